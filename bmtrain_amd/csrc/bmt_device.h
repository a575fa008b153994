// Device-side helpers shared by the gfx950 kernels: 16-bit float conversions,
// vector types, wave64 / workgroup reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bmt {

typedef float    f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;  // gfx950 wavefront

// ---- element types -------------------------------------------------------
// A 16-bit float travels as its bit pattern; the tag type picks the converters.
struct Half {  // IEEE binary16
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return (float)__builtin_bit_cast(_Float16, b);          // exact, subnormals kept
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        // The empty asm makes `f` exist as a rounded fp32 value.  Without it the compiler folds
        // the multiply / fma that produced `f` into v_fma_mixlo_f16, which rounds the exact
        // result once, straight to fp16, instead of to fp32 and then to fp16 as the reference
        // arithmetic does; the two differ by one fp16 ulp near ties.
        asm("" : "+v"(f));
        return __builtin_bit_cast(uint16_t, (_Float16)f);        // v_cvt_f16_f32, round-nearest-even
    }
    static constexpr uint32_t kExpMask2 = 0x7C007C00u;   // exponent field of both halves of a dword
    static constexpr uint32_t kExpCarry2 = 0x04000400u;  // exponent all-ones + this carries into bit 15
};
struct BFloat16 {  // bfloat16 = upper half of binary32
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) {  // round-nearest-even, NaN quieted
        uint32_t u = __builtin_bit_cast(uint32_t, f);
        uint32_t r = u + 0x7FFFu + ((u >> 16) & 1u);
        uint32_t q = u | 0x00400000u;
        return (uint16_t)(((u & 0x7FFFFFFFu) > 0x7F800000u ? q : r) >> 16);
    }
    static constexpr uint32_t kExpMask2 = 0x7F807F80u;
    static constexpr uint32_t kExpCarry2 = 0x00800080u;
};

template <typename T>
__device__ __forceinline__ float lo_f32(uint32_t packed) { return T::to_f32((uint16_t)(packed & 0xFFFFu)); }
template <typename T>
__device__ __forceinline__ float hi_f32(uint32_t packed) { return T::to_f32((uint16_t)(packed >> 16)); }
template <>
__device__ __forceinline__ float lo_f32<BFloat16>(uint32_t packed) { return __builtin_bit_cast(float, packed << 16); }
template <>
__device__ __forceinline__ float hi_f32<BFloat16>(uint32_t packed) { return __builtin_bit_cast(float, packed & 0xFFFF0000u); }

// Two fp32 values -> one dword of two 16-bit values, round-to-nearest-even, with the packed
// hardware converts of gfx950 (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32).
typedef float  f32x2_t  __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<BFloat16>(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
template <>
__device__ __forceinline__ uint32_t pack2<Half>(float lo, float hi) {
    asm("" : "+v"(lo), "+v"(hi));   // keep the fp32 rounding step (see Half::from_f32)
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, f16x2_t));
}

// ---- wave64 reductions ----------------------------------------------------
// Butterfly over the 64 lanes: every lane ends with the full result.
__device__ __forceinline__ float wave_allreduce_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_allreduce_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Workgroup all-reduce through LDS: one float per wave, every thread returns the result.
// `slots` must hold blockDim.x / 64 floats and may be reused after the call returns
// only after another barrier.
template <bool IsMax>
__device__ __forceinline__ float block_allreduce(float v, float *slots) {
    v = IsMax ? wave_allreduce_max(v) : wave_allreduce_sum(v);
    const int nwaves = (int)(blockDim.x / kWave);
    if (nwaves == 1) return v;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) slots[wave] = v;
    __syncthreads();
    float r = slots[0];
    for (int w = 1; w < nwaves; w++) r = IsMax ? fmaxf(r, slots[w]) : r + slots[w];
    return r;
}

// ---- vector memory instructions of the resident streaming kernels ---------------------------
// Those kernels keep one tile of loads in flight while they compute and store the tile before, which
// the compiler's wait-count insertion cannot express; their loads, stores and ticket atomics are asm
// statements and they place `s_waitcnt vmcnt(N)` themselves (see adam.hip).  A 16-byte store is
// followed by `s_nop 1`: it reads its data registers for two more cycles, and the compiler pads that
// hazard only for stores it emits itself.
__device__ __forceinline__ void stream_load(f32x4 &dst, const f32x4 *src) {
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(src) : "memory");
}
__device__ __forceinline__ void stream_load(u32x2 &dst, const u32x2 *src) {
    asm volatile("global_load_dwordx2 %0, %1, off nt" : "=v"(dst) : "v"(src) : "memory");
}
__device__ __forceinline__ void stream_store(f32x4 *dst, const f32x4 &v) {
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
}
__device__ __forceinline__ void stream_store(u32x2 *dst, const u32x2 &v) {
    asm volatile("global_store_dwordx2 %0, %1, off nt" : : "v"(dst), "v"(v) : "memory");
}
__device__ __forceinline__ void stream_load(u32x4 &dst, const u32x4 *src) {
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(dst) : "v"(src) : "memory");
}
__device__ __forceinline__ void stream_store(u32x4 *dst, const u32x4 &v) {
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 1" : : "v"(dst), "v"(v) : "memory");
}
__device__ __forceinline__ void stream_draw(uint32_t &ticket, uint32_t *counter) {
    const uint32_t one = 1u;
    asm volatile("global_atomic_add %0, %1, %2, off sc0" : "=v"(ticket) : "v"(counter), "v"(one) : "memory");
}

// ---- ticket counters that the library keeps for a stream (host side: stream_slot_for in bmt_host.h) ------------
// A slot is a group of kSlotCounters counters, 4 KiB apart (counter c: word c * 1024 of the slot), plus a count of the
// workgroups that have left the running launch (word 1).  The counters start at zero (the array is zero when the
// library is loaded) and a launch leaves them at zero: every workgroup has received its last ticket before it leaves
// (it waits for it), so when the last one leaves nothing is drawing any more; that workgroup puts the counters and
// the count of leavers back to zero and then writes the launch's number into the slot's word of pinned host memory
// (a release, so that the zeros are in memory first): from then on the host may hand the slot to another stream.
constexpr int kSlotCounters = 8;
__device__ __forceinline__ void stream_slot_leave(uint32_t *slot, uint32_t *done_word, uint32_t launch_number) {
    if (threadIdx.x == 0) {
        const uint32_t left = __hip_atomic_fetch_add(slot + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (left + 1 == gridDim.x) {
#pragma unroll
            for (int c = 0; c < kSlotCounters; c++)
                __hip_atomic_store(slot + c * 1024, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(slot + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(done_word, launch_number, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

}  // namespace bmt
