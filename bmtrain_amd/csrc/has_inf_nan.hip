// Loss-scale overflow check for gfx950: does a 16-bit float buffer hold an inf or NaN?
// Replaces csrc/cuda/has_inf_nan.cu:35-138 of the reference (two kernels and a
// 1024-byte intermediate) by one streaming kernel.
//
// An element is inf/NaN iff its exponent field is all ones.  Two elements are
// tested per dword without unpacking: mask the exponent fields and add the value
// that makes an all-ones field carry into bit 15 of its half; no other field value
// reaches bit 15, and the mask keeps the low half's carry out of the high half:
//     hit |= ((w & EXP_MASK2) + EXP_CARRY2) & 0x80008000
// Each lane ORs its dwords, the wave votes with one ballot, and one lane of a wave
// that saw a hit issues a relaxed atomic byte store out[0] = 1 (after a look at the
// flag: once it is up nobody stores again).  When nothing is found the kernel writes
// nothing, which keeps the flag sticky across calls.
#include <atomic>
#include "bmt_device.h"
#include "bmt_host.h"
#include "../../include/bmt_hip.h"

namespace bmt {

// One workgroup scans one tile of kScanThreads * UNROLL 16-byte vectors and exits (short
// workgroups stream faster here than a resident grid that loops; one vector per lane and no
// workgroup-level meeting point measured 94 % of HBM peak, two vectors with an LDS word and two
// barriers 89 %).
constexpr int kScanThreads = 1024;
constexpr int kScanUnroll = 1;
// The statistics kernel ends in a workgroup-wide sum; a four times larger tile (128 KiB) spreads
// that cost and keeps eight loads per lane in flight.
constexpr int kStatsUnroll = 8;

template <typename T>
__device__ __forceinline__ uint32_t exp_all_ones2(uint32_t w) {
    return ((w & T::kExpMask2) + T::kExpCarry2) & 0x80008000u;
}

template <typename T, int UNROLL>
__global__ __launch_bounds__(kScanThreads) void has_inf_nan_kernel(
    const uint16_t *__restrict__ g, int64_t head, int64_t nvec, int64_t n, uint8_t *__restrict__ out) {
    uint32_t hit = 0;
    const u32x4 *body = (const u32x4 *)(g + head);
    const int64_t base = (int64_t)blockIdx.x * (kScanThreads * UNROLL) + threadIdx.x;
    u32x4 w[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kScanThreads;
        if (i < nvec) w[u] = __builtin_nontemporal_load(body + i);
        else w[u] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++)
        hit |= exp_all_ones2<T>(w[u].x) | exp_all_ones2<T>(w[u].y) | exp_all_ones2<T>(w[u].z) | exp_all_ones2<T>(w[u].w);
    // Unaligned head (< 8 elements) and tail (< 8 elements): workgroup 0, one element per lane.
    if (blockIdx.x == 0) {
        const int64_t tail_lo = head + nvec * 8;
        const int64_t edge = head + (n - tail_lo);
        if ((int64_t)threadIdx.x < edge) {
            const int64_t i = (int64_t)threadIdx.x < head ? (int64_t)threadIdx.x : tail_lo + ((int64_t)threadIdx.x - head);
            hit |= exp_all_ones2<T>((uint32_t)g[i]);
        }
    }
    // Each wave votes on its own (no LDS, no barrier); a wave that saw a hit raises the flag unless
    // it is up already, so a buffer full of NaNs costs a few stores, not one per wave.
    if (__builtin_amdgcn_ballot_w64(hit != 0) != 0 && (threadIdx.x & (kWave - 1)) == 0 &&
        __hip_atomic_load(out, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
        __hip_atomic_store(out, (uint8_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T>
static int scan(int64_t n, const void *g, void *out, void *stream, const char *who) {
    if (n <= 0) return 0;  // has_inf_nan.cu:108,:128
    if (!g || !out) return fail(-1, "has_nan_inf launcher: null pointer");
    const uintptr_t a = (uintptr_t)g;
    if (a & 1u) return fail(-1, "has_nan_inf launcher: gradient pointer is not 2-byte aligned");
    int64_t head = (int64_t)(((16 - (a & 15u)) & 15u) / 2);
    if (head > n) head = n;
    const int64_t nvec = (n - head) / 8;
    constexpr int UNROLL = kScanUnroll;
    const int64_t tile = (int64_t)kScanThreads * UNROLL;
    const int64_t ntiles = (nvec + tile - 1) / tile;
    if (ntiles > 0x7FFFFFFF) return fail(-1, "has_nan_inf launcher: buffer too large for one launch");
    const int64_t grid = ntiles < 1 ? 1 : ntiles;
    hipLaunchKernelGGL((has_inf_nan_kernel<T, UNROLL>), dim3((unsigned)grid), dim3(kScanThreads), 0, (hipStream_t)stream,
                       (const uint16_t *)g, head, nvec, n, (uint8_t *)out);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}


// ---- gradient statistics: overflow flag and sum of squares in one pass -----------------
// For gradient clipping the reference computes, per tensor, g.float().norm(2) (a 4-byte copy of
// every gradient is written and read back, optim_manager.py:186-190) and, separately, the
// overflow flag.  This kernel reads the gradient once (2 B / element) and produces both: the
// flag as above, and per workgroup one fp32 partial sum of squares, which a second, single
// workgroup adds up in double precision in a fixed order and accumulates into `sumsq[0]`.
// acc + lo(w)^2 + hi(w)^2 in one instruction (v_dot2_f32_f16 / v_dot2_f32_bf16): the products of
// 16-bit values are exact in fp32, so this is the unpack-and-fma sequence without the unpacking.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
template <typename T> __device__ __forceinline__ float sumsq2(uint32_t w, float acc);
template <> __device__ __forceinline__ float sumsq2<Half>(uint32_t w, float acc) {
    const half2_t h = __builtin_bit_cast(half2_t, w);
    return __builtin_amdgcn_fdot2(h, h, acc, false);
}
template <> __device__ __forceinline__ float sumsq2<BFloat16>(uint32_t w, float acc) {
    const bf16x2_t h = __builtin_bit_cast(bf16x2_t, w);
    return __builtin_amdgcn_fdot2_f32_bf16(h, h, acc, false);
}

template <typename T, int UNROLL>
__global__ __launch_bounds__(kScanThreads) void grad_stats_kernel(
    const uint16_t *__restrict__ g, int64_t head, int64_t nvec, int64_t n, uint8_t *__restrict__ flag,
    float *__restrict__ partials) {
    uint32_t hit = 0;
    float acc = 0.f;
    const u32x4 *body = (const u32x4 *)(g + head);
    const int64_t base = (int64_t)blockIdx.x * (kScanThreads * UNROLL) + threadIdx.x;
    u32x4 w[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kScanThreads;
        if (i < nvec) w[u] = __builtin_nontemporal_load(body + i);
        else w[u] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            hit |= exp_all_ones2<T>(w[u][k]);
            acc = sumsq2<T>(w[u][k], acc);
        }
    }
    if (blockIdx.x == 0) {   // unaligned head and tail, one element per lane
        const int64_t tail_lo = head + nvec * 8;
        const int64_t edge = head + (n - tail_lo);
        if ((int64_t)threadIdx.x < edge) {
            const int64_t i = (int64_t)threadIdx.x < head ? (int64_t)threadIdx.x : tail_lo + ((int64_t)threadIdx.x - head);
            hit |= exp_all_ones2<T>((uint32_t)g[i]);
            const float x = T::to_f32(g[i]);
            acc = __builtin_fmaf(x, x, acc);
        }
    }
    __shared__ float slots[kScanThreads / kWave];
    __shared__ uint32_t any_wave;
    if (threadIdx.x == 0) any_wave = 0;
    __syncthreads();
    if (__builtin_amdgcn_ballot_w64(hit != 0) != 0 && (threadIdx.x & (kWave - 1)) == 0) any_wave = 1;
    const float total = block_allreduce<false>(acc, slots);   // contains a barrier
    if (threadIdx.x == 0) {
        partials[blockIdx.x] = total;
        if (any_wave) __hip_atomic_store(flag, (uint8_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// One workgroup: lane t adds partials t, t + 1024, ... in double, then a fixed tree over the lanes.
__global__ __launch_bounds__(kScanThreads) void grad_stats_finish_kernel(const float *__restrict__ partials, int64_t count,
                                                                        double *__restrict__ sumsq) {
    __shared__ double lanes[kScanThreads];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < count; i += kScanThreads) acc += (double)partials[i];
    lanes[threadIdx.x] = acc;
    __syncthreads();
    for (int stride = kScanThreads / 2; stride > 0; stride >>= 1) {
        if ((int)threadIdx.x < stride) lanes[threadIdx.x] += lanes[threadIdx.x + stride];
        __syncthreads();
    }
    if (threadIdx.x == 0) sumsq[0] += lanes[0];
}

static int64_t stats_tiles(int64_t n, const void *g, int64_t *head_out, int64_t *nvec_out) {
    const uintptr_t a = (uintptr_t)g;
    int64_t head = (int64_t)(((16 - (a & 15u)) & 15u) / 2);
    if (head > n) head = n;
    const int64_t nvec = (n - head) / 8;
    const int64_t tile = (int64_t)kScanThreads * kStatsUnroll;
    const int64_t ntiles = (nvec + tile - 1) / tile;
    if (head_out) *head_out = head;
    if (nvec_out) *nvec_out = nvec;
    return ntiles < 1 ? 1 : ntiles;
}

template <typename T>
static int grad_stats(int64_t n, const void *g, void *sumsq, void *flag, void *workspace, void *stream, const char *who) {
    if (n <= 0) return 0;
    if (!g || !sumsq || !flag || !workspace) return fail(-1, "grad_stats launcher: null pointer");
    if ((uintptr_t)g & 1u) return fail(-1, "grad_stats launcher: gradient pointer is not 2-byte aligned");
    if ((uintptr_t)sumsq & 7u) return fail(-1, "grad_stats launcher: sumsq must be 8-byte aligned");
    int64_t head = 0, nvec = 0;
    const int64_t grid = stats_tiles(n, g, &head, &nvec);
    if (grid > 0x7FFFFFFF) return fail(-1, "grad_stats launcher: buffer too large for one launch");
    hipLaunchKernelGGL((grad_stats_kernel<T, kStatsUnroll>), dim3((unsigned)grid), dim3(kScanThreads), 0, (hipStream_t)stream,
                       (const uint16_t *)g, head, nvec, n, (uint8_t *)flag, (float *)workspace);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, who, e);
    hipLaunchKernelGGL(grad_stats_finish_kernel, dim3(1), dim3(kScanThreads), 0, (hipStream_t)stream,
                       (const float *)workspace, grid, (double *)sumsq);
    e = hipGetLastError();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}

// ---- the same pass for callers that cannot allocate -------------------------------------------
// The partial sums go to a fixed array in device memory instead of a caller's workspace.  Every GPU the
// library runs on holds its own copy of the array at its own address; the address is looked up once per
// device (with that device current) and used from then on — the array's name is only a host-side handle.
constexpr int64_t kStaticPartials = (int64_t)1 << 20;                     // 4 MiB: gradients of up to 2^36 elements
static __device__ __align__(256) float stats_scratch[kStaticPartials];
static std::atomic<float *> stats_scratch_ptr[64];                         // per device, null until looked up

static float *static_partials(hipStream_t stream, const char **why) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) { *why = "grad_stats_noalloc_launcher: no current device"; return nullptr; }
    // the array used is the current device's copy: a stream of another device would run the kernels over there
    hipDevice_t owner = -1;
    if (stream != hipStreamPerThread && (hipStreamGetDevice(stream, &owner) != hipSuccess || (int)owner != dev)) {
        (void)hipGetLastError();
        *why = "grad_stats_noalloc_launcher: the stream does not belong to the current device";
        return nullptr;
    }
    float *ptr = stats_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(stats_scratch));
        if (e != hipSuccess || ptr == nullptr) { *why = "grad_stats_noalloc_launcher: hipGetSymbolAddress failed"; return nullptr; }
        stats_scratch_ptr[dev].store(ptr, std::memory_order_release);     // every thread finds the same address
    }
    return ptr;
}

// ---- the same two passes over several gradient tensors at once ------------------------------------
// A model whose gradients are separate allocations is scanned tensor by tensor otherwise: the 291 tensors of a
// 6.74 B-parameter model cost 2.35 ms (flag) / 3.46 ms (flag and sum of squares, two launches each) against
// 1.8 / 1.9 ms for one flat buffer, all of the difference launches; here 1.88 / 1.96 ms.  Up to kScanBatch tensors
// travel in the kernel arguments; tiles are numbered through the tensors, a workgroup finds its tensor from the
// table in the arguments, and the first tile of a tensor also takes that tensor's elements in front of and behind
// its 16-byte vectors.  The partial sums are one per tile, as in the single-tensor kernel.
constexpr int kScanBatch = 64;
// Vectors per lane of the flag-only pass: the search in front makes a workgroup's start longer than the
// single-tensor kernel's, and two vectors spread it (1 / 2 / 3 vectors: 48 / 89.5 / 85.5 % of the HBM peak over
// the 291 gradient tensors of a 6.74 B-parameter model).
constexpr int kScanMultiUnroll = 2;
// Tensors travel in sets of four: first[i] is the number of the first tile of the set's tensor i (0xFFFFFFFF
// behind the last tensor of the launch; every tensor has at least one tile, so the used entries rise strictly),
// and every_4th[j] repeats four[j].first[0].  A workgroup finds its tensor with two rounds of scalar loads - the
// 16 entries of every_4th, then one set with its pointers and counts - instead of the six dependent loads of a
// bisection and a seventh for pointer and count: the search runs in front of the workgroup's only loads of data,
// so every round of it is time in which that workgroup's share of the memory pipeline stands idle.
struct ScanFour {
    uint32_t first[4];
    const uint16_t *g[4];
    int64_t n[4];
};
struct ScanBatch {
    ScanFour four[kScanBatch / 4];
    uint32_t every_4th[kScanBatch / 4];
};

template <typename T, bool STATS>
__global__ __launch_bounds__(kScanThreads) void scan_multi_kernel(ScanBatch batch, uint8_t *__restrict__ flag,
                                                                   float *__restrict__ partials) {
    constexpr int UNROLL = STATS ? kStatsUnroll : kScanMultiUnroll;
    int group = -1;                                    // every_4th[group] <= blockIdx.x < every_4th[group + 1]
#pragma unroll
    for (int j = 0; j < kScanBatch / 4; j++) group += batch.every_4th[j] <= blockIdx.x ? 1 : 0;
    const ScanFour &set = batch.four[group];
    const uint32_t f0 = set.first[0], f1 = set.first[1], f2 = set.first[2], f3 = set.first[3];
    const uint16_t *g0 = set.g[0], *g1 = set.g[1], *g2 = set.g[2], *g3 = set.g[3];
    const int64_t n0 = set.n[0], n1 = set.n[1], n2 = set.n[2], n3 = set.n[3];
    const int within = (f1 <= blockIdx.x ? 1 : 0) + (f2 <= blockIdx.x ? 1 : 0) + (f3 <= blockIdx.x ? 1 : 0);
    const uint32_t first = within == 0 ? f0 : within == 1 ? f1 : within == 2 ? f2 : f3;
    const uint16_t *g = within == 0 ? g0 : within == 1 ? g1 : within == 2 ? g2 : g3;
    const int64_t n = within == 0 ? n0 : within == 1 ? n1 : within == 2 ? n2 : n3;
    const uint32_t tile = blockIdx.x - first;
    int64_t head = (int64_t)(((16 - ((uintptr_t)g & 15u)) & 15u) / 2);
    if (head > n) head = n;
    const int64_t nvec = (n - head) / 8;
    const u32x4 *body = (const u32x4 *)(g + head);
    const int64_t base = (int64_t)tile * (kScanThreads * UNROLL) + threadIdx.x;
    uint32_t hit = 0;
    float acc = 0.f;
    u32x4 w[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kScanThreads;
        if (i < nvec) w[u] = __builtin_nontemporal_load(body + i);
        else w[u] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            hit |= exp_all_ones2<T>(w[u][k]);
            if (STATS) acc = sumsq2<T>(w[u][k], acc);
        }
    }
    if (tile == 0) {   // unaligned head and tail of this tensor, one element per lane
        const int64_t tail_lo = head + nvec * 8;
        const int64_t edge = head + (n - tail_lo);
        if ((int64_t)threadIdx.x < edge) {
            const int64_t i = (int64_t)threadIdx.x < head ? (int64_t)threadIdx.x : tail_lo + ((int64_t)threadIdx.x - head);
            hit |= exp_all_ones2<T>((uint32_t)g[i]);
            if (STATS) {
                const float x = T::to_f32(g[i]);
                acc = __builtin_fmaf(x, x, acc);
            }
        }
    }
    if (!STATS) {
        if (__builtin_amdgcn_ballot_w64(hit != 0) != 0 && (threadIdx.x & (kWave - 1)) == 0 &&
            __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
            __hip_atomic_store(flag, (uint8_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    __shared__ float slots[kScanThreads / kWave];
    __shared__ uint32_t any_wave;
    if (threadIdx.x == 0) any_wave = 0;
    __syncthreads();
    if (__builtin_amdgcn_ballot_w64(hit != 0) != 0 && (threadIdx.x & (kWave - 1)) == 0) any_wave = 1;
    const float total = block_allreduce<false>(acc, slots);   // contains a barrier
    if (threadIdx.x == 0) {
        partials[blockIdx.x] = total;
        if (any_wave) __hip_atomic_store(flag, (uint8_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

template <typename T>
static int scan_multi(int32_t count, const bmt_scan_tensor *tensors, void *sumsq, void *flag, void *workspace, void *stream,
                      const char *who) {
    if (count <= 0) return 0;
    if (!tensors) return fail(-1, "grad_stats_multi_launcher: null tensor table");
    if (!flag) return fail(-1, "grad_stats_multi_launcher: null flag");
    if (sumsq && !workspace) return fail(-1, "grad_stats_multi_launcher: sumsq without workspace");
    if ((uintptr_t)sumsq & 7u) return fail(-1, "grad_stats_multi_launcher: sumsq must be 8-byte aligned");
    const int64_t per_tile = (int64_t)kScanThreads * (sumsq ? kStatsUnroll : kScanMultiUnroll) * 8;     // elements
    for (int32_t k = 0; k < count; k++) {              // the whole table first: an error means nothing was launched
        if (tensors[k].n <= 0) continue;
        if (!tensors[k].g_16) return fail(-1, "grad_stats_multi_launcher: null pointer");
        if ((uintptr_t)tensors[k].g_16 & 1u) return fail(-1, "grad_stats_multi_launcher: gradient pointer is not 2-byte aligned");
        if (tensors[k].n / per_tile + 1 > 0x3FFFFFFF) return fail(-1, "grad_stats_multi_launcher: tensor too large for one launch");
    }
    ScanBatch batch;
    int held = 0;                                      // tensors in the batch
    uint32_t tiles_held = 0;                           // and their tiles
    auto flush = [&]() -> hipError_t {
        if (held == 0) return hipSuccess;
        for (int k = held; k < kScanBatch; k++) {      // behind the last tensor: never found, never dereferenced
            batch.four[k / 4].first[k % 4] = 0xFFFFFFFFu;
            batch.four[k / 4].g[k % 4] = nullptr;
            batch.four[k / 4].n[k % 4] = 0;
        }
        for (int j = 0; j < kScanBatch / 4; j++) batch.every_4th[j] = batch.four[j].first[0];
        const uint32_t tiles = tiles_held;
        if (sumsq) {
            hipLaunchKernelGGL((scan_multi_kernel<T, true>), dim3(tiles), dim3(kScanThreads), 0, (hipStream_t)stream, batch,
                               (uint8_t *)flag, (float *)workspace);
            hipLaunchKernelGGL(grad_stats_finish_kernel, dim3(1), dim3(kScanThreads), 0, (hipStream_t)stream,
                               (const float *)workspace, (int64_t)tiles, (double *)sumsq);
        } else {
            hipLaunchKernelGGL((scan_multi_kernel<T, false>), dim3(tiles), dim3(kScanThreads), 0, (hipStream_t)stream, batch,
                               (uint8_t *)flag, (float *)nullptr);
        }
        held = 0;
        tiles_held = 0;
        return hipGetLastError();
    };
    for (int32_t k = 0; k < count; k++) {
        const int64_t n = tensors[k].n;
        if (n <= 0) continue;
        const uintptr_t a = (uintptr_t)tensors[k].g_16;
        int64_t head = (int64_t)(((16 - (a & 15u)) & 15u) / 2);
        if (head > n) head = n;
        const int64_t nvec = (n - head) / 8;
        int64_t tiles = (nvec * 8 + per_tile - 1) / per_tile;
        if (tiles < 1) tiles = 1;
        if (held == kScanBatch || (int64_t)tiles_held + tiles > 0x7FFFFFFF) {
            hipError_t e = flush();
            if (e != hipSuccess) return fail((int)e, who, e);
        }
        batch.four[held / 4].first[held % 4] = tiles_held;
        batch.four[held / 4].g[held % 4] = (const uint16_t *)tensors[k].g_16;
        batch.four[held / 4].n[held % 4] = n;
        tiles_held += (uint32_t)tiles;
        held++;
    }
    hipError_t e = flush();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}

}  // namespace bmt

extern "C" int grad_stats_noalloc_launcher(int64_t n, const void *g_16, int32_t is_bf16, void *sumsq, void *flag, void *stream) {
    if (n <= 0) return 0;
    if (bmt::stats_tiles(n, g_16, nullptr, nullptr) > bmt::kStaticPartials)
        return bmt::fail(-1, "grad_stats_noalloc_launcher: more than 2^36 elements; use grad_stats_*_launcher with a workspace");
    const char *why = "";
    float *partials = bmt::static_partials((hipStream_t)stream, &why);
    if (partials == nullptr) return bmt::fail(-1, why);
    return is_bf16 ? bmt::grad_stats<bmt::BFloat16>(n, g_16, sumsq, flag, partials, stream, "grad_stats_noalloc_launcher")
                   : bmt::grad_stats<bmt::Half>(n, g_16, sumsq, flag, partials, stream, "grad_stats_noalloc_launcher");
}

extern "C" int has_nan_inf_fp16_launcher(int64_t n, const void *g_fp16, void *mid, void *out, void *stream) {
    (void)mid;
    return bmt::scan<bmt::Half>(n, g_fp16, out, stream, "has_nan_inf_fp16_launcher");
}
extern "C" int has_nan_inf_bf16_launcher(int64_t n, const void *g_bf16, void *mid, void *out, void *stream) {
    (void)mid;
    return bmt::scan<bmt::BFloat16>(n, g_bf16, out, stream, "has_nan_inf_bf16_launcher");
}

extern "C" int64_t grad_stats_workspace_floats(int64_t n) {
    // the worst case over base alignments: no head elements, every vector in the body
    if (n <= 0) return 1;
    const int64_t tile = (int64_t)bmt::kScanThreads * bmt::kStatsUnroll * 8;
    return (n + tile - 1) / tile + 1;
}
extern "C" int grad_stats_fp16_launcher(int64_t n, const void *g_fp16, void *sumsq, void *flag, void *workspace,
                                        void *stream) {
    return bmt::grad_stats<bmt::Half>(n, g_fp16, sumsq, flag, workspace, stream, "grad_stats_fp16_launcher");
}
extern "C" int grad_stats_bf16_launcher(int64_t n, const void *g_bf16, void *sumsq, void *flag, void *workspace,
                                        void *stream) {
    return bmt::grad_stats<bmt::BFloat16>(n, g_bf16, sumsq, flag, workspace, stream, "grad_stats_bf16_launcher");
}

extern "C" int grad_stats_multi_launcher(int32_t count, const bmt_scan_tensor *tensors, int32_t is_bf16, void *sumsq, void *flag,
                                         void *workspace, void *stream) {
    return is_bf16 ? bmt::scan_multi<bmt::BFloat16>(count, tensors, sumsq, flag, workspace, stream, "grad_stats_multi_launcher")
                   : bmt::scan_multi<bmt::Half>(count, tensors, sumsq, flag, workspace, stream, "grad_stats_multi_launcher");
}
