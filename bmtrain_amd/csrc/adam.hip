// Fused mixed-precision Adam step for gfx950 (MI355X).
//
// One streaming pass: per element it reads the fp32 master parameter, the two
// moments and the 16-bit gradient (14 B for bf16, 12 B for fp16) and writes the
// fp32 master, the moments and the 16-bit parameter copy (14 B / 12 B).  The
// kernel is HBM-bound; the design goal is full-width (16 B / lane) coalesced
// accesses, all loads of a workgroup issued before its arithmetic starts, and
// many short workgroups so that every CU always has fresh waves to issue from.
//
// Arithmetic (replaces csrc/cuda/adam_cuda.cu:8-72 of the reference).  The
// expression tree is fixed — this file is compiled with -ffp-contract=off and
// the only fused multiply-adds are the explicit ones below; `/` and sqrtf are
// correctly rounded — so that results are reproducible bit-for-bit on a CPU:
//   bf16:  g  = float(g16) / scale
//          m' = fma(b1, m, (1-b1)*g)
//          v' = fma(b2, v, ((1-b2)*g)*g)
//          p' = fma(-(lr*wd), p, p - ((lr*m')/bc1) / (sqrt(v'/bc2) + eps))
//   fp16:  g  = float(g16)                      (moments stay multiplied by scale)
//          m' = fma(b1, float(m16), (1-b1)*g)
//          v' = fma(b2, v, (((1-b2)*g)*g) / scale)
//          p' = fma(-(lr*wd), p, p - ((lr*m')/bc1) / (sqrt((v'*scale)/bc2) + eps*scale))
// This is the reference's expression with the multiply-adds contracted the way
// its own host compiler contracts the identical CPU loop (adam_cpu.hpp:265-276).
#include <type_traits>
#include "bmt_device.h"
#include "bmt_host.h"
#include "../../include/bmt_hip.h"

#pragma clang fp contract(off)

namespace bmt {

struct AdamHyper {
    float b1, b2, eps, lr, scale, wd, bc1, bc2;
    float gcoef = 1.0f;   // gradient clipping factor applied on the fly (1: none), see clip16
};

// Gradient clipping folded into the step.  Eagerly, clipping multiplies the 16-bit gradient in
// place: fp32 product of the gradient and the (16-bit-rounded) factor, rounded back to 16 bits.
// Doing exactly that to the value in flight gives the same bits without the extra pass over the
// gradients.
template <typename T>
__device__ __forceinline__ float clip16(float g, float coef) {
    return coef == 1.0f ? g : T::to_f32(T::from_f32(g * coef));
}

// Per-element update, bf16 flavour (plain fp32 moments).
__device__ __forceinline__ void adam_elem_unscaled(float g16f, float &m, float &v, float &p, const AdamHyper &h,
                                                   float omb1, float omb2, float lrwd) {
    float g = g16f / h.scale;
    float mm = __builtin_fmaf(h.b1, m, omb1 * g);
    float vv = __builtin_fmaf(h.b2, v, (omb2 * g) * g);
    float den = __builtin_sqrtf(vv / h.bc2) + h.eps;
    float upd = ((h.lr * mm) / h.bc1) / den;
    float np = __builtin_fmaf(-lrwd, p, p - upd);
    m = mm; v = vv; p = np;
}

// Per-element update, fp16 flavour (moments pre-multiplied by the loss scale).
__device__ __forceinline__ void adam_elem_scaled(float g, float &m, float &v, float &p, const AdamHyper &h,
                                                 float omb1, float omb2, float lrwd, float eps_s) {
    float mm = __builtin_fmaf(h.b1, m, omb1 * g);
    float vv = __builtin_fmaf(h.b2, v, ((omb2 * g) * g) / h.scale);
    float den = __builtin_sqrtf((vv * h.scale) / h.bc2) + eps_s;
    float upd = ((h.lr * mm) / h.bc1) / den;
    float np = __builtin_fmaf(-lrwd, p, p - upd);
    m = mm; v = vv; p = np;
}

// The same for the four packed gradients of a group, with the hardware's packed round-to-nearest-even converts.
template <typename T>
__device__ __forceinline__ u32x2 clip_group(u32x2 g, float coef) {
    if (coef == 1.0f) return g;
    return u32x2{pack2<T>(lo_f32<T>(g.x) * coef, hi_f32<T>(g.x) * coef), pack2<T>(lo_f32<T>(g.y) * coef, hi_f32<T>(g.y) * coef)};
}

// Four elements at once: gradients arrive as two packed dwords.
template <typename T>
__device__ __forceinline__ void adam_group_unscaled(u32x2 g, f32x4 &m, f32x4 &v, f32x4 &p, const AdamHyper &h, float omb1,
                                                    float omb2, float lrwd) {
    g = clip_group<T>(g, h.gcoef);
    float gm[4] = {lo_f32<T>(g.x), hi_f32<T>(g.x), lo_f32<T>(g.y), hi_f32<T>(g.y)};
    float ma[4] = {m.x, m.y, m.z, m.w}, va[4] = {v.x, v.y, v.z, v.w}, pa[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int k = 0; k < 4; k++) adam_elem_unscaled(gm[k], ma[k], va[k], pa[k], h, omb1, omb2, lrwd);
    m = f32x4{ma[0], ma[1], ma[2], ma[3]};
    v = f32x4{va[0], va[1], va[2], va[3]};
    p = f32x4{pa[0], pa[1], pa[2], pa[3]};
}
template <typename T>
__device__ __forceinline__ void adam_group_scaled(u32x2 g, f32x4 &m, f32x4 &v, f32x4 &p, const AdamHyper &h, float omb1,
                                                  float omb2, float lrwd, float eps_s) {
    g = clip_group<T>(g, h.gcoef);
    float gm[4] = {lo_f32<T>(g.x), hi_f32<T>(g.x), lo_f32<T>(g.y), hi_f32<T>(g.y)};
    float ma[4] = {m.x, m.y, m.z, m.w}, va[4] = {v.x, v.y, v.z, v.w}, pa[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int k = 0; k < 4; k++) adam_elem_scaled(gm[k], ma[k], va[k], pa[k], h, omb1, omb2, lrwd, eps_s);
    m = f32x4{ma[0], ma[1], ma[2], ma[3]};
    v = f32x4{va[0], va[1], va[2], va[3]};
    p = f32x4{pa[0], pa[1], pa[2], pa[3]};
}

template <typename T>
__device__ __forceinline__ T ld(const T *p) { return __builtin_nontemporal_load(p); }
template <typename T>
__device__ __forceinline__ void st(T *p, T v) { __builtin_nontemporal_store(v, p); }

// Launch shape of the short vector kernels: one workgroup owns one tile and exits.
constexpr int kAdamThreads = 1024;
constexpr int kAdamUnroll = 1;

// A call's elements in front of and behind its vector body (the arrays may start anywhere): lane t < head takes
// element t - head, lane head + k takes the k-th element behind the body; indices count from the body's first element.
// The first workgroup of the one-tile kernels steps them next to its tile, with the per-element routine that the
// element kernels use, so such a call stays one launch.
__device__ __forceinline__ int64_t edge_element(int64_t nvec, int32_t head) {
    const int32_t t = (int32_t)threadIdx.x;
    return t < head ? (int64_t)t - head : 4 * nvec + (t - head);
}

// Vector body, bf16.  `nvec` = number of 4-element groups; every pointer is aligned for its
// vector type.  A tile is kAdamThreads * UNROLL groups; group u of a lane sits kAdamThreads groups
// after group u-1, so each load instruction of a wave covers 64 consecutive vectors (1 KiB of fp32).
template <int UNROLL>
__global__ __launch_bounds__(kAdamThreads) void adam_bf16_vec_kernel(
    int64_t nvec, f32x4 *__restrict__ p32, u32x2 *__restrict__ p16, const u32x2 *__restrict__ g16,
    f32x4 *__restrict__ mom, f32x4 *__restrict__ var, AdamHyper h, int32_t head, int32_t tail) {
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd;
    if (blockIdx.x == 0 && (int)threadIdx.x < head + tail) {      // the elements around the vector body, one per lane
        const int64_t e = edge_element(nvec, head);
        float *p1 = (float *)p32 + e, *m1 = (float *)mom + e, *v1 = (float *)var + e;
        float p = *p1, m = *m1, v = *v1;
        adam_elem_unscaled(clip16<BFloat16>(BFloat16::to_f32(((const uint16_t *)g16)[e]), h.gcoef), m, v, p, h, omb1, omb2, lrwd);
        *p1 = p; *m1 = m; *v1 = v; ((uint16_t *)p16)[e] = BFloat16::from_f32(p);
    }
    const int64_t base = (int64_t)blockIdx.x * (kAdamThreads * UNROLL) + threadIdx.x;
    f32x4 p[UNROLL], m[UNROLL], v[UNROLL];
    u32x2 g[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kAdamThreads;
        ok[u] = i < nvec;
        if (ok[u]) { g[u] = ld(g16 + i); p[u] = ld(p32 + i); m[u] = ld(mom + i); v[u] = ld(var + i); }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        if (!ok[u]) continue;
        const int64_t i = base + (int64_t)u * kAdamThreads;
        adam_group_unscaled<BFloat16>(g[u], m[u], v[u], p[u], h, omb1, omb2, lrwd);
        u32x2 o;
        o.x = pack2<BFloat16>(p[u].x, p[u].y);
        o.y = pack2<BFloat16>(p[u].z, p[u].w);
        st(p32 + i, p[u]); st(mom + i, m[u]); st(var + i, v[u]); st(p16 + i, o);
    }
}

// Vector body, fp16: the first moment is a 16-bit array as well.
template <int UNROLL>
__global__ __launch_bounds__(kAdamThreads) void adam_fp16_vec_kernel(
    int64_t nvec, f32x4 *__restrict__ p32, u32x2 *__restrict__ p16, const u32x2 *__restrict__ g16,
    u32x2 *__restrict__ mom, f32x4 *__restrict__ var, AdamHyper h, int32_t head, int32_t tail) {
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd, eps_s = h.eps * h.scale;
    if (blockIdx.x == 0 && (int)threadIdx.x < head + tail) {      // the elements around the vector body, one per lane
        const int64_t e = edge_element(nvec, head);
        float *p1 = (float *)p32 + e, *v1 = (float *)var + e;
        uint16_t *m1 = (uint16_t *)mom + e;
        float p = *p1, m = Half::to_f32(*m1), v = *v1;
        adam_elem_scaled(clip16<Half>(Half::to_f32(((const uint16_t *)g16)[e]), h.gcoef), m, v, p, h, omb1, omb2, lrwd, eps_s);
        *p1 = p; *m1 = Half::from_f32(m); *v1 = v; ((uint16_t *)p16)[e] = Half::from_f32(p);
    }
    const int64_t base = (int64_t)blockIdx.x * (kAdamThreads * UNROLL) + threadIdx.x;
    f32x4 p[UNROLL], v[UNROLL];
    u32x2 g[UNROLL], mh[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const int64_t i = base + (int64_t)u * kAdamThreads;
        ok[u] = i < nvec;
        if (ok[u]) { g[u] = ld(g16 + i); mh[u] = ld(mom + i); p[u] = ld(p32 + i); v[u] = ld(var + i); }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        if (!ok[u]) continue;
        const int64_t i = base + (int64_t)u * kAdamThreads;
        f32x4 mm;
        mm.x = lo_f32<Half>(mh[u].x); mm.y = hi_f32<Half>(mh[u].x);
        mm.z = lo_f32<Half>(mh[u].y); mm.w = hi_f32<Half>(mh[u].y);
        adam_group_scaled<Half>(g[u], mm, v[u], p[u], h, omb1, omb2, lrwd, eps_s);
        u32x2 o, mo;
        o.x = pack2<Half>(p[u].x, p[u].y);  o.y = pack2<Half>(p[u].z, p[u].w);
        mo.x = pack2<Half>(mm.x, mm.y); mo.y = pack2<Half>(mm.z, mm.w);
        st(p32 + i, p[u]); st(var + i, v[u]); st(mom + i, mo); st(p16 + i, o);
    }
}

// ---- long launches: a resident grid that streams ---------------------------------------------
// From kStreamMinVecBf16 / kStreamMinVecFp16 4-element groups on, the step runs as one workgroup of 256 lanes per compute
// unit that stays resident and works through tiles of 256 groups (4 KiB of each fp32 array, the
// granularity at which HBM channels interleave; tiles of other sizes measured up to 15 points
// slower).  What decides the rate of this 1:1 read/write stream is how narrow the window of
// addresses is that the whole chip touches at any moment, and how few bytes are in flight beyond
// what hides the latency:
//   * tiles are handed out by atomic tickets in the order in which workgroups ask for them, so
//     all compute units work within a few MiB of each other in every array (with tiles bound to
//     workgroup ids the eight XCDs drift apart);
//   * a same-address atomic takes about 11 ns on this part, which would cap a launch at one tile
//     per 11 ns; four counters in different 4 KiB blocks serve the tiles t = 4 * ticket + k
//     (k = 0..3; workgroup w uses counter (w / 8) % 4, so every XCD feeds every counter);
//   * each wave keeps exactly one tile of loads in flight while it computes and stores the one
//     before (software pipeline of depth 1, two register sets); deeper prefetch, more waves per
//     compute unit and larger tiles all measured slower;
//   * the ticket for the tile after the next is drawn one stage ahead by lane 0 and handed to
//     the workgroup through LDS, so nobody waits for the atomic's round trip.
// The compiler's own wait-count insertion cannot express this pipeline (it drains the loads that
// were just issued before the arithmetic starts), so the vector memory instructions of the loop
// and their waits are written by hand:  `s_waitcnt vmcnt(4)` right after the four loads of the
// next tile means "everything older has completed" — the current tile's data, the ticket drawn a
// stage ago, and the stores of the tile before — whatever the order in which loads, stores and
// atomics retire.  A 16-byte store is followed by `s_nop 1`: the instruction reads its data
// registers for two more cycles, and the compiler, which pads that hazard itself for stores it
// emits, does not see through an asm statement.
//
// Where the four counters live depends on the stream.  A stream that has an entry in the library's
// stream table (stream_slot_for, bmt_host.h) uses that entry's counters in the library's own device
// array: one kernel, the last workgroup to leave puts the counters back to zero.  Otherwise (a stream
// under graph capture, the per-thread default stream, a busy table; the multi-tensor kernel always)
// they live in the caller's 16-bit parameter output, the only memory of the call that the step never
// reads: word 0 of the 8-byte vectors nvec-1, nvec-513, nvec-1025 and nvec-1537.  A one-workgroup
// kernel in front zeroes them; the lanes that own those four groups step them like any other but do
// not store their 16-bit result; a one-workgroup kernel behind derives those four vectors from the
// fp32 parameters just written (the 16-bit copy is by definition the rounded fp32 value).  All three
// run on the caller's stream, so the ordering between the zeroing, the atomics (performed in memory,
// beyond the per-XCD L2s) and the final plain stores is that of kernel boundaries.  Measured, slot
// against output-hosted counters: bf16 12.6 M elements 73.6 / 72.3 % of peak, 16.8 M 77.6 / 76.1,
// 45 M 82.4 / 81.8, from 131 M on the same; 3.5 against 9.2 us of host time per call.
constexpr int kStreamThreads = 256;
constexpr int kStreamCounters = 4;
constexpr int64_t kStreamCounterStride = 512;            // in 8-byte vectors: 4 KiB
// Smallest launch (in 4-element groups) that runs as the resident grid, where it overtakes one workgroup per
// tile.  Measured per flavour, launches back to back, % of peak of one workgroup per tile / of the resident grid
// with the stream's own counters (a single kernel):
//   bf16    8.4 M elements 73.5 / 67.7;  10.5 M 73.6 / 74.4;  12.6 M 72.5 / 75.9;  16.8 M 73.5 / 78.7;  33.6 M 72.3 / 81.9
//   fp16   16.8 M 75.1 / 72.7;  21.0 M 75.5 / 74.1;  25.2 M 74.3 / 75.0;  33.6 M 76.3 / 77.2;  45 M 74.6 / 76.4;  202 M 72.8 / 80
// Multi-tensor batches keep their counters in a 16-bit output (three kernels) and change over a little later:
//   bf16   10.5 M: 71 either way;  12.6 M: 71.7 / 74.3;  14.7 M: 73.9 / 76.2
constexpr int64_t kStreamMinVecBf16 = (int64_t)5 << 19;        // 10,485,760 elements
constexpr int64_t kStreamMinVecFp16 = (int64_t)3 << 21;        // 25,165,824 elements
constexpr int64_t kStreamMultiMinVecBf16 = (int64_t)3 << 20;   // 12,582,912 elements
constexpr int64_t kStreamMultiMinVecFp16 = (int64_t)3 << 21;   // 25,165,824 elements

__device__ __forceinline__ bool holds_stream_counter(int64_t i, int64_t nvec) {
    const int64_t d = nvec - 1 - i;
    return (d & (kStreamCounterStride - 1)) == 0 && d < kStreamCounters * kStreamCounterStride;
}
// Every workgroup starts on two tiles it can name itself (see stream_first_tickets), so a ticket drawn from a
// counter (which starts at zero) counts from twice the number of workgroups that share the counter.
__global__ void adam_stream_reset_kernel(u32x2 *p16, int64_t nvec) {
    if (threadIdx.x < kStreamCounters) p16[nvec - 1 - threadIdx.x * kStreamCounterStride] = u32x2{0u, 0u};
}
// The grid of the resident kernels: one workgroup per compute unit, rounded down to a multiple of 32
// (8 XCDs x 4 counters), at least 32.
// The fp16 flavour moves fewer bytes per tile (its first moment is a 16-bit array) and runs 1 % faster with a
// quarter more workgroups (1.6 B elements: 81.3 % of peak with 320 workgroups, 80.1 % with 256, 80.6 % with 384, 78 % with
// 512); the bf16 flavour is fastest with exactly one per compute unit (84 %; 288: 82 %, 320: 81 %).
// With the counters taken in turn (launches of 2^31 elements or more) the fp16 flavour is fastest with two per compute
// unit (6.74 B elements: 83.7 % with 512 workgroups, 83.2 % with 320 or 384, 82.1 % with 256; bf16: 84.6 % with 256,
// 84.1 % with 288, 83.2 % with 512).
static unsigned stream_grid(bool fp16 = false, bool turns = false) {
    int cus = device_cu_count();
    if (fp16) cus += turns ? cus : cus / 4;
    return (unsigned)(cus >= 32 ? cus / 32 * 32 : 32);
}
// Workgroup b draws from counter (b / 8) % 4.  Its first two tickets need no atomic: it is workgroup number q
// among the gridDim / 4 that share the counter, and takes tickets q and q + gridDim / 4.
__device__ __forceinline__ void stream_first_tickets(int &which, uint32_t &t0, uint32_t &t1) {
    which = (int)((blockIdx.x >> 3) & (kStreamCounters - 1));
    const uint32_t q = ((blockIdx.x >> 5) << 3) | (blockIdx.x & 7u);
    t0 = q;
    t1 = q + (gridDim.x >> 2);
}
// A workgroup takes its tiles from the counters in turn (its own, the next one, ...), so that all counters are drawn
// from at the same rate whatever the pace of the single workgroups is.  With every workgroup on one counter of its
// own the four interleaved tile sequences drift apart over a long launch when some compute units run slower than
// others, the chip's window on the arrays widens, and launches over 6.74 B elements of a freshly allocated state took
// 27.65 to 28.7 ms (mean 28.05); in turn: 27.34 to 27.37 ms, every launch (86.2 % of the HBM peak against 84 %; 2.4 to
// 4.8 B elements: 87.5 against 85 %).  A counter's sequence only goes up, so a workgroup is done when it has met a tile
// past the end from every counter in a row.
// TURNS = false keeps every workgroup on its own counter (and lets it leave at its first tile past the end): launches
// below 2^31 elements, which are over before the sequences have drifted, run up to 2 % faster that way, and short ones
// save the three last draws (12.6 M elements: 3 to 5 %).
template <bool TURNS>
__device__ __forceinline__ int stream_next_counter(int c) { return TURNS ? (c + 1) & (kStreamCounters - 1) : c; }
constexpr int64_t kStreamTurnsMinVec = (int64_t)1 << 29;       // 2^31 elements

template <typename T>
__global__ void adam_stream_finish_kernel(const f32x4 *__restrict__ p32, u32x2 *__restrict__ p16, int64_t nvec) {
    if (threadIdx.x < kStreamCounters) {
        const int64_t i = nvec - 1 - threadIdx.x * kStreamCounterStride;
        const f32x4 p = p32[i];
        p16[i] = u32x2{pack2<T>(p.x, p.y), pack2<T>(p.z, p.w)};
    }
}

template <bool FP16> struct MomentVec { typedef f32x4 type; };
template <> struct MomentVec<true> { typedef u32x2 type; };
template <bool FP16>
struct StreamSet {
    f32x4 p, v;
    typename MomentVec<FP16>::type m;
    u32x2 g;
    int64_t i;      // group index of this lane in the tile
    bool ok;        // the group exists
};

// SLOT: the counters are a slot of the library's own array (stream_slot_for) instead of places in the 16-bit output;
// every group then stores its 16-bit result, nothing runs in front of or behind the kernel, and the last workgroup to
// leave puts the slot back (stream_slot_leave).
template <bool FP16, bool SLOT, bool TURNS>
__global__ __launch_bounds__(kStreamThreads) void adam_stream_kernel(
    int64_t nvec, int64_t ntiles, f32x4 *__restrict__ p32, u32x2 *__restrict__ p16, const u32x2 *__restrict__ g16,
    typename MomentVec<FP16>::type *__restrict__ mom, f32x4 *__restrict__ var, AdamHyper h, uint32_t *__restrict__ slot,
    uint32_t *__restrict__ done_word, uint32_t launch_number) {
    typedef StreamSet<FP16> Set;
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd, eps_s = h.eps * h.scale;
    __shared__ uint32_t handed[2];
    int which;
    uint32_t t0, t1;
    stream_first_tickets(which, t0, t1);
    auto counter_of = [&](int c) -> uint32_t * {
        return SLOT ? slot + c * 1024 : (uint32_t *)(p16 + (nvec - 1 - c * kStreamCounterStride));
    };
    const uint32_t drawn_base = gridDim.x >> 1;                       // two tickets per counter and workgroup of its group are taken already
    const int64_t first = (int64_t)t0 * kStreamCounters + which;
    int64_t ahead = (int64_t)t1 * kStreamCounters + stream_next_counter<TURNS>(which);   // the tile after the one in flight
    if (first >= ntiles) {
        if (SLOT) stream_slot_leave(slot, done_word, launch_number);
        return;
    }
    int drawing = stream_next_counter<TURNS>(stream_next_counter<TURNS>(which));    // counter of the ticket on its way
    uint32_t *const counter = counter_of(drawing);                    // TURNS = false: the only one
    uint32_t drawn = 0;                                               // lane 0: that ticket
    if (threadIdx.x == 0) stream_draw(drawn, counter);

    auto issue = [&](Set &s, int64_t tile) {
        s.i = tile * kStreamThreads + threadIdx.x;
        s.ok = tile < ntiles && s.i < nvec;
        const int64_t j = s.ok ? s.i : 0;          // lanes without a group load group 0 and drop it
        stream_load(s.g, g16 + j);
        stream_load(s.p, p32 + j);
        stream_load(s.m, mom + j);
        stream_load(s.v, var + j);
    };
    auto finish = [&](Set &s) {
        if (!s.ok) return;
        u32x2 o;
        if constexpr (FP16) {
            f32x4 mm = f32x4{lo_f32<Half>(s.m.x), hi_f32<Half>(s.m.x), lo_f32<Half>(s.m.y), hi_f32<Half>(s.m.y)};
            adam_group_scaled<Half>(s.g, mm, s.v, s.p, h, omb1, omb2, lrwd, eps_s);
            s.m = u32x2{pack2<Half>(mm.x, mm.y), pack2<Half>(mm.z, mm.w)};
            o = u32x2{pack2<Half>(s.p.x, s.p.y), pack2<Half>(s.p.z, s.p.w)};
        } else {
            adam_group_unscaled<BFloat16>(s.g, s.m, s.v, s.p, h, omb1, omb2, lrwd);
            o = u32x2{pack2<BFloat16>(s.p.x, s.p.y), pack2<BFloat16>(s.p.z, s.p.w)};
        }
        stream_store(p32 + s.i, s.p);
        stream_store(mom + s.i, s.m);
        stream_store(var + s.i, s.v);
        if (SLOT || !holds_stream_counter(s.i, nvec)) stream_store(p16 + s.i, o);
    };
    // One stage: the loads of the tile after `cur` go out, then `cur` is computed and stored.
    // Returns the tile whose loads went out.
    auto stage = [&](Set &cur, Set &next, int turn) -> int64_t {
        const int64_t tile = ahead;
        issue(next, tile);
        asm volatile("s_waitcnt vmcnt(4)" : "+v"(cur.g), "+v"(cur.p), "+v"(cur.m), "+v"(cur.v), "+v"(drawn));
        if (threadIdx.x == 0) handed[turn] = drawn;
        __syncthreads();
        if constexpr (TURNS) {
            ahead = (int64_t)(handed[turn] + drawn_base) * kStreamCounters + drawing;
            drawing = stream_next_counter<TURNS>(drawing);
            if (threadIdx.x == 0) stream_draw(drawn, counter_of(drawing));
        } else {
            ahead = (int64_t)(handed[turn] + drawn_base) * kStreamCounters + which;
            if (threadIdx.x == 0) stream_draw(drawn, counter);
        }
        finish(cur);
        return tile;
    };
    Set a, b;
    issue(a, first);
    if constexpr (TURNS) {
        int beyond = 0;  // tiles past the end in a row: one from every counter means that all counters have run out
        while (true) {
            beyond = stage(a, b, 0) >= ntiles ? beyond + 1 : 0;
            if (beyond == kStreamCounters) break;
            beyond = stage(b, a, 1) >= ntiles ? beyond + 1 : 0;
            if (beyond == kStreamCounters) break;
        }
    } else {
        while (true) {
            if (stage(a, b, 0) >= ntiles) break;
            if (stage(b, a, 1) >= ntiles) break;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");   // loads of the tile nobody owns, the last ticket
    if (SLOT) stream_slot_leave(slot, done_word, launch_number);
}

constexpr int kAdamScalarThreads = 256;
// Element-at-a-time kernels: the unaligned head/tail of a vectorised call, or the
// whole call when the five arrays do not share one alignment phase.
__global__ __launch_bounds__(kAdamScalarThreads) void adam_bf16_scalar_kernel(
    int64_t lo0, int64_t hi0, int64_t lo1, int64_t hi1, float *p32, uint16_t *p16, const uint16_t *g16,
    float *mom, float *var, AdamHyper h) {
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd;
    const int64_t n0 = hi0 - lo0, total = n0 + (hi1 - lo1);
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < total; k += (int64_t)gridDim.x * blockDim.x) {
        const int64_t i = k < n0 ? lo0 + k : lo1 + (k - n0);
        float p = p32[i], m = mom[i], v = var[i];
        adam_elem_unscaled(clip16<BFloat16>(BFloat16::to_f32(g16[i]), h.gcoef), m, v, p, h, omb1, omb2, lrwd);
        p32[i] = p; mom[i] = m; var[i] = v; p16[i] = BFloat16::from_f32(p);
    }
}
__global__ __launch_bounds__(kAdamScalarThreads) void adam_fp16_scalar_kernel(
    int64_t lo0, int64_t hi0, int64_t lo1, int64_t hi1, float *p32, uint16_t *p16, const uint16_t *g16,
    uint16_t *mom, float *var, AdamHyper h) {
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd, eps_s = h.eps * h.scale;
    const int64_t n0 = hi0 - lo0, total = n0 + (hi1 - lo1);
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < total; k += (int64_t)gridDim.x * blockDim.x) {
        const int64_t i = k < n0 ? lo0 + k : lo1 + (k - n0);
        float p = p32[i], m = Half::to_f32(mom[i]), v = var[i];
        adam_elem_scaled(clip16<Half>(Half::to_f32(g16[i]), h.gcoef), m, v, p, h, omb1, omb2, lrwd, eps_s);
        p32[i] = p; mom[i] = Half::from_f32(m); var[i] = v; p16[i] = Half::from_f32(p);
    }
}

constexpr int64_t kLineAlignMinVec = 4096;       // 16,384 elements: below that the head would be a visible share of the call
// Splits [0, n) into a scalar head, a vector body of 4-element groups and a scalar
// tail, given the addresses of the fp32 arrays (16-byte vectors) and the 16-bit
// arrays (8-byte vectors).  Returns false when the arrays do not share one phase.
static bool split_for_vectors(int64_t n, const uintptr_t *addr32, int n32, const uintptr_t *addr16, int n16,
                              int64_t resident_min_vec, int64_t *head, int64_t *nvec) {
    // Elements to skip until the address is vector-aligned; must agree across arrays.
    int64_t want = -1;
    for (int k = 0; k < n32; k++) {
        if (addr32[k] & 3u) return false;
        int64_t skip = (int64_t)(((16 - (addr32[k] & 15u)) & 15u) / 4);
        if (want < 0) want = skip; else if (want != skip) return false;
    }
    for (int k = 0; k < n16; k++) {
        if (addr16[k] & 1u) return false;
        int64_t skip = (int64_t)(((8 - (addr16[k] & 7u)) & 7u) / 2);
        if (want < 0) want = skip; else if (want != skip) return false;
    }
    if (want > n) want = n;
    // Tiles are 4 KiB blocks of the fp32 arrays (the granularity at which HBM channels interleave) counted from the
    // first group, so a body that starts off that grid makes every tile straddle two blocks: one transformer block
    // stepped through views 8 elements into its buffers runs at 77.5 % of peak, 256 elements in at 81.5 %, 1,024
    // elements in (on the grid again) at 84 %.  Calls that run as the resident grid therefore hand the elements up to
    // the fp32 parameters' next 4 KiB boundary (at most 1,023) to the element kernel as well; the step to that boundary
    // is the step to the next 16-byte boundary plus whole vectors, so it suits every array of the call.
    // The one-tile kernel of shorter calls only needs whole lines and would pay for the extra launch (2^23 elements,
    // 64 elements in: 72 % as it is, 67 % with the longer head).
    const int64_t to_grid = (int64_t)(((4096 - (addr32[0] & 4095u)) & 4095u) / 4);     // = want modulo 4
    // Shorter calls start their body on a 256-byte boundary of the fp32 parameters (a 128-byte line of the 16-bit
    // arrays; 2^23 elements reached through views 8 or 1,000 elements into their buffers: 65-67 % of peak as they
    // are, 72 % on the lines); the up to 63 elements in front are stepped by the vector kernel's first workgroup.
    const int64_t to_line = (int64_t)(((256 - (addr32[0] & 255u)) & 255u) / 4);        // = want modulo 4
    if (to_grid > want && (n - to_grid) / 4 >= resident_min_vec) want = to_grid;
    else if (to_line > want && (n - to_line) / 4 >= kLineAlignMinVec) want = to_line;
    *head = want;
    *nvec = (n - want) / 4;
    return true;
}

// Launches the vector body over [head, head + 4 * nvec) and, unless the vector launch has stepped them itself
// (it says so), the element kernel over what is left.
template <typename VecLaunch, typename ScalarLaunch>
static hipError_t launch_split(int64_t n, bool vectorisable, int64_t head, int64_t nvec, const VecLaunch &vec,
                               const ScalarLaunch &scalar) {
    if (!vectorisable) {
        const int64_t blocks = (n + kAdamScalarThreads - 1) / kAdamScalarThreads;
        const int64_t cap = (int64_t)device_cu_count() * 32;
        scalar((unsigned)(blocks < cap ? blocks : cap), (int64_t)0, n, (int64_t)0, (int64_t)0);
        return hipGetLastError();
    }
    if (nvec > 0) {
        const int64_t tile = (int64_t)kAdamThreads * kAdamUnroll;
        const int64_t ntiles = (nvec + tile - 1) / tile;
        if (ntiles > 0x7FFFFFFF) return hipErrorInvalidValue;
        const bool edges_done = vec((unsigned)ntiles, (int32_t)(head <= 1023 ? head : -1), (int32_t)(n - head - nvec * 4));
        hipError_t e = hipGetLastError();
        if (e != hipSuccess || edges_done) return e;
    }
    const int64_t tail_lo = head + nvec * 4;
    if (head > 0 || tail_lo < n) {
        scalar(1u, (int64_t)0, head, tail_lo, n);
        return hipGetLastError();
    }
    return hipSuccess;
}

// The 16-bit parameter array is output only and hosts the tile counters of long launches: it must not share
// memory with anything the step reads.
static bool overlaps(const void *a, int64_t a_bytes, const void *b, int64_t b_bytes) {
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a0 < b0 + (uintptr_t)b_bytes && b0 < a0 + (uintptr_t)a_bytes;
}
static bool output16_overlaps_input(int64_t n, const void *p16, const void *p32, const void *g, const void *m, int64_t m_size,
                                    const void *v) {
    return overlaps(p16, 2 * n, p32, 4 * n) || overlaps(p16, 2 * n, g, 2 * n) || overlaps(p16, 2 * n, m, m_size * n) ||
           overlaps(p16, 2 * n, v, 4 * n);
}

static hipError_t launch_bf16(int64_t n, float *p32, uint16_t *p16, const uint16_t *g, float *m, float *v,
                              const AdamHyper &h, hipStream_t s) {
    uintptr_t a32[3] = {(uintptr_t)p32, (uintptr_t)m, (uintptr_t)v};
    uintptr_t a16[2] = {(uintptr_t)p16, (uintptr_t)g};
    int64_t head = 0, nvec = 0;
    const bool vectorisable = split_for_vectors(n, a32, 3, a16, 2, kStreamMinVecBf16, &head, &nvec);
    return launch_split(
        n, vectorisable, head, nvec,
        [&](unsigned grid, int32_t head_elements, int32_t tail_elements) -> bool {
            u32x2 *out16 = (u32x2 *)(p16 + head);
            if (nvec >= kStreamMinVecBf16) {
                const int64_t ntiles = (nvec + kStreamThreads - 1) / kStreamThreads;
                StreamSlot slot;
                if (stream_slot_for(s, &slot, false)) {
                    auto kern = nvec >= kStreamTurnsMinVec ? adam_stream_kernel<false, true, true> : adam_stream_kernel<false, true, false>;
                    hipLaunchKernelGGL(kern, dim3(stream_grid()), dim3(kStreamThreads), 0, s, nvec,
                                       ntiles, (f32x4 *)(p32 + head), out16, (const u32x2 *)(g + head), (f32x4 *)(m + head),
                                       (f32x4 *)(v + head), h, slot.tickets, slot.done_word, slot.number);
                    return false;
                }
                hipLaunchKernelGGL(adam_stream_reset_kernel, dim3(1), dim3(64), 0, s, out16, nvec);
                auto hosted = nvec >= kStreamTurnsMinVec ? adam_stream_kernel<false, false, true> : adam_stream_kernel<false, false, false>;
                hipLaunchKernelGGL(hosted, dim3(stream_grid()), dim3(kStreamThreads), 0, s, nvec,
                                   ntiles, (f32x4 *)(p32 + head), out16, (const u32x2 *)(g + head), (f32x4 *)(m + head),
                                   (f32x4 *)(v + head), h, (uint32_t *)nullptr, (uint32_t *)nullptr, 0u);
                hipLaunchKernelGGL((adam_stream_finish_kernel<BFloat16>), dim3(1), dim3(64), 0, s, (const f32x4 *)(p32 + head),
                                   out16, nvec);
                return false;
            }
            const bool with_edges = head_elements >= 0 && head_elements + tail_elements <= kAdamThreads;
            hipLaunchKernelGGL((adam_bf16_vec_kernel<kAdamUnroll>), dim3(grid), dim3(kAdamThreads), 0, s, nvec,
                               (f32x4 *)(p32 + head), out16, (const u32x2 *)(g + head), (f32x4 *)(m + head),
                               (f32x4 *)(v + head), h, with_edges ? head_elements : 0, with_edges ? tail_elements : 0);
            return with_edges;
        },
        [&](unsigned grid, int64_t lo0, int64_t hi0, int64_t lo1, int64_t hi1) {
            hipLaunchKernelGGL(adam_bf16_scalar_kernel, dim3(grid), dim3(kAdamScalarThreads), 0, s, lo0, hi0, lo1, hi1,
                               p32, p16, g, m, v, h);
        });
}

static hipError_t launch_fp16(int64_t n, float *p32, uint16_t *p16, const uint16_t *g, uint16_t *m, float *v,
                              const AdamHyper &h, hipStream_t s) {
    uintptr_t a32[2] = {(uintptr_t)p32, (uintptr_t)v};
    uintptr_t a16[3] = {(uintptr_t)p16, (uintptr_t)g, (uintptr_t)m};
    int64_t head = 0, nvec = 0;
    const bool vectorisable = split_for_vectors(n, a32, 2, a16, 3, kStreamMinVecFp16, &head, &nvec);
    return launch_split(
        n, vectorisable, head, nvec,
        [&](unsigned grid, int32_t head_elements, int32_t tail_elements) -> bool {
            u32x2 *out16 = (u32x2 *)(p16 + head);
            if (nvec >= kStreamMinVecFp16) {
                const int64_t ntiles = (nvec + kStreamThreads - 1) / kStreamThreads;
                StreamSlot slot;
                if (stream_slot_for(s, &slot, false)) {
                    auto kern = nvec >= kStreamTurnsMinVec ? adam_stream_kernel<true, true, true> : adam_stream_kernel<true, true, false>;
                    hipLaunchKernelGGL(kern, dim3(stream_grid(true, nvec >= kStreamTurnsMinVec)), dim3(kStreamThreads), 0, s, nvec,
                                       ntiles, (f32x4 *)(p32 + head), out16, (const u32x2 *)(g + head), (u32x2 *)(m + head),
                                       (f32x4 *)(v + head), h, slot.tickets, slot.done_word, slot.number);
                    return false;
                }
                hipLaunchKernelGGL(adam_stream_reset_kernel, dim3(1), dim3(64), 0, s, out16, nvec);
                auto hosted = nvec >= kStreamTurnsMinVec ? adam_stream_kernel<true, false, true> : adam_stream_kernel<true, false, false>;
                hipLaunchKernelGGL(hosted, dim3(stream_grid(true, nvec >= kStreamTurnsMinVec)), dim3(kStreamThreads), 0, s, nvec,
                                   ntiles, (f32x4 *)(p32 + head), out16, (const u32x2 *)(g + head), (u32x2 *)(m + head),
                                   (f32x4 *)(v + head), h, (uint32_t *)nullptr, (uint32_t *)nullptr, 0u);
                hipLaunchKernelGGL((adam_stream_finish_kernel<Half>), dim3(1), dim3(64), 0, s, (const f32x4 *)(p32 + head),
                                   out16, nvec);
                return false;
            }
            const bool with_edges = head_elements >= 0 && head_elements + tail_elements <= kAdamThreads;
            hipLaunchKernelGGL((adam_fp16_vec_kernel<kAdamUnroll>), dim3(grid), dim3(kAdamThreads), 0, s, nvec,
                               (f32x4 *)(p32 + head), out16, (const u32x2 *)(g + head), (u32x2 *)(m + head),
                               (f32x4 *)(v + head), h, with_edges ? head_elements : 0, with_edges ? tail_elements : 0);
            return with_edges;
        },
        [&](unsigned grid, int64_t lo0, int64_t hi0, int64_t lo1, int64_t hi1) {
            hipLaunchKernelGGL(adam_fp16_scalar_kernel, dim3(grid), dim3(kAdamScalarThreads), 0, s, lo0, hi0, lo1, hi1,
                               p32, p16, g, m, v, h);
        });
}


// ---- several tensors in one launch ---------------------------------------------------------
// An optimizer steps one tensor per launch in the reference (adam.py:72-159); for models with
// many small tensors the launches, not the bytes, set the pace.  Up to kBatch tensors that share
// their hyper-parameters are described in the kernel argument itself (no device-side table to
// upload): workgroup b finds its tensor by scanning the running tile counts, then works on one
// tile of that tensor exactly as the single-tensor kernel does.  The last tile of a tensor also
// steps the up to three elements that do not fill a 4-element group.
constexpr int kBatch = 32;
struct AdamBatch {
    float *p32[kBatch];
    uint16_t *p16[kBatch];
    const uint16_t *g16[kBatch];
    void *mom[kBatch];          // float * (bf16 flavour) or uint16_t * (fp16 flavour)
    float *var[kBatch];
    int64_t n[kBatch];
    uint32_t first_tile[kBatch + 1];
    int32_t count;
    // long batches (adam_stream_multi_kernel): tiles of kStreamThreads groups, vector part of each tensor only
    uint32_t stream_first[kBatch + 1];
    int32_t counter_tensor;     // the tensor whose 16-bit output hosts the four tile counters
};

template <bool FP16>
__global__ __launch_bounds__(kAdamThreads) void adam_multi_kernel(AdamBatch batch, AdamHyper h) {
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd, eps_s = h.eps * h.scale;
    const uint32_t tile = blockIdx.x;
    int t = 0;
    while (t + 1 < batch.count && tile >= batch.first_tile[t + 1]) t++;
    const int64_t n = batch.n[t];
    const int64_t nvec = n / 4;
    const int64_t i = (int64_t)(tile - batch.first_tile[t]) * kAdamThreads + threadIdx.x;
    float *p32 = batch.p32[t];
    float *var = batch.var[t];
    uint16_t *p16 = batch.p16[t];
    const uint16_t *g16 = batch.g16[t];
    if (i < nvec) {
        u32x2 g = ld((const u32x2 *)g16 + i);
        f32x4 p = ld((const f32x4 *)p32 + i), v = ld((const f32x4 *)var + i), m;
        u32x2 o;
        if (FP16) {
            u32x2 mh = ld((const u32x2 *)batch.mom[t] + i);
            m = f32x4{lo_f32<Half>(mh.x), hi_f32<Half>(mh.x), lo_f32<Half>(mh.y), hi_f32<Half>(mh.y)};
            adam_group_scaled<Half>(g, m, v, p, h, omb1, omb2, lrwd, eps_s);
            st((u32x2 *)batch.mom[t] + i, u32x2{pack2<Half>(m.x, m.y), pack2<Half>(m.z, m.w)});
            o = u32x2{pack2<Half>(p.x, p.y), pack2<Half>(p.z, p.w)};
        } else {
            m = ld((const f32x4 *)batch.mom[t] + i);
            adam_group_unscaled<BFloat16>(g, m, v, p, h, omb1, omb2, lrwd);
            st((f32x4 *)batch.mom[t] + i, m);
            o = u32x2{pack2<BFloat16>(p.x, p.y), pack2<BFloat16>(p.z, p.w)};
        }
        st((f32x4 *)p32 + i, p); st((f32x4 *)var + i, v); st((u32x2 *)p16 + i, o);
    } else if (i - nvec < n - nvec * 4) {   // lanes right after the last group take the leftover elements
        const int64_t e = nvec * 4 + (i - nvec);
        float p = p32[e], v = var[e];
        if (FP16) {
            uint16_t *mom = (uint16_t *)batch.mom[t];
            float m = Half::to_f32(mom[e]);
            adam_elem_scaled(clip16<Half>(Half::to_f32(g16[e]), h.gcoef), m, v, p, h, omb1, omb2, lrwd, eps_s);
            mom[e] = Half::from_f32(m); p16[e] = Half::from_f32(p);
        } else {
            float *mom = (float *)batch.mom[t];
            float m = mom[e];
            adam_elem_unscaled(clip16<BFloat16>(BFloat16::to_f32(g16[e]), h.gcoef), m, v, p, h, omb1, omb2, lrwd);
            mom[e] = m; p16[e] = BFloat16::from_f32(p);
        }
        p32[e] = p; var[e] = v;
    }
}

// ---- long batches: the resident grid over several tensors ---------------------------------------
// The streaming scheme of adam_stream_kernel with the tile -> tensor mapping of adam_multi_kernel: tiles of
// kStreamThreads groups are numbered through the vector parts of all tensors of the batch
// (batch.stream_first), handed out by ticket, and each stage looks its tensor up in the kernel
// argument (the tile is uniform, so the look-up runs on the scalar unit).  The four counters live in the
// 16-bit output of batch.counter_tensor.  The elements that do not fill a 4-element group (up to three per
// tensor) and the four vectors that hosted the counters are finished by adam_stream_multi_finish_kernel.
template <bool FP16, bool TURNS>
__global__ __launch_bounds__(kStreamThreads) void adam_stream_multi_kernel(AdamBatch batch, AdamHyper h) {
    typedef typename MomentVec<FP16>::type mom_t;
    typedef StreamSet<FP16> Set;
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd, eps_s = h.eps * h.scale;
    __shared__ uint32_t handed[2];
    int which;
    uint32_t t0, t1;
    stream_first_tickets(which, t0, t1);
    const int64_t ntiles = batch.stream_first[batch.count];
    const int ct = batch.counter_tensor;
    const int64_t ct_nvec = batch.n[ct] / 4;
    auto counter_of = [&](int c) -> uint32_t * {
        return (uint32_t *)((u32x2 *)batch.p16[ct] + (ct_nvec - 1 - c * kStreamCounterStride));
    };
    const int64_t first = (int64_t)t0 * kStreamCounters + which;
    int64_t ahead = (int64_t)t1 * kStreamCounters + stream_next_counter<TURNS>(which);
    if (first >= ntiles) return;
    int drawing = stream_next_counter<TURNS>(stream_next_counter<TURNS>(which));    // counter of the ticket on its way
    uint32_t *const counter = counter_of(drawing);                    // TURNS = false: the only one
    uint32_t drawn = 0;
    if (threadIdx.x == 0) stream_draw(drawn, counter);

    // The tiles of a workgroup stay close to each other (the counters move together, and each of them only goes up),
    // so the tensor of a tile is found by walking from the tensor of the tile before, mostly not at all, and its
    // pointers are read from the kernel argument only when it changes; each register set remembers the pointers its
    // tile was loaded through.
    struct Where { float *p32; uint16_t *p16; const uint16_t *g16; void *mom; float *var; int64_t nvec; bool hosts_counters; };
    int t = 0;
    uint32_t t_first = 0, t_end = batch.stream_first[1];       // tensor t owns the tiles [t_first, t_end)
    auto where_of = [&](int k) {
        return Where{batch.p32[k], batch.p16[k], batch.g16[k], batch.mom[k], batch.var[k], batch.n[k] / 4, k == ct};
    };
    Where cur_where = where_of(0), wa = cur_where, wb = cur_where;
    auto issue = [&](Set &s, Where &w, int64_t tile_in) {
        const bool real = tile_in < ntiles;
        if (real) {
            const uint32_t tile = __builtin_amdgcn_readfirstlane((uint32_t)tile_in);
            bool moved = false;
            while (tile >= t_end) { t++; t_first = t_end; t_end = batch.stream_first[t + 1]; moved = true; }
            while (tile < t_first) { t--; t_end = t_first; t_first = batch.stream_first[t]; moved = true; }
            if (moved) cur_where = where_of(t);
            s.i = (int64_t)(tile - t_first) * kStreamThreads + threadIdx.x;
        } else {
            s.i = 0;
        }
        w = cur_where;
        s.ok = real && s.i < w.nvec;
        const int64_t j = s.ok ? s.i : 0;          // lanes without a group load group 0 of some tensor and drop it
        stream_load(s.g, (const u32x2 *)w.g16 + j);
        stream_load(s.p, (const f32x4 *)w.p32 + j);
        stream_load(s.m, (const mom_t *)w.mom + j);
        stream_load(s.v, (const f32x4 *)w.var + j);
    };
    auto finish = [&](Set &s, const Where &w) {
        if (!s.ok) return;
        u32x2 o;
        if constexpr (FP16) {
            f32x4 mm = f32x4{lo_f32<Half>(s.m.x), hi_f32<Half>(s.m.x), lo_f32<Half>(s.m.y), hi_f32<Half>(s.m.y)};
            adam_group_scaled<Half>(s.g, mm, s.v, s.p, h, omb1, omb2, lrwd, eps_s);
            s.m = u32x2{pack2<Half>(mm.x, mm.y), pack2<Half>(mm.z, mm.w)};
            o = u32x2{pack2<Half>(s.p.x, s.p.y), pack2<Half>(s.p.z, s.p.w)};
        } else {
            adam_group_unscaled<BFloat16>(s.g, s.m, s.v, s.p, h, omb1, omb2, lrwd);
            o = u32x2{pack2<BFloat16>(s.p.x, s.p.y), pack2<BFloat16>(s.p.z, s.p.w)};
        }
        stream_store((f32x4 *)w.p32 + s.i, s.p);
        stream_store((mom_t *)w.mom + s.i, s.m);
        stream_store((f32x4 *)w.var + s.i, s.v);
        if (!(w.hosts_counters && holds_stream_counter(s.i, ct_nvec))) stream_store((u32x2 *)w.p16 + s.i, o);
    };
    auto stage = [&](Set &cur, const Where &wcur, Set &next, Where &wnext, int slot) -> int64_t {
        const int64_t tile = ahead;
        issue(next, wnext, tile);
        asm volatile("s_waitcnt vmcnt(4)" : "+v"(cur.g), "+v"(cur.p), "+v"(cur.m), "+v"(cur.v), "+v"(drawn));
        if (threadIdx.x == 0) handed[slot] = drawn;
        __syncthreads();
        if constexpr (TURNS) {
            ahead = (int64_t)(handed[slot] + (gridDim.x >> 1)) * kStreamCounters + drawing;
            drawing = stream_next_counter<TURNS>(drawing);
            if (threadIdx.x == 0) stream_draw(drawn, counter_of(drawing));
        } else {
            ahead = (int64_t)(handed[slot] + (gridDim.x >> 1)) * kStreamCounters + which;
            if (threadIdx.x == 0) stream_draw(drawn, counter);
        }
        finish(cur, wcur);
        return tile;
    };
    Set a, b;
    issue(a, wa, first);
    if constexpr (TURNS) {
        int beyond = 0;  // see adam_stream_kernel
        while (true) {
            beyond = stage(a, wa, b, wb, 0) >= ntiles ? beyond + 1 : 0;
            if (beyond == kStreamCounters) break;
            beyond = stage(b, wb, a, wa, 1) >= ntiles ? beyond + 1 : 0;
            if (beyond == kStreamCounters) break;
        }
    } else {
        while (true) {
            if (stage(a, wa, b, wb, 0) >= ntiles) break;
            if (stage(b, wb, a, wa, 1) >= ntiles) break;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
}

// One workgroup: lanes 0..3 write the four 16-bit vectors that hosted the counters (from the fp32 parameters
// just written); lane 4 * t + k steps leftover element k of tensor t.
template <bool FP16>
__global__ __launch_bounds__(4 * kBatch + 64) void adam_stream_multi_finish_kernel(AdamBatch batch, AdamHyper h) {
    typedef typename std::conditional<FP16, Half, BFloat16>::type T;
    const float omb1 = 1.0f - h.b1, omb2 = 1.0f - h.b2, lrwd = h.lr * h.wd, eps_s = h.eps * h.scale;
    const int lane = threadIdx.x;
    if (lane < kStreamCounters) {
        const int ct = batch.counter_tensor;
        const int64_t i = batch.n[ct] / 4 - 1 - lane * kStreamCounterStride;
        const f32x4 p = ((const f32x4 *)batch.p32[ct])[i];
        ((u32x2 *)batch.p16[ct])[i] = u32x2{pack2<T>(p.x, p.y), pack2<T>(p.z, p.w)};
    }
    const int t = (lane - 64) / 4, k = (lane - 64) % 4;
    if (lane >= 64 && t < batch.count) {
        const int64_t n = batch.n[t], e = (n / 4) * 4 + k;
        if (e < n) {
            float *p32 = batch.p32[t], *var = batch.var[t];
            uint16_t *p16 = batch.p16[t];
            const uint16_t *g16 = batch.g16[t];
            float p = p32[e], v = var[e];
            if (FP16) {
                uint16_t *mom = (uint16_t *)batch.mom[t];
                float m = Half::to_f32(mom[e]);
                adam_elem_scaled(clip16<Half>(Half::to_f32(g16[e]), h.gcoef), m, v, p, h, omb1, omb2, lrwd, eps_s);
                mom[e] = Half::from_f32(m); p16[e] = Half::from_f32(p);
            } else {
                float *mom = (float *)batch.mom[t];
                float m = mom[e];
                adam_elem_unscaled(clip16<BFloat16>(BFloat16::to_f32(g16[e]), h.gcoef), m, v, p, h, omb1, omb2, lrwd);
                mom[e] = m; p16[e] = BFloat16::from_f32(p);
            }
            p32[e] = p; var[e] = v;
        }
    }
}

// Tiles of one tensor: its 4-element groups plus one lane per leftover element.
static int64_t multi_tiles(int64_t n) { return (n / 4 + (n % 4) + kAdamThreads - 1) / kAdamThreads; }

template <bool FP16>
static int adam_multi(int32_t count, const bmt_adam_tensor *tensors, const AdamHyper &h, hipStream_t s, const char *who) {
    if (count <= 0) return 0;
    if (!tensors) return fail(-1, "adam multi launcher: null tensor table");
    // The whole table is checked before the first launch, so that an error status means nothing was stepped.
    for (int32_t k = 0; k < count; k++) {
        const bmt_adam_tensor &t = tensors[k];
        if (t.n <= 0) continue;
        if (!t.param_fp32 || !t.param_16 || !t.grad_16 || !t.m || !t.v) return fail(-1, "adam multi launcher: null pointer");
        if (output16_overlaps_input(t.n, t.param_16, t.param_fp32, t.grad_16, t.m, FP16 ? 2 : 4, t.v))
            return fail(-1, "adam multi launcher: param_16 overlaps an input array");
    }
    AdamBatch batch;
    auto flush = [&]() -> hipError_t {
        if (batch.count == 0) return hipSuccess;
        const uint32_t tiles = batch.first_tile[batch.count];
        // Batches of kStreamMultiMinVec* groups or more run as the resident grid; the tensor with the most groups (at
        // least 3 * 2^20 / 32 of them, so the four counter places exist) lends its 16-bit output to the counters.
        int64_t groups = 0, most = -1;
        batch.stream_first[0] = 0;
        batch.counter_tensor = 0;
        for (int c = 0; c < batch.count; c++) {
            const int64_t nvec = batch.n[c] / 4;
            groups += nvec;
            if (nvec > most) { most = nvec; batch.counter_tensor = c; }
            batch.stream_first[c + 1] = batch.stream_first[c] + (uint32_t)((nvec + kStreamThreads - 1) / kStreamThreads);
        }
        // The counters occupy the last kStreamCounters * kStreamCounterStride 8-byte vectors of that output while the
        // launch runs: no array of any other tensor of the batch may share that memory (a table that names one
        // tensor twice, say).  Such a batch takes the workgroup-per-tile kernel, which keeps no counters.
        bool counters_clear = true;
        {
            const int ct = batch.counter_tensor;
            const int64_t span = kStreamCounters * kStreamCounterStride < most ? kStreamCounters * kStreamCounterStride : most;
            const char *lo = (const char *)batch.p16[ct] + (most - span) * 8;
            for (int c = 0; c < batch.count && counters_clear; c++) {
                if (c == ct) continue;
                const int64_t nc = batch.n[c];
                counters_clear = !overlaps(lo, span * 8, batch.p32[c], 4 * nc) && !overlaps(lo, span * 8, batch.g16[c], 2 * nc) &&
                                 !overlaps(lo, span * 8, batch.mom[c], (FP16 ? 2 : 4) * nc) && !overlaps(lo, span * 8, batch.var[c], 4 * nc) &&
                                 !overlaps(lo, span * 8, batch.p16[c], 2 * nc);
            }
        }
        if (counters_clear && groups >= (FP16 ? kStreamMultiMinVecFp16 : kStreamMultiMinVecBf16)) {
            hipLaunchKernelGGL(adam_stream_reset_kernel, dim3(1), dim3(64), 0, s, (u32x2 *)batch.p16[batch.counter_tensor], most);
            auto resident = groups >= kStreamTurnsMinVec ? adam_stream_multi_kernel<FP16, true> : adam_stream_multi_kernel<FP16, false>;
            hipLaunchKernelGGL(resident, dim3(stream_grid(FP16, groups >= kStreamTurnsMinVec)), dim3(kStreamThreads), 0, s, batch, h);
            hipLaunchKernelGGL((adam_stream_multi_finish_kernel<FP16>), dim3(1), dim3(4 * kBatch + 64), 0, s, batch, h);
        } else {
            hipLaunchKernelGGL((adam_multi_kernel<FP16>), dim3(tiles), dim3(kAdamThreads), 0, s, batch, h);
        }
        batch.count = 0;
        batch.first_tile[0] = 0;
        return hipGetLastError();
    };
    batch.count = 0;
    batch.first_tile[0] = 0;
    for (int32_t k = 0; k < count; k++) {
        const bmt_adam_tensor &t = tensors[k];
        if (t.n <= 0) continue;
        const bool aligned = (((uintptr_t)t.param_fp32 | (uintptr_t)t.v | (FP16 ? 0 : (uintptr_t)t.m)) & 15u) == 0 &&
                             (((uintptr_t)t.param_16 | (uintptr_t)t.grad_16 | (FP16 ? (uintptr_t)t.m : 0)) & 7u) == 0;
        const int64_t tiles = multi_tiles(t.n);
        if (!aligned || tiles > 0x0FFFFFFF) {
            // tensors the batch kernel does not take (unaligned views, gigantic buffers) go alone
            hipError_t e = FP16 ? launch_fp16(t.n, (float *)t.param_fp32, (uint16_t *)t.param_16, (const uint16_t *)t.grad_16,
                                              (uint16_t *)t.m, (float *)t.v, h, s)
                                : launch_bf16(t.n, (float *)t.param_fp32, (uint16_t *)t.param_16, (const uint16_t *)t.grad_16,
                                              (float *)t.m, (float *)t.v, h, s);
            if (e != hipSuccess) return fail((int)e, who, e);
            continue;
        }
        if (batch.count == kBatch || (int64_t)batch.first_tile[batch.count] + tiles > 0x0FFFFFFF) {
            hipError_t e = flush();
            if (e != hipSuccess) return fail((int)e, who, e);
        }
        const int c = batch.count;
        batch.p32[c] = (float *)t.param_fp32; batch.p16[c] = (uint16_t *)t.param_16; batch.g16[c] = (const uint16_t *)t.grad_16;
        batch.mom[c] = t.m; batch.var[c] = (float *)t.v; batch.n[c] = t.n;
        batch.first_tile[c + 1] = batch.first_tile[c] + (uint32_t)tiles;
        batch.count = c + 1;
    }
    hipError_t e = flush();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}

}  // namespace bmt

using namespace bmt;

extern "C" int adam_bf16_launcher(int64_t n, void *param_fp32, void *param_bf16, const void *g_bf16, void *m_fp32,
                                  void *v_fp32, float beta1, float beta2, float eps, float lr, float scale,
                                  float weight_decay, float bias_correction1, float bias_correction2, void *stream) {
    if (n <= 0) return 0;  // adam_cuda.cu:118
    if (!param_fp32 || !param_bf16 || !g_bf16 || !m_fp32 || !v_fp32) return fail(-1, "adam_bf16_launcher: null pointer");
    if (output16_overlaps_input(n, param_bf16, param_fp32, g_bf16, m_fp32, 4, v_fp32))
        return fail(-1, "adam_bf16_launcher: param_bf16 overlaps an input array");
    AdamHyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2};
    hipError_t e = launch_bf16(n, (float *)param_fp32, (uint16_t *)param_bf16, (const uint16_t *)g_bf16, (float *)m_fp32,
                               (float *)v_fp32, h, (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail((int)e, "adam_bf16_launcher", e);
}

extern "C" int adam_fp16_launcher(int64_t n, void *param_fp32, void *param_fp16, const void *g_fp16, void *m_fp16,
                                  void *v_fp32, float beta1, float beta2, float eps, float lr, float scale,
                                  float weight_decay, float bias_correction1, float bias_correction2, void *stream) {
    if (n <= 0) return 0;  // adam_cuda.cu:91
    if (!param_fp32 || !param_fp16 || !g_fp16 || !m_fp16 || !v_fp32) return fail(-1, "adam_fp16_launcher: null pointer");
    if (output16_overlaps_input(n, param_fp16, param_fp32, g_fp16, m_fp16, 2, v_fp32))
        return fail(-1, "adam_fp16_launcher: param_fp16 overlaps an input array");
    AdamHyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2};
    hipError_t e = launch_fp16(n, (float *)param_fp32, (uint16_t *)param_fp16, (const uint16_t *)g_fp16,
                                  (uint16_t *)m_fp16, (float *)v_fp32, h, (hipStream_t)stream);
    return e == hipSuccess ? 0 : fail((int)e, "adam_fp16_launcher", e);
}

extern "C" int adam_bf16_multi_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2, float eps,
                                        float lr, float scale, float weight_decay, float bias_correction1,
                                        float bias_correction2, void *stream) {
    AdamHyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2};
    return adam_multi<false>(count, tensors, h, (hipStream_t)stream, "adam_bf16_multi_launcher");
}
extern "C" int adam_fp16_multi_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2, float eps,
                                        float lr, float scale, float weight_decay, float bias_correction1,
                                        float bias_correction2, void *stream) {
    AdamHyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2};
    return adam_multi<true>(count, tensors, h, (hipStream_t)stream, "adam_fp16_multi_launcher");
}

extern "C" int adam_bf16_multi_clip_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2,
                                             float eps, float lr, float scale, float weight_decay,
                                             float bias_correction1, float bias_correction2, float grad_coef,
                                             void *stream) {
    AdamHyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2, grad_coef};
    return adam_multi<false>(count, tensors, h, (hipStream_t)stream, "adam_bf16_multi_clip_launcher");
}
extern "C" int adam_fp16_multi_clip_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2,
                                             float eps, float lr, float scale, float weight_decay,
                                             float bias_correction1, float bias_correction2, float grad_coef,
                                             void *stream) {
    AdamHyper h{beta1, beta2, eps, lr, scale, weight_decay, bias_correction1, bias_correction2, grad_coef};
    return adam_multi<true>(count, tensors, h, (hipStream_t)stream, "adam_fp16_multi_clip_launcher");
}
