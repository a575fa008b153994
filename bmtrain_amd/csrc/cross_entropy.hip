// Fused cross-entropy forward / in-place backward for gfx950 (MI355X), plus the two
// row helpers used by the vocabulary-parallel loss.  Replaces
// csrc/cuda/cross_entropy.cu of the reference.
//
// Forward (reference kernels :9-43, :63-101) per row r of the [m, n] logits:
//   M = max(max_i x_i, -1e6);  S = sum_i expf(x_i - M) + 1e-10
//   softmax[r, i] = to16(expf(x_i - M) / S)
//   out[r] = target[r] != ignore ? (-x[target[r]] + M) + logf(S) : 0
// The reference walks each row three times from global memory.  Here rows move as 16-byte
// vectors; rows of up to 512 elements share a wave (ce_forward_small_kernel), longer ones get a
// workgroup each:
//   * up to 32,768 elements the row is read once into registers; maximum, exponentials (kept in
//     fp32 registers), sum and quotient all work on registers (ce_forward_row_kernel);
//   * longer rows are streamed once while a per-lane running maximum / sum is kept; 4 vectors
//     per lane stay in registers and up to 4 in LDS (65,536 elements), the remainder is fetched a
//     second time for the output sweep (ce_forward_retain_kernel).
// Reductions are a wave64 butterfly followed by one LDS slot per wave.  Rows may have any length
// and start at any 2-byte offset: each row is split into a head of fewer than 8 elements, whole
// 16-byte vectors and a tail (RowSpan).  Only when logits and softmax sit at different offsets
// from a 16-byte boundary does a three-sweep kernel with element loads take over
// (ce_forward_sweep_kernel).
//
// Backward (reference kernels :46-60, :104-121), element-wise and in place on the
// stored softmax: x[r, i] = to16((x[r, i] - (i == target[r])) * grad_output[r]).
#include <atomic>
#include <mutex>
#include "bmt_device.h"
#include "bmt_host.h"
#include "../../include/bmt_hip.h"

namespace bmt {

template <typename T> __device__ __forceinline__ uint32_t neg_inf2();
template <> __device__ __forceinline__ uint32_t neg_inf2<Half>() { return 0xFC00FC00u; }
template <> __device__ __forceinline__ uint32_t neg_inf2<BFloat16>() { return 0xFF80FF80u; }

__device__ __forceinline__ float add_tiny(float s) { return (float)((double)s + 1e-10); }  // cross_entropy.cu:28

// ---- exponentials and the quotient -------------------------------------------------
// All exponentials here are e^(x - M) with x <= M.  They are produced multiplied by 2^16
// ("biased"): v_exp_f32 returns 0 for results below 2^-126, and the bias keeps everything that
// can still matter after the division in the normal range — the smallest quotient a 16-bit
// output can hold is 2^-134 (half the least bf16 subnormal), and with a divisor of at least 1 its
// exponential is at least 2^-134, biased 2^-118.  The factor is removed again, exactly, by the
// reciprocal used for the quotient.
//
// The forward kernels are close to ALU-bound (a v_exp_f32 costs four issue slots and every
// element needs one or two), so the exponential is three instructions and the quotient one.
// Errors stay far below half an ulp of the 16-bit result.  The largest is the one rounding of
// (x - M) * log2(e) + 16, half an ulp of a number between -16 and 16, i.e. 2^-21 to 2^-23 for most
// elements (which is why the bias is no larger than it has to be: with 64 in its place that
// rounding alone was 2^-19, and the stored softmax differed from a libm-based evaluation on 1.4 to
// 1.8 elements in 10,000; now 0.3 to 0.4); then 2^-22 from v_exp_f32, 2^-23 from the reciprocal and
// the product.
constexpr float kLog2e = 1.44269502162933349609375f;       // fp32 nearest to log2(e)
constexpr int kBiasLog2 = 16;
constexpr float kBias = (float)kBiasLog2;
constexpr float kTwoPowMinusBias = 1.0f / (float)(1 << kBiasLog2);   // 2^-16, exact

// 2^16 * e^(x - M).  The difference is formed first (folding M into the constant would save an
// instruction, but rounds 16 - M * log2(e) to an error that grows with |M| and overflows for huge
// M); x = -inf gives 0, NaN gives NaN.
__device__ __forceinline__ float exp_biased(float x, float M) {
    return __builtin_amdgcn_exp2f(__builtin_fmaf(x - M, kLog2e, kBias));
}
// The row's divisor in the two forms the kernels need.
struct RowSum {
    float S;      // sum of exponentials + 1e-10, unbiased (for the loss)
    float scaled_reciprocal;    // 2^-16 / S: multiplying a biased exponential by it gives the softmax value
};
__device__ __forceinline__ RowSum make_row_sum(float biased_sum) {
    RowSum rs;
    rs.S = add_tiny(biased_sum * kTwoPowMinusBias);
    rs.scaled_reciprocal = (1.0f / rs.S) * kTwoPowMinusBias;
    return rs;
}
__device__ __forceinline__ float quotient(float e_biased, const RowSum &rs) { return e_biased * rs.scaled_reciprocal; }

// Loss of one row; an out-of-range target that is not ignore_index yields NaN instead
// of the reference's out-of-bounds read.
template <typename T>
__device__ __forceinline__ float row_loss(const uint16_t *row, int32_t n, int32_t t, int32_t ignore_index, float M,
                                          float S) {
    if (t == ignore_index) return 0.f;
    if (t < 0 || t >= n) return __builtin_nanf("");
    return (-T::to_f32(row[t]) + M) + logf(S);
}

// How one row splits into 16-byte vectors.  A row may start anywhere (rows of odd length start at
// every 2-byte offset in turn): `head` elements before the first boundary, whole vectors, up to 7
// elements after the last one.  The edge elements are handled by the first lanes of the workgroup,
// one element each, next to their share of the vectors.
//
// The boundary is a 16-byte one (`align` = 8 elements, at most 14 edge elements) or, in the kernels with
// 256 lanes or more, a 128-byte one (`align` = 64, at most 70 edge elements): a wave then loads and stores
// whole 128-byte lines.  Rows whose length is not a multiple of 64 elements start off the line grid, and a
// workgroup that reads such a row and then writes it reaches 66 % of peak with vectors placed from the first
// 16-byte boundary and 72 % with vectors placed from the first line boundary (bare access pattern, rows of
// 256 KB; aligned rows: 72 %).  The launcher says which rows use it and what it measures on the kernels.
struct RowSpan {
    const uint16_t *row;   // first element of the row
    int32_t head;          // elements before the first vector
    int32_t nvec;          // whole vectors
    int32_t nedge;         // head + tail elements
    __device__ __forceinline__ int32_t edge_index(int lane) const {   // lane < nedge
        return lane < head ? lane : head + 8 * nvec + (lane - head);
    }
};
__device__ __forceinline__ RowSpan row_span(const uint16_t *x, int64_t row, int32_t n, uint32_t align = 8u) {
    RowSpan sp;
    sp.row = x + row * n;
    sp.head = (int32_t)((align - (uint32_t)(((uintptr_t)sp.row >> 1) & (align - 1u))) & (align - 1u));
    if (sp.head > n) sp.head = n;
    sp.nvec = (n - sp.head) >> 3;
    sp.nedge = n - 8 * sp.nvec;
    return sp;
}

// The row of workgroup b when every XCD is to work on its own run of consecutive rows.  Workgroups are handed to
// the eight XCDs in turn (b % 8), so XCD k takes the k-th eighth of the rows, in order; the rows past the last
// multiple of eight keep their index.  This is a choice of order only: every row is still processed exactly once
// whatever the hardware's placement is.  Measured on rows of 32 to 64 KiB (one workgroup of 1024 lanes reading its
// row and then writing it): 68-74 % of peak with row = b, 77-79 % with this order; rows of 16 KiB or less lose 2-4
// points and rows beyond 80 KiB gain or lose about one, so only the 1024-lane register-resident kernels use it.
__device__ __forceinline__ int64_t xcd_contiguous_row(uint32_t b, uint32_t rows) {
    const uint32_t whole = rows & ~7u;
    return b < whole ? (int64_t)(b & 7u) * (whole >> 3) + (b >> 3) : (int64_t)b;
}

// The same idea in runs: XCD k works through 128 consecutive rows, then through the 128 rows that lie 1,024 further
// on.  This is the order of the long-row kernel.  Measured against row = b, alternating in one process, on arrays of
// 2^29 elements with rows of 36,864 to 151,936 classes: runs of 32, 64 and 128 rows are 2 % faster on average (65,536
// classes: 2.8 %, 98,304: 5 to 6 %, 151,936: 2 to 3 %; never more than 1 % slower); at 8,192 x 128,256 runs of 128 are
// 0.7 % faster (0.7453 against 0.7505 ms; runs of 32: 0.7515, of 64: 0.7484), runs of 8 are 1.3 % slower.  One run per
// XCD for the whole launch, as above, is ahead at some lengths and up to 4 % behind at others.
constexpr uint32_t kXcdRunRows = 128;
__device__ __forceinline__ int64_t xcd_run_row(uint32_t b, uint32_t rows) {
    const uint32_t whole = rows / (8u * kXcdRunRows) * (8u * kXcdRunRows);
    if (b >= whole) return (int64_t)b;
    const uint32_t xcd = b & 7u, turn = b >> 3;
    return (int64_t)(turn / kXcdRunRows) * (8u * kXcdRunRows) + xcd * kXcdRunRows + (turn % kXcdRunRows);
}

// ---- forward, register-resident row ------------------------------------------
// One workgroup of THREADS lanes per row; lane t owns vectors t, t+THREADS, ...
// (CHUNKS of them, 8 elements each).  The 8*CHUNKS exponentials of a lane stay in fp32
// registers between the sum and the quotient: one exponential per element.
template <typename T, int THREADS, int CHUNKS>
__global__ __launch_bounds__(THREADS) void ce_forward_row_kernel(
    int32_t n, const uint16_t *__restrict__ x, const int32_t *__restrict__ target,
    uint16_t *__restrict__ softmax, float *__restrict__ out, int32_t ignore_index, uint32_t align) {
    __shared__ float slots[2][THREADS / kWave];
    const int64_t row = THREADS == 1024 ? xcd_contiguous_row(blockIdx.x, gridDim.x) : (int64_t)blockIdx.x;
    const RowSpan sp = row_span(x, row, n, THREADS >= 256 ? align : 8u);
    const int32_t nvec = sp.nvec;
    const u32x4 *xr = (const u32x4 *)(sp.row + sp.head);
    uint16_t *srow = softmax + row * n;
    u32x4 *sr = (u32x4 *)(srow + sp.head);
    const int tid = threadIdx.x;

    u32x4 w[CHUNKS];
    const uint32_t pad = neg_inf2<T>();
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
        const int j = c * THREADS + tid;
        if (j < nvec) w[c] = __builtin_nontemporal_load(xr + j);
        else { w[c].x = pad; w[c].y = pad; w[c].z = pad; w[c].w = pad; }
    }

    // Lanes past the end of the row skip the arithmetic (whole waves do, when the row is much
    // shorter than the launch shape's capacity): these kernels are close to ALU-bound.
    float mx = -INFINITY;
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
        if (c * THREADS + tid < nvec) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                mx = fmaxf(lo_f32<T>(w[c][k]), mx);
                mx = fmaxf(hi_f32<T>(w[c][k]), mx);
            }
        }
    }
    float edge = -INFINITY;
    if (tid < sp.nedge) {
        edge = T::to_f32(sp.row[sp.edge_index(tid)]);
        mx = fmaxf(edge, mx);
    }
    const float M = fmaxf(block_allreduce<true>(mx, slots[0]), -1e6f);

    float e[CHUNKS][8];
    float sum = 0.f;
    if (tid < sp.nedge) {
        edge = exp_biased(edge, M);
        sum = edge;
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
        if (c * THREADS + tid < nvec) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                e[c][2 * k] = exp_biased(lo_f32<T>(w[c][k]), M);
                e[c][2 * k + 1] = exp_biased(hi_f32<T>(w[c][k]), M);
                sum += e[c][2 * k];
                sum += e[c][2 * k + 1];
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) e[c][k] = 0.f;
        }
    }
    const RowSum rs = make_row_sum(block_allreduce<false>(sum, slots[1]));

#pragma unroll
    for (int c = 0; c < CHUNKS; c++) {
        const int j = c * THREADS + tid;
        if (j < nvec) {
            u32x4 o;
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = pack2<T>(quotient(e[c][2 * k], rs), quotient(e[c][2 * k + 1], rs));
            __builtin_nontemporal_store(o, sr + j);
        }
    }
    if (tid < sp.nedge) srow[sp.edge_index(tid)] = T::from_f32(quotient(edge, rs));
    if (tid == 0) out[row] = row_loss<T>(sp.row, n, target[row], ignore_index, M, rs.S);
}

// ---- helpers on one 16-byte vector (8 elements) ------------------------------------------
// Returns `w` through an empty asm: the compiler then cannot keep the unpacked fp32 values of
// one sweep alive for the next one, which would double the registers a resident row occupies.
__device__ __forceinline__ u32x4 reread(u32x4 w) {
    asm volatile("" : "+v"(w));
    return w;
}

template <typename T>
__device__ __forceinline__ void vec_max(const u32x4 &w, float &mx) {
#pragma unroll
    for (int k = 0; k < 4; k++) { mx = fmaxf(lo_f32<T>(w[k]), mx); mx = fmaxf(hi_f32<T>(w[k]), mx); }
}
template <typename T>
__device__ __forceinline__ void vec_sumexp(const u32x4 &w, float m, float &sum) {
#pragma unroll
    for (int k = 0; k < 4; k++) { sum += exp_biased(lo_f32<T>(w[k]), m); sum += exp_biased(hi_f32<T>(w[k]), m); }
}
template <typename T>
__device__ __forceinline__ u32x4 vec_softmax(const u32x4 &w, float M, const RowSum &rs) {
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; k++)
        o[k] = pack2<T>(quotient(exp_biased(lo_f32<T>(w[k]), M), rs), quotient(exp_biased(hi_f32<T>(w[k]), M), rs));
    return o;
}

// ---- forward, short rows ---------------------------------------------------------------
// Rows of up to 64 vectors.  LANES (8..64) adjacent lanes own one row, one vector per lane, so a
// wave holds 64 / LANES rows side by side; it works on R such sets at once, with all loads issued
// first (a single 1 KiB row per wave in flight would leave HBM idle).  Reductions are butterflies
// inside the lane group; no LDS, no barriers.  256 lanes per workgroup.
constexpr int kSmallThreads = 256;
template <int LANES, bool IsMax>
__device__ __forceinline__ float group_allreduce(float v) {
#pragma unroll
    for (int off = LANES / 2; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off, kWave);
        v = IsMax ? fmaxf(v, o) : v + o;
    }
    return v;
}
template <typename T, int LANES, int R>
__global__ __launch_bounds__(kSmallThreads) void ce_forward_small_kernel(
    int32_t m, int32_t n, const uint16_t *__restrict__ x, const int32_t *__restrict__ target,
    uint16_t *__restrict__ softmax, float *__restrict__ out, int32_t ignore_index) {
    constexpr int GROUPS = kWave / LANES;                          // rows side by side in a wave
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane & (LANES - 1);                            // lane inside its row
    const int64_t wave_id = (int64_t)blockIdx.x * (kSmallThreads / kWave) + threadIdx.x / kWave;
    const int64_t row0 = wave_id * (R * GROUPS) + lane / LANES;     // set r covers rows row0 + r * GROUPS

    RowSpan sp[R];
    u32x4 w[R];
    bool live[R];                                                  // this lane holds a vector of its row
    const uint32_t pad = neg_inf2<T>();
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int64_t row = row0 + (int64_t)r * GROUPS;
        const bool row_ok = row < m;
        sp[r] = row_span(x, row_ok ? row : 0, n);
        if (!row_ok) { sp[r].nvec = 0; sp[r].nedge = 0; }
        live[r] = sub < sp[r].nvec;
        if (live[r]) w[r] = __builtin_nontemporal_load((const u32x4 *)(sp[r].row + sp[r].head) + sub);
        else { w[r].x = pad; w[r].y = pad; w[r].z = pad; w[r].w = pad; }
    }
    float M[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float mx = -INFINITY;
        if (live[r]) vec_max<T>(w[r], mx);
        for (int e = sub; e < sp[r].nedge; e += LANES) mx = fmaxf(T::to_f32(sp[r].row[sp[r].edge_index(e)]), mx);
        M[r] = fmaxf(group_allreduce<LANES, true>(mx), -1e6f);
    }
    float ex[R][8];
    RowSum rs[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float sum = 0.f;
        if (live[r]) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                ex[r][2 * k] = exp_biased(lo_f32<T>(w[r][k]), M[r]);
                ex[r][2 * k + 1] = exp_biased(hi_f32<T>(w[r][k]), M[r]);
                sum += ex[r][2 * k];
                sum += ex[r][2 * k + 1];
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) ex[r][k] = 0.f;
        }
        for (int e = sub; e < sp[r].nedge; e += LANES) sum += exp_biased(T::to_f32(sp[r].row[sp[r].edge_index(e)]), M[r]);
        rs[r] = make_row_sum(group_allreduce<LANES, false>(sum));
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int64_t row = row0 + (int64_t)r * GROUPS;
        if (row >= m) continue;
        uint16_t *srow = softmax + row * n;
        if (live[r]) {
            u32x4 o;
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = pack2<T>(quotient(ex[r][2 * k], rs[r]), quotient(ex[r][2 * k + 1], rs[r]));
            __builtin_nontemporal_store(o, (u32x4 *)(srow + sp[r].head) + sub);
        }
        for (int e = sub; e < sp[r].nedge; e += LANES) {
            const int32_t i = sp[r].edge_index(e);
            srow[i] = T::from_f32(quotient(exp_biased(T::to_f32(sp[r].row[i]), M[r]), rs[r]));
        }
        if (sub == 0) out[row] = row_loss<T>(sp[r].row, n, target[row], ignore_index, M[r], rs[r].S);
    }
}

// ---- forward, long rows: stream once, keep most of the row on chip ---------------------
// 1024 lanes per row, two workgroups per CU (<= 64 VGPRs, <= 64 KiB LDS each).  Sweep 1 streams
// the row from HBM in `chunks` vectors per lane while each lane keeps a running maximum and the sum
// of exponentials relative to it (rescaled when the maximum grows).  The first RK vectors of a
// lane stay in registers and the next LK in LDS; the remaining ones are dropped.  Sweep 2 walks the
// row backwards: the dropped vectors — the most recently fetched, so the likeliest to sit in L2
// still — are loaded again, then the LDS and register parts follow without memory traffic.
// Cache policy decides what that second fetch costs: the first fetch of the dropped part uses the default
// policy so that the lines stay in L2 and the memory-side cache (fetched non-temporally, the second fetch
// comes from HBM and the kernel takes 0.92 ms instead of 0.76 at 8,192 x 128,256; each pair of chunks fetched
// that way costs 0.02-0.05 ms), and the second fetch is non-temporal — its lines are dead afterwards —
// which gains 1.2 %.  With the first fetch cached, the second one is free: a timing probe that skips it
// altogether runs no faster.
// Fine-grained load/compute interleaving in both sweeps lets the 32 waves of a CU hide each
// other's latencies, which a whole-row-resident scheme with one or two workgroups per CU cannot.
//
// XR > 0 (rows of more than 10,240 vectors) keeps three more chunks: one in what is left of the CU's LDS — two
// workgroups share 160 KiB, so all lanes but the last 16 find room for a fifth vector — and the two after it in
// registers (58 VGPRs), and issues the four loads of the register part before it folds the first of them.  Together
// 0.8 % at 128,256 classes (0.7597 -> 0.7529 ms, nine alternating rounds in one process); on rows that have no
// dropped part the same code is 2 % slower, and so it is on rows of 9 or 10 chunks (8,192 x 81,920: 0.4575 against
// 0.4511 ms); from 11 chunks on it is ahead (90,112: 0.5230 against 0.5327; 98,304: 0.5761 against 0.6067), hence the
// condition.  Chunks are folded into the running sums two at a
// time in row order either way, so the results do not depend on RK / LK / XR.
template <typename T, int RK, int LK, int XR>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(8, 8))) void ce_forward_retain_kernel(
    int32_t n, const uint16_t *__restrict__ x, const int32_t *__restrict__ target,
    uint16_t *__restrict__ softmax, float *__restrict__ out, int32_t ignore_index, int32_t chunks, uint32_t align) {
    constexpr int THREADS = 1024;
    constexpr int GROUP = 2;
    static_assert(RK % GROUP == 0 && LK % GROUP == 0, "chunk counts must be even");   // and so is `chunks`
    static_assert(XR == 0 || XR == 2, "none, or chunk RK + LK in LDS and the two after it in registers");
    constexpr int kPartialLanes = THREADS - 16;                 // lanes whose vector of chunk RK + LK fits into LDS
    constexpr int DROP0 = RK + LK + (XR > 0 ? 2 * GROUP : 0);   // first chunk that every lane fetches twice
    extern __shared__ u32x4 staged[];  // LK * 1024 vectors, and kPartialLanes more when XR > 0
    __shared__ float slots[2][THREADS / kWave];
    const int64_t row = xcd_run_row(blockIdx.x, gridDim.x);
    const RowSpan sp = row_span(x, row, n, align);
    const int32_t nvec = sp.nvec;
    const u32x4 *xr = (const u32x4 *)(sp.row + sp.head);
    uint16_t *srow = softmax + row * n;
    u32x4 *sr = (u32x4 *)(srow + sp.head);
    const int tid = threadIdx.x;
    const uint32_t pad = neg_inf2<T>();
    const u32x4 pad4 = {pad, pad, pad, pad};

    float m = -1e6f;   // running maximum of this lane, never below the reference's clamp
    float s = 0.f;     // sum of 2^16 * e^(x - m) over this lane's elements so far
    // Folds GROUP vectors into (m, s).
    auto absorb = [&](const u32x4 (&v)[GROUP], int c0) {
        if (c0 * THREADS + (tid & ~(kWave - 1)) >= nvec) return;   // this wave is past the end of the row
        float vm = -INFINITY;
#pragma unroll
        for (int g = 0; g < GROUP; g++) vec_max<T>(v[g], vm);
        if (vm > m) {
            s *= __builtin_amdgcn_exp2f((m - vm) * kLog2e);
            m = vm;
        }
#pragma unroll
        for (int g = 0; g < GROUP; g++) vec_sumexp<T>(v[g], m, s);
    };
    u32x4 w[RK > 0 ? RK : 1];
    u32x4 wx = pad4, wy = pad4;
    // register part
    if constexpr (XR > 0) {
#pragma unroll
        for (int c = 0; c < RK; c++) {
            const int j = c * THREADS + tid;
            w[c] = j < nvec ? __builtin_nontemporal_load(xr + j) : pad4;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c0 = 0; c0 < RK; c0 += GROUP) {
            u32x4 v[GROUP];
#pragma unroll
            for (int g = 0; g < GROUP; g++) v[g] = w[c0 + g];
            absorb(v, c0);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
#pragma unroll
        for (int c0 = 0; c0 < RK; c0 += GROUP) {
            u32x4 v[GROUP];
#pragma unroll
            for (int g = 0; g < GROUP; g++) {
                const int j = (c0 + g) * THREADS + tid;
                v[g] = j < nvec ? __builtin_nontemporal_load(xr + j) : pad4;
            }
            absorb(v, c0);
#pragma unroll
            for (int g = 0; g < GROUP; g++) w[c0 + g] = v[g];
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // LDS part
#pragma unroll 1
    for (int c0 = RK; c0 < RK + LK; c0 += GROUP) {
        u32x4 v[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; g++) {
            const int j = (c0 + g) * THREADS + tid;
            v[g] = j < nvec ? __builtin_nontemporal_load(xr + j) : pad4;
        }
        absorb(v, c0);
#pragma unroll
        for (int g = 0; g < GROUP; g++) staged[(c0 + g - RK) * THREADS + tid] = v[g];
    }
    if constexpr (XR > 0) {
        // chunk RK + LK: to LDS where there is room (the last 16 lanes fetch theirs twice), RK + LK + 1: register
        {
            u32x4 v[GROUP];
            const int j0 = (RK + LK) * THREADS + tid, j1 = j0 + THREADS;
            if (tid < kPartialLanes) v[0] = j0 < nvec ? __builtin_nontemporal_load(xr + j0) : pad4;
            else v[0] = j0 < nvec ? xr[j0] : pad4;
            v[1] = j1 < nvec ? __builtin_nontemporal_load(xr + j1) : pad4;
            absorb(v, RK + LK);
            if (tid < kPartialLanes) staged[LK * THREADS + tid] = v[0];
            wx = v[1];
        }
        // chunk RK + LK + 2: register, RK + LK + 3: fetched twice
        {
            u32x4 v[GROUP];
            const int j0 = (RK + LK + 2) * THREADS + tid, j1 = j0 + THREADS;
            v[0] = j0 < nvec ? __builtin_nontemporal_load(xr + j0) : pad4;
            v[1] = j1 < nvec ? xr[j1] : pad4;
            absorb(v, RK + LK + 2);
            wy = v[0];
        }
    }
    // dropped part: default cache policy, so that the second fetch finds it in L2 or the memory-side cache
#pragma unroll 1
    for (int c0 = DROP0; c0 < chunks; c0 += GROUP) {
        u32x4 v[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; g++) {
            const int j = (c0 + g) * THREADS + tid;
            v[g] = j < nvec ? xr[j] : pad4;
        }
        absorb(v, c0);
    }
    if (tid < sp.nedge) {
        const float edge = T::to_f32(sp.row[sp.edge_index(tid)]);
        if (edge > m) {
            s *= __builtin_amdgcn_exp2f((m - edge) * kLog2e);
            m = edge;
        }
        s += exp_biased(edge, m);
    }
    const float M = block_allreduce<true>(m, slots[0]);
    s *= __builtin_amdgcn_exp2f((m - M) * kLog2e);
    const RowSum rs = make_row_sum(block_allreduce<false>(s, slots[1]));
    if (tid < sp.nedge) {
        const int32_t i = sp.edge_index(tid);
        srow[i] = T::from_f32(quotient(exp_biased(T::to_f32(sp.row[i]), M), rs));
    }

    // dropped part, last fetched first; its lines are not needed again (non-temporal)
#pragma unroll 1
    for (int c0 = chunks - GROUP; c0 >= DROP0; c0 -= GROUP) {
        u32x4 v[GROUP];
#pragma unroll
        for (int g = GROUP - 1; g >= 0; g--) {
            const int j = (c0 + g) * THREADS + tid;
            v[g] = j < nvec ? __builtin_nontemporal_load(xr + j) : pad4;
        }
#pragma unroll
        for (int g = GROUP - 1; g >= 0; g--) {
            const int j = (c0 + g) * THREADS + tid;
            if (j < nvec) __builtin_nontemporal_store(vec_softmax<T>(v[g], M, rs), sr + j);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (XR > 0) {
        {
            const int j0 = (RK + LK + 2) * THREADS + tid, j1 = j0 + THREADS;
            const u32x4 v1 = j1 < nvec ? __builtin_nontemporal_load(xr + j1) : pad4;
            if (j1 < nvec) __builtin_nontemporal_store(vec_softmax<T>(v1, M, rs), sr + j1);
            if (j0 < nvec) __builtin_nontemporal_store(vec_softmax<T>(reread(wy), M, rs), sr + j0);
        }
        {
            const int j0 = (RK + LK) * THREADS + tid, j1 = j0 + THREADS;
            u32x4 v0 = pad4;
            if (tid >= kPartialLanes && j0 < nvec) v0 = __builtin_nontemporal_load(xr + j0);
            if (j1 < nvec) __builtin_nontemporal_store(vec_softmax<T>(reread(wx), M, rs), sr + j1);
            if (tid < kPartialLanes) v0 = staged[LK * THREADS + tid];
            if (j0 < nvec) __builtin_nontemporal_store(vec_softmax<T>(v0, M, rs), sr + j0);
        }
    }
    // LDS part (each lane reads the slots it wrote itself)
#pragma unroll 1
    for (int c = LK - 1; c >= 0; c--) {
        const int j = (RK + c) * THREADS + tid;
        if (j < nvec) __builtin_nontemporal_store(vec_softmax<T>(staged[c * THREADS + tid], M, rs), sr + j);
    }
    // register part
#pragma unroll
    for (int c = RK - 1; c >= 0; c--) {
        const int j = c * THREADS + tid;
        if (j < nvec) __builtin_nontemporal_store(vec_softmax<T>(reread(w[c]), M, rs), sr + j);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (tid == 0) out[row] = row_loss<T>(sp.row, n, target[row], ignore_index, M, rs.S);
}

// ---- forward, any row length / alignment ---------------------------------------
// One workgroup per row, three sweeps with 2-byte loads (max; sum of exponentials;
// quotient).  The second and third sweep re-read the row through the caches.
constexpr int kSweepThreads = 256;
template <typename T>
__global__ __launch_bounds__(kSweepThreads) void ce_forward_sweep_kernel(
    int32_t n, const uint16_t *__restrict__ x, const int32_t *__restrict__ target, uint16_t *__restrict__ softmax,
    float *__restrict__ out, int32_t ignore_index) {
    __shared__ float slots[2][kSweepThreads / kWave];
    const int64_t row = blockIdx.x;
    const uint16_t *xr = x + row * n;
    uint16_t *sr = softmax + row * n;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < n; i += kSweepThreads) mx = fmaxf(T::to_f32(xr[i]), mx);
    const float M = fmaxf(block_allreduce<true>(mx, slots[0]), -1e6f);
    float sum = 0.f;
    for (int i = threadIdx.x; i < n; i += kSweepThreads) sum += exp_biased(T::to_f32(xr[i]), M);
    const RowSum rs = make_row_sum(block_allreduce<false>(sum, slots[1]));
    const float S = rs.S;
    for (int i = threadIdx.x; i < n; i += kSweepThreads) sr[i] = T::from_f32(quotient(exp_biased(T::to_f32(xr[i]), M), rs));
    if (threadIdx.x == 0) out[row] = row_loss<T>(xr, n, target[row], ignore_index, M, S);
}

// ---- element-wise kernels over the flat [m * n] array -----------------------------
// OP 0: backward in place.  OP 1: softmax in place from given max / sum.
constexpr int kFlatThreads = 1024;
constexpr int kFlatUnroll = 1;
constexpr int kFlatScalarThreads = 256;

template <typename T, int OP>
__device__ __forceinline__ float flat_elem(float s, bool is_target, float a, float b) {
    if (OP == 0) return is_target ? (s - 1.f) * a : s * a;  // a = grad_output[r]
    return exp_biased(s, a) * b;                            // a = max, b = 2^-16 / sum
}
// Second per-row scalar of the flat kernels: nothing for the backward, 2^-16 / sum for the softmax.
template <int OP>
__device__ __forceinline__ float flat_row_b(const float *row_b, int64_t row) {
    return OP == 1 ? kTwoPowMinusBias / row_b[row] : 0.f;
}

// One workgroup transforms one tile of kFlatThreads * kFlatUnroll vectors and exits.  The array is
// taken as one run of m * n elements: `head` elements up to the first 16-byte boundary, total_vec
// vectors, and a tail of fewer than 8 elements (head and tail: first lanes of workgroup 0).  With a
// row length that is not a multiple of 8 a vector can hold the end of one row and the start of
// the next (n >= 8: never more than two rows).  RAGGED = false promises n % 8 == 0 and head == 0.
template <typename T, int OP, bool RAGGED>
__global__ __launch_bounds__(kFlatThreads) void ce_flat_vec_kernel(
    int32_t n, int32_t head, int64_t total_vec, int64_t total, uint16_t *__restrict__ x,
    const float *__restrict__ row_a, const float *__restrict__ row_b, const int32_t *__restrict__ target) {
    u32x4 *xv = (u32x4 *)(x + head);
    const int64_t start = (int64_t)blockIdx.x * (kFlatThreads * kFlatUnroll);   // first vector of the tile
    const int64_t first = (int64_t)head + 8 * start;                            // its first element
    const int64_t row0 = first / n;
    const uint32_t col0 = (uint32_t)(first - row0 * n);
    u32x4 w[kFlatUnroll];
    bool ok[kFlatUnroll];
#pragma unroll
    for (int u = 0; u < kFlatUnroll; u++) {
        const int64_t g = start + (int64_t)u * kFlatThreads + threadIdx.x;
        ok[u] = g < total_vec;
        if (ok[u]) w[u] = __builtin_nontemporal_load(xv + g);
    }
#pragma unroll
    for (int u = 0; u < kFlatUnroll; u++) {
        if (!ok[u]) continue;
        const int64_t g = start + (int64_t)u * kFlatThreads + threadIdx.x;
        const uint32_t off = col0 + 8u * (uint32_t)(u * kFlatThreads + threadIdx.x);
        const uint32_t dr = off / (uint32_t)n;
        const int64_t row = row0 + dr;
        const int32_t col = (int32_t)(off - dr * (uint32_t)n);
        const float a = row_a[row];
        const float b = flat_row_b<OP>(row_b, row);
        const int32_t tk = OP == 0 ? target[row] - col : -1;  // position of the target inside this vector
        u32x4 o;
        if (!RAGGED || col + 8 <= n) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const float lo = flat_elem<T, OP>(lo_f32<T>(w[u][k]), tk == 2 * k, a, b);
                const float hi = flat_elem<T, OP>(hi_f32<T>(w[u][k]), tk == 2 * k + 1, a, b);
                o[k] = pack2<T>(lo, hi);
            }
        } else {   // elements from position `split` on belong to the next row
            const int32_t split = n - col;
            const float a1 = row_a[row + 1];
            const float b1 = flat_row_b<OP>(row_b, row + 1);
            const int32_t tk1 = OP == 0 ? target[row + 1] + split : -1;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const bool lo_next = 2 * k >= split, hi_next = 2 * k + 1 >= split;
                const float lo = flat_elem<T, OP>(lo_f32<T>(w[u][k]), (lo_next ? tk1 : tk) == 2 * k, lo_next ? a1 : a,
                                                  lo_next ? b1 : b);
                const float hi = flat_elem<T, OP>(hi_f32<T>(w[u][k]), (hi_next ? tk1 : tk) == 2 * k + 1,
                                                  hi_next ? a1 : a, hi_next ? b1 : b);
                o[k] = pack2<T>(lo, hi);
            }
        }
        __builtin_nontemporal_store(o, xv + g);
    }
    if (RAGGED && blockIdx.x == 0) {
        const int64_t tail_lo = (int64_t)head + 8 * total_vec;
        const int64_t nedge = (int64_t)head + (total - tail_lo);
        if ((int64_t)threadIdx.x < nedge) {
            const int64_t i = (int64_t)threadIdx.x < head ? (int64_t)threadIdx.x : tail_lo + ((int64_t)threadIdx.x - head);
            const int64_t row = i / n;
            const int32_t col = (int32_t)(i - row * n);
            const bool is_t = OP == 0 ? (target[row] == col) : false;
            x[i] = T::from_f32(flat_elem<T, OP>(T::to_f32(x[i]), is_t, row_a[row], flat_row_b<OP>(row_b, row)));
        }
    }
}

// ---- the element-wise kernels as a resident grid --------------------------------------------
// Large arrays with rows of at least 8,192 elements run the way the
// long Adam launches do (see adam.hip): one workgroup of 256 lanes per compute unit stays resident and works
// through tiles of 1,024 vectors (16 KiB = four 4 KiB blocks, one load per lane and block) handed out by atomic
// tickets, with the loads of the next tile in flight while the current one is computed and stored; the vector
// memory instructions of the loop and their waits are written by hand.  A tile spans at most two rows, so the
// per-row scalars (grad_output / max, target / sum) of both are fetched with scalar loads, outside the vector
// memory counter.
//
// The array is transformed in place and the call has no output-only memory, so the ticket counters cannot live
// in a caller's buffer: they live in a small fixed array in the library's device image, one group of eight
// counters per stream that has been seen on the device (up to kFlatSlots; launches on one stream follow each other,
// so a group is never shared by two running launches).  Launches on a stream that is being captured into a graph,
// on the per-thread default stream, or beyond the slot table keep the workgroup-per-tile kernel.
constexpr int kFlatStreamThreads = 256;
constexpr int kFlatStreamVecs = 4;                    // vectors per lane and tile
constexpr int kFlatCounters = kSlotCounters;
constexpr int kFlatSlots = 256;
// Smallest array (in 16-byte vectors) that runs as the resident grid: 2^27 elements, 256 MiB.  Measured against one
// workgroup per tile, launches back to back on rows of 16,384 bf16 elements (% of peak, resident / per tile):
// 2^25 elements 66.6 / 73.5, 2^26 76.3 / 79.3, 2^27 81.4 / 81.8, 2^28 83.1 / 82.4, 2^29 83.8 / 81.6, 2^30 (8,192 x 128,256)
// 83.7 / 78; fp16 rows of 32,000: 6.6e7 elements 76.0 / 79.0, 1.3e8 81.2 / 81.6, 5.2e8 84.0 / 81.
constexpr int64_t kFlatStreamMinVec = (int64_t)1 << 24;
constexpr int32_t kFlatStreamMinRow = kFlatStreamThreads * kFlatStreamVecs * 8;
// counter c of slot s: word c * 1024 + s * 4 (the counters of one launch sit 4 KiB apart); word s * 4 + 1 counts the
// workgroups of the running launch that have left
static __device__ __align__(256) uint32_t flat_tickets[kFlatCounters * 1024];

// RAGGED: rows of any length from 8,192 elements on and any 2-byte aligned base (an unpadded vocabulary): the vectors are
// counted from the array's first 16-byte boundary, `head` elements in, so a tile starts at any column and the vector
// that holds the end of one row and the start of the next takes the scalars of both; the fewer than 8 elements in
// front of the first vector and behind the last one are transformed by the first lanes of workgroup 0 before its
// first tile.  The array must hold fewer than 2^32 elements (the row of a tile comes from one 32-bit division).
// TURNS: a workgroup takes its tiles from the counters in turn, as the long Adam launches do (see stream_next_counter in
// adam.hip), so that all counters move at the same rate; it then leaves after it has met a tile past the end from
// every counter in a row, seven draws later than with a counter of its own.  Measured against each other, alternating
// in one process: 2^27 elements 78.2 against 81.0 % of peak, 2^28 82.0 / 82.8, 2^29 83.7 / 83.4, 16,384 x 32,000 83.7 / 83.2,
// 8,192 x 128,256 84.5 / 83.7 - hence from 2^29 elements on.
constexpr int64_t kFlatTurnsMinVec = (int64_t)1 << 26;
template <typename T, int OP, bool RAGGED, bool TURNS>
__global__ __launch_bounds__(kFlatStreamThreads) void ce_flat_stream_kernel(
    int32_t n, int64_t total_vec, int64_t ntiles, u32x4 *__restrict__ xv, const float *__restrict__ row_a,
    const float *__restrict__ row_b, const int32_t *__restrict__ target, uint32_t *__restrict__ tickets,
    uint32_t *__restrict__ done_word, uint32_t launch_number, uint32_t head, uint32_t total) {
    constexpr int V = kFlatStreamVecs;
    constexpr int64_t kTileVecs = (int64_t)kFlatStreamThreads * V;
    struct Set {
        u32x4 w[V];
        int64_t base;        // first vector of the tile
        float a0, a1, b0, b1;
        int32_t t0, t1;      // targets of the tile's first row and of the row after it
        uint32_t col0;       // column of the tile's first element
        bool real;
    };
    __shared__ uint32_t handed[2];
    const int which = (int)((blockIdx.x >> 3) & (kFlatCounters - 1));
    const uint32_t q = ((blockIdx.x >> 6) << 3) | (blockIdx.x & 7u);      // number among the workgroups of this counter
    auto next_counter = [](int c) { return TURNS ? (c + 1) & (kFlatCounters - 1) : c; };
    const int64_t first = (int64_t)q * kFlatCounters + which;
    int64_t ahead = (int64_t)(q + (gridDim.x >> 3)) * kFlatCounters + next_counter(which);
    const uint32_t drawn_base = 2u * (gridDim.x >> 3);      // the first two tiles of a workgroup follow from its number
    if (RAGGED && blockIdx.x == 0) {     // the elements outside the vectors; no vector of any tile holds them
        const uint32_t tail_lo = head + 8u * (uint32_t)total_vec;
        const uint32_t nedge = head + (total - tail_lo);
        if (threadIdx.x < nedge) {
            uint16_t *x = (uint16_t *)xv - head;
            const uint32_t i = threadIdx.x < head ? threadIdx.x : tail_lo + (threadIdx.x - head);
            const uint32_t row = i / (uint32_t)n;
            const int32_t col = (int32_t)(i - row * (uint32_t)n);
            const bool is_t = OP == 0 ? (target[row] == col) : false;
            x[i] = T::from_f32(flat_elem<T, OP>(T::to_f32(x[i]), is_t, row_a[row], flat_row_b<OP>(row_b, row)));
        }
    }
    if (first >= ntiles) { stream_slot_leave(tickets, done_word, launch_number); return; }
    int drawing = next_counter(next_counter(which));        // counter of the ticket on its way
    uint32_t *const counter = tickets + drawing * 1024;     // TURNS = false: the only one
    uint32_t drawn = 0;
    if (threadIdx.x == 0) stream_draw(drawn, counter);
    const uint32_t row_vecs = (uint32_t)n >> 3;
    const uint32_t last_row = RAGGED ? total / (uint32_t)n - 1 : (uint32_t)total_vec / row_vecs - 1;

    auto issue = [&](Set &s, int64_t tile_in) {
        s.real = tile_in < ntiles;
        // the tile number is the same in every lane (it came through LDS): saying so puts the row arithmetic and the
        // loads of the per-row scalars below on the scalar unit, outside the vector memory counter
        const int64_t tile = s.real ? (int64_t)__builtin_amdgcn_readfirstlane((uint32_t)tile_in) : 0;
        s.base = tile * kTileVecs;
        uint32_t row0;
        if (RAGGED) {
            const uint32_t first_elem = head + 8u * (uint32_t)s.base;      // the launcher keeps the array below 2^32 elements
            row0 = first_elem / (uint32_t)n;
            s.col0 = first_elem - row0 * (uint32_t)n;
        } else {
            row0 = (uint32_t)s.base / row_vecs;                  // the launcher keeps total_vec below 2^32
            s.col0 = 8u * ((uint32_t)s.base - row0 * row_vecs);
        }
        const uint32_t row1 = row0 == last_row ? row0 : row0 + 1;     // the last row has no successor
        s.a0 = row_a[row0]; s.a1 = row_a[row1];
        if (OP == 0) { s.t0 = target[row0]; s.t1 = target[row1]; s.b0 = s.b1 = 0.f; }
        else { s.b0 = kTwoPowMinusBias / row_b[row0]; s.b1 = kTwoPowMinusBias / row_b[row1]; s.t0 = s.t1 = -1; }
#pragma unroll
        for (int u = 0; u < V; u++) {
            const int64_t g = s.base + u * kFlatStreamThreads + threadIdx.x;
            stream_load(s.w[u], xv + (s.real && g < total_vec ? g : 0));
        }
    };
    auto finish = [&](Set &s) {
        if (!s.real) return;
#pragma unroll
        for (int u = 0; u < V; u++) {
            const int64_t g = s.base + u * kFlatStreamThreads + threadIdx.x;
            if (g >= total_vec) continue;
            const uint32_t off = s.col0 + 8u * (uint32_t)(u * kFlatStreamThreads + threadIdx.x);
            u32x4 o;
            if (RAGGED) {
                // element k of the vector lies in the tile's first row while k < split, in the row after it otherwise
                const int32_t split = n - (int32_t)off;
                const int32_t tk0 = OP == 0 ? s.t0 - (int32_t)off : -1;       // position of either row's target in the vector
                const int32_t tk1 = OP == 0 ? s.t1 + split : -1;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const bool lo_next = 2 * k >= split, hi_next = 2 * k + 1 >= split;
                    const float lo = flat_elem<T, OP>(lo_f32<T>(s.w[u][k]), (lo_next ? tk1 : tk0) == 2 * k,
                                                      lo_next ? s.a1 : s.a0, lo_next ? s.b1 : s.b0);
                    const float hi = flat_elem<T, OP>(hi_f32<T>(s.w[u][k]), (hi_next ? tk1 : tk0) == 2 * k + 1,
                                                      hi_next ? s.a1 : s.a0, hi_next ? s.b1 : s.b0);
                    o[k] = pack2<T>(lo, hi);
                }
            } else {
                const bool next_row = off >= (uint32_t)n;
                const int32_t col = (int32_t)(next_row ? off - (uint32_t)n : off);
                const float a = next_row ? s.a1 : s.a0, b = next_row ? s.b1 : s.b0;
                const int32_t tk = OP == 0 ? (next_row ? s.t1 : s.t0) - col : -1;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float lo = flat_elem<T, OP>(lo_f32<T>(s.w[u][k]), tk == 2 * k, a, b);
                    const float hi = flat_elem<T, OP>(hi_f32<T>(s.w[u][k]), tk == 2 * k + 1, a, b);
                    o[k] = pack2<T>(lo, hi);
                }
            }
            stream_store(xv + g, o);
        }
    };
    auto stage = [&](Set &cur, Set &next, int slot) -> int64_t {
        const int64_t tile = ahead;
        issue(next, tile);
        asm volatile("s_waitcnt vmcnt(4)" : "+v"(cur.w[0]), "+v"(cur.w[1]), "+v"(cur.w[2]), "+v"(cur.w[3]), "+v"(drawn));
        if (threadIdx.x == 0) handed[slot] = drawn;
        __syncthreads();
        if constexpr (TURNS) {
            ahead = (int64_t)(handed[slot] + drawn_base) * kFlatCounters + drawing;
            drawing = next_counter(drawing);
            if (threadIdx.x == 0) stream_draw(drawn, tickets + drawing * 1024);
        } else {
            ahead = (int64_t)(handed[slot] + drawn_base) * kFlatCounters + which;
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
            if (beyond == kFlatCounters) break;
            beyond = stage(b, a, 1) >= ntiles ? beyond + 1 : 0;
            if (beyond == kFlatCounters) break;
        }
    } else {
        while (true) {
            if (stage(a, b, 0) >= ntiles) break;
            if (stage(b, a, 1) >= ntiles) break;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    stream_slot_leave(tickets, done_word, launch_number);
}

template <typename T, int OP>
__global__ __launch_bounds__(kFlatScalarThreads) void ce_flat_scalar_kernel(
    int32_t n, int64_t total, uint16_t *__restrict__ x, const float *__restrict__ row_a,
    const float *__restrict__ row_b, const int32_t *__restrict__ target) {
    for (int64_t g = (int64_t)blockIdx.x * kFlatScalarThreads + threadIdx.x; g < total;
         g += (int64_t)gridDim.x * kFlatScalarThreads) {
        const int64_t row = g / n;
        const int32_t col = (int32_t)(g - row * n);
        const float a = row_a[row];
        const float b = flat_row_b<OP>(row_b, row);
        const bool is_t = OP == 0 ? (target[row] == col) : false;
        x[g] = T::from_f32(flat_elem<T, OP>(T::to_f32(x[g]), is_t, a, b));
    }
}

// ---- row sum of exponentials given the row maximum ---------------------------------
// One workgroup of THREADS lanes per row, two vectors per lane in flight.  The exponentials are the
// biased ones of the forward kernels; the factor 2^16 is taken out of the sum at the end.
template <typename T, int THREADS>
__global__ __launch_bounds__(THREADS) void sumexp_kernel(int32_t n, const uint16_t *__restrict__ x,
                                                         const float *__restrict__ row_max,
                                                         float *__restrict__ row_sum) {
    __shared__ float slots[THREADS / kWave];
    const int64_t row = blockIdx.x;
    const RowSpan sp = row_span(x, row, n);
    const u32x4 *xr = (const u32x4 *)(sp.row + sp.head);
    const float M = row_max[row];
    const uint32_t pad = neg_inf2<T>();
    const u32x4 pad4 = {pad, pad, pad, pad};
    float sum = 0.f;
    for (int j0 = 0; j0 < sp.nvec; j0 += 2 * THREADS) {
        const int ja = j0 + threadIdx.x, jb = ja + THREADS;
        const u32x4 wa = ja < sp.nvec ? __builtin_nontemporal_load(xr + ja) : pad4;
        const u32x4 wb = jb < sp.nvec ? __builtin_nontemporal_load(xr + jb) : pad4;
        vec_sumexp<T>(wa, M, sum);
        vec_sumexp<T>(wb, M, sum);
    }
    if ((int)threadIdx.x < sp.nedge) sum += exp_biased(T::to_f32(sp.row[sp.edge_index(threadIdx.x)]), M);
    sum = block_allreduce<false>(sum, slots);
    if (threadIdx.x == 0) row_sum[row] = sum * kTwoPowMinusBias;
}

// ---- host side ------------------------------------------------------------------
// The forward kernels move input and output rows as 16-byte vectors with one split per row, which
// needs the two arrays to sit at the same offset from a 16-byte boundary.
static bool same_vector_phase(const void *a, const void *b) {
    return ((((uintptr_t)a) ^ ((uintptr_t)b)) & 15u) == 0;
}

static int flat_grid(int64_t work_items, int threads_times_unroll) {
    const int64_t tiles = (work_items + threads_times_unroll - 1) / threads_times_unroll;
    const int64_t cap = (int64_t)device_cu_count() * 16;
    return (int)(tiles < 1 ? 1 : (tiles < cap ? tiles : cap));
}

#define BMT_CE_ROW(THREADS, CHUNKS)                                                                                \
    hipLaunchKernelGGL((ce_forward_row_kernel<T, THREADS, CHUNKS>), dim3((unsigned)m), dim3(THREADS), 0, s, n,         \
                       (const uint16_t *)input, (const int32_t *)target, (uint16_t *)softmax, (float *)output,     \
                       ignore_index, align)

#define BMT_CE_SMALL(LANES)                                                                                       \
    do {                                                                                                           \
        constexpr int R = 2;                                                                                       \
        const int64_t rows_per_group = (int64_t)(kSmallThreads / kWave) * R * (kWave / (LANES));                   \
        hipLaunchKernelGGL((ce_forward_small_kernel<T, LANES, R>), dim3((unsigned)((m + rows_per_group - 1) / rows_per_group)), \
                           dim3(kSmallThreads), 0, s, m, n, (const uint16_t *)input, (const int32_t *)target,      \
                           (uint16_t *)softmax, (float *)output, ignore_index);                                    \
    } while (0)

#define BMT_CE_RETAIN(CHUNKS, RK, LK, XR)                                                                          \
    do {                                                                                                           \
        auto kern = ce_forward_retain_kernel<T, RK, LK, XR>;                                                       \
        const size_t lds = ((size_t)(LK) * 1024 + ((XR) > 0 ? 1024 - 16 : 0)) * sizeof(u32x4);                     \
        static std::atomic<uint64_t> allowed{0};   /* devices on which this kernel may use `lds` bytes */         \
        int dev = 0;                                                                                               \
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 63;                                    \
        if (dev == 63 || !((allowed.load(std::memory_order_relaxed) >> dev) & 1u)) {                               \
            const hipError_t attr = hipFuncSetAttribute((const void *)kern,                                        \
                                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);     \
            if (attr != hipSuccess) return fail((int)attr, who, attr);                                             \
            allowed.fetch_or((uint64_t)1 << dev, std::memory_order_relaxed);                                       \
        }                                                                                                          \
        hipLaunchKernelGGL(kern, dim3((unsigned)m), dim3(1024), lds, s, n, (const uint16_t *)input,                \
                           (const int32_t *)target, (uint16_t *)softmax, (float *)output, ignore_index,            \
                           (int32_t)(CHUNKS), align);                                                              \
    } while (0)

template <typename T>
static int ce_forward(int32_t m, int32_t n, const void *input, const void *target, void *softmax, void *output,
                      int32_t ignore_index, void *stream, const char *who) {
    if (m <= 0 || n <= 0) return 0;
    if (!input || !target || !softmax || !output) return fail(-1, "cross_entropy_forward launcher: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if ((((uintptr_t)input | (uintptr_t)softmax) & 1u) != 0)
        return fail(-1, "cross_entropy_forward launcher: pointer is not 2-byte aligned");
    // Not an in-place operation: the loss reads input[r, target[r]] after the row's softmax has been stored (in the
    // reference as well, cross_entropy.cu:30-36), and the kernels here fetch parts of a row a second time.
    {
        const uintptr_t a = (uintptr_t)input, b = (uintptr_t)softmax, bytes = (uintptr_t)2 * (uintptr_t)m * (uintptr_t)n;
        if (a < b + bytes && b < a + bytes) return fail(-1, "cross_entropy_forward launcher: softmax overlaps input");
    }
    const int32_t nvec = n / 8;   // the most vectors a row can have
    // Rows of more than 16,384 elements: vectors are placed from the first 128-byte line boundary of a row where both
    // arrays sit at the same offset from one (any two torch allocations do), else from the first 16-byte boundary.
    // Measured on rows that start off the line grid (2^29 elements in all, ms with 16-byte / with 128-byte placement):
    // 8,192 x 86,583: 0.529 / 0.472; 128,257: 0.812 / 0.750; 16,384 x 32,001: 0.354 / 0.337; 65,544: 0.421 / 0.386;
    // 20,488: 0.372 / 0.356; 16,392: 0.372 / 0.369; shorter rows gain or lose up to 5 % either way (up to 70 elements
    // of a row then go through the one-element path), 2,056: 0.109 / 0.125.  Rows on the line grid are not affected.
    const uint32_t align = (nvec > 2048 && ((((uintptr_t)input) ^ ((uintptr_t)softmax)) & 127u) == 0) ? 64u : 8u;
    if (same_vector_phase(input, softmax)) {
        // rows up to 32,768 elements live in the registers of their workgroup
        // short rows: several rows per wave
        if (nvec <= 8) BMT_CE_SMALL(8);
        else if (nvec <= 16) BMT_CE_SMALL(16);
        else if (nvec <= 32) BMT_CE_SMALL(32);
        else if (nvec <= 64) BMT_CE_SMALL(64);
        else if (nvec <= 128) BMT_CE_ROW(64, 2);
        else if (nvec <= 192) BMT_CE_ROW(64, 3);
        else if (nvec <= 256) BMT_CE_ROW(64, 4);
        else if (nvec <= 512) BMT_CE_ROW(256, 2);
        else if (nvec <= 768) BMT_CE_ROW(256, 3);
        else if (nvec <= 1024) BMT_CE_ROW(256, 4);
        else if (nvec <= 1536) BMT_CE_ROW(512, 3);
        else if (nvec <= 2048) BMT_CE_ROW(1024, 2);
        else if (nvec <= 3072) BMT_CE_ROW(1024, 3);
        else if (nvec <= 4096) BMT_CE_ROW(1024, 4);
        // up to 65,536 elements: 4 vectors per lane in registers, the rest in LDS, two workgroups per CU
        else if (nvec <= 6144) BMT_CE_RETAIN(6, 2, 4, 0);
        // up to 81,920 elements: 8 vectors per lane kept, the rest fetched twice
        else if (nvec <= 10240) BMT_CE_RETAIN(2 * ((nvec + 2047) / 2048), 4, 4, 0);
        // longer rows: 11 vectors per lane kept (all but 16 lanes)
        else BMT_CE_RETAIN(2 * ((nvec + 2047) / 2048), 4, 4, 2);
    } else {
        hipLaunchKernelGGL((ce_forward_sweep_kernel<T>), dim3((unsigned)m), dim3(kSweepThreads), 0, s, n,
                           (const uint16_t *)input, (const int32_t *)target, (uint16_t *)softmax, (float *)output,
                           ignore_index);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}

// The ticket counters of the resident element-wise kernel for `stream`, or null when the launch has to use the
// workgroup-per-tile kernel (see ce_flat_stream_kernel): a stream under graph capture, the per-thread default stream,
// a stream that belongs to another device than the current one, or a full table with nothing to evict.
//
// Every device keeps a table of up to kFlatSlots stream handles; a stream's slot is its group of eight counters.
// Launches that use a slot are numbered, and the last workgroup of a launch writes that number into the slot's word
// of a small pinned host array (stream_slot_leave).  When the table is full, the least recently used slot whose word shows
// its latest launch — so nothing can still be drawing from its counters, whether or not its stream still exists — is
// given to the new stream.  The handles in the table are only ever compared, never passed to the runtime: a stream
// may have been destroyed since.  A process that creates and destroys streams therefore keeps the resident kernel.
struct FlatStreamStats { int64_t resident = 0, fallback = 0, evictions = 0; };
static FlatStreamStats flat_stats[64];
static std::mutex flat_mutex;
struct FlatSlot { hipStream_t stream; uint64_t last_use; uint32_t launches; };
struct FlatDevice {
    uint32_t *base = nullptr;
    volatile uint32_t *done = nullptr;          // pinned host memory, one word per slot, written by the device
    FlatSlot slots[kFlatSlots];
    int used = 0;
    uint64_t clock = 0;
};
static FlatDevice flat_devices[64];
bool stream_slot_for(hipStream_t stream, StreamSlot *launch, bool counted) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    auto fallback = [&]() -> bool {
        (void)hipGetLastError();
        std::lock_guard<std::mutex> lock(flat_mutex);
        if (counted) flat_stats[dev].fallback++;
        return false;
    };
    if (stream == hipStreamPerThread) return fallback();
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) return fallback();
    hipDevice_t owner = -1;
    if (hipStreamGetDevice(stream, &owner) != hipSuccess || (int)owner != dev) return fallback();   // counters are per device
    std::lock_guard<std::mutex> lock(flat_mutex);
    FlatDevice &d = flat_devices[dev];
    if (d.base == nullptr) {
        uint32_t *base = nullptr;
        void *done = nullptr;
        if (hipGetSymbolAddress((void **)&base, HIP_SYMBOL(flat_tickets)) != hipSuccess ||
            hipHostMalloc(&done, kFlatSlots * sizeof(uint32_t), hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            if (counted) flat_stats[dev].fallback++;
            return false;
        }
        for (int k = 0; k < kFlatSlots; k++) ((uint32_t *)done)[k] = 0u;
        d.base = base;
        d.done = (volatile uint32_t *)done;
    }
    int slot = 0;
    while (slot < d.used && d.slots[slot].stream != stream) slot++;
    if (slot == d.used) {
        if (d.used < kFlatSlots) {
            d.slots[slot] = FlatSlot{stream, 0, 0u};
            d.used++;
        } else {
            slot = -1;
            uint64_t tried_up_to = 0;
            for (int attempt = 0; attempt < 16 && slot < 0; attempt++) {       // least recently used first
                int oldest = -1;
                for (int k = 0; k < kFlatSlots; k++)
                    if (d.slots[k].last_use > tried_up_to && (oldest < 0 || d.slots[k].last_use < d.slots[oldest].last_use)) oldest = k;
                if (oldest < 0) break;
                tried_up_to = d.slots[oldest].last_use;
                if (d.done[oldest] == d.slots[oldest].launches) slot = oldest;
            }
            if (slot < 0) { if (counted) flat_stats[dev].fallback++; return false; }
            flat_stats[dev].evictions++;
            d.slots[slot].stream = stream;
        }
    }
    d.slots[slot].last_use = ++d.clock;
    launch->number = ++d.slots[slot].launches;
    launch->tickets = d.base + slot * 4;
    launch->done_word = (uint32_t *)d.done + slot;
    if (counted) flat_stats[dev].resident++;
    return true;
}

template <typename T, int OP>
static int ce_flat(int32_t m, int32_t n, void *x, const void *row_a, const void *row_b, const void *target, void *stream,
                   const char *who) {
    if (m <= 0 || n <= 0) return 0;
    if (!x || !row_a || (OP == 1 && !row_b) || (OP == 0 && !target)) return fail(-1, "cross_entropy launcher: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (((uintptr_t)x & 1u) != 0) return fail(-1, "cross_entropy launcher: pointer is not 2-byte aligned");
    if (n >= 8) {
        const int64_t total = (int64_t)m * n;
        int64_t head = (int64_t)(((16 - ((uintptr_t)x & 15u)) & 15u) / 2);
        if (head > total) head = total;
        const int64_t total_vec = (total - head) / 8;
        int64_t tiles = (total_vec + kFlatThreads * kFlatUnroll - 1) / (kFlatThreads * kFlatUnroll);
        if (tiles < 1) tiles = 1;
        if (tiles > 0x7FFFFFFF) return fail(-1, "cross_entropy launcher: tensor too large for one launch");
        const bool even = n % 8 == 0 && head == 0;
        if (n >= kFlatStreamMinRow && total_vec >= kFlatStreamMinVec &&
            (even ? total_vec < ((int64_t)1 << 32) : total < ((int64_t)1 << 32))) {
            StreamSlot fl;
            if (stream_slot_for(s, &fl, true)) {
                uint32_t *tickets = fl.tickets;
                const int cus = device_cu_count();
                const unsigned grid = (unsigned)(cus >= 64 ? cus / 64 * 64 : 64);      // 8 XCDs x 8 counters
                const int64_t per_tile = (int64_t)kFlatStreamThreads * kFlatStreamVecs;
                const bool turns = total_vec >= kFlatTurnsMinVec;
                auto resident = even ? (turns ? ce_flat_stream_kernel<T, OP, false, true> : ce_flat_stream_kernel<T, OP, false, false>)
                                     : (turns ? ce_flat_stream_kernel<T, OP, true, true> : ce_flat_stream_kernel<T, OP, true, false>);
                hipLaunchKernelGGL(resident, dim3(grid), dim3(kFlatStreamThreads), 0, s, n, total_vec,
                                   (total_vec + per_tile - 1) / per_tile, (u32x4 *)((uint16_t *)x + head), (const float *)row_a,
                                   (const float *)row_b, (const int32_t *)target, tickets, fl.done_word, fl.number, (uint32_t)head,
                                   (uint32_t)total);
                hipError_t e = hipGetLastError();
                return e == hipSuccess ? 0 : fail((int)e, who, e);
            }
        }
        auto kern = even ? ce_flat_vec_kernel<T, OP, false> : ce_flat_vec_kernel<T, OP, true>;
        hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(kFlatThreads), 0, s, n, (int32_t)head, total_vec, total,
                           (uint16_t *)x, (const float *)row_a, (const float *)row_b, (const int32_t *)target);
    } else {
        const int64_t total = (int64_t)m * n;
        hipLaunchKernelGGL((ce_flat_scalar_kernel<T, OP>), dim3(flat_grid(total, kFlatScalarThreads)), dim3(kFlatScalarThreads), 0, s, n,
                           total, (uint16_t *)x, (const float *)row_a, (const float *)row_b, (const int32_t *)target);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}

template <typename T>
static int sumexp(int32_t m, int32_t n, const void *logits, const void *row_max, void *row_sum, void *stream,
                  const char *who) {
    if (m <= 0 || n <= 0) return 0;
    if (!logits || !row_max || !row_sum) return fail(-1, "fused_sumexp launcher: null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (((uintptr_t)logits & 1u) != 0) return fail(-1, "fused_sumexp launcher: pointer is not 2-byte aligned");
    if (n > 16384)
        hipLaunchKernelGGL((sumexp_kernel<T, 1024>), dim3((unsigned)m), dim3(1024), 0, s, n, (const uint16_t *)logits,
                           (const float *)row_max, (float *)row_sum);
    else
        hipLaunchKernelGGL((sumexp_kernel<T, 256>), dim3((unsigned)m), dim3(256), 0, s, n, (const uint16_t *)logits,
                           (const float *)row_max, (float *)row_sum);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : fail((int)e, who, e);
}

}  // namespace bmt

using namespace bmt;

extern "C" int bmt_hip_flat_stream_stats(int64_t *out) {
    if (!out) return fail(-1, "bmt_hip_flat_stream_stats: null pointer");
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(-1, "bmt_hip_flat_stream_stats: no current device");
    std::lock_guard<std::mutex> lock(flat_mutex);
    out[0] = flat_stats[dev].resident;
    out[1] = flat_stats[dev].fallback;
    out[2] = flat_stats[dev].evictions;
    return 0;
}

extern "C" int cross_entropy_forward_fp16_launcher(int32_t m, int32_t n, const void *input, const void *target,
                                                   void *softmax, void *output, int32_t ignore_index, void *stream) {
    return ce_forward<Half>(m, n, input, target, softmax, output, ignore_index, stream, "cross_entropy_forward_fp16_launcher");
}
extern "C" int cross_entropy_forward_bf16_launcher(int32_t m, int32_t n, const void *input, const void *target,
                                                   void *softmax, void *output, int32_t ignore_index, void *stream) {
    return ce_forward<BFloat16>(m, n, input, target, softmax, output, ignore_index, stream, "cross_entropy_forward_bf16_launcher");
}
extern "C" int cross_entropy_backward_inplace_fp16_launcher(int32_t m, int32_t n, const void *grad_output,
                                                            const void *target, void *x, int32_t ignore_index,
                                                            void *stream) {
    (void)ignore_index;  // cross_entropy.cu:46-60 never reads it
    return ce_flat<Half, 0>(m, n, x, grad_output, nullptr, target, stream, "cross_entropy_backward_inplace_fp16_launcher");
}
extern "C" int cross_entropy_backward_inplace_bf16_launcher(int32_t m, int32_t n, const void *grad_output,
                                                            const void *target, void *x, int32_t ignore_index,
                                                            void *stream) {
    (void)ignore_index;
    return ce_flat<BFloat16, 0>(m, n, x, grad_output, nullptr, target, stream, "cross_entropy_backward_inplace_bf16_launcher");
}
extern "C" int fused_sumexp_fp16_launcher(int32_t m, int32_t n, const void *logits, const void *max_logits,
                                          void *sum_exp_logits, void *stream) {
    return sumexp<Half>(m, n, logits, max_logits, sum_exp_logits, stream, "fused_sumexp_fp16_launcher");
}
extern "C" int fused_sumexp_bf16_launcher(int32_t m, int32_t n, const void *logits, const void *max_logits,
                                          void *sum_exp_logits, void *stream) {
    return sumexp<BFloat16>(m, n, logits, max_logits, sum_exp_logits, stream, "fused_sumexp_bf16_launcher");
}
extern "C" int fused_softmax_inplace_fp16_launcher(int32_t m, int32_t n, void *logits, const void *max_logits,
                                                   const void *sum_exp_logits, void *stream) {
    return ce_flat<Half, 1>(m, n, logits, max_logits, sum_exp_logits, nullptr, stream, "fused_softmax_inplace_fp16_launcher");
}
extern "C" int fused_softmax_inplace_bf16_launcher(int32_t m, int32_t n, void *logits, const void *max_logits,
                                                   const void *sum_exp_logits, void *stream) {
    return ce_flat<BFloat16, 1>(m, n, logits, max_logits, sum_exp_logits, nullptr, stream, "fused_softmax_inplace_bf16_launcher");
}
