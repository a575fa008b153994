// Reduction of the per-row cross-entropy losses for gfx950: what FusedCrossEntropy does after the forward kernel
// (bmtrain/loss/cross_entropy.py:243-260) with about ten [m]-sized torch operations and what autograd does on the
// way back with six more:
//     w_r    = (target_r == ignore_index) ? 0 : (weight ? weight[target_r] : 1)
//     sum    : result = sum_r w_r * loss_r
//     mean   : result = (sum_r w_r * loss_r) / (sum_r w_r)
//     back   : grad_r = (upstream / sum_r w_r) * w_r          (mean)       grad_r = upstream * w_r       (sum)
// Each side is one launch here.  The products w_r * loss_r are rounded to fp32 as the reference's are; the two sums
// are taken in double in a fixed order and rounded to fp32 once (torch adds in fp32 in an order of its own), the
// quotient is one correctly rounded fp32 division as in the reference, and the gradient per row is the same two
// fp32 operations in the same order, so it is bit-identical to what autograd computes from the same two sums.
#include "bmt_device.h"
#include "bmt_host.h"
#include "../../include/bmt_hip.h"

namespace bmt {

constexpr int kReduceThreads = 1024;

__device__ __forceinline__ float row_weight(int32_t t, const float *__restrict__ weight, int32_t n_classes, int32_t ignore_index) {
    if (t == ignore_index) return 0.f;
    if (!weight) return 1.f;
    return (uint32_t)t < (uint32_t)n_classes ? weight[t] : 0.f;       // a class outside the table weighs nothing
}

// One workgroup; lane t takes rows t, t + 1024, ... four at a time, then a fixed tree over the lanes.
__global__ __launch_bounds__(kReduceThreads) void loss_reduce_kernel(
    int64_t m, const float *__restrict__ losses, const int32_t *__restrict__ target, const float *__restrict__ weight,
    int32_t n_classes, int32_t ignore_index, int32_t mean, float *__restrict__ result, float *__restrict__ weight_sum) {
    double s = 0.0, w = 0.0;
    for (int64_t base = threadIdx.x; base < m; base += 4 * kReduceThreads) {
        float l[4];
        int32_t t[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int64_t i = base + (int64_t)u * kReduceThreads;
            l[u] = i < m ? losses[i] : 0.f;
            t[u] = i < m ? target[i] : ignore_index;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const float wi = row_weight(t[u], weight, n_classes, ignore_index);
            float prod = wi * l[u];
            asm("" : "+v"(prod));                  // the fp32 product exists as such before it is widened
            s += (double)prod;
            w += (double)wi;
        }
    }
    __shared__ double lanes_s[kReduceThreads], lanes_w[kReduceThreads];
    lanes_s[threadIdx.x] = s;
    lanes_w[threadIdx.x] = w;
    __syncthreads();
    for (int stride = kReduceThreads / 2; stride > 0; stride >>= 1) {
        if ((int)threadIdx.x < stride) {
            lanes_s[threadIdx.x] += lanes_s[threadIdx.x + stride];
            lanes_w[threadIdx.x] += lanes_w[threadIdx.x + stride];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float sum = (float)lanes_s[0], wsum = (float)lanes_w[0];
        weight_sum[0] = wsum;
        result[0] = mean ? sum / wsum : sum;       // 0 / 0 = NaN when every row is ignored, as in the reference
    }
}

__global__ __launch_bounds__(256) void loss_reduce_backward_kernel(
    int64_t m, const int32_t *__restrict__ target, const float *__restrict__ weight, int32_t n_classes, int32_t ignore_index,
    int32_t mean, const float *__restrict__ weight_sum, const float *__restrict__ upstream, float *__restrict__ grad_rows) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= m) return;
    float coef = upstream[0];
    if (mean) coef = coef / weight_sum[0];
    asm("" : "+v"(coef));
    grad_rows[i] = coef * row_weight(target[i], weight, n_classes, ignore_index);
}

}  // namespace bmt

extern "C" int cross_entropy_reduce_forward_launcher(int64_t m, const void *losses, const void *target, const void *weight,
                                                     int32_t n_classes, int32_t ignore_index, int32_t mean, void *result,
                                                     void *weight_sum, void *stream) {
    if (m < 0) return bmt::fail(-1, "cross_entropy_reduce_forward_launcher: negative row count");
    if (!result || !weight_sum || (m > 0 && (!losses || !target)))
        return bmt::fail(-1, "cross_entropy_reduce_forward_launcher: null pointer");
    if (weight && n_classes <= 0) return bmt::fail(-1, "cross_entropy_reduce_forward_launcher: weights without classes");
    hipLaunchKernelGGL(bmt::loss_reduce_kernel, dim3(1), dim3(bmt::kReduceThreads), 0, (hipStream_t)stream, m,
                       (const float *)losses, (const int32_t *)target, (const float *)weight, n_classes, ignore_index, mean,
                       (float *)result, (float *)weight_sum);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : bmt::fail((int)e, "cross_entropy_reduce_forward_launcher", e);
}

extern "C" int cross_entropy_reduce_backward_launcher(int64_t m, const void *target, const void *weight, int32_t n_classes,
                                                      int32_t ignore_index, int32_t mean, const void *weight_sum,
                                                      const void *upstream, void *grad_rows, void *stream) {
    if (m <= 0) return m < 0 ? bmt::fail(-1, "cross_entropy_reduce_backward_launcher: negative row count") : 0;
    if (!target || !upstream || !grad_rows || (mean && !weight_sum))
        return bmt::fail(-1, "cross_entropy_reduce_backward_launcher: null pointer");
    if (weight && n_classes <= 0) return bmt::fail(-1, "cross_entropy_reduce_backward_launcher: weights without classes");
    const int64_t grid = (m + 255) / 256;
    if (grid > 0x7FFFFFFF) return bmt::fail(-1, "cross_entropy_reduce_backward_launcher: too many rows for one launch");
    hipLaunchKernelGGL(bmt::loss_reduce_backward_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, m,
                       (const int32_t *)target, (const float *)weight, n_classes, ignore_index, mean, (const float *)weight_sum,
                       (const float *)upstream, (float *)grad_rows);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : bmt::fail((int)e, "cross_entropy_reduce_backward_launcher", e);
}
