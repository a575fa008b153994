/*
 * C ABI of libbmt_hip.so — the MI355X (gfx950) replacement for the hot-path
 * part of BMTrain's compiled extension `bmtrain.C`.
 *
 * Every entry point has the name and positional argument order of the function
 * that the reference registers under `bmtrain.C` (csrc/bind.cpp:3-35, prototypes
 * in csrc/include/bind.hpp:5-111 and csrc/include/adam_cpu.hpp), so that a
 * binding layer can forward its arguments unchanged.  Differences, all supersets:
 *   - element counts are int64_t (the reference takes int/int32_t for the GPU
 *     launchers); flat buffers beyond 2^31 elements are supported;
 *   - pointers are typed `void *` instead of std::uintptr_t integers;
 *   - every function returns int: 0 on success, otherwise a hipError_t value
 *     (GPU launchers) or -1 (invalid argument); the reference returns void and
 *     never looks at the launch status.  bmt_hip_last_error() describes the last
 *     failure of the calling thread.
 *
 * Ownership: the caller owns every buffer; the library allocates no device memory
 * and retains no pointer into a caller's buffer.  GPU launchers are asynchronous on
 * `stream` (a hipStream_t; NULL = the default stream) and never synchronise.
 * Device pointers and the stream must belong to the device that is current at the call.
 *
 * State the library does keep (everything else is stateless, as the reference's launchers are):
 *   - host side: the parked worker threads of adam_cpu_*_launcher; per device, a table of up to 256
 *     stream handles (which stream uses which group of ticket counters below) behind one mutex, 1 KiB of pinned host memory, the
 *     looked-up addresses of the two device arrays, and the cached compute-unit count;
 *   - device side, two fixed arrays in the library's own code object, one copy per GPU: 32 KiB of
 *     ticket counters for the in-place cross-entropy kernels and the long single-tensor Adam launches
 *     (eight counters per stream in the table; every launch leaves them at zero)
 *     and the 4 MiB of partial sums of grad_stats_noalloc_launcher;
 *   - in a caller's buffer, only for the duration of a launch: long Adam launches on a stream without a
 *     table entry, and long multi-tensor launches, keep four tile counters in the 16-bit parameter
 *     output (see adam_fp16_launcher).
 * Launches that use a table entry are numbered, and the last workgroup of each writes its number into a
 * word of pinned host memory (1 KiB per device, allocated at the first such launch).  When the table is
 * full, the least recently used entry whose latest launch has left is given to the new stream; if the
 * entries looked at are all busy the launch does without an entry: the cross-entropy kernels run their
 * one-tile-per-workgroup form, Adam keeps its counters in param_16 (same results, a few per cent
 * slower).  Stream handles in the table are only compared, never handed to the runtime.  Launches on a
 * stream under graph capture, on hipStreamPerThread or on a stream of another device never get an entry.
 */
#ifndef BMT_HIP_H
#define BMT_HIP_H

#include <stdint.h>

/* The library is built with hidden visibility; only these entry points are exported. */
#define BMT_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

/* csrc/cuda/has_inf_nan.cu:140-145.  Always 1 on gfx950. */
BMT_API int is_bf16_supported(void);

/* Human-readable text for the last non-zero return value on this thread. */
BMT_API const char *bmt_hip_last_error(void);

/*
 * has_nan_inf_{fp16,bf16}_launcher — csrc/cuda/has_inf_nan.cu:101-138 (bind.hpp:7-8).
 * Sets out[0] = 1 (uint8) iff some g[i], 0 <= i < n, is +-inf or NaN; leaves out[0]
 * untouched otherwise (the flag is sticky across calls).  n <= 0 is a no-op.
 * `mid` is the reference's uint8[1024] scratch; it is accepted and not used.
 */
BMT_API int has_nan_inf_fp16_launcher(int64_t n, const void *g_fp16, void *mid, void *out, void *stream);
BMT_API int has_nan_inf_bf16_launcher(int64_t n, const void *g_bf16, void *mid, void *out, void *stream);

/*
 * adam_fp16_launcher — csrc/cuda/adam_cuda.cu:76-101 (kernel :8-37; bind.hpp:82-96).
 * One fused step over n elements.  fp16 flavour: g is the loss-scaled gradient and
 * the moments are kept multiplied by `scale` (m in fp16, v in fp32).
 * Writes param_fp32, param_fp16 (round-to-nearest-even), m_fp16, v_fp32.  n <= 0: no-op.
 * param_fp16 is output only and its previous contents are never read.  A launch of 25,165,824 elements
 * or more (bf16 flavour: 10,485,760 or more) hands out its tiles through counters: those of the
 * stream's entry in the library's table (see "State" above) or, where the stream has none (graph
 * capture, hipStreamPerThread, table busy), four of the last 1,537 8-byte groups of param_fp16,
 * which then hold counters while the launch is in flight (set by a small kernel in front, replaced
 * by the real values by one behind, in stream order).  A call whose param_fp16 overlaps g_fp16,
 * param_fp32, m_fp16 or v_fp32 returns -1, at any size and on any stream.
 */
BMT_API int adam_fp16_launcher(int64_t n, void *param_fp32, void *param_fp16, const void *g_fp16,
                       void *m_fp16, void *v_fp32,
                       float beta1, float beta2, float eps, float lr, float scale,
                       float weight_decay, float bias_correction1, float bias_correction2,
                       void *stream);

/*
 * adam_bf16_launcher — csrc/cuda/adam_cuda.cu:103-126 (kernel :39-72; bind.hpp:97-111).
 * bf16 flavour: g is divided by `scale`; m and v are plain fp32 moments.
 */
BMT_API int adam_bf16_launcher(int64_t n, void *param_fp32, void *param_bf16, const void *g_bf16,
                       void *m_fp32, void *v_fp32,
                       float beta1, float beta2, float eps, float lr, float scale,
                       float weight_decay, float bias_correction1, float bias_correction2,
                       void *stream);

/*
 * adam_cpu_{fp16,bf16}_launcher — csrc/include/adam_cpu.hpp:504-533 and :535-557.
 * Host-memory (optimizer-offload) Adam step; all pointers are host pointers.
 * delta_info is NULL or float[4] receiving {mean, variance, sum, sum of squares} of the
 * per-element update m/bc1/(sqrt(v/bc2)+eps) + wd*p.  The fp16 copy is rounded to
 * nearest even, the bf16 copy is truncated, as in the reference.
 */
BMT_API int adam_cpu_fp16_launcher(int64_t n, void *param_fp32, void *param_fp16, void *delta_info,
                           const void *g_fp16, void *m_fp32, void *v_fp32,
                           float beta1, float beta2, float eps, float lr, float scale,
                           float weight_decay, float bias_correction1, float bias_correction2);
BMT_API int adam_cpu_bf16_launcher(int64_t n, void *param_fp32, void *param_bf16, void *delta_info,
                           const void *g_bf16, void *m_fp32, void *v_fp32,
                           float beta1, float beta2, float eps, float lr, float scale,
                           float weight_decay, float bias_correction1, float bias_correction2);

/*
 * to_fp16_from_fp32 / to_bf16_from_fp32 — bind.cpp:4-5 ->
 * fp16_from_fp32_value_launcher / bf16_from_fp32_value_launcher
 * (csrc/include/adam_cpu.hpp:139-175).  Host pointers.  fp16: round to nearest even;
 * bf16: truncation.
 */
BMT_API int to_fp16_from_fp32(int64_t n, const void *param_fp32, void *param_fp16);
BMT_API int to_bf16_from_fp32(int64_t n, const void *param_fp32, void *param_bf16);

/*
 * cross_entropy_forward_{fp16,bf16}_launcher — csrc/cuda/cross_entropy.cu:202-217,
 * :234-247 (kernels :9-43, :63-101; bind.hpp:20-28, :38-46).
 * input, softmax: [m, n] row-major 16-bit; target: int32[m]; output: float[m].
 *   softmax[r, :] = softmax(input[r, :]) rounded to the 16-bit type,
 *   output[r]     = target[r] != ignore_index ? logsumexp(input[r, :]) - input[r, target[r]] : 0.
 * m <= 0 or n <= 0 is a no-op (the reference would issue an invalid launch).
 * softmax must not share memory with input: the loss is taken from input[r, target[r]] after
 * the row's softmax has been stored (cross_entropy.cu:30-36 has the same order and gives an
 * undefined loss in place); an overlapping pair is refused with status -1.
 */
BMT_API int cross_entropy_forward_fp16_launcher(int32_t m, int32_t n, const void *input, const void *target,
                                        void *softmax, void *output, int32_t ignore_index, void *stream);
BMT_API int cross_entropy_forward_bf16_launcher(int32_t m, int32_t n, const void *input, const void *target,
                                        void *softmax, void *output, int32_t ignore_index, void *stream);

/*
 * cross_entropy_backward_inplace_{fp16,bf16}_launcher — csrc/cuda/cross_entropy.cu:219-232,
 * :249-261 (kernels :46-60, :104-121; bind.hpp:29-37, :47-53).
 * x holds the softmax written by the forward call and is overwritten with the gradient:
 *   x[r, i] = to16((x[r, i] - (i == target[r])) * grad_output[r]).
 * As in the reference, ignore_index is not consulted: ignored rows are zeroed by the caller
 * passing grad_output[r] = 0.
 */
BMT_API int cross_entropy_backward_inplace_fp16_launcher(int32_t m, int32_t n, const void *grad_output,
                                                 const void *target, void *x, int32_t ignore_index,
                                                 void *stream);
BMT_API int cross_entropy_backward_inplace_bf16_launcher(int32_t m, int32_t n, const void *grad_output,
                                                 const void *target, void *x, int32_t ignore_index,
                                                 void *stream);

/*
 * fused_sumexp_{fp16,bf16}_launcher — csrc/cuda/cross_entropy.cu:263-288 (kernels :124-164;
 * bind.hpp:54-67).  sum_exp_logits[r] = sum_i expf(logits[r, i] - max_logits[r]).
 */
BMT_API int fused_sumexp_fp16_launcher(int32_t m, int32_t n, const void *logits, const void *max_logits,
                               void *sum_exp_logits, void *stream);
BMT_API int fused_sumexp_bf16_launcher(int32_t m, int32_t n, const void *logits, const void *max_logits,
                               void *sum_exp_logits, void *stream);

/*
 * fused_softmax_inplace_{fp16,bf16}_launcher — csrc/cuda/cross_entropy.cu:290-315
 * (kernels :167-199; bind.hpp:68-81).
 * logits[r, i] = to16(expf(logits[r, i] - max_logits[r]) / sum_exp_logits[r]).
 */
BMT_API int fused_softmax_inplace_fp16_launcher(int32_t m, int32_t n, void *logits, const void *max_logits,
                                        const void *sum_exp_logits, void *stream);
BMT_API int fused_softmax_inplace_bf16_launcher(int32_t m, int32_t n, void *logits, const void *max_logits,
                                        const void *sum_exp_logits, void *stream);

/*
 * cross_entropy_reduce_{forward,backward}_launcher — no counterpart in the reference's extension: the
 * reduction of the per-row losses that FusedCrossEntropy.forward spells out in torch operations
 * (bmtrain/loss/cross_entropy.py:243-260) and its autograd backward, one launch each.
 *   w_r = target[r] == ignore_index ? 0 : (weight ? weight[target[r]] : 1)       (weight: float[n_classes] or NULL;
 *                                                                                 a class outside the table weighs 0)
 *   forward:  weight_sum[0] = sum_r w_r;  result[0] = sum_r w_r * losses[r], divided by weight_sum[0] when `mean`
 *   backward: grad_rows[r] = (mean ? upstream[0] / weight_sum[0] : upstream[0]) * w_r
 * losses, grad_rows: float[m]; target: int32[m]; result, weight_sum, upstream: one float each, all on the device.
 * The sums are taken in double in a fixed order and rounded to float once; the forward launch is one workgroup
 * (meant for row counts up to about a million).
 */
BMT_API int cross_entropy_reduce_forward_launcher(int64_t m, const void *losses, const void *target, const void *weight,
                                                  int32_t n_classes, int32_t ignore_index, int32_t mean, void *result,
                                                  void *weight_sum, void *stream);
BMT_API int cross_entropy_reduce_backward_launcher(int64_t m, const void *target, const void *weight, int32_t n_classes,
                                                   int32_t ignore_index, int32_t mean, const void *weight_sum,
                                                   const void *upstream, void *grad_rows, void *stream);

/*
 * adam_{fp16,bf16}_multi_launcher — no counterpart in the reference's extension, which is called once
 * per parameter tensor from the Python loop of AdamOptimizer.step (bmtrain/optim/adam.py:72-159).  Steps
 * `count` tensors that share their hyper-parameters (same group, same step count) in as few launches as
 * possible; per element the arithmetic is that of adam_{fp16,bf16}_launcher, bit for bit.
 * `tensors` is a host array; `m` is float[n] for bf16 and half[n] for fp16.  Entries with n <= 0 are skipped.
 * param_16 is output only; a launch over 25,165,824 elements or more (bf16: 12,582,912 or more) keeps four tile counters in the
 * param_16 of its largest tensor while it runs (as adam_fp16_launcher does).  The whole table is checked before
 * the first launch: the call returns -1, and no tensor has been stepped, if any entry has a null pointer or a
 * param_16 that overlaps an input of the same tensor.  A batch in which another entry shares memory with the
 * counters' place runs on the kernel that keeps no counters.
 */
typedef struct bmt_adam_tensor {
    void *param_fp32;
    void *param_16;
    const void *grad_16;
    void *m;
    void *v;
    int64_t n;
} bmt_adam_tensor;
BMT_API int adam_bf16_multi_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2, float eps,
                             float lr, float scale, float weight_decay, float bias_correction1,
                             float bias_correction2, void *stream);
BMT_API int adam_fp16_multi_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2, float eps,
                             float lr, float scale, float weight_decay, float bias_correction1,
                             float bias_correction2, void *stream);

/*
 * adam_{fp16,bf16}_multi_clip_launcher — no counterpart in the reference's extension.  The same step with
 * gradient clipping applied on the fly: every gradient element enters as to16(float(g) * grad_coef), which is
 * what the reference's eager clipping (`p.grad.mul_(clip_coef)`, bmtrain/optim/optim_manager.py:196-199)
 * leaves in memory when grad_coef is the clipping factor rounded to the gradient's 16-bit type; the gradients
 * themselves are not modified.  grad_coef = 1 is the unclipped step.
 */
BMT_API int adam_bf16_multi_clip_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2, float eps,
                                  float lr, float scale, float weight_decay, float bias_correction1,
                                  float bias_correction2, float grad_coef, void *stream);
BMT_API int adam_fp16_multi_clip_launcher(int32_t count, const bmt_adam_tensor *tensors, float beta1, float beta2, float eps,
                                  float lr, float scale, float weight_decay, float bias_correction1,
                                  float bias_correction2, float grad_coef, void *stream);

/*
 * grad_stats_{fp16,bf16}_launcher — no single counterpart in the reference's extension: one pass over
 * a gradient buffer that yields both quantities OptimManager needs before a step, where the reference
 * makes several (optim_manager.py:9-21 `check_overflow` via has_nan_inf_*_launcher, and :186-190
 * `g.float().norm(2) ** 2` through torch, which writes and re-reads an fp32 copy of every gradient).
 *   flag[0]  (uint8)  = 1 iff some g[i] is +-inf or NaN, else untouched (sticky, as has_nan_inf_*);
 *   sumsq[0] (double) += sum_i g[i]^2   (accumulated, so that several tensors add into one total).
 * workspace: float[grad_stats_workspace_floats(n)] of device memory owned by the caller; its content
 * is overwritten.  The summation order is fixed, so equal inputs give equal bits.  n <= 0 is a no-op.
 */
BMT_API int64_t grad_stats_workspace_floats(int64_t n);
BMT_API int grad_stats_fp16_launcher(int64_t n, const void *g_fp16, void *sumsq, void *flag, void *workspace,
                             void *stream);
BMT_API int grad_stats_bf16_launcher(int64_t n, const void *g_bf16, void *sumsq, void *flag, void *workspace,
                             void *stream);

/*
 * grad_stats_noalloc_launcher — no counterpart in the reference.  For callers that cannot allocate device
 * memory (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc): the pass of
 * grad_stats_{fp16,bf16}_launcher with its partial sums kept in a fixed 4 MiB array inside the library's own
 * device image instead of a caller's workspace, so the call allocates nothing.  is_bf16: 0 = fp16 gradients,
 * otherwise bf16.  Same results as the workspace form, bit for bit.  n above 2^36 elements is refused (-1).
 * Every call on one GPU uses that GPU's one array: calls that overlap in time on the same GPU (two streams, two
 * threads) race on it; calls that follow each other on one stream do not.
 */
BMT_API int grad_stats_noalloc_launcher(int64_t n, const void *g_16, int32_t is_bf16, void *sumsq, void *flag,
                                        void *stream);

/*
 * grad_stats_multi_launcher — no counterpart in the reference, whose overflow check and gradient norm loop
 * over the parameters (bmtrain/optim/optim_manager.py:9-21, :186-190).  The passes of has_nan_inf_*_launcher
 * (sumsq == NULL: only the sticky flag) or of grad_stats_*_launcher (sumsq != NULL: flag, and the sum of squares
 * of all tensors accumulated into sumsq[0]) over `count` gradient tensors of one 16-bit type in as few launches
 * as possible (64 tensors each).  `tensors` is a host array; entries with n <= 0 are skipped; the tensors may
 * start at any 2-byte aligned address.  `workspace` (device, floats): at least the sum over the tensors of
 * grad_stats_workspace_floats(n); not used when sumsq is NULL.  The table is checked before the first launch.
 */
typedef struct bmt_scan_tensor {
    const void *g_16;
    int64_t n;
} bmt_scan_tensor;
BMT_API int grad_stats_multi_launcher(int32_t count, const bmt_scan_tensor *tensors, int32_t is_bf16, void *sumsq,
                                      void *flag, void *workspace, void *stream);

/*
 * bmt_hip_flat_stream_stats — diagnostics, no counterpart in the reference.  For the current device, since the
 * library was loaded: out[0] = launches of the in-place cross-entropy / softmax kernels that ran as the resident
 * ticket-ordered grid, out[1] = large launches that could not get ticket counters (stream under capture,
 * hipStreamPerThread, stream of another device, stream table full of busy streams) and took the
 * workgroup-per-tile kernel, out[2] = stream-table entries handed from one stream to another.
 */
BMT_API int bmt_hip_flat_stream_stats(int64_t *out);

#ifdef __cplusplus
}
#endif
#endif /* BMT_HIP_H */
