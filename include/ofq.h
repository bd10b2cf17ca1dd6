/*
 * ofq.h -- C ABI of the MI355X (gfx950) kernels for OneFlow's quantized-inference op family.
 *
 * One entry point per OneFlow user op.  Each is what the op's `user_op::OpKernel::Compute`
 * would call after unpacking its `KernelComputeContext`: raw DEVICE pointers to contiguous
 * tensors, sizes, the op's attributes, and the HIP stream of `ctx->stream()`.
 *
 * Contract shared by every entry point (it mirrors what the OneFlow runtime guarantees a kernel,
 * oneflow/core/framework/op_kernel.h:287-324, oneflow/core/vm/op_call_instruction_policy.cpp:49-82):
 *   - the caller owns every buffer, including the workspace ("tmp_buffer"); nothing is allocated,
 *     freed or synchronised here, work is only enqueued on `stream` (a hipStream_t, may be NULL
 *     for the default stream), so the calls are safe under stream capture;
 *   - the return value is an ofq_status; invalid arguments are reported, never aborted on, and
 *     nothing is launched when the status is not OFQ_OK;
 *   - calls on different streams, and on different devices, may run concurrently.  The only
 *     state the library keeps is, per kernel, one bit per device saying that the kernel's
 *     dynamic-LDS limit has been raised there (set at the first launch on the device that is
 *     current in the calling thread; the caller makes the device of `stream` current, as the
 *     OneFlow worker thread that owns a stream does, oneflow/core/ep/cuda/cuda_stream.cpp:209-213);
 * Pointers must be aligned to 16 bytes (OneFlow's allocator aligns to 512,
 * oneflow/core/common/util.h:158-160).
 */
#ifndef OFQ_H_
#define OFQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  OFQ_OK = 0,
  OFQ_ERR_NULL_POINTER = 1,    /* a required tensor pointer is NULL, or an optional one is
                                  present/absent against `symmetric` */
  OFQ_ERR_BAD_DTYPE = 2,       /* dtype code not valid for this argument */
  OFQ_ERR_BAD_SHAPE = 3,       /* sizes inconsistent (divisibility, packing, limits) */
  OFQ_ERR_BAD_ATTR = 4,        /* attribute outside the op's domain */
  OFQ_ERR_UNSUPPORTED = 5,     /* valid for the op, but no kernel covers the combination */
  OFQ_ERR_WORKSPACE = 6,       /* workspace missing or smaller than *_workspace_bytes() */
  OFQ_ERR_MISALIGNED = 7,      /* a pointer is not 16-byte aligned */
  OFQ_ERR_LAUNCH = 8,          /* hipGetLastError() after the launch was not hipSuccess */
  OFQ_ERR_TOO_LARGE = 9        /* input beyond the fixed capacity of an entry point that
                                  allocates nothing and takes no workspace */
} ofq_status;

/* element types; values follow no OneFlow enum on purpose (the adapter maps DataType) */
typedef enum {
  OFQ_F32 = 0,
  OFQ_F16 = 1,
  OFQ_BF16 = 2,
  OFQ_F64 = 3,
  OFQ_I8 = 4,
  OFQ_U8 = 5
} ofq_dtype;

typedef enum { OFQ_SCHEME_SYMMETRIC = 0, OFQ_SCHEME_AFFINE = 1 } ofq_scheme;
typedef enum { OFQ_FORMULA_GOOGLE = 0, OFQ_FORMULA_CAMBRICON = 1 } ofq_formula;
/* how `quantization`/`fake_quantization` read an affine zero point:
 *   OFQ_ZP_FLOAT     as stored (the rule of the CUDA kernels this library replaces,
 *                    oneflow/user/kernels/quantization_kernel.cu:65-67),
 *   OFQ_ZP_UINT8     rounded to uint8 first (the rule of the CPU kernels,
 *                    oneflow/user/kernels/quantization_kernel.cpp:41-43). */
typedef enum { OFQ_ZP_FLOAT = 0, OFQ_ZP_UINT8 = 1 } ofq_zp_mode;
/* how LayerNorm takes the mean and the variance of a row:
 *   OFQ_LN_STATS_FP32  accumulated in fp32 (the reference's precision,
 *                      oneflow/core/cuda/layer_norm.cuh:212-233; the last bit of mean / inv then
 *                      depends on the order of summation, there as here)
 *   OFQ_LN_STATS_FP64  accumulated in fp64 and rounded once: the correctly rounded fp32 mean and
 *                      inv of the row, whatever the order -- y, scale and the codes made from them
 *                      are then reproducible bit for bit by any implementation of the same rule */
typedef enum { OFQ_LN_STATS_FP32 = 0, OFQ_LN_STATS_FP64 = 1 } ofq_ln_statistics;

const char* ofq_status_string(int status);
/* library ABI version; bumped on any signature change */
int ofq_abi_version(void);

/*
 * groupwise_dequantize
 * replaces GroupwiseDequantizeKernel<T>::Compute and its launchers,
 *   oneflow/user/kernels/groupwise_quantization_kernels.cu:394-454 (and :170-392).
 * The caller flattens the tensor the way the reference does (:436-437):
 *   outer = Count(0, group_dim) * num_groups, inner = Count(group_dim + 1) of the OUTPUT shape;
 *   out[outer][group_size][inner] = T(q) * scale[outer][inner] + zero[outer][inner], in T.
 * in:      in_dtype OFQ_U8 | OFQ_I8, codes packed along the tensor's last axis
 *          (num_bits 4: element 2i = high nibble of byte i); asymmetric requires OFQ_U8.
 * scale:   t_dtype OFQ_F16 | OFQ_BF16 | OFQ_F32, `outer*inner` elements.
 * zero:    same as scale; NULL iff symmetric != 0.
 * out:     t_dtype, outer*group_size*inner elements.
 */
int ofq_groupwise_dequantize(void* stream, const void* in, const void* scale, const void* zero,
                             void* out, int in_dtype, int t_dtype, int num_bits, int symmetric,
                             int64_t outer, int64_t group_size, int64_t inner);

/*
 * fused_linear_with_groupwise_quantized_weight
 * replaces FusedLinearWithGroupwiseQuantizedWeightKernel<T>::Compute and DispatchMatmulBias,
 *   oneflow/user/kernels/groupwise_quantization_kernels.cu:760-839 (and :465-749),
 * and, for m > 8, the dequantize -> matmul decomposition of the functor,
 *   oneflow/core/functional/impl/quantization.cpp:341-350.
 * x[m,k] (t_dtype), w[n, k*num_bits/8] (w_dtype OFQ_U8|OFQ_I8), w_scale / w_zero:
 *   [n, k/group_size] for group_dim 1, [n/group_size, k] for group_dim 0 (t_dtype),
 *   w_zero NULL iff symmetric, b[n] (t_dtype) or NULL, out[m,n] (t_dtype).
 * out = T( sum_k float(x * w~) + float(b) ), w~ = T(T(q)*scale) + zero as in groupwise_dequantize.
 *   One family of kernels departs from the rounding of w~: fp16, 4-bit symmetric codes in an
 *   int8 container (no zero term), groups along K with 128 | group_size, m <= 16 -- the Llama
 *   decode case.  There the group scale multiplies the exact fp32 sum of x*q over the group, so
 *   q*scale is never rounded to fp16; the result is closer to exact arithmetic and differs from
 *   the composition above by ~3e-4 rel-L2 (contract: 1e-3).  The same codes with groups along
 *   N (16 | group_size, 256 | k) at m = 1 take a kernel of that family in which the scale meets
 *   x instead (x*scale is rounded to fp16 once per k, q*scale never): the same ~3e-4.  Neither
 *   kernel rescales x by a constant: x meets the codes as stored, and x*scale is brought to a
 *   common power of two per 32 k before its rounding, so the bound holds for any magnitude of x
 *   and of the scales whose outputs are normal halves (tested from 1e-3 to hundreds).  Every
 *   other combination (uint8 container, a zero term, 8 bit, bf16, fp32, m > 16, groups along N
 *   otherwise) forms w~ with the two roundings of groupwise_dequantize.  The same weights in the two containers can therefore
 *   differ in the last bits of the output.
 * Any m is accepted (the reference kernel has no m limit either, :473,590).
 * workspace: optional.  ofq_fused_linear_gq_workspace_bytes() is non-zero only for large m on the
 *   GEMM path (n*k*sizeof(T)): with it the weight is dequantised once into the workspace and a
 *   copy-fed MFMA GEMM runs on the result (the functor's own m > 8 decomposition); with NULL or
 *   a smaller buffer the weight tiles are dequantised inside the GEMM instead (same results up to
 *   fp32 summation order, slower at large m).  With group_dim 0 it is n*k*sizeof(T) for m > 64
 *   (same decomposition; plus fp32 partial sums of K slices when there are few output tiles);
 *   without it the streaming kernel takes x 64 rows at a time.
 */
size_t ofq_fused_linear_gq_workspace_bytes(int w_dtype, int t_dtype, int num_bits, int symmetric,
                                           int group_dim, int64_t group_size, int64_t m,
                                           int64_t n, int64_t k);
int ofq_fused_linear_gq(void* stream, const void* x, const void* w, const void* w_scale,
                        const void* w_zero, const void* b, void* out, int w_dtype, int t_dtype,
                        int num_bits, int symmetric, int group_dim, int64_t group_size, int64_t m,
                        int64_t n, int64_t k, void* workspace, size_t workspace_bytes);

/*
 * min_max_observer
 * replaces GpuMinMaxObserverKernel<T>::Compute,
 *   oneflow/user/kernels/min_max_observer_kernel.cu:186-237 (arithmetic :117-163; CPU twin
 *   oneflow/user/kernels/min_max_observer_kernel.cpp:22-58).
 * in: in_dtype OFQ_F32 | OFQ_F64, elem_cnt elements; channels = 1 (per_layer_quantization) or
 * in.shape[0]; scale, zero_point: `channels` elements of in_dtype.
 * workspace: ofq_min_max_observer_workspace_bytes() (the op's "tmp_buffer", :247-254).
 */
size_t ofq_min_max_observer_workspace_bytes(int in_dtype, int64_t elem_cnt, int64_t channels);
int ofq_min_max_observer(void* stream, const void* in, void* scale, void* zero_point,
                         int in_dtype, int64_t elem_cnt, int64_t channels, int quantization_bit,
                         int scheme, int formula, void* workspace, size_t workspace_bytes);

/*
 * moving_average_min_max_observer (per-tensor only)
 * Replaces GpuMovingAverageMinMaxObserverKernel<T>::Compute,
 *   oneflow/user/kernels/moving_average_min_max_observer_kernel.cu:217-300
 * with the arithmetic of the CPU kernel, moving_average_min_max_observer_kernel.cpp:22-107.
 * in: elem_cnt values (OFQ_F32 | OFQ_F64); current_train_step: one int64 ON THE DEVICE (read by
 * the kernel: no host synchronisation, unlike the reference's cudaMemcpy at .cu:249-251);
 * moving_max / moving_min: one value each, updated in place while
 * `training && *current_train_step <= stop_update_after_iters`; scale / zero_point: one value each.
 * workspace: ofq_moving_average_min_max_observer_workspace_bytes().
 */
size_t ofq_moving_average_min_max_observer_workspace_bytes(int in_dtype, int64_t elem_cnt);
int ofq_moving_average_min_max_observer(void* stream, const void* in,
                                        const int64_t* current_train_step, void* moving_max,
                                        void* moving_min, void* scale, void* zero_point,
                                        int in_dtype, int64_t elem_cnt, int quantization_bit,
                                        int scheme, int formula, float momentum,
                                        int64_t stop_update_after_iters, int training,
                                        void* workspace, size_t workspace_bytes);

/*
 * quantization / fake_quantization
 * replace GpuQuantizationKernel<T>::Compute, oneflow/user/kernels/quantization_kernel.cu:107-144
 * (arithmetic :24-95) and GpuFakeQuantizationKernel<T>::Compute,
 * oneflow/user/kernels/fake_quantization_kernel.cu:24-96.
 * in: in_dtype OFQ_F32 | OFQ_F64 (the reference's types) or OFQ_F16 | OFQ_BF16 (dynamic
 *     activation path: scale/zero_point are then fp32 and the divide is done in fp32).
 * out: out_dtype == in_dtype (the reference: codes stored in the input type) or, for
 *     `quantization` only, OFQ_I8 (symmetric) / OFQ_U8 (affine) integer codes.
 * scale_size 1 = per-layer, else per-channel with scale_size == shape0 and panel = elem_cnt/shape0.
 */
int ofq_quantization(void* stream, const void* in, const void* scale, const void* zero_point,
                     void* out, int in_dtype, int out_dtype, int64_t elem_cnt, int64_t scale_size,
                     int quantization_bit, int scheme, int formula, int zp_mode);
int ofq_fake_quantization(void* stream, const void* in, const void* scale,
                          const void* zero_point, void* out, int in_dtype, int64_t elem_cnt,
                          int64_t scale_size, int quantization_bit, int scheme, int formula,
                          int zp_mode);

/*
 * fused_layer_norm_min_max_observer
 * The op is named by the task but absent from the reference tree; it composes
 *   LayerNorm over the last axis (oneflow/core/cuda/layer_norm.cuh:212-233,377-380 and the
 *   affine store of oneflow/user/kernels/layer_norm_gpu_kernel.cu:40-70) with a per-tensor
 *   symmetric min_max_observer (min_max_observer_kernel.cu:117-131) of the normalised output.
 * x, y: [rows, cols] t_dtype OFQ_F16 | OFQ_BF16 | OFQ_F32; gamma, beta: [cols] t_dtype or NULL;
 * scale, zero_point: one fp32 each.
 */
size_t ofq_fused_layer_norm_min_max_observer_workspace_bytes(int t_dtype, int64_t rows,
                                                             int64_t cols);
int ofq_fused_layer_norm_min_max_observer(void* stream, const void* x, const void* gamma,
                                          const void* beta, void* y, float* scale,
                                          float* zero_point, int t_dtype, int64_t rows,
                                          int64_t cols, double epsilon, int quantization_bit,
                                          void* workspace, size_t workspace_bytes);

/*
 * fused_layer_norm_min_max_observer for callers that cannot allocate device memory.
 * No counterpart in the reference (there the framework allocates every tmp_buffer before Compute):
 * it is for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc.  Same arguments and results (bit for bit) as the entry point above without the
 * workspace; the per-row partial maxima go to a fixed array in the library's device image
 * (OFQ_LN_STATIC_MAX_ROWS floats = 256 KB, present on every device the library runs on), whose
 * address is looked up once per device at the first call made with that device current (make
 * that first call outside stream capture).  Calls no hipMalloc / hipFree or allocating routine.
 * rows > 65536 returns OFQ_ERR_TOO_LARGE and launches nothing.  All calls on one device share
 * the array: calls that overlap on one device (different streams) race; calls on one stream do not.
 */
int ofq_fused_layer_norm_min_max_observer_static(void* stream, const void* x, const void* gamma,
                                                 const void* beta, void* y, float* scale,
                                                 float* zero_point, int t_dtype, int64_t rows,
                                                 int64_t cols, double epsilon,
                                                 int quantization_bit);

/*
 * fused_skip_layer_norm_min_max_observer: the op above on the input of skip_layer_norm,
 *   oneflow/user/kernels/skip_layer_norm_kernel.cu:36-67 (functional signature
 *   oneflow/core/functional/functional_api.yaml:1545-1546): the row that is normalised is
 *   (x + bias[c]) + skip * T(alpha), every operation in t_dtype; bias ([cols]) and skip
 *   ([rows, cols]) may each be NULL and then enter as zero.  Workspace as above.
 */
int ofq_fused_skip_layer_norm_min_max_observer(void* stream, const void* x, const void* bias,
                                               const void* skip, double alpha, const void* gamma,
                                               const void* beta, void* y, float* scale,
                                               float* zero_point, int t_dtype, int64_t rows,
                                               int64_t cols, double epsilon, int quantization_bit,
                                               void* workspace, size_t workspace_bytes);

/*
 * The two ops above with the precision of the row statistics as an attribute (ofq_ln_statistics).
 * No reference interface (the ops themselves are absent there).  with_skip = 0: the plain op
 * (bias, skip, alpha ignored); with_skip != 0: the skip_layer_norm input.  OFQ_LN_STATS_FP32 runs
 * the same kernels as the entry points above.
 */
int ofq_fused_layer_norm_min_max_observer_stats(
    void* stream, const void* x, const void* bias, const void* skip, double alpha, int with_skip,
    const void* gamma, const void* beta, void* y, float* scale, float* zero_point, int t_dtype,
    int64_t rows, int64_t cols, double epsilon, int quantization_bit, int statistics,
    void* workspace, size_t workspace_bytes);

/*
 * fused_layer_norm_quantization: fused_layer_norm_min_max_observer followed by `quantization`
 *   (symmetric, per layer, google formula, the same quantization_bit) of its output, without the
 *   normalised tensor reaching memory: codes[rows, cols] (int8), scale[1], zero_point[1] = 0.
 *   No reference interface: it is the dynamic activation quantisation in front of matmul_quant,
 *   i.e. the composition of the op above with
 *   oneflow/user/kernels/quantization_kernel.cu:107-156; the codes and the scale carry the same
 *   bits as that composition.  statistics as in ofq_fused_layer_norm_min_max_observer_stats.
 *   Served: fp16 rows of 512, 1024, 2048 or 4096 elements with gamma and beta, 16-byte aligned;
 *   any other case returns OFQ_ERR_UNSUPPORTED (nothing is launched) and the caller runs the two
 *   ops.  workspace: ofq_fused_layer_norm_quantization_workspace_bytes(), 16-byte aligned.
 */
size_t ofq_fused_layer_norm_quantization_workspace_bytes(int t_dtype, int64_t rows, int64_t cols);
int ofq_fused_layer_norm_quantization(void* stream, const void* x, const void* gamma,
                                      const void* beta, void* codes, float* scale,
                                      float* zero_point, int t_dtype, int64_t rows, int64_t cols,
                                      double epsilon, int quantization_bit, int statistics,
                                      void* workspace, size_t workspace_bytes);

/*
 * groupwise_quantize: the producer of the weight format of the two ops above.
 * The reference defines that format only through the helpers of its own test,
 *   python/oneflow/test/modules/test_groupwise_quantization.py:26-35 (int4 packing) and :46-81
 *   (`_quantize`),
 * whose fp32 arithmetic this follows exactly: x[n,k] (t_dtype) -> q[n, k*num_bits/8] (q_dtype
 * OFQ_U8 | OFQ_I8; asymmetric => OFQ_U8), scale and zero (t_dtype; zero NULL iff symmetric) of
 * shape [n, k/group_size] (group_dim 1) or [n/group_size, k] (group_dim 0).
 *   symmetric : scale = absmax/(2^(b-1)-1), q = rint(x/scale + offset), offset = 2^(b-1)-1 for
 *               OFQ_U8 and 0 for OFQ_I8;  asymmetric: scale = (max-min)/(2^b-1),
 *               q = rint((x-min)/scale), zero = min.
 * Codes use the unrounded fp32 scale; a group with scale 0 gets the code of value 0.
 */
int ofq_groupwise_quantize(void* stream, const void* x, void* q, void* scale, void* zero,
                           int t_dtype, int q_dtype, int num_bits, int symmetric, int group_dim,
                           int64_t group_size, int64_t n, int64_t k);

/*
 * grouped linear with groupwise-quantised weights: `count` (<= 64) independent problems
 *   outs[i][m_i, n_i] = fused_linear_with_groupwise_quantized_weight(xs[i], ws[i], ...)
 * in one call, the quantised counterpart of grouped_matmul_bias
 * (oneflow/user/kernels/grouped_matmul_bias.cu:153-204; functional signature
 * oneflow/core/functional/functional_api.yaml:2759-2760: TensorTuple xs, weights, biases -> ys).
 * As there, problems are grouped by shape: those of equal (m, k) with m <= 16 run as ONE launch
 * (any n_i; e.g. the q, k and v projections, or gate and up, of a decode step), the rest one
 * after the other.  All problems share the dtypes and the quantisation attributes.
 * xs, ws, w_scales, w_zeros, bs, outs: HOST arrays of `count` device pointers (w_zeros NULL iff
 * symmetric; bs NULL or with NULL entries for "no bias"); ms, ns, ks: HOST arrays.
 */
int ofq_grouped_linear_gq(void* stream, int count, const void* const* xs, const void* const* ws,
                          const void* const* w_scales, const void* const* w_zeros,
                          const void* const* bs, void* const* outs, const int64_t* ms,
                          const int64_t* ns, const int64_t* ks, int w_dtype, int t_dtype,
                          int num_bits, int symmetric, int group_dim, int64_t group_size);

/*
 * fused_glu with groupwise-quantised weights, the quantised counterpart of fused_glu
 * (oneflow/user/kernels/fused_glu_kernel.cu:303-347 for the gating, :566-770 for Compute;
 * functional signature oneflow/core/functional/functional_api.yaml:774-775 and the argument
 * rules of oneflow/core/functional/impl/nn_functor.cpp:3724-3800):
 *   matmul_wx = x w~^T + b, matmul_vx = x v~^T + c      (outputs, t_dtype [m, n])
 *   y = matmul_wx * act(matmul_vx)                       (act in fp32 on the widened gate,
 *                                                         rounded to t_dtype; product rounded)
 * Split mode (v != NULL): w and v are [n, k*bits/8] with their own scales / zeros, c NULL iff b
 * NULL.  Otherwise w is [2n, k*bits/8] (hidden-state rows first, gate rows second), b [2n] or
 * NULL, matmul_wx is [m, 2n] and v, v_scale, v_zero, c, matmul_vx are NULL.
 * activation: OFQ_ACT_*.  For m <= 16 the two linears of split mode are one launch.
 */
enum {
  OFQ_ACT_NONE = 0,
  OFQ_ACT_SIGMOID = 1,
  OFQ_ACT_RELU = 2,
  OFQ_ACT_GELU = 3,
  OFQ_ACT_FAST_GELU = 4,
  OFQ_ACT_SILU = 5
};
int ofq_fused_glu_gq(void* stream, const void* x, const void* w, const void* w_scale,
                     const void* w_zero, const void* b, const void* v, const void* v_scale,
                     const void* v_zero, const void* c, void* y, void* matmul_wx,
                     void* matmul_vx, int activation, int w_dtype, int t_dtype, int num_bits,
                     int symmetric, int group_dim, int64_t group_size, int64_t m, int64_t n,
                     int64_t k);

/*
 * matmul_quant
 * The op is named by the task but absent from the reference tree (only the env-var name
 * ONEFLOW_MLIR_GROUP_MATMUL_QUANT, python/oneflow/framework/infer_compiler/with_fx_graph.py:63);
 * operand conventions follow fused_matmul_bias (oneflow/ir/include/OneFlow/OneFlowUserOps.td:5615-5633):
 * a[m,k] int8, b[n,k] int8 (weight layout), exact int32 accumulation,
 * out[m,n] = T( float(acc) * (a_scale[0] * b_scale[n]) + float(bias[n]) ), out_dtype OFQ_F16 |
 * OFQ_BF16 | OFQ_F32; a_scale: one fp32 on the device; b_scale: fp32[n]; bias: out_dtype[n] or NULL.
 * k has to be a multiple of 64.  m <= 64 streams the weights once (decode); larger m runs the
 * tiled int8 MFMA GEMM (k a multiple of 128; else 64 rows of a per pass of the streaming kernel).
 */
int ofq_matmul_quant(void* stream, const void* a, const void* b, const float* a_scale,
                     const float* b_scale, const void* bias, void* out, int out_dtype, int64_t m,
                     int64_t n, int64_t k);
/*
 * The same op with an optional workspace (the op's tmp_buffer).  ofq_matmul_quant_workspace_bytes()
 * is non-zero when 64 < m and the 128-wide output tiles alone would leave most CUs without a
 * block: K is then cut into up to 8 slices that run as separate blocks, each writing its int32
 * partial sums to the workspace (splits * m * n * 4 bytes), and a second kernel adds the slices
 * (integer addition: the result does not depend on the order) and applies the epilogue.  Same
 * bits as ofq_matmul_quant, which is this call with workspace NULL.
 */
size_t ofq_matmul_quant_workspace_bytes(int64_t m, int64_t n, int64_t k);
int ofq_matmul_quant_ws(void* stream, const void* a, const void* b, const float* a_scale,
                        const float* b_scale, const void* bias, void* out, int out_dtype,
                        int64_t m, int64_t n, int64_t k, void* workspace, size_t workspace_bytes);

/*
 * Offline tile-major copy of 4-bit weights for the decode kernels at 2 to 16 rows of x.  No
 * counterpart in the reference, whose only weight format is the row-major [n, k/2] array of
 * python/oneflow/test/modules/test_groupwise_quantization.py:26-81; this is the pre-shuffled
 * variant of that format.  The row-balanced decode kernel gives every block of its grid
 * rows_per_block consecutive weight rows (a function of n alone) and walks them as 16-row
 * tiles, a lane (k-slot kb, row r) taking 16 bytes of each 64-byte chunk of its row: in the
 * row-major array one request of a wave is 16 pieces of 64 bytes.  The copy stores, for block b,
 * tile t and chunk c, those 64 x 16 bytes as one contiguous KB in lane order,
 *   tiled[((b * tiles_per_block + t) * (k/128) + c) * 1024 + (kb * 16 + r) * 16 + 0..15]
 *     = w[b * rows_per_block + 16 t + r][64 c + 16 kb + 0..15],
 * zeros for rows beyond the block's share.  Scales, zeros and bias keep the reference layout.
 * ofq_groupwise_repack_bytes: size of the copy (0: no tile-major form for this shape; 4-bit
 * codes and 128 | k only).  ofq_fused_linear_gq_tiled: ofq_fused_linear_gq on the copy, same
 * argument meaning, same bits in `out` as the row-major call (tested); OFQ_ERR_UNSUPPORTED
 * outside fp16, groups of a multiple of 128 along K, m <= 16 and m * k * 2 bytes of x within
 * LDS -- callers keep the row-major array for everything else (prefill, one row of x, where the
 * kernel that reads whole rows is the faster one).
 */
size_t ofq_groupwise_repack_bytes(int num_bits, int64_t n, int64_t k);
int ofq_groupwise_repack(void* stream, const void* w, void* w_tiled, int num_bits, int64_t n,
                         int64_t k);
int ofq_fused_linear_gq_tiled(void* stream, const void* x, const void* w_tiled,
                              const void* w_scale, const void* w_zero, const void* b, void* out,
                              int w_dtype, int t_dtype, int num_bits, int symmetric,
                              int group_dim, int64_t group_size, int64_t m, int64_t n, int64_t k);

#ifdef __cplusplus
}
#endif
#endif /* OFQ_H_ */
