/*
 * libattorch_hip — C ABI of the MI355X (gfx950) kernels behind the attorch layer API.
 *
 * The reference (BobMcDear/attorch) has no FFI: its device boundary is the Triton launch
 * `kernel[grid](tensor pointers, dims, strides, constexpr flags)` inside each
 * torch.autograd.Function.  Every entry point below replaces one such launch (or the torch
 * call the reference delegates to) and keeps its argument meaning; the reference site is
 * cited above each declaration as attorch/<file>:<lines>.
 *
 * Rules common to every entry point
 *   - all pointers are device pointers; the caller allocates every output and every
 *     workspace (the library never allocates, frees or keeps device memory)
 *   - "nullable" pointers are null exactly where the reference passes None
 *   - tensors are row-major with unit stride in the last dimension; row strides are given
 *     in elements
 *   - dtype arguments take AT_DTYPE_*; arithmetic is always fp32
 *   - the work is enqueued on `stream` (a hipStream_t, null = default stream); no call
 *     synchronises the device
 *   - return value: 0 on success, > 0 a hipError_t from the launch, < 0 an AT_ERR_* argument
 *     error (checked before any device call, so argument errors are reported without a GPU)
 *   - results are bit-reproducible: no floating-point atomics are used anywhere
 */
#ifndef ATTORCH_HIP_H
#define ATTORCH_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AT_OK 0
#define AT_ERR_NULL (-1)        /* a required pointer is null */
#define AT_ERR_DIM (-2)         /* a dimension or stride is out of range */
#define AT_ERR_DTYPE (-3)       /* unknown dtype or unsupported dtype combination */
#define AT_ERR_ACT (-4)         /* unknown activation id */
#define AT_ERR_WORKSPACE (-5)   /* workspace missing or too small */
#define AT_ERR_ALIGN (-6)       /* pointer or stride alignment the kernel cannot serve */
#define AT_ERR_UNSUPPORTED (-7) /* valid arguments, configuration not implemented */

#define AT_DTYPE_F32 0
#define AT_DTYPE_F16 1
#define AT_DTYPE_BF16 2

/* Activation ids: the strings accepted by attorch/linear_layer.py:42-49 and dispatched by
 * apply_act_func / apply_act_func_grad, attorch/act_kernels.py:631-837. */
#define AT_ACT_NONE 0
#define AT_ACT_SIGMOID 1
#define AT_ACT_LOGSIGMOID 2
#define AT_ACT_TANH 3
#define AT_ACT_RELU 4
#define AT_ACT_GELU 5
#define AT_ACT_GELUAPPROX 6
#define AT_ACT_SILU 7
#define AT_ACT_RELU6 8
#define AT_ACT_HARDSIGMOID 9
#define AT_ACT_HARDTANH 10
#define AT_ACT_HARDSWISH 11
#define AT_ACT_SELU 12
#define AT_ACT_MISH 13
#define AT_ACT_SOFTPLUS 14
#define AT_ACT_SOFTSIGN 15
#define AT_ACT_TANHSHRINK 16
#define AT_ACT_LEAKY_RELU 17
#define AT_ACT_ELU 18
#define AT_ACT_CELU 19
#define AT_ACT_HARDSHRINK 20
#define AT_ACT_SOFTSHRINK 21
#define AT_ACT_COUNT 22

typedef void* at_stream_t;

/* Library version (major * 10000 + minor * 100 + patch). */
int at_version(void);

/* Static description of a return code of this library (never null). */
const char* at_error_string(int code);

/* Measurement aid with no counterpart in the reference: v_mfma_f32_32x32x16_bf16 back to back on
 * every CU (two workgroups of four waves each), operands and accumulators in registers, no memory
 * traffic.  random_operands != 0: the operands are pseudo-random values in [-1, 1) that change
 * from one MFMA to the next, as in a real product; 0: one constant pair.  The caller times the
 * launch; at_mfma_probe_flop(iters) is the arithmetic it performs.  scratch4: 4 writable bytes of
 * device memory (never written in practice).  The rate with changing operands is what the matrix
 * cores of this device sustain under their power limit; the nominal peak is only reached with
 * constant operands. */
int at_mfma_probe(int64_t iters, int random_operands, void* scratch4, at_stream_t stream);
int64_t at_mfma_probe_flop(int64_t iters);

/* ------------------------------------------------------------------------------------------
 * RMSNorm — replaces rms_norm_forward_kernel / rms_norm_backward_kernel,
 * attorch/rms_norm_kernels.py:21-88 and :98-193, launched from attorch/rms_norm_layer.py:68-75
 * and :114-124.
 *   fwd: inv_rms = rsqrt(sum(x^2)/feat + eps); y = x * inv_rms (* weight)
 *   bwd: g = weight*dy; dx = inv_rms*(g - x*sum(x*g)*inv_rms^2/feat); weight_grad = sum_rows dy*x*inv_rms
 * weight (nullable) = scale_by_weight False; inv_rms (nullable in fwd) = save_stats False.
 * weight_grad is fp32 [feat] and is the finished column sum (the reference writes per-program
 * partial rows and sums them with torch, rms_norm_layer.py:126-127; here the partial rows live in
 * `workspace`, at least at_norm_bwd_workspace_bytes(batch, feat, 1) bytes, and are reduced by a
 * second launch in fixed order).
 * ------------------------------------------------------------------------------------------ */
int at_rms_norm_fwd(const void* x, const void* weight, float* inv_rms, void* y,
                    int64_t batch, int64_t feat, int64_t x_stride, int64_t y_stride, float eps,
                    int x_dtype, int weight_dtype, int y_dtype, at_stream_t stream);

int at_rms_norm_bwd(const void* dy, const void* x, const float* inv_rms, const void* weight,
                    void* dx, float* weight_grad, void* workspace, int64_t workspace_bytes,
                    int64_t batch, int64_t feat, int64_t dy_stride, int64_t x_stride,
                    int64_t dx_stride, int dy_dtype, int x_dtype, int weight_dtype, int dx_dtype,
                    at_stream_t stream);

/* Bytes of workspace the norm backward kernels need for `n_param_grads` (1 = weight only,
 * 2 = weight and bias) fp32 parameter gradients; 0 when n_param_grads is 0. */
int64_t at_norm_bwd_workspace_bytes(int64_t batch, int64_t feat, int n_param_grads);

/* ------------------------------------------------------------------------------------------
 * LayerNorm — replaces layer_norm_forward_kernel / layer_norm_backward_kernel,
 * attorch/layer_norm_kernels.py:21-101 and :111-224, launched from
 * attorch/layer_norm_layer.py:77-85 and :137-148 (+ the torch sums at :150-153).
 *   fwd: mean = sum(x)/feat; inv_std = rsqrt(sum((x-mean)^2)/feat + eps);
 *        y = (x-mean)*inv_std (* weight (+ bias))
 *   bwd: xh = (x-mean)*inv_std; g = weight*dy;
 *        dx = inv_std*(g - xh*mean(xh*g) - mean(g)); weight_grad = sum_rows dy*xh; bias_grad = sum_rows dy
 * bias is ignored when weight is null (layer_norm_layer.py:60). mean/inv_std nullable in fwd.
 * ------------------------------------------------------------------------------------------ */
int at_layer_norm_fwd(const void* x, const void* weight, const void* bias, float* mean,
                      float* inv_std, void* y, int64_t batch, int64_t feat, int64_t x_stride,
                      int64_t y_stride, float eps, int x_dtype, int weight_dtype, int y_dtype,
                      at_stream_t stream);

int at_layer_norm_bwd(const void* dy, const void* x, const float* mean, const float* inv_std,
                      const void* weight, void* dx, float* weight_grad, float* bias_grad,
                      void* workspace, int64_t workspace_bytes, int64_t batch, int64_t feat,
                      int64_t dy_stride, int64_t x_stride, int64_t dx_stride, int dy_dtype,
                      int x_dtype, int weight_dtype, int dx_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Softmax / LogSoftmax / Softmin over the last dimension — replaces softmax_forward_kernel /
 * softmax_backward_kernel, attorch/softmax_kernels.py:43-103 and :113-181, launched from
 * attorch/softmax_layers.py:50-52 and :82-86.  neg = softmin, log = log-softmax.
 *   bwd (from the saved OUTPUT y): softmax dx = y*(dy - sum(dy*y)); log dx = dy - exp(y)*sum(dy);
 *   negated when neg.
 * ------------------------------------------------------------------------------------------ */
int at_softmax_fwd(const void* x, void* y, int64_t batch, int64_t feat, int64_t x_stride,
                   int64_t y_stride, int neg, int log, int x_dtype, int y_dtype, at_stream_t stream);

int at_softmax_bwd(const void* dy, const void* y, void* dx, int64_t batch, int64_t feat,
                   int64_t dy_stride, int64_t y_stride, int64_t dx_stride, int neg, int log,
                   int dy_dtype, int y_dtype, int dx_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Cross entropy (mean reduction, optional class weights, ignore_index) — replaces
 * cross_entropy_loss_forward_kernel / cross_entropy_loss_backward_kernel,
 * attorch/cross_entropy_loss_kernels.py:21-86 and :96-172, the torch sums at
 * attorch/cross_entropy_loss_layer.py:76-80, and adds ignore_index (absent upstream, :144).
 * One pass over the logits produces the loss and, when dlogits is non-null, the gradient for an
 * upstream gradient of 1:  dlogits = (softmax - onehot(target)) * w[target] / denom, with
 * denom = sum of w[target] over kept rows (or the kept-row count when weight is null).
 * Rows whose target equals ignore_index — or lies outside [0, feat) — contribute nothing and
 * get an all-zero gradient row. loss is one element of loss_dtype, dlogits has out_dtype;
 * workspace needs at_cross_entropy_workspace_bytes(batch) bytes; on return workspace[0] (fp32)
 * holds denom.  dlogits may have the dtype of the logits or be fp32 (the reference's autocast
 * policy computes an fp32 loss and gradient for 16-bit logits, cross_entropy_loss_layer.py:59,108;
 * autograd then rounds that gradient to the dtype of the logits, which out_dtype = logits_dtype
 * with loss_dtype = fp32 produces in one step).
 * at_cross_entropy_bwd is the reference's backward kernel (cross_entropy_loss_kernels.py:96-172):
 * dlogits = output_grad * (softmax - onehot) * w[target] / denom, recomputed from the logits,
 * with output_grad read on the device as one element of grad_dtype (:155) and multiplied in
 * fp32 before the one rounding.  `workspace` is the one the forward call filled (it only reads
 * workspace[0], the divisor).  holds_unit_grad != 0 states that dlogits already holds the
 * gradient the forward call produced (upstream gradient 1): the call then leaves it untouched
 * when output_grad is exactly 1 and overwrites it otherwise.
 * at_cross_entropy_scale_grad multiplies dlogits in place by the upstream gradient (it returns
 * without touching memory when that value is exactly 1); the product is rounded from the
 * already rounded gradient, so prefer at_cross_entropy_bwd for 16-bit gradients.
 * ------------------------------------------------------------------------------------------ */
int64_t at_cross_entropy_workspace_bytes(int64_t batch);

int at_cross_entropy_fwd_bwd(const void* logits, const int64_t* target, const void* weight,
                             void* loss, void* dlogits, void* workspace, int64_t workspace_bytes,
                             int64_t batch, int64_t feat, int64_t logits_stride,
                             int64_t dlogits_stride, int64_t ignore_index, int logits_dtype,
                             int weight_dtype, int out_dtype, int loss_dtype, at_stream_t stream);

int at_cross_entropy_bwd(const void* logits, const int64_t* target, const void* weight,
                         const void* output_grad, const void* workspace, void* dlogits,
                         int64_t batch, int64_t feat, int64_t logits_stride,
                         int64_t dlogits_stride, int64_t ignore_index, int holds_unit_grad,
                         int logits_dtype, int weight_dtype, int grad_dtype, int out_dtype,
                         at_stream_t stream);

int at_cross_entropy_scale_grad(void* dlogits, const void* output_grad, int64_t batch,
                                int64_t feat, int64_t dlogits_stride, int dlogits_dtype,
                                int grad_dtype, at_stream_t stream);

/* at_cross_entropy_fwd_bwd without a workspace argument and without any allocation.  It has no
 * counterpart in the reference: it is for callers that cannot allocate device memory (code
 * under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The divisor and
 * the per-row losses live in a 256 KiB device array inside the library (one copy per GPU,
 * held until the process ends), so batch is limited to at_cross_entropy_static_max_batch()
 * = 65536 rows; larger batches return AT_ERR_WORKSPACE.  Every call on a GPU shares that
 * GPU's array: calls that overlap in time on one GPU (two streams) race; calls ordered on one
 * stream do not.  The first call on a device looks up the address of that array
 * (hipGetDevice + hipGetSymbolAddress, no allocation): make it outside a graph capture; later
 * calls are kernel launches only.  Arguments and results otherwise as
 * at_cross_entropy_fwd_bwd. */
int64_t at_cross_entropy_static_max_batch(void);

int at_cross_entropy_fwd_bwd_static(const void* logits, const int64_t* target,
                                    const void* weight, void* loss, void* dlogits,
                                    int64_t batch, int64_t feat, int64_t logits_stride,
                                    int64_t dlogits_stride, int64_t ignore_index,
                                    int logits_dtype, int weight_dtype, int out_dtype,
                                    int loss_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Negative log likelihood loss — replaces nll_loss_forward_kernel / nll_loss_backward_kernel,
 * attorch/nll_loss_kernels.py:39-138 and :141-235, and the torch sums and the division by the
 * summed weights at attorch/nll_loss_layer.py:88-93.
 * input is contiguous [batch, feat, spatial] log-probabilities, target [batch, spatial].
 *   forward : l[b, s] = -w[target] * input[b, target, s]  (w = 1 when weight is null)
 *             AT_REDUCTION_NONE: output[batch, spatial] = l;  _SUM: output[1] = sum(l);
 *             _MEAN: output[1] = sum(l) / sum(w[target])  (= sum(l) / (batch * spatial) unweighted)
 *   backward: input_grad[b, c, s] = -output_grad * w[c] / denominator where c == target[b, s],
 *             zero elsewhere; every element of input_grad is written (no prior zero fill).
 * output_grad is [batch, spatial] for AT_REDUCTION_NONE and one element otherwise.  The
 * reductions need at_nll_loss_workspace_bytes bytes of workspace; sum_weights (one fp32,
 * optional in the forward call) receives sum(w[target]) and is what the backward call of a
 * weighted mean divides by.  A target outside [0, feat) contributes no loss, weight or gradient
 * (the reference reads out of bounds there; it has no ignore_index, nll_loss_layer.py:162).
 * ------------------------------------------------------------------------------------------ */
#define AT_REDUCTION_NONE 0
#define AT_REDUCTION_MEAN 1
#define AT_REDUCTION_SUM 2

int64_t at_nll_loss_workspace_bytes(int64_t batch, int64_t spatial);

int at_nll_loss_fwd(const void* input, const int64_t* target, const void* weight, void* output,
                    float* sum_weights, void* workspace, int64_t workspace_bytes, int64_t batch,
                    int64_t feat, int64_t spatial, int reduction, int in_dtype, int weight_dtype,
                    int out_dtype, at_stream_t stream);

int at_nll_loss_bwd(const void* output_grad, const int64_t* target, const void* weight,
                    const float* sum_weights, void* input_grad, int64_t batch, int64_t feat,
                    int64_t spatial, int reduction, int grad_dtype, int weight_dtype,
                    int out_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Regression losses of d = input - target — replace p_loss_forward_kernel /
 * p_loss_backward_kernel, attorch/p_loss_kernels.py:17-79 and :82-143, and the torch sum at
 * attorch/p_loss_layers.py:71-73.  The ids are the reference's p_loss integers
 * (p_loss_layers.py:39-40); param is beta (smooth L1) or delta (Huber).
 *   forward : AT_REDUCTION_NONE: output[size] = loss(d); _SUM: output[1] = sum; _MEAN: sum / size
 *   backward: input_grad = output_grad * loss'(d) (/ size for the mean), target_grad = -input_grad;
 *             either gradient pointer may be null.  At d == 0 the L1-type slope is +1, as in
 *             the reference (p_loss_kernels.py:128-136).
 * input and target are contiguous, of one dtype; output_grad is [size] for AT_REDUCTION_NONE
 * and one element otherwise.  Reductions need at_p_loss_workspace_bytes bytes of workspace.
 * ------------------------------------------------------------------------------------------ */
#define AT_P_LOSS_SMOOTH_L1 0
#define AT_P_LOSS_L1 1
#define AT_P_LOSS_MSE 2
#define AT_P_LOSS_HUBER 3

int64_t at_p_loss_workspace_bytes(int64_t size);

int at_p_loss_fwd(const void* input, const void* target, void* output, void* workspace,
                  int64_t workspace_bytes, int64_t size, int p_loss, int reduction, float param,
                  int in_dtype, int out_dtype, at_stream_t stream);

int at_p_loss_bwd(const void* output_grad, const void* input, const void* target,
                  void* input_grad, void* target_grad, int64_t size, int p_loss, int reduction,
                  float param, int in_dtype, int grad_dtype, int out_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Gated linear unit with an arbitrary activation — replaces glu_forward_kernel /
 * glu_backward_kernel, attorch/glu_kernels.py:18-57 and :60-105, together with the chunk /
 * contiguous / concat copies around them (attorch/glu_layer.py:60-62, :113).
 * input is addressed as [outer][2][half]: for a contiguous tensor gated along dimension d,
 * outer = product of the sizes before d and half = (size of d / 2) * product of the sizes after d.
 *   forward : output[outer][half] = x1 * act(x2)
 *   backward: input_grad[outer][2][half] = (output_grad * act(x2), output_grad * x1 * act'(x2))
 * act is an AT_ACT_* id other than AT_ACT_NONE.
 * ------------------------------------------------------------------------------------------ */
int at_glu_fwd(const void* input, void* output, int64_t outer, int64_t half, int act, float param,
               int dtype, at_stream_t stream);

int at_glu_bwd(const void* output_grad, const void* input, void* input_grad, int64_t outer,
               int64_t half, int act, float param, int dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Linear — replaces linear_forward_kernel, attorch/linear_kernels.py:59-188 (launched from
 * attorch/linear_layer.py:90-98), act_func_backward_kernel, attorch/act_kernels.py:888-927
 * (launched from linear_layer.py:144-146 and batch_norm_layer.py:204-206), and the torch calls
 * at linear_layer.py:152-156 (two matmuls and a column sum).
 *   fwd:  output = act(input @ weight + bias), weight is [in_feat, out_feat] (row stride
 *         weight_stride); fp32 accumulation; when act != AT_ACT_NONE and pre_act is non-null
 *         (and != output) the accumulator is also stored there before the activation
 *         (save_pre_act).  bias nullable (add_bias False).  in_dtype is the dtype of input and
 *         weight; bias may have its own dtype.
 *   bwd_input:  input_grad[batch, in_feat]   = pre_act_grad[batch, out_feat] @ weight^T
 *   bwd_weight: weight_grad[in_feat, out_feat] = input^T @ pre_act_grad
 *   act_bwd:    input_grad = output_grad * act'(input) over a [rows, cols] matrix (a flat
 *               tensor is rows = 1); input_grad has input's dtype (linear_layer.py:138).  When
 *               bias_grad is non-null the column sums of input_grad (linear_layer.py:156) come
 *               out of the same pass; that needs at_act_bwd_workspace_bytes(rows, cols) bytes.
 *   colsum:     out[cols] = sum over rows (bias gradient, linear_layer.py:156); workspace of
 *               at_colsum_workspace_bytes(rows, cols) bytes; fixed summation order.
 * 16-bit operands whose pointers and strides are 16-byte aligned (and K, plus the contiguous
 * extent of a transposed operand, a multiple of 8) run on the 256x256x64 MFMA kernel; any
 * other case (fp32, odd sizes, small problems) runs on the generic fp32-MFMA kernel.
 * ------------------------------------------------------------------------------------------ */
int at_linear_fwd(const void* input, const void* weight, const void* bias, void* pre_act,
                  void* output, int64_t batch, int64_t in_feat, int64_t out_feat,
                  int64_t input_stride, int64_t weight_stride, int64_t pre_act_stride,
                  int64_t output_stride, int act, float param, int in_dtype, int bias_dtype,
                  int out_dtype, at_stream_t stream);

int at_linear_bwd_input(const void* pre_act_grad, const void* weight, void* input_grad,
                        int64_t batch, int64_t in_feat, int64_t out_feat, int64_t grad_stride,
                        int64_t weight_stride, int64_t input_grad_stride, int in_dtype,
                        int out_dtype, at_stream_t stream);

/* The two backward products take out_dtype = fp32 with 16-bit operands: the result is the product
 * rounded to the operand dtype and then widened, i.e. what the reference's 16-bit products under
 * torch.autocast (attorch/linear_layer.py:152-155) give once autograd has cast them to a float32
 * leaf — written in one pass instead of a 16-bit store and a cast kernel.  The tiled kernels do
 * this in their epilogue; at_linear_bwd_wide_output_supported tells (1 / 0) whether both products
 * of a layer with contiguous, 16-byte aligned operands of these extents run on them (otherwise
 * the generic kernels still give the same values, only slower than a 16-bit result plus a cast). */
int at_linear_bwd_wide_output_supported(int64_t batch, int64_t in_feat, int64_t out_feat, int dtype);

/* Scratch for at_linear_bwd_weight: with it, a weight gradient whose [in_feat, out_feat] tile
 * grid is small next to the GPU is computed in several slices of the batch at once (fp32 partial
 * sums, added in a fixed order); so is the weight gradient of a layer with at most 16 output
 * features.  0 when the product runs in one piece anyway.  The workspace is optional: NULL (or a
 * short one) selects the one-piece path. */
int64_t at_linear_bwd_weight_workspace_bytes(int64_t batch, int64_t in_feat, int64_t out_feat,
                                             int dtype);

int at_linear_bwd_weight(const void* input, const void* pre_act_grad, void* weight_grad,
                         void* workspace, int64_t workspace_bytes, int64_t batch,
                         int64_t in_feat, int64_t out_feat, int64_t input_stride,
                         int64_t grad_stride, int64_t weight_grad_stride, int in_dtype,
                         int out_dtype, at_stream_t stream);

/* The whole backward pass of a small fp32 layer in one launch — act_func_backward
 * (attorch/linear_layer.py:143-149 with act_kernels.py), the two products of :152-155 and the
 * bias sum of :157: input_grad = dZ W^T, weight_grad = X^T dZ and, when bias_grad is non-null,
 * bias_grad = column sums of dZ, with dZ = output_grad * act'(pre_act) formed on the fly and
 * never stored (act = AT_ACT_NONE: dZ = output_grad, pre_act may be null; a null input_grad
 * skips that product).  For layers whose
 * gradients have too few tiles to fill the GPU, where launches cost more than arithmetic:
 * at_linear_bwd_small_supported tells (1 / 0) whether a shape and dtype qualify (fp32, feature
 * extents multiples of 4, both gradients smaller than one 64x64 tile per CU); other arguments
 * return AT_ERR_UNSUPPORTED and the caller takes at_act_bwd + at_linear_bwd_input +
 * at_linear_bwd_weight.  Results are summed in a fixed order. */
int at_linear_bwd_small_supported(int64_t batch, int64_t in_feat, int64_t out_feat, int dtype);

int at_linear_bwd_small(const void* output_grad, const void* pre_act, const void* input,
                        const void* weight, void* input_grad, void* weight_grad, void* bias_grad,
                        int64_t batch, int64_t in_feat, int64_t out_feat,
                        int64_t output_grad_stride, int64_t pre_act_stride, int64_t input_stride,
                        int64_t weight_stride, int64_t input_grad_stride,
                        int64_t weight_grad_stride, int act, float param, int dtype,
                        at_stream_t stream);

int64_t at_act_bwd_workspace_bytes(int64_t rows, int64_t cols);

int at_act_bwd(const void* output_grad, const void* input, void* input_grad, void* bias_grad,
               void* workspace, int64_t workspace_bytes, int64_t rows, int64_t cols,
               int64_t output_grad_stride, int64_t input_stride, int64_t input_grad_stride, int act,
               float param, int grad_dtype, int input_dtype, int bias_grad_dtype,
               at_stream_t stream);

int64_t at_colsum_workspace_bytes(int64_t rows, int64_t cols);

int at_colsum(const void* x, void* out, void* workspace, int64_t workspace_bytes, int64_t rows,
              int64_t cols, int64_t x_stride, int x_dtype, int out_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * BatchNorm with fused affine, residual, pre-activation store and activation — replaces
 * batch_norm_forward_kernel / batch_norm_backward_kernel, attorch/batch_norm_kernels.py:44-236
 * and :246-381 (launched from attorch/batch_norm_layer.py:142-157 and :227-233) and the
 * act_func_backward_kernel launch at batch_norm_layer.py:204-206.
 * Tensors are contiguous [batch, feat, spatial] (NC, NCL or NCHW flattened; spatial = 1 for 2D
 * inputs) — no transposed view is needed.  All tensors of one call share `dtype`; weight/bias
 * share param_dtype; running statistics share running_dtype.
 *   fwd: batch statistics when is_train or !track_running_stats (biased variance normalises,
 *        running statistics are updated in place with the unbiased variance when is_train and
 *        track_running_stats), running statistics otherwise;
 *        output = act(weight*(input-mean)*inv_std + bias + pre_act_add); affine only when both
 *        weight and bias are non-null; pre_act_add nullable (add_pre_act False); pre_act
 *        non-null (and != output) stores the value before the activation (save_pre_act);
 *        mean / inv_std nullable (save_stats False).
 *   bwd: g = output_grad * act'(pre_act) is written to pre_act_grad (required when
 *        act != AT_ACT_NONE; it is also the residual gradient, batch_norm_layer.py:244);
 *        input_grad = inv_std*(weight*g - (sum(x_hat*g)*weight/n * x_hat + sum(g)*weight/n));
 *        weight_grad = sum(x_hat*g), bias_grad = sum(g) (fp32 [feat], nullable).
 * workspace: at_batch_norm_workspace_bytes(feat) bytes for either direction.
 * ------------------------------------------------------------------------------------------ */
int64_t at_batch_norm_workspace_bytes(int64_t feat);

int at_batch_norm_fwd(const void* input, const void* weight, const void* bias, float* mean,
                      float* inv_std, const void* pre_act_add, void* pre_act, void* output,
                      void* running_mean, void* running_var, void* workspace,
                      int64_t workspace_bytes, int64_t batch, int64_t feat, int64_t spatial,
                      float momentum, float eps, int act, float param, int track_running_stats,
                      int is_train, int dtype, int param_dtype, int running_dtype,
                      at_stream_t stream);

int at_batch_norm_bwd(const void* output_grad, const void* pre_act, const void* input,
                      const float* mean, const float* inv_std, const void* weight,
                      void* input_grad, void* pre_act_grad, float* weight_grad, float* bias_grad,
                      void* workspace, int64_t workspace_bytes, int64_t batch, int64_t feat,
                      int64_t spatial, int act, float param, int dtype, int param_dtype,
                      at_stream_t stream);

/* The same two calls for tensors that are channels-last in memory ([batch, spatial..., feat], a
 * [batch * spatial, feat] matrix with statistics per column): same arguments, meanings and
 * workspace.  The reference reads its input through strides (batch_norm_layer.py:130-157), so
 * such tensors are within its interface.  Covered when feat is a multiple of the 16-byte vector
 * (8 for 16-bit, 4 for fp32 tensors) — at_batch_norm_nhwc_supported tells; rows wider than 256
 * vectors are processed in column slabs.  Otherwise the calls return AT_ERR_UNSUPPORTED and the
 * caller converts to channels-first.  With spatial = 1 these are the calls for [batch, feat]
 * inputs. */
int at_batch_norm_nhwc_supported(int64_t feat, int dtype);

int at_batch_norm_fwd_nhwc(const void* input, const void* weight, const void* bias, float* mean,
                           float* inv_std, const void* pre_act_add, void* pre_act, void* output,
                           void* running_mean, void* running_var, void* workspace,
                           int64_t workspace_bytes, int64_t batch, int64_t feat, int64_t spatial,
                           float momentum, float eps, int act, float param,
                           int track_running_stats, int is_train, int dtype, int param_dtype,
                           int running_dtype, at_stream_t stream);

int at_batch_norm_bwd_nhwc(const void* output_grad, const void* pre_act, const void* input,
                           const float* mean, const float* inv_std, const void* weight,
                           void* input_grad, void* pre_act_grad, float* weight_grad,
                           float* bias_grad, void* workspace, int64_t workspace_bytes,
                           int64_t batch, int64_t feat, int64_t spatial, int act, float param,
                           int dtype, int param_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Conv2d (NCHW, zero padding, stride, groups, no dilation) — replaces conv2d_forward_kernel,
 * attorch/conv_kernels.py:68-207 (launched from attorch/conv_layer.py:102-112), the bias add
 * at conv_layer.py:114-116, and the torch calls of the backward pass at conv_layer.py:153-162
 * (torch.nn.grad.conv2d_input, conv2d_weight and the bias sum).
 * Tensors are contiguous: input [batch, in_feat, in_height, in_width], weight
 * [out_feat, in_feat / groups, kernel_height, kernel_width], output
 * [batch, out_feat, out_height, out_width] with out = (in + 2*padding - kernel) / stride + 1
 * (conv_layer.py:18-36), which the call checks.  bias nullable.
 *   Workspace: 16-bit tensors run on the matrix cores from channels-last copies kept in
 *   caller-provided workspace when the contraction channels per group (input channels for
 *   forward, output channels for bwd_input) are a multiple of 64 or at least 16 (the copy is
 *   then padded with zero channels to the next multiple), for bwd_input with
 *   stride_height * stride_width <= 4 (the gradient is spread out by the strides first) and for
 *   bwd_weight with channel counts per group in multiples of 8; each
 *   at_conv2d_*_workspace_bytes(...) returns the bytes that path wants for the given shape
 *   (0: no such path).  forward and bwd_input fall back to the generic kernel when the
 *   workspace is null or smaller; bwd_weight always needs its workspace (split-K partials).
 *   Channels-last copies can be shared between calls: at_conv2d_fwd leaves the copy of the
 *   input ([batch, height, width, feat]) at the start of its workspace when
 *   at_conv2d_fwd_leaves_nhwc(...) returns 1 (no channel padding was needed), at_nchw_to_nhwc makes
 *   one of any 16-bit NCHW tensor, and the backward entry points take such copies through
 *   their nullable *_nhwc arguments instead of making their own (matrix-core path only).
 *   at_channel_sum: out[feat] = sum over batch and space of a [batch, feat, spatial] tensor.
 * ------------------------------------------------------------------------------------------ */
int64_t at_conv2d_fwd_workspace_bytes(int64_t batch, int64_t in_feat, int64_t in_height,
                                      int64_t in_width, int64_t out_feat, int64_t out_height,
                                      int64_t out_width, int64_t kernel_height,
                                      int64_t kernel_width, int64_t stride_height,
                                      int64_t stride_width, int64_t padding_height,
                                      int64_t padding_width, int64_t groups, int in_dtype,
                                      int out_dtype);

int at_conv2d_fwd_leaves_nhwc(int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width,
                              int64_t out_feat, int64_t out_height, int64_t out_width,
                              int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                              int64_t stride_width, int64_t padding_height,
                              int64_t padding_width, int64_t groups, int in_dtype, int out_dtype);

int at_conv2d_fwd(const void* input, const void* weight, const void* bias, void* output,
                  void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat,
                  int64_t in_height, int64_t in_width, int64_t out_feat, int64_t out_height,
                  int64_t out_width, int64_t kernel_height, int64_t kernel_width,
                  int64_t stride_height, int64_t stride_width, int64_t padding_height,
                  int64_t padding_width, int64_t groups, int in_dtype, int bias_dtype,
                  int out_dtype, at_stream_t stream);

int64_t at_conv2d_bwd_input_workspace_bytes(int64_t batch, int64_t in_feat, int64_t in_height,
                                            int64_t in_width, int64_t out_feat,
                                            int64_t out_height, int64_t out_width,
                                            int64_t kernel_height, int64_t kernel_width,
                                            int64_t stride_height, int64_t stride_width,
                                            int64_t padding_height, int64_t padding_width,
                                            int64_t groups, int dtype);

int at_conv2d_bwd_input(const void* output_grad, const void* output_grad_nhwc,
                        const void* weight, void* input_grad, void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat,
                        int64_t in_height, int64_t in_width, int64_t out_feat,
                        int64_t out_height, int64_t out_width, int64_t kernel_height,
                        int64_t kernel_width, int64_t stride_height, int64_t stride_width,
                        int64_t padding_height, int64_t padding_width, int64_t groups, int dtype,
                        at_stream_t stream);

int64_t at_conv2d_bwd_weight_workspace_bytes(int64_t batch, int64_t in_feat, int64_t in_height,
                                             int64_t in_width, int64_t out_feat,
                                             int64_t out_height, int64_t out_width,
                                             int64_t kernel_height, int64_t kernel_width,
                                             int64_t stride_height, int64_t stride_width,
                                             int64_t padding_height, int64_t padding_width,
                                             int64_t groups, int dtype);

int at_conv2d_bwd_weight(const void* output_grad, const void* output_grad_nhwc,
                         const void* input, const void* input_nhwc, void* weight_grad,
                         void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat,
                         int64_t in_height, int64_t in_width, int64_t out_feat, int64_t out_height,
                         int64_t out_width, int64_t kernel_height, int64_t kernel_width,
                         int64_t stride_height, int64_t stride_width, int64_t padding_height,
                         int64_t padding_width, int64_t groups, int dtype, at_stream_t stream);

/* The same three products for tensors that are channels-last in memory ([batch, height, width,
 * feat], what torch.channels_last gives a [batch, feat, height, width] tensor) — the layout the
 * matrix-core kernels work in, so nothing is copied: input and output of every call are
 * channels-last, the weight ([out_feat, in_feat / groups, kh, kw]) and its gradient are not.
 * The reference's kernels take any strides (attorch/conv_layer.py:102-116 passes them on), so
 * such tensors are within its interface.  16-bit tensors only; forward needs in_feat / groups,
 * bwd_input out_feat / groups in multiples of 64 (and stride 1), bwd_weight both in multiples
 * of 8.  at_conv2d_nhwc_workspace_bytes(pass, ...) (pass 0 forward, 1 bwd_input, 2 bwd_weight)
 * returns the workspace the call needs, 0 when this path does not cover the shape (the calls
 * then return AT_ERR_UNSUPPORTED and the caller converts to channels-first). */
int64_t at_conv2d_nhwc_workspace_bytes(int pass, int64_t batch, int64_t in_feat, int64_t in_height,
                                       int64_t in_width, int64_t out_feat, int64_t out_height, int64_t out_width,
                                       int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                                       int64_t stride_width, int64_t padding_height, int64_t padding_width,
                                       int64_t groups, int dtype);

int at_conv2d_fwd_nhwc(const void* input, const void* weight, const void* bias, void* output,
                       void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height,
                       int64_t in_width, int64_t out_feat, int64_t out_height, int64_t out_width,
                       int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                       int64_t stride_width, int64_t padding_height, int64_t padding_width,
                       int64_t groups, int dtype, int bias_dtype, at_stream_t stream);

int at_conv2d_bwd_input_nhwc(const void* output_grad, const void* weight, void* input_grad,
                             void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height,
                             int64_t in_width, int64_t out_feat, int64_t out_height, int64_t out_width,
                             int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                             int64_t stride_width, int64_t padding_height, int64_t padding_width,
                             int64_t groups, int dtype, at_stream_t stream);

int at_conv2d_bwd_weight_nhwc(const void* output_grad, const void* input, void* weight_grad,
                              void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height,
                              int64_t in_width, int64_t out_feat, int64_t out_height, int64_t out_width,
                              int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                              int64_t stride_width, int64_t padding_height, int64_t padding_width,
                              int64_t groups, int dtype, at_stream_t stream);

int at_nchw_to_nhwc(const void* src, void* dst, int64_t batch, int64_t feat, int64_t spatial,
                    int dtype, at_stream_t stream);

int at_channel_sum(const void* x, void* out, int64_t batch, int64_t feat, int64_t spatial,
                   int x_dtype, int out_dtype, at_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Standalone activation layers with fused dropout, and Dropout — replace
 * act_func_forward_kernel / act_func_backward_kernel, attorch/act_kernels.py:845-927 (launched
 * from attorch/act_layers.py:78-80,108-111), and dropout_forward_kernel /
 * dropout_backward_kernel, attorch/dropout_kernels.py:54-112 (launched from
 * attorch/dropout_layer.py:53-58,88-93).  Flat tensors of `size` elements, one dtype.
 *   fwd: output     = dropout(act(input))                   (act_kernels.py:729-730)
 *   bwd: input_grad = dropout'(output_grad) * act'(input)   (act_kernels.py:834-837)
 * act = AT_ACT_NONE gives plain dropout (input may then be null in bwd).  drop_p = 0 disables
 * dropout (pass 0 outside training).  A dropped element is exactly zero, kept ones are scaled
 * by 1 / (1 - drop_p) (dropout_kernels.py:26-27).  The mask is a pure function of (seed,
 * element index) — Philox4x32-7 (16 bits per element), not Triton's generator, so masks differ from the
 * reference's for equal seeds; forward and backward of one call pair agree.
 * ------------------------------------------------------------------------------------------ */
int at_act_dropout_fwd(const void* input, void* output, int64_t size, int act, float param,
                       float drop_p, uint32_t seed, int dtype, at_stream_t stream);

int at_act_dropout_bwd(const void* output_grad, const void* input, void* input_grad,
                       int64_t size, int act, float param, float drop_p, uint32_t seed,
                       int dtype, at_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* ATTORCH_HIP_H */
