// Implicit-GEMM convolution on the 16-bit matrix cores (bf16 / fp16, fp32 accumulate).
//
// The kernels work on channels-last copies of the activations: with the channel index
// contiguous, one 16-byte access holds 8 consecutive values of the contraction index, which is
// what a matrix-core operand wants, and a filter tap outside the image is a whole row of zeros.
// The tensors of the C ABI stay NCHW; the copies live in caller-provided workspace.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace at_hip {

struct ConvProblem {
  int64_t N, C, H, W, O, KH, KW, sh, sw, ph, pw, groups, OH, OW;
  int dtype;   // AT_DTYPE_F16 or AT_DTYPE_BF16 for every tensor
};

// True when the 16-bit implicit-GEMM kernels cover the problem: 32-bit addressable tensors;
// contraction channels per group (input channels for the forward product, output channels for the
// input gradient) in multiples of 64, or at least 16 (padded with zeros to the next multiple in
// the channels-last copy); strides of the input gradient with sh * sw <= 4 (the gradient is
// spread out by the strides); channel counts per group in multiples of 8 for the weight gradient.
bool conv_igemm_supports_fwd(const ConvProblem& p);
bool conv_igemm_supports_dx(const ConvProblem& p);
bool conv_igemm_supports_dw(const ConvProblem& p);
// True when the forward workspace afterwards begins with a plain [N][H][W][C] copy of the input
// (no channel padding), which conv_igemm_dw accepts as x_nhwc.
bool conv_igemm_fwd_leaves_nhwc(const ConvProblem& p);

int64_t conv_igemm_fwd_workspace(const ConvProblem& p);
int64_t conv_igemm_dx_workspace(const ConvProblem& p);
int64_t conv_igemm_dw_workspace(const ConvProblem& p);

// Y = conv(X, W) + bias, all NCHW.
int conv_igemm_fwd(const ConvProblem& p, const void* x, const void* w, const void* bias, int bias_dt,
                   void* y, void* workspace, hipStream_t stream);
// dX = conv_transpose(dY, W), all NCHW.  dy_nhwc: optional channels-last copy of dY the caller
// already holds (saves the copy made here when the product can read it as it is: stride 1 and
// output channels per group a multiple of 64).
int conv_igemm_dx(const ConvProblem& p, const void* dy, const void* dy_nhwc, const void* w, void* dx,
                  void* workspace, hipStream_t stream);
// dW[O][C/groups][KH][KW] = correlation of dY with X, all NCHW.  dy_nhwc / x_nhwc: optional
// channels-last copies the caller already holds.
int conv_igemm_dw(const ConvProblem& p, const void* dy, const void* dy_nhwc, const void* x, const void* x_nhwc,
                  void* dw, void* workspace, hipStream_t stream);
// The same products on channels-last tensors ([N][H][W][C]) in and out: no layout copies, the
// workspace holds the reordered weights only.  Input channels per group (forward) / output
// channels per group (input gradient, stride 1 only) in multiples of 64.  The weight gradient of
// channels-last tensors is conv_igemm_dw with both *_nhwc arguments given.
bool conv_igemm_supports_fwd_last(const ConvProblem& p);
bool conv_igemm_supports_dx_last(const ConvProblem& p);
int64_t conv_igemm_fwd_last_workspace(const ConvProblem& p);
int64_t conv_igemm_dx_last_workspace(const ConvProblem& p);
int conv_igemm_fwd_last(const ConvProblem& p, const void* x_last, const void* w, const void* bias, int bias_dt,
                        void* y_last, void* workspace, hipStream_t stream);
int conv_igemm_dx_last(const ConvProblem& p, const void* dy_last, const void* w, void* dx_last, void* workspace,
                       hipStream_t stream);
// [N][C][HW] -> [N][HW][C] for a 16-bit dtype.
int conv_nchw_to_nhwc(const void* src, void* dst, int64_t N, int64_t C, int64_t HW, int dtype,
                      hipStream_t stream);

}  // namespace at_hip
