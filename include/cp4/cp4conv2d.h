// C++ operator API of the fused CP4 Conv2d: the reference's namespace CP
// (Cuda_kernels/cp4Conv2d.cuh:6-33) and its raw-pointer launchers
// (cp4Conv2dForward.cuh:7-14, cp4Conv2dBackwardData.cuh:7-14,
// cp4Conv2dBackwardFilter.cuh:7-47), implemented on top of the C ABI in
// cp4/capi.h.  Factor order everywhere: FT (out-channel), FC, FY, FX.
#ifndef CP4_CP4CONV2D_H
#define CP4_CP4CONV2D_H

#include <utility>

#include "cp4/tensor.h"

namespace CP {

// Cuda_kernels/cp4Conv2d.cu:14-43.  N,C,H,W from Input, T and Rank from FT, Y
// from FY, X from FX; returns Out{N,T,H,W}.
Tensor Conv2dForward(Tensor const& Input, Tensor const& FT, Tensor const& FC,
                     Tensor const& FY, Tensor const& FX, unsigned pad = 1);

// Restores the reference's disabled wrapper (cp4Conv2d.cu:48-77): N,T,H,W from
// Upstream, C from FC; returns dInput{N,C,H,W}.
Tensor Conv2dBackwardData(Tensor const& Upstream, Tensor const& FT, Tensor const& FC,
                          Tensor const& FY, Tensor const& FX, unsigned pad = 1);

// Restores cp4Conv2d.cu:83-153, returning the four factor gradients themselves
// (the disabled reference code recomposed them into a dense tensor, which is
// not the dense filter gradient).
struct FilterGradients {
  Tensor dFT, dFC, dFY, dFX;
};
FilterGradients Conv2dBackwardFilter(Tensor const& dLdO, Tensor const& In, Tensor const& FT,
                                     Tensor const& FC, Tensor const& FY, Tensor const& FX,
                                     unsigned pad = 1);

// Cuda_kernels/cp4Conv2d.cu:158-190: device buffers of the given shape
// (contents unspecified), one untimed then PROFCOUNT timed forward launches; returns
// {mean microseconds, algorithmic bytes 4*(N*T*H*W + N*C*H*W + Rank*(T+C+X+Y))}.
std::pair<float, unsigned> run_convolution(tensor_shape, unsigned PROFCOUNT = 1);

}  // namespace CP

// Raw-pointer launchers with the reference's signatures.  Pointers may be
// device pointers or host pointers (the reference is handed both managed and
// plain device memory); host data is staged through HBM.  All return the mean
// microseconds per launch over PROFCOUNT launches, synchronise before
// returning, and on a runtime error print it and exit like the reference's
// ErrChk (Cuda_kernels/cp4Conv2dForward.cu:10-19).
float cp4_conv2d_forward_gpu(tensor_shape, const float* In, const float* FT, const float* FC,
                             const float* FY, const float* FX, float* Out,
                             unsigned PROFCOUNT = 1);
float cp4_conv2d_backward_data_gpu(tensor_shape, const float* Upstream, const float* FT,
                                   const float* FC, const float* FY, const float* FX,
                                   float* Out, unsigned PROFCOUNT = 1);
// Dense filter gradient FF[T,C,Y,X] += ... (cp4Conv2dBackwardFilter.cu:23-59).
float cp4_conv2d_backward_filter_full_gpu(tensor_shape, float* FF, const float* In,
                                          const float* dLdO, unsigned PROFCOUNT = 1);
// Factor gradients; each ADDS into its output like the reference's loops
// (cp4Conv2dBackwardFilter.cu:99,150,200,249) and takes the other three
// factors in T, C, Y, X order.
float cp4_conv2d_backward_filter_t_gpu(tensor_shape, float* dFT, const float* In,
                                       const float* dLdO, const float* FC, const float* FY,
                                       const float* FX, unsigned PROFCOUNT = 1);
float cp4_conv2d_backward_filter_c_gpu(tensor_shape, float* dFC, const float* In,
                                       const float* dLdO, const float* FT, const float* FY,
                                       const float* FX, unsigned PROFCOUNT = 1);
float cp4_conv2d_backward_filter_y_gpu(tensor_shape, float* dFY, const float* In,
                                       const float* dLdO, const float* FT, const float* FC,
                                       const float* FX, unsigned PROFCOUNT = 1);
float cp4_conv2d_backward_filter_x_gpu(tensor_shape, float* dFX, const float* In,
                                       const float* dLdO, const float* FT, const float* FC,
                                       const float* FY, unsigned PROFCOUNT = 1);

#endif  // CP4_CP4CONV2D_H
