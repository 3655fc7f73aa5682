// Dense convolution through the vendor library, the comparator of the CP4
// operators: the reference's namespace NV (Cuda_kernels/NVConv2d.cuh:7-17),
// which calls cuDNN there and MIOpen here.  The namespace keeps the
// reference's name so that its tests and bench drivers read unchanged.
// Needs libcp4dense.so (and 2*pad = Y-1 = X-1: the output is H x W).
#ifndef CP4_NVCONV2D_H
#define CP4_NVCONV2D_H

#include <utility>

#include "cp4/tensor.h"

namespace NV {

// In[N,C,H,W] (*) K[T,C,Y,X] -> [N,T,H,W]            (NVConv2d.cu:154-171)
Tensor Conv2dForward(Tensor const& In, Tensor const& K, unsigned pad);
// Upstream[N,T,H,W], K[T,C,Y,X] -> dIn[N,C,H,W]      (NVConv2d.cu:296-314)
Tensor Conv2dBackwardData(Tensor const& Upstream, Tensor const& K, unsigned pad);
// dLdO[N,T,H,W], Input[N,C,H,W] -> dK with Filter's shape [T,C,Y,X]; only
// the shape of Filter is used                         (NVConv2d.cu:439-461)
Tensor Conv2dBackwardFilter(Tensor const& dLdO, Tensor const& Input, Tensor const& Filter,
                            unsigned pad);
// (mean microseconds of PROFCOUNT forward calls on uninitialised device
// buffers, bytes of In + Filter + Out)                (NVConv2d.cu:471-489)
std::pair<float, unsigned> run_convolution(tensor_shape, unsigned PROFCOUNT = 1);

}  // namespace NV

#endif  // CP4_NVCONV2D_H
