// Test / bench helpers of the reference (Cuda_kernels/Utils.cuh:9-13).
#ifndef CP4_UTILS_H
#define CP4_UTILS_H

#include <initializer_list>

#include "cp4/tensor.h"

// Uniform (0,1] values from a fixed seed (1234), generated on the GPU: like the
// reference (Utils.cu:22-33) every call yields the same stream prefix.
Tensor random_fill(std::initializer_list<unsigned> lst);

// Dense filter K[T,C,Y,X] = sum_r FT[t,r] FC[c,r] FY[y,r] FX[x,r] (Utils.cu:36-98).
Tensor cp4recom(Tensor const& FT, Tensor const& FC, Tensor const& FY, Tensor const& FX);

// True if no element's symmetric relative error exceeds the tolerance
// (absolute error where either value is 0) (Utils.cu:143-180).
bool AllClose(Tensor const& A, Tensor const& B, float tolerance = 1e-3);

#endif  // CP4_UTILS_H
