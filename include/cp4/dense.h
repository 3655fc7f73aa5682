/*
 * C ABI of the dense-convolution comparator: the vendor library's (MIOpen's)
 * fp32 NCHW cross-correlation on the same device buffers the CP4 path uses.
 * It stands where the reference calls cuDNN (Cuda_kernels/NVConv2d.cu): as the
 * independent check of a CP4 result against the dense convolution with the
 * recomposed filter, and as the "dense" column of the timing tables.
 *
 * Stride 1, no dilation, zero padding `pad`, and an H x W output: 2*pad must
 * equal Y-1 and X-1 (the only case in which the reference's wrappers, which
 * allocate [N,T,H,W], are consistent with the library's output size).
 * Lives in its own shared library (libcp4dense.so) so that libcp4conv.so does
 * not depend on MIOpen.  All pointers are DEVICE pointers to contiguous fp32.
 */
#ifndef CP4_DENSE_H
#define CP4_DENSE_H

#include "cp4/capi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Detail of the calling thread's last failure in this library ("" if none). */
const char* cp4_dense_last_error_message(void);

/* Replaces conv2d_forward_gpu (Cuda_kernels/NVConv2d.cu:18-148) without its
 * timing loop: x[N,C,H,W] (*) K[T,C,Y,X] -> y[N,T,H,W].  shape->Rank is
 * ignored. */
cp4_status cp4_dense_conv2d_forward(const cp4_shape* shape, const float* x,
                                    const float* K, float* y, cp4_stream stream);

/* Replaces conv2d_backward_data_gpu (NVConv2d.cu:178-290):
 * dy[N,T,H,W], K[T,C,Y,X] -> dx[N,C,H,W]. */
cp4_status cp4_dense_conv2d_backward_data(const cp4_shape* shape, const float* dy,
                                          const float* K, float* dx,
                                          cp4_stream stream);

/* Replaces conv2d_backward_filter_gpu (NVConv2d.cu:322-433):
 * x[N,C,H,W], dy[N,T,H,W] -> dK[T,C,Y,X] (overwritten). */
cp4_status cp4_dense_conv2d_backward_filter(const cp4_shape* shape, const float* x,
                                            const float* dy, float* dK,
                                            cp4_stream stream);

/* Replaces the PROFCOUNT loop of conv2d_forward_gpu (NVConv2d.cu:118-140):
 * `warmup` untimed forward calls, then `profcount` calls between one pair of
 * HIP events on `stream`; *mean_us = elapsed / profcount. */
cp4_status cp4_dense_time_forward(const cp4_shape* shape, const float* x,
                                  const float* K, float* y, unsigned warmup,
                                  unsigned profcount, float* mean_us,
                                  cp4_stream stream);

/* Drops the cached library handle, problem descriptors and workspaces. */
void cp4_dense_release(void);

#ifdef __cplusplus
}
#endif
#endif /* CP4_DENSE_H */
