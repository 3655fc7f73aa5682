// Internal interface between the C ABI (cp4_capi.hip) and the kernel
// translation units.  Every launcher validates nothing: the C ABI has already
// checked pointers and shape, and each launcher's own `*_supported` predicate
// says whether its kernel's assumptions hold for a shape.
#ifndef CP4_INTERNAL_H
#define CP4_INTERNAL_H

#include <hip/hip_runtime.h>

#include "cp4/capi.h"

namespace cp4 {

// Operands of one forward-shaped launch.  Backward-data is the same kernel
// with x<-dy, Cin<-T, Cout<-C, Fin<-FK, Fout<-FC and flipped taps
// (Cuda_kernels/cp4Conv2dBackwardData.cu:79-87,98-108).
struct FwdArgs {
  const float* x;     // [N, Cin, H, W]
  const float* Fin;   // [Cin, R]
  const float* Fout;  // [Cout, R]
  const float* FH;    // [Y, R]
  const float* FW;    // [X, R]
  float* y;           // [N, Cout, H, W]
  int N, Cin, Cout, H, W, pad, Y, X, R;
  int flip;           // 1: tap index t reads factor row (taps-1-t)
  // Output epilogue y = act(conv + bias[k]); only kernels that say so apply it
  // (the caller runs bias_act_launch after the others).
  const float* bias;  // [Cout] or null
  int act;            // 0: none, 1: max(., 0)
  // Rank and channel passes (rank-pass build of the producer / consumer kernel only): the
  // factor pointers may address a column block of wider matrices - ldf is their row
  // stride in floats (0: R) -, x a slice of Cin channels out of wider images - ldx is
  // the distance between images in elements (0: Cin * H * W) - and accumulate != 0 adds
  // to y instead of overwriting it.
  int ldf;
  size_t ldx;
  int accumulate;
  // 2-D-tap build of the producer / consumer kernel only: depthwise filter
  // [Y, X, R] used instead of the outer product FH x FW (FH, FW unused then).
  const float* taps2d;
  // Producer / consumer kernel: a tuned strip height (tile height in the tiled
  // build), log2 of the tile width (tiled build) and role split (1: off) that
  // replace the planner's choice; 0 leaves it to the planner.
  int tune_th, tune_lgwt, tune_split2;
  // Producer / consumer kernel: polls before a wait between waves gives up
  // (0: the default) and the device's fault record, four ints (may be null).
  int spin_limit;
  int* fault;
  // Layer geometry beyond the reference's (stride 1, `pad` zeros before the image,
  // an H x W output): output pixel (ho, wo) reads x at (sh*ho + i - pt, sw*wo + j - pl),
  // the output plane is Ho x Wo.  sh == 0: the reference's geometry, the other
  // fields unused.  Only kernels that say so take sh != 0.
  int sh, sw, pt, pl, Ho, Wo;
  // Strided build of the producer / consumer kernel only: the adjoint of a strided
  // layer (its backward-data pass).  The H x W input plane is then the strided
  // layer's output gradient and the Ho x Wo output plane its input gradient:
  // output pixel (h, w) sums tap (i, j) times input pixel ((h + pt - i) / sh,
  // (w + pl - j) / sw) wherever both divisions are exact and land inside the plane
  // (flip unused).
  int transposed;
  // Strided build only, set by its own entry points: a filter of ty x tx taps that runs as
  // the square window of Y = X taps around it (even and rectangular filters); 0: Y, X.
  int ty, tx;
  // Recomposed-filter kernel only: the dense filter [Cout, Cin, Y, X] itself, taps in
  // the order the pass reads them; the four factors are unused then.
  const float* dense;
};

// The geometry of a launch with the defaults filled in.
struct Geometry {
  int sh, sw, pt, pl, Ho, Wo;
};
inline Geometry geometry_of(const FwdArgs& a) {
  if (a.sh == 0) return Geometry{1, 1, a.pad, a.pad, a.H, a.W};
  return Geometry{a.sh, a.sw, a.pt, a.pl, a.Ho, a.Wo};
}

// Compute units of the current device (256 when no device can be asked).
int num_compute_units();


// The matrix-core kernels index pixels, strips and work items with 32-bit
// integers: planes up to 2^24 pixels and batch x plane products that keep every
// such count below 2^31.  Larger problems run on the general kernels, whose
// indices are 64-bit throughout.
inline bool fits_int_indexing(int N, int H, int W) {
  const size_t HW = (size_t)H * W;
  return HW <= (1u << 24) && (size_t)N * HW < (1ull << 35) && (size_t)N * H < (1ull << 30);
}

bool fwd_general_supported(const FwdArgs&);
hipError_t fwd_general_launch(const FwdArgs&, hipStream_t);
// Recomposed-filter direct convolution for very few channels on both sides.
bool fwd_dense_small_supported(const FwdArgs&);
hipError_t fwd_dense_small_launch(const FwdArgs&, hipStream_t);
// Its plan for a shape: 16 x 64 tiles in all and LDS bytes per workgroup (false: no plan).
bool fwd_dense_small_plan_info(const FwdArgs&, long* tiles, size_t* lds_bytes);
bool fwd_mfma_supported(const FwdArgs&);
hipError_t fwd_mfma_launch(const FwdArgs&, hipStream_t);
bool fwd_split_supported(const FwdArgs&);
hipError_t fwd_split_launch(const FwdArgs&, hipStream_t);
// Few short phases in small workgroups, for small problems (ranks up to 32).
bool fwd_light_supported(const FwdArgs&);
hipError_t fwd_light_launch(const FwdArgs&, hipStream_t);
// Persistent small workgroups over 2-D tiles, taps and output contraction in registers:
// few channels (up to 64 in), up to 16 ranks, planes of any width.
bool fwd_few_supported(const FwdArgs&);
hipError_t fwd_few_launch(const FwdArgs&, hipStream_t);
bool fwd_few_plan(const FwdArgs&, int* rows, int* cols, int* workgroups);
bool fwd_pipe_supported(const FwdArgs&);
hipError_t fwd_pipe_launch(const FwdArgs&, hipStream_t);
// Rows per strip and workgroups of the whole-row strip plan (false: no plan).
bool fwd_pipe_strip_plan(const FwdArgs&, int* rows, int* workgroups);
// Producer / consumer kernel with a 64-rank plane: ranks 33 - 64 in one pass (1x1 and 3x3
// filters, up to 256 input channels); honours FwdArgs::ldf, ldx and accumulate.
bool fwd_pipe64_supported(const FwdArgs&);
hipError_t fwd_pipe64_launch(const FwdArgs&, hipStream_t);
bool fwd_pipe64_plan(const FwdArgs&, int* rows, int* workgroups);
// The same kernel compiled with the bias / activation epilogue in its stores.
bool fwd_pipe_epi_supported(const FwdArgs&);
hipError_t fwd_pipe_epi_launch(const FwdArgs&, hipStream_t);
// The same kernel with bfloat16 x and y in memory (FwdArgs::x / y point at
// 16-bit elements; factors and bias stay fp32), epilogue included.
bool fwd_pipe_io16_supported(const FwdArgs&);
hipError_t fwd_pipe_io16_launch(const FwdArgs&, hipStream_t);
// The same with IEEE half-precision x and y in memory.
bool fwd_pipe_iof16_supported(const FwdArgs&);
hipError_t fwd_pipe_iof16_launch(const FwdArgs&, hipStream_t);
// The same kernel honouring FwdArgs::ldf and FwdArgs::accumulate (rank passes).
bool fwd_pipe_rankpass_supported(const FwdArgs&);
hipError_t fwd_pipe_rankpass_launch(const FwdArgs&, hipStream_t);
// The same kernel on tiles of TH rows x Wt columns (wide planes).
bool fwd_pipe_tiled_supported(const FwdArgs&);
hipError_t fwd_pipe_tiled_launch(const FwdArgs&, hipStream_t);
bool fwd_pipe_tiled_epi_supported(const FwdArgs&);          // ... with the bias / activation epilogue
hipError_t fwd_pipe_tiled_epi_launch(const FwdArgs&, hipStream_t);
// The same kernel for a stride or an output plane of its own (FwdArgs::sh ...
// all filled in by the caller).
bool fwd_pipe_strided_supported(const FwdArgs&);
hipError_t fwd_pipe_strided_launch(const FwdArgs&, hipStream_t);
// The same kernel with a depthwise Y x X filter (FwdArgs::taps2d) in its tap step.
bool fwd_pipe_taps2d_supported(const FwdArgs&);
hipError_t fwd_pipe_taps2d_launch(const FwdArgs&, hipStream_t);
// In-place y[n,k,:] = act(y[n,k,:] + bias[k]) for variants without the epilogue.
hipError_t bias_act_launch(float* y, const float* bias, int act, size_t N, size_t K, size_t HW,
                           hipStream_t);

// Backward-filter (factor gradients).
struct BwdFilterArgs {
  const float *x, *dy, *FK, *FC, *FH, *FW;
  float *dFK, *dFC, *dFH, *dFW;
  void* workspace;
  int N, C, T, H, W, pad, Y, X, R;
  // Matrix-core variant only, 3-factor CP op: a depthwise filter [Y, X, R] in place
  // of FH x FW and its gradient (FH, FW, dFH, dFW unused then).
  const float* taps2d;
  float* dtaps2d;
};
// general (VALU, any shape) and matrix-core variants
size_t bwd_filter_workspace_bytes(const cp4_shape&);
hipError_t bwd_filter_launch(const BwdFilterArgs&, hipStream_t);
bool bwd_filter_mfma_supported(const cp4_shape&);
size_t bwd_filter_mfma_workspace_bytes(const cp4_shape&);
bool bwd_filter_mfma_taps2d_supported(const cp4_shape&);   // with BwdFilterArgs::taps2d
hipError_t bwd_filter_mfma_launch(const BwdFilterArgs&, hipStream_t);
// Matrix-core variant with the tap step inside the gradient GEMMs (three launches;
// square odd filters up to 5 with 2 * pad == Y - 1, channel counts multiples of 16,
// H * W a multiple of 4, x / dy / workspace 16-byte aligned).
bool bwd_filter_fused_supported(const cp4_shape&);
// Where the three-launch variant is the faster one (small and medium problems, whose
// time is launches and first-load latencies rather than bandwidth).
bool bwd_filter_fused_preferred(const cp4_shape&);
size_t bwd_filter_fused_workspace_bytes(const cp4_shape&);
hipError_t bwd_filter_fused_launch(const BwdFilterArgs&, hipStream_t);
// Few channels on both sides (square filters of 1, 3, 5 taps; T * C up to 256 with plain
// multiply-adds, or up to 64 output channels and 16384 entries of the dense gradient on the
// matrix cores): the dense filter gradient over tiles of pixels, then the chain rule onto the
// factors (three launches, no [N, R, H, W] intermediates).
bool bwd_filter_dense_tiles_supported(const cp4_shape&);
bool bwd_filter_dense_tiles_preferred(const cp4_shape&);
size_t bwd_filter_dense_tiles_workspace_bytes(const cp4_shape&);
hipError_t bwd_filter_dense_tiles_launch(const BwdFilterArgs&, hipStream_t);
// 0: the plain multiply-add tile kernel, 1: the matrix-core one, wherever both can run the
// shape; anything else: the route's own choice.
void bwd_filter_dense_tiles_force_kernel(int which);
// A layer with a stride and zeros of its own before the image (BwdFilterArgs::H, W: the
// input plane; pad unused; dy on the geometry's Ho x Wo grid).
bool bwd_filter_mfma_strided_supported(const cp4_shape&, const Geometry&);
size_t bwd_filter_mfma_strided_workspace_bytes(const cp4_shape&, const Geometry&);
hipError_t bwd_filter_mfma_strided_launch(const BwdFilterArgs&, const Geometry&, hipStream_t);
// The same with bfloat16 x and dy in memory (BwdFilterArgs::x / dy point at 16-bit
// elements); split-bf16 kernels only: C and T multiples of 16.
bool bwd_filter_mfma_io16_supported(const cp4_shape&);
size_t bwd_filter_mfma_io16_workspace_bytes(const cp4_shape&);
hipError_t bwd_filter_mfma_io16_launch(const BwdFilterArgs&, hipStream_t);
// The same with IEEE half-precision x and dy in memory.
bool bwd_filter_mfma_iof16_supported(const cp4_shape&);
size_t bwd_filter_mfma_iof16_workspace_bytes(const cp4_shape&);
hipError_t bwd_filter_mfma_iof16_launch(const BwdFilterArgs&, hipStream_t);
hipError_t bwd_filter_full_launch(const cp4_shape&, const float* x,
                                  const float* dy, float* dK, int accumulate,
                                  hipStream_t);

// Utilities.
hipError_t recompose_launch(const cp4_shape&, const float* FK, const float* FC,
                            const float* FH, const float* FW, float* K,
                            hipStream_t);
hipError_t count_exceeding_launch(const float* A, const float* B, size_t n,
                                  float tol, unsigned long long* d_count,
                                  hipStream_t);
hipError_t random_uniform_launch(float* dst, size_t n, unsigned long long seed,
                                 hipStream_t);
// 3-factor CP sibling op: its factors as a CP4 of rank Y*Rank (s.Rank is the CP
// rank), and the fold of the CP4 factor gradients back onto the three factors.
hipError_t cp3_expand_launch(const cp4_shape& s, const float* K0, const float* K1,
                             const float* K2, float* FK, float* FC, float* FH, float* FW,
                             hipStream_t);
hipError_t cp3_fold_launch(const cp4_shape& s, const float* dFK, const float* dFC,
                           const float* dFW, float* dK0, float* dK1, float* dK2, hipStream_t);
// dst[row*ld_dst + c] = src[row*ld_src + c], c < cols (column blocks of factor matrices)
hipError_t copy_columns_launch(const float* src, int ld_src, float* dst, int ld_dst, int rows,
                               int cols, hipStream_t);
// dst[plane][ot + sh*u][ol + sw*v] = src[plane][u][v] on `planes` planes of h x w
// set into canvases of Hc x Wc; every other canvas cell is written as zero.
hipError_t embed_launch(const float* src, float* dst, size_t planes, int h, int w, int Hc, int Wc,
                        int ot, int ol, int sh, int sw, hipStream_t);
// Reshaped-CP sibling op: its dense filter (transposed != 0: the input-gradient
// pass's filter [C][T][Y][X], taps reversed) and the fold of a dense filter
// gradient [T][C][Y][X] back onto K0 [S0,T0,R], K1 [S1,T1,R], KC [Y,X,R].
hipError_t rcp_recompose_launch(const float* K0, const float* K1, const float* KC, float* out,
                                int S0, int S1, int T0, int T1, int Y, int X, int R,
                                int transposed, hipStream_t);
hipError_t rcp_fold_launch(const float* dK, const float* K0, const float* K1, const float* KC,
                           float* dK0, float* dK1, float* dKC, int S0, int S1, int T0, int T1,
                           int Y, int X, int R, hipStream_t);
// dst [cols, rows] = transpose of src [rows, cols]
hipError_t transpose_f32_launch(const float* src, float* dst, int rows, int cols, hipStream_t);
hipError_t copy_f32_launch(float* dst, const float* src, size_t n, hipStream_t);
hipError_t add_f32_launch(float* dst, const float* src, size_t n, hipStream_t);   // dst += src
// dst [groups][rows_padded][row_elems] = src [groups][rows][row_elems] with zero rows appended
hipError_t pad_rows_launch(const float* src, float* dst, size_t groups, size_t rows,
                           size_t rows_padded, size_t row_elems, hipStream_t);
// Fill kernel rather than a memset node, so that callers may capture the
// empty-batch paths into a graph like every other launch.
hipError_t zero_f32_launch(float* dst, size_t n, hipStream_t);

}  // namespace cp4
#endif
