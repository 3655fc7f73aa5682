/*
 * C ABI of the MI355X (gfx950) fused CP4-decomposed Conv2d library.
 *
 *   y[n,k,h,w] = sum_r FK[k,r] sum_c FC[c,r] sum_{i,j} FH[i,r] FW[j,r]
 *                x[n,c,h+i-pad,w+j-pad]            (zero padding, stride 1)
 *
 * Plain pointers and sizes only.  Every data pointer is a DEVICE pointer to
 * contiguous fp32; activations are NCHW, the four factor matrices row-major
 * [dim, Rank] in the reference's argument order (out-channel FK = "FT",
 * in-channel FC, height FH = "FY", width FW = "FX").  The passes keep no state
 * between calls, so calls on different streams may overlap; what the library
 * does keep per process is listed where it is set: the tuner's choices
 * (cp4_tune_*), the bound of the in-kernel waits (cp4_set_spin_limit) and, on
 * each device, the sticky fault record read by cp4_device_status.  Functions
 * return a status code and never exit the process.
 *
 * Non-finite inputs: the matrix-core kernels form every product from exact
 * three-way splits of the fp32 operands, and Inf - trunc(Inf) is NaN.  An Inf or
 * NaN in an activation or a factor therefore yields NaN in every output element
 * whose sum it enters - also where plain fp32 arithmetic would give +-Inf or, for
 * 0 * Inf, NaN anyway - and leaves all other elements exact.  Finite inputs
 * whose products overflow fp32 behave like fp32 (+-Inf).
 */
#ifndef CP4_CAPI_H
#define CP4_CAPI_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The nine unsigned fields of the reference's tensor_shape, same order
 * (Cuda_kernels/Tensor.cuh:10-19).  T = out-channel count K. */
typedef struct cp4_shape {
  unsigned N, H, W, pad, T, C, Y, X, Rank;
} cp4_shape;

typedef enum cp4_status {
  CP4_OK = 0,
  CP4_ERR_NULL_POINTER = 1,
  CP4_ERR_SHAPE = 2,       /* zero dim, sizes beyond the documented limits ... */
  CP4_ERR_HIP = 3,         /* a HIP runtime call failed; see cp4_last_error_message */
  CP4_ERR_WORKSPACE = 4,   /* workspace missing or too small */
  CP4_ERR_UNSUPPORTED = 5, /* requested kernel variant cannot run this shape */
  CP4_ERR_DEVICE = 6       /* a kernel gave up a wait between its waves: outputs incomplete */
} cp4_status;

/* A hipStream_t passed as void*; NULL is the default stream. */
typedef void* cp4_stream;

const char* cp4_status_string(cp4_status);
/* Detail of the calling thread's last failure ("" if none). */
const char* cp4_last_error_message(void);

/* ---- device-side failures --------------------------------------------------
 * The producer / consumer kernels (the default for most shapes of forward and
 * backward-data) hand work between the waves of a workgroup through counters in
 * LDS and wait for them with a bounded number of polls.  A wait that runs out -
 * which takes a bug in the library or a wave stalled for about a quarter of a
 * second - never lets its wave go on: the wave records the fault on the device,
 * the workgroup's other waves stop waiting, and the waves that gave up store
 * nothing further, so the outputs of that launch are incomplete rather than
 * silently wrong.  Launches are asynchronous, so the launch itself still
 * returns CP4_OK; the record is sticky until somebody reads it:
 *
 * cp4_device_status synchronises `stream`, reads and clears the current device's
 * record and returns CP4_ERR_DEVICE if a wait has run out since the last call
 * (CP4_OK otherwise).  detail, if not NULL, receives {flag, workgroup, wave, wait
 * site}.  The cp4_time_* and cp4_tune_* loops, which synchronise anyway, call it
 * themselves and return its status; so do the synchronous C++ launchers of
 * cp4conv2d.h.
 *
 * cp4_set_spin_limit sets the number of polls after which a wait gives up, for
 * every later launch of the process (0: the default, 2^19).  For fault-injection
 * tests of callers' error handling: with a limit of 1 the first wait of every
 * workgroup runs out, every wave still ends normally, and cp4_device_status
 * reports the fault. */
cp4_status cp4_device_status(cp4_stream stream, int* detail);
void cp4_set_spin_limit(int polls);

/* ---- the three passes --------------------------------------------------- */

/* Replaces cp4_conv2d_forward_gpu (Cuda_kernels/cp4Conv2dForward.cuh:7-14,
 * .cu:187-328): x[N,C,H,W] -> y[N,T,H,W].  Asynchronous on `stream`. */
cp4_status cp4_conv2d_forward(const cp4_shape* shape, const float* x,
                              const float* FK, const float* FC,
                              const float* FH, const float* FW, float* y,
                              cp4_stream stream);

/* Forward with the layer's epilogue fused into the stores:
 * y[n,t,h,w] = act(conv[n,t,h,w] + bias[t]).  The reference adds the bias as a
 * separate framework op after the convolution (test/layers.py:282, use_bias) and
 * applies the activation in another; here neither re-reads y.  bias is [T] in
 * device memory or NULL; activation is a cp4_activation. */
typedef enum cp4_activation { CP4_ACT_NONE = 0, CP4_ACT_RELU = 1 } cp4_activation;
cp4_status cp4_conv2d_forward_bias_act(const cp4_shape* shape, const float* x,
                                       const float* FK, const float* FC,
                                       const float* FH, const float* FW,
                                       const float* bias, int activation, float* y,
                                       cp4_stream stream);

/* Forward and backward-data with bfloat16 activations in memory: x / dy and
 * y / dx are NCHW arrays of 16-bit bfloat16, the four factors and the bias stay
 * fp32 and so does all arithmetic (exact products of the bf16 inputs with the
 * fp32 factors, fp32 accumulation, one rounding to nearest-even at the store).
 * Half the HBM bytes of the fp32 entry points.  The reference has fp32 only; this
 * is the layer's mixed-precision form.  Runs on the producer / consumer kernel
 * alone: CP4_ERR_UNSUPPORTED for shapes it does not take (Rank > 32, more than
 * 768 input channels, filters other than square 1/3/5/7, rows too long for its
 * whole-row strips);
 * cp4_bf16_supported answers beforehand (backward_data != 0: the shape is read
 * as that pass's, channels swapped). */
int cp4_bf16_supported(const cp4_shape* shape, int backward_data);
cp4_status cp4_conv2d_forward_bf16(const cp4_shape* shape, const void* x_bf16,
                                   const float* FK, const float* FC,
                                   const float* FH, const float* FW,
                                   const float* bias, int activation,
                                   void* y_bf16, cp4_stream stream);
cp4_status cp4_conv2d_backward_data_bf16(const cp4_shape* shape, const void* dy_bf16,
                                         const float* FK, const float* FC,
                                         const float* FH, const float* FW,
                                         void* dx_bf16, cp4_stream stream);
/* The same two passes with IEEE half-precision (fp16) activations in memory: a
 * half is exactly two bfloat16 parts, so the products with the fp32 factors are
 * still exact; y / dx are rounded once, to nearest-even (values beyond 65504
 * become infinities, as in any fp16 store).  Same shape limits as the bfloat16
 * entry points (cp4_bf16_supported answers for both). */
cp4_status cp4_conv2d_forward_f16(const cp4_shape* shape, const void* x_f16,
                                  const float* FK, const float* FC,
                                  const float* FH, const float* FW,
                                  const float* bias, int activation,
                                  void* y_f16, cp4_stream stream);
cp4_status cp4_conv2d_backward_data_f16(const cp4_shape* shape, const void* dy_f16,
                                        const float* FK, const float* FC,
                                        const float* FH, const float* FW,
                                        void* dx_f16, cp4_stream stream);
/* Backward-filter with bfloat16 (_bf16) or IEEE half (_f16) x and dy in memory;
 * factors, gradients, the workspace (cp4_conv2d_backward_filter_workspace_bytes)
 * and all arithmetic stay fp32: a bfloat16 value is one bf16 part, a half value two,
 * so the products are exact as in the fp32 pass.  Matrix-core path only: Rank <= 64,
 * C and T multiples of 16 (cp4_bf16_backward_filter_supported answers for both);
 * CP4_ERR_UNSUPPORTED otherwise. */
int cp4_bf16_backward_filter_supported(const cp4_shape* shape);
cp4_status cp4_conv2d_backward_filter_bf16(const cp4_shape* shape, const void* x_bf16,
                                           const void* dy_bf16, const float* FK,
                                           const float* FC, const float* FH,
                                           const float* FW, float* dFK, float* dFC,
                                           float* dFH, float* dFW, void* workspace,
                                           size_t workspace_bytes, cp4_stream stream);
cp4_status cp4_conv2d_backward_filter_f16(const cp4_shape* shape, const void* x_f16,
                                          const void* dy_f16, const float* FK,
                                          const float* FC, const float* FH,
                                          const float* FW, float* dFK, float* dFC,
                                          float* dFH, float* dFW, void* workspace,
                                          size_t workspace_bytes, cp4_stream stream);

/* Replaces cp4_conv2d_backward_data_gpu
 * (Cuda_kernels/cp4Conv2dBackwardData.cuh:7-14, .cu:112-282):
 * dy[N,T,H,W] -> dx[N,C,H,W] with the reference's flipped taps. */
cp4_status cp4_conv2d_backward_data(const cp4_shape* shape, const float* dy,
                                    const float* FK, const float* FC,
                                    const float* FH, const float* FW,
                                    float* dx, cp4_stream stream);

/* Replaces the four host loop nests cp4_conv2d_backward_filter_{t,c,y,x}_gpu
 * (Cuda_kernels/cp4Conv2dBackwardFilter.cuh:13-47, .cu:64-257) with one fused
 * call producing dFK[T,R], dFC[C,R], dFH[Y,R], dFW[X,R].  Outputs are
 * OVERWRITTEN (the reference's per-factor functions accumulate; the C++
 * wrappers of the same names keep that).  `workspace` must hold at least
 * cp4_conv2d_backward_filter_workspace_bytes(shape) bytes of device memory;
 * its contents are scratch.  Deterministic: no floating-point atomics.
 * The matrix-core variants want x, dy and the workspace on 16-byte boundaries, and
 * the routes that run them on copies - rank tiles beyond 64 ranks; zero channels
 * appended where a channel count is odd (on planes of an odd number of pixels: not a
 * multiple of 16), a first layer's three input channels say - the workspace on a
 * 256-byte one; operands aligned to less run the general kernel, same results. */
size_t cp4_conv2d_backward_filter_workspace_bytes(const cp4_shape* shape);
cp4_status cp4_conv2d_backward_filter(const cp4_shape* shape, const float* x,
                                      const float* dy, const float* FK,
                                      const float* FC, const float* FH,
                                      const float* FW, float* dFK, float* dFC,
                                      float* dFH, float* dFW, void* workspace,
                                      size_t workspace_bytes,
                                      cp4_stream stream);

/* cp4_conv2d_backward_filter for callers that cannot allocate.  It has no
 * counterpart in the reference; it is for code under HIP graph capture, tight
 * serving loops and harnesses that forbid hipMalloc, which cannot provide the
 * workspace above.  Same arguments without the workspace, same kernels, same
 * results bit for bit: the planes and partial sums live in a static device array
 * inside the library instead (CP4_NOALLOC_SCRATCH_BYTES per GPU the library runs
 * on, held until the process ends; its address is looked up once per device on
 * the first call there).  The call allocates and frees nothing.  Shapes whose
 * cp4_conv2d_backward_filter_workspace_bytes exceeds the array return
 * CP4_ERR_WORKSPACE (config C5, N64 C256 K256 14x14 R64, needs 23.6 MB and fits).
 * All calls on one GPU share the array: calls that overlap in time on one GPU -
 * different streams, or different host threads - race; serialise them. */
#define CP4_NOALLOC_SCRATCH_BYTES (32u << 20)
size_t cp4_noalloc_scratch_bytes(void);
cp4_status cp4_conv2d_backward_filter_noalloc(const cp4_shape* shape, const float* x,
                                              const float* dy, const float* FK,
                                              const float* FC, const float* FH,
                                              const float* FW, float* dFK, float* dFC,
                                              float* dFH, float* dFW, cp4_stream stream);

/* Same, with the kernel variant chosen by the caller: -1 library's choice,
 * 0 general (any shape), 1 matrix cores in four launches (contraction, taps,
 * gradient GEMMs, sum), 2 matrix cores in three launches with the tap step inside
 * the gradient GEMMs (square odd filters up to 5x5 with 2 * pad == Y - 1, channel
 * counts multiples of 16, H * W a multiple of 4, W >= 8, 16-byte aligned x / dy /
 * workspace), 3 the dense filter gradient over tiles of pixels followed by the chain
 * rule onto the factors, for few channels on both sides (T * C <= 256 with plain
 * multiply-adds, or on the matrix cores T <= 64, T * C * Y * X <= 16384 and a tile of
 * all channels within the LDS: 64 + 64 channels under a 1x1 filter, about 80 together
 * under 3x3; square filters of 1, 3 or 5
 * taps, pad <= Y - 1; any alignment); CP4_ERR_UNSUPPORTED if the shape does not qualify
 * for 1, 2 or 3. */
cp4_status cp4_conv2d_backward_filter_variant(const cp4_shape* shape, const float* x,
                                              const float* dy, const float* FK,
                                              const float* FC, const float* FH,
                                              const float* FW, float* dFK, float* dFC,
                                              float* dFH, float* dFW, void* workspace,
                                              size_t workspace_bytes, int variant,
                                              cp4_stream stream);

/* Variant 3 has two tile kernels and picks one by the shape (one or two output channels
 * under a 3x3 or 5x5 filter on inputs of ten million cells or more: plain multiply-adds;
 * else the matrix cores).
 * cp4_set_backward_filter_tile_kernel overrides that for every later launch of the process
 * where both can run the shape: 0 plain multiply-adds, 1 matrix cores, anything else the
 * library's choice again.  For A/B measurements and for tests that run both kernels on the
 * same inputs; no counterpart in the reference (cp4Conv2dBackwardFilter.cu has one kernel
 * sequence). */
void cp4_set_backward_filter_tile_kernel(int which);

/* Replaces cp4_conv2d_backward_filter_full_gpu
 * (Cuda_kernels/cp4Conv2dBackwardFilter.cuh:7-11, .cu:23-59): dense filter
 * gradient dK[T,C,Y,X]; accumulate != 0 adds into dK as the reference does. */
cp4_status cp4_conv2d_backward_filter_full(const cp4_shape* shape,
                                           const float* x, const float* dy,
                                           float* dK, int accumulate,
                                           cp4_stream stream);

/* ---- layer geometry: stride, explicit padding, an output plane of its own ---
 * The reference's kernels are stride 1 with an H x W output; its layer library
 * passes strides and padding = "SAME" / "VALID" on to the framework's convolutions
 * (test/layers.py:264-279).  With a cp4_geometry the operator is
 *   y[n,t,ho,wo] = sum_{c,r} FK[t,r] FC[c,r] sum_{i,j} FH[i,r] FW[j,r]
 *                  x[n,c, stride_h*ho + i - pad_top, stride_w*wo + j - pad_left]
 * on an out_h x out_w output plane; reads outside the image are zero (so the
 * padding after the image is implied by the output size).  shape->pad is not
 * used by the _ex entry points; shape->H, W describe x.  Limits: strides >= 1,
 * pad_top <= Y - 1, pad_left <= X - 1, every output window overlapping the padded
 * image (stride*(out-1) - pad < image size).  cp4_geometry_same / _valid /
 * _symmetric fill in the three usual cases: the framework's "SAME" (out =
 * ceil(in / stride), the smaller half of the zeros before the image - on even
 * sizes not the symmetric padding of a PyTorch layer), "VALID" (no zeros) and
 * `pad` zeros on every side (out = (in + 2 pad - filter) / stride + 1). */
typedef struct cp4_geometry {
  unsigned stride_h, stride_w, pad_top, pad_left, out_h, out_w;
} cp4_geometry;
cp4_status cp4_geometry_same(const cp4_shape* shape, unsigned stride_h, unsigned stride_w,
                             cp4_geometry* g);
cp4_status cp4_geometry_valid(const cp4_shape* shape, unsigned stride_h, unsigned stride_w,
                              cp4_geometry* g);
cp4_status cp4_geometry_symmetric(const cp4_shape* shape, unsigned stride_h, unsigned stride_w,
                                  unsigned pad_h, unsigned pad_w, cp4_geometry* g);
/* Forward x[N,C,H,W] -> y[N,T,out_h,out_w] = act(conv + bias) (bias [T] or NULL,
 * activation a cp4_activation).  Only the kept outputs are filtered, contracted
 * and stored: the producer / consumer kernel's strided build (square 1/3/5/7
 * filters, Rank <= 32; bias and activation fused into its stores), else the
 * general kernel followed by the in-place bias / activation kernel. */
cp4_status cp4_conv2d_forward_ex(const cp4_shape* shape, const cp4_geometry* g, const float* x,
                                 const float* FK, const float* FC, const float* FH,
                                 const float* FW, const float* bias, int activation, float* y,
                                 cp4_stream stream);
/* The two gradients of that map: dx[N,C,H,W] (the exact adjoint, whatever the
 * padding) from dy[N,T,out_h,out_w], and the four factor gradients.  With a
 * stride both read dy as it is where the matrix-core kernels take the shape: the
 * strided build's adjoint mode for dx, and for the factors a pass whose planes
 * live on two grids (A, G1 on the input's, G3, Cc on the output's).  Otherwise dy
 * is first spread out with zeros to stride 1 and the stride-1 kernels run.
 * `workspace`: device memory of at least cp4_conv2d_backward_ex_workspace_bytes
 * (sized for either route), 256-byte aligned. */
size_t cp4_conv2d_backward_ex_workspace_bytes(const cp4_shape* shape, const cp4_geometry* g);
cp4_status cp4_conv2d_backward_data_ex(const cp4_shape* shape, const cp4_geometry* g,
                                       const float* dy, const float* FK, const float* FC,
                                       const float* FH, const float* FW, float* dx,
                                       void* workspace, size_t workspace_bytes,
                                       cp4_stream stream);
cp4_status cp4_conv2d_backward_filter_ex(const cp4_shape* shape, const cp4_geometry* g,
                                         const float* x, const float* dy, const float* FK,
                                         const float* FC, const float* FH, const float* FW,
                                         float* dFK, float* dFC, float* dFH, float* dFW,
                                         void* workspace, size_t workspace_bytes,
                                         cp4_stream stream);

/* ---- timed launches: the reference's PROFCOUNT loop ---------------------- */

/* Replace the event-timed loops of cp4Conv2dForward.cu:245-327 and
 * cp4Conv2dBackwardData.cu:165-281: `warmup` untimed launches, then
 * `profcount` launches bracketed by ONE pair of HIP events on `stream` with no
 * host synchronisation in between; *mean_us = elapsed / profcount. */
cp4_status cp4_time_forward(const cp4_shape* shape, const float* x,
                            const float* FK, const float* FC, const float* FH,
                            const float* FW, float* y, unsigned warmup,
                            unsigned profcount, float* mean_us,
                            cp4_stream stream);
/* The same loop over `nsets` distinct input / output buffer sets taken in turn
 * (launch i uses xs[i % nsets], ys[i % nsets]; host arrays of device pointers).
 * The reference's loop re-launches on one set, whose 2 x 103 MB at the
 * ResNet-stage shape stay in the part's 256 MB memory-side cache; with enough sets
 * to exceed it every launch streams from and to HBM, as a training step does. */
cp4_status cp4_time_forward_sets(const cp4_shape* shape, const float* const* xs,
                                 float* const* ys, unsigned nsets, const float* FK,
                                 const float* FC, const float* FH, const float* FW,
                                 unsigned warmup, unsigned profcount, float* mean_us,
                                 cp4_stream stream);
cp4_status cp4_time_backward_data(const cp4_shape* shape, const float* dy,
                                  const float* FK, const float* FC,
                                  const float* FH, const float* FW, float* dx,
                                  unsigned warmup, unsigned profcount,
                                  float* mean_us, cp4_stream stream);
cp4_status cp4_time_backward_filter(const cp4_shape* shape, const float* x,
                                    const float* dy, const float* FK,
                                    const float* FC, const float* FH,
                                    const float* FW, float* dFK, float* dFC,
                                    float* dFH, float* dFW, void* workspace,
                                    size_t workspace_bytes, unsigned warmup,
                                    unsigned profcount, float* mean_us,
                                    cp4_stream stream);

/* ---- kernel variants and the tuner --------------------------------------- */

/* Replaces the reference's tile heuristic (cp4Conv2dForward.cu:228-233).  The
 * forward / backward-data pass has several kernel variants; variant -1 means
 * "library's choice" (a tuned entry for this shape if cp4_tune_forward has
 * run, else a size heuristic; the environment variable
 * CP4_FORWARD_VARIANT=<variant name>, read once at the first launch of the
 * process, overrides the heuristic for the shapes that variant supports). */
int cp4_forward_variant_count(void);
const char* cp4_forward_variant_name(int variant);
/* CP4_OK if `variant` can run `shape`, else CP4_ERR_UNSUPPORTED. */
cp4_status cp4_forward_variant_supported(const cp4_shape* shape, int variant);
/* The variant the library's choice falls on for `shape` (forward, or the
 * backward-data pass of that layer): the tuned entry if there is one, else the
 * heuristic - the CP4_FORWARD_VARIANT override included, so this names what a launch
 * would run, not what the heuristic alone would pick; -1 if the shape is invalid or
 * no variant takes it. */
int cp4_forward_default_variant(const cp4_shape* shape, int backward_data);
cp4_status cp4_conv2d_forward_variant(const cp4_shape* shape, const float* x,
                                      const float* FK, const float* FC,
                                      const float* FH, const float* FW,
                                      float* y, int variant,
                                      cp4_stream stream);
/* Times every variant that supports `shape` (warmup + profcount launches
 * each) on the caller's buffers - the producer / consumer variants once per
 * strip height (tile height x width for wide planes) up to 16 rows and with each
 * of the consumers' schedules (role split by the kernel's rule, off, whole pixel
 * groups per wave); the few-channel tiled variant once per tile height, tile
 * width (32, 64, 128 columns) and workgroup size (schedule 0: eight waves, 2:
 * four, 1: its own rule) - remembers the fastest for this shape for the
 * rest of the process (a process-wide table behind a mutex; cp4_tune_clear
 * empties it) and reports it.  cp4_tune_backward_data does the same for that
 * pass, cp4_tune_backward_filter chooses between that pass's three variants.
 * cp4_tuned_choice reports what a shape would run with now: the variant, the
 * tuned tile (rows, columns; 0 = the kernel's own planner) and the consumers'
 * schedule (1 = the kernel's rule, 0 = no role split, 2 = whole groups per wave). */
cp4_status cp4_tune_forward(const cp4_shape* shape, const float* x,
                            const float* FK, const float* FC, const float* FH,
                            const float* FW, float* y, unsigned warmup,
                            unsigned profcount, int* best_variant,
                            float* best_us, cp4_stream stream);
cp4_status cp4_tune_backward_data(const cp4_shape* shape, const float* dy,
                                  const float* FK, const float* FC, const float* FH,
                                  const float* FW, float* dx, unsigned warmup,
                                  unsigned profcount, int* best_variant,
                                  float* best_us, cp4_stream stream);
cp4_status cp4_tune_backward_filter(const cp4_shape* shape, const float* x, const float* dy,
                                    const float* FK, const float* FC, const float* FH,
                                    const float* FW, float* dFK, float* dFC, float* dFH,
                                    float* dFW, void* workspace, size_t workspace_bytes,
                                    unsigned warmup, unsigned profcount, int* best_variant,
                                    float* best_us, cp4_stream stream);
cp4_status cp4_tuned_choice(const cp4_shape* shape, int backward_data, int* variant,
                            int* tile_rows, int* tile_cols, int* role_split);
/* What a launch of `shape` would run with now, for reports and benchmarks: pass 0 =
 * forward, 1 = backward-data, 2 = backward-filter.  `variant` indexes
 * cp4_forward_variant_name (passes 0, 1) or cp4_backward_filter_variant_name (pass 2,
 * for operands and a workspace aligned to 16 bytes); for the whole-row strip kernels
 * (32 and 64 ranks) and the few-channel tiled kernel `strip_rows` and `workgroups` are
 * the planner's strip / tile height and grid, else 0.
 * No counterpart in the reference, whose kernel has one fixed tile
 * (reference/kernels/cp4Conv2dForward.cu:183-198). */
cp4_status cp4_plan_query(const cp4_shape* shape, int pass, int* variant, int* strip_rows,
                          int* workgroups);
/* Enters a choice into the table as cp4_tune_forward / cp4_tune_backward_data
 * would (one saved from an earlier process, say), in cp4_tuned_choice's terms.
 * `tile_cols` is 0, 32, 64, 128 or 256 (which of them a variant takes is its own matter).
 * CP4_ERR_UNSUPPORTED if the variant does not take the shape with that tile. */
cp4_status cp4_set_tuned_choice(const cp4_shape* shape, int backward_data, int variant,
                                int tile_rows, int tile_cols, int schedule);
/* The table of cp4_tune_forward / cp4_tune_backward_data as a list, in
 * cp4_tuned_choice's terms: a process can save it and a later one re-enter it
 * with cp4_set_tuned_choice (variant numbers are those of this build of the
 * library: keep cp4_forward_variant_name beside them). */
int cp4_tuned_count(void);
cp4_status cp4_tuned_entry(int index, cp4_shape* shape, int* backward_data, int* variant,
                           int* tile_rows, int* tile_cols, int* schedule);
/* The backward-filter tuner's table (cp4_tune_backward_filter): enumeration, entry by
 * hand and the names of that pass's variants (NULL past the last), so that a table can
 * be carried from one process to the next like the forward one. */
const char* cp4_backward_filter_variant_name(int variant);
int cp4_tuned_filter_count(void);
cp4_status cp4_tuned_filter_entry(int index, cp4_shape* shape, int* variant);
cp4_status cp4_set_tuned_filter_choice(const cp4_shape* shape, int variant);
void cp4_tune_clear(void);

/* ---- device allocator / copy helpers (the reference's Tensor uses
 * cudaMallocManaged, Cuda_kernels/Tensor.cu:8-39) ------------------------- */
cp4_status cp4_set_device(int ordinal);
cp4_status cp4_device_malloc(void** ptr, size_t bytes);
cp4_status cp4_device_free(void* ptr);
cp4_status cp4_host_malloc(void** ptr, size_t bytes); /* pinned */
cp4_status cp4_host_free(void* ptr);
cp4_status cp4_memcpy_h2d(void* dst, const void* src, size_t bytes, cp4_stream);
cp4_status cp4_memcpy_d2h(void* dst, const void* src, size_t bytes, cp4_stream);
cp4_status cp4_memcpy_d2d(void* dst, const void* src, size_t bytes, cp4_stream);
cp4_status cp4_memset_zero(void* dst, size_t bytes, cp4_stream);
/* *is_device = 1 if ptr is device (HBM) memory, 0 for host memory of any
 * kind (pinned, pageable, unknown to the runtime). */
cp4_status cp4_pointer_is_device(const void* ptr, int* is_device);
cp4_status cp4_stream_synchronize(cp4_stream);
cp4_status cp4_device_synchronize(void);

/* ---- 3-factor CP sibling op ------------------------------------------------
 * Stands where the reference registers its TensorFlow op Conv2dCpFusedNchw
 * (Kernels/cp_fused_nchw.cc:6-30, launcher Conv2dCpFusedNchwKernelLauncher :33):
 *   y[n,t,h,w] = sum_r K2[r,t] sum_{i,j} K1[i,j,r] sum_c K0[c,r] x[n,c,h+i-pad,w+j-pad]
 * with K0 [C,Rank], K1 [Y,X,Rank], K2 [Rank,T] (the reference's op is a generated
 * kernel for the single shape N1 C16 32x32 3x3 Rank 6 T16; any shape here).
 * The op runs on the CP4 kernels: cp3_expand_factors writes the equivalent CP4
 * factors of rank Y*Rank (FK [T,Y*Rank], FC [C,Y*Rank], FH [Y,Y*Rank] - unit
 * columns -, FW [X,Y*Rank]); the products with those ones and zeros are exact for
 * finite inputs.  For training, run cp4_conv2d_backward_data / _backward_filter
 * on the expanded factors (shape.Rank = Y*Rank) and cp3_fold_gradients on the
 * result: dK0 [C,Rank], dK1 [Y,X,Rank], dK2 [Rank,T], fixed summation order.
 * In every cp3_* call shape->Rank is the CP rank. */
cp4_status cp3_expand_factors(const cp4_shape* shape, const float* K0,
                              const float* K1, const float* K2, float* FK,
                              float* FC, float* FH, float* FW, cp4_stream stream);
cp4_status cp3_fold_gradients(const cp4_shape* shape, const float* dFK,
                              const float* dFC, const float* dFW, float* dK0,
                              float* dK1, float* dK2, cp4_stream stream);
/* Forward and input gradient in one call each; `workspace` (device memory, at
 * least cp3_conv2d_forward_workspace_bytes(shape) bytes, either pass) is scratch
 * for rewritten factors.  With Rank <= 32 and a 1x1 or 3x3 filter the producer /
 * consumer kernel applies K1 itself in its tap step (only K2 is transposed);
 * other shapes run on the expanded factors.  The input gradient uses the
 * reference's backward-data convention (flipped taps at offset +y-pad,
 * Cuda_kernels/cp4Conv2dBackwardData.cu:79-87): the adjoint of the forward when
 * 2*pad = Y-1 = X-1. */
size_t cp3_conv2d_forward_workspace_bytes(const cp4_shape* shape);
cp4_status cp3_conv2d_forward(const cp4_shape* shape, const float* x,
                              const float* K0, const float* K1, const float* K2,
                              float* y, void* workspace, size_t workspace_bytes,
                              cp4_stream stream);
cp4_status cp3_conv2d_backward_data(const cp4_shape* shape, const float* dy,
                                    const float* K0, const float* K1,
                                    const float* K2, float* dx, void* workspace,
                                    size_t workspace_bytes, cp4_stream stream);

/* The factor gradients of the 3-factor op in one call: dK0 [C,Rank], dK1 [Y,X,Rank],
 * dK2 [Rank,T].  `workspace`: cp3_conv2d_backward_filter_workspace_bytes.  With more
 * than 32 expanded ranks (Y*Rank), where the matrix-core backward-filter applies and
 * a plane pair fits LDS (H*W up to about 8000), the pass runs on Rank planes with
 * K1 applied as it is - the channel contractions and gradient products do a Y-th
 * of the work of the rewriting; other shapes run cp3_expand_factors, the CP4 pass
 * at rank Y*Rank and cp3_fold_gradients. */
size_t cp3_conv2d_backward_filter_workspace_bytes(const cp4_shape* shape);
cp4_status cp3_conv2d_backward_filter(const cp4_shape* shape, const float* x, const float* dy,
                                      const float* K0, const float* K1, const float* K2,
                                      float* dK0, float* dK1, float* dK2, void* workspace,
                                      size_t workspace_bytes, cp4_stream stream);

/* ---- reshaped-CP sibling op -------------------------------------------------
 * Stands where the reference registers its TensorFlow op Conv2dRcpFusedNchw
 * (Kernels/rcp_fused_nchw.cc:6-12, launcher Conv2dRcpFusedNchwKernelLauncher :32; a
 * generated kernel for the single shape 1 x (4,4) x 32 x 32, rank 11; defined by
 * test/test_conv2d_rcp.py:38-41 and the layer test/layers.py:687-760): the C = S0*S1
 * input channels are the pairs (a,b) of a grid, the T = T0*T1 output channels the
 * pairs (x,y), and
 *   y[n,(x,y),h,w] = sum_{a,b,i,j,r} K0[a,x,r] K1[b,y,r] KC[i,j,r] x[n,(a,b),h+i-pad,w+j-pad]
 * with K0 [S0,T0,Rank], K1 [S1,T1,Rank], KC [Y,X,Rank], channel (a,b) = a*S1 + b.
 * Each rank couples every input channel with every output channel, so there is no
 * [N,Rank,H,W] intermediate to pass through as in the CP ops; for the channel
 * counts the op is meant for (16 in the reference) the cheaper order is the dense
 * filter, recomposed on the device, in a direct convolution (the recomposed-filter
 * kernel of the CP4 passes; with more than 8192 / (8*Y*X) input channels - 113 at
 * 3x3 - the filter's weights stream through LDS by channel chunk).  Square odd
 * filters up to 17x17, pad <= Y - 1; CP4_ERR_UNSUPPORTED beyond.  shape->C and shape->T must equal
 * S0*S1 and T0*T1.  `workspace`: device memory of rcp_conv2d_workspace_bytes (the
 * dense filter and, for the factor gradients, its gradient).  The input gradient
 * follows the reference's backward-data convention (reversed taps at offset
 * +y-pad): the adjoint of the forward when 2*pad = Y-1 = X-1. */
typedef struct rcp_dims {
  unsigned S0, S1, T0, T1;
} rcp_dims;
size_t rcp_conv2d_workspace_bytes(const cp4_shape* shape, const rcp_dims* dims);
cp4_status rcp_conv2d_forward(const cp4_shape* shape, const rcp_dims* dims, const float* x,
                              const float* K0, const float* K1, const float* KC, float* y,
                              void* workspace, size_t workspace_bytes, cp4_stream stream);
cp4_status rcp_conv2d_backward_data(const cp4_shape* shape, const rcp_dims* dims, const float* dy,
                                    const float* K0, const float* K1, const float* KC, float* dx,
                                    void* workspace, size_t workspace_bytes, cp4_stream stream);
cp4_status rcp_conv2d_backward_filter(const cp4_shape* shape, const rcp_dims* dims,
                                      const float* x, const float* dy, const float* K0,
                                      const float* K1, const float* KC, float* dK0, float* dK1,
                                      float* dKC, void* workspace, size_t workspace_bytes,
                                      cp4_stream stream);

/* ---- test / bench utilities (Cuda_kernels/Utils.cuh:9-13) ---------------- */

/* Replaces cp_recompose (Utils.cu:36-98): K[T,C,Y,X] = sum_r FK FC FH FW. */
cp4_status cp4_recompose(const cp4_shape* shape, const float* FK,
                         const float* FC, const float* FH, const float* FW,
                         float* K, cp4_stream stream);
/* Replaces arrayRelativeDelta / AllClose (Utils.cu:143-180): *count = number
 * of elements with symmetric relative error > tol (absolute error if either
 * value is 0).  Synchronises `stream`. */
cp4_status cp4_count_exceeding(const float* A, const float* B, size_t n,
                               float tol, long long* count, cp4_stream stream);
/* Replaces random_fill's generator (Utils.cu:22-33): uniform in (0,1], a
 * counter-based hash of (seed, index), reproducible on any device. */
cp4_status cp4_random_uniform(float* dst, size_t n, unsigned long long seed,
                              cp4_stream stream);
/* Plain streaming copy (one read + one write per element); the calibration
 * kernel for bandwidth and for hardware-counter scale factors. */
cp4_status cp4_copy_f32(float* dst, const float* src, size_t n, cp4_stream);
cp4_status cp4_time_copy_f32(float* dst, const float* src, size_t n,
                             unsigned warmup, unsigned profcount,
                             float* mean_us, cp4_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* CP4_CAPI_H */
