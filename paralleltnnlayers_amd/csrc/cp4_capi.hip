// C ABI entry points: argument checks, kernel-variant choice, the PROFCOUNT
// timing loops and the device allocator / copy helpers.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "cp4_internal.h"

namespace {

using cp4::FwdArgs;

thread_local char g_err[256] = "";

// Sticky record of the first in-kernel wait that ran out on this device since the
// last cp4_device_status: {nonzero, workgroup, wave, wait site}.  One copy per GPU.
__device__ int g_device_fault[4];

// Scratch of cp4_conv2d_backward_filter_noalloc: the planes and partial sums the
// backward-filter kernels otherwise keep in the caller's workspace.  Every GPU the
// library runs on holds its own copy, at its own address, until the process ends.
// In host code the array's name is only a stand-in for those copies: the address
// to hand to kernels comes from hipGetSymbolAddress (scratch_of_current_device).
constexpr size_t kScratchBytes = (size_t)CP4_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_dev_mu;
int* g_fault_ptr[kMaxDevices];
void* g_scratch_ptr[kMaxDevices];
int g_num_cus[kMaxDevices];
std::atomic<int> g_spin_limit{0};

cp4_status fail(cp4_status st, const char* what) {
  std::snprintf(g_err, sizeof(g_err), "%s", what);
  return st;
}
cp4_status hip_fail(hipError_t e, const char* where) {
  std::snprintf(g_err, sizeof(g_err), "%s: %s", where, hipGetErrorString(e));
  return CP4_ERR_HIP;
}
#define CP4_HIP(call)                                  \
  do {                                                 \
    hipError_t e_ = (call);                            \
    if (e_ != hipSuccess) return hip_fail(e_, #call);  \
  } while (0)

hipStream_t as_stream(cp4_stream s) { return static_cast<hipStream_t>(s); }

// Address of this device's fault record (null if the runtime cannot say).
int* fault_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_dev_mu);
  if (!g_fault_ptr[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(g_device_fault)) != hipSuccess) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_fault_ptr[dev] = static_cast<int*>(p);
  }
  return g_fault_ptr[dev];
}

// Address of the current device's copy of `scratch`: looked up once per device,
// with that device current, and kept.
cp4_status scratch_of_current_device(void** out) {
  int dev = -1;
  CP4_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(CP4_ERR_UNSUPPORTED, "device ordinal beyond the library's table");
  std::lock_guard<std::mutex> lk(g_dev_mu);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    CP4_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return fail(CP4_ERR_HIP, "hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return CP4_OK;
}

// The launch context every producer / consumer launch carries.  A launch without a
// fault record could give up a wait unseen, so an unresolved record is an error.
cp4_status arm(FwdArgs& a) {
  a.fault = fault_of_current_device();
  if (!a.fault)
    return fail(CP4_ERR_HIP, "the device's fault record could not be resolved (hipGetSymbolAddress)");
  a.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
  return CP4_OK;
}
#define CP4_ARM(a)                     \
  do {                                 \
    const cp4_status rc_ = arm(a);     \
    if (rc_ != CP4_OK) return rc_;     \
  } while (0)

// Synchronise `st`, read and clear the device's fault record.
cp4_status device_status(hipStream_t st, int* detail) {
  CP4_HIP(hipStreamSynchronize(st));
  int rec[4] = {0, 0, 0, 0};
  int* p = fault_of_current_device();
  if (p) {
    CP4_HIP(hipMemcpy(rec, p, sizeof(rec), hipMemcpyDeviceToHost));
    if (rec[0]) {
      const int zero[4] = {0, 0, 0, 0};
      CP4_HIP(hipMemcpy(p, zero, sizeof(zero), hipMemcpyHostToDevice));
    }
  }
  if (detail) memcpy(detail, rec, sizeof(rec));
  if (!rec[0]) return CP4_OK;
  std::snprintf(g_err, sizeof(g_err),
                "a wait between waves ran out in workgroup %d, wave %d, wait site %d: the "
                "outputs of launches since the last status check are incomplete",
                rec[1], rec[2], rec[3]);
  return CP4_ERR_DEVICE;
}

// Shape rules shared by the three passes.  N == 0 is a valid empty batch.
cp4_status check_shape(const cp4_shape* s) {
  if (!s) return fail(CP4_ERR_NULL_POINTER, "shape is NULL");
  if (!s->H || !s->W || !s->T || !s->C || !s->Y || !s->X || !s->Rank)
    return fail(CP4_ERR_SHAPE, "H, W, T, C, Y, X and Rank must be >= 1");
  if ((unsigned long long)s->H * s->W >= (1ull << 31))
    return fail(CP4_ERR_SHAPE, "H*W must be below 2^31");
  if (s->N > 65535u) return fail(CP4_ERR_SHAPE, "N must be <= 65535");
  if (s->T > 65535u || s->C > 65535u || s->Rank > 65535u)
    return fail(CP4_ERR_SHAPE, "T, C and Rank must be <= 65535");
  if (s->Y > 1024u || s->X > 1024u || s->pad > 1024u)
    return fail(CP4_ERR_SHAPE, "Y, X and pad must be <= 1024");
  return CP4_OK;
}

FwdArgs forward_args(const cp4_shape& s, const float* x, const float* FK,
                     const float* FC, const float* FH, const float* FW,
                     float* y) {
  FwdArgs a{};
  a.x = x; a.Fin = FC; a.Fout = FK; a.FH = FH; a.FW = FW; a.y = y;
  a.N = s.N; a.Cin = s.C; a.Cout = s.T; a.H = s.H; a.W = s.W; a.pad = s.pad;
  a.Y = s.Y; a.X = s.X; a.R = s.Rank; a.flip = 0;
  return a;
}
// Backward-data is the forward kernel on dy with the channel factors swapped
// and the taps read in reverse (cp4Conv2dBackwardData.cu:79-87,98-108).
FwdArgs backward_data_args(const cp4_shape& s, const float* dy, const float* FK,
                           const float* FC, const float* FH, const float* FW,
                           float* dx) {
  FwdArgs a{};
  a.x = dy; a.Fin = FK; a.Fout = FC; a.FH = FH; a.FW = FW; a.y = dx;
  a.N = s.N; a.Cin = s.T; a.Cout = s.C; a.H = s.H; a.W = s.W; a.pad = s.pad;
  a.Y = s.Y; a.X = s.X; a.R = s.Rank; a.flip = 1;
  return a;
}

struct Variant {
  const char* name;
  bool (*supported)(const FwdArgs&);
  hipError_t (*launch)(const FwdArgs&, hipStream_t);
};
// More than 32 ranks or more than 768 input channels on the producer / consumer kernel
// (which holds 32 and 768): the sum over ranks splits, and so does the sum over input
// channels, so the kernel runs on ranks [0, 32) of the first channels, then with y += on
// the next 32 ranks, and so on through every (channel slice, rank tile) pair - the factor
// pointers moved 32 columns in per rank tile (row stride unchanged) and a slice's rows
// down, x moved a slice's planes in (image stride unchanged).  Every pass reads its slice
// of x again (and y, after the first).  Without the channel slices a layer with 1024
// input channels - or the backward-data pass of one with 1000 outputs - ran the general
// VALU kernel (N4 C512 K1000 32x32 R64 backward-data: 3.3 ms).
constexpr int kMaxPasses = 16;        // rank tiles x channel slices
constexpr int kPassMaxChannels = 768;   // one pass up to here ...
constexpr int kSliceMaxChannels = 512;  // ... slices no wider than this (98 KB of factor fragments in LDS)
int rank_passes(const FwdArgs& a) { return (a.R + 31) / 32; }
int channel_slices(const FwdArgs& a) {
  return a.Cin <= kPassMaxChannels ? 1 : (a.Cin + kSliceMaxChannels - 1) / kSliceMaxChannels;
}
int slice_channels(const FwdArgs& a) {          // channels per slice, a multiple of 16
  const int n = channel_slices(a);
  return ((a.Cin + n - 1) / n + 15) / 16 * 16;
}
FwdArgs pass_args(const FwdArgs& a, int slice, int tile) {
  FwdArgs b = a;
  b.ldf = a.R;
  const int r0 = 32 * tile, c0 = slice_channels(a) * slice;
  b.R = a.R - r0 < 32 ? a.R - r0 : 32;
  b.Cin = a.Cin - c0 < slice_channels(a) ? a.Cin - c0 : slice_channels(a);
  b.ldx = (size_t)a.Cin * a.H * a.W;
  b.x = a.x + (size_t)c0 * a.H * a.W;
  b.Fin += (size_t)c0 * a.R + r0; b.Fout += r0; b.FH += r0; b.FW += r0;
  b.accumulate = slice > 0 || tile > 0;
  return b;
}
// A build of the kernel that honours the pass arguments, run over every (channel slice,
// rank tile) pair of a layer it cannot take in one launch.
struct PassBuild {
  bool (*supported)(const FwdArgs&);
  hipError_t (*launch)(const FwdArgs&, hipStream_t);
};
bool passes_supported(const FwdArgs& a, const PassBuild& b) {
  if ((a.R <= 32 && a.Cin <= kPassMaxChannels) || rank_passes(a) * channel_slices(a) > kMaxPasses ||
      a.ldf || a.ldx || a.accumulate || a.bias || a.act)
    return false;
  // (the passes differ in their rank and channel counts only: the first and the last decide)
  return b.supported(pass_args(a, 0, 0)) &&
         b.supported(pass_args(a, channel_slices(a) - 1, rank_passes(a) - 1));
}
hipError_t passes_launch(const FwdArgs& a, const PassBuild& b, hipStream_t st) {
  for (int t = 0; t < rank_passes(a); ++t)
    for (int c = 0; c < channel_slices(a); ++c) {
      const hipError_t e = b.launch(pass_args(a, c, t), st);
      if (e != hipSuccess) return e;
    }
  return hipSuccess;
}
constexpr PassBuild kRankPassBuild{cp4::fwd_pipe_rankpass_supported, cp4::fwd_pipe_rankpass_launch};
bool fwd_pipe2_supported(const FwdArgs& a) { return passes_supported(a, kRankPassBuild); }
hipError_t fwd_pipe2_launch(const FwdArgs& a, hipStream_t st) {
  return passes_launch(a, kRankPassBuild, st);
}

// Passes with tiles of 64 ranks: the 64-rank single-pass kernel (which holds 33 - 64 ranks
// and 256 input channels) once per (tile of 64 ranks, slice of up to 256 channels), and the
// 32-rank build above for a last tile of up to 32 ranks.  Against passes of 32 ranks x is
// read once per 64 ranks instead of once per 32, and a layer with 33 - 64 ranks and more
// than 256 input channels reads x once in all.
constexpr int kWideTileRanks = 64, kWideSliceChannels = 256;
struct WidePass {
  int r0, rn, c0, cn;
  bool wide;            // the 64-rank kernel; else the 32-rank build
};
// The passes of a layer in launch order; 0 if there would be more than kMaxPasses.
int wide_passes(const FwdArgs& a, WidePass* out) {
  int n = 0;
  for (int r0 = 0; r0 < a.R; r0 += kWideTileRanks) {
    const int rn = a.R - r0 < kWideTileRanks ? a.R - r0 : kWideTileRanks;
    const bool wide = rn > 32;
    const int cap = wide ? kWideSliceChannels : kPassMaxChannels;
    const int most = wide ? kWideSliceChannels : kSliceMaxChannels;
    const int slices = a.Cin <= cap ? 1 : (a.Cin + most - 1) / most;
    const int per = ((a.Cin + slices - 1) / slices + 15) / 16 * 16;
    for (int c0 = 0; c0 < a.Cin; c0 += per) {
      if (n == kMaxPasses) return 0;
      out[n++] = WidePass{r0, rn, c0, a.Cin - c0 < per ? a.Cin - c0 : per, wide};
    }
  }
  return n;
}
FwdArgs wide_pass_args(const FwdArgs& a, const WidePass& p, bool first) {
  FwdArgs b = a;
  b.ldf = a.R;
  b.R = p.rn;
  b.Cin = p.cn;
  b.ldx = (size_t)a.Cin * a.H * a.W;
  b.x = a.x + (size_t)p.c0 * a.H * a.W;
  b.Fin += (size_t)p.c0 * a.R + p.r0; b.Fout += p.r0; b.FH += p.r0; b.FW += p.r0;
  b.accumulate = !first;
  return b;
}
bool fwd_pipe64_passes_supported(const FwdArgs& a) {
  if (a.R <= 32 || (a.R <= kWideTileRanks && a.Cin <= kWideSliceChannels) || a.ldf || a.ldx ||
      a.accumulate || a.bias || a.act)
    return false;
  WidePass ps[kMaxPasses];
  const int n = wide_passes(a, ps);
  for (int i = 0; i < n; ++i) {
    const FwdArgs b = wide_pass_args(a, ps[i], i == 0);
    if (!(ps[i].wide ? cp4::fwd_pipe64_supported(b) : cp4::fwd_pipe_rankpass_supported(b)))
      return false;
  }
  return n > 0;
}
hipError_t fwd_pipe64_passes_launch(const FwdArgs& a, hipStream_t st) {
  WidePass ps[kMaxPasses];
  const int n = wide_passes(a, ps);
  for (int i = 0; i < n; ++i) {
    const FwdArgs b = wide_pass_args(a, ps[i], i == 0);
    const hipError_t e = ps[i].wide ? cp4::fwd_pipe64_launch(b, st) : cp4::fwd_pipe_rankpass_launch(b, st);
    if (e != hipSuccess) return e;
  }
  return n > 0 ? hipSuccess : hipErrorInvalidValue;
}
// Channel planes moved per pixel by the passes of either kind: x once per rank tile, y
// written by every pass and read back by all but the first.
long pass_traffic(const FwdArgs& a, bool wide) {
  if (wide) {
    WidePass ps[kMaxPasses];
    const int n = wide_passes(a, ps);
    return (long)((a.R + kWideTileRanks - 1) / kWideTileRanks) * a.Cin + (long)(2 * n - 1) * a.Cout;
  }
  return (long)rank_passes(a) * a.Cin + (long)(2 * rank_passes(a) * channel_slices(a) - 1) * a.Cout;
}

// The strided build in passes over rank tiles and channel slices (more than 32 ranks or
// 768 input channels; a downsampling 1x1 layer with 1024 inputs, its backward-data pass
// with 2048): as fwd_pipe2_* for the reference's geometry, without the epilogue.
constexpr PassBuild kStridedPassBuild{cp4::fwd_pipe_strided_supported,
                                      cp4::fwd_pipe_strided_launch};
FwdArgs without_epilogue(FwdArgs a) {
  a.bias = nullptr;
  a.act = 0;
  return a;
}
bool strided_passes_supported(const FwdArgs& a) {
  return passes_supported(without_epilogue(a), kStridedPassBuild);
}
hipError_t strided_passes_launch(const FwdArgs& a, hipStream_t st) {
  return passes_launch(without_epilogue(a), kStridedPassBuild, st);
}

// Even and rectangular filters of up to 7 taps a side (2x2, 4x4, 1x7, 7x1 ...) on the matrix
// cores: the strided build runs them as the next odd square window around the filter, here
// on the reference's geometry (stride 1, `pad` zeros before the image, an H x W output), in
// passes where one launch does not hold the layer.  (Such layers ran the fp32 strip kernel
// where its LDS plan fits - N32 C256 K256 56x56 2x2 R32: 68 us, here 46 - and the general
// kernel elsewhere: N16 C192 K192 17x17 1x7 R32 400 us, here 16.)
FwdArgs on_reference_geometry(FwdArgs a) {
  a.sh = a.sw = 1;
  a.pt = a.pl = a.pad;
  a.Ho = a.H;
  a.Wo = a.W;
  return a;
}
bool fwd_window_supported(const FwdArgs& a) {
  if (a.sh || a.dense || a.taps2d || a.bias || a.act || a.accumulate || a.ldf || a.ldx) return false;
  if ((a.Y == a.X && (a.Y & 1)) || a.Y > 7 || a.X > 7) return false;   // square odd filters: the other builds
  const FwdArgs g = on_reference_geometry(a);
  return cp4::fwd_pipe_strided_supported(g) || strided_passes_supported(g);
}
hipError_t fwd_window_launch(const FwdArgs& a, hipStream_t st) {
  const FwdArgs g = on_reference_geometry(a);
  if (cp4::fwd_pipe_strided_supported(g)) return cp4::fwd_pipe_strided_launch(g, st);
  return strided_passes_launch(g, st);
}

// Order = preference of the untuned heuristic, last to first.
const Variant kVariants[] = {
    {"general_valu", cp4::fwd_general_supported, cp4::fwd_general_launch},
    {"dense_small_valu", cp4::fwd_dense_small_supported, cp4::fwd_dense_small_launch},
    {"mfma_f32_strip", cp4::fwd_mfma_supported, cp4::fwd_mfma_launch},
    {"mfma_bf16x3_strip", cp4::fwd_split_supported, cp4::fwd_split_launch},
    {"mfma_bf16x3_pipe_window", fwd_window_supported, fwd_window_launch},
    {"mfma_bf16x3_few", cp4::fwd_few_supported, cp4::fwd_few_launch},
    {"mfma_bf16x3_light", cp4::fwd_light_supported, cp4::fwd_light_launch},
    {"mfma_bf16x3_pipe_tiled", cp4::fwd_pipe_tiled_supported, cp4::fwd_pipe_tiled_launch},
    {"mfma_bf16x3_pipe", cp4::fwd_pipe_supported, cp4::fwd_pipe_launch},
    {"mfma_bf16x3_pipe_rank_passes", fwd_pipe2_supported, fwd_pipe2_launch},
    {"mfma_bf16x3_pipe64", cp4::fwd_pipe64_supported, cp4::fwd_pipe64_launch},
    {"mfma_bf16x3_pipe64_passes", fwd_pipe64_passes_supported, fwd_pipe64_passes_launch},
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

// ---- choice of kernel variant and of its tile ------------------------------------

// What runs a shape: a variant and, for the producer / consumer kernels, the tile
// the tuner measured to be best (zeros: the kernel's own planner).
struct Choice {
  int variant;
  int th, lgwt, split2;
};

using TuneKey = std::tuple<int, int, int, int, int, int, int, int, int, int>;
std::mutex g_tune_mu;
std::map<TuneKey, Choice> g_tuned;          // filled by cp4_tune_forward / _backward_data only
std::map<TuneKey, int> g_tuned_filter;      // filled by cp4_tune_backward_filter only

TuneKey key_of(const FwdArgs& a) {
  return TuneKey(a.N, a.Cin, a.Cout, a.H, a.W, a.pad, a.Y, a.X, a.R, a.flip);
}
TuneKey key_of(const cp4_shape& s) {
  return TuneKey(s.N, s.C, s.T, s.H, s.W, s.pad, s.Y, s.X, s.Rank, 2);
}

int variant_named(const char* name) {
  for (int v = 0; v < kNumVariants; ++v)
    if (!strcmp(kVariants[v].name, name)) return v;
  return -1;
}
bool is_variant(int v, const char* name) { return v >= 0 && !strcmp(kVariants[v].name, name); }

// Thresholds of the untuned heuristic, each the measured crossover on MI355X.
// Above 256 input channels the producer / consumer kernel keeps its factor in LDS
// and its strips get short; from this many pixels on, the phase-by-phase split
// kernel is then the faster one where it applies (even widths).
constexpr long kPipeLdsFactorMaxPixels = 8192;
constexpr int kPipeRegisterFactorMaxCin = 256;
// Fewer channels than this on both sides together and a rank of one or two leave
// the 32 x 32 matrix tiles almost empty: the general VALU kernel, whose cost
// follows the real counts, wins (N1 C3 K128 512x512 R1: 28 against 31 us; at rank
// 16 the matrix-core kernels win at every channel count: N1 C3 K16 512x512 27
// against 36 us, N8 C8 K8 256x256 47 against 73 us).
constexpr int kMatrixMinChannels = 24;
constexpr int kMatrixMinRank = 2;
// The recomposed-filter kernel against the kernel that would run otherwise:
// estimated microseconds per 2^18 pixels, fitted to measurements on MI355X.
// Recomposed: bound by its LDS segment reads (Cin * FS * (FS + 3) / 4 per pixel)
// more than by its Cout * Cin * FS^2 multiply-adds.  Matrix-core kernels: about
// 18 us whatever the (small) channel counts.  General VALU kernel: grows with the
// factored order's R * (Cin + Cout + Y + X).  (N1 512x512 3x3 R16: C16 K1 14
// against 25 us matrix-core, C128 K1 107 against 43; 17x17 C3 K1: 24 against 240
// us general at R16, 22 against 13 at R1.)
double dense_small_estimate(const FwdArgs& a) {
  const int groups = (a.Cout + 7) / 8;       // the segment reads repeat per group of 8 outputs
  return 8.0 + 0.155 * groups * a.Cin * a.Y * (a.X + 3) / 4.0 +
         0.0025 * a.Cout * a.Cin * a.Y * a.X;
}
constexpr double kMatrixSmallChannelEstimate = 26.0;
// Below about a million pixels the recomposed-filter kernel is bound not by that rate
// but by the time of one workgroup: each thread runs the multiply-adds of its four
// pixels in series, Cin filter rows' segment reads and Cin x min(Cout, 8) filter rows
// of multiply-adds, with one wave per vector unit to hide the LDS latency behind
// (measured on 16 x 64 tiles, 3x3, any size from a thousand pixels up: 3 -> 1 channels
// 7.4 us, 4 -> 4 12.8, 3 -> 16 15.7, 16 -> 1 23, 8 -> 8 31, 16 -> 3 34), times the
// rounds of workgroups the grid needs at six tenths of the occupancy its LDS allows
// (co-resident workgroups share the vector units).  The matrix-core kernels take
// 6 us + 16.5 us per 2^18 pixels there (few channels, rank 16: 12 us at 100,000
// pixels, 18 at 200,000, 56 at 800,000).
constexpr long kDenseSmallRateFromPixels = 1l << 20;
double dense_small_floor(const FwdArgs& a) {
  const double ko = a.Cout < 8 ? a.Cout : 8;
  // rows of whole 64-column tiles are loaded sixteen bytes a lane: the per-channel part
  // shrinks (N1 512x512, 16 -> 1: 15.4 us, 8 -> 1: 8.1, 3 -> 8: 13.8)
  const double v = a.W % 64 == 0 ? 0.65 : 1.0;
  return 3.8 * v + a.Cin * (a.Y / 3.0) * (1.2 * v + 0.34 * (ko - 1));   // (5x5, 3 -> 16: 24 us)
}
bool dense_small_loses_to_matrix(const FwdArgs& a) {
  const long pixels = (long)a.N * a.H * a.W;
  if (pixels > kDenseSmallRateFromPixels) return false;
  long tiles = 0;
  size_t lds = 0;
  if (!cp4::fwd_dense_small_plan_info(a, &tiles, &lds)) return false;
  long occ = (long)(160 * 1024 / (lds ? lds : 1));
  occ = occ < 1 ? 1 : (occ > 8 ? 8 : occ);
  const double rounds = (double)tiles / (0.6 * occ * cp4::num_compute_units());
  const double dense = dense_small_floor(a) * (rounds > 1.0 ? rounds : 1.0);
  // (the matrix-core kernels' tap step grows with the filter: 28 us per 2^18 pixels at
  // 5x5, 52 at 7x7)
  return dense > 6.0 + 16.5 * (a.Y * a.X + 9) / 18.0 * pixels / 262144.0;
}
// The few-channel tiled kernel (persistent small workgroups, taps and output contraction in
// registers) against the other kernels, over 1620 layers (3 - 64 channels in, 1 - 128 out,
// 1x1 / 3x3 / 5x5, ranks 4 and 16, a thousand to a million pixels): with up to 32 input and
// 64 output channels it is the faster one from about 60,000 pixels on - by 1.05 - 1.3 at 64
// output channels, 1.3 - 2.7 below (N16 C16 K16 512x512 R16: 271 -> 160 us, N32 C16 K16 56x56
// 13.1 -> 7.5, N16 C8 K32 256x256 84 -> 35) - and with a 1x1 filter and up to 32 output
// channels at any size (1.05 - 1.35); below that size the others are within 0.93 - 1.08 and
// stay.  Against the recomposed-filter kernel it is weighed by time: its own 4.2 us + a rate
// per 2^18 pixels (6 - 9 with up to 16 input channels, 10 - 16 with 32; 3x3; two thirds of
// that at 1x1, 1.35 times at 5x5) against the
// larger of that kernel's workgroup floor times its rounds and its rate (measured at a million
// pixels: 3 -> 1 channels 1.9 us per 2^18 pixels, 3 -> 16 7.9, 8 -> 8 8.5, 16 -> 1 8.4).
constexpr long kFewMinPixels = 60000;
constexpr int kFewMaxCin = 32, kFewMaxCout = 64, kFewPointwiseMaxCout = 32;
double few_time(const FwdArgs& a) {
  const double rate = a.Cin <= 16 ? 5.8 + 0.1 * a.Cout : 10.0 + 0.2 * a.Cout;
  return 4.2 + rate * (0.49 + 0.17 * a.Y) * (double)a.N * a.H * a.W / 262144.0;
}
double dense_small_time(const FwdArgs& a) {
  long tiles = 0;
  size_t lds = 0;
  if (!cp4::fwd_dense_small_plan_info(a, &tiles, &lds)) return 1e30;
  long occ = (long)(160 * 1024 / (lds ? lds : 1));
  occ = occ < 1 ? 1 : (occ > 8 ? 8 : occ);
  const double rounds = (double)tiles / (0.6 * occ * cp4::num_compute_units());
  const double floor_time = dense_small_floor(a) * (rounds > 1.0 ? rounds : 1.0);
  const int groups = (a.Cout + 7) / 8;
  const double rate = 1.0 + 0.1 * a.Cin * groups * a.Y + 0.011 * a.Cout * a.Cin * a.Y * a.X;
  const double rate_time = rate * (double)a.N * a.H * a.W / 262144.0;
  return floor_time > rate_time ? floor_time : rate_time;
}
bool few_preferred(const FwdArgs& a, bool over_dense_small) {
  if (a.Cin > kFewMaxCin || a.Cout > kFewMaxCout) return false;
  const long pixels = (long)a.N * a.H * a.W;
  if (pixels < kFewMinPixels && !(a.Y == 1 && a.Cout <= kFewPointwiseMaxCout)) return false;
  return !over_dense_small || few_time(a) < dense_small_time(a);
}
double general_estimate(const FwdArgs& a) {
  return 10.0 + 0.3 * a.R * (a.Cin + a.Cout + a.Y + a.X);
}

// Rows longer than this may leave whole-row strips only a row or two (2 at
// W = 224 and 32 ranks): tiles of TH x Wt then pay less for their halo.  Where the
// strips still get a few rows (up to 16 ranks the LDS plane holds half the rank
// rows) they win - long contiguous rows, no column halo: N8 C128 224x224 R16 96
// against 112 us, N16 C256 160x160 R16 203 against 254 - unless too few of them
// fill the chip or, with few channels, the halo rows cost more than they save
// (N8 C32 150x300 R16: 45 against 30 us).
constexpr int kWholeRowMaxWidth = 128;
// What the halo rows add to a strip's traffic, (rows read x Cin + rows written x
// Cout) over the same without halo: up to 1.35 with 128 input channels or more
// (1.5 with 256 on rows up to 192 pixels), else up to 1.15 on strips of at least
// four rows that fill the chip.
constexpr double kStripMaxTraffic = 1.15, kStripMaxTrafficManyChannels = 1.35;
constexpr int kStripManyChannels = 128, kStripMinRows = 4;
// With 256 input channels even two-row strips (32 ranks) beat tiles up to this
// width (N16 C256 160x160 R32: 225 against 265 us; 192 wide: 190 against 204;
// 224 wide: 291 against 249).
constexpr int kStripTwoRowMaxWidth = 192;
bool strips_on_wide_plane(const FwdArgs& a) {
  int rows = 0, wgs = 0;
  if (!cp4::fwd_pipe_strip_plan(a, &rows, &wgs)) return false;
  const double traffic =
      1.0 + (double)(a.Y - 1) * a.Cin / ((double)rows * (a.Cin + a.Cout));
  if (a.Cin >= kStripManyChannels)
    return traffic <= kStripMaxTrafficManyChannels ||
           (a.Cin >= 2 * kStripManyChannels && a.W <= kStripTwoRowMaxWidth && traffic <= 1.5);
  const bool fills = 4 * wgs >= 3 * cp4::num_compute_units();
  return traffic <= kStripMaxTraffic && rows >= kStripMinRows && fills;
}

// Two rank passes read x twice and y once more; below this many activation
// elements the fp32 matrix-core strip kernel is the faster one for ranks 33-64.
constexpr long kTwoPassMinElements = 16l << 20;

// Ranks 33-64 in one pass (the 64-rank kernel) against the fp32 strip kernel, over 248
// layers with C = K in {32 ... 256}, planes of 7 - 56 pixels a side, 1 - 64 images, 40 and 64
// ranks: the fp32 kernel is the faster one (by 1.05 - 1.9) with a 3x3 filter and up to 64
// channels below 8 M activation elements, with up to 128 channels on batches of 8 - 32
// thousand pixels (1.1 - 1.25); with a 1x1 filter and everywhere else the 64-rank kernel
// is (within 1.0 - 1.2 at 32 channels, by up to 5x at 256).
constexpr int kF32StripFewChannels = 64, kF32StripMidChannels = 128;
constexpr long kF32StripFewMaxElements = 8l << 20;
constexpr long kF32StripMidMinPixels = 8192, kF32StripMidMaxPixels = 32768;
bool f32_strip_beats_pipe64(const FwdArgs& a) {
  const long px = (long)a.N * a.H * a.W;
  const int ch = (a.Cin + a.Cout + 1) / 2;
  if (a.Y == 1) return false;
  if (ch <= kF32StripFewChannels) return px * (a.Cin + a.Cout) < kF32StripFewMaxElements;
  return ch <= kF32StripMidChannels && px >= kF32StripMidMinPixels && px < kF32StripMidMaxPixels;
}

// Passes with tiles of 64 ranks against passes of 32 ranks.  Without channel slices (up to
// 256 input channels) the 64-rank tiles read x half as often and win throughout (N32 C256
// 56x56 R96: 150 against 182 us, R128 162 / 248, R200 314 / 461; N32 C128 28x28 R128 53 /
// 66).  With more than 256 input channels they run more, shorter passes, each adding y
// once more: they win on large batches where they move a tenth less (N32 C512 K512 28x28
// R64: 132 against 157 us) and lose on small ones (N32 C1024 K256 14x14 1x1 R64: 81 / 62;
// N8 C384 K384 28x28 R96 83 / 64; N4 C512 K1000 32x32 R64 71 / 51).
constexpr long kWideSlicesMinPixels = 16384;
bool wide_passes_preferred(const FwdArgs& a) {
  if (a.Cin <= kWideSliceChannels) return true;
  return (long)a.N * a.H * a.W >= kWideSlicesMinPixels &&
         10 * pass_traffic(a, true) <= 9 * pass_traffic(a, false);
}

// Where the light kernel beats the producer / consumer kernel (and, below a few
// tens of thousands of pixels, the recomposed-filter kernel, whose threads each run
// Cout x Cin x Y x X multiply-adds per pixel quad in series): measured over 90 shapes
// it takes 0.61-0.97 of the other's time inside these bounds - N8 C16 56x56 R16 9.3 ->
// 5.7 us, N4 C32 112x112 R16 11.1 -> 9.1, N16 C8 32x32 R16 29.9 -> 5.6 - and more
// outside them: 1.0-1.1 with 48-64 input channels or 32 ranks, 1.2-2.3 from 100,000
// pixels on (its grid then needs several rounds of workgroups of 200 registers a lane).
// (whole rows: on rows beyond 128 pixels the tiled kernel stays ahead, N1 C3 K64 224x224
// 9.4 against 10.1 us)
constexpr long kLightMaxPixels = 50176;      // 4 x 112 x 112
constexpr int kLightMaxCin = 32, kLightMaxCout = 64, kLightMaxRank = 16;
constexpr double kLightMinDenseFloor = 6.0;  // us

// CP4_FORWARD_VARIANT=<name> overrides the heuristic where that variant can run the
// shape (profiling and A/B runs of unmodified callers).  Read once, at the first launch:
// the process's environment is not consulted per call.
int forced_variant() {
  static const int forced = [] {
    const char* want = getenv("CP4_FORWARD_VARIANT");
    return want ? variant_named(want) : -1;
  }();
  return forced;
}

int heuristic_variant(const FwdArgs& a) {
  const int forced = forced_variant();
  if (forced >= 0 && kVariants[forced].supported(a)) return forced;
  int pick = -1;
  for (int v = kNumVariants - 1; v >= 0 && pick < 0; --v)
    if (kVariants[v].supported(a) && !is_variant(v, "dense_small_valu")) pick = v;
  auto prefer = [&](const char* name) {
    const int v = variant_named(name);
    if (v >= 0 && kVariants[v].supported(a)) pick = v;
  };
  if (is_variant(pick, "mfma_bf16x3_pipe") && a.Cin > kPipeRegisterFactorMaxCin &&
      (long)a.N * a.H * a.W > kPipeLdsFactorMaxPixels)
    prefer("mfma_bf16x3_strip");
  if (pick >= 0 && !strncmp(kVariants[pick].name, "mfma_bf16x3_pipe", 16) &&
      a.Cin + a.Cout < kMatrixMinChannels && a.R <= kMatrixMinRank)
    prefer("general_valu");
  if (is_variant(pick, "mfma_bf16x3_pipe") && a.W > kWholeRowMaxWidth && !strips_on_wide_plane(a))
    prefer("mfma_bf16x3_pipe_tiled");
  if (is_variant(pick, "mfma_bf16x3_pipe64_passes") && fwd_pipe2_supported(a) &&
      !wide_passes_preferred(a))
    prefer("mfma_bf16x3_pipe_rank_passes");
  if (is_variant(pick, "mfma_bf16x3_pipe64")) {
    if (f32_strip_beats_pipe64(a)) prefer("mfma_f32_strip");
  } else if ((is_variant(pick, "mfma_bf16x3_pipe_rank_passes") ||
              is_variant(pick, "mfma_bf16x3_pipe64_passes")) && a.R <= 64 &&
             (long)a.N * a.H * a.W * (a.Cin + a.Cout) < kTwoPassMinElements) {
    prefer("mfma_f32_strip");
  }
  // A handful of channels on both sides: the recomposed filter costs fewer
  // multiply-adds per pixel than the factor-by-factor order.
  if (cp4::fwd_dense_small_supported(a)) {
    const bool matrix = pick >= 0 && !strncmp(kVariants[pick].name, "mfma_", 5);
    if (dense_small_estimate(a) <= (matrix ? kMatrixSmallChannelEstimate : general_estimate(a)) &&
        !(matrix && dense_small_loses_to_matrix(a)))
      prefer("dense_small_valu");
  }
  // Small problems with few channels: the light kernel's three short phases.
  // (not where the recomposed-filter kernel was picked and is as quick: 3 -> 1 channels on
  // whole tiles, 4.8 us)
  if ((long)a.N * a.H * a.W <= kLightMaxPixels && a.W <= kWholeRowMaxWidth &&
      a.Cin <= kLightMaxCin && a.Cout <= kLightMaxCout && a.R <= kLightMaxRank &&
      !(is_variant(pick, "dense_small_valu") && dense_small_floor(a) <= kLightMinDenseFloor))
    prefer("mfma_bf16x3_light");
  // Few channels from a few tens of thousands of pixels on: the tiled few-channel kernel.
  if (pick >= 0 && !is_variant(pick, "general_valu") && cp4::fwd_few_supported(a) &&
      few_preferred(a, is_variant(pick, "dense_small_valu")))
    prefer("mfma_bf16x3_few");
  return pick;
}

// The heuristic's pick per shape and operand alignment, remembered: evaluating it asks
// every kernel for its plan, several microseconds of host time that a small layer's launch
// (5 us on the device) would otherwise wait for.
std::map<std::tuple<TuneKey, unsigned>, int> g_heuristic_picks;
Choice choose(const FwdArgs& a) {
  const std::tuple<TuneKey, unsigned> hk(
      key_of(a), (unsigned)((reinterpret_cast<uintptr_t>(a.x) & 15) << 4 |
                            (reinterpret_cast<uintptr_t>(a.y) & 15)));
  {
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = g_tuned.find(key_of(a));
    if (it != g_tuned.end()) return it->second;
    auto ih = g_heuristic_picks.find(hk);
    if (ih != g_heuristic_picks.end()) return Choice{ih->second, 0, 0, 0};
  }
  const int pick = heuristic_variant(a);
  std::lock_guard<std::mutex> lk(g_tune_mu);
  if (g_heuristic_picks.size() > 4096) g_heuristic_picks.clear();
  g_heuristic_picks[hk] = pick;
  return Choice{pick, 0, 0, 0};
}

FwdArgs with_tile(const FwdArgs& a, const Choice& c) {
  FwdArgs b = a;
  b.tune_th = c.th;
  b.tune_lgwt = c.lgwt;
  b.tune_split2 = c.split2;
  return b;
}

cp4_status run_choice(const FwdArgs& a0, const Choice& c, hipStream_t st) {
  if (c.variant < 0 || c.variant >= kNumVariants)
    return fail(CP4_ERR_UNSUPPORTED, "no kernel variant supports this shape");
  FwdArgs a = with_tile(a0, c);
  if (!kVariants[c.variant].supported(a))
    return fail(CP4_ERR_UNSUPPORTED, "no kernel variant supports this shape");
  CP4_ARM(a);
  CP4_HIP(kVariants[c.variant].launch(a, st));
  return CP4_OK;
}

cp4_status run_forward_like(const FwdArgs& a, int variant, hipStream_t st) {
  if (a.N == 0) return CP4_OK;
  return run_choice(a, variant < 0 ? choose(a) : Choice{variant, 0, 0, 0}, st);
}

// Backward-filter with more than 64 ranks on the matrix-core kernels (which hold
// 64): the gradient columns of a rank depend on that rank's factor columns only,
// so the pass runs once per tile of 64 ranks on compact copies of the factor
// columns and its gradients are copied back into their columns.
constexpr unsigned kFilterRankTile = 64;
// (tiles of 32 ranks where the contraction's 64-rank factor tile of the wider channel
// side would not fit LDS: more than 640 channels)
unsigned filter_tile_ranks(const cp4_shape& s) {
  cp4_shape t = s;
  t.Rank = kFilterRankTile;
  return cp4::bwd_filter_mfma_supported(t) ? kFilterRankTile : 32;
}
cp4_shape filter_rank_tile(const cp4_shape& s, unsigned r0) {
  cp4_shape t = s;
  const unsigned tile = filter_tile_ranks(s);
  t.Rank = s.Rank - r0 < tile ? s.Rank - r0 : tile;
  return t;
}
size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }
bool filter_rank_tiles_supported(const cp4_shape& s) {
  const unsigned tile = filter_tile_ranks(s);
  return s.Rank > tile && cp4::bwd_filter_mfma_supported(filter_rank_tile(s, 0)) &&
         cp4::bwd_filter_mfma_supported(filter_rank_tile(s, (s.Rank - 1) / tile * tile));
}
size_t filter_rank_tile_floats(const cp4_shape& s) {   // compact factors or gradients of a tile
  return align256((size_t)(s.T + s.C + s.Y + s.X) * kFilterRankTile * sizeof(float)) / sizeof(float);
}

// Channel counts the matrix-core backward-filter kernels do not take - odd ones, and on
// planes of an odd number of pixels anything but multiples of 16 (a first layer's three
// input channels, a single output channel) - run them all the same on copies of x and dy
// with zero channels appended and factors with zero rows appended: the appended channels
// add nothing to A, G3 or the tap gradients, and their own gradient rows are dropped.
// The copies cost a pass over x and dy; the general kernel such a layer would otherwise
// run takes 50 to 1000 times the forward pass (N8 C3 K1 512x512 R16: 14.5 ms).
cp4_shape filter_padded_shape(const cp4_shape& s) {
  const unsigned m = ((size_t)s.H * s.W) & 1 ? 16 : 2;
  cp4_shape t = s;
  t.C = (s.C + m - 1) / m * m;
  t.T = (s.T + m - 1) / m * m;
  return t;
}
// (Also on the smallest layers: N2 C3 K5 8x8 R4 24.8 against 42.3 us.)
bool filter_pad_route(const cp4_shape& s) {
  if (cp4::bwd_filter_mfma_supported(s) || filter_rank_tiles_supported(s)) return false;
  const cp4_shape t = filter_padded_shape(s);
  if (t.C == s.C && t.T == s.T) return false;
  if (t.C > 65535 || t.T > 65535) return false;
  return cp4::bwd_filter_mfma_supported(t) || filter_rank_tiles_supported(t);
}
// Floats at the head of the workspace: padded x, dy (only where a channel is appended),
// factors FC, FK and gradients dFC, dFK, each on a 256-byte boundary.
struct FilterPadLayout {
  size_t x, dy, fc, fk, gfc, gfk, head;   // offsets in floats; head = floats before the inner workspace
};
FilterPadLayout filter_pad_layout(const cp4_shape& s, const cp4_shape& t) {
  FilterPadLayout l{};
  const size_t hw = (size_t)s.H * s.W;
  auto take = [&](size_t floats) {
    const size_t at = l.head;
    l.head += align256(floats * sizeof(float)) / sizeof(float);
    return at;
  };
  l.x = take(t.C != s.C ? (size_t)s.N * t.C * hw : 0);
  l.dy = take(t.T != s.T ? (size_t)s.N * t.T * hw : 0);
  l.fc = take((size_t)t.C * s.Rank);
  l.fk = take((size_t)t.T * s.Rank);
  l.gfc = take((size_t)t.C * s.Rank);
  l.gfk = take((size_t)t.T * s.Rank);
  return l;
}

// One workspace size serves every backward-filter variant.
size_t filter_workspace(const cp4_shape& s) {
  if (filter_pad_route(s)) {
    const cp4_shape t = filter_padded_shape(s);
    const size_t general = cp4::bwd_filter_workspace_bytes(s);
    const size_t padded = filter_pad_layout(s, t).head * sizeof(float) + filter_workspace(t);
    const size_t dense =
        cp4::bwd_filter_dense_tiles_supported(s) ? cp4::bwd_filter_dense_tiles_workspace_bytes(s) : 0;
    const size_t most = padded > general ? padded : general;
    return most > dense ? most : dense;
  }
  size_t b = cp4::bwd_filter_workspace_bytes(s);
  if (cp4::bwd_filter_mfma_supported(s)) {
    const size_t m = cp4::bwd_filter_mfma_workspace_bytes(s);
    if (m > b) b = m;
  }
  if (cp4::bwd_filter_fused_supported(s)) {
    const size_t m = cp4::bwd_filter_fused_workspace_bytes(s);
    if (m > b) b = m;
  }
  if (cp4::bwd_filter_dense_tiles_supported(s)) {
    const size_t m = cp4::bwd_filter_dense_tiles_workspace_bytes(s);
    if (m > b) b = m;
  }
  if (filter_rank_tiles_supported(s)) {
    size_t inner = cp4::bwd_filter_mfma_workspace_bytes(filter_rank_tile(s, 0));
    if (cp4::bwd_filter_fused_supported(filter_rank_tile(s, 0))) {
      const size_t f = cp4::bwd_filter_fused_workspace_bytes(filter_rank_tile(s, 0));
      if (f > inner) inner = f;
    }
    const size_t m = 2 * filter_rank_tile_floats(s) * sizeof(float) + inner;
    if (m > b) b = m;
  }
  return b;
}

cp4_status check_forward_ptrs(const void* x, const void* FK, const void* FC,
                              const void* FH, const void* FW, const void* y) {
  if (!x || !FK || !FC || !FH || !FW || !y)
    return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  return CP4_OK;
}

// `warmup` untimed launches then `profcount` launches between one event pair.
template <class Launch>
cp4_status time_loop(Launch&& launch, unsigned warmup, unsigned profcount,
                     float* mean_us, hipStream_t st) {
  if (!mean_us) return fail(CP4_ERR_NULL_POINTER, "mean_us is NULL");
  if (profcount == 0) return fail(CP4_ERR_SHAPE, "profcount must be >= 1");
  hipEvent_t e0, e1;
  CP4_HIP(hipEventCreate(&e0));
  CP4_HIP(hipEventCreate(&e1));
  cp4_status rc = CP4_OK;
  for (unsigned i = 0; i < warmup && rc == CP4_OK; ++i) rc = launch();
  hipError_t e = hipSuccess;
  if (rc == CP4_OK) e = hipEventRecord(e0, st);
  for (unsigned i = 0; i < profcount && rc == CP4_OK && e == hipSuccess; ++i)
    rc = launch();
  if (rc == CP4_OK && e == hipSuccess) e = hipEventRecord(e1, st);
  if (rc == CP4_OK && e == hipSuccess) e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (rc == CP4_OK && e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != CP4_OK) return rc;
  if (e != hipSuccess) return hip_fail(e, "timing loop");
  *mean_us = ms * 1e3f / (float)profcount;
  return device_status(st, nullptr);    // the launches are done: did any give up a wait?
}

}  // namespace

namespace cp4 {
int num_compute_units() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return 256;
  }
  std::lock_guard<std::mutex> lk(g_dev_mu);
  if (!g_num_cus[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    g_num_cus[dev] = n;
  }
  return g_num_cus[dev];
}
}  // namespace cp4

extern "C" {

const char* cp4_status_string(cp4_status s) {
  switch (s) {
    case CP4_OK: return "ok";
    case CP4_ERR_NULL_POINTER: return "null pointer";
    case CP4_ERR_SHAPE: return "invalid shape";
    case CP4_ERR_HIP: return "HIP runtime error";
    case CP4_ERR_WORKSPACE: return "workspace missing or too small";
    case CP4_ERR_UNSUPPORTED: return "unsupported kernel variant for this shape";
    case CP4_ERR_DEVICE: return "a kernel gave up a wait between its waves";
  }
  return "unknown status";
}

const char* cp4_last_error_message(void) { return g_err; }

cp4_status cp4_conv2d_forward_variant(const cp4_shape* shape, const float* x,
                                      const float* FK, const float* FC,
                                      const float* FH, const float* FW,
                                      float* y, int variant,
                                      cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(x, FK, FC, FH, FW, y);
  if (rc != CP4_OK) return rc;
  return run_forward_like(forward_args(*shape, x, FK, FC, FH, FW, y), variant,
                          as_stream(stream));
}

cp4_status cp4_conv2d_forward(const cp4_shape* shape, const float* x,
                              const float* FK, const float* FC,
                              const float* FH, const float* FW, float* y,
                              cp4_stream stream) {
  return cp4_conv2d_forward_variant(shape, x, FK, FC, FH, FW, y, -1, stream);
}

cp4_status cp4_conv2d_forward_bias_act(const cp4_shape* shape, const float* x,
                                       const float* FK, const float* FC,
                                       const float* FH, const float* FW,
                                       const float* bias, int activation, float* y,
                                       cp4_stream stream) {
  if (activation != CP4_ACT_NONE && activation != CP4_ACT_RELU)
    return fail(CP4_ERR_UNSUPPORTED, "activation must be CP4_ACT_NONE or CP4_ACT_RELU");
  if (!bias && activation == CP4_ACT_NONE)
    return cp4_conv2d_forward(shape, x, FK, FC, FH, FW, y, stream);
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(x, FK, FC, FH, FW, y);
  if (rc != CP4_OK) return rc;
  FwdArgs a = forward_args(*shape, x, FK, FC, FH, FW, y);
  a.bias = bias;
  a.act = activation;
  hipStream_t st = as_stream(stream);
  // The kernel the plain forward would pick decides: when that is the producer /
  // consumer kernel its epilogue build runs, otherwise the chosen variant is
  // followed by the in-place bias / activation kernel.
  FwdArgs plain = a;
  plain.bias = nullptr;
  plain.act = 0;
  const Choice c = choose(plain);
  if (c.variant < 0) return fail(CP4_ERR_UNSUPPORTED, "no kernel variant supports this shape");
  if (is_variant(c.variant, "mfma_bf16x3_pipe")) {
    FwdArgs e = with_tile(a, c);
    if (cp4::fwd_pipe_epi_supported(e)) {
      CP4_ARM(e);
      CP4_HIP(cp4::fwd_pipe_epi_launch(e, st));
      return CP4_OK;
    }
  }
  if (is_variant(c.variant, "mfma_bf16x3_pipe_tiled")) {
    // (the tiled build's epilogue sibling)
    FwdArgs e = with_tile(a, c);
    if (cp4::fwd_pipe_tiled_epi_supported(e)) {
      CP4_ARM(e);
      CP4_HIP(cp4::fwd_pipe_tiled_epi_launch(e, st));
      return CP4_OK;
    }
  }
  if (is_variant(c.variant, "dense_small_valu") && cp4::fwd_dense_small_supported(a)) {
    CP4_HIP(cp4::fwd_dense_small_launch(a, st));    // applies bias / activation in its stores
    return CP4_OK;
  }
  if (is_variant(c.variant, "mfma_bf16x3_light")) {
    FwdArgs e = with_tile(a, c);
    if (cp4::fwd_light_supported(e)) {
      CP4_HIP(cp4::fwd_light_launch(e, st));        // the same
      return CP4_OK;
    }
  }
  if (is_variant(c.variant, "mfma_bf16x3_few")) {
    FwdArgs e = with_tile(a, c);
    if (cp4::fwd_few_supported(e)) {
      CP4_HIP(cp4::fwd_few_launch(e, st));          // the same
      return CP4_OK;
    }
  }
  rc = run_choice(plain, c, st);
  if (rc != CP4_OK) return rc;
  CP4_HIP(cp4::bias_act_launch(y, bias, activation, shape->N, shape->T,
                               (size_t)shape->H * shape->W, st));
  return CP4_OK;
}

cp4_status cp4_conv2d_backward_data(const cp4_shape* shape, const float* dy,
                                    const float* FK, const float* FC,
                                    const float* FH, const float* FW,
                                    float* dx, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(dy, FK, FC, FH, FW, dx);
  if (rc != CP4_OK) return rc;
  return run_forward_like(backward_data_args(*shape, dy, FK, FC, FH, FW, dx),
                          -1, as_stream(stream));
}

size_t cp4_conv2d_backward_filter_workspace_bytes(const cp4_shape* shape) {
  if (check_shape(shape) != CP4_OK || shape->N == 0) return 0;
  return filter_workspace(*shape);
}

int cp4_bf16_supported(const cp4_shape* shape, int backward_data) {
  if (check_shape(shape) != CP4_OK) return 0;
  const FwdArgs a = backward_data
                        ? backward_data_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr)
                        : forward_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
  return cp4::fwd_pipe_io16_supported(a) ? 1 : 0;
}

cp4_status cp4_conv2d_forward_bf16(const cp4_shape* shape, const void* x_bf16,
                                   const float* FK, const float* FC,
                                   const float* FH, const float* FW,
                                   const float* bias, int activation,
                                   void* y_bf16, cp4_stream stream) {
  if (activation != CP4_ACT_NONE && activation != CP4_ACT_RELU)
    return fail(CP4_ERR_UNSUPPORTED, "activation must be CP4_ACT_NONE or CP4_ACT_RELU");
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(x_bf16, FK, FC, FH, FW, y_bf16);
  if (rc != CP4_OK) return rc;
  // the kernel reads FwdArgs::x / y as 16-bit elements
  FwdArgs a = forward_args(*shape, static_cast<const float*>(x_bf16), FK, FC, FH, FW,
                           static_cast<float*>(y_bf16));
  a.bias = bias;
  a.act = activation;
  CP4_ARM(a);
  if (!cp4::fwd_pipe_io16_supported(a))
    return fail(CP4_ERR_UNSUPPORTED, "bfloat16 I/O: shape not taken by the producer/consumer kernel");
  CP4_HIP(cp4::fwd_pipe_io16_launch(a, as_stream(stream)));
  return CP4_OK;
}

cp4_status cp4_conv2d_backward_data_bf16(const cp4_shape* shape, const void* dy_bf16,
                                         const float* FK, const float* FC,
                                         const float* FH, const float* FW,
                                         void* dx_bf16, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(dy_bf16, FK, FC, FH, FW, dx_bf16);
  if (rc != CP4_OK) return rc;
  FwdArgs a = backward_data_args(*shape, static_cast<const float*>(dy_bf16), FK, FC, FH, FW,
                                 static_cast<float*>(dx_bf16));
  CP4_ARM(a);
  if (!cp4::fwd_pipe_io16_supported(a))
    return fail(CP4_ERR_UNSUPPORTED, "bfloat16 I/O: shape not taken by the producer/consumer kernel");
  CP4_HIP(cp4::fwd_pipe_io16_launch(a, as_stream(stream)));
  return CP4_OK;
}

cp4_status cp4_conv2d_forward_f16(const cp4_shape* shape, const void* x_f16,
                                   const float* FK, const float* FC,
                                   const float* FH, const float* FW,
                                   const float* bias, int activation,
                                   void* y_f16, cp4_stream stream) {
  if (activation != CP4_ACT_NONE && activation != CP4_ACT_RELU)
    return fail(CP4_ERR_UNSUPPORTED, "activation must be CP4_ACT_NONE or CP4_ACT_RELU");
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(x_f16, FK, FC, FH, FW, y_f16);
  if (rc != CP4_OK) return rc;
  // the kernel reads FwdArgs::x / y as 16-bit elements
  FwdArgs a = forward_args(*shape, static_cast<const float*>(x_f16), FK, FC, FH, FW,
                           static_cast<float*>(y_f16));
  a.bias = bias;
  a.act = activation;
  CP4_ARM(a);
  if (!cp4::fwd_pipe_iof16_supported(a))
    return fail(CP4_ERR_UNSUPPORTED, "half-precision I/O: shape not taken by the producer/consumer kernel");
  CP4_HIP(cp4::fwd_pipe_iof16_launch(a, as_stream(stream)));
  return CP4_OK;
}

cp4_status cp4_conv2d_backward_data_f16(const cp4_shape* shape, const void* dy_f16,
                                         const float* FK, const float* FC,
                                         const float* FH, const float* FW,
                                         void* dx_f16, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(dy_f16, FK, FC, FH, FW, dx_f16);
  if (rc != CP4_OK) return rc;
  FwdArgs a = backward_data_args(*shape, static_cast<const float*>(dy_f16), FK, FC, FH, FW,
                                 static_cast<float*>(dx_f16));
  CP4_ARM(a);
  if (!cp4::fwd_pipe_iof16_supported(a))
    return fail(CP4_ERR_UNSUPPORTED, "half-precision I/O: shape not taken by the producer/consumer kernel");
  CP4_HIP(cp4::fwd_pipe_iof16_launch(a, as_stream(stream)));
  return CP4_OK;
}

namespace {
// Which backward-filter variants can run a shape whose operands and workspace are aligned to
// `align` bytes (variant 1 and the rank-tile route need 8, variant 2 needs 16, the rank-tile
// route a workspace on a 256-byte boundary as well), and the one a launch picks: the tuned
// entry if it can run, else the three-launch variant where it is preferred or the only
// matrix-core one, else four launches, else the general kernel.
struct FilterRoutes {
  bool tiles_ok, mfma_ok, fused_ok;
  bool dense_ok;      // variant 3: the dense filter gradient over tiles, then the chain rule
};
FilterRoutes filter_routes(const cp4_shape& s, bool aligned8, bool aligned16, bool ws256) {
  FilterRoutes r;
  r.tiles_ok = filter_rank_tiles_supported(s) && aligned8 && ws256;
  r.mfma_ok = (cp4::bwd_filter_mfma_supported(s) && aligned8) || r.tiles_ok;
  // more than 64 ranks: the fused variant runs per rank tile when every tile qualifies
  const bool fused_tiles =
      r.tiles_ok && cp4::bwd_filter_fused_supported(filter_rank_tile(s, 0)) &&
      cp4::bwd_filter_fused_supported(
          filter_rank_tile(s, (s.Rank - 1) / filter_tile_ranks(s) * filter_tile_ranks(s)));
  r.fused_ok = aligned16 && (cp4::bwd_filter_fused_supported(s) || fused_tiles);
  r.dense_ok = cp4::bwd_filter_dense_tiles_supported(s);
  return r;
}
int default_filter_variant(const cp4_shape& s, const FilterRoutes& r) {
  {
    std::lock_guard<std::mutex> lk(g_tune_mu);
    auto it = g_tuned_filter.find(key_of(s));
    if (it != g_tuned_filter.end() &&
        (it->second == 0 || (it->second == 1 && r.mfma_ok) || (it->second == 2 && r.fused_ok) ||
         (it->second == 3 && r.dense_ok)))
      return it->second;
  }
  if (r.dense_ok && cp4::bwd_filter_dense_tiles_preferred(s)) return 3;
  const bool prefer_fused =
      r.fused_ok && (cp4::bwd_filter_fused_preferred(
                         s.Rank > filter_tile_ranks(s) ? filter_rank_tile(s, 0) : s) ||
                     !r.mfma_ok);
  return prefer_fused ? 2 : (r.mfma_ok ? 1 : 0);
}
}  // namespace

cp4_status cp4_conv2d_backward_filter(const cp4_shape* shape, const float* x,
                                      const float* dy, const float* FK,
                                      const float* FC, const float* FH,
                                      const float* FW, float* dFK, float* dFC,
                                      float* dFH, float* dFW, void* workspace,
                                      size_t workspace_bytes,
                                      cp4_stream stream) {
  return cp4_conv2d_backward_filter_variant(shape, x, dy, FK, FC, FH, FW, dFK, dFC, dFH, dFW,
                                            workspace, workspace_bytes, -1, stream);
}

cp4_status cp4_conv2d_backward_filter_variant(const cp4_shape* shape, const float* x,
                                              const float* dy, const float* FK,
                                              const float* FC, const float* FH,
                                              const float* FW, float* dFK, float* dFC,
                                              float* dFH, float* dFW, void* workspace,
                                              size_t workspace_bytes, int variant,
                                              cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (!FK || !FC || !FH || !FW || !dFK || !dFC || !dFH || !dFW)
    return fail(CP4_ERR_NULL_POINTER, "a factor or gradient pointer is NULL");
  const cp4_shape& s = *shape;
  hipStream_t st = as_stream(stream);
  if (s.N == 0) {  // empty batch: the gradients are zero
    CP4_HIP(cp4::zero_f32_launch(dFK, (size_t)s.T * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dFC, (size_t)s.C * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dFH, (size_t)s.Y * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dFW, (size_t)s.X * s.Rank, st));
    return CP4_OK;
  }
  if (!x || !dy) return fail(CP4_ERR_NULL_POINTER, "x or dy is NULL");
  if (!workspace || workspace_bytes < filter_workspace(s))
    return fail(CP4_ERR_WORKSPACE,
                "workspace smaller than cp4_conv2d_backward_filter_workspace_bytes");
  const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy) |
                         reinterpret_cast<uintptr_t>(workspace);
  const FilterRoutes routes = filter_routes(s, (bits & 7) == 0, (bits & 15) == 0,
                                            (reinterpret_cast<uintptr_t>(workspace) & 255) == 0);
  const bool tiles_ok = routes.tiles_ok;
  if (variant > 3 || (variant == 1 && !routes.mfma_ok) || (variant == 2 && !routes.fused_ok) ||
      (variant == 3 && !routes.dense_ok))
    return fail(CP4_ERR_UNSUPPORTED, "backward-filter variant cannot run this shape");
  cp4::BwdFilterArgs a{};
  a.x = x; a.dy = dy; a.FK = FK; a.FC = FC; a.FH = FH; a.FW = FW;
  a.dFK = dFK; a.dFC = dFC; a.dFH = dFH; a.dFW = dFW; a.workspace = workspace;
  a.N = s.N; a.C = s.C; a.T = s.T; a.H = s.H; a.W = s.W; a.pad = s.pad;
  a.Y = s.Y; a.X = s.X; a.R = s.Rank;
  // few channels on both sides: the dense-gradient route takes any channel count as it is
  if (variant < 0 && default_filter_variant(s, routes) == 3) variant = 3;
  if (variant == 3) {
    CP4_HIP(cp4::bwd_filter_dense_tiles_launch(a, st));
    return CP4_OK;
  }
  if (variant < 0 && filter_pad_route(s) && (bits & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(workspace) & 255) == 0) {
    bool tuned_general = false;
    {
      std::lock_guard<std::mutex> lk(g_tune_mu);
      auto it = g_tuned_filter.find(key_of(s));
      tuned_general = it != g_tuned_filter.end() && it->second == 0;
    }
    if (!tuned_general) {
      // zero channels appended: the matrix-core variants on copies (see filter_padded_shape)
      const cp4_shape t = filter_padded_shape(s);
      const FilterPadLayout l = filter_pad_layout(s, t);
      float* w = static_cast<float*>(workspace);
      const size_t hw = (size_t)s.H * s.W;
      const float *xp = x, *dyp = dy;
      if (t.C != s.C) {
        CP4_HIP(cp4::pad_rows_launch(x, w + l.x, s.N, s.C, t.C, hw, st));
        xp = w + l.x;
      }
      if (t.T != s.T) {
        CP4_HIP(cp4::pad_rows_launch(dy, w + l.dy, s.N, s.T, t.T, hw, st));
        dyp = w + l.dy;
      }
      CP4_HIP(cp4::pad_rows_launch(FC, w + l.fc, 1, s.C, t.C, s.Rank, st));
      CP4_HIP(cp4::pad_rows_launch(FK, w + l.fk, 1, s.T, t.T, s.Rank, st));
      rc = cp4_conv2d_backward_filter_variant(&t, xp, dyp, w + l.fk, w + l.fc, FH, FW, w + l.gfk,
                                              w + l.gfc, dFH, dFW, w + l.head,
                                              workspace_bytes - l.head * sizeof(float), -1, stream);
      if (rc != CP4_OK) return rc;
      CP4_HIP(cp4::copy_f32_launch(dFC, w + l.gfc, (size_t)s.C * s.Rank, st));
      CP4_HIP(cp4::copy_f32_launch(dFK, w + l.gfk, (size_t)s.T * s.Rank, st));
      return CP4_OK;
    }
  }
  if (variant < 0) variant = default_filter_variant(s, routes);
  if (variant >= 1 && tiles_ok) {
    float* cf = static_cast<float*>(workspace);                 // compact factors of a tile
    float* cg = cf + filter_rank_tile_floats(s);                // compact gradients
    void* inner = cg + filter_rank_tile_floats(s);
    const int R = (int)s.Rank;
    const float* fac[4] = {FK, FC, FH, FW};
    float* grad[4] = {dFK, dFC, dFH, dFW};
    const int rows[4] = {(int)s.T, (int)s.C, (int)s.Y, (int)s.X};
    for (unsigned r0 = 0; r0 < s.Rank; r0 += filter_tile_ranks(s)) {
      const cp4_shape t = filter_rank_tile(s, r0);
      const int rt = (int)t.Rank;
      float *f[4], *g[4];
      size_t off = 0;
      for (int i = 0; i < 4; ++i) {
        f[i] = cf + off;
        g[i] = cg + off;
        off += (size_t)rows[i] * rt;
        CP4_HIP(cp4::copy_columns_launch(fac[i] + r0, R, f[i], rt, rows[i], rt, st));
      }
      cp4::BwdFilterArgs b = a;
      b.FK = f[0]; b.FC = f[1]; b.FH = f[2]; b.FW = f[3];
      b.dFK = g[0]; b.dFC = g[1]; b.dFH = g[2]; b.dFW = g[3];
      b.R = rt;
      b.workspace = inner;
      if (variant == 2) CP4_HIP(cp4::bwd_filter_fused_launch(b, st));
      else CP4_HIP(cp4::bwd_filter_mfma_launch(b, st));
      for (int i = 0; i < 4; ++i)
        CP4_HIP(cp4::copy_columns_launch(g[i], rt, grad[i] + r0, R, rows[i], rt, st));
    }
    return CP4_OK;
  }
  if (variant == 2) CP4_HIP(cp4::bwd_filter_fused_launch(a, st));
  else if (variant == 1) CP4_HIP(cp4::bwd_filter_mfma_launch(a, st));
  else CP4_HIP(cp4::bwd_filter_launch(a, st));
  return CP4_OK;
}

size_t cp4_noalloc_scratch_bytes(void) { return kScratchBytes; }

cp4_status cp4_conv2d_backward_filter_noalloc(const cp4_shape* shape, const float* x,
                                              const float* dy, const float* FK,
                                              const float* FC, const float* FH,
                                              const float* FW, float* dFK, float* dFC,
                                              float* dFH, float* dFW, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  const size_t need = shape->N ? filter_workspace(*shape) : 0;
  if (need > kScratchBytes) {
    std::snprintf(g_err, sizeof(g_err),
                  "this shape needs %zu bytes of scratch, the library's static scratch holds "
                  "%zu: use cp4_conv2d_backward_filter with a workspace",
                  need, kScratchBytes);
    return CP4_ERR_WORKSPACE;
  }
  void* ws = nullptr;
  rc = scratch_of_current_device(&ws);
  if (rc != CP4_OK) return rc;
  // The kernels write every scratch word before they read it (planes, then
  // per-workgroup partial sums, then the fixed-order reduce), so nothing has to be
  // cleared between calls; two calls in flight on one GPU would share the array.
  return cp4_conv2d_backward_filter_variant(shape, x, dy, FK, FC, FH, FW, dFK, dFC, dFH, dFW,
                                            ws, kScratchBytes, -1, stream);
}

int cp4_bf16_backward_filter_supported(const cp4_shape* shape) {
  return check_shape(shape) == CP4_OK && cp4::bwd_filter_mfma_io16_supported(*shape) ? 1 : 0;
}

namespace {
// The two 16-bit backward-filter entry points: same checks, the build for the element type.
cp4_status backward_filter_16(const cp4_shape* shape, const void* x16, const void* dy16,
                              const float* FK, const float* FC, const float* FH, const float* FW,
                              float* dFK, float* dFC, float* dFH, float* dFW, void* workspace,
                              size_t workspace_bytes, bool half, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (!FK || !FC || !FH || !FW || !dFK || !dFC || !dFH || !dFW)
    return fail(CP4_ERR_NULL_POINTER, "a factor or gradient pointer is NULL");
  const cp4_shape& s = *shape;
  hipStream_t st = as_stream(stream);
  if (s.N == 0) {  // empty batch: the gradients are zero
    CP4_HIP(cp4::zero_f32_launch(dFK, (size_t)s.T * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dFC, (size_t)s.C * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dFH, (size_t)s.Y * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dFW, (size_t)s.X * s.Rank, st));
    return CP4_OK;
  }
  if (!x16 || !dy16) return fail(CP4_ERR_NULL_POINTER, "x or dy is NULL");
  if (!cp4::bwd_filter_mfma_io16_supported(s))
    return fail(CP4_ERR_UNSUPPORTED,
                "16-bit backward-filter needs Rank <= 64 and C, T multiples of 16");
  if (!workspace || workspace_bytes < cp4::bwd_filter_mfma_io16_workspace_bytes(s))
    return fail(CP4_ERR_WORKSPACE,
                "workspace smaller than cp4_conv2d_backward_filter_workspace_bytes");
  if ((reinterpret_cast<uintptr_t>(workspace) & 7) != 0)
    return fail(CP4_ERR_WORKSPACE, "workspace must be 8-byte aligned");
  cp4::BwdFilterArgs a{};
  // the 16-bit kernels read BwdFilterArgs::x / dy as 16-bit elements
  a.x = static_cast<const float*>(x16);
  a.dy = static_cast<const float*>(dy16);
  a.FK = FK; a.FC = FC; a.FH = FH; a.FW = FW;
  a.dFK = dFK; a.dFC = dFC; a.dFH = dFH; a.dFW = dFW; a.workspace = workspace;
  a.N = s.N; a.C = s.C; a.T = s.T; a.H = s.H; a.W = s.W; a.pad = s.pad;
  a.Y = s.Y; a.X = s.X; a.R = s.Rank;
  if (half) CP4_HIP(cp4::bwd_filter_mfma_iof16_launch(a, st));
  else CP4_HIP(cp4::bwd_filter_mfma_io16_launch(a, st));
  return CP4_OK;
}
}  // namespace

cp4_status cp4_conv2d_backward_filter_bf16(const cp4_shape* shape, const void* x_bf16,
                                           const void* dy_bf16, const float* FK,
                                           const float* FC, const float* FH,
                                           const float* FW, float* dFK, float* dFC,
                                           float* dFH, float* dFW, void* workspace,
                                           size_t workspace_bytes, cp4_stream stream) {
  return backward_filter_16(shape, x_bf16, dy_bf16, FK, FC, FH, FW, dFK, dFC, dFH, dFW, workspace,
                            workspace_bytes, false, stream);
}

cp4_status cp4_conv2d_backward_filter_f16(const cp4_shape* shape, const void* x_f16,
                                          const void* dy_f16, const float* FK,
                                          const float* FC, const float* FH,
                                          const float* FW, float* dFK, float* dFC,
                                          float* dFH, float* dFW, void* workspace,
                                          size_t workspace_bytes, cp4_stream stream) {
  return backward_filter_16(shape, x_f16, dy_f16, FK, FC, FH, FW, dFK, dFC, dFH, dFW, workspace,
                            workspace_bytes, true, stream);
}

cp4_status cp4_conv2d_backward_filter_full(const cp4_shape* shape,
                                           const float* x, const float* dy,
                                           float* dK, int accumulate,
                                           cp4_stream stream) {
  cp4_shape s;
  if (!shape) return fail(CP4_ERR_NULL_POINTER, "shape is NULL");
  s = *shape;
  if (s.Rank == 0) s.Rank = 1;  // the dense gradient does not involve the rank
  cp4_status rc = check_shape(&s);
  if (rc != CP4_OK) return rc;
  if (!dK) return fail(CP4_ERR_NULL_POINTER, "dK is NULL");
  hipStream_t st = as_stream(stream);
  if (s.N == 0) {
    if (!accumulate)
      CP4_HIP(cp4::zero_f32_launch(dK, (size_t)s.T * s.C * s.Y * s.X, st));
    return CP4_OK;
  }
  if (!x || !dy) return fail(CP4_ERR_NULL_POINTER, "x or dy is NULL");
  CP4_HIP(cp4::bwd_filter_full_launch(s, x, dy, dK, accumulate, st));
  return CP4_OK;
}

// ---- layer geometry ---------------------------------------------------------

namespace {
cp4_status check_geometry(const cp4_shape* s, const cp4_geometry* g) {
  cp4_status rc = check_shape(s);
  if (rc != CP4_OK) return rc;
  if (!g) return fail(CP4_ERR_NULL_POINTER, "geometry is NULL");
  if (!g->stride_h || !g->stride_w || !g->out_h || !g->out_w)
    return fail(CP4_ERR_SHAPE, "strides and output sizes must be >= 1");
  if (g->stride_h > 1024u || g->stride_w > 1024u)
    return fail(CP4_ERR_SHAPE, "strides must be <= 1024");
  if (g->pad_top > s->Y - 1 || g->pad_left > s->X - 1)
    return fail(CP4_ERR_SHAPE, "pad_top must be <= Y - 1 and pad_left <= X - 1");
  if ((unsigned long long)g->out_h * g->out_w >= (1ull << 31))
    return fail(CP4_ERR_SHAPE, "out_h*out_w must be below 2^31");
  // the last window still starts inside the padded image
  if ((unsigned long long)g->stride_h * (g->out_h - 1) >= (unsigned long long)s->H + g->pad_top ||
      (unsigned long long)g->stride_w * (g->out_w - 1) >= (unsigned long long)s->W + g->pad_left)
    return fail(CP4_ERR_SHAPE, "the output plane reaches past the padded image");
  return CP4_OK;
}
bool is_reference_geometry(const cp4_shape& s, const cp4_geometry& g) {
  return g.stride_h == 1 && g.stride_w == 1 && g.pad_top == g.pad_left && g.out_h == s.H &&
         g.out_w == s.W;
}
void set_geometry(FwdArgs& a, const cp4_geometry& g) {
  a.sh = (int)g.stride_h; a.sw = (int)g.stride_w; a.pt = (int)g.pad_top; a.pl = (int)g.pad_left;
  a.Ho = (int)g.out_h; a.Wo = (int)g.out_w;
}

// A launch with a geometry: the strided build of the producer / consumer kernel
// where it applies and the matrix tiles are not mostly padding (in passes where one launch
// does not hold the layer), else the general kernel.
// (The strided build carries the bias / activation epilogue: a.bias / a.act are applied
// there in a single launch; *epilogue_done says whether they were.)
cp4_status run_geometry(FwdArgs a, hipStream_t st, bool* epilogue_done = nullptr) {
  if (epilogue_done) *epilogue_done = false;
  if (a.N == 0) return CP4_OK;
  CP4_ARM(a);
  if (cp4::fwd_pipe_strided_supported(a) && a.Cin + a.Cout >= kMatrixMinChannels) {
    CP4_HIP(cp4::fwd_pipe_strided_launch(a, st));
    if (epilogue_done) *epilogue_done = true;
    return CP4_OK;
  }
  if (strided_passes_supported(a)) {
    CP4_HIP(strided_passes_launch(a, st));
    return CP4_OK;
  }
  if (cp4::fwd_general_supported(a)) {
    CP4_HIP(cp4::fwd_general_launch(a, st));
    return CP4_OK;
  }
  // few channels on a geometry whose rows do not fit the general kernel's LDS tile:
  // the matrix-core build takes it after all, below the channel count it pays from
  if (cp4::fwd_pipe_strided_supported(a)) {
    CP4_HIP(cp4::fwd_pipe_strided_launch(a, st));
    if (epilogue_done) *epilogue_done = true;
    return CP4_OK;
  }
  return fail(CP4_ERR_UNSUPPORTED, "no kernel variant supports this shape and geometry");
}
// Stride-1 canvas that carries the strided layer (backward-filter): pad P on every
// side, x set in at (ot, ol), dy spread out with zeros from the origin.  The
// stride-1 layer reads canvas row h + i - P = x row h + i - P - ot, which must be
// x row h + i - pad_top: P is the smaller of the two pads and the side with more
// zeros before the image gets the difference as rows (columns) of zeros in the canvas.
struct Canvas {
  unsigned P, ot, ol, Hc, Wc;
  bool x_in_place, dy_in_place;
};
Canvas canvas_of(const cp4_shape& s, const cp4_geometry& g) {
  Canvas c;
  c.P = g.pad_top < g.pad_left ? g.pad_top : g.pad_left;
  c.ot = g.pad_top - c.P;
  c.ol = g.pad_left - c.P;
  const unsigned hu = g.stride_h * (g.out_h - 1) + 1, wu = g.stride_w * (g.out_w - 1) + 1;
  c.Hc = c.ot + s.H > hu ? c.ot + s.H : hu;
  c.Wc = c.ol + s.W > wu ? c.ol + s.W : wu;
  c.x_in_place = c.ot == 0 && c.ol == 0 && c.Hc == s.H && c.Wc == s.W;
  c.dy_in_place = g.stride_h == 1 && g.stride_w == 1 && g.out_h == c.Hc && g.out_w == c.Wc;
  return c;
}
}  // namespace

cp4_status cp4_geometry_same(const cp4_shape* s, unsigned sh, unsigned sw, cp4_geometry* g) {
  cp4_status rc = check_shape(s);
  if (rc != CP4_OK) return rc;
  if (!g) return fail(CP4_ERR_NULL_POINTER, "geometry is NULL");
  if (!sh || !sw) return fail(CP4_ERR_SHAPE, "strides must be >= 1");
  g->stride_h = sh; g->stride_w = sw;
  g->out_h = (s->H + sh - 1) / sh;
  g->out_w = (s->W + sw - 1) / sw;
  const long th = (long)(g->out_h - 1) * sh + s->Y - s->H, tw = (long)(g->out_w - 1) * sw + s->X - s->W;
  g->pad_top = th > 0 ? (unsigned)(th / 2) : 0;
  g->pad_left = tw > 0 ? (unsigned)(tw / 2) : 0;
  return CP4_OK;
}

cp4_status cp4_geometry_valid(const cp4_shape* s, unsigned sh, unsigned sw, cp4_geometry* g) {
  cp4_status rc = check_shape(s);
  if (rc != CP4_OK) return rc;
  if (!g) return fail(CP4_ERR_NULL_POINTER, "geometry is NULL");
  if (!sh || !sw) return fail(CP4_ERR_SHAPE, "strides must be >= 1");
  if (s->H < s->Y || s->W < s->X) return fail(CP4_ERR_SHAPE, "the filter is larger than the image");
  *g = cp4_geometry{sh, sw, 0, 0, (s->H - s->Y) / sh + 1, (s->W - s->X) / sw + 1};
  return CP4_OK;
}

cp4_status cp4_geometry_symmetric(const cp4_shape* s, unsigned sh, unsigned sw, unsigned ph,
                                  unsigned pw, cp4_geometry* g) {
  cp4_status rc = check_shape(s);
  if (rc != CP4_OK) return rc;
  if (!g) return fail(CP4_ERR_NULL_POINTER, "geometry is NULL");
  if (!sh || !sw) return fail(CP4_ERR_SHAPE, "strides must be >= 1");
  if (s->H + 2 * ph < s->Y || s->W + 2 * pw < s->X)
    return fail(CP4_ERR_SHAPE, "the filter is larger than the padded image");
  // the layer entry points take at most Y - 1 / X - 1 zeros before the image (a window
  // that lies wholly in the padding would produce outputs of zero): say so here, not
  // at the first launch
  if (ph > s->Y - 1 || pw > s->X - 1)
    return fail(CP4_ERR_SHAPE, "padding must be <= Y - 1 rows and <= X - 1 columns");
  *g = cp4_geometry{sh, sw, ph, pw, (s->H + 2 * ph - s->Y) / sh + 1, (s->W + 2 * pw - s->X) / sw + 1};
  return CP4_OK;
}

cp4_status cp4_conv2d_forward_ex(const cp4_shape* shape, const cp4_geometry* g, const float* x,
                                 const float* FK, const float* FC, const float* FH,
                                 const float* FW, const float* bias, int activation, float* y,
                                 cp4_stream stream) {
  if (activation != CP4_ACT_NONE && activation != CP4_ACT_RELU)
    return fail(CP4_ERR_UNSUPPORTED, "activation must be CP4_ACT_NONE or CP4_ACT_RELU");
  cp4_status rc = check_geometry(shape, g);
  if (rc != CP4_OK) return rc;
  if (is_reference_geometry(*shape, *g)) {
    cp4_shape s = *shape;
    s.pad = g->pad_top;
    return cp4_conv2d_forward_bias_act(&s, x, FK, FC, FH, FW, bias, activation, y, stream);
  }
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(x, FK, FC, FH, FW, y);
  if (rc != CP4_OK) return rc;
  FwdArgs a = forward_args(*shape, x, FK, FC, FH, FW, y);
  set_geometry(a, *g);
  a.bias = bias;
  a.act = activation;
  hipStream_t st = as_stream(stream);
  bool fused = false;
  rc = run_geometry(a, st, &fused);
  if (rc != CP4_OK) return rc;
  if (!fused && (bias || activation != CP4_ACT_NONE))
    CP4_HIP(cp4::bias_act_launch(y, bias, activation, shape->N, shape->T,
                                 (size_t)g->out_h * g->out_w, st));
  return CP4_OK;
}

size_t cp4_conv2d_backward_ex_workspace_bytes(const cp4_shape* shape, const cp4_geometry* g) {
  if (check_geometry(shape, g) != CP4_OK || shape->N == 0) return 0;
  const Canvas c = canvas_of(*shape, *g);
  cp4_shape sc = *shape;
  sc.H = c.Hc; sc.W = c.Wc; sc.pad = c.P;
  const size_t plane = (size_t)c.Hc * c.Wc * sizeof(float);
  // backward-filter: canvas x (unless in place), canvas dy, the stride-1 pass's workspace;
  // backward-data needs only dy spread out, which is no larger than canvas dy
  const size_t canvas = align256(c.x_in_place ? 0 : (size_t)shape->N * shape->C * plane) +
                        align256((size_t)shape->N * shape->T * plane) + filter_workspace(sc);
  // (the strided matrix-core pass needs far less; the maximum keeps either route open)
  const cp4::Geometry gg{(int)g->stride_h, (int)g->stride_w, (int)g->pad_top, (int)g->pad_left,
                         (int)g->out_h, (int)g->out_w};
  const size_t strided = cp4::bwd_filter_mfma_strided_supported(*shape, gg)
                             ? cp4::bwd_filter_mfma_strided_workspace_bytes(*shape, gg)
                             : 0;
  return canvas > strided ? canvas : strided;
}

cp4_status cp4_conv2d_backward_data_ex(const cp4_shape* shape, const cp4_geometry* g,
                                       const float* dy, const float* FK, const float* FC,
                                       const float* FH, const float* FW, float* dx,
                                       void* workspace, size_t workspace_bytes,
                                       cp4_stream stream) {
  cp4_status rc = check_geometry(shape, g);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  rc = check_forward_ptrs(dy, FK, FC, FH, FW, dx);
  if (rc != CP4_OK) return rc;
  const cp4_shape& s = *shape;
  hipStream_t st = as_stream(stream);
  if (is_reference_geometry(s, *g) && 2 * g->pad_top == s.Y - 1 && 2 * g->pad_left == s.X - 1) {
    // the reference's own layer: its backward-data pass is this adjoint, and has every variant
    cp4_shape r = s;
    r.pad = g->pad_top;
    return cp4_conv2d_backward_data(&r, dy, FK, FC, FH, FW, dx, stream);
  }
  // In general: dx[h,w] = sum_{i,j} K[i,j] dyu[h + pad_top - i, w + pad_left - j] with dyu = dy spread
  // out with zeros: a stride-1 pass over dyu with the taps in reverse order, Y - 1 - pad_top
  // zeros before it and an H x W output.
  if (g->stride_h > 1 || g->stride_w > 1) {
    // The strided build's adjoint mode reads dy as it is: tap (i, j) of input pixel
    // (h, w) takes dy at ((h + pad_top - i) / sh, (w + pad_left - j) / sw) where
    // both divisions are exact.
    cp4_shape sd = s;
    sd.H = g->out_h; sd.W = g->out_w;
    FwdArgs t = backward_data_args(sd, dy, FK, FC, FH, FW, dx);
    t.flip = 0;
    t.transposed = 1;
    t.sh = (int)g->stride_h; t.sw = (int)g->stride_w;
    t.pt = (int)g->pad_top; t.pl = (int)g->pad_left;
    t.Ho = (int)s.H; t.Wo = (int)s.W;
    if (cp4::fwd_pipe_strided_supported(t) && t.Cin + t.Cout >= kMatrixMinChannels) {
      CP4_ARM(t);
      CP4_HIP(cp4::fwd_pipe_strided_launch(t, st));
      return CP4_OK;
    }
    if (strided_passes_supported(t)) {
      CP4_ARM(t);
      CP4_HIP(strided_passes_launch(t, st));
      return CP4_OK;
    }
  }
  const unsigned hu = g->stride_h * (g->out_h - 1) + 1, wu = g->stride_w * (g->out_w - 1) + 1;
  const float* src = dy;
  if (g->stride_h > 1 || g->stride_w > 1) {
    const size_t need = (size_t)s.N * s.T * hu * wu * sizeof(float);
    if (!workspace || workspace_bytes < need)
      return fail(CP4_ERR_WORKSPACE, "workspace smaller than cp4_conv2d_backward_ex_workspace_bytes");
    CP4_HIP(cp4::embed_launch(dy, static_cast<float*>(workspace), (size_t)s.N * s.T, (int)g->out_h,
                              (int)g->out_w, (int)hu, (int)wu, 0, 0, (int)g->stride_h,
                              (int)g->stride_w, st));
    src = static_cast<const float*>(workspace);
  }
  cp4_shape su = s;
  su.H = hu; su.W = wu;
  FwdArgs a = backward_data_args(su, src, FK, FC, FH, FW, dx);
  a.sh = 1; a.sw = 1;
  a.pt = (int)(s.Y - 1 - g->pad_top);
  a.pl = (int)(s.X - 1 - g->pad_left);
  a.Ho = (int)s.H; a.Wo = (int)s.W;
  return run_geometry(a, st);
}

cp4_status cp4_conv2d_backward_filter_ex(const cp4_shape* shape, const cp4_geometry* g,
                                         const float* x, const float* dy, const float* FK,
                                         const float* FC, const float* FH, const float* FW,
                                         float* dFK, float* dFC, float* dFH, float* dFW,
                                         void* workspace, size_t workspace_bytes,
                                         cp4_stream stream) {
  cp4_status rc = check_geometry(shape, g);
  if (rc != CP4_OK) return rc;
  const cp4_shape& s = *shape;
  const Canvas c = canvas_of(s, *g);
  cp4_shape sc = s;
  sc.H = c.Hc; sc.W = c.Wc; sc.pad = c.P;
  if (s.N == 0 || (c.x_in_place && c.dy_in_place))
    return cp4_conv2d_backward_filter(&sc, x, dy, FK, FC, FH, FW, dFK, dFC, dFH, dFW, workspace,
                                      workspace_bytes, stream);
  if (!x || !dy) return fail(CP4_ERR_NULL_POINTER, "x or dy is NULL");
  if (!workspace || workspace_bytes < cp4_conv2d_backward_ex_workspace_bytes(shape, g))
    return fail(CP4_ERR_WORKSPACE, "workspace smaller than cp4_conv2d_backward_ex_workspace_bytes");
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
    return fail(CP4_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  hipStream_t st = as_stream(stream);
  if (g->stride_h > 1 || g->stride_w > 1) {
    // With a stride: the matrix-core pass on planes of two sizes (A, G1 on the input's
    // grid, G3, Cc on the output's), dy read as it is.
    const cp4::Geometry gg{(int)g->stride_h, (int)g->stride_w, (int)g->pad_top, (int)g->pad_left,
                           (int)g->out_h, (int)g->out_w};
    if (cp4::bwd_filter_mfma_strided_supported(s, gg)) {
      if (!FK || !FC || !FH || !FW || !dFK || !dFC || !dFH || !dFW)
        return fail(CP4_ERR_NULL_POINTER, "a factor or gradient pointer is NULL");
      cp4::BwdFilterArgs b{};
      b.x = x; b.dy = dy; b.FK = FK; b.FC = FC; b.FH = FH; b.FW = FW;
      b.dFK = dFK; b.dFC = dFC; b.dFH = dFH; b.dFW = dFW;
      b.workspace = workspace;
      b.N = (int)s.N; b.C = (int)s.C; b.T = (int)s.T; b.H = (int)s.H; b.W = (int)s.W; b.pad = 0;
      b.Y = (int)s.Y; b.X = (int)s.X; b.R = (int)s.Rank;
      CP4_HIP(cp4::bwd_filter_mfma_strided_launch(b, gg, st));
      return CP4_OK;
    }
  }
  // Otherwise the stride-1 layer on a canvas: it computes y1[sh*ho, sw*wo] = y[ho, wo]; with
  // dy spread out with zeros the loss and so the factor gradients are the same.
  unsigned char* w = static_cast<unsigned char*>(workspace);
  const size_t plane = (size_t)c.Hc * c.Wc * sizeof(float);
  const float* xc = x;
  if (!c.x_in_place) {
    CP4_HIP(cp4::embed_launch(x, reinterpret_cast<float*>(w), (size_t)s.N * s.C, (int)s.H, (int)s.W,
                              (int)c.Hc, (int)c.Wc, (int)c.ot, (int)c.ol, 1, 1, st));
    xc = reinterpret_cast<const float*>(w);
    w += align256((size_t)s.N * s.C * plane);
  }
  float* dyc = reinterpret_cast<float*>(w);
  CP4_HIP(cp4::embed_launch(dy, dyc, (size_t)s.N * s.T, (int)g->out_h, (int)g->out_w, (int)c.Hc,
                            (int)c.Wc, 0, 0, (int)g->stride_h, (int)g->stride_w, st));
  w += align256((size_t)s.N * s.T * plane);
  const size_t used = (size_t)(w - static_cast<unsigned char*>(workspace));
  return cp4_conv2d_backward_filter(&sc, xc, dyc, FK, FC, FH, FW, dFK, dFC, dFH, dFW, w,
                                    workspace_bytes - used, stream);
}

cp4_status cp4_time_forward(const cp4_shape* shape, const float* x,
                            const float* FK, const float* FC, const float* FH,
                            const float* FW, float* y, unsigned warmup,
                            unsigned profcount, float* mean_us,
                            cp4_stream stream) {
  return time_loop(
      [&] { return cp4_conv2d_forward(shape, x, FK, FC, FH, FW, y, stream); },
      warmup, profcount, mean_us, as_stream(stream));
}

cp4_status cp4_time_forward_sets(const cp4_shape* shape, const float* const* xs,
                                 float* const* ys, unsigned nsets, const float* FK,
                                 const float* FC, const float* FH, const float* FW,
                                 unsigned warmup, unsigned profcount, float* mean_us,
                                 cp4_stream stream) {
  if (!xs || !ys) return fail(CP4_ERR_NULL_POINTER, "xs or ys is NULL");
  if (nsets == 0) return fail(CP4_ERR_SHAPE, "nsets must be >= 1");
  unsigned i = 0;
  return time_loop(
      [&] {
        const unsigned k = i++ % nsets;
        return cp4_conv2d_forward(shape, xs[k], FK, FC, FH, FW, ys[k], stream);
      },
      warmup, profcount, mean_us, as_stream(stream));
}

cp4_status cp4_time_backward_data(const cp4_shape* shape, const float* dy,
                                  const float* FK, const float* FC,
                                  const float* FH, const float* FW, float* dx,
                                  unsigned warmup, unsigned profcount,
                                  float* mean_us, cp4_stream stream) {
  return time_loop(
      [&] { return cp4_conv2d_backward_data(shape, dy, FK, FC, FH, FW, dx, stream); },
      warmup, profcount, mean_us, as_stream(stream));
}

cp4_status cp4_time_backward_filter(const cp4_shape* shape, const float* x,
                                    const float* dy, const float* FK,
                                    const float* FC, const float* FH,
                                    const float* FW, float* dFK, float* dFC,
                                    float* dFH, float* dFW, void* workspace,
                                    size_t workspace_bytes, unsigned warmup,
                                    unsigned profcount, float* mean_us,
                                    cp4_stream stream) {
  return time_loop(
      [&] {
        return cp4_conv2d_backward_filter(shape, x, dy, FK, FC, FH, FW, dFK, dFC,
                                          dFH, dFW, workspace, workspace_bytes,
                                          stream);
      },
      warmup, profcount, mean_us, as_stream(stream));
}

int cp4_forward_variant_count(void) { return kNumVariants; }

const char* cp4_forward_variant_name(int v) {
  return (v >= 0 && v < kNumVariants) ? kVariants[v].name : "";
}

cp4_status cp4_forward_variant_supported(const cp4_shape* shape, int variant) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (variant < 0 || variant >= kNumVariants)
    return fail(CP4_ERR_UNSUPPORTED, "variant index out of range");
  const FwdArgs a = forward_args(*shape, nullptr, nullptr, nullptr, nullptr,
                                 nullptr, nullptr);
  return kVariants[variant].supported(a)
             ? CP4_OK
             : fail(CP4_ERR_UNSUPPORTED, "variant does not support this shape");
}

int cp4_forward_default_variant(const cp4_shape* shape, int backward_data) {
  if (check_shape(shape) != CP4_OK) return -1;
  const FwdArgs a =
      backward_data
          ? backward_data_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr)
          : forward_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
  return choose(a).variant;
}

namespace {
// Times every variant that can run the shape and, for the producer / consumer
// kernels, every strip height (tile height and width) and role split they can
// run it with; remembers the fastest.
cp4_status tune_forward_like(const FwdArgs& a, unsigned warmup, unsigned profcount,
                             int* best_variant, float* best_us, hipStream_t st) {
  Choice best{-1, 0, 0, 0};
  float best_t = 0.f;
  auto consider = [&](const Choice& c) -> cp4_status {
    if (!kVariants[c.variant].supported(with_tile(a, c))) return CP4_OK;
    float us = 0.f;
    const cp4_status rc =
        time_loop([&] { return run_choice(a, c, st); }, warmup, profcount, &us, st);
    if (rc != CP4_OK) return rc;
    if (best.variant < 0 || us < best_t) {
      best = c;
      best_t = us;
    }
    return CP4_OK;
  };
  for (int v = 0; v < kNumVariants; ++v) {
    if (!kVariants[v].supported(a)) continue;
    cp4_status rc = consider(Choice{v, 0, 0, 0});     // the kernel's own planner
    if (rc != CP4_OK) return rc;
    const bool strips = is_variant(v, "mfma_bf16x3_pipe") || is_variant(v, "mfma_bf16x3_pipe_rank_passes");
    const bool tiles = is_variant(v, "mfma_bf16x3_pipe_tiled");
    const bool few = is_variant(v, "mfma_bf16x3_few");      // tiles of 32, 64 or 128 columns
    if (!strips && !tiles && !few) continue;
    const int max_th = a.H < 16 ? a.H : 16;
    for (int lgwt = tiles ? 6 : (few ? 5 : 0); lgwt <= (tiles ? 8 : (few ? 7 : 0)); ++lgwt)
      for (int th = 1; th <= max_th; ++th)
        for (int split2 = 0; split2 <= 2; ++split2) {   // 2: consumer waves with groups of their own
          rc = consider(Choice{v, th, lgwt, split2});
          if (rc != CP4_OK) return rc;
        }
  }
  if (best.variant < 0) return fail(CP4_ERR_UNSUPPORTED, "no kernel variant supports this shape");
  {
    std::lock_guard<std::mutex> lk(g_tune_mu);
    g_tuned[key_of(a)] = best;
  }
  if (best_variant) *best_variant = best.variant;
  if (best_us) *best_us = best_t;
  return CP4_OK;
}
}  // namespace

cp4_status cp4_tune_forward(const cp4_shape* shape, const float* x,
                            const float* FK, const float* FC, const float* FH,
                            const float* FW, float* y, unsigned warmup,
                            unsigned profcount, int* best_variant,
                            float* best_us, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  rc = check_forward_ptrs(x, FK, FC, FH, FW, y);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return fail(CP4_ERR_SHAPE, "cannot tune an empty batch");
  return tune_forward_like(forward_args(*shape, x, FK, FC, FH, FW, y), warmup, profcount,
                           best_variant, best_us, as_stream(stream));
}

cp4_status cp4_tune_backward_data(const cp4_shape* shape, const float* dy,
                                  const float* FK, const float* FC, const float* FH,
                                  const float* FW, float* dx, unsigned warmup,
                                  unsigned profcount, int* best_variant,
                                  float* best_us, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  rc = check_forward_ptrs(dy, FK, FC, FH, FW, dx);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return fail(CP4_ERR_SHAPE, "cannot tune an empty batch");
  return tune_forward_like(backward_data_args(*shape, dy, FK, FC, FH, FW, dx), warmup,
                           profcount, best_variant, best_us, as_stream(stream));
}

cp4_status cp4_tune_backward_filter(const cp4_shape* shape, const float* x, const float* dy,
                                    const float* FK, const float* FC, const float* FH,
                                    const float* FW, float* dFK, float* dFC, float* dFH,
                                    float* dFW, void* workspace, size_t workspace_bytes,
                                    unsigned warmup, unsigned profcount, int* best_variant,
                                    float* best_us, cp4_stream stream) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return fail(CP4_ERR_SHAPE, "cannot tune an empty batch");
  int best = -1;
  float best_t = 0.f;
  for (int v = 0; v < 4; ++v) {
    float us = 0.f;
    rc = time_loop(
        [&] {
          return cp4_conv2d_backward_filter_variant(shape, x, dy, FK, FC, FH, FW, dFK, dFC, dFH,
                                                    dFW, workspace, workspace_bytes, v, stream);
        },
        warmup, profcount, &us, as_stream(stream));
    if (rc == CP4_ERR_UNSUPPORTED) continue;
    if (rc != CP4_OK) return rc;
    if (best < 0 || us < best_t) { best = v; best_t = us; }
  }
  if (best < 0) return fail(CP4_ERR_UNSUPPORTED, "no kernel variant supports this shape");
  {
    std::lock_guard<std::mutex> lk(g_tune_mu);
    g_tuned_filter[key_of(*shape)] = best;
  }
  if (best_variant) *best_variant = best;
  if (best_us) *best_us = best_t;
  return CP4_OK;
}

cp4_status cp4_tuned_choice(const cp4_shape* shape, int backward_data, int* variant,
                            int* tile_rows, int* tile_cols, int* role_split) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  const FwdArgs a =
      backward_data
          ? backward_data_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr)
          : forward_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
  const Choice c = choose(a);
  if (variant) *variant = c.variant;
  if (tile_rows) *tile_rows = c.th;
  if (tile_cols) *tile_cols = c.lgwt ? 1 << c.lgwt : 0;
  if (role_split) *role_split = c.split2 == 1 ? 0 : (c.split2 == 2 ? 2 : 1);
  return CP4_OK;
}

cp4_status cp4_plan_query(const cp4_shape* shape, int pass, int* variant, int* strip_rows,
                          int* workgroups) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (pass < 0 || pass > 2) return fail(CP4_ERR_SHAPE, "pass must be 0, 1 or 2");
  int v = -1, rows = 0, wgs = 0;
  if (pass == 2) {
    // the choice for operands aligned as every allocator returns them
    v = default_filter_variant(*shape, filter_routes(*shape, true, true, true));
    if (v == 0 && filter_pad_route(*shape)) {   // runs on copies with zero channels appended
      const cp4_shape t = filter_padded_shape(*shape);
      v = default_filter_variant(t, filter_routes(t, true, true, true));
    }
  } else {
    FwdArgs a = pass == 1
        ? backward_data_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr)
        : forward_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
    const Choice c = choose(a);
    v = c.variant;
    if (is_variant(v, "mfma_bf16x3_pipe")) {
      a.tune_th = c.th;
      if (!cp4::fwd_pipe_strip_plan(a, &rows, &wgs)) rows = wgs = 0;
    }
    if (is_variant(v, "mfma_bf16x3_pipe64")) {
      a.tune_th = c.th;
      if (!cp4::fwd_pipe64_plan(a, &rows, &wgs)) rows = wgs = 0;
    }
    if (is_variant(v, "mfma_bf16x3_few")) {       // (tile rows; its persistent workgroups)
      int cols = 0;
      a.tune_th = c.th;
      a.tune_lgwt = c.lgwt;
      a.tune_split2 = c.split2;
      if (!cp4::fwd_few_plan(a, &rows, &cols, &wgs)) rows = wgs = 0;
    }
  }
  if (variant) *variant = v;
  if (strip_rows) *strip_rows = rows;
  if (workgroups) *workgroups = wgs;
  return CP4_OK;
}

cp4_status cp4_set_tuned_choice(const cp4_shape* shape, int backward_data, int variant,
                                int tile_rows, int tile_cols, int schedule) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (variant < 0 || variant >= kNumVariants) return fail(CP4_ERR_SHAPE, "variant out of range");
  int lgwt = 0;
  if (tile_cols) {
    while ((1 << lgwt) < tile_cols) ++lgwt;
    if ((1 << lgwt) != tile_cols || lgwt < 5 || lgwt > 8)
      return fail(CP4_ERR_SHAPE, "tile_cols must be 0, 32, 64, 128 or 256");
  }
  if (tile_rows < 0 || schedule < 0 || schedule > 2)
    return fail(CP4_ERR_SHAPE, "tile_rows >= 0 and schedule 0, 1 or 2 expected");
  const FwdArgs a =
      backward_data
          ? backward_data_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr)
          : forward_args(*shape, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr);
  // (schedule as cp4_tuned_choice reports it: 1 the kernel's rule, 0 no role split, 2 whole groups)
  const Choice c{variant, tile_rows, lgwt, schedule == 1 ? 0 : (schedule == 0 ? 1 : 2)};
  if (!kVariants[variant].supported(with_tile(a, c)))
    return fail(CP4_ERR_UNSUPPORTED, "the variant does not take this shape with this tile");
  std::lock_guard<std::mutex> lk(g_tune_mu);
  g_tuned[key_of(a)] = c;
  return CP4_OK;
}

int cp4_tuned_count(void) {
  std::lock_guard<std::mutex> lk(g_tune_mu);
  return (int)g_tuned.size();
}

cp4_status cp4_tuned_entry(int index, cp4_shape* shape, int* backward_data, int* variant,
                           int* tile_rows, int* tile_cols, int* schedule) {
  if (!shape) return fail(CP4_ERR_NULL_POINTER, "shape is NULL");
  std::lock_guard<std::mutex> lk(g_tune_mu);
  if (index < 0 || index >= (int)g_tuned.size()) return fail(CP4_ERR_SHAPE, "index out of range");
  auto it = g_tuned.begin();
  std::advance(it, index);
  const TuneKey& k = it->first;                    // N, Cin, Cout, H, W, pad, Y, X, R, flip
  const bool bwd = std::get<9>(k) == 1;
  shape->N = (unsigned)std::get<0>(k);
  shape->C = (unsigned)(bwd ? std::get<2>(k) : std::get<1>(k));
  shape->T = (unsigned)(bwd ? std::get<1>(k) : std::get<2>(k));
  shape->H = (unsigned)std::get<3>(k);
  shape->W = (unsigned)std::get<4>(k);
  shape->pad = (unsigned)std::get<5>(k);
  shape->Y = (unsigned)std::get<6>(k);
  shape->X = (unsigned)std::get<7>(k);
  shape->Rank = (unsigned)std::get<8>(k);
  const Choice& c = it->second;
  if (backward_data) *backward_data = bwd ? 1 : 0;
  if (variant) *variant = c.variant;
  if (tile_rows) *tile_rows = c.th;
  if (tile_cols) *tile_cols = c.lgwt ? 1 << c.lgwt : 0;
  if (schedule) *schedule = c.split2 == 1 ? 0 : (c.split2 == 2 ? 2 : 1);
  return CP4_OK;
}

const char* cp4_backward_filter_variant_name(int variant) {
  static const char* const names[4] = {"general_valu", "mfma_four_launches", "mfma_fused_taps",
                                       "dense_gradient_tiles"};
  return variant >= 0 && variant < 4 ? names[variant] : nullptr;
}

int cp4_tuned_filter_count(void) {
  std::lock_guard<std::mutex> lk(g_tune_mu);
  return (int)g_tuned_filter.size();
}

cp4_status cp4_tuned_filter_entry(int index, cp4_shape* shape, int* variant) {
  if (!shape) return fail(CP4_ERR_NULL_POINTER, "shape is NULL");
  std::lock_guard<std::mutex> lk(g_tune_mu);
  if (index < 0 || index >= (int)g_tuned_filter.size())
    return fail(CP4_ERR_SHAPE, "index out of range");
  auto it = g_tuned_filter.begin();
  std::advance(it, index);
  const TuneKey& k = it->first;                    // N, C, T, H, W, pad, Y, X, Rank, 2
  shape->N = (unsigned)std::get<0>(k);
  shape->C = (unsigned)std::get<1>(k);
  shape->T = (unsigned)std::get<2>(k);
  shape->H = (unsigned)std::get<3>(k);
  shape->W = (unsigned)std::get<4>(k);
  shape->pad = (unsigned)std::get<5>(k);
  shape->Y = (unsigned)std::get<6>(k);
  shape->X = (unsigned)std::get<7>(k);
  shape->Rank = (unsigned)std::get<8>(k);
  if (variant) *variant = it->second;
  return CP4_OK;
}

cp4_status cp4_set_tuned_filter_choice(const cp4_shape* shape, int variant) {
  cp4_status rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (variant < 0 || variant > 3)
    return fail(CP4_ERR_UNSUPPORTED, "backward-filter variants are numbered 0 to 3");
  // (a choice the shape or the caller's alignment does not allow is ignored at launch)
  std::lock_guard<std::mutex> lk(g_tune_mu);
  g_tuned_filter[key_of(*shape)] = variant;
  return CP4_OK;
}

void cp4_tune_clear(void) {
  std::lock_guard<std::mutex> lk(g_tune_mu);
  g_tuned.clear();
  g_tuned_filter.clear();
  g_heuristic_picks.clear();
}

cp4_status cp4_device_status(cp4_stream stream, int* detail) {
  return device_status(as_stream(stream), detail);
}

void cp4_set_spin_limit(int polls) { g_spin_limit.store(polls > 0 ? polls : 0); }

void cp4_set_backward_filter_tile_kernel(int which) {
  cp4::bwd_filter_dense_tiles_force_kernel(which);
}

cp4_status cp4_set_device(int ordinal) {
  CP4_HIP(hipSetDevice(ordinal));
  return CP4_OK;
}
cp4_status cp4_device_malloc(void** ptr, size_t bytes) {
  if (!ptr) return fail(CP4_ERR_NULL_POINTER, "ptr is NULL");
  *ptr = nullptr;
  if (bytes == 0) return CP4_OK;
  CP4_HIP(hipMalloc(ptr, bytes));
  return CP4_OK;
}
cp4_status cp4_device_free(void* ptr) {
  if (ptr) CP4_HIP(hipFree(ptr));
  return CP4_OK;
}
cp4_status cp4_host_malloc(void** ptr, size_t bytes) {
  if (!ptr) return fail(CP4_ERR_NULL_POINTER, "ptr is NULL");
  *ptr = nullptr;
  if (bytes == 0) return CP4_OK;
  CP4_HIP(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return CP4_OK;
}
cp4_status cp4_host_free(void* ptr) {
  if (ptr) CP4_HIP(hipHostFree(ptr));
  return CP4_OK;
}
cp4_status cp4_memcpy_h2d(void* dst, const void* src, size_t bytes, cp4_stream s) {
  if (bytes == 0) return CP4_OK;
  if (!dst || !src) return fail(CP4_ERR_NULL_POINTER, "memcpy pointer is NULL");
  CP4_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(s)));
  return CP4_OK;
}
cp4_status cp4_memcpy_d2h(void* dst, const void* src, size_t bytes, cp4_stream s) {
  if (bytes == 0) return CP4_OK;
  if (!dst || !src) return fail(CP4_ERR_NULL_POINTER, "memcpy pointer is NULL");
  CP4_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(s)));
  return CP4_OK;
}
cp4_status cp4_memcpy_d2d(void* dst, const void* src, size_t bytes, cp4_stream s) {
  if (bytes == 0) return CP4_OK;
  if (!dst || !src) return fail(CP4_ERR_NULL_POINTER, "memcpy pointer is NULL");
  CP4_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(s)));
  return CP4_OK;
}
cp4_status cp4_memset_zero(void* dst, size_t bytes, cp4_stream s) {
  if (bytes == 0) return CP4_OK;
  if (!dst) return fail(CP4_ERR_NULL_POINTER, "memset pointer is NULL");
  CP4_HIP(hipMemsetAsync(dst, 0, bytes, as_stream(s)));
  return CP4_OK;
}
cp4_status cp4_pointer_is_device(const void* ptr, int* is_device) {
  if (!is_device) return fail(CP4_ERR_NULL_POINTER, "is_device is NULL");
  *is_device = 0;
  if (!ptr) return CP4_OK;
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // plain host memory the runtime has never seen
    return CP4_OK;
  }
  *is_device = attr.type == hipMemoryTypeDevice ? 1 : 0;
  return CP4_OK;
}
cp4_status cp4_stream_synchronize(cp4_stream s) {
  CP4_HIP(hipStreamSynchronize(as_stream(s)));
  return CP4_OK;
}
cp4_status cp4_device_synchronize(void) {
  CP4_HIP(hipDeviceSynchronize());
  return CP4_OK;
}

cp4_status cp4_recompose(const cp4_shape* shape, const float* FK,
                         const float* FC, const float* FH, const float* FW,
                         float* K, cp4_stream stream) {
  if (!shape) return fail(CP4_ERR_NULL_POINTER, "shape is NULL");
  if (!shape->T || !shape->C || !shape->Y || !shape->X || !shape->Rank)
    return fail(CP4_ERR_SHAPE, "T, C, Y, X and Rank must be >= 1");
  if (!FK || !FC || !FH || !FW || !K)
    return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  CP4_HIP(cp4::recompose_launch(*shape, FK, FC, FH, FW, K, as_stream(stream)));
  return CP4_OK;
}

// ---- 3-factor CP sibling op ---------------------------------------------------

namespace {
size_t cp3_align(size_t floats) { return (floats + 63) & ~(size_t)63; }   // 256-byte slices

cp4_status cp3_check(const cp4_shape* s) {
  if (!s) return fail(CP4_ERR_NULL_POINTER, "shape is NULL");
  if (!s->T || !s->C || !s->Y || !s->X || !s->Rank)
    return fail(CP4_ERR_SHAPE, "T, C, Y, X and Rank must be >= 1");
  if ((unsigned long long)s->Y * s->Rank > 65535ull)
    return fail(CP4_ERR_SHAPE, "Y * Rank must be <= 65535");
  return CP4_OK;
}
}  // namespace

cp4_status cp3_expand_factors(const cp4_shape* shape, const float* K0, const float* K1,
                              const float* K2, float* FK, float* FC, float* FH, float* FW,
                              cp4_stream stream) {
  cp4_status rc = cp3_check(shape);
  if (rc != CP4_OK) return rc;
  if (!K0 || !K1 || !K2 || !FK || !FC || !FH || !FW)
    return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  CP4_HIP(cp4::cp3_expand_launch(*shape, K0, K1, K2, FK, FC, FH, FW, as_stream(stream)));
  return CP4_OK;
}

cp4_status cp3_fold_gradients(const cp4_shape* shape, const float* dFK, const float* dFC,
                              const float* dFW, float* dK0, float* dK1, float* dK2,
                              cp4_stream stream) {
  cp4_status rc = cp3_check(shape);
  if (rc != CP4_OK) return rc;
  if (!dFK || !dFC || !dFW || !dK0 || !dK1 || !dK2)
    return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  CP4_HIP(cp4::cp3_fold_launch(*shape, dFK, dFC, dFW, dK0, dK1, dK2, as_stream(stream)));
  return CP4_OK;
}

size_t cp3_conv2d_forward_workspace_bytes(const cp4_shape* s) {
  if (!s) return 0;
  const size_t Q = (size_t)s->Y * s->Rank;
  return sizeof(float) * (cp3_align(s->T * Q) + cp3_align(s->C * Q) + cp3_align(s->Y * Q) +
                          cp3_align(s->X * Q));
}

namespace {
// The pass on the producer / consumer kernel's 2-D-tap build when that kernel is
// the right one for the shape (whole-row strips that fit, enough channels to
// fill its tiles, at most 256 input channels on large problems), else on the
// expanded CP4 factors through the usual choice of variants.
cp4_status cp3_run(const cp4_shape* shape, const float* in, const float* K0, const float* K1,
                   const float* K2, float* out, void* workspace, size_t workspace_bytes,
                   bool backward, cp4_stream stream) {
  cp4_status rc = cp3_check(shape);
  if (rc != CP4_OK) return rc;
  rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  if (!in || !K0 || !K1 || !K2 || !out)
    return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  if (!workspace || workspace_bytes < cp3_conv2d_forward_workspace_bytes(shape))
    return fail(CP4_ERR_WORKSPACE, "workspace missing or smaller than "
                                   "cp3_conv2d_forward_workspace_bytes(shape)");
  hipStream_t st = as_stream(stream);
  const size_t Q = (size_t)shape->Y * shape->Rank;
  float* FK = static_cast<float*>(workspace);

  // K2 [R,T] as an out-channel factor [T,R]; K0 is an in-channel factor as it is
  FwdArgs a = backward ? backward_data_args(*shape, in, FK, K0, nullptr, nullptr, out)
                       : forward_args(*shape, in, FK, K0, nullptr, nullptr, out);
  a.taps2d = K1;
  CP4_ARM(a);
  const size_t pixels = (size_t)a.N * a.H * a.W;
  if (cp4::fwd_pipe_taps2d_supported(a) && a.W <= 128 && a.Cin + a.Cout >= 24 &&
      !(a.Cin > 256 && pixels > 8192)) {
    CP4_HIP(cp4::transpose_f32_launch(K2, FK, (int)shape->Rank, (int)shape->T, st));
    CP4_HIP(cp4::fwd_pipe_taps2d_launch(a, st));
    return CP4_OK;
  }
  // more than 32 ranks (or 768 input channels): the same build in passes with y +=, R ranks
  // in tiles of 32 instead of Y * R expanded ones (N32 C256 K256 56x56 3x3 R48: two passes
  // against five)
  auto tap_pass = [&](int slice, int tile) {
    FwdArgs b = pass_args(a, slice, tile);
    b.FH = b.FW = nullptr;
    b.taps2d = a.taps2d + 32 * tile;
    return b;
  };
  if ((a.R > 32 || a.Cin > kPassMaxChannels) && a.W <= 128 && a.Cin + a.Cout >= 24 &&
      rank_passes(a) * channel_slices(a) <= kMaxPasses &&
      cp4::fwd_pipe_taps2d_supported(tap_pass(0, 0)) &&
      cp4::fwd_pipe_taps2d_supported(tap_pass(channel_slices(a) - 1, rank_passes(a) - 1))) {
    CP4_HIP(cp4::transpose_f32_launch(K2, FK, (int)shape->Rank, (int)shape->T, st));
    for (int t = 0; t < rank_passes(a); ++t)
      for (int c = 0; c < channel_slices(a); ++c)
        CP4_HIP(cp4::fwd_pipe_taps2d_launch(tap_pass(c, t), st));
    return CP4_OK;
  }

  float* FC = FK + cp3_align(shape->T * Q);
  float* FH = FC + cp3_align(shape->C * Q);
  float* FW = FH + cp3_align(shape->Y * Q);
  rc = cp3_expand_factors(shape, K0, K1, K2, FK, FC, FH, FW, stream);
  if (rc != CP4_OK) return rc;
  cp4_shape wide = *shape;
  wide.Rank = (unsigned)Q;
  return backward ? cp4_conv2d_backward_data(&wide, in, FK, FC, FH, FW, out, stream)
                  : cp4_conv2d_forward(&wide, in, FK, FC, FH, FW, out, stream);
}
}  // namespace

cp4_status cp3_conv2d_forward(const cp4_shape* shape, const float* x, const float* K0,
                              const float* K1, const float* K2, float* y, void* workspace,
                              size_t workspace_bytes, cp4_stream stream) {
  return cp3_run(shape, x, K0, K1, K2, y, workspace, workspace_bytes, false, stream);
}

cp4_status cp3_conv2d_backward_data(const cp4_shape* shape, const float* dy, const float* K0,
                                    const float* K1, const float* K2, float* dx,
                                    void* workspace, size_t workspace_bytes,
                                    cp4_stream stream) {
  return cp3_run(shape, dy, K0, K1, K2, dx, workspace, workspace_bytes, true, stream);
}

namespace {
// workspace of cp3_conv2d_backward_filter: [FK^T | dFK | inner] on the direct path,
// [expanded factors | their gradients | inner] on the rewriting
struct Cp3FilterLayout {
  bool direct;
  size_t fk, dfk, inner_off, inner_bytes, total;      // bytes
  cp4_shape wide;                                      // rank Y*R shape of the rewriting
};
Cp3FilterLayout cp3_filter_layout(const cp4_shape& s) {
  Cp3FilterLayout l{};
  // Up to 32 expanded ranks the rewriting is one pass of 32-rank tiles with the
  // fast separable tap kernels and wins (N32 C64 56x56 R10: 65 against 89 us); above,
  // Y times fewer planes win (N32 C256 56x56 R16: 137 against 168 us).
  l.direct = cp4::bwd_filter_mfma_taps2d_supported(s) && (size_t)s.Y * s.Rank > 32;
  l.wide = s;
  l.wide.Rank = s.Y * s.Rank;
  if (l.direct) {
    l.fk = 0;
    l.dfk = align256((size_t)s.T * s.Rank * sizeof(float));
    l.inner_off = 2 * l.dfk;
    l.inner_bytes = cp4::bwd_filter_mfma_workspace_bytes(s);
  } else {
    const size_t Q = l.wide.Rank;
    const size_t fac = sizeof(float) * (cp3_align(s.T * Q) + cp3_align(s.C * Q) +
                                        cp3_align(s.Y * Q) + cp3_align(s.X * Q));
    l.fk = 0;
    l.dfk = fac;
    l.inner_off = 2 * fac;
    l.inner_bytes = filter_workspace(l.wide);
  }
  l.total = l.inner_off + align256(l.inner_bytes);
  return l;
}
}  // namespace

size_t cp3_conv2d_backward_filter_workspace_bytes(const cp4_shape* s) {
  if (cp3_check(s) != CP4_OK || check_shape(s) != CP4_OK || s->N == 0) return 0;
  return cp3_filter_layout(*s).total;
}

cp4_status cp3_conv2d_backward_filter(const cp4_shape* shape, const float* x, const float* dy,
                                      const float* K0, const float* K1, const float* K2,
                                      float* dK0, float* dK1, float* dK2, void* workspace,
                                      size_t workspace_bytes, cp4_stream stream) {
  cp4_status rc = cp3_check(shape);
  if (rc != CP4_OK) return rc;
  rc = check_shape(shape);
  if (rc != CP4_OK) return rc;
  if (!K0 || !K1 || !K2 || !dK0 || !dK1 || !dK2)
    return fail(CP4_ERR_NULL_POINTER, "a factor or gradient pointer is NULL");
  const cp4_shape& s = *shape;
  hipStream_t st = as_stream(stream);
  if (s.N == 0) {
    CP4_HIP(cp4::zero_f32_launch(dK0, (size_t)s.C * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dK1, (size_t)s.Y * s.X * s.Rank, st));
    CP4_HIP(cp4::zero_f32_launch(dK2, (size_t)s.Rank * s.T, st));
    return CP4_OK;
  }
  if (!x || !dy) return fail(CP4_ERR_NULL_POINTER, "x or dy is NULL");
  const Cp3FilterLayout l = cp3_filter_layout(s);
  if (!workspace || workspace_bytes < l.total)
    return fail(CP4_ERR_WORKSPACE, "workspace smaller than cp3_conv2d_backward_filter_workspace_bytes");
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
    return fail(CP4_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  unsigned char* w = static_cast<unsigned char*>(workspace);
  const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(dy)) & 7) == 0;
  if (l.direct && aligned) {
    float* FK = reinterpret_cast<float*>(w + l.fk);
    float* dFK = reinterpret_cast<float*>(w + l.dfk);
    CP4_HIP(cp4::transpose_f32_launch(K2, FK, (int)s.Rank, (int)s.T, st));     // [R,T] -> [T,R]
    cp4::BwdFilterArgs a{};
    a.x = x; a.dy = dy; a.FK = FK; a.FC = K0; a.taps2d = K1;
    a.dFK = dFK; a.dFC = dK0; a.dtaps2d = dK1;
    a.workspace = w + l.inner_off;
    a.N = s.N; a.C = s.C; a.T = s.T; a.H = s.H; a.W = s.W; a.pad = s.pad;
    a.Y = s.Y; a.X = s.X; a.R = s.Rank;
    CP4_HIP(cp4::bwd_filter_mfma_launch(a, st));
    CP4_HIP(cp4::transpose_f32_launch(dFK, dK2, (int)s.T, (int)s.Rank, st));   // [T,R] -> [R,T]
    return CP4_OK;
  }
  // the rewriting as a CP4 of rank Y*R
  const size_t Q = l.wide.Rank;
  float* FK = reinterpret_cast<float*>(w + l.fk);
  float* FC = FK + cp3_align(s.T * Q);
  float* FH = FC + cp3_align(s.C * Q);
  float* FW = FH + cp3_align(s.Y * Q);
  float* dFK = reinterpret_cast<float*>(w + l.dfk);
  float* dFC = dFK + cp3_align(s.T * Q);
  float* dFH = dFC + cp3_align(s.C * Q);
  float* dFW = dFH + cp3_align(s.Y * Q);
  rc = cp3_expand_factors(shape, K0, K1, K2, FK, FC, FH, FW, stream);
  if (rc != CP4_OK) return rc;
  rc = cp4_conv2d_backward_filter(&l.wide, x, dy, FK, FC, FH, FW, dFK, dFC, dFH, dFW,
                                  w + l.inner_off, workspace_bytes - l.inner_off, stream);
  if (rc != CP4_OK) return rc;
  return cp3_fold_gradients(shape, dFK, dFC, dFW, dK0, dK1, dK2, stream);
}

// ---- reshaped-CP sibling op ------------------------------------------------------

namespace {
cp4_status rcp_check(const cp4_shape* s, const rcp_dims* d) {
  cp4_status rc = check_shape(s);
  if (rc != CP4_OK) return rc;
  if (!d) return fail(CP4_ERR_NULL_POINTER, "dims is NULL");
  if (!d->S0 || !d->S1 || !d->T0 || !d->T1 ||
      (unsigned long long)d->S0 * d->S1 != s->C || (unsigned long long)d->T0 * d->T1 != s->T)
    return fail(CP4_ERR_SHAPE, "S0*S1 must equal C and T0*T1 must equal T");
  return CP4_OK;
}
size_t rcp_filter_floats(const cp4_shape& s) { return (size_t)s.T * s.C * s.Y * s.X; }

// One dense pass of the op on the recomposed filter in `K`.
cp4_status rcp_dense_pass(const cp4_shape& s, const float* in, float* out, const float* K,
                          bool backward, hipStream_t st) {
  FwdArgs a{};
  a.x = in; a.y = out; a.dense = K;
  a.N = s.N; a.Cin = backward ? s.T : s.C; a.Cout = backward ? s.C : s.T;
  a.H = s.H; a.W = s.W; a.pad = s.pad; a.Y = s.Y; a.X = s.X; a.R = s.Rank;
  if (!cp4::fwd_dense_small_supported(a))
    return fail(CP4_ERR_UNSUPPORTED,
                "reshaped-CP op: square odd filters up to 17x17 with pad <= Y-1");
  CP4_HIP(cp4::fwd_dense_small_launch(a, st));
  return CP4_OK;
}
}  // namespace

size_t rcp_conv2d_workspace_bytes(const cp4_shape* s, const rcp_dims* d) {
  if (rcp_check(s, d) != CP4_OK) return 0;
  return 2 * align256(rcp_filter_floats(*s) * sizeof(float));
}

cp4_status rcp_conv2d_forward(const cp4_shape* shape, const rcp_dims* d, const float* x,
                              const float* K0, const float* K1, const float* KC, float* y,
                              void* workspace, size_t workspace_bytes, cp4_stream stream) {
  cp4_status rc = rcp_check(shape, d);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  if (!x || !K0 || !K1 || !KC || !y) return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  if (!workspace || workspace_bytes < rcp_conv2d_workspace_bytes(shape, d))
    return fail(CP4_ERR_WORKSPACE, "workspace smaller than rcp_conv2d_workspace_bytes");
  hipStream_t st = as_stream(stream);
  float* K = static_cast<float*>(workspace);
  CP4_HIP(cp4::rcp_recompose_launch(K0, K1, KC, K, d->S0, d->S1, d->T0, d->T1, shape->Y, shape->X,
                                    shape->Rank, 0, st));
  return rcp_dense_pass(*shape, x, y, K, false, st);
}

cp4_status rcp_conv2d_backward_data(const cp4_shape* shape, const rcp_dims* d, const float* dy,
                                    const float* K0, const float* K1, const float* KC, float* dx,
                                    void* workspace, size_t workspace_bytes, cp4_stream stream) {
  cp4_status rc = rcp_check(shape, d);
  if (rc != CP4_OK) return rc;
  if (shape->N == 0) return CP4_OK;
  if (!dy || !K0 || !K1 || !KC || !dx) return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  if (!workspace || workspace_bytes < rcp_conv2d_workspace_bytes(shape, d))
    return fail(CP4_ERR_WORKSPACE, "workspace smaller than rcp_conv2d_workspace_bytes");
  hipStream_t st = as_stream(stream);
  float* K = static_cast<float*>(workspace);
  CP4_HIP(cp4::rcp_recompose_launch(K0, K1, KC, K, d->S0, d->S1, d->T0, d->T1, shape->Y, shape->X,
                                    shape->Rank, 1, st));
  return rcp_dense_pass(*shape, dy, dx, K, true, st);
}

cp4_status rcp_conv2d_backward_filter(const cp4_shape* shape, const rcp_dims* d, const float* x,
                                      const float* dy, const float* K0, const float* K1,
                                      const float* KC, float* dK0, float* dK1, float* dKC,
                                      void* workspace, size_t workspace_bytes,
                                      cp4_stream stream) {
  cp4_status rc = rcp_check(shape, d);
  if (rc != CP4_OK) return rc;
  if (!K0 || !K1 || !KC || !dK0 || !dK1 || !dKC)
    return fail(CP4_ERR_NULL_POINTER, "a factor or gradient pointer is NULL");
  if (!workspace || workspace_bytes < rcp_conv2d_workspace_bytes(shape, d))
    return fail(CP4_ERR_WORKSPACE, "workspace smaller than rcp_conv2d_workspace_bytes");
  hipStream_t st = as_stream(stream);
  // dense filter gradient (cp4Conv2dBackwardFilter.cu:23-59), then the chain rule
  float* dK = static_cast<float*>(workspace) + align256(rcp_filter_floats(*shape) * sizeof(float)) / sizeof(float);
  rc = cp4_conv2d_backward_filter_full(shape, x, dy, dK, 0, stream);
  if (rc != CP4_OK) return rc;
  CP4_HIP(cp4::rcp_fold_launch(dK, K0, K1, KC, dK0, dK1, dKC, d->S0, d->S1, d->T0, d->T1, shape->Y,
                               shape->X, shape->Rank, st));
  return CP4_OK;
}

cp4_status cp4_count_exceeding(const float* A, const float* B, size_t n,
                               float tol, long long* count, cp4_stream stream) {
  if (!count) return fail(CP4_ERR_NULL_POINTER, "count is NULL");
  *count = 0;
  if (n == 0) return CP4_OK;
  if (!A || !B) return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  hipStream_t st = as_stream(stream);
  unsigned long long* d = nullptr;
  CP4_HIP(hipMalloc(&d, sizeof(*d)));
  unsigned long long h = 0;
  hipError_t e = hipMemsetAsync(d, 0, sizeof(*d), st);
  if (e == hipSuccess) e = cp4::count_exceeding_launch(A, B, n, tol, d, st);
  if (e == hipSuccess) e = hipMemcpyAsync(&h, d, sizeof(h), hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  (void)hipFree(d);
  if (e != hipSuccess) return hip_fail(e, "cp4_count_exceeding");
  *count = (long long)h;
  return CP4_OK;
}

cp4_status cp4_random_uniform(float* dst, size_t n, unsigned long long seed,
                              cp4_stream stream) {
  if (n == 0) return CP4_OK;
  if (!dst) return fail(CP4_ERR_NULL_POINTER, "dst is NULL");
  CP4_HIP(cp4::random_uniform_launch(dst, n, seed, as_stream(stream)));
  return CP4_OK;
}

cp4_status cp4_copy_f32(float* dst, const float* src, size_t n, cp4_stream stream) {
  if (n == 0) return CP4_OK;
  if (!dst || !src) return fail(CP4_ERR_NULL_POINTER, "a data pointer is NULL");
  CP4_HIP(cp4::copy_f32_launch(dst, src, n, as_stream(stream)));
  return CP4_OK;
}

cp4_status cp4_time_copy_f32(float* dst, const float* src, size_t n,
                             unsigned warmup, unsigned profcount,
                             float* mean_us, cp4_stream stream) {
  return time_loop([&] { return cp4_copy_f32(dst, src, n, stream); }, warmup,
                   profcount, mean_us, as_stream(stream));
}

}  // extern "C"
