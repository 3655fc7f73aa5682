// Fused forward / backward-data kernel, producer / consumer form of the
// split-precision strip kernel (ranks up to 32).
//
// Arithmetic and fragments are those of fwd_mfma_split.hip: every fp32 operand
// is split exactly into three bf16 parts and a product is six bf16 MFMAs
// accumulated in fp32 (fp32-equivalent accuracy).  What changes is the
// schedule.  With one strip of TH rows per workgroup the output contraction of
// a pixel cannot start before the channel contraction of its whole 3x3
// neighbourhood is done, so a phase-by-phase kernel reads x, then writes y, and
// HBM never sees both directions at once.  Here the 16 waves take roles:
//
//   waves 0-7  producers: the strip (+ halo rows) is swept in rounds of two
//              32-pixel blocks; in a round wave w works on block (w & 1) of the
//              pair for channel quarter w >> 1 (its slice of the input factor,
//              pre-split, sits in registers up to 256 input channels and in
//              LDS above): it streams x (ring of KR
//              16-channel chunks in flight, refilled across round boundaries),
//              splits, runs the MFMAs and adds its partial fp32 A[r][q] into
//              LDS.  The four quarters of a block add in fixed order (an LDS
//              word per block counts the quarters done), so the sum is
//              deterministic; the word reaching 4 publishes the block.
//   waves 8-15 consumers: for each group of 64 output pixels, in sweep order,
//              wait until the producers have finished every block the group's
//              taps touch, apply the taps (one wave per rank quad, lane =
//              pixel), split the result into MFMA B fragments in one of three
//              rotating LDS tiles and signal an LDS arrival counter; then run
//              the rank -> output-channel MFMAs for their 32-channel block of
//              the previous group and store y (float2 per lane).
//
// Reads of later blocks therefore overlap the writes of earlier groups.  Odd
// strips sweep bottom-up, even strips top-down: neighbouring strips then read
// the halo rows they share at about the same time and the second reader finds
// them in L2 instead of fetching them from HBM again.
// All waits are on LDS words written by waves of the same workgroup, which are
// co-resident by construction: a producer waits only for the lower channel
// quarters of its own block, consumers wait for producers and for each other's
// arrivals, nothing waits for a consumer's stores, so every wait is eventually
// satisfied.  The spins are bounded all the same.
// Arithmetic follows the reassociated form of
// Cuda_kernels/cp4Conv2dForward.cu:84-133 (backward-data:
// cp4Conv2dBackwardData.cu:57-108 through swapped factors and flipped taps).
//
// This file is compiled ten times: as is; with CP4_PIPE_EPILOGUE defined, which
// adds y = act(conv + bias[k]) to the stores (the bias, padded to whole channel
// blocks, waits in LDS and is what the accumulators start from) and exports
// the entry points under the names fwd_pipe_epi_*; and with CP4_PIPE_IO16, where
// x and y are bfloat16 in memory (factors, bias and all arithmetic stay fp32):
// a bf16 activation is its own high part, so the channel contraction needs
// neither the split nor the three MFMAs of the lower parts, and y is rounded to
// nearest-even as pixel pairs (entry points fwd_pipe_io16_*, epilogue included;
// CP4_PIPE_IO16=2: IEEE half precision instead - a half is two bfloat16 parts, five
// MFMAs per chunk - entry points fwd_pipe_iof16_*);
// and with CP4_PIPE_RANKPASS, the build behind the two-pass variant for ranks
// 33-64: factor matrices with a row stride of their own (FwdArgs::ldf) and stores
// that add to y (FwdArgs::accumulate), entry points fwd_pipe_rankpass_*;
// and with CP4_PIPE_TILED, for wide planes: a workgroup's tile is TH rows by Wt
// columns (Wt a power of two, at least 64) instead of TH whole rows; the LDS
// plane holds the tile plus its halo in rows of Wt + FS - 1 cells, so the taps
// need no border masks (cells outside the image are stored as zeros) and every
// 64-pixel output group is one row segment; entry points fwd_pipe_tiled_*;
// and with CP4_PIPE_TAPS2D, for the 3-factor CP sibling op: the tap step weighs
// the Y x X cells it reads with a depthwise filter FwdArgs::taps2d [Y, X, R]
// instead of the outer product FH x FW (1x1 and 3x3 filters: 36 wave-uniform
// weights per wave), entry points fwd_pipe_taps2d_*;
// and with CP4_PIPE_STRIDED, for layers with a stride or an output plane that is
// not the input's (FwdArgs::sh ...): a strip is TH rows of the OUTPUT, its LDS
// plane the sh*(TH-1) + Y input rows under them; the tap step of output pixel
// (ho, wo) reads the plane at row sh*ho, column sw*wo - pl, so only the kept
// outputs are filtered, contracted and stored; entry points fwd_pipe_strided_*.
#include <cstdlib>
#include <type_traits>

#include "cp4_internal.h"
#include "split_bf16.h"
#include "pipe_wait.h"
#ifdef CP4_DEBUG_PHASES
#include "cp4_debug.h"
#endif

#ifdef CP4_PIPE_IO16
#define CP4_PIPE_EPILOGUE 1
#endif

// Passes over rank tiles and channel slices (FwdArgs::ldf, ldx, accumulate): the rank-pass
// build, the strided build and the 2-D-tap build honour them.
#if defined(CP4_PIPE_RANKPASS) || defined(CP4_PIPE_STRIDED) || defined(CP4_PIPE_TAPS2D)
#define CP4_PIPE_PASSES 1
#endif

namespace cp4 {
namespace {

#ifdef CP4_PIPE_IO16
using io_t = unsigned short;     // bfloat16 bits (CP4_PIPE_IO16 == 2: IEEE half bits)
__device__ __forceinline__ unsigned short to_io(float v) {
#if CP4_PIPE_IO16 == 2
  return __builtin_bit_cast(unsigned short, static_cast<_Float16>(v));   // round to nearest even
#else
  return __builtin_bit_cast(unsigned short, static_cast<__bf16>(v));   // round to nearest even
#endif
}
#else
using io_t = float;
#endif
constexpr int kIoBytes = (int)sizeof(io_t);

using namespace split;

constexpr int kThreads = 1024;
constexpr int kProd = 8, kCons = 8;          // producer / consumer waves (4 per SIMD in all)
constexpr int kRP = 32;
constexpr int kCcBuf = 24 * 512;             // bytes of one Cc fragment tile (64 pixels)
constexpr size_t kLdsLimit = 160 * 1024;
[[maybe_unused]] constexpr int kOwnGroupsMaxRank = 4;         // ranks up to which consumer waves take whole groups by default
#ifndef CP4_WHOLE_BLOCK_MIN
#define CP4_WHOLE_BLOCK_MIN 16
#endif
// What a workgroup spends before its pipeline runs (first loads, factor
// fragments, the consumers' wait for the first rows: 7-8 us), in the planners'
// unit of one channel of one cell read or written (7-11 thousand per us).
constexpr double kTileStartCost = 50000.0;
// C3 (56-pixel rows): 7-row strips, 256 workgroups, 39.6 us on one buffer set and
// 61.6 us on rotating sets; 8-row strips, 224 workgroups, 38.1 and 56.0 us.
[[maybe_unused]] constexpr double kUnalignedStripCost = 1.12;
constexpr int kWholeBlockMin = CP4_WHOLE_BLOCK_MIN;   // blocks per plane from which 17-64 channels go unsplit
constexpr int kSpinLimit = 1 << 19;      // default bound of a wait: about a quarter of a second at the longest nap
constexpr int kMaxBlk = 64;                  // per-block progress words in LDS

struct PipePlan {
  int TH, strips, nWG;
  int nblk;        // 32-pixel producer blocks of a workgroup's plane
  int QA;          // cells (of four ranks each) per rank quad of the A plane in LDS
  int fin_off;     // byte offsets inside LDS; factor fragments only above 256 input channels
  int cc_off;
  int flag_off;
  size_t lds_bytes;
  int Wt, lgWt, cols;       // tiled build: tile width, its log2, column tiles per row strip
  unsigned wl_magic;        // tiled build: 2^32 / (Wt + FS - 1) + 1, for the division by the row length
  int split2;               // consumer waves split roles also above 16 ranks / 4 channel blocks
  int own;                  // consumer waves take whole groups each (few ranks and channel blocks)
  int spin_limit;           // polls before a wait between waves gives up
  // Few strips (one image, small planes) leave compute units idle: the output channels are
  // then cut into kparts slices of kslice channels (a multiple of 32), one workgroup per
  // (strip, slice) - blockIdx.y is the slice; every slice's workgroup contracts the strip's
  // A plane again and writes its own channels.  1: no slices.
  int kparts = 1, kslice = 0;
#ifdef CP4_DEBUG_PHASES
  long long* dbg;
#endif
};

// NQ: channel splits of the producers (4: quarters, two blocks per round; 1: up to
// 16 input channels, every producer wave takes a whole block of its own, eight
// blocks per round and no partial sums to chain).
// PAIR (16-bit activations, even row length): a producer lane loads two adjacent
// pixels as one dword, a wave's block is 64 pixels (128-byte pieces of every
// channel row instead of 64-byte ones) and holds two accumulators, one per pixel
// parity; the progress words stay per 32 pixels.
template <int FS, int CPQ, int KR, int NQ = 4, bool PAIR = false>
__global__ __launch_bounds__(kThreads) void fwd_pipe_kernel(FwdArgs a, PipePlan pl) {
  extern __shared__ float lds[];
  // A plane: [rank quad][QA cells] of four fp32 each (the quad's ranks side by side:
  // one 16-byte LDS access moves a cell's four ranks)
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  f32x4* As4 = reinterpret_cast<f32x4*>(lds);
  unsigned char* ldsb = reinterpret_cast<unsigned char*>(lds);
  unsigned char* Fb = ldsb + pl.fin_off;     // Fin fragments [chunk][part][hi][r] x 16 B (CPQ == 0)
  unsigned char* Cb = ldsb + pl.cc_off;      // 3 x Cc fragment tiles
  // [0..kMaxBlk) quarters done per block (sweep order), then 4 consumer arrival
  // counters, then the 4 contraction counters of the split-role schedule, then
  // the abort word
  int* flags = reinterpret_cast<int*>(ldsb + pl.flag_off);
#ifdef CP4_PIPE_EPILOGUE
  float* biasL = reinterpret_cast<float*>(flags + kMaxBlk + 16);   // [32 * nkb], zero past Cout
#endif

  const int per = (pl.nWG + 7) >> 3;
  const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);         // XCD-contiguous tile order
  if (t >= pl.nWG) return;
#ifdef CP4_PIPE_TILED
  const int per_img = pl.strips * pl.cols;
  const int n = t / per_img, trem = t - n * per_img;
  const int strip = trem / pl.cols, h0 = strip * pl.TH, w0 = (trem - strip * pl.cols) * pl.Wt;
  const bool rev = false;
#else
  const int n = t / pl.strips, strip = t - n * pl.strips, h0 = strip * pl.TH;
  const bool rev = strip & 1;                    // odd strips sweep bottom-up
#endif

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const WaitCtx wx{pl.spin_limit, flags + kMaxBlk + 8, a.fault, t, wave};
#ifdef CP4_DEBUG_PHASES
#define STAMP(i) if (pl.dbg && lane == 0 && (i) < 32) { pl.dbg[((size_t)t * 16 + wave) * 32 + (i)] = wall_clock64(); }
#if CP4_DEBUG_PHASES > 1
#define STAMPX(i) STAMP(i)
#else
#define STAMPX(i)
#endif
#else
#define STAMP(i)
#define STAMPX(i)
#endif
  STAMP(0)
#ifdef CP4_DEBUG_PHASES
  if (pl.dbg && lane == 0) pl.dbg[((size_t)t * 16 + wave) * 32 + 30] = clock64();
#endif
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin;
  // this workgroup's output channels [k0, k0 + Cout) of the layer's CoutAll
  const int CoutAll = a.Cout;
  const int k0 = pl.kparts > 1 ? (int)blockIdx.y * pl.kslice : 0;
  const int Cout = pl.kparts > 1 ? min(pl.kslice, CoutAll - k0) : CoutAll;
#ifdef CP4_PIPE_STRIDED
  // output plane, stride, zeros before the image; h0 counts output rows
  const int Ho = a.Ho, Wo = a.Wo, HWo = Ho * Wo, SH = a.sh, SW = a.sw, PT = a.pt, PL = a.pl;
  // a filter of FY x FX taps set into the FS x FS window (even or rectangular filters):
  // the plane holds the rows FY taps reach, taps past FY / FX weigh nothing
  const int FY = a.ty ? a.ty : FS, FX = a.tx ? a.tx : FS;
#else
  [[maybe_unused]] const int Ho = H, Wo = W, HWo = HW;
#endif
  const int QA = pl.QA;
#ifdef CP4_PIPE_PASSES
  const int ldf = a.ldf ? a.ldf : R;             // row stride of the factor matrices
#else
  const int ldf = R;
#endif
  const int rows = min(pl.TH, Ho - h0);
#ifdef CP4_PIPE_TILED
  const int Wt = pl.Wt, lgWt = pl.lgWt, WL = Wt + FS - 1;   // tile width, LDS row length
  const int wcols = min(Wt, W - w0);             // tile columns inside the image
  const int nvalid = rows * Wt;                  // output cells of the tile (a multiple of 64)
  const int gshift = 0;
  const int ngroups = nvalid >> 6;
#else
  const int nvalid = rows * Wo;                  // output pixels inside the image
  // 64-pixel output groups start `gshift` pixels before the strip so that their
  // boundaries fall on 128-byte lines of y (pixel h0*W + 64*g - gshift is a
  // multiple of 32); pixels before the strip are computed and not stored.
  const int gshift = (h0 * Wo) & 31;
  const int ngroups = (nvalid + gshift + 63) >> 6;
#endif
  const int nkb = (Cout + 31) >> 5;
#ifdef CP4_PIPE_TILED
  const int QLEN = (pl.TH + FS - 1) * WL;
#else
#ifdef CP4_PIPE_STRIDED
  // adjoint of a strided layer: the plane holds the input rows trow0 ... that the
  // strip's output rows h0 ... h0 + TH - 1 can draw on, (h + PT - i) / SH
  const bool TR = a.transposed != 0;
  const int trow0 = h0 + PT - (FY - 1) <= 0 ? 0 : (h0 + PT - (FY - 1) + SH - 1) / SH;
  const int qbase = TR ? trow0 * W : (SH * h0 - PT) * W;   // global flat pixel of LDS column 0
  const int QLEN = TR ? ((pl.TH + FY - 2) / SH + 1) * W : (SH * (pl.TH - 1) + FY) * W;
#else
  const int qbase = (h0 - a.pad) * W;            // global flat pixel of LDS column 0
  const int QLEN = (pl.TH + FS - 1) * W;
#endif
#endif
  const int nblk = (QLEN + 31) >> 5;             // 32-pixel producer blocks
  const bool low16 = R <= 16;                    // the plane holds rank rows 0 ... 15 only
  const bool backoff = nblk >= 4;                // growing naps in the spin waits

  // ---- prologue: clear the progress words; above 256 input channels the input
  // factor does not fit the producers' registers and goes to LDS, pre-split ----
  constexpr bool FLDS = CPQ == 0;
  constexpr int NB = kProd / NQ;                   // blocks per producer round
  const int cpq = FLDS ? (Cin + 63) >> 6 : CPQ;    // 16-channel chunks per channel split
  if (tid < kMaxBlk + 16) flags[tid] = 0;
#ifdef CP4_PIPE_EPILOGUE
  for (int k = tid; k < 32 * nkb; k += kThreads) biasL[k] = (a.bias && k < Cout) ? a.bias[k0 + k] : 0.f;
#endif
  if (FLDS) {
    for (int it = tid; it < 8 * cpq * 32; it += kThreads) {
      const int o = it >> 5, r = it & 31;          // channel octet (of the padded count), rank
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = (r < R && 8 * o + e < Cin) ? a.Fin[(size_t)(8 * o + e) * ldf + r] : 0.f;
      u32x4 h, m, l;
      split8(v, h, m, l);
      u32x4* dst = reinterpret_cast<u32x4*>(Fb + ((size_t)(o >> 1) * 6 + (o & 1)) * 512 + r * 16);
      dst[0] = h;          // part stride: 2 planes of 512 B
      dst[64] = m;
      dst[128] = l;
    }
  }
  __syncthreads();
  STAMP(1)

  if (wave < kProd) {
    // =========================== producers ==================================
    const int bsel = wave % NB, cq = wave / NB;    // block within the round, channel split
    const int nrounds = PAIR ? (((nblk + 1) >> 1) + NB - 1) / NB : (nblk + NB - 1) / NB;
    // lane's channel 16*(cpq*cq + chunk) + 8*hi + e
    // (channel groups past Cin count as zero: their factor rows are, and x reads there return 0)
    const int cg0 = 16 * cpq * cq + 8 * hi;        // lane's first channel of chunk 0
    // x is read through a buffer descriptor over this image: the address is
    // (descriptor base) + (32-bit lane offset) + (scalar offset), so the walk
    // over channels runs on the scalar unit and no 64-bit vector adds sit between
    // the MFMAs; reads past the last channel (padded channel groups) return 0.
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
#ifdef CP4_PIPE_PASSES
        // (channel passes: this launch's Cin channels are a slice of wider images)
        const_cast<io_t*>(reinterpret_cast<const io_t*>(a.x) +
                          (size_t)n * (a.ldx ? (size_t)a.ldx : (size_t)Cin * HW)), 0,
#else
        const_cast<io_t*>(reinterpret_cast<const io_t*>(a.x) + (size_t)n * Cin * HW), 0,
#endif
        Cin * HW * kIoBytes, 0x00020000);
    const unsigned sbase =
        (unsigned)(16 * cpq * cq) * (unsigned)HW * (unsigned)kIoBytes;   // uniform byte offset
    // This wave's slice of the input factor stays in registers for the whole
    // sweep, already split: lane holds rank l32, channels 16*(cpq*cq+c) + 8*hi + e.
    constexpr int NF = FLDS ? 1 : CPQ;
    u32x4 fh[NF], fm[NF], fl[NF];
    if (!FLDS) {
      // (two copies of the loop on purpose: with whole chunks of channels the loads of
      // a slice sit under one condition and go out together - the start of every
      // workgroup waits for them; with a ragged channel count each has its own)
      if ((Cin & (16 * NQ - 1)) == 0) {
#pragma unroll
        for (int c = 0; c < NF; ++c) {
          float v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = l32 < R ? a.Fin[(size_t)(cg0 + 16 * c + e) * ldf + l32] : 0.f;
          split8(v, fh[c], fm[c], fl[c]);
        }
      } else {
#pragma unroll
        for (int c = 0; c < NF; ++c) {
          float v[8];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = (l32 < R && cg0 + 16 * c + e < Cin)
                       ? a.Fin[(size_t)(cg0 + 16 * c + e) * ldf + l32]
                       : 0.f;
          split8(v, fh[c], fm[c], fl[c]);
        }
      }
    }
    const u32x4* fbase =
        reinterpret_cast<const u32x4*>(Fb + hi * 512 + l32 * 16) + (size_t)(cq * cpq) * (6 * 32);
    // Block of round r: sweep index j, LDS column qa of this lane, whether the
    // lane's pixel exists, and the lane's byte offset (clamped pixel, channel 8*hi).
    auto geom = [&](int r, int& j, int& qa, bool& valid, [[maybe_unused]] bool& ex) -> unsigned {
#ifdef CP4_PIPE_IO16
      if constexpr (PAIR) {
        // span NB * r + bsel of the sweep: its 32-pixel blocks j and j + 1 (sweep
        // order), 64 plane cells from s0 (-32 when the sweep runs backwards and
        // the last span has one block only); the lane's pixels are cells qa, qa + 1
        j = 2 * (NB * r + bsel);
        const int s0 = rev ? 32 * (nblk - 2 - j) : 32 * j;
        qa = s0 + 2 * l32;
        const int q = qbase + qa;                  // even: W is
        ex = j < nblk && qa >= 0 && qa < 32 * nblk;
        valid = ex && q >= 0 && q < HW && qa < QLEN;
        const int qc = q < 0 ? 0 : (q > HW - 2 ? HW - 2 : q);
        return (unsigned)(8 * hi * HW + qc) * (unsigned)kIoBytes;
      }
#endif
      j = NB * r + bsel;
      const int b = rev ? nblk - 1 - j : j;        // j == nblk happens when nblk is odd
      qa = 32 * b + l32;
#ifdef CP4_PIPE_TILED
      // cell qa of the tile plane: row lr, column lc -> image pixel (grow, gcol)
      const int lr = (int)__umulhi((unsigned)qa, pl.wl_magic), lc = qa - lr * WL;
      const int grow = h0 - a.pad + lr, gcol = w0 - a.pad + lc;
      valid = j < nblk && qa < QLEN && grow >= 0 && grow < H && gcol >= 0 && gcol < W;
      const int qc = valid ? grow * W + gcol : 0;
#else
      const int q = qbase + qa;
      valid = j < nblk && q >= 0 && q < HW && qa < QLEN;
      const int qc = q < 0 ? 0 : (q > HW - 1 ? HW - 1 : q);
#endif
      return (unsigned)(8 * hi * HW + qc) * (unsigned)kIoBytes;
    };
#ifdef CP4_PIPE_IO16
    // ring entries hold the raw bfloat16 bits, zero-extended
    using ring_t = unsigned;
    auto ld_chunk = [&](ring_t (&dst)[8], unsigned voff, int chunk) {   // chunk < cpq
      const unsigned soff = sbase + (unsigned)(16 * chunk) * (unsigned)HW * 2u;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if constexpr (PAIR)
          dst[e] = __builtin_amdgcn_raw_buffer_load_b32(xrs, voff, soff + (unsigned)e * HW * 2u, 0);
        else
          dst[e] = (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(
              xrs, voff, soff + (unsigned)e * HW * 2u, 0);
      }
    };
#else
    using ring_t = float;
    auto ld_chunk = [&](ring_t (&dst)[8], unsigned voff, int chunk) {   // chunk < cpq
      const unsigned soff = sbase + (unsigned)(16 * chunk) * (unsigned)HW * 4u;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        dst[e] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(xrs, voff, soff + (unsigned)e * HW * 4u, 0));
    };
#endif
    ring_t xb[KR][8];
    int j, qa;
    bool valid, ex = true;
    unsigned xp = geom(0, j, qa, valid, ex);
#pragma unroll
    for (int u = 0; u < KR; ++u) ld_chunk(xb[u], xp, u);
    for (int r = 0; r < nrounds; ++r) {
      int jn, qan;
      bool validn, exn = true;
      const unsigned xpn = geom(r + 1 < nrounds ? r + 1 : r, jn, qan, validn, exn);
      f32x16 acc = (f32x16)(0.f);
      [[maybe_unused]] f32x16 acc2 = (f32x16)(0.f);      // PAIR: the odd pixels
      auto step = [&](int ch, int u) {
#if CP4_PIPE_IO16 == 2
        // half-precision activations: 11 significand bits are two bfloat16 parts
        // (h + m exactly, l = 0), so five of the six partial products remain
        if constexpr (PAIR) {
          float xe[8], xo[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            xe[e] = (float)__builtin_bit_cast(_Float16, (unsigned short)xb[u][e]);
            xo[e] = (float)__builtin_bit_cast(_Float16, (unsigned short)(xb[u][e] >> 16));
          }
          u32x4 eh, em, el, oh, om, ol;
          split8(xe, eh, em, el);
          split8(xo, oh, om, ol);
          u32x4 tl, tm, th;
          if (FLDS) {
            const u32x4* fp = fbase + (size_t)(ch + u) * (6 * 32);
            th = fp[0], tm = fp[64], tl = fp[128];
          } else {
            th = fh[FLDS ? 0 : ch + u], tm = fm[FLDS ? 0 : ch + u], tl = fl[FLDS ? 0 : ch + u];
          }
          acc = mfma16(tl, eh, acc);
          acc = mfma16(tm, em, acc);
          acc = mfma16(tm, eh, acc);
          acc = mfma16(th, em, acc);
          acc = mfma16(th, eh, acc);
          acc2 = mfma16(tl, oh, acc2);
          acc2 = mfma16(tm, om, acc2);
          acc2 = mfma16(tm, oh, acc2);
          acc2 = mfma16(th, om, acc2);
          acc2 = mfma16(th, oh, acc2);
        } else {
        float xv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          xv[e] = (float)__builtin_bit_cast(_Float16, (unsigned short)xb[u][e]);
        u32x4 xh, xm, xl;
        split8(xv, xh, xm, xl);
        if (FLDS) {
          const u32x4* fp = fbase + (size_t)(ch + u) * (6 * 32);
          acc = mfma16(fp[128], xh, acc);
          acc = mfma16(fp[64], xm, acc);
          acc = mfma16(fp[64], xh, acc);
          acc = mfma16(fp[0], xm, acc);
          acc = mfma16(fp[0], xh, acc);
        } else {
          acc = mfma16(fl[FLDS ? 0 : ch + u], xh, acc);
          acc = mfma16(fm[FLDS ? 0 : ch + u], xm, acc);
          acc = mfma16(fm[FLDS ? 0 : ch + u], xh, acc);
          acc = mfma16(fh[FLDS ? 0 : ch + u], xm, acc);
          acc = mfma16(fh[FLDS ? 0 : ch + u], xh, acc);
        }
        }
#elif defined(CP4_PIPE_IO16)
        // the activations are bfloat16 already: pack pairs, multiply by the three
        // factor parts (smallest first)
        u32x4 xh;
        [[maybe_unused]] u32x4 xo;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          if constexpr (PAIR) {
            // low halves: the even pixel of channels 2d, 2d + 1; high halves: the odd one
            xh[d] = __builtin_amdgcn_perm(xb[u][2 * d + 1], xb[u][2 * d], 0x05040100u);
            xo[d] = __builtin_amdgcn_perm(xb[u][2 * d + 1], xb[u][2 * d], 0x07060302u);
          } else {
            xh[d] = xb[u][2 * d] | (xb[u][2 * d + 1] << 16);
          }
        }
        if (FLDS) {
          const u32x4* fp = fbase + (size_t)(ch + u) * (6 * 32);
          acc = mfma16(fp[128], xh, acc);
          acc = mfma16(fp[64], xh, acc);
          acc = mfma16(fp[0], xh, acc);
          if constexpr (PAIR) {
            acc2 = mfma16(fp[128], xo, acc2);
            acc2 = mfma16(fp[64], xo, acc2);
            acc2 = mfma16(fp[0], xo, acc2);
          }
        } else {
          acc = mfma16(fl[FLDS ? 0 : ch + u], xh, acc);
          acc = mfma16(fm[FLDS ? 0 : ch + u], xh, acc);
          acc = mfma16(fh[FLDS ? 0 : ch + u], xh, acc);
          if constexpr (PAIR) {
            acc2 = mfma16(fl[FLDS ? 0 : ch + u], xo, acc2);
            acc2 = mfma16(fm[FLDS ? 0 : ch + u], xo, acc2);
            acc2 = mfma16(fh[FLDS ? 0 : ch + u], xo, acc2);
          }
        }
#else
        u32x4 xh, xm, xl;
        split8(xb[u], xh, xm, xl);
        if (FLDS) {
          const u32x4* fp = fbase + (size_t)(ch + u) * (6 * 32);
          acc = mfma_split(fp[0], fp[64], fp[128], xh, xm, xl, acc);
        } else {
          acc = mfma_split(fh[FLDS ? 0 : ch + u], fm[FLDS ? 0 : ch + u], fl[FLDS ? 0 : ch + u], xh,
                           xm, xl, acc);
        }
#endif
        // refill this ring slot: same round, or the first chunks of the next
        const int nxt = ch + u + KR;
        if (nxt < cpq)
          ld_chunk(xb[u], xp, nxt);
        else
          ld_chunk(xb[u], xpn, nxt - cpq);
        // keep use-then-refill order per chunk so KR chunks stay in flight
        __builtin_amdgcn_sched_barrier(0);
      };
      if (FLDS) {
        for (int ch = 0; ch < cpq; ch += KR) {
#pragma unroll
          for (int u = 0; u < KR; ++u) step(ch, u);
        }
      } else {
#pragma unroll
        for (int ch = 0; ch < NF; ch += KR) {
#pragma unroll
          for (int u = 0; u < KR; ++u) step(ch, u);
        }
      }
      if (j < nblk) {
        // add this quarter's partial sums after the lower quarters
        int* bf = &flags[j];
        // accumulator elements 4*g ... 4*g + 3 are ranks 8*g + 4*hi ...: rank quad 2*g + hi
        f32x4* dst = As4 + (size_t)hi * QA + qa;
        const int ng = low16 ? 2 : 4;              // the plane holds rank quads 0 ... 3 only
        if constexpr (PAIR) {
          // cells qa (even pixel) and qa + 1 (odd pixel); lanes whose half of the
          // span has no block touch nothing
          if (cq == 0) {
            if (ex) {
#pragma unroll
              for (int g = 0; g < 4; ++g)
                if (g < ng) {
                  const int v = 4 * g;
                  dst[(2 * g) * QA] = valid ? f32x4{acc[v], acc[v + 1], acc[v + 2], acc[v + 3]}
                                            : f32x4{0.f, 0.f, 0.f, 0.f};
                  dst[(2 * g) * QA + 1] =
                      valid ? f32x4{acc2[v], acc2[v + 1], acc2[v + 2], acc2[v + 3]}
                            : f32x4{0.f, 0.f, 0.f, 0.f};
                }
            }
          } else {
            wait_ge(bf, cq, backoff, wx, 1);
            if (ex && valid) {
#pragma unroll
              for (int g = 0; g < 4; ++g)
                if (g < ng) {
                  const int v = 4 * g;
                  const f32x4 o0 = dst[(2 * g) * QA], o1 = dst[(2 * g) * QA + 1];
                  dst[(2 * g) * QA] = o0 + f32x4{acc[v], acc[v + 1], acc[v + 2], acc[v + 3]};
                  dst[(2 * g) * QA + 1] = o1 + f32x4{acc2[v], acc2[v + 1], acc2[v + 2], acc2[v + 3]};
                }
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          if (lane == 0) {
            __hip_atomic_store(bf, cq + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (j + 1 < nblk)
              __hip_atomic_store(bf + 1, cq + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
          }
        } else {
        if (cq == 0) {
#pragma unroll
          for (int g = 0; g < 4; ++g)
            if (g < ng)
              dst[(2 * g) * QA] = valid ? f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]}
                                        : f32x4{0.f, 0.f, 0.f, 0.f};
        } else {
          wait_ge(bf, cq, backoff, wx, 1);
          // read, add, write two quads at a time: one LDS round trip per half
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            if (half == 1 && low16) break;
            f32x4 old[2];
#pragma unroll
            for (int g = 0; g < 2; ++g) old[g] = dst[(2 * (2 * half + g)) * QA];
#pragma unroll
            for (int g = 0; g < 2; ++g) {
              const int v = 4 * (2 * half + g);
              dst[(2 * (2 * half + g)) * QA] =
                  valid ? old[g] + f32x4{acc[v], acc[v + 1], acc[v + 2], acc[v + 3]} : old[g];
            }
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0)
          __hip_atomic_store(bf, cq + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
      }
      STAMP(2 + r)
      xp = xpn;
      j = jn;
      qa = qan;
      valid = validn;
      ex = exn;
    }
#ifdef CP4_DEBUG_PHASES
    if (pl.dbg && lane == 0) pl.dbg[((size_t)t * 16 + wave) * 32 + 31] = clock64();
#endif
  } else {
    // =========================== consumers ==================================
    const int wc = wave - kProd;                   // 0..7: rank quad in the tap step
    // Output-factor fragment of this wave's 32-channel block kb = wc (reloaded per
    // item only when there are more blocks than consumer waves): lane holds row
    // 32*kb + l32, ranks 16*c + 8*hi + e.
    // (slot 1: second block of a contraction wave in the wide split-role schedule)
    u32x4 fkh[2][2], fkm[2][2], fkl[2][2];
#ifdef CP4_PIPE_EPILOGUE
    const bool relu = a.act != 0;
#endif
    auto load_fk = [&](int kb, auto slot_c) {
      constexpr int slot = decltype(slot_c)::value;
      const int k = 32 * kb + l32;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int r = 16 * c + 8 * hi + e;
          v[e] = (k < Cout && r < R) ? a.Fout[(size_t)(k0 + k) * ldf + r] : 0.f;
        }
        split8(v, fkh[slot][c], fkm[slot][c], fkl[slot][c]);
      }
    };
    constexpr std::integral_constant<int, 0> slot0{};
    [[maybe_unused]] constexpr std::integral_constant<int, 1> slot1{};
    const bool fk_cached = nkb <= kCons;
    // With at most 16 ranks and at most 4 channel blocks only four waves have
    // ranks in the tap step and only four have a block to contract: the roles
    // are then split - waves 4-7 run the taps (rank quad wc - 4), waves 0-3 the
    // contractions - so that the tap step of one group overlaps the contraction
    // of the previous one, and the contraction skips the empty upper rank chunk.
    // Above that, up to 8 channel blocks (wide split): a tap wave takes two rank
    // quads (wq and wq + 4), a contraction wave two channel blocks (wc and
    // wc + 4, both output-factor fragments in registers).
    // With at most 16 ranks and one or two channel blocks even that leaves most
    // waves idle and every group's latency in series; a strip of many groups then
    // runs them side by side instead (own groups): consumer wave wc takes groups
    // wc, wc + 8, ... whole - the taps of all rank quads into a tile of its own,
    // then the contractions - with no hand-over between consumer waves at all.
    // (Only in the builds for up to 64 input channels, whose producers leave the
    // registers for it.)
#ifdef CP4_PIPE_TAPS2D
    constexpr bool own_groups = false;
#else
    const bool own_groups = NQ == 1 && pl.own && ngroups >= 4;   // (the host checked ranks, blocks, filter)
#endif
    const bool split_narrow = !own_groups && FS <= 5 && R <= 16 && nkb <= 4;  // (7x7: no registers to spare)
#if defined(CP4_PIPE_TAPS2D)
    // (twice the 2-D weights would not fit)
    const bool split_wide = false;
#else
    // It pays with six or more channel blocks, or once the groups of a strip form a
    // pipeline (a single group gains nothing from overlapping with its neighbours).
    // Not for the accumulating rank pass: its stores read y first, and a
    // contraction wave would wait for that twice per group, one block after the other.
    // (5x5: the weights of a second rank quad do not fit - up to 16 ranks only)
    const bool split_wide = !split_narrow && pl.split2 && (FS <= 3 || (FS == 5 && R <= 16)) &&
                            nkb <= 8 && (nkb >= 6 || ngroups >= 3) && !a.accumulate;
#endif
    const bool split_roles = split_narrow || split_wide;
    const int wq = split_roles ? (wc >= 4 ? wc - 4 : 0) : wc;     // (first) rank quad in the tap step
    // Narrow split with one or two channel blocks: the contraction waves left over
    // take alternate groups (wave wc: block wc % nkb of the groups i = wc / nkb
    // modulo crep), so two or four groups' contractions and stores are in flight.
    // (From eight groups on; on shorter strips the extra waves' set-up costs more than
    // they gain: C2 7.1 -> 7.3 us.)
    const int crep = split_narrow && nkb <= 2 && ngroups >= 8 ? 4 / nkb : 1;
    if (!split_wide && fk_cached && wc < nkb * crep) {
      load_fk(wc % nkb, slot0);
    }
    // Tap weights of this wave's 4 ranks (wave-uniform values).
#ifdef CP4_PIPE_TAPS2D
    constexpr int NTQ = 1;
    float w2[NTQ][4][FS][FS];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr)
#pragma unroll
      for (int ti = 0; ti < FS; ++ti)
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          const int ty = a.flip ? FS - 1 - ti : ti, tx = a.flip ? FS - 1 - j : j, r = 4 * wq + rr;
          w2[0][rr][ti][j] = r < R ? a.taps2d[(ty * FS + tx) * ldf + r] : 0.f;
        }
#else
    constexpr int NTQ = FS <= 3 ? 2 : 1;           // quads a tap wave may take (wide split)
    float fh[NTQ][4][FS], fw[NTQ][4][FS];
    auto load_taps = [&](auto qi_c) {
      constexpr int qi = decltype(qi_c)::value;
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
#pragma unroll
        for (int j = 0; j < FS; ++j) {
#ifdef CP4_PIPE_STRIDED
          const int r = 4 * (wq + 4 * qi) + rr;
          const int tap = a.flip ? FY - 1 - j : j, tapw = a.flip ? FX - 1 - j : j;
          fh[qi][rr][j] = r < R && j < FY ? a.FH[tap * ldf + r] : 0.f;
          fw[qi][rr][j] = r < R && j < FX ? a.FW[tapw * ldf + r] : 0.f;
#else
          const int tap = a.flip ? FS - 1 - j : j, r = 4 * (wq + 4 * qi) + rr;
          fh[qi][rr][j] = r < R ? a.FH[tap * ldf + r] : 0.f;
          fw[qi][rr][j] = r < R ? a.FW[tap * ldf + r] : 0.f;
#endif
        }
    };
    load_taps(std::integral_constant<int, 0>{});
#endif
#ifdef CP4_PIPE_TILED
    io_t* yn = reinterpret_cast<io_t*>(a.y) + ((size_t)n * CoutAll + k0) * HW + (size_t)h0 * W + w0;
#else
    io_t* yn = reinterpret_cast<io_t*>(a.y) + ((size_t)n * CoutAll + k0) * HWo + (size_t)h0 * Wo;
#endif
    [[maybe_unused]] const bool accumulate = a.accumulate != 0;
    const bool pair_stores =                       // one store per pixel pair is legal
        ((Wo | HWo) & 1) == 0 && (reinterpret_cast<uintptr_t>(a.y) & (2 * kIoBytes - 1)) == 0;
#if !defined(CP4_PIPE_TILED) && !defined(CP4_PIPE_STRIDED)
    const int reach = (FS - 1) * (W + 1);          // how far past a pixel its taps read in A
#endif

    int frontier = 0;                              // blocks [0, frontier) of the sweep are complete
    int* arrivals = flags + kMaxBlk;               // [4] tap-step arrivals, slot = step & 3
    int* cdone = flags + kMaxBlk + 4;              // [4] split roles: contractions done, slot = step & 3

    // Tap step i of the sweep (pixel group g), `taps` below: wait for the
    // producers of every block the group's taps touch, compute pixel 64*g + lane
    // for ranks 4*wc .. 4*wc + 3, write the split fragments into fragment tile
    // `cb`, then signal arrival.
    // Highest sweep index among the blocks the taps of step i touch: the taps of
    // pixel p read A columns p - pad .. p + (FS-1)*(W+1) - pad.
    auto need_of = [&](int i) {
#ifdef CP4_PIPE_TILED
      // group i is the row segment (h, w .. w + 63): its taps read plane rows
      // h .. h + FS - 1, columns w .. w + 62 + FS
      const int h = (64 * i) >> lgWt, w = (64 * i) & (Wt - 1);
      const int last = ((h + FS - 1) * WL + w + 63 + FS - 1) >> 5;
      return last > nblk - 1 ? nblk - 1 : last;
#elif defined(CP4_PIPE_STRIDED)
      // group g holds output pixels 64*g - gshift ... + 63 of the strip: its taps
      // read the plane rows SH*h ... SH*h + FS - 1 of its first to last output row h
      const int g = rev ? ngroups - 1 - i : i;
      const int pf = max(64 * g - gshift, 0), pz = min(64 * g - gshift + 63, nvalid - 1);
      if (TR) {
        // output rows hf ... hz draw on the input rows ceil((hf + PT - FS + 1) / SH)
        // ... floor((hz + PT) / SH)
        const int hf = h0 + pf / Wo, hz = h0 + pz / Wo;
        if (rev) {
          const int num = hf + PT - (FY - 1);
          const int first = (num <= 0 ? 0 : (num + SH - 1) / SH) - trow0;   // >= 0
          const int b = (first * W) >> 5;
          return b > nblk - 1 ? 0 : nblk - 1 - b;
        }
        const int lastrow = min((hz + PT) / SH, H - 1) - trow0;
        if (lastrow < 0) return 0;
        const int last = ((lastrow + 1) * W - 1) >> 5;
        return last > nblk - 1 ? nblk - 1 : last;
      }
      if (rev) return nblk - 1 - ((SH * (pf / Wo) * W) >> 5);
      const int last = ((SH * (pz / Wo) + FY - 1) * W + W - 1) >> 5;
      return last > nblk - 1 ? nblk - 1 : last;
#else
      const int g = rev ? ngroups - 1 - i : i;
      int last = max(64 * g - gshift + 63 + reach, 0) >> 5;
      if (last > nblk - 1) last = nblk - 1;
      const int first = max(64 * g - gshift - a.pad, 0) >> 5;
      return rev ? nblk - 1 - first : last;
#endif
    };
    // Non-blocking: advance the frontier over finished blocks, say whether step
    // i could run its taps now.
    auto ready = [&](int i) {
      const int need = need_of(i);
      while (frontier <= need &&
             __hip_atomic_load(&flags[frontier], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) >= NQ)
        ++frontier;
      return frontier > need;
    };
    // Where the taps of pixel group g read the plane: first plane row h of the
    // lane's pixel, row length RL, and per tap column the (clamped) plane column
    // and whether it lies inside the image.
    struct TapPos {
      int roff[FS];                                // plane offset of tap row ti
      bool rin[FS];                                // ... and whether that row exists
      int off[FS];
      bool in[FS];
    };
    auto tap_pos = [&](int g) {
      TapPos tp;
#ifdef CP4_PIPE_TILED
      // the plane carries the halo columns: tap (ti, j) of cell (h, w) is plane
      // cell (h + ti, w + j), no border cases
      const int p = 64 * g + lane;
      const int w = p & (Wt - 1), h = p >> lgWt;
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        tp.in[j] = true;
        tp.off[j] = w + j;
        tp.rin[j] = true;
        tp.roff[j] = (h + j) * WL;                 // WL: row length of the plane
      }
#elif defined(CP4_PIPE_STRIDED)
      // lanes before or past the strip's outputs: any valid pixel (not stored)
      const int p = min(max(64 * g - gshift + lane, 0), nvalid - 1);
      const int ho = p / Wo, wo = p - ho * Wo;
      if (TR) {
        // tap row ti: input row (h + PT - ti) / SH where that is exact and inside the
        // plane; quotient and remainder step down with ti (one division per lane)
        int qh = (h0 + ho + PT) / SH, rh = (h0 + ho + PT) - qh * SH;
        int qw = (wo + PL) / SW, rw = (wo + PL) - qw * SW;
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          tp.rin[j] = rh == 0 && qh >= 0 && qh < H && j < FY;
          tp.roff[j] = tp.rin[j] ? (qh - trow0) * W : 0;
          tp.in[j] = rw == 0 && qw >= 0 && qw < W && j < FX;
          tp.off[j] = tp.in[j] ? qw : 0;
          if (--rh < 0) {
            rh += SH;
            --qh;
          }
          if (--rw < 0) {
            rw += SW;
            --qw;
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          const int ww = SW * wo + j - PL;
          tp.in[j] = ww >= 0 && ww < W;
          tp.off[j] = ww < 0 ? 0 : (ww >= W ? W - 1 : ww);   // clamped: weight is 0 there
          tp.rin[j] = j < FY;                      // (rows past the filter's own: not in the plane)
          tp.roff[j] = j < FY ? (SH * ho + j) * W : 0;   // plane row SH * ho is the first tap row
        }
      }
#else
      const int p = max(64 * g - gshift + lane, 0);      // lanes before the strip: any valid column
      const int h = p / W;
      const int w = p - h * W;
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        const int ww = w + j - a.pad;
        tp.in[j] = ww >= 0 && ww < W;
        tp.off[j] = ww < 0 ? 0 : (ww >= W ? W - 1 : ww);   // clamped: weight is 0 there
        tp.rin[j] = true;
        tp.roff[j] = (h + j) * W;
      }
#endif
      return tp;
    };
    // The taps of rank quad q at the lane's pixel, split exactly and written into
    // fragment tile cb.  wa / wb: the quad's weights (2-D taps: wa[rank][row][col];
    // else rows wa[rank][row] and columns wb[rank][col]).
    auto tap_quad = [&](const TapPos& tp, int q, const auto& wa, [[maybe_unused]] const auto& wb,
                        unsigned char* cb) {
      // (a quad past the last rank has zero weights; it reads quad 0's cells, the
      // plane may end before its own, and writes zeros)
      const bool live = 4 * q < R;
      const f32x4* ab = As4 + (size_t)(live ? q : 0) * QA;
      float o[4];
      // One 16-byte read per tap cell brings the quad's four ranks.  3x3 and
      // smaller: all cells go out together, then the arithmetic; larger filters:
      // tap row by tap row (registers).
      if constexpr (FS <= 3) {
        f32x4 av[FS][FS];
#pragma unroll
        for (int ti = 0; ti < FS; ++ti)
#pragma unroll
          for (int j = 0; j < FS; ++j) av[ti][j] = ab[tp.roff[ti] + tp.off[j]];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          float s = 0.f;
#pragma unroll
          for (int ti = 0; ti < FS; ++ti) {
#ifdef CP4_PIPE_TAPS2D
#pragma unroll
            for (int j = 0; j < FS; ++j)
              s += (tp.in[j] && tp.rin[ti] ? wa[rr][ti][j] : 0.f) * av[ti][j][rr];
#else
            float hs = 0.f;
#pragma unroll
            for (int j = 0; j < FS; ++j) hs += (tp.in[j] ? wb[rr][j] : 0.f) * av[ti][j][rr];
            s += (tp.rin[ti] ? wa[rr][ti] : 0.f) * hs;
#endif
          }
          o[rr] = live ? s : 0.f;
        }
      } else {
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ti = 0; ti < FS; ++ti) {
          f32x4 av[FS];
#pragma unroll
          for (int j = 0; j < FS; ++j) av[j] = ab[tp.roff[ti] + tp.off[j]];
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
#ifdef CP4_PIPE_TAPS2D
#pragma unroll
            for (int j = 0; j < FS; ++j)
              s[rr] += (tp.in[j] && tp.rin[ti] ? wa[rr][ti][j] : 0.f) * av[j][rr];
#else
            float hs = 0.f;
#pragma unroll
            for (int j = 0; j < FS; ++j) hs += (tp.in[j] ? wb[rr][j] : 0.f) * av[j][rr];
            s[rr] += (tp.rin[ti] ? wa[rr][ti] : 0.f) * hs;
#endif
          }
        }
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) o[rr] = live ? s[rr] : 0.f;
      }
      // exact split of the four values: two dwords per part
      u32x2 ph, pm, pl2;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const float x0 = o[2 * d], x1 = o[2 * d + 1];
        ph[d] = pack_hi16(x0, x1);
        const float r0 = x0 - trunc_bf16(x0), r1 = x1 - trunc_bf16(x1);
        pm[d] = pack_hi16(r0, r1);
        pl2[d] = pack_hi16(r0 - trunc_bf16(r0), r1 - trunc_bf16(r1));
      }
      // plane ((part*2 + chunk)*2 + hi)*2 + parity, 512 B each; entry lane >> 1;
      // this quad is the low or high 8 bytes of the 16-byte entry
      unsigned char* dst = cb + ((((q >> 2) * 2 + ((q >> 1) & 1)) * 2 + (lane & 1)) * 512) +
                           (lane >> 1) * 16 + (q & 1) * 8;
      *reinterpret_cast<u32x2*>(dst) = ph;
      *reinterpret_cast<u32x2*>(dst + 8 * 512) = pm;
      *reinterpret_cast<u32x2*>(dst + 16 * 512) = pl2;
    };
    auto await_blocks = [&](int i) {
      const int need = need_of(i);
      while (frontier <= need) {
        wait_ge(&flags[frontier], NQ, backoff, wx, 2);
        ++frontier;
      }
    };
    auto taps = [&](int i, unsigned char* cb, auto ntq_c) {
      const int g = rev ? ngroups - 1 - i : i;
      await_blocks(i);
      STAMPX(2 + 4 * i)
      const TapPos tp = tap_pos(g);
#pragma unroll
      for (int qi = 0; qi < decltype(ntq_c)::value; ++qi) {
#ifdef CP4_PIPE_TAPS2D
        tap_quad(tp, wq + 4 * qi, w2[qi], w2[qi], cb);
#else
        tap_quad(tp, wq + 4 * qi, fh[qi], fw[qi], cb);
#endif
      }
      STAMPX(3 + 4 * i)
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane == 0)
        __hip_atomic_fetch_add(&arrivals[i & 3], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };

    // Contraction ranks -> the 32 output channels of block kb for pixel group g
    // from fragment tile cb (nch rank chunks of 16), epilogue, stores.
    auto contract_block = [&](const unsigned char* cb, int g, int kb, auto nch, bool signal,
                              int step, auto slot_c, auto seq_c) {
      constexpr int slot = decltype(slot_c)::value;
#ifdef CP4_PIPE_EPILOGUE
      // the accumulators start at the bias of their rows (from LDS) instead of zero
      f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
      if (a.bias) {                                // (the same for all waves)
        const float* bkb = biasL + 32 * kb + 4 * hi;
        acc0 = f32x16{bkb[0],  bkb[1],  bkb[2],  bkb[3],  bkb[8],  bkb[9],  bkb[10], bkb[11],
                      bkb[16], bkb[17], bkb[18], bkb[19], bkb[24], bkb[25], bkb[26], bkb[27]};
        acc1 = f32x16{bkb[0],  bkb[1],  bkb[2],  bkb[3],  bkb[8],  bkb[9],  bkb[10], bkb[11],
                      bkb[16], bkb[17], bkb[18], bkb[19], bkb[24], bkb[25], bkb[26], bkb[27]};
      }
      __builtin_amdgcn_sched_barrier(0);
#else
      f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
#endif
#pragma unroll
      for (int c = 0; c < decltype(nch)::value; ++c) {
        const unsigned char* bp = cb + ((c * 2 + hi) * 2) * 512 + l32 * 16;
        if constexpr (decltype(seq_c)::value) {
          // wide split (two output-factor fragments in registers): one pixel
          // parity's fragments live at a time
          {
            const u32x4 b0h = *reinterpret_cast<const u32x4*>(bp);
            const u32x4 b0m = *reinterpret_cast<const u32x4*>(bp + 8 * 512);
            const u32x4 b0l = *reinterpret_cast<const u32x4*>(bp + 16 * 512);
            acc0 = mfma_split(fkh[slot][c], fkm[slot][c], fkl[slot][c], b0h, b0m, b0l, acc0);
          }
          __builtin_amdgcn_sched_barrier(0);
          {
            const u32x4 b1h = *reinterpret_cast<const u32x4*>(bp + 512);
            const u32x4 b1m = *reinterpret_cast<const u32x4*>(bp + 9 * 512);
            const u32x4 b1l = *reinterpret_cast<const u32x4*>(bp + 17 * 512);
            acc1 = mfma_split(fkh[slot][c], fkm[slot][c], fkl[slot][c], b1h, b1m, b1l, acc1);
          }
        } else {
          const u32x4 b0h = *reinterpret_cast<const u32x4*>(bp);
          const u32x4 b1h = *reinterpret_cast<const u32x4*>(bp + 512);
          const u32x4 b0m = *reinterpret_cast<const u32x4*>(bp + 8 * 512);
          const u32x4 b1m = *reinterpret_cast<const u32x4*>(bp + 9 * 512);
          const u32x4 b0l = *reinterpret_cast<const u32x4*>(bp + 16 * 512);
          const u32x4 b1l = *reinterpret_cast<const u32x4*>(bp + 17 * 512);
          acc0 = mfma_split(fkh[slot][c], fkm[slot][c], fkl[slot][c], b0h, b0m, b0l, acc0);
          acc1 = mfma_split(fkh[slot][c], fkm[slot][c], fkl[slot][c], b1h, b1m, b1l, acc1);
        }
        __builtin_amdgcn_sched_barrier(0);     // one chunk's fragments live at a time
      }
      if (signal) {
        // the tile has been read: the tap waves may write it again three steps on
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0)
          __hip_atomic_fetch_add(&cdone[step & 3], 1, __ATOMIC_RELEASE,
                                 __HIP_MEMORY_SCOPE_WORKGROUP);
      }
      // The activation goes onto each value as it is stored (rewriting the
      // accumulators in place costs the compiler some 150 spilled registers).
#ifdef CP4_PIPE_EPILOGUE
#define EPI(val, v) (relu && (val) < 0.f ? 0.f : (val))          // (a NaN stays a NaN)
#else
#define EPI(val, v) (val)
#endif
      // store rows: uniform row base + one 32-bit lane offset
      const int p = 64 * g - gshift + 2 * l32;       // lane's pixel pair p, p + 1
#ifdef CP4_PIPE_TILED
      // tile cell p = (row, column) -> offset in the image plane from the tile's corner
      const int pcol = p & (Wt - 1);
      const int pofs = (p >> lgWt) * W + pcol;
      const bool pin0 = pcol < wcols, pin1 = pcol + 1 < wcols;
#else
      const int pofs = p;
      const bool pin0 = p >= 0 && p < nvalid, pin1 = p + 1 >= 0 && p + 1 < nvalid;
#endif
      io_t* rowbase = yn + (size_t)(32 * kb) * HWo;
      // the lane's pixel pair as one store: float2, or two bfloat16 in a dword
      auto store_pair = [&](io_t* dst, float v0, float v1) {
#ifdef CP4_PIPE_IO16
        *reinterpret_cast<unsigned*>(dst) = (unsigned)to_io(v0) | ((unsigned)to_io(v1) << 16);
#else
        float2 o;
        o.x = v0;
        o.y = v1;
#ifdef CP4_PIPE_PASSES
        if (accumulate) {                        // second rank pass: y += (wave-uniform)
          const float2 old = *reinterpret_cast<const float2*>(dst);
          o.x += old.x;
          o.y += old.y;
        }
#endif
        *reinterpret_cast<float2*>(dst) = o;
#endif
      };
      auto store_one = [&](io_t* dst, float v) {
#ifdef CP4_PIPE_IO16
        *dst = to_io(v);
#else
#ifdef CP4_PIPE_PASSES
        *dst = accumulate ? *dst + v : v;
#else
        *dst = v;
#endif
#endif
      };
      if (pair_stores) {
        // W and H*W even, y aligned to a pair: p is even and the pair is one store
        if (pin0) {
          const unsigned lofs = (unsigned)(4 * hi * HWo + pofs);
          if (32 * kb + 32 <= Cout) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
              store_pair(rowbase + (size_t)(8 * (v >> 2) + (v & 3)) * HWo + lofs, EPI(acc0[v], v), EPI(acc1[v], v));
          } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int kk = 8 * (v >> 2) + (v & 3);         // + 4*hi is in lofs
              if (32 * kb + kk + 4 * hi < Cout)
                store_pair(rowbase + (size_t)kk * HWo + lofs, EPI(acc0[v], v), EPI(acc1[v], v));
            }
          }
        }
      } else {
        // odd widths or planes: the two pixels are stored and bounded one by one
        const bool in0 = pin0, in1 = pin1;
        const long lofs = (long)(4 * hi) * HWo + pofs;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kk = 8 * (v >> 2) + (v & 3);
          if (32 * kb + kk + 4 * hi < Cout) {
            io_t* rp = rowbase + (size_t)kk * HWo + lofs;
            if (in0) store_one(rp, EPI(acc0[v], v));
            if (in1) store_one(rp + 1, EPI(acc1[v], v));
          }
        }
      }
    };

    constexpr std::integral_constant<int, 1> one{};
    constexpr std::integral_constant<int, 2> two{};
    [[maybe_unused]] constexpr std::integral_constant<bool, true> yes{};
    constexpr std::integral_constant<bool, false> no{};
#ifndef CP4_PIPE_TAPS2D
    if constexpr (NQ == 1) {
    if (own_groups) {
      // Two waves share a 12 KB tile buffer: with one rank chunk a group's
      // fragments fill only the chunk-0 planes of each part, and the chunk-1
      // planes (4 * 512 bytes further) hold the other wave's.
      unsigned char* cb = Cb + (wc >> 1) * kCcBuf + (wc & 1) * (4 * 512);
      const int nq = (R + 3) >> 2;
      load_fk(0, slot0);
      if (nkb > 1) load_fk(1, slot1);
      // the quads past the last rank: zeros, written once (the tile is never
      // anyone else's)
      for (int q = nq; q < 4; ++q) {
        unsigned char* dst = cb + ((((q >> 1) & 1) * 2 + (lane & 1)) * 512) + (lane >> 1) * 16 + (q & 1) * 8;
        const u32x2 zero = {0u, 0u};
        *reinterpret_cast<u32x2*>(dst) = zero;
        *reinterpret_cast<u32x2*>(dst + 8 * 512) = zero;
        *reinterpret_cast<u32x2*>(dst + 16 * 512) = zero;
      }
      for (int i = wc; i < ngroups; i += kCons) {
        const int g = rev ? ngroups - 1 - i : i;
        await_blocks(i);
        STAMPX(2 + 4 * (i >> 3))
        const TapPos tp = tap_pos(g);
        for (int q = 0; q < nq; ++q) {
          float qh[4][FS], qw[4][FS];               // wave-uniform loads
#pragma unroll
          for (int rr = 0; rr < 4; ++rr)
#pragma unroll
            for (int j = 0; j < FS; ++j) {
#ifdef CP4_PIPE_STRIDED
              const int r = 4 * q + rr;
              const int tap = a.flip ? FY - 1 - j : j, tapw = a.flip ? FX - 1 - j : j;
              qh[rr][j] = r < R && j < FY ? a.FH[tap * ldf + r] : 0.f;
              qw[rr][j] = r < R && j < FX ? a.FW[tapw * ldf + r] : 0.f;
#else
              const int tap = a.flip ? FS - 1 - j : j, r = 4 * q + rr;
              qh[rr][j] = r < R ? a.FH[tap * ldf + r] : 0.f;
              qw[rr][j] = r < R ? a.FW[tap * ldf + r] : 0.f;
#endif
            }
          tap_quad(tp, q, qh, qw, cb);
        }
        STAMPX(3 + 4 * (i >> 3))
        // (the tile is this wave's own: its LDS writes and reads stay in order)
        contract_block(cb, g, 0, one, false, i, slot0, yes);
        if (nkb > 1) {
          contract_block(cb, g, 1, one, false, i, slot1, yes);
        }
        STAMPX(5 + 4 * (i >> 3))
      }
      return;
    }
    }
    if (split_wide) {
      // As the narrow split below, with two rank quads per tap wave and up to two
      // channel blocks per contraction wave; the tile is free again once every
      // contraction wave has read it for its last block.
      const int ncw = nkb < 4 ? nkb : 4;           // contraction waves with a block
      if (wc >= 4) {
        // (up to 16 ranks: the second rank chunk is never read, one quad each)
        if constexpr (NTQ == 2) {
          if (R > 16) load_taps(std::integral_constant<int, 1>{});
        }
        for (int i = 0; i < ngroups; ++i) {
          if (i >= 3) wait_ge(&cdone[(i - 3) & 3], ncw * (((i - 3) >> 2) + 1), backoff, wx, 3);
          if constexpr (NTQ == 2) {
            if (R > 16) {
              taps(i, Cb + (i % 3) * kCcBuf, two);
              continue;
            }
          }
          taps(i, Cb + (i % 3) * kCcBuf, one);
        }
      } else if (wc < nkb) {
        const bool second = wc + 4 < nkb;
        load_fk(wc, slot0);
        if (second) load_fk(wc + 4, slot1);
        for (int i = 0; i < ngroups; ++i) {
          const int g = rev ? ngroups - 1 - i : i;
          const unsigned char* cb = Cb + (i % 3) * kCcBuf;
          wait_ge(&arrivals[i & 3], 4 * ((i >> 2) + 1), backoff, wx, 4);
          STAMPX(4 + 4 * i)
          if (R <= 16) {
            contract_block(cb, g, wc, one, !second, i, slot0, yes);
          } else {
            contract_block(cb, g, wc, two, !second, i, slot0, yes);
          }
          if (second) {
            if (R <= 16) {
              contract_block(cb, g, wc + 4, one, true, i, slot1, yes);
            } else {
              contract_block(cb, g, wc + 4, two, true, i, slot1, yes);
            }
          }
          STAMP(5 + 4 * i)
        }
      }
      return;
    }
#endif
    if (split_roles) {
      // The tile of step i is i % 3; the tap waves write it after every
      // contraction wave has read it for step i - 3.  cdone[s] counts one per
      // contraction wave for the steps = s mod 4 (a single running total would
      // not do: a fast wave's later steps could stand in for a slow wave's
      // missing one); like the arrivals, a slot cannot run a whole cycle ahead.
      // A tap wave whose rank quad lies past the last rank (up to 12 ranks) has
      // nothing to compute: it zeroes its quad's entries in the three tiles once,
      // arrives once (counted with step 0) and ends; the steps then count the
      // live tap waves only.
      // Up to 16 ranks a tile fills only the planes of its first rank chunk, so the
      // first two of the three tiles share a buffer (the second in the planes of
      // the unused chunk, 4 * 512 bytes further) and the plane gets the room.
      auto tile3 = [&](int k) { return Cb + (k >> 1) * kCcBuf + (k & 1) * (4 * 512); };
      const int nlive = min(4, (R + 3) >> 2), ndead = 4 - nlive;
      if (wc >= 4) {
        if (4 * wq >= R) {
          const u32x2 zero = {0u, 0u};
#pragma unroll
          for (int tb = 0; tb < 3; ++tb) {
            unsigned char* dst = tile3(tb) + ((((wq >> 1) & 1) * 2 + (lane & 1)) * 512) +
                                 (lane >> 1) * 16 + (wq & 1) * 8;
            *reinterpret_cast<u32x2*>(dst) = zero;
            *reinterpret_cast<u32x2*>(dst + 8 * 512) = zero;
            *reinterpret_cast<u32x2*>(dst + 16 * 512) = zero;
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
          if (lane == 0)
            __hip_atomic_fetch_add(&arrivals[0], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
          return;
        }
        for (int i = 0; i < ngroups; ++i) {
          if (i >= 3) wait_ge(&cdone[(i - 3) & 3], nkb * (((i - 3) >> 2) + 1), backoff, wx, 5);
          taps(i, tile3(i % 3), one);
        }
      } else if (wc < nkb * crep) {
        // (a slot of cdone still gets its nkb signals per step, all from the same
        // waves in step order)
        const int kb = wc % nkb;
        for (int i = wc / nkb; i < ngroups; i += crep) {
          const int g = rev ? ngroups - 1 - i : i;
          wait_ge(&arrivals[i & 3], nlive * ((i >> 2) + 1) + ((i & 3) == 0 ? ndead : 0), backoff, wx,
                  6);
          contract_block(tile3(i % 3), g, kb, one, true, i, slot0, no);
        }
      }
      return;
    }
    // Three fragment tiles in rotation.  Iteration i: once every consumer wave
    // has arrived for step i (which also means it has finished the contraction
    // of step i-2, the last reader of the tile written next), do the tap step
    // i+1 and contract step i, in either order.  The arrival of step i was
    // signalled about one contraction earlier, so this wait seldom stalls.
    unsigned char* cb_cur = Cb;
    unsigned char* cb_next = Cb + kCcBuf;
    unsigned char* cb_free = Cb + 2 * kCcBuf;
    taps(0, cb_cur, one);
    for (int i = 0; i < ngroups; ++i) {
      const int g = rev ? ngroups - 1 - i : i;
      wait_ge(&arrivals[i & 3], kCons * ((i >> 2) + 1), backoff, wx, 7);
      STAMPX(4 + 4 * i)
      // tap step i+1 goes first when its blocks are there (keeps the stores of
      // consecutive groups close), else after this group's contraction
      const bool early = i + 1 < ngroups && ready(i + 1);
      if (early) taps(i + 1, cb_next, one);
      // ---- rank -> output-channel contraction for this wave's blocks --------
      const unsigned char* cb = cb_cur;
      for (int kb = wc; kb < nkb; kb += kCons) {
        if (!fk_cached) {
          load_fk(kb, slot0);
        }
        contract_block(cb, g, kb, two, false, i, slot0, no);
      }
      STAMP(5 + 4 * i)
      if (i + 1 < ngroups && !early) taps(i + 1, cb_next, one);
      unsigned char* tmp = cb_cur;
      cb_cur = cb_next;
      cb_next = cb_free;
      cb_free = tmp;
    }
  }
}

int round_up(int v, int m) { return (v + m - 1) / m * m; }

// After the fragment tiles: the progress words and, in the builds with the bias /
// activation epilogue, the bias padded to whole 32-channel blocks.
size_t tail_bytes(const FwdArgs& a) {
  size_t b = (kMaxBlk + 16) * sizeof(int);
#ifdef CP4_PIPE_EPILOGUE
  b += (size_t)((a.Cout + 31) & ~31) * sizeof(float);
#endif
  return b;
}

// Fragment tiles: three in rotation, or one per consumer wave (two to a buffer)
// where the kernel may give every wave groups of its own.
bool own_groups_wanted(const FwdArgs& a) {
#ifdef CP4_PIPE_TAPS2D
  return false;
#else
  const bool legal = a.R <= 16 && a.Cout <= 64 && a.Cin <= 64 && a.Y <= 5 && !a.accumulate;
  // by default where one rank quad is the whole tap step (the other schedules
  // would run three empty quads beside it), with 3x3 and smaller filters and at
  // most 32 channels on one side also for two quads (16 x 16 x 512 x 512 at rank 8:
  // 213 against 262 us; 64 -> 64 channels 224 x 224: 49 against 47; 5x5: 27 against
  // 22); above that only when tuned so
  // (tune_split2: 0 this rule, 1 no role split at all, 2 own groups)
  const bool by_rule = a.R <= kOwnGroupsMaxRank ||
                       (a.R <= 2 * kOwnGroupsMaxRank && a.Y <= 3 && (a.Cin <= 32 || a.Cout <= 32));
  return legal && (a.tune_split2 == 2 || (a.tune_split2 == 0 && by_rule));
#endif
}
size_t cc_region_bytes(const FwdArgs& a) {
  if (own_groups_wanted(a)) return (size_t)4 * kCcBuf;
  // the narrow role split (the kernel's rule: up to 16 ranks, 4 channel blocks, 5x5)
  // packs its first two tiles into one buffer; the third ends after 20 planes
  if (a.R <= 16 && a.Cout <= 128 && a.Y <= 5) return (size_t)kCcBuf + 20 * 512;
  return (size_t)3 * kCcBuf;
}

// Rank rows of the A plane in LDS: the producers' 32 x 32 products carry 32, of
// which the upper 16 are zero (and neither written nor read) up to 16 ranks.
int plane_rows(const FwdArgs& a) { return a.R <= 16 ? 16 : kRP; }

[[maybe_unused]] bool layout(const FwdArgs& a, int TH, PipePlan* pl) {
  const long QLEN = (long)(TH + a.Y - 1) * a.W;
  // the taps of the last (partly filled) 64-pixel group may read past QLEN; the
  // groups start up to 31 pixels before the strip, so they end up to 31 + 63 past it
  const long QA =
      round_up((int)(round_up(TH * a.W + 31, 64) + (long)(a.Y - 1) * (a.W + 1) + 1), 64) + 8;
  const size_t a_bytes = (size_t)plane_rows(a) * QA * sizeof(float);
  // above 256 input channels: pre-split factor fragments, 192 B per (padded) channel
  const size_t fin_bytes = a.Cin > 256 ? (size_t)((a.Cin + 63) & ~63) * 192 : 0;
  const size_t bytes = a_bytes + fin_bytes + cc_region_bytes(a) + tail_bytes(a);
  if ((QLEN + 31) / 32 + 1 > kMaxBlk) return false;
  if (bytes > kLdsLimit) return false;
  pl->TH = TH;
  pl->nblk = (int)((QLEN + 31) / 32);
  pl->strips = (a.H + TH - 1) / TH;
  pl->nWG = a.N * pl->strips;
  pl->QA = (int)QA;
  pl->fin_off = (int)a_bytes;
  pl->cc_off = (int)(a_bytes + fin_bytes);
  pl->flag_off = (int)(a_bytes + fin_bytes + cc_region_bytes(a));
  pl->lds_bytes = bytes;
  return true;
}

// Strips (tiles) that fill at most half the chip, four or more blocks of 32 output channels: as
// many slices of at least two blocks as bring the grid up to the compute units
// (N1 C512 K512 28x28: 28 strips, 16 blocks -> 8 slices of two).
void choose_output_slices(const FwdArgs& a, int cus, PipePlan* pl) {
  const int nkb = (a.Cout + 31) / 32;
  if (a.tune_th > 0 || 2 * pl->nWG > cus || nkb < 4) return;
  int parts = cus / pl->nWG;
  if (parts > nkb / 2) parts = nkb / 2;
  if (parts < 2) return;
  const int blocks = (nkb + parts - 1) / parts;     // blocks per slice
  pl->kslice = 32 * blocks;
  pl->kparts = (nkb + blocks - 1) / blocks;
}
#ifdef CP4_PIPE_STRIDED
// Strip of TH output rows: plane of the sh * (TH - 1) + Y input rows under them.
bool layout_strided(const FwdArgs& a, int TH, PipePlan* pl) {
  const int FY = a.ty ? a.ty : a.Y;              // the filter's own rows (window: a.Y)
  const long QLEN = a.transposed ? ((long)(TH + FY - 2) / a.sh + 1) * a.W
                                 : ((long)a.sh * (TH - 1) + FY) * a.W;
  const long QA = round_up((int)QLEN, 64) + 8;
  const size_t a_bytes = (size_t)plane_rows(a) * QA * sizeof(float);
  const size_t fin_bytes = a.Cin > 256 ? (size_t)((a.Cin + 63) & ~63) * 192 : 0;
  const size_t bytes = a_bytes + fin_bytes + cc_region_bytes(a) + tail_bytes(a);
  if ((QLEN + 31) / 32 + 1 > kMaxBlk) return false;
  if (bytes > kLdsLimit) return false;
  pl->TH = TH;
  pl->nblk = (int)((QLEN + 31) / 32);
  pl->strips = (a.Ho + TH - 1) / TH;
  pl->nWG = a.N * pl->strips;
  pl->QA = (int)QA;
  pl->fin_off = (int)a_bytes;
  pl->cc_off = (int)(a_bytes + fin_bytes);
  pl->flag_off = (int)(a_bytes + fin_bytes + cc_region_bytes(a));
  pl->lds_bytes = bytes;
  return true;
}
bool plan(const FwdArgs& a, PipePlan* best) {
  double best_cost = 0;
  bool found = false;
  if (a.tune_th > 0) return a.tune_th <= a.Ho && layout_strided(a, a.tune_th, best);
  const int cus = num_compute_units();
  for (int TH = 1; TH <= a.Ho; ++TH) {
    PipePlan pl;
    if (!layout_strided(a, TH, &pl)) break;
    const double rounds = (pl.nWG + cus - 1) / cus;
    // cells read per channel and cells written per channel
    const double cost = rounds * ((double)pl.nblk * 32 * a.Cin +
                                  (double)TH * a.Wo * a.Cout + kTileStartCost);
    if (!found || cost <= best_cost) {
      best_cost = cost;
      *best = pl;
      found = true;
    }
  }
  if (found) choose_output_slices(a, cus, best);
  return found;
}
#elif defined(CP4_PIPE_TILED)
// Tile of TH rows x Wt columns: plane of (TH + Y - 1) rows of Wt + Y - 1 cells.
bool layout_tiled(const FwdArgs& a, int TH, int lgWt, PipePlan* pl) {
  const int Wt = 1 << lgWt, WL = Wt + a.Y - 1;
  const long QLEN = (long)(TH + a.Y - 1) * WL;
  const long QA = round_up((int)QLEN, 64) + 8;
  const size_t a_bytes = (size_t)plane_rows(a) * QA * sizeof(float);
  const size_t fin_bytes = a.Cin > 256 ? (size_t)((a.Cin + 63) & ~63) * 192 : 0;
  const size_t bytes = a_bytes + fin_bytes + cc_region_bytes(a) + tail_bytes(a);
  if ((QLEN + 31) / 32 + 1 > kMaxBlk) return false;
  if (bytes > kLdsLimit) return false;
  pl->TH = TH;
  pl->nblk = (int)((QLEN + 31) / 32);
  pl->strips = (a.H + TH - 1) / TH;
  pl->Wt = Wt;
  pl->lgWt = lgWt;
  pl->cols = (a.W + Wt - 1) / Wt;
  pl->wl_magic = (unsigned)(0x100000000ull / (unsigned)WL) + 1u;   // exact quotients below 2^16
  pl->nWG = a.N * pl->strips * pl->cols;
  pl->QA = (int)QA;
  pl->fin_off = (int)a_bytes;
  pl->cc_off = (int)(a_bytes + fin_bytes);
  pl->flag_off = (int)(a_bytes + fin_bytes + cc_region_bytes(a));
  pl->lds_bytes = bytes;
  return true;
}
bool plan(const FwdArgs& a, PipePlan* best) {
  double best_cost = 0;
  bool found = false;
  // a tuned tile (cp4_tune_forward) replaces the cost model
  if (a.tune_th > 0 && a.tune_lgwt >= 6 && a.tune_lgwt <= 8)
    return a.tune_th <= a.H && layout_tiled(a, a.tune_th, a.tune_lgwt, best);
  const int cus = num_compute_units();
  for (int lgWt = 6; lgWt <= 8; ++lgWt)
    for (int TH = 1; TH <= a.H; ++TH) {
      PipePlan pl;
      if (!layout_tiled(a, TH, lgWt, &pl)) break;
      const double rounds = (pl.nWG + cus - 1) / cus;
      // cells read per channel and cells written per channel, with the tiles of the
      // last column counted whole
      const double cost = rounds * ((double)(TH + a.Y - 1) * (pl.Wt + a.Y - 1) * a.Cin +
                                    (double)TH * pl.Wt * a.Cout + kTileStartCost);
      // on equal cost (1x1 filters: no halo) the larger tile: fewer workgroups
      if (!found || cost <= best_cost) {
        best_cost = cost;
        *best = pl;
        found = true;
      }
    }
  if (found) choose_output_slices(a, cus, best);
  return found;
}
#endif
#if !defined(CP4_PIPE_TILED) && !defined(CP4_PIPE_STRIDED)
bool plan(const FwdArgs& a, PipePlan* best) {
  double best_cost = 0;
  bool found = false;
  // a tuned strip height (cp4_tune_forward) replaces the cost model
  if (a.tune_th > 0) return a.tune_th <= a.H && layout(a, a.tune_th, best);
  const int cus = num_compute_units();
  for (int TH = 1; TH <= a.H; ++TH) {
    PipePlan pl;
    if (!layout(a, TH, &pl)) break;
    const double rounds = (pl.nWG + cus - 1) / cus;
    double cost = rounds * ((double)(TH + a.Y - 1) * a.Cin + (double)TH * a.Cout +
                            kTileStartCost / a.W);
    // Strips that do not end on a 128-byte line of y share that line with their
    // neighbour (two partial writes) and start with a partly masked group.
    if (((long)TH * a.W * kIoBytes) % 128 != 0 && TH < a.H) cost *= kUnalignedStripCost;
    // on equal cost (1x1 filters: no halo rows) the taller strip: fewer workgroups
    if (!found || cost <= best_cost) {
      best_cost = cost;
      *best = pl;
      found = true;
    }
  }
  if (found) choose_output_slices(a, cus, best);
  return found;
}
#endif

template <int FS, int CPQ, int KR, int NQ = 4>
hipError_t launch_as(const FwdArgs& a, const PipePlan& pl, hipStream_t st) {
#ifdef CP4_PIPE_IO16
  // even rows, activations on a 4-byte boundary: the producers load pixel pairs
  if ((a.W & 1) == 0 && (reinterpret_cast<uintptr_t>(a.x) & 3) == 0) {
    const void* fp = reinterpret_cast<const void*>(fwd_pipe_kernel<FS, CPQ, KR, NQ, true>);
    hipError_t ep = hipFuncSetAttribute(fp, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)pl.lds_bytes);
    if (ep != hipSuccess) return ep;
    fwd_pipe_kernel<FS, CPQ, KR, NQ, true>
        <<<dim3(8u * ((pl.nWG + 7) / 8), pl.kparts), kThreads, pl.lds_bytes, st>>>(a, pl);
    return hipGetLastError();
  }
#endif
  const void* fn = reinterpret_cast<const void*>(fwd_pipe_kernel<FS, CPQ, KR, NQ>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)pl.lds_bytes);
  if (e != hipSuccess) return e;
  const dim3 grid(8u * ((pl.nWG + 7) / 8), pl.kparts);
  fwd_pipe_kernel<FS, CPQ, KR, NQ><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}

template <int FS>
hipError_t launch_cpq(const FwdArgs& a, const PipePlan& pl, hipStream_t st) {
  const int cpq = (a.Cin + 63) >> 6;             // 16-channel chunks per channel quarter
  switch (cpq) {
    case 1: return launch_as<FS, 1, 1>(a, pl, st);
    case 2: return launch_as<FS, 2, 2>(a, pl, st);
    case 3: return launch_as<FS, 3, 1>(a, pl, st);
    case 4: return launch_as<FS, 4, 2>(a, pl, st);
    default:                                      // factor fragments in LDS
      return (cpq & 1) ? launch_as<FS, 0, 1>(a, pl, st) : launch_as<FS, 0, 2>(a, pl, st);
  }
}

template <int FS>
hipError_t launch_fs(const FwdArgs& a, const PipePlan& pl, hipStream_t st) {
  // Up to 16 input channels (one chunk): no channel split - every producer wave
  // contracts a whole block of its own, eight blocks per round, nothing to chain.
  // (With 17-64 channels the four-way split is the faster one: C2 7.3 us against
  // 8.1 us; a wave would run its 2-4 chunks one after the other.)
  if (a.Cin <= 16) return launch_as<FS, 1, 1, 1>(a, pl, st);
  // On planes of many blocks the waves' arithmetic bounds the sweep, not the
  // latency of one block, and the split's four chained LDS accumulations per block
  // are half of the producers' instructions at 17-64 channels: there, too, every
  // producer wave contracts whole blocks (N32 C32 112x112 R16: 63 -> 47 us).
  if (a.Cin <= 64 && pl.nblk >= kWholeBlockMin) {
    switch ((a.Cin + 15) >> 4) {
      case 2: return launch_as<FS, 2, 2, 1>(a, pl, st);
      case 3: return launch_as<FS, 3, 1, 1>(a, pl, st);
      default: return launch_as<FS, 4, 2, 1>(a, pl, st);
    }
  }
  return launch_cpq<FS>(a, pl, st);
}

}  // namespace

#if defined(CP4_PIPE_STRIDED)
#define fwd_pipe_supported fwd_pipe_strided_supported
#define fwd_pipe_launch fwd_pipe_strided_launch
#elif defined(CP4_PIPE_TAPS2D)
#define fwd_pipe_supported fwd_pipe_taps2d_supported
#define fwd_pipe_launch fwd_pipe_taps2d_launch
#elif defined(CP4_PIPE_TILED) && defined(CP4_PIPE_EPILOGUE)
#define fwd_pipe_supported fwd_pipe_tiled_epi_supported
#define fwd_pipe_launch fwd_pipe_tiled_epi_launch
#elif defined(CP4_PIPE_TILED)
#define fwd_pipe_supported fwd_pipe_tiled_supported
#define fwd_pipe_launch fwd_pipe_tiled_launch
#elif defined(CP4_PIPE_RANKPASS)
#define fwd_pipe_supported fwd_pipe_rankpass_supported
#define fwd_pipe_launch fwd_pipe_rankpass_launch
#elif defined(CP4_PIPE_IO16) && CP4_PIPE_IO16 == 2
#define fwd_pipe_supported fwd_pipe_iof16_supported
#define fwd_pipe_launch fwd_pipe_iof16_launch
#elif defined(CP4_PIPE_IO16)
#define fwd_pipe_supported fwd_pipe_io16_supported
#define fwd_pipe_launch fwd_pipe_io16_launch
#elif defined(CP4_PIPE_EPILOGUE)
#define fwd_pipe_supported fwd_pipe_epi_supported
#define fwd_pipe_launch fwd_pipe_epi_launch
#endif

#ifdef CP4_PIPE_STRIDED
// Even and rectangular filters up to 7 taps a side run as the square window of the next odd
// size: FwdArgs::ty / tx keep the filter's own rows and columns (the plane holds the rows
// ty taps reach; the taps past ty / tx weigh nothing), Y = X the window.
FwdArgs in_window(const FwdArgs& a) {
  FwdArgs b = a;
  if (a.ty || a.tx) return b;
  const int m = a.Y > a.X ? a.Y : a.X;
  if (m > 7 || (a.Y == a.X && (a.Y & 1))) return b;
  b.ty = a.Y;
  b.tx = a.X;
  b.Y = b.X = m | 1;
  return b;
}
#endif

bool fwd_pipe_supported(const FwdArgs& a_in) {
#ifdef CP4_PIPE_STRIDED
  const FwdArgs a = in_window(a_in);
  if (a.ty > a.Y || a.tx > a.X || a.ty < 0 || a.tx < 0) return false;
#else
  const FwdArgs& a = a_in;
#endif
  if (a.R > kRP || a.Cin > 768) return false;
#ifndef CP4_PIPE_PASSES
  if (a.accumulate || a.ldf || a.ldx) return false;   // only the rank-pass, strided and 2-D-tap builds have these
#endif
  if (!fits_int_indexing(a.N, a.H, a.W)) return false;
#ifdef CP4_PIPE_STRIDED
  // the caller fills in the whole geometry; every output row reads at least one image row
  if (a.sh < 1 || a.sw < 1 || a.Ho < 1 || a.Wo < 1 || a.pt < 0 || a.pl < 0) return false;
  if (!fits_int_indexing(a.N, a.Ho, a.Wo)) return false;
  if ((size_t)a.Cout * a.Ho * a.Wo * sizeof(io_t) >= (1ull << 31)) return false;
#else
  if (a.sh) return false;                        // only the strided build takes a geometry
#endif
  if ((size_t)a.Cin * a.H * a.W * sizeof(io_t) >= (1ull << 31)) return false;   // buffer offsets
  if (a.Y != a.X || !(a.Y == 1 || a.Y == 3 || a.Y == 5 || a.Y == 7)) return false;
#ifdef CP4_PIPE_TAPS2D
  if (!a.taps2d || a.Y > 3) return false;        // 4 * Y * X weights per wave in registers
#endif
  PipePlan pl;
  return plan(a, &pl);
}

#if !defined(CP4_PIPE_STRIDED) && !defined(CP4_PIPE_TAPS2D) && !defined(CP4_PIPE_TILED) && \
    !defined(CP4_PIPE_RANKPASS) && !defined(CP4_PIPE_IO16) && !defined(CP4_PIPE_EPILOGUE)
// What the planner gives a shape as whole-row strips: rows per strip and
// workgroups (the variant choice weighs them against tiles on wide planes).
bool fwd_pipe_strip_plan(const FwdArgs& a, int* rows, int* workgroups) {
  PipePlan pl;
  if (!fwd_pipe_supported(a) || !plan(a, &pl)) return false;
  *rows = pl.TH;
  *workgroups = pl.nWG * pl.kparts;
  return true;
}
#endif

hipError_t fwd_pipe_launch(const FwdArgs& a_in, hipStream_t st) {
#ifdef CP4_PIPE_STRIDED
  const FwdArgs a = in_window(a_in);
#else
  const FwdArgs& a = a_in;
#endif
  PipePlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
  pl.split2 = a.tune_split2 != 1;               // 0: the kernel's own rule, 1: off
  pl.own = own_groups_wanted(a);
  pl.spin_limit = a.spin_limit > 0 ? a.spin_limit : kSpinLimit;
#ifdef CP4_DEBUG_PHASES
  pl.dbg = debug_stamp_buffer();
#endif
  switch (a.Y) {
    case 1: return launch_fs<1>(a, pl, st);
    case 3: return launch_fs<3>(a, pl, st);
#ifdef CP4_PIPE_TAPS2D
    default: return hipErrorInvalidValue;          // larger filters: the weights would spill
#else
    case 5: return launch_fs<5>(a, pl, st);
    default: return launch_fs<7>(a, pl, st);
#endif
  }
}

}  // namespace cp4
