// Fused forward / backward-data kernel for ranks 33 - 64 in one pass: the producer /
// consumer strip kernel (fwd_mfma_pipe.hip) with a 64-rank A plane.
//
// Two passes of 32 ranks read x twice and read y back once; here x is read once and
// y written once.  What changes against the 32-rank kernel:
//
//   producers (waves 0-7): all eight work on the same 32-pixel block, wave w on
//              channel eighth w (up to 256 input channels: 32 a wave, whose slice of
//              the input factor for BOTH 32-rank tiles sits in registers, pre-split -
//              48 registers, what a channel quarter of one tile takes there).  A chunk of
//              x is split once and multiplied into two accumulators.  The eight partial
//              sums of a block are added into LDS in fixed order (an LDS word per block
//              counts the eighths done; 8 publishes the block), so the sum is
//              deterministic.
//   consumers (waves 8-15): the tap step of a 64-pixel group takes two rank quads per
//              wave (w and w + 8), the contraction of a wave's 32-channel block runs
//              over three or four 16-rank chunks.  The fragment tiles hold 48 or 64
//              ranks (18 or 24 KB); where three of them would leave the plane too few
//              rows two rotate, and a wave then starts the next group's taps only after
//              its own contraction.
//
// A 64-rank plane of a whole strip plus halo would leave a strip four rows (56-pixel
// rows), so the plane is a ring of L cells per rank quad: plane cell c lives at c mod L,
// the producers overwrite a block's cells once every tap step that reads them has been
// done by all consumer waves (the arrival counters say so), and the strip can be as tall
// as the grid wants.  A tap step reads a span of at most (63 + (FS-1)(W+1) + pad) / 32 + 2
// blocks; with L at least three blocks more the producers always have room to run ahead
// of the step the consumers wait for, so the two kinds of wait cannot lock each other
// (all waits stay bounded as well).  Where the whole plane fits, L covers it and nothing
// wraps.
//
// Exact-split arithmetic, flat pixel index, sweep directions, waits and their bounds
// are those of fwd_mfma_pipe.hip.  3x3 and 1x1 filters (two quads of larger filters'
// tap weights do not fit the scalar registers), stride 1.  Honours FwdArgs::ldf, ldx and
// accumulate (rank tiles of 64 beyond 64 ranks).
// Arithmetic follows the reassociated form of Cuda_kernels/cp4Conv2dForward.cu:84-133
// (backward-data: cp4Conv2dBackwardData.cu:57-108 through swapped factors and flipped
// taps).
#include <cstdlib>
#include <type_traits>

#include "cp4_internal.h"
#include "split_bf16.h"
#include "pipe_wait.h"

namespace cp4 {
namespace {

using namespace split;
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 1024;
constexpr int kProd = 8, kCons = 8;          // producer / consumer waves (4 per SIMD in all)
constexpr size_t kLdsLimit = 160 * 1024;
constexpr int kMaxBlk = 128;                 // per-block progress words in LDS
constexpr int kSpinLimit = 1 << 19;          // default bound of a wait
// the planner's terms, as in fwd_mfma_pipe.hip: what a workgroup spends before its
// pipeline runs, in channel-cells; strips that do not end on a 128-byte line of y;
// two fragment tiles instead of three (the tap step of a group waits for the
// contraction of the one before)
constexpr double kTileStartCost = 50000.0;
constexpr double kUnalignedStripCost = 1.12;
constexpr double kTwoTileCost = 1.06;

struct Plan64 {
  int TH, strips, nWG;
  int nblk;          // 32-pixel producer blocks of a workgroup's plane
  int L;             // cells of the plane's ring per rank quad, a multiple of 32
  int QA;            // distance between rank quads of the plane in LDS, in cells
  int ntiles;        // fragment tiles in rotation: 3 or 2
  int cc_off, flag_off;
  size_t lds_bytes;
  int kparts, kslice;   // output-channel slices (blockIdx.y), as in fwd_mfma_pipe.hip
  int spin_limit;
};

// FS: filter size; CPQ: 16-channel chunks per channel eighth (1: up to 128 input
// channels, 2: up to 256); NCH: 16-rank chunks (3: up to 48 ranks, 4: up to 64).
template <int FS, int CPQ, int NCH>
__global__ __launch_bounds__(kThreads) void fwd_pipe64_kernel(FwdArgs a, Plan64 pl) {
  extern __shared__ float lds[];
  // A plane: [rank quad][QA cells] of four fp32 each
  f32x4* As4 = reinterpret_cast<f32x4*>(lds);
  unsigned char* ldsb = reinterpret_cast<unsigned char*>(lds);
  unsigned char* Cb = ldsb + pl.cc_off;      // fragment tiles
  // [0..kMaxBlk) eighths done per block (sweep order), then 4 consumer arrival
  // counters, then (at + 8) the abort word
  int* flags = reinterpret_cast<int*>(ldsb + pl.flag_off);
  constexpr int NQD = 4 * NCH;               // rank quads of the plane
  constexpr int PS = NCH * 4 * 512;          // bytes of one part of a fragment tile
  constexpr int kCc = 3 * PS;                // ... and of a tile

  const int per = (pl.nWG + 7) >> 3;
  const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);         // XCD-contiguous strip order
  if (t >= pl.nWG) return;
  const int n = t / pl.strips, strip = t - n * pl.strips, h0 = strip * pl.TH;
  const bool rev = strip & 1;                    // odd strips sweep bottom-up

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const WaitCtx wx{pl.spin_limit, flags + kMaxBlk + 8, a.fault, t, wave};
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin;
  const int CoutAll = a.Cout;
  const int k0 = pl.kparts > 1 ? (int)blockIdx.y * pl.kslice : 0;
  const int Cout = pl.kparts > 1 ? min(pl.kslice, CoutAll - k0) : CoutAll;
  const int QA = pl.QA;
  const int ldf = a.ldf ? a.ldf : R;             // row stride of the factor matrices
  const int rows = min(pl.TH, H - h0);
  const int nvalid = rows * W;                   // output pixels inside the image
  // 64-pixel output groups start `gshift` pixels before the strip so that their
  // boundaries fall on 128-byte lines of y
  const int gshift = (h0 * W) & 31;
  const int ngroups = (nvalid + gshift + 63) >> 6;
  const int nkb = (Cout + 31) >> 5;
  const int qbase = (h0 - a.pad) * W;            // global flat pixel of LDS column 0
  // The plane covers the strip's own rows (the image's last strip may have fewer than
  // TH): every block of the sweep is then read by some tap step, which the ring's
  // producer-side wait relies on.
  const int QLEN = (rows + FS - 1) * W;
  const int nblk = (QLEN + 31) >> 5;             // 32-pixel producer blocks
  const bool backoff = nblk >= 4;                // growing naps in the spin waits
  const int L = pl.L, NBL = L >> 5;              // the plane's ring: cells, blocks
  const int reach = (FS - 1) * (W + 1);          // how far past a pixel its taps read in A
  int* arrivals = flags + kMaxBlk;               // [4] tap-step arrivals, slot = step & 3
  // Sweep indices of the first and the last block the taps of step i touch: the taps of
  // pixel p read plane cells p - pad .. p + (FS-1)*(W+1) - pad.
  auto span_of = [&](int i, int& lo, int& hi) {
    const int g = rev ? ngroups - 1 - i : i;
    int last = max(64 * g - gshift + 63 + reach, 0) >> 5;
    if (last > nblk - 1) last = nblk - 1;
    int first = max(64 * g - gshift - a.pad, 0) >> 5;
    if (first > nblk - 1) first = nblk - 1;
    lo = rev ? nblk - 1 - last : first;
    hi = rev ? nblk - 1 - first : last;
  };

  if (tid < kMaxBlk + 16) flags[tid] = 0;
  __syncthreads();

  if (wave < kProd) {
    // =========================== producers ==================================
    const int cq = wave;                           // channel eighth
    // lane's channel 16*(CPQ*cq + chunk) + 8*hi + e (channels past Cin count as zero:
    // their factor rows are, and x reads there return 0)
    const int cg0 = 16 * CPQ * cq + 8 * hi;
    // x through a buffer descriptor over this image's channels: (base) + (lane
    // offset) + (scalar offset), the sum range-checked - reads past the last channel
    // return 0
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(a.x) + (size_t)n * (a.ldx ? (size_t)a.ldx : (size_t)Cin * HW), 0,
        Cin * HW * 4, 0x00020000);
    const unsigned sbase = (unsigned)(16 * CPQ * cq) * (unsigned)HW * 4u;
    // factor slices of both rank tiles: lane holds rank l32 + 32*rb
    u32x4 fh[2][CPQ], fm[2][CPQ], fl[2][CPQ];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int c = 0; c < CPQ; ++c) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[e] = (l32 + 32 * rb < R && cg0 + 16 * c + e < Cin)
                     ? a.Fin[(size_t)(cg0 + 16 * c + e) * ldf + l32 + 32 * rb]
                     : 0.f;
        split8(v, fh[rb][c], fm[rb][c], fl[rb][c]);
      }
    // Block of round r: whether the lane's pixel exists, and the lane's byte offset
    // (clamped pixel, channel 8*hi).
    auto geom = [&](int r, bool& valid) -> unsigned {
      const int b = rev ? nblk - 1 - r : r;
      const int qa = 32 * b + l32;
      const int q = qbase + qa;
      valid = q >= 0 && q < HW && qa < QLEN;
      const int qc = q < 0 ? 0 : (q > HW - 1 ? HW - 1 : q);
      return (unsigned)(8 * hi * HW + qc) * 4u;
    };
    int bm = (rev ? nblk - 1 : 0) % NBL;           // the round's plane block modulo the ring
    int istar = 0;                                 // last tap step that reads the block about to go
    auto ld_chunk = [&](float (&dst)[8], unsigned voff, int chunk) {   // chunk < CPQ
      const unsigned soff = sbase + (unsigned)(16 * chunk) * (unsigned)HW * 4u;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        dst[e] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(xrs, voff, soff + (unsigned)e * HW * 4u, 0));
    };
    // ring of two chunks: the steps (round, chunk) in order, step s in slot s & 1
    float xb[2][8];
    {
      bool v0;
      ld_chunk(xb[0], geom(0, v0), 0);
      if (CPQ == 2) ld_chunk(xb[1], geom(0, v0), 1);
      else ld_chunk(xb[1], geom(nblk > 1 ? 1 : 0, v0), 0);
    }
    // one round: the block's CPQ chunks (the first in ring slot S0), then the sum
    auto round = [&](int r, auto s0_c) {
      constexpr int S0 = decltype(s0_c)::value;
      bool valid, validn;
      geom(r, valid);
      const int qa = 32 * bm + l32;                // the lane's cell in the ring
      // the slot freed by a step is refilled with the step two further on: the
      // same chunk of the next round (two chunks a round) or the round after it
      const int rn = r + (CPQ == 2 ? 1 : 2);
      const unsigned xpn = geom(rn < nblk ? rn : nblk - 1, validn);
      f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
#pragma unroll
      for (int ch = 0; ch < CPQ; ++ch) {
        const int slot = (S0 + ch) & 1;
        u32x4 xh, xm, xl;
        split8(xb[slot], xh, xm, xl);
        acc0 = mfma_split(fh[0][ch], fm[0][ch], fl[0][ch], xh, xm, xl, acc0);
        acc1 = mfma_split(fh[1][ch], fm[1][ch], fl[1][ch], xh, xm, xl, acc1);
        ld_chunk(xb[slot], xpn, ch);
        // keep use-then-refill order per chunk so two chunks stay in flight
        __builtin_amdgcn_sched_barrier(0);
      }
      // add this eighth's partial sums after the lower eighths
      int* bf = &flags[r];
      // accumulator elements 4*g ... 4*g + 3 of tile rb are ranks 32*rb + 8*g + 4*hi ...:
      // rank quad 8*rb + 2*g + hi
      f32x4* dst = As4 + (size_t)hi * QA + qa;
      if (cq == 0) {
        if (r >= NBL) {
          // these cells still hold block r - NBL of the sweep: every tap step that
          // reads it must have been done by all consumer waves
          const int jb = r - NBL;
          for (;;) {
            int lo, hi2;
            if (istar + 1 >= ngroups) break;
            span_of(istar + 1, lo, hi2);
            if (lo > jb) break;
            ++istar;
          }
          wait_ge(&arrivals[istar & 3], kCons * ((istar >> 2) + 1), backoff, wx, 8);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          dst[(2 * g) * QA] = valid ? f32x4{acc0[4 * g], acc0[4 * g + 1], acc0[4 * g + 2], acc0[4 * g + 3]}
                                    : f32x4{0.f, 0.f, 0.f, 0.f};
          if (8 + 2 * g < NQD)
            dst[(8 + 2 * g) * QA] =
                valid ? f32x4{acc1[4 * g], acc1[4 * g + 1], acc1[4 * g + 2], acc1[4 * g + 3]}
                      : f32x4{0.f, 0.f, 0.f, 0.f};
        }
      } else {
        wait_ge(bf, cq, backoff, wx, 1);
        // read, add, write two quads at a time: one LDS round trip per pair
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          f32x4 old[2];
#pragma unroll
          for (int g = 0; g < 2; ++g) old[g] = dst[(2 * (2 * half + g)) * QA];
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            const int v = 4 * (2 * half + g);
            dst[(2 * (2 * half + g)) * QA] =
                valid ? old[g] + f32x4{acc0[v], acc0[v + 1], acc0[v + 2], acc0[v + 3]} : old[g];
          }
        }
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          if (8 + 4 * half >= NQD) break;          // (48 ranks: quads 8 ... 11 only)
          f32x4 old[2];
#pragma unroll
          for (int g = 0; g < 2; ++g) old[g] = dst[(8 + 2 * (2 * half + g)) * QA];
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            const int v = 4 * (2 * half + g);
            dst[(8 + 2 * (2 * half + g)) * QA] =
                valid ? old[g] + f32x4{acc1[v], acc1[v + 1], acc1[v + 2], acc1[v + 3]} : old[g];
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane == 0) __hip_atomic_store(bf, cq + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      if (rev) bm = bm == 0 ? NBL - 1 : bm - 1;
      else bm = bm + 1 == NBL ? 0 : bm + 1;
    };
    constexpr std::integral_constant<int, 0> s0{};
    constexpr std::integral_constant<int, 1> s1{};
    if (CPQ == 2) {
      for (int r = 0; r < nblk; ++r) round(r, s0);
    } else {
      for (int r = 0; r < nblk; r += 2) {
        round(r, s0);
        if (r + 1 < nblk) round(r + 1, s1);
      }
    }
  } else {
    // =========================== consumers ==================================
    const int wc = wave - kProd;                   // 0..7: first rank quad in the tap step
    const bool second = wc + 8 < NQD;              // ... and quad wc + 8
    // Output-factor fragment of this wave's 32-channel block (reloaded per block only
    // when there are more blocks than consumer waves): lane holds row 32*kb + l32,
    // ranks 16*c + 8*hi + e.
    u32x4 fkh[NCH], fkm[NCH], fkl[NCH];
    auto load_fk = [&](int kb) {
      const int k = 32 * kb + l32;
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int r = 16 * c + 8 * hi + e;
          v[e] = (k < Cout && r < R) ? a.Fout[(size_t)(k0 + k) * ldf + r] : 0.f;
        }
        split8(v, fkh[c], fkm[c], fkl[c]);
      }
    };
    const bool fk_cached = nkb <= kCons;
    if (fk_cached && wc < nkb) load_fk(wc);
    // Tap weights of this wave's two rank quads (wave-uniform values).
    float fh[2][4][FS], fw[2][4][FS];
#pragma unroll
    for (int qi = 0; qi < 2; ++qi)
#pragma unroll
      for (int rr = 0; rr < 4; ++rr)
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          const int tap = a.flip ? FS - 1 - j : j, r = 4 * (wc + 8 * qi) + rr;
          fh[qi][rr][j] = r < R ? a.FH[tap * ldf + r] : 0.f;
          fw[qi][rr][j] = r < R ? a.FW[tap * ldf + r] : 0.f;
        }
    float* yn = a.y + ((size_t)n * CoutAll + k0) * HW + (size_t)h0 * W;
    const bool accumulate = a.accumulate != 0;
    const bool pair_stores =                       // one store per pixel pair is legal
        ((W | HW) & 1) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 7) == 0;

    int frontier = 0;                              // blocks [0, frontier) of the sweep are complete
    auto need_of = [&](int i) {
      int lo, hi2;
      span_of(i, lo, hi2);
      return hi2;
    };
    // Non-blocking: advance the frontier over finished blocks, say whether step i
    // could run its taps now.
    auto ready = [&](int i) {
      const int need = need_of(i);
      while (frontier <= need &&
             __hip_atomic_load(&flags[frontier], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) >= kProd)
        ++frontier;
      return frontier > need;
    };
    auto await_blocks = [&](int i) {
      const int need = need_of(i);
      while (frontier <= need) {
        wait_ge(&flags[frontier], kProd, backoff, wx, 2);
        ++frontier;
      }
    };
    // The taps of rank quad q at the lane's pixel of group g, split exactly and
    // written into fragment tile cb.
    // Where the taps of pixel group g read the ring: the cell of the lane's pixel row
    // for every tap row, and per tap column the (clamped) column and whether it lies
    // inside the image.
    struct TapPos {
      int roff[FS];
      int off[FS];
      bool in[FS];
    };
    auto tap_pos = [&](int g) {
      TapPos tp;
      const int p = max(64 * g - gshift + lane, 0);      // lanes before the strip: any valid column
      const int h = p / W;
      const int w = p - h * W;
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        const int ww = w + j - a.pad;
        tp.in[j] = ww >= 0 && ww < W;
        tp.off[j] = ww < 0 ? 0 : (ww >= W ? W - 1 : ww);   // clamped: weight is 0 there
      }
      tp.roff[0] = (int)((unsigned)(h * W) % (unsigned)L);
#pragma unroll
      for (int ti = 1; ti < FS; ++ti) {
        const int nx = tp.roff[ti - 1] + W;              // (W <= L)
        tp.roff[ti] = nx >= L ? nx - L : nx;
      }
      return tp;
    };
    auto tap_quad = [&](const TapPos& tp, int q, const float (&wa)[4][FS], const float (&wb)[4][FS],
                        unsigned char* cb) {
      // (a quad past the last rank has zero weights and writes zeros)
      const bool live = 4 * q < R;
      const f32x4* ab = As4 + (size_t)q * QA;
      f32x4 av[FS][FS];
#pragma unroll
      for (int ti = 0; ti < FS; ++ti)
#pragma unroll
        for (int j = 0; j < FS; ++j) {
          const int c = tp.roff[ti] + tp.off[j];
          av[ti][j] = ab[c >= L ? c - L : c];
        }
      float o[4];
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        float s = 0.f;
#pragma unroll
        for (int ti = 0; ti < FS; ++ti) {
          float hs = 0.f;
#pragma unroll
          for (int j = 0; j < FS; ++j) hs += (tp.in[j] ? wb[rr][j] : 0.f) * av[ti][j][rr];
          s += wa[rr][ti] * hs;
        }
        o[rr] = live ? s : 0.f;
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
      // plane ((part*NCH + chunk)*2 + hi)*2 + parity, 512 B each; entry lane >> 1;
      // this quad is the low or high 8 bytes of the 16-byte entry
      unsigned char* dst = cb + ((((q >> 2) * 2 + ((q >> 1) & 1)) * 2 + (lane & 1)) * 512) +
                           (lane >> 1) * 16 + (q & 1) * 8;
      *reinterpret_cast<u32x2*>(dst) = ph;
      *reinterpret_cast<u32x2*>(dst + PS) = pm;
      *reinterpret_cast<u32x2*>(dst + 2 * PS) = pl2;
    };
    auto taps = [&](int i, unsigned char* cb) {
      const int g = rev ? ngroups - 1 - i : i;
      await_blocks(i);
      const TapPos tp = tap_pos(g);
      tap_quad(tp, wc, fh[0], fw[0], cb);
      if (second) tap_quad(tp, wc + 8, fh[1], fw[1], cb);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      if (lane == 0)
        __hip_atomic_fetch_add(&arrivals[i & 3], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    // Contraction ranks -> the 32 output channels of block kb for pixel group g from
    // fragment tile cb, stores.
    auto contract_block = [&](const unsigned char* cb, int g, int kb) {
      f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        const unsigned char* bp = cb + ((c * 2 + hi) * 2) * 512 + l32 * 16;
        const u32x4 b0h = *reinterpret_cast<const u32x4*>(bp);
        const u32x4 b1h = *reinterpret_cast<const u32x4*>(bp + 512);
        const u32x4 b0m = *reinterpret_cast<const u32x4*>(bp + PS);
        const u32x4 b1m = *reinterpret_cast<const u32x4*>(bp + PS + 512);
        const u32x4 b0l = *reinterpret_cast<const u32x4*>(bp + 2 * PS);
        const u32x4 b1l = *reinterpret_cast<const u32x4*>(bp + 2 * PS + 512);
        acc0 = mfma_split(fkh[c], fkm[c], fkl[c], b0h, b0m, b0l, acc0);
        acc1 = mfma_split(fkh[c], fkm[c], fkl[c], b1h, b1m, b1l, acc1);
        __builtin_amdgcn_sched_barrier(0);     // one chunk's fragments live at a time
      }
      // store rows: uniform row base + one 32-bit lane offset
      const int p = 64 * g - gshift + 2 * l32;       // lane's pixel pair p, p + 1
      const bool pin0 = p >= 0 && p < nvalid, pin1 = p + 1 >= 0 && p + 1 < nvalid;
      float* rowbase = yn + (size_t)(32 * kb) * HW;
      if (pair_stores) {
        // W and H*W even, y aligned to a pair: p is even and the pair is one store
        if (pin0) {
          const unsigned lofs = (unsigned)(4 * hi * HW + p);
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int kk = 8 * (v >> 2) + (v & 3);         // + 4*hi is in lofs
            if (32 * kb + kk + 4 * hi < Cout) {
              float2* dst = reinterpret_cast<float2*>(rowbase + (size_t)kk * HW + lofs);
              float2 o;
              o.x = acc0[v];
              o.y = acc1[v];
              if (accumulate) {                      // a later pass: y += (wave-uniform)
                const float2 old = *dst;
                o.x += old.x;
                o.y += old.y;
              }
              *dst = o;
            }
          }
        }
      } else {
        // odd widths or planes: the two pixels are stored and bounded one by one
        const long lofs = (long)(4 * hi) * HW + p;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kk = 8 * (v >> 2) + (v & 3);
          if (32 * kb + kk + 4 * hi < Cout) {
            float* rp = rowbase + (size_t)kk * HW + lofs;
            if (pin0) rp[0] = accumulate ? rp[0] + acc0[v] : acc0[v];
            if (pin1) rp[1] = accumulate ? rp[1] + acc1[v] : acc1[v];
          }
        }
      }
    };

    // Fragment tiles in rotation.  Iteration i: once every consumer wave has arrived
    // for step i, contract step i and do the tap step i + 1.  With three tiles the
    // tile written by step i + 1 was last read by step i - 2, which every wave
    // finished before it arrived for step i: the taps may go first when their blocks
    // are there.  With two tiles it was last read by step i - 1: every wave signals
    // its arrival for step i only after its own contraction of step i - 1 (the taps
    // never go first), so after the wait the tile is free as well.
    const int NT = pl.ntiles;
    taps(0, Cb);
    for (int i = 0; i < ngroups; ++i) {
      const int g = rev ? ngroups - 1 - i : i;
      wait_ge(&arrivals[i & 3], kCons * ((i >> 2) + 1), backoff, wx, 7);
      unsigned char* cb_next = Cb + ((i + 1) % NT) * kCc;
      const bool early = NT == 3 && i + 1 < ngroups && ready(i + 1);
      if (early) taps(i + 1, cb_next);
      const unsigned char* cb = Cb + (i % NT) * kCc;
      for (int kb = wc; kb < nkb; kb += kCons) {
        if (!fk_cached) load_fk(kb);
        contract_block(cb, g, kb);
      }
      if (i + 1 < ngroups && !early) taps(i + 1, cb_next);
    }
  }
}

int round_up(int v, int m) { return (v + m - 1) / m * m; }
int rank_chunks(const FwdArgs& a) { return a.R <= 48 ? 3 : 4; }

bool layout(const FwdArgs& a, int TH, int ntiles, Plan64* pl) {
  const long QLEN = (long)(TH + a.Y - 1) * a.W;
  // the taps of the last (partly filled) 64-pixel group may read past QLEN; the
  // groups start up to 31 pixels before the strip, so they end up to 31 + 63 past it
  const long whole = round_up(TH * a.W + 31, 64) + (long)(a.Y - 1) * (a.W + 1) + 1;
  const int nch = rank_chunks(a);
  const size_t cc_bytes = (size_t)ntiles * nch * 12 * 512;
  const size_t tail = (kMaxBlk + 16) * sizeof(int);
  if ((QLEN + 31) / 32 + 1 > kMaxBlk || cc_bytes + tail >= kLdsLimit) return false;
  // ring blocks the LDS leaves room for; the whole plane where it fits, else a ring of
  // at least a tap step's span of blocks plus three
  const long room = (long)((kLdsLimit - cc_bytes - tail) / ((size_t)(4 * nch) * 16)) - 8;
  const long nbl_max = room / 32, nbl_whole = (whole + 31) / 32;
  const long span = (63 + (long)(a.Y - 1) * (a.W + 1) + a.pad) / 32 + 2;
  long nbl = nbl_whole;
  if (nbl_max < nbl_whole) {
    nbl = nbl_max;
    if (nbl < span + 3 || 32 * nbl < a.W) return false;
  }
  const long QA = 32 * nbl + 8;
  const size_t a_bytes = (size_t)(4 * nch) * QA * 16;
  const size_t bytes = a_bytes + cc_bytes + tail;
  if (bytes > kLdsLimit) return false;
  pl->L = (int)(32 * nbl);
  pl->TH = TH;
  pl->nblk = (int)((QLEN + 31) / 32);
  pl->strips = (a.H + TH - 1) / TH;
  pl->nWG = a.N * pl->strips;
  pl->QA = (int)QA;
  pl->ntiles = ntiles;
  pl->cc_off = (int)a_bytes;
  pl->flag_off = (int)(a_bytes + cc_bytes);
  pl->lds_bytes = bytes;
  pl->kparts = 1;
  pl->kslice = 0;
  return true;
}

// Strips that fill at most half the chip, four or more blocks of 32 output channels: as
// many slices of at least two blocks as bring the grid up to the compute units.
void choose_output_slices(const FwdArgs& a, int cus, Plan64* pl) {
  const int nkb = (a.Cout + 31) / 32;
  if (a.tune_th > 0 || 2 * pl->nWG > cus || nkb < 4) return;
  int parts = cus / pl->nWG;
  if (parts > nkb / 2) parts = nkb / 2;
  if (parts < 2) return;
  const int blocks = (nkb + parts - 1) / parts;     // blocks per slice
  pl->kslice = 32 * blocks;
  pl->kparts = (nkb + blocks - 1) / blocks;
}

bool plan(const FwdArgs& a, Plan64* best) {
  double best_cost = 0;
  bool found = false;
  // a tuned strip height replaces the cost model (three tiles where they fit)
  // (tune_split2 == 1 asks for two fragment tiles)
  if (a.tune_th > 0)
    return a.tune_th <= a.H && ((a.tune_split2 != 1 && layout(a, a.tune_th, 3, best)) ||
                                layout(a, a.tune_th, 2, best));
  const int cus = num_compute_units();
  for (int nt = a.tune_split2 == 1 ? 2 : 3; nt >= 2; --nt)
    for (int TH = 1; TH <= a.H; ++TH) {
      Plan64 pl;
      if (!layout(a, TH, nt, &pl)) break;
      const double rounds = (pl.nWG + cus - 1) / cus;
      double cost = rounds * ((double)(TH + a.Y - 1) * a.Cin + (double)TH * a.Cout +
                              kTileStartCost / a.W);
      if (((long)TH * a.W * 4) % 128 != 0 && TH < a.H) cost *= kUnalignedStripCost;
      if (nt == 2) cost *= kTwoTileCost;
      if (!found || cost < best_cost) {
        best_cost = cost;
        *best = pl;
        found = true;
      }
    }
  if (found) choose_output_slices(a, cus, best);
  return found;
}

template <int FS, int CPQ, int NCH>
hipError_t launch_as(const FwdArgs& a, const Plan64& pl, hipStream_t st) {
  const void* fn = reinterpret_cast<const void*>(fwd_pipe64_kernel<FS, CPQ, NCH>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)pl.lds_bytes);
  if (e != hipSuccess) return e;
  const dim3 grid(8u * ((pl.nWG + 7) / 8), pl.kparts);
  fwd_pipe64_kernel<FS, CPQ, NCH><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}

template <int FS>
hipError_t launch_fs(const FwdArgs& a, const Plan64& pl, hipStream_t st) {
  const bool two = a.Cin > 128, four = rank_chunks(a) == 4;
  if (two) return four ? launch_as<FS, 2, 4>(a, pl, st) : launch_as<FS, 2, 3>(a, pl, st);
  return four ? launch_as<FS, 1, 4>(a, pl, st) : launch_as<FS, 1, 3>(a, pl, st);
}

}  // namespace

bool fwd_pipe64_supported(const FwdArgs& a) {
  if (a.R <= 32 || a.R > 64 || a.Cin > 256) return false;
  if (a.sh || a.dense || a.taps2d || a.bias || a.act) return false;
  if (a.Y != a.X || !(a.Y == 1 || a.Y == 3)) return false;
  if (!fits_int_indexing(a.N, a.H, a.W)) return false;
  if ((size_t)a.Cin * a.H * a.W * sizeof(float) >= (1ull << 31)) return false;   // buffer offsets
  Plan64 pl;
  return plan(a, &pl);
}

bool fwd_pipe64_plan(const FwdArgs& a, int* rows, int* workgroups) {
  Plan64 pl;
  if (!fwd_pipe64_supported(a) || !plan(a, &pl)) return false;
  *rows = pl.TH;
  *workgroups = pl.nWG * pl.kparts;
  return true;
}

hipError_t fwd_pipe64_launch(const FwdArgs& a, hipStream_t st) {
  Plan64 pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
  pl.spin_limit = a.spin_limit > 0 ? a.spin_limit : kSpinLimit;
  return a.Y == 1 ? launch_fs<1>(a, pl, st) : launch_fs<3>(a, pl, st);
}

}  // namespace cp4
