// Fused forward / backward-data kernel on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32) for ranks up to 64.
//
// One workgroup (8 wave64) owns a strip of TH image rows of one image, full
// width.  Each channel plane of a strip plus its halo rows is one contiguous
// run of floats in NCHW, so pixels are handled as a flat index q.
//
//   P0  Fin[Cin,R] -> LDS, zero-padded to RP = 32*RB columns.
//   P1  A[r,q] = sum_c Fin[c,r] x[c,q] for the strip + halo rows.  Each wave
//       owns blocks of 64 consecutive pixels; a lane streams float2 (two
//       pixels) per channel straight from HBM into a ring of kRing registers
//       (kRing channel pairs in flight per lane) and feeds them as the B
//       operand of the MFMA; the A operand is 64 consecutive floats of the
//       LDS copy of Fin.  The accumulators go to LDS as A[r][q]; rows outside
//       the image become 0.
//   P2  the separable taps, VALU out of LDS: a thread owns one (rank, column)
//       pair, walks down the strip's rows keeping the last FS horizontally
//       filtered rows in registers, and writes Cc[r][p].
//   P3  y[k,p] = sum_r Fout[k,r] Cc[r,p]: a wave keeps the Fout fragment of
//       its 32-output-channel block in registers, reads Cc pairs from LDS as
//       the B operand and stores float2 per lane, 256 contiguous bytes per
//       half-wave and output row.
//
// x is read once from HBM (halo rows are shared with the neighbouring strip,
// which the XCD-aware tile order places on the same L2), y is written once,
// and no intermediate leaves the CU.  Arithmetic follows the reassociated form
// of Cuda_kernels/cp4Conv2dForward.cu:84-133 (backward-data:
// cp4Conv2dBackwardData.cu:57-108 through swapped factors and flipped taps).
#include <cstdlib>
#include <type_traits>

#include "cp4_internal.h"
#ifdef CP4_DEBUG_PHASES
#include "cp4_debug.h"
#endif

namespace cp4 {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 512, kWaves = kThreads / 64;
constexpr size_t kLdsLimit = 160 * 1024;     // gfx950 LDS per workgroup

struct StripPlan {
  int TH;       // output rows per strip
  int strips;   // strips per image
  int nWG;      // N * strips
  int QA;       // LDS row stride of A (floats)
  int QC;       // LDS row stride of Cc (floats)
  int QB;       // LDS row stride of B (generic tap path only)
  int padoff;   // leading floats of each B row (>= pad, even)
  int r2_off;   // float offset of the second LDS region
  size_t lds_bytes;
  int phases;   // debug: bit0 P1, bit1 P2, bit2 P3
#ifdef CP4_DEBUG_PHASES
  long long* dbg;
#endif
};

__device__ __forceinline__ f32x16 mfma32(float a, float b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// FS: square filter size known at compile time (1, 3, 5, 7), 0 = any Y, X.
// NS: Cin / 2 known at compile time (P1 fully unrolled), 0 = any even Cin.
template <int RB, int FS, int NS>
__global__ __launch_bounds__(kThreads) void fwd_mfma_strip_kernel(FwdArgs a, StripPlan pl) {
  constexpr int RP = 32 * RB;
  constexpr int kRing = 32 / RB;   // channel pairs in flight per lane
  extern __shared__ float lds[];
  float* As = lds;                 // [RP][QA]: A after P1 (Cc on the generic tap path)
  float* R2 = lds + pl.r2_off;     // Fin tile [Cin][RP] in P1; Cc [RP][QC] (or B) after

  // XCD-aware tile order: workgroup b runs on XCD b % 8; give each XCD a
  // contiguous range of tiles so neighbouring strips share an L2.
  const int per = (pl.nWG + 7) >> 3;
  const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (t >= pl.nWG) return;
  const int n = t / pl.strips, h0 = (t - n * pl.strips) * pl.TH;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#ifdef CP4_DEBUG_PHASES
#define STAMP(i) if (pl.dbg && lane == 0) { pl.dbg[((size_t)t * 8 + wave) * 8 + (i)] = wall_clock64(); pl.dbg[262144 + ((size_t)t * 8 + wave) * 8 + (i)] = clock64(); }
#else
#define STAMP(i)
#endif
  STAMP(0)
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin, Cout = a.Cout;
  const int QA = pl.QA;

  const int rows = min(pl.TH, H - h0);
  const int nvalid = rows * W;               // output pixels of this strip
  const int npo = (nvalid + 63) >> 6;
  const int nkb = (Cout + 31) >> 5;
  const int nitems = nkb * npo;

  // Output-channel factor fragment of a 32-channel block: lane holds
  // Fout[32*kb + l32][2*s + hi].  The block is 32 contiguous rows of Fout, so it
  // is read coalesced into a per-wave LDS staging tile (row stride RP + 1, in
  // the A region while that is free) and picked up from there without bank
  // conflicts; a direct gather would touch 64 cache lines per load.
  float fk[RP / 2];
  int cur_kb = -1;
  auto fk_issue = [&](int kb, float (&v)[RP / 2]) {
    cur_kb = kb;
#pragma unroll
    for (int j = 0; j < RP / 2; ++j) {
      const int idx = lane + 64 * j, kk = idx / RP, r = idx - kk * RP;
      const int k = 32 * kb + kk;
      v[j] = (k < Cout && r < R) ? a.Fout[(size_t)k * R + r] : 0.f;
    }
  };
  auto fk_finish = [&](const float (&v)[RP / 2]) {
    float* stage = As + wave * (32 * (RP + 1));
#pragma unroll
    for (int j = 0; j < RP / 2; ++j) {
      const int idx = lane + 64 * j, kk = idx / RP, r = idx - kk * RP;
      stage[kk * (RP + 1) + r] = v[j];
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int s = 0; s < RP / 2; ++s) fk[s] = stage[l32 * (RP + 1) + 2 * s + hi];
  };
  auto load_fk_staged = [&](int kb) {
    float v[RP / 2];
    fk_issue(kb, v);
    fk_finish(v);
  };
  auto load_fk_gather = [&](int kb) {
    cur_kb = kb;
    const int k = 32 * kb + l32;
#pragma unroll
    for (int s = 0; s < RP / 2; ++s) {
      const int r = 2 * s + hi;
      fk[s] = (k < Cout && r < R) ? a.Fout[(size_t)k * R + r] : 0.f;
    }
  };

  // ---- P1 set-up ----------------------------------------------------------
  const int qbase = (h0 - a.pad) * W;          // global flat pixel of LDS column 0
  const int QLEN = (pl.TH + a.Y - 1) * W;
  const int npair = (QLEN + 63) >> 6;
  const float* xn = a.x + (size_t)n * Cin * HW;
  const int nsteps = NS > 0 ? NS : Cin >> 1;   // channel pairs
  float2 xb[kRing];
  unsigned loff = 0;   // per-lane float offset inside the image; the channel-pair base stays scalar
  bool valid = false;
  int qa = 0;
  auto block_setup = [&](int pb) {
    qa = pb * 64 + 2 * l32;
    const int q = qbase + qa;
    valid = q >= 0 && q < HW && qa < QLEN;
    const int qc = q < 0 ? 0 : (q > HW - 2 ? HW - 2 : q);
    loff = (unsigned)(hi * HW + qc);           // channel (2*step + hi)
  };
  // Step indices are clamped instead of branched on: a redundant load of a
  // valid address is cheaper than a branch per ring slot.
  auto ldx = [&](int step) {
    step = step < nsteps ? step : nsteps - 1;
    return *reinterpret_cast<const float2*>(xn + (size_t)(2 * step) * HW + loff);
  };
  auto ring_fill = [&]() {
#pragma unroll
    for (int s = 0; s < kRing; ++s) xb[s] = ldx(s);
  };
  // Prologue: put every global load the first phases need in flight at once
  // (oldest first, the order the in-order load counter releases them): this
  // wave's Fout block for P3, the first chunk of the Fin tile, the x ring.
  constexpr int kP0 = 16;                       // Fin elements per thread and chunk
  const int fin_total = Cin * RP;
  float fkv[RP / 2], finv[kP0];
  if (wave < nitems) fk_issue(wave % nkb, fkv);
  auto fin_issue = [&](int i0) {
#pragma unroll
    for (int u = 0; u < kP0; ++u) {
      const int i = i0 + u * kThreads;
      const int c = i / RP, r = i - c * RP;
      finv[u] = (i < fin_total && r < R) ? a.Fin[(size_t)c * R + r] : 0.f;
    }
  };
  auto fin_store = [&](int i0) {
#pragma unroll
    for (int u = 0; u < kP0; ++u) {
      const int i = i0 + u * kThreads;
      if (i < fin_total) R2[i] = finv[u];
    }
  };
  fin_issue(tid);
  bool filled = false;
  if (wave < npair) {
    block_setup(wave);
    if (__any(valid)) {
      ring_fill();
      filled = true;
    }
  }
  if (wave < nitems) fk_finish(fkv);
  fin_store(tid);
  for (int i0 = tid + kThreads * kP0; i0 < fin_total; i0 += kThreads * kP0) {
    fin_issue(i0);
    fin_store(i0);
  }
  STAMP(1)
  __syncthreads();
  STAMP(2)

  // ---- P1: channel -> rank contraction ------------------------------------
  if (pl.phases & 1)
  for (int pb = wave; pb < npair; pb += kWaves) {
    f32x16 acc[RB][2];
#pragma unroll
    for (int mb = 0; mb < RB; ++mb) {
      acc[mb][0] = (f32x16)(0.f);
      acc[mb][1] = (f32x16)(0.f);
    }
    if (pb != wave) {
      block_setup(pb);
      filled = false;
    }
    if (__any(valid)) {
      if (!filled) ring_fill();
      // Fin[2*step + hi][32*mb + l32]; one LDS read per step and rank block,
      // issued one step ahead of the MFMAs that use it.
      const float* fp = R2 + hi * RP + l32;
      if constexpr (NS > 0) {
        // straight-line: x slot st % kRing is consumed at step st and refilled
        // for step st + kRing right after, so kRing loads stay in flight per
        // lane; the Fin operand runs kAhead steps ahead the same way
        constexpr int kAhead = 4;
        float aopr[kAhead][RB];
#pragma unroll
        for (int u = 0; u < kAhead; ++u)
#pragma unroll
          for (int mb = 0; mb < RB; ++mb)
            aopr[u][mb] = fp[(u < NS ? u : NS - 1) * 2 * RP + 32 * mb];
#pragma unroll
        for (int st = 0; st < NS; ++st) {
          const int slot = st % kRing, as = st % kAhead;
#pragma unroll
          for (int mb = 0; mb < RB; ++mb) {
            acc[mb][0] = mfma32(aopr[as][mb], xb[slot].x, acc[mb][0]);
            acc[mb][1] = mfma32(aopr[as][mb], xb[slot].y, acc[mb][1]);
          }
          if (st + kRing < NS) xb[slot] = ldx(st + kRing);
          if (st + kAhead < NS) {
#pragma unroll
            for (int mb = 0; mb < RB; ++mb)
              aopr[as][mb] = fp[(st + kAhead) * 2 * RP + 32 * mb];
          }
          // keep the issue order use-then-refill per step: without it the
          // scheduler sinks the refills to the end and the ring no longer
          // overlaps loads with the matrix work
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        float aop[RB], aopn[RB];
#pragma unroll
        for (int mb = 0; mb < RB; ++mb) aop[mb] = fp[32 * mb];
        int base = 0;
        for (; base + kRing <= nsteps; base += kRing) {
#pragma unroll
          for (int s = 0; s < kRing; ++s) {
            const int st = base + s;
            const int stn = st + 1 < nsteps ? st + 1 : nsteps - 1;
#pragma unroll
            for (int mb = 0; mb < RB; ++mb) aopn[mb] = fp[stn * 2 * RP + 32 * mb];
#pragma unroll
            for (int mb = 0; mb < RB; ++mb) {
              acc[mb][0] = mfma32(aop[mb], xb[s].x, acc[mb][0]);
              acc[mb][1] = mfma32(aop[mb], xb[s].y, acc[mb][1]);
            }
            xb[s] = ldx(st + kRing);   // refill this slot kRing steps ahead
#pragma unroll
            for (int mb = 0; mb < RB; ++mb) aop[mb] = aopn[mb];
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        // fewer than kRing steps left: they are already in the ring
        for (int s = 0; base + s < nsteps; ++s) {
          float2 cur = xb[0];
#pragma unroll
          for (int u = 1; u < kRing; ++u) cur = (u == s) ? xb[u] : cur;
#pragma unroll
          for (int mb = 0; mb < RB; ++mb) {
            const float f = fp[(base + s) * 2 * RP + 32 * mb];
            acc[mb][0] = mfma32(f, cur.x, acc[mb][0]);
            acc[mb][1] = mfma32(f, cur.y, acc[mb][1]);
          }
        }
      }
    }
    // accumulator (v, lane) holds rank row 8*(v/4) + 4*hi + v%4, pixel column l32
#pragma unroll
    for (int mb = 0; mb < RB; ++mb)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = 32 * mb + 8 * (v >> 2) + 4 * hi + (v & 3);
        float2 o;
        o.x = valid ? acc[mb][0][v] : 0.f;
        o.y = valid ? acc[mb][1][v] : 0.f;
        *reinterpret_cast<float2*>(As + r * QA + qa) = o;
      }
  }
  STAMP(3)
  __syncthreads();
  STAMP(4)

  // ---- P2: the separable taps ----------------------------------------------
  const float* Cc;   // [RP][QCs] for P3
  int QCs;
  if constexpr (FS > 0) {
    // One (rank, column) pair per thread; rows stream through a register window.
    float* Cs = R2;
    const int QC = pl.QC;
    Cc = Cs;
    QCs = QC;
    const int nin = pl.TH + FS - 1;
    if (pl.phases & 2)
    for (int pr = tid; pr < R * W; pr += kThreads) {
      const int r = pr / W, w = pr - r * W;
      float fh[FS], fw[FS];
      int off[FS];
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        const int tap = a.flip ? FS - 1 - j : j;
        fh[j] = a.FH[tap * R + r];
        const int ww = w + j - a.pad;
        const bool in = ww >= 0 && ww < W;
        fw[j] = in ? a.FW[tap * R + r] : 0.f;
        off[j] = ww < 0 ? 0 : (ww >= W ? W - 1 : ww);   // clamped: weight is 0 there
      }
      const float* ar = As + r * QA;
      float* cr = Cs + r * QC + w;
      float win[FS];
#pragma unroll
      for (int j = 0; j < FS; ++j) win[j] = 0.f;
      for (int hh = 0; hh < nin; ++hh) {
        float hs = 0.f;
#pragma unroll
        for (int j = 0; j < FS; ++j) hs += fw[j] * ar[hh * W + off[j]];
#pragma unroll
        for (int j = 0; j + 1 < FS; ++j) win[j] = win[j + 1];
        win[FS - 1] = hs;
        if (hh >= FS - 1) {
          float o = 0.f;
#pragma unroll
          for (int i = 0; i < FS; ++i) o += fh[i] * win[i];
          cr[(hh - (FS - 1)) * W] = o;
        }
      }
    }
    // ranks beyond R meet a zero factor in P3 but must not hold NaN bit patterns
    for (int i = R * QC + tid; i < RP * QC; i += kThreads) Cs[i] = 0.f;
  } else {
    // Any filter shape: taps along H (A -> B), then along W (B -> Cc over A).
    const int QB = pl.QB;
    const int npix = pl.TH * W;
    float* Bs = R2 + pl.padoff;
    Cc = As;
    QCs = QA;
    for (int rr = wave; rr < R; rr += kWaves) {
      const float* ar = As + rr * QA;
      float* br = Bs + rr * QB;
      for (int p = lane; p < npix; p += 64) {
        float s = 0.f;
        for (int i = 0; i < a.Y; ++i)
          s += a.FH[(a.flip ? a.Y - 1 - i : i) * R + rr] * ar[p + i * W];
        br[p] = s;
      }
    }
    __syncthreads();
    for (int p = lane; p < npix; p += 64) {
      const int w = p % W;
      for (int rr = wave; rr < RP; rr += kWaves) {
        const float* br = Bs + rr * QB;
        float s = 0.f;
        if (rr < R) {
          for (int j = 0; j < a.X; ++j) {
            const int ww = w + j - a.pad;
            const float bv = (ww >= 0 && ww < W) ? br[p + j - a.pad] : 0.f;
            s += a.FW[(a.flip ? a.X - 1 - j : j) * R + rr] * bv;
          }
        }
        As[rr * QA + p] = s;
      }
    }
  }
  STAMP(5)
  __syncthreads();
  STAMP(6)

  // ---- P3: rank -> output-channel contraction -----------------------------
  float* yn = a.y + (size_t)n * Cout * HW + (size_t)h0 * W;
  auto ensure_fk = [&](int kb) {
    if (kb != cur_kb) {
      if constexpr (FS > 0) load_fk_staged(kb);   // A region is free again
      else load_fk_gather(kb);
    }
  };
  if constexpr (RB == 1) {
    // Software-pipelined over this wave's items (item j = wave + 8*j): while
    // the MFMAs of item j run, the Cc operands of item j+1 are read from LDS
    // and the rows of item j-1 are stored, one of each per MFMA pair, so a
    // wave keeps the matrix pipe fed on its own.
    const int nmy = wave < nitems ? (nitems - wave + kWaves - 1) / kWaves : 0;
    float2 bA[RP / 2], bB[RP / 2];
    f32x16 aA0 = (f32x16)(0.f), aA1 = aA0, aB0 = aA0, aB1 = aA0;
    auto cp_of = [&](int j) -> const float* {
      if (j >= nmy) return nullptr;
      const int pp = (wave + kWaves * j) / nkb;
      return Cc + hi * QCs + pp * 64 + 2 * l32;
    };
    // per-lane pointer to output row 32*kb + 4*hi of item j, or null if this lane stores nothing
    auto yp_of = [&](int j, int& krem) -> float* {
      krem = 0;
      if (j < 0 || j >= nmy) return nullptr;
      const int item = wave + kWaves * j, pp = item / nkb, kb = item - pp * nkb;
      const int p = pp * 64 + 2 * l32;
      krem = Cout - (32 * kb + 4 * hi);
#ifdef CP4_DEBUG_PHASES
      if (pl.phases & 8) return nullptr;
#endif
      return p < nvalid ? yn + (size_t)(32 * kb + 4 * hi) * HW + p : nullptr;
    };
    // full: every lane and every row of the item is inside the output, so the
    // store needs no predicate
    auto store_row = [&](const f32x16& p0, const f32x16& p1, int v, float* yp, int krem,
                         auto full) {
      const int ro = 8 * (v >> 2) + (v & 3);
      if (full.value || (yp && ro < krem)) {
        float2 o;
        o.x = p0[v];
        o.y = p1[v];
        *reinterpret_cast<float2*>(yp + (size_t)ro * HW) = o;
      }
    };
    // One item's 32 MFMAs with, per MFMA pair, one Cc read for the next item
    // (has_next) and one row store of the previous item (has_prev); the three
    // flags are wave-uniform and compiled in, so the steady state is branch-free.
    auto stage = [&](const float2 (&bc)[RP / 2], f32x16& c0, f32x16& c1, float2 (&bn)[RP / 2],
                     const float* cpn, const f32x16& p0, const f32x16& p1, float* yp, int krem,
                     auto has_next, auto has_prev, auto prev_full) {
      c0 = (f32x16)(0.f);
      c1 = (f32x16)(0.f);
#pragma unroll
      for (int s = 0; s < RP / 2; ++s) {
#ifdef CP4_DEBUG_PHASES
        if (!(pl.phases & 16)) {
#endif
        c0 = mfma32(fk[s], bc[s].x, c0);
        c1 = mfma32(fk[s], bc[s].y, c1);
#ifdef CP4_DEBUG_PHASES
        }
#endif
        if constexpr (has_next.value) bn[s] = *reinterpret_cast<const float2*>(cpn + 2 * s * QCs);
        if constexpr (has_prev.value) store_row(p0, p1, s, yp, krem, prev_full);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    using T = std::true_type;
    using F = std::false_type;
    auto run_stage = [&](const float2 (&bc)[RP / 2], f32x16& c0, f32x16& c1,
                         float2 (&bn)[RP / 2], int jnext, const f32x16& p0, const f32x16& p1,
                         int jprev) {
      int krem;
      const float* cpn = cp_of(jnext);
      float* yp = yp_of(jprev, krem);
      const bool next = jnext < nmy, prev = jprev >= 0;
      bool full = false;
      if (prev) {
        const int item = wave + kWaves * jprev, pp = item / nkb, kb = item - pp * nkb;
        full = pp * 64 + 64 <= nvalid && 32 * kb + 32 <= Cout;
#ifdef CP4_DEBUG_PHASES
        if (pl.phases & 8) full = false;
#endif
      }
      if (next) {
        if (!prev) stage(bc, c0, c1, bn, cpn, p0, p1, yp, krem, T{}, F{}, F{});
        else if (full) stage(bc, c0, c1, bn, cpn, p0, p1, yp, krem, T{}, T{}, T{});
        else stage(bc, c0, c1, bn, cpn, p0, p1, yp, krem, T{}, T{}, F{});
      } else {
        if (!prev) stage(bc, c0, c1, bn, cpn, p0, p1, yp, krem, F{}, F{}, F{});
        else if (full) stage(bc, c0, c1, bn, cpn, p0, p1, yp, krem, F{}, T{}, T{});
        else stage(bc, c0, c1, bn, cpn, p0, p1, yp, krem, F{}, T{}, F{});
      }
    };
    if (pl.phases & 4)
    if (nmy > 0) {
      const float* cp0 = cp_of(0);
#pragma unroll
      for (int s = 0; s < RP / 2; ++s) bA[s] = *reinterpret_cast<const float2*>(cp0 + 2 * s * QCs);
      for (int j = 0; j < nmy; j += 2) {
        ensure_fk((wave + kWaves * j) % nkb);
        run_stage(bA, aA0, aA1, bB, j + 1, aB0, aB1, j - 1);
        if (j + 1 < nmy) {
          ensure_fk((wave + kWaves * (j + 1)) % nkb);
          run_stage(bB, aB0, aB1, bA, j + 2, aA0, aA1, j);
        }
      }
      int krem;
      float* yp = yp_of(nmy - 1, krem);
      if (nmy & 1) {
#pragma unroll
        for (int v = 0; v < 16; ++v) store_row(aA0, aA1, v, yp, krem, F{});
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) store_row(aB0, aB1, v, yp, krem, F{});
      }
    }
  } else {
    if (pl.phases & 4)
    for (int item = wave; item < nitems; item += kWaves) {
      const int pp = item / nkb, kb = item - pp * nkb;
      ensure_fk(kb);
      f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
      const float* cp = Cc + hi * QCs + pp * 64 + 2 * l32;
#pragma unroll
      for (int s = 0; s < RP / 2; ++s) {
        const float2 b = *reinterpret_cast<const float2*>(cp + 2 * s * QCs);
        acc0 = mfma32(fk[s], b.x, acc0);
        acc1 = mfma32(fk[s], b.y, acc1);
      }
      const int p = pp * 64 + 2 * l32;
      if (p < nvalid) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int k = 32 * kb + 8 * (v >> 2) + 4 * hi + (v & 3);
          if (k < Cout) {
            float2 o;
            o.x = acc0[v];
            o.y = acc1[v];
            *reinterpret_cast<float2*>(yn + (size_t)k * HW + p) = o;
          }
        }
      }
    }
  }
  STAMP(7)
}

int round_up(int v, int m) { return (v + m - 1) / m * m; }

bool fast_taps(const FwdArgs& a) {
  return a.Y == a.X && (a.Y == 1 || a.Y == 3 || a.Y == 5 || a.Y == 7);
}

// LDS layout for a strip height; returns false if it does not fit.
bool layout(const FwdArgs& a, int TH, StripPlan* pl) {
  const long RP = a.R <= 32 ? 32 : 64;
  const long QLEN = (long)(TH + a.Y - 1) * a.W;
  const long QA = round_up((int)QLEN, 64) + 8;
  const long QC = round_up(TH * a.W, 64) + 8;
  const int padoff = round_up(a.pad, 2);
  const long QB = round_up(TH * a.W + padoff + a.X, 2);
  long r2 = (long)a.Cin * RP;
  const long second = fast_taps(a) ? RP * QC : RP * QB;
  if (second > r2) r2 = second;
  long r1 = RP * QA;                              // A region, at least the
  const long stage = kWaves * 32 * (RP + 1);      // 8 per-wave Fout staging tiles
  if (stage > r1) r1 = stage;
  const size_t bytes = (size_t)(r1 + r2) * sizeof(float);
  if (bytes > kLdsLimit) return false;
  pl->TH = TH;
  pl->strips = (a.H + TH - 1) / TH;
  pl->nWG = a.N * pl->strips;
  pl->QA = (int)QA;
  pl->QC = (int)QC;
  pl->QB = (int)QB;
  pl->padoff = padoff;
  pl->r2_off = (int)r1;
  pl->lds_bytes = bytes;
  pl->phases = 7;
  return true;
}

// Strip height: fewest rounds of one workgroup per compute unit times the per-strip matrix work
// (halo rows repeat the channel->rank contraction).
bool plan(const FwdArgs& a, StripPlan* best) {
  double best_cost = 0;
  bool found = false;
  const int cus = num_compute_units();
  for (int TH = 1; TH <= a.H; ++TH) {
    StripPlan pl;
    if (!layout(a, TH, &pl)) break;
    const double rounds = (pl.nWG + cus - 1) / cus;
    const double cost = rounds * ((double)(TH + a.Y - 1) * a.Cin + (double)TH * a.Cout);
    if (!found || cost < best_cost) {
      best_cost = cost;
      *best = pl;
      found = true;
    }
  }
  return found;
}

template <int RB, int FS, int NS>
hipError_t launch_ns(const FwdArgs& a, const StripPlan& pl, hipStream_t st) {
  const void* fn = reinterpret_cast<const void*>(fwd_mfma_strip_kernel<RB, FS, NS>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)pl.lds_bytes);
  if (e != hipSuccess) return e;
  const unsigned grid = 8u * ((pl.nWG + 7) / 8);
  fwd_mfma_strip_kernel<RB, FS, NS><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}

// The channel counts of common layers get the fully unrolled P1.
template <int RB, int FS>
hipError_t launch_as(const FwdArgs& a, const StripPlan& pl, hipStream_t st) {
  if constexpr (FS == 3 || FS == 5) {
    switch (a.Cin) {
      case 64: return launch_ns<RB, FS, 32>(a, pl, st);
      case 128: return launch_ns<RB, FS, 64>(a, pl, st);
      case 256: return launch_ns<RB, FS, 128>(a, pl, st);
      default: break;
    }
  }
  return launch_ns<RB, FS, 0>(a, pl, st);
}

template <int RB>
hipError_t launch_rb(const FwdArgs& a, const StripPlan& pl, hipStream_t st) {
  if (!fast_taps(a)) return launch_as<RB, 0>(a, pl, st);
  switch (a.Y) {
    case 1: return launch_as<RB, 1>(a, pl, st);
    case 3: return launch_as<RB, 3>(a, pl, st);
    case 5: return launch_as<RB, 5>(a, pl, st);
    default: return launch_as<RB, 7>(a, pl, st);
  }
}

}  // namespace

bool fwd_mfma_supported(const FwdArgs& a) {
  if (a.R > 64 || (a.W & 1) || (a.Cin & 1) || a.sh) return false;
  if (!fits_int_indexing(a.N, a.H, a.W)) return false;
  if (a.x && (reinterpret_cast<uintptr_t>(a.x) & 7)) return false;
  if (a.y && (reinterpret_cast<uintptr_t>(a.y) & 7)) return false;
  StripPlan pl;
  return plan(a, &pl);
}

hipError_t fwd_mfma_launch(const FwdArgs& a, hipStream_t st) {
  StripPlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
#ifdef CP4_DEBUG_PHASES
  pl.phases = debug_phase_limit(pl.phases);
  pl.dbg = debug_stamp_buffer();
#endif
  return a.R <= 32 ? launch_rb<1>(a, pl, st) : launch_rb<2>(a, pl, st);
}

}  // namespace cp4
