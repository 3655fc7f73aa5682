// Fused forward / backward-data kernel on the bf16 matrix cores with an exact
// three-way operand split (fp32-equivalent accuracy), ranks up to 32.
//
// An fp32 value has 24 significand bits; truncating to bf16 three times,
//   h = bf16(x), m = bf16(x - h), l = x - h - m,
// gives three bf16 numbers of 8 significand bits each whose sum is x exactly.
// A product x*f is then  xh*fh + (xh*fm + xm*fh) + (xh*fl + xm*fm + xl*fh)
// plus terms below 2^-24 of |x*f|, i.e. six bf16 MFMAs accumulated in fp32 give
// the fp32 product to within fp32 rounding.  v_mfma_f32_32x32x16_bf16 runs 16x
// the flops per cycle of the fp32 MFMA, so the six-term split is ~2.7x faster
// than v_mfma_f32_32x32x2_f32 and moves the kernel from matrix-bound to
// memory-bound; the split itself is 5.5 VALU ops per value.
//
// Structure (one workgroup of 8 wave64 per strip of TH image rows, flat pixel
// index q inside the strip plus its halo rows):
//   P0  Fin[Cin,R] -> split -> LDS, laid out as MFMA A fragments.
//   P1  A[r,q] = sum_c Fin[c,r] x[c,q]: a lane streams float2 (two pixels) of 8
//       channels per 16-channel chunk from HBM (4 chunks = 32 loads in flight),
//       splits them in registers and issues 12 MFMAs per chunk; fp32 A -> LDS.
//   P2  separable taps in fp32 (VALU, register window per (rank quad, column)),
//       result split and written to LDS as MFMA B fragments.
//   P3  y[k,p] = sum_r Fout[k,r] Cc[r,p]: Fout fragment split in registers,
//       Cc fragments read 16 bytes per lane from LDS, 24 MFMAs per 32x64 tile,
//       float2 stores (256 contiguous bytes per half-wave and output row).
// Arithmetic follows the reassociated form of
// Cuda_kernels/cp4Conv2dForward.cu:84-133 (backward-data:
// cp4Conv2dBackwardData.cu:57-108 through swapped factors and flipped taps).
#include <cstdlib>

#include "cp4_internal.h"
#ifdef CP4_DEBUG_PHASES
#include "cp4_debug.h"
#endif

namespace cp4 {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 512, kWaves = kThreads / 64;
constexpr int kRP = 32;                      // rank padded to one MFMA tile
#ifndef CP4_SPLIT_RING
#define CP4_SPLIT_RING 4
#endif
constexpr int kRing = CP4_SPLIT_RING;                     // 16-channel chunks in flight per lane
constexpr size_t kLdsLimit = 160 * 1024;     // gfx950 LDS per workgroup

struct SplitPlan {
  int TH, strips, nWG;
  int QA;             // LDS row stride of A (floats)
  int plane_bytes;    // bytes of one Cc fragment plane
  int r2_off;         // float offset of the second LDS region
  size_t lds_bytes;
#ifdef CP4_DEBUG_PHASES
  long long* dbg;
#endif
};

__device__ __forceinline__ f32x16 mfma16(u32x4 a, u32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                 __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// upper halves of two floats' bit patterns -> one dword (a in the low half)
__device__ __forceinline__ unsigned pack_hi16(float a, float b) {
  return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}
__device__ __forceinline__ float trunc_bf16(float v) {
  return __uint_as_float(__float_as_uint(v) & 0xffff0000u);
}

// Exact split of N floats (N even) into bf16 parts h, m, l, N/2 dwords each.
template <int N, class V>
__device__ __forceinline__ void split_exact(const float (&v)[N], V& h, V& m, V& l) {
#pragma unroll
  for (int d = 0; d < N / 2; ++d) {
    const float a = v[2 * d], b = v[2 * d + 1];
    h[d] = pack_hi16(a, b);
    const float ra = a - trunc_bf16(a), rb = b - trunc_bf16(b);
    m[d] = pack_hi16(ra, rb);
    const float sa = ra - trunc_bf16(ra), sb = rb - trunc_bf16(rb);
    l[d] = pack_hi16(sa, sb);
  }
}

// acc += A * B with both operands split; smallest terms first.
__device__ __forceinline__ f32x16 mfma_split(u32x4 ah, u32x4 am, u32x4 al, u32x4 bh, u32x4 bm,
                                             u32x4 bl, f32x16 acc) {
  acc = mfma16(al, bh, acc);
  acc = mfma16(am, bm, acc);
  acc = mfma16(ah, bl, acc);
  acc = mfma16(am, bh, acc);
  acc = mfma16(ah, bm, acc);
  acc = mfma16(ah, bh, acc);
  return acc;
}

template <int FS>
__global__ __launch_bounds__(kThreads) void fwd_split_kernel(FwdArgs a, SplitPlan pl) {
  extern __shared__ float lds[];
  float* As = lds;                                      // [32][QA] fp32
  unsigned char* R2 = reinterpret_cast<unsigned char*>(lds + pl.r2_off);
  // R2 holds the Fin fragments in P0/P1: [chunk][part][hi][r] x 16 B, and the
  // Cc fragments in P2/P3: plane (part, chunk, hi, pixel parity) of
  // [pixel >> 1] x 16 B (8 consecutive ranks of one pixel).

  const int per = (pl.nWG + 7) >> 3;
  const int t = (blockIdx.x & 7) * per + (blockIdx.x >> 3);   // XCD-contiguous tile order
  if (t >= pl.nWG) return;
  const int n = t / pl.strips, h0 = (t - n * pl.strips) * pl.TH;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#ifdef CP4_DEBUG_PHASES
#define STAMP(i) if (pl.dbg && lane == 0) { pl.dbg[((size_t)t * 8 + wave) * 8 + (i)] = wall_clock64(); pl.dbg[262144 + ((size_t)t * 8 + wave) * 8 + (i)] = clock64(); }
#define STAMP2(i) if (pl.dbg && lane == 0) { pl.dbg[65536 + ((size_t)t * 8 + wave) * 8 + (i)] = wall_clock64(); }
#else
#define STAMP(i)
#define STAMP2(i)
#endif
  STAMP(0)
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin, Cout = a.Cout;
  const int QA = pl.QA;
  const int rows = min(pl.TH, H - h0);
  const int nvalid = rows * W;
  const int npo = (nvalid + 63) >> 6;
  const int nkb = (Cout + 31) >> 5;
  const int nitems = nkb * npo;

  // ---- prologue: every global load the first phases need goes out at once,
  // oldest first in the order they are consumed (the load counter releases in
  // order): the Fin tile, this wave's raw Fout block (split only before P3),
  // then the first ring of x chunks.
  const int fin_items = (Cin >> 3) * 32;                  // (channel octet, rank)
  float finv[2][8];
  auto fin_issue = [&](float (&v)[8], int it) {
    const int o = it >> 5, r = it & 31;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      v[e] = (it < fin_items && r < R) ? a.Fin[(size_t)(8 * o + e) * R + r] : 0.f;
  };
  auto fin_store = [&](const float (&v)[8], int it) {
    if (it >= fin_items) return;
    const int o = it >> 5, r = it & 31;
    u32x4 h, m, l;
    split_exact<8>(v, h, m, l);
    u32x4* dst = reinterpret_cast<u32x4*>(R2 + ((size_t)(o >> 1) * 6 + (o & 1)) * 512 + r * 16);
    dst[0] = h;        // part stride: 2 planes of 512 B = 64 x 16 B
    dst[64] = m;
    dst[128] = l;
  };
  STAMP2(0)
  fin_issue(finv[0], tid);
  fin_issue(finv[1], tid + kThreads);
  STAMP2(1)

  // Fout block of 32 output channels: lane holds row 32*kb + l32, ranks
  // 16*c + 8*hi + e, read as two float4 per 16-rank chunk when R allows.
  float fkraw[2][8];
  u32x4 fkh[2], fkm[2], fkl[2];
  int cur_kb = -1;
  const bool fk_vec = (R & 7) == 0 && (reinterpret_cast<uintptr_t>(a.Fout) & 15) == 0;
  auto fk_issue = [&](int kb) {
    cur_kb = kb;
    const int k = 32 * kb + l32;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int r0 = 16 * c + 8 * hi;
      if (fk_vec) {
        float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi4 = lo;
        if (k < Cout && r0 < R) {
          const float4* src = reinterpret_cast<const float4*>(a.Fout + (size_t)k * R + r0);
          lo = src[0];
          hi4 = src[1];
        }
        fkraw[c][0] = lo.x; fkraw[c][1] = lo.y; fkraw[c][2] = lo.z; fkraw[c][3] = lo.w;
        fkraw[c][4] = hi4.x; fkraw[c][5] = hi4.y; fkraw[c][6] = hi4.z; fkraw[c][7] = hi4.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          fkraw[c][e] = (k < Cout && r0 + e < R) ? a.Fout[(size_t)k * R + r0 + e] : 0.f;
      }
    }
  };
  auto fk_split = [&]() {
#pragma unroll
    for (int c = 0; c < 2; ++c) split_exact<8>(fkraw[c], fkh[c], fkm[c], fkl[c]);
  };
  if (wave < nitems) fk_issue(wave % nkb);

  const int qbase = (h0 - a.pad) * W;
  const int QLEN = (pl.TH + FS - 1) * W;
  const int npair = (QLEN + 63) >> 6;
  const int nch = Cin >> 4;                              // 16-channel chunks
  const float* xn = a.x + (size_t)n * Cin * HW;
  float2 xb[kRing][8];
  unsigned loff = 0;
  bool valid = false;
  int qa = 0;
  auto block_setup = [&](int pb) {
    qa = pb * 64 + 2 * l32;
    const int q = qbase + qa;
    valid = q >= 0 && q < HW && qa < QLEN;
    const int qc = q < 0 ? 0 : (q > HW - 2 ? HW - 2 : q);
    loff = (unsigned)(8 * hi * HW + qc);                 // channel 16*chunk + 8*hi + e
  };
  auto ld_chunk = [&](float2 (&b)[8], int ch) {
    ch = ch < nch ? ch : nch - 1;                        // clamped, not branched
    const float* base = xn + (size_t)(16 * ch) * HW + loff;
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = *reinterpret_cast<const float2*>(base + (size_t)e * HW);
  };
  bool filled = false;
  if (wave < npair) {
    block_setup(wave);
    if (__any(valid)) {
#pragma unroll
      for (int u = 0; u < kRing; ++u) ld_chunk(xb[u], u);
      filled = true;
    }
  }

  STAMP2(2)
  // ---- P0: Fin -> split -> LDS fragments ----------------------------------
  fin_store(finv[0], tid);
  STAMP2(3)
  fin_store(finv[1], tid + kThreads);
  STAMP2(4)
  for (int it = tid + 2 * kThreads; it < fin_items; it += kThreads) {
    fin_issue(finv[0], it);
    fin_store(finv[0], it);
  }
  STAMP(1)
  __syncthreads();
  STAMP(2)

  // ---- P1: channel -> rank contraction ------------------------------------
  for (int pb = wave; pb < npair; pb += kWaves) {
    f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
    if (pb != wave) {
      block_setup(pb);
      filled = false;
    }
    if (__any(valid)) {
      if (!filled) {
#pragma unroll
        for (int u = 0; u < kRing; ++u) ld_chunk(xb[u], u);
      }
      const u32x4* fbase = reinterpret_cast<const u32x4*>(R2 + hi * 512 + l32 * 16);
      for (int ch = 0; ch < nch; ch += kRing) {
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
          const u32x4* fp = fbase + (size_t)(ch + u) * (6 * 32);   // 6 planes of 32 x 16 B per chunk
          const u32x4 fh = fp[0], fm = fp[64], fl = fp[128];
          float vx[8], vy[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            vx[e] = xb[u][e].x;
            vy[e] = xb[u][e].y;
          }
          u32x4 xh, xm, xl;
          split_exact<8>(vx, xh, xm, xl);
          acc0 = mfma_split(fh, fm, fl, xh, xm, xl, acc0);
          split_exact<8>(vy, xh, xm, xl);
          acc1 = mfma_split(fh, fm, fl, xh, xm, xl, acc1);
          ld_chunk(xb[u], ch + u + kRing);               // refill this ring slot
          // keep use-then-refill order per chunk so kRing chunks stay in flight
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int r = 8 * (v >> 2) + 4 * hi + (v & 3);
      float2 o;
      o.x = valid ? acc0[v] : 0.f;
      o.y = valid ? acc1[v] : 0.f;
      *reinterpret_cast<float2*>(As + r * QA + qa) = o;
    }
  }
  STAMP(3)
  __syncthreads();
  STAMP(4)

  // ---- P2: separable taps, then split into B fragments ---------------------
  const int pbytes = pl.plane_bytes;
  if (R < kRP) {   // fragments of ranks >= R must be zero, not stale bits
    for (int i = tid; i < 24 * (pbytes >> 2); i += kThreads)
      reinterpret_cast<unsigned*>(R2)[i] = 0u;
    __syncthreads();
  }
  {
    const int nin = pl.TH + FS - 1;
    const int nq = (R + 3) >> 2;                         // rank quads
    for (int it = tid; it < nq * W; it += kThreads) {
      const int rq = it / W, w = it - rq * W;
      float fh[4][FS], fw[4][FS];
      int off[FS];
#pragma unroll
      for (int j = 0; j < FS; ++j) {
        const int tap = a.flip ? FS - 1 - j : j;
        const int ww = w + j - a.pad;
        const bool in = ww >= 0 && ww < W;
        off[j] = ww < 0 ? 0 : (ww >= W ? W - 1 : ww);    // clamped: weight is 0 there
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int r = 4 * rq + q;
          fh[q][j] = r < R ? a.FH[tap * R + r] : 0.f;
          fw[q][j] = (in && r < R) ? a.FW[tap * R + r] : 0.f;
        }
      }
      const float* ar = As + (4 * rq) * QA;
      // plane (part, chunk, hi, parity): chunk = rq >> 2, hi = (rq >> 1) & 1; this
      // quad is the low or high 8 bytes of the 16-byte entry
      unsigned char* cbase = R2 + (size_t)(((rq >> 2) * 2 + ((rq >> 1) & 1)) * 2) * pbytes +
                             (rq & 1) * 8;
      float win[4][FS];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < FS; ++j) win[q][j] = 0.f;
      for (int hh = 0; hh < nin; ++hh) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float hs = 0.f;
#pragma unroll
          for (int j = 0; j < FS; ++j) hs += fw[q][j] * ar[q * QA + hh * W + off[j]];
#pragma unroll
          for (int j = 0; j + 1 < FS; ++j) win[q][j] = win[q][j + 1];
          win[q][FS - 1] = hs;
        }
        if (hh >= FS - 1) {
          float o[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            o[q] = 0.f;
#pragma unroll
            for (int i = 0; i < FS; ++i) o[q] += fh[q][i] * win[q][i];
          }
          u32x2 ph, pm, pl2;
          split_exact<4>(o, ph, pm, pl2);
          const int p = (hh - (FS - 1)) * W + w;
          unsigned char* dst = cbase + (size_t)(p & 1) * pbytes + (p >> 1) * 16;
          *reinterpret_cast<u32x2*>(dst) = ph;                       // part stride: 8 planes
          *reinterpret_cast<u32x2*>(dst + (size_t)8 * pbytes) = pm;
          *reinterpret_cast<u32x2*>(dst + (size_t)16 * pbytes) = pl2;
        }
      }
    }
  }
  STAMP(5)
  __syncthreads();
  STAMP(6)

  // ---- P3: rank -> output-channel contraction -----------------------------
  float* yn = a.y + (size_t)n * Cout * HW + (size_t)h0 * W;
  if (wave < nitems) fk_split();   // the block loaded in the prologue
  for (int item = wave; item < nitems; item += kWaves) {
    const int pp = item / nkb, kb = item - pp * nkb;
    if (kb != cur_kb) {
      fk_issue(kb);
      fk_split();
    }
    f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      // plane index ((part*2 + c)*2 + hi)*2 + parity; entry 32*pp + l32
      const unsigned char* bp = R2 + (size_t)((c * 2 + hi) * 2) * pbytes + (32 * pp + l32) * 16;
      const u32x4 b0h = *reinterpret_cast<const u32x4*>(bp);
      const u32x4 b1h = *reinterpret_cast<const u32x4*>(bp + pbytes);
      const u32x4 b0m = *reinterpret_cast<const u32x4*>(bp + (size_t)8 * pbytes);
      const u32x4 b1m = *reinterpret_cast<const u32x4*>(bp + (size_t)9 * pbytes);
      const u32x4 b0l = *reinterpret_cast<const u32x4*>(bp + (size_t)16 * pbytes);
      const u32x4 b1l = *reinterpret_cast<const u32x4*>(bp + (size_t)17 * pbytes);
      acc0 = mfma_split(fkh[c], fkm[c], fkl[c], b0h, b0m, b0l, acc0);
      acc1 = mfma_split(fkh[c], fkm[c], fkl[c], b1h, b1m, b1l, acc1);
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
  STAMP(7)
}

int round_up(int v, int m) { return (v + m - 1) / m * m; }

bool layout(const FwdArgs& a, int TH, SplitPlan* pl) {
  const long QLEN = (long)(TH + a.Y - 1) * a.W;
  const long QA = round_up((int)QLEN, 64) + 8;
  const long npo = (TH * a.W + 63) / 64;
  const long plane_bytes = npo * 32 * 16;               // 32 entries of 16 B per 64-pixel block
  const long r1 = kRP * QA;                              // floats
  long r2_bytes = (long)a.Cin * 192;                     // Fin fragments: Cin*32 values, 3 parts x 2 B
  if (24 * plane_bytes > r2_bytes) r2_bytes = 24 * plane_bytes;
  const size_t bytes = (size_t)r1 * sizeof(float) + (size_t)r2_bytes;
  if (bytes > kLdsLimit) return false;
  pl->TH = TH;
  pl->strips = (a.H + TH - 1) / TH;
  pl->nWG = a.N * pl->strips;
  pl->QA = (int)QA;
  pl->plane_bytes = (int)plane_bytes;
  pl->r2_off = (int)r1;
  pl->lds_bytes = bytes;
  return true;
}

// Strip height: fewest rounds of one workgroup per compute unit times the rows each strip
// reads (with halo) and writes.
bool plan(const FwdArgs& a, SplitPlan* best) {
  double best_cost = 0;
  bool found = false;
  const int cus = num_compute_units();
  for (int TH = 1; TH <= a.H; ++TH) {
    SplitPlan pl;
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

template <int FS>
hipError_t launch_fs(const FwdArgs& a, const SplitPlan& pl, hipStream_t st) {
  const void* fn = reinterpret_cast<const void*>(fwd_split_kernel<FS>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)pl.lds_bytes);
  if (e != hipSuccess) return e;
  const unsigned grid = 8u * ((pl.nWG + 7) / 8);
  fwd_split_kernel<FS><<<grid, kThreads, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}

}  // namespace

bool fwd_split_supported(const FwdArgs& a) {
  if (a.R > kRP || (a.W & 1) || (a.Cin & 63) || a.sh) return false;
  if (!fits_int_indexing(a.N, a.H, a.W)) return false;
  if (a.Y != a.X || !(a.Y == 1 || a.Y == 3 || a.Y == 5 || a.Y == 7)) return false;
  if (a.x && (reinterpret_cast<uintptr_t>(a.x) & 7)) return false;
  if (a.y && (reinterpret_cast<uintptr_t>(a.y) & 7)) return false;
  SplitPlan pl;
  return plan(a, &pl);
}

hipError_t fwd_split_launch(const FwdArgs& a, hipStream_t st) {
  SplitPlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
#ifdef CP4_DEBUG_PHASES
  pl.dbg = debug_stamp_buffer();
#endif
  switch (a.Y) {
    case 1: return launch_fs<1>(a, pl, st);
    case 3: return launch_fs<3>(a, pl, st);
    case 5: return launch_fs<5>(a, pl, st);
    default: return launch_fs<7>(a, pl, st);
  }
}

}  // namespace cp4
