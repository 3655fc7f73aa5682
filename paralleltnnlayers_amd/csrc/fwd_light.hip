// Fused forward / backward-data kernel for small problems: few, short phases and
// many small workgroups, where the producer / consumer kernel's sixteen-wave
// pipeline spends most of a launch filling and draining.
//
// Same arithmetic as the other matrix-core kernels (the reassociated form of
// Cuda_kernels/cp4Conv2dForward.cu:84-133; backward-data,
// cp4Conv2dBackwardData.cu:57-108, through swapped factors and reversed taps):
// exact fp32 products as six bf16 MFMAs on three-way split operands, taps in fp32
// on the vector units.  Ranks up to 32.
//
// A workgroup of four or eight waves owns a strip of TH rows of one image (full
// width; with its FS - 1 halo rows a contiguous run of floats per channel plane,
// so pixels are a flat index q).  Three phases, two barriers:
//   P1  A[r,q] = sum_c Fin[c,r] x[c,q]: a wave takes 32-pixel blocks; both
//       operands come straight from memory through a register ring of
//       16-channel chunks (the factor slice as well: no staging phase before the
//       first product), are split in registers and meet in six MFMAs per chunk.
//       A goes to LDS by rank quads, [r / 4][q][r % 4], zero outside the image.
//   P2  a thread takes (rank quad, output pixel): FS x FS cells of A as 16-byte
//       LDS reads, tap weights from LDS, the four results split into the MFMA B
//       fragment layout in LDS.
//   P3  y[k,p] = sum_r Fout[k,r] Cc[r,p]: a wave takes (64 pixels, 32 output
//       channels); even and odd pixels in two accumulators, float2 stores with
//       the bias / activation epilogue (FwdArgs::bias, act) applied on the way.
#include "cp4_internal.h"
#include "split_bf16.h"

namespace cp4 {
namespace {

using namespace split;

constexpr int kRing = 4;                     // 16-channel chunks in flight per lane
constexpr int kMaxWG = 4;                    // workgroups the planner wants per compute unit at most

struct LightPlan {
  int TH, strips, nWG;
  int nw;          // waves per workgroup (4 or 8)
  int QA;          // cells of the A plane per rank quad (a multiple of 32)
  int npo;         // 64-pixel output groups
  int quads;       // rank quads of A
  int nc;          // 16-rank chunks of the output contraction (1 or 2)
  int pbytes;      // bytes of one fragment plane
  int cf_off;      // byte offset of the fragment planes in LDS
  int w_off;       // byte offset of the tap weights in LDS
  unsigned wmagic; // ceil(2^32 / W)
  size_t lds_bytes;
};

template <int FS, int NW>
__global__ __launch_bounds__(64 * NW) void fwd_light_kernel(FwdArgs a, LightPlan pl) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float4* As4 = reinterpret_cast<float4*>(lds_raw);                  // [quads][QA]
  unsigned char* Cf = lds_raw + pl.cf_off;   // plane ((part*nc + c)*2 + hi)*2 + parity: [pixel >> 1] x 16 B
  float* wl = reinterpret_cast<float*>(lds_raw + pl.w_off);          // FH then FW, [FS][32] each

  const int t = blockIdx.x;
  const int n = t / pl.strips, h0 = (t - n * pl.strips) * pl.TH;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin, Cout = a.Cout;
  const int QA = pl.QA, NC = pl.nc;
  const int rows = min(pl.TH, H - h0);
  const int nvalid = rows * W;
  const int nkb = (Cout + 31) >> 5;
  const int nitems = nkb * pl.npo;
  const int qbase = (h0 - a.pad) * W;
  const int QLEN = (rows + FS - 1) * W;
  const int nblk = (QLEN + 31) >> 5;
  const int nch = (Cin + 15) >> 4;

  // ---- every load the first products need goes out before anything waits ----
  // x through a buffer descriptor over this image: reads past its last channel return 0
  const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(a.x + (size_t)n * Cin * HW), 0, Cin * HW * 4, 0x00020000);
  const bool frow = l32 < R;
  const float* fin = a.Fin + (frow ? l32 : 0);
  float xb[kRing][8], fb[kRing][8];
  unsigned voff = 0;
  int qa = 0;
  bool valid = false;
  auto block_setup = [&](int b) {
    qa = 32 * b + l32;
    const int q = qbase + qa;
    valid = q >= 0 && q < HW && qa < QLEN;
    const int qc = q < 0 ? 0 : (q > HW - 1 ? HW - 1 : q);
    voff = (unsigned)(8 * hi * HW + qc) * 4u;
  };
  auto ld_chunk = [&](int u, int ch) {
    ch = ch < nch ? ch : nch - 1;                        // clamped, not branched
    const unsigned soff = (unsigned)(16 * ch) * (unsigned)HW * 4u;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      xb[u][e] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(xrs, voff, soff + (unsigned)e * HW * 4u, 0));
    const int c0 = 16 * ch + 8 * hi;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int c = c0 + e < Cin ? c0 + e : Cin - 1;
      fb[u][e] = fin[(size_t)c * R];
    }
  };
  if (wave < nblk) {
    block_setup(wave);
#pragma unroll
    for (int u = 0; u < kRing; ++u)
      if (u < nch) ld_chunk(u, u);
  }
  // tap weights -> LDS (rows of 32 ranks, zero past the last rank)
  for (int i = tid; i < 2 * FS * 32; i += 64 * NW) {
    const int which = i / (FS * 32), rem = i - which * FS * 32;
    const int j = rem >> 5, r = rem & 31;
    const int tap = a.flip ? FS - 1 - j : j;
    const float* src = which ? a.FW : a.FH;
    wl[i] = r < R ? src[tap * R + r] : 0.f;
  }
  // the first output-factor block of this wave: row 32*kb + l32, ranks 16*c + 8*hi + e
  float fkraw[2][8];
  int cur_kb = -1;
  auto fk_issue = [&](int kb) {
    cur_kb = kb;
    const int k = 32 * kb + l32;
    const float* src = a.Fout + (size_t)(k < Cout ? k : Cout - 1) * R;
#pragma unroll
    for (int c = 0; c < 2; ++c)
      if (c < NC) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int r = 16 * c + 8 * hi + e;
          const float v = src[r < R ? r : R - 1];
          fkraw[c][e] = (k < Cout && r < R) ? v : 0.f;
        }
      }
  };
  if (wave < nitems) fk_issue(wave % nkb);

  // ---- P1: channel -> rank contraction ------------------------------------
  for (int b = wave; b < nblk; b += NW) {
    if (b != wave) {
      block_setup(b);
#pragma unroll
      for (int u = 0; u < kRing; ++u)
        if (u < nch) ld_chunk(u, u);
    }
    f32x16 acc = (f32x16)(0.f);
    for (int ch0 = 0; ch0 < nch; ch0 += kRing) {
#pragma unroll
      for (int u = 0; u < kRing; ++u) {
        if (ch0 + u < nch) {                             // (the same for all lanes)
          float fv[8];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            fv[e] = (frow && 16 * (ch0 + u) + 8 * hi + e < Cin) ? fb[u][e] : 0.f;
          u32x4 fh, fm, fl, xh, xm, xl;
          split8(fv, fh, fm, fl);
          split8(xb[u], xh, xm, xl);
          acc = mfma_split(fh, fm, fl, xh, xm, xl, acc);
        }
        if (ch0 + kRing < nch) ld_chunk(u, ch0 + u + kRing);   // refill (uniform)
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // accumulator element v: rank 8*(v >> 2) + 4*hi + (v & 3), i.e. quad 2*(v >> 2) + hi
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int quad = 2 * j + hi;
      if (quad < pl.quads) {
        float4 o;
        o.x = valid ? acc[4 * j] : 0.f;
        o.y = valid ? acc[4 * j + 1] : 0.f;
        o.z = valid ? acc[4 * j + 2] : 0.f;
        o.w = valid ? acc[4 * j + 3] : 0.f;
        As4[quad * QA + qa] = o;
      }
    }
  }
  __syncthreads();

  // ---- P2: separable taps, results split into B fragments -------------------
  {
    const int PW = 64 * pl.npo;                          // padded output pixels
    const int total = 4 * NC * PW;
    const int pbytes = pl.pbytes;
    for (int it = tid; it < total; it += 64 * NW) {
      const int rq = it / PW, p = it - rq * PW;
      float o[4] = {0.f, 0.f, 0.f, 0.f};
      if (rq < pl.quads && p < nvalid) {
        const int h = (int)__umulhi((unsigned)p, pl.wmagic), w = p - h * W;
        const float4* ar = As4 + rq * QA + h * W + w - a.pad;
        const float* wh = wl + 4 * rq;                   // FH rows
        const float* ww = wl + FS * 32 + 4 * rq;         // FW rows
        float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < FS; ++i) {
          float hs[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < FS; ++j) {
            const int wc = w + j - a.pad;
            const bool in = wc >= 0 && wc < W;
            const float4 v = ar[i * W + (in ? j : a.pad - w)];   // outside: any cell of the row
            const float4 f = *reinterpret_cast<const float4*>(ww + 32 * j);
            hs[0] += (in ? f.x : 0.f) * v.x;
            hs[1] += (in ? f.y : 0.f) * v.y;
            hs[2] += (in ? f.z : 0.f) * v.z;
            hs[3] += (in ? f.w : 0.f) * v.w;
          }
          const float4 g = *reinterpret_cast<const float4*>(wh + 32 * i);
          s[0] += g.x * hs[0];
          s[1] += g.y * hs[1];
          s[2] += g.z * hs[2];
          s[3] += g.w * hs[3];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) o[q] = s[q];
      }
      u32x2 ph, pm, pl2;
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const float x0 = o[2 * d], x1 = o[2 * d + 1];
        ph[d] = pack_hi16(x0, x1);
        const float r0 = x0 - trunc_bf16(x0), r1 = x1 - trunc_bf16(x1);
        pm[d] = pack_hi16(r0, r1);
        pl2[d] = pack_hi16(r0 - trunc_bf16(r0), r1 - trunc_bf16(r1));
      }
      // chunk rq >> 2, half (rq >> 1) & 1 of the chunk; the quad is the low or high 8 bytes
      unsigned char* dst = Cf + (size_t)((((rq >> 2) * 2 + ((rq >> 1) & 1)) * 2) + (p & 1)) * pbytes +
                           (p >> 1) * 16 + (rq & 1) * 8;
      const size_t part = (size_t)NC * 4 * pbytes;
      *reinterpret_cast<u32x2*>(dst) = ph;
      *reinterpret_cast<u32x2*>(dst + part) = pm;
      *reinterpret_cast<u32x2*>(dst + 2 * part) = pl2;
    }
  }
  __syncthreads();

  // ---- P3: rank -> output-channel contraction -------------------------------
  float* yn = a.y + (size_t)n * Cout * HW + (size_t)h0 * W;
  for (int item = wave; item < nitems; item += NW) {
    const int pp = item / nkb, kb = item - pp * nkb;
    if (kb != cur_kb) fk_issue(kb);
    f32x16 acc0 = (f32x16)(0.f), acc1 = (f32x16)(0.f);
    const size_t part = (size_t)NC * 4 * pl.pbytes;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      if (c < NC) {
        u32x4 kh, km, kl;
        split8(fkraw[c], kh, km, kl);
        const unsigned char* bp = Cf + (size_t)((c * 2 + hi) * 2) * pl.pbytes + (32 * pp + l32) * 16;
        const u32x4 b0h = *reinterpret_cast<const u32x4*>(bp);
        const u32x4 b1h = *reinterpret_cast<const u32x4*>(bp + pl.pbytes);
        const u32x4 b0m = *reinterpret_cast<const u32x4*>(bp + part);
        const u32x4 b1m = *reinterpret_cast<const u32x4*>(bp + part + pl.pbytes);
        const u32x4 b0l = *reinterpret_cast<const u32x4*>(bp + 2 * part);
        const u32x4 b1l = *reinterpret_cast<const u32x4*>(bp + 2 * part + pl.pbytes);
        acc0 = mfma_split(kh, km, kl, b0h, b0m, b0l, acc0);
        acc1 = mfma_split(kh, km, kl, b1h, b1m, b1l, acc1);
      }
    }
    const int p = pp * 64 + 2 * l32;
    // epilogue y = act(conv + bias[k]), applied as a value is stored
    float bv[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) bv[v] = 0.f;
    if (a.bias) {                                        // (the same for all lanes)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int k = 32 * kb + 8 * (v >> 2) + 4 * hi + (v & 3);
        bv[v] = a.bias[k < Cout ? k : Cout - 1];
      }
    }
    const bool relu = a.act == 1;
    if (p < nvalid) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int k = 32 * kb + 8 * (v >> 2) + 4 * hi + (v & 3);
        if (k < Cout) {
          float2 o;
          o.x = acc0[v] + bv[v];
          o.y = acc1[v] + bv[v];
          if (relu) {                                    // (a NaN stays a NaN)
            o.x = o.x < 0.f ? 0.f : o.x;
            o.y = o.y < 0.f ? 0.f : o.y;
          }
          *reinterpret_cast<float2*>(yn + (size_t)k * HW + p) = o;
        }
      }
    }
  }
}

// Strip height: the serial work of a workgroup's busiest wave in the three phases,
// for as long as the grid still fits the chip at once.
bool plan(const FwdArgs& a, LightPlan* best) {
  const int cus = num_compute_units();
  const int nch = (a.Cin + 15) / 16, nkb = (a.Cout + 31) / 32;
  const int nc = a.R > 16 ? 2 : 1, quads = (a.R + 3) / 4;
  double best_cost = 0;
  bool found = false;
  const int th_lo = a.tune_th > 0 ? a.tune_th : 1, th_hi = a.tune_th > 0 ? a.tune_th : a.H;
  for (int TH = th_lo; TH <= th_hi && TH <= a.H; ++TH) {
    const long QLEN = (long)(TH + a.Y - 1) * a.W;
    const long nblk = (QLEN + 31) / 32, npo = ((long)TH * a.W + 63) / 64;
    if (nblk > 64) break;
    const int nw = nblk > 4 || npo * nkb > 4 ? 8 : 4;
    const long QA = nblk * 32;
    const long pbytes = npo * 512;
    const long as_bytes = quads * QA * 16, cf_bytes = 12l * nc * pbytes, w_bytes = 2l * a.Y * 32 * 4;
    const long lds = as_bytes + cf_bytes + w_bytes;
    if (lds > 64 * 1024) break;
    const long strips = (a.H + TH - 1) / TH, nwg = a.N * strips;
    const double rounds = (double)((nwg + (long)cus * kMaxWG - 1) / ((long)cus * kMaxWG));
    const double p1 = (double)((nblk + nw - 1) / nw) * (nch + 2.0);
    const double p2 = (double)((4 * nc * npo + nw - 1) / nw) * 0.25 * a.Y;
    const double p3 = (double)((npo * nkb + nw - 1) / nw) * (nc + 1.0);
    // workgroups beyond one per compute unit share its vector units
    const double share = nwg > cus ? (double)nwg / cus : 1.0;
    const double cost = rounds * (p1 + p2 + p3 + 3.0) * (share > kMaxWG ? kMaxWG : share);
    if (!found || cost < best_cost) {
      best_cost = cost;
      found = true;
      best->TH = TH;
      best->strips = (int)strips;
      best->nWG = (int)nwg;
      best->nw = nw;
      best->QA = (int)QA;
      best->npo = (int)npo;
      best->quads = quads;
      best->nc = nc;
      best->pbytes = (int)pbytes;
      best->cf_off = (int)as_bytes;
      best->w_off = (int)(as_bytes + cf_bytes);
      best->wmagic = (unsigned)((0x100000000ull + a.W - 1) / a.W);
      best->lds_bytes = (size_t)lds;
    }
  }
  return found;
}

template <int FS, int NW>
hipError_t launch_nw(const FwdArgs& a, const LightPlan& pl, hipStream_t st) {
  const void* fn = reinterpret_cast<const void*>(fwd_light_kernel<FS, NW>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)pl.lds_bytes);
  if (e != hipSuccess) return e;
  fwd_light_kernel<FS, NW><<<pl.nWG, 64 * NW, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}
template <int FS>
hipError_t launch_fs(const FwdArgs& a, const LightPlan& pl, hipStream_t st) {
  return pl.nw == 4 ? launch_nw<FS, 4>(a, pl, st) : launch_nw<FS, 8>(a, pl, st);
}

}  // namespace

bool fwd_light_supported(const FwdArgs& a) {
  if (a.R > 32 || (a.W & 1) || a.sh || a.dense || a.taps2d || a.ldf || a.accumulate) return false;
  if (a.Y != a.X || !(a.Y == 1 || a.Y == 3 || a.Y == 5) || a.pad > a.Y - 1) return false;
  if (!fits_int_indexing(a.N, a.H, a.W) || (size_t)a.Cin * a.H * a.W >= (1u << 29)) return false;
  if (a.y && (reinterpret_cast<uintptr_t>(a.y) & 7)) return false;
  if (a.x && (reinterpret_cast<uintptr_t>(a.x) & 3)) return false;
  LightPlan pl;
  return plan(a, &pl);
}

hipError_t fwd_light_launch(const FwdArgs& a, hipStream_t st) {
  LightPlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
  switch (a.Y) {
    case 1: return launch_fs<1>(a, pl, st);
    case 3: return launch_fs<3>(a, pl, st);
    default: return launch_fs<5>(a, pl, st);
  }
}

}  // namespace cp4
