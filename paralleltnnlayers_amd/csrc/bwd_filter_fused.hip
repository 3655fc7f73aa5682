// Backward-filter in three launches, the tap step fused into the gradient GEMMs.
//
// Same reassociation of the reference's 8-deep sums
// (Cuda_kernels/cp4Conv2dBackwardFilter.cu:64-257) as the other variants:
//   A = FC^T x,  G3 = FK^T dy,  Cc = FW *h (FH *v A),  G1 = adjoint taps of G3
//   dFK = dy . Cc^T     dFC = x . G1^T
//   dFH[i] = sum G3[h,w] sum_j FW[j] A[h+i-P, w+j-P]     dFW[j] = sum G3[h,w] sum_i FH[i] A[h+i-P, w+j-P]
// but only A and G3 ever reach memory:
//   1. contract_all_kernel: both channel -> rank contractions as exact split-bf16
//      products; a wave splits its x / dy chunk once and multiplies it with every
//      32-rank block of the factor (pre-split MFMA fragments in LDS).
//   2. grad_fused_kernel: a workgroup owns (gradient, channel group) and walks over
//      (image, row strip) items.  Per item it copies the strip of A (dFK) or G3
//      (dFC) plus halo rows into a zero-bordered LDS plane, applies the taps there
//      and leaves Cc / G1 of the strip as split MFMA B fragments in LDS; its waves
//      then stream their 32 channel rows of dy / x straight from memory as the A
//      operand.  Accumulators live in registers across all items of the workgroup,
//      so there are as many partial sums as workgroups per (gradient, channel
//      group), not one per image.  The workgroups of channel group 0 of dFK also
//      form the tap gradients from the A window they already hold.
//   3. reduce_fused_kernel: fixed-order sum of the partials (bit-reproducible; no
//      floating-point atomics anywhere).
#include <cstdint>

#include "cp4_internal.h"
#include "split_bf16.h"

namespace cp4 {
namespace {

using namespace split;
typedef float f32x4 __attribute__((ext_vector_type(4)));


constexpr int kFillTasks = 4;     // factor-tile tasks whose loads a thread requests together
constexpr int kFragBytes = 3072;  // one (16-element step, 32-rank block): [part][half][rank] x 16 B

// ---- 1. Z[n,r,p] = sum_c F[c,r] src[n,c,p] for x -> A and dy -> G3 -----------------
// (Operands of the two contractions as separate fields, picked with selects: indexing an
// array in the kernel-argument segment by blockIdx would cost a dependent scalar load.)
struct ContractAllArgs {
  const float *src0, *src1;   // x, dy
  const float *F0, *F1;       // FC, FK
  float *Z0, *Z1;             // A, G3
  int Cin0, Cin1;
  int R, HW, npb, items;   // items per operand = N * npb (32-pixel blocks)
  int vecfill;             // both factors 16-byte aligned and R a multiple of 4
};

// x / dy and the factor are read through buffer descriptors: an address is
// (descriptor base) + (32-bit lane offset) + (scalar offset), so the walk over
// channels runs on the scalar unit and a load costs no vector instruction.
template <int RB, int KS, int RING>
__global__ __launch_bounds__(512) void contract_all_kernel(ContractAllArgs a) {
  extern __shared__ float Fs[];
  unsigned char* Fb = reinterpret_cast<unsigned char*>(Fs);
  const int which = blockIdx.y;
  const int Cin = which ? a.Cin1 : a.Cin0, R = a.R, HW = a.HW;
  const float* src = which ? a.src1 : a.src0;
  const float* F = which ? a.F1 : a.F0;
  float* Z = which ? a.Z1 : a.Z0;
  const int tid = threadIdx.x, lane = tid & 63, nthr = blockDim.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nw = nthr >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  // This wave's (item, channel split); waves past the end do nothing but reach the barriers.
  const int slot = blockIdx.x * nw + wave;
  const int item = slot / KS, part = slot - item * KS;
  const bool has_item = item < a.items;
  const int n = has_item ? item / a.npb : 0, pb = has_item ? item - n * a.npb : 0;
  const int p = pb * 32 + l32;
  const bool valid = has_item && p < HW;
  const int pc = p < HW ? p : HW - 1;
  const int nch = (Cin >> 4) / KS, c0 = part * nch;   // this wave's chunks c0 .. c0 + nch - 1
  const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(src + (size_t)n * Cin * HW), 0, Cin * HW * 4, 0x00020000);
  const unsigned voff = (unsigned)(8 * hi * HW + pc) * 4u;   // lane's channel 16*chunk + 8*hi + e
  const unsigned sbase = (unsigned)(16 * c0) * (unsigned)HW * 4u;
  float xb[RING][8];
  // (Every load of the sweep is issued on every path - chunks past the wave's last are
  // clamped to it - so that the count of loads in flight at each wait is a constant the
  // compiler can put into the wait instruction; a load skipped on some path makes it
  // wait for the youngest load instead of the one it needs.)
  auto ld_chunk = [&](float (&dst)[8], int ch) {
    ch = ch < nch ? ch : nch - 1;
    const unsigned soff = sbase + (unsigned)(16 * ch) * (unsigned)HW * 4u;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      dst[e] = __builtin_bit_cast(
          float, __builtin_amdgcn_raw_buffer_load_b32(xrs, voff, soff + (unsigned)e * HW * 4u, 0));
  };
  // the first activation chunks are requested before the factor tile is built
#pragma unroll
  for (int u = 0; u < RING; ++u) ld_chunk(xb[u], u);
  // factor tile: fragment entry (channel octet o, rank rr) = the three bf16 parts of
  // F[8o .. 8o+7][rr], 16 bytes each
  {
    const __amdgpu_buffer_rsrc_t frs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(F), 0, Cin * R * 4, 0x00020000);
    constexpr int RPt = 32 * RB;
    auto put = [&](const float (&v)[8], int o, int rr) {
      u32x4 h, m, l;
      split8(v, h, m, l);
      u32x4* dst = reinterpret_cast<u32x4*>(Fb + ((size_t)(o >> 1) * RB + (rr >> 5)) * kFragBytes +
                                            (o & 1) * 512 + (rr & 31) * 16);
      dst[0] = h;            // part stride: 2 halves x 32 ranks x 16 B
      dst[64] = m;
      dst[128] = l;
    };
    if (a.vecfill) {
      // rows of F are 16-byte aligned and R is a multiple of 4: a task is (octet, four
      // ranks), eight 16-byte loads; two tasks' loads are requested together (tasks
      // past the end repeat the last one)
      const int ntask = (Cin >> 3) * (RPt / 4);
      for (int it0 = tid; it0 < ntask; it0 += 2 * nthr) {
        f32x4 w[2][8];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int it = min(it0 + t * nthr, ntask - 1);
          const int o = it / (RPt / 4), rq = it - o * (RPt / 4);
          // rank quads past R read past the descriptor's end: 0
          const unsigned fo = 4 * rq < R ? (unsigned)(8 * o * R + 4 * rq) * 4u : 0x80000000u;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            w[t][e] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                                                    frs, fo, (unsigned)(e * R) * 4u, 0));
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int it = min(it0 + t * nthr, ntask - 1);
          const int o = it / (RPt / 4), rq = it - o * (RPt / 4);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const f32x4 q = w[t][e];
              v[e] = j == 0 ? q.x : (j == 1 ? q.y : (j == 2 ? q.z : q.w));
            }
            put(v, o, 4 * rq + j);
          }
        }
      }
    } else {
      // element by element: a thread requests the loads of kFillTasks entries before it splits any
      const int nfill = (Cin >> 3) * RPt;
      for (int it0 = tid; it0 < nfill; it0 += kFillTasks * nthr) {
        float v[kFillTasks][8];
#pragma unroll
        for (int t = 0; t < kFillTasks; ++t) {
          const int it = min(it0 + t * nthr, nfill - 1);
          const int o = it / RPt, rr = it - o * RPt;
          const unsigned fo = rr < R ? (unsigned)(8 * o * R + rr) * 4u : 0x80000000u;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[t][e] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(frs, fo, (unsigned)(e * R) * 4u, 0));
        }
#pragma unroll
        for (int t = 0; t < kFillTasks; ++t) {
          const int it = min(it0 + t * nthr, nfill - 1);
          put(v[t], it / RPt, it % RPt);
        }
      }
    }
  }
  for (int i = tid; i < RB * (kFragBytes / 16); i += nthr)
    reinterpret_cast<u32x4*>(Fb + (size_t)(Cin >> 4) * RB * kFragBytes)[i] = u32x4{0u, 0u, 0u, 0u};
  __syncthreads();
  f32x16 acc[2] = {(f32x16)(0.f), (f32x16)(0.f)};   // RB == 2: one per rank block; RB == 1: alternating
  {
    const u32x4* fbase = reinterpret_cast<const u32x4*>(Fb + hi * 512 + l32 * 16);
    const int zero_chunk = Cin >> 4;                   // an all-zero fragment block behind the tile
    u32x4 xh, xm, xl;
    split8(xb[0], xh, xm, xl);
    ld_chunk(xb[0], RING);
    // rounds of RING chunks; chunks past the last multiply the zero block
    for (int ch = 0; ch < nch; ch += RING) {
#pragma unroll
      for (int u = 0; u < RING; ++u) {
        const int c = ch + u;                          // chunk whose parts are in xh / xm / xl
        const u32x4* fp = fbase + (size_t)(c < nch ? c0 + c : zero_chunk) * RB * (kFragBytes / 16);
        float (&nx)[8] = xb[(u + 1) % RING];
        u32x4 nh, nm, nl;
        auto piece = [&](int d) {                      // a quarter of the next chunk's split
          const float x0 = nx[2 * d], x1 = nx[2 * d + 1];
          nh[d] = pack_hi16(x0, x1);
          const float r0 = x0 - trunc_bf16(x0), r1 = x1 - trunc_bf16(x1);
          nm[d] = pack_hi16(r0, r1);
          nl[d] = pack_hi16(r0 - trunc_bf16(r0), r1 - trunc_bf16(r1));
        };
        if (RB == 1) {
          const u32x4 fh = fp[0], fm = fp[64], fl = fp[128];
          acc[0] = mfma16(fl, xh, acc[0]);
          piece(0);
          __builtin_amdgcn_sched_barrier(0);
          acc[1] = mfma16(fm, xm, acc[1]);
          piece(1);
          __builtin_amdgcn_sched_barrier(0);
          acc[0] = mfma16(fh, xl, acc[0]);
          piece(2);
          __builtin_amdgcn_sched_barrier(0);
          acc[1] = mfma16(fm, xh, acc[1]);
          piece(3);
          __builtin_amdgcn_sched_barrier(0);
          acc[0] = mfma16(fh, xm, acc[0]);
          acc[1] = mfma16(fh, xh, acc[1]);
        } else {
          const u32x4 fh0 = fp[0], fm0 = fp[64], fl0 = fp[128];
          const u32x4 fh1 = fp[kFragBytes / 16], fm1 = fp[kFragBytes / 16 + 64],
                      fl1 = fp[kFragBytes / 16 + 128];
          acc[0] = mfma16(fl0, xh, acc[0]);
          piece(0);
          __builtin_amdgcn_sched_barrier(0);
          acc[1] = mfma16(fl1, xh, acc[1]);
          piece(1);
          __builtin_amdgcn_sched_barrier(0);
          acc[0] = mfma16(fm0, xm, acc[0]);
          piece(2);
          __builtin_amdgcn_sched_barrier(0);
          acc[1] = mfma16(fm1, xm, acc[1]);
          piece(3);
          __builtin_amdgcn_sched_barrier(0);
          acc[0] = mfma16(fh0, xl, acc[0]);
          acc[1] = mfma16(fh1, xl, acc[1]);
          acc[0] = mfma16(fm0, xh, acc[0]);
          acc[1] = mfma16(fm1, xh, acc[1]);
          acc[0] = mfma16(fh0, xm, acc[0]);
          acc[1] = mfma16(fh1, xm, acc[1]);
          acc[0] = mfma16(fh0, xh, acc[0]);
          acc[1] = mfma16(fh1, xh, acc[1]);
        }
        ld_chunk(nx, c + 1 + RING);                    // refill the slot just split
        xh = nh;
        xm = nm;
        xl = nl;
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (RB == 1) acc[0] = acc[0] + acc[1];
  }
  float* zn = Z + (size_t)n * R * HW + p;
  if (KS == 1) {
    if (valid) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int r = 32 * rb + 8 * (v >> 2) + 4 * hi + (v & 3);
          if (r < R) zn[(size_t)r * HW] = acc[rb][v];
        }
    }
    return;
  }
  // KS waves hold partial sums of one item: exchange through LDS (over the factor
  // tile, which nobody reads any more); wave `part` adds and stores rows
  // v = part, part + KS, ... in the fixed order of the splits.
  __syncthreads();
  float* red = Fs;                                     // [wave][rb * 16 + v][lane]
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int v = 0; v < 16; ++v) red[((wave * RB + rb) * 16 + v) * 64 + lane] = acc[rb][v];
  __syncthreads();
  if (!has_item) return;
  const int w0 = wave - part;                          // first wave of this item
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int j = 0; j < 16 / KS; ++j) {
      const int v = part + KS * j;
      float sum = 0.f;
#pragma unroll
      for (int q = 0; q < KS; ++q) sum += red[(((w0 + q) * RB + rb) * 16 + v) * 64 + lane];
      const int r = 32 * rb + 8 * (v >> 2) + 4 * hi + (v & 3);
      if (valid && r < R) zn[(size_t)r * HW] = sum;
    }
}

// ---- 2. taps in LDS + gradient GEMMs + tap gradients --------------------------------
struct FusedArgs {
  const float *act0, *act1;     // dy, x            (gradient 0: dFK, 1: dFC)
  const float *Zsrc0, *Zsrc1;   // A, G3            the plane the taps are applied to (G3 also
                                //                  feeds the tap gradients)
  const float *FH, *FW;
  float *part0, *part1;         // [S][D][R]
  float *partH, *partW;         // [S * TG][FS][R]
  int D0, D1;
  int N, R, H, W, P, HW;
  int TG;                     // channel groups of dFK that share the tap gradients (1 or 2)
  int TH, NS, items, S, MT;   // strip rows, strips per image, items = N * NS, workgroups per
                              // (gradient, channel group), 32-channel tiles per workgroup (4 or 8)
  int Wp, PSt, KSmax;         // padded row pitch, plane stride (odd), 16-pixel steps per strip
  unsigned wmagic;            // floor(2^32 / W) + 1: q / W == umulhi(q, wmagic) for q < 2^32 / W
};

// Workgroup: 512 threads.  LDS: [RP][PSt] plane | [RB][KSmax] fragment steps.
// Square odd filters with "same" padding P = (FS-1)/2, so the zero border of the
// plane is Q = P cells on every side and both chains read the same window.
template <int FS, int RB>
__global__ __launch_bounds__(512) void grad_fused_kernel(FusedArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int RP = 32 * RB;
  constexpr int Q = (FS - 1) / 2;
  constexpr int NX = 8 + 2 * Q;        // window positions that can hold a pixel of the octet
  constexpr int WN = NX + FS - 1;      // window columns read per tap row
  constexpr int kRing = 4;             // 16-pixel steps in flight per wave
  const int which = blockIdx.z, cg = blockIdx.y, sidx = blockIdx.x;
  const int D = which ? a.D1 : a.D0, R = a.R, H = a.H, W = a.W, HW = a.HW;
  const int MT = a.MT, KH = 8 / MT;
  if (cg * 32 * MT >= D) return;                       // whole workgroup
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  const int Wp = a.Wp, PSt = a.PSt;
  float* plane = lds;
  u32x4* frag = reinterpret_cast<u32x4*>(lds + (size_t)RP * PSt);
  // the tap gradients are shared by the first TG channel groups of dFK: group g takes
  // the octets o with o % TG == g
  const int TG = a.TG;
  const bool tapgroup = which == 0 && cg < TG;
  // taps of this thread's rank (fixed: 512 % RP == 0); the adjoint chain (dFC) reads
  // the same window with both weight vectors reversed
  const int r = tid & (RP - 1);
  float fh[FS], fw[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) fh[i] = fw[i] = 0.f;
  float gh[FS], gw[FS];
#pragma unroll
  for (int i = 0; i < FS; ++i) gh[i] = gw[i] = 0.f;
  // the zero step behind each rank block's fragment steps (read first after a barrier)
  for (int i = tid; i < RB * (kFragBytes / 16); i += 512)
    frag[(size_t)((i / (kFragBytes / 16)) * (a.KSmax + 1) + a.KSmax) * (kFragBytes / 16) +
         i % (kFragBytes / 16)] = u32x4{0u, 0u, 0u, 0u};
  // GEMM role of this wave: 32 channel rows, every KH-th 16-pixel step
  const int mt = wave / KH, kh = wave - mt * KH;
  const int d = cg * 32 * MT + 32 * mt + l32;
  const bool drow = d < D;
  f32x16 acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) acc[rb] = (f32x16)(0.f);
  const float* Zs = which ? a.Zsrc1 : a.Zsrc0;
  const float* act = which ? a.act1 : a.act0;

  for (int item = sidx; item < a.items; item += a.S) {
    const int n = item / a.NS, st = item - n * a.NS;
    const int h0 = st * a.TH, h1 = min(H, h0 + a.TH);
    const int q0 = h0 * W, q1 = h1 * W;
    const int KS = (q1 - q0 + 15) >> 4;
    // this wave's first activation steps, requested before the tap step
    const float* arow = act + ((size_t)n * D + (drow ? d : 0)) * HW;
    float4 ring[kRing][2];
    // Every load of the sweep is issued on every path (steps past the strip's last
    // and pixels past the plane's end are clamped into this channel row, rows past D
    // to row 0: they multiply zero fragments or land in rows that are not stored), so
    // that the loads in flight at each wait are a constant.
    auto issue = [&](float4 (&dst)[2], int s) {
      s = s < KS ? s : KS - 1;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int px = min(q0 + 16 * s + 8 * hi + 4 * j, HW - 4);
        dst[j] = *reinterpret_cast<const float4*>(arow + px);
      }
    };

    // (b) rows hlo .. hhi-1 of every rank of the source plane are one contiguous run
    // per rank: wave w takes ranks w, w + 8, ... in 64-element pieces, a batch of
    // JM x KM loads in flight at once (buffer loads: the rank walk is a scalar offset).
    // Pieces past the run and ranks past R are not branched around: their loads are
    // clamped and their stores go to a cell nothing reads.
    constexpr int JM = 4 * RB, KM = 32 / JM;
    const int hlo = max(0, h0 - Q), hhi = min(H, h1 + Q);
    const int run = (hhi - hlo) * W;
    const int per = (run + 63) >> 6;
    const int cbase = (hlo - h0 + Q) * Wp + Q;         // cell of (hlo, 0)
    const int dummy = PSt - 1;
    const __amdgpu_buffer_rsrc_t zrs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(Zs + (size_t)n * R * HW + (size_t)hlo * W), 0, ((R - 1) * HW + run) * 4,
        0x00020000);
    float pv[JM * KM];
    int cellk[KM];
    auto plane_load = [&](int kb) {
#pragma unroll
      for (int kk = 0; kk < KM; ++kk) {
        const int i = lane + 64 * (kb * KM + kk);
        const int row = (int)__umulhi((unsigned)i, a.wmagic);
        cellk[kk] = i < run ? cbase + i + row * 2 * Q : dummy;
        const unsigned vo = (unsigned)min(i, run - 1) * 4u;   // (lanes past the run: a valid cell, for the dummy)
        if (kb * KM + kk < per) {                      // wave-uniform
#pragma unroll
          for (int jj = 0; jj < JM; ++jj) {
            const int rr = min(wave + 8 * jj, R - 1);
            pv[jj * KM + kk] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(zrs, vo,
                                                            (unsigned)(rr * HW) * 4u, 0));
          }
        }
      }
    };
    auto plane_store = [&](int kb) {
#pragma unroll
      for (int kk = 0; kk < KM; ++kk) {
        if (kb * KM + kk < per) {
#pragma unroll
          for (int jj = 0; jj < JM; ++jj) {
            const int rr = wave + 8 * jj;              // wave-uniform
            plane[min(rr, R - 1) * PSt + (rr < R ? cellk[kk] : dummy)] = pv[jj * KM + kk];
          }
        }
      }
    };
    plane_load(0);
    // this wave's first activation steps, requested behind the plane so that the plane arrives first
#pragma unroll
    for (int u = 0; u < kRing; ++u) issue(ring[u], kh + u * KH);
    if (item == sidx) {
      // the tap weights, requested behind the first loads and first used in the tap
      // step; padding ranks read rank 0's weights: their plane rows are all zero
#pragma unroll
      for (int i = 0; i < FS; ++i) {
        const int src = which ? FS - 1 - i : i;
        fh[i] = a.FH[src * R + (r < R ? r : 0)];
        fw[i] = a.FW[src * R + (r < R ? r : 0)];
      }
    }
    // (a) clear the plane (borders, halo rows outside the image, padding ranks); the
    // previous item's tap step is over (barrier before its GEMM), its GEMM reads fragments only
    {
      float4* p4 = reinterpret_cast<float4*>(plane);
      for (int i = tid; i < (RP * PSt) >> 2; i += 512) p4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();
    plane_store(0);
    for (int kb = 1; kb * KM < per; ++kb) {
      plane_load(kb);
      plane_store(kb);
    }
    __syncthreads();
    // (c) taps: unit = (rank r, octet o of the strip's pixels) -> 8 values of Cc / G1,
    // split into the B fragment entry of (step o/2, half o&1, rank)
    for (int u = tid; u < RP * 2 * KS; u += 512) {
      const int o = u / RP;
      const int qb = q0 + 8 * o;
      u32x4* dst = frag + ((size_t)((r >> 5) * (a.KSmax + 1) + (o >> 1)) * 6 + (o & 1)) * 32 + (r & 31);
      if (qb >= q1) {                                  // an octet past the strip
        const u32x4 z = {0u, 0u, 0u, 0u};
        dst[0] = z;
        dst[64] = z;
        dst[128] = z;
        continue;
      }
      const int h = (int)__umulhi((unsigned)qb, a.wmagic), w = qb - h * W;
      const int k = W - w;       // pixels j < k lie in row h (window position j), the others
                                 // in row h + 1 (window position j + 2Q, past the two borders)
      const float* c0 = plane + (size_t)r * PSt + (h - h0) * Wp + w;
      const bool tapgrad = tapgroup && (TG == 1 || ((o >> (RB == 1 ? 1 : 0)) & 1) == cg);   // wave-uniform
      float B[WN];
#pragma unroll
      for (int x = 0; x < WN; ++x) B[x] = 0.f;
      // tap gradients: G3 of the octet, spread to window positions
      float gx[NX];
      if (tapgrad) {
        float g[8];
        const float* gp = a.Zsrc1 + ((size_t)n * R + (r < R ? r : 0)) * HW + qb;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
          if (qb + 4 * j < HW) v = *reinterpret_cast<const float4*>(gp + 4 * j);
          g[4 * j] = v.x; g[4 * j + 1] = v.y; g[4 * j + 2] = v.z; g[4 * j + 3] = v.w;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (qb + j >= q1) g[j] = 0.f;
#pragma unroll
        for (int x = 0; x < NX; ++x) {
          const float lo = x < 8 ? g[x < 8 ? x : 0] : 0.f;
          const float up = x >= 2 * Q ? g[x >= 2 * Q ? x - 2 * Q : 0] : 0.f;
          gx[x] = x < k ? lo : (x >= k + 2 * Q ? up : 0.f);
        }
      }
#pragma unroll
      for (int i = 0; i < FS; ++i) {
        float av[WN];
#pragma unroll
        for (int x = 0; x < WN; ++x) av[x] = c0[i * Wp + x];
#pragma unroll
        for (int x = 0; x < WN; ++x) B[x] += fh[i] * av[x];
        if (tapgrad) {
          float s = 0.f;
#pragma unroll
          for (int x = 0; x < NX; ++x) {
            float hr = 0.f;
#pragma unroll
            for (int t = 0; t < FS; ++t) hr += fw[t] * av[x + t];
            s += gx[x] * hr;
          }
          gh[i] += s;
        }
      }
      float call[NX];
#pragma unroll
      for (int x = 0; x < NX; ++x) {
        float s = 0.f;
#pragma unroll
        for (int t = 0; t < FS; ++t) s += fw[t] * B[x + t];
        call[x] = s;
      }
      if (tapgrad) {
#pragma unroll
        for (int t = 0; t < FS; ++t) {
          float s = 0.f;
#pragma unroll
          for (int x = 0; x < NX; ++x) s += gx[x] * B[x + t];
          gw[t] += s;
        }
      }
      float out[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float v = j < k ? call[j] : call[j + 2 * Q];
        out[j] = (qb + j < q1) ? v : 0.f;
      }
      u32x4 ph, pm, pl;
      split8(out, ph, pm, pl);
      dst[0] = ph;
      dst[64] = pm;
      dst[128] = pl;
    }
    __syncthreads();
    // (d) this wave's steps of the GEMM: acc[rb] += act[32 rows][16 px] . Z[16 px][32 ranks]
    auto gemm_step = [&](const float4 (&rv)[2], int s) {
      const float v[8] = {rv[0].x, rv[0].y, rv[0].z, rv[0].w, rv[1].x, rv[1].y, rv[1].z, rv[1].w};
      u32x4 ah, am, al;
      split8(v, ah, am, al);
      const int sf = s < KS ? s : a.KSmax;             // steps past the last: the zero step
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const u32x4* zp = frag + ((size_t)(rb * (a.KSmax + 1) + sf) * 6 + hi) * 32 + l32;
        acc[rb] = mfma_split(ah, am, al, zp[0], zp[64], zp[128], acc[rb]);
      }
    };
    for (int sb = kh; sb < KS; sb += KH * kRing) {
#pragma unroll
      for (int u = 0; u < kRing; ++u) {
        const int s = sb + u * KH;
        float4 rv[2] = {ring[u][0], ring[u][1]};
        issue(ring[u], s + kRing * KH);
        gemm_step(rv, s);
        // keep the steps in program order: the refill above must stay behind the loads
        // of the following steps, or their waits would cover it too
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- tail: partial sums of this workgroup ----
  __syncthreads();
  float* red = lds;
  if (KH > 1) {
    // the KH waves of a channel tile hold the sums of interleaved steps: added in wave order
    if (kh > 0) {
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) red[((wave * RB + rb) * 16 + v) * 64 + lane] = acc[rb][v];
    }
    __syncthreads();
    if (kh == 0) {
      for (int k2 = 1; k2 < KH; ++k2)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int v = 0; v < 16; ++v)
            acc[rb][v] += red[(((wave + k2) * RB + rb) * 16 + v) * 64 + lane];
    }
    __syncthreads();
  }
  if (kh == 0) {
    // ranks past R are masked through the lane offset; D is a multiple of 16, so a
    // 32-row tile is valid as a whole, in its first 16 rows (v < 8) or not at all
    const __amdgpu_buffer_rsrc_t ors = __builtin_amdgcn_make_buffer_rsrc(
        (which ? a.part1 : a.part0) + (size_t)sidx * D * R, 0, D * R * 4, 0x00020000);
    const int dbase = cg * 32 * MT + 32 * mt;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int rr = 32 * rb + l32;
      const unsigned vo = rr < R ? (unsigned)((dbase + 4 * hi) * R + rr) * 4u : 0x80000000u;
#pragma unroll
      for (int v = 0; v < 16; ++v)
        if (dbase + 16 * (v >> 3) < D) {                // wave-uniform
          const float val = acc[rb][v];
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), ors, vo,
                                                (unsigned)((8 * (v >> 2) + (v & 3)) * R) * 4u, 0);
        }
    }
  }
  if (tapgroup) {
    // thread t holds sums of rank t % RP: fixed-order sum over the 512 / RP threads of a rank
#pragma unroll
    for (int i = 0; i < FS; ++i) {
      red[i * 512 + tid] = gh[i];
      red[(FS + i) * 512 + tid] = gw[i];
    }
    __syncthreads();
    for (int e = tid; e < 2 * FS * RP; e += 512) {
      const int t = e / RP, rr = e - t * RP;
      float s = 0.f;
      for (int k2 = 0; k2 < 512 / RP; ++k2) s += red[t * 512 + k2 * RP + rr];
      if (rr < R) {
        if (t < FS) a.partH[((size_t)(sidx * TG + cg) * FS + t) * R + rr] = s;
        else a.partW[((size_t)(sidx * TG + cg) * FS + (t - FS)) * R + rr] = s;
      }
    }
  }
}

// ---- 3. out[i] = sum_s partial[s][i], four segments in one launch -------------------
struct ReduceFusedArgs {
  const float* part[4];
  float* out[4];
  int count[4], S[4];
};
// A workgroup owns 64 consecutive outputs; its four waves each sum a quarter of the
// S partials in index order, then the quarter sums are added in wave order.
__global__ __launch_bounds__(256) void reduce_fused_kernel(ReduceFusedArgs a) {
  __shared__ float quarter[4][64];
  const int seg = blockIdx.y;
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int i = blockIdx.x * 64 + lane;
  const int count = a.count[seg], S = a.S[seg];
  if ((int)blockIdx.x * 64 >= count) return;           // whole workgroup
  const int k0 = (int)((long)S * q / 4), k1 = (int)((long)S * (q + 1) / 4);
  float s = 0.f;
  if (i < count) {
    const float* p = a.part[seg] + i;
    const size_t stride = count;
    // sixteen loads in flight (one round trip for up to 64 partial sets), summed in index order
    for (int k = k0; k < k1; k += 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = k + u < k1 ? p[(size_t)(k + u) * stride] : 0.f;
#pragma unroll
      for (int u = 0; u < 16; ++u) s += v[u];
    }
  }
  quarter[q][lane] = s;
  __syncthreads();
  if (q == 0 && i < count)
    a.out[seg][i] = ((quarter[0][lane] + quarter[1][lane]) + quarter[2][lane]) + quarter[3][lane];
}

// ---- host side -----------------------------------------------------------------------
constexpr size_t kLdsBudget = 150 * 1024;

struct FusedPlan {
  bool ok;
  int RB, MT, ncg, TG, TH, NS, items, S, Q, Wp, PSt, KSmax;
  size_t lds;
  int ks, nw, ring;           // contraction: channel splits per item, waves per workgroup, chunks in flight
  size_t lds_contract;
  size_t plane, part_elems;   // floats
};

FusedPlan make_fused_plan(const cp4_shape& s) {
  FusedPlan p{};
  const int N = s.N, C = s.C, T = s.T, H = s.H, W = s.W, FS = s.Y, R = s.Rank;
  const int HW = H * W;
  p.RB = R <= 32 ? 1 : 2;
  const int RP = 32 * p.RB;
  p.Q = (FS - 1) / 2;
  p.Wp = W + 2 * p.Q;
  const int dmax = T > C ? T : C;
  const int cus = num_compute_units();
  double best = -1.;
  // 32-channel tiles per workgroup: no more than the channels fill, the eight waves
  // sharing a tile's pixel steps among them when there are fewer
  const int mt_max = dmax > 128 ? 8 : (dmax > 64 ? 4 : (dmax > 32 ? 2 : 1));
  for (int MT = mt_max; MT >= (mt_max > 4 ? 4 : mt_max); MT >>= 1) {
    const int ncg = (dmax + 32 * MT - 1) / (32 * MT);
    const int s_target = cus / (2 * ncg) > 0 ? cus / (2 * ncg) : 1;
    for (int TH = H; TH >= 1; --TH) {
      const int NS = (H + TH - 1) / TH;
      if (NS > 1 && ((TH * W) & 3)) continue;          // strips start on a 16-byte boundary
      int pst = (TH + 2 * p.Q + 1) * p.Wp + 16;
      pst |= 1;
      const int KS = (TH * W + 15) / 16;
      const size_t lds = (size_t)RP * pst * 4 + (size_t)p.RB * (KS + 1) * kFragBytes;
      if (lds > kLdsBudget) continue;
      const int items = N * NS;
      const int S = items < s_target ? items : s_target;
      const int rounds = (items + S - 1) / S;
      // per item: the GEMM steps of a wave, the tap step (replicated per channel
      // group), and barriers / first-load latency
      const double item_cost = (double)TH * W * (MT / 8.0) + 0.6 * (TH + 2 * p.Q) * W + 400.;
      const double cost = rounds * item_cost;
      if (best < 0 || cost < best) {
        best = cost;
        p.ok = true;
        p.MT = MT; p.ncg = ncg; p.TH = TH; p.NS = NS; p.items = items; p.S = S;
        p.PSt = pst; p.KSmax = KS; p.lds = lds;
      }
    }
  }
  if (!p.ok) return p;
  // the tail's cross-wave sums use the same allocation
  const size_t tail_gemm = (size_t)8 * p.RB * 16 * 64 * 4, tail_taps = (size_t)2 * FS * 512 * 4;
  if (p.lds < tail_gemm) p.lds = tail_gemm;
  if (p.lds < tail_taps) p.lds = tail_taps;
  // contraction: 32-pixel blocks of x and of dy are the wave items; with few of them
  // 2 or 4 waves share an item (a slice of the channels each) until there are about
  // three waves per compute unit, and a workgroup is four waves (one per SIMD, an
  // eight-chunk load ring) unless the items alone fill the chip twice over
  const int npb = (HW + 31) / 32;
  const long wave_items = 2L * N * npb;
  p.ks = 1;
  const int nch_min = (C < T ? C : T) >> 4;
  while (p.ks < 4 && wave_items * p.ks < 3L * cus && ((C >> 4) % (2 * p.ks)) == 0 &&
         ((T >> 4) % (2 * p.ks)) == 0 && nch_min / (2 * p.ks) >= 2)
    p.ks *= 2;
  p.nw = wave_items * p.ks <= 5L * cus ? 4 : 8;
  p.ring = p.nw == 4 ? 8 : 4;
  p.lds_contract = ((size_t)dmax / 16 + 1) * p.RB * kFragBytes;   // + the zero block
  const size_t red = (size_t)p.nw * p.RB * 16 * 64 * 4;
  if (p.ks > 1 && p.lds_contract < red) p.lds_contract = red;
  p.plane = ((size_t)N * R * HW + 63) & ~(size_t)63;
  p.TG = (T + 32 * p.MT - 1) / (32 * p.MT) >= 2 ? 2 : 1;   // among dFK's own channel groups
  p.part_elems = (size_t)p.S * R * ((size_t)T + C + 2 * FS * p.TG);
  return p;
}

}  // namespace

bool bwd_filter_fused_supported(const cp4_shape& s) {
  const bool odd_square = s.Y == s.X && (s.Y == 1 || s.Y == 3 || s.Y == 5);
  if (!odd_square || 2 * s.pad != s.Y - 1 || s.Rank > 64) return false;
  if ((s.C & 15) || (s.T & 15) || ((s.H * s.W) & 3) || s.W < 8 || s.W > 4096) return false;
  if (!fits_int_indexing((int)s.N, (int)s.H, (int)s.W) || (size_t)s.H * s.W > (1u << 20)) return false;
  const size_t dmax = s.C > s.T ? s.C : s.T;
  if ((dmax / 16 + 1) * (s.Rank <= 32 ? 1 : 2) * kFragBytes > kLdsBudget) return false;
  if (dmax * s.H * s.W >= ((size_t)1 << 29)) return false;    // an image's channels behind one 32-bit descriptor
  return make_fused_plan(s).ok;
}

// Measured on one MI355X against the four-launch variant over 150 shapes (the library's
// own timed loop): the three-launch variant is ahead wherever the batch holds up to
// 25,000 pixels or so (17-20 us against 21-25 on the smallest layers, N16 C128 28x28
// R16 19.9 against 26.6, N8 C256 56x56 R32 36.3 against 38.5), and on planes of up to
// 32 x 32 pixels up to 65,000 (N64 C256 28x28 R64: 93.7 against 105.9 us).  Beyond
// that, and from 50,000 pixels on planes of 56 x 56 and more, its plane copy, tap step
// and GEMM - one after the other in a workgroup that has the compute unit to itself -
// cost more than the launch and the planes they save (N16 C64 56x56 R16: 37.3 against
// 32.7 us, N8 C32 112x112: 63.9 against 44.9).  On planes of up to 256 pixels with more
// than 32 ranks one partial set per image outweighs the planes from about 10 MB of
// activations on (N64 C256 14x14 R64: 36.3 against 34.0 us).
bool bwd_filter_fused_preferred(const cp4_shape& s) {
  if (!bwd_filter_fused_supported(s)) return false;
  const long plane = (long)s.H * s.W, pixels = plane * s.N;
  if (plane <= 256 && s.Rank > 32) return 4e-6 * s.N * ((double)s.C + s.T) * plane <= 10.;
  return pixels <= 25088 || (plane <= 1024 && pixels <= 65536);
}

size_t bwd_filter_fused_workspace_bytes(const cp4_shape& s) {
  const FusedPlan p = make_fused_plan(s);
  return (2 * p.plane + p.part_elems) * sizeof(float);
}

hipError_t bwd_filter_fused_launch(const BwdFilterArgs& a, hipStream_t st) {
  cp4_shape s{};
  s.N = a.N; s.C = a.C; s.T = a.T; s.H = a.H; s.W = a.W; s.pad = a.pad; s.Y = a.Y; s.X = a.X;
  s.Rank = a.R;
  const FusedPlan p = make_fused_plan(s);
  if (!p.ok) return hipErrorInvalidValue;
  const int HW = a.H * a.W, R = a.R, N = a.N, FS = a.Y;
  float* ws = static_cast<float*>(a.workspace);
  float *A = ws, *G3 = ws + p.plane, *part = ws + 2 * p.plane;
  float* pK = part;
  float* pC = pK + (size_t)p.S * a.T * R;
  float* pH = pC + (size_t)p.S * a.C * R;
  float* pW = pH + (size_t)p.S * p.TG * FS * R;

  ContractAllArgs c{};
  c.src0 = a.x; c.F0 = a.FC; c.Z0 = A; c.Cin0 = a.C;
  c.src1 = a.dy; c.F1 = a.FK; c.Z1 = G3; c.Cin1 = a.T;
  c.R = R; c.HW = HW; c.npb = (HW + 31) / 32; c.items = N * c.npb;
  c.vecfill = (R & 3) == 0 && ((reinterpret_cast<uintptr_t>(a.FC) | reinterpret_cast<uintptr_t>(a.FK)) & 15) == 0;
  const long slots = (long)c.items * p.ks;
  const dim3 cgrid((unsigned)((slots + p.nw - 1) / p.nw), 2);
  hipError_t e;
#define CP4_CONTRACT(RB_, KS_, RING_)                                                          \
  {                                                                                            \
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(contract_all_kernel<RB_, KS_, RING_>), \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)p.lds_contract);  \
    if (e != hipSuccess) return e;                                                             \
    contract_all_kernel<RB_, KS_, RING_><<<cgrid, p.nw * 64, p.lds_contract, st>>>(c);         \
  }
#define CP4_CONTRACT_KS(RB_, RING_)                                                            \
  {                                                                                            \
    if (p.ks == 1) CP4_CONTRACT(RB_, 1, RING_)                                                 \
    else if (p.ks == 2) CP4_CONTRACT(RB_, 2, RING_)                                            \
    else CP4_CONTRACT(RB_, 4, RING_)                                                           \
  }
  if (p.RB == 1) {
    if (p.ring == 8) CP4_CONTRACT_KS(1, 8) else CP4_CONTRACT_KS(1, 4)
  } else {
    if (p.ring == 8) CP4_CONTRACT_KS(2, 8) else CP4_CONTRACT_KS(2, 4)
  }
#undef CP4_CONTRACT_KS
#undef CP4_CONTRACT

  FusedArgs g{};
  g.act0 = a.dy; g.Zsrc0 = A; g.part0 = pK; g.D0 = a.T;
  g.act1 = a.x; g.Zsrc1 = G3; g.part1 = pC; g.D1 = a.C;
  g.FH = a.FH; g.FW = a.FW; g.partH = pH; g.partW = pW;
  g.N = N; g.R = R; g.H = a.H; g.W = a.W; g.P = a.pad; g.HW = HW;
  g.TG = p.TG; g.TH = p.TH; g.NS = p.NS; g.items = p.items; g.S = p.S; g.MT = p.MT;
  g.Wp = p.Wp; g.PSt = p.PSt; g.KSmax = p.KSmax;
  g.wmagic = (unsigned)(0x100000000ull / (unsigned)a.W) + 1u;
  const dim3 ggrid(p.S, p.ncg, 2);
#define CP4_FUSED(FS_, RB_)                                                                   \
  {                                                                                           \
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(grad_fused_kernel<FS_, RB_>),       \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)p.lds);          \
    if (e != hipSuccess) return e;                                                            \
    grad_fused_kernel<FS_, RB_><<<ggrid, 512, p.lds, st>>>(g);                                \
  }
#define CP4_FUSED_FS(FS_)                                 \
  {                                                       \
    if (p.RB == 1) CP4_FUSED(FS_, 1) else CP4_FUSED(FS_, 2) \
  }
  switch (FS) {
    case 1: CP4_FUSED_FS(1) break;
    case 3: CP4_FUSED_FS(3) break;
    default: CP4_FUSED_FS(5) break;
  }
#undef CP4_FUSED_FS
#undef CP4_FUSED

  ReduceFusedArgs r{};
  const float* parts[4] = {pK, pC, pH, pW};
  float* outs[4] = {a.dFK, a.dFC, a.dFH, a.dFW};
  const int counts[4] = {a.T * R, a.C * R, FS * R, FS * R};
  int maxc = 0;
  for (int i = 0; i < 4; ++i) {
    r.part[i] = parts[i]; r.out[i] = outs[i]; r.count[i] = counts[i];
    r.S[i] = i < 2 ? p.S : p.S * p.TG;
    if (counts[i] > maxc) maxc = counts[i];
  }
  reduce_fused_kernel<<<dim3((maxc + 63) / 64, 4), 256, 0, st>>>(r);
  return hipGetLastError();
}


}  // namespace cp4
