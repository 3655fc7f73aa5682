// Fused forward / backward-data kernel for layers with few channels and up to 16 ranks on
// planes of any width: persistent four-wave workgroups over 2-D tiles, the tap step and
// the output contraction in registers.
//
// Same arithmetic as the other matrix-core kernels (the reassociated form of
// Cuda_kernels/cp4Conv2dForward.cu:84-133; backward-data,
// cp4Conv2dBackwardData.cu:57-108, through swapped factors and reversed taps): exact fp32
// products as six bf16 MFMAs on three-way split operands, taps in fp32 on the vector units.
//
// With 16 channels a side the sixteen-wave producer / consumer kernel is bound by what a
// workgroup spends before and after its pipeline runs (thousands of tiles, each a
// workgroup of its own) and by LDS round trips between its waves.  Here
//   * a workgroup of four waves keeps its factor fragments and walks over tiles of
//     TH x TW output pixels (TW = 32, 64 or 128); up to four workgroups share a compute
//     unit, so one's loads overlap another's arithmetic;
//   * P1  A[r, cell] = sum_c Fin[c, r] x[c, cell] over the tile and its halo (a plane of
//     (TH + FS - 1) x (TW + FS - 1) cells, zero outside the image): a wave takes 32-cell
//     blocks, x straight from memory through a register ring that runs across blocks; A
//     goes to LDS by rank quads, [r / 4][cell][r % 4];
//   * barrier;
//   * P2 + P3  a wave takes 64 consecutive pixels of a tile row: the lane that holds
//     ranks 8*hi ... 8*hi + 7 of pixels 2*l32 and 2*l32 + 1 in the MFMA B operand computes
//     exactly those tap results (two rank quads, two neighbouring pixels: a 3 x 4 window
//     of 16-byte LDS cells per quad), splits them in registers and multiplies by the
//     output factor: no fragment tile in LDS, no barrier between the two steps.  float2
//     stores with the bias / activation epilogue;
//   * barrier (the plane is free for the next tile).
// Out-of-image cells are zeros in the plane, so the tap step needs no masks.
#include <cstring>

#include "cp4_internal.h"
#include "split_bf16.h"

namespace cp4 {
namespace {

using namespace split;

constexpr int kMaxRank = 16;

struct FewPlan {
  int TH, TW, lgTW;
  int tilesX, tilesY, ntiles;
  int PS;              // cells per plane row: TW + FS - 1
  int cells;           // plane cells: (TH + FS - 1) * PS
  int nblk_first;      // 32-cell blocks of the whole plane (a run's first tile)
  int nblk_next;       // ... and of a tile's TH new rows (the tiles below it)
  int seg, parts;      // tiles per run; runs per column of tiles
  int nunits;          // runs in all
  int QA;              // cells per rank quad in LDS (a multiple of 32)
  int quads;           // rank quads of A
  int ngroups;         // 64-pixel groups of a tile
  int nkb;             // blocks of 32 output channels
  unsigned psmagic;    // ceil(2^32 / PS)
  unsigned ptmagic;    // ceil(2^32 / (parts * tilesX))
  unsigned txmagic;    // ceil(2^32 / tilesX)
  int w_off;           // byte offset of the tap weights in LDS
  int f_off;           // ... and of the factor fragments
  int nw;              // waves per workgroup (4 or 8)
  int grid;
  size_t lds_bytes;
};

// FS: filter size; NCH: 16-channel chunks of the input (1, 2 or 4); RING: chunk loads in
// flight per lane, a multiple of NCH; OCC: waves per SIMD the register budget is set for.
template <int FS, int NCH, int RING, int OCC, int NW>
__global__ __launch_bounds__(64 * NW, OCC) void fwd_few_kernel(FwdArgs a, FewPlan pl) {
  constexpr int kWaves = NW;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float4* As4 = reinterpret_cast<float4*>(lds_raw);                  // [quads][QA]
  float* wl = reinterpret_cast<float*>(lds_raw + pl.w_off);          // FH then FW, [FS][16] each

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  const int H = a.H, W = a.W, HW = H * W, R = a.R, Cin = a.Cin, Cout = a.Cout;
  const int QA = pl.QA, PS = pl.PS, TW = pl.TW;

  u32x4* frag = reinterpret_cast<u32x4*>(lds_raw + pl.f_off);      // [NCH + nkb][3][64]
  const int nkb = pl.nkb;

  // Work units are runs of `seg` vertically adjacent tiles (a column of the image, or a part
  // of one): a workgroup walks down its run and keeps the last FS - 1 rows of a tile's A
  // plane in LDS for the tile below, so only a run's first tile contracts halo rows.  The
  // plane's rows are a ring: row r of a run (counted from the run's first plane row) lives
  // in slot r mod PH.  An XCD (workgroup index mod 8) gets a contiguous range of units,
  // which its workgroups walk through side by side: runs that share halo columns are read
  // at about the same time through the same L2.
  constexpr bool kSlide = FS > 1;
  const int PH = pl.TH + FS - 1;
  const int per = (pl.nunits + 7) >> 3;
  const int xcd = blockIdx.x & 7, gj = gridDim.x >> 3;
  // Where a tile lies: image, first output row and column; the ring slot of its first plane
  // row; whether it is the first of its run (its whole plane is contracted).
  struct Tile {
    int n, h0, w0, slot0, first;
  };
  struct Cursor {
    int ju, k, cnt, n, ty0, tx;
    int slot0;       // (k * TH) mod PH, kept as the cursor moves
  };
  auto unit_at = [&](int ju) {
    const int u = xcd * per + ju;
    const int pt = pl.parts * pl.tilesX;
    // (divisions by multiplication: a division proper is some forty instructions before
    // a tile's first load can go out; the host has checked that the products are exact)
    const int n = pt == 1 ? u : (int)__umulhi((unsigned)u, pl.ptmagic), rem = u - n * pt;
    const int part = pl.tilesX == 1 ? rem : (int)__umulhi((unsigned)rem, pl.txmagic);
    const int tx = rem - part * pl.tilesX;
    const int ty0 = part * pl.seg;
    const int cnt = pl.tilesY - ty0 < pl.seg ? pl.tilesY - ty0 : pl.seg;
    // (the high products come from the vector unit: say that they are wave-uniform)
    return Cursor{ju, 0, __builtin_amdgcn_readfirstlane(cnt), __builtin_amdgcn_readfirstlane(n),
                  __builtin_amdgcn_readfirstlane(ty0), __builtin_amdgcn_readfirstlane(tx), 0};
  };
  auto has_unit = [&](int ju) { return ju < per && xcd * per + ju < pl.nunits; };
  auto tile_at = [&](const Cursor& c) {
    return Tile{c.n, (c.ty0 + c.k) * pl.TH, c.tx * TW, kSlide ? c.slot0 : 0, !kSlide || c.k == 0};
  };
  // The cursor after c, and whether there is one.
  auto advance = [&](const Cursor& c, bool& more) {
    if (c.k + 1 < c.cnt) {
      more = true;
      Cursor d = c;
      d.k = c.k + 1;
      d.slot0 = c.slot0 + pl.TH >= PH ? c.slot0 + pl.TH - PH : c.slot0 + pl.TH;
      return d;
    }
    more = has_unit(c.ju + gj);
    return more ? unit_at(c.ju + gj) : c;
  };

  // P1's loads: the wave's (block, chunk) steps of a tile in order, step s in ring slot
  // s % RING; the ring runs on across tiles, so the first loads of the next tile are in
  // flight while this one's taps and output contraction run.  A run's first tile has
  // nblk_first blocks (the whole plane), the others nblk_next (their TH new rows).
  auto steps_of = [&](bool first) {
    const int nblk = first ? pl.nblk_first : pl.nblk_next;
    return (wave < nblk ? (nblk - wave + kWaves - 1) / kWaves : 0) * NCH;
  };
  // ... padded to whole turns of the ring, so that a step of any tile has the same slot;
  // the padding steps load the tile's last chunk again and are not used
  auto padded = [&](int nsteps) { return (nsteps + RING - 1) / RING * RING; };
  float xb[RING][8];
  int cellv[RING];     // the slot's LDS cell; bit 30: outside the image (zero); -1: not a cell
  auto issue = [&](int slot, const Tile& tl, int step, int c) {   // c == step % NCH, given statically
    const int rows = tl.first ? PH : pl.TH, prow0 = tl.first ? 0 : FS - 1;
    const int qa = 32 * (wave + kWaves * (step / NCH)) + l32;
    const int pr = (int)__umulhi((unsigned)qa, pl.psmagic), pc = qa - pr * PS;
    const int prow = prow0 + pr;                        // row of the tile's plane
    const int h = tl.h0 - a.pad + prow, w = tl.w0 - a.pad + pc;
    const bool cell = pr < rows;
    const bool inside = h >= 0 && h < H && w >= 0 && w < W;
    const int hc = h < 0 ? 0 : (h > H - 1 ? H - 1 : h), wc = w < 0 ? 0 : (w > W - 1 ? W - 1 : w);
    const unsigned voff = (unsigned)(8 * hi * HW + hc * W + wc) * 4u;
    // x through a buffer descriptor over the tile's image: reads past its last channel return 0
    const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(a.x + (size_t)tl.n * Cin * HW), 0, Cin * HW * 4, 0x00020000);
    const unsigned soff = (unsigned)(16 * c) * (unsigned)HW * 4u;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      xb[slot][e] = __builtin_bit_cast(          // (the scalar offset said to be wave-uniform: held in
          float,                                   // a vector register it would cost a loop per load)
          __builtin_amdgcn_raw_buffer_load_b32(
              xrs, voff, __builtin_amdgcn_readfirstlane(soff + (unsigned)e * HW * 4u), 0));
    int ring_row = tl.slot0 + prow;
    ring_row = ring_row >= PH ? ring_row - PH : ring_row;
    cellv[slot] = !cell ? -1 : (ring_row * PS + pc) | (inside ? 0 : 0x40000000);
  };
  // Step `step` of the tile (or, past its last step, of the tile after it; with no tile
  // after it the last step once more: loads stay unconditional).
  auto issue_from = [&](int slot, const Tile& cur, const Tile& nxt, bool more, int step, int c) {
    const bool over = step >= padded(steps_of(cur.first)) && more;
    const int nsteps = steps_of(over ? nxt.first : cur.first);
    int st = over ? step - padded(steps_of(cur.first)) : step;
    st = st < nsteps ? st : nsteps - NCH + c;
    st = st < 0 ? c : st;                               // (a tile of which this wave has no block)
    Tile tl;
    tl.n = over ? nxt.n : cur.n;
    tl.h0 = over ? nxt.h0 : cur.h0;
    tl.w0 = over ? nxt.w0 : cur.w0;
    tl.slot0 = over ? nxt.slot0 : cur.slot0;
    tl.first = over ? nxt.first : cur.first;
    issue(slot, tl, st, c);
  };

  if (!has_unit(blockIdx.x >> 3)) return;
  Cursor cu = unit_at(blockIdx.x >> 3);
  Tile cur = tile_at(cu);
  const bool loads = steps_of(true) > 0;                // (a wave with no block of any tile loads nothing)
  if (loads) {
    const int nsteps = steps_of(true);
#pragma unroll
    for (int u = 0; u < RING; ++u) issue(u, cur, u < nsteps ? u : nsteps - NCH + u % NCH, u % NCH);
  }
  // (the first tile's loads are out: what follows waits for memory of its own)

  // tap weights -> LDS (rows of 16 ranks, zero past the last rank)
  for (int i = tid; i < 2 * FS * 16; i += 64 * kWaves) {
    const int which = i / (FS * 16), rem = i - which * FS * 16;
    const int j = rem >> 4, r = rem & 15;
    const int tap = a.flip ? FS - 1 - j : j;
    const float* src = which ? a.FW : a.FH;
    wl[i] = r < R ? src[tap * R + r] : 0.f;
  }
  // Factor fragments, pre-split, in LDS as the lanes read them back (48 bytes a lane: parts
  // h, m, l of 8 bf16 each): kept in registers they would cost a quarter of a wave's budget.
  // Input factor: chunk c, lane (l32, hi) holds rank l32, channels 16*c + 8*hi + e.
  // Output factor: block kb, lane holds row 32*kb + l32, ranks 8*hi + e.
  for (int item = wave; item < NCH + nkb; item += kWaves) {
    float v[8];
    if (item < NCH) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int ch = 16 * item + 8 * hi + e;
        v[e] = (l32 < R && ch < Cin) ? a.Fin[(size_t)ch * R + l32] : 0.f;
      }
    } else {
      const int k = 32 * (item - NCH) + l32;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int r = 8 * hi + e;
        v[e] = (k < Cout && r < R) ? a.Fout[(size_t)k * R + r] : 0.f;
      }
    }
    u32x4 h, m, l;
    split8(v, h, m, l);
    frag[(item * 3 + 0) * 64 + lane] = h;
    frag[(item * 3 + 1) * 64 + lane] = m;
    frag[(item * 3 + 2) * 64 + lane] = l;
  }
  __syncthreads();

  for (;;) {
    bool more;
    const Cursor cn = advance(cu, more);
    const Tile nxt = more ? tile_at(cn) : cur;
    const int n = cur.n, h0 = cur.h0, w0 = cur.w0;

    // ---- P1: channel -> rank contraction over the tile's new plane rows -------------
    if (loads) {
      const int nsteps = steps_of(cur.first);
      f32x16 acc = (f32x16)(0.f);
      for (int s0 = 0; s0 < nsteps; s0 += RING) {
#pragma unroll
        for (int u = 0; u < RING; ++u) {
          const int c = u % NCH;
          if (s0 + u < nsteps) {                        // (the same for all lanes)
            if (c == 0) acc = (f32x16)(0.f);
            u32x4 xh, xm, xl;
            split8(xb[u], xh, xm, xl);
            acc = mfma_split(frag[(c * 3 + 0) * 64 + lane], frag[(c * 3 + 1) * 64 + lane],
                             frag[(c * 3 + 2) * 64 + lane], xh, xm, xl, acc);
            if (c == NCH - 1 && cellv[u] >= 0) {
              const int cell = cellv[u] & 0x3fffffff;
              const bool valid = !(cellv[u] & 0x40000000);
              // accumulator element v: rank 8*(v >> 2) + 4*hi + (v & 3), i.e. quad 2*(v >> 2) + hi
#pragma unroll
              for (int q2 = 0; q2 < 2; ++q2) {
                const int quad = 2 * q2 + hi;
                if (quad < pl.quads) {
                  float4 o;
                  o.x = valid ? acc[4 * q2] : 0.f;
                  o.y = valid ? acc[4 * q2 + 1] : 0.f;
                  o.z = valid ? acc[4 * q2 + 2] : 0.f;
                  o.w = valid ? acc[4 * q2 + 3] : 0.f;
                  As4[quad * QA + cell] = o;
                }
              }
            }
          }
          issue_from(u, cur, nxt, more, s0 + u + RING, c);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    __syncthreads();

    // ---- P2 + P3: taps in registers, rank -> output-channel contraction ------------
    const __amdgpu_buffer_rsrc_t yrs = __builtin_amdgcn_make_buffer_rsrc(
        a.y + (size_t)n * Cout * HW, 0, Cout * HW * 4, 0x00020000);
    const bool pair_ok = (W & 1) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 7) == 0;
    for (int g = wave; g < pl.ngroups; g += kWaves) {
      const int p0 = 64 * g + 2 * l32;                 // the lane's pixels p0, p0 + 1 of the tile
      const int row = p0 >> pl.lgTW, col = p0 & (TW - 1);
      int ring_row[FS];                                // ring slots of the FS plane rows under the pixel
#pragma unroll
      for (int i = 0; i < FS; ++i) {
        int r = cur.slot0 + row + i;                   // (below 2 * PH)
        ring_row[i] = r >= PH ? r - PH : r;
      }
      float v0[8], v1[8];
#pragma unroll
      for (int qi = 0; qi < 2; ++qi) {
        const int quad = 2 * hi + qi;
        const bool live = quad < pl.quads;
        const float4* ar = As4 + (live ? quad : 0) * QA + col;
        const float* wq = wl + 4 * quad;
        float s0[4] = {0.f, 0.f, 0.f, 0.f}, s1[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < FS; ++i) {
          float4 cell[FS + 1];
#pragma unroll
          for (int jj = 0; jj <= FS; ++jj) cell[jj] = ar[__mul24(ring_row[i], PS) + jj];
          float h0s[4] = {0.f, 0.f, 0.f, 0.f}, h1s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int jj = 0; jj < FS; ++jj) {
            const float4 f = *reinterpret_cast<const float4*>(wq + FS * 16 + 16 * jj);
            h0s[0] += f.x * cell[jj].x;
            h0s[1] += f.y * cell[jj].y;
            h0s[2] += f.z * cell[jj].z;
            h0s[3] += f.w * cell[jj].w;
            h1s[0] += f.x * cell[jj + 1].x;
            h1s[1] += f.y * cell[jj + 1].y;
            h1s[2] += f.z * cell[jj + 1].z;
            h1s[3] += f.w * cell[jj + 1].w;
          }
          const float4 gq = *reinterpret_cast<const float4*>(wq + 16 * i);
          s0[0] += gq.x * h0s[0];
          s0[1] += gq.y * h0s[1];
          s0[2] += gq.z * h0s[2];
          s0[3] += gq.w * h0s[3];
          s1[0] += gq.x * h1s[0];
          s1[1] += gq.y * h1s[1];
          s1[2] += gq.z * h1s[2];
          s1[3] += gq.w * h1s[3];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          v0[4 * qi + q] = live ? s0[q] : 0.f;
          v1[4 * qi + q] = live ? s1[q] : 0.f;
        }
      }
      const int h = h0 + row, w = w0 + col;
      const bool in0 = h < H && w < W, in1 = h < H && w + 1 < W;
      // Stores through a buffer descriptor over the image's output planes: a store past its
      // range is dropped, so channels past the last one need no test, and a pixel outside
      // the image gets an offset past the range.
      const unsigned vo = (unsigned)(4 * hi * HW + h * W + w) * 4u;
      const unsigned vo0 = in0 ? vo : 0x80000000u, vo1 = in1 ? vo + 4u : 0x80000000u;
      const bool relu = a.act == 1;
      for (int kb = 0; kb < nkb; ++kb) {
        const u32x4 kh = frag[((NCH + kb) * 3 + 0) * 64 + lane];
        const u32x4 km = frag[((NCH + kb) * 3 + 1) * 64 + lane];
        const u32x4 kl = frag[((NCH + kb) * 3 + 2) * 64 + lane];
        f32x16 acc0, acc1;
        {
          u32x4 bh, bm, bl;
          split8(v0, bh, bm, bl);
          acc0 = mfma_split(kh, km, kl, bh, bm, bl, (f32x16)(0.f));
        }
        {
          u32x4 bh, bm, bl;
          split8(v1, bh, bm, bl);
          acc1 = mfma_split(kh, km, kl, bh, bm, bl, (f32x16)(0.f));
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int kk = 32 * kb + 8 * (v >> 2) + (v & 3);       // + 4*hi is in the lane offset
          if (kk < Cout) {                                       // (the same for all lanes)
            float o0 = acc0[v], o1 = acc1[v];
            if (a.bias) {
              const int k = kk + 4 * hi;
              const float bv = a.bias[k < Cout ? k : Cout - 1];
              o0 += bv;
              o1 += bv;
            }
            if (relu) {                                          // (a NaN stays a NaN)
              o0 = o0 < 0.f ? 0.f : o0;
              o1 = o1 < 0.f ? 0.f : o1;
            }
            const unsigned so = __builtin_amdgcn_readfirstlane((unsigned)kk * (unsigned)HW * 4u);
            if (pair_ok) {                                       // (W even: both pixels or neither)
              u32x2 o = {__float_as_uint(o0), __float_as_uint(o1)};
              __builtin_amdgcn_raw_buffer_store_b64(o, yrs, vo0, so, 0);
            } else {
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(o0), yrs, vo0, so, 0);
              __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(o1), yrs, vo1, so, 0);
            }
          }
        }
      }
    }
    __syncthreads();
    if (!more) break;
    cur = nxt;
    cu = cn;
  }
}

bool layout(const FwdArgs& a, int TH, int lgTW, int nw, int cus, FewPlan* pl) {
  const int TW = 1 << lgTW, FS = a.Y;
  const long PS = TW + FS - 1, PH = TH + FS - 1, cells = PH * PS;
  const long QA = (cells + 31) / 32 * 32;
  const int quads = (a.R + 3) / 4, nkb = (a.Cout + 31) / 32, nch = a.Cin <= 16 ? 1 : (a.Cin <= 32 ? 2 : 4);
  const long as_bytes = quads * QA * 16, w_bytes = 2l * FS * 16 * 4, f_bytes = (long)(nch + nkb) * 3 * 64 * 16;
  const long lds = as_bytes + w_bytes + f_bytes;
  if (lds > 64 * 1024 || (TH * TW) % 64 != 0) return false;
  pl->TH = TH;
  pl->TW = TW;
  pl->lgTW = lgTW;
  pl->nw = nw;
  pl->tilesX = (a.W + TW - 1) / TW;
  pl->tilesY = (a.H + TH - 1) / TH;
  pl->ntiles = a.N * pl->tilesX * pl->tilesY;
  // Runs of vertically adjacent tiles: whole columns where those already give every workgroup
  // slot one, else as many parts of a column as bring the runs up to the slots.
  const long slots = (long)cus * (16 / nw), cols = (long)a.N * pl->tilesX;
  long parts = cols >= slots ? 1 : (slots + cols - 1) / cols;
  parts = parts > pl->tilesY ? pl->tilesY : parts;
  pl->seg = (int)((pl->tilesY + parts - 1) / parts);
  pl->parts = (pl->tilesY + pl->seg - 1) / pl->seg;
  pl->nunits = (int)(cols * pl->parts);
  pl->PS = (int)PS;
  pl->nblk_first = (int)((cells + 31) / 32);
  pl->nblk_next = (int)(((long)TH * PS + 31) / 32);
  pl->QA = (int)QA;
  pl->quads = quads;
  pl->ngroups = TH * TW / 64;
  pl->nkb = nkb;
  pl->psmagic = (unsigned)((0x100000000ull + PS - 1) / PS);
  // n / d as the high word of n * ceil(2^32 / d), exact while n * d < 2^32; a divisor of one
  // has no such multiplier and is tested for in the kernel
  const unsigned long long pt = (unsigned long long)pl->parts * pl->tilesX;
  if ((unsigned long long)pl->nunits * pt >= (1ull << 31)) return false;
  pl->ptmagic = pt < 2 ? 0u : (unsigned)((0x100000000ull + pt - 1) / pt);
  pl->txmagic = pl->tilesX < 2 ? 0u : (unsigned)((0x100000000ull + pl->tilesX - 1) / pl->tilesX);
  pl->w_off = (int)as_bytes;
  pl->f_off = (int)(as_bytes + w_bytes);
  pl->lds_bytes = (size_t)lds;
  const long grid = pl->nunits < slots ? pl->nunits : slots;
  pl->grid = (int)((grid + 7) / 8 * 8);
  return true;
}

// Tile and workgroup size by a model of the serial work of a workgroup's busiest wave per
// tile (blocks of the plane per wave in P1 - a run's first tile the whole plane, the others
// their new rows -, 64-pixel groups per wave in P2 + P3, the barriers), times the tiles a
// workgroup walks through, times what the waves that share a vector unit cost one another.
// Eight waves on tiles of 256 pixels or more, four on smaller ones; a tuned height / width /
// schedule (0: eight waves, 2: four) replaces the choice.
constexpr double kBlockCost = 1.0, kBlockFixed = 0.3, kGroupCost = 4.0, kGroupBlockCost = 2.0,
                 kTileFixed = 2.0, kNarrowTileCost = 8.0, kShareCost = 0.6;
bool plan_uncached(const FwdArgs& a, FewPlan* best);
// The plan of the last shape asked for, per thread: a launch asks twice (whether the kernel
// takes the shape, then with what), a training loop for the same few shapes over and over.
bool plan(const FwdArgs& a, FewPlan* best) {
  struct Key {
    int v[13];
    bool operator==(const Key& o) const { return !memcmp(v, o.v, sizeof(v)); }
  };
  static thread_local Key last_key{};
  static thread_local FewPlan last_plan{};
  static thread_local int last_ok = -1;
  const Key k{{a.N, a.Cin, a.Cout, a.H, a.W, a.pad, a.Y, a.X, a.R, a.tune_th, a.tune_lgwt, a.tune_split2,
               num_compute_units()}};
  if (last_ok < 0 || !(k == last_key)) {
    last_ok = plan_uncached(a, &last_plan) ? 1 : 0;
    last_key = k;
  }
  if (last_ok == 1) *best = last_plan;
  return last_ok == 1;
}
bool plan_uncached(const FwdArgs& a, FewPlan* best) {
  const int cus = num_compute_units();
  bool found = false;
  double best_cost = 0;
  const double nch = a.Cin <= 16 ? 1 : (a.Cin <= 32 ? 2 : 4);
  for (int lg = 5; lg <= 7; ++lg) {
    if (a.tune_lgwt && lg != a.tune_lgwt) continue;
    for (int TH = 1; TH <= 32; ++TH) {
      if (a.tune_th > 0 && TH != a.tune_th) continue;
      const int nw = a.tune_split2 == 1 ? 8 : (a.tune_split2 == 2 ? 4 : ((TH << lg) >= 256 ? 8 : 4));
      FewPlan pl;
      if (!layout(a, TH, lg, nw, cus, &pl)) continue;
      const long slots = (long)cus * (16 / nw);            // sixteen waves a compute unit
      auto per_wave = [&](int n) { return (double)((n + nw - 1) / nw); };
      // a run's tiles: one with the whole plane, seg - 1 with their new rows
      const double blocks = (per_wave(pl.nblk_first) + (pl.seg - 1) * per_wave(pl.nblk_next)) / pl.seg;
      const double wave_work = blocks * (kBlockCost * nch + kBlockFixed) +
                               per_wave(pl.ngroups) * (kGroupCost + kGroupBlockCost * pl.nkb) + kTileFixed;
      const long resident = pl.nunits >= slots ? 16 / nw : (pl.nunits + cus - 1) / cus;
      // beyond two waves a vector unit they share it, less what they hide of one another's waits
      const double share = resident * nw > 8 ? 1.0 + kShareCost * (resident * nw / 8.0 - 1.0) : 1.0;
      const double turns = (double)((pl.nunits + slots - 1) / slots) * pl.seg;
      // (short rows cost more per byte moved: 128-byte pieces at 32 columns, 512 at 128)
      const double cost = turns * wave_work * share * (1.0 + kNarrowTileCost / pl.TW);
      if (!found || cost < best_cost) {
        best_cost = cost;
        *best = pl;
        found = true;
      }
    }
  }
  return found;
}

template <int FS, int NCH, int RING, int OCC, int NW>
hipError_t launch_as(const FwdArgs& a, const FewPlan& pl, hipStream_t st) {
  fwd_few_kernel<FS, NCH, RING, OCC, NW><<<pl.grid, 64 * NW, pl.lds_bytes, st>>>(a, pl);
  return hipGetLastError();
}
template <int FS>
hipError_t launch_fs(const FwdArgs& a, const FewPlan& pl, hipStream_t st) {
  if (a.Cin <= 16) return pl.nw == 8 ? launch_as<FS, 1, 2, 4, 8>(a, pl, st) : launch_as<FS, 1, 2, 4, 4>(a, pl, st);
  if (a.Cin <= 32) return pl.nw == 8 ? launch_as<FS, 2, 2, 4, 8>(a, pl, st) : launch_as<FS, 2, 2, 4, 4>(a, pl, st);
  return pl.nw == 8 ? launch_as<FS, 4, 4, 4, 8>(a, pl, st) : launch_as<FS, 4, 4, 4, 4>(a, pl, st);
}

}  // namespace

bool fwd_few_supported(const FwdArgs& a) {
  if (a.R > kMaxRank || a.Cin > 64 || a.sh || a.dense || a.taps2d || a.ldf || a.ldx || a.accumulate)
    return false;
  if (a.Y != a.X || !(a.Y == 1 || a.Y == 3 || a.Y == 5) || a.pad > a.Y - 1) return false;
  if (!fits_int_indexing(a.N, a.H, a.W) || (size_t)a.Cin * a.H * a.W >= (1u << 28) ||
      (size_t)a.Cout * a.H * a.W >= (1u << 28))          // 32-bit buffer offsets, stores past the range dropped
    return false;
  if (a.x && (reinterpret_cast<uintptr_t>(a.x) & 3)) return false;
  FewPlan pl;
  return plan(a, &pl);
}

bool fwd_few_plan(const FwdArgs& a, int* rows, int* cols, int* workgroups) {
  FewPlan pl;
  if (!fwd_few_supported(a) || !plan(a, &pl)) return false;
  *rows = pl.TH;
  *cols = pl.TW;
  *workgroups = pl.grid;
  return true;
}

hipError_t fwd_few_launch(const FwdArgs& a, hipStream_t st) {
  FewPlan pl;
  if (!plan(a, &pl)) return hipErrorInvalidValue;
  switch (a.Y) {
    case 1: return launch_fs<1>(a, pl, st);
    case 3: return launch_fs<3>(a, pl, st);
    default: return launch_fs<5>(a, pl, st);
  }
}

}  // namespace cp4
