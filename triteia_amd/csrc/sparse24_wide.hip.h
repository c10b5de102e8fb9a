// Wide-tile form of the fp16 x (int4, 2:4-sparse) grouped GEMM for gfx950: the
// variant for groups with many tokens (prefill / hot deltas), where the work is
// bound by the matrix cores rather than by HBM.
//
// Same packed layout, dequantisation and sparse-MFMA operand mapping as
// sparse24_grouped_kernel (sparse24_gemm.hip.h).  Differences:
//   * a workgroup owns a 64-token x 512-column tile: its 4 wavefronts take 4
//     adjacent 128-column blocks and each runs the whole K range (no K split, no
//     cross-wave reduction; every dequantised weight fragment feeds 4 MFMAs);
//   * the 64 x 128 activation tile of each K step is fetched from global memory
//     once per workgroup into LDS (double buffered) and read by all 4 wavefronts,
//     instead of once per wavefront: one barrier per K step;
//   * outputs go straight from the accumulators to memory (each lane holds 32
//     consecutive features of one token).
// LDS rows are padded to 272 B so that the 16 token rows read by one
// ds_read_b128 fall into distinct banks.
#pragma once
#include "sparse24_gemm.hip.h"

namespace triteia_hip {

constexpr int kWideTokens = 64;
constexpr int kWideRowHalfs = 136;   // 128 k + 8 halfs of padding

template <int DEPTH>
__global__ __launch_bounds__(256) void sparse24_wide_kernel(const Sparse24Args p) {
  constexpr int NT = kWideTokens / 16;
  __shared__ _Float16 xs[2][kWideTokens][kWideRowHalfs];
  __shared__ int s_rows[kWideTokens];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int r = lane & 15;
  const int q = lane >> 4;

  // unit = (group, group of 4 column blocks); column-block groups are padded to a multiple of
  // 8 per group and renumbered so that each XCD (own L2) owns a contiguous run of them for
  // every token tile of a delta
  const int col_blocks = p.m >> 7;
  const int cgs = (col_blocks + 3) >> 2;
  const int cg_pad = (cgs + 7) & ~7;
  const int unit = blockIdx.x;
  const int grp = unit / cg_pad;
  const int i = unit - grp * cg_pad;
  const int cg = p.xcd_swizzle ? (i & 7) * (cg_pad >> 3) + (i >> 3) : i;
  if (cg >= cgs) return;
  int delta, start, count;
  if (p.tiles) {
    const int4 d = p.tiles[grp];
    delta = d.x;
    start = d.y;
    count = d.z;
  } else {
    const int chunks = (p.uniform_count + kWideTokens - 1) / kWideTokens;
    const int gi = grp / chunks, tc = grp - gi * chunks;
    delta = gi * p.delta_step;
    start = gi * p.uniform_stride + p.uniform_first + tc * kWideTokens;
    count = min(kWideTokens, p.uniform_count - tc * kWideTokens);
  }
  const int n_groups = p.n_groups_dev ? *p.n_groups_dev : p.n_groups;
  if (grp >= n_groups) return;
  if (delta < 0 || delta >= p.n_deltas || count <= 0) return;
  const int cnt = min(count, kWideTokens);

  const int cb = 4 * cg + wave;
  const bool active = cb < col_blocks;          // the last group of a matrix may be partial
  const int cbc = active ? cb : col_blocks - 1;  // idle waves still run the barriers

  const int k_rows = p.k >> 5;
  const int n_steps = (k_rows + 3) >> 2;
  const long qrow = p.m >> 1;
  const long mrow = p.m >> 2;
  const uint4_t* qw_lane = p.qweight + (long)delta * p.qweight_stride + (long)cbc * 64 + 4 * r;
  const uint4_t* mt_lane = p.meta + (long)delta * p.meta_stride + (long)cbc * 32 + (r >> 3) * 16 + (r & 7);

  // token rows of the tile (slots past the end repeat the last row; their outputs are dropped)
  if (tid < kWideTokens) {
    const int slot = min(tid, cnt - 1);
    s_rows[tid] = p.perm ? p.perm[start + slot] : start + slot;
  }
  __syncthreads();

  // cooperative activation fetch: thread t moves 16-byte chunk (t % 16) of rows t/16 + 16 i
  const int xc = tid & 15;
  const _Float16* xsrc[4];
#pragma unroll
  for (int ii = 0; ii < 4; ii++) xsrc[ii] = p.x + (long)s_rows[(tid >> 4) + 16 * ii] * p.x_stride + xc * 8;
  uint4_t xg[4];
  auto load_xg = [&](int st) {
    // the last step may be half empty (k % 128 == 64): chunks past K are zeroed at the store
    const int koff = min(st * 128 + xc * 8, p.k - 8) - xc * 8;
#pragma unroll
    for (int ii = 0; ii < 4; ii++) xg[ii] = *reinterpret_cast<const uint4_t*>(xsrc[ii] + koff);
  };
  auto store_xg = [&](int stage, int st) {
    const bool in_k = st * 128 + xc * 8 < p.k;
#pragma unroll
    for (int ii = 0; ii < 4; ii++) {
      const uint4_t v = in_k ? xg[ii] : uint4_t{0u, 0u, 0u, 0u};
      *reinterpret_cast<uint4_t*>(&xs[stage][(tid >> 4) + 16 * ii][xc * 8]) = v;
    }
  };

  struct WFrag {
    uint4_t wq[4];
    uint4_t mt[2];
  };
  auto load_w = [&](WFrag& f, int st) {
    const int tr0 = (st < n_steps ? st : 0) << 2;
    const int tr = min(tr0 + q, k_rows - 1);   // rows past the end of K meet zero activations
    const uint4_t* wp = qw_lane + (long)tr * qrow;
    const uint4_t* mp = mt_lane + (long)tr * mrow;
#pragma unroll
    for (int a = 0; a < 4; a++) f.wq[a] = wp[a];
    f.mt[0] = mp[0];
    f.mt[1] = mp[8];
  };

  float4_t acc[8][NT];
#pragma unroll
  for (int cc = 0; cc < 8; cc++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[cc][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

  // B operand of lane (n = r, qb = q): k offsets 8*(q%2) + {0..7} of packed rows q/2 and 2 + q/2
  // of the step, i.e. halfs [32*(q/2) + 8*(q%2) + 16u, +8) and the same + 64
  const int xb_off = 32 * (q >> 1) + 8 * (q & 1);
  auto compute_step = [&](const WFrag& f, int stage) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
      half8_t A[8];
      int idx[8];
#pragma unroll
      for (int cc = 0; cc < 8; cc++) {
        const int w = cc & 3;
        const int b2 = cc >> 2;
        uint4_t av;
#pragma unroll
        for (int a = 0; a < 4; a++) {
          uint32_t word = f.wq[a][w];
          if (b2) word >>= 8;
          av[a] = u ? dequant_odd(word) : dequant_even(word);
        }
        A[cc] = __builtin_bit_cast(half8_t, av);
        idx[cc] = (int)f.mt[(cc >> 1) & 1][(cc & 1) * 2 + u];
      }
#pragma unroll
      for (int nt = 0; nt < NT; nt++) {
        const _Float16* row = &xs[stage][nt * 16 + r][xb_off + 16 * u];
        typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
        const uint4_t lo = *reinterpret_cast<const uint4_t*>(row);
        const uint4_t hi = *reinterpret_cast<const uint4_t*>(row + 64);
        const uint8_t_v bb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const half16_t b = __builtin_bit_cast(half16_t, bb);
#pragma unroll
        for (int cc = 0; cc < 8; cc++) {
          if (cc >> 2)
            acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A[cc], b, acc[cc][nt], idx[cc], 0, 1);
          else
            acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A[cc], b, acc[cc][nt], idx[cc], 0, 0);
        }
      }
    }
  };

  // pipeline: weights DEPTH steps ahead in registers, activations one step ahead through LDS
  WFrag ring[DEPTH];
#pragma unroll
  for (int j = 0; j < DEPTH; j++) load_w(ring[j], j);
  load_xg(0);
  store_xg(0, 0);
  lds_barrier();
  constexpr int TURN = DEPTH % 2 == 0 ? DEPTH : 2 * DEPTH;   // whole ring turns and LDS stage pairs
  for (int s0 = 0; s0 < n_steps; s0 += TURN) {
#pragma unroll
    for (int j = 0; j < TURN; j++) {
      const int st = s0 + j;
      // the same loads and stores every iteration (the step after the last one re-reads the
      // last tile into the stage nobody reads), so that load-counter waits stay exact
      const int nxt = min(st + 1, n_steps - 1);
      load_xg(nxt);
      if (st < n_steps && active) compute_step(ring[j % DEPTH], j & 1);
      load_w(ring[j % DEPTH], st + DEPTH);
      store_xg((j + 1) & 1, nxt);
      lds_barrier();
    }
  }

  if (!active) return;
  // epilogue: lane (n = r, qq = q) holds features 32q + 8j + c of token n for every 16-token tile
  const _Float16* sc = p.scales + (long)delta * p.scales_stride + cb * 128 + 32 * q;
  half8_t sv[4];
#pragma unroll
  for (int j = 0; j < 4; j++) sv[j] = *reinterpret_cast<const half8_t*>(sc + 8 * j);
#pragma unroll
  for (int nt = 0; nt < NT; nt++) {
    const int slot = nt * 16 + r;
    if (slot >= cnt) continue;
    _Float16* op = p.out + (long)s_rows[slot] * p.out_stride + cb * 128 + 32 * q;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      half8_t o;
      if (p.accumulate) {
        const half8_t old = *reinterpret_cast<const half8_t*>(op + 8 * j);
#pragma unroll
        for (int cc = 0; cc < 8; cc++) o[cc] = (_Float16)((float)old[cc] + acc[cc][nt][j] * (float)sv[j][cc]);
      } else {
#pragma unroll
        for (int cc = 0; cc < 8; cc++) o[cc] = (_Float16)(acc[cc][nt][j] * (float)sv[j][cc]);
      }
      *reinterpret_cast<half8_t*>(op + 8 * j) = o;
    }
  }
}

}  // namespace triteia_hip
