// Wide-tile form of the fp16 x (int4, 2:4-sparse) grouped GEMM for gfx950: the
// variant for groups with many tokens (prefill / hot deltas), where the work is
// bound by the matrix cores rather than by HBM.
//
// Same packed layout, dequantisation and sparse-MFMA operand mapping as
// sparse24_grouped_kernel (sparse24_gemm.hip.h).  Differences:
//   * a workgroup owns a 64-token x 512-column tile: its 4 wavefronts take 4
//     adjacent 128-column blocks and each runs the whole K range (no K split, no
//     cross-wave reduction; every dequantised weight fragment feeds 4 MFMAs);
//   * the 64 x 128 activation tile of each K step is fetched once per workgroup,
//     straight from global memory into LDS (global_load_lds_dwordx4, no registers in
//     between), three steps ahead of its use in a 4-stage ring, and read by all 4
//     wavefronts: one barrier per K step;
//   * outputs go straight from the accumulators to memory (each lane holds 32
//     consecutive features of one token).
// An LDS row is the 256 B of one token; the 16-byte chunk c of row n is stored at chunk
// position c ^ (n % 16), so that the 16 token rows read by one ds_read_b128 fall into
// distinct banks while every direct-to-LDS load still writes 1 KB of consecutive LDS.
// Needs k % 128 == 0 (a direct load cannot zero-fill a partial K step).
#pragma once
#include "sparse24_gemm.hip.h"

namespace triteia_hip {

constexpr int kWideTokens = 64;
constexpr int kWideStages = 4;        // activation tiles in flight (LDS ring)

template <int DEPTH>
__global__ __launch_bounds__(256, 2) void sparse24_wide_kernel(const Sparse24Args p) {
  constexpr int NT = kWideTokens / 16;
  __shared__ __attribute__((aligned(1024))) _Float16 xs[kWideStages][kWideTokens][128];
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
  if (p.wide_min_units && (long)n_groups * p.wide_gate < p.wide_min_units) return;   // the narrow kernel has taken these tokens
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

  // cooperative activation fetch.  One direct-to-LDS instruction of a wavefront writes 64
  // consecutive 16-byte chunks = 4 token rows; instruction ii of wave w covers rows
  // 16 ii + 4 w + lane/16.  Lane l fills chunk position l % 16 of its row, which holds the
  // row's chunk (l % 16) ^ (row % 16).
  const _Float16* xsrc[4];
#pragma unroll
  for (int ii = 0; ii < 4; ii++) {
    const int row = 16 * ii + 4 * wave + (lane >> 4);
    const int chunk = (lane & 15) ^ (row & 15);
    xsrc[ii] = p.x + (long)s_rows[row] * p.x_stride + chunk * 8;
  }
  auto issue_x = [&](int st) {
    const int stc = min(st, n_steps - 1);   // past the end: refetch the last tile (never read)
    const int stage = st & (kWideStages - 1);
#pragma unroll
    for (int ii = 0; ii < 4; ii++)
      __builtin_amdgcn_global_load_lds(xsrc[ii] + stc * 128, &xs[stage][16 * ii + 4 * wave][0], 16, 0, 0);
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
  // reads the B fragment (16 halfs) of 16-token tile nt, k-half u from the LDS stage
  auto read_b = [&](int stage, int nt, int u) {
    // chunks c and c + 8 of token row nt*16 + r, at their swizzled positions
    const int c = (xb_off >> 3) + 2 * u;
    const _Float16* row = &xs[stage][nt * 16 + r][0];
    typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
    const uint4_t lo = *reinterpret_cast<const uint4_t*>(row + ((c ^ r) << 3));
    const uint4_t hi = *reinterpret_cast<const uint4_t*>(row + (((c + 8) ^ r) << 3));
    const uint8_t_v bb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(half16_t, bb);
  };
  auto compute_step = [&](const WFrag& f, int stage) {
    // Per k-half u and per half of the 8 columns: dequantise 4 weight fragments, then run them
    // against the four 16-token B fragments.  B fragments are read one ahead of the MFMAs that
    // use them, so that the LDS latency hides behind 4 MFMAs instead of stalling in front of them.
    half16_t b_nxt = read_b(stage, 0, 0);
#pragma unroll
    for (int u = 0; u < 2; u++) {
#pragma unroll
      for (int b2 = 0; b2 < 2; b2++) {
        half8_t A[4];
#pragma unroll
        for (int w = 0; w < 4; w++) {
          uint4_t av;
#pragma unroll
          for (int a = 0; a < 4; a++) {
            uint32_t word = f.wq[a][w];
            if (b2) word >>= 8;
            av[a] = u ? dequant_odd(word) : dequant_even(word);
          }
          A[w] = __builtin_bit_cast(half8_t, av);
        }
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
          const half16_t b = b_nxt;
          if (nt + 1 < NT) b_nxt = read_b(stage, nt + 1, u);
          else if (b2 == 0) b_nxt = read_b(stage, 0, u);
          else if (u == 0) b_nxt = read_b(stage, 0, 1);
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const int cc = 4 * b2 + w;
            const int idx = (int)f.mt[(cc >> 1) & 1][(cc & 1) * 2 + u];
            if (b2)
              acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A[w], b, acc[cc][nt], idx, 0, 1);
            else
              acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A[w], b, acc[cc][nt], idx, 0, 0);
          }
        }
      }
    }
  };

  // pipeline: weights DEPTH steps ahead in registers; activation tiles 3 steps ahead in the
  // LDS ring.  At the top of step st this wave waits until its own direct loads of tile st
  // have landed (everything it issued since then is allowed to stay in flight: 4 loads for each
  // of tiles st+1 and st+2 at least), then the barrier makes all four waves' parts visible
  // and also says that tile st-1 has been read by everyone, so its stage can be refilled.
  WFrag ring[DEPTH];
#pragma unroll
  for (int j = 0; j < DEPTH; j++) load_w(ring[j], j);
  issue_x(0);
  issue_x(1);
  issue_x(2);
  constexpr int TURN = DEPTH > 4 ? DEPTH : 4;   // whole ring turns of both rings (DEPTH divides 4)
  for (int s0 = 0; s0 < n_steps; s0 += TURN) {
#pragma unroll
    for (int j = 0; j < TURN; j++) {
      const int st = s0 + j;
      __builtin_amdgcn_s_waitcnt(0x0F70 | 8);   // vmcnt(8), nothing else
      lds_barrier();
      issue_x(st + 3);
      if (st < n_steps && active) compute_step(ring[j % DEPTH], j & (kWideStages - 1));
      load_w(ring[j % DEPTH], st + DEPTH);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): no direct load may outlive the block's LDS

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
      half8_t old = {0, 0, 0, 0, 0, 0, 0, 0};
      if (p.accumulate) old = *reinterpret_cast<const half8_t*>(op + 8 * j);
      half8_t o;
#pragma unroll
      for (int cc = 0; cc < 8; cc++) o[cc] = scaled_sum_f16(old[cc], acc[cc][nt][j], sv[j][cc]);
      *reinterpret_cast<half8_t*>(op + 8 * j) = o;
    }
  }
}

}  // namespace triteia_hip
