// 128-token form of the wide fp16 x (int4, 2:4-sparse) GEMM tile for gfx950: the variant for
// groups with hundreds of tokens (prefill), where the matrix cores are the bound.
//
// Same packed layout, dequantisation and sparse-MFMA operand mapping as sparse24_wide_kernel
// (sparse24_wide.hip.h), with twice the tokens per dequantised weight fragment:
//   * a workgroup owns a 128-token x 512-column tile; each of its 4 wavefronts keeps the
//     128 x 128 fp32 accumulators of one column block (256 registers per lane, so one workgroup
//     per CU and one wavefront per SIMD);
//   * every dequantised weight fragment feeds 8 MFMAs and every activation fragment read from
//     LDS feeds 8 MFMAs (all 8 columns of the lane's block);
//   * with a single wavefront per SIMD nothing else fills a stall, so the kernel is software
//     pipelined by hand: everything it reads from global memory goes straight into LDS
//     (global_load_lds_dwordx4) two steps ahead of its use, and the fragments for the next half
//     step are dequantised while the MFMAs of the current half step run.
// LDS (dynamic, 144.5 KB): a 3-stage ring of 128 x 128 activation tiles (32 KB each, shared by
// the 4 waves, swizzled as in the 64-token kernel), and per wave a 2-stage ring of its own
// packed weights and metadata of one K step (6 KB each: no register is the target of a load
// that is still in flight, so nothing depends on how the compiler moves registers around).
// Needs k % 128 == 0.
#pragma once
#include "sparse24_gemm.hip.h"

namespace triteia_hip {

constexpr int kWide128Tokens = 128;
constexpr int kWide128Lookahead = 2;
constexpr int kWide128Stages = 3;                                   // activation tiles
constexpr int kWide128XBytes = kWide128Stages * kWide128Tokens * 256;
constexpr int kWide128WStageBytes = 6 * 1024;                       // per wave: 4 weight + 2 metadata vectors per lane
constexpr int kWide128WBytes = 4 * 2 * kWide128WStageBytes;
constexpr int kWide128LdsBytes = kWide128XBytes + kWide128WBytes + kWide128Tokens * 4;

__global__ __launch_bounds__(256, 1) void sparse24_wide128_kernel(const Sparse24Args p) {
  constexpr int NT = kWide128Tokens / 16;
  extern __shared__ __attribute__((aligned(1024))) unsigned char wide128_lds[];
  typedef _Float16 XsTile[kWide128Tokens][128];
  XsTile* xs = reinterpret_cast<XsTile*>(wide128_lds);
  unsigned char* ws_lds = wide128_lds + kWide128XBytes;
  int* s_rows = reinterpret_cast<int*>(wide128_lds + kWide128XBytes + kWide128WBytes);

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int r = lane & 15;
  const int q = lane >> 4;

  // unit = (group, group of 4 column blocks), numbered as in sparse24_wide_kernel
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
    const int chunks = (p.uniform_count + kWide128Tokens - 1) / kWide128Tokens;
    const int gi = grp / chunks, tc = grp - gi * chunks;
    delta = gi * p.delta_step;
    start = gi * p.uniform_stride + p.uniform_first + tc * kWide128Tokens;
    count = min(kWide128Tokens, p.uniform_count - tc * kWide128Tokens);
  }
  const int n_groups = p.n_groups_dev ? *p.n_groups_dev : p.n_groups;
  if (p.wide_min_units && (long)n_groups * p.wide_gate < p.wide_min_units) return;   // the narrow kernel has taken these tokens
  if (grp >= n_groups) return;
  if (delta < 0 || delta >= p.n_deltas || count <= 0) return;
  const int cnt = min(count, kWide128Tokens);

  const int cb = 4 * cg + wave;
  const bool active = cb < col_blocks;
  const int cbc = active ? cb : col_blocks - 1;

  const int k_rows = p.k >> 5;
  const int n_steps = k_rows >> 2;
  const long qrow = p.m >> 1;
  const long mrow = p.m >> 2;

  if (tid < kWide128Tokens) {
    const int slot = min(tid, cnt - 1);
    s_rows[tid] = p.perm ? p.perm[start + slot] : start + slot;
  }
  __syncthreads();

  // One direct-to-LDS instruction of a wavefront writes 64 consecutive 16-byte chunks = 4 token
  // rows; instruction ii of wave w covers rows 16 ii + 4 w + lane/16.  Lane l fills chunk
  // position l % 16 of its row, which holds the row's chunk (l % 16) ^ (row % 16).  Addresses
  // are a scalar base (which advances with the K step) plus a 32-bit byte offset per lane
  // (the launcher only picks this kernel for activations below 4 GiB).
  uint32_t xoff[NT];
#pragma unroll
  for (int ii = 0; ii < NT; ii++) {
    const int row = 16 * ii + 4 * wave + (lane >> 4);
    const int chunk = (lane & 15) ^ (row & 15);
    xoff[ii] = (uint32_t)(((long)s_rows[row] * p.x_stride + chunk * 8) * 2);
  }
  // All global memory requests of the main loop are direct-to-LDS loads written as inline
  // assembly, and so are the waits for them.  (The compiler's own wait insertion would drain
  // every outstanding request at each barrier: it counts direct-to-LDS loads as LDS writes
  // that a release fence must complete, which would cut the prefetch distance to a fraction
  // of a step.)  The LDS address of a request is M0 + 16 * lane.
  const uint32_t lds_x_wave = (uint32_t)(uintptr_t)&xs[0][4 * wave][0];
  auto issue_x = [&](int st, int stage) {
    const int stc = min(st, n_steps - 1);   // past the end: refetch the last tile (never read)
    const _Float16* base = p.x + stc * 128;
#pragma unroll
    for (int ii = 0; ii < NT; ii++) {
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_x_wave + (stage * kWide128Tokens + 16 * ii) * 256);
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(xoff[ii]), "s"(base), "s"(dst) : "memory");
    }
  };
  // weights and metadata of step st -> this wave's weight stage `stage`: vector a of lane l at
  // byte 1024 a + 16 l.  Scalar base = packed row 4 st of the delta, lane offsets fixed.
  unsigned char* ws_wave = ws_lds + wave * 2 * kWide128WStageBytes;
  const uint32_t lds_w_wave = (uint32_t)(uintptr_t)ws_wave;
  const uint4_t* qw_delta = p.qweight + (long)delta * p.qweight_stride;
  const uint4_t* mt_delta = p.meta + (long)delta * p.meta_stride;
  uint32_t woff[4], moff[2];
#pragma unroll
  for (int a = 0; a < 4; a++) woff[a] = (uint32_t)((q * qrow + (long)cbc * 64 + 4 * r + a) * 16);
  moff[0] = (uint32_t)((q * mrow + (long)cbc * 32 + (r >> 3) * 16 + (r & 7)) * 16);
  moff[1] = moff[0] + 128;
  auto issue_w = [&](int st, int stage) {
    const long tr0 = (st < n_steps ? st : 0) << 2;   // past the end: any valid rows (never used)
    const uint4_t* wb = qw_delta + tr0 * qrow;
    const uint4_t* mb = mt_delta + tr0 * mrow;
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_w_wave + stage * kWide128WStageBytes);
#pragma unroll
    for (int a = 0; a < 4; a++)
      asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(woff[a]), "s"(wb), "s"(dst + 1024 * a) : "memory");
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(moff[0]), "s"(mb), "s"(dst + 4096) : "memory");
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(moff[1]), "s"(mb), "s"(dst + 5120) : "memory");
  };

  struct WFrag {
    uint4_t wq[4];
    uint4_t mt[2];
  };
  // LDS weight stage -> registers (ordinary LDS reads, which the compiler tracks itself)
  auto read_w = [&](WFrag& f, int stage) {
    const uint4_t* src = reinterpret_cast<const uint4_t*>(ws_wave + stage * kWide128WStageBytes) + lane;
#pragma unroll
    for (int a = 0; a < 4; a++) f.wq[a] = src[64 * a];
    f.mt[0] = src[256];
    f.mt[1] = src[320];
  };

  float4_t acc[8][NT];
#pragma unroll
  for (int cc = 0; cc < 8; cc++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[cc][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

  const int xb_off = 32 * (q >> 1) + 8 * (q & 1);
  auto read_b = [&](int stage, int nt, int u) {
    const int c = (xb_off >> 3) + 2 * u;
    const _Float16* row = &xs[stage][nt * 16 + r][0];
    typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
    const uint4_t lo = *reinterpret_cast<const uint4_t*>(row + ((c ^ r) << 3));
    const uint4_t hi = *reinterpret_cast<const uint4_t*>(row + (((c + 8) ^ r) << 3));
    const uint8_t_v bb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(half16_t, bb);
  };
  // the 8 A fragments (one per column of the lane's block) of k-half u
  auto dequant = [&](half8_t (&A)[8], const WFrag& f, int u) {
#pragma unroll
    for (int cc = 0; cc < 8; cc++) {
      uint4_t av;
#pragma unroll
      for (int a = 0; a < 4; a++) {
        uint32_t word = f.wq[a][cc & 3];
        if (cc >> 2) word >>= 8;
        av[a] = u ? dequant_odd(word) : dequant_even(word);
      }
      A[cc] = __builtin_bit_cast(half8_t, av);
    }
  };
  // Requests, in this order: W0 X0 W1 X1 W2, then per step s: X(s+2) at its top, W(s+3) at
  // its end (X = the 8 requests of an activation tile, W = the 6 of a weight stage).
  // Requests complete in order.  At the top of step s tile s must be there: the 20 requests
  // after it (W(s+1) X(s+1) W(s+2)) may stay in flight.  In the middle of step s weights s+1
  // must be there: the 22 requests after them (X(s+1) W(s+2) X(s+2)) may stay in flight.
  // The barrier at the top of step s also says that every wave has finished step s-1, whose
  // activation stage then takes tile s+2.  A weight stage is refilled (with step s+3) at the
  // end of the step that read its content (step s+1) into registers.
  WFrag wr[2];
  half8_t A0[8], A1[8];
  issue_w(0, 0);
  issue_x(0, 0);
  issue_w(1, 1);
  issue_x(1, 1);
  asm volatile("s_waitcnt vmcnt(22)" ::: "memory");
  read_w(wr[0], 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  issue_w(2, 0);
  dequant(A0, wr[0], 0);   // idle waves (partial last group of columns) only run the requests and barriers
  constexpr int LA = kWide128Lookahead;   // B fragments requested ahead of the MFMAs that use them
  for (int s0 = 0; s0 < n_steps; s0 += 6) {
#pragma unroll
    for (int j = 0; j < 6; j++) {
      const int st = s0 + j;
      asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
      lds_barrier();
      issue_x(st + 2, (j + 2) % 3);
      if (st < n_steps && active) {
        // the step's 16 B fragments (k-half u = f / 8, token tile f % 8) form one stream; fragment f
        // feeds the 8 MFMAs of the lane's 8 columns
        const WFrag& wc = wr[j & 1];
        WFrag& wn = wr[(j + 1) & 1];
        half16_t bq[LA + 1];
#pragma unroll
        for (int f = 0; f < LA; f++) bq[f] = read_b(j % 3, f & 7, f >> 3);
        dequant(A1, wc, 1);
#pragma unroll
        for (int f = 0; f < 16; f++) {
          if (f == 8) {
            // A0 has served its last MFMA of this step: prepare it for the next one
            asm volatile("s_waitcnt vmcnt(22)" ::: "memory");
            read_w(wn, (j + 1) & 1);
            dequant(A0, wn, 0);
          }
          if (f + LA < 16) bq[(f + LA) % (LA + 1)] = read_b(j % 3, (f + LA) & 7, (f + LA) >> 3);
          const half16_t b = bq[f % (LA + 1)];
          const int u = f >> 3, nt = f & 7;
#pragma unroll
          for (int cc = 0; cc < 8; cc++) {
            const int idx = (int)wc.mt[(cc >> 1) & 1][(cc & 1) * 2 + u];
            const half8_t a = u ? A1[cc] : A0[cc];
            if (cc >> 2)
              acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a, b, acc[cc][nt], idx, 0, 1);
            else
              acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a, b, acc[cc][nt], idx, 0, 0);
          }
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave has read the stage that is refilled now
      issue_w(st + 3, (j + 1) & 1);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive the block's LDS

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
