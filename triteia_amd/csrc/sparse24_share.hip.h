// Decode-size form of the fp16 x (int4, 2:4-sparse) product for gfx950: at most 16 tokens per matrix and so few
// 128-column blocks in the whole launch that one workgroup per block would leave most CUs idle (a single
// 4096 x 4096 matrix has 32).  Such a launch is bound by the chain of dependent steps of each workgroup, not by
// bytes: here a workgroup takes a share of 16 T output columns (T = 1, 2, 4: the narrowest that leaves at most a workgroup
// per CU), and
//   * the 16 rows of a sparse MFMA are 16 adjacent columns of the share (in sparse24_grouped_kernel they are the sixteen
//     8-column blocks of a 128-column block, one MFMA per column of a block): 2 T MFMAs and 8 T conversions per step
//     instead of 16 and 64, and a lane holds one 32-bit word of each of its four weight vectors and two metadata
//     words per 16 columns and step instead of six 16-byte vectors;
//   * with so few registers per step, every wavefront requests all of its steps of a chunk of K at once (DEPTH steps,
//     k = 4096 on eight wavefronts: the whole of K): one round trip to memory instead of one per step.
// Packed layout, dequantisation, B operand and the order of every fp32 sum are those of sparse24_grouped_kernel with
// the same number of wavefronts (wavefront w takes steps w, w + KW, ... in order; the wavefronts' sums are added in
// the order of w), so a launch gives the same bits through either kernel.
#pragma once
#include "sparse24_gemm.hip.h"

namespace triteia_hip {

// T: 16-column tiles of a share (1, 2 or 4).  ROUTED: the groups are the deltas that a batch of at most 16 tokens uses,
// worked out by every wavefront from the batch's indices (Sparse24Args::raw_indices), as sparse24_grouped_kernel does
// for batches of up to 256; with KW = 4, the number of wavefronts that kernel keeps for routed tokens, so that a token's
// bits do not depend on which of the two kernels its batch went to.
template <int KW, int DEPTH, int T, bool ROUTED = false>
__global__ __launch_bounds__(64 * KW, 2) void sparse24_share16_kernel(const Sparse24Args p) {
  constexpr int kShareCols = 16 * T;
  __shared__ float red[KW][16][kShareCols + 4];   // [wavefront][token][column of the share] (+ pad)

  // unit = (group, share); the shares of a group are numbered so that each XCD owns a contiguous run of them
  const int shares = p.m / kShareCols;            // (m is a multiple of 128)
  const int sh_pad = (shares + 7) & ~7;
  const int unit = blockIdx.x;
  const int grp = unit / sh_pad;
  const int i = unit - grp * sh_pad;
  const int sh = p.xcd_swizzle ? (i & 7) * (sh_pad >> 3) + (i >> 3) : i;
  if (sh >= shares || grp >= p.n_groups) return;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int rho = lane & 15;     // A: column rho of the share; B and D: token rho
  const int q = lane >> 4;       // A, B: packed row tr0 + q resp. k slots; D: columns 4q .. 4q + 3
  int delta, start, cnt;
  int list = 0;                  // ROUTED: lane s holds the batch position of the group's s-th token
  if (ROUTED) {
    // lane l < raw_count looks at token l; group g is the g-th delta in use, in ascending order
    int d = p.raw_indices[min(lane, p.raw_count - 1)] - p.raw_offset;
    if (lane >= p.raw_count || lane >= 16 || d < 0 || d >= p.n_deltas || d >= 64) d = -1;
    unsigned long long used = d >= 0 ? (1ull << d) : 0ull;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const unsigned lo = __shfl_xor((unsigned)used, off, 64);
      const unsigned hi = __shfl_xor((unsigned)(used >> 32), off, 64);
      used |= ((unsigned long long)hi << 32) | lo;
    }
    if (grp >= __popcll(used)) return;
    for (int g = 0; g < grp; g++) used &= used - 1;
    delta = __ffsll((long long)used) - 1;
    const unsigned long long members = __ballot(d == delta);
    cnt = __popcll(members);
    const int rank = __popcll(members & ((1ull << lane) - 1ull));
    const int dest = (d == delta) ? rank : cnt + (lane - rank);   // a permutation: members first, in batch order
    list = __builtin_amdgcn_ds_permute(dest << 2, lane);
    start = 0;
  } else {
    // uniform groups: group g = delta g * delta_step with uniform_count (<= 16) rows
    delta = grp * p.delta_step;
    start = grp * p.uniform_stride + p.uniform_first;
    cnt = min(p.uniform_count, 16);
  }
  if (delta < 0 || delta >= p.n_deltas || cnt <= 0) return;

  const int k_rows = p.k >> 5;
  const int n_steps = (k_rows + 3) >> 2;
  const int rot = (int)(((unsigned)delta * (unsigned)p.rot_spread) % (unsigned)n_steps);

  // this lane's column of tile 0: 8-column block `ra` of column block `cb`, column `c` inside it (tile t: block ra + 2 t)
  const int cb = sh / (8 / T);
  const int ra = 2 * T * (sh % (8 / T)) + (rho >> 3);
  const int c = rho & 7;
  const long qrow_w = (long)(p.m >> 1) * 4;   // 32-bit words per packed row (weights, metadata)
  const long mrow_w = (long)(p.m >> 2) * 4;
  // weights: word c % 4 of the vectors 4 ra + a (a = 0..3), byte c / 4 of each 16-bit half of the word
  // (tile t: 8 vectors = 32 words further)
  const uint32_t* qw = reinterpret_cast<const uint32_t*>(p.qweight + (long)delta * p.qweight_stride + (long)cb * 64 + 4 * ra) + (c & 3);
  // metadata: words 2 (c % 2) + u (u = 0, 1) of vector (c / 2) % 2 of the block's pair, 16-bit half c / 4
  // (block ra + 2 t lies in the same half of the column block as ra -- shares do not straddle 64 columns --: 2 t vectors further)
  const uint32_t* mt = reinterpret_cast<const uint32_t*>(p.meta + (long)delta * p.meta_stride + (long)(cb * 2 + (ra >> 3)) * 16 +
                                                         (ra & 7) + 8 * ((c >> 1) & 1)) + 2 * (c & 1);
  const int w_shift = (c >> 2) * 8;
  const int m_shift = (c >> 2) * 16;
  // B operand: token slot rho (slots past the end repeat the last row; their results are dropped)
  const long row = ROUTED ? __shfl(list, min(rho, cnt - 1), 64) : start + min(rho, cnt - 1);
  const _Float16* xrow = p.x + row * p.x_stride + 32 * (q >> 1) + 8 * (q & 1);

  struct Frag {
    uint32_t w[T][4];
    uint32_t m[T][2];
    uint4_t xa[2], xb[2];
  };
  auto phys = [&](int st) {
    const int ps = st + rot;
    return st < n_steps ? (ps < n_steps ? ps : ps - n_steps) : 0;   // steps past the end read step 0 (never multiplied)
  };
  auto load = [&](Frag& f, int st) {
    const int tr0 = phys(st) << 2;
    const int tr = min(tr0 + q, k_rows - 1);   // rows past the end of K are cancelled by a zero B
    const uint32_t* wp = qw + (long)tr * qrow_w;
    const uint32_t* mp = mt + (long)tr * mrow_w;
#pragma unroll
    for (int t = 0; t < T; t++) {
#pragma unroll
      for (int a = 0; a < 4; a++) f.w[t][a] = wp[32 * t + 4 * a];
      const uint2 mm = *reinterpret_cast<const uint2*>(mp + 8 * t);
      f.m[t][0] = mm.x;
      f.m[t][1] = mm.y;
    }
    const long xoff_a = (long)min(tr0, k_rows - 1 - (q >> 1)) * 32;
    const long xoff_b = (long)min(tr0 + 2, k_rows - 1 - (q >> 1)) * 32;
    f.xa[0] = *reinterpret_cast<const uint4_t*>(xrow + xoff_a);
    f.xa[1] = *reinterpret_cast<const uint4_t*>(xrow + xoff_a + 16);
    f.xb[0] = *reinterpret_cast<const uint4_t*>(xrow + xoff_b);
    f.xb[1] = *reinterpret_cast<const uint4_t*>(xrow + xoff_b + 16);
  };
  float4_t acc[T];
#pragma unroll
  for (int t = 0; t < T; t++) acc[t] = float4_t{0.f, 0.f, 0.f, 0.f};
  auto compute = [&](const Frag& f, int st) {
    const int tr0 = phys(st) << 2;
    const bool tail = tr0 + 4 > k_rows;
    const bool ok_a = (tr0 + (q >> 1)) < k_rows;
    const bool ok_b = (tr0 + 2 + (q >> 1)) < k_rows;
#pragma unroll
    for (int u = 0; u < 2; u++) {
      typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
      uint8_t_v bb = {f.xa[u][0], f.xa[u][1], f.xa[u][2], f.xa[u][3], f.xb[u][0], f.xb[u][1], f.xb[u][2], f.xb[u][3]};
      if (tail) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
          if (!ok_a) bb[e] = 0u;
          if (!ok_b) bb[4 + e] = 0u;
        }
      }
#pragma unroll
      for (int t = 0; t < T; t++) {
        uint4_t av;
#pragma unroll
        for (int a = 0; a < 4; a++) {
          const uint32_t word = f.w[t][a] >> w_shift;
          av[a] = u ? dequant_odd(word) : dequant_even(word);
        }
        const int idx = (int)(f.m[t][u] >> m_shift);
        acc[t] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(__builtin_bit_cast(half8_t, av), __builtin_bit_cast(half16_t, bb), acc[t], idx, 0, 0);
      }
    }
  };

  // wavefront w takes steps w, w + KW, ...; a chunk = DEPTH of them, all requested before the first is used
  for (int base = wave; base < n_steps; base += DEPTH * KW) {
    Frag f[DEPTH];
#pragma unroll
    for (int j = 0; j < DEPTH; j++) load(f[j], base + j * KW);
#pragma unroll
    for (int j = 0; j < DEPTH; j++)
      if (base + j * KW < n_steps) compute(f[j], base + j * KW);
  }

  // D: lane (token rho, q) holds columns 16 t + 4q + j of the share
#pragma unroll
  for (int t = 0; t < T; t++) *reinterpret_cast<float4_t*>(&red[wave][rho][16 * t + 4 * q]) = acc[t];
  __syncthreads();
  // (the row of a routed token is fetched from the lane that holds it while every lane is active)
  const long orow_routed = ROUTED ? __shfl(list, (tid / (2 * T)) & 15, 64) : 0;
  if (tid < 32 * T) {
    const int tok = tid / (2 * T), f0 = (tid % (2 * T)) * 8;
    if (tok < cnt) {
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; e++) v[e] = 0.f;
#pragma unroll
      for (int w = 0; w < KW; w++) {
        const float4_t a0 = *reinterpret_cast<const float4_t*>(&red[w][tok][f0]);
        const float4_t a1 = *reinterpret_cast<const float4_t*>(&red[w][tok][f0 + 4]);
#pragma unroll
        for (int e = 0; e < 4; e++) { v[e] += a0[e]; v[4 + e] += a1[e]; }
      }
      const half8_t sv = *reinterpret_cast<const half8_t*>(p.scales + (long)delta * p.scales_stride + sh * kShareCols + f0);
      const long orow = ROUTED ? orow_routed : start + tok;
      _Float16* op = p.out + orow * p.out_stride + sh * kShareCols + f0;
      half8_t old = {0, 0, 0, 0, 0, 0, 0, 0};
      if (p.accumulate) old = *reinterpret_cast<const half8_t*>(op);
      half8_t o;
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = scaled_sum_f16(old[e], v[e], sv[e]);
      *reinterpret_cast<half8_t*>(op) = o;
    }
  }
}

}  // namespace triteia_hip
