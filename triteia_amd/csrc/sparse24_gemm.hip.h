// fp16 x (int4, 2:4-sparse) grouped GEMM for gfx950 (MI355X).
//
// One kernel serves matmul_4bit_2_4, bmm_4bit_2_4 and the routed
// sbmm_4bit_2_4 / ldmm delta path: the work is a list of *groups*, each group
// being (delta matrix, list of token rows).  A workgroup owns one
// (group, 128-output-column block) and streams that slice of the packed
// weights from HBM exactly once per 16*NT tokens.
//
// Packed layout consumed directly (no repacking), as produced by the
// reference's packer (triteia/python/nn/linear.py:79-141,
// triteia/python/ops/utils/sparsity.py:35-61,134-161):
//   qweight [k/32][2m] int32 : per 32-dense-k row `tr`, 64 output columns are
//       128 consecutive int32 = 32 x 16-byte vectors.  Vector i holds output
//       columns 8*(i/4)..+7 and compressed-k entries {2a,2a+1,2a+8,2a+9},
//       a = i%4, i.e. 2:4 groups a and a+4 of the 8 groups in the row.
//   meta [k/32][m][2] int16 (physical order): per `tr`, 64 columns are 128
//       int16 whose index has bits [b1 b5 b4 b3 b0 h b2] (b = column bits,
//       h = which 16-k half); each int16 = four 4-bit (lo | hi<<2) codes.
//   scales [m] fp16 per output column.
//
// Mapping onto V_SMFMAC_F32_16X16X64_F16 (sparse A = weights, dense B =
// activations, D = out^T tile):
//   lane l = (r = l%16, q = l/16).  Row r of the MFMA is the 8-column block r
//   of the 128-column block; quarter q covers packed row tr0+q.  For output
//   column c (0..7) inside the block and k-half u (0/1) one MFMA consumes, per
//   lane, the 4 groups {4u..4u+3} of that column: one half2 from each of the
//   lane's four 16-byte weight vectors, and exactly one 16-bit metadata word
//   as the index operand (ABID selects the half of the 32-bit word).  The
//   dequantised half2 comes from the (nibble | 0x6400) - 1032 trick, so the
//   weights go HBM -> VGPR -> MFMA with ~2 VALU ops per pair.
//   B operand of lane (n = l%16, qb = l/16): 8 halfs from
//   x[token n][32*(tr0 + qb/2) + 16u + 8*(qb%2) ..] and 8 from the same
//   offset two packed rows further (the instruction's K order for B is
//   {8qb..8qb+7, 32+8qb..}).
//   D: lane (n, qq) holds rows 4qq+j => output features 32qq + 8j + c: 32
//   consecutive features of token n.
//
// The KW wavefronts of a workgroup split K between them and reduce through
// LDS in a fixed order (deterministic, no atomics, no global scratch).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace triteia_hip {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

struct Sparse24Args {
  const _Float16* x;        // [T, k] activations
  long x_stride;            // elements between token rows
  const uint4_t* qweight;   // [N][k/32][m/2] 16-byte vectors
  long qweight_stride;      // vectors between deltas
  const uint4_t* meta;      // [N][k/32][m/4] 16-byte vectors (physical order)
  long meta_stride;         // vectors between deltas
  const _Float16* scales;   // [N][m]; with scale_groups > 0 (GS builds): [N][scale_groups][m], one row per 128 dense k,
                            // each run of 8 columns stored in the order 0 4 1 5 2 6 3 7 (the reference's grouped layout)
  long scales_stride;       // elements between deltas
  _Float16* out;            // [T, m]
  long out_stride;          // elements between rows
  int m;                    // output features
  int k;                    // input features
  // groups, one of three forms:
  //   tiles   : packed {delta, start, count, 0} per group (the routing plan's tile list)
  //   g_*     : three separate arrays (the reference's run table)
  //   none    : group j = delta j*delta_step with uniform_count rows from
  //             j*uniform_stride + uniform_first
  //   raw_indices : (takes precedence) the batch's per-token delta indices, at most 256 tokens
  //             and 64 deltas: every workgroup derives its group itself ("fused routing"),
  //             group j = the j-th delta in use, in ascending order
  const int4* tiles;
  const int* raw_indices;
  int raw_count;
  int raw_offset;
  const int* g_delta;
  const int* g_start;
  const int* g_count;
  const int* perm;          // row of the i-th listed token (nullptr: identity)
  const int* n_groups_dev;  // device-side group count (nullptr: n_groups)
  // A routing plan with wide tiles lists its tokens twice: as {wide tiles + narrow rest} and as
  // narrow tiles only.  Which of the two runs is decided on the device, where the number of wide
  // tiles is known: the wide kernel only pays when its launch fills the chip, i.e. when
  // wide tiles x wide_gate (column groups per tile) >= wide_min_units.  For the narrow kernel
  // tiles_alt is the narrow-only list and n_groups_dev points at the plan header ([0] narrow rest
  // tiles, [4] wide tiles, [5] tiles of the narrow-only list); for the wide kernels n_groups_dev
  // points at header[4] and wide_min_units != 0 switches the check on.
  const int4* tiles_alt;
  int wide_gate;
  int wide_min_units;
  int n_groups;             // upper bound on the number of groups
  int uniform_count;
  int uniform_stride;
  int uniform_first;
  int delta_step;
  int n_deltas;             // deltas with index outside [0, n_deltas) are skipped
  int accumulate;           // 0: out = result, 1: out += result
  int raw_static;           // fused routing with group g = delta g: weights are requested before the indices arrive
  int rot_spread;           // steps between the starting points of consecutive deltas' walks over K (0: all start at step 0)
  int xcd_swizzle;          // 1: remap column blocks so that each XCD owns a contiguous run; 5 (streaming kernel): whole groups per XCD
  int xcd_cgs;              // wide kernel, order 4: column groups (of 512) in the block that one XCD takes
  // K split across workgroups (uniform groups only): blockIdx.z = z takes the steps [z * ksplit_steps, (z + 1) * ksplit_steps)
  // of K and writes its fp32 sums, unscaled, to partial[z][row][column]; splitk_reduce_kernel adds the splits in
  // the order of z and finishes the rows.  ksplit_steps = 0: no split.
  float* partial;
  long partial_rows;        // rows of one split's block in `partial` (= rows of `out`)
  int ksplit_steps;
  // A workgroup takes 128 >> sub_shift columns of a column block (0..3): launches of a few dozen workgroups are bound
  // by what one CU's memory pipeline delivers (about 30 GB/s however many wavefronts and requests it has in flight),
  // so the same work spread over more CUs is faster.  Each output column is still summed over K by the same wavefronts
  // in the same order: the bits do not depend on sub_shift.
  int sub_shift;
  // 1: the plan's tiles hold up to 64 tokens and the 32-token build of the wide kernel takes each as two halves
  // (workgroups 2g and 2g + 1 of a column group; a half without tokens returns at once)
  int tile_halves;
  int scale_groups;         // 0: one scale per output column; else k / 128 groups of K, each with a scale per column
  // A plan with wide tiles on a layer whose wide launch fills the chip.  The wide kernel leaves a delta's last tokens
  // (fewer than 64) to the narrow kernel, a second stream of that delta's weights.  Where ONE list of 64-token tiles
  // over all tokens (tiles_all64; plan_header[all64_index] of them) needs no more rounds of the workgroups that run
  // together than the wide tiles alone, the wide kernel takes that list and the narrow kernel returns at once: decided
  // on the device, by both kernels alike, from the numbers of tiles in the plan's header.  nullptr: never.
  const int4* tiles_all64;
  const int* plan_header;
  int all64_index;
};

// workgroups of the 64-token wide kernel that run together: two on each of 256 CUs
constexpr int kWideSlots = 512;
__device__ __forceinline__ bool plan_takes_all64(const Sparse24Args& p) {
  const int wide = p.plan_header[4], all = p.plan_header[p.all64_index];
  if ((long)wide * p.wide_gate < p.wide_min_units) return false;   // (no wide launch at all: the narrow kernel takes every token)
  // wide_gate = column groups of the layer = workgroups per tile
  return (all * p.wide_gate + kWideSlots - 1) / kWideSlots <= (wide * p.wide_gate + kWideSlots - 1) / kWideSlots;
}

__device__ __forceinline__ uint32_t h2_bits(half2_t v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ half2_t bits_h2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

// (w & mask) | 0x64006400 in one instruction: a bitfield insert of w's masked bits into the fp16
// pair (1024, 1024).  (The compiler would emit an AND and an OR: VOP3 takes no two literals.)
__device__ __forceinline__ uint32_t insert_into_1024(uint32_t w, uint32_t mask) {
  uint32_t r;
  const uint32_t magic = 0x64006400u;
  asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(r) : "s"(mask), "v"(w), "v"(magic));
  return r;
}
// nibbles 0 and 4 of w -> (n0 - 8, n4 - 8)
__device__ __forceinline__ uint32_t dequant_even(uint32_t w) {
  const half2_t bias = {(_Float16)1032.0f, (_Float16)1032.0f};
  return h2_bits(bits_h2(insert_into_1024(w, 0x000f000fu)) - bias);
}
// nibbles 1 and 5 of w -> (n1 - 8, n5 - 8):  (1024 + 16 n) / 16 - 72
__device__ __forceinline__ uint32_t dequant_odd(uint32_t w) {
  const half2_t mul = {(_Float16)0.0625f, (_Float16)0.0625f};
  const half2_t add = {(_Float16)-72.0f, (_Float16)-72.0f};
  return h2_bits(bits_h2(insert_into_1024(w, 0x00f000f0u)) * mul + add);
}

// fp16(old + acc * scale) with every step rounded on its own (fp32 product, fp32 sum, then fp16), and
// the same expression whether or not there is an `old` to add to (0 otherwise).  Left to itself
// the compiler fuses some instances of this into a single-rounding mixed-precision fma and not
// others, so that the same row could differ in its last bit between two builds of the kernel
// (token-tile sizes, accumulate or not); results must not depend on which kernel ran.
__device__ __forceinline__ _Float16 scaled_sum_f16(_Float16 old, float acc, _Float16 scale) {
#pragma clang fp contract(off)
  const float prod = acc * (float)scale;
  const float sum = (float)old + prod;
  return (_Float16)sum;
}

// Workgroup barrier that orders LDS traffic only: outstanding global loads (the prefetch
// ring) are not waited for.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int NT>
struct StepFrag {
  uint4_t wq[4];        // weights: groups a and a+4 (a = vector index) of 8 columns
  uint4_t mt[2];        // metadata vectors (b1 = 0, 1)
  uint4_t xa[NT][2];    // B slots 0..7 for u = 0, 1
  uint4_t xb[NT][2];    // B slots 8..15 for u = 0, 1
  uint4_t gs[4];        // grouped scales only: the step's scales of this lane's 4 x 8 output columns
};

// weights and metadata of one step, requested ahead of a tile pass
struct WPre {
  uint4_t wq[4];
  uint4_t mt[2];
};

constexpr int kRawParts = 4;     // fused routing: tokens per lane, i.e. batches of up to 256 tokens

constexpr int kRedStride = 132;  // floats per token row in the reduction buffer (128 + pad)

// Everything one workgroup knows about its (group, column block) before touching tokens.
struct TileCtx {
  const uint4_t* qw_lane;   // this lane's first weight vector in packed row 0
  const uint4_t* mt_lane;   // this lane's first metadata vector in packed row 0
  const _Float16* sc;       // scales of the 128 columns
  long qrow, mrow;          // vectors per packed row (weights, metadata)
  int k_rows, n_steps;      // packed rows, 128-k steps
  int rot;                  // this delta's walk over K starts at step `rot` and wraps around
  int step0;                // first step of this workgroup's share of K (K split across workgroups), else 0
  int cb;                   // column block
  int ra;                   // the 8-column block (0..15) of the column block whose weights this lane loads: r, or with
                            // sub_shift > 0 one of the 16 >> sub_shift blocks of this workgroup's share
  int col0;                 // first column of this workgroup's share inside the column block
  int nblk_shift;           // log2 of the 8-column blocks in the share (4 - sub_shift)
  int tid, wave, lane, r, q;
  // fused routing (up to kRawParts x 64 tokens, kRawParts per lane): for part j of the batch (tokens
  // 64 j .. 64 j + 63), lane s of raw_list[j] holds the s-th of the group's tokens in that part, and
  // raw_before[j] counts the group's tokens in the parts before it.  The group's slots run through
  // the parts in order.
  int raw_list[kRawParts];
  int raw_before[kRawParts + 1];
};

// One pass over K for up to 16*NTT tokens of one group: loads, sparse MFMAs, cross-wave
// reduction, scaled fp16 store.  `first` = index of the pass's first token in the group's list.
// NPRE: the weights of this wave's first NPRE (<= DEPTH) steps are already on their way in `pre`.
// GS: grouped scales (one scale per column and 128-k step instead of one per column): each step's MFMAs start from
// zero and their sums enter the running sums times the step's scales.
template <int NTT, int KW, int DEPTH, int NPRE = 0, bool GS = false>
__device__ __forceinline__ void tile_pass(const Sparse24Args& p, TileCtx& c, int first, int cnt,
                                          float (*red)[16][kRedStride], int* s_rows, const WPre* pre = nullptr) {
  const int r = c.r, q = c.q, wave = c.wave;
  const int k_rows = c.k_rows, n_steps = c.n_steps;
  // The i-th step of a delta's walk over K is step (i + rot) mod n_steps of the matrix: deltas
  // that are streamed side by side sit a power of two apart in memory, and in lockstep they
  // would hit the same DRAM banks at the same moment (measured: 16 deltas of 4096 x 4096
  // stream at 4.8 TB/s in lockstep, at 5.7 TB/s with their walks spread around the ring).
  auto phys = [&](int st) {
    const int ps = st + c.rot;
    return c.step0 + (st < n_steps ? (ps < n_steps ? ps : ps - n_steps) : 0);
  };

  // Steps past the end of K (st >= n_steps) read step 0 again: cheap cache hits that keep the
  // load count per iteration constant; they are never multiplied.
  auto load_w = [&](StepFrag<NTT>& f, int st) {
    const int tr0 = phys(st) << 2;
    const int tr = min(tr0 + q, k_rows - 1);  // clamped: rows past the end are cancelled by zero B
    const uint4_t* wp = c.qw_lane + (long)tr * c.qrow;
    const uint4_t* mp = c.mt_lane + (long)tr * c.mrow;
#pragma unroll
    for (int a = 0; a < 4; a++) f.wq[a] = wp[a];
    f.mt[0] = mp[0];
    f.mt[1] = mp[8];
    if constexpr (GS) {
      // D rows 4q + j of this lane = columns 8 (4q + j) .. + 7 of the column block
      const _Float16* sp = c.sc + (long)phys(st) * p.m + 32 * q;
#pragma unroll
      for (int j = 0; j < 4; j++) f.gs[j] = *reinterpret_cast<const uint4_t*>(sp + 8 * j);
    }
  };

  // Start-up order matters (vector loads return in order): first the tiny per-lane read of
  // this lane's token rows, then the weight stream (which only needs the delta id), and the
  // activation loads once the rows have arrived.  No barrier is needed before the K loop.
  int rows[NTT];
#pragma unroll
  for (int nt = 0; nt < NTT; nt++) {
    const int slot = min(nt * 16 + r, cnt - 1);   // slots past the end re-read the last row
    if (p.raw_indices) {
      const int sigma = first + slot;
      int row = 0;
#pragma unroll
      for (int j = 0; j < kRawParts; j++) {
        const int v = __shfl(c.raw_list[j], sigma - c.raw_before[j], 64);
        if (sigma >= c.raw_before[j] && sigma < c.raw_before[j + 1]) row = v;
      }
      rows[nt] = row;
    } else rows[nt] = p.perm ? p.perm[first + slot] : first + slot;
  }
  StepFrag<NTT> ring[DEPTH];
#pragma unroll
  for (int j = 0; j < DEPTH; j++) {
    if (j < NPRE) {
#pragma unroll
      for (int a = 0; a < 4; a++) ring[j].wq[a] = pre[j].wq[a];
      ring[j].mt[0] = pre[j].mt[0];
      ring[j].mt[1] = pre[j].mt[1];
    } else {
      load_w(ring[j], wave + j * KW);
    }
  }

  // The scales of this thread's 8 output features, for the epilogue: requested here, behind the first
  // weights, so that no wait for them can land ahead of a request (requested before the loop over
  // passes they were waited for at the loop's entry: a full memory round trip before the first weights).
  half8_t sv = {1, 1, 1, 1, 1, 1, 1, 1};
  if constexpr (!GS) sv = *reinterpret_cast<const half8_t*>(c.sc + c.col0 + (c.tid & ((1 << c.nblk_shift) - 1)) * 8);

  // Every lane always loads from a valid address, so that the number of loads per step is
  // fixed and the hardware load counter can be waited on exactly (the output columns of the
  // duplicated slots are never stored).
  const _Float16* xrow[NTT];
#pragma unroll
  for (int nt = 0; nt < NTT; nt++) {
    // B operand slot layout: this lane supplies k offsets 8*(q%2) + {0..7} of
    // packed rows tr0 + q/2 and tr0 + 2 + q/2
    xrow[nt] = p.x + (long)rows[nt] * p.x_stride + 32 * (q >> 1) + 8 * (q & 1);
  }
  if (wave == 0 && q == 0) {
#pragma unroll
    for (int nt = 0; nt < NTT; nt++) s_rows[nt * 16 + r] = (nt * 16 + r < cnt) ? rows[nt] : -1;
  }

  float4_t acc[8][NTT];
#pragma unroll
  for (int cc = 0; cc < 8; cc++)
#pragma unroll
    for (int nt = 0; nt < NTT; nt++) acc[cc][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

  auto load_x = [&](StepFrag<NTT>& f, int st) {
    const int tr0 = phys(st) << 2;
    // rows tr0+2.. may lie past the end of K in the last step: clamp the address, zero at use
    const long xoff_a = (long)min(tr0, k_rows - 1 - (q >> 1)) * 32;
    const long xoff_b = (long)min(tr0 + 2, k_rows - 1 - (q >> 1)) * 32;
#pragma unroll
    for (int nt = 0; nt < NTT; nt++) {
      f.xa[nt][0] = *reinterpret_cast<const uint4_t*>(xrow[nt] + xoff_a);
      f.xa[nt][1] = *reinterpret_cast<const uint4_t*>(xrow[nt] + xoff_a + 16);
      f.xb[nt][0] = *reinterpret_cast<const uint4_t*>(xrow[nt] + xoff_b);
      f.xb[nt][1] = *reinterpret_cast<const uint4_t*>(xrow[nt] + xoff_b + 16);
    }
  };

  auto compute_step = [&](const StepFrag<NTT>& f, int st) {
    const int tr0 = phys(st) << 2;
    const bool tail = tr0 + 4 > k_rows;            // wave-uniform: only the last, partial step
    const bool ok_a = (tr0 + (q >> 1)) < k_rows;
    const bool ok_b = (tr0 + 2 + (q >> 1)) < k_rows;
    if constexpr (GS) {
      // (K is a whole number of steps here.)  Column by column: the two MFMAs of a column (k halves u = 0, 1) start
      // from zero, and their sum enters the running sum times the scale of (this step, that column).
      half16_t b[2][NTT];
#pragma unroll
      for (int u = 0; u < 2; u++)
#pragma unroll
        for (int nt = 0; nt < NTT; nt++) {
          typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
          const uint8_t_v bb = {f.xa[nt][u][0], f.xa[nt][u][1], f.xa[nt][u][2], f.xa[nt][u][3],
                                f.xb[nt][u][0], f.xb[nt][u][1], f.xb[nt][u][2], f.xb[nt][u][3]};
          b[u][nt] = __builtin_bit_cast(half16_t, bb);
        }
#pragma unroll
      for (int cc = 0; cc < 8; cc++) {
        const int w = cc & 3, b2 = cc >> 2;
        float4_t part[NTT];
#pragma unroll
        for (int nt = 0; nt < NTT; nt++) part[nt] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 2; u++) {
          uint4_t av;
#pragma unroll
          for (int a = 0; a < 4; a++) {
            uint32_t word = f.wq[a][w];
            if (b2) word >>= 8;
            av[a] = u ? dequant_odd(word) : dequant_even(word);
          }
          const half8_t A = __builtin_bit_cast(half8_t, av);
          const int idx = (int)f.mt[(cc >> 1) & 1][(cc & 1) * 2 + u];
#pragma unroll
          for (int nt = 0; nt < NTT; nt++) {
            if (b2)
              part[nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A, b[u][nt], part[nt], idx, 0, 1);
            else
              part[nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A, b[u][nt], part[nt], idx, 0, 0);
          }
        }
        // column cc of a run of 8 is stored at position 0 2 4 6 1 3 5 7 [cc] of the run
        constexpr int kPos[8] = {0, 2, 4, 6, 1, 3, 5, 7};
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const half2_t pair = bits_h2(f.gs[j][kPos[cc] >> 1]);
          const float sc = (float)pair[kPos[cc] & 1];
#pragma unroll
          for (int nt = 0; nt < NTT; nt++) acc[cc][nt][j] = __builtin_fmaf(part[nt][j], sc, acc[cc][nt][j]);
        }
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      half16_t b[NTT];
#pragma unroll
      for (int nt = 0; nt < NTT; nt++) {
        typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
        uint8_t_v bb = {f.xa[nt][u][0], f.xa[nt][u][1], f.xa[nt][u][2], f.xa[nt][u][3],
                        f.xb[nt][u][0], f.xb[nt][u][1], f.xb[nt][u][2], f.xb[nt][u][3]};
        if (tail) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            if (!ok_a) bb[i] = 0u;
            if (!ok_b) bb[4 + i] = 0u;
          }
        }
        b[nt] = __builtin_bit_cast(half16_t, bb);
      }
#pragma unroll
      for (int cc = 0; cc < 8; cc++) {
        const int w = cc & 3;         // word inside each weight vector
        const int b2 = cc >> 2;       // upper / lower 4 columns of the 8-column block
        uint4_t av;
#pragma unroll
        for (int a = 0; a < 4; a++) {
          uint32_t word = f.wq[a][w];
          if (b2) word >>= 8;
          av[a] = u ? dequant_odd(word) : dequant_even(word);
        }
        const half8_t A = __builtin_bit_cast(half8_t, av);
        const int idx = (int)f.mt[(cc >> 1) & 1][(cc & 1) * 2 + u];
#pragma unroll
        for (int nt = 0; nt < NTT; nt++) {
          if (b2)
            acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A, b[nt], acc[cc][nt], idx, 0, 1);
          else
            acc[cc][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(A, b[nt], acc[cc][nt], idx, 0, 0);
        }
      }
    }
  };

  // K loop: wave w takes steps w, w + KW, ...; DEPTH steps of loads are kept in flight in
  // registers (ring of fragments, statically indexed through the unrolled inner loop).
  // The body is branch-free apart from the wave-uniform "is this step real" test around the
  // arithmetic, so each iteration issues the same loads and waits for exactly its own.
#pragma unroll
  for (int j = 0; j < DEPTH; j++) load_x(ring[j], wave + j * KW);
  for (int st = wave; st < n_steps; st += DEPTH * KW) {
#pragma unroll
    for (int j = 0; j < DEPTH; j++) {
      const int cur = st + j * KW;
      if (cur < n_steps) compute_step(ring[j], cur);
      load_w(ring[j], cur + DEPTH * KW);
      load_x(ring[j], cur + DEPTH * KW);
    }
  }

  // cross-wave reduction + epilogue, one 16-token tile at a time
#pragma unroll
  for (int nt = 0; nt < NTT; nt++) {
    if (nt * 16 >= cnt) break;
    if (nt > 0) lds_barrier();
    // D: lane (n = r, qq = q) owns rows 4q + j of the MFMA, i.e. columns 8 (4q + j) + c of the workgroup's share (rows
    // past the share, when it is narrower than 128 columns, repeat its blocks and are never read back)
    float* dst = &red[wave][r][32 * q];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      float4_t lo = {acc[0][nt][j], acc[1][nt][j], acc[2][nt][j], acc[3][nt][j]};
      float4_t hi = {acc[4][nt][j], acc[5][nt][j], acc[6][nt][j], acc[7][nt][j]};
      *reinterpret_cast<float4_t*>(dst + 8 * j) = lo;
      *reinterpret_cast<float4_t*>(dst + 8 * j + 4) = hi;
    }
    lds_barrier();
    // 16 tokens x (128 >> sub_shift) features in chunks of 8 features
    for (int ch = c.tid; ch < (16 << c.nblk_shift); ch += 64 * KW) {
      const int tok = ch >> c.nblk_shift;
      const int f0 = (ch & ((1 << c.nblk_shift) - 1)) * 8;
      const int row = s_rows[nt * 16 + tok];
      if (row < 0) continue;
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = 0.f;
#pragma unroll
      for (int w = 0; w < KW; w++) {
        const float4_t a0 = *reinterpret_cast<const float4_t*>(&red[w][tok][f0]);
        const float4_t a1 = *reinterpret_cast<const float4_t*>(&red[w][tok][f0 + 4]);
#pragma unroll
        for (int i = 0; i < 4; i++) { v[i] += a0[i]; v[4 + i] += a1[i]; }
      }
      if (p.ksplit_steps) {
        // this workgroup's share of K only: the sums go to its block of the partial buffer as they are
        float* pp = p.partial + ((long)blockIdx.z * p.partial_rows + row) * p.m + c.cb * 128 + c.col0 + f0;
        *reinterpret_cast<float4_t*>(pp) = float4_t{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<float4_t*>(pp + 4) = float4_t{v[4], v[5], v[6], v[7]};
        continue;
      }
      // (sv: f0 is the same for every chunk of a thread, 64 * KW being a multiple of 16)
      _Float16* op = p.out + (long)row * p.out_stride + c.cb * 128 + c.col0 + f0;
      half8_t old = {0, 0, 0, 0, 0, 0, 0, 0};
      if (p.accumulate) old = *reinterpret_cast<const half8_t*>(op);
      half8_t o;
#pragma unroll
      for (int i = 0; i < 8; i++) o[i] = scaled_sum_f16(old[i], v[i], sv[i]);
      *reinterpret_cast<half8_t*>(op) = o;
    }
  }
}

// NT = widest token tile (16*NT tokens per pass) the instantiation supports; narrower passes
// take the cheaper code path (fewer activation loads and MFMAs) at the same register budget.
// EAGER: fused routing with group g = delta g (Sparse24Args::raw_static): the weights of the first
// step are requested at once, together with the indices, instead of one memory round trip later.
template <int NT, int KW, int DEPTH, bool EAGER = false, bool GS = false>
__global__ __launch_bounds__(64 * KW, (NT == 1 ? (DEPTH == 1 && !GS ? 3 : 2) : (NT == 2 && !GS ? 2 : 1))) void sparse24_grouped_kernel(const Sparse24Args p) {
  // steps per wave requested ahead of the routing in the EAGER build (the 32- and 64-token builds
  // also hold narrower passes with a ring of their own depth: one step fits them all)
  constexpr int NPRE = EAGER ? (NT == 1 ? DEPTH : 1) : 0;
  __shared__ float red[KW][16][kRedStride];
  __shared__ int s_rows[16 * NT];

  // Unit = (group, column block).  Workgroups are dealt round-robin to the 8 XCDs (each with
  // its own L2); the column blocks of a group are numbered so that every XCD owns a contiguous
  // run of them: the per-group unit count is padded to a multiple of 8 (padding units exit).
  // (with sub_shift > 0 the same holds for the shares of column blocks)
  const int col_units = (p.m >> 7) << p.sub_shift;
  const int cu_pad = (col_units + 7) & ~7;
  const int unit = blockIdx.x;
  int grp = unit / cu_pad;
  int i = unit - grp * cu_pad;
  int cu = p.xcd_swizzle ? (i & 7) * (cu_pad >> 3) + (i >> 3) : i;
  if (p.xcd_swizzle == 5) {
    // Whole groups per XCD, for launches whose groups all have work (the host asks for this order only then): the
    // first 8 * gpx groups go gpx to an XCD, with all their column units, so that an XCD's L2 fetches the activations
    // of its own groups only and streams whole matrices; the groups that are left over keep the order above.
    const int gpx = p.n_groups >> 3;
    if (unit < 8 * gpx * cu_pad) {
      const int xcd = unit & 7, s = unit >> 3;
      grp = xcd * gpx + s / cu_pad;
      cu = s - (s / cu_pad) * cu_pad;
    }
  }
  if (cu >= col_units) return;
  const int cb = cu >> p.sub_shift;

  TileCtx c;
  c.tid = threadIdx.x;
  c.wave = c.tid >> 6;
  c.lane = c.tid & 63;
  c.r = c.lane & 15;
  c.q = c.lane >> 4;
  c.cb = cb;
  c.nblk_shift = 4 - p.sub_shift;
  {
    const int sub = cu & ((1 << p.sub_shift) - 1);
    c.ra = (sub << c.nblk_shift) + (c.r & ((1 << c.nblk_shift) - 1));
    c.col0 = sub << (7 - p.sub_shift);
  }
#pragma unroll
  for (int j = 0; j < kRawParts; j++) c.raw_list[j] = c.raw_before[j] = 0;
  c.raw_before[kRawParts] = 0;
  c.k_rows = p.k >> 5;                 // packed rows (32 dense k each)
  c.n_steps = (c.k_rows + 3) >> 2;     // 128 dense k per step
  c.step0 = 0;
  if (p.ksplit_steps) {                // this workgroup's share of the steps (the last share may be short, never empty)
    c.step0 = blockIdx.z * p.ksplit_steps;
    c.n_steps = min(p.ksplit_steps, c.n_steps - c.step0);
  }
  c.qrow = p.m >> 1;
  c.mrow = p.m >> 2;
  // everything that depends on the delta: operand pointers and the request for this thread's scales
  auto bind_delta = [&](int delta) {
    c.qw_lane = p.qweight + (long)delta * p.qweight_stride + (long)cb * 64 + 4 * c.ra;
    c.mt_lane = p.meta + (long)delta * p.meta_stride + (long)(cb * 2 + (c.ra >> 3)) * 16 + (c.ra & 7);
    c.sc = p.scales + (long)delta * p.scales_stride + cb * 128;   // (GS: row 0 of the delta's groups)
    // side-by-side deltas start their walks spread around the ring of steps (by the delta's index,
    // so that a result does not depend on where the weights happen to lie in memory)
    // (32-bit arithmetic: a 64-bit remainder is a routine of some 150 instructions ahead of the first request;
    // any value in [0, n_steps) is a valid start, so a wrapped product for a huge delta index does no harm)
    c.rot = (int)(((unsigned)delta * (unsigned)p.rot_spread) % (unsigned)c.n_steps);
  };

  // group descriptor and live group count are fetched side by side (no dependent chain);
  // grp < p.n_groups (the host's upper bound) keeps the descriptor reads in bounds
  int delta, start, count;
  bool alt_list = false;
  WPre pre[NPRE > 0 ? NPRE : 1];
  if (EAGER || p.raw_indices) {   // (the eager build serves this form only: the others compile away)
    // Fused routing for small batches: every wavefront looks at all (<= 64) indices, one per
    // lane, and works out its delta and the rows routed to it -- a few dozen instructions
    // instead of a separate routing launch and a dependent descriptor read.
    int d[kRawParts];     // this lane's tokens: lane, 64 + lane, ...
#pragma unroll
    // (every lane loads from a valid address, the last index standing in for those past the end: loads under a branch
    // make the compiler wait for everything in flight -- the weights requested below included -- before the first use
    // of an index, instead of for the indices alone)
    for (int j = 0; j < kRawParts; j++) d[j] = p.raw_indices[min(64 * j + c.lane, p.raw_count - 1)];
    if (EAGER) {
      // group g is delta g: its first weights are requested right behind the indices
      if (grp >= p.n_deltas) return;
      delta = grp;
      bind_delta(delta);
      // Only the workgroup that takes a group's first tokens needs them: the others of a launch that splits a group's
      // tokens over blockIdx.y mostly find nothing to do, and a step each would be traffic for nothing.  They issue the
      // same loads on packed row 0 instead (one hot piece per column block), because requests under a branch would make
      // the compiler wait for everything in flight before the first use of an index: where two paths meet it assumes
      // the shorter queue, and "all but the newest 0" then includes these weights, a cold round trip to HBM, ahead of
      // the routing.
      const bool lead = blockIdx.y == 0;
#pragma unroll
      for (int j = 0; j < NPRE; j++) {
        const int st = c.wave + j * KW;              // this wave's j-th step (beyond the end of K: loads go unused)
        int ps = st + c.rot;
        if (ps >= c.n_steps) ps -= c.n_steps;
        if (st >= c.n_steps) ps = 0;
        const int tr = lead ? min((ps << 2) + c.q, c.k_rows - 1) : 0;
        const uint4_t* wp = c.qw_lane + (long)tr * c.qrow;
        const uint4_t* mp = c.mt_lane + (long)tr * c.mrow;
#pragma unroll
        for (int a = 0; a < 4; a++) pre[j].wq[a] = wp[a];
        pre[j].mt[0] = mp[0];
        pre[j].mt[1] = mp[8];
      }
      // nothing that needs the indices may be scheduled (with its wait) ahead of these requests
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int j = 0; j < kRawParts; j++) {
      const int v = d[j] - p.raw_offset;
      d[j] = (64 * j + c.lane < p.raw_count && v >= 0 && v < p.n_deltas) ? v : -1;
    }
    const unsigned long long below = (1ull << c.lane) - 1ull;
    if (!EAGER) {
      // the grp-th delta in use
      unsigned long long used = 0ull;
#pragma unroll
      for (int j = 0; j < kRawParts; j++) used |= d[j] >= 0 ? (1ull << d[j]) : 0ull;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const unsigned lo = __shfl_xor((unsigned)used, off, 64);
        const unsigned hi = __shfl_xor((unsigned)(used >> 32), off, 64);
        used |= ((unsigned long long)hi << 32) | lo;
      }
      if (grp >= __popcll(used)) return;
      const bool is_grp = ((used >> c.lane) & 1ull) && __popcll(used & below) == grp;
      delta = __ffsll((long long)__ballot(is_grp)) - 1;
    }
    // slot s of the group = its s-th member token.  Per part of the batch, a full permutation sends
    // every member's token id to the lane of its rank (non-members fill the lanes after the members)
    count = 0;
    start = 0;
#pragma unroll
    for (int j = 0; j < kRawParts; j++) {
      const unsigned long long members = __ballot(d[j] == delta);
      const int cj = __popcll(members);
      const int rank = __popcll(members & below);
      const int dest = (d[j] == delta) ? rank : cj + (c.lane - rank);
      c.raw_list[j] = __builtin_amdgcn_ds_permute(dest << 2, 64 * j + c.lane);
      c.raw_before[j] = count;
      count += cj;
    }
    c.raw_before[kRawParts] = count;
    if (EAGER && count <= 0) {
      __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): let the requested weights land before the wave ends
      return;
    }
  } else if (p.tiles) {
    int4 d = p.tiles[grp];
    if (p.tiles_alt) {
      // both candidates and the header are requested together; the choice costs no extra round trip
      const int4 d_alt = p.tiles_alt[grp];
      if ((long)p.n_groups_dev[4] * p.wide_gate < p.wide_min_units) {
        d = d_alt;
        alt_list = true;
      } else if (p.tiles_all64 && plan_takes_all64(p)) {
        return;   // the wide kernel takes every token of this plan
      }
    }
    delta = d.x;
    start = d.y;
    count = d.z;
  } else if (p.g_delta) {
    delta = p.g_delta[grp];
    start = p.g_start[grp];
    count = p.g_count[grp];
  } else {
    delta = grp * p.delta_step;
    start = grp * p.uniform_stride + p.uniform_first;
    count = p.uniform_count;
  }
  if (!EAGER) {
    const int n_groups = p.n_groups_dev ? p.n_groups_dev[alt_list ? 5 : 0] : p.n_groups;
    if (grp >= n_groups) return;
    if (delta < 0 || delta >= p.n_deltas || count <= 0) return;
    bind_delta(delta);
  }

  // blockIdx.y splits a group's tokens between workgroups (each re-streams the weights)
  int t0 = blockIdx.y * 16 * NT;
  if (EAGER && blockIdx.y == 0 && t0 < count) {
    // The pass that uses the weights requested ahead of the routing stands on its own, ahead of the loop over the
    // other passes: inside that loop the compiler has to keep `pre` alive for every iteration, cannot let the K loop's
    // ring take over its registers, and copies it into the ring instead -- with a wait for those weights, a cold round
    // trip to HBM, ahead of the first activation request (measured: 1.8 us between the routing and that request).
    const int cnt = min(count - t0, 16 * NT);
    if (NT == 1 || cnt <= 16) {
      tile_pass<1, KW, (NT == 1 ? DEPTH : 2), NPRE>(p, c, start + t0, cnt, red, s_rows, pre);
    } else if (NT == 2 || cnt <= 32) {
      tile_pass<(NT >= 2 ? 2 : 1), KW, (NT == 2 ? DEPTH : 2), NPRE>(p, c, start + t0, cnt, red, s_rows, pre);
    } else {
      tile_pass<NT, KW, DEPTH, NPRE>(p, c, start + t0, cnt, red, s_rows, pre);
    }
    t0 += gridDim.y * 16 * NT;
    if (t0 < count) lds_barrier();    // the next pass over this group's tokens reuses s_rows / red
  }
  for (; t0 < count; t0 += gridDim.y * 16 * NT) {
    const int cnt = min(count - t0, 16 * NT);
    if (NT == 1 || cnt <= 16) {
      tile_pass<1, KW, (NT == 1 ? DEPTH : 2), 0, GS>(p, c, start + t0, cnt, red, s_rows);
    } else if (NT == 2 || cnt <= 32) {
      tile_pass<(NT >= 2 ? 2 : 1), KW, (NT == 2 ? DEPTH : 2), 0, GS>(p, c, start + t0, cnt, red, s_rows);
    } else {
      tile_pass<NT, KW, DEPTH, 0, GS>(p, c, start + t0, cnt, red, s_rows);
    }
    // the next pass over this group's tokens reuses s_rows / red
    if (t0 + gridDim.y * 16 * NT < count) lds_barrier();
  }
}

// Second pass of a K split across workgroups: out[row] = fp16(sum over splits, in the order of the splits, x scale).
// One thread per 8 columns of a row; `rows_per_group` rows in a row share a delta (delta = group x delta_step).
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int splits, long rows, int m,
                                                           const _Float16* __restrict__ scales, long scales_stride,
                                                           int rows_per_group, int delta_step, _Float16* __restrict__ out,
                                                           long out_stride) {
  const long chunk = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_row = m >> 3;
  const long row = chunk / per_row;
  if (row >= rows) return;
  const int f0 = (int)(chunk - row * per_row) * 8;
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; i++) v[i] = 0.f;
  for (int z = 0; z < splits; z++) {
    const float* pp = partial + ((long)z * rows + row) * m + f0;
    const float4_t a0 = *reinterpret_cast<const float4_t*>(pp);
    const float4_t a1 = *reinterpret_cast<const float4_t*>(pp + 4);
#pragma unroll
    for (int i = 0; i < 4; i++) { v[i] += a0[i]; v[4 + i] += a1[i]; }
  }
  const long delta = (row / rows_per_group) * delta_step;
  const half8_t sv = *reinterpret_cast<const half8_t*>(scales + delta * scales_stride + f0);
  half8_t o;
#pragma unroll
  for (int i = 0; i < 8; i++) o[i] = scaled_sum_f16((_Float16)0, v[i], sv[i]);
  *reinterpret_cast<half8_t*>(out + row * out_stride + f0) = o;
}

}  // namespace triteia_hip
