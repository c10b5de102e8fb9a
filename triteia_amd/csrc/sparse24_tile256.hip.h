// 256-token x 256-column workgroup tiles of the fp16 x (int4, 2:4-sparse) GEMM for gfx950: the form for
// groups with hundreds of tokens, where the matrix cores bound the work.
//
// Same packed layout and sparse-MFMA instruction as sparse24_grouped_kernel (sparse24_gemm.hip.h).  What is
// different is who dequantises what.  A workgroup has 8 wavefronts; wavefront (tq, cj) owns the 64 tokens
// tq (of 4) x the 128-column block cj (of 2) of the tile, i.e. 32 accumulator fragments of 16 x 16.  A
// dequantised weight fragment (the A operand of one MFMA) is the same for the four wavefronts of a column
// block, so each of them converts a quarter of the block's fragments into LDS and all four read them back:
// int4 -> fp16 conversion work per MFMA is a quarter of what a wavefront that converts for itself spends,
// and one 16-byte LDS read feeds 4 MFMAs.
//
// K is walked in steps of 64 (two packed rows).  The MFMA's K = 64 is laid out so that one step is exactly
// one contiguous 128-byte piece of every token row: lane quarter q of the A operand takes packed row
// 2t + q/2, 2:4 groups 4(q%2) .. 4(q%2)+3 (dense k 32(q/2) + 16(q%2) .. +15 of the step), and the metadata word
// of that (column, 16-k block) is its index operand unchanged; the B operand of lane (n, q) is the 16-byte
// chunks q and q + 4 of token n's 128 bytes.
//
// Every byte comes from global memory by direct-to-LDS loads (global_load_lds_dwordx4, no registers in
// between), issued a fixed number per wavefront and step, so one hand-counted s_waitcnt per step says "my
// part of this step's operands has landed" and nothing the compiler tracks is ever in flight across a
// barrier:
//   x tiles   [3 stages][256 tokens][128 B]   requested 3 steps ahead of the MFMAs (2 ahead of the LDS reads); chunk c of token n sits at chunk
//                                             position c ^ ((n >> 1) & 7), which makes the 16 rows of one
//                                             ds_read_b128 fall into distinct banks
//   staging   [5 stages][2 blocks][3 KB]      packed weights (2 rows x 1 KB) and metadata (2 rows x 512 B) of
//                                             a step, requested 4 steps ahead (3 ahead of its conversion)
//   fragments [2][2 blocks][8][64 lanes][16 B] dequantised A operands of a step, written one step ahead
// One barrier per step.  Needs activations below 4 GiB (32-bit lane offsets) and k % 64 == 0.
#pragma once
#include <type_traits>

#include "sparse24_gemm.hip.h"

namespace triteia_hip {

constexpr int kT256Tokens = 256;
constexpr int kT256XStages = 3;
constexpr int kT256WStages = 5;                    // staging ring: requested 4 steps ahead of the step that multiplies it
constexpr int kT256XStageBytes = kT256Tokens * 128;
constexpr int kT256WStageBytes = 2 * 3 * 1024;
constexpr int kT256FragBytes = 2 * 8 * 64 * 16;    // one step, both column blocks
constexpr int kT256LdsBytes = kT256XStages * kT256XStageBytes + kT256WStages * kT256WStageBytes + 2 * kT256FragBytes + kT256Tokens * 4;

// unit = (token tile, pair of column blocks).  Consecutive workgroup ids go to the 8 XCDs in turn (each has
// its own L2): id % 8 is the XCD, and each XCD is given whole token tiles (all column pairs of a tile share
// the tile's activations through that L2) when there are at least 8 tiles, else whole column pairs (their
// token tiles share the pair's weights).  Ids past the padded ranges exit.
struct T256Unit { int tile, cp; bool valid; };
__host__ __device__ inline long t256_grid(long tiles, long ncp) {
  return tiles >= 8 ? 8 * ((tiles + 7) / 8) * ncp : 8 * ((ncp + 7) / 8) * tiles;
}
__device__ __forceinline__ T256Unit t256_unit(int id, int tiles, int ncp, int swizzle) {
  T256Unit u;
  if (!swizzle) {
    u.tile = id / ncp;
    u.cp = id - u.tile * ncp;
  } else {
    const int xcd = id & 7, slot = id >> 3;
    if (tiles >= 8) {
      const int j = slot / ncp;
      u.tile = xcd + 8 * j;
      u.cp = slot - j * ncp;
    } else {
      const int j = slot / tiles;
      u.cp = xcd + 8 * j;
      u.tile = slot - j * tiles;
    }
  }
  u.valid = u.tile < tiles && u.cp < ncp;
  return u;
}

__global__ __launch_bounds__(512, 1) void sparse24_tile256_kernel(const Sparse24Args p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char t256_lds[];
  unsigned char* const xs = t256_lds;                                              // x tiles
  unsigned char* const stg = xs + kT256XStages * kT256XStageBytes;                 // staging ring
  unsigned char* const frg = stg + kT256WStages * kT256WStageBytes;                // fragments, double-buffered
  int* const s_rows = reinterpret_cast<int*>(frg + 2 * kT256FragBytes);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tq = wave & 3;          // token quarter of the tile; also: which quarter of the fragments this wave converts
  const int cj = wave >> 2;         // column block of the pair
  const int lane = tid & 63;
  const int r = lane & 15;
  const int q = lane >> 4;

  // ---- which unit
  const int col_blocks = p.m >> 7;
  const int ncp = (col_blocks + 1) >> 1;
  const int chunks = (p.uniform_count + kT256Tokens - 1) / kT256Tokens;
  const int tiles = p.n_groups * chunks;      // n_groups = groups of the launch (uniform form only)
  const T256Unit un = t256_unit(blockIdx.x, tiles, ncp, p.xcd_swizzle);
  if (!un.valid) return;
  const int gi = un.tile / chunks, tc = un.tile - gi * chunks;
  const int delta = gi * p.delta_step;
  const int start = gi * p.uniform_stride + p.uniform_first + tc * kT256Tokens;
  const int cnt = min(kT256Tokens, p.uniform_count - tc * kT256Tokens);
  if (delta < 0 || delta >= p.n_deltas || cnt <= 0) return;

  const int cb = 2 * un.cp + cj;
  const bool active = cb < col_blocks && tq * 64 < cnt;     // (a wave without columns or tokens still loads, converts and syncs)
  const int nk = p.k >> 6;                                   // steps of 64
  const long qrow = (long)(p.m >> 1) * 16;                   // bytes per packed row: weights
  const long mrow = (long)(p.m >> 2) * 16;                   //                       metadata

  // ---- token rows of the tile (slots past the end repeat the last row; their outputs are dropped)
  if (tid < kT256Tokens) {
    const int slot = min(tid, cnt - 1);
    s_rows[tid] = p.perm ? p.perm[start + slot] : start + slot;
  }
  __syncthreads();

  // (Walking K in lockstep is what the L2 wants here: the 16 workgroups of an XCD that share a token tile ask for the
  // same piece of it at the same time and one fill serves them all.  Spreading their walks around the ring of steps
  // was measured: 40 % of the L2 requests then miss instead of the compulsory 13 %, and the launch is 5 % slower.)
  auto phys = [&](int t) { return min(t, nk - 1); };   // (steps past the end refetch the last one: never read)

  // ---- direct-to-LDS requests.  One instruction of a wavefront writes 1 KB of consecutive LDS (M0 + 16 * lane).
  // x tile of a step: 32 instructions, 4 per wave; instruction g = 4 * wave + ii covers token rows 8g .. 8g+7,
  // lane l the chunk position l % 8 of row 8g + l / 8, which holds the row's chunk (l % 8) ^ ((row >> 1) & 7).
  uint32_t xoff[4];
#pragma unroll
  for (int ii = 0; ii < 4; ii++) {
    const int row = 8 * (4 * wave + ii) + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    xoff[ii] = (uint32_t)(((long)s_rows[row] * p.x_stride + chunk * 8) * 2);
  }
  const uint32_t lds_x = (uint32_t)(uintptr_t)xs + 4096 * wave;
  // staging of a step: per column block two packed rows of weights (64 vectors each) and one instruction for the
  // metadata of both rows (32 vectors each); waves 0..5 issue one of the six each.  Weight vector 4r + a of a row
  // (8-column block r, 2:4 groups a and a + 4) goes to slot r + 16a of its KB: the conversion's 8-byte reads then
  // spread over the banks (in global order they would hit the same few).
  const int sj = wave / 3, sp = wave - 3 * sj;            // (block, part) for waves 0..5
  const int scb = min(2 * un.cp + sj, col_blocks - 1);
  const unsigned char* sbase;                              // global address of this wave's part in step 0, without the lane
  uint32_t soff, sstep;                                    // lane offset; bytes per step
  if (sp < 2) {
    sbase = reinterpret_cast<const unsigned char*>(p.qweight + (long)delta * p.qweight_stride) + sp * qrow + (long)scb * 1024;
    soff = 16 * (4 * (lane & 15) + (lane >> 4));
    sstep = (uint32_t)(2 * qrow);
  } else {
    sbase = reinterpret_cast<const unsigned char*>(p.meta + (long)delta * p.meta_stride) + (long)scb * 512;
    soff = (uint32_t)((lane >> 5) * mrow + 16 * (lane & 31));
    sstep = (uint32_t)(2 * mrow);
  }
  const uint32_t lds_s = (uint32_t)(uintptr_t)stg + (3 * sj + sp) * 1024;
  const bool stager = wave < 6;

  // A request group = the x tile of step tx (4 instructions), then this wave's part of the staging of step ts.
  // `xst` / `sst`: byte offsets of the stages they go to.  Part i (0..3: x, 4: staging) can be issued on its own: inside
  // a step the five instructions are spread over the MFMA groups, one each -- issued in one burst by all eight waves
  // right behind the barrier they fill the address unit's queue, and every wave then sits behind its own requests
  // (a wave issues in order) while the matrix cores idle: measured 0.3 us of a 1.2 us step.
  auto issue_part = [&](int i, int tx, uint32_t xst, int ts, uint32_t sst) {
    if (i < 4) {
      const _Float16* xb = p.x + phys(tx) * 64;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_x + xst + 1024 * i);
      asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(xoff[i]), "s"(xb), "{m0}"(dst) : "memory");
    } else if (stager) {
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_s + sst);
      const unsigned char* base = sbase + (long)phys(ts) * sstep;
      asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(soff), "s"(base), "{m0}"(dst) : "memory");
    }
  };
  auto issue = [&](int tx, uint32_t xst, int ts, uint32_t sst) {
#pragma unroll
    for (int i = 0; i < 5; i++) issue_part(i, tx, xst, ts, sst);
  };
  // waits until only the wave's newest `G` request groups, and the staging part of the one before them, are in flight
  auto wait_groups = [&](auto groups) {
    constexpr int G = decltype(groups)::value;
    if (stager) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(5 * G + 1) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" : : "n"(4 * G) : "memory");
  };

  // ---- conversion duty of this wave: columns c0, c0 + 1 of every 8-column block of its column block, i.e. words
  // w0, w0 + 1 of the weight vectors, upper or lower byte pair by b2.  Lane (r, vp = q % 2, rho = q / 2) takes packed row
  // rho, vectors 2 vp and 2 vp + 1 (2:4 groups a and a + 4 for a = 2 vp, 2 vp + 1) and writes the halves (e = 0, 1) of
  // both into the slots of lanes (r, 2 rho + e).
  const int b2 = tq >> 1;
  const int w0 = 2 * (tq & 1);
  const int vp = q & 1, rho = q >> 1;
  const uint32_t conv_src = (uint32_t)(cj * 3072 + rho * 1024 + (r + 32 * vp) * 16 + w0 * 4);
  const uint32_t conv_dst = (uint32_t)(cj * 8192 + (4 * b2 + w0) * 1024 + (r + 32 * rho) * 16 + 8 * vp);
  typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));
  struct Packed { uint2_t va, vb; };
  auto convert_load = [&](uint32_t sst) {   // this lane's packed words of a step: vectors 2 vp and 2 vp + 1, words w0, w0 + 1
    const unsigned char* src = stg + sst + conv_src;
    Packed pk;
    pk.va = *reinterpret_cast<const uint2_t*>(src);
    pk.vb = *reinterpret_cast<const uint2_t*>(src + 256);
    return pk;
  };
  auto convert_store = [&](int t, const Packed& pk, int ww) {   // fragments of column c0 + ww of step t
    unsigned char* dst = frg + (t & 1) * kT256FragBytes + conv_dst + ww * 1024;
    uint32_t a = pk.va[ww], b = pk.vb[ww];
    if (b2) { a >>= 8; b >>= 8; }
    const uint2_t even = {dequant_even(a), dequant_even(b)};
    const uint2_t odd = {dequant_odd(a), dequant_odd(b)};
    *reinterpret_cast<uint2_t*>(dst) = even;            // slot lane (r, 2 rho)
    *reinterpret_cast<uint2_t*>(dst + 256) = odd;       // slot lane (r, 2 rho + 1)
  };

  float4_t acc[8][4];
#pragma unroll
  for (int c = 0; c < 8; c++)
#pragma unroll
    for (int nt = 0; nt < 4; nt++) acc[c][nt] = float4_t{0.f, 0.f, 0.f, 0.f};

  // per-lane read addresses
  const uint32_t b_lo = (uint32_t)((tq * 64 + r) * 128 + ((q ^ (r >> 1)) << 4));     // chunk q of token row tq*64 + r (+ 16 nt)
  const uint32_t a_off = (uint32_t)(cj * 8192 + lane * 16);
  // metadata word of slot lane (r, q): packed row q / 2 of the step, 16-k block q % 2, vectors v0 and v0 + 8 of the row
  const uint32_t i_off = (uint32_t)(cj * 3072 + 2048 + (q >> 1) * 512 + ((r >> 3) * 16 + (r & 7)) * 16 + 4 * (q & 1));

  // B operand (16 halfs) of 16-token tile nt of this wave, from the x stage at byte offset xst
  auto read_b = [&](uint32_t xst, int nt) {
    const unsigned char* xp = xs + xst + nt * 2048;
    typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
    const uint4_t lo = *reinterpret_cast<const uint4_t*>(xp + b_lo);
    const uint4_t hi = *reinterpret_cast<const uint4_t*>(xp + (b_lo ^ 64));
    const uint8_t_v bb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(half16_t, bb);
  };
  auto mfma4 = [&](int c, const uint4_t& a, const half16_t (&b)[4], int index, int nt0 = 0, int nt1 = 4) {
    const half8_t Ah = __builtin_bit_cast(half8_t, a);
#pragma unroll
    for (int nt = nt0; nt < nt1; nt++) {
      if (c >= 4) acc[c][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(Ah, b[nt], acc[c][nt], index, 0, 1);
      else acc[c][nt] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(Ah, b[nt], acc[c][nt], index, 0, 0);
    }
  };

  // ring positions (byte offsets of stages), advanced once per step
  uint32_t x_cur = 0;     // x stage of step t, which is also where the tile of step t + 3 goes
  uint32_t s_cur = 0;     // staging stage of step t
  auto x_next = [&](uint32_t o) { return o == (kT256XStages - 1) * kT256XStageBytes ? 0u : o + kT256XStageBytes; };
  auto s_next = [&](uint32_t o) { return o == (kT256WStages - 1) * kT256WStageBytes ? 0u : o + kT256WStageBytes; };
  auto s_prev = [&](uint32_t o) { return o == 0u ? (kT256WStages - 1) * kT256WStageBytes : o - kT256WStageBytes; };

  // One step: 32 MFMAs on the B operands `bc` (read from LDS during the step before), with the reads for the next
  // step (`bn`), the A operands (one 16-byte read per 4 MFMAs, three ahead) and this wave's share of the next step's
  // conversion spread between them, so that LDS and the matrix cores work side by side.  The last eight MFMAs of a
  // step (columns 6 and 7) are held back and issued at the top of the next step, right behind its barrier: they cover
  // the latency of the first fragment reads that the barrier has just allowed, and the address arithmetic of the
  // requests.  (`bn` still holds the step before's B operands at that point; its registers are refilled afterwards.)
  uint4_t a_held[2] = {{0u, 0u, 0u, 0u}, {0u, 0u, 0u, 0u}};
  int i_held[2] = {0, 0};
  auto step = [&](int t, const half16_t (&bc)[4], half16_t (&bn)[4]) {
    const unsigned char* fst = frg + (t & 1) * kT256FragBytes + a_off;
    const unsigned char* ist = stg + s_cur + i_off;
    const uint32_t x_nxt = x_next(x_cur), s_nxt = s_next(s_cur);
    uint4_t A[4];
    A[0] = *reinterpret_cast<const uint4_t*>(fst);
    A[1] = *reinterpret_cast<const uint4_t*>(fst + 1024);
    A[2] = *reinterpret_cast<const uint4_t*>(fst + 2048);
    // index words: columns w (low half) and w + 4 (high half) for w = 0..3
    int idx[4];
    idx[0] = *reinterpret_cast<const int*>(ist);
    idx[1] = *reinterpret_cast<const int*>(ist + 8);
    idx[2] = *reinterpret_cast<const int*>(ist + 128);
    idx[3] = *reinterpret_cast<const int*>(ist + 136);
    const Packed pk = convert_load(s_nxt);
    if (t > 0) {
      mfma4(6, a_held[0], bn, i_held[0]);
      mfma4(7, a_held[1], bn, i_held[1]);
    }
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t s_prv = s_prev(s_cur);
#pragma unroll
    for (int c = 0; c < 6; c++) {
      if (c + 3 < 8) A[(c + 3) & 3] = *reinterpret_cast<const uint4_t*>(fst + (c + 3) * 1024);
      if (c < 4) bn[c] = read_b(x_nxt, c);
      if (c == 1) convert_store(t + 1, pk, 0);
      if (c == 2) convert_store(t + 1, pk, 1);
      // (a wave without tokens or columns of its own multiplies what it finds: its sums are dropped)
      mfma4(c, A[c & 3], bc, idx[c & 3], 0, 2);
      __builtin_amdgcn_sched_barrier(0);
      if (c < 5) issue_part(c, t + 3, x_cur, t + 4, s_prv);
      __builtin_amdgcn_sched_barrier(0);
      mfma4(c, A[c & 3], bc, idx[c & 3], 2, 4);
      __builtin_amdgcn_sched_barrier(0);
    }
    a_held[0] = A[2];
    a_held[1] = A[3];
    i_held[0] = idx[2];
    i_held[1] = idx[3];
    x_cur = x_nxt;
    s_cur = s_nxt;
  };

  // ---- pipeline.  Requests, in order: staging 0; groups (x 0, staging 1), (x 1, staging 2), (x 2, staging 3); then
  // in step t the group (x t + 3, staging t + 4).  A wave's requests complete in order, so "everything but the newest
  // ... has landed" is one counter wait.  At the barrier of step t: x tile t + 1 and staging t + 1 have landed
  // (everyone's parts), the fragments of step t are written, and what step t - 1 read (x tile t, fragments t - 1,
  // staging t - 1) is free.
  if (stager) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_s);
    const unsigned char* base = sbase + (long)phys(0) * sstep;
    asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(soff), "s"(base), "{m0}"(dst) : "memory");
  }
  issue(0, 0, 1, kT256WStageBytes);
  issue(1, kT256XStageBytes, 2, 2 * kT256WStageBytes);
  issue(2, 2 * kT256XStageBytes, 3, 3 * kT256WStageBytes);
  wait_groups(std::integral_constant<int, 2>{});     // staging 0 and x tile 0 are in LDS
  lds_barrier();
  {
    const Packed pk = convert_load(0);
    convert_store(0, pk, 0);
    convert_store(0, pk, 1);
  }
  half16_t b0[4], b1[4];
#pragma unroll
  for (int nt = 0; nt < 4; nt++) b0[nt] = read_b(0, nt);
  for (int t = 0; t < nk; t += 2) {
    wait_groups(std::integral_constant<int, 1>{});
    lds_barrier();
    step(t, b0, b1);
    if (t + 1 < nk) {
      wait_groups(std::integral_constant<int, 1>{});
      lds_barrier();
      step(t + 1, b1, b0);
    }
  }
  // the last step's held MFMAs: its B operands are in b0 for an odd number of steps, else in b1
  if (nk & 1) {
    mfma4(6, a_held[0], b0, i_held[0]);
    mfma4(7, a_held[1], b0, i_held[1]);
  } else {
    mfma4(6, a_held[0], b1, i_held[0]);
    mfma4(7, a_held[1], b1, i_held[1]);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive the block's LDS

  if (!active) return;
  // epilogue: lane (n = r, qq = q) holds features 32q + 8j + c of token tq*64 + 16nt + r
  const _Float16* sc = p.scales + (long)delta * p.scales_stride + cb * 128 + 32 * q;
  half8_t sv[4];
#pragma unroll
  for (int j = 0; j < 4; j++) sv[j] = *reinterpret_cast<const half8_t*>(sc + 8 * j);
#pragma unroll
  for (int nt = 0; nt < 4; nt++) {
    const int slot = tq * 64 + nt * 16 + r;
    if (slot >= cnt) continue;
    _Float16* op = p.out + (long)s_rows[slot] * p.out_stride + cb * 128 + 32 * q;
    // (when the sums are added to what is there: a token's four pieces are requested together, ahead of the arithmetic)
    half8_t olds[4];
#pragma unroll
    for (int j = 0; j < 4; j++) olds[j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (p.accumulate) {
#pragma unroll
      for (int j = 0; j < 4; j++) olds[j] = *reinterpret_cast<const half8_t*>(op + 8 * j);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      half8_t o;
#pragma unroll
      for (int c = 0; c < 8; c++) o[c] = scaled_sum_f16(olds[j][c], acc[c][nt][j], sv[j][c]);
      *reinterpret_cast<half8_t*>(op + 8 * j) = o;
    }
  }
}

}  // namespace triteia_hip
