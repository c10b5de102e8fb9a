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
#include <type_traits>

#include "sparse24_gemm.hip.h"

namespace triteia_hip {

constexpr int kWideTokens = 64;
constexpr int kWideStages = 4;        // activation tiles in flight (LDS ring)

// TOK: token rows of a tile (64, or 32 for the narrow tiles of a routing plan and for uniform groups in launches
// that do not fill the chip).  PLAN_ALL: the kernel stands in for the narrow kernel on a routing plan: it takes the
// plan's narrow tiles, or its narrow-only list.  DEPTH: steps of weights in flight per wavefront.
// KS = 2: eight wavefronts; wavefronts 4..7 take the second half of the K steps of the same four column blocks (an
// activation ring of their own) and hand their sums to wavefronts 0..3 through LDS at the end: half as long a chain
// of steps per wavefront, for launches of at most one workgroup per CU.
template <int DEPTH, int TOK = kWideTokens, bool PLAN_ALL = false, int KS = 1>
__global__ __launch_bounds__(256 * KS, KS == 1 ? 2 : 1) void sparse24_wide_kernel(const Sparse24Args p) {
  constexpr int NT = TOK / 16;
  __shared__ __attribute__((aligned(1024))) _Float16 xs[KS][kWideStages][TOK][128];
  __shared__ int s_rows[TOK];

  const int tid = threadIdx.x;
  const int wave = (tid >> 6) & 3;   // column block of the group
  const int kh = KS == 1 ? 0 : __builtin_amdgcn_readfirstlane(tid >> 8);   // half of K (KS = 2); wave-uniform
  const int lane = tid & 63;
  const int r = lane & 15;
  const int q = lane >> 4;

  // unit = (group, group of 4 column blocks); column-block groups are padded to a multiple of
  // 8 per group and renumbered so that each XCD (own L2) owns a contiguous run of them for
  // every token tile of a delta.  Where cgs % 8 leaves XCDs short of work, the host asks for one of two other orders
  // (workgroup u runs on XCD u % 8): xcd_swizzle = 3 puts the idle slots of the padding to work, xcd_swizzle = 2
  // numbers the units without padding (unit u = column group u % cgs of group u / cgs: balanced, but a delta's token
  // tiles then read a column group through different L2s).
  const int col_blocks = p.m >> 7;
  const int cgs = (col_blocks + 3) >> 2;
  const int cg_pad = (cgs + 7) & ~7;
  const int unit = blockIdx.x;
  int grp = unit / cg_pad;
  int i = unit - grp * cg_pad;
  const int rows_of_tiles = p.n_groups * (PLAN_ALL && TOK == 32 && p.tile_halves ? 2 : 1);   // the host's bound
  int cg;
  if (p.xcd_swizzle == 2) {
    grp = unit / cgs;
    cg = unit - grp * cgs;
    if (grp >= rows_of_tiles) return;
  } else if (p.xcd_swizzle == 3) {
    // padded rows whose idle slots work: R rows of slots serve R + 1 tiles, the last of them through the rows' idle
    // slots (R * pad >= cgs), so that the XCDs that hold the padding get as many units as the others while all but one
    // tile in R + 1 keep each column group on one XCD
    const int pad = cg_pad - cgs;   // > 0: the host asks for this order only then
    const int R = (cgs + pad - 1) / pad;
    const int sg = grp / R, row = grp - sg * R;
    const int c = (i & 7) * (cg_pad >> 3) + (i >> 3);
    if (c < cgs) {
      grp = sg * (R + 1) + row;
      cg = c;
    } else {
      grp = sg * (R + 1) + R;
      cg = row * pad + (c - cgs);
    }
    if (grp >= rows_of_tiles) return;
  } else if (p.xcd_swizzle == 4) {
    // an XCD takes a block of xcd_cgs column groups x a block of tiles: the bytes that its L2 has to fetch are the
    // block's weights plus the block's activations, least when the two are of about the same size
    // (a plan's list: the blocks of tiles are cut from the list's real length, which the device knows, so that the
    // live tiles spread over all the XCDs; the launch is sized for the host's bound on it)
    int rows_live = rows_of_tiles;
    if (p.tiles && p.n_groups_dev) {
      const bool alt = PLAN_ALL && p.tiles_alt && (long)p.n_groups_dev[4] * p.wide_gate < p.wide_min_units;
      int live = p.n_groups_dev[alt ? 5 : 0];
      if (!PLAN_ALL && p.tiles_all64 && plan_takes_all64(p)) live = p.plan_header[p.all64_index];   // (the list chosen below)
      rows_live = min(rows_of_tiles, live * (PLAN_ALL && TOK == 32 && p.tile_halves ? 2 : 1));
    }
    const int n_cgb = cg_pad / p.xcd_cgs;             // blocks of column groups (a divisor of 8)
    const int tbs = 8 / n_cgb;                         // blocks of tiles
    const int tpb = (rows_live + tbs - 1) / tbs;       // tiles per block
    const int xcd = unit & 7, slot = unit >> 3;
    cg = (xcd % n_cgb) * p.xcd_cgs + slot % p.xcd_cgs;
    const int tslot = slot / p.xcd_cgs;
    grp = (xcd / n_cgb) * tpb + tslot;
    if (tslot >= tpb || grp >= rows_live) return;
  } else {
    cg = p.xcd_swizzle ? (i & 7) * (cg_pad >> 3) + (i >> 3) : i;
  }
  if (cg >= cgs) return;
  int half = 0;
  if (PLAN_ALL && TOK == 32 && p.tile_halves) {
    half = grp & 1;
    grp >>= 1;
  }
  int delta, start, count;
  bool alt_list = false;
  int all64_live = -1;
  if (p.tiles) {
    const int4* list = p.tiles;
    if (!PLAN_ALL && p.tiles_all64) {
      // the plan's wide tiles, or one list of 64-token tiles over all its tokens (the choice comes first: the launch
      // is sized for the longer of the two lists, and a workgroup past the end of the chosen one reads no tile)
      if (plan_takes_all64(p)) {
        list = p.tiles_all64;
        all64_live = p.plan_header[p.all64_index];
      }
      if (grp >= (all64_live >= 0 ? all64_live : p.n_groups_dev[0])) return;
    }
    int4 d = list[grp];
    if (PLAN_ALL && p.tiles_alt) {
      // this build stands in for the narrow kernel on a plan's narrow tiles: like that kernel it takes
      // the narrow-only list when the plan's wide tiles do not fill the chip (both candidates are requested together)
      const int4 d_alt = p.tiles_alt[grp];
      if ((long)p.n_groups_dev[4] * p.wide_gate < p.wide_min_units) {
        d = d_alt;
        alt_list = true;
      }
    }
    delta = d.x;
    start = d.y + 32 * half;
    count = d.z - 32 * half;
  } else {
    const int chunks = (p.uniform_count + TOK - 1) / TOK;
    const int gi = grp / chunks, tc = grp - gi * chunks;
    delta = gi * p.delta_step;
    start = gi * p.uniform_stride + p.uniform_first + tc * TOK;
    count = min(TOK, p.uniform_count - tc * TOK);
  }
  const int n_groups = all64_live >= 0 ? all64_live : (p.n_groups_dev ? p.n_groups_dev[alt_list ? 5 : 0] : p.n_groups);
  if (!PLAN_ALL && all64_live < 0 && p.wide_min_units && (long)n_groups * p.wide_gate < p.wide_min_units) return;   // the narrow kernel has taken these tokens
  if (grp >= n_groups) return;
  if (delta < 0 || delta >= p.n_deltas || count <= 0) return;
  const int cnt = min(count, TOK);

  const int cb = 4 * cg + wave;
  const bool active = cb < col_blocks;          // the last group of a matrix may be partial
  const int cbc = active ? cb : col_blocks - 1;  // idle waves still run the barriers

  const int k_rows = p.k >> 5;
  const int all_steps = (k_rows + 3) >> 2;
  // this wavefront's steps: [step0, step0 + n_steps); every wavefront runs `loop_steps` rounds of the loop (barriers)
  const int loop_steps = (all_steps + KS - 1) / KS;
  const int step0 = kh == 0 ? 0 : loop_steps;
  const int n_steps = kh == 0 ? loop_steps : all_steps - loop_steps;
  const long qrow = p.m >> 1;
  const long mrow = p.m >> 2;
  // operand addresses = a base that is the same for the whole wave (scalar registers) + a 32-bit byte
  // offset per lane: two registers per lane fewer for each pointer that stays alive across the K loop
  const uint4_t* qw_delta = p.qweight + (long)delta * p.qweight_stride;
  const uint4_t* mt_delta = p.meta + (long)delta * p.meta_stride;
  const uint32_t woff = (uint32_t)((q * qrow + (long)cbc * 64 + 4 * r) * 16);
  const uint32_t moff = (uint32_t)((q * mrow + (long)cbc * 32 + (r >> 3) * 16 + (r & 7)) * 16);

  // token rows of the tile (slots past the end repeat the last row; their outputs are dropped)
  if (tid < TOK) {
    const int slot = min(tid, cnt - 1);
    s_rows[tid] = p.perm ? p.perm[start + slot] : start + slot;
  }
  __syncthreads();

  // cooperative activation fetch.  One direct-to-LDS instruction of a wavefront writes 64
  // consecutive 16-byte chunks = 4 token rows; instruction ii of wave w covers rows
  // 16 ii + 4 w + lane/16.  Lane l fills chunk position l % 16 of its row, which holds the
  // row's chunk (l % 16) ^ (row % 16).
  uint32_t xoff[NT];   // byte offsets into x (the launcher sends activations of 4 GiB and more elsewhere)
#pragma unroll
  for (int ii = 0; ii < NT; ii++) {
    const int row = 16 * ii + 4 * wave + (lane >> 4);
    const int chunk = (lane & 15) ^ (row & 15);
    xoff[ii] = (uint32_t)(((long)s_rows[row] * p.x_stride + chunk * 8) * 2);
  }
  // Direct-to-LDS loads and the waits for them are written as inline assembly: the compiler
  // counts a direct-to-LDS load as an LDS write, which the release fence of every barrier and
  // the first LDS read behind it must complete, i.e. it drains every outstanding request (the
  // weights requested a moment ago included) once per K step.  The LDS address of a request is
  // M0 + 16 * lane; M0 is an input operand of the statement, so the compiler writes it and knows it is live.
  const uint32_t lds_x_wave = (uint32_t)(uintptr_t)&xs[kh][0][4 * wave][0];
  // (`nta`: the 16-token tiles that hold tokens; the others are neither fetched nor multiplied)
  auto issue_x = [&](int st, int nta) {   // (nta: a constant where this is called)
    const int stc = min(step0 + min(st, n_steps - 1), all_steps - 1);   // past the end: refetch a valid tile (never read)
    const int stage = st & (kWideStages - 1);
#pragma unroll
    for (int ii = 0; ii < NT; ii++) {
      if (ii >= nta) break;
      const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_x_wave + (stage * TOK + 16 * ii) * 256);
      const _Float16* base = p.x + stc * 128;
      asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(xoff[ii]), "s"(base), "{m0}"(dst) : "memory");
    }
  };

  struct WFrag {
    uint4_t wq[4];
    uint4_t mt[2];
  };
  auto load_w = [&](WFrag& f, int st) {
    const long tr0 = (st < n_steps ? step0 + st : 0) << 2;   // past the end: any valid rows (never used); k % 128 == 0, so
    const char* wb = reinterpret_cast<const char*>(qw_delta + tr0 * qrow);   // rows tr0 .. tr0 + 3 always exist
    const char* mb = reinterpret_cast<const char*>(mt_delta + tr0 * mrow);
#pragma unroll
    for (int a = 0; a < 4; a++) f.wq[a] = *reinterpret_cast<const uint4_t*>(wb + woff + 16 * a);
    f.mt[0] = *reinterpret_cast<const uint4_t*>(mb + moff);
    f.mt[1] = *reinterpret_cast<const uint4_t*>(mb + moff + 128);
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
    const _Float16* row = &xs[kh][stage][nt * 16 + r][0];
    typedef uint32_t uint8_t_v __attribute__((ext_vector_type(8)));
    const uint4_t lo = *reinterpret_cast<const uint4_t*>(row + ((c ^ r) << 3));
    const uint4_t hi = *reinterpret_cast<const uint4_t*>(row + (((c + 8) ^ r) << 3));
    const uint8_t_v bb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(half16_t, bb);
  };
  // `mid(g)`: called behind the MFMAs of group g = 2 u + b2 (requests that a step issues between its groups)
  auto compute_step = [&](const WFrag& f, int stage, auto nta, auto&& mid) {
    constexpr int NTA = decltype(nta)::value;
    // Per k-half u and per half of the 8 columns: dequantise 4 weight fragments, then run them
    // against the four 16-token B fragments.  B fragments are read one ahead of the MFMAs that
    // use them, so that the LDS latency hides behind 4 MFMAs instead of stalling in front of them.
    half16_t b_nxt;
    if (DEPTH < 2) b_nxt = read_b(stage, 0, 0);
#pragma unroll
    for (int u = 0; u < 2; u++) {
#pragma unroll
      for (int b2 = 0; b2 < 2; b2++) {
        if (DEPTH >= 2) __builtin_amdgcn_sched_barrier(0);   // (keeps the scheduler from pulling later fragments ahead: registers)
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
        for (int nt = 0; nt < NTA; nt++) {
          half16_t b;
          if (DEPTH < 2) {
            b = b_nxt;
            if (nt + 1 < NTA) b_nxt = read_b(stage, nt + 1, u);
            else if (b2 == 0) b_nxt = read_b(stage, 0, u);
            else if (u == 0) b_nxt = read_b(stage, 0, 1);
          } else {
            b = read_b(stage, nt, u);   // (two steps of weights in flight leave no registers for a fragment ahead)
          }
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
        mid(2 * u + b2);
      }
    }
  };
  auto no_mid = [](int) {};

  // pipeline: weights DEPTH steps ahead in registers (requests the compiler tracks), activation tiles
  // 3 steps ahead in the LDS ring (requests it does not see).  Requests complete in order, and every
  // step issues its activation tile first and its weights last, so the compiler's wait for the weights of
  // step st ("all but the newest 6 (DEPTH - 1) requests") is exact for DEPTH = 2: the weights of step
  // st + 1 stay in flight across the step.  The hand-written wait at the top of a step says that this
  // wave's part of tile st has landed: behind it in the queue are at most the tiles st+1, st+2 (one
  // request per occupied 16-token tile each) and DEPTH sets of weights (6 each); the barrier then makes all four waves' parts visible and
  // also says that tile st-1 has been read by everyone, so its stage can be refilled.
  // EARLY (the 32-token builds with two steps of weights in flight): a third slot in the ring of weights, so that the
  // requests of a step need not wait for its arithmetic to release a slot.  They are issued between the step's groups
  // of MFMAs -- the activation tile of step st + 3 behind the first group (its stage was read in step st - 1, and every
  // wavefront is past this step's barrier), the weights of step st + 2 behind the second (into the slot of step st - 1)
  // -- instead of in one burst behind the last MFMA, where the wavefront stands at the address unit's queue with
  // nothing else to issue.  The order of the requests (tile, then weights, once per step) and with it both counts
  // above are unchanged, and so are the sums.  Measured: plans of 16 deltas of 4096 x 4096 with 768 / 1024 tokens
  // 48.7 -> 45.6, 60.8 -> 58.6 us, 8 deltas of 8192 x 8192 with 512 tokens 98.5 -> 95.0 us; uniform launches the same
  // within 3 %.
  constexpr bool EARLY = DEPTH == 2 && TOK == 32;
  constexpr int RING = EARLY ? 3 : DEPTH;
  WFrag ring[RING];
  auto k_loop = [&](auto nta) {
    constexpr int NTA = decltype(nta)::value;
    issue_x(0, NTA);
    issue_x(1, NTA);
    issue_x(2, NTA);
#pragma unroll
    for (int j = 0; j < DEPTH; j++) load_w(ring[j], j);
    constexpr int TURN = EARLY ? 12 : (DEPTH > 4 ? DEPTH : 4);   // whole ring turns of both rings (DEPTH divides 4; EARLY: 3 and 4 slots)
    // Whole turns run without a condition around the arithmetic (a wavefront past the last column block works on
    // the block before it and stores nothing): behind a skipped step the compiler has to assume that step's weights
    // still in flight and waits for everything before it requests the next ones.
    // (with K halved inside the workgroup the second half can be a step shorter: both halves run the same
    // number of barriers, so the unconditional part covers the steps that both have)
    const int whole = (KS == 1 ? all_steps : all_steps - loop_steps) / TURN * TURN;
    for (int s0 = 0; s0 < whole; s0 += TURN) {
#pragma unroll
      for (int j = 0; j < TURN; j++) {
        const int st = s0 + j;
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * NTA + 6 * DEPTH) : "memory");
        lds_barrier();
        if constexpr (EARLY) {
          compute_step(ring[j % 3], j & (kWideStages - 1), nta, [&](int g) {
            if (g > 1) return;
            __builtin_amdgcn_sched_barrier(0);
            if (g == 0) issue_x(st + 3, NTA);
            else load_w(ring[(j + 2) % 3], st + 2);
            __builtin_amdgcn_sched_barrier(0);
          });
        } else {
          compute_step(ring[j % DEPTH], j & (kWideStages - 1), nta, no_mid);
          __builtin_amdgcn_sched_barrier(0);   // (requests stay behind the step's arithmetic, where its registers are free)
          issue_x(st + 3, NTA);
          load_w(ring[j % DEPTH], st + DEPTH);
        }
      }
    }
    for (int s0 = whole; s0 < loop_steps; s0 += TURN) {
#pragma unroll
      for (int j = 0; j < TURN; j++) {
        const int st = s0 + j;
        if (EARLY && st >= loop_steps) break;   // (a turn of 12 can be longer than what is left)
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * NTA + 6 * DEPTH) : "memory");
        lds_barrier();
        if (st < n_steps) compute_step(ring[j % RING], j & (kWideStages - 1), nta, no_mid);
        issue_x(st + 3, NTA);
        load_w(ring[(j + DEPTH) % RING], st + DEPTH);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive the block's LDS
  };
  // A plan's tiles are often far from full (a delta with a handful of tokens): a tile whose tokens fit the first half of
  // its 16-token tiles walks K in a copy of the loop that leaves the other half out (the matrix cores, not the weight
  // stream, bound a CU that holds three such workgroups).  The count is the same for the whole workgroup.
  if (PLAN_ALL && cnt <= TOK / 2)
    k_loop(std::integral_constant<int, NT / 2>{});
  else
    k_loop(std::integral_constant<int, NT>{});

  if (KS == 2) {
    // the second half's sums go to the first half through the memory of the activation rings (same size:
    // 2048 * TOK bytes), register by register with consecutive lanes side by side
    __syncthreads();   // every wavefront has read its last tile
    float* red = reinterpret_cast<float*>(&xs[0][0][0][0]) + wave * (32 * NT * 64) + lane;
    if (kh == 1) {
#pragma unroll
      for (int cc = 0; cc < 8; cc++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
          for (int j = 0; j < 4; j++) red[((cc * NT + nt) * 4 + j) * 64] = acc[cc][nt][j];
    }
    __syncthreads();
    if (kh == 1) return;
#pragma unroll
    for (int cc = 0; cc < 8; cc++)
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[cc][nt][j] += red[((cc * NT + nt) * 4 + j) * 64];
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
    // (when the sums are added to what is there: a token's four pieces are requested together, ahead of the arithmetic
    // -- one round trip per 16-token tile instead of one per 8 columns.  All tiles at once would be one round trip in
    // all, but holds 16 registers per tile, which the 64-token builds do not have.)
    constexpr bool TOGETHER = !(TOK == 64 && KS == 2);   // (that build is out of registers as it is)
    half8_t olds[4];
#pragma unroll
    for (int j = 0; j < 4; j++) olds[j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (TOGETHER && p.accumulate) {
#pragma unroll
      for (int j = 0; j < 4; j++) olds[j] = *reinterpret_cast<const half8_t*>(op + 8 * j);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      if (!TOGETHER && p.accumulate) olds[j] = *reinterpret_cast<const half8_t*>(op + 8 * j);
      half8_t o;
#pragma unroll
      for (int cc = 0; cc < 8; cc++) o[cc] = scaled_sum_f16(olds[j][cc], acc[cc][nt][j], sv[j][cc]);
      *reinterpret_cast<half8_t*>(op + 8 * j) = o;
    }
  }
}

}  // namespace triteia_hip
