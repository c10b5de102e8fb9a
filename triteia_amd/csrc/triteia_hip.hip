// extern "C" boundary of libtriteia_hip.so: argument checks, launch geometry,
// stream / device handling.  Kernels live in the headers next to this file.
#include "../../include/triteia_hip.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "lora.hip.h"
#include "lora_mfma.hip.h"
#include "route_plan.hip.h"
#include "sparse24_gemm.hip.h"
#include "sparse24_share.hip.h"
#include "sparse24_tile256.hip.h"
#include "sparse24_wide.hip.h"

namespace {

using namespace triteia_hip;

thread_local char g_err[512] = "";
constexpr int kMaxDevicesForAttr = 64;

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Makes `dev` current for the duration of a call and restores the previous device.
struct DeviceGuard {
  int prev = -1;
  bool ok = true;
  explicit DeviceGuard(int dev) {
    if (hipGetDevice(&prev) != hipSuccess) { ok = false; return; }
    if (dev >= 0 && dev != prev) ok = hipSetDevice(dev) == hipSuccess; else prev = -1;
  }
  ~DeviceGuard() { if (prev >= 0) (void)hipSetDevice(prev); }
};

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TRITEIA_HIP_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
  return TRITEIA_HIP_OK;
}

// Tuning knobs.  Each can be set through an environment variable of the same name in capitals with the
// prefix TRITEIA_HIP_ (for tests and measurements); the variables are read ONCE, at the first call into the
// library, and again only when triteia_hip_reload_env() is called: an ordinary call does no getenv.
// kUnset marks knobs whose default depends on the launch.
constexpr int kUnset = -0x7fffffff;
struct Knobs {
  int nt = 0, xcd_swizzle = 1, xcd_cgs = 0 /* 0: the rule, n > 0: blocks of n column groups, -1: never */, wide_order_min_idle = kUnset, pass_nt = 0;
  int wide = 1, wide_min_units = kUnset, wide_min_batch = 256, plan_wide_min_units = kUnset;
  int wide32_min_units = kUnset, wide32_max_units = kUnset, wide32_ksplit_max_units = kUnset, wide64_ksplit_max_units = kUnset;
  int mid = 1, mid64_max_k = 0x7fffffff, mid_min_column_groups = 16, mid_min_units = kUnset, mid_min_half_tokens = 7, mid_narrow = 1, mid_depth = 0, plan_big = 1, plan_all64 = 1, lora_mfma = 1;
  int eager = 1, fused_route = 1;
  int tile256 = 1, tile256_min_units = kUnset, tile256_max_units = kUnset, ksplit = 1, sub_shift = kUnset, share16 = 1, share16_max_blocks = kUnset;
};
Knobs g_knobs;
std::once_flag g_knobs_once;

void read_knobs() {
  Knobs k;
  struct { const char* name; int* dst; } table[] = {
      {"NT", &k.nt}, {"XCD_SWIZZLE", &k.xcd_swizzle}, {"XCD_CGS", &k.xcd_cgs}, {"WIDE_ORDER_MIN_IDLE", &k.wide_order_min_idle},
      {"PASS_NT", &k.pass_nt}, {"WIDE", &k.wide}, {"WIDE_MIN_UNITS", &k.wide_min_units},
      {"WIDE_MIN_BATCH", &k.wide_min_batch}, {"PLAN_WIDE_MIN_UNITS", &k.plan_wide_min_units},
      {"WIDE32_MIN_UNITS", &k.wide32_min_units}, {"WIDE32_MAX_UNITS", &k.wide32_max_units},
      {"WIDE32_KSPLIT_MAX_UNITS", &k.wide32_ksplit_max_units}, {"WIDE64_KSPLIT_MAX_UNITS", &k.wide64_ksplit_max_units},
      {"MID", &k.mid}, {"MID64_MAX_K", &k.mid64_max_k}, {"MID_MIN_COLUMN_GROUPS", &k.mid_min_column_groups},
      {"MID_MIN_UNITS", &k.mid_min_units}, {"MID_MIN_HALF_TOKENS", &k.mid_min_half_tokens}, {"MID_NARROW", &k.mid_narrow}, {"MID_DEPTH", &k.mid_depth}, {"PLAN_BIG", &k.plan_big}, {"PLAN_ALL64", &k.plan_all64}, {"LORA_MFMA", &k.lora_mfma}, {"EAGER", &k.eager}, {"FUSED_ROUTE", &k.fused_route},
      {"TILE256", &k.tile256}, {"TILE256_MIN_UNITS", &k.tile256_min_units}, {"TILE256_MAX_UNITS", &k.tile256_max_units},
      {"KSPLIT", &k.ksplit}, {"SUB_SHIFT", &k.sub_shift}, {"SHARE16", &k.share16}, {"SHARE16_MAX_BLOCKS", &k.share16_max_blocks},
  };
  char name[64];
  for (auto& e : table) {
    snprintf(name, sizeof(name), "TRITEIA_HIP_%s", e.name);
    const char* v = getenv(name);
    if (v && *v) *e.dst = atoi(v);
  }
  g_knobs = k;
}

const Knobs& knobs() {
  std::call_once(g_knobs_once, read_knobs);
  return g_knobs;
}

// value of a knob whose default depends on the launch
inline int knob_or(int v, long dflt) { return v == kUnset ? (int)dflt : v; }

// Scale groups along K that the launchers accept, in the reference's unit (compressed k, i.e. dense k / 2): -1, one scale
// per column, and 64 = 128 dense k = one K step of the kernels (marlin_nm.cu:68,102-111: group_blocks -1 or 4).
constexpr int kGroupsize = 64;
int check_gemm_shape(int prob_m, int prob_n, int prob_k, int groupsize, bool grouped_ok = false) {
  if (groupsize != -1 && !(grouped_ok && groupsize == kGroupsize))
    return fail(TRITEIA_HIP_ERR_KERN_SHAPE, grouped_ok ? "groupsize=%d: scales per column (groupsize=-1) or per column and 128 dense k (groupsize=64) are implemented"
                                                       : "groupsize=%d: only per-channel scales (groupsize=-1) are implemented by this entry point", groupsize);
  if (groupsize != -1 && prob_k % 128 != 0)
    return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "k=%d is not a whole number of scale groups of 128", prob_k);
  if (prob_m < 0 || prob_n < 0 || prob_k < 0 || prob_m % 128 != 0 || prob_k % 64 != 0)
    return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "problem (m=%d, n=%d, k=%d) needs m %% 128 == 0 and k %% 64 == 0", prob_m, prob_n, prob_k);
  return TRITEIA_HIP_OK;
}

// Token tile of the grouped kernel: 16 * NT rows share one pass over the weights.  Chosen from
// what the host knows (tokens, groups); the routing plan cuts groups into tiles of this size.
int pick_nt(long tokens, long groups) {
  const int forced = knobs().nt;
  if (forced == 1 || forced == 2 || forced == 4) return forced;
  if (groups < 1) groups = 1;
  if (tokens <= 16) return 1;
  // small batches spread thinly: groups well under 16 tokens (a rare larger one takes a second pass);
  // with more tokens some delta of a skewed batch is always hot and 32-token tiles win
  if (tokens <= 64 && tokens <= 4 * groups) return 1;
  if (tokens <= 24 * groups) return 2;   // typical group well under 32 tokens
  // few tiles in all (64-token tiles: one per 64 tokens and a last one per group): 32-token tiles make twice as
  // many workgroups of them (4 deltas of 4096 x 4096 with 1024 tokens: 55 -> 46 us; 16 deltas: 66 -> 61.5 us with 1024
  // tokens, 86.6 -> 82.1 with 2048; 32 deltas of 11008 x 4096 with 1024: 184 -> 156 us)
  if (tokens / 64 + groups <= 48) return 2;
  return 4;
}

// Uniform groups (matmul, bmm): tokens per group are known exactly.  A launch of few workgroups is
// bound by latency, not by the weights it re-reads from cache: the widest tile that still leaves
// one workgroup per CU, else 16-token tiles with the tokens split across workgroups (measured on
// one 4096 x 4096 matrix: 64 tokens 24.4 -> 12.2 us, 128 tokens 24.2 -> 12.4 us, 256 tokens 24.4 -> 19.1 us).
int pick_nt_uniform(long tokens, long groups, long col_blocks) {
  const int forced = knobs().nt;
  if (forced == 1 || forced == 2 || forced == 4) return forced;
  for (int nt = 4; nt >= 2; nt /= 2) {
    if (tokens <= 8 * nt) continue;   // a narrower tile holds them all
    if (groups * col_blocks * ((tokens + 16 * nt - 1) / (16 * nt)) >= 256) return nt;
  }
  return 1;
}

template <int NT, int KW, int DEPTH, bool EAGER = false>
void launch_one(const Sparse24Args& a, dim3 grid, hipStream_t st) {
  hipLaunchKernelGGL((sparse24_grouped_kernel<NT, KW, DEPTH, EAGER>), grid, dim3(64 * KW), 0, st, a);
}

// `nt`: token tile class; `tsplit`: workgroups along y sharing one group's tokens (run-table form
// only: plan tiles never exceed one pass, uniform groups are cut into chunks by the kernel).
// Decode-size uniform launches of at most 128 column blocks in all (a single matrix of up to 16384 columns): shares of
// 16, 32 or 64 columns -- the narrowest that leaves at most one workgroup per CU -- on the kernel whose MFMA rows are
// a share's columns and whose wavefronts request all their steps at once (sparse24_share.hip.h); same sums in the same
// order as the eight-wavefront streaming kernel that took them before.  Returns the 16-column tiles per share, 0 = no.
constexpr long kShare16MaxBlocks = 128;
static int share16_tiles(long n_groups, int m, int tokens_per_group) {
  if (tokens_per_group > 16 || !knobs().share16 || knobs().sub_shift != kUnset || knobs().nt != 0)
    return 0;
  const long blocks = n_groups * (m / 128);
  if (blocks > knob_or(knobs().share16_max_blocks, kShare16MaxBlocks)) return 0;
  return blocks <= 32 ? 1 : blocks <= 64 ? 2 : 4;
}
int launch_sparse24(Sparse24Args a, int nt, long tsplit, hipStream_t st, int zsplit = 1) {
  if (a.n_groups <= 0 || a.m == 0 || a.k == 0) return TRITEIA_HIP_OK;
  if (tsplit < 1) tsplit = 1;
  if (tsplit > 65535) tsplit = 65535;
  // Uniform launches of few workgroups give each workgroup a share of a column block (128 >> sub_shift columns)
  // instead of a whole one, halving the share while the launch stays within one workgroup per CU: more CUs take part,
  // and the sums do not change (see Sparse24Args::sub_shift).  The gain is small, because every share still reads all
  // the activations: 16 tokens on 4096 x 4096 (32 column blocks) 11.4 -> 10.1 us in shares of 16 columns, on 4096 x 11008
  // (86) 12.4 -> 11.1 us in shares of 64 (in shares of 32, 344 workgroups: 18.2 us); one token on each of 8 matrices of
  // 4096 x 4096 (256 column blocks already) 13.2 -> 16.5 us in shares of 64, which the rule does not do.
  const bool uniform = !a.raw_indices && !a.tiles && !a.g_delta;
  {
    int s = 0;
    const long blocks = (long)a.n_groups * (a.m / 128) * tsplit * zsplit;
    if (uniform && nt == 1 && zsplit == 1)
      while (s < 3 && (blocks << (s + 1)) <= 256) s++;
    a.sub_shift = knob_or(knobs().sub_shift, s);
    if (a.sub_shift < 0 || a.sub_shift > 3) a.sub_shift = 0;
  }
  const long cb_pad = (((long)(a.m / 128) << a.sub_shift) + 7) / 8 * 8;   // column shares padded to the 8 XCDs
  // A launch of at most one workgroup per CU runs 8 wavefronts per workgroup with one step in
  // flight each: more waves, not more bytes per wave, is what raises the rate there (measured:
  // cfg1 14.3 -> 13.6 us, 16-token matmul 12.3 -> 11.4 us; 16 wavefronts and two steps per wave are slower).
  // Only for uniform groups (matmul, bmm): the split of K among the wavefronts fixes the order of the
  // fp32 sums, and a routed token must have the same bits whatever the size of its batch.
  const bool one_per_cu = uniform && zsplit == 1 && (nt == 1 || nt == 2) && (long)a.n_groups * cb_pad * tsplit <= 256;
  const int kw = one_per_cu ? 8 : 4;
  // register budget: the 16-token kernel runs 3 workgroups per CU with one step in flight (2 with
  // two), the 32-token kernel 2 per CU with two, the 64-token kernel 1 per CU with one.  Fused
  // routing in its eager form keeps one step in flight (measured: a second step requested ahead of
  // the routing makes the 16-delta case slower, 23.1 against 22.0 us).
  const bool eager = a.raw_indices && a.raw_static;
  // A launch of at most one live workgroup per CU is bound by the latency of each wave's chain of requests rather
  // than by bandwidth: a second step in flight pays there, while from two workgroups on some CUs on it costs time
  // (16 deltas of 4096 x 4096: 8 tokens on 5 deltas, 160 workgroups, 14.6 -> 13.4 us with two steps; 16 tokens on
  // 11 deltas, 352 workgroups, 18.3 -> 20.3 us; 8192 x 8192: 8 tokens on 6 deltas, 384 workgroups, 31.2 -> 34.0 us;
  // 11008 x 4096 with 16 tokens on 8 deltas, 256 workgroups, 32.3 -> 29.8 us).  A batch routed inside the kernel
  // launches a workgroup for every delta that could be in use; the ones that find tokens are estimated as under a
  // uniform routing, deltas x (1 - (1 - 1 / deltas) ^ tokens).
  double live_groups = a.n_groups;
  if (a.raw_indices && !a.raw_static && a.n_deltas > 0) {
    double none = 1.0;
    for (int t = 0; t < a.raw_count && none > 1e-9; t++) none *= 1.0 - 1.0 / a.n_deltas;
    live_groups = a.n_deltas * (1.0 - none);
    if (live_groups > a.n_groups) live_groups = a.n_groups;
  }
  const bool small = live_groups * cb_pad * tsplit * zsplit <= 256.5;
  const int depth = eager || kw == 8 ? 1 : (nt == 2 || (nt == 1 && small) ? 2 : 1);
  // About 512 workgroups run at a time.  When those belong to four or more deltas (narrow matrices),
  // the deltas start their walks over K spread evenly around the ring of steps; wide matrices are
  // streamed one or two at a time anyway and walk from step 0.
  // (counted in whole column blocks, whatever the share a workgroup takes: the start of a delta's walk fixes the order
  // of its fp32 sums, which must not depend on the share)
  {
    const long side_by_side = 512 / (((long)(a.m / 128) + 7) / 8 * 8);
    const int n_steps = (a.k / 32 + 3) / 4;
    const long spread = side_by_side >= 4 ? n_steps / (side_by_side < 16 ? side_by_side : 16) : 0;
    a.rot_spread = (int)spread;
  }
  if (const int tiles = uniform && nt == 1 && tsplit == 1 && zsplit == 1 && !a.ksplit_steps ? share16_tiles(a.n_groups, a.m, a.uniform_count) : 0) {
    const long sh_pad = ((long)(a.m / (16 * tiles)) + 7) / 8 * 8;
    const dim3 grid((unsigned)(a.n_groups * sh_pad));
    if (tiles == 1) hipLaunchKernelGGL((sparse24_share16_kernel<8, 4, 1>), grid, dim3(512), 0, st, a);
    else if (tiles == 2) hipLaunchKernelGGL((sparse24_share16_kernel<8, 4, 2>), grid, dim3(512), 0, st, a);
    else hipLaunchKernelGGL((sparse24_share16_kernel<8, 4, 4>), grid, dim3(512), 0, st, a);
    return check_launch("sparse24_share16_kernel");
  }
  // The same for a routed batch of at most 16 tokens that is routed inside the kernel (one group per delta in use, at
  // most min(tokens, deltas) of them): on four wavefronts, like every routed launch.
  if (const int tiles = a.raw_indices && !a.raw_static && nt == 1 && tsplit == 1 && zsplit == 1 ? share16_tiles(a.n_groups, a.m, a.raw_count) : 0) {
    const long sh_pad = ((long)(a.m / (16 * tiles)) + 7) / 8 * 8;
    const dim3 grid((unsigned)(a.n_groups * sh_pad));
    if (tiles == 1) hipLaunchKernelGGL((sparse24_share16_kernel<4, 8, 1, true>), grid, dim3(256), 0, st, a);
    else if (tiles == 2) hipLaunchKernelGGL((sparse24_share16_kernel<4, 4, 2, true>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((sparse24_share16_kernel<4, 4, 4, true>), grid, dim3(256), 0, st, a);
    return check_launch("sparse24_share16_kernel (routed)");
  }
  const long units = (long)a.n_groups * cb_pad;
  if (units > 0x7fffffffL) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "too many work units (%ld)", units);
  // Launches whose groups all have work -- uniform groups, and a batch routed in the kernel with a group per delta --
  // give whole groups to an XCD (Sparse24Args::xcd_swizzle = 5) instead of a run of column blocks of every group:
  // each XCD's L2 then fetches the activations and indices of its own groups only (the counters showed them fetched once
  // per XCD: 5.6 % on top of the algorithmic bytes of the 64-token batch over 16 deltas of 4096 x 4096) and streams whole
  // matrices.  Measured: that batch 22.9 -> 22.3 us (four pairs of runs, each ahead); 8 matrices of 4096 x 4096 with a token
  // each 13.9 -> 13.7 us; 12 deltas with 64 tokens 20.5 -> 20.2 us.  The sums do not depend on which workgroup takes which unit.
  // Only for launches of a single round (at most the 512 workgroups that run together): there every XCD's share is
  // resident at once whatever its size, while a longer launch needs the even split of every group over the XCDs
  // (8 matrices of 4096 x 11008 with a token each, 704 workgroups: 30.4 -> 31.1 us; 16 deltas of 4096 x 11008 with 128
  // tokens 63.0 -> 64.8 us).
  if (a.xcd_swizzle == 1 && a.n_groups >= 8 && units * tsplit * zsplit <= 512 && (uniform || (a.raw_indices && a.raw_static))) a.xcd_swizzle = 5;
  else if (a.xcd_swizzle == 5) a.xcd_swizzle = 1;
  const dim3 grid((unsigned)units, (unsigned)tsplit, (unsigned)zsplit);
#define TRY(NT_, KW_, D_) if (nt == NT_ && kw == KW_ && depth == D_) { launch_one<NT_, KW_, D_>(a, grid, st); return check_launch("sparse24_grouped_kernel"); }
#define TRY_EAGER(NT_, KW_, D_) if (nt == NT_ && kw == KW_ && depth == D_) { launch_one<NT_, KW_, D_, true>(a, grid, st); return check_launch("sparse24_grouped_kernel"); }
  if (a.raw_indices && a.raw_static) {
    TRY_EAGER(1, 4, 1) TRY_EAGER(2, 4, 1) TRY_EAGER(4, 4, 1)
  }
  TRY(1, 4, 1) TRY(1, 4, 2) TRY(1, 8, 1)
  TRY(2, 4, 2) TRY(2, 8, 1)
  TRY(4, 4, 1)
#undef TRY
#undef TRY_EAGER
  return fail(TRITEIA_HIP_ERR_KERN_SHAPE, "no kernel variant for NT=%d KW=%d DEPTH=%d", nt, kw, depth);
}

// One matrix whose scales come per column and 128-k step (Sparse24Args::scale_groups): the streaming kernel's GS build,
// whole column blocks, four wavefronts, one step in flight, the tokens in passes of 16 or 32 spread over blockIdx.y
// (a compatibility path: the reference's own module and converter never produce such scales).
int launch_grouped_scales(Sparse24Args a, int tokens, hipStream_t st) {
  a.n_groups = 1;
  a.uniform_count = tokens;
  a.uniform_stride = tokens;
  a.delta_step = 0;
  const int nt = tokens <= 16 ? 1 : 2;
  long tsplit = (tokens + 16 * nt - 1) / (16 * nt);
  if (tsplit > 65535) tsplit = 65535;
  const long cb_pad = ((long)(a.m / 128) + 7) / 8 * 8;
  const dim3 grid((unsigned)cb_pad, (unsigned)tsplit, 1);
  if (nt == 1) hipLaunchKernelGGL((sparse24_grouped_kernel<1, 4, 1, false, true>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((sparse24_grouped_kernel<2, 4, 1, false, true>), grid, dim3(256), 0, st, a);
  return check_launch("sparse24_grouped_kernel (grouped scales)");
}

void fill_weights(Sparse24Args& a, const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m,
                  int prob_k, int n_deltas) {
  a = Sparse24Args{};   // every field the caller does not set is zero / null
  a.x = static_cast<const _Float16*>(A);
  a.x_stride = prob_k;
  a.qweight = static_cast<const uint4_t*>(B);
  a.qweight_stride = (long)(prob_k / 32) * (prob_m / 2);
  a.meta = static_cast<const uint4_t*>(meta);
  a.meta_stride = (long)(prob_k / 32) * (prob_m / 4);
  a.scales = static_cast<const _Float16*>(s);
  a.scales_stride = prob_m;
  a.out = static_cast<_Float16*>(C);
  a.out_stride = prob_m;
  a.m = prob_m;
  a.k = prob_k;
  a.n_deltas = n_deltas;
  a.xcd_swizzle = knobs().xcd_swizzle;
}


// 32-token launches of at most one workgroup per CU run with eight wavefronts per workgroup (K split in two inside the
// workgroup): 20-27 % faster from 160 to 256 units, slower beyond (two rounds of workgroups that fill a CU each).
constexpr long kWide32KSplitMaxUnits = 256;
// The same for 64-token tiles (256 registers, 128 KiB of LDS): 9-20 % faster than the 32-token build with four wavefronts
// at 257-448 of its units and than the 64-token build with four wavefronts up to 256 units (one workgroup per CU).
constexpr long kWide64KSplitMaxUnits = 256;
// Wide (64-token x 512-column) tiles: groups from a plan's wide list or uniform groups.  `tok` = 32: uniform groups
// in 32-token tiles on the 32-token build with two steps of weights in flight (launches that do not fill the chip).
// Order of the wide kernel's units over the XCDs (workgroup u runs on XCD u % 8).  Column groups padded to a multiple of
// 8 keep a column group of a delta on one XCD for all its token tiles, but with 28 groups (m = 14336) the eighth XCD gets
// none of a tile's 32 slots, with 10 (m = 5120) three get none and with 4 (m = 2048) four.  From three idle slots per
// tile on, the idle slots are put to work (order 3 of sparse24_wide_kernel: R rows of slots serve R + 1 tiles).
// Measured, padded -> order 3: plans over deltas of 4096 x 14336, Zipf(1.2)-routed, 1024 tokens over 4 / 8 / 32 deltas
// 118.5 -> 86.0, 120.7 -> 90.9, 204.8 -> 189.0 us; 5120 x 13824 with 1024 tokens over 8 deltas 145.4 -> 106.8 us; 5120 x 5120
// with 1024 tokens over 32 deltas 124.6 -> 94.4 us, one matrix with 4096 tokens 178.2 -> 138.6 us; 8192 x 2048, one matrix
// with 2048 / 4096 tokens 95.9 -> 68.4, 141.1 -> 102.2 us; 4096 x 6144 with 1024 tokens over 8 / 32 deltas 67.3 -> 56.8,
// 103.3 -> 83.4 us.  Numbering the units without padding (order 2) balances as well but lets every tile of a delta read
// a column group through another L2: the same on most of these, 4-7 % behind on 5120 x 13824 and 5120 x 5120 (4096 tokens
// on one matrix 333 against 310 us, 143 against 138 us).  With two idle slots in 24 (m = 11008) neither order gains (cfg3's
// delta kernel 86.3 -> 87.6-92.7 us with order 3, 85.4 -> 89.2 us with order 2; one matrix with 4096 tokens 218 -> 215 us): its
// launches fit the three workgroups per CU either way, and the busiest CU decides.
constexpr int kWideOrderMinIdleSlots = 3;
static int wide_unit_order(int m) {
  const int cgs = (m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
  if (knobs().xcd_swizzle == 3 && cg_pad == cgs) return 1;   // (no padding to put to work)
  // (order 3 divides by the number of padding slots: never without any, whatever the knob says)
  return knobs().xcd_swizzle == 1 && cg_pad > cgs && cg_pad - cgs >= knob_or(knobs().wide_order_min_idle, kWideOrderMinIdleSlots) ? 3 : knobs().xcd_swizzle;
}
// Workgroups of a wide-kernel launch over `rows` tiles (or halves of tiles) in the given order of units.
static long wide_grid_units(long rows, int m, int order) {
  const long cgs = (m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
  if (order == 2) return rows * cgs;
  if (order == 3) {
    const long pad = cg_pad - cgs, R = (cgs + pad - 1) / pad;
    return (rows / (R + 1) * R + rows % (R + 1)) * cg_pad;
  }
  return rows * cg_pad;
}
// Workgroups of a wide-kernel launch over `rows` tiles in blocks of `xc` column groups x blocks of tiles per XCD
// (order 4); -1 where 8 XCDs cannot be cut into blocks of that many column groups on this layer.
static long wide_block_grid_units(long rows, int m, long xc) {
  const long cgs = (m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
  if (xc <= 0 || cg_pad % xc != 0 || cg_pad / xc > 8 || 8 % (cg_pad / xc) != 0) return -1;
  const long tbs = 8 / (cg_pad / xc);
  return 8 * xc * ((rows + tbs - 1) / tbs);
}
// Workgroups of a wide-kernel launch over a plan's list of at most `rows` tiles (or halves of tiles) of `tok` tokens,
// and the order of its units.  Where the layer's order is the plain one (1: every XCD takes a run of column groups for
// every tile, so that every XCD's L2 fetches every tile's activations), blocks of column groups x blocks of tiles per
// XCD (order 4; the blocks of tiles are cut on the device from the list's real length) make the L2s fetch fewer bytes
// once the batch has tokens enough: while the `window` workgroups that an XCD holds at a time walk K, its L2 fetches the
// weights of their distinct (delta, column group) pairs and the activations of their distinct tiles; with units numbered
// column group first and about `tiles_per_delta` adjacent tiles per delta, blocks of c column groups fetch
// c x ceil(window / c / tiles_per_delta) x (a column group's weights) + window / c x (a tile's activations).
// Measured (order 1 -> blocks): 16 deltas of 4096 x 4096 with 1024 / 2048 tokens 56.4 -> 54.5, 76.5 -> 74.8 us (blocks of
// 4 or 8); 32 deltas of 4096 x 11008 with 1024 / 4096 tokens 154-158 -> 146, 290-300 -> 284 us (blocks of 12; of 24:
// 165 and 296); 64 deltas of 8192 x 28672 with 256 / 1024 tokens: the plain order stays ahead (644 against 662 us in
// blocks of 14).  The knob xcd_cgs forces a block size (> 0) or the plain order (-1).
static unsigned plan_wide_grid(Sparse24Args& b, long rows, int m, int tok, int prob_n, int n_deltas, int window) {
  const long cgs = (m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
  const long forced = knobs().xcd_cgs;
  long best = cg_pad / 8;
  if (b.xcd_swizzle == 1 && forced >= 0) {
    const double groups = n_deltas < prob_n ? n_deltas : prob_n;
    const double tpd = prob_n / (tok * groups) > 1.0 ? prob_n / (tok * groups) : 1.0;          // tiles per delta
    const double per_tile = prob_n / groups < tok ? prob_n / groups : tok;                      // tokens per tile
    const double w_cg = 512.0 * b.k * 0.375, x_tile = per_tile * b.k * 2.0;
    auto fetched = [&](long xc) {
      const double tiles = (double)window / xc > 1.0 ? (double)window / xc : 1.0;
      double deltas = tiles / tpd > 1.0 ? tiles / tpd : 1.0;
      if (deltas > groups) deltas = groups;
      return xc * deltas * w_cg + tiles * x_tile;
    };
    double best_bytes = fetched(best);
    for (long xc = 1; xc <= cg_pad; xc++) {
      if (cg_pad % xc != 0 || cg_pad / xc > 8 || 8 % (cg_pad / xc) != 0) continue;
      if (forced > 0) {
        if (xc == forced) best = xc;
        continue;
      }
      // (tiles of a plan are ragged: a block of tiles is shared by two XCDs at least, so that the XCDs' loads stay alike;
      // blocks of all 24 column groups of 4096 x 11008 measured 4 % behind the plain order)
      if (cg_pad / xc >= 2 && fetched(xc) < 0.95 * best_bytes) { best = xc; best_bytes = fetched(xc); }
    }
  }
  if (best != cg_pad / 8 || (forced > 0 && best == forced && b.xcd_swizzle == 1)) {
    b.xcd_swizzle = 4;
    b.xcd_cgs = (int)best;
    return (unsigned)wide_block_grid_units(rows, m, best);
  }
  return (unsigned)wide_grid_units(rows, m, b.xcd_swizzle);
}
// (`plan_tokens`, `plan_deltas`: the batch behind a plan's list of tiles, for the order of its units; 0 for uniform groups)
int launch_wide(const Sparse24Args& a, hipStream_t st, int tok = kWideTokens, int plan_tokens = 0, int plan_deltas = 0) {
  if (a.n_groups <= 0 || a.m == 0 || a.k == 0) return TRITEIA_HIP_OK;
  const long cgs = (a.m / 128 + 3) / 4;
  const long cg_pad = (cgs + 7) / 8 * 8;
  const long chunks = a.tiles ? 1 : (a.uniform_count + tok - 1) / tok;
  const long units = (long)a.n_groups * chunks * cg_pad;   // (the rules below count padded units)
  if (units > 0x7fffffffL) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "too many work units (%ld)", units);
  Sparse24Args b = a;
  if (!b.tiles) b.n_groups = (int)(a.n_groups * chunks);
  b.xcd_swizzle = wide_unit_order(a.m);
  unsigned grid = a.tiles && plan_tokens > 0 ? plan_wide_grid(b, (long)a.n_groups * chunks, a.m, tok, plan_tokens, plan_deltas, 64)
                                             : (unsigned)wide_grid_units((long)a.n_groups * chunks, a.m, b.xcd_swizzle);
  // Uniform launches: an XCD takes a block of column groups x a block of token tiles (order 4) where that makes its
  // L2 fetch fewer bytes than a run of column groups for every tile (order 1).  While the workgroups that an XCD holds at
  // a time (32 CUs x 1 or 2) walk K, its L2 fetches the packed weights of their distinct column groups and the
  // activations of their distinct tiles once each: with units numbered column group first, a window of W units over
  // blocks of c column groups fetches c x (weights of a column group) + W / c x (activations of a tile), least near
  // c = sqrt(W x tile / column group).  Measured (order 1 -> the rule): 4096 x 4096 with 640 / 1024 / 1536 / 2048 tokens
  // 28.3 -> 27.1, 32.1 -> 30.6, 43.8 -> 41.6, 50.5 -> 46.8 us; 8192 x 8192 with 1000 tokens 81.2 -> 79.7 us; 11008 x 4096 with
  // 1280 tokens 92.5 -> 88.6 us; 4096 x 11008 and 8192 x 28672 the same either way (blocks of 14 column groups on the
  // latter, which a count over the whole launch instead of the window would pick, measured 1.7 % slower).
  // The sums do not depend on which workgroup takes which unit.
  const bool eight_waves = !a.tiles && ((tok == 32 && units <= knob_or(knobs().wide32_ksplit_max_units, kWide32KSplitMaxUnits)) ||
                                        (tok != 32 && units <= knob_or(knobs().wide64_ksplit_max_units, kWide64KSplitMaxUnits)));
  if (!a.tiles && b.xcd_swizzle == 1 && knobs().xcd_cgs >= 0) {
    const long rows = (long)a.n_groups * chunks;
    const double w_cg = 512.0 * a.k * 0.375, x_tile = (double)tok * a.k * 2.0;
    const long window = 32 * (eight_waves ? 1 : 2);                       // workgroups an XCD holds at a time
    auto fetched = [&](long xc) {
      const long tbs = 8 / (cg_pad / xc);
      long slots = xc * ((rows + tbs - 1) / tbs);
      if (slots > window) slots = window;
      return (double)xc * w_cg + (double)((slots + xc - 1) / xc) * x_tile;
    };
    long best = cg_pad / 8;
    double best_bytes = fetched(best);
    for (long xc = 1; xc <= cg_pad; xc++) {
      if (cg_pad % xc != 0 || cg_pad / xc > 8 || 8 % (cg_pad / xc) != 0) continue;
      if (knobs().xcd_cgs > 0) {                                           // (forced, for measurements)
        if (xc == knobs().xcd_cgs) best = xc;
        continue;
      }
      if (fetched(xc) < 0.95 * best_bytes) { best = xc; best_bytes = fetched(xc); }
    }
    if (best != cg_pad / 8 || knobs().xcd_cgs > 0) {
      b.xcd_swizzle = 4;
      b.xcd_cgs = (int)best;
      grid = (unsigned)wide_block_grid_units(rows, a.m, best);
    }
  }
  if (tok == 32 && units <= knob_or(knobs().wide32_ksplit_max_units, kWide32KSplitMaxUnits))
    hipLaunchKernelGGL((sparse24_wide_kernel<2, 32, false, 2>), dim3(grid), dim3(512), 0, st, b);
  else if (tok == 32)
    hipLaunchKernelGGL((sparse24_wide_kernel<2, 32, false>), dim3(grid), dim3(256), 0, st, b);
  else if (units <= knob_or(knobs().wide64_ksplit_max_units, kWide64KSplitMaxUnits) &&
           !a.tiles)   // (a plan's launch is sized by an upper bound on its tiles; at 190-230 real units it measured the same either way)
    hipLaunchKernelGGL((sparse24_wide_kernel<1, kWideTokens, false, 2>), dim3(grid), dim3(512), 0, st, b);
  else
    hipLaunchKernelGGL((sparse24_wide_kernel<1>), dim3(grid), dim3(256), 0, st, b);
  return check_launch("sparse24_wide_kernel");
}

// 256-token x 256-column tiles on workgroups of eight wavefronts (153 KB of dynamic LDS, one workgroup per CU):
// uniform groups only.
bool g_tile256_ready[kMaxDevicesForAttr] = {};
std::mutex g_tile256_mutex;
int launch_tile256(const Sparse24Args& a, hipStream_t st) {
  if (a.n_groups <= 0 || a.m == 0 || a.k == 0 || a.uniform_count <= 0) return TRITEIA_HIP_OK;
  const long ncp = (a.m / 128 + 1) / 2;
  const long tiles = (long)a.n_groups * ((a.uniform_count + kT256Tokens - 1) / kT256Tokens);
  const long units = t256_grid(tiles, ncp);
  if (units > 0x7fffffffL) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "too many work units (%ld)", units);
  {
    // more than 64 KB of LDS has to be granted once per device
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevicesForAttr)
      return fail(TRITEIA_HIP_ERR_RUNTIME, "sparse24_tile256_kernel: no current device");
    std::lock_guard<std::mutex> lock(g_tile256_mutex);
    if (!g_tile256_ready[dev]) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&sparse24_tile256_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kT256LdsBytes) != hipSuccess)
        return fail(TRITEIA_HIP_ERR_RUNTIME, "sparse24_tile256_kernel: cannot reserve %d bytes of LDS", kT256LdsBytes);
      g_tile256_ready[dev] = true;
    }
  }
  hipLaunchKernelGGL(sparse24_tile256_kernel, dim3((unsigned)units), dim3(512), kT256LdsBytes, st, a);
  return check_launch("sparse24_tile256_kernel");
}
// (token tile, column pair) units for which a uniform launch takes this kernel: launches of one round of workgroups
// (one per CU) that fill most of the chip.  Measured against 64-token tiles: 4096 tokens on 4096 x 4096 (256 units) 89.1
// against 95.8 us (82.8 against 83.4 on another box), on 8192 x 8192 (512 units) 290 against 294 us; 4096 x 11008
// (688 units) 228 against 227 us; 8192 x 28672 (1792 units) 994 against 950 us; 2048 tokens on 4096 x 11008 (344 units:
// a second round of a third of the chip) 139 against 116 us; on 4096 x 4096 (128 units: half the CUs idle) 72 against 55 us.
constexpr long kTile256MinUnits = 192, kTile256MaxUnits = 256;

// The wide kernel pays off when there are enough tiles to occupy the GPU; below that the narrow
// kernel's smaller units win.  Knob `wide` = 0 disables it; `wide_min_units` moves the threshold.
bool wide_enabled() { return knobs().wide != 0; }
constexpr long kWideMinUnits = 160;   // 4096 x 4096: 1024 tokens (128 tiles) 54.9 us wide against 46.5 us narrow, 1536 tokens (192) 60.8 against 71.1
constexpr long kWide32MinUnits = 160, kWide32MaxUnits = 448;   // (32-token tile, 512-column group) units: see launch_uniform

// ---- uniform groups (matmul, bmm): `tokens` rows per group.  Which kernel takes which rows is decided by
// decide_uniform (a pure function of the shapes and the knobs, also behind triteia_hip_uniform_kernel) and carried
// out by launch_uniform.
enum UniformKind { kUniNarrow = 0, kUniWide32 = 32, kUniWide64 = 64, kUniTile256 = 256, kUniSplitK = 1000 };
struct UniformSegment { int kind, first, count, ksplit; };
struct UniformPlan { UniformSegment seg[3]; int n = 0; };

// K split across workgroups for launches that leave most of the chip idle on a long K: (groups x column blocks x
// token passes) well below the number of CUs and at least 64 steps of K.  Every workgroup takes 1 / ksplit of the K
// steps and writes fp32 partial sums to a scratch buffer of the caller's; a second, tiny launch adds them in a fixed
// order.  Returns the number of splits (1: none).  Measured (16 tokens, unsplit -> split in 4): 8192 x 8192 18.5 -> 14.2 us,
// 11008 x 4096 22.5 -> 14.5 us.  A K of 4096 is too short to pay for the second launch (4096 x 4096: 11.4 -> 11.0 us in 4,
// 12.4 in 8; with 64 tokens 11.0 -> 12.3; 4096 x 11008 12.5 -> 12.7), and so is a launch that has a workgroup per CU
// already (8 matrices of 4096 x 4096 with one token each: 13.4 -> 16.5 us).
constexpr long kSplitKMaxUnits = 64;    // launches of at most this many unsplit workgroups are split ...
constexpr int kSplitKMinSteps = 64;     // ... if K has at least this many steps of 128 ...
constexpr int kSplitKStepsPerSplit = 16;   // ... into shares of about this many steps
static int share16_tiles(long n_groups, int m, int tokens_per_group);
int pick_ksplit(long tokens, long n_groups, int m, int k) {
  if (!knobs().ksplit || tokens <= 0) return 1;
  const long cb_pad = (m / 128 + 7) / 8 * 8;
  const int nt = tokens <= 16 ? 1 : pick_nt_uniform(tokens, n_groups, m / 128);
  const long units = n_groups * cb_pad * ((tokens + 16 * nt - 1) / (16 * nt));
  const int n_steps = (k / 32 + 3) / 4;
  if (knobs().ksplit > 1) return knobs().ksplit <= n_steps ? knobs().ksplit : n_steps;   // forced (tests, measurements)
  if (units > kSplitKMaxUnits || n_steps < kSplitKMinSteps) return 1;
  // A handful of tokens: the column-share kernel (one launch, all of a wavefront's requests at once) is ahead of the
  // split and its second launch as long as the activations that every share reads again are few (1 / 8 tokens on
  // 8192 x 8192 11.4 / 12.7 against 13.4 / 13.9 us, on 11008 x 4096 10.4 / 13.5 against 13.3 / 14.0; 2 / 4 tokens on
  // 14336 x 4096 13.3 / 15.2 against 13.9 / 14.2; 16 tokens on 11008 x 4096 16.8 against 14.6 us).
  if (share16_tiles(n_groups, m, (int)tokens) && (tokens * (long)k <= 49152 || (k <= 11008 && tokens <= 8))) return 1;
  long ks = n_steps / kSplitKStepsPerSplit;
  if (ks > 512 / units) ks = 512 / units;
  if (ks > 16) ks = 16;
  return ks < 2 ? 1 : (int)ks;
}

UniformPlan decide_uniform(int tokens, int stride, int n_groups, int m, int k, long x_stride, bool have_scratch) {
  UniformPlan up;
  auto add = [&](int kind, int first, int count, int ksplit = 1) { up.seg[up.n++] = UniformSegment{kind, first, count, ksplit}; };
  const long cgs = (m / 128 + 3) / 4;
  int done = 0;
  bool ks64 = false;   // the whole launch goes to 64-token tiles on workgroups of eight wavefronts
  // (the wide kernels address activations with 32-bit byte offsets)
  const bool x_below_4g = ((long)(n_groups - 1) * stride + tokens) * x_stride * 2 < (1L << 32);
  // Launches of a few dozen workgroups: K split across workgroups.
  if (have_scratch) {
    const int ks = pick_ksplit(tokens, n_groups, m, k);
    if (ks > 1) {
      add(kUniSplitK, 0, tokens, ks);
      return up;
    }
  }
  // Groups of hundreds of tokens: 256-token x 256-column tiles whose wavefronts share the dequantised weights.
  // On layers of fewer than 8 column groups of 512 (m < 3584) only: elsewhere the 64-token kernel, since its units go to
  // the XCDs in blocks of column groups x token tiles, is as fast or faster inside this window (4096 x 4096 with 3072 /
  // 3584 / 4096 tokens 80.5 -> 66.8, 80.7 -> 72.4, 81.7 -> 78.2 us; 4096 x 8192 with 2048 tokens 81.5 -> 78.8; 8192 x 4096
  // and 11008 x 4096 with 4096 tokens 147.3 -> 145, 193 -> 192 us), while 4096 x 2048 with 8192 tokens, whose four column
  // groups leave half of a padded tile's slots idle, keeps it (81 against 85 us).  The knob tile256 = 2 lifts the limit.
  if (knobs().tile256 && (cgs < 8 || knobs().tile256 > 1) && wide_enabled() && x_below_4g) {
    const long ncp = (m / 128 + 1) / 2;
    const long min_units = knob_or(knobs().tile256_min_units, kTile256MinUnits);
    int t = tokens / kT256Tokens * kT256Tokens;
    if (tokens - t >= kT256Tokens / 2 || min_units <= 1) t = tokens;     // a rest of half a tile and more is a tile
    const long units = (long)n_groups * ((t + kT256Tokens - 1) / kT256Tokens) * ncp;
    if (t > 0 && units >= min_units && units <= knob_or(knobs().tile256_max_units, kTile256MaxUnits)) {
      add(kUniTile256, 0, t);
      done = t;
    }
  }
  // A launch of at most two 32-token workgroups per CU, but of more than the narrow kernel fills well, is bound by
  // the latency of each workgroup's chain of steps, not by the matrix cores: there the 32-token build of the wide
  // kernel with two steps of weights in flight per wavefront beats both the narrow kernel and 64-token tiles.
  // Measured (narrow or 64-token -> this): 4096 x 4096 with 640 / 1024 / 1536 / 2048 tokens 45.7 -> 37.2, 46.5 -> 38.2,
  // 54.5 -> 49.7, 60.8 -> 55.6 us; 4096 x 11008 with 384 / 512 tokens 66 -> 46.7, 54.7 -> 48.5 us; 8192 x 8192 with
  // 384 / 768 tokens 76.5 -> 66.5, 94.7 -> 86.9 us; 8192 x 28672 with 128 / 256 tokens 79 -> 69.3, 99.5 -> 95.5 us.
  // At 160 units: 4096 x 4096 with 640 tokens 45 -> 36.7, 8192 x 8192 with 320 tokens 76.5 -> 66.2, 11008 x 4096 with 640
  // tokens 98.8 -> 89.5 us.  Outside the window it loses: 8192 x 8192 with 288 tokens (144 units) 61.7 -> 65.7 us,
  // 4096 x 11008 with 160 tokens (110 units) 28.9 -> 37 us, with 768 tokens (528 units) 64 -> 76 us; inside it one
  // case measured slower: 8192 x 28672 with 96 tokens (168 units) 64 -> 69 us.
  {
    // (a last tile of any size counts: in a launch of one round its workgroups cost nothing, a separate launch of
    // the narrow kernel for them streams the weights once more)
    const long units32 = (long)n_groups * ((tokens + 31) / 32) * cgs;
    // past the launches that the 32-token build runs with eight wavefronts, 64-token tiles with eight wavefronts
    // are ahead while they make one workgroup per CU at most (4096 x 4096 with 1280 / 1536 tokens 49.7 -> 44.2,
    // 50.8 -> 46.0 us; 4096 x 11008 with 384 / 640 tokens 47.2 -> 43.0, 51.4 -> 46.0 us; 8192 x 8192 with 768 tokens 88.7 ->
    // 72.5 us; 8192 x 28672 with 192 tokens 89.4 -> 73.0 us)
    ks64 = done == 0 && wide_enabled() && k % 128 == 0 && x_below_4g && tokens >= kWideTokens &&
           units32 > knob_or(knobs().wide32_ksplit_max_units, kWide32KSplitMaxUnits) &&
           (long)n_groups * ((tokens + kWideTokens - 1) / kWideTokens) * ((cgs + 7) / 8 * 8) <=
               knob_or(knobs().wide64_ksplit_max_units, kWide64KSplitMaxUnits);
    if (done == 0 && !ks64 && wide_enabled() && k % 128 == 0 && x_below_4g && tokens >= 32 &&
        units32 >= knob_or(knobs().wide32_min_units, kWide32MinUnits) &&
        units32 <= knob_or(knobs().wide32_max_units, kWide32MaxUnits)) {
      add(kUniWide32, 0, tokens);
      done = tokens;
    }
  }
  int rest = tokens - done;
  if (rest > 0 && wide_enabled() && k % 128 == 0 && x_below_4g &&
      (done > 0 ? rest >= kPlanWideMinRest
                : ks64 || (long)n_groups * (rest / kWideTokens) * cgs >= knob_or(knobs().wide_min_units, kWideMinUnits))) {
    int t = rest / kWideTokens * kWideTokens;
    // A rest above half a tile becomes a tile of its own; a smaller one too while the launch stays within one
    // round of workgroups (two per CU), where its workgroups cost nothing and a launch of the narrow kernel for them
    // would stream the weights once more (288 tokens on 8192 x 28672: 130.6 -> 111.5 us; 2056 on 4096 x 4096 69.3 ->
    // 67.4 us).  Past one round the extra tile starts a round of its own (4104 tokens on 4096 x 4096: 88 -> 111 us).
    const bool one_round = (long)n_groups * (rest / kWideTokens + 1) * cgs <= 512;
    if (rest - t >= (one_round ? 1 : kPlanWideMinRest)) t = rest;
    add(kUniWide64, done, t);
    done += t;
  }
  rest = tokens - done;
  if (rest > 0) add(kUniNarrow, done, rest);
  return up;
}

// bytes of fp32 partial sums that a K split of this launch writes (0: the launch is not split)
size_t uniform_scratch_bytes(int tokens, int n_groups, int m, int k) {
  const int ks = pick_ksplit(tokens, n_groups, m, k);
  return ks > 1 ? sizeof(float) * (size_t)ks * (size_t)n_groups * (size_t)tokens * (size_t)m : 0;
}

int launch_uniform(Sparse24Args a, int tokens, int stride, int delta_step, int n_groups, hipStream_t st,
                   void* scratch = nullptr, size_t scratch_bytes = 0) {
  a.n_groups = n_groups;
  a.uniform_stride = stride;
  a.delta_step = delta_step;
  const bool have_scratch = scratch && stride == tokens && reinterpret_cast<uintptr_t>(scratch) % 16 == 0 &&
                            scratch_bytes >= uniform_scratch_bytes(tokens, n_groups, a.m, a.k) &&
                            uniform_scratch_bytes(tokens, n_groups, a.m, a.k) > 0;
  const UniformPlan up = decide_uniform(tokens, stride, n_groups, a.m, a.k, a.x_stride, have_scratch);
  for (int i = 0; i < up.n; i++) {
    const UniformSegment& sg = up.seg[i];
    a.uniform_first = sg.first;
    a.uniform_count = sg.count;
    int e = TRITEIA_HIP_OK;
    if (sg.kind == kUniTile256) e = launch_tile256(a, st);
    else if (sg.kind == kUniWide32) e = launch_wide(a, st, 32);
    else if (sg.kind == kUniWide64) e = launch_wide(a, st);
    else if (sg.kind == kUniSplitK) {
      const int n_steps = (a.k / 32 + 3) / 4;
      Sparse24Args b = a;
      b.partial = static_cast<float*>(scratch);
      b.partial_rows = (long)n_groups * tokens;
      b.ksplit_steps = (n_steps + sg.ksplit - 1) / sg.ksplit;
      const int splits = (n_steps + b.ksplit_steps - 1) / b.ksplit_steps;   // (every split has a step)
      const int nt = sg.count <= 16 ? 1 : pick_nt_uniform(sg.count, n_groups, a.m / 128);
      e = launch_sparse24(b, nt, (sg.count + 16 * nt - 1) / (16 * nt), st, splits);
      if (e) return e;
      const long chunks = b.partial_rows * (a.m / 8);
      hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, b.partial, splits,
                         b.partial_rows, a.m, a.scales, a.scales_stride, tokens, delta_step, a.out, a.out_stride);
      e = check_launch("splitk_reduce_kernel");
    } else {
      const int nt = pick_nt_uniform(sg.count, n_groups, a.m / 128);
      e = launch_sparse24(a, nt, (sg.count + 16 * nt - 1) / (16 * nt), st);
    }
    if (e) return e;
  }
  return TRITEIA_HIP_OK;
}

// Routing-plan scratch of triteia_hip_sbmm_2_4_routed_static: owned by the library, one copy per GPU (each
// device that loads this code object holds its own instance of the array at its own address).  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels get the per-device address it returns.
constexpr size_t kStaticPlanBytes = 256 * 1024;
__device__ __align__(256) unsigned char g_static_plan[kStaticPlanBytes];

constexpr int kMaxDevices = 64;
void* g_static_plan_addr[kMaxDevices] = {};
std::mutex g_static_plan_mutex;

// Address of the current device's instance of g_static_plan (looked up once per device, with that device current).
int static_plan_address(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(TRITEIA_HIP_ERR_RUNTIME, "sbmm_2_4_routed_static: no current device");
  std::lock_guard<std::mutex> lock(g_static_plan_mutex);
  if (!g_static_plan_addr[dev]) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_plan));
    if (e != hipSuccess || !ptr)
      return fail(TRITEIA_HIP_ERR_RUNTIME, "sbmm_2_4_routed_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_static_plan_addr[dev] = ptr;
  }
  *out = g_static_plan_addr[dev];
  return TRITEIA_HIP_OK;
}

}  // namespace

extern "C" {

int triteia_hip_version(void) { return 1001; }

void triteia_hip_reload_env(void) {
  knobs();        // (so that a first call later on does not overwrite what is read here)
  read_knobs();
}

const char* triteia_hip_last_error(void) { return g_err; }

int triteia_hip_mul_2_4(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m, int prob_n,
                        int prob_k, void* workspace, int groupsize, int dev, void* stream, int thread_k, int thread_m,
                        int sms, int max_par) {
  (void)workspace; (void)thread_k; (void)thread_m; (void)sms; (void)max_par;
  if (int e = check_gemm_shape(prob_m, prob_n, prob_k, groupsize, true)) return e;
  if (prob_m == 0 || prob_n == 0 || prob_k == 0) return TRITEIA_HIP_OK;
  if (!A || !B || !meta || !C || !s) return fail(TRITEIA_HIP_ERR_ARGUMENT, "mul_2_4: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  Sparse24Args a;
  fill_weights(a, A, B, meta, C, s, prob_m, prob_k, 1);
  if (groupsize != -1) {
    a.scale_groups = prob_k / 128;
    a.scales_stride = (long)a.scale_groups * prob_m;
    return launch_grouped_scales(a, prob_n, static_cast<hipStream_t>(stream));
  }
  return launch_uniform(a, prob_n, prob_n, 0, 1, static_cast<hipStream_t>(stream));
}

int triteia_hip_bmm_2_4_tokens_scratch(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m,
                                       int batch, int tokens, int prob_k, void* scratch, size_t scratch_bytes, int dev,
                                       void* stream) {
  if (int e = check_gemm_shape(prob_m, batch, prob_k, -1)) return e;
  if (tokens < 0) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "bmm_2_4: tokens=%d", tokens);
  if (prob_m == 0 || batch == 0 || prob_k == 0 || tokens == 0) return TRITEIA_HIP_OK;
  if (!A || !B || !meta || !C || !s) return fail(TRITEIA_HIP_ERR_ARGUMENT, "bmm_2_4: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  Sparse24Args a;
  fill_weights(a, A, B, meta, C, s, prob_m, prob_k, batch);
  return launch_uniform(a, tokens, tokens, 1, batch, static_cast<hipStream_t>(stream), scratch, scratch_bytes);
}

int triteia_hip_bmm_2_4_tokens(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m,
                               int batch, int tokens, int prob_k, int dev, void* stream) {
  return triteia_hip_bmm_2_4_tokens_scratch(A, B, meta, C, s, prob_m, batch, tokens, prob_k, nullptr, 0, dev, stream);
}

size_t triteia_hip_bmm_scratch_bytes(int prob_m, int batch, int tokens, int prob_k) {
  if (prob_m <= 0 || batch <= 0 || tokens <= 0 || prob_k <= 0 || prob_m % 128 != 0 || prob_k % 64 != 0) return 0;
  return uniform_scratch_bytes(tokens, batch, prob_m, prob_k);
}

int triteia_hip_uniform_kernel(int prob_m, int batch, int tokens, int prob_k, int with_scratch) {
  if (prob_m <= 0 || batch <= 0 || tokens <= 0 || prob_k <= 0 || prob_m % 128 != 0 || prob_k % 64 != 0) return -1;
  const bool sc = with_scratch && uniform_scratch_bytes(tokens, batch, prob_m, prob_k) > 0;
  const UniformPlan up = decide_uniform(tokens, tokens, batch, prob_m, prob_k, prob_k, sc);
  if (up.n == 0) return -1;
  // the segment that takes the most rows
  int best = 0;
  for (int i = 1; i < up.n; i++) if (up.seg[i].count > up.seg[best].count) best = i;
  const UniformSegment& sg = up.seg[best];
  if (sg.kind == kUniSplitK) return kUniSplitK + sg.ksplit;
  if (sg.kind == kUniNarrow) return share16_tiles(batch, prob_m, sg.count) ? 16 : 0;
  // 32- and 64-token tiles: + 1 when the launch runs on workgroups of eight wavefronts (halves of K)
  const long cgs = (prob_m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
  if (sg.kind == kUniWide32)
    return 32 + ((long)batch * ((sg.count + 31) / 32) * cg_pad <= knob_or(knobs().wide32_ksplit_max_units, kWide32KSplitMaxUnits) ? 1 : 0);
  if (sg.kind == kUniWide64)
    return 64 + ((long)batch * ((sg.count + 63) / 64) * cg_pad <= knob_or(knobs().wide64_ksplit_max_units, kWide64KSplitMaxUnits) ? 1 : 0);
  return sg.kind;
}

int triteia_hip_bmm_2_4(const void* A, const void* B, const void* meta, void* C, const void* s, int prob_m, int prob_n,
                        int prob_k, void* workspace, int groupsize, int dev, void* stream, int thread_k, int thread_m,
                        int sms, int max_par) {
  (void)workspace; (void)thread_k; (void)thread_m; (void)sms; (void)max_par;
  if (int e = check_gemm_shape(prob_m, prob_n, prob_k, groupsize)) return e;
  return triteia_hip_bmm_2_4_tokens(A, B, meta, C, s, prob_m, prob_n, 1, prob_k, dev, stream);
}

int triteia_hip_sbmm_2_4_bounded(const void* A, const void* B, const void* meta, void* C, const void* s,
                                 const void* indices, const void* starts, const void* counts, int prob_m, int prob_n,
                                 int prob_k, int prob_r, void* workspace, int groupsize, int dev, void* stream,
                                 int thread_k, int thread_m, int sms, int max_par, int n_deltas) {
  (void)workspace; (void)thread_k; (void)thread_m; (void)sms; (void)max_par;
  if (int e = check_gemm_shape(prob_m, prob_n, prob_k, groupsize)) return e;
  if (prob_r < 0 || n_deltas < 0) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "sbmm_2_4: runs=%d deltas=%d", prob_r, n_deltas);
  if (prob_m == 0 || prob_n == 0 || prob_k == 0 || prob_r == 0) return TRITEIA_HIP_OK;
  if (!A || !B || !meta || !C || !s || !indices || !starts || !counts)
    return fail(TRITEIA_HIP_ERR_ARGUMENT, "sbmm_2_4: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  Sparse24Args a;
  fill_weights(a, A, B, meta, C, s, prob_m, prob_k, n_deltas);
  a.g_delta = static_cast<const int*>(indices);
  a.g_start = static_cast<const int*>(starts);
  a.g_count = static_cast<const int*>(counts);
  a.n_groups = prob_r;
  // run lengths live on the device: size the tile and the token split for a few times the average run
  const int nt = pick_nt(prob_n, prob_r);
  long tsplit = (4L * prob_n / prob_r + 16 * nt - 1) / (16 * nt);
  if (tsplit > 16) tsplit = 16;
  return launch_sparse24(a, nt, tsplit, static_cast<hipStream_t>(stream));
}

int triteia_hip_sbmm_2_4(const void* A, const void* B, const void* meta, void* C, const void* s, const void* indices,
                         const void* starts, const void* counts, int prob_m, int prob_n, int prob_k, int prob_r,
                         void* workspace, int groupsize, int dev, void* stream, int thread_k, int thread_m, int sms,
                         int max_par) {
  // the reference's argument list carries no number of matrices: every non-negative index is taken as valid
  return triteia_hip_sbmm_2_4_bounded(A, B, meta, C, s, indices, starts, counts, prob_m, prob_n, prob_k, prob_r, workspace,
                                      groupsize, dev, stream, thread_k, thread_m, sms, max_par, 0x7fffffff);
}

size_t triteia_hip_sbmm_routed_workspace_bytes(int prob_n, int n_deltas) {
  if (prob_n < 0 || n_deltas < 0) return 0;
  return sizeof(int) * (size_t)plan_layout(prob_n, n_deltas).total;
}

int triteia_hip_plan_tile_tokens(int prob_n, int n_deltas) {
  const int groups = prob_n < n_deltas ? prob_n : n_deltas;
  int nt = pick_nt(prob_n, groups);
  // A plan for 33 .. 64 tokens over more than 16 deltas: under a skewed routing the hot delta has more than 16 tokens,
  // and a second 16-token tile streams its weights again (64 tokens, Zipf(1.2) over 32 deltas: 11008 x 4096 70.5 us in
  // 16-token tiles, 65.6 in 32-token tiles, 64.0 in 64-token tiles; 4096 x 11008 59.5 / 58.9 / 70.8 us).
  if (nt == 1 && prob_n > 32 && groups > 16 && knobs().nt == 0) nt = 2;
  return 16 * nt;
}

// A plan carries wide (64-token) tiles, next to a narrow-only cut of the same tokens, for batches
// with at least 8 tokens per delta on average (the plan is independent of the layer shape, so the
// rule only looks at the batch).  Which of the two cuts a layer uses is decided on the device:
// the wide kernel takes its tiles only if they fill the chip (wide tiles x column groups of the
// layer >= kPlanWideMinUnits); otherwise re-reading a hot delta's weights from cache in narrow
// tiles is cheaper than a second, poorly filled launch, and the wide launch returns at once.
// (measured between the two: launches of 152-176 wide units are 16-23 % faster on the wide kernel, 4 deltas of 4096 x 11008
// with 512 tokens 73 -> 61 us, 2 of 8192 x 8192 with 640 tokens 118 -> 99 us; launches of 128 are 12-20 % slower there)
constexpr int kPlanWideMinUnits = 150;
// A plan's 32-token tiles on a wide layer go to the 32-token build of the wide kernel (four column blocks of a
// workgroup share each activation tile through LDS, every wavefront walks all of K) instead of the K-split narrow
// kernel, whose column-block workgroups each fetch the tile's activations again: 5-10 % faster once there are
// about 450 (tile, 512-column group) units (cfg3 at 128 / 256 / 512 tokens 66.6 -> 62.7, 97 -> 88, 133 -> 126.5 us;
// 8 deltas of 8192 x 28672 with 96 tokens 142 -> 128.5 us), slower below (16 deltas of 4096 x 4096 with 256 tokens
// 24.9 -> 42.4 us).  The host only has the upper bound on the tiles; 600 on that bound separates the measured cases.
constexpr int kMidMinUnits = 480;
constexpr int kMidNarrowMinUnits = 280, kMidNarrowMinUnits64 = 150, kMidNarrowMinTokens = 768, kMidNarrowMaxTokens = 2048;
// A plan launch of at most two workgroups per CU (in 32-token tiles x 512-column groups, on the plan's upper bound of
// tiles) runs on the 32-token build with two steps of weights in flight per wavefront, a 64-token plan tile as two
// halves: with so few wavefronts per SIMD one step in flight leaves the memory latency of every step in the open.
// Measured with evenly routed batches of 256 .. 2048 tokens over 4 .. 32 deltas (against one step in flight / against
// what the rules chose before): 16 deltas of 4096 x 4096 with 768 / 1024 / 1536 tokens 43.5 / 43.9 -> 39.3, 47.5 / 47.8 ->
// 42.3, 57.3 / 59.4 -> 55.0 us; 8 of 8192 x 8192 with 512 tokens 83.2 / 93.5 -> 74.6; 4 of 4096 x 11008 with 512 tokens
// 52.8 / 60.7 -> 50.2; 32 of 11008 x 4096 with 1024 tokens 126.8 / 130.0 -> 117.1 us; with randomly routed batches the
// gain is 4-10 % (16 deltas of 4096 x 4096 with 768 / 1024 tokens 49.6 -> 45.0, 57.0 -> 54.7 us).  Past two workgroups
// per CU the third workgroup of the one-deep build is worth more (16 deltas of 4096 x 4096 with 2048 randomly routed
// tokens, 640 units on the bound: 76.2 -> 84.8 us; 4 / 8 of 4096 x 11008 with 768 tokens 66.5 -> 77.4, 73.6 -> 83.6 us), so
// the bound itself must fit; below 240 units the K-split narrow kernel is faster (16 deltas of 4096 x 4096 with 320 / 384
// randomly routed tokens, 208 / 224 units: 29.0 against 34.5, 31.4 against 34.6 us), and so it is with few tokens per tile
// (256 tokens, Zipf(1.2) over 32 deltas of 11008 x 4096, 6.4 per tile on the bound: 89.6 against 102.6 us).
// The lower end was 288 before the requests of this build moved in between its groups of MFMAs: its time is now flat
// in the tokens up to a launch of one round (34 us on k = 4096, 57 on 8192, 74 on 11008), while the narrow kernel pays
// a second round of workgroups from about 240 units on.  Randomly routed, narrow kernel -> this build: 16 deltas of
// 4096 x 4096 with 448 / 512 tokens 37.9 -> 34.9, 42.0 -> 38.6 us, 8 with 704 45.0 -> 37.2, 20 with 384 38.5 -> 34.9; 4 of
// 4096 x 11008 with 192 / 224 36.0 -> 33.2, 42.6 -> 33.3, 2 with 288 46.5 -> 32.5; 16 of 11008 x 4096 with 448 / 512 84 -> 74,
// 90 -> 73.6; 8 / 4 of 8192 x 8192 with 288 / 352 / 416 62 -> 57.5, 68 -> 56.6, 69 -> 57.3; 2 of 8192 x 28672 with 96 65.5 -> 58.6 us.
// It loses where the bound is far above the real tiles: 2 of 4096 x 11008 with 256 tokens a third of them unrouted
// 31.0 -> 32.6, 8 of 8192 x 8192 with 224 54.0 -> 57.8, one 8192 x 28672 with 128 tokens half of them unrouted 50.0 -> 55.8 us.
constexpr long kMidDeepMinUnits = 240, kMidDeepMaxUnits = 512, kMidDeepMinTokensPerTile = 12;
static long mid_units32(int prob_n, int n_deltas, int prob_m, int tile) {
  const long cgs = (prob_m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
  return (long)plan_max_tiles(prob_n, n_deltas, tile) * (tile == 64 ? 2 : 1) * cg_pad;
}
static bool mid_deep(int prob_n, int n_deltas, int prob_m, int tile) {
  const int forced = knobs().mid_depth;
  if (forced == 1 || forced == 2) return forced == 2;
  return mid_units32(prob_n, n_deltas, prob_m, tile) <= kMidDeepMaxUnits;
}
static bool mid_tiles(int prob_n, int n_deltas, int prob_m, int prob_k) {
  const int tile = triteia_hip_plan_tile_tokens(prob_n, n_deltas);
  // (64-token plans as well, on the 64-token build: cfg3 at 1024 / 2048 tokens 196 -> 170 / 250 -> 214 us; 8192 x 28672
  // with 2048 / 4096 tokens over 64 deltas 1454 -> 1317 / 1920 -> 1736 us, 2048 tokens over 32 deltas 985 -> 864 us;
  // 8192 x 8192 with 4096 tokens over 64 deltas 408 -> 381 us; k = 11008 .. 28672: 0-3 % faster.  The knob mid64_max_k
  // can cap it: before the wide kernel's loop lost its conditional waits, k >= 8192 was better off on the narrow kernel.)
  const bool mid64 = tile == 64 && prob_k < knobs().mid64_max_k;
  if (!knobs().mid || (tile != 32 && !mid64)) return false;
  if (prob_k % 128 != 0 || (long)prob_n * prob_k * 2 >= (1L << 32)) return false;   // whole K steps, 32-bit activation offsets
  const long tiles = (n_deltas < prob_n ? n_deltas : prob_n) + prob_n / tile;
  // (and only with a few tokens per tile at least: with two or three the shared activation tile saves nothing
  // and the longer workgroups cost: 200 tokens over 65 of 512 resident deltas of 4096 x 11008 212 -> 238 us; at 3.6 per
  // tile on the bound, 128 tokens over 32 deltas of 4096 x 11008, it depends on the routing: 82 -> 92 us under Zipf(1.0),
  // 76 -> 66 us under Zipf(1.2))
  if (2 * (long)prob_n < (long)knobs().mid_min_half_tokens * tiles) return false;
  if (tile == 32 || tile == 64) {
    const long u32 = mid_units32(prob_n, n_deltas, prob_m, tile);
    if (knobs().mid_depth != 1 && u32 >= kMidDeepMinUnits && u32 <= kMidDeepMaxUnits && prob_n >= kMidDeepMinTokensPerTile * tiles)
      return true;
  }
  const long cgs = (prob_m / 128 + 3) / 4;
  if (cgs < knobs().mid_min_column_groups) {
    // A layer of fewer than 16 column groups (m = 4096): with few tokens per tile it is even at best (64 deltas with 8
    // tokens each 80 us both ways) or loses (128 deltas with 6 each 146 -> 164 us); with a thousand tokens in tiles
    // that are mostly full it wins (4 / 16 / 64 deltas of 4096 x 4096, 1024 tokens: 65 -> 56, 72 -> 65, 107 -> 103 us),
    // as long as the launch has work for the chip (16 deltas with 512 tokens, 256 units on the bound: 45 -> 50 us) and
    // the batch is not one whose hot deltas fill the chip with 64-token tiles of their own (16 deltas, 4096 tokens:
    // 134 -> 153 us).
    // Past 2047 tokens the same holds for as long as the batch's 64-token tiles (tokens / 64 and half a tile per delta,
    // as a randomly routed batch leaves them) fit one round of the 512 workgroups of the 64-token kernel that run
    // together, with 48 tokens per delta and more (emptier tiles lose): 16 deltas with 2048 / 3072 tokens 77-80 -> 70-72,
    // 92 -> 78 us, while with 4096 tokens (a third of a round too many) the split stays ahead, 102 against 118 us.
    const long groups = n_deltas < prob_n ? n_deltas : prob_n;
    const bool one_round = prob_n >= 48 * groups && (prob_n / 64 + (groups + 1) / 2) * cgs <= 512;
    return knobs().mid_narrow && prob_n >= kMidNarrowMinTokens && (prob_n < kMidNarrowMaxTokens || one_round) &&
           tiles * cgs >= (tile == 64 ? kMidNarrowMinUnits64 : kMidNarrowMinUnits);
  }
  return tiles * cgs >= knob_or(knobs().mid_min_units, kMidMinUnits);
}
constexpr int kFusedMaxTokens = 64 * kRawParts;   // kRawParts tokens per lane of a wavefront
// The routed entry point routes inside the multiply kernel (one launch, no plan) or builds a plan first:
static bool routed_eager_ok(int prob_n, int n_deltas) {
  return n_deltas <= 16 && prob_n >= (prob_n > 64 ? 4 : 2) * n_deltas && knobs().eager;
}
static bool routed_in_kernel(int prob_n, int n_deltas, int prob_m, int prob_k) {
  // (more than 32 tokens over more than 16 deltas of a large layer: a skewed batch then has a delta with several
  // 16-token passes, which a plan spreads over workgroups while the in-kernel form runs them one after the other, and
  // the plan's launch is small against the kernel.  64 tokens, Zipf(1.2): 32 deltas of 4096 x 11008 63 -> 58 us,
  // of 11008 x 4096 69 -> 64 us, 64 deltas of 8192 x 28672 375 -> 352 us; on 4096 x 4096 the in-kernel form stays ahead,
  // 30.6 against 32-33 us)
  // (knob fused_route = 2: in the kernel wherever the kernel can -- at most 64 tokens over at most 64 deltas, at most
  // 256 over at most 32 -- whatever the rules below say; for measurements)
  if (knobs().fused_route == 2) return prob_n <= kFusedMaxTokens && n_deltas <= (prob_n > 64 ? 32 : 64);
  if (prob_n > 32 && !routed_eager_ok(prob_n, n_deltas) && (long)prob_k * prob_m >= (1L << 25)) return false;
  return prob_n <= kFusedMaxTokens &&
         n_deltas <= (prob_n > 64 ? 16 : 64) && knobs().fused_route &&
         !(prob_n >= 128 && ((!routed_eager_ok(prob_n, n_deltas) && mid_tiles(prob_n, n_deltas, prob_m, prob_k)) ||
                             (long)prob_k * prob_m >= (1L << 27)));
}
static int plan_has_wide(int prob_n, int n_deltas) {
  const long groups = n_deltas < prob_n ? n_deltas : prob_n;
  return wide_enabled() && prob_n >= knobs().wide_min_batch && prob_n >= 8 * groups;
}

// A batch of 48 tokens per delta and more that pick_nt cuts in 32-token tiles, because it has few tiles in all and
// narrow layers then get twice the workgroups: its plan also lists the tokens in 64-token tiles, and a layer of 16
// column groups and more whose plan tiles go to the wide kernel, in a launch past two workgroups per CU, takes
// those on the 64-token build.  Measured (32-token tiles -> 64-token tiles, evenly routed): 4096 x 11008 with
// 768 / 1024 / 2048 tokens over 8 deltas 78.5 -> 68.9, 86.9 -> 78.5, 156.8 -> 129.3 us; 8192 x 8192 with 1536 / 2048
// over 8 deltas 159.6 -> 141.3, 210.7 -> 161.3 us; 8192 x 28672 with 512 / 1024 tokens over 8 deltas 232.9 -> 179.9,
// 370.9 -> 319.3 us, with 1024 Zipf(1.2)-routed tokens over 8 / 16 deltas 398.6 -> 334.2, 493.7 -> 459.0 us.  With 32 tokens
// per delta, where every second half of a 64-token tile is empty, it loses (4096 x 11008 with 1024 tokens over 32
// deltas 122.9 -> 136.8 us), and narrow layers are better off with the workgroups of 32-token tiles.
// Between 24 and 48 tokens per delta the 64-token tiles pay only where the launch is several rounds of workgroups long
// (from 2304 units of 32-token tiles on the plan's bound: three rounds), where an empty half here and there no longer
// decides a round: 8192 x 28672 with 1024 tokens over 24 / 32 deltas, randomly routed 547 -> 502, 634 -> 593 us,
// Zipf(1.2) 564 -> 546, 693 -> 675 us; on 7B-size layers it is a coin flip at those ratios (4096 x 14336 with 512 tokens
// over 16 deltas 78 -> 83 us randomly routed, 90 -> 111 us Zipf-routed; 8192 x 8192 with 1024 over 32: 184 -> 165 and
// 204 -> 222 us).  The plan lists the 64-token tiles from 24 tokens per delta on; each layer decides.
constexpr int kPlanBigMinTokensPerDelta = 24, kMidBigMinTokensPerDelta = 48;
constexpr long kMidBigManyUnits = 2304;
static int plan_has_big(int prob_n, int n_deltas) {
  const long groups = n_deltas < prob_n ? n_deltas : prob_n;
  const long bar = knobs().plan_big == 1 ? kPlanBigMinTokensPerDelta : knobs().plan_big;   // (a knob above 1 is the bar itself)
  return knobs().plan_big && prob_n >= bar * groups && triteia_hip_plan_tile_tokens(prob_n, n_deltas) == 32;
}
static bool mid_big(int prob_n, int n_deltas, int prob_m, int prob_k) {
  const long groups = n_deltas < prob_n ? n_deltas : prob_n;
  return plan_has_big(prob_n, n_deltas) && (prob_m / 128 + 3) / 4 >= knobs().mid_min_column_groups &&
         (knobs().plan_big > 1 || prob_n >= kMidBigMinTokensPerDelta * groups || mid_units32(prob_n, n_deltas, prob_m, 32) >= kMidBigManyUnits) &&
         mid_tiles(prob_n, n_deltas, prob_m, prob_k) && !mid_deep(prob_n, n_deltas, prob_m, 32);
}
int triteia_hip_wide_unit_order(int prob_m) { return prob_m >= 128 ? wide_unit_order(prob_m) : 0; }
long triteia_hip_wide_grid_units(long rows, int prob_m, int order) {
  if (rows <= 0 || prob_m < 128) return 0;
  if (order == 3 && ((prob_m / 128 + 3) / 4) % 8 == 0) order = 1;
  return wide_grid_units(rows, prob_m, order);
}
long triteia_hip_wide_block_grid_units(long rows, int prob_m, int block_column_groups) {
  if (rows <= 0 || prob_m < 128) return 0;
  return wide_block_grid_units(rows, prob_m, block_column_groups);
}
int triteia_hip_planned_tile_kernel(int prob_n, int n_deltas, int prob_m, int prob_k) {
  if (prob_n <= 0 || n_deltas <= 0 || prob_m <= 0 || prob_k <= 0) return 0;
  if (mid_big(prob_n, n_deltas, prob_m, prob_k)) return 64;
  return mid_tiles(prob_n, n_deltas, prob_m, prob_k) ? triteia_hip_plan_tile_tokens(prob_n, n_deltas) : 0;
}

int triteia_hip_routed_in_kernel(int prob_n, int n_deltas, int prob_m, int prob_k) {
  if (prob_n <= 0 || n_deltas <= 0 || prob_m <= 0 || prob_k <= 0) return 0;
  if (!routed_in_kernel(prob_n, n_deltas, prob_m, prob_k)) return 0;
  // (the launch that sbmm_2_4_routed makes of it: route first unless there are two tokens per delta; 16-token passes)
  const bool shares = prob_n <= 16 && !routed_eager_ok(prob_n, n_deltas) && pick_nt(prob_n, prob_n < n_deltas ? prob_n : n_deltas) == 1 &&
                      share16_tiles(prob_n < n_deltas ? prob_n : n_deltas, prob_m, prob_n);
  return shares ? 2 : 1;
}

int triteia_hip_route_plan(const void* token_indices, int index_offset, int n_deltas, int prob_n, void* workspace,
                           size_t workspace_bytes, int dev, void* stream) {
  if (prob_n < 0 || n_deltas < 0) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "route_plan: tokens=%d deltas=%d", prob_n, n_deltas);
  if (n_deltas > kPlanMaxDeltas)
    return fail(TRITEIA_HIP_ERR_KERN_SHAPE, "route_plan: at most %d deltas per call (got %d)", kPlanMaxDeltas, n_deltas);
  if (!workspace || workspace_bytes < triteia_hip_sbmm_routed_workspace_bytes(prob_n, n_deltas))
    return fail(TRITEIA_HIP_ERR_ARGUMENT, "route_plan: workspace must hold %zu bytes (got %zu)",
                triteia_hip_sbmm_routed_workspace_bytes(prob_n, n_deltas), workspace_bytes);
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
    return fail(TRITEIA_HIP_ERR_ARGUMENT, "route_plan: workspace must be 16-byte aligned");
  if (prob_n > 0 && !token_indices) return fail(TRITEIA_HIP_ERR_ARGUMENT, "route_plan: null indices");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  hipLaunchKernelGGL(route_plan_kernel, dim3(1), dim3(kPlanThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const int*>(token_indices), prob_n, n_deltas, index_offset,
                     triteia_hip_plan_tile_tokens(prob_n, n_deltas), plan_has_wide(prob_n, n_deltas), plan_has_big(prob_n, n_deltas),
                     static_cast<int*>(workspace));
  return check_launch("route_plan_kernel");
}

int triteia_hip_sbmm_2_4_planned(const void* A, const void* B, const void* meta, void* C, const void* s,
                                 const void* plan, int n_deltas, int prob_m, int prob_n, int prob_k, int accumulate,
                                 int dev, void* stream) {
  if (int e = check_gemm_shape(prob_m, prob_n, prob_k, -1)) return e;
  if (accumulate != 0 && accumulate != 1) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sbmm_2_4_planned: accumulate=%d", accumulate);
  if (n_deltas < 0) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "sbmm_2_4_planned: deltas=%d", n_deltas);
  if (prob_m == 0 || prob_n == 0 || prob_k == 0 || n_deltas == 0) return TRITEIA_HIP_OK;
  if (!A || !B || !meta || !C || !s || !plan) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sbmm_2_4_planned: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  const PlanLayout L = plan_layout(prob_n, n_deltas);
  const int* ws = static_cast<const int*>(plan);
  const int tile = triteia_hip_plan_tile_tokens(prob_n, n_deltas);
  Sparse24Args a;
  fill_weights(a, A, B, meta, C, s, prob_m, prob_k, n_deltas);
  a.tiles = reinterpret_cast<const int4*>(ws + L.tiles);
  a.perm = ws + L.perm;
  a.n_groups_dev = ws + L.header;
  a.n_groups = plan_max_tiles(prob_n, n_deltas, tile);
  a.accumulate = accumulate;
  const bool wide = plan_has_wide(prob_n, n_deltas);
  const bool mid = mid_tiles(prob_n, n_deltas, prob_m, prob_k);
  bool wide_launch = false;
  if (wide) {
    a.tiles_alt = reinterpret_cast<const int4*>(ws + L.all);
    a.wide_gate = (prob_m / 128 + 3) / 4;
    a.wide_min_units = knob_or(knobs().plan_wide_min_units, kPlanWideMinUnits);
    // The wide kernel needs whole 128-deep K steps, and a batch that could not reach the bar
    // even with most of its tokens in wide tiles (one per 48 tokens) is not worth the empty
    // launch: then the bar is out of reach on the device too and every tile list is the narrow-only one.
    // (and it addresses activations with 32-bit byte offsets)
    // Nor is it where the 32-token wide kernel takes the plan's tiles: that kernel on the narrow-only list is
    // as fast or faster than a split between the two (cfg4 at 512 / 768 tokens 955 -> 913 / 1075 -> 1032 us).
    wide_launch = !mid && prob_k % 128 == 0 && (long)prob_n * prob_k * 2 < (1L << 32) &&
                  (long)(prob_n / 48 + 1) * a.wide_gate >= a.wide_min_units;
    if (!wide_launch) a.wide_min_units = 0x7fffffff;
    // One list of 64-token tiles over all tokens, for the device to take instead of {wide tiles, narrow rest} where that
    // costs no further round of workgroups (Sparse24Args::tiles_all64): the plan's narrow-only list when it is cut in
    // 64-token tiles, else its list of 64-token tiles beside the 32-token ones, if it has one.  Measured by forcing that
    // list on 16 deltas of 4096 x 4096: 2048 / 3072 tokens 77 -> 70, 92 -> 78 us, 8 deltas with 4096 tokens 98 -> 83 us
    // (the same rounds either way), 16 / 32 deltas with 4096 tokens 102 -> 118, 119 -> 130 us (a further round: the
    // split stays).
    if (wide_launch && knobs().plan_all64) {
      a.plan_header = ws + L.header;
      if (tile == 64) {
        a.tiles_all64 = reinterpret_cast<const int4*>(ws + L.all);
        a.all64_index = 5;
      } else if (plan_has_big(prob_n, n_deltas)) {
        a.tiles_all64 = reinterpret_cast<const int4*>(ws + L.big);
        a.all64_index = 6;
      }
    }
  }
  // The plan's tiles are cut without knowledge of the layer.  Where they make a launch of very few
  // workgroups on this layer (one or two deltas, a narrow matrix: fewer than 200 even on the plan's
  // upper bound of tiles), the kernel takes them in narrower passes split over workgroups (the weights
  // re-read that way come from cache) until there is a workgroup per CU.  Measured on 4096 x 4096: one
  // delta with 64 / 128 tokens 24.4 -> 12.7 / 24.2 -> 18.8 us, two deltas with 256 tokens 24.6 -> 18.5 us;
  // launches of 250 workgroups and more lose 10 % that way and keep the plan's tile.
  int pass_nt = tile / 16;
  {
    const long cb_pad = (prob_m / 128 + 7) / 8 * 8;
    if ((long)a.n_groups * cb_pad < 200)
      while (pass_nt > 1 && (long)a.n_groups * cb_pad * (tile / (16 * pass_nt)) < 256) pass_nt /= 2;
    const int forced = knobs().pass_nt;
    if ((forced == 1 || forced == 2 || forced == 4) && 16 * forced <= tile) pass_nt = forced;
  }
  if (mid) a.xcd_swizzle = wide_unit_order(prob_m);
  if (mid && mid_big(prob_n, n_deltas, prob_m, prob_k)) {
    // the plan's own list of 64-token tiles, whole, on the 64-token build
    const long cgs = (a.m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
    a.tiles = reinterpret_cast<const int4*>(ws + L.big);
    a.tiles_alt = nullptr;
    a.n_groups_dev = ws + L.header + 6;
    a.n_groups = L.max_big;
    if ((long)a.n_groups * cg_pad > 0x7fffffffL) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "too many work units");
    hipLaunchKernelGGL((sparse24_wide_kernel<1, 64, true>), dim3(plan_wide_grid(a, a.n_groups, prob_m, 64, prob_n, n_deltas, 64)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a);
    if (int e = check_launch("sparse24_wide_kernel (plan tiles)")) return e;
  } else if (mid) {
    const long cgs = (a.m / 128 + 3) / 4, cg_pad = (cgs + 7) / 8 * 8;
    if ((long)a.n_groups * cg_pad > 0x7fffffffL) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "too many work units");
    const long units32 = (long)a.n_groups * (tile == 64 ? 2 : 1) * cg_pad;   // in 32-token tiles, on the plan's bound
    if (mid_deep(prob_n, n_deltas, prob_m, tile) && units32 <= 0x7fffffffL) {
      a.tile_halves = tile == 64;
      hipLaunchKernelGGL((sparse24_wide_kernel<2, 32, true>), dim3(plan_wide_grid(a, (long)a.n_groups * (tile == 64 ? 2 : 1), prob_m, 32, prob_n, n_deltas, 64)), dim3(256), 0,
                         static_cast<hipStream_t>(stream), a);
      a.tile_halves = 0;
    } else if (tile == 32)
      hipLaunchKernelGGL((sparse24_wide_kernel<1, 32, true>), dim3(plan_wide_grid(a, a.n_groups, prob_m, 32, prob_n, n_deltas, 64)), dim3(256), 0,
                         static_cast<hipStream_t>(stream), a);
    else
      hipLaunchKernelGGL((sparse24_wide_kernel<1, 64, true>), dim3(plan_wide_grid(a, a.n_groups, prob_m, 64, prob_n, n_deltas, 64)), dim3(256), 0,
                         static_cast<hipStream_t>(stream), a);
    if (int e = check_launch("sparse24_wide_kernel (plan tiles)")) return e;
  } else
  if (int e = launch_sparse24(a, pass_nt, tile / (16 * pass_nt), static_cast<hipStream_t>(stream))) return e;
  if (wide_launch) {
    a.tiles = reinterpret_cast<const int4*>(ws + L.wide);
    a.tiles_alt = nullptr;
    a.n_groups_dev = ws + L.header + 4;
    a.n_groups = L.max_wide;
    if (a.tiles_all64) {   // (the launch covers the longer of the two lists the device may choose from)
      const int all64_max = a.all64_index == 5 ? plan_max_tiles(prob_n, n_deltas, 64) : L.max_big;
      if (all64_max > a.n_groups) a.n_groups = all64_max;
    }
    return launch_wide(a, static_cast<hipStream_t>(stream), kWideTokens, prob_n, n_deltas);
  }
  return TRITEIA_HIP_OK;
}

int triteia_hip_sbmm_2_4_routed(const void* A, const void* B, const void* meta, void* C, const void* s,
                                const void* token_indices, int index_offset, int n_deltas, int prob_m, int prob_n,
                                int prob_k, void* workspace, size_t workspace_bytes, int accumulate, int dev,
                                void* stream) {
  if (int e = check_gemm_shape(prob_m, prob_n, prob_k, -1)) return e;
  if (accumulate != 0 && accumulate != 1) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sbmm_2_4_routed: accumulate=%d", accumulate);
  if (n_deltas < 0) return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "sbmm_2_4_routed: deltas=%d", n_deltas);
  if (prob_m == 0 || prob_n == 0 || prob_k == 0 || n_deltas == 0) return TRITEIA_HIP_OK;
  if (!A || !B || !meta || !C || !s) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sbmm_2_4_routed: null tensor pointer");
  // (above 64 tokens only for at most 16 deltas, whose weights can be requested ahead of the routing: with 32 deltas of
  // 11008 x 4096 and 256 tokens a plan is 10-15 % faster, with 64 deltas of 8192 x 28672 under a skewed routing 1-2 %)
  // (and from 128 tokens on, a batch whose deltas' weights are not requested ahead of the routing is better
  // off with a plan where the plan's tiles go to the 32-token wide kernel: 32 deltas of 4096 x 11008,
  // 128 / 256 tokens: 69 -> 65.5 / 96 -> 89.5 us including the plan; on very large layers (k x m >= 2^27) a
  // plan pays from 128 tokens on whatever the number of deltas, the plan launch being small against the kernel
  // and the wide kernels taking hot deltas: 8 / 4 deltas of 8192 x 28672 with 128 / 256 tokens 145 -> 130 /
  // 160 -> 122 us, while 8 or 16 deltas of 4096 x 11008 stay 8-12 % faster routed inside the kernel)
  const bool eager_ok = routed_eager_ok(prob_n, n_deltas);
  if (routed_in_kernel(prob_n, n_deltas, prob_m, prob_k)) {
    // small batch: the multiply kernel routes by itself, no plan, no workspace traffic
    if (!token_indices) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sbmm_2_4_routed: null indices");
    DeviceGuard g(dev);
    if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
    Sparse24Args a;
    fill_weights(a, A, B, meta, C, s, prob_m, prob_k, n_deltas);
    a.raw_indices = static_cast<const int*>(token_indices);
    a.raw_count = prob_n;
    a.raw_offset = index_offset;
    a.n_groups = prob_n < n_deltas ? prob_n : n_deltas;
    a.accumulate = accumulate;
    const int nt = pick_nt(prob_n, a.n_groups);
    // With at least two tokens per delta on average (four for batches above 64 tokens) nearly every
    // delta is in use: one group per delta, whose weights are requested before the indices have
    // arrived (a delta without tokens costs one prefetched step per wave).  Sparser batches route
    // first.  Only for at most 16 deltas: under a skewed routing larger sets leave many deltas
    // without a token (Zipf(1.5) over 32: 14 in use at 64 tokens, and the prefetched steps of the
    // other 18 make the launch 10 % slower than routing first).
    if (eager_ok) {
      a.raw_static = 1;
      a.n_groups = n_deltas;
    }
    // Above 64 tokens a delta may hold several passes' worth of tokens (a skewed routing, or few deltas): its passes are
    // spread over up to four workgroups instead of running one after the other in one (4 deltas of 4096 x 4096 with 256
    // tokens: 44 -> 21 us; the workgroups that find no pass of their own leave after the routing).
    // (from 33 tokens on already where the weights are not requested ahead of the routing, i.e. where a workgroup without
    // a pass costs nothing but its routing: 64 tokens under Zipf(1.2) over 32 deltas of 11008 x 4096, 70 -> 64 us)
    const long tsplit = prob_n <= (eager_ok ? 64 : 32) ? 1 : (prob_n <= 128 ? 2 : 4);
    return launch_sparse24(a, nt, tsplit, static_cast<hipStream_t>(stream));
  }
  if (int e = triteia_hip_route_plan(token_indices, index_offset, n_deltas, prob_n, workspace, workspace_bytes, dev, stream))
    return e;
  return triteia_hip_sbmm_2_4_planned(A, B, meta, C, s, workspace, n_deltas, prob_m, prob_n, prob_k, accumulate, dev, stream);
}

size_t triteia_hip_sbmm_routed_static_max_bytes(void) { return kStaticPlanBytes; }

int triteia_hip_sbmm_2_4_routed_static(const void* A, const void* B, const void* meta, void* C, const void* s,
                                       const void* token_indices, int index_offset, int n_deltas, int prob_m,
                                       int prob_n, int prob_k, int accumulate, int dev, void* stream) {
  if (prob_n < 0 || n_deltas < 0)
    return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "sbmm_2_4_routed_static: tokens=%d deltas=%d", prob_n, n_deltas);
  const size_t need = triteia_hip_sbmm_routed_workspace_bytes(prob_n, n_deltas);
  if (need > kStaticPlanBytes)
    return fail(TRITEIA_HIP_ERR_KERN_SHAPE,
                "sbmm_2_4_routed_static: the routing plan of %d tokens over %d deltas takes %zu bytes, the library's "
                "scratch holds %zu; use triteia_hip_sbmm_2_4_routed with a workspace of the caller's",
                prob_n, n_deltas, need, kStaticPlanBytes);
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  void* plan = nullptr;
  if (int e = static_plan_address(&plan)) return e;
  // (the plan kernel writes every word of the plan that the multiply kernels read: nothing to clear)
  return triteia_hip_sbmm_2_4_routed(A, B, meta, C, s, token_indices, index_offset, n_deltas, prob_m, prob_n, prob_k, plan,
                                     kStaticPlanBytes, accumulate, -1, stream);
}

}  // extern "C"

namespace {
typedef __bf16 bf16_t;

template <class T, bool ACC = true>
int bgmv_impl(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out, int num_layers,
              int layer_idx, float scale, int dev, void* stream) {
  if (batch < 0 || h_in <= 0 || h_out <= 0 || num_layers <= 0 || layer_idx < 0 || layer_idx >= num_layers)
    return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "bgmv: batch=%d h_in=%d h_out=%d layers=%d layer=%d", batch, h_in, h_out, num_layers, layer_idx);
  const int narrow = h_in < h_out ? h_in : h_out;
  if (h_in % 8 != 0 || h_out % 8 != 0 || narrow > kLoraMaxNarrow)
    return fail(TRITEIA_HIP_ERR_KERN_SHAPE, "No suitable kernel. h_in=%d h_out=%d", h_in, h_out);
  if (batch == 0) return TRITEIA_HIP_OK;
  if (!Y || !X || !W || !indices) return fail(TRITEIA_HIP_ERR_ARGUMENT, "bgmv: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (h_in >= h_out) {
    hipLaunchKernelGGL((bgmv_shrink_kernel<T, ACC>), dim3(batch), dim3(256), 0, st, static_cast<T*>(Y), static_cast<const T*>(X),
                       static_cast<const T*>(W), static_cast<const long long*>(indices), h_in, h_out, (long)num_layers,
                       (long)layer_idx, scale);
  } else if (h_in == 8 || h_in == 16 || h_in == 32 || h_in == 64 || h_in == 128) {
    // weight rows spread over neighbouring lanes (whole cache lines per load instruction), four tokens per block
    constexpr int Q = 8, TB = 4;
    const int rows_per_block = 4 * Q * 64 / (h_in / 8);
    const dim3 grid((h_out + rows_per_block - 1) / rows_per_block, (batch + TB - 1) / TB);
#define BGMV_LINES(LPR_) hipLaunchKernelGGL((bgmv_expand_lines_kernel<T, LPR_, Q, TB, ACC>), grid, dim3(256), 0, st, static_cast<T*>(Y), \
      static_cast<const T*>(X), static_cast<const T*>(W), static_cast<const long long*>(indices), batch, h_out, (long)num_layers, \
      (long)layer_idx, scale)
    if (h_in == 8) BGMV_LINES(1); else if (h_in == 16) BGMV_LINES(2); else if (h_in == 32) BGMV_LINES(4);
    else if (h_in == 64) BGMV_LINES(8); else BGMV_LINES(16);
#undef BGMV_LINES
  } else {
    hipLaunchKernelGGL((bgmv_expand_kernel<T, ACC>), dim3((h_out + 2047) / 2048, batch), dim3(256), 0, st, static_cast<T*>(Y),
                       static_cast<const T*>(X), static_cast<const T*>(W), static_cast<const long long*>(indices), h_in,
                       h_out, (long)num_layers, (long)layer_idx, scale);
  }
  return check_launch("bgmv kernel");
}

#ifndef TRITEIA_SHRINK_ROWS16
#define TRITEIA_SHRINK_ROWS16 2
#endif
#ifndef TRITEIA_EXPAND_ROWS16
#define TRITEIA_EXPAND_ROWS16 4
#endif
constexpr int kShrinkRows16 = TRITEIA_SHRINK_ROWS16;   // token rows a block of the rank <= 16 shrink kernel takes at a time
constexpr int kExpandRows16 = TRITEIA_EXPAND_ROWS16;

// Adapters of rank 32, 64 or 128 run on the matrix cores (lora_mfma.hip.h): the expand always (512 tokens over 8
// adapters of rank 64 on 4096 columns 42.9 -> 7.5 us, 256 over 32 on 11008 columns 291 -> 15 us); the shrink, where a
// workgroup pulls the whole adapter through one CU per pass of tokens, from 128 rows per group on (`rows_per_group`:
// what the caller knows of the average, 0 = nothing; 2048 tokens over 4 adapters of rank 64 / 128 on k = 4096 46.4 -> 28.9 /
// 81.1 -> 32.5 us, 512 over 8 20.0 -> 23.2 us).  The knob lora_mfma = 2 sends every launch there that the kernels can
// take (the shrink also at rank 16), 0 none.
constexpr int kLoraMfmaShrinkMinRows = 128;
template <class T>
bool launch_sgmv_mfma(const SgmvArgsT<T>& a, int max_rows, int rows_per_group, hipStream_t st) {
  const int mode = knobs().lora_mfma;
  if (mode == 0) return false;
  int row_slots = max_rows < 1 ? 1 : max_rows;
  if (a.d_in >= a.d_out) {
    if (mode == 1 && rows_per_group < kLoraMfmaShrinkMinRows) return false;
    if (a.d_in % 32 != 0 || !(a.d_out == 32 || a.d_out == 64 || a.d_out == 128 || (a.d_out == 16 && mode == 2))) return false;
    if (row_slots > 256) row_slots = 256;
#define SHRINK_MFMA(R16_, TT_) hipLaunchKernelGGL((sgmv_shrink_mfma_kernel<T, R16_, TT_>), dim3(a.n_groups, (row_slots + 16 * TT_ - 1) / (16 * TT_)), dim3(256), 0, st, a)
    if (a.d_out == 16) SHRINK_MFMA(1, 4); else if (a.d_out == 32) SHRINK_MFMA(2, 4); else if (a.d_out == 64) SHRINK_MFMA(4, 4); else SHRINK_MFMA(8, 2);
#undef SHRINK_MFMA
    return true;
  }
  if (!(a.d_in == 32 || a.d_in == 64 || a.d_in == 128)) return false;
  if (row_slots > 64) row_slots = 64;
  const dim3 grid(a.n_groups, (a.d_out + 127) / 128, (row_slots + 15) / 16);
  if (a.d_in == 32) hipLaunchKernelGGL((sgmv_expand_mfma_kernel<T, 1>), grid, dim3(256), 0, st, a);
  else if (a.d_in == 64) hipLaunchKernelGGL((sgmv_expand_mfma_kernel<T, 2>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((sgmv_expand_mfma_kernel<T, 4>), grid, dim3(256), 0, st, a);
  return true;
}

template <class T>
int launch_sgmv(SgmvArgsT<T> a, int max_rows, hipStream_t st, int rows_per_group = 0) {
  const int narrow = a.d_in < a.d_out ? a.d_in : a.d_out;
  if (a.d_in % 8 != 0 || a.d_out % 8 != 0 || narrow > kLoraMaxNarrow)
    return fail(TRITEIA_HIP_ERR_KERN_SHAPE, "No suitable kernel. d_in=%d d_out=%d", a.d_in, a.d_out);
  if (a.n_groups <= 0) return TRITEIA_HIP_OK;
  if (launch_sgmv_mfma(a, max_rows, rows_per_group, st)) return check_launch("sgmv kernel (matrix cores)");
  // rows of a group are spread over y (shrink) / z (expand); group sizes live on the device
  int row_slots = max_rows < 64 ? max_rows : 64;
  if (row_slots < 1) row_slots = 1;
  auto slots = [&](int rows_per_block) { return (row_slots + rows_per_block - 1) / rows_per_block; };
  if (a.d_in >= a.d_out) {
    if (a.d_out <= 16) hipLaunchKernelGGL((sgmv_shrink_kernel<16, kShrinkRows16, T>), dim3(a.n_groups, slots(kShrinkRows16)), dim3(256), 0, st, a);
    else if (a.d_out <= 32) hipLaunchKernelGGL((sgmv_shrink_kernel<32, 2, T>), dim3(a.n_groups, slots(2)), dim3(256), 0, st, a);
    else if (a.d_out <= 64) hipLaunchKernelGGL((sgmv_shrink_kernel<64, 1, T>), dim3(a.n_groups, slots(1)), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((sgmv_shrink_kernel<128, 1, T>), dim3(a.n_groups, slots(1)), dim3(256), 0, st, a);
  } else {
    const int rz = row_slots < 8 ? row_slots : 8;
    const dim3 grid(a.n_groups, (a.d_out + 255) / 256, rz);
    const int col_blocks = (a.d_out + 2047) / 2048;
    if (a.d_in <= 16 && a.accumulate) hipLaunchKernelGGL((sgmv_expand_vec_kernel<16, kExpandRows16, T, true>), dim3(a.n_groups, col_blocks, slots(kExpandRows16)), dim3(256), 0, st, a);
    else if (a.d_in <= 16) hipLaunchKernelGGL((sgmv_expand_vec_kernel<16, kExpandRows16, T, false>), dim3(a.n_groups, col_blocks, slots(kExpandRows16)), dim3(256), 0, st, a);
    else if (a.d_in <= 32 && a.accumulate) hipLaunchKernelGGL((sgmv_expand_vec_kernel<32, 2, T, true>), dim3(a.n_groups, col_blocks, slots(2)), dim3(256), 0, st, a);
    else if (a.d_in <= 32) hipLaunchKernelGGL((sgmv_expand_vec_kernel<32, 2, T, false>), dim3(a.n_groups, col_blocks, slots(2)), dim3(256), 0, st, a);
    else if (a.d_in <= 64) hipLaunchKernelGGL((sgmv_expand_kernel<64, T>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((sgmv_expand_kernel<128, T>), grid, dim3(256), 0, st, a);
  }
  return check_launch("sgmv kernel");
}

template <class T>
int sgmv_impl(void* y, const void* x, const void* w_ptrs, const void* s, int num_problems, int d_in, int d_out, int layer_idx,
              int accumulate, int dev, void* stream) {
  if (num_problems < 0 || d_in <= 0 || d_out <= 0 || layer_idx < 0)
    return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "sgmv: problems=%d d_in=%d d_out=%d layer=%d", num_problems, d_in, d_out, layer_idx);
  if (num_problems == 0) return TRITEIA_HIP_OK;
  if (!y || !x || !w_ptrs || !s) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sgmv: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  SgmvArgsT<T> a;
  memset(&a, 0, sizeof(a));
  a.y = static_cast<T*>(y);
  a.y_stride = d_out;
  a.x = static_cast<const T*>(x);
  a.x_stride = d_in;
  a.d_in = d_in;
  a.d_out = d_out;
  a.w_ptrs = static_cast<const long long*>(w_ptrs);
  a.layer_off = (long)layer_idx * d_in * d_out;
  a.seg = static_cast<const int*>(s);
  a.n_groups = num_problems;
  a.n_adapters = num_problems;
  a.scale = 1.0f;
  a.accumulate = accumulate;
  // segment lengths live on the device; size the row-tile dimension for a few rows per segment
  return launch_sgmv(a, 64, static_cast<hipStream_t>(stream));
}

template <class T>
int sgmv_routed_impl(void* y, long y_stride, const void* x, long x_stride, const void* w_base, long w_stride, int n_adapters,
                     int d_in, int d_out, float scale, const void* plan, int prob_n, int accumulate, int dev, void* stream) {
  if (accumulate != 0 && accumulate != 1) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sgmv_routed: accumulate=%d", accumulate);
  if (prob_n < 0 || n_adapters < 0 || d_in <= 0 || d_out <= 0)
    return fail(TRITEIA_HIP_ERR_PROB_SHAPE, "sgmv_routed: tokens=%d adapters=%d d_in=%d d_out=%d", prob_n, n_adapters, d_in, d_out);
  if (prob_n == 0 || n_adapters == 0) return TRITEIA_HIP_OK;
  if (!y || !x || !w_base || !plan) return fail(TRITEIA_HIP_ERR_ARGUMENT, "sgmv_routed: null tensor pointer");
  DeviceGuard g(dev);
  if (!g.ok) return fail(TRITEIA_HIP_ERR_RUNTIME, "cannot select device %d", dev);
  const PlanLayout L = plan_layout(prob_n, n_adapters);
  const int* ws = static_cast<const int*>(plan);
  SgmvArgsT<T> a;
  memset(&a, 0, sizeof(a));
  a.y = static_cast<T*>(y);
  a.y_stride = y_stride;
  a.x = static_cast<const T*>(x);
  a.x_stride = x_stride;
  a.d_in = d_in;
  a.d_out = d_out;
  a.w_base = static_cast<const T*>(w_base);
  a.w_stride = w_stride;
  // a plan with wide tiles also lists all its tokens in narrow tiles: that is the cut for LoRA
  const bool wide = plan_has_wide(prob_n, n_adapters);
  a.tiles = reinterpret_cast<const int4*>(ws + (wide ? L.all : L.tiles));
  a.perm = ws + L.perm;
  a.n_groups_dev = ws + L.header + (wide ? 5 : 0);
  a.n_groups = plan_max_tiles(prob_n, n_adapters, triteia_hip_plan_tile_tokens(prob_n, n_adapters));
  a.n_adapters = n_adapters;
  a.scale = scale;
  a.accumulate = accumulate;
  return launch_sgmv(a, prob_n, static_cast<hipStream_t>(stream), prob_n / (n_adapters < prob_n ? n_adapters : prob_n));
}

}  // namespace

extern "C" {

int triteia_hip_bgmv(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                     int num_layers, int layer_idx, float scale, int dev, void* stream) {
  return bgmv_impl<_Float16>(Y, X, W, indices, batch, h_in, h_out, num_layers, layer_idx, scale, dev, stream);
}
int triteia_hip_bgmv_bf16(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                          int num_layers, int layer_idx, float scale, int dev, void* stream) {
  return bgmv_impl<bf16_t>(Y, X, W, indices, batch, h_in, h_out, num_layers, layer_idx, scale, dev, stream);
}
int triteia_hip_bgmv_store(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                           int num_layers, int layer_idx, float scale, int dev, void* stream) {
  return bgmv_impl<_Float16, false>(Y, X, W, indices, batch, h_in, h_out, num_layers, layer_idx, scale, dev, stream);
}
int triteia_hip_bgmv_store_bf16(void* Y, const void* X, const void* W, const void* indices, int batch, int h_in, int h_out,
                                int num_layers, int layer_idx, float scale, int dev, void* stream) {
  return bgmv_impl<bf16_t, false>(Y, X, W, indices, batch, h_in, h_out, num_layers, layer_idx, scale, dev, stream);
}

size_t triteia_hip_sgmv_tmp_size(int num_problems) {
  // the reference's CUTLASS argument block: 60 bytes per problem (sgmv.cuh:48-52)
  return num_problems > 0 ? (size_t)60 * (size_t)num_problems : 0;
}

int triteia_hip_sgmv(void* y, const void* x, const void* w_ptrs, const void* s, void* tmp, int num_problems, int d_in,
                     int d_out, int layer_idx, int dev, void* stream) {
  (void)tmp;
  return sgmv_impl<_Float16>(y, x, w_ptrs, s, num_problems, d_in, d_out, layer_idx, 1, dev, stream);
}
int triteia_hip_sgmv_bf16(void* y, const void* x, const void* w_ptrs, const void* s, void* tmp, int num_problems, int d_in,
                          int d_out, int layer_idx, int dev, void* stream) {
  (void)tmp;
  return sgmv_impl<bf16_t>(y, x, w_ptrs, s, num_problems, d_in, d_out, layer_idx, 1, dev, stream);
}
int triteia_hip_sgmv_store(void* y, const void* x, const void* w_ptrs, const void* s, int num_problems, int d_in, int d_out,
                           int layer_idx, int dev, void* stream) {
  return sgmv_impl<_Float16>(y, x, w_ptrs, s, num_problems, d_in, d_out, layer_idx, 0, dev, stream);
}
int triteia_hip_sgmv_store_bf16(void* y, const void* x, const void* w_ptrs, const void* s, int num_problems, int d_in, int d_out,
                                int layer_idx, int dev, void* stream) {
  return sgmv_impl<bf16_t>(y, x, w_ptrs, s, num_problems, d_in, d_out, layer_idx, 0, dev, stream);
}

int triteia_hip_sgmv_routed(void* y, long y_stride, const void* x, long x_stride, const void* w_base, long w_stride,
                            int n_adapters, int d_in, int d_out, float scale, const void* plan, int prob_n,
                            int accumulate, int dev, void* stream) {
  return sgmv_routed_impl<_Float16>(y, y_stride, x, x_stride, w_base, w_stride, n_adapters, d_in, d_out, scale, plan, prob_n, accumulate, dev, stream);
}
int triteia_hip_sgmv_routed_bf16(void* y, long y_stride, const void* x, long x_stride, const void* w_base, long w_stride,
                                 int n_adapters, int d_in, int d_out, float scale, const void* plan, int prob_n,
                                 int accumulate, int dev, void* stream) {
  return sgmv_routed_impl<bf16_t>(y, y_stride, x, x_stride, w_base, w_stride, n_adapters, d_in, d_out, scale, plan, prob_n, accumulate, dev, stream);
}

}  // extern "C"
