// Device-side routing prep for the indexed ops: groups the tokens of one batch
// by delta index without any host round trip.
//
// Replaces the host-side prep of the reference
// (triteia/python/ops/matmul/sbmm.py:94-123: torch.all / unique_consecutive /
// where()[0][0] / cumsum, each a device->host sync) and, unlike it, accepts
// indices in any order with -1 (no delta) anywhere.
//
// Output (all int32, in the caller's workspace):
//   header[0] = number of narrow tiles, header[1] = number of routed tokens,
//   header[2] = number of deltas that have at least one token, header[3] = narrow tile size,
//   header[4] = number of wide tiles, header[5] = number of tiles in all[], header[6] = number of tiles in big[],
//   header[7] = 0
//   tiles[..] = {delta, start, count, 0}: `count` <= tile size tokens of one delta,
//               listed at perm[start .. start+count); ascending delta id, a delta's
//               tiles are adjacent
//   wide[..]  = same, for 64-token tiles (only when built with wide = 1): a delta with c
//               tokens gets c/64 full wide tiles, one more if the rest exceeds 32 tokens,
//               and narrow tiles (in tiles[]) for a smaller rest
//   perm[routed] = token rows, grouped by delta, original order kept inside a
//               delta (stable)
//   all[..]   = (only with wide = 1) the same tokens cut into narrow tiles only: the consumer
//               chooses between {tiles, wide} and {all} per weight shape, on the device
//   big[..]   = (only when built with big = 1) the same tokens cut into 64-token tiles only, for the layers on which
//               the consumer prefers those to the narrow tiles the plan was cut in
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace triteia_hip {

constexpr int kPlanHeaderInts = 8;
constexpr int kPlanWideTile = 64;      // tokens per wide tile
constexpr int kPlanWideMinRest = 33;   // a rest of at least this many tokens still forms a wide tile
constexpr int kPlanMaxDeltas = 8192;  // per-delta cursors live in LDS
constexpr int kPlanThreads = 1024;     // 16 wavefronts
constexpr int kPlanCachedTokens = 8192;  // token indices kept in LDS between the two passes
constexpr int kPlanMinTile = 16;      // smallest tile size a plan can be built for

struct PlanLayout {
  int header, tiles, wide, perm, all, big, total;  // offsets in ints
  int max_tiles, max_wide, max_big;
};

// The layout depends only on (tokens, deltas), not on the tile size the plan is built
// for, so that every consumer finds `perm` without knowing it.
__host__ __device__ inline PlanLayout plan_layout(int n_tokens, int n_deltas) {
  const int g = n_deltas < n_tokens ? n_deltas : n_tokens;
  PlanLayout l;
  l.max_tiles = g + n_tokens / kPlanMinTile;
  l.max_wide = n_tokens / kPlanWideMinRest + 1;
  l.header = 0;
  l.tiles = kPlanHeaderInts;
  l.wide = l.tiles + 4 * l.max_tiles;
  l.perm = l.wide + 4 * l.max_wide;
  l.all = (l.perm + n_tokens + 3) & ~3;
  l.big = l.all + 4 * l.max_tiles;
  l.max_big = g + n_tokens / kPlanWideTile;
  l.total = l.big + 4 * l.max_big;
  return l;
}

__host__ __device__ inline int plan_max_tiles(int n_tokens, int n_deltas, int tile) {
  const int g = n_deltas < n_tokens ? n_deltas : n_tokens;
  return g + n_tokens / tile;
}

__device__ __forceinline__ int wave_excl_scan(int v, int lane, int* total) {
  int incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  *total = __shfl(incl, 63, 64);
  return incl - v;
}

// One workgroup.  indices[t] - index_offset outside [0, n_deltas) means "no delta".
//
// The tokens are cut into `shares` of whole 64-token pieces, one per wavefront (as many as the 8192 LDS counters
// allow: 16 shares up to 512 deltas, one at 8192).  Every token is counted under (share, delta); the scan over the
// deltas then turns the counts of a delta's shares into the shares' first slots in perm, one behind the other, so
// that the wavefronts can place their shares side by side and the order inside a delta is still the batch's.
__global__ __launch_bounds__(kPlanThreads) void route_plan_kernel(const int* __restrict__ indices, int n_tokens,
                                                                 int n_deltas, int index_offset, int tile, int wide,
                                                                 int big, int* __restrict__ ws) {
  __shared__ int s_cursor[kPlanMaxDeltas];     // [share][delta]: counts, then cursors into perm
  __shared__ int s_delta[kPlanCachedTokens];   // pass 1 leaves each token's delta here for pass 2
  const PlanLayout L = plan_layout(n_tokens, n_deltas);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  int shares = kPlanThreads / 64;
  if (n_deltas > 0 && shares > kPlanMaxDeltas / n_deltas) shares = kPlanMaxDeltas / n_deltas;
  if (shares > (n_tokens + 63) / 64) shares = (n_tokens + 63) / 64;
  if (shares < 1) shares = 1;
  const int share_tokens = (((n_tokens + shares - 1) / shares) + 63) & ~63;   // whole 64-token pieces

  for (int i = tid; i < shares * n_deltas; i += kPlanThreads) s_cursor[i] = 0;
  __syncthreads();
  for (int t = tid; t < n_tokens; t += kPlanThreads) {
    int d = indices[t] - index_offset;
    if (d < 0 || d >= n_deltas) d = -1;
    if (t < kPlanCachedTokens) s_delta[t] = d;
    if (d >= 0) atomicAdd(&s_cursor[(t / share_tokens) * n_deltas + d], 1);
  }
  __syncthreads();

  if (wave == 0) {
    // exclusive scans over the deltas, 64 per iteration: token counts -> first slot in perm,
    // tile counts -> first tile
    int running = 0, tiles = 0, wides = 0, alls = 0, bigs = 0, groups = 0;
    int4* tile_out = reinterpret_cast<int4*>(ws + L.tiles);
    int4* wide_out = reinterpret_cast<int4*>(ws + L.wide);
    int4* all_out = reinterpret_cast<int4*>(ws + L.all);
    int4* big_out = reinterpret_cast<int4*>(ws + L.big);
    for (int base = 0; base < n_deltas; base += 64) {
      const int d = base + lane;
      int c = 0;
      if (d < n_deltas)
        for (int w = 0; w < shares; w++) c += s_cursor[w * n_deltas + d];
      int chunk_tokens, chunk_tiles, chunk_wides, chunk_alls;
      const int offs = running + wave_excl_scan(c, lane, &chunk_tokens);
      // split this delta's tokens: wide tiles first, the rest in narrow tiles
      int nw = 0, c_wide = 0;
      if (wide) {
        nw = c / kPlanWideTile;
        c_wide = nw * kPlanWideTile;
        if (c - c_wide >= kPlanWideMinRest) { nw++; c_wide = c; }
      }
      const int c_rest = c - c_wide;
      const int nt = (c_rest + tile - 1) / tile;
      const int wpos = wides + wave_excl_scan(nw, lane, &chunk_wides);
      const int tpos = tiles + wave_excl_scan(nt, lane, &chunk_tiles);
      for (int i = 0; i < nw; i++) {
        const int first = i * kPlanWideTile;
        wide_out[wpos + i] = make_int4(d, offs + first, min(kPlanWideTile, c_wide - first), 0);
      }
      for (int i = 0; i < nt; i++) {
        const int first = i * tile;
        tile_out[tpos + i] = make_int4(d, offs + c_wide + first, min(tile, c_rest - first), 0);
      }
      if (wide) {
        const int na = (c + tile - 1) / tile;
        const int apos = alls + wave_excl_scan(na, lane, &chunk_alls);
        for (int i = 0; i < na; i++) {
          const int first = i * tile;
          all_out[apos + i] = make_int4(d, offs + first, min(tile, c - first), 0);
        }
        alls += chunk_alls;
      }
      if (big) {
        int chunk_bigs;
        const int nb = (c + kPlanWideTile - 1) / kPlanWideTile;
        const int bpos = bigs + wave_excl_scan(nb, lane, &chunk_bigs);
        for (int i = 0; i < nb; i++) {
          const int first = i * kPlanWideTile;
          big_out[bpos + i] = make_int4(d, offs + first, min(kPlanWideTile, c - first), 0);
        }
        bigs += chunk_bigs;
      }
      if (d < n_deltas) {
        // the shares' pieces of this delta's run of slots, in the order of the shares
        int before = 0;
        for (int w = 0; w < shares; w++) {
          const int mine = s_cursor[w * n_deltas + d];
          s_cursor[w * n_deltas + d] = offs + before;
          before += mine;
        }
      }
      running += chunk_tokens;
      tiles += chunk_tiles;
      wides += chunk_wides;
      groups += __popcll(__ballot(c > 0));
    }
    if (lane == 0) {
      ws[L.header + 0] = tiles;
      ws[L.header + 1] = running;
      ws[L.header + 2] = groups;
      ws[L.header + 3] = tile;
      ws[L.header + 4] = wides;
      ws[L.header + 5] = alls;
      ws[L.header + 6] = bigs;
      ws[L.header + 7] = 0;
    }
  }
  __syncthreads();

  if (wave < shares) {
    // stable placement of this wavefront's share: 64 tokens at a time, tokens with equal delta ranked by lane order
    int* cursor = s_cursor + wave * n_deltas;
    const int end = min(n_tokens, (wave + 1) * share_tokens);
    for (int base = wave * share_tokens; base < end; base += 64) {
      const int t = base + lane;
      int d = -1;
      if (t < end) {
        if (t < kPlanCachedTokens) {
          d = s_delta[t];
        } else {
          d = indices[t] - index_offset;
          if (d < 0 || d >= n_deltas) d = -1;
        }
      }
      // lanes holding the same delta, found for all lanes at once: intersect, bit by bit of the
      // delta id, the lanes that agree with this lane on that bit
      const unsigned long long valid = __ballot(d >= 0);
      unsigned long long same = valid;
      for (int bit = 0; (1 << bit) < n_deltas; bit++) {
        const unsigned long long set = __ballot((d >> bit) & 1);
        same &= ((d >> bit) & 1) ? set : ~set;
      }
      if (d >= 0) {
        const int rank = __popcll(same & ((1ull << lane) - 1ull));
        const int first = cursor[d];
        ws[L.perm + first + rank] = t;
        // every lane of the group has read the cursor before its first lane moves it
        __builtin_amdgcn_wave_barrier();
        if (rank == 0) cursor[d] = first + __popcll(same);
      }
    }
  }
}

}  // namespace triteia_hip
