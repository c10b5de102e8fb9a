// Device-side routing prep for the indexed ops: groups the tokens of one batch
// by delta index without any host round trip.
//
// Replaces the host-side prep of the reference
// (triteia/python/ops/matmul/sbmm.py:94-123: torch.all / unique_consecutive /
// where()[0][0] / cumsum, each a device->host sync) and, unlike it, accepts
// indices in any order with -1 (no delta) anywhere.
//
// Output (all int32, in the caller's workspace):
//   header[0] = number of groups G (deltas that have at least one token)
//   header[1] = number of routed tokens
//   g_delta[G], g_start[G], g_count[G] : per group, ascending delta id
//   perm[routed] : token rows, grouped by delta, original order kept inside a
//                  group (stable), g_start indexes into it
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace triteia_hip {

constexpr int kPlanHeaderInts = 4;
constexpr int kPlanMaxDeltas = 8192;  // per-delta cursors live in LDS
constexpr int kPlanThreads = 256;

struct PlanLayout {
  int header, g_delta, g_start, g_count, perm, total;  // offsets in ints
};

__host__ __device__ inline PlanLayout plan_layout(int n_tokens, int n_deltas) {
  const int g = n_deltas < n_tokens ? n_deltas : n_tokens;
  PlanLayout l;
  l.header = 0;
  l.g_delta = kPlanHeaderInts;
  l.g_start = l.g_delta + g;
  l.g_count = l.g_start + g;
  l.perm = l.g_count + g;
  l.total = l.perm + n_tokens;
  return l;
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

// One workgroup.  indices[t] outside [0, n_deltas) means "no delta".
__global__ __launch_bounds__(kPlanThreads) void route_plan_kernel(const int* __restrict__ indices, int n_tokens,
                                                                 int n_deltas, int index_offset, int* __restrict__ ws) {
  __shared__ int s_cursor[kPlanMaxDeltas];
  const PlanLayout L = plan_layout(n_tokens, n_deltas);
  const int tid = threadIdx.x;
  const int lane = tid & 63;

  for (int d = tid; d < n_deltas; d += kPlanThreads) s_cursor[d] = 0;
  __syncthreads();
  for (int t = tid; t < n_tokens; t += kPlanThreads) {
    const int d = indices[t] - index_offset;
    if (d >= 0 && d < n_deltas) atomicAdd(&s_cursor[d], 1);
  }
  __syncthreads();

  if (tid < 64) {
    // exclusive scan of the counts (-> first slot of every delta) and compaction
    // of the deltas that have tokens, 64 deltas per iteration
    int running = 0, groups = 0;
    for (int base = 0; base < n_deltas; base += 64) {
      const int d = base + lane;
      const int c = d < n_deltas ? s_cursor[d] : 0;
      int chunk_total;
      const int offs = running + wave_excl_scan(c, lane, &chunk_total);
      const unsigned long long act = __ballot(c > 0);
      if (c > 0) {
        const int pos = groups + __popcll(act & ((1ull << lane) - 1ull));
        ws[L.g_delta + pos] = d;
        ws[L.g_start + pos] = offs;
        ws[L.g_count + pos] = c;
      }
      if (d < n_deltas) s_cursor[d] = offs;
      running += chunk_total;
      groups += __popcll(act);
    }
    if (lane == 0) {
      ws[L.header + 0] = groups;
      ws[L.header + 1] = running;
      ws[L.header + 2] = 0;
      ws[L.header + 3] = 0;
    }
    // stable placement: 64 tokens at a time, tokens with equal delta ranked by lane order
    for (int base = 0; base < n_tokens; base += 64) {
      const int t = base + lane;
      int d = -1;
      if (t < n_tokens) {
        d = indices[t] - index_offset;
        if (d < 0 || d >= n_deltas) d = -1;
      }
      unsigned long long todo = __ballot(d >= 0);
      while (todo) {
        const int leader = __ffsll((long long)todo) - 1;
        const int dl = __shfl(d, leader, 64);
        const unsigned long long same = __ballot(d == dl) & todo;
        const int first = s_cursor[dl];
        if (d == dl && ((same >> lane) & 1ull)) ws[L.perm + first + __popcll(same & ((1ull << lane) - 1ull))] = t;
        // every lane has read s_cursor[dl] before the leader bumps it
        __builtin_amdgcn_wave_barrier();
        if (lane == leader) s_cursor[dl] = first + __popcll(same);
        __builtin_amdgcn_wave_barrier();
        todo &= ~same;
      }
    }
  }
}

}  // namespace triteia_hip
