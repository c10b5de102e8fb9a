// LoRA matrix-vector kernels for gfx950: BGMV (one adapter per token) and SGMV
// (one adapter per segment / group of tokens).  Element type T = fp16 or bf16 (the reference
// instantiates both: triteia/csrc/ops/bgmv_all.cu:4-5, sgmv.cu:10), fp32 accumulate,
// read-modify-write of y in T.
//
// Semantics follow the reference:
//   BGMV  Y[b, j] += scale * sum_i W[idx_b * L + layer][j][i] * X[b][i]
//         (triteia/csrc/ops/bgmv_impl.cuh:14-183, weights stored out-major)
//   SGMV  y[s_g : s_g+1] += x[s_g : s_g+1] @ W_g, W_g row-major [d_in, d_out]
//         (triteia/csrc/ops/sgmv.cuh:61-174, alpha = beta = 1)
// Any (d_in, d_out) with the narrow side <= 128 and both sides multiples of 8
// is accepted at run time (the reference enumerates shapes at compile time,
// triteia/csrc/ops/bgmv_config.h:11-36).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef TRITEIA_SHRINK_UNROLL
#define TRITEIA_SHRINK_UNROLL 4
#endif

namespace triteia_hip {

template <class T> using lvec8 = T __attribute__((ext_vector_type(8)));
template <class T> using lvec2 = T __attribute__((ext_vector_type(2)));

constexpr int kLoraMaxNarrow = 128;

// Load through a pointer that is known to point into global memory.  (An adapter pointer read from the
// caller's pointer table is a generic pointer to the compiler: its loads become flat loads, which count
// against the LDS / scalar counter as well and are waited for more conservatively.)
template <class T>
__device__ __forceinline__ T load_global(const T* p) {
  return *(const __attribute__((address_space(1))) T*)(uintptr_t)p;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---------------------------------------------------------------- BGMV ----

// wide -> narrow: grid (B), block 256.  The block walks the token's activations once per 16 outputs: thread t takes the
// 8-element pieces t, t + 256, ... of x and of each of the 16 weight rows (all of a piece's loads are independent, so
// they are in flight together), then the 16 partial sums are added over the wavefront by shuffles and over the four
// wavefronts through LDS.
// ACC: the result is added to what Y holds (the reference's semantics); otherwise it is stored, and Y is not read
// (rows whose index is negative are left alone either way).
template <class T, bool ACC = true>
__global__ __launch_bounds__(256) void bgmv_shrink_kernel(T* __restrict__ Y, const T* __restrict__ X,
                                                         const T* __restrict__ W,
                                                         const long long* __restrict__ indices, int h_in, int h_out,
                                                         long num_layers, long layer_idx, float scale) {
  __shared__ float red[4][16];
  const int b = blockIdx.x;
  const long idx = indices[b];
  if (idx < 0) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* w = W + (idx * num_layers + layer_idx) * (long)h_out * h_in;
  const T* x = X + (long)b * h_in;
  for (int oc = 0; oc < h_out; oc += 16) {
    const int n_out = h_out - oc < 16 ? h_out - oc : 16;      // 16, or 8 for the last chunk (h_out is a multiple of 8)
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; j++) acc[j] = 0.f;
    for (int i = threadIdx.x * 8; i < h_in; i += 2048) {
      const lvec8<T> xv = *reinterpret_cast<const lvec8<T>*>(x + i);
      lvec8<T> wv[16];
#pragma unroll
      for (int j = 0; j < 16; j++)   // (rows past the chunk re-read its first row: no branch around a load)
        wv[j] = *reinterpret_cast<const lvec8<T>*>(w + (long)(oc + (j < n_out ? j : 0)) * h_in + i);
#pragma unroll
      for (int j = 0; j < 16; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[j] += (float)wv[j][e] * (float)xv[e];
    }
#pragma unroll
    for (int j = 0; j < 16; j++) {
      const float sum = wave_sum(acc[j]);
      if (lane == 0) red[wave][j] = sum;
    }
    __syncthreads();
    if (threadIdx.x < n_out) {
      const float sum = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
      T* yp = Y + (long)b * h_out + oc + threadIdx.x;
      *yp = (T)((ACC ? (float)*yp : 0.f) + sum * scale);
    }
    __syncthreads();
  }
}

// narrow -> wide: grid (ceil(h_out / 2048), B), block 256.  A thread owns 8 consecutive outputs: their 8 weight rows are
// one contiguous piece of memory (h_in elements each), the token's h_in activations are the same address in every lane,
// and the old outputs are one 16-byte load; everything is requested before the first result is used.
template <class T, bool ACC = true>
__global__ __launch_bounds__(256) void bgmv_expand_kernel(T* __restrict__ Y, const T* __restrict__ X,
                                                         const T* __restrict__ W,
                                                         const long long* __restrict__ indices, int h_in, int h_out,
                                                         long num_layers, long layer_idx, float scale) {
  const int b = blockIdx.y;
  const long idx = indices[b];
  if (idx < 0) return;
  const int j0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (j0 >= h_out) return;
  const T* w = W + ((idx * num_layers + layer_idx) * (long)h_out + j0) * h_in;
  const T* x = X + (long)b * h_in;
  T* yp = Y + (long)b * h_out + j0;
  lvec8<T> old = lvec8<T>{0, 0, 0, 0, 0, 0, 0, 0};
  if (ACC) old = *reinterpret_cast<const lvec8<T>*>(yp);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++) acc[e] = 0.f;
  for (int i = 0; i < h_in; i += 8) {
    const lvec8<T> xv = *reinterpret_cast<const lvec8<T>*>(x + i);
    lvec8<T> wv[8];
#pragma unroll
    for (int e = 0; e < 8; e++) wv[e] = *reinterpret_cast<const lvec8<T>*>(w + (long)e * h_in + i);
#pragma unroll
    for (int e = 0; e < 8; e++)
#pragma unroll
      for (int q = 0; q < 8; q++) acc[e] += (float)wv[e][q] * (float)xv[q];
  }
  lvec8<T> o;
#pragma unroll
  for (int e = 0; e < 8; e++) o[e] = (T)((float)old[e] + acc[e] * scale);
  *reinterpret_cast<lvec8<T>*>(yp) = o;
}

// The same for h_in = 8 LPR with LPR a power of two (h_in = 8 .. 128), written around whole cache lines: a weight row
// (h_in elements) is spread over LPR neighbouring lanes, 8 elements each, so that one load instruction of a wavefront
// covers 1 KB of consecutive memory (64 / LPR rows); with a thread per 8 rows, as above, every load instruction touches
// 64 different lines for 16 bytes each, and the address unit, not memory, bounds the kernel (measured at rank 16:
// 18.5 us for 256 tokens on 11008 outputs).  The LPR partial dot products of a row are added by shuffles; lane 0 of the row
// updates the output.  A block takes TB consecutive tokens; the weights stay in registers from one token to the next
// and are fetched again only when the adapter changes (sorted batches, the hot adapter of a skewed one).
// grid (ceil(h_out / (4 Q 64 / LPR)), ceil(B / TB)), block 256.
template <class T, int LPR, int Q, int TB, bool ACC = true>
__global__ __launch_bounds__(256) void bgmv_expand_lines_kernel(T* __restrict__ Y, const T* __restrict__ X,
                                                               const T* __restrict__ W,
                                                               const long long* __restrict__ indices, int batch, int h_out,
                                                               long num_layers, long layer_idx, float scale) {
  constexpr int h_in = 8 * LPR;
  constexpr int RPL = 64 / LPR;                      // rows per load instruction of a wavefront
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = lane % LPR, rl = lane / LPR;
  const int row0 = (blockIdx.x * 4 + wave) * Q * RPL + rl;
  if ((blockIdx.x * 4 + wave) * Q * RPL >= h_out) return;      // (wave-uniform)
  const int b0 = blockIdx.y * TB;
  long idx[TB];
#pragma unroll
  for (int t = 0; t < TB; t++) idx[t] = indices[b0 + t < batch ? b0 + t : batch - 1];
  lvec8<T> wv[Q];
  long have = -1;
#pragma unroll
  for (int t = 0; t < TB; t++) {
    const int b = b0 + t;
    if (b >= batch || idx[t] < 0) continue;          // (uniform over the block)
    const lvec8<T> xv = *reinterpret_cast<const lvec8<T>*>(X + (long)b * h_in + sub * 8);
    T* yrow = Y + (long)b * h_out;
    T old[Q];
#pragma unroll
    for (int q = 0; q < Q; q++) {                     // (rows past the end re-read the last row; their sums are dropped)
      const int row = row0 + q * RPL < h_out ? row0 + q * RPL : h_out - 1;
      old[q] = ACC ? yrow[row] : (T)0;
    }
    if (idx[t] != have) {
      const T* w = W + (idx[t] * num_layers + layer_idx) * (long)h_out * h_in + sub * 8;
#pragma unroll
      for (int q = 0; q < Q; q++) {
        const int row = row0 + q * RPL < h_out ? row0 + q * RPL : h_out - 1;
        wv[q] = *reinterpret_cast<const lvec8<T>*>(w + (long)row * h_in);
      }
      have = idx[t];
    }
#pragma unroll
    for (int q = 0; q < Q; q++) {
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) acc += (float)wv[q][e] * (float)xv[e];
#pragma unroll
      for (int off = 1; off < LPR; off <<= 1) acc += __shfl_xor(acc, off, 64);
      const int row = row0 + q * RPL;
      if (sub == 0 && row < h_out) yrow[row] = (T)((float)old[q] + acc * scale);
    }
  }
}

// ---------------------------------------------------------------- SGMV ----

template <class T>
struct SgmvArgsT {
  T* y;
  long y_stride;
  const T* x;
  long x_stride;
  int d_in, d_out;
  // weights: pointer per group (w_ptrs) or w_base + adapter * w_stride; layer_off added to either
  const long long* w_ptrs;
  const T* w_base;
  long w_stride;
  long layer_off;
  // groups: indptr `seg` (group g = rows seg[g]..seg[g+1], adapter g), or the
  // routing plan's tile list {adapter, start, count, 0} + perm
  const int* seg;
  const int4* tiles;
  const int* perm;
  const int* n_groups_dev;
  int n_groups;               // blocks along x: segments, or the maximum length of the tile list
  int n_adapters;
  float scale;
  int accumulate;             // 1: y += result (the reference's semantics); 0: y = result, y is not read
};

using SgmvArgs = SgmvArgsT<_Float16>;

template <class T>
struct SgmvGroupT {
  const T* w;
  int start, count;
};

template <class T>
__device__ __forceinline__ bool sgmv_group(const SgmvArgsT<T>& a, int g, SgmvGroupT<T>* out) {
  int adapter, n = a.n_groups;
  if (a.seg) {
    adapter = g;
    out->start = a.seg[g];
    out->count = a.seg[g + 1] - out->start;
  } else {
    // the tile is read together with the tile count (the list is allocated at its maximum
    // length, g is inside it); whether it is a live one is decided afterwards
    const int4 d = a.tiles[g];
    n = *a.n_groups_dev;
    if (g >= n) return false;
    adapter = d.x;
    out->start = d.y;
    out->count = d.z;
  }
  if (out->count <= 0 || adapter < 0 || adapter >= a.n_adapters) return false;
  const T* base = a.w_ptrs ? reinterpret_cast<const T*>(a.w_ptrs[adapter]) : a.w_base + adapter * a.w_stride;
  out->w = base + a.layer_off;
  return true;
}

template <class T>
__device__ __forceinline__ int sgmv_row(const SgmvArgsT<T>& a, int i) { return a.perm ? a.perm[i] : i; }

// The rows of R consecutive list positions (positions past the end of the group repeat `first`).  The list
// entries are requested together and without a branch around the loads (a load under a branch is waited for
// where the branches join: one memory round trip per row); without a list the same loads read the head of
// the activations, which is always there, and their values are dropped.
template <int R, class T>
__device__ __forceinline__ void sgmv_rows(const SgmvArgsT<T>& a, int first, int n_left, int (&rows)[R]) {
  const int* list = a.perm ? a.perm : reinterpret_cast<const int*>(a.x);
  int pos[R], listed[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    pos[r] = first + (r < n_left ? r : 0);
    listed[r] = list[a.perm ? pos[r] : 0];
  }
#pragma unroll
  for (int r = 0; r < R; r++) rows[r] = a.perm ? listed[r] : pos[r];
}

// wide -> narrow (d_out <= DOUT <= 128): grid (n_groups, row slots), block 256; a block takes
// R token rows of its group at a time and walks all of d_in once for them.  With CB = d_out / 8
// column blocks, thread (kp, cb) = (tid / CB, tid % CB) reads the 16-byte pieces [k][cb*8 .. +8] of
// the adapter rows k = 2 kp and 2 kp + 1, then 2 (256 / CB) rows further on, and so on, so that a
// wavefront's loads cover consecutive memory; the matching two activations of a row are one dword.
// Each thread keeps R x 8 partial sums; they are summed over the threads of a column block in two
// passes through LDS (row stride 8 R + 1 floats, so neither pass has bank conflicts worth naming).
template <int DOUT, int R, class T>
__global__ __launch_bounds__(256) void sgmv_shrink_kernel(const SgmvArgsT<T> a) {
  constexpr int V = 8 * R;
  __shared__ float part[256 * (V + 1)];
  __shared__ float part2[256];
  SgmvGroupT<T> g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  const int tid = threadIdx.x;
  const int dn = a.d_out;
  const int CB = dn >> 3;
  const int KP = 256 / CB;               // k pairs per sweep of the block
  const int cb = tid % CB, kp = tid / CB;
  const bool worker = kp < KP;
  // second pass: thread (v, cb2, part) adds every P-th partial of output v of column block cb2
  const int P = 256 / (V * CB);
  const int v2 = tid % V, cb2 = (tid / V) % CB, part_id = tid / (V * CB);
  for (int r0 = blockIdx.y * R; r0 < g.count; r0 += gridDim.y * R) {
    int rows[R];
    const T* xr[R];
    sgmv_rows<R, T>(a, g.start + r0, g.count - r0, rows);
#pragma unroll
    for (int r = 0; r < R; r++) xr[r] = a.x + (long)rows[r] * a.x_stride;
    float acc[R][8];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[r][j] = 0.f;
    if (worker) {
      // U sweeps at a time: their loads are all requested before the first is used (no branch between them:
      // a sweep past the end of K re-reads the batch's first rows and meets zero activations), so a thread
      // has U times the requests in flight and a U-th of the round trips in sequence.  Sums are taken in
      // the order of k, as without the batching, each product added by one fused multiply-add written out (left to the
      // compiler's contraction the two products of a k pair were first added to each other: 256 tokens over 32 adapters of
      // rank 16 on k = 4096 8.5 -> 7.4 us, on k = 11008 15.4 -> 12.7 us).  Requesting the next batch ahead of the sums of
      // the current one (two sets of registers) was measured slower (7.4 -> 8.3 us).
      constexpr int U = TRITEIA_SHRINK_UNROLL;
      const T* wp = g.w + cb * 8;
      const int kstep = 2 * KP;
      for (int k0 = 2 * kp; k0 < a.d_in; k0 += U * kstep) {
        lvec8<T> w0[U], w1[U];
        lvec2<T> xv[U][R];
#pragma unroll
        for (int u = 0; u < U; u++) {
          const int k = k0 + u * kstep;
          const int kc = k < a.d_in ? k : k0;
          w0[u] = load_global(reinterpret_cast<const lvec8<T>*>(wp + (long)kc * dn));
          w1[u] = load_global(reinterpret_cast<const lvec8<T>*>(wp + (long)(kc + 1) * dn));
#pragma unroll
          for (int r = 0; r < R; r++) xv[u][r] = *reinterpret_cast<const lvec2<T>*>(xr[r] + kc);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
          const bool live = k0 + u * kstep < a.d_in;
#pragma unroll
          for (int r = 0; r < R; r++) {
            const float x0 = live ? (float)xv[u][r][0] : 0.f, x1 = live ? (float)xv[u][r][1] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) acc[r][j] = __builtin_fmaf(x1, (float)w1[u][j], __builtin_fmaf(x0, (float)w0[u][j], acc[r][j]));
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int j = 0; j < 8; j++) part[tid * (V + 1) + r * 8 + j] = acc[r][j];
    __syncthreads();
    if (part_id < P) {
      float s = 0.f;
      for (int i = part_id; i < KP; i += P) s += part[(cb2 + CB * i) * (V + 1) + v2];
      part2[tid] = s;
    }
    __syncthreads();
    if (tid < V * CB) {
      float sum = 0.f;
      for (int p = 0; p < P; p++) sum += part2[tid + V * CB * p];
      const int r = v2 >> 3;
      if (r0 + r < g.count) {
        int row = rows[0];
#pragma unroll
        for (int q = 1; q < R; q++) row = r == q ? rows[q] : row;
        T* yp = a.y + (long)row * a.y_stride + cb2 * 8 + (v2 & 7);
        *yp = (T)((a.accumulate ? (float)*yp : 0.f) + sum * a.scale);
      }
    }
  }
}

// narrow -> wide (d_in <= 128): grid (n_groups, ceil(d_out / 256)), block 256;
// each thread keeps its weight column in registers and walks the group's rows.
template <int DIN, class T>
__global__ __launch_bounds__(256) void sgmv_expand_kernel(const SgmvArgsT<T> a) {
  __shared__ float xs[DIN];
  SgmvGroupT<T> g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  const int j = blockIdx.y * 256 + threadIdx.x;
  const bool ok = j < a.d_out;
  float w[DIN];
#pragma unroll
  for (int i = 0; i < DIN; i++) w[i] = (ok && i < a.d_in) ? (float)g.w[(long)i * a.d_out + j] : 0.f;
  for (int rr = blockIdx.z; rr < g.count; rr += gridDim.z) {
    const int row = sgmv_row(a, g.start + rr);
    __syncthreads();
    if (threadIdx.x < DIN) xs[threadIdx.x] = threadIdx.x < a.d_in ? (float)a.x[(long)row * a.x_stride + threadIdx.x] : 0.f;
    __syncthreads();
    if (ok) {
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < DIN; i++) acc += w[i] * xs[i];
      T* yp = a.y + (long)row * a.y_stride + j;
      *yp = (T)((a.accumulate ? (float)*yp : 0.f) + acc * a.scale);
    }
  }
}

// narrow -> wide for d_in <= DIN <= 32: grid (n_groups, ceil(d_out / 2048), row slots), block 256.
// A thread owns 8 consecutive output columns: its d_in x 8 weight patch stays in registers while
// it walks the group's rows R at a time (16-byte loads and stores throughout, no barriers; the R
// rows' loads are independent, so they are in flight together).
template <int DIN, int R, class T, bool ACC = true>
__global__ __launch_bounds__(256) void sgmv_expand_vec_kernel(const SgmvArgsT<T> a) {
  SgmvGroupT<T> g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  const int j0 = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (j0 >= a.d_out) return;
  int r0 = blockIdx.z * R;
  if (r0 >= g.count) return;
  // Order of the requests: the first rows' list entries, then the weight patch, then (once the rows are
  // known) their activations and old outputs; nothing is waited for before all of these are on their way.
  int rows[R];
  sgmv_rows<R, T>(a, g.start + r0, g.count - r0, rows);
  lvec8<T> w[DIN];
#pragma unroll
  for (int i = 0; i < DIN; i++)   // (no branch around a load: rows past d_in re-read the last one and are zeroed below)
    w[i] = load_global(reinterpret_cast<const lvec8<T>*>(g.w + (long)(i < a.d_in ? i : a.d_in - 1) * a.d_out + j0));
  bool patch_ready = false;
  for (;;) {
    lvec8<T> xv[R][DIN / 8], old[R];
    T* yp[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const T* xr = a.x + (long)rows[r] * a.x_stride;
      yp[r] = a.y + (long)rows[r] * a.y_stride + j0;
#pragma unroll
      for (int i0 = 0; i0 < DIN / 8; i0++)
        xv[r][i0] = *reinterpret_cast<const lvec8<T>*>(xr + (i0 * 8 < a.d_in ? i0 * 8 : 0));   // same address in every lane
      old[r] = ACC ? *reinterpret_cast<const lvec8<T>*>(yp[r]) : lvec8<T>{0, 0, 0, 0, 0, 0, 0, 0};
    }
    __builtin_amdgcn_sched_barrier(0);   // every request above is issued before the first result is touched
    if (!patch_ready) {
#pragma unroll
      for (int i = 0; i < DIN; i++)
        if (i >= a.d_in) w[i] = lvec8<T>{0, 0, 0, 0, 0, 0, 0, 0};
      patch_ready = true;
    }
    const int n_left = g.count - r0;
#pragma unroll
    for (int r = 0; r < R; r++) {
      float acc[8];
#pragma unroll
      for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll
      for (int i = 0; i < DIN; i++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = __builtin_fmaf((float)xv[r][i / 8][i % 8], (float)w[i][e], acc[e]);
      lvec8<T> o;
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = (T)__builtin_fmaf(acc[e], a.scale, (float)old[r][e]);
      if (r == 0 || r < n_left) *reinterpret_cast<lvec8<T>*>(yp[r]) = o;
    }
    r0 += gridDim.z * R;
    if (r0 >= g.count) break;
    sgmv_rows<R, T>(a, g.start + r0, g.count - r0, rows);
  }
}

}  // namespace triteia_hip
