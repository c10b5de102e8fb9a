// LoRA matrix-vector kernels for gfx950: BGMV (one adapter per token) and SGMV
// (one adapter per segment / group of tokens).  fp16 in, fp32 accumulate,
// fp16 read-modify-write of y.
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
#define TRITEIA_SHRINK_UNROLL 8
#endif

namespace triteia_hip {

typedef _Float16 lhalf8_t __attribute__((ext_vector_type(8)));
typedef _Float16 lhalf2_t __attribute__((ext_vector_type(2)));

constexpr int kLoraMaxNarrow = 128;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// ---------------------------------------------------------------- BGMV ----

// wide -> narrow: grid (B), block 256.  Wave w computes outputs j = w, w+4, ...
__global__ __launch_bounds__(256) void bgmv_shrink_kernel(_Float16* __restrict__ Y, const _Float16* __restrict__ X,
                                                         const _Float16* __restrict__ W,
                                                         const long long* __restrict__ indices, int h_in, int h_out,
                                                         long num_layers, long layer_idx, float scale) {
  const int b = blockIdx.x;
  const long idx = indices[b];
  if (idx < 0) return;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const _Float16* w = W + (idx * num_layers + layer_idx) * (long)h_out * h_in;
  const _Float16* x = X + (long)b * h_in;
  for (int j = wave; j < h_out; j += 4) {
    const _Float16* wj = w + (long)j * h_in;
    float acc = 0.f;
    for (int i = lane * 8; i < h_in; i += 512) {
      const lhalf8_t wv = *reinterpret_cast<const lhalf8_t*>(wj + i);
      const lhalf8_t xv = *reinterpret_cast<const lhalf8_t*>(x + i);
#pragma unroll
      for (int e = 0; e < 8; e++) acc += (float)wv[e] * (float)xv[e];
    }
    acc = wave_sum(acc) * scale;
    if (lane == 0) Y[(long)b * h_out + j] = (_Float16)((float)Y[(long)b * h_out + j] + acc);
  }
}

// narrow -> wide: grid (ceil(h_out / 256), B), block 256, one output per thread
__global__ __launch_bounds__(256) void bgmv_expand_kernel(_Float16* __restrict__ Y, const _Float16* __restrict__ X,
                                                         const _Float16* __restrict__ W,
                                                         const long long* __restrict__ indices, int h_in, int h_out,
                                                         long num_layers, long layer_idx, float scale) {
  __shared__ float xs[kLoraMaxNarrow];
  const int b = blockIdx.y;
  const long idx = indices[b];
  if (idx < 0) return;
  if (threadIdx.x < h_in) xs[threadIdx.x] = (float)X[(long)b * h_in + threadIdx.x];
  __syncthreads();
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= h_out) return;
  const _Float16* wj = W + ((idx * num_layers + layer_idx) * (long)h_out + j) * h_in;
  float acc = 0.f;
  for (int i = 0; i < h_in; i += 8) {
    const lhalf8_t wv = *reinterpret_cast<const lhalf8_t*>(wj + i);
#pragma unroll
    for (int e = 0; e < 8; e++) acc += (float)wv[e] * xs[i + e];
  }
  _Float16* yp = Y + (long)b * h_out + j;
  *yp = (_Float16)((float)*yp + acc * scale);
}

// ---------------------------------------------------------------- SGMV ----

struct SgmvArgs {
  _Float16* y;
  long y_stride;
  const _Float16* x;
  long x_stride;
  int d_in, d_out;
  // weights: pointer per group (w_ptrs) or w_base + adapter * w_stride; layer_off added to either
  const long long* w_ptrs;
  const _Float16* w_base;
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
};

struct SgmvGroup {
  const _Float16* w;
  int start, count;
};

__device__ __forceinline__ bool sgmv_group(const SgmvArgs& a, int g, SgmvGroup* out) {
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
  const _Float16* base = a.w_ptrs ? reinterpret_cast<const _Float16*>(a.w_ptrs[adapter]) : a.w_base + adapter * a.w_stride;
  out->w = base + a.layer_off;
  return true;
}

__device__ __forceinline__ int sgmv_row(const SgmvArgs& a, int i) { return a.perm ? a.perm[i] : i; }

// wide -> narrow (d_out <= DOUT <= 128): grid (n_groups, row slots), block 256; a block takes
// R token rows of its group at a time and walks all of d_in once for them.  With CB = d_out / 8
// column blocks, thread (kp, cb) = (tid / CB, tid % CB) reads the 16-byte pieces [k][cb*8 .. +8] of
// the adapter rows k = 2 kp and 2 kp + 1, then 2 (256 / CB) rows further on, and so on, so that a
// wavefront's loads cover consecutive memory; the matching two activations of a row are one dword.
// Each thread keeps R x 8 partial sums; they are summed over the threads of a column block in two
// passes through LDS (row stride 8 R + 1 floats, so neither pass has bank conflicts worth naming).
template <int DOUT, int R>
__global__ __launch_bounds__(256) void sgmv_shrink_kernel(const SgmvArgs a) {
  constexpr int V = 8 * R;
  __shared__ float part[256 * (V + 1)];
  __shared__ float part2[256];
  SgmvGroup g;
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
    const _Float16* xr[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      rows[r] = sgmv_row(a, g.start + (r0 + r < g.count ? r0 + r : r0));
      xr[r] = a.x + (long)rows[r] * a.x_stride;
    }
    float acc[R][8];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
      for (int j = 0; j < 8; j++) acc[r][j] = 0.f;
    if (worker) {
      const _Float16* wp = g.w + cb * 8;
#pragma unroll TRITEIA_SHRINK_UNROLL
      for (int k = 2 * kp; k < a.d_in; k += 2 * KP) {
        const lhalf8_t w0 = *reinterpret_cast<const lhalf8_t*>(wp + (long)k * dn);
        const lhalf8_t w1 = *reinterpret_cast<const lhalf8_t*>(wp + (long)(k + 1) * dn);
#pragma unroll
        for (int r = 0; r < R; r++) {
          const lhalf2_t xv = *reinterpret_cast<const lhalf2_t*>(xr[r] + k);
          const float x0 = (float)xv[0], x1 = (float)xv[1];
#pragma unroll
          for (int j = 0; j < 8; j++) acc[r][j] += x0 * (float)w0[j] + x1 * (float)w1[j];
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
        _Float16* yp = a.y + (long)row * a.y_stride + cb2 * 8 + (v2 & 7);
        *yp = (_Float16)((float)*yp + sum * a.scale);
      }
    }
  }
}

// narrow -> wide (d_in <= 128): grid (n_groups, ceil(d_out / 256)), block 256;
// each thread keeps its weight column in registers and walks the group's rows.
template <int DIN>
__global__ __launch_bounds__(256) void sgmv_expand_kernel(const SgmvArgs a) {
  __shared__ float xs[DIN];
  SgmvGroup g;
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
      _Float16* yp = a.y + (long)row * a.y_stride + j;
      *yp = (_Float16)((float)*yp + acc * a.scale);
    }
  }
}

// narrow -> wide for d_in <= DIN <= 32: grid (n_groups, ceil(d_out / 2048), row slots), block 256.
// A thread owns 8 consecutive output columns: its d_in x 8 weight patch stays in registers while
// it walks the group's rows R at a time (16-byte loads and stores throughout, no barriers; the R
// rows' loads are independent, so they are in flight together).
template <int DIN, int R>
__global__ __launch_bounds__(256) void sgmv_expand_vec_kernel(const SgmvArgs a) {
  SgmvGroup g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  const int j0 = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (j0 >= a.d_out) return;
  lhalf8_t w[DIN];
#pragma unroll
  for (int i = 0; i < DIN; i++) {
    if (i < a.d_in) w[i] = *reinterpret_cast<const lhalf8_t*>(g.w + (long)i * a.d_out + j0);
    else w[i] = lhalf8_t{0, 0, 0, 0, 0, 0, 0, 0};
  }
  for (int r0 = blockIdx.z * R; r0 < g.count; r0 += gridDim.z * R) {
    lhalf8_t xv[R][DIN / 8], old[R];
    _Float16* yp[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const int row = sgmv_row(a, g.start + (r0 + r < g.count ? r0 + r : r0));
      const _Float16* xr = a.x + (long)row * a.x_stride;
      yp[r] = a.y + (long)row * a.y_stride + j0;
#pragma unroll
      for (int i0 = 0; i0 < DIN / 8; i0++)
        xv[r][i0] = i0 * 8 < a.d_in ? *reinterpret_cast<const lhalf8_t*>(xr + i0 * 8)   // same address in every lane
                                    : lhalf8_t{0, 0, 0, 0, 0, 0, 0, 0};
      old[r] = *reinterpret_cast<const lhalf8_t*>(yp[r]);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
      float acc[8];
#pragma unroll
      for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll
      for (int i = 0; i < DIN; i++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] += (float)xv[r][i / 8][i % 8] * (float)w[i][e];
      lhalf8_t o;
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = (_Float16)((float)old[r][e] + acc[e] * a.scale);
      if (r == 0 || r0 + r < g.count) *reinterpret_cast<lhalf8_t*>(yp[r]) = o;
    }
  }
}

}  // namespace triteia_hip
