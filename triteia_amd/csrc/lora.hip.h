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

namespace triteia_hip {

typedef _Float16 lhalf8_t __attribute__((ext_vector_type(8)));

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
  const int4* tiles2;         // second tile list (the plan's wide tiles), after the first
  const int* perm;
  const int* n_groups_dev;
  const int* n_groups2_dev;
  int n_groups;
  int n_adapters;
  float scale;
};

struct SgmvGroup {
  const _Float16* w;
  int start, count;
};

__device__ __forceinline__ bool sgmv_group(const SgmvArgs& a, int g, SgmvGroup* out) {
  const int n = a.n_groups_dev ? *a.n_groups_dev : a.n_groups;
  const int n2 = a.n_groups2_dev ? *a.n_groups2_dev : 0;
  if (g >= n + n2) return false;
  int adapter;
  if (a.seg) {
    adapter = g;
    out->start = a.seg[g];
    out->count = a.seg[g + 1] - a.seg[g];
  } else {
    const int4 d = g < n ? a.tiles[g] : a.tiles2[g - n];
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

// wide -> narrow (d_out <= DOUT <= 128): grid (n_groups, row slots), block 256; a block computes
// one token row at a time.  Thread j takes the 8-row slabs j, j + 256, ... of the adapter matrix
// (8 * d_out consecutive halfs, so a wavefront reads 64 slabs back to back) against 8 activations,
// keeping d_out partial sums; the 256 partial vectors are then summed by shuffles and LDS.
template <int DOUT>
__global__ __launch_bounds__(256) void sgmv_shrink_kernel(const SgmvArgs a) {
  __shared__ float part[4][DOUT];
  SgmvGroup g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int dn = a.d_out;
  for (int rr = blockIdx.y; rr < g.count; rr += gridDim.y) {
    const int row = sgmv_row(a, g.start + rr);
    const _Float16* x = a.x + (long)row * a.x_stride;
    float acc[DOUT];
#pragma unroll
    for (int j = 0; j < DOUT; j++) acc[j] = 0.f;
    for (int k0 = tid * 8; k0 < a.d_in; k0 += 256 * 8) {
      const lhalf8_t xv = *reinterpret_cast<const lhalf8_t*>(x + k0);
      const _Float16* wk = g.w + (long)k0 * dn;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float xe = (float)xv[e];
#pragma unroll
        for (int j0 = 0; j0 < DOUT; j0 += 8) {
          if (j0 < dn) {
            const lhalf8_t wv = *reinterpret_cast<const lhalf8_t*>(wk + (long)e * dn + j0);
#pragma unroll
            for (int j = 0; j < 8; j++) acc[j0 + j] += xe * (float)wv[j];
          }
        }
      }
    }
#pragma unroll
    for (int j = 0; j < DOUT; j++) {
      const float v = wave_sum(acc[j]);
      if (lane == 0) part[wave][j] = v;
    }
    __syncthreads();
    if (tid < dn) {
      const float sum = part[0][tid] + part[1][tid] + part[2][tid] + part[3][tid];
      _Float16* yp = a.y + (long)row * a.y_stride + tid;
      *yp = (_Float16)((float)*yp + sum * a.scale);
    }
    __syncthreads();
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
// it walks the group's rows (16-byte loads and stores throughout, no barriers).
template <int DIN>
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
  for (int rr = blockIdx.z; rr < g.count; rr += gridDim.z) {
    const int row = sgmv_row(a, g.start + rr);
    const _Float16* xr = a.x + (long)row * a.x_stride;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll
    for (int i0 = 0; i0 < DIN; i0 += 8) {
      if (i0 < a.d_in) {
        const lhalf8_t xv = *reinterpret_cast<const lhalf8_t*>(xr + i0);   // same address in every lane
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
          for (int e = 0; e < 8; e++) acc[e] += (float)xv[i] * (float)w[i0 + i][e];
      }
    }
    _Float16* yp = a.y + (long)row * a.y_stride + j0;
    const lhalf8_t old = *reinterpret_cast<const lhalf8_t*>(yp);
    lhalf8_t o;
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = (_Float16)((float)old[e] + acc[e] * a.scale);
    *reinterpret_cast<lhalf8_t*>(yp) = o;
  }
}

}  // namespace triteia_hip
