// SGMV on the matrix cores of gfx950, for adapters of rank 32, 64 or 128 (and the shrink at rank 16): the form the
// reference's SGMV has (a tensor-core grouped GEMM, triteia/csrc/ops/sgmv.cuh:84-125,129-171), next to the VALU kernels
// of lora.hip.h, which stay for other ranks and for the shapes these kernels do not take.
//
//   y[rows of group g] (+)= scale * x[rows of group g] @ W_g,   W_g row-major [d_in, d_out]
//
// Both kernels compute the transposed product out^T = W^T x^T with V_MFMA_F32_16X16X32_{F16,BF16}:
//   A operand (16 rows x 32 k)  = W^T: row i = output column, lane (i, kq) holds W[k0 + 8 kq + t][n0 + i], t = 0..7
//   B operand (32 k x 16 cols)  = x^T: column j = token, lane (j, kq) holds x[token j][k0 + 8 kq .. + 7]
//   D (16 x 16)                 : lane (j, q) holds output columns n0 + 4 q .. + 3 of token j
// x is read straight from global memory (16 contiguous bytes per lane); so is the result (8 contiguous bytes per
// lane).  W is row-major with the output column as the fast index, i.e. strided in k: a tile of it is copied to LDS
// as it lies in memory and the A operands are gathered from there, eight 2-byte reads per operand, with a row stride
// that sends the four k-groups of a read to different banks.
// The contraction pairs slot (kq, t) of A with slot (kq, t) of B whatever k the hardware gives that slot, so the
// only layout fact the code depends on is D's (measured for the sparse instruction of the same shape).
//
// Shrink (d_in long, d_out = rank): the four wavefronts of a workgroup split K (steps of 32, two in flight in
// registers), each copying its own steps of W through its own LDS slab, and add their sums in a fixed order at the end.
// Expand (d_in = rank, d_out long): a workgroup copies the adapter's [rank x 128 columns] once, every wavefront keeps the
// A operands of its 32 columns in registers and walks the group's token tiles.
#pragma once
#include "lora.hip.h"

namespace triteia_hip {

typedef float lm_float4 __attribute__((ext_vector_type(4)));

template <class T> struct LoraMfma;
template <> struct LoraMfma<_Float16> {
  typedef _Float16 v8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ lm_float4 run(v8 a, v8 b, lm_float4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};
template <> struct LoraMfma<__bf16> {
  typedef __bf16 v8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ lm_float4 run(v8 a, v8 b, lm_float4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};

template <class T> using lvec4 = T __attribute__((ext_vector_type(4)));

// row of list position first + j of a group; positions past the group's `n_left` remaining ones (a tile past the end
// has none) stand for the group's first row, `fallback`: always a valid one, and their results are dropped
template <class T>
__device__ __forceinline__ int lm_row(const SgmvArgsT<T>& a, int first, int j, int n_left, int fallback) {
  const int pos = j < n_left ? first + j : fallback;
  return a.perm ? a.perm[pos] : pos;
}

// ---- shrink: grid (groups, token chunks), block 256.  R16 = d_out / 16 (1, 2, 4 or 8), TT = 16-token tiles per pass.
template <class T, int R16, int TT>
__global__ __launch_bounds__(256) void sgmv_shrink_mfma_kernel(const SgmvArgsT<T> a) {
  typedef typename LoraMfma<T>::v8 v8;
  constexpr int R = 16 * R16;
  constexpr int LDW = R + 4;                       // elements per staged row: an 8-byte aligned stride of 2 (mod 8) dwords,
                                                   // so that the four k-groups of a gather fall into four different quarters of the banks
  constexpr int kStageBytes = 4 * 32 * LDW * 2;    // four wavefronts' slabs
  constexpr int kRedBytes = 3 * TT * R16 * 1024;   // the sums of wavefronts 1..3
  __shared__ __attribute__((aligned(16))) unsigned char smem[kStageBytes > kRedBytes ? kStageBytes : kRedBytes];
  SgmvGroupT<T> g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int j = lane & 15, kq = lane >> 4;
  T* const slab = reinterpret_cast<T*>(smem) + wave * 32 * LDW;
  const int nsteps = a.d_in >> 5;                  // (the launcher sends d_in % 32 != 0 elsewhere)

  struct Frag {
    lvec8<T> w[R16];      // this lane's 16-byte pieces of the step's 32 x R tile of W (piece lane + 64 i of 4 R)
    lvec8<T> x[TT];       // B operands
  };
  for (int r0 = blockIdx.y * 16 * TT; r0 < g.count; r0 += gridDim.y * 16 * TT) {
    int rows[TT];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) rows[tt] = lm_row(a, g.start + r0 + 16 * tt, j, g.count - r0 - 16 * tt, g.start);
    const T* xr[TT];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) xr[tt] = a.x + (long)rows[tt] * a.x_stride + 8 * kq;
    auto load = [&](Frag& f, int ks) {
      const int k0 = (ks < nsteps ? ks : nsteps - 1) << 5;        // past the end: the last step again (never multiplied)
      const T* wp = g.w + (long)k0 * R + lane * 8;                 // the step's tile is 32 R consecutive elements
#pragma unroll
      for (int i = 0; i < R16; i++) f.w[i] = load_global(reinterpret_cast<const lvec8<T>*>(wp + 512 * i));
#pragma unroll
      for (int tt = 0; tt < TT; tt++) f.x[tt] = *reinterpret_cast<const lvec8<T>*>(xr[tt] + k0);
    };
    lm_float4 acc[R16][TT];
#pragma unroll
    for (int rt = 0; rt < R16; rt++)
#pragma unroll
      for (int tt = 0; tt < TT; tt++) acc[rt][tt] = lm_float4{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const Frag& f) {
      // the tile of W to this wavefront's slab, as it lies in memory (row = piece / (R / 8))
#pragma unroll
      for (int i = 0; i < R16; i++) {
        const int piece = lane + 64 * i;
        T* dst = slab + (piece / (R / 8)) * LDW + (piece % (R / 8)) * 8;
        const lvec4<T> lo = {f.w[i][0], f.w[i][1], f.w[i][2], f.w[i][3]}, hi = {f.w[i][4], f.w[i][5], f.w[i][6], f.w[i][7]};
        *reinterpret_cast<lvec4<T>*>(dst) = lo;
        *reinterpret_cast<lvec4<T>*>(dst + 4) = hi;
      }
#pragma unroll
      for (int rt = 0; rt < R16; rt++) {
        v8 A;
#pragma unroll
        for (int t = 0; t < 8; t++) A[t] = slab[(8 * kq + t) * LDW + 16 * rt + j];
#pragma unroll
        for (int tt = 0; tt < TT; tt++) acc[rt][tt] = LoraMfma<T>::run(A, f.x[tt], acc[rt][tt]);
      }
    };
    Frag ring[2];
    load(ring[0], wave);
    load(ring[1], wave + 4);
    for (int ks = wave; ks < nsteps; ks += 8) {
#pragma unroll
      for (int b = 0; b < 2; b++) {
        if (ks + 4 * b < nsteps) multiply(ring[b]);
        load(ring[b], ks + 4 * b + 8);
      }
    }
    // the four wavefronts' sums, added in the order of the wavefronts
    __syncthreads();      // every slab has been read for the last time
    lm_float4* red = reinterpret_cast<lm_float4*>(smem);
    if (wave > 0) {
#pragma unroll
      for (int rt = 0; rt < R16; rt++)
#pragma unroll
        for (int tt = 0; tt < TT; tt++) red[(((wave - 1) * TT + tt) * R16 + rt) * 64 + lane] = acc[rt][tt];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int tt = 0; tt < TT; tt++) {
        if (r0 + 16 * tt + j >= g.count) continue;
        T* yp = a.y + (long)rows[tt] * a.y_stride + 4 * kq;
        lvec4<T> old[R16];
#pragma unroll
        for (int rt = 0; rt < R16; rt++) old[rt] = lvec4<T>{0, 0, 0, 0};
        if (a.accumulate) {
#pragma unroll
          for (int rt = 0; rt < R16; rt++) old[rt] = *reinterpret_cast<const lvec4<T>*>(yp + 16 * rt);
        }
#pragma unroll
        for (int rt = 0; rt < R16; rt++) {
          lm_float4 s = acc[rt][tt];
#pragma unroll
          for (int w = 0; w < 3; w++) {
            const lm_float4 o = red[((w * TT + tt) * R16 + rt) * 64 + lane];
#pragma unroll
            for (int e = 0; e < 4; e++) s[e] += o[e];
          }
          lvec4<T> out;
#pragma unroll
          for (int e = 0; e < 4; e++) out[e] = (T)((float)old[rt][e] + s[e] * a.scale);
          *reinterpret_cast<lvec4<T>*>(yp + 16 * rt) = out;
        }
      }
    }
    __syncthreads();      // the next pass stages into the same memory
  }
}

// ---- expand: grid (groups, ceil(d_out / 128), token-tile slots), block 256.  KS = d_in / 32 (1, 2 or 4).
template <class T, int KS>
__global__ __launch_bounds__(256) void sgmv_expand_mfma_kernel(const SgmvArgsT<T> a) {
  typedef typename LoraMfma<T>::v8 v8;
  constexpr int RK = 32 * KS;
  constexpr int LDW = 128 + 4;
  __shared__ __attribute__((aligned(16))) T wl[RK * LDW];   // (rows are 8-byte aligned)
  SgmvGroupT<T> g;
  if (!sgmv_group(a, blockIdx.x, &g)) return;
  if ((int)blockIdx.z * 16 >= g.count) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int j = lane & 15, kq = lane >> 4;
  const int c0 = blockIdx.y * 128;
  // the adapter's [rank x 128 columns] to LDS (columns past d_out: zeros)
#pragma unroll
  for (int i = 0; i < RK / 16; i++) {
    const int piece = tid + 256 * i, row = piece >> 4, c8 = piece & 15;
    const int col = c0 + 8 * c8;
    lvec8<T> v = lvec8<T>{0, 0, 0, 0, 0, 0, 0, 0};
    const lvec8<T> w = load_global(reinterpret_cast<const lvec8<T>*>(g.w + (long)row * a.d_out + (col < a.d_out ? col : 0)));
    if (col < a.d_out) v = w;
    const lvec4<T> lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
    *reinterpret_cast<lvec4<T>*>(wl + row * LDW + 8 * c8) = lo;
    *reinterpret_cast<lvec4<T>*>(wl + row * LDW + 8 * c8 + 4) = hi;
  }
  __syncthreads();
  v8 A[2][KS];
#pragma unroll
  for (int nt = 0; nt < 2; nt++)
#pragma unroll
    for (int ks = 0; ks < KS; ks++)
#pragma unroll
      for (int t = 0; t < 8; t++) A[nt][ks][t] = wl[(32 * ks + 8 * kq + t) * LDW + 32 * wave + 16 * nt + j];
  const int col = c0 + 32 * wave + 4 * kq;          // this lane's first output column (tile nt: + 16 nt)
  for (int tile = blockIdx.z; tile * 16 < g.count; tile += gridDim.z) {
    const int n_left = g.count - 16 * tile;
    const int row = lm_row(a, g.start + 16 * tile, j, n_left, g.start);
    const T* xr = a.x + (long)row * a.x_stride + 8 * kq;
    T* yp = a.y + (long)row * a.y_stride + col;
    v8 B[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) B[ks] = *reinterpret_cast<const v8*>(xr + 32 * ks);
    lvec4<T> old[2];
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
      old[nt] = lvec4<T>{0, 0, 0, 0};
      // (a column group of four lies wholly inside or outside d_out, which is a multiple of 8)
      if (a.accumulate) old[nt] = *reinterpret_cast<const lvec4<T>*>(col + 16 * nt < a.d_out ? yp + 16 * nt : yp - col);
    }
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
      lm_float4 s = lm_float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ks++) s = LoraMfma<T>::run(A[nt][ks], B[ks], s);
      lvec4<T> out;
#pragma unroll
      for (int e = 0; e < 4; e++) out[e] = (T)((float)old[nt][e] + s[e] * a.scale);
      if (j < n_left && col + 16 * nt < a.d_out) *reinterpret_cast<lvec4<T>*>(yp + 16 * nt) = out;
    }
  }
}

}  // namespace triteia_hip
