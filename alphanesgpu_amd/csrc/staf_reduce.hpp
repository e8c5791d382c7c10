// Second pass of every parameter-gradient op and small fills.
#pragma once
#include "staf_common.hpp"

namespace staf {

constexpr int RED_ELEMS = 32;   // consecutive output elements per block (one coalesced row segment)
constexpr int RED_PARTS = 8;    // threads that share one output element
constexpr int RED_SLICES = 32;  // row slices of the first pass when there are many partial rows

// Sums workgroup partials partial[g*nout + e] over the rows g of this block's slice (blockIdx.y), in a fixed
// order: thread `part` adds rows part, part+8, ... of the slice in ascending order, then the 8 part sums are
// added in ascending order -- independent of scheduling, so the result is bit-reproducible.
// FINAL = false: the slice sums go to tmp[slice*nout + e].
// FINAL = true: element e < n0 goes to out0[e], element n0 <= e < n0+n1 to out1[e-n0]; out0 is padded with zeros
// up to z0 elements and out1 up to z1 (z0 >= n0, z1 >= n1; out1 may be null when z1 == 0).
template <typename real, bool FINAL>
__global__ __launch_bounds__(RED_ELEMS* RED_PARTS) void reduce_partials_kernel(const real* __restrict__ partial,
                                                                                int nblocks, int rows_per_slice,
                                                                                int nout, real* out0, int n0, int z0,
                                                                                real* out1, int n1, int z1) {
  __shared__ real sh[RED_PARTS][RED_ELEMS];
  const int el = threadIdx.x % RED_ELEMS;
  const int part = threadIdx.x / RED_ELEMS;
  const int e = blockIdx.x * RED_ELEMS + el;
  // FINAL indexes the padded output space: [0, z0) -> out0, [z0, z0+z1) -> out1
  int src = e;
  if (FINAL) src = e < z0 ? (e < n0 ? e : -1) : ((e - z0) < n1 ? n0 + (e - z0) : -1);
  const int g0 = blockIdx.y * rows_per_slice;
  const int g1 = (g0 + rows_per_slice) < nblocks ? (g0 + rows_per_slice) : nblocks;
  real s = 0;
  if (src >= 0 && src < nout) {
    int g = g0 + part;
    for (; g + 7 * RED_PARTS < g1; g += 8 * RED_PARTS) {
      real v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = partial[(size_t)(g + u * RED_PARTS) * nout + src];
#pragma unroll
      for (int u = 0; u < 8; u++) s += v[u];
    }
    for (; g < g1; g += RED_PARTS) s += partial[(size_t)g * nout + src];
  }
  sh[part][el] = s;
  __syncthreads();
  if (part == 0) {
    real t = 0;
#pragma unroll
    for (int p = 0; p < RED_PARTS; p++) t += sh[p][el];
    if (!FINAL) {
      if (e < nout) out0[(size_t)blockIdx.y * nout + e] = t;
    } else if (e < z0) {
      out0[e] = t;
    } else if (e - z0 < z1) {
      out1[e - z0] = t;
    }
  }
}

// tmp: RED_SLICES * nout reals of scratch for the first pass (may be null: single pass).
template <typename real>
inline void launch_reduce_partials(const real* partial, int nblocks, int nout, real* out0, int n0, int z0, real* out1,
                                   int n1, int z1, real* tmp, hipStream_t stream) {
  const real* src = partial;
  int rows = nblocks;
  if (tmp && nblocks > 8 * RED_SLICES) {
    const int per = (nblocks + RED_SLICES - 1) / RED_SLICES;
    hipLaunchKernelGGL((reduce_partials_kernel<real, false>), dim3((nout + RED_ELEMS - 1) / RED_ELEMS, RED_SLICES),
                       dim3(RED_ELEMS * RED_PARTS), 0, stream, partial, nblocks, per, nout, tmp, 0, 0, (real*)nullptr,
                       0, 0);
    src = tmp;
    rows = RED_SLICES;
  }
  const int etot = z0 + z1;
  hipLaunchKernelGGL((reduce_partials_kernel<real, true>), dim3((etot + RED_ELEMS - 1) / RED_ELEMS, 1),
                     dim3(RED_ELEMS * RED_PARTS), 0, stream, src, rows, rows, nout, out0, n0, z0, out1, n1, z1);
}

template <typename real>
__global__ void fill_zero_kernel(real* p, int n) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < n) p[e] = 0;
}

template <typename real>
inline void launch_fill_zero(real* p, int n, hipStream_t stream) {
  if (n > 0) hipLaunchKernelGGL(fill_zero_kernel<real>, dim3((n + 255) / 256), dim3(256), 0, stream, p, n);
}

}  // namespace staf
