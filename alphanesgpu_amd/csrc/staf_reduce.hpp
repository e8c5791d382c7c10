// Second pass of every parameter-gradient op and small fills.
#pragma once
#include "staf_common.hpp"

namespace staf {

constexpr int RED_ELEMS = 8;    // output elements per block
constexpr int RED_PARTS = 32;   // threads that share one output element

// out[e] = sum over the nblocks workgroup partials partial[g*nout + e].  The
// order is fixed: thread `part` adds blocks part, part+32, ... in ascending
// order, then the 32 part sums are added in ascending order -- independent of
// scheduling, so the result is bit-reproducible.  out0 receives the first n0
// elements, out1 (may be null) the next n1.
template <typename real>
__global__ __launch_bounds__(RED_ELEMS* RED_PARTS) void reduce_partials_kernel(const real* __restrict__ partial,
                                                                                int nblocks, int nout, real* out0,
                                                                                int n0, real* out1, int n1) {
  __shared__ real sh[RED_ELEMS][RED_PARTS + 1];
  const int el = threadIdx.x % RED_ELEMS;
  const int part = threadIdx.x / RED_ELEMS;
  const int e = blockIdx.x * RED_ELEMS + el;
  real s = 0;
  if (e < nout)
    for (int g = part; g < nblocks; g += RED_PARTS) s += partial[(size_t)g * nout + e];
  sh[el][part] = s;
  __syncthreads();
  if (part == 0 && e < nout) {
    real t = 0;
#pragma unroll
    for (int p = 0; p < RED_PARTS; p++) t += sh[el][p];
    if (e < n0) out0[e] = t;
    else if (out1 && e - n0 < n1) out1[e - n0] = t;
  }
}

template <typename real>
inline void launch_reduce_partials(const real* partial, int nblocks, int nout, real* out0, int n0, real* out1, int n1,
                                   hipStream_t stream) {
  hipLaunchKernelGGL(reduce_partials_kernel<real>, dim3((nout + RED_ELEMS - 1) / RED_ELEMS),
                     dim3(RED_ELEMS * RED_PARTS), 0, stream, partial, nblocks, nout, out0, n0, out1, n1);
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
