// Second pass of every parameter-gradient op and small fills.
#pragma once
#include "staf_common.hpp"

namespace staf {

constexpr int RED_THREADS = 256;   // larger workgroups wait for a whole CU to drain when other kernels share the GPU
constexpr int RED_SLICES = 32;  // rows callers still reserve behind their partial rows (the reduction no longer uses them)

// Sums workgroup partials partial[g*nout + e] over all rows g in one launch and a fixed order, so the result is
// bit-reproducible.  A workgroup owns one 64-byte segment of the output row (8 doubles / 16 floats: whole memory
// sectors of every partial row); thread (part, el) adds rows part, part+PARTS, ... in ascending order, the parts
// of a wavefront are combined by a butterfly over the lane bits above the element index, the four wavefronts'
// sums in ascending order by the first lanes.  One launch instead of a sliced first pass and a final one: the
// partial rows are a few MB and a segment's column a few hundred KB, which one CU reads in the time a launch costs.
// Element e of the padded output space [0, z0) -> out0, [z0, z0+z1) -> out1: e < n0 takes column e, z0 <= e < z0+n1
// column n0 + (e - z0), the rest is written as zero (z0 >= n0, z1 >= n1; out1 may be null when z1 == 0).
template <typename real>
__global__ __launch_bounds__(RED_THREADS) void reduce_partials_kernel(const real* __restrict__ partial, int nblocks,
                                                                      int nout, real* out0, int n0, int z0, real* out1,
                                                                      int n1, int z1) {
  constexpr int EL = 64 / (int)sizeof(real);
  constexpr int PARTS = RED_THREADS / EL;
  constexpr int NWV = RED_THREADS / WAVE;
  __shared__ real sh[NWV][EL];
  const int tid = threadIdx.x;
  const int el = tid % EL, part = tid / EL;
  const int e = blockIdx.x * EL + el;
  const int src = e < z0 ? (e < n0 ? e : -1) : ((e - z0) < n1 ? n0 + (e - z0) : -1);
  real s = 0;
  if (src >= 0 && src < nout) {
    int g = part;
    for (; g + 7 * PARTS < nblocks; g += 8 * PARTS) {
      real v[8];
#pragma unroll
      for (int u = 0; u < 8; u++) v[u] = partial[(size_t)(g + u * PARTS) * nout + src];
#pragma unroll
      for (int u = 0; u < 8; u++) s += v[u];
    }
    for (; g < nblocks; g += PARTS) s += partial[(size_t)g * nout + src];
  }
#pragma unroll
  for (int d = EL; d < WAVE; d <<= 1) s += __shfl_xor(s, d, WAVE);
  if ((tid & (WAVE - 1)) < EL) sh[tid / WAVE][el] = s;
  __syncthreads();
  if (tid < EL) {
    real t = 0;
#pragma unroll
    for (int w = 0; w < NWV; w++) t += sh[w][tid];
    if (e < z0) out0[e] = t;
    else if (e - z0 < z1) out1[e - z0] = t;
  }
}

// tmp is not used (callers reserve it with their partial rows).
template <typename real>
inline void launch_reduce_partials(const real* partial, int nblocks, int nout, real* out0, int n0, int z0, real* out1,
                                   int n1, int z1, real* tmp, hipStream_t stream) {
  (void)tmp;
  constexpr int EL = 64 / (int)sizeof(real);
  const int etot = z0 + z1;
  hipLaunchKernelGGL(reduce_partials_kernel<real>, dim3((etot + EL - 1) / EL), dim3(RED_THREADS), 0, stream, partial,
                     nblocks, nout, out0, n0, z0, out1, n1, z1);
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
