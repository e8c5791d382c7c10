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
// The padded output space is a sequence of up to three pieces: piece i takes the next n[i] columns of the partial
// rows and is z[i] >= n[i] elements long, the rest written as zero (a piece with n = 0 is a zero fill).
struct ReduceOut {
  void* out[3];
  int n[3], z[3];
};
template <typename real>
__global__ __launch_bounds__(RED_THREADS) void reduce_partials_kernel(const real* __restrict__ partial, int nblocks,
                                                                      int nout, ReduceOut O) {
  constexpr int EL = 64 / (int)sizeof(real);
  constexpr int PARTS = RED_THREADS / EL;
  constexpr int NWV = RED_THREADS / WAVE;
  __shared__ real sh[NWV][EL];
  const int tid = threadIdx.x;
  const int el = tid % EL, part = tid / EL;
  const int e = blockIdx.x * EL + el;
  // piece and position of element e, column of the partial rows it sums (-1: padding)
  int piece = 0, at = e, col0 = 0;
  while (piece < 2 && at >= O.z[piece]) { at -= O.z[piece]; col0 += O.n[piece]; piece++; }
  const int src = at < O.n[piece] ? col0 + at : -1;
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
    if (at < O.z[piece]) ((real*)O.out[piece])[at] = t;
  }
}

// tmp is not used (callers reserve it with their partial rows).
template <typename real>
inline void launch_reduce_partials(const real* partial, int nblocks, int nout, real* out0, int n0, int z0, real* out1,
                                   int n1, int z1, real* tmp, hipStream_t stream, real* out2 = nullptr, int n2 = 0,
                                   int z2 = 0) {
  (void)tmp;
  constexpr int EL = 64 / (int)sizeof(real);
  const int etot = z0 + z1 + z2;
  ReduceOut O;
  O.out[0] = out0; O.n[0] = n0; O.z[0] = z0;
  O.out[1] = out1; O.n[1] = n1; O.z[1] = z1;
  O.out[2] = out2; O.n[2] = n2; O.z[2] = z2;
  hipLaunchKernelGGL(reduce_partials_kernel<real>, dim3((etot + EL - 1) / EL), dim3(RED_THREADS), 0, stream, partial,
                     nblocks, nout, O);
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
