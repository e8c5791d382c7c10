// 2-body fingerprints of one centre by one wavefront:
//   AF2[a] = sum_s D_s exp(alpha[t_s,a] D_s) c2[t_s,a]
// (radialAFs_kernel, STAF/src/fingerprint/rad/reforce.cu.cc:12-64).  Shared by af2_kernel (a wave per centre, four
// centres per workgroup) and by the launch that computes a centre's descriptors and fingerprints in one workgroup,
// so that both give the same bits.
#pragma once
#include "staf_tile.hpp"
#include "staf_tri.hpp"

namespace staf {

// Parameter tables of a workgroup in LDS: p_al[nt*Ar] = alpha in the units of the hot exponential, p_c2[nt*Ar].
// All threads of the workgroup call; a barrier must follow before the tables are read.
template <typename real>
__device__ inline void af2_tables(const real* __restrict__ alpha2b, const real* __restrict__ emb2b, int n,
                                  real* p_al, real* p_c2) {
  for (int q = threadIdx.x; q < n; q += blockDim.x) {
    p_al[q] = HotExp<real>::scale(alpha2b[q]);
    p_c2[q] = emb2b[q];
  }
}

// The wave's loads of its centre: slot descriptors and species offsets into myD, myT (nr entries each, the wave's
// own LDS rows); returns the number of slots.  A barrier (or a wave-level wait) must follow before af2_wave_sum.
template <typename real>
__device__ inline int af2_wave_load(const real* __restrict__ Drow, const int* __restrict__ im,
                                    const int* __restrict__ type_map, int nr, int Ar, real* myD, int* myT, int lane) {
  int cnt = im[0];
  if (cnt > nr) cnt = nr;
  for (int s = lane; s < cnt; s += WAVE) { myD[s] = Drow[s]; myT[s] = type_map[im[1 + s]] * Ar; }
  return cnt;
}

// Lane <-> (channel, slot subset); the subsets of a channel are combined in a fixed order.
template <typename real>
__device__ inline void af2_wave_sum(const real* p_al, const real* p_c2, const real* myD, const int* myT, int cnt,
                                    int Ar, real* __restrict__ out_row, int lane) {
  using HE = HotExp<real>;
  const ChanSub cs(lane, Ar);
  for (int a0 = 0; a0 < Ar; a0 += cs.chunk) {
    const int a = a0 + cs.a;
    const bool on = cs.sub < cs.nsub && a < Ar;
    real acc = 0;
    if (on) {
      for (int s = cs.sub; s < cnt; s += cs.nsub) {
        const real d = myD[s];
        const int ta = myT[s] + a;
        acc += d * (HE::eval(p_al[ta] * d) * p_c2[ta]);
      }
    }
    acc = cs.combine(acc, lane);
    if (on && cs.sub == 0) out_row[a] = acc;
  }
}

}  // namespace staf
