// Per-atom neighbour tile and per-class channel tables shared by the 3-body
// kernels (fingerprint forward, force, and both parameter-gradient ops).
//
// The reference walks an atom's triplets in storage order and evaluates every
// channel for each of them.  Here the triplets of one centre are enumerated by
// species class instead: the first m sorted neighbour slots are grouped by
// species, and the pairs (j<k) are visited class by class -- (ta,ta) triangles
// and (ta,tb) rectangles.  Inside a class the parameter row sigma = ta+tb is
// the same for every lane of a wavefront, so (1) alpha/beta/embedding values
// are wave-uniform and (2) channels whose squared embedding is exactly 0 --
// two thirds of them with the reference's block embeddings -- are skipped for
// the whole wave instead of being multiplied by zero lane by lane.
// The storage index nn of a pair is recovered from its two slots, so tensors
// laid out by nn (angdescr, der3b) are read in place.
#pragma once
#include "staf_common.hpp"

namespace staf {

// Compacted parameters of the active channels of every parameter row sigma.
// Lives in LDS, built once per workgroup.
template <typename real>
struct ChanTable {
  real* a1;   // [nsig*Aa]
  real* a2;   // [nsig*Aa]
  real* be;   // [nsig*Aa]
  real* c3;   // [nsig*Aa]
  int* ch;    // [nsig*Aa] channel id of the compacted entry
  int* nact;  // [nsig]
  int Aa, nsig;
  __device__ unsigned char* carve(unsigned char* p, int nsig_, int Aa_) {
    Aa = Aa_; nsig = nsig_;
    a1 = (real*)p; a2 = a1 + nsig * Aa; be = a2 + nsig * Aa; c3 = be + nsig * Aa;
    ch = (int*)(c3 + nsig * Aa); nact = ch + nsig * Aa;
    // the next carve-out may hold doubles: keep 16-byte alignment
    return p + ((((size_t)nsig * Aa * (4 * sizeof(real) + sizeof(int)) + (size_t)nsig * sizeof(int)) + 15) & ~(size_t)15);
  }
  // alpha3b [ntc, 3*Aa] as (alpha1, alpha2, beta) per channel, emb3b [ntc, Aa].
  // Waves of the block split the rows; a __syncthreads() must follow.
  __device__ void build(const real* alpha3b, const real* emb3b) {
    const int lane = lane_id();
    const int wave = threadIdx.x / WAVE, nwaves = blockDim.x / WAVE;
    for (int sg = wave; sg < nsig; sg += nwaves) {
      int base = 0;
      for (int a0 = 0; a0 < Aa; a0 += WAVE) {
        const int a = a0 + lane;
        real c = 0;
        if (a < Aa) c = emb3b[sg * Aa + a];
        const bool on = (a < Aa) && (c != real(0));
        const unsigned long long mask = __ballot(on);
        if (on) {
          const int pos = base + __popcll(mask & ((1ull << lane) - 1ull));
          const real* al = alpha3b + ((size_t)sg * Aa + a) * 3;
          a1[sg * Aa + pos] = al[0];
          a2[sg * Aa + pos] = al[1];
          be[sg * Aa + pos] = al[2];
          c3[sg * Aa + pos] = c;
          ch[sg * Aa + pos] = a;
        }
        base += __popcll(mask);
      }
      if (lane == 0) nact[sg] = base;
    }
  }
};

template <typename real>
__host__ __device__ inline size_t chan_table_bytes(int nsig, int Aa) {
  return (((size_t)nsig * Aa * (4 * sizeof(real) + sizeof(int)) + (size_t)nsig * sizeof(int)) + 15) & ~(size_t)15;
}

// Slots of one centre grouped by neighbour species (ascending slot inside a
// species).  lst [m] and off [nt+1] live in LDS (per wave or per block).
// Called by one full wavefront; stp [m] holds the species of every slot (LDS).
__device__ inline void group_slots_by_type(int m, int nt, const int* stp, int* lst, int* off) {
  const int lane = lane_id();
  int base = 0;
  for (int t = 0; t < nt; t++) {
    if (lane == 0) off[t] = base;
    for (int s0 = 0; s0 < m; s0 += WAVE) {
      const int s = s0 + lane;
      bool on = false;
      if (s < m) on = (stp[s] == t);
      const unsigned long long mask = __ballot(on);
      if (on) lst[base + __popcll(mask & ((1ull << lane) - 1ull))] = s;
      base += __popcll(mask);
    }
  }
  if (lane == 0) off[nt] = base;
}

// The same for m <= 64 with the species of slot `lane` in a register (t_mine; anything for lane >= m): no memory
// is read, so the wave that loaded the species needs no barrier before it groups.
__device__ inline void group_slots_by_type_reg(int m, int nt, int t_mine, int* lst, int* off) {
  const int lane = lane_id();
  int base = 0;
  for (int t = 0; t < nt; t++) {
    if (lane == 0) off[t] = base;
    const bool on = lane < m && t_mine == t;
    const unsigned long long mask = __ballot(on);
    if (on) lst[base + __popcll(mask & ((1ull << lane) - 1ull))] = lane;
    base += __popcll(mask);
  }
  if (lane == 0) off[nt] = base;
}

// Class (ta,tb) pair index q -> slots (j<k) and storage index nn.
// na_ = population of ta, nb_ = population of tb; la/lb the two slot lists.
__device__ inline void class_pair(int q, bool same, int nb_, const int* la, const int* lb, int m, int& j, int& k,
                                  int& nn) {
  int x, y;
  if (same) {
    // triangle over the na_ == nb_ slots of one species
    tri_decode_xy(q, nb_, x, y);
  } else {
    x = q / nb_;
    y = q - x * nb_;
  }
  const int s1 = la[x], s2 = lb[y];
  j = s1 < s2 ? s1 : s2;
  k = s1 < s2 ? s2 : s1;
  nn = tri_rowstart(j, m) + k - j - 1;
}

// Lane <-> (channel, slot subset) for the 2-body kernels: with Ar channels the 64 lanes hold 64 / Ar subsets that
// walk the slots with that stride, so most lanes work even for few channels (Ar = 20: 60 lanes).  More than 64
// channels are taken in chunks of 64 with one subset.
struct ChanSub {
  int chunk, nsub, sub, a;
  __device__ ChanSub(int lane, int Ar) {
    chunk = Ar < WAVE ? Ar : WAVE;
    nsub = WAVE / chunk;
    sub = lane / chunk;
    a = lane - sub * chunk;
  }
  // sum over the subsets of a channel, valid in the lanes of subset 0 (fixed order)
  template <typename real>
  __device__ real combine(real v, int lane) const {
    real tot = v;
    for (int k = 1; k < nsub; k++) tot += __shfl(v, lane + k * chunk, WAVE);
    return tot;
  }
};

}  // namespace staf
