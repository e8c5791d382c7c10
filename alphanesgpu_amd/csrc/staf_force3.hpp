// 3-body force, pass A: one 256-thread workgroup per centre atom, four barriers per centre.
// Replaces computeforce_tripl_kernel (STAF/src/force/ang/reforce.cu.cc:96-214).
//
// The kernel is bound by vector-ALU issue and by latency, so the layout keeps the per-(triplet, channel) work
// minimal, keeps everything else out of the inner loop and avoids workgroup barriers:
//   * lane <-> triplet in storage order (nn = 64*pass + lane, passes dealt round-robin to the four waves):
//     angdescr and der3b are read coalesced, once; the triplets of a wave's NP passes (T, the three channel
//     sums, packed indices) stay in registers from the first read to the slot sums.
//   * exp(a1 D_s) and exp(a2 D_s) of every (channel ia, slot s, partner species tb) are tabulated in LDS once
//     per centre (a row per (tb, s): the parameter row is sigma = t_s + tb; channels whose squared embedding is
//     exactly 0 are compacted away), so that exp(a1 Dj + a2 Dk) = E[ia][tk,j].x * E[ia][tj,k].y costs two
//     multiplies.  Per triplet and channel only exp(beta T) remains: one multiply and the hardware exp2 in fp32.
//       Sd  += h (1 + beta T)(sim1 + sim2)              h = 1/4 G c3 e^{beta T}   (1/2 of E, 1/2 of T)
//       SBj += h (a1 sim2 + a2 sim1)  SBk += h (a1 sim1 + a2 sim2)               (times T at the end)
//   * der3b contraction in the same lanes: the contributions to slot j of a pass form contiguous lane groups
//     (rows of the triplet triangle) and are summed with one inclusive scan per value; the contributions to
//     slot k are added to the wave's own LDS accumulators row by row (inside a row the k are distinct).  The
//     four waves' accumulators are added in a fixed order: results are bit-reproducible.
//     F_s = sum_p Sd(s,p) dT/dd_s(s,p) + (sum_p SB_s(s,p)) grad fc_s
#pragma once
#include "staf_tri.hpp"

namespace staf {

// register-to-register inclusive prefix sum over the 64 lanes (same tree as wave_sum_to_last)
template <typename T>
__device__ inline T wave_scan(T v) { return wave_sum_to_last(v); }

template <typename real>
struct Force3Cfg {
  static constexpr int THREADS = 256;
  static constexpr int NW = THREADS / WAVE;
  static constexpr int NP = 4;                              // passes of 64 triplets a wave holds in registers
  static constexpr int CAP = sizeof(real) == 8 ? 8 : 16;    // channels tabulated at a time
  __host__ __device__ static bool fits(int nr, int nt) { return nr <= 255 && nt <= NT_MAX; }   // slots packed in 8 bits
  __host__ __device__ static size_t n_reals(int nr, int Aa, int nt) {
    const int nsig = 2 * nt - 1;
    return (size_t)CAP * nt * nr * 2 /*E*/ + (size_t)nsig * Aa * 4 /*prm*/ + (size_t)NW * 8 * nr /*accJ, accK per wave*/ +
           nr /*D*/ + 3 * nr /*grad fc*/ + (size_t)NW * 4 * WAVE /*scan exchange per wave*/ + 3 * nr /*fs*/;
  }
  __host__ __device__ static size_t bytes(int nr, int Aa, int nt) {
    return n_reals(nr, Aa, nt) * sizeof(real) + (size_t)(16 + nr) * sizeof(int);
  }
};

template <typename real>
__global__ __launch_bounds__(Force3Cfg<real>::THREADS) void force3_kernel(
    const real* __restrict__ G, const real* __restrict__ Dsup, const real* __restrict__ Tang,
    const real* __restrict__ dDsup, const real* __restrict__ d3b, const int* __restrict__ im2,
    const real* __restrict__ alpha3b, const real* __restrict__ emb3b, const int* __restrict__ type_map,
    const int* __restrict__ numtriplet, real* __restrict__ gslot, real* __restrict__ self, int* bcnt, int* bent,
    int cap, int* status, int nf, int N, int Nl, int ld, int nr, int na, int Aa, int nt) {
  using real2 = typename Vec2<real>::type;
  using HE = HotExp<real>;
  using L = Force3Cfg<real>;
  constexpr int NP = L::NP, NW = L::NW, THREADS = L::THREADS, CAP = L::CAP;
  extern __shared__ __align__(16) unsigned char smem[];
  const int nsig = 2 * nt - 1;
  const int RT = nt * nr;                                  // table rows (tb, s)
  real2* E = (real2*)smem;                                 // [CAP][RT]
  real* prm = (real*)(E + (size_t)CAP * RT);               // [nsig*Aa][4] = a1, a2, scaled beta, 1/4 G c3 (active channels)
  real* acc = prm + (size_t)nsig * Aa * 4;                 // [NW][8][nr]: per wave, slot sums as j (4) and as k (4)
  real* sD = acc + (size_t)NW * 8 * nr;                    // [nr]
  real* sg = sD + nr;                                      // [3*nr] grad fc (der3bsupp)
  real* xch = sg + 3 * nr;                                 // [NW][4][64] prefix sums of a pass
  real* fs = xch + NW * 4 * WAVE;                          // [3*nr]
  int* nact = (int*)(fs + 3 * nr);                         // [16] active channels per sigma (0 beyond nsig)
  int* stp = nact + 16;                                    // [nr] species of every slot
  PHASE_CLOCK_BEGIN();

  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int atom = blockIdx.x;
  const int b = atom / Nl, p_ = atom - b * Nl;
  const size_t rowAtom = (size_t)b * ld + p_;
  const int* im = im2 + rowAtom * (nr + 1);
  int m = numtriplet[rowAtom];
  if (m > nr) m = nr;
  int ntri = (m * (m - 1)) / 2;
  if (ntri > na) ntri = na;
  const real* Trow = Tang + rowAtom * na;
  const real2* d3 = (const real2*)d3b + rowAtom * 3 * na;
  real* accJ = acc + (size_t)wave * 8 * nr;
  real* accK = accJ + 4 * nr;
  real* myx = xch + wave * 4 * WAVE;

  // ---- set-up.  Global reads are issued level by level, back to back: (1) everything addressed by the centre
  // alone -- slot rows (read up to nr: padded slots hold index 0), the T of the first sweep, the parameter rows;
  // (2) what needs a neighbour index -- its species and its registration with the receiving atom (an integer
  // atomic whose return is only used for a store at the very end).  Holding the der3b rows of the first sweep in
  // registers from here on was measured and is slower: it only adds to the burst of reads every workgroup of
  // the launch issues at the same moment.
  int nj = 0;
  real d_s = 0, g_s[3] = {0, 0, 0};
  if (tid < nr) {
    nj = im[1 + tid];
    d_s = Dsup[rowAtom * nr + tid];
#pragma unroll
    for (int c = 0; c < 3; c++) g_s[c] = dDsup[rowAtom * 3 * nr + c * nr + tid];
  }
  real Tpre[NP];
#pragma unroll
  for (int p = 0; p < NP; p++) {
    const int nn = (p * NW + wave) * WAVE + lane;
    Tpre[p] = nn < na ? Trow[nn] : real(0);
  }
  if (tid >= nsig && tid < 16) nact[tid] = 0;
  for (int q = tid; q < NW * 8 * nr; q += THREADS) acc[q] = 0;
  for (int sgm = wave; sgm < nsig; sgm += NW) {
    int base = 0;
    for (int a0 = 0; a0 < Aa; a0 += WAVE) {
      const int a = a0 + lane;
      real c = 0, al0 = 0, al1 = 0, al2 = 0, gv = 0;
      if (a < Aa) {
        const real* al = alpha3b + ((size_t)sgm * Aa + a) * 3;
        c = emb3b[sgm * Aa + a];
        al0 = al[0]; al1 = al[1]; al2 = al[2];
        gv = G[(size_t)atom * Aa + a];
      }
      const bool on = (a < Aa) && (c != real(0));
      const unsigned long long mask = __ballot(on);
      if (on) {
        real* o = prm + ((size_t)sgm * Aa + base + __popcll(mask & ((1ull << lane) - 1ull))) * 4;
        o[0] = al0;
        o[1] = al1;
        o[2] = HE::scale(al2);   // beta in the units of the hot exponential
        o[3] = real(0.25) * gv * c;
      }
      base += __popcll(mask);
    }
    // parameter rows beyond the active ones are read (and weighted with 0) by lanes of another sigma
    for (int q = base * 4 + lane; q < Aa * 4; q += WAVE) prm[(size_t)sgm * Aa * 4 + q] = 0;
    if (lane == 0) nact[sgm] = base;
  }
  int bpos = 0;
  const bool slot = tid < m;
  if (slot) {
    stp[tid] = type_map[nj];
    bpos = atomicAdd(&bcnt[(size_t)b * N + nj], 1);
  }
  if (tid < nr) {
    sD[tid] = d_s;
#pragma unroll
    for (int c = 0; c < 3; c++) sg[c * nr + tid] = g_s[c];
  }
  __syncthreads();
  PHASE_MARK(0);
  int maxact = 0;
  for (int sgm = 0; sgm < nsig; sgm++) {
    const int n_ = uniform(nact[sgm]);
    maxact = n_ > maxact ? n_ : maxact;
  }
  const int mrows = nt * m;
  const float inv_mrows = mrows > 0 ? 1.0f / (float)mrows : 0.f, inv_m = m > 0 ? 1.0f / (float)m : 0.f;

  for (int w0 = 0; w0 < ntri; w0 += NW * NP * WAVE) {
    // ---- this wave's triplets of the sweep: T, packed table rows / sigma, packed slots / active-channel count
    real T[NP], Sd[NP], S1[NP], S2[NP];
    int rj[NP], rk[NP], rp[NP], jk[NP];   // table rows of slot j and slot k, first parameter row of sigma, packed j|k|count
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int nn = w0 + (p * NW + wave) * WAVE + lane;
      T[p] = 0; Sd[p] = 0; S1[p] = 0; S2[p] = 0;
      rj[p] = 0; rk[p] = 0; rp[p] = 0;
      jk[p] = 0;                // count 0: no active channel
      if (nn < ntri) {
        int j, k;
        tri_decode(nn, m, j, k);
        T[p] = w0 == 0 ? Tpre[p] : Trow[nn];
        const int tj = stp[j], tk = stp[k];
        rj[p] = tk * nr + j;
        rk[p] = tj * nr + k;
        rp[p] = (tj + tk) * Aa;
        jk[p] = j | (k << 8) | (nact[tj + tk] << 16);
      }
    }
    PHASE_MARK(1);

    for (int c0 = 0; c0 < maxact; c0 += CAP) {
      const int nch = (maxact - c0) < CAP ? (maxact - c0) : CAP;
      if (c0 > 0 || w0 > 0) __syncthreads();   // readers of the previous tables are done
      // E[ia][(tb, s)] = (exp(a1 D_s), exp(a2 D_s)) with the parameters of sigma = t_s + tb
      for (int e = tid; e < nch * mrows; e += THREADS) {
        const int ia = small_div(e, mrows, inv_mrows), r = e - ia * mrows;
        const int tb = small_div(r, m, inv_m), s = r - tb * m;
        const int sgm = stp[s] + tb;
        // an entry without a channel is read by lanes of another sigma (and weighted with 0): it must be finite
        real2 v;
        v.x = 0; v.y = 0;
        if (c0 + ia < nact[sgm]) {
          const real* o = prm + ((size_t)sgm * Aa + c0 + ia) * 4;
          const real d = sD[s];
          v.x = HE::eval(HE::scale(o[0]) * d);
          v.y = HE::eval(HE::scale(o[1]) * d);
        }
        E[ia * RT + tb * nr + s] = v;
      }
      __syncthreads();
      PHASE_MARK(2);
      for (int ia = 0; ia < nch; ia++) {
        const real2* Ei = E + ia * RT;
        const real* prmi = prm + (size_t)(c0 + ia) * 4;
#pragma unroll
        for (int p = 0; p < NP; p++) {
          if (w0 + (p * NW + wave) * WAVE >= ntri) break;   // this wave has no further pass in the sweep
          // A lane whose sigma has no channel c0+ia reads parameters and table entries that are not its own
          // (finite values of another channel or the zeros the table starts with) and weights them with 0.
          const real* o = prmi + rp[p] * 4;
          const real a1 = o[0], a2 = o[1], bes = o[2];
          const real nc = (c0 + ia) < (jk[p] >> 16) ? o[3] : real(0);
          const real2 e1 = Ei[rj[p]];
          const real2 e2 = Ei[rk[p]];
          const real sim2 = e1.x * e2.y;   // exp(a1 Dj + a2 Dk)
          const real sim1 = e1.y * e2.x;   // exp(a2 Dj + a1 Dk)
          const real bts = bes * T[p];
          const real h = HE::eval(bts) * nc;
          Sd[p] += h * r_fma(bts, HE::unscale(), real(1)) * (sim1 + sim2);
          S1[p] += h * (a1 * sim2 + a2 * sim1);
          S2[p] += h * (a1 * sim1 + a2 * sim2);
        }
      }
      PHASE_MARK(3);
    }

    // ---- contraction with der3b, slot sums of this wave.  The reads of all passes are issued together.
    real2 dv[NP][3];
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int nn = w0 + (p * NW + wave) * WAVE + lane;
#pragma unroll
      for (int c = 0; c < 3; c++) {
        dv[p][c].x = 0; dv[p][c].y = 0;
        if (nn < ntri) dv[p][c] = d3[c * na + nn];
      }
    }
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int nn0 = w0 + (p * NW + wave) * WAVE;   // first storage index of the pass
      if (nn0 >= ntri) break;
      const int nn = nn0 + lane;
      const bool valid = nn < ntri;
      const int j = jk[p] & 0xff, k = (jk[p] >> 8) & 0xff;
      real vj[4] = {0, 0, 0, 0}, vk[4] = {0, 0, 0, 0};
      if (valid) {
        const real2 d0 = dv[p][0], d1 = dv[p][1], d2 = dv[p][2];
        vj[0] = Sd[p] * d0.x; vj[1] = Sd[p] * d1.x; vj[2] = Sd[p] * d2.x; vj[3] = S1[p] * T[p];
        vk[0] = Sd[p] * d0.y; vk[1] = Sd[p] * d1.y; vk[2] = Sd[p] * d2.y; vk[3] = S2[p] * T[p];
      }
      // slot j: the lanes of a row are contiguous.  Row sum = prefix at the row's last lane minus prefix
      // before its first lane of this pass.
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int c = 0; c < 4; c++) {
        vj[c] = wave_scan(vj[c]);
        myx[c * WAVE + lane] = vj[c];
      }
      __builtin_amdgcn_wave_barrier();
      const int jn = __shfl_down(valid ? j : -1, 1, WAVE);
      const bool row_end = valid && (lane == WAVE - 1 || jn != j);
      if (row_end) {
        const int first = lane - (k - j - 1);   // lane of the row's first triplet (not positive: starts earlier)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          real s = vj[c];
          if (first > 0) s -= myx[c * WAVE + first - 1];
          accJ[c * nr + j] += s;
        }
      }
      // slot k: row by row (the k of one row are distinct)
      const int jlo = __builtin_amdgcn_readfirstlane(j);
      const int nlast = (ntri - 1 - nn0) < (WAVE - 1) ? (ntri - 1 - nn0) : (WAVE - 1);
      const int jhi = __builtin_amdgcn_readlane(j, nlast);
      for (int g = jlo; g <= jhi; g++) {
        if (valid && j == g) {
#pragma unroll
          for (int c = 0; c < 4; c++) accK[c * nr + k] += vk[c];
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
    PHASE_MARK(4);
  }
  __syncthreads();
  PHASE_MARK(5);

  // ---- slot forces (waves added in a fixed order), centre's own force
  for (int s = tid; s < m; s += THREADS) {
    real t4[4];
#pragma unroll
    for (int c = 0; c < 4; c++) {
      real t = 0;
#pragma unroll
      for (int w = 0; w < NW; w++) t += acc[((size_t)w * 8 + c) * nr + s] + acc[((size_t)w * 8 + 4 + c) * nr + s];
      t4[c] = t;
    }
#pragma unroll
    for (int c = 0; c < 3; c++) fs[c * nr + s] = t4[c] + t4[3] * sg[c * nr + s];
  }
  __syncthreads();
  // global stores after the last barrier: nothing waits for them
  for (int s = tid; s < m; s += THREADS) {
#pragma unroll
    for (int c = 0; c < 3; c++) gslot[((size_t)atom * nr + s) * 3 + c] = fs[c * nr + s];
  }
  if (tid < WAVE) {
#pragma unroll
    for (int c = 0; c < 3; c++) {
      real a = 0;
      for (int s = tid; s < m; s += WAVE) a -= fs[c * nr + s];
      a = wave_sum(a);
      if (tid == 0) self[(size_t)atom * 3 + c] = a;
    }
  }
  if (slot) {   // the slot's place in the bucket of its receiving atom
    if (bpos < cap) bent[((size_t)b * N + nj) * cap + bpos] = p_ * nr + tid;
    else atomicOr(status, 2);
  }
  PHASE_MARK(6);
  PHASE_CLOCK_END();
}

}  // namespace staf
