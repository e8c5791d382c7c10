// 3-body force, pass A: one workgroup of four waves per centre atom, four barriers per centre.
// Replaces computeforce_tripl_kernel (STAF/src/force/ang/reforce.cu.cc:96-214).
//
// The kernel is bound by vector-ALU issue and LDS bandwidth in its channel loop (an item reads its parameter entry
// and two table entries: 32 bytes per lane in single, 64 in double precision, which keeps a CU's LDS as busy as the
// item's 13 / 30 instructions keep its vector units) and by latency around it, so the layout keeps the
// per-(triplet, channel) work minimal, keeps everything else out of the inner loop and avoids workgroup barriers:
//   * lane <-> triplet in storage order (nn = 64*pass + lane, passes dealt round-robin to the waves):
//     angdescr and der3b are read coalesced, once; the triplets of a wave's NP passes (T, the three channel
//     sums, packed indices) stay in registers from the first read to the slot sums.
//   * exp(a1 D_s) and exp(a2 D_s) of every (channel ia, slot s, partner species tb) are tabulated in LDS once
//     per centre (a row per (tb, s): the parameter row is sigma = t_s + tb; channels whose squared embedding is
//     exactly 0 are compacted away), so that exp(a1 Dj + a2 Dk) = E[ia][tk,j].x * E[ia][tj,k].y costs two
//     multiplies.  Per triplet and channel only exp(beta T) remains: one multiply and the hardware exp2 in fp32.
//     With sim2 = exp(a1 Dj + a2 Dk), sim1 = exp(a2 Dj + a1 Dk), P = sim1 + sim2, M = sim2 - sim1:
//       Sd += h (1 + beta T) P                          h = 1/4 G c3 e^{beta T}   (1/2 of E, 1/2 of T)
//       U  += h (a1 + a2) P     V += h (a1 - a2) M
//       SBj = (U + V)/2 = sum h (a1 sim2 + a2 sim1)     SBk = (U - V)/2          (times T at the end)
//     The table is stored row-major ([row][channel], rows padded against bank conflicts, see ROWP) and the
//     channel loop is unrolled, so that every LDS read of the loop is a per-triplet base address plus an
//     immediate offset.
//   * der3b contraction in the same lanes: the contributions to slot j of a pass form contiguous lane groups
//     (rows of the triplet triangle) and are summed with one inclusive scan per value (the prefix before a row's
//     first lane is taken with a lane read); the contributions to slot k are added to the wave's own LDS
//     accumulators row by row (inside a row the k are distinct).  One accumulator per wave and slot takes both;
//     the waves' accumulators are added in a fixed order: results are bit-reproducible.
//     F_s = sum_p Sd(s,p) dT/dd_s(s,p) + (sum_p SB_s(s,p)) grad fc_s
// The slot forces go to scratch or to the caller's arrays (gslot, and the centre's own force to self); the atoms
// that receive them collect them in gather_kernel (per op) or force_total_kernel (all species at once) through the
// neighbour map.
#pragma once
#include <type_traits>

#include "staf_tri.hpp"

namespace staf {

// register-to-register inclusive prefix sums over the 64 lanes of four values at once (same tree as
// wave_sum_to_last; the four chains are interleaved step by step, so that the wait states a lane move needs after
// the instruction that wrote its source are filled by the other chains)
template <typename T>
__device__ inline void wave_scan4(T (&v)[4]) {
  T s[4];
#pragma unroll
  for (int c = 0; c < 4; c++) s[c] = v[c] + dpp_get<0x111, 0xf>(v[c]);
#pragma unroll
  for (int c = 0; c < 4; c++) s[c] += dpp_get<0x112, 0xf>(v[c]);
#pragma unroll
  for (int c = 0; c < 4; c++) s[c] += dpp_get<0x113, 0xf>(v[c]);
#pragma unroll
  for (int c = 0; c < 4; c++) s[c] += dpp_get<0x114, 0xf>(s[c]);
#pragma unroll
  for (int c = 0; c < 4; c++) s[c] += dpp_get<0x118, 0xf>(s[c]);
  dpp_rows_carry(s[0], s[1], s[2], s[3]);
#pragma unroll
  for (int c = 0; c < 4; c++) v[c] = s[c];
}

// NW_: waves per workgroup, 4 or 8 (the launches use 4, see force_tripl).  A sweep takes 16 passes of 64 triplets
// either way; with eight waves a wave holds two of them, so that a centre's critical path and a wave's registers
// are about half of what they are with four.
template <typename real, int NW_ = 4>
struct Force3Cfg {
  static_assert(NW_ == 4 || NW_ == 8, "four or eight waves per workgroup");
  static constexpr int NW = NW_;
  static constexpr int THREADS = NW * WAVE;
  static constexpr int NP = 16 / NW;                        // passes of 64 triplets a wave holds in registers
  static constexpr int CAP = sizeof(real) == 8 ? 8 : 16;    // channels tabulated at a time
  // Exponential table: one row per (partner species, slot), ROWP reals long.
  //   float:  (x, y) pairs of the CAP channels, then one pair of padding: 8-byte reads, rows 136 bytes apart
  //   double: the CAP x values, the CAP y values, one real of padding: two 8-byte reads per entry (one instruction
  //           with two offsets), rows 136 bytes apart as well
  // With 136 = 8 x 17 bytes between the rows of consecutive slots, the 8-byte reads of the lanes of a wave -- a few
  // runs of consecutive slots, since a wave's triplets span two or three rows of the triplet triangle -- fall on the
  // same banks only for slots 32 apart.  (16-byte entries in double precision, 144 bytes apart, collide for slots
  // 16 apart: measured 1.9 conflict cycles per LDS instruction of the whole kernel.)
  static constexpr int ROWP = sizeof(real) == 8 ? 2 * CAP + 1 : 2 * (CAP + 1);
  // der3b rows requested one sweep ahead and held in registers across the channel loop: measured, no gain in
  // fp32 (the kernel is bound by vector-ALU issue) and slower in fp64 (a third of the resident waves lost)
  // (measured and not faster either: the rows of a wave's first pass alone requested ahead of the channel loop,
  // rolling requests in single precision, one element of every 128-byte line of the rows requested at the kernel's
  // start to have the lines in the L2)
  static constexpr bool PREFETCH = false;
  // waves per SIMD the register allocation is held to: with four waves per workgroup what the LDS footprint of the
  // reference's sizes admits (six workgroups per CU in single precision, four in double), with eight waves the
  // hardware's eight waves per SIMD in single precision
  static constexpr int MIN_WAVES = NW == 8 ? (sizeof(real) == 8 ? 6 : 8) : (sizeof(real) == 8 ? 4 : 6);
  __host__ __device__ static bool fits(int nr, int nt) { return nr <= 255 && nt <= NT_MAX; }   // slots packed in 8 bits
  __host__ __device__ static int pitch(int Aa) { return (Aa + 3) & ~3; }   // parameter row pitch (channels)
  // Distance, in channels, between the weight rows of consecutive sigma.  The lanes of a wave read the 16- or 32-byte
  // entry of one channel from the rows of two or three different sigma at once: with a row of pitch(Aa) entries
  // (a multiple of 128 bytes for the usual channel counts) those entries would share their banks; one entry more
  // puts consecutive rows one entry apart.
  __host__ __device__ static int rowp(int Aa) { return pitch(Aa) + 1; }
  // Ar2 > 0: the 2-body pair forces are added (Ar2 radial channels)
  __host__ __device__ static size_t n_reals(int nr, int Aa, int nt, bool fused = false, int Ar2 = 0) {
    const int nsig = 2 * nt - 1;
    return (size_t)nsig * rowp(Aa) * 4 /*prm*/ + (size_t)nsig * pitch(Aa) * 2 /*prE*/ +
           (((size_t)ROWP * nt * nr + 1) & ~(size_t)1) /*E*/ +
           (size_t)NW * 4 * nr /*slot sums per wave*/ + nr /*D*/ + 3 * nr /*grad fc*/ +
           (size_t)NW * 4 /*the waves' shares of the centre's own force*/ + (fused ? 4 * nr : 0) /*unit vectors, 1/r*/ +
           (Ar2 > 0 ? (size_t)NW * nr + nr + (size_t)(2 * nt + 1) * Ar2 : 0) /*2-body: the waves' shares of the pair
           weights, D, parameter rows, the centre's dE/dAF2*/;
  }
  __host__ __device__ static size_t bytes(int nr, int Aa, int nt, bool fused = false, int Ar2 = 0) {
    return n_reals(nr, Aa, nt, fused, Ar2) * sizeof(real) + (size_t)(16 + nr) * sizeof(int);
  }
};

// FUSED (the MD entry): Tang and d3b are not read; a triplet's angular descriptor and its Jacobian are rebuilt from
// the slots' unit vectors u, 1/r, cutoff values fc and their gradients (DescriptorsAngular_kernel,
// STAF/src/descriptor_builder/reforce.cu.cc:195-228), with c = u_j . u_k, h = (c + 1)/2:
//   T = h fc_j fc_k,   dT/dd_j = 1/2 fc_j fc_k / r_j (u_k - c u_j) + h fc_k grad fc_j,   j <-> k for dT/dd_k
// `unit` is [nf, ld, 4, nr] = (u_x, u_y, u_z, 1/r) per sorted neighbour, written by the radial-only descriptor call.
// The 2-body pair forces of the same centre, added to its slot forces (W2B): with g(i,s) = 1/2 sum_ch G2[i,ch]
// c2[t_s,ch] e^{alpha[t_s,ch] D(i,s)} (1 + alpha[t_s,ch] D(i,s)) grad D(i,s) (computeforce_doublets_kernel,
// STAF/src/force/rad/reforce.cu.cc:70-131) the slot force becomes 3-body + g, over all im2[0] radial neighbours.
template <typename real, bool FUSED = false, int NWAVES = 4, bool W2B = false>
__global__ __launch_bounds__((Force3Cfg<real, NWAVES>::THREADS), (Force3Cfg<real, NWAVES>::MIN_WAVES)) void force3_kernel(
    const real* __restrict__ G, const real* __restrict__ Dsup, const real* __restrict__ Tang,
    const real* __restrict__ dDsup, const real* __restrict__ d3b, const real* __restrict__ unit,
    const int* __restrict__ im2,
    const real* __restrict__ alpha3b, const real* __restrict__ emb3b, const int* __restrict__ type_map,
    const int* __restrict__ numtriplet, real* __restrict__ gslot, real* __restrict__ self, int nf, int N, int Nl,
    int ld, int nr, int na, int Aa, int nt, Force2In<real> B2) {
  using real2 = typename Vec2<real>::type;
  using real4 = typename Vec4<real>::type;
  using HE = HotExp<real>;
  using L = Force3Cfg<real, NWAVES>;
  constexpr int NP = L::NP, NW = L::NW, THREADS = L::THREADS, CAP = L::CAP, ROWP = L::ROWP;
  extern __shared__ __align__(16) unsigned char smem[];
  const int nsig = 2 * nt - 1;
  const int RT = nt * nr;                                  // table rows (tb, s)
  const int Ap = L::pitch(Aa), Apr = L::rowp(Aa);
  real* prm = (real*)smem;                                 // [nsig][Apr][4] = a1+a2, a1-a2, scaled beta, 1/4 G c3 (active channels)
  real* prE = prm + (size_t)nsig * Apr * 4;                // [nsig*Ap][2] = a1, a2 in the units of the hot exponential
  real* E = prE + (size_t)nsig * Ap * 2;                   // [RT][ROWP], see Force3Cfg::ROWP
  real* acc = E + (((size_t)RT * ROWP + 1) & ~(size_t)1);  // [NW][4 nr]: per wave, slot sums (as j and as k), see accW
  real* sD = acc + (size_t)NW * 4 * nr;                    // [nr]
  real* sg = sD + nr;                                      // [3*nr] grad fc (der3bsupp)
  real* xch = sg + 3 * nr;                                 // [NW][4] the waves' shares of the centre's own force
  real* sU = xch + NW * 4;                                 // FUSED: [4][nr] unit vector, 1/r
  real* w2p = sU + (FUSED ? 4 * nr : 0);                   // W2B: [NW][nr] the waves' shares of the 2-body pair weights
  real* sD2 = w2p + (W2B ? NW * nr : 0);                   // W2B: [nr] raddescr of the slots
  real* p2 = sD2 + (W2B ? nr : 0);                         // W2B: alpha2b [nt*Ar], emb2b [nt*Ar], dE/dAF2 of the centre [Ar]
  int* nact = (int*)(p2 + (W2B ? (2 * nt + 1) * B2.Ar : 0));   // [16] active channels per sigma (0 beyond nsig)
  int* stp = nact + 16;                                    // [nr] species of every slot

  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), wave = uniform(tid / WAVE);
  const int atom = blockIdx.x;
  const int b = atom / Nl, p_ = atom - b * Nl;
  const size_t rowAtom = (size_t)b * ld + p_;
  const int* im = im2 + rowAtom * (nr + 1);
  int m = numtriplet[rowAtom];
  m = m > nr ? nr : (m < 0 ? 0 : m);
  int ntri = (m * (m - 1)) / 2;
  if (ntri > na) ntri = na;
  const real* Trow = Tang + rowAtom * na;
  const real2* d3 = (const real2*)d3b + rowAtom * 3 * na;
  // A wave's slot sums (force x, y, z, radial factor).  Single precision: one 16-byte entry per slot.  Double
  // precision: two arrays of 16-byte halves, (x, y) and (z, w), so that the lanes of a row, which hold consecutive
  // slots, read consecutive 16-byte words (32-byte entries would put every other lane on the same banks).
  real* accW = acc + (size_t)wave * 4 * nr;
  auto acc_get = [&](const real* base, int s_) -> real4 {
    if constexpr (sizeof(real) == 8) {
      const real2 a = ((const real2*)base)[s_], b2 = ((const real2*)base)[nr + s_];
      real4 t;
      t.x = a.x; t.y = a.y; t.z = b2.x; t.w = b2.y;
      return t;
    } else {
      return ((const real4*)base)[s_];
    }
  };
  auto acc_put = [&](real* base, int s_, const real4& t) {
    if constexpr (sizeof(real) == 8) {
      real2 a, b2;
      a.x = t.x; a.y = t.y; b2.x = t.z; b2.y = t.w;
      ((real2*)base)[s_] = a;
      ((real2*)base)[nr + s_] = b2;
    } else {
      ((real4*)base)[s_] = t;
    }
  };

  // ---- set-up.  Global reads are issued back to back in two levels: (1) everything addressed by the centre alone,
  // the neighbour index first (read up to nr: padded slots are never used); (2) the neighbour's species, which
  // needs only that index and overlaps the parameter rows.
  // Holding the der3b rows of the first sweep in registers from here on was measured and is slower.
  unsigned nj = 0;   // unsigned: no sign extension (and so no wait for the read) ahead of the reads that follow
  real d_s = 0, g_s[3] = {0, 0, 0}, u_s[4] = {0, 0, 0, 0};
  int cnt2 = 0;      // W2B: radial neighbours of the centre
  real d2_s = 0;
  if constexpr (W2B) {
    cnt2 = im[0];
    if (tid < nr) d2_s = B2.D[rowAtom * nr + tid];
    const int npar = nt * B2.Ar;
    for (int q = tid; q < 2 * npar + B2.Ar; q += THREADS)
      p2[q] = q < npar ? B2.alpha2b[q] : (q < 2 * npar ? B2.emb2b[q - npar] : B2.G2[(size_t)atom * B2.Ar + (q - 2 * npar)]);
  }
  if (tid < nr) {
    nj = (unsigned)im[1 + tid];
    d_s = Dsup[rowAtom * nr + tid];
#pragma unroll
    for (int c = 0; c < 3; c++) g_s[c] = dDsup[rowAtom * 3 * nr + c * nr + tid];
    if constexpr (FUSED) {
#pragma unroll
      for (int c = 0; c < 4; c++) u_s[c] = unit[(rowAtom * 4 + c) * nr + tid];
    }
  }
  // Reads of per-triplet rows are never predicated: a lane past the last triplet re-reads the last one (row element
  // 0 if there is none) and its value is masked where it is used.  With every read issued on every path the waits
  // can name how many later reads may stay in flight, which is what lets the prefetches below overlap.
  const int nlast = ntri > 0 ? ntri - 1 : 0;
  real Tn[NP];
  if constexpr (!FUSED) {
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int nn = (p * NW + wave) * WAVE + lane;
      Tn[p] = Trow[nn < nlast ? nn : nlast];
    }
  }
  if constexpr (W2B) cnt2 = cnt2 > nr ? nr : cnt2;
  const bool slot = tid < m;
  const bool slot_t = W2B ? tid < cnt2 : slot;   // slots whose species is needed: with the pair forces, all radial ones
  int t_s = 0;
  if (slot_t) t_s = type_map[nj];
  if (tid >= nsig && tid < 16) nact[tid] = 0;
  {
    real4 z;
    z.x = z.y = z.z = z.w = 0;
    for (int q = tid; q < NW * nr; q += THREADS) ((real4*)acc)[q] = z;
  }
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
        const int cpos = base + __popcll(mask & ((1ull << lane) - 1ull));
        real4 o;
        o.x = al0 + al1;
        o.y = al0 - al1;
        o.z = HE::scale(al2);   // beta in the units of the hot exponential
        o.w = real(0.25) * gv * c;
        *(real4*)(prm + (size_t)(sgm * Apr + cpos) * 4) = o;
        real2 e;
        e.x = HE::scale(al0);
        e.y = HE::scale(al1);
        *(real2*)(prE + (size_t)(sgm * Ap + cpos) * 2) = e;
      }
      base += __popcll(mask);
    }
    // Rows are Ap long and zero beyond the active channels: a triplet whose sigma has fewer channels than the
    // workgroup's maximum reads weight 0 (and exponent 0: table entries 1) there.
    for (int q = base * 4 + lane; q < Ap * 4; q += WAVE) prm[(size_t)sgm * Apr * 4 + q] = 0;
    for (int q = base * 2 + lane; q < Ap * 2; q += WAVE) prE[(size_t)sgm * Ap * 2 + q] = 0;
    if (lane == 0) nact[sgm] = base;
  }
  if (tid < nr) {
    sD[tid] = d_s;
#pragma unroll
    for (int c = 0; c < 3; c++) sg[c * nr + tid] = g_s[c];
    if constexpr (FUSED) {
#pragma unroll
      for (int c = 0; c < 4; c++) sU[c * nr + tid] = u_s[c];
    }
  }
  if (slot_t) stp[tid] = t_s;
  if constexpr (W2B) {
    if (tid < nr) sD2[tid] = d2_s;
  }
  __syncthreads();
  if constexpr (W2B) {
    // 2-body pair weights: lane <-> slot, wave w takes every NW-th channel; the waves' shares are added in a fixed
    // order where the slot forces are formed (several barriers from here)
    const int Ar = B2.Ar;
    for (int s_ = lane; s_ < nr; s_ += WAVE) {
      real w = 0;
      if (s_ < cnt2) {
        const real d2 = sD2[s_];
        const real* al = p2 + mul24(stp[s_], Ar);
        const real* c2 = al + mul24(nt, Ar);
        const real* g2 = p2 + 2 * mul24(nt, Ar);
        for (int ch = wave; ch < Ar; ch += NW) {
          const real ad = al[ch] * d2;
          w += g2[ch] * (c2[ch] * HE::eval(HE::scale(ad)) * (real(1) + ad));
        }
      }
      w2p[wave * nr + s_] = w;
    }
  }
  int maxact = 0;
  for (int sgm = 0; sgm < nsig; sgm++) {
    const int n_ = uniform(nact[sgm]);
    maxact = n_ > maxact ? n_ : maxact;
  }
  // The der3b rows of a sweep are requested one sweep ahead (those of the first here, after the last wait of the
  // set-up): all workgroups of a launch run in step, so reads issued only where they are needed arrive as one
  // burst with the vector units idle.
  // LATE: the products of a pass are formed where the pass is reduced.  Always so in the fused form; in double
  // precision too, where in addition the der3b rows of a pass are requested while the pass before it is reduced (all
  // passes' rows or products at once do not fit the registers of four waves per SIMD).
  constexpr bool LATE = FUSED || sizeof(real) == 8;
  constexpr bool ROLL = !FUSED && LATE && !L::PREFETCH;
  real2 dn[NP][3];
  if constexpr (L::PREFETCH && !FUSED) {
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int nn = (p * NW + wave) * WAVE + lane;
#pragma unroll
      for (int c = 0; c < 3; c++) dn[p][c] = d3[c * na + (nn < nlast ? nn : nlast)];
    }
  }

  for (int w0 = 0; w0 < ntri; w0 += NW * NP * WAVE) {
    // ---- this wave's triplets of the sweep: T, table rows of slot j and slot k, parameter row of sigma, packed j|k
    real T[NP], Sd[NP], U[NP], V[NP];
    int rj[NP], rk[NP], rp[NP], jk[NP];
    int npass = 0;   // passes of the sweep this wave has triplets in (a prefix of the NP)
#pragma unroll
    for (int p = 0; p < NP; p++) {
      const int nn0 = w0 + (p * NW + wave) * WAVE, nn = nn0 + lane;
      if (nn0 < ntri) npass = p + 1;
      T[p] = 0; Sd[p] = 0; U[p] = 0; V[p] = 0;
      rj[p] = 0; rk[p] = 0; rp[p] = 0; jk[p] = 0;   // lanes past the last triplet compute on row 0: finite, never used
      if (nn < ntri) {
        int j, k;
        tri_decode(nn, m, j, k);
        if constexpr (FUSED) {
          const real cs = sU[j] * sU[k] + sU[nr + j] * sU[nr + k] + sU[2 * nr + j] * sU[2 * nr + k];
          T[p] = (real(0.5) * (cs + real(1))) * (sD[j] * sD[k]);
        } else {
          T[p] = Tn[p];
        }
        const int tj = stp[j], tk = stp[k];
        rj[p] = mul24(mul24(tk, nr) + j, ROWP);
        rk[p] = mul24(mul24(tj, nr) + k, ROWP);
        rp[p] = mul24(tj + tk, Apr * 4);
        jk[p] = j | (k << 8);
      }
    }
    for (int c0 = 0; c0 < maxact; c0 += CAP) {
      const int nch = (maxact - c0) < CAP ? (maxact - c0) : CAP;
      const int nch2 = (nch + 1) & ~1;            // the channel loop runs in pairs (c0 + nch2 <= Ap)
      if (c0 > 0 || w0 > 0) __syncthreads();      // readers of the previous tables are done
      // E[(tb, s)][ia] = (exp(a1 D_s), exp(a2 D_s)) with the parameters of sigma = t_s + tb
      // thread <-> (channel ia, rows r0, r0 + RPI, ...): no index division, a row's channels written contiguously
      {
        constexpr int RPI = THREADS / CAP;
        const int ia = tid & (CAP - 1), r0 = tid / CAP;
        if (ia < nch2) {
          for (int tb = 0; tb < nt; tb++) {
            for (int s_ = r0; s_ < m; s_ += RPI) {
              const real2 o = *(const real2*)(prE + (mul24(stp[s_] + tb, Ap) + c0 + ia) * 2);
              const real d = sD[s_];
              real2 v;
              v.x = HE::eval(o.x * d);
              v.y = HE::eval(o.y * d);
              real* row = E + mul24(mul24(tb, nr) + s_, ROWP);
              if constexpr (sizeof(real) == 8) {
                row[ia] = v.x;
                row[CAP + ia] = v.y;
              } else {
                ((real2*)row)[ia] = v;
              }
            }
          }
        }
      }
      __syncthreads();
      // One copy of the loop per number of passes, so that no branch separates the (triplet, channel) items and
      // the LDS reads of the next items are in flight while the current ones are computed.
      auto channels = [&](auto npass_c) {
        constexpr int NPASS = decltype(npass_c)::value;
        const real* pj[NPASS];
        const real* pk[NPASS];
        const real* po[NPASS];
        auto entry = [](const real* row, int c) -> real2 {   // (exp(a1 D), exp(a2 D)) of channel c of a table row
          if constexpr (sizeof(real) == 8) {
            real2 v;
            v.x = row[c];
            v.y = row[CAP + c];
            return v;
          } else {
            return ((const real2*)row)[c];
          }
        };
#pragma unroll
        for (int p = 0; p < NPASS; p++) {
          pj[p] = E + rj[p];
          pk[p] = E + rk[p];
          po[p] = prm + rp[p] + c0 * 4;
        }
        // fully unrolled with an early exit: every LDS address of the loop is a per-pass base plus an immediate
        // offset, no pointer is stepped
#pragma unroll
        for (int ia = 0; ia < CAP; ia += 2) {
          if (ia >= nch2) break;
#pragma unroll
          for (int u = 0; u < 2; u++) {
            // the reads of one channel's items are in flight together; hoisting those of more channels would
            // cost more registers than the occupancy can afford
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < NPASS; p++) {
              const real4 o = *(const real4*)(po[p] + (ia + u) * 4);   // a1+a2, a1-a2, scaled beta, weight
              const real2 e1 = entry(pj[p], ia + u);
              const real2 e2 = entry(pk[p], ia + u);
              const real bts = o.z * T[p];
              const real h = HE::eval(bts) * o.w;
              const real sim1 = e1.y * e2.x;                      // exp(a2 Dj + a1 Dk)
              const real P = r_fma(e1.x, e2.y, sim1);             // + exp(a1 Dj + a2 Dk)
              const real M = r_fma(e1.x, e2.y, -sim1);
              const real hp = h * P, hm = h * M;
              Sd[p] = r_fma(hp, r_fma(bts, HE::unscale(), real(1)), Sd[p]);
              U[p] = r_fma(hp, o.x, U[p]);
              V[p] = r_fma(hm, o.y, V[p]);
            }
          }
        }
      };
      static_assert(NP == 4 || NP == 2, "one case per pass count below");
      if constexpr (NP == 4) {
        switch (npass) {
          case 1: channels(std::integral_constant<int, 1>{}); break;
          case 2: channels(std::integral_constant<int, 2>{}); break;
          case 3: channels(std::integral_constant<int, 3>{}); break;
          case 4: channels(std::integral_constant<int, 4>{}); break;
          default: break;
        }
      } else {
        switch (npass) {
          case 1: channels(std::integral_constant<int, 1>{}); break;
          case 2: channels(std::integral_constant<int, 2>{}); break;
          default: break;
        }
      }
    }

    // ---- contraction with der3b, slot sums of this wave.  Lanes past the last triplet hold T = 0 and finite sums
    // computed on row 0: their products are forced to 0.
    if constexpr (FUSED) {
      // nothing to load: a pass's Jacobian is rebuilt from the slot tile where it is used
    } else if constexpr (!L::PREFETCH) {
#pragma unroll
      for (int p = 0; p < (ROLL ? 1 : NP); p++) {
        const int nn = w0 + (p * NW + wave) * WAVE + lane;
#pragma unroll
        for (int c = 0; c < 3; c++) dn[p][c] = d3[c * na + (nn < nlast ? nn : nlast)];
      }
    }
    // A pass's contributions to its slots j and k: (force x, y, z, radial factor).  The loaded rows are turned into
    // products here, all passes at once, so that their registers are free again before the rows of the next sweep
    // are requested; the fused form rebuilds a pass's Jacobian only where the pass is reduced (its tile reads are
    // LDS reads, and holding all passes' products at once would cost half the resident waves in double precision).
    real vjs[NP][4], vks[NP][4];
    auto pass_products = [&](int p, real (&vj)[4], real (&vk)[4]) {
      const bool valid = w0 + (p * NW + wave) * WAVE + lane < ntri;
      const real sd = valid ? Sd[p] : real(0);
      const real hT = real(0.5) * T[p];
      if constexpr (FUSED) {
        // lanes past the last triplet hold j = k = 0: finite values, masked by sd = 0 and T = 0
        const int j = jk[p] & 0xff, k = jk[p] >> 8;
        const real uj[3] = {sU[j], sU[nr + j], sU[2 * nr + j]}, uk[3] = {sU[k], sU[nr + k], sU[2 * nr + k]};
        const real cs = uj[0] * uk[0] + uj[1] * uk[1] + uj[2] * uk[2];
        const real fj = sD[j], fk = sD[k];
        const real half = real(0.5) * (cs + real(1)), ff = fj * fk;
        const real aj = sd * (real(0.5) * sU[3 * nr + j] * ff), ak = sd * (real(0.5) * sU[3 * nr + k] * ff);
        const real hk = sd * (half * fk), hj = sd * (half * fj);
#pragma unroll
        for (int c = 0; c < 3; c++) {
          vj[c] = aj * (uk[c] - cs * uj[c]) + hk * sg[c * nr + j];
          vk[c] = ak * (uj[c] - cs * uk[c]) + hj * sg[c * nr + k];
        }
      } else {
#pragma unroll
        for (int c = 0; c < 3; c++) {
          vj[c] = sd * dn[p][c].x;
          vk[c] = sd * dn[p][c].y;
        }
      }
      vj[3] = (U[p] + V[p]) * hT;
      vk[3] = (U[p] - V[p]) * hT;
    };
    if constexpr (!LATE) {
#pragma unroll
      for (int p = 0; p < NP; p++) pass_products(p, vjs[p], vks[p]);
    }
    if (!FUSED && w0 + NW * NP * WAVE < ntri) {   // rows of the next sweep
#pragma unroll
      for (int p = 0; p < NP; p++) {
        const int nn = w0 + NW * NP * WAVE + (p * NW + wave) * WAVE + lane;
        Tn[p] = Trow[nn < nlast ? nn : nlast];
      }
      if constexpr (L::PREFETCH && !FUSED) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
          const int nn = w0 + NW * NP * WAVE + (p * NW + wave) * WAVE + lane;
#pragma unroll
          for (int c = 0; c < 3; c++) dn[p][c] = d3[c * na + (nn < nlast ? nn : nlast)];
        }
      }
    }
#pragma unroll
    for (int p = 0; p < NP; p++) {
      if (p >= npass) break;
      const int nn0 = w0 + (p * NW + wave) * WAVE;   // first storage index of the pass
      const int nn = nn0 + lane;
      const bool valid = nn < ntri;
      const int j = jk[p] & 0xff, k = jk[p] >> 8;
      real vj[4], vk[4];
      if constexpr (ROLL) {
        if (p + 1 < NP) {   // rows of the next pass (a pass this wave has no triplets in re-reads the last triplet)
          const int nx = w0 + ((p + 1) * NW + wave) * WAVE + lane;
#pragma unroll
          for (int c = 0; c < 3; c++) dn[(p + 1) % NP][c] = d3[c * na + (nx < nlast ? nx : nlast)];
        }
      }
      if constexpr (LATE) {
        pass_products(p, vj, vk);
      } else {
#pragma unroll
        for (int c = 0; c < 4; c++) { vj[c] = vjs[p][c]; vk[c] = vks[p][c]; }
      }
      // slot j: the lanes of a row are contiguous.  Row sum = prefix at the row's last lane minus prefix
      // before its first lane of this pass (taken with a lane read: no memory is involved).
      wave_scan4(vj);
      const int first = lane - (k - j - 1);   // lane of the row's first triplet (not positive: starts earlier)
      const int before = first > 0 ? first - 1 : 0;   // lanes past the last triplet hold j = k = 0: their own lane
      real pre[4];
#pragma unroll
      for (int c = 0; c < 4; c++) pre[c] = __shfl(vj[c], before, WAVE);
      const int jn = __shfl_down(valid ? j : -1, 1, WAVE);
      const bool row_end = valid && (lane == WAVE - 1 || jn != j);
      if (row_end) {
        real4 t = acc_get(accW, j);
        t.x += vj[0] - (first > 0 ? pre[0] : real(0));
        t.y += vj[1] - (first > 0 ? pre[1] : real(0));
        t.z += vj[2] - (first > 0 ? pre[2] : real(0));
        t.w += vj[3] - (first > 0 ? pre[3] : real(0));
        acc_put(accW, j, t);
      }
      __builtin_amdgcn_wave_barrier();   // the wave's memory operations stay in program order: slot k sums follow
      // slot k: row by row (the k of one row are distinct).  LDS floating-point adds instead of this loop were
      // measured: much slower in fp32 (1.6x the kernel), a few percent faster in fp64.
      const int jlo = __builtin_amdgcn_readfirstlane(j);
      const int llast = (ntri - 1 - nn0) < (WAVE - 1) ? (ntri - 1 - nn0) : (WAVE - 1);
      const int jhi = __builtin_amdgcn_readlane(j, llast);
      for (int g = jlo; g <= jhi; g++) {
        if (valid && j == g) {
          real4 t = acc_get(accW, k);
          t.x += vk[0]; t.y += vk[1]; t.z += vk[2]; t.w += vk[3];
          acc_put(accW, k, t);
        }
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
  __syncthreads();

  // ---- slot forces (waves added in a fixed order; one slot per thread: m <= nr < THREADS), centre's own force.
  // Only the waves that hold slots (the first one for up to 64 slots) form sums; the others' share is zero.
  real f3[3] = {0, 0, 0};
  if (wave * WAVE < nr) {
    if (slot) {
      real t4[4] = {0, 0, 0, 0};
#pragma unroll
      for (int w = 0; w < NW; w++) {
        const real4 a = acc_get(acc + (size_t)w * 4 * nr, tid);
        t4[0] += a.x; t4[1] += a.y; t4[2] += a.z; t4[3] += a.w;
      }
#pragma unroll
      for (int c = 0; c < 3; c++) f3[c] = t4[c] + t4[3] * sg[c * nr + tid];
    }
    if constexpr (W2B) {
      // the pair force of slot tid (zero weight beyond the radial neighbours); slots beyond the angular cutoff carry it alone
      if (tid < nr) {
        real w = 0;
#pragma unroll
        for (int w_ = 0; w_ < NW; w_++) w += w2p[w_ * nr + tid];
        w *= real(0.5);
#pragma unroll
        for (int c = 0; c < 3; c++) f3[c] += w * B2.dD[rowAtom * 3 * nr + c * nr + tid];
      }
    }
#pragma unroll
    for (int c = 0; c < 3; c++) {
      const real t = wave_sum_to_last(f3[c]);
      if (lane == WAVE - 1) xch[wave * 4 + c] = t;
    }
  } else if (lane < 3) {
    xch[wave * 4 + lane] = 0;
  }
  __syncthreads();
  // global stores after the last barrier: nothing waits for them
  // every slot of the row is written: the atoms that gather see all slots of the neighbour map, also those beyond
  // the angular cutoff, which carry no 3-body force (f3 = 0 there)
  if (tid < nr) {
#pragma unroll
    for (int c = 0; c < 3; c++) gslot[((size_t)atom * nr + tid) * 3 + c] = f3[c];
  }
  if (tid < 3) {
    real a = 0;
#pragma unroll
    for (int w = 0; w < NW; w++) a += xch[w * 4 + tid];
    self[(size_t)atom * 3 + tid] = -a;
  }
}

}  // namespace staf
