// Triplet kernels that reduce over an atom's triplets: 3-body fingerprints
// (MODE 0), their parameter gradient (MODE 1) and the gradient of the 3-body
// force op (MODE 2).  One 256-thread workgroup per centre atom (persistent
// over atoms for the gradient modes).
//
// Work decomposition inside a species class (ta,tb) of the centre's triplets
// (see staf_tile.hpp for the class enumeration):
//   * exp(a1*D_s), exp(a2*D_s) are tabulated in LDS once per (slot, channel)
//     of the class, so that exp(a1 Dj + a2 Dk) = E1[j]*E2[k] costs two
//     multiplies instead of an exp: O(m * channels) transcendental calls for
//     the pair factors instead of O(m^2 * channels).  Only exp(beta*T) stays
//     per (triplet, channel).
//   * thread <-> (channel, triplet subset): the threads of a wave that share a
//     subset walk the same triplets and differ in the channel, so every thread
//     accumulates its own channel privately -- no cross-lane reduction per
//     channel, parameters live in registers, table reads are contiguous in the
//     channel.  Subsets are combined once per class through LDS in a fixed
//     order (bit-reproducible).
//   * triplets are staged in LDS in blocks (packed pair index, T, and for
//     MODE 2 the contraction U of der3b with dL/dF), so tensors laid out by
//     the storage index nn are read exactly once.
#pragma once
#include "staf_tile.hpp"

namespace staf {

constexpr int TRI_BLOCK = 256;
constexpr int TRI_CAP = 16;    // channels tabulated per pass
constexpr int TRI_QB = 512;    // triplets staged per block
constexpr int TRI_GRID_MAX = 2048;  // workgroups of the persistent gradient modes (one partial row each)

template <typename real>
struct TriArgs {
  const real* Dsup;       // des3bsupp  [nf, ld, nr]
  const real* Tang;       // angdescr   [nf, ld, na]
  const int* im2;         // intmap2b   [nf, ld, nr+1]
  const real* alpha3b;    // [ntc, 3*Aa]
  const real* emb3b;      // [ntc, Aa]
  const int* type_map;    // [N]
  const int* numtriplet;  // [nf, ld]
  const real* P;          // MODE 1: dL/dAF3, MODE 2: netderiv  [nf, Nl, Aa] contiguous
  const real* Q;          // MODE 2: dL/dF [nf, 3N]
  const real* dDsup;      // MODE 2: der3bsupp [nf, ld, 3, nr]
  const real* d3b;        // MODE 2: der3b [nf, ld, 3, na, 2]
  const int* tipos;       // MODE 2
  const int* actual_type; // MODE 2
  const real* Qvir;       // MODE 2, virial form: dL/dW [nf, 9] (else null)
  const real* pos;        // MODE 2, virial form: positions [nf, 3N]
  const real* box;        // MODE 2, virial form: [nf, 6]
  int skip_pbc;           // MODE 2, virial form: no minimum-image wrap
  real* out;              // MODE 0: AF3, MODE 2: gradnet  [nf, Nl, Aa] contiguous
  real* partial;          // MODE 1/2: [gridDim.x, nsig*Aa*3]
  int nf, N, Nl, ld, nr, na, Aa, nt;
};

template <typename real, int MODE>
struct TriLds {
  static constexpr int NV = (MODE == 0) ? 1 : (MODE == 1 ? 3 : 4);
  // bytes of the staging region (packed pairs + T (+ U)) followed by the per-thread partials of the class reduction
  __host__ __device__ static size_t stage_bytes() {
    size_t st = (size_t)TRI_QB * (sizeof(int) + sizeof(real) * (MODE == 2 ? 2 : 1));
    size_t rd = (size_t)TRI_BLOCK * NV * sizeof(real);
    return ((st + 15) & ~(size_t)15) + ((rd + 15) & ~(size_t)15);
  }
  __host__ __device__ static size_t bytes(int nr, int Aa, int nt) {
    const int nsig = 2 * nt - 1;
    size_t b = chan_table_bytes<real>(nsig, Aa);
    size_t reals = (size_t)Aa /*out_ch*/ + nr /*sD*/ + Aa /*sP*/ + (size_t)nr * TRI_CAP * 2 /*pair tables*/;
    if (MODE != 0) reals += (size_t)nsig * Aa * 3;
    if (MODE == 2) reals += (size_t)4 * nr;  // sV, sQ
    b += reals * sizeof(real);
    b = (b + 15) & ~(size_t)15;
    b += stage_bytes();
    b += (size_t)(2 * nr + NT_MAX + 1) * sizeof(int);
    return b;
  }
};

template <typename real, int MODE>
__global__ __launch_bounds__(TRI_BLOCK) void tri_reduce_kernel(TriArgs<real> A) {
  using real2 = typename Vec2<real>::type;
  constexpr int NV = TriLds<real, MODE>::NV;
  extern __shared__ __align__(16) unsigned char smem[];
  const int nr = A.nr, na = A.na, Aa = A.Aa, nt = A.nt;
  const int nsig = 2 * nt - 1;
  ChanTable<real> tab;
  unsigned char* sp = tab.carve(smem, nsig, Aa);
  real* rp = (real*)sp;   // 16-byte aligned: the pair tables come first
  real2* tabA = (real2*)rp; rp += (size_t)nr * TRI_CAP * 2;   // both species of a class: at most m <= nr rows
  real* out_ch = rp; rp += Aa;
  real* sD = rp; rp += nr;
  real* sP = rp; rp += Aa;
  real* acc_par = rp;
  if (MODE != 0) rp += (size_t)nsig * Aa * 3;
  real* sV = rp;
  real* sQ = rp + nr;
  if (MODE == 2) rp += (size_t)4 * nr;
  unsigned char* stg = (unsigned char*)((((size_t)rp) + 15) & ~(size_t)15);
  real* sT = (real*)stg;                       // [TRI_QB]
  real* sU = sT + TRI_QB;                      // [TRI_QB] (MODE 2)
  int* pk = (int*)(sT + TRI_QB * (MODE == 2 ? 2 : 1));   // [TRI_QB]
  real* red = (real*)(stg + (((size_t)TRI_QB * (sizeof(int) + sizeof(real) * (MODE == 2 ? 2 : 1)) + 15) & ~(size_t)15));
  int* lst = (int*)(stg + TriLds<real, MODE>::stage_bytes());
  int* stp = lst + nr;
  int* off = stp + nr;

  const int tid = threadIdx.x;
  tab.build(A.alpha3b, A.emb3b);
  if (MODE != 0)
    for (int q = tid; q < nsig * Aa * 3; q += TRI_BLOCK) acc_par[q] = 0;
  int shift = 0;
  if (MODE == 2) {
    const int at = A.actual_type[0];
    for (int y = 0; y < at; y++) shift += A.tipos[y];
  }
  __syncthreads();

  const int total = A.nf * A.Nl;
  for (int atom = blockIdx.x; atom < total; atom += gridDim.x) {
    const int b = atom / A.Nl, p = atom - b * A.Nl;
    const size_t rowAtom = (size_t)b * A.ld + p;
    const int* im = A.im2 + rowAtom * (nr + 1);
    int m = A.numtriplet[rowAtom];
    if (m > nr) m = nr;
    const real* Trow = A.Tang + rowAtom * na;
    const real2* d3 = (const real2*)A.d3b + rowAtom * 3 * na;
    // ---- per-atom slot data
    for (int s = tid; s < m; s += TRI_BLOCK) {
      sD[s] = A.Dsup[rowAtom * nr + s];
      const int nj = im[1 + s];
      stp[s] = A.type_map[nj];
      if (MODE == 2) {
        const real* Qj = A.Q + ((size_t)b * A.N + nj) * 3;
        const real* Qi = A.Q + ((size_t)b * A.N + p + shift) * 3;
        real q0 = Qj[0] - Qi[0], q1 = Qj[1] - Qi[1], q2 = Qj[2] - Qi[2];
        if (A.Qvir) {
          // virial form: dL/dg_a = (dL/dF_j - dL/dF_i)_a - sum_e (dL/dW)_ae r_e (grad_force/ang/reforce.cu.cc:391-394)
          real r[3];
          mic_cart_from_cart(A.pos + ((size_t)b * A.N + p + shift) * 3, A.pos + ((size_t)b * A.N + nj) * 3,
                             A.box + (size_t)b * 6, A.skip_pbc, r);
          const real* Wg = A.Qvir + (size_t)b * 9;
          q0 -= Wg[0] * r[0] + Wg[1] * r[1] + Wg[2] * r[2];
          q1 -= Wg[3] * r[0] + Wg[4] * r[1] + Wg[5] * r[2];
          q2 -= Wg[6] * r[0] + Wg[7] * r[1] + Wg[8] * r[2];
        }
        const real* gr = A.dDsup + rowAtom * 3 * nr + s;
        sQ[3 * s] = q0; sQ[3 * s + 1] = q1; sQ[3 * s + 2] = q2;
        sV[s] = q0 * gr[0] + q1 * gr[nr] + q2 * gr[2 * nr];
      }
    }
    for (int a = tid; a < Aa; a += TRI_BLOCK) {
      out_ch[a] = 0;
      if (MODE != 0) sP[a] = A.P[(size_t)atom * Aa + a];
    }
    __syncthreads();
    if (tid < WAVE) group_slots_by_type(m, nt, stp, lst, off);
    __syncthreads();

    for (int ta = 0; ta < nt; ta++) {
      const int oa = off[ta];
      const int na_ = off[ta + 1] - oa;
      if (na_ == 0) continue;
      for (int tb = ta; tb < nt; tb++) {
        const int ob = off[tb];
        const int nb_ = off[tb + 1] - ob;
        const bool same = (ta == tb);
        const int size = same ? (na_ * (na_ - 1)) / 2 : na_ * nb_;
        if (size == 0) continue;
        const int sg = ta + tb;
        const int nact = tab.nact[sg];
        const int pb = sg * Aa;
        const int* la = lst + oa;
        const int* lb = lst + ob;
        real2* tabB = tabA + (size_t)na_ * TRI_CAP;   // rows of the second species follow the first
        for (int c0 = 0; c0 < nact; c0 += TRI_CAP) {
          const int nch = (nact - c0) < TRI_CAP ? (nact - c0) : TRI_CAP;
          // ---- tables of the class: E[x][ia] = (exp(a1 D), exp(a2 D))
          {
            const int ea = na_ * nch, eb_ = same ? 0 : nb_ * nch;
            for (int e = tid; e < ea + eb_; e += TRI_BLOCK) {
              const bool second = e >= ea;
              const int ee = second ? e - ea : e;
              const int x = ee / nch, ia = ee - x * nch;
              const real d = sD[second ? lb[x] : la[x]];
              real2 v;
              v.x = r_exp(tab.a1[pb + c0 + ia] * d);
              v.y = r_exp(tab.a2[pb + c0 + ia] * d);
              (second ? tabB : tabA)[x * TRI_CAP + ia] = v;
            }
          }
          const real2* tB = same ? tabA : tabB;
          const int S = TRI_BLOCK / nch;
          const int sub = tid / nch, ia = tid - sub * nch;
          const bool worker = sub < S;
          real be = 0;
          if (worker) be = tab.be[pb + c0 + ia];
          real acc[NV];
#pragma unroll
          for (int v = 0; v < NV; v++) acc[v] = 0;
          for (int q0 = 0; q0 < size; q0 += TRI_QB) {
            const int nq = (size - q0) < TRI_QB ? (size - q0) : TRI_QB;
            if (q0 > 0) __syncthreads();   // previous block consumed
            // ---- stage a block of triplets
            for (int qq = tid; qq < nq; qq += TRI_BLOCK) {
              const int q = q0 + qq;
              int x, y;
              if (same) tri_decode_xy(q, nb_, x, y);
              else { x = q / nb_; y = q - x * nb_; }
              const int s1 = la[x], s2 = lb[y];
              const int j = s1 < s2 ? s1 : s2, k = s1 < s2 ? s2 : s1;
              const int nn = tri_rowstart(j, m) + k - j - 1;
              const bool ok = nn < na;
              pk[qq] = x | (y << 16);
              real T = 0;
              if (ok) T = Trow[nn];
              sT[qq] = T;
              if (MODE == 2) {
                real U = 0;
                if (ok) {
#pragma unroll
                  for (int c = 0; c < 3; c++) {
                    const real2 dv = d3[c * na + nn];
                    U += sQ[3 * j + c] * dv.x + sQ[3 * k + c] * dv.y;
                  }
                }
                sU[qq] = U;
              }
            }
            __syncthreads();
            // ---- thread <-> (channel ia, subset sub)
            if (worker) {
              for (int qq = sub; qq < nq; qq += S) {
                const int xy = pk[qq];
                const int x = xy & 0xffff, y = xy >> 16;
                const real T = sT[qq];
                const real2 e1 = tabA[x * TRI_CAP + ia];
                const real2 e2 = tB[y * TRI_CAP + ia];
                const real ebt = r_exp(be * T);
                const real sim2 = e1.x * e2.y;   // exp(a1 D1 + a2 D2)
                const real sim1 = e1.y * e2.x;   // exp(a2 D1 + a1 D2)
                if (MODE == 0) {
                  acc[0] += T * (sim1 + sim2) * ebt;
                } else if (MODE == 1) {
                  const real D1 = sD[la[x]], D2 = sD[lb[y]];
                  const real w = ebt * T;
                  acc[0] += (sim2 * D1 + sim1 * D2) * w;
                  acc[1] += (sim2 * D2 + sim1 * D1) * w;
                  acc[NV - 1] += (sim1 + sim2) * w * T;
                } else {
                  const int s1 = la[x], s2 = lb[y];
                  const real D1 = sD[s1], D2 = sD[s2];
                  const real V1 = sV[s1], V2 = sV[s2];
                  const real U = sU[qq];
                  const real a1 = tab.a1[pb + c0 + ia], a2 = tab.a2[pb + c0 + ia];
                  const real ss = sim1 + sim2;
                  const real opb = real(1) + be * T;
                  const real hT = real(0.5) * ebt * T;
                  const real hU = real(0.5) * ebt * opb * U;
                  const real sup1 = a1 * sim2 + a2 * sim1;   // multiplies V1 (slot paired with a1 in sim2)
                  const real sup2 = a1 * sim1 + a2 * sim2;
                  acc[0] += hU * ss + hT * (sup1 * V1 + sup2 * V2);
                  acc[1] += hU * (sim1 * D2 + sim2 * D1) +
                            hT * ((sim2 + a1 * sim2 * D1 + a2 * sim1 * D2) * V1 +
                                  (sim1 + a1 * sim1 * D2 + a2 * sim2 * D1) * V2);
                  acc[2] += hU * (sim1 * D1 + sim2 * D2) +
                            hT * ((sim1 + a2 * sim1 * D1 + a1 * sim2 * D2) * V1 +
                                  (sim2 + a2 * sim2 * D2 + a1 * sim1 * D1) * V2);
                  acc[NV - 1] += hT * (real(2) + be * T) * ss * U + hT * T * (sup1 * V1 + sup2 * V2);
                }
              }
            }
          }
          // ---- combine the subsets of each channel in a fixed order.  `red` is its own region: the
          // previous pass's combine finished before the barrier that followed this pass's staging.
#pragma unroll
          for (int v = 0; v < NV; v++) red[tid * NV + v] = acc[v];
          __syncthreads();
          if (tid < nch * NV) {
            const int ia2 = tid / NV, v = tid - ia2 * NV;
            real s = 0;
            for (int u = 0; u < S; u++) s += red[(u * nch + ia2) * NV + v];
            const int a = tab.ch[pb + c0 + ia2];
            const real c3h = tab.c3[pb + c0 + ia2] * real(0.5);
            if (MODE == 0) {
              out_ch[a] += s * c3h;
            } else if (MODE == 1) {
              acc_par[(sg * Aa + a) * 3 + v] += s * c3h * sP[a];
            } else {
              if (v == 0) out_ch[a] += s * c3h;
              else acc_par[(sg * Aa + a) * 3 + (v - 1)] += s * c3h * sP[a];
            }
          }
          // the next pass starts with a __syncthreads() before red/staging/tables are rewritten
        }
      }
    }
    __syncthreads();
    if (MODE != 1)
      for (int a = tid; a < Aa; a += TRI_BLOCK) A.out[(size_t)atom * Aa + a] = out_ch[a];
    __syncthreads();
  }
  if (MODE != 0) {
    const int nacc = nsig * Aa * 3;
    for (int q = tid; q < nacc; q += TRI_BLOCK) A.partial[(size_t)blockIdx.x * nacc + q] = acc_par[q];
  }
}

}  // namespace staf
