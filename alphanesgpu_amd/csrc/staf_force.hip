// Forces (2-body, 3-body) and the gradients of the force ops.
// Replaces computeforce_doublets_kernel, computeforce_tripl_kernel,
// back_prop_grad_force2b_kernel and gradforce_tripl_kernel
// (STAF/src/force/{rad,ang}/reforce.cu.cc, STAF/src/grad_force/{rad,ang}/reforce.cu.cc).
//
// Force scatter is owner-computes and deterministic: every atom collects the pair forces of the slots that point
// at it, in a fixed order and with a fixed tree -- no floating-point atomics.  Which slots point at an atom comes
// from the neighbour map itself when the library's own search wrote it (symmetric: the atom's own neighbours, the
// slot looked up in the neighbour's row), else from a transposed map (staf_transpose.hpp).
//   2-body op  one kernel, one wave per atom of the frame: it evaluates the pair force of each of its own slots
//              (as a centre of the op's species) and of each slot that lists it (read from that centre's rows).
//   3-body op  pass A (per centre) slot forces -> scratch gslot[b,i,s,3], centre's own force -> self[b,i,3];
//              pass B (per receiving atom) gathers them.
// The 120x re-read of der3b by the reference's gradient kernel (one pass per
// channel and species pair) is gone: der3b is contracted once per triplet with
// dL/dF into three scalars, and all channels are evaluated from those.
#include "staf_tile.hpp"
#include "staf_reduce.hpp"
#include "staf_transpose.hpp"
#include "staf_tri.hpp"

namespace staf {

constexpr int F_BLOCK = 256;
constexpr int F_WAVES = F_BLOCK / WAVE;
constexpr int GRAD_MAX_BLOCKS_F = 1024;  // workgroups (partial rows) of the 2-body force-gradient kernel

// Process-wide switch of the virial forms: 0 = minimum-image wrap of r_i - r_j (periodic box, default),
// 1 = no wrap (neighbours are explicit periodic images).  Same role as staf_force_skip_pbc of the reference
// (STAF/include/staf_force_pbc.cuh:5-10, libstaf/vendor/jmd/src_nn/staf_force_pbc.cu).
static int g_force_skip_pbc = 0;

__device__ inline int species_shift(const int* tipos, const int* actual_type) {
  const int at = actual_type[0];
  int s = 0;
  for (int y = 0; y < at; y++) s += tipos[y];
  return s;
}

}  // namespace staf
#include "staf_force3.hpp"
namespace staf {

// ---------------------------------------------------------------------------
// 2-body force.  One wave per atom a of the frame, lane <-> slot.
//   g(i,s) = 1/2 sum_ch G[i,ch] c2[t,ch] e^{alpha[t,ch] D}(1 + alpha[t,ch] D) * grad D(i,s),  t = species of the
//   neighbour in slot s of centre i
//   F_a = - sum_s g(a,s)  [a is a centre of the op's species]  + sum_{(i,s) listing a} g(i,s)
// The second sum runs over the keys of a in the transposed map whose centre belongs to the op's rows.  VIRIAL: the
// wave also leaves its centre's 3x3 sum - sum_s g(a,s) (x) r(a,s) in vpart.
// ---------------------------------------------------------------------------
template <typename real>
struct Force2Args {
  const real* G;         // [nf, Nl, Ar]
  const real* D;         // raddescr [nf, ld, nr]
  const real* dD;        // der2b [nf, ld, 3, nr]
  const int* im2;        // [nf, ld, nr+1]
  const real* alpha2b;
  const real* emb2b;
  const int* type_map;
  const int* tipos;
  const int* actual_type;
  real* force;           // [nf, 3N]
  real* vpart;           // VIRIAL: [nf, Nl, 9]
  const real* pos;
  const real* box;
  TransposeRef tr;
  int* status;
  int host_shift;        // first atom of the centre species when the host knows it (a view of a descriptor output:
                         // its offset in that tensor), else -1: taken from tipos / actual_type on the device
  int skip_pbc, nf, N, Nl, ld, nr, Ar, nt;
};

template <typename real, bool VIRIAL>
__global__ __launch_bounds__(F_BLOCK) void force2_kernel(Force2Args<real> A) {
  using HE = HotExp<real>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int Ar = A.Ar, nt = A.nt, nr = A.nr, Nl = A.Nl;
  real* p_al = (real*)smem;      // [nt*Ar]
  real* p_c2 = p_al + nt * Ar;   // [nt*Ar]
  for (int q = threadIdx.x; q < nt * Ar; q += blockDim.x) { p_al[q] = A.alpha2b[q]; p_c2[q] = A.emb2b[q]; }
  __syncthreads();
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  const int recv = blockIdx.x * F_WAVES + wave;
  if (recv >= A.nf * A.N) return;
  const int b = recv / A.N, a = recv - b * A.N;
  // The species' first atom: known on the host for a view of a descriptor output, which spares every wave two
  // dependent reads ahead of all its other reads; the device's own figure is then only compared with it.
  const int shift = A.host_shift >= 0 ? A.host_shift : species_shift(A.tipos, A.actual_type);
  if (A.host_shift >= 0 && recv == 0 && lane == 0 && species_shift(A.tipos, A.actual_type) != A.host_shift)
    atomicOr(A.status, 4);
  const int pl = a - shift;
  real f[3] = {0, 0, 0};
  real v[9];
#pragma unroll
  for (int c = 0; c < 9; c++) v[c] = 0;
  // weight of the pair force of slot s of centre row `row` (row of G: gr), neighbour species t
  auto pair_weight = [&](size_t row, size_t gr, int s, int t) -> real {
    const real d = A.D[row * nr + s];
    const real* g = A.G + gr * Ar;
    real w = 0;
    for (int ch = 0; ch < Ar; ch++) {
      const real ad = p_al[t * Ar + ch] * d;
      w += g[ch] * (p_c2[t * Ar + ch] * HE::eval(HE::scale(ad)) * (real(1) + ad));
    }
    return w * real(0.5);
  };
  if (pl >= 0 && pl < Nl) {
    // own slots
    const size_t row = (size_t)b * A.ld + pl;
    const int* im = A.im2 + row * (nr + 1);
    int cnt = im[0];
    if (cnt > nr) cnt = nr;
    for (int s = lane; s < nr; s += WAVE) {
      const int nj = im[1 + s];   // read up to nr, not up to the count just requested: padded slots hold atom 0
      if (s >= cnt) break;
      const real w = pair_weight(row, (size_t)b * Nl + pl, s, A.type_map[nj]);
      real g[3];
#pragma unroll
      for (int c = 0; c < 3; c++) {
        g[c] = w * A.dD[row * 3 * nr + c * nr + s];
        f[c] -= g[c];
      }
      if (VIRIAL) {
        real r[3];
        mic_cart_from_cart(A.pos + ((size_t)b * A.N + a) * 3, A.pos + ((size_t)b * A.N + nj) * 3,
                           A.box + (size_t)b * 6, A.skip_pbc, r);
#pragma unroll
        for (int c = 0; c < 3; c++)
#pragma unroll
          for (int e = 0; e < 3; e++) v[c * 3 + e] -= g[c] * r[e];
      }
    }
  }
  // slots of the op's centres that list this atom
  const int ta = A.type_map[a];
  if (A.tr.symmetric) {
    // the centres that list a are a's own neighbours (row of a in the full map); lane <-> own slot
    const int* mine = A.tr.full + ((size_t)b * A.N + a) * (nr + 1);
    int cnt = mine[0];
    if (cnt > nr) cnt = nr;
    unsigned hsum = 0;
    for (int t = lane; t < nr; t += WAVE) {
      const int i = mine[1 + t];
      if (t >= cnt) break;
      hsum += row_hash(i, t);
      const int p = i - A.tr.key_shift;
      if (p < 0 || p >= Nl) continue;
      const int s = slot_of(A.tr.full, b, A.N, nr, i, a);
      if (s < 0) { atomicOr(A.status, 4); continue; }   // a lists i but i does not list a
      const size_t row = (size_t)b * A.ld + p;
      const real w = pair_weight(row, (size_t)b * Nl + p, s, ta);
#pragma unroll
      for (int c = 0; c < 3; c++) f[c] += w * A.dD[row * 3 * nr + c * nr + s];
    }
    row_check(A.tr, (size_t)b * A.N + a, cnt, hsum, lane, A.status);
  } else {
    const int L = A.tr.cnt[recv];
    const int* keys = A.tr.keys + (size_t)recv * A.tr.cap;
    for (int e = lane; e < L; e += WAVE) {
      const int key = keys[e];
      const int p = key_centre(key) - A.tr.key_shift, s = key_slot(key);
      if (p < 0 || p >= Nl) continue;
      const size_t row = (size_t)b * A.ld + p;
      if (A.im2[row * (nr + 1) + 1 + s] != a) { atomicOr(A.status, 4); continue; }   // the map is not the one transposed
      const real w = pair_weight(row, (size_t)b * Nl + p, s, ta);
#pragma unroll
      for (int c = 0; c < 3; c++) f[c] += w * A.dD[row * 3 * nr + c * nr + s];
    }
  }
#pragma unroll
  for (int c = 0; c < 3; c++) f[c] = wave_sum(f[c]);
  if (lane < 3) A.force[((size_t)b * A.N + a) * 3 + lane] = lane == 0 ? f[0] : (lane == 1 ? f[1] : f[2]);
  if (VIRIAL && pl >= 0 && pl < Nl) {
#pragma unroll
    for (int c = 0; c < 9; c++) {
      const real t = wave_sum(v[c]);
      if (lane == 0) A.vpart[((size_t)b * Nl + pl) * 9 + c] = t;
    }
  }
}

// ---------------------------------------------------------------------------
// Virial forms (ComputeForceRadialVirial / ComputeForceTriplVirial).  The reference adds W_ab -= g_a r_b for
// every pair force g it scatters, r = minimum-image r_centre - r_neighbour.  Summed over the triplets of a
// centre, the pair forces on one slot add up to that slot's entry of gslot, so W = - sum_(centre,slot)
// gslot (x) r: one wave per centre builds its 3x3 contribution, a second kernel adds the centres of a frame
// in ascending order.
// ---------------------------------------------------------------------------
template <typename real>
__global__ __launch_bounds__(F_BLOCK) void virial_centre_kernel(const real* __restrict__ gslot,
                                                                const int* __restrict__ im2,
                                                                const int* __restrict__ counts,
                                                                const real* __restrict__ pos,
                                                                const real* __restrict__ box,
                                                                const int* __restrict__ tipos,
                                                                const int* __restrict__ actual_type,
                                                                real* __restrict__ vpart, int nf, int N, int Nl,
                                                                int ld, int nr, int skip_pbc) {
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  const int atom = blockIdx.x * F_WAVES + wave;
  if (atom >= nf * Nl) return;
  const int b = atom / Nl, p = atom - b * Nl;
  const size_t rowAtom = (size_t)b * ld + p;
  const int* im = im2 + rowAtom * (nr + 1);
  int cnt = counts ? counts[rowAtom] : im[0];
  if (cnt > nr) cnt = nr;
  const int shift = species_shift(tipos, actual_type);
  const real* pi = pos + ((size_t)b * N + p + shift) * 3;
  const real* bx = box + (size_t)b * 6;
  real v[9];
#pragma unroll
  for (int c = 0; c < 9; c++) v[c] = 0;
  for (int s = lane; s < cnt; s += WAVE) {
    const int nj = im[1 + s];
    real r[3];
    mic_cart_from_cart(pi, pos + ((size_t)b * N + nj) * 3, bx, skip_pbc, r);
    const real* g = gslot + ((size_t)atom * nr + s) * 3;
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
      for (int e = 0; e < 3; e++) v[a * 3 + e] -= g[a] * r[e];
  }
#pragma unroll
  for (int c = 0; c < 9; c++) {
    const real t = wave_sum(v[c]);
    if (lane == 0) vpart[(size_t)atom * 9 + c] = t;
  }
}

template <typename real>
__global__ __launch_bounds__(F_BLOCK) void virial_frame_kernel(const real* __restrict__ vpart,
                                                               real* __restrict__ virial, int Nl) {
  __shared__ real sh[F_BLOCK * 9];
  const int b = blockIdx.x, tid = threadIdx.x;
  real v[9];
#pragma unroll
  for (int c = 0; c < 9; c++) v[c] = 0;
  for (int p = tid; p < Nl; p += F_BLOCK)
#pragma unroll
    for (int c = 0; c < 9; c++) v[c] += vpart[((size_t)b * Nl + p) * 9 + c];
#pragma unroll
  for (int c = 0; c < 9; c++) sh[tid * 9 + c] = v[c];
  __syncthreads();
  if (tid < 9) {
    real t = 0;
    for (int u = 0; u < F_BLOCK; u++) t += sh[u * 9 + tid];
    virial[b * 9 + tid] = t;
  }
}

// ---------------------------------------------------------------------------
// 3-body force, pass B: one wave per receiving atom.  The keys of the atom in the transposed map are in ascending
// (centre, slot) order; lane e takes keys e, e + 64, ... whose centre is one of the op's rows, and the lanes are
// added with a fixed tree.  The centre's own force is added when the receiver belongs to the centre species.
// ---------------------------------------------------------------------------
template <typename real>
__global__ __launch_bounds__(F_BLOCK) void gather_kernel(const real* __restrict__ gslot,
                                                         const real* __restrict__ self,
                                                         const int* __restrict__ im2, TransposeRef tr,
                                                         const int* __restrict__ tipos,
                                                         const int* __restrict__ actual_type,
                                                         real* __restrict__ force, int* status, int host_shift,
                                                         int nf, int N, int Nl, int ld, int nr) {
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  const int recv = blockIdx.x * F_WAVES + wave;
  if (recv >= nf * N) return;
  const int b = recv / N, a = recv - b * N;
  // the species' first atom: see force2_kernel
  const int shift = host_shift >= 0 ? host_shift : species_shift(tipos, actual_type);
  if (host_shift >= 0 && recv == 0 && lane == 0 && species_shift(tipos, actual_type) != host_shift)
    atomicOr(status, 4);
  real f[3] = {0, 0, 0};
  if (tr.symmetric) {
    // the centres that list a are a's own neighbours (row of a in the full map); lane <-> own slot
    const int* mine = tr.full + ((size_t)b * N + a) * (nr + 1);
    int cnt = mine[0];
    if (cnt > nr) cnt = nr;
    unsigned hsum = 0;
    for (int t = lane; t < nr; t += WAVE) {
      const int i = mine[1 + t];
      if (t >= cnt) break;
      hsum += row_hash(i, t);
      const int p = i - tr.key_shift;
      if (p < 0 || p >= Nl) continue;
      const int s = slot_of(tr.full, b, N, nr, i, a);
      if (s < 0) { atomicOr(status, 4); continue; }   // a lists i but i does not list a
      const real* g = gslot + (((size_t)b * Nl + p) * nr + s) * 3;
      f[0] += g[0];
      f[1] += g[1];
      f[2] += g[2];
    }
    row_check(tr, (size_t)b * N + a, cnt, hsum, lane, status);
  } else {
    const int L = tr.cnt[recv];
    const int* keys = tr.keys + (size_t)recv * tr.cap;
    for (int e = lane; e < L; e += WAVE) {
      const int key = keys[e];
      const int p = key_centre(key) - tr.key_shift, s = key_slot(key);
      if (p < 0 || p >= Nl) continue;
      if (im2[((size_t)b * ld + p) * (nr + 1) + 1 + s] != a) { atomicOr(status, 4); continue; }
      const real* g = gslot + (((size_t)b * Nl + p) * nr + s) * 3;
      f[0] += g[0];
      f[1] += g[1];
      f[2] += g[2];
    }
  }
#pragma unroll
  for (int c = 0; c < 3; c++) f[c] = wave_sum(f[c]);
  if (lane < 3) {
    real o = lane == 0 ? f[0] : (lane == 1 ? f[1] : f[2]);
    const int pl = a - shift;
    if (pl >= 0 && pl < Nl) o += self[((size_t)b * Nl + pl) * 3 + lane];
    force[((size_t)b * N + a) * 3 + lane] = o;
  }
}

// ---------------------------------------------------------------------------
// Total force in one launch: for every atom the 3-body forces of all centre species (what gather_kernel does per
// species, from the slot forces force3_kernel left) and the per-op force arrays the caller adds to them (the 2-body
// forces), summed in the order 2-body of species 0, 3-body of species 0, 2-body of species 1, ...  One wave per
// atom; the lane sums of a species run over the same lanes in the same tree as in gather_kernel, so the result has
// the bits of the per-op outputs added in that order.  The map must be one the library's own neighbour search
// wrote (symmetric); atoms are species-sorted, first[k] is the first atom of species k.
// ---------------------------------------------------------------------------
template <typename real>
struct TotalArgs {
  const real* gslot[NT_MAX];   // [nf, Nl_k, nr, 3] slot forces of centre species k (null: no 3-body term of k)
  const real* self[NT_MAX];    // [nf, Nl_k, 3]
  const real* f2[NT_MAX];      // [nf, 3N] a per-op force array added ahead of the 3-body term of species k (or null)
  int first[NT_MAX + 1];
  const int* full;             // intmap2b [nf, N, nr+1]
  real* total;                 // [nf, 3N]
  int* status;
  const unsigned* rowsum;   // checksums of the map's rows as written (TransposeRef::rowsum), or null
  int nf, N, nr, nt;
};

template <typename real, int NT>   // NT: species the unrolled selections below cover (nt <= NT)
__global__ __launch_bounds__(F_BLOCK) void force_total_kernel(TotalArgs<real> A) {
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  const int recv = blockIdx.x * F_WAVES + wave;
  if (recv >= A.nf * A.N) return;
  const int nr = A.nr, N = A.N, nt = A.nt;
  const int b = recv / N, a = recv - b * N;
  real acc[NT][3];
#pragma unroll
  for (int k = 0; k < NT; k++) acc[k][0] = acc[k][1] = acc[k][2] = 0;
  const int* mine = A.full + ((size_t)b * N + a) * (nr + 1);
  int cnt = mine[0];
  if (cnt > nr) cnt = nr;
  unsigned hsum = 0;
  for (int t = lane; t < nr; t += WAVE) {
    const int i = mine[1 + t];
    if (t >= cnt) break;
    hsum += row_hash(i, t);
    int k = 0;
#pragma unroll
    for (int q = 1; q < NT; q++) k += (q < nt && i >= A.first[q]) ? 1 : 0;
    const real* gs = nullptr;
#pragma unroll
    for (int q = 0; q < NT; q++) gs = (q == k) ? A.gslot[q] : gs;
    if (!gs) continue;
    const int s = slot_of(A.full, b, N, nr, i, a);
    if (s < 0) { atomicOr(A.status, 4); continue; }   // a lists i but i does not list a
    int f0 = 0, f1 = 0;
#pragma unroll
    for (int q = 0; q < NT; q++) { f0 = (q == k) ? A.first[q] : f0; f1 = (q == k) ? A.first[q + 1] : f1; }
    const real* g = gs + (((size_t)b * (f1 - f0) + (i - f0)) * nr + s) * 3;
    const real g0 = g[0], g1 = g[1], g2 = g[2];
#pragma unroll
    for (int q = 0; q < NT; q++) {
      if (q == k) { acc[q][0] += g0; acc[q][1] += g1; acc[q][2] += g2; }
    }
  }
  {
    const unsigned h = wave_sum_to_last(hsum) + (unsigned)cnt;
    if (lane == WAVE - 1 && A.rowsum && h != A.rowsum[(size_t)b * N + a]) atomicOr(A.status, 4);
  }
  real tot = 0;
  bool have = false;
#pragma unroll
  for (int k = 0; k < NT; k++) {
    if (k >= nt) break;
    if (A.f2[k]) {
      real v = 0;
      if (lane < 3) v = A.f2[k][((size_t)b * N + a) * 3 + lane];
      tot = have ? tot + v : v;
      have = true;
    }
    if (A.gslot[k]) {
      const real s0 = wave_sum(acc[k][0]), s1 = wave_sum(acc[k][1]), s2 = wave_sum(acc[k][2]);
      real o = lane == 0 ? s0 : (lane == 1 ? s1 : s2);
      const int pl = a - A.first[k];
      if (lane < 3 && pl >= 0 && a < A.first[k + 1]) o += A.self[k][((size_t)b * (A.first[k + 1] - A.first[k]) + pl) * 3 + lane];
      tot = have ? tot + o : o;
      have = true;
    }
  }
  if (lane < 3) A.total[((size_t)b * N + a) * 3 + lane] = tot;
}

// ---------------------------------------------------------------------------
// gradient of the 2-body force op.  Q = dL/dF.
//   w_s   = sum_c (Q[j_s,c] - Q[i,c]) * 1/2 dD_s,c
//   dG[a]      = sum_s w_s c2 e(1+alpha D)
//   dalpha[t,a]= sum w_s G[a] c2 e D (2+alpha D),  dc2[t,a] = sum w_s G[a] e (1+alpha D)
// ---------------------------------------------------------------------------
template <typename real>
__global__ __launch_bounds__(F_BLOCK) void gradforce2_kernel(
    const real* __restrict__ Q, const real* __restrict__ G, const real* __restrict__ D, const real* __restrict__ dD,
    const int* __restrict__ im2, const real* __restrict__ alpha2b, const real* __restrict__ emb2b,
    const int* __restrict__ type_map, const int* __restrict__ tipos, const int* __restrict__ actual_type,
    real* __restrict__ gnet, real* __restrict__ partial, const real* __restrict__ Qvir,
    const real* __restrict__ pos, const real* __restrict__ box, int skip_pbc, int nf, int N, int Nl, int ld, int nr,
    int Ar, int nt) {
  using HE = HotExp<real>;
  extern __shared__ __align__(16) unsigned char smem[];
  real* p_al = (real*)smem;                     // [nt*Ar]
  real* p_c2 = p_al + nt * Ar;                  // [nt*Ar]
  real* w_acc = p_c2 + nt * Ar;                 // [F_WAVES][2*nt*Ar]
  real* w_D = w_acc + F_WAVES * 2 * nt * Ar;    // [F_WAVES][nr]  D, w of the slots in grouped order
  real* w_w = w_D + F_WAVES * nr;               // [F_WAVES][nr]
  int* w_t = (int*)(w_w + F_WAVES * nr);        // [F_WAVES][nr]  species of the slot
  int* w_l = w_t + F_WAVES * nr;                // [F_WAVES][nr]  slots grouped by species
  int* w_o = w_l + F_WAVES * nr;                // [F_WAVES][NT_MAX+1]
  for (int q = threadIdx.x; q < nt * Ar; q += blockDim.x) { p_al[q] = alpha2b[q]; p_c2[q] = emb2b[q]; }
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  real* myD = w_D + wave * nr;
  real* myW = w_w + wave * nr;
  int* myT = w_t + wave * nr;
  int* myL = w_l + wave * nr;
  int* myO = w_o + wave * (NT_MAX + 1);
  const int nout = 2 * nt * Ar;
  real* myAcc = w_acc + wave * nout;
  for (int q = lane; q < nout; q += WAVE) myAcc[q] = 0;
  const int shift = species_shift(tipos, actual_type);
  __syncthreads();
  const ChanSub cs(lane, Ar);
  const int total = nf * Nl;
  const int stride = gridDim.x * F_WAVES;
  for (int atom = blockIdx.x * F_WAVES + wave; atom < total; atom += stride) {
    const int b = atom / Nl, p = atom - b * Nl;
    const size_t rowAtom = (size_t)b * ld + p;
    const int* im = im2 + rowAtom * (nr + 1);
    int cnt = im[0];
    if (cnt > nr) cnt = nr;
    for (int s = lane; s < cnt; s += WAVE) myT[s] = type_map[im[1 + s]];
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    group_slots_by_type(cnt, nt, myT, myL, myO);
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    const real* Qi = Q + ((size_t)b * N + p + shift) * 3;
    const real qi0 = Qi[0], qi1 = Qi[1], qi2 = Qi[2];
    for (int q = lane; q < cnt; q += WAVE) {
      const int s = myL[q];
      const int nj = im[1 + s];
      const real* Qj = Q + ((size_t)b * N + nj) * 3;
      const real* dr = dD + rowAtom * 3 * nr + s;
      real q0 = Qj[0] - qi0, q1 = Qj[1] - qi1, q2 = Qj[2] - qi2;
      if (Qvir) {
        // virial form: dL/dg_a = (dL/dF_j - dL/dF_i)_a - sum_e (dL/dW)_ae r_e  (grad_force/rad/reforce.cu.cc:213-216)
        real r[3];
        mic_cart_from_cart(pos + ((size_t)b * N + p + shift) * 3, pos + ((size_t)b * N + nj) * 3, box + (size_t)b * 6,
                           skip_pbc, r);
        const real* Wg = Qvir + (size_t)b * 9;
        q0 -= Wg[0] * r[0] + Wg[1] * r[1] + Wg[2] * r[2];
        q1 -= Wg[3] * r[0] + Wg[4] * r[1] + Wg[5] * r[2];
        q2 -= Wg[6] * r[0] + Wg[7] * r[1] + Wg[8] * r[2];
      }
      myW[q] = real(0.5) * (q0 * dr[0] + q1 * dr[nr] + q2 * dr[2 * nr]);
      myD[q] = D[rowAtom * nr + s];
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    for (int a0 = 0; a0 < Ar; a0 += cs.chunk) {
      const int a = a0 + cs.a;
      const bool on = cs.sub < cs.nsub && a < Ar;
      const real g = on ? G[(size_t)atom * Ar + a] : real(0);
      real dg = 0;
      for (int t = 0; t < nt; t++) {
        const int q0 = uniform(myO[t]), q1 = uniform(myO[t + 1]);
        if (q0 == q1) continue;
        real ga = 0, ge = 0;
        if (on) {
          const real al = p_al[t * Ar + a], c2 = p_c2[t * Ar + a];
          const real als = HE::scale(al);
          for (int q = q0 + cs.sub; q < q1; q += cs.nsub) {
            const real d = myD[q], w = myW[q];
            const real ad = al * d;
            const real we = w * HE::eval(als * d);
            ge += we * (real(1) + ad);           // sum w e (1 + alpha D)
            ga += we * d * (real(2) + ad);       // sum w e D (2 + alpha D)
          }
          dg += c2 * ge;
          ga *= g * c2;
          ge *= g;
        }
        ga = cs.combine(ga, lane);
        ge = cs.combine(ge, lane);
        if (on && cs.sub == 0) { myAcc[t * Ar + a] += ga; myAcc[nt * Ar + t * Ar + a] += ge; }
      }
      dg = cs.combine(dg, lane);
      if (on && cs.sub == 0) gnet[(size_t)atom * Ar + a] = dg;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  __syncthreads();
  for (int q = threadIdx.x; q < nout; q += blockDim.x) {
    real s = 0;
#pragma unroll
    for (int w = 0; w < F_WAVES; w++) s += w_acc[w * nout + q];
    partial[(size_t)blockIdx.x * nout + q] = s;
  }
}

// ---- host launchers --------------------------------------------------------

static inline int grad_blocks_f(int atoms) {
  int nb = (atoms + F_WAVES - 1) / F_WAVES;
  return nb < GRAD_MAX_BLOCKS_F ? nb : GRAD_MAX_BLOCKS_F;
}

// The transposed neighbour map for a force op: the one the descriptor op left beside the tensor `im2` points into,
// or, for any other copy of the map, one built here in the stream's work area (push + sort launches).
static int force_transpose(DeviceState* st, const int* im2, int nf, int N, int Nl, int ld, int nr, hipStream_t stream,
                           TransposeRef* tr, bool* cached) {
  *cached = transpose_find(st, im2, nf, N, Nl, ld, nr, tr);
  if (*cached) return STAF_OK;
  const int cap = 4 * nr;
  if ((size_t)TR_WAVES * cap * sizeof(int) > 64 * 1024) return STAF_E_LIMIT;
  if (!bucket_reserve(st, (size_t)nf * N, cap, stream, tr)) return reserve_failure(stream);
  const int total = nf * Nl * nr;
  hipLaunchKernelGGL(transpose_push_kernel, dim3((total + TR_BLOCK - 1) / TR_BLOCK), dim3(TR_BLOCK), 0, stream, im2,
                     tr->build_cnt, tr->keys, tr->cap, status_word(st, stream), nf, N, Nl, ld, nr);
  launch_transpose_sort(*tr, nf * N, stream);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

// A species without atoms in these frames contributes no force (and no virial): the op still fills its outputs.
template <typename real>
static int empty_species_force(real* force, real* virial, int nf, int N, void* stream_) {
  launch_fill_zero<real>(force, nf * 3 * N, (hipStream_t)stream_);
  if (virial) launch_fill_zero<real>(virial, nf * 9, (hipStream_t)stream_);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

// The same for the gradient of a force op: no centre, so the sums over centres are empty and gradnet has no rows.
template <typename real>
static int empty_species_grad(real* g_alpha, int n_alpha, real* g_emb, int n_emb, void* stream_) {
  launch_fill_zero<real>(g_alpha, n_alpha, (hipStream_t)stream_);
  launch_fill_zero<real>(g_emb, n_emb, (hipStream_t)stream_);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

template <typename real>
int force_doublets(const real* G, const real* D, const real* dD, const int* im2, int nr, int N, int nf, int Ar,
                   const real* alpha2b, const real* emb2b, int nt, const int* tipos, const int* actual_type,
                   real* force, const int* type_map, int Nl, real* virial, const real* pos, const real* box, int ld,
                   int skip_pbc, void* stream_) {
  if ((virial || pos || box) && !(virial && pos && box)) return STAF_E_BAD_ARG;
  if (Nl == 0 && nf > 0 && N > 0 && force) return empty_species_force<real>(force, virial, nf, N, stream_);
  if (!G || !D || !dD || !im2 || !alpha2b || !emb2b || !tipos || !actual_type || !force || !type_map || nr <= 0 ||
      N <= 0 || nf <= 0 || Ar <= 0 || nt <= 0 || Nl <= 0 || Nl > N)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX || nr > (1 << KEY_SLOT_BITS) || N >= (1 << (31 - KEY_SLOT_BITS))) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  hipStream_t stream = (hipStream_t)stream_;
  Force2Args<real> A;
  bool cached = false;
  int rc = force_transpose(st, im2, nf, N, Nl, ld, nr, stream, &A.tr, &cached);
  if (rc) return rc;
  A.G = G; A.D = D; A.dD = dD; A.im2 = im2; A.alpha2b = alpha2b; A.emb2b = emb2b; A.type_map = type_map;
  A.tipos = tipos; A.actual_type = actual_type; A.force = force; A.vpart = nullptr; A.pos = pos; A.box = box;
  A.status = status_word(st, stream); A.skip_pbc = skip_pbc;
  A.host_shift = cached ? A.tr.key_shift : -1;
  A.nf = nf; A.N = N; A.Nl = Nl; A.ld = ld; A.nr = nr; A.Ar = Ar; A.nt = nt;
  if (virial) {
    A.vpart = (real*)scratch_reserve(st, stream, (size_t)nf * Nl * 9 * sizeof(real));
    if (!A.vpart) return reserve_failure(stream);
  }
  const size_t lds = (size_t)2 * nt * Ar * sizeof(real);
  if (lds > 64 * 1024) return STAF_E_LIMIT;
  const int atoms = nf * N;
  {
    KernelTimer kt_("force2_kernel", stream);
    if (virial)
      hipLaunchKernelGGL((force2_kernel<real, true>), dim3((atoms + F_WAVES - 1) / F_WAVES), dim3(F_BLOCK), lds,
                         stream, A);
    else
      hipLaunchKernelGGL((force2_kernel<real, false>), dim3((atoms + F_WAVES - 1) / F_WAVES), dim3(F_BLOCK), lds,
                         stream, A);
  }
  if (virial)
    hipLaunchKernelGGL(virial_frame_kernel<real>, dim3(nf), dim3(F_BLOCK), 0, stream, (const real*)A.vpart, virial,
                       Nl);
  return finish_op(st, stream);
}

template <typename real>
int force_tripl(const real* G, const real* Dsup, const real* Tang, const real* dDsup, const real* d3b,
                const real* unit, const int* im2, const int* im3, int nr, int na, int N, int nf, int Aa,
                const real* emb3b, int nt,
                const int* tipos, const int* actual_type, real* force, const int* numtriplet, const real* alpha3b,
                const int* type_map, int Nl, real* virial, const real* pos, const real* box, int ld, int skip_pbc,
                void* stream_, real* slots_out, real* self_out, const Force2In<real>* two_body) {
  (void)im3;
  if ((virial || pos || box) && !(virial && pos && box)) return STAF_E_BAD_ARG;
  // slots_out / self_out: the slot forces [nf, Nl, nr, 3] and the centres' own forces [nf, Nl, 3] go to the caller
  // instead of the library's work area and no atom gathers them here (force is not written and may be null)
  const bool deferred = slots_out != nullptr;
  if (deferred && (!self_out || virial)) return STAF_E_BAD_ARG;
  // two_body: the 2-body pair forces of the same centres are added to the slot forces (slot outputs only)
  if (two_body && (!deferred || !two_body->G2 || !two_body->D || !two_body->dD || !two_body->alpha2b ||
                   !two_body->emb2b || two_body->Ar <= 0))
    return STAF_E_BAD_ARG;
  if (deferred && Nl == 0) return STAF_OK;
  if (Nl == 0 && nf > 0 && N > 0 && force) return empty_species_force<real>(force, virial, nf, N, stream_);
  if (!G || !Dsup || (!unit && (!Tang || !d3b)) || !dDsup || !im2 || !emb3b || !tipos || !actual_type ||
      (!force && !deferred) ||
      !numtriplet || !alpha3b || !type_map || nr <= 0 || na <= 0 || N <= 0 || nf <= 0 || Aa <= 0 || nt <= 0 ||
      Nl <= 0 || Nl > N)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  hipStream_t stream = (hipStream_t)stream_;
  if (!Force3Cfg<real, 4>::fits(nr, nt) || N >= (1 << (31 - KEY_SLOT_BITS))) return STAF_E_LIMIT;
  TransposeRef tr;
  bool cached = false;
  int rc = deferred ? STAF_OK : force_transpose(st, im2, nf, N, Nl, ld, nr, stream, &tr, &cached);
  if (rc) return rc;
  const size_t ng = (size_t)nf * Nl * nr * 3, ns = (size_t)nf * Nl * 3, nv = virial ? (size_t)nf * Nl * 9 : 0;
  real* gslot = deferred ? slots_out : (real*)scratch_reserve(st, stream, (ng + ns + nv) * sizeof(real));
  if (!gslot) return reserve_failure(stream);
  real* self = deferred ? self_out : gslot + ng;
  real* vpart = self + ns;
  const bool fused = unit != nullptr;   // the MD entry: T and its Jacobian rebuilt from the unit vectors
  // Four waves per workgroup in both precisions.  Eight (Force3Cfg<real, 8>) are faster in single precision when
  // the launch has the GPU to itself (a wave's registers then admit eight waves per SIMD and a centre's critical path
  // is half as long: 32.0 against 34.0 us for 2048 centres) but slower inside a step, where its workgroups share the
  // CUs with those of other launches: an eight-wave workgroup needs two free wave slots on every SIMD of a CU at
  // once and waits while four-wave workgroups around it end one by one (the 3-body force launches of a step held
  // 0.7-0.8 of the wave slots, 0.9 when alone; 4 frames of 768 atoms: 104.1 against 105.8 us per step, 8 frames
  // with the gradient ops: 330 against 345).  In double precision eight measured no faster even alone.
  constexpr int NWV = 4;
  auto launch = [&](auto fused_c, auto w2b_c) -> int {
    constexpr bool FUSED = decltype(fused_c)::value, W2B = decltype(w2b_c)::value;
    using L = Force3Cfg<real, NWV>;
    const size_t lds = L::bytes(nr, Aa, nt, FUSED, W2B ? two_body->Ar : 0);
    if (lds > 64 * 1024) {
      if (lds > 160 * 1024 || hipFuncSetAttribute((const void*)force3_kernel<real, FUSED, NWV, W2B>,
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
        return STAF_E_LIMIT;
    }
    KernelTimer kt_("force3_kernel", stream);
    hipLaunchKernelGGL((force3_kernel<real, FUSED, NWV, W2B>), dim3(nf * Nl), dim3(L::THREADS), lds, stream, G, Dsup,
                       Tang, dDsup, d3b, unit, im2, alpha3b, emb3b, type_map, numtriplet, gslot, self, nf, N, Nl, ld, nr,
                       na, Aa, nt, two_body ? *two_body : Force2In<real>{});
    return STAF_OK;
  };
  using T_ = std::integral_constant<bool, true>;
  using F_ = std::integral_constant<bool, false>;
  rc = fused ? (two_body ? launch(T_{}, T_{}) : launch(T_{}, F_{})) : (two_body ? launch(F_{}, T_{}) : launch(F_{}, F_{}));
  if (rc) return rc;
  if (deferred) return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  if (virial) {
    const int atoms = nf * Nl;
    hipLaunchKernelGGL(virial_centre_kernel<real>, dim3((atoms + F_WAVES - 1) / F_WAVES), dim3(F_BLOCK), 0, stream,
                       (const real*)gslot, im2, numtriplet, pos, box, tipos, actual_type, vpart, nf, N, Nl, ld, nr,
                       skip_pbc);
    hipLaunchKernelGGL(virial_frame_kernel<real>, dim3(nf), dim3(F_BLOCK), 0, stream, (const real*)vpart, virial, Nl);
  }
  {
    KernelTimer kt_("gather_kernel", stream);
    const int recv = nf * N;
    hipLaunchKernelGGL(gather_kernel<real>, dim3((recv + F_WAVES - 1) / F_WAVES), dim3(F_BLOCK), 0, stream,
                       (const real*)gslot, (const real*)self, im2, tr, tipos, actual_type, force, status_word(st, stream),
                       cached ? tr.key_shift : -1, nf, N, Nl, ld, nr);
  }
  return finish_op(st, stream);
}

template int force_doublets<double>(const double*, const double*, const double*, const int*, int, int, int, int,
                                    const double*, const double*, int, const int*, const int*, double*, const int*,
                                    int, double*, const double*, const double*, int, int, void*);
template int force_tripl<double>(const double*, const double*, const double*, const double*, const double*,
                                 const double*, const int*, const int*, int, int, int, int, int, const double*, int,
                                 const int*,
                                 const int*, double*, const int*, const double*, const int*, int, double*,
                                 const double*, const double*, int, int, void*, double*, double*,
                                 const Force2In<double>*);

template <typename real>
static int gradforce_2b(const real* Q, const real* D, int nr, const real* alpha2b, int Ar, const real* dD,
                        const int* im2, int nf, int N, int Nl, const real* G, const real* emb2b, int nt,
                        const int* type_map, const int* tipos, const int* actual_type, real* gnet, real* g_alpha,
                        real* g_emb, const real* Qvir, const real* pos, const real* box, int ld, int skip_pbc,
                        void* stream_) {
  if ((Qvir || pos || box) && !(Qvir && pos && box)) return STAF_E_BAD_ARG;
  if (Nl == 0 && nf > 0 && Ar > 0 && nt > 0 && g_alpha && g_emb)
    return empty_species_grad<real>(g_alpha, nt * Ar, g_emb, nt * Ar, stream_);
  if (!Q || !D || !alpha2b || !dD || !im2 || !G || !emb2b || !type_map || !tipos || !actual_type || !gnet ||
      !g_alpha || !g_emb || nr <= 0 || Ar <= 0 || nf <= 0 || N <= 0 || Nl <= 0 || Nl > N || nt <= 0)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  hipStream_t stream = (hipStream_t)stream_;
  const int nout = 2 * nt * Ar;
  const int nb = grad_blocks_f(nf * Nl);
  real* partial = (real*)scratch_reserve(st, stream, ((size_t)nb + RED_SLICES) * nout * sizeof(real));
  real* red_tmp = partial ? partial + (size_t)nb * nout : nullptr;
  if (!partial) return reserve_failure(stream);
  size_t lds = (size_t)(2 * nt * Ar + F_WAVES * nout + 2 * F_WAVES * nr) * sizeof(real) +
               (size_t)F_WAVES * (2 * nr + NT_MAX + 1) * sizeof(int);
  if (lds > 64 * 1024) return STAF_E_LIMIT;
  {
    KernelTimer kt_("gradforce2_kernel", stream);
    hipLaunchKernelGGL(gradforce2_kernel<real>, dim3(nb), dim3(F_BLOCK), lds, stream, Q, G, D, dD, im2, alpha2b, emb2b,
                       type_map, tipos, actual_type, gnet, partial, Qvir, pos, box, skip_pbc, nf, N, Nl, ld, nr,
                       Ar, nt);
  }
  launch_reduce_partials<real>(partial, nb, nout, g_alpha, nt * Ar, nt * Ar, g_emb, nt * Ar, nt * Ar, red_tmp, stream);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

template <typename real>
static int gradforce_tripl(const real* Q, const real* G, const real* Dsup, const real* Tang, const real* dDsup,
                           const real* d3b, const int* im2, const int* im3, int nr, int na, int N, int nf, int Aa,
                           const real* emb3b, int nt, const int* tipos, const int* actual_type, const int* numtriplet,
                           const real* alpha3b, const int* type_map, int Nl, real* gnet, real* g_alpha, real* g_emb,
                           const real* Qvir, const real* pos, const real* box, int ld, int skip_pbc, void* stream_) {
  (void)im3;
  if ((Qvir || pos || box) && !(Qvir && pos && box)) return STAF_E_BAD_ARG;
  if (Nl == 0 && nf > 0 && Aa > 0 && nt > 0 && g_alpha && g_emb) {
    const int ntc = nt * (nt + 1) / 2;
    return empty_species_grad<real>(g_alpha, ntc * Aa * 3, g_emb, ntc * Aa, stream_);
  }
  if (!Q || !G || !Dsup || !Tang || !dDsup || !d3b || !im2 || !emb3b || !tipos || !actual_type || !numtriplet ||
      !alpha3b || !type_map || !gnet || !g_alpha || !g_emb || nr <= 0 || na <= 0 || N <= 0 || nf <= 0 || Aa <= 0 ||
      nt <= 0 || Nl <= 0 || Nl > N)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  hipStream_t stream = (hipStream_t)stream_;
  const int ntc = nt * (nt + 1) / 2;
  const int nsig = 2 * nt - 1;
  const int nout = nsig * Aa * 3;
  const int nb_max = nf * Nl < TRI_GRID_MAX ? nf * Nl : TRI_GRID_MAX;   // the work area does not depend on occupancy
  real* partial = (real*)scratch_reserve(st, stream, ((size_t)nb_max + RED_SLICES) * nout * sizeof(real));
  real* red_tmp = partial ? partial + (size_t)nb_max * nout : nullptr;
  if (!partial) return reserve_failure(stream);
  size_t lds = TriLds<real, 2>::bytes(nr, Aa, nt);
  if (!lds_request(tri_reduce_kernel<real, 2>, lds)) return STAF_E_LIMIT;
  const int nb = tri_grid((const void*)tri_reduce_kernel<real, 2>, lds, nf * Nl);
  const int nall = ntc * Aa * 3;
  TriArgs<real> A = {};
  A.Dsup = Dsup; A.Tang = Tang; A.im2 = im2; A.alpha3b = alpha3b; A.emb3b = emb3b; A.type_map = type_map;
  A.numtriplet = numtriplet; A.P = G; A.Q = Q; A.dDsup = dDsup; A.d3b = d3b; A.tipos = tipos;
  A.actual_type = actual_type; A.out = gnet; A.partial = partial; A.Qvir = Qvir; A.pos = pos; A.box = box;
  A.skip_pbc = skip_pbc;
  A.nf = nf; A.N = N; A.Nl = Nl; A.ld = ld; A.nr = nr; A.na = na; A.Aa = Aa; A.nt = nt;
  {
    KernelTimer kt_("gradforce3_kernel", stream);
    hipLaunchKernelGGL((tri_reduce_kernel<real, 2>), dim3(nb), dim3(TRI_BLOCK), lds, stream, A);
  }
  // parameter rows sigma >= nsig and the embedding gradient (identically zero in the reference) are zero-filled here
  launch_reduce_partials<real>(partial, nb, nout, g_alpha, nout, nall, g_emb, 0, ntc * Aa, red_tmp, stream);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

// Virial of slot forces (2-body, 3-body or both in one array): W = - sum over centres and radial slots of
// gslot (x) r, r = minimum-image r_centre - r_neighbour (virial_centre_kernel, virial_frame_kernel above).
template <typename real>
int slots_virial(const real* gslot, const int* im2, const real* pos, const real* box, const int* tipos,
                 const int* actual_type, real* virial, int nf, int N, int Nl, int ld, int nr, int skip_pbc,
                 void* stream_) {
  if (!gslot || !im2 || !pos || !box || !tipos || !actual_type || !virial || nf <= 0 || N <= 0 || Nl <= 0 || nr <= 0)
    return STAF_E_BAD_ARG;
  hipStream_t stream = (hipStream_t)stream_;
  DeviceState* st = device_state(stream);
  if (!st) return reserve_failure(stream);
  if (ld <= 0) ld = Nl;
  real* vpart = (real*)scratch_reserve(st, stream, (size_t)nf * Nl * 9 * sizeof(real));
  if (!vpart) return reserve_failure(stream);
  const int atoms = nf * Nl;
  hipLaunchKernelGGL(virial_centre_kernel<real>, dim3((atoms + F_WAVES - 1) / F_WAVES), dim3(F_BLOCK), 0, stream, gslot,
                     im2, (const int*)nullptr, pos, box, tipos, actual_type, vpart, nf, N, Nl, ld, nr, skip_pbc);
  hipLaunchKernelGGL(virial_frame_kernel<real>, dim3(nf), dim3(F_BLOCK), 0, stream, (const real*)vpart, virial, Nl);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}
template int slots_virial<double>(const double*, const int*, const double*, const double*, const int*, const int*,
                                  double*, int, int, int, int, int, int, void*);

template <typename real>
int force_total(const int* im2_full, int nr, int N, int nf, int nt, const int* n_local,
                       const real* const* slot_forces, const real* const* self_forces, const real* const* force_2b,
                       real* total, void* stream_) {
  if (!im2_full || !n_local || !slot_forces || !self_forces || !total || nr <= 0 || N <= 0 || nf <= 0 || nt <= 0)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  hipStream_t stream = (hipStream_t)stream_;
  DeviceState* st = device_state(stream);
  if (!st) return reserve_failure(stream);
  TotalArgs<real> A;
  int sum = 0;
  bool any = false;
  for (int k = 0; k < NT_MAX; k++) {
    A.first[k] = sum;
    A.gslot[k] = A.self[k] = A.f2[k] = nullptr;
    if (k >= nt) continue;
    if (n_local[k] < 0) return STAF_E_BAD_ARG;
    if (n_local[k] > 0 && slot_forces[k]) {
      if (!self_forces[k]) return STAF_E_BAD_ARG;
      A.gslot[k] = slot_forces[k];
      A.self[k] = self_forces[k];
      any = true;
    }
    if (force_2b && force_2b[k]) { A.f2[k] = force_2b[k]; any = true; }
    sum += n_local[k];
  }
  A.first[NT_MAX] = sum;
  for (int k = nt; k < NT_MAX; k++) A.first[k] = sum;
  if (sum != N) return STAF_E_BAD_ARG;
  if (!any) {
    launch_fill_zero<real>(total, nf * 3 * N, stream);
    return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  }
  // the slots that list an atom are found through the atom's own row: only a map the library's own neighbour search
  // wrote, and remembers, is known to be symmetric
  TransposeRef tr;
  if (!transpose_find(st, im2_full, nf, N, N, N, nr, &tr) || !tr.symmetric || tr.key_shift != 0) return STAF_E_BAD_ARG;
  A.full = im2_full; A.total = total; A.status = status_word(st, stream); A.rowsum = tr.rowsum;
  A.nf = nf; A.N = N; A.nr = nr; A.nt = nt;
  {
    KernelTimer kt_("force_total_kernel", stream);
    const int recv = nf * N;
    const dim3 grid((recv + F_WAVES - 1) / F_WAVES);
    if (nt <= 2) hipLaunchKernelGGL((force_total_kernel<real, 2>), grid, dim3(F_BLOCK), 0, stream, A);
    else if (nt <= 4) hipLaunchKernelGGL((force_total_kernel<real, 4>), grid, dim3(F_BLOCK), 0, stream, A);
    else hipLaunchKernelGGL((force_total_kernel<real, NT_MAX>), grid, dim3(F_BLOCK), 0, stream, A);
  }
  return finish_op(st, stream);
}

template int force_total<double>(const int*, int, int, int, int, const int*, const double* const*, const double* const*,
                                 const double* const*, double*, void*);
template int force_total<float>(const int*, int, int, int, int, const int*, const float* const*, const float* const*,
                                const float* const*, float*, void*);

// Both 3-body parameter gradients of a training step in one pass (tri_reduce_kernel<3>): the gradient of the force
// op (gradnet, dL/dalpha3b from dL/dF) and the gradient of the fingerprint op (dL/dalpha3b from dL/dAF3).  Outputs
// as the two separate ops give them; the embedding gradient (identically zero in both, as in the reference) once.
template <typename real>
static int grads_tripl_fused(const real* Q, const real* G, const real* PE, const real* Dsup, const real* Tang,
                             const real* dDsup, const real* d3b, const int* im2, const int* im3, int nr, int na, int N,
                             int nf, int Aa, const real* emb3b, int nt, const int* tipos, const int* actual_type,
                             const int* numtriplet, const real* alpha3b, const int* type_map, int Nl, real* gnet,
                             real* g_alpha_force, real* g_alpha_energy, real* g_emb, const real* Qvir, const real* pos,
                             const real* box, int ld, int skip_pbc, void* stream_) {
  (void)im3;
  if ((Qvir || pos || box) && !(Qvir && pos && box)) return STAF_E_BAD_ARG;
  const int ntc = nt * (nt + 1) / 2;
  if (Nl == 0 && nf > 0 && Aa > 0 && nt > 0 && g_alpha_force && g_alpha_energy && g_emb) {
    launch_fill_zero<real>(g_alpha_force, ntc * Aa * 3, (hipStream_t)stream_);
    launch_fill_zero<real>(g_alpha_energy, ntc * Aa * 3, (hipStream_t)stream_);
    launch_fill_zero<real>(g_emb, ntc * Aa, (hipStream_t)stream_);
    return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  }
  if (!Q || !G || !PE || !Dsup || !Tang || !dDsup || !d3b || !im2 || !emb3b || !tipos || !actual_type || !numtriplet ||
      !alpha3b || !type_map || !gnet || !g_alpha_force || !g_alpha_energy || !g_emb || nr <= 0 || na <= 0 || N <= 0 ||
      nf <= 0 || Aa <= 0 || nt <= 0 || Nl <= 0 || Nl > N)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  hipStream_t stream = (hipStream_t)stream_;
  const int nsig = 2 * nt - 1;
  const int nacc = nsig * Aa * 3, nout = 2 * nacc;
  const int nb_max = nf * Nl < TRI_GRID_MAX ? nf * Nl : TRI_GRID_MAX;   // the work area does not depend on occupancy
  real* partial = (real*)scratch_reserve(st, stream, (size_t)nb_max * nout * sizeof(real));
  if (!partial) return reserve_failure(stream);
  size_t lds = TriLds<real, 3>::bytes(nr, Aa, nt);
  if (!lds_request(tri_reduce_kernel<real, 3>, lds)) return STAF_E_LIMIT;
  const int nb = tri_grid((const void*)tri_reduce_kernel<real, 3>, lds, nf * Nl);
  const int nall = ntc * Aa * 3;
  TriArgs<real> A = {};
  A.Dsup = Dsup; A.Tang = Tang; A.im2 = im2; A.alpha3b = alpha3b; A.emb3b = emb3b; A.type_map = type_map;
  A.numtriplet = numtriplet; A.P = G; A.PE = PE; A.Q = Q; A.dDsup = dDsup; A.d3b = d3b; A.tipos = tipos;
  A.actual_type = actual_type; A.out = gnet; A.partial = partial; A.Qvir = Qvir; A.pos = pos; A.box = box;
  A.skip_pbc = skip_pbc;
  A.nf = nf; A.N = N; A.Nl = Nl; A.ld = ld; A.nr = nr; A.na = na; A.Aa = Aa; A.nt = nt;
  {
    KernelTimer kt_("grads3_kernel", stream);
    hipLaunchKernelGGL((tri_reduce_kernel<real, 3>), dim3(nb), dim3(TRI_BLOCK), lds, stream, A);
  }
  // rows sigma >= nsig of both parameter gradients and the embedding gradient are zero-filled by the same launch
  launch_reduce_partials<real>(partial, nb, nout, g_alpha_force, nacc, nall, g_alpha_energy, nacc, nall, nullptr, stream,
                               g_emb, 0, ntc * Aa);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

}  // namespace staf

extern "C" {

void staf_op_force_set_skip_pbc(int skip) { staf::g_force_skip_pbc = skip ? 1 : 0; }

#define STAF_FORCE_ENTRY(real, SFX)                                                                                    \
  int staf_op_force_doublets_##SFX(const real* netderiv, const real* des_r, const real* intderiv_r,                    \
                                   const int* intmap_r, int nr, int N, int dimbat, int num_alpha_radiale,              \
                                   const real* alpha_radiale, const real* type_emb2b, int nt, const int* tipos,        \
                                   const int* actual_type, real* forces2b, const int* type_map, int N_local,           \
                                   real* virial, const real* pos, const real* box, int ld_atoms, void* stream) {       \
    return staf::force_doublets<real>(netderiv, des_r, intderiv_r, intmap_r, nr, N, dimbat, num_alpha_radiale,         \
                                      alpha_radiale, type_emb2b, nt, tipos, actual_type, forces2b, type_map, N_local,  \
                                      virial, pos, box, ld_atoms, staf::g_force_skip_pbc, stream);                     \
  }                                                                                                                    \
  int staf_op_force_tripl_##SFX(const real* netderiv, const real* desr, const real* desa, const real* intderiv_r,      \
                                const real* intderiv_a, const int* intmap_r, const int* intmap_a, int nr, int na,      \
                                int N, int dimbat, int num_finger, const real* type_emb3b, int nt, const int* tipos,   \
                                const int* actual_type, real* forces3b, const int* num_triplets, const real* smooth_a, \
                                const int* type_map, int N_local, real* virial, const real* pos, const real* box,      \
                                int ld_atoms, void* stream) {                                                          \
    return staf::force_tripl<real>(netderiv, desr, desa, intderiv_r, intderiv_a, (const real*)nullptr, intmap_r,      \
                                   intmap_a, nr, na, N,                                                                \
                                   dimbat, num_finger, type_emb3b, nt, tipos, actual_type, forces3b, num_triplets,     \
                                   smooth_a, type_map, N_local, virial, pos, box, ld_atoms, staf::g_force_skip_pbc,    \
                                   stream, (real*)nullptr, (real*)nullptr, (const staf::Force2In<real>*)nullptr);      \
  }                                                                                                                    \
  int staf_op_force_tripl_slots_##SFX(const real* netderiv, const real* desr, const real* desa,                        \
                                      const real* intderiv_r, const real* intderiv_a, const int* intmap_r,             \
                                      const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,          \
                                      const real* type_emb3b, int nt, const int* tipos, const int* actual_type,        \
                                      real* slot_forces, real* self_forces, const int* num_triplets,                   \
                                      const real* smooth_a, const int* type_map, int N_local, int ld_atoms,            \
                                      void* stream) {                                                                  \
    if (!slot_forces || !self_forces) return STAF_E_BAD_ARG;                                                           \
    return staf::force_tripl<real>(netderiv, desr, desa, intderiv_r, intderiv_a, (const real*)nullptr, intmap_r,      \
                                   intmap_a, nr, na, N, dimbat, num_finger, type_emb3b, nt, tipos, actual_type,        \
                                   (real*)nullptr, num_triplets, smooth_a, type_map, N_local, (real*)nullptr,          \
                                   (const real*)nullptr, (const real*)nullptr, ld_atoms, staf::g_force_skip_pbc,       \
                                   stream, slot_forces, self_forces, (const staf::Force2In<real>*)nullptr);           \
  }                                                                                                                    \
  int staf_op_forces_slots_##SFX(const real* netderiv3b, const real* netderiv2b, const real* desr, const real* desa,   \
                                 const real* intderiv_r, const real* intderiv_a, const real* des_r2b,                  \
                                 const real* intderiv_r2b, const int* intmap_r, const int* intmap_a, int nr, int na,   \
                                 int N, int dimbat, int num_finger, int num_alpha_radiale, const real* type_emb3b,     \
                                 const real* smooth_a, const real* alpha_radiale, const real* type_emb2b, int nt,      \
                                 const int* tipos, const int* actual_type, real* slot_forces, real* self_forces,       \
                                 const int* num_triplets, const int* type_map, int N_local, int ld_atoms,              \
                                 void* stream) {                                                                       \
    if (!slot_forces || !self_forces) return STAF_E_BAD_ARG;                                                           \
    staf::Force2In<real> two;                                                                                          \
    two.G2 = netderiv2b; two.D = des_r2b; two.dD = intderiv_r2b; two.alpha2b = alpha_radiale; two.emb2b = type_emb2b;  \
    two.Ar = num_alpha_radiale;                                                                                        \
    return staf::force_tripl<real>(netderiv3b, desr, desa, intderiv_r, intderiv_a, (const real*)nullptr, intmap_r,    \
                                   intmap_a, nr, na, N, dimbat, num_finger, type_emb3b, nt, tipos, actual_type,        \
                                   (real*)nullptr, num_triplets, smooth_a, type_map, N_local, (real*)nullptr,          \
                                   (const real*)nullptr, (const real*)nullptr, ld_atoms, staf::g_force_skip_pbc,       \
                                   stream, slot_forces, self_forces, &two);                                            \
  }                                                                                                                    \
  int staf_op_force_total_##SFX(const int* intmap_r_full, int nr, int N, int dimbat, int nt, const int* n_local,       \
                                const real* const* slot_forces, const real* const* self_forces,                        \
                                const real* const* forces2b, real* total, void* stream) {                              \
    return staf::force_total<real>(intmap_r_full, nr, N, dimbat, nt, n_local, slot_forces, self_forces, forces2b,      \
                                   total, stream);                                                                     \
  }                                                                                                                    \
  int staf_op_gradforce_2b_##SFX(const real* prevgrad, const real* radiale, int nr, const real* alpha_radiale,         \
                                 int num_finger, const real* desder, const int* intmap_r, int dimbat, int N,           \
                                 int N_local, const real* netderiv, const real* type_emb2b, int nt,                    \
                                 const int* type_map, const int* tipos, const int* actual_type, real* grad_net,        \
                                 real* grad_alpha2b, real* grad_emb2b, const real* prevgrad_virial, const real* pos,   \
                                 const real* box, int ld_atoms, void* stream) {                                        \
    return staf::gradforce_2b<real>(prevgrad, radiale, nr, alpha_radiale, num_finger, desder, intmap_r, dimbat, N,     \
                                    N_local, netderiv, type_emb2b, nt, type_map, tipos, actual_type, grad_net,         \
                                    grad_alpha2b, grad_emb2b, prevgrad_virial, pos, box, ld_atoms,                     \
                                    staf::g_force_skip_pbc, stream);                                                   \
  }                                                                                                                    \
  int staf_op_gradforce_tripl_##SFX(const real* prevgrad, const real* netderiv, const real* desr, const real* desa,    \
                                    const real* intderiv_r, const real* intderiv_a, const int* intmap_r,               \
                                    const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,            \
                                    const real* type_emb3b, int nt, const int* tipos, const int* actual_type,          \
                                    const int* num_triplets, const real* smooth_a, const int* type_map, int N_local,   \
                                    real* gradnet_3b, real* grad_alpha3b, real* grad_emb3b,                            \
                                    const real* prevgrad_virial, const real* pos, const real* box, int ld_atoms,       \
                                    void* stream) {                                                                    \
    return staf::gradforce_tripl<real>(prevgrad, netderiv, desr, desa, intderiv_r, intderiv_a, intmap_r, intmap_a, nr, \
                                       na, N, dimbat, num_finger, type_emb3b, nt, tipos, actual_type, num_triplets,    \
                                       smooth_a, type_map, N_local, gradnet_3b, grad_alpha3b, grad_emb3b,              \
                                       prevgrad_virial, pos, box, ld_atoms, staf::g_force_skip_pbc, stream);           \
  }

STAF_FORCE_ENTRY(float, f32)
STAF_FORCE_ENTRY(double, f64)

#define STAF_FUSED_GRAD_ENTRY(real, SFX)                                                                               \
  int staf_op_grads_tripl_fused_##SFX(                                                                                 \
      const real* prevgrad_force, const real* netderiv, const real* prevgrad_energy, const real* desr,                 \
      const real* desa, const real* intderiv_r, const real* intderiv_a, const int* intmap_r, const int* intmap_a,      \
      int nr, int na, int N, int dimbat, int num_finger, const real* type_emb3b, int nt, const int* tipos,             \
      const int* actual_type, const int* num_triplets, const real* smooth_a, const int* type_map, int N_local,         \
      real* gradnet_3b, real* grad_alpha3b_force, real* grad_alpha3b_energy, real* grad_emb3b,                         \
      const real* prevgrad_virial, const real* pos, const real* box, int ld_atoms, void* stream) {                     \
    return staf::grads_tripl_fused<real>(prevgrad_force, netderiv, prevgrad_energy, desr, desa, intderiv_r,            \
                                         intderiv_a, intmap_r, intmap_a, nr, na, N, dimbat, num_finger, type_emb3b,    \
                                         nt, tipos, actual_type, num_triplets, smooth_a, type_map, N_local,            \
                                         gradnet_3b, grad_alpha3b_force, grad_alpha3b_energy, grad_emb3b,              \
                                         prevgrad_virial, pos, box, ld_atoms, staf::g_force_skip_pbc, stream);         \
  }
STAF_FUSED_GRAD_ENTRY(float, f32)
STAF_FUSED_GRAD_ENTRY(double, f64)

}  // extern "C"
