// Descriptor op: neighbour list under minimum-image PBC + radial and angular
// descriptors with their Jacobians, one kernel launch for the whole batch.
//
// Replaces the reference chain convert_carte_to_int -> celleBuild -> imeBuild ->
// sort_neighbors -> DescriptorsRadial -> DescriptorsAngular
// (STAF/src/descriptor_builder/celle_gpu.cu.cc:11-201, reforce.cu.cc:17-236).
//
// Layout of the work: one 256-thread workgroup per (frame, centre atom).
//   1. all-pairs candidate scan of the frame (positions are a few KB and stay
//      in L2), accepted neighbours compacted into LDS;
//   2. rank sort on the key (dist2, index) -> canonical order, independent of
//      the order candidates arrived in;
//   3. per-slot radial quantities written coalesced along the slot axis and
//      kept in LDS as the neighbour tile (unit vector, 1/r, fc, grad fc);
//   4. the j<k triplets of the tile are enumerated over the lanes, each lane
//      owning consecutive triplet indices so that angdescr / intmap3b / der3b
//      rows are written as contiguous vectors.
// The neighbour list never touches HBM; the only HBM traffic is the position
// read and the nine op outputs.  Every output element is written exactly once,
// padding as 0 -- the reference zeroes angdescr, intmap2b, intmap3b and
// numtriplet before its kernels run (reforce.cc:357-358,375-376,385-386,420-421)
// -- with one exception: der3b beyond an atom's triplets, which the reference
// leaves uninitialised too, is only written when the zero_padding option is set.
#include "staf_common.hpp"
#include "staf_reduce.hpp"
#include "staf_transpose.hpp"
#include "staf_tri.hpp"
#include "staf_af2.hpp"

#include <math.h>
#include <stdio.h>
#include <mutex>

namespace staf {

template <typename real>
struct DescArgs {
  const real* pos;         // [nf, 3*Npos] Cartesian
  const real* box;
  const int* inj_howmany;  // injected neighbour list (else null): [nf, N]
  const int* inj_with;     // [nf, N, nr], sorted by distance, indices into the Npos atoms
  int nf, N, Npos, nr, na;
  int skip_pbc;            // no minimum-image wrap (neighbours carry their periodic image)
  real Rc, Ra, Rs, cA, cB, cC, pa, pb;
  int dist2_fma, zero_padding;
  // cell list of the frames (cell_dims null: every atom is a candidate), see cell_build_kernel
  const int* cell_dims;    // [nf, 8] cells along a, b, c (1: the axis is not divided), number of cells, counter set
  const int* cell_counts;  // [2 sets][cell_set_ints]; of a set: [nf, cell_max] atoms per cell (may exceed cell_cap)
  const void* cell_recs;   // [nf, cell_max, cell_cap] CellRec<real>: position and index of the atoms of every cell
  const int* cell_of;      // [nf, N] cell of every atom: its three coordinates in the grid, 10 bits each
  int* cell_toggle;        // the counter set the next build uses (flipped by this launch)
  size_t cell_set_ints;    // ints between the two counter sets
  int cell_max, cell_cap;  // cells a frame may have, atoms a cell holds
  real* raddescr;
  real* angdescr;
  real* des3bsupp;
  int* intmap2b;
  int* intmap3b;
  real* der2b;
  real* der3b;
  real* der3bsupp;
  int* numtriplet;
  // Radial-only mode of the MD entry: angular = 0 skips the triplet fill (angdescr, intmap3b, der3b are not touched
  // and may be null) and unit receives, per sorted neighbour, the unit vector centre - neighbour and 1/r,
  // [nf, N, 4, nr] -- with des3bsupp and der3bsupp all a 3-body kernel needs to rebuild T and its Jacobian itself.
  real* unit;
  int angular;
  int* status;
  TransposeRef tr;         // transposed neighbour map kept beside intmap2b (receiving atoms: the Npos positions)
};

// Everything that decides an integer output (which atoms are neighbours, their
// order, how many fall inside Ra) is computed without FMA contraction, in the
// operation order of the reference source, so that it matches a plain IEEE
// evaluation bit for bit.
template <typename real>
__device__ inline void inverse_box(const real* b, real* inv) {
#pragma clang fp contract(off)
  inv[0] = real(1.) / b[0];
  inv[1] = -b[1] / (b[0] * b[3]);
  inv[2] = (b[1] * b[4]) / (b[0] * b[3] * b[5]) - b[2] / (b[0] * b[5]);
  inv[3] = real(1.) / b[3];
  inv[4] = -b[4] / (b[3] * b[5]);
  inv[5] = real(1.) / b[5];
}

template <typename real>
__device__ inline void to_frac(const real* inv, real px, real py, real pz, real* s) {
#pragma clang fp contract(off)
  s[0] = (inv[0] * px + inv[1] * py + inv[2] * pz);
  s[1] = (inv[3] * py + inv[4] * pz);
  s[2] = (inv[5] * pz);
}

// d = H * ((sa - sb) - rint(sa - sb)), returns |d|^2 as the neighbour test sees it.
template <typename real>
__device__ inline real mic_delta(const real* box, const real* sa, const real* sb, int fma_mode, int skip_pbc, real* d) {
#pragma clang fp contract(off)
  real ox = sa[0] - sb[0], oy = sa[1] - sb[1], oz = sa[2] - sb[2];
  if (!skip_pbc) {
    ox -= r_rint(ox);
    oy -= r_rint(oy);
    oz -= r_rint(oz);
  }
  d[0] = box[0] * ox + box[1] * oy + box[2] * oz;
  d[1] = box[3] * oy + box[4] * oz;
  d[2] = box[5] * oz;
  if (fma_mode) return r_fma(d[2], d[2], r_fma(d[1], d[1], d[0] * d[0]));
  return (d[0] * d[0] + d[1] * d[1]) + d[2] * d[2];
}

template <typename real>
__device__ inline real norm_plain(const real* d) {
#pragma clang fp contract(off)
  return r_sqrt((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
}

// ---------------------------------------------------------------------------
// Cell list for large frames (replaces the binning kernels of celle_gpu.cu.cc:11-101; the grid rule is this
// library's own).  The box is cut into nx x ny x nz cells in fractional coordinates with every cell at least Rc
// wide measured perpendicular to its faces, so that all atoms within Rc of a centre (minimum image by rounding the
// fractional difference, as the scan does) lie in the centre's cell or one of its 26 neighbours.  An axis with
// fewer than three such cells is not divided (its two neighbours would coincide).
// A cell holds up to `cap` atoms as packed position+index records; a thread per atom takes the atom's place in
// its cell with one atomic add on the cell's counter, so a frame is binned by as many workgroups as it has
// 256-atom pieces (one workgroup per frame, with a prefix sum over the cells between a counting and a fill pass,
// took 13-16 us for 6144 atoms: a single CU's memory pipeline).  The order of the atoms inside a cell is
// arbitrary: the neighbour search sorts what it finds.  A cell that counts more atoms than it holds lacks some of
// them: the search of a centre in or beside such a cell tests every atom of the frame instead.
// The counters must read zero when a build starts.  There are two sets of them: a build takes the set the
// device-side toggle names, clears the whole other set, and the descriptor launch that follows flips the toggle --
// no launch of its own for the clearing, and nothing a replayed graph would have to be told.
// ---------------------------------------------------------------------------
constexpr int CELL_THREADS = 256;

// An atom as the neighbour search reads it: Cartesian position and index in one 16-byte (float) or 32-byte (double)
// record.
template <typename real> struct CellRec;
template <> struct __align__(16) CellRec<float> { float x, y, z; int j; };
template <> struct __align__(16) CellRec<double> { double x, y, z; int j, pad; };

template <typename real>
__global__ __launch_bounds__(CELL_THREADS) void cell_build_kernel(const real* __restrict__ pos, const real* __restrict__ boxes,
                                                         int N, real Rc, const int* __restrict__ toggle,
                                                         size_t set_ints, int cell_max, int cap,
                                                         int* __restrict__ cell_dims, int* __restrict__ counts,
                                                         CellRec<real>* __restrict__ cell_recs,
                                                         int* __restrict__ cell_of) {
  __shared__ int dims[4];
  const int tid = threadIdx.x, b = blockIdx.y;
  const int a = blockIdx.x * CELL_THREADS + tid;
  real box[6], inv[6];
#pragma unroll
  for (int c = 0; c < 6; c++) box[c] = boxes[b * 6 + c];
  const real* pf = pos + (size_t)b * N * 3;
  real px = 0, py = 0, pz = 0;
  if (a < N) { px = pf[3 * a]; py = pf[3 * a + 1]; pz = pf[3 * a + 2]; }
  const int set = toggle[0] & 1;
  // the other set is cleared, all of it (what earlier calls of other shapes counted included)
  {
    int* other = counts + (size_t)(1 - set) * set_ints;
    const size_t step = (size_t)gridDim.x * gridDim.y * CELL_THREADS;
    for (size_t e = ((size_t)b * gridDim.x + blockIdx.x) * CELL_THREADS + tid; e < set_ints; e += step) other[e] = 0;
  }
  inverse_box(box, inv);
  if (tid == 0) {
    // lattice vectors a = (b0,0,0), b = (b1,b3,0), c = (b2,b4,b5); heights = volume / area of the opposite face
    const double ax = box[0], bx = box[1], by = box[3], cx = box[2], cy = box[4], cz = box[5];
    const double vol = fabs(ax * by * cz);
    const double bcx = by * cz, bcy = -bx * cz, bcz = bx * cy - by * cx;   // b x c
    const double cax = 0.0, cay = cz * ax, caz = -cy * ax;                 // c x a
    const double ha = vol / sqrt(bcx * bcx + bcy * bcy + bcz * bcz);
    const double hb = vol / sqrt(cax * cax + cay * cay + caz * caz);
    const double hc = vol / fabs(ax * by);
    int n[3] = {(int)(ha / (double)Rc), (int)(hb / (double)Rc), (int)(hc / (double)Rc)};
    for (int c = 0; c < 3; c++) n[c] = n[c] < 3 ? 1 : (n[c] > 1023 ? 1023 : n[c]);   // (10 bits each in cell_of)
    // coarser cells only widen the search: all axes by the same factor first, then the longest one step at a time
    if ((long long)n[0] * n[1] * n[2] > cell_max) {
      const double f = cbrt((double)cell_max / ((double)n[0] * n[1] * n[2]));
      for (int c = 0; c < 3; c++)
        if (n[c] > 1) {
          int m = (int)(n[c] * f) + 1;
          m = m < 3 ? 3 : m;
          n[c] = m < n[c] ? m : n[c];   // never finer than the cut-off allows
        }
    }
    while ((long long)n[0] * n[1] * n[2] > cell_max) {
      int big = n[0] >= n[1] && n[0] >= n[2] ? 0 : (n[1] >= n[2] ? 1 : 2);
      n[big] = n[big] - 1 < 3 ? 1 : n[big] - 1;
    }
    dims[0] = n[0]; dims[1] = n[1]; dims[2] = n[2]; dims[3] = n[0] * n[1] * n[2];
    if (blockIdx.x == 0) {
      for (int c = 0; c < 4; c++) cell_dims[b * 8 + c] = dims[c];
      cell_dims[b * 8 + 4] = set;
    }
  }
  __syncthreads();
  if (a >= N) return;
  const int nx = dims[0], ny = dims[1], nz = dims[2];
  real s3[3];
  to_frac(inv, px, py, pz, s3);
  int c3[3];
  const int nn[3] = {nx, ny, nz};
#pragma unroll
  for (int c = 0; c < 3; c++) {
    const real f = s3[c] - r_floor(s3[c]);   // [0, 1]
    int q = (int)(f * (real)nn[c]);
    c3[c] = q < 0 ? 0 : (q >= nn[c] ? nn[c] - 1 : q);
  }
  const int cell = (c3[0] * ny + c3[1]) * nz + c3[2];
  cell_of[(size_t)b * N + a] = c3[0] | c3[1] << 10 | c3[2] << 20;
  int* cnt = counts + (size_t)set * set_ints + (size_t)b * cell_max;
  const int slot = atomicAdd(&cnt[cell], 1);
  if (slot < cap) {   // (the centres around a cell whose count has passed its places test every atom of the frame)
    CellRec<real> r;
    r.x = px; r.y = py; r.z = pz; r.j = a;
    cell_recs[((size_t)b * cell_max + cell) * cap + slot] = r;
  }
}

// Zeroes nbytes (a multiple of 4) from p (4-byte aligned), all threads of a 256-thread workgroup calling: single
// words up to the first 16-byte boundary and after the last, 16-byte stores between.
__device__ inline void zero_fill(char* p, unsigned nbytes, int tid) {
  const unsigned head_max = (unsigned)((16 - ((size_t)p & 15)) & 15);
  const unsigned head = head_max < nbytes ? head_max : nbytes;
  const unsigned body = (nbytes - head) & ~15u;
  const unsigned tail = nbytes - head - body;
  if ((unsigned)tid * 4u < head) *(int*)(p + tid * 4u) = 0;
  char* q = p + head;
  for (unsigned o = (unsigned)tid * 16u; o < body; o += 256u * 16u) *(int4*)(q + o) = make_int4(0, 0, 0, 0);
  if ((unsigned)tid * 4u < tail) *(int*)(q + body + tid * 4u) = 0;
}

// Waves per SIMD the allocation is held to: without a bound the single-precision kernel takes 112 scalar registers
// (seven waves: 1792 resident workgroups for the 3072 centres of four 768-atom frames) and the double-precision
// one 104 vector registers (four waves); at eight and five the launch needs fewer rounds of workgroups.
constexpr int DESC_MIN_WAVES_F32 = 8, DESC_MIN_WAVES_F64 = 5, DESC_RADIAL_MIN_WAVES_F64 = 7;
// The kernel's body for the 256-thread workgroup of centre `centre` (frame-major over all N atoms): desc_kernel
// below, and the launch that goes on to the centre's fingerprints in the same workgroup.
template <typename real, bool ANGULAR = true>
__device__ __forceinline__ void desc_body(const DescArgs<real> A, const int centre) {
  using real2 = typename Vec2<real>::type;
  extern __shared__ __align__(16) unsigned char smem[];
  const int nr = A.nr, na = A.na, N = A.N;
  // LDS carve-up
  real* c_d2 = (real*)smem;            // [nr] candidate dist2
  real* c_d = c_d2 + nr;               // [3*nr] candidate delta (neighbour - centre)
  // Per sorted neighbour: unit vector centre - neighbour (3), 1/r, grad of fc wrt d (3), fc, kept as 16-byte pieces
  // in REC_P arrays of nr pieces each (piece q of slot s at s_rec[q * nr + s]): the lanes of a wave hold consecutive
  // triplets, i.e. one j and consecutive k, so a piece of the k records is read from consecutive 16-byte words (no
  // bank conflict) and of the j record as a broadcast, with one address and REC_P wide reads per record.
  using rec_t = typename Vec16<real>::type;
  constexpr int REC_P = 8 * (int)sizeof(real) / 16, REC_N = 16 / (int)sizeof(real);
  rec_t* s_rec = (rec_t*)(c_d + 3 * nr);
  int* c_j = (int*)((real*)s_rec + 8 * nr);   // [nr] candidate index
  int* s_j = c_j + nr;                 // [nr] sorted neighbour index
  int* s_rank = s_j + nr;              // [nr] rank of every candidate
  __shared__ int cnt_all, cnt_ang;
  __shared__ int nb_groups;      // cell search: groups of records to test; -1: a cell holds more atoms than it has places
  __shared__ unsigned row_sum;   // checksum of the row being written (row_hash over its slots)
  __shared__ real sinv[6];

  const int tid = threadIdx.x;
  const int b = centre / N;
  const int i = centre - b * N;
  if (tid == 0) { cnt_all = 0; cnt_ang = 0; row_sum = 0; }
  for (int e = tid; e < nr; e += blockDim.x) s_rank[e] = 0;
  // Box and centre position are the same for the whole workgroup: every thread reads them itself (reads of
  // workgroup-uniform addresses).  The inverse box costs six divisions -- in double precision more instructions
  // than a thread's whole share of the candidate scan -- so one wave computes it for all.
  const real* pf = A.pos + (size_t)b * A.Npos * 3;
  real box[6], inv[6];
#pragma unroll
  for (int c = 0; c < 6; c++) box[c] = A.box[b * 6 + c];
  const real pix = pf[3 * i], piy = pf[3 * i + 1], piz = pf[3 * i + 2];
  if (tid < WAVE) {
    inverse_box(box, inv);
    if (tid < 6) sinv[tid] = tid == 0 ? inv[0] : tid == 1 ? inv[1] : tid == 2 ? inv[2] : tid == 3 ? inv[3]
                                                 : tid == 4 ? inv[4] : inv[5];
  }
  __syncthreads();
#pragma unroll
  for (int c = 0; c < 6; c++) inv[c] = sinv[c];
  real si[3];
  to_frac(inv, pix, piy, piz, si);
  const real rc2 = A.Rc * A.Rc;

  // 1. candidate scan -- or the caller's list (already cut off and sorted by distance)
  const bool injected = A.inj_howmany != nullptr;
  // (the launch that reads a build's counters is the one that hands the next build the other set)
  if (A.cell_dims && blockIdx.x == 0 && tid == 0) A.cell_toggle[0] ^= 1;
  // A candidate within reach takes the next place of the candidate arrays.  The lanes of a wave that have found one
  // take their places together: one add on the counter per wave instead of one per lane (adds of several lanes on one
  // LDS word are done one after the other).
  auto keep = [&](const bool hit, const int j, const real d2, const real (&d)[3]) {
    const unsigned long long m = __ballot(hit);
    if (m == 0) return;
    const int leader = __ffsll((long long)m) - 1;
    int first = 0;
    if ((tid & (WAVE - 1)) == leader) first = atomicAdd(&cnt_all, __popcll(m));
    first = __builtin_amdgcn_readlane(first, leader);
    if (hit) {
      const int slot = first + (int)__builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0));
      if (slot < nr) {
        c_j[slot] = j;
        c_d2[slot] = d2;
        c_d[3 * slot] = d[0];
        c_d[3 * slot + 1] = d[1];
        c_d[3 * slot + 2] = d[2];
      }
    }
  };
  bool by_cells = false;
  if (!injected && A.cell_dims) {
    // Candidates = the atoms of the centre's cell and its neighbours (every atom appears once: an axis has one cell or
    // at least three).  The records of the up to 27 cells are taken in groups of 16 consecutive ones (a cell's last
    // group may be short), listed in a table that lies where the sorted neighbours' records will go: thread <-> place
    // in a group, one table read per candidate, and four candidates per thread are requested before the first is used.
    constexpr int CELLS = 27, BATCH = 4, GROUP = 16;
    int* group = (int*)s_rec;   // [groups] (first record / GROUP) << 5 | records
    const int* dm = A.cell_dims + b * 8;
    const int nx = dm[0], ny = dm[1], nz = dm[2];
    const int* cell_cnt = A.cell_counts + (size_t)dm[4] * A.cell_set_ints + (size_t)b * A.cell_max;
    const int cap = A.cell_cap;   // a multiple of 2 * GROUP
    const CellRec<real>* recs = (const CellRec<real>*)A.cell_recs + (size_t)b * A.cell_max * cap;
    if (tid < WAVE) {   // lane <-> cell
      int c = 0, l = 0;
      if (tid < CELLS) {
        const int ci = A.cell_of[(size_t)b * N + i];
        const int cx = ci & 1023, cy = ci >> 10 & 1023, cz = ci >> 20;
        const int dx = tid / 9 - 1, dy = (tid / 3) % 3 - 1, dz = tid % 3 - 1;
        if ((nx > 1 || dx == 0) && (ny > 1 || dy == 0) && (nz > 1 || dz == 0)) {
          int x = cx + dx, y = cy + dy, z = cz + dz;
          x = x < 0 ? x + nx : (x >= nx ? x - nx : x);
          y = y < 0 ? y + ny : (y >= ny ? y - ny : y);
          z = z < 0 ? z + nz : (z >= nz ? z - nz : z);
          c = (x * ny + y) * nz + z;
          l = cell_cnt[c];
        }
      }
      // groups before a lane's own: a prefix sum over the lanes, register to register (same tree as wave_scan4)
      const unsigned g = (unsigned)(l + GROUP - 1) / GROUP;
      unsigned incl = g + dpp_get<0x111, 0xf>(g);
      incl += dpp_get<0x112, 0xf>(g);
      incl += dpp_get<0x113, 0xf>(g);
      incl += dpp_get<0x114, 0xf>(incl);
      incl += dpp_get<0x118, 0xf>(incl);
      dpp_rows_carry(incl);
      const bool over = __any(l > cap);
      if (tid == CELLS) nb_groups = over ? -1 : (int)incl;   // (this lane has no cell: the sum of all before it)
      if (!over) {
        const int first = (int)(incl - g), base = c * (cap / GROUP);
        for (int k = 0; k < (int)g; k++)
          group[first + k] = (base + k) << 5 | (l - k * GROUP < GROUP ? l - k * GROUP : GROUP);
      }
    }
    __syncthreads();
    // (an overfull cell lacks the records of some of its atoms: this centre then tests every atom of the frame)
    by_cells = nb_groups >= 0;
    const int total = by_cells ? nb_groups * GROUP : 0;
    for (int t0 = 0; t0 < total; t0 += BATCH * 256) {
      CellRec<real> rc_[BATCH];
      bool have[BATCH];
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        const int t = t0 + u * 256 + tid;
        have[u] = false;
        if (t < total) {
          const int w = group[t / GROUP], e = t % GROUP;
          have[u] = e < (w & 31);
          if (have[u]) rc_[u] = recs[(size_t)(w >> 5) * GROUP + e];
        }
      }
#pragma unroll
      for (int u = 0; u < BATCH; u++) {
        real sj[3], d[3] = {0, 0, 0};
        real d2 = rc2;
        int j = i;
        if (have[u]) {
          j = rc_[u].j;
          to_frac(inv, rc_[u].x, rc_[u].y, rc_[u].z, sj);
          d2 = mic_delta(box, sj, si, A.dist2_fma, A.skip_pbc, d);
        }
        keep(d2 < rc2 && j != i, j, d2, d);
      }
    }
  }
  if (by_cells) {
  } else if (!injected) {
    // the position reads of four candidates per thread are issued together
    for (int j0 = tid; j0 < A.Npos; j0 += 4 * 256) {
      real px[4], py[4], pz[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int j = j0 + u * 256;
        px[u] = py[u] = pz[u] = 0;
        if (j < A.Npos) { px[u] = pf[3 * j]; py[u] = pf[3 * j + 1]; pz[u] = pf[3 * j + 2]; }
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int j = j0 + u * 256;
        if (j >= A.Npos) break;
        real sj[3], d[3];
        to_frac(inv, px[u], py[u], pz[u], sj);
        real d2 = mic_delta(box, sj, si, A.dist2_fma, A.skip_pbc, d);
        keep(d2 < rc2 && j != i, j, d2, d);
      }
    }
  } else {
    const int cnt = A.inj_howmany[(size_t)b * N + i];
    if (tid == 0) cnt_all = cnt;
    const int* wl = A.inj_with + ((size_t)b * N + i) * nr;
    for (int e = tid; e < cnt && e < nr; e += blockDim.x) {
      const int j = wl[e];
      real sj[3], d[3];
      to_frac(inv, pf[3 * j], pf[3 * j + 1], pf[3 * j + 2], sj);
      c_d2[e] = mic_delta(box, sj, si, A.dist2_fma, A.skip_pbc, d);
      c_j[e] = j;
      c_d[3 * e] = d[0];
      c_d[3 * e + 1] = d[1];
      c_d[3 * e + 2] = d[2];
    }
  }
  __syncthreads();
  const int hm = cnt_all;
  const int n = hm < nr ? hm : nr;
  if (hm > nr && tid == 0) atomicOr(A.status, 1);

  const size_t atom = (size_t)b * N + i;
  const size_t row = atom * nr;
  const size_t row3 = atom * 3 * nr;
  int* im = A.intmap2b + atom * (nr + 1);
  const real PI = pi_ref<real>();

  // 2. rank of every candidate in (dist2, index) order: the four waves each count a quarter of the others
  if (!injected) {
    const int e = tid & (WAVE - 1), part = tid / WAVE;
    for (int e0 = 0; e0 < n; e0 += WAVE) {
      const int ee = e0 + e;
      if (ee < n) {
        const real d2 = c_d2[ee];
        const int j = c_j[ee];
        int rank = 0;
        for (int o = part; o < n; o += 4) {
          const real od2 = c_d2[o];
          const int oj = c_j[o];
          rank += (od2 < d2 || (od2 == d2 && oj < j)) ? 1 : 0;
        }
        if (rank) atomicAdd(&s_rank[ee], rank);
      }
    }
    __syncthreads();
  }
  // A caller's list: every slot registers with the atom it points at (the transposed map the force ops gather
  // through; the library's own lists are symmetric and need none).  The second wave does it while the first one
  // fills the radial rows.
  if (A.tr.keys && tid >= WAVE && tid < 2 * WAVE) {
    for (int e = tid - WAVE; e < n; e += WAVE)
      transpose_push(A.tr.build_cnt, A.tr.keys, A.tr.cap, (size_t)b * A.Npos + c_j[e], i, injected ? e : s_rank[e],
                     A.status);
  }
  // 3. radial fill
  const bool same_cut = A.Ra == A.Rc;
  const bool std_pow = A.pa == real(1) && A.pb == real(-30);   // the exponents fill_repulsion uses
  unsigned hloc = 0;   // this thread's share of the row's checksum
  for (int e = tid; e < nr; e += blockDim.x) {
    if (e < n) {
      const int j = c_j[e];
      const int rank = injected ? e : s_rank[e];   // the caller's order is kept
      // centre - neighbour: exact negation of the scan's neighbour - centre
      real d[3] = {-c_d[3 * e], -c_d[3 * e + 1], -c_d[3 * e + 2]};
      const real r = norm_plain(d);
      const real invr = real(1) / r;
      real sc, cc;
      r_sincos_0pi(PI * r / A.Rc, &sc, &cc);   // r < Rc: the argument lies in [0, pi]
      real fc = 0, dfc = 0;
      if (r < A.Ra) {
        atomicAdd(&cnt_ang, 1);
        real sa = sc, ca = cc;
        if (!same_cut) r_sincos_0pi(PI * r / A.Ra, &sa, &ca);   // r < Ra
        fc = real(0.5) * (ca + real(1));
        dfc = -real(0.5) * sa * PI / A.Ra;
      }
      real D, dD;
      if (r < A.Rs) {
        if (std_pow) {
          // A/r + B r^30 + C and its derivative, r^30 by squarings
          const real r2 = r * r, r4 = r2 * r2, r8 = r4 * r4, r16 = r8 * r8;
          const real r28 = r16 * r8 * r4, r29 = r28 * r;
          D = A.cA * invr + A.cB * (r29 * r) + A.cC;
          dD = -A.cA * invr * invr + real(30) * A.cB * r29;
        } else {
          D = A.cA / r_pow(r, A.pa) + A.cB / r_pow(r, A.pb) + A.cC;
          dD = -A.pa * A.cA / r_pow(r, A.pa + real(1)) - A.pb * A.cB / r_pow(r, A.pb + real(1));
        }
      } else {
        D = real(0.5) * (cc + real(1));
        dD = -real(0.5) * sc * PI / A.Rc;
      }
      A.raddescr[row + rank] = D;
      A.des3bsupp[row + rank] = fc;
      im[1 + rank] = j;
      hloc += row_hash(j, rank);
      s_j[rank] = j;
      if (A.unit) A.unit[(atom * 4 + 3) * nr + rank] = invr;
      alignas(16) real rec[8];
      rec[3] = invr;
      rec[7] = fc;
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const real u = d[c] * invr;
        A.der2b[row3 + c * nr + rank] = dD * u;
        A.der3bsupp[row3 + c * nr + rank] = dfc * u;
        rec[c] = u;
        rec[4 + c] = dfc * u;
        if (A.unit) A.unit[(atom * 4 + c) * nr + rank] = u;
      }
#pragma unroll
      for (int q = 0; q < REC_P; q++) s_rec[q * nr + rank] = *(const rec_t*)(rec + q * REC_N);
    } else {
      if (A.unit) {
#pragma unroll
        for (int c = 0; c < 4; c++) A.unit[(atom * 4 + c) * nr + e] = 0;
      }
      A.raddescr[row + e] = 0;
      A.des3bsupp[row + e] = 0;
      im[1 + e] = 0;
#pragma unroll
      for (int c = 0; c < 3; c++) {
        A.der2b[row3 + c * nr + e] = 0;
        A.der3bsupp[row3 + c * nr + e] = 0;
      }
    }
  }
  if (A.tr.rowsum && tid < ((nr + WAVE - 1) & ~(WAVE - 1))) {   // the waves that hold slots: a lane sum each, one LDS add per wave
    const unsigned hw = wave_sum_to_last(hloc);
    if ((tid & (WAVE - 1)) == WAVE - 1) atomicAdd(&row_sum, hw);
  }
  __syncthreads();
  const int m = cnt_ang;
  if (tid == 0) {
    im[0] = hm;
    A.numtriplet[atom] = m;
    if (A.tr.rowsum) const_cast<unsigned*>(A.tr.rowsum)[atom] = row_sum + (unsigned)n;
  }

  if (!ANGULAR || !A.angular) return;
  // 4. angular fill: triplet nn <-> (j<k) over the first m sorted neighbours
  int ntr = (m * (m - 1)) / 2;
  if (ntr > na) ntr = na;
  real* ang = A.angdescr + atom * na;
  int2* im3 = (int2*)A.intmap3b + atom * na;
  real2* d3 = (real2*)A.der3b + atom * 3 * na;
  // Consecutive lanes take consecutive triplets: the stores of a wave are whole cache lines.  (Four consecutive
  // triplets per thread with one index decode was measured: fewer instructions, but the strided stores made the
  // kernel a third slower.)  Row bases are workgroup-uniform and element offsets unsigned 32-bit byte counts, so a
  // store's address is a scalar base plus a vector offset.
  char* angp = (char*)ang;
  char* im3p = (char*)im3;
  char* d3p0 = (char*)d3;
  char* d3p1 = (char*)(d3 + na);
  char* d3p2 = (char*)(d3 + 2 * (size_t)na);
  for (unsigned nn = tid; nn < (unsigned)ntr; nn += 256u) {
    int j, k;
    tri_decode((int)nn, m, j, k);
    alignas(16) real rj[8];
    alignas(16) real rk[8];
#pragma unroll
    for (int q = 0; q < REC_P; q++) {
      *(rec_t*)(rj + q * REC_N) = s_rec[q * nr + j];
      *(rec_t*)(rk + q * REC_N) = s_rec[q * nr + k];
    }
    const real uj0 = rj[0], uj1 = rj[1], uj2 = rj[2];
    const real uk0 = rk[0], uk1 = rk[1], uk2 = rk[2];
    const real cs = uj0 * uk0 + uj1 * uk1 + uj2 * uk2;
    const real fj = rj[7], fk = rk[7];
    const real half = real(0.5) * (cs + real(1));
    const real ff = fj * fk;
    const real aj = real(0.5) * rj[3] * ff, ak = real(0.5) * rk[3] * ff;
    const real hk = half * fk, hj = half * fj;
    const unsigned o1 = nn * (unsigned)sizeof(real), o2 = nn * (unsigned)sizeof(real2);
    *(real*)(angp + o1) = half * ff;
    *(int2*)(im3p + nn * 8u) = make_int2(s_j[j], s_j[k]);
    real2 o;
    o.x = aj * (uk0 - cs * uj0) + hk * rj[4];
    o.y = ak * (uj0 - cs * uk0) + hj * rk[4];
    *(real2*)(d3p0 + o2) = o;
    o.x = aj * (uk1 - cs * uj1) + hk * rj[5];
    o.y = ak * (uj1 - cs * uk1) + hj * rk[5];
    *(real2*)(d3p1 + o2) = o;
    o.x = aj * (uk2 - cs * uj2) + hk * rj[6];
    o.y = ak * (uj2 - cs * uk2) + hj * rk[6];
    *(real2*)(d3p2 + o2) = o;
  }
  // angdescr and intmap3b are written over the whole row (the reference zeroes both tensors before its kernels
  // run, STAF/src/descriptor_builder/reforce.cc:357-358,385-386); der3b beyond the triplets only on request
  const unsigned npad = (unsigned)(na - ntr);
  zero_fill(angp + (size_t)ntr * sizeof(real), npad * (unsigned)sizeof(real), tid);
  zero_fill(im3p + (size_t)ntr * 8, npad * 8u, tid);
  if (A.zero_padding) {
    zero_fill(d3p0 + (size_t)ntr * sizeof(real2), npad * (unsigned)sizeof(real2), tid);
    zero_fill(d3p1 + (size_t)ntr * sizeof(real2), npad * (unsigned)sizeof(real2), tid);
    zero_fill(d3p2 + (size_t)ntr * sizeof(real2), npad * (unsigned)sizeof(real2), tid);
  }
}

template <typename real>
__global__ __launch_bounds__(256, sizeof(real) == 4 ? DESC_MIN_WAVES_F32 : DESC_MIN_WAVES_F64) void
desc_kernel(DescArgs<real> A) {
  desc_body<real>(A, (int)blockIdx.x);
}

// The radial-only launch (MD entry) without the code of the triplet fill: fewer registers, more workgroups per CU
// to hide the chain of dependent reads and barriers the search and the sort are.
template <typename real>
__global__ __launch_bounds__(256, sizeof(real) == 4 ? DESC_MIN_WAVES_F32 : DESC_RADIAL_MIN_WAVES_F64) void desc_radial_kernel(DescArgs<real> A) {
  desc_body<real, false>(A, (int)blockIdx.x);
}

template <typename real>
size_t desc_lds_bytes(int nr) {
  return (size_t)nr * (12 * sizeof(real) + 3 * sizeof(int));
}

// ---------------------------------------------------------------------------
// Descriptors and fingerprints of a centre in one workgroup.  A centre's fingerprints need nothing but the rows its
// own descriptor workgroup writes, so the three launches of a step's first stage (descriptors, 2-body and 3-body
// fingerprints of every species) can be one: a workgroup runs the descriptor body, then -- behind a barrier, reading
// back through the cache of its own CU what it has just written -- the 3-body fingerprint body of tri_reduce_kernel
// and, in its first wave, the 2-body fingerprints as af2_kernel computes them (same code, same bits).  No launch
// of the stage then waits for another one's last workgroup, and the species' centres share one grid: entry e of
// the launch is a species, the species with the most centres first.
// ---------------------------------------------------------------------------
template <typename real>
struct Af2Args {
  const real* alpha2b;   // [nt, Ar] of the centre species
  const real* emb2b;     // [nt, Ar]
  real* out;             // [nf, Nl, Ar]
};
template <typename real>
struct FingerprintArgs {
  TriArgs<real> tri[NT_MAX];   // 3-body fingerprint arguments of the entry's species (views of the descriptor outputs)
  Af2Args<real> rad[NT_MAX];
  int first[NT_MAX + 1];       // first workgroup of the entry
  int shift[NT_MAX];           // first atom of the entry's species within a frame
  int entries;
  int Ar;                      // 0: no 2-body fingerprints
  const real* raddescr;        // what the descriptor body writes, for the 2-body part
  const int* intmap2b;
};

template <typename real>
__global__ __launch_bounds__(256, sizeof(real) == 4 ? DESC_MIN_WAVES_F32 : DESC_MIN_WAVES_F64) void
desc_fingerprints_kernel(DescArgs<real> D, FingerprintArgs<real> M) {
  static_assert(TRI_BLOCK == 256 && TriCfg<float, 0>::MIN_WAVES == DESC_MIN_WAVES_F32 &&
                    TriCfg<double, 0>::MIN_WAVES == DESC_MIN_WAVES_F64,
                "both bodies are written for this workgroup size and register budget");
  int e = 0;
  while (e + 1 < M.entries && (int)blockIdx.x >= M.first[e + 1]) e++;
  const TriArgs<real>& T = M.tri[e];
  const int c = (int)blockIdx.x - M.first[e];   // centre within the species, frame-major
  const int b = c / T.Nl, p = c - b * T.Nl;
  const int centre = b * D.N + M.shift[e] + p;
  desc_body<real>(D, centre);
  __syncthreads();   // the rows written above are read below by other threads of this workgroup
  tri_reduce_body<real, 0, false>(T, c, 0x3fffffff, 0);
  if (M.Ar) {
    // (the 3-body body ends behind a barrier: its LDS is free)
    extern __shared__ __align__(16) unsigned char smem[];
    const int Ar = M.Ar, nr = D.nr, npar = T.nt * Ar;
    real* p_al = (real*)smem;
    real* p_c2 = p_al + npar;
    real* myD = p_c2 + npar;
    int* myT = (int*)(myD + nr);
    const Af2Args<real>& R = M.rad[e];
    af2_tables(R.alpha2b, R.emb2b, npar, p_al, p_c2);
    int cnt = 0;
    if (threadIdx.x < WAVE)
      cnt = af2_wave_load(M.raddescr + (size_t)centre * nr, M.intmap2b + (size_t)centre * (nr + 1), T.type_map, nr, Ar,
                          myD, myT, (int)threadIdx.x);
    __syncthreads();
    if (threadIdx.x < WAVE) af2_wave_sum(p_al, p_c2, myD, myT, cnt, Ar, R.out + (size_t)c * Ar, (int)threadIdx.x);
  }
}

template <typename real>
size_t desc_fingerprints_lds_bytes(int nr, int Aa, int Ar, int nt) {
  size_t b = desc_lds_bytes<real>(nr);
  const size_t t = TriLds<real, 0>::bytes(nr, Aa, nt, false);
  const size_t r = (size_t)2 * nt * Ar * sizeof(real) + (size_t)nr * (sizeof(real) + sizeof(int));
  b = b > t ? b : t;
  return b > r ? b : r;
}

// ---- host side -------------------------------------------------------------

static std::mutex g_cfg_mu;
// Frames of at least this many atoms search through a cell list.  Testing every atom of a 4096-atom frame costs a
// centre's workgroup about what the launch that builds the cells costs the call (measured: the search over all
// atoms is 3-8 us per call faster up to 3456 atoms, level at 4608-6144, twice as slow at 20736).
static int g_cell_threshold = 4096;
// Geometry set by construct: one configuration per device and precision.  construct() stores it for the device
// that is current and as the process default, which serves devices construct() was never called on (the
// reference keeps one process-wide configuration, STAF/src/descriptor_builder/reforce.cc:97-158).
template <typename real>
struct CfgStore {
  DescConfig<real> dflt;
  std::unordered_map<int, DescConfig<real>> dev;
  DescConfig<real>& current() {   // g_cfg_mu held
    int d = 0;
    if (hipGetDevice(&d) != hipSuccess) return dflt;
    auto it = dev.find(d);
    return it == dev.end() ? dflt : it->second;
  }
  void store(const DescConfig<real>& c) {   // g_cfg_mu held
    int d = 0;
    if (hipGetDevice(&d) == hipSuccess) dev[d] = c;
    dflt = c;
  }
};
static CfgStore<float> g_cfg_f;
static CfgStore<double> g_cfg_d;
template <typename real> CfgStore<real>& cfg();
template <> CfgStore<float>& cfg<float>() { return g_cfg_f; }
template <> CfgStore<double>& cfg<double>() { return g_cfg_d; }

// Short-range coefficients of D(r) = A/r^alpha + B/r^beta + C matching value,
// slope and curvature of the cosine cutoff at rs; evaluated in `real` like
// fill_repulsion, STAF/src/descriptor_builder/reforce.cc:101-125.
template <typename real>
static void repulsion_coefficients(DescConfig<real>& c) {
  const real PI = pi_ref<real>();
  const real al = 1., be = -30.;
  const real rs = c.Rs, rc = c.Rc;
  const real cs = std::cos(PI * rs / rc), sn = std::sin(PI * rs / rc);
  const real f = 0.5 * (cs + 1);
  const real f1 = -0.5 * PI / rc * sn;
  const real f2r = -0.5 * (PI / rc) * (PI / rc) * cs * (rs * rs);
  const real inv = 1. / (al - be);
  const real gam_r = inv * al - 1;
  const real del_r = inv * (f * (al - be) - f1 * rs - f * al);
  const real eta_r = -al / (al - be);
  const real eps_r = inv * (rs * f1 + al * f);
  const real c2r = al * (al + 1) * del_r + be * (be + 1) * eps_r;
  const real c1r = al * (al + 1) * gam_r + be * (be + 1) * eta_r;
  c.cC = (f2r - c2r) / c1r;
  const real rsb = std::pow(rs, be), rsa = std::pow(rs, al);
  const real eta = -al * rsb / (al - be);
  const real eps = rsb / (al - be) * (rs * f1 + al * f);
  c.cB = eta * c.cC + eps;
  const real gam = rsa / (al - be) * al - rsa;
  const real del = rsa / (al - be) * (f * (al - be) - f1 * rs - f * al);
  c.cA = gam * c.cC + del;
  c.pa = al;
  c.pb = be;
}

template <typename real>
static int construct(real Rc, int nr, int na, int numpar, real Rs, real Ra, int max_batch, const char* curve_path) {
  if (nr <= 0 || na <= 0 || numpar <= 0 || max_batch <= 0 || !(Rc > 0) || !(Ra > 0)) return STAF_E_BAD_ARG;
  if (nr > 1024) return STAF_E_LIMIT;
  DescConfig<real> c;
  c.nr = nr; c.na = na; c.n_max = numpar; c.max_batch = max_batch;
  c.Rc = Rc; c.Rs = Rs; c.Ra = Ra;
  repulsion_coefficients(c);
  c.ready = true;
  if (curve_path) {
    FILE* f = fopen(curve_path, "w");
    if (!f) return STAF_E_BAD_ARG;
    const real PI = pi_ref<real>();
    real dx = Rc / 1000., x = 0;
    for (int k = 0; k < 1000; k++) {
      x = x + dx;
      if (x < Rs)
        fprintf(f, "%g %g\n", x, c.cA / std::pow(x, c.pa) + c.cB / std::pow(x, c.pb) + c.cC);
      else
        fprintf(f, "%g %g\n", x, 0.5 * (1 + std::cos(PI * x / Rc)));
    }
    fclose(f);
  }
  std::lock_guard<std::mutex> lock(g_cfg_mu);
  cfg<real>().store(c);   // the options go back to their defaults: a mode set for an earlier geometry does not linger
  return STAF_OK;
}

// What a descriptor launch goes on to compute for every centre (desc_fingerprints_kernel): host arrays of nt
// device pointers, one per centre species.
template <typename real>
struct FingerprintStep {
  int nt;
  int first_species, n_species;  // the centres of these species only
  const int* n_local;            // host [nt] atoms per species (species-sorted atoms, summing to N)
  const int* type_map;           // device [N]
  int Aa;
  const real* const* alpha3b;    // [ntc, 3*Aa] each
  const real* const* emb3b;      // [ntc, Aa] each
  real* const* af3;              // [nf, n_local[k], Aa] each
  int Ar;                        // 0: no 2-body fingerprints
  const real* const* alpha2b;    // [nt, Ar] each
  const real* const* emb2b;
  real* const* af2;              // [nf, n_local[k], Ar] each
};

template <typename real>
static int desc_launch_impl(const DescConfig<real>& c, const real* pos, const real* box, int nf, int N, int Npos,
                            const int* inj_howmany, const int* inj_with, int skip_pbc, real* raddescr,
                            real* angdescr, real* des3bsupp, int* intmap2b, int* intmap3b, real* der2b, real* der3b,
                            real* der3bsupp, int* numtriplet, real* unit, hipStream_t stream,
                            const FingerprintStep<real>* fp) {
  if (!c.ready) return STAF_E_NOT_CONSTRUCTED;
  const bool angular = unit == nullptr;   // with `unit` the call is radial-only
  if (!pos || !box || !raddescr || !des3bsupp || !intmap2b || !der2b || !der3bsupp || !numtriplet || nf <= 0 ||
      N <= 0 || Npos < N || (inj_howmany && !inj_with) || (angular && (!angdescr || !intmap3b || !der3b)))
    return STAF_E_BAD_ARG;
  DeviceState* st = device_state(stream);
  if (!st) return reserve_failure(stream);
  DescArgs<real> A;
  A.pos = pos; A.box = box; A.nf = nf; A.N = N; A.Npos = Npos; A.nr = c.nr; A.na = c.na;
  A.inj_howmany = inj_howmany; A.inj_with = inj_with; A.skip_pbc = skip_pbc;
  A.Rc = c.Rc; A.Ra = c.Ra; A.Rs = c.Rs; A.cA = c.cA; A.cB = c.cB; A.cC = c.cC; A.pa = c.pa; A.pb = c.pb;
  A.dist2_fma = c.dist2_fma; A.zero_padding = c.zero_padding;
  A.raddescr = raddescr; A.angdescr = angdescr; A.des3bsupp = des3bsupp; A.intmap2b = intmap2b;
  A.intmap3b = intmap3b; A.der2b = der2b; A.der3b = der3b; A.der3bsupp = der3bsupp; A.numtriplet = numtriplet;
  A.unit = unit; A.angular = angular ? 1 : 0;
  A.status = status_word(st, stream);
  if (N >= (1 << (31 - KEY_SLOT_BITS))) return STAF_E_LIMIT;
  // The library's own search finds j from i exactly when it finds i from j (the squared distance is computed from
  // the negated difference vector: same bits), so the map it writes needs no transposing; a caller's list may name
  // ghost atoms, which list nobody, and from more centres than nr.
  const bool symmetric = inj_howmany == nullptr;
  if (!transpose_for_descriptor(st, intmap2b, nf, N, Npos, c.nr, 4 * c.nr, symmetric, stream, &A.tr))
    return reserve_failure(stream);
  A.cell_dims = A.cell_counts = A.cell_of = nullptr;
  A.cell_recs = nullptr;
  const int cell_from = g_cell_threshold;
  // The cell list is built by the launch below, just before the kernel that reads it (and that hands the next
  // build its counters: the two go together).
  auto build_cells = [&]() -> bool {
    if (inj_howmany || cell_from <= 0 || N < cell_from || c.nr < 8) return true;   // (the search keeps a table of
                                                                                   // nr * 27 / 16 + 54 ints in 8 * nr words)
    // A cell is at least Rc wide and at most 4/3 of that per axis, a sphere of radius Rc holds at most nr atoms: a
    // cell of nr places overflows only in frames far denser in one spot than on average (and those are searched
    // atom by atom).  More cells than an eighth of the atoms would be mostly empty.
    const int cap = std::min(256, (c.nr + 31) / 32 * 32);
    // (the search numbers a cell's groups of 16 records in 26 bits)
    const int cell_max = (int)std::min<long long>((1ll << 26) / (cap / 16) - 1, std::max(27, N / 8));
    const size_t counters = (size_t)nf * cell_max;
    const size_t rec_bytes = (size_t)nf * cell_max * cap * sizeof(CellRec<real>);
    const size_t ints = (size_t)nf * (8 + (size_t)N);
    CellBlock blk;
    if (!cells_reserve(st, stream, counters, rec_bytes + ints * sizeof(int), &blk)) return false;
    CellRec<real>* recs = (CellRec<real>*)blk.rest;   // records first (aligned), then the integer tables
    int* dims = (int*)(blk.rest + rec_bytes);
    int* of = dims + (size_t)nf * 8;
    KernelTimer kt_("cell_build_kernel", stream);
    hipLaunchKernelGGL(cell_build_kernel<real>, dim3((N + CELL_THREADS - 1) / CELL_THREADS, nf), dim3(CELL_THREADS), 0,
                       stream, pos, box, N, c.Rc, blk.toggle, blk.set_ints, cell_max, cap, dims, blk.counts, recs, of);
    A.cell_dims = dims; A.cell_counts = blk.counts; A.cell_recs = recs; A.cell_of = of;
    A.cell_toggle = blk.toggle; A.cell_set_ints = blk.set_ints; A.cell_max = cell_max; A.cell_cap = cap;
    return true;
  };
  size_t lds = desc_lds_bytes<real>(c.nr);
  if (lds > 60 * 1024) return STAF_E_LIMIT;
  if (fp) {
    FingerprintArgs<real> M = {};
    const int nt = fp->nt;
    int order[NT_MAX], shift[NT_MAX], sum = 0;
    for (int k = 0; k < nt; k++) { order[k] = k; shift[k] = sum; sum += fp->n_local[k]; }
    // the species with the most centres first (stable): its workgroups are the first to be dispatched
    for (int a = 1; a < nt; a++)
      for (int q = a; q > 0 && fp->n_local[order[q]] > fp->n_local[order[q - 1]]; q--) std::swap(order[q], order[q - 1]);
    int e = 0, wg = 0;
    for (int o = 0; o < nt; o++) {
      const int k = order[o], Nl = fp->n_local[k];
      if (Nl == 0 || k < fp->first_species || k >= fp->first_species + fp->n_species) continue;
      TriArgs<real>& T = M.tri[e];
      T.Dsup = des3bsupp + (size_t)shift[k] * c.nr;
      T.Tang = angdescr + (size_t)shift[k] * c.na;
      T.im2 = intmap2b + (size_t)shift[k] * (c.nr + 1);
      T.numtriplet = numtriplet + shift[k];
      T.alpha3b = fp->alpha3b[k]; T.emb3b = fp->emb3b[k]; T.type_map = fp->type_map; T.out = fp->af3[k];
      T.nf = nf; T.N = N; T.Nl = Nl; T.ld = N; T.nr = c.nr; T.na = c.na; T.Aa = fp->Aa; T.nt = nt;
      if (fp->Ar) { M.rad[e].alpha2b = fp->alpha2b[k]; M.rad[e].emb2b = fp->emb2b[k]; M.rad[e].out = fp->af2[k]; }
      M.first[e] = wg; M.shift[e] = shift[k];
      wg += nf * Nl;
      e++;
    }
    M.first[e] = wg; M.entries = e; M.Ar = fp->Ar; M.raddescr = raddescr; M.intmap2b = intmap2b;
    if (wg == 0) return finish_op(st, stream);   // no centre of these species in the frames
    lds = desc_fingerprints_lds_bytes<real>(c.nr, fp->Aa, fp->Ar, nt);
    if (!lds_request(desc_fingerprints_kernel<real>, lds)) return STAF_E_LIMIT;
    if (!build_cells()) return reserve_failure(stream);
    KernelTimer kt_("desc_fp_kernel", stream);
    hipLaunchKernelGGL(desc_fingerprints_kernel<real>, dim3((unsigned)wg), dim3(256), lds, stream, A, M);
  } else {
    if (!build_cells()) return reserve_failure(stream);
    KernelTimer kt_("desc_kernel", stream);
    if (angular) hipLaunchKernelGGL(desc_kernel<real>, dim3((unsigned)(nf * N)), dim3(256), lds, stream, A);
    else hipLaunchKernelGGL(desc_radial_kernel<real>, dim3((unsigned)(nf * N)), dim3(256), lds, stream, A);
  }
  if (!symmetric) {
    KernelTimer kt_("transpose_sort_kernel", stream);
    launch_transpose_sort(A.tr, nf * Npos, stream);
  }
  return finish_op(st, stream);
}

template <typename real>
int desc_launch(const DescConfig<real>& c, const real* pos, const real* box, int nf, int N, int Npos,
                const int* inj_howmany, const int* inj_with, int skip_pbc, real* raddescr, real* angdescr,
                real* des3bsupp, int* intmap2b, int* intmap3b, real* der2b, real* der3b, real* der3bsupp,
                int* numtriplet, real* unit, hipStream_t stream) {
  return desc_launch_impl<real>(c, pos, box, nf, N, Npos, inj_howmany, inj_with, skip_pbc, raddescr, angdescr,
                                des3bsupp, intmap2b, intmap3b, der2b, der3b, der3bsupp, numtriplet, unit, stream,
                                (const FingerprintStep<real>*)nullptr);
}
template int desc_launch<float>(const DescConfig<float>&, const float*, const float*, int, int, int, const int*,
                                const int*, int, float*, float*, float*, int*, int*, float*, float*, float*, int*,
                                float*, hipStream_t);
template int desc_launch<double>(const DescConfig<double>&, const double*, const double*, int, int, int, const int*,
                                 const int*, int, double*, double*, double*, int*, int*, double*, double*, double*,
                                 int*, double*, hipStream_t);

template <typename real>
int desc_configure(DescConfig<real>& c, real Rc, int nr, int na, real Rs, real Ra) {
  if (nr <= 0 || na <= 0 || !(Rc > 0) || !(Ra > 0)) return STAF_E_BAD_ARG;
  if (nr > 1024) return STAF_E_LIMIT;
  c = DescConfig<real>();
  c.nr = nr; c.na = na; c.Rc = Rc; c.Rs = Rs; c.Ra = Ra;
  repulsion_coefficients(c);
  c.ready = true;
  return STAF_OK;
}
template int desc_configure<double>(DescConfig<double>&, double, int, int, double, double);

template <typename real>
static int compute(const real* pos, const real* box, int nf, int N, real* raddescr, real* angdescr, real* des3bsupp,
                   int* intmap2b, int* intmap3b, real* der2b, real* der3b, real* der3bsupp, int* numtriplet,
                   void* stream_) {
  DescConfig<real> c;
  {
    std::lock_guard<std::mutex> lock(g_cfg_mu);
    c = cfg<real>().current();
  }
  return desc_launch<real>(c, pos, box, nf, N, N, nullptr, nullptr, 0, raddescr, angdescr, des3bsupp, intmap2b,
                           intmap3b, der2b, der3b, der3bsupp, numtriplet, (real*)nullptr, (hipStream_t)stream_);
}

// Descriptors and fingerprints of every species in one launch (the library's own neighbour search, all N atoms
// local).
template <typename real>
static int compute_with_fingerprints(const real* pos, const real* box, int nf, int N, real* raddescr, real* angdescr,
                                     real* des3bsupp, int* intmap2b, int* intmap3b, real* der2b, real* der3b,
                                     real* der3bsupp, int* numtriplet, int nt, const int* n_local,
                                     int first_species, int n_species, const int* type_map, int Aa, const real* const* alpha3b,
                                     const real* const* emb3b, real* const* af3, int Ar, const real* const* alpha2b,
                                     const real* const* emb2b, real* const* af2, void* stream_) {
  if (nt <= 0 || !n_local || first_species < 0 || n_species <= 0 || first_species + n_species > nt || !type_map ||
      Aa <= 0 || !alpha3b || !emb3b || !af3 || Ar < 0 ||
      (Ar > 0 && (!alpha2b || !emb2b || !af2)) || !angdescr)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  long sum = 0;
  for (int k = 0; k < nt; k++) {
    if (n_local[k] < 0) return STAF_E_BAD_ARG;
    sum += n_local[k];
    const bool mine = k >= first_species && k < first_species + n_species;
    if (mine && n_local[k] > 0 && (!alpha3b[k] || !emb3b[k] || !af3[k] || (Ar > 0 && (!alpha2b[k] || !emb2b[k] || !af2[k]))))
      return STAF_E_BAD_ARG;
  }
  if (sum != N) return STAF_E_BAD_ARG;
  DescConfig<real> c;
  {
    std::lock_guard<std::mutex> lock(g_cfg_mu);
    c = cfg<real>().current();
  }
  FingerprintStep<real> fp = {nt, first_species, n_species, n_local, type_map, Aa, alpha3b, emb3b, af3, Ar, alpha2b, emb2b, af2};
  return desc_launch_impl<real>(c, pos, box, nf, N, N, nullptr, nullptr, 0, raddescr, angdescr, des3bsupp, intmap2b,
                                intmap3b, der2b, der3b, der3bsupp, numtriplet, (real*)nullptr,
                                (hipStream_t)stream_, &fp);
}

}  // namespace staf

extern "C" {

int staf_op_descriptors_fingerprints_f32(const float* positions, const float* boxer, int nf, int N, float* raddescr,
                                         float* angdescr, float* des3bsupp, int* intmap2b, int* intmap3b,
                                         float* der2b, float* der3b, float* der3bsupp, int* numtriplet, int nt,
                                         const int* n_local, int first_species, int n_species, const int* type_map,
                                         int nsmooth_a, const float* const* alpha3b, const float* const* type_emb3b,
                                         float* const* three_body_AFs, int nalpha_r, const float* const* alpha2b,
                                         const float* const* type_emb2b, float* const* radial_AFs, void* stream) {
  return staf::compute_with_fingerprints<float>(positions, boxer, nf, N, raddescr, angdescr, des3bsupp, intmap2b,
                                                intmap3b, der2b, der3b, der3bsupp, numtriplet, nt, n_local,
                                                first_species, n_species, type_map, nsmooth_a, alpha3b, type_emb3b, three_body_AFs, nalpha_r, alpha2b,
                                                type_emb2b, radial_AFs, stream);
}
int staf_op_descriptors_fingerprints_f64(const double* positions, const double* boxer, int nf, int N,
                                         double* raddescr, double* angdescr, double* des3bsupp, int* intmap2b,
                                         int* intmap3b, double* der2b, double* der3b, double* der3bsupp,
                                         int* numtriplet, int nt, const int* n_local, int first_species,
                                         int n_species, const int* type_map, int nsmooth_a,
                                         const double* const* alpha3b,
                                         const double* const* type_emb3b, double* const* three_body_AFs,
                                         int nalpha_r, const double* const* alpha2b,
                                         const double* const* type_emb2b, double* const* radial_AFs, void* stream) {
  return staf::compute_with_fingerprints<double>(positions, boxer, nf, N, raddescr, angdescr, des3bsupp, intmap2b,
                                                 intmap3b, der2b, der3b, der3bsupp, numtriplet, nt, n_local,
                                                 first_species, n_species, type_map, nsmooth_a, alpha3b, type_emb3b, three_body_AFs, nalpha_r,
                                                 alpha2b, type_emb2b, radial_AFs, stream);
}

int staf_op_construct_descriptors_light_f32(float rc, int nr, int na, int numpar, float rs, float ra, int max_batch,
                                            const char* path) {
  return staf::construct<float>(rc, nr, na, numpar, rs, ra, max_batch, path);
}
int staf_op_construct_descriptors_light_f64(double rc, int nr, int na, int numpar, double rs, double ra,
                                            int max_batch, const char* path) {
  return staf::construct<double>(rc, nr, na, numpar, rs, ra, max_batch, path);
}

int staf_op_descriptor_cell_threshold(int n_atoms) {
  std::lock_guard<std::mutex> lock(staf::g_cfg_mu);
  staf::g_cell_threshold = n_atoms;
  return STAF_OK;
}

int staf_op_descriptor_options(int dist2_fma, int zero_padding) {
  std::lock_guard<std::mutex> lock(staf::g_cfg_mu);
  auto set = [&](auto& c) { c.dist2_fma = dist2_fma ? 1 : 0; c.zero_padding = zero_padding ? 1 : 0; };
  set(staf::g_cfg_f.current()); set(staf::g_cfg_d.current());
  set(staf::g_cfg_f.dflt); set(staf::g_cfg_d.dflt);
  return STAF_OK;
}

int staf_op_descriptor_coefficients_f32(float* o) {
  std::lock_guard<std::mutex> lock(staf::g_cfg_mu);
  const staf::DescConfig<float>& c = staf::g_cfg_f.current();
  if (!c.ready) return STAF_E_NOT_CONSTRUCTED;
  if (!o) return STAF_E_BAD_ARG;
  o[0] = c.cA; o[1] = c.cB; o[2] = c.cC; o[3] = c.pa; o[4] = c.pb;
  return STAF_OK;
}
int staf_op_descriptor_coefficients_f64(double* o) {
  std::lock_guard<std::mutex> lock(staf::g_cfg_mu);
  const staf::DescConfig<double>& c = staf::g_cfg_d.current();
  if (!c.ready) return STAF_E_NOT_CONSTRUCTED;
  if (!o) return STAF_E_BAD_ARG;
  o[0] = c.cA; o[1] = c.cB; o[2] = c.cC; o[3] = c.pa; o[4] = c.pb;
  return STAF_OK;
}

int staf_op_compute_descriptors_light_f32(const float* pos, const float* box, int nf, int N, float* raddescr,
                                          float* angdescr, float* des3bsupp, int* intmap2b, int* intmap3b,
                                          float* der2b, float* der3b, float* der3bsupp, int* numtriplet,
                                          void* stream) {
  return staf::compute<float>(pos, box, nf, N, raddescr, angdescr, des3bsupp, intmap2b, intmap3b, der2b, der3b,
                              der3bsupp, numtriplet, stream);
}
int staf_op_compute_descriptors_light_f64(const double* pos, const double* box, int nf, int N, double* raddescr,
                                          double* angdescr, double* des3bsupp, int* intmap2b, int* intmap3b,
                                          double* der2b, double* der3b, double* der3bsupp, int* numtriplet,
                                          void* stream) {
  return staf::compute<double>(pos, box, nf, N, raddescr, angdescr, des3bsupp, intmap2b, intmap3b, der2b, der3b,
                               der3bsupp, numtriplet, stream);
}

}  // extern "C"
