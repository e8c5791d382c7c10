// TEST INFRASTRUCTURE ONLY -- CPU oracle for the STAF fingerprint hot path.
//
// A scalar C++ restatement of the reference's CUDA kernels, one function per
// op, with the op's exact tensor layouts.  It exists to check the HIP library;
// nothing in the product may link, import or call it.  Only tests/, the smoke
// entry and the cpu_baseline leg of the benchmark use it.
//
// Single templated source, instantiated for float and double.  The reference
// fp32 build evaluates several sub-expressions in double because of untyped
// literals (0.5, 1.); those expressions are written here with the same literal
// types so that ordinary C++ promotion reproduces them.  Build with
// -ffp-contract=off (see Makefile): no FMA contraction anywhere.
//
// Conventions: nf frames, N atoms per frame, nr radial buffer, na angular
// buffer, box6 = [Lx, xy, xz, Ly, yz, Lz].  Padded slots of every output are
// written as 0 (the reference leaves raddescr/des3bsupp/der2b/der3bsupp/der3b
// padding uninitialised; comparisons must mask by the counts).
// Sums that the reference accumulates with atomicAdd (arbitrary order) are
// accumulated here in (frame, atom, slot, channel) loop order, in `real`.
//
// Pinning status (what fixes each function besides this restatement) is kept
// in tests/test_oracle_*.py; functions with no independent check are listed
// there as "parity unpinned" -- currently none.

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include <algorithm>
#include <chrono>

namespace {

template <typename real> struct M;
template <> struct M<float> {
  static float exp(float x) { return expf(x); }
  static float cos(float x) { return cosf(x); }
  static float sin(float x) { return sinf(x); }
  static float sqrt(float x) { return sqrtf(x); }
  static float pow(float x, float n) { return powf(x, n); }
  static float rint(float x) { return rintf(x); }
};
template <> struct M<double> {
  static double exp(double x) { return ::exp(x); }
  static double cos(double x) { return ::cos(x); }
  static double sin(double x) { return ::sin(x); }
  static double sqrt(double x) { return ::sqrt(x); }
  static double pow(double x, double n) { return ::pow(x, n); }
  static double rint(double x) { return ::rint(x); }
};

// STAF/src/descriptor_builder/reforce.cu.cc:15 and reforce.cc:23 -- the
// reference uses this 10-digit literal, not pi.
template <typename real> inline real PIc() { return real(3.141592654); }

template <typename real> inline real sqr(real x) { return x * x; }

// ---------------------------------------------------------------------------
// fill_repulsion -- STAF/src/descriptor_builder/reforce.cc:101-141
// Coefficients A,B,C of D(r)=A/r^alpha+B/r^beta+C (alpha=1, beta=-30) joining
// the cosine cutoff at rs with continuous value, slope and curvature.
// out5 = {A, B, C, alpha, beta}
// ---------------------------------------------------------------------------
template <typename real>
void fill_repulsion(real rc, real rs, real* out5) {
  const real PI = PIc<real>();
  real alpha = 1.;
  real beta = -30.;
  real f = 0.5 * (M<real>::cos(PI * rs / rc) + 1);
  real f1 = -0.5 * PI / rc * M<real>::sin(PI * rs / rc);
  real f2_red = -0.5 * sqr(PI / rc) * M<real>::cos(PI * rs / rc) * sqr(rs);
  real gamma_red = 1. / (alpha - beta) * alpha - 1;
  real delta_red = 1. / (alpha - beta) * (f * (alpha - beta) - f1 * rs - f * alpha);
  real eta_red = -alpha / (alpha - beta);
  real epsilon_red = 1. / (alpha - beta) * (rs * f1 + alpha * f);
  real c2_red = alpha * (alpha + 1) * delta_red + beta * (beta + 1) * epsilon_red;
  real c1_red = alpha * (alpha + 1) * gamma_red + beta * (beta + 1) * eta_red;
  real C = (f2_red - c2_red) / c1_red;
  real eta = -alpha * M<real>::pow(rs, beta) / (alpha - beta);
  real epsilon = M<real>::pow(rs, beta) / (alpha - beta) * (rs * f1 + alpha * f);
  real B = eta * C + epsilon;
  real gamma = M<real>::pow(rs, alpha) / (alpha - beta) * alpha - M<real>::pow(rs, alpha);
  real delta = M<real>::pow(rs, alpha) / (alpha - beta) * (f * (alpha - beta) - f1 * rs - f * alpha);
  real A = gamma * C + delta;
  out5[0] = A; out5[1] = B; out5[2] = C; out5[3] = alpha; out5[4] = beta;
}

// cutoff_curve.dat rows -- STAF/src/descriptor_builder/reforce.cc:127-140
template <typename real>
void cutoff_curve(real rc, real rs, const real* c5, int n, real* xs, real* ys) {
  const real PI = PIc<real>();
  real dx = rc / 1000.;
  real x = 0;
  for (int k = 0; k < n; k++) {
    x = x + dx;
    xs[k] = x;
    if (x < rs)
      ys[k] = c5[0] / M<real>::pow(x, c5[3]) + c5[1] / M<real>::pow(x, c5[4]) + c5[2];
    else
      ys[k] = 0.5 * (1 + M<real>::cos(PI * x / rc));
  }
}

// ---------------------------------------------------------------------------
// inverse box -- STAF/src/descriptor_builder/reforce.cc:283-299 (host, in real)
// ---------------------------------------------------------------------------
template <typename real>
void inverse_box(const real* b, real* inv) {
  inv[0] = real(1.) / b[0];
  inv[1] = -b[1] / (b[0] * b[3]);
  inv[2] = (b[1] * b[4]) / (b[0] * b[3] * b[5]) - b[2] / (b[0] * b[5]);
  inv[3] = real(1.) / b[3];
  inv[4] = -b[4] / (b[3] * b[5]);
  inv[5] = real(1.) / b[5];
}

// cart -> frac -- STAF/src/descriptor_builder/celle_gpu.cu.cc:11-28
template <typename real>
void cart_to_frac(int nf, int N, const real* pos, const real* box, real* frac) {
  for (int b = 0; b < nf; b++) {
    real inv[6];
    inverse_box(box + 6 * b, inv);
    for (int p = 0; p < N; p++) {
      real px = pos[(b * N + p) * 3 + 0], py = pos[(b * N + p) * 3 + 1], pz = pos[(b * N + p) * 3 + 2];
      frac[(b * N + p) * 3 + 0] = (inv[0] * px + inv[1] * py + inv[2] * pz);
      frac[(b * N + p) * 3 + 1] = (inv[3] * py + inv[4] * pz);
      frac[(b * N + p) * 3 + 2] = (inv[5] * pz);
    }
  }
}

// minimum-image Cartesian separation from fractional coordinates, sign
// convention s_a - s_b.  celle_gpu.cu.cc:95-107 (a = neighbour, b = centre),
// reforce.cu.cc:56-67 (a = centre, b = neighbour).
template <typename real>
inline void mic_cart(const real* sa, const real* sb, const real* box, real* d) {
  real ox = sa[0] - sb[0], oy = sa[1] - sb[1], oz = sa[2] - sb[2];
  ox -= M<real>::rint(ox);
  oy -= M<real>::rint(oy);
  oz -= M<real>::rint(oz);
  d[0] = box[0] * ox + box[1] * oy + box[2] * oz;
  d[1] = box[3] * oy + box[4] * oz;
  d[2] = box[5] * oz;
}

// dist2 = x^2+y^2+z^2 -- celle_gpu.cu.cc:109.  The only contraction-sensitive
// expression that decides an integer output.  fma_mode 0: ((x*x)+(y*y))+(z*z)
// (what an uncontracted build and the legacy CPU list, cell_list.cu.cc:1147-1159,
// compute); fma_mode 1: fma(z,z,fma(y,y,x*x)) (nvcc --fmad=true contraction).
template <typename real>
inline real dist2_of(const real* d, int fma_mode) {
  if (fma_mode) return std::fma(d[2], d[2], std::fma(d[1], d[1], d[0] * d[0]));
  return sqr(d[0]) + sqr(d[1]) + sqr(d[2]);
}

// ---------------------------------------------------------------------------
// cell grid -- celleCompute, celle_gpu.cu.cc:203-228
// ---------------------------------------------------------------------------
template <typename real>
void cell_dims(const real* box, real cutoff, int N, int* nxyz) {
  real volume = box[0] * box[3] * box[5];
  int nx = (int)(volume / (std::sqrt(box[3] * box[3] * box[5] * box[5] + box[5] * box[5] * box[1] * box[1] +
                                     box[3] * box[3] * box[2] * box[2] + box[4] * box[4] * box[1] * box[1]) *
                           cutoff));
  int ny = (int)(volume / (box[0] * std::sqrt(box[5] * box[5] + box[4] * box[4]) * cutoff));
  int nz = (int)(volume / (box[0] * box[3] * cutoff));
  while ((nx * ny * nz > 27) && (nx * ny * nz > N)) {
    int* mx = (nx > ny ? &nx : &ny);
    mx = (*mx > nz ? mx : &nz);
    (*mx)--;
  }
  if (nx < 3) nx = 3;
  if (ny < 3) ny = 3;
  if (nz < 3) nz = 3;
  nxyz[0] = nx; nxyz[1] = ny; nxyz[2] = nz;
}

// stable insertion sort by dist2 -- sort_neighbors, celle_gpu.cu.cc:128-152
template <typename real>
void sort_row(int* w, real* r2, int n) {
  for (int a = 1; a < n; ++a) {
    real kr = r2[a];
    int kw = w[a];
    int b = a - 1;
    while (b >= 0 && r2[b] > kr) { r2[b + 1] = r2[b]; w[b + 1] = w[b]; --b; }
    r2[b + 1] = kr; w[b + 1] = kw;
  }
}

// ---------------------------------------------------------------------------
// neighbour list, all-pairs form.  Same acceptance test and sort as
// imeBuild + sort_neighbors (celle_gpu.cu.cc:40-152); candidates arrive in
// ascending j, so exact dist2 ties end in ascending j (the reference's tie
// order is the arrival order of atomicAdd in celleBuild, i.e. unspecified).
// howmany keeps counting past nr; only the first nr arrivals are stored
// (celle_gpu.cu.cc:111-117).  Returns max(howmany).
// ---------------------------------------------------------------------------
template <typename real>
int neighbor_list(int nf, int N, const real* frac, const real* box, real cutoff, int nr, int fma_mode,
                  int* with, real* with_d2, int* howmany) {
  int mx = 0;
  for (int b = 0; b < nf; b++) {
    const real* bx = box + 6 * b;
    for (int i = 0; i < N; i++) {
      int cnt = 0;
      int* w = with + ((size_t)b * N + i) * nr;
      real* r2 = with_d2 + ((size_t)b * N + i) * nr;
      for (int k = 0; k < nr; k++) { w[k] = 0; r2[k] = 0; }
      for (int j = 0; j < N; j++) {
        real d[3];
        mic_cart(frac + ((size_t)b * N + j) * 3, frac + ((size_t)b * N + i) * 3, bx, d);
        real d2 = dist2_of(d, fma_mode);
        if (d2 < cutoff * cutoff && i != j) {
          int slot = cnt++;
          if (slot < nr) { w[slot] = j; r2[slot] = d2; }
        }
      }
      howmany[b * N + i] = cnt;
      sort_row(w, r2, cnt < nr ? cnt : nr);
      if (cnt > mx) mx = cnt;
    }
  }
  return mx;
}

// neighbour list through the linked-cell grid, as the reference launches it:
// celleBuild (celle_gpu.cu.cc:176-201) with atoms entered in ascending index
// (one of the orders the atomicAdd there can produce), imeBuild over the 27
// neighbour cells in the (i,j,k) loop order of celle_gpu.cu.cc:58-82, then
// sort_neighbors.  MAX_PARTICLE_CELLS as reforce.cc:306-309, atoms beyond it
// in a cell are dropped as in the reference.  Returns max(howmany).
template <typename real>
int neighbor_list_cells(int nf, int N, const real* frac, const real* box, real cutoff, int nr, int fma_mode,
                        int* with, real* with_d2, int* howmany) {
  int mpc = N / 3;
  if (mpc < 1) mpc = 1;
  if (mpc > 256) mpc = 256;
  int mx = 0;
  for (int b = 0; b < nf; b++) {
    const real* bx = box + 6 * b;
    const real* s = frac + (size_t)b * N * 3;
    int n3[3];
    cell_dims(bx, cutoff, N, n3);
    int nx = n3[0], ny = n3[1], nz = n3[2];
    real cx = real(1.) / (real)nx, cy = real(1.) / (real)ny, cz = real(1.) / (real)nz;
    std::vector<int> cells((size_t)nx * ny * nz * mpc, 0), chow((size_t)nx * ny * nz, 0);
    for (int t = 0; t < N; t++) {
      int px = (int)std::floor(s[3 * t + 0] / cx); px = px % nx; while (px < 0) px += nx;
      int py = (int)std::floor(s[3 * t + 1] / cy); py = py % ny; while (py < 0) py += ny;
      int pz = (int)std::floor(s[3 * t + 2] / cz); pz = pz % nz; while (pz < 0) pz += nz;
      int c = px + py * nx + pz * (nx * ny);
      int n = chow[c]++;
      if (n < mpc) cells[(size_t)c * mpc + n] = t;
    }
    int* hm = howmany + b * N;
    for (int i = 0; i < N; i++) hm[i] = 0;
    for (size_t q = 0; q < (size_t)N * nr; q++) { with[(size_t)b * N * nr + q] = 0; with_d2[(size_t)b * N * nr + q] = 0; }
    for (int bz = 0; bz < nz; bz++) for (int by = 0; by < ny; by++) for (int bxi = 0; bxi < nx; bxi++) {
      int cc = bxi + by * nx + bz * nx * ny;
      int ncc = chow[cc] < mpc ? chow[cc] : mpc;
      for (int di = -1; di < 2; di++) {
        int bi = bxi + di; if (bi < 0) bi = nx - 1; else if (bi == nx) bi = 0;
        for (int dj = -1; dj < 2; dj++) {
          int bj = by + dj; if (bj < 0) bj = ny - 1; else if (bj == ny) bj = 0;
          for (int dk = -1; dk < 2; dk++) {
            int bk = bz + dk; if (bk < 0) bk = nz - 1; else if (bk == nz) bk = 0;
            int nc = bi + bj * nx + bk * nx * ny;
            int nnc = chow[nc] < mpc ? chow[nc] : mpc;
            for (int ti = 0; ti < ncc; ti++) {
              int me = cells[(size_t)cc * mpc + ti];
              for (int n = 0; n < nnc; n++) {
                int he = cells[(size_t)nc * mpc + n];
                real d[3];
                mic_cart(s + 3 * he, s + 3 * me, bx, d);
                real d2 = dist2_of(d, fma_mode);
                if (d2 < cutoff * cutoff && me != he) {
                  int slot = hm[me]++;
                  if (slot < nr) {
                    with[((size_t)b * N + me) * nr + slot] = he;
                    with_d2[((size_t)b * N + me) * nr + slot] = d2;
                  }
                }
              }
            }
          }
        }
      }
    }
    for (int i = 0; i < N; i++) {
      sort_row(with + ((size_t)b * N + i) * nr, with_d2 + ((size_t)b * N + i) * nr, hm[i] < nr ? hm[i] : nr);
      if (hm[i] > mx) mx = hm[i];
    }
  }
  return mx;
}

// ---------------------------------------------------------------------------
// DescriptorsRadial_kernel -- STAF/src/descriptor_builder/reforce.cu.cc:17-110
// Npos = atoms per frame in `frac` (N for the training ops; nlocal+nghost for
// the libstaf variant); skip_pbc != 0 drops the rint() (ghost images,
// libstaf/vendor/jmd/src_nn/descriptor_builder/reforce.cu:17-23).
// ---------------------------------------------------------------------------
template <typename real>
void descriptors_radial(int nf, int N, int Npos, int nr, const real* frac, const real* box, const int* howmany,
                        const int* with, real Rc, real Ra, real rs, real cA, real cB, real cC, real pa, real pb,
                        int skip_pbc, real* raddescr, int* intmap2b, real* der2b, real* des3bsupp, real* der3bsupp,
                        int* numtriplet) {
  const real PI = PIc<real>();
  for (int b = 0; b < nf; b++) {
    const real* bx = box + 6 * b;
    for (int i = 0; i < N; i++) {
      size_t row = ((size_t)b * N + i) * nr;
      size_t row3 = ((size_t)b * N + i) * 3 * nr;
      int* im = intmap2b + ((size_t)b * N + i) * (nr + 1);
      for (int k = 0; k < nr + 1; k++) im[k] = 0;
      for (int k = 0; k < nr; k++) {
        raddescr[row + k] = 0; des3bsupp[row + k] = 0;
        for (int c = 0; c < 3; c++) { der2b[row3 + c * nr + k] = 0; der3bsupp[row3 + c * nr + k] = 0; }
      }
      int hm = howmany[b * N + i];
      im[0] = hm;
      int ntrip = 0;
      for (int k = 0; k < nr && k < hm; k++) {
        int j = with[row + k];
        real od[3], d[3];
        const real* si = frac + ((size_t)b * Npos + i) * 3;
        const real* sj = frac + ((size_t)b * Npos + j) * 3;
        for (int c = 0; c < 3; c++) {
          od[c] = si[c] - sj[c];
          if (!skip_pbc) od[c] -= M<real>::rint(od[c]);
        }
        d[0] = bx[0] * od[0] + bx[1] * od[1] + bx[2] * od[2];
        d[1] = bx[3] * od[1] + bx[4] * od[2];
        d[2] = bx[5] * od[2];
        real r = M<real>::sqrt(sqr(d[0]) + sqr(d[1]) + sqr(d[2]));
        if (r < Ra) {
          ntrip += 1;
          des3bsupp[row + k] = 0.5 * (M<real>::cos(PI * r / Ra) + 1);
          for (int c = 0; c < 3; c++)
            der3bsupp[row3 + c * nr + k] = -0.5 * M<real>::sin(PI * r / Ra) * PI / Ra * d[c] / r;
        }
        if (r < rs) {
          raddescr[row + k] = cA / M<real>::pow(r, pa) + cB / M<real>::pow(r, pb) + cC;
          for (int c = 0; c < 3; c++) {
            // pow(real, real + 1.): the double literal makes the call ISO-ambiguous
            // for real=float; gcc (and nvcc's front end in gcc mode) pick pow(double,double).
            der2b[row3 + c * nr + k] =
                (-pa * cA / std::pow((double)r, pa + 1.) - pb * cB / std::pow((double)r, pb + 1.)) * d[c] / r;
          }
        } else {
          raddescr[row + k] = 0.5 * (M<real>::cos(PI * r / Rc) + 1);
          for (int c = 0; c < 3; c++)
            der2b[row3 + c * nr + k] = -0.5 * M<real>::sin(PI * r / Rc) * PI / Rc * d[c] / r;
        }
        im[1 + k] = j;
      }
      numtriplet[b * N + i] = ntrip;
    }
  }
}

// triplet index nn -> (j,k), row-major upper triangle over the first m sorted
// neighbours -- reforce.cu.cc:137-146
inline void decode_triplet(int nn, int m, int* jo, int* ko) {
  int j = 0, prev_row = 0, next_row = m - j - 1;
  while (nn >= next_row) { j += 1; prev_row = next_row; next_row += m - j - 1; }
  *jo = j; *ko = nn - prev_row + 1 + j;
}

// ---------------------------------------------------------------------------
// DescriptorsAngular_kernel -- STAF/src/descriptor_builder/reforce.cu.cc:112-236
// ---------------------------------------------------------------------------
template <typename real>
void descriptors_angular(int nf, int N, int Npos, int nr, int na, const real* frac, const real* box, const int* with,
                         real Ra, const int* numtriplet, int skip_pbc, real* angdescr, int* intmap3b, real* der3b) {
  const real PI = PIc<real>();
  for (int b = 0; b < nf; b++) {
    const real* bx = box + 6 * b;
    for (int i = 0; i < N; i++) {
      size_t arow = ((size_t)b * N + i) * na;
      for (int nn = 0; nn < na; nn++) {
        angdescr[arow + nn] = 0;
        intmap3b[(arow + nn) * 2] = 0; intmap3b[(arow + nn) * 2 + 1] = 0;
        for (int c = 0; c < 3; c++) { der3b[((arow * 3) + (size_t)c * na + nn) * 2] = 0; der3b[((arow * 3) + (size_t)c * na + nn) * 2 + 1] = 0; }
      }
      int m = numtriplet[b * N + i];
      int ntr = m * (m - 1) / 2;
      const int* w = with + ((size_t)b * N + i) * nr;
      const real* si = frac + ((size_t)b * Npos + i) * 3;
      for (int nn = 0; nn < na && nn < ntr; nn++) {
        int j, k;
        decode_triplet(nn, m, &j, &k);
        int jw = w[j], kw = w[k];
        intmap3b[(arow + nn) * 2] = jw;
        intmap3b[(arow + nn) * 2 + 1] = kw;
        real dj[3], dk[3], od[3];
        const real* sj = frac + ((size_t)b * Npos + jw) * 3;
        const real* sk = frac + ((size_t)b * Npos + kw) * 3;
        for (int c = 0; c < 3; c++) { od[c] = si[c] - sj[c]; if (!skip_pbc) od[c] -= M<real>::rint(od[c]); }
        dj[0] = bx[0] * od[0] + bx[1] * od[1] + bx[2] * od[2]; dj[1] = bx[3] * od[1] + bx[4] * od[2]; dj[2] = bx[5] * od[2];
        real rj = M<real>::sqrt(sqr(dj[0]) + sqr(dj[1]) + sqr(dj[2]));
        for (int c = 0; c < 3; c++) { od[c] = si[c] - sk[c]; if (!skip_pbc) od[c] -= M<real>::rint(od[c]); }
        dk[0] = bx[0] * od[0] + bx[1] * od[1] + bx[2] * od[2]; dk[1] = bx[3] * od[1] + bx[4] * od[2]; dk[2] = bx[5] * od[2];
        real rk = M<real>::sqrt(sqr(dk[0]) + sqr(dk[1]) + sqr(dk[2]));
        real dot = dj[0] * dk[0] + dj[1] * dk[1] + dj[2] * dk[2];
        real angle = dot / (rj * rk);
        real cj = real(0.5) * (real(1.) + M<real>::cos(PI * rj / Ra));
        real ck = real(0.5) * (real(1.) + M<real>::cos(PI * rk / Ra));
        real tijk = 0.5 * (angle + 1) * cj * ck;
        for (int c = 0; c < 3; c++) {
          real dcj = -real(0.5) * M<real>::sin(PI * rj / Ra) * PI / Ra / rj * dj[c];
          real dck = -real(0.5) * M<real>::sin(PI * rk / Ra) * PI / Ra / rk * dk[c];
          real daj = 0.5 * (sqr(rj) * dk[c] - dj[c] * dot) / (rj * rj * rj * rk);
          real dak = 0.5 * (sqr(rk) * dj[c] - dk[c] * dot) / (rk * rk * rk * rj);
          size_t o = ((arow * 3) + (size_t)c * na + nn) * 2;
          der3b[o] = daj * cj * ck + 0.5 * (angle + 1) * dcj * ck;
          der3b[o + 1] = dak * cj * ck + 0.5 * (angle + 1) * cj * dck;
        }
        angdescr[arow + nn] = tijk;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// radialAFs_kernel (ComputeSortProj) -- STAF/src/fingerprint/rad/reforce.cu.cc:12-48
// ---------------------------------------------------------------------------
template <typename real>
void radial_afs(int nf, int Nl, int nr, int Ar, const real* raddescr, const int* intmap2b, const real* alpha2b,
                const real* emb2b, const int* type_map, real* af2) {
  for (size_t q = 0; q < (size_t)nf * Nl * Ar; q++) af2[q] = 0;
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    const int* im = intmap2b + ((size_t)b * Nl + p) * (nr + 1);
    int cnt = im[0];
    for (int j = 0; j < nr && j < cnt; j++) {
      real d = raddescr[((size_t)b * Nl + p) * nr + j];
      int ct = type_map[im[1 + j]];
      for (int a = 0; a < Ar; a++) {
        real w = M<real>::exp(alpha2b[Ar * ct + a] * d) * emb2b[Ar * ct + a];
        af2[((size_t)b * Nl + p) * Ar + a] += d * w;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// angularAFs_kernel (ComputeSortProj3body) -- STAF/src/fingerprint/ang/reforce.cu.cc:13-71
// ds = des3bsupp (the op's "radial_descriptor" input), T = angdescr.
// ---------------------------------------------------------------------------
template <typename real>
void angular_afs(int nf, int Nl, int nr, int na, int Aa, const real* ds, const real* T, const int* intmap3b,
                 const real* alpha3b, const real* emb3b, const int* type_map, const int* numtriplet, real* af3) {
  for (size_t q = 0; q < (size_t)nf * Nl * Aa; q++) af3[q] = 0;
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    int m = numtriplet[b * Nl + p];
    int ntr = (m * (m - 1)) / 2;
    size_t act = ((size_t)b * Nl + p) * nr, acta = ((size_t)b * Nl + p) * na;
    for (int nn = 0; nn < na && nn < ntr; nn++) {
      int j, k;
      decode_triplet(nn, m, &j, &k);
      int sum = type_map[intmap3b[(acta + nn) * 2]] + type_map[intmap3b[(acta + nn) * 2 + 1]];
      real t = T[acta + nn];
      for (int a = 0; a < Aa; a++) {
        const real* al = alpha3b + ((size_t)sum * Aa + a) * 3;
        real c = emb3b[sum * Aa + a];
        real w = M<real>::exp(al[0] * ds[act + j] + al[1] * ds[act + k]);
        w += M<real>::exp(al[1] * ds[act + j] + al[0] * ds[act + k]);
        w *= M<real>::exp(al[2] * t);
        af3[((size_t)b * Nl + p) * Aa + a] += t * w * c / real(2.);
      }
    }
  }
}

inline int species_shift(const int* tipos, int actual_type) {
  int s = 0;
  for (int y = 0; y < actual_type; y++) s += tipos[y];
  return s;
}

// MIC Cartesian separation r_i - r_j from Cartesian positions --
// STAF/include/staf_force_pbc.cuh:16-49
template <typename real>
inline void mic_cart_from_cart(const real* pi, const real* pj, const real* bx, int skip_pbc, real* d) {
  real inv[6];
  inv[0] = real(1.) / bx[0];
  inv[1] = -bx[1] / (bx[0] * bx[3]);
  inv[2] = (bx[1] * bx[4]) / (bx[0] * bx[3] * bx[5]) - bx[2] / (bx[0] * bx[5]);
  inv[3] = real(1.) / bx[3];
  inv[4] = -bx[4] / (bx[3] * bx[5]);
  inv[5] = real(1.) / bx[5];
  real fi[3] = {inv[0] * pi[0] + inv[1] * pi[1] + inv[2] * pi[2], inv[3] * pi[1] + inv[4] * pi[2], inv[5] * pi[2]};
  real fj[3] = {inv[0] * pj[0] + inv[1] * pj[1] + inv[2] * pj[2], inv[3] * pj[1] + inv[4] * pj[2], inv[5] * pj[2]};
  real r[3] = {fi[0] - fj[0], fi[1] - fj[1], fi[2] - fj[2]};
  if (!skip_pbc) for (int c = 0; c < 3; c++) r[c] -= M<real>::rint(r[c]);
  d[0] = bx[0] * r[0] + bx[1] * r[1] + bx[2] * r[2];
  d[1] = bx[3] * r[1] + bx[4] * r[2];
  d[2] = bx[5] * r[2];
}

// ---------------------------------------------------------------------------
// computeforce_doublets[_virial]_kernel (ComputeForceRadial[Virial]) --
// STAF/src/force/rad/reforce.cu.cc:45-136, 174-287.  virial/pos/box may be
// null (plain op).  force [nf,3N] and virial [nf,9] are zeroed here as the op
// shells do (force/rad/reforce.cc:118, 218-221).
// ---------------------------------------------------------------------------
template <typename real>
void force_doublets(int nf, int N, int nr, int Ar, const real* netderiv, const real* des_r, const real* der2b,
                    const int* intmap2b, const real* alpha2b, const real* emb2b, const int* type_map,
                    const int* tipos, int actual_type, real* force, real* virial, const real* pos, const real* box) {
  int Nl = tipos[actual_type];
  int shift = species_shift(tipos, actual_type);
  for (size_t q = 0; q < (size_t)nf * 3 * N; q++) force[q] = 0;
  if (virial) for (int q = 0; q < nf * 9; q++) virial[q] = 0;
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    int ap = p + shift;
    const int* im = intmap2b + ((size_t)b * Nl + p) * (nr + 1);
    int cnt = im[0];
    real self[3] = {0, 0, 0};
    real vloc[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int j = 0; j < nr && j < cnt; j++) {
      int nj = im[1 + j];
      real d = des_r[((size_t)b * Nl + p) * nr + j];
      int ct = type_map[nj];
      real id[3];
      for (int c = 0; c < 3; c++) id[c] = der2b[((size_t)b * Nl + p) * 3 * nr + c * nr + j];
      real dij[3] = {0, 0, 0};
      if (virial) mic_cart_from_cart(pos + ((size_t)b * N + ap) * 3, pos + ((size_t)b * N + nj) * 3, box + 6 * b, 0, dij);
      real other[3] = {0, 0, 0};
      real fslot[3] = {0, 0, 0};
      for (int a = 0; a < Ar; a++) {
        real al = alpha2b[Ar * ct + a];
        real ch = emb2b[Ar * ct + a];
        real sds = ch * M<real>::exp(al * d);
        sds *= (real(1.) + al * d);
        real pg = netderiv[((size_t)b * Nl + p) * Ar + a];
        if (!virial) {
          for (int c = 0; c < 3; c++) {
            real tmp = real(0.5) * sds * id[c];
            fslot[c] -= pg * tmp;
            other[c] += pg * tmp;
          }
        } else {
          real g[3];
          for (int c = 0; c < 3; c++) { g[c] = pg * real(0.5) * sds * id[c]; fslot[c] -= g[c]; other[c] += g[c]; }
          for (int c = 0; c < 3; c++) for (int e = 0; e < 3; e++) vloc[c * 3 + e] -= g[c] * dij[e];
        }
      }
      for (int c = 0; c < 3; c++) { force[((size_t)b * N + nj) * 3 + c] += other[c]; self[c] += fslot[c]; }
    }
    for (int c = 0; c < 3; c++) force[((size_t)b * N + ap) * 3 + c] += self[c];
    if (virial) for (int c = 0; c < 9; c++) virial[b * 9 + c] += vloc[c];
  }
}

// per-(triplet, channel) force coefficients shared by the 3-body force op
// and its gradient -- force/ang/reforce.cu.cc:140-160
template <typename real>
struct TripCoef { real delta, Bpj, Bpk; };
template <typename real>
inline TripCoef<real> trip_coef(real a1, real a2, real be, real T, real Dj, real Dk) {
  real expbeta = M<real>::exp(be * T);
  real sim1 = M<real>::exp(a2 * Dj + a1 * Dk);
  real sim2 = M<real>::exp(a1 * Dj + a2 * Dk);
  TripCoef<real> o;
  o.delta = expbeta * (1. + be * T) * (sim1 + sim2) * real(0.5);
  real suppj = (a1 * sim2 + a2 * sim1) * expbeta * real(0.5);
  real suppk = (a1 * sim1 + a2 * sim2) * expbeta * real(0.5);
  o.Bpj = suppj * T;
  o.Bpk = suppk * T;
  return o;
}

// ---------------------------------------------------------------------------
// computeforce_tripl[_virial]_kernel (ComputeForceTripl[Virial]) --
// STAF/src/force/ang/reforce.cu.cc:48-232, 269-457
// desr = des3bsupp, desa = angdescr, der_r = der3bsupp, der_a = der3b.
// ---------------------------------------------------------------------------
template <typename real>
void force_tripl(int nf, int N, int nr, int na, int Aa, const real* netderiv, const real* desr, const real* desa,
                 const real* der_r, const real* der_a, const int* intmap3b, const real* alpha3b, const real* emb3b,
                 const int* type_map, const int* tipos, int actual_type, const int* numtriplet, real* force,
                 real* virial, const real* pos, const real* box) {
  int Nl = tipos[actual_type];
  int shift = species_shift(tipos, actual_type);
  for (size_t q = 0; q < (size_t)nf * 3 * N; q++) force[q] = 0;
  if (virial) for (int q = 0; q < nf * 9; q++) virial[q] = 0;
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    int ap = p + shift;
    int m = numtriplet[b * Nl + p];
    int ntr = (m * (m - 1)) / 2;
    size_t act = ((size_t)b * Nl + p) * nr, acta = ((size_t)b * Nl + p) * na, actg = ((size_t)b * Nl + p) * Aa;
    real self[3] = {0, 0, 0};
    real vloc[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int nn = 0; nn < na && nn < ntr; nn++) {
      int j, k;
      decode_triplet(nn, m, &j, &k);
      int nj = intmap3b[(acta + nn) * 2], nk = intmap3b[(acta + nn) * 2 + 1];
      int sum = type_map[nj] + type_map[nk];
      real T = desa[acta + nn], Dj = desr[act + j], Dk = desr[act + k];
      real dij[3] = {0, 0, 0}, dik[3] = {0, 0, 0};
      if (virial) {
        mic_cart_from_cart(pos + ((size_t)b * N + ap) * 3, pos + ((size_t)b * N + nj) * 3, box + 6 * b, 0, dij);
        mic_cart_from_cart(pos + ((size_t)b * N + ap) * 3, pos + ((size_t)b * N + nk) * 3, box + 6 * b, 0, dik);
      }
      real oj[3] = {0, 0, 0}, ok[3] = {0, 0, 0}, fs[3] = {0, 0, 0};
      for (int a = 0; a < Aa; a++) {
        const real* al = alpha3b + ((size_t)sum * Aa + a) * 3;
        real net = real(0.5) * netderiv[actg + a] * emb3b[sum * Aa + a];
        TripCoef<real> tc = trip_coef<real>(al[0], al[1], al[2], T, Dj, Dk);
        for (int c = 0; c < 3; c++) {
          size_t o = ((acta * 3) + (size_t)c * na + nn) * 2;
          real fij = net * (tc.delta * der_a[o] + tc.Bpj * der_r[act * 3 + c * nr + j]);
          real fik = net * (tc.delta * der_a[o + 1] + tc.Bpk * der_r[act * 3 + c * nr + k]);
          fs[c] -= (fij + fik);
          oj[c] += fij;
          ok[c] += fik;
          if (virial) for (int e = 0; e < 3; e++) vloc[c * 3 + e] -= fij * dij[e] + fik * dik[e];
        }
      }
      for (int c = 0; c < 3; c++) {
        force[((size_t)b * N + nj) * 3 + c] += oj[c];
        force[((size_t)b * N + nk) * 3 + c] += ok[c];
        self[c] += fs[c];
      }
    }
    for (int c = 0; c < 3; c++) force[((size_t)b * N + ap) * 3 + c] += self[c];
    if (virial) for (int c = 0; c < 9; c++) virial[b * 9 + c] += vloc[c];
  }
}

// ---------------------------------------------------------------------------
// alphagrad_dist_kernel (ComputeTwoBodyParGrad) -- STAF/src/grad_finger/rad/reforce.cu.cc:12-47
// ---------------------------------------------------------------------------
template <typename real>
void alphagrad_dist(int nf, int Nl, int nr, int Ar, int nt, const real* prevgrad, const real* raddescr,
                    const int* intmap2b, const real* alpha2b, const real* emb2b, const int* type_map,
                    real* g_alpha2b, real* g_emb2b) {
  for (int q = 0; q < nt * Ar; q++) { g_alpha2b[q] = 0; g_emb2b[q] = 0; }
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    const int* im = intmap2b + ((size_t)b * Nl + p) * (nr + 1);
    int cnt = im[0];
    for (int j = 0; j < nr && j < cnt; j++) {
      real d = raddescr[((size_t)b * Nl + p) * nr + j];
      int ct = type_map[im[1 + j]];
      for (int a = 0; a < Ar; a++) {
        real pg = prevgrad[((size_t)b * Nl + p) * Ar + a];
        real tw = emb2b[ct * Ar + a];
        real acc = d * d;
        acc *= M<real>::exp(alpha2b[ct * Ar + a] * d) * tw * pg;
        g_alpha2b[ct * Ar + a] += acc;
        acc = d;
        acc *= M<real>::exp(alpha2b[ct * Ar + a] * d) * pg;
        g_emb2b[ct * Ar + a] += acc;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// alphagrad_ang_kernel (ComputeSortProj3bodyGrad) -- STAF/src/grad_finger/ang/reforce.cu.cc:13-111
// g_emb3b is allocated, zeroed and never written by the reference.
// ---------------------------------------------------------------------------
template <typename real>
void alphagrad_ang(int nf, int Nl, int nr, int na, int Aa, int ntc, const real* prevgrad, const real* T,
                   const real* ds, const int* intmap3b, const real* alpha3b, const real* emb3b, const int* type_map,
                   const int* numtriplet, real* g_alpha3b, real* g_emb3b) {
  for (int q = 0; q < ntc * Aa * 3; q++) g_alpha3b[q] = 0;
  for (int q = 0; q < ntc * Aa; q++) g_emb3b[q] = 0;
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    int m = numtriplet[b * Nl + p];
    int ntr = (m * (m - 1)) / 2;
    size_t act = ((size_t)b * Nl + p) * nr, acta = ((size_t)b * Nl + p) * na;
    for (int nn = 0; nn < na && nn < ntr; nn++) {
      int j, k;
      decode_triplet(nn, m, &j, &k);
      int sum = type_map[intmap3b[(acta + nn) * 2]] + type_map[intmap3b[(acta + nn) * 2 + 1]];
      if (sum >= ntc) continue;
      real dj = ds[act + j], dy = ds[act + k], Tjy = T[acta + nn];
      for (int a = 0; a < Aa; a++) {
        const real* al = alpha3b + ((size_t)sum * Aa + a) * 3;
        real c = emb3b[sum * Aa + a];
        real pg = prevgrad[((size_t)b * Nl + p) * Aa + a];
        real e1 = M<real>::exp(al[0] * dj + al[1] * dy);
        real e2 = M<real>::exp(al[0] * dy + al[1] * dj);
        real bt = M<real>::exp(al[2] * Tjy);
        real* g = g_alpha3b + ((size_t)sum * Aa + a) * 3;
        g[0] += pg * c * (e1 * dj + e2 * dy) * bt * Tjy / real(2.);
        g[1] += pg * c * (e1 * dy + e2 * dj) * bt * Tjy / real(2.);
        g[2] += pg * c * (e1 + e2) * bt * Tjy * Tjy / real(2.);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// back_prop_grad_force2b[_virial]_kernel (ComputeForceRadial[Virial]Grad) --
// STAF/src/grad_force/rad/reforce.cu.cc:46-123, 165-234
// prevgrad = dL/dF [nf,3N]; pg_vir = dL/dW [nf,9] or null.
// ---------------------------------------------------------------------------
template <typename real>
void gradforce_2b(int nf, int N, int nr, int Ar, int nt, const real* prevgrad, const real* netderiv, const real* ds,
                  const real* der2b, const int* intmap2b, const real* alpha2b, const real* emb2b, const int* type_map,
                  const int* tipos, int actual_type, real* g_net, real* g_alpha2b, real* g_emb2b, const real* pg_vir,
                  const real* pos, const real* box) {
  int Nl = tipos[actual_type];
  int shift = species_shift(tipos, actual_type);
  for (size_t q = 0; q < (size_t)nf * Nl * Ar; q++) g_net[q] = 0;
  for (int q = 0; q < nt * Ar; q++) { g_alpha2b[q] = 0; g_emb2b[q] = 0; }
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    int ap = p + shift;
    const int* im = intmap2b + ((size_t)b * Nl + p) * (nr + 1);
    int cnt = im[0];
    for (int j = 0; j < nr && j < cnt; j++) {
      int nj = im[1 + j];
      int ct = type_map[nj];
      real d = ds[((size_t)b * Nl + p) * nr + j];
      real rij[3] = {0, 0, 0};
      if (pg_vir) mic_cart_from_cart(pos + ((size_t)b * N + ap) * 3, pos + ((size_t)b * N + nj) * 3, box + 6 * b, 0, rij);
      for (int a = 0; a < Ar; a++) {
        real a1 = 0, a2 = 0, a3 = 0;
        for (int c = 0; c < 3; c++) {
          real pe = prevgrad[((size_t)b * N + ap) * 3 + c];
          real pn = prevgrad[((size_t)b * N + nj) * 3 + c];
          real common = real(0.5) * der2b[((size_t)b * Nl + p) * 3 * nr + c * nr + j];
          real al = alpha2b[Ar * ct + a];
          real ch = emb2b[Ar * ct + a];
          real s1 = M<real>::exp(al * d);
          real sds = s1 * (real(1.) + al * d);
          real buff_alpha = ch * s1 * d * (real(2.) + al * d);
          real NG = netderiv[((size_t)b * Nl + p) * Ar + a];
          if (!pg_vir) {
            a1 -= pe * common * ch * sds;
            a1 += pn * common * ch * sds;
            a2 -= pe * NG * buff_alpha * common;
            a2 += pn * NG * buff_alpha * common;
            a3 -= pe * NG * sds * common;
            a3 += pn * NG * sds * common;
          } else {
            const real* Wg = pg_vir + b * 9;
            real wdot = Wg[c * 3 + 0] * rij[0] + Wg[c * 3 + 1] * rij[1] + Wg[c * 3 + 2] * rij[2];
            real coeff = pn - pe - wdot;
            a1 += coeff * common * ch * sds;
            a2 += coeff * NG * buff_alpha * common;
            a3 += coeff * NG * sds * common;
          }
        }
        g_net[((size_t)b * Nl + p) * Ar + a] += a1;
        g_alpha2b[Ar * ct + a] += a2;
        g_emb2b[Ar * ct + a] += a3;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// gradforce_tripl[_virial]_kernel (ComputeForceTripl[Virial]Grad) --
// STAF/src/grad_force/ang/reforce.cu.cc:47-231, 274-446
// g_emb3b is zeroed and never written by the reference.
// ---------------------------------------------------------------------------
template <typename real>
void gradforce_tripl(int nf, int N, int nr, int na, int Aa, int nt, const real* prevgrad, const real* netderiv,
                     const real* desr, const real* desa, const real* der_r, const real* der_a, const int* intmap3b,
                     const real* alpha3b, const real* emb3b, const int* type_map, const int* tipos, int actual_type,
                     const int* numtriplet, real* g_net, real* g_alpha3b, real* g_emb3b, const real* pg_vir,
                     const real* pos, const real* box) {
  int Nl = tipos[actual_type];
  int shift = species_shift(tipos, actual_type);
  int ntc = nt * (nt + 1) / 2;
  for (size_t q = 0; q < (size_t)nf * Nl * Aa; q++) g_net[q] = 0;
  for (int q = 0; q < ntc * Aa * 3; q++) g_alpha3b[q] = 0;
  for (int q = 0; q < ntc * Aa; q++) g_emb3b[q] = 0;
  for (int b = 0; b < nf; b++) for (int p = 0; p < Nl; p++) {
    int ap = p + shift;
    int m = numtriplet[b * Nl + p];
    int ntr = (m * (m - 1)) / 2;
    size_t act = ((size_t)b * Nl + p) * nr, acta = ((size_t)b * Nl + p) * na, actg = ((size_t)b * Nl + p) * Aa;
    for (int nn = 0; nn < na && nn < ntr; nn++) {
      int j, k;
      decode_triplet(nn, m, &j, &k);
      int nj = intmap3b[(acta + nn) * 2], nk = intmap3b[(acta + nn) * 2 + 1];
      int sum = type_map[nj] + type_map[nk];
      if (sum >= ntc) continue;
      real T = desa[acta + nn], Dj = desr[act + j], Dk = desr[act + k];
      real rij[3] = {0, 0, 0}, rik[3] = {0, 0, 0};
      if (pg_vir) {
        mic_cart_from_cart(pos + ((size_t)b * N + ap) * 3, pos + ((size_t)b * N + nj) * 3, box + 6 * b, 0, rij);
        mic_cart_from_cart(pos + ((size_t)b * N + ap) * 3, pos + ((size_t)b * N + nk) * 3, box + 6 * b, 0, rik);
      }
      for (int a = 0; a < Aa; a++) {
        real acc1 = 0, acc3 = 0, acc4 = 0, acc5 = 0;
        real NG = netderiv[actg + a];
        const real* al = alpha3b + ((size_t)sum * Aa + a) * 3;
        real a1 = al[0], a2 = al[1], be = al[2];
        real ch = emb3b[sum * Aa + a];
        real expbeta = M<real>::exp(be * T);
        real sim1 = M<real>::exp(a2 * Dj + a1 * Dk);
        real sim2 = M<real>::exp(a1 * Dj + a2 * Dk);
        real sum_sim = sim1 + sim2;
        real delta = expbeta * (real(1.0) + be * T) * sum_sim * real(0.5);
        real suppj = (a1 * sim2 + a2 * sim1) * expbeta;
        real suppk = (a1 * sim1 + a2 * sim2) * expbeta;
        real Bpj = suppj * T * real(0.5);
        real Bpk = suppk * T * real(0.5);
        for (int c = 0; c < 3; c++) {
          size_t o = ((acta * 3) + (size_t)c * na + nn) * 2;
          real ix = der_a[o], iy = der_a[o + 1];
          real irj = der_r[act * 3 + c * nr + j], irk = der_r[act * 3 + c * nr + k];
          real pl = prevgrad[((size_t)b * N + ap) * 3 + c];
          real pj = prevgrad[((size_t)b * N + nj) * 3 + c];
          real pk = prevgrad[((size_t)b * N + nk) * 3 + c];
          real gxij = ch * delta * ix + ch * Bpj * irj;
          real gxik = ch * delta * iy + ch * Bpk * irk;
          real b_a1_ang = expbeta * (real(1.) + be * T) * (sim1 * Dk + sim2 * Dj) * real(0.5);
          real b_a2_ang = expbeta * (real(1.) + be * T) * (sim1 * Dj + sim2 * Dk) * real(0.5);
          real b_be_ang = expbeta * T * (real(2.) + be * T) * sum_sim * real(0.5);
          real b_be_rj = suppj * T * T * real(0.5);
          real b_be_rk = suppk * T * T * real(0.5);
          real b_a1_rj = (sim2 + a1 * sim2 * Dj + a2 * sim1 * Dk) * expbeta * real(0.5) * T;
          real b_a2_rj = (sim1 + a2 * sim1 * Dj + a1 * sim2 * Dk) * expbeta * real(0.5) * T;
          real b_a1_rk = (sim1 + a1 * sim1 * Dk + a2 * sim2 * Dj) * expbeta * real(0.5) * T;
          real b_a2_rk = (sim2 + a2 * sim2 * Dk + a1 * sim1 * Dj) * expbeta * real(0.5) * T;
          real g1ij = ch * b_a1_ang * ix + ch * b_a1_rj * irj;
          real g1ik = ch * b_a1_ang * iy + ch * b_a1_rk * irk;
          real g2ij = ch * b_a2_ang * ix + ch * b_a2_rj * irj;
          real g2ik = ch * b_a2_ang * iy + ch * b_a2_rk * irk;
          real gbij = ch * b_be_ang * ix + ch * b_be_rj * irj;
          real gbik = ch * b_be_ang * iy + ch * b_be_rk * irk;
          if (!pg_vir) {
            acc1 += -pl * real(0.5) * (gxij + gxik);
            acc1 += pj * real(0.5) * gxij + pk * real(0.5) * gxik;
            acc3 += -pl * real(0.5) * NG * (g1ij + g1ik) + pj * real(0.5) * NG * g1ij + pk * real(0.5) * NG * g1ik;
            acc4 += -pl * real(0.5) * NG * (g2ij + g2ik) + pj * real(0.5) * NG * g2ij + pk * real(0.5) * NG * g2ik;
            acc5 += -pl * real(0.5) * NG * (gbij + gbik) + pj * real(0.5) * NG * gbij + pk * real(0.5) * NG * gbik;
          } else {
            const real* Wg = pg_vir + b * 9;
            real wij = Wg[c * 3 + 0] * rij[0] + Wg[c * 3 + 1] * rij[1] + Wg[c * 3 + 2] * rij[2];
            real wik = Wg[c * 3 + 0] * rik[0] + Wg[c * 3 + 1] * rik[1] + Wg[c * 3 + 2] * rik[2];
            real cj = pj - pl - wij, ck = pk - pl - wik;
            acc1 += cj * real(0.5) * gxij + ck * real(0.5) * gxik;
            acc3 += cj * real(0.5) * NG * g1ij + ck * real(0.5) * NG * g1ik;
            acc4 += cj * real(0.5) * NG * g2ij + ck * real(0.5) * NG * g2ik;
            acc5 += cj * real(0.5) * NG * gbij + ck * real(0.5) * NG * gbik;
          }
        }
        g_net[actg + a] += acc1;
        real* g = g_alpha3b + ((size_t)sum * Aa + a) * 3;
        g[0] += acc3; g[1] += acc4; g[2] += acc5;
      }
    }
  }
}

// whole descriptor op -- ComputeDescriptorsLightOp::Compute, reforce.cc:262-444
template <typename real>
int compute_descriptors_light(int nf, int N, int nr, int na, const real* pos, const real* box, real Rc, real Ra,
                              real Rs, int fma_mode, real* raddescr, real* angdescr, real* des3bsupp, int* intmap2b,
                              int* intmap3b, real* der2b, real* der3b, real* der3bsupp, int* numtriplet,
                              int* with_out, int* howmany_out) {
  std::vector<real> frac((size_t)nf * N * 3), d2((size_t)nf * N * nr);
  std::vector<int> with((size_t)nf * N * nr), hm((size_t)nf * N);
  real c5[5];
  fill_repulsion<real>(Rc, Rs, c5);
  cart_to_frac(nf, N, pos, box, frac.data());
  int mx = neighbor_list(nf, N, frac.data(), box, Rc, nr, fma_mode, with.data(), d2.data(), hm.data());
  if (with_out) memcpy(with_out, with.data(), with.size() * sizeof(int));
  if (howmany_out) memcpy(howmany_out, hm.data(), hm.size() * sizeof(int));
  if (mx > nr) return mx;  // reference aborts here (reforce.cc:329-337)
  descriptors_radial(nf, N, N, nr, frac.data(), box, hm.data(), with.data(), Rc, Ra, Rs, c5[0], c5[1], c5[2], c5[3],
                     c5[4], 0, raddescr, intmap2b, der2b, des3bsupp, der3bsupp, numtriplet);
  descriptors_angular(nf, N, N, nr, na, frac.data(), box, with.data(), Ra, numtriplet, 0, angdescr, intmap3b, der3b);
  return mx;
}

}  // namespace

#define ORACLE_INSTANTIATE(real, SFX)                                                                                  \
  extern "C" {                                                                                                         \
  void oracle_fill_repulsion_##SFX(real rc, real rs, real* out5) { fill_repulsion<real>(rc, rs, out5); }               \
  void oracle_cutoff_curve_##SFX(real rc, real rs, const real* c5, int n, real* xs, real* ys) {                        \
    cutoff_curve<real>(rc, rs, c5, n, xs, ys);                                                                         \
  }                                                                                                                    \
  void oracle_inverse_box_##SFX(const real* b, real* inv) { inverse_box<real>(b, inv); }                               \
  void oracle_cart_to_frac_##SFX(int nf, int N, const real* pos, const real* box, real* frac) {                        \
    cart_to_frac<real>(nf, N, pos, box, frac);                                                                         \
  }                                                                                                                    \
  void oracle_cell_dims_##SFX(const real* box, real cutoff, int N, int* nxyz) { cell_dims<real>(box, cutoff, N, nxyz); } \
  int oracle_neighbor_list_##SFX(int nf, int N, const real* frac, const real* box, real cutoff, int nr, int fma_mode,  \
                                 int* with, real* d2, int* hm) {                                                       \
    return neighbor_list<real>(nf, N, frac, box, cutoff, nr, fma_mode, with, d2, hm);                                  \
  }                                                                                                                    \
  int oracle_neighbor_list_cells_##SFX(int nf, int N, const real* frac, const real* box, real cutoff, int nr,          \
                                       int fma_mode, int* with, real* d2, int* hm) {                                   \
    return neighbor_list_cells<real>(nf, N, frac, box, cutoff, nr, fma_mode, with, d2, hm);                            \
  }                                                                                                                    \
  void oracle_descriptors_radial_##SFX(int nf, int N, int Npos, int nr, const real* frac, const real* box,             \
                                       const int* hm, const int* with, real Rc, real Ra, real rs, real cA, real cB,    \
                                       real cC, real pa, real pb, int skip_pbc, real* raddescr, int* intmap2b,         \
                                       real* der2b, real* des3bsupp, real* der3bsupp, int* numtriplet) {               \
    descriptors_radial<real>(nf, N, Npos, nr, frac, box, hm, with, Rc, Ra, rs, cA, cB, cC, pa, pb, skip_pbc, raddescr, \
                             intmap2b, der2b, des3bsupp, der3bsupp, numtriplet);                                       \
  }                                                                                                                    \
  void oracle_descriptors_angular_##SFX(int nf, int N, int Npos, int nr, int na, const real* frac, const real* box,    \
                                        const int* with, real Ra, const int* numtriplet, int skip_pbc, real* angdescr, \
                                        int* intmap3b, real* der3b) {                                                  \
    descriptors_angular<real>(nf, N, Npos, nr, na, frac, box, with, Ra, numtriplet, skip_pbc, angdescr, intmap3b,      \
                              der3b);                                                                                  \
  }                                                                                                                    \
  int oracle_compute_descriptors_light_##SFX(int nf, int N, int nr, int na, const real* pos, const real* box, real Rc, \
                                             real Ra, real Rs, int fma_mode, real* raddescr, real* angdescr,           \
                                             real* des3bsupp, int* intmap2b, int* intmap3b, real* der2b, real* der3b,  \
                                             real* der3bsupp, int* numtriplet, int* with_out, int* howmany_out) {      \
    return compute_descriptors_light<real>(nf, N, nr, na, pos, box, Rc, Ra, Rs, fma_mode, raddescr, angdescr,          \
                                           des3bsupp, intmap2b, intmap3b, der2b, der3b, der3bsupp, numtriplet,         \
                                           with_out, howmany_out);                                                     \
  }                                                                                                                    \
  void oracle_radial_afs_##SFX(int nf, int Nl, int nr, int Ar, const real* raddescr, const int* intmap2b,              \
                               const real* alpha2b, const real* emb2b, const int* type_map, real* af2) {               \
    radial_afs<real>(nf, Nl, nr, Ar, raddescr, intmap2b, alpha2b, emb2b, type_map, af2);                               \
  }                                                                                                                    \
  void oracle_angular_afs_##SFX(int nf, int Nl, int nr, int na, int Aa, const real* ds, const real* T,                 \
                                const int* intmap3b, const real* alpha3b, const real* emb3b, const int* type_map,      \
                                const int* numtriplet, real* af3) {                                                    \
    angular_afs<real>(nf, Nl, nr, na, Aa, ds, T, intmap3b, alpha3b, emb3b, type_map, numtriplet, af3);                 \
  }                                                                                                                    \
  void oracle_force_doublets_##SFX(int nf, int N, int nr, int Ar, const real* netderiv, const real* des_r,             \
                                   const real* der2b, const int* intmap2b, const real* alpha2b, const real* emb2b,     \
                                   const int* type_map, const int* tipos, int actual_type, real* force, real* virial,  \
                                   const real* pos, const real* box) {                                                 \
    force_doublets<real>(nf, N, nr, Ar, netderiv, des_r, der2b, intmap2b, alpha2b, emb2b, type_map, tipos,             \
                         actual_type, force, virial, pos, box);                                                        \
  }                                                                                                                    \
  void oracle_force_tripl_##SFX(int nf, int N, int nr, int na, int Aa, const real* netderiv, const real* desr,         \
                                const real* desa, const real* der_r, const real* der_a, const int* intmap3b,           \
                                const real* alpha3b, const real* emb3b, const int* type_map, const int* tipos,         \
                                int actual_type, const int* numtriplet, real* force, real* virial, const real* pos,    \
                                const real* box) {                                                                     \
    force_tripl<real>(nf, N, nr, na, Aa, netderiv, desr, desa, der_r, der_a, intmap3b, alpha3b, emb3b, type_map,       \
                      tipos, actual_type, numtriplet, force, virial, pos, box);                                        \
  }                                                                                                                    \
  void oracle_alphagrad_dist_##SFX(int nf, int Nl, int nr, int Ar, int nt, const real* prevgrad,                       \
                                   const real* raddescr, const int* intmap2b, const real* alpha2b, const real* emb2b,  \
                                   const int* type_map, real* g_alpha2b, real* g_emb2b) {                              \
    alphagrad_dist<real>(nf, Nl, nr, Ar, nt, prevgrad, raddescr, intmap2b, alpha2b, emb2b, type_map, g_alpha2b,        \
                         g_emb2b);                                                                                     \
  }                                                                                                                    \
  void oracle_alphagrad_ang_##SFX(int nf, int Nl, int nr, int na, int Aa, int ntc, const real* prevgrad,               \
                                  const real* T, const real* ds, const int* intmap3b, const real* alpha3b,             \
                                  const real* emb3b, const int* type_map, const int* numtriplet, real* g_alpha3b,      \
                                  real* g_emb3b) {                                                                     \
    alphagrad_ang<real>(nf, Nl, nr, na, Aa, ntc, prevgrad, T, ds, intmap3b, alpha3b, emb3b, type_map, numtriplet,      \
                        g_alpha3b, g_emb3b);                                                                           \
  }                                                                                                                    \
  void oracle_gradforce_2b_##SFX(int nf, int N, int nr, int Ar, int nt, const real* prevgrad, const real* netderiv,    \
                                 const real* ds, const real* der2b, const int* intmap2b, const real* alpha2b,          \
                                 const real* emb2b, const int* type_map, const int* tipos, int actual_type,            \
                                 real* g_net, real* g_alpha2b, real* g_emb2b, const real* pg_vir, const real* pos,     \
                                 const real* box) {                                                                    \
    gradforce_2b<real>(nf, N, nr, Ar, nt, prevgrad, netderiv, ds, der2b, intmap2b, alpha2b, emb2b, type_map, tipos,    \
                       actual_type, g_net, g_alpha2b, g_emb2b, pg_vir, pos, box);                                      \
  }                                                                                                                    \
  void oracle_gradforce_tripl_##SFX(int nf, int N, int nr, int na, int Aa, int nt, const real* prevgrad,               \
                                    const real* netderiv, const real* desr, const real* desa, const real* der_r,       \
                                    const real* der_a, const int* intmap3b, const real* alpha3b, const real* emb3b,    \
                                    const int* type_map, const int* tipos, int actual_type, const int* numtriplet,     \
                                    real* g_net, real* g_alpha3b, real* g_emb3b, const real* pg_vir, const real* pos,  \
                                    const real* box) {                                                                 \
    gradforce_tripl<real>(nf, N, nr, na, Aa, nt, prevgrad, netderiv, desr, desa, der_r, der_a, intmap3b, alpha3b,      \
                          emb3b, type_map, tipos, actual_type, numtriplet, g_net, g_alpha3b, g_emb3b, pg_vir, pos,     \
                          box);                                                                                        \
  }                                                                                                                    \
  }

ORACLE_INSTANTIATE(float, f32)
ORACLE_INSTANTIATE(double, f64)
