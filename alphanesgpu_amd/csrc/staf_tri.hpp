// Triplet kernels that reduce over an atom's triplets: 3-body fingerprints
// (MODE 0), their parameter gradient (MODE 1), the gradient of the 3-body
// force op (MODE 2), and both gradients in one pass (MODE 3: a training step
// needs both, and everything but the last few accumulations per item -- set-up,
// tables, staging, the exponential, the pair factors -- is shared).  One
// 256-thread workgroup per centre atom at a time; a launch has as many
// workgroups as the device holds at once (or a whole number of such rounds,
// tri_grid) and a workgroup walks over its centres.  These kernels are bound
// by vector-ALU issue, so the layout below is chosen to keep the instruction
// count per (triplet, channel) item low.
//
// Work decomposition inside a species class (ta,tb) of the centre's triplets
// (see staf_tile.hpp for the class enumeration):
//   * exp(a1*D_s), exp(a2*D_s) are tabulated in LDS once per (slot, channel)
//     of the class, so that exp(a1 Dj + a2 Dk) = E1[j]*E2[k] costs two
//     multiplies instead of an exp: O(m * channels) transcendental calls for
//     the pair factors instead of O(m^2 * channels).  Only exp(beta*T) stays
//     per (triplet, channel).
//   * thread <-> (channel ia = tid & 15, triplet subset sub = tid >> 4): the
//     16 lanes of a subset walk the same triplets and differ in the channel,
//     so every thread accumulates its own channel privately with its
//     parameters in registers, and table reads are contiguous in the channel.
//     The four subsets of a wave are combined with two cross-lane adds and
//     added into per-wave fingerprint accumulators in LDS, which are summed once
//     per atom in a fixed order.  The parameter-gradient sums of a pass go through
//     a small per-wave exchange buffer and are added, waves in ascending order, to
//     the workgroup's single accumulator set by the first 16 threads after the next
//     barrier the kernel needs anyway (bit-reproducible, no barrier of its own; one
//     set instead of one per wave keeps the LDS footprint at four workgroups per CU).
//   * triplets are staged in LDS in blocks (table row offsets, T, and for
//     MODE 2 the contraction U of der3b with dL/dF), so tensors laid out by
//     the storage index nn are read exactly once.
#pragma once
#include <map>
#include <mutex>
#include <type_traits>
#include <utility>

#include "staf_tile.hpp"

namespace staf {

constexpr int TRI_BLOCK = 256;
constexpr int TRI_WAVES = TRI_BLOCK / WAVE;
constexpr int TRI_CAP = 16;    // channels tabulated per pass = lanes of a subset
constexpr int TRI_CAPP = TRI_CAP + 1;   // table row pitch: the entry after a row's channels holds (D, V) of its slot
constexpr int TRI_SUBS = TRI_BLOCK / TRI_CAP;
template <typename real, int MODE, bool FUSED = false>
struct TriCfg {
  // triplets staged per block.  The double-precision pass that gives both gradients stages 256: with 512 its LDS
  // footprint would admit three workgroups per CU instead of four; with 256 it is 40496 bytes, 32 of the 128
  // pieces of 1280 bytes a CU hands out, which is exactly a fourth (192, counted on 40 KB per workgroup, was the
  // earlier choice: 336.7 -> 333.3 us per fp64 training step; 272, not a power of two, is slower again).
  // The fused double-precision fingerprint kernel (the MD entry: thousands of centres per launch, several per
  // workgroup) stages 160: five workgroups per CU instead of four.  The plain double-precision fingerprint kernel
  // stages 448: a CU hands out its 160 KB of LDS in pieces of 1280 bytes, so the 32496 bytes that 512 staged triplets
  // make count as 33280 and four workgroups fit, not the five that the occupancy query of the runtime reports
  // (measured with a kernel that counts its resident workgroups per CU); with 448 it is 31472 bytes and five
  // (6144-atom step 360.6 -> 356.8 us).
  static constexpr int QB = sizeof(real) == 8 ? (MODE == 3 ? 256 : MODE == 2 ? 448 : FUSED ? 160 : MODE == 0 ? 448 : 512) : 512;
  // waves per SIMD the register allocation is held to: without a bound the allocation comes out a few registers
  // above the next occupancy step.  The
  // single-precision pass for both gradients is held to six (80 registers, 56 bytes of spill per lane outside the
  // item loop) where it would take 95 and run four: 146 against 168 us per 8-frame step; seven (with a staging block
  // of 256 so that seven workgroups fit a CU's LDS) is slower again (156 us).
  static constexpr int MIN_WAVES = sizeof(real) == 8 ? (MODE == 0 ? 5 : 4)   // also the fused fingerprint kernel's
                                                     : (MODE == 0 ? 8 : MODE == 1 ? 7 : MODE == 3 ? 6 : 5);
  static constexpr bool FORCE_BRANCH = MODE == 2 || MODE == 3;    // dL/dF comes in: der3b, der3bsupp are read
  static constexpr bool ENERGY_BRANCH = MODE == 1 || MODE == 3;   // dL/dAF3 comes in
};
constexpr int TRI_GRID_MAX = 2048;  // workgroups of the persistent gradient modes (one partial row each)

// Workgroups of a persistent gradient launch over `centres` centres.  Workgroup w takes centres w, w + W, ...: the
// launch lasts about ceil(W / resident) rounds of workgroups times ceil(centres / W) centres each, `resident` being
// the workgroups the device holds at once for this kernel and LDS size.  Within a number of rounds the largest W
// is best, so one candidate per number of rounds; ties go to the larger W (more, shorter workgroups even out the
// centres' unequal work).  E.g. 4096 centres, 1792 resident: 1792 workgroups (1 round x 3) rather than 2048 (2 x 2).
inline int tri_grid(const void* kernel, size_t lds, int centres) {
  const int wmax = centres < TRI_GRID_MAX ? centres : TRI_GRID_MAX;
  static int cus = 0;   // one device kind per process
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = -1;
  }
  // the occupancy query is made once per (kernel, LDS size)
  static std::mutex mu;
  static std::map<std::pair<const void*, size_t>, int> known;
  int per_cu = 0;
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = known.find({kernel, lds});
    if (it != known.end()) {
      per_cu = it->second;
    } else {
      if (cus <= 0 || hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, TRI_BLOCK, lds) != hipSuccess) {
        (void)hipGetLastError();
        per_cu = 0;
      }
      known[{kernel, lds}] = per_cu;
    }
  }
  if (per_cu <= 0) return wmax;
  const long resident = (long)per_cu * cus;
  int best = wmax;
  long best_span = ((wmax + resident - 1) / resident) * (long)((centres + wmax - 1) / wmax);
  for (long k = (wmax + resident - 1) / resident - 1; k >= 1; k--) {
    const int w = (int)(k * resident);   // < wmax
    const long span = k * (long)((centres + w - 1) / w);
    if (span < best_span) { best = w; best_span = span; }
  }
  return best;
}

// Exponential of the hot loops.
// float: the argument is pre-scaled by log2(e) and fed to the hardware exp2 (two instructions; the rounding of the
// scaled product is of the same size as the rounding of the unscaled product inside expf).
// double: Cody-Waite reduction x = n ln2 + r, |r| <= ln2/2, degree-12 Taylor polynomial in Horner form (truncation
// 1.7e-16), ldexp; 18 instructions, measured maximum relative error 3.2e-16 over [-60, 60] against the C library.
// The 3-body kernels use the tabulated form below it (eval(x, table in LDS)).
// Overflow gives inf, underflow 0, NaN stays NaN; exp(+inf) gives NaN (arguments here are finite products).
template <typename real> struct HotExp;
template <> struct HotExp<float> {
  static constexpr int TABLE_REALS = 0;   // no table in LDS
  __device__ static float scale(float a) { return a * 1.44269504088896341f; }
  __device__ static float eval(float t) { return __builtin_amdgcn_exp2f(t); }
  __device__ static float eval(float t, const float*) { return __builtin_amdgcn_exp2f(t); }
  __device__ static float unscale() { return 0.693147180559945309f; }   // scaled argument -> natural argument
  __device__ static void fill(float*, int, int) {}
};
// 2^(i/128), i = 0..127, correctly rounded
static __device__ const double exp2_frac_128[128] = {
    1, 1.0054299011128027, 1.0108892860517005, 1.0163783149109531,
    1.0218971486541166, 1.0274459491187637, 1.0330248790212284, 1.0386341019613787,
    1.0442737824274138, 1.0499440858006872, 1.0556451783605572, 1.0613772272892621,
    1.0671404006768237, 1.0729348675259756, 1.0787607977571199, 1.0846183622133092,
    1.0905077326652577, 1.0964290818163769, 1.1023825833078409, 1.1083684117236787,
    1.1143867425958924, 1.1204377524096067, 1.1265216186082418, 1.1326385195987192,
    1.1387886347566916, 1.1449721444318042, 1.1511892299529827, 1.1574400736337511,
    1.1637248587775775, 1.1700437696832502, 1.1763969916502812, 1.182784710984341,
    1.189207115002721, 1.1956643920398273, 1.2021567314527031, 1.2086843236265816,
    1.215247359980469, 1.2218460329727576, 1.22848053610687, 1.2351510639369334,
    1.241857812073484, 1.2486009771892048, 1.2553807570246911, 1.2621973503942507,
    1.2690509571917332, 1.275941778396392, 1.2828700160787783, 1.2898358734066657,
    1.2968395546510096, 1.3038812651919358, 1.3109612115247644, 1.318079601266064,
    1.3252366431597413, 1.3324325470831615, 1.3396675240533029, 1.3469417862329458,
    1.3542555469368927, 1.3616090206382248, 1.3690024229745905, 1.3764359707545302,
    1.383909881963832, 1.3914243757719262, 1.3989796725383112, 1.4065759938190154,
    1.4142135623730951, 1.4218926021691656, 1.42961333839197, 1.4373759974489824,
    1.4451808069770467, 1.4530279958490526, 1.460917794180647, 1.4688504333369818,
    1.4768261459394993, 1.4848451658727524, 1.4929077282912648, 1.5010140696264256,
    1.5091644275934228, 1.5173590411982147, 1.5255981507445384, 1.5338819978409559,
    1.5422108254079407, 1.550584877685, 1.5590044002378369, 1.567469639965553,
    1.5759808451078865, 1.5845382652524937, 1.593142151342267, 1.6017927556826934,
    1.6104903319492543, 1.6192351351948637, 1.6280274218573478, 1.6368674497669644,
    1.6457554781539649, 1.6546917676561943, 1.6636765803267364, 1.6727101796415966,
    1.681792830507429, 1.6909247992693053, 1.7001063537185235, 1.7093377631004629,
    1.7186192981224779, 1.7279512309618377, 1.7373338352737062, 1.746767386199169,
    1.7562521603732995, 1.7657884359332727, 1.7753764925265212, 1.785016611318935,
    1.7947090750031072, 1.8044541678066239, 1.8142521755003989, 1.8241033854070534,
    1.8340080864093424, 1.843966568958626, 1.8539791250833855, 1.864046048397789,
    1.8741676341103, 1.8843441790323345, 1.8945759815869656, 1.9048633418176741,
    1.9152065613971474, 1.925605943636125, 1.9360617934922943, 1.9465744175792332,
    1.9571441241754002, 1.9677712232331759, 1.9784560263879509, 1.9891988469672663};
template <> struct HotExp<double> {
  static constexpr int TABLE_REALS = 128;   // 2^(i/128) in LDS for the tabulated form
  __device__ static double scale(double a) { return a; }
  __device__ static double eval(double x) {
    const double t = rint(x * 1.4426950408889634);
    double r = fma(t, -6.93147180369123816490e-01, x);
    r = fma(t, -1.90821492927058770002e-10, r);
    double p = 2.08767569878680989792e-09;        // 1/12!
    p = fma(p, r, 2.50521083854417187751e-08);
    p = fma(p, r, 2.75573192239858906526e-07);
    p = fma(p, r, 2.75573192239858906526e-06);
    p = fma(p, r, 2.48015873015873015873e-05);
    p = fma(p, r, 1.98412698412698412698e-04);
    p = fma(p, r, 1.38888888888888888889e-03);
    p = fma(p, r, 8.33333333333333333333e-03);
    p = fma(p, r, 4.16666666666666666667e-02);
    p = fma(p, r, 1.66666666666666666667e-01);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    return ldexp(p, (int)t);
  }
  // The same function with the reduction x = (128 k + i) ln2/128 + r, |r| <= ln2/256: e^x = 2^k 2^(i/128) e^r with
  // 2^(i/128) from `tab` (LDS, filled by fill()) and e^r by its Taylor polynomial of degree 5 (truncation 5e-19):
  // 15 vector instructions and one LDS read instead of 18; measured maximum relative error 3.0e-16 over [-60, 60]
  // against a 60-digit evaluation, as the form above.  Limits as above (inf, 0, NaN through ldexp and r).
  __device__ static double eval(double x, const double* tab) {
    const double t = rint(x * 184.6649652337873);              // 128 / ln2
    double r = fma(t, -0.00541521234663378, x);                // ln2/128, 32 significant bits: t times it is exact
    r = fma(t, -1.4907929134926466e-12, r);
    const int i = (int)t;
    const double f = tab[i & 127];
    double p = fma(r, 8.33333333333333333333e-03, 4.16666666666666666667e-02);
    p = fma(p, r, 1.66666666666666666667e-01);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    return ldexp(f * p, i >> 7);
  }
  __device__ static double unscale() { return 1.0; }
  __device__ static void fill(double* tab, int tid, int nthreads) {
    for (int i = tid; i < TABLE_REALS; i += nthreads) tab[i] = exp2_frac_128[i];
  }
};

// q / n for 0 <= q < 2^22, 1 <= n <= 2^11 without the integer-division sequence
__device__ inline int small_div(int q, int n, float inv_n) {
  int x = (int)(((float)q + 0.5f) * inv_n);
  if (x * n > q) --x;
  else if ((x + 1) * n <= q) ++x;
  return x;
}

template <typename real>
struct TriArgs {
  const real* Dsup;       // des3bsupp  [nf, ld, nr]
  const real* Tang;       // angdescr   [nf, ld, na] (not read by the FUSED kernel)
  const real* unit;       // FUSED: unit vectors centre - neighbour and 1/r of the sorted neighbours [nf, ld, 4, nr]
  const int* im2;         // intmap2b   [nf, ld, nr+1]
  const real* alpha3b;    // [ntc, 3*Aa]
  const real* emb3b;      // [ntc, Aa]
  const int* type_map;    // [N]
  const int* numtriplet;  // [nf, ld]
  const real* P;          // MODE 1: dL/dAF3, MODE 2 and 3: netderiv  [nf, Nl, Aa] contiguous
  const real* PE;         // MODE 3: dL/dAF3 [nf, Nl, Aa] contiguous
  const real* Q;          // MODE 2, 3: dL/dF [nf, 3N]
  const real* dDsup;      // MODE 2: der3bsupp [nf, ld, 3, nr]
  const real* d3b;        // MODE 2: der3b [nf, ld, 3, na, 2]
  const int* tipos;       // MODE 2
  const int* actual_type; // MODE 2
  const real* Qvir;       // MODE 2, virial form: dL/dW [nf, 9] (else null)
  const real* pos;        // MODE 2, virial form: positions [nf, 3N]
  const real* box;        // MODE 2, virial form: [nf, 6]
  int skip_pbc;           // MODE 2, virial form: no minimum-image wrap
  real* out;              // MODE 0: AF3, MODE 2, 3: gradnet  [nf, Nl, Aa] contiguous
  real* partial;          // MODE 1, 2: [gridDim.x, nsig*Aa*3]; MODE 3: [gridDim.x, 2, nsig*Aa*3] force branch, energy branch
  int nf, N, Nl, ld, nr, na, Aa, nt;
};

// A staged triplet: the offsets of its two table rows (16 bits each, in one word), T and -- force gradient -- the
// contraction U, laid out so that the inner loop takes them with one LDS read (two in the double-precision force
// gradient, whose LDS budget has no room for padding): every lane of a subset reads the same record.
//   float,  fingerprint / its gradient: {ab, T}          8 bytes
//   float,  force gradient:             {ab, T, U, -}   16 bytes
//   double, fingerprint / its gradient: {ab, -, T}      16 bytes
//   double, force gradient:             {T, U} 16 bytes in one array, ab in a second one
template <typename real, int MODE>
struct TriStage {
  static constexpr bool WITH_U = MODE == 2 || MODE == 3;
  static constexpr bool SPLIT = WITH_U && sizeof(real) == 8;
  static constexpr int BYTES = SPLIT ? 20 : ((sizeof(real) == 4 && !WITH_U) ? 8 : 16);
  unsigned char* base;   // 16-byte aligned; SPLIT: QB records of 16 bytes, then QB words
  int qb;
  __device__ void put(int qq, unsigned ab, real T, real U) const {
    if constexpr (SPLIT) {
      double2 v;
      v.x = T; v.y = U;
      ((double2*)base)[qq] = v;
      ((unsigned*)(base + (size_t)qb * 16))[qq] = ab;
    } else if constexpr (sizeof(real) == 4 && !WITH_U) {
      ((uint2*)base)[qq] = make_uint2(ab, __float_as_uint((float)T));
    } else if constexpr (sizeof(real) == 4) {
      ((uint4*)base)[qq] = make_uint4(ab, __float_as_uint((float)T), __float_as_uint((float)U), 0u);
    } else {
      const unsigned long long t = (unsigned long long)__double_as_longlong((double)T);
      ((uint4*)base)[qq] = make_uint4(ab, 0u, (unsigned)(t & 0xffffffffull), (unsigned)(t >> 32));
    }
  }
  __device__ void get(int qq, unsigned& ab, real& T, real& U) const {
    if constexpr (SPLIT) {
      const double2 v = ((const double2*)base)[qq];
      T = (real)v.x; U = (real)v.y;
      ab = ((const unsigned*)(base + (size_t)qb * 16))[qq];
    } else if constexpr (sizeof(real) == 4 && !WITH_U) {
      const uint2 v = ((const uint2*)base)[qq];
      ab = v.x; T = (real)__uint_as_float(v.y); U = 0;
    } else if constexpr (sizeof(real) == 4) {
      const uint4 v = ((const uint4*)base)[qq];
      ab = v.x; T = (real)__uint_as_float(v.y); U = (real)__uint_as_float(v.z);
    } else {
      const uint4 v = ((const uint4*)base)[qq];
      ab = v.x;
      T = (real)__longlong_as_double((long long)(((unsigned long long)v.w << 32) | v.z));
      U = 0;
    }
  }
};

template <typename real, int MODE, bool FUSED = false>
struct TriLds {
  static constexpr int NV = (MODE == 0) ? 1 : (MODE == 1 ? 3 : (MODE == 2 ? 4 : 7));
  static constexpr int NG = MODE == 3 ? 2 : 1;   // parameter-gradient sets (force branch, energy branch)
  static constexpr int QB = TriCfg<real, MODE, FUSED>::QB;
  __host__ __device__ static size_t n_reals(int nr, int Aa, int nt, bool fused = false) {
    const int nsig = 2 * nt - 1;
    size_t r = (size_t)nr * TRI_CAPP * 2;                   // pair tables (real2 per (row, channel)), + (D, V) per row
    if (fused) r += (size_t)3 * nr;                         // unit vectors of the slots
    r += nr;                                                // sD
    r += (size_t)NG * Aa;                                   // sP (and sPE)
    r += (size_t)TRI_WAVES * Aa;                            // per-wave channel sums
    if (MODE != 0) r += (size_t)NG * nsig * Aa * 3;         // parameter-gradient sums of the workgroup
    if (MODE != 0) r += (size_t)NG * TRI_WAVES * TRI_CAP * 3;   // exchange buffer of a pass
    if (MODE == 2 || MODE == 3) r += (size_t)4 * nr;        // sV, sQ
    return r;
  }
  __host__ __device__ static size_t bytes(int nr, int Aa, int nt, bool fused = false) {
    size_t b = chan_table_bytes<real>(2 * nt - 1, Aa) + n_reals(nr, Aa, nt, fused) * sizeof(real);
    b += (size_t)HotExp<real>::TABLE_REALS * sizeof(real);  // table of the exponential
    b += 16 + (size_t)QB * TriStage<real, MODE>::BYTES;     // staged triplets, 16-byte aligned
    b += (size_t)(2 * nr + NT_MAX + 1) * sizeof(int);
    return (b + 15) & ~(size_t)15;
  }
};

// FUSED (MODE 0 only, the MD entry): the angular descriptor of a triplet is not read from angdescr but rebuilt from
// the slots' unit vectors and cutoff values, T = 1/2 (u_j . u_k + 1) fc_j fc_k
// (DescriptorsAngular_kernel, STAF/src/descriptor_builder/reforce.cu.cc:195-212), so no na-wide tensor exists.
// The kernel's body, for a workgroup that takes centres first, first + stride, ... (row-major over frames and the
// species' atoms) and leaves its parameter-gradient sums in row part_row of A.partial: tri_reduce_kernel below,
// and the launch that computes descriptors and fingerprints of a centre in one workgroup.
template <typename real, int MODE, bool FUSED = false>
__device__ __forceinline__ void tri_reduce_body(const TriArgs<real> A, const int first_centre, const int stride,
                                                const int part_row) {
  static_assert(!FUSED || MODE == 0, "only the fingerprint mode rebuilds T");
  using real2 = typename Vec2<real>::type;
  using HE = HotExp<real>;
  constexpr int NV = TriLds<real, MODE>::NV, NG = TriLds<real, MODE>::NG;
  constexpr int TRI_QB = TriCfg<real, MODE, FUSED>::QB;
  constexpr bool FB = TriCfg<real, MODE>::FORCE_BRANCH;
  extern __shared__ __align__(16) unsigned char smem[];
  const int nr = A.nr, na = A.na, Aa = A.Aa, nt = A.nt;
  const int nsig = 2 * nt - 1;
  const int nacc = nsig * Aa * 3;
  ChanTable<real> tab;
  unsigned char* sp = tab.carve(smem, nsig, Aa);
  real* rp = (real*)sp;   // 16-byte aligned: the pair tables come first
  real2* tabE = (real2*)rp; rp += (size_t)nr * TRI_CAPP * 2;   // rows of both species of a class: at most m <= nr
  real* sUn = rp; if (FUSED) rp += (size_t)3 * nr;             // [3][nr] unit vectors
  real* sD = rp; rp += nr;
  real* sP = rp; rp += Aa;
  real* sPE = rp; if (MODE == 3) rp += Aa;                     // MODE 3: dL/dAF3 of the centre beside its netderiv
  real* outw = rp; rp += (size_t)TRI_WAVES * Aa;
  real* accw = rp; if (MODE != 0) rp += (size_t)NG * nacc;     // [NG][nacc]
  real* xch = rp; if (MODE != 0) rp += (size_t)TRI_WAVES * TRI_CAP * 3 * NG;   // [wave][channel][3 NG]
  real* sV = rp;
  real* sQ = rp + nr;
  if (FB) rp += (size_t)4 * nr;
  real* etab = rp; rp += HE::TABLE_REALS;   // table of the exponential (double precision)
  TriStage<real, MODE> stage;                   // [TRI_QB] staged triplets
  stage.base = smem + ((((unsigned char*)rp - smem) + 15) & ~(ptrdiff_t)15);   // an offset into smem, not an integer cast
  stage.qb = TRI_QB;
  int* lst = (int*)(stage.base + (size_t)TRI_QB * TriStage<real, MODE>::BYTES);
  int* stp = lst + nr;
  int* off = stp + nr;

  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int ia = tid & (TRI_CAP - 1), sub = tid / TRI_CAP;
  // The reads of the workgroup's first centre that need no other read's result (triplet count, neighbour index and
  // descriptor values of slot tid) are issued ahead of everything else, together with the parameter rows: a centre
  // then waits for two rounds of global reads (these, and what the neighbour index addresses) instead of four.
  // Slots are read up to nr whatever the count: rows are nr long.
  int m0, nj0 = 0;
  real d0 = 0, gr0[3] = {0, 0, 0}, un0[3] = {0, 0, 0};
  {
    const int b0 = first_centre / A.Nl, p0 = first_centre - b0 * A.Nl;
    const size_t row0 = (size_t)b0 * A.ld + p0;
    m0 = A.numtriplet[row0];
    if (tid < nr) {
      nj0 = A.im2[row0 * (nr + 1) + 1 + tid];
      d0 = A.Dsup[row0 * nr + tid];
      if (FB) {
#pragma unroll
        for (int c = 0; c < 3; c++) gr0[c] = A.dDsup[row0 * 3 * nr + c * nr + tid];
      }
      if (FUSED) {
#pragma unroll
        for (int c = 0; c < 3; c++) un0[c] = A.unit[(row0 * 4 + c) * nr + tid];
      }
    }
  }
  tab.build(A.alpha3b, A.emb3b);
  HE::fill(etab, tid, TRI_BLOCK);
  if (MODE != 0)
    for (int q = tid; q < NG * nacc; q += TRI_BLOCK) accw[q] = 0;
  int shift = 0;
  if (FB) {
    const int at = A.actual_type[0];
    for (int y = 0; y < at; y++) shift += A.tipos[y];
  }
  real* my_out = outw + wave * Aa;
  real* my_xch = xch + (size_t)wave * TRI_CAP * 3 * NG;
  // Parameter-gradient sums of the last pass: thread ia < 16 of the workgroup adds the four waves' values of its
  // channel to accumulator row `pending` (-1: nothing to add).  Called right after a barrier that follows the pass
  // and before the next one, so that the exchange buffer is complete and not yet rewritten.
  int pending = -1;
  auto flush_pass = [&]() {
    if (MODE != 0 && tid < TRI_CAP && pending >= 0) {
#pragma unroll
      for (int g = 0; g < NG; g++) {
#pragma unroll
        for (int v = 0; v < 3; v++) {
          real s = xch[ia * 3 * NG + g * 3 + v];
#pragma unroll
          for (int w = 1; w < TRI_WAVES; w++) s += xch[(w * TRI_CAP + ia) * 3 * NG + g * 3 + v];
          accw[g * nacc + pending + v] += s;
        }
      }
    }
    pending = -1;
  };
  __syncthreads();

  const int total = A.nf * A.Nl;
  // Per-centre set-up: slot data into LDS.  The first centre takes what was read at the kernel's start (a separate
  // copy of the code, so that those registers are free afterwards); later centres of a persistent workgroup read here.
  int m = 0, t_mine = -1;   // neighbours inside the angular cutoff; species of slot tid
  const real* Trow = nullptr;
  const real2* d3 = nullptr;
  auto centre_setup = [&](int atom, auto early_c) {
    const int b = atom / A.Nl, p = atom - b * A.Nl;
    const size_t rowAtom = (size_t)b * A.ld + p;
    const int* im = A.im2 + rowAtom * (nr + 1);
    constexpr bool early = decltype(early_c)::value;   // the centre whose first reads were issued at the kernel's start
    m = early ? m0 : A.numtriplet[rowAtom];
    m = m > nr ? nr : (m < 0 ? 0 : m);
    Trow = A.Tang + rowAtom * na;
    d3 = (const real2*)A.d3b + rowAtom * 3 * na;
    // ---- per-atom slot data
    t_mine = -1;
    for (int s = tid; s < m; s += TRI_BLOCK) {
      const bool have = early && s == tid;
      sD[s] = have ? d0 : A.Dsup[rowAtom * nr + s];
      if (FUSED) {
#pragma unroll
        for (int c = 0; c < 3; c++) sUn[c * nr + s] = have ? un0[c] : A.unit[(rowAtom * 4 + c) * nr + s];
      }
      const int nj = have ? nj0 : im[1 + s];
      const int t_s = A.type_map[nj];
      stp[s] = t_s;
      if (s == tid) t_mine = t_s;
      if (FB) {
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
        const real g0 = have ? gr0[0] : gr[0], g1 = have ? gr0[1] : gr[nr], g2 = have ? gr0[2] : gr[2 * nr];
        sQ[3 * s] = q0; sQ[3 * s + 1] = q1; sQ[3 * s + 2] = q2;
        sV[s] = q0 * g0 + q1 * g1 + q2 * g2;
      }
    }
    for (int a = tid; a < Aa; a += TRI_BLOCK) {
      if (MODE != 0) sP[a] = A.P[(size_t)atom * Aa + a];
      if (MODE == 3) sPE[a] = A.PE[(size_t)atom * Aa + a];
    }
    for (int q = tid; q < TRI_WAVES * Aa; q += TRI_BLOCK) outw[q] = 0;
  };
  int atom = first_centre;
  centre_setup(atom, std::true_type{});
  while (true) {
    if (m <= WAVE) {
      // all slots are in the first wave's registers: it groups them by species before the barrier
      if (tid < WAVE) group_slots_by_type_reg(m, nt, t_mine, lst, off);
      __syncthreads();
    } else {
      __syncthreads();
      if (tid < WAVE) group_slots_by_type(m, nt, stp, lst, off);
      __syncthreads();
    }

    bool first = true;
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
        const int nrows = same ? na_ : na_ + nb_;   // rows of the second species follow the first
        const int rowB0 = same ? 0 : na_;
        const float inv_nb = 1.0f / (float)nb_;
        for (int c0 = 0; c0 < nact; c0 += TRI_CAP) {
          const int nch = (nact - c0) < TRI_CAP ? (nact - c0) : TRI_CAP;
          const bool chan = ia < nch;
          real a1 = 0, a2 = 0, be = 0;
          if (chan) { a1 = tab.a1[pb + c0 + ia]; a2 = tab.a2[pb + c0 + ia]; be = tab.be[pb + c0 + ia]; }
          const real a1s = HE::scale(a1), a2s = HE::scale(a2), bes = HE::scale(be);
          if (!first) {
            __syncthreads();   // tables and staged block of the previous pass fully consumed
            flush_pass();
          }
          first = false;
          // ---- tables of the class: E[row][ia] = (exp(a1 D), exp(a2 D)), D (and V) by row
          for (int row = sub; row < nrows; row += TRI_SUBS) {
            const int s = row < na_ ? la[row] : lb[row - na_];
            const real d = sD[s];
            if (chan) {
              real2 v;
              v.x = HE::eval(a1s * d, etab);
              v.y = HE::eval(a2s * d, etab);
              tabE[row * TRI_CAPP + ia] = v;
            }
            if (ia == 0) {
              real2 v;
              v.x = d;
              v.y = FB ? sV[s] : real(0);
              tabE[row * TRI_CAPP + TRI_CAP] = v;
            }
          }
          real acc[NV];
#pragma unroll
          for (int v = 0; v < NV; v++) acc[v] = 0;
          for (int q0 = 0; q0 < size; q0 += TRI_QB) {
            const int nq = (size - q0) < TRI_QB ? (size - q0) : TRI_QB;
            // The block is padded to a whole number of rounds of the TRI_SUBS subsets with triplets of T = U = 0 on
            // table row 0 (they add exact zeros): every subset then makes the same number of steps, and the loop below
            // runs on a scalar counter.
            const int nq_pad = (nq + TRI_SUBS - 1) & ~(TRI_SUBS - 1);
            if (q0 > 0) __syncthreads();   // previous block consumed
            // ---- stage a block of triplets
            for (int qq = nq + tid; qq < nq_pad; qq += TRI_BLOCK) stage.put(qq, 0u, real(0), real(0));
            for (int qq = tid; qq < nq; qq += TRI_BLOCK) {
              const int q = q0 + qq;
              int x, y;
              if (same) tri_decode_xy(q, nb_, x, y);
              else { x = small_div(q, nb_, inv_nb); y = q - x * nb_; }
              const int s1 = la[x], s2 = lb[y];
              const int j = s1 < s2 ? s1 : s2, k = s1 < s2 ? s2 : s1;
              const int nn = tri_rowstart(j, m) + k - j - 1;
              const bool ok = nn < na;
              const unsigned ab = (unsigned)(x * TRI_CAPP) | ((unsigned)((rowB0 + y) * TRI_CAPP) << 16);
              real T = 0, U = 0;
              if (ok) {
                if constexpr (FUSED) {
                  const real cs = sUn[j] * sUn[k] + sUn[nr + j] * sUn[nr + k] + sUn[2 * nr + j] * sUn[2 * nr + k];
                  T = (real(0.5) * (cs + real(1))) * (sD[j] * sD[k]);
                } else {
                  T = Trow[nn];
                }
              }
              if (FB) {
                if (ok) {
#pragma unroll
                  for (int c = 0; c < 3; c++) {
                    const real2 dv = d3[c * na + nn];
                    U += sQ[3 * j + c] * dv.x + sQ[3 * k + c] * dv.y;
                  }
                }
              }
              stage.put(qq, ab, T, U);
            }
            __syncthreads();
            // ---- thread <-> (channel ia, subset sub)
            if (chan) {
              const int rounds = nq_pad / TRI_SUBS;
#pragma unroll 2
              for (int it = 0; it < rounds; it++) {
                const int qq = sub + it * TRI_SUBS;
                unsigned ab;
                real T, U;
                stage.get(qq, ab, T, U);
                const real2* r1 = tabE + (ab & 0xffffu);
                const real2* r2 = tabE + (ab >> 16);
                const real2 e1 = r1[ia];
                const real2 e2 = r2[ia];
                const real ebt = HE::eval(bes * T, etab);
                const real sim2 = e1.x * e2.y;   // exp(a1 D1 + a2 D2)
                const real sim1 = e1.y * e2.x;   // exp(a2 D1 + a1 D2)
                if constexpr (MODE == 0) {
                  acc[0] += T * (sim1 + sim2) * ebt;
                } else if constexpr (MODE == 1) {
                  const real D1 = r1[TRI_CAP].x, D2 = r2[TRI_CAP].x;
                  const real w = ebt * T;
                  acc[0] += (sim2 * D1 + sim1 * D2) * w;
                  acc[1] += (sim2 * D2 + sim1 * D1) * w;
                  acc[NV - 1] += (sim1 + sim2) * w * T;
                } else {
                  const real2 g1 = r1[TRI_CAP], g2 = r2[TRI_CAP];
                  const real D1 = g1.x, D2 = g2.x, V1 = g1.y, V2 = g2.y;
                  // With A = a1 V1 + a2 V2, B = a1 V2 + a2 V1 (the factor 1/2 of both weights is applied once per
                  // channel at the end) and W = sim2 A + sim1 B:
                  //   d/dG      : hU ss + hT W                         hT = e^{bT} T,  hU = e^{bT} (1 + bT) U
                  //   d/da1     : hU (sim2 D1 + sim1 D2) + hT (sim2 (V1 + D1 A) + sim1 (V2 + D2 B))
                  //   d/da2     : hU (sim1 D1 + sim2 D2) + hT (sim1 (V1 + D1 B) + sim2 (V2 + D2 A))
                  //   d/dbeta   : hT ((2 + bT) ss U + T W) = T (hU ss + hT W + e^{bT} U ss): T times (the d/dG term + eU ss)
                  // (the sums of the reference's per-term products, STAF/src/grad_force/ang/reforce.cu.cc:120-200,
                  // with the common factors taken out: 38 operations per item beside the exponential)
                  const real bT = be * T;
                  const real hT = ebt * T;
                  const real eU = ebt * U;
                  const real hU = r_fma(eU, bT, eU);
                  const real ss = sim1 + sim2;
                  const real Aw = r_fma(a1, V1, a2 * V2);
                  const real Bw = r_fma(a1, V2, a2 * V1);
                  const real W = r_fma(sim2, Aw, sim1 * Bw);
                  const real dG = r_fma(hT, W, hU * ss);
                  acc[0] += dG;
                  const real pq = r_fma(sim2, D1, sim1 * D2);
                  const real rt = r_fma(sim1, D1, sim2 * D2);
                  acc[1] = r_fma(hU, pq, acc[1]);
                  acc[1] = r_fma(hT, r_fma(sim2, r_fma(D1, Aw, V1), sim1 * r_fma(D2, Bw, V2)), acc[1]);
                  acc[2] = r_fma(hU, rt, acc[2]);
                  acc[2] = r_fma(hT, r_fma(sim1, r_fma(D1, Bw, V1), sim2 * r_fma(D2, Aw, V2)), acc[2]);
                  acc[3] = r_fma(T, r_fma(eU, ss, dG), acc[3]);
                  if constexpr (MODE == 3) {
                    // the energy branch's sums of the same item (MODE 1 above with w = hT):
                    // d/da1: (sim2 D1 + sim1 D2) w,  d/da2: (sim2 D2 + sim1 D1) w,  d/dbeta: (sim1 + sim2) w T
                    acc[4] = r_fma(pq, hT, acc[4]);
                    acc[5] = r_fma(rt, hT, acc[5]);
                    acc[6] = r_fma(ss * hT, T, acc[6]);
                  }
                }
              }
            }
          }
          // ---- the wave's four subsets of every channel, then the wave's own accumulators (fixed order)
#pragma unroll
          for (int v = 0; v < NV; v++) {
            real s = acc[v];
            s += __shfl_xor(s, 16, WAVE);
            s += __shfl_xor(s, 32, WAVE);
            acc[v] = s;
          }
          if (lane < TRI_CAP && chan) {
            const int a = tab.ch[pb + c0 + ia];
            const real c3h = tab.c3[pb + c0 + ia] * real(FB ? 0.25 : 0.5);
            if constexpr (MODE == 0) {
              my_out[a] += acc[0] * c3h;
            } else if constexpr (MODE == 1) {
              const real f = c3h * sP[a];
#pragma unroll
              for (int v = 0; v < 3; v++) my_xch[ia * 3 + v] = acc[v] * f;
            } else {
              my_out[a] += acc[0] * c3h;
              const real f = c3h * sP[a];
#pragma unroll
              for (int v = 0; v < 3; v++) my_xch[ia * 3 * NG + v] = acc[v + 1] * f;
              if constexpr (MODE == 3) {
                const real fe = (c3h + c3h) * sPE[a];   // 1/2 c3 dL/dAF3: the energy branch's weight
#pragma unroll
                for (int v = 0; v < 3; v++) my_xch[ia * 6 + 3 + v] = acc[v + 4] * fe;
              }
            }
            if (MODE != 0) pending = (sg * Aa + a) * 3;
          }
        }
      }
    }
    __syncthreads();
    flush_pass();
    if (MODE != 1)
      for (int a = tid; a < Aa; a += TRI_BLOCK) {
        real s = 0;
#pragma unroll
        for (int w = 0; w < TRI_WAVES; w++) s += outw[w * Aa + a];
        A.out[(size_t)atom * Aa + a] = s;
      }
    __syncthreads();
    if (stride > total - 1 - atom) break;   // (no overflow of atom + stride)
    atom += stride;
    centre_setup(atom, std::false_type{});
  }
  if (MODE != 0) {
    for (int q = tid; q < NG * nacc; q += TRI_BLOCK) A.partial[(size_t)part_row * NG * nacc + q] = accw[q];
  }
}

template <typename real, int MODE, bool FUSED = false>
__global__ __launch_bounds__(TRI_BLOCK, (TriCfg<real, MODE, FUSED>::MIN_WAVES)) void
tri_reduce_kernel(TriArgs<real> A) {
  tri_reduce_body<real, MODE, FUSED>(A, (int)blockIdx.x, (int)gridDim.x, (int)blockIdx.x);
}

}  // namespace staf
