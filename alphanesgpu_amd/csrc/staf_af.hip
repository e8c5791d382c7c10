// Atomic fingerprints (2-body, 3-body) and their parameter gradients from the
// energy branch.  Replaces radialAFs_kernel, angularAFs_kernel,
// alphagrad_dist_kernel and alphagrad_ang_kernel
// (STAF/src/fingerprint/{rad,ang}/reforce.cu.cc, STAF/src/grad_finger/{rad,ang}/reforce.cu.cc).
//
// One wavefront owns one centre atom.  Sums over an atom's slots/triplets are
// reduced inside the wave with a fixed butterfly; sums over atoms (the
// parameter gradients) go through per-workgroup partials and a second,
// fixed-order pass.  There are no floating-point atomics, so results are
// bit-reproducible from run to run.
#include "staf_tile.hpp"
#include "staf_reduce.hpp"
#include "staf_tri.hpp"
#include "staf_af2.hpp"

#include <stdio.h>
#include <mutex>
#include <unordered_map>

namespace staf {

constexpr int AF_BLOCK = 256;
constexpr int AF_WAVES = AF_BLOCK / WAVE;
constexpr int GRAD_MAX_BLOCKS = 1024;

// ---------------------------------------------------------------------------
// 2-body fingerprints: AF2[b,p,a] = sum_s D_s exp(alpha[t_s,a] D_s) c2[t_s,a]
// ---------------------------------------------------------------------------
template <typename real>
__global__ __launch_bounds__(AF_BLOCK) void af2_kernel(const real* __restrict__ D, const int* __restrict__ im2,
                                                       const real* __restrict__ alpha2b,
                                                       const real* __restrict__ emb2b,
                                                       const int* __restrict__ type_map, real* __restrict__ out,
                                                       int nf, int Nl, int ld, int nr, int Ar, int nt) {
  extern __shared__ __align__(16) unsigned char smem[];
  real* p_al = (real*)smem;          // [nt*Ar] alpha in the units of the hot exponential
  real* p_c2 = p_al + nt * Ar;       // [nt*Ar]
  real* w_D = p_c2 + nt * Ar;        // [AF_WAVES][nr]
  int* w_t = (int*)(w_D + AF_WAVES * nr);  // [AF_WAVES][nr]
  af2_tables(alpha2b, emb2b, nt * Ar, p_al, p_c2);
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  real* myD = w_D + wave * nr;
  int* myT = w_t + wave * nr;
  const int atom = blockIdx.x * AF_WAVES + wave;
  int cnt = 0;
  if (atom < nf * Nl) {
    const int b = atom / Nl, p = atom - b * Nl;
    const size_t rowAtom = (size_t)b * ld + p;
    cnt = af2_wave_load(D + rowAtom * nr, im2 + rowAtom * (nr + 1), type_map, nr, Ar, myD, myT, lane);
  }
  __syncthreads();
  if (atom >= nf * Nl) return;
  af2_wave_sum(p_al, p_c2, myD, myT, cnt, Ar, out + (size_t)atom * Ar, lane);
}

// ---------------------------------------------------------------------------
// dL/dalpha2b, dL/demb2b from P = dL/dAF2:
//   dalpha[t,a] += P c2 D^2 e^{alpha D},  demb[t,a] += P D e^{alpha D}
// The slots of a centre are grouped by neighbour species, so that a lane's running sums belong to one species at
// a time; workgroup partials.
// ---------------------------------------------------------------------------
template <typename real>
__global__ __launch_bounds__(AF_BLOCK) void grad2_kernel(const real* __restrict__ D, const int* __restrict__ im2,
                                                         const real* __restrict__ alpha2b,
                                                         const real* __restrict__ emb2b,
                                                         const int* __restrict__ type_map,
                                                         const real* __restrict__ P, real* __restrict__ partial,
                                                         int nf, int Nl, int ld, int nr, int Ar, int nt) {
  using HE = HotExp<real>;
  extern __shared__ __align__(16) unsigned char smem[];
  real* p_al = (real*)smem;                 // [nt*Ar] alpha in the units of the hot exponential
  real* p_c2 = p_al + nt * Ar;              // [nt*Ar]
  real* w_acc = p_c2 + nt * Ar;             // [AF_WAVES][2*nt*Ar]
  real* w_D = w_acc + AF_WAVES * 2 * nt * Ar;  // [AF_WAVES][nr] D of the slots in grouped order
  int* w_t = (int*)(w_D + AF_WAVES * nr);   // [AF_WAVES][nr] species of the slot
  int* w_l = w_t + AF_WAVES * nr;           // [AF_WAVES][nr] slots grouped by species
  int* w_o = w_l + AF_WAVES * nr;           // [AF_WAVES][NT_MAX+1] first grouped position of a species
  for (int q = threadIdx.x; q < nt * Ar; q += blockDim.x) { p_al[q] = HE::scale(alpha2b[q]); p_c2[q] = emb2b[q]; }
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  real* myD = w_D + wave * nr;
  int* myT = w_t + wave * nr;
  int* myL = w_l + wave * nr;
  int* myO = w_o + wave * (NT_MAX + 1);
  real* myAcc = w_acc + wave * 2 * nt * Ar;
  for (int q = lane; q < 2 * nt * Ar; q += WAVE) myAcc[q] = 0;
  __syncthreads();
  const ChanSub cs(lane, Ar);
  const int total = nf * Nl;
  const int stride = gridDim.x * AF_WAVES;
  for (int atom = blockIdx.x * AF_WAVES + wave; atom < total; atom += stride) {
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
    for (int q = lane; q < cnt; q += WAVE) myD[q] = D[rowAtom * nr + myL[q]];
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    for (int a0 = 0; a0 < Ar; a0 += cs.chunk) {
      const int a = a0 + cs.a;
      const bool on = cs.sub < cs.nsub && a < Ar;
      const real pg = on ? P[(size_t)atom * Ar + a] : real(0);
      for (int t = 0; t < nt; t++) {
        const int q0 = uniform(myO[t]), q1 = uniform(myO[t + 1]);
        if (q0 == q1) continue;
        real ga = 0, ge = 0;
        if (on) {
          const real al = p_al[t * Ar + a];
          for (int q = q0 + cs.sub; q < q1; q += cs.nsub) {
            const real d = myD[q];
            const real de = d * HE::eval(al * d);
            ge += de;
            ga += d * de;
          }
          ga *= p_c2[t * Ar + a] * pg;
          ge *= pg;
        }
        ga = cs.combine(ga, lane);
        ge = cs.combine(ge, lane);
        if (on && cs.sub == 0) { myAcc[t * Ar + a] += ga; myAcc[nt * Ar + t * Ar + a] += ge; }
      }
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
  __syncthreads();
  const int nout = 2 * nt * Ar;
  for (int q = threadIdx.x; q < nout; q += blockDim.x) {
    real s = 0;
#pragma unroll
    for (int w = 0; w < AF_WAVES; w++) s += w_acc[w * nout + q];
    partial[(size_t)blockIdx.x * nout + q] = s;
  }
}

// ---- host launchers --------------------------------------------------------

static inline int grad_blocks(int atoms) {
  int nb = (atoms + AF_WAVES - 1) / AF_WAVES;
  return nb < GRAD_MAX_BLOCKS ? nb : GRAD_MAX_BLOCKS;
}

template <typename real>
static int radial_afs(const real* D, int nr, const real* alpha2b, int Ar, real* out, int nf, int Nl, const int* im2,
                      const real* emb2b, const int* type_map, int nt, int ld, void* stream_) {
  if (Nl == 0 && nf > 0 && Ar > 0) return STAF_OK;   // a species without atoms in these frames: nothing to write
  if (!D || !alpha2b || !out || !im2 || !emb2b || !type_map || nr <= 0 || Ar <= 0 || nf <= 0 || Nl <= 0 || nt <= 0)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  size_t lds = (size_t)2 * nt * Ar * sizeof(real) + (size_t)AF_WAVES * nr * (sizeof(real) + sizeof(int));
  if (lds > 64 * 1024) return STAF_E_LIMIT;
  const int atoms = nf * Nl;
  {
    KernelTimer kt_("af2_kernel", (hipStream_t)stream_);
    hipLaunchKernelGGL(af2_kernel<real>, dim3((atoms + AF_WAVES - 1) / AF_WAVES), dim3(AF_BLOCK), lds,
                       (hipStream_t)stream_, D, im2, alpha2b, emb2b, type_map, out, nf, Nl, ld, nr, Ar, nt);
  }
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

// Work area of the 2-body parameter gradient: one row of 2*nt*Ar partial sums per workgroup of grad2_kernel, then
// RED_SLICES spare rows (an earlier form of the reduction used them; the size is part of the documented limit of
// the entry point that allocates nothing).
static inline size_t grad2_work_reals(int nf, int Nl, int nt, int Ar) {
  return ((size_t)grad_blocks(nf * Nl) + RED_SLICES) * 2 * nt * Ar;
}

template <typename real>
static int alpha_dist_grad_check(const real* D, int nr, const real* alpha2b, int Ar, real* g_alpha, int nf, int Nl,
                                 const int* im2, const real* P, const real* emb2b, const int* type_map, real* g_emb,
                                 int nt) {
  if (!D || !alpha2b || !g_alpha || !g_emb || !im2 || !P || !emb2b || !type_map || nr <= 0 || Ar <= 0 || nf <= 0 ||
      Nl <= 0 || nt <= 0)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  const size_t lds = (size_t)(2 * nt * Ar + AF_WAVES * 2 * nt * Ar + AF_WAVES * nr) * sizeof(real) +
                     (size_t)AF_WAVES * (2 * nr + NT_MAX + 1) * sizeof(int);
  if (lds > 64 * 1024) return STAF_E_LIMIT;
  return STAF_OK;
}

// Launches grad2_kernel and the fixed-order reduction on `work` (grad2_work_reals reals, every element written
// before it is read: nothing has to be cleared).  timed: bracket the kernel with events when timing is switched on.
template <typename real>
static int alpha_dist_grad_launch(const real* D, int nr, const real* alpha2b, int Ar, real* g_alpha, int nf, int Nl,
                                  const int* im2, const real* P, const real* emb2b, const int* type_map, real* g_emb,
                                  int nt, int ld, real* work, bool timed, hipStream_t stream) {
  const int nout = 2 * nt * Ar;
  const int nb = grad_blocks(nf * Nl);
  real* partial = work;
  real* red_tmp = work + (size_t)nb * nout;
  const size_t lds = (size_t)(2 * nt * Ar + AF_WAVES * nout + AF_WAVES * nr) * sizeof(real) +
                     (size_t)AF_WAVES * (2 * nr + NT_MAX + 1) * sizeof(int);
  if (timed) {
    KernelTimer kt_("grad2_kernel", stream);
    hipLaunchKernelGGL(grad2_kernel<real>, dim3(nb), dim3(AF_BLOCK), lds, stream, D, im2, alpha2b, emb2b, type_map, P,
                       partial, nf, Nl, ld, nr, Ar, nt);
  } else {
    hipLaunchKernelGGL(grad2_kernel<real>, dim3(nb), dim3(AF_BLOCK), lds, stream, D, im2, alpha2b, emb2b, type_map, P,
                       partial, nf, Nl, ld, nr, Ar, nt);
  }
  launch_reduce_partials<real>(partial, nb, nout, g_alpha, nt * Ar, nt * Ar, g_emb, nt * Ar, nt * Ar, red_tmp, stream);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

template <typename real>
static int alpha_dist_grad(const real* D, int nr, const real* alpha2b, int Ar, real* g_alpha, int nf, int Nl,
                           const int* im2, const real* P, const real* emb2b, const int* type_map, real* g_emb, int nt,
                           int ld, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (Nl == 0 && nf > 0 && Ar > 0 && nt > 0 && g_alpha && g_emb) {
    // a species without atoms in these frames: its sums are empty
    launch_fill_zero<real>(g_alpha, nt * Ar, stream);
    launch_fill_zero<real>(g_emb, nt * Ar, stream);
    return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  }
  const int rc = alpha_dist_grad_check<real>(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt);
  if (rc) return rc;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  real* work = (real*)scratch_reserve(st, stream, grad2_work_reals(nf, Nl, nt, Ar) * sizeof(real));
  if (!work) return reserve_failure(stream);
  return alpha_dist_grad_launch<real>(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt, ld,
                                      work, true, stream);
}

// ---- the same op for callers that cannot allocate -------------------------------------------------------------
// Work area in the library's own image instead of hipMalloc'ed memory: each GPU the library is loaded on holds its
// own copy of this array, at its own address, until the process ends.  The name below is a host-side handle only;
// the device address is asked for once per device (noalloc_work) and that address is what kernels are given.
constexpr size_t NOALLOC_WORK_BYTES = (size_t)1 << 20;
static __device__ __align__(256) unsigned char scratch[NOALLOC_WORK_BYTES];

static std::mutex g_noalloc_mu;
static std::unordered_map<int, void*> g_noalloc_ptr;   // device ordinal -> device address of `scratch` there

static void* noalloc_work() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_noalloc_mu);
  auto it = g_noalloc_ptr.find(dev);
  if (it != g_noalloc_ptr.end()) return it->second;
  void* ptr = nullptr;
  if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
    (void)hipGetLastError();
    return nullptr;
  }
  g_noalloc_ptr.emplace(dev, ptr);
  return ptr;
}

static int alpha_dist_grad_noalloc(const double* D, int nr, const double* alpha2b, int Ar, double* g_alpha, int nf,
                                   int Nl, const int* im2, const double* P, const double* emb2b, const int* type_map,
                                   double* g_emb, int nt, int ld, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (Nl == 0 && nf > 0 && Ar > 0 && nt > 0 && g_alpha && g_emb) {
    launch_fill_zero<double>(g_alpha, nt * Ar, stream);
    launch_fill_zero<double>(g_emb, nt * Ar, stream);
    return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  }
  const int rc = alpha_dist_grad_check<double>(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt);
  if (rc) return rc;
  const size_t need = grad2_work_reals(nf, Nl, nt, Ar) * sizeof(double);
  if (need > NOALLOC_WORK_BYTES) {
    fprintf(stderr,
            "staf_op_alpha_dist_grad_noalloc_f64: nt = %d, nalpha_r = %d need a work area of %zu bytes, the built-in "
            "one holds %zu (nt * nalpha_r <= %zu); use staf_op_alpha_dist_grad_f64\n",
            nt, Ar, need, NOALLOC_WORK_BYTES,
            NOALLOC_WORK_BYTES / (sizeof(double) * 2 * ((size_t)GRAD_MAX_BLOCKS + RED_SLICES)));
    return STAF_E_LIMIT;
  }
  if (ld <= 0) ld = Nl;
  double* work = (double*)noalloc_work();
  if (!work) return STAF_E_HIP;
  return alpha_dist_grad_launch<double>(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt, ld,
                                        work, false, stream);
}

// unit != null (the MD entry): the fused kernel, which rebuilds the angular descriptor from the slots' unit vectors
// instead of reading Tang (may be null then).
template <typename real>
int angular_afs(const real* Dsup, const real* Tang, const real* unit, int nr, int na, real* out, int nf, int Nl,
                const int* im3, const int* im2, const real* alpha3b, int Aa, const real* emb3b, const int* type_map,
                const int* numtriplet, int nt, int ld, void* stream_) {
  (void)im3;
  if (Nl == 0 && nf > 0 && Aa > 0) return STAF_OK;   // a species without atoms in these frames: nothing to write
  if (!Dsup || (!Tang && !unit) || !out || !im2 || !alpha3b || !emb3b || !type_map || !numtriplet || nr <= 0 ||
      na <= 0 || Aa <= 0 || nf <= 0 || Nl <= 0 || nt <= 0)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  size_t lds = unit ? TriLds<real, 0, true>::bytes(nr, Aa, nt, true) : TriLds<real, 0>::bytes(nr, Aa, nt, false);
  if (!(unit ? lds_request(tri_reduce_kernel<real, 0, true>, lds) : lds_request(tri_reduce_kernel<real, 0>, lds)))
    return STAF_E_LIMIT;
  TriArgs<real> A = {};
  A.Dsup = Dsup; A.Tang = Tang; A.unit = unit; A.im2 = im2; A.alpha3b = alpha3b; A.emb3b = emb3b;
  A.type_map = type_map; A.numtriplet = numtriplet; A.out = out;
  A.nf = nf; A.Nl = Nl; A.ld = ld; A.nr = nr; A.na = na; A.Aa = Aa; A.nt = nt;
  {
    KernelTimer kt_("af3_kernel", (hipStream_t)stream_);
    // as many workgroups as the device holds at once (or a whole number of such rounds), each taking several centres
    if (unit)
      hipLaunchKernelGGL((tri_reduce_kernel<real, 0, true>),
                         dim3(tri_grid((const void*)tri_reduce_kernel<real, 0, true>, lds, nf * Nl)), dim3(TRI_BLOCK), lds,
                         (hipStream_t)stream_, A);
    else
      hipLaunchKernelGGL((tri_reduce_kernel<real, 0>),
                         dim3(tri_grid((const void*)tri_reduce_kernel<real, 0>, lds, nf * Nl)), dim3(TRI_BLOCK), lds,
                         (hipStream_t)stream_, A);
  }
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}
template int angular_afs<double>(const double*, const double*, const double*, int, int, double*, int, int, const int*,
                                 const int*, const double*, int, const double*, const int*, const int*, int, int,
                                 void*);

template <typename real>
static int alphagrad_ang(const real* Dsup, const real* Tang, int nr, int na, const real* P, int nf, int Nl,
                         const int* im3, const int* im2, const real* alpha3b, int Aa, real* g_alpha,
                         const real* emb3b, const int* type_map, real* g_emb, const int* numtriplet, int ntc, int nt,
                         int ld, void* stream_) {
  (void)im3;
  if (Nl == 0 && nf > 0 && Aa > 0 && nt > 0 && ntc >= 2 * nt - 1 && g_alpha && g_emb) {
    // a species without atoms in these frames: its sums are empty
    launch_fill_zero<real>(g_alpha, ntc * Aa * 3, (hipStream_t)stream_);
    launch_fill_zero<real>(g_emb, ntc * Aa, (hipStream_t)stream_);
    return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  }
  if (!Dsup || !Tang || !P || !im2 || !alpha3b || !g_alpha || !g_emb || !emb3b || !type_map || !numtriplet ||
      nr <= 0 || na <= 0 || Aa <= 0 || nf <= 0 || Nl <= 0 || nt <= 0 || ntc < 2 * nt - 1)
    return STAF_E_BAD_ARG;
  if (nt > NT_MAX) return STAF_E_LIMIT;
  if (ld <= 0) ld = Nl;
  DeviceState* st = device_state((hipStream_t)stream_);
  if (!st) return reserve_failure((hipStream_t)stream_);
  hipStream_t stream = (hipStream_t)stream_;
  const int nsig = 2 * nt - 1;
  const int nout = nsig * Aa * 3;
  const int nb_max = nf * Nl < TRI_GRID_MAX ? nf * Nl : TRI_GRID_MAX;   // the work area does not depend on occupancy
  real* partial = (real*)scratch_reserve(st, stream, ((size_t)nb_max + RED_SLICES) * nout * sizeof(real));
  real* red_tmp = partial ? partial + (size_t)nb_max * nout : nullptr;
  if (!partial) return reserve_failure(stream);
  size_t lds = TriLds<real, 1>::bytes(nr, Aa, nt);
  if (!lds_request(tri_reduce_kernel<real, 1>, lds)) return STAF_E_LIMIT;
  const int nb = tri_grid((const void*)tri_reduce_kernel<real, 1>, lds, nf * Nl);
  // rows sigma >= nsig of the outputs receive no contribution
  const int nall = ntc * Aa * 3;
  TriArgs<real> A = {};
  A.Dsup = Dsup; A.Tang = Tang; A.im2 = im2; A.alpha3b = alpha3b; A.emb3b = emb3b; A.type_map = type_map;
  A.numtriplet = numtriplet; A.P = P; A.partial = partial;
  A.nf = nf; A.Nl = Nl; A.ld = ld; A.nr = nr; A.na = na; A.Aa = Aa; A.nt = nt;
  {
    KernelTimer kt_("grad3_kernel", stream);
    hipLaunchKernelGGL((tri_reduce_kernel<real, 1>), dim3(nb), dim3(TRI_BLOCK), lds, stream, A);
  }
  // parameter rows sigma >= nsig and the embedding gradient (identically zero in the reference) are zero-filled here
  launch_reduce_partials<real>(partial, nb, nout, g_alpha, nout, nall, g_emb, 0, ntc * Aa, red_tmp, stream);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

}  // namespace staf

extern "C" {

int staf_op_radial_afs_f32(const float* D, int nr, const float* alpha2b, int Ar, float* out, int nf, int Nl,
                           const int* im2, const float* emb2b, const int* type_map, int nt, int ld, void* stream) {
  return staf::radial_afs<float>(D, nr, alpha2b, Ar, out, nf, Nl, im2, emb2b, type_map, nt, ld, stream);
}
int staf_op_radial_afs_f64(const double* D, int nr, const double* alpha2b, int Ar, double* out, int nf, int Nl,
                           const int* im2, const double* emb2b, const int* type_map, int nt, int ld, void* stream) {
  return staf::radial_afs<double>(D, nr, alpha2b, Ar, out, nf, Nl, im2, emb2b, type_map, nt, ld, stream);
}
int staf_op_angular_afs_f32(const float* Dsup, const float* Tang, int nr, int na, float* out, int nf, int Nl,
                            const int* im3, const int* im2, const float* alpha3b, int Aa, const float* emb3b,
                            const int* type_map, const int* numtriplet, int nt, int ld, void* stream) {
  return staf::angular_afs<float>(Dsup, Tang, (const float*)nullptr, nr, na, out, nf, Nl, im3, im2, alpha3b, Aa, emb3b,
                                  type_map, numtriplet, nt, ld, stream);
}
int staf_op_angular_afs_f64(const double* Dsup, const double* Tang, int nr, int na, double* out, int nf, int Nl,
                            const int* im3, const int* im2, const double* alpha3b, int Aa, const double* emb3b,
                            const int* type_map, const int* numtriplet, int nt, int ld, void* stream) {
  return staf::angular_afs<double>(Dsup, Tang, (const double*)nullptr, nr, na, out, nf, Nl, im3, im2, alpha3b, Aa,
                                   emb3b, type_map, numtriplet, nt, ld, stream);
}
int staf_op_alpha_dist_grad_f32(const float* D, int nr, const float* alpha2b, int Ar, float* g_alpha, int nf, int Nl,
                                const int* im2, const float* P, const float* emb2b, const int* type_map,
                                float* g_emb, int nt, int ld, void* stream) {
  return staf::alpha_dist_grad<float>(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt, ld,
                                      stream);
}
int staf_op_alpha_dist_grad_f64(const double* D, int nr, const double* alpha2b, int Ar, double* g_alpha, int nf,
                                int Nl, const int* im2, const double* P, const double* emb2b, const int* type_map,
                                double* g_emb, int nt, int ld, void* stream) {
  return staf::alpha_dist_grad<double>(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt, ld,
                                       stream);
}
int staf_op_alpha_dist_grad_noalloc_f64(const double* D, int nr, const double* alpha2b, int Ar, double* g_alpha,
                                        int nf, int Nl, const int* im2, const double* P, const double* emb2b,
                                        const int* type_map, double* g_emb, int nt, int ld, void* stream) {
  return staf::alpha_dist_grad_noalloc(D, nr, alpha2b, Ar, g_alpha, nf, Nl, im2, P, emb2b, type_map, g_emb, nt, ld,
                                       stream);
}
int staf_op_alphagrad_ang_f32(const float* Dsup, const float* Tang, int nr, int na, const float* P, int nf, int Nl,
                              const int* im3, const int* im2, const float* alpha3b, int Aa, float* g_alpha,
                              const float* emb3b, const int* type_map, float* g_emb, const int* numtriplet, int ntc,
                              int nt, int ld, void* stream) {
  return staf::alphagrad_ang<float>(Dsup, Tang, nr, na, P, nf, Nl, im3, im2, alpha3b, Aa, g_alpha, emb3b, type_map,
                                    g_emb, numtriplet, ntc, nt, ld, stream);
}
int staf_op_alphagrad_ang_f64(const double* Dsup, const double* Tang, int nr, int na, const double* P, int nf, int Nl,
                              const int* im3, const int* im2, const double* alpha3b, int Aa, double* g_alpha,
                              const double* emb3b, const int* type_map, double* g_emb, const int* numtriplet, int ntc,
                              int nt, int ld, void* stream) {
  return staf::alphagrad_ang<double>(Dsup, Tang, nr, na, P, nf, Nl, im3, im2, alpha3b, Aa, g_alpha, emb3b, type_map,
                                     g_emb, numtriplet, ntc, nt, ld, stream);
}

}  // extern "C"
