// Device-resident evaluation of the per-species MLP of the MD entry: x = log(af + 1e-3) - mu, Dense stack
// (tanh / relu / linear), atomic energy, and dE/d af by back-propagation -- the step between the fingerprint and
// the force kernels that the reference does on the host or through ONNX Runtime
// (Compute_NNEnergyandGradient_all, libstaf/vendor/jmd/nn_nn_mlp.cu:657-768; native evaluation
// libstaf/src/mlp/staf_mlp_ort.cc:186-233).  The network is tiny (60 -> 140 -> 140 -> 1 in the reference's models):
// one workgroup evaluates TA (2 or 4) atoms; a matrix-vector product is spread over the workgroup as (output neuron,
// slice of the inner dimension), so that all weight reads of a layer are in flight together (coalesced; a
// transposed copy serves the backward pass); each weight read serves the TA atoms of the workgroup.
#include "staf_mlp_dev.hpp"

#include <vector>

namespace staf {

// Atoms per workgroup (template parameter TA of the kernel).  Every product reads one activation from LDS (a
// wave-wide broadcast), which is what a workgroup's time goes into; a weight read serves TA atoms.  Small systems
// take 2 atoms per workgroup (short critical path, the workgroups still fit the GPU at once), large ones 4 (half
// the weight traffic per atom).
constexpr int MLP_TA_MAX = 4;
constexpr int MLP_BLOCK = 1024;
static_assert(MLP_TA_MAX <= MLP_BLOCK / WAVE, "the output neuron is summed by one wave per atom");

template <typename T>
struct MlpArgs {
  int nl, n_af, tot, maxw, Ar, Aa, Nl;
  int act[DEV_MLP_MAX_LAYERS], in_f[DEV_MLP_MAX_LAYERS], out_f[DEV_MLP_MAX_LAYERS];
  const T* W[DEV_MLP_MAX_LAYERS];    // [in, out]
  const T* Wt[DEV_MLP_MAX_LAYERS];   // [out, in]
  const T* b[DEV_MLP_MAX_LAYERS];
  const T* mu;
  const double* af2;   // [Nl, Ar]
  const double* af3;   // [Nl, Aa]
  double* e_atom;      // [Nl]
  double* g2;          // [Nl, Ar]
  double* g3;          // [Nl, Aa]
};

__device__ inline float m_log(float x) { return logf(x); }
__device__ inline double m_log(double x) { return log(x); }
__device__ inline float m_tanh(float x) { return tanhf(x); }
__device__ inline double m_tanh(double x) { return tanh(x); }

// value of v in lane `src` (a compile-time constant after unrolling), as a wave-uniform scalar
__device__ inline float lane_value(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ inline double lane_value(double v, int src) {
  const long long b = __double_as_longlong(v);
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(b & 0xffffffffll), src);
  const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(b >> 32), src);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// y[t][j] (+)= sum_k x[t][k] M[k][j] for the MLP_TA atoms of the workgroup, M [K, J] row-major in global memory.
// The K range is cut into slices: thread <-> (column j, slice), every thread keeps sixteen weight reads in flight,
// slice sums go to part[slice][t][j] in LDS and are added by the caller in ascending slice order (fixed order:
// bit-reproducible).  Returns the number of slices.
template <typename T, int MLP_TA>
__device__ inline int matvec_slices(const T* __restrict__ M, int K, int J, const T* x, int xs, T* part) {
  const int JP = (J + WAVE - 1) & ~(WAVE - 1);        // a wave holds one slice
  const int KS = JP <= MLP_BLOCK ? MLP_BLOCK / JP : 1;
  const int KC = (K + KS - 1) / KS;
  for (int idx = threadIdx.x; idx < KS * JP; idx += MLP_BLOCK) {
    const int ks = idx / JP, j = idx - ks * JP;
    // lanes beyond the last column stay in step with their wave (they hold activations the others read) on the
    // last column, and store nothing
    const bool live = j < J;
    const int jc = live ? j : J - 1;
    const int k0 = ks * KC;
    const int k1 = (k0 + KC) < K ? (k0 + KC) : K;
    T acc[MLP_TA];
#pragma unroll
    for (int t = 0; t < MLP_TA; t++) acc[t] = 0;
    // Sixteen rows at a time.  The weight reads are all issued before the first is used: rows beyond the slice are
    // read at its last row (always inside the matrix) and enter with weight zero, so the reads carry no condition.
    // The activations of the sixteen rows are the same for every lane of the wave (a wave holds one slice): lane u
    // reads row u's value once, and the products take it from that lane (a register read instead of sixteen LDS
    // broadcasts, which is what the workgroup's time went into).
    const int lane = threadIdx.x & (WAVE - 1);
    for (int kb = k0; kb < k1; kb += 16) {
      T w[16];
#pragma unroll
      for (int u = 0; u < 16; u++) {
        const int k = (kb + u) < k1 ? (kb + u) : (k1 - 1);
        w[u] = M[(size_t)k * J + jc];
      }
      T xl[MLP_TA];
      {
        const int k = (kb + (lane & 15)) < k1 ? (kb + (lane & 15)) : (k1 - 1);
#pragma unroll
        for (int t = 0; t < MLP_TA; t++) xl[t] = x[t * xs + k];
      }
#pragma unroll
      for (int u = 0; u < 16; u++) {
        const T wu = (kb + u) < k1 ? w[u] : T(0);
#pragma unroll
        for (int t = 0; t < MLP_TA; t++) acc[t] += lane_value(xl[t], u) * wu;
      }
    }
    if (live) {
#pragma unroll
      for (int t = 0; t < MLP_TA; t++) part[((size_t)ks * MLP_TA + t) * J + j] = acc[t];
    }
  }
  return KS;
}

template <typename T, int MLP_TA>
__global__ __launch_bounds__(MLP_BLOCK) void mlp_kernel(MlpArgs<T> A) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* buf = (T*)smem;                       // [MLP_TA][tot]: input and every layer's output
  T* dl = buf + MLP_TA * A.tot;            // [MLP_TA][maxw]: back-propagated deltas
  T* part = dl + MLP_TA * A.maxw;          // [slices][MLP_TA][width]: slice sums of the current product
  const int tid = threadIdx.x;
  const int a0 = blockIdx.x * MLP_TA;
  const int n_af = A.n_af;
  PHASE_CLOCK_BEGIN();
  for (int q = tid; q < MLP_TA * n_af; q += MLP_BLOCK) {
    const int t = q / n_af, i = q - t * n_af;
    const int atom = a0 + t;
    T v = 0;
    if (atom < A.Nl) {
      const T afv = (T)(i < A.Ar ? A.af2[(size_t)atom * A.Ar + i] : A.af3[(size_t)atom * A.Aa + (i - A.Ar)]);
      v = m_log(afv + T(1e-3)) - A.mu[i];
    }
    buf[t * A.tot + i] = v;
  }
  __syncthreads();
  PHASE_MARK(0);
  // ---- forward
  int off_in = 0;
  for (int l = 0; l < A.nl; l++) {
    const int in_f = A.in_f[l], out_f = A.out_f[l];
    const int off_out = off_in + in_f;
    if (out_f == 1) {
      // the output neuron of the stack: wave t sums atom t's products over the lanes (fixed order)
      const int t = tid / WAVE, lane = tid & (WAVE - 1);
      if (t < MLP_TA) {
        T p = 0;
        for (int i = lane; i < in_f; i += WAVE) p += buf[t * A.tot + off_in + i] * A.W[l][i];
        p = wave_sum(p);
        if (lane == 0) {
          T y = p + A.b[l][0];
          if (A.act[l] == 1) y = m_tanh(y);
          else if (A.act[l] == 2) y = y > T(0) ? y : T(0);
          buf[t * A.tot + off_out] = y;
        }
      }
    } else {
      const int KS = matvec_slices<T, MLP_TA>(A.W[l], in_f, out_f, buf + off_in, A.tot, part);
      __syncthreads();
      PHASE_MARK(1);
      for (int q = tid; q < MLP_TA * out_f; q += MLP_BLOCK) {
        const int t = q / out_f, j = q - t * out_f;
        T y = A.b[l][j];
        for (int ks = 0; ks < KS; ks++) y += part[((size_t)ks * MLP_TA + t) * out_f + j];
        if (A.act[l] == 1) y = m_tanh(y);
        else if (A.act[l] == 2) y = y > T(0) ? y : T(0);
        buf[t * A.tot + off_out + j] = y;
      }
    }
    __syncthreads();
    PHASE_MARK(2);
    off_in = off_out;
  }
  // off_in is now the offset of the last layer's output (one value per atom)
  if (tid < MLP_TA && a0 + tid < A.Nl) A.e_atom[a0 + tid] = (double)buf[tid * A.tot + off_in];
  // ---- backward: delta of the summed atomic energy
  for (int q = tid; q < MLP_TA; q += MLP_BLOCK) dl[q * A.maxw] = T(1);
  __syncthreads();
  int off_out = off_in;
  for (int l = A.nl - 1; l >= 0; l--) {
    const int in_f = A.in_f[l], out_f = A.out_f[l];
    const int off_i = off_out - in_f;
    // delta times the activation derivative, in place
    for (int q = tid; q < MLP_TA * out_f; q += MLP_BLOCK) {
      const int t = q / out_f, j = q - t * out_f;
      const T y = buf[t * A.tot + off_out + j];
      T g = dl[t * A.maxw + j];
      if (A.act[l] == 1) g *= (T(1) - y * y);
      else if (A.act[l] == 2 && y <= T(0)) g = T(0);
      dl[t * A.maxw + j] = g;
    }
    __syncthreads();
    // delta of the layer's input: Wt [out, in] is the matrix, the delta the vector
    PHASE_MARK(3);
    const int KS = matvec_slices<T, MLP_TA>(A.Wt[l], out_f, in_f, dl, A.maxw, part);
    __syncthreads();
    PHASE_MARK(4);
    for (int q = tid; q < MLP_TA * in_f; q += MLP_BLOCK) {
      const int t = q / in_f, i = q - t * in_f;
      T g = 0;
      for (int ks = 0; ks < KS; ks++) g += part[((size_t)ks * MLP_TA + t) * in_f + i];
      dl[t * A.maxw + i] = g;
    }
    __syncthreads();
    PHASE_MARK(5);
    off_out = off_i;
  }
  // ---- d sum(atomic) / d af = delta / (af + 1e-3)
  for (int q = tid; q < MLP_TA * n_af; q += MLP_BLOCK) {
    const int t = q / n_af, i = q - t * n_af;
    const int atom = a0 + t;
    if (atom >= A.Nl) continue;
    const bool two = i < A.Ar;
    const T afv = (T)(two ? A.af2[(size_t)atom * A.Ar + i] : A.af3[(size_t)atom * A.Aa + (i - A.Ar)]);
    const double g = (double)(dl[t * A.maxw + i] / (afv + T(1e-3)));
    if (two) A.g2[(size_t)atom * A.Ar + i] = g;
    else A.g3[(size_t)atom * A.Aa + (i - A.Ar)] = g;
  }
  PHASE_MARK(6);
  PHASE_CLOCK_END();
}

// LDS of one workgroup of ta atoms: activations, deltas, and slice sums (slices * ta * width <= ta * max(MLP_BLOCK,
// rounded width))
template <typename T>
static size_t mlp_lds_bytes(const DevMlpNet& net, int ta) {
  const int wpad = (net.maxw + WAVE - 1) & ~(WAVE - 1);
  const size_t npart = (size_t)ta * (wpad > MLP_BLOCK ? wpad : MLP_BLOCK);
  return ((size_t)ta * net.tot + (size_t)ta * net.maxw + npart) * sizeof(T);
}

template <typename T>
static bool upload_net(const StafMlp* mlp, int type, DevMlpNet* net) {
  const int nl = staf_mlp_internal_nlayers(mlp, type);
  if (nl <= 0 || nl > DEV_MLP_MAX_LAYERS) return false;
  net->nl = nl;
  net->n_af = staf_mlp_n_af(mlp, type);
  net->tot = net->n_af;
  net->maxw = net->n_af;
  if (hipMalloc(&net->mu, net->n_af * sizeof(T)) != hipSuccess) return false;
  if (hipMemcpy(net->mu, staf_mlp_internal_mu(mlp, type), net->n_af * sizeof(T), hipMemcpyHostToDevice) != hipSuccess)
    return false;
  for (int l = 0; l < nl; l++) {
    const void *W, *b;
    if (staf_mlp_internal_layer(mlp, type, l, &net->act[l], &net->in_f[l], &net->out_f[l], &W, &b) != 0) return false;
    const int in_f = net->in_f[l], out_f = net->out_f[l];
    net->tot += out_f;
    net->maxw = out_f > net->maxw ? out_f : net->maxw;
    std::vector<T> wt((size_t)in_f * out_f);
    const T* w = (const T*)W;
    for (int i = 0; i < in_f; i++)
      for (int j = 0; j < out_f; j++) wt[(size_t)j * in_f + i] = w[(size_t)i * out_f + j];
    const size_t nb = (size_t)in_f * out_f * sizeof(T);
    if (hipMalloc(&net->W[l], nb) != hipSuccess || hipMalloc(&net->Wt[l], nb) != hipSuccess ||
        hipMalloc(&net->b[l], out_f * sizeof(T)) != hipSuccess)
      return false;
    if (hipMemcpy(net->W[l], W, nb, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(net->Wt[l], wt.data(), nb, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(net->b[l], b, out_f * sizeof(T), hipMemcpyHostToDevice) != hipSuccess)
      return false;
  }
  // a stack too wide for the kernel's LDS is left to the host evaluation
  return net->out_f[nl - 1] == 1 && net->in_f[0] == net->n_af && mlp_lds_bytes<T>(*net, MLP_TA_MAX) <= 64 * 1024;
}

bool dev_mlp_upload(const StafMlp* mlp, int type, DevMlpNet* net) {
  *net = DevMlpNet();
  net->precision = staf_mlp_precision(mlp);
  return net->precision ? upload_net<double>(mlp, type, net) : upload_net<float>(mlp, type, net);
}

void dev_mlp_free(DevMlpNet* net) {
  if (net->mu) (void)hipFree(net->mu);
  for (int l = 0; l < DEV_MLP_MAX_LAYERS; l++) {
    if (net->W[l]) (void)hipFree(net->W[l]);
    if (net->Wt[l]) (void)hipFree(net->Wt[l]);
    if (net->b[l]) (void)hipFree(net->b[l]);
  }
  *net = DevMlpNet();
}

template <typename T>
static int eval_net(const DevMlpNet& net, const double* af2, int Ar, const double* af3, int Aa, int Nl, double* e_atom,
                    double* g2, double* g3, hipStream_t stream) {
  MlpArgs<T> A;
  A.nl = net.nl; A.n_af = net.n_af; A.tot = net.tot; A.maxw = net.maxw; A.Ar = Ar; A.Aa = Aa; A.Nl = Nl;
  for (int l = 0; l < net.nl; l++) {
    A.act[l] = net.act[l]; A.in_f[l] = net.in_f[l]; A.out_f[l] = net.out_f[l];
    A.W[l] = (const T*)net.W[l]; A.Wt[l] = (const T*)net.Wt[l]; A.b[l] = (const T*)net.b[l];
  }
  A.mu = (const T*)net.mu;
  A.af2 = af2; A.af3 = af3; A.e_atom = e_atom; A.g2 = g2; A.g3 = g3;
  const int ta = Nl <= 2 * 256 ? 2 : 4;   // up to 256 workgroups (one per CU) take 2 atoms each
  const size_t lds = mlp_lds_bytes<T>(net, ta);
  if (lds > 64 * 1024) return STAF_E_LIMIT;
  if (ta == 2)
    hipLaunchKernelGGL((mlp_kernel<T, 2>), dim3((Nl + 1) / 2), dim3(MLP_BLOCK), lds, stream, A);
  else
    hipLaunchKernelGGL((mlp_kernel<T, 4>), dim3((Nl + 3) / 4), dim3(MLP_BLOCK), lds, stream, A);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

int dev_mlp_eval(const DevMlpNet& net, const double* af2, int Ar, const double* af3, int Aa, int Nl, double* e_atom,
                 double* g2, double* g3, hipStream_t stream) {
  if (Ar + Aa != net.n_af || Nl <= 0) return STAF_E_BAD_ARG;
  return net.precision ? eval_net<double>(net, af2, Ar, af3, Aa, Nl, e_atom, g2, g3, stream)
                       : eval_net<float>(net, af2, Ar, af3, Aa, Nl, e_atom, g2, g3, stream);
}

}  // namespace staf

PHASE_CLOCK_READER(staf_debug_phase_clock_mlp)
