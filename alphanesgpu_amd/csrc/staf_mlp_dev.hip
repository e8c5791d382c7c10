// Device-resident evaluation of the per-species MLP of the MD entry: x = log(af + 1e-3) - mu, Dense stack
// (tanh / relu / linear), atomic energy, and dE/d af by back-propagation -- the step between the fingerprint and
// the force kernels that the reference does on the host or through ONNX Runtime
// (Compute_NNEnergyandGradient_all, libstaf/vendor/jmd/nn_nn_mlp.cu:657-768; native evaluation
// libstaf/src/mlp/staf_mlp_ort.cc:186-233).  The network is tiny (60 -> 140 -> 140 -> 1 in the reference's models):
// one workgroup evaluates MLP_TA atoms, thread <-> output neuron, the weight matrix is read once per workgroup
// (coalesced; a transposed copy serves the backward pass) and reused for its atoms from registers.
#include "staf_mlp_dev.hpp"

#include <vector>

namespace staf {

constexpr int MLP_TA = 4;        // atoms per workgroup
constexpr int MLP_BLOCK = 256;
static_assert(MLP_TA <= MLP_BLOCK / WAVE, "the output neuron is summed by one wave per atom");

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

template <typename T>
__global__ __launch_bounds__(MLP_BLOCK) void mlp_kernel(MlpArgs<T> A) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* buf = (T*)smem;                       // [MLP_TA][tot]: input and every layer's output
  T* dl = buf + MLP_TA * A.tot;            // [2][MLP_TA][maxw]: back-propagated deltas, ping-pong
  const int tid = threadIdx.x;
  const int a0 = blockIdx.x * MLP_TA;
  const int n_af = A.n_af;
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
  // ---- forward
  int off_in = 0;
  for (int l = 0; l < A.nl; l++) {
    const int in_f = A.in_f[l], out_f = A.out_f[l];
    const int off_out = off_in + in_f;
    if (out_f == 1) {
      // the output neuron of the stack: wave t sums atom t's products over the lanes (fixed order)
      const int t = tid / WAVE, lane = tid & (WAVE - 1);
      if (t < MLP_TA) {
        T part = 0;
        for (int i = lane; i < in_f; i += WAVE) part += buf[t * A.tot + off_in + i] * A.W[l][i];
        part = wave_sum(part);
        if (lane == 0) {
          T y = part + A.b[l][0];
          if (A.act[l] == 1) y = m_tanh(y);
          else if (A.act[l] == 2) y = y > T(0) ? y : T(0);
          buf[t * A.tot + off_out] = y;
        }
      }
    } else
    for (int j = tid; j < out_f; j += MLP_BLOCK) {
      T acc[MLP_TA];
      const T bj = A.b[l][j];
#pragma unroll
      for (int t = 0; t < MLP_TA; t++) acc[t] = bj;
      // the weight reads of twenty steps are in flight together (the loop is bound by their latency otherwise)
#pragma unroll 20
      for (int i = 0; i < in_f; i++) {
        const T w = A.W[l][(size_t)i * out_f + j];
#pragma unroll
        for (int t = 0; t < MLP_TA; t++) acc[t] += buf[t * A.tot + off_in + i] * w;
      }
#pragma unroll
      for (int t = 0; t < MLP_TA; t++) {
        T y = acc[t];
        if (A.act[l] == 1) y = m_tanh(y);
        else if (A.act[l] == 2) y = y > T(0) ? y : T(0);
        buf[t * A.tot + off_out + j] = y;
      }
    }
    __syncthreads();
    off_in = off_out;
  }
  // off_in is now the offset of the last layer's output (one value per atom)
  if (tid < MLP_TA && a0 + tid < A.Nl) A.e_atom[a0 + tid] = (double)buf[tid * A.tot + off_in];
  // ---- backward: delta of the summed atomic energy
  int cur = 0;
  for (int q = tid; q < MLP_TA; q += MLP_BLOCK) dl[(cur * MLP_TA + q) * A.maxw] = T(1);
  __syncthreads();
  int off_out = off_in;
  for (int l = A.nl - 1; l >= 0; l--) {
    const int in_f = A.in_f[l], out_f = A.out_f[l];
    const int off_i = off_out - in_f;
    // delta times the activation derivative, in place
    for (int q = tid; q < MLP_TA * out_f; q += MLP_BLOCK) {
      const int t = q / out_f, j = q - t * out_f;
      const T y = buf[t * A.tot + off_out + j];
      T g = dl[(cur * MLP_TA + t) * A.maxw + j];
      if (A.act[l] == 1) g *= (T(1) - y * y);
      else if (A.act[l] == 2 && y <= T(0)) g = T(0);
      dl[(cur * MLP_TA + t) * A.maxw + j] = g;
    }
    __syncthreads();
    for (int i = tid; i < in_f; i += MLP_BLOCK) {
      T acc[MLP_TA];
#pragma unroll
      for (int t = 0; t < MLP_TA; t++) acc[t] = 0;
#pragma unroll 20
      for (int j = 0; j < out_f; j++) {
        const T w = A.Wt[l][(size_t)j * in_f + i];
#pragma unroll
        for (int t = 0; t < MLP_TA; t++) acc[t] += dl[(cur * MLP_TA + t) * A.maxw + j] * w;
      }
#pragma unroll
      for (int t = 0; t < MLP_TA; t++) dl[((1 - cur) * MLP_TA + t) * A.maxw + i] = acc[t];
    }
    __syncthreads();
    cur = 1 - cur;
    off_out = off_i;
  }
  // ---- d sum(atomic) / d af = delta / (af + 1e-3)
  for (int q = tid; q < MLP_TA * n_af; q += MLP_BLOCK) {
    const int t = q / n_af, i = q - t * n_af;
    const int atom = a0 + t;
    if (atom >= A.Nl) continue;
    const bool two = i < A.Ar;
    const T afv = (T)(two ? A.af2[(size_t)atom * A.Ar + i] : A.af3[(size_t)atom * A.Aa + (i - A.Ar)]);
    const double g = (double)(dl[(cur * MLP_TA + t) * A.maxw + i] / (afv + T(1e-3)));
    if (two) A.g2[(size_t)atom * A.Ar + i] = g;
    else A.g3[(size_t)atom * A.Aa + (i - A.Ar)] = g;
  }
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
  return net->out_f[nl - 1] == 1 && net->in_f[0] == net->n_af;
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
  const size_t lds = (size_t)(MLP_TA * net.tot + 2 * MLP_TA * net.maxw) * sizeof(T);
  if (lds > 64 * 1024) return STAF_E_LIMIT;
  hipLaunchKernelGGL(mlp_kernel<T>, dim3((Nl + MLP_TA - 1) / MLP_TA), dim3(MLP_BLOCK), lds, stream, A);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

int dev_mlp_eval(const DevMlpNet& net, const double* af2, int Ar, const double* af3, int Aa, int Nl, double* e_atom,
                 double* g2, double* g3, hipStream_t stream) {
  if (Ar + Aa != net.n_af || Nl <= 0) return STAF_E_BAD_ARG;
  return net.precision ? eval_net<double>(net, af2, Ar, af3, Aa, Nl, e_atom, g2, g3, stream)
                       : eval_net<float>(net, af2, Ar, af3, Aa, Nl, e_atom, g2, g3, stream);
}

}  // namespace staf
