// Device-resident evaluation of the per-species MLP of the MD entry: x = log(af + 1e-3) - mu, Dense stack
// (tanh / relu / linear), atomic energy, and dE/d af by back-propagation -- the step between the fingerprint and
// the force kernels that the reference does on the host or through ONNX Runtime
// (Compute_NNEnergyandGradient_all, libstaf/vendor/jmd/nn_nn_mlp.cu:657-768; native evaluation
// libstaf/src/mlp/staf_mlp_ort.cc:186-233).  The network is tiny (60 -> 140 -> 140 -> 1 in the reference's models):
// one workgroup evaluates TA (2 or 4) atoms; a matrix-vector product is spread over the workgroup as (output neuron,
// slice of the inner dimension), so that all weight reads of a layer are in flight together (coalesced; a
// transposed copy serves the backward pass); each weight read serves the TA atoms of the workgroup.
#include "staf_mlp_dev.hpp"

#include <stdlib.h>
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
    const int KS = matvec_slices<T, MLP_TA>(A.Wt[l], out_f, in_f, dl, A.maxw, part);
    __syncthreads();
    for (int q = tid; q < MLP_TA * in_f; q += MLP_BLOCK) {
      const int t = q / in_f, i = q - t * in_f;
      T g = 0;
      for (int ks = 0; ks < KS; ks++) g += part[((size_t)ks * MLP_TA + t) * in_f + i];
      dl[t * A.maxw + i] = g;
    }
    __syncthreads();
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
}

// ---------------------------------------------------------------------------------------------------------------
// Matrix-core form of the same evaluation.  The Dense layers are small dense matrix products ([atoms, in] x
// [in, out]), the one place on this path where the matrix cores fit: a workgroup takes 16 atoms (the rows of a
// 16x16x4 MFMA tile), so the weight matrices stream through a CU once per 16 atoms instead of once per 2-4, which is
// what bounds the vector kernel above.  Activations live in LDS as X[feature][16 atoms]; a unit of work is (tile of
// 16 output columns, slice of the inner dimension) with up to MM_STEPS weight reads in flight per lane; units are
// dealt round-robin to the 16 waves; slice sums meet in LDS and are added in ascending slice order (fixed order).
constexpr int MM_TA = 16;
// Pitch of a column of slice sums in LDS: the lanes of a tile write the same atom row of 16 consecutive columns at
// once, and 16 atoms (128 bytes in double precision) between them would put all of them on the same banks.
constexpr int MM_TP = MM_TA + 1;
constexpr int MM_BLOCK = 1024;
constexpr int MM_WAVES = MM_BLOCK / WAVE;
constexpr int MM_STEPS = 12;      // MFMA steps (4 rows of the inner dimension each) per batch of weight reads
constexpr int MM_SLICES = 4;      // at most this many slices of the inner dimension

template <typename T> struct MfmaOp;
template <> struct MfmaOp<double> {
  typedef double acc_t __attribute__((ext_vector_type(4)));
  __device__ static acc_t run(double a, double b, acc_t c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  __device__ static int acc_row(int lane, int v) { return lane / 16 + 4 * v; }
};
template <> struct MfmaOp<float> {
  typedef float acc_t __attribute__((ext_vector_type(4)));
  __device__ static acc_t run(float a, float b, acc_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  __device__ static int acc_row(int lane, int v) { return 4 * (lane / 16) + v; }
};
// operand layout of the 16x16x4 tiles: A[row = lane % 16][k = lane / 16], B[k = lane / 16][col = lane % 16];
// accumulator element v of a lane: col = lane % 16, row = acc_row(lane, v) (the two precisions differ)

__host__ __device__ inline int mm_slices(int K) {
  const int nstep = (K + 3) / 4;
  const int s = (nstep + MM_STEPS - 1) / MM_STEPS;
  return s < 1 ? 1 : (s > MM_SLICES ? MM_SLICES : s);
}

// part[slice][j][atom] = sum over the slice's rows k of X[k][atom] * M[k][j];  M [K, J] row-major in global memory,
// X [K][MM_TA] in LDS.  Returns the number of slices.
template <typename T>
__device__ inline int mm_products(const T* __restrict__ M, int K, int J, const T* X, T* part) {
  typedef typename MfmaOp<T>::acc_t acc_t;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int ntile = (J + 15) / 16;
  const int nstep = (K + 3) / 4;
  const int nsl = mm_slices(K);
  const int per = (nstep + nsl - 1) / nsl;
  const int kq = lane / 16, c16 = lane % 16;
  for (int u = wave; u < ntile * nsl; u += MM_WAVES) {
    const int tile = u % ntile, sl = u / ntile;
    const int s0 = sl * per;
    const int s1 = (s0 + per) < nstep ? (s0 + per) : nstep;
    const int col = tile * 16 + c16;
    const int colc = col < J ? col : J - 1;
    acc_t acc = {0, 0, 0, 0};
    for (int sb = s0; sb < s1; sb += MM_STEPS) {
      T b[MM_STEPS], a[MM_STEPS];
      // rows beyond the slice or the matrix are read at the last row (inside the matrix) and enter as zeros
#pragma unroll
      for (int q = 0; q < MM_STEPS; q++) {
        const int k = 4 * (sb + q) + kq;
        const int kc = k < K ? k : K - 1;
        b[q] = M[(size_t)kc * J + colc];
      }
#pragma unroll
      for (int q = 0; q < MM_STEPS; q++) {
        const int k = 4 * (sb + q) + kq;
        const int kc = k < K ? k : K - 1;
        a[q] = X[kc * MM_TA + c16];
      }
#pragma unroll
      for (int q = 0; q < MM_STEPS; q++) {
        const int k = 4 * (sb + q) + kq;
        const bool in = (sb + q) < s1 && k < K;
        acc = MfmaOp<T>::run(in ? a[q] : T(0), (in && col < J) ? b[q] : T(0), acc);
      }
    }
    if (col < J) {
#pragma unroll
      for (int v = 0; v < 4; v++) part[((size_t)sl * J + col) * MM_TP + MfmaOp<T>::acc_row(lane, v)] = acc[v];
    }
  }
  return nsl;
}

template <typename T>
__global__ __launch_bounds__(MM_BLOCK) void mlp_matrix_kernel(MlpArgs<T> A) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* X = (T*)smem;                            // [tot][MM_TA]: input and every layer's output
  T* dl = X + (size_t)A.tot * MM_TA;          // [maxw][MM_TA]: back-propagated deltas
  T* part = dl + (size_t)A.maxw * MM_TA;      // [slices][width][MM_TP]
  const int tid = threadIdx.x;
  const int a0 = blockIdx.x * MM_TA;
  const int n_af = A.n_af;
  for (int q = tid; q < MM_TA * n_af; q += MM_BLOCK) {
    const int t = q / n_af, i = q - t * n_af;
    const int atom = a0 + t;
    T v = 0;
    if (atom < A.Nl) {
      const T afv = (T)(i < A.Ar ? A.af2[(size_t)atom * A.Ar + i] : A.af3[(size_t)atom * A.Aa + (i - A.Ar)]);
      v = m_log(afv + T(1e-3)) - A.mu[i];
    }
    X[i * MM_TA + t] = v;
  }
  __syncthreads();
  // ---- forward
  int off_in = 0;
  for (int l = 0; l < A.nl; l++) {
    const int in_f = A.in_f[l], out_f = A.out_f[l];
    const int off_out = off_in + in_f;
    const int nsl = mm_products<T>(A.W[l], in_f, out_f, X + (size_t)off_in * MM_TA, part);
    __syncthreads();
    for (int q = tid; q < out_f * MM_TA; q += MM_BLOCK) {
      const int j = q / MM_TA, t = q - j * MM_TA;
      T y = A.b[l][j];
      for (int sl = 0; sl < nsl; sl++) y += part[((size_t)sl * out_f + j) * MM_TP + t];
      if (A.act[l] == 1) y = m_tanh(y);
      else if (A.act[l] == 2) y = y > T(0) ? y : T(0);
      X[(size_t)off_out * MM_TA + q] = y;
    }
    __syncthreads();
    off_in = off_out;
  }
  // off_in is now the offset of the last layer's output (one value per atom)
  if (tid < MM_TA && a0 + tid < A.Nl) A.e_atom[a0 + tid] = (double)X[(size_t)off_in * MM_TA + tid];
  // ---- backward: delta of the summed atomic energy
  for (int q = tid; q < MM_TA; q += MM_BLOCK) dl[q] = T(1);
  __syncthreads();
  int off_out = off_in;
  for (int l = A.nl - 1; l >= 0; l--) {
    const int in_f = A.in_f[l], out_f = A.out_f[l];
    const int off_i = off_out - in_f;
    // delta times the activation derivative, in place
    for (int q = tid; q < out_f * MM_TA; q += MM_BLOCK) {
      const T y = X[(size_t)off_out * MM_TA + q];
      T g = dl[q];
      if (A.act[l] == 1) g *= (T(1) - y * y);
      else if (A.act[l] == 2 && y <= T(0)) g = T(0);
      dl[q] = g;
    }
    __syncthreads();
    // delta of the layer's input: Wt [out, in] is the matrix, the deltas [out][atoms] the vectors
    const int nsl = mm_products<T>(A.Wt[l], out_f, in_f, dl, part);
    __syncthreads();
    for (int q = tid; q < in_f * MM_TA; q += MM_BLOCK) {
      T g = 0;
      const int j = q / MM_TA, t = q - j * MM_TA;
      for (int sl = 0; sl < nsl; sl++) g += part[((size_t)sl * in_f + j) * MM_TP + t];
      dl[q] = g;
    }
    __syncthreads();
    off_out = off_i;
  }
  // ---- d sum(atomic) / d af = delta / (af + 1e-3)
  for (int q = tid; q < MM_TA * n_af; q += MM_BLOCK) {
    const int t = q / n_af, i = q - t * n_af;
    const int atom = a0 + t;
    if (atom >= A.Nl) continue;
    const bool two = i < A.Ar;
    const T afv = (T)(two ? A.af2[(size_t)atom * A.Ar + i] : A.af3[(size_t)atom * A.Aa + (i - A.Ar)]);
    const double g = (double)(dl[i * MM_TA + t] / (afv + T(1e-3)));
    if (two) A.g2[(size_t)atom * A.Ar + i] = g;
    else A.g3[(size_t)atom * A.Aa + (i - A.Ar)] = g;
  }
}

// LDS of a workgroup of the matrix kernel: activations, deltas, slice sums of the widest product
template <typename T>
static size_t mm_lds_bytes(const DevMlpNet& net) {
  size_t npart = 0;
  for (int l = 0; l < net.nl; l++) {
    const size_t f = (size_t)mm_slices(net.in_f[l]) * net.out_f[l];
    const size_t b = (size_t)mm_slices(net.out_f[l]) * net.in_f[l];
    npart = f > npart ? f : npart;
    npart = b > npart ? b : npart;
  }
  return (((size_t)net.tot + net.maxw) * MM_TA + npart * MM_TP) * sizeof(T);
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
static bool upload_net(const StafMlp* mlp, int type, DevMlpNet* net, hipStream_t stream) {
  const int nl = staf_mlp_internal_nlayers(mlp, type);
  if (nl <= 0 || nl > DEV_MLP_MAX_LAYERS) return false;
  net->nl = nl;
  net->n_af = staf_mlp_n_af(mlp, type);
  net->tot = net->n_af;
  net->maxw = net->n_af;
  // every parameter of the stack in one block (one upload, neighbouring pages): [mu | per layer W, Wt, b], each part
  // on a 256-byte boundary
  std::vector<T> host;
  auto place = [&](const T* src, size_t n) {
    const size_t at = (host.size() + 31) & ~(size_t)31;
    host.resize(at + n, T(0));
    for (size_t i = 0; i < n; i++) host[at + i] = src[i];
    return at;
  };
  const size_t at_mu = place((const T*)staf_mlp_internal_mu(mlp, type), net->n_af);
  size_t at_W[DEV_MLP_MAX_LAYERS], at_Wt[DEV_MLP_MAX_LAYERS], at_b[DEV_MLP_MAX_LAYERS];
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
    at_W[l] = place(w, (size_t)in_f * out_f);
    at_Wt[l] = place(wt.data(), (size_t)in_f * out_f);
    at_b[l] = place((const T*)b, out_f);
  }
  T* block = nullptr;
  if (hipMalloc((void**)&block, host.size() * sizeof(T)) != hipSuccess) return false;
  net->mu = block;   // the block's address: freed through it
  // on the model's stream, not the legacy default stream (another host thread may be recording a graph)
  if (hipMemcpyAsync(block, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice, stream) != hipSuccess ||
      hipStreamSynchronize(stream) != hipSuccess)
    return false;
  (void)at_mu;       // 0: mu leads the block
  for (int l = 0; l < nl; l++) {
    net->W[l] = block + at_W[l];
    net->Wt[l] = block + at_Wt[l];
    net->b[l] = block + at_b[l];
  }
  if (net->out_f[nl - 1] != 1 || net->in_f[0] != net->n_af) return false;
  // The matrix kernel needs more LDS than the 64 KB a kernel gets by default (160 KB per CU exist): ask once.
  // (the attribute is per kernel, not per launch: it is set to the largest request seen, on the device in use)
  static size_t largest = 0;
  const size_t mm = mm_lds_bytes<T>(*net);
  if (mm <= 64 * 1024) {
    net->matrix_path = true;
  } else if (mm <= 152 * 1024) {
    const size_t want = mm > largest ? mm : largest;
    if (hipFuncSetAttribute((const void*)mlp_matrix_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)want) == hipSuccess) {
      largest = want;
      net->matrix_path = true;
    }
  }
  (void)hipGetLastError();
  // a stack too wide for either kernel's LDS is left to the host evaluation
  return net->matrix_path || mlp_lds_bytes<T>(*net, MLP_TA_MAX) <= 64 * 1024;
}

bool dev_mlp_upload(const StafMlp* mlp, int type, DevMlpNet* net, hipStream_t stream) {
  *net = DevMlpNet();
  net->precision = staf_mlp_precision(mlp);
  return net->precision ? upload_net<double>(mlp, type, net, stream) : upload_net<float>(mlp, type, net, stream);
}

void dev_mlp_free(DevMlpNet* net) {
  if (net->mu) (void)hipFree(net->mu);   // one block holds mu and every layer
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
  // Which kernel: one workgroup of either takes 25-35 us for the reference's 60-140-140-1 stack whatever its atom
  // count (the weight matrices stream through its CU layer by layer), so the vector kernel (2-4 atoms a workgroup)
  // serves up to ~1000 atoms in one round of workgroups and the matrix kernel (16 atoms) sixteen times as many; in
  // single precision the matrix kernel is the faster one throughout.  STAF_MLP_VECTOR / STAF_MLP_MATRIX in the
  // environment force one of them (tests).
  const bool prefer_matrix = sizeof(T) == 4 || Nl > 1024 || getenv("STAF_MLP_MATRIX");
  if (net.matrix_path && prefer_matrix && !getenv("STAF_MLP_VECTOR")) {
    hipLaunchKernelGGL((mlp_matrix_kernel<T>), dim3((Nl + MM_TA - 1) / MM_TA), dim3(MM_BLOCK), mm_lds_bytes<T>(net),
                       stream, A);
    return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
  }
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
