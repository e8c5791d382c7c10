// Per-species MLP plug-in on the host: x = log(af + 1e-3) - mu, Dense stack (tanh / relu / linear), and the
// analytical gradient of the summed atomic energy with respect to the fingerprints.
// Interface and file format of the reference: libstaf/include/staf_mlp.h:19-41, "STAFMLP1" reader and native
// evaluation libstaf/src/mlp/staf_mlp_ort.cc:99-165,186-233 (energy = 0.5 * sum atomic, dE_daf = d sum / d af).
#include "../../include/staf_mlp.h"

#include <math.h>
#include <stdio.h>
#include <string.h>

#include <string>
#include <vector>

namespace {

enum { ACT_LINEAR = 0, ACT_TANH = 1, ACT_RELU = 2 };

template <typename T>
struct Layer {
  int act = 0, in_f = 0, out_f = 0;
  std::vector<T> W;  // [in_f, out_f] row-major
  std::vector<T> b;  // [out_f]
};

template <typename T>
struct Net {
  int n_af = 0;
  std::vector<T> mu;
  std::vector<Layer<T>> layers;
};

template <typename S, typename T>
bool read_vec(FILE* f, size_t n, std::vector<T>& out) {
  std::vector<S> tmp(n);
  if (fread(tmp.data(), sizeof(S), n, f) != n) return false;
  out.assign(tmp.begin(), tmp.end());
  return true;
}

// File: "STAFMLP1", int32 {precision, n_af, n_layers}, mu[n_af], then per layer int32 {act, in, out},
// W[in*out], b[out]; floats or doubles according to `precision`.
template <typename T>
bool load_bin(const std::string& path, Net<T>& net) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return false;
  char magic[8];
  int hdr[3];
  bool ok = fread(magic, 1, 8, f) == 8 && memcmp(magic, "STAFMLP1", 8) == 0 && fread(hdr, sizeof(int), 3, f) == 3;
  if (ok) {
    const bool dbl = hdr[0] == 1;
    net.n_af = hdr[1];
    ok = hdr[1] > 0 && hdr[2] > 0 && hdr[2] < 64 &&
         (dbl ? read_vec<double>(f, net.n_af, net.mu) : read_vec<float>(f, net.n_af, net.mu));
    net.layers.resize(ok ? hdr[2] : 0);
    for (size_t li = 0; ok && li < net.layers.size(); li++) {
      int meta[3];
      ok = fread(meta, sizeof(int), 3, f) == 3 && meta[1] > 0 && meta[2] > 0;
      if (!ok) break;
      Layer<T>& L = net.layers[li];
      L.act = meta[0]; L.in_f = meta[1]; L.out_f = meta[2];
      const size_t nw = (size_t)L.in_f * L.out_f;
      ok = dbl ? (read_vec<double>(f, nw, L.W) && read_vec<double>(f, L.out_f, L.b))
               : (read_vec<float>(f, nw, L.W) && read_vec<float>(f, L.out_f, L.b));
    }
    if (ok) ok = net.layers.front().in_f == net.n_af && net.layers.back().out_f == 1;
  }
  fclose(f);
  if (!ok) fprintf(stderr, "staf_mlp: cannot read %s\n", path.c_str());
  return ok;
}

// Forward and backward over all atoms of one species.  Returns sum of atomic energies.
template <typename T>
T eval_net(const Net<T>& net, const T* af, int n_atoms, T* dE_daf) {
  const int n_af = net.n_af;
  std::vector<std::vector<T>> acts(net.layers.size() + 1);
  acts[0].resize((size_t)n_atoms * n_af);
  for (int a = 0; a < n_atoms; a++)
    for (int i = 0; i < n_af; i++) acts[0][(size_t)a * n_af + i] = std::log(af[(size_t)a * n_af + i] + T(1e-3)) - net.mu[i];
  for (size_t li = 0; li < net.layers.size(); li++) {
    const Layer<T>& L = net.layers[li];
    acts[li + 1].assign((size_t)n_atoms * L.out_f, T(0));
    for (int a = 0; a < n_atoms; a++) {
      const T* x = &acts[li][(size_t)a * L.in_f];
      T* y = &acts[li + 1][(size_t)a * L.out_f];
      for (int j = 0; j < L.out_f; j++) y[j] = L.b[j];
      for (int i = 0; i < L.in_f; i++) {
        const T xi = x[i];
        const T* w = &L.W[(size_t)i * L.out_f];
        for (int j = 0; j < L.out_f; j++) y[j] += xi * w[j];
      }
      if (L.act == ACT_TANH)
        for (int j = 0; j < L.out_f; j++) y[j] = std::tanh(y[j]);
      else if (L.act == ACT_RELU)
        for (int j = 0; j < L.out_f; j++) y[j] = y[j] > T(0) ? y[j] : T(0);
    }
  }
  T e = T(0);
  for (int a = 0; a < n_atoms; a++) e += acts.back()[a];
  std::vector<T> delta((size_t)n_atoms, T(1)), next;
  for (int li = (int)net.layers.size() - 1; li >= 0; li--) {
    const Layer<T>& L = net.layers[li];
    next.assign((size_t)n_atoms * L.in_f, T(0));
    for (int a = 0; a < n_atoms; a++) {
      const T* y = &acts[li + 1][(size_t)a * L.out_f];
      const T* dy = &delta[(size_t)a * L.out_f];
      T* dx = &next[(size_t)a * L.in_f];
      for (int j = 0; j < L.out_f; j++) {
        T g = dy[j];
        if (L.act == ACT_TANH) g *= (T(1) - y[j] * y[j]);
        else if (L.act == ACT_RELU && y[j] <= T(0)) g = T(0);
        for (int i = 0; i < L.in_f; i++) dx[i] += g * L.W[(size_t)i * L.out_f + j];
      }
    }
    delta.swap(next);
  }
  for (int a = 0; a < n_atoms; a++)
    for (int i = 0; i < n_af; i++)
      dE_daf[(size_t)a * n_af + i] = delta[(size_t)a * n_af + i] / (af[(size_t)a * n_af + i] + T(1e-3));
  return e;
}

}  // namespace

struct StafMlp {
  int precision = 0;
  StafMlpBackend backend = STAF_MLP_NATIVE;
  std::vector<Net<float>> nets_f;
  std::vector<Net<double>> nets_d;
};

extern "C" {

StafMlp* staf_mlp_create(StafMlpBackend backend, const char* model_dir, int precision, int device_id) {
  (void)device_id;
  if (!model_dir) return NULL;
  StafMlp* m = new StafMlp();
  m->precision = precision ? 1 : 0;
  m->backend = backend;
  if (backend == STAF_MLP_ORT)
    fprintf(stderr, "staf_mlp: ONNX Runtime backend not available in this build, using the native Dense evaluation "
                    "of mlp_type*.bin\n");
  for (int k = 0; k < 32; k++) {
    const std::string path = std::string(model_dir) + "/mlp_type" + std::to_string(k) + ".bin";
    FILE* t = fopen(path.c_str(), "rb");
    if (!t) break;
    fclose(t);
    bool ok;
    if (m->precision) { m->nets_d.emplace_back(); ok = load_bin(path, m->nets_d.back()); }
    else { m->nets_f.emplace_back(); ok = load_bin(path, m->nets_f.back()); }
    if (!ok) { delete m; return NULL; }
  }
  if (m->nets_f.empty() && m->nets_d.empty()) {
    fprintf(stderr, "staf_mlp: no mlp_type*.bin under %s\n", model_dir);
    delete m;
    return NULL;
  }
  return m;
}

int staf_mlp_eval(StafMlp* mlp, StafMlpEval* io) {
  if (!mlp || !io || !io->n_atoms || !io->n_af) return -1;
  const int n_type = staf_mlp_ntypes(mlp);
  size_t off = 0;
  if (mlp->precision == 0) {
    if (!io->af_f32 || !io->energy_f32 || !io->dE_daf_f32) return -1;
    float e_tot = 0.f;
    for (int t = 0; t < n_type; t++) {
      if (io->n_af[t] != mlp->nets_f[t].n_af) return -3;
      e_tot += 0.5f * eval_net<float>(mlp->nets_f[t], io->af_f32 + off, io->n_atoms[t], io->dE_daf_f32 + off);
      off += (size_t)io->n_atoms[t] * io->n_af[t];
    }
    io->energy_f32[0] = e_tot;
    return 0;
  }
  if (!io->af_f64 || !io->energy_f64 || !io->dE_daf_f64) return -1;
  double e_tot = 0.0;
  for (int t = 0; t < n_type; t++) {
    if (io->n_af[t] != mlp->nets_d[t].n_af) return -3;
    e_tot += 0.5 * eval_net<double>(mlp->nets_d[t], io->af_f64 + off, io->n_atoms[t], io->dE_daf_f64 + off);
    off += (size_t)io->n_atoms[t] * io->n_af[t];
  }
  io->energy_f64[0] = e_tot;
  return 0;
}

void staf_mlp_destroy(StafMlp* mlp) { delete mlp; }

int staf_mlp_ntypes(const StafMlp* mlp) {
  if (!mlp) return 0;
  return (int)(mlp->precision ? mlp->nets_d.size() : mlp->nets_f.size());
}

int staf_mlp_n_af(const StafMlp* mlp, int type) {
  if (!mlp || type < 0 || type >= staf_mlp_ntypes(mlp)) return -1;
  return mlp->precision ? mlp->nets_d[type].n_af : mlp->nets_f[type].n_af;
}

int staf_mlp_precision(const StafMlp* mlp) { return mlp ? mlp->precision : -1; }

// ---- library-internal access to the loaded weights (staf_mlp_internal.h): the device-resident evaluation of the
// MD entry uploads them once at load time.
int staf_mlp_internal_nlayers(const StafMlp* mlp, int type) {
  if (!mlp || type < 0 || type >= staf_mlp_ntypes(mlp)) return -1;
  return (int)(mlp->precision ? mlp->nets_d[type].layers.size() : mlp->nets_f[type].layers.size());
}

const void* staf_mlp_internal_mu(const StafMlp* mlp, int type) {
  if (staf_mlp_internal_nlayers(mlp, type) < 0) return NULL;
  return mlp->precision ? (const void*)mlp->nets_d[type].mu.data() : (const void*)mlp->nets_f[type].mu.data();
}

int staf_mlp_internal_layer(const StafMlp* mlp, int type, int layer, int* act, int* in_f, int* out_f, const void** W,
                            const void** b) {
  const int nl = staf_mlp_internal_nlayers(mlp, type);
  if (nl < 0 || layer < 0 || layer >= nl) return -1;
  if (mlp->precision) {
    const auto& L = mlp->nets_d[type].layers[layer];
    *act = L.act; *in_f = L.in_f; *out_f = L.out_f; *W = L.W.data(); *b = L.b.data();
  } else {
    const auto& L = mlp->nets_f[type].layers[layer];
    *act = L.act; *in_f = L.in_f; *out_f = L.out_f; *W = L.W.data(); *b = L.b.data();
  }
  return 0;
}

}  // extern "C"
