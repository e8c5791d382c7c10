// MD-facing entry (LAMMPS `pair_style staf`): staf_load / staf_compute / staf_free of include/staf.h.
//
// Host logic follows libstaf/src/staf_api.cpp:192-412 (validation and return codes, species-sorted packing of
// the owned atoms, ghosts appended, neighbour-index remapping, un-packing of forces) and the step order of
// calculateforces (libstaf/vendor/jmd/nn_nn_mlp.cu:838-889): neighbour list (own, or the caller's with no
// periodic wrap) -> descriptors -> fingerprints of every species -> MLP -> 2-body + 3-body forces with virial.
// Everything on the GPU runs in float64.  The path is fused in the sense that matters for memory: no tensor of the
// angular buffer's width exists.  The descriptor kernel runs radial-only and leaves, per centre, its sorted
// neighbour list with unit vectors, 1/r, cutoff values and their gradients (nr-wide rows); the 3-body fingerprint
// and force kernels rebuild every triplet's angular descriptor and Jacobian from those rows in LDS.  HBM traffic of a
// call is positions and types in, forces out, and those nr-wide rows.  The MLP is the per-species Dense stack,
// evaluated on the GPU between the fingerprint and the force kernels (or on the host, staf_mlp.cpp, on request).
#include "staf_common.hpp"
#include "staf_reduce.hpp"
#include "staf_mlp_dev.hpp"
#include "../../include/staf.h"
#include "../../include/staf_mlp.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <algorithm>
#include <vector>

namespace {

template <typename T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  bool reserve(size_t want) {
    if (want <= n) return true;
    if (p) (void)hipFree(p);
    p = nullptr;
    n = 0;
    if (hipMalloc((void**)&p, want * sizeof(T)) != hipSuccess) return false;
    n = want;
    return true;
  }
  void release() {
    if (p) (void)hipFree(p);
    p = nullptr;
    n = 0;
  }
};

// Pinned host staging (allocated pinned, never registered): one block for everything a call sends, one for what it
// brings back, so that a call makes one copy each way.
template <typename T>
struct PinBuf {
  T* p = nullptr;
  size_t n = 0;
  bool reserve(size_t want) {
    if (want <= n) return true;
    if (p) (void)hipHostFree(p);
    p = nullptr;
    n = 0;
    want += want / 4;
    if (hipHostMalloc((void**)&p, want * sizeof(T), hipHostMallocDefault) != hipSuccess) return false;
    n = want;
    return true;
  }
  void release() {
    if (p) (void)hipHostFree(p);
    p = nullptr;
    n = 0;
  }
};

__global__ void add_into_kernel(double* dst, const double* src, int n) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < n) dst[e] += src[e];
}

// Host-to-device copy that is complete when it returns, on a stream of the model: a blocking hipMemcpy runs on the
// legacy default stream, and work on that stream while another host thread records a graph (every handle records
// its own) is refused by the runtime and spoils that thread's recording.
static bool upload_sync(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  return hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream) == hipSuccess &&
         hipStreamSynchronize(stream) == hipSuccess;
}

// dst[e] = sum over the nb op outputs src[b*n + e], b ascending (fixed order); the same for the 3x3 virials
__global__ void combine_kernel(double* dst, const double* src, int n, int nb, double* vdst, const double* vsrc) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < n) {
    double s = 0;
    for (int b = 0; b < nb; b++) s += src[(size_t)b * n + e];
    dst[e] = s;
  }
  if (e < 9) {
    double s = 0;
    if (vsrc)
      for (int b = 0; b < nb; b++) s += vsrc[b * 9 + e];
    vdst[e] = s;
  }
}

bool read_numbers(const std::string& path, std::vector<double>& out, int* rows) {
  FILE* f = fopen(path.c_str(), "r");
  if (!f) return false;
  out.clear();
  int nrows = 0;
  char line[1 << 16];
  while (fgets(line, sizeof(line), f)) {
    char* s = line;
    int got = 0;
    for (;;) {
      char* e;
      double v = strtod(s, &e);
      if (e == s) break;
      out.push_back(v);
      s = e;
      got++;
    }
    if (got) nrows++;
  }
  fclose(f);
  if (rows) *rows = nrows;
  return !out.empty();
}

}  // namespace

struct StafModel {
  StafOptions opt;
  std::string dir;
  StafMlp* mlp = nullptr;
  int nt = 0, ntc = 0, nr = 60, na = 1770;
  double Rc = 4.5, Ra = 4.5, Rs = 2.25;
  std::vector<int> Ar, Aa;
  std::vector<DevBuf<double>> alpha2b, alpha3b, emb2b, emb3b;
  staf::DescConfig<double> cfg;
  hipStream_t stream = nullptr;            // the call's stream (descriptors, copies, final sum)
  std::vector<hipStream_t> sstream;        // one per centre species: their op chains are independent
  hipEvent_t ev_fork = nullptr;
  std::vector<hipEvent_t> ev_join;
  // device buffers
  // in_d  = [pos nall*3 | box 6 | howmany nlocal ints | with nlocal*nr ints]   (mirror of in_h, one copy per call)
  // out_d = [force nall*3 | virial 9 | atomic energies nlocal]                 (mirror of out_h, one copy per call)
  DevBuf<double> in_d, out_d, force_op, virial_op, af2, af3, g2, g3;
  PinBuf<double> in_h, out_h;
  std::vector<int> type_map_up, tipos_up;   // what the device copies of type_map and tipos hold
  bool actual_type_up = false;
  // The kernel sequence of a call (descriptors .. sum of the forces), recorded as a HIP graph once a configuration
  // of the same shape has been evaluated eagerly (which also sizes every scratch buffer), then replayed: an MD run
  // repeats one shape for many steps, and issuing ~27 launches costs the host more than the GPU needs to run them.
  struct Replay {
    int state = 0;             // 0: nothing, 1: shape seen (eagerly), 2: graph ready
    // Recording costs about as much as six replays save.  A shape is recorded when it has come `need` times in a
    // row; a graph that was dropped young (the shape changed after few replays, as when atoms migrate between
    // ranks every few steps) doubles `need`, one that lived long resets it.
    int seen = 0, replays = 0, need = 2;
    int nlocal = 0, nall = 0, ext = 0, want_w = 0;
    unsigned epoch = 0;        // staf::release_epoch() when the shape was first seen
    std::vector<int> tipos;
    const void* in_d = nullptr;
    const void* out_d = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    void drop() {
      if (exec) (void)hipGraphExecDestroy(exec);
      if (graph) (void)hipGraphDestroy(graph);
      exec = nullptr;
      graph = nullptr;
      state = 0;
    }
  } replay;
  bool use_graph = true;
  // device-resident MLP (default); false: the host evaluation of staf_mlp.cpp between the kernels
  bool dev_mlp = false;
  std::vector<staf::DevMlpNet> dnets;
  DevBuf<double> raddescr, des3bsupp, der2b, der3bsupp, unit;   // nr-wide rows per owned atom; unit = (u, 1/r)
  DevBuf<double> slotf, selff;   // slot forces [nlocal, nr, 3] and centres' own forces [nlocal, 3] (own-list calls)
  DevBuf<int> intmap2b, numtriplet, type_map, tipos, actual_type;
  // host staging
  std::vector<double> af_h, gr_h, tmp2, tmp3;
  std::vector<float> af_f, gr_f;
  std::vector<int> order_to_slot, slot_to_order, type_map_h;
};

static bool load_species_params(StafModel* m) {
  const int nt = m->nt, ntc = m->ntc;
  m->Ar.assign(nt, 0);
  m->Aa.assign(nt, 0);
  m->alpha2b.resize(nt);
  m->alpha3b.resize(nt);
  m->emb2b.resize(nt);
  m->emb3b.resize(nt);
  for (int k = 0; k < nt; k++) {
    const std::string pre = m->dir + "/type" + std::to_string(k) + "_";
    std::vector<double> a2, a3, e2, e3;
    int rows = 0;
    if (!read_numbers(pre + "alpha_2body.dat", a2, &rows) || rows != nt || a2.size() % nt) return false;
    if (!read_numbers(pre + "alpha_3body.dat", a3, &rows) || rows != ntc || a3.size() % (3 * ntc)) return false;
    m->Ar[k] = (int)(a2.size() / nt);
    m->Aa[k] = (int)(a3.size() / (3 * ntc));
    // the kernels take the squared embeddings (what the reference's Python layers feed its ops)
    if (!read_numbers(pre + "type_emb_2b_sq.dat", e2, nullptr)) {
      if (!read_numbers(pre + "type_emb_2b.dat", e2, nullptr)) return false;
      for (double& v : e2) v *= v;
    }
    if (!read_numbers(pre + "type_emb_3b_sq.dat", e3, nullptr)) {
      if (!read_numbers(pre + "type_emb_3b.dat", e3, nullptr)) return false;
      for (double& v : e3) v *= v;
    }
    if ((int)e2.size() != nt * m->Ar[k] || (int)e3.size() != ntc * m->Aa[k]) return false;
    struct { DevBuf<double>* d; std::vector<double>* h; } up[4] = {
        {&m->alpha2b[k], &a2}, {&m->alpha3b[k], &a3}, {&m->emb2b[k], &e2}, {&m->emb3b[k], &e3}};
    for (auto& u : up) {
      if (!u.d->reserve(u.h->size())) return false;
      if (!upload_sync(u.d->p, u.h->data(), u.h->size() * sizeof(double), m->stream)) return false;
    }
  }
  return true;
}

// staf_jmd.cfg: "key = value" lines (test/test-lammps-smoke/staf_jmd.cfg); missing file or keys -> the defaults
// the reference writes into its auto-generated cfg (libstaf/src/staf_api.cpp:139-148).
static void read_cfg(StafModel* m) {
  FILE* f = fopen((m->dir + "/staf_jmd.cfg").c_str(), "r");
  if (!f) return;
  char line[4096];
  while (fgets(line, sizeof(line), f)) {
    char key[256];
    double v;
    if (sscanf(line, " %255[A-Za-z_] = %lf", key, &v) != 2) continue;
    if (!strcmp(key, "Buffer_radial_descriptors")) m->nr = (int)v;
    else if (!strcmp(key, "Buffer_angular_descriptors")) m->na = (int)v;
    else if (!strcmp(key, "Cutoff")) m->Rc = v;
    else if (!strcmp(key, "Cutoff_Angular")) m->Ra = v;
    else if (!strcmp(key, "Hardcore_Cutoff")) m->Rs = v;
    else if (!strcmp(key, "number_of_types")) m->nt = (int)v;
  }
  fclose(f);
}

extern "C" {

void staf_options_default(StafOptions* opt) {
  if (!opt) return;
  memset(opt, 0, sizeof(*opt));
  opt->mlp_backend = STAF_MLP_ORT;
  opt->device_id = 0;
  opt->precision = 0;
}

int staf_cuda_set_device(int device_id) {
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev <= 0) {
    fprintf(stderr, "staf_cuda_set_device: no GPU\n");
    return -1;
  }
  if (device_id < 0) device_id = 0;
  device_id %= ndev;
  if (hipSetDevice(device_id) != hipSuccess) return -1;
  return device_id;
}

void staf_free(StafModel* m) {
  if (!m) return;
  if (m->stream) (void)hipStreamSynchronize(m->stream);
  m->replay.drop();
  for (hipStream_t s : m->sstream)
    if (s) { (void)hipStreamSynchronize(s); (void)hipStreamDestroy(s); }
  for (hipEvent_t e : m->ev_join)
    if (e) (void)hipEventDestroy(e);
  if (m->ev_fork) (void)hipEventDestroy(m->ev_fork);
  if (m->stream) (void)hipStreamDestroy(m->stream);
  if (m->mlp) staf_mlp_destroy(m->mlp);
  for (auto& n : m->dnets) staf::dev_mlp_free(&n);
  for (auto* v : {&m->alpha2b, &m->alpha3b, &m->emb2b, &m->emb3b})
    for (auto& b : *v) b.release();
  m->in_h.release();
  m->out_h.release();
  for (DevBuf<double>* b : {&m->in_d, &m->out_d, &m->force_op, &m->virial_op, &m->af2, &m->af3, &m->g2, &m->g3,
                            &m->raddescr, &m->des3bsupp, &m->der2b, &m->der3bsupp, &m->unit})
    b->release();
  for (DevBuf<int>* b : {&m->intmap2b, &m->numtriplet, &m->type_map, &m->tipos, &m->actual_type})
    b->release();
  delete m;
}

StafModel* staf_load(const char* model_dir, const StafOptions* opt) {
  if (!model_dir) return NULL;
  StafModel* m = new StafModel();
  staf_options_default(&m->opt);
  if (opt) m->opt = *opt;
  const int dev = staf_cuda_set_device(m->opt.device_id);
  if (dev < 0) { delete m; return NULL; }
  m->opt.device_id = dev;
  m->dir = model_dir;
  m->mlp = staf_mlp_create(m->opt.mlp_backend, model_dir, m->opt.precision, dev);
  if (!m->mlp) {
    fprintf(stderr, "staf_load: staf_mlp_create failed for %s\n", model_dir);
    staf_free(m);
    return NULL;
  }
  m->nt = staf_mlp_ntypes(m->mlp);
  read_cfg(m);
  if (m->nt != staf_mlp_ntypes(m->mlp) || m->nt < 1 || m->nt > staf::NT_MAX) {
    fprintf(stderr, "staf_load: %d species in staf_jmd.cfg, %d MLP files\n", m->nt, staf_mlp_ntypes(m->mlp));
    staf_free(m);
    return NULL;
  }
  m->ntc = m->nt * (m->nt + 1) / 2;
  // Streams of the model (default priority; non-blocking: no implicit ordering with the legacy default stream).
  bool ok = hipStreamCreateWithFlags(&m->stream, hipStreamNonBlocking) == hipSuccess &&
            hipEventCreateWithFlags(&m->ev_fork, hipEventDisableTiming) == hipSuccess;
  m->sstream.assign(m->nt, nullptr);
  m->ev_join.assign(m->nt, nullptr);
  for (int k = 0; k < m->nt && ok; k++)
    ok = hipStreamCreateWithFlags(&m->sstream[k], hipStreamNonBlocking) == hipSuccess &&
         hipEventCreateWithFlags(&m->ev_join[k], hipEventDisableTiming) == hipSuccess;
  if (!ok) {
    fprintf(stderr, "staf_load: cannot create the model's streams\n");
    staf_free(m);
    return NULL;
  }
  if (!load_species_params(m)) {
    fprintf(stderr, "staf_load: cannot read the type*_alpha_*.dat / type*_type_emb_*.dat files of %s\n", model_dir);
    staf_free(m);
    return NULL;
  }
  for (int k = 0; k < m->nt; k++)
    if (staf_mlp_n_af(m->mlp, k) != m->Ar[k] + m->Aa[k]) {
      fprintf(stderr, "staf_load: species %d: MLP input width %d != %d + %d fingerprints\n", k,
              staf_mlp_n_af(m->mlp, k), m->Ar[k], m->Aa[k]);
      staf_free(m);
      return NULL;
    }
  // The kernel sequence of a repeated shape is replayed as a HIP graph unless the caller asks for eager launches
  // (StafOptions.reserved bit 2, or STAF_MD_EAGER=1 in the environment).
  m->use_graph = !(m->opt.reserved & 4) && !getenv("STAF_MD_EAGER");
  // The MLP runs on the GPU between the fingerprint and the force kernels unless the caller asks for the host
  // evaluation (StafOptions.reserved bit 1, or STAF_MLP_HOST=1 in the environment).
  if (!(m->opt.reserved & 2) && !getenv("STAF_MLP_HOST")) {
    m->dnets.resize(m->nt);
    m->dev_mlp = true;
    for (int k = 0; k < m->nt && m->dev_mlp; k++) m->dev_mlp = staf::dev_mlp_upload(m->mlp, k, &m->dnets[k], m->stream);
    if (!m->dev_mlp) {
      for (auto& n : m->dnets) staf::dev_mlp_free(&n);
      m->dnets.clear();
      fprintf(stderr, "staf_load: MLP not representable on the device path, evaluating it on the host\n");
    }
  }
  if (staf::desc_configure<double>(m->cfg, m->Rc, m->nr, m->na, m->Rs, m->Ra) != STAF_OK) {
    staf_free(m);
    return NULL;
  }
  return m;
}

// A GPU runtime failure: -20 to the caller; with STAF_DEBUG set in the environment, where it came from on stderr.
static int gpu_failure(int line, int code) {
  static const bool verbose = getenv("STAF_DEBUG") != nullptr;
  if (verbose) fprintf(stderr, "staf_compute: GPU runtime failure at staf_api.hip:%d (code %d)\n", line, code);
  return -20;
}
#define STAF_HIP_OK(x) do { const hipError_t e_ = (x); if (e_ != hipSuccess) return gpu_failure(__LINE__, (int)e_); } while (0)

int staf_compute(StafModel* m, int nlocal, int nghost, const double* x, const double* box, const int* type,
                 const int* howmany, const int* with, int maxneigh, double* e_rank, double* f, double* virial) {
  if (!m || !m->mlp) return -1;
  const bool ext = (howmany != NULL);
  const int nall = ext ? (nlocal + nghost) : nlocal;
  if (nlocal <= 0) return -3;
  if (!x || !box || (ext && !with)) return -1;
  if (box[0] == 0.0 || box[3] == 0.0 || box[5] == 0.0) return -7;
  if (hipSetDevice(m->opt.device_id) != hipSuccess) return gpu_failure(__LINE__, 0);
  const int nt = m->nt, nr = m->nr, na = m->na;

  // ---- owned atoms species-sorted into slots [0, nlocal), ghosts keep their order behind them
  std::vector<int> tipos(nt, 0), cursor(nt, 0);
  for (int i = 0; i < nlocal; i++) {
    const int sp = type ? type[i] : 0;
    if (sp < 0 || sp >= nt) {
      fprintf(stderr, "staf_compute: unsupported type %d at atom %d\n", sp, i);
      return -8;
    }
    tipos[sp]++;
  }
  for (int t = 1; t < nt; t++) cursor[t] = cursor[t - 1] + tipos[t - 1];
  m->order_to_slot.resize(nall);
  m->slot_to_order.resize(nall);
  m->type_map_h.resize(nall);
  for (int i = 0; i < nlocal; i++) {
    const int sp = type ? type[i] : 0;
    const int slot = cursor[sp]++;
    m->order_to_slot[i] = slot;
    m->slot_to_order[slot] = i;
    m->type_map_h[slot] = sp;
  }
  for (int i = nlocal; i < nall; i++) {
    const int sp = type ? type[i] : 0;
    if (sp < 0 || sp >= nt) return -8;
    m->order_to_slot[i] = i;
    m->slot_to_order[i] = i;
    m->type_map_h[i] = sp;
  }
  // ---- the call's input block, written straight into pinned memory
  const size_t L = (size_t)nlocal;
  const size_t n_in_d = (size_t)nall * 3 + 6;                                 // doubles
  const size_t n_in_i = ext ? L + L * nr : 0;                                 // ints behind them
  const size_t n_in = n_in_d + (n_in_i + 1) / 2;
  const size_t n_out = (size_t)nall * 3 + 9 + L;
  if (!m->in_h.reserve(n_in) || !m->out_h.reserve(n_out)) return -1;
  double* pos_h = m->in_h.p;
  int* how_h = (int*)(m->in_h.p + n_in_d);
  int* with_h = how_h + L;
  if (ext) {
    memset(how_h, 0, n_in_i * sizeof(int));
    for (int i = 0; i < nlocal; i++) {
      const int slot = m->order_to_slot[i];
      int nn = howmany[i];
      if (nn < 0) nn = 0;
      if (nn > nr) nn = nr;   // truncated like the reference (staf_api.cpp:321-323)
      if (nn > maxneigh) nn = maxneigh;
      how_h[slot] = nn;
      for (int k = 0; k < nn; k++) {
        const int j = with[(size_t)i * maxneigh + k];
        if (j < 0 || j >= nall) {
          fprintf(stderr, "staf_compute: neighbor index %d out of range [0,%d)\n", j, nall);
          return -9;
        }
        with_h[(size_t)slot * nr + k] = m->order_to_slot[j];
      }
    }
  }
  for (int i = 0; i < nall; i++) {
    const int s = m->order_to_slot[i];
    pos_h[3 * s] = x[3 * i];
    pos_h[3 * s + 1] = x[3 * i + 1];
    pos_h[3 * s + 2] = x[3 * i + 2];
  }
  memcpy(pos_h + (size_t)nall * 3, box, 6 * sizeof(double));

  // ---- device buffers
  int amax2 = 0, amax3 = 0;
  for (int k = 0; k < nt; k++) { amax2 = m->Ar[k] > amax2 ? m->Ar[k] : amax2; amax3 = m->Aa[k] > amax3 ? m->Aa[k] : amax3; }
  const int* type_map_before = m->type_map.p;
  bool ok = m->in_d.reserve(n_in) && m->out_d.reserve(n_out) &&
            m->force_op.reserve((size_t)nall * 3 * 2 * nt) && m->virial_op.reserve((size_t)9 * 2 * nt) && m->af2.reserve(L * amax2) &&
            m->af3.reserve(L * amax3) && m->g2.reserve(L * amax2) && m->g3.reserve(L * amax3) &&
            m->raddescr.reserve(L * nr) && m->des3bsupp.reserve(L * nr) && m->der2b.reserve(L * 3 * nr) &&
            m->der3bsupp.reserve(L * 3 * nr) && m->unit.reserve(L * 4 * nr) && m->intmap2b.reserve(L * (nr + 1)) &&
            m->numtriplet.reserve(L) && m->slotf.reserve(L * nr * 3) && m->selff.reserve(L * 3) &&
            m->type_map.reserve(nall) && m->tipos.reserve(nt) && m->actual_type.reserve(nt);
  if (!ok) return -1;
  if (m->type_map.p != type_map_before) m->type_map_up.clear();   // a new block holds nothing yet
  hipStream_t st = m->stream;
  double* const d_pos = m->in_d.p;
  double* const d_box = d_pos + (size_t)nall * 3;
  int* const d_how = (int*)(m->in_d.p + n_in_d);
  int* const d_with = d_how + L;
  double* const d_force = m->out_d.p;
  double* const d_W = d_force + (size_t)nall * 3;
  double* const d_e = d_W + 9;
  STAF_HIP_OK(hipMemcpyAsync(m->in_d.p, m->in_h.p, n_in * sizeof(double), hipMemcpyHostToDevice, st));
  // species of the slots and atoms per species: sent when they differ from what the device holds (in MD they change
  // when atoms migrate, not every step); the blocking copies read host vectors that the next lines may replace
  if (m->type_map_up != m->type_map_h) {
    if (!upload_sync(m->type_map.p, m->type_map_h.data(), (size_t)nall * sizeof(int), st)) return gpu_failure(__LINE__, 0);
    m->type_map_up = m->type_map_h;
  }
  if (m->tipos_up != tipos) {
    if (!upload_sync(m->tipos.p, tipos.data(), nt * sizeof(int), st)) return gpu_failure(__LINE__, 0);
    m->tipos_up = tipos;
  }
  if (!m->actual_type_up) {
    std::vector<int> ats(nt);
    for (int k = 0; k < nt; k++) ats[k] = k;
    if (!upload_sync(m->actual_type.p, ats.data(), nt * sizeof(int), st)) return gpu_failure(__LINE__, 0);
    m->actual_type_up = true;
  }
  // No synchronisation here: the pinned input block outlives the call's final synchronisation.
  staf::DeferStatus defer;   // conditions the kernels detect are read once, after the last kernel

  // ---- descriptors (own minimum-image list, or the caller's list with explicit images)
  auto descriptors = [&]() -> int {
    return staf::desc_launch<double>(m->cfg, d_pos, d_box, 1, nlocal, nall, ext ? d_how : nullptr,
                                     ext ? d_with : nullptr, ext ? 1 : 0, m->raddescr.p, nullptr, m->des3bsupp.p,
                                     m->intmap2b.p, nullptr, m->der2b.p, nullptr, m->der3bsupp.p, m->numtriplet.p,
                                     m->unit.p, st) == STAF_OK ? 0 : -20;
  };
  int rc = 0;
  double energy = 0.0;
  double W[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
  const int n3 = nall * 3;
  const bool want_w = virial != nullptr;
  const int skip_pbc = ext ? 1 : 0;   // the caller's neighbours are explicit periodic images
  // ---- everything stays on the device: per species fingerprints -> MLP -> forces, one stream per species (the
  // chains meet only in the sum of the forces); one synchronisation at the end of the call
  auto device_sequence = [&]() -> int {
    if (descriptors() != 0) return gpu_failure(__LINE__, 0);
    // every species stream branches off right behind the descriptors, and the call's stream waits for all of
    // them only after the last chain has been issued: a recorded graph then holds independent branches
    STAF_HIP_OK(hipEventRecord(m->ev_fork, st));
    for (int k = 0; k < nt; k++)
      if (tipos[k] > 0) STAF_HIP_OK(hipStreamWaitEvent(m->sstream[k], m->ev_fork, 0));
    // The chains are issued step by step across the species (all fingerprint ops, then all networks, ...): the host
    // -- also when it replays a recorded graph -- submits launches one after the other, and a chain issued as a
    // whole would have run before the next one is even submitted.
    int nops = 0;
    // Within a step the species with the most atoms comes first: launches (and the nodes of a replayed graph) are
    // submitted in issue order, and the longest chain should not be the one that starts last.
    std::vector<int> first_atom(nt, 0), op_slot(nt, 0), by_size;
    for (int k = 0, at = 0, sl = 0; k < nt; at += tipos[k], k++) {
      first_atom[k] = at;
      if (tipos[k] > 0) { op_slot[k] = sl++; by_size.push_back(k); }
    }
    std::stable_sort(by_size.begin(), by_size.end(), [&](int a, int b) { return tipos[a] > tipos[b]; });
    // With the library's own neighbour list (a symmetric map) the forces take the step-level route: per species one
    // launch leaves the 2-body + 3-body forces on the centres' neighbour slots (and their virial), and after the
    // join one launch lets every atom collect them.  A caller's list (ghosts, not symmetric) keeps one force op per
    // body and species, each with its own gather.
    const bool slots_route = !ext;
    for (int step = 0; step < 5; step++) {
      if (slots_route && step == 3) continue;
      for (int k : by_size) {
        const int Nl = tipos[k], Ar = m->Ar[k], Aa = m->Aa[k];
        const int shift = first_atom[k], slot = op_slot[k];
        hipStream_t sk = m->sstream[k];
        const size_t o = (size_t)shift;
        double* af2 = m->af2.p + o * amax2;
        double* af3 = m->af3.p + o * amax3;
        double* g2 = m->g2.p + o * amax2;
        double* g3 = m->g3.p + o * amax3;
        const int op = 2 * slot + (step - 3);          // output slot of the force ops (steps 3 and 4)
        double* fo = m->force_op.p + (size_t)(op < 0 ? 0 : op) * n3;
        double* wo = want_w ? m->virial_op.p + (op < 0 ? 0 : op) * 9 : nullptr;
        const double* px = want_w ? d_pos : nullptr;
        const double* bx = want_w ? d_box : nullptr;
        switch (step) {
          case 0:
            rc = staf_op_radial_afs_f64(m->raddescr.p + o * nr, nr, m->alpha2b[k].p, Ar, af2, 1, Nl,
                                        m->intmap2b.p + o * (nr + 1), m->emb2b[k].p, m->type_map.p, nt, nlocal, sk);
            break;
          case 1:
            rc = staf::angular_afs<double>(m->des3bsupp.p + o * nr, nullptr, m->unit.p + o * 4 * nr, nr, na, af3, 1,
                                           Nl, nullptr, m->intmap2b.p + o * (nr + 1), m->alpha3b[k].p, Aa,
                                           m->emb3b[k].p, m->type_map.p, m->numtriplet.p + o, nt, nlocal, sk);
            break;
          case 2:
            rc = staf::dev_mlp_eval(m->dnets[k], af2, Ar, af3, Aa, Nl, d_e + o, g2, g3, sk);
            break;
          case 3:
            rc = staf::force_doublets<double>(g2, m->raddescr.p + o * nr, m->der2b.p + o * 3 * nr,
                                              m->intmap2b.p + o * (nr + 1), nr, nall, 1, Ar, m->alpha2b[k].p,
                                              m->emb2b[k].p, nt, m->tipos.p, m->actual_type.p + k, fo, m->type_map.p,
                                              Nl, wo, px, bx, nlocal, skip_pbc, sk);
            break;
          default:
            if (slots_route) {
              staf::Force2In<double> two;
              two.G2 = g2; two.D = m->raddescr.p + o * nr; two.dD = m->der2b.p + o * 3 * nr;
              two.alpha2b = m->alpha2b[k].p; two.emb2b = m->emb2b[k].p; two.Ar = Ar;
              double* sf = m->slotf.p + o * nr * 3;
              rc = staf::force_tripl<double>(g3, m->des3bsupp.p + o * nr, nullptr, m->der3bsupp.p + o * 3 * nr, nullptr,
                                             m->unit.p + o * 4 * nr, m->intmap2b.p + o * (nr + 1), nullptr, nr, na,
                                             nall, 1, Aa, m->emb3b[k].p, nt, m->tipos.p, m->actual_type.p + k, nullptr,
                                             m->numtriplet.p + o, m->alpha3b[k].p, m->type_map.p, Nl, nullptr, nullptr,
                                             nullptr, nlocal, skip_pbc, sk, sf, m->selff.p + o * 3, &two);
              if (rc == STAF_OK && want_w)
                rc = staf::slots_virial<double>(sf, m->intmap2b.p + o * (nr + 1), d_pos, d_box, m->tipos.p,
                                                m->actual_type.p + k, m->virial_op.p + slot * 9, 1, nall, Nl, nlocal, nr,
                                                skip_pbc, sk);
              STAF_HIP_OK(hipEventRecord(m->ev_join[k], sk));
              if (rc != STAF_OK) return gpu_failure(__LINE__, rc);
              nops = slot + 1 > nops ? slot + 1 : nops;
              continue;
            }
            rc = staf::force_tripl<double>(g3, m->des3bsupp.p + o * nr, nullptr, m->der3bsupp.p + o * 3 * nr, nullptr,
                                           m->unit.p + o * 4 * nr, m->intmap2b.p + o * (nr + 1), nullptr, nr, na, nall,
                                           1, Aa, m->emb3b[k].p, nt, m->tipos.p, m->actual_type.p + k, fo,
                                           m->numtriplet.p + o, m->alpha3b[k].p, m->type_map.p, Nl, wo, px, bx, nlocal,
                                           skip_pbc, sk);
            STAF_HIP_OK(hipEventRecord(m->ev_join[k], sk));
            break;
        }
        if (rc != STAF_OK) return gpu_failure(__LINE__, rc);
        if (step >= 3) nops = op + 1 > nops ? op + 1 : nops;
      }
    }
    for (int k = 0; k < nt; k++)
      if (tipos[k] > 0) STAF_HIP_OK(hipStreamWaitEvent(st, m->ev_join[k], 0));
    if (slots_route) {
      std::vector<const double*> sl(nt, nullptr), se(nt, nullptr);
      for (int k = 0; k < nt; k++)
        if (tipos[k] > 0) { sl[k] = m->slotf.p + (size_t)first_atom[k] * nr * 3; se[k] = m->selff.p + (size_t)first_atom[k] * 3; }
      if (staf::force_total<double>(m->intmap2b.p, nr, nlocal, 1, nt, tipos.data(), sl.data(), se.data(), nullptr,
                                    d_force, st) != STAF_OK)
        return gpu_failure(__LINE__, 0);
      // the species' virials (nothing to add to the forces: n = 0)
      hipLaunchKernelGGL(combine_kernel, dim3(1), dim3(256), 0, st, d_force, m->force_op.p, 0, nops, d_W,
                         want_w ? m->virial_op.p : nullptr);
      return hipGetLastError() == hipSuccess ? 0 : -20;
    }
    hipLaunchKernelGGL(combine_kernel, dim3((n3 + 255) / 256), dim3(256), 0, st, d_force, m->force_op.p, n3, nops,
                       d_W, want_w ? m->virial_op.p : nullptr);
    return hipGetLastError() == hipSuccess ? 0 : -20;
  };
  if (m->dev_mlp) {
    StafModel::Replay& rp = m->replay;
    const bool same = rp.state > 0 && rp.nlocal == nlocal && rp.nall == nall && rp.ext == (int)ext &&
                      rp.want_w == (int)want_w && rp.tipos == tipos && rp.in_d == m->in_d.p && rp.out_d == m->out_d.p &&
                      rp.epoch == staf::release_epoch();   // staf_ops_release frees what a recorded graph points into
    if (!m->use_graph || !same) {
      if (rp.state == 2) rp.need = rp.replays < 12 ? (rp.need < 64 ? 2 * rp.need : 64) : 2;
      rp.drop();
      if (device_sequence() != 0) return gpu_failure(__LINE__, 0);
      if (m->use_graph) {
        rp.state = 1;
        rp.seen = 1;
        rp.replays = 0;
        rp.nlocal = nlocal; rp.nall = nall; rp.ext = ext; rp.want_w = want_w; rp.tipos = tipos;
        rp.in_d = m->in_d.p; rp.out_d = m->out_d.p;
        rp.epoch = staf::release_epoch();
      }
    } else if (rp.state == 1 && ++rp.seen < rp.need) {
      if (device_sequence() != 0) return gpu_failure(__LINE__, 0);
    } else {
      if (rp.state == 1) {
        // the shape keeps coming and every buffer and scratch block has its final size: record the sequence
        STAF_HIP_OK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        const int issued = device_sequence();
        hipGraph_t g = nullptr;
        const hipError_t ended = hipStreamEndCapture(st, &g);
        if (issued != 0 || ended != hipSuccess || !g) {
          if (g) (void)hipGraphDestroy(g);
          (void)hipGetLastError();
          rp.drop();
          return gpu_failure(__LINE__, 0);
        }
        rp.graph = g;
        if (hipGraphInstantiate(&rp.exec, rp.graph, nullptr, nullptr, 0) != hipSuccess) {
          rp.drop();
          return gpu_failure(__LINE__, 0);
        }
        rp.state = 2;
      }
      STAF_HIP_OK(hipGraphLaunch(rp.exec, st));
      rp.replays++;
    }
  } else {
    if (descriptors() != 0) return gpu_failure(__LINE__, 0);
    // ---- fingerprints of every species, packed rows [Ar+Aa] for the MLP
    size_t total = 0;
    for (int k = 0; k < nt; k++) total += (size_t)tipos[k] * (m->Ar[k] + m->Aa[k]);
    m->af_h.resize(total);
    m->gr_h.assign(total, 0.0);
    size_t off = 0;
    int shift = 0;
    for (int k = 0; k < nt; shift += tipos[k], k++) {
      const int Nl = tipos[k], Ar = m->Ar[k], Aa = m->Aa[k];
      if (Nl == 0) continue;
      const size_t o = (size_t)shift;
      rc = staf_op_radial_afs_f64(m->raddescr.p + o * nr, nr, m->alpha2b[k].p, Ar, m->af2.p, 1, Nl,
                                  m->intmap2b.p + o * (nr + 1), m->emb2b[k].p, m->type_map.p, nt, nlocal, st);
      if (rc == STAF_OK)
        rc = staf::angular_afs<double>(m->des3bsupp.p + o * nr, nullptr, m->unit.p + o * 4 * nr, nr, na, m->af3.p, 1, Nl,
                                       nullptr, m->intmap2b.p + o * (nr + 1), m->alpha3b[k].p, Aa, m->emb3b[k].p,
                                       m->type_map.p, m->numtriplet.p + o, nt, nlocal, st);
      if (rc != STAF_OK) return gpu_failure(__LINE__, rc);
      m->tmp2.resize((size_t)Nl * Ar);
      m->tmp3.resize((size_t)Nl * Aa);
      STAF_HIP_OK(hipMemcpyAsync(m->tmp2.data(), m->af2.p, m->tmp2.size() * sizeof(double), hipMemcpyDeviceToHost, st));
      STAF_HIP_OK(hipMemcpyAsync(m->tmp3.data(), m->af3.p, m->tmp3.size() * sizeof(double), hipMemcpyDeviceToHost, st));
      STAF_HIP_OK(hipStreamSynchronize(st));
      for (int a = 0; a < Nl; a++) {
        double* row = &m->af_h[off + (size_t)a * (Ar + Aa)];
        memcpy(row, &m->tmp2[(size_t)a * Ar], Ar * sizeof(double));
        memcpy(row + Ar, &m->tmp3[(size_t)a * Aa], Aa * sizeof(double));
      }
      off += (size_t)Nl * (Ar + Aa);
    }

    // ---- MLP on the host (libstaf/vendor/jmd/nn_nn_mlp.cu:657-768): float32 nets see float32 fingerprints
    std::vector<int> n_af(nt);
    for (int k = 0; k < nt; k++) n_af[k] = m->Ar[k] + m->Aa[k];
    StafMlpEval ev;
    memset(&ev, 0, sizeof(ev));
    ev.n_type = nt;
    ev.n_atoms = tipos.data();
    ev.n_af = n_af.data();
    energy = 0.0;
    if (staf_mlp_precision(m->mlp) == 0) {
      m->af_f.resize(total);
      m->gr_f.assign(total, 0.f);
      for (size_t i = 0; i < total; i++) m->af_f[i] = (float)m->af_h[i];
      float e_f = 0.f;
      ev.af_f32 = m->af_f.data();
      ev.energy_f32 = &e_f;
      ev.dE_daf_f32 = m->gr_f.data();
      if (staf_mlp_eval(m->mlp, &ev) != 0) return gpu_failure(__LINE__, 0);
      energy = (double)e_f;
      for (size_t i = 0; i < total; i++) m->gr_h[i] = (double)m->gr_f[i];
    } else {
      ev.af_f64 = m->af_h.data();
      ev.energy_f64 = &energy;
      ev.dE_daf_f64 = m->gr_h.data();
      if (staf_mlp_eval(m->mlp, &ev) != 0) return gpu_failure(__LINE__, 0);
    }
    if (!isfinite(energy))
      fprintf(stderr, "staf_compute: non-finite energy=%g nlocal=%d nghost=%d\n", energy, nlocal, nghost);

    // ---- forces: 2-body + 3-body of every centre species, with the virial
    staf::launch_fill_zero<double>(d_force, nall * 3, st);
    double Wk[9];
    off = 0;
    shift = 0;
    for (int k = 0; k < nt; shift += tipos[k], k++) {
      const int Nl = tipos[k], Ar = m->Ar[k], Aa = m->Aa[k];
      if (Nl == 0) continue;
      const size_t o = (size_t)shift;
      m->tmp2.resize((size_t)Nl * Ar);
      m->tmp3.resize((size_t)Nl * Aa);
      for (int a = 0; a < Nl; a++) {
        const double* row = &m->gr_h[off + (size_t)a * (Ar + Aa)];
        memcpy(&m->tmp2[(size_t)a * Ar], row, Ar * sizeof(double));
        memcpy(&m->tmp3[(size_t)a * Aa], row + Ar, Aa * sizeof(double));
      }
      off += (size_t)Nl * (Ar + Aa);
      STAF_HIP_OK(hipMemcpyAsync(m->g2.p, m->tmp2.data(), m->tmp2.size() * sizeof(double), hipMemcpyHostToDevice, st));
      STAF_HIP_OK(hipMemcpyAsync(m->g3.p, m->tmp3.data(), m->tmp3.size() * sizeof(double), hipMemcpyHostToDevice, st));
      STAF_HIP_OK(hipStreamSynchronize(st));
      for (int body = 2; body <= 3; body++) {
        if (body == 2)
          rc = staf::force_doublets<double>(m->g2.p, m->raddescr.p + o * nr, m->der2b.p + o * 3 * nr,
                                            m->intmap2b.p + o * (nr + 1), nr, nall, 1, Ar, m->alpha2b[k].p,
                                            m->emb2b[k].p, nt, m->tipos.p, m->actual_type.p + k, m->force_op.p,
                                            m->type_map.p, Nl, m->virial_op.p, d_pos, d_box, nlocal, skip_pbc, st);
        else
          rc = staf::force_tripl<double>(m->g3.p, m->des3bsupp.p + o * nr, nullptr, m->der3bsupp.p + o * 3 * nr, nullptr,
                                         m->unit.p + o * 4 * nr, m->intmap2b.p + o * (nr + 1), nullptr, nr, na, nall, 1,
                                         Aa, m->emb3b[k].p, nt, m->tipos.p, m->actual_type.p + k, m->force_op.p,
                                         m->numtriplet.p + o, m->alpha3b[k].p, m->type_map.p, Nl, m->virial_op.p,
                                         d_pos, d_box, nlocal, skip_pbc, st);
        if (rc != STAF_OK) return gpu_failure(__LINE__, rc);
        hipLaunchKernelGGL(add_into_kernel, dim3((n3 + 255) / 256), dim3(256), 0, st, d_force, m->force_op.p, n3);
        STAF_HIP_OK(hipMemcpyAsync(Wk, m->virial_op.p, 9 * sizeof(double), hipMemcpyDeviceToHost, st));
        STAF_HIP_OK(hipStreamSynchronize(st));
        for (int c = 0; c < 9; c++) W[c] += Wk[c];
      }
    }
  }
  // forces, and on the device path the virial and the atomic energies behind them, in one copy
  const size_t n_back = m->dev_mlp ? n_out : (size_t)n3;
  STAF_HIP_OK(hipMemcpyAsync(m->out_h.p, m->out_d.p, n_back * sizeof(double), hipMemcpyDeviceToHost, st));
  const double* force_h = m->out_h.p;
  // the call's synchronisation: results are on the host, and so is what the kernels reported
  rc = staf_ops_poll_status(st);
  if (rc == STAF_E_RADIAL_OVERFLOW) return -10;
  if (rc == STAF_E_SCATTER_OVERFLOW) return -11;
  if (rc != STAF_OK) return gpu_failure(__LINE__, rc);
  if (m->dev_mlp) {
    const double* e_atom_h = m->out_h.p + (size_t)n3 + 9;
    for (int c = 0; c < 9; c++) W[c] = m->out_h.p[(size_t)n3 + c];
    for (int a = 0; a < nlocal; a++) energy += e_atom_h[a];   // slot order: fixed
    energy *= 0.5;
    if (!isfinite(energy))
      fprintf(stderr, "staf_compute: non-finite energy=%g nlocal=%d nghost=%d\n", energy, nlocal, nghost);
  }

  if (e_rank) *e_rank = energy;
  if (f)
    for (int s = 0; s < nall; s++) {
      const int i = m->slot_to_order[s];
      f[3 * i] = force_h[3 * s];
      f[3 * i + 1] = force_h[3 * s + 1];
      f[3 * i + 2] = force_h[3 * s + 2];
    }
  if (virial) {
    virial[0] = W[0];
    virial[1] = W[4];
    virial[2] = W[8];
    virial[3] = virial[4] = virial[5] = 0.0;   // the reference fills the diagonal only (staf_api.cpp:398-403)
    if (m->opt.reserved & 1) {
      virial[3] = 0.5 * (W[1] + W[3]);
      virial[4] = 0.5 * (W[2] + W[6]);
      virial[5] = 0.5 * (W[5] + W[7]);
    }
  }
  return 0;
}

}  // extern "C"
