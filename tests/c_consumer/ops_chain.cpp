// A caller of the op-level C ABI (include/staf_ops.h) that is neither Python nor torch: device memory from
// hipMalloc, one stream, every staf_op_*_f64 entry point in the order the reference's Python layers call the ops
// (STAF/source_routine/descriptor_builder.py:31-37, physics_layer_mod.py:33-46, force_layer_mod.py:24-42, then the
// gradient ops of STAF/gradient_utility/*.py), per centre species, on views of the descriptor outputs -- the way
// ComputeSortProjOp::Compute hands its tensors to radialAFs_Launcher (STAF/src/fingerprint/rad/reforce.cc:33-76).
//
//   ops_chain <fixture>      exit code 0: every output matches the expected arrays of the fixture
//
// The fixture is written by the test that runs this program (inputs, and the CPU oracle's outputs as expected
// values): a sequence of records  name[32] | kind int32 (0 = int32, 1 = float64) | count int64 | data.
// Integers must match exactly; float64 arrays within 1e-12 both in max|a-b|/max|b| and element-wise
// |a-b| <= 1e-12 (|b| + rms(b)).
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <map>
#include <string>
#include <vector>

#include "staf_ops.h"

namespace {

struct Array {
  int kind = 0;
  std::vector<int> i;
  std::vector<double> d;
};
std::map<std::string, Array> fx;

bool load_fixture(const char* path) {
  FILE* f = fopen(path, "rb");
  if (!f) return false;
  for (;;) {
    char name[32];
    int32_t kind;
    int64_t count;
    if (fread(name, 1, 32, f) != 32) break;
    if (fread(&kind, 4, 1, f) != 1 || fread(&count, 8, 1, f) != 1) { fclose(f); return false; }
    name[31] = 0;
    Array a;
    a.kind = kind;
    size_t got;
    if (kind == 0) { a.i.resize(count); got = fread(a.i.data(), 4, count, f); }
    else { a.d.resize(count); got = fread(a.d.data(), 8, count, f); }
    if ((int64_t)got != count) { fclose(f); return false; }
    fx[name] = std::move(a);
  }
  fclose(f);
  return !fx.empty();
}

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
  fprintf(stderr, "ops_chain: %s -> %s\n", #x, hipGetErrorString(e_)); exit(3); } } while (0)
#define STAF_CALL(x) do { int rc_ = (x); if (rc_ != STAF_OK) { \
  fprintf(stderr, "ops_chain: %s -> %d\n", #x, rc_); exit(4); } } while (0)

template <typename T>
T* dev_alloc(size_t n) {
  T* p = nullptr;
  HIP_OK(hipMalloc((void**)&p, (n ? n : 1) * sizeof(T)));
  return p;
}
const double* up_d(const std::string& name) {
  const Array& a = fx.at(name);
  double* p = dev_alloc<double>(a.d.size());
  HIP_OK(hipMemcpy(p, a.d.data(), a.d.size() * 8, hipMemcpyHostToDevice));
  return p;
}
const int* up_i(const std::string& name) {
  const Array& a = fx.at(name);
  int* p = dev_alloc<int>(a.i.size());
  HIP_OK(hipMemcpy(p, a.i.data(), a.i.size() * 4, hipMemcpyHostToDevice));
  return p;
}

int failures = 0;

void check_d(const std::string& name, const double* dev, size_t n) {
  const std::vector<double>& want = fx.at(name).d;
  if (want.size() != n) { printf("%-12s size %zu, expected %zu\n", name.c_str(), n, want.size()); failures++; return; }
  std::vector<double> got(n);
  HIP_OK(hipMemcpy(got.data(), dev, n * 8, hipMemcpyDeviceToHost));
  double mx = 0, md = 0, sq = 0;
  for (size_t e = 0; e < n; e++) { mx = fmax(mx, fabs(want[e])); md = fmax(md, fabs(got[e] - want[e])); sq += want[e] * want[e]; }
  const double rms = n ? sqrt(sq / n) : 0.0;
  double el = 0;
  for (size_t e = 0; e < n; e++) {
    const double den = fabs(want[e]) + rms;
    const double r = den > 0 ? fabs(got[e] - want[e]) / den : fabs(got[e] - want[e]);
    if (!(r <= el)) el = r;   // NaN lands here too
  }
  const double nerr = mx > 0 ? md / mx : md;
  const bool ok = nerr <= 1e-12 && el <= 1e-12;
  printf("%-12s %9zu doubles  max-norm error %.2e  element-wise %.2e  %s\n", name.c_str(), n, nerr, el, ok ? "ok" : "FAIL");
  if (!ok) failures++;
}

void check_i(const std::string& name, const int* dev, size_t n) {
  const std::vector<int>& want = fx.at(name).i;
  if (want.size() != n) { printf("%-12s size %zu, expected %zu\n", name.c_str(), n, want.size()); failures++; return; }
  std::vector<int> got(n);
  HIP_OK(hipMemcpy(got.data(), dev, n * 4, hipMemcpyDeviceToHost));
  size_t bad = 0;
  for (size_t e = 0; e < n; e++) bad += got[e] != want[e];
  printf("%-12s %9zu ints     %zu differ  %s\n", name.c_str(), n, bad, bad ? "FAIL" : "ok");
  if (bad) failures++;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc != 2 || !load_fixture(argv[1])) {
    fprintf(stderr, "usage: ops_chain <fixture>\n");
    return 2;
  }
  const std::vector<int>& dims = fx.at("dims").i;
  const int nf = dims[0], N = dims[1], nt = dims[2], nr = dims[3], na = dims[4];
  const int ntc = nt * (nt + 1) / 2;
  const std::vector<double>& geom = fx.at("geom").d;   // Rc, Rs, Ra
  const std::vector<int>& tipos_h = fx.at("tipos").i;
  HIP_OK(hipSetDevice(0));
  hipStream_t stream;
  HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));

  // ---- descriptor layer
  STAF_CALL(staf_op_construct_descriptors_light_f64(geom[0], nr, na, N, geom[1], geom[2], nf, nullptr));
  STAF_CALL(staf_op_descriptor_options(0, 1));   // der3b padding as 0, so that the whole tensor can be compared
  for (int (*init)(int) : {staf_op_init_force_radial, staf_op_init_grad_force_radial}) STAF_CALL(init(nr));
  for (int (*init)(int) : {staf_op_init_force_tripl, staf_op_init_grad_force_tripl}) STAF_CALL(init(na));
  const double* pos = up_d("pos");
  const double* box = up_d("box");
  const int* type_map = up_i("type_map");
  const int* tipos = up_i("tipos");
  const size_t A = (size_t)nf * N;
  double* rad = dev_alloc<double>(A * nr);
  double* ang = dev_alloc<double>(A * na);
  double* sup = dev_alloc<double>(A * nr);
  int* im2 = dev_alloc<int>(A * (nr + 1));
  int* im3 = dev_alloc<int>(A * 2 * na);
  double* d2 = dev_alloc<double>(A * 3 * nr);
  double* d3 = dev_alloc<double>(A * 6 * na);
  double* d3s = dev_alloc<double>(A * 3 * nr);
  int* ntr = dev_alloc<int>(A);
  STAF_CALL(staf_op_compute_descriptors_light_f64(pos, box, nf, N, rad, ang, sup, im2, im3, d2, d3, d3s, ntr, stream));
  HIP_OK(hipStreamSynchronize(stream));
  check_d("raddescr", rad, A * nr);
  check_d("angdescr", ang, A * na);
  check_d("des3bsupp", sup, A * nr);
  check_i("intmap2b", im2, A * (nr + 1));
  check_i("intmap3b", im3, A * 2 * na);
  check_d("der2b", d2, A * 3 * nr);
  check_d("der3b", d3, A * 6 * na);
  check_d("der3bsupp", d3s, A * 3 * nr);
  check_i("numtriplet", ntr, A);

  const double* Q = up_d("Q");
  // per species: the force ops' outputs and the slot forces, kept for the collecting launch after the loop
  std::vector<const double*> f2_of(nt), f3_of(nt), slots_of(nt), selfs_of(nt), both_slots_of(nt), both_selfs_of(nt);
  std::vector<const double*> a2_of(nt), e2_of(nt), a3_of(nt), e3_of(nt);
  int Ar_all = 0, Aa_all = 0;
  int first = 0;   // first atom of the centre species: its rows are views into the descriptor outputs (ld_atoms = N)
  for (int k = 0; k < nt; first += tipos_h[k], k++) {
    const int Nl = tipos_h[k];
    const std::string s = std::to_string(k);
    const int Ar = (int)fx.at("alpha2b_" + s).d.size() / nt;
    const int Aa = (int)fx.at("alpha3b_" + s).d.size() / (3 * ntc);
    const double* a2 = up_d("alpha2b_" + s);
    const double* e2 = up_d("emb2b_" + s);
    const double* a3 = up_d("alpha3b_" + s);
    const double* e3 = up_d("emb3b_" + s);
    const double* G2 = up_d("G2_" + s);
    const double* G3 = up_d("G3_" + s);
    const double* P2 = up_d("P2_" + s);
    const double* P3 = up_d("P3_" + s);
    const int actual_h = k;
    int* actual = dev_alloc<int>(1);
    HIP_OK(hipMemcpy(actual, &actual_h, 4, hipMemcpyHostToDevice));
    const double* radk = rad + (size_t)first * nr;
    const double* angk = ang + (size_t)first * na;
    const double* supk = sup + (size_t)first * nr;
    const int* im2k = im2 + (size_t)first * (nr + 1);
    const int* im3k = im3 + (size_t)first * 2 * na;
    const double* d2k = d2 + (size_t)first * 3 * nr;
    const double* d3k = d3 + (size_t)first * 6 * na;
    const double* d3sk = d3s + (size_t)first * 3 * nr;
    const int* ntrk = ntr + first;
    const size_t L = (size_t)nf * Nl;
    double* af2 = dev_alloc<double>(L * Ar);
    double* af3 = dev_alloc<double>(L * Aa);
    double* f2 = dev_alloc<double>((size_t)nf * 3 * N);
    double* f3 = dev_alloc<double>((size_t)nf * 3 * N);
    double* g2a = dev_alloc<double>(nt * Ar);
    double* g2e = dev_alloc<double>(nt * Ar);
    double* g3a = dev_alloc<double>(ntc * 3 * Aa);
    double* g3e = dev_alloc<double>(ntc * Aa);
    double* gf2n = dev_alloc<double>(L * Ar);
    double* gf2a = dev_alloc<double>(nt * Ar);
    double* gf2e = dev_alloc<double>(nt * Ar);
    double* gf3n = dev_alloc<double>(L * Aa);
    double* gf3a = dev_alloc<double>(ntc * 3 * Aa);
    double* gf3e = dev_alloc<double>(ntc * Aa);
    // physics layer
    STAF_CALL(staf_op_radial_afs_f64(radk, nr, a2, Ar, af2, nf, Nl, im2k, e2, type_map, nt, N, stream));
    STAF_CALL(staf_op_angular_afs_f64(supk, angk, nr, na, af3, nf, Nl, im3k, im2k, a3, Aa, e3, type_map, ntrk, nt, N,
                                      stream));
    // force layer
    STAF_CALL(staf_op_force_doublets_f64(G2, radk, d2k, im2k, nr, N, nf, Ar, a2, e2, nt, tipos, actual, f2, type_map,
                                         Nl, nullptr, nullptr, nullptr, N, stream));
    STAF_CALL(staf_op_force_tripl_f64(G3, supk, angk, d3sk, d3k, im2k, im3k, nr, na, N, nf, Aa, e3, nt, tipos, actual,
                                      f3, ntrk, a3, type_map, Nl, nullptr, nullptr, nullptr, N, stream));
    // registered gradients
    STAF_CALL(staf_op_alpha_dist_grad_f64(radk, nr, a2, Ar, g2a, nf, Nl, im2k, P2, e2, type_map, g2e, nt, N, stream));
    STAF_CALL(staf_op_alphagrad_ang_f64(supk, angk, nr, na, P3, nf, Nl, im3k, im2k, a3, Aa, g3a, e3, type_map, g3e,
                                        ntrk, ntc, nt, N, stream));
    STAF_CALL(staf_op_gradforce_2b_f64(Q, radk, nr, a2, Ar, d2k, im2k, nf, N, Nl, G2, e2, nt, type_map, tipos, actual,
                                       gf2n, gf2a, gf2e, nullptr, nullptr, nullptr, N, stream));
    STAF_CALL(staf_op_gradforce_tripl_f64(Q, G3, supk, angk, d3sk, d3k, im2k, im3k, nr, na, N, nf, Aa, e3, nt, tipos,
                                          actual, ntrk, a3, type_map, Nl, gf3n, gf3a, gf3e, nullptr, nullptr, nullptr,
                                          N, stream));
    // step-level entry points: both 3-body gradients in one pass; the 3-body force (alone, and with the 2-body pair
    // forces) left on the neighbour slots for staf_op_force_total
    double* fgn = dev_alloc<double>(L * Aa);
    double* fgaf = dev_alloc<double>(ntc * 3 * Aa);
    double* fgae = dev_alloc<double>(ntc * 3 * Aa);
    double* fge = dev_alloc<double>(ntc * Aa);
    double* slots = dev_alloc<double>(L * nr * 3);
    double* selfs = dev_alloc<double>(L * 3);
    double* both_slots = dev_alloc<double>(L * nr * 3);
    double* both_selfs = dev_alloc<double>(L * 3);
    STAF_CALL(staf_op_grads_tripl_fused_f64(Q, G3, P3, supk, angk, d3sk, d3k, im2k, im3k, nr, na, N, nf, Aa, e3, nt,
                                            tipos, actual, ntrk, a3, type_map, Nl, fgn, fgaf, fgae, fge, nullptr,
                                            nullptr, nullptr, N, stream));
    STAF_CALL(staf_op_force_tripl_slots_f64(G3, supk, angk, d3sk, d3k, im2k, im3k, nr, na, N, nf, Aa, e3, nt, tipos,
                                            actual, slots, selfs, ntrk, a3, type_map, Nl, N, stream));
    STAF_CALL(staf_op_forces_slots_f64(G3, G2, supk, angk, d3sk, d3k, radk, d2k, im2k, im3k, nr, na, N, nf, Aa, Ar, e3,
                                       a3, a2, e2, nt, tipos, actual, both_slots, both_selfs, ntrk, type_map, Nl, N,
                                       stream));
    a2_of[k] = a2, e2_of[k] = e2, a3_of[k] = a3, e3_of[k] = e3, Ar_all = Ar, Aa_all = Aa;
    f2_of[k] = f2, f3_of[k] = f3, slots_of[k] = slots, selfs_of[k] = selfs;
    both_slots_of[k] = both_slots, both_selfs_of[k] = both_selfs;
    HIP_OK(hipStreamSynchronize(stream));
    check_d("gf3n_" + s, fgn, L * Aa);
    check_d("gf3a_" + s, fgaf, ntc * 3 * Aa);
    check_d("g3a_" + s, fgae, ntc * 3 * Aa);
    check_d("g3e_" + s, fge, ntc * Aa);
    check_d("af2_" + s, af2, L * Ar);
    check_d("af3_" + s, af3, L * Aa);
    check_d("f2_" + s, f2, (size_t)nf * 3 * N);
    check_d("f3_" + s, f3, (size_t)nf * 3 * N);
    check_d("g2a_" + s, g2a, nt * Ar);
    check_d("g2e_" + s, g2e, nt * Ar);
    check_d("g3a_" + s, g3a, ntc * 3 * Aa);
    check_d("g3e_" + s, g3e, ntc * Aa);
    check_d("gf2n_" + s, gf2n, L * Ar);
    check_d("gf2a_" + s, gf2a, nt * Ar);
    check_d("gf2e_" + s, gf2e, nt * Ar);
    check_d("gf3n_" + s, gf3n, L * Aa);
    check_d("gf3a_" + s, gf3a, ntc * 3 * Aa);
    check_d("gf3e_" + s, gf3e, ntc * Aa);
  }
  // ---- descriptors and fingerprints of every species in one launch, into fresh tensors
  {
    double* rad1 = dev_alloc<double>(A * nr);
    double* ang1 = dev_alloc<double>(A * na);
    double* sup1 = dev_alloc<double>(A * nr);
    int* im21 = dev_alloc<int>(A * (nr + 1));
    int* im31 = dev_alloc<int>(A * 2 * na);
    double* d21 = dev_alloc<double>(A * 3 * nr);
    double* d31 = dev_alloc<double>(A * 6 * na);
    double* d3s1 = dev_alloc<double>(A * 3 * nr);
    int* ntr1 = dev_alloc<int>(A);
    std::vector<double*> af3_of(nt), af2_of(nt);
    for (int k = 0; k < nt; k++) {
      af3_of[k] = dev_alloc<double>((size_t)nf * tipos_h[k] * Aa_all);
      af2_of[k] = dev_alloc<double>((size_t)nf * tipos_h[k] * Ar_all);
    }
    STAF_CALL(staf_op_descriptors_fingerprints_f64(pos, box, nf, N, rad1, ang1, sup1, im21, im31, d21, d31, d3s1, ntr1,
                                                   nt, tipos_h.data(), 0, nt, type_map, Aa_all, a3_of.data(),
                                                   e3_of.data(), af3_of.data(), Ar_all, a2_of.data(), e2_of.data(),
                                                   af2_of.data(), stream));
    HIP_OK(hipStreamSynchronize(stream));
    check_d("raddescr", rad1, A * nr);
    check_d("angdescr", ang1, A * na);
    check_d("des3bsupp", sup1, A * nr);
    check_i("intmap2b", im21, A * (nr + 1));
    check_i("intmap3b", im31, A * 2 * na);
    check_d("der2b", d21, A * 3 * nr);
    check_d("der3b", d31, A * 6 * na);
    check_d("der3bsupp", d3s1, A * 3 * nr);
    check_i("numtriplet", ntr1, A);
    for (int k = 0; k < nt; k++) {
      check_d("af3_" + std::to_string(k), af3_of[k], (size_t)nf * tipos_h[k] * Aa_all);
      check_d("af2_" + std::to_string(k), af2_of[k], (size_t)nf * tipos_h[k] * Ar_all);
    }
  }
  // ---- the collecting launch: total force of the step from the slot forces of every centre species
  const size_t F = (size_t)nf * 3 * N;
  double* total = dev_alloc<double>(F);
  double* total_both = dev_alloc<double>(F);
  STAF_CALL(staf_op_force_total_f64(im2, nr, N, nf, nt, tipos_h.data(), slots_of.data(), selfs_of.data(),
                                    f2_of.data(), total, stream));
  STAF_CALL(staf_op_force_total_f64(im2, nr, N, nf, nt, tipos_h.data(), both_slots_of.data(), both_selfs_of.data(),
                                    nullptr, total_both, stream));
  HIP_OK(hipStreamSynchronize(stream));
  check_d("ftot", total, F);
  check_d("ftot", total_both, F);
  {
    // the same bits as the per-op force arrays added in the order f2[0], f3[0], f2[1], f3[1], ...
    std::vector<double> want(F), part(F), got(F);
    for (int k = 0; k < nt; k++)
      for (const double* src : {f2_of[k], f3_of[k]}) {
        HIP_OK(hipMemcpy(part.data(), src, F * 8, hipMemcpyDeviceToHost));
        const bool start = k == 0 && src == f2_of[0];
        for (size_t e = 0; e < F; e++) want[e] = start ? part[e] : want[e] + part[e];
      }
    HIP_OK(hipMemcpy(got.data(), total, F * 8, hipMemcpyDeviceToHost));
    size_t bad = 0;
    for (size_t e = 0; e < F; e++) bad += memcmp(&got[e], &want[e], 8) != 0;
    printf("%-12s %9zu doubles  %zu differ in bits from the per-op arrays added  %s\n", "ftot", F, bad,
           bad ? "FAIL" : "ok");
    if (bad) failures++;
  }
  staf_ops_release();
  printf("ops_chain: %s\n", failures ? "FAILED" : "OK");
  return failures ? 1 : 0;
}
