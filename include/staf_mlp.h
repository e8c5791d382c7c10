/* staf_mlp.h -- per-species MLP plug-in: fingerprints -> energy and d(energy)/d(fingerprint).
 *
 * Same interface as the reference's libstaf/include/staf_mlp.h:19-41.  Convention (":13" there):
 * energy = 0.5 * sum(atomic energies), dE_daf = d(sum of atomic energies)/d(af).
 * This build evaluates the Dense stack of mlp_type{k}.bin natively (libstaf/src/mlp/staf_mlp_ort.cc:99-233).
 */
#ifndef STAF_MLP_H
#define STAF_MLP_H

#ifdef __cplusplus
extern "C" {
#endif

#include "staf.h"

typedef struct StafMlp StafMlp;

typedef struct StafMlpEval {
  int n_type;
  const int* n_atoms;      /* [n_type] */
  const int* n_af;         /* [n_type] */
  const float* af_f32;     /* packed per type: type 0 atoms, then type 1, ...; rows [n_atoms_k, n_af_k] */
  const double* af_f64;
  float* energy_f32;       /* [1], all types */
  double* energy_f64;
  float* dE_daf_f32;       /* packed like af */
  double* dE_daf_f64;
} StafMlpEval;

StafMlp* staf_mlp_create(StafMlpBackend backend, const char* model_dir, int precision, int device_id);
int staf_mlp_eval(StafMlp* mlp, StafMlpEval* io);
void staf_mlp_destroy(StafMlp* mlp);
int staf_mlp_ntypes(const StafMlp* mlp);
int staf_mlp_n_af(const StafMlp* mlp, int type);
int staf_mlp_precision(const StafMlp* mlp); /* 0 = float32, 1 = float64 */

#ifdef __cplusplus
}
#endif
#endif /* STAF_MLP_H */
