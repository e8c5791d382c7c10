// Device-resident per-species MLP of the MD entry (staf_mlp_dev.hip).
#pragma once
#include "staf_common.hpp"
#include "staf_mlp_internal.h"

namespace staf {

constexpr int DEV_MLP_MAX_LAYERS = 8;

struct DevMlpNet {
  int precision = 0;   // 0: float weights and arithmetic, 1: double
  int nl = 0, n_af = 0, tot = 0, maxw = 0;
  int act[DEV_MLP_MAX_LAYERS] = {0}, in_f[DEV_MLP_MAX_LAYERS] = {0}, out_f[DEV_MLP_MAX_LAYERS] = {0};
  void* W[DEV_MLP_MAX_LAYERS] = {nullptr};
  void* Wt[DEV_MLP_MAX_LAYERS] = {nullptr};
  void* b[DEV_MLP_MAX_LAYERS] = {nullptr};
  void* mu = nullptr;
  bool matrix_path = false;   // the matrix-core kernel can hold this stack (LDS), else the vector kernel runs
};

bool dev_mlp_upload(const StafMlp* mlp, int type, DevMlpNet* net, hipStream_t stream);   // false: not representable (fall back to host)
void dev_mlp_free(DevMlpNet* net);
// af2 [Nl, Ar], af3 [Nl, Aa] (float64 fingerprints) -> atomic energies e_atom [Nl] and d sum(e) / d af split into
// g2 [Nl, Ar], g3 [Nl, Aa] (float64; computed in the network's precision like the host evaluation).
int dev_mlp_eval(const DevMlpNet& net, const double* af2, int Ar, const double* af3, int Aa, int Nl, double* e_atom,
                 double* g2, double* g3, hipStream_t stream);

}  // namespace staf
