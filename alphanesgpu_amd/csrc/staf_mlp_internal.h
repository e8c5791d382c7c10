// Library-internal view of a loaded StafMlp (staf_mlp.cpp): layer shapes and host pointers to the weights in the
// model's precision (float for precision 0, double for 1).  W is [in_f, out_f] row-major.  Activation codes:
// 0 linear, 1 tanh, 2 relu (the codes of the "STAFMLP1" file, libstaf/src/mlp/staf_mlp_ort.cc:99-165).
#pragma once
#include "../../include/staf_mlp.h"

#ifdef __cplusplus
extern "C" {
#endif
int staf_mlp_internal_nlayers(const StafMlp* mlp, int type);
const void* staf_mlp_internal_mu(const StafMlp* mlp, int type);
int staf_mlp_internal_layer(const StafMlp* mlp, int type, int layer, int* act, int* in_f, int* out_f, const void** W,
                            const void** b);
#ifdef __cplusplus
}
#endif
