// TensorFlow custom-op shells over libstaf_hip.so: one shared object registers every op of the reference's
// STAF/src/**/reforce.cc (same op names, input order, dtypes and output shapes), and each Compute() only marshals
// tensors into the matching staf_op_* entry point of include/staf_ops.h.
//
// NOT built in this repository (no TensorFlow in the build image); it is the reference-side file a maintainer adds.
// Build one library per precision, like the reference's ops_float / ops_double trees (STAF/staf_paths.py:55-73):
//   hipcc -std=c++17 -shared -fPIC [-DSTAF_REAL_DOUBLE] staf_tf_ops.cc -o reforce.so \
//         $(python -c 'import tensorflow as tf; print(" ".join(tf.sysconfig.get_compile_flags()))') \
//         -I<repo>/include -L<repo>/alphanesgpu_amd/lib -lstaf_hip \
//         $(python -c 'import tensorflow as tf; print(" ".join(tf.sysconfig.get_link_flags()))')
// and point every entry of STAF/staf_paths.py at that one file (tf.load_op_library may load it once; all ops are in it).
//
// Per-species tensors arrive as tf.split copies, i.e. contiguous [nf, N_local, ...]: ld_atoms = N_local.
#define EIGEN_USE_GPU
#include <atomic>

#include "staf_ops.h"
#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/framework/shape_inference.h"

using namespace tensorflow;

#ifdef STAF_REAL_DOUBLE
using real = double;
#define STAF_TF_DTYPE "double"
#define STAF_FN(name) name##_f64
#else
using real = float;
#define STAF_TF_DTYPE "float"
#define STAF_FN(name) name##_f32
#endif

namespace {

// geometry of the last ConstructDescriptorsLight, needed for the output shapes of ComputeDescriptorsLight
std::atomic<int> g_nr{0}, g_na{0};

inline void* stream_of(OpKernelContext* c) { return (void*)c->eigen_device<Eigen::GpuDevice>().stream(); }
inline const real* R(OpKernelContext* c, int i) { return c->input(i).flat<real>().data(); }
inline const int* I(OpKernelContext* c, int i) { return c->input(i).flat<int32>().data(); }
inline int dim(OpKernelContext* c, int i, int d) { return (int)c->input(i).shape().dim_size(d); }

inline real* out_real(OpKernelContext* c, int i, std::initializer_list<int64_t> shape) {
  Tensor* t = nullptr;
  if (!c->allocate_output(i, TensorShape(shape), &t).ok()) return nullptr;
  return t->flat<real>().data();
}
inline int* out_int(OpKernelContext* c, int i, std::initializer_list<int64_t> shape) {
  Tensor* t = nullptr;
  if (!c->allocate_output(i, TensorShape(shape), &t).ok()) return nullptr;
  return t->flat<int32>().data();
}
inline int species_count(int nt_couple) {   // rows of alpha3b = nt (nt + 1) / 2
  int nt = 1;
  while (nt * (nt + 1) / 2 < nt_couple) ++nt;
  return nt;
}
#define STAF_CHECK(ctx, rc, what) \
  OP_REQUIRES(ctx, (rc) == STAF_OK, errors::Internal(what, " failed with STAF code ", (rc)))

}  // namespace

// ---- descriptor ops (STAF/src/descriptor_builder/reforce.cc:182-252) -------------------------------------------
REGISTER_OP("ConstructDescriptorsLight")
    .Input("radial_cutoff: " STAF_TF_DTYPE).Input("radial_buffer: int32").Input("angular_buffer: int32")
    .Input("numpar: int32").Input("boxer: " STAF_TF_DTYPE).Input("rs: " STAF_TF_DTYPE)
    .Input("ra: " STAF_TF_DTYPE).Input("max_batch: int32").Output("exitcode: int32");

class ConstructDescriptorsLightOp : public OpKernel {   // host op: scalars live in host memory
 public:
  explicit ConstructDescriptorsLightOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    auto sr = [&](int i) { return c->input(i).flat<real>()(0); };
    auto si = [&](int i) { return c->input(i).flat<int32>()(0); };
    const int rc = STAF_FN(staf_op_construct_descriptors_light)(sr(0), si(1), si(2), si(3), sr(5), sr(6), si(7),
                                                                "cutoff_curve.dat");
    STAF_CHECK(c, rc, "ConstructDescriptorsLight");
    g_nr = si(1);
    g_na = si(2);
    Tensor* code = nullptr;
    OP_REQUIRES_OK(c, c->allocate_output(0, TensorShape({1}), &code));
    code->flat<int32>()(0) = 0;
  }
};
REGISTER_KERNEL_BUILDER(Name("ConstructDescriptorsLight").Device(DEVICE_CPU), ConstructDescriptorsLightOp);

REGISTER_OP("ComputeDescriptorsLight")
    .Input("positions: " STAF_TF_DTYPE).Input("boxer: " STAF_TF_DTYPE)
    .Output("raddescr: " STAF_TF_DTYPE).Output("angdescr: " STAF_TF_DTYPE).Output("des3bsupp: " STAF_TF_DTYPE)
    .Output("intmap2b: int32").Output("intmap3b: int32").Output("der2b: " STAF_TF_DTYPE)
    .Output("der3b: " STAF_TF_DTYPE).Output("der3bsupp: " STAF_TF_DTYPE).Output("numtriplet: int32");

class ComputeDescriptorsLightOp : public OpKernel {
 public:
  explicit ComputeDescriptorsLightOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 1, 0), N = dim(c, 0, 1) / 3, nr = g_nr, na = g_na;
    OP_REQUIRES(c, nr > 0 && na > 0, errors::FailedPrecondition("ConstructDescriptorsLight has not run"));
    real* rad = out_real(c, 0, {nf, N, nr});
    real* ang = out_real(c, 1, {nf, N, na});
    real* sup = out_real(c, 2, {nf, N, nr});
    int* im2 = out_int(c, 3, {nf, N, nr + 1});
    int* im3 = out_int(c, 4, {nf, N, 2 * na});
    real* d2 = out_real(c, 5, {nf, N, 3, nr});
    real* d3 = out_real(c, 6, {nf, N, 3, 2 * na});
    real* d3s = out_real(c, 7, {nf, N, 3, nr});
    int* ntr = out_int(c, 8, {nf, N});
    OP_REQUIRES(c, rad && ang && sup && im2 && im3 && d2 && d3 && d3s && ntr,
                errors::ResourceExhausted("ComputeDescriptorsLight: output allocation"));
    // no set_tensor_to_zero launches: the library writes the zeros the reference's memsets leave
    const int rc = STAF_FN(staf_op_compute_descriptors_light)(R(c, 0), R(c, 1), nf, N, rad, ang, sup, im2, im3, d2,
                                                              d3, d3s, ntr, stream_of(c));
    // the reference ends the process on a full neighbour buffer (reforce.cc:329-337); here the step fails cleanly
    STAF_CHECK(c, rc, "ComputeDescriptorsLight");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeDescriptorsLight").Device(DEVICE_GPU), ComputeDescriptorsLightOp);

// ---- fingerprints (fingerprint/rad/reforce.cc:13-19, fingerprint/ang/reforce.cc:15-24) ---------------------------
REGISTER_OP("ComputeSortProj")
    .Input("radial_descriptor: " STAF_TF_DTYPE).Input("interaction_map_rad: int32")
    .Input("alpha2b_parameters: " STAF_TF_DTYPE).Input("type_emb2b_parameters: " STAF_TF_DTYPE)
    .Input("type_map: int32").Output("two_body_afs: " STAF_TF_DTYPE);

class ComputeSortProjOp : public OpKernel {
 public:
  explicit ComputeSortProjOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 0, 0), Nl = dim(c, 0, 1), nr = dim(c, 0, 2), nt = dim(c, 2, 0), Ar = dim(c, 2, 1);
    real* out = out_real(c, 0, {nf, Nl, Ar});
    OP_REQUIRES(c, out || nf * Nl * Ar == 0, errors::ResourceExhausted("ComputeSortProj: output allocation"));
    STAF_CHECK(c, STAF_FN(staf_op_radial_afs)(R(c, 0), nr, R(c, 2), Ar, out, nf, Nl, I(c, 1), R(c, 3), I(c, 4), nt,
                                              Nl, stream_of(c)),
               "ComputeSortProj");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeSortProj").Device(DEVICE_GPU), ComputeSortProjOp);

REGISTER_OP("ComputeSortProj3body")
    .Input("angular_descriptor: " STAF_TF_DTYPE).Input("radial_descriptor: " STAF_TF_DTYPE)
    .Input("interaction_map_angular: int32").Input("interaction_map_rad: int32")
    .Input("alpha3b_parameters: " STAF_TF_DTYPE).Input("type_emb3b_parameters: " STAF_TF_DTYPE)
    .Input("type_map: int32").Input("num_triplet: int32").Output("three_body_afs: " STAF_TF_DTYPE);

class ComputeSortProj3bodyOp : public OpKernel {
 public:
  explicit ComputeSortProj3bodyOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 0, 0), Nl = dim(c, 0, 1), na = dim(c, 0, 2), nr = dim(c, 1, 2);
    const int ntc = dim(c, 4, 0), Aa = dim(c, 4, 1) / 3;
    real* out = out_real(c, 0, {nf, Nl, Aa});
    OP_REQUIRES(c, out || nf * Nl * Aa == 0, errors::ResourceExhausted("ComputeSortProj3body: output allocation"));
    STAF_CHECK(c, STAF_FN(staf_op_angular_afs)(R(c, 1), R(c, 0), nr, na, out, nf, Nl, I(c, 2), I(c, 3), R(c, 4), Aa,
                                               R(c, 5), I(c, 6), I(c, 7), species_count(ntc), Nl, stream_of(c)),
               "ComputeSortProj3body");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeSortProj3body").Device(DEVICE_GPU), ComputeSortProj3bodyOp);

// ---- Init* ops: the reference picks a CUDA block size there; nothing to pick here, the ops stay for the graphs
// that call them (force/rad/reforce.cc:13-36 and its three siblings) ------------------------------------------------
#define STAF_INIT_OP(OPNAME, FN)                                                              \
  REGISTER_OP(#OPNAME).Input("buffdim: int32").Output("code: int32");                         \
  class OPNAME##Op : public OpKernel {                                                        \
   public:                                                                                    \
    explicit OPNAME##Op(OpKernelConstruction* c) : OpKernel(c) {}                             \
    void Compute(OpKernelContext* c) override {                                               \
      STAF_CHECK(c, FN(c->input(0).flat<int32>()(0)), #OPNAME);                               \
      Tensor* code = nullptr;                                                                 \
      OP_REQUIRES_OK(c, c->allocate_output(0, TensorShape({1}), &code));                      \
      code->flat<int32>()(0) = 0;                                                             \
    }                                                                                         \
  };                                                                                          \
  REGISTER_KERNEL_BUILDER(Name(#OPNAME).Device(DEVICE_CPU), OPNAME##Op);
STAF_INIT_OP(InitForceRadial, staf_op_init_force_radial)
STAF_INIT_OP(InitForceTripl, staf_op_init_force_tripl)
STAF_INIT_OP(InitGradForceRadial, staf_op_init_grad_force_radial)
STAF_INIT_OP(InitGradForceTripl, staf_op_init_grad_force_tripl)

// ---- force ops and their virial forms (force/rad/reforce.cc:39-49,133-146; force/ang/reforce.cc:44-58,159-176) ---
#define STAF_FORCE2_INPUTS                                                                                  \
  .Input("netderiv: " STAF_TF_DTYPE).Input("descriptor_derivative_rad: " STAF_TF_DTYPE)                     \
  .Input("interaction_map_rad: int32").Input("radial_descriptor: " STAF_TF_DTYPE)                           \
  .Input("alpha2b_parameters: " STAF_TF_DTYPE).Input("type_emb2b_parameters: " STAF_TF_DTYPE)               \
  .Input("type_map: int32").Input("tipos: int32").Input("actual_type: int32")
REGISTER_OP("ComputeForceRadial") STAF_FORCE2_INPUTS.Output("force: " STAF_TF_DTYPE);
REGISTER_OP("ComputeForceRadialVirial") STAF_FORCE2_INPUTS.Input("pos: " STAF_TF_DTYPE).Input("box: " STAF_TF_DTYPE)
    .Output("force: " STAF_TF_DTYPE).Output("virial: " STAF_TF_DTYPE);

template <bool VIRIAL>
class ComputeForceRadialOp : public OpKernel {
 public:
  explicit ComputeForceRadialOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 0, 0), Nl = dim(c, 0, 1), Ar = dim(c, 0, 2), nr = dim(c, 3, 2);
    const int nt = dim(c, 4, 0), N = dim(c, 6, 0);
    real* force = out_real(c, 0, {nf, 3 * N});
    real* W = VIRIAL ? out_real(c, 1, {nf, 9}) : nullptr;
    OP_REQUIRES(c, force && (W || !VIRIAL), errors::ResourceExhausted("ComputeForceRadial: output allocation"));
    STAF_CHECK(c, STAF_FN(staf_op_force_doublets)(R(c, 0), R(c, 3), R(c, 1), I(c, 2), nr, N, nf, Ar, R(c, 4), R(c, 5),
                                                  nt, I(c, 7), I(c, 8), force, I(c, 6), Nl, W,
                                                  VIRIAL ? R(c, 9) : nullptr, VIRIAL ? R(c, 10) : nullptr, Nl,
                                                  stream_of(c)),
               "ComputeForceRadial");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeForceRadial").Device(DEVICE_GPU), ComputeForceRadialOp<false>);
REGISTER_KERNEL_BUILDER(Name("ComputeForceRadialVirial").Device(DEVICE_GPU), ComputeForceRadialOp<true>);

#define STAF_FORCE3_INPUTS                                                                                  \
  .Input("netderiv: " STAF_TF_DTYPE).Input("radial_descriptor: " STAF_TF_DTYPE)                             \
  .Input("angular_descriptor: " STAF_TF_DTYPE).Input("descriptor_derivative_rad: " STAF_TF_DTYPE)           \
  .Input("descriptor_derivative_ang: " STAF_TF_DTYPE).Input("interaction_map_rad: int32")                   \
  .Input("interaction_map_ang: int32").Input("alpha3b_parameters: " STAF_TF_DTYPE)                          \
  .Input("type_emb3b_parameters: " STAF_TF_DTYPE).Input("type_map: int32").Input("tipos: int32")            \
  .Input("actual_type: int32").Input("num_triplets: int32")
REGISTER_OP("ComputeForceTripl") STAF_FORCE3_INPUTS.Output("force: " STAF_TF_DTYPE);
REGISTER_OP("ComputeForceTriplVirial") STAF_FORCE3_INPUTS.Input("pos: " STAF_TF_DTYPE).Input("box: " STAF_TF_DTYPE)
    .Output("force: " STAF_TF_DTYPE).Output("virial: " STAF_TF_DTYPE);

template <bool VIRIAL>
class ComputeForceTriplOp : public OpKernel {
 public:
  explicit ComputeForceTriplOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 0, 0), Nl = dim(c, 0, 1), Aa = dim(c, 0, 2), nr = dim(c, 1, 2), na = dim(c, 2, 2);
    const int nt = species_count(dim(c, 7, 0)), N = dim(c, 9, 0);
    real* force = out_real(c, 0, {nf, 3 * N});
    real* W = VIRIAL ? out_real(c, 1, {nf, 9}) : nullptr;
    OP_REQUIRES(c, force && (W || !VIRIAL), errors::ResourceExhausted("ComputeForceTripl: output allocation"));
    STAF_CHECK(c, STAF_FN(staf_op_force_tripl)(R(c, 0), R(c, 1), R(c, 2), R(c, 3), R(c, 4), I(c, 5), I(c, 6), nr, na,
                                               N, nf, Aa, R(c, 8), nt, I(c, 10), I(c, 11), force, I(c, 12), R(c, 7),
                                               I(c, 9), Nl, W, VIRIAL ? R(c, 13) : nullptr,
                                               VIRIAL ? R(c, 14) : nullptr, Nl, stream_of(c)),
               "ComputeForceTripl");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeForceTripl").Device(DEVICE_GPU), ComputeForceTriplOp<false>);
REGISTER_KERNEL_BUILDER(Name("ComputeForceTriplVirial").Device(DEVICE_GPU), ComputeForceTriplOp<true>);

// ---- parameter gradients of the fingerprint ops (grad_finger/rad/reforce.cc:14-22, grad_finger/ang/reforce.cc:12-23)
REGISTER_OP("ComputeTwoBodyParGrad")
    .Input("prev_grad: " STAF_TF_DTYPE).Input("radial_descriptor: " STAF_TF_DTYPE)
    .Input("interaction_map_rad: int32").Input("alpha2b_parameters: " STAF_TF_DTYPE)
    .Input("type_emb2b_parameters: " STAF_TF_DTYPE).Input("type_map: int32")
    .Output("nextgrad_alpha2b: " STAF_TF_DTYPE).Output("nextgrad_emb2b: " STAF_TF_DTYPE);

class ComputeTwoBodyParGradOp : public OpKernel {
 public:
  explicit ComputeTwoBodyParGradOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 1, 0), Nl = dim(c, 1, 1), nr = dim(c, 1, 2), nt = dim(c, 3, 0), Ar = dim(c, 3, 1);
    real* ga = out_real(c, 0, {nt, Ar});
    real* ge = out_real(c, 1, {nt, Ar});
    OP_REQUIRES(c, ga && ge, errors::ResourceExhausted("ComputeTwoBodyParGrad: output allocation"));
    STAF_CHECK(c, STAF_FN(staf_op_alpha_dist_grad)(R(c, 1), nr, R(c, 3), Ar, ga, nf, Nl, I(c, 2), R(c, 0), R(c, 4),
                                                   I(c, 5), ge, nt, Nl, stream_of(c)),
               "ComputeTwoBodyParGrad");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeTwoBodyParGrad").Device(DEVICE_GPU), ComputeTwoBodyParGradOp);

REGISTER_OP("ComputeSortProj3bodyGrad")
    .Input("previous_gradient: " STAF_TF_DTYPE).Input("angular_desciptors: " STAF_TF_DTYPE)
    .Input("radial_descriptors: " STAF_TF_DTYPE).Input("intmap3b: int32").Input("intmap2b: int32")
    .Input("alpha3b_parameters: " STAF_TF_DTYPE).Input("type_emb3b: " STAF_TF_DTYPE).Input("type_map: int32")
    .Input("num_triplets: int32")
    .Output("alphagrad3body: " STAF_TF_DTYPE).Output("nextgrad_emb3b: " STAF_TF_DTYPE);

class ComputeSortProj3bodyGradOp : public OpKernel {
 public:
  explicit ComputeSortProj3bodyGradOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    const int nf = dim(c, 1, 0), Nl = dim(c, 1, 1), na = dim(c, 1, 2), nr = dim(c, 2, 2);
    const int ntc = dim(c, 5, 0), Aa = dim(c, 5, 1) / 3;
    real* ga = out_real(c, 0, {ntc, 3 * Aa});
    real* ge = out_real(c, 1, {ntc, Aa});
    OP_REQUIRES(c, ga && ge, errors::ResourceExhausted("ComputeSortProj3bodyGrad: output allocation"));
    STAF_CHECK(c, STAF_FN(staf_op_alphagrad_ang)(R(c, 2), R(c, 1), nr, na, R(c, 0), nf, Nl, I(c, 3), I(c, 4), R(c, 5),
                                                 Aa, ga, R(c, 6), I(c, 7), ge, I(c, 8), ntc, species_count(ntc), Nl,
                                                 stream_of(c)),
               "ComputeSortProj3bodyGrad");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeSortProj3bodyGrad").Device(DEVICE_GPU), ComputeSortProj3bodyGradOp);

// ---- gradients of the force ops (grad_force/rad/reforce.cc:42-55,160-176; grad_force/ang/reforce.cc:39-56,186-206)
// The virial forms carry prevgrad_virial as their second input, so the remaining inputs sit one place further on.
#define STAF_GRADFORCE2_TAIL                                                                                \
  .Input("netderiv: " STAF_TF_DTYPE).Input("descriptor_derivative_rad: " STAF_TF_DTYPE)                     \
  .Input("interaction_map_rad: int32").Input("radial_descriptor: " STAF_TF_DTYPE)                           \
  .Input("alpha2b_parameters: " STAF_TF_DTYPE).Input("type_emb2b_parameters: " STAF_TF_DTYPE)               \
  .Input("type_map: int32").Input("tipos: int32").Input("actual_type: int32")
#define STAF_GRADFORCE2_OUT \
  .Output("gradnet: " STAF_TF_DTYPE).Output("grad_alpha2b: " STAF_TF_DTYPE).Output("grad_emb2b: " STAF_TF_DTYPE)
REGISTER_OP("ComputeForceRadialGrad").Input("prevgrad: " STAF_TF_DTYPE) STAF_GRADFORCE2_TAIL STAF_GRADFORCE2_OUT;
REGISTER_OP("ComputeForceRadialVirialGrad").Input("prevgrad: " STAF_TF_DTYPE)
    .Input("prevgrad_virial: " STAF_TF_DTYPE) STAF_GRADFORCE2_TAIL
    .Input("pos: " STAF_TF_DTYPE).Input("box: " STAF_TF_DTYPE) STAF_GRADFORCE2_OUT;

template <bool VIRIAL>
class ComputeForceRadialGradOp : public OpKernel {
 public:
  explicit ComputeForceRadialGradOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    constexpr int o = VIRIAL ? 1 : 0;   // shift of the inputs behind prevgrad
    const int nf = dim(c, 1 + o, 0), Nl = dim(c, 1 + o, 1), Ar = dim(c, 1 + o, 2), nr = dim(c, 4 + o, 2);
    const int nt = dim(c, 5 + o, 0), N = dim(c, 7 + o, 0);
    real* gn = out_real(c, 0, {nf, Nl, Ar});
    real* ga = out_real(c, 1, {nt, Ar});
    real* ge = out_real(c, 2, {nt, Ar});
    OP_REQUIRES(c, ga && ge && (gn || nf * Nl == 0), errors::ResourceExhausted("ComputeForceRadialGrad: outputs"));
    STAF_CHECK(c, STAF_FN(staf_op_gradforce_2b)(R(c, 0), R(c, 4 + o), nr, R(c, 5 + o), Ar, R(c, 2 + o), I(c, 3 + o),
                                                nf, N, Nl, R(c, 1 + o), R(c, 6 + o), nt, I(c, 7 + o), I(c, 8 + o),
                                                I(c, 9 + o), gn, ga, ge, VIRIAL ? R(c, 1) : nullptr,
                                                VIRIAL ? R(c, 11) : nullptr, VIRIAL ? R(c, 12) : nullptr, Nl,
                                                stream_of(c)),
               "ComputeForceRadialGrad");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeForceRadialGrad").Device(DEVICE_GPU), ComputeForceRadialGradOp<false>);
REGISTER_KERNEL_BUILDER(Name("ComputeForceRadialVirialGrad").Device(DEVICE_GPU), ComputeForceRadialGradOp<true>);

#define STAF_GRADFORCE3_OUT \
  .Output("gradnet: " STAF_TF_DTYPE).Output("gradalpha: " STAF_TF_DTYPE).Output("gradck: " STAF_TF_DTYPE)
REGISTER_OP("ComputeForceTriplGrad").Input("prevgrad: " STAF_TF_DTYPE) STAF_FORCE3_INPUTS STAF_GRADFORCE3_OUT;
REGISTER_OP("ComputeForceTriplVirialGrad").Input("prevgrad: " STAF_TF_DTYPE)
    .Input("prevgrad_virial: " STAF_TF_DTYPE) STAF_FORCE3_INPUTS
    .Input("pos: " STAF_TF_DTYPE).Input("box: " STAF_TF_DTYPE) STAF_GRADFORCE3_OUT;

template <bool VIRIAL>
class ComputeForceTriplGradOp : public OpKernel {
 public:
  explicit ComputeForceTriplGradOp(OpKernelConstruction* c) : OpKernel(c) {}
  void Compute(OpKernelContext* c) override {
    constexpr int o = VIRIAL ? 2 : 1;   // first input of the STAF_FORCE3_INPUTS block (netderiv)
    const int nf = dim(c, o, 0), Nl = dim(c, o, 1), Aa = dim(c, o, 2), nr = dim(c, o + 1, 2), na = dim(c, o + 2, 2);
    const int ntc = dim(c, o + 7, 0), nt = species_count(ntc), N = dim(c, o + 9, 0);
    real* gn = out_real(c, 0, {nf, Nl, Aa});
    real* ga = out_real(c, 1, {ntc, 3 * Aa});
    real* ge = out_real(c, 2, {ntc, Aa});
    OP_REQUIRES(c, ga && ge && (gn || nf * Nl == 0), errors::ResourceExhausted("ComputeForceTriplGrad: outputs"));
    STAF_CHECK(c, STAF_FN(staf_op_gradforce_tripl)(R(c, 0), R(c, o), R(c, o + 1), R(c, o + 2), R(c, o + 3), R(c, o + 4),
                                                   I(c, o + 5), I(c, o + 6), nr, na, N, nf, Aa, R(c, o + 8), nt,
                                                   I(c, o + 10), I(c, o + 11), I(c, o + 12), R(c, o + 7), I(c, o + 9),
                                                   Nl, gn, ga, ge, VIRIAL ? R(c, 1) : nullptr,
                                                   VIRIAL ? R(c, o + 13) : nullptr, VIRIAL ? R(c, o + 14) : nullptr,
                                                   Nl, stream_of(c)),
               "ComputeForceTriplGrad");
  }
};
REGISTER_KERNEL_BUILDER(Name("ComputeForceTriplGrad").Device(DEVICE_GPU), ComputeForceTriplGradOp<false>);
REGISTER_KERNEL_BUILDER(Name("ComputeForceTriplVirialGrad").Device(DEVICE_GPU), ComputeForceTriplGradOp<true>);
