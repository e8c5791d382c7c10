/* staf.h -- C API of the MD-facing entry of libstaf_hip.so (LAMMPS `pair_style staf`, standalone MD).
 *
 * Binary-compatible with the reference's libstaf/include/staf.h:20-61: same type layouts, enum values, function
 * names, argument meaning and return codes, so lammps/USER-STAF/pair_staf.cpp links against it unchanged.
 * (The function is still called staf_cuda_set_device because that is the symbol the callers bind; it selects a
 * HIP device.)
 */
#ifndef STAF_H
#define STAF_H

#ifdef __cplusplus
extern "C" {
#endif

typedef struct StafModel StafModel;

typedef enum StafMlpBackend {
  STAF_MLP_ORT = 0,    /* reference default (ONNX Runtime).  Not available here: served by the native Dense
                          evaluation of mlp_type{k}.bin, the reference's own fallback path */
  STAF_MLP_TF_C = 1,   /* legacy SavedModel in the reference; treated like STAF_MLP_NATIVE */
  STAF_MLP_NATIVE = 2  /* Dense stack read from mlp_type{k}.bin ("STAFMLP1") */
} StafMlpBackend;

typedef struct StafOptions {
  StafMlpBackend mlp_backend;
  int device_id;  /* GPU of this rank; taken modulo the device count */
  int precision;  /* 0 = the MLP runs in float32, 1 = float64 (descriptors, fingerprints, forces: always float64) */
  int reserved;   /* bit 0 set: fill all six virial components (reference: diagonal only, off-diagonals 0);
                   * bit 1 set: evaluate the MLP on the host between the kernels (default: on the GPU);
                   * bit 2 set: launch every kernel of every call eagerly (default: once a shape -- same atom counts
                   *            per species, same list mode -- has come twice in a row, more often if shapes change
                   *            every few calls, the call's kernel sequence is recorded as a HIP graph and replayed) */
} StafOptions;

/* Defaults of the reference (libstaf/src/staf_api.cpp:39-45): ORT backend, device 0, float32 MLP. */
void staf_options_default(StafOptions* opt);

/* Selects the GPU for this process.  Returns the device id actually selected (device_id modulo the number of
 * devices, negative ids -> 0) or -1 when no device is usable (libstaf/src/staf_api.cpp:47-68). */
int staf_cuda_set_device(int device_id);

/* Loads a model directory: type.dat, type{k}_alpha_{2,3}body.dat, type{k}_type_emb_{2b,3b}[_sq].dat,
 * mlp_type{k}.bin, optional staf_jmd.cfg (buffers and cutoffs; the reference's defaults otherwise).
 * Returns NULL on failure (libstaf/src/staf_api.cpp:70-107). */
StafModel* staf_load(const char* model_dir, const StafOptions* opt);

/* Energy, forces and virial of one configuration (libstaf/src/staf_api.cpp:192-412).
 *   nall = nlocal + nghost; x [nall*3] Cartesian; box [6] = {Lx, xy, xz, Ly, yz, Lz}; type [nall] 0-based.
 *   howmany/with == NULL: the library builds its own minimum-image neighbour list over the nlocal atoms
 *   (nghost is ignored).  Otherwise howmany [nlocal] and with [nlocal*maxneigh] give, for every owned atom, its
 *   neighbours sorted by distance as indices into x (0..nall-1); ghosts carry their periodic image in x, and no
 *   minimum-image wrap is applied.
 *   e_rank: 1/2 sum of the atomic energies of the owned atoms; f [nall*3] (ghost entries are the forces to be
 *   reverse-communicated); virial [6] = xx yy zz xy xz yz.
 * Returns 0, or: -1 null model / allocation, -3 nlocal <= 0, -4 model files unreadable, -7 zero box diagonal,
 * -8 species out of range, -9 neighbour index out of range, -10 more neighbours than the radial buffer,
 * -11 (this library only) an atom of a caller's list is named by more than 4 x the radial buffer centres, which
 * no list cut at the model's cutoff can hold while -10 does not occur, -20 GPU runtime failure.  (-2 and -5 of the
 * reference, "built without engine" and "cwd", cannot occur.) */
int staf_compute(StafModel* m, int nlocal, int nghost, const double* x, const double* box, const int* type,
                 const int* howmany, const int* with, int maxneigh, double* e_rank, double* f, double* virial);

void staf_free(StafModel* m);

#ifdef __cplusplus
}
#endif
#endif /* STAF_H */
