/* staf_ops.h -- C ABI of libstaf_hip.so: the STAF fingerprint hot path on MI355X (gfx950).
 *
 * One entry point per launcher the reference's TensorFlow op shells call
 * (device pointers + integer dims + one stream).  Each entry point exists
 * twice, suffixed _f32 and _f64 (the reference builds one .so per precision
 * with -DSTAF_REAL_DOUBLE); `real` below stands for float / double.
 *
 * Conventions
 *   - all tensor pointers are DEVICE pointers, row-major, caller-owned;
 *     outputs are pre-allocated by the caller and fully written by the call
 *     (no pre-zeroing needed), except where a note says "padding".
 *   - `stream` is a hipStream_t passed as void* (NULL = default stream).
 *   - return value: 0 on success, a negative STAF_E_* code otherwise.  No
 *     entry point ever calls exit().
 *   - per-species ops take tensors sliced to one centre species, [nf, Nl, ...].
 *     `ld_atoms` is the distance, in atoms, between consecutive frames of the
 *     descriptor-derived tensors of the call (raddescr, des3bsupp, angdescr,
 *     der2b, der3bsupp, der3b, intmap2b, intmap3b, numtriplet): Nl (or 0) for
 *     the contiguous tensors tf.split produces, N when the pointers are views
 *     into the descriptor op's [nf, N, ...] outputs (pointer pre-offset to the
 *     species' first atom).  Channel-width tensors (fingerprints, netderiv,
 *     prevgrad of the fingerprint ops, gradnet outputs) are always contiguous
 *     [nf, Nl, channels].
 *   - type_map [N] int32 species of every atom of a frame; tipos [nt] int32
 *     atoms per species; actual_type [1] int32 centre species -- device
 *     pointers, as the reference ops receive them.
 *   - type-embedding arguments are the SQUARED embeddings (the reference's
 *     Python layers square them before the op call).
 *   - N_local = 0 (a species with no atom in these frames) is a valid call of
 *     the per-species ops: fingerprint ops write nothing, force ops fill force
 *     (and virial) with zeros, gradient ops fill the parameter gradients with
 *     zeros; the other pointers are not read.
 *   - state is per device.  Work areas are kept per stream, so calls issued on
 *     different streams of a device may overlap; calls on one stream are ordered.
 *     Error words are per stream too (the first 63 streams that use a device
 *     get their own, later ones share one): the synchronising return of an op
 *     reports what its own stream raised; staf_ops_poll_status reports what
 *     any stream of the device raised.
 *   - the force ops are owner-computes: every atom collects the pair forces of
 *     the slots that list it.  The descriptor op remembers, by address, the
 *     intmap2b tensors it has written (the 8 most recent per device); such a
 *     map is symmetric (i lists j exactly when j lists i), so a force op whose
 *     interaction_map_rad points into one (ld_atoms = N) finds the slots that
 *     list an atom from the atom's own row.  The tensor must then still hold
 *     what the descriptor op wrote (a broken pairing is reported as
 *     STAF_E_STALE_MAP).  Any other copy of the map (tf.split output,
 *     ld_atoms = N_local) is transposed by the force op itself, at the price of
 *     two more launches.
 *   - graph capture: every entry point may be captured once the same call (same
 *     shapes, same stream, same output tensors for the descriptor op) has run
 *     eagerly, which sizes the library's work areas; a call that would have to
 *     allocate under capture returns STAF_E_CAPTURE and allocates nothing.
 *     Outgrown work areas stay allocated until staf_ops_release, so graphs
 *     recorded earlier keep valid addresses.
 *     Tested bound: a capture that forks the op chains onto at most THREE
 *     streams beside the capture stream (captured, instantiated, replayed and
 *     compared bit for bit with the eager step).  A capture that forked onto
 *     four side streams has ended the process inside the end of the capture /
 *     the instantiation of the graph, twice, with the cause unknown; under
 *     capture the library itself only looks up per-stream state it already
 *     holds and launches kernels, exactly as with three streams.  Keep a
 *     captured step to three forked streams.
 */
#ifndef STAF_OPS_H
#define STAF_OPS_H

#ifdef __cplusplus
extern "C" {
#endif

#define STAF_OK 0
#define STAF_E_NOT_CONSTRUCTED (-1)  /* compute before construct (reference: exit(1), reforce.cc:145-148) */
#define STAF_E_BAD_ARG (-2)          /* null pointer / non-positive dimension / dims beyond the constructed maxima */
#define STAF_E_HIP (-3)              /* a HIP runtime call failed */
#define STAF_E_RADIAL_OVERFLOW (-10) /* an atom has more than radial_buffer neighbours (reference: exit(0), reforce.cc:329-337) */
#define STAF_E_SCATTER_OVERFLOW (-11)/* an atom is listed by more centres than the force scatter can hold (4*nr) */
#define STAF_E_LIMIT (-12)           /* nt, channels or buffers beyond the kernels' compile-time limits */
#define STAF_E_CAPTURE (-13)         /* the stream is being captured into a graph and the call would have to allocate:
                                        run the same call once outside the capture first */
#define STAF_E_STALE_MAP (-14)       /* a force op was handed a view of a descriptor output whose intmap2b no longer
                                        holds what the descriptor op wrote there, or whose first row is not the
                                        first atom of the centre species (tipos, actual_type) */

/* ---- library state ------------------------------------------------------ */

/* Version string "major.minor". */
const char* staf_ops_version(void);

/* Error reporting of conditions only the GPU can detect (neighbour-buffer overflow,
 * scatter overflow).  mode 1 (default, reference behaviour): the call that can hit
 * the condition synchronises its stream and returns the code -- except on a stream
 * that is being captured into a graph, which cannot be waited for: there the call
 * behaves as in mode 0.  mode 0: nothing synchronises; conditions accumulate in
 * the stream's device word, read by staf_ops_poll_status. */
void staf_ops_set_sync_errors(int mode);

/* Synchronises `stream`, returns the accumulated device-side status of every
 * stream of the device (0 or a negative STAF_E_* code) and clears it.  Work on
 * other streams that `stream` has not been made to wait for may still raise
 * conditions afterwards; they stay for the next poll. */
int staf_ops_poll_status(void* stream);

/* Measurement aid with no counterpart in the reference: when enabled, the library brackets its kernels with HIP
 * events on the stream they are launched on.  staf_ops_kernel_time waits for the device, returns the summed duration
 * and the number of launches of the named kernel ("desc_kernel", "af2_kernel", "af3_kernel", "force2_kernel",
 * "force3_kernel", "gather_kernel", "grad2_kernel", "grad3_kernel", "gradforce2_kernel", "gradforce3_kernel",
 * "grads3_kernel", "force_total_kernel", "transpose_sort_kernel", "cell_build_kernel")
 * since the last call for that name, and forgets them. */
void staf_ops_kernel_timing(int enable);
int staf_ops_kernel_time(const char* kernel, double* total_ms, int* launches);

/* Waits for the current device and frees all device memory the library holds on it (work areas, remembered
 * neighbour maps, error words); the next call builds them again.  Graphs the caller captured before point into the
 * freed areas and must not be replayed afterwards; a handle of the MD entry (staf.h) notices the release and records
 * its own graph again. */
void staf_ops_release(void);

/* ---- descriptor op ------------------------------------------------------ */

/* ConstructDescriptorsLight -- STAF/src/descriptor_builder/reforce.cc:182-238 (+ fill_repulsion :101-141).
 * Stores the geometry for all later compute calls and derives the short-range coefficients.
 * cutoff_curve_path: where to write the 1000-row "%g %g" curve the reference writes to
 * ./cutoff_curve.dat; NULL skips the file. */
int staf_op_construct_descriptors_light_f32(float radial_cutoff, int radial_buffer, int angular_buffer, int numpar,
                                            float rs, float ra, int max_batch, const char* cutoff_curve_path);
int staf_op_construct_descriptors_light_f64(double radial_cutoff, int radial_buffer, int angular_buffer, int numpar,
                                            double rs, double ra, int max_batch, const char* cutoff_curve_path);

/* Options of the descriptor op (apply to both precisions on the current device; construct resets them to their
 * defaults, so call this after construct).
 *   dist2_fma     0: dist2 = (x*x+y*y)+z*z uncontracted (default); 1: fma(z,z,fma(y,y,x*x))
 *   zero_padding  0: der3b beyond an atom's triplets is left untouched (default; the reference leaves it
 *                    uninitialised as well); 1: it is written as 0.
 * All other padding is always written as 0: angdescr, intmap2b, intmap3b and numtriplet are zeroed by the reference
 * op before its kernels run (reforce.cc:357-358,375-376,385-386,420-421), and the padded slots of raddescr,
 * des3bsupp, der2b and der3bsupp, which the reference leaves uninitialised, are written as 0 too. */
int staf_op_descriptor_options(int dist2_fma, int zero_padding);

/* Frames of at least n_atoms atoms find their neighbours through a cell list (the role of the binning kernels of
 * celle_gpu.cu.cc:11-101), smaller ones test every atom of the frame; default 4096, n_atoms <= 0: never.  The
 * outputs are the same either way. */
int staf_op_descriptor_cell_threshold(int n_atoms);

/* Reads back {A, B, C, pow_alpha, pow_beta} computed by construct. */
int staf_op_descriptor_coefficients_f32(float* out5);
int staf_op_descriptor_coefficients_f64(double* out5);

/* ComputeDescriptorsLight -- STAF/src/descriptor_builder/reforce.cc:241-444, kernels
 * celle_gpu.cu.cc:11-201 (cart->frac, cell list, neighbour search, sort) and
 * reforce.cu.cc:17-236 (radial + angular fill).
 *   positions [nf, 3N] Cartesian, boxer [nf, 6] = [Lx, xy, xz, Ly, yz, Lz]
 *   raddescr [nf,N,nr]  angdescr [nf,N,na]  des3bsupp [nf,N,nr]  intmap2b [nf,N,nr+1]
 *   intmap3b [nf,N,2*na]  der2b [nf,N,3,nr]  der3b [nf,N,3,2*na]  der3bsupp [nf,N,3,nr]  numtriplet [nf,N]
 * Padded slots are written as 0 (der3b: see staf_op_descriptor_options).  The library notes the address of intmap2b
 * as that of a map of its own making (see the conventions above). */
int staf_op_compute_descriptors_light_f32(const float* positions, const float* boxer, int nf, int N, float* raddescr,
                                          float* angdescr, float* des3bsupp, int* intmap2b, int* intmap3b,
                                          float* der2b, float* der3b, float* der3bsupp, int* numtriplet,
                                          void* stream);
int staf_op_compute_descriptors_light_f64(const double* positions, const double* boxer, int nf, int N,
                                          double* raddescr, double* angdescr, double* des3bsupp, int* intmap2b,
                                          int* intmap3b, double* der2b, double* der3b, double* der3bsupp,
                                          int* numtriplet, void* stream);

/* Descriptors and the fingerprints of the centre species first_species .. first_species + n_species - 1 in one
 * launch: a workgroup per centre goes from the neighbour search to the centre's 3-body and 2-body fingerprints (a
 * centre's fingerprints need only the rows its own descriptor workgroup writes).  No counterpart as one op in the
 * reference; replaces, for those centres, staf_op_compute_descriptors_light followed by staf_op_angular_afs and
 * staf_op_radial_afs per species, with the same bits in every output.
 *   descriptor arguments and outputs as staf_op_compute_descriptors_light (whole tensors; the rows of the centres of
 *   other species are not touched: call once with (0, nt), or once per species -- each call on a stream of its own
 *   lets what follows a species' fingerprints start when that species is through, 105 against 114 us for a
 *   single-precision step of 4 x 768 atoms; with more than about 4000 centres per step the separate ops are faster).
 *   nt species, n_local: HOST array of the atoms per species (atoms stored species-sorted, summing to N), type_map [N].
 *   alpha3b, type_emb3b, three_body_AFs: HOST arrays of nt device pointers, per centre species [ntc,3*nsmooth_a],
 *   [ntc,nsmooth_a] and the output [nf,n_local[k],nsmooth_a]; alpha2b, type_emb2b, radial_AFs likewise
 *   ([nt,nalpha_r], [nt,nalpha_r], output [nf,n_local[k],nalpha_r]); nalpha_r = 0 (and null arrays): no 2-body
 *   fingerprints.  Entries of species outside the range, and of species without atoms, are not read.
 * The library's own neighbour search only (no injected list), all N atoms local. */
int staf_op_descriptors_fingerprints_f32(const float* positions, const float* boxer, int nf, int N, float* raddescr,
                                         float* angdescr, float* des3bsupp, int* intmap2b, int* intmap3b,
                                         float* der2b, float* der3b, float* der3bsupp, int* numtriplet, int nt,
                                         const int* n_local, int first_species, int n_species, const int* type_map,
                                         int nsmooth_a, const float* const* alpha3b, const float* const* type_emb3b,
                                         float* const* three_body_AFs, int nalpha_r, const float* const* alpha2b,
                                         const float* const* type_emb2b, float* const* radial_AFs, void* stream);
int staf_op_descriptors_fingerprints_f64(const double* positions, const double* boxer, int nf, int N,
                                         double* raddescr, double* angdescr, double* des3bsupp, int* intmap2b,
                                         int* intmap3b, double* der2b, double* der3b, double* der3bsupp,
                                         int* numtriplet, int nt, const int* n_local, int first_species,
                                         int n_species, const int* type_map, int nsmooth_a,
                                         const double* const* alpha3b, const double* const* type_emb3b,
                                         double* const* three_body_AFs, int nalpha_r, const double* const* alpha2b,
                                         const double* const* type_emb2b, double* const* radial_AFs, void* stream);

/* ---- atomic fingerprints (forward) -------------------------------------- */

/* radialAFs_Launcher (ComputeSortProj) -- STAF/src/fingerprint/rad/reforce.cc:13-24, reforce.cu.cc:12-64.
 *   radial_AFs [nf,Nl,nalpha_r] = sum_k D_k exp(alpha2b[t_k,a] D_k) emb2b[t_k,a];  alpha2b, emb2b [nt,nalpha_r] */
int staf_op_radial_afs_f32(const float* radial_descriptor, int nr, const float* alpha2b, int nalpha_r,
                           float* radial_AFs, int dimbat, int N_local, const int* interaction_map_rad,
                           const float* type_emb2b, const int* type_map, int nt, int ld_atoms, void* stream);
int staf_op_radial_afs_f64(const double* radial_descriptor, int nr, const double* alpha2b, int nalpha_r,
                           double* radial_AFs, int dimbat, int N_local, const int* interaction_map_rad,
                           const double* type_emb2b, const int* type_map, int nt, int ld_atoms, void* stream);

/* angularAFs_Launcher (ComputeSortProj3body) -- STAF/src/fingerprint/ang/reforce.cc:15-30, reforce.cu.cc:13-86.
 *   radial_descriptor = des3bsupp [nf,Nl,nr]; angular_descriptor [nf,Nl,na]; alpha3b [ntc,3*nsmooth_a]
 *   (alpha1,alpha2,beta per channel), type_emb3b [ntc,nsmooth_a]; row = t_j + t_k.
 *   interaction_map_rad [nf,Nl,nr+1] supplies the neighbour species; interaction_map_angular must be the
 *   one the descriptor op produced with it (it is not re-read).
 *   num_triplets [nf,Nl] = neighbours inside the angular cutoff; every 3-body op of this library takes an entry
 *   below 0 as 0 and an entry above nr as nr, so no kernel leaves its rows whatever the tensor holds. */
int staf_op_angular_afs_f32(const float* radial_descriptor, const float* angular_descriptor, int nr, int na,
                            float* three_body_AFs, int dimbat, int N_local, const int* interaction_map_angular,
                            const int* interaction_map_rad, const float* alpha3b, int nsmooth_a,
                            const float* type_emb3b, const int* type_map, const int* num_triplets, int nt,
                            int ld_atoms, void* stream);
int staf_op_angular_afs_f64(const double* radial_descriptor, const double* angular_descriptor, int nr, int na,
                            double* three_body_AFs, int dimbat, int N_local, const int* interaction_map_angular,
                            const int* interaction_map_rad, const double* alpha3b, int nsmooth_a,
                            const double* type_emb3b, const int* type_map, const int* num_triplets, int nt,
                            int ld_atoms, void* stream);

/* ---- forces -------------------------------------------------------------- */

/* init_block_dim (InitForceRadial / InitForceTripl / InitGradForceRadial / InitGradForceTripl) --
 * STAF/src/force/rad/reforce.cc:13-36, force/ang/reforce.cc:14-37, grad_force/rad/reforce.cc:15-38,
 * grad_force/ang/reforce.cc:14-37.  The reference picks a CUDA block size dividing the buffer; these
 * kernels need none, so the calls only validate the argument and return the op's output code [0]. */
int staf_op_init_force_radial(int buffdim);
int staf_op_init_force_tripl(int buffdim);
int staf_op_init_grad_force_radial(int buffdim);
int staf_op_init_grad_force_tripl(int buffdim);

/* Virial forms only: 0 (default) = r_i - r_j is wrapped to the minimum image of the periodic box; 1 = no wrap, the
 * neighbour positions already are the periodic images (domain-decomposed MD with ghost atoms).  Process-wide, like
 * staf_force_skip_pbc of the reference (STAF/include/staf_force_pbc.cuh:5-10); read by the staf_op_* entry points of
 * this header only (staf_compute of staf.h decides per call and neither reads nor changes it). */
void staf_op_force_set_skip_pbc(int skip);

/* computeforce_doublets_Launcher (ComputeForceRadial) -- STAF/src/force/rad/reforce.cc:39-57, reforce.cu.cc:45-172
 * and computeforce_doublets_virial_Launcher (ComputeForceRadialVirial) -- reforce.cc:124-146, reforce.cu.cc:174-314.
 *   forces2b [nf,3N] (all atoms; fully written).  virial [nf,9] row-major W_ab -= g_a r_b, pos [nf,3N]
 *   Cartesian, box [nf,6]; pass virial = pos = box = NULL for the plain op.
 * Deterministic: every atom gathers the pair forces of the slots that list it, in a fixed order; no float atomics. */
int staf_op_force_doublets_f32(const float* netderiv, const float* des_r, const float* intderiv_r,
                               const int* intmap_r, int nr, int N, int dimbat, int num_alpha_radiale,
                               const float* alpha_radiale, const float* type_emb2b, int nt, const int* tipos,
                               const int* actual_type, float* forces2b, const int* type_map, int N_local,
                               float* virial, const float* pos, const float* box, int ld_atoms, void* stream);
int staf_op_force_doublets_f64(const double* netderiv, const double* des_r, const double* intderiv_r,
                               const int* intmap_r, int nr, int N, int dimbat, int num_alpha_radiale,
                               const double* alpha_radiale, const double* type_emb2b, int nt, const int* tipos,
                               const int* actual_type, double* forces2b, const int* type_map, int N_local,
                               double* virial, const double* pos, const double* box, int ld_atoms, void* stream);

/* computeforce_tripl_Launcher (ComputeForceTripl) -- STAF/src/force/ang/reforce.cc:44-66, reforce.cu.cc:48-248
 * and computeforce_tripl_virial_Launcher (ComputeForceTriplVirial) -- reforce.cc:151-176, reforce.cu.cc:269-482.
 *   desr = des3bsupp, desa = angdescr, intderiv_r = der3bsupp, intderiv_a = der3b. */
int staf_op_force_tripl_f32(const float* netderiv, const float* desr, const float* desa, const float* intderiv_r,
                            const float* intderiv_a, const int* intmap_r, const int* intmap_a, int nr, int na, int N,
                            int dimbat, int num_finger, const float* type_emb3b, int nt, const int* tipos,
                            const int* actual_type, float* forces3b, const int* num_triplets, const float* smooth_a,
                            const int* type_map, int N_local, float* virial, const float* pos, const float* box,
                            int ld_atoms, void* stream);
int staf_op_force_tripl_f64(const double* netderiv, const double* desr, const double* desa,
                            const double* intderiv_r, const double* intderiv_a, const int* intmap_r,
                            const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,
                            const double* type_emb3b, int nt, const int* tipos, const int* actual_type,
                            double* forces3b, const int* num_triplets, const double* smooth_a, const int* type_map,
                            int N_local, double* virial, const double* pos, const double* box, int ld_atoms,
                            void* stream);

/* ---- parameter gradients from the energy branch ------------------------- */

/* alpha_dist_grad_Launcher (ComputeTwoBodyParGrad) -- STAF/src/grad_finger/rad/reforce.cc:14-29, reforce.cu.cc:12-66.
 *   prevgrad [nf,Nl,nalpha_r] = dL/dAF2 -> nextgrad_alpha2b, nextgrad_emb2b [nt,nalpha_r] */
int staf_op_alpha_dist_grad_f32(const float* radial_descriptor, int nr, const float* alpha2b, int nalpha_r,
                                float* nextgrad_alpha2b, int dimbat, int N_local, const int* interaction_map_rad,
                                const float* prevgrad, const float* type_emb2b, const int* type_map,
                                float* nextgrad_emb2b, int nt, int ld_atoms, void* stream);
int staf_op_alpha_dist_grad_f64(const double* radial_descriptor, int nr, const double* alpha2b, int nalpha_r,
                                double* nextgrad_alpha2b, int dimbat, int N_local, const int* interaction_map_rad,
                                const double* prevgrad, const double* type_emb2b, const int* type_map,
                                double* nextgrad_emb2b, int nt, int ld_atoms, void* stream);

/* The same op for callers that cannot allocate device memory (code under HIP graph capture that has not run the
 * call eagerly before, serving loops and harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Arguments and results as staf_op_alpha_dist_grad_f64, bit for bit; the work area (partial sums of the workgroups)
 * is a 1 MiB array in the library's own device image instead of memory grown on demand, which limits the call to
 * (min(ceil(dimbat * N_local / 4), 1024) + 32) * 2 * nt * nalpha_r * 8 bytes <= 1 MiB -- any batch with
 * nt * nalpha_r <= 62 -- and returns STAF_E_LIMIT with a message on stderr beyond that.  The call allocates nothing and frees
 * nothing.  All calls on one GPU share that array: calls that overlap on one GPU (different streams or threads)
 * race.  The first call on a device looks up the array's device address (hipGetSymbolAddress): make it outside a
 * capture. */
int staf_op_alpha_dist_grad_noalloc_f64(const double* radial_descriptor, int nr, const double* alpha2b, int nalpha_r,
                                        double* nextgrad_alpha2b, int dimbat, int N_local,
                                        const int* interaction_map_rad, const double* prevgrad,
                                        const double* type_emb2b, const int* type_map, double* nextgrad_emb2b, int nt,
                                        int ld_atoms, void* stream);

/* alphagrad_ang_Launcher (ComputeSortProj3bodyGrad) -- STAF/src/grad_finger/ang/reforce.cc:12-31, reforce.cu.cc:13-133.
 *   prevgrad [nf,Nl,nsmooth_a] = dL/dAF3 -> next_alpha3b_grad [nt_couple,3*nsmooth_a],
 *   next_emb3b_grad [nt_couple,nsmooth_a] (identically zero, as in the reference). */
int staf_op_alphagrad_ang_f32(const float* radial_descriptor, const float* angular_descriptor, int nr, int na,
                              const float* prevgrad, int dimbat, int N_local, const int* intmap3b,
                              const int* intmap2b, const float* alpha3b, int nsmooth_a, float* next_alpha3b_grad,
                              const float* type_emb3b, const int* type_map, float* next_emb3b_grad,
                              const int* num_triplets, int nt_couple, int nt, int ld_atoms, void* stream);
int staf_op_alphagrad_ang_f64(const double* radial_descriptor, const double* angular_descriptor, int nr, int na,
                              const double* prevgrad, int dimbat, int N_local, const int* intmap3b,
                              const int* intmap2b, const double* alpha3b, int nsmooth_a, double* next_alpha3b_grad,
                              const double* type_emb3b, const int* type_map, double* next_emb3b_grad,
                              const int* num_triplets, int nt_couple, int nt, int ld_atoms, void* stream);

/* ---- gradients of the force ops ----------------------------------------- */

/* back_prop_grad_force2b_Launcher (ComputeForceRadialGrad) -- STAF/src/grad_force/rad/reforce.cc:42-63,
 * reforce.cu.cc:46-147, and back_prop_grad_force2b_virial_Launcher (ComputeForceRadialVirialGrad) --
 * reforce.cc:149-176, reforce.cu.cc:165-261.
 *   prevgrad [nf,3N] = dL/dF -> grad_net [nf,Nl,num_finger], grad_alpha2b, grad_emb2b [nt,num_finger].
 *   prevgrad_virial [nf,9] = dL/dW with pos, box for the virial form; NULL for the plain op. */
int staf_op_gradforce_2b_f32(const float* prevgrad, const float* radiale, int nr, const float* alpha_radiale,
                             int num_finger, const float* desder, const int* intmap_r, int dimbat, int N,
                             int N_local, const float* netderiv, const float* type_emb2b, int nt,
                             const int* type_map, const int* tipos, const int* actual_type, float* grad_net,
                             float* grad_alpha2b, float* grad_emb2b, const float* prevgrad_virial, const float* pos,
                             const float* box, int ld_atoms, void* stream);
int staf_op_gradforce_2b_f64(const double* prevgrad, const double* radiale, int nr, const double* alpha_radiale,
                             int num_finger, const double* desder, const int* intmap_r, int dimbat, int N,
                             int N_local, const double* netderiv, const double* type_emb2b, int nt,
                             const int* type_map, const int* tipos, const int* actual_type, double* grad_net,
                             double* grad_alpha2b, double* grad_emb2b, const double* prevgrad_virial,
                             const double* pos, const double* box, int ld_atoms, void* stream);

/* gradforce_tripl_Launcher (ComputeForceTriplGrad) -- STAF/src/grad_force/ang/reforce.cc:39-66, reforce.cu.cc:47-254,
 * and gradforce_tripl_virial_Launcher (ComputeForceTriplVirialGrad) -- reforce.cc:172-206, reforce.cu.cc:274-477.
 *   -> gradnet_3b [nf,Nl,num_finger], grad_alpha3b [ntc,3*num_finger], grad_emb3b [ntc,num_finger] (zero). */
int staf_op_gradforce_tripl_f32(const float* prevgrad, const float* netderiv, const float* desr, const float* desa,
                                const float* intderiv_r, const float* intderiv_a, const int* intmap_r,
                                const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,
                                const float* type_emb3b, int nt, const int* tipos, const int* actual_type,
                                const int* num_triplets, const float* smooth_a, const int* type_map, int N_local,
                                float* gradnet_3b, float* grad_alpha3b, float* grad_emb3b,
                                const float* prevgrad_virial, const float* pos, const float* box, int ld_atoms,
                                void* stream);
int staf_op_gradforce_tripl_f64(const double* prevgrad, const double* netderiv, const double* desr,
                                const double* desa, const double* intderiv_r, const double* intderiv_a,
                                const int* intmap_r, const int* intmap_a, int nr, int na, int N, int dimbat,
                                int num_finger, const double* type_emb3b, int nt, const int* tipos,
                                const int* actual_type, const int* num_triplets, const double* smooth_a,
                                const int* type_map, int N_local, double* gradnet_3b, double* grad_alpha3b,
                                double* grad_emb3b, const double* prevgrad_virial, const double* pos,
                                const double* box, int ld_atoms, void* stream);

/* Both 3-body parameter gradients of a training step in one launch.  No counterpart as one op in the reference: it
 * stands for the pair ComputeForceTriplGrad (STAF/src/grad_force/ang/reforce.cc:39-66, reforce.cu.cc:47-254; with
 * prevgrad_virial/pos/box the virial form, :172-206) and ComputeSortProj3bodyGrad (STAF/src/grad_finger/ang/
 * reforce.cc:24-31, reforce.cu.cc:13-111), which the modules of STAF/gradient_utility register as the gradients of the 3-body
 * force op and of the 3-body fingerprint op and which every energy+force training step runs on the same descriptor
 * tensors.  They share the species grouping, the exponential tables, the staged triplets and exp(beta T) of every
 * (triplet, channel), so one pass costs about what the force-branch op costs alone.
 *   prevgrad_force [nf,3N] = dL/dF, netderiv [nf,Nl,num_finger] = dE/dAF3, prevgrad_energy [nf,Nl,num_finger] = dL/dAF3
 *   -> gradnet_3b [nf,Nl,num_finger] and grad_alpha3b_force [ntc,3*num_finger] as staf_op_gradforce_tripl,
 *      grad_alpha3b_energy [ntc,3*num_finger] as staf_op_alphagrad_ang, grad_emb3b [ntc,num_finger] (zero, once).
 * Results agree with the separate ops to rounding (same sums, other order of a few operations).
 * grad_alpha3b_energy is linear in prevgrad_energy, which must be complete when the pass runs: where dL/dAF3 has a
 * part that is itself derived from gradnet_3b (a force loss back-propagated through the network's second
 * derivative), that part is added afterwards with staf_op_alphagrad_ang. */
int staf_op_grads_tripl_fused_f32(const float* prevgrad_force, const float* netderiv, const float* prevgrad_energy,
                                  const float* desr, const float* desa, const float* intderiv_r,
                                  const float* intderiv_a, const int* intmap_r, const int* intmap_a, int nr, int na,
                                  int N, int dimbat, int num_finger, const float* type_emb3b, int nt,
                                  const int* tipos, const int* actual_type, const int* num_triplets,
                                  const float* smooth_a, const int* type_map, int N_local, float* gradnet_3b,
                                  float* grad_alpha3b_force, float* grad_alpha3b_energy, float* grad_emb3b,
                                  const float* prevgrad_virial, const float* pos, const float* box, int ld_atoms,
                                  void* stream);
int staf_op_grads_tripl_fused_f64(const double* prevgrad_force, const double* netderiv, const double* prevgrad_energy,
                                  const double* desr, const double* desa, const double* intderiv_r,
                                  const double* intderiv_a, const int* intmap_r, const int* intmap_a, int nr, int na,
                                  int N, int dimbat, int num_finger, const double* type_emb3b, int nt,
                                  const int* tipos, const int* actual_type, const int* num_triplets,
                                  const double* smooth_a, const int* type_map, int N_local, double* gradnet_3b,
                                  double* grad_alpha3b_force, double* grad_alpha3b_energy, double* grad_emb3b,
                                  const double* prevgrad_virial, const double* pos, const double* box, int ld_atoms,
                                  void* stream);

/* The 3-body force op in two halves, for a caller that owns the whole step.  No counterpart in the reference, whose
 * ComputeForceTripl (STAF/src/force/ang/reforce.cc:44-66) scatters with atomicAdd inside the op and whose callers
 * then add the per-op force arrays (force_radial + force_angular, STAF/source_routine/force_layer_mod.py:24-43;
 * tf.math.add_n over the species, STAF/staf_models/staf_model.py:210).
 *
 * staf_op_force_tripl_slots: arguments of staf_op_force_tripl (no virial form); instead of forces3b it returns the
 *   force of every centre on each of its neighbour slots, slot_forces [nf,N_local,nr,3], and on the centre itself,
 *   self_forces [nf,N_local,3] (caller-owned, fully written).  No atom collects anything yet.
 * staf_op_force_total: one launch that, for every atom, collects the slot forces of all centre species and adds
 *   the per-op force arrays to them: total [nf,3N] = sum over species k = 0..nt-1, in this order, of forces2b[k]
 *   (any [nf,3N] array, e.g. the output of staf_op_force_doublets for centre species k; null to skip) and of the
 *   3-body forces of centre species k (slot_forces[k], self_forces[k]; null to skip).  The result has the bits of
 *   the per-op outputs added in that order.  slot_forces, self_forces, forces2b are HOST arrays of nt device
 *   pointers; n_local is a HOST array of the atoms per species (atoms are stored species-sorted, summing to N);
 *   intmap_r_full is the whole [nf,N,nr+1] tensor the descriptor op wrote and still remembers (its own neighbour
 *   search: the map is symmetric), else STAF_E_BAD_ARG -- callers with other maps use staf_op_force_tripl. */
int staf_op_force_tripl_slots_f32(const float* netderiv, const float* desr, const float* desa,
                                  const float* intderiv_r, const float* intderiv_a, const int* intmap_r,
                                  const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,
                                  const float* type_emb3b, int nt, const int* tipos, const int* actual_type,
                                  float* slot_forces, float* self_forces, const int* num_triplets,
                                  const float* smooth_a, const int* type_map, int N_local, int ld_atoms,
                                  void* stream);
int staf_op_force_tripl_slots_f64(const double* netderiv, const double* desr, const double* desa,
                                  const double* intderiv_r, const double* intderiv_a, const int* intmap_r,
                                  const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,
                                  const double* type_emb3b, int nt, const int* tipos, const int* actual_type,
                                  double* slot_forces, double* self_forces, const int* num_triplets,
                                  const double* smooth_a, const int* type_map, int N_local, int ld_atoms,
                                  void* stream);
/* staf_op_force_tripl_slots with the 2-body pair forces of the same centre species added to the slot forces in the
 * same launch (the arguments of staf_op_force_doublets beside those of staf_op_force_tripl: netderiv2b
 * [nf,N_local,num_alpha_radiale], des_r2b = raddescr, intderiv_r2b = der2b, alpha_radiale, type_emb2b): slot_forces and
 * self_forces then hold 2-body + 3-body, and staf_op_force_total gives the total force of a step without any per-op
 * force array.  Agrees with the sum of the two ops' outputs to rounding (other order of the additions). */
int staf_op_forces_slots_f32(const float* netderiv3b, const float* netderiv2b, const float* desr, const float* desa,
                             const float* intderiv_r, const float* intderiv_a, const float* des_r2b,
                             const float* intderiv_r2b, const int* intmap_r, const int* intmap_a, int nr, int na,
                             int N, int dimbat, int num_finger, int num_alpha_radiale, const float* type_emb3b,
                             const float* smooth_a, const float* alpha_radiale, const float* type_emb2b, int nt,
                             const int* tipos, const int* actual_type, float* slot_forces, float* self_forces,
                             const int* num_triplets, const int* type_map, int N_local, int ld_atoms, void* stream);
int staf_op_forces_slots_f64(const double* netderiv3b, const double* netderiv2b, const double* desr,
                             const double* desa, const double* intderiv_r, const double* intderiv_a,
                             const double* des_r2b, const double* intderiv_r2b, const int* intmap_r,
                             const int* intmap_a, int nr, int na, int N, int dimbat, int num_finger,
                             int num_alpha_radiale, const double* type_emb3b, const double* smooth_a,
                             const double* alpha_radiale, const double* type_emb2b, int nt, const int* tipos,
                             const int* actual_type, double* slot_forces, double* self_forces,
                             const int* num_triplets, const int* type_map, int N_local, int ld_atoms, void* stream);
int staf_op_force_total_f32(const int* intmap_r_full, int nr, int N, int dimbat, int nt, const int* n_local,
                            const float* const* slot_forces, const float* const* self_forces,
                            const float* const* forces2b, float* total, void* stream);
int staf_op_force_total_f64(const int* intmap_r_full, int nr, int N, int dimbat, int nt, const int* n_local,
                            const double* const* slot_forces, const double* const* self_forces,
                            const double* const* forces2b, double* total, void* stream);

/* Sum of up to four arrays of n elements, dst[e] = ((a[e] + b[e]) + c[e]) + d[e] (c, d may be null), in one launch:
 * what the callers do with the per-op force arrays (force_radial + force_angular in
 * STAF/source_routine/force_layer_mod.py:43, tf.math.add_n over the species in
 * STAF/staf_models/staf_model.py:210).  dst may be one of the inputs.  No counterpart among the reference's ops. */
int staf_op_add_n_f32(float* dst, const float* a, const float* b, const float* c, const float* d, int n,
                      void* stream);
int staf_op_add_n_f64(double* dst, const double* a, const double* b, const double* c, const double* d, int n,
                      void* stream);

#ifdef __cplusplus
}
#endif
#endif /* STAF_OPS_H */
