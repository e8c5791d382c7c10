// Shared device/host helpers of the gfx950 STAF kernels.
//
// One templated source serves fp32 and fp64: every kernel is a template on
// `real` and the extern "C" entry points instantiate it twice (_f32/_f64).
// Wavefronts are 64 lanes wide; all cross-lane reductions below use a fixed
// butterfly tree, so a sum's rounding does not depend on scheduling.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <unordered_map>
#include <vector>

#include "../../include/staf_ops.h"

namespace staf {

constexpr int WAVE = 64;
constexpr int NT_MAX = 8;  // species supported by the per-type bookkeeping

template <typename real> struct Vec2;
template <> struct Vec2<float> { using type = float2; };
template <> struct Vec2<double> { using type = double2; };
// 16 bytes of reals: the widest LDS and global access
template <typename real> struct Vec16;
template <> struct Vec16<float> { using type = float4; };
template <> struct Vec16<double> { using type = double2; };
template <typename real> struct Vec4;
template <> struct Vec4<float> { using type = float4; };
template <> struct Vec4<double> { using type = double4; };

// The reference's value of pi (STAF/src/descriptor_builder/reforce.cu.cc:15).
template <typename real> __host__ __device__ inline real pi_ref() { return real(3.141592654); }

__device__ inline float r_exp(float x) { return expf(x); }
__device__ inline double r_exp(double x) { return exp(x); }
__device__ inline float r_cos(float x) { return cosf(x); }
__device__ inline double r_cos(double x) { return cos(x); }
__device__ inline float r_sin(float x) { return sinf(x); }
__device__ inline double r_sin(double x) { return sin(x); }
__device__ inline void r_sincos(float x, float* s, float* c) { sincosf(x, s, c); }
__device__ inline void r_sincos(double x, double* s, double* c) { sincos(x, s, c); }
// sin and cos of an argument in [0, pi] (the cutoff functions' pi r / Rc, r < Rc): reduction by a multiple of pi/2 in
// two parts, then the polynomials of fdlibm's kernel_sin / kernel_cos on [-pi/4, pi/4].  Maximum error 1.1e-16
// absolute over the range against the C library's sin and cos; an eighth of the instructions of the general routine,
// which has to cope with any argument.  Single precision keeps the library routine.
__device__ inline void r_sincos_0pi(float x, float* s, float* c) { sincosf(x, s, c); }
__device__ inline void r_sincos_0pi(double x, double* sn, double* cs) {
  const double k = rint(x * 0.63661977236758134308);
  double y = fma(-k, 1.57079632673412561417e+00, x);
  y = fma(-k, 6.07710050650619224932e-11, y);
  const double z = y * y;
  double ps = 1.58969099521155010221e-10;
  ps = fma(ps, z, -2.50507602534068634195e-08);
  ps = fma(ps, z, 2.75573137070700676789e-06);
  ps = fma(ps, z, -1.98412698298579493134e-04);
  ps = fma(ps, z, 8.33333333332248946124e-03);
  ps = fma(ps, z, -1.66666666666666324348e-01);
  const double s = fma(y * z, ps, y);
  double pc = -1.13596475577881948265e-11;
  pc = fma(pc, z, 2.08757232129817482790e-09);
  pc = fma(pc, z, -2.75573143513906633035e-07);
  pc = fma(pc, z, 2.48015872894767294178e-05);
  pc = fma(pc, z, -1.38888888888741095749e-03);
  pc = fma(pc, z, 4.16666666666666019037e-02);
  const double c = 1.0 - (0.5 * z - z * z * pc);
  const int q = (int)k;   // 0, 1 or 2
  *sn = q == 0 ? s : (q == 1 ? c : -s);
  *cs = q == 0 ? c : (q == 1 ? -s : -c);
}
__device__ inline float r_sqrt(float x) { return sqrtf(x); }
__device__ inline double r_sqrt(double x) { return sqrt(x); }
__device__ inline float r_pow(float x, float n) { return powf(x, n); }
__device__ inline double r_pow(double x, double n) { return pow(x, n); }
__device__ inline float r_rint(float x) { return rintf(x); }
__device__ inline double r_rint(double x) { return rint(x); }
__device__ inline float r_floor(float x) { return floorf(x); }
__device__ inline double r_floor(double x) { return floor(x); }
__device__ inline float r_fma(float a, float b, float c) { return fmaf(a, b, c); }
__device__ inline double r_fma(double a, double b, double c) { return fma(a, b, c); }

__device__ inline int lane_id() { return threadIdx.x & (WAVE - 1); }

// Butterfly all-reduce over the 64 lanes of a wave; every lane returns the sum.
template <typename T>
__device__ inline T wave_sum(T v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
// Data-parallel-primitive lane moves: lane l receives the value of another lane of its row of 16 (or of the
// previous rows for the broadcasts); lanes without a source receive 0.
template <int CTRL, int ROW_MASK>
__device__ inline float dpp_get(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK>
__device__ inline unsigned dpp_get(unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
template <int CTRL, int ROW_MASK>
__device__ inline double dpp_get(double v) {
  const long long b = __double_as_longlong(v);
  const int lo = __builtin_amdgcn_update_dpp(0, (int)(b & 0xffffffffll), CTRL, ROW_MASK, 0xf, false);
  const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, ROW_MASK, 0xf, false);
  return __longlong_as_double(((long long)hi << 32) | (unsigned int)lo);
}
// The two steps that carry a prefix across the rows of 16 lanes: s += (lane 15 of the row before) in rows 1 and 3,
// then s += (lane 31) in rows 2 and 3.  Written as `s += dpp_get<..>(s)` each costs a zero, a move and an add,
// because the rows that receive nothing need a 0 to add; as one add whose result is written in the selected rows
// only (the others keep s) it is a single instruction.  Single precision only: the lane moves are 32 bits wide.
// A lane move reads a register two cycles after the instruction that wrote it at the earliest: the idle cycles
// stand in front of the moves, and behind them for whatever lane operation follows.
__device__ inline void dpp_rows_carry(float& a) {
  asm("s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa\n\t"
      "s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc\n\t"
      "s_nop 1"
      : "+v"(a));
}
__device__ inline void dpp_rows_carry(float& a, float& b, float& c, float& d) {
  asm("s_nop 1\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa\n\t"
      "v_add_f32_dpp %1, %1, %1 row_bcast:15 row_mask:0xa\n\t"
      "v_add_f32_dpp %2, %2, %2 row_bcast:15 row_mask:0xa\n\t"
      "v_add_f32_dpp %3, %3, %3 row_bcast:15 row_mask:0xa\n\t"
      "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc\n\t"
      "v_add_f32_dpp %1, %1, %1 row_bcast:31 row_mask:0xc\n\t"
      "v_add_f32_dpp %2, %2, %2 row_bcast:31 row_mask:0xc\n\t"
      "v_add_f32_dpp %3, %3, %3 row_bcast:31 row_mask:0xc\n\t"
      "s_nop 1"
      : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ inline void dpp_rows_carry(unsigned& a) {
  asm("s_nop 1\n\t"
      "v_add_u32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa\n\t"
      "s_nop 1\n\t"
      "v_add_u32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc\n\t"
      "s_nop 1"
      : "+v"(a));
}
__device__ inline void dpp_rows_carry(double& s) {
  s += dpp_get<0x142, 0xa>(s);   // lane 15 of a row -> every lane of the next row (rows 1 and 3 take it)
  s += dpp_get<0x143, 0xc>(s);   // lane 31 -> rows 2 and 3
}
__device__ inline void dpp_rows_carry(double& a, double& b, double& c, double& d) {
  a += dpp_get<0x142, 0xa>(a); b += dpp_get<0x142, 0xa>(b); c += dpp_get<0x142, 0xa>(c); d += dpp_get<0x142, 0xa>(d);
  a += dpp_get<0x143, 0xc>(a); b += dpp_get<0x143, 0xc>(b); c += dpp_get<0x143, 0xc>(c); d += dpp_get<0x143, 0xc>(d);
}

// Sum over the 64 lanes with register-to-register lane moves only; the total is valid in lane 63 alone.
// Fixed tree: prefix steps 1,2,3,4,8 inside each row of 16, then row 0->1, 2->3, and rows 0-1 -> 2-3.
template <typename T>
__device__ inline T wave_sum_to_last(T v) {
  T s = v + dpp_get<0x111, 0xf>(v);
  s += dpp_get<0x112, 0xf>(v);
  s += dpp_get<0x113, 0xf>(v);
  s += dpp_get<0x114, 0xf>(s);
  s += dpp_get<0x118, 0xf>(s);
  dpp_rows_carry(s);
  return s;
}
// Wave-uniform value loaded through a vector path (e.g. from LDS) moved to a scalar register, so that loop
// bounds and addresses derived from it stay scalar.
__device__ inline int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

__device__ inline int wave_max(int v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Index arithmetic of the hot kernels uses the 24-bit multiplier (full rate; the 32-bit integer multiply takes
// four times as long): operands here are slot, species and channel counts far below 2^23.
__device__ inline int mul24(int a, int b) { return __mul24(a, b); }

// First flat index of row j in the row-major upper triangle over m items
// (pairs j<k): the reference's triplet numbering,
// STAF/src/descriptor_builder/reforce.cu.cc:137-146.  j m - j (j + 1) / 2 = j (2 m - 1 - j) / 2, m <= 2048.
__device__ inline int tri_rowstart(int j, int m) { return mul24(j, 2 * m - 1 - j) >> 1; }

// Inverse of the numbering: nn -> (j,k), 0 <= nn < m(m-1)/2, m <= 2048.
// With t = 2m - 1 the row is j = floor((t - sqrt(t^2 - 8 nn)) / 2); the root is an integer exactly at a row's first
// pair, where a rounding error would decide the row.
// m <= 255: the root is taken of t^2 - 8 nn - 4 instead, which moves the quotient 1/(t - 2j) >= 0.002 away from the
// integers on either side (up at a row's first pair, down at the last pair of the row before) -- sixty times the
// error of the single-precision root and subtraction, so the truncation is the row and no correction step follows
// (checked for every m <= 255 and every nn, with the root off by up to two units in the last place).
// m > 255: the hardware square root (1 ulp) puts the row estimate within one of the exact row (two steps each way
// are taken); the row start follows the row in steps of the row length m - 1 - j, so that the comparisons with the
// exact integer row starts cost no multiply.
__device__ inline void tri_decode(int nn, int m, int& j, int& k) {
  const int t = 2 * m - 1;
  if (m <= 255) {
    const int jj = (int)(((float)t - __builtin_amdgcn_sqrtf((float)(mul24(t, t) - 4 - 8 * nn))) * 0.5f);
    j = jj;
    k = nn - (mul24(jj, t - jj) >> 1) + jj + 1;
    return;
  }
  int jj = (int)(((float)t - __builtin_amdgcn_sqrtf((float)(mul24(t, t) - 8 * nn))) * 0.5f);
  jj = jj < 0 ? 0 : (jj > m - 2 ? m - 2 : jj);
  int rs = mul24(jj, t - jj) >> 1;
#pragma unroll
  for (int it = 0; it < 2; it++) {   // row 0 starts at 0 <= nn: never stepped below
    const bool down = rs > nn;
    rs = down ? rs - (m - jj) : rs;
    jj = down ? jj - 1 : jj;
  }
#pragma unroll
  for (int it = 0; it < 2; it++) {   // the row after row m - 2 would start at m (m - 1) / 2 > nn: never stepped to
    const int next = rs + (m - 1 - jj);
    const bool up = next <= nn;
    rs = up ? next : rs;
    jj = up ? jj + 1 : jj;
  }
  j = jj;
  k = nn - rs + jj + 1;
}

// Minimum-image Cartesian separation r_i - r_j from Cartesian positions and
// box6 = [Lx, xy, xz, Ly, yz, Lz]: cart -> frac, rint, back to cart
// (STAF/include/staf_force_pbc.cuh:16-49; used by the virial forms only).  skip_pbc: no wrap, the neighbour
// already carries its periodic image (staf_force_skip_pbc there).
template <typename real>
__device__ inline void mic_cart_from_cart(const real* pi, const real* pj, const real* bx, int skip_pbc, real* d) {
  const real i0 = real(1) / bx[0];
  const real i1 = -bx[1] / (bx[0] * bx[3]);
  const real i2 = (bx[1] * bx[4]) / (bx[0] * bx[3] * bx[5]) - bx[2] / (bx[0] * bx[5]);
  const real i3 = real(1) / bx[3];
  const real i4 = -bx[4] / (bx[3] * bx[5]);
  const real i5 = real(1) / bx[5];
  real rx = (i0 * pi[0] + i1 * pi[1] + i2 * pi[2]) - (i0 * pj[0] + i1 * pj[1] + i2 * pj[2]);
  real ry = (i3 * pi[1] + i4 * pi[2]) - (i3 * pj[1] + i4 * pj[2]);
  real rz = i5 * pi[2] - i5 * pj[2];
  if (!skip_pbc) {
    rx -= r_rint(rx);
    ry -= r_rint(ry);
    rz -= r_rint(rz);
  }
  d[0] = bx[0] * rx + bx[1] * ry + bx[2] * rz;
  d[1] = bx[3] * ry + bx[4] * rz;
  d[2] = bx[5] * rz;
}

// Pair index q inside an n-item triangle (x<y) -> (x,y); same numbering.
__device__ inline void tri_decode_xy(int q, int n, int& x, int& y) { tri_decode(q, n, x, y); }

// ---- library-owned device state (per device) -------------------------------
struct Workspace {
  void* buf = nullptr;
  size_t bytes = 0;
};

// Work areas are kept per stream: ops issued on different streams of one device (e.g. the per-species op chains,
// which do not depend on each other) never share scratch, so they may run concurrently.
struct StreamWork {
  Workspace scratch;         // per-slot partial forces / partial sums
  Workspace buckets;         // transpose a force op builds for itself: build counters, counts, keys
  size_t bucket_counters = 0;    // capacity, in ints, of each of the two counter parts
  size_t bucket_entries = 0;     // capacity, in ints, of the key part
  Workspace cells;           // cell list of the descriptor op: set toggle, two sets of cell counters, tables, records
  size_t cell_counters = 0;      // capacity, in ints, of each of the two counter sets
};

// The cell-list block of a stream (see cell_build_kernel).  The toggle and the counters live as long as the block:
// the counter set the toggle names reads zero whenever a descriptor call starts, whatever the shapes of the calls
// before it (a fresh block is cleared on the caller's stream).
struct CellBlock {
  int* toggle = nullptr;     // [1]
  int* counts = nullptr;     // [2][set_ints]
  size_t set_ints = 0;
  char* rest = nullptr;      // rest_bytes, 256-byte aligned: tables and records of this call
};

// What a force kernel needs to find the slots that list an atom (see staf_transpose.hpp).  Two forms:
//   symmetric = 1  the map is one the library's own neighbour search wrote for all N atoms of the frames: i lists
//                  j exactly when j lists i, so an atom's own row names the centres that list it, and the slot is
//                  found by looking the atom up in that centre's row.  `full` is the whole tensor [nf, N, nr+1].
//   symmetric = 0  a transposed map, receiver -> sorted (centre, slot) keys (caller-supplied lists, where ghost
//                  atoms are listed without listing anybody; maps of unknown origin).
struct TransposeRef {
  int symmetric = 0;
  const int* full = nullptr; // symmetric: the intmap2b tensor the view points into
  const unsigned* rowsum = nullptr;   // symmetric: [nf * N] checksum of every row as the descriptor op wrote it (row_hash
                                      // in staf_transpose.hpp), or null where no block could be had: an atom that
                                      // collects through its own row compares, and reports a stale map on a difference
  int* build_cnt = nullptr;  // [nf * Nrecv] fill cursors of a build, all zero between builds
  int* cnt = nullptr;        // [nf * Nrecv] keys per receiving atom
  int* keys = nullptr;       // [nf * Nrecv, cap]
  int cap = 0;
  int key_shift = 0;         // centre number (row in `full`) of row 0 of the map the force op was handed
};

// Transpose the descriptor op keeps beside an intmap2b tensor it has written.
struct Transpose {
  const int* im2 = nullptr;  // the intmap2b tensor [nf, N, nr+1] it was built from
  int nf = 0, N = 0, Nrecv = 0, nr = 0;
  TransposeRef ref;
  Workspace buf;
  size_t cap_recv = 0, cap_keys = 0;   // capacities of buf, in ints, of a counter part and of the key part
  unsigned long long stamp = 0;        // last use, for replacement
};
constexpr int TRANSPOSE_SLOTS = 8;     // descriptor output tensors whose transposes are kept at a time
constexpr int STATUS_WORDS = 64;       // error words of a device, one per stream

struct DeviceState {
  int device = -1;
  // Error words kernels OR their bits into: one per stream that has used the device (STATUS_WORDS of them, allocated
  // with the state; later streams share the last one).  The synchronising return of an op reports and clears the word
  // of the op's own stream, so a condition goes to the caller that raised it; a poll reports and clears all of them.
  int* status_d = nullptr;   // [STATUS_WORDS]
  int* status_h = nullptr;   // pinned host mirror, [STATUS_WORDS]
  std::unordered_map<hipStream_t, int> status_slot;
  std::unordered_map<hipStream_t, StreamWork> work;
  Transpose transposes[TRANSPOSE_SLOTS];
  std::vector<void*> retired;   // outgrown blocks, freed by staf_ops_release
  unsigned long long transpose_clock = 0;
};

// For the current device, created on the first call (which allocates and synchronises: refused with null while
// `stream` is being captured).
DeviceState* device_state(hipStream_t stream);
// True while `stream` is being captured into a graph: memory may then neither be freed nor allocated, and a fill
// launched to initialise a fresh block would become part of the graph.
bool stream_is_capturing(hipStream_t stream);
// Counts the calls of staf_ops_release: work-area addresses recorded anywhere (a captured graph of the MD entry)
// are valid only while it stands still.
unsigned release_epoch();
// Dynamic LDS of a launch of `kernel`: up to 64 KB needs nothing, up to the 160 KB of a CU is requested for the
// kernel (host-side attribute, no stream work).  False: the launch cannot be made (STAF_E_LIMIT).
template <typename K>
inline bool lds_request(K kernel, size_t lds) {
  if (lds <= 64 * 1024) return true;
  return lds <= 160 * 1024 &&
         hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess;
}
// The error word of `stream` on this device (see DeviceState::status_d).
int* status_word(DeviceState* st, hipStream_t stream);
// Both grow on demand and never shrink; under capture a request that does not fit what the stream already holds
// returns null (the caller reports STAF_E_CAPTURE) instead of freeing and allocating.
void* scratch_reserve(DeviceState* st, hipStream_t stream, size_t bytes);
bool cells_reserve(DeviceState* st, hipStream_t stream, size_t counters, size_t rest_bytes, CellBlock* out);
// Transpose a force op builds for itself (n_recv receiving atoms, cap keys each), in the stream's own work area.
bool bucket_reserve(DeviceState* st, size_t n_recv, int cap, hipStream_t stream, TransposeRef* out);
// What the library keeps beside the intmap2b tensor `im2` the descriptor op is about to write (nf frames, N centres,
// Nrecv receiving atoms): for its own neighbour search (symmetric) only the fact, for a caller's list a transposed
// map of cap keys per receiver.  No block to be had -> false.
bool transpose_for_descriptor(DeviceState* st, const int* im2, int nf, int N, int Nrecv, int nr, int cap,
                              bool symmetric, hipStream_t stream, TransposeRef* out);
// The transpose that covers the map view a force op was handed (pointer into a descriptor output, frame stride ld),
// if the library holds one.
bool transpose_find(DeviceState* st, const int* im2_view, int nf, int Nrecv, int Nl, int ld, int nr, TransposeRef* out);
int finish_op(DeviceState* st, hipStream_t stream);            // launch check (+ optional sync & status fetch)
// STAF_E_CAPTURE when the stream is being captured, else STAF_E_HIP: the code for a work area that could not be had
int reserve_failure(hipStream_t stream);
bool sync_errors_enabled();
struct DeferStatus {   // while one is alive, the calling thread's ops do not synchronise to report device conditions
  DeferStatus();
  ~DeferStatus();
};

// Optional timing of single kernels with HIP events on the stream they are launched on (off by default; switched on
// with staf_ops_kernel_timing).  A KernelTimer brackets one launch; the pairs are summed by staf_ops_kernel_time.
bool kernel_timing_enabled();
void kernel_timing_record(const char* kernel, hipEvent_t a, hipEvent_t b);
struct KernelTimer {
  hipEvent_t a = nullptr, b = nullptr;
  hipStream_t stream;
  const char* name;
  KernelTimer(const char* kernel, hipStream_t s) : stream(s), name(kernel) {
    if (!kernel_timing_enabled()) return;
    if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) { a = b = nullptr; return; }
    (void)hipEventRecord(a, stream);
  }
  ~KernelTimer() {
    if (!a) return;
    (void)hipEventRecord(b, stream);
    kernel_timing_record(name, a, b);
  }
};

// Descriptor geometry shared by all devices (set by construct_descriptors_light).
template <typename real>
struct DescConfig {
  bool ready = false;
  int nr = 0, na = 0, n_max = 0, max_batch = 0;
  real Rc = 0, Rs = 0, Ra = 0;
  real cA = 0, cB = 0, cC = 0, pa = 0, pb = 0;
  int dist2_fma = 0;
  int zero_padding = 0;
};

// Internal launchers shared with the MD entry (staf_api): descriptor op with an explicit configuration, an
// optional caller-supplied neighbour list (owned centres only, Npos >= N positions) and optional no-wrap mode.
// unit != null: radial-only call -- no triplet tensor is written (angdescr, intmap3b, der3b may be null) and unit
// [nf, N, 4, nr] receives the unit vectors centre - neighbour and 1/r of the sorted neighbours.
template <typename real>
int desc_configure(DescConfig<real>& c, real Rc, int nr, int na, real Rs, real Ra);
template <typename real>
int desc_launch(const DescConfig<real>& c, const real* pos, const real* box, int nf, int N, int Npos,
                const int* inj_howmany, const int* inj_with, int skip_pbc, real* raddescr, real* angdescr,
                real* des3bsupp, int* intmap2b, int* intmap3b, real* der2b, real* der3b, real* der3bsupp,
                int* numtriplet, real* unit, hipStream_t stream);


// Force ops with the wrap switch of the virial forms given per call (skip_pbc = 1: neighbour positions already are
// periodic images; the extern "C" entry points pass the process-wide setting of staf_op_force_set_skip_pbc, the MD
// entry its own per call).  Argument lists as in include/staf_ops.h.
template <typename real>
int force_doublets(const real* G, const real* D, const real* dD, const int* im2, int nr, int N, int nf, int Ar,
                   const real* alpha2b, const real* emb2b, int nt, const int* tipos, const int* actual_type,
                   real* force, const int* type_map, int Nl, real* virial, const real* pos, const real* box, int ld,
                   int skip_pbc, void* stream);
// unit != null: the fused forms of the MD entry (T and its Jacobian rebuilt from the radial-only descriptor call's
// unit vectors; Tang, d3b, im3 are not read and may be null).
template <typename real>
int angular_afs(const real* Dsup, const real* Tang, const real* unit, int nr, int na, real* out, int nf, int Nl,
                const int* im3, const int* im2, const real* alpha3b, int Aa, const real* emb3b, const int* type_map,
                const int* numtriplet, int nt, int ld, void* stream);
// The 2-body inputs of the force launch that adds the pair forces to the 3-body slot forces (staf_force3.hpp).
template <typename real>
struct Force2In {
  const real* G2;       // [nf, Nl, Ar] dE/dAF2
  const real* D;        // raddescr [nf, ld, nr]
  const real* dD;       // der2b [nf, ld, 3, nr]
  const real* alpha2b;  // [nt, Ar]
  const real* emb2b;    // [nt, Ar]
  int Ar;
};

template <typename real>
int force_tripl(const real* G, const real* Dsup, const real* Tang, const real* dDsup, const real* d3b,
                const real* unit, const int* im2, const int* im3, int nr, int na, int N, int nf, int Aa,
                const real* emb3b, int nt,
                const int* tipos, const int* actual_type, real* force, const int* numtriplet, const real* alpha3b,
                const int* type_map, int Nl, real* virial, const real* pos, const real* box, int ld, int skip_pbc,
                void* stream, real* slots_out = nullptr, real* self_out = nullptr,
                const Force2In<real>* two_body = nullptr);
// Virial of slot forces (of 2-body, 3-body or both bodies in one array) and the total force collected from the slot
// forces of all species: the internal forms of staf_op_force_total and of the virial kernels of the force ops.
template <typename real>
int slots_virial(const real* gslot, const int* im2, const real* pos, const real* box, const int* tipos,
                 const int* actual_type, real* virial, int nf, int N, int Nl, int ld, int nr, int skip_pbc, void* stream);
template <typename real>
int force_total(const int* im2_full, int nr, int N, int nf, int nt, const int* n_local, const real* const* slot_forces,
                const real* const* self_forces, const real* const* force_2b, real* total, void* stream);

}  // namespace staf
