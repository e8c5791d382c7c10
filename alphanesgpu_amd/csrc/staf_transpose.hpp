// Transpose of the neighbour map: for every receiving atom the (centre, slot) pairs that list it.
//
// The reference scatters pair forces with floating-point atomicAdd (STAF/src/force/rad/reforce.cu.cc:112-131,
// STAF/src/force/ang/reforce.cu.cc:206-231).  Here the force on an atom is gathered by the atom itself from the
// slots that point at it, which needs intmap2b transposed: receiver -> sorted list of keys (centre, slot).  The
// transpose depends on intmap2b alone, so it is built once by the descriptor op that writes intmap2b (pushes from
// desc_kernel, one sort launch) and kept by the library beside that tensor; every force op that is handed a view of
// that tensor finds it by address.  A force op that is handed some other copy of the map builds a transpose of its
// own first (push + sort launches).
//
// Building uses integer atomics only (the arrival order they leave is removed by the sort); every list ends up in
// ascending (centre, slot) order, so sums taken over it have a fixed order.
//
// None of this is needed for the maps the library's own neighbour search writes: those are symmetric, the centres
// that list an atom are the atom's own neighbours, and the slot is found by looking the atom up in the centre's row
// (slot_of below).  Sums then run in the order of the atom's own (distance-sorted) row.
#pragma once
#include "staf_common.hpp"

namespace staf {

constexpr int KEY_SLOT_BITS = 10;   // key = centre << 10 | slot; slots < 1024 (the descriptor op's limit on nr)
constexpr int TR_BLOCK = 256;
constexpr int TR_WAVES = TR_BLOCK / WAVE;

__device__ inline int key_make(int centre, int slot) { return (centre << KEY_SLOT_BITS) | slot; }
__device__ inline int key_centre(int key) { return key >> KEY_SLOT_BITS; }
__device__ inline int key_slot(int key) { return key & ((1 << KEY_SLOT_BITS) - 1); }

// Registers slot `slot` of centre `centre` with receiving atom `recv` (index into [nf * Nrecv]).
__device__ inline void transpose_push(int* build_cnt, int* keys, int cap, size_t recv, int centre, int slot,
                                      int* status) {
  const int pos = atomicAdd(&build_cnt[recv], 1);
  if (pos < cap) keys[recv * cap + pos] = key_make(centre, slot);
  else atomicOr(status, 2);
}

// Checksum of a row of a map, order-free: the sum over its slots of row_hash(neighbour, slot), plus the count.  The
// descriptor op stores it for every row of a map it writes; a kernel that takes an atom's own row as the list of
// centres that list the atom recomputes it, so that other content at a remembered address (a caller's list copied
// there, a tensor of another call at a recycled address) is reported instead of read as symmetric.
__device__ inline unsigned row_hash(int neighbour, int slot) {
  return ((unsigned)neighbour + 1u) * (2u * (unsigned)slot + 1u) * 0x9E3779B1u;
}
// `partial`: the lane's share of the sum over the row's slots below `cnt`; the last lane holds the sum and reports.
__device__ inline void row_check(const TransposeRef& tr, size_t row, int cnt, unsigned partial, int lane, int* status) {
  if (!tr.rowsum) return;
  const unsigned h = wave_sum_to_last(partial) + (unsigned)cnt;
  if (lane == WAVE - 1 && h != tr.rowsum[row]) atomicOr(status, 4);
}

// Slot of atom `a` in the row of centre `i` of frame b of the symmetric map `full` [nf, N, nr+1], or -1 (the map is
// not symmetric after all: reported by the caller).  The whole row is requested at once, sixteen entries per round
// in four 16-byte reads (rows are only 4-byte aligned), and compared without an early exit: one round trip to
// memory instead of one per entry.
struct __attribute__((packed, aligned(4))) Int4U { int x, y, z, w; };
__device__ inline int slot_of(const int* __restrict__ full, int b, int N, int nr, int i, int a) {
  const int* r = full + ((size_t)b * N + i) * (nr + 1);
  int cnt = r[0];
  if (cnt > nr) cnt = nr;
  const int* e = r + 1;
  int found = -1;
  int s0 = 0;
  for (; s0 + 16 <= nr; s0 += 16) {
    Int4U v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) v[u] = *(const Int4U*)(e + s0 + 4 * u);
#pragma unroll
    for (int u = 0; u < 4; u++) {
      found = (v[u].x == a && s0 + 4 * u < cnt) ? s0 + 4 * u : found;
      found = (v[u].y == a && s0 + 4 * u + 1 < cnt) ? s0 + 4 * u + 1 : found;
      found = (v[u].z == a && s0 + 4 * u + 2 < cnt) ? s0 + 4 * u + 2 : found;
      found = (v[u].w == a && s0 + 4 * u + 3 < cnt) ? s0 + 4 * u + 3 : found;
    }
  }
  for (; s0 < nr; s0 += 4) {   // ragged end of the row, entry by entry (never beyond the row)
    int v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) v[u] = s0 + u < nr ? e[s0 + u] : -1;
#pragma unroll
    for (int u = 0; u < 4; u++) found = (v[u] == a && s0 + u < cnt) ? s0 + u : found;
  }
  // (padded entries hold 0, which is also an atom: only slots below the count are the centre's neighbours)
  return found;
}

// One thread per (frame, centre, slot) of a map [nf, ld (Nl used), nr+1]: the push pass of a transpose built by a
// force op itself.  Centres are numbered from 0 at the first row of the view.
static __global__ __launch_bounds__(TR_BLOCK) void transpose_push_kernel(const int* __restrict__ im2, int* build_cnt,
                                                                         int* keys, int cap, int* status, int nf,
                                                                         int Nrecv, int Nl, int ld, int nr) {
  const int t = blockIdx.x * TR_BLOCK + threadIdx.x;
  const int total = nf * Nl * nr;
  if (t >= total) return;
  const int s = t % nr;
  const int atom = t / nr;
  const int b = atom / Nl, p = atom - b * Nl;
  const int* im = im2 + ((size_t)b * ld + p) * (nr + 1);
  int cnt = im[0];
  if (cnt > nr) cnt = nr;
  if (s >= cnt) return;
  const int nj = im[1 + s];
  if (nj < 0 || nj >= Nrecv) { atomicOr(status, 2); return; }
  transpose_push(build_cnt, keys, cap, (size_t)b * Nrecv + nj, p, s, status);
}

// One wave per receiving atom: its keys are put in ascending order in place, the final count goes to cnt and the
// build counter back to 0 for the next build.
static __global__ __launch_bounds__(TR_BLOCK) void transpose_sort_kernel(int* build_cnt, int* __restrict__ cnt,
                                                                         int* keys, int cap, int n_recv) {
  extern __shared__ __align__(16) unsigned char smem[];
  int* w_key = (int*)smem;   // [TR_WAVES][cap]
  const int wave = threadIdx.x / WAVE, lane = lane_id();
  int* key = w_key + wave * cap;
  const int recv = blockIdx.x * TR_WAVES + wave;
  if (recv >= n_recv) return;
  int L = uniform(build_cnt[recv]);
  if (L > cap) L = cap;
  int* mine = keys + (size_t)recv * cap;
  for (int e = lane; e < L; e += WAVE) key[e] = mine[e];
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();
  if (lane == 0) {
    cnt[recv] = L;
    if (L > 0) build_cnt[recv] = 0;
  }
  for (int e = lane; e < L; e += WAVE) {
    const int ke = key[e];
    int rank = 0;
    for (int o = 0; o < L; o++) rank += (key[o] < ke) ? 1 : 0;   // keys of one receiver are distinct
    mine[rank] = ke;
  }
}

inline void launch_transpose_sort(const TransposeRef& t, int n_recv, hipStream_t stream) {
  hipLaunchKernelGGL(transpose_sort_kernel, dim3((n_recv + TR_WAVES - 1) / TR_WAVES), dim3(TR_BLOCK),
                     (size_t)TR_WAVES * t.cap * sizeof(int), stream, t.build_cnt, t.cnt, t.keys, t.cap, n_recv);
}

}  // namespace staf
