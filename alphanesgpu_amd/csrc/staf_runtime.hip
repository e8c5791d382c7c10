// Library-owned per-device state: status word, scratch and scatter buckets.
#include "staf_common.hpp"
#include "staf_reduce.hpp"

#include <atomic>
#include <mutex>
#include <unordered_map>
#include <memory>
#include <stdio.h>
#include <string>
#include <utility>
#include <vector>

namespace staf {

static std::mutex g_mu;
static std::atomic<unsigned> g_release_epoch{0};
unsigned release_epoch() { return g_release_epoch.load(); }
static std::unordered_map<int, std::unique_ptr<DeviceState>> g_state;
static int g_sync_errors = 1;
// Calls made by this thread leave their device-detected conditions in the status word (no synchronisation per op)
// while the count is positive: the MD entry runs its whole op sequence this way and reads the word once at the end.
static thread_local int tl_defer_status = 0;
DeferStatus::DeferStatus() { ++tl_defer_status; }
DeferStatus::~DeferStatus() { --tl_defer_status; }

bool sync_errors_enabled() { return g_sync_errors != 0 && tl_defer_status == 0; }

static int g_kernel_timing = 0;
static std::unordered_map<std::string, std::vector<std::pair<hipEvent_t, hipEvent_t>>> g_kernel_events;
bool kernel_timing_enabled() { return g_kernel_timing != 0; }
void kernel_timing_record(const char* kernel, hipEvent_t a, hipEvent_t b) {
  std::lock_guard<std::mutex> lock(g_mu);
  g_kernel_events[kernel].emplace_back(a, b);
}

DeviceState* device_state(hipStream_t stream) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_state.find(dev);
  if (it != g_state.end()) return it->second.get();
  // the first call on a device allocates and synchronises: not while the caller's stream is being captured
  if (stream_is_capturing(stream)) return nullptr;
  auto st = std::unique_ptr<DeviceState>(new DeviceState());
  st->device = dev;
  if (hipMalloc((void**)&st->status_d, STATUS_WORDS * sizeof(int)) != hipSuccess) return nullptr;
  // the clear runs on the legacy default stream: wait for it, callers' streams need not be ordered after that one
  if (hipMemset(st->status_d, 0, STATUS_WORDS * sizeof(int)) != hipSuccess || hipDeviceSynchronize() != hipSuccess)
    return nullptr;
  if (hipHostMalloc((void**)&st->status_h, STATUS_WORDS * sizeof(int), hipHostMallocDefault) != hipSuccess)
    return nullptr;
  for (int w = 0; w < STATUS_WORDS; w++) st->status_h[w] = 0;
  DeviceState* raw = st.get();
  g_state.emplace(dev, std::move(st));
  return raw;
}

int* status_word(DeviceState* st, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = st->status_slot.find(stream);
  if (it == st->status_slot.end()) {
    const int n = (int)st->status_slot.size();
    it = st->status_slot.emplace(stream, n < STATUS_WORDS ? n : STATUS_WORDS - 1).first;
  }
  return st->status_d + it->second;
}

static StreamWork* stream_work(DeviceState* st, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mu);
  return &st->work[stream];   // references into an unordered_map stay valid when it grows
}

bool stream_is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cs) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return cs != hipStreamCaptureStatusNone;
}

int reserve_failure(hipStream_t stream) { return stream_is_capturing(stream) ? STAF_E_CAPTURE : STAF_E_HIP; }

// A block that has become too small is not freed but retired until staf_ops_release: kernels in flight, and graphs
// instantiated while it was current, may still address it.  Blocks grow by half, so the retired ones of a work area
// add up to less than twice its final size.
static bool grow(DeviceState* st, Workspace* w, size_t bytes, hipStream_t stream) {
  if (stream_is_capturing(stream)) return false;
  void* fresh = nullptr;
  const size_t want = bytes + bytes / 2;
  if (hipMalloc(&fresh, want) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  if (w->buf) st->retired.push_back(w->buf);
  w->buf = fresh;
  w->bytes = want;
  return true;
}

void* scratch_reserve(DeviceState* st, hipStream_t stream, size_t bytes) {
  StreamWork* w = stream_work(st, stream);
  if (bytes <= w->scratch.bytes) return w->scratch.buf;
  std::lock_guard<std::mutex> lock(g_mu);
  return grow(st, &w->scratch, bytes, stream) ? w->scratch.buf : nullptr;
}

// Layout of a cell-list block: [toggle, padded to 256 bytes | two counter sets | this call's tables and records].
bool cells_reserve(DeviceState* st, hipStream_t stream, size_t counters, size_t rest_bytes, CellBlock* out) {
  constexpr size_t HEAD = 64;   // ints
  StreamWork* w = stream_work(st, stream);
  std::lock_guard<std::mutex> lock(g_mu);
  counters = (counters + 63) / 64 * 64;
  const size_t have = w->cell_counters;
  const size_t cnt = counters > have ? counters : have;
  const size_t bytes = (HEAD + 2 * cnt) * sizeof(int) + rest_bytes;
  if (cnt > have || bytes > w->cells.bytes) {
    if (!grow(st, &w->cells, bytes, stream)) return false;
    w->cell_counters = cnt;
    launch_fill_zero<int>((int*)w->cells.buf, (int)(HEAD + 2 * cnt), stream);
    if (hipGetLastError() != hipSuccess) return false;
  }
  out->toggle = (int*)w->cells.buf;
  out->counts = out->toggle + HEAD;
  out->set_ints = w->cell_counters;
  out->rest = (char*)(out->counts + 2 * w->cell_counters);
  return true;
}

// Layout of a transpose block: [build counters | counts | keys].  The build counters must read zero when a build
// starts: a fresh block is cleared once, on the caller's stream (a clear on the default stream is not ordered
// before work on a non-blocking stream), and every build's sort pass leaves them at zero again.
static bool transpose_block(DeviceState* st, Workspace* buf, size_t* cap_recv, size_t* cap_keys, size_t n_recv,
                            size_t n_keys, hipStream_t stream) {
  if (n_recv > *cap_recv || n_keys > *cap_keys) {
    const size_t r = n_recv > *cap_recv ? n_recv : *cap_recv;
    const size_t k = n_keys > *cap_keys ? n_keys : *cap_keys;
    if (!grow(st, buf, (2 * r + k) * sizeof(int), stream)) return false;
    // the whole grown block is handed out in the same proportions
    const size_t have = buf->bytes / sizeof(int);
    *cap_recv = r + (have - (2 * r + k)) / 4;
    *cap_keys = have - 2 * *cap_recv;
    launch_fill_zero<int>((int*)buf->buf, (int)*cap_recv, stream);
    if (hipGetLastError() != hipSuccess) return false;
  }
  return true;
}

bool bucket_reserve(DeviceState* st, size_t n_recv, int cap, hipStream_t stream, TransposeRef* out) {
  StreamWork* w = stream_work(st, stream);
  std::lock_guard<std::mutex> lock(g_mu);
  if (!transpose_block(st, &w->buckets, &w->bucket_counters, &w->bucket_entries, n_recv, n_recv * cap, stream))
    return false;
  *out = TransposeRef();
  out->build_cnt = (int*)w->buckets.buf;
  out->cnt = out->build_cnt + w->bucket_counters;
  out->keys = out->cnt + w->bucket_counters;
  out->cap = cap;
  out->key_shift = 0;
  return true;
}

bool transpose_for_descriptor(DeviceState* st, const int* im2, int nf, int N, int Nrecv, int nr, int cap,
                              bool symmetric, hipStream_t stream, TransposeRef* out) {
  std::lock_guard<std::mutex> lock(g_mu);
  // a symmetric map needs no transpose, only one word per row for the rows' checksums (the counter part of a block)
  const size_t want_recv = (size_t)nf * Nrecv, want_keys = symmetric ? 0 : want_recv * cap;
  Transpose* t = nullptr;
  for (auto& e : st->transposes)
    if (e.im2 == im2) { t = &e; break; }
  if (!t) {
    // A tensor not seen before takes the place that has not been used for the longest time.  Under capture nothing
    // can be allocated, so only places whose block is already large enough qualify (a graph recorded earlier with
    // such a place rebuilds the transpose in it on every replay, before it reads it).
    const bool capturing = stream_is_capturing(stream);
    for (auto& e : st->transposes) {
      if (capturing && !symmetric && (e.cap_recv < want_recv || e.cap_keys < want_keys)) continue;
      if (!t || e.stamp < t->stamp) t = &e;
    }
    if (!t) return false;
  }
  // (a symmetric map whose place has no block for the checksums and cannot get one now -- a tensor first seen while
  // its stream is captured -- goes without them)
  bool have_block = true;
  if (symmetric && stream_is_capturing(stream) && (t->cap_recv < want_recv))
    have_block = false;
  else if (!transpose_block(st, &t->buf, &t->cap_recv, &t->cap_keys, want_recv, want_keys, stream))
    return false;
  t->im2 = im2; t->nf = nf; t->N = N; t->Nrecv = Nrecv; t->nr = nr;
  t->ref = TransposeRef();
  t->ref.symmetric = symmetric ? 1 : 0;
  t->ref.full = im2;
  if (symmetric && have_block) t->ref.rowsum = (const unsigned*)t->buf.buf;
  if (!symmetric) {
    t->ref.build_cnt = (int*)t->buf.buf;
    t->ref.cnt = t->ref.build_cnt + t->cap_recv;
    t->ref.keys = t->ref.cnt + t->cap_recv;
    t->ref.cap = cap;
  }
  t->stamp = ++st->transpose_clock;
  *out = t->ref;
  return true;
}

bool transpose_find(DeviceState* st, const int* im2_view, int nf, int Nrecv, int Nl, int ld, int nr,
                    TransposeRef* out) {
  std::lock_guard<std::mutex> lock(g_mu);
  for (auto& e : st->transposes) {
    if (!e.im2 || e.nr != nr || e.nf != nf || e.Nrecv != Nrecv || e.N != ld) continue;
    if (im2_view < e.im2) continue;
    const size_t off = (size_t)(im2_view - e.im2);
    if (off % (size_t)(nr + 1)) continue;
    const size_t first = off / (size_t)(nr + 1);
    if (first + (size_t)Nl > (size_t)e.N) continue;
    e.stamp = ++st->transpose_clock;
    *out = e.ref;
    out->key_shift = (int)first;
    return true;
  }
  return false;
}

template <typename real>
__global__ void add_n_kernel(real* dst, const real* a, const real* b, const real* c, const real* d, int n) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= n) return;
  real s = a[e] + b[e];
  if (c) s += c[e];
  if (d) s += d[e];
  dst[e] = s;
}

template <typename real>
static int add_n(real* dst, const real* a, const real* b, const real* c, const real* d, int n, void* stream) {
  if (!dst || !a || !b || n <= 0 || (d && !c)) return STAF_E_BAD_ARG;
  hipLaunchKernelGGL(add_n_kernel<real>, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream, dst, a, b, c, d, n);
  return hipGetLastError() == hipSuccess ? STAF_OK : STAF_E_HIP;
}

static int decode_status(int bits) {
  if (bits & 1) return STAF_E_RADIAL_OVERFLOW;
  if (bits & 2) return STAF_E_SCATTER_OVERFLOW;
  if (bits & 4) return STAF_E_STALE_MAP;
  return STAF_OK;
}

// Clears in every error word exactly the bits the host has just read: a bit a kernel of another stream sets between
// the read and this clear stays for the next poll (a plain fill of the words would lose it).
struct StatusSeen { int bits[STATUS_WORDS]; };
__global__ void status_clear_kernel(int* word, StatusSeen seen, int nw) {
  const int w = threadIdx.x;
  if (w < nw && seen.bits[w]) atomicAnd(&word[w], ~seen.bits[w]);
}

// Reads and clears, after waiting for `stream`, the stream's own error word (all = false) or every word of the
// device (all = true: the poll, whose caller has waited for the other streams itself).
static int fetch_status(DeviceState* st, hipStream_t stream, bool all) {
  static std::mutex mirror_mu;   // one pinned mirror per device
  std::lock_guard<std::mutex> lock(mirror_mu);
  int* word = all ? st->status_d : status_word(st, stream);
  const int nw = all ? STATUS_WORDS : 1;
  int* host = st->status_h + (word - st->status_d);
  if (hipMemcpyAsync(host, word, nw * sizeof(int), hipMemcpyDeviceToHost, stream) != hipSuccess) return STAF_E_HIP;
  if (hipStreamSynchronize(stream) != hipSuccess) return STAF_E_HIP;
  int bits = 0;
  StatusSeen seen;
  for (int w = 0; w < STATUS_WORDS; w++) seen.bits[w] = w < nw ? host[w] : 0;
  for (int w = 0; w < nw; w++) bits |= host[w];
  if (bits) {
    hipLaunchKernelGGL(status_clear_kernel, dim3(1), dim3(STATUS_WORDS), 0, stream, word, seen, nw);
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) return STAF_E_HIP;
    if (bits & 4) {
      // A remembered neighbour map no longer holds what the descriptor op wrote: nothing remembered is trusted any
      // more.  Force ops then transpose the map they are handed themselves until the descriptor op writes again.
      std::lock_guard<std::mutex> lock2(g_mu);
      for (auto& e : st->transposes) e.im2 = nullptr;
    }
  }
  return decode_status(bits);
}

int finish_op(DeviceState* st, hipStream_t stream) {
  if (hipGetLastError() != hipSuccess) return STAF_E_HIP;
  if (!sync_errors_enabled()) return STAF_OK;
  // A stream that is being captured cannot be waited for (and the copy and the clear would become nodes of the
  // graph): the condition stays in the status word for staf_ops_poll_status after a replay.
  if (stream_is_capturing(stream)) return STAF_OK;
  return fetch_status(st, stream, false);
}

}  // namespace staf

extern "C" {

const char* staf_ops_version(void) { return "0.1"; }

void staf_ops_set_sync_errors(int mode) { staf::g_sync_errors = mode ? 1 : 0; }

int staf_ops_poll_status(void* stream) {
  staf::DeviceState* st = staf::device_state((hipStream_t)stream);
  if (!st) return staf::reserve_failure((hipStream_t)stream);
  return staf::fetch_status(st, (hipStream_t)stream, true);
}

void staf_ops_kernel_timing(int enable) { staf::g_kernel_timing = enable ? 1 : 0; }

int staf_ops_kernel_time(const char* kernel, double* total_ms, int* launches) {
  if (!kernel || !total_ms || !launches) return STAF_E_BAD_ARG;
  if (hipDeviceSynchronize() != hipSuccess) return STAF_E_HIP;
  std::lock_guard<std::mutex> lock(staf::g_mu);
  *total_ms = 0.0;
  *launches = 0;
  auto it = staf::g_kernel_events.find(kernel);
  if (it == staf::g_kernel_events.end()) return STAF_OK;
  for (auto& ev : it->second) {
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, ev.first, ev.second) == hipSuccess) { *total_ms += ms; ++*launches; }
    (void)hipEventDestroy(ev.first);
    (void)hipEventDestroy(ev.second);
  }
  it->second.clear();
  return STAF_OK;
}

void staf_ops_release(void) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return;
  std::lock_guard<std::mutex> lock(staf::g_mu);
  staf::g_release_epoch++;
  auto it = staf::g_state.find(dev);
  if (it == staf::g_state.end()) return;
  staf::DeviceState* st = it->second.get();
  (void)hipDeviceSynchronize();
  for (auto& kv : st->work) {
    if (kv.second.scratch.buf) (void)hipFree(kv.second.scratch.buf);
    if (kv.second.buckets.buf) (void)hipFree(kv.second.buckets.buf);
    if (kv.second.cells.buf) (void)hipFree(kv.second.cells.buf);
  }
  for (auto& t : st->transposes)
    if (t.buf.buf) (void)hipFree(t.buf.buf);
  for (void* p : st->retired) (void)hipFree(p);
  if (st->status_d) (void)hipFree(st->status_d);
  if (st->status_h) (void)hipHostFree(st->status_h);
  staf::g_state.erase(it);
}

int staf_op_add_n_f32(float* dst, const float* a, const float* b, const float* c, const float* d, int n,
                      void* stream) {
  return staf::add_n<float>(dst, a, b, c, d, n, stream);
}
int staf_op_add_n_f64(double* dst, const double* a, const double* b, const double* c, const double* d, int n,
                      void* stream) {
  return staf::add_n<double>(dst, a, b, c, d, n, stream);
}

int staf_op_init_force_radial(int buffdim) { return buffdim > 0 ? STAF_OK : STAF_E_BAD_ARG; }
int staf_op_init_force_tripl(int buffdim) { return buffdim > 0 ? STAF_OK : STAF_E_BAD_ARG; }
int staf_op_init_grad_force_radial(int buffdim) { return buffdim > 0 ? STAF_OK : STAF_E_BAD_ARG; }
int staf_op_init_grad_force_tripl(int buffdim) { return buffdim > 0 ? STAF_OK : STAF_E_BAD_ARG; }

}  // extern "C"
