// Library-owned per-device state: status word, scratch and scatter buckets.
#include "staf_common.hpp"
#include "staf_reduce.hpp"

#include <mutex>
#include <unordered_map>
#include <memory>
#include <stdio.h>
#include <string>
#include <utility>
#include <vector>

namespace staf {

static std::mutex g_mu;
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

DeviceState* device_state() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = g_state.find(dev);
  if (it != g_state.end()) return it->second.get();
  auto st = std::unique_ptr<DeviceState>(new DeviceState());
  st->device = dev;
  if (hipMalloc((void**)&st->status_d, sizeof(int)) != hipSuccess) return nullptr;
  // the clear runs on the legacy default stream: wait for it, callers' streams need not be ordered after that one
  if (hipMemset(st->status_d, 0, sizeof(int)) != hipSuccess || hipDeviceSynchronize() != hipSuccess) return nullptr;
  if (hipHostMalloc((void**)&st->status_h, sizeof(int), hipHostMallocDefault) != hipSuccess) return nullptr;
  *st->status_h = 0;
  DeviceState* raw = st.get();
  g_state.emplace(dev, std::move(st));
  return raw;
}

static StreamWork* stream_work(DeviceState* st, hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_mu);
  return &st->work[stream];   // references into an unordered_map stay valid when it grows
}

void* scratch_reserve(DeviceState* st, hipStream_t stream, size_t bytes) {
  StreamWork* w = stream_work(st, stream);
  if (bytes <= w->scratch.bytes) return w->scratch.buf;
  if (w->scratch.buf) {
    // hipFree waits for in-flight work that may still read the old block
    if (hipFree(w->scratch.buf) != hipSuccess) return nullptr;
    w->scratch.buf = nullptr;
    w->scratch.bytes = 0;
  }
  size_t want = bytes + bytes / 4;
  if (hipMalloc(&w->scratch.buf, want) != hipSuccess) return nullptr;
  w->scratch.bytes = want;
  return w->scratch.buf;
}

// Scatter buckets: n_counters ints (kept all-zero between calls: the gather
// kernel clears every counter it consumes) followed by n_entries ints.
int* bucket_reserve(DeviceState* st, size_t n_counters, size_t n_entries, hipStream_t stream, int** entries) {
  StreamWork* w = stream_work(st, stream);
  if (n_counters > w->bucket_counters || n_entries > w->bucket_entries) {
    if (w->buckets.buf) {
      if (hipFree(w->buckets.buf) != hipSuccess) return nullptr;
      w->buckets.buf = nullptr;
      w->buckets.bytes = 0;
    }
    size_t cnt = n_counters + n_counters / 4;
    size_t ent = n_entries + n_entries / 4;
    size_t want = (cnt + ent) * sizeof(int);
    if (hipMalloc(&w->buckets.buf, want) != hipSuccess) return nullptr;
    // cleared on the caller's stream, ahead of the kernels that count into it (a clear on the default stream is
    // not ordered before work on a non-blocking stream)
    launch_fill_zero<int>((int*)w->buckets.buf, (int)cnt, stream);
    if (hipGetLastError() != hipSuccess) return nullptr;
    w->buckets.bytes = want;
    w->bucket_counters = cnt;
    w->bucket_entries = ent;
  }
  *entries = (int*)w->buckets.buf + w->bucket_counters;
  return (int*)w->buckets.buf;
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
  return STAF_OK;
}

static int fetch_status(DeviceState* st, hipStream_t stream) {
  if (hipMemcpyAsync(st->status_h, st->status_d, sizeof(int), hipMemcpyDeviceToHost, stream) != hipSuccess)
    return STAF_E_HIP;
  if (hipStreamSynchronize(stream) != hipSuccess) return STAF_E_HIP;
  int bits = *st->status_h;
  if (bits) {
    if (hipMemsetAsync(st->status_d, 0, sizeof(int), stream) != hipSuccess) return STAF_E_HIP;
    if (hipStreamSynchronize(stream) != hipSuccess) return STAF_E_HIP;
  }
  return decode_status(bits);
}

int finish_op(DeviceState* st, hipStream_t stream) {
  if (hipGetLastError() != hipSuccess) return STAF_E_HIP;
  if (!sync_errors_enabled()) return STAF_OK;
  return fetch_status(st, stream);
}

}  // namespace staf

extern "C" {

const char* staf_ops_version(void) { return "0.1"; }

void staf_ops_set_sync_errors(int mode) { staf::g_sync_errors = mode ? 1 : 0; }

int staf_ops_poll_status(void* stream) {
  staf::DeviceState* st = staf::device_state();
  if (!st) return STAF_E_HIP;
  return staf::fetch_status(st, (hipStream_t)stream);
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
  auto it = staf::g_state.find(dev);
  if (it == staf::g_state.end()) return;
  staf::DeviceState* st = it->second.get();
  (void)hipDeviceSynchronize();
  for (auto& kv : st->work) {
    if (kv.second.scratch.buf) (void)hipFree(kv.second.scratch.buf);
    if (kv.second.buckets.buf) (void)hipFree(kv.second.buckets.buf);
  }
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
