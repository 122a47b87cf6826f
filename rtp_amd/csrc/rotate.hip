// Shard rotation on one GPU: a two-slot staging buffer fed by a copy kernel on a side stream, fenced
// against the consuming stream with events, plus the error/device plumbing of the C ABI.
#include "common.h"

#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace rtp {

char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

struct ProfileRecord {
  hipEvent_t start, stop;  // host-recorded timing events, or null when the launch stamps a device slot
  int slot;                // index into the device stamp buffer, or -1
  const char* name;
  double flops, bytes;
};
static std::mutex g_profile_mutex;
static int g_profile_mode = 0;  // 0 off, 1 HIP events around every launch, 2 device time stamps (GEMM kernels)
static std::vector<ProfileRecord> g_profile_records;
// Mode 2: a launch that supports it receives a slot of two 64-bit words in device memory; its first workgroup to
// start stores the earliest value of the constant-rate wall clock there (atomic min), its last to end the latest
// (atomic max).  The slot address is a kernel argument, so a launch recorded into a HIP graph stamps its slot at
// every replay -- which HIP timing events recorded during a capture do not do.
constexpr int kTraceSlots = 8192;
// Words of a slot: earliest start, latest end, then sums over the launch's workgroups of the wall-clock ticks from the
// launch's... (see ProfileScope::trace_slot): [2] workgroup start, [3] entry -> first operands in LDS, [4] the K loop,
// [5] the epilogue, [6] the number of workgroups that reported.
constexpr int kTraceWords = 8;
static unsigned long long* g_trace_buf = nullptr;
static int g_trace_next = 0;

ProfileScope::ProfileScope(hipStream_t stream, const char* name, double flops, double bytes)
    : stream_(stream), name_(name), flops_(flops), bytes_(bytes) {
  if (g_profile_mode != 1) return;
  // Timing events recorded while a stream is captured read 0 after a replay (observed): such launches are not timed
  // in this mode -- device time stamps (mode 2) are for them.
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream_, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return;
  if (hipEventCreate(&start_) != hipSuccess) {
    start_ = nullptr;
    return;
  }
  (void)hipEventRecord(start_, stream_);
}

ProfileScope::~ProfileScope() {
  if (!start_) return;
  hipEvent_t stop = nullptr;
  if (hipEventCreate(&stop) != hipSuccess) {
    (void)hipEventDestroy(start_);
    return;
  }
  (void)hipEventRecord(stop, stream_);
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  g_profile_records.push_back({start_, stop, -1, name_, flops_, bytes_});
}

unsigned long long* ProfileScope::trace_slot() {
  if (g_profile_mode != 2) return nullptr;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  if (!g_trace_buf || g_trace_next >= kTraceSlots) return nullptr;
  const int slot = g_trace_next++;
  g_profile_records.push_back({nullptr, nullptr, slot, name_, flops_, bytes_});
  return g_trace_buf + kTraceWords * (size_t)slot;
}

__global__ void trace_reset_kernel(unsigned long long* buf, int slots) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < slots) {
    buf[kTraceWords * i] = ~0ull;
#pragma unroll
    for (int w = 1; w < kTraceWords; ++w) buf[kTraceWords * i + w] = 0ull;
  }
}

struct Ring {
  hipStream_t side = nullptr;
  hipEvent_t join = nullptr;  // a point on the consuming stream the side stream must not run ahead of
  hipEvent_t copied[2] = {nullptr, nullptr};
  hipEvent_t consumed[2] = {nullptr, nullptr};
  bool consumed_pending[2] = {false, false};
  bool join_recorded = false;  // `join` holds a fence that the next prefetch still has to wait for
  bool need_join = true;       // nothing orders the side stream after the consuming stream yet
  int device = -1;
};

static bool is_capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) return false;
  return st == hipStreamCaptureStatusActive;
}

// 16 bytes per thread per iteration, grid-stride; the ragged head/tail (when the two pointers share
// an alignment phase) and fully unaligned pairs go byte by byte.
__global__ __launch_bounds__(256) void copy_kernel(char* dst, const char* src, size_t bytes, int aligned) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t nthreads = (size_t)gridDim.x * blockDim.x;
  if (aligned) {
    const size_t nvec = bytes >> 4;
    const uint4* s = reinterpret_cast<const uint4*>(src);
    uint4* d = reinterpret_cast<uint4*>(dst);
    size_t i = tid;
    for (; i + 3 * nthreads < nvec; i += 4 * nthreads) {
      // the source is read once per pass; the destination is about to be read by the matrix products
      uint4 v0 = nt_load(s + i), v1 = nt_load(s + i + nthreads), v2 = nt_load(s + i + 2 * nthreads),
            v3 = nt_load(s + i + 3 * nthreads);
      d[i] = v0;
      d[i + nthreads] = v1;
      d[i + 2 * nthreads] = v2;
      d[i + 3 * nthreads] = v3;
    }
    for (; i < nvec; i += nthreads) d[i] = s[i];
    for (size_t b = (nvec << 4) + tid; b < bytes; b += nthreads) dst[b] = src[b];
  } else {
    for (size_t b = tid; b < bytes; b += nthreads) dst[b] = src[b];
  }
}

// Reads `bytes` at `src` and keeps nothing: the lines end up in the 256 MiB memory-side cache (and pass through the
// L2), from where the products that need them next take them at cached-operand speed.  Weights are read once per
// pass, so at their turn they would otherwise come from HBM, whose latency the products' load pipeline does not
// cover.  One workgroup per CU, like the background copy: the kernel runs under the products of the layer before.
__global__ __launch_bounds__(256) void warm_kernel(const char* src, size_t bytes, unsigned* sink, int nt) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t nthreads = (size_t)gridDim.x * blockDim.x;
  const size_t nvec = bytes >> 4;
  const uint4* s = reinterpret_cast<const uint4*>(src);
  unsigned acc = 0;
  size_t i = tid;
  if (nt) {
    for (; i + 3 * nthreads < nvec; i += 4 * nthreads) {
      const uint4 v0 = nt_load(s + i), v1 = nt_load(s + i + nthreads), v2 = nt_load(s + i + 2 * nthreads),
                  v3 = nt_load(s + i + 3 * nthreads);
      acc |= v0.x & v1.x & v2.x & v3.x;
    }
  } else {
    for (; i + 3 * nthreads < nvec; i += 4 * nthreads) {
      const uint4 v0 = s[i], v1 = s[i + nthreads], v2 = s[i + 2 * nthreads], v3 = s[i + 3 * nthreads];
      acc |= v0.x & v1.x & v2.x & v3.x;
    }
  }
  for (; i < nvec; i += nthreads) acc |= s[i].x;
  // never true for the value the host passes (sink == nullptr): the loads cannot be optimised away
  if (sink != nullptr && acc == 0x9e3779b9u) *sink = acc;
}

__global__ __launch_bounds__(256) void zero_kernel(char* dst, size_t bytes, int aligned) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t nthreads = (size_t)gridDim.x * blockDim.x;
  if (aligned) {
    const size_t nvec = bytes >> 4;
    uint4* d = reinterpret_cast<uint4*>(dst);
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (size_t i = tid; i < nvec; i += nthreads) d[i] = z;
    for (size_t b = (nvec << 4) + tid; b < bytes; b += nthreads) dst[b] = 0;
  } else {
    for (size_t b = tid; b < bytes; b += nthreads) dst[b] = 0;
  }
}

// `background`: the copy runs on the ring's side stream under the matrix products of the layer before.  One
// workgroup per CU then: a grid that covers the CUs eight times over (the fastest for a copy that has the GPU to
// itself) floods every CU's memory pipeline and the products' own loads queue behind it (measured on the 10-layer LM
// step: 4.30 ms with 2048 workgroups, 4.24 ms with 256, 4.28 ms with 128, 4.49 ms with 64).
static unsigned copy_grid(size_t bytes, bool background) {
  static const size_t cap_env = [] {
    const char* e = getenv("RTP_COPY_BLOCKS");
    return e ? (size_t)atoi(e) : (size_t)0;
  }();
  const size_t cap = background ? (cap_env ? cap_env : (size_t)256) : (size_t)2048;
  size_t blocks = (bytes + 4095) / 4096;
  if (blocks < 1) blocks = 1;
  if (blocks > cap) blocks = cap;
  return (unsigned)blocks;
}

static int launch_copy(hipStream_t s, void* dst, const void* src, size_t bytes, bool background) {
  if (bytes == 0) return RTP_OK;
  RTP_REQUIRE(dst && src, "shard copy: null pointer");
  const int aligned = (((uintptr_t)dst | (uintptr_t)src) & 15) == 0;
  ProfileScope prof(s, "shard_copy", 0.0, 2.0 * (double)bytes);
  hipLaunchKernelGGL(copy_kernel, dim3(copy_grid(bytes, background)), dim3(256), 0, s, (char*)dst, (const char*)src,
                     bytes, aligned);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

}  // namespace rtp

using namespace rtp;

extern "C" const char* rtp_last_error(void) { return error_buffer(); }

extern "C" int rtp_abi_version(void) { return 5; }

extern "C" int rtp_device_check(char* name_out, int name_len) {
  int dev = 0;
  RTP_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  RTP_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  if (name_out && name_len > 0) {
    strncpy(name_out, prop.gcnArchName, (size_t)name_len - 1);
    name_out[name_len - 1] = 0;
  }
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(RTP_ERR_DEVICE, "device %d is %s; this library is built for gfx950 only", dev, prop.gcnArchName);
  // per-device set-up: the address of the built-in scratch of rtp_gate_wgrad_static on this device
  return gate_static_setup();
}

extern "C" int rtp_cache_warm(void* stream, const void* src, size_t bytes, int flags) {
  if (bytes == 0) return RTP_OK;
  RTP_REQUIRE(src && ((uintptr_t)src & 15) == 0, "rtp_cache_warm: source must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  ProfileScope prof(s, "cache_warm", 0.0, (double)bytes);
  hipLaunchKernelGGL(warm_kernel, dim3(copy_grid(bytes, true)), dim3(256), 0, s, (const char*)src, bytes,
                     (unsigned*)nullptr, flags & 1);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_ring_create(void** ring_out) {
  RTP_REQUIRE(ring_out, "rtp_ring_create: null out pointer");
  Ring* r = new Ring();
  RTP_HIP_TRY(hipGetDevice(&r->device));
  // Default priority on purpose: mixed stream priorities are not used anywhere in this library.
  RTP_HIP_TRY(hipStreamCreateWithFlags(&r->side, hipStreamNonBlocking));
  RTP_HIP_TRY(hipEventCreateWithFlags(&r->join, hipEventDisableTiming));
  for (int i = 0; i < 2; ++i) {
    RTP_HIP_TRY(hipEventCreateWithFlags(&r->copied[i], hipEventDisableTiming));
    RTP_HIP_TRY(hipEventCreateWithFlags(&r->consumed[i], hipEventDisableTiming));
  }
  *ring_out = r;
  return RTP_OK;
}

extern "C" int rtp_ring_destroy(void* ring) {
  if (!ring) return RTP_OK;
  Ring* r = (Ring*)ring;
  if (r->side) (void)hipStreamSynchronize(r->side);
  for (int i = 0; i < 2; ++i) {
    if (r->copied[i]) (void)hipEventDestroy(r->copied[i]);
    if (r->consumed[i]) (void)hipEventDestroy(r->consumed[i]);
  }
  if (r->join) (void)hipEventDestroy(r->join);
  if (r->side) (void)hipStreamDestroy(r->side);
  delete r;
  return RTP_OK;
}

extern "C" int rtp_ring_fence(void* ring, void* main_stream) {
  RTP_REQUIRE(ring, "rtp_ring_fence: null ring");
  Ring* r = (Ring*)ring;
  RTP_HIP_TRY(hipEventRecord(r->join, (hipStream_t)main_stream));
  r->join_recorded = true;
  r->need_join = true;
  // everything that consumed a slot so far is queued before the fence
  r->consumed_pending[0] = r->consumed_pending[1] = false;
  return RTP_OK;
}

extern "C" int rtp_ring_prefetch(void* ring, void* main_stream, int slot, void* dst, const void* src,
                                 size_t bytes) {
  RTP_REQUIRE(ring, "rtp_ring_prefetch: null ring");
  RTP_REQUIRE(slot == 0 || slot == 1, "rtp_ring_prefetch: slot %d not in {0,1}", slot);
  Ring* r = (Ring*)ring;
  hipStream_t main = (hipStream_t)main_stream;
  // While `main` is being captured into a graph the side stream has to be forked from it, or the copy
  // would run now instead of being recorded.
  if (is_capturing(main) && !is_capturing(r->side)) r->need_join = true, r->join_recorded = false;
  if (r->need_join) {
    if (!r->join_recorded) {
      RTP_HIP_TRY(hipEventRecord(r->join, main));
      r->consumed_pending[0] = r->consumed_pending[1] = false;
    }
    RTP_HIP_TRY(hipStreamWaitEvent(r->side, r->join, 0));
    r->need_join = false;
    r->join_recorded = false;
  }
  if (r->consumed_pending[slot]) {
    RTP_HIP_TRY(hipStreamWaitEvent(r->side, r->consumed[slot], 0));
    r->consumed_pending[slot] = false;
  }
  int rc = launch_copy(r->side, dst, src, bytes, true);
  if (rc != RTP_OK) return rc;
  RTP_HIP_TRY(hipEventRecord(r->copied[slot], r->side));
  return RTP_OK;
}

extern "C" int rtp_ring_acquire(void* ring, void* main_stream, int slot) {
  RTP_REQUIRE(ring, "rtp_ring_acquire: null ring");
  RTP_REQUIRE(slot == 0 || slot == 1, "rtp_ring_acquire: slot %d not in {0,1}", slot);
  Ring* r = (Ring*)ring;
  RTP_HIP_TRY(hipStreamWaitEvent((hipStream_t)main_stream, r->copied[slot], 0));
  return RTP_OK;
}

extern "C" int rtp_ring_release(void* ring, void* main_stream, int slot) {
  RTP_REQUIRE(ring, "rtp_ring_release: null ring");
  RTP_REQUIRE(slot == 0 || slot == 1, "rtp_ring_release: slot %d not in {0,1}", slot);
  Ring* r = (Ring*)ring;
  RTP_HIP_TRY(hipEventRecord(r->consumed[slot], (hipStream_t)main_stream));
  r->consumed_pending[slot] = true;
  return RTP_OK;
}

extern "C" int rtp_shard_copy_async(void* stream, void* dst, const void* src, size_t bytes) {
  return launch_copy((hipStream_t)stream, dst, src, bytes, false);
}

extern "C" int rtp_zero_async(void* stream, void* dst, size_t bytes) {
  if (bytes == 0) return RTP_OK;
  RTP_REQUIRE(dst, "rtp_zero_async: null pointer");
  const int aligned = ((uintptr_t)dst & 15) == 0;
  hipLaunchKernelGGL(zero_kernel, dim3(copy_grid(bytes, false)), dim3(256), 0, (hipStream_t)stream, (char*)dst, bytes,
                     aligned);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

extern "C" int rtp_profile_enable(int mode) {
  RTP_REQUIRE(mode >= 0 && mode <= 2, "rtp_profile_enable: mode 0 (off), 1 (events) or 2 (device time stamps)");
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  if (mode == 2 && !g_trace_buf) {
    RTP_HIP_TRY(hipMalloc((void**)&g_trace_buf, sizeof(unsigned long long) * kTraceWords * kTraceSlots));
    hipLaunchKernelGGL(trace_reset_kernel, dim3((kTraceSlots + 255) / 256), dim3(256), 0, nullptr, g_trace_buf, kTraceSlots);
    RTP_LAUNCH_CHECK();
    RTP_HIP_TRY(hipDeviceSynchronize());
  }
  g_profile_mode = mode;
  return RTP_OK;
}

extern "C" int rtp_profile_reset_stamps(void* stream) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  if (!g_trace_buf || g_trace_next == 0) return RTP_OK;
  hipLaunchKernelGGL(trace_reset_kernel, dim3((g_trace_next + 255) / 256), dim3(256), 0, (hipStream_t)stream, g_trace_buf,
                     g_trace_next);
  RTP_LAUNCH_CHECK();
  return RTP_OK;
}

// Sums the recorded launches per kernel name.  `clear`: destroy the event pairs and forget the stamp slots afterwards.
// Without it the stamp slots stay booked -- what a replayed HIP graph needs whose launches carry them: every replay
// stamps them anew, and a read after a replay returns that replay's durations.
static int profile_sum(rtp_kernel_stat* out, int max_out, int* n_out, bool clear) {
  RTP_REQUIRE(out && n_out && max_out > 0, "rtp_profile_collect: bad arguments");
  RTP_HIP_TRY(hipDeviceSynchronize());
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  std::vector<unsigned long long> stamps;
  double ticks_per_ms = 1e5;  // the wall clock runs at 100 MHz unless the device says otherwise
  if (g_trace_buf && g_trace_next > 0) {
    stamps.resize((size_t)kTraceWords * g_trace_next);
    RTP_HIP_TRY(hipMemcpy(stamps.data(), g_trace_buf, stamps.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) == hipSuccess && khz > 0)
      ticks_per_ms = (double)khz;
  }
  std::map<std::string, rtp_kernel_stat> agg;
  for (const ProfileRecord& r : g_profile_records) {
    float ms = 0.0f;
    double phase[4] = {0.0, 0.0, 0.0, 0.0};
    if (r.slot >= 0) {
      const unsigned long long* w = &stamps[(size_t)kTraceWords * r.slot];
      const unsigned long long t0 = w[0], t1 = w[1];
      if (t1 < t0) continue;  // the launch did not run since the last reset
      ms = (float)((double)(t1 - t0) / ticks_per_ms);
      if (w[6] > 0) {  // per-workgroup phases, averaged over the workgroups of the launch
        const double n = (double)w[6];
        phase[0] = ((double)w[2] / n - (double)t0) / ticks_per_ms;
        for (int i = 1; i < 4; ++i) phase[i] = (double)w[2 + i] / n / ticks_per_ms;
      }
    } else {
      if (hipEventElapsedTime(&ms, r.start, r.stop) != hipSuccess) ms = 0.0f;
      if (clear) {
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
      }
    }
    rtp_kernel_stat& st = agg[r.name];
    if (st.launches == 0) {
      memset(&st, 0, sizeof(st));
      strncpy(st.name, r.name, sizeof(st.name) - 1);
    }
    st.launches += 1;
    st.total_ms += ms;
    st.flops += r.flops;
    st.bytes += r.bytes;
    for (int i = 0; i < 4; ++i) st.phase_ms[i] += phase[i];
  }
  if (clear) {
    g_profile_records.clear();
    g_trace_next = 0;
  }
  int n = 0;
  for (auto& kv : agg) {
    if (n >= max_out) break;
    out[n++] = kv.second;
  }
  *n_out = n;
  return RTP_OK;
}

extern "C" int rtp_profile_collect(rtp_kernel_stat* out, int max_out, int* n_out) {
  return profile_sum(out, max_out, n_out, true);
}

extern "C" int rtp_profile_read(rtp_kernel_stat* out, int max_out, int* n_out) {
  return profile_sum(out, max_out, n_out, false);
}
