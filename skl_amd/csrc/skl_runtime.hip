// skl_runtime.hip - the runtime shim declared in include/skl-hip.h: device
// selection, buffers, the per-thread stream, pointer classification and the
// thread-local error channel of the `void` kernel entry points.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

#include "../../include/skl-hip.h"
#include "skl_device.hpp"

namespace {

constexpr int kMaxDevices = 16;

// A block that only ever grows. The block it replaces is kept until shutdown: another thread may have been
// handed its address and not launched yet, and kernels in flight may still use it.
struct Scratch {
  void *ptr = nullptr;
  size_t bytes = 0;
};

// Scratch memory belongs to one stream of one device: kernels of different streams may run at the same time, and
// each scratch block carries data from one kernel to the next (or between the workgroups of one kernel).
struct StreamState {
  hipStream_t stream = nullptr;
  Scratch workspace;       // partial sums of the split reductions (never more than kWorkspaceBytes are asked for)
  Scratch operands;        // copies of operands in another layout; apart from the workspace so that a launch which
                           // uses the workspace keeps the copies it was given
  Scratch converted;       // an operand converted to another element type ahead of a GEMM that may itself copy operands
  void *zeroed = nullptr;  // block that is zero between launches (sums and counters shared by workgroups)
  size_t zeroed_bytes = 0;
  std::vector<void *> retired;  // blocks this stream outgrew: kept while work that was handed their address may still
                                // run, freed when the stream is released (or at shutdown)
};

// Streams with scratch of their own per device. A further stream gets none (its calls run on the kernels that need
// no scratch and an error is recorded) until skl_hip_release_stream() has given a slot back.
constexpr size_t kMaxStreamStates = 32;

struct DeviceState {
  std::vector<StreamState> streams;
};

constexpr size_t kWorkspaceBytes = size_t(64) << 20;
constexpr size_t kOperandBytes = size_t(4) << 20;

std::mutex g_mutex;
DeviceState g_devices[kMaxDevices];

thread_local hipStream_t t_stream = nullptr;
thread_local int t_pointer_mode = SKL_HIP_POINTERS_AUTO;
thread_local int t_beta_zero_mode = -1;  // not set by this thread: the process's default (the environment) counts
thread_local int t_error = SKL_HIP_OK;
thread_local char t_error_text[256] = "no error";

}  // namespace

extern "C" void skl_hip_withdraw_error(int code) {
  if (t_error == code) t_error = SKL_HIP_OK;
}

extern "C" int skl_hip_pending_error(void) { return t_error; }

extern "C" void skl_hip_record_error(int code, const char *what) {
  if (code == SKL_HIP_OK || t_error != SKL_HIP_OK) return;  // keep the first error until it is read
  t_error = code;
  const char *detail = "";
  if (code > 0) detail = hipGetErrorString((hipError_t)code);
  else if (code == SKL_HIP_ERR_MIXED_POINTERS) detail = "host and device pointers mixed in one call";
  else if (code == SKL_HIP_ERR_BAD_ARGUMENT) detail = "bad argument";
  else if (code == SKL_HIP_ERR_NO_DEVICE) detail = "no usable GPU";
  else if (code == SKL_HIP_ERR_WORKSPACE) detail = "workspace allocation failed";
  snprintf(t_error_text, sizeof t_error_text, "%s: %s", what ? what : "skl", detail);
}

int skl_check_hip(hipError_t e, const char *what) {
  if (e == hipSuccess) return SKL_HIP_OK;
  skl_hip_record_error((int)e, what);
  return (int)e;
}

hipStream_t skl_current_stream() { return t_stream; }

namespace {

std::recursive_mutex g_sequence;

// Under g_mutex. At least `floor` bytes, and at least twice the block replaced, so that retired blocks add up to
// less than the live one.
void *grow(StreamState &st, Scratch &sc, size_t bytes, size_t floor, const char *what, bool record) {
  if (sc.ptr && sc.bytes >= bytes) return sc.ptr;
  size_t want = bytes < floor ? floor : bytes;
  if (want < 2 * sc.bytes) want = 2 * sc.bytes;
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess && (want == bytes || hipMalloc(&p, want = bytes) != hipSuccess)) {
    (void)hipGetLastError();
    if (record) skl_hip_record_error(SKL_HIP_ERR_WORKSPACE, what);
    return nullptr;
  }
  (void)hipGetLastError();
  if (sc.ptr) st.retired.push_back(sc.ptr);
  sc.ptr = p;
  sc.bytes = want;
  return p;
}

DeviceState *current_device_state() {
  int dev = 0;
  if (skl_check_hip(hipGetDevice(&dev), "hipGetDevice") != 0 || dev >= kMaxDevices) return nullptr;
  return &g_devices[dev];
}

// Under g_mutex: the scratch of the calling thread's stream on this device; nullptr when every slot belongs to
// another stream (two streams on one slot would mix their partial sums and counters).
StreamState *current_stream_state(DeviceState &st) {
  for (StreamState &s : st.streams)
    if (s.stream == t_stream) return &s;
  if (st.streams.size() >= kMaxStreamStates) {
    skl_hip_record_error(SKL_HIP_ERR_STREAM_SLOTS, "scratch memory: 32 streams hold a slot on this device - release one (skl_hip_release_stream)");
    return nullptr;
  }
  st.streams.emplace_back();
  st.streams.back().stream = t_stream;
  return &st.streams.back();
}

}  // namespace

void *skl_workspace(size_t bytes) {
  DeviceState *st = current_device_state();
  if (!st) return nullptr;
  std::lock_guard<std::mutex> lock(g_mutex);
  StreamState *ss = current_stream_state(*st);
  return ss ? grow(*ss, ss->workspace, bytes, kWorkspaceBytes, "skl_workspace", true) : nullptr;
}

void *skl_zeroed_scratch(size_t bytes) {
  DeviceState *st = current_device_state();
  if (!st) return nullptr;
  std::lock_guard<std::mutex> lock(g_mutex);
  StreamState *slot = current_stream_state(*st);
  if (!slot) return nullptr;
  StreamState &ss = *slot;
  if (ss.zeroed) {
    if (bytes <= ss.zeroed_bytes) return ss.zeroed;
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, "skl_zeroed_scratch: size differs from the first request");
    return nullptr;
  }
  void *p = nullptr;
  if (hipMalloc(&p, bytes) != hipSuccess) {
    (void)hipGetLastError();
    skl_hip_record_error(SKL_HIP_ERR_WORKSPACE, "zeroed scratch");
    return nullptr;
  }
  // Cleared on the stream that will use it, and finished before any other stream can be handed the block.
  if (skl_check_hip(hipMemsetAsync(p, 0, bytes, t_stream), "zeroed scratch clear") != 0 ||
      skl_check_hip(hipStreamSynchronize(t_stream), "zeroed scratch clear") != 0) {
    (void)hipFree(p);
    return nullptr;
  }
  ss.zeroed = p;
  ss.zeroed_bytes = bytes;
  return p;
}

extern "C" {

int skl_hip_init(int device) {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    skl_hip_record_error(SKL_HIP_ERR_NO_DEVICE, "skl_hip_init");
    return SKL_HIP_ERR_NO_DEVICE;
  }
  if (device < 0 || device >= count || device >= kMaxDevices) {
    skl_hip_record_error(SKL_HIP_ERR_BAD_ARGUMENT, "skl_hip_init: device index");
    return SKL_HIP_ERR_BAD_ARGUMENT;
  }
  int rc = skl_check_hip(hipSetDevice(device), "hipSetDevice");
  if (rc != 0) return rc;
  rc = skl_hip_noalloc_setup();  // the static scratch of the entry point that allocates nothing, on this device
  if (rc != 0) return rc;
  return skl_workspace(1) ? SKL_HIP_OK : SKL_HIP_ERR_WORKSPACE;
}

void *skl_hip_operand_scratch(size_t bytes) {
  DeviceState *st = current_device_state();
  if (!st) return nullptr;
  std::lock_guard<std::mutex> lock(g_mutex);
  // not recorded as an error: the caller falls back to a kernel that needs no copy
  StreamState *ss = current_stream_state(*st);
  return ss ? grow(*ss, ss->operands, bytes, kOperandBytes, "skl_hip_operand_scratch", false) : nullptr;
}

int skl_hip_release_stream(void *stream) {
  DeviceState *st = current_device_state();
  if (!st) return SKL_HIP_ERR_NO_DEVICE;
  // The stream's work may still use the blocks: wait for it before they go (outside the lock; the caller has
  // promised not to issue more work on the stream meanwhile).
  int rc = skl_check_hip(hipStreamSynchronize((hipStream_t)stream), "skl_hip_release_stream");
  if (rc != 0) return rc;
  std::lock_guard<std::mutex> lock(g_mutex);
  for (size_t i = 0; i < st->streams.size(); ++i) {
    StreamState &s = st->streams[i];
    if (s.stream != (hipStream_t)stream) continue;
    if (s.workspace.ptr) (void)hipFree(s.workspace.ptr);
    if (s.operands.ptr) (void)hipFree(s.operands.ptr);
    if (s.converted.ptr) (void)hipFree(s.converted.ptr);
    if (s.zeroed) (void)hipFree(s.zeroed);
    for (void *p : s.retired) (void)hipFree(p);
    st->streams.erase(st->streams.begin() + (long)i);
    break;
  }
  return SKL_HIP_OK;
}

void *skl_hip_converted_scratch(size_t bytes) {
  DeviceState *st = current_device_state();
  if (!st) return nullptr;
  std::lock_guard<std::mutex> lock(g_mutex);
  StreamState *ss = current_stream_state(*st);
  return ss ? grow(*ss, ss->converted, bytes, kOperandBytes, "skl_hip_converted_scratch", true) : nullptr;
}

void skl_hip_sequence_begin(void) { g_sequence.lock(); }
void skl_hip_sequence_end(void) { g_sequence.unlock(); }

void skl_hip_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  int prev = 0;
  if (hipGetDevice(&prev) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  for (int d = 0; d < kMaxDevices; ++d) {
    DeviceState &st = g_devices[d];
    if (st.streams.empty()) continue;
    if (hipSetDevice(d) == hipSuccess) {
      (void)hipDeviceSynchronize();
      for (StreamState &s : st.streams) {
        if (s.workspace.ptr) (void)hipFree(s.workspace.ptr);
        if (s.operands.ptr) (void)hipFree(s.operands.ptr);
        if (s.converted.ptr) (void)hipFree(s.converted.ptr);
        if (s.zeroed) (void)hipFree(s.zeroed);
        for (void *p : s.retired) (void)hipFree(p);
      }
    }
    st = DeviceState{};
  }
  (void)hipSetDevice(prev);
}

void *skl_hip_malloc(size_t bytes) {
  void *p = nullptr;
  if (bytes == 0) bytes = 1;
  if (skl_check_hip(hipMalloc(&p, bytes), "skl_hip_malloc") != 0) return nullptr;
  return p;
}

void skl_hip_free(void *ptr) {
  if (ptr) (void)skl_check_hip(hipFree(ptr), "skl_hip_free");
}

// Copies are ordered with the current stream and complete before returning, so
// a caller can touch the host buffer immediately.
static int copy_sync(void *dst, const void *src, size_t bytes, hipMemcpyKind kind, const char *what) {
  if (bytes == 0) return SKL_HIP_OK;
  int rc = skl_check_hip(hipMemcpyAsync(dst, src, bytes, kind, t_stream), what);
  if (rc != 0) return rc;
  return skl_check_hip(hipStreamSynchronize(t_stream), what);
}

int skl_hip_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  return copy_sync(dst, src, bytes, hipMemcpyHostToDevice, "skl_hip_memcpy_h2d");
}
int skl_hip_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  return copy_sync(dst, src, bytes, hipMemcpyDeviceToHost, "skl_hip_memcpy_d2h");
}
int skl_hip_memcpy_d2d(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return SKL_HIP_OK;
  return skl_check_hip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, t_stream),
                       "skl_hip_memcpy_d2d");
}
int skl_hip_memset(void *dst, int byte, size_t bytes) {
  if (bytes == 0) return SKL_HIP_OK;
  return skl_check_hip(hipMemsetAsync(dst, byte, bytes, t_stream), "skl_hip_memset");
}

void skl_hip_set_stream(void *stream) { t_stream = (hipStream_t)stream; }
void *skl_hip_get_stream(void) { return (void *)t_stream; }
int skl_hip_synchronize(void) { return skl_check_hip(hipStreamSynchronize(t_stream), "skl_hip_synchronize"); }

void skl_hip_set_pointer_mode(int mode) {
  t_pointer_mode = (mode == SKL_HIP_POINTERS_DEVICE) ? SKL_HIP_POINTERS_DEVICE : SKL_HIP_POINTERS_AUTO;
}
int skl_hip_get_pointer_mode(void) { return t_pointer_mode; }

void skl_hip_set_beta_zero_mode(int mode) {
  t_beta_zero_mode = (mode == SKL_HIP_BETA_ZERO_AS_REFERENCE) ? SKL_HIP_BETA_ZERO_AS_REFERENCE : SKL_HIP_BETA_ZERO_INITIALISES;
}
int skl_hip_get_beta_zero_mode(void) {
  // A thread that has not chosen takes the process's default: SKL_HIP_BETA_ZERO=reference in the environment makes
  // the reference's evaluation the default for callers that cannot be changed to call the setter.
  static const int process_default = [] {
    const char *e = std::getenv("SKL_HIP_BETA_ZERO");
    return (e && std::strcmp(e, "reference") == 0) ? SKL_HIP_BETA_ZERO_AS_REFERENCE : SKL_HIP_BETA_ZERO_INITIALISES;
  }();
  return t_beta_zero_mode < 0 ? process_default : t_beta_zero_mode;
}

int skl_hip_pointer_is_device(const void *ptr) {
  if (t_pointer_mode == SKL_HIP_POINTERS_DEVICE) return 1;
  if (!ptr) return 0;
  hipPointerAttribute_t attr;
  memset(&attr, 0, sizeof attr);
  hipError_t e = hipPointerGetAttributes(&attr, ptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // ordinary host memory is reported as an error: not ours to keep
    return 0;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged ||
         attr.type == hipMemoryTypeHost;
}

int skl_hip_last_error(void) {
  int e = t_error;
  t_error = SKL_HIP_OK;
  return e;
}

const char *skl_hip_last_error_string(void) { return t_error_text; }

size_t skl_hip_te(void) { return 64; }

void *skl_hip_event_create(void) {
  hipEvent_t ev = nullptr;
  if (skl_check_hip(hipEventCreate(&ev), "hipEventCreate") != 0) return nullptr;
  return (void *)ev;
}
void skl_hip_event_destroy(void *event) {
  if (event) (void)skl_check_hip(hipEventDestroy((hipEvent_t)event), "hipEventDestroy");
}
int skl_hip_event_record(void *event) {
  return skl_check_hip(hipEventRecord((hipEvent_t)event, t_stream), "hipEventRecord");
}
float skl_hip_event_elapsed_ms(void *start, void *stop) {
  if (skl_check_hip(hipEventSynchronize((hipEvent_t)stop), "hipEventSynchronize") != 0) return -1.0f;
  float ms = -1.0f;
  if (skl_check_hip(hipEventElapsedTime(&ms, (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime") != 0)
    return -1.0f;
  return ms;
}

int skl_hip_device_info(char *name, size_t name_len, int *compute_units, int *clock_mhz) {
  int dev = 0;
  int rc = skl_check_hip(hipGetDevice(&dev), "hipGetDevice");
  if (rc != 0) return rc;
  hipDeviceProp_t prop;
  rc = skl_check_hip(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties");
  if (rc != 0) return rc;
  if (name && name_len) {
    // Some driver stacks report no marketing name; the architecture string is always there.
    snprintf(name, name_len, "%s (%s)", prop.name[0] ? prop.name : "unnamed AMD GPU", prop.gcnArchName);
  }
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
  return SKL_HIP_OK;
}

}  // extern "C"
