// Library-level entry points: version, device selection, error text, descriptor validation and
// the unpacking of the reference's packed `main(void**)` parameter array.
#include <cstring>

#include <mutex>
#include <vector>

#include "common.hpp"

namespace llc {

static thread_local char g_err[512] = "";

int set_error(int status, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return status;
}

int make_view(const llc_tensor* t, const char* what, View* v) {
  if (!t) return set_error(LLC_ERR_BAD_ARG, "%s: null tensor descriptor", what);
  if (t->rank > LLC_MAX_RANK) return set_error(LLC_ERR_SHAPE, "%s: rank %zu > %d", what, t->rank, LLC_MAX_RANK);
  size_t es = dtype_size(t->type);
  if (es == 0) return set_error(LLC_ERR_DTYPE, "%s: unknown element type code %zu", what, t->type);
  if (t->rank > 0 && (!t->size || !t->stride)) return set_error(LLC_ERR_BAD_ARG, "%s: null size/stride array", what);
  v->dtype = (int)t->type;
  v->rank = (int)t->rank;
  int64_t n = 1;
  for (size_t i = 0; i < t->rank; ++i) {
    v->size[i] = (int64_t)t->size[i];
    v->stride[i] = (int64_t)t->stride[i];
    if (v->size[i] < 0) return set_error(LLC_ERR_SHAPE, "%s: negative extent", what);
    n *= v->size[i];
  }
  if (n > 0 && !t->data) return set_error(LLC_ERR_BAD_ARG, "%s: null data pointer", what);
  v->ptr = (char*)t->data + t->offset * es;
  return LLC_OK;
}

int check_launch(const char* kernel) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(LLC_ERR_HIP, "launch of %s failed: %s", kernel, hipGetErrorString(e));
  return LLC_OK;
}

namespace {
constexpr int kMaxDevices = 64;
// Scratch buffers of op entry points called outside a plan: one per (device, stream), so that calls on different
// streams never share partial sums.  A buffer that was outgrown moves to `retired` (launches already queued may still
// address it) until llc_hip_trim frees it.
struct StreamScratch {
  hipStream_t stream;
  void* ptr;
  size_t cap;
};
struct DeviceScratch {
  std::vector<StreamScratch> live;
  std::vector<StreamScratch> retired;
};
DeviceScratch g_scratch[kMaxDevices];
std::mutex g_scratch_mu;
}  // namespace

int allow_dynamic_lds(const void* kernel, int bytes, std::atomic<uint32_t>& done) {
  int dev = 0;
  LLC_HIP_TRY(hipGetDevice(&dev));
  const uint32_t bit = 1u << (dev & 31);
  if (done.load(std::memory_order_acquire) & bit) return LLC_OK;
  LLC_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  done.fetch_or(bit, std::memory_order_release);
  return LLC_OK;
}

namespace {
thread_local void* t_ws_ptr = nullptr;
thread_local size_t t_ws_cap = 0;
thread_local bool t_ws_active = false;
thread_local size_t* t_ws_high_water = nullptr;
}  // namespace

WorkspaceScope::WorkspaceScope(void* ptr, size_t capacity) : prev_ptr_(t_ws_ptr), prev_cap_(t_ws_cap), prev_active_(t_ws_active) {
  t_ws_ptr = ptr;
  t_ws_cap = capacity;
  t_ws_active = true;
}
WorkspaceScope::~WorkspaceScope() {
  t_ws_ptr = prev_ptr_;
  t_ws_cap = prev_cap_;
  t_ws_active = prev_active_;
}
void workspace_track(size_t* high_water) { t_ws_high_water = high_water; }

int get_workspace(size_t bytes, void** out, hipStream_t stream) {
  if (t_ws_high_water && bytes > *t_ws_high_water) *t_ws_high_water = bytes;
  if (t_ws_active) {
    if (bytes > t_ws_cap)
      return set_error(LLC_ERR_TOO_LARGE, "this call needs %zu bytes of scratch memory, %zu are provided and nothing may be allocated here",
                       bytes, t_ws_cap);
    *out = t_ws_ptr;
    return LLC_OK;
  }
  int dev = 0;
  LLC_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return set_error(LLC_ERR_BAD_ARG, "workspace: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  DeviceScratch& d = g_scratch[dev];
  StreamScratch* mine = nullptr;
  for (StreamScratch& e : d.live)
    if (e.stream == stream) mine = &e;
  if (!mine || bytes > mine->cap) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone)
      return set_error(LLC_ERR_UNSUPPORTED, "this call needs %zu bytes of scratch memory and the stream is being captured: run it once on this stream "
                       "outside the capture, or record it into a plan", bytes);
    const size_t cap_bytes = ((bytes + bytes / 2) + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
    void* fresh = nullptr;
    LLC_HIP_TRY(hipMalloc(&fresh, cap_bytes));
    if (mine) {
      d.retired.push_back(*mine);  // queued launches and captured graphs may still address it
      mine->ptr = fresh;
      mine->cap = cap_bytes;
    } else {
      d.live.push_back(StreamScratch{stream, fresh, cap_bytes});
      mine = &d.live.back();
    }
  }
  *out = mine->ptr;
  return LLC_OK;
}

int scratch_bytes(int dev, size_t* live, size_t* retired) {
  if (dev < 0 || dev >= kMaxDevices) return set_error(LLC_ERR_BAD_ARG, "scratch: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  size_t a = 0, b = 0;
  for (const StreamScratch& e : g_scratch[dev].live) a += e.cap;
  for (const StreamScratch& e : g_scratch[dev].retired) b += e.cap;
  if (live) *live = a;
  if (retired) *retired = b;
  return LLC_OK;
}

int scratch_trim(int all) {
  int dev = 0;
  LLC_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return set_error(LLC_ERR_BAD_ARG, "scratch: device %d", dev);
  // nothing queued may still address what is freed
  LLC_HIP_TRY(hipDeviceSynchronize());
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  DeviceScratch& d = g_scratch[dev];
  for (StreamScratch& e : d.retired) (void)hipFree(e.ptr);
  d.retired.clear();
  if (all) {
    for (StreamScratch& e : d.live) (void)hipFree(e.ptr);
    d.live.clear();
  }
  return LLC_OK;
}

}  // namespace llc

using namespace llc;

extern "C" int llc_hip_abi_version(void) { return LLC_HIP_ABI_VERSION; }

extern "C" const char* llc_hip_last_error(void) { return g_err; }

extern "C" const char* llc_hip_status_string(int status) {
  switch (status) {
    case LLC_OK: return "ok";
    case LLC_ERR_BAD_ARG: return "bad argument";
    case LLC_ERR_DTYPE: return "unsupported or mismatched element type";
    case LLC_ERR_SHAPE: return "shape mismatch";
    case LLC_ERR_LAYOUT: return "unsupported strides";
    case LLC_ERR_UNSUPPORTED: return "unsupported attribute combination";
    case LLC_ERR_HIP: return "HIP runtime error";
    case LLC_ERR_NO_DEVICE: return "no usable gfx950 device";
    case LLC_ERR_TOO_LARGE: return "tensor too large for this kernel";
  }
  return "unknown status";
}

extern "C" int llc_hip_init(int device) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return set_error(LLC_ERR_NO_DEVICE, "no HIP device visible");
  if (device < 0 || device >= n) return set_error(LLC_ERR_BAD_ARG, "device %d out of range (0..%d)", device, n - 1);
  LLC_HIP_TRY(hipSetDevice(device));
  hipDeviceProp_t prop;
  LLC_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(LLC_ERR_NO_DEVICE, "device %d is %s; this library carries gfx950 code only", device,
                     prop.gcnArchName);
  // the scratch array of the allocation-free entry point has an address of its own on every device
  return llc_impl_static_scratch_setup();
}

extern "C" int llc_hip_scratch_bytes(int device, size_t* live_bytes, size_t* retired_bytes) {
  return scratch_bytes(device, live_bytes, retired_bytes);
}

extern "C" int llc_hip_trim(int release_live) { return scratch_trim(release_live); }

extern "C" int llc_hip_unpack_params(void* const* params, size_t n_tensors, const size_t* ranks, const size_t* types,
                                     llc_tensor* tensors_out, const int64_t** symbols_out) {
  if (!params || (n_tensors && (!ranks || !types || !tensors_out)))
    return set_error(LLC_ERR_BAD_ARG, "unpack_params: null argument");
  if (symbols_out) *symbols_out = (const int64_t*)params[0];
  size_t slot = 1;
  for (size_t i = 0; i < n_tensors; ++i) {
    llc_tensor* t = &tensors_out[i];
    if (ranks[i] > LLC_MAX_RANK) return set_error(LLC_ERR_SHAPE, "unpack_params: tensor %zu has rank %zu", i, ranks[i]);
    t->base = params[slot + 0];
    t->data = params[slot + 1];
    const size_t* off = (const size_t*)params[slot + 2];
    if (!off) return set_error(LLC_ERR_BAD_ARG, "unpack_params: tensor %zu has a null offset slot", i);
    t->offset = *off;
    t->type = types[i];
    t->rank = ranks[i];
    t->size = (const size_t*)params[slot + 3];
    t->stride = (const size_t*)params[slot + 4];
    if (ranks[i] && (!t->size || !t->stride))
      return set_error(LLC_ERR_BAD_ARG, "unpack_params: tensor %zu has null size/stride slots", i);
    slot += 5;
  }
  return (int)slot;
}
