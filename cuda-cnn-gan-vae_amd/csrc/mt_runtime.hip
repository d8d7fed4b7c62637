// Runtime of libmi355tensor: device selection, the work stream, memory and the error latch.
// Replaces CCUDADeviceVector (cuda/ccudadevicevector.cu.h) and HANDLE_ERROR (cuda/handle_error.cu.h):
// errors are reported to the caller instead of ending the process.
#include <stdarg.h>
#include <string.h>

#include "mt_common.h"

namespace {
char g_error[512] = "";
hipStream_t g_own_stream = nullptr;
hipStream_t g_stream = nullptr;
bool g_ready = false;
}  // namespace

namespace mt {

hipStream_t stream() { return g_stream; }

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char *what) {
  (void)hipGetLastError();  // the runtime keeps the error until it is read: the next launch check must not see it again
  return fail(MT_E_HIP + (int)e, "%s: %s", what, hipGetErrorString(e));
}

}  // namespace mt

extern "C" {

const char *mt_last_error(void) { return g_error; }

int mt_init(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) return mt::fail(MT_E_UNAVAILABLE, "mt_init: no HIP device (%s)", hipGetErrorString(e));
  if (device < 0 || device >= n) return mt::fail(MT_E_ARGUMENT, "mt_init: device %d out of range (0..%d)", device, n - 1);
  hipDeviceProp_t prop;
  MT_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return mt::fail(MT_E_UNAVAILABLE, "mt_init: device %d is %s, this library holds gfx950 code only", device, prop.gcnArchName);
  MT_HIP(hipSetDevice(device));
  if (g_own_stream == nullptr) MT_HIP(hipStreamCreateWithFlags(&g_own_stream, hipStreamNonBlocking));
  g_stream = g_own_stream;
  g_ready = true;
  return MT_OK;
}

int mt_malloc(void **ptr, size_t bytes) {
  if (ptr == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_malloc: null result pointer");
  if (!g_ready) { int rc = mt_init(0); if (rc) return rc; }
  *ptr = nullptr;
  if (bytes == 0) return MT_OK;
  MT_HIP(hipMalloc(ptr, bytes));
  return MT_OK;
}

int mt_free(void *ptr) {
  if (ptr == nullptr) return MT_OK;
  MT_HIP(hipStreamSynchronize(g_stream));  // queued kernels may still use it
  MT_HIP(hipFree(ptr));
  return MT_OK;
}

int mt_copy_h2d(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return MT_OK;
  if (dst == nullptr || src == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_copy_h2d: null pointer");
  MT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
  MT_HIP(hipStreamSynchronize(g_stream));  // the host buffer may be reused on return
  return MT_OK;
}

int mt_copy_d2h(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return MT_OK;
  if (dst == nullptr || src == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_copy_d2h: null pointer");
  MT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
  MT_HIP(hipStreamSynchronize(g_stream));
  return MT_OK;
}

int mt_copy_d2d(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return MT_OK;
  if (dst == nullptr || src == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_copy_d2d: null pointer");
  MT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
  return MT_OK;
}

int mt_synchronize(void) {
  if (!g_ready) return MT_OK;
  MT_HIP(hipStreamSynchronize(g_stream));
  return MT_OK;
}

void *mt_get_stream(void) { return (void *)g_stream; }

int mt_set_option(const char *name, int value) {
  if (name && strcmp(name, "conv_path") == 0) return mt::set_conv_path(value);
  if (name && strcmp(name, "igemm_tile") == 0) return mt::set_igemm_tile(value);
  if (name && strcmp(name, "wgrad_groups") == 0) return mt::set_wgrad_groups(value);
  if (name && strcmp(name, "patch_blocks") == 0) return mt::set_patch_blocks(value);
  return mt::fail(MT_E_ARGUMENT, "mt_set_option: unknown option '%s'", name ? name : "(null)");
}

// ---- interval timer on the work stream: the two events of the reference's CCUDATimeSpent ----
namespace {
struct Timer {
  hipEvent_t start, stop;
};
}  // namespace

int mt_timer_create(void **timer) {
  if (timer == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_timer_create: null pointer");
  Timer *t = new Timer;
  hipError_t e = hipEventCreate(&t->start);
  if (e == hipSuccess && (e = hipEventCreate(&t->stop)) != hipSuccess) (void)hipEventDestroy(t->start);
  if (e != hipSuccess) { delete t; return mt::hip_fail(e, "hipEventCreate"); }
  *timer = t;
  return MT_OK;
}
int mt_timer_start(void *timer) {
  if (timer == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_timer_start: null timer");
  MT_HIP(hipEventRecord(static_cast<Timer *>(timer)->start, mt::stream()));
  return MT_OK;
}
int mt_timer_stop(void *timer, float *milliseconds) {
  if (timer == nullptr || milliseconds == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_timer_stop: null argument");
  Timer *t = static_cast<Timer *>(timer);
  MT_HIP(hipEventRecord(t->stop, mt::stream()));
  MT_HIP(hipEventSynchronize(t->stop));
  MT_HIP(hipEventElapsedTime(milliseconds, t->start, t->stop));
  return MT_OK;
}
int mt_timer_destroy(void *timer) {
  if (timer == nullptr) return MT_OK;
  Timer *t = static_cast<Timer *>(timer);
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
  return MT_OK;
}

int mt_set_stream(void *hip_stream) {
  if (!g_ready) { int rc = mt_init(0); if (rc) return rc; }
  g_stream = hip_stream ? (hipStream_t)hip_stream : g_own_stream;
  return MT_OK;
}

}  // extern "C"
