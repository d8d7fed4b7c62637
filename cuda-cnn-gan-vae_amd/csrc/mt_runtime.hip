// Runtime of libmi355tensor: device selection, the work stream, memory and the error latch.
// Replaces CCUDADeviceVector (cuda/ccudadevicevector.cu.h) and HANDLE_ERROR (cuda/handle_error.cu.h):
// errors are reported to the caller instead of ending the process.
#include <stdarg.h>
#include <string.h>

#include <map>
#include <unordered_map>
#include <vector>

#include "mt_common.h"

namespace {
char g_error[512] = "";
hipStream_t g_own_stream = nullptr;
hipStream_t g_stream = nullptr;
bool g_ready = false;
int g_device = -1;
uint64_t g_driver_allocs = 0;
std::vector<float *> g_retired;  // outgrown workspace blocks that a recorded graph may still use
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

int workspace_get(Workspace &ws, const char *what, size_t floats, float **p) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (g_stream != nullptr) (void)hipStreamIsCapturing(g_stream, &capture);
  const bool capturing = capture != hipStreamCaptureStatusNone;
  if (floats > ws.floats) {
    if (capturing)
      return fail(MT_E_ARGUMENT, "%s: %zu bytes are needed but %zu exist, and the stream is being captured: run the sequence once before recording it",
                  what, floats * sizeof(float), ws.floats * sizeof(float));
    const size_t want = floats + floats / 4 + 1024;
    float *fresh = nullptr;
    MT_HIP(hipMalloc((void **)&fresh, want * sizeof(float)));
    g_driver_allocs++;
    if (ws.p != nullptr) {
      if (ws.captured) {
        g_retired.push_back(ws.p);  // a recorded graph may still name it: kept until the process ends
      } else {
        hipError_t e = hipStreamSynchronize(g_stream);  // queued kernels may still use the old block
        if (e == hipSuccess) e = hipFree(ws.p);
        if (e != hipSuccess) { (void)hipFree(fresh); return hip_fail(e, "workspace growth"); }
      }
    }
    ws.p = fresh; ws.floats = want; ws.captured = false;
  }
  if (capturing) ws.captured = true;
  *p = ws.p;
  return MT_OK;
}

size_t retired_workspaces() { return g_retired.size(); }
void count_driver_allocation() { g_driver_allocs++; }

}  // namespace mt

extern "C" {

const char *mt_last_error(void) { return g_error; }

int mt_init(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n <= 0) return mt::fail(MT_E_UNAVAILABLE, "mt_init: no HIP device (%s)", hipGetErrorString(e));
  if (device < 0 || device >= n) return mt::fail(MT_E_ARGUMENT, "mt_init: device %d out of range (0..%d)", device, n - 1);
  if (g_ready && device != g_device)
    return mt::fail(MT_E_ARGUMENT, "mt_init: the library already runs on device %d (its stream, workspaces and memory pool live there)", g_device);
  hipDeviceProp_t prop;
  MT_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return mt::fail(MT_E_UNAVAILABLE, "mt_init: device %d is %s, this library holds gfx950 code only", device, prop.gcnArchName);
  MT_HIP(hipSetDevice(device));
  if (g_own_stream == nullptr) MT_HIP(hipStreamCreateWithFlags(&g_own_stream, hipStreamNonBlocking));
  if (!g_ready) g_stream = g_own_stream;
  int rc = mt::static_scratch_setup();  // the entry point that allocates nothing finds its array's address here
  if (rc) return rc;
  g_device = device;
  g_ready = true;
  return MT_OK;
}

// ---- device memory: a stream-ordered pool ---------------------------------------------------------------------------
// All work of the library runs on one stream.  A block that the caller frees may still be read by kernels that are
// queued, but whatever the next owner of the block does is queued behind them on the same stream: the block can be
// handed out again at once, without waiting.  Freed blocks are kept per size; memory goes back to the driver only when
// the pool holds more than its limit or an allocation fails (then the stream is drained first).  The unchanged layers
// of the reference create temporaries on every call (netlayer/cnetlayerconvolution.cu.h:494), which this makes cheap.
namespace {
constexpr size_t POOL_GRANULE = 512;                  // block sizes are multiples of this
constexpr size_t POOL_LARGEST = (size_t)1 << 30;      // larger blocks are not kept
size_t g_pool_limit = (size_t)4 << 30;                // bytes the pool may hold in free blocks
size_t g_pool_bytes = 0;
bool g_pool_on = true;
uint64_t g_pool_reused = 0;
// A block is LIVE (the caller holds it), POOLED (free, waiting for the next mt_malloc of its size) or RETIRED: freed
// while the stream was being captured, or handed out during a capture.  A recorded graph names such a block's address
// in its kernels, and every replay writes there again; handing the block to another tensor would let replays scribble
// over it.  A retired block stays allocated and is never handed out again (the cost of recording a sequence that creates
// temporaries: its temporaries, once per recording).
enum BlockState : uint8_t { LIVE, POOLED, RETIRED };
struct Block {
  size_t size;
  BlockState state;
  bool in_capture;  // handed out while the stream was being captured
};
std::unordered_map<void *, Block> g_blocks;           // every block mt_malloc ever got from the driver and still holds
std::map<size_t, std::vector<void *>> g_pool;         // free blocks by size
size_t g_retired_blocks = 0, g_retired_bytes = 0;

bool capturing_now() {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (g_stream != nullptr) (void)hipStreamIsCapturing(g_stream, &capture);
  return capture != hipStreamCaptureStatusNone;
}

// gives every pooled block back to the driver; the bookkeeping is complete before a failure is reported
int pool_release_all() {
  if (g_pool_bytes == 0) return MT_OK;
  hipError_t first = hipStreamSynchronize(g_stream);
  for (auto &kv : g_pool)
    for (void *p : kv.second) {
      g_blocks.erase(p);
      const hipError_t e = hipFree(p);
      if (first == hipSuccess) first = e;
    }
  g_pool.clear();
  g_pool_bytes = 0;
  return first == hipSuccess ? MT_OK : mt::hip_fail(first, "returning pooled blocks to the driver");
}
}  // namespace

int mt_malloc(void **ptr, size_t bytes) {
  if (ptr == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_malloc: null result pointer");
  if (!g_ready) { int rc = mt_init(0); if (rc) return rc; }
  *ptr = nullptr;
  if (bytes == 0) return MT_OK;
  const size_t size = (bytes + POOL_GRANULE - 1) / POOL_GRANULE * POOL_GRANULE;
  const bool capturing = capturing_now();
  auto it = g_pool.find(size);
  if (it != g_pool.end() && !it->second.empty()) {
    *ptr = it->second.back();
    it->second.pop_back();
    g_pool_bytes -= size;
    g_pool_reused++;
    Block &b = g_blocks[*ptr];
    b.state = LIVE;
    b.in_capture = capturing;
    return MT_OK;
  }
  hipError_t e = hipMalloc(ptr, size);
  if (e == hipErrorOutOfMemory && g_pool_bytes && !capturing) {
    (void)hipGetLastError();
    int rc = pool_release_all();
    if (rc) return rc;
    e = hipMalloc(ptr, size);
  }
  if (e != hipSuccess) { *ptr = nullptr; return mt::hip_fail(e, "hipMalloc"); }
  g_driver_allocs++;
  g_blocks[*ptr] = Block{size, LIVE, capturing};
  return MT_OK;
}

int mt_free(void *ptr) {
  if (ptr == nullptr) return MT_OK;
  auto it = g_blocks.find(ptr);
  if (it != g_blocks.end() && it->second.state != LIVE)
    return mt::fail(MT_E_ARGUMENT, "mt_free: block %p was freed already (%s)", ptr, it->second.state == POOLED ? "it waits in the pool" : "a recorded graph holds it");
  const size_t size = it == g_blocks.end() ? 0 : it->second.size;
  // whatever was derived from the block's contents (re-ordered weights) must not outlive it: the address may come back
  mt::note_write(ptr, size ? size : ~(size_t)0 - (size_t)(uintptr_t)ptr);
  const bool capturing = capturing_now();
  if (it != g_blocks.end() && (capturing || it->second.in_capture)) {
    it->second.state = RETIRED;  // a recorded graph may write here on every replay
    g_retired_blocks++;
    g_retired_bytes += size;
    return MT_OK;
  }
  mt::forget_graph_writes(ptr, size);
  if (g_pool_on && size && size <= POOL_LARGEST) {
    if (g_pool_bytes + size > g_pool_limit) { int rc = pool_release_all(); if (rc) return rc; }
    it->second.state = POOLED;
    g_pool[size].push_back(ptr);
    g_pool_bytes += size;
    return MT_OK;
  }
  if (it != g_blocks.end()) g_blocks.erase(it);
  if (!capturing) MT_HIP(hipStreamSynchronize(g_stream));  // queued kernels may still use it
  MT_HIP(hipFree(ptr));
  return MT_OK;
}

// Small uploads (a layer's time steps, a batch of noise, a label) go through pinned staging slots: the caller's buffer is
// copied at once and may be reused on return, the copy to the device is queued like a kernel -- waiting for it here would
// wait for everything queued in front of it, and a layer that uploads 128 bytes per forward pass would drain the queue
// every time.  A slot is taken again when its own copy is over (an event per slot).
namespace {
constexpr size_t STAGE_SLOT_BYTES = (size_t)64 << 10;
constexpr int STAGE_SLOTS = 64;
char *g_stage = nullptr;
hipEvent_t g_stage_done[STAGE_SLOTS];
bool g_stage_used[STAGE_SLOTS];
int g_stage_next = 0, g_staged_uploads = 1;
uint64_t g_staged_count = 0;
}  // namespace

int mt_copy_h2d(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return MT_OK;
  if (dst == nullptr || src == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_copy_h2d: null pointer");
  mt::note_write(dst, bytes);
  if (g_staged_uploads && bytes <= STAGE_SLOT_BYTES && !capturing_now()) {
    if (g_stage == nullptr) {
      MT_HIP(hipHostMalloc((void **)&g_stage, STAGE_SLOT_BYTES * STAGE_SLOTS, hipHostMallocPortable));
      for (int i = 0; i < STAGE_SLOTS; i++) {
        MT_HIP(hipEventCreateWithFlags(&g_stage_done[i], hipEventDisableTiming));
        g_stage_used[i] = false;
      }
    }
    const int slot = g_stage_next;
    g_stage_next = (slot + 1) % STAGE_SLOTS;
    if (g_stage_used[slot]) MT_HIP(hipEventSynchronize(g_stage_done[slot]));
    char *staged = g_stage + (size_t)slot * STAGE_SLOT_BYTES;
    memcpy(staged, src, bytes);
    MT_HIP(hipMemcpyAsync(dst, staged, bytes, hipMemcpyHostToDevice, g_stream));
    MT_HIP(hipEventRecord(g_stage_done[slot], g_stream));
    g_stage_used[slot] = true;
    g_staged_count++;
    return MT_OK;
  }
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
  mt::note_write(dst, bytes);
  MT_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g_stream));
  return MT_OK;
}

int mt_invalidate(const void *ptr, size_t bytes) {
  if (ptr == nullptr || bytes == 0) return MT_OK;
  mt::note_write(ptr, bytes);
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
  if (name && strcmp(name, "pack_cache") == 0) return mt::set_pack_cache(value);
  if (name && strcmp(name, "tconv_walk") == 0) return mt::set_tconv_walk(value);
  if (name && strcmp(name, "conv_walk") == 0) return mt::set_conv_walk(value);
  if (name && strcmp(name, "wgrad_walk") == 0) return mt::set_wgrad_walk(value);
  if (name && strcmp(name, "upconv_walk") == 0) return mt::set_upconv_walk(value);
  if (name && strcmp(name, "upconv_split") == 0) return mt::set_upconv_split(value);
  if (name && strcmp(name, "walk_wide") == 0) return mt::set_walk_wide(value);
  if (name && strcmp(name, "wgrad_parts") == 0) return mt::set_wgrad_parts(value);
  if (name && strcmp(name, "wgrad_pad") == 0) return mt::set_wgrad_pad(value);
  if (name && strcmp(name, "wgrad_patch") == 0) return mt::set_wgrad_patch(value);
  if (name && strcmp(name, "tconv_patch") == 0) return mt::set_tconv_patch(value);
  if (name && strcmp(name, "tconv_merge") == 0) return mt::set_tconv_merge(value);
  if (name && strcmp(name, "tconv_as_conv") == 0) return mt::set_tconv_as_conv(value);
  if (name && strcmp(name, "conv_patch") == 0) return mt::set_conv_patch(value);
  if (name && strcmp(name, "pack_refresh") == 0) return mt::set_pack_refresh(value);
  if (name && strcmp(name, "adam_vec") == 0) return mt::set_adam_vec(value);
  if (name && strcmp(name, "nontemporal") == 0) return mt::set_nontemporal(value);
  if (name && strcmp(name, "image_strip") == 0) return mt::set_image_strip(value);
  if (name && strcmp(name, "first_layer") == 0) return mt::set_first_layer(value);
  if (name && strcmp(name, "walk_blocks") == 0) return mt::set_walk_blocks(value);
  if (name && strcmp(name, "image_mfma") == 0) return mt::set_image_mfma(value);
  if (name && strcmp(name, "walk_waves") == 0) return mt::set_walk_waves(value);
  if (name && strcmp(name, "walk_tm") == 0) return mt::set_walk_tm(value);
  if (name && strcmp(name, "walk_order") == 0) return mt::set_walk_order(value);
  if (name && strcmp(name, "walk_fair") == 0) return mt::set_walk_fair(value);
  if (name && strcmp(name, "igemm_fair") == 0) return mt::set_igemm_fair(value);
  if (name && strcmp(name, "staged_uploads") == 0) {
    if (value != 0 && value != 1) return mt::fail(MT_E_ARGUMENT, "staged_uploads must be 0 or 1");
    g_staged_uploads = value;
    return MT_OK;
  }
  if (name && strcmp(name, "pool") == 0) {
    if (value != 0 && value != 1) return mt::fail(MT_E_ARGUMENT, "pool must be 0 (every mt_free goes to the driver) or 1");
    g_pool_on = value != 0;
    return g_pool_on ? MT_OK : pool_release_all();
  }
  if (name && strcmp(name, "pool_limit_mib") == 0) {
    if (value < 0) return mt::fail(MT_E_ARGUMENT, "pool_limit_mib must not be negative");
    g_pool_limit = (size_t)value << 20;
    return g_pool_bytes > g_pool_limit ? pool_release_all() : MT_OK;
  }
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
  hipStream_t next = hip_stream ? (hipStream_t)hip_stream : g_own_stream;
  if (next == g_stream) return MT_OK;
  // pooled blocks, workspaces and re-ordered weights are reused in the order of ONE stream: the old stream's work
  // must be complete before anything is queued on the new one
  MT_HIP(hipStreamSynchronize(g_stream));
  g_stream = next;
  return MT_OK;
}

int mt_get_info(const char *name, int64_t *value) {
  if (name == nullptr || value == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_get_info: null argument");
  if (strcmp(name, "pool_bytes") == 0) { *value = (int64_t)g_pool_bytes; return MT_OK; }
  if (strcmp(name, "pool_reused") == 0) { *value = (int64_t)g_pool_reused; return MT_OK; }
  if (strcmp(name, "driver_allocations") == 0) { *value = (int64_t)g_driver_allocs; return MT_OK; }
  if (strcmp(name, "staged_uploads") == 0) { *value = (int64_t)g_staged_count; return MT_OK; }
  if (strcmp(name, "retired_workspaces") == 0) { *value = (int64_t)mt::retired_workspaces(); return MT_OK; }
  if (strcmp(name, "retired_blocks") == 0) { *value = (int64_t)g_retired_blocks; return MT_OK; }
  if (strcmp(name, "retired_bytes") == 0) { *value = (int64_t)g_retired_bytes; return MT_OK; }
  if (mt::pack_cache_info(name, value)) return MT_OK;
  return mt::fail(MT_E_ARGUMENT, "mt_get_info: unknown name '%s'", name);
}

}  // extern "C"
