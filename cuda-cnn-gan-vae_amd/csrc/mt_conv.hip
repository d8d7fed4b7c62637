// CTensorConv on gfx950: forward convolution, transposed convolution (also the input delta of a convolution)
// and the per-sample weight / bias gradient.
//
// Fast path: implicit GEMM on the fp32 matrix cores (mt_igemm.h).
//   forward      C[k][(b,oy,ox)]   = sum_{c,ky,kx} kernel[k][(c,ky,kx)] * image[b][c][oy*s-p+ky][ox*s-p+kx]
//   transposed   the output is split into its sy*sx stride phases.  All pixels of one phase use the same subset of
//                kernel taps, so each phase is a dense stride-1 convolution of the (un-dilated) delta with a packed
//                sub-kernel: only non-zero taps are multiplied, 1/(sy*sx) of the dense-over-zeros product.
//   gradient     per sample, dK[f][(c,i,j)] += sum_{oy,ox} delta[f][(oy,ox)] * image[c][oy*s-p+i][ox*s-p+j]
// Slow path ("direct"): one thread per output element, same loop and summation order as the CPU path, used
// for shapes the fast path does not cover (kernels that differ per sample, strides above 4) and as a
// bit-for-bit cross-check of the fast path in the tests.
#include <string.h>

#include <initializer_list>
#include <utility>
#include <vector>

#include "mt_igemm.h"
#include "mt_walk.h"
#include "mt_firstlayer.h"
#include "mt_wgradpatch.h"
#include "mt_convpatch.h"

namespace {

using namespace mt::igemm;
using mt::cdiv;

int g_conv_path = 0;  // 0 auto, 1 direct, 2 implicit GEMM wherever it applies
int g_first_layer = 1; // forward convolutions of 3-channel images: 0 never on the kernel that keeps the input patch in LDS and the weights in registers, 1 wherever the shape allows
int g_conv_walk = 1;   // forward convolutions whose taps tile the k step: 0 never on the kernel whose blocks walk over the batch, 1 wherever the shape allows and gives 512 blocks, 2 wherever the shape allows
int g_walk_wide = 1;       // 1: layers whose output channels are a multiple of 32 but not of 64 walk in blocks of 32 rows x 128 columns, 0: never
int g_upconv_split = 1;    // 1: up-sampling convolutions with fewer than 512 walking blocks share a tile's k steps between blocks
int g_upconv_walk = 512;   // blocks from which the up-sampling convolution takes the walking kernel (0: never; measured on the
                           // shipped GAN generator at batch 32: 768 blocks 67.7 -> 54.6 and 58.6 -> 54.0 us, 384 blocks 65.1 -> 69 us)
uint64_t g_wgrad_walk_launches = 0, g_wgrad_patch_launches = 0, g_tconv_patch_launches = 0, g_tconv_merge_launches = 0, g_tconv_as_conv_launches = 0, g_conv_patch_launches = 0;
int g_conv_patch = 1;     // 1: a 3x3 stride-1 forward convolution from at most 32 channels to g_conv_patch_min..64 filters on large images multiplies patches held in LDS, 0: never
int g_conv_patch_min = 5;
int g_tconv_as_conv = 1;   // 1: a stride-1 transposed convolution whose taps do not tile the k step (3x3) runs as the forward convolution with flipped kernels, 0: never
int g_tconv_merge = 1;   // 1: a 5x5 stride-2 padding-2 transposed convolution to 5..16 channels runs as one 3x3 convolution to (channel, phase) rows, 0: never
int g_tconv_patch = 1;   // 1: a 3x3 stride-1 transposed convolution from at most 32 filters to at most 64 channels on large images multiplies patches held in LDS (tconv3x3_patch_kernel), 0: never
int g_wgrad_patch = 1;   // 1: the batch-summed weight gradient of a 3x3 stride-1 layer with at most 32 filters on large images multiplies patches held in LDS (wgrad_patch3x3_kernel), 0: never
int g_wgrad_pad = 1;     // 1: the batch-summed weight gradient pads delta's images with rows of zeros when their pixels do not fill whole k steps, 0: per-sample gradients then
int g_wgrad_parts = 1;   // 1: the general batch-summed weight gradient cuts samples into bands of output rows when samples x tiles are too few blocks, 0: never, n > 1: n bands
int g_wgrad_walk = 1;    // 1: the batch-summed weight gradient runs as one k loop per block where its shape allows (wgrad_walk_kernel), 0: never
int g_wgrad_groups = 0;  // 0 auto, else the number of batch groups of the batch-summed weight gradient (if it divides the batch)

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

// Calls f with a row-major, k-contiguous source; 128-bit loads when the layout allows them.
template <class F>
int with_row_k(const float *p, uint32_t ld, uint32_t R, uint32_t K, Batch bt, F &&f) {
  if (ld % 4 == 0 && K % 4 == 0 && aligned16(p) && bt.stride % 4 == 0) {
    SrcRowK<true> s{};
    s.p = p; s.ld = ld; s.R = R; s.K = K; s.bt = bt;
    return f(s);
  }
  SrcRowK<false> s{};
  s.p = p; s.ld = ld; s.R = R; s.K = K; s.bt = bt;
  return f(s);
}

// ---- library-owned workspace: the partial sums of the batch-summed gradients, up-sampled images, and re-ordered
// weights while they cannot be kept (see below)
mt::Workspace g_ws, g_stats_ws, g_norm_ws, g_pad_ws, g_merge_ws;   // (one per use: a call that takes its input from one of them may need another)
int workspace(size_t floats, float **p) { return mt::workspace_get(g_ws, "convolution workspace", floats, p); }

// ---- re-ordered weights, kept between calls ---------------------------------------------------------------------
// A layer passes the same kernel tensor on every forward call (netlayer/cnetlayerbackconvolution.cu.h:303-315); it
// changes only when the optimiser steps.  The per-phase sub-kernels and bias sums of a transposed convolution, the
// tap-major order of a 3x3 / 5x5 forward kernel and the coefficient sums of "up-sampling, then 3x3" are therefore
// made once per (kernel address and sizes, bias address and sizes, geometry, layout) and made again only after a write
// to the kernel's or the bias' memory: every library call that writes device memory reports its output range
// (mt::note_write), and writers outside the library call mt_invalidate.  Every entry owns its buffer, so the order of
// uses on the stream keeps readers of the old contents ahead of the kernel that re-makes them.  While the stream is
// being captured nothing is kept or looked up (the recorded graph must re-order the weights it will meet at every
// replay): the re-ordered weights then live in the workspace, as they do with the cache switched off.
struct PackKey {
  int kind;  // 0 transposed convolution, 1 tap-major forward kernel, 2 up-sampling + 3x3 coefficient sums
  const float *kernel, *bias;
  uint32_t kernel_dims[4], bias_dims[4];
  int32_t geo[12];
  bool operator==(const PackKey &o) const {
    if (kind != o.kind || kernel != o.kernel || bias != o.bias) return false;
    for (int i = 0; i < 4; i++)
      if (kernel_dims[i] != o.kernel_dims[i] || bias_dims[i] != o.bias_dims[i]) return false;
    for (int i = 0; i < 12; i++)
      if (geo[i] != o.geo[i]) return false;
    return true;
  }
};
// What an optimiser step needs to write the re-ordered copy of a 4x4 stride-2 transposed convolution itself (see
// mt::pack_refresh_find): where the sub-kernel of each phase starts behind the bias sums, and which phase owns which
// parity of a flipped coefficient.
struct PackK4S2 {
  bool on = false;
  uint32_t sums = 0, CO = 0, CI = 0, co_stride = 0, ci_stride = 0, begin[4] = {0, 0, 0, 0};  // coefficient (co, ci, tap) of phase f: begin[f] + co*co_stride + ci*ci_stride + tap
  uint8_t phase_of[4] = {0, 0, 0, 0};  // [(3 - ky) % 2 * 2 + (3 - kx) % 2]
};
struct PackEntry {
  PackKey key;
  PackK4S2 k4s2;
  float *buf = nullptr;
  size_t floats = 0;
  bool valid = false;
  bool pinned = false;  // a recorded graph writes and reads the buffer: it is never freed
  uint64_t used = 0;
};
constexpr size_t PACK_MAX_ENTRIES = 64, PACK_MAX_BYTES = (size_t)512 << 20;
std::vector<PackEntry> g_packs;
bool g_pack_cache = true;
uint64_t g_pack_clock = 0, g_pack_hits = 0, g_pack_made = 0, g_pack_refreshed = 0;
int g_pack_refresh = 1;  // 1: mt_adam_many writes the re-ordered copies of the weights it updates (4x4 stride-2 transposed convolutions), 0: never
// Memory that calls recorded into a graph write.  A replay changes it without the library seeing a call, so copies made
// from such memory are never trusted: they are made again on every use (training weights that a recorded step updates).
std::vector<std::pair<uintptr_t, uintptr_t>> g_graph_written;
bool g_graph_writes_anything = false;  // the list overflowed: nothing is trusted any more
constexpr size_t GRAPH_WRITTEN_MAX = 4096;

PackKey pack_key(int kind, const mt_tensor *kernel, const mt_tensor *bias, std::initializer_list<int32_t> geo) {
  PackKey k{};
  k.kind = kind;
  k.kernel = kernel->p;
  k.kernel_dims[0] = kernel->w; k.kernel_dims[1] = kernel->z; k.kernel_dims[2] = kernel->y; k.kernel_dims[3] = kernel->x;
  if (bias) { k.bias = bias->p; k.bias_dims[0] = bias->w; k.bias_dims[1] = bias->z; k.bias_dims[2] = bias->y; k.bias_dims[3] = bias->x; }
  int i = 0;
  for (int32_t g : geo) k.geo[i++] = g;
  return k;
}

bool capturing() {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (mt::stream() != nullptr) (void)hipStreamIsCapturing(mt::stream(), &st);
  return st != hipStreamCaptureStatusNone;
}

inline bool overlaps(const float *p, size_t floats, uintptr_t lo, uintptr_t hi) {
  const uintptr_t a = (uintptr_t)p, b = a + floats * sizeof(float);
  return p != nullptr && a < hi && lo < b;
}
inline size_t key_floats(const uint32_t (&d)[4]) { return (size_t)d[0] * d[1] * d[2] * d[3]; }

bool written_by_a_graph(const PackKey &k) {
  if (g_graph_writes_anything) return true;
  for (const auto &r : g_graph_written)
    if (overlaps(k.kernel, key_floats(k.kernel_dims), r.first, r.second) || overlaps(k.bias, key_floats(k.bias_dims), r.first, r.second)) return true;
  return false;
}

// Buffers of evicted entries that a recorded graph may still name: they stay allocated, are counted
// ("pack_cache_spare_bytes") and serve the same key again when it comes back.
std::vector<PackEntry> g_pack_spare;

void drop_entry(size_t i) {  // the stream is idle
  if (g_packs[i].pinned) {
    g_packs[i].valid = false;
    g_pack_spare.push_back(g_packs[i]);
  } else {
    (void)hipFree(g_packs[i].buf);
  }
  g_packs.erase(g_packs.begin() + i);
}

// Where the re-ordered weights of `key` live: *fresh tells the caller to make them (again).
// While the stream is captured the recording makes them itself at every replay -- into the entry's own buffer when
// the weights have been used before (the buffer is then never freed), else into the workspace.
int pack_buffer(const PackKey &key, size_t floats, float **buf, bool *fresh) {
  *fresh = true;
  if (!g_pack_cache || floats * sizeof(float) > PACK_MAX_BYTES / 4) return workspace(floats, buf);
  const bool recording = capturing();
  g_pack_clock++;
  for (PackEntry &e : g_packs)
    if (e.key == key && e.floats == floats) {
      e.used = g_pack_clock;
      *buf = e.buf;
      if (recording) { e.pinned = true; return MT_OK; }
      *fresh = !e.valid || written_by_a_graph(key);
      e.valid = true;
      if (*fresh) g_pack_made++; else g_pack_hits++;
      return MT_OK;
    }
  if (recording) return workspace(floats, buf);
  size_t bytes = floats * sizeof(float);
  for (const PackEntry &e : g_packs) bytes += e.floats * sizeof(float);
  while (!g_packs.empty() && (g_packs.size() >= PACK_MAX_ENTRIES || bytes > PACK_MAX_BYTES)) {  // least recently used goes
    size_t lru = 0;
    for (size_t i = 1; i < g_packs.size(); i++)
      if (g_packs[i].used < g_packs[lru].used) lru = i;
    MT_HIP(hipStreamSynchronize(mt::stream()));
    bytes -= g_packs[lru].floats * sizeof(float);
    drop_entry(lru);
  }
  PackEntry e;
  e.key = key; e.floats = floats; e.valid = true; e.used = g_pack_clock;
  for (size_t i = 0; i < g_pack_spare.size(); i++)
    if (g_pack_spare[i].key == key && g_pack_spare[i].floats == floats) {  // the buffer a graph still names: the same weights again
      e.buf = g_pack_spare[i].buf;
      e.pinned = true;
      g_pack_spare.erase(g_pack_spare.begin() + i);
      break;
    }
  if (e.buf == nullptr) {
    MT_HIP(hipMalloc((void **)&e.buf, floats * sizeof(float)));
    mt::count_driver_allocation();
  }
  g_packs.push_back(e);
  g_pack_made++;
  *buf = e.buf;
  return MT_OK;
}

struct ConvGeo {
  uint32_t out_w, in_w, ker_w, bias_w;
  int32_t C, H, W;      // input depth and size (image of a forward conv, delta of a transposed one)
  int32_t KA;           // kernel_amount
  int32_t KY, KX, SY, SX, PY, PX;
  int32_t OH, OW, OZ;   // output size and depth
  uint32_t ker_ld, ker_rows;
};

// ---- direct kernels: CPU loop order, no contraction, so results equal the CPU path bit for bit ------------------
__global__ __launch_bounds__(256) void fwd_direct_kernel(float *out, const float *image, const float *kernel, const float *bias, ConvGeo g, size_t total) {
  size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int32_t x = idx % g.OW, y = (idx / g.OW) % g.OH, k = (idx / ((size_t)g.OW * g.OH)) % g.OZ;
  uint32_t w = idx / ((size_t)g.OW * g.OH * g.OZ);
  const float *img = image + (size_t)(w % g.in_w) * g.C * g.H * g.W;
  const float *ker = kernel + ((size_t)(w % g.ker_w) * g.ker_rows + k) * g.ker_ld;
  float acc = bias[(size_t)(w % g.bias_w) * g.KA + k];
  int32_t taps = g.KX * g.KY;
  for (int32_t ky = 0; ky < g.KY; ky++) {
    int32_t iy = g.SY * y + ky - g.PY;
    if (iy < 0 || iy >= g.H) continue;
    for (int32_t kx = 0; kx < g.KX; kx++) {
      int32_t ix = g.SX * x + kx - g.PX;
      if (ix < 0 || ix >= g.W) continue;
      for (int32_t c = 0; c < g.C; c++) acc += ker[c * taps + ky * g.KX + kx] * img[((size_t)c * g.H + iy) * g.W + ix];
    }
  }
  out[idx] = acc;
}

__global__ __launch_bounds__(256) void tconv_direct_kernel(float *out, const float *delta, const float *kernel, const float *bias, ConvGeo g, size_t total, int func) {
  size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int32_t x = idx % g.OW, y = (idx / g.OW) % g.OH, z = (idx / ((size_t)g.OW * g.OH)) % g.OZ;
  uint32_t w = idx / ((size_t)g.OW * g.OH * g.OZ);
  const float *dl = delta + (size_t)(w % g.in_w) * g.C * g.H * g.W;
  const float *ker = kernel + (size_t)(w % g.ker_w) * g.ker_rows * g.ker_ld;
  const float *bs = bias + (size_t)(w % g.bias_w) * g.KA;
  int32_t pad_y = g.KY - 1 - g.PY, pad_x = g.KX - 1 - g.PX, taps = g.KX * g.KY;
  float acc = 0.f;
  for (int32_t ky = 0; ky < g.KY; ky++) {
    int32_t py = y + ky - pad_y;
    if (py % g.SY != 0) continue;
    int32_t dy = py / g.SY;
    if (dy < 0 || dy >= g.H) continue;
    for (int32_t kx = 0; kx < g.KX; kx++) {
      int32_t px = x + kx - pad_x;
      if (px % g.SX != 0) continue;
      int32_t dx = px / g.SX;
      if (dx < 0 || dx >= g.W) continue;
      int32_t col = z * taps + (g.KY - 1 - ky) * g.KX + (g.KX - 1 - kx);
      for (int32_t f = 0; f < g.KA; f++) {
        acc += bs[f];
        acc += ker[(size_t)f * g.ker_ld + col] * dl[((size_t)f * g.H + dy) * g.W + dx];
      }
    }
  }
  out[idx] = mt::apply_func(func, acc);
}

// one thread per gradient coefficient (w, f, c, i, j); pixels are visited in the CPU order
__global__ __launch_bounds__(256) void wgrad_direct_kernel(float *dk, const float *image, const float *delta, ConvGeo g, uint32_t delta_w, int32_t DH, int32_t DW, size_t total) {
  size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  int32_t taps = g.KX * g.KY, ncol = g.C * taps;
  int32_t col = idx % ncol, f = (idx / ncol) % g.KA;
  uint32_t w = idx / ((size_t)ncol * g.KA);
  int32_t c = col / taps, i = (col % taps) / g.KX, j = col % g.KX;
  const float *img = image + ((size_t)(w % g.in_w) * g.C + c) * g.H * g.W;
  const float *dl = delta + ((size_t)(w % delta_w) * g.KA + f) * DH * DW;
  float *dst = dk + ((size_t)w * g.ker_rows + f) * g.ker_ld + col;
  float acc = *dst;
  for (int32_t oy = 0; oy < DH; oy++) {
    int32_t iy = i + oy * g.SY - g.PY;
    if (iy < 0 || iy >= g.H) continue;
    for (int32_t ox = 0; ox < DW; ox++) {
      int32_t ix = j + ox * g.SX - g.PX;
      if (ix < 0 || ix >= g.W) continue;
      acc += dl[oy * DW + ox] * img[(size_t)iy * g.W + ix];
    }
  }
  *dst = acc;
}

// bias gradient, CPU order: for each stored row (wb, f), samples w = wb, wb + Wb, ... then pixels in order
__global__ __launch_bounds__(256) void dbias_serial_kernel(float *dbias, uint32_t dbias_w, const float *delta, uint32_t delta_w, uint32_t KA, uint32_t DHW, uint32_t W) {
  uint32_t idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= dbias_w * KA) return;
  uint32_t wb = idx / KA, f = idx % KA;
  float b = dbias[idx];
  for (uint32_t w = wb; w < W; w += dbias_w) {
    const float *dl = delta + ((size_t)(w % delta_w) * KA + f) * DHW;
    for (uint32_t i = 0; i < DHW; i++) b += dl[i];
  }
  dbias[idx] = b;
}

// bias gradient when every sample owns its row of dbias: one wavefront per (w, f)
__global__ __launch_bounds__(256) void dbias_wave_kernel(float *dbias, const float *delta, uint32_t delta_w, uint32_t KA, uint32_t DHW, uint32_t rows) {
  uint32_t row = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
  if (row >= rows) return;
  uint32_t w = row / KA, f = row % KA;
  const float *dl = delta + ((size_t)(w % delta_w) * KA + f) * DHW;
  float s = 0.f;
  for (uint32_t i = lane; i < DHW; i += 64) s += dl[i];
  s = mt::wave_sum(s);
  if (lane == 0) dbias[row] += s;
}

// Sum over the whole batch and all pixels of delta[w][f], one value per filter.  Block (f, c) adds the samples
// c*per .. (c+1)*per-1 of filter f (V = float4 when the rows allow it, else float) and writes partial[f*chunks + c],
// or adds to dbias[f] itself when chunks == 1.  The partials are added in a fixed order by dbias_finish_kernel.
template <class V>
__global__ __launch_bounds__(256) void dbias_batch_sum_kernel(float *dbias, float *partial, const V *delta, uint32_t per, uint32_t KA, uint32_t DV, uint32_t chunks) {
  const uint32_t f = blockIdx.x, c = blockIdx.y, t = threadIdx.x;
  const uint32_t count = per * DV;  // vectors of this block
  const V *base = delta + ((size_t)c * per * KA + f) * DV;
  const size_t sample = (size_t)KA * DV;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  auto at = [&](uint32_t i) -> float {
    if (i >= count) return 0.f;
    const uint32_t w = i / DV, x = i - w * DV;
    const V v = base[(size_t)w * sample + x];
    if constexpr (sizeof(V) == 16) return (v.x + v.y) + (v.z + v.w);
    else return v;
  };
  for (uint32_t i = t; i < count; i += 1024) {
    s0 += at(i); s1 += at(i + 256); s2 += at(i + 512); s3 += at(i + 768);
  }
  __shared__ float part[4];
  const float s = mt::wave_sum((s0 + s1) + (s2 + s3));
  if (t % 64 == 0) part[t / 64] = s;
  __syncthreads();
  if (t == 0) {
    const float sum = (part[0] + part[1]) + (part[2] + part[3]);
    if (chunks == 1) dbias[f] += sum;
    else partial[f * chunks + c] = sum;
  }
}
__global__ __launch_bounds__(256) void dbias_finish_kernel(float *dbias, const float *partial, uint32_t KA, uint32_t chunks) {
  const uint32_t f = blockIdx.x * 256 + threadIdx.x;
  if (f >= KA) return;
  float s = 0.f;
  for (uint32_t c = 0; c < chunks; c++) s += partial[f * chunks + c];
  dbias[f] += s;
}
// chunks of the batch per filter: enough blocks to fill the device, each with at least a few thousand values
uint32_t dbias_chunks(uint32_t B, uint32_t KA, uint32_t DHW) {
  uint32_t chunks = 1;
  while (chunks * 2 <= B && B % (chunks * 2) == 0 && KA * chunks < 1024 && (size_t)(B / (chunks * 2)) * DHW >= 4096) chunks *= 2;
  return chunks;
}
int dbias_batch_sum(const char *name, float *dbias, float *partial, const float *delta, uint32_t B, uint32_t KA, uint32_t DHW, uint32_t chunks) {
  const dim3 grid(KA, chunks);
  if (DHW % 4 == 0 && ((uintptr_t)delta & 15u) == 0)
    dbias_batch_sum_kernel<float4><<<grid, 256, 0, mt::stream()>>>(dbias, partial, (const float4 *)delta, B / chunks, KA, DHW / 4, chunks);
  else
    dbias_batch_sum_kernel<float><<<grid, 256, 0, mt::stream()>>>(dbias, partial, delta, B / chunks, KA, DHW, chunks);
  MT_LAUNCH_CHECK(name);
  if (chunks > 1) {
    dbias_finish_kernel<<<cdiv(KA, 256), 256, 0, mt::stream()>>>(dbias, partial, KA, chunks);
    MT_LAUNCH_CHECK(name);
  }
  return MT_OK;
}

// ---- transposed convolution: phase geometry, kernel packing, bias sums ----------------------------------------
struct Phase1D {
  int32_t k0, taps, off, q;  // first tap, tap count, input offset, number of output rows/columns in the phase
};
// outputs y = q*s + ph (q = 0..); taps ky = k0 + t*s; the input row of (q, t) is q + t + off
Phase1D phase_1d(int32_t ph, int32_t K, int32_t s, int32_t p, int32_t O) {
  int32_t pad = K - 1 - p;
  Phase1D r;
  r.k0 = ((pad - ph) % s + s) % s;
  r.taps = r.k0 < K ? (K - r.k0 + s - 1) / s : 0;
  r.off = (ph + r.k0 - pad) / s;  // exact: ph + k0 - pad is a multiple of s
  r.q = O > ph ? (O - ph + s - 1) / s : 0;
  return r;
}

// One launch prepares a transposed convolution: blockIdx.y < nphase packs that phase's sub-kernel,
//   packed_f[co][(ci, ty, tx)] = kernel[ci][co*KY*KX + (KY-1-(ky0+ty*sy))*KX + (KX-1-(kx0+tx*sx))],
// (or, with other strides, [ci][phase][co][taps] for the kernel that reads all coefficients of a channel at once)
// and blockIdx.y == nphase sums the biases of every bias layer (the CPU path adds all of them per tap).
struct PackPhase {
  uint32_t begin, kp, ld;  // offset of the phase in the packed buffer (floats), coefficients per row, padded row length
  int32_t ky0, kx0, ty, tx;
  uint32_t co_stride, ci_stride;  // coefficient (co, ci, t) goes to begin + co*co_stride + ci*ci_stride + t
};
struct PackArgs {
  PackPhase ph[MAX_PHASES];
  uint32_t nphase, ker_ld, bias_w;
  int32_t CO, CI, KY, KX, SY, SX;
};
__global__ __launch_bounds__(256) void tconv_prepare_kernel(float *packed, float *sums, const float *kernel, const float *bias, PackArgs pa) {
  if (blockIdx.y == pa.nphase) {
    uint32_t wave = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64, waves = gridDim.x * 4;
    for (uint32_t w = wave; w < pa.bias_w; w += waves) {
      float acc = 0.f;
      for (uint32_t i = lane; i < (uint32_t)pa.CI; i += 64) acc += bias[(size_t)w * pa.CI + i];
      acc = mt::wave_sum(acc);
      if (lane == 0) sums[w] = acc;
    }
    return;
  }
  const PackPhase ph = pa.ph[blockIdx.y];
  const uint32_t taps = ph.ty * ph.tx, total = (uint32_t)pa.CO * ph.ld;
  for (uint32_t idx = blockIdx.x * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
    uint32_t co = idx / ph.ld, k = idx % ph.ld;
    if (k < ph.kp) {
      uint32_t ci = k / taps, t = k % taps, ty = t / ph.tx, tx = t % ph.tx;
      int32_t ky = ph.ky0 + ty * pa.SY, kx = ph.kx0 + tx * pa.SX;
      packed[ph.begin + co * ph.co_stride + ci * ph.ci_stride + t] =
          kernel[(size_t)ci * pa.ker_ld + co * pa.KY * pa.KX + (pa.KY - 1 - ky) * pa.KX + (pa.KX - 1 - kx)];
    } else {
      packed[ph.begin + idx] = 0.f;  // rows [co][k] are zero-padded to a multiple of four coefficients
    }
  }
}

// The same preparation for the common geometry kernel 4x4, stride 2 (four phases of 2x2 taps): one thread per
// (input channel, output channel) reads the 16 contiguous coefficients of that pair once (four 128-bit loads) and
// writes each phase its four; consecutive threads take consecutive input channels, so the writes of a wavefront are
// contiguous.  blockIdx.y == CO sums the biases.
__global__ __launch_bounds__(256) void tconv_prepare_k4s2_kernel(float *packed, float *sums, const float *kernel, const float *bias, PackArgs pa) {
  if (blockIdx.y == (uint32_t)pa.CO) {
    uint32_t wave = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64, waves = gridDim.x * 4;
    for (uint32_t w = wave; w < pa.bias_w; w += waves) {
      float acc = 0.f;
      for (uint32_t i = lane; i < (uint32_t)pa.CI; i += 64) acc += bias[(size_t)w * pa.CI + i];
      acc = mt::wave_sum(acc);
      if (lane == 0) sums[w] = acc;
    }
    return;
  }
  const uint32_t ci = blockIdx.x * 256 + threadIdx.x, co = blockIdx.y;
  if (ci >= (uint32_t)pa.CI) return;
  float k[16];
  const float4 *src = reinterpret_cast<const float4 *>(kernel + (size_t)ci * pa.ker_ld + co * 16);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float4 t = src[i];
    k[4 * i] = t.x; k[4 * i + 1] = t.y; k[4 * i + 2] = t.z; k[4 * i + 3] = t.w;
  }
#pragma unroll
  for (int f = 0; f < 4; f++) {
    const PackPhase &ph = pa.ph[f];
    float4 o;
    // tap (ty, tx) of the phase is coefficient (3 - (ky0 + 2*ty), 3 - (kx0 + 2*tx)) of the kernel
    float v[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
      const int ky = ph.ky0 + 2 * (t / 2), kx = ph.kx0 + 2 * (t % 2);
      const int idx = (3 - ky) * 4 + (3 - kx);
      float r = k[0];
#pragma unroll
      for (int q = 1; q < 16; q++) r = idx == q ? k[q] : r;   // ky0, kx0 are uniform: selects, no indexed registers
      v[t] = r;
    }
    o = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4 *>(packed + ph.begin + (size_t)co * ph.co_stride + (size_t)ci * ph.ci_stride) = o;
  }
}

// ---- transposed convolution with very few output channels (the image-producing last layer) --------------------
// A 32-row matrix-core tile would be 90% padding for 3 output channels, so this case runs on the vector ALUs:
// one thread per output pixel of one stride phase (blockIdx.y), CO accumulators, the packed sub-kernel read
// through the scalar cache (its address is uniform), the delta read with lanes along x (coalesced, neighbours
// share cache lines).  TY/TX = 0 means "tap counts known only at run time".
template <int CO, int TY, int TX>
__global__ __launch_bounds__(256) void tconv_small_kernel(TconvArgs args) {
  const TconvPhase ph = args.ph[blockIdx.y];
  const uint32_t qhw = ph.qh * ph.qw, N = args.out_w * qhw;
  const uint32_t n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  const int ty_cnt = TY ? TY : ph.taps_y, tx_cnt = TX ? TX : ph.taps_x;
  const uint32_t g = n / qhw, r = n % qhw, qy = r / ph.qw, qx = r % ph.qw;
  const uint32_t H = args.H, W = args.W, C = args.C;
  const float *in = args.delta + (size_t)(g % args.in_w) * C * H * W;
  const int32_t y0 = (int32_t)qy + ph.offy, x0 = (int32_t)qx + ph.offx;
  float acc[CO];
#pragma unroll
  for (int co = 0; co < CO; co++) acc[co] = 0.f;
  const uint32_t taps = ty_cnt * tx_cnt;
  for (uint32_t ci = 0; ci < C; ci++) {
    const float *plane = in + (size_t)ci * H * W;
    const float *wrow = ph.packed + ci * taps;
#pragma unroll
    for (int ty = 0; ty < (TY ? TY : 4); ty++) {
      if (!TY && ty >= ty_cnt) break;
      const int32_t iy = y0 + ty;
      const bool yok = (uint32_t)iy < H;
#pragma unroll
      for (int tx = 0; tx < (TX ? TX : 4); tx++) {
        if (!TX && tx >= tx_cnt) break;
        const int32_t ix = x0 + tx;
        const bool ok = yok && (uint32_t)ix < W;
        const float v = ok ? plane[(size_t)(ok ? iy : 0) * W + (ok ? ix : 0)] : 0.f;
#pragma unroll
        for (int co = 0; co < CO; co++)
          if (co < (int)args.M) acc[co] = __builtin_fmaf(wrow[(size_t)co * ph.ld + ty * tx_cnt + tx], v, acc[co]);
      }
    }
  }
  Epilogue ep = args.ep;
  ep.inner = qhw; ep.qw = ph.qw; ep.py = ph.py; ep.px = ph.px;
  ep.ty_cnt = ph.taps_y; ep.tx_cnt = ph.taps_x; ep.offy = ph.offy; ep.offx = ph.offx;
  Epilogue::Col col = ep.column(n);
#pragma unroll
  for (int co = 0; co < CO; co++)
    if (co < (int)args.M) ep.store(col, co, acc[co]);
}

// The same case for the common geometry kernel 4x4, stride 2, padding 1 (output exactly twice the input):
// one thread per INPUT pixel computes the 2x2 output pixels it maps to, i.e. all four stride phases, for CO output
// channels.  The four phases together read the 3x3 neighbourhood of the input pixel, so per input channel a
// thread issues 9 loads for 16*CO multiply-adds.  The loads are buffer loads whose 9 byte offsets (or the
// out-of-range marker for neighbours outside the image) are computed once; the channel advances through the
// scalar offset.  The 16*CO coefficients of a channel are uniform and come through the scalar cache.
// The input channels are split over the 4 wavefronts of a block (64 input pixels per block): four times as many
// loads in flight, partial sums combined through LDS.
template <int CO>
__global__ __launch_bounds__(256) void tconv_k4s2_small_kernel(TconvArgs args) {
  constexpr int SLICES = 4, PIX = 64;
  __shared__ float part[SLICES - 1][4 * CO][PIX];
  const uint32_t H = args.H, W = args.W, C = args.C, HW = H * W;
  const uint32_t pix = threadIdx.x % PIX, slice = threadIdx.x / PIX;   // the slice is uniform over a wavefront
  const uint32_t n = blockIdx.x * PIX + pix;
  const bool live = n < args.out_w * HW;
  const uint32_t g = (live ? n : 0) / HW, r = (live ? n : 0) % HW, qy = r / W, qx = r % W;
  __amdgpu_buffer_rsrc_t rsrc = make_rsrc(args.delta, args.in_w * C * HW * 4u);
  const uint32_t imgoff = (g % args.in_w) * C * HW * 4u;
  uint32_t voff[3][3];
#pragma unroll
  for (int dy = 0; dy < 3; dy++)
#pragma unroll
    for (int dx = 0; dx < 3; dx++) {
      int32_t iy = (int32_t)qy + dy - 1, ix = (int32_t)qx + dx - 1;
      bool ok = live && (uint32_t)iy < H && (uint32_t)ix < W;
      voff[dy][dx] = ok ? imgoff + ((uint32_t)iy * W + (uint32_t)ix) * 4u : OOB;
    }
  float acc[2][2][CO];
#pragma unroll
  for (int i = 0; i < 4 * CO; i++) (&acc[0][0][0])[i] = 0.f;
  const uint32_t M = args.M;
  const uint32_t per = (C + SLICES - 1) / SLICES;
  const uint32_t c_begin = __builtin_amdgcn_readfirstlane(slice * per);
  const uint32_t c_end = c_begin + per < C ? c_begin + per : C;
#pragma unroll 4
  for (uint32_t ci = c_begin; ci < c_end; ci++) {
    const uint32_t soff = ci * HW * 4u;
    float v[3][3];
#pragma unroll
    for (int dy = 0; dy < 3; dy++)
#pragma unroll
      for (int dx = 0; dx < 3; dx++) v[dy][dx] = buf_load(rsrc, voff[dy][dx], soff);
#pragma unroll
    for (int py = 0; py < 2; py++)
#pragma unroll
      for (int px = 0; px < 2; px++) {
        const TconvPhase &ph = args.ph[py * 2 + px];
#pragma unroll
        for (int co = 0; co < CO; co++) {
          if (co >= (int)M) continue;
          const float4 w = *reinterpret_cast<const float4 *>(ph.packed + (size_t)co * ph.ld + ci * 4u);  // taps (ty,tx) = 00 01 10 11
          float a = acc[py][px][co];
          a = __builtin_fmaf(w.x, v[py][px], a);
          a = __builtin_fmaf(w.y, v[py][px + 1], a);
          a = __builtin_fmaf(w.z, v[py + 1][px], a);
          a = __builtin_fmaf(w.w, v[py + 1][px + 1], a);
          acc[py][px][co] = a;
        }
      }
  }
  if (slice > 0) {
#pragma unroll
    for (int i = 0; i < 4 * CO; i++) part[slice - 1][i][pix] = (&acc[0][0][0])[i];
  }
  __syncthreads();
  if (slice > 0 || !live) return;
#pragma unroll
  for (int i = 0; i < 4 * CO; i++)
#pragma unroll
    for (int sl = 0; sl < SLICES - 1; sl++) (&acc[0][0][0])[i] += part[sl][i][pix];
  const uint32_t OW = 2 * W, OHW = 4 * HW;
  const float bsum = args.ep.tap_bias ? args.ep.tap_bias[g % args.ep.bias_w] : 0.f;
#pragma unroll
  for (int py = 0; py < 2; py++) {
    // contributing taps of output row 2*qy+py are input rows qy+py-1 and qy+py
    const int ny = ((uint32_t)((int32_t)qy + py - 1) < H) + ((uint32_t)((int32_t)qy + py) < H);
    const int nx0 = ((uint32_t)((int32_t)qx - 1) < W) + 1, nx1 = 1 + ((uint32_t)((int32_t)qx + 1) < W);
#pragma unroll
    for (int co = 0; co < CO; co++) {
      if (co >= (int)M) continue;
      float2 o;
      o.x = mt::apply_func_epilogue(args.ep.func, acc[py][0][co] + bsum * (float)(ny * nx0));
      o.y = mt::apply_func_epilogue(args.ep.func, acc[py][1][co] + bsum * (float)(ny * nx1));
      float *dst = args.ep.C + ((size_t)g * M + co) * OHW + (size_t)(2 * qy + py) * OW + 2 * qx;
      *reinterpret_cast<float2 *>(dst) = o;
    }
  }
}

// The same for kernel 5x5, stride 2, padding 2 (output exactly twice the input: the first layer of a discriminator on
// images, backwards): output pixel (2*qy + py, 2*qx + px) reads input rows qy + py - 1 .. qy + 1 and columns
// qx + px - 1 .. qx + 1, so the four phases -- 3x3, 3x2, 2x3 and 2x2 taps -- again share the 3x3 neighbourhood of the input
// pixel: per input channel a thread issues 9 loads for 25*CO multiply-adds.  Phase (py, px) has 3-py by 3-px taps with
// offsets (py-1, px-1); tap (ty, tx) multiplies neighbour (py + ty, px + tx).
template <int CO>
__global__ __launch_bounds__(256) void tconv_k5s2_small_kernel(TconvArgs args) {
  constexpr int SLICES = 4, PIX = 64;
  __shared__ float part[SLICES - 1][4 * CO][PIX];
  const uint32_t H = args.H, W = args.W, C = args.C, HW = H * W;
  const uint32_t pix = threadIdx.x % PIX, slice = threadIdx.x / PIX;   // the slice is uniform over a wavefront
  const uint32_t n = blockIdx.x * PIX + pix;
  const bool live = n < args.out_w * HW;
  const uint32_t g = (live ? n : 0) / HW, r = (live ? n : 0) % HW, qy = r / W, qx = r % W;
  __amdgpu_buffer_rsrc_t rsrc = make_rsrc(args.delta, args.in_w * C * HW * 4u);
  const uint32_t imgoff = (g % args.in_w) * C * HW * 4u;
  uint32_t voff[3][3];
#pragma unroll
  for (int dy = 0; dy < 3; dy++)
#pragma unroll
    for (int dx = 0; dx < 3; dx++) {
      int32_t iy = (int32_t)qy + dy - 1, ix = (int32_t)qx + dx - 1;
      bool ok = live && (uint32_t)iy < H && (uint32_t)ix < W;
      voff[dy][dx] = ok ? imgoff + ((uint32_t)iy * W + (uint32_t)ix) * 4u : OOB;
    }
  float acc[2][2][CO];
#pragma unroll
  for (int i = 0; i < 4 * CO; i++) (&acc[0][0][0])[i] = 0.f;
  const uint32_t M = args.M;
  const uint32_t per = (C + SLICES - 1) / SLICES;
  const uint32_t c_begin = __builtin_amdgcn_readfirstlane(slice * per);
  const uint32_t c_end = c_begin + per < C ? c_begin + per : C;
#pragma unroll 2
  for (uint32_t ci = c_begin; ci < c_end; ci++) {
    const uint32_t soff = ci * HW * 4u;
    float v[3][3];
#pragma unroll
    for (int dy = 0; dy < 3; dy++)
#pragma unroll
      for (int dx = 0; dx < 3; dx++) v[dy][dx] = buf_load(rsrc, voff[dy][dx], soff);
#pragma unroll
    for (int py = 0; py < 2; py++)
#pragma unroll
      for (int px = 0; px < 2; px++) {
        const TconvPhase &ph = args.ph[py * 2 + px];
        const int ty_cnt = 3 - py, tx_cnt = 3 - px;
#pragma unroll
        for (int co = 0; co < CO; co++) {
          if (co >= (int)M) continue;
          const float *w = ph.packed + (size_t)co * ph.ld + ci * (uint32_t)(ty_cnt * tx_cnt);   // uniform: through the scalar cache
          float a = acc[py][px][co];
#pragma unroll
          for (int ty = 0; ty < ty_cnt; ty++)
#pragma unroll
            for (int tx = 0; tx < tx_cnt; tx++) a = __builtin_fmaf(w[ty * tx_cnt + tx], v[py + ty][px + tx], a);
          acc[py][px][co] = a;
        }
      }
  }
  if (slice > 0) {
#pragma unroll
    for (int i = 0; i < 4 * CO; i++) part[slice - 1][i][pix] = (&acc[0][0][0])[i];
  }
  __syncthreads();
  if (slice > 0 || !live) return;
#pragma unroll
  for (int i = 0; i < 4 * CO; i++)
#pragma unroll
    for (int sl = 0; sl < SLICES - 1; sl++) (&acc[0][0][0])[i] += part[sl][i][pix];
  const uint32_t OW = 2 * W, OHW = 4 * HW;
  const float bsum = args.ep.tap_bias ? args.ep.tap_bias[g % args.ep.bias_w] : 0.f;
  const int up = (uint32_t)((int32_t)qy - 1) < H, down = (uint32_t)((int32_t)qy + 1) < H;
  const int left = (uint32_t)((int32_t)qx - 1) < W, right = (uint32_t)((int32_t)qx + 1) < W;
#pragma unroll
  for (int py = 0; py < 2; py++) {
    // contributing input rows of output row 2*qy+py: qy-1 (py = 0 only), qy, qy+1; columns alike
    const int ny = (py == 0 ? up : 0) + 1 + down;
    const int nx0 = left + 1 + right, nx1 = 1 + right;
#pragma unroll
    for (int co = 0; co < CO; co++) {
      if (co >= (int)M) continue;
      float2 o;
      o.x = mt::apply_func_epilogue(args.ep.func, acc[py][0][co] + bsum * (float)(ny * nx0));
      o.y = mt::apply_func_epilogue(args.ep.func, acc[py][1][co] + bsum * (float)(ny * nx1));
      float *dst = args.ep.C + ((size_t)g * M + co) * OHW + (size_t)(2 * qy + py) * OW + 2 * qx;
      *reinterpret_cast<float2 *>(dst) = o;
    }
  }
}

// Staging of an input tile with a one-pixel halo through registers into LDS, shared by the vector-ALU kernels below:
// per channel (TH+2) rows of [x0-1 | x0 .. x0+TW-1 | x0+TW] (PITCH floats, the tile itself starts at column 1), CC
// channels per chunk.  The tile columns are fetched with 128-bit buffer loads, the two halo columns with 32-bit ones;
// everything outside the image comes back as zero through the range check.  The byte offsets of a thread's pieces are
// computed once; the chunk advances through the scalar offset.  Needs W % 4 == 0 and 16-byte aligned rows.
// NORM: the input still owes func(scale * x + shift) with one (scale, shift) pair per element [C][H][W]; the pairs of a
// piece are fetched beside it (two 128-bit loads for the four pairs of a 128-bit piece) and applied on the way to LDS.
// Pieces outside the image load their pairs out of range as well: func(0 * 0 + 0) = 0 keeps the padding zero.
template <int TW, int TH, int CC, bool NORM = false>
struct HaloTile {
  static constexpr int PITCH = TW + 4, ROWS = TH + 2, FLOATS = CC * ROWS * PITCH;
  static constexpr int VEC = CC * ROWS * (TW / 4), NVEC = (VEC + 255) / 256;
  static constexpr int EDGE = CC * ROWS * 2, NEDGE = (EDGE + 255) / 256;
  __amdgpu_buffer_rsrc_t rsrc, prsrc;
  uint32_t voff[NVEC], eoff[NEDGE], vdst[NVEC], edst[NEDGE], chunk_bytes, image_bytes;
  int in_func;
  floatx4 rv[NVEC];
  float re[NEDGE];
  floatx4 pv[NORM ? NVEC : 1][2];
  floatx2 pe[NORM ? NEDGE : 1];
  __device__ void setup(const float *p, uint32_t bytes, uint32_t imgoff, uint32_t H, uint32_t W, uint32_t x0, uint32_t y0, uint32_t tid,
                        const float *pairs = nullptr, uint32_t channels = 0, int func = MT_F_NONE) {
    rsrc = make_rsrc(p, bytes);
    prsrc = rsrc;
    if (NORM) prsrc = make_rsrc(pairs, channels * H * W * 8u);
    in_func = func;
    image_bytes = imgoff;
    chunk_bytes = CC * H * W * 4u;
#pragma unroll
    for (int i = 0; i < NVEC; i++) {
      const uint32_t idx = tid + i * 256, row = idx / (TW / 4), seg = idx % (TW / 4), c = row / ROWS, yy = row % ROWS;
      const int32_t iy = (int32_t)(y0 + yy) - 1;
      const uint32_t ix = x0 + seg * 4;
      const bool ok = idx < VEC && (uint32_t)iy < H && ix < W;
      voff[i] = ok ? imgoff + ((c * H + (uint32_t)iy) * W + ix) * 4u : OOB;
      vdst[i] = idx < VEC ? (c * ROWS + yy) * PITCH + 1 + seg * 4 : 0xffffffffu;
    }
#pragma unroll
    for (int i = 0; i < NEDGE; i++) {
      const uint32_t idx = tid + i * 256, row = idx / 2, side = idx % 2, c = row / ROWS, yy = row % ROWS;
      const int32_t iy = (int32_t)(y0 + yy) - 1, ix = side ? (int32_t)(x0 + TW) : (int32_t)x0 - 1;
      const bool ok = idx < EDGE && (uint32_t)iy < H && (uint32_t)ix < W;
      eoff[i] = ok ? imgoff + ((c * H + (uint32_t)iy) * W + (uint32_t)ix) * 4u : OOB;
      edst[i] = idx < EDGE ? (c * ROWS + yy) * PITCH + (side ? TW + 1 : 0) : 0xffffffffu;
    }
  }
  __device__ void fetch(uint32_t chunk) {
    const uint32_t soff = chunk * chunk_bytes;
#pragma unroll
    for (int i = 0; i < NVEC; i++) rv[i] = buf_load4(rsrc, voff[i], soff);
#pragma unroll
    for (int i = 0; i < NEDGE; i++) re[i] = buf_load(rsrc, eoff[i], soff);
    if constexpr (NORM) {  // the pairs of an element sit at twice its byte offset inside the sample
#pragma unroll
      for (int i = 0; i < NVEC; i++) {
        const uint32_t po = voff[i] == OOB ? OOB : (voff[i] - image_bytes) * 2u;
        pv[i][0] = buf_load4(prsrc, po, 2u * soff);
        pv[i][1] = buf_load4(prsrc, po == OOB ? OOB : po + 16u, 2u * soff);
      }
#pragma unroll
      for (int i = 0; i < NEDGE; i++) pe[i] = buf_load2(prsrc, eoff[i] == OOB ? OOB : (eoff[i] - image_bytes) * 2u, 2u * soff);
    }
  }
  __device__ void put(float *t) const {
#pragma unroll
    for (int i = 0; i < NVEC; i++)
      if (vdst[i] != 0xffffffffu) {  // the tile starts at an odd column: 4 + 8 + 4 bytes
        floatx4 v = rv[i];
        if constexpr (NORM) {
          v.x = mt::apply_func_cheap(in_func, pv[i][0].x * v.x + pv[i][0].y);
          v.y = mt::apply_func_cheap(in_func, pv[i][0].z * v.y + pv[i][0].w);
          v.z = mt::apply_func_cheap(in_func, pv[i][1].x * v.z + pv[i][1].y);
          v.w = mt::apply_func_cheap(in_func, pv[i][1].z * v.w + pv[i][1].w);
        }
        t[vdst[i]] = v.x;
        *reinterpret_cast<float2 *>(t + vdst[i] + 1) = make_float2(v.y, v.z);
        t[vdst[i] + 3] = v.w;
      }
#pragma unroll
    for (int i = 0; i < NEDGE; i++)
      if (edst[i] != 0xffffffffu) {
        float v = re[i];
        if constexpr (NORM) v = mt::apply_func_cheap(in_func, pe[i].x * v + pe[i].y);
        t[edst[i]] = v;
      }
  }
};

// The same geometry with the input staged through LDS: a block owns a tile of 32 x 16 input pixels of one image
// (64 x 32 output pixels) and walks the input channels in chunks of CC.  A chunk's (16+2) x (32+2) halo tile per
// channel is fetched with 128-bit buffer loads (zero outside the image through the range check), kept in registers
// while the previous chunk is multiplied, then written to the other LDS buffer: one barrier per chunk.  A thread
// computes two neighbouring input pixels, i.e. 2 x 4 output pixels: per channel 6 LDS reads for 32*CO multiply-adds
// instead of 9 global loads for 16*CO, which moves the kernel from the texture-address path to the vector ALUs.
// Needs W % 4 == 0, C % CC == 0, 16-byte aligned rows, exactly CO output channels and the coefficients packed
// as [ci][phase][co][taps].
// PP = 2 as described; PP = 1: one input pixel per thread and tiles of 16 x 16, twice the wavefronts (and twice the LDS
// reads per multiply-add) for inputs so small that the grid would otherwise not give every SIMD two wavefronts.
// SPLIT = 2: the block is two halves of 256 threads that take every other chunk of (then four) channels, each with its
// own pair of LDS buffers, and add their sums at the end: twice the wavefronts per SIMD for a grid of two blocks per
// compute unit, where the multiply-adds of one wavefront otherwise wait for its own LDS and scalar loads.
template <int CO, int PP, int SPLIT, bool NORM>
__global__ __launch_bounds__(256 * SPLIT) void tconv_k4s2_tile_kernel(TconvArgs args) {
  constexpr int CC = SPLIT == 2 ? 4 : 8;
  using Tile = HaloTile<16 * PP, 16, CC, NORM>;
  constexpr int TW = 16 * PP, TH = 16, PITCH = Tile::PITCH, ROWS = Tile::ROWS;
  __shared__ __attribute__((aligned(16))) float tiles[SPLIT][2][CC][ROWS][PITCH];
  static_assert(SPLIT == 1 || sizeof(tiles) >= sizeof(float) * 256 * PP * 4 * CO, "the sums of the second half fit into the tile memory");
  const uint32_t H = args.H, W = args.W, C = args.C, HW = H * W, M = args.M;
  const uint32_t tiles_x = (W + TW - 1) / TW;
  // (an XCD takes a contiguous range of (image, tile): neighbouring tiles read each other's edge lines from one L2)
  const uint32_t logical = xcd_swizzle(blockIdx.y * gridDim.x + blockIdx.x, gridDim.x * gridDim.y);
  const uint32_t tile_id = logical % gridDim.x, g = logical / gridDim.x;
  const uint32_t x0 = (tile_id % tiles_x) * TW, y0 = (tile_id / tiles_x) * TH;
  const uint32_t half = SPLIT == 2 ? __builtin_amdgcn_readfirstlane(threadIdx.x / 256) : 0u, tid = threadIdx.x % 256, tx = tid % 16, ty = tid / 16;
  auto &tile = tiles[half];
  Tile stage;
  stage.setup(args.delta, args.in_w * C * HW * 4u, (g % args.in_w) * C * HW * 4u, H, W, x0, y0, tid, args.in_scale_shift, C, args.in_func);
  auto fetch = [&](uint32_t step) { stage.fetch(step * SPLIT + half); };
  auto put = [&](int buf) { stage.put(&tile[buf][0][0][0]); };

  float acc[PP][2][2][CO];  // [pixel][py][px][co]
#pragma unroll
  for (int i = 0; i < PP * 4 * CO; i++) (&acc[0][0][0][0])[i] = 0.f;
  const uint32_t chunks = C / (CC * SPLIT);  // steps of a half
  const float *coeff = args.ph[0].packed;
  fetch(0);
  put(0);
  __syncthreads();
  for (uint32_t ch = 0; ch < chunks; ch++) {
    const int cur = ch & 1;
    if (ch + 1 < chunks) fetch(ch + 1);
#pragma unroll 2
    for (int c = 0; c < CC; c++) {
      const uint32_t ci = (ch * SPLIT + half) * CC + c;
      float v[3][PP + 2];  // rows y-1..y+1, columns x-1..x+PP of the thread's pixels (x .. x+PP-1)
#pragma unroll
      for (int dy = 0; dy < 3; dy++) {
        const float *rowp = &tile[cur][c][ty + dy][PP * tx];
        if constexpr (PP == 2) {
          const float2 lo = *reinterpret_cast<const float2 *>(rowp), hi = *reinterpret_cast<const float2 *>(rowp + 2);
          v[dy][0] = lo.x; v[dy][1] = lo.y; v[dy][2] = hi.x; v[dy][3] = hi.y;
        } else {
          v[dy][0] = rowp[0]; v[dy][1] = rowp[1]; v[dy][2] = rowp[2];
        }
      }
      // all 16*CO coefficients of a channel are contiguous, [ci][phase][co][taps (ty,tx) = 00 01 10 11]: CO uniform
      // 64-byte loads through the scalar cache
      floatx16 wv[CO];
#pragma unroll
      for (int j = 0; j < CO; j++) wv[j] = reinterpret_cast<const floatx16 *>(coeff + (size_t)ci * (16 * CO))[j];
#pragma unroll
      for (int py = 0; py < 2; py++)
#pragma unroll
        for (int px = 0; px < 2; px++) {
#pragma unroll
          for (int co = 0; co < CO; co++) {
            const int f = ((py * 2 + px) * CO + co) * 4;
            const float4 w = make_float4(wv[f / 16][f % 16], wv[f / 16][f % 16 + 1], wv[f / 16][f % 16 + 2], wv[f / 16][f % 16 + 3]);
#pragma unroll
            for (int p = 0; p < PP; p++) {
              float a = acc[p][py][px][co];
              a = __builtin_fmaf(w.x, v[py][p + px], a);
              a = __builtin_fmaf(w.y, v[py][p + px + 1], a);
              a = __builtin_fmaf(w.z, v[py + 1][p + px], a);
              a = __builtin_fmaf(w.w, v[py + 1][p + px + 1], a);
              acc[p][py][px][co] = a;
            }
          }
        }
    }
    if (ch + 1 < chunks) put(cur ^ 1);
    __syncthreads();
  }
  if constexpr (SPLIT == 2) {  // the second half hands its sums over through the tile memory (nobody reads tiles any more)
    float *sums = &tiles[0][0][0][0][0];
    if (half == 1) {
#pragma unroll
      for (int i = 0; i < PP * 4 * CO; i++) sums[i * 256 + tid] = (&acc[0][0][0][0])[i];
    }
    __syncthreads();
    if (half == 1) return;
#pragma unroll
    for (int i = 0; i < PP * 4 * CO; i++) (&acc[0][0][0][0])[i] += sums[i * 256 + tid];
  }

  const uint32_t qy = y0 + ty, qx = x0 + PP * tx;
  if (qy >= H || qx >= W) return;  // W is even: a pair is inside or outside as a whole
  const uint32_t OW = 2 * W, OHW = 4 * HW;
  const float bsum = args.ep.tap_bias ? args.ep.tap_bias[g % args.ep.bias_w] : 0.f;
  const int func = args.ep.func;
#pragma unroll
  for (int py = 0; py < 2; py++) {
    // contributing taps of output row 2*qy+py are input rows qy+py-1 and qy+py; likewise along x
    const int ny = ((uint32_t)((int32_t)qy + py - 1) < H) + ((uint32_t)((int32_t)qy + py) < H);
    int nx[2 * PP];  // output column 2*qx+i: two taps inside the row, one fewer at the image's left and right edge
#pragma unroll
    for (int i = 0; i < 2 * PP; i++) nx[i] = 2;
    nx[0] = ((uint32_t)((int32_t)qx - 1) < W) + 1;
    nx[2 * PP - 1] = 1 + ((uint32_t)((int32_t)qx + PP) < W);
#pragma unroll
    for (int co = 0; co < CO; co++) {
      float o[2 * PP];
#pragma unroll
      for (int i = 0; i < 2 * PP; i++) o[i] = acc[i / 2][py][i % 2][co] + bsum * (float)(ny * nx[i]);
#pragma unroll
      for (int i = 0; i < 2 * PP; i++) o[i] = mt::apply_func_epilogue(func, o[i]);  // tanh / sigmoid: hardware exp and reciprocal
      float *dst = args.ep.C + ((size_t)g * M + co) * OHW + (size_t)(2 * qy + py) * OW + 2 * qx;
      if constexpr (PP == 2) *reinterpret_cast<float4 *>(dst) = make_float4(o[0], o[1], o[2], o[3]);
      else *reinterpret_cast<float2 *>(dst) = make_float2(o[0], o[1]);
    }
  }
}

template <int... I, class F>
__device__ __forceinline__ void static_for(std::integer_sequence<int, I...>, F &&f) {
  (f(std::integral_constant<int, I>{}), ...);
}

// The same layer on the matrix cores.  v_mfma_f32_4x4x1_16B_f32 multiplies sixteen independent 4x1 by 1x4 blocks: with
// the four rows as output channels (at most 4: the image layer has 3) and the 64 lanes as 64 input pixels, one
// instruction adds one (channel, tap) term to 4 output channels of 64 pixels -- the same rate as the large matrix
// instructions, 3/4 of it useful.  Lane l supplies the input value of ITS pixel (operand B); operand A, the coefficients,
// uses the instruction's block broadcast: a register holds in lanes 4b..4b+3 the coefficients of the four output
// channels for input channel b of a chunk of 16, and the instruction with broadcast block b takes just those -- one
// register per (phase, tap) carries 16 channels, so the 16 (phase, tap) combinations of a chunk are 16 registers read
// from LDS once per chunk.
//
// A block (4 wavefronts) owns 8 rows x 32 columns of input pixels of one image; a wavefront two rows.  The input patch
// behind the tile (10 x 34 pixels) is staged per chunk of 16 channels in LDS as [pixel][channel], 80 bytes per pixel:
// a lane's 3x3 neighbours are 128-bit reads of four channels each, free of bank conflicts like the operand tiles of
// the large kernels.  Global loads walk the image rows (lanes along x, four channels per thread gathered into one
// 128-bit LDS write); the next chunk's values travel while the current chunk is multiplied (two LDS buffers).  NORM:
// func(scale * x + shift) on the way to LDS, see HaloTile.  The four phases of an output row pair are stored as 8-byte
// pairs (px = 0, 1), whole lines per wavefront.
// Needs W % 32 == 0, C % 16 == 0, at most 4 output channels, coefficients packed [ci][phase][co][taps].
template <bool NORM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void tconv_k4s2_mfma_kernel(TconvArgs args, uint32_t tiles_x, uint32_t tiles_y) {
  constexpr int TR = 8, TC = 32, PR = TR + 2, PC = TC + 2, PS = 20, CH = 16;
  constexpr int PIX = PR * PC, ITEMS = PIX * (CH / 4), NIT = (ITEMS + 255) / 256;
  __shared__ __attribute__((aligned(16))) float patch[2][PIX * PS];
  __shared__ __attribute__((aligned(16))) float coeff[2][64 * 16];  // [lane][phase * 4 + tap]
  const uint32_t H = args.H, W = args.W, C = args.C, HW = H * W, M = args.M;
  const uint32_t tile = blockIdx.x % (tiles_x * tiles_y), g = blockIdx.x / (tiles_x * tiles_y);
  const uint32_t x0 = (tile % tiles_x) * TC, y0 = (tile / tiles_x) * TR;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(args.delta, args.in_w * C * HW * 4u);
  __amdgpu_buffer_rsrc_t prsrc = rsrc;
  if (NORM) prsrc = make_rsrc(args.in_scale_shift, C * HW * 8u);
  const uint32_t image_bytes = (g % args.in_w) * C * HW * 4u;

  // staging items: (pixel of the patch, quad of channels); byte offset of channel 4*quad at that pixel, or out of range
  uint32_t it_off[NIT], it_dst[NIT];
#pragma unroll
  for (int i = 0; i < NIT; i++) {
    const uint32_t id = (uint32_t)tid + i * 256u, quad = id / PIX, pix = id % PIX, yy = pix / PC, xx = pix % PC;
    const int32_t y = (int32_t)(y0 + yy) - 1, x = (int32_t)(x0 + xx) - 1;
    const bool ok = id < ITEMS && (uint32_t)y < H && (uint32_t)x < W;
    it_off[i] = ok ? ((quad * 4u * H + (uint32_t)y) * W + (uint32_t)x) * 4u : OOB;
    it_dst[i] = id < ITEMS ? pix * PS + quad * 4u : 0xffffffffu;
  }
  floatx4 sv[NIT];
  floatx2 sp[NORM ? NIT : 1][4];
  float cw[4];
  const int in_func = args.in_func;
  const float *packed = args.ph[0].packed;
  auto fetch = [&](uint32_t chunk) {
    const uint32_t soff = image_bytes + chunk * CH * HW * 4u;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) sv[i][j] = buf_load(rsrc, it_off[i] == OOB ? OOB : it_off[i] + (uint32_t)j * HW * 4u, soff);
      if constexpr (NORM) {
#pragma unroll
        for (int j = 0; j < 4; j++) sp[i][j] = buf_load2(prsrc, it_off[i] == OOB ? OOB : (it_off[i] + (uint32_t)j * HW * 4u) * 2u, 2u * chunk * CH * HW * 4u);
      }
    }
    // coefficients of the chunk: thread (lane l = 4b + i, four of the 16 combinations) reads packed[ci = chunk*16 + b][phase][co = i][tap]
    const uint32_t l = (uint32_t)tid & 63u, b = l >> 2, co = l & 3u, f = (uint32_t)tid >> 6;
    const float *src = packed + ((size_t)(chunk * CH + b) * 4u + f) * (4u * M) + co * 4u;
#pragma unroll
    for (int t = 0; t < 4; t++) cw[t] = co < M ? src[t] : 0.f;
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NIT; i++)
      if (it_dst[i] != 0xffffffffu) {
        floatx4 v = sv[i];
        if constexpr (NORM) {
#pragma unroll
          for (int j = 0; j < 4; j++) v[j] = mt::apply_func_cheap(in_func, sp[i][j].x * v[j] + sp[i][j].y);
        }
        *reinterpret_cast<floatx4 *>(&patch[buf][it_dst[i]]) = v;
      }
    *reinterpret_cast<floatx4 *>(&coeff[buf][((uint32_t)tid & 63u) * 16u + ((uint32_t)tid >> 6) * 4u]) = floatx4{cw[0], cw[1], cw[2], cw[3]};
  };

  floatx4acc acc[4];
#pragma unroll
  for (int f = 0; f < 4; f++) acc[f] = floatx4acc{0.f, 0.f, 0.f, 0.f};
  const uint32_t rr = (uint32_t)lane >> 5, lx = (uint32_t)lane & 31u;
  const float *centre = &patch[0][((wave * 2 + rr + 1) * PC + lx + 1) * PS];  // the lane's pixel in the patch (buffer 0)
  const uint32_t chunks = C / CH;
  fetch(0);
  put(0);
  __syncthreads();
  for (uint32_t ch = 0; ch < chunks; ch++) {
    const int cur = ch & 1;
    if (ch + 1 < chunks) fetch(ch + 1);
    floatx4 av[4];  // av[f][t]: coefficients of phase f, tap t for the 16 channels of the chunk (this lane's slot)
#pragma unroll
    for (int f = 0; f < 4; f++) av[f] = *reinterpret_cast<const floatx4 *>(&coeff[cur][lane * 16 + f * 4]);
    const float *pc = centre + cur * PIX * PS;
    static_for(std::make_integer_sequence<int, CH / 4>{}, [&](auto qc) {
      constexpr int q = decltype(qc)::value;
      floatx4 xv[3][3];  // four channels of the nine neighbours
#pragma unroll
      for (int dy = 0; dy < 3; dy++)
#pragma unroll
        for (int dx = 0; dx < 3; dx++) xv[dy][dx] = *reinterpret_cast<const floatx4 *>(pc + ((dy - 1) * PC + (dx - 1)) * PS + q * 4);
      static_for(std::make_integer_sequence<int, 4>{}, [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        // channel 4q+j of the chunk (broadcast block 4q+j): tap (ty, tx) of phase (py, px) reads neighbour
        // (py + ty - 1, px + tx - 1); consecutive instructions go to different accumulators
#pragma unroll
        for (int t = 0; t < 4; t++)
#pragma unroll
          for (int f = 0; f < 4; f++) {
            const int py = f >> 1, px = f & 1, ty = t >> 1, tx = t & 1;
            acc[f] = __builtin_amdgcn_mfma_f32_4x4x1f32(av[f][t], xv[py + ty][px + tx][j], acc[f], 4, q * 4 + j, 0);
          }
      });
    });
    if (ch + 1 < chunks) put(cur ^ 1);
    __syncthreads();
  }

  const uint32_t qy = y0 + wave * 2 + rr, qx = x0 + lx;
  if (qy >= H) return;
  const uint32_t OW = 2 * W, OHW = 4 * HW;
  const float bsum = args.ep.tap_bias ? args.ep.tap_bias[g % args.ep.bias_w] : 0.f;
  const int func = args.ep.func;
#pragma unroll
  for (int py = 0; py < 2; py++) {
    const int ny = ((uint32_t)((int32_t)qy + py - 1) < H) + ((uint32_t)((int32_t)qy + py) < H);
    const int nx0 = ((uint32_t)((int32_t)qx - 1) < W) + 1, nx1 = 1 + ((uint32_t)((int32_t)qx + 1) < W);
#pragma unroll
    for (int co = 0; co < 4; co++) {
      if ((uint32_t)co >= M) break;
      float2 o;
      o.x = mt::apply_func_epilogue(func, acc[py * 2][co] + bsum * (float)(ny * nx0));
      o.y = mt::apply_func_epilogue(func, acc[py * 2 + 1][co] + bsum * (float)(ny * nx1));
      *reinterpret_cast<float2 *>(args.ep.C + ((size_t)g * M + co) * OHW + (size_t)(2 * qy + py) * OW + 2 * qx) = o;
    }
  }
}

// The same layer as a product WITHOUT neighbourhoods, then a cheap combination.  A stride-2 transposed convolution
// scatters: input pixel (y, x) adds kernel tap (phase, tap) times its value to one output pixel near (2y, 2x).  So
//   P[(tap of 16, co)][pixel] = sum over ci of coefficient[(tap, co)][ci] * in[ci][pixel]
// is an ordinary product with 16*CO rows, K = C and the raw input pixels as columns -- no patch, no halo, no padding
// rows: with CO = 3 the 48 rows are exactly three 16-row tiles of v_mfma_f32_16x16x4_f32.  Every output pixel is then
// the sum of four P values of neighbouring input pixels.
//
// A block owns one image (W = 32, H <= 32 rows, one wavefront per two rows).  Lane (n, g) of a wavefront supplies, per
// k step of four channels, channel 4s + g of pixels x = 2n, 2n+1 in both rows: two 64-bit loads straight from global
// memory into the matrix operand (the input is read exactly once, in whole lines; no LDS for it), DEPTH k steps ahead
// in a register ring.  The coefficients are re-ordered once per block into LDS as [k step][tile][lane], one 32-bit read
// per tile and k step, from the [ci][phase][co][taps] order of the tile kernel.  NORM: func(scale * x + shift) on the
// operand registers, the pairs fetched beside the values.
//
// Rows of a tile are (a, b) = ((py, ty), (px, tx)): the product of category a lands in output row 2y + {2, 0, 1, -1}[a],
// of category b in output column 2x + {2, 0, 1, -1}[b].  The accumulator layout puts a into the lane group g and b into
// the register index, so the combination along x is four additions per output row piece, two of them with the
// neighbouring lane's value (a DPP shift inside the 16 lanes that hold one image row: what it shifts in at either end is
// the zero beyond the image), and the combination along y goes once through LDS ([row][a][co][64 columns]), from where
// every lane takes the two pieces of its output row, adds the bias term, applies the function and stores 16 bytes of a
// whole output line.
// Needs W == 32, H even and at most 32, C a multiple of 4 * DEPTH, exactly CO output channels, 8-byte aligned input.
//
// STRIP: images of W == 64.  A block owns a strip of R input rows of one image and has R + 2 wavefronts, one per input
// row from the row above the strip to the row below it (the neighbours' pieces are computed again rather than fetched
// from another block; rows outside the image load zeros and contribute zeros).  A wavefront's four pixel groups are the
// two halves of its row (the second half is 128 bytes on, exactly where the next row is for W == 32, so the loads and
// the products are the same instructions); along x the two halves exchange their edge pixels through a DPP rotation of
// the 16 lanes; the first R wavefronts then finish two output rows each, 32 lanes per row.
template <int CO, int NORM, int DEPTH, bool STRIP = false>   // NORM: 0 plain input, 1 ReLU(scale * x + shift), 2 any of the cheap functions
__global__ __launch_bounds__(1024) void tconv_k4s2_products_kernel(TconvArgs args) {
  extern __shared__ __attribute__((aligned(16))) float pieces[];  // [rows][4][CO][2 W], then the coefficients [C/4][CO][64]
  constexpr uint32_t W = STRIP ? 64u : 32u, OW = 2u * W;
  const uint32_t H = args.H, C = args.C, HW = H * W;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t R = STRIP ? blockDim.x / 64u - 2u : H;            // input rows whose output rows the block writes
  const uint32_t strips = STRIP ? H / R : 1u;
  const uint32_t block = STRIP ? xcd_swizzle(blockIdx.x, gridDim.x) : blockIdx.x;   // neighbouring strips share two input rows: one L2 for both
  const uint32_t img = block / strips, y0 = (block % strips) * R;
  const uint32_t n = (uint32_t)lane & 15u, g = (uint32_t)lane >> 4;
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(args.delta, args.in_w * C * HW * 4u);
  __amdgpu_buffer_rsrc_t prsrc = rsrc;
  if (NORM) prsrc = make_rsrc(args.in_scale_shift, C * HW * 8u);
  // value offsets: channel g of the k step, the wavefront's (first) row, pixels 2n, 2n+1; the second pair is 128 bytes on
  const int32_t row = STRIP ? (int32_t)y0 - 1 + wave : 2 * wave;
  const bool row_in = !STRIP || (uint32_t)row < H;
  const uint32_t in_sample = row_in ? ((g * H + (uint32_t)row) * W + 2u * n) * 4u : 0u;
  const uint32_t b_voff = row_in ? (img % args.in_w) * C * HW * 4u + in_sample : OOB, b_step = 4u * HW * 4u;
  const uint32_t steps = C / 4u;
  const int in_func = args.in_func;
  float *coeff = pieces + (STRIP ? R + 2u : H) * 4u * CO * OW;

  floatx2 rb[DEPTH][2];
  floatx4 rp[NORM ? DEPTH : 1][2];
  float rc[2][CO];
  auto fetch = [&](int slot, uint32_t s) {
    const bool live = s < steps && row_in;   // uniform; loads beyond the last step are dropped by the range check
    const uint32_t bo = live ? b_voff : OOB;
#pragma unroll
    for (int yy = 0; yy < 2; yy++) rb[slot][yy] = buf_load2(rsrc, bo == OOB ? OOB : bo + (uint32_t)yy * 128u, s * b_step);
    if constexpr (NORM != 0) {
      const uint32_t po = live ? in_sample * 2u : OOB;
#pragma unroll
      for (int yy = 0; yy < 2; yy++) rp[slot][yy] = buf_load4(prsrc, po == OOB ? OOB : po + (uint32_t)yy * 256u, s * b_step * 2u);
    }
  };

  floatx4acc acc[CO][4];   // [tile = co][pixel group (yy, xx)]
#pragma unroll
  for (int co = 0; co < CO; co++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[co][j] = floatx4acc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int d = 0; d < DEPTH; d++) fetch(d, (uint32_t)d);
  // The coefficients in the order the matrix instruction takes them.  Row i = lane % 16 of a tile is
  // (a, b) = (i / 4, i % 4) = ((py, ty), (px, tx)); lane / 16 is the channel within the k step.
  for (uint32_t idx = (uint32_t)tid; idx < steps * CO * 64u; idx += blockDim.x) {
    const uint32_t l = idx & 63u, co = (idx >> 6) % CO, s = idx / (64u * CO), i = l & 15u;
    const uint32_t f = ((i >> 2) >> 1) * 2u + ((i & 3u) >> 1), t = ((i >> 2) & 1u) * 2u + (i & 1u);
    coeff[idx] = args.ph[0].packed[((4u * s + (l >> 4)) * 16u + f * 4u) * CO + co * 4u + t];
  }
  __syncthreads();
  const float *cget = coeff + lane;
#pragma unroll
  for (int co = 0; co < CO; co++) rc[0][co] = cget[co * 64];
  for (uint32_t s0 = 0; s0 < steps; s0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      {
        const uint32_t sn = s0 + (uint32_t)d + 1u < steps ? s0 + (uint32_t)d + 1u : 0u;   // (the last step reads something it does not use)
#pragma unroll
        for (int co = 0; co < CO; co++) rc[(d + 1) & 1][co] = cget[(sn * CO + co) * 64u];
      }
      __builtin_amdgcn_sched_barrier(0);
      float v[4] = {rb[d][0].x, rb[d][0].y, rb[d][1].x, rb[d][1].y};   // (yy, xx) = 00 01 10 11
      if constexpr (NORM != 0) {
        const float sc[4] = {rp[d][0].x, rp[d][0].z, rp[d][1].x, rp[d][1].z}, sh[4] = {rp[d][0].y, rp[d][0].w, rp[d][1].y, rp[d][1].w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float u = sc[j] * v[j] + sh[j];
          v[j] = NORM == 1 ? (u > 0.f ? u : 0.f) : mt::apply_func_cheap(in_func, u);
        }
      }
#pragma unroll
      for (int j = 0; j < 4; j++)
#pragma unroll
        for (int co = 0; co < CO; co++) acc[co][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(rc[d & 1][co], v[j], acc[co][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      fetch(d, s0 + (uint32_t)d + DEPTH);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- along x: output columns 4n .. 4n+3 of row category a = g, for both input rows and every channel
  auto from_left = [](float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x111, 0xf, 0xf, true)); };   // row_shr:1
  auto from_right = [](float x) { return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x101, 0xf, 0xf, true)); };  // row_shl:1
#pragma unroll
  for (int yy = 0; yy < 2; yy++)
#pragma unroll
    for (int co = 0; co < CO; co++) {
      const floatx4acc &e = acc[co][yy * 2], &o = acc[co][yy * 2 + 1];   // pixels x = 2n and 2n + 1; register = category b
      floatx4 r;
      r.x = e[1] + from_left(o[0]);    // column 4n:     x = 2n as 2x, x = 2n - 1 as 2x + 2
      r.y = e[2] + o[3];               // column 4n + 1: x = 2n as 2x + 1, x = 2n + 1 as 2x - 1
      r.z = o[1] + e[0];               // column 4n + 2: x = 2n + 1 as 2x, x = 2n as 2x + 2
      r.w = o[2] + from_right(e[3]);   // column 4n + 3: x = 2n + 1 as 2x + 1, x = 2n + 2 as 2x - 1
      if constexpr (STRIP) {
        // yy is the half of the row: pixel 31's neighbour to the right is pixel 32, lane 0 of the other half, and the other
        // way round (a rotation of the 16 lanes; lanes without a source in the shift keep that value)
        if (yy == 0) {
          const float edge = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc[co][2][3]), 0x12f, 0xf, 0xf, false));   // row_ror:15: lane 15 <- lane 0
          r.w = o[2] + __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(edge), __float_as_int(e[3]), 0x101, 0xf, 0xf, false));
        } else {
          const float edge = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(acc[co][1][0]), 0x121, 0xf, 0xf, false));   // row_ror:1: lane 0 <- lane 15
          r.x = e[1] + __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(edge), __float_as_int(o[0]), 0x111, 0xf, 0xf, false));
        }
        *reinterpret_cast<floatx4 *>(&pieces[((((uint32_t)wave) * 4u + g) * CO + co) * OW + 64u * (uint32_t)yy + 4u * n]) = r;
      } else {
        *reinterpret_cast<floatx4 *>(&pieces[((((uint32_t)(2 * wave + yy)) * 4u + g) * CO + co) * 64u + 4u * n]) = r;
      }
    }

  __syncthreads();
  if constexpr (STRIP) {
    // ---- along y: wavefront w finishes output rows 2m and 2m + 1 of input row m = y0 + w (local row w + 1), 32 lanes each
    if ((uint32_t)wave >= R) return;
    const uint32_t odd = (uint32_t)lane >> 5, q = (uint32_t)lane & 31u, m = y0 + (uint32_t)wave, local = (uint32_t)wave + 1u;
    const uint32_t a_own = odd ? 2u : 1u, a_other = odd ? 3u : 0u, local_other = odd ? local + 1u : local - 1u;
    const bool other = (uint32_t)((int32_t)m + (odd ? 1 : -1)) < H;   // (a row outside the image holds zeros: only the bias count differs)
    const uint32_t OHW = 4u * HW, oy = 2u * m + odd;
    const float bsum = args.ep.tap_bias ? args.ep.tap_bias[img % args.ep.bias_w] : 0.f;
    const float ny = other ? 2.f : 1.f;
    const float nx[4] = {q == 0 ? 1.f : 2.f, 2.f, 2.f, q == 31 ? 1.f : 2.f};
    float o[CO][4];
#pragma unroll
    for (int co = 0; co < CO; co++) {
      floatx4 r = *reinterpret_cast<const floatx4 *>(&pieces[((local * 4u + a_own) * CO + co) * OW + 4u * q]);
      const floatx4 t = *reinterpret_cast<const floatx4 *>(&pieces[((local_other * 4u + a_other) * CO + co) * OW + 4u * q]);
#pragma unroll
      for (int i = 0; i < 4; i++) o[co][i] = (r[i] + t[i]) + bsum * (ny * nx[i]);
    }
    mt::apply_func_epilogue_many<4 * CO>(args.ep.func, &o[0][0]);
#pragma unroll
    for (int co = 0; co < CO; co++)
      *reinterpret_cast<float4 *>(args.ep.C + ((size_t)img * CO + co) * OHW + (size_t)oy * OW + 4u * q) = make_float4(o[co][0], o[co][1], o[co][2], o[co][3]);
    return;
  }

  // ---- along y: output row 2m is input row m in category 1 plus row m - 1 in category 0; output row 2m + 1 is row m in
  // category 2 plus row m + 1 in category 3.  The lane takes row 4*wave + g, columns 4n .. 4n+3, every channel.
  const uint32_t oy = 4u * (uint32_t)wave + g, m = oy >> 1, odd = oy & 1u;
  const uint32_t a_own = odd ? 2u : 1u, a_other = odd ? 3u : 0u;
  const int32_t y_other = odd ? (int32_t)m + 1 : (int32_t)m - 1;
  const bool other = (uint32_t)y_other < H;
  const uint32_t OHW = 4u * HW;
  const float bsum = args.ep.tap_bias ? args.ep.tap_bias[img % args.ep.bias_w] : 0.f;
  const float ny = other ? 2.f : 1.f;
  // contributing input columns of an output column: two, one at the image's left and right edge
  const float nx[4] = {n == 0 ? 1.f : 2.f, 2.f, 2.f, n == 15 ? 1.f : 2.f};
  float o[CO][4];
#pragma unroll
  for (int co = 0; co < CO; co++) {
    floatx4 r = *reinterpret_cast<const floatx4 *>(&pieces[((m * 4u + a_own) * CO + co) * 64u + 4u * n]);
    if (other) {
      const floatx4 q = *reinterpret_cast<const floatx4 *>(&pieces[(((uint32_t)y_other * 4u + a_other) * CO + co) * 64u + 4u * n]);
      r.x = r.x + q.x; r.y = r.y + q.y; r.z = r.z + q.z; r.w = r.w + q.w;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) o[co][i] = r[i] + bsum * (ny * nx[i]);
  }
  mt::apply_func_epilogue_many<4 * CO>(args.ep.func, &o[0][0]);
#pragma unroll
  for (int co = 0; co < CO; co++)
    *reinterpret_cast<float4 *>(args.ep.C + ((size_t)img * CO + co) * OHW + (size_t)oy * 64u + 4u * n) = make_float4(o[co][0], o[co][1], o[co][2], o[co][3]);
}

// Forward convolution 3x3, stride 1, padding 1 with at most 4 output channels (an image-producing last layer) on the
// vector ALUs, same staging: a thread computes two neighbouring output pixels for all KA channels, per input channel
// 6 LDS reads and 18*KA multiply-adds; the 9 coefficients of (k, c) are contiguous in the kernel tensor and come
// through the scalar cache.  Needs W % 4 == 0, C % 8 == 0, 16-byte aligned rows.
// CC channels per chunk: 8, or 4 for images of few channels (more chunks to overlap loading with, and half the LDS,
// so that more blocks share a compute unit).
template <int KA, int CC>
__global__ __launch_bounds__(256) void conv3x3_tile_kernel(float *out, const float *image, const float *kernel, const float *bias, ConvGeo g, int func) {
  using Tile = HaloTile<32, 16, CC>;
  constexpr int TW = 32, TH = 16, PITCH = Tile::PITCH, ROWS = Tile::ROWS;
  __shared__ __attribute__((aligned(16))) float tile[2][CC][ROWS][PITCH];
  const uint32_t H = g.H, W = g.W, C = g.C, HW = H * W;
  const uint32_t tiles_x = (W + TW - 1) / TW;
  // Neighbouring tiles read each other's edge columns and rows: an XCD (its own L2) takes a contiguous range of
  // (image, tile) instead of every eighth block, so that those lines are fetched once (2.8 times the input was read
  // from the fabric before, 5.9 TB/s of it: the kernel was bound by its own re-reads).
  const uint32_t logical = mt::igemm::xcd_swizzle(blockIdx.y * gridDim.x + blockIdx.x, gridDim.x * gridDim.y);
  const uint32_t tile_id = logical % gridDim.x, w = logical / gridDim.x;
  const uint32_t x0 = (tile_id % tiles_x) * TW, y0 = (tile_id / tiles_x) * TH;
  const uint32_t tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  Tile stage;
  stage.setup(image, g.in_w * C * HW * 4u, (w % g.in_w) * C * HW * 4u, H, W, x0, y0, tid);
  float acc[2][KA];
#pragma unroll
  for (int k = 0; k < KA; k++) acc[0][k] = acc[1][k] = bias[(size_t)(w % g.bias_w) * KA + k];
  const uint32_t chunks = C / CC;
  stage.fetch(0);
  stage.put(&tile[0][0][0][0]);
  __syncthreads();
  for (uint32_t ch = 0; ch < chunks; ch++) {
    const int cur = ch & 1;
    if (ch + 1 < chunks) stage.fetch(ch + 1);
#pragma unroll 2
    for (int c = 0; c < CC; c++) {
      const uint32_t ci = ch * CC + c;
      float v[3][4];  // rows y-1..y+1, columns x-1..x+2 of the pixel pair (x, x+1)
#pragma unroll
      for (int dy = 0; dy < 3; dy++) {
        const float *rowp = &tile[cur][c][ty + dy][2 * tx];
        const float2 lo = *reinterpret_cast<const float2 *>(rowp), hi = *reinterpret_cast<const float2 *>(rowp + 2);
        v[dy][0] = lo.x; v[dy][1] = lo.y; v[dy][2] = hi.x; v[dy][3] = hi.y;
      }
#pragma unroll
      for (int k = 0; k < KA; k++) {
        const float *wk = kernel + (size_t)k * g.ker_ld + ci * 9u;
#pragma unroll
        for (int dy = 0; dy < 3; dy++)
#pragma unroll
          for (int dx = 0; dx < 3; dx++) {
            const float wv = wk[dy * 3 + dx];
            acc[0][k] = __builtin_fmaf(wv, v[dy][dx], acc[0][k]);
            acc[1][k] = __builtin_fmaf(wv, v[dy][dx + 1], acc[1][k]);
          }
      }
    }
    if (ch + 1 < chunks) stage.put(&tile[cur ^ 1][0][0][0]);
    __syncthreads();
  }
  const uint32_t y = y0 + ty, x = x0 + 2 * tx;
  if (y >= H || x >= W) return;  // W is even: a pair is inside or outside as a whole
#pragma unroll
  for (int k = 0; k < KA; k++) {
    float2 o;
    o.x = mt::apply_func_epilogue(func, acc[0][k]);
    o.y = mt::apply_func_epilogue(func, acc[1][k]);
    *reinterpret_cast<float2 *>(out + ((size_t)w * KA + k) * HW + (size_t)y * W + x) = o;
  }
}

// kernel 4x4, stride 2, padding 1, at most 4 output channels, and the shape the tile kernel is written for
bool tile_kernel_fits(const mt_tensor *out, const mt_tensor *delta, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, int32_t sx, int32_t sy, int32_t px,
                      int32_t py) {
  return kz <= 4 && kx == 4 && ky == 4 && sx == 2 && sy == 2 && px == 1 && py == 1 && out->y == 2 * delta->y && out->x == 2 * delta->x &&
         delta->x % 4 == 0 && ka % 8 == 0 && ka >= 16 && ((uintptr_t)out->p & 15u) == 0 && ((uintptr_t)delta->p & 15u) == 0 && out->w <= 65535u;
}
template <bool NORM>
int launch_tconv_tile_norm(const char *name, TconvArgs &args) {
  mt::ProfileScope prof(mt::profiling() ? mt::intern_label(name, "vector ALU, few output channels") : name);
  dim3 gt(cdiv(args.W, 32) * cdiv(args.H, 16), args.out_w);
  if ((size_t)gt.x * gt.y < 512) {  // fewer than two blocks per compute unit: one pixel per thread, twice the blocks
    dim3 g1(cdiv(args.W, 16) * cdiv(args.H, 16), args.out_w);
    if (args.M == 1) tconv_k4s2_tile_kernel<1, 1, 1, NORM><<<g1, 256, 0, mt::stream()>>>(args);
    else if (args.M == 2) tconv_k4s2_tile_kernel<2, 1, 1, NORM><<<g1, 256, 0, mt::stream()>>>(args);
    else if (args.M == 3) tconv_k4s2_tile_kernel<3, 1, 1, NORM><<<g1, 256, 0, mt::stream()>>>(args);
    else tconv_k4s2_tile_kernel<4, 1, 1, NORM><<<g1, 256, 0, mt::stream()>>>(args);
  } else if ((size_t)gt.x * gt.y < 1024 && args.C % 16 == 0) {  // two to four blocks per compute unit: the channels split over two halves of a block
    if (args.M == 1) tconv_k4s2_tile_kernel<1, 2, 2, NORM><<<gt, 512, 0, mt::stream()>>>(args);
    else if (args.M == 2) tconv_k4s2_tile_kernel<2, 2, 2, NORM><<<gt, 512, 0, mt::stream()>>>(args);
    else if (args.M == 3) tconv_k4s2_tile_kernel<3, 2, 2, NORM><<<gt, 512, 0, mt::stream()>>>(args);
    else tconv_k4s2_tile_kernel<4, 2, 2, NORM><<<gt, 512, 0, mt::stream()>>>(args);
  } else if (args.M == 1) tconv_k4s2_tile_kernel<1, 2, 1, NORM><<<gt, 256, 0, mt::stream()>>>(args);
  else if (args.M == 2) tconv_k4s2_tile_kernel<2, 2, 1, NORM><<<gt, 256, 0, mt::stream()>>>(args);
  else if (args.M == 3) tconv_k4s2_tile_kernel<3, 2, 1, NORM><<<gt, 256, 0, mt::stream()>>>(args);
  else tconv_k4s2_tile_kernel<4, 2, 1, NORM><<<gt, 256, 0, mt::stream()>>>(args);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}
// Which kernel runs the image layer: 0 the vector ALUs; 1 the 4x4x1 matrix instruction where the shape allows (measured
// on an MI355X for [256,64,32,32] -> [256,3,64,64]: 35.0 us against 35.3 us, with the normalising loader 47.8 against
// 40.3 us: kept selectable and tested); 2 (default) products per input pixel on the 16x16x4 matrix instruction where the
// shape allows (22.7 us, 25.1 us with the normalising loader), the vector ALUs elsewhere.
int g_image_mfma = 2;
template <int CO, int NORM>
int launch_tconv_products(const char *name, const TconvArgs &args) {
  constexpr int DEPTH = NORM == 2 || (CO == 4 && NORM != 0) ? 2 : 4;   // k steps in flight: what 128 registers hold beside the accumulators
  static bool prepared = false;
  const size_t lds = ((size_t)args.H * 4u * CO * 64u + (size_t)args.C / 4u * CO * 64u) * sizeof(float);   // the pieces, then the coefficients
  if (!prepared) {
    MT_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&tconv_k4s2_products_kernel<CO, NORM, DEPTH>), hipFuncAttributeMaxDynamicSharedMemorySize,
                               160 * 1024));
    prepared = true;
  }
  tconv_k4s2_products_kernel<CO, NORM, DEPTH><<<args.out_w, args.H * 32u, lds, mt::stream()>>>(args);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}
// Rows per strip of the same kernel for images of 64 columns: 8 (two blocks of ten wavefronts per compute unit), else 4
int g_image_strip = 0;   // 0: choose; else rows per strip (measurements only; must divide the image height)
uint32_t products_strip_rows(const TconvArgs &args) {
  if (g_image_strip > 0 && args.H % (uint32_t)g_image_strip == 0) return (uint32_t)g_image_strip;
  return args.H % 8 == 0 ? 8u : 4u;
}
template <int CO, int NORM>
int launch_tconv_products_strip(const char *name, const TconvArgs &args) {
  constexpr int DEPTH = NORM == 2 || (CO == 4 && NORM != 0) ? 2 : 4;
  static bool prepared = false;
  const uint32_t rows = products_strip_rows(args);
  const size_t lds = ((size_t)(rows + 2u) * 4u * CO * 128u + (size_t)args.C / 4u * CO * 64u) * sizeof(float);
  if (!prepared) {
    MT_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&tconv_k4s2_products_kernel<CO, NORM, DEPTH, true>), hipFuncAttributeMaxDynamicSharedMemorySize,
                               160 * 1024));
    prepared = true;
  }
  tconv_k4s2_products_kernel<CO, NORM, DEPTH, true><<<args.out_w * (args.H / rows), (rows + 2u) * 64u, lds, mt::stream()>>>(args);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}
template <int CO>
int launch_tconv_products_norm(const char *name, const TconvArgs &args) {
  if (args.W == 64) {
    if (!args.in_scale_shift) return launch_tconv_products_strip<CO, 0>(name, args);
    return args.in_func == MT_F_RELU ? launch_tconv_products_strip<CO, 1>(name, args) : launch_tconv_products_strip<CO, 2>(name, args);
  }
  if (!args.in_scale_shift) return launch_tconv_products<CO, 0>(name, args);
  return args.in_func == MT_F_RELU ? launch_tconv_products<CO, 1>(name, args) : launch_tconv_products<CO, 2>(name, args);
}
bool products_kernel_fits(const TconvArgs &args) {
  if (args.C % 16 != 0 || args.M < 1 || args.M > 4) return false;
  if (args.W == 64) {  // strips of rows, one wavefront per input row
    const uint32_t rows = products_strip_rows(args);
    return args.H % 4 == 0 && args.H >= 4 && (uint64_t)args.out_w * (args.H / rows) <= 0x7fffffffu &&
           ((size_t)(rows + 2u) * 4u * 128u + args.C / 4u * 64u) * args.M * sizeof(float) <= 160u * 1024u;
  }
  // (the pieces of the output rows and the coefficients share the 160 KB of LDS)
  return args.W == 32 && args.H % 2 == 0 && args.H >= 2 && args.H <= 32 && args.out_w <= 0x7fffffffu &&
         ((size_t)args.H * 4u + args.C / 4u) * args.M * 64u * sizeof(float) <= 160u * 1024u;
}
int launch_tconv_tile(const char *name, TconvArgs &args) {
  if (g_image_mfma == 2 && products_kernel_fits(args)) {
    mt::ProfileScope prof(mt::profiling() ? mt::intern_label(name, "products per input pixel on 16x16x4, few output channels") : name);
    switch (args.M) {
      case 1: return launch_tconv_products_norm<1>(name, args);
      case 2: return launch_tconv_products_norm<2>(name, args);
      case 3: return launch_tconv_products_norm<3>(name, args);
      default: return launch_tconv_products_norm<4>(name, args);
    }
  }
  if (g_image_mfma == 1 && args.W % 32 == 0 && args.C % 16 == 0 && args.M <= 4) {
    mt::ProfileScope prof(mt::profiling() ? mt::intern_label(name, "4x4x1 matrix instructions, few output channels") : name);
    const uint32_t tiles_x = args.W / 32, tiles_y = cdiv(args.H, 8);
    const size_t blocks = (size_t)tiles_x * tiles_y * args.out_w;
    if (blocks <= 0x7fffffffu) {
      if (args.in_scale_shift) tconv_k4s2_mfma_kernel<true><<<(uint32_t)blocks, 256, 0, mt::stream()>>>(args, tiles_x, tiles_y);
      else tconv_k4s2_mfma_kernel<false><<<(uint32_t)blocks, 256, 0, mt::stream()>>>(args, tiles_x, tiles_y);
      MT_LAUNCH_CHECK(name);
      return MT_OK;
    }
  }
  return args.in_scale_shift ? launch_tconv_tile_norm<true>(name, args) : launch_tconv_tile_norm<false>(name, args);
}

int launch_tconv_small(const char *name, TconvArgs &args, uint32_t max_n) {
  mt::ProfileScope prof(mt::profiling() ? mt::intern_label(name, "vector ALU, few output channels") : name);
  dim3 grid(cdiv(max_n, 256), args.nphase);
  bool t22 = true, small = true;
  for (uint32_t f = 0; f < args.nphase; f++) {
    t22 = t22 && args.ph[f].taps_y == 2 && args.ph[f].taps_x == 2;
    small = small && args.ph[f].taps_y <= 4 && args.ph[f].taps_x <= 4;
  }
  if (!small) return -1;  // caller falls back to the matrix-core path
  // kernel 4x4, stride 2, padding 1 with the natural output size: four 2x2-tap phases with offsets -1 / 0
  bool k4s2 = t22 && args.nphase == 4 && args.ep.sy == 2 && args.ep.sx == 2 && args.ep.OW == 2 * args.W && args.ep.row_stride == 4 * args.H * args.W &&
              ((uintptr_t)args.ep.C & 7u) == 0;
  for (uint32_t f = 0; k4s2 && f < 4; f++)
    k4s2 = args.ph[f].py == f / 2 && args.ph[f].px == f % 2 && args.ph[f].offy == (int32_t)(f / 2) - 1 && args.ph[f].offx == (int32_t)(f % 2) - 1 &&
           args.ph[f].qh == args.H && args.ph[f].qw == args.W;
  if (k4s2) {
    dim3 g4(cdiv((size_t)args.out_w * args.H * args.W, 64));
    if (args.M <= 1) tconv_k4s2_small_kernel<1><<<g4, 256, 0, mt::stream()>>>(args);
    else if (args.M <= 2) tconv_k4s2_small_kernel<2><<<g4, 256, 0, mt::stream()>>>(args);
    else if (args.M == 3) tconv_k4s2_small_kernel<3><<<g4, 256, 0, mt::stream()>>>(args);
    else tconv_k4s2_small_kernel<4><<<g4, 256, 0, mt::stream()>>>(args);
    MT_LAUNCH_CHECK(name);
    return MT_OK;
  }
  // kernel 5x5, stride 2, padding 2 with the natural output size: phases of 3-py by 3-px taps with offsets py-1, px-1
  bool k5s2 = args.nphase == 4 && args.ep.sy == 2 && args.ep.sx == 2 && args.ep.OW == 2 * args.W && args.ep.row_stride == 4 * args.H * args.W &&
              ((uintptr_t)args.ep.C & 7u) == 0 && mt::fits_buffer((size_t)args.in_w * args.C * args.H * args.W);
  for (uint32_t f = 0; k5s2 && f < 4; f++)
    k5s2 = args.ph[f].py == f / 2 && args.ph[f].px == f % 2 && args.ph[f].offy == (int32_t)(f / 2) - 1 && args.ph[f].offx == (int32_t)(f % 2) - 1 &&
           args.ph[f].taps_y == 3 - (int32_t)(f / 2) && args.ph[f].taps_x == 3 - (int32_t)(f % 2) && args.ph[f].qh == args.H && args.ph[f].qw == args.W;
  if (k5s2) {
    dim3 g5(cdiv((size_t)args.out_w * args.H * args.W, 64));
    if (args.M <= 1) tconv_k5s2_small_kernel<1><<<g5, 256, 0, mt::stream()>>>(args);
    else if (args.M <= 2) tconv_k5s2_small_kernel<2><<<g5, 256, 0, mt::stream()>>>(args);
    else if (args.M == 3) tconv_k5s2_small_kernel<3><<<g5, 256, 0, mt::stream()>>>(args);
    else tconv_k5s2_small_kernel<4><<<g5, 256, 0, mt::stream()>>>(args);
    MT_LAUNCH_CHECK(name);
    return MT_OK;
  }
  if (t22) {
    if (args.M <= 2) tconv_small_kernel<2, 2, 2><<<grid, 256, 0, mt::stream()>>>(args);
    else tconv_small_kernel<4, 2, 2><<<grid, 256, 0, mt::stream()>>>(args);
  } else {
    if (args.M <= 2) tconv_small_kernel<2, 0, 0><<<grid, 256, 0, mt::stream()>>>(args);
    else tconv_small_kernel<4, 0, 0><<<grid, 256, 0, mt::stream()>>>(args);
  }
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

// Weights of a forward convolution re-ordered tap-major for SrcIm2colTap: packed[m][t*C + c] = kernel[m][c*taps + t]
__global__ __launch_bounds__(256) void conv_pack_tap_major_kernel(float *packed, const float *kernel, uint32_t ker_ld, uint32_t KA, uint32_t C, uint32_t taps) {
  const uint32_t K = C * taps;
  const size_t total = (size_t)KA * K;
  for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
    const uint32_t m = (uint32_t)(idx / K), k = (uint32_t)(idx % K), t = k / C, c = k % C;
    packed[idx] = kernel[(size_t)m * ker_ld + c * taps + t];
  }
}

// ---- argument checks shared by the plain and the fused entry points ---------------------------------------------
int check_forward(const char *name, const mt_tensor *out, const mt_tensor *image, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz,
                  uint32_t ka, const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  if (mt::bad(out) || mt::bad(image) || mt::bad(kernel) || mt::bad(bias)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(out);
  if (ka == 0) return mt::fail(MT_E_NO_KERNELS, "%s: at least one kernel is required", name);
  if (ka != bias->z) return mt::fail(MT_E_BIAS_COUNT, "%s: kernel_amount %u but %u biases", name, ka, bias->z);
  if (kx <= 0 || ky <= 0 || sx <= 0 || sy <= 0 || px < 0 || py < 0) return mt::fail(MT_E_ARGUMENT, "%s: kernel and stride must be positive, padding non-negative", name);
  int32_t ox = ((int32_t)image->x - kx + 2 * px) / sx + 1, oy = ((int32_t)image->y - ky + 2 * py) / sy + 1;
  if ((int32_t)out->x != ox || (int32_t)out->y != oy || out->z != ka) return mt::fail(MT_E_OUTPUT_SHAPE, "%s: output must be [W,%u,%d,%d]", name, ka, oy, ox);
  if ((int32_t)image->z != kz) return mt::fail(MT_E_DEPTH, "%s: image depth %u but kernel depth %d", name, image->z, kz);
  return MT_OK;
}

int check_kernel_tensor(const char *name, const mt_tensor *kernel, uint32_t rows, uint32_t cols) {
  if (kernel->w == 0 || kernel->z == 0 || kernel->y < rows || kernel->x < cols)
    return mt::fail(MT_E_ARGUMENT, "%s: kernel tensor [%u,%u,%u,%u] is smaller than [1,1,%u,%u]", name, kernel->w, kernel->z, kernel->y, kernel->x, rows, cols);
  return MT_OK;
}

int forward(const char *name, const mt_tensor *out, const mt_tensor *image, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz, uint32_t ka,
            const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func) {
  int rc = check_forward(name, out, image, kernel, kx, ky, kz, ka, bias, sx, sy, px, py);
  if (rc) return rc;
  if (mt::count(out) == 0) return MT_OK;
  if (image->w == 0 || bias->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  uint32_t K = (uint32_t)kz * kx * ky;
  if ((rc = check_kernel_tensor(name, kernel, ka, K))) return rc;
  ConvGeo g{out->w, image->w, kernel->w, bias->w, kz, (int32_t)image->y, (int32_t)image->x, (int32_t)ka, ky, kx, sy, sx, py, px,
            (int32_t)out->y, (int32_t)out->x, (int32_t)ka, kernel->x, kernel->z * kernel->y};
  bool direct = g_conv_path == 1;
  const size_t image_sample = (size_t)kz * image->y * image->x;
  if (!direct && kernel->w == 1 && !mt::fits_buffer(image)) {
    // the folded batch is addressed through one 32-bit descriptor: run it in parts of less than 2 GiB of input
    if (image->w == out->w && bias->w == 1 && mt::fits_buffer(image_sample)) {
      const uint32_t part = (uint32_t)((0x80000000ull / 4 - 1) / image_sample);
      const size_t out_sample = (size_t)ka * out->y * out->x;
      for (uint32_t w0 = 0; w0 < out->w; w0 += part) {
        const uint32_t n = out->w - w0 < part ? out->w - w0 : part;
        mt_tensor o{out->p + w0 * out_sample, n, out->z, out->y, out->x}, im{image->p + w0 * image_sample, n, image->z, image->y, image->x};
        if ((rc = forward(name, &o, &im, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func))) return rc;
      }
      return MT_OK;
    }
    direct = true;
  }
  if (!direct && kernel->w != 1 && !mt::fits_buffer(image_sample)) direct = true;
  if (direct) {
    size_t total = mt::count(out);
    mt::ProfileScope prof("fwd_direct");
    fwd_direct_kernel<<<cdiv(total, 256), 256, 0, mt::stream()>>>(out->p, image->p, kernel->p, bias->p, g, total);
    MT_LAUNCH_CHECK(name);
    if (func != MT_F_NONE) return mt_apply_func(out, out, func);
    return MT_OK;
  }
  if (ka <= 4 && kernel->w == 1 && mt::igemm::tile_override() < 0 && kx == 3 && ky == 3 && sx == 1 && sy == 1 && px == 1 && py == 1 &&
      image->x % 4 == 0 && kz % 8 == 0 && ((uintptr_t)image->p & 15u) == 0 && ((uintptr_t)out->p & 7u) == 0 && out->w <= 65535u) {
    mt::ProfileScope prof(mt::profiling() ? mt::intern_label(name, "vector ALU, few output channels") : name);
    dim3 grid(cdiv(image->x, 32) * cdiv(image->y, 16), out->w);
#define MT_CONV3X3_TILE(KA)                                                                                                   \
  do {                                                                                                                        \
    if (kz <= 32) conv3x3_tile_kernel<KA, 4><<<grid, 256, 0, mt::stream()>>>(out->p, image->p, kernel->p, bias->p, g, func);  \
    else conv3x3_tile_kernel<KA, 8><<<grid, 256, 0, mt::stream()>>>(out->p, image->p, kernel->p, bias->p, g, func);           \
  } while (0)
    if (ka == 1) MT_CONV3X3_TILE(1);
    else if (ka == 2) MT_CONV3X3_TILE(2);
    else if (ka == 3) MT_CONV3X3_TILE(3);
    else MT_CONV3X3_TILE(4);
#undef MT_CONV3X3_TILE
    MT_LAUNCH_CHECK(name);
    return MT_OK;
  }
  uint32_t OHW = out->y * out->x;
  // an image of three channels (a first layer): input patch in LDS, weights in registers, 128-bit stores (mt_firstlayer.h)
  if (g_first_layer && kz == 3 && kernel->w == 1 && bias->w == 1 && image->w == out->w && mt::igemm::tile_override() < 0 && sx == sy && px >= 0 && py >= 0 &&
      mt::fits_buffer(image)) {
    FirstLayerArgs fl{};
    fl.image = image->p; fl.kernel = kernel->p; fl.bias = bias->p; fl.out = out->p;
    fl.ld = kernel->x; fl.KA = ka; fl.H = image->y; fl.W = image->x; fl.OH = out->y; fl.OW = out->x; fl.batch = out->w;
    fl.pad_y = py; fl.pad_x = px;
    fl.func = mt::epilogue_func(func) ? func : MT_F_NONE;
    char tag[96];
    snprintf(tag, sizeof tag, "input patch M%u N%u K%u x1", ka, out->w * OHW, K);
    mt::ProfileScope prof(mt::profiling() ? mt::intern_label(name, tag) : name);
    if (first_layer_launch(name, fl, kz, ky, kx, sx, &rc)) {
      if (rc) return rc;
      return mt::epilogue_func(func) ? MT_OK : mt_apply_func(out, out, func);
    }
  }
  // 3 x 3, stride 1, padding 1 from at most 32 channels on large images: the nine taps share one patch of the image in LDS,
  // the weights live in registers (mt_convpatch.h)
  if (g_conv_patch && kx == 3 && ky == 3 && sx == 1 && sy == 1 && px == 1 && py == 1 && kernel->w == 1 && bias->w == 1 && image->w == out->w &&
      mt::igemm::tile_override() < 0 && kz <= 32 && ka >= (uint32_t)g_conv_patch_min && ka <= 64 && (kz <= 16 || ka <= 16) && image->y == out->y &&
      image->x == out->x) {   // (32 channels to 32 or 64 filters: the general kernel is as fast or faster, 322 against 364 us at 192 x 256, batch 32)
    mt::igemm::TconvPatchArgs cp{};
    cp.delta = image->p; cp.kernel = kernel->p; cp.bias = bias->p; cp.out = out->p;
    cp.B = out->w; cp.F = (uint32_t)kz; cp.C = ka; cp.H = out->y; cp.W = out->x; cp.ld = kernel->x;
    cp.func = mt::epilogue_func(func) ? func : MT_F_NONE;
    if (mt::igemm::tconv_patch_plan(cp)) {
      {
        mt::ProfileScope prof(mt::profiling() ? shape_label(name, T16x256, ka, out->w * OHW, K, 1) : name);
        if ((rc = mt::igemm::launch_conv_patch(name, cp))) return rc;
      }
      g_conv_patch_launches++;
      return mt::epilogue_func(func) ? MT_OK : mt_apply_func(out, out, func);
    }
  }
  // Taps that tile the k step (4x4, 2x2, 1x1 kernels), one kernel and bias set, whole 64-channel row tiles: the kernel whose
  // blocks walk over the batch runs it (see mt_walk.h) when that gives at least two blocks per compute unit; products
  // with fewer tiles and a long k axis are better cut over k (launch_split below).
  if (g_conv_walk && kernel->w == 1 && bias->w == 1 && image->w == out->w && mt::igemm::tile_override() < 0 && BK % ((uint32_t)ky * kx) == 0 &&
      ((uintptr_t)kernel->p & 15u) == 0 && mt::fits_buffer(out)) {
    WalkArgs walk{};
    walk.nphase = 1;
    walk.ph[0] = TconvPhase{kernel->p, K, kernel->x, out->y, out->x, ky, kx, -py, -px, 0u, 0u};
    walk.M = ka; walk.batch = out->w;
    walk.delta = image->p; walk.C = (uint32_t)kz; walk.H = image->y; walk.W = image->x;
    walk.in_sy = (uint32_t)sy; walk.in_sx = (uint32_t)sx;
    walk.out = out->p; walk.OW = out->x; walk.OHW = OHW; walk.sy = 1; walk.sx = 1;
    walk.row_bias = bias->p; walk.tap_bias = nullptr;
    walk.func = mt::epilogue_func(func) ? func : MT_F_NONE;
    if (tconv_walk_plan(walk, (uint32_t)mt::igemm::walk_blocks(), 1) && ((size_t)walk.tiles_m * walk.qtiles * walk.groups >= 512 || g_conv_walk == 2)) {
      {
        mt::ProfileScope prof(mt::profiling() ? shape_label(name, T64x64, ka, out->w * OHW, K, 1) : name);
        if ((rc = launch_tconv_walk(name, walk, false, false, 1))) return rc;
      }
      return mt::epilogue_func(func) ? MT_OK : mt_apply_func(out, out, func);
    }
  }
  SrcIm2col b{};
  b.p = image->p; b.in_w = image->w; b.C = kz; b.H = image->y; b.W = image->x; b.KY = ky; b.KX = kx; b.OHW = OHW; b.OW = out->x; b.K = K;
  b.sy = sy; b.sx = sx; b.py = py; b.px = px;
  Epilogue ep{};
  ep.C = out->p; ep.row_stride = OHW; ep.inner = OHW; ep.g_stride = (size_t)ka * OHW;
  ep.bias = bias->p; ep.bias_mode = 1; ep.bias_w = bias->w; ep.bias_stride = ka;
  const bool func_later = !mt::epilogue_func(func);
  ep.func = func_later ? MT_F_NONE : func;
  if (kernel->w == 1) {  // one kernel set for the whole batch: fold the batch into the columns
    b.R = out->w * OHW;
    const uint32_t taps = (uint32_t)ky * kx, N = out->w * OHW;
    const size_t out_floats = mt::count(out);
    // one product, split over k when it has few output tiles (needs one bias set: the partial sums are added flat)
    auto run = [&](auto a, auto src) {
      if (bias->w == 1) return launch_split(name, a, src, ep, ka, N, K, out_floats, OHW, ka);
      return launch(name, a, src, ep, ka, N, K, 1);
    };
    if (BK % taps == 0 && (uint32_t)kz % (BK / taps) == 0) {  // taps tile the k step: offsets precomputed per thread
      SrcIm2colFixed bf{};
      bf.p = b.p; bf.in_w = b.in_w; bf.C = b.C; bf.H = b.H; bf.W = b.W; bf.KY = b.KY; bf.KX = b.KX; bf.OHW = b.OHW; bf.OW = b.OW; bf.R = b.R; bf.K = b.K;
      bf.sy = sy; bf.sx = sx; bf.py = py; bf.px = px;
      rc = with_row_k(kernel->p, kernel->x, ka, K, Batch{}, [&](auto a) { return run(a, bf); });
    } else if ((uint32_t)kz % BK == 0 && ka >= 16) {
      // k ordered tap-major, 16 channels of one tap per k step; the weights are re-ordered to match (one small launch)
      float *packed = nullptr;
      bool fresh = true;
      if ((rc = pack_buffer(pack_key(1, kernel, nullptr, {kx, ky, kz, (int32_t)ka}), (size_t)ka * K, &packed, &fresh))) return rc;
      if (fresh) {
        mt::ProfileScope prof("conv_pack_tap_major");
        unsigned gx = cdiv((size_t)ka * K, 256 * 4);
        conv_pack_tap_major_kernel<<<gx > 2048 ? 2048 : gx, 256, 0, mt::stream()>>>(packed, kernel->p, kernel->x, ka, (uint32_t)kz, taps);
        MT_LAUNCH_CHECK("conv_pack_tap_major");
      }
      SrcIm2colTap bt{};
      bt.p = b.p; bt.in_w = b.in_w; bt.C = b.C; bt.H = b.H; bt.W = b.W; bt.KY = b.KY; bt.KX = b.KX; bt.OHW = b.OHW; bt.OW = b.OW; bt.R = b.R; bt.K = b.K;
      bt.sy = sy; bt.sx = sx; bt.py = py; bt.px = px;
      rc = with_row_k(packed, K, ka, K, Batch{}, [&](auto a) { return run(a, bt); });
    } else {
      rc = with_row_k(kernel->p, kernel->x, ka, K, Batch{}, [&](auto a) { return run(a, b); });
    }
  } else {
    // kernels differ per sample: one product per output image
    Batch abt;
    abt.wmod = kernel->w; abt.stride = (size_t)kernel->z * kernel->y * kernel->x;
    b.bt.wmod = image->w; b.bt.stride = (size_t)kz * image->y * image->x; b.in_w = 1; b.R = OHW;
    ep.bt.wmod = out->w; ep.bt.stride = (size_t)ka * OHW;
    rc = with_row_k(kernel->p, kernel->x, ka, K, abt, [&](auto a) { return launch(name, a, b, ep, ka, OHW, K, out->w); });
  }
  return rc == MT_OK && func_later ? mt_apply_func(out, out, func) : rc;
}

// What a transposed convolution can take over from the batch-norm layers around it (see mt_walk.h).
struct NormIn {   // the input tensor stands for func(scale * x + shift), the pairs (scale, shift) per element [C][H][W]
  const float *scale_shift;
  int func;
};
struct BnOut {    // statistics of the output over the batch, turned into (scale, shift) for the consumer of the output
  const mt_tensor *gamma, *beta, *scale_shift, *ivar, *mean, *var, *new_mean, *new_var;
  float momentum, epsilon;
};
int g_tconv_walk = 1;  // plain calls (no batch norm folded in): 0 never walk, 1 walk wherever the shape allows

// ---- transposed convolution 5x5, stride 2, padding 2 to few channels as ONE 3x3 convolution ------------------------
// Output pixel (2*qy + py, 2*qx + px) reads input rows qy + py - 1 .. qy + 1 and columns qx + px - 1 .. qx + 1: the four
// stride phases are 3x3 stride-1 convolutions of the same input with (3 - py) x (3 - px) of the nine taps set, so all of
// them are one convolution to 4 x CO "channels" (c, phase) -- 64 rows instead of four products of 16 -- whose result is
// spread over the output afterwards.  36/25 of the multiplications, but one gather of the input instead of four, and
// tiles of the size the matrix-core kernels are built for.
// merged[(c*4 + py*2 + px)][f*9 + a*3 + b] = kernel[f][c*25 + (4 - (py + 2*(a - py)))*5 + (4 - (px + 2*(b - px)))] for
// a >= py, b >= px (tap (a - py, b - px) of the phase, whose first coefficient is py, px), else 0; `zeros`: 4*CO zeros
// behind it (the convolution's bias).
__global__ __launch_bounds__(256) void tconv_k5s2_merge_kernel(float *merged, const float *kernel, uint32_t ker_ld, uint32_t CO, uint32_t F) {
  const uint32_t cols = F * 9, total = 4 * CO * cols;
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= total + 4 * CO) return;
  if (i >= total) { merged[i] = 0.f; return; }
  const uint32_t r = i / cols, k = i % cols, c = r / 4, py = (r / 2) % 2, px = r % 2, f = k / 9, a = (k % 9) / 3, b = k % 3;
  float v = 0.f;
  if (a >= py && b >= px) v = kernel[(size_t)f * ker_ld + c * 25 + (4 - (py + 2 * (a - py))) * 5 + (4 - (px + 2 * (b - px)))];
  merged[i] = v;
}
// out[w][c][2y + py][2x + px] = func(planes[w][c*4 + py*2 + px][y][x] + bias_sum * taps inside the image)
__global__ __launch_bounds__(256) void tconv_k5s2_spread_kernel(float *out, const float *planes, const float *bias, uint32_t F, uint32_t rows, uint32_t H, uint32_t W, int func) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;   // (w, c, y, x)
  if (i >= (size_t)rows * H * W) return;
  const uint32_t x = (uint32_t)(i % W), y = (uint32_t)((i / W) % H);
  const size_t row = i / ((size_t)W * H);   // w * CO + c
  float bias_sum = 0.f;
  for (uint32_t f = 0; f < F; f++) bias_sum += bias[f];
  const size_t HW = (size_t)H * W;
  const float *p = planes + row * 4 * HW + (size_t)y * W + x;
  const float up = y > 0 ? 1.f : 0.f, down = y + 1 < H ? 1.f : 0.f, left = x > 0 ? 1.f : 0.f, right = x + 1 < W ? 1.f : 0.f;
  const float ny0 = up + 1.f + down, ny1 = 1.f + down, nx0 = left + 1.f + right, nx1 = 1.f + right;
  float2 top, bottom;
  top.x = mt::apply_func_epilogue(func, p[0] + bias_sum * (ny0 * nx0));
  top.y = mt::apply_func_epilogue(func, p[HW] + bias_sum * (ny0 * nx1));
  bottom.x = mt::apply_func_epilogue(func, p[2 * HW] + bias_sum * (ny1 * nx0));
  bottom.y = mt::apply_func_epilogue(func, p[3 * HW] + bias_sum * (ny1 * nx1));
  float *dst = out + row * 4 * HW + (size_t)(2 * y) * (2 * W) + 2 * x;
  *reinterpret_cast<float2 *>(dst) = top;
  *reinterpret_cast<float2 *>(dst + 2 * W) = bottom;
}

// ---- stride-1 transposed convolution as the forward convolution it is ---------------------------------------------------
// out[c][y][x] = sum over (f, a, b) of kernel[f][c*taps + a*KX + b] * delta[f][y - a + py][x - b + px] is the forward
// convolution of delta with the kernels flipped and transposed, padding K - 1 - p: flipped[c][f*taps + t] =
// kernel[f][c*taps + taps - 1 - t].  The forward path orders k tap-major (16 channels of one tap per k step: one input
// offset per step), which a kernel whose taps do not tile the k step (3 x 3) cannot have in the phase formulation above.
// Behind the flipped weights: CO zeros (the convolution's bias) and the sum of the filters' biases, which the reference
// adds once per tap inside the image (cpu/ctensorconv.h:204-268).
__global__ __launch_bounds__(256) void tconv_s1_flip_kernel(float *flipped, const float *kernel, const float *bias, uint32_t ker_ld, uint32_t CO, uint32_t F, uint32_t taps) {
  const uint32_t cols = F * taps, total = CO * cols;
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < total) {
    const uint32_t c = i / cols, k = i % cols, f = k / taps, t = k % taps;
    flipped[i] = kernel[(size_t)f * ker_ld + c * taps + (taps - 1 - t)];
  } else if (i < total + CO) {
    flipped[i] = 0.f;
  } else if (i == total + CO) {
    float sum = 0.f;
    for (uint32_t f = 0; f < F; f++) sum += bias[f];
    flipped[i] = sum;
  }
}
// out[row][y][x] += bias_sum * (taps of (y, x) inside the input image); nothing to do when the sum is zero (a layer's
// backward pass hands over zeroed biases)
__global__ __launch_bounds__(256) void tconv_s1_bias_kernel(float *out, const float *bias_sum, size_t total, uint32_t OH, uint32_t OW, uint32_t IH, uint32_t IW,
                                                            int32_t KY, int32_t KX, int32_t pad_y, int32_t pad_x) {
  const float sum = *bias_sum;
  if (sum == 0.f) return;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const uint32_t x = (uint32_t)(i % OW), y = (uint32_t)((i / OW) % OH);
    int ny = 0, nx = 0;
    for (int32_t t = 0; t < KY; t++) ny += (uint32_t)((int32_t)y + t - pad_y) < IH;
    for (int32_t t = 0; t < KX; t++) nx += (uint32_t)((int32_t)x + t - pad_x) < IW;
    out[i] += sum * (float)(ny * nx);
  }
}

// norm / bn: only the kernel that walks over the batch implements them.  `handled` (required with either) tells the
// caller whether it ran; if not, nothing was launched and the caller composes the result from separate passes.
int backward(const char *name, const mt_tensor *out, const mt_tensor *delta, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz, uint32_t ka,
             const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func, const NormIn *norm = nullptr, const BnOut *bn = nullptr,
             bool *handled = nullptr) {
  const bool fused = norm != nullptr || bn != nullptr;
  if (handled) *handled = false;
  if (mt::bad(out) || mt::bad(delta) || mt::bad(kernel) || mt::bad(bias)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(out);
  if (ka == 0) return mt::fail(MT_E_NO_KERNELS, "%s: at least one kernel is required", name);
  if (ka != bias->z) return mt::fail(MT_E_BIAS_COUNT, "%s: kernel_amount %u but %u biases", name, ka, bias->z);
  if (kx <= 0 || ky <= 0 || kz <= 0 || sx <= 0 || sy <= 0) return mt::fail(MT_E_ARGUMENT, "%s: kernel and stride must be positive", name);
  if (out->z != (uint32_t)kz) return mt::fail(MT_E_OUTPUT_SHAPE, "%s: output depth %u but kernel depth %d", name, out->z, kz);
  if (delta->z != ka) return mt::fail(MT_E_DEPTH, "%s: delta depth %u but kernel_amount %u", name, delta->z, ka);
  if (mt::count(out) == 0) return MT_OK;
  if (delta->w == 0 || bias->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  int rc = check_kernel_tensor(name, kernel, ka, (uint32_t)kz * kx * ky);
  if (rc) return rc;
  ConvGeo g{out->w, delta->w, kernel->w, bias->w, (int32_t)ka, (int32_t)delta->y, (int32_t)delta->x, (int32_t)ka, ky, kx, sy, sx, py, px,
            (int32_t)out->y, (int32_t)out->x, kz, kernel->x, kernel->z * kernel->y};
  bool direct = g_conv_path == 1 || kernel->w != 1 || sx > 4 || sy > 4 || delta->y == 0 || delta->x == 0;
  if (!direct && fused && !mt::fits_buffer(delta)) return MT_OK;
  if (!direct && !mt::fits_buffer(delta)) {
    // the batch is addressed through one 32-bit descriptor: run it in parts of less than 2 GiB of input
    const size_t delta_sample = (size_t)ka * delta->y * delta->x, out_sample = (size_t)kz * out->y * out->x;
    if (delta->w == out->w && bias->w == 1 && mt::fits_buffer(delta_sample)) {
      const uint32_t part = (uint32_t)((0x80000000ull / 4 - 1) / delta_sample);
      for (uint32_t w0 = 0; w0 < out->w; w0 += part) {
        const uint32_t n = out->w - w0 < part ? out->w - w0 : part;
        mt_tensor o{out->p + w0 * out_sample, n, out->z, out->y, out->x}, d{delta->p + w0 * delta_sample, n, delta->z, delta->y, delta->x};
        if ((rc = backward(name, &o, &d, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func))) return rc;
      }
      return MT_OK;
    }
    direct = true;
  }
  if (direct && fused) return MT_OK;
  if (direct) {
    size_t total = mt::count(out);
    mt::ProfileScope prof("tconv_direct");
    tconv_direct_kernel<<<cdiv(total, 256), 256, 0, mt::stream()>>>(out->p, delta->p, kernel->p, bias->p, g, total, func);
    MT_LAUNCH_CHECK(name);
    return MT_OK;
  }

  // 5 x 5, stride 2, padding 2 to 5..16 channels at twice the input size: the four phases as one 3 x 3 convolution to
  // (channel, phase) rows, spread over the output afterwards
  if (g_tconv_merge && !fused && mt::igemm::tile_override() < 0 && kx == 5 && ky == 5 && sx == 2 && sy == 2 && px == 2 && py == 2 && bias->w == 1 &&
      delta->w == out->w && out->y == 2 * delta->y && out->x == 2 * delta->x && kz > 4 && kz <= 16 && ka >= 16 && mt::epilogue_func(func) &&
      ((uintptr_t)out->p & 7u) == 0 && mt::fits_buffer(mt::count(out)) && (size_t)out->w * delta->y * delta->x >= 16384) {
    const uint32_t rows4 = 4u * (uint32_t)kz, cols = ka * 9u;
    const size_t merged_floats = ((size_t)rows4 * cols + rows4 + 3) & ~(size_t)3, plane_floats = mt::count(out);
    float *buf = nullptr;
    if ((rc = mt::workspace_get(g_merge_ws, "merged phases", merged_floats + plane_floats, &buf))) return rc;
    float *planes = buf + merged_floats;
    {
      mt::ProfileScope prof("tconv_prepare");
      tconv_k5s2_merge_kernel<<<cdiv((size_t)rows4 * cols + rows4, 256), 256, 0, mt::stream()>>>(buf, kernel->p, kernel->x, (uint32_t)kz, ka);
      MT_LAUNCH_CHECK(name);
    }
    mt::note_write(buf, (merged_floats + plane_floats) * sizeof(float));   // (a copy of these weights that the forward pass kept is stale)
    mt_tensor merged{buf, 1, 1, rows4, cols}, zeros{buf + (size_t)rows4 * cols, 1, rows4, 1, 1}, wide{planes, out->w, rows4, delta->y, delta->x};
    if ((rc = forward(name, &wide, delta, &merged, 3, 3, (int32_t)ka, rows4, &zeros, 1, 1, 1, 1, MT_F_NONE))) return rc;
    {
      mt::ProfileScope prof("tconv_spread");
      tconv_k5s2_spread_kernel<<<cdiv(plane_floats / 4, 256), 256, 0, mt::stream()>>>(out->p, planes, bias->p, ka, out->w * (uint32_t)kz, delta->y, delta->x, func);
      MT_LAUNCH_CHECK(name);
    }
    g_tconv_merge_launches++;
    return MT_OK;
  }
  // few filters of 3 x 3, stride 1, padding 1 on large images: the nine taps share one patch of delta in LDS, the weights are
  // read as they lie
  // (stride 1, taps that do not tile the k step: also the forward convolution with flipped, transposed kernels, below; from 32
  // filters on it is the faster of the two: 680 against 740 us for 32 filters to 64 channels at 256 x 256, batch 32)
  const bool as_conv = g_tconv_as_conv && !fused && mt::igemm::tile_override() < 0 && sx == 1 && sy == 1 && BK % (uint32_t)(kx * ky) != 0 && ka % BK == 0 &&
                       kz >= 16 && bias->w == 1 && delta->w == out->w && px <= kx - 1 && py <= ky - 1 && out->y == delta->y + (uint32_t)(ky - 1 - 2 * py) &&
                       out->x == delta->x + (uint32_t)(kx - 1 - 2 * px) && func == MT_F_NONE && kernel->x == (uint32_t)(kz * kx * ky) &&
                       (size_t)ka * kx * ky >= 256 && mt::fits_buffer(out) && mt::fits_buffer(delta);
  if (g_tconv_patch && !fused && mt::igemm::tile_override() < 0 && kx == 3 && ky == 3 && sx == 1 && sy == 1 && px == 1 && py == 1 && bias->w == 1 &&
      delta->w == out->w && delta->y == out->y && delta->x == out->x && !(as_conv && ka > 16)) {
    mt::igemm::TconvPatchArgs tp{};
    tp.delta = delta->p; tp.kernel = kernel->p; tp.bias = bias->p; tp.out = out->p;
    tp.B = out->w; tp.F = ka; tp.C = (uint32_t)kz; tp.H = out->y; tp.W = out->x; tp.ld = kernel->x;
    if (mt::igemm::tconv_patch_plan(tp)) {
      {
        mt::ProfileScope prof(mt::profiling() ? shape_label(name, T16x256, (uint32_t)kz, out->w * out->y * out->x, ka * 9, 1) : name);
        if ((rc = mt::igemm::launch_tconv_patch(name, tp))) return rc;
      }
      g_tconv_patch_launches++;
      return func == MT_F_NONE ? MT_OK : mt_apply_func(out, out, func);
    }
  }
  // stride 1, taps that do not tile the k step (3 x 3, 5 x 5): the forward convolution with flipped, transposed kernels
  if (as_conv) {
    const uint32_t taps = (uint32_t)(kx * ky), cols = ka * taps;
    const size_t flip_floats = ((size_t)kz * cols + (size_t)kz + 1 + 3) & ~(size_t)3;
    float *buf = nullptr;
    if ((rc = mt::workspace_get(g_merge_ws, "flipped kernels", flip_floats, &buf))) return rc;
    {
      mt::ProfileScope prof("tconv_prepare");
      tconv_s1_flip_kernel<<<cdiv((size_t)kz * cols + kz + 1, 256), 256, 0, mt::stream()>>>(buf, kernel->p, bias->p, kernel->x, (uint32_t)kz, ka, taps);
      MT_LAUNCH_CHECK(name);
    }
    mt::note_write(buf, flip_floats * sizeof(float));   // (a re-ordered copy of these weights that the forward path kept is stale)
    mt_tensor flipped{buf, 1, 1, (uint32_t)kz, cols}, zeros{buf + (size_t)kz * cols, 1, (uint32_t)kz, 1, 1};
    if ((rc = forward(name, out, delta, &flipped, kx, ky, (int32_t)ka, (uint32_t)kz, &zeros, 1, 1, kx - 1 - px, ky - 1 - py, MT_F_NONE))) return rc;
    {
      mt::ProfileScope prof("tconv_tap_bias");
      tconv_s1_bias_kernel<<<1024, 256, 0, mt::stream()>>>(out->p, buf + (size_t)kz * cols + kz, mt::count(out), out->y, out->x, delta->y, delta->x, ky, kx,
                                                           ky - 1 - py, kx - 1 - px);
      MT_LAUNCH_CHECK(name);
    }
    g_tconv_as_conv_launches++;
    return MT_OK;
  }
  // workspace: [bias sums (bias_w, padded to 64)] [packed sub-kernels of all phases: kz*ka*ky*kx floats + alignment]
  size_t sums = (bias->w + 63u) & ~(size_t)63u;
  float *ws = nullptr;
  bool fresh = true;
  const bool tile = mt::igemm::tile_override() < 0 && tile_kernel_fits(out, delta, kx, ky, kz, ka, sx, sy, px, py);
  const bool tile_norm = tile && norm && !bn;   // the image layer's kernel normalises its input on the way to LDS
  if (fused && !tile_norm && (tile || kz <= 4 || mt::igemm::tile_override() >= 0)) return MT_OK;
  // the phases depend on the output size as well (an odd output has phases of different sizes and may lack one)
  if ((rc = pack_buffer(pack_key(0, kernel, bias, {kx, ky, kz, (int32_t)ka, sx, sy, px, py, (int32_t)out->x, (int32_t)out->y, tile ? 1 : 0}),
                        sums + (size_t)kz * ka * ky * kx + (size_t)4 * kz * sy * sx + 64, &ws, &fresh)))
    return rc;
  float *packed = ws + sums;

  TconvArgs args{};
  PackArgs pa{};
  pa.ker_ld = kernel->x; pa.bias_w = bias->w; pa.CO = kz; pa.CI = ka; pa.KY = ky; pa.KX = kx; pa.SY = sy; pa.SX = sx;
  uint32_t max_n = 0, max_pack = 0, begin = 0;
  const uint32_t OHW = out->y * out->x;
  for (int32_t phy = 0; phy < sy; phy++) {
    Phase1D Y = phase_1d(phy, ky, sy, py, out->y);
    if (Y.q == 0) continue;
    for (int32_t phx = 0; phx < sx; phx++) {
      Phase1D X = phase_1d(phx, kx, sx, px, out->x);
      if (X.q == 0) continue;
      uint32_t kp = ka * Y.taps * X.taps, ld = (kp + 3u) & ~3u, f = args.nphase++;
      pa.ph[f] = PackPhase{begin, kp, ld, Y.k0, X.k0, Y.taps, X.taps, ld, (uint32_t)(Y.taps * X.taps)};
      if (tile) {  // [ci][phase][co][2x2 taps]
        pa.ph[f].begin = f * 4u * (uint32_t)kz; pa.ph[f].co_stride = 4; pa.ph[f].ci_stride = 16u * (uint32_t)kz;
      }
      args.ph[f] = TconvPhase{packed + pa.ph[f].begin, kp, ld, (uint32_t)Y.q, (uint32_t)X.q, Y.taps, X.taps, Y.off, X.off, (uint32_t)phy, (uint32_t)phx};
      begin += (uint32_t)kz * ld;  // a multiple of four floats: every phase starts 16-byte aligned
      uint32_t n = out->w * Y.q * X.q;
      if (n > max_n) max_n = n;
      if ((uint32_t)kz * ld > max_pack) max_pack = (uint32_t)kz * ld;
    }
  }
  pa.nphase = args.nphase;
  // blocks that walk over the batch: the statistics of the output, the normalisation of the input, and for plain calls
  // the saving of a cold start per tile
  WalkArgs walk{};
  bool walks = false;
  uint32_t walk_tm = 1;
  if (!tile && kz > 4 && mt::igemm::tile_override() < 0 && (fused || g_tconv_walk) && bias->w == 1 && delta->w == out->w && (int32_t)args.nphase == sy * sx &&
      mt::fits_buffer((size_t)ka * delta->y * delta->x * 2)) {
    for (uint32_t f = 0; f < args.nphase; f++) walk.ph[f] = args.ph[f];
    walk.nphase = args.nphase; walk.M = (uint32_t)kz; walk.batch = out->w;
    walk.delta = delta->p; walk.C = ka; walk.H = delta->y; walk.W = delta->x;
    walk.out = out->p; walk.OW = out->x; walk.OHW = OHW; walk.sy = (uint32_t)sy; walk.sx = (uint32_t)sx;
    walk.func = bn || !mt::epilogue_func(func) ? MT_F_NONE : func;   // any other function runs as a pass of its own afterwards
    if (norm) { walk.scale_shift = norm->scale_shift; walk.in_func = norm->func; }
    size_t covered = 0;
    for (uint32_t f = 0; f < args.nphase; f++) covered += (size_t)args.ph[f].qh * args.ph[f].qw;
    walk_tm = mt::igemm::walk_tm() == 2 && kz % 128 == 0 ? 2u : 1u;
    walk.wide = g_walk_wide && !norm && !bn && kz % 64 != 0 && kz % 32 == 0 ? 1u : 0u;
    if (walk.wide) walk_tm = 1;
    walks = covered == OHW && tconv_walk_plan(walk, (uint32_t)mt::igemm::walk_blocks(), walk_tm);
  }
  bool k4s2 = kx == 4 && ky == 4 && sx == 2 && sy == 2 && args.nphase == 4 && kernel->x % 4 == 0 && ((uintptr_t)kernel->p & 15u) == 0 && kz <= 65534;
  for (uint32_t f = 0; k4s2 && f < 4; f++) k4s2 = pa.ph[f].ty == 2 && pa.ph[f].tx == 2 && pa.ph[f].ci_stride % 4 == 0 && pa.ph[f].co_stride % 4 == 0;
  if (k4s2 && kernel->x == (uint32_t)kz * 16u) {
    // an optimiser step may keep this copy current: tell the cache entry (if the copy lives in one) how it is laid out
    PackK4S2 info;
    info.on = true; info.sums = (uint32_t)sums; info.CO = (uint32_t)kz; info.CI = ka; info.co_stride = pa.ph[0].co_stride; info.ci_stride = pa.ph[0].ci_stride;
    uint32_t seen = 0;
    for (uint32_t f = 0; f < 4; f++) {
      info.begin[f] = pa.ph[f].begin;
      info.on = info.on && (uint32_t)pa.ph[f].ky0 < 2u && (uint32_t)pa.ph[f].kx0 < 2u && pa.ph[f].co_stride == info.co_stride && pa.ph[f].ci_stride == info.ci_stride;
      if (info.on) { info.phase_of[pa.ph[f].ky0 * 2 + pa.ph[f].kx0] = (uint8_t)f; seen |= 1u << (pa.ph[f].ky0 * 2 + pa.ph[f].kx0); }
    }
    if (info.on && seen == 15u)
      for (PackEntry &e : g_packs)
        if (e.buf == ws) e.k4s2 = info;
  }
  if (fresh) {
    mt::ProfileScope prof("tconv_prepare");
    if (k4s2) {
      tconv_prepare_k4s2_kernel<<<dim3(cdiv(ka, 256), kz + 1), 256, 0, mt::stream()>>>(packed, ws, kernel->p, bias->p, pa);
    } else {
      unsigned gx = cdiv(max_pack ? max_pack : 1, 256 * 4);
      if (gx > 1024) gx = 1024;
      tconv_prepare_kernel<<<dim3(gx ? gx : 1, args.nphase + 1), 256, 0, mt::stream()>>>(packed, ws, kernel->p, bias->p, pa);
    }
    MT_LAUNCH_CHECK("tconv_prepare");
  }
  args.M = kz; args.out_w = out->w;
  args.delta = delta->p; args.in_w = delta->w; args.C = ka; args.H = delta->y; args.W = delta->x;
  args.ep.C = out->p; args.ep.row_stride = OHW; args.ep.g_stride = (size_t)kz * OHW;
  args.ep.sy = sy; args.ep.sx = sx; args.ep.OW = out->x;
  args.ep.tap_bias = ws; args.ep.bias_w = bias->w; args.ep.IH = delta->y; args.ep.IW = delta->x;
  args.ep.func = func;
  if (fused && !walks && !tile_norm) return MT_OK;
  if (walks) {
    const size_t S = (size_t)kz * OHW;
    if (bn) {
      float *part = nullptr;
      if ((rc = mt::workspace_get(g_stats_ws, "batch-norm partial statistics", 2 * (size_t)walk.groups * S, &part))) return rc;
      walk.part_mean = part; walk.part_m2 = part + (size_t)walk.groups * S;
    }
    walk.tap_bias = ws;
    {
      mt::ProfileScope prof(mt::profiling() ? shape_label(name, walk.wide ? T32x128 : T64x64, walk.M, out->w * args.ph[0].qh * args.ph[0].qw, args.ph[0].kp, args.nphase) : name);
      if ((rc = launch_tconv_walk(name, walk, norm != nullptr, bn != nullptr, walk_tm))) return rc;
    }
    if (bn) {
      mt::ProfileScope prof("bn_finish");
      const float mom_new = (float)(1.0 - (double)bn->momentum);
      bn_finish_kernel<<<cdiv(S, 64), 256, 0, mt::stream()>>>(bn->scale_shift->p, bn->mean ? bn->mean->p : nullptr, bn->var ? bn->var->p : nullptr,
                                                              bn->ivar ? bn->ivar->p : nullptr, bn->new_mean ? bn->new_mean->p : nullptr,
                                                              bn->new_var ? bn->new_var->p : nullptr, walk.part_mean, walk.part_m2, walk.groups,
                                                              (float)(walk.per * (64u >> walk.px_log)), (uint32_t)S, bn->gamma->p, bn->beta->p, bn->epsilon,
                                                              bn->momentum, mom_new);
      MT_LAUNCH_CHECK("bn_finish");
    }
    if (handled) *handled = true;
    return !bn && !mt::epilogue_func(func) ? mt_apply_func(out, out, func) : MT_OK;
  }
  if (tile_norm) {
    args.in_scale_shift = norm->scale_shift; args.in_func = norm->func;
    if (handled) *handled = true;
  }
  if (tile) return launch_tconv_tile(name, args);
  // (a small output behind a long k axis -- 128 filters to one channel at 16 x 16 -- has too few pixels for one thread each:
  // the matrix-core path cuts its k axis over blocks)
  const bool few_pixels = (size_t)max_n * args.nphase < 32768 && (size_t)ka * ky * kx >= 512;
  if (kz <= 4 && mt::igemm::tile_override() < 0 && !few_pixels) {
    rc = launch_tconv_small(name, args, max_n);
    if (rc >= 0) return rc;
  }
  if (mt::epilogue_func(func)) return launch_tconv(name, args, max_n, mt::count(out));
  args.ep.func = MT_F_NONE;
  rc = launch_tconv(name, args, max_n, mt::count(out));
  return rc == MT_OK ? mt_apply_func(out, out, func) : rc;
}

// A transposed convolution between two batch-norm layers: the input may still owe its normalisation and activation
// (scale_shift [1,C,H,2*W], delta_func), and the statistics of the output may be wanted as the (scale, shift) pairs of
// the NEXT batch normalisation.  One kernel when the blocks can walk over the batch; otherwise the same result from
// separate passes: normalise into the workspace, convolve, statistics over the output.
int backward_between_norms(const char *name, const mt_tensor *out, const mt_tensor *delta, const mt_tensor *scale_shift, int delta_func, const mt_tensor *kernel,
                           int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func,
                           const BnOut *bn) {
  if (mt::bad(out) || mt::bad(delta)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  if (scale_shift) {
    if (mt::bad(scale_shift) || scale_shift->w == 0 || scale_shift->z != delta->z || scale_shift->y != delta->y || scale_shift->x != 2 * delta->x)
      return mt::fail(MT_E_SHAPE, "%s: the (scale, shift) pairs of the input must be [1,%u,%u,%u]", name, delta->z, delta->y, 2 * delta->x);
    if (!mt::epilogue_func(delta_func)) return mt::fail(MT_E_ARGUMENT, "%s: the input's function must be none, linear, ReLU or leaky ReLU", name);
  }
  if (bn) {
    const mt_tensor *same[7] = {bn->gamma, bn->beta, bn->ivar, bn->mean, bn->var, bn->new_mean, bn->new_var};
    for (int i = 0; i < 7; i++) {
      if (i < 2 && mt::bad(same[i])) return mt::fail(MT_E_ARGUMENT, "%s: gamma and beta are required", name);
      if (same[i] && (mt::bad(same[i]) || !mt::same_zyx(same[i], out) || same[i]->w == 0)) return mt::fail(MT_E_SHAPE, "%s: statistics and parameters must be [1,Z,Y,X] of the output", name);
    }
    if (mt::bad(bn->scale_shift) || bn->scale_shift->w == 0 || bn->scale_shift->z != out->z || bn->scale_shift->y != out->y || bn->scale_shift->x != 2 * out->x)
      return mt::fail(MT_E_SHAPE, "%s: the (scale, shift) pairs of the output must be [1,%u,%u,%u]", name, out->z, out->y, 2 * out->x);
    for (auto t : {bn->scale_shift, bn->ivar, bn->mean, bn->var, bn->new_mean, bn->new_var}) mt::note_write(t);
  }
  if (!scale_shift && !bn) return backward(name, out, delta, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func);  // nothing folded in: the plain call, once
  NormIn norm{scale_shift ? scale_shift->p : nullptr, delta_func};
  bool handled = false;
  int rc = backward(name, out, delta, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func, scale_shift ? &norm : nullptr, bn, &handled);
  if (rc || handled) return rc;
  mt_tensor in = *delta;
  if (scale_shift && mt::count(delta)) {
    float *tmp = nullptr;
    if ((rc = mt::workspace_get(g_norm_ws, "normalised input", mt::count(delta), &tmp))) return rc;
    in.p = tmp;
    if ((rc = mt::norm_apply(&in, delta, scale_shift->p, delta_func))) return rc;
  }
  if ((rc = backward(name, out, &in, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, bn ? MT_F_NONE : func))) return rc;
  if (!bn) return MT_OK;
  return mt::bn_statistics(out, bn->gamma, bn->beta, bn->scale_shift, bn->ivar, bn->mean, bn->var, bn->new_mean, bn->new_var, bn->momentum, bn->epsilon);
}

// Whether the weight gradient's image operand can use fixed per-thread offsets (SrcWgradImageFixed): the output
// pixels must tile the k step for the number of pixels a thread loads in the block tile that will be chosen.
bool wgrad_image_fixed(uint32_t M, uint32_t N, uint32_t batches, const mt_tensor *delta, const mt_tensor *image, int32_t kz, uint32_t per, int32_t px,
                       int32_t py) {
  if (px < 0 || py < 0) return false;
  const Tile tile = pick_tile(M, N, batches);
  const uint32_t pixels = tile_cols(tile) * BK / THREADS;
  const size_t span = (size_t)per * kz * image->y * image->x + (size_t)py * image->x + px;
  return SrcWgradImageFixed::fits(delta->y, delta->x, pixels) && mt::fits_buffer(span);
}

int wgrad(const char *name, const mt_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *db, const mt_tensor *image,
          const mt_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py, bool bias_too) {
  if (mt::bad(dk) || mt::bad(db) || mt::bad(image) || mt::bad(delta)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(dk);
  mt::note_write(db);
  if (ka == 0) return mt::fail(MT_E_NO_KERNELS, "%s: at least one kernel gradient is required", name);
  if (db->z != ka) return mt::fail(MT_E_BIAS_COUNT, "%s: kernel_amount %u but %u bias gradients", name, ka, db->z);
  if (kx <= 0 || ky <= 0 || kz <= 0 || sx <= 0 || sy <= 0) return mt::fail(MT_E_ARGUMENT, "%s: kernel and stride must be positive", name);
  if ((uint32_t)kz != image->z) return mt::fail(MT_E_SHAPE, "%s: kernel depth %d but image depth %u", name, kz, image->z);
  if (delta->z != ka) return mt::fail(MT_E_DEPTH, "%s: delta depth %u but kernel_amount %u", name, delta->z, ka);
  if (dk->w == 0) return MT_OK;
  if (image->w == 0 || delta->w == 0 || db->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  uint32_t ncol = (uint32_t)kz * kx * ky, DHW = delta->y * delta->x;
  int rc = check_kernel_tensor(name, dk, ka, ncol);
  if (rc) return rc;
  if (DHW == 0) return MT_OK;
  ConvGeo g{dk->w, image->w, dk->w, db->w, kz, (int32_t)image->y, (int32_t)image->x, (int32_t)ka, ky, kx, sy, sx, py, px, 0, 0, 0, dk->x, dk->z * dk->y};
  bool direct = g_conv_path == 1 || dk->w > 65535u || !mt::fits_buffer((size_t)kz * image->y * image->x) || !mt::fits_buffer((size_t)ka * DHW);
  if (direct) {
    size_t total = (size_t)dk->w * ka * ncol;
    wgrad_direct_kernel<<<cdiv(total, 256), 256, 0, mt::stream()>>>(dk->p, image->p, delta->p, g, delta->w, delta->y, delta->x, total);
    MT_LAUNCH_CHECK(name);
  } else {
    Batch abt;
    abt.wmod = delta->w; abt.stride = (size_t)ka * DHW;
    SrcWgradImage b{};
    b.p = image->p; b.C = kz; b.H = image->y; b.W = image->x; b.KY = ky; b.KX = kx; b.OW = delta->x; b.R = ncol; b.K = DHW; b.sy = sy; b.sx = sx; b.py = py; b.px = px;
    b.bt.wmod = image->w; b.bt.stride = (size_t)kz * image->y * image->x;
    Epilogue ep{};
    ep.C = dk->p; ep.row_stride = dk->x; ep.inner = ncol; ep.g_stride = 0; ep.accumulate = true;
    ep.bt.wmod = dk->w; ep.bt.stride = (size_t)dk->z * dk->y * dk->x;
    if (wgrad_image_fixed(ka, ncol, dk->w, delta, image, kz, 1, px, py)) {
      SrcWgradImageFixed bf{};
      bf.p = b.p; bf.C = b.C; bf.H = b.H; bf.W = b.W; bf.KY = b.KY; bf.KX = b.KX; bf.OW = b.OW; bf.OH = 0; bf.R = b.R; bf.K = b.K;
      bf.sy = sy; bf.sx = sx; bf.py = py; bf.px = px; bf.bt = b.bt;
      rc = with_row_k(delta->p, DHW, ka, DHW, abt, [&](auto a) { return launch(name, a, bf, ep, ka, ncol, DHW, dk->w); });
    } else {
      rc = with_row_k(delta->p, DHW, ka, DHW, abt, [&](auto a) { return launch(name, a, b, ep, ka, ncol, DHW, dk->w); });
    }
    if (rc) return rc;
  }
  if (!bias_too) return MT_OK;
  if (db->y != 1 || db->x != 1) return mt::fail(MT_E_ARGUMENT, "%s: bias gradient must be [W,Z,1,1]", name);
  if (db->w >= dk->w && g_conv_path != 1) {
    uint32_t rows = dk->w * ka;
    dbias_wave_kernel<<<cdiv(rows, 4), 256, 0, mt::stream()>>>(db->p, delta->p, delta->w, ka, DHW, rows);
  } else {
    uint32_t wb = db->w < dk->w ? db->w : dk->w;
    dbias_serial_kernel<<<cdiv((size_t)wb * ka, 256), 256, 0, mt::stream()>>>(db->p, wb, delta->p, delta->w, ka, DHW, dk->w);
  }
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

// delta with rows of zeros appended to every image: [rows][hw] -> [rows][hw2]
__global__ __launch_bounds__(256) void pad_rows_kernel(float *out, const float *in, uint32_t hw, uint32_t hw2, size_t total) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const size_t row = i / hw2;
  const uint32_t k = (uint32_t)(i - row * hw2);
  out[i] = k < hw ? in[row * hw + k] : 0.f;
}

// Weight and bias gradient of a convolution layer summed over the batch in one product: K runs over (sample, output
// pixel), so dK[f][(c,i,j)] += sum_w sum_(oy,ox) delta[w][f][oy][ox] * image[w][c][oy*s-p+i][ox*s-p+j] without the
// per-sample gradients ever being written.  When the product has few output tiles the batch is split into groups
// whose partial sums go to the workspace and are added afterwards (fixed order: the result does not depend on timing).
int wgrad_batch_sum(const char *name, const mt_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *db, const mt_tensor *image,
                    const mt_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  if (mt::bad(dk) || mt::bad(db) || mt::bad(image) || mt::bad(delta)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(dk);
  mt::note_write(db);
  if (ka == 0) return mt::fail(MT_E_NO_KERNELS, "%s: at least one kernel gradient is required", name);
  if (db->z != ka) return mt::fail(MT_E_BIAS_COUNT, "%s: kernel_amount %u but %u bias gradients", name, ka, db->z);
  if (kx <= 0 || ky <= 0 || kz <= 0 || sx <= 0 || sy <= 0) return mt::fail(MT_E_ARGUMENT, "%s: kernel and stride must be positive", name);
  if ((uint32_t)kz != image->z) return mt::fail(MT_E_SHAPE, "%s: kernel depth %d but image depth %u", name, kz, image->z);
  if (delta->z != ka) return mt::fail(MT_E_DEPTH, "%s: delta depth %u but kernel_amount %u", name, delta->z, ka);
  if (dk->w != 1 || db->w != 1 || db->y != 1 || db->x != 1) return mt::fail(MT_E_ARGUMENT, "%s: the summed gradients are [1,1,Kamt,C*Ky*Kx] and [1,Kamt,1,1]", name);
  if (image->w != delta->w) return mt::fail(MT_E_SHAPE, "%s: image and delta batch sizes differ", name);
  const uint32_t B = delta->w, ncol = (uint32_t)kz * kx * ky, DHW = delta->y * delta->x;
  int rc = check_kernel_tensor(name, dk, ka, ncol);
  if (rc) return rc;
  if (B == 0 || DHW == 0) return MT_OK;
  const size_t sample_image = (size_t)kz * image->y * image->x, sample_delta = (size_t)ka * DHW;
  if (g_conv_path != 1 && DHW % BK != 0 && g_wgrad_pad && sample_image * 4 < 0x80000000ull) {
    // Output images whose pixels do not fill whole k steps (3 x 4 at the end of a discriminator): the same sums with rows of
    // zeros appended to every image of delta -- the image rows those would meet are inside the tensor or masked like any
    // row below the image, and a zero times either adds nothing
    uint32_t oh2 = delta->y;
    while ((oh2 * delta->x) % BK != 0 && oh2 <= 2 * delta->y) oh2++;
    const size_t padded_floats = (size_t)B * ka * oh2 * delta->x;
    if ((oh2 * delta->x) % BK == 0 && oh2 <= 2 * delta->y && padded_floats * 4 < 0x80000000ull) {
      float *buf = nullptr;
      if ((rc = mt::workspace_get(g_pad_ws, "padded delta", padded_floats, &buf))) return rc;
      {
        mt::ProfileScope prof("pad_rows");
        pad_rows_kernel<<<cdiv(padded_floats, 256), 256, 0, mt::stream()>>>(buf, delta->p, DHW, oh2 * delta->x, padded_floats);
        MT_LAUNCH_CHECK(name);
      }
      mt_tensor padded{buf, B, ka, oh2, delta->x};
      return wgrad_batch_sum(name, dk, kx, ky, kz, ka, db, image, &padded, sx, sy, px, py);
    }
  }
  if (g_conv_path == 1 || DHW % BK != 0 || sample_image * 4 >= 0x80000000ull || sample_delta * 4 >= 0x80000000ull) {
    // per-sample gradients into the workspace, then their sum: the op sequence of the layer itself
    float *ws = nullptr;
    if ((rc = workspace((size_t)B * ka * ncol + (size_t)B * ka, &ws))) return rc;
    mt_tensor dkb{ws, B, 1, ka, ncol}, dbb{ws + (size_t)B * ka * ncol, B, ka, 1, 1};
    if ((rc = mt_fill(&dkb, 0.f)) || (rc = mt_fill(&dbb, 0.f))) return rc;
    if ((rc = wgrad(name, &dkb, kx, ky, kz, ka, &dbb, image, delta, sx, sy, px, py, true))) return rc;
    mt_tensor flat{dk->p, 1, 1, ka, ncol};
    const mt_tensor *dst = (dk->x == ncol && dk->z * dk->y == ka) ? &flat : nullptr;
    if (!dst) return mt::fail(MT_E_ARGUMENT, "%s: the summed kernel gradient must be exactly [1,1,%u,%u]", name, ka, ncol);
    if ((rc = mt_add_sum_w(dst, dst, &dkb, 1.f, 1.f))) return rc;
    return mt_add_sum_w(db, db, &dbb, 1.f, 1.f);
  }
  // few filters of 3 x 3, stride 1, padding 1 on large images: the nine taps share one patch in LDS
  if (g_wgrad_patch && kx == 3 && ky == 3 && sx == 1 && sy == 1 && px == 1 && py == 1 && image->y == delta->y && image->x == delta->x &&
      dk->x == ncol && dk->z * dk->y == ka) {
    mt::igemm::WgradPatchArgs pa{};
    pa.delta = delta->p; pa.image = image->p; pa.B = B; pa.KA = ka; pa.C = (uint32_t)kz; pa.H = delta->y; pa.W = delta->x;
    if (mt::igemm::wgrad_patch_plan(pa)) {
      const uint32_t sums = 2 * pa.groups, chunks = dbias_chunks(B, ka, DHW);
      float *ws = nullptr;
      if ((rc = workspace((size_t)sums * ka * ncol + (chunks > 1 ? (size_t)ka * chunks : 0), &ws))) return rc;
      pa.partial = ws;
      {
        mt::ProfileScope prof(mt::profiling() ? shape_label(name, T64x64, ka, ncol, B * DHW, pa.groups * pa.slabs) : name);
        if ((rc = mt::igemm::launch_wgrad_patch(name, pa))) return rc;
      }
      g_wgrad_patch_launches++;
      mt_tensor pt{ws, sums, 1, ka, ncol}, flat{dk->p, 1, 1, ka, ncol};
      if ((rc = mt_add_sum_w(&flat, &flat, &pt, 1.f, 1.f))) return rc;
      return dbias_batch_sum(name, db->p, ws + (size_t)sums * ka * ncol, delta->p, B, ka, DHW, chunks);
    }
  }
  // groups: enough blocks for every compute unit, and a divisor of the batch so that all groups have the same K
  const uint32_t tiles = cdiv(ka, 64) * cdiv(ncol, 64);
  uint32_t groups = 1;
  while (groups < B && tiles * groups < 1024) {
    uint32_t g = groups + 1;
    while (g < B && B % g) g++;
    groups = g;
  }
  if (g_wgrad_groups > 0 && B % (uint32_t)g_wgrad_groups == 0) groups = (uint32_t)g_wgrad_groups;
  while (groups < B && (!mt::fits_buffer((size_t)(B / groups) * sample_image) || !mt::fits_buffer((size_t)(B / groups) * sample_delta))) {
    uint32_t g = groups + 1;   // a group's samples are addressed through one descriptor: keep its span below 2 GiB
    while (g < B && B % g) g++;
    groups = g;
  }
  const uint32_t per = B / groups;
  // rows of delta against a gather from the image with fixed offsets, one k loop per block (wgrad_walk_kernel), where the
  // shape allows; it may cut the samples themselves into groups when the batch alone gives few blocks
  mt::igemm::WgradWalkArgs wa{};
  bool walks = false;
  if (g_wgrad_walk && dk->x == ncol && dk->z * dk->y == ka) {
    wa.delta = delta->p; wa.image = image->p;
    wa.M = ka; wa.N = ncol; wa.C = (uint32_t)kz; wa.H = image->y; wa.W = image->x; wa.OH = delta->y; wa.OW = delta->x; wa.KY = (uint32_t)ky; wa.KX = (uint32_t)kx;
    wa.sy = sy; wa.sx = sx; wa.py = py; wa.px = px; wa.groups = groups;
    walks = mt::igemm::wgrad_walk_plan(wa, B, g_wgrad_groups == 0);
  }
  float *partial = nullptr, *dbias_partial = nullptr;
  const uint32_t chunks = dbias_chunks(B, ka, DHW);
  const size_t wgrad_floats = walks ? (size_t)wa.groups * ka * ncol : groups > 1 ? (size_t)groups * ka * ncol : 0;
  if (groups > 1 && (dk->x != ncol || dk->z * dk->y != ka))
    return mt::fail(MT_E_ARGUMENT, "%s: the summed kernel gradient must be exactly [1,1,%u,%u]", name, ka, ncol);
  const size_t dbias_floats = walks ? (size_t)ka * wa.groups : chunks > 1 ? (size_t)ka * chunks : 0;   // (the walking kernel sums delta as it passes)
  if (wgrad_floats + dbias_floats > 0) {
    if ((rc = workspace(wgrad_floats + dbias_floats, &partial))) return rc;
    dbias_partial = partial + wgrad_floats;
  }
  if (walks) {
    wa.partial = partial;
    wa.bias_partial = dbias_partial;
    {
      mt::ProfileScope prof(mt::profiling() ? shape_label(name, T64x64, ka, ncol, wa.steps * BK, wa.groups) : name);
      if ((rc = mt::igemm::launch_wgrad_walk(name, wa))) return rc;
    }
    g_wgrad_walk_launches++;
    return mt::add_sum_w_pair(dk->p, partial, (size_t)ka * ncol, db->p, dbias_partial, ka, wa.groups);  // the groups in order, one launch for both
  }
  // Few filters on large images (the last layers of a generator: 16 filters at 192 x 256) leave fewer tiles x samples than
  // the chip has compute units even with one group per sample: the groups then become equal bands of output rows of one
  // sample each (`parts` per sample), for the source that gathers with fixed offsets
  uint32_t parts = 1;
  if (g_wgrad_parts && groups == B && DHW % 4 == 0 && ((uintptr_t)delta->p & 15u) == 0 && dk->x == ncol && dk->z * dk->y == ka) {
    const uint32_t OH = delta->y, OW = delta->x;
    auto fits = [&](uint32_t n) {
      return OH % n == 0 && ((OH / n) * OW) % BK == 0 && (OH / n) * OW >= 32u * BK && (size_t)B * n * ka * ncol <= ((size_t)1 << 26) &&
             wgrad_image_fixed(ka, ncol, B * n, delta, image, kz, 1, px, py);
    };
    auto blocks = [&](uint32_t n) {   // with the tile that the product of B * n groups will get
      const Tile tile = pick_tile(ka, ncol, B * n);
      return (size_t)cdiv(ka, tile_rows(tile)) * cdiv(ncol, tile_cols(tile)) * B * n;
    };
    while (blocks(parts) < 1024 && parts < 256 && fits(parts * 2)) parts *= 2;
    if (g_wgrad_parts > 1 && fits((uint32_t)g_wgrad_parts)) parts = (uint32_t)g_wgrad_parts;
  }
  if (parts > 1) {
    const uint32_t total = B * parts, rows = delta->y / parts, chunk = rows * delta->x;
    float *band_sums = nullptr;
    if ((rc = workspace((size_t)total * ka * ncol + (chunks > 1 ? (size_t)ka * chunks : 0), &band_sums))) return rc;
    SrcRowK<true> a{};
    a.p = delta->p; a.ld = DHW; a.R = ka; a.K = chunk;
    a.bt.wmod = B; a.bt.zcount = parts; a.bt.wstride = sample_delta; a.bt.stride = chunk;
    SrcWgradImageFixed bf{};
    bf.p = image->p; bf.C = kz; bf.H = image->y; bf.W = image->x; bf.KY = ky; bf.KX = kx; bf.OW = delta->x; bf.OH = 0; bf.R = ncol; bf.K = chunk;
    bf.sy = sy; bf.sx = sx; bf.py = py; bf.px = px; bf.part_rows = rows;
    bf.bt.wmod = B; bf.bt.zcount = parts; bf.bt.wstride = sample_image; bf.bt.stride = 0;
    Epilogue ep{};
    ep.inner = ncol; ep.g_stride = 0;
    ep.C = band_sums; ep.row_stride = ncol; ep.bt.wmod = total; ep.bt.stride = (size_t)ka * ncol;
    if ((rc = launch(name, a, bf, ep, ka, ncol, chunk, total))) return rc;
    mt_tensor pt{band_sums, total, 1, ka, ncol}, flat{dk->p, 1, 1, ka, ncol};
    if ((rc = mt_add_sum_w(&flat, &flat, &pt, 1.f, 1.f))) return rc;
    return dbias_batch_sum(name, db->p, band_sums + (size_t)total * ka * ncol, delta->p, B, ka, DHW, chunks);
  }
  SrcRowK<true> a{};
  a.p = delta->p; a.ld = DHW; a.R = ka; a.K = per * DHW; a.seg = DHW; a.seg_stride = (uint32_t)sample_delta;
  a.bt.wmod = groups; a.bt.stride = (size_t)per * sample_delta;
  SrcWgradImage b{};
  b.p = image->p; b.C = kz; b.H = image->y; b.W = image->x; b.KY = ky; b.KX = kx; b.OW = delta->x; b.OH = delta->y; b.R = ncol; b.K = per * DHW;
  b.sy = sy; b.sx = sx; b.py = py; b.px = px;
  b.bt.wmod = groups; b.bt.stride = (size_t)per * sample_image;
  Epilogue ep{};
  ep.inner = ncol; ep.g_stride = 0;
  if (groups > 1) {
    ep.C = partial; ep.row_stride = ncol; ep.bt.wmod = groups; ep.bt.stride = (size_t)ka * ncol;
  } else {
    ep.C = dk->p; ep.row_stride = dk->x; ep.accumulate = true;
  }
  if (DHW % 4 == 0 && ((uintptr_t)delta->p & 15u) == 0) {
    if (wgrad_image_fixed(ka, ncol, groups, delta, image, kz, per, px, py)) {
      SrcWgradImageFixed bf{};
      bf.p = b.p; bf.C = b.C; bf.H = b.H; bf.W = b.W; bf.KY = b.KY; bf.KX = b.KX; bf.OW = b.OW; bf.OH = b.OH; bf.R = b.R; bf.K = b.K;
      bf.sy = sy; bf.sx = sx; bf.py = py; bf.px = px; bf.bt = b.bt;
      rc = launch(name, a, bf, ep, ka, ncol, per * DHW, groups);
    } else {
      rc = launch(name, a, b, ep, ka, ncol, per * DHW, groups);
    }
  } else {
    SrcRowK<false> as{};
    as.p = a.p; as.ld = a.ld; as.R = a.R; as.K = a.K; as.seg = a.seg; as.seg_stride = a.seg_stride; as.bt = a.bt;
    rc = launch(name, as, b, ep, ka, ncol, per * DHW, groups);
  }
  if (rc) return rc;
  if (groups > 1) {
    mt_tensor pt{partial, groups, 1, ka, ncol}, flat{dk->p, 1, 1, ka, ncol};
    if ((rc = mt_add_sum_w(&flat, &flat, &pt, 1.f, 1.f))) return rc;
  }
  return dbias_batch_sum(name, db->p, dbias_partial, delta->p, B, ka, DHW, chunks);
}

// ---- nearest-neighbour up-sampling x2 followed by a 3x3 convolution (stride 1, padding 1), without the up-sampled image --
// Output row 2q reads up-sampled rows 2q-1, 2q, 2q+1 = input rows q-1, q, q; output row 2q+1 reads input rows q, q, q+1.
// So each of the four output phases (row parity, column parity) is a 2x2 convolution of the input itself, with
// coefficients that are sums of the 3x3 ones: 4 taps instead of 9, and the up-sampled image (four times the input)
// is neither written nor read.  This is the phase structure of a transposed convolution 4x4 stride 2 padding 1, so the
// same kernel runs it.  Rows outside the up-sampled image are rows outside the input: the zero padding carries over.
// One thread per (co, ci): packed[phase][co][ci*4 + ty*2 + tx] = sum of w[co][ci][ky][kx] over ky in Y(phase_y, ty),
// kx in X(phase_x, tx), with  (parity 0: tap 0 = {0}, tap 1 = {1, 2};  parity 1: tap 0 = {0, 1}, tap 1 = {2}).
__global__ __launch_bounds__(256) void upconv_prepare_kernel(float *packed, const float *kernel, uint32_t ker_ld, uint32_t CO, uint32_t CI) {
  const uint32_t ci = blockIdx.x * 256 + threadIdx.x, co = blockIdx.y;
  if (ci >= CI) return;
  float w[3][3];
#pragma unroll
  for (int i = 0; i < 9; i++) w[i / 3][i % 3] = kernel[(size_t)co * ker_ld + ci * 9 + i];
  // rows summed per (parity, tap): r[parity][tap][kx]
  float r[2][2][3];
#pragma unroll
  for (int x = 0; x < 3; x++) {
    r[0][0][x] = w[0][x]; r[0][1][x] = w[1][x] + w[2][x];
    r[1][0][x] = w[0][x] + w[1][x]; r[1][1][x] = w[2][x];
  }
  const uint32_t ld = CI * 4;
#pragma unroll
  for (int py = 0; py < 2; py++)
#pragma unroll
    for (int px = 0; px < 2; px++) {
      float4 q;
      const float(&a)[3] = r[py][0], (&b)[3] = r[py][1];
      if (px == 0) q = make_float4(a[0], a[1] + a[2], b[0], b[1] + b[2]);
      else q = make_float4(a[0] + a[1], a[2], b[0] + b[1], b[2]);
      *reinterpret_cast<float4 *>(packed + ((size_t)(py * 2 + px) * CO + co) * ld + ci * 4) = q;
    }
}

int upsampling_convolution(const char *name, const mt_tensor *out, const mt_tensor *image, uint32_t ux, uint32_t uy, const mt_tensor *kernel, int32_t kx,
                           int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func) {
  if (mt::bad(out) || mt::bad(image) || mt::bad(kernel) || mt::bad(bias)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(out);
  if (ux == 0 || uy == 0) return mt::fail(MT_E_ARGUMENT, "%s: up-sampling factors must be positive", name);
  if ((uint64_t)image->y * uy > 0x7fffffffu || (uint64_t)image->x * ux > 0x7fffffffu) return mt::fail(MT_E_ARGUMENT, "%s: image too large", name);
  const mt_tensor up_shape{image->p, image->w, image->z, image->y * uy, image->x * ux};  // sizes only: the pointer is not used
  int rc = check_forward(name, out, &up_shape, kernel, kx, ky, kz, ka, bias, sx, sy, px, py);
  if (rc) return rc;
  if (mt::count(out) == 0) return MT_OK;
  if (image->w == 0 || bias->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  const uint32_t K = (uint32_t)kz * kx * ky;
  if ((rc = check_kernel_tensor(name, kernel, ka, K))) return rc;
  const bool phases = ux == 2 && uy == 2 && kx == 3 && ky == 3 && sx == 1 && sy == 1 && px == 1 && py == 1 && kernel->w == 1 && bias->w == 1 &&
                      image->w == out->w && g_conv_path != 1 && mt::fits_buffer(image) && kz <= 0x0fffffff / 16;
  if (!phases) {
    // any other geometry: the two layers one after the other, the up-sampled image in the workspace behind the
    // region the convolution may use for re-ordered weights
    const size_t head = ((size_t)ka * K + 63) & ~(size_t)63;
    float *ws = nullptr;
    if ((rc = workspace(head + mt::count(&up_shape), &ws))) return rc;
    mt_tensor up = up_shape;
    up.p = ws + head;
    if ((rc = mt_upsampling(&up, image, ux, uy))) return rc;
    return forward(name, out, &up, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func);
  }
  const uint32_t ld = (uint32_t)kz * 4;
  float *packed = nullptr;
  bool fresh = true;
  if ((rc = pack_buffer(pack_key(2, kernel, nullptr, {kz, (int32_t)ka}), (size_t)4 * ka * ld, &packed, &fresh))) return rc;
  if (fresh) {
    mt::ProfileScope prof("upconv_prepare");
    upconv_prepare_kernel<<<dim3(cdiv((uint32_t)kz, 256), ka), 256, 0, mt::stream()>>>(packed, kernel->p, kernel->x, ka, (uint32_t)kz);
    MT_LAUNCH_CHECK("upconv_prepare");
  }
  TconvArgs args{};
  uint32_t max_n = 0;
  for (int32_t phy = 0; phy < 2; phy++) {
    const Phase1D Y = phase_1d(phy, 4, 2, 1, out->y);
    for (int32_t phx = 0; phx < 2; phx++) {
      const Phase1D X = phase_1d(phx, 4, 2, 1, out->x);
      const uint32_t f = args.nphase++;
      args.ph[f] = TconvPhase{packed + (size_t)(phy * 2 + phx) * ka * ld, ld, ld, (uint32_t)Y.q, (uint32_t)X.q, Y.taps, X.taps, Y.off, X.off, (uint32_t)phy, (uint32_t)phx};
      const uint32_t n = out->w * Y.q * X.q;
      if (n > max_n) max_n = n;
    }
  }
  const uint32_t OHW = out->y * out->x;
  args.M = ka; args.out_w = out->w;
  args.delta = image->p; args.in_w = image->w; args.C = kz; args.H = image->y; args.W = image->x;
  args.ep.C = out->p; args.ep.row_stride = OHW; args.ep.g_stride = (size_t)ka * OHW;
  args.ep.sy = 2; args.ep.sx = 2; args.ep.OW = out->x;
  args.ep.bias = bias->p; args.ep.bias_mode = 1; args.ep.bias_w = 1; args.ep.bias_stride = 0;
  args.ep.IH = image->y; args.ep.IW = image->x;
  const bool func_later = !mt::epilogue_func(func);
  args.ep.func = func_later ? MT_F_NONE : func;
  if (g_upconv_walk) {
    // the same four phases on the kernel whose blocks walk over the batch, where the shape allows (see mt_walk.h)
    mt::igemm::WalkArgs walk{};
    walk.nphase = args.nphase;
    for (uint32_t f = 0; f < args.nphase; f++) walk.ph[f] = args.ph[f];
    walk.M = ka; walk.batch = out->w; walk.delta = image->p; walk.C = (uint32_t)kz; walk.H = image->y; walk.W = image->x;
    walk.out = out->p; walk.OW = out->x; walk.OHW = OHW; walk.sy = 2; walk.sx = 2;
    walk.row_bias = bias->p; walk.tap_bias = nullptr; walk.func = args.ep.func;
    walk.wide = g_walk_wide && ka % 64 != 0 && ka % 32 == 0 ? 1u : 0u;   // 32 filters (or 96, ...): blocks of 32 rows x 128 columns
    if (mt::igemm::tconv_walk_plan(walk, (uint32_t)mt::igemm::walk_blocks(), 1) || mt::igemm::tconv_walk_plan_flat(walk)) {
      // too few tiles for the chip (small images, many channels): two or four blocks share a tile's k steps, their sums
      // are added afterwards together with the bias and the function
      const size_t blocks = (size_t)walk.nphase * walk.tiles_m * walk.qtiles * walk.groups;
      uint32_t share = 1;
      if (g_upconv_split && walk.per == 1 && blocks < 512 && mt::count(out) <= (1u << 22))
        while (share < 4 && blocks * share < 512 && walk.nk % (4 * share) == 0 && walk.nk / (2 * share) >= 8) share *= 2;
      if (share > 1) {
        float *partial = nullptr;
        if ((rc = mt::split_workspace((size_t)share * mt::count(out), &partial))) return rc;
        walk.ksplit = share; walk.nk /= share; walk.split_stride = mt::count(out);
        walk.out = partial; walk.row_bias = nullptr; walk.func = MT_F_NONE;
        mt::ProfileScope prof(mt::profiling() ? shape_label(name, walk.wide ? T32x128 : T64x64, ka, out->w * args.ph[0].qh * args.ph[0].qw, walk.nk * mt::igemm::BK, args.nphase * share) : name);
        if ((rc = mt::igemm::launch_tconv_walk(name, walk, false, false, 1))) return rc;
        return mt::split_reduce(name, out->p, partial, share, mt::count(out), bias->p, OHW, ka, func);
      }
      if (blocks >= (size_t)g_upconv_walk) {
        {
          mt::ProfileScope prof(mt::profiling() ? shape_label(name, walk.wide ? T32x128 : T64x64, ka, out->w * args.ph[0].qh * args.ph[0].qw, args.ph[0].kp, args.nphase) : name);
          if ((rc = mt::igemm::launch_tconv_walk(name, walk, false, false, 1))) return rc;
        }
        return func_later ? mt_apply_func(out, out, func) : MT_OK;
      }
    }
  }
  rc = launch_tconv(name, args, max_n, mt::count(out));
  return rc == MT_OK && func_later ? mt_apply_func(out, out, func) : rc;
}

}  // namespace

namespace mt {
namespace igemm {
int &tile_override() {
  static int v = -1;
  return v;
}
int &patch_blocks() {
  static int v = 512;
  return v;
}
int &walk_blocks() {
  static int v = 1024;
  return v;
}
int &walk_waves() {
  static int v = 4;
  return v;
}
int &walk_tm() {
  static int v = 1;
  return v;
}
int &walk_order() {
  static int v = -1;
  return v;
}
int &igemm_fair() {
  static int v = -1;
  return v;
}
int &walk_fair() {
  static int v = 0x842;
  return v;
}
}  // namespace igemm
void note_write(const void *p, size_t bytes) {
  if (p == nullptr || bytes == 0) return;
  const uintptr_t lo = (uintptr_t)p, hi = lo + bytes < lo ? ~(uintptr_t)0 : lo + bytes;
  if (g_pack_cache && !g_graph_writes_anything && capturing()) {  // a replay will write this range unseen
    bool known = false;
    for (const auto &r : g_graph_written) known = known || (r.first <= lo && hi <= r.second);
    if (!known) {
      if (g_graph_written.size() >= GRAPH_WRITTEN_MAX) g_graph_writes_anything = true;
      else g_graph_written.emplace_back(lo, hi);
    }
  }
  for (PackEntry &e : g_packs) {
    if (!e.valid) continue;
    if (overlaps(e.key.kernel, key_floats(e.key.kernel_dims), lo, hi) || overlaps(e.key.bias, key_floats(e.key.bias_dims), lo, hi)) e.valid = false;
  }
}
// The kept re-ordered copy of the weights at `kernel` that mt_adam_many can write while it updates them, if there is one:
// a 4x4 stride-2 transposed convolution's, not while a graph is recorded (a replay would write a copy that the cache
// cannot vouch for) and not for weights that a recorded graph writes.
bool pack_refresh_find(const float *kernel, size_t floats, PackRefresh *r) {
  if (!g_pack_cache || !g_pack_refresh || capturing()) return false;
  for (size_t i = 0; i < g_packs.size(); i++) {
    const PackEntry &e = g_packs[i];
    if (e.key.kind != 0 || !e.valid || !e.k4s2.on || e.key.kernel != kernel || key_floats(e.key.kernel_dims) != floats || floats != (size_t)e.k4s2.CI * e.k4s2.CO * 16u) continue;
    if (written_by_a_graph(e.key)) continue;
    r->packed = e.buf + e.k4s2.sums; r->ker_ld = e.k4s2.CO * 16u; r->co_stride = e.k4s2.co_stride; r->ci_stride = e.k4s2.ci_stride; r->entry = i;
    for (int f = 0; f < 4; f++) { r->begin[f] = e.k4s2.begin[f]; r->phase_of[f] = e.k4s2.phase_of[f]; }
    return true;
  }
  return false;
}
// After the launch that wrote the copy (and after the write to the weights was reported, which marked the entry stale):
// the copy is current again unless the same step also wrote the bias whose sums the entry holds.
void pack_refresh_commit(const PackRefresh &r, const mt_tensor *const *weight, const mt_tensor *const *m, const mt_tensor *const *v, uint32_t count) {
  if (r.entry >= g_packs.size()) return;
  PackEntry &e = g_packs[r.entry];
  for (const mt_tensor *const *written : {weight, m, v})
    for (uint32_t i = 0; i < count; i++) {
      const uintptr_t lo = (uintptr_t)written[i]->p, hi = lo + mt::count(written[i]) * sizeof(float);
      if (overlaps(e.key.bias, key_floats(e.key.bias_dims), lo, hi)) return;
      if (written != weight && overlaps(e.key.kernel, key_floats(e.key.kernel_dims), lo, hi)) return;  // (moments that alias the weights: nothing to vouch for)
    }
  e.valid = true;
  g_pack_refreshed++;
}
// A block goes back to the pool or the driver (not under capture): what recorded graphs write into it no longer matters
// to the cache.  Replaying such a graph now would write into whoever owns the block next -- the caller's error, as
// with any use of freed memory -- so nothing recorded can change what the next owner keeps there, and copies made of the
// next owner's weights can be trusted again.
void forget_graph_writes(const void *p, size_t bytes) {
  if (p == nullptr || bytes == 0 || g_graph_written.empty()) return;
  const uintptr_t lo = (uintptr_t)p, hi = lo + bytes < lo ? ~(uintptr_t)0 : lo + bytes;
  size_t kept = 0;
  for (size_t i = 0; i < g_graph_written.size(); i++)
    if (!(lo <= g_graph_written[i].first && g_graph_written[i].second <= hi)) g_graph_written[kept++] = g_graph_written[i];
  g_graph_written.resize(kept);
}
int set_pack_refresh(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "pack_refresh must be 0 or 1");
  g_pack_refresh = v;
  return MT_OK;
}
int set_pack_cache(int on) {
  if (on != 0 && on != 1) return fail(MT_E_ARGUMENT, "pack_cache must be 0 (re-order the weights on every call) or 1 (keep them between calls)");
  g_pack_cache = on != 0;
  if (!g_pack_cache && !g_packs.empty()) {
    MT_HIP(hipStreamSynchronize(stream()));
    while (!g_packs.empty()) drop_entry(g_packs.size() - 1);
  }
  return MT_OK;
}
bool pack_cache_info(const char *name, int64_t *value) {
  if (strcmp(name, "pack_cache_entries") == 0) { *value = (int64_t)g_packs.size(); return true; }
  if (strcmp(name, "pack_cache_valid") == 0) { int64_t n = 0; for (const PackEntry &e : g_packs) n += e.valid; *value = n; return true; }
  if (strcmp(name, "pack_cache_hits") == 0) { *value = (int64_t)g_pack_hits; return true; }
  if (strcmp(name, "pack_cache_made") == 0) { *value = (int64_t)g_pack_made; return true; }
  if (strcmp(name, "pack_cache_refreshed") == 0) { *value = (int64_t)g_pack_refreshed; return true; }
  if (strcmp(name, "pack_cache_bytes") == 0) { int64_t n = 0; for (const PackEntry &e : g_packs) n += (int64_t)(e.floats * sizeof(float)); *value = n; return true; }
  if (strcmp(name, "pack_cache_spare_bytes") == 0) { int64_t n = 0; for (const PackEntry &e : g_pack_spare) n += (int64_t)(e.floats * sizeof(float)); *value = n; return true; }
  if (strcmp(name, "graph_written_ranges") == 0) { *value = (int64_t)g_graph_written.size(); return true; }
  if (strcmp(name, "graph_writes_anything") == 0) { *value = g_graph_writes_anything ? 1 : 0; return true; }
  if (strcmp(name, "convolution_workspace_bytes") == 0) { *value = (int64_t)(g_ws.floats * sizeof(float)); return true; }
  if (strcmp(name, "wgrad_walk_launches") == 0) { *value = (int64_t)g_wgrad_walk_launches; return true; }
  if (strcmp(name, "wgrad_patch_launches") == 0) { *value = (int64_t)g_wgrad_patch_launches; return true; }
  if (strcmp(name, "conv_patch_launches") == 0) { *value = (int64_t)g_conv_patch_launches; return true; }
  if (strcmp(name, "tconv_as_conv_launches") == 0) { *value = (int64_t)g_tconv_as_conv_launches; return true; }
  if (strcmp(name, "tconv_merge_launches") == 0) { *value = (int64_t)g_tconv_merge_launches; return true; }
  if (strcmp(name, "tconv_patch_launches") == 0) { *value = (int64_t)g_tconv_patch_launches; return true; }
  return false;
}
int set_image_strip(int v) {
  if (v < 0 || v > 14) return fail(MT_E_ARGUMENT, "image_strip must be 0 (choose) or 1..14 rows");
  g_image_strip = v;
  return MT_OK;
}
int set_image_mfma(int v) {
  if (v < 0 || v > 2) return fail(MT_E_ARGUMENT, "image_mfma must be 0, 1 or 2");
  g_image_mfma = v;
  return MT_OK;
}
int set_tconv_walk(int v) {
  if (v < 0 || v > 1) return fail(MT_E_ARGUMENT, "tconv_walk must be 0 (never for plain calls) or 1 (wherever the shape allows)");
  g_tconv_walk = v;
  return MT_OK;
}
int set_first_layer(int v) {
  if (v < 0 || v > 1) return fail(MT_E_ARGUMENT, "first_layer must be 0 (never) or 1 (wherever the shape allows)");
  g_first_layer = v;
  return MT_OK;
}
int set_conv_walk(int v) {
  if (v < 0 || v > 2) return fail(MT_E_ARGUMENT, "conv_walk must be 0 (never), 1 (wherever the shape allows and the grid fills the chip) or 2 (wherever the shape allows)");
  g_conv_walk = v;
  return MT_OK;
}
int set_walk_blocks(int v) {
  if (v < 1 || v > 65536) return fail(MT_E_ARGUMENT, "walk_blocks must be 1..65536");
  igemm::walk_blocks() = v;
  return MT_OK;
}
int set_walk_order(int v) {
  if (v < -1 || v > 1) return fail(MT_E_ARGUMENT, "walk_order must be -1 (per layer), 0 (batch groups first) or 1 (row tiles first)");
  igemm::walk_order() = v;
  return MT_OK;
}
int set_walk_fair(int v) {
  if (v < 0 || v > 0xfff) return fail(MT_E_ARGUMENT, "walk_fair must be 0 or three hexadecimal digits (sixteenths of a block's steps)");
  igemm::walk_fair() = v;
  return MT_OK;
}
int set_igemm_fair(int v) {
  if (v < -1 || v > 0xfff) return fail(MT_E_ARGUMENT, "igemm_fair must be -1 (per launch), 0 or three hexadecimal digits (sixteenths of a block's steps)");
  igemm::igemm_fair() = v;
  return MT_OK;
}
int set_walk_tm(int v) {
  if (v != 1 && v != 2) return fail(MT_E_ARGUMENT, "walk_tm must be 1 or 2");
  igemm::walk_tm() = v;
  return MT_OK;
}
int set_walk_waves(int v) {
  if (v != 4 && v != 5) return fail(MT_E_ARGUMENT, "walk_waves must be 4 or 5");
  igemm::walk_waves() = v;
  return MT_OK;
}
int set_patch_blocks(int v) {
  if (v < 1 || v > 65536) return fail(MT_E_ARGUMENT, "patch_blocks must be 1..65536");
  igemm::patch_blocks() = v;
  return MT_OK;
}
int set_igemm_tile(int v) {
  if (v < -1 || v > 4) return fail(MT_E_ARGUMENT, "igemm_tile must be -1 (auto) or 0..4");
  igemm::tile_override() = v;
  return MT_OK;
}
int set_walk_wide(int v) {
  if (v < 0 || v > 1) return fail(MT_E_ARGUMENT, "walk_wide must be 0 or 1");
  g_walk_wide = v;
  return MT_OK;
}
int set_upconv_split(int v) {
  if (v < 0 || v > 1) return fail(MT_E_ARGUMENT, "upconv_split must be 0 (never) or 1 (where too few tiles would fill the chip)");
  g_upconv_split = v;
  return MT_OK;
}
int set_upconv_walk(int v) {
  if (v < 0) return fail(MT_E_ARGUMENT, "upconv_walk must be 0 (never) or the number of blocks from which the walking kernel is taken");
  g_upconv_walk = v;
  return MT_OK;
}
int set_conv_patch(int v) {
  if (v < 0 || v > 64) return fail(MT_E_ARGUMENT, "conv_patch must be 0 (never), 1 (from 5 filters on) or the smallest number of filters (2..64)");
  g_conv_patch = v != 0;
  g_conv_patch_min = v <= 1 ? 5 : v;
  return MT_OK;
}
int set_tconv_as_conv(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "tconv_as_conv must be 0 or 1");
  g_tconv_as_conv = v;
  return MT_OK;
}
int set_tconv_merge(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "tconv_merge must be 0 or 1");
  g_tconv_merge = v;
  return MT_OK;
}
int set_tconv_patch(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "tconv_patch must be 0 or 1");
  g_tconv_patch = v;
  return MT_OK;
}
int set_wgrad_patch(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "wgrad_patch must be 0 or 1");
  g_wgrad_patch = v;
  return MT_OK;
}
int set_wgrad_pad(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "wgrad_pad must be 0 or 1");
  g_wgrad_pad = v;
  return MT_OK;
}
int set_wgrad_parts(int v) {
  if (v < 0 || v > 256) return fail(MT_E_ARGUMENT, "wgrad_parts must be 0 (never), 1 (choose) or the number of bands per sample (2..256)");
  g_wgrad_parts = v;
  return MT_OK;
}
int set_wgrad_walk(int v) {
  if (v != 0 && v != 1) return fail(MT_E_ARGUMENT, "wgrad_walk must be 0 or 1");
  g_wgrad_walk = v;
  return MT_OK;
}

int set_wgrad_groups(int v) {
  if (v < 0) return fail(MT_E_ARGUMENT, "wgrad_groups must be 0 (auto) or a positive divisor of the batch");
  g_wgrad_groups = v;
  return MT_OK;
}
int set_conv_path(int v) {
  if (v < 0 || v > 2) return fail(MT_E_ARGUMENT, "conv_path must be 0 (auto), 1 (direct) or 2 (matrix cores)");
  g_conv_path = v;
  return MT_OK;
}
}  // namespace mt

extern "C" {

int mt_forward_convolution(const mt_tensor *out, const mt_tensor *image, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz, uint32_t ka,
                           const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  return forward("mt_forward_convolution", out, image, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, MT_F_NONE);
}

int mt_forward_convolution_func(const mt_tensor *out, const mt_tensor *image, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz, uint32_t ka,
                                const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func) {
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "mt_forward_convolution_func: unknown function id %d", func);
  return forward("mt_forward_convolution_func", out, image, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func);
}

int mt_upsampling_convolution_func(const mt_tensor *out, const mt_tensor *image, uint32_t ux, uint32_t uy, const mt_tensor *kernel, int32_t kx, int32_t ky,
                                   int32_t kz, uint32_t ka, const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func) {
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "mt_upsampling_convolution_func: unknown function id %d", func);
  return upsampling_convolution("mt_upsampling_convolution_func", out, image, ux, uy, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func);
}

int mt_backward_convolution(const mt_tensor *out, const mt_tensor *delta, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz, uint32_t ka,
                            const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  return backward("mt_backward_convolution", out, delta, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, MT_F_NONE);
}

int mt_backward_convolution_func(const mt_tensor *out, const mt_tensor *delta, const mt_tensor *kernel, int32_t kx, int32_t ky, int32_t kz, uint32_t ka,
                                 const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func) {
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "mt_backward_convolution_func: unknown function id %d", func);
  return backward("mt_backward_convolution_func", out, delta, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func);
}

int mt_backward_convolution_norm_func(const mt_tensor *out, const mt_tensor *delta, const mt_tensor *delta_scale_shift, int delta_func, const mt_tensor *kernel,
                                      int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py, int func) {
  if (!mt::valid_func(func, true) || !mt::valid_func(delta_func, true)) return mt::fail(MT_E_ARGUMENT, "mt_backward_convolution_norm_func: unknown function id");
  return backward_between_norms("mt_backward_convolution_norm_func", out, delta, delta_scale_shift, delta_func, kernel, kx, ky, kz, ka, bias, sx, sy, px, py, func, nullptr);
}

int mt_backward_convolution_norm_stats(const mt_tensor *out, const mt_tensor *delta, const mt_tensor *delta_scale_shift, int delta_func, const mt_tensor *kernel,
                                       int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py,
                                       const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *scale_shift, const mt_tensor *ivar,
                                       const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean, const mt_tensor *new_variable,
                                       float momentum, float epsilon) {
  if (!mt::valid_func(delta_func, true)) return mt::fail(MT_E_ARGUMENT, "mt_backward_convolution_norm_stats: unknown function id %d", delta_func);
  const BnOut bn{gamma, beta, scale_shift, ivar, batch_mean, batch_var, new_mean, new_variable, momentum, epsilon};
  return backward_between_norms("mt_backward_convolution_norm_stats", out, delta, delta_scale_shift, delta_func, kernel, kx, ky, kz, ka, bias, sx, sy, px, py,
                                MT_F_NONE, &bn);
}

int mt_create_delta_weight_and_bias(const mt_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *db, const mt_tensor *image,
                                    const mt_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  return wgrad("mt_create_delta_weight_and_bias", dk, kx, ky, kz, ka, db, image, delta, sx, sy, px, py, true);
}

int mt_convolution_backward_weights_sum(const mt_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *db, const mt_tensor *image,
                                        const mt_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  return wgrad_batch_sum("mt_convolution_backward_weights_sum", dk, kx, ky, kz, ka, db, image, delta, sx, sy, px, py);
}

// the transposed layer: image and delta trade places, and the bias gradient is cleared (cpu/ctensorconv.h:393-397)
int mt_create_back_delta_weight_and_bias(const mt_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, const mt_tensor *db, const mt_tensor *image,
                                         const mt_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py) {
  int rc = wgrad("mt_create_back_delta_weight_and_bias", dk, kx, ky, kz, ka, db, delta, image, sx, sy, px, py, false);
  if (rc) return rc;
  return mt_fill(db, 0.f);
}

}  // extern "C"
