// HBM-bound part of the tensor-op path for gfx950: elementwise ops, reductions over the batch axis
// and over Y*X, resampling, pooling, Adam and the activation functions.
//
// Layout rule shared by every kernel here: the output is walked as [W][S] with S = Z*Y*X;
// blockIdx.y is the output layer w, so a broadcast operand (w % W_operand) costs no per-element
// division, and threads along blockIdx.x/threadIdx.x touch consecutive addresses (coalesced,
// 16-byte vectors when S and the pointers allow it).
#include <type_traits>
#include "mt_common.h"

namespace {

using mt::cdiv;

constexpr int EW_THREADS = 256;
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Tensors that are streamed once and exceed what the caches hold (4 MiB of L2 per XCD, 256 MiB of Infinity Cache) are
// read and written with non-temporal accesses: measured on 268 MB and 1 GB tensors, 2x2 up-sampling goes from 4.9 to
// 6.7 TB/s, max pooling backward from 5.1 to 6.7, max pooling from 5.2 to 6.2, down-sampling from 4.9 to 5.7.  Tensors that
// fit are left to the caches: the next kernel finds them there (max pooling of a 67 MB input: 6.6 TB/s, 5.6 when
// it is read past the caches).  The plain elementwise kernels (one contiguous store per thread) measured no difference
// and keep ordinary accesses.
int g_nontemporal = 2;   // 0 never, 1 always, 2 by size (default)
inline bool streamed(size_t bytes) { return g_nontemporal == 1 || (g_nontemporal == 2 && bytes >= ((size_t)128 << 20)); }

struct Operand {
  const float *p;
  uint32_t w;  // layers; layer used for output layer w is w % this
};

__device__ __forceinline__ const float *layer(const Operand &o, uint32_t w, size_t S) {
  return o.p + (size_t)(o.w == 1 ? 0u : w % o.w) * S;
}

// out[w][i] = f(a[w%Wa][i])
template <class F>
__global__ __launch_bounds__(EW_THREADS) void ew1_kernel(float *out, Operand a, uint32_t S, uint32_t W, bool vec, F f) {
  for (uint32_t w = blockIdx.y; w < W; w += gridDim.y) {
    const float *pa = layer(a, w, S);
    float *po = out + (size_t)w * S;
    uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
    if (vec) {
      if (i * 4 < S) {
        float4 v = reinterpret_cast<const float4 *>(pa)[i];
        v.x = f(v.x); v.y = f(v.y); v.z = f(v.z); v.w = f(v.w);
        reinterpret_cast<float4 *>(po)[i] = v;
      }
    } else if (i < S) {
      po[i] = f(pa[i]);
    }
  }
}

// out[w][i] = f(a[w%Wa][i], b[w%Wb][i])
template <class F>
__global__ __launch_bounds__(EW_THREADS) void ew2_kernel(float *out, Operand a, Operand b, uint32_t S, uint32_t W, bool vec, F f) {
  for (uint32_t w = blockIdx.y; w < W; w += gridDim.y) {
    const float *pa = layer(a, w, S), *pb = layer(b, w, S);
    float *po = out + (size_t)w * S;
    uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
    if (vec) {
      if (i * 4 < S) {
        float4 x = reinterpret_cast<const float4 *>(pa)[i], y = reinterpret_cast<const float4 *>(pb)[i], o;
        o.x = f(x.x, y.x); o.y = f(x.y, y.y); o.z = f(x.z, y.z); o.w = f(x.w, y.w);
        reinterpret_cast<float4 *>(po)[i] = o;
      }
    } else if (i < S) {
      po[i] = f(pa[i], pb[i]);
    }
  }
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }
// grid.y of the kernels that loop over planes: enough blocks to fill the machine, few enough that a thread's index
// arithmetic is spread over several planes
inline unsigned plane_blocks(unsigned blocks_x, uint32_t planes) {
  unsigned want = blocks_x >= 8192u ? 1u : 8192u / blocks_x;
  return planes < want ? planes : want;
}

template <class F>
int launch1(const char *name, const mt_tensor *out, const mt_tensor *in, F f) {
  if (mt::bad(out) || mt::bad(in)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(out);
  if (!mt::same_zyx(in, out)) return mt::fail(MT_E_SHAPE, "%s: Z/Y/X of input and output differ", name);
  size_t S = (size_t)out->z * out->y * out->x;
  if (S == 0 || out->w == 0) return MT_OK;
  if (in->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty input", name);
  bool vec = (S % 4 == 0) && aligned16(out->p) && aligned16(in->p);
  dim3 grid(cdiv(vec ? S / 4 : S, EW_THREADS), out->w < 65535u ? out->w : 65535u);
  mt::ProfileScope prof(name);
  ew1_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, Operand{in->p, in->w}, (uint32_t)S, out->w, vec, f);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

template <class F>
int launch2(const char *name, const mt_tensor *out, const mt_tensor *l, const mt_tensor *r, F f) {
  if (mt::bad(out) || mt::bad(l) || mt::bad(r)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(out);
  if (!mt::same_zyx(l, r) || !mt::same_zyx(out, r)) return mt::fail(MT_E_SHAPE, "%s: Z/Y/X of the operands differ", name);
  size_t S = (size_t)out->z * out->y * out->x;
  if (S == 0 || out->w == 0) return MT_OK;
  if (l->w == 0 || r->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  bool vec = (S % 4 == 0) && aligned16(out->p) && aligned16(l->p) && aligned16(r->p);
  dim3 grid(cdiv(vec ? S / 4 : S, EW_THREADS), out->w < 65535u ? out->w : 65535u);
  mt::ProfileScope prof(name);
  ew2_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, Operand{l->p, l->w}, Operand{r->p, r->w}, (uint32_t)S, out->w, vec, f);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

// ---- functors: arithmetic exactly as the CPU path writes it (no fused multiply-add: see the build flags) ----
struct FInv { __device__ float operator()(float i) const { return (float)(1.0 / (double)i); } };
struct FPow2 { float s; __device__ float operator()(float i) const { return i * i * s; } };
struct FSqrt { float s, add; __device__ float operator()(float i) const { return sqrtf(i + add) * s; } };
struct FScale { float v; __device__ float operator()(float i) const { return i * v; } };
struct FAffine { float s, add; __device__ float operator()(float i) const { return i * s + add; } };
struct FClip { float lo, hi; __device__ float operator()(float v) const { if (v < lo) v = lo; if (v > hi) v = hi; return v; } };
struct FSign { __device__ float operator()(float v) const { if (v < 0.f) v = -1.f; if (v > 0.f) v = 1.f; return v; } };
struct FFunc { int func; __device__ float operator()(float v) const { return mt::apply_func(func, v); } };
struct FAdd { float ls, rs; __device__ float operator()(float l, float r) const { return (ls * l) + (rs * r); } };
struct FSub { float ls, rs; __device__ float operator()(float l, float r) const { return (ls * l) - (rs * r); } };
struct FDiv { float ls, rs; __device__ float operator()(float l, float r) const { return (ls * l) / (rs * r); } };
struct FMul { __device__ float operator()(float l, float r) const { return l * r; } };

__global__ __launch_bounds__(EW_THREADS) void fill4_kernel(float4 *out, size_t n4, float v) {
  size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * EW_THREADS;
  const float4 q = make_float4(v, v, v, v);
  for (; i < n4; i += stride) out[i] = q;
}
__global__ __launch_bounds__(EW_THREADS) void fill_kernel(float *out, size_t n, float v) {
  size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;
  size_t stride = (size_t)gridDim.x * EW_THREADS;
  for (; i < n; i += stride) out[i] = v;
}

// ---- AddSumW: out[0][r] = ls*sum_w L[w][r] + rs*sum_w R[w][r], out[w>0][r] = 0 --------------------------------
// A block owns RB consecutive r and splits the batch axis over WS = 256/RB slices that are combined in LDS,
// so short tensors (S of a few thousand) still fill the chip and every load is coalesced along r.
template <int RB>
__global__ __launch_bounds__(EW_THREADS) void add_sum_w_kernel(float *out, uint32_t Wout, const float *L, uint32_t Wl, const float *R,
                                                               uint32_t Wr, uint32_t S, float ls, float rs) {
  constexpr int WS = EW_THREADS / RB;
  __shared__ float part[2][WS][RB];
  int rl = threadIdx.x % RB, ws = threadIdx.x / RB;
  uint32_t r = blockIdx.x * RB + rl;
  float sl = 0.f, sr = 0.f;
  if (r < S) {
    for (uint32_t w = ws; w < Wl; w += WS) sl += L[(size_t)w * S + r];
    for (uint32_t w = ws; w < Wr; w += WS) sr += R[(size_t)w * S + r];
  }
  part[0][ws][rl] = sl;
  part[1][ws][rl] = sr;
  __syncthreads();
  if (ws == 0 && r < S) {
    sl = 0.f; sr = 0.f;
#pragma unroll
    for (int i = 0; i < WS; i++) { sl += part[0][i][rl]; sr += part[1][i][rl]; }
    sl *= ls;
    sr *= rs;
    out[r] = sl + sr;
  }
  if (r < S)
    for (uint32_t w = 1 + ws; w < Wout; w += WS) out[(size_t)w * S + r] = 0.f;
}

// ---- SummXY: one wavefront per (w,z) row of Y*X elements ---------------------------------------------------------
__global__ __launch_bounds__(EW_THREADS) void summ_xy_kernel(float *out, const float *in, uint32_t Win, uint32_t Z, uint32_t YX, uint32_t rows) {
  uint32_t row = blockIdx.x * (EW_THREADS / 64) + threadIdx.x / 64;
  if (row >= rows) return;
  uint32_t w = row / Z, z = row % Z, lane = threadIdx.x % 64;
  const float *p = in + ((size_t)(w % Win) * Z + z) * YX;
  float s = 0.f;
  if (YX % 4 == 0 && ((uintptr_t)p & 15u) == 0) {  // 128-bit loads, four partial sums per lane
    float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
    for (uint32_t i = lane; i < YX / 4; i += 64) {
      const float4 v = reinterpret_cast<const float4 *>(p)[i];
      q.x += v.x; q.y += v.y; q.z += v.z; q.w += v.w;
    }
    s = (q.x + q.y) + (q.z + q.w);
  } else {
    for (uint32_t i = lane; i < YX; i += 64) s += p[i];
  }
  s = mt::wave_sum(s);
  if (lane == 0) out[row] = s;
}

// ---- AddBias: working[w][z][.] += bias[w%Wb][z] ------------------------------------------------------------------
// The same with 128-bit accesses: a block owns RB groups of four columns and splits the batch over WS = 256 / RB slices;
// the slice loops are unrolled so that several loads per thread are in flight.  Slices are combined inside a wavefront by
// lane exchanges (the lanes that differ above the column bits), the four wavefronts in LDS.  RB = 256 is one thread per
// group of columns, no exchange at all: tensors with few samples and many columns (two or eight partial weight gradients);
// RB = 4 gives 64 slices: few columns and many samples (hundreds of partial gradients of a first layer).
template <int RB>
__device__ __forceinline__ void add_sum_w_vec_body(uint32_t block, float *out, uint32_t Wout, const float *L, uint32_t Wl, const float *R, uint32_t Wr,
                                                   uint32_t S, float ls, float rs) {
  constexpr int WS = EW_THREADS / RB, WAVES = EW_THREADS / 64;
  constexpr int IN_WAVE = RB >= 64 ? 1 : 64 / RB;   // slices inside one wavefront
  __shared__ float4 part[2][WS > 1 ? WAVES : 1][RB < 64 ? RB : 64];
  const int rl = threadIdx.x % RB, ws = threadIdx.x / RB;
  const uint32_t r = (block * RB + rl) * 4;
  float4 sl = make_float4(0.f, 0.f, 0.f, 0.f), sr = sl;
  if (r < S) {
#pragma unroll 4
    for (uint32_t w = ws; w < Wl; w += WS) {
      const float4 q = *reinterpret_cast<const float4 *>(L + (size_t)w * S + r);
      sl.x += q.x; sl.y += q.y; sl.z += q.z; sl.w += q.w;
    }
#pragma unroll 8
    for (uint32_t w = ws; w < Wr; w += WS) {
      const float4 q = *reinterpret_cast<const float4 *>(R + (size_t)w * S + r);
      sr.x += q.x; sr.y += q.y; sr.z += q.z; sr.w += q.w;
    }
  }
  if constexpr (WS > 1) {
#pragma unroll
    for (int d = RB; d < RB * IN_WAVE; d <<= 1) {
      sl.x += __shfl_xor(sl.x, d, 64); sl.y += __shfl_xor(sl.y, d, 64); sl.z += __shfl_xor(sl.z, d, 64); sl.w += __shfl_xor(sl.w, d, 64);
      sr.x += __shfl_xor(sr.x, d, 64); sr.y += __shfl_xor(sr.y, d, 64); sr.z += __shfl_xor(sr.z, d, 64); sr.w += __shfl_xor(sr.w, d, 64);
    }
    static_assert(RB <= 64, "several slices: a wavefront holds whole slices");
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    if (lane < RB) { part[0][wave][lane] = sl; part[1][wave][lane] = sr; }
    __syncthreads();
    if (r >= S) return;
    if (ws == 0) {
      sl = make_float4(0.f, 0.f, 0.f, 0.f); sr = sl;
#pragma unroll
      for (int i = 0; i < WAVES; i++) {
        const float4 a = part[0][i][rl], b = part[1][i][rl];
        sl.x += a.x; sl.y += a.y; sl.z += a.z; sl.w += a.w;
        sr.x += b.x; sr.y += b.y; sr.z += b.z; sr.w += b.w;
      }
    }
  } else {
    if (r >= S) return;
  }
  if (ws == 0) {
    float4 o;
    o.x = sl.x * ls + sr.x * rs; o.y = sl.y * ls + sr.y * rs; o.z = sl.z * ls + sr.z * rs; o.w = sl.w * ls + sr.w * rs;
    *reinterpret_cast<float4 *>(out + r) = o;
  }
  for (uint32_t w = 1 + ws; w < Wout; w += WS) *reinterpret_cast<float4 *>(out + (size_t)w * S + r) = make_float4(0.f, 0.f, 0.f, 0.f);
}
template <int RB>
__global__ __launch_bounds__(EW_THREADS) void add_sum_w_vec_kernel(float *out, uint32_t Wout, const float *L, uint32_t Wl, const float *R, uint32_t Wr,
                                                                   uint32_t S, float ls, float rs) {
  add_sum_w_vec_body<RB>(blockIdx.x, out, Wout, L, Wl, R, Wr, S, ls, rs);
}
// Two sums in one launch, out[i] += sum over w of R[w][i] for each: the first `blocks` blocks own the first one.  (The
// partial weight gradients of a layer and the partial sums of its bias gradient: the second is too small for a launch of
// its own to be worth its start.)
struct SumJob {
  float *out;
  const float *R;
  uint32_t S, blocks;
};
template <int RB>
__global__ __launch_bounds__(EW_THREADS) void add_sum_w_pair_kernel(SumJob a, SumJob b, uint32_t W) {
  const bool first = blockIdx.x < a.blocks;  // (uniform over the block: the barrier inside the body is reached by all of its threads)
  const SumJob &j = first ? a : b;
  add_sum_w_vec_body<RB>(first ? blockIdx.x : blockIdx.x - a.blocks, j.out, 1, j.out, 1, j.R, W, j.S, 1.f, 1.f);
}

__global__ __launch_bounds__(EW_THREADS) void add_bias4_kernel(float *t, const float *bias, uint32_t Wb, uint32_t Z, uint32_t YX4, uint32_t rows) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
  if (i >= YX4) return;
  for (uint32_t row = blockIdx.y; row < rows; row += gridDim.y) {
    const uint32_t w = row / Z, z = row % Z;
    const float b = bias[(size_t)(w % Wb) * Z + z];
    float4 *p = reinterpret_cast<float4 *>(t + (size_t)row * YX4 * 4) + i;
    float4 q = *p;
    q.x += b; q.y += b; q.z += b; q.w += b;
    *p = q;
  }
}
__global__ __launch_bounds__(EW_THREADS) void add_bias_kernel(float *t, const float *bias, uint32_t Wb, uint32_t Z, uint32_t YX, uint32_t rows) {
  for (uint32_t row = blockIdx.y; row < rows; row += gridDim.y) {
    uint32_t w = row / Z, z = row % Z;
    float b = bias[(size_t)(w % Wb) * Z + z];
    uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
    if (i < YX) t[(size_t)row * YX + i] += b;
  }
}

// ---- Transponse ---------------------------------------------------------------------------------------------------
__global__ void transponse_kernel(float *out, const float *in, uint32_t Y, uint32_t X) {
  __shared__ float tile[32][33];
  const float *pi = in + (size_t)blockIdx.z * Y * X;
  float *po = out + (size_t)blockIdx.z * Y * X;
  uint32_t x = blockIdx.x * 32 + threadIdx.x;
  for (int j = threadIdx.y; j < 32; j += 8) {
    uint32_t y = blockIdx.y * 32 + j;
    if (x < X && y < Y) tile[j][threadIdx.x] = pi[(size_t)y * X + x];
  }
  __syncthreads();
  uint32_t oy = blockIdx.y * 32 + threadIdx.x;  // becomes the fast index of the output
  for (int j = threadIdx.y; j < 32; j += 8) {
    uint32_t ox = blockIdx.x * 32 + j;
    if (ox < X && oy < Y) po[(size_t)ox * Y + oy] = tile[threadIdx.x][j];
  }
}

// ---- resampling and pooling: one thread per output element, x fastest ---------------------------------------------
struct Geo {
  uint32_t Win, Z, iy, ix, oy, ox;  // input layers, depth, input / output rows and columns
};

__global__ __launch_bounds__(EW_THREADS) void upsampling_kernel(float *out, const float *in, Geo g, uint32_t ux, uint32_t uy, uint32_t planes) {
  uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, n = g.oy * g.ox;
  if (i >= n) return;
  uint32_t y = i / g.ox, x = i % g.ox, sy = y / uy, sx = x / ux;
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    uint32_t w = pl / g.Z, z = pl % g.Z;
    float v = 0.f;
    if (sx < g.ix && sy < g.iy) v = in[(((size_t)(w % g.Win) * g.Z + z) * g.iy + sy) * g.ix + sx];
    out[(size_t)pl * n + i] = v;
  }
}

// Four consecutive output columns per thread (one 128-bit store); ox is a multiple of 4, the input is not empty.
// Source indices are clamped into the input and the out-of-range columns zeroed afterwards, so the loads carry no
// condition and four planes are in flight per thread.
__global__ __launch_bounds__(EW_THREADS) void upsampling4_kernel(float *out, const float *in, Geo g, uint32_t ux, uint32_t uy, uint32_t planes) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, ox4 = g.ox / 4, n4 = g.oy * ox4;
  if (i >= n4) return;
  const uint32_t y = i / ox4, x = (i % ox4) * 4, sy = y / uy;
  const uint32_t syc = sy < g.iy ? sy : g.iy - 1;
  uint32_t sx[4];
  bool ok[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t c = (x + k) / ux;
    ok[k] = sy < g.iy && c < g.ix;
    sx[k] = c < g.ix ? c : g.ix - 1;
  }
  const size_t plane_in = (size_t)g.iy * g.ix, plane_out = (size_t)g.oy * g.ox;
  const bool same_w = g.Win * g.Z == planes;  // no broadcast over the batch: plane pl of the input
#pragma unroll 4
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const uint32_t ipl = same_w ? pl : (pl / g.Z % g.Win) * g.Z + pl % g.Z;
    const float *src = in + (size_t)ipl * plane_in + (size_t)syc * g.ix;
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = src[sx[k]];
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = ok[k] ? v[k] : 0.f;
    reinterpret_cast<float4 *>(out + (size_t)pl * plane_out)[i] = make_float4(v[0], v[1], v[2], v[3]);
  }
}
// x2 in both directions, output exactly twice the input, even input width: a thread reads two input pixels (64 bits)
// and writes their 2x4 output pixels as two 128-bit stores; the same index map, without divisions.
template <bool NT>
__global__ __launch_bounds__(EW_THREADS) void upsampling2x2_kernel(float *out, const float *in, Geo g, uint32_t planes) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, ix2 = g.ix / 2, n2 = g.iy * ix2;
  if (i >= n2) return;
  const uint32_t y = i / ix2, x2 = i % ix2;
  const size_t plane_in = (size_t)g.iy * g.ix, plane_out = (size_t)g.oy * g.ox;
  const size_t o0 = (size_t)(2 * y) * g.ox + 4 * x2;
  const bool same_w = g.Win * g.Z == planes;
#pragma unroll 4
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const uint32_t ipl = same_w ? pl : (pl / g.Z % g.Win) * g.Z + pl % g.Z;
    const float2 v = reinterpret_cast<const float2 *>(in + (size_t)ipl * plane_in)[i];
    const floatx4 q = {v.x, v.x, v.y, v.y};
    float *dst = out + (size_t)pl * plane_out + o0;
    if constexpr (NT) {  // an output beyond what the caches hold: written once, not kept
      __builtin_nontemporal_store(q, reinterpret_cast<floatx4 *>(dst));
      __builtin_nontemporal_store(q, reinterpret_cast<floatx4 *>(dst + g.ox));
    } else {
      *reinterpret_cast<floatx4 *>(dst) = q;
      *reinterpret_cast<floatx4 *>(dst + g.ox) = q;
    }
  }
}
__global__ __launch_bounds__(EW_THREADS) void max_pooling_backward4_kernel(float *out, const mt_spos *pos, uint32_t Wpos, const float *in, Geo g, uint32_t px_, uint32_t py_, uint32_t planes) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, ox4 = g.ox / 4, n4 = g.oy * ox4;
  if (i >= n4) return;
  const uint32_t y = i / ox4, x = (i % ox4) * 4, sy = y / py_;
  const uint32_t syc = sy < g.iy ? sy : g.iy - 1;
  uint32_t sx[4];
  bool ok[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const uint32_t c = (x + k) / px_;
    ok[k] = sy < g.iy && c < g.ix;
    sx[k] = c < g.ix ? c : g.ix - 1;
  }
  const size_t plane_in = (size_t)g.iy * g.ix, plane_out = (size_t)g.oy * g.ox;
#pragma unroll 2
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const uint32_t w = pl / g.Z, z = pl % g.Z;
    const mt_spos *prow = pos + ((size_t)(w % Wpos) * g.Z + z) * plane_in + (size_t)syc * g.ix;
    const float *irow = in + (size_t)pl * plane_in + (size_t)syc * g.ix;
    mt_spos s[4];
    float v[4];
#pragma unroll
    for (int k = 0; k < 4; k++) { s[k] = prow[sx[k]]; v[k] = irow[sx[k]]; }
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = (ok[k] && s[k].X == x + k && s[k].Y == y) ? v[k] : 0.f;
    reinterpret_cast<float4 *>(out + (size_t)pl * plane_out)[i] = make_float4(v[0], v[1], v[2], v[3]);
  }
}
__global__ __launch_bounds__(EW_THREADS) void downsampling_kernel(float *out, const float *in, Geo g, uint32_t dsx, uint32_t dsy, uint32_t planes) {
  uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, n = g.oy * g.ox;
  if (i >= n) return;
  uint32_t y = i / g.ox, x = i % g.ox;
  float div = (float)(dsx * dsy);
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const float *p = in + (size_t)pl * g.iy * g.ix;
    float s = 0.f;
    for (uint32_t dx = 0; dx < dsx; dx++) {  // dx outer, dy inner: the CPU path's summation order
      uint32_t xp = x * dsx + dx;
      if (xp >= g.ix) continue;
      for (uint32_t dy = 0; dy < dsy; dy++) {
        uint32_t yp = y * dsy + dy;
        if (yp >= g.iy) continue;
        s += p[(size_t)yp * g.ix + xp];
      }
    }
    out[(size_t)pl * n + i] = s / div;
  }
}

__global__ __launch_bounds__(EW_THREADS) void max_pooling_kernel(float *out, mt_spos *pos, uint32_t Wpos, const float *in, Geo g, uint32_t px_, uint32_t py_, uint32_t planes) {
  uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, n = g.oy * g.ox;
  if (i >= n) return;
  uint32_t y = i / g.ox, x = i % g.ox, ix = x * px_, iy = y * py_;
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    uint32_t w = pl / g.Z, z = pl % g.Z;
    const float *p = in + (size_t)pl * g.iy * g.ix;
    float best = p[(size_t)iy * g.ix + ix];
    uint32_t bx = ix, by = iy;
    for (uint32_t py = 0; py < py_; py++)
      for (uint32_t px = 0; px < px_; px++) {
        float e = p[(size_t)(iy + py) * g.ix + ix + px];
        if (e > best) { best = e; bx = ix + px; by = iy + py; }  // first strict maximum, rows then columns
      }
    out[(size_t)pl * n + i] = best;
    mt_spos s; s.X = bx; s.Y = by;
    pos[((size_t)(w % Wpos) * g.Z + z) * n + i] = s;
  }
}

// 2x2 windows over an input of exactly twice the output and a width that is a multiple of four: a thread reads
// 2x4 input pixels (two 128-bit loads) and produces two outputs; same arithmetic and scan order as the kernels above.
template <bool NT>
__global__ __launch_bounds__(EW_THREADS) void downsampling2x2_kernel(float *out, const float *in, Geo g, uint32_t planes) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, ox2 = g.ox / 2, n2 = g.oy * ox2;
  if (i >= n2) return;
  const uint32_t y = i / ox2, x2 = i % ox2;
  const size_t plane_in = (size_t)g.iy * g.ix, plane_out = (size_t)g.oy * g.ox;
  const size_t i0 = (size_t)(2 * y) * g.ix + 4 * x2;
#pragma unroll 4
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const float *p = in + (size_t)pl * plane_in + i0;
    floatx4 a, b;
    if constexpr (NT) {  // an input beyond what the caches hold: read once, not kept
      a = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(p));
      b = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(p + g.ix));
    } else {
      a = *reinterpret_cast<const floatx4 *>(p);
      b = *reinterpret_cast<const floatx4 *>(p + g.ix);
    }
    float2 r;
    r.x = ((((0.f + a.x) + b.x) + a.y) + b.y) / 4.f;  // columns outer, rows inner
    r.y = ((((0.f + a.z) + b.z) + a.w) + b.w) / 4.f;
    reinterpret_cast<float2 *>(out + (size_t)pl * plane_out)[i] = r;
  }
}
template <bool NT>
__global__ __launch_bounds__(EW_THREADS) void max_pooling2x2_kernel(float *out, mt_spos *pos, uint32_t Wpos, const float *in, Geo g, uint32_t planes) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, ox2 = g.ox / 2, n2 = g.oy * ox2;
  if (i >= n2) return;
  const uint32_t y = i / ox2, x2 = i % ox2, iy = 2 * y, ix = 4 * x2;
  const size_t plane_in = (size_t)g.iy * g.ix, plane_out = (size_t)g.oy * g.ox;
  const size_t i0 = (size_t)iy * g.ix + ix;
  const bool same_w = Wpos * g.Z == planes;
#pragma unroll 4
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const float *p = in + (size_t)pl * plane_in + i0;
    floatx4 a, b;
    if constexpr (NT) {
      a = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(p));
      b = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(p + g.ix));
    } else {
      a = *reinterpret_cast<const floatx4 *>(p);
      b = *reinterpret_cast<const floatx4 *>(p + g.ix);
    }
    const float e[2][4] = {{a.x, a.y, b.x, b.y}, {a.z, a.w, b.z, b.w}};  // window scan order: rows, then columns
    float best[2];
    uint4 where;
    uint32_t wh[4];
#pragma unroll
    for (int k = 0; k < 2; k++) {
      best[k] = e[k][0];
      uint32_t bx = ix + 2 * k, by = iy;
#pragma unroll
      for (int t = 0; t < 4; t++)
        if (e[k][t] > best[k]) { best[k] = e[k][t]; bx = ix + 2 * k + (t & 1); by = iy + (t >> 1); }  // first strict maximum
      wh[2 * k] = bx; wh[2 * k + 1] = by;
    }
    where = make_uint4(wh[0], wh[1], wh[2], wh[3]);
    reinterpret_cast<float2 *>(out + (size_t)pl * plane_out)[i] = make_float2(best[0], best[1]);
    const uint32_t ppl = same_w ? pl : (pl / g.Z % Wpos) * g.Z + pl % g.Z;
    reinterpret_cast<uint4 *>(pos + (size_t)ppl * plane_out)[i] = where;
  }
}

// MaxPoolingBackward for 2x2 windows and an output of exactly twice the input: a thread owns two neighbouring windows
// (one 128-bit load of their positions, one 64-bit load of their deltas) and writes their 2 x 4 output pixels as two
// 128-bit stores; same rule as the gather kernel below.
template <bool NT>
__global__ __launch_bounds__(EW_THREADS) void max_pooling_backward2x2_kernel(float *out, const mt_spos *pos, uint32_t Wpos, const float *in, Geo g, uint32_t planes) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, ix2 = g.ix / 2, n2 = g.iy * ix2;
  if (i >= n2) return;
  const uint32_t y = i / ix2, x2 = i % ix2, oy = 2 * y, ox = 4 * x2;
  const size_t plane_in = (size_t)g.iy * g.ix, plane_out = (size_t)g.oy * g.ox;
  const size_t o0 = (size_t)oy * g.ox + ox;
  const bool same_w = Wpos * g.Z == planes;
#pragma unroll 4
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const uint32_t ppl = same_w ? pl : (pl / g.Z % Wpos) * g.Z + pl % g.Z;
    const uint4 s = reinterpret_cast<const uint4 *>(pos + (size_t)ppl * plane_in)[i];  // {X0, Y0, X1, Y1}
    const float2 d = reinterpret_cast<const float2 *>(in + (size_t)pl * plane_in)[i];
    floatx4 r[2];
#pragma unroll
    for (uint32_t dy = 0; dy < 2; dy++) {
      r[dy].x = (s.x == ox && s.y == oy + dy) ? d.x : 0.f;
      r[dy].y = (s.x == ox + 1 && s.y == oy + dy) ? d.x : 0.f;
      r[dy].z = (s.z == ox + 2 && s.w == oy + dy) ? d.y : 0.f;
      r[dy].w = (s.z == ox + 3 && s.w == oy + dy) ? d.y : 0.f;
    }
    float *dst = out + (size_t)pl * plane_out + o0;
    if constexpr (NT) {
      __builtin_nontemporal_store(r[0], reinterpret_cast<floatx4 *>(dst));
      __builtin_nontemporal_store(r[1], reinterpret_cast<floatx4 *>(dst + g.ox));
    } else {
      *reinterpret_cast<floatx4 *>(dst) = r[0];
      *reinterpret_cast<floatx4 *>(dst + g.ox) = r[1];
    }
  }
}

// Gather form of the CPU path's scatter: output (y,x) takes the delta of its window when that window's stored
// maximum is (x,y), else 0.  Equal to the scatter for positions that lie inside their own window, which is what
// max_pooling writes.
__global__ __launch_bounds__(EW_THREADS) void max_pooling_backward_kernel(float *out, const mt_spos *pos, uint32_t Wpos, const float *in, Geo g, uint32_t px_, uint32_t py_, uint32_t planes) {
  uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x, n = g.oy * g.ox;
  if (i >= n) return;
  uint32_t y = i / g.ox, x = i % g.ox, sy = y / py_, sx = x / px_;
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    uint32_t w = pl / g.Z, z = pl % g.Z;
    float v = 0.f;
    if (sy < g.iy && sx < g.ix) {
      size_t k = (size_t)sy * g.ix + sx;
      mt_spos s = pos[((size_t)(w % Wpos) * g.Z + z) * g.iy * g.ix + k];
      if (s.X == x && s.Y == y) v = in[(size_t)pl * g.iy * g.ix + k];
    }
    out[(size_t)pl * n + i] = v;
  }
}

// ---- Adam: fp32 state, update arithmetic in double as on the CPU path ------------------------------------------------
struct AdamStep {
  float batch;
  double speed, beta1, beta2, epsilon, c1, c2;
};
// one element: the new weight; mi and vi are updated in place
__device__ __forceinline__ float adam_element(float w, float dw, float &mi, float &vi, const AdamStep &a) {
  const double speed = a.speed, beta1 = a.beta1, beta2 = a.beta2, epsilon = a.epsilon, c1 = a.c1, c2 = a.c2;
  dw = dw / a.batch;
  mi = (float)(beta1 * (double)mi + (1.0 - beta1) * (double)dw);
  vi = (float)(beta2 * (double)vi + (1.0 - beta2) * (double)dw * (double)dw);
  float mc = (float)((double)mi / c1);  // c1 = 1 - beta1^iteration
  float vc = (float)((double)vi / c2);
  dw = (float)(speed * (double)mc / ((double)sqrtf(vc) + epsilon));
  return w - dw;
}
__device__ __forceinline__ float adam_update(float *weight, const float *dweight, float *m, float *v, size_t i, const AdamStep &a) {
  float mi = m[i], vi = v[i];
  const float w = adam_element(weight[i], dweight[i], mi, vi, a);
  m[i] = mi;
  v[i] = vi;
  weight[i] = w;
  return w;
}
// four consecutive elements (16-byte aligned tensors), the same arithmetic per element
__device__ __forceinline__ float4 adam_update4(float *weight, const float *dweight, float *m, float *v, size_t i4, const AdamStep &a) {
  float4 w = reinterpret_cast<const float4 *>(weight)[i4], mi = reinterpret_cast<const float4 *>(m)[i4], vi = reinterpret_cast<const float4 *>(v)[i4];
  const float4 dw = reinterpret_cast<const float4 *>(dweight)[i4];
  w.x = adam_element(w.x, dw.x, mi.x, vi.x, a);
  w.y = adam_element(w.y, dw.y, mi.y, vi.y, a);
  w.z = adam_element(w.z, dw.z, mi.z, vi.z, a);
  w.w = adam_element(w.w, dw.w, mi.w, vi.w, a);
  reinterpret_cast<float4 *>(m)[i4] = mi;
  reinterpret_cast<float4 *>(v)[i4] = vi;
  reinterpret_cast<float4 *>(weight)[i4] = w;
  return w;
}
__global__ __launch_bounds__(EW_THREADS) void adam_kernel(float *weight, const float *dweight, float *m, float *v, size_t n, AdamStep a) {
  size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x;
  if (i < n) adam_update(weight, dweight, m, v, i, a);
}

// ---- one launch over several tensors (all gradients of a network, all its parameters) ------------------------------
// Tensor t owns the blocks first_block[t] .. first_block[t+1]-1, which walk it with a grid stride.
constexpr int MANY = 32;
struct ManyFill {
  float *p[MANY];
  size_t n[MANY];
  uint32_t first_block[MANY + 1];
};
struct ManyAdam {
  float *weight[MANY];
  const float *dweight[MANY];
  float *m[MANY], *v[MANY];
  size_t n[MANY];
  uint32_t first_block[MANY + 1];
  uint32_t vec;  // bit t: tensor t is updated four elements at a time (a multiple of four elements, 16-byte aligned)
};
template <class T>
__device__ __forceinline__ uint32_t many_owner(const T &a, uint32_t count) {
  uint32_t t = 0;
  while (t + 1 < count && blockIdx.x >= a.first_block[t + 1]) t++;
  return t;
}
__global__ __launch_bounds__(EW_THREADS) void fill_many_kernel(ManyFill a, uint32_t count, float value) {
  const uint32_t t = many_owner(a, count);
  const size_t stride = (size_t)(a.first_block[t + 1] - a.first_block[t]) * EW_THREADS;
  float *p = a.p[t];
  for (size_t i = (size_t)(blockIdx.x - a.first_block[t]) * EW_THREADS + threadIdx.x; i < a.n[t]; i += stride) p[i] = value;
}
// Weights whose re-ordered copy for the transposed convolution 4x4 stride 2 (the input gradient of a 4x4 stride-2
// convolution layer) is kept between calls: the step writes the new value to its place in the copy as well, so the next
// backward pass finds it current.  Coefficient (ky, kx) of filter ci, channel co is tap ((3-ky)/2, (3-kx)/2) of the phase
// that owns the parities of (3-ky, 3-kx); a phase's sub-kernel is [co][ci*4 + tap].
constexpr int MANY_PACKS = 8;
int g_adam_vec = 1;  // 1: mt_adam_many updates four elements per thread in the tiles that also write a re-ordered copy; 2: wherever the tensors allow; 0: never (measurements only)
struct AdamPack {
  float *packed;
  uint32_t ker_ld, co_stride, ci_stride, begin[4];
  uint8_t phase_of[4];
  uint32_t tiles_co;  // 0: element by element; else tiles of 16 filters x 16 channels, this many along the channels
};
struct ManyAdamPacks {
  int8_t slot[MANY];  // -1: no copy to keep
  AdamPack pack[MANY_PACKS];
};
__device__ __forceinline__ void adam_many_plain(const ManyAdam &a, uint32_t t, const AdamStep &step) {
  const size_t stride = (size_t)(a.first_block[t + 1] - a.first_block[t]) * EW_THREADS;
  const size_t first = (size_t)(blockIdx.x - a.first_block[t]) * EW_THREADS + threadIdx.x;
  if (a.vec >> t & 1u) {
    for (size_t i = first; i < a.n[t] / 4; i += stride) adam_update4(a.weight[t], a.dweight[t], a.m[t], a.v[t], i, step);
  } else {
    for (size_t i = first; i < a.n[t]; i += stride) adam_update(a.weight[t], a.dweight[t], a.m[t], a.v[t], i, step);
  }
}
__global__ __launch_bounds__(EW_THREADS) void adam_many_kernel(ManyAdam a, uint32_t count, AdamStep step) {
  adam_many_plain(a, many_owner(a, count), step);
}
__global__ __launch_bounds__(EW_THREADS) void adam_many_packs_kernel(ManyAdam a, ManyAdamPacks packs, uint32_t count, AdamStep step) {
  const uint32_t t = many_owner(a, count);
  const int slot = packs.slot[t];
  if (slot < 0) {
    adam_many_plain(a, t, step);
    return;
  }
  const AdamPack &p = packs.pack[slot];
  const uint32_t begin[4] = {p.begin[0], p.begin[1], p.begin[2], p.begin[3]};
  const uint32_t phase_of = (uint32_t)p.phase_of[0] | (uint32_t)p.phase_of[1] << 8 | (uint32_t)p.phase_of[2] << 16 | (uint32_t)p.phase_of[3] << 24;
  if (p.tiles_co) {
    // Tiles of 16 filters x 16 channels (16 rows of 256 consecutive weights): updated with 128-bit accesses along the
    // rows, the new values staged in LDS, then written to the copy as the 256 contiguous bytes that sixteen filters fill
    // of a (phase, channel) row -- whole lines instead of 16-byte pieces from blocks that run at different times.
    constexpr int ROW = 256 + 1;
    __shared__ float tile[16 * ROW];
    const uint32_t tiles = (uint32_t)(a.n[t] / 4096), blocks = a.first_block[t + 1] - a.first_block[t];
    const uint32_t tid = threadIdx.x, r4 = tid / 64, c4 = tid % 64;   // row within a pass of four rows, float4 within the row
    for (uint32_t tl = blockIdx.x - a.first_block[t]; tl < tiles; tl += blocks) {
      const uint32_t ci0 = (tl / p.tiles_co) * 16u, co0 = (tl % p.tiles_co) * 16u;
#pragma unroll
      for (int pass = 0; pass < 4; pass++) {
        const uint32_t r = pass * 4 + r4;
        const size_t i4 = ((size_t)(ci0 + r) * p.ker_ld + co0 * 16u) / 4 + c4;
        const float4 w = adam_update4(a.weight[t], a.dweight[t], a.m[t], a.v[t], i4, step);
        float *d = tile + r * ROW + c4 * 4;
        d[0] = w.x; d[1] = w.y; d[2] = w.z; d[3] = w.w;
      }
      __syncthreads();
#pragma unroll
      for (int j = 0; j < 4; j++) {   // j = parities of the flipped coefficient: (ky' % 2, kx' % 2)
        const uint32_t ci = tid % 16, co = tid / 16, f = (phase_of >> (8u * j)) & 255u;
        const uint32_t b = f == 0 ? begin[0] : f == 1 ? begin[1] : f == 2 ? begin[2] : begin[3];
        const float *src = tile + ci * ROW + co * 16;
        float4 q;   // taps (ty, tx): coefficient (3 - (ky0 + 2 ty), 3 - (kx0 + 2 tx)) with ky0 = j / 2, kx0 = j % 2
        const uint32_t ky0 = (uint32_t)j >> 1, kx0 = (uint32_t)j & 1u;
        q.x = src[(3 - ky0) * 4 + (3 - kx0)];
        q.y = src[(3 - ky0) * 4 + (1 - kx0)];
        q.z = src[(1 - ky0) * 4 + (3 - kx0)];
        q.w = src[(1 - ky0) * 4 + (1 - kx0)];
        *reinterpret_cast<float4 *>(p.packed + (size_t)b + (size_t)(co0 + co) * p.co_stride + (ci0 + ci) * 4u) = q;
      }
      __syncthreads();
    }
    return;
  }
  const size_t stride = (size_t)(a.first_block[t + 1] - a.first_block[t]) * EW_THREADS;
  for (size_t i = (size_t)(blockIdx.x - a.first_block[t]) * EW_THREADS + threadIdx.x; i < a.n[t]; i += stride) {
    const float w = adam_update(a.weight[t], a.dweight[t], a.m[t], a.v[t], i, step);
    const uint32_t e = (uint32_t)i, ci = e / p.ker_ld, col = e - ci * p.ker_ld, co = col >> 4, tap = col & 15u;
    const uint32_t ky = 3u - (tap >> 2), kx = 3u - (tap & 3u);
    const uint32_t f = (phase_of >> (8u * ((ky & 1u) * 2u + (kx & 1u)))) & 255u;
    const uint32_t b = f == 0 ? begin[0] : f == 1 ? begin[1] : f == 2 ? begin[2] : begin[3];
    p.packed[(size_t)b + (size_t)co * p.co_stride + (size_t)ci * p.ci_stride + (ky >> 1) * 2u + (kx >> 1)] = w;
  }
}

// ---- batch normalisation over the batch axis, statistics per element (z,y,x) --------------------------------------
// Pass 1: per column r, sums of d = x - x[0][r] and d*d over w (the shift keeps the one-pass variance stable).
// A block owns 32 column groups of V columns (V = 4: 128-bit loads) and splits the batch over 8 slices that are
// combined in LDS; the slice loop is unrolled so that several loads per thread are in flight.
// Produces mean, biased variance and 1/sqrt(var+eps), and blends the running statistics.
template <int V>
__global__ __launch_bounds__(EW_THREADS) void bn_stats_kernel(const float *x, uint32_t W, uint32_t S, float inv_n, float eps, float *mean,
                                                              float *var, float *ivar, float *new_mean, float *new_var, float mom_old, float mom_new,
                                                              const float *old_mean, const float *old_var) {
  constexpr int RB = 32, WS = EW_THREADS / RB;
  __shared__ float part[2][WS][RB * V];
  const int rl = threadIdx.x % RB, ws = threadIdx.x / RB;
  const uint32_t r = (blockIdx.x * RB + rl) * V;
  float s1[V], s2[V], shift[V];
#pragma unroll
  for (int v = 0; v < V; v++) { s1[v] = 0.f; s2[v] = 0.f; shift[v] = 0.f; }
  if (r < S) {
    if constexpr (V == 4) {
      float4 t = *reinterpret_cast<const float4 *>(x + r);
      shift[0] = t.x; shift[1] = t.y; shift[2] = t.z; shift[3] = t.w;
#pragma unroll 4
      for (uint32_t w = ws; w < W; w += WS) {
        float4 q = *reinterpret_cast<const float4 *>(x + (size_t)w * S + r);
        float d0 = q.x - shift[0], d1 = q.y - shift[1], d2 = q.z - shift[2], d3 = q.w - shift[3];
        s1[0] += d0; s1[1] += d1; s1[2] += d2; s1[3] += d3;
        s2[0] += d0 * d0; s2[1] += d1 * d1; s2[2] += d2 * d2; s2[3] += d3 * d3;
      }
    } else {
      shift[0] = x[r];
#pragma unroll 4
      for (uint32_t w = ws; w < W; w += WS) {
        float d = x[(size_t)w * S + r] - shift[0];
        s1[0] += d;
        s2[0] += d * d;
      }
    }
  }
#pragma unroll
  for (int v = 0; v < V; v++) { part[0][ws][rl * V + v] = s1[v]; part[1][ws][rl * V + v] = s2[v]; }
  __syncthreads();
  // the first RB*V threads finish one column each
  const int c = threadIdx.x;
  if (c >= RB * V) return;
  const uint32_t rc = blockIdx.x * RB * V + c;
  if (rc >= S) return;
  float a1 = 0.f, a2 = 0.f;
#pragma unroll
  for (int i = 0; i < WS; i++) { a1 += part[0][i][c]; a2 += part[1][i][c]; }
  const float sh = x[rc];
  float md = a1 * inv_n;                  // mean of the shifted data
  float mu = sh + md;
  float vr = (a2 - a1 * md) * inv_n;      // sum((d-md)^2)/N
  if (vr < 0.f) vr = 0.f;
  float iv = (float)(1.0 / (double)(sqrtf(vr + eps) * 1.f));
  mean[rc] = mu;
  var[rc] = vr;
  ivar[rc] = iv;
  if (new_mean) new_mean[rc] = (mom_old * old_mean[rc]) + (mom_new * mu);   // (old_*: the same tensors unless the caller blends from others)
  if (new_var) new_var[rc] = (mom_old * old_var[rc]) + (mom_new * vr);
}

// Pass 2: out = func(gamma * ((x - mean) * ivar) + beta), optionally storing xhat and the value in front of the function.
__global__ __launch_bounds__(EW_THREADS) void bn_apply_kernel(float *out, float *xhat, const float *x, const float *mean, const float *ivar,
                                                              const float *gamma, const float *beta, uint32_t S, uint32_t W, bool vec, int func,
                                                              float *pre = nullptr) {
  uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
  if (vec) {
    if (i * 4 >= S) return;
    float4 mu = reinterpret_cast<const float4 *>(mean)[i], iv = reinterpret_cast<const float4 *>(ivar)[i];
    float4 g = reinterpret_cast<const float4 *>(gamma)[i], b = reinterpret_cast<const float4 *>(beta)[i];
    for (uint32_t w = blockIdx.y; w < W; w += gridDim.y) {
      float4 v = reinterpret_cast<const float4 *>(x + (size_t)w * S)[i], h, o;
      h.x = (v.x - mu.x) * iv.x; h.y = (v.y - mu.y) * iv.y; h.z = (v.z - mu.z) * iv.z; h.w = (v.w - mu.w) * iv.w;
      const float4 z = make_float4((g.x * h.x) + b.x, (g.y * h.y) + b.y, (g.z * h.z) + b.z, (g.w * h.w) + b.w);
      o.x = mt::apply_func(func, z.x); o.y = mt::apply_func(func, z.y);
      o.z = mt::apply_func(func, z.z); o.w = mt::apply_func(func, z.w);
      if (xhat) reinterpret_cast<float4 *>(xhat + (size_t)w * S)[i] = h;
      if (pre) reinterpret_cast<float4 *>(pre + (size_t)w * S)[i] = z;
      reinterpret_cast<float4 *>(out + (size_t)w * S)[i] = o;
    }
  } else {
    if (i >= S) return;
    float mu = mean[i], iv = ivar[i], g = gamma[i], b = beta[i];
    for (uint32_t w = blockIdx.y; w < W; w += gridDim.y) {
      float h = (x[(size_t)w * S + i] - mu) * iv;
      if (xhat) xhat[(size_t)w * S + i] = h;
      if (pre) pre[(size_t)w * S + i] = (g * h) + b;
      out[(size_t)w * S + i] = mt::apply_func(func, (g * h) + b);
    }
  }
}

// Both passes in one kernel when a thread's share of the batch fits in registers: a block owns RB groups of four
// columns and splits the batch over 256/RB slices; a thread keeps its NW rows (128-bit each) in registers between
// the statistics and the normalisation, so the input is read once.  Same sums, in the same order per thread, as
// bn_stats_kernel<4>; only the cheap functions are applied here (see mt::epilogue_func).
// T = 1024 threads for batches of more than 512: 64 or 128 slices, so that a thread's share is still 16 rows at most; the
// slices that sit in one wavefront are added by lane exchanges first, one partial per wavefront goes through LDS.
template <int RB, int NW, int T = EW_THREADS, bool NT = false>
__global__ __launch_bounds__(T) void bn_fused_kernel(float *out, float *xhat, const float *x, uint32_t W, uint32_t S, float inv_n, float eps,
                                                     float *mean, float *var, float *ivar, float *new_mean, float *new_var, float mom_old,
                                                     float mom_new, const float *gamma, const float *beta, int func, const float *old_mean,
                                                     const float *old_var, float *pre) {
  constexpr int WS = T / RB, PARTS = T > EW_THREADS ? T / 64 : WS;
  __shared__ __attribute__((aligned(16))) float part[2][PARTS][RB * 4];
  __shared__ __attribute__((aligned(16))) float col_mean[RB * 4], col_ivar[RB * 4];
  const int rl = threadIdx.x % RB, ws = threadIdx.x / RB;
  const uint32_t r = (blockIdx.x * RB + rl) * 4;
  float4 q[NW];
  float4 s1 = make_float4(0.f, 0.f, 0.f, 0.f), s2 = s1;
  if (r < S) {
    const float4 sh = *reinterpret_cast<const float4 *>(x + r);
#pragma unroll
    for (int i = 0; i < NW; i++) {
      const uint32_t w = ws + i * WS;  // rows past the batch re-read its last row (a plain global load) and are not summed
      if constexpr (NT) {
        const floatx4 t = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(x + (size_t)(w < W ? w : W - 1) * S + r));
        q[i] = make_float4(t.x, t.y, t.z, t.w);
      } else {
        q[i] = *reinterpret_cast<const float4 *>(x + (size_t)(w < W ? w : W - 1) * S + r);
      }
    }
#pragma unroll
    for (int i = 0; i < NW; i++) {
      if (ws + i * WS < W) {
        float d0 = q[i].x - sh.x, d1 = q[i].y - sh.y, d2 = q[i].z - sh.z, d3 = q[i].w - sh.w;
        s1.x += d0; s1.y += d1; s1.z += d2; s1.w += d3;
        s2.x += d0 * d0; s2.y += d1 * d1; s2.z += d2 * d2; s2.w += d3 * d3;
      }
    }
  }
  if constexpr (T > EW_THREADS) {
    static_assert(RB < 64, "several slices per wavefront");
#pragma unroll
    for (int d = RB; d < 64; d <<= 1) {
      s1.x += __shfl_xor(s1.x, d, 64); s1.y += __shfl_xor(s1.y, d, 64); s1.z += __shfl_xor(s1.z, d, 64); s1.w += __shfl_xor(s1.w, d, 64);
      s2.x += __shfl_xor(s2.x, d, 64); s2.y += __shfl_xor(s2.y, d, 64); s2.z += __shfl_xor(s2.z, d, 64); s2.w += __shfl_xor(s2.w, d, 64);
    }
    if ((threadIdx.x & 63) < RB) {
      *reinterpret_cast<float4 *>(&part[0][threadIdx.x / 64][rl * 4]) = s1;
      *reinterpret_cast<float4 *>(&part[1][threadIdx.x / 64][rl * 4]) = s2;
    }
  } else {
    *reinterpret_cast<float4 *>(&part[0][ws][rl * 4]) = s1;
    *reinterpret_cast<float4 *>(&part[1][ws][rl * 4]) = s2;
  }
  __syncthreads();
  const int c = threadIdx.x;
  const uint32_t rc = blockIdx.x * RB * 4 + c;
  if (c < RB * 4 && rc < S) {  // the first RB*4 threads finish one column each
    float a1 = 0.f, a2 = 0.f;
#pragma unroll
    for (int i = 0; i < PARTS; i++) { a1 += part[0][i][c]; a2 += part[1][i][c]; }
    const float sh = x[rc];
    float md = a1 * inv_n;
    float mu = sh + md;
    float vr = (a2 - a1 * md) * inv_n;
    if (vr < 0.f) vr = 0.f;
    float iv = (float)(1.0 / (double)(sqrtf(vr + eps) * 1.f));
    mean[rc] = mu;
    var[rc] = vr;
    ivar[rc] = iv;
    if (new_mean) new_mean[rc] = (mom_old * old_mean[rc]) + (mom_new * mu);
    if (new_var) new_var[rc] = (mom_old * old_var[rc]) + (mom_new * vr);
    col_mean[c] = mu;
    col_ivar[c] = iv;
  }
  __syncthreads();
  if (r >= S) return;
  const float4 mu = *reinterpret_cast<const float4 *>(col_mean + rl * 4), iv = *reinterpret_cast<const float4 *>(col_ivar + rl * 4);
  const float4 g = *reinterpret_cast<const float4 *>(gamma + r), b = *reinterpret_cast<const float4 *>(beta + r);
  // one look at the function and at the optional output for the whole loop, not one per value
  auto emit = [&](auto f, auto keep) {
#pragma unroll
    for (int i = 0; i < NW; i++) {
      const uint32_t w = ws + i * WS;
      if (w >= W) break;
      float4 h, o;
      h.x = (q[i].x - mu.x) * iv.x; h.y = (q[i].y - mu.y) * iv.y; h.z = (q[i].z - mu.z) * iv.z; h.w = (q[i].w - mu.w) * iv.w;
      const float4 z = make_float4((g.x * h.x) + b.x, (g.y * h.y) + b.y, (g.z * h.z) + b.z, (g.w * h.w) + b.w);
      o.x = f(z.x); o.y = f(z.y); o.z = f(z.z); o.w = f(z.w);
      if (pre) *reinterpret_cast<float4 *>(pre + (size_t)w * S + r) = z;   // (the value in front of the function, for callers that keep both)
      if constexpr (NT) {
        if constexpr (decltype(keep)::value) __builtin_nontemporal_store(floatx4{h.x, h.y, h.z, h.w}, reinterpret_cast<floatx4 *>(xhat + (size_t)w * S + r));
        __builtin_nontemporal_store(floatx4{o.x, o.y, o.z, o.w}, reinterpret_cast<floatx4 *>(out + (size_t)w * S + r));
      } else {
        if constexpr (decltype(keep)::value) *reinterpret_cast<float4 *>(xhat + (size_t)w * S + r) = h;
        *reinterpret_cast<float4 *>(out + (size_t)w * S + r) = o;
      }
    }
  };
  auto with_func = [&](auto keep) {
    if (func == MT_F_RELU) emit([](float v) { return v > 0.f ? v : 0.f; }, keep);
    else if (func == MT_F_LEAKY_RELU) emit([](float v) { return v > 0.f ? v : (float)(0.1 * (double)v); }, keep);
    else emit([](float v) { return v; }, keep);
  };
  if (xhat) with_func(std::true_type{}); else with_func(std::false_type{});
}

// Backward pass of the same layer in one kernel (netlayer/cnetlayerbatchnormalization.cu.h:578-604):
//   dxhat = delta*gamma;  s1 = sum_w dxhat;  s2 = sum_w dxhat*xhat;  dgamma += sum_w delta*xhat;  dbeta += sum_w delta;
//   error = ((N*dxhat - xhat*s2) - s1) * ivar * (1/N)            (each step rounded to fp32, in this order)
// Block layout as bn_fused_kernel.  NW > 0: a thread keeps its NW rows of delta and xhat in registers between the
// sums and the error; NW == 0: any batch size, the rows are read a second time.
// func (ReLU or leaky ReLU, else MT_F_NONE): the layer's output went through that function and `delta` is the
// gradient behind it; the function layer's step delta * f'(gamma*xhat + beta) happens as delta is loaded (keep_front:
// that product is stored too, where the function layer itself leaves it).
template <int RB, int NW, int T = EW_THREADS>   // T = 1024: see bn_fused_kernel
__global__ __launch_bounds__(T) void bn_backward_kernel(float *err, float *dgamma, float *dbeta, const float *delta, const float *gamma,
                                                        const float *beta, const float *xhat, const float *ivar, uint32_t W, uint32_t S, float n,
                                                        float inv_n, int func, float *keep_dxhat, float *keep_s1, float *keep_s2, float *keep_front) {
  constexpr int WS = T / RB, HOLD = NW > 0 ? NW : 1, PARTS = T > EW_THREADS ? T / 64 : WS;
  __shared__ float part[4][PARTS][RB * 4];
  __shared__ float col_s1[RB * 4], col_s2[RB * 4];
  const int rl = threadIdx.x % RB, ws = threadIdx.x / RB;
  const uint32_t r = (blockIdx.x * RB + rl) * 4;
  float4 qd[HOLD], qx[HOLD];
  float acc[4][4] = {};
  float4 g = make_float4(0.f, 0.f, 0.f, 0.f), bt = g;
  const float below = func == MT_F_RELU ? 0.f : 0.1f;  // f'(z) for z < 0
  auto behind = [&](float4 d, const float4 &x) {  // the gradient in front of the function
    if (func != MT_F_NONE) {
      d.x = d.x * (((g.x * x.x) + bt.x) >= 0.f ? 1.f : below);
      d.y = d.y * (((g.y * x.y) + bt.y) >= 0.f ? 1.f : below);
      d.z = d.z * (((g.z * x.z) + bt.z) >= 0.f ? 1.f : below);
      d.w = d.w * (((g.w * x.w) + bt.w) >= 0.f ? 1.f : below);
    }
    return d;
  };
  auto add = [&](const float4 &d, const float4 &x) {
    const float dv[4] = {d.x, d.y, d.z, d.w}, xv[4] = {x.x, x.y, x.z, x.w}, gv[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const float dx = dv[v] * gv[v];
      acc[0][v] += dx;
      acc[1][v] += dx * xv[v];
      acc[2][v] += dv[v] * xv[v];
      acc[3][v] += dv[v];
    }
  };
  if (r < S) {
    g = *reinterpret_cast<const float4 *>(gamma + r);
    if (func != MT_F_NONE) bt = *reinterpret_cast<const float4 *>(beta + r);
    if constexpr (NW > 0) {
#pragma unroll
      for (int i = 0; i < NW; i++) {
        const uint32_t w = ws + i * WS;
        if (w < W) {
          qd[i] = *reinterpret_cast<const float4 *>(delta + (size_t)w * S + r);
          qx[i] = *reinterpret_cast<const float4 *>(xhat + (size_t)w * S + r);
        }
      }
#pragma unroll
      for (int i = 0; i < NW; i++)
        if (ws + i * WS < W) {
          qd[i] = behind(qd[i], qx[i]);
          add(qd[i], qx[i]);
        }
    } else {
#pragma unroll 8
      for (uint32_t w = ws; w < W; w += WS) {
        const float4 x = *reinterpret_cast<const float4 *>(xhat + (size_t)w * S + r);
        add(behind(*reinterpret_cast<const float4 *>(delta + (size_t)w * S + r), x), x);
      }
    }
  }
  if constexpr (T > EW_THREADS) {
    static_assert(RB < 64, "several slices per wavefront");
#pragma unroll
    for (int d = RB; d < 64; d <<= 1)
#pragma unroll
      for (int q = 0; q < 4; q++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[q][v] += __shfl_xor(acc[q][v], d, 64);
    if ((threadIdx.x & 63) < RB) {
#pragma unroll
      for (int q = 0; q < 4; q++)
#pragma unroll
        for (int v = 0; v < 4; v++) part[q][threadIdx.x / 64][rl * 4 + v] = acc[q][v];
    }
  } else {
#pragma unroll
    for (int q = 0; q < 4; q++)
#pragma unroll
      for (int v = 0; v < 4; v++) part[q][ws][rl * 4 + v] = acc[q][v];
  }
  __syncthreads();
  const int c = threadIdx.x;
  const uint32_t rc = blockIdx.x * RB * 4 + c;
  if (c < RB * 4 && rc < S) {  // the first RB*4 threads finish one column each
    float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < PARTS; i++)
#pragma unroll
      for (int q = 0; q < 4; q++) t[q] += part[q][i][c];
    col_s1[c] = t[0];
    col_s2[c] = t[1];
    if (keep_s1) keep_s1[rc] = t[0];
    if (keep_s2) keep_s2[rc] = t[1];
    if (dgamma) dgamma[rc] = dgamma[rc] + t[2];
    if (dbeta) dbeta[rc] = dbeta[rc] + t[3];
  }
  __syncthreads();
  if (r >= S) return;
  const float4 s1 = *reinterpret_cast<const float4 *>(col_s1 + rl * 4), s2 = *reinterpret_cast<const float4 *>(col_s2 + rl * 4);
  const float4 iv = *reinterpret_cast<const float4 *>(ivar + r);
  auto error = [&](const float4 &d, const float4 &x) {
    float4 e;
    e.x = (((n * (d.x * g.x)) - (x.x * s2.x)) - s1.x) * iv.x * inv_n;
    e.y = (((n * (d.y * g.y)) - (x.y * s2.y)) - s1.y) * iv.y * inv_n;
    e.z = (((n * (d.z * g.z)) - (x.z * s2.z)) - s1.z) * iv.z * inv_n;
    e.w = (((n * (d.w * g.w)) - (x.w * s2.w)) - s1.w) * iv.w * inv_n;
    return e;
  };
  auto times_gamma = [&](const float4 &d) { return make_float4(d.x * g.x, d.y * g.y, d.z * g.z, d.w * g.w); };
  if constexpr (NW > 0) {
    if (keep_dxhat) {  // (one look at the optional output for the whole loop)
#pragma unroll
      for (int i = 0; i < NW; i++) {
        const uint32_t w = ws + i * WS;
        if (w >= W) break;
        *reinterpret_cast<float4 *>(keep_dxhat + (size_t)w * S + r) = times_gamma(qd[i]);
      }
    }
    if (keep_front) {
#pragma unroll
      for (int i = 0; i < NW; i++) {
        const uint32_t w = ws + i * WS;
        if (w >= W) break;
        *reinterpret_cast<float4 *>(keep_front + (size_t)w * S + r) = qd[i];
      }
    }
#pragma unroll
    for (int i = 0; i < NW; i++) {
      const uint32_t w = ws + i * WS;
      if (w >= W) break;
      *reinterpret_cast<float4 *>(err + (size_t)w * S + r) = error(qd[i], qx[i]);
    }
  } else {
    for (uint32_t w = ws; w < W; w += WS) {
      const float4 x = *reinterpret_cast<const float4 *>(xhat + (size_t)w * S + r);
      const float4 d = behind(*reinterpret_cast<const float4 *>(delta + (size_t)w * S + r), x);
      if (keep_dxhat) *reinterpret_cast<float4 *>(keep_dxhat + (size_t)w * S + r) = times_gamma(d);
      if (keep_front) *reinterpret_cast<float4 *>(keep_front + (size_t)w * S + r) = d;
      *reinterpret_cast<float4 *>(err + (size_t)w * S + r) = error(d, x);
    }
  }
}

// VAE coder output (netlayer/cnetlayervaecoderoutput.cu.h:252-286, a host loop there): out = mu + exp(clamp(lv)/2)*eps
// and per block the partial sum of 1 + lv - mu^2 - exp(lv); vae_kl_kernel adds the partials in block order.
__global__ __launch_bounds__(EW_THREADS) void vae_coder_kernel(float *out, float *partial, const float *mu, const float *logvar, const float *eps, size_t n) {
  __shared__ float red[EW_THREADS / 64];
  float s = 0.f;
  for (size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += (size_t)gridDim.x * EW_THREADS) {
    float m = mu[i], lv = logvar[i];
    if (lv > 10.f) lv = 10.f;
    if (lv < -10.f) lv = -10.f;
    const float e = (float)exp((double)lv / 2.0);
    out[i] = m + e * eps[i];
    s += 1.f + lv - m * m - expf(lv);
  }
  s = mt::wave_sum(s);
  if (threadIdx.x % 64 == 0) red[threadIdx.x / 64] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int i = 0; i < EW_THREADS / 64; i++) t += red[i];
    partial[blockIdx.x] = t;
  }
}
__global__ void vae_kl_kernel(float *kl, const float *partial, uint32_t blocks, float batch) {
  float t = 0.f;
  for (uint32_t i = 0; i < blocks; i++) t += partial[i];
  t = (float)((double)t * -0.5);
  kl[0] = t / batch;
}

// ---- functions of the reference's GPU class that have no CPU counterpart (cuda/ctensormath.cu.h:473-598, 3029-3262) ----
// ConcatecationZ / SplitZ: plane (w, z) of the wide tensor is plane (w % Wa, z) of A or (w % Wb, z - Za) of B.
// TO_WIDE: the wide tensor is written (concatenation), else read (split; w then runs over the wide tensor's batch).
template <bool TO_WIDE, class V>
__global__ __launch_bounds__(EW_THREADS) void concat_split_z_kernel(V *wide, V *a, V *b, uint32_t Wwide, uint32_t Z, uint32_t Wa, uint32_t Za, uint32_t Wb,
                                                                     uint32_t yx) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
  if (i >= yx) return;
  const uint32_t planes = Wwide * Z, Zb = Z - Za;
  for (uint32_t pl = blockIdx.y; pl < planes; pl += gridDim.y) {
    const uint32_t w = pl / Z, z = pl % Z;
    V *narrow = z < Za ? a + ((size_t)(w % Wa) * Za + z) * yx : b + ((size_t)(w % Wb) * Zb + (z - Za)) * yx;
    if (TO_WIDE) wide[(size_t)pl * yx + i] = narrow[i];
    else narrow[i] = wide[(size_t)pl * yx + i];
  }
}

// SetTimeStep: out = in + (pos even ? sin : cos)(t[w] / 10000^(pos/size)), pos = element index within the sample
__global__ __launch_bounds__(EW_THREADS) void set_time_step_kernel(float *out, const float *in, const uint32_t *time_step, uint32_t size, uint32_t W) {
  const uint32_t pos = blockIdx.x * EW_THREADS + threadIdx.x;
  if (pos >= size) return;
  const float scale = powf(10000.0f, (float)pos / (float)size);
  for (uint32_t w = blockIdx.y; w < W; w += gridDim.y) {
    const float angle = (float)time_step[w] / scale;
    out[(size_t)w * size + pos] = in[(size_t)w * size + pos] + ((pos & 1u) == 0 ? sinf(angle) : cosf(angle));
  }
}

// Philox4x32-10 (Salmon et al., SC'11): key = seed, counter = (element index, 0, 0); one block of four words per element.
__device__ __forceinline__ void philox4x32_10(uint64_t seed, uint64_t index, uint32_t (&r)[4]) {
  uint32_t c0 = (uint32_t)index, c1 = (uint32_t)(index >> 32), c2 = 0u, c3 = 0u, k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int round = 0; round < 10; round++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  r[0] = c0; r[1] = c1; r[2] = c2; r[3] = c3;
}
__device__ __forceinline__ float philox_uniform(const uint32_t (&r)[4]) { return (float)(r[0] >> 8) * (1.0f / 16777216.0f); }  // [0, 1)
__device__ __forceinline__ float philox_normal(const uint32_t (&r)[4]) {  // Box-Muller: u1 in (0, 1], u2 in [0, 1)
  const float u1 = (float)((r[0] >> 8) + 1u) * (1.0f / 16777216.0f), u2 = (float)(r[1] >> 8) * (1.0f / 16777216.0f);
  return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
}
__global__ __launch_bounds__(EW_THREADS) void drop_out_kernel(float *out, size_t n, float drop_out, float mult, uint64_t seed) {
  for (size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += (size_t)gridDim.x * EW_THREADS) {
    uint32_t r[4];
    philox4x32_10(seed, i, r);
    out[i] = philox_uniform(r) >= drop_out ? mult : 0.f;
  }
}
// noise = N(0,1); with an image: noisy = sa[w] * image + sb[w] * noise
__global__ __launch_bounds__(EW_THREADS) void normal_noise_kernel(float *noise, float *noisy, const float *image, const float *sa, uint32_t sa_stride,
                                                                   const float *sb, uint32_t sb_stride, size_t per, size_t n, uint64_t seed) {
  for (size_t i = (size_t)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += (size_t)gridDim.x * EW_THREADS) {
    uint32_t r[4];
    philox4x32_10(seed, i, r);
    const float e = philox_normal(r);
    noise[i] = e;
    if (noisy) {
      const size_t w = i / per;
      noisy[i] = (sa[w * sa_stride] * image[i]) + (sb[w * sb_stride] * e);
    }
  }
}

__global__ __launch_bounds__(EW_THREADS) void bn_ivar_kernel(float *ivar, const float *var, uint32_t S, float eps) {
  uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
  if (i < S) ivar[i] = (float)(1.0 / (double)sqrtf(var[i] + eps));
}

}  // namespace

// a small pool of scratch statistics for the fused batch-norm entry points when the caller passes NULL
namespace {
mt::Workspace g_bn_ws;
int bn_scratch(size_t floats, float **p) { return mt::workspace_get(g_bn_ws, "batch-norm scratch", floats, p); }

// The same scratch for callers that cannot allocate: a fixed array in the code object's own device memory, one copy
// per device that loads the library, held until the process ends.  Host code never uses the array's name as an
// address: the device address is looked up once per device (with that device current) and kept.
constexpr size_t STATIC_SCRATCH_FLOATS = 3u * 262144u;  // mean, variance, 1/sqrt(variance + eps) of up to 262144 elements: 3 MiB
constexpr int MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];
float *g_static_scratch[MAX_DEVICES] = {};
int static_scratch(float **p) {
  int dev = -1;
  MT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= MAX_DEVICES) return mt::fail(MT_E_UNAVAILABLE, "static scratch: device %d is beyond the %d devices the library keeps an address for", dev, MAX_DEVICES);
  if (g_static_scratch[dev] == nullptr) {
    void *q = nullptr;
    MT_HIP(hipGetSymbolAddress(&q, HIP_SYMBOL(scratch)));
    if (q == nullptr) return mt::fail(MT_E_UNAVAILABLE, "static scratch: no device address for the array on device %d", dev);
    g_static_scratch[dev] = static_cast<float *>(q);
  }
  *p = g_static_scratch[dev];
  return MT_OK;
}
}  // namespace

namespace {
__global__ __launch_bounds__(EW_THREADS) void norm_apply_kernel(float *out, const float *in, const float2 *ss, uint32_t S, uint32_t W, int func) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
  if (i >= S) return;
  const float2 p = ss[i];
  for (uint32_t w = blockIdx.y; w < W; w += gridDim.y) out[(size_t)w * S + i] = mt::apply_func_cheap(func, p.x * in[(size_t)w * S + i] + p.y);
}
__global__ __launch_bounds__(EW_THREADS) void bn_scale_shift_kernel(float2 *ss, const float *mean, const float *ivar, const float *gamma, const float *beta, uint32_t S) {
  const uint32_t i = blockIdx.x * EW_THREADS + threadIdx.x;
  if (i >= S) return;
  const float scale = gamma[i] * ivar[i];
  ss[i] = make_float2(scale, beta[i] - mean[i] * scale);
}
}  // namespace

namespace mt {
int set_nontemporal(int v) {
  if (v < 0 || v > 2) return fail(MT_E_ARGUMENT, "nontemporal must be 0 (never), 1 (always) or 2 (tensors of 128 MiB and more)");
  g_nontemporal = v;
  return MT_OK;
}
int norm_apply(const mt_tensor *out, const mt_tensor *in, const float *scale_shift, int func) {
  const size_t S = (size_t)in->z * in->y * in->x;
  if (S == 0 || in->w == 0) return MT_OK;
  mt::ProfileScope prof("norm_apply");
  norm_apply_kernel<<<dim3(cdiv(S, EW_THREADS), in->w < 16 ? in->w : 16), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, reinterpret_cast<const float2 *>(scale_shift),
                                                                                                         (uint32_t)S, in->w, func);
  MT_LAUNCH_CHECK("norm_apply");
  return MT_OK;
}

int bn_statistics(const mt_tensor *x, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *scale_shift, const mt_tensor *ivar,
                  const mt_tensor *mean, const mt_tensor *var, const mt_tensor *new_mean, const mt_tensor *new_var, float momentum, float epsilon) {
  const size_t S = (size_t)x->z * x->y * x->x;
  const uint32_t W = x->w;
  if (S == 0 || W == 0) return MT_OK;
  float *spare = nullptr;
  int rc = bn_scratch(3 * S, &spare);
  if (rc) return rc;
  float *pm = mean ? mean->p : spare, *pv = var ? var->p : spare + S, *pi = ivar ? ivar->p : spare + 2 * S;
  const float inv_n = (float)(1.0 / (double)(float)W), mom_new = (float)(1.0 - (double)momentum);
  float *nm = new_mean ? new_mean->p : nullptr, *nv = new_var ? new_var->p : nullptr;
  {
    mt::ProfileScope prof("bn_stats");
    if (S % 4 == 0 && aligned16(x->p))
      bn_stats_kernel<4><<<cdiv(S, 128), EW_THREADS, 0, mt::stream()>>>(x->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, nm, nv);
    else
      bn_stats_kernel<1><<<cdiv(S, 32), EW_THREADS, 0, mt::stream()>>>(x->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, nm, nv);
    MT_LAUNCH_CHECK("bn_stats");
  }
  bn_scale_shift_kernel<<<cdiv(S, EW_THREADS), EW_THREADS, 0, mt::stream()>>>(reinterpret_cast<float2 *>(scale_shift->p), pm, pi, gamma->p, beta->p, (uint32_t)S);
  MT_LAUNCH_CHECK("bn_scale_shift");
  return MT_OK;
}

int static_scratch_setup() {
  float *p = nullptr;
  return static_scratch(&p);
}
}  // namespace mt

namespace {
template <bool TO_WIDE>
int concat_split(const char *name, const mt_tensor *wide, const mt_tensor *a, const mt_tensor *b) {
  if (mt::bad(wide) || mt::bad(a) || mt::bad(b)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  if (TO_WIDE) mt::note_write(wide); else { mt::note_write(a); mt::note_write(b); }
  if (wide->x != a->x || wide->x != b->x || wide->y != a->y || wide->y != b->y || wide->z != a->z + b->z)
    return mt::fail(MT_E_SHAPE, "%s: sizes do not match", name);
  const uint32_t yx = wide->y * wide->x, planes = wide->w * wide->z;
  if (yx == 0 || planes == 0) return MT_OK;
  if ((a->z && a->w == 0) || (b->z && b->w == 0)) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  const uint32_t wa = a->w ? a->w : 1, wb = b->w ? b->w : 1;
  if (yx % 4 == 0 && aligned16(wide->p) && aligned16(a->p) && aligned16(b->p)) {
    const unsigned bx = cdiv(yx / 4, EW_THREADS);
    concat_split_z_kernel<TO_WIDE, float4><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(
        (float4 *)wide->p, (float4 *)a->p, (float4 *)b->p, wide->w, wide->z, wa, a->z, wb, yx / 4);
  } else {
    const unsigned bx = cdiv(yx, EW_THREADS);
    concat_split_z_kernel<TO_WIDE, float><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(wide->p, a->p, b->p, wide->w, wide->z, wa, a->z,
                                                                                                               wb, yx);
  }
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}
unsigned stream_blocks(size_t n) {
  const unsigned blocks = cdiv(n, EW_THREADS);
  return blocks > 16384u ? 16384u : blocks;
}
}  // namespace

static int bn_backward_any(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta, const mt_tensor *gamma,
                           const mt_tensor *beta, const mt_tensor *xhat, const mt_tensor *ivar, int func, const mt_tensor *keep_dxhat, const mt_tensor *keep_s1,
                           const mt_tensor *keep_s2, const mt_tensor *keep_front = nullptr);

namespace mt {
int set_adam_vec(int v) {
  if (v < 0 || v > 2) return fail(MT_E_ARGUMENT, "adam_vec must be 0, 1 or 2");
  g_adam_vec = v;
  return MT_OK;
}
// out1[i] += sum over w of r1[w][i] and out2[i] += sum over w of r2[w][i], both over the same W: one launch where the
// 128-bit kernel takes both (sizes that are multiples of four, aligned), else two calls of mt_add_sum_w.
int add_sum_w_pair(float *out1, const float *r1, size_t S1, float *out2, const float *r2, size_t S2, uint32_t W) {
  if (S1 == 0 || S2 == 0 || W == 0) return fail(MT_E_ARGUMENT, "add_sum_w_pair: empty operand");
  if (S1 % 4 || S2 % 4 || S1 < 1024 || S1 > 0xffffffffu || S2 > 0xffffffffu || !aligned16(out1) || !aligned16(r1) || !aligned16(out2) || !aligned16(r2)) {
    const mt_tensor o1{out1, 1, 1, 1, (uint32_t)S1}, p1{const_cast<float *>(r1), W, 1, 1, (uint32_t)S1};
    const mt_tensor o2{out2, 1, 1, 1, (uint32_t)S2}, p2{const_cast<float *>(r2), W, 1, 1, (uint32_t)S2};
    if (S1 > 0xffffffffu || S2 > 0xffffffffu) return fail(MT_E_ARGUMENT, "add_sum_w_pair: more than 2^32 elements");
    const int rc = mt_add_sum_w(&o1, &o1, &p1, 1.f, 1.f);
    return rc ? rc : mt_add_sum_w(&o2, &o2, &p2, 1.f, 1.f);
  }
  note_write(out1, S1 * sizeof(float));
  note_write(out2, S2 * sizeof(float));
  char shape[64];
  if (profiling()) snprintf(shape, sizeof shape, "S %zu and %zu W 1 + %u", S1, S2, W);
  ProfileScope prof(profiling() ? intern_label("mt_add_sum_w", shape) : "mt_add_sum_w");
  const size_t cols = S1 / 4;
  int rb = cols / 256 >= 1024 && W <= 4 ? 256 : cols / 32 >= 256 ? 32 : cols / 8 >= 256 ? 8 : 4;   // as in mt_add_sum_w, chosen for the first sum
  if (rb == 4 && W < 64) rb = 8;
  if (rb == 8 && W < 32) rb = 32;
  if (rb == 32 && W < 8 && cols / 256 >= 64) rb = 256;
  SumJob a{out1, r1, (uint32_t)S1, cdiv(cols, (size_t)rb)}, b{out2, r2, (uint32_t)S2, cdiv(S2 / 4, (size_t)rb)};
  const uint32_t grid = a.blocks + b.blocks;
  hipStream_t st = stream();
  if (rb == 256) add_sum_w_pair_kernel<256><<<grid, EW_THREADS, 0, st>>>(a, b, W);
  else if (rb == 32) add_sum_w_pair_kernel<32><<<grid, EW_THREADS, 0, st>>>(a, b, W);
  else if (rb == 8) add_sum_w_pair_kernel<8><<<grid, EW_THREADS, 0, st>>>(a, b, W);
  else add_sum_w_pair_kernel<4><<<grid, EW_THREADS, 0, st>>>(a, b, W);
  MT_LAUNCH_CHECK("mt_add_sum_w");
  return MT_OK;
}
}  // namespace mt

extern "C" {

int mt_fill(const mt_tensor *out, float value) {
  if (mt::bad(out)) return mt::fail(MT_E_ARGUMENT, "mt_fill: null tensor");
  mt::note_write(out);
  size_t n = mt::count(out);
  if (n == 0) return MT_OK;
  if (n % 4 == 0 && aligned16(out->p)) {
    unsigned blocks = cdiv(n / 4, EW_THREADS);
    if (blocks > 8192u) blocks = 8192u;
    fill4_kernel<<<blocks, EW_THREADS, 0, mt::stream()>>>(reinterpret_cast<float4 *>(out->p), n / 4, value);
    MT_LAUNCH_CHECK("mt_fill");
    return MT_OK;
  }
  unsigned blocks = cdiv(n, EW_THREADS);
  if (blocks > 65536u * 4) blocks = 65536u * 4;
  fill_kernel<<<blocks, EW_THREADS, 0, mt::stream()>>>(out->p, n, value);
  MT_LAUNCH_CHECK("mt_fill");
  return MT_OK;
}

int mt_inv(const mt_tensor *out, const mt_tensor *in) { return launch1("mt_inv", out, in, FInv{}); }
int mt_pow2(const mt_tensor *out, const mt_tensor *in, float scale) { return launch1("mt_pow2", out, in, FPow2{scale}); }
int mt_sqrt(const mt_tensor *out, const mt_tensor *in, float scale, float add) { return launch1("mt_sqrt", out, in, FSqrt{scale, add}); }
int mt_mul_value(const mt_tensor *out, const mt_tensor *in, float v) { return launch1("mt_mul_value", out, in, FScale{v}); }
int mt_add_value(const mt_tensor *out, const mt_tensor *in, float s, float v) { return launch1("mt_add_value", out, in, FAffine{s, v}); }
int mt_sub_value(const mt_tensor *out, const mt_tensor *in, float s, float v) { return launch1("mt_sub_value", out, in, FAffine{s, -v}); }
int mt_set(const mt_tensor *out, const mt_tensor *in, float s, float add) { return launch1("mt_set", out, in, FAffine{s, add}); }
int mt_clip(const mt_tensor *t, float lo, float hi) { return launch1("mt_clip", t, t, FClip{lo, hi}); }
int mt_signum(const mt_tensor *t) { return launch1("mt_signum", t, t, FSign{}); }

int mt_add(const mt_tensor *out, const mt_tensor *l, const mt_tensor *r, float ls, float rs) { return launch2("mt_add", out, l, r, FAdd{ls, rs}); }
int mt_sub(const mt_tensor *out, const mt_tensor *l, const mt_tensor *r, float ls, float rs) { return launch2("mt_sub", out, l, r, FSub{ls, rs}); }
int mt_div(const mt_tensor *out, const mt_tensor *l, const mt_tensor *r, float ls, float rs) { return launch2("mt_div", out, l, r, FDiv{ls, rs}); }
int mt_tensor_item_production(const mt_tensor *out, const mt_tensor *l, const mt_tensor *r) { return launch2("mt_tensor_item_production", out, l, r, FMul{}); }

int mt_apply_func(const mt_tensor *out, const mt_tensor *in, int func) {
  if (!mt::valid_func(func, false)) return mt::fail(MT_E_ARGUMENT, "mt_apply_func: unknown function id %d", func);
  if (mt::bad(out) || mt::bad(in)) return mt::fail(MT_E_ARGUMENT, "mt_apply_func: null tensor");
  if (!mt::same_zyx(in, out) || in->w != out->w) return mt::fail(MT_E_SHAPE, "mt_apply_func: sizes of input and output differ");
  return launch1("mt_apply_func", out, in, FFunc{func});
}

int mt_add_sum_w(const mt_tensor *out, const mt_tensor *l, const mt_tensor *r, float ls, float rs) {
  if (mt::bad(out) || mt::bad(l) || mt::bad(r)) return mt::fail(MT_E_ARGUMENT, "mt_add_sum_w: null tensor");
  mt::note_write(out);
  if (!mt::same_zyx(l, r) || !mt::same_zyx(out, r)) return mt::fail(MT_E_SHAPE, "mt_add_sum_w: Z/Y/X of the operands differ");
  size_t S = (size_t)out->z * out->y * out->x;
  if (S == 0 || out->w == 0) return MT_OK;
  char shape[64];
  if (mt::profiling()) snprintf(shape, sizeof shape, "S %zu W %u + %u", S, l->w, r->w);
  mt::ProfileScope prof(mt::profiling() ? mt::intern_label("mt_add_sum_w", shape) : "mt_add_sum_w");
  // the output may alias an operand (dW = dW + sum_w TmpdW): every column is read completely before it is written
  if (S % 4 == 0 && S >= 1024 && aligned16(out->p) && aligned16(l->p) && aligned16(r->p)) {
    // groups of four columns per block: as many as still give about a thousand blocks, but no more slices than samples
    const size_t cols = S / 4;
    const uint32_t W = l->w > r->w ? l->w : r->w;
    int rb = cols / 256 >= 1024 && W <= 4 ? 256 : cols / 32 >= 256 ? 32 : cols / 8 >= 256 ? 8 : 4;
    if (rb == 4 && W < 64) rb = 8;
    if (rb == 8 && W < 32) rb = 32;
    if (rb == 32 && W < 8 && cols / 256 >= 64) rb = 256;
    hipStream_t st = mt::stream();
    const uint32_t n = (uint32_t)S;
    if (rb == 256) add_sum_w_vec_kernel<256><<<cdiv(cols, 256), EW_THREADS, 0, st>>>(out->p, out->w, l->p, l->w, r->p, r->w, n, ls, rs);
    else if (rb == 32) add_sum_w_vec_kernel<32><<<cdiv(cols, 32), EW_THREADS, 0, st>>>(out->p, out->w, l->p, l->w, r->p, r->w, n, ls, rs);
    else if (rb == 8) add_sum_w_vec_kernel<8><<<cdiv(cols, 8), EW_THREADS, 0, st>>>(out->p, out->w, l->p, l->w, r->p, r->w, n, ls, rs);
    else add_sum_w_vec_kernel<4><<<cdiv(cols, 4), EW_THREADS, 0, st>>>(out->p, out->w, l->p, l->w, r->p, r->w, n, ls, rs);
  } else if (S >= 65536)
    add_sum_w_kernel<256><<<cdiv(S, 256), EW_THREADS, 0, mt::stream()>>>(out->p, out->w, l->p, l->w, r->p, r->w, (uint32_t)S, ls, rs);
  else if ((l->w >= 512 || r->w >= 512) && S <= 4096)   // many short slices (partial sums of a small gradient): 64 threads share a column
    add_sum_w_kernel<4><<<cdiv(S, 4), EW_THREADS, 0, mt::stream()>>>(out->p, out->w, l->p, l->w, r->p, r->w, (uint32_t)S, ls, rs);
  else
    add_sum_w_kernel<32><<<cdiv(S, 32), EW_THREADS, 0, mt::stream()>>>(out->p, out->w, l->p, l->w, r->p, r->w, (uint32_t)S, ls, rs);
  MT_LAUNCH_CHECK("mt_add_sum_w");
  return MT_OK;
}

int mt_summ_xy(const mt_tensor *out, const mt_tensor *in) {
  if (mt::bad(out) || mt::bad(in)) return mt::fail(MT_E_ARGUMENT, "mt_summ_xy: null tensor");
  mt::note_write(out);
  if (in->z != out->z) return mt::fail(MT_E_SHAPE, "mt_summ_xy: depth of input and output differ");
  uint32_t rows = out->w * out->z;
  if (rows == 0) return MT_OK;
  if (in->w == 0) return mt::fail(MT_E_ARGUMENT, "mt_summ_xy: empty input");
  if (out->y != 1 || out->x != 1) {  // the reference writes element (w,z,0,0) of a larger output; keep that addressing
    return mt::fail(MT_E_ARGUMENT, "mt_summ_xy: output must be [W,Z,1,1]");
  }
  summ_xy_kernel<<<cdiv(rows, EW_THREADS / 64), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, in->w, in->z, in->y * in->x, rows);
  MT_LAUNCH_CHECK("mt_summ_xy");
  return MT_OK;
}

int mt_add_bias(const mt_tensor *t, const mt_tensor *bias) {
  if (mt::bad(t) || mt::bad(bias)) return mt::fail(MT_E_ARGUMENT, "mt_add_bias: null tensor");
  mt::note_write(t);
  if (t->z != bias->z) return mt::fail(MT_E_SHAPE, "mt_add_bias: depth of tensor and bias differ");
  uint32_t rows = t->w * t->z, YX = t->y * t->x;
  if (rows == 0 || YX == 0) return MT_OK;
  if (bias->w == 0 || bias->y != 1 || bias->x != 1) return mt::fail(MT_E_ARGUMENT, "mt_add_bias: bias must be [W,Z,1,1], W >= 1");
  if (YX % 4 == 0 && aligned16(t->p)) {
    dim3 grid4(cdiv(YX / 4, EW_THREADS), plane_blocks(cdiv(YX / 4, EW_THREADS), rows));
    add_bias4_kernel<<<grid4, EW_THREADS, 0, mt::stream()>>>(t->p, bias->p, bias->w, t->z, YX / 4, rows);
    MT_LAUNCH_CHECK("mt_add_bias");
    return MT_OK;
  }
  dim3 grid(cdiv(YX, EW_THREADS), rows < 65535u ? rows : 65535u);
  add_bias_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(t->p, bias->p, bias->w, t->z, YX, rows);
  MT_LAUNCH_CHECK("mt_add_bias");
  return MT_OK;
}

int mt_transponse(const mt_tensor *out, const mt_tensor *in) {
  if (mt::bad(out) || mt::bad(in)) return mt::fail(MT_E_ARGUMENT, "mt_transponse: null tensor");
  mt::note_write(out);
  if (out->y != in->x || out->x != in->y || out->z != in->z || out->w != in->w) return mt::fail(MT_E_SHAPE, "mt_transponse: sizes do not match");
  if (mt::count(in) == 0) return MT_OK;
  uint32_t planes = in->w * in->z;
  if (planes > 65535u) return mt::fail(MT_E_ARGUMENT, "mt_transponse: more than 65535 matrices");
  dim3 grid(cdiv(in->x, 32), cdiv(in->y, 32), planes);
  transponse_kernel<<<grid, dim3(32, 8), 0, mt::stream()>>>(out->p, in->p, in->y, in->x);
  MT_LAUNCH_CHECK("mt_transponse");
  return MT_OK;
}

int mt_upsampling(const mt_tensor *out, const mt_tensor *in, uint32_t ux, uint32_t uy) {
  if (mt::bad(out) || mt::bad(in) || ux == 0 || uy == 0) return mt::fail(MT_E_ARGUMENT, "mt_upsampling: bad argument");
  mt::note_write(out);
  if (in->x != out->x / ux || in->y != out->y / uy || in->z != out->z) return mt::fail(MT_E_SHAPE, "mt_upsampling: sizes do not match");
  uint32_t planes = out->w * out->z, n = out->y * out->x;
  if (planes == 0 || n == 0) return MT_OK;
  if (in->w == 0) return mt::fail(MT_E_ARGUMENT, "mt_upsampling: empty input");
  Geo g{in->w, in->z, in->y, in->x, out->y, out->x};
  if (ux == 2 && uy == 2 && out->x == 2 * in->x && out->y == 2 * in->y && in->x % 2 == 0 && in->x > 0 && aligned16(out->p) && ((uintptr_t)in->p & 7u) == 0) {
    const unsigned bx = cdiv(n / 8, EW_THREADS);
    if (streamed(mt::count(out) * sizeof(float))) upsampling2x2_kernel<true><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, planes);
    else upsampling2x2_kernel<false><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, planes);
    MT_LAUNCH_CHECK("mt_upsampling");
    return MT_OK;
  }
  if (out->x % 4 == 0 && aligned16(out->p) && in->x > 0 && in->y > 0) {
    dim3 grid4(cdiv(n / 4, EW_THREADS), plane_blocks(cdiv(n / 4, EW_THREADS), planes));
    upsampling4_kernel<<<grid4, EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, ux, uy, planes);
    MT_LAUNCH_CHECK("mt_upsampling");
    return MT_OK;
  }
  dim3 grid(cdiv(n, EW_THREADS), planes < 65535u ? planes : 65535u);
  upsampling_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, ux, uy, planes);
  MT_LAUNCH_CHECK("mt_upsampling");
  return MT_OK;
}

int mt_downsampling(const mt_tensor *out, const mt_tensor *in, uint32_t dx, uint32_t dy) {
  if (mt::bad(out) || mt::bad(in) || dx == 0 || dy == 0) return mt::fail(MT_E_ARGUMENT, "mt_downsampling: bad argument");
  mt::note_write(out);
  if (in->x / dx != out->x || in->y / dy != out->y || in->z != out->z || in->w != out->w) return mt::fail(MT_E_SHAPE, "mt_downsampling: sizes do not match");
  uint32_t planes = out->w * out->z, n = out->y * out->x;
  if (planes == 0 || n == 0) return MT_OK;
  Geo g{in->w, in->z, in->y, in->x, out->y, out->x};
  if (dx == 2 && dy == 2 && in->x == 2 * out->x && in->y == 2 * out->y && out->x % 2 == 0 && aligned16(in->p) && ((uintptr_t)out->p & 7u) == 0) {
    const unsigned bx = cdiv(n / 2, EW_THREADS);
    if (streamed(mt::count(in) * sizeof(float))) downsampling2x2_kernel<true><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, planes);
    else downsampling2x2_kernel<false><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, planes);
    MT_LAUNCH_CHECK("mt_downsampling");
    return MT_OK;
  }
  dim3 grid(cdiv(n, EW_THREADS), planes < 65535u ? planes : 65535u);
  downsampling_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, in->p, g, dx, dy, planes);
  MT_LAUNCH_CHECK("mt_downsampling");
  return MT_OK;
}

int mt_max_pooling(const mt_tensor *out, const mt_pos_tensor *pos, const mt_tensor *in, uint32_t px, uint32_t py) {
  if (mt::bad(out) || mt::bad(in) || pos == nullptr || px == 0 || py == 0) return mt::fail(MT_E_ARGUMENT, "mt_max_pooling: bad argument");
  mt::note_write(out);
  mt::note_write(pos->p, (size_t)pos->w * pos->z * pos->y * pos->x * sizeof(mt_spos));
  if (in->x / px != out->x || in->y / py != out->y || in->z != out->z || in->w != out->w) return mt::fail(MT_E_SHAPE, "mt_max_pooling: sizes do not match");
  uint32_t planes = out->w * out->z, n = out->y * out->x;
  if (planes == 0 || n == 0) return MT_OK;
  if (pos->p == nullptr || pos->w == 0 || pos->z != out->z || pos->y != out->y || pos->x != out->x)
    return mt::fail(MT_E_ARGUMENT, "mt_max_pooling: position tensor must be [W',Z,Y,X] of the output");
  Geo g{in->w, in->z, in->y, in->x, out->y, out->x};
  if (px == 2 && py == 2 && in->x == 2 * out->x && in->y == 2 * out->y && out->x % 2 == 0 && aligned16(in->p) && ((uintptr_t)out->p & 7u) == 0 &&
      aligned16(pos->p)) {
    const unsigned bx = cdiv(n / 2, EW_THREADS);
    if (streamed(mt::count(in) * sizeof(float))) max_pooling2x2_kernel<true><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, planes);
    else max_pooling2x2_kernel<false><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, planes);
    MT_LAUNCH_CHECK("mt_max_pooling");
    return MT_OK;
  }
  dim3 grid(cdiv(n, EW_THREADS), planes < 65535u ? planes : 65535u);
  max_pooling_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, px, py, planes);
  MT_LAUNCH_CHECK("mt_max_pooling");
  return MT_OK;
}

int mt_max_pooling_backward(const mt_tensor *out, const mt_pos_tensor *pos, const mt_tensor *in, uint32_t px, uint32_t py) {
  if (mt::bad(out) || mt::bad(in) || pos == nullptr || px == 0 || py == 0) return mt::fail(MT_E_ARGUMENT, "mt_max_pooling_backward: bad argument");
  mt::note_write(out);
  if (in->x != out->x / px || in->y != out->y / py || in->z != out->z || in->w != out->w) return mt::fail(MT_E_SHAPE, "mt_max_pooling_backward: sizes do not match");
  uint32_t planes = out->w * out->z, n = out->y * out->x;
  if (planes == 0 || n == 0) return MT_OK;
  if (pos->p == nullptr || pos->w == 0 || pos->z != in->z || pos->y != in->y || pos->x != in->x)
    return mt::fail(MT_E_ARGUMENT, "mt_max_pooling_backward: position tensor must be [W',Z,Y,X] of the input");
  Geo g{in->w, in->z, in->y, in->x, out->y, out->x};
  if (px == 2 && py == 2 && out->x == 2 * in->x && out->y == 2 * in->y && in->x % 2 == 0 && in->x > 0 && aligned16(out->p) && aligned16(pos->p) &&
      ((uintptr_t)in->p & 7u) == 0) {
    const unsigned bx = cdiv(n / 8, EW_THREADS);
    if (streamed(mt::count(out) * sizeof(float))) max_pooling_backward2x2_kernel<true><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, planes);
    else max_pooling_backward2x2_kernel<false><<<dim3(bx, plane_blocks(bx, planes)), EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, planes);
    MT_LAUNCH_CHECK("mt_max_pooling_backward");
    return MT_OK;
  }
  if (out->x % 4 == 0 && aligned16(out->p) && in->x > 0 && in->y > 0) {
    dim3 grid4(cdiv(n / 4, EW_THREADS), plane_blocks(cdiv(n / 4, EW_THREADS), planes));
    max_pooling_backward4_kernel<<<grid4, EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, px, py, planes);
    MT_LAUNCH_CHECK("mt_max_pooling_backward");
    return MT_OK;
  }
  dim3 grid(cdiv(n, EW_THREADS), planes < 65535u ? planes : 65535u);
  max_pooling_backward_kernel<<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, pos->p, pos->w, in->p, g, px, py, planes);
  MT_LAUNCH_CHECK("mt_max_pooling_backward");
  return MT_OK;
}

int mt_concatecation_z(const mt_tensor *out, const mt_tensor *a, const mt_tensor *b) { return concat_split<true>("mt_concatecation_z", out, a, b); }
int mt_split_z(const mt_tensor *out_a, const mt_tensor *out_b, const mt_tensor *in) { return concat_split<false>("mt_split_z", in, out_a, out_b); }

int mt_set_time_step(const mt_tensor *out, const mt_tensor *in, const mt_u32_tensor *time_step) {
  if (mt::bad(out) || mt::bad(in) || time_step == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_set_time_step: null tensor");
  mt::note_write(out);
  if (!mt::same_zyx(in, out) || in->w != out->w || time_step->w != in->w || time_step->z != 1 || time_step->y != 1 || time_step->x != 1)
    return mt::fail(MT_E_SHAPE, "mt_set_time_step: sizes do not match");
  const size_t size = (size_t)in->z * in->y * in->x;
  if (size == 0 || in->w == 0) return MT_OK;
  if (time_step->p == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_set_time_step: null tensor");
  if (size > 0xffffffffu) return mt::fail(MT_E_ARGUMENT, "mt_set_time_step: sample too large");
  const unsigned bx = cdiv(size, EW_THREADS);
  set_time_step_kernel<<<dim3(bx, plane_blocks(bx, in->w)), EW_THREADS, 0, mt::stream()>>>(out->p, in->p, time_step->p, (uint32_t)size, in->w);
  MT_LAUNCH_CHECK("mt_set_time_step");
  return MT_OK;
}

int mt_create_drop_out_matrix(const mt_tensor *out, float drop_out, uint64_t seed) {
  if (mt::bad(out)) return mt::fail(MT_E_ARGUMENT, "mt_create_drop_out_matrix: null tensor");
  mt::note_write(out);
  const size_t n = mt::count(out);
  if (n == 0) return MT_OK;
  drop_out_kernel<<<stream_blocks(n), EW_THREADS, 0, mt::stream()>>>(out->p, n, drop_out, (float)(1.0 / (1.0 - (double)drop_out)), seed);
  MT_LAUNCH_CHECK("mt_create_drop_out_matrix");
  return MT_OK;
}

int mt_set_normal_noise(const mt_tensor *out, uint64_t seed) {
  if (mt::bad(out)) return mt::fail(MT_E_ARGUMENT, "mt_set_normal_noise: null tensor");
  mt::note_write(out);
  const size_t n = mt::count(out);
  if (n == 0) return MT_OK;
  normal_noise_kernel<<<stream_blocks(n), EW_THREADS, 0, mt::stream()>>>(out->p, nullptr, nullptr, nullptr, 0, nullptr, 0, 1, n, seed);
  MT_LAUNCH_CHECK("mt_set_normal_noise");
  return MT_OK;
}

int mt_get_noise_image_and_noise(const mt_tensor *noisy, const mt_tensor *noise, const mt_tensor *image, const mt_tensor *sqrt_alpha_bar,
                                 const mt_tensor *sqrt_one_minus_alpha_bar, uint64_t seed) {
  const mt_tensor *all[5] = {noisy, noise, image, sqrt_alpha_bar, sqrt_one_minus_alpha_bar};
  for (auto t : all)
    if (mt::bad(t)) return mt::fail(MT_E_ARGUMENT, "mt_get_noise_image_and_noise: null tensor");
  mt::note_write(noisy);
  mt::note_write(noise);
  if (!mt::same_zyx(noisy, noise) || noisy->w != noise->w) return mt::fail(MT_E_SHAPE, "mt_get_noise_image_and_noise: sizes of NoisyImage and Noise differ");
  if (!mt::same_zyx(noisy, image) || noisy->w != image->w) return mt::fail(MT_E_SHAPE, "mt_get_noise_image_and_noise: sizes of NoisyImage and Image differ");
  if (sqrt_alpha_bar->w != image->w || sqrt_one_minus_alpha_bar->w != image->w)
    return mt::fail(MT_E_SHAPE, "mt_get_noise_image_and_noise: SqrtAlphaBar / SqrtOneMinusAlphaBar need one value per sample");
  const size_t n = mt::count(image), per = (size_t)image->z * image->y * image->x;
  if (n == 0) return MT_OK;
  const size_t sa = (size_t)sqrt_alpha_bar->z * sqrt_alpha_bar->y * sqrt_alpha_bar->x, sb = (size_t)sqrt_one_minus_alpha_bar->z * sqrt_one_minus_alpha_bar->y * sqrt_one_minus_alpha_bar->x;
  if (sa == 0 || sb == 0 || sa > 0xffffffffu || sb > 0xffffffffu) return mt::fail(MT_E_SHAPE, "mt_get_noise_image_and_noise: SqrtAlphaBar / SqrtOneMinusAlphaBar need one value per sample");
  normal_noise_kernel<<<stream_blocks(n), EW_THREADS, 0, mt::stream()>>>(noise->p, noisy->p, image->p, sqrt_alpha_bar->p, (uint32_t)sa, sqrt_one_minus_alpha_bar->p,
                                                                         (uint32_t)sb, per, n, seed);
  MT_LAUNCH_CHECK("mt_get_noise_image_and_noise");
  return MT_OK;
}

int mt_adam(const mt_tensor *weight, const mt_tensor *dweight, const mt_tensor *m, const mt_tensor *v, uint32_t batch_size, double speed,
            double beta1, double beta2, double epsilon, double iteration) {
  if (mt::bad(weight) || mt::bad(dweight) || mt::bad(m) || mt::bad(v)) return mt::fail(MT_E_ARGUMENT, "mt_adam: null tensor");
  mt::note_write(weight);
  mt::note_write(m);
  mt::note_write(v);
  const mt_tensor *o[3] = {dweight, m, v};
  for (auto t : o)
    if (!mt::same_zyx(weight, t) || weight->w != t->w) return mt::fail(MT_E_SHAPE, "mt_adam: sizes do not match");
  size_t n = mt::count(weight);
  if (n == 0) return MT_OK;
  const AdamStep step{(float)batch_size, speed, beta1, beta2, epsilon, 1.0 - pow(beta1, iteration), 1.0 - pow(beta2, iteration)};
  adam_kernel<<<cdiv(n, EW_THREADS), EW_THREADS, 0, mt::stream()>>>(weight->p, dweight->p, m->p, v->p, n, step);
  MT_LAUNCH_CHECK("mt_adam");
  return MT_OK;
}

int mt_fill_many(uint32_t count, const mt_tensor *const *tensors, float value) {
  if (count && tensors == nullptr) return mt::fail(MT_E_ARGUMENT, "mt_fill_many: null list");
  for (uint32_t i = 0; i < count; i++)
    if (mt::bad(tensors[i])) return mt::fail(MT_E_ARGUMENT, "mt_fill_many: null tensor (entry %u)", i);
  for (uint32_t i = 0; i < count; i++) mt::note_write(tensors[i]);
  for (uint32_t first = 0; first < count;) {
    ManyFill a{};
    uint32_t used = 0;
    for (; first < count && used < (uint32_t)MANY; first++) {
      const size_t n = mt::count(tensors[first]);
      if (n == 0) continue;
      unsigned blocks = cdiv(n, (size_t)EW_THREADS * 4);  // a few stores per thread
      if (blocks > 2048u) blocks = 2048u;
      a.p[used] = tensors[first]->p; a.n[used] = n; a.first_block[used + 1] = a.first_block[used] + blocks;
      used++;
    }
    if (used == 0) continue;
    mt::ProfileScope prof("mt_fill_many");
    fill_many_kernel<<<a.first_block[used], EW_THREADS, 0, mt::stream()>>>(a, used, value);
    MT_LAUNCH_CHECK("mt_fill_many");
  }
  return MT_OK;
}

int mt_adam_many(uint32_t count, const mt_tensor *const *weight, const mt_tensor *const *dweight, const mt_tensor *const *m, const mt_tensor *const *v,
                 uint32_t batch_size, double speed, double beta1, double beta2, double epsilon, double iteration) {
  if (count && (weight == nullptr || dweight == nullptr || m == nullptr || v == nullptr)) return mt::fail(MT_E_ARGUMENT, "mt_adam_many: null list");
  mt::PackRefresh found[MANY_PACKS];
  uint32_t found_for[MANY_PACKS], nfound = 0;
  for (uint32_t i = 0; i < count; i++) {
    if (mt::bad(weight[i]) || mt::bad(dweight[i]) || mt::bad(m[i]) || mt::bad(v[i])) return mt::fail(MT_E_ARGUMENT, "mt_adam_many: null tensor (entry %u)", i);
    // (looked up before the write is reported: only a copy that is current now can be kept current by this step)
    if (nfound < (uint32_t)MANY_PACKS && mt::count(weight[i]) <= 0xffffffffu && mt::pack_refresh_find(weight[i]->p, mt::count(weight[i]), &found[nfound])) found_for[nfound++] = i;
    mt::note_write(weight[i]);
    mt::note_write(m[i]);
    mt::note_write(v[i]);
    const mt_tensor *o[3] = {dweight[i], m[i], v[i]};
    for (auto t : o)
      if (!mt::same_zyx(weight[i], t) || weight[i]->w != t->w) return mt::fail(MT_E_SHAPE, "mt_adam_many: sizes do not match (entry %u)", i);
  }
  const AdamStep step{(float)batch_size, speed, beta1, beta2, epsilon, 1.0 - pow(beta1, iteration), 1.0 - pow(beta2, iteration)};
  for (uint32_t first = 0; first < count;) {
    ManyAdam a{};
    ManyAdamPacks packs{};
    uint32_t refresh[MANY_PACKS];
    uint32_t used = 0, kept = 0;
    for (; first < count && used < (uint32_t)MANY; first++) {
      const size_t n = mt::count(weight[first]);
      if (n == 0) continue;
      const bool vec = g_adam_vec && n % 4 == 0 && aligned16(weight[first]->p) && aligned16(dweight[first]->p) && aligned16(m[first]->p) && aligned16(v[first]->p);
      unsigned blocks = cdiv(vec ? n / 4 : n, EW_THREADS);
      a.weight[used] = weight[first]->p; a.dweight[used] = dweight[first]->p; a.m[used] = m[first]->p; a.v[used] = v[first]->p;
      a.n[used] = n;
      if (vec) a.vec |= 1u << used;
      packs.slot[used] = -1;
      uint32_t k = 0;
      while (k < nfound && found_for[k] != first) k++;
      if (k < nfound) {
        const mt::PackRefresh &r = found[k];
        refresh[kept] = k;
        AdamPack &p = packs.pack[kept];
        p.packed = r.packed; p.ker_ld = r.ker_ld; p.co_stride = r.co_stride; p.ci_stride = r.ci_stride;
        for (int f = 0; f < 4; f++) { p.begin[f] = r.begin[f]; p.phase_of[f] = r.phase_of[f]; }
        const uint32_t CO = r.ker_ld / 16u, CI = (uint32_t)(n / r.ker_ld);
        p.tiles_co = vec && CO % 16 == 0 && CI % 16 == 0 && r.ci_stride == 4 && r.co_stride % 4 == 0 && aligned16(r.packed) ? CO / 16u : 0u;
        if (p.tiles_co) blocks = (unsigned)(n / 4096);
        else { blocks = cdiv(n, EW_THREADS); a.vec &= ~(1u << used); }
        packs.slot[used] = (int8_t)kept++;
      } else if (vec && g_adam_vec == 1) {
        blocks = cdiv(n, EW_THREADS); a.vec &= ~(1u << used);
      }
      if (blocks > 4096u) blocks = 4096u;
      a.first_block[used + 1] = a.first_block[used] + blocks;
      used++;
    }
    if (used == 0) continue;
    mt::ProfileScope prof("mt_adam_many");
    if (kept) adam_many_packs_kernel<<<a.first_block[used], EW_THREADS, 0, mt::stream()>>>(a, packs, used, step);
    else adam_many_kernel<<<a.first_block[used], EW_THREADS, 0, mt::stream()>>>(a, used, step);
    MT_LAUNCH_CHECK("mt_adam_many");
    for (uint32_t k = 0; k < kept; k++) mt::pack_refresh_commit(found[refresh[k]], weight, m, v, count);
  }
  return MT_OK;
}

// fixed_scratch: the entry point that allocates nothing -- statistics the caller does not ask for go to the library's
// fixed array (at most STATIC_SCRATCH_FLOATS / 3 elements per sample) and no launch is bracketed by profiling events.
static int bn_forward_train(const mt_tensor *out, const mt_tensor *in, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *xhat,
                            const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean,
                            const mt_tensor *new_variable, float momentum, float epsilon, int func, bool fixed_scratch,
                            const mt_tensor *old_mean = nullptr, const mt_tensor *old_variable = nullptr, const mt_tensor *pre = nullptr) {
  if (pre && (mt::bad(pre) || !mt::same_zyx(pre, in) || pre->w != in->w || pre->p == out->p || (xhat && pre->p == xhat->p) || pre->p == in->p))
    return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_train_from: the tensor for gamma*xhat+beta must have the input's sizes and be a tensor of its own");
  mt::note_write(pre);
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_forward_train_func: unknown function id %d", func);
  if ((old_mean && !new_mean) || (old_variable && !new_variable)) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_forward_train_from: a statistic to blend from needs one to blend into");
  for (auto t : {old_mean, old_variable})
    if (t && (mt::bad(t) || !mt::same_zyx(t, in) || t->w == 0)) return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_train_from: statistics must be [1,Z,Y,X]");
  if (mt::bad(out) || mt::bad(in) || mt::bad(gamma) || mt::bad(beta)) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_forward_train_func: null tensor");
  for (auto t : {out, xhat, ivar, batch_mean, batch_var, new_mean, new_variable}) mt::note_write(t);
  if (!mt::same_zyx(in, out) || in->w != out->w || !mt::same_zyx(gamma, in) || !mt::same_zyx(beta, in) || gamma->w == 0 || beta->w == 0)
    return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_train_func: sizes do not match");
  const mt_tensor *stats[5] = {ivar, batch_mean, batch_var, new_mean, new_variable};
  for (auto t : stats)
    if (t && (mt::bad(t) || !mt::same_zyx(t, in) || t->w == 0)) return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_train_func: statistics must be [1,Z,Y,X]");
  if (xhat && (mt::bad(xhat) || !mt::same_zyx(xhat, in) || xhat->w != in->w)) return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_train_func: xhat must match the input");
  size_t S = (size_t)in->z * in->y * in->x;
  uint32_t W = in->w;
  if (S == 0 || W == 0) return MT_OK;
  float *spare = nullptr;
  int rc = MT_OK;
  if (fixed_scratch) {
    if (3 * S > STATIC_SCRATCH_FLOATS)
      return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_forward_train_func_noalloc: %zu elements per sample, the fixed scratch array holds statistics for at most %zu",
                      S, STATIC_SCRATCH_FLOATS / 3);
    rc = static_scratch(&spare);
  } else {
    rc = bn_scratch(3 * S, &spare);
  }
  if (rc) return rc;
  mt::ProfileMute mute(fixed_scratch);
  float *pm = batch_mean ? batch_mean->p : spare, *pv = batch_var ? batch_var->p : spare + S, *pi = ivar ? ivar->p : spare + 2 * S;
  float inv_n = (float)(1.0 / (double)(float)W);  // the layer passes 1.0/N with N a float
  float mom_new = (float)(1.0 - (double)momentum);  // and 1.0-Momentum, rounded once
  float *nm = new_mean ? new_mean->p : nullptr, *nv = new_variable ? new_variable->p : nullptr;
  const float *om = old_mean ? old_mean->p : nm, *ov = old_variable ? old_variable->p : nv;
  float *pp = pre ? pre->p : nullptr;
  bool vec = (S % 4 == 0) && aligned16(out->p) && aligned16(in->p) && aligned16(gamma->p) && aligned16(beta->p) && aligned16(pm) && aligned16(pi) && (!xhat || aligned16(xhat->p)) &&
             (!pp || aligned16(pp));
  if (vec && mt::epilogue_func(func)) {
    // one pass: the widest column block that still gives every compute unit a few blocks, if the batch share fits
    // (a small batch on a large tensor: 64 column groups, so that a thread still has 8 to 16 loads in flight)
    int rb = S / 256 >= 512 && cdiv(W, 4) <= 16 ? 64 : S / 128 >= 512 ? 32 : S / 64 >= 512 ? 16 : 8;
    if (W > 512 && W <= 2048) {
      // a large batch: blocks of 1024 threads, 64 slices of 16 column groups (128 of 8 beyond a batch of 1024)
      mt::ProfileScope prof("bn_fused");
      const int big_rb = W <= 1024 ? 16 : 8;
      const unsigned grid = cdiv(S, (size_t)big_rb * 4);
#define MT_BN_FUSED_BIG(RB, NT) \
  bn_fused_kernel<RB, 16, 1024, NT><<<grid, 1024, 0, mt::stream()>>>(out->p, xhat ? xhat->p : nullptr, in->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, gamma->p, beta->p, func, om, ov, pp)
      const bool past_caches = streamed(S * W * sizeof(float));   // (116 against 125 us for a 268 MB tensor)
      if (big_rb == 16 && past_caches) MT_BN_FUSED_BIG(16, true); else if (big_rb == 16) MT_BN_FUSED_BIG(16, false);
      else if (past_caches) MT_BN_FUSED_BIG(8, true); else MT_BN_FUSED_BIG(8, false);
#undef MT_BN_FUSED_BIG
      MT_LAUNCH_CHECK("bn_fused");
      return MT_OK;
    }
    const uint32_t nw = cdiv(W, EW_THREADS / rb);
    if (nw <= 32) {
      mt::ProfileScope prof("bn_fused");
      const unsigned grid = cdiv(S, (size_t)rb * 4);
#define MT_BN_FUSED(RB, NW) \
  bn_fused_kernel<RB, NW><<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, xhat ? xhat->p : nullptr, in->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, gamma->p, beta->p, func, om, ov, pp)
#define MT_BN_FUSED_NW(RB) \
  do { if (nw <= 8) MT_BN_FUSED(RB, 8); else if (nw <= 16) MT_BN_FUSED(RB, 16); else MT_BN_FUSED(RB, 32); } while (0)
      if (rb == 64 && streamed(S * W * sizeof(float))) {   // a large tensor, every element touched once: past the caches
#define MT_BN_FUSED_NT(NW) \
  bn_fused_kernel<64, NW, EW_THREADS, true><<<grid, EW_THREADS, 0, mt::stream()>>>(out->p, xhat ? xhat->p : nullptr, in->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, gamma->p, beta->p, func, om, ov, pp)
        if (nw <= 8) MT_BN_FUSED_NT(8); else MT_BN_FUSED_NT(16);
#undef MT_BN_FUSED_NT
      }
      else if (rb == 64) { if (nw <= 8) MT_BN_FUSED(64, 8); else MT_BN_FUSED(64, 16); }
      else if (rb == 32) MT_BN_FUSED_NW(32); else if (rb == 16) MT_BN_FUSED_NW(16); else MT_BN_FUSED_NW(8);
#undef MT_BN_FUSED_NW
#undef MT_BN_FUSED
      MT_LAUNCH_CHECK("bn_fused");
      return MT_OK;
    }
  }
  {
  mt::ProfileScope prof("bn_stats");
  if (S % 4 == 0 && aligned16(in->p))
    bn_stats_kernel<4><<<cdiv(S, 128), EW_THREADS, 0, mt::stream()>>>(in->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, om, ov);
  else
    bn_stats_kernel<1><<<cdiv(S, 32), EW_THREADS, 0, mt::stream()>>>(in->p, W, (uint32_t)S, inv_n, epsilon, pm, pv, pi, nm, nv, momentum, mom_new, om, ov);
  }
  MT_LAUNCH_CHECK("bn_stats");
  unsigned gx = cdiv(vec ? S / 4 : S, EW_THREADS);
  unsigned gy = W < 16 ? W : 16;  // a few batch slices per column block keeps the per-column loads in registers
  mt::ProfileScope prof("bn_apply");
  bn_apply_kernel<<<dim3(gx, gy), EW_THREADS, 0, mt::stream()>>>(out->p, xhat ? xhat->p : nullptr, in->p, pm, pi, gamma->p, beta->p, (uint32_t)S, W, vec, func, pp);
  MT_LAUNCH_CHECK("bn_apply");
  return MT_OK;
}

int mt_batchnorm_forward_train_func(const mt_tensor *out, const mt_tensor *in, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *xhat,
                                    const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean,
                                    const mt_tensor *new_variable, float momentum, float epsilon, int func) {
  return bn_forward_train(out, in, gamma, beta, xhat, ivar, batch_mean, batch_var, new_mean, new_variable, momentum, epsilon, func, false);
}

int mt_batchnorm_forward_train_from(const mt_tensor *out, const mt_tensor *in, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *xhat,
                                    const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean,
                                    const mt_tensor *new_variable, const mt_tensor *old_mean, const mt_tensor *old_variable, float momentum, float epsilon,
                                    int func, const mt_tensor *pre_function) {
  return bn_forward_train(out, in, gamma, beta, xhat, ivar, batch_mean, batch_var, new_mean, new_variable, momentum, epsilon, func, false, old_mean, old_variable,
                          pre_function);
}

int mt_batchnorm_forward_train_func_noalloc(const mt_tensor *out, const mt_tensor *in, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *xhat,
                                            const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean,
                                            const mt_tensor *new_variable, float momentum, float epsilon, int func) {
  return bn_forward_train(out, in, gamma, beta, xhat, ivar, batch_mean, batch_var, new_mean, new_variable, momentum, epsilon, func, true);
}

int mt_batchnorm_forward_infer_func(const mt_tensor *out, const mt_tensor *in, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *mean,
                                    const mt_tensor *variable, float epsilon, int func) {
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_forward_infer_func: unknown function id %d", func);
  const mt_tensor *all[6] = {out, in, gamma, beta, mean, variable};
  for (auto t : all)
    if (mt::bad(t)) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_forward_infer_func: null tensor");
  mt::note_write(out);
  if (!mt::same_zyx(in, out) || in->w != out->w) return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_infer_func: sizes do not match");
  for (int i = 2; i < 6; i++)
    if (!mt::same_zyx(all[i], in) || all[i]->w == 0) return mt::fail(MT_E_SHAPE, "mt_batchnorm_forward_infer_func: parameters must be [1,Z,Y,X]");
  size_t S = (size_t)in->z * in->y * in->x;
  uint32_t W = in->w;
  if (S == 0 || W == 0) return MT_OK;
  float *scratch = nullptr;
  int rc = bn_scratch(3 * S, &scratch);
  if (rc) return rc;
  bn_ivar_kernel<<<cdiv(S, EW_THREADS), EW_THREADS, 0, mt::stream()>>>(scratch, variable->p, (uint32_t)S, epsilon);
  MT_LAUNCH_CHECK("bn_ivar");
  bool vec = (S % 4 == 0) && aligned16(out->p) && aligned16(in->p) && aligned16(gamma->p) && aligned16(beta->p) && aligned16(mean->p);
  unsigned gx = cdiv(vec ? S / 4 : S, EW_THREADS);
  unsigned gy = W < 16 ? W : 16;
  bn_apply_kernel<<<dim3(gx, gy), EW_THREADS, 0, mt::stream()>>>(out->p, nullptr, in->p, mean->p, scratch, gamma->p, beta->p, (uint32_t)S, W, vec, func);
  MT_LAUNCH_CHECK("bn_apply");
  return MT_OK;
}

int mt_batchnorm_backward(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta, const mt_tensor *gamma,
                          const mt_tensor *xhat, const mt_tensor *ivar) {
  return mt_batchnorm_backward_func(error, dgamma, dbeta, delta, gamma, nullptr, xhat, ivar, MT_F_NONE);
}

int mt_batchnorm_backward_func(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta, const mt_tensor *gamma,
                               const mt_tensor *beta, const mt_tensor *xhat, const mt_tensor *ivar, int func) {
  return bn_backward_any(error, dgamma, dbeta, delta, gamma, beta, xhat, ivar, func, nullptr, nullptr, nullptr);
}

int mt_batchnorm_backward_keep(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta, const mt_tensor *gamma,
                               const mt_tensor *xhat, const mt_tensor *ivar, const mt_tensor *dxhat, const mt_tensor *sum_dxhat, const mt_tensor *sum_dxhat_xhat) {
  return bn_backward_any(error, dgamma, dbeta, delta, gamma, nullptr, xhat, ivar, MT_F_NONE, dxhat, sum_dxhat, sum_dxhat_xhat);
}

int mt_batchnorm_backward_func_keep(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta, const mt_tensor *gamma,
                                    const mt_tensor *beta, const mt_tensor *xhat, const mt_tensor *ivar, int func, const mt_tensor *dxhat,
                                    const mt_tensor *sum_dxhat, const mt_tensor *sum_dxhat_xhat, const mt_tensor *delta_front) {
  return bn_backward_any(error, dgamma, dbeta, delta, gamma, beta, xhat, ivar, func, dxhat, sum_dxhat, sum_dxhat_xhat, delta_front);
}

}  // extern "C"

static int bn_backward_any(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta, const mt_tensor *gamma,
                           const mt_tensor *beta, const mt_tensor *xhat, const mt_tensor *ivar, int func, const mt_tensor *keep_dxhat, const mt_tensor *keep_s1,
                           const mt_tensor *keep_s2, const mt_tensor *keep_front) {
  if (!mt::valid_func(func, true) || (func != MT_F_NONE && (func & MT_F_DIFFERENTIAL))) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_backward: unknown function id %d", func);
  if (func == MT_F_LINEAR) func = MT_F_NONE;  // derivative 1
  const mt_tensor *need[5] = {error, delta, gamma, xhat, ivar};
  for (auto t : need)
    if (mt::bad(t)) return mt::fail(MT_E_ARGUMENT, "mt_batchnorm_backward: null tensor");
  for (auto t : {error, dgamma, dbeta, keep_dxhat, keep_s1, keep_s2, keep_front}) mt::note_write(t);
  if (keep_front && (mt::bad(keep_front) || !mt::same_zyx(keep_front, delta) || keep_front->w != delta->w || keep_front->p == error->p ||
                     (keep_dxhat && keep_front->p == keep_dxhat->p)))
    return mt::fail(MT_E_SHAPE, "mt_batchnorm_backward_func_keep: delta_front must have the sizes of delta and be neither the error nor dxhat");
  if (keep_dxhat && (mt::bad(keep_dxhat) || !mt::same_zyx(keep_dxhat, delta) || keep_dxhat->w != delta->w || keep_dxhat->p == delta->p || keep_dxhat->p == error->p))
    return mt::fail(MT_E_SHAPE, "mt_batchnorm_backward_keep: dxhat must be a tensor of its own with the sizes of delta");
  for (auto t : {keep_s1, keep_s2})
    if (t && (mt::bad(t) || !mt::same_zyx(t, delta) || t->w == 0)) return mt::fail(MT_E_SHAPE, "mt_batchnorm_backward_keep: the sums must be [1,Z,Y,X]");
  if (func != MT_F_NONE && (mt::bad(beta) || !mt::same_zyx(beta, delta) || beta->w == 0))
    return mt::fail(MT_E_SHAPE, "mt_batchnorm_backward: beta must be [1,Z,Y,X] when a function is given");
  if (!mt::same_zyx(error, delta) || error->w != delta->w || !mt::same_zyx(xhat, delta) || xhat->w != delta->w || !mt::same_zyx(gamma, delta) ||
      !mt::same_zyx(ivar, delta) || gamma->w == 0 || ivar->w == 0)
    return mt::fail(MT_E_SHAPE, "mt_batchnorm_backward: sizes do not match");
  for (auto t : {dgamma, dbeta})
    if (t && (mt::bad(t) || !mt::same_zyx(t, delta) || t->w == 0)) return mt::fail(MT_E_SHAPE, "mt_batchnorm_backward: gradients must be [1,Z,Y,X]");
  const size_t S = (size_t)delta->z * delta->y * delta->x;
  const uint32_t W = delta->w;
  if (S == 0 || W == 0) return MT_OK;
  const float n = (float)W, inv_n = (float)(1.0 / (double)n);
  float *pg = dgamma ? dgamma->p : nullptr, *pb = dbeta ? dbeta->p : nullptr;
  const bool cheap = func == MT_F_NONE || func == MT_F_RELU || func == MT_F_LEAKY_RELU;
  const bool vec = cheap && S % 4 == 0 && aligned16(error->p) && aligned16(delta->p) && aligned16(gamma->p) && aligned16(xhat->p) && aligned16(ivar->p) &&
                   (func == MT_F_NONE || aligned16(beta->p)) && (!keep_dxhat || aligned16(keep_dxhat->p)) && (!keep_front || aligned16(keep_front->p));
  if (!vec) {
    // any layout, any function: the layers' own sequences of tensor operations, on workspace tensors
    float *ws = nullptr;
    int rc = bn_scratch(2 * S + 3 * (size_t)W * S, &ws);
    if (rc) return rc;
    mt_tensor s1{keep_s1 ? keep_s1->p : ws, 1, delta->z, delta->y, delta->x}, s2{keep_s2 ? keep_s2->p : ws + S, 1, delta->z, delta->y, delta->x};
    mt_tensor dx{keep_dxhat ? keep_dxhat->p : ws + 2 * S, W, delta->z, delta->y, delta->x}, t{ws + 2 * S + (size_t)W * S, W, delta->z, delta->y, delta->x};
    mt_tensor front{keep_front ? keep_front->p : ws + 2 * S + 2 * (size_t)W * S, W, delta->z, delta->y, delta->x};
    if (func != MT_F_NONE) {  // the function layer: delta * f'(gamma*xhat + beta)
      if ((rc = mt_tensor_item_production(&t, gamma, xhat)) || (rc = mt_add(&t, &t, beta, 1.f, 1.f))) return rc;
      if ((rc = mt_apply_func(&t, &t, MT_F_DIFFERENTIAL + func)) || (rc = mt_tensor_item_production(&front, delta, &t))) return rc;
      delta = &front;
    } else if (keep_front && keep_front->p != delta->p) {
      if ((rc = mt_set(&front, delta, 1.f, 0.f))) return rc;
    }
    if ((rc = mt_fill(&s1, 0.f)) || (rc = mt_fill(&s2, 0.f))) return rc;
    if ((rc = mt_tensor_item_production(&dx, delta, gamma)) || (rc = mt_add_sum_w(&s1, &s1, &dx, 1.f, 1.f))) return rc;
    if ((rc = mt_tensor_item_production(&t, &dx, xhat)) || (rc = mt_add_sum_w(&s2, &s2, &t, 1.f, 1.f))) return rc;
    if (dgamma && ((rc = mt_tensor_item_production(&t, delta, xhat)) || (rc = mt_add_sum_w(dgamma, dgamma, &t, 1.f, 1.f)))) return rc;
    if (dbeta && (rc = mt_add_sum_w(dbeta, dbeta, delta, 1.f, 1.f))) return rc;
    if ((rc = mt_mul_value(error, &dx, n)) || (rc = mt_tensor_item_production(&t, xhat, &s2))) return rc;
    if ((rc = mt_sub(error, error, &t, 1.f, 1.f)) || (rc = mt_sub(error, error, &s1, 1.f, 1.f))) return rc;
    if ((rc = mt_tensor_item_production(error, error, ivar))) return rc;
    return mt_mul_value(error, error, inv_n);
  }
  mt::ProfileScope prof("bn_backward");
  if (W > 512 && W <= 1024) {  // a large batch: 1024 threads, 128 slices of 8 column groups, 8 rows of both tensors per thread
    bn_backward_kernel<8, 8, 1024><<<cdiv(S, (size_t)32), 1024, 0, mt::stream()>>>(error->p, pg, pb, delta->p, gamma->p, beta ? beta->p : nullptr, xhat->p, ivar->p, W,
                                                                               (uint32_t)S, n, inv_n, func, keep_dxhat ? keep_dxhat->p : nullptr,
                                                                               keep_s1 ? keep_s1->p : nullptr, keep_s2 ? keep_s2->p : nullptr,
                                                                               keep_front ? keep_front->p : nullptr);
    MT_LAUNCH_CHECK("mt_batchnorm_backward");
    return MT_OK;
  }
  int rb = S / 128 >= 512 ? 32 : S / 64 >= 512 ? 16 : 8;
  while (rb > 8 && cdiv(W, EW_THREADS / rb) > 16) rb /= 2;
  const uint32_t nw = cdiv(W, EW_THREADS / rb);
  const unsigned grid = cdiv(S, (size_t)rb * 4);
#define MT_BN_BWD(RB, NW) \
  bn_backward_kernel<RB, NW><<<grid, EW_THREADS, 0, mt::stream()>>>(error->p, pg, pb, delta->p, gamma->p, beta ? beta->p : nullptr, xhat->p, ivar->p, W, \
                                                                    (uint32_t)S, n, inv_n, func, keep_dxhat ? keep_dxhat->p : nullptr, keep_s1 ? keep_s1->p : nullptr, \
                                                                    keep_s2 ? keep_s2->p : nullptr, keep_front ? keep_front->p : nullptr)
#define MT_BN_BWD_NW(RB) \
  do { if (nw <= 4) MT_BN_BWD(RB, 4); else if (nw <= 8) MT_BN_BWD(RB, 8); else if (nw <= 16) MT_BN_BWD(RB, 16); else MT_BN_BWD(RB, 0); } while (0)
  if (rb == 32) MT_BN_BWD_NW(32); else if (rb == 16) MT_BN_BWD_NW(16); else MT_BN_BWD_NW(8);
#undef MT_BN_BWD_NW
#undef MT_BN_BWD
  MT_LAUNCH_CHECK("mt_batchnorm_backward");
  return MT_OK;
}

extern "C" {

int mt_vae_coder_output(const mt_tensor *out, const mt_tensor *kl_loss, const mt_tensor *mu, const mt_tensor *logvar, const mt_tensor *epsilon) {
  const mt_tensor *need[4] = {out, mu, logvar, epsilon};
  for (auto t : need)
    if (mt::bad(t)) return mt::fail(MT_E_ARGUMENT, "mt_vae_coder_output: null tensor");
  mt::note_write(out);
  mt::note_write(kl_loss);
  for (auto t : {mu, logvar, epsilon})
    if (!mt::same_zyx(t, out) || t->w != out->w) return mt::fail(MT_E_SHAPE, "mt_vae_coder_output: sizes do not match");
  if (kl_loss && (mt::bad(kl_loss) || mt::count(kl_loss) < 1)) return mt::fail(MT_E_ARGUMENT, "mt_vae_coder_output: kl_loss must hold one value");
  const size_t n = mt::count(out);
  if (n == 0) return MT_OK;
  unsigned blocks = cdiv(n, (size_t)EW_THREADS * 4);
  if (blocks > 1024) blocks = 1024;
  float *partial = nullptr;
  int rc = bn_scratch(blocks, &partial);
  if (rc) return rc;
  vae_coder_kernel<<<blocks, EW_THREADS, 0, mt::stream()>>>(out->p, partial, mu->p, logvar->p, epsilon->p, n);
  MT_LAUNCH_CHECK("mt_vae_coder_output");
  if (kl_loss) {
    vae_kl_kernel<<<1, 1, 0, mt::stream()>>>(kl_loss->p, partial, blocks, (float)out->w);
    MT_LAUNCH_CHECK("mt_vae_coder_output");
  }
  return MT_OK;
}

}  // extern "C"
