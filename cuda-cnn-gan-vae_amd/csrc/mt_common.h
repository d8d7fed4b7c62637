// Shared host/device helpers of libmi355tensor (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "mi355_tensor.h"

namespace mt {

// ---- host side: stream, error latch -------------------------------------------------------
hipStream_t stream();
int fail(int code, const char *fmt, ...);  // records the message, returns `code`
int hip_fail(hipError_t e, const char *what);
// split-K: workspace for S partial results, and out[i] = func(sum_s partial[s][i] + bias[(i / bias_div) % bias_mod])
int split_workspace(size_t floats, float **p);
int split_reduce(const char *name, float *out, const float *partial, uint32_t S, size_t n, const float *bias, uint32_t bias_div, uint32_t bias_mod, int func);
int set_conv_path(int v);  // 0 auto, 1 direct kernels, 2 matrix cores wherever they apply
int set_igemm_tile(int v); // -1 auto, 0..4 force one block tile of the matrix-core kernels
int set_patch_blocks(int v);
int set_image_mfma(int v);
int set_walk_blocks(int v);
int set_walk_waves(int v);
int set_walk_tm(int v);
int set_walk_order(int v);
int set_walk_fair(int v);
int set_igemm_fair(int v);
int set_first_layer(int v);   // forward convolutions of 3-channel images on the input-patch kernel: 0 never, 1 wherever the shape allows
int set_nontemporal(int v);   // streaming kernels read and write past the caches: 0 never, 1 always, 2 tensors of 128 MiB and more
int set_image_strip(int v);   // rows per strip of the image layer's product kernel on 64-column images (0: choose)
int set_conv_patch(int v);     // 3x3 stride-1 forward convolutions from at most 32 channels on large images from patches in LDS: 1 (default) / 0 never / n: from n filters on
int set_tconv_as_conv(int v);  // stride-1 transposed convolutions with 3x3 (5x5 ...) taps as forward convolutions with flipped kernels: 1 (default) / 0 never
int set_tconv_merge(int v);  // 5x5 stride-2 padding-2 transposed convolutions to 5..16 channels as one 3x3 convolution to (channel, phase) rows: 1 (default) / 0 never
int set_tconv_patch(int v);  // 3x3 stride-1 transposed convolutions from at most 32 filters on large images from patches in LDS: 1 (default) / 0 never
int set_wgrad_patch(int v);  // the batch-summed weight gradient of 3x3 stride-1 layers with at most 32 filters on large images from patches in LDS: 1 (default) / 0 never
int set_wgrad_pad(int v);    // the batch-summed weight gradient on delta padded with rows of zeros where its images do not fill whole k steps: 1 (default) / 0 never
int set_wgrad_parts(int v);  // the general batch-summed weight gradient in bands of output rows per sample: 1 (default) where samples x tiles are few, 0 never, n bands
int set_walk_wide(int v);    // 1 (default): the walking kernel in blocks of 32 rows x 128 columns for 32 (96, ...) output channels; 0: never
int set_upconv_split(int v); // 1 (default): up-sampling convolutions with too few tiles share a tile's k steps between blocks; 0: never
int set_upconv_walk(int v);  // mt_upsampling_convolution_func on the walking kernel from this many blocks (0: never)
int set_wgrad_walk(int v);    // batch-summed weight gradients as one k loop per block: 0 never, 1 wherever the shape allows
int set_conv_walk(int v);     // forward convolutions on the kernel whose blocks walk over the batch: 0 never, 1 wherever the shape allows
int set_tconv_walk(int v);    // blocks of a transposed convolution that walk over the batch: 0 never for plain calls, 1 wherever the shape allows
// out = func(scale * in + shift) with the pairs (scale, shift) per element [Z][Y][X] of one sample (func: a cheap one)
int norm_apply(const mt_tensor *out, const mt_tensor *in, const float *scale_shift, int func);
// statistics of x over the batch as a separate pass: (scale, shift) pairs of the batch normalisation that follows, and
// the optional outputs of mt_batchnorm_forward_train_func
int bn_statistics(const mt_tensor *x, const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *scale_shift, const mt_tensor *ivar,
                  const mt_tensor *mean, const mt_tensor *var, const mt_tensor *new_mean, const mt_tensor *new_var, float momentum, float epsilon);  // persistent blocks of the input-patch transposed convolution (default 512)
int set_wgrad_groups(int v);  // 0 auto, else batch groups of the batch-summed weight gradient

// A library-owned device buffer that grows on demand.  Recorded HIP graphs keep the pointers of the recording:
// a request that does not fit while the stream is being captured is an error (run the sequence once eagerly
// first), and a block that a capture may have seen is kept alive when a later request outgrows it.
struct Workspace {
  float *p = nullptr;
  size_t floats = 0;
  bool captured = false;  // handed out while the work stream was being captured
};
int workspace_get(Workspace &ws, const char *what, size_t floats, float **p);
size_t retired_workspaces();
void count_driver_allocation();  // every hipMalloc of the library is counted (mt_get_info "driver_allocations")
// Re-ordered copies of weights are kept between calls, keyed by the weights' address and shape.  Every library call
// that writes device memory reports the range here (so does mt_invalidate for writers outside the library); copies
// made from an overlapping range are then made again on their next use.
void note_write(const void *p, size_t bytes);
void forget_graph_writes(const void *p, size_t bytes);  // the block at p is released: recorded writes into it no longer count
int add_sum_w_pair(float *out1, const float *r1, size_t S1, float *out2, const float *r2, size_t S2, uint32_t W);  // two batch sums, one launch
int set_pack_cache(int on);
int set_adam_vec(int v);      // mt_adam_many updates four elements per thread: 1 (default) in the tiles that also write a re-ordered copy, 2 wherever the tensors allow, 0 never (measurements only)
int set_pack_refresh(int v);  // 1 (default): mt_adam_many keeps the re-ordered copies of 4x4 stride-2 transposed-convolution weights current; 0: never
struct PackRefresh {          // where mt_adam_many writes such a copy: tap t of (channel co, filter ci) in phase f at packed[begin[f] + co*co_stride + ci*ci_stride + t]
  float *packed;
  uint32_t ker_ld, co_stride, ci_stride, begin[4];
  uint8_t phase_of[4];
  size_t entry;
};
bool pack_refresh_find(const float *kernel, size_t floats, PackRefresh *r);
void pack_refresh_commit(const PackRefresh &r, const mt_tensor *const *weight, const mt_tensor *const *m, const mt_tensor *const *v, uint32_t count);
bool pack_cache_info(const char *name, int64_t *value);
int static_scratch_setup();  // looks up the device address of the fixed scratch array for the current device

// Brackets the launches made inside its lifetime with two events on the work stream when profiling is enabled
// (mt_profile_enable); `label` must be a string literal.
struct ProfileScope {
  explicit ProfileScope(const char *label);
  ~ProfileScope();
  int slot;
};
bool profiling();
struct ProfileMute {  // while alive (and `on`): scopes record nothing, so no event is created
  explicit ProfileMute(bool on);
  ~ProfileMute();
  bool on;
};
const char *intern_label(const char *name, const char *suffix);  // "name[suffix]" with process lifetime

#define MT_HIP(call)                                         \
  do {                                                       \
    hipError_t e_ = (call);                                  \
    if (e_ != hipSuccess) return mt::hip_fail(e_, #call);    \
  } while (0)

// after a kernel launch
#define MT_LAUNCH_CHECK(name)                                \
  do {                                                       \
    hipError_t e_ = hipGetLastError();                       \
    if (e_ != hipSuccess) return mt::hip_fail(e_, name);     \
  } while (0)

inline bool same_zyx(const mt_tensor *a, const mt_tensor *b) { return a->x == b->x && a->y == b->y && a->z == b->z; }
inline size_t count(const mt_tensor *t) { return (size_t)t->w * t->z * t->y * t->x; }
inline void note_write(const mt_tensor *t) { if (t && t->p) note_write(t->p, count(t) * sizeof(float)); }
inline bool bad(const mt_tensor *t) { return t == nullptr || (t->p == nullptr && count(t) != 0); }
inline unsigned cdiv(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }
// The matrix-core kernels address an operand through a 32-bit buffer descriptor, with 0x80000000 as "outside".
inline bool fits_buffer(size_t floats) { return floats * 4 < 0x80000000ull; }
inline bool fits_buffer(const mt_tensor *t) { return fits_buffer(count(t)); }

// ---- device side ---------------------------------------------------------------------------
// The reference's scalar functions (cpu/ctensorapplyfunc.h:111-255) with the same float/double
// promotions, so that results differ from the CPU path only by the libm implementation.
__device__ __forceinline__ float f_sigmoid(float v) {
  if (v > 30.f) v = 29.99999f;
  if (v < -30.f) v = -29.99999f;
  return (float)(1.0 / (1.0 + (double)expf(-v)));
}
__device__ __forceinline__ float f_tangence(float v) {
  if (v > 30.f) v = 29.99999f;
  if (v < -30.f) v = -29.99999f;
  return tanhf(v);
}
__device__ __forceinline__ float f_gelu_inner(float v) {
  const float pi = 3.141592654f;
  double dv = v;
  return (float)((double)sqrtf(2.f / pi) * (dv + 0.044715 * dv * dv * dv));
}
__device__ __forceinline__ float f_gelu(float v) {
  float ft = tanhf(f_gelu_inner(v));
  return (float)(0.5 * (double)v * (double)(1.f + ft));
}
__device__ __forceinline__ float f_dgelu(float v) {
  const float pi = 3.141592654f;
  double dv = v;
  float ft = f_gelu_inner(v);
  float fa = (float)((double)sqrtf(2.f / pi) * (1.0 + 3 * 0.044715 * dv * dv));
  float sech = 1.f / coshf(ft);
  return (float)(0.5 * ((double)(1.f + tanhf(ft)) + 0.5 * dv * (double)sech * (double)sech) * (double)fa);
}

__device__ __forceinline__ float apply_func(int func, float v) {
  switch (func) {
    case MT_F_SIGMOID: return f_sigmoid(v);
    case MT_F_RELU: return v > 0.f ? v : 0.f;
    case MT_F_GELU: return f_gelu(v);
    case MT_F_LEAKY_RELU: return v > 0.f ? v : (float)(0.1 * (double)v);
    case MT_F_LINEAR: return v;
    case MT_F_TANGENCE: return f_tangence(v);
    case MT_F_DIFFERENTIAL + MT_F_SIGMOID: { float s = f_sigmoid(v); return (float)((1.0 - (double)s) * (double)s); }
    case MT_F_DIFFERENTIAL + MT_F_RELU: return v >= 0.f ? 1.f : 0.f;
    case MT_F_DIFFERENTIAL + MT_F_GELU: return f_dgelu(v);
    case MT_F_DIFFERENTIAL + MT_F_LEAKY_RELU: return v >= 0.f ? 1.f : 0.1f;
    case MT_F_DIFFERENTIAL + MT_F_LINEAR: return 1.f;
    case MT_F_DIFFERENTIAL + MT_F_TANGENCE: { float t = f_tangence(v); return 1.f - t * t; }
    default: return v;  // MT_F_NONE
  }
}

// Functions cheap enough to live in the epilogue of a matrix-core kernel; after the others the host runs the
// elementwise kernel over the output (same arithmetic, one more pass).
inline bool epilogue_func(int func) { return func == MT_F_NONE || func == MT_F_LINEAR || func == MT_F_RELU || func == MT_F_LEAKY_RELU; }

__device__ __forceinline__ float apply_func_cheap(int func, float v) {  // func satisfies epilogue_func()
  if (func == MT_F_RELU) return v > 0.f ? v : 0.f;
  if (func == MT_F_LEAKY_RELU) return v > 0.f ? v : (float)(0.1 * (double)v);
  return v;
}

// The same for N values at once: one look at the (uniform) function, then straight-line code.
template <int N>
__device__ __forceinline__ void apply_func_cheap_many(int func, float *v) {
  if (func == MT_F_RELU) {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = v[i] > 0.f ? v[i] : 0.f;
  } else if (func == MT_F_LEAKY_RELU) {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = v[i] > 0.f ? v[i] : (float)(0.1 * (double)v[i]);
  }
}

// tanh and sigmoid for the end of a compute-bound kernel (the image layer of a generator applies one of them to 24
// values per thread; with the library routines that was a third of the kernel's vector-ALU time).  Hardware exp and
// reciprocal: absolute error below 3e-7 against the functions above, the same results beyond their clamps.
__device__ __forceinline__ float f_tangence_fast(float v) {
  // (the clamps of the function above change nothing here: beyond +-30 the result is +-1 with or without them --
  // exp overflows to infinity, whose reciprocal is 0, or underflows to 0)
  const float e = __expf(2.f * v);
  return 1.f - 2.f * __frcp_rn(e + 1.f);
}
__device__ __forceinline__ float f_sigmoid_fast(float v) {
  if (v > 30.f) v = 29.99999f;
  if (v < -30.f) v = -29.99999f;
  return __frcp_rn(1.f + __expf(-v));
}

// For kernels that hold few values per thread: the cheap functions stay inline, the transcendental ones are one
// shared out-of-line body (func is uniform, so the branch costs nothing).
__device__ __attribute__((noinline)) inline float apply_func_outlined(int func, float v) { return apply_func(func, v); }
__device__ __forceinline__ float apply_func_epilogue(int func, float v) {
  if (func == MT_F_NONE || func == MT_F_LINEAR) return v;
  if (func == MT_F_RELU) return v > 0.f ? v : 0.f;
  if (func == MT_F_LEAKY_RELU) return v > 0.f ? v : (float)(0.1 * (double)v);
  if (func == MT_F_TANGENCE) return f_tangence_fast(v);
  if (func == MT_F_SIGMOID) return f_sigmoid_fast(v);
  return apply_func_outlined(func, v);
}
// The same for N values at once: one look at the (uniform) function, then straight-line code.
template <int N>
__device__ __forceinline__ void apply_func_epilogue_many(int func, float *v) {
  if (func == MT_F_NONE || func == MT_F_LINEAR) return;
  if (func == MT_F_TANGENCE) {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = f_tangence_fast(v[i]);
  } else if (func == MT_F_SIGMOID) {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = f_sigmoid_fast(v[i]);
  } else if (func == MT_F_RELU) {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = v[i] > 0.f ? v[i] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < N; i++) v[i] = apply_func_epilogue(func, v[i]);
  }
}

inline bool valid_func(int func, bool allow_none) {
  if (func == MT_F_NONE) return allow_none;
  int base = func & ~MT_F_DIFFERENTIAL;
  return func >= 0 && func < 16 && base >= MT_F_SIGMOID && base <= MT_F_TANGENCE;
}

// 64-lane wavefront sum
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

}  // namespace mt
