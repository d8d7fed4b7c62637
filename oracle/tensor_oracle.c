/*
 * TEST INFRASTRUCTURE ONLY -- see tensor_oracle.h.
 *
 * Build: gcc -O2 -ffp-contract=off -std=c99 (no fast-math, no OpenMP): the
 * reference CPU path is single threaded (its only OpenMP pragma sits behind an
 * undefined GOFAST, cpu/ctensormath.h:663) and is built without FMA contraction.
 *
 * Parity pins (tests/test_oracle_*.py):
 *   - every function is bit-compared with the reference headers compiled from
 *     /root/reference (oracle/_ref) on seeded random and edge-case inputs;
 *   - convolutions, products and reductions are also checked against the
 *     reference's own known-answer vectors (cuda/ctensortest.cu.h) and against
 *     float64 closed forms (torch conv2d / conv_transpose2d / autograd, numpy).
 */
#include "tensor_oracle.h"

#include <math.h>
#include <string.h>

#define AT(t, w_, z_, y_, x_) \
  ((t)->p[(size_t)(x_) + (size_t)(t)->x * ((size_t)(y_) + (size_t)(t)->y * ((size_t)(z_) + (size_t)(t)->z * (size_t)(w_)))])

static size_t count(const ot_tensor *t) { return (size_t)t->w * t->z * t->y * t->x; }
static int same_zyx(const ot_tensor *a, const ot_tensor *b) { return a->x == b->x && a->y == b->y && a->z == b->z; }
static uint32_t umin(uint32_t a, uint32_t b) { return a < b ? a : b; }

/* ------------------------------------------------------------------------ */
/* cpu/ctensorconv.h:84-148 -- cross-correlation, bias first, taps ky->kx->c */
int oracle_forward_convolution(ot_tensor *out, const ot_tensor *image, const ot_tensor *kernel,
                               int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                               const ot_tensor *bias, int32_t stride_x, int32_t stride_y,
                               int32_t padding_x, int32_t padding_y) {
  int32_t out_z = (int32_t)kernel_amount;
  if (out_z == 0) return ORACLE_E_NO_KERNELS;
  if ((uint32_t)out_z != bias->z) return ORACLE_E_BIAS_COUNT;
  int32_t in_y = (int32_t)image->y, in_x = (int32_t)image->x, in_z = (int32_t)image->z;
  int32_t out_x = (in_x - kernel_x + 2 * padding_x) / stride_x + 1;
  int32_t out_y = (in_y - kernel_y + 2 * padding_y) / stride_y + 1;
  if (out->x != (uint32_t)out_x || out->y != (uint32_t)out_y || out->z != (uint32_t)out_z) return ORACLE_E_OUTPUT_SHAPE;
  if (in_z != kernel_z) return ORACLE_E_DEPTH;

  int32_t taps = kernel_x * kernel_y;
  for (uint32_t w = 0; w < out->w; w++) {
    uint32_t wi = w % image->w, wk = w % kernel->w, wb = w % bias->w;
    for (int32_t k = 0; k < out_z; k++)
      for (int32_t y = 0; y < out_y; y++)
        for (int32_t x = 0; x < out_x; x++) {
          float acc = AT(bias, wb, k, 0, 0);
          for (int32_t ky = 0; ky < kernel_y; ky++) {
            int32_t sy = stride_y * y + ky - padding_y;
            if (sy < 0 || sy >= in_y) continue;
            for (int32_t kx = 0; kx < kernel_x; kx++) {
              int32_t sx = stride_x * x + kx - padding_x;
              if (sx < 0 || sx >= in_x) continue;
              for (int32_t c = 0; c < in_z; c++) {
                float kv = AT(kernel, wk, 0, k, c * taps + ky * kernel_x + kx);
                float iv = AT(image, wi, c, sy, sx);
                acc += kv * iv;
              }
            }
          }
          AT(out, w, k, y, x) = acc;
        }
  }
  return ORACLE_OK;
}

/* cpu/ctensorconv.h:196-266 -- transposed convolution / input delta.
 * Flipped kernel, padding K-1-p, only taps landing on a stride multiple count.
 * The bias of filter f is added once per contributing (ky,kx,f) tap, before
 * the product (line 255).  Output Y/X come from the output tensor itself. */
int oracle_backward_convolution(ot_tensor *out_delta, const ot_tensor *delta, const ot_tensor *kernel,
                                int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                const ot_tensor *bias, int32_t stride_x, int32_t stride_y,
                                int32_t padding_x, int32_t padding_y) {
  if (kernel_amount == 0) return ORACLE_E_NO_KERNELS;
  if (kernel_amount != bias->z) return ORACLE_E_BIAS_COUNT;
  int32_t in_y = (int32_t)delta->y, in_x = (int32_t)delta->x, in_z = (int32_t)delta->z;
  int32_t pad_x = kernel_x - 1 - padding_x, pad_y = kernel_y - 1 - padding_y;
  int32_t out_x = (int32_t)out_delta->x, out_y = (int32_t)out_delta->y, out_z = kernel_z;
  if (out_delta->z != (uint32_t)out_z) return ORACLE_E_OUTPUT_SHAPE;
  if ((uint32_t)in_z != kernel_amount) return ORACLE_E_DEPTH;

  int32_t taps = kernel_x * kernel_y;
  for (uint32_t w = 0; w < out_delta->w; w++) {
    uint32_t wi = w % delta->w, wk = w % kernel->w, wb = w % bias->w;
    for (int32_t y = 0; y < out_y; y++)
      for (int32_t x = 0; x < out_x; x++)
        for (int32_t z = 0; z < out_z; z++) {
          float acc = 0;
          for (int32_t ky = 0; ky < kernel_y; ky++) {
            int32_t py = y + ky - pad_y;
            if (py % stride_y != 0) continue;
            int32_t dy = py / stride_y;
            if (dy < 0 || dy >= in_y) continue;
            for (int32_t kx = 0; kx < kernel_x; kx++) {
              int32_t px = x + kx - pad_x;
              if (px % stride_x != 0) continue;
              int32_t dx = px / stride_x;
              if (dx < 0 || dx >= in_x) continue;
              int32_t col = z * taps + (kernel_y - 1 - ky) * kernel_x + (kernel_x - 1 - kx);
              for (int32_t f = 0; f < (int32_t)kernel_amount; f++) {
                acc += AT(bias, wb, f, 0, 0);
                float kv = AT(kernel, wk, 0, f, col);
                float dv = AT(delta, wi, f, dy, dx);
                acc += kv * dv;
              }
            }
          }
          AT(out_delta, w, z, y, x) = acc;
        }
  }
  return ORACLE_OK;
}

/* cpu/ctensorconv.h:319-386 -- per-sample weight and bias gradient, ACCUMULATED
 * into dkernel/dbias; W loop runs over dkernel->w; order f -> oy -> ox -> i -> j -> c. */
int oracle_create_delta_weight_and_bias(ot_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                        uint32_t dkernel_amount, ot_tensor *dbias, const ot_tensor *image,
                                        const ot_tensor *delta, int32_t stride_x, int32_t stride_y,
                                        int32_t padding_x, int32_t padding_y) {
  if (dkernel_amount == 0) return ORACLE_E_NO_KERNELS;
  if (dbias->z != dkernel_amount) return ORACLE_E_BIAS_COUNT;
  int32_t img_x = (int32_t)image->x, img_y = (int32_t)image->y, img_z = (int32_t)image->z;
  int32_t d_x = (int32_t)delta->x, d_y = (int32_t)delta->y;
  if (dkernel_z != img_z) return ORACLE_E_SHAPE;
  if (delta->z != dkernel_amount) return ORACLE_E_DEPTH;

  /* the reference walks a zero-dilated delta of size s*(d-1)+1 and skips the holes */
  int32_t dil_x = stride_x * (d_x - 1) + 1, dil_y = stride_y * (d_y - 1) + 1;
  int32_t taps = dkernel_x * dkernel_y;
  for (uint32_t w = 0; w < dkernel->w; w++) {
    uint32_t wi = w % image->w, wd = w % delta->w, wb = w % dbias->w;
    for (int32_t f = 0; f < (int32_t)dkernel_amount; f++)
      for (int32_t y = 0; y < dil_y; y++) {
        if (y % stride_y != 0) continue;
        for (int32_t x = 0; x < dil_x; x++) {
          if (x % stride_x != 0) continue;
          float g = AT(delta, wd, f, y / stride_y, x / stride_x);
          for (int32_t i = 0; i < dkernel_y; i++) {
            int32_t iy = i + y - padding_y;
            if (iy < 0 || iy >= img_y) continue;
            for (int32_t j = 0; j < dkernel_x; j++) {
              int32_t ix = j + x - padding_x;
              if (ix < 0 || ix >= img_x) continue;
              for (int32_t c = 0; c < dkernel_z; c++) {
                float dk = AT(dkernel, w, 0, f, c * taps + i * dkernel_x + j);
                dk += g * AT(image, wi, c, iy, ix);
                AT(dkernel, w, 0, f, c * taps + i * dkernel_x + j) = dk;
              }
            }
          }
          float b = AT(dbias, wb, f, 0, 0);
          b += g;
          AT(dbias, wb, f, 0, 0) = b;
        }
      }
  }
  return ORACLE_OK;
}

/* cpu/ctensorconv.h:393-397 -- gradient of the transposed layer: image and
 * delta trade places, then the bias gradient is cleared. */
int oracle_create_back_delta_weight_and_bias(ot_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                             uint32_t dkernel_amount, ot_tensor *dbias, const ot_tensor *image,
                                             const ot_tensor *delta, int32_t stride_x, int32_t stride_y,
                                             int32_t padding_x, int32_t padding_y) {
  int rc = oracle_create_delta_weight_and_bias(dkernel, dkernel_x, dkernel_y, dkernel_z, dkernel_amount, dbias, delta,
                                               image, stride_x, stride_y, padding_x, padding_y);
  if (rc) return rc;
  return oracle_fill(dbias, 0.0f);
}

/* ------------------------------------------------------------------------ */
/* cpu/ctensormath.h:531-595 -- C = A*B, 32-blocked yy->kk->xx, inner y->k->x */
int oracle_mul(ot_tensor *out, const ot_tensor *left, const ot_tensor *right) {
  if (left->x != right->y || left->z != right->z || out->y != left->y || out->x != right->x || out->z != right->z)
    return ORACLE_E_SHAPE;
  uint32_t M = left->y, K = left->x, N = right->x, Z = left->z;
  memset(out->p, 0, count(out) * sizeof(float));
  const uint32_t BS = 32;
  for (uint32_t w = 0; w < out->w; w++)
    for (uint32_t z = 0; z < Z; z++) {
      const float *a = &AT(left, w % left->w, z, 0, 0);
      const float *b = &AT(right, w % right->w, z, 0, 0);
      float *c = &AT(out, w, z, 0, 0);
      for (uint32_t y0 = 0; y0 < M; y0 += BS)
        for (uint32_t k0 = 0; k0 < K; k0 += BS)
          for (uint32_t x0 = 0; x0 < N; x0 += BS) {
            uint32_t y1 = umin(y0 + BS, M), k1 = umin(k0 + BS, K), x1 = umin(x0 + BS, N);
            for (uint32_t y = y0; y < y1; y++)
              for (uint32_t k = k0; k < k1; k++) {
                float av = a[(size_t)y * K + k];
                for (uint32_t x = x0; x < x1; x++) c[(size_t)y * N + x] += av * b[(size_t)k * N + x];
              }
          }
    }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:643-712 -- C = A^T*B, A stored [K,M]; 32-blocked kk->yy->xx, inner k->y->x */
int oracle_transponse_mul(ot_tensor *out, const ot_tensor *left, const ot_tensor *right) {
  if (left->y != right->y || left->z != right->z || out->y != left->x || out->x != right->x || out->z != right->z)
    return ORACLE_E_SHAPE;
  uint32_t K = left->y, M = left->x, N = right->x, Z = left->z;
  memset(out->p, 0, count(out) * sizeof(float));
  const uint32_t BS = 32;
  for (uint32_t w = 0; w < out->w; w++)
    for (uint32_t z = 0; z < Z; z++) {
      const float *a = &AT(left, w % left->w, z, 0, 0);
      const float *b = &AT(right, w % right->w, z, 0, 0);
      float *c = &AT(out, w, z, 0, 0);
      for (uint32_t k0 = 0; k0 < K; k0 += BS)
        for (uint32_t y0 = 0; y0 < M; y0 += BS)
          for (uint32_t x0 = 0; x0 < N; x0 += BS) {
            uint32_t k1 = umin(k0 + BS, K), y1 = umin(y0 + BS, M), x1 = umin(x0 + BS, N);
            for (uint32_t k = k0; k < k1; k++)
              for (uint32_t y = y0; y < y1; y++) {
                float av = a[(size_t)k * M + y];
                for (uint32_t x = x0; x < x1; x++) c[(size_t)y * N + x] += av * b[(size_t)k * N + x];
              }
          }
    }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:787-816 */
int oracle_transponse(ot_tensor *out, const ot_tensor *in) {
  if (out->y != in->x || out->x != in->y || out->z != in->z || out->w != in->w) return ORACLE_E_SHAPE;
  for (uint32_t w = 0; w < out->w; w++)
    for (uint32_t z = 0; z < in->z; z++)
      for (uint32_t y = 0; y < in->y; y++)
        for (uint32_t x = 0; x < in->x; x++) AT(out, w, z, x, y) = AT(in, w, z, y, x);
  return ORACLE_OK;
}

/* ------------------------------------------------------------------------ */
/* one- and two-operand elementwise loops with the reference's W broadcasting */
#define UNARY_LOOP(EXPR)                                            \
  for (uint32_t w = 0; w < out->w; w++) {                           \
    uint32_t wi = w % in->w;                                        \
    for (uint32_t z = 0; z < out->z; z++)                           \
      for (uint32_t y = 0; y < out->y; y++)                         \
        for (uint32_t x = 0; x < out->x; x++) {                     \
          float i = AT(in, wi, z, y, x);                            \
          AT(out, w, z, y, x) = (EXPR);                             \
        }                                                           \
  }
#define BINARY_LOOP(EXPR)                                           \
  for (uint32_t w = 0; w < out->w; w++) {                           \
    uint32_t wl = w % left->w, wr = w % right->w;                   \
    for (uint32_t z = 0; z < out->z; z++)                           \
      for (uint32_t y = 0; y < out->y; y++)                         \
        for (uint32_t x = 0; x < out->x; x++) {                     \
          float l = AT(left, wl, z, y, x), r = AT(right, wr, z, y, x); \
          AT(out, w, z, y, x) = (EXPR);                             \
        }                                                           \
  }

/* cpu/ctensor.h Fill via cpu/ctensormath.h:154-157 */
int oracle_fill(ot_tensor *out, float value) {
  size_t n = count(out);
  for (size_t i = 0; i < n; i++) out->p[i] = value;
  return ORACLE_OK;
}

/* cpu/ctensormath.h:163-190 -- the division is carried out in double */
int oracle_inv(ot_tensor *out, const ot_tensor *in) {
  if (!same_zyx(in, out)) return ORACLE_E_SHAPE;
  UNARY_LOOP((float)(1.0 / (double)i))
  return ORACLE_OK;
}

/* cpu/ctensormath.h:197-229 */
int oracle_div(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale) {
  if (!same_zyx(left, right) || !same_zyx(out, right)) return ORACLE_E_SHAPE;
  BINARY_LOOP((left_scale * l) / (right_scale * r))
  return ORACLE_OK;
}

/* cpu/ctensormath.h:235-266 */
int oracle_add(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale) {
  if (!same_zyx(left, right) || !same_zyx(out, right)) return ORACLE_E_SHAPE;
  BINARY_LOOP((left_scale * l) + (right_scale * r))
  return ORACLE_OK;
}

/* cpu/ctensormath.h:314-346 */
int oracle_sub(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale) {
  if (!same_zyx(left, right) || !same_zyx(out, right)) return ORACLE_E_SHAPE;
  BINARY_LOOP((left_scale * l) - (right_scale * r))
  return ORACLE_OK;
}

/* cpu/ctensormath.h:273-307 -- sums over W go to layer 0, every other layer of the output is zeroed */
int oracle_add_sum_w(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale) {
  if (!same_zyx(left, right) || !same_zyx(out, right)) return ORACLE_E_SHAPE;
  for (uint32_t z = 0; z < left->z; z++)
    for (uint32_t y = 0; y < left->y; y++)
      for (uint32_t x = 0; x < left->x; x++) {
        float sl = 0, sr = 0;
        for (uint32_t w = 0; w < left->w; w++) sl += AT(left, w, z, y, x);
        sl *= left_scale;
        for (uint32_t w = 0; w < right->w; w++) sr += AT(right, w, z, y, x);
        sr *= right_scale;
        AT(out, 0, z, y, x) = sl + sr;
        for (uint32_t w = 1; w < out->w; w++) AT(out, w, z, y, x) = 0;
      }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:352-381 */
int oracle_add_bias(ot_tensor *working, const ot_tensor *bias) {
  if (working->z != bias->z) return ORACLE_E_SHAPE;
  for (uint32_t w = 0; w < working->w; w++)
    for (uint32_t z = 0; z < working->z; z++) {
      float b = AT(bias, w % bias->w, z, 0, 0);
      for (uint32_t y = 0; y < working->y; y++)
        for (uint32_t x = 0; x < working->x; x++) AT(working, w, z, y, x) += b;
    }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:387-415 */
int oracle_pow2(ot_tensor *out, const ot_tensor *in, float scale) {
  if (!same_zyx(in, out)) return ORACLE_E_SHAPE;
  UNARY_LOOP(i * i * scale)
  return ORACLE_OK;
}

/* cpu/ctensormath.h:421-449 */
int oracle_sqrt(ot_tensor *out, const ot_tensor *in, float scale, float add_sqrt_value) {
  if (!same_zyx(in, out)) return ORACLE_E_SHAPE;
  UNARY_LOOP(sqrtf(i + add_sqrt_value) * scale)
  return ORACLE_OK;
}

/* cpu/ctensormath.h:455-483 */
int oracle_summ_xy(ot_tensor *out, const ot_tensor *in) {
  if (in->z != out->z) return ORACLE_E_SHAPE;
  for (uint32_t w = 0; w < out->w; w++) {
    uint32_t wi = w % in->w;
    for (uint32_t z = 0; z < in->z; z++) {
      float s = 0;
      for (uint32_t y = 0; y < in->y; y++)
        for (uint32_t x = 0; x < in->x; x++) s += AT(in, wi, z, y, x);
      AT(out, w, z, 0, 0) = s;
    }
  }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:721-782 (both scalar overloads compute the same product) */
int oracle_mul_value(ot_tensor *out, const ot_tensor *in, float value) {
  if (!same_zyx(in, out)) return ORACLE_E_SHAPE;
  UNARY_LOOP(i * value)
  return ORACLE_OK;
}

/* cpu/ctensormath.h:822-851 */
int oracle_tensor_item_production(ot_tensor *out, const ot_tensor *left, const ot_tensor *right) {
  if (!same_zyx(left, right) || !same_zyx(out, right)) return ORACLE_E_SHAPE;
  BINARY_LOOP(l * r)
  return ORACLE_OK;
}

/* cpu/ctensormath.h:1061-1084 */
int oracle_clip(ot_tensor *t, float min_value, float max_value) {
  size_t n = count(t);
  for (size_t i = 0; i < n; i++) {
    if (t->p[i] < min_value) t->p[i] = min_value;
    if (t->p[i] > max_value) t->p[i] = max_value;
  }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:1090-1113 */
int oracle_signum(ot_tensor *t) {
  size_t n = count(t);
  for (size_t i = 0; i < n; i++) {
    if (t->p[i] < 0) t->p[i] = -1;
    if (t->p[i] > 0) t->p[i] = 1;
  }
  return ORACLE_OK;
}

/* cuda/ctensormath.cu.h:957-979 (kernel), :985 (host) */
int oracle_add_value(ot_tensor *out, const ot_tensor *in, float tensor_scale, float value) {
  if (!same_zyx(in, out)) return ORACLE_E_SHAPE;
  UNARY_LOOP(i * tensor_scale + value)
  return ORACLE_OK;
}
/* cuda/ctensormath.cu.h:1061 -- AddValue with the value negated */
int oracle_sub_value(ot_tensor *out, const ot_tensor *in, float tensor_scale, float value) {
  return oracle_add_value(out, in, tensor_scale, -value);
}
/* cuda/ctensormath.cu.h:1098-1122 */
int oracle_set(ot_tensor *out, const ot_tensor *in, float scale, float add_value) {
  if (!same_zyx(in, out)) return ORACLE_E_SHAPE;
  UNARY_LOOP(i * scale + add_value)
  return ORACLE_OK;
}

/* ------------------------------------------------------------------------ */
/* cpu/ctensormath.h:868-902 -- nearest neighbour, integer division, 0 outside the input */
int oracle_upsampling(ot_tensor *out, const ot_tensor *in, uint32_t ux, uint32_t uy) {
  if (in->x != out->x / ux || in->y != out->y / uy || in->z != out->z) return ORACLE_E_SHAPE;
  for (uint32_t w = 0; w < out->w; w++) {
    uint32_t wi = w % in->w;
    for (uint32_t z = 0; z < out->z; z++)
      for (uint32_t y = 0; y < out->y; y++) {
        uint32_t iy = y / uy;
        for (uint32_t x = 0; x < out->x; x++) {
          uint32_t ix = x / ux;
          AT(out, w, z, y, x) = (ix >= in->x || iy >= in->y) ? 0.0f : AT(in, wi, z, iy, ix);
        }
      }
  }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:908-949 -- box mean; taps outside are skipped but the divisor stays dx*dy; dx outer, dy inner */
int oracle_downsampling(ot_tensor *out, const ot_tensor *in, uint32_t dsx, uint32_t dsy) {
  if (in->x / dsx != out->x || in->y / dsy != out->y || in->z != out->z || in->w != out->w) return ORACLE_E_SHAPE;
  for (uint32_t w = 0; w < out->w; w++)
    for (uint32_t z = 0; z < out->z; z++)
      for (uint32_t y = 0; y < out->y; y++)
        for (uint32_t x = 0; x < out->x; x++) {
          float s = 0;
          for (uint32_t dx = 0; dx < dsx; dx++) {
            uint32_t xp = x * dsx + dx;
            if (xp >= in->x) continue;
            for (uint32_t dy = 0; dy < dsy; dy++) {
              uint32_t yp = y * dsy + dy;
              if (yp >= in->y) continue;
              s += AT(in, w, z, yp, xp);
            }
          }
          s /= (float)(dsx * dsy);
          AT(out, w, z, y, x) = s;
        }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:955-1013 -- seed is the top-left element, strict '>' scanning py then px */
int oracle_max_pooling(ot_tensor *out, ot_pos_tensor *pos, const ot_tensor *in, uint32_t px_, uint32_t py_) {
  if (in->x / px_ != out->x || in->y / py_ != out->y || in->z != out->z || in->w != out->w) return ORACLE_E_SHAPE;
  for (uint32_t w = 0; w < out->w; w++) {
    uint32_t wp = w % pos->w;
    for (uint32_t z = 0; z < out->z; z++)
      for (uint32_t y = 0; y < out->y; y++)
        for (uint32_t x = 0; x < out->x; x++) {
          uint32_t ix = x * px_, iy = y * py_;
          float best = AT(in, w, z, iy, ix);
          uint32_t bx = ix, by = iy;
          for (uint32_t py = 0; py < py_; py++)
            for (uint32_t px = 0; px < px_; px++) {
              float e = AT(in, w, z, iy + py, ix + px);
              if (e > best) { best = e; bx = ix + px; by = iy + py; }
            }
          AT(out, w, z, y, x) = best;
          ot_spos s; s.X = bx; s.Y = by;
          AT(pos, wp, z, y, x) = s;
        }
  }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:1019-1055 -- zero, then scatter each delta to its stored position */
int oracle_max_pooling_backward(ot_tensor *out, const ot_pos_tensor *pos, const ot_tensor *in, uint32_t px_, uint32_t py_) {
  if (in->x != out->x / px_ || in->y != out->y / py_ || in->z != out->z || in->w != out->w) return ORACLE_E_SHAPE;
  memset(out->p, 0, count(out) * sizeof(float));
  for (uint32_t w = 0; w < out->w; w++) {
    uint32_t wp = w % pos->w;
    for (uint32_t z = 0; z < in->z; z++)
      for (uint32_t y = 0; y < in->y; y++)
        for (uint32_t x = 0; x < in->x; x++) {
          ot_spos s = AT(pos, wp, z, y, x);
          AT(out, w, z, s.Y, s.X) = AT(in, w, z, y, x);
        }
  }
  return ORACLE_OK;
}

/* cpu/ctensormath.h:1119-1165 -- moments are fp32 state, the update arithmetic is double;
 * `iteration` is used as passed (no +1, unlike the GPU kernel of the reference). */
int oracle_adam(ot_tensor *weight, const ot_tensor *dweight, ot_tensor *m, ot_tensor *v, uint32_t batch_size,
                double speed, double beta1, double beta2, double epsilon, double iteration) {
  if (!same_zyx(weight, dweight) || weight->w != dweight->w || !same_zyx(weight, m) || weight->w != m->w ||
      !same_zyx(weight, v) || weight->w != v->w)
    return ORACLE_E_SHAPE;
  size_t n = count(weight);
  for (size_t i = 0; i < n; i++) {
    float dw = dweight->p[i], mi = m->p[i], vi = v->p[i];
    dw /= (float)batch_size;
    mi = (float)(beta1 * mi + (1.0 - beta1) * dw);
    vi = (float)(beta2 * vi + (1.0 - beta2) * dw * dw);
    float mc = (float)(mi / (1.0 - pow(beta1, iteration)));
    float vc = (float)(vi / (1.0 - pow(beta2, iteration)));
    dw = (float)(speed * mc / (sqrtf(vc) + epsilon));
    m->p[i] = mi;
    v->p[i] = vi;
    weight->p[i] = weight->p[i] - dw;
  }
  return ORACLE_OK;
}

/* netlayer/cnetlayervaecoderoutput.cu.h:252-286 with type_t = float: log_var/2.0 is a double division, exp of it a
 * double exp rounded to float; exp(log_var) in the KL term is the float overload; the sum runs in float in
 * w, z, y, x order; "*=-0.5" multiplies in double, "/=BatchSize" divides by the batch size converted to float. */
int oracle_vae_coder_output(ot_tensor *out, float *kl, const ot_tensor *mu, const ot_tensor *logvar, const ot_tensor *epsilon) {
  if (!same_zyx(out, mu) || out->w != mu->w || !same_zyx(out, logvar) || out->w != logvar->w || !same_zyx(out, epsilon) ||
      out->w != epsilon->w)
    return ORACLE_E_SHAPE;
  size_t n = count(out);
  float kl_loss = 0;
  for (size_t i = 0; i < n; i++) {
    float m = mu->p[i], log_var = logvar->p[i];
    if (log_var > 10) log_var = 10;
    if (log_var < -10) log_var = -10;
    float e = (float)exp(log_var / 2.0);
    out->p[i] = m + e * epsilon->p[i];
    kl_loss += 1 + log_var - m * m - expf(log_var);
  }
  kl_loss = (float)(kl_loss * -0.5);
  kl_loss /= (float)out->w;
  if (kl) *kl = kl_loss;
  return ORACLE_OK;
}

/* ------------------------------------------------------------------------ */
/* Functions that exist only in the GPU class of the reference (no CPU body to follow): restated from the CUDA kernels. */

/* cuda/ctensormath.cu.h:473-533: out[w][z] = z < Za ? a[w % Wa][z] : b[w % Wb][z - Za], w over the output's W */
int oracle_concatecation_z(ot_tensor *out, const ot_tensor *a, const ot_tensor *b) {
  if (out->x != a->x || out->x != b->x || out->y != a->y || out->y != b->y || out->z != a->z + b->z) return ORACLE_E_SHAPE;
  size_t yx = (size_t)out->y * out->x;
  for (uint32_t w = 0; w < out->w; w++)
    for (uint32_t z = 0; z < out->z; z++) {
      const float *src = z < a->z ? a->p + ((size_t)(w % a->w) * a->z + z) * yx : b->p + ((size_t)(w % b->w) * b->z + (z - a->z)) * yx;
      memcpy(out->p + ((size_t)w * out->z + z) * yx, src, yx * sizeof(float));
    }
  return ORACLE_OK;
}

/* cuda/ctensormath.cu.h:538-598: the inverse; w runs over the input's W, outputs are indexed by w % their W */
int oracle_split_z(ot_tensor *out_a, ot_tensor *out_b, const ot_tensor *in) {
  if (out_a->x != in->x || out_b->x != in->x || out_a->y != in->y || out_b->y != in->y || out_a->z + out_b->z != in->z) return ORACLE_E_SHAPE;
  size_t yx = (size_t)in->y * in->x;
  for (uint32_t w = 0; w < in->w; w++)
    for (uint32_t z = 0; z < in->z; z++) {
      float *dst = z < out_a->z ? out_a->p + ((size_t)(w % out_a->w) * out_a->z + z) * yx
                                : out_b->p + ((size_t)(w % out_b->w) * out_b->z + (z - out_a->z)) * yx;
      memcpy(dst, in->p + ((size_t)w * in->z + z) * yx, yx * sizeof(float));
    }
  return ORACLE_OK;
}

/* cuda/ctensormath.cu.h:3029-3059, type_t = float: pos = x + X*y + X*Y*z, size = X*Y*Z,
 * angle = t / powf(10000, (float)pos / (float)size); even pos adds sin(angle), odd pos adds cos(angle) */
int oracle_set_time_step(ot_tensor *out, const ot_tensor *in, const uint32_t *time_step, uint32_t time_step_w) {
  if (!same_zyx(in, out) || in->w != out->w || time_step_w != in->w) return ORACLE_E_SHAPE;
  uint32_t size = in->x * in->y * in->z;
  for (uint32_t w = 0; w < in->w; w++) {
    float t = (float)time_step[w];
    for (uint32_t pos = 0; pos < size; pos++) {
      float angle = t / powf(10000.0f, (float)pos / (float)size);
      float v = in->p[(size_t)w * size + pos];
      v += (pos & 1u) == 0 ? sinf(angle) : cosf(angle);
      out->p[(size_t)w * size + pos] = v;
    }
  }
  return ORACLE_OK;
}

/* The reference draws with cuRAND seeded by rand() (cuda/ctensormath.cu.h:3117-3123, 3169-3174, 3218-3225): no
 * sequence to reproduce.  The generator specified here instead is Philox4x32-10 (Salmon et al., SC'11) with
 * key = (seed low, seed high) and counter = (element index low, element index high, 0, 0), one block per element. */
void oracle_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = counter[0], c1 = counter[1], c2 = counter[2], c3 = counter[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; r++) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n1 = (uint32_t)p1, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1, n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
static void element_random(uint64_t seed, uint64_t index, uint32_t r[4]) {
  uint32_t counter[4] = {(uint32_t)index, (uint32_t)(index >> 32), 0u, 0u}, key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  oracle_philox4x32_10(counter, key, r);
}
/* uniform in [0, 1): the top 24 bits of word 0 */
static float element_uniform(const uint32_t r[4]) { return (float)(r[0] >> 8) * (1.0f / 16777216.0f); }
/* standard normal by Box-Muller from words 0 and 1: sqrt(-2 ln u1) cos(2 pi u2), u1 in (0, 1], u2 in [0, 1) */
static float element_normal(const uint32_t r[4]) {
  float u1 = (float)((r[0] >> 8) + 1u) * (1.0f / 16777216.0f), u2 = (float)(r[1] >> 8) * (1.0f / 16777216.0f);
  return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530717958647692f * u2);
}

/* cuda/ctensormath.cu.h:3093-3123: out = uniform >= drop_out ? (float)(1.0 / (1.0 - drop_out)) : 0 */
int oracle_create_drop_out_matrix(ot_tensor *out, float drop_out, uint64_t seed) {
  size_t n = count(out);
  float mult = (float)(1.0 / (1.0 - drop_out));
  for (size_t i = 0; i < n; i++) {
    uint32_t r[4];
    element_random(seed, i, r);
    out->p[i] = element_uniform(r) >= drop_out ? mult : 0.0f;
  }
  return ORACLE_OK;
}

/* cuda/ctensormath.cu.h:3143-3174 */
int oracle_set_normal_noise(ot_tensor *out, uint64_t seed) {
  size_t n = count(out);
  for (size_t i = 0; i < n; i++) {
    uint32_t r[4];
    element_random(seed, i, r);
    out->p[i] = element_normal(r);
  }
  return ORACLE_OK;
}

/* cuda/ctensormath.cu.h:3179-3262: noise as above; noisy = sqrt_alpha_bar[w] * image + sqrt_one_minus_alpha_bar[w] * noise */
int oracle_get_noise_image_and_noise(ot_tensor *noisy, ot_tensor *noise, const ot_tensor *image, const ot_tensor *sqrt_alpha_bar,
                                     const ot_tensor *sqrt_one_minus_alpha_bar, uint64_t seed) {
  if (!same_zyx(noisy, noise) || noisy->w != noise->w || !same_zyx(noisy, image) || noisy->w != image->w) return ORACLE_E_SHAPE;
  if (sqrt_alpha_bar->w != image->w || sqrt_one_minus_alpha_bar->w != image->w) return ORACLE_E_SHAPE;
  size_t per = (size_t)image->z * image->y * image->x;
  size_t sa = (size_t)sqrt_alpha_bar->z * sqrt_alpha_bar->y * sqrt_alpha_bar->x;
  size_t sb = (size_t)sqrt_one_minus_alpha_bar->z * sqrt_one_minus_alpha_bar->y * sqrt_one_minus_alpha_bar->x;
  for (uint32_t w = 0; w < image->w; w++)
    for (size_t i = 0; i < per; i++) {
      uint32_t r[4];
      element_random(seed, (size_t)w * per + i, r);
      float e = element_normal(r);
      noise->p[(size_t)w * per + i] = e;
      noisy->p[(size_t)w * per + i] = sqrt_alpha_bar->p[w * sa] * image->p[(size_t)w * per + i] + sqrt_one_minus_alpha_bar->p[w * sb] * e;
    }
  return ORACLE_OK;
}

/* ------------------------------------------------------------------------ */
/* cpu/ctensorapplyfunc.h:111-255.  The float/double mix follows the C++
 * overload resolution of the reference with type_t=float: math calls on a
 * float argument are the float versions, bare literals such as 1.0, 0.5, 0.1
 * and 0.044715 promote the surrounding product to double. */
static float f_sigmoid(float v) {
  if (v > 30) v = 29.99999f;
  if (v < -30) v = -29.99999f;
  return (float)(1.0 / (1.0 + expf(-v)));
}
static float f_tangence(float v) {
  if (v > 30) v = 29.99999f;
  if (v < -30) v = -29.99999f;
  return tanhf(v);
}
static const float GELU_PI = 3.141592654f;
static float f_gelu_inner(float v) { return (float)(sqrtf(2 / GELU_PI) * (v + 0.044715 * v * v * v)); }
static float f_gelu(float v) {
  float ft = tanhf(f_gelu_inner(v));
  return (float)(0.5 * v * (1 + ft));
}
static float f_sech(float v) { return 1 / coshf(v); }
/* as written in the reference (lines 220-229); it is not the textbook derivative */
static float f_dgelu(float v) {
  float ft = f_gelu_inner(v);
  float fa = (float)(sqrtf(2 / GELU_PI) * (1 + 3 * 0.044715 * v * v));
  return (float)(0.5 * ((1 + tanhf(ft)) + 0.5 * v * f_sech(ft) * f_sech(ft)) * fa);
}

float oracle_func_scalar(int func, float v) {
  switch (func) {
    case ORACLE_F_SIGMOID: return f_sigmoid(v);
    case ORACLE_F_RELU: return v > 0 ? v : 0.0f;
    case ORACLE_F_GELU: return f_gelu(v);
    case ORACLE_F_LEAKY_RELU: return v > 0 ? v : (float)(0.1 * v);
    case ORACLE_F_LINEAR: return v;
    case ORACLE_F_TANGENCE: return f_tangence(v);
    case ORACLE_F_DIFFERENTIAL + ORACLE_F_SIGMOID: { float s = f_sigmoid(v); return (float)((1.0 - s) * s); }
    case ORACLE_F_DIFFERENTIAL + ORACLE_F_RELU: return v >= 0 ? 1.0f : 0.0f;
    case ORACLE_F_DIFFERENTIAL + ORACLE_F_GELU: return f_dgelu(v);
    case ORACLE_F_DIFFERENTIAL + ORACLE_F_LEAKY_RELU: return v >= 0 ? 1.0f : (float)0.1;
    case ORACLE_F_DIFFERENTIAL + ORACLE_F_LINEAR: return 1.0f;
    case ORACLE_F_DIFFERENTIAL + ORACLE_F_TANGENCE: { float t = f_tangence(v); return 1 - t * t; }
  }
  return NAN;
}

/* cpu/ctensorapplyfunc.h:261-629 -- shapes must match in all four sizes */
int oracle_apply_func(ot_tensor *out, const ot_tensor *in, int func) {
  if (!same_zyx(in, out) || in->w != out->w) return ORACLE_E_SHAPE;
  size_t n = count(in);
  for (size_t i = 0; i < n; i++) out->p[i] = oracle_func_scalar(func, in->p[i]);
  return ORACLE_OK;
}
