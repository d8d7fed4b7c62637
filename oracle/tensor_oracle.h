/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the tensor-op hot path.
 *
 * A single-threaded, plain-C restatement of the reference's CPU tensor path
 * (cpu/ctensorconv.h, cpu/ctensormath.h, cpu/ctensorapplyfunc.h, cpu/ctensor.h).
 * Every function keeps the reference's loop nest, accumulation order and
 * float/double promotion so that its fp32 results are bit-equal to the
 * reference headers compiled with `g++ -O2 -ffp-contract=off`.
 *
 * Nothing that ships may link or call this library: it is used by tests/,
 * by the smoke check and by the CPU-baseline leg of the benchmark, always as
 * the checker and never as the product.
 *
 * Tensors are dense [W,Z,Y,X] fp32 arrays with X contiguous; element
 * (w,z,y,x) lives at x + X*(y + Y*(z + Z*w))            (cpu/ctensor.h:259).
 * An operand whose W is smaller than the output's broadcasts by w % W.
 *
 * Return value: 0 on success, or one of the ORACLE_E_* codes where the
 * reference would `throw` a precondition message.
 */
#ifndef TENSOR_ORACLE_H
#define TENSOR_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
  float *p;
  uint32_t w, z, y, x;
} ot_tensor;

/* absolute input coordinates of a pooling maximum (cpu/ctensormath.h:35-39) */
typedef struct {
  uint32_t X, Y;
} ot_spos;

typedef struct {
  ot_spos *p;
  uint32_t w, z, y, x;
} ot_pos_tensor;

enum {
  ORACLE_OK = 0,
  ORACLE_E_NO_KERNELS = 1,     /* kernel_amount == 0                           */
  ORACLE_E_BIAS_COUNT = 2,     /* bias Z != kernel_amount                      */
  ORACLE_E_OUTPUT_SHAPE = 3,   /* output tensor has the wrong Z/Y/X            */
  ORACLE_E_DEPTH = 4,          /* image/delta depth does not match the kernels */
  ORACLE_E_SHAPE = 5           /* generic "sizes do not match" of tensor math  */
};

/* ---- convolutions (cpu/ctensorconv.h) ---------------------------------- */
int oracle_forward_convolution(ot_tensor *out, const ot_tensor *image, const ot_tensor *kernel,
                               int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                               const ot_tensor *bias, int32_t stride_x, int32_t stride_y,
                               int32_t padding_x, int32_t padding_y);
int oracle_backward_convolution(ot_tensor *out_delta, const ot_tensor *delta, const ot_tensor *kernel,
                                int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                const ot_tensor *bias, int32_t stride_x, int32_t stride_y,
                                int32_t padding_x, int32_t padding_y);
int oracle_create_delta_weight_and_bias(ot_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                        uint32_t dkernel_amount, ot_tensor *dbias, const ot_tensor *image,
                                        const ot_tensor *delta, int32_t stride_x, int32_t stride_y,
                                        int32_t padding_x, int32_t padding_y);
int oracle_create_back_delta_weight_and_bias(ot_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                             uint32_t dkernel_amount, ot_tensor *dbias, const ot_tensor *image,
                                             const ot_tensor *delta, int32_t stride_x, int32_t stride_y,
                                             int32_t padding_x, int32_t padding_y);

/* ---- matrix products (cpu/ctensormath.h:531-712, 787-816) -------------- */
int oracle_mul(ot_tensor *out, const ot_tensor *left, const ot_tensor *right);
int oracle_transponse_mul(ot_tensor *out, const ot_tensor *left, const ot_tensor *right);
int oracle_transponse(ot_tensor *out, const ot_tensor *in);

/* ---- elementwise / reductions (cpu/ctensormath.h) ----------------------- */
int oracle_fill(ot_tensor *out, float value);
int oracle_inv(ot_tensor *out, const ot_tensor *in);
int oracle_div(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale);
int oracle_add(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale);
int oracle_sub(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale);
int oracle_add_sum_w(ot_tensor *out, const ot_tensor *left, const ot_tensor *right, float left_scale, float right_scale);
int oracle_add_bias(ot_tensor *working, const ot_tensor *bias);
int oracle_pow2(ot_tensor *out, const ot_tensor *in, float scale);
int oracle_sqrt(ot_tensor *out, const ot_tensor *in, float scale, float add_sqrt_value);
int oracle_summ_xy(ot_tensor *out, const ot_tensor *in);
int oracle_mul_value(ot_tensor *out, const ot_tensor *in, float value);
int oracle_tensor_item_production(ot_tensor *out, const ot_tensor *left, const ot_tensor *right);
int oracle_clip(ot_tensor *t, float min_value, float max_value);
int oracle_signum(ot_tensor *t);
/* present only in the GPU class of the reference (cuda/ctensormath.cu.h:957-979, 1098-1122) */
int oracle_add_value(ot_tensor *out, const ot_tensor *in, float tensor_scale, float value);
int oracle_sub_value(ot_tensor *out, const ot_tensor *in, float tensor_scale, float value);
int oracle_set(ot_tensor *out, const ot_tensor *in, float scale, float add_value);

/* ---- resampling / pooling (cpu/ctensormath.h:868-1055) ------------------ */
int oracle_upsampling(ot_tensor *out, const ot_tensor *in, uint32_t upsampling_x, uint32_t upsampling_y);
int oracle_downsampling(ot_tensor *out, const ot_tensor *in, uint32_t downsampling_x, uint32_t downsampling_y);
int oracle_max_pooling(ot_tensor *out, ot_pos_tensor *pos, const ot_tensor *in, uint32_t pooling_x, uint32_t pooling_y);
int oracle_max_pooling_backward(ot_tensor *out, const ot_pos_tensor *pos, const ot_tensor *in, uint32_t pooling_x,
                                uint32_t pooling_y);

/* ---- optimiser (cpu/ctensormath.h:1119-1165) ---------------------------- */
int oracle_adam(ot_tensor *weight, const ot_tensor *dweight, ot_tensor *m, ot_tensor *v, uint32_t batch_size,
                double speed, double beta1, double beta2, double epsilon, double iteration);

/* ---- VAE coder output (netlayer/cnetlayervaecoderoutput.cu.h:244-287) ----
 * The layer's host loop with the noise given instead of drawn: out = mu + exp(clamp(logvar,-10,10)/2) * epsilon and
 * *kl = -0.5 * sum(1 + logvar - mu^2 - exp(logvar)) / W (clamped logvar).  Pinned by its float64 closed form and by
 * special cases (tests/test_oracle_math.py); the layer itself draws from an unseedable generator. */
int oracle_vae_coder_output(ot_tensor *out, float *kl, const ot_tensor *mu, const ot_tensor *logvar, const ot_tensor *epsilon);

/* ---- functions of the GPU class only (cuda/ctensormath.cu.h:473-598, 3029-3262) -----------------------------------
 * No CPU body exists in the reference: restated from the CUDA kernels.  Concatenation and split are data movement,
 * pinned by numpy's concatenate / slicing; the time step by its float64 closed form.  The three random fills follow
 * the reference's formulas, but the reference draws from cuRAND seeded with rand(), a sequence nobody can reproduce:
 * the generator is specified here (Philox4x32-10, pinned by the published known-answer vectors of Random123) and
 * the fills are checked for their distribution; their parity with the reference's own draws is unpinned by nature. */
int oracle_concatecation_z(ot_tensor *out, const ot_tensor *a, const ot_tensor *b);
int oracle_split_z(ot_tensor *out_a, ot_tensor *out_b, const ot_tensor *in);
int oracle_set_time_step(ot_tensor *out, const ot_tensor *in, const uint32_t *time_step, uint32_t time_step_w);
void oracle_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);
int oracle_create_drop_out_matrix(ot_tensor *out, float drop_out, uint64_t seed);
int oracle_set_normal_noise(ot_tensor *out, uint64_t seed);
int oracle_get_noise_image_and_noise(ot_tensor *noisy, ot_tensor *noise, const ot_tensor *image, const ot_tensor *sqrt_alpha_bar,
                                     const ot_tensor *sqrt_one_minus_alpha_bar, uint64_t seed);

/* ---- activations (cpu/ctensorapplyfunc.h) -------------------------------
 * func ids: 0 sigmoid, 1 ReLU, 2 GeLU, 3 LeakyReLU(0.1), 4 linear, 5 tanh;
 * add 8 for the derivative of the same function. */
enum {
  ORACLE_F_SIGMOID = 0, ORACLE_F_RELU = 1, ORACLE_F_GELU = 2, ORACLE_F_LEAKY_RELU = 3,
  ORACLE_F_LINEAR = 4, ORACLE_F_TANGENCE = 5, ORACLE_F_DIFFERENTIAL = 8
};
float oracle_func_scalar(int func, float v);
int oracle_apply_func(ot_tensor *out, const ot_tensor *in, int func);

#ifdef __cplusplus
}
#endif
#endif
