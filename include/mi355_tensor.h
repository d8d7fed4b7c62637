/*
 * mi355_tensor.h -- C ABI of libmi355tensor.so, the MI355X (gfx950) tensor-op library
 * that backs the reference's CTensor / CTensorMath / CTensorConv / CTensorApplyFunc
 * classes.  Each entry point below replaces one static member function of the
 * reference's GPU classes (file:line given per function, relative to the reference
 * tree) and keeps its argument order, argument meaning and precondition checks.
 *
 * Conventions
 *  - Tensors are dense fp32 [W,Z,Y,X] arrays in DEVICE memory, X contiguous; element
 *    (w,z,y,x) is at x + X*(y + Y*(z + Z*w))  (cuda/ctensor.cu.h:293).  The library
 *    borrows the pointers for the duration of the call and never owns them.
 *  - An operand whose W is smaller than the output's broadcasts by w % W
 *    (cuda/ctensormath.cu.h:141-145).
 *  - Every function returns 0 on success.  MT_E_* (1..5) are the reference's
 *    precondition failures (where the C++ classes `throw` a message); values >= 1000
 *    are 1000 + hipError_t.  mt_last_error() returns a readable message.
 *  - Work is enqueued on one HIP stream (mt_get_stream) and is asynchronous with
 *    respect to the host; mt_copy_d2h and mt_synchronize wait for it.  The reference
 *    blocks after every launch (cudaDeviceSynchronize); callers see the same results
 *    because every host read goes through mt_copy_d2h.
 *  - Not thread safe: one host thread per process, as in the reference.
 */
#ifndef MI355_TENSOR_H
#define MI355_TENSOR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
  float *p;            /* device pointer */
  uint32_t w, z, y, x; /* sizes, [W,Z,Y,X] */
} mt_tensor;

/* CTensorMath<T>::SPos (cuda/ctensormath.cu.h:63-67): absolute input coordinates of a pooling maximum */
typedef struct {
  uint32_t X, Y;
} mt_spos;

typedef struct {
  mt_spos *p; /* device pointer */
  uint32_t w, z, y, x;
} mt_pos_tensor;

/* CTensor<uint32_t> (time steps of the diffusion model, cuda/ctensormath.cu.h:3064) */
typedef struct {
  uint32_t *p; /* device pointer */
  uint32_t w, z, y, x;
} mt_u32_tensor;

enum {
  MT_OK = 0,
  MT_E_NO_KERNELS = 1,   /* kernel_amount == 0                                  (cpu/ctensorconv.h:88,199,321)  */
  MT_E_BIAS_COUNT = 2,   /* bias Z != kernel_amount                             (cpu/ctensorconv.h:89,200,322)  */
  MT_E_OUTPUT_SHAPE = 3, /* output tensor has the wrong Z/Y/X                   (cpu/ctensorconv.h:103,220)     */
  MT_E_DEPTH = 4,        /* image/delta depth does not match the kernels        (cpu/ctensorconv.h:105,221,335) */
  MT_E_SHAPE = 5,        /* "sizes do not match" of the tensor-math functions   (cpu/ctensormath.h, every head) */
  MT_E_ARGUMENT = 6,     /* null pointer, zero stride, unknown function id ...  (no counterpart: the C++ API cannot express these) */
  MT_E_UNAVAILABLE = 7,  /* no usable gfx950 device; a single matrix of 2 GiB+   */
  MT_E_HIP = 1000        /* + hipError_t                                         (cuda/handle_error.cu.h:7-19)  */
};

/* activation ids (cuda/ctensorapplyfunc.cu.h:60-...): add MT_F_DIFFERENTIAL for the derivative */
enum {
  MT_F_SIGMOID = 0, MT_F_RELU = 1, MT_F_GELU = 2, MT_F_LEAKY_RELU = 3, MT_F_LINEAR = 4, MT_F_TANGENCE = 5,
  MT_F_DIFFERENTIAL = 8,
  MT_F_NONE = -1 /* fused entry points only: no activation */
};

/* ---- runtime: replaces CCUDADeviceVector (cuda/ccudadevicevector.cu.h:41-72) and HANDLE_ERROR ---- */
int mt_init(int device);                 /* cuda/cuda.cu:81 (cudaSetDevice); checks the device is gfx950 */
const char *mt_last_error(void);
int mt_malloc(void **ptr, size_t bytes); /* ccudadevicevector.cu.h resize   */
int mt_free(void *ptr);                  /* ccudadevicevector.cu.h clear    */
int mt_copy_h2d(void *dst, const void *src, size_t bytes); /* copy_host_to_device; src may be reused on return; the copy is in
                                                             stream order (at most 64 KiB: queued, not waited for) */
int mt_copy_d2h(void *dst, const void *src, size_t bytes); /* copy_device_to_host; waits for queued work */
int mt_copy_d2d(void *dst, const void *src, size_t bytes); /* operator= (device copy, :159-170) */
/* Tells the library that someone else (another library's kernel, a hipMemcpy of the caller's) wrote [ptr, ptr+bytes).
 * The library keeps re-ordered copies of convolution weights between calls (the layers pass the same kernel tensor on
 * every forward call, netlayer/cnetlayerbackconvolution.cu.h:303-315) and makes them again after any write to the
 * weights that goes through this ABI -- mt_copy_h2d, mt_copy_d2d, mt_free, every function with an output tensor --
 * or is announced here.  No counterpart in the reference: its CTensor writes device memory through its own calls only. */
int mt_invalidate(const void *ptr, size_t bytes);
int mt_synchronize(void);
void *mt_get_stream(void);               /* the hipStream_t all work is queued on */
int mt_set_stream(void *hip_stream);     /* queue on a caller-owned stream (NULL: back to the library's own) */
/* CCUDATimeSpent (cuda/ccudatimespent.cu:9-52): two events on the work stream; stop waits for the second one and
 * returns the milliseconds between them.  The timer must have been started before it is stopped. */
int mt_timer_create(void **timer);
int mt_timer_start(void *timer);
int mt_timer_stop(void *timer, float *milliseconds);
int mt_timer_destroy(void *timer);
/* Options, for tests and measurements (results agree within fp32 rounding whatever is chosen).  No counterpart in the
 * reference.  One line per option: name, values, meaning.
 *   "conv_path"      0 (default) choose per shape / 1 one-thread-per-output kernels in the CPU path's summation order /
 *                    2 matrix-core kernels wherever they apply
 *   "igemm_tile"     -1 (default) choose per shape / 0..4 force the block tile 128x128, 64x128, 32x128, 64x64, 16x256 of the
 *                    matrix-core kernels (a forced tile also switches off the kernels chosen by shape beside them)
 *   "igemm_fair"     -1 (default) falling wavefront priorities where the chip holds the whole grid at once / 0 never /
 *                    three hexadecimal digits: sixteenths of a block's k steps left at which the priority drops to 2, 1, 0
 *   "patch_blocks"   persistent blocks of the input-patch transposed convolution (default 512, two per compute unit)
 *   "wgrad_groups"   0 (default) choose per shape / n split the batch of mt_convolution_backward_weights_sum into n groups
 *                    (when n divides the batch)
 *   "wgrad_parts"    1 (default) the general kernel of mt_convolution_backward_weights_sum cuts every sample into equal bands of
 *                    output rows (one partial sum per band) when samples x tiles are fewer blocks than the chip needs: layers
 *                    with few filters on large images / 0 never / n bands per sample (2..256, where the rows divide)
 *   "wgrad_pad"      1 (default) mt_convolution_backward_weights_sum appends rows of zeros to delta's images when their pixels
 *                    are not a multiple of 16 (3 x 4 at the end of a discriminator), so that the sum over the batch stays
 *                    one product / 0 per-sample gradients and their sum then
 *   "conv_patch"     1 (default) mt_forward_convolution 3x3, stride 1, padding 1 from at most 32 channels to 5..64 filters on large
 *                    images (rows a multiple of 64 pixels, an even number of rows, at least 1024 tiles of 2 x 64 pixels in the
 *                    batch) multiplies image patches held in LDS, nine taps per patch / 0 never / n (2..64) from n filters on
 *   "tconv_as_conv"  1 (default) mt_backward_convolution with stride 1 and a kernel whose taps do not tile a k step of 16 (3x3, 5x5),
 *                    a multiple of 16 filters and at least 16 channels runs as the forward convolution with flipped, transposed
 *                    kernels (k ordered tap-major) / 0 as a transposed convolution
 *   "tconv_merge"    1 (default) mt_backward_convolution 5x5 stride 2 padding 2 to 5..16 channels at twice the input size runs its
 *                    four stride phases as one 3x3 convolution to (channel, phase) rows and spreads them over the output / 0 never
 *   "tconv_patch"    1 (default) mt_backward_convolution of a 3x3 layer with stride 1, padding 1, at most 32 filters and at most 64
 *                    channels on large images (rows a multiple of 64 pixels, an even number of rows, at least 1024 tiles of
 *                    2 x 64 pixels in the batch) multiplies patches of delta held in LDS, nine taps per patch / 0 never
 *   "wgrad_patch"    1 (default) mt_convolution_backward_weights_sum of a 3x3 layer with stride 1, padding 1 and at most 32
 *                    filters on large images (rows a multiple of 64 pixels, an even number of rows, at least 1024 tiles of
 *                    2 x 64 pixels in the batch) multiplies image patches held in LDS, nine taps per patch / 0 never
 *   "pack_cache"     1 (default) keep re-ordered weights between calls / 0 re-order on every call
 *   "tconv_walk"     1 (default) plain transposed convolutions use the kernel whose blocks walk over the batch wherever
 *                    the shape allows / 0 never
 *   "conv_walk"      1 (default) forward convolutions whose taps tile the k step (4x4, 2x2, 1x1) use the same walking kernel
 *                    wherever the shape allows and gives at least 512 blocks / 2 wherever the shape allows / 0 never
 *   "wgrad_walk"     1 (default) mt_convolution_backward_weights_sum runs each group of samples as one k loop per block, with
 *                    fixed gather offsets, where the shape allows (output rows of 4, 8 or 16 pixels, filters a multiple of 64) /
 *                    0 never
 *   "upconv_walk"    512 (default) mt_upsampling_convolution_func (x2, 3x3) uses the walking kernel when that gives at least this
 *                    many blocks / 1 wherever the shape allows / 0 never
 *   "upconv_split"   1 (default) where that kernel would get fewer than 512 blocks (small images, many channels), two or four
 *                    blocks share a tile's sum over (channel, tap) and a second kernel adds their parts, the bias and the function /
 *                    0 never
 *   "walk_wide"      1 (default) transposed and up-sampling convolutions whose output channels are a multiple of 32 but not of 64
 *                    walk in blocks of 32 rows x 128 columns / 0 they run on the one-tile kernels
 *   "pack_refresh"   1 (default) mt_adam_many writes each new weight also into the kept re-ordered copy that the 4x4 stride-2
 *                    transposed convolution (the input gradient of a 4x4 stride-2 convolution layer) made of those weights, so a
 *                    training loop re-orders nothing per step; not while a graph is recorded / 0 the step only reports its write
 *   "adam_vec"       1 (default) mt_adam_many updates four elements per thread in the tiles that also write a re-ordered copy /
 *                    2 wherever the tensors allow / 0 never (measurements only; the results are the same bit for bit)
 *   "first_layer"    1 (default) forward convolutions of 3-channel images (3x3, 4x4, 5x5 kernels to 32 or 64 filters) keep the
 *                    input patch in LDS and the weights in registers wherever the shape allows / 0 never
 *   "walk_blocks"    blocks wanted per launch of the walking kernel (default 1024)
 *   "walk_waves"     4 (default) or 5 wavefronts per SIMD for its plain variant
 *   "walk_tm"        1 (default) or 2 accumulators per wavefront
 *   "walk_order"     -1 (default) per layer / 0 batch groups first / 1 row tiles first
 *   "walk_fair"      0x842 (default): a wavefront's priority drops at 8/16, 4/16 and 2/16 of its steps left / 0 none
 *   "image_mfma"     kernel of a generator's image layer (transposed convolution 4x4, stride 2, to at most 4 channels):
 *                    2 (default) products per input pixel on the 16x16x4 matrix instruction where the shape allows /
 *                    1 the 4x4x1 matrix instruction where the shape allows / 0 the vector ALUs
 *   "image_strip"    rows per strip of the image layer's product kernel on images of 64 columns (0, default: 8 or 4)
 *   "nontemporal"    2 (default) the re-sampling, pooling and large-batch batch-norm kernels read and write tensors of 128 MiB
 *                    and more past the caches (each element is touched once) / 1 always / 0 never
 *   "staged_uploads" 1 (default) mt_copy_h2d of at most 64 KiB copies the caller's buffer into a pinned slot at once and queues
 *                    the copy to the device behind the work already queued, without waiting for it / 0 every upload waits
 *   "pool"           1 (default) mt_free keeps blocks for the next mt_malloc of the same size (stream-ordered reuse, no
 *                    wait) / 0 every mt_free waits for the stream and returns the block to the driver
 *   "pool_limit_mib" MiB the pool may hold in free blocks (default 4096) */
int mt_set_option(const char *name, int value);
/* Counters of the runtime, for tests and measurements (no counterpart in the reference):
 *   "pool_bytes", "pool_reused", "driver_allocations"      the memory pool behind mt_malloc / mt_free
 *   "retired_blocks", "retired_bytes"                      blocks freed (or handed out) while the stream was being captured:
 *                                                          a recorded graph names them, so they are never handed out again
 *   "staged_uploads"                                       uploads that went through a pinned slot (option "staged_uploads")
 *   "retired_workspaces"                                   outgrown workspaces that a recorded graph may still use
 *   "convolution_workspace_bytes"                          size of the convolutions' workspace (it only grows)
 *   "pack_cache_entries", "pack_cache_valid", "pack_cache_hits", "pack_cache_made", "pack_cache_bytes"
 *                                                          the re-ordered weights kept between calls
 *   "pack_cache_refreshed"                                 copies that an mt_adam_many call wrote itself (option "pack_refresh")
 *   "pack_cache_spare_bytes"                               buffers of evicted entries that a recorded graph still names
 *   "graph_written_ranges", "graph_writes_anything"        memory written by recorded calls: weights inside such a range
 *                                                          are re-ordered on every use, until the block that holds the
 *                                                          range is freed; after 4096 ranges everything is
 *                                                          (graph_writes_anything = 1, for the rest of the process)
 *   "wgrad_walk_launches"                                  calls of mt_convolution_backward_weights_sum that ran as one k loop
 *                                                          per block (option "wgrad_walk")
 *   "wgrad_patch_launches"                                 calls of it that multiplied patches held in LDS (option "wgrad_patch")
 *   "conv_patch_launches"                                  calls of mt_forward_convolution that multiplied patches held in LDS (option "conv_patch")
 *   "tconv_as_conv_launches"                               calls of mt_backward_convolution that ran as a forward convolution (option "tconv_as_conv")
 *   "tconv_merge_launches"                                 calls of mt_backward_convolution that ran as one merged convolution (option "tconv_merge")
 *   "tconv_patch_launches"                                 calls of mt_backward_convolution that did (option "tconv_patch") */
int mt_get_info(const char *name, int64_t *value);

/* ---- convolutions: CTensorConv<T> (cuda/ctensorconv.cu.h:63-66) ---- */
/* ForwardConvolution, cuda/ctensorconv.cu.h:276-315 (+ the AddBias launch it ends with); CPU: cpu/ctensorconv.h:84-148 */
int mt_forward_convolution(const mt_tensor *output, const mt_tensor *image, const mt_tensor *kernel,
                           int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                           const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y);
/* BackwardConvolution, cuda/ctensorconv.cu.h:683-725; CPU: cpu/ctensorconv.h:196-266 (the per-tap bias of the CPU path is kept) */
int mt_backward_convolution(const mt_tensor *output_delta, const mt_tensor *delta, const mt_tensor *kernel,
                            int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                            const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y);
/* CreateDeltaWeightAndBias, cuda/ctensorconv.cu.h:1168-1211; CPU: cpu/ctensorconv.h:319-386. Accumulates into dkernel and dbias. */
int mt_create_delta_weight_and_bias(const mt_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                    uint32_t dkernel_amount, const mt_tensor *dbias, const mt_tensor *image,
                                    const mt_tensor *delta, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y);
/* CreateBackDeltaWeightAndBias, cuda/ctensorconv.cu.h:1218-1222; CPU: cpu/ctensorconv.h:393-397 */
int mt_create_back_delta_weight_and_bias(const mt_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                         uint32_t dkernel_amount, const mt_tensor *dbias, const mt_tensor *image,
                                         const mt_tensor *delta, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y);

/* ---- matrix products: CTensorMath<T> ---- */
int mt_mul(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right);            /* Mul, cuda/ctensormath.cu.h:2237-2243 (MulAbstract :1949-2067); CPU :531-595 */
int mt_transponse_mul(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right); /* TransponseMul, cuda :2249-2255; CPU :643-712 */
int mt_transponse(const mt_tensor *output, const mt_tensor *input);                            /* Transponse, cuda :2362 (a host loop there); CPU :787-816 */

/* ---- elementwise and reductions: CTensorMath<T> (line numbers: cuda/ctensormath.cu.h host entry; CPU twin in cpu/ctensormath.h) ---- */
int mt_fill(const mt_tensor *output, float value);                                                                               /* Fill :637; CPU :154-157 */
int mt_inv(const mt_tensor *output, const mt_tensor *input);                                                                     /* Inv :702; CPU :163-190 */
int mt_div(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right, float left_scale, float right_scale);         /* Div :768; CPU :197-229 */
int mt_add(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right, float left_scale, float right_scale);         /* Add :837; CPU :235-266 */
int mt_sub(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right, float left_scale, float right_scale);         /* Sub :1021; CPU :314-346 */
int mt_add_sum_w(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right, float left_scale, float right_scale);   /* AddSumW :914; CPU :273-307 */
int mt_add_bias(const mt_tensor *working, const mt_tensor *bias);                                                                /* AddBias :1328; CPU :352-381 */
int mt_pow2(const mt_tensor *output, const mt_tensor *input, float scale);                                                       /* Pow2 :1196; CPU :387-415 */
int mt_sqrt(const mt_tensor *output, const mt_tensor *input, float scale, float add_sqrt_value);                                 /* SQRT :1262; CPU :421-449 */
int mt_summ_xy(const mt_tensor *output, const mt_tensor *input);                                                                 /* SummXY :1396; CPU :455-483 */
int mt_mul_value(const mt_tensor *output, const mt_tensor *input, float value);                                                  /* Mul(T,scalar) x2 :2291,:2326; CPU :721-782 */
int mt_tensor_item_production(const mt_tensor *output, const mt_tensor *left, const mt_tensor *right);                           /* TensorItemProduction :2425; CPU :822-851 */
int mt_clip(const mt_tensor *tensor, float min_value, float max_value);                                                          /* Clip :2834; CPU :1061-1084 */
int mt_signum(const mt_tensor *tensor);                                                                                          /* Signum :2892; CPU :1090-1113 */
int mt_add_value(const mt_tensor *output, const mt_tensor *input, float tensor_scale, float value);                              /* AddValue :985 (GPU class only) */
int mt_sub_value(const mt_tensor *output, const mt_tensor *input, float tensor_scale, float value);                              /* SubValue :1061 (GPU class only) */
int mt_set(const mt_tensor *output, const mt_tensor *input, float scale, float add_value);                                       /* Set :1128 (GPU class only) */

/* ---- resampling and pooling: CTensorMath<T> ---- */
int mt_upsampling(const mt_tensor *output, const mt_tensor *input, uint32_t upsampling_x, uint32_t upsampling_y);       /* UpSampling :2518; CPU :868-902 */
int mt_downsampling(const mt_tensor *output, const mt_tensor *input, uint32_t downsampling_x, uint32_t downsampling_y); /* DownSampling :2600; CPU :908-949 (CPU edge rule kept) */
int mt_max_pooling(const mt_tensor *output, const mt_pos_tensor *position, const mt_tensor *input, uint32_t pooling_x, uint32_t pooling_y);          /* MaxPooling :2693; CPU :955-1013 */
int mt_max_pooling_backward(const mt_tensor *output, const mt_pos_tensor *position, const mt_tensor *input, uint32_t pooling_x, uint32_t pooling_y); /* MaxPoolingBackward :2767; CPU :1019-1055 */

/* ---- optimiser: Adam, cuda/ctensormath.cu.h:2978-3022; CPU :1119-1165 (`iteration` used as passed, as on the CPU path) ---- */
int mt_adam(const mt_tensor *weight, const mt_tensor *dweight, const mt_tensor *m, const mt_tensor *v, uint32_t batch_size,
            double speed, double beta1, double beta2, double epsilon, double iteration);

/* ---- activations: CTensorApplyFunc<T>::Apply* / ApplyDifferential* (cuda/ctensorapplyfunc.cu.h:297-866; CPU :261-629) ---- */
int mt_apply_func(const mt_tensor *output, const mt_tensor *input, int func);

/* ---- fused entry points -----------------------------------------------------------------------
 * Each one is the exact op sequence of one reference layer's Forward(), lowered to fewer launches.
 * They have no single counterpart function in the reference; the sequence each replaces is cited.
 * Numerics of `func`: ReLU, leaky ReLU, linear and GeLU are the arithmetic of mt_apply_func.  Sigmoid and tangence,
 * where they run at the end of a convolution or transposed-convolution kernel (the image layer of a generator and the
 * small-channel-count kernels), use the hardware's exponential and reciprocal (v_exp_f32, v_rcp_f32) with the same
 * clamp at +-30 instead of the library exp and the division of mt_apply_func, and differ from mt_apply_func on the
 * same input by at most 3e-7 absolute (outputs lie in [-1, 1]). */

/* CNetLayerConvolution::Forward + CNetLayerFunction::Forward (netlayer/cnetlayerconvolution.cu.h:310-322,
 * netlayer/cnetlayerfunction.cu.h:203-213): convolution, bias and activation `func` in one kernel. */
int mt_forward_convolution_func(const mt_tensor *output, const mt_tensor *image, const mt_tensor *kernel,
                                int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y, int func);
/* CNetLayerBackConvolution::Forward + CNetLayerFunction::Forward (netlayer/cnetlayerbackconvolution.cu.h:303-315) */
int mt_backward_convolution_func(const mt_tensor *output, const mt_tensor *delta, const mt_tensor *kernel,
                                 int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                 const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y, int func);
/* CNetLayerUpSampling::Forward (netlayer/cnetlayerupsampling.cu.h:233-252) + CNetLayerConvolution::Forward
 * (netlayer/cnetlayerconvolution.cu.h:310-322) + CNetLayerFunction::Forward: output = func(conv(UpSampling(image))).
 * `image` is the input of the up-sampling layer, [W,kernel_z,H,Wd]; output must be the convolution's output for the
 * up-sampled image [W,kernel_z,H*upsampling_y,Wd*upsampling_x].  For x2 up-sampling and a 3x3 kernel with stride 1 and
 * padding 1 (the reference's GAN generator) the up-sampled image is never formed: each output parity is a 2x2
 * convolution of the input with sums of the 3x3 coefficients. */
int mt_upsampling_convolution_func(const mt_tensor *output, const mt_tensor *image, uint32_t upsampling_x, uint32_t upsampling_y,
                                   const mt_tensor *kernel, int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                   const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y, int func);
/* A transposed-convolution layer between two batch-norm layers, with the batch normalisations folded into it
 * (CNetLayerBatchNormalization::Forward in training mode + CNetLayerFunction::Forward,
 * netlayer/cnetlayerbatchnormalization.cu.h:301-371, around CNetLayerBackConvolution::Forward,
 * netlayer/cnetlayerbackconvolution.cu.h:303-315).  A batch normalisation is split at its statistics: the layer in
 * front of it produces, beside its raw output x, the pair (scale, shift) = (gamma*ivar, beta - mean*gamma*ivar) per
 * element, and the layer behind it applies func(scale*x + shift) as it loads x.  The normalised tensor is never
 * written or read.  A tensor of pairs is [1,Z,Y,2*X]: element (z,y,x) holds its scale at 2*x and its shift at 2*x+1.
 *
 * mt_backward_convolution_norm_func:  output = func(BackwardConvolution(delta_func(scale*delta + shift), kernel, bias)).
 *   delta_scale_shift [1,kernel_amount,H,2*W] may be NULL (delta is used as it is); delta_func is none, linear, ReLU or
 *   leaky ReLU.
 * mt_backward_convolution_norm_stats: the same with func none, plus the statistics of `output` over the batch for the batch
 *   normalisation (gamma, beta [1,Z,Y,X] of the output) that follows: scale_shift [1,Z,Y,2*X] of the output, and
 *   optionally ivar, batch mean, batch variance and the blended running statistics exactly as
 *   mt_batchnorm_forward_train_func gives them.  xhat of that layer is (output - batch_mean) * ivar.
 * Where the shape allows (one kernel set and one bias set for the batch, equal batch sizes, output channels a
 * multiple of 64, phase images of a multiple of 16 pixels, batch a multiple of 4) this is one matrix-core kernel whose
 * blocks walk over the batch and a small kernel that combines per-block statistics in a fixed order; otherwise the
 * same results come from separate passes.  Results equal the layer-by-layer path within fp32 rounding
 * (scale*x + shift against gamma*((x - mean)*ivar) + beta: a few units in the last place of |mean*scale| + |x*scale|). */
int mt_backward_convolution_norm_func(const mt_tensor *output, const mt_tensor *delta, const mt_tensor *delta_scale_shift, int delta_func,
                                      const mt_tensor *kernel, int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                      const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y, int func);
int mt_backward_convolution_norm_stats(const mt_tensor *output, const mt_tensor *delta, const mt_tensor *delta_scale_shift, int delta_func,
                                       const mt_tensor *kernel, int32_t kernel_x, int32_t kernel_y, int32_t kernel_z, uint32_t kernel_amount,
                                       const mt_tensor *bias, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y,
                                       const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *scale_shift, const mt_tensor *ivar,
                                       const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean, const mt_tensor *new_variable,
                                       float momentum, float epsilon);
/* CNetLayerLinear::Forward + CNetLayerFunction::Forward (netlayer/cnetlayerlinear.cu.h:262-282): output[B,1,Out,1] =
 * func(weight[1,1,Out,In] * input[B,1,In,1] + bias[1,1,Out,1]); `input` may have any [B,Z,Y,X] with Z*Y*X == In. */
int mt_linear_forward_func(const mt_tensor *output, const mt_tensor *weight, const mt_tensor *input, const mt_tensor *bias, int func);
/* CNetLayerLinear::Forward (netlayer/cnetlayerlinear.cu.h:262-282), CNetLayerBatchNormalization::Forward in training mode
 * (netlayer/cnetlayerbatchnormalization.cu.h:301-371) and CNetLayerFunction::Forward as one launch for batches of at most
 * 256: output [B,...] = func(gamma * xhat + beta) with xhat = (weight * input + bias - mean) * ivar, mean and variance per
 * output feature over the batch, computed on the product's accumulators (a block holds the whole batch of its 16
 * features).  weight, input, bias as for mt_linear_forward_func; gamma, beta and the optional statistics hold Out values
 * ([1,Z,Y,X] with Z*Y*X == Out, like the output's sample); optional linear_output (the Linear layer's own output) and
 * xhat hold [B,Out] values; NULL skips an optional tensor.  Larger batches run as the two calls. */
int mt_linear_batchnorm_forward_func(const mt_tensor *output, const mt_tensor *weight, const mt_tensor *input, const mt_tensor *bias,
                                     const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *linear_output, const mt_tensor *xhat,
                                     const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean,
                                     const mt_tensor *new_variable, float momentum, float epsilon, int func);
/* CNetLayerBatchNormalization::Forward in training mode followed by CNetLayerFunction::Forward
 * (netlayer/cnetlayerbatchnormalization.cu.h:301-371): statistics per element (z,y,x) over the batch axis W.
 * Writes output = func(gamma*xhat+beta); optionally xhat [B,Z,Y,X], ivar / batch mean / batch variance [1,Z,Y,X]
 * (NULL to skip), and blends new_mean / new_variable with `momentum` as lines 311 and 324 do (NULL to skip). */
int mt_batchnorm_forward_train_func(const mt_tensor *output, const mt_tensor *input, const mt_tensor *gamma, const mt_tensor *beta,
                                    const mt_tensor *xhat, const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var,
                                    const mt_tensor *new_mean, const mt_tensor *new_variable, float momentum, float epsilon, int func);
/* The same call with the running statistics blended FROM other tensors: new_mean = momentum * old_mean + (1 - momentum) * batch
 * mean, likewise the variance (lines 311 and 324 with cTensor_NewMean sharing its memory with cTensor_Mean, as it does after
 * TrainingResetDeltaWeight, netlayer/cnetlayerbatchnormalization.cu.h:617-618, in a container whose copies share storage);
 * old_mean / old_variable NULL: blended in place.  pre_function [B,Z,Y,X] (NULL to skip): gamma*xhat+beta, the batch-norm
 * layer's own output tensor when `output` is the function layer's (netlayer/cnetlayerfunction.cu.h:202-212); a tensor of
 * its own. */
int mt_batchnorm_forward_train_from(const mt_tensor *output, const mt_tensor *input, const mt_tensor *gamma, const mt_tensor *beta,
                                    const mt_tensor *xhat, const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var,
                                    const mt_tensor *new_mean, const mt_tensor *new_variable, const mt_tensor *old_mean,
                                    const mt_tensor *old_variable, float momentum, float epsilon, int func, const mt_tensor *pre_function);
/* The same call for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Statistics the caller does not ask for go to a
 * fixed array inside the library's code object (3 MiB per GPU, held until the process ends) instead of a workspace
 * that grows: Z*Y*X of the input must not exceed 262144 (MT_E_ARGUMENT otherwise); nothing is allocated or freed, no
 * profiling event is created.  Same kernels and results as mt_batchnorm_forward_train_func.  All calls on one GPU
 * share the array: calls that overlap in time on one GPU (two streams, two threads) race. */
int mt_batchnorm_forward_train_func_noalloc(const mt_tensor *output, const mt_tensor *input, const mt_tensor *gamma, const mt_tensor *beta,
                                            const mt_tensor *xhat, const mt_tensor *ivar, const mt_tensor *batch_mean, const mt_tensor *batch_var,
                                            const mt_tensor *new_mean, const mt_tensor *new_variable, float momentum, float epsilon, int func);
/* The same layer in inference mode (netlayer/cnetlayerbatchnormalization.cu.h:326-371): stored mean / variable instead of
 * batch statistics. */
int mt_batchnorm_forward_infer_func(const mt_tensor *output, const mt_tensor *input, const mt_tensor *gamma, const mt_tensor *beta,
                                    const mt_tensor *mean, const mt_tensor *variable, float epsilon, int func);

/* CNetLayerVAECoderOutput::Forward, netlayer/cnetlayervaecoderoutput.cu.h:244-287 (a host loop over GetElement there),
 * with the noise supplied by the caller instead of drawn from an unseedable generator:
 * output = mu + exp(clamp(logvar, -10, 10) / 2) * epsilon;  kl_loss[0] = -0.5 * sum(1 + logvar - mu^2 - exp(logvar)) / W
 * (kl_loss: device tensor of at least one value, NULL to skip). */
int mt_vae_coder_output(const mt_tensor *output, const mt_tensor *kl_loss, const mt_tensor *mu, const mt_tensor *logvar, const mt_tensor *epsilon);

/* ---- fused backward sequences ---- */
/* CNetLayerBatchNormalization::TrainingBackward, netlayer/cnetlayerbatchnormalization.cu.h:578-604, as one kernel:
 * error [B,Z,Y,X] = ((N*dxhat - xhat*sum_w(dxhat*xhat)) - sum_w(dxhat)) * ivar * (1/N) with dxhat = delta*gamma;
 * dgamma [1,Z,Y,X] += sum_w(delta*xhat), dbeta += sum_w(delta) (NULL to skip, as create_delta_weight == false does).
 * `error` may be the same tensor as `delta`. */
int mt_batchnorm_backward(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta,
                          const mt_tensor *gamma, const mt_tensor *xhat, const mt_tensor *ivar);
/* The same behind a function layer (CNetLayerFunction::SetOutputError, netlayer/cnetlayerfunction.cu.h:347-358, then the
 * sequence above): `delta` is the gradient of func(gamma*xhat+beta) as the forward pass wrote it with that `func`; it is
 * multiplied by f'(gamma*xhat+beta) on the way in.  `beta` [1,Z,Y,X] is needed unless func is MT_F_NONE / MT_F_LINEAR. */
int mt_batchnorm_backward_func(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta,
                               const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *xhat, const mt_tensor *ivar, int func);
/* CNetLayerBatchNormalization::TrainingBackward (netlayer/cnetlayerbatchnormalization.cu.h:578-604) as one kernel that also
 * leaves the tensors the literal sequence leaves behind, for callers that replace the sequence behind an unchanged layer:
 * dxhat [B,Z,Y,X] = delta*gamma (line 581), sum_dxhat [1,Z,Y,X] = sum_w dxhat (line 582), sum_dxhat_xhat = sum_w dxhat*xhat
 * (line 585); NULL skips any of them.  dxhat must not be the error or the delta tensor. */
int mt_batchnorm_backward_keep(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta,
                               const mt_tensor *gamma, const mt_tensor *xhat, const mt_tensor *ivar, const mt_tensor *dxhat,
                               const mt_tensor *sum_dxhat, const mt_tensor *sum_dxhat_xhat);
/* Both of the above: CNetLayerFunction::SetOutputError (netlayer/cnetlayerfunction.cu.h:347-358) and the batch-norm layer's
 * TrainingBackward (netlayer/cnetlayerbatchnormalization.cu.h:578-604) as one kernel that leaves what the two literal sequences
 * leave: delta_front [B,Z,Y,X] = delta * f'(gamma*xhat+beta) (the function layer's own delta tensor; may be the same tensor
 * as delta, not the error or dxhat), dxhat = delta_front*gamma, the two sums; NULL skips any of them. */
int mt_batchnorm_backward_func_keep(const mt_tensor *error, const mt_tensor *dgamma, const mt_tensor *dbeta, const mt_tensor *delta,
                                    const mt_tensor *gamma, const mt_tensor *beta, const mt_tensor *xhat, const mt_tensor *ivar, int func,
                                    const mt_tensor *dxhat, const mt_tensor *sum_dxhat, const mt_tensor *sum_dxhat_xhat,
                                    const mt_tensor *delta_front);
/* CNetLayerConvolution::TrainingBackward, netlayer/cnetlayerconvolution.cu.h:501-508, without the per-sample round trip:
 * dkernel [1,1,Kamt,C*Ky*Kx] += sum over the batch of the per-sample weight gradients (CreateDeltaWeightAndBias into a
 * zeroed batch tensor, then AddSumW), dbias [1,Kamt,1,1] += sum over the batch and the pixels of delta. */
int mt_convolution_backward_weights_sum(const mt_tensor *dkernel, int32_t dkernel_x, int32_t dkernel_y, int32_t dkernel_z,
                                        uint32_t dkernel_amount, const mt_tensor *dbias, const mt_tensor *image,
                                        const mt_tensor *delta, int32_t stride_x, int32_t stride_y, int32_t padding_x, int32_t padding_y);

/* TrainingResetDeltaWeight of every layer of a network (netlayer/cnetlayerconvolution.cu.h:522-526 and the same
 * function of the other layers) as one launch: Fill(tensors[i], value) for i < count. */
int mt_fill_many(uint32_t count, const mt_tensor *const *tensors, float value);
/* TrainingUpdateWeight of every layer in Adam mode (netlayer/cnetlayerconvolution.cu.h:533-539 and the same function of
 * the other layers) as one launch: mt_adam on (weight[i], dweight[i], m[i], v[i]) for i < count, same arithmetic. */
int mt_adam_many(uint32_t count, const mt_tensor *const *weight, const mt_tensor *const *dweight, const mt_tensor *const *m,
                 const mt_tensor *const *v, uint32_t batch_size, double speed, double beta1, double beta2, double epsilon, double iteration);

/* ---- functions that only the GPU class of the reference has (no CPU body) ----
 * CTensorMath::ConcatecationZ, cuda/ctensormath.cu.h:473-533: output[w][z] = z < Za ? a[w % Wa][z] : b[w % Wb][z - Za]. */
int mt_concatecation_z(const mt_tensor *output, const mt_tensor *input_a, const mt_tensor *input_b);
/* CTensorMath::SplitZ, cuda/ctensormath.cu.h:538-598: the inverse; w runs over the input's W. */
int mt_split_z(const mt_tensor *output_a, const mt_tensor *output_b, const mt_tensor *input);
/* CTensorMath::SetTimeStep, cuda/ctensormath.cu.h:3029-3091: output = input + sin (even pos) or cos (odd pos) of
 * time_step[w] / 10000^(pos/size), pos the element index within a sample; time_step is [W,1,1,1]. */
int mt_set_time_step(const mt_tensor *output, const mt_tensor *input, const mt_u32_tensor *time_step);
/* CTensorMath::CreateDropOutMatrix / SetNormalNoise / GetNoiseImageAndNoise, cuda/ctensormath.cu.h:3093-3262.  The
 * reference seeds cuRAND with rand(); here the caller passes the seed and the generator is Philox4x32-10 with
 * key = seed and counter = element index: element i of the output depends on (seed, i) only.
 *   drop-out matrix: uniform[0,1) >= drop_out ? 1/(1-drop_out) : 0;   noise: standard normal (Box-Muller);
 *   noisy_image = sqrt_alpha_bar[w] * image + sqrt_one_minus_alpha_bar[w] * noise. */
int mt_create_drop_out_matrix(const mt_tensor *output, float drop_out, uint64_t seed);
int mt_set_normal_noise(const mt_tensor *output, uint64_t seed);
int mt_get_noise_image_and_noise(const mt_tensor *noisy_image, const mt_tensor *noise, const mt_tensor *image, const mt_tensor *sqrt_alpha_bar,
                                 const mt_tensor *sqrt_one_minus_alpha_bar, uint64_t seed);

/* ---- timing: replaces CCUDATimeSpent / CTimeStamp (cuda/ccudatimespent.cu:38-52, cuda/ctimestamp.cu:17-32) ----
 * While enabled, every kernel launch of the hot path is bracketed by two events on the work stream and its
 * duration is accumulated under the kernel's label.  mt_profile_entries() waits for the stream and returns the
 * number of labels seen since profiling was enabled; mt_profile_entry() reads one of them. */
int mt_profile_enable(int on);
int mt_profile_entries(void);
int mt_profile_entry(int index, const char **label, uint64_t *launches, double *total_ms);

#ifdef __cplusplus
}
#endif
#endif
