// CTensorMath::Mul / TransponseMul and the Linear layer's forward pass on the fp32 matrix cores.
//
// The reference runs one small product per batch entry (grid.z = W, N = 1 for a Linear layer).  Here a batch
// that shares one operand is folded into a single wide product before it reaches the matrix cores:
//   left  has W == 1:  C[w] = A * B[w]   ->  one product with N' = W*N columns
//   right has W == 1:  C[w] = A[w] * B   ->  one product with M' = W*M rows
// With N == 1 (matrix times a batch of vectors) the folded product is computed transposed, C'[w][m], so that
// the 64 lanes of a wavefront write consecutive addresses.
#include "mt_igemm.h"

namespace {

using namespace mt::igemm;
using mt::cdiv;

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
SrcColK col_k(const float *p, uint32_t ld, uint32_t R, uint32_t K, uint32_t inner, size_t gstride) {
  SrcColK s{};
  s.p = p; s.ld = ld; s.R = R; s.K = K; s.inner = inner; s.gstride = gstride;
  s.groups = inner ? (R + inner - 1) / inner : 1;
  return s;
}

// ---- split-K support (see launch_split in mt_igemm.h): workspace for the partial results and the kernel that adds them
mt::Workspace g_split_ws;

// out[i] = func(sum_s partial[s][i] + bias[(i / bias_div) % bias_mod])
__global__ __launch_bounds__(256) void splitk_reduce_kernel(float *out, const float *partial, uint32_t S, size_t n, const float *bias, uint32_t bias_div,
                                                            uint32_t bias_mod, int func) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float acc = 0.f;
  const float *p = partial + i;
  uint32_t s = 0;
  for (; s + 4 <= S; s += 4, p += 4 * n) {  // four loads in flight
    const float v0 = p[0], v1 = p[n], v2 = p[2 * n], v3 = p[3 * n];
    acc += v0; acc += v1; acc += v2; acc += v3;
  }
  for (; s < S; s++, p += n) acc += p[0];
  if (bias) acc += bias[(i / bias_div) % bias_mod];
  out[i] = mt::apply_func(func, acc);
}
// The same for a small output: 16 outputs per block, 16 threads per output each adding every 16th partial, then the
// 16 sums in a fixed order (one thread per output over all S partials would be a long chain of dependent loads).
__global__ __launch_bounds__(256) void splitk_reduce_small_kernel(float *out, const float *partial, uint32_t S, uint32_t n, const float *bias, uint32_t bias_div,
                                                                  uint32_t bias_mod, int func) {
  const uint32_t t = threadIdx.x, il = t % 16, g = t / 16, i = blockIdx.x * 16 + il;
  __shared__ float part[16][17];
  float acc = 0.f;
  if (i < n)
    for (uint32_t s = g; s < S; s += 16) acc += partial[(size_t)s * n + i];
  part[g][il] = acc;
  __syncthreads();
  if (g == 0 && i < n) {
    float sum = 0.f;
#pragma unroll
    for (uint32_t k = 0; k < 16; k++) sum += part[k][il];
    if (bias) sum += bias[(i / bias_div) % bias_mod];
    out[i] = mt::apply_func(func, sum);
  }
}

// C[w,z] = op(A[w%Wa,z]) * B[w%Wb,z];  op = transpose when `ta` (A stored [K][M]).
// bias (optional) holds one value per output row m; func is applied last.
int product(const char *name, const mt_tensor *out, const mt_tensor *left, const mt_tensor *right, bool ta, const float *bias, int func) {
  if (mt::bad(out) || mt::bad(left) || mt::bad(right)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  mt::note_write(out);
  const uint32_t M = ta ? left->x : left->y, K = ta ? left->y : left->x, N = right->x, Z = left->z;
  if (K != right->y || left->z != right->z || out->y != M || out->x != N || out->z != right->z)
    return mt::fail(MT_E_SHAPE, "%s: sizes do not match", name);
  const uint32_t W = out->w;
  if (W == 0 || Z == 0 || M == 0 || N == 0) return MT_OK;
  if (left->w == 0 || right->w == 0) return mt::fail(MT_E_ARGUMENT, "%s: empty operand", name);
  if (K == 0) return mt_fill(out, 0.f);

  Epilogue ep{};
  ep.C = out->p;
  ep.func = func;
  // a folded batch is addressed through one 32-bit descriptor; otherwise every matrix has its own
  const bool fold_ok = Z == 1 && W > 1 && mt::fits_buffer(left) && mt::fits_buffer(right);
  if (!mt::fits_buffer((size_t)M * K) || !mt::fits_buffer((size_t)K * N))
    return mt::fail(MT_E_UNAVAILABLE, "%s: a single matrix of 2 GiB or more is not supported", name);
  const Batch none{};

  if (fold_ok && left->w == 1 && right->w >= W) {
    if (N == 1) {
      // C'[w][m] = sum_k B[w][k] * op(A)[m][k]: rows are batch entries, columns are the output rows m
      ep.row_stride = M; ep.inner = M; ep.g_stride = 0;
      if (bias) { ep.bias = bias; ep.bias_mode = 2; }
      // bias per output row m = flat index % M
      return with_row_k(right->p, K, W, K, none, [&](auto a) {
        if (ta) return launch_split(name, a, col_k(left->p, M, M, K, M, 0), ep, W, M, K, (size_t)W * M, 1, M);
        return with_row_k(left->p, K, M, K, none, [&](auto b) { return launch_split(name, a, b, ep, W, M, K, (size_t)W * M, 1, M); });
      });
    }
    // one product with N' = W*N columns; column n' = (w, n)
    ep.row_stride = N; ep.inner = N; ep.g_stride = (size_t)M * N;
    if (bias) { ep.bias = bias; ep.bias_mode = 1; }
    // output [w][m][n]: bias per row m = (flat index / N) % M
    SrcColK b = col_k(right->p, N, W * N, K, N, (size_t)K * N);
    if (ta) return launch_split(name, col_k(left->p, M, M, K, M, 0), b, ep, M, W * N, K, (size_t)W * M * N, N, M);
    return with_row_k(left->p, K, M, K, none, [&](auto a) { return launch_split(name, a, b, ep, M, W * N, K, (size_t)W * M * N, N, M); });
  }
  if (fold_ok && right->w == 1 && left->w >= W && !ta && !bias) {
    // rows (w, m) of A and of C are contiguous: one product with M' = W*M rows
    ep.row_stride = N; ep.inner = N; ep.g_stride = 0;
    SrcColK b = col_k(right->p, N, N, K, N, 0);
    return with_row_k(left->p, K, W * M, K, none, [&](auto a) { return launch_split(name, a, b, ep, W * M, N, K, (size_t)W * M * N, 1, 1); });
  }

  // general case: one product per (w, z)
  ep.row_stride = N; ep.inner = N; ep.g_stride = 0;
  ep.bt.wmod = W; ep.bt.zcount = Z; ep.bt.stride = (size_t)M * N;
  if (bias) { ep.bias = bias; ep.bias_mode = 1; }
  SrcColK b = col_k(right->p, N, N, K, N, 0);
  b.bt.wmod = right->w; b.bt.zcount = Z; b.bt.stride = (size_t)K * N;
  if (ta) {
    SrcColK a = col_k(left->p, M, M, K, M, 0);
    a.bt.wmod = left->w; a.bt.zcount = Z; a.bt.stride = (size_t)K * M;
    return launch(name, a, b, ep, M, N, K, W * Z);
  }
  Batch abt;
  abt.wmod = left->w; abt.zcount = Z; abt.stride = (size_t)M * K;
  return with_row_k(left->p, K, M, K, abt, [&](auto a) { return launch(name, a, b, ep, M, N, K, W * Z); });
}

}  // namespace

namespace mt {
int split_workspace(size_t floats, float **p) { return workspace_get(g_split_ws, "split-K workspace", floats, p); }
int split_reduce(const char *name, float *out, const float *partial, uint32_t S, size_t n, const float *bias, uint32_t bias_div, uint32_t bias_mod, int func) {
  if (n <= 16384 && S >= 32)
    splitk_reduce_small_kernel<<<cdiv(n, 16), 256, 0, stream()>>>(out, partial, S, (uint32_t)n, bias, bias_div, bias_mod, func);
  else
    splitk_reduce_kernel<<<cdiv(n, 256), 256, 0, stream()>>>(out, partial, S, n, bias, bias_div, bias_mod, func);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}
}  // namespace mt

extern "C" {

int mt_mul(const mt_tensor *out, const mt_tensor *left, const mt_tensor *right) { return product("mt_mul", out, left, right, false, nullptr, MT_F_NONE); }

int mt_transponse_mul(const mt_tensor *out, const mt_tensor *left, const mt_tensor *right) {
  return product("mt_transponse_mul", out, left, right, true, nullptr, MT_F_NONE);
}

int mt_linear_forward_func(const mt_tensor *out, const mt_tensor *weight, const mt_tensor *input, const mt_tensor *bias, int func) {
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "mt_linear_forward_func: unknown function id %d", func);
  if (mt::bad(out) || mt::bad(weight) || mt::bad(input) || mt::bad(bias)) return mt::fail(MT_E_ARGUMENT, "mt_linear_forward_func: null tensor");
  // the layer views its input as [B,1,In,1] (ReinterpretSize, netlayer/cnetlayerlinear.cu.h:271)
  mt_tensor in = *input;
  in.y = input->z * input->y * input->x;
  in.z = 1;
  in.x = 1;
  if (weight->w != 1 || weight->z != 1 || bias->w != 1 || bias->z != 1 || bias->x != 1 || bias->y != weight->y || out->w != input->w)
    return mt::fail(MT_E_SHAPE, "mt_linear_forward_func: weight must be [1,1,Out,In], bias [1,1,Out,1], output [B,1,Out,1]");
  if (mt::epilogue_func(func)) return product("mt_linear_forward_func", out, weight, &in, false, bias->p, func);
  int rc = product("mt_linear_forward_func", out, weight, &in, false, bias->p, MT_F_NONE);
  return rc == MT_OK ? mt_apply_func(out, out, func) : rc;
}

// CNetLayerLinear::Forward, CNetLayerBatchNormalization::Forward in training mode and CNetLayerFunction::Forward as one
// launch: features are the rows of the product, the batch its columns, and a 16 x 256 block holds the whole batch of its
// 16 features, so the statistics over the batch are sums inside the block (lane shuffles, then the four wavefronts
// through LDS).  Batches above 256 take the two calls.
int mt_linear_batchnorm_forward_func(const mt_tensor *out, const mt_tensor *weight, const mt_tensor *input, const mt_tensor *bias, const mt_tensor *gamma,
                                     const mt_tensor *beta, const mt_tensor *linear_output, const mt_tensor *xhat, const mt_tensor *ivar,
                                     const mt_tensor *batch_mean, const mt_tensor *batch_var, const mt_tensor *new_mean, const mt_tensor *new_variable,
                                     float momentum, float epsilon, int func) {
  const char *name = "mt_linear_batchnorm_forward_func";
  if (!mt::valid_func(func, true)) return mt::fail(MT_E_ARGUMENT, "%s: unknown function id %d", name, func);
  if (mt::bad(out) || mt::bad(weight) || mt::bad(input) || mt::bad(bias) || mt::bad(gamma) || mt::bad(beta)) return mt::fail(MT_E_ARGUMENT, "%s: null tensor", name);
  for (auto t : {out, linear_output, xhat, ivar, batch_mean, batch_var, new_mean, new_variable}) mt::note_write(t);
  const uint32_t B = input->w, In = input->z * input->y * input->x, Out = weight->y;
  if (weight->w != 1 || weight->z != 1 || weight->x != In || bias->w != 1 || bias->z != 1 || bias->x != 1 || bias->y != Out)
    return mt::fail(MT_E_SHAPE, "%s: weight must be [1,1,Out,In], bias [1,1,Out,1]", name);
  const size_t S = Out;
  if (out->w != B || (size_t)out->z * out->y * out->x != S) return mt::fail(MT_E_SHAPE, "%s: output must hold [B,Out] values", name);
  for (auto t : {gamma, beta, ivar, batch_mean, batch_var, new_mean, new_variable})
    if (t && (t->p == nullptr || t->w == 0 || (size_t)t->z * t->y * t->x != S)) return mt::fail(MT_E_SHAPE, "%s: parameters and statistics are [1,...] tensors of Out values", name);
  for (auto t : {linear_output, xhat})
    if (t && (t->p == nullptr || t->w != B || (size_t)t->z * t->y * t->x != S)) return mt::fail(MT_E_SHAPE, "%s: linear_output and xhat hold [B,Out] values", name);
  if (B == 0 || Out == 0) return MT_OK;
  const bool fast = B <= 256 && In > 0 && mt::fits_buffer((size_t)Out * In) && mt::fits_buffer((size_t)B * In) && aligned16(out->p) && (!xhat || aligned16(xhat->p)) &&
                    Out <= 0x7fffffffu / 16u;
  if (!fast) {
    // the layers one after the other; the Linear output goes to its own tensor if there is one, else through `out`
    mt_tensor lin = linear_output ? *linear_output : *out;
    lin.z = 1; lin.y = Out; lin.x = 1;
    int rc = mt_linear_forward_func(&lin, weight, input, bias, MT_F_NONE);
    if (rc) return rc;
    mt_tensor x = *out;   // the same values seen with the output's sizes
    x.p = lin.p;
    return mt_batchnorm_forward_train_func(out, &x, gamma, beta, xhat, ivar, batch_mean, batch_var, new_mean, new_variable, momentum, epsilon, func);
  }
  Epilogue ep{};
  ep.C = out->p; ep.row_stride = 1; ep.inner = 1; ep.g_stride = Out;
  ep.bias = bias->p; ep.bias_mode = 1; ep.func = func;
  ep.bn.gamma = gamma->p; ep.bn.beta = beta->p;
  ep.bn.raw = linear_output ? linear_output->p : nullptr;
  ep.bn.xhat = xhat ? xhat->p : nullptr;
  ep.bn.ivar = ivar ? ivar->p : nullptr;
  ep.bn.mean = batch_mean ? batch_mean->p : nullptr;
  ep.bn.var = batch_var ? batch_var->p : nullptr;
  ep.bn.new_mean = new_mean ? new_mean->p : nullptr;
  ep.bn.new_var = new_variable ? new_variable->p : nullptr;
  ep.bn.inv_n = (float)(1.0 / (double)(float)B);
  ep.bn.eps = epsilon;
  ep.bn.mom_old = momentum;
  ep.bn.mom_new = (float)(1.0 - (double)momentum);
  const uint32_t tiles = cdiv(Out, 16);
  mt::ProfileScope prof(mt::profiling() ? shape_label(name, T16x256, Out, B, In, 1) : name);
  const Batch none{};
  int rc = with_row_k(weight->p, In, Out, In, none, [&](auto a) {
    return with_row_k(input->p, In, B, In, none, [&](auto b) {
      igemm_kernel<1, 2, 1, 4, true, true><<<tiles, THREADS, 0, mt::stream()>>>(a, b, ep, Out, B, In, tiles, 1);
      return MT_OK;
    });
  });
  if (rc) return rc;
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

}  // extern "C"
