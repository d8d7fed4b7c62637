// Implicit-GEMM core for gfx950: C[M,N] (+)= A[M,K] * B[K,N] on the fp32 matrix cores.
//
//  * 256 threads = 4 wavefronts of 64 lanes; every wavefront owns a (TM*32) x (TN*32) block of C held in
//    TM*TN accumulators of v_mfma_f32_32x32x2_f32 (16 VGPRs each).
//  * A and B never exist as matrices in memory.  Each is an "operand source" that maps (row, k) to an
//    address -- a row-major or column-major matrix, an im2col view of an NCHW image, one stride phase of a
//    transposed convolution, the image view of a weight gradient -- and is staged through LDS as
//    [BK][rows] tiles, double buffered: global loads of tile t+1 are in flight while tile t is multiplied.
//  * A thread always loads the same row (its m or its n) and E consecutive k.  The expensive part of an
//    implicit-GEMM address, decomposing the row into (image, y, x), is therefore done once per thread;
//    the k part is decomposed once per tile and advanced by increments (no per-element division).
//  * For sources whose rows are contiguous in memory the 64 lanes of a wavefront read 64 consecutive
//    rows of one k (coalesced NCHW rows); for k-contiguous sources each thread reads a 16/32-byte vector.
#pragma once

#include "mt_common.h"

namespace mt {
namespace igemm {

constexpr int BK = 16;
constexpr int THREADS = 256;

typedef float floatx16 __attribute__((ext_vector_type(16)));

// matrix index of batch entry bz = (w, z) for an operand with Wop layers of Z matrices each
struct Batch {
  uint32_t wmod = 1, zcount = 1;
  size_t stride = 0;
  __device__ size_t offset(uint32_t bz) const {
    uint32_t w = bz / zcount, z = bz % zcount;
    return (size_t)((w % wmod) * zcount + z) * stride;
  }
};

// element(row, k) = p[row*ld + k]: k contiguous (weights [M][K], Linear activations [B][In])
struct SrcRowK {
  static constexpr bool K_CONTIG = true;
  const float *p;
  uint32_t ld, R, K;
  bool vec;  // ld % 4 == 0 and p 16-byte aligned: vector loads allowed
  Batch bt;
  const float *rowp;
  bool rowok;
  __device__ void batch(uint32_t bz) { p += bt.offset(bz); }
  __device__ void bind(uint32_t row) {
    rowok = row < R;
    rowp = p + (size_t)(rowok ? row : 0) * ld;
  }
  template <int E>
  __device__ void fetch(uint32_t k0, float (&v)[E]) const {
    if (rowok && vec && k0 + E <= K) {
      if constexpr (E % 4 == 0) {
#pragma unroll
        for (int i = 0; i < E; i += 4) {
          float4 t = *reinterpret_cast<const float4 *>(rowp + k0 + i);
          v[i] = t.x; v[i + 1] = t.y; v[i + 2] = t.z; v[i + 3] = t.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < E; i += 2) {
          float2 t = *reinterpret_cast<const float2 *>(rowp + k0 + i);
          v[i] = t.x; v[i + 1] = t.y;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < E; i++) v[i] = (rowok && k0 + i < K) ? rowp[k0 + i] : 0.f;
    }
  }
};

// element(row, k) = p[(row/inner)*gstride + k*ld + row%inner]: rows contiguous (B of Mul, A of TransponseMul);
// `inner` < R folds a batch of matrices that share the other operand into one wide matrix.
struct SrcColK {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t ld, R, K, inner;
  size_t gstride;
  Batch bt;
  const float *rowp;
  bool rowok;
  __device__ void batch(uint32_t bz) { p += bt.offset(bz); }
  __device__ void bind(uint32_t row) {
    rowok = row < R;
    uint32_t r = rowok ? row : 0;
    rowp = p + (size_t)(r / inner) * gstride + r % inner;
  }
  template <int E>
  __device__ void fetch(uint32_t k0, float (&v)[E]) const {
#pragma unroll
    for (int i = 0; i < E; i++) v[i] = (rowok && k0 + i < K) ? rowp[(size_t)(k0 + i) * ld] : 0.f;
  }
};

// im2col view of NCHW images: row = (b, oy, ox), k = (c, ky, kx) with kx fastest;
// element = image[b % in_w][c][oy*sy - py + ky][ox*sx - px + kx], 0 outside the image.
// One stride phase of a transposed convolution is the same view with stride 1 and a (possibly negative) padding.
struct SrcIm2col {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t in_w, C, H, W, KY, KX, OHW, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;  // per-image batching (kernels that differ per sample): stride = C*H*W, wmod = in_w
  const float *base;
  int32_t iy0, ix0;
  bool rowok;
  __device__ void batch(uint32_t bz) { p += bt.offset(bz); }
  __device__ void bind(uint32_t row) {
    rowok = row < R;
    uint32_t r = rowok ? row : 0;
    uint32_t b = r / OHW, q = r % OHW, oy = q / OW, ox = q % OW;
    base = p + (size_t)(b % in_w) * C * H * W;
    iy0 = (int32_t)oy * sy - py;
    ix0 = (int32_t)ox * sx - px;
  }
  template <int E>
  __device__ void fetch(uint32_t k0, float (&v)[E]) const {
    uint32_t taps = KY * KX;
    uint32_t c = k0 / taps, rem = k0 % taps, ky = rem / KX, kx = rem % KX;
#pragma unroll
    for (int i = 0; i < E; i++) {
      int32_t iy = iy0 + (int32_t)ky, ix = ix0 + (int32_t)kx;
      bool ok = rowok && (k0 + i < K) && (uint32_t)iy < H && (uint32_t)ix < W;
      v[i] = ok ? base[((size_t)c * H + (uint32_t)iy) * W + (uint32_t)ix] : 0.f;
      if (++kx == KX) { kx = 0; if (++ky == KY) { ky = 0; ++c; } }
    }
  }
};

// image view of a weight gradient: row = (c, i, j) (a kernel coefficient), k = (oy, ox) (an output pixel);
// element = image[c][oy*sy - py + i][ox*sx - px + j], 0 outside.
struct SrcWgradImage {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t H, W, KY, KX, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;
  const float *base;
  int32_t iy0, ix0;
  bool rowok;
  __device__ void batch(uint32_t bz) { p += bt.offset(bz); }
  __device__ void bind(uint32_t row) {
    rowok = row < R;
    uint32_t r = rowok ? row : 0;
    uint32_t taps = KY * KX, c = r / taps, q = r % taps, i = q / KX, j = q % KX;
    base = p + (size_t)c * H * W;
    iy0 = (int32_t)i - py;
    ix0 = (int32_t)j - px;
  }
  template <int E>
  __device__ void fetch(uint32_t k0, float (&v)[E]) const {
    uint32_t oy = k0 / OW, ox = k0 % OW;
#pragma unroll
    for (int i = 0; i < E; i++) {
      int32_t iy = iy0 + (int32_t)oy * sy, ix = ix0 + (int32_t)ox * sx;
      bool ok = rowok && (k0 + i < K) && (uint32_t)iy < H && (uint32_t)ix < W;
      v[i] = ok ? base[(size_t)(uint32_t)iy * W + (uint32_t)ix] : 0.f;
      if (++ox == OW) { ox = 0; ++oy; }
    }
  }
};

// Where C goes.  Column n decomposes as g = n / inner, r = n % inner; with qw > 0, r is a pixel (qy, qx) of a
// stride phase and lands at ((qy*sy + py) * OW + qx*sx + px).  Element (m, n) is at col(n) + m*row_stride.
// value = acc [+ old C] [+ bias (per row m, or per inner column r)] [+ tap_bias[g % bias_w] * taps(y, x)], then func.
struct Epilogue {
  float *C;
  uint32_t row_stride, inner;
  size_t g_stride;
  uint32_t qw = 0, sy = 1, sx = 1, py = 0, px = 0, OW = 0;
  const float *bias = nullptr;
  int bias_mode = 1;  // 1: one value per row m (and per g % bias_w); 2: one value per inner column r
  uint32_t bias_w = 1, bias_stride = 0;
  // transposed convolution only: the CPU path adds the bias of every filter once per contributing tap
  const float *tap_bias = nullptr;
  int32_t ty_cnt = 0, tx_cnt = 0, offy = 0, offx = 0;
  uint32_t IH = 0, IW = 0;
  int func = MT_F_NONE;
  bool accumulate = false;
  Batch bt;
  uint32_t g0 = 0;  // batched launches: the batch entry's w, so that per-sample biases still index by w

  struct Col {
    size_t off;
    uint32_t g;
    float extra;
  };
  __device__ void batch(uint32_t bz) { C += bt.offset(bz); g0 = bz / bt.zcount; }
  __device__ Col column(uint32_t n) const {
    Col c;
    c.g = g0 + n / inner;
    uint32_t r = n % inner;
    c.extra = (bias && bias_mode == 2) ? bias[r] : 0.f;
    if (qw) {
      uint32_t qy = r / qw, qx = r % qw;
      r = (qy * sy + py) * OW + qx * sx + px;
      if (tap_bias) {
        int ny = 0, nx = 0;
        for (int t = 0; t < ty_cnt; t++) ny += (uint32_t)((int32_t)qy + offy + t) < IH;
        for (int t = 0; t < tx_cnt; t++) nx += (uint32_t)((int32_t)qx + offx + t) < IW;
        c.extra += tap_bias[c.g % bias_w] * (float)(ny * nx);
      }
    }
    c.off = (size_t)(c.g - g0) * g_stride + r;
    return c;
  }
  __device__ void store(const Col &c, uint32_t m, float v) const {
    float *dst = C + c.off + (size_t)m * row_stride;
    if (accumulate) v += *dst;
    if (bias && bias_mode == 1) v += bias[(size_t)(c.g % bias_w) * bias_stride + m];
    v += c.extra;
    *dst = apply_func_epilogue(func, v);
  }
};

template <int TM, int TN, int WGM, int WGN, class SrcA, class SrcB>
__global__ __launch_bounds__(THREADS) void igemm_kernel(SrcA a, SrcB b, Epilogue ep, uint32_t M, uint32_t N, uint32_t K) {
  static_assert(WGM * WGN == 4, "four wavefronts per block");
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int EA = BM * BK / THREADS, EB = BN * BK / THREADS;
  static_assert(EA >= 2 && EB >= 2, "tile too small for the loader");
  __shared__ float As[2][BK][BM];
  __shared__ float Bs[2][BK][BN];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;
  const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  a.batch(blockIdx.z);
  b.batch(blockIdx.z);
  ep.batch(blockIdx.z);

  int a_row, a_k, b_row, b_k;
  if (SrcA::K_CONTIG) { constexpr int TPR = BK / EA; a_row = tid / TPR; a_k = (tid % TPR) * EA; }
  else { a_row = tid % BM; a_k = (tid / BM) * EA; }
  if (SrcB::K_CONTIG) { constexpr int TPR = BK / EB; b_row = tid / TPR; b_k = (tid % TPR) * EB; }
  else { b_row = tid % BN; b_k = (tid / BN) * EB; }
  // with 64 or more rows per tile a wavefront shares one k range: keep its decomposition on the scalar unit
  if (!SrcA::K_CONTIG && BM >= 64) a_k = __builtin_amdgcn_readfirstlane(a_k);
  if (!SrcB::K_CONTIG && BN >= 64) b_k = __builtin_amdgcn_readfirstlane(b_k);
  a.bind(m0 + a_row);
  b.bind(n0 + b_row);

  float ra[EA], rb[EB];
  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const uint32_t nk = (K + BK - 1) / BK;
  a.template fetch<EA>(a_k, ra);
  b.template fetch<EB>(b_k, rb);
#pragma unroll
  for (int i = 0; i < EA; i++) As[0][a_k + i][a_row] = ra[i];
#pragma unroll
  for (int i = 0; i < EB; i++) Bs[0][b_k + i][b_row] = rb[i];
  __syncthreads();

  const int lrow = lane & 31, lk = lane >> 5;
  for (uint32_t kt = 0; kt < nk; kt++) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      a.template fetch<EA>((kt + 1) * BK + a_k, ra);
      b.template fetch<EB>((kt + 1) * BK + b_k, rb);
    }
#pragma unroll
    for (int ks = 0; ks < BK; ks += 2) {
      float av[TM], bv[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) av[i] = As[cur][ks + lk][(wm * TM + i) * 32 + lrow];
#pragma unroll
      for (int j = 0; j < TN; j++) bv[j] = Bs[cur][ks + lk][(wn * TN + j) * 32 + lrow];
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
#pragma unroll
      for (int i = 0; i < EA; i++) As[cur ^ 1][a_k + i][a_row] = ra[i];
#pragma unroll
      for (int i = 0; i < EB; i++) Bs[cur ^ 1][b_k + i][b_row] = rb[i];
    }
    __syncthreads();
  }

  // accumulator layout of v_mfma_f32_32x32x2_f32: register r of lane l holds C[8*(r/4) + 4*(l/32) + r%4][l%32]
#pragma unroll
  for (int j = 0; j < TN; j++) {
    uint32_t n = n0 + (wn * TN + j) * 32 + lrow;
    if (n >= N) continue;
    Epilogue::Col col = ep.column(n);
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        uint32_t m = m0 + (wm * TM + i) * 32 + 8 * (r / 4) + 4 * lk + (r & 3);
        if (m < M) ep.store(col, m, acc[i][j][r]);
      }
    }
  }
}

enum Tile { T128x128, T64x128, T32x128, T64x64 };

inline Tile pick_tile(uint32_t M, uint32_t N) {
  if (M <= 32) return T32x128;
  if (M <= 64) return N >= 8192 ? T64x128 : T64x64;
  size_t big = (size_t)cdiv(M, 128) * cdiv(N, 128);
  if (big >= 512) return T128x128;  // at least two 128x128 blocks per compute unit
  return T64x128;
}

template <class SrcA, class SrcB>
int launch(const char *name, SrcA a, SrcB b, Epilogue ep, uint32_t M, uint32_t N, uint32_t K, uint32_t batches) {
  if (M == 0 || N == 0 || batches == 0) return MT_OK;
  if (batches > 65535u) return fail(MT_E_ARGUMENT, "%s: more than 65535 batched products", name);
  hipStream_t s = stream();
  const Tile tile = pick_tile(M, N);
  static const char *const tile_names[] = {"128x128", "64x128", "32x128", "64x64"};
  ProfileScope prof(profiling() ? intern_label(name, tile_names[tile]) : name);
  switch (tile) {
    case T128x128:
      igemm_kernel<2, 2, 2, 2><<<dim3(cdiv(N, 128), cdiv(M, 128), batches), THREADS, 0, s>>>(a, b, ep, M, N, K);
      break;
    case T64x128:
      igemm_kernel<2, 1, 1, 4><<<dim3(cdiv(N, 128), cdiv(M, 64), batches), THREADS, 0, s>>>(a, b, ep, M, N, K);
      break;
    case T32x128:
      igemm_kernel<1, 1, 1, 4><<<dim3(cdiv(N, 128), cdiv(M, 32), batches), THREADS, 0, s>>>(a, b, ep, M, N, K);
      break;
    case T64x64:
      igemm_kernel<1, 1, 2, 2><<<dim3(cdiv(N, 64), cdiv(M, 64), batches), THREADS, 0, s>>>(a, b, ep, M, N, K);
      break;
  }
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

}  // namespace igemm
}  // namespace mt
