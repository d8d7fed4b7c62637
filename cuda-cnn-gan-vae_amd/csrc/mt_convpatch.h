// Transposed convolution 3 x 3, stride 1, padding 1 (the backward pass of such a convolution layer) from FEW filters on LARGE
// images -- the last layers of a generator: 16 or 3 filters at 192 x 256 -- on the fp32 matrix cores.
//
//   out[c][y][x] = sum over filters f and taps (a, b) of  kernel[f][c*9 + a*3 + b] * delta[f][y - a + 1][x - b + 1]
//                  + (sum of the filters' biases) * (number of taps inside the image)          (cpu/ctensorconv.h:204-268)
//
// As an implicit GEMM the k axis (filters x taps) is 27 ... 288 long: a block is all prologue and epilogue, and every value
// of delta is gathered nine times.  Here
//   * a block owns tiles of ROWS x 64 output pixels of one sample and loads the patch of delta behind it ((ROWS + 2) x 66
//     values per filter, zeros outside the image) ONCE into LDS, in whole rows;
//   * v_mfma_f32_16x16x4_f32 multiplies 16 pixels x 4 filters by 4 filters x 16 output channels: its first operand is the
//     patch read in place (lane l: pixel l % 16 of filter 4q + l / 16, at an address that differs between taps by
//     constants), the second -- the weights of (filter 4q + l / 16, channel l % 16, tap) -- never changes and lives in
//     registers for the life of the block;
//   * a wave owns 16 output channels and a share of the tile's pixels; a lane's accumulator registers are four
//     neighbouring pixels of one channel: 128-bit stores;
//   * blocks are persistent and walk over the tiles; the next tile's patch travels into registers while the current one is
//     multiplied.
#pragma once

#include "mt_igemm.h"

namespace mt {
namespace igemm {

struct TconvPatchArgs {
  const float *delta;    // [B][F][H][W]
  const float *kernel;   // [F][ld], column c*9 + a*3 + b
  const float *bias;     // [F]
  float *out;            // [B][C][H][W]
  uint32_t B, F, C, H, W, ld;
  uint32_t groups;       // persistent blocks
  int func;              // forward convolution only: the function behind it (none, linear, ReLU, leaky ReLU)
};

namespace tpatch {
constexpr int PX = 64, ROWS = 2;
constexpr int P_ROW = PX + 8;                       // the 64 pixels at 4 .. 67 (128-bit stores), the halo at 3 and 68
constexpr int P_PLANE = (ROWS + 2) * P_ROW + 16;    // = 16 mod 32 banks: the four filters of an instruction read disjoint banks
}  // namespace tpatch

// FQ: filters / 4, rounded up to 1, 2, 4 or 8; NC: output channels / 16, rounded up (1, 2 or 4).
// FWD: the forward convolution of such a layer on the same machine -- `delta` is the image (F channels), `kernel` is
// [C][ld] with column f*9 + a*3 + b, tap (a, b) reads image[f][y + a - 1][x + b - 1], `bias` holds one value per output
// channel and `func` follows:  out[c][y][x] = func(bias[c] + sum kernel[c][f*9 + a*3 + b] * image[f][y + a - 1][x + b - 1]).
template <int FQ, int NC, bool FWD = false>
__global__ __launch_bounds__(THREADS) void tconv3x3_patch_kernel(TconvPatchArgs a) {
  using namespace tpatch;
  constexpr int NP = FQ * 4;             // planes of the patch
  constexpr int NPB = 2 * NC;            // blocks of 16 pixels per wave (a tile has 8)
  __shared__ __attribute__((aligned(16))) float patch[NP * P_PLANE];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t g = blockIdx.x;
  const uint32_t segs = a.W / PX, bands = a.H / ROWS, tiles = a.B * bands * segs;
  const uint32_t cb = wave % NC, pb0 = (wave / NC) * NPB;
  const uint32_t first = a.groups % 8 == 0 ? (g % 8) * (a.groups / 8) + g / 8 : g;   // one XCD takes neighbouring tiles at a time
  // the weights of (filter 4q + lane / 16, channel cb*16 + lane % 16), all nine taps
  float wreg[9][FQ];
  const uint32_t c = cb * 16 + (lane & 15u);
#pragma unroll
  for (int q = 0; q < FQ; q++) {
    const uint32_t f = 4 * q + (lane >> 4);
#pragma unroll
    for (int t = 0; t < 9; t++)
      wreg[t][q] = f < a.F && c < a.C ? (FWD ? a.kernel[(size_t)c * a.ld + f * 9 + t] : a.kernel[(size_t)f * a.ld + c * 9 + t]) : 0.f;
  }
  float bias_sum = 0.f;   // backward: the sum of the filters' biases; forward: the output channel's own
  if constexpr (FWD) {
    bias_sum = c < a.C ? a.bias[c] : 0.f;
  } else {
    for (uint32_t f = 0; f < a.F; f++) bias_sum += a.bias[f];
  }
  // loader: 16 neighbouring threads load one row of 64 pixels; a thread keeps its patch row and quad and steps over the
  // filters.  The halo: thread -> (filter, patch row, side).
  const uint32_t p_q = tid & 15u, p_rr = (tid >> 4) & 3u;
  const uint32_t h_side = tid & 1u, h_rr = (tid >> 1) & 3u, h_f = tid >> 3;
  const size_t plane = (size_t)a.H * a.W;
  floatx4 p_reg[FQ];
  float h_reg = 0.f;
  auto fetch = [&](uint32_t t) {
    const uint32_t seg = t % segs, band = (t / segs) % bands, w = t / (segs * bands);
    const uint32_t y0 = band * ROWS, x0 = seg * PX;
    const int y = (int)y0 - 1 + (int)p_rr;
    const bool row_ok = y >= 0 && y < (int)a.H;
    const float *src = a.delta + ((size_t)w * a.F + wave) * plane + (size_t)(row_ok ? (uint32_t)y : 0u) * a.W + x0 + 4 * p_q;
#pragma unroll
    for (int k = 0; k < FQ; k++) {   // filters wave, wave + 4, ...
      p_reg[k] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (row_ok && wave + 4 * k < a.F) p_reg[k] = *(const floatx4 *)(src + (size_t)(4 * k) * plane);
    }
    const int hy = (int)y0 - 1 + (int)h_rr;
    const bool h_ok = h_f < a.F && hy >= 0 && hy < (int)a.H && (h_side ? x0 + PX < a.W : x0 > 0);
    h_reg = 0.f;
    if (h_ok) h_reg = a.delta[((size_t)w * a.F + h_f) * plane + (size_t)hy * a.W + (h_side ? x0 + PX : x0 - 1)];
  };
  if (first < tiles) fetch(first);
  for (uint32_t t = first; t < tiles; t += a.groups) {
    const uint32_t seg = t % segs, band = (t / segs) % bands, w = t / (segs * bands);
    const uint32_t y0 = band * ROWS, x0 = seg * PX;
    __syncthreads();   // the previous tile has been multiplied
    {
      float *dst = patch + wave * P_PLANE + p_rr * P_ROW + 4 + 4 * p_q;
#pragma unroll
      for (int k = 0; k < FQ; k++) *(floatx4 *)(dst + 4 * k * P_PLANE) = p_reg[k];
      if (h_f < NP) patch[h_f * P_PLANE + h_rr * P_ROW + (h_side ? PX + 4 : 3)] = h_reg;
    }
    __syncthreads();
    if (t + a.groups < tiles) fetch(t + a.groups);
    floatx4 acc[NPB];
#pragma unroll
    for (int i = 0; i < NPB; i++) acc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    // lane l reads pixel l % 16 of filter 4q + l / 16; output row r needs patch rows r + 2 - a, column x + 5 - b
    // (forward: rows r + a, column x + 3 + b)
    const float *pa = patch + (lane >> 4) * P_PLANE + (lane & 15u) + (FWD ? 3 : 5);
#pragma unroll
    for (int i = 0; i < NPB; i++) {
      const uint32_t pb = pb0 + i, r = pb >> 2, xb = pb & 3u;
      const float *pr = pa + (r + (FWD ? 0 : 2)) * P_ROW + xb * 16;
#pragma unroll
      for (int ta = 0; ta < 3; ta++)
#pragma unroll
        for (int tb = 0; tb < 3; tb++)
#pragma unroll
          for (int q = 0; q < FQ; q++)
            acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(FWD ? pr[4 * q * P_PLANE + ta * P_ROW + tb] : pr[4 * q * P_PLANE - ta * P_ROW - tb], wreg[ta * 3 + tb][q],
                                                          acc[i], 0, 0, 0);
    }
    // register v of lane l holds (pixel 4 * (l / 16) + v, channel l % 16) of its block of 16 pixels
    if (c < a.C) {
#pragma unroll
      for (int i = 0; i < NPB; i++) {
        const uint32_t pb = pb0 + i, r = pb >> 2, xb = pb & 3u;
        const uint32_t y = y0 + r, x = x0 + xb * 16 + 4 * (lane >> 4);
        floatx4 v = acc[i];
        if constexpr (FWD) {
          v.x = apply_func_epilogue(a.func, v.x + bias_sum);
          v.y = apply_func_epilogue(a.func, v.y + bias_sum);
          v.z = apply_func_epilogue(a.func, v.z + bias_sum);
          v.w = apply_func_epilogue(a.func, v.w + bias_sum);
        } else {
          const float ny = 3.f - (y == 0 ? 1.f : 0.f) - (y + 1 == a.H ? 1.f : 0.f);
          const float inner = bias_sum * (ny * 3.f);
          v.x += x == 0 ? bias_sum * (ny * 2.f) : inner;
          v.y += inner;
          v.z += inner;
          v.w += x + 4 == a.W ? bias_sum * (ny * 2.f) : inner;
        }
        *(floatx4 *)(a.out + ((size_t)w * a.C + c) * plane + (size_t)y * a.W + x) = v;
      }
    }
  }
}

// Whether the layer is one for this kernel; fills the number of persistent blocks.
inline bool tconv_patch_plan(TconvPatchArgs &a) {
  using namespace tpatch;
  if (a.F == 0 || a.F > 32 || a.C == 0 || a.C > 64 || a.W % PX != 0 || a.H % ROWS != 0) return false;
  if (((uintptr_t)a.delta & 15u) != 0 || ((uintptr_t)a.out & 15u) != 0) return false;
  const size_t tiles = (size_t)a.B * (a.H / ROWS) * (a.W / PX);
  if (tiles < 1024 || tiles >= 0x40000000ull) return false;
  a.groups = 768;
  return true;
}

template <int FQ, bool FWD>
inline void launch_tconv_patch_nc(const TconvPatchArgs &a) {
  const uint32_t nc = (a.C + 15) / 16;
  if (nc == 1) tconv3x3_patch_kernel<FQ, 1, FWD><<<a.groups, THREADS, 0, stream()>>>(a);
  else if (nc == 2) tconv3x3_patch_kernel<FQ, 2, FWD><<<a.groups, THREADS, 0, stream()>>>(a);
  else tconv3x3_patch_kernel<FQ, 4, FWD><<<a.groups, THREADS, 0, stream()>>>(a);
}

template <bool FWD>
inline int launch_patch(const char *name, const TconvPatchArgs &a) {
  if (a.F <= 4) launch_tconv_patch_nc<1, FWD>(a);
  else if (a.F <= 8) launch_tconv_patch_nc<2, FWD>(a);
  else if (a.F <= 16) launch_tconv_patch_nc<4, FWD>(a);
  else launch_tconv_patch_nc<8, FWD>(a);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}
inline int launch_tconv_patch(const char *name, const TconvPatchArgs &a) { return launch_patch<false>(name, a); }
inline int launch_conv_patch(const char *name, const TconvPatchArgs &a) { return launch_patch<true>(name, a); }

}  // namespace igemm
}  // namespace mt
