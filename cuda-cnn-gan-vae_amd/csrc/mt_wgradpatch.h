// Weight gradient, summed over the batch, of a 3 x 3 convolution with stride 1 and padding 1 that has FEW filters on LARGE
// images (the last layers of a generator: 16 or 3 filters at 192 x 256), on the fp32 matrix cores.
//
//   dK[f][c][i][j] = sum over samples and pixels (y, x) of  delta[f][y][x] * image[c][y + i - 1][x + j - 1]
//
// As one product with K = (sample, pixel) the second operand is a gather of single floats, nine per image element, and
// with 16 filters a 64-row tile is three quarters padding.  Here the nine taps share what they read:
//   * a block owns tiles of ROWS x 64 pixels of one sample for a slab of 32 channels; it loads delta's tile (all filters)
//     and the image patch behind it ((ROWS + 2) x 66 per channel, zeros outside the image) ONCE into LDS, in whole rows;
//   * v_mfma_f32_16x16x4_f32 multiplies 16 filters x 4 pixels by 4 pixels x 16 channels: the image operand of tap (i, j)
//     is the patch read at a constant offset, so nine instructions share one delta operand and one patch;
//   * a wave owns 16 channels and one row of the tile, and keeps the 9 x FB accumulators (FB blocks of 16 filters) for the
//     life of the block: blocks are persistent and walk over the tiles, their sums go to the workspace once, as
//     [group][filter][c * 9 + tap], and are added afterwards in a fixed order.
#pragma once

#include "mt_igemm.h"

namespace mt {
namespace igemm {

struct WgradPatchArgs {
  const float *delta;   // [B][KA][H][W]
  const float *image;   // [B][C][H][W]
  float *partial;       // [2 * groups][KA][C * 9]
  uint32_t B, KA, C, H, W;
  uint32_t groups;      // persistent blocks per slab of 32 channels
  uint32_t slabs;       // ceil(C / 32)
};

namespace patch3 {
constexpr int PX = 64, ROWS = 2, SLAB = 32;
constexpr int P_ROW = PX + 8;                      // a patch row: the 64 pixels at 4 .. 67 (128-bit stores), the halo at 3 and 68
constexpr int P_PLANE = (ROWS + 2) * P_ROW + 4;    // a channel's patch; = 4 mod 32 banks: lanes (channel, pixel) spread over the banks
constexpr int D_ROW = ROWS * PX + 4;               // a filter's row of the delta tile, same spread
}  // namespace patch3

// FB: filters / 16, rounded up (1 or 2)
template <int FB>
__global__ __launch_bounds__(THREADS) void wgrad_patch3x3_kernel(WgradPatchArgs a) {
  using namespace patch3;
  static_assert(THREADS == SLAB * (ROWS + 2) * 2, "one thread per halo element of the patch");
  __shared__ __attribute__((aligned(16))) float patch[SLAB * P_PLANE];
  __shared__ __attribute__((aligned(16))) float dtile[FB * 16 * D_ROW];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
  const uint32_t slab = blockIdx.x / a.groups, g = blockIdx.x % a.groups;
  const uint32_t c0 = slab * SLAB;
  const uint32_t segs = a.W / PX, bands = a.H / ROWS, tiles = a.B * bands * segs;
  const uint32_t chunk = wave & 1u, r = wave >> 1;   // the wave's 16 channels and its row of the tile
  // Blocks are dealt to the eight XCDs in turn: the blocks of one XCD take neighbouring tiles at a time, so that the rows two
  // bands share are read through one L2.
  const uint32_t first = a.groups % 8 == 0 ? (g % 8) * (a.groups / 8) + g / 8 : g;
  floatx4 acc[9][FB];
#pragma unroll
  for (int t = 0; t < 9; t++)
#pragma unroll
    for (int fb = 0; fb < FB; fb++) acc[t][fb] = floatx4{0.f, 0.f, 0.f, 0.f};
  // patch loader: 16 neighbouring threads load one row of 64 pixels; a thread keeps its patch row and quad and steps
  // over the channels.  The halo: thread -> (channel, patch row, side).
  const uint32_t p_q = tid & 15u, p_rr = (tid >> 4) & 3u;
  const uint32_t h_side = tid & 1u, h_rr = (tid >> 1) & 3u, h_c = tid >> 3;
  const float *const pa = dtile + (lane & 15u) * D_ROW + r * PX + (lane >> 4);
  const float *const pb = patch + (chunk * 16 + (lane & 15u)) * P_PLANE + r * P_ROW + (lane >> 4) + 3;
  // The loads of the next tile travel into registers while the current one is multiplied.
  floatx4 d_reg[FB * 2], p_reg[SLAB / 4];
  float h_reg = 0.f;
  const size_t plane = (size_t)a.H * a.W;
  auto fetch = [&](uint32_t t) {
    const uint32_t seg = t % segs, band = (t / segs) % bands, w = t / (segs * bands);
    const uint32_t y0 = band * ROWS, x0 = seg * PX;
#pragma unroll
    for (int k = 0; k < FB * 2; k++) {   // delta: FB*16 filters x ROWS rows x 16 quads
      const uint32_t idx = tid + k * THREADS, f = idx >> 5, rr = (idx >> 4) & 1u, q = idx & 15u;
      d_reg[k] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (f < a.KA) d_reg[k] = *(const floatx4 *)(a.delta + (((size_t)w * a.KA + f) * a.H + y0 + rr) * a.W + x0 + 4 * q);
    }
    const int y = (int)y0 - 1 + (int)p_rr;
    const bool row_ok = y >= 0 && y < (int)a.H;
    const float *src = a.image + ((size_t)w * a.C + c0 + wave) * plane + (size_t)(row_ok ? (uint32_t)y : 0u) * a.W + x0 + 4 * p_q;
#pragma unroll
    for (int k = 0; k < SLAB / 4; k++) {   // channels wave, wave + 4, ...
      p_reg[k] = floatx4{0.f, 0.f, 0.f, 0.f};
      if (row_ok && c0 + wave + 4 * k < a.C) p_reg[k] = *(const floatx4 *)(src + (size_t)(4 * k) * plane);
    }
    const int hy = (int)y0 - 1 + (int)h_rr;
    const bool h_ok = c0 + h_c < a.C && hy >= 0 && hy < (int)a.H && (h_side ? x0 + PX < a.W : x0 > 0);
    h_reg = 0.f;
    if (h_ok) h_reg = a.image[((size_t)w * a.C + c0 + h_c) * plane + (size_t)hy * a.W + (h_side ? x0 + PX : x0 - 1)];
  };
  if (first < tiles) fetch(first);
  for (uint32_t t = first; t < tiles; t += a.groups) {
    __syncthreads();   // the previous tile has been multiplied
#pragma unroll
    for (int k = 0; k < FB * 2; k++) {
      const uint32_t idx = tid + k * THREADS, f = idx >> 5, rr = (idx >> 4) & 1u, q = idx & 15u;
      *(floatx4 *)(dtile + f * D_ROW + rr * PX + 4 * q) = d_reg[k];
    }
    {
      float *dst = patch + wave * P_PLANE + p_rr * P_ROW + 4 + 4 * p_q;
#pragma unroll
      for (int k = 0; k < SLAB / 4; k++) *(floatx4 *)(dst + 4 * k * P_PLANE) = p_reg[k];
      patch[h_c * P_PLANE + h_rr * P_ROW + (h_side ? PX + 4 : 3)] = h_reg;
    }
    __syncthreads();
    if (t + a.groups < tiles) fetch(t + a.groups);
#pragma unroll 4
    for (int ks = 0; ks < PX / 4; ks++) {
      float av[FB];
#pragma unroll
      for (int fb = 0; fb < FB; fb++) av[fb] = pa[fb * 16 * D_ROW + 4 * ks];
#pragma unroll
      for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++) {
          const float bv = pb[i * P_ROW + 4 * ks + j];
#pragma unroll
          for (int fb = 0; fb < FB; fb++) acc[i * 3 + j][fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[fb], bv, acc[i * 3 + j][fb], 0, 0, 0);
        }
    }
  }
  // register v of lane l holds (filter 4 * (l / 16) + v, channel l % 16) of its 16 x 16 block
  const uint32_t c = c0 + chunk * 16 + (lane & 15u), ncol = a.C * 9;
  if (c < a.C) {
    float *out = a.partial + (size_t)(g * 2 + r) * a.KA * ncol + c * 9;
#pragma unroll
    for (int fb = 0; fb < FB; fb++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const uint32_t f = fb * 16 + 4 * (lane >> 4) + v;
        if (f < a.KA) {
#pragma unroll
          for (int t = 0; t < 9; t++) out[(size_t)f * ncol + t] = acc[t][fb][v];
        }
      }
  }
}

// Whether the layer is one for this kernel; fills the grid's shape.
inline bool wgrad_patch_plan(WgradPatchArgs &a) {
  using namespace patch3;
  if (a.KA == 0 || a.KA > 32 || a.C == 0 || a.W % PX != 0 || a.H % ROWS != 0) return false;
  if (((uintptr_t)a.delta & 15u) != 0 || ((uintptr_t)a.image & 15u) != 0) return false;
  const size_t tiles = (size_t)a.B * (a.H / ROWS) * (a.W / PX);
  if (tiles < 1024 || tiles >= 0x40000000ull) return false;   // a large image: the persistent blocks need several tiles each
  a.slabs = (a.C + SLAB - 1) / SLAB;
  if (a.C % SLAB != 0 && a.C % SLAB < 16 && a.slabs > 1) return false;   // (a last slab that is mostly padding)
  uint32_t groups = 768 / a.slabs;
  if (groups < 64) return false;
  if (tiles < groups) groups = (uint32_t)tiles;
  a.groups = groups;
  return true;
}

inline int launch_wgrad_patch(const char *name, const WgradPatchArgs &a) {
  const uint32_t grid = a.slabs * a.groups;
  if (a.KA <= 16) wgrad_patch3x3_kernel<1><<<grid, THREADS, 0, stream()>>>(a);
  else wgrad_patch3x3_kernel<2><<<grid, THREADS, 0, stream()>>>(a);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

}  // namespace igemm
}  // namespace mt
