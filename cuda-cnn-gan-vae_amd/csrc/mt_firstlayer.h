// Forward convolution of an image with very few channels (the first layer of a discriminator or an encoder: 3 channels,
// K = C*KY*KX = 27 ... 75) on the fp32 matrix cores.
//
// As an implicit GEMM this layer is all prologue and epilogue: two to five k steps per 64 x 64 tile, a gather of single
// floats per element, and an output (the layer's only real traffic) written 4 bytes per lane.  Here
//   * a block owns a tile of TH x TW output pixels of one image and loads the input patch behind it ONCE, in whole rows,
//     into LDS; the matrix instruction reads it in place: the first operand of v_mfma_f32_32x32x2_f32 is the patch value
//     of (pixel = lane % 32, tap k), an LDS read whose address is a per-lane base plus a compile-time constant;
//   * the second operand, the weights of (filter = lane % 32, tap k), never changes: it lives in registers for the
//     life of the block (all NS k steps, loaded once through LDS);
//   * pixels are the ROWS of the product, so a lane's accumulator registers 4j .. 4j+3 are four neighbouring pixels of
//     one filter: the output is written with 128-bit stores;
//   * blocks are persistent and walk over the tiles: the patches of the next two tiles travel into registers while the
//     current one is multiplied (the loads' latency is longer than a tile's multiplications), one barrier per tile.
// k order.  An instruction multiplies two taps: lanes 0-31 supply tap a, lanes 32-63 tap b.  The taps are paired so that
// the LDS address of b is that of a plus a constant per pair class (the next column, or the next row for the last column
// of a kernel with an odd width); a tap without a partner is multiplied with a zero weight in the other half.
#pragma once

#include "mt_igemm.h"

namespace mt {
namespace igemm {

struct FirstLayerArgs {
  const float *image;   // [W][C][H][Wd]
  const float *kernel;  // [KA][ld], k = (c, ky, kx)
  const float *bias;    // [KA]
  float *out;           // [W][KA][OH][OW]
  uint32_t ld, KA, H, W, OH, OW, batch;
  int32_t pad_y, pad_x;
  uint32_t tiles_x, tiles_y, tiles;
  int func;
};

__device__ __forceinline__ floatx4 make_floatx4(float x, float y, float z, float w) {
  floatx4 v;
  v.x = x; v.y = y; v.z = z; v.w = w;
  return v;
}

template <int C, int KY, int KX>
struct FirstLayerSteps {
  static constexpr int PAIRS_X = KY * (KX / 2);                        // (kx, kx+1) in one row
  static constexpr int PER_C = PAIRS_X + (KX % 2 ? (KY + 1) / 2 : 0);  // + the last column, rows two by two
  static constexpr int NS = C * PER_C;
  // tap a of step i; cls: 0 -> b is the next column, 1 -> b is the next row, 2 -> no b
  __host__ __device__ static constexpr int chan(int i) { return i / PER_C; }
  __host__ __device__ static constexpr int ky(int i) { return (i % PER_C) < PAIRS_X ? (i % PER_C) / (KX / 2 > 0 ? KX / 2 : 1) : 2 * ((i % PER_C) - PAIRS_X); }
  __host__ __device__ static constexpr int kx(int i) { return (i % PER_C) < PAIRS_X ? 2 * ((i % PER_C) % (KX / 2 > 0 ? KX / 2 : 1)) : KX - 1; }
  __host__ __device__ static constexpr int cls(int i) { return (i % PER_C) < PAIRS_X ? 0 : (ky(i) + 1 < KY ? 1 : 2); }
};

// S: stride; NF: filters / 32 (1 or 2); TH x (32*GX): output pixels of a tile
template <int C, int KY, int KX, int S, int NF, int TH, int GX>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 4))) void first_layer_kernel(FirstLayerArgs a) {
  using St = FirstLayerSteps<C, KY, KX>;
  constexpr int NS = St::NS, K = C * KY * KX;
  constexpr int TW = 32 * GX;
  constexpr int PR = (TH - 1) * S + KY, PW = (TW - 1) * S + KX;   // patch rows and columns
  constexpr int PWP = PW | 1;                                     // odd row pitch
  constexpr int PLANE = PR * PWP, PATCH = C * PLANE;
  constexpr int ROWS = C * PR;                                    // (channel, row) pairs of a patch
  constexpr int RW = (ROWS + 3) / 4;                              // ... per wavefront: pair j belongs to wavefront j % 4
  constexpr int CH = (PW + 63) / 64;                              // 64-lane pieces of a patch row
  constexpr int GROUPS = TH * GX;                                 // groups of 32 pixels per tile
  static_assert(GROUPS % 4 == 0, "every wavefront takes the same number of pixel groups");
  constexpr int WROW = K + 1;                                     // weights in LDS: [32*NF][K + 1] (odd pitch)
  __shared__ float patch[2][PATCH + 64];   // (+ 64 floats that take the writes of lanes beyond a row's end: no branch around a write)
  __shared__ float wlds[32 * NF * WROW];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 31, half = lane >> 5;
  const uint32_t HW = a.H * a.W;
  const __amdgpu_buffer_rsrc_t i_rsrc = make_rsrc(a.image, a.batch * C * HW * 4u);
  const uint32_t sample_bytes = a.KA * a.OH * a.OW * 4u;
  const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(a.out, a.batch * sample_bytes);   // (the output is below 2 GiB: checked on the host)

  // ---- the patch of a tile.  One load instruction fetches (a 64-lane piece of) one patch row: the lane's column is the
  // vector offset, image, channel and row are the scalar offset (scalar additions only).  Columns outside the image are
  // out of range per lane, rows outside the image (or a tile that does not exist) for the whole instruction: they read
  // as zero, which is the padding.  Two tiles ahead of the one being multiplied, in two register sets.
  float pv[2][RW * CH];
  auto request = [&](uint32_t tile, auto slot) {
    constexpr int SL = decltype(slot)::value;
    tile = __builtin_amdgcn_readfirstlane(tile);
    const bool exists = tile < a.tiles;
    const uint32_t tx = tile % a.tiles_x, ty = (tile / a.tiles_x) % a.tiles_y, w = exists ? tile / (a.tiles_x * a.tiles_y) : 0u;
    const int32_t iy0 = (int32_t)(ty * TH * S) - a.pad_y, ix0 = (int32_t)(tx * TW * S) - a.pad_x;
    uint32_t voff[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ch++) {
      const int32_t x = ch * 64 + lane, ix = ix0 + x;
      voff[ch] = x < PW && (uint32_t)ix < a.W ? (uint32_t)ix * 4u : OOB;
    }
    const uint32_t image_off = w * C * HW * 4u;
#pragma unroll
    for (int jj = 0; jj < RW; jj++) {
      const int j = jj * 4 + wave, c = j / PR, r = j % PR;   // (uniform: scalar registers)
      const int32_t iy = iy0 + r;
      const bool row = exists && j < ROWS && (uint32_t)iy < a.H;
      const uint32_t soff = row ? image_off + ((uint32_t)c * HW + (uint32_t)iy * a.W) * 4u : 0u, outside = row ? 0u : OOB;   // (scalar selects)
#pragma unroll
      for (int ch = 0; ch < CH; ch++) pv[SL][jj * CH + ch] = buf_load(i_rsrc, voff[ch] | outside, soff);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto deposit = [&](auto slot, int buf) {
    constexpr int SL = decltype(slot)::value;
#pragma unroll
    for (int jj = 0; jj < RW; jj++) {
      const int j = jj * 4 + wave, c = j / PR, r = j % PR;
      float *row = patch[buf] + c * PLANE + r * PWP, *spare = patch[buf] + PATCH;
#pragma unroll
      for (int ch = 0; ch < CH; ch++) {
        float *dst = j < ROWS && ch * 64 + lane < PW ? row + ch * 64 + lane : spare + lane;
        *dst = pv[SL][jj * CH + ch];
      }
    }
  };
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;

  // neighbouring tiles share patch rows and columns: the blocks of an XCD (one L2) take neighbouring tiles of every round
  uint32_t tile = __builtin_amdgcn_readfirstlane(xcd_swizzle(blockIdx.x, gridDim.x));
  if (tile >= a.tiles) return;
  request(tile, Slot0{});
  request(tile + gridDim.x, Slot1{});
  // ---- weights: the kernel tensor through LDS (coalesced), then every lane's NS * NF values for the life of the block
  // (all of a thread's weights requested at once: a loop of load-then-store would pay the memory latency once per round)
  constexpr int WREG = (32 * NF * K + THREADS - 1) / THREADS;
  const __amdgpu_buffer_rsrc_t k_rsrc = make_rsrc(a.kernel, ((a.KA - 1u) * a.ld + K) * 4u);
  float wv[WREG];
#pragma unroll
  for (int q = 0; q < WREG; q++) {
    const int e = q * THREADS + tid, f = e / K, k = e % K;
    wv[q] = buf_load(k_rsrc, e < 32 * NF * K && (uint32_t)f < a.KA ? ((uint32_t)f * a.ld + (uint32_t)k) * 4u : OOB, 0);
  }
#pragma unroll
  for (int q = 0; q < WREG; q++) {
    const int e = q * THREADS + tid, f = e / K, k = e % K;
    if (e < 32 * NF * K) wlds[f * WROW + k] = wv[q];
  }
  deposit(Slot0{}, 0);
  __syncthreads();
  float wr[NS][NF];
#pragma unroll
  for (int i = 0; i < NS; i++) {
    const int ka = St::chan(i) * KY * KX + St::ky(i) * KX + St::kx(i);
    const int kb = St::cls(i) == 0 ? ka + 1 : ka + KX;
#pragma unroll
    for (int f = 0; f < NF; f++) {
      const float wa = wlds[(f * 32 + col) * WROW + ka], wb = St::cls(i) == 2 ? 0.f : wlds[(f * 32 + col) * WROW + kb];
      wr[i][f] = half ? wb : wa;
    }
  }
  float bias_f[NF];
#pragma unroll
  for (int f = 0; f < NF; f++) bias_f[f] = (uint32_t)(f * 32 + col) < a.KA ? a.bias[f * 32 + col] : 0.f;
  const int func = a.func;

  // one tile: LDS buffer `buf` holds it; the register set of the same parity is free (its tile is in LDS) and takes the
  // tile after next; the other set holds the next tile, which goes to the other LDS buffer behind the multiplications
  auto one_tile = [&](auto parity) {
    constexpr int buf = decltype(parity)::value;
    request(tile + 2 * gridDim.x, parity);   // (beyond the last tile: nothing is read)
    const uint32_t tx = tile % a.tiles_x, ty = (tile / a.tiles_x) % a.tiles_y, w = tile / (a.tiles_x * a.tiles_y);
    const float *pl = patch[buf];
#pragma unroll
    for (int gi = 0; gi < GROUPS / 4; gi++) {
      const int g = gi * 4 + wave, gy = g / GX, gx = g % GX;     // the group's row and 32-pixel column block inside the tile
      // LDS address of (pixel = col of the group, first tap): per pair class the other half's displacement
      const int base = (gy * S) * PWP + (gx * 32 + col) * S;
      const float *p0 = pl + base + (half ? 1 : 0), *p1 = pl + base + (half ? PWP : 0), *p2 = pl + base;
      floatx16 acc[NF];
#pragma unroll
      for (int f = 0; f < NF; f++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[f][r] = 0.f;
#pragma unroll
      for (int i = 0; i < NS; i++) {
        const int off = St::chan(i) * PLANE + St::ky(i) * PWP + St::kx(i);
        const float v = St::cls(i) == 0 ? p0[off] : St::cls(i) == 1 ? p1[off] : p2[off];
#pragma unroll
        for (int f = 0; f < NF; f++) acc[f] = __builtin_amdgcn_mfma_f32_32x32x2f32(v, wr[i][f], acc[f], 0, 0, 0);
      }
      // register 4j + q of lane (filter col, half): pixel 8j + 4*half + q of the group.  Stores go through a buffer
      // descriptor: a filter or a row beyond the tensor is an out-of-range offset, not a branch (the count of memory
      // operations in flight stays exact, so the wait before the next patch goes to LDS names only the loads it needs).
      const uint32_t oy = ty * TH + gy, ox = tx * TW + gx * 32 + 4 * half;
#pragma unroll
      for (int f = 0; f < NF; f++) {
        const uint32_t filt = f * 32 + col;
        float v[16];
#pragma unroll
        for (int r = 0; r < 16; r++) v[r] = acc[f][r] + bias_f[f];
        apply_func_cheap_many<16>(func, v);
        const uint32_t voff = filt < a.KA && oy < a.OH ? ((filt * a.OH + oy) * a.OW + ox) * 4u : OOB;
#pragma unroll
        for (int j = 0; j < 4; j++)
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((ext_vector_type(4))) int, make_floatx4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3])), o_rsrc,
                                                 (int)(voff + 32u * j), (int)(w * sample_bytes), 0);
      }
    }
    if (tile + gridDim.x < a.tiles) deposit(std::integral_constant<int, buf ^ 1>{}, buf ^ 1);
    lds_barrier();   // orders LDS traffic only: the loads of the tile after next and this tile's stores stay in flight
    tile = __builtin_amdgcn_readfirstlane(tile + gridDim.x);
  };
#pragma unroll 1
  while (tile < a.tiles) {
    one_tile(Slot0{});
    if (tile >= a.tiles) break;
    one_tile(Slot1{});
  }
}

// the shapes the kernel is built for; returns false when the layer is not one of them
inline bool first_layer_launch(const char *name, FirstLayerArgs &a, int C, int KY, int KX, int S, int *rc) {
  *rc = MT_OK;
  if (a.OW % 32 != 0 || a.OW % 4 != 0 || ((uintptr_t)a.out & 15u) || a.KA < 8 || a.KA > 64 || !epilogue_func(a.func)) return false;   // (filters beyond KA in the last block of 32: zero weights, stores out of range)
  if (!fits_buffer((size_t)a.batch * a.KA * a.OH * a.OW)) return false;
  hipStream_t s = stream();
  auto go = [&](auto kernel, int th, int gx) {
    a.tiles_x = a.OW / (32 * gx);
    a.tiles_y = cdiv(a.OH, th);
    const size_t tiles = (size_t)a.tiles_x * a.tiles_y * a.batch;
    if (tiles > 0x7fffffffu) return false;
    a.tiles = (uint32_t)tiles;
    const uint32_t most = 512;  // persistent blocks, two per compute unit
    kernel<<<a.tiles < most ? a.tiles : most, THREADS, 0, s>>>(a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) *rc = hip_fail(e, name);
    return true;
  };
  const int nf = ((int)a.KA + 31) / 32;
  if (C == 3 && KY == 5 && KX == 5 && S == 1 && nf == 1 && a.OW % 64 == 0) return go(first_layer_kernel<3, 5, 5, 1, 1, 2, 2>, 2, 2);
  if (C == 3 && KY == 5 && KX == 5 && S == 2 && nf == 1) return go(first_layer_kernel<3, 5, 5, 2, 1, 4, 1>, 4, 1);
  if (C == 3 && KY == 3 && KX == 3 && S == 2 && nf == 1 && a.OW % 64 == 0) return go(first_layer_kernel<3, 3, 3, 2, 1, 4, 2>, 4, 2);
  if (C == 3 && KY == 3 && KX == 3 && S == 1 && nf == 1 && a.OW % 64 == 0) return go(first_layer_kernel<3, 3, 3, 1, 1, 4, 2>, 4, 2);
  if (C == 3 && KY == 4 && KX == 4 && S == 2 && nf == 2) return go(first_layer_kernel<3, 4, 4, 2, 2, 4, 1>, 4, 1);
  if (C == 3 && KY == 4 && KX == 4 && S == 2 && nf == 1) return go(first_layer_kernel<3, 4, 4, 2, 1, 4, 1>, 4, 1);
  return false;
}

}  // namespace igemm
}  // namespace mt
