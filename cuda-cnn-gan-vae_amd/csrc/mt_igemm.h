// Implicit-GEMM core for gfx950: C[M,N] (+)= A[M,K] * B[K,N] on the fp32 matrix cores.
//
//  * 256 threads = 4 wavefronts of 64 lanes; every wavefront owns a (TM*32) x (TN*32) block of C held in
//    TM*TN accumulators of v_mfma_f32_32x32x2_f32 (16 VGPRs each).  Products of at most 16 rows use
//    v_mfma_f32_16x16x4_f32 instead (R16: a 16 x 256 block, four 16 x 16 accumulators per wavefront), which
//    runs at the same rate and leaves no half of the matrix unit multiplying padding.
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

#include <initializer_list>
#include <type_traits>

#include "mt_common.h"

namespace mt {
namespace igemm {

constexpr int BK = 16;
constexpr int THREADS = 256;

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4acc __attribute__((ext_vector_type(4)));

// matrix index of batch entry bz = (w, z) for an operand with Wop layers of Z matrices each
struct Batch {
  uint32_t wmod = 1, zcount = 1;
  size_t stride = 0;
  size_t wstride = 0;  // > 0: entry (w, z) lies at (w % wmod) * wstride + z * stride (parts of a sample that are not the whole sample)
  __device__ size_t offset(uint32_t bz) const {
    uint32_t w = bz / zcount, z = bz % zcount;
    if (wstride) return (size_t)(w % wmod) * wstride + (size_t)z * stride;
    return (size_t)((w % wmod) * zcount + z) * stride;
  }
};

// ---- operand sources ----------------------------------------------------------------------------------------
// Every source reads through a raw buffer descriptor (buffer_load_dword / _dwordx4).  The hardware range check
// returns 0 for a lane whose byte offset is >= the buffer size, so "outside the operand" is encoded as the offset
// OOB and costs no compare-and-select after the load and no branch around it: the loop body is straight-line
// code and the loads of the next tile stay in flight behind the matrix instructions of the current one.
// The scalar offset operand (uniform over the wavefront) carries what advances from tile to tile.
// Operands must be smaller than 2 GiB (checked on the host); OOB plus any in-range offset stays out of range.
//
// Protocol:  bind(row) once per thread;  seek<E>(k) position at the thread's first k;  fetch<E>(v) load E
// consecutive k;  next<E>() advance by BK.
constexpr uint32_t OOB = 0x80000000u;
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0));
}
__device__ __forceinline__ floatx2 buf_load2(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(floatx2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)soff, 0));
}
__device__ __forceinline__ void buf_store(__amdgpu_buffer_rsrc_t r, float v, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, v), r, (int)voff, (int)soff, 0);
}
__device__ __forceinline__ floatx4 buf_load4(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
}

// element(row, k) = p[row*ld + k]: k contiguous (weights [M][K], Linear activations [B][In]).
// VEC: ld % 4 == 0, K % 4 == 0 and p 16-byte aligned, so every aligned group of 4 (or 2) k is all real or all padding.
// seg > 0: k runs over several matrices of seg columns each (seg a multiple of BK), seg_stride floats apart -- the
// deltas of a whole batch, [w][row][seg], as one long k axis.
template <bool VEC>
struct SrcRowK {
  static constexpr bool K_CONTIG = true;
  const float *p;
  uint32_t ld, R, K;
  Batch bt;
  uint32_t seg = 0, seg_stride = 0;
  uint32_t ksplit = 0;  // > 0: batch entry bz covers k in [bz*ksplit, (bz+1)*ksplit) of one matrix (split-K)
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t voff, kthread, ktile, kseg, segjump;
  __device__ void batch(uint32_t bz) {
    if (ksplit) {
      const uint32_t k0 = bz * ksplit;
      p += k0;
      K = K > k0 ? (K - k0 < ksplit ? K - k0 : ksplit) : 0;
    } else {
      p += bt.offset(bz);
    }
  }
  __device__ void bind(uint32_t row) {
    // the range check applies to vector + scalar offset, so the descriptor spans every matrix of the k axis
    rsrc = make_rsrc(p, seg ? ((K / seg - 1) * seg_stride + R * ld) * 4u : R * ld * 4u);
    voff = row < R ? row * ld * 4u : OOB;
  }
  template <int E>
  __device__ void seek(uint32_t k0) {
    kthread = k0;
    ktile = 0; kseg = 0; segjump = 0;
    if (voff != OOB) voff += k0 * 4u;
  }
  template <int E>
  __device__ void next() {
    ktile += BK;
    if (seg) {
      kseg += BK;
      if (kseg >= seg) { kseg = 0; segjump += (seg_stride - seg) * 4u; }
    }
  }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
    const uint32_t soff = ktile * 4u + segjump, k = kthread + ktile;
    if constexpr (VEC && E % 4 == 0) {
#pragma unroll
      for (int i = 0; i < E; i += 4) {
        floatx4 t = buf_load4(rsrc, k + i + 4 <= K ? voff + i * 4u : OOB, soff);
        v[i] = t.x; v[i + 1] = t.y; v[i + 2] = t.z; v[i + 3] = t.w;
      }
    } else if constexpr (VEC) {
#pragma unroll
      for (int i = 0; i < E; i += 2) {
        floatx2 t = buf_load2(rsrc, k + i + 2 <= K ? voff + i * 4u : OOB, soff);
        v[i] = t.x; v[i + 1] = t.y;
      }
    } else {
#pragma unroll
      for (int i = 0; i < E; i++) v[i] = buf_load(rsrc, k + i < K ? voff + i * 4u : OOB, soff);
    }
  }
};

// element(row, k) = p[(row/inner)*gstride + k*ld + row%inner]: rows contiguous (B of Mul, A of TransponseMul);
// `inner` < R folds a batch of matrices that share the other operand into one wide matrix.
struct SrcColK {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t ld, R, K, inner, groups;  // groups = number of folded matrices (1 when not folded)
  size_t gstride;
  Batch bt;
  uint32_t ksplit = 0;  // > 0: batch entry bz covers k in [bz*ksplit, (bz+1)*ksplit) (split-K)
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t voff, k;
  __device__ void batch(uint32_t bz) {
    if (ksplit) {
      const uint32_t k0 = bz * ksplit;
      p += (size_t)k0 * ld;
      K = K > k0 ? (K - k0 < ksplit ? K - k0 : ksplit) : 0;
    } else {
      p += bt.offset(bz);
    }
  }
  __device__ void bind(uint32_t row) {
    rsrc = make_rsrc(p, (uint32_t)(((size_t)(groups - 1) * gstride + (size_t)K * ld) * 4u));
    voff = row < R ? (uint32_t)((row / inner) * gstride + row % inner) * 4u : OOB;
  }
  template <int E>
  __device__ void seek(uint32_t k0) { k = k0; }
  template <int E>
  __device__ void next() { k += BK; }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
#pragma unroll
    for (int i = 0; i < E; i++) v[i] = buf_load(rsrc, k + i < K ? voff + (k + i) * ld * 4u : OOB, 0);
  }
};

// im2col view of NCHW images: row = (b, oy, ox), k = (c, ky, kx) with kx fastest;
// element = image[b % in_w][c][oy*sy - py + ky][ox*sx - px + kx], 0 outside the image.
// One stride phase of a transposed convolution is the same view with stride 1 and a (possibly negative) padding.
// The k position is kept as (c, ky, kx); it is uniform over a wavefront (scalar registers) for tiles of >= 64 rows.
struct SrcIm2col {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t in_w, C, H, W, KY, KX, OHW, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;  // per-image batching (kernels that differ per sample): stride = C*H*W, wmod = in_w
  uint32_t ksplit = 0, kbase = 0;  // ksplit > 0: batch entry bz covers k in [bz*ksplit, (bz+1)*ksplit) (split-K)
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t imgoff;  // byte offset of the row's image, OOB for rows outside the operand
  int32_t iy0, ix0;
  uint32_t k, c, ky, kx;
  uint32_t step_c, step_ky, step_kx;  // BK = step_c*KY*KX + step_ky*KX + step_kx
  __device__ void batch(uint32_t bz) {
    if (ksplit) {
      kbase = bz * ksplit;
      if (K > kbase + ksplit) K = kbase + ksplit;
    } else {
      p += bt.offset(bz);
    }
  }
  __device__ void bind(uint32_t row) {
    rsrc = make_rsrc(p, in_w * C * H * W * 4u);
    uint32_t r = row < R ? row : 0;
    uint32_t b = r / OHW, q = r % OHW, oy = q / OW, ox = q % OW;
    imgoff = row < R ? (b % in_w) * C * H * W * 4u : OOB;
    iy0 = (int32_t)oy * sy - py;
    ix0 = (int32_t)ox * sx - px;
  }
  template <int E>
  __device__ void seek(uint32_t k0) {
    uint32_t taps = KY * KX;
    k0 += kbase;
    k = k0; c = k0 / taps;
    uint32_t rem = k0 % taps;
    ky = rem / KX; kx = rem % KX;
    step_c = BK / taps;
    rem = BK % taps;
    step_ky = rem / KX; step_kx = rem % KX;
  }
  template <int E>
  __device__ void next() {
    k += BK;
    kx += step_kx;
    if (kx >= KX) { kx -= KX; ky++; }
    ky += step_ky;
    if (ky >= KY) { ky -= KY; c++; }
    c += step_c;
  }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
    uint32_t cc = c, yy = ky, xx = kx;
#pragma unroll
    for (int i = 0; i < E; i++) {
      int32_t iy = iy0 + (int32_t)yy, ix = ix0 + (int32_t)xx;
      bool ok = (k + i < K) && (uint32_t)iy < H && (uint32_t)ix < W;
      uint32_t off = imgoff + ((cc * H + (uint32_t)iy) * W + (uint32_t)ix) * 4u;
      v[i] = buf_load(rsrc, ok ? off : OOB, 0);  // imgoff == OOB keeps a row outside the operand out of range
      if (++xx == KX) { xx = 0; if (++yy == KY) { yy = 0; ++cc; } }
    }
  }
};

// The same view when the taps tile the k step: KY*KX divides BK and C is a multiple of BK/(KY*KX) (so K is a
// multiple of BK).  Then a thread's E elements always hit the same taps; their byte offsets (or OOB) are computed
// once, and from tile to tile only the channel moves -- by the scalar offset.  Per tile: E loads, no vector ALU work.
struct SrcIm2colFixed {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t in_w, C, H, W, KY, KX, OHW, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t imgoff;
  int32_t iy0, ix0;
  uint32_t ksplit = 0;  // > 0: batch entry bz covers k in [bz*ksplit, (bz+1)*ksplit), ksplit a multiple of BK (split-K)
  uint32_t voff[16];
  uint32_t soff, sstep, kpos, kend, kbase = 0;
  __device__ void batch(uint32_t bz) {
    if (ksplit) kbase = bz * ksplit;
    else p += bt.offset(bz);
  }
  __device__ void range() {  // [kpos, kend): this batch entry's part of the k axis
    kpos = kbase;
    kend = ksplit && K > kbase + ksplit ? kbase + ksplit : K;
  }
  __device__ void bind(uint32_t row) {
    rsrc = make_rsrc(p, in_w * C * H * W * 4u);
    uint32_t r = row < R ? row : 0;
    uint32_t b = r / OHW, q = r % OHW, oy = q / OW, ox = q % OW;
    imgoff = row < R ? (b % in_w) * C * H * W * 4u : OOB;
    iy0 = (int32_t)oy * sy - py;
    ix0 = (int32_t)ox * sx - px;
  }
  template <int E>
  __device__ void seek(uint32_t k0) {  // k0 < BK
    static_assert(E <= 16, "at most sixteen elements per thread");
    const uint32_t taps = KY * KX;  // taps divides BK = 16, so taps and KX are powers of two
    const int lt = __builtin_ctz(taps), lx = __builtin_ctz(KX);
#pragma unroll
    for (int i = 0; i < E; i++) {
      uint32_t kk = k0 + i, cc = kk >> lt, t = kk & (taps - 1), ty = t >> lx, tx = t & (KX - 1);
      int32_t iy = iy0 + (int32_t)ty, ix = ix0 + (int32_t)tx;
      bool ok = imgoff != OOB && (uint32_t)iy < H && (uint32_t)ix < W;
      voff[i] = ok ? imgoff + ((cc * H + (uint32_t)iy) * W + (uint32_t)ix) * 4u : OOB;
    }
    range();
    sstep = (BK / taps) * H * W * 4u;
    soff = (kpos / BK) * sstep;
  }
  template <int E>
  __device__ void next() { soff += sstep; kpos += BK; }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
    const uint32_t so = kpos < kend ? soff : OOB;  // beyond this range of k: out of range for every lane (uniform select)
#pragma unroll
    for (int i = 0; i < E; i++) v[i] = buf_load(rsrc, voff[i], so);
  }
};

// The same view with k ordered tap-major, k = (ky*KX + kx)*C + c, for kernels whose taps do not tile the k step (3x3,
// 5x5): C is a multiple of BK, so a tile holds 16 consecutive channels of ONE tap.  A thread's E elements are E
// channels of the same input pixel: their byte offsets (or OOB) are recomputed only when the tap changes, every C/BK
// tiles; in between only the scalar channel offset moves.  The weight matrix must be packed in the same k order.
struct SrcIm2colTap {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t in_w, C, H, W, KY, KX, OHW, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;
  uint32_t ksplit = 0;  // > 0: batch entry bz covers k in [bz*ksplit, (bz+1)*ksplit), ksplit a multiple of BK (split-K)
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t imgoff, kthread;
  int32_t iy0, ix0;
  uint32_t voff[16];
  uint32_t ky, kx, ctile, tiles_per_tap, kpos, kend, kbase = 0;
  __device__ void batch(uint32_t bz) {
    if (ksplit) kbase = bz * ksplit;
    else p += bt.offset(bz);
  }
  __device__ void range() {  // [kpos, kend): this batch entry's part of the k axis
    kpos = kbase;
    kend = ksplit && K > kbase + ksplit ? kbase + ksplit : K;
  }
  __device__ void bind(uint32_t row) {
    rsrc = make_rsrc(p, in_w * C * H * W * 4u);
    uint32_t r = row < R ? row : 0;
    uint32_t b = r / OHW, q = r % OHW, oy = q / OW, ox = q % OW;
    imgoff = row < R ? (b % in_w) * C * H * W * 4u : OOB;
    iy0 = (int32_t)oy * sy - py;
    ix0 = (int32_t)ox * sx - px;
  }
  template <int E>
  __device__ void retap() {
    const int32_t iy = iy0 + (int32_t)ky, ix = ix0 + (int32_t)kx;
    const bool ok = imgoff != OOB && ky < KY && (uint32_t)iy < H && (uint32_t)ix < W;
    const uint32_t base = imgoff + ((kthread * H + (uint32_t)iy) * W + (uint32_t)ix) * 4u;
#pragma unroll
    for (int i = 0; i < E; i++) voff[i] = ok ? base + (uint32_t)i * H * W * 4u : OOB;
  }
  template <int E>
  __device__ void seek(uint32_t k0) {  // k0 < BK: the thread's first channel within a tile
    static_assert(E <= 16, "at most sixteen elements per thread");
    kthread = k0;
    range();
    tiles_per_tap = C / BK;
    const uint32_t tile = kpos / BK, t = tile / tiles_per_tap;
    ctile = tile % tiles_per_tap;
    ky = t / KX; kx = t % KX;
    retap<E>();
  }
  template <int E>
  __device__ void next() {
    kpos += BK;
    if (++ctile == tiles_per_tap) {  // uniform: next tap
      ctile = 0;
      if (++kx == KX) { kx = 0; ++ky; }
      retap<E>();
    }
  }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
    const uint32_t so = kpos < kend ? ctile * BK * H * W * 4u : OOB;
#pragma unroll
    for (int i = 0; i < E; i++) v[i] = buf_load(rsrc, voff[i], so);
  }
};

// image view of a weight gradient: row = (c, i, j) (a kernel coefficient), k = (oy, ox) (an output pixel);
// element = image[c][oy*sy - py + i][ox*sx - px + j], 0 outside.
// OH > 0: k runs over the output pixels of several images in turn, (w, oy, ox), OH*OW a multiple of BK.
struct SrcWgradImage {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t C, H, W, KY, KX, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;
  uint32_t OH = 0;
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t chanoff, woff;
  int32_t iy0, ix0;
  uint32_t k, oy, ox, step_y, step_x;  // BK = step_y*OW + step_x
  __device__ void batch(uint32_t bz) { p += bt.offset(bz); }
  __device__ void bind(uint32_t row) {
    rsrc = make_rsrc(p, (OH ? K / (OH * OW) : 1u) * C * H * W * 4u);  // all images of the k axis: the range check sees vector + scalar offset
    uint32_t r = row < R ? row : 0;
    uint32_t taps = KY * KX, c = r / taps, q = r % taps, i = q / KX, j = q % KX;
    chanoff = row < R ? c * H * W * 4u : OOB;
    iy0 = (int32_t)i - py;
    ix0 = (int32_t)j - px;
  }
  template <int E>
  __device__ void seek(uint32_t k0) {
    k = k0; oy = k0 / OW; ox = k0 % OW; woff = 0;
    step_y = BK / OW; step_x = BK % OW;
    if (OH) { step_y %= OH; }  // a tile may be longer than a whole image of very few pixels
  }
  template <int E>
  __device__ void next() {
    k += BK;
    ox += step_x;
    if (ox >= OW) { ox -= OW; oy++; }
    oy += step_y;
    if (OH) {
      woff += (BK / (OH * OW)) * C * H * W * 4u;
      if (oy >= OH) { oy -= OH; woff += C * H * W * 4u; }
    }
  }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
    if (OW % E == 0) {  // the E elements are consecutive pixels of one output row (k and ox are multiples of E)
      const int32_t iy = iy0 + (int32_t)oy * sy;
      int32_t ix = ix0 + (int32_t)ox * sx;
      const bool row_ok = k < K && (uint32_t)iy < H;
      uint32_t off = chanoff + ((uint32_t)iy * W + (uint32_t)ix) * 4u;
#pragma unroll
      for (int i = 0; i < E; i++) {
        v[i] = buf_load(rsrc, row_ok && (uint32_t)ix < W ? off : OOB, woff);
        ix += sx;
        off += (uint32_t)sx * 4u;
      }
      return;
    }
    uint32_t yy = oy, xx = ox;
#pragma unroll
    for (int i = 0; i < E; i++) {
      int32_t iy = iy0 + (int32_t)yy * sy, ix = ix0 + (int32_t)xx * sx;
      bool ok = (k + i < K) && (uint32_t)iy < H && (uint32_t)ix < W;
      uint32_t off = chanoff + ((uint32_t)iy * W + (uint32_t)ix) * 4u;
      v[i] = buf_load(rsrc, ok ? off : OOB, woff);
      if (++xx == OW) { xx = 0; ++yy; }
    }
  }
};

// The same view when the 16 pixels of a k step are consecutive pixels of one output row (OW % 16 == 0) or a whole
// number of output rows of one image (16 % OW == 0 and OH*OW % 16 == 0), and OW is a multiple of the E pixels a thread
// loads: those pixels then keep their place inside the step's block of pixels, so their byte offsets relative to the
// block's first pixel are computed once.  A step moves the block origin (scalar unit) and re-tests the image borders:
// one test for the row, one per pixel for the column.  K is a multiple of 16 here, every step is complete.
struct SrcWgradImageFixed {
  static constexpr bool K_CONTIG = false;
  const float *p;
  uint32_t C, H, W, KY, KX, OW, R, K;
  int32_t sy, sx, py, px;
  Batch bt;
  uint32_t OH = 0;  // > 0: k runs over the pixels of several images in turn
  uint32_t part_rows = 0;  // > 0: batch entry (w, z) covers the output rows z * part_rows .. of image w only (OH = 0 then)
  __amdgpu_buffer_rsrc_t rsrc;
  uint32_t voff;       // byte offset of the thread's first pixel for the block origin (image 0, row 0, column 0), from p - bias
  int32_t iyc, ixc;    // input row / column of that pixel for that origin
  uint32_t oy, ox, woff, soff, oy0 = 0;
  int32_t Y, X;        // input row / column displacement of the current origin
  static __host__ __device__ bool fits(uint32_t OH_, uint32_t OW_, uint32_t e) {
    return OW_ % e == 0 && (OW_ % BK == 0 || (BK % OW_ == 0 && (OH_ * OW_) % BK == 0));
  }
  __device__ void batch(uint32_t bz) {
    p += bt.offset(bz);
    if (part_rows) oy0 = (bz % bt.zcount) * part_rows;
  }
  __device__ void bind(uint32_t row) {
    // offsets are taken from (py rows + px pixels) in front of the image so that none is negative; elements that would
    // lie in front of the image are masked before they are loaded
    const uint32_t bias = (uint32_t)py * W + (uint32_t)px;
    rsrc = make_rsrc(p - bias, ((OH ? K / (OH * OW) : 1u) * C * H * W + bias) * 4u);
    const uint32_t r = row < R ? row : 0;
    const uint32_t taps = KY * KX, c = r / taps, q = r % taps, i = q / KX, j = q % KX;
    voff = (c * H * W + i * W + j) * 4u;
    iyc = row < R ? (int32_t)i - py : 0x40000000;  // rows beyond R never pass the row test
    ixc = (int32_t)j - px;
  }
  template <int E>
  __device__ void seek(uint32_t k0) {
    const uint32_t dy = k0 / OW, dx = k0 % OW;  // the thread's first pixel inside the block of 16
    voff += (dy * (uint32_t)sy * W + dx * (uint32_t)sx) * 4u;
    iyc += (int32_t)dy * sy;
    ixc += (int32_t)dx * sx;
    oy = oy0; ox = 0; woff = 0; X = 0;
    Y = (int32_t)oy * sy;
    soff = (uint32_t)Y * W * 4u;
  }
  template <int E>
  __device__ void next() {
    if (OW > BK) {
      ox += BK;
      if (ox == OW) { ox = 0; oy++; }
    } else {
      oy += BK / OW;
    }
    if (OH && oy >= OH) { oy = 0; woff += C * H * W * 4u; }
    Y = (int32_t)oy * sy;
    X = (int32_t)ox * sx;
    soff = woff + ((uint32_t)Y * W + (uint32_t)X) * 4u;
  }
  template <int E>
  __device__ void fetch(float (&v)[E]) const {
    const bool row_ok = (uint32_t)(iyc + Y) < H;
    int32_t ix = ixc + X;
    uint32_t off = voff;
#pragma unroll
    for (int i = 0; i < E; i++) {
      v[i] = buf_load(rsrc, row_ok && (uint32_t)ix < W ? off : OOB, soff);
      ix += sx;
      off += (uint32_t)sx * 4u;
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
  uint32_t fair = 0;    // wavefront priorities by remaining k steps (three hexadecimal digits, sixteenths), 0: none
  int func = MT_F_NONE;
  bool accumulate = false;
  Batch bt;
  uint32_t g0 = 0;  // batched launches: the batch entry's w, so that per-sample biases still index by w
  // Batch normalisation over the columns of a block that holds all of them (BN_TAIL kernels only): row m is a feature,
  // the N columns are the batch.  gamma, beta and the statistics are indexed by m.
  struct BnTail {
    const float *gamma = nullptr, *beta = nullptr;
    float *raw = nullptr, *xhat = nullptr, *ivar = nullptr, *mean = nullptr, *var = nullptr, *new_mean = nullptr, *new_var = nullptr;
    float inv_n = 0.f, eps = 0.f, mom_old = 0.f, mom_new = 0.f;
  } bn;

  struct Col {
    size_t off;
    uint32_t g, bias_row;
    float extra;
  };
  __device__ void batch(uint32_t bz) { C += bt.offset(bz); g0 = bz / bt.zcount; }
  __device__ Col column(uint32_t n) const {
    Col c;
    c.g = g0 + n / inner;
    uint32_t r = n % inner;
    c.bias_row = (c.g % bias_w) * bias_stride;
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
  // one value (kernels that hold few values per thread)
  __device__ void store(const Col &c, uint32_t m, float v) const {
    float *dst = C + c.off + (size_t)m * row_stride;
    if (accumulate) v += *dst;
    if (bias && bias_mode == 1) v += bias[c.bias_row + m];
    v += c.extra;
    *dst = apply_func_epilogue(func, v);
  }
  // One accumulator of v_mfma_f32_32x32x2_f32 for column c: register r holds row m_base + 8*(r/4) + r%4.
  // Every option is tested once for the sixteen values, not once per value: old C, then the bias of the row, then
  // the column's extra term, then the function (none, linear, ReLU or leaky ReLU), in this order.
  template <bool FULL>
  __device__ __forceinline__ void store_rows(const Col &c, uint32_t m_base, uint32_t M, floatx16 &v) const {
    float *dst = C + c.off + (size_t)m_base * row_stride;
#define MT_EACH_ROW(body)                                    \
  _Pragma("unroll") for (int r = 0; r < 16; r++) {           \
    const uint32_t dm = 8 * (r / 4) + (r & 3);               \
    if (FULL || m_base + dm < M) { body; }                   \
  }
    if (accumulate) MT_EACH_ROW(v[r] += dst[(size_t)dm * row_stride]);
    if (bias && bias_mode == 1) {
      const float *bp = bias + c.bias_row + m_base;
      MT_EACH_ROW(v[r] += bp[dm]);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) v[r] += c.extra;
    if (func == MT_F_RELU) {
#pragma unroll
      for (int r = 0; r < 16; r++) v[r] = v[r] > 0.f ? v[r] : 0.f;
    } else if (func == MT_F_LEAKY_RELU) {
#pragma unroll
      for (int r = 0; r < 16; r++) v[r] = v[r] > 0.f ? v[r] : (float)(0.1 * (double)v[r]);
    }  // any other function is applied by the host in a pass of its own (see epilogue_func)
    MT_EACH_ROW(dst[(size_t)dm * row_stride] = v[r]);
#undef MT_EACH_ROW
  }
  // One accumulator of v_mfma_f32_16x16x4_f32 for column c: register r holds row m_base + r.  Same order of terms.
  __device__ __forceinline__ void store_quad(const Col &c, uint32_t m_base, uint32_t M, floatx4acc &v) const {
    if (m_base >= M) return;
    float *dst = C + c.off + (size_t)m_base * row_stride;
    const uint32_t rows = M - m_base < 4 ? M - m_base : 4;
    if (accumulate) {
#pragma unroll
      for (int r = 0; r < 4; r++) if ((uint32_t)r < rows) v[r] += dst[(size_t)r * row_stride];
    }
    if (bias && bias_mode == 1) {
      const float *bp = bias + c.bias_row + m_base;
#pragma unroll
      for (int r = 0; r < 4; r++) if ((uint32_t)r < rows) v[r] += bp[r];
    }
#pragma unroll
    for (int r = 0; r < 4; r++) v[r] += c.extra;
    if (func == MT_F_RELU) {
#pragma unroll
      for (int r = 0; r < 4; r++) v[r] = v[r] > 0.f ? v[r] : 0.f;
    } else if (func == MT_F_LEAKY_RELU) {
#pragma unroll
      for (int r = 0; r < 4; r++) v[r] = v[r] > 0.f ? v[r] : (float)(0.1 * (double)v[r]);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) if ((uint32_t)r < rows) dst[(size_t)r * row_stride] = v[r];
  }
  __device__ __forceinline__ void store_block(const Col &c, uint32_t m_base, uint32_t M, floatx16 &v) const {
    if (m_base >= M) return;
    if (m_base + 28 <= M) store_rows<true>(c, m_base, M, v);
    else store_rows<false>(c, m_base, M, v);
  }
};

// LDS tiles are [rows][LDK] with the 16 k of a tile contiguous per row and 4 floats of padding: a row is 80 bytes,
// so eight consecutive rows start in eight different 16-byte bank groups and 128-bit LDS reads and writes of
// consecutive rows are conflict free.
constexpr int LDK = BK + 4;

template <int TM, int TN, int WGM, int WGN>
struct TileShape {
  static constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  static constexpr int LDS_FLOATS = 2 * (BM + BN) * LDK;
};

template <int E>
__device__ __forceinline__ void lds_put(float *dst, const float (&v)[E]) {
  if constexpr (E % 4 == 0) {
#pragma unroll
    for (int i = 0; i < E; i += 4) *reinterpret_cast<float4 *>(dst + i) = make_float4(v[i], v[i + 1], v[i + 2], v[i + 3]);
  } else {
#pragma unroll
    for (int i = 0; i < E; i += 2) *reinterpret_cast<float2 *>(dst + i) = make_float2(v[i], v[i + 1]);
  }
}

// Workgroup barrier that orders LDS traffic only: global loads issued before it stay in flight across it
// (__syncthreads() would also wait for them).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// One (BM x BN) block of C at (m0, n0).  `smem` holds LDS_FLOATS floats, 16-byte aligned.
//
// Feeding v_mfma_f32_32x32x2_f32: lanes 0-31 supply k = 2s and lanes 32-63 supply k = 2s+1 of step s, for the row
// (lane % 32) of A and the column (lane % 32) of B.  Which k of the tile a step multiplies is free as long as A and
// B agree, so lanes 0-31 take k = 0..3 and lanes 32-63 k = 4..7 from ONE 128-bit LDS read (steps 0-3), then
// k = 8..11 / 12..15 from a second one (steps 4-7): two LDS reads per 32 rows and tile instead of eight.
//
// R16 (with TM = 1, WGM = 1): the block is 16 rows of C.  A is still staged 32 rows at a time (two k per thread,
// rows beyond the sixteenth are never read back), and a wavefront's TN*32 columns are 2*TN accumulators of
// v_mfma_f32_16x16x4_f32: lane l supplies row (or column) l % 16 at k slot l / 16, so ONE 128-bit LDS read at
// k offset 4*(l/16) feeds four instructions that together cover the 16 k of a tile (instruction c multiplies
// k = c, 4+c, 8+c, 12+c).  The two halves of a pipeline step are then the two halves of the wavefront's columns.
template <int TM, int TN, int WGM, int WGN, bool R16, bool BN_TAIL = false, class SrcA, class SrcB>
__device__ __forceinline__ void igemm_body(SrcA &a, SrcB &b, const Epilogue &ep, uint32_t M, uint32_t N, uint32_t K, uint32_t m0, uint32_t n0, float *smem) {
  static_assert(WGM * WGN == 4, "four wavefronts per block");
  static_assert(!R16 || (TM == 1 && WGM == 1), "a 16-row block is one row of wavefronts");
  static_assert(!BN_TAIL || R16, "the batch-norm tail belongs to the 16-row block, whose 256 columns hold a whole batch");
  constexpr int BM = WGM * TM * 32, BN = WGN * TN * 32;
  constexpr int EA = BM * BK / THREADS, EB = BN * BK / THREADS;
  static_assert(EA >= 2 && EB >= 2, "tile too small for the loader");
  float *As = smem;                      // [2][BM][LDK]
  float *Bs = smem + 2 * BM * LDK;       // [2][BN][LDK]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  int a_row, a_k, b_row, b_k;
  // k-contiguous sources: TPR threads share a row.  With four threads per row (128 bits each) the LDS takes two rows
  // per cycle, and rows of 80 bytes fill the 32 banks exactly when they are r and r+4 (r and r+1 would share four
  // banks): eight consecutive threads take rows r, r+4.
  auto row_of = [](int t, int tpr) { return tpr == 4 ? ((t / 8) / 4) * 8 + ((t / 8) % 4) + 4 * ((t % 8) / 4) : t / tpr; };
  if (SrcA::K_CONTIG) { constexpr int TPR = BK / EA; a_row = row_of(tid, TPR); a_k = (tid % TPR) * EA; }
  else { a_row = tid % BM; a_k = (tid / BM) * EA; }
  if (SrcB::K_CONTIG) { constexpr int TPR = BK / EB; b_row = row_of(tid, TPR); b_k = (tid % TPR) * EB; }
  else { b_row = tid % BN; b_k = (tid / BN) * EB; }
  // with 64 or more rows per tile a wavefront shares one k range: keep its decomposition on the scalar unit
  if (!SrcA::K_CONTIG && BM >= 64) a_k = __builtin_amdgcn_readfirstlane(a_k);
  if (!SrcB::K_CONTIG && BN >= 64) b_k = __builtin_amdgcn_readfirstlane(b_k);
  a.bind(m0 + a_row);
  b.bind(n0 + b_row);

  float ra[2][EA], rb[2][EB];  // two register sets: the global loads run two tiles ahead of the LDS writes
  floatx16 acc[TM][TN];
  floatx4acc acc16[2 * TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
#pragma unroll
  for (int j = 0; j < 2 * TN; j++)
#pragma unroll
    for (int r = 0; r < 4; r++) acc16[j][r] = 0.f;

  const uint32_t nk = (K + BK - 1) / BK;
  a.template seek<EA>(a_k);
  b.template seek<EB>(b_k);
  float *a_put = As + a_row * LDK + a_k, *b_put = Bs + b_row * LDK + b_k;
  // tile 0 goes to LDS, tiles 1 and 2 (where they exist) are requested; the two cases are separate straight-line
  // paths so that the count of loads in flight is known at compile time on each of them
  auto load_tile = [&](int set, bool advance) {
    // the same issue order everywhere (A, then B), so that the wait before an LDS write names exactly the loads
    // it needs and leaves the younger ones in flight
    if (advance) { a.template next<EA>(); b.template next<EB>(); }
    __builtin_amdgcn_sched_barrier(0);
    a.template fetch<EA>(ra[set]);
    __builtin_amdgcn_sched_barrier(0);
    b.template fetch<EB>(rb[set]);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto prologue = [&](auto tiles) {
    load_tile(0, false);
    lds_put<EA>(a_put, ra[0]);
    lds_put<EB>(b_put, rb[0]);
    if constexpr (decltype(tiles)::value > 1) load_tile(1, true);
    if constexpr (decltype(tiles)::value > 2) load_tile(0, true);
    lds_barrier();
  };

  const int lrow = R16 ? (lane & 15) : (lane & 31), lk = R16 ? (lane >> 4) : (lane >> 5);
  const float *a_get = As + (wm * TM * 32 + lrow) * LDK + lk * 4;
  const float *b_get = Bs + (wn * TN * 32 + lrow) * LDK + lk * 4;
  // fragments of one half: one 128-bit LDS read per 32 rows and 8 k, or (R16) per 16 rows and 16 k
  float4 fa[2][TM], fb[2][TN];
  auto read_half = [&](float4 (&av)[TM], float4 (&bv)[TN], int buf, int half) {
    if constexpr (R16) {
      av[0] = *reinterpret_cast<const float4 *>(a_get + buf * BM * LDK);
#pragma unroll
      for (int j = 0; j < TN; j++) bv[j] = *reinterpret_cast<const float4 *>(b_get + buf * BN * LDK + (half * TN + j) * 16 * LDK);
    } else {
#pragma unroll
      for (int i = 0; i < TM; i++) av[i] = *reinterpret_cast<const float4 *>(a_get + buf * BM * LDK + i * 32 * LDK + half * 8);
#pragma unroll
      for (int j = 0; j < TN; j++) bv[j] = *reinterpret_cast<const float4 *>(b_get + buf * BN * LDK + j * 32 * LDK + half * 8);
    }
  };
  auto multiply = [&](auto half, const float4 (&av)[TM], const float4 (&bv)[TN]) {
#pragma unroll
    for (int c = 0; c < 4; c++)  // consecutive matrix instructions go to different accumulators
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          float x = c == 0 ? av[i].x : c == 1 ? av[i].y : c == 2 ? av[i].z : av[i].w;
          float y = c == 0 ? bv[j].x : c == 1 ? bv[j].y : c == 2 ? bv[j].z : bv[j].w;
          if constexpr (R16) {
            constexpr int blk = decltype(half)::value * TN;
            acc16[blk + j] = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, acc16[blk + j], 0, 0, 0);
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, acc[i][j], 0, 0, 0);
          }
        }
  };

  // Software pipeline, two half tiles per step.  While the matrix instructions of one half run, the wavefront
  // already holds the fragments of the next half in registers, tile t+1 is being written to the other LDS buffer
  // and the global loads of tiles t+2 and t+3 are in flight, so a wavefront keeps its matrix pipe busy on its own:
  //
  //   first half   read fragments (t, half 1) | write tile t+1 to LDS | issue loads of tile t+3 | multiply (t, half 0)
  //   barrier      tile t+1 is complete in LDS and nobody reads the buffer of tile t any more
  //   second half  read fragments (t+1, half 0) | multiply (t, half 1)
  //
  // Steps come in pairs so that the LDS buffer and the register set of a step are compile-time constants, and the
  // last (up to four) steps, which have less left to write or load, are peeled: every step is free of branches, the
  // compiler counts outstanding memory operations exactly and waits for no more than it must.  Nothing is loaded
  // past K.
  auto step = [&](auto parity, auto write_next, auto load_ahead) {
    constexpr int cur = decltype(parity)::value, nxt = cur ^ 1;  // tile t lives in LDS buffer cur, tile t+1 in register set nxt
    read_half(fa[1], fb[1], cur, 1);
    if constexpr (decltype(write_next)::value) {
      lds_put<EA>(a_put + nxt * BM * LDK, ra[nxt]);
      lds_put<EB>(b_put + nxt * BN * LDK, rb[nxt]);
    }
    if constexpr (decltype(load_ahead)::value) load_tile(nxt, true);
    __builtin_amdgcn_sched_barrier(0);  // memory instructions first, their latency hides behind the multiplies
    multiply(std::integral_constant<int, 0>{}, fa[0], fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    if constexpr (decltype(write_next)::value) read_half(fa[0], fb[0], nxt, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(std::integral_constant<int, 1>{}, fa[1], fb[1]);
    __builtin_amdgcn_sched_barrier(0);
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;
  if (nk >= 3) {
    prologue(std::integral_constant<int, 3>{});
    read_half(fa[0], fb[0], 0, 0);
    uint32_t left = nk;
    uint32_t lower2 = 0, lower1 = 0, lower0 = 0;   // see tconv_walk_kernel
    if (ep.fair) {
      lower2 = (left * ((ep.fair >> 8) & 15u) / 16u) & ~1u; lower1 = (left * ((ep.fair >> 4) & 15u) / 16u) & ~1u; lower0 = (left * (ep.fair & 15u) / 16u) & ~1u;
      __builtin_amdgcn_s_setprio(3);
    }
    for (; left > 4; left -= 2) {
      if (ep.fair) {
        if (left == lower2) __builtin_amdgcn_s_setprio(2);
        else if (left == lower1) __builtin_amdgcn_s_setprio(1);
        else if (left == lower0) __builtin_amdgcn_s_setprio(0);
      }
      step(Even{}, Yes{}, Yes{});
      step(Odd{}, Yes{}, Yes{});
    }
    if (left == 4) {
      step(Even{}, Yes{}, Yes{});
      step(Odd{}, Yes{}, No{});
      step(Even{}, Yes{}, No{});
      step(Odd{}, No{}, No{});
    } else {
      step(Even{}, Yes{}, No{});
      step(Odd{}, Yes{}, No{});
      step(Even{}, No{}, No{});
    }
  } else if (nk == 2) {
    prologue(std::integral_constant<int, 2>{});
    read_half(fa[0], fb[0], 0, 0);
    step(Even{}, Yes{}, No{});
    step(Odd{}, No{}, No{});
  } else {
    prologue(std::integral_constant<int, 1>{});
    read_half(fa[0], fb[0], 0, 0);
    step(Even{}, No{}, No{});
  }

  if constexpr (BN_TAIL) {
    // The block's columns are the whole batch (n0 == 0, N <= BN): Linear bias, then the batch normalisation of the
    // layer behind it (netlayer/cnetlayerbatchnormalization.cu.h:301-371) on the accumulators, then the function.
    // Register r of accumulator j of lane l holds C[4*(l/16) + r][wn*TN*32 + 16*j + l%16]: a row's values sit in the 16
    // lanes that share l/16 (lane shuffles), in the 2*TN accumulators of a lane and in the four wavefronts (LDS).
    __syncthreads();                           // every wavefront has read its last operand fragments: the tiles' memory is free
    float *red = smem;                         // [4 wavefronts][16 rows]
    const uint32_t m4 = m0 + 4 * lk;
    const Epilogue::BnTail &bn = ep.bn;
    float v[2 * TN][4];
    bool ok[2 * TN];
    float bias_r[4], gamma_r[4], beta_r[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const bool row = m4 + r < M;
      bias_r[r] = ep.bias && row ? ep.bias[m4 + r] : 0.f;
      gamma_r[r] = row ? bn.gamma[m4 + r] : 0.f;
      beta_r[r] = row ? bn.beta[m4 + r] : 0.f;
    }
    auto row_sums = [&](float (&s)[4]) {       // over the batch: lanes, then wavefronts; every lane gets the totals of its rows
#pragma unroll
      for (int off = 1; off < 16; off <<= 1)
#pragma unroll
        for (int r = 0; r < 4; r++) s[r] += __shfl_xor(s[r], off, 64);
      if (lrow == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) red[wave * 16 + 4 * lk + r] = s[r];
      }
      __syncthreads();
#pragma unroll
      for (int r = 0; r < 4; r++) s[r] = ((red[4 * lk + r] + red[16 + 4 * lk + r]) + red[32 + 4 * lk + r]) + red[48 + 4 * lk + r];
      __syncthreads();
    };
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 2 * TN; j++) {
      ok[j] = n0 + wn * TN * 32 + j * 16 + lrow < N;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        v[j][r] = acc16[j][r] + bias_r[r];
        s[r] += ok[j] ? v[j][r] : 0.f;
      }
    }
    row_sums(s);
    float mean[4], q[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; r++) mean[r] = s[r] * bn.inv_n;
#pragma unroll
    for (int j = 0; j < 2 * TN; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const float raw = v[j][r];
        if (bn.raw && ok[j] && m4 + r < M) bn.raw[(size_t)(n0 + wn * TN * 32 + j * 16 + lrow) * M + m4 + r] = raw;
        v[j][r] = raw - mean[r];
        q[r] += ok[j] ? v[j][r] * v[j][r] : 0.f;
      }
    row_sums(q);
    float iv[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const float vr = q[r] * bn.inv_n;
      iv[r] = (float)(1.0 / (double)sqrtf(vr + bn.eps));
      if (wave == 0 && lrow == 0 && m4 + r < M) {
        const uint32_t m = m4 + r;
        if (bn.mean) bn.mean[m] = mean[r];
        if (bn.var) bn.var[m] = vr;
        if (bn.ivar) bn.ivar[m] = iv[r];
        if (bn.new_mean) bn.new_mean[m] = (bn.mom_old * bn.new_mean[m]) + (bn.mom_new * mean[r]);
        if (bn.new_var) bn.new_var[m] = (bn.mom_old * bn.new_var[m]) + (bn.mom_new * vr);
      }
    }
    const bool whole = m4 + 4 <= M && M % 4 == 0;   // the lane's four rows are one aligned 16-byte piece of a sample
    // xhat in place of the centred values, then the outputs: one look at the function for all of them
    float o[2 * TN][4];
#pragma unroll
    for (int j = 0; j < 2 * TN; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        v[j][r] = v[j][r] * iv[r];
        o[j][r] = gamma_r[r] * v[j][r] + beta_r[r];
      }
    apply_func_epilogue_many<8 * TN>(ep.func, &o[0][0]);
#pragma unroll
    for (int j = 0; j < 2 * TN; j++) {
      if (!ok[j]) continue;
      const size_t at = (size_t)(n0 + wn * TN * 32 + j * 16 + lrow) * M + m4;   // output [batch][features]
      if (whole) {
        *reinterpret_cast<float4 *>(ep.C + at) = make_float4(o[j][0], o[j][1], o[j][2], o[j][3]);
        if (bn.xhat) *reinterpret_cast<float4 *>(bn.xhat + at) = make_float4(v[j][0], v[j][1], v[j][2], v[j][3]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++)
          if (m4 + r < M) {
            ep.C[at + r] = o[j][r];
            if (bn.xhat) bn.xhat[at + r] = v[j][r];
          }
      }
    }
    return;
  }
  if constexpr (R16) {
    // accumulator layout of v_mfma_f32_16x16x4_f32: register r of lane l holds C[4*(l/16) + r][l%16]
#pragma unroll
    for (int j = 0; j < 2 * TN; j++) {
      uint32_t n = n0 + wn * TN * 32 + j * 16 + lrow;
      if (n >= N) continue;
      Epilogue::Col col = ep.column(n);
      ep.store_quad(col, m0 + 4 * lk, M, acc16[j]);
    }
    return;
  }
  // accumulator layout of v_mfma_f32_32x32x2_f32: register r of lane l holds C[8*(r/4) + 4*(l/32) + r%4][l%32]
#pragma unroll
  for (int j = 0; j < TN; j++) {
    uint32_t n = n0 + (wn * TN + j) * 32 + lrow;
    if (n >= N) continue;
    Epilogue::Col col = ep.column(n);
#pragma unroll
    for (int i = 0; i < TM; i++) ep.store_block(col, m0 + (wm * TM + i) * 32 + 4 * lk, M, acc[i][j]);
  }
}

// The hardware hands workgroup L of a 1-D grid to XCD (L % 8), each XCD with its own L2.  Renumbering gives
// XCD x the contiguous logical range [x*total/8, (x+1)*total/8), so blocks that share operand tiles (neighbouring
// logical indices) meet in one L2 instead of eight.
__device__ __forceinline__ uint32_t xcd_swizzle(uint32_t L, uint32_t total) {
  uint32_t per = total / 8;
  if (L >= per * 8) return L;
  return (L % 8) * per + L / 8;
}

__device__ __forceinline__ constexpr uint32_t igemm_group_n() { return 8; }

// Generic launch: logical block index = (n tile, batch entry, m tile), n slowest, so concurrently running blocks
// of one XCD share their B tile (the activations) and cycle through the A tiles (the weights).
template <int TM, int TN, int WGM, int WGN, bool R16, bool BN_TAIL = false, class SrcA, class SrcB>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(TM * TN == 1 ? 5 : TM * TN == 2 ? 3 : 2))) void igemm_kernel(SrcA a, SrcB b, Epilogue ep, uint32_t M, uint32_t N, uint32_t K, uint32_t tiles_m, uint32_t batches) {
  using TS = TileShape<TM, TN, WGM, WGN>;
  __shared__ float4 smem[TS::LDS_FLOATS / 4];
  uint32_t j = xcd_swizzle(blockIdx.x, gridDim.x);
  uint32_t group = tiles_m * batches;
  uint32_t nt = j / group, rem = j % group, bz = rem / tiles_m, mt = rem % tiles_m;
  if (batches == 1 && tiles_m >= 16) {
    // One large product: with m fastest, the blocks that run together (some 160 per XCD) would cover all row tiles of two or
    // three column tiles and stream the whole of A through the L2 once per column tile.  Groups of eight column tiles, column
    // fastest inside a group: the same blocks cover a patch of about 20 x 8 tiles and fetch 28 operand panels instead of 66.
    const uint32_t tiles_n = gridDim.x / tiles_m, per_group = igemm_group_n() * tiles_m, g = j / per_group, idx = j % per_group;
    const uint32_t first = g * igemm_group_n(), gn = tiles_n - first < igemm_group_n() ? tiles_n - first : igemm_group_n();
    mt = idx / gn;
    nt = first + idx % gn;
  }
  a.batch(bz);
  b.batch(bz);
  ep.batch(bz);
  igemm_body<TM, TN, WGM, WGN, R16, BN_TAIL>(a, b, ep, M, N, K, mt * (R16 ? 16 : TS::BM), nt * TS::BN, reinterpret_cast<float *>(smem));
}

enum Tile { T128x128, T64x128, T32x128, T64x64, T16x256 };
static const char *const tile_names[] = {"128x128", "64x128", "32x128", "64x64", "16x256"};
inline uint32_t tile_rows(Tile t) { return t == T128x128 ? 128 : t == T32x128 ? 32 : t == T16x256 ? 16 : 64; }
inline uint32_t tile_cols(Tile t) { return t == T64x64 ? 64 : t == T16x256 ? 256 : 128; }

int &tile_override();  // -1: choose per shape; 0..4: force a Tile (measurements only)
int &patch_blocks();   // persistent blocks of tconv_patch16_kernel (measurements only); default two per compute unit

inline const char *shape_label(const char *name, Tile tile, uint32_t M, uint32_t N, uint32_t K, uint32_t batches) {
  char buf[96];
  snprintf(buf, sizeof buf, "%s M%u N%u K%u x%u", tile_names[tile], M, N, K, batches);
  return intern_label(name, buf);
}

int &igemm_fair();   // wavefront priorities of the one-tile kernels: -1 choose per launch (default), 0 none, else Epilogue::fair as given (measurements only)
// A grid that the chip holds all at once (at least two blocks per compute unit) with long k loops behaves like the kernel
// whose blocks walk over the batch: its blocks start together, and should finish together (see tconv_walk_kernel).
inline uint32_t fair_for(Tile tile, size_t blocks, uint32_t k) {
  if (igemm_fair() >= 0) return (uint32_t)igemm_fair();
  const size_t per_cu = tile == T128x128 ? 2 : tile == T64x128 ? 3 : 5;
  return blocks >= 512 && blocks <= 256 * per_cu && k >= 16 * BK ? 0x842u : 0u;
}
inline Tile pick_tile(uint32_t M, uint32_t N, uint32_t batches) {
  if (tile_override() >= 0) return (Tile)tile_override();
  // the 16x16x4 instruction: no half of the matrix unit multiplies padding; with few columns the narrower block of the
  // 32-row tile gives twice the blocks, which matters more
  if (M <= 16 && (size_t)cdiv(N, 256) * batches >= 256) return T16x256;
  if (M <= 32) return T32x128;
  if (M <= 64) return T64x64;
  // 64x64 blocks need only 20 KB of LDS and 60 registers, so eight of them share a compute unit and hide each
  // other's barriers and load latency; larger blocks only pay off when the grid is huge anyway
  size_t big = (size_t)cdiv(M, 128) * cdiv(N, 128) * batches;
  // (two 128x128 blocks share a compute unit: a grid that is a whole number of rounds of 512, or many rounds.  Measured after
  // a warm-up: 4096^3 1040 us against 1135 us with 64x64 blocks, 4096 x 4096 x 2048 522 against 586; but 3072^3, 576 blocks,
  // 639 against 506, and 2048^3 174 against 172)
  if (big >= 512 && (big % 512 == 0 || big >= 2048)) return T128x128;
  return T64x64;
}

template <class SrcA, class SrcB>
int launch(const char *name, SrcA a, SrcB b, Epilogue ep, uint32_t M, uint32_t N, uint32_t K, uint32_t batches) {
  if (M == 0 || N == 0 || batches == 0) return MT_OK;
  hipStream_t s = stream();
  const Tile tile = pick_tile(M, N, batches);
  ProfileScope prof(profiling() ? shape_label(name, tile, M, N, K, batches) : name);
  const uint32_t bm = tile_rows(tile), bn = tile_cols(tile);
  const uint32_t tm = cdiv(M, bm), tn = cdiv(N, bn);
  const size_t total = (size_t)tm * tn * batches;
  if (total > 0x7fffffffu) return fail(MT_E_ARGUMENT, "%s: problem too large for one launch", name);
  ep.fair = fair_for(tile, total, K);
  switch (tile) {
    case T128x128: igemm_kernel<2, 2, 2, 2, false><<<(uint32_t)total, THREADS, 0, s>>>(a, b, ep, M, N, K, tm, batches); break;
    case T64x128: igemm_kernel<2, 1, 1, 4, false><<<(uint32_t)total, THREADS, 0, s>>>(a, b, ep, M, N, K, tm, batches); break;
    case T32x128: igemm_kernel<1, 1, 1, 4, false><<<(uint32_t)total, THREADS, 0, s>>>(a, b, ep, M, N, K, tm, batches); break;
    case T64x64: igemm_kernel<1, 1, 2, 2, false><<<(uint32_t)total, THREADS, 0, s>>>(a, b, ep, M, N, K, tm, batches); break;
    case T16x256: igemm_kernel<1, 2, 1, 4, true><<<(uint32_t)total, THREADS, 0, s>>>(a, b, ep, M, N, K, tm, batches); break;
  }
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

// ---- split-K: one product with few output tiles and a long k axis ------------------------------------------------
// A product of fewer than 128 output tiles would leave most compute units idle while a few blocks walk the whole k
// axis (a Linear layer 8192 -> 1 for a batch of 128 is two blocks of 512 steps; a 3x3 convolution of 512 channels on
// 6x8 pixels is 96 blocks of 288 steps).  The k axis is cut into S ranges, each range is an ordinary product into its
// own partial result in the library's workspace, and one elementwise kernel adds the S partials in a fixed order,
// then bias and activation.  `out_floats`: the contiguous output the epilogue addresses from ep.C; the bias is given
// as (divisor, modulus) over the flat output index.  Sources must understand `ksplit`.
template <class SrcA, class SrcB>
int launch_split(const char *name, SrcA a, SrcB b, Epilogue ep, uint32_t M, uint32_t N, uint32_t K, size_t out_floats, uint32_t bias_div, uint32_t bias_mod) {
  const size_t tiles = (size_t)cdiv(M, 64) * cdiv(N, 64);
  // up to two blocks per compute unit (one wave per SIMD each) and a long k axis: split down to ranges of 64 steps
  const bool few = tiles < 128 && K >= 512, thin = tiles >= 128 && tiles <= 512 && K >= 2048;
  if (!(few || thin) || out_floats > (1u << 22) || ep.accumulate) return launch(name, a, b, ep, M, N, K, 1);
  uint32_t want = (uint32_t)((few ? 512 : 1024) / tiles);        // ranges wanted
  uint32_t kc = (cdiv(K, want) + BK - 1) / BK * BK;              // range length, a multiple of the k step
  if (kc < 2 * BK) kc = 2 * BK;
  if (thin && kc < 64 * BK) kc = 64 * BK;
  const uint32_t S = cdiv(K, kc);
  if (S < 2) return launch(name, a, b, ep, M, N, K, 1);
  float *partial = nullptr;
  int rc = split_workspace((size_t)S * out_floats, &partial);
  if (rc) return rc;
  float *out = ep.C;
  const float *bias = ep.bias;
  const int func = ep.func;
  a.ksplit = kc; b.ksplit = kc;
  ep.C = partial; ep.bias = nullptr; ep.func = MT_F_NONE;
  ep.bt.wmod = S; ep.bt.zcount = 1; ep.bt.stride = out_floats;
  if ((rc = launch(name, a, b, ep, M, N, kc, S))) return rc;
  return split_reduce(name, out, partial, S, out_floats, bias, bias_div, bias_mod, func);
}

// ---- all stride phases of a transposed convolution in one launch -------------------------------------------------
// Phase f multiplies its packed sub-kernel [M][kp] with the stride-1 im2col view of the delta that has
// taps_y x taps_x taps and offsets (offy, offx), and scatters to output pixels (qy*sy + py, qx*sx + px).
struct TconvPhase {
  const float *packed;
  uint32_t kp, ld, qh, qw;  // packed rows hold kp coefficients, zero-padded to ld (a multiple of 4)
  int32_t taps_y, taps_x, offy, offx;
  uint32_t py, px;
};
constexpr int MAX_PHASES = 16;
struct TconvArgs {
  TconvPhase ph[MAX_PHASES];
  uint32_t nphase, tiles_m, M, out_w;
  uint32_t nsplit = 1, ksplit = 0;  // split-K: slice s of nsplit covers k in [s*ksplit, (s+1)*ksplit) of every phase and
  size_t split_stride = 0;          // writes its own copy of the output, split_stride floats after the previous one
  const float *delta;          // [in_w][C][H][W]
  uint32_t in_w, C, H, W;
  const float *in_scale_shift = nullptr;  // kernels that normalise their input: (scale, shift) pairs [C][H][W][2], and the
  int in_func = MT_F_NONE;                // function applied to scale * x + shift
  Epilogue ep;   // C, row_stride, g_stride, sy, sx, OW, tap_bias, bias_w, IH, IW, func filled in
};

// FIXED: every phase has taps that tile the k step (see SrcIm2colFixed)
template <int TM, int TN, int WGM, int WGN, bool FIXED, bool R16>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(TM * TN == 1 ? 5 : TM * TN == 2 ? 3 : 2))) void tconv_kernel(TconvArgs args) {
  using TS = TileShape<TM, TN, WGM, WGN>;
  __shared__ float4 smem[TS::LDS_FLOATS / 4];
  uint32_t j = xcd_swizzle(blockIdx.x, gridDim.x);
  const uint32_t per_slice = gridDim.x / args.nsplit, slice = j / per_slice;
  j %= per_slice;
  uint32_t group = args.tiles_m * args.nphase;
  uint32_t nt = j / group, rem = j % group, f = rem / args.tiles_m, mt = rem % args.tiles_m;
  const TconvPhase &ph = args.ph[f];
  const uint32_t qhw = ph.qh * ph.qw, N = args.out_w * qhw;
  if (nt * TS::BN >= N) return;  // phases of an odd-sized output differ in size
  const uint32_t k_first = slice * args.ksplit;
  if (k_first >= ph.kp && slice) return;  // a phase with fewer taps has fewer slices; its other copies stay zero
  SrcRowK<true> a{};
  a.p = ph.packed; a.ld = ph.ld; a.R = args.M; a.K = ph.ld;  // rows are zero-padded to ld (a multiple of 4)
  typename std::conditional<FIXED, SrcIm2colFixed, SrcIm2col>::type b{};
  b.p = args.delta; b.in_w = args.in_w; b.C = args.C; b.H = args.H; b.W = args.W;
  b.KY = ph.taps_y ? ph.taps_y : 1; b.KX = ph.taps_x ? ph.taps_x : 1; b.OHW = qhw; b.OW = ph.qw; b.R = N; b.K = ph.kp;
  b.sy = 1; b.sx = 1; b.py = -ph.offy; b.px = -ph.offx;
  Epilogue ep = args.ep;
  ep.inner = qhw; ep.qw = ph.qw; ep.py = ph.py; ep.px = ph.px;
  ep.ty_cnt = ph.taps_y; ep.tx_cnt = ph.taps_x; ep.offy = ph.offy; ep.offx = ph.offx;
  uint32_t klen = ph.kp;
  if (args.nsplit > 1) {
    a.ksplit = args.ksplit; a.batch(slice);   // A rows are zero-padded to ld: its K is ld, the slice may end inside the padding
    b.ksplit = args.ksplit; b.batch(slice);
    klen = ph.kp - k_first < args.ksplit ? ph.kp - k_first : args.ksplit;
    ep.C += (size_t)slice * args.split_stride;
    if (slice) { ep.bias = nullptr; ep.tap_bias = nullptr; }  // the biases enter once, through slice 0
  }
  igemm_body<TM, TN, WGM, WGN, R16>(a, b, ep, args.M, N, klen, mt * (R16 ? 16 : TS::BM), nt * TS::BN, reinterpret_cast<float *>(smem));
}


// ---- stride-2 transposed convolution to at most 16 channels, operands taken from an input patch in LDS -----------
// The four stride phases of a 4x4 stride-2 padding-1 transposed convolution (and of "up-sampling x2, then 3x3
// convolution") are 2x2 convolutions of the SAME input pixels.  As implicit GEMMs every input value is gathered
// 16 times (4 taps x 4 phases) through the texture path, which then limits a layer with few channels.  Here a block
// loads the C x 10 x 34 input patch behind 8 x 32 input pixels once, and the matrix unit reads it in place:
// v_mfma_f32_16x16x4_f32 takes k slot s from lanes 16s..16s+15; one instruction multiplies tap t of the four
// channels 4i..4i+3, so lane l reads patch[4i + l/16][y + py + t/2][x + l%16 + px + t%2] -- a 32-bit LDS read whose
// address differs between (i, t, phase, block of pixels) by constants -- and the four taps of channel 4i + l/16 of
// its row l%16 as one 128-bit read of the packed sub-kernels (k order: channel, tap), which a block keeps in LDS too.
// A wavefront owns 2 x 32 input pixels = four blocks of 16, for both px of one py at a time, and writes the two px
// of an output pixel pair together: whole 128-byte lines.
// Requires: 4 phases of 2x2 taps with offsets (py-1, px-1), phase size = input size, M <= 16, C = CH, bias per row
// or per tap, output 8-byte aligned.
//
// Blocks are persistent (two per compute unit) and walk over the tiles: while the matrix unit works on a tile, the
// next tile's patch is already on its way into registers (half of it requested before each of the two py passes,
// so that never more loads are outstanding than the hardware counts), and the stores of a pass drain behind the
// next pass.  Reads, matrix work and writes of the whole chip then overlap instead of coming in bursts.
template <int CH>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void tconv_patch16_kernel(TconvArgs args, uint32_t tiles_x, uint32_t tiles_y, uint32_t tiles) {
  constexpr int TY = 8, TX = 32, P = TX + 2, ROWS = TY + 2;
  constexpr int PLANE = ROWS * P + 28;  // 368: planes of consecutive channels start 16 banks apart
  static_assert(PLANE % 32 == 16 && CH % 4 == 0, "LDS layout");
  constexpr int PAIRS = CH / 4 * ROWS;  // (channel, row) pairs per wavefront, requested in two halves
  static_assert(CH % 8 == 0 && PAIRS / 2 <= 40, "two batches of loads, each within the outstanding-load counter");
  constexpr int WROW = CH * 4 + 4;       // a row of coefficients plus 16 bytes: 128-bit reads of 8 rows hit 8 bank groups
  __shared__ float patch[CH * PLANE];
  __shared__ float coeff[4 * 16 * WROW];  // [phase][row][channel*4 + tap], rows beyond M zero
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int jj = lane & 15, slot = lane >> 4;
  const uint32_t H = args.H, W = args.W, HW = H * W;

  // the patch: every (channel, row) pair is one load instruction of 34 lanes; a wavefront takes a quarter of the
  // channels.  The lane's column goes into the vector offset, channel and row into the scalar offset (additions
  // only); either may be out of range.
  float v[PAIRS];
  auto request_patch = [&](uint32_t tile, auto half) {  // tile >= tiles: every load is out of range (no branch)
    tile = __builtin_amdgcn_readfirstlane(tile);  // uniform by construction: keeps the offsets below on the scalar unit
    const uint32_t none = tile < tiles ? 0u : OOB;
    const uint32_t bx = tile % tiles_x, by = (tile / tiles_x) % tiles_y, w = tile / (tiles_x * tiles_y);
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(args.delta + (size_t)(w % args.in_w) * CH * HW, CH * HW * 4u);
    const int32_t gx = (int32_t)(bx * TX) - 1 + lane;
    const uint32_t voff = lane < P && (uint32_t)gx < W ? (uint32_t)gx * 4u : OOB;
    constexpr int C0 = decltype(half)::value * (CH / 8);
    // scalar offsets: one per row (exactly 2^31 for rows outside the image or a tile that does not exist: with the
    // channel offset, below 2^31, the sum stays out of range) plus one per channel; a load costs one scalar addition
    uint32_t row_off[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; r++) {
      const int32_t row = (int32_t)(by * TY) - 1 + r;
      const uint32_t outside = (uint32_t)((row | ((int32_t)H - 1 - row)) >> 31) | (none ? ~0u : 0u);  // all ones for row < 0 or row >= H
      row_off[r] = (((uint32_t)row * W * 4u) & ~outside) | (outside & OOB);
    }
    uint32_t s_chan = (uint32_t)(wave * (CH / 4) + C0) * HW * 4u;
#pragma unroll
    for (int cl = C0; cl < C0 + CH / 8; cl++) {
#pragma unroll
      for (int r = 0; r < ROWS; r++) v[cl * ROWS + r] = buf_load(rsrc, voff, s_chan + row_off[r]);
      s_chan += HW * 4u;
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto store_patch = [&]() {
    float *dst = patch + wave * (CH / 4) * PLANE + lane;
#pragma unroll
    for (int i = 0; i < PAIRS; i++)
      if (lane < P) dst[(i / ROWS) * PLANE + (i % ROWS) * P] = v[i];
  };
  using First = std::integral_constant<int, 0>;
  using Second = std::integral_constant<int, 1>;

  // neighbouring tiles share patch rows and columns: the blocks of an XCD (one L2) take neighbouring tiles of every round
  uint32_t tile = __builtin_amdgcn_readfirstlane(xcd_swizzle(blockIdx.x, gridDim.x));
  if (tile >= tiles) return;
  request_patch(tile, First{});
  request_patch(tile, Second{});
  // the coefficients of all four phases, once per block (their loads travel with those of the first patch)
  {
    constexpr int VEC = 4 * 16 * CH;  // 128-bit pieces
    static_assert(VEC % THREADS == 0, "whole rounds of loads");
#pragma unroll
    for (int i = 0; i < VEC / THREADS; i++) {
      const int e = i * THREADS + tid, f = e / (16 * CH), row = (e / CH) % 16, piece = e % CH;
      const TconvPhase &ph = args.ph[f];
      const __amdgpu_buffer_rsrc_t rs = make_rsrc(ph.packed, args.M * ph.ld * 4u);
      const floatx4 t = buf_load4(rs, (uint32_t)row < args.M ? ((uint32_t)row * ph.ld + (uint32_t)piece * 4u) * 4u : OOB, 0);
      *reinterpret_cast<floatx4 *>(coeff + (f * 16 + row) * WROW + piece * 4) = t;
    }
  }
  store_patch();
  const float *b_lane = patch + slot * PLANE + wave * 2 * P + jj;
  __syncthreads();

#pragma unroll 1
  for (; tile < tiles; tile = __builtin_amdgcn_readfirstlane(tile + gridDim.x)) {
    const uint32_t bx = tile % tiles_x, by = (tile / tiles_x) % tiles_y, w = tile / (tiles_x * tiles_y);
    const uint32_t y0 = by * TY, x0 = bx * TX;
    const uint32_t next = tile + gridDim.x;
    // bias of the lane's four rows (per row, and per sample where the caller has one set per sample)
    float row_bias[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const uint32_t m = (uint32_t)(slot * 4 + r);
      row_bias[r] = args.ep.bias && m < args.M ? args.ep.bias[(w % args.ep.bias_w) * args.ep.bias_stride + m] : 0.f;
    }
#pragma unroll
    for (uint32_t py = 0; py < 2; py++) {
      if (py == 0) request_patch(next, First{});
      else request_patch(next, Second{});
      floatx4acc acc[4][2];
#pragma unroll
      for (int b = 0; b < 4; b++)
#pragma unroll
        for (int px = 0; px < 2; px++)
#pragma unroll
          for (int r = 0; r < 4; r++) acc[b][px][r] = 0.f;
      // the patch values of step (i, t) + 1 are read while the eight matrix instructions of step (i, t) run; the
      // two px of a block are neighbours in LDS
      const float *b_py = b_lane + py * P;
      float bv[2][4][2];
      auto read_step = [&](int set, int step) {
        const int i = step >> 2, t = step & 3;
#pragma unroll
        for (int b = 0; b < 4; b++) {
          const float *q = b_py + i * 4 * PLANE + ((b >> 1) + (t >> 1)) * P + (b & 1) * 16 + (t & 1);
          bv[set][b][0] = q[0];
          bv[set][b][1] = q[1];
        }
      };
      // coefficients of the phases (py, 0) and (py, 1) for the lane's row and the channels 4i + slot: read one
      // group of four steps ahead
      const float *a_py = coeff + (py * 2 * 16 + jj) * WROW + slot * 4;
      floatx4 av[2][2];
      auto read_coefficients = [&](int set, int i) {
#pragma unroll
        for (int px = 0; px < 2; px++) av[set][px] = *reinterpret_cast<const floatx4 *>(a_py + px * 16 * WROW + i * 16);
      };
      read_coefficients(0, 0);
      read_step(0, 0);
#pragma unroll
      for (int step = 0; step < CH; step++) {
        if (step + 1 < CH) read_step((step + 1) & 1, step + 1);
        if ((step & 3) == 0 && step + 4 < CH) read_coefficients(((step >> 2) + 1) & 1, (step >> 2) + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int px = 0; px < 2; px++)
            acc[b][px] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[(step >> 2) & 1][px][step & 3], bv[step & 1][b][px], acc[b][px], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // accumulator layout: register r of lane l holds channel 4*(l/16) + r of pixel l%16.  value = acc + bias of
      // the row + bias of every filter once per contributing tap (as the CPU path adds it), then the function: the
      // order of the other kernels.  Output pixel (2*qy + py, 2*qx + px): the two px are written together.
      float *image = args.ep.C + (size_t)w * args.ep.g_stride;
      if (args.ep.tap_bias) {
        const float tap_bias = args.ep.tap_bias[w % args.ep.bias_w];
#pragma unroll
        for (int b = 0; b < 4; b++) {
          const uint32_t qy = y0 + wave * 2 + (b >> 1), qx = x0 + (b & 1) * 16 + jj;
          const int ny = (int)((uint32_t)(qy + py - 1) < H) + (int)((uint32_t)(qy + py) < H);
          const float extra0 = tap_bias * (float)(ny * ((int)((uint32_t)(qx - 1) < W) + 1));
          const float extra1 = tap_bias * (float)(ny * (1 + (int)(qx + 1 < W)));
#pragma unroll
          for (int r = 0; r < 4; r++) {
            acc[b][0][r] = acc[b][0][r] + row_bias[r] + extra0;
            acc[b][1][r] = acc[b][1][r] + row_bias[r] + extra1;
          }
        }
      } else {  // (vector instructions of one wavefront do not overlap with the matrix instructions of another: fewer is faster)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int r = 0; r < 4; r++) {
            acc[b][0][r] += row_bias[r];
            acc[b][1][r] += row_bias[r];
          }
      }
      // the function is tested once for the 32 values (callers pass none, linear, ReLU or leaky ReLU)
      if (args.ep.func == MT_F_RELU) {
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int px = 0; px < 2; px++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[b][px][r] = acc[b][px][r] > 0.f ? acc[b][px][r] : 0.f;
      } else if (args.ep.func == MT_F_LEAKY_RELU) {
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
          for (int px = 0; px < 2; px++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[b][px][r] = acc[b][px][r] > 0.f ? acc[b][px][r] : (float)(0.1 * (double)acc[b][px][r]);
      }
#pragma unroll
      for (int b = 0; b < 4; b++) {
        const uint32_t qy = y0 + wave * 2 + (b >> 1), qx = x0 + (b & 1) * 16 + jj;
        const bool pixel = qy < H && qx < W;
        const uint32_t off = (2 * qy + py) * args.ep.OW + 2 * qx;
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const uint32_t m = (uint32_t)(slot * 4 + r);
          if (pixel && m < args.M) *reinterpret_cast<float2 *>(image + (m * args.ep.row_stride + off)) = make_float2(acc[b][0][r], acc[b][1][r]);
        }
      }
    }
    if (next < tiles) {  // barriers that order LDS traffic only: the stores of this tile keep draining behind them
      lds_barrier();     // nobody reads the old patch any more
      store_patch();
      lds_barrier();
    }
  }
}

// whether the launch is the shape tconv_patch16_kernel covers; on success `order` maps (py, px) to the phase index
inline bool tconv_patch16_fits(const TconvArgs &args) {
  if (args.nphase != 4 || args.M > 16 || (args.C != 16 && args.C != 32) || args.ep.sy != 2 || args.ep.sx != 2 || args.ep.accumulate || !epilogue_func(args.ep.func)) return false;
  if ((args.ep.bias && args.ep.bias_mode != 1) || ((uintptr_t)args.ep.C & 7u) || args.ep.row_stride % 2 || args.ep.g_stride % 2 || args.ep.OW != 2 * args.W) return false;
  if ((uint64_t)args.M * args.ep.row_stride >= (1u << 30) || (args.ep.tap_bias && args.ep.IH != args.H) || (args.ep.tap_bias && args.ep.IW != args.W)) return false;
  for (uint32_t f = 0; f < 4; f++) {
    const TconvPhase &ph = args.ph[f];
    if (ph.py != f / 2 || ph.px != f % 2 || ph.taps_y != 2 || ph.taps_x != 2 || ph.offy != (int32_t)ph.py - 1 || ph.offx != (int32_t)ph.px - 1 ||
        ph.qh != args.H || ph.qw != args.W || ph.kp != args.C * 4)
      return false;
  }
  return true;
}

// out_floats > 0: the whole output tensor (args.ep.C, out_floats values, every pixel written by exactly one phase) may be
// produced as the sum of k ranges when the launch has few blocks and a long k axis (see launch_split): every range
// writes its own copy of the output in the workspace, the copies are added in a fixed order, then the function.
inline int launch_tconv(const char *name, TconvArgs &args, uint32_t max_n, size_t out_floats = 0) {
  if (args.M == 0 || max_n == 0 || args.nphase == 0) return MT_OK;
  hipStream_t s = stream();
  if (tile_override() < 0 && tconv_patch16_fits(args)) {
    const uint32_t tiles_x = cdiv(args.W, 32), tiles_y = cdiv(args.H, 8);
    const size_t tiles = (size_t)tiles_x * tiles_y * args.out_w;
    if (tiles <= 0x7fffffffu) {
      ProfileScope prof(profiling() ? shape_label(name, T16x256, args.M, max_n, args.C * 4, 4) : name);
      args.nsplit = 1;
      const uint32_t most = (uint32_t)patch_blocks();  // persistent blocks, two per compute unit
      const uint32_t grid = tiles < most ? (uint32_t)tiles : most;
      if (args.C == 16) tconv_patch16_kernel<16><<<grid, THREADS, 0, s>>>(args, tiles_x, tiles_y, (uint32_t)tiles);
      else tconv_patch16_kernel<32><<<grid, THREADS, 0, s>>>(args, tiles_x, tiles_y, (uint32_t)tiles);
      MT_LAUNCH_CHECK(name);
      return MT_OK;
    }
  }
  const Tile tile = pick_tile(args.M, max_n, args.nphase);
  const uint32_t bm = tile_rows(tile), bn = tile_cols(tile);
  args.tiles_m = cdiv(args.M, bm);
  size_t total = (size_t)args.tiles_m * cdiv(max_n, bn) * args.nphase;
  uint32_t kmax = 0, kmin = 0xffffffffu;
  for (uint32_t f = 0; f < args.nphase; f++) {
    kmax = args.ph[f].kp > kmax ? args.ph[f].kp : kmax;
    kmin = args.ph[f].kp < kmin ? args.ph[f].kp : kmin;
  }
  float *out = args.ep.C;
  const int func_in_kernel = args.ep.func;
  args.nsplit = 1;
  // (two blocks on every compute unit already keep the matrix pipes busy: splitting 512 blocks cost more in the extra
  // pass over the output than it gained)
  if (out_floats && out_floats <= (1u << 22) && total <= 384 && kmin >= 1024) {
    const uint32_t want = (uint32_t)(1024 / total);
    uint32_t kc = (cdiv(kmax, want) + BK - 1) / BK * BK;
    if (kc < 32 * BK) kc = 32 * BK;
    const uint32_t S = cdiv(kmax, kc);
    if (S >= 2) {
      float *partial = nullptr;
      int rc = split_workspace((size_t)S * out_floats, &partial);
      if (rc) return rc;
      if (kmin != kmax) {  // phases with fewer taps leave some copies untouched: those must read as zero
        const mt_tensor all{partial, 1, 1, S, (uint32_t)out_floats};
        if ((rc = mt_fill(&all, 0.f))) return rc;
      }
      args.nsplit = S; args.ksplit = kc; args.split_stride = out_floats;
      args.ep.C = partial; args.ep.func = MT_F_NONE;
      total *= S;
    }
  }
  ProfileScope prof(profiling() ? shape_label(name, tile, args.M, max_n, args.nsplit > 1 ? args.ksplit : args.ph[0].kp, args.nphase * args.nsplit) : name);
  if (total > 0x7fffffffu) return fail(MT_E_ARGUMENT, "%s: problem too large for one launch", name);
  bool fixed = true;
  for (uint32_t f = 0; f < args.nphase; f++) {
    uint32_t taps = args.ph[f].taps_y * args.ph[f].taps_x;
    fixed = fixed && taps != 0 && BK % taps == 0 && args.C % (BK / taps) == 0;
  }
  const uint32_t grid = (uint32_t)total;
  args.ep.fair = fair_for(tile, total, args.nsplit > 1 ? args.ksplit : args.ph[0].kp);
  if (fixed) {
    switch (tile) {
      case T128x128: tconv_kernel<2, 2, 2, 2, true, false><<<grid, THREADS, 0, s>>>(args); break;
      case T64x128: tconv_kernel<2, 1, 1, 4, true, false><<<grid, THREADS, 0, s>>>(args); break;
      case T32x128: tconv_kernel<1, 1, 1, 4, true, false><<<grid, THREADS, 0, s>>>(args); break;
      case T64x64: tconv_kernel<1, 1, 2, 2, true, false><<<grid, THREADS, 0, s>>>(args); break;
      case T16x256: tconv_kernel<1, 2, 1, 4, true, true><<<grid, THREADS, 0, s>>>(args); break;
    }
  } else {
    switch (tile) {
      case T128x128: tconv_kernel<2, 2, 2, 2, false, false><<<grid, THREADS, 0, s>>>(args); break;
      case T64x128: tconv_kernel<2, 1, 1, 4, false, false><<<grid, THREADS, 0, s>>>(args); break;
      case T32x128: tconv_kernel<1, 1, 1, 4, false, false><<<grid, THREADS, 0, s>>>(args); break;
      case T64x64: tconv_kernel<1, 1, 2, 2, false, false><<<grid, THREADS, 0, s>>>(args); break;
      case T16x256: tconv_kernel<1, 2, 1, 4, false, true><<<grid, THREADS, 0, s>>>(args); break;
    }
  }
  MT_LAUNCH_CHECK(name);
  if (args.nsplit > 1) {
    const float *partial = args.ep.C;
    const uint32_t S = args.nsplit;
    args.ep.C = out; args.ep.func = func_in_kernel; args.nsplit = 1;
    return split_reduce(name, out, partial, S, out_floats, nullptr, 1, 1, func_in_kernel);
  }
  return MT_OK;
}

}  // namespace igemm
}  // namespace mt
