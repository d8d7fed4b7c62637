// Transposed convolution on the fp32 matrix cores whose blocks walk over the batch, with the two halves of a batch
// normalisation folded into it: the statistics of the layer's own output (epilogue) and the normalisation + activation
// that its input still owes (loader).  A forward convolution whose taps tile the k step (4x4, 2x2, 1x1 kernels) is the
// same kernel with one "phase": the operand is gathered with the convolution's stride (in_sy, in_sx), the weights are
// the layer's kernel tensor as it is, and every output channel has its bias (ROWBIAS).
//
// A block owns one stride phase, 64 output channels and one tile of PX pixels x SP samples (PX * SP = 64 columns), and
// walks from one group of SP samples to the next, `per` groups in all.  Going to the next group changes nothing but a
// scalar byte offset of the operand loads, so the walk is ONE long k loop: the loads of the next group's first tiles
// are in flight while the last tiles of the current one are multiplied, and the only pause of the matrix pipe is the
// epilogue itself (the stores of a group drain behind the multiplications of the next).  The one-tile blocks of
// tconv_kernel pay a cold start and a drain per tile.
//
// STATS.  Walking the batch is what makes the statistics cheap: a block sees per * SP samples of every output element
// it owns.  Each lane keeps a running mean and sum of squared deviations (Welford) of its sixteen elements over the
// groups it walks, merges the SP samples of a tile at the end (lane shuffles for samples that sit in one wavefront's
// columns, LDS between the two wavefronts along the columns) and writes ONE (mean, M2) pair per element and block.
// The pairs of the blocks are combined in a fixed order by a small kernel afterwards: no pass over the activation, and
// a result that does not depend on timing.
//
// NORM.  The input is the raw output of a layer whose batch normalisation and activation are still owed: every value
// becomes func(scale * x + shift) on its way from the load to LDS, with (scale, shift) per element (c, y, x) fetched as
// one 64-bit value beside it.  Elements outside the image stay exactly zero: their pair is loaded out of range as well,
// and func(0 * 0 + 0) = 0 for the functions allowed here.
#pragma once

#include "mt_igemm.h"

namespace mt {
namespace igemm {

struct WalkArgs {
  TconvPhase ph[MAX_PHASES];
  uint32_t nphase, tiles_m, M, batch;
  uint32_t px_log, qtiles, groups, per;  // PX = 1 << px_log pixels per tile; pixel tiles per phase; batch groups; steps per block
  uint32_t nk;                           // k steps of one block's tile (the same for every phase): all of them, or one of ksplit equal shares
  uint32_t ksplit = 1;                   // blocks that share a tile's k steps; block ks writes its sums to out + ks * split_stride (per = 1 then)
  size_t split_stride = 0;               // floats
  uint32_t wide = 0;                     // 1: blocks of 32 rows x 128 columns (set by the caller before planning; plain variant only)
  uint32_t flat = 0;                     // 1: the columns are (sample, pixel) pairs counted through the whole batch, 64 to a tile (qtiles of
                                         // them, the last one may be ragged), for pixel counts that no tile of 16, 32 or 64 divides; no walk
  uint32_t weights_major;                // block order, see tconv_walk_kernel
  uint32_t fair;                         // 0, or three hexadecimal digits: sixteenths of the steps left at which a wavefront's priority drops to 2, 1, 0
  const float *delta;                    // [batch][C][H][W]
  const float *scale_shift;              // NORM: [C][H][W][2]
  int in_func;                           // NORM: none, linear, ReLU or leaky ReLU
  uint32_t C, H, W;
  float *out;                            // [batch][M][OH][OW]
  uint32_t OW, OHW, sy, sx;
  uint32_t in_sy = 1, in_sx = 1;         // stride of the gather: input pixel = output pixel * stride + offset + tap (1 for a transposed convolution)
  const float *row_bias = nullptr;       // ROWBIAS: one value per output channel, [M]
  const float *tap_bias;                 // sum of the filters' biases, added once per contributing tap (may be null)
  int func;                              // applied to the output (cheap functions only); with STATS: none
  float *part_mean, *part_m2;            // STATS: [groups][M * OHW] each
};

// Merges two sets of n samples each, given as (mean, sum of squared deviations): Chan's update for equal counts.
__device__ __forceinline__ void welford_merge_equal(float &mean, float &m2, float other_mean, float other_m2, float half_n) {
  const float d = other_mean - mean;
  mean = mean + 0.5f * d;
  m2 = (m2 + other_m2) + (d * d) * half_n;
}

// TM: 32-row accumulators per wavefront (the block is 64*TM rows x 64 columns, 2 x 2 wavefronts)
// NORM: 0 the input is used as it is, 1 ReLU(scale * x + shift), 2 any of the cheap functions of it (chosen at run time: a
// branch per element in the loader, which the one case that generators use should not pay)
// WIDE: the block is 32 rows x 128 columns, four wavefronts side by side (layers with 32 output channels; plain variant
// only: no statistics, no normalisation of the input, one accumulator per wavefront)
template <int NORM, bool STATS, int WAVES, int TM, bool ROWBIAS = false, bool WIDE = false>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) void tconv_walk_kernel(WalkArgs a) {
  static_assert(!WIDE || (NORM == 0 && !STATS && TM == 1), "the 32 x 128 block exists as the plain variant only");
  constexpr int BM = WIDE ? 32 : 64 * TM, BN = WIDE ? 128 : 64, E = 4;  // four elements per thread, operand and 64 rows
  constexpr int NB = BN / 64;   // sets of four k per thread and step in operand B (a step is 16 k of BN columns)
  __shared__ float4 smem4[2 * (BM + BN) * LDK / 4];
  float *smem = reinterpret_cast<float *>(smem4);
  float *As = smem, *Bs = smem + 2 * BM * LDK;

  // An XCD runs a contiguous range of logical blocks.  Ordered by batch group first, the blocks of an XCD share the
  // samples of a few groups in its L2 and between them read every packed weight.  When the weights of the layer do not
  // fit an L2 beside the rest (weights_major), the order is by row tile first: an XCD then reads one row tile's weights
  // (all phases) again and again from its own L2 and streams its share of the input through once; the phases of a
  // tile stay neighbours, so their stores, which interleave pixel by pixel, still meet in one L2.
  uint32_t j = xcd_swizzle(blockIdx.x, gridDim.x), mt, f, qt, g, ks = 0;
  if (a.ksplit > 1) { ks = j % a.ksplit; j /= a.ksplit; }
  if (a.weights_major) {
    f = j % a.nphase; j /= a.nphase;
    qt = j % a.qtiles; j /= a.qtiles;
    g = j % a.groups; mt = j / a.groups;
  } else {
    mt = j % a.tiles_m; j /= a.tiles_m;
    f = j % a.nphase; j /= a.nphase;
    qt = j % a.qtiles; g = j / a.qtiles;
  }
  const TconvPhase &ph = a.ph[f];
  const uint32_t m0 = mt * BM, HW = a.H * a.W, sp = (uint32_t)BN >> a.px_log, px_mask = (1u << a.px_log) - 1u;

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = WIDE ? 0 : wave >> 1, wn = WIDE ? wave : wave & 1;
  const bool a_loader = !WIDE || wave < 2;   // 32 rows of A are one 128-bit load for 128 threads

  // ---- operand A: packed sub-kernel of the phase, [M][ld], one 128-bit load per thread and step
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(ph.packed, a.M * ph.ld * 4u);
  // Four threads write one 64-byte piece of a row to LDS (128-bit each); the LDS takes eight lanes per cycle, i.e. two
  // rows, and rows of 80 bytes that are r and r+4 apart fill the 32 banks exactly (r and r+1 would share four banks).
  const uint32_t a_oct = (uint32_t)tid / 8u, a_row = (a_oct / 4u) * 8u + (a_oct % 4u) + 4u * (((uint32_t)tid % 8u) / 4u), a_k = ((uint32_t)tid % 4u) * E;
  const uint32_t a_voff = ((m0 + a_row) * ph.ld + a_k) * 4u;  // M is a multiple of the block's rows; the next 64 rows are 64*ld further
  // ---- operand B: the thread's column (pixel p of sample s of the group) and its E consecutive k (channel, tap)
  // (with 128 columns a thread's two sets are k = b_k .. b_k+3 and b_k+8 .. b_k+11)
  const uint32_t b_col = (uint32_t)tid % BN, b_k = (uint32_t)__builtin_amdgcn_readfirstlane((tid / BN) * E);
  constexpr uint32_t B_SET = (THREADS / BN) * E;
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc(a.delta, a.batch * a.C * HW * 4u);
  __amdgpu_buffer_rsrc_t s_rsrc = b_rsrc;
  if (NORM) s_rsrc = make_rsrc(a.scale_shift, a.C * HW * 8u);
  uint32_t b_voff[NB][E], sample_bytes;  // (the offsets of the pairs follow from b_voff: twice the offset inside the sample)
  uint32_t sstep;
  {
    const uint32_t qhw = ph.qh * ph.qw, n = qt * BN + b_col;
    const uint32_t q = a.flat ? n % qhw : qt * (px_mask + 1u) + (b_col & px_mask);
    const uint32_t qy = q / ph.qw, qx = q % ph.qw;
    const uint32_t sample = a.flat ? n / qhw : g * a.per * sp + (b_col >> a.px_log);
    const uint32_t tx_cnt = (uint32_t)ph.taps_x, taps = (uint32_t)(ph.taps_y * ph.taps_x);  // taps divides BK: powers of two
    const int lt = __builtin_ctz(taps), lx = __builtin_ctz(tx_cnt);
    const bool col_ok = q < ph.qh * ph.qw && sample < a.batch;
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
      for (int i = 0; i < E; i++) {
        const uint32_t kk = b_k + (uint32_t)j * B_SET + i, cc = kk >> lt, t = kk & (taps - 1u), ty = t >> lx, tx = t & (tx_cnt - 1u);
        const int32_t iy = (int32_t)(qy * a.in_sy) + ph.offy + (int32_t)ty, ix = (int32_t)(qx * a.in_sx) + ph.offx + (int32_t)tx;
        const bool ok = col_ok && (uint32_t)iy < a.H && (uint32_t)ix < a.W;
        const uint32_t pixel = (cc * a.H + (uint32_t)iy) * a.W + (uint32_t)ix;
        b_voff[j][i] = ok ? (sample * a.C * HW + pixel) * 4u : OOB;
      }
    sample_bytes = sample * a.C * HW * 4u;
    sstep = (BK / taps) * HW * 4u;
  }
  const uint32_t group_step = sp * a.C * HW * 4u, nk = a.nk;
  const uint32_t a_first = ks * nk * BK * 4u;  // the block's share of the k steps starts here
  uint32_t a_soff = a_first, b_soff = ks * nk * sstep, ctile = 0;
  auto advance = [&]() {  // scalar unit only
    ctile++;
    a_soff += BK * 4u; b_soff += sstep;
    if (ctile == nk) { ctile = 0; a_soff = a_first; b_soff += group_step - nk * sstep; }
  };

  // Register sets: A and B are loaded two steps before they are written to LDS (two sets, tile t+3 requested while
  // tile t is multiplied).  The (scale, shift) pairs come from the L2 cache and are requested one step ahead into a
  // single set -- in front of the A and B loads of the same step, so that waiting for them leaves those in flight.
  float ra[2][TM][E], rb[2][NB][E];
  floatx2 rs[NORM ? E : 1];
  const uint32_t s_first = 2u * ks * nk * sstep;
  uint32_t s_next = s_first;  // scalar offset of the pairs of the tile that is written to LDS next
  auto load_pairs = [&]() {
    if constexpr (NORM) {
#pragma unroll
      for (int i = 0; i < E; i++) rs[i] = buf_load2(s_rsrc, b_voff[0][i] == OOB ? OOB : (b_voff[0][i] - sample_bytes) * 2u, s_next);
      s_next += 2u * sstep;
      if (s_next == s_first + 2u * sstep * nk) s_next = s_first;
    }
  };
  auto load_tile = [&](int set, bool adv) {
    if (adv) advance();
    __builtin_amdgcn_sched_barrier(0);
    if (a_loader) {
#pragma unroll
      for (int i = 0; i < TM; i++) {
        const floatx4 t = buf_load4(a_rsrc, a_voff + (uint32_t)i * 64u * ph.ld * 4u, a_soff);
        ra[set][i][0] = t.x; ra[set][i][1] = t.y; ra[set][i][2] = t.z; ra[set][i][3] = t.w;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < NB; j++)
#pragma unroll
      for (int i = 0; i < E; i++) rb[set][j][i] = buf_load(b_rsrc, b_voff[j][i], b_soff);
    __builtin_amdgcn_sched_barrier(0);
  };
  float *a_put = As + a_row * LDK + a_k, *b_put = Bs + b_col * LDK + b_k;
  const int in_func = a.in_func;
  auto put_tile = [&](int set, int buf) {
    if (a_loader) {
#pragma unroll
      for (int i = 0; i < TM; i++) lds_put<E>(a_put + buf * BM * LDK + i * 64 * LDK, ra[set][i]);
    }
    if constexpr (NORM) {
      float v[E];
#pragma unroll
      for (int i = 0; i < E; i++) {
        const float u = rs[i].x * rb[set][0][i] + rs[i].y;
        v[i] = NORM == 1 ? (u > 0.f ? u : 0.f) : apply_func_cheap(in_func, u);
      }
      lds_put<E>(b_put + buf * BN * LDK, v);
    } else {
#pragma unroll
      for (int j = 0; j < NB; j++) lds_put<E>(b_put + buf * BN * LDK + j * (int)B_SET, rb[set][j]);
    }
  };

  const int lrow = lane & 31, lk = lane >> 5;
  const float *a_get = As + (wm * TM * 32 + lrow) * LDK + lk * 4;
  const float *b_get = Bs + (wn * 32 + lrow) * LDK + lk * 4;
  floatx16 acc[TM];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  float4 fa[2][TM], fb[2];
  auto read_half = [&](float4 (&av)[TM], float4 &bv, int buf, int half) {
#pragma unroll
    for (int i = 0; i < TM; i++) av[i] = *reinterpret_cast<const float4 *>(a_get + buf * BM * LDK + i * 32 * LDK + half * 8);
    bv = *reinterpret_cast<const float4 *>(b_get + buf * BN * LDK + half * 8);
  };
  auto multiply = [&](const float4 (&av)[TM], const float4 &bv) {
#pragma unroll
    for (int c = 0; c < 4; c++)  // consecutive matrix instructions go to different accumulators
#pragma unroll
      for (int i = 0; i < TM; i++) {
        const float x = c == 0 ? av[i].x : c == 1 ? av[i].y : c == 2 ? av[i].z : av[i].w;
        const float y = c == 0 ? bv.x : c == 1 ? bv.y : c == 2 ? bv.z : bv.w;
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, acc[i], 0, 0, 0);
      }
  };
  auto step = [&](auto parity, auto write_next, auto load_ahead, auto pairs_ahead) {
    constexpr int cur = decltype(parity)::value, nxt = cur ^ 1;
    read_half(fa[1], fb[1], cur, 1);
    if constexpr (decltype(write_next)::value) {
      put_tile(nxt, nxt);
      if constexpr (decltype(pairs_ahead)::value) load_pairs();  // the pairs of tile t+2, wanted by the next step
    }
    if constexpr (decltype(load_ahead)::value) load_tile(nxt, true);
    __builtin_amdgcn_sched_barrier(0);
    multiply(fa[0], fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    if constexpr (decltype(write_next)::value) read_half(fa[0], fb[0], nxt, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(fa[1], fb[1]);
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- the lane's column of C: pixel and sample of the first group; register r is row m_lane + 8*(r/4) + r%4
  const uint32_t c_col = (uint32_t)(wn * 32 + lrow);
  const uint32_t c_n = qt * BN + c_col, c_qhw = ph.qh * ph.qw;
  const uint32_t c_q = a.flat ? c_n % c_qhw : qt * (px_mask + 1u) + (c_col & px_mask);
  const uint32_t c_sample = a.flat ? c_n / c_qhw : g * a.per * sp + (c_col >> a.px_log);
  const uint32_t c_qy = c_q / ph.qw, c_qx = c_q % ph.qw;
  const uint32_t pix = (c_qy * a.sy + ph.py) * a.OW + c_qx * a.sx + ph.px;
  const uint32_t m_lane = m0 + (uint32_t)(wm * TM * 32 + 4 * lk);  // whole blocks of rows and whole pixel tiles: no row or column tests
  float rbias[ROWBIAS ? 16 * TM : 1];
  if constexpr (ROWBIAS) {
#pragma unroll
    for (int r = 0; r < 16 * TM; r++) rbias[r] = a.row_bias[m_lane + 32u * (r / 16) + 8u * ((r % 16) / 4) + (r & 3)];
  }
  float extra = 0.f;
  if (a.tap_bias) {  // the CPU path adds the bias of every filter once per contributing tap
    int ny = 0, nx = 0;
    for (int t = 0; t < ph.taps_y; t++) ny += (uint32_t)((int32_t)c_qy + ph.offy + t) < a.H;
    for (int t = 0; t < ph.taps_x; t++) nx += (uint32_t)((int32_t)c_qx + ph.offx + t) < a.W;
    extra = a.tap_bias[0] * (float)(ny * nx);
  }
  // element offsets fit 32 bits (the output is addressed like the input: less than 2 GiB)
  uint32_t dst = c_sample < a.batch ? (c_sample * a.M + m_lane) * a.OHW + pix : OOB / 4u;  // (columns past the batch: only in a ragged flat tile)
  const uint32_t dst_step = sp * a.M * a.OHW;
  const int func = a.func;
  constexpr int NS = STATS ? 16 * TM : 1;
  float w_mean[NS], w_m2[NS];
  if constexpr (STATS) {
#pragma unroll
    for (int r = 0; r < NS; r++) { w_mean[r] = 0.f; w_m2[r] = 0.f; }
  }
  uint32_t seen = 0;  // groups finished
  // The output is addressed like the input, through a buffer descriptor (less than 2 GiB): the lane's first element as
  // a 32-bit byte offset, the row of register r as a scalar offset -- no 64-bit address arithmetic per store, and one
  // look at the output function for all sixteen values instead of a chain of branches per value.
  const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(a.out + (size_t)ks * a.split_stride, a.batch * a.M * a.OHW * 4u);
  const uint32_t row_bytes = a.OHW * 4u;
  auto flush = [&]() {
    seen++;
    const float inv_seen = 1.0f / (float)seen;
    float v[16 * TM];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) v[16 * i + r] = ROWBIAS ? acc[i][r] + rbias[16 * i + r] : acc[i][r] + extra;
    if constexpr (STATS) {
#pragma unroll
      for (int e = 0; e < 16 * TM; e++) {
        const float d = v[e] - w_mean[e];
        w_mean[e] = w_mean[e] + d * inv_seen;
        w_m2[e] = w_m2[e] + d * (v[e] - w_mean[e]);
      }
    } else {
      apply_func_cheap_many<16 * TM>(func, v);
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const uint32_t dm = 32u * i + 8u * (r / 4) + (r & 3);
        buf_store(o_rsrc, v[16 * i + r], dst * 4u, dm * row_bytes);
        acc[i][r] = 0.f;
      }
    dst += dst_step;
  };

  // ---- the walk: per * nk steps as one software pipeline (see igemm_body for the pipeline itself)
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;
  load_pairs();              // pairs of tile 0
  load_tile(0, false);
  put_tile(0, 0);
  load_pairs();              // pairs of tile 1
  load_tile(1, true);
  load_tile(0, true);
  lds_barrier();
  read_half(fa[0], fb[0], 0, 0);
  uint32_t left = a.per * nk, kleft = nk;  // nk is even and at least 4, so the last four steps belong to the last group
  // The blocks that share a compute unit (one wavefront each per SIMD) do the same work, but a SIMD serves the oldest
  // ready wavefront first: left alone, one block runs ahead and finishes early (the first after less than half of the
  // kernel's time), and the last ones multiply with ever fewer neighbours to cover their waits.  A wavefront therefore
  // lowers its own priority as its work shrinks -- four levels, at 1/2, 1/4 and 1/8 of its steps left -- so whoever is
  // behind is served first and the blocks of a compute unit stay together to the end (they also ask for the same
  // weights at the same time).
  uint32_t lower2 = 0, lower1 = 0, lower0 = 0;   // steps left at which the priority drops to 2, 1, 0 (even numbers)
  if (a.fair) { lower2 = (left * ((a.fair >> 8) & 15u) / 16u) & ~1u; lower1 = (left * ((a.fair >> 4) & 15u) / 16u) & ~1u; lower0 = (left * (a.fair & 15u) / 16u) & ~1u; }
  if (a.fair) __builtin_amdgcn_s_setprio(3);
  for (; left > 4; left -= 2) {
    if (a.fair) {
      if (left == lower2) __builtin_amdgcn_s_setprio(2);
      else if (left == lower1) __builtin_amdgcn_s_setprio(1);
      else if (left == lower0) __builtin_amdgcn_s_setprio(0);
    }
    step(Even{}, Yes{}, Yes{}, Yes{});
    step(Odd{}, Yes{}, Yes{}, Yes{});
    kleft -= 2;
    if (kleft == 0) { flush(); kleft = nk; }
  }
  step(Even{}, Yes{}, Yes{}, Yes{});   // writes tile left-3, requests the pairs of tile left-2
  step(Odd{}, Yes{}, No{}, Yes{});     // writes tile left-2, requests the pairs of the last tile
  step(Even{}, Yes{}, No{}, No{});     // writes the last tile
  step(Odd{}, No{}, No{}, No{});
  flush();

  if constexpr (STATS) {
    // samples of the tile that sit in one wavefront's 32 columns: lanes that differ in the bits at and above px_log
    float half_n = 0.5f * (float)a.per;  // half of the samples each side of a merge holds
    for (uint32_t bit = px_mask + 1u; bit < 32u; bit <<= 1) {
#pragma unroll
      for (int r = 0; r < NS; r++) {
        const float om = __shfl_xor(w_mean[r], (int)bit, 64), o2 = __shfl_xor(w_m2[r], (int)bit, 64);
        welford_merge_equal(w_mean[r], w_m2[r], om, o2, half_n);
      }
      half_n *= 2.f;
    }
    const bool across = a.px_log <= 5;  // both wavefronts along the columns hold the same pixels (other samples)
    if (across) {
      // no wavefront reads operand tiles any more: every LDS read of the last step came before its barrier
      float *xch = smem + (wm * 64 + lane) * (NS + 1);  // 2 x 64 x (NS + 1) floats, used twice: within the tiles' memory
      static_assert(2 * 64 * (NS + 1) <= 2 * (BM + BN) * LDK, "the exchange fits into the tiles' memory");
      float other_mean[NS];
      if (wn == 1) {
#pragma unroll
        for (int r = 0; r < NS; r++) xch[r] = w_mean[r];
      }
      __syncthreads();
      if (wn == 0) {
#pragma unroll
        for (int r = 0; r < NS; r++) other_mean[r] = xch[r];
      }
      __syncthreads();
      if (wn == 1) {
#pragma unroll
        for (int r = 0; r < NS; r++) xch[r] = w_m2[r];
      }
      __syncthreads();
      if (wn == 0) {
#pragma unroll
        for (int r = 0; r < NS; r++) welford_merge_equal(w_mean[r], w_m2[r], other_mean[r], xch[r], half_n);
      }
    }
    const uint32_t keep = px_mask + 1u < 32u ? px_mask + 1u : 32u;  // lanes that hold distinct pixels
    if ((!across || wn == 0) && (uint32_t)lrow < keep) {
      const size_t S = (size_t)a.M * a.OHW;
      float *pm = a.part_mean + (size_t)g * S + (size_t)m_lane * a.OHW + pix, *p2 = a.part_m2 + (size_t)g * S + (size_t)m_lane * a.OHW + pix;
#pragma unroll
      for (int r = 0; r < NS; r++) {
        const uint32_t dm = 32u * (r / 16) + 8u * ((r % 16) / 4) + (r & 3);
        pm[(size_t)dm * a.OHW] = w_mean[r];
        p2[(size_t)dm * a.OHW] = w_m2[r];
      }
    }
  }
}

// ---- batch-summed weight gradient on the same pipeline ----------------------------------------------------------------
//   dK[f][(c,i,j)] = sum over (w, oy, ox) of delta[w][f][oy][ox] * image[w][c][oy*sy + i - py][ox*sx + j - px]
// as one product per group of k steps: rows = filters (operand A: rows of delta, 16 consecutive pixels per k step, one
// 128-bit load per thread), columns = kernel coefficients (c, i, j) (operand B: a gather from the image whose per-thread
// byte offsets never change: a k step is a block of 16 output pixels -- whole output rows, 16 / OW of them, or a 16-pixel
// piece of one row -- so the pixels keep their place inside the block and a step moves a scalar offset), k = (sample,
// output pixel).  A block owns one 64 x 64 tile of dK for its group -- whole samples, or an equal share of one sample's
// steps -- and runs it as ONE k loop; the groups' tiles are added afterwards in group order.
// Image borders: rows can only fall outside the image in the first row block of a sample (above it) and in the last one
// (below it), so a thread keeps one mask for each and a step ORs in the one that applies -- two vector instructions per
// step and one per load, against a bounds test per element in the general kernel.  Columns outside the image are out of
// range for good when a step covers whole rows (folded into the offsets); when a row takes several steps (WIDE) they can
// only occur in its first and last step, with a mask per element for each.
struct WgradWalkArgs {
  const float *delta;   // [B][M][OH][OW]
  const float *image;   // [B][C][H][W]
  float *partial;       // [groups][M][N]
  float *bias_partial;  // [groups][M]: the groups' sums of delta per filter (the bias gradient), or null
  uint32_t M, N, C, H, W, OH, OW, KY, KX;
  int32_t sy, sx, py, px;
  uint32_t steps, groups, tiles_m, tiles_n, fair;   // steps: k steps of a group (of B * OH * OW / 16 in all)
};

template <bool WIDE, int WAVES>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(WAVES, WAVES))) void wgrad_walk_kernel(WgradWalkArgs a) {
  constexpr int BM = 64, BN = 64, E = 4;
  __shared__ float4 smem4[2 * (BM + BN) * LDK / 4];
  float *smem = reinterpret_cast<float *>(smem4);
  float *As = smem, *Bs = smem + 2 * BM * LDK;

  // an XCD runs a contiguous range of logical blocks: a few groups (their slices of delta and of the image) per range
  uint32_t j = xcd_swizzle(blockIdx.x, gridDim.x);
  const uint32_t mt = j % a.tiles_m; j /= a.tiles_m;
  const uint32_t nt = j % a.tiles_n, g = j / a.tiles_n;
  const uint32_t m0 = mt * BM, n0 = nt * BN, DHW = a.OH * a.OW, HW = a.H * a.W;
  // a sample is yblocks row blocks of xsteps k steps each
  const uint32_t rows_per_step = WIDE ? 1u : BK / a.OW, xsteps = WIDE ? a.OW / BK : 1u, yblocks = a.OH / rows_per_step, nb = yblocks * xsteps;
  const uint32_t first = g * a.steps, sample0 = first / nb, rem = first % nb;   // the group's first step: sample and step inside it
  const uint32_t samples = (rem + a.steps + nb - 1) / nb;                        // samples the group touches (1 when it is a share of one)

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // ---- operand A: delta[w][m0 + row][16 pixels of the step], four pixels per thread
  const uint32_t a_oct = (uint32_t)tid / 8u, a_row = (a_oct / 4u) * 8u + (a_oct % 4u) + 4u * (((uint32_t)tid % 8u) / 4u), a_k = ((uint32_t)tid % 4u) * E;
  const __amdgpu_buffer_rsrc_t a_rsrc = make_rsrc(a.delta + (size_t)sample0 * a.M * DHW, samples * a.M * DHW * 4u);
  const uint32_t a_voff = ((m0 + a_row) * DHW + a_k) * 4u;
  // ---- operand B: column n = (c, i, j), pixels b_k .. b_k + 3 of the step's block
  const uint32_t b_col = (uint32_t)tid % BN, b_k = (uint32_t)__builtin_amdgcn_readfirstlane((tid / BN) * E);
  const uint32_t front = (uint32_t)a.py * a.W + (uint32_t)a.px;   // offsets are taken from (py rows + px pixels) in front of the image: none is negative
  const __amdgpu_buffer_rsrc_t b_rsrc = make_rsrc(a.image + (size_t)sample0 * a.C * HW - front, (samples * a.C * HW + front) * 4u);
  uint32_t b_voff[E], m_top, m_bottom, m_left[WIDE ? E : 1], m_right[WIDE ? E : 1];
  {
    const uint32_t n = n0 + b_col, taps = a.KY * a.KX, c = n / taps, t = n % taps, ki = t / a.KX, kj = t % a.KX;
    const uint32_t dy = WIDE ? 0u : b_k / a.OW, dx0 = WIDE ? b_k : b_k % a.OW;   // the four pixels are neighbours in one output row (OW is a multiple of 4)
    const int32_t iy_first = (int32_t)(dy * a.sy + ki) - a.py;                                  // input row in the first row block of a sample
    const int32_t iy_last = (int32_t)((a.OH - rows_per_step + dy) * a.sy + ki) - a.py;          // ... and in the last one
    m_top = iy_first < 0 ? OOB : 0u;
    m_bottom = iy_last >= (int32_t)a.H ? OOB : 0u;
#pragma unroll
    for (int e = 0; e < E; e++) {
      const int32_t ix = (int32_t)((dx0 + e) * a.sx + kj) - a.px;   // input column in the first step of a row
      bool ok = n < a.N;
      if constexpr (WIDE) {
        m_left[e] = ix < 0 ? OOB : 0u;
        m_right[e] = ix + (int32_t)((a.OW - BK) * a.sx) >= (int32_t)a.W ? OOB : 0u;
      } else {
        ok = ok && (uint32_t)ix < a.W;
      }
      b_voff[e] = ok ? ((c * a.H + dy * a.sy + ki) * a.W + (dx0 + e) * a.sx + kj) * 4u : OOB;
    }
  }
  const uint32_t a_sample = (a.M * DHW - DHW) * 4u;
  const uint32_t x_bytes = WIDE ? BK * (uint32_t)a.sx * 4u : 0u;                                  // a step along a row
  const uint32_t y_bytes = rows_per_step * (uint32_t)a.sy * a.W * 4u, y_jump = y_bytes - xsteps * x_bytes;   // to the next row block
  const uint32_t b_sample = (a.C * HW) * 4u - yblocks * y_bytes;
  uint32_t yb = rem / xsteps, xb = rem % xsteps;   // the step's row block inside its sample, its place in the row
  uint32_t a_soff = rem * BK * 4u, b_soff = yb * y_bytes + xb * x_bytes;
  auto edges = [&]() { return (yb == 0 ? 1u : 0u) | (yb == yblocks - 1 ? 2u : 0u) | (xb == 0 ? 4u : 0u) | (xb == xsteps - 1 ? 8u : 0u); };
  uint32_t edge = edges();
  auto advance = [&]() {  // scalar unit only
    a_soff += BK * 4u;
    if constexpr (WIDE) { b_soff += x_bytes; xb++; }
    if (!WIDE || xb == xsteps) {
      xb = 0; yb++; b_soff += y_jump;
      if (yb == yblocks) { yb = 0; a_soff += a_sample; b_soff += b_sample; }
    }
    edge = edges();
  };
  float ra[2][E], rb[2][E];
  auto load_tile = [&](int set, bool adv) {
    if (adv) advance();
    const uint32_t top = edge & 1u ? ~0u : 0u, bottom = edge & 2u ? ~0u : 0u;   // (scalar selects)
    const uint32_t mask = (m_top & top) | (m_bottom & bottom);
    __builtin_amdgcn_sched_barrier(0);
    {
      const floatx4 t = buf_load4(a_rsrc, a_voff, a_soff);
      ra[set][0] = t.x; ra[set][1] = t.y; ra[set][2] = t.z; ra[set][3] = t.w;
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (WIDE) {
      const uint32_t left = edge & 4u ? ~0u : 0u, right = edge & 8u ? ~0u : 0u;
#pragma unroll
      for (int i = 0; i < E; i++) rb[set][i] = buf_load(b_rsrc, b_voff[i] | mask | (m_left[i] & left) | (m_right[i] & right), b_soff);
    } else {
#pragma unroll
      for (int i = 0; i < E; i++) rb[set][i] = buf_load(b_rsrc, b_voff[i] | mask, b_soff);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  float *a_put = As + a_row * LDK + a_k, *b_put = Bs + b_col * LDK + b_k;
  // the bias gradient is the sum of delta over samples and pixels: the row sums of operand A, which the blocks of the
  // first column tile add up as the tiles pass through their registers
  const bool row_sums = a.bias_partial != nullptr && nt == 0;
  float row_sum = 0.f;
  auto put_tile = [&](int set, int buf) {
    lds_put<E>(a_put + buf * BM * LDK, ra[set]);
    lds_put<E>(b_put + buf * BN * LDK, rb[set]);
    if (row_sums) row_sum += (ra[set][0] + ra[set][1]) + (ra[set][2] + ra[set][3]);
  };
  const int lrow = lane & 31, lk = lane >> 5;
  const float *a_get = As + (wm * 32 + lrow) * LDK + lk * 4;
  const float *b_get = Bs + (wn * 32 + lrow) * LDK + lk * 4;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  float4 fa[2], fb[2];
  auto read_half = [&](float4 &av, float4 &bv, int buf, int half) {
    av = *reinterpret_cast<const float4 *>(a_get + buf * BM * LDK + half * 8);
    bv = *reinterpret_cast<const float4 *>(b_get + buf * BN * LDK + half * 8);
  };
  auto multiply = [&](const float4 &av, const float4 &bv) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.x, bv.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.y, bv.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.z, bv.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av.w, bv.w, acc, 0, 0, 0);
  };
  auto step = [&](auto parity, auto write_next, auto load_ahead) {   // (the pipeline of igemm_body)
    constexpr int cur = decltype(parity)::value, nxt = cur ^ 1;
    read_half(fa[1], fb[1], cur, 1);
    if constexpr (decltype(write_next)::value) put_tile(nxt, nxt);
    if constexpr (decltype(load_ahead)::value) load_tile(nxt, true);
    __builtin_amdgcn_sched_barrier(0);
    multiply(fa[0], fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    if constexpr (decltype(write_next)::value) read_half(fa[0], fb[0], nxt, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(fa[1], fb[1]);
    __builtin_amdgcn_sched_barrier(0);
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;
  load_tile(0, false);
  put_tile(0, 0);
  load_tile(1, true);
  load_tile(0, true);
  lds_barrier();
  read_half(fa[0], fb[0], 0, 0);
  uint32_t left = a.steps;   // even and at least 4 (checked on the host)
  uint32_t lower2 = 0, lower1 = 0, lower0 = 0;   // wavefront priorities that fall with the work left (see tconv_walk_kernel)
  if (a.fair) { lower2 = (left * ((a.fair >> 8) & 15u) / 16u) & ~1u; lower1 = (left * ((a.fair >> 4) & 15u) / 16u) & ~1u; lower0 = (left * (a.fair & 15u) / 16u) & ~1u; }
  if (a.fair) __builtin_amdgcn_s_setprio(3);
  for (; left > 4; left -= 2) {
    if (a.fair) {
      if (left == lower2) __builtin_amdgcn_s_setprio(2);
      else if (left == lower1) __builtin_amdgcn_s_setprio(1);
      else if (left == lower0) __builtin_amdgcn_s_setprio(0);
    }
    step(Even{}, Yes{}, Yes{});
    step(Odd{}, Yes{}, Yes{});
  }
  step(Even{}, Yes{}, Yes{});
  step(Odd{}, Yes{}, No{});
  step(Even{}, Yes{}, No{});
  step(Odd{}, No{}, No{});
  // the group's tile: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the wavefront's 32 x 32 quarter
  const uint32_t n = n0 + (uint32_t)(wn * 32 + lrow), m_lane = m0 + (uint32_t)(wm * 32 + 4 * lk);
  const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(a.partial, a.groups * a.M * a.N * 4u);
  const uint32_t dst = n < a.N ? ((g * a.M + m_lane) * a.N + n) * 4u : OOB, row_bytes = a.N * 4u;
#pragma unroll
  for (int r = 0; r < 16; r++) buf_store(o_rsrc, acc[r], dst, (8u * (r / 4) + (r & 3)) * row_bytes);
  if (row_sums) {  // four neighbouring lanes hold the four quarters of a row's k steps
    row_sum += __shfl_xor(row_sum, 1, 64);
    row_sum += __shfl_xor(row_sum, 2, 64);
    if ((tid & 3) == 0) a.bias_partial[(size_t)g * a.M + (m0 + a_row)] = row_sum;
  }
}

// Chan's update: (n, mean, m2) takes in another set of samples given the same way
__device__ __forceinline__ void welford_merge(float &n, float &mean, float &m2, float on, float om, float o2) {
  if (on == 0.f) return;
  if (n == 0.f) { n = on; mean = om; m2 = o2; return; }
  const float total = n + on, d = om - mean, w = __frcp_rn(total);
  mean = mean + d * (on * w);
  m2 = (m2 + o2) + (d * d) * (n * on * w);
  n = total;
}

// Combines the per-block (mean, M2) pairs of one element in a fixed order (every block holds n_block samples) and turns
// them into what the consumer of the normalised tensor needs:
//   mean, biased variance, ivar = 1/sqrt(var + eps);  scale = gamma * ivar,  shift = beta - mean * scale
// scale_shift is [S][2]; the other outputs are optional.  A block finishes 64 elements: thread (element, quarter) merges
// the blocks quarter, quarter + 4, ... with eight loads in flight, then the four quarters are merged in order.
__global__ __launch_bounds__(256) void bn_finish_kernel(float *scale_shift, float *mean_out, float *var_out, float *ivar_out, float *new_mean, float *new_var,
                                                        const float *part_mean, const float *part_m2, uint32_t blocks, float n_block, uint32_t S,
                                                        const float *gamma, const float *beta, float eps, float mom_old, float mom_new) {
  __shared__ float xn[3][64], xm[3][64], x2[3][64];
  const uint32_t el = threadIdx.x % 64, quarter = threadIdx.x / 64, e = blockIdx.x * 64 + el;
  float n = 0.f, mean = 0.f, m2 = 0.f;
  if (e < S) {
    uint32_t b = quarter;
    for (; b + 12 < blocks; b += 16) {
      float om[4], o2[4];
#pragma unroll
      for (int i = 0; i < 4; i++) { om[i] = part_mean[(size_t)(b + 4 * i) * S + e]; o2[i] = part_m2[(size_t)(b + 4 * i) * S + e]; }
#pragma unroll
      for (int i = 0; i < 4; i++) welford_merge(n, mean, m2, n_block, om[i], o2[i]);
    }
    for (; b < blocks; b += 4) welford_merge(n, mean, m2, n_block, part_mean[(size_t)b * S + e], part_m2[(size_t)b * S + e]);
  }
  if (quarter) { xn[quarter - 1][el] = n; xm[quarter - 1][el] = mean; x2[quarter - 1][el] = m2; }
  __syncthreads();
  if (quarter || e >= S) return;
#pragma unroll
  for (int q = 0; q < 3; q++) welford_merge(n, mean, m2, xn[q][el], xm[q][el], x2[q][el]);
  float var = m2 / n;
  if (var < 0.f) var = 0.f;
  const float ivar = (float)(1.0 / (double)sqrtf(var + eps));
  const float scale = gamma[e] * ivar;
  reinterpret_cast<float2 *>(scale_shift)[e] = make_float2(scale, beta[e] - mean * scale);
  if (mean_out) mean_out[e] = mean;
  if (var_out) var_out[e] = var;
  if (ivar_out) ivar_out[e] = ivar;
  if (new_mean) new_mean[e] = (mom_old * new_mean[e]) + (mom_new * mean);
  if (new_var) new_var[e] = (mom_old * new_var[e]) + (mom_new * var);
}

int &walk_order();    // -1 choose per layer (default), 0 batch groups first, 1 row tiles first (measurements only)
int &walk_fair();     // 0x842 (default): wavefronts lower their priority at 8/16, 4/16, 2/16 of their steps left; 0: no priorities (measurements only)
// What every use of tconv_walk_kernel needs of the phases and the sizes.
inline bool tconv_walk_fits(const WalkArgs &a, uint32_t tm) {
  if (a.nphase == 0 || a.M == 0 || a.batch == 0) return false;
  const TconvPhase &p0 = a.ph[0];
  const uint32_t qhw = p0.qh * p0.qw;
  for (uint32_t f = 0; f < a.nphase; f++) {
    const TconvPhase &ph = a.ph[f];
    const uint32_t taps = (uint32_t)(ph.taps_y * ph.taps_x);
    if (ph.qh * ph.qw != qhw || ph.kp != p0.kp || taps == 0 || BK % taps != 0 || (taps & (taps - 1)) != 0 || (ph.taps_x & (ph.taps_x - 1)) != 0) return false;
    if (a.C % (BK / taps) != 0 || ph.ld < ph.kp || ph.ld % 4 != 0) return false;
  }
  if (p0.kp % (2 * BK) != 0 || p0.kp < 4 * BK || a.M % (a.wide ? 32 : 64 * tm) != 0 || (a.wide && tm != 1)) return false;
  return (uint64_t)a.batch * a.M * a.OHW * 4u < 0x80000000ull && (uint64_t)a.batch * a.C * a.H * a.W * 4u < 0x80000000ull;
}
// Whether (and how) a transposed convolution can walk: fills px_log, qtiles, groups, per, nk.
inline bool tconv_walk_plan(WalkArgs &a, uint32_t want_blocks, uint32_t tm) {
  if (!tconv_walk_fits(a, tm)) return false;
  const TconvPhase &p0 = a.ph[0];
  const uint32_t qhw = p0.qh * p0.qw;
  a.flat = 0;
  a.nk = p0.kp / BK;
  // pixels per tile: 16 (four samples per tile: two per wavefront, merged by a lane shuffle), else 32 or 64; twice
  // that for the blocks of 128 columns
  const uint32_t cols = a.wide ? 128u : 64u, lo = a.wide ? 5u : 4u;
  uint32_t px_log = 0;
  for (uint32_t cand = lo; cand < lo + 3u; cand++)
    if (qhw % (1u << cand) == 0 && a.batch % (cols >> cand) == 0) { px_log = cand; break; }
  if (px_log == 0) return false;
  a.px_log = px_log;
  a.qtiles = qhw >> px_log;
  const uint32_t sp = cols >> px_log, sample_groups = a.batch / sp;
  a.tiles_m = a.M / (a.wide ? 32 : 64 * tm);
  const uint32_t base = a.nphase * a.tiles_m * a.qtiles;
  // batch groups: as many as give about want_blocks blocks, a divisor of the number of sample groups
  uint32_t groups = base >= want_blocks ? 1u : want_blocks / base;
  if (groups > sample_groups) groups = sample_groups;
  while (groups > 1 && sample_groups % groups) groups--;
  a.groups = groups;
  a.per = sample_groups / groups;
  // more packed weights than an XCD's L2 holds (4 MiB), and several row tiles to deal out
  a.fair = (uint32_t)walk_fair();
  a.ksplit = 1; a.split_stride = 0;
  a.weights_major = walk_order() >= 0 ? (uint32_t)walk_order() : ((uint64_t)a.nphase * a.M * p0.kp * 4u > (4u << 20) && a.tiles_m > 1 ? 1u : 0u);
  return (uint64_t)base * groups <= 0x7fffffffu;
}

// The same kernel without a walk, for any number of pixels per sample: tiles of 64 (sample, pixel) columns through the
// whole batch, every block one tile over all k steps (64-row blocks only, no statistics).
inline bool tconv_walk_plan_flat(WalkArgs &a) {
  if (!tconv_walk_fits(a, 1)) return false;
  const TconvPhase &p0 = a.ph[0];
  const uint64_t n = (uint64_t)a.batch * p0.qh * p0.qw;
  a.flat = 1;
  a.nk = p0.kp / BK;
  const uint32_t cols = a.wide ? 128u : 64u;
  a.px_log = a.wide ? 7 : 6; a.qtiles = (uint32_t)((n + cols - 1) / cols); a.groups = 1; a.per = 1;
  a.tiles_m = a.M / (a.wide ? 32 : 64);
  a.fair = (uint32_t)walk_fair();
  a.ksplit = 1; a.split_stride = 0;
  a.weights_major = walk_order() >= 0 ? (uint32_t)walk_order() : ((uint64_t)a.nphase * a.M * p0.kp * 4u > (4u << 20) && a.tiles_m > 1 ? 1u : 0u);
  return (uint64_t)a.nphase * a.tiles_m * a.qtiles <= 0x7fffffu;
}

int &walk_blocks();   // blocks wanted per launch (measurements only); default 1024, or 1280 for the plain variant
int &walk_waves();
int &walk_tm();       // 1 or 2 accumulators per wavefront (2 where the output channels allow; measurements only)    // 4 or 5 wavefronts per SIMD for the plain variant (measurements only)

inline int launch_tconv_walk(const char *name, const WalkArgs &a, bool norm, bool stats, uint32_t tm) {
  const uint32_t grid = a.nphase * a.tiles_m * a.qtiles * a.groups * a.ksplit;
  hipStream_t s = stream();
  const int n = !norm ? 0 : a.in_func == MT_F_RELU ? 1 : 2;
  if (a.flat && (stats || tm != 1 || a.per != 1 || a.groups != 1)) return fail(MT_E_ARGUMENT, "%s: flat column tiles do not walk and keep no statistics", name);
  if (a.ksplit > 1 && (stats || a.per != 1 || a.nk < 4 || a.nk % 2 != 0 || a.row_bias || a.tap_bias || a.func != MT_F_NONE))
    return fail(MT_E_ARGUMENT, "%s: blocks that share a tile's k steps write plain sums of one batch group", name);
  if (a.wide) {
    if (norm || stats || tm != 1) return fail(MT_E_ARGUMENT, "%s: blocks of 32 rows walk without batch-norm folding", name);
    if (a.row_bias) tconv_walk_kernel<0, false, 4, 1, true, true><<<grid, THREADS, 0, s>>>(a);
    else tconv_walk_kernel<0, false, 4, 1, false, true><<<grid, THREADS, 0, s>>>(a);
    MT_LAUNCH_CHECK(name);
    return MT_OK;
  }
  if (a.row_bias) {  // forward convolution: plain variant only
    if (norm || stats || tm != 1) return fail(MT_E_ARGUMENT, "%s: a forward convolution walks without batch-norm folding", name);
    tconv_walk_kernel<0, false, 4, 1, true><<<grid, THREADS, 0, s>>>(a);
    MT_LAUNCH_CHECK(name);
    return MT_OK;
  }
  if (tm == 2) {
    if (n == 1 && stats) tconv_walk_kernel<1, true, 2, 2><<<grid, THREADS, 0, s>>>(a);
    else if (n == 2 && stats) tconv_walk_kernel<2, true, 2, 2><<<grid, THREADS, 0, s>>>(a);
    else if (n == 1) tconv_walk_kernel<1, false, 3, 2><<<grid, THREADS, 0, s>>>(a);
    else if (n == 2) tconv_walk_kernel<2, false, 3, 2><<<grid, THREADS, 0, s>>>(a);
    else if (stats) tconv_walk_kernel<0, true, 3, 2><<<grid, THREADS, 0, s>>>(a);
    else tconv_walk_kernel<0, false, 4, 2><<<grid, THREADS, 0, s>>>(a);
  } else if (n == 1 && stats) tconv_walk_kernel<1, true, 4, 1><<<grid, THREADS, 0, s>>>(a);
  else if (n == 2 && stats) tconv_walk_kernel<2, true, 4, 1><<<grid, THREADS, 0, s>>>(a);
  else if (n == 1) tconv_walk_kernel<1, false, 4, 1><<<grid, THREADS, 0, s>>>(a);
  else if (n == 2) tconv_walk_kernel<2, false, 4, 1><<<grid, THREADS, 0, s>>>(a);
  else if (stats) tconv_walk_kernel<0, true, 4, 1><<<grid, THREADS, 0, s>>>(a);
  else if (walk_waves() == 5) tconv_walk_kernel<0, false, 5, 1><<<grid, THREADS, 0, s>>>(a);
  else tconv_walk_kernel<0, false, 4, 1><<<grid, THREADS, 0, s>>>(a);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

// Whether the batch-summed weight gradient can run as wgrad_walk_kernel, and with how many groups: `groups` comes in as
// the caller's choice (a divisor of the batch) and may go up to an equal share of one sample's steps per group when the
// batch alone gives too few blocks.  Fills steps, groups, tiles_m, tiles_n.
inline bool wgrad_walk_plan(WgradWalkArgs &a, uint32_t batch, bool may_split_samples) {
  if (a.groups == 0 || batch % a.groups != 0 || a.M % 64 != 0 || a.py < 0 || a.px < 0) return false;
  const bool wide = a.OW > (uint32_t)BK;
  if (wide ? a.OW % BK != 0 : (a.OW < 4 || BK % a.OW != 0 || a.OH % (BK / a.OW) != 0)) return false;   // a k step is whole output rows or a piece of one
  const uint32_t rows = wide ? 1u : BK / a.OW, yblocks = a.OH / rows, xsteps = wide ? a.OW / BK : 1u, nb = yblocks * xsteps;
  // rows above the image only in the first row block of a sample, rows below it only in the last one; columns left and
  // right of it only in the first and last step of a row
  for (uint32_t yb = 0; yb < yblocks; yb++)
    for (uint32_t dy = 0; dy < rows; dy++)
      for (uint32_t ki = 0; ki < a.KY; ki++) {
        const int64_t iy = (int64_t)(yb * rows + dy) * a.sy + ki - a.py;
        if (iy < 0 && yb != 0) return false;
        if (iy >= (int64_t)a.H && yb != yblocks - 1) return false;
      }
  if (wide)
    for (uint32_t xb = 0; xb < xsteps; xb++)
      for (uint32_t dx = 0; dx < (uint32_t)BK; dx++)
        for (uint32_t kj = 0; kj < a.KX; kj++) {
          const int64_t ix = (int64_t)(xb * BK + dx) * a.sx + kj - a.px;
          if (ix < 0 && xb != 0) return false;
          if (ix >= (int64_t)a.W && xb != xsteps - 1) return false;
        }
  a.tiles_m = a.M / 64;
  a.tiles_n = (a.N + 63) / 64;
  uint32_t steps = batch / a.groups * nb;
  if (may_split_samples && a.groups == batch)   // one sample per group and still few blocks: equal shares of a sample's steps
    while (steps % 2 == 0 && steps / 2 >= 16 && (uint64_t)a.tiles_m * a.tiles_n * a.groups < 512) { steps /= 2; a.groups *= 2; }
  if (may_split_samples && steps >= 48) {
    // The blocks come in rounds of one per compute unit: 576 blocks are three rounds, the last an eighth full.  More groups of
    // fewer steps each can fill the rounds (a group need not end with a sample); a group's first loads and its tile's way
    // out cost about eight steps' time.
    const uint64_t tiles = (uint64_t)a.tiles_m * a.tiles_n;
    auto cost = [&](uint64_t groups, uint32_t st) { return (double)((tiles * groups + 255) / 256) / (double)groups * (1.0 + 8.0 / (double)st); };
    double best = cost(a.groups, steps);
    uint32_t pick = 1;
    for (uint32_t m : {2u, 3u, 4u, 6u, 8u, 12u, 16u}) {
      if (steps % m != 0 || (steps / m) % 2 != 0 || steps / m < 24) continue;
      if ((uint64_t)a.groups * m * a.M * a.N > ((uint64_t)1 << 26)) continue;   // (the groups' tiles: at most 256 MB)
      const double c = cost((uint64_t)a.groups * m, steps / m);
      if (c < 0.97 * best) { best = c; pick = m; }
    }
    steps /= pick; a.groups *= pick;
  }
  if (a.groups < 2 || steps < 4 || steps % 2 != 0) return false;
  a.steps = steps;
  const uint64_t samples = (steps + nb - 1) / nb, front = (uint64_t)a.py * a.W + a.px;
  if (samples * a.M * a.OH * a.OW * 4u >= 0x80000000ull || (samples * a.C * a.H * a.W + front + (uint64_t)a.KY * a.W) * 4u >= 0x80000000ull ||
      (uint64_t)a.groups * a.M * a.N * 4u >= 0x80000000ull)
    return false;
  if (((uintptr_t)a.delta & 15u) != 0) return false;
  a.fair = (uint32_t)walk_fair();
  return (uint64_t)a.tiles_m * a.tiles_n * a.groups <= 0x7fffffffu;
}

inline int launch_wgrad_walk(const char *name, const WgradWalkArgs &a) {
  const uint32_t grid = a.tiles_m * a.tiles_n * a.groups;
  if (a.OW > (uint32_t)BK) wgrad_walk_kernel<true, 4><<<grid, THREADS, 0, stream()>>>(a);
  else wgrad_walk_kernel<false, 4><<<grid, THREADS, 0, stream()>>>(a);
  MT_LAUNCH_CHECK(name);
  return MT_OK;
}

}  // namespace igemm
}  // namespace mt
