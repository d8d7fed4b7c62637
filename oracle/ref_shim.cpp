// TEST INFRASTRUCTURE ONLY.
//
// Thin C wrapper that exposes the reference's own CPU tensor classes, compiled
// from the headers where they lie under /root/reference, through the flat API of
// tensor_oracle.h.  It exists to (1) pin the C restatement bit-for-bit and
// (2) serve as the "reference" CPU baseline.  It is built only where
// /root/reference is present, into oracle/_ref/ (not tracked by git); no
// reference source is copied into this repository.
//
// The reference headers rely on transitive includes, so the standard headers
// come first; its two console helpers come from the reference's own
// system/system.cpp, which oracle/Makefile compiles beside this file.
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <math.h>
#include <string>
#include <vector>
#include <algorithm>

#include "cpu/tensor.h"   // resolved with -I/root/reference

#include "tensor_oracle.h"

namespace
{
const int REF_THROW = 100;  // any precondition `throw` of the reference

typedef CTensor<float> T;

T load(const ot_tensor *t)
{
 T c(t->w, t->z, t->y, t->x);
 uint32_t n = t->w * t->z * t->y * t->x;
 if (n) c.CopyItemToHost(t->p, n);
 return c;
}
void store(ot_tensor *t, T &c)
{
 uint32_t n = t->w * t->z * t->y * t->x;
 if (n) memcpy(t->p, c.GetColumnPtr(0, 0, 0), n * sizeof(float));
}
}  // namespace

#define GUARD(BODY) try { BODY } catch (const char *) { return REF_THROW; } return 0;

extern "C" {

int oracle_forward_convolution(ot_tensor *out, const ot_tensor *image, const ot_tensor *kernel, int32_t kx, int32_t ky,
                               int32_t kz, uint32_t ka, const ot_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py)
{
 GUARD(T o = load(out); T i = load(image); T k = load(kernel); T b = load(bias);
       CTensorConv<float>::ForwardConvolution(o, i, k, kx, ky, kz, ka, b, sx, sy, px, py); store(out, o);)
}
int oracle_backward_convolution(ot_tensor *out, const ot_tensor *delta, const ot_tensor *kernel, int32_t kx, int32_t ky,
                                int32_t kz, uint32_t ka, const ot_tensor *bias, int32_t sx, int32_t sy, int32_t px, int32_t py)
{
 GUARD(T o = load(out); T d = load(delta); T k = load(kernel); T b = load(bias);
       CTensorConv<float>::BackwardConvolution(o, d, k, kx, ky, kz, ka, b, sx, sy, px, py); store(out, o);)
}
int oracle_create_delta_weight_and_bias(ot_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, ot_tensor *db,
                                        const ot_tensor *image, const ot_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py)
{
 GUARD(T k = load(dk); T b = load(db); T i = load(image); T d = load(delta);
       CTensorConv<float>::CreateDeltaWeightAndBias(k, kx, ky, kz, ka, b, i, d, sx, sy, px, py); store(dk, k); store(db, b);)
}
int oracle_create_back_delta_weight_and_bias(ot_tensor *dk, int32_t kx, int32_t ky, int32_t kz, uint32_t ka, ot_tensor *db,
                                             const ot_tensor *image, const ot_tensor *delta, int32_t sx, int32_t sy, int32_t px, int32_t py)
{
 GUARD(T k = load(dk); T b = load(db); T i = load(image); T d = load(delta);
       CTensorConv<float>::CreateBackDeltaWeightAndBias(k, kx, ky, kz, ka, b, i, d, sx, sy, px, py); store(dk, k); store(db, b);)
}

int oracle_mul(ot_tensor *out, const ot_tensor *l, const ot_tensor *r)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::Mul(o, a, b); store(out, o);)
}
int oracle_transponse_mul(ot_tensor *out, const ot_tensor *l, const ot_tensor *r)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::TransponseMul(o, a, b); store(out, o);)
}
int oracle_transponse(ot_tensor *out, const ot_tensor *in)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::Transponse(o, a); store(out, o);)
}

int oracle_fill(ot_tensor *out, float v) { GUARD(T o = load(out); CTensorMath<float>::Fill(o, v); store(out, o);) }
int oracle_inv(ot_tensor *out, const ot_tensor *in)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::Inv(o, a); store(out, o);)
}
int oracle_div(ot_tensor *out, const ot_tensor *l, const ot_tensor *r, float ls, float rs)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::Div(o, a, b, ls, rs); store(out, o);)
}
int oracle_add(ot_tensor *out, const ot_tensor *l, const ot_tensor *r, float ls, float rs)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::Add(o, a, b, ls, rs); store(out, o);)
}
int oracle_sub(ot_tensor *out, const ot_tensor *l, const ot_tensor *r, float ls, float rs)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::Sub(o, a, b, ls, rs); store(out, o);)
}
int oracle_add_sum_w(ot_tensor *out, const ot_tensor *l, const ot_tensor *r, float ls, float rs)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::AddSumW(o, a, b, ls, rs); store(out, o);)
}
int oracle_add_bias(ot_tensor *working, const ot_tensor *bias)
{
 GUARD(T o = load(working); T b = load(bias); CTensorMath<float>::AddBias(o, b); store(working, o);)
}
int oracle_pow2(ot_tensor *out, const ot_tensor *in, float s)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::Pow2(o, a, s); store(out, o);)
}
int oracle_sqrt(ot_tensor *out, const ot_tensor *in, float s, float add)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::SQRT(o, a, s, add); store(out, o);)
}
int oracle_summ_xy(ot_tensor *out, const ot_tensor *in)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::SummXY(o, a); store(out, o);)
}
int oracle_mul_value(ot_tensor *out, const ot_tensor *in, float v)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::Mul(o, a, v); store(out, o);)
}
int oracle_tensor_item_production(ot_tensor *out, const ot_tensor *l, const ot_tensor *r)
{
 GUARD(T o = load(out); T a = load(l); T b = load(r); CTensorMath<float>::TensorItemProduction(o, a, b); store(out, o);)
}
int oracle_clip(ot_tensor *t, float lo, float hi) { GUARD(T o = load(t); CTensorMath<float>::Clip(o, lo, hi); store(t, o);) }
int oracle_signum(ot_tensor *t) { GUARD(T o = load(t); CTensorMath<float>::Signum(o); store(t, o);) }

// AddValue / SubValue / Set exist only in the GPU class of the reference, which cannot be built here.
int oracle_add_value(ot_tensor *, const ot_tensor *, float, float) { return -1; }
int oracle_sub_value(ot_tensor *, const ot_tensor *, float, float) { return -1; }
int oracle_set(ot_tensor *, const ot_tensor *, float, float) { return -1; }

int oracle_upsampling(ot_tensor *out, const ot_tensor *in, uint32_t ux, uint32_t uy)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::UpSampling(o, a, ux, uy); store(out, o);)
}
int oracle_downsampling(ot_tensor *out, const ot_tensor *in, uint32_t dx, uint32_t dy)
{
 GUARD(T o = load(out); T a = load(in); CTensorMath<float>::DownSampling(o, a, dx, dy); store(out, o);)
}
int oracle_max_pooling(ot_tensor *out, ot_pos_tensor *pos, const ot_tensor *in, uint32_t px, uint32_t py)
{
 GUARD(T o = load(out); T a = load(in); CTensor<SPos> p(pos->w, pos->z, pos->y, pos->x);
       CTensorMath<float>::MaxPooling(o, p, a, px, py); store(out, o);
       uint32_t n = pos->w * pos->z * pos->y * pos->x;
       if (n) memcpy(pos->p, p.GetColumnPtr(0, 0, 0), n * sizeof(SPos));)
}
int oracle_max_pooling_backward(ot_tensor *out, const ot_pos_tensor *pos, const ot_tensor *in, uint32_t px, uint32_t py)
{
 GUARD(T o = load(out); T a = load(in); CTensor<SPos> p(pos->w, pos->z, pos->y, pos->x);
       uint32_t n = pos->w * pos->z * pos->y * pos->x;
       if (n) p.CopyItemToHost(reinterpret_cast<SPos *>(pos->p), n);
       CTensorMath<float>::MaxPoolingBackward(o, p, a, px, py); store(out, o);)
}
int oracle_adam(ot_tensor *w, const ot_tensor *dw, ot_tensor *m, ot_tensor *v, uint32_t batch, double speed, double b1,
                double b2, double eps, double it)
{
 GUARD(T tw = load(w); T tdw = load(dw); T tm = load(m); T tv = load(v);
       CTensorMath<float>::Adam(tw, tdw, tm, tv, batch, speed, b1, b2, eps, it); store(w, tw); store(m, tm); store(v, tv);)
}

float oracle_func_scalar(int func, float v)
{
 typedef CTensorApplyFunc<float> F;
 switch (func)
 {
  case 0: return F::Sigmoid(v);
  case 1: return F::ReLU(v);
  case 2: return F::GeLU(v);
  case 3: return F::LeakyReLU(v);
  case 4: return F::Linear(v);
  case 5: return F::Tangence(v);
  case 8: return F::dSigmoid(v);
  case 9: return F::dReLU(v);
  case 10: return F::dGeLU(v);
  case 11: return F::dLeakyReLU(v);
  case 12: return F::dLinear(v);
  case 13: return F::dTangence(v);
 }
 return NAN;
}
int oracle_apply_func(ot_tensor *out, const ot_tensor *in, int func)
{
 typedef CTensorApplyFunc<float> F;
 GUARD(T o = load(out); T a = load(in);
       switch (func)
       {
        case 0: F::ApplySigmoid(o, a); break;
        case 1: F::ApplyReLU(o, a); break;
        case 2: F::ApplyGeLU(o, a); break;
        case 3: F::ApplyLeakyReLU(o, a); break;
        case 4: F::ApplyLinear(o, a); break;
        case 5: F::ApplyTangence(o, a); break;
        case 8: F::ApplyDifferentialSigmoid(o, a); break;
        case 9: F::ApplyDifferentialReLU(o, a); break;
        case 10: F::ApplyDifferentialGeLU(o, a); break;
        case 11: F::ApplyDifferentialLeakyReLU(o, a); break;
        case 12: F::ApplyDifferentialLinear(o, a); break;
        case 13: F::ApplyDifferentialTangence(o, a); break;
        default: return -1;
       }
       store(out, o);)
}

}  // extern "C"
