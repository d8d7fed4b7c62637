"""numpy-in / numpy-out front end of the C ABI with the same method names as oracle_api.Oracle,
so that a parity test is `gpu.f(*args)` against `oracle.f(*args)`.  Every call uploads its inputs,
runs the HIP path through libmi355tensor.so and downloads the result."""
import numpy as np

import mi355tensor as mt
from mi355tensor import CTensor, CTensorApplyFunc, CTensorConv, CTensorMath, Fused


def up(a):
    return CTensor.from_numpy(np.ascontiguousarray(a, dtype=np.float32))


up_ = up   # for methods with a parameter called `up`


class Gpu:
    def __init__(self):
        mt.init(0)

    # ---- convolutions ---------------------------------------------------
    def forward_convolution(self, image, kernel, bias, kx, ky, kz, ka, sx, sy, px, py, out_w=None, out_shape=None, func=None):
        image, kernel, bias = (np.asarray(a, np.float32) for a in (image, kernel, bias))
        if out_shape is None:
            out_shape = (out_w or image.shape[0], ka, (image.shape[2] - ky + 2 * py) // sy + 1, (image.shape[3] - kx + 2 * px) // sx + 1)
        out = CTensor(*out_shape)
        CTensorConv.ForwardConvolution(out, up(image), up(kernel), kx, ky, kz, ka, up(bias), sx, sy, px, py, func=func)
        return out.numpy()

    def backward_convolution(self, delta, kernel, bias, kx, ky, kz, ka, sx, sy, px, py, out_shape, func=None):
        out = CTensor(*out_shape)
        CTensorConv.BackwardConvolution(out, up(delta), up(kernel), kx, ky, kz, ka, up(bias), sx, sy, px, py, func=func)
        return out.numpy()

    def create_delta_weight_and_bias(self, dkernel, dbias, image, delta, kx, ky, kz, ka, sx, sy, px, py, back=False):
        dk, db = up(dkernel), up(dbias)
        fn = CTensorConv.CreateBackDeltaWeightAndBias if back else CTensorConv.CreateDeltaWeightAndBias
        fn(dk, kx, ky, kz, ka, db, up(image), up(delta), sx, sy, px, py)
        return dk.numpy(), db.numpy()

    def convolution_backward_weights_sum(self, dkernel, dbias, image, delta, kx, ky, kz, ka, sx, sy, px, py):
        dk, db = up(dkernel), up(dbias)
        Fused.ConvolutionBackwardWeightsSum(dk, kx, ky, kz, ka, db, up(image), up(delta), sx, sy, px, py)
        return dk.numpy(), db.numpy()

    # ---- products -------------------------------------------------------
    def mul(self, left, right, out_w=None):
        left, right = np.asarray(left, np.float32), np.asarray(right, np.float32)
        out = CTensor(out_w or max(left.shape[0], right.shape[0]), right.shape[1], left.shape[2], right.shape[3])
        CTensorMath.Mul(out, up(left), up(right))
        return out.numpy()

    def transponse_mul(self, left, right, out_w=None):
        left, right = np.asarray(left, np.float32), np.asarray(right, np.float32)
        out = CTensor(out_w or max(left.shape[0], right.shape[0]), right.shape[1], left.shape[3], right.shape[3])
        CTensorMath.TransponseMul(out, up(left), up(right))
        return out.numpy()

    def transponse(self, a):
        a = np.asarray(a, np.float32)
        out = CTensor(a.shape[0], a.shape[1], a.shape[3], a.shape[2])
        CTensorMath.Transponse(out, up(a))
        return out.numpy()

    # ---- elementwise / reductions --------------------------------------------
    def _binary(self, fn, left, right, *scalars, out_shape=None):
        left, right = np.asarray(left, np.float32), np.asarray(right, np.float32)
        if out_shape is None:
            out_shape = (max(left.shape[0], right.shape[0]),) + right.shape[1:]
        out = CTensor(*out_shape)
        fn(out, up(left), up(right), *scalars)
        return out.numpy()

    def add(self, left, right, ls=1.0, rs=1.0, out_shape=None):
        return self._binary(CTensorMath.Add, left, right, ls, rs, out_shape=out_shape)

    def sub(self, left, right, ls=1.0, rs=1.0, out_shape=None):
        return self._binary(CTensorMath.Sub, left, right, ls, rs, out_shape=out_shape)

    def div(self, left, right, ls=1.0, rs=1.0, out_shape=None):
        return self._binary(CTensorMath.Div, left, right, ls, rs, out_shape=out_shape)

    def tensor_item_production(self, left, right, out_shape=None):
        return self._binary(CTensorMath.TensorItemProduction, left, right, out_shape=out_shape)

    def add_sum_w(self, left, right, ls=1.0, rs=1.0, out_w=1, out_init=None):
        right = np.asarray(right, np.float32)
        out = up(np.full((out_w,) + right.shape[1:], 7.0, np.float32) if out_init is None else out_init)
        CTensorMath.AddSumW(out, up(left), up(right), ls, rs)
        return out.numpy()

    def _unary(self, fn, a, *scalars, out_w=None):
        a = np.asarray(a, np.float32)
        out = CTensor(out_w or a.shape[0], *a.shape[1:])
        fn(out, up(a), *scalars)
        return out.numpy()

    def inv(self, a, out_w=None):
        return self._unary(CTensorMath.Inv, a, out_w=out_w)

    def pow2(self, a, scale=1.0, out_w=None):
        return self._unary(CTensorMath.Pow2, a, scale, out_w=out_w)

    def sqrt(self, a, scale, add, out_w=None):
        return self._unary(CTensorMath.SQRT, a, scale, add, out_w=out_w)

    def mul_value(self, a, value, out_w=None):
        return self._unary(CTensorMath.Mul, a, float(value), out_w=out_w)

    def add_value(self, a, scale, value, out_w=None):
        return self._unary(CTensorMath.AddValue, a, scale, value, out_w=out_w)

    def sub_value(self, a, scale, value, out_w=None):
        return self._unary(CTensorMath.SubValue, a, scale, value, out_w=out_w)

    def set(self, a, scale=1.0, add=0.0, out_w=None):
        return self._unary(CTensorMath.Set, a, scale, add, out_w=out_w)

    def fill(self, shape, value):
        out = CTensor(*shape)
        CTensorMath.Fill(out, value)
        return out.numpy()

    def add_bias(self, working, bias):
        t = up(working)
        CTensorMath.AddBias(t, up(bias))
        return t.numpy()

    def summ_xy(self, a, out_w=None):
        a = np.asarray(a, np.float32)
        out = CTensor(out_w or a.shape[0], a.shape[1], 1, 1)
        CTensorMath.SummXY(out, up(a))
        return out.numpy()

    def clip(self, a, lo, hi):
        t = up(a)
        CTensorMath.Clip(t, lo, hi)
        return t.numpy()

    def signum(self, a):
        t = up(a)
        CTensorMath.Signum(t)
        return t.numpy()

    # ---- resampling / pooling ------------------------------------------------
    def upsampling(self, a, ux, uy, out_shape=None):
        a = np.asarray(a, np.float32)
        out = up(np.full(out_shape or (a.shape[0], a.shape[1], a.shape[2] * uy, a.shape[3] * ux), 7.0, np.float32))
        CTensorMath.UpSampling(out, up(a), ux, uy)
        return out.numpy()

    def downsampling(self, a, dx, dy):
        a = np.asarray(a, np.float32)
        out = CTensor(a.shape[0], a.shape[1], a.shape[2] // dy, a.shape[3] // dx)
        CTensorMath.DownSampling(out, up(a), dx, dy)
        return out.numpy()

    def max_pooling(self, a, px, py):
        a = np.asarray(a, np.float32)
        shape = (a.shape[0], a.shape[1], a.shape[2] // py, a.shape[3] // px)
        out, pos = CTensor(*shape), CTensor(*shape, pos=True)
        CTensorMath.MaxPooling(out, pos, up(a), px, py)
        return out.numpy(), pos.numpy()

    def max_pooling_backward(self, delta, pos, px, py, out_shape):
        pos = np.ascontiguousarray(pos, dtype=np.uint32)
        p = CTensor(*pos.shape[:4], pos=True)
        p.upload(pos)
        out = up(np.full(out_shape, 7.0, np.float32))
        CTensorMath.MaxPoolingBackward(out, p, up(delta), px, py)
        return out.numpy()

    # ---- optimiser / activations -----------------------------------------------
    def adam(self, weight, dweight, m, v, batch_size, speed, beta1, beta2, epsilon, iteration):
        w, mm, vv = up(weight), up(m), up(v)
        CTensorMath.Adam(w, up(dweight), mm, vv, batch_size, speed, beta1, beta2, epsilon, iteration)
        return w.numpy(), mm.numpy(), vv.numpy()

    def apply_func(self, a, func, differential=False):
        a = np.asarray(a, np.float32)
        out = CTensor(*a.shape)
        CTensorApplyFunc.Apply(out, up(a), func, differential)
        return out.numpy()

    # ---- fused layers -------------------------------------------------------------
    def linear_forward(self, weight, x, bias, func=None):
        x = np.asarray(x, np.float32)
        out = CTensor(x.shape[0], 1, weight.shape[2], 1)
        Fused.LinearForward(out, up(weight), up(x), up(bias), func)
        return out.numpy()

    def batchnorm_train(self, x, gamma, beta, momentum=0.9, eps=1e-6, func=None, new_mean=None, new_var=None):
        x = np.asarray(x, np.float32)
        s = (1,) + x.shape[1:]
        out, xhat, ivar, mean, var = CTensor(*x.shape), CTensor(*x.shape), CTensor(*s), CTensor(*s), CTensor(*s)
        nm = up(new_mean) if new_mean is not None else None
        nv = up(new_var) if new_var is not None else None
        Fused.BatchNormForwardTrain(out, up(x), up(gamma), up(beta), xhat, ivar, mean, var, nm, nv, momentum, eps, func)
        res = dict(out=out.numpy(), xhat=xhat.numpy(), ivar=ivar.numpy(), mean=mean.numpy(), var=var.numpy())
        if nm is not None:
            res["new_mean"], res["new_var"] = nm.numpy(), nv.numpy()
        return res

    def batchnorm_backward(self, delta, gamma, xhat, ivar, dgamma0, dbeta0, beta=None, func=None):
        delta = np.asarray(delta, np.float32)
        err, dg, db = CTensor(*delta.shape), up(dgamma0), up(dbeta0)
        Fused.BatchNormBackward(err, dg, db, up(delta), up(gamma), up(xhat), up(ivar), beta=up(beta) if beta is not None else None, func=func)
        return err.numpy(), dg.numpy(), db.numpy()

    def upsampling_convolution(self, image, kernel, bias, k, kz, ka, up=2, s=1, p=1, func=None):
        image = np.asarray(image, np.float32)
        oy, ox = (image.shape[2] * up - k + 2 * p) // s + 1, (image.shape[3] * up - k + 2 * p) // s + 1
        out = up_(np.full((image.shape[0], ka, oy, ox), 7.0, np.float32))
        Fused.UpSamplingConvolution(out, up_(image), up, up, up_(kernel), k, k, kz, ka, up_(bias), s, s, p, p, func)
        return out.numpy()

    # ---- functions of the reference's GPU class only ---------------------------
    def concatecation_z(self, a, b, out_w=None):
        a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
        out = up(np.full((out_w or max(a.shape[0], b.shape[0]), a.shape[1] + b.shape[1], a.shape[2], a.shape[3]), 7.0, np.float32))
        CTensorMath.ConcatecationZ(out, up(a), up(b))
        return out.numpy()

    def split_z(self, a, za, out_w=None):
        a = np.asarray(a, np.float32)
        w = out_w or a.shape[0]
        oa, ob = up(np.full((w, za) + a.shape[2:], 7.0, np.float32)), up(np.full((w, a.shape[1] - za) + a.shape[2:], 7.0, np.float32))
        CTensorMath.SplitZ(oa, ob, up(a))
        return oa.numpy(), ob.numpy()

    def set_time_step(self, a, time_step):
        a = np.asarray(a, np.float32)
        t = CTensor(a.shape[0], 1, 1, 1, u32=True)
        t.upload(np.asarray(time_step, np.uint32))
        out = CTensor(*a.shape)
        CTensorMath.SetTimeStep(out, up(a), t)
        return out.numpy()

    def create_drop_out_matrix(self, shape, drop_out, seed):
        out = CTensor(*shape)
        CTensorMath.CreateDropOutMatrix(out, drop_out, seed)
        return out.numpy()

    def set_normal_noise(self, shape, seed):
        out = CTensor(*shape)
        CTensorMath.SetNormalNoise(out, seed)
        return out.numpy()

    def get_noise_image_and_noise(self, image, sqrt_alpha_bar, sqrt_one_minus_alpha_bar, seed):
        image = np.asarray(image, np.float32)
        noisy, noise = CTensor(*image.shape), CTensor(*image.shape)
        CTensorMath.GetNoiseImageAndNoise(noisy, noise, up(image), up(sqrt_alpha_bar), up(sqrt_one_minus_alpha_bar), seed)
        return noisy.numpy(), noise.numpy()

    def fill_many(self, arrays, value):
        ts = [up(a) for a in arrays]
        Fused.FillMany(ts, value)
        return [t.numpy() for t in ts]

    def adam_many(self, weights, dweights, ms, vs, batch_size, speed, beta1, beta2, epsilon, iteration):
        w, dw, m, v = ([up(a) for a in group] for group in (weights, dweights, ms, vs))
        Fused.AdamMany(w, dw, m, v, batch_size, speed, beta1, beta2, epsilon, iteration)
        return [t.numpy() for t in w], [t.numpy() for t in m], [t.numpy() for t in v]

    def vae_coder_output(self, mu, logvar, epsilon):
        mu = np.asarray(mu, np.float32)
        out, kl = CTensor(*mu.shape), CTensor(1, 1, 1, 1)
        Fused.VaeCoderOutput(out, kl, up(mu), up(logvar), up(epsilon))
        return out.numpy(), float(kl.numpy().ravel()[0])

    def batchnorm_infer(self, x, gamma, beta, mean, var, eps=1e-6, func=None):
        x = np.asarray(x, np.float32)
        out = CTensor(*x.shape)
        Fused.BatchNormForwardInfer(out, up(x), up(gamma), up(beta), up(mean), up(var), eps, func)
        return out.numpy()
