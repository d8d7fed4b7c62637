"""TEST INFRASTRUCTURE ONLY -- ctypes front end of the CPU oracle.

Loads ``oracle/liboracle.so`` (the C restatement) or, with ``which="ref"``,
``oracle/_ref/libtensor_ref.so`` (the reference's own CPU headers compiled in the
authoring container).  Both export the flat API of ``tensor_oracle.h``.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the product never does.

All tensors are numpy float32 arrays of shape ``[W, Z, Y, X]``.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
PATHS = {
    "oracle": os.path.join(HERE, "liboracle.so"),
    "ref": os.path.join(HERE, "_ref", "libtensor_ref.so"),
}

FUNC = {"sigmoid": 0, "relu": 1, "gelu": 2, "leaky_relu": 3, "linear": 4, "tangence": 5}
DIFFERENTIAL = 8


class OtTensor(C.Structure):
    _fields_ = [("p", C.c_void_p), ("w", C.c_uint32), ("z", C.c_uint32), ("y", C.c_uint32), ("x", C.c_uint32)]


class OracleError(RuntimeError):
    def __init__(self, name, code):
        super().__init__("%s failed with code %d" % (name, code))
        self.code = code


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    assert a.ndim == 4, "tensors are [W,Z,Y,X]"
    return a


def _desc(a):
    return OtTensor(a.ctypes.data, *a.shape)


def available(which="oracle"):
    return os.path.exists(PATHS[which])


class Oracle:
    """One loaded oracle library. Method names follow the reference's function names."""

    def __init__(self, which="oracle"):
        self.which = which
        self.lib = C.CDLL(PATHS[which])
        self.lib.oracle_func_scalar.restype = C.c_float
        self.lib.oracle_func_scalar.argtypes = [C.c_int, C.c_float]

    def _call(self, name, *args):
        fn = getattr(self.lib, "oracle_" + name)
        fn.restype = C.c_int
        rc = fn(*args)
        if rc != 0:
            raise OracleError(name, rc)

    @staticmethod
    def _p(a):
        d = _desc(a)
        return C.byref(d)

    # ---- convolutions -------------------------------------------------
    def forward_convolution(self, image, kernel, bias, kx, ky, kz, ka, sx, sy, px, py, out_w=None, out_shape=None):
        image, kernel, bias = _f32(image), _f32(kernel), _f32(bias)
        if out_shape is None:
            oy = (image.shape[2] - ky + 2 * py) // sy + 1
            ox = (image.shape[3] - kx + 2 * px) // sx + 1
            out_shape = (out_w or image.shape[0], ka, oy, ox)
        out = np.zeros(out_shape, np.float32)
        self._call("forward_convolution", self._p(out), self._p(image), self._p(kernel), C.c_int32(kx), C.c_int32(ky),
                   C.c_int32(kz), C.c_uint32(ka), self._p(bias), C.c_int32(sx), C.c_int32(sy), C.c_int32(px), C.c_int32(py))
        return out

    def backward_convolution(self, delta, kernel, bias, kx, ky, kz, ka, sx, sy, px, py, out_shape):
        delta, kernel, bias = _f32(delta), _f32(kernel), _f32(bias)
        out = np.zeros(out_shape, np.float32)
        self._call("backward_convolution", self._p(out), self._p(delta), self._p(kernel), C.c_int32(kx), C.c_int32(ky),
                   C.c_int32(kz), C.c_uint32(ka), self._p(bias), C.c_int32(sx), C.c_int32(sy), C.c_int32(px), C.c_int32(py))
        return out

    def create_delta_weight_and_bias(self, dkernel, dbias, image, delta, kx, ky, kz, ka, sx, sy, px, py, back=False):
        """Accumulates into copies of dkernel/dbias and returns them."""
        dkernel, dbias = _f32(dkernel).copy(), _f32(dbias).copy()
        image, delta = _f32(image), _f32(delta)
        name = "create_back_delta_weight_and_bias" if back else "create_delta_weight_and_bias"
        self._call(name, self._p(dkernel), C.c_int32(kx), C.c_int32(ky), C.c_int32(kz), C.c_uint32(ka), self._p(dbias),
                   self._p(image), self._p(delta), C.c_int32(sx), C.c_int32(sy), C.c_int32(px), C.c_int32(py))
        return dkernel, dbias

    # ---- products -----------------------------------------------------
    def mul(self, left, right, out_w=None):
        left, right = _f32(left), _f32(right)
        out = np.zeros((out_w or max(left.shape[0], right.shape[0]), right.shape[1], left.shape[2], right.shape[3]), np.float32)
        self._call("mul", self._p(out), self._p(left), self._p(right))
        return out

    def transponse_mul(self, left, right, out_w=None):
        left, right = _f32(left), _f32(right)
        out = np.zeros((out_w or max(left.shape[0], right.shape[0]), right.shape[1], left.shape[3], right.shape[3]), np.float32)
        self._call("transponse_mul", self._p(out), self._p(left), self._p(right))
        return out

    def transponse(self, a):
        a = _f32(a)
        out = np.zeros((a.shape[0], a.shape[1], a.shape[3], a.shape[2]), np.float32)
        self._call("transponse", self._p(out), self._p(a))
        return out

    # ---- elementwise / reductions -------------------------------------
    def _binary(self, name, left, right, ls, rs, out_shape=None):
        left, right = _f32(left), _f32(right)
        if out_shape is None:
            out_shape = (max(left.shape[0], right.shape[0]),) + right.shape[1:]
        out = np.zeros(out_shape, np.float32)
        self._call(name, self._p(out), self._p(left), self._p(right), C.c_float(ls), C.c_float(rs))
        return out

    def add(self, left, right, ls=1.0, rs=1.0, out_shape=None):
        return self._binary("add", left, right, ls, rs, out_shape)

    def sub(self, left, right, ls=1.0, rs=1.0, out_shape=None):
        return self._binary("sub", left, right, ls, rs, out_shape)

    def div(self, left, right, ls=1.0, rs=1.0, out_shape=None):
        return self._binary("div", left, right, ls, rs, out_shape)

    def add_sum_w(self, left, right, ls=1.0, rs=1.0, out_w=1, out_init=None):
        left, right = _f32(left), _f32(right)
        out = np.full((out_w,) + right.shape[1:], 7.0, np.float32) if out_init is None else _f32(out_init).copy()
        self._call("add_sum_w", self._p(out), self._p(left), self._p(right), C.c_float(ls), C.c_float(rs))
        return out

    def tensor_item_production(self, left, right, out_shape=None):
        left, right = _f32(left), _f32(right)
        if out_shape is None:
            out_shape = (max(left.shape[0], right.shape[0]),) + right.shape[1:]
        out = np.zeros(out_shape, np.float32)
        self._call("tensor_item_production", self._p(out), self._p(left), self._p(right))
        return out

    def _unary(self, name, a, *scalars, out_w=None):
        a = _f32(a)
        out = np.zeros((out_w or a.shape[0],) + a.shape[1:], np.float32)
        self._call(name, self._p(out), self._p(a), *[C.c_float(s) for s in scalars])
        return out

    def inv(self, a, out_w=None):
        return self._unary("inv", a, out_w=out_w)

    def pow2(self, a, scale=1.0, out_w=None):
        return self._unary("pow2", a, scale, out_w=out_w)

    def sqrt(self, a, scale, add, out_w=None):
        return self._unary("sqrt", a, scale, add, out_w=out_w)

    def mul_value(self, a, value, out_w=None):
        return self._unary("mul_value", a, value, out_w=out_w)

    def add_value(self, a, scale, value, out_w=None):
        return self._unary("add_value", a, scale, value, out_w=out_w)

    def sub_value(self, a, scale, value, out_w=None):
        return self._unary("sub_value", a, scale, value, out_w=out_w)

    def set(self, a, scale=1.0, add=0.0, out_w=None):
        return self._unary("set", a, scale, add, out_w=out_w)

    def fill(self, shape, value):
        out = np.zeros(shape, np.float32)
        self._call("fill", self._p(out), C.c_float(value))
        return out

    def add_bias(self, working, bias):
        working, bias = _f32(working).copy(), _f32(bias)
        self._call("add_bias", self._p(working), self._p(bias))
        return working

    def summ_xy(self, a, out_w=None):
        a = _f32(a)
        out = np.zeros((out_w or a.shape[0], a.shape[1], 1, 1), np.float32)
        self._call("summ_xy", self._p(out), self._p(a))
        return out

    def clip(self, a, lo, hi):
        a = _f32(a).copy()
        self._call("clip", self._p(a), C.c_float(lo), C.c_float(hi))
        return a

    def signum(self, a):
        a = _f32(a).copy()
        self._call("signum", self._p(a))
        return a

    # ---- resampling / pooling -----------------------------------------
    def upsampling(self, a, ux, uy, out_shape=None):
        a = _f32(a)
        if out_shape is None:
            out_shape = (a.shape[0], a.shape[1], a.shape[2] * uy, a.shape[3] * ux)
        out = np.full(out_shape, 7.0, np.float32)
        self._call("upsampling", self._p(out), self._p(a), C.c_uint32(ux), C.c_uint32(uy))
        return out

    def downsampling(self, a, dx, dy):
        a = _f32(a)
        out = np.zeros((a.shape[0], a.shape[1], a.shape[2] // dy, a.shape[3] // dx), np.float32)
        self._call("downsampling", self._p(out), self._p(a), C.c_uint32(dx), C.c_uint32(dy))
        return out

    def max_pooling(self, a, px, py):
        """Returns (pooled, positions) with positions as uint32 [W,Z,Y,X,2] = (X, Y) pairs."""
        a = _f32(a)
        shape = (a.shape[0], a.shape[1], a.shape[2] // py, a.shape[3] // px)
        out = np.zeros(shape, np.float32)
        pos = np.zeros(shape + (2,), np.uint32)
        pd = OtTensor(pos.ctypes.data, *shape)
        self._call("max_pooling", self._p(out), C.byref(pd), self._p(a), C.c_uint32(px), C.c_uint32(py))
        return out, pos

    def max_pooling_backward(self, delta, pos, px, py, out_shape):
        delta = _f32(delta)
        pos = np.ascontiguousarray(pos, dtype=np.uint32)
        out = np.full(out_shape, 7.0, np.float32)
        pd = OtTensor(pos.ctypes.data, *pos.shape[:4])
        self._call("max_pooling_backward", self._p(out), C.byref(pd), self._p(delta), C.c_uint32(px), C.c_uint32(py))
        return out

    # ---- optimiser ----------------------------------------------------
    def adam(self, weight, dweight, m, v, batch_size, speed, beta1, beta2, epsilon, iteration):
        weight, m, v = _f32(weight).copy(), _f32(m).copy(), _f32(v).copy()
        dweight = _f32(dweight)
        self._call("adam", self._p(weight), self._p(dweight), self._p(m), self._p(v), C.c_uint32(batch_size),
                   C.c_double(speed), C.c_double(beta1), C.c_double(beta2), C.c_double(epsilon), C.c_double(iteration))
        return weight, m, v

    # ---- VAE coder output ----------------------------------------------
    def vae_coder_output(self, mu, logvar, epsilon):
        mu, logvar, epsilon = _f32(mu), _f32(logvar), _f32(epsilon)
        out, kl = np.zeros(mu.shape, np.float32), C.c_float()
        self._call("vae_coder_output", self._p(out), C.byref(kl), self._p(mu), self._p(logvar), self._p(epsilon))
        return out, kl.value

    # ---- functions of the reference's GPU class only ---------------------
    def concatecation_z(self, a, b, out_w=None):
        a, b = _f32(a), _f32(b)
        out = np.zeros((out_w or max(a.shape[0], b.shape[0]), a.shape[1] + b.shape[1], a.shape[2], a.shape[3]), np.float32)
        self._call("concatecation_z", self._p(out), self._p(a), self._p(b))
        return out

    def split_z(self, a, za, out_w=None):
        a = _f32(a)
        w = out_w or a.shape[0]
        oa, ob = np.zeros((w, za) + a.shape[2:], np.float32), np.zeros((w, a.shape[1] - za) + a.shape[2:], np.float32)
        self._call("split_z", self._p(oa), self._p(ob), self._p(a))
        return oa, ob

    def set_time_step(self, a, time_step):
        a, t = _f32(a), np.ascontiguousarray(time_step, dtype=np.uint32).ravel()
        out = np.zeros(a.shape, np.float32)
        self._call("set_time_step", self._p(out), self._p(a), t.ctypes.data_as(C.POINTER(C.c_uint32)), C.c_uint32(t.size))
        return out

    def philox4x32_10(self, counter, key):
        c, k, out = (C.c_uint32 * 4)(*counter), (C.c_uint32 * 2)(*key), (C.c_uint32 * 4)()
        self.lib.oracle_philox4x32_10.restype = None
        self.lib.oracle_philox4x32_10(c, k, out)
        return tuple(out)

    def create_drop_out_matrix(self, shape, drop_out, seed):
        out = np.zeros(shape, np.float32)
        self._call("create_drop_out_matrix", self._p(out), C.c_float(drop_out), C.c_uint64(seed))
        return out

    def set_normal_noise(self, shape, seed):
        out = np.zeros(shape, np.float32)
        self._call("set_normal_noise", self._p(out), C.c_uint64(seed))
        return out

    def get_noise_image_and_noise(self, image, sqrt_alpha_bar, sqrt_one_minus_alpha_bar, seed):
        image, sa, sb = _f32(image), _f32(sqrt_alpha_bar), _f32(sqrt_one_minus_alpha_bar)
        noisy, noise = np.zeros(image.shape, np.float32), np.zeros(image.shape, np.float32)
        self._call("get_noise_image_and_noise", self._p(noisy), self._p(noise), self._p(image), self._p(sa), self._p(sb), C.c_uint64(seed))
        return noisy, noise

    # ---- activations --------------------------------------------------
    def apply_func(self, a, func, differential=False):
        a = _f32(a)
        out = np.zeros(a.shape, np.float32)
        code = FUNC[func] + (DIFFERENTIAL if differential else 0)
        self._call("apply_func", self._p(out), self._p(a), C.c_int(code))
        return out

    def func_scalar(self, v, func, differential=False):
        return float(self.lib.oracle_func_scalar(FUNC[func] + (DIFFERENTIAL if differential else 0), C.c_float(v)))
