"""ctypes binding of libmi355tensor.so for tests and benchmarks.

The names mirror the reference's C++ classes (`CTensor`, `CTensorMath`, `CTensorConv`,
`CTensorApplyFunc`; cuda/ctensor.cu.h:69-168, cuda/ctensormath.cu.h:52-138,
cuda/ctensorconv.cu.h:48-69, cuda/ctensorapplyfunc.cu.h) with the same argument order, so a test
written against the reference reads the same here.  Every call goes through the C ABI declared in
include/mi355_tensor.h; there is no CPU fallback: without the built library and a gfx950 device
this module raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmi355tensor.so")

FUNC = {"sigmoid": 0, "relu": 1, "gelu": 2, "leaky_relu": 3, "linear": 4, "tangence": 5, None: -1, "none": -1}
DIFFERENTIAL = 8


class MtTensor(C.Structure):
    _fields_ = [("p", C.c_void_p), ("w", C.c_uint32), ("z", C.c_uint32), ("y", C.c_uint32), ("x", C.c_uint32)]


class TensorError(RuntimeError):
    """A non-zero status of the C ABI (the C++ classes `throw` a message in the same place)."""

    def __init__(self, name, code, message):
        super().__init__("%s failed with code %d: %s" % (name, code, message))
        self.code = code


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libmi355tensor.so is not built: run `make -C cuda-cnn-gan-vae_amd` (or __graft_entry__.build())")
        _lib = C.CDLL(LIB_PATH)
        _lib.mt_last_error.restype = C.c_char_p
        _lib.mt_get_stream.restype = C.c_void_p
        _lib.mt_malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        _lib.mt_free.argtypes = [C.c_void_p]
        for f in ("mt_copy_h2d", "mt_copy_d2h", "mt_copy_d2d"):
            getattr(_lib, f).argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        _lib.mt_set_stream.argtypes = [C.c_void_p]
        _lib.mt_set_option.argtypes = [C.c_char_p, C.c_int]
        _lib.mt_get_info.argtypes = [C.c_char_p, C.POINTER(C.c_int64)]
        _lib.mt_invalidate.argtypes = [C.c_void_p, C.c_size_t]
    return _lib


def call(name, *args):
    rc = getattr(_lib or lib(), name)(*args)   # ctypes' default result type is int
    if rc != 0:
        raise TensorError(name, rc, lib().mt_last_error().decode(errors="replace"))


def init(device=0):
    call("mt_init", C.c_int(device))


def synchronize():
    call("mt_synchronize")


def set_option(name, value):
    call("mt_set_option", name.encode(), C.c_int(value))


def get_info(name):
    """A counter of the runtime (memory pool, kept re-ordered weights, retired workspaces); see mt_get_info."""
    v = C.c_int64()
    call("mt_get_info", name.encode(), C.byref(v))
    return v.value


def invalidate(ptr, nbytes):
    """Announce a write to device memory that did not go through this library (see mt_invalidate)."""
    call("mt_invalidate", C.c_void_p(ptr), C.c_size_t(nbytes))


def profile_enable(on=True):
    call("mt_profile_enable", C.c_int(1 if on else 0))


def profile_report():
    """{label: (launches, total_ms)} of the kernels launched since profile_enable(True); waits for the stream."""
    n = lib().mt_profile_entries()
    if n < 0:
        raise TensorError("mt_profile_entries", n, lib().mt_last_error().decode(errors="replace"))
    out = {}
    for i in range(n):
        label, launches, ms = C.c_char_p(), C.c_uint64(), C.c_double()
        call("mt_profile_entry", C.c_int(i), C.byref(label), C.byref(launches), C.byref(ms))
        out[label.value.decode()] = (launches.value, ms.value)
    return out


def get_stream():
    return lib().mt_get_stream()


def set_stream(handle):
    call("mt_set_stream", C.c_void_p(handle))


class Timer:
    """Milliseconds of queued work between start() and stop() (two events on the work stream; the reference's
    CCUDATimeSpent, cuda/ccudatimespent.cu:9-52)."""

    def __init__(self):
        self._t = C.c_void_p()
        call("mt_timer_create", C.byref(self._t))

    def start(self):
        call("mt_timer_start", self._t)

    def stop(self):
        ms = C.c_float()
        call("mt_timer_stop", self._t, C.byref(ms))
        return ms.value

    def __del__(self):
        try:
            if self._t:
                call("mt_timer_destroy", self._t)
        except Exception:
            pass


class Graph:
    """A sequence of library calls recorded once as a HIP graph and replayed with one launch: for steps made of many
    short kernels, where the host would otherwise be the bottleneck.  Everything the calls allocate (workspaces) must
    exist before the recording, so run the sequence once eagerly first.  The recorded kernels keep the pointers and
    sizes of the recording."""

    def __init__(self, record):
        hip = C.CDLL("libamdhip64.so")
        self._hip, self._stream = hip, C.c_void_p(get_stream())
        graph, self._exec = C.c_void_p(), C.c_void_p()
        self._check(hip.hipStreamBeginCapture(self._stream, C.c_int(2)), "hipStreamBeginCapture")   # relaxed mode
        try:
            record()
        finally:
            rc = hip.hipStreamEndCapture(self._stream, C.byref(graph))
        self._check(rc, "hipStreamEndCapture")
        self._check(hip.hipGraphInstantiate(C.byref(self._exec), graph, None, None, C.c_size_t(0)), "hipGraphInstantiate")
        hip.hipGraphDestroy(graph)

    @staticmethod
    def _check(rc, what):
        if rc != 0:
            raise RuntimeError("%s failed with hipError %d" % (what, rc))

    def launch(self):
        self._check(self._hip.hipGraphLaunch(self._exec, self._stream), "hipGraphLaunch")

    def __del__(self):
        try:
            if self._exec:
                self._hip.hipGraphExecDestroy(self._exec)
        except Exception:
            pass


class CTensor:
    """Device-resident [W,Z,Y,X] fp32 tensor (uint32 pairs for pooling positions when `pos` is set)."""

    def __init__(self, size_w=1, size_z=1, size_y=1, size_x=1, pos=False, u32=False):
        self.shape = (int(size_w), int(size_z), int(size_y), int(size_x))
        self.pos, self.u32 = pos, u32     # u32: CTensor<uint32_t> (time steps)
        self.item = 8 if pos else 4
        self.ptr = C.c_void_p()
        self.owned = True
        call("mt_malloc", C.byref(self.ptr), C.c_size_t(self.count * self.item))

    @property
    def count(self):
        w, z, y, x = self.shape
        return w * z * y * x

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        assert a.ndim == 4, "tensors are [W,Z,Y,X]"
        t = cls(*a.shape)
        t.upload(a)
        return t

    @classmethod
    def wrap(cls, ptr, shape):
        """Borrow device memory owned by someone else (e.g. a torch tensor's data_ptr())."""
        t = cls.__new__(cls)
        t.shape, t.pos, t.u32, t.item, t.ptr, t.owned = tuple(int(s) for s in shape), False, False, 4, C.c_void_p(ptr), False
        return t

    def upload(self, a):
        a = np.ascontiguousarray(a, dtype=np.uint32 if self.pos or self.u32 else np.float32)
        assert a.size == self.count * (2 if self.pos else 1)
        if a.size:
            call("mt_copy_h2d", self.ptr, C.c_void_p(a.ctypes.data), C.c_size_t(a.nbytes))

    def numpy(self):
        out = np.empty(self.shape + ((2,) if self.pos else ()), np.uint32 if self.pos or self.u32 else np.float32)
        if out.size:
            call("mt_copy_d2h", C.c_void_p(out.ctypes.data), self.ptr, C.c_size_t(out.nbytes))
        else:
            synchronize()
        return out

    def Save(self, f):
        """CTensor::Save (cuda/ctensor.cu.h:525-537): copy back from the device, four sizes, then the values as doubles."""
        import wire_format
        assert not (self.pos or self.u32), "only CTensor<type_t> tensors are part of a checkpoint"
        wire_format.write_tensor(f, self.numpy())

    def Load(self, f, check_size=True):
        """CTensor::Load (cuda/ctensor.cu.h:541-571).  With `check_size` the sizes in the stream must be this tensor's own
        (TensorError, as the reference throws); without it the tensor takes the stream's sizes and new device memory."""
        import wire_format
        a = wire_format.read_tensor(f)
        if a.shape != self.shape:
            if check_size:
                axis = "WZYX"[[i for i in range(4) if a.shape[i] != self.shape[i]][0]]
                raise TensorError("CTensor::Load", -1, "the stream holds %s, the tensor is %s: wrong size %s" % (a.shape, self.shape, axis))
            assert self.owned, "a borrowed view cannot change its size"
            self.free()
            self.__dict__.pop("_ref", None)
            self.shape = a.shape
            call("mt_malloc", C.byref(self.ptr), C.c_size_t(self.count * self.item))
        self.upload(a)

    def reinterpret(self, w, z, y, x):
        """ReinterpretSize: the same memory under other sizes (cuda/ctensor.cu.h:587-601)."""
        assert w * z * y * x == self.count, "the element count must not change"
        t = CTensor.wrap(self.ptr.value, (w, z, y, x))
        t._base = self   # the view must not outlive the memory it looks at
        return t

    def desc(self):
        return MtTensor(self.ptr.value, *self.shape)

    def ref(self):
        """Pointer to this tensor's descriptor for a C-ABI call (built once: pointer and sizes never change)."""
        r = self.__dict__.get("_ref")
        if r is None:
            if not self.ptr and self.count:
                raise RuntimeError("the tensor's device memory has been freed")
            self._desc = self.desc()
            r = self._ref = C.byref(self._desc)
        return r

    def free(self):
        if self.owned and self.ptr:
            call("mt_free", self.ptr)
            self.ptr = C.c_void_p()
            self.__dict__.pop("_ref", None)
            self.__dict__.pop("_desc", None)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _d(t):
    return t.ref()


def _list(tensors):
    """Array of descriptor pointers for the entry points that take several tensors."""
    descs = [t.ref() and t._desc for t in tensors]
    return (C.POINTER(MtTensor) * len(descs))(*[C.pointer(d) for d in descs])


def _i(v):
    return C.c_int32(int(v))


def _u(v):
    return C.c_uint32(int(v))


def _f(v):
    return C.c_float(float(v))


class CTensorConv:
    @staticmethod
    def ForwardConvolution(out, image, kernel, kernel_x, kernel_y, kernel_z, kernel_amount, bias, stride_x, stride_y, padding_x, padding_y, func=None):
        args = (_d(out), _d(image), _d(kernel), _i(kernel_x), _i(kernel_y), _i(kernel_z), _u(kernel_amount), _d(bias), _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y))
        if func is None:
            call("mt_forward_convolution", *args)
        else:
            call("mt_forward_convolution_func", *args, C.c_int(FUNC[func]))

    @staticmethod
    def BackwardConvolution(out, delta, kernel, kernel_x, kernel_y, kernel_z, kernel_amount, bias, stride_x, stride_y, padding_x, padding_y, func=None):
        args = (_d(out), _d(delta), _d(kernel), _i(kernel_x), _i(kernel_y), _i(kernel_z), _u(kernel_amount), _d(bias), _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y))
        if func is None:
            call("mt_backward_convolution", *args)
        else:
            call("mt_backward_convolution_func", *args, C.c_int(FUNC[func]))

    @staticmethod
    def CreateDeltaWeightAndBias(dkernel, dkernel_x, dkernel_y, dkernel_z, dkernel_amount, dbias, image, delta, stride_x, stride_y, padding_x, padding_y):
        call("mt_create_delta_weight_and_bias", _d(dkernel), _i(dkernel_x), _i(dkernel_y), _i(dkernel_z), _u(dkernel_amount), _d(dbias), _d(image), _d(delta),
             _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y))

    @staticmethod
    def CreateBackDeltaWeightAndBias(dkernel, dkernel_x, dkernel_y, dkernel_z, dkernel_amount, dbias, image, delta, stride_x, stride_y, padding_x, padding_y):
        call("mt_create_back_delta_weight_and_bias", _d(dkernel), _i(dkernel_x), _i(dkernel_y), _i(dkernel_z), _u(dkernel_amount), _d(dbias), _d(image), _d(delta),
             _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y))


class CTensorMath:
    @staticmethod
    def Fill(out, value=0.0):
        call("mt_fill", _d(out), _f(value))

    @staticmethod
    def Inv(out, inp):
        call("mt_inv", _d(out), _d(inp))

    @staticmethod
    def Div(out, left, right, left_scale=1.0, right_scale=1.0):
        call("mt_div", _d(out), _d(left), _d(right), _f(left_scale), _f(right_scale))

    @staticmethod
    def Add(out, left, right, left_scale=1.0, right_scale=1.0):
        call("mt_add", _d(out), _d(left), _d(right), _f(left_scale), _f(right_scale))

    @staticmethod
    def Sub(out, left, right, left_scale=1.0, right_scale=1.0):
        call("mt_sub", _d(out), _d(left), _d(right), _f(left_scale), _f(right_scale))

    @staticmethod
    def AddSumW(out, left, right, left_scale=1.0, right_scale=1.0):
        call("mt_add_sum_w", _d(out), _d(left), _d(right), _f(left_scale), _f(right_scale))

    @staticmethod
    def AddValue(out, inp, tensor_scale, value):
        call("mt_add_value", _d(out), _d(inp), _f(tensor_scale), _f(value))

    @staticmethod
    def SubValue(out, inp, tensor_scale, value):
        call("mt_sub_value", _d(out), _d(inp), _f(tensor_scale), _f(value))

    @staticmethod
    def Set(out, inp, scale=1.0, add_value=0.0):
        call("mt_set", _d(out), _d(inp), _f(scale), _f(add_value))

    @staticmethod
    def Pow2(out, inp, scale=1.0):
        call("mt_pow2", _d(out), _d(inp), _f(scale))

    @staticmethod
    def SQRT(out, inp, scale, add_sqrt_value):
        call("mt_sqrt", _d(out), _d(inp), _f(scale), _f(add_sqrt_value))

    @staticmethod
    def AddBias(working, bias):
        call("mt_add_bias", _d(working), _d(bias))

    @staticmethod
    def SummXY(out, inp):
        call("mt_summ_xy", _d(out), _d(inp))

    @staticmethod
    def Mul(out, left, right):
        """Tensor * tensor, or tensor * scalar / scalar * tensor (the reference overloads Mul the same way)."""
        if isinstance(right, (int, float)):
            call("mt_mul_value", _d(out), _d(left), _f(right))
        elif isinstance(left, (int, float)):
            call("mt_mul_value", _d(out), _d(right), _f(left))
        else:
            call("mt_mul", _d(out), _d(left), _d(right))

    @staticmethod
    def TransponseMul(out, left, right):
        call("mt_transponse_mul", _d(out), _d(left), _d(right))

    @staticmethod
    def Transponse(out, inp):
        call("mt_transponse", _d(out), _d(inp))

    @staticmethod
    def TensorItemProduction(out, left, right):
        call("mt_tensor_item_production", _d(out), _d(left), _d(right))

    @staticmethod
    def UpSampling(out, inp, upsampling_x, upsampling_y):
        call("mt_upsampling", _d(out), _d(inp), _u(upsampling_x), _u(upsampling_y))

    @staticmethod
    def DownSampling(out, inp, downsampling_x, downsampling_y):
        call("mt_downsampling", _d(out), _d(inp), _u(downsampling_x), _u(downsampling_y))

    @staticmethod
    def MaxPooling(out, position, inp, pooling_x, pooling_y):
        call("mt_max_pooling", _d(out), _d(position), _d(inp), _u(pooling_x), _u(pooling_y))

    @staticmethod
    def MaxPoolingBackward(out, position, inp, pooling_x, pooling_y):
        call("mt_max_pooling_backward", _d(out), _d(position), _d(inp), _u(pooling_x), _u(pooling_y))

    @staticmethod
    def Clip(tensor, min_value, max_value):
        call("mt_clip", _d(tensor), _f(min_value), _f(max_value))

    @staticmethod
    def Signum(tensor):
        call("mt_signum", _d(tensor))

    @staticmethod
    def Adam(weight, dweight, m, v, batch_size, speed, beta1, beta2, epsilon, iteration):
        call("mt_adam", _d(weight), _d(dweight), _d(m), _d(v), _u(batch_size), C.c_double(speed), C.c_double(beta1), C.c_double(beta2),
             C.c_double(epsilon), C.c_double(iteration))


    # ---- functions of the reference's GPU class only (cuda/ctensormath.cu.h:92-93, 128-134); seeds are explicit here
    @staticmethod
    def ConcatecationZ(out, a, b):
        call("mt_concatecation_z", _d(out), _d(a), _d(b))

    @staticmethod
    def SplitZ(out_a, out_b, inp):
        call("mt_split_z", _d(out_a), _d(out_b), _d(inp))

    @staticmethod
    def SetTimeStep(out, inp, time_step):
        call("mt_set_time_step", _d(out), _d(inp), _d(time_step))

    @staticmethod
    def CreateDropOutMatrix(out, drop_out, seed):
        call("mt_create_drop_out_matrix", _d(out), _f(drop_out), C.c_uint64(seed))

    @staticmethod
    def SetNormalNoise(out, seed):
        call("mt_set_normal_noise", _d(out), C.c_uint64(seed))

    @staticmethod
    def GetNoiseImageAndNoise(noisy_image, noise, image, sqrt_alpha_bar, sqrt_one_minus_alpha_bar, seed):
        call("mt_get_noise_image_and_noise", _d(noisy_image), _d(noise), _d(image), _d(sqrt_alpha_bar), _d(sqrt_one_minus_alpha_bar), C.c_uint64(seed))


class CTensorApplyFunc:
    @staticmethod
    def Apply(out, inp, func, differential=False):
        call("mt_apply_func", _d(out), _d(inp), C.c_int(FUNC[func] + (DIFFERENTIAL if differential else 0)))


for _name, _key in (("Sigmoid", "sigmoid"), ("ReLU", "relu"), ("GeLU", "gelu"), ("LeakyReLU", "leaky_relu"), ("Linear", "linear"), ("Tangence", "tangence")):
    setattr(CTensorApplyFunc, "Apply" + _name, staticmethod(lambda out, inp, k=_key: CTensorApplyFunc.Apply(out, inp, k)))
    setattr(CTensorApplyFunc, "ApplyDifferential" + _name, staticmethod(lambda out, inp, k=_key: CTensorApplyFunc.Apply(out, inp, k, True)))


class Fused:
    """The fused layer entry points of the C ABI (one reference layer Forward() each)."""

    @staticmethod
    def LinearForward(out, weight, inp, bias, func=None):
        call("mt_linear_forward_func", _d(out), _d(weight), _d(inp), _d(bias), C.c_int(FUNC[func]))

    @staticmethod
    def LinearBatchNormForwardTrain(out, weight, inp, bias, gamma, beta, linear_output=None, xhat=None, ivar=None, batch_mean=None, batch_var=None,
                                    new_mean=None, new_variable=None, momentum=0.9, epsilon=1e-6, func=None):
        """Linear layer, batch normalisation in training mode and function layer in one launch (batches of at most 256;
        larger ones run as the two calls inside the library)."""
        opt = lambda t: _d(t) if t is not None else None
        call("mt_linear_batchnorm_forward_func", _d(out), _d(weight), _d(inp), _d(bias), _d(gamma), _d(beta), opt(linear_output), opt(xhat), opt(ivar),
             opt(batch_mean), opt(batch_var), opt(new_mean), opt(new_variable), _f(momentum), _f(epsilon), C.c_int(FUNC[func]))

    @staticmethod
    def BatchNormForwardTrain(out, inp, gamma, beta, xhat=None, ivar=None, batch_mean=None, batch_var=None, new_mean=None, new_variable=None,
                              momentum=0.9, epsilon=1e-6, func=None, old_mean=None, old_variable=None, pre_function=None):
        """old_mean / old_variable: the running statistics are blended from these tensors into new_mean / new_variable;
        pre_function: gamma*xhat+beta is written there beside func of it."""
        opt = lambda t: _d(t) if t is not None else None
        if old_mean is not None or old_variable is not None or pre_function is not None:
            return call("mt_batchnorm_forward_train_from", _d(out), _d(inp), _d(gamma), _d(beta), opt(xhat), opt(ivar), opt(batch_mean), opt(batch_var),
                        opt(new_mean), opt(new_variable), opt(old_mean), opt(old_variable), _f(momentum), _f(epsilon), C.c_int(FUNC[func]), opt(pre_function))
        call("mt_batchnorm_forward_train_func", _d(out), _d(inp), _d(gamma), _d(beta), opt(xhat), opt(ivar), opt(batch_mean), opt(batch_var),
             opt(new_mean), opt(new_variable), _f(momentum), _f(epsilon), C.c_int(FUNC[func]))

    @staticmethod
    def BatchNormForwardTrainNoAlloc(out, inp, gamma, beta, xhat=None, ivar=None, batch_mean=None, batch_var=None, new_mean=None, new_variable=None,
                                     momentum=0.9, epsilon=1e-6, func=None):
        """The same call through the entry point that allocates nothing (statistics in the library's fixed array)."""
        opt = lambda t: _d(t) if t is not None else None
        call("mt_batchnorm_forward_train_func_noalloc", _d(out), _d(inp), _d(gamma), _d(beta), opt(xhat), opt(ivar), opt(batch_mean), opt(batch_var),
             opt(new_mean), opt(new_variable), _f(momentum), _f(epsilon), C.c_int(FUNC[func]))

    @staticmethod
    def VaeCoderOutput(out, kl_loss, mu, logvar, epsilon):
        call("mt_vae_coder_output", _d(out), _d(kl_loss) if kl_loss is not None else None, _d(mu), _d(logvar), _d(epsilon))

    @staticmethod
    def BatchNormBackward(error, dgamma, dbeta, delta, gamma, xhat, ivar, beta=None, func=None):
        """func: the function the forward pass applied to gamma*xhat+beta (`delta` is the gradient behind it)."""
        opt = lambda t: _d(t) if t is not None else None
        if func is None:
            call("mt_batchnorm_backward", _d(error), opt(dgamma), opt(dbeta), _d(delta), _d(gamma), _d(xhat), _d(ivar))
        else:
            call("mt_batchnorm_backward_func", _d(error), opt(dgamma), opt(dbeta), _d(delta), _d(gamma), opt(beta), _d(xhat), _d(ivar), C.c_int(FUNC[func]))

    @staticmethod
    def BatchNormBackwardKeep(error, dgamma, dbeta, delta, gamma, xhat, ivar, dxhat=None, sum_dxhat=None, sum_dxhat_xhat=None):
        """The backward pass that also leaves the intermediate tensors of the layer's own sequence."""
        opt = lambda t: _d(t) if t is not None else None
        call("mt_batchnorm_backward_keep", _d(error), opt(dgamma), opt(dbeta), _d(delta), _d(gamma), _d(xhat), _d(ivar), opt(dxhat), opt(sum_dxhat), opt(sum_dxhat_xhat))

    @staticmethod
    def BatchNormBackwardFuncKeep(error, dgamma, dbeta, delta, gamma, beta, xhat, ivar, func, dxhat=None, sum_dxhat=None, sum_dxhat_xhat=None, delta_front=None):
        """The function layer's backward step and the batch-norm layer's backward pass in one kernel, leaving what both sequences leave."""
        opt = lambda t: _d(t) if t is not None else None
        call("mt_batchnorm_backward_func_keep", _d(error), opt(dgamma), opt(dbeta), _d(delta), _d(gamma), opt(beta), _d(xhat), _d(ivar), C.c_int(FUNC[func]),
             opt(dxhat), opt(sum_dxhat), opt(sum_dxhat_xhat), opt(delta_front))

    @staticmethod
    def UpSamplingConvolution(out, image, upsampling_x, upsampling_y, kernel, kernel_x, kernel_y, kernel_z, kernel_amount, bias, stride_x, stride_y,
                              padding_x, padding_y, func=None):
        call("mt_upsampling_convolution_func", _d(out), _d(image), _u(upsampling_x), _u(upsampling_y), _d(kernel), _i(kernel_x), _i(kernel_y), _i(kernel_z),
             _u(kernel_amount), _d(bias), _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y), C.c_int(FUNC[func]))

    @staticmethod
    def BackwardConvolutionNorm(out, delta, delta_scale_shift, delta_func, kernel, kernel_x, kernel_y, kernel_z, kernel_amount, bias, stride_x, stride_y,
                                padding_x, padding_y, func=None, bn=None):
        """A transposed convolution whose input still owes func(scale*x+shift) (delta_scale_shift may be None).  With
        `bn` (a dict: gamma, beta, scale_shift and optionally ivar, batch_mean, batch_var, new_mean, new_variable, momentum,
        epsilon) the statistics of the output for the batch normalisation that follows are produced as well."""
        opt = lambda t: _d(t) if t is not None else None
        head = (_d(out), _d(delta), opt(delta_scale_shift), C.c_int(FUNC[delta_func]), _d(kernel), _i(kernel_x), _i(kernel_y), _i(kernel_z), _u(kernel_amount),
                _d(bias), _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y))
        if bn is None:
            call("mt_backward_convolution_norm_func", *head, C.c_int(FUNC[func]))
        else:
            g = bn.get
            call("mt_backward_convolution_norm_stats", *head, _d(bn["gamma"]), _d(bn["beta"]), _d(bn["scale_shift"]), opt(g("ivar")), opt(g("batch_mean")),
                 opt(g("batch_var")), opt(g("new_mean")), opt(g("new_variable")), _f(g("momentum", 0.9)), _f(g("epsilon", 1e-6)))

    @staticmethod
    def FillMany(tensors, value):
        call("mt_fill_many", _u(len(tensors)), _list(tensors), _f(value))

    @staticmethod
    def AdamMany(weights, dweights, ms, vs, batch_size, speed, beta1, beta2, epsilon, iteration):
        call("mt_adam_many", _u(len(weights)), _list(weights), _list(dweights), _list(ms), _list(vs), _u(batch_size), C.c_double(speed),
             C.c_double(beta1), C.c_double(beta2), C.c_double(epsilon), C.c_double(iteration))

    @staticmethod
    def ConvolutionBackwardWeightsSum(dkernel, dkernel_x, dkernel_y, dkernel_z, dkernel_amount, dbias, image, delta, stride_x, stride_y, padding_x, padding_y):
        call("mt_convolution_backward_weights_sum", _d(dkernel), _i(dkernel_x), _i(dkernel_y), _i(dkernel_z), _u(dkernel_amount), _d(dbias), _d(image),
             _d(delta), _i(stride_x), _i(stride_y), _i(padding_x), _i(padding_y))

    @staticmethod
    def BatchNormForwardInfer(out, inp, gamma, beta, mean, variable, epsilon=1e-6, func=None):
        call("mt_batchnorm_forward_infer_func", _d(out), _d(inp), _d(gamma), _d(beta), _d(mean), _d(variable), _f(epsilon), C.c_int(FUNC[func]))


def exported_symbols():
    """Names declared in include/mi355_tensor.h (used by the CPU-side ABI test)."""
    import re
    header = open(os.path.join(HERE, "..", "include", "mi355_tensor.h")).read()
    return sorted(set(re.findall(r"\b(mt_[a-z0-9_]+)\s*\(", header)))
