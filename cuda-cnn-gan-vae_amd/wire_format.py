"""The reference's checkpoint wire format, read and written from Python.

A stream is a sequence of host-endian values without framing (common/cdatastreamfile.cpp: Save<T> / Load<T> copy
the bytes of T).  What the layers put into it:

    tensor               4 x uint32 (W, Z, Y, X), then W*Z*Y*X doubles          cuda/ctensor.cu.h:525-571
    convolution layer    8 x int32 (kernel amount, kernel x, y, z, stride x, y, padding x, y), kernel tensor
                         [1,1,amount,z*y*x], bias tensor [1,amount,1,1]        netlayer/cnetlayerconvolution.cu.h:351-400
    transposed conv.     the same header and tensors (kernel rows = input channels)  netlayer/cnetlayerbackconvolution.cu.h
    linear layer         weight tensor [1,1,out,in], bias tensor [1,1,out,1]    netlayer/cnetlayerlinear.cu.h:309-327
    batch normalisation  beta, gamma, mean, variable tensors [1,Z,Y,X], momentum as one double
                                                                                netlayer/cnetlayerbatchnormalization.cu.h:409-417

Values are float32 in memory and double on the wire: writing and reading back is exact.
"""
import struct

import numpy as np

CONV_HEADER = ("kernel_amount", "kernel_x", "kernel_y", "kernel_z", "stride_x", "stride_y", "padding_x", "padding_y")


def read_tensor(f):
    head = f.read(16)
    if len(head) != 16:
        raise EOFError("stream ends inside a tensor header")
    w, z, y, x = struct.unpack("=4I", head)
    n = w * z * y * x
    data = f.read(8 * n)
    if len(data) != 8 * n:
        raise EOFError("stream ends inside a tensor of [%d,%d,%d,%d]" % (w, z, y, x))
    return np.frombuffer(data, dtype=np.float64).astype(np.float32).reshape(w, z, y, x)


def write_tensor(f, a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    assert a.ndim == 4, "tensors are [W,Z,Y,X]"
    f.write(struct.pack("=4I", *a.shape))
    f.write(a.astype(np.float64).tobytes())


def read_convolution_layer(f):
    """Returns (header dict, kernel, bias)."""
    raw = f.read(32)
    if len(raw) != 32:
        raise EOFError("stream ends inside a convolution header")
    values = struct.unpack("=I7i", raw)          # the amount is written as int32 and read back as uint32
    return dict(zip(CONV_HEADER, values)), read_tensor(f), read_tensor(f)


def write_convolution_layer(f, header, kernel, bias):
    f.write(struct.pack("=I7i", *(int(header[k]) for k in CONV_HEADER)))
    write_tensor(f, kernel)
    write_tensor(f, bias)


def read_linear_layer(f):
    """Returns (weight [1,1,out,in], bias [1,1,out,1])."""
    return read_tensor(f), read_tensor(f)


def write_linear_layer(f, weight, bias):
    write_tensor(f, weight)
    write_tensor(f, bias)


def read_batchnorm_layer(f):
    """Returns (beta, gamma, mean, variable, momentum)."""
    tensors = [read_tensor(f) for _ in range(4)]
    raw = f.read(8)
    if len(raw) != 8:
        raise EOFError("stream ends before the momentum")
    return tuple(tensors) + (struct.unpack("=d", raw)[0],)


def write_batchnorm_layer(f, beta, gamma, mean, variable, momentum):
    for t in (beta, gamma, mean, variable):
        write_tensor(f, t)
    f.write(struct.pack("=d", float(momentum)))


# Whole networks.  CModelMain::SaveNetLayers (cuda/netmodel/cmodelmain.cu.h:296-300) calls Save() of every layer in
# order, with nothing between them; what the other layer kinds write:
#     function                 uint32 id of netlayer/neuron.cu.h:21-26 (not the id of the tensor-level function)
#     up-sampling, max pooling, max de-pooling, average pooling      2 x uint32 (x, y)
#     drop-out                 one double
#     input, time embedding, concatenator, splitter, VAE coder output, soft-max      nothing
NEURON_FUNCTION = {"sigmoid": 0, "relu": 1, "leaky_relu": 2, "linear": 3, "tangence": 4, "gelu": 5}
_NEURON_NAME = {v: k for k, v in NEURON_FUNCTION.items()}
_EMPTY = ("input", "time_embedding", "concatenator", "splitter", "vae_coder_output", "softmax")
_PAIR = ("upsampling", "maxpooling", "maxdepooling", "averagepooling")


def _take(f, fmt, what):
    raw = f.read(struct.calcsize(fmt))
    if len(raw) != struct.calcsize(fmt):
        raise EOFError("stream ends inside " + what)
    return struct.unpack(fmt, raw)


def write_net(f, layers):
    """`layers`: a list of (kind, fields) in the order of the network's layer vector, e.g.
    ("convolution", {"header": {...}, "kernel": a, "bias": b}), ("batchnorm", {"beta":…, "gamma":…, "mean":…,
    "variable":…, "momentum": 0.9}), ("function", {"name": "leaky_relu"}), ("upsampling", {"x": 2, "y": 2}),
    ("linear", {"weight":…, "bias":…}), ("dropout", {"rate": 0.3}), ("input", {})."""
    for kind, p in layers:
        if kind in ("convolution", "backconvolution"):
            write_convolution_layer(f, p["header"], p["kernel"], p["bias"])
        elif kind == "linear":
            write_linear_layer(f, p["weight"], p["bias"])
        elif kind == "batchnorm":
            write_batchnorm_layer(f, p["beta"], p["gamma"], p["mean"], p["variable"], p["momentum"])
        elif kind == "function":
            f.write(struct.pack("=I", NEURON_FUNCTION[p["name"]]))
        elif kind in _PAIR:
            f.write(struct.pack("=2I", int(p["x"]), int(p["y"])))
        elif kind == "dropout":
            f.write(struct.pack("=d", float(p["rate"])))
        elif kind not in _EMPTY:
            raise ValueError("unknown layer kind " + repr(kind))


def read_net(f, kinds):
    """The inverse: `kinds` names the layer kinds in order (the format carries no tags, the reader must know the
    topology, as the reference's LoadNetLayers does).  Returns the list write_net takes."""
    out = []
    for kind in kinds:
        if kind in ("convolution", "backconvolution"):
            header, kernel, bias = read_convolution_layer(f)
            p = {"header": header, "kernel": kernel, "bias": bias}
        elif kind == "linear":
            weight, bias = read_linear_layer(f)
            p = {"weight": weight, "bias": bias}
        elif kind == "batchnorm":
            beta, gamma, mean, variable, momentum = read_batchnorm_layer(f)
            p = {"beta": beta, "gamma": gamma, "mean": mean, "variable": variable, "momentum": momentum}
        elif kind == "function":
            ident = _take(f, "=I", "a function layer")[0]
            if ident not in _NEURON_NAME:
                raise ValueError("unknown neuron function %d" % ident)
            p = {"name": _NEURON_NAME[ident]}
        elif kind in _PAIR:
            x, y = _take(f, "=2I", "a " + kind + " layer")
            p = {"x": x, "y": y}
        elif kind == "dropout":
            p = {"rate": _take(f, "=d", "a drop-out layer")[0]}
        elif kind in _EMPTY:
            p = {}
        else:
            raise ValueError("unknown layer kind " + repr(kind))
        out.append((kind, p))
    return out


# Training state.  CModelMain::SaveNetLayersTrainingParam (cuda/netmodel/cmodelmain.cu.h:368-373) writes the iteration
# as one uint32, then SaveTrainingParam() of every layer in order: four tensors for the layers that Adam updates --
# first moment and second moment of the weights, then of the biases (convolution / transposed convolution: MK, VK,
# MB, VB, netlayer/cnetlayerconvolution.cu.h; linear: MW, VW, MB, VB; batch normalisation: MK, VK for gamma and MB, VB
# for beta, netlayer/cnetlayerbatchnormalization.cu.h:639-640) -- and nothing for every other kind.
_TRAINED = ("convolution", "backconvolution", "linear", "batchnorm")


def write_training_params(f, iteration, layers):
    """`layers`: a list of (kind, fields) in network order; for the kinds Adam updates the fields are "m_weight",
    "v_weight", "m_bias", "v_bias" (for batch normalisation the weight is gamma, the bias beta)."""
    f.write(struct.pack("=I", int(iteration)))
    for kind, p in layers:
        if kind in _TRAINED:
            for name in ("m_weight", "v_weight", "m_bias", "v_bias"):
                write_tensor(f, p[name])
        elif kind not in _EMPTY and kind not in _PAIR and kind not in ("function", "dropout"):
            raise ValueError("unknown layer kind " + repr(kind))


def read_training_params(f, kinds):
    """Returns (iteration, layers) as write_training_params takes them."""
    iteration = _take(f, "=I", "the iteration")[0]
    out = []
    for kind in kinds:
        if kind in _TRAINED:
            out.append((kind, {name: read_tensor(f) for name in ("m_weight", "v_weight", "m_bias", "v_bias")}))
        elif kind in _EMPTY or kind in _PAIR or kind in ("function", "dropout"):
            out.append((kind, {}))
        else:
            raise ValueError("unknown layer kind " + repr(kind))
    return iteration, out


# Averaged weights.  CModelMain::SaveNetLayersEMAWeight (cuda/netmodel/cmodelmain.cu.h:332-336) calls SaveEMAWeight() of
# every layer in order (backwards through the vector when asked to), and every layer writes the record of its Save()
# with the averaged tensors in place of the trained ones: convolution / transposed convolution the eight header values,
# Kernel_EMA, Bias_EMA (netlayer/cnetlayerconvolution.cu.h:679-692); linear W_EMA, B_EMA (cnetlayerlinear.cu.h:590-595);
# batch normalisation Beta_EMA, Gamma_EMA, Mean_EMA, Variable_EMA and the momentum (cnetlayerbatchnormalization.cu.h:
# 770-778); the other kinds what their Save() writes.  A layer whose averaging was never enabled holds [1,1,1,1] tensors
# there (EnableEMA(false), the constructors' state) and writes those.  TrainingUpdateWeight blends
# ema = EMA_K * ema + (1 - EMA_K) * weight with EMA_K = 0.999 (netlayer/inetlayer.cu.h:67) after every step.
EMA_K = 0.999


def write_ema(f, layers, backward=False):
    """`layers` as write_net takes them, the tensor fields holding the averaged weights."""
    write_net(f, list(reversed(layers)) if backward else layers)


def read_ema(f, kinds, backward=False):
    """Returns the layers in network order, whichever way the stream was written."""
    if not backward:
        return read_net(f, kinds)
    return list(reversed(read_net(f, list(reversed(kinds)))))


def ema_disabled(kind):
    """The fields a layer of this kind writes when its averaging was never enabled (for write_ema)."""
    one = np.zeros((1, 1, 1, 1), np.float32)
    if kind in ("convolution", "backconvolution"):
        return {"kernel": one, "bias": one}
    if kind == "linear":
        return {"weight": one, "bias": one}
    if kind == "batchnorm":
        return {"beta": one, "gamma": one, "mean": one, "variable": one}
    return {}
