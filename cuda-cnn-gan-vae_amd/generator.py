"""DCGAN-64 generator forward pass as the reference's layers would run it, on device-resident tensors.

Layer stack (the reference's layer classes in brackets):
    latent [B,1,100,1]
    -> Linear 100 -> 512*4*4              [CNetLayerLinear, netlayer/cnetlayerlinear.cu.h:262-282]
    -> BatchNorm (batch statistics) + ReLU [CNetLayerBatchNormalization :268-380, CNetLayerFunction :203-213]
    -> transposed conv 4x4 s2 p1, 512 -> 256 -> 128 -> 64, each followed by BatchNorm + ReLU
                                           [CNetLayerBackConvolution, netlayer/cnetlayerbackconvolution.cu.h:303-315]
    -> transposed conv 4x4 s2 p1, 64 -> 3, tanh -> images [B,3,64,64]

Batch-norm statistics are per element (z,y,x) over the batch axis, as in the reference.
`forward_fused` uses the fused C-ABI entry points (one or two launches per layer); `forward_literal`
issues the reference layers' exact op sequences, one C-ABI call per tensor op.
"""
import numpy as np

import mi355tensor as mt
from mi355tensor import CTensor, CTensorApplyFunc, CTensorConv, CTensorMath, Fused

LATENT = 100
CHANNELS = (512, 256, 128, 64, 3)
BN_EPSILON = 1e-6
MOMENTUM = 0.9
FOLD = (3,)
FUSE_LINEAR_BN = False


def make_parameters(seed=3, std=0.02):
    """Random-init parameters (N(0, std)), biases 0, gamma 1, beta 0, as numpy arrays in the reference's layouts."""
    rng = np.random.default_rng(seed)
    p = {"lin_w": (rng.standard_normal((1, 1, CHANNELS[0] * 16, LATENT)) * std).astype(np.float32),
         "lin_b": np.zeros((1, 1, CHANNELS[0] * 16, 1), np.float32)}
    size = 4
    for i in range(4):
        cin, cout = CHANNELS[i], CHANNELS[i + 1]
        p["gamma%d" % i] = np.ones((1, cin, size, size), np.float32)
        p["beta%d" % i] = np.zeros((1, cin, size, size), np.float32)
        # kernel of BackwardConvolution: row f = input channel, column z*16 + i*4 + j (cpu/ctensorconv.h:256)
        p["kernel%d" % i] = (rng.standard_normal((1, 1, cin, cout * 16)) * std).astype(np.float32)
        p["bias%d" % i] = np.zeros((1, cin, 1, 1), np.float32)
        size *= 2
    return p


def make_latent(batch, seed=3):
    return np.random.default_rng(seed + 1000).standard_normal((batch, 1, LATENT, 1)).astype(np.float32)


def conv_flops(batch):
    """Algorithmic FLOPs (2*MAC, non-zero taps only) of the four transposed convolutions, per layer."""
    out, size = [], 4
    for i in range(4):
        out.append(2.0 * batch * CHANNELS[i] * size * size * CHANNELS[i + 1] * 16)
        size *= 2
    return out


class DcganGenerator:
    def __init__(self, batch, params=None):
        mt.init(0)
        self.batch = batch
        host = params or make_parameters()
        self.p = {k: CTensor.from_numpy(v) for k, v in host.items()}
        b = batch
        self.latent = CTensor(b, 1, LATENT, 1)
        self.h = [CTensor(b, CHANNELS[0], 4, 4)]            # pre-normalisation activations
        self.a = []                                          # post BN+ReLU activations
        size = 4
        for i in range(4):
            self.a.append(CTensor(b, CHANNELS[i], size, size))
            size *= 2
            self.h.append(CTensor(b, CHANNELS[i + 1], size, size))
        self.lin_out = self.h[0].reinterpret(b, 1, CHANNELS[0] * 16, 1)
        self.literal_tmp = None
        # (scale, shift) pairs of the batch normalisations that are folded into the convolutions around them
        self.pairs = [CTensor(1, CHANNELS[i], 4 << i, 2 * (4 << i)) for i in range(4)]
        # Which batch normalisations forward_fused folds: i in FOLD means layer i's statistics come from the epilogue of
        # the transposed convolution in front of it and its normalisation + ReLU happen in the loader of the one behind
        # it.  Measured per layer on an MI355X at batch 256; the others keep the one-pass batch-norm kernel.
        self.fold = FOLD
        # forward_fused can run the Linear layer and its batch norm as one launch (the Linear layer's own output h[0] is
        # then written only when somebody wants to look at it) or as two
        self.fuse_linear_bn = FUSE_LINEAR_BN
        self.keep_linear_output = False

    def set_latent(self, z):
        self.latent.upload(z)

    @property
    def output(self):
        return self.h[4]

    def activation(self, i):
        """Output of batch norm i + ReLU as a numpy array: the tensor itself, or -- when the layer is folded and the tensor
        never exists on the device -- what the consuming convolution computes from the raw activation and the pairs."""
        if i in self.fold and i > 0:
            pairs = self.pairs[i].numpy().reshape(1, CHANNELS[i], 4 << i, 4 << i, 2)
            return np.maximum(pairs[..., 0] * self.h[i].numpy() + pairs[..., 1], np.float32(0))
        return self.a[i].numpy()

    def forward_fused(self):
        """One or two launches per layer.  Batch norm 0 sits in the epilogue of the Linear layer's product (a block holds
        the whole batch of its features); a batch norm i in self.fold never writes its output: the convolution in front of
        it leaves the raw activation h[i] and the pairs (scale, shift), the convolution behind it normalises as it loads.
        Running statistics: this class measures the forward pass in training mode and keeps none (no new_mean /
        new_variable is passed; the reference's layer would blend its NewMean / NewVariable here and, without a weight update
        behind the pass, discard the blend at its next reset, netlayer/cnetlayerbatchnormalization.cu.h:620-621)."""
        p = self.p
        if self.fuse_linear_bn:
            Fused.LinearBatchNormForwardTrain(self.a[0], p["lin_w"], self.latent, p["lin_b"], p["gamma0"], p["beta0"],
                                              linear_output=self.lin_out if self.keep_linear_output else None,
                                              momentum=MOMENTUM, epsilon=BN_EPSILON, func="relu")
        else:
            Fused.LinearForward(self.lin_out, p["lin_w"], self.latent, p["lin_b"], None)
            Fused.BatchNormForwardTrain(self.a[0], self.h[0], p["gamma0"], p["beta0"], momentum=MOMENTUM, epsilon=BN_EPSILON, func="relu")
        for i in range(4):
            folded, next_folded = i in self.fold and i > 0, (i + 1) in self.fold and i < 3
            if not folded and i > 0:
                Fused.BatchNormForwardTrain(self.a[i], self.h[i], p["gamma%d" % i], p["beta%d" % i], momentum=MOMENTUM, epsilon=BN_EPSILON, func="relu")
            if not folded and not next_folded:
                CTensorConv.BackwardConvolution(self.h[i + 1], self.a[i], p["kernel%d" % i], 4, 4, CHANNELS[i + 1], CHANNELS[i], p["bias%d" % i], 2, 2, 1, 1,
                                                func="tangence" if i == 3 else None)
                continue
            bn = dict(gamma=p["gamma%d" % (i + 1)], beta=p["beta%d" % (i + 1)], scale_shift=self.pairs[i + 1], momentum=MOMENTUM,
                      epsilon=BN_EPSILON) if next_folded else None
            Fused.BackwardConvolutionNorm(self.h[i + 1], self.h[i] if folded else self.a[i], self.pairs[i] if folded else None, "relu" if folded else None,
                                          p["kernel%d" % i], 4, 4, CHANNELS[i + 1], CHANNELS[i], p["bias%d" % i], 2, 2, 1, 1,
                                          func="tangence" if i == 3 else None, bn=bn)
        return self.h[4]

    def forward_literal(self):
        """Every layer as the reference issues it: Mul + Add; the 11 tensor ops of a training-mode batch norm;
        ApplyReLU; BackwardConvolution; ApplyTangence."""
        p = self.p
        if self.literal_tmp is None:
            self.literal_tmp = []
            for i in range(4):
                s = self.h[i].shape
                one = (1,) + s[1:]
                self.literal_tmp.append(dict(mean=CTensor(*one), var=CTensor(*one), sqrtvar=CTensor(*one), ivar=CTensor(*one),
                                             xhat=CTensor(*s), tmp=CTensor(*s), bn=CTensor(*s)))
        CTensorMath.Mul(self.lin_out, p["lin_w"], self.latent)
        CTensorMath.Add(self.lin_out, self.lin_out, p["lin_b"])
        inv_n = float(np.float32(1.0 / np.float64(np.float32(self.batch))))
        for i in range(4):
            t, x = self.literal_tmp[i], self.h[i]
            CTensorMath.Fill(t["mean"], 0)
            CTensorMath.AddSumW(t["mean"], t["mean"], x, 1, inv_n)
            CTensorMath.Sub(t["xhat"], x, t["mean"], 1.0, 1.0)
            CTensorMath.Fill(t["var"], 0)
            CTensorMath.Pow2(t["tmp"], t["xhat"], 1)
            CTensorMath.AddSumW(t["var"], t["var"], t["tmp"], 1, inv_n)
            CTensorMath.SQRT(t["sqrtvar"], t["var"], 1, BN_EPSILON)
            CTensorMath.Inv(t["ivar"], t["sqrtvar"])
            CTensorMath.TensorItemProduction(t["xhat"], t["xhat"], t["ivar"])
            CTensorMath.TensorItemProduction(t["tmp"], p["gamma%d" % i], t["xhat"])
            CTensorMath.Add(t["bn"], t["tmp"], p["beta%d" % i])
            CTensorApplyFunc.ApplyReLU(self.a[i], t["bn"])
            CTensorConv.BackwardConvolution(self.h[i + 1], self.a[i], p["kernel%d" % i], 4, 4, CHANNELS[i + 1], CHANNELS[i], p["bias%d" % i], 2, 2, 1, 1)
        CTensorApplyFunc.ApplyTangence(self.h[4], self.h[4])
        return self.h[4]
