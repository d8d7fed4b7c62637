"""Convolutional VAE forward pass (encoder, reparameterisation, decoder) on device-resident tensors, as a stack of the
reference's layers through the fused C-ABI entry points.

    image [B,3,128,128]
    -> conv 3x3 stride 2 padding 1, 3 -> 32 -> 64 -> 128 -> 256, each followed by BatchNorm (batch statistics) and
       leaky ReLU                [CNetLayerConvolution, CNetLayerBatchNormalization, CNetLayerFunction]
    -> two Linear heads 256*8*8 -> latent: mean and log-variance          [CNetLayerLinear]
    -> z = mu + exp(clamp(logvar, +-10) / 2) * eps, KL loss               [CNetLayerVAECoderOutput,
                                                                            netlayer/cnetlayervaecoderoutput.cu.h:244-287]
    -> Linear latent -> 256*8*8, leaky ReLU, viewed [B,256,8,8]
    -> transposed conv 4x4 stride 2 padding 1, 256 -> 128 -> 64 -> 32 -> 3, leaky ReLU between, sigmoid at the end
                                 [CNetLayerBackConvolution, netlayer/cnetlayerbackconvolution.cu.h:303-315]

The noise eps is an input (the reference draws it from a generator that cannot be seeded).
"""
import numpy as np

import mi355tensor as mt
from mi355tensor import CTensor, CTensorConv, Fused

ENCODER = (3, 32, 64, 128, 256)
DECODER = (256, 128, 64, 32, 3)
IMAGE = 128
LATENT = 128
BN_EPSILON = 1e-6
MOMENTUM = 0.9


def make_parameters(latent=LATENT, seed=4):
    """He-normal kernels, small biases, gamma in [0.5, 1.5], beta in [-0.2, 0.2], Linear biases 0.1 (the reference's
    initial value, netlayer/cnetlayerlinear.cu.h:222-226), as numpy arrays in the reference's layouts."""
    rng = np.random.default_rng(seed)
    p, size = {}, IMAGE
    for i in range(4):
        cin, cout = ENCODER[i], ENCODER[i + 1]
        size //= 2
        p["ekernel%d" % i] = (rng.standard_normal((1, 1, cout, cin * 9)) * np.sqrt(2.0 / (cin * 9))).astype(np.float32)
        p["ebias%d" % i] = (rng.standard_normal((1, cout, 1, 1)) * 0.05).astype(np.float32)
        p["egamma%d" % i] = rng.uniform(0.5, 1.5, (1, cout, size, size)).astype(np.float32)
        p["ebeta%d" % i] = rng.uniform(-0.2, 0.2, (1, cout, size, size)).astype(np.float32)
    flat = ENCODER[4] * size * size
    for head in ("mu", "lv"):
        p[head + "_w"] = (rng.standard_normal((1, 1, latent, flat)) / np.sqrt(flat)).astype(np.float32)
        p[head + "_b"] = np.full((1, 1, latent, 1), 0.1, np.float32)
    p["dec_w"] = (rng.standard_normal((1, 1, flat, latent)) / np.sqrt(latent)).astype(np.float32)
    p["dec_b"] = np.full((1, 1, flat, 1), 0.1, np.float32)
    for i in range(4):
        cin, cout = DECODER[i], DECODER[i + 1]
        # kernel of BackwardConvolution: row f = input channel, column z*16 + i*4 + j (cpu/ctensorconv.h:256)
        p["dkernel%d" % i] = (rng.standard_normal((1, 1, cin, cout * 16)) * np.sqrt(1.0 / (cin * 4))).astype(np.float32)
        p["dbias%d" % i] = np.zeros((1, cin, 1, 1), np.float32)
    return p


def make_batch(batch, seed=4):
    """Images uniform in [0, 1] and standard normal noise for the latent."""
    rng = np.random.default_rng(seed + 1000)
    return rng.uniform(0.0, 1.0, (batch, 3, IMAGE, IMAGE)).astype(np.float32), rng.standard_normal((batch, 1, LATENT, 1)).astype(np.float32)


def flops(batch):
    """Algorithmic FLOPs (2*MAC, non-zero taps only): encoder convolutions, the three Linear layers, decoder transposed
    convolutions."""
    enc, dec, size = 0.0, 0.0, IMAGE
    for i in range(4):
        size //= 2
        enc += 2.0 * batch * ENCODER[i + 1] * size * size * ENCODER[i] * 9
    flat = ENCODER[4] * size * size
    lin = 2.0 * batch * flat * LATENT * 3
    for i in range(4):
        dec += 2.0 * batch * DECODER[i] * size * size * DECODER[i + 1] * 16
        size *= 2
    return {"encoder_conv": enc, "linear": lin, "decoder_tconv": dec}


class Vae:
    def __init__(self, batch, params=None):
        mt.init(0)
        self.batch = b = batch
        host = params or make_parameters()
        self.p = {k: CTensor.from_numpy(v) for k, v in host.items()}
        self.x, self.eps = CTensor(b, 3, IMAGE, IMAGE), CTensor(b, 1, LATENT, 1)
        self.ec, self.eh, size = [], [], IMAGE
        for i in range(4):
            size //= 2
            self.ec.append(CTensor(b, ENCODER[i + 1], size, size))
            self.eh.append(CTensor(b, ENCODER[i + 1], size, size))
        self.mu, self.logvar, self.z, self.kl = CTensor(b, 1, LATENT, 1), CTensor(b, 1, LATENT, 1), CTensor(b, 1, LATENT, 1), CTensor(1, 1, 1, 1)
        self.dh = [CTensor(b, DECODER[0], size, size)]
        for i in range(4):
            size *= 2
            self.dh.append(CTensor(b, DECODER[i + 1], size, size))
        self.dec_flat = self.dh[0].reinterpret(b, 1, DECODER[0] * 64, 1)

    def set_batch(self, images, eps):
        self.x.upload(images)
        self.eps.upload(eps)

    @property
    def output(self):
        return self.dh[4]

    def forward(self):
        # batch norm in training mode (batch statistics); running statistics are not kept here: a forward pass without a
        # weight update leaves the reference's Mean / Variable unchanged too (its NewMean is reset from Mean,
        # netlayer/cnetlayerbatchnormalization.cu.h:620-621)
        p, h = self.p, self.x
        for i in range(4):
            CTensorConv.ForwardConvolution(self.ec[i], h, p["ekernel%d" % i], 3, 3, ENCODER[i], ENCODER[i + 1], p["ebias%d" % i], 2, 2, 1, 1)
            Fused.BatchNormForwardTrain(self.eh[i], self.ec[i], p["egamma%d" % i], p["ebeta%d" % i], momentum=MOMENTUM, epsilon=BN_EPSILON, func="leaky_relu")
            h = self.eh[i]
        Fused.LinearForward(self.mu, p["mu_w"], h, p["mu_b"])
        Fused.LinearForward(self.logvar, p["lv_w"], h, p["lv_b"])
        Fused.VaeCoderOutput(self.z, self.kl, self.mu, self.logvar, self.eps)
        Fused.LinearForward(self.dec_flat, p["dec_w"], self.z, p["dec_b"], "leaky_relu")
        for i in range(4):
            CTensorConv.BackwardConvolution(self.dh[i + 1], self.dh[i], p["dkernel%d" % i], 4, 4, DECODER[i + 1], DECODER[i], p["dbias%d" % i], 2, 2, 1, 1,
                                            func="leaky_relu" if i < 3 else "sigmoid")
        return self.dh[4]
