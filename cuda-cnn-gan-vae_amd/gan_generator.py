"""The generator of the reference's own GAN model (cuda/netmodel/cmodel_gan.cu.h:121-200) on device-resident tensors:

    noise [B,1,N,1]
    -> Linear N -> 3*4*C0, leaky ReLU, viewed [B,C0,3,4]                [CNetLayerLinear, CNetLayerFunction]
    -> six times: up-sampling x2, convolution 3x3 stride 1 padding 1, BatchNorm (batch statistics), leaky ReLU
                                                                         [CNetLayerUpSampling, CNetLayerConvolution,
                                                                          CNetLayerBatchNormalization, CNetLayerFunction]
    -> convolution 3x3 to the image depth, tanh -> images [B,3,192,256]

The shipped model: N = 1024, C0 = 512, widths 512, 256, 128, 64, 32, 16, batch 32.
`forward(fused=False)` issues the layers one after the other (up-sampled image written, then read by the convolution);
`forward(fused=True)` uses the entry point that computes the convolution of the up-sampled image from the input itself.
"""
import numpy as np

import mi355tensor as mt
from mi355tensor import CTensor, CTensorConv, CTensorMath, Fused

NOISE = 1024
CHANNELS = (512, 512, 256, 128, 64, 32, 16)   # C0, then the six convolution widths
IMAGE_DEPTH = 3
BATCH = 32
BN_EPSILON = 1e-6
MOMENTUM = 0.9


def make_parameters(channels=CHANNELS, noise=NOISE, seed=6):
    """He-normal kernels, small biases, gamma in [0.5, 1.5], beta in [-0.2, 0.2], as numpy arrays in the reference's layouts.
    Names: lin_w, lin_b, kernel0..6, bias0..6, gamma0..5, beta0..5."""
    rng = np.random.default_rng(seed)
    p = {"lin_w": (rng.standard_normal((1, 1, 12 * channels[0], noise)) * (0.1 * np.sqrt(64.0 / noise))).astype(np.float32),
         "lin_b": np.full((1, 1, 12 * channels[0], 1), 0.1, np.float32)}
    size, widths = (3, 4), tuple(channels[1:]) + (IMAGE_DEPTH,)
    for i in range(7):
        cin, cout = (channels[0] if i == 0 else widths[i - 1]), widths[i]
        p["kernel%d" % i] = (rng.standard_normal((1, 1, cout, cin * 9)) * np.sqrt(2.0 / (cin * 9))).astype(np.float32)
        p["bias%d" % i] = (rng.standard_normal((1, cout, 1, 1)) * 0.05).astype(np.float32)
        if i < 6:
            size = (size[0] * 2, size[1] * 2)
            p["gamma%d" % i] = rng.uniform(0.5, 1.5, (1, cout) + size).astype(np.float32)
            p["beta%d" % i] = rng.uniform(-0.2, 0.2, (1, cout) + size).astype(np.float32)
    return p


def make_statistics(channels=CHANNELS):
    """Running mean and variable of the six batch-norm layers as a fresh layer holds them
    (Reset, netlayer/cnetlayerbatchnormalization.cu.h:239-240): 0 and 1."""
    s, size = {}, (3, 4)
    for i in range(6):
        size = (size[0] * 2, size[1] * 2)
        s["mean%d" % i] = np.zeros((1, channels[i + 1]) + size, np.float32)
        s["variable%d" % i] = np.ones((1, channels[i + 1]) + size, np.float32)
    return s


# cmodel_gan.cu.h:136-225: the input holder is a Linear layer without a predecessor, which saves two [1,1,1,1] tensors
# (netlayer/cnetlayerlinear.cu.h:175-178)
LAYER_KINDS = ["linear", "linear", "function"] + ["upsampling", "convolution", "batchnorm", "function"] * 6 + ["convolution", "function"]


def net_layers(host, channels=CHANNELS):
    """Parameters and running statistics (numpy, keys of make_parameters + make_statistics) as the layer list that
    wire_format.write_net takes, in the order SaveNetLayers writes the reference's generator
    (cuda/netmodel/cmodelmain.cu.h:296-300)."""
    one = np.zeros((1, 1, 1, 1), np.float32)
    layers = [("linear", {"weight": one, "bias": one}), ("linear", {"weight": host["lin_w"], "bias": host["lin_b"]}), ("function", {"name": "leaky_relu"})]
    widths = tuple(channels[1:]) + (IMAGE_DEPTH,)
    for i in range(7):
        header = dict(kernel_amount=widths[i], kernel_x=3, kernel_y=3, kernel_z=channels[i], stride_x=1, stride_y=1, padding_x=1, padding_y=1)
        if i < 6:
            layers.append(("upsampling", {"x": 2, "y": 2}))
        layers.append(("convolution", {"header": header, "kernel": host["kernel%d" % i], "bias": host["bias%d" % i]}))
        if i < 6:
            layers.append(("batchnorm", {"beta": host["beta%d" % i], "gamma": host["gamma%d" % i], "mean": host["mean%d" % i],
                                         "variable": host["variable%d" % i], "momentum": MOMENTUM}))
            layers.append(("function", {"name": "leaky_relu"}))
    layers.append(("function", {"name": "tangence"}))
    return layers


def host_from_layers(layers):
    """The inverse, for a list read with wire_format.read_net(f, LAYER_KINDS)."""
    host = {"lin_w": layers[1][1]["weight"], "lin_b": layers[1][1]["bias"]}
    for i, c in enumerate(p for kind, p in layers if kind == "convolution"):
        host["kernel%d" % i], host["bias%d" % i] = c["kernel"], c["bias"]
    for i, n in enumerate(p for kind, p in layers if kind == "batchnorm"):
        for name in ("gamma", "beta", "mean", "variable"):
            host["%s%d" % (name, i)] = n[name]
    return host


def make_noise(batch, noise=NOISE, seed=6):
    return np.random.default_rng(seed + 1000).standard_normal((batch, 1, noise, 1)).astype(np.float32)


def conv_flops(batch, channels=CHANNELS):
    """Algorithmic FLOPs (2*MAC) of the seven convolutions as the reference's layers compute them (nine taps per
    up-sampled pixel), per layer."""
    out, size, widths = [], (3, 4), tuple(channels[1:]) + (IMAGE_DEPTH,)
    for i in range(7):
        cin, cout = (channels[0] if i == 0 else widths[i - 1]), widths[i]
        if i < 6:
            size = (size[0] * 2, size[1] * 2)
        out.append(2.0 * batch * cout * size[0] * size[1] * cin * 9)
    return out


class GanGenerator:
    def __init__(self, batch=BATCH, params=None, channels=CHANNELS, noise=NOISE):
        mt.init(0)
        self.batch, self.channels = batch, tuple(channels)
        host = params or make_parameters(channels, noise)
        self.p = {k: CTensor.from_numpy(v) for k, v in host.items() if not k.startswith(("mean", "variable"))}
        # running statistics: one tensor serves as the layer's Mean / Variable and as its NewMean / NewVariable, which the
        # layer copies into each other at both ends of a training step (netlayer/cnetlayerbatchnormalization.cu.h:620-621,
        # 650-651); the training-mode forward pass blends into it.  The layer itself discards the blend of a forward pass
        # that no weight update follows (NewMean = Mean at the next reset); this class keeps it: forward passes here are
        # meant as the forward half of training steps
        self.stats = {k: CTensor.from_numpy(host[k] if k in host else v) for k, v in make_statistics(self.channels).items()}
        b = batch
        self.noise = CTensor(b, 1, noise, 1)
        self.h = [CTensor(b, channels[0], 3, 4)]          # layer outputs after the function
        self.lin_out = self.h[0].reinterpret(b, 1, 12 * channels[0], 1)
        self.up, self.c, size, cin = [], [], (3, 4), channels[0]
        for i in range(6):
            size = (size[0] * 2, size[1] * 2)
            self.up.append(None)                          # up-sampled images: allocated by the layer-by-layer pass only
            self.c.append(CTensor(b, channels[i + 1], *size))
            self.h.append(CTensor(b, channels[i + 1], *size))
            cin = channels[i + 1]
        self.image = CTensor(b, IMAGE_DEPTH, *size)

    def set_noise(self, z):
        self.noise.upload(z)

    # ---- network file ----------------------------------------------------------------------------------------
    LAYER_KINDS = LAYER_KINDS

    def host_state(self):
        host = {k: t.numpy() for k, t in self.p.items()}
        host.update({k: t.numpy() for k, t in self.stats.items()})
        return host

    def save_net(self, f):
        """Parameters and running statistics as SaveNetLayers writes the reference's generator
        (cuda/netmodel/cmodelmain.cu.h:296-300)."""
        import wire_format
        wire_format.write_net(f, net_layers(self.host_state(), self.channels))

    def load_net(self, f):
        """The inverse; tensor sizes in the file must be this network's (the reference loads with check_size)."""
        import wire_format
        found = host_from_layers(wire_format.read_net(f, self.LAYER_KINDS))
        for name, a in found.items():
            t = self.stats[name] if name in self.stats else self.p[name]
            if a.shape != t.shape:
                raise ValueError("%s: the file holds %s, the network %s" % (name, a.shape, t.shape))
        for name, a in found.items():
            (self.stats[name] if name in self.stats else self.p[name]).upload(a)

    def forward(self, fused=True):
        p, ch = self.p, self.channels
        Fused.LinearForward(self.lin_out, p["lin_w"], self.noise, p["lin_b"], "leaky_relu")
        for i in range(6):
            cin, cout = ch[i], ch[i + 1]
            if fused:
                Fused.UpSamplingConvolution(self.c[i], self.h[i], 2, 2, p["kernel%d" % i], 3, 3, cin, cout, p["bias%d" % i], 1, 1, 1, 1)
            else:
                if self.up[i] is None:
                    s = self.h[i].shape
                    self.up[i] = CTensor(s[0], s[1], s[2] * 2, s[3] * 2)
                CTensorMath.UpSampling(self.up[i], self.h[i], 2, 2)
                CTensorConv.ForwardConvolution(self.c[i], self.up[i], p["kernel%d" % i], 3, 3, cin, cout, p["bias%d" % i], 1, 1, 1, 1)
            Fused.BatchNormForwardTrain(self.h[i + 1], self.c[i], p["gamma%d" % i], p["beta%d" % i], new_mean=self.stats["mean%d" % i],
                                        new_variable=self.stats["variable%d" % i], momentum=MOMENTUM, epsilon=BN_EPSILON, func="leaky_relu")
        CTensorConv.ForwardConvolution(self.image, self.h[6], p["kernel6"], 3, 3, ch[6], IMAGE_DEPTH, p["bias6"], 1, 1, 1, 1, func="tangence")
        return self.image
