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
        self.p = {k: CTensor.from_numpy(v) for k, v in host.items()}
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
    # cmodel_gan.cu.h:136-225: the input holder is a Linear layer without a predecessor, which saves two [1,1,1,1] tensors
    # (netlayer/cnetlayerlinear.cu.h:175-178)
    LAYER_KINDS = ["linear", "linear", "function"] + ["upsampling", "convolution", "batchnorm", "function"] * 6 + ["convolution", "function"]

    def save_net(self, f):
        """The parameters as SaveNetLayers writes the reference's generator (cuda/netmodel/cmodelmain.cu.h:296-300).  This
        class keeps no running statistics: mean 0 and variable 1 are written, the values of a fresh layer."""
        import wire_format
        one = np.zeros((1, 1, 1, 1), np.float32)
        layers = [("linear", {"weight": one, "bias": one}),
                  ("linear", {"weight": self.p["lin_w"].numpy(), "bias": self.p["lin_b"].numpy()}), ("function", {"name": "leaky_relu"})]
        widths = self.channels[1:] + (IMAGE_DEPTH,)
        for i in range(7):
            cin = self.channels[i]
            header = dict(kernel_amount=widths[i], kernel_x=3, kernel_y=3, kernel_z=cin, stride_x=1, stride_y=1, padding_x=1, padding_y=1)
            if i < 6:
                layers.append(("upsampling", {"x": 2, "y": 2}))
            layers.append(("convolution", {"header": header, "kernel": self.p["kernel%d" % i].numpy(), "bias": self.p["bias%d" % i].numpy()}))
            if i < 6:
                beta = self.p["beta%d" % i].numpy()
                layers.append(("batchnorm", {"beta": beta, "gamma": self.p["gamma%d" % i].numpy(), "mean": np.zeros_like(beta),
                                             "variable": np.ones_like(beta), "momentum": MOMENTUM}))
                layers.append(("function", {"name": "leaky_relu"}))
        layers.append(("function", {"name": "tangence"}))
        wire_format.write_net(f, layers)

    def load_net(self, f):
        """The inverse; tensor sizes in the file must be this network's (the reference loads with check_size)."""
        import wire_format
        layers = wire_format.read_net(f, self.LAYER_KINDS)
        found = {"lin_w": layers[1][1]["weight"], "lin_b": layers[1][1]["bias"]}
        convs = [p for kind, p in layers if kind == "convolution"]
        norms = [p for kind, p in layers if kind == "batchnorm"]
        for i, c in enumerate(convs):
            found["kernel%d" % i], found["bias%d" % i] = c["kernel"], c["bias"]
        for i, n in enumerate(norms):
            found["gamma%d" % i], found["beta%d" % i] = n["gamma"], n["beta"]
        for name, a in found.items():
            if a.shape != self.p[name].shape:
                raise ValueError("%s: the file holds %s, the network %s" % (name, a.shape, self.p[name].shape))
        for name, a in found.items():
            self.p[name].upload(a)

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
            Fused.BatchNormForwardTrain(self.h[i + 1], self.c[i], p["gamma%d" % i], p["beta%d" % i], momentum=MOMENTUM, epsilon=BN_EPSILON, func="leaky_relu")
        CTensorConv.ForwardConvolution(self.image, self.h[6], p["kernel6"], 3, 3, ch[6], IMAGE_DEPTH, p["bias6"], 1, 1, 1, 1, func="tangence")
        return self.image
