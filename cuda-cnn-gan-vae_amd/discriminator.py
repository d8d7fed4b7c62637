"""DCGAN-64 discriminator training step as the reference's layers would run it, on device-resident tensors.

Layer stack (the reference's layer classes in brackets):
    images [B,3,64,64]
    -> conv 4x4 s2 p1, 3 -> 64 -> 128 -> 256 -> 512   [CNetLayerConvolution, netlayer/cnetlayerconvolution.cu.h:310-322]
       each followed by BatchNorm (batch statistics)   [CNetLayerBatchNormalization :268-380]
       and leaky ReLU                                  [CNetLayerFunction :203-213]
    -> Linear 8192 -> 1, sigmoid                       [CNetLayerLinear :262-282]

`forward` / `backward` issue the layers' op sequences one C-ABI call per tensor op (TrainingBackward of
cnetlayerfunction.cu.h:347-358, cnetlayerbatchnormalization.cu.h:578-604, cnetlayerconvolution.cu.h:484-516,
cnetlayerlinear.cu.h:415-447); `update` is the layers' TrainingUpdateWeight (Adam).  The error fed to the last
function layer is p - label.
"""
import numpy as np

import mi355tensor as mt
from mi355tensor import CTensor, CTensorApplyFunc, CTensorConv, CTensorMath, Fused

CHANNELS = (3, 64, 128, 256, 512)
IMAGE = 64
BN_EPSILON = 1e-6
MOMENTUM = 0.9


def make_parameters(seed=5, std=0.02):
    """Random-init parameters as numpy arrays in the reference's layouts (kernel [1,1,Cout,Cin*16], bias [1,Cout,1,1])."""
    rng = np.random.default_rng(seed)
    p, size = {}, IMAGE
    for i in range(4):
        cin, cout = CHANNELS[i], CHANNELS[i + 1]
        size //= 2
        p["kernel%d" % i] = (rng.standard_normal((1, 1, cout, cin * 16)) * std).astype(np.float32)
        p["bias%d" % i] = np.zeros((1, cout, 1, 1), np.float32)
        p["gamma%d" % i] = np.ones((1, cout, size, size), np.float32)
        p["beta%d" % i] = np.zeros((1, cout, size, size), np.float32)
    p["lin_w"] = (rng.standard_normal((1, 1, 1, CHANNELS[4] * 16)) * std).astype(np.float32)
    p["lin_b"] = np.full((1, 1, 1, 1), 0.1, np.float32)
    return p


def make_statistics():
    """Running mean and variable of the four batch-norm layers as a fresh layer holds them
    (Reset, netlayer/cnetlayerbatchnormalization.cu.h:239-240): 0 and 1."""
    s, size = {}, IMAGE
    for i in range(4):
        size //= 2
        s["mean%d" % i] = np.zeros((1, CHANNELS[i + 1], size, size), np.float32)
        s["variable%d" % i] = np.ones((1, CHANNELS[i + 1], size, size), np.float32)
    return s


LAYER_KINDS = ["input"] + ["convolution", "batchnorm", "function"] * 4 + ["linear", "function"]


def net_layers(host):
    """Parameters and running statistics (numpy, keys of make_parameters + make_statistics) as the layer list that
    wire_format.write_net takes, in the order SaveNetLayers writes this stack (cuda/netmodel/cmodelmain.cu.h:296-300)."""
    layers = [("input", {})]
    for i in range(4):
        header = dict(kernel_amount=CHANNELS[i + 1], kernel_x=4, kernel_y=4, kernel_z=CHANNELS[i], stride_x=2, stride_y=2, padding_x=1, padding_y=1)
        layers.append(("convolution", {"header": header, "kernel": host["kernel%d" % i], "bias": host["bias%d" % i]}))
        layers.append(("batchnorm", {"beta": host["beta%d" % i], "gamma": host["gamma%d" % i], "mean": host["mean%d" % i],
                                     "variable": host["variable%d" % i], "momentum": MOMENTUM}))
        layers.append(("function", {"name": "leaky_relu"}))
    layers.append(("linear", {"weight": host["lin_w"], "bias": host["lin_b"]}))
    layers.append(("function", {"name": "sigmoid"}))
    return layers


def host_from_layers(layers):
    """The inverse, for a list read with wire_format.read_net(f, LAYER_KINDS); layer settings in the file must be this
    stack's (the reference loads with check_size)."""
    import wire_format
    host = {}
    for i in range(4):
        conv, bn, func = (layers[1 + 3 * i + j][1] for j in range(3))
        h = conv["header"]
        want = (CHANNELS[i + 1], 4, 4, CHANNELS[i], 2, 2, 1, 1)
        if tuple(h[k] for k in wire_format.CONV_HEADER) != want or func["name"] != "leaky_relu":
            raise ValueError("layer %d of the file is not this network's: %r, %s" % (i, h, func["name"]))
        for name, a in (("kernel", conv["kernel"]), ("bias", conv["bias"]), ("gamma", bn["gamma"]), ("beta", bn["beta"]), ("mean", bn["mean"]),
                        ("variable", bn["variable"])):
            host["%s%d" % (name, i)] = a
    if layers[14][1]["name"] != "sigmoid":
        raise ValueError("the last layers of the file are not this network's")
    host["lin_w"], host["lin_b"] = layers[13][1]["weight"], layers[13][1]["bias"]
    return host


def make_batch(batch, seed=5):
    rng = np.random.default_rng(seed + 1000)
    x = rng.uniform(-1, 1, size=(batch, 3, IMAGE, IMAGE)).astype(np.float32)
    labels = (rng.uniform(size=(batch, 1, 1, 1)) < 0.5).astype(np.float32)
    return x, labels


def conv_flops(batch):
    """Algorithmic FLOPs (2*MAC) of one pass over the four convolutions; forward, input gradient and weight
    gradient each cost this much."""
    out, size = [], IMAGE
    for i in range(4):
        size //= 2
        out.append(2.0 * batch * CHANNELS[i + 1] * size * size * CHANNELS[i] * 16)
    return out


class Discriminator:
    def __init__(self, batch, params=None):
        mt.init(0)
        self.batch = b = batch
        host = params or make_parameters()
        self.p = {k: CTensor.from_numpy(v) for k, v in host.items() if not k.startswith(("mean", "variable"))}
        # Running statistics of the batch-norm layers.  The layer keeps Mean / Variable (saved, used in inference mode)
        # and NewMean / NewVariable (blended by every training-mode forward pass), and copies one pair to the other at
        # both ends of a training step (netlayer/cnetlayerbatchnormalization.cu.h:620-621, 650-651).  Here one tensor
        # serves as both: the training-mode forward pass blends into it, the two copies are no-ops.  Inside a complete
        # step (reset, forward, backward, update) the two are the same.  They differ for a training-mode forward pass that
        # is NOT followed by the update: the layer throws its blend away at the next reset (NewMean = Mean), this class
        # keeps it.  step() always runs the whole sequence; a caller that only wants outputs in training mode and the
        # reference's statistics afterwards saves self.stats before and restores them after.
        self.stats = {k: CTensor.from_numpy(host[k] if k in host else v) for k, v in make_statistics().items()}
        self.x, self.labels = CTensor(b, 3, IMAGE, IMAGE), CTensor(b, 1, 1, 1)
        self.c, self.bn, self.a, self.xhat, self.ivar = [], [], [], [], []
        self.d_a, self.d_bn, self.d_c = [], [], []
        self.dk_batch, self.db_batch, self.g = [], [], {}
        self.stat = []
        size = IMAGE
        for i in range(4):
            cin, cout = CHANNELS[i], CHANNELS[i + 1]
            size //= 2
            shape, s1 = (b, cout, size, size), (1, cout, size, size)
            for lst in (self.c, self.bn, self.a, self.xhat, self.d_a, self.d_bn, self.d_c):
                lst.append(CTensor(*shape))
            self.ivar.append(CTensor(*s1))
            self.stat.append([CTensor(*s1) for _ in range(4)])      # scratch of the batch-norm backward pass
            self.dk_batch.append(CTensor(b, 1, cout, cin * 16))
            self.db_batch.append(CTensor(b, cout, 1, 1))
            for name in ("kernel", "bias", "gamma", "beta"):
                self.g["%s%d" % (name, i)] = CTensor(*host["%s%d" % (name, i)].shape)
        self.d_x = CTensor(b, 3, IMAGE, IMAGE)
        self.logit, self.prob, self.err, self.d_logit = (CTensor(b, 1, 1, 1) for _ in range(4))
        self.tmp = [CTensor(*t.shape) for t in self.c]               # elementwise scratch, one per layer size
        self.tmp_dw = CTensor(b, 1, 1, CHANNELS[4] * 16)
        self.g["lin_w"], self.g["lin_b"] = CTensor(1, 1, 1, CHANNELS[4] * 16), CTensor(1, 1, 1, 1)
        self.zero_bias = [CTensor.from_numpy(np.zeros((1, CHANNELS[i + 1], 1, 1), np.float32)) for i in range(4)]
        self.m = {k: CTensor.from_numpy(np.zeros(t.shape, np.float32)) for k, t in self.p.items()}
        self.v = {k: CTensor.from_numpy(np.zeros(t.shape, np.float32)) for k, t in self.p.items()}
        self.iteration = 0

    def set_batch(self, x, labels):
        self.x.upload(x)
        self.labels.upload(labels)

    # ---- network file ----------------------------------------------------------------------------------------
    LAYER_KINDS = LAYER_KINDS

    def host_state(self):
        """Parameters and running statistics as numpy arrays."""
        host = {k: t.numpy() for k, t in self.p.items()}
        host.update({k: t.numpy() for k, t in self.stats.items()})
        return host

    def save_net(self, f):
        """The parameters and the running statistics as the reference's SaveNetLayers would write this stack
        (cuda/netmodel/cmodelmain.cu.h:296-300; batch norm: beta, gamma, mean, variable, momentum,
        netlayer/cnetlayerbatchnormalization.cu.h:409-417): a C++ network of the same layers on the drop-in classes
        loads the file and runs inference with the statistics trained here."""
        import wire_format
        wire_format.write_net(f, net_layers(self.host_state()))

    def load_net(self, f):
        """The inverse; sizes and layer settings in the file must be this stack's (the reference loads with check_size)."""
        import wire_format
        host = host_from_layers(wire_format.read_net(f, self.LAYER_KINDS))
        for name, a in host.items():
            t = self.stats[name] if name in self.stats else self.p[name]
            if a.shape != t.shape:
                raise ValueError("%s: the file holds %s, the network %s" % (name, a.shape, t.shape))
        for name, a in host.items():
            (self.stats[name] if name in self.stats else self.p[name]).upload(a)

    def save_training(self, f):
        """Iteration and Adam moments in the layout of SaveNetLayersTrainingParam (cuda/netmodel/cmodelmain.cu.h:368-373):
        per convolution, batch-norm and linear layer first and second moment of the weights, then of the biases (for a
        batch norm: of gamma, then of beta)."""
        import wire_format
        pick = lambda w, b: {"m_weight": self.m[w].numpy(), "v_weight": self.v[w].numpy(), "m_bias": self.m[b].numpy(), "v_bias": self.v[b].numpy()}
        layers = [("input", {})]
        for i in range(4):
            layers += [("convolution", pick("kernel%d" % i, "bias%d" % i)), ("batchnorm", pick("gamma%d" % i, "beta%d" % i)), ("function", {})]
        layers += [("linear", pick("lin_w", "lin_b")), ("function", {})]
        wire_format.write_training_params(f, self.iteration, layers)

    def load_training(self, f):
        import wire_format
        iteration, layers = wire_format.read_training_params(f, self.LAYER_KINDS)
        names = [None]
        for i in range(4):
            names += [("kernel%d" % i, "bias%d" % i), ("gamma%d" % i, "beta%d" % i), None]
        names += [("lin_w", "lin_b"), None]
        for (kind, p), pair in zip(layers, names):
            if pair is None:
                continue
            for key, name in (("m_weight", pair[0]), ("v_weight", pair[0]), ("m_bias", pair[1]), ("v_bias", pair[1])):
                target = (self.m if key[0] == "m" else self.v)[name]
                if p[key].shape != target.shape:
                    raise ValueError("%s of %s: the file holds %s, the network %s" % (key, name, p[key].shape, target.shape))
                target.upload(p[key])
        self.iteration = iteration

    # ---- forward -------------------------------------------------------------------------------------------
    def forward(self, fused=False):
        h, p = self.x, self.p
        for i in range(4):
            cin, cout = CHANNELS[i], CHANNELS[i + 1]
            CTensorConv.ForwardConvolution(self.c[i], h, p["kernel%d" % i], 4, 4, cin, cout, p["bias%d" % i], 2, 2, 1, 1)
            if fused:  # batch norm and the function layer behind it in one pass
                Fused.BatchNormForwardTrain(self.a[i], self.c[i], p["gamma%d" % i], p["beta%d" % i], self.xhat[i], self.ivar[i],
                                            new_mean=self.stats["mean%d" % i], new_variable=self.stats["variable%d" % i],
                                            momentum=MOMENTUM, epsilon=BN_EPSILON, func="leaky_relu")
            else:
                self._batchnorm_literal(i)
                CTensorApplyFunc.ApplyLeakyReLU(self.a[i], self.bn[i])
            h = self.a[i]
        flat = h.reinterpret(self.batch, 1, CHANNELS[4] * 16, 1)
        if fused:
            Fused.LinearForward(self.logit, p["lin_w"], flat, p["lin_b"])
        else:
            CTensorMath.Mul(self.logit, p["lin_w"], flat)
            CTensorMath.Add(self.logit, self.logit, p["lin_b"])
        CTensorApplyFunc.ApplySigmoid(self.prob, self.logit)
        return self.prob

    def _batchnorm_literal(self, i):
        """Training-mode forward of cnetlayerbatchnormalization.cu.h:301-371, op by op."""
        x, p = self.c[i], self.p
        mean, var, sq = self.stat[i][0], self.stat[i][1], self.stat[i][2]
        inv_n = float(np.float32(1.0 / np.float64(np.float32(self.batch))))
        CTensorMath.Fill(mean, 0.0)
        CTensorMath.AddSumW(mean, mean, x, 1.0, inv_n)
        keep = float(np.float32(1.0 - np.float64(np.float32(MOMENTUM))))      # the layer passes 1.0-Momentum, rounded to float
        CTensorMath.Add(self.stats["mean%d" % i], self.stats["mean%d" % i], mean, MOMENTUM, keep)
        xmu = self.tmp[i]
        CTensorMath.Sub(xmu, x, mean, 1.0, 1.0)
        CTensorMath.Pow2(self.xhat[i], xmu, 1.0)
        CTensorMath.Fill(var, 0.0)
        CTensorMath.AddSumW(var, var, self.xhat[i], 1.0, inv_n)
        CTensorMath.Add(self.stats["variable%d" % i], self.stats["variable%d" % i], var, MOMENTUM, keep)
        CTensorMath.SQRT(sq, var, 1.0, BN_EPSILON)
        CTensorMath.Inv(self.ivar[i], sq)
        CTensorMath.TensorItemProduction(self.xhat[i], xmu, self.ivar[i])
        CTensorMath.TensorItemProduction(self.bn[i], p["gamma%d" % i], self.xhat[i])
        CTensorMath.Add(self.bn[i], self.bn[i], p["beta%d" % i])

    # ---- backward ------------------------------------------------------------------------------------------
    def backward(self, fused=False):
        """fused: function and batch-norm backward as one kernel, the batch-summed weight gradient as one product and
        one launch that zeroes every gradient, instead of the layers' sequences of tensor operations."""
        b, p, g = self.batch, self.p, self.g
        if fused:
            Fused.FillMany([g[k] for k in g if k != "lin_w"], 0.0)      # lin_w is written, not accumulated
        CTensorMath.Sub(self.err, self.prob, self.labels)
        CTensorApplyFunc.ApplyDifferentialSigmoid(self.d_logit, self.logit)
        CTensorMath.TensorItemProduction(self.d_logit, self.err, self.d_logit)
        # Linear: previous error, per-sample outer products, their sum over the batch
        flat_err = self.d_a[3].reinterpret(b, 1, CHANNELS[4] * 16, 1)
        CTensorMath.TransponseMul(flat_err, p["lin_w"], self.d_logit)
        if fused:
            # dW = sum_b delta_b (x) h_b is one product delta^T * H over the batch axis: the same tensors viewed as
            # [1,1,B,Out] and [1,1,B,In] (ReinterpretSize), no per-sample outer products
            CTensorMath.TransponseMul(g["lin_w"], self.d_logit.reinterpret(1, 1, b, 1), self.a[3].reinterpret(1, 1, b, CHANNELS[4] * 16))
        else:
            CTensorMath.Mul(self.tmp_dw, self.d_logit, self.a[3].reinterpret(b, 1, 1, CHANNELS[4] * 16))
            CTensorMath.Fill(g["lin_w"], 0.0)
            CTensorMath.AddSumW(g["lin_w"], g["lin_w"], self.tmp_dw)
        if not fused:
            CTensorMath.Fill(g["lin_b"], 0.0)
        CTensorMath.AddSumW(g["lin_b"], g["lin_b"], self.d_logit)
        for i in (3, 2, 1, 0):
            cin, cout = CHANNELS[i], CHANNELS[i + 1]
            if fused:  # function layer and batch norm
                Fused.BatchNormBackward(self.d_c[i], g["gamma%d" % i], g["beta%d" % i], self.d_a[i], p["gamma%d" % i], self.xhat[i], self.ivar[i],
                                        beta=p["beta%d" % i], func="leaky_relu")
            else:
                CTensorApplyFunc.ApplyDifferentialLeakyReLU(self.d_bn[i], self.bn[i])
                CTensorMath.TensorItemProduction(self.d_bn[i], self.d_a[i], self.d_bn[i])
                self._batchnorm_backward(i)
            # convolution layer
            inp, prev = (self.a[i - 1], self.d_a[i - 1]) if i else (self.x, self.d_x)
            CTensorConv.BackwardConvolution(prev, self.d_c[i], p["kernel%d" % i], 4, 4, cin, cout, self.zero_bias[i], 2, 2, 1, 1)
            if not fused:
                CTensorMath.Fill(g["kernel%d" % i], 0.0)
                CTensorMath.Fill(g["bias%d" % i], 0.0)
            if fused:
                Fused.ConvolutionBackwardWeightsSum(g["kernel%d" % i], 4, 4, cin, cout, g["bias%d" % i], inp, self.d_c[i], 2, 2, 1, 1)
                continue
            CTensorMath.Fill(self.dk_batch[i], 0.0)
            CTensorMath.Fill(self.db_batch[i], 0.0)
            CTensorConv.CreateDeltaWeightAndBias(self.dk_batch[i], 4, 4, cin, cout, self.db_batch[i], inp, self.d_c[i], 2, 2, 1, 1)
            CTensorMath.AddSumW(g["kernel%d" % i], g["kernel%d" % i], self.dk_batch[i])
            CTensorMath.AddSumW(g["bias%d" % i], g["bias%d" % i], self.db_batch[i])

    def _batchnorm_backward(self, i):
        """cnetlayerbatchnormalization.cu.h:578-604."""
        n = np.float32(self.batch)
        delta, gamma, xhat, ivar, g = self.d_bn[i], self.p["gamma%d" % i], self.xhat[i], self.ivar[i], self.g
        s1, s2 = self.stat[i][0], self.stat[i][1]
        dxhat, t, out = self.tmp[i], self.c[i], self.d_c[i]          # the conv output is no longer needed: reuse it as scratch
        CTensorMath.TensorItemProduction(dxhat, delta, gamma)
        CTensorMath.Fill(s1, 0.0)
        CTensorMath.AddSumW(s1, s1, dxhat)
        CTensorMath.TensorItemProduction(t, dxhat, xhat)
        CTensorMath.Fill(s2, 0.0)
        CTensorMath.AddSumW(s2, s2, t)
        CTensorMath.TensorItemProduction(t, delta, xhat)
        CTensorMath.Fill(g["gamma%d" % i], 0.0)
        CTensorMath.AddSumW(g["gamma%d" % i], g["gamma%d" % i], t)
        CTensorMath.Fill(g["beta%d" % i], 0.0)
        CTensorMath.AddSumW(g["beta%d" % i], g["beta%d" % i], delta)
        CTensorMath.Mul(out, dxhat, float(n))
        CTensorMath.TensorItemProduction(t, xhat, s2)
        CTensorMath.Sub(out, out, t)
        CTensorMath.Sub(out, out, s1)
        CTensorMath.TensorItemProduction(out, out, ivar)
        CTensorMath.Mul(out, out, float(np.float32(1.0 / np.float64(n))))

    # ---- optimiser ------------------------------------------------------------------------------------------
    def update(self, speed=2e-4, beta1=0.5, beta2=0.999, epsilon=1e-8, fused=False):
        self.iteration += 1
        if fused:
            keys = list(self.p)
            Fused.AdamMany([self.p[k] for k in keys], [self.g[k] for k in keys], [self.m[k] for k in keys], [self.v[k] for k in keys],
                           self.batch, speed, beta1, beta2, epsilon, float(self.iteration))
            return
        for k in self.p:
            CTensorMath.Adam(self.p[k], self.g[k], self.m[k], self.v[k], self.batch, speed, beta1, beta2, epsilon, float(self.iteration))

    def step(self, fused=False):
        self.forward(fused)
        self.backward(fused)
        self.update(fused=fused)
