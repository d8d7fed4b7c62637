"""TEST INFRASTRUCTURE ONLY (checker side).

The reference layers' Forward()/TrainingBackward() as literal sequences of tensor ops, written
against the shared numpy API of oracle_api.Oracle and gpu_api.Gpu.  Running one sequence on both
back ends is the "same op sequence on oracle vs GPU" parity check; the fused C-ABI entry points
are compared with the oracle's literal sequence."""
import numpy as np

BN_EPSILON = 1e-6  # netlayer/cnetlayerbatchnormalization.cu.h:26


def flat(x):
    """ReinterpretSize(B,1,Z*Y*X,1) (netlayer/cnetlayerlinear.cu.h:268-271)."""
    return np.ascontiguousarray(x).reshape(x.shape[0], 1, -1, 1)


def linear_forward(lib, weight, x, bias):
    """CNetLayerLinear::Forward, netlayer/cnetlayerlinear.cu.h:262-280: Mul then Add of the bias."""
    h = lib.mul(weight, flat(x))
    return lib.add(h, bias)


def linear_backward(lib, weight, delta, h_prev):
    """CNetLayerLinear::TrainingBackward, netlayer/cnetlayerlinear.cu.h:415-447.
    Returns (previous layer error, dW, dB) starting from zero gradients."""
    prev_err = lib.transponse_mul(weight, delta)
    b = delta.shape[0]
    tmp = lib.mul(delta, np.ascontiguousarray(h_prev).reshape(b, 1, 1, -1))          # per-sample outer products
    zero_w = np.zeros((1, 1) + weight.shape[2:], np.float32)
    dw = lib.add_sum_w(zero_w, tmp, out_init=zero_w)
    zero_b = np.zeros((1, 1, weight.shape[2], 1), np.float32)
    db = lib.add_sum_w(zero_b, delta, out_init=zero_b)
    return prev_err, dw, db


def function_forward(lib, x, func):
    """CNetLayerFunction::Forward, netlayer/cnetlayerfunction.cu.h:203-213."""
    return lib.apply_func(x, func)


def batchnorm_forward_train(lib, x, gamma, beta, new_mean=None, new_var=None, momentum=0.9):
    """CNetLayerBatchNormalization::Forward in training mode, netlayer/cnetlayerbatchnormalization.cu.h:301-371.
    Statistics are per element (z,y,x) over the batch axis.  Returns a dict of every tensor the layer keeps."""
    n = np.float32(x.shape[0])
    inv_n = float(np.float32(1.0 / np.float64(n)))
    zero = np.zeros((1,) + x.shape[1:], np.float32)
    mean = lib.add_sum_w(zero, x, 1.0, inv_n, out_init=zero)                        # :308-309
    res = {}
    if new_mean is not None:
        res["new_mean"] = lib.add(new_mean, mean, momentum, float(np.float32(1.0 - np.float64(np.float32(momentum)))))  # :311
    xmu = lib.sub(x, mean, 1.0, 1.0)                                               # :315
    sq = lib.pow2(xmu, 1.0)                                                        # :321
    var = lib.add_sum_w(zero, sq, 1.0, inv_n, out_init=zero)                       # :322
    if new_var is not None:
        res["new_var"] = lib.add(new_var, var, momentum, float(np.float32(1.0 - np.float64(np.float32(momentum)))))     # :324
    sqrtvar = lib.sqrt(var, 1.0, BN_EPSILON)                                       # :356
    ivar = lib.inv(sqrtvar)                                                        # :359
    xhat = lib.tensor_item_production(xmu, ivar)                                   # :363
    gx = lib.tensor_item_production(gamma, xhat)                                   # :369
    out = lib.add(gx, beta)                                                        # :371
    res.update(out=out, xhat=xhat, ivar=ivar, mean=mean, var=var)
    return res


def batchnorm_forward_infer(lib, x, gamma, beta, mean, var):
    """The same layer in inference mode, lines 326-371."""
    xmu = lib.sub(x, mean, 1.0, 1.0)
    ivar = lib.inv(lib.sqrt(var, 1.0, BN_EPSILON))
    xhat = lib.tensor_item_production(xmu, ivar)
    return lib.add(lib.tensor_item_production(gamma, xhat), beta)


def batchnorm_backward(lib, delta, gamma, xhat, ivar):
    """CNetLayerBatchNormalization::TrainingBackward, lines 578-604 (with create_delta_weight).
    Returns (previous layer error, dGamma, dBeta) starting from zero gradients."""
    n = np.float32(delta.shape[0])
    zero = np.zeros((1,) + delta.shape[1:], np.float32)
    dxhat = lib.tensor_item_production(delta, gamma)
    s1 = lib.add_sum_w(zero, dxhat, out_init=zero)
    s2 = lib.add_sum_w(zero, lib.tensor_item_production(dxhat, xhat), out_init=zero)
    dgamma = lib.add_sum_w(zero, lib.tensor_item_production(delta, xhat), out_init=zero)
    dbeta = lib.add_sum_w(zero, delta, out_init=zero)
    err = lib.mul_value(dxhat, float(n))
    err = lib.sub(err, lib.tensor_item_production(xhat, s2))
    err = lib.sub(err, s1)
    err = lib.tensor_item_production(err, ivar)
    err = lib.mul_value(err, float(np.float32(1.0 / np.float64(n))))
    return err, dgamma, dbeta


def conv_forward(lib, x, kernel, bias, k, s, p):
    """CNetLayerConvolution::Forward, netlayer/cnetlayerconvolution.cu.h:310-322."""
    ka, c = kernel.shape[2], x.shape[1]
    return lib.forward_convolution(x, kernel, bias, k, k, c, ka, s, s, p, p)


def conv_backward(lib, x, kernel, delta, k, s, p):
    """CNetLayerConvolution::TrainingBackward, netlayer/cnetlayerconvolution.cu.h:484-516: input delta with a zero
    bias, per-sample gradients, then their sum over the batch.  Returns (previous layer error, dK, dB)."""
    b, c, ka = x.shape[0], x.shape[1], kernel.shape[2]
    zero_bias = np.zeros((1, ka, 1, 1), np.float32)
    prev_err = lib.backward_convolution(delta, kernel, zero_bias, k, k, c, ka, s, s, p, p, x.shape)
    dk_batch, db_batch = lib.create_delta_weight_and_bias(np.zeros((b, 1, ka, c * k * k), np.float32), np.zeros((b, ka, 1, 1), np.float32),
                                                          x, delta, k, k, c, ka, s, s, p, p)
    zk, zb = np.zeros((1, 1, ka, c * k * k), np.float32), np.zeros((1, ka, 1, 1), np.float32)
    dk = lib.add_sum_w(zk, dk_batch, out_init=zk)
    db = lib.add_sum_w(zb, db_batch, out_init=zb)
    return prev_err, dk, db


def backconv_forward(lib, x, kernel, bias, k, s, p, out_depth):
    """CNetLayerBackConvolution::Forward, netlayer/cnetlayerbackconvolution.cu.h:303-315; output size
    s*(in-1)+k-2p (lines 198-232).  kernel is [1,1,Cin,Cout*k*k]."""
    b, cin, h, w = x.shape
    oh, ow = s * (h - 1) + k - 2 * p, s * (w - 1) + k - 2 * p
    return lib.backward_convolution(x, kernel, bias, k, k, out_depth, cin, s, s, p, p, (b, out_depth, oh, ow))


def dcgan_generator_forward(lib, params, latent, channels=(512, 256, 128, 64, 3)):
    """DCGAN-64 generator forward as a stack of the reference's layers: Linear, then four times
    (BatchNorm in training mode, ReLU, transposed conv 4x4 stride 2 padding 1), tanh on the last output.
    `params` uses the names of generator.make_parameters().  Returns every layer output."""
    b = latent.shape[0]
    h = linear_forward(lib, params["lin_w"], latent, params["lin_b"]).reshape(b, channels[0], 4, 4)
    outs = {"h0": h}
    for i in range(4):
        bn = batchnorm_forward_train(lib, h, params["gamma%d" % i], params["beta%d" % i])["out"]
        a = function_forward(lib, bn, "relu")
        h = backconv_forward(lib, a, params["kernel%d" % i], params["bias%d" % i], 4, 2, 1, channels[i + 1])
        outs["a%d" % i], outs["h%d" % (i + 1)] = a, h
    outs["image"] = function_forward(lib, h, "tangence")
    return outs


def function_backward(lib, error, layer_input, func):
    """CNetLayerFunction::SetOutputError, netlayer/cnetlayerfunction.cu.h:347-358: delta = error * f'(input)."""
    return lib.tensor_item_production(error, lib.apply_func(layer_input, func, differential=True))


def discriminator_forward(lib, params, x, channels=(3, 64, 128, 256, 512)):
    """DCGAN-64 discriminator forward as a stack of the reference's layers: four times (conv 4x4 stride 2 padding 1,
    BatchNorm in training mode, leaky ReLU), Linear to one logit, sigmoid.  `params` uses the names of
    discriminator.make_parameters().  Returns every tensor the layers keep."""
    acts, h = {"x": x}, x
    for i in range(4):
        c = conv_forward(lib, h, params["kernel%d" % i], params["bias%d" % i], 4, 2, 1)
        bn = batchnorm_forward_train(lib, c, params["gamma%d" % i], params["beta%d" % i])
        h = function_forward(lib, bn["out"], "leaky_relu")
        acts["c%d" % i], acts["bn%d" % i], acts["a%d" % i] = c, bn, h
    acts["logit"] = linear_forward(lib, params["lin_w"], h, params["lin_b"])
    acts["prob"] = function_forward(lib, acts["logit"], "sigmoid")
    return acts


def discriminator_backward(lib, params, acts, labels):
    """TrainingBackward of the same stack with the error p - label fed to the last function layer.
    Returns the gradient of every parameter (same names) and "d_x", the error that reaches the images."""
    grads = {}
    err = lib.sub(acts["prob"], labels)
    delta = function_backward(lib, err, acts["logit"], "sigmoid")
    prev, grads["lin_w"], grads["lin_b"] = linear_backward(lib, params["lin_w"], delta, acts["a3"])
    err = prev.reshape(acts["a3"].shape)
    for i in (3, 2, 1, 0):
        bn = acts["bn%d" % i]
        d_bn = function_backward(lib, err, bn["out"], "leaky_relu")
        d_c, grads["gamma%d" % i], grads["beta%d" % i] = batchnorm_backward(lib, d_bn, params["gamma%d" % i], bn["xhat"], bn["ivar"])
        inp = acts["a%d" % (i - 1)] if i else acts["x"]
        err, grads["kernel%d" % i], grads["bias%d" % i] = conv_backward(lib, inp, params["kernel%d" % i], d_c, 4, 2, 1)
        grads["d_c%d" % i] = d_c
    grads["d_x"] = err
    return grads


def upsampling_forward(lib, x, u):
    """CNetLayerUpSampling::Forward, netlayer/cnetlayerupsampling.cu.h:233-252."""
    return lib.upsampling(x, u, u)


def gan_generator_forward(lib, params, noise, channels=(512, 512, 256, 128, 64, 32, 16), image_depth=3):
    """The generator the reference ships (cuda/netmodel/cmodel_gan.cu.h:131-230): Linear to 3*4*C0, leaky ReLU, viewed as
    [B,C0,3,4]; six times (up-sampling x2, conv 3x3 stride 1 padding 1, BatchNorm in training mode, leaky ReLU); conv 3x3
    to the image depth, tanh: [B,depth,192,256].  `channels[0]` is C0, `channels[1:]` the six convolution widths;
    parameter names: lin_w, lin_b, kernel0..6, bias0..6, gamma0..5, beta0..5."""
    b = noise.shape[0]
    h = function_forward(lib, linear_forward(lib, params["lin_w"], noise, params["lin_b"]), "leaky_relu")
    h = np.ascontiguousarray(h).reshape(b, channels[0], 3, 4)
    outs = {"h0": h}
    for i in range(6):
        c = conv_forward(lib, upsampling_forward(lib, h, 2), params["kernel%d" % i], params["bias%d" % i], 3, 1, 1)
        bn = batchnorm_forward_train(lib, c, params["gamma%d" % i], params["beta%d" % i])["out"]
        h = function_forward(lib, bn, "leaky_relu")
        outs["c%d" % i], outs["h%d" % (i + 1)] = c, h
    outs["image"] = function_forward(lib, conv_forward(lib, h, params["kernel6"], params["bias6"], 3, 1, 1), "tangence")
    return outs


VAE_ENCODER = (3, 32, 64, 128, 256)
VAE_DECODER = (256, 128, 64, 32, 3)


def vae_encoder_forward(lib, params, x):
    """VAE encoder of configuration 4: conv 3x3 stride 2 padding 1, 3 -> 32 -> 64 -> 128 -> 256, each followed by
    BatchNorm (training mode) and leaky ReLU; two Linear heads to the mean and the log-variance of the latent
    (netlayer/cnetlayervaecoderoutput.cu.h consumes them).  Parameter names: ekernel0..3, ebias0..3, egamma0..3,
    ebeta0..3, mu_w, mu_b, lv_w, lv_b."""
    outs, h = {}, x
    for i in range(4):
        c = conv_forward(lib, h, params["ekernel%d" % i], params["ebias%d" % i], 3, 2, 1)
        bn = batchnorm_forward_train(lib, c, params["egamma%d" % i], params["ebeta%d" % i])["out"]
        h = function_forward(lib, bn, "leaky_relu")
        outs["ec%d" % i], outs["eh%d" % i] = c, h
    outs["mu"] = linear_forward(lib, params["mu_w"], h, params["mu_b"])
    outs["logvar"] = linear_forward(lib, params["lv_w"], h, params["lv_b"])
    return outs


def vae_reparameterize(mu, logvar, eps):
    """z = mu + exp(clamp(logvar, -10, 10) / 2) * eps (netlayer/cnetlayervaecoderoutput.cu.h:266-274), on the host:
    the same numbers feed both back ends."""
    return (mu + np.exp(np.clip(logvar, -10.0, 10.0) * 0.5) * eps).astype(np.float32)


def vae_decoder_forward(lib, params, z, size=8):
    """VAE decoder: Linear latent -> 256*size*size, leaky ReLU, viewed [B,256,size,size]; transposed conv 4x4 stride 2
    padding 1, 256 -> 128 -> 64 -> 32 -> 3 with leaky ReLU between, sigmoid at the end.  Parameter names: dec_w, dec_b,
    dkernel0..3, dbias0..3."""
    b = z.shape[0]
    h = function_forward(lib, linear_forward(lib, params["dec_w"], z, params["dec_b"]), "leaky_relu")
    h = np.ascontiguousarray(h).reshape(b, VAE_DECODER[0], size, size)
    outs = {"dh0": h}
    for i in range(4):
        h = backconv_forward(lib, h, params["dkernel%d" % i], params["dbias%d" % i], 4, 2, 1, VAE_DECODER[i + 1])
        h = function_forward(lib, h, "leaky_relu" if i < 3 else "sigmoid")
        outs["dh%d" % (i + 1)] = h
    return outs
