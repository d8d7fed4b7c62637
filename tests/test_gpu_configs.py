"""The benchmark configurations through the C ABI: the DCGAN-64 generator (the measured workload) against
the CPU oracle at a batch the oracle finishes in seconds, and at the full batch of 256 through
size-independent properties; the Linear stack and the single-conv configuration at full size."""
import numpy as np
import pytest

import layer_sequences as seq
from cases import rng_normal as Nrm, rng_uniform as U
from conftest import rel_err

pytestmark = pytest.mark.gpu

REL = 1e-4  # max|gpu-cpu| / max|cpu| per tensor, fp32


@pytest.fixture(scope="module")
def gpu():
    from gpu_api import Gpu
    return Gpu()


def test_config1_single_conv_layer(gpu, oracle):
    """16x3x64x64 uniform[-1,1], 32 filters 5x5x3 He-normal seed 1, bias 0, stride 1, padding 2, leaky ReLU."""
    image = U(1, 16, 3, 64, 64)
    kernel = Nrm(1, 1, 1, 32, 75, std=float(np.sqrt(2.0 / 75)))
    bias = np.zeros((1, 32, 1, 1), np.float32)
    want = oracle.apply_func(oracle.forward_convolution(image, kernel, bias, 5, 5, 3, 32, 1, 1, 2, 2), "leaky_relu")  # slope 0.1, the reference's
    got = gpu.forward_convolution(image, kernel, bias, 5, 5, 3, 32, 1, 1, 2, 2, func="leaky_relu")
    assert got.shape == (16, 32, 64, 64) and rel_err(got, want) <= REL
    lit = gpu.apply_func(gpu.forward_convolution(image, kernel, bias, 5, 5, 3, 32, 1, 1, 2, 2), "leaky_relu")
    assert rel_err(lit, want) <= REL


def test_config2_linear_stack(gpu, oracle):
    """Batch 256, 4096 -> 3072 -> ReLU -> 768, Xavier-uniform seed 2."""
    x = Nrm(2, 256, 1, 4096, 1)
    w1 = U(3, 1, 1, 3072, 4096, lo=-np.sqrt(6 / 7168), hi=np.sqrt(6 / 7168))
    w2 = U(4, 1, 1, 768, 3072, lo=-np.sqrt(6 / 3840), hi=np.sqrt(6 / 3840))
    b1, b2 = np.full((1, 1, 3072, 1), 0.1, np.float32), np.full((1, 1, 768, 1), 0.1, np.float32)
    h = oracle.apply_func(seq.linear_forward(oracle, w1, x, b1), "relu")
    want = seq.linear_forward(oracle, w2, h, b2)
    got = gpu.linear_forward(w2, gpu.linear_forward(w1, x, b1, func="relu"), b2)
    assert got.shape == (256, 1, 768, 1) and rel_err(got, want) <= REL
    lit = seq.linear_forward(gpu, w2, gpu.apply_func(seq.linear_forward(gpu, w1, x, b1), "relu"), b2)
    assert rel_err(lit, want) <= REL


def test_config3_generator_against_oracle(gpu, oracle):
    """DCGAN-64 generator forward, every layer output, batch 8 (the oracle needs ~0.2 GFLOP per image): the literal op
    sequence, and the fused path with no, one and all batch norms folded into the convolutions around them."""
    import generator as G
    params, z = G.make_parameters(), G.make_latent(8)
    want = seq.dcgan_generator_forward(oracle, params, z)
    net = G.DcganGenerator(8, params)
    net.keep_linear_output = True
    net.set_latent(z)
    for forward, fold, one_launch in ((net.forward_fused, (), False), (net.forward_fused, (3,), True), (net.forward_fused, (3,), False),
                                      (net.forward_fused, (1, 2, 3), False), (net.forward_literal, (), False)):
        net.fold = fold
        net.fuse_linear_bn = one_launch   # the Linear layer and its batch norm as one launch or two
        for t in net.h + net.a:
            mt_fill(t, 7.0)
        forward()
        assert rel_err(net.h[0].numpy(), want["h0"]) <= REL
        for i in range(4):
            assert rel_err(net.activation(i), want["a%d" % i]) <= REL, ("a%d" % i, fold)
            if i < 3:
                assert rel_err(net.h[i + 1].numpy(), want["h%d" % (i + 1)]) <= REL, ("h%d" % (i + 1), fold)
        image = net.output.numpy()
        assert image.shape == (8, 3, 64, 64) and rel_err(image, want["image"]) <= REL, fold


def mt_fill(t, value):
    import mi355tensor as mt
    mt.CTensorMath.Fill(t, value)


def test_config3_full_batch_properties(gpu, oracle):
    """Batch 256: (1) the fused path (with the batch norms folded that the benchmark folds, and with all of them) and the
    literal op sequences agree; (2) the transposed convolutions are linear and per-sample independent, so any sample of
    the big batch equals the same sample run alone through the oracle."""
    import generator as G
    params, z = G.make_parameters(), G.make_latent(256)
    net = G.DcganGenerator(256, params)
    net.keep_linear_output = True
    net.set_latent(z)
    literal = net.forward_literal().numpy()
    for fold, one_launch in (((), False), (G.FOLD, False), (G.FOLD, True), ((1, 2, 3), False)):
        net.fold = fold
        net.fuse_linear_bn = one_launch
        fused = net.forward_fused().numpy()
        a = [net.activation(i) for i in range(4)]
        h = [t.numpy() for t in net.h[:4]]
        assert fused.shape == (256, 3, 64, 64) and np.all(np.isfinite(fused)) and np.all(np.abs(fused) <= 1)
        assert rel_err(fused, literal) <= REL, fold
        for i in range(4):
            # batch-norm output before ReLU has zero mean and unit variance over the batch, per element
            x = h[i].astype(np.float64)
            xhat = (x - x.mean(0)) / np.sqrt(x.var(0) + G.BN_EPSILON)
            assert rel_err(a[i], np.maximum(xhat, 0)) <= REL, (i, fold)
        for i, sample in ((0, 255), (1, 17), (2, 100), (3, 3)):
            cin, cout = G.CHANNELS[i], G.CHANNELS[i + 1]
            want = seq.backconv_forward(oracle, a[i][sample:sample + 1], params["kernel%d" % i], params["bias%d" % i], 4, 2, 1, cout)
            got = h[i + 1][sample:sample + 1] if i < 3 else None
            if i == 3:
                want, got = oracle.apply_func(want, "tangence"), fused[sample:sample + 1]
            assert rel_err(got, want) <= REL, ("layer %d" % i, fold)


def test_config5_training_step_against_oracle(gpu, oracle):
    """DCGAN-64 discriminator: forward, backward (input, weight and bias gradients, batch-norm gradients) and one Adam
    step at batch 4, every tensor against the CPU oracle running the same layer sequences."""
    import discriminator as D
    params = D.make_parameters()
    x, labels = D.make_batch(4)
    acts = seq.discriminator_forward(oracle, params, x)
    want = seq.discriminator_backward(oracle, params, acts, labels)
    net = D.Discriminator(4, params)
    net.set_batch(x, labels)
    for fused in (False, True):
        net.forward(fused)
        for i in range(4):
            assert rel_err(net.c[i].numpy(), acts["c%d" % i]) <= REL, "conv %d" % i
            assert rel_err(net.xhat[i].numpy(), acts["bn%d" % i]["xhat"]) <= REL, "xhat %d" % i
            assert rel_err(net.ivar[i].numpy(), acts["bn%d" % i]["ivar"]) <= REL, "ivar %d" % i
            assert rel_err(net.a[i].numpy(), acts["a%d" % i]) <= REL, "activation %d" % i
        assert rel_err(net.prob.numpy(), acts["prob"]) <= REL
    net.backward()
    for name in sorted(params):
        if name.startswith("bias"):
            # a bias in front of a batch norm has zero gradient: what is left is the rounding of a sum of cancelling
            # terms, so the error is measured against the size of the summands
            scale = np.abs(want["d_c" + name[4:]]).sum(axis=(0, 2, 3)).max()
            assert np.max(np.abs(net.g[name].numpy() - want[name])) <= REL * scale, name
        else:
            assert rel_err(net.g[name].numpy(), want[name]) <= REL, name
    for i in range(4):
        assert rel_err(net.d_c[i].numpy(), want["d_c%d" % i]) <= REL, "delta %d" % i
    assert rel_err(net.d_x.numpy(), want["d_x"]) <= REL
    # Adam normalises every step to about +-speed, so it is checked on identical inputs: the device's own gradients
    grads = {name: net.g[name].numpy() for name in ("kernel3", "gamma1", "lin_w")}
    net.update()
    for name, grad in grads.items():
        zero = np.zeros_like(params[name])
        w, m, v = oracle.adam(params[name], grad, zero, zero, 4, 2e-4, 0.5, 0.999, 1e-8, 1.0)
        assert np.max(np.abs(net.p[name].numpy() - w)) <= 1e-7, name
        assert rel_err(net.m[name].numpy(), m) <= 1e-6 and rel_err(net.v[name].numpy(), v) <= 1e-6, name


def test_config5_network_file_round_trip(gpu):
    """The discriminator's parameters after a training step, written in the reference's network-file layout, loaded
    into a differently initialised copy: the copy computes the same outputs bit for bit; a file of another topology
    is refused."""
    import io
    import discriminator as D
    import wire_format as wf
    x, labels = D.make_batch(4)
    net = D.Discriminator(4)
    net.set_batch(x, labels)
    net.step(fused=True)
    f = io.BytesIO()
    net.save_net(f)
    # size: 4 conv headers, 4 function ids + the last one, 4 momenta, 26 tensors
    tensors = sum(int(np.prod(t.shape)) for t in net.p.values()) + sum(int(np.prod(t.shape)) for t in net.stats.values())
    assert len(f.getvalue()) == 4 * 32 + 5 * 4 + 4 * 8 + 26 * 16 + 8 * tensors
    other = D.Discriminator(4, D.make_parameters(seed=77))
    other.set_batch(x, labels)
    f.seek(0)
    other.load_net(f)
    for name in net.p:
        assert np.array_equal(net.p[name].numpy(), other.p[name].numpy()), name
    for name in net.stats:      # the running statistics travel too, and saving what was loaded gives the same bytes
        assert np.array_equal(net.stats[name].numpy(), other.stats[name].numpy()), name
    again = io.BytesIO()
    other.save_net(again)
    assert again.getvalue() == f.getvalue()
    assert np.array_equal(net.forward(True).numpy(), other.forward(True).numpy())
    # the training state (iteration, Adam moments) travels the same way: after loading both, the next step is the same
    g = io.BytesIO()
    net.save_training(g)
    g.seek(0)
    other.load_training(g)
    assert other.iteration == net.iteration == 1
    net.step(fused=True)
    other.step(fused=True)
    for name in net.p:
        assert np.array_equal(net.p[name].numpy(), other.p[name].numpy()), name
        assert np.array_equal(net.m[name].numpy(), other.m[name].numpy()), name
    layers = wf.read_net(io.BytesIO(f.getvalue()), D.Discriminator.LAYER_KINDS)
    layers[1][1]["header"]["stride_x"] = 1
    g = io.BytesIO()
    wf.write_net(g, layers)
    g.seek(0)
    with pytest.raises(ValueError):
        other.load_net(g)


def test_config5_running_statistics(gpu, oracle):
    """The running mean and variable of the batch-norm layers after two training steps, fused and literal: the
    oracle's blend Add(momentum, 1-momentum) of the batch statistics of the layer's input
    (netlayer/cnetlayerbatchnormalization.cu.h:311, 324), starting from 0 and 1."""
    import discriminator as D
    for fused in (True, False):
        net = D.Discriminator(6)
        want = D.make_statistics()
        for seed in (70, 71):
            net.set_batch(*D.make_batch(6, seed=seed))
            net.forward(fused)
            for i in range(4):
                zero = np.zeros_like(want["mean%d" % i])
                r = seq.batchnorm_forward_train(oracle, net.c[i].numpy(), zero + 1, zero, new_mean=want["mean%d" % i], new_var=want["variable%d" % i],
                                                momentum=D.MOMENTUM)
                want["mean%d" % i], want["variable%d" % i] = r["new_mean"], r["new_var"]
            net.backward(fused)
            net.update(fused=fused)
        for name in want:
            assert rel_err(net.stats[name].numpy(), want[name]) <= 1e-5, (fused, name)
            assert np.abs(want[name] - D.make_statistics()[name]).max() > 1e-3, name


def test_config5_full_batch_properties(gpu, oracle):
    """Batch 128: (1) the fused and the literal forward agree; (2) convolution, its input gradient and its per-sample
    weight gradient are independent per sample, so one sample of the big batch equals that sample alone through the
    oracle; (3) the batch sum of the per-sample gradients equals their float64 sum."""
    import discriminator as D
    params = D.make_parameters()
    x, labels = D.make_batch(128)
    net = D.Discriminator(128, params)
    net.set_batch(x, labels)
    fus = net.forward(True).numpy()
    a_fus = [t.numpy() for t in net.a]
    lit = net.forward(False).numpy()
    assert np.all(np.isfinite(fus)) and np.all((fus > 0) & (fus < 1)) and rel_err(fus, lit) <= REL
    for i in range(4):
        assert rel_err(a_fus[i], net.a[i].numpy()) <= REL
    # both backward passes start from the literal forward pass: the same xhat, so the same side of zero for every
    # leaky ReLU input (after different forward passes a few inputs next to zero change sides)
    net.backward()
    for i, sample in ((0, 127), (1, 5), (2, 64), (3, 0)):
        cin, cout = D.CHANNELS[i], D.CHANNELS[i + 1]
        inp = (net.a[i - 1] if i else net.x).numpy()[sample:sample + 1]
        delta = net.d_c[i].numpy()[sample:sample + 1]
        zero_bias = np.zeros((1, cout, 1, 1), np.float32)
        want_prev = oracle.backward_convolution(delta, params["kernel%d" % i], zero_bias, 4, 4, cin, cout, 2, 2, 1, 1, inp.shape)
        got_prev = (net.d_a[i - 1] if i else net.d_x).numpy()[sample:sample + 1]
        assert rel_err(got_prev, want_prev) <= REL, "input gradient %d" % i
        dk, db = oracle.create_delta_weight_and_bias(np.zeros((1, 1, cout, cin * 16), np.float32), np.zeros((1, cout, 1, 1), np.float32),
                                                     inp, delta, 4, 4, cin, cout, 2, 2, 1, 1)
        dk_batch, db_batch = net.dk_batch[i].numpy(), net.db_batch[i].numpy()
        assert rel_err(dk_batch[sample:sample + 1], dk) <= REL, "weight gradient %d" % i
        assert rel_err(db_batch[sample:sample + 1], db) <= REL, "bias gradient %d" % i
        assert rel_err(net.g["kernel%d" % i].numpy(), dk_batch.astype(np.float64).sum(0, keepdims=True)) <= REL
        assert np.max(np.abs(net.g["bias%d" % i].numpy() - db_batch.astype(np.float64).sum(0, keepdims=True))) <= REL * np.abs(db_batch).sum(0).max()
    # (4) the batch-summed weight gradient in one product gives the same gradients
    literal = {name: t.numpy() for name, t in net.g.items()}
    net.backward(fused=True)
    for name, want in literal.items():
        if name.startswith("bias"):
            i = int(name[4:])
            assert np.max(np.abs(net.g[name].numpy() - want)) <= REL * np.abs(net.db_batch[i].numpy()).sum(0).max(), name
        else:
            assert rel_err(net.g[name].numpy(), want) <= REL, name


def test_shipped_gan_generator_topology(gpu, oracle):
    """The generator of the reference's own GAN model (Linear, then up-sampling + conv 3x3 + BatchNorm + leaky ReLU six
    times, conv 3x3 + tanh; 3x4 -> 192x256), every layer output against the oracle, at a quarter of the shipped widths
    and batch 4 so that the CPU side finishes in seconds."""
    import gan_generator as GG
    channels, noise_size, b = (128, 128, 64, 32, 16, 8, 4), 64, 4
    params, noise = GG.make_parameters(channels, noise_size), GG.make_noise(b, noise_size)
    widths = channels[1:] + (3,)
    want = seq.gan_generator_forward(oracle, params, noise, channels)
    # layer by layer on the oracle's own inputs: a batch norm over four samples divides by spreads that can be tiny, so
    # rounding differences of one layer would otherwise be amplified by the next ones
    h0 = seq.function_forward(gpu, seq.linear_forward(gpu, params["lin_w"], noise, params["lin_b"]), "leaky_relu")
    assert rel_err(h0.reshape(want["h0"].shape), want["h0"]) <= REL
    for i in range(6):
        up = seq.upsampling_forward(oracle, want["h%d" % i], 2)
        assert np.array_equal(seq.upsampling_forward(gpu, want["h%d" % i], 2), up), "up-sampling %d is an index map: bit-exact" % i
        assert rel_err(seq.conv_forward(gpu, up, params["kernel%d" % i], params["bias%d" % i], 3, 1, 1), want["c%d" % i]) <= REL, "conv %d" % i
        bn = seq.batchnorm_forward_train(gpu, want["c%d" % i], params["gamma%d" % i], params["beta%d" % i])["out"]
        assert rel_err(seq.function_forward(gpu, bn, "leaky_relu"), want["h%d" % (i + 1)]) <= REL, "batch norm %d" % i
        fused = gpu.batchnorm_train(want["c%d" % i], params["gamma%d" % i], params["beta%d" % i], func="leaky_relu")["out"]
        assert rel_err(fused, want["h%d" % (i + 1)]) <= REL, "fused batch norm %d" % i
    image = gpu.forward_convolution(want["h6"], params["kernel6"], params["bias6"], 3, 3, widths[5], 3, 1, 1, 1, 1, func="tangence")
    assert rel_err(image, want["image"]) <= REL
    # end to end: the whole stack on the device, seven layers of accumulated rounding
    got = seq.gan_generator_forward(gpu, params, noise, channels)
    assert got["image"].shape == (b, 3, 192, 256) and rel_err(got["image"], want["image"]) <= 2e-3
    # the same stack on device-resident tensors, layer by layer and with up-sampling + convolution as one call
    net = GG.GanGenerator(b, params, channels, noise_size)
    net.set_noise(noise)
    for fused in (False, True):
        image = net.forward(fused).numpy()
        assert rel_err(net.c[0].numpy(), want["c0"]) <= REL        # same input as the oracle's first convolution
        assert rel_err(image, want["image"]) <= 2e-3, "fused" if fused else "layer by layer"
    for i in range(6):   # one call against two layers, each on the oracle's input
        one = gpu.upsampling_convolution(want["h%d" % i], params["kernel%d" % i], params["bias%d" % i], 3, want["h%d" % i].shape[1], widths[i])
        assert rel_err(one, want["c%d" % i]) <= REL, "up-sampling + conv %d" % i


def test_gan_generator_network_file_round_trip(gpu):
    """The generator's parameters in the layer order of the reference's GAN model (two Linear layers, the first one the
    input holder with 1x1 tensors), loaded into a differently initialised copy: same image bit for bit."""
    import io
    import gan_generator as GG
    import wire_format as wf
    channels, noise_size, b = (64, 64, 32, 16, 16, 8, 4), 32, 2
    net = GG.GanGenerator(b, GG.make_parameters(channels, noise_size), channels, noise_size)
    other = GG.GanGenerator(b, GG.make_parameters(channels, noise_size, seed=99), channels, noise_size)
    noise = GG.make_noise(b, noise_size)
    net.set_noise(noise)
    other.set_noise(noise)
    f = io.BytesIO()
    net.save_net(f)
    raw = f.getvalue()
    head = wf.read_net(io.BytesIO(raw), GG.GanGenerator.LAYER_KINDS[:5])
    assert head[0][1]["weight"].shape == (1, 1, 1, 1) and head[2][1]["name"] == "leaky_relu" and head[3][1] == {"x": 2, "y": 2}
    assert head[4][1]["header"]["kernel_amount"] == 64 and head[4][1]["kernel"].shape == (1, 1, 64, 64 * 9)
    assert not np.array_equal(net.forward(True).numpy(), other.forward(True).numpy())
    other.load_net(io.BytesIO(raw))
    assert np.array_equal(net.forward(True).numpy(), other.forward(True).numpy())
    with pytest.raises(ValueError):
        GG.GanGenerator(b, None, (64, 64, 32, 16, 16, 8, 8), noise_size).load_net(io.BytesIO(raw))


def vae_parameters():
    import vae
    return vae.make_parameters()


def test_config4_vae_against_oracle(gpu, oracle):
    """VAE of configuration 4 at batch 4: encoder (conv 3x3 s2 p1 + BatchNorm + leaky ReLU x4, two Linear heads 16384 ->
    128), reparameterisation on the host, decoder (Linear 128 -> 16384, transposed conv 4x4 s2 p1 x4, sigmoid)."""
    params = vae_parameters()
    x = U(40, 4, 3, 128, 128, lo=0.0, hi=1.0)
    want = seq.vae_encoder_forward(oracle, params, x)
    # layer by layer on the oracle's inputs (batch norms over four samples amplify rounding between layers)
    h = x
    for i in range(4):
        c = seq.conv_forward(gpu, h, params["ekernel%d" % i], params["ebias%d" % i], 3, 2, 1)
        assert rel_err(c, want["ec%d" % i]) <= REL, "encoder conv %d" % i
        a = gpu.batchnorm_train(want["ec%d" % i], params["egamma%d" % i], params["ebeta%d" % i], func="leaky_relu")["out"]
        assert rel_err(a, want["eh%d" % i]) <= REL, "encoder batch norm %d" % i
        h = want["eh%d" % i]
    for head, key in (("mu", "mu"), ("lv", "logvar")):   # 16384 -> 128 at batch 4: split over k
        assert rel_err(gpu.linear_forward(params[head + "_w"], h, params[head + "_b"]), want[key]) <= REL, key
    z = seq.vae_reparameterize(want["mu"], want["logvar"], Nrm(41, *want["mu"].shape))
    dwant = seq.vae_decoder_forward(oracle, params, z)
    dgot = seq.vae_decoder_forward(gpu, params, z)
    for name in dwant:
        assert rel_err(dgot[name], dwant[name]) <= REL, name
    assert dgot["dh4"].shape == (4, 3, 128, 128) and np.all((dgot["dh4"] > 0) & (dgot["dh4"] < 1))
    # the encoder end to end on the device
    got = seq.vae_encoder_forward(gpu, params, x)
    assert rel_err(got["mu"], want["mu"]) <= 2e-3 and rel_err(got["logvar"], want["logvar"]) <= 2e-3


def test_config4_device_resident_model(gpu, oracle):
    """vae.Vae (every tensor on the device, fused entry points) at batch 4: latent statistics against the oracle's
    encoder, the latent against the closed form on the device's own statistics, the decoder against the oracle's
    decoder fed with the device's latent."""
    import vae
    params = vae.make_parameters()
    x, eps = vae.make_batch(4)
    net = vae.Vae(4, params)
    net.set_batch(x, eps)
    out = net.forward().numpy()
    want = seq.vae_encoder_forward(oracle, params, x)
    for i in range(4):   # four batch norms over four samples amplify rounding from layer to layer
        assert rel_err(net.eh[i].numpy(), want["eh%d" % i]) <= 2e-3, "encoder stage %d" % i
    mu, logvar = net.mu.numpy(), net.logvar.numpy()
    assert rel_err(mu, want["mu"]) <= 2e-3 and rel_err(logvar, want["logvar"]) <= 2e-3
    z, kl = oracle.vae_coder_output(mu, logvar, eps)
    assert rel_err(net.z.numpy(), z) <= 1e-6 and abs(float(net.kl.numpy().ravel()[0]) - kl) <= 1e-5 * abs(kl)
    dwant = seq.vae_decoder_forward(oracle, params, net.z.numpy())
    for i in range(5):
        assert rel_err(net.dh[i].numpy(), dwant["dh%d" % i]) <= REL, "decoder stage %d" % i
    assert out.shape == (4, 3, 128, 128) and np.all((out > 0) & (out < 1))


def test_config4_full_batch_properties(gpu, oracle):
    """Batch 64: convolutions and transposed convolutions are independent per sample, so one sample of the full batch
    equals that sample alone through the oracle; the Linear heads likewise."""
    params = vae_parameters()
    x = U(42, 64, 3, 128, 128, lo=0.0, hi=1.0)
    h = x
    for i, sample in ((0, 63), (1, 7)):
        c = seq.conv_forward(gpu, h, params["ekernel%d" % i], params["ebias%d" % i], 3, 2, 1)
        one = seq.conv_forward(oracle, h[sample:sample + 1], params["ekernel%d" % i], params["ebias%d" % i], 3, 2, 1)
        assert rel_err(c[sample:sample + 1], one) <= REL, "encoder conv %d" % i
        h = gpu.batchnorm_train(c, params["egamma%d" % i], params["ebeta%d" % i], func="leaky_relu")["out"]
        x64 = c.astype(np.float64)
        exact = params["egamma%d" % i] * (x64 - x64.mean(0)) / np.sqrt(x64.var(0) + seq.BN_EPSILON) + params["ebeta%d" % i]
        assert rel_err(h, np.where(exact > 0, exact, 0.1 * exact)) <= REL, "batch norm %d" % i
    z = Nrm(43, 64, 1, 128, 1)
    d = seq.vae_decoder_forward(gpu, params, z)
    one = seq.vae_decoder_forward(oracle, params, z[20:21])
    for name in one:
        assert rel_err(d[name][20:21], one[name]) <= REL, name


def test_recorded_graph_replays(gpu, oracle):
    """A discriminator forward pass recorded as a HIP graph: every replay, with eager work and synchronisations of the
    program between the replays, gives the eager result for the input that is in the tensors at that moment."""
    import discriminator as D
    import mi355tensor as mt
    net = D.Discriminator(8)
    batches = [D.make_batch(8, seed=s) for s in (60, 61, 62, 63)]
    net.set_batch(*batches[0])
    net.forward(True)                                   # allocates the workspaces
    mt.synchronize()
    graph = mt.Graph(lambda: net.forward(True))
    for x, labels in batches:
        net.set_batch(x, labels)
        eager = net.forward(True).numpy()
        acts = [t.numpy() for t in net.a]
        for t in net.a + [net.prob]:
            mt.CTensorMath.Fill(t, 7.0)                 # eager work in between; the replay must overwrite it
        mt.synchronize()
        graph.launch()
        assert np.array_equal(net.prob.numpy(), eager)
        for t, want in zip(net.a, acts):
            assert np.array_equal(t.numpy(), want)
