"""The drop-in boundary on the GPU, from C++:

* `ctensor_selftest` -- the checks of the reference's CTensorTest::Test() written against the drop-in
  CTensor / CTensorMath / CTensorConv classes (every op runs through libmi355tensor.so);
* `layers_mi355` vs `layers_cpu` -- the reference's OWN layer classes (convolution, transposed convolution, linear,
  function, batch normalisation), compiled in the authoring container from /root/reference, once on the drop-in
  classes and once on the reference's CPU classes: forward outputs, back-propagated deltas and the weights after
  one gradient step must agree within 1e-4 (max|a-b| / max|b| per tensor).  Skipped where those binaries are absent.
"""
import os
import struct
import subprocess

import numpy as np
import pytest

import layer_sequences as seq
from conftest import ROOT, rel_err

pytestmark = pytest.mark.gpu

SELFTEST = os.path.join(ROOT, "cuda-cnn-gan-vae_amd", "dropin", "ctensor_selftest")
LAYERS_GPU = os.path.join(ROOT, "oracle", "_ref", "layers_mi355")
LAYERS_CPU = os.path.join(ROOT, "oracle", "_ref", "layers_cpu")


RANDOM = ("H.drop_output", "H.drop_prev_delta", "H.vae_output", "H.vae_delta_logvar0", "H.vae_delta_logvar")


def read_dump(path):
    out, data, pos = {}, open(path, "rb").read(), 0
    while pos < len(data):
        name = data[pos:pos + 32].split(b"\0")[0].decode()
        dims = struct.unpack_from("<4I", data, pos + 32)
        n = int(np.prod(dims))
        out[name] = np.frombuffer(data, np.float32, n, pos + 48).reshape(dims)
        pos += 48 + 4 * n
    return out


def test_cpp_selftest_on_the_dropin_classes():
    assert os.path.exists(SELFTEST), "build it with `make -C cuda-cnn-gan-vae_amd`"
    run = subprocess.run([SELFTEST], capture_output=True, text=True, timeout=120)
    print(run.stdout[-3000:], run.stderr[-2000:])
    assert run.returncode == 0 and "ALL PASS" in run.stdout and "FAIL" not in run.stdout
    assert run.stdout.count("PASS") >= 32


@pytest.fixture(scope="module")
def dumps(tmp_path_factory):
    if not (os.path.exists(LAYERS_GPU) and os.path.exists(LAYERS_CPU)):
        pytest.skip("oracle/_ref/layers_* not built (they need /root/reference)")
    d = tmp_path_factory.mktemp("layers")
    files = {}
    for tag, exe in (("gpu", LAYERS_GPU), ("cpu", LAYERS_CPU)):
        files[tag] = str(d / (tag + ".bin"))
        run = subprocess.run([exe, files[tag]], capture_output=True, text=True, timeout=180)
        assert run.returncode == 0, run.stderr
    return read_dump(files["gpu"]), read_dump(files["cpu"])


def test_reference_layers_agree_on_both_tensor_paths(dumps):
    gpu, cpu = dumps
    # streams are bytes, compared by tests of their own; drop-out and the VAE coder output draw from std::random_device
    shared = [k for k in cpu if k in gpu and not k.endswith("_stream") and k not in RANDOM]
    assert "A.sigmoid_ema" in shared and "H.soft_delta" in shared and "H.split_delta" in shared and "H.depool_prev_delta" in shared
    assert len(shared) >= 16 and any(k.startswith("B.") for k in shared)
    for key in shared:
        assert gpu[key].shape == cpu[key].shape, key
        assert rel_err(gpu[key], cpu[key]) <= 1e-4, key
    # the update step really moved the weights (the comparison above is not between two untouched copies)
    assert not np.array_equal(cpu["A.conv_updated.0"], cpu["A.conv_updated.0"] * 0)


def test_reference_batchnorm_layer_matches_the_oracle_sequence(dumps, oracle):
    """The reference's batch-norm layer does not build on its own CPU classes, so its run on the drop-in classes is
    checked against the oracle's restatement of the layer's op sequence."""
    gpu, _ = dumps
    x, gamma, beta, err = gpu["C.input"], gpu["C.gamma"], gpu["C.beta"], gpu["C.error"]
    want = seq.batchnorm_forward_train(oracle, x, gamma, beta)
    assert rel_err(gpu["C.bn"], want["out"]) <= 1e-4
    assert rel_err(gpu["C.relu"], oracle.apply_func(want["out"], "relu")) <= 1e-4
    delta = oracle.tensor_item_production(err, oracle.apply_func(want["out"], "relu", differential=True))
    assert rel_err(gpu["C.delta_bn"], delta) <= 1e-4


def test_reference_layers_of_the_gpu_class_only_match_the_oracle(dumps, oracle):
    """Concatenator, time embedding and max pooling build on the reference's GPU tensor class only; their runs on the
    drop-in classes are checked against the oracle (and the resampling chain D is among the shared keys above)."""
    gpu, cpu = dumps
    assert "D.average" in cpu and "D.delta_upsampling" in cpu
    cat = oracle.concatecation_z(gpu["E.a"], gpu["E.b"])
    assert np.array_equal(gpu["E.concatenated"], cat)
    steps = gpu["E.steps"].ravel().astype(np.uint32)
    assert steps.max() == 35
    assert np.max(np.abs(gpu["E.time"] - oracle.set_time_step(cat, steps))) <= 2e-5
    pooled, pos = oracle.max_pooling(gpu["F.input"], 2, 2)
    assert np.array_equal(gpu["F.maxpool"], pooled)
    assert np.array_equal(gpu["F.prev_error"], oracle.max_pooling_backward(gpu["F.error"], pos, 2, 2, gpu["F.input"].shape))


def test_reference_batchnorm_layer_saved_stream(dumps, oracle):
    """CNetLayerBatchNormalization::Save on the drop-in classes (tensors copied back from the device), parsed by the
    Python reader of the wire format: all four tensors as loaded and the momentum."""
    import io
    import wire_format as wf
    gpu, _ = dumps
    stream = io.BytesIO(gpu["C.bn_stream"].tobytes())
    beta, gamma, mean, variable, momentum = wf.read_batchnorm_layer(stream)
    assert stream.read() == b""
    assert momentum == float(np.float32(0.9))
    assert np.array_equal(beta, gpu["C.beta"]) and np.array_equal(gamma, gpu["C.gamma"])
    # the saved statistics change only in TrainingUpdateWeight (cnetlayerbatchnormalization.cu.h:650), which this chain
    # does not call: they are the loaded ones
    assert np.array_equal(mean, np.zeros_like(beta)) and np.array_equal(variable, np.ones_like(beta))
    # the conv and linear streams of the drop-in build carry the same layout as the reference's CPU build
    header, kernel, bias = wf.read_convolution_layer(io.BytesIO(gpu["A.conv_stream"].tobytes()))
    assert np.array_equal(kernel, gpu["A.conv_updated.0"]) and np.array_equal(bias, gpu["A.conv_updated.1"])


def test_reference_batchnorm_layer_trained_statistics(dumps, oracle):
    """The running statistics the reference's batch-norm layer saves after one and two training steps on the drop-in
    classes are the oracle's blends Add(momentum, 1-momentum) of the batch statistics (cnetlayerbatchnormalization.cu.h:311,
    324, 650-651), and its inference-mode forward pass uses them."""
    import io
    import wire_format as wf
    gpu, _ = dumps
    beta, gamma = gpu["C.beta"], gpu["C.gamma"]
    zero, one = np.zeros_like(beta), np.ones_like(beta)
    first = seq.batchnorm_forward_train(oracle, gpu["C.input"], gamma, beta, new_mean=zero, new_var=one, momentum=0.9)
    _, _, mean1, var1, momentum = wf.read_batchnorm_layer(io.BytesIO(gpu["C.bn_trained_stream"].tobytes()))
    assert momentum == float(np.float32(0.9))
    assert rel_err(mean1, first["new_mean"]) <= 1e-6 and rel_err(var1, first["new_var"]) <= 1e-6
    assert np.abs(mean1).max() > 0.01 and np.abs(var1 - 1.0).max() > 0.01        # non-trivial
    # the second step runs with gamma and beta after one gradient step; the statistics do not depend on them
    second = seq.batchnorm_forward_train(oracle, gpu["C.input2"], gamma, beta, new_mean=first["new_mean"], new_var=first["new_var"], momentum=0.9)
    beta2, gamma2, mean2, var2, _ = wf.read_batchnorm_layer(io.BytesIO(gpu["C.bn_trained2_stream"].tobytes()))
    assert rel_err(mean2, second["new_mean"]) <= 1e-6 and rel_err(var2, second["new_var"]) <= 1e-6
    want = seq.batchnorm_forward_infer(oracle, gpu["C.input2"], gamma2, beta2, mean2, var2)
    assert rel_err(gpu["C.bn_inference"], want) <= 1e-4


def test_dropin_layers_load_a_network_written_from_python(oracle, tmp_path):
    """A network file written by wire_format.py, loaded by the reference's layers on the drop-in classes: forward on the
    GPU against the oracle on the same weights."""
    if not os.path.exists(LAYERS_GPU):
        pytest.skip("oracle/_ref/layers_mi355 not built (it needs /root/reference)")
    from test_wire_format import chain_g_network, run_chain_g, expected_chain_g
    layers = chain_g_network(seed=4)
    got = run_chain_g(LAYERS_GPU, layers, tmp_path)
    leaky, prob = expected_chain_g(oracle, layers, got["G.input"])
    assert rel_err(got["G.leaky"], leaky) <= 1e-4
    assert rel_err(got["G.sigmoid"], prob.reshape(got["G.sigmoid"].shape)) <= 1e-4


def test_reference_host_side_layers_on_the_dropin_classes(dumps):
    """Soft-max, splitter, drop-out, VAE coder output and max de-pooling read and write their tensors element by element
    (GetElement / SetElement on device-resident drop-in tensors) and mix that with tensor-library calls; the same checks
    that pin the numpy restatements on the reference's CPU build."""
    import host_layers
    gpu, _ = dumps
    host_layers.check_chain_h({k: v for k, v in gpu.items() if k.startswith("H.")}, tol=1e-5)


def test_reference_layers_averaged_weights_on_the_dropin_classes(dumps):
    """SaveEMAWeight on the drop-in classes: the convolution and linear streams against the CPU build's (same layout, values
    within rounding), the batch-norm layer's (GPU class only) against EMA_K * loaded + (1 - EMA_K) * trained."""
    import io
    import wire_format as wf
    gpu, cpu = dumps
    kinds = ["input", "convolution", "function", "linear", "function"]
    mine, theirs = (wf.read_ema(io.BytesIO(d["A.ema_stream"].tobytes()), kinds) for d in (gpu, cpu))
    assert mine[1][1]["header"] == theirs[1][1]["header"] and mine[2][1] == theirs[2][1]
    for i, field in ((1, "kernel"), (1, "bias"), (3, "weight"), (3, "bias")):
        assert rel_err(mine[i][1][field], theirs[i][1][field]) <= 1e-5, field
    off = wf.read_ema(io.BytesIO(gpu["A.ema_off_stream"].tobytes()), kinds)
    assert off[1][1]["kernel"].shape == off[3][1]["weight"].shape == (1, 1, 1, 1)
    beta, gamma, mean, variable, momentum = wf.read_batchnorm_layer(io.BytesIO(gpu["C.bn_ema_stream"].tobytes()))
    trained = wf.read_batchnorm_layer(io.BytesIO(gpu["C.bn_trained_stream"].tobytes()))
    loaded = (gpu["C.beta"], gpu["C.gamma"], np.zeros_like(beta), np.ones_like(beta))
    assert momentum == trained[4]
    k = np.float32(wf.EMA_K)
    for got, w0, w1 in zip((beta, gamma, mean, variable), loaded, trained[:4]):
        assert np.abs(w1 - w0).max() > 1e-3
        assert rel_err(got, k * w0 + (np.float32(1) - k) * w1) <= 1e-6


def test_reference_gan_generator_with_deferred_upsampling(tmp_path):
    """The generator of the reference's GAN model on its own layer classes (six times UpSampling 2x2 + Convolution 3x3):
    the drop-in classes compute each convolution from the up-sampling layer's input; the images are those of the run
    with every call made at once (same weights: a row of the last image summed, 256 values after seven layers)."""
    import json
    if not os.path.exists(LAYERS_GPU):
        pytest.skip("oracle/_ref/layers_mi355 not built (it needs /root/reference)")
    run = subprocess.run([LAYERS_GPU, str(tmp_path / "t.bin"), "time", "2", "1", "literal"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr + run.stdout[-2000:]
    lines = [json.loads(l) for l in run.stdout.splitlines() if l.startswith("{")]
    gan = [l for l in lines if l["chain"] == "gan_generator_forward"]
    assert len(gan) == 2 and gan[0]["output"] == [32, 3, 192, 256]
    deferred, literal = gan[0]["last_row_abs_sum"], gan[1]["last_row_abs_sum"]
    assert literal > 1.0 and abs(deferred - literal) <= 1e-5 * literal


def test_deferred_weight_gradients_in_the_reference_layers(tmp_path):
    """Two training steps (forward, backward, gradient descent) of the DCGAN-64 discriminator at batch 16 on the reference's own layer
    classes: the drop-in classes defer the per-sample weight gradients of the last two convolution layers (their sums
    over the batch are computed directly); the updated weights must be those of the run with every call made at once."""
    if not os.path.exists(LAYERS_GPU):
        pytest.skip("oracle/_ref/layers_mi355 not built (it needs /root/reference)")
    path = str(tmp_path / "k.bin")
    run = subprocess.run([LAYERS_GPU, path, "deferred"], capture_output=True, text=True, timeout=180)
    assert run.returncode == 0, run.stderr + run.stdout[-2000:]
    d = read_dump(path)
    for layer in (1, 2, 3, 4):
        for part in (0, 1):
            a, b = d["K.deferred.conv%d.%d" % (layer, part)], d["K.eager.conv%d.%d" % (layer, part)]
            assert a.shape == b.shape
            # (the biases sit in front of a batch normalisation: their gradients are rounding noise around zero)
            assert np.abs(a - b).max() <= 1e-6 + 1e-4 * np.abs(b).max(), (layer, part, np.abs(a - b).max(), np.abs(b).max())
    assert rel_err(d["K.deferred.out"], d["K.eager.out"]) <= 1e-4
    kernel = d["K.eager.conv4.0"]
    assert kernel.shape == (1, 1, 512, 4096) and kernel.std() > 0.005
