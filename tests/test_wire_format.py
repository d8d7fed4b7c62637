"""The checkpoint wire format (wire_format.py): round trips, and the byte streams that the reference's OWN layer classes
write with Save() -- `oracle/_ref/layers_cpu` is the reference's convolution and linear layers on its CPU tensor classes,
compiled in the authoring container; it stores those streams byte for byte in its dump (entries `*_stream`)."""
import io
import os
import struct
import subprocess

import numpy as np
import pytest

import wire_format as wf
from conftest import ROOT

LAYERS_CPU = os.path.join(ROOT, "oracle", "_ref", "layers_cpu")


def read_dump_bytes(path):
    """name -> (dims, raw bytes of the float32 slots)"""
    out, data, pos = {}, open(path, "rb").read(), 0
    while pos < len(data):
        name = data[pos:pos + 32].split(b"\0")[0].decode()
        dims = struct.unpack_from("<4I", data, pos + 32)
        n = int(np.prod(dims))
        out[name] = (dims, data[pos + 48:pos + 48 + 4 * n])
        pos += 48 + 4 * n
    return out


def as_array(entry):
    return np.frombuffer(entry[1], np.float32).reshape(entry[0])


def test_tensor_round_trip_is_exact():
    rng = np.random.default_rng(1)
    a = rng.standard_normal((2, 3, 4, 5)).astype(np.float32)
    a[0, 0, 0, :3] = (np.float32(1e-40), np.float32(3.4e38), np.float32(-0.0))       # denormal, near the maximum, signed zero
    f = io.BytesIO()
    wf.write_tensor(f, a)
    assert len(f.getvalue()) == 16 + 8 * a.size
    assert struct.unpack_from("=4I", f.getvalue()) == (2, 3, 4, 5)
    f.seek(0)
    b = wf.read_tensor(f)
    assert b.dtype == np.float32 and np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_empty_tensor_and_truncated_streams():
    f = io.BytesIO()
    wf.write_tensor(f, np.zeros((0, 1, 1, 1), np.float32))      # the reference writes the four sizes and no values
    assert len(f.getvalue()) == 16
    f.seek(0)
    assert wf.read_tensor(f).shape == (0, 1, 1, 1)
    with pytest.raises(EOFError):
        wf.read_tensor(io.BytesIO(b"\x01\0\0\0"))
    with pytest.raises(EOFError):
        wf.read_tensor(io.BytesIO(struct.pack("=4I", 1, 1, 1, 2) + b"\0" * 8))


def test_layer_round_trips():
    rng = np.random.default_rng(2)
    header = dict(kernel_amount=4, kernel_x=3, kernel_y=2, kernel_z=5, stride_x=2, stride_y=1, padding_x=1, padding_y=0)
    kernel, bias = rng.standard_normal((1, 1, 4, 30)).astype(np.float32), rng.standard_normal((1, 4, 1, 1)).astype(np.float32)
    f = io.BytesIO()
    wf.write_convolution_layer(f, header, kernel, bias)
    wf.write_linear_layer(f, kernel, bias.reshape(1, 1, 4, 1))
    bn = [rng.standard_normal((1, 2, 3, 3)).astype(np.float32) for _ in range(4)]
    wf.write_batchnorm_layer(f, *bn, momentum=0.9)
    f.seek(0)
    h, k, b = wf.read_convolution_layer(f)
    assert h == header and np.array_equal(k, kernel) and np.array_equal(b, bias)
    w, lb = wf.read_linear_layer(f)
    assert np.array_equal(w, kernel) and lb.shape == (1, 1, 4, 1)
    got = wf.read_batchnorm_layer(f)
    assert all(np.array_equal(g, t) for g, t in zip(got[:4], bn)) and got[4] == 0.9
    assert f.read() == b""


@pytest.fixture(scope="module")
def cpu_dump(tmp_path_factory):
    if not os.path.exists(LAYERS_CPU):
        pytest.skip("oracle/_ref/layers_cpu not built (it needs /root/reference)")
    path = str(tmp_path_factory.mktemp("wire") / "cpu.bin")
    run = subprocess.run([LAYERS_CPU, path], capture_output=True, text=True, timeout=180)
    assert run.returncode == 0, run.stderr
    return read_dump_bytes(path)


def test_streams_written_by_the_reference_layers(cpu_dump):
    """CNetLayerConvolution::Save and CNetLayerLinear::Save of the reference, parsed here; the tensors must equal the ones
    the harness itself read back from the same streams with the reference's stream interface."""
    header, kernel, bias = wf.read_convolution_layer(io.BytesIO(cpu_dump["A.conv_stream"][1]))
    want_k, want_b = as_array(cpu_dump["A.conv_updated.0"]), as_array(cpu_dump["A.conv_updated.1"])
    assert kernel.shape == want_k.shape and np.array_equal(kernel, want_k)
    assert bias.shape == want_b.shape and np.array_equal(bias, want_b)
    assert header["kernel_amount"] == kernel.shape[2]
    assert header["kernel_x"] * header["kernel_y"] * header["kernel_z"] == kernel.shape[3]
    assert header["stride_x"] >= 1 and header["stride_y"] >= 1 and header["padding_x"] >= 0 and header["padding_y"] >= 0

    stream = io.BytesIO(cpu_dump["A.linear_stream"][1])
    weight, lbias = wf.read_linear_layer(stream)
    assert stream.read() == b""
    assert np.array_equal(weight, as_array(cpu_dump["A.linear_updated.0"]))
    assert np.array_equal(lbias, as_array(cpu_dump["A.linear_updated.1"]))

    # written back, the bytes are the reference's own
    f = io.BytesIO()
    wf.write_convolution_layer(f, header, kernel, bias)
    assert f.getvalue() == cpu_dump["A.conv_stream"][1]
    f = io.BytesIO()
    wf.write_linear_layer(f, weight, lbias)
    assert f.getvalue() == cpu_dump["A.linear_stream"][1]


def test_whole_networks_written_by_the_reference(cpu_dump):
    """Every layer of a chain saved into one stream, the way CModelMain::SaveNetLayers writes a network file."""
    raw = cpu_dump["A.net_stream"][1]
    kinds = ["input", "convolution", "function", "linear", "function"]
    net = wf.read_net(io.BytesIO(raw), kinds)
    assert [k for k, _ in net] == kinds
    assert net[2][1]["name"] == "leaky_relu" and net[4][1]["name"] == "sigmoid"
    assert np.array_equal(net[1][1]["kernel"], as_array(cpu_dump["A.conv_updated.0"]))
    assert np.array_equal(net[3][1]["bias"], as_array(cpu_dump["A.linear_updated.1"]))
    f = io.BytesIO()
    wf.write_net(f, net)
    assert f.getvalue() == raw

    raw = cpu_dump["D.net_stream"][1]
    net = wf.read_net(io.BytesIO(raw), ["input", "upsampling", "averagepooling"])
    assert net[1][1] == {"x": 2, "y": 2} and net[2][1] == {"x": 4, "y": 4}
    f = io.BytesIO()
    wf.write_net(f, net)
    assert f.getvalue() == raw

    header, kernel, _ = wf.read_convolution_layer(io.BytesIO(cpu_dump["B.tconv_stream"][1]))   # transposed convolution
    assert np.array_equal(kernel, as_array(cpu_dump["B.tconv_updated.0"]))
    assert (header["kernel_amount"], header["kernel_z"]) == (kernel.shape[2], kernel.shape[3] // 16)


def test_net_round_trip_of_the_other_layer_kinds():
    f = io.BytesIO()
    layers = [("input", {}), ("dropout", {"rate": 0.25}), ("maxpooling", {"x": 2, "y": 3}), ("function", {"name": "gelu"}),
              ("softmax", {}), ("splitter", {}), ("vae_coder_output", {}), ("concatenator", {}), ("time_embedding", {})]
    wf.write_net(f, layers)
    assert len(f.getvalue()) == 8 + 8 + 4
    f.seek(0)
    assert wf.read_net(f, [k for k, _ in layers]) == layers
    with pytest.raises(ValueError):
        wf.read_net(io.BytesIO(struct.pack("=I", 9)), ["function"])
    with pytest.raises(EOFError):
        wf.read_net(io.BytesIO(b""), ["upsampling"])


def chain_g_network(seed=3):
    """The layers of the harness's chain G with weights of our own."""
    rng = np.random.default_rng(seed)
    header = dict(kernel_amount=8, kernel_x=4, kernel_y=4, kernel_z=3, stride_x=2, stride_y=2, padding_x=1, padding_y=1)
    return [("input", {}),
            ("convolution", {"header": header, "kernel": (rng.standard_normal((1, 1, 8, 48)) * 0.2).astype(np.float32),
                             "bias": (rng.standard_normal((1, 8, 1, 1)) * 0.1).astype(np.float32)}),
            ("function", {"name": "leaky_relu"}),
            ("linear", {"weight": (rng.standard_normal((1, 1, 24, 512)) * 0.08).astype(np.float32),
                        "bias": (rng.standard_normal((1, 1, 24, 1)) * 0.1).astype(np.float32)}),
            ("function", {"name": "sigmoid"})]


def run_chain_g(exe, layers, tmp_path):
    net, dump = str(tmp_path / "net.bin"), str(tmp_path / "g.bin")
    with open(net, "wb") as f:
        wf.write_net(f, layers)
    run = subprocess.run([exe, dump, net], capture_output=True, text=True, timeout=180)
    assert run.returncode == 0, run.stderr
    return {k: as_array(v) for k, v in read_dump_bytes(dump).items()}


def expected_chain_g(lib, layers, image):
    import layer_sequences as seq
    conv, lin = layers[1][1], layers[3][1]
    a = lib.apply_func(seq.conv_forward(lib, image, conv["kernel"], conv["bias"], 4, 2, 1), "leaky_relu")
    out = seq.linear_forward(lib, lin["weight"], a.reshape(a.shape[0], 1, -1, 1), lin["bias"])
    return a, lib.apply_func(out, "sigmoid")


def test_reference_layers_load_a_network_written_here(oracle, tmp_path):
    """The other direction: a network file written by wire_format.py, loaded by the reference's own convolution, function
    and linear layers (on the reference's CPU tensor classes) with Load(); their forward pass must be the oracle's on
    the same weights.  The function layer is constructed as a sigmoid and becomes a leaky ReLU by loading."""
    if not os.path.exists(LAYERS_CPU):
        pytest.skip("oracle/_ref/layers_cpu not built (it needs /root/reference)")
    layers = chain_g_network()
    got = run_chain_g(LAYERS_CPU, layers, tmp_path)
    leaky, prob = expected_chain_g(oracle, layers, got["G.input"])
    assert np.array_equal(got["G.leaky"], leaky)
    assert np.max(np.abs(got["G.sigmoid"] - prob.reshape(got["G.sigmoid"].shape))) <= 1e-6


def test_training_state_written_by_the_reference(cpu_dump):
    """Iteration and Adam moments of chain A as SaveNetLayersTrainingParam writes them: the moments have the shapes of
    the parameters, the convolution's come back in the order they were loaded in, and the bytes survive a round trip."""
    raw = cpu_dump["A.train_stream"][1]
    kinds = ["input", "convolution", "function", "linear", "function"]
    iteration, layers = wf.read_training_params(io.BytesIO(raw), kinds)
    assert iteration == 7
    conv, lin = layers[1][1], layers[3][1]
    assert conv["m_weight"].shape == conv["v_weight"].shape == as_array(cpu_dump["A.conv_updated.0"]).shape
    assert conv["m_bias"].shape == as_array(cpu_dump["A.conv_updated.1"]).shape
    assert lin["m_weight"].shape == as_array(cpu_dump["A.linear_updated.0"]).shape and lin["v_bias"].shape == as_array(cpu_dump["A.linear_updated.1"]).shape
    # the convolution layer was given known moments through its LoadTrainingParam: their order in the stream
    for name, key in (("m_weight", "A.mk"), ("v_weight", "A.vk"), ("m_bias", "A.mb"), ("v_bias", "A.vb")):
        assert np.array_equal(conv[name], as_array(cpu_dump[key])) and np.abs(conv[name]).max() > 0, name
    assert not np.array_equal(conv["m_weight"], conv["v_weight"])
    f = io.BytesIO()
    wf.write_training_params(f, iteration, layers)
    assert f.getvalue() == raw


@pytest.mark.parametrize("model", ["discriminator", "gan_generator"])
def test_model_files_keep_the_running_statistics(model):
    """What the Python models write for a network and read back (host side, no device): a stream whose batch-norm layers
    carry trained running statistics, read into the model's parameter dictionary and written again, is the same bytes,
    so loading a trained network and saving it loses nothing."""
    import importlib
    mod = importlib.import_module(model)
    rng = np.random.default_rng(7)
    if model == "discriminator":
        host = dict(mod.make_parameters(), **mod.make_statistics())
        layers_of, kinds = mod.net_layers, mod.LAYER_KINDS
    else:
        channels = (8, 8, 4, 4, 2, 2, 2)
        host = dict(mod.make_parameters(channels, 16), **mod.make_statistics(channels))
        layers_of, kinds = (lambda h: mod.net_layers(h, channels)), mod.LAYER_KINDS
    for name in host:
        if name.startswith("mean"):
            host[name] = rng.standard_normal(host[name].shape).astype(np.float32)
        if name.startswith("variable"):
            host[name] = rng.uniform(0.2, 3.0, host[name].shape).astype(np.float32)
    first = io.BytesIO()
    wf.write_net(first, layers_of(host))
    back = mod.host_from_layers(wf.read_net(io.BytesIO(first.getvalue()), kinds))
    assert sorted(back) == sorted(host)
    for name in host:
        assert np.array_equal(back[name], host[name]), name
    second = io.BytesIO()
    wf.write_net(second, layers_of(back))
    assert second.getvalue() == first.getvalue()
    # the statistics sit where the reference's layer reads them: third and fourth tensor of a batch-norm layer
    norm = [p for kind, p in wf.read_net(io.BytesIO(first.getvalue()), kinds) if kind == "batchnorm"][0]
    assert np.array_equal(norm["mean"], host["mean0"]) and np.array_equal(norm["variable"], host["variable0"])


def test_averaged_weights_written_by_the_reference(cpu_dump):
    """SaveEMAWeight of every layer of chain A after one update step with averaging enabled: the stream has the layout of
    the network stream, its tensors are EMA_K * loaded + (1 - EMA_K) * updated (netlayer/cnetlayerconvolution.cu.h:547-551,
    cnetlayerlinear.cu.h:478-482), and writing them back gives the reference's bytes."""
    kinds = ["input", "convolution", "function", "linear", "function"]
    raw = cpu_dump["A.ema_stream"][1]
    net = wf.read_ema(io.BytesIO(raw), kinds)
    conv, lin = net[1][1], net[3][1]
    assert np.array_equal(conv["kernel"], as_array(cpu_dump["A.conv_ema.0"])) and np.array_equal(conv["bias"], as_array(cpu_dump["A.conv_ema.1"]))
    assert np.array_equal(lin["weight"], as_array(cpu_dump["A.linear_ema.0"])) and np.array_equal(lin["bias"], as_array(cpu_dump["A.linear_ema.1"]))
    assert net[2][1]["name"] == "leaky_relu" and conv["header"]["kernel_amount"] == 8
    k, rest = np.float32(wf.EMA_K), np.float32(1.0 - wf.EMA_K)
    for got, loaded, updated in ((conv["kernel"], "A.conv_loaded.0", "A.conv_updated.0"), (conv["bias"], "A.conv_loaded.1", "A.conv_updated.1"),
                                 (lin["weight"], "A.linear_loaded.0", "A.linear_updated.0"), (lin["bias"], "A.linear_loaded.1", "A.linear_updated.1")):
        w0, w1 = as_array(cpu_dump[loaded]), as_array(cpu_dump[updated])
        assert np.abs(w1 - w0).max() > 1e-4                               # the step moved the weights
        assert np.array_equal(got, k * w0 + rest * w1), loaded            # rounded product by product, like CTensorMath::Add
        assert not np.array_equal(got, w0) and not np.array_equal(got, w1)
    f = io.BytesIO()
    wf.write_ema(f, net)
    assert f.getvalue() == raw
    # written from the last layer to the first (SaveNetLayersEMAWeight with backward = true) and read back in network order
    f = io.BytesIO()
    wf.write_ema(f, net, backward=True)
    assert f.getvalue() != raw and len(f.getvalue()) == len(raw)
    back = wf.read_ema(io.BytesIO(f.getvalue()), kinds, backward=True)
    assert [k for k, _ in back] == kinds and np.array_equal(back[3][1]["weight"], lin["weight"])


def test_averaged_weights_of_a_network_that_never_enabled_them(cpu_dump):
    """Before EnableEMA(true) the layers hold [1,1,1,1] tensors in place of the averages and write those."""
    kinds = ["input", "convolution", "function", "linear", "function"]
    raw = cpu_dump["A.ema_off_stream"][1]
    net = wf.read_ema(io.BytesIO(raw), kinds)
    assert net[1][1]["kernel"].shape == net[1][1]["bias"].shape == net[3][1]["weight"].shape == (1, 1, 1, 1)
    header = net[1][1]["header"]
    mine = [("input", {}), ("convolution", dict(wf.ema_disabled("convolution"), header=header)), ("function", {"name": "leaky_relu"}),
            ("linear", wf.ema_disabled("linear")), ("function", {"name": "sigmoid"})]
    f = io.BytesIO()
    wf.write_ema(f, mine)
    assert f.getvalue() == raw


def test_host_side_layers_of_the_reference(cpu_dump):
    """Soft-max, splitter, drop-out, VAE coder output and max de-pooling of the reference on its CPU tensor classes against
    the numpy restatements in host_layers.py (which the GPU tests then use on the drop-in build of the same classes)."""
    import host_layers
    host_layers.check_chain_h({k: as_array(v) for k, v in cpu_dump.items() if k.startswith("H.")})
    layers = wf.read_net(io.BytesIO(cpu_dump["H.drop_stream"][1] + cpu_dump["H.depool_stream"][1]), ["dropout", "maxdepooling"])
    assert layers == [("dropout", {"rate": 0.25}), ("maxdepooling", {"x": 3, "y": 2})]
