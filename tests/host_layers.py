"""numpy restatements of the reference layers that work on the host, element by element, through CTensor::GetElement /
SetElement (no tensor-library call to compare with), and the checks of what the reference's own classes produce for
them in chain H of oracle/ref_layers_harness.cpp.  Used on the dump of the reference's CPU build (no GPU needed: this
pins the restatements) and on the dump of the same classes on the drop-in tensors."""
import io
import struct

import numpy as np


def softmax_forward(x):
    """netlayer/cnetlayersoftmax.cu.h:235-271: exp(x) over the sum of exp over all elements of the sample (double sum)."""
    e = np.exp(x.astype(np.float32))
    total = e.astype(np.float64).reshape(len(x), -1).sum(axis=1).reshape(-1, 1, 1, 1)
    return (e / total).astype(np.float32)


def softmax_backward(x, error):
    """netlayer/cnetlayersoftmax.cu.h:420-470: delta_i = sum_{k != i} (-e_i e_k / S^2) c_k + e_i (S - e_i) / S^2 c_i."""
    b = len(x)
    e = np.exp(x.astype(np.float64)).reshape(b, -1)
    c = error.astype(np.float64).reshape(b, -1)
    s = e.sum(axis=1, keepdims=True)
    dot = (e * c).sum(axis=1, keepdims=True)
    delta = -e * (dot - e * c) / s ** 2 + e * (s - e) / s ** 2 * c
    return delta.reshape(x.shape).astype(np.float32)


def depool_forward(x, py, px):
    """netlayer/cnetlayermaxdepooling.cu.h:246-290: every input element fills its py x px block (no division)."""
    return np.repeat(np.repeat(x, py, axis=2), px, axis=3)


def depool_backward(error, py, px):
    """netlayer/cnetlayermaxdepooling.cu.h:383-431: the mean of the block's errors."""
    b, z, y, x = error.shape
    return (error.reshape(b, z, y // py, py, x // px, px).sum(axis=(3, 5), dtype=np.float32) / np.float32(py * px)).astype(np.float32)


def check_chain_h(d, tol=2e-6):
    """`d`: name -> array, the dump of one harness build.  Raises AssertionError with the entry's name."""
    def close(name, want, t=tol):
        got = d[name]
        assert got.shape == want.shape, name
        err = np.max(np.abs(got.astype(np.float64) - want)) / max(np.max(np.abs(want)), 1e-30)
        assert err <= t, (name, err)

    # soft-max
    close("H.softmax", softmax_forward(d["H.soft_input"]))
    assert np.allclose(d["H.softmax"].reshape(len(d["H.softmax"]), -1).sum(axis=1), 1.0, atol=1e-5)
    close("H.soft_delta", softmax_backward(d["H.soft_input"], d["H.soft_error"]), 2e-5)

    # splitter (netlayer/cnetlayersplitter.cu.h:229-232, 374-383): output = input; the two consumers' errors add up
    assert np.array_equal(d["H.split_output"], d["H.split_input"])
    close("H.split_tanh", np.tanh(d["H.split_input"].astype(np.float64)), 1e-6)
    through_tanh = d["H.split_error_b"] * (np.float32(1) - d["H.split_tanh"] * d["H.split_tanh"])
    close("H.split_delta", (d["H.split_error_a"] + through_tanh).astype(np.float64), 1e-6)
    assert np.array_equal(d["H.split_prev_delta"], d["H.split_delta"])

    # drop-out (netlayer/cnetlayerdropout.cu.h:199-226, 330-336): mask elements are 0 or 1/(1-p); the error passes the same mask
    x, out = d["H.drop_input"], d["H.drop_output"]
    assert np.array_equal(d["H.drop_inference"], x)
    scale = np.float32(1.0 / (1.0 - 0.25))
    kept = out != 0
    assert np.array_equal(out[kept], (x * scale)[kept]) and np.all(x[~kept] != 0)
    assert 0.65 <= kept.mean() <= 0.85, kept.mean()                     # 1536 draws at p = 0.75: +-0.1 is nine sigma
    assert np.array_equal(d["H.drop_prev_delta"], np.where(kept, d["H.drop_error"] * scale, np.float32(0)))
    assert struct.unpack("=d", d["H.drop_stream"].tobytes()) == (0.25,)

    # output of a VAE coder (netlayer/cnetlayervaecoderoutput.cu.h:243-282, 438-470); the noise is recovered from the output
    mu, logvar, out, err = (d[k].astype(np.float64) for k in ("H.vae_mu", "H.vae_logvar", "H.vae_output", "H.vae_error"))
    assert np.abs(logvar).max() > 10                                   # the forward pass clamps, the error pass does not
    sigma = np.exp(np.clip(logvar, -10, 10) / 2)
    noise = (out - mu) / sigma
    assert abs(noise.mean()) < 0.5 and 0.6 < noise.std() < 1.4, (noise.mean(), noise.std())    # 96 draws of N(0,1)
    assert np.array_equal(d["H.vae_delta_mu0"], d["H.vae_error"])
    # relative to the largest term: the recovered noise carries the rounding of `out`
    want0 = err * 0.5 * noise * np.exp(logvar / 2)
    close("H.vae_delta_logvar0", want0, 2e-4)
    k = 0.125
    close("H.vae_delta_mu", err + mu * k, 1e-6)
    close("H.vae_delta_logvar", want0 - 0.5 * (1 - np.exp(logvar)) * k, 2e-4)

    # max de-pooling, constructed with (y, x) = (2, 3)
    close("H.depool_output", depool_forward(d["H.depool_input"], 2, 3).astype(np.float64), 0)
    close("H.depool_prev_delta", depool_backward(d["H.depool_error"], 2, 3).astype(np.float64), 1e-6)
    assert struct.unpack("=2I", d["H.depool_stream"].tobytes()) == (3, 2)
