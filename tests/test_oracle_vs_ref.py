"""The C restatement against the reference's own CPU headers (oracle/_ref), bit for bit,
on seeded random and edge-case inputs.  Skipped where the reference build is absent."""
import numpy as np
import pytest

import oracle_api
from cases import rng_uniform as U


def same(a, b):
    return np.array_equal(a, b, equal_nan=True)


CONV_CASES = [
    # W, C, H, Wd, K_amount, kx, ky, sx, sy, px, py, kernel_W, bias_W
    (2, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1),
    (3, 2, 9, 7, 5, 2, 4, 2, 1, 0, 2, 1, 1),
    (2, 1, 6, 6, 1, 5, 5, 2, 2, 2, 2, 2, 2),
    (4, 3, 16, 16, 8, 4, 4, 2, 2, 1, 1, 1, 1),
    (1, 5, 5, 5, 3, 5, 5, 1, 1, 0, 0, 1, 1),
    (2, 2, 7, 10, 3, 3, 3, 3, 2, 1, 0, 1, 2),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_forward_convolution(oracle, ref, case):
    W, C, H, Wd, KA, kx, ky, sx, sy, px, py, kw, bw = case
    image, kernel, bias = U(1, W, C, H, Wd), U(2, kw, 1, KA, C * kx * ky), U(3, bw, KA, 1, 1)
    args = (image, kernel, bias, kx, ky, C, KA, sx, sy, px, py)
    assert same(oracle.forward_convolution(*args), ref.forward_convolution(*args))
    # image broadcast over a larger output batch
    assert same(oracle.forward_convolution(*args, out_w=W + 2), ref.forward_convolution(*args, out_w=W + 2))


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("with_bias", [False, True])
def test_backward_convolution(oracle, ref, case, with_bias):
    W, C, H, Wd, KA, kx, ky, sx, sy, px, py, kw, bw = case
    oy, ox = (H - ky + 2 * py) // sy + 1, (Wd - kx + 2 * px) // sx + 1
    delta, kernel = U(4, W, KA, oy, ox), U(5, kw, 1, KA, C * kx * ky)
    bias = U(6, bw, KA, 1, 1) if with_bias else np.zeros((bw, KA, 1, 1), np.float32)
    # the layer's natural output size, and a deliberately different one (the size comes from the output tensor)
    for shape in ((W, C, H, Wd), (W, C, H + 1, Wd - 1)):
        args = (delta, kernel, bias, kx, ky, C, KA, sx, sy, px, py, shape)
        assert same(oracle.backward_convolution(*args), ref.backward_convolution(*args))


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("back", [False, True])
def test_create_delta_weight_and_bias(oracle, ref, case, back):
    W, C, H, Wd, KA, kx, ky, sx, sy, px, py, kw, bw = case
    oy, ox = (H - ky + 2 * py) // sy + 1, (Wd - kx + 2 * px) // sx + 1
    big, small = U(7, W, C, H, Wd), U(8, W, KA, oy, ox)
    dk0, db0 = U(9, W, 1, KA, C * kx * ky), U(10, W, KA, 1, 1)
    if back:  # the transposed layer passes its (small) input as "image" and the (big) output delta as "delta"
        args = (dk0, db0, small, big, kx, ky, C, KA, sx, sy, px, py)
    else:
        args = (dk0, db0, big, small, kx, ky, C, KA, sx, sy, px, py)
    a, b = oracle.create_delta_weight_and_bias(*args, back=back), ref.create_delta_weight_and_bias(*args, back=back)
    assert same(a[0], b[0]) and same(a[1], b[1])


def test_wgrad_w_broadcast(oracle, ref):
    # dKernel batch larger than image/delta batch; shared dBias row (w % W)
    image, delta = U(1, 2, 2, 6, 6), U(2, 1, 3, 6, 6)
    dk0, db0 = np.zeros((4, 1, 3, 18), np.float32), np.zeros((2, 3, 1, 1), np.float32)
    args = (dk0, db0, image, delta, 3, 3, 2, 3, 1, 1, 1, 1)
    a, b = oracle.create_delta_weight_and_bias(*args), ref.create_delta_weight_and_bias(*args)
    assert same(a[0], b[0]) and same(a[1], b[1])


@pytest.mark.parametrize("m,k,n,wl,wr,z", [(1, 1, 1, 1, 1, 1), (33, 65, 31, 1, 3, 2), (64, 100, 1, 1, 5, 1), (70, 32, 96, 2, 2, 1), (5, 300, 7, 3, 1, 1)])
def test_products(oracle, ref, m, k, n, wl, wr, z):
    a, b, at = U(1, wl, z, m, k), U(2, wr, z, k, n), U(3, wl, z, k, m)
    assert same(oracle.mul(a, b), ref.mul(a, b))
    assert same(oracle.transponse_mul(at, b), ref.transponse_mul(at, b))
    assert same(oracle.transponse(a), ref.transponse(a))


def test_elementwise(oracle, ref):
    l, r, one = U(1, 3, 2, 5, 7), U(2, 3, 2, 5, 7), U(3, 1, 2, 5, 7)
    for name in ("add", "sub", "div"):
        for (a, b) in ((l, r), (l, one), (one, r)):
            assert same(getattr(oracle, name)(a, b, 0.3, -1.7), getattr(ref, name)(a, b, 0.3, -1.7))
    assert same(oracle.tensor_item_production(l, one), ref.tensor_item_production(l, one))
    assert same(oracle.tensor_item_production(one, r), ref.tensor_item_production(one, r))
    pos = np.abs(l) + 0.01
    assert same(oracle.inv(l), ref.inv(l))
    assert same(oracle.inv(one, out_w=4), ref.inv(one, out_w=4))
    assert same(oracle.pow2(l, 0.37), ref.pow2(l, 0.37))
    assert same(oracle.sqrt(pos, 1.3, 1e-6), ref.sqrt(pos, 1.3, 1e-6))
    assert same(oracle.sqrt(l, 1.0, 0.0), ref.sqrt(l, 1.0, 0.0))  # negative inputs -> NaN alike
    assert same(oracle.mul_value(l, -2.5), ref.mul_value(l, -2.5))
    assert same(oracle.fill((2, 3, 4, 5), 0.1), ref.fill((2, 3, 4, 5), 0.1))
    assert same(oracle.add_bias(l, U(4, 1, 2, 1, 1)), ref.add_bias(l, U(4, 1, 2, 1, 1)))
    assert same(oracle.add_bias(l, U(4, 3, 2, 1, 1)), ref.add_bias(l, U(4, 3, 2, 1, 1)))
    assert same(oracle.summ_xy(l), ref.summ_xy(l))
    assert same(oracle.summ_xy(one, out_w=3), ref.summ_xy(one, out_w=3))
    assert same(oracle.clip(l, -0.3, 0.4), ref.clip(l, -0.3, 0.4))
    assert same(oracle.signum(np.round(l * 2)), ref.signum(np.round(l * 2)))
    big = U(5, 64, 2, 5, 7) * 100
    assert same(oracle.add_sum_w(l, big, 1.0, 1.0 / 64), ref.add_sum_w(l, big, 1.0, 1.0 / 64))
    assert same(oracle.add_sum_w(l, big, 0.5, 2.0, out_w=2), ref.add_sum_w(l, big, 0.5, 2.0, out_w=2))


def test_resampling_and_pooling(oracle, ref):
    a = U(1, 2, 3, 12, 10)
    for ux, uy in ((2, 2), (1, 3), (4, 1)):
        assert same(oracle.upsampling(a, ux, uy), ref.upsampling(a, ux, uy))
    assert same(oracle.upsampling(a, 2, 2, out_shape=(2, 3, 25, 21)), ref.upsampling(a, 2, 2, out_shape=(2, 3, 25, 21)))
    assert same(oracle.upsampling(a[:1], 2, 2, out_shape=(3, 3, 24, 20)), ref.upsampling(a[:1], 2, 2, out_shape=(3, 3, 24, 20)))
    for dx, dy in ((2, 2), (3, 5), (1, 1), (4, 3)):
        assert same(oracle.downsampling(a, dx, dy), ref.downsampling(a, dx, dy))
        ties = np.round(a * 3)
        o, r = oracle.max_pooling(ties, dx, dy), ref.max_pooling(ties, dx, dy)
        assert same(o[0], r[0]) and same(o[1], r[1])
        d = U(2, *o[0].shape)
        shape = a.shape
        assert same(oracle.max_pooling_backward(d, o[1], dx, dy, shape), ref.max_pooling_backward(d, o[1], dx, dy, shape))


@pytest.mark.parametrize("name", sorted(oracle_api.FUNC))
def test_activations(oracle, ref, name):
    x = np.concatenate([U(1, 4000) * 12, U(2, 2000) * 40, np.array([0.0, -0.0, 30, -30, 30.000002, -30.000002, np.inf, -np.inf], np.float32)])
    x = x.reshape(1, 1, 1, -1)
    for d in (False, True):
        assert same(oracle.apply_func(x, name, d), ref.apply_func(x, name, d))
    assert oracle.func_scalar(0.25, name) == ref.func_scalar(0.25, name)


def test_adam(oracle, ref):
    w, dw, m, v = U(1, 2, 1, 6, 9), U(2, 2, 1, 6, 9) * 30, U(3, 2, 1, 6, 9) * 0.2, np.abs(U(4, 2, 1, 6, 9)) * 0.05
    for it in (1.0, 2.0, 1000.0):
        a, b = oracle.adam(w, dw, m, v, 32, 1e-3, 0.9, 0.999, 1e-8, it), ref.adam(w, dw, m, v, 32, 1e-3, 0.9, 0.999, 1e-8, it)
        assert all(same(x, y) for x, y in zip(a, b))


def test_precondition_failures_agree(oracle, ref):
    """Where the reference throws, the restatement returns an error code (and vice versa)."""
    img, ker, bias = U(1, 1, 2, 5, 5), U(2, 1, 1, 3, 18), U(3, 1, 3, 1, 1)

    def fails(lib, fn):
        try:
            fn(lib)
            return False
        except oracle_api.OracleError:
            return True

    probes = [
        lambda L: L.forward_convolution(img, ker, bias, 3, 3, 2, 3, 1, 1, 1, 1),                          # fine
        lambda L: L.forward_convolution(img, ker, bias, 3, 3, 2, 0, 1, 1, 1, 1),                          # no kernels
        lambda L: L.forward_convolution(img, ker, U(3, 1, 2, 1, 1), 3, 3, 2, 3, 1, 1, 1, 1),              # bias count
        lambda L: L.forward_convolution(img, ker, bias, 3, 3, 2, 3, 1, 1, 1, 1, out_shape=(1, 3, 4, 5)),  # output shape
        lambda L: L.forward_convolution(img, ker, bias, 3, 3, 3, 3, 1, 1, 1, 1),                          # depth
        lambda L: L.backward_convolution(U(4, 1, 3, 5, 5), ker, bias, 3, 3, 2, 3, 1, 1, 1, 1, (1, 2, 5, 5)),
        lambda L: L.backward_convolution(U(4, 1, 3, 5, 5), ker, bias, 3, 3, 2, 3, 1, 1, 1, 1, (1, 3, 5, 5)),
        lambda L: L.backward_convolution(U(4, 1, 2, 5, 5), ker, bias, 3, 3, 2, 3, 1, 1, 1, 1, (1, 2, 5, 5)),
        lambda L: L.create_delta_weight_and_bias(np.zeros((1, 1, 3, 18)), np.zeros((1, 3, 1, 1)), img, U(4, 1, 3, 5, 5), 3, 3, 2, 3, 1, 1, 1, 1),
        lambda L: L.create_delta_weight_and_bias(np.zeros((1, 1, 3, 18)), np.zeros((1, 2, 1, 1)), img, U(4, 1, 3, 5, 5), 3, 3, 2, 3, 1, 1, 1, 1),
        lambda L: L.create_delta_weight_and_bias(np.zeros((1, 1, 3, 18)), np.zeros((1, 3, 1, 1)), img, U(4, 1, 2, 5, 5), 3, 3, 2, 3, 1, 1, 1, 1),
        lambda L: L.create_delta_weight_and_bias(np.zeros((1, 1, 3, 27)), np.zeros((1, 3, 1, 1)), img, U(4, 1, 3, 5, 5), 3, 3, 3, 3, 1, 1, 1, 1),
        lambda L: L.mul(U(1, 1, 1, 3, 4), U(2, 1, 1, 5, 2)),
        lambda L: L.transponse_mul(U(1, 1, 1, 3, 4), U(2, 1, 1, 5, 2)),
        lambda L: L.add(U(1, 1, 1, 3, 4), U(2, 1, 1, 4, 3)),
        lambda L: L.add_sum_w(U(1, 1, 1, 3, 4), U(2, 1, 2, 3, 4)),
        lambda L: L.add_bias(U(1, 1, 2, 3, 4), U(2, 1, 3, 1, 1)),
        lambda L: L.upsampling(U(1, 1, 1, 3, 4), 2, 2, out_shape=(1, 1, 8, 8)),
        lambda L: L.apply_func(U(1, 1, 1, 3, 4), "relu"),
    ]
    for i, probe in enumerate(probes):
        assert fails(oracle, probe) == fails(ref, probe), "probe %d" % i
    assert not fails(oracle, probes[0]) and fails(oracle, probes[1])
