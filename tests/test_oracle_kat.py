"""The CPU oracle against every known-answer vector the reference's self-test holds
(cuda/ctensortest.cu.h) and against the committed vectors produced by the compiled
reference headers (tests/golden/ref_vectors.npz).  Integer-valued KATs and all
golden vectors must match bit for bit."""
import numpy as np
import pytest

import oracle_api
from cases import batch, rule


def test_kat_forward_convolution(oracle, kat):
    k = kat["forward_convolution"]
    image = batch(np.array(k["image"], np.float32).reshape(1, *k["image_shape"]))
    kernel = np.array(k["kernels"], np.float32).reshape(1, 1, 2, 12)
    out = oracle.forward_convolution(image, kernel, np.zeros((1, 2, 1, 1)), 2, 2, 3, 2, 1, 1, 0, 0)
    want = np.array(k["expected"], np.float32).reshape(k["expected_shape"])
    for w in range(10):
        assert np.array_equal(out[w], want)


def test_kat_forward_convolution_step_padding(oracle, kat, golden):
    k = kat["forward_convolution_step_padding"]
    image = batch(np.array(k["image"], np.float32).reshape(1, *k["image_shape"]))
    kernel = np.array(k["kernels"], np.float32).reshape(1, 1, 2, 27)
    out = oracle.forward_convolution(image, kernel, np.zeros((1, 2, 1, 1)), 3, 3, 3, 2, 2, 2, 1, 1)
    assert out.shape == (10, 2, 3, 3)
    for w in range(10):
        assert np.array_equal(out[w], golden["fwd_s2p1_out"][0])


def test_kat_delta_weight_step_padding(oracle, kat):
    k = kat["delta_weight_step_padding"]
    image, delta = batch(rule((7, 7), 7)), batch(rule((4, 4), 4))
    dk, db = oracle.create_delta_weight_and_bias(np.zeros((10, 1, 1, 25)), np.zeros((10, 1, 1, 1)), image, delta,
                                                 5, 5, 1, 1, 2, 2, 2, 2)
    for w in range(10):
        assert np.array_equal(dk[w].ravel(), np.array(k["expected_dkernel"], np.float32))
        assert db[w, 0, 0, 0] == 136  # 1+2+...+16


def test_kat_delta_weight(oracle, kat):
    k = kat["delta_weight"]
    image = batch(np.array(k["image"], np.float32).reshape(1, 1, 4, 4))
    delta = batch(np.array(k["delta"], np.float32).reshape(1, 1, 2, 2))
    dk, db = oracle.create_delta_weight_and_bias(np.zeros((10, 1, 1, 9)), np.zeros((10, 1, 1, 1)), image, delta,
                                                 3, 3, 1, 1, 1, 1, 0, 0)
    for w in range(10):
        assert np.array_equal(dk[w].ravel(), np.array(k["expected_dkernel"], np.float32))


def test_kat_backward_convolution_step_padding(oracle, kat):
    k = kat["backward_convolution_step_padding"]
    kernel = rule((5, 5), 5).reshape(1, 1, 1, 25)
    delta = batch(rule((4, 4), 4))
    out = oracle.backward_convolution(delta, kernel, np.zeros((1, 1, 1, 1)), 5, 5, 1, 1, 2, 2, 2, 2, (10, 1, 7, 7))
    want = np.array(k["expected"], np.float32).reshape(1, 7, 7)
    for w in range(10):
        assert np.array_equal(out[w], want)


def test_kat_matrix_ops(oracle, kat):
    k = kat["matrix"]
    a = batch(np.array(k["a"], np.float32).reshape(1, 1, 2, 2))
    b = batch(np.array(k["b"], np.float32).reshape(1, 1, 2, 2))
    one = a[:1]
    arr = lambda key: np.array(k[key], np.float32).reshape(2, 2)
    assert all(np.array_equal(oracle.mul_value(a, 2.0)[w, 0], arr("scaled_by_2")) for w in range(10))
    for left, right in ((a, b), (one, b), (a, one)):  # W broadcast both ways (ctensortest.cu.h:816-842)
        out = oracle.mul(left, right)
        assert out.shape == (10, 1, 2, 2)
        assert all(np.array_equal(out[w, 0], arr("mul")) for w in range(10))
    assert np.array_equal(oracle.sub(a, b)[3, 0], arr("sub"))
    assert np.array_equal(oracle.add(a, b)[3, 0], arr("add"))
    assert np.array_equal(oracle.transponse(a)[3, 0], arr("transpose_a"))
    assert np.array_equal(oracle.tensor_item_production(a, b)[3, 0], arr("item_production"))


def test_kat_summ_xy(oracle, kat):
    w, z = kat["summ_xy"]["shape_wz"]
    for s in kat["summ_xy"]["sizes"][:6]:  # 1..161; larger sizes repeat the same path
        out = oracle.summ_xy(np.ones((w, z, s, s), np.float32))
        assert out.shape == (w, z, 1, 1)
        assert np.all(out == s * s)


# ---- vectors written by the compiled reference -------------------------------

def test_golden_forward(oracle, golden):
    g = golden
    out = oracle.forward_convolution(g["fwd_image"], g["fwd_kernel"], g["fwd_bias"], 2, 3, 4, 5, 2, 1, 1, 2)
    assert np.array_equal(out, g["fwd_out"])


@pytest.mark.parametrize("key,stride,pad,shape", [("tconv_out_s2", 2, 1, (2, 2, 8, 10)), ("tconv_out_s3", 3, 0, (2, 2, 13, 16)),
                                                   ("tconv_out_s1", 1, 2, (2, 2, 3, 4))])
def test_golden_tconv_nonzero_bias(oracle, golden, key, stride, pad, shape):
    g = golden
    out = oracle.backward_convolution(g["tconv_delta"], g["tconv_kernel"], g["tconv_bias"], 4, 4, 2, 3, stride, stride, pad, pad, shape)
    assert np.array_equal(out, g[key])


def test_golden_wgrad(oracle, golden):
    g = golden
    dk, db = oracle.create_delta_weight_and_bias(g["wgrad_dk0"], g["wgrad_db0"], g["wgrad_image"], g["wgrad_delta"], 3, 3, 2, 4, 2, 2, 1, 1)
    assert np.array_equal(dk, g["wgrad_dk"]) and np.array_equal(db, g["wgrad_db"])


def test_golden_max_pooling(oracle, golden):
    g = golden
    pooled, pos = oracle.max_pooling(g["maxpool_in"], 2, 3)
    assert np.array_equal(pos, g["maxpool_pos"])
    assert np.array_equal(pooled, g["maxpool_out"], equal_nan=True)
    back = oracle.max_pooling_backward(g["maxpool_back_delta"], g["maxpool_pos"], 2, 3, (2, 2, 6, 6))
    assert np.array_equal(back, g["maxpool_back_out"])


@pytest.mark.parametrize("name", sorted(oracle_api.FUNC))
def test_golden_activations(oracle, golden, name):
    assert np.array_equal(oracle.apply_func(golden["act_in"], name), golden["act_" + name])
    assert np.array_equal(oracle.apply_func(golden["act_in"], name, differential=True), golden["dact_" + name])


def test_golden_resampling(oracle, golden):
    assert np.array_equal(oracle.downsampling(golden["down_in"], 2, 3), golden["down_out"])
    assert np.array_equal(oracle.upsampling(golden["down_in"], 2, 3, out_shape=(2, 2, 23, 19)), golden["up_out"])


def test_golden_add_sum_w(oracle, golden):
    out = oracle.add_sum_w(golden["addsumw_l"], golden["addsumw_r"], 0.5, 1.0 / 5.0, out_w=3)
    assert np.array_equal(out, golden["addsumw_out"])
    assert np.all(out[1:] == 0)


@pytest.mark.parametrize("it", [1, 7])
def test_golden_adam(oracle, golden, it):
    g = golden
    w, m, v = oracle.adam(g["adam_w"], g["adam_dw"], g["adam_m"], g["adam_v"], 16, 0.0002, 0.5, 0.9, 1e-8, float(it))
    assert np.array_equal(w, g["adam_w_it%d" % it])
    assert np.array_equal(m, g["adam_m_it%d" % it])
    assert np.array_equal(v, g["adam_v_it%d" % it])


def test_golden_products(oracle, golden):
    assert np.array_equal(oracle.mul(golden["mul_a"], golden["mul_b"]), golden["mul_out"])
    assert np.array_equal(oracle.transponse_mul(golden["tmul_a"], golden["mul_b"]), golden["tmul_out"])
