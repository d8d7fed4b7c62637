"""The CPU oracle against what the mathematics fixes, independently of the compiled
reference: float64 library routines (torch conv2d / conv_transpose2d / autograd,
numpy matmul), closed forms and invariants.  A dropped term, a wrong sign or index
or a transposed operand fails at least one of these."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from cases import rng_uniform as U
from conftest import rel_err

TOL = 2e-6  # fp32 accumulation vs a float64 routine on these small sizes


def t64(a):
    return torch.from_numpy(np.asarray(a, np.float64))


CASES = [  # W, C, H, Wd, KA, k, s, p
    (2, 3, 8, 8, 4, 3, 1, 1), (2, 2, 9, 9, 3, 5, 2, 2), (3, 4, 16, 16, 6, 4, 2, 1), (1, 3, 7, 7, 2, 3, 3, 0), (2, 1, 5, 5, 1, 1, 1, 0),
]


@pytest.mark.parametrize("W,C,H,Wd,KA,k,s,p", CASES)
def test_forward_is_conv2d(oracle, W, C, H, Wd, KA, k, s, p):
    image, kernel, bias = U(1, W, C, H, Wd), U(2, 1, 1, KA, C * k * k), U(3, 1, KA, 1, 1)
    got = oracle.forward_convolution(image, kernel, bias, k, k, C, KA, s, s, p, p)
    want = F.conv2d(t64(image), t64(kernel).reshape(KA, C, k, k), t64(bias).reshape(KA), stride=s, padding=p).numpy()
    assert got.shape == want.shape and rel_err(got, want) < TOL


@pytest.mark.parametrize("W,C,H,Wd,KA,k,s,p", CASES)
def test_backward_is_conv_transpose2d(oracle, W, C, H, Wd, KA, k, s, p):
    oy = (H - k + 2 * p) // s + 1
    delta, kernel = U(4, W, KA, oy, oy), U(5, 1, 1, KA, C * k * k)
    natural = s * (oy - 1) + k - 2 * p  # conv_transpose2d's own output size (no output_padding)
    got = oracle.backward_convolution(delta, kernel, np.zeros((1, KA, 1, 1)), k, k, C, KA, s, s, p, p, (W, C, natural, natural))
    want = F.conv_transpose2d(t64(delta), t64(kernel).reshape(KA, C, k, k), stride=s, padding=p).numpy()
    assert got.shape == want.shape and rel_err(got, want) < TOL


@pytest.mark.parametrize("W,C,H,Wd,KA,k,s,p", CASES)
def test_adjointness(oracle, W, C, H, Wd, KA, k, s, p):
    """<conv(x), y> == <x, tconv(y)> for zero bias: the input delta is the adjoint of the forward pass."""
    oy = (H - k + 2 * p) // s + 1
    x, y, kernel = U(6, W, C, H, Wd), U(7, W, KA, oy, oy), U(8, 1, 1, KA, C * k * k)
    zero = np.zeros((1, KA, 1, 1))
    cx = oracle.forward_convolution(x, kernel, zero, k, k, C, KA, s, s, p, p)
    ty = oracle.backward_convolution(y, kernel, zero, k, k, C, KA, s, s, p, p, x.shape)
    lhs, rhs = np.sum(cx.astype(np.float64) * y), np.sum(x.astype(np.float64) * ty)
    assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))


@pytest.mark.parametrize("W,C,H,Wd,KA,k,s,p", CASES)
def test_wgrad_is_autograd(oracle, W, C, H, Wd, KA, k, s, p):
    oy = (H - k + 2 * p) // s + 1
    image, delta = U(9, W, C, H, Wd), U(10, W, KA, oy, oy)
    dk, db = oracle.create_delta_weight_and_bias(np.zeros((W, 1, KA, C * k * k)), np.zeros((W, KA, 1, 1)), image, delta,
                                                 k, k, C, KA, s, s, p, p)
    for w in range(W):  # per-sample gradients
        wt = torch.zeros(KA, C, k, k, dtype=torch.float64, requires_grad=True)
        bt = torch.zeros(KA, dtype=torch.float64, requires_grad=True)
        out = F.conv2d(t64(image[w:w + 1]), wt, bt, stride=s, padding=p)
        out.backward(t64(delta[w:w + 1]))
        assert rel_err(dk[w].reshape(KA, C, k, k), wt.grad.numpy()) < TOL
        assert rel_err(db[w].ravel(), bt.grad.numpy()) < TOL


def test_wgrad_accumulates(oracle):
    image, delta = U(1, 2, 2, 6, 6), U(2, 2, 3, 6, 6)
    dk0, db0 = U(3, 2, 1, 3, 18), U(4, 2, 3, 1, 1)
    z = oracle.create_delta_weight_and_bias(np.zeros_like(dk0), np.zeros_like(db0), image, delta, 3, 3, 2, 3, 1, 1, 1, 1)
    a = oracle.create_delta_weight_and_bias(dk0, db0, image, delta, 3, 3, 2, 3, 1, 1, 1, 1)
    assert rel_err(a[0], dk0 + z[0]) < TOL and rel_err(a[1], db0 + z[1]) < TOL


def test_back_wgrad_swaps_operands_and_clears_bias(oracle):
    big, small = U(1, 2, 2, 8, 8), U(2, 2, 3, 4, 4)
    z_dk, z_db = np.zeros((2, 1, 3, 2 * 16), np.float32), np.full((2, 3, 1, 1), 5.0, np.float32)
    a = oracle.create_delta_weight_and_bias(z_dk, np.zeros_like(z_db), big, small, 4, 4, 2, 3, 2, 2, 1, 1)
    b = oracle.create_delta_weight_and_bias(z_dk, z_db, small, big, 4, 4, 2, 3, 2, 2, 1, 1, back=True)
    assert np.array_equal(a[0], b[0]) and np.all(b[1] == 0)


def test_identity_kernel_copies(oracle):
    x = U(1, 2, 3, 6, 5)
    eye = np.eye(3, dtype=np.float32).reshape(1, 1, 3, 3)
    assert np.array_equal(oracle.forward_convolution(x, eye, np.zeros((1, 3, 1, 1)), 1, 1, 3, 3, 1, 1, 0, 0), x)
    assert np.array_equal(oracle.backward_convolution(x, eye, np.zeros((1, 3, 1, 1)), 1, 1, 3, 3, 1, 1, 0, 0, x.shape), x)


def test_tconv_bias_counts_taps(oracle):
    """With a zero kernel the transposed conv returns bias-sum times the number of contributing taps."""
    delta = U(1, 1, 2, 3, 3)
    bias = np.array([0.5, 0.25], np.float32).reshape(1, 2, 1, 1)
    out = oracle.backward_convolution(delta, np.zeros((1, 1, 2, 16)), bias, 4, 4, 1, 2, 2, 2, 1, 1, (1, 1, 6, 6))
    ones = F.conv_transpose2d(torch.ones(1, 1, 3, 3, dtype=torch.float64), torch.ones(1, 1, 4, 4, dtype=torch.float64), stride=2, padding=1).numpy()
    assert np.array_equal(out, (ones * 0.75).astype(np.float32))


@pytest.mark.parametrize("m,k,n,wl,wr", [(7, 13, 5, 1, 4), (64, 100, 1, 1, 8), (40, 33, 70, 2, 2)])
def test_products_are_matmul(oracle, m, k, n, wl, wr):
    a, b, at = U(1, wl, 2, m, k), U(2, wr, 2, k, n), U(3, wl, 2, k, m)
    W = max(wl, wr)
    want = np.stack([[a[w % wl, z].astype(np.float64) @ b[w % wr, z] for z in range(2)] for w in range(W)])
    assert rel_err(oracle.mul(a, b), want) < TOL
    want = np.stack([[at[w % wl, z].astype(np.float64).T @ b[w % wr, z] for z in range(2)] for w in range(W)])
    assert rel_err(oracle.transponse_mul(at, b), want) < TOL
    assert np.array_equal(oracle.transponse(a), np.swapaxes(a, 2, 3))


def test_reductions_and_elementwise(oracle):
    l, r = U(1, 6, 2, 3, 4), U(2, 6, 2, 3, 4)
    out = oracle.add_sum_w(l, r, 0.5, 1.0 / 6, out_w=2)
    assert rel_err(out[0], 0.5 * l.sum(0, dtype=np.float64) + r.sum(0, dtype=np.float64) / 6) < TOL and np.all(out[1] == 0)
    assert rel_err(oracle.summ_xy(l)[..., 0, 0], l.sum((2, 3), dtype=np.float64)) < TOL
    assert np.array_equal(oracle.add(l, r, 2.0, -3.0), np.float32(2) * l + np.float32(-3) * r)
    assert np.array_equal(oracle.sub(l, r[:1], 1.0, 1.0), l - r[:1])
    assert np.array_equal(oracle.tensor_item_production(l, r), l * r)
    assert np.array_equal(oracle.pow2(l, 3.0), l * l * np.float32(3))
    assert np.array_equal(oracle.inv(l), (1.0 / l.astype(np.float64)).astype(np.float32))
    assert np.array_equal(oracle.sqrt(np.abs(l), 2.0, 1e-6), np.sqrt(np.abs(l) + np.float32(1e-6)) * np.float32(2))
    assert np.array_equal(oracle.add_bias(l, r[:1, :, :1, :1]), l + r[:1, :, :1, :1])
    assert np.array_equal(oracle.add_value(l, 2.0, 0.5), l * np.float32(2) + np.float32(0.5))
    assert np.array_equal(oracle.sub_value(l, 2.0, 0.5), l * np.float32(2) - np.float32(0.5))
    assert np.array_equal(oracle.set(l, 0.25, -1.0), l * np.float32(0.25) + np.float32(-1.0))
    assert np.array_equal(oracle.clip(l, -0.2, 0.3), np.clip(l, np.float32(-0.2), np.float32(0.3)))
    assert np.array_equal(oracle.signum(np.round(l)), np.sign(np.round(l)))


def test_batchnorm_chain_closed_form(oracle):
    """The BN layer's op sequence (netlayer/cnetlayerbatchnormalization.cu.h:301-371) equals
    gamma*(x-mean_w)/sqrt(var_w+eps)+beta with the biased variance over the batch axis, per element."""
    x, gamma, beta = U(1, 16, 3, 4, 5) * 3 + 1, U(2, 1, 3, 4, 5), U(3, 1, 3, 4, 5)
    n = np.float32(16)
    zero = np.zeros((1, 3, 4, 5), np.float32)
    mean = oracle.add_sum_w(zero, x, 1.0, float(np.float32(1.0) / n))
    xmu = oracle.sub(x, mean)
    var = oracle.add_sum_w(zero, oracle.pow2(xmu, 1.0), 1.0, float(np.float32(1.0) / n))
    ivar = oracle.inv(oracle.sqrt(var, 1.0, 1e-6))
    xhat = oracle.tensor_item_production(xmu, ivar)
    out = oracle.add(oracle.tensor_item_production(gamma, xhat), beta)
    x64 = x.astype(np.float64)
    want = gamma * (x64 - x64.mean(0)) / np.sqrt(x64.var(0) + 1e-6) + beta
    assert rel_err(out, want) < 1e-5


def test_resampling_closed_forms(oracle):
    a = U(1, 2, 2, 6, 8)
    assert np.array_equal(oracle.upsampling(a, 2, 3), np.repeat(np.repeat(a, 3, axis=2), 2, axis=3))
    want = a.reshape(2, 2, 3, 2, 2, 4).astype(np.float64).mean((3, 5))
    assert rel_err(oracle.downsampling(a, 4, 2), want) < TOL
    # max pooling by brute force, first strict maximum scanning rows then columns
    b = np.round(U(2, 1, 2, 6, 6) * 3)
    pooled, pos = oracle.max_pooling(b, 3, 2)
    for z in range(2):
        for y in range(3):
            for x in range(2):
                win = b[0, z, y * 2:y * 2 + 2, x * 3:x * 3 + 3]
                iy, ix = np.unravel_index(np.argmax(win), win.shape)  # argmax returns the first maximum in row-major order
                assert pooled[0, z, y, x] == win.max()
                assert tuple(pos[0, z, y, x]) == (x * 3 + ix, y * 2 + iy)
    d = U(3, 1, 2, 3, 2)
    back = oracle.max_pooling_backward(d, pos, 3, 2, b.shape)
    assert np.count_nonzero(back) <= d.size and np.isclose(back.sum(), d.sum())
    for z in range(2):
        for y in range(3):
            for x in range(2):
                px, py = pos[0, z, y, x]
                assert back[0, z, py, px] == d[0, z, y, x]


def test_activation_closed_forms(oracle):
    x = (U(1, 1, 1, 1, 2000) * 10)
    x64 = x.astype(np.float64)
    assert rel_err(oracle.apply_func(x, "sigmoid"), 1 / (1 + np.exp(-x64))) < 1e-6
    assert rel_err(oracle.apply_func(x, "tangence"), np.tanh(x64)) < 1e-6
    assert np.array_equal(oracle.apply_func(x, "relu"), np.maximum(x, 0))
    assert np.array_equal(oracle.apply_func(x, "leaky_relu"), np.where(x > 0, x, (0.1 * x64).astype(np.float32)))
    assert np.array_equal(oracle.apply_func(x, "linear"), x)
    gelu = 0.5 * x64 * (1 + np.tanh(np.sqrt(2 / np.pi) * (x64 + 0.044715 * x64 ** 3)))
    assert rel_err(oracle.apply_func(x, "gelu"), gelu) < 1e-6
    s = 1 / (1 + np.exp(-x64))
    assert rel_err(oracle.apply_func(x, "sigmoid", True), s * (1 - s)) < 1e-6
    assert rel_err(oracle.apply_func(x, "tangence", True), 1 - np.tanh(x64) ** 2) < 1e-6
    assert np.array_equal(oracle.apply_func(x, "relu", True), (x >= 0).astype(np.float32))
    assert np.array_equal(oracle.apply_func(x, "leaky_relu", True), np.where(x >= 0, np.float32(1), np.float32(0.1)))
    assert np.all(oracle.apply_func(x, "linear", True) == 1)
    # derivative of GeLU exactly as the reference writes it (cpu/ctensorapplyfunc.h:220-229)
    c = np.sqrt(2 / np.float64(np.float32(3.141592654)))
    ft, fa = c * (x64 + 0.044715 * x64 ** 3), c * (1 + 3 * 0.044715 * x64 ** 2)
    want = 0.5 * ((1 + np.tanh(ft)) + 0.5 * x64 / np.cosh(ft) ** 2) * fa
    assert rel_err(oracle.apply_func(x, "gelu", True), want) < 1e-5
    # clamps: beyond +-30 the argument is replaced by +-29.99999
    for name in ("sigmoid", "tangence"):
        assert oracle.func_scalar(1000.0, name) == oracle.func_scalar(29.99999, name)
        assert oracle.func_scalar(-1000.0, name) == oracle.func_scalar(-29.99999, name)


def test_adam_closed_form(oracle):
    w, dw, m, v = U(1, 1, 1, 5, 5), U(2, 1, 1, 5, 5) * 8, U(3, 1, 1, 5, 5) * 0.1, np.abs(U(4, 1, 1, 5, 5)) * 0.1
    b1, b2, lr, eps, it, bs = 0.9, 0.999, 1e-3, 1e-8, 3.0, 8
    w1, m1, v1 = oracle.adam(w, dw, m, v, bs, lr, b1, b2, eps, it)
    g = dw.astype(np.float64) / bs
    m64 = b1 * m + (1 - b1) * g
    v64 = b2 * v + (1 - b2) * g * g
    step = lr * (m64 / (1 - b1 ** it)) / (np.sqrt(v64 / (1 - b2 ** it)) + eps)
    assert rel_err(m1, m64) < 1e-6 and rel_err(v1, v64) < 1e-6 and rel_err(w1, w - step) < 1e-6


def test_vae_coder_output_closed_form(oracle):
    """out = mu + exp(clamp(logvar)/2)*eps and the KL term against float64; special cases that a dropped term, a wrong
    sign or a missing clamp would break."""
    rng = np.random.default_rng(7)
    mu, lv, eps = (rng.standard_normal((5, 1, 64, 1)).astype(np.float32) for _ in range(3))
    lv *= 7                                                     # some beyond +-10
    out, kl = oracle.vae_coder_output(mu, lv, eps)
    c = np.clip(lv.astype(np.float64), -10, 10)
    assert np.max(np.abs(out - (mu + np.exp(c / 2) * eps))) <= 1e-5 * np.abs(out).max()
    exact = -0.5 * np.sum(1 + c - mu.astype(np.float64) ** 2 - np.exp(c)) / 5
    assert abs(kl - exact) <= 1e-5 * abs(exact)
    zero = np.zeros((3, 1, 8, 1), np.float32)
    out, kl = oracle.vae_coder_output(zero + 0.5, zero, zero)   # no noise: the mean comes through; KL = 0.5*mu^2 per element
    assert np.array_equal(out, zero + 0.5) and abs(kl - 0.5 * 0.25 * 8) <= 1e-6
    out, kl = oracle.vae_coder_output(zero, zero, zero + 2)     # unit variance: the noise comes through, KL = 0
    assert np.array_equal(out, zero + 2) and kl == 0
    out, _ = oracle.vae_coder_output(zero, zero + 50, zero + 1)  # clamp at 10: exp(5)
    assert np.allclose(out, np.exp(5.0), rtol=1e-6)
    out, _ = oracle.vae_coder_output(zero, zero - 50, zero + 1)
    assert np.allclose(out, np.exp(-5.0), rtol=1e-6)


# ---- functions that only the reference's GPU class has (cuda/ctensormath.cu.h:473-598, 3029-3262) ----------------

def test_concatenation_and_split_are_numpy_slicing(oracle):
    a, b = U(1, 3, 2, 4, 5), U(2, 3, 3, 4, 5)
    cat = oracle.concatecation_z(a, b)
    assert np.array_equal(cat, np.concatenate([a, b], axis=1))
    # an operand with fewer samples repeats by w % W
    one = oracle.concatecation_z(a, b[:1])
    assert np.array_equal(one, np.concatenate([a, np.repeat(b[:1], 3, axis=0)], axis=1))
    sa, sb = oracle.split_z(cat, 2)
    assert np.array_equal(sa, a) and np.array_equal(sb, b)
    with pytest.raises(Exception):
        oracle.concatecation_z(a, U(3, 3, 3, 4, 6))


def test_time_step_closed_form(oracle):
    x = U(1, 3, 2, 4, 6)
    steps = np.array([0, 7, 999], np.uint32)
    got = oracle.set_time_step(x, steps)
    size = 2 * 4 * 6
    pos = np.arange(size, dtype=np.float64)
    for w, t in enumerate(steps):
        angle = float(t) / 10000.0 ** (pos / size)
        want = x[w].ravel().astype(np.float64) + np.where(pos % 2 == 0, np.sin(angle), np.cos(angle))
        # the angle is a float quotient of up to 1000: its rounding (6e-5) is the error of the sine
        assert np.max(np.abs(got[w].ravel() - want)) <= 2e-4
    assert np.array_equal(got[0].ravel()[0::2], x[0].ravel()[0::2])        # t = 0: sin 0 added to even positions
    assert np.allclose(got[0].ravel()[1::2], x[0].ravel()[1::2] + 1.0)     # and cos 0 to odd ones


def test_philox_known_answers(oracle):
    """Philox4x32-10 against the known-answer vectors published with Random123 (kat_vectors)."""
    assert oracle.philox4x32_10((0, 0, 0, 0), (0, 0)) == (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)
    assert oracle.philox4x32_10((0xffffffff,) * 4, (0xffffffff,) * 2) == (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)
    assert oracle.philox4x32_10((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0)) == (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)


def test_random_fills_have_the_reference_distributions(oracle):
    shape = (4, 8, 64, 64)   # 131072 draws
    n = float(np.prod(shape))
    for p in (0.0, 0.3, 0.5):
        d = oracle.create_drop_out_matrix(shape, p, 11)
        kept = d != 0
        assert np.all(d[kept] == np.float32(1.0 / (1.0 - p)))
        assert abs(kept.mean() - (1.0 - p)) <= 4 * np.sqrt(p * (1 - p) / n) + 1e-12          # four standard errors
    assert not np.array_equal(oracle.create_drop_out_matrix(shape, 0.3, 11), oracle.create_drop_out_matrix(shape, 0.3, 12))
    z = oracle.set_normal_noise(shape, 5).astype(np.float64)
    assert abs(z.mean()) <= 4 / np.sqrt(n) and abs(z.var() - 1.0) <= 4 * np.sqrt(2.0 / n)
    assert abs((z ** 3).mean()) <= 4 * np.sqrt(15.0 / n) and abs((z ** 4).mean() - 3.0) <= 4 * np.sqrt(96.0 / n)
    assert abs((np.abs(z) < 1.0).mean() - 0.682689) <= 4 * np.sqrt(0.68 * 0.32 / n)
    assert abs(np.corrcoef(z.ravel()[:-1], z.ravel()[1:])[0, 1]) <= 4 / np.sqrt(n)           # neighbours are independent
    image = U(3, *shape)
    sa, sb = U(4, 4, 1, 1, 1) * 0.5 + 0.5, U(5, 4, 1, 1, 1) * 0.5 + 0.5
    noisy, noise = oracle.get_noise_image_and_noise(image, sa, sb, 5)
    assert np.array_equal(noise, oracle.set_normal_noise(shape, 5))                          # the same draws per element
    assert np.allclose(noisy, sa * image + sb * noise, rtol=0, atol=1e-6)
