"""Writes tests/golden/ref_vectors.npz from the reference's own CPU headers.

Run in the authoring container only (it needs oracle/_ref/libtensor_ref.so,
which `make -C oracle` builds from the headers under /root/reference):

    python tests/golden/make_golden.py

The vectors cover the behaviours that nothing but the compiled reference can
pin: transposed convolution with a non-zero bias (added once per tap), the
tie/NaN rule of max pooling, the activation clamps and the derivative of GeLU as
written, box down-sampling at ragged edges, the zero fill of AddSumW, Adam's
mixed float/double arithmetic, and the un-asserted stride-2/padding-1 forward
convolution of the reference self-test.  Inputs are stored beside the outputs so
the tests need no generator.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
import oracle_api  # noqa: E402


def main():
    ref = oracle_api.Oracle("ref")
    rng = np.random.default_rng(20240607)
    out = {}

    def u(*shape, lo=-1.0, hi=1.0):
        return rng.uniform(lo, hi, size=shape).astype(np.float32)

    # 1. self-test conv with stride 2 / padding 1 (inputs from the reference, no expected values there)
    kat = json.load(open(os.path.join(HERE, "ctensortest_kat.json")))["forward_convolution_step_padding"]
    img = np.array(kat["image"], np.float32).reshape(1, 3, 5, 5)
    ker = np.array(kat["kernels"], np.float32).reshape(1, 1, 2, 27)
    out["fwd_s2p1_out"] = ref.forward_convolution(img, ker, np.zeros((1, 2, 1, 1), np.float32), 3, 3, 3, 2, 2, 2, 1, 1)

    # 2. forward conv, random, rectangular kernel/stride/padding, batch broadcast of the kernel
    image = u(3, 4, 9, 11)
    kernel = u(1, 1, 5, 4 * 3 * 2)
    bias = u(1, 5, 1, 1)
    out["fwd_image"], out["fwd_kernel"], out["fwd_bias"] = image, kernel, bias
    out["fwd_out"] = ref.forward_convolution(image, kernel, bias, 2, 3, 4, 5, 2, 1, 1, 2)  # kx=2 ky=3 sx=2 sy=1 px=1 py=2

    # 3. transposed conv with NON-ZERO bias, stride 2 and stride 3
    delta = u(2, 3, 4, 5)
    tk = u(1, 1, 3, 2 * 4 * 4)
    tb = u(1, 3, 1, 1)
    out["tconv_delta"], out["tconv_kernel"], out["tconv_bias"] = delta, tk, tb
    out["tconv_out_s2"] = ref.backward_convolution(delta, tk, tb, 4, 4, 2, 3, 2, 2, 1, 1, (2, 2, 8, 10))
    out["tconv_out_s3"] = ref.backward_convolution(delta, tk, tb, 4, 4, 2, 3, 3, 3, 0, 0, (2, 2, 13, 16))
    out["tconv_out_s1"] = ref.backward_convolution(delta, tk, tb, 4, 4, 2, 3, 1, 1, 2, 2, (2, 2, 3, 4))

    # 4. weight gradient accumulating into non-zero dK/dB, stride 2
    wimg = u(3, 2, 8, 8)
    wdelta = u(3, 4, 4, 4)
    dk0 = u(3, 1, 4, 2 * 9)
    db0 = u(3, 4, 1, 1)
    out["wgrad_image"], out["wgrad_delta"], out["wgrad_dk0"], out["wgrad_db0"] = wimg, wdelta, dk0, db0
    out["wgrad_dk"], out["wgrad_db"] = ref.create_delta_weight_and_bias(dk0, db0, wimg, wdelta, 3, 3, 2, 4, 2, 2, 1, 1)

    # 5. max pooling with ties, negative zero and NaN
    mp = np.round(u(2, 2, 6, 6) * 2).astype(np.float32)          # many ties
    mp[0, 0, 0, 0] = np.nan
    mp[0, 0, 2, 3] = np.nan
    mp[1, 1, 4, 4] = -0.0
    out["maxpool_in"] = mp
    pooled, pos = ref.max_pooling(mp, 2, 3)
    out["maxpool_out"], out["maxpool_pos"] = pooled, pos
    md = u(2, 2, 2, 3)
    out["maxpool_back_delta"] = md
    out["maxpool_back_out"] = ref.max_pooling_backward(md, pos, 2, 3, (2, 2, 6, 6))

    # 6. activations on a grid with the clamp boundaries
    grid = np.concatenate([np.linspace(-8, 8, 161), [-31, -30.5, -30, -29.99999, 29.99999, 30, 30.5, 31, 0.0, -0.0, 1e-8, -1e-8]])
    grid = grid.astype(np.float32).reshape(1, 1, 1, -1)
    out["act_in"] = grid
    for name in oracle_api.FUNC:
        out["act_" + name] = ref.apply_func(grid, name)
        out["dact_" + name] = ref.apply_func(grid, name, differential=True)

    # 7. down-sampling with ragged edges and up-sampling into a larger-than-multiple output
    ds = u(2, 2, 7, 9)
    out["down_in"] = ds
    out["down_out"] = ref.downsampling(ds, 2, 3)
    out["up_out"] = ref.upsampling(ds, 2, 3, out_shape=(2, 2, 23, 19))

    # 8. AddSumW: zero fill of w>0, scales
    al, ar = u(3, 2, 3, 4), u(5, 2, 3, 4)
    out["addsumw_l"], out["addsumw_r"] = al, ar
    out["addsumw_out"] = ref.add_sum_w(al, ar, 0.5, 1.0 / 5.0, out_w=3)

    # 9. Adam, two different iterations
    w0, dw, m0, v0 = u(1, 1, 4, 8), u(1, 1, 4, 8) * 10, u(1, 1, 4, 8) * 0.1, np.abs(u(1, 1, 4, 8)) * 0.01
    out["adam_w"], out["adam_dw"], out["adam_m"], out["adam_v"] = w0, dw, m0, v0
    for it in (1.0, 7.0):
        w1, m1, v1 = ref.adam(w0, dw, m0, v0, 16, 0.0002, 0.5, 0.9, 1e-8, it)
        out["adam_w_it%d" % it], out["adam_m_it%d" % it], out["adam_v_it%d" % it] = w1, m1, v1

    # 10. matrix products with ragged sizes and W broadcast
    a, b = u(1, 2, 37, 45), u(3, 2, 45, 33)
    out["mul_a"], out["mul_b"] = a, b
    out["mul_out"] = ref.mul(a, b)
    at = u(1, 2, 45, 37)
    out["tmul_a"] = at
    out["tmul_out"] = ref.transponse_mul(at, b)

    path = os.path.join(HERE, "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
