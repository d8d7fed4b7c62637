"""The entry point that allocates nothing (mt_batchnorm_forward_train_func_noalloc) against the entry point it is a
variant of, through the C ABI: bit-identical results on two calls in a row, the second with a smaller input; the
size limit of the fixed scratch array is enforced with a clear error; no device memory is requested from the driver."""
import numpy as np
import pytest

from cases import rng_normal as Nrm

pytestmark = pytest.mark.gpu


def run(fn, x, gamma, beta, func, want_stats):
    import mi355tensor as mt
    from mi355tensor import CTensor
    shape = x.shape
    one = (1,) + shape[1:]
    tx, tg, tb, out = CTensor.from_numpy(x), CTensor.from_numpy(gamma), CTensor.from_numpy(beta), CTensor(*shape)
    mt.CTensorMath.Fill(out, -3.0)
    stats = {}
    if want_stats:
        stats = dict(xhat=CTensor(*shape), ivar=CTensor(*one), batch_mean=CTensor(*one), batch_var=CTensor(*one),
                     new_mean=CTensor.from_numpy(np.zeros(one, np.float32)), new_variable=CTensor.from_numpy(np.ones(one, np.float32)))
    before = mt.get_info("driver_allocations")
    fn(out, tx, tg, tb, momentum=0.9, epsilon=1e-6, func=func, **stats)
    allocated = mt.get_info("driver_allocations") - before
    return dict({"out": out.numpy()}, **{k: t.numpy() for k, t in stats.items()}), allocated


def test_no_alloc_entry_point_matches_the_allocating_one():
    import mi355tensor as mt
    from mi355tensor import Fused
    mt.init(0)
    # two calls in a row on the shared array, the second smaller: what the first call left behind must not be read
    for seed, shape, func, want_stats in ((11, (32, 64, 32, 32), "relu", False), (12, (5, 3, 7, 9), "leaky_relu", False),
                                          (13, (16, 8, 4, 4), None, True), (14, (3, 1, 1, 5), "tangence", False)):
        x = Nrm(seed, *shape) * 3.0 + 1.5
        gamma, beta = Nrm(seed + 100, 1, *shape[1:]), Nrm(seed + 200, 1, *shape[1:])
        want, _ = run(Fused.BatchNormForwardTrain, x, gamma, beta, func, want_stats)
        got, allocated = run(Fused.BatchNormForwardTrainNoAlloc, x, gamma, beta, func, want_stats)
        assert allocated == 0, "the entry point asked the driver for device memory"
        for k in want:
            assert np.array_equal(got[k], want[k]), (shape, k)
        assert np.isfinite(got["out"]).all()
    # bit-exact for integer-valued data as well (a constant batch: variance 0, output beta)
    x = np.full((4, 2, 3, 3), 5.0, np.float32)
    got, _ = run(Fused.BatchNormForwardTrainNoAlloc, x, np.ones((1, 2, 3, 3), np.float32), np.full((1, 2, 3, 3), 2.0, np.float32), None, False)
    assert np.array_equal(got["out"], np.full((4, 2, 3, 3), 2.0, np.float32))


def test_no_alloc_entry_point_rejects_what_does_not_fit():
    import mi355tensor as mt
    from mi355tensor import CTensor, Fused
    mt.init(0)
    shape = (2, 1, 513, 512)   # 262656 elements per sample: 512 more than the fixed array has statistics for
    x, g, b, out = (CTensor(*s) for s in (shape, (1,) + shape[1:], (1,) + shape[1:], shape))
    with pytest.raises(mt.TensorError) as e:
        Fused.BatchNormForwardTrainNoAlloc(out, x, g, b)
    assert e.value.code == 6 and "262144" in str(e.value)
    Fused.BatchNormForwardTrain(out, x, g, b)   # the allocating entry point takes the same input
    mt.synchronize()
