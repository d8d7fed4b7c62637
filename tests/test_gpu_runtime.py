"""The runtime around the kernels, through the C ABI: re-ordered weights kept between calls and made again after every
kind of write, the stream-ordered memory pool, and workspaces that grow while recorded graphs exist."""
import ctypes as C

import numpy as np
import pytest

from cases import rng_normal as Nrm

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mt():
    import mi355tensor as m
    m.init(0)
    return m


def tconv(mt, out, x, kernel, bias, cout, cin, func=None):
    mt.CTensorConv.BackwardConvolution(out, x, kernel, 4, 4, cout, cin, bias, 2, 2, 1, 1, func=func)
    return out.numpy()


def test_kept_weights_follow_every_write_path(mt):
    """A transposed convolution whose weights change through each call that can write them gives, every time, exactly
    the result of the same call with the cache switched off; unchanged weights are not re-ordered again."""
    from mi355tensor import CTensor, CTensorMath as M, Fused
    cin, cout, b = 32, 48, 4
    x = CTensor.from_numpy(Nrm(1, b, cin, 8, 8))
    w0 = Nrm(2, 1, 1, cin, cout * 16, std=0.05)
    kernel, bias = CTensor.from_numpy(w0), CTensor.from_numpy(Nrm(3, 1, cin, 1, 1, std=0.1))
    out = CTensor(b, cout, 16, 16)
    other, mom, vel = CTensor.from_numpy(Nrm(4, 1, 1, cin, cout * 16, std=0.05)), CTensor(1, 1, cin, cout * 16), CTensor(1, 1, cin, cout * 16)
    M.Fill(mom, 0.0)
    M.Fill(vel, 0.0)
    host = np.ascontiguousarray(Nrm(5, 1, 1, cin, cout * 16, std=0.05))
    part = kernel.reinterpret(1, 1, 1, cin * cout * 16)
    writes = [
        ("nothing", lambda: None, False),
        ("mt_copy_h2d", lambda: kernel.upload(host), True),
        ("mt_copy_d2d", lambda: mt.call("mt_copy_d2d", kernel.ptr, other.ptr, C.c_size_t(kernel.count * 4)), True),
        ("mt_fill", lambda: M.Fill(kernel, 0.01), True),
        ("mt_adam", lambda: M.Adam(kernel, other, mom, vel, 4, 1e-2, 0.9, 0.999, 1e-8, 1.0), True),
        # (the step over several tensors writes the re-ordered copy itself: nothing is made again, the result is the same)
        ("mt_adam_many", lambda: Fused.AdamMany([kernel], [other], [mom], [vel], 4, 1e-2, 0.9, 0.999, 1e-8, 2.0), False),
        ("mt_fill_many", lambda: Fused.FillMany([kernel, mom], 0.02), True),
        ("mt_add into the weights", lambda: M.Add(kernel, kernel, other, 1.0, 0.5), True),
        ("mt_mul_value on a view of the weights", lambda: M.Mul(part, part, 1.5), True),
        ("mt_apply_func", lambda: mt.CTensorApplyFunc.ApplyTangence(kernel, kernel), True),
        ("mt_set_normal_noise", lambda: M.SetNormalNoise(kernel, 7), True),
        ("mt_invalidate after a foreign write", lambda: (mt.call("mt_copy_d2d", bias.ptr, bias.ptr, C.c_size_t(0)), mt.invalidate(kernel.ptr.value, 64)), True),
        ("a write to the bias", lambda: M.Fill(bias, 0.25), True),
        ("a write next to the weights", lambda: M.Fill(other, 0.0), False),
    ]
    tconv(mt, out, x, kernel, bias, cout, cin)
    for name, write, changes in writes:
        write()
        made = mt.get_info("pack_cache_made")
        got = tconv(mt, out, x, kernel, bias, cout, cin)
        assert (mt.get_info("pack_cache_made") - made == 1) == changes, name
        mt.set_option("pack_cache", 0)
        want = tconv(mt, out, x, kernel, bias, cout, cin)
        mt.set_option("pack_cache", 1)
        assert np.array_equal(got, want), name
        tconv(mt, out, x, kernel, bias, cout, cin)   # the entry exists again for the next write
    hits = mt.get_info("pack_cache_hits")
    tconv(mt, out, x, kernel, bias, cout, cin)
    assert mt.get_info("pack_cache_hits") == hits + 1


def test_optimiser_step_keeps_the_reordered_copy_current(mt):
    """mt_adam_many writes every new weight into the kept copy for the 4x4 stride-2 transposed convolution as well: the
    next input gradient re-orders nothing and is bit for bit what a fresh re-ordering gives, over several steps and four
    layers in one call.  A step that also changes the bias whose sums the copy holds, a copy that was stale before the
    step, and the option switched off all fall back to re-ordering."""
    from mi355tensor import CTensor, CTensorMath as M, Fused
    layers = []
    # (the third: no tiles of 16 x 16, element by element; the last: an image layer, whose kernel has a layout of its own)
    for n, (cin, cout, hw) in enumerate([(64, 32, 8), (128, 64, 4), (24, 20, 4), (64, 3, 16)]):
        kernel, grad = CTensor.from_numpy(Nrm(160 + n, 1, 1, cin, cout * 16, std=0.05)), CTensor.from_numpy(Nrm(62 + n, 1, 1, cin, cout * 16, std=0.05))
        mom, vel = CTensor(1, 1, cin, cout * 16), CTensor(1, 1, cin, cout * 16)
        M.Fill(mom, 0.0)
        M.Fill(vel, 0.0)
        layers.append(dict(cin=cin, cout=cout, x=CTensor.from_numpy(Nrm(64 + n, 4, cin, hw, hw)), out=CTensor(4, cout, 2 * hw, 2 * hw), kernel=kernel, grad=grad,
                           mom=mom, vel=vel, bias=CTensor.from_numpy(Nrm(66 + n, 1, cin, 1, 1, std=0.1))))
    run = lambda l: tconv(mt, l["out"], l["x"], l["kernel"], l["bias"], l["cout"], l["cin"])
    fresh = lambda l: (mt.set_option("pack_cache", 0), run(l), mt.set_option("pack_cache", 1))[1]
    lists = lambda key: [l[key] for l in layers]
    for l in layers:
        run(l)
    # (weights at an address that a graph recorded by an earlier test wrote are never vouched for: the pool may hand such a
    # block to this test, and that layer is then re-ordered on every use, as it must be)
    trusted = mt.get_info("graph_written_ranges") == 0 and mt.get_info("graph_writes_anything") == 0
    for step in range(1, 4):
        refreshed, made = mt.get_info("pack_cache_refreshed"), mt.get_info("pack_cache_made")
        Fused.AdamMany(lists("kernel"), lists("grad"), lists("mom"), lists("vel"), 4, 1e-2, 0.9, 0.999, 1e-8, float(step))
        kept = mt.get_info("pack_cache_refreshed") - refreshed
        assert kept == 4 if trusted else 0 <= kept <= 4
        got = [run(l) for l in layers]
        assert mt.get_info("pack_cache_made") - made == 4 - kept, "a copy was neither kept current nor made again"
        for l, g in zip(layers, got):
            assert np.array_equal(g, fresh(l)), step
        for l in layers:
            run(l)  # (switching the cache off dropped every entry: they exist again for the next step)
    # the bias in the same step: its sums in the entry are stale, so the copy is made again
    l = layers[0]
    bias_grad, bias_mom, bias_vel = CTensor.from_numpy(Nrm(70, 1, l["cin"], 1, 1)), CTensor(1, l["cin"], 1, 1), CTensor(1, l["cin"], 1, 1)
    M.Fill(bias_mom, 0.0)
    M.Fill(bias_vel, 0.0)
    made = mt.get_info("pack_cache_made")
    Fused.AdamMany([l["kernel"], l["bias"]], [l["grad"], bias_grad], [l["mom"], bias_mom], [l["vel"], bias_vel], 4, 1e-2, 0.9, 0.999, 1e-8, 4.0)
    got = run(l)
    assert mt.get_info("pack_cache_made") == made + 1
    assert np.array_equal(got, fresh(l))
    run(l)
    # a copy that is stale before the step (the bias was written on its own) is not vouched for by the step
    M.Fill(l["bias"], 0.125)
    made = mt.get_info("pack_cache_made")
    refreshed = mt.get_info("pack_cache_refreshed")
    Fused.AdamMany([l["kernel"]], [l["grad"]], [l["mom"]], [l["vel"]], 4, 1e-2, 0.9, 0.999, 1e-8, 5.0)
    got = run(l)
    assert mt.get_info("pack_cache_made") == made + 1 and mt.get_info("pack_cache_refreshed") == refreshed
    assert np.array_equal(got, fresh(l))
    run(l)
    # switched off: the step only reports its write
    mt.set_option("pack_refresh", 0)
    try:
        made, refreshed = mt.get_info("pack_cache_made"), mt.get_info("pack_cache_refreshed")
        Fused.AdamMany([l["kernel"]], [l["grad"]], [l["mom"]], [l["vel"]], 4, 1e-2, 0.9, 0.999, 1e-8, 6.0)
        got = run(l)
        assert mt.get_info("pack_cache_made") == made + 1 and mt.get_info("pack_cache_refreshed") == refreshed
        assert np.array_equal(got, fresh(l))
    finally:
        mt.set_option("pack_refresh", 1)


def test_kept_weights_of_the_other_layouts(mt):
    """Tap-major forward kernels, the image layer's layout and the coefficient sums of up-sampling + 3x3: the second call
    re-orders nothing and gives the first call's result; freed weights never serve a new tensor at the same address."""
    from mi355tensor import CTensor, CTensorConv as Cv, CTensorMath as M, Fused
    image = CTensor.from_numpy(Nrm(20, 2, 16, 12, 12))
    k3, b3, out3 = CTensor.from_numpy(Nrm(21, 1, 1, 32, 16 * 9, std=0.1)), CTensor.from_numpy(Nrm(22, 1, 32, 1, 1)), CTensor(2, 32, 12, 12)
    up_out = CTensor(2, 32, 24, 24)
    img_k, img_b, img_out = CTensor.from_numpy(Nrm(23, 1, 1, 16, 3 * 16, std=0.1)), CTensor.from_numpy(np.zeros((1, 16, 1, 1), np.float32)), CTensor(2, 3, 24, 24)
    calls = [lambda: (Cv.ForwardConvolution(out3, image, k3, 3, 3, 16, 32, b3, 1, 1, 1, 1, func="relu"), out3.numpy())[1],
             lambda: (Fused.UpSamplingConvolution(up_out, image, 2, 2, k3, 3, 3, 16, 32, b3, 1, 1, 1, 1, func="leaky_relu"), up_out.numpy())[1],
             lambda: (Cv.BackwardConvolution(img_out, image, img_k, 4, 4, 3, 16, img_b, 2, 2, 1, 1, func="tangence"), img_out.numpy())[1]]
    for call in calls:
        first = call()
        made = mt.get_info("pack_cache_made")
        assert np.array_equal(call(), first) and mt.get_info("pack_cache_made") == made
        mt.set_option("pack_cache", 0)
        assert np.array_equal(call(), first)
        mt.set_option("pack_cache", 1)
    # the same address with other contents: mt_free forgets what was derived from the block
    shape, results = (1, 1, 32, 16 * 9), []
    for seed in (30, 31):
        k = CTensor.from_numpy(Nrm(seed, *shape, std=0.1))
        Cv.ForwardConvolution(out3, image, k, 3, 3, 16, 32, b3, 1, 1, 1, 1)
        results.append((k.ptr.value, out3.numpy()))
        k.free()
    assert results[0][0] == results[1][0], "the pool hands the freed block to the next tensor of the same size"
    assert not np.array_equal(results[0][1], results[1][1])


def test_recording_never_uses_kept_weights(mt):
    """While the stream is captured the weights are re-ordered inside the recording: a replay after the weights changed
    (by a write the recording itself does not contain) gives the eager result for the new weights."""
    from mi355tensor import CTensor, CTensorMath as M
    cin, cout = 32, 32
    x, out = CTensor.from_numpy(Nrm(40, 2, cin, 4, 4)), CTensor(2, cout, 8, 8)
    kernel, bias = CTensor.from_numpy(Nrm(41, 1, 1, cin, cout * 16, std=0.05)), CTensor.from_numpy(np.zeros((1, cin, 1, 1), np.float32))
    step = lambda: mt.CTensorConv.BackwardConvolution(out, x, kernel, 4, 4, cout, cin, bias, 2, 2, 1, 1)
    mt.set_option("pack_cache", 0)
    step()                       # the workspace the recording will use exists
    mt.set_option("pack_cache", 1)
    step()
    mt.synchronize()
    graph = mt.Graph(step)
    for value in (0.01, -0.02, 0.03):
        M.Fill(kernel, value)
        step()
        eager = out.numpy()
        M.Fill(out, 9.0)
        mt.synchronize()
        graph.launch()
        assert np.array_equal(out.numpy(), eager)


def test_weights_that_a_recording_updates_are_never_trusted(mt):
    """A recorded step that changes the weights (an optimiser step inside the graph): replays write the weights without
    the library seeing a call, so an eager call after a replay must re-order them again although no eager write happened;
    and a recording made after eager use of the weights needs no workspace of its own."""
    from mi355tensor import CTensor, CTensorMath as M
    cin, cout = 32, 64
    x, out = CTensor.from_numpy(Nrm(60, 4, cin, 4, 4)), CTensor(4, cout, 8, 8)
    kernel, bias = CTensor.from_numpy(Nrm(61, 1, 1, cin, cout * 16, std=0.05)), CTensor.from_numpy(np.zeros((1, cin, 1, 1), np.float32))
    other = CTensor.from_numpy(Nrm(62, 1, 1, cin, cout * 16, std=0.05))
    conv = lambda: mt.CTensorConv.BackwardConvolution(out, x, kernel, 4, 4, cout, cin, bias, 2, 2, 1, 1)

    def step():
        M.Add(kernel, kernel, other, 1.0, 0.5)
        conv()
    conv()                      # the kept copy exists and is valid
    mt.synchronize()
    graph = mt.Graph(step)      # records into the kept copy's own buffer
    for _ in range(3):
        graph.launch()
        replayed = out.numpy()
        hits = mt.get_info("pack_cache_hits")
        conv()                  # eager, after an unseen write
        assert mt.get_info("pack_cache_hits") == hits, "the copy of weights that a graph writes was trusted"
        eager = out.numpy()
        mt.set_option("pack_cache", 0)
        conv()
        mt.set_option("pack_cache", 1)
        assert np.array_equal(eager, out.numpy()) and np.array_equal(replayed, eager)
        conv()
    # Once the weights' block is given back, what the recording writes there no longer counts (replaying it now would be a
    # use of freed memory): the next tensor at that address is trusted like any other.
    ranges, address = mt.get_info("graph_written_ranges"), kernel.ptr.value
    kernel.free()
    assert mt.get_info("graph_written_ranges") < ranges
    kernel = CTensor.from_numpy(Nrm(63, 1, 1, cin, cout * 16, std=0.05))
    assert kernel.ptr.value == address, "the pool hands the freed block to the next tensor of the same size"
    conv()
    hits = mt.get_info("pack_cache_hits")
    conv()
    assert mt.get_info("pack_cache_hits") == hits + 1


def test_pool_reuses_blocks_in_stream_order(mt):
    """A temporary that is freed while the kernel that reads it is still queued (the reference's layers do this on
    every backward call, netlayer/cnetlayerconvolution.cu.h:494) and whose block is handed out again at once."""
    from mi355tensor import CTensor, CTensorMath as M
    n = 1 << 22
    a = CTensor.from_numpy(np.arange(n, dtype=np.float32).reshape(1, 1, 1 << 11, 1 << 11) % 1000.0)
    out1, out2 = CTensor(1, 1, 1 << 11, 1 << 11), CTensor(1, 1, 1 << 11, 1 << 11)
    allocs = mt.get_info("driver_allocations")
    for rounds in range(3):
        tmp = CTensor(1, 1, 1 << 11, 1 << 11)
        M.Set(tmp, a, 2.0, 1.0)                # tmp = 2a + 1
        for _ in range(20):
            M.Add(out1, tmp, a, 1.0, 1.0)      # queued readers of tmp: 3a + 1
        ptr = tmp.ptr.value
        tmp.free()                             # no wait: the block goes to the pool while its readers are queued
        again = CTensor(1, 1, 1 << 11, 1 << 11)
        assert again.ptr.value == ptr
        M.Fill(again, -5.0)                    # queued behind the readers
        M.Add(out2, again, a, 1.0, 1.0)
        want = a.numpy()
        assert np.array_equal(out1.numpy(), 3.0 * want + 1.0)
        assert np.array_equal(out2.numpy(), want - 5.0)
        again.free()
    assert mt.get_info("driver_allocations") <= allocs + 1   # (one block for all three rounds; none when an earlier test left one of this size in the pool)
    assert mt.get_info("pool_reused") >= 5
    mt.set_option("pool", 0)
    assert mt.get_info("pool_bytes") == 0
    mt.set_option("pool", 1)


def test_temporaries_of_a_recording_are_never_handed_out_again(mt):
    """A recorded sequence that creates and frees a temporary, as the reference's layers do on every backward call
    (netlayer/cnetlayerconvolution.cu.h:494): the graph's kernels name the temporary's address, so its block must not
    serve another tensor afterwards -- replays would write over that tensor.  A block freed twice is refused."""
    from mi355tensor import CTensor, CTensorMath as M, Graph
    shape = (1, 1, 1 << 10, 1 << 10)
    a = CTensor.from_numpy(np.arange(1 << 20, dtype=np.float32).reshape(shape) % 977.0)
    out = CTensor(*shape)
    seen = {}

    def step():
        tmp = CTensor(*shape)
        seen["ptr"] = tmp.ptr.value
        M.Set(tmp, a, 2.0, 1.0)
        M.Add(out, tmp, a, 1.0, 1.0)
        tmp.free()

    step()                                       # eager first: the temporary's block now waits in the pool
    want = out.numpy()
    retired = mt.get_info("retired_blocks")
    graph = Graph(step)
    assert mt.get_info("retired_blocks") == retired + 1
    later = [CTensor(*shape) for _ in range(3)]  # same size as the temporary
    assert all(t.ptr.value != seen["ptr"] for t in later)
    for t in later:
        M.Fill(t, 7.0)
    for _ in range(3):
        M.Fill(out, 0.0)
        graph.launch()
        assert np.array_equal(out.numpy(), want)
        for t in later:
            assert np.array_equal(t.numpy(), np.full(shape, 7.0, np.float32))
    # a block handed out during a recording is retired when it is freed later, too
    held = {}

    def allocate_only():
        held["t"] = CTensor(*shape)
        M.Set(held["t"], a, 1.0, 0.0)

    graph2 = Graph(allocate_only)
    ptr = held["t"].ptr.value
    retired = mt.get_info("retired_blocks")
    held["t"].free()
    assert mt.get_info("retired_blocks") == retired + 1
    again = CTensor(*shape)
    assert again.ptr.value != ptr
    del graph2
    # double free: the second call names a block that waits in the pool
    t = CTensor(1, 1, 8, 8)
    raw = C.c_void_p(t.ptr.value)
    t.free()
    with pytest.raises(mt.TensorError) as e:
        mt.call("mt_free", raw)
    assert "freed already" in str(e.value)


def test_workspace_growth_around_a_recording(mt):
    """A request that outgrows a workspace while the stream is captured is refused with a message; a workspace that a
    recording has seen is kept alive when a later call outgrows it."""
    from mi355tensor import CTensor, CTensorMath as M
    mt.set_option("pack_cache", 0)     # the re-ordered weights then live in the convolution workspace
    try:
        def layer(cin, cout, size):
            x, out = CTensor.from_numpy(Nrm(50, 1, cin, size, size)), CTensor(1, cout, 2 * size, 2 * size)
            k, b = CTensor.from_numpy(Nrm(51, 1, 1, cin, cout * 16, std=0.05)), CTensor.from_numpy(np.zeros((1, cin, 1, 1), np.float32))
            return lambda: mt.CTensorConv.BackwardConvolution(out, x, k, 4, 4, cout, cin, b, 2, 2, 1, 1), out
        small, small_out = layer(16, 16, 4)
        small()
        mt.synchronize()
        retired = mt.get_info("retired_workspaces")
        hip = C.CDLL("libamdhip64.so")
        stream, graph = C.c_void_p(mt.get_stream()), C.c_void_p()
        # larger than anything the process has run so far, so the workspace must grow
        exists = mt.get_info("convolution_workspace_bytes") // 4
        huge, _ = layer(1024, max(1024, 16 * (exists // (1024 * 16 * 16) + 2)) + 16 * retired, 2)
        assert hip.hipStreamBeginCapture(stream, C.c_int(2)) == 0
        try:
            small()
            with pytest.raises(mt.TensorError) as e:
                huge()
            assert "captured" in str(e.value)
        finally:
            assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        hip.hipGraphDestroy(graph)
        eager = small_out.numpy()
        huge()                                           # grows now: the block the recording saw is retired, not freed
        assert mt.get_info("retired_workspaces") == retired + 1
        small()
        assert np.array_equal(small_out.numpy(), eager)
    finally:
        mt.set_option("pack_cache", 1)


def test_small_uploads_go_through_pinned_slots(mt):
    """Uploads of at most 64 KiB are queued behind the work already queued instead of waiting for it: the caller's buffer is
    copied at once (it is overwritten right after the call here), the slots are taken again after 64 uploads, and the
    order with the kernels around them is kept.  Larger uploads and the option's other value wait as before."""
    from mi355tensor import CTensor, CTensorMath as M
    big = CTensor.from_numpy(Nrm(60, 8, 16, 64, 64))         # some queued work in front of every upload
    acc = CTensor.from_numpy(np.zeros((1, 1, 8, 16), np.float32))
    want = np.zeros((1, 1, 8, 16), np.float32)
    try:
        for staged in (1, 0):
            mt.set_option("staged_uploads", staged)
            before = mt.get_info("staged_uploads")
            buf = np.zeros((1, 1, 8, 16), np.float32)
            t = CTensor(1, 1, 8, 16)
            for i in range(150):                              # more uploads than there are slots
                buf[...] = float(i + 1)
                t.upload(buf)
                buf[...] = -1.0                               # the caller's buffer is free again
                M.Add(big, big, big, 0.5, 0.5)                # queued work between the uploads
                M.Add(acc, acc, t, 1.0, 1.0)
                want += float(i + 1)
            assert mt.get_info("staged_uploads") - before == (150 if staged else 0)
            assert np.array_equal(acc.numpy(), want)
        mt.set_option("staged_uploads", 1)
        before = mt.get_info("staged_uploads")
        large = Nrm(61, 1, 1, 256, 128)                       # 128 KiB: waits, as before
        assert np.array_equal(CTensor.from_numpy(large).numpy(), large)
        assert mt.get_info("staged_uploads") == before
    finally:
        mt.set_option("staged_uploads", 1)
