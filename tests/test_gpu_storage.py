"""Storage contract of the backend (register / write / read / dispose / memory / time /
moveData) through the C ABI, after tfjs-backend-wasm/src/index_test.ts:29-49,
backends/cpu/backend_cpu_test.ts:135-175 and engine_test.ts:307-368, 452-609."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tfhip
    tfhip.set_backend("hip")
    return tfhip


def test_write_read_round_trip_all_dtypes(tf):
    with tf.tidy():
        f = tf.tensor(np.array([1.5, -2.25, 2.0 ** 35], np.float32))
        i = tf.tensor(np.array([1, -2, 2 ** 31 - 1], np.int32))
        b = tf.tensor(np.array([True, False, True]))
        assert f.data_sync().tolist() == [1.5, -2.25, 2.0 ** 35] and f.dtype == "float32"
        assert i.data_sync().tolist() == [1, -2, 2 ** 31 - 1] and i.dtype == "int32"
        assert b.data_sync().tolist() == [1, 0, 1] and b.dtype == "bool"
        z = tf.tensor(np.zeros((0, 3), np.float32))
        assert z.data_sync().shape == (0, 3)


def test_overwrite_live_buffer(tf):
    with tf.tidy():
        t = tf.tensor(np.zeros(4, np.float32))
        tf.backend().write(t.data_id, np.arange(4, dtype=np.float32))
        assert t.data_sync().tolist() == [0, 1, 2, 3]


def test_register_twice_and_null_write_throw(tf):
    be = tf.backend()
    with tf.tidy():
        t = tf.tensor(np.zeros(4, np.float32))
        with pytest.raises(RuntimeError, match="already registered"):
            be.register(t.data_id, (4,), "float32")
        with pytest.raises(ValueError, match="can not be null"):
            be.write(t.data_id, None)
    # the C ABI itself reports the same two conditions
    h = 10 ** 9
    shape = (C.c_int32 * 1)(4)
    assert be.lib.tfhip_register(be.ctx, h, shape, 1, 0) == 0
    assert be.lib.tfhip_register(be.ctx, h, shape, 1, 0) != 0
    assert b"already registered" in be.lib.tfhip_last_error(be.ctx)
    assert be.lib.tfhip_write(be.ctx, h, None, 16) != 0
    assert be.lib.tfhip_write(be.ctx, h, None, 8) != 0      # wrong size
    assert be.lib.tfhip_read(be.ctx, h + 1, None, 0) != 0   # unknown id
    assert be.lib.tfhip_dispose(be.ctx, h) == 0
    assert be.lib.tfhip_dispose(be.ctx, h) == 0             # disposing again is a no-op


def test_memory_accounting_and_pool_reuse(tf):
    """Freed blocks are reused: allocate / free cycles do not grow the device footprint
    (index_test.ts:41-49 'allocation reuse')."""
    be = tf.backend()
    base = tf.memory()
    t = tf.tensor(np.zeros(1000, np.float32))
    m1 = tf.memory()
    assert m1["numTensors"] == base["numTensors"] + 1
    assert m1["numBytes"] == base["numBytes"] + 4000
    assert m1["numDeviceBuffers"] == base["numDeviceBuffers"] + 1
    t.dispose()
    total = lambda m: m["numBytesInGPU"] + m["numBytesInGPUPool"]
    footprint = total(tf.memory())
    for _ in range(6):
        tf.tensor(np.ones(1000, np.float32)).dispose()
    assert total(tf.memory()) == footprint
    assert tf.memory()["numTensors"] == base["numTensors"]


def test_reshape_and_widening_cast_alias_the_buffer(tf):
    with tf.tidy():
        a = tf.tensor(np.array([1, 2, 3, 4], np.int32))
        n0 = tf.memory()["numDataBuffers"]
        r = tf.reshape(a, (2, 2))
        f = tf.cast(a, "float32")       # int32 -> float32: same data id, int32 storage
        assert tf.memory()["numDataBuffers"] == n0
        assert r.data_id is a.data_id and f.data_id is a.data_id
        # kernels convert from the stored dtype
        s = tf.add(f, tf.tensor(np.float32(0.5)))
        assert s.dtype == "float32" and s.data_sync().tolist() == [1.5, 2.5, 3.5, 4.5]
        m = tf.matmul(tf.reshape(f, (2, 2)), tf.tensor(np.eye(2, dtype=np.float32)))
        assert m.data_sync().ravel().tolist() == [1, 2, 3, 4]
        a.dispose()
        assert r.data_sync().ravel().tolist() == [1, 2, 3, 4], "alias keeps the buffer alive"
        i = tf.cast(tf.tensor(np.array([1.9, -1.9], np.float32)), "int32")   # narrowing: copy
        assert i.data_sync().tolist() == [1, -1]
        b = tf.cast(tf.tensor(np.array([0.0, 2.0, np.nan], np.float32)), "bool")
        assert b.data_sync().tolist() == [0, 1, 1]


def test_move_data_from_another_backend(tf):
    """A tensor created on another backend is moved on first use (engine.ts:361-363)."""
    from test_host_logic import FakeBackend
    from tfhip.engine import ENGINE
    fake = FakeBackend()
    tf.register_backend("fake-move", lambda: fake, 0)
    try:
        tf.set_backend("fake-move")
        a = tf.tensor(np.array([1, 2, 3], np.float32))
        assert len(fake.live) == 1
        tf.set_backend("hip")
        r = tf.add(a, tf.tensor(np.float32(1)))
        assert r.data_sync().tolist() == [2, 3, 4]
        assert len(fake.live) == 0, "data left the source backend"
        a.dispose()
        r.dispose()
    finally:
        tf.set_backend("hip")
        tf.remove_backend("fake-move")


def test_time_returns_kernel_ms(tf):
    with tf.tidy():
        a = tf.tensor(np.ones((512, 512), np.float32))
        info = tf.time(lambda: tf.matmul(a, a))
        assert info["kernelMs"] > 0
    assert tf.backend().float_precision() == 32 and tf.backend().epsilon() == 1e-7


def test_errors_come_back_as_exceptions(tf):
    with tf.tidy():
        a = tf.tensor(np.ones((2, 3), np.float32))
        with pytest.raises(ValueError, match="inner shapes"):
            tf.matmul(a, a)
        with pytest.raises(ValueError, match="could not be broadcast"):
            tf.add(a, tf.tensor(np.ones((2, 2), np.float32)))
        with pytest.raises(ValueError, match="has not been implemented"):
            tf.fused.matmul(a, tf.tensor(np.ones((3, 2), np.float32)), activation="elu")
        with pytest.raises(ValueError, match="depth of input"):
            tf.conv2d(tf.tensor(np.ones((1, 4, 4, 3), np.float32)),
                      tf.tensor(np.ones((3, 3, 2, 8), np.float32)), 1, "same")


def test_captured_graph_replays_match_eager_runs():
    """A chain of conv / depthwise / pointwise / pool / matmul / softmax kernels captured once and
    replayed several times, with eager work, new input data and synchronisations between the
    replays: every replay must equal the eager result for the input then in place, the blocks
    the graph wrote must not be handed to other tensors while it lives, and destroying it returns
    them to the pool."""
    import tfhip as tf
    tf.set_backend("hip")
    rng = np.random.default_rng(91)
    f32 = lambda *s: rng.standard_normal(s).astype(np.float32)
    w0, b0 = f32(3, 3, 3, 16) * 0.3, f32(16) * 0.1
    dw, w1, b1 = f32(3, 3, 16, 1) * 0.3, f32(1, 1, 16, 32) * 0.3, f32(32) * 0.1
    fc = f32(32, 10) * 0.3
    with tf.tidy():
        wt = [tf.tensor(a) for a in (w0, b0, dw, w1, b1, fc)]
        x = tf.tensor(f32(2, 16, 16, 3))

        def net():
            h = tf.fused.conv2d(x, wt[0], 2, "same", bias=wt[1], activation="relu6")
            h = tf.depthwise_conv2d(h, wt[2], 1, "same")
            h = tf.fused.conv2d(h, wt[3], 1, "same", bias=wt[4], activation="relu")
            h = tf.avg_pool(h, 8, 8, "valid")
            return tf.softmax(tf.matmul(tf.reshape(h, (2, 32)), wt[5]))

        def eager():
            with tf.tidy():
                return net().data_sync()

        before = tf.memory()
        g = tf.capture_graph(net)
        out = g.outputs
        for k in range(4):
            new_x = f32(2, 16, 16, 3)
            tf.backend().write(x.data_id, new_x)          # new data into the same tensor
            want = eager()                                 # eager work between the replays
            junk = [tf.tensor(f32(2, 8, 8, 16)) for _ in range(6)]   # takes blocks from the pool
            junk_want = [t.data_sync() for t in junk]
            g.replay()
            got = out.data_sync()                          # synchronises
            np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-7, err_msg="replay %d" % k)
            for t, wv in zip(junk, junk_want):             # the replay wrote none of their blocks
                assert np.array_equal(t.data_sync(), wv)
                t.dispose()
        # write / read are refused inside a capture and the capture still ends cleanly
        tf.backend().lib.tfhip_graph_begin(tf.backend().ctx)
        with pytest.raises(Exception, match="graph capture"):
            with tf.tidy():
                tf.tensor(f32(4))
        import ctypes
        gid = ctypes.c_int64()
        if tf.backend().lib.tfhip_graph_end(tf.backend().ctx, ctypes.byref(gid)) == 0:
            assert tf.backend().lib.tfhip_graph_destroy(tf.backend().ctx, gid.value) == 0
        with tf.tidy():
            assert tf.tensor(f32(4)).data_sync().shape == (4,)  # eager work goes on afterwards
        g.dispose()
        after = tf.memory()
        assert after["numDeviceBuffers"] == before["numDeviceBuffers"]
        assert after["numBytesInGPU"] == before["numBytesInGPU"]


# ---- copies that overlap with kernels ------------------------------------------------------
def _chain(tf, x, w):
    """A few milliseconds of dependent kernels whose result depends on every element of x."""
    h = x
    for _ in range(6):
        h = tf.relu(tf.matmul(h, w))
    return h


def test_large_pageable_and_pinned_uploads_arrive_whole(tf):
    """Writes above the ring-slot size run on the upload stream; the first kernel that reads
    the tensor waits for the copy.  Checked for ordinary and for page-locked source memory, on
    fresh blocks and on blocks that come back from the pool with kernels still reading them."""
    rng = np.random.default_rng(21)
    n = 1 << 20
    pinned = tf.pinned_array("float32", (n,))
    for round_ in range(6):
        src = rng.standard_normal(n).astype(np.float32)
        if round_ % 2:
            pinned[:] = src
            src_arr = pinned
        else:
            src_arr = src
        with tf.tidy():
            t = tf.tensor(src_arr)
            y = tf.add(tf.mul(t, t), t)      # reads the block while the next round's tensor ...
            got = y.data_sync()
        np.testing.assert_array_equal(got, src * src + src)
        # ... is registered here into the block t just gave back


def test_upload_overlapping_a_running_step_never_tears(tf):
    """A pipelined loop as the benchmark runs it: batch i+1 is uploaded from pinned memory
    while the kernels of batch i run, input blocks cycle through the pool, results are read
    asynchronously two steps late.  Every result must equal the eager, fully synchronised
    one: a kernel that read a half-written input, or an upload that overwrote an input still
    being read, would differ."""
    rng = np.random.default_rng(22)
    m = 1024
    w_np = (rng.standard_normal((m, m)) / np.sqrt(m)).astype(np.float32)
    batches = [rng.standard_normal((m, m)).astype(np.float32) for _ in range(4)]
    slots = [tf.pinned_array("float32", (m, m)) for _ in range(2)]
    w = tf.tensor(w_np)
    want = []
    for b in batches:
        with tf.tidy():
            want.append(_chain(tf, tf.tensor(b), w).data_sync())
        tf.backend().sync()
    steps = 24
    pending, got = [], []
    slots[0][:] = batches[0]
    nxt = tf.tensor(slots[0])
    for i in range(steps):
        cur = nxt
        if i + 1 < steps:
            # the slot was the source of batch i-1, whose result has been waited for below
            slots[(i + 1) % 2][:] = batches[(i + 1) % 4]
            nxt = tf.tensor(slots[(i + 1) % 2])          # upload overlaps with the step below
        out = _chain(tf, cur, w)
        cur.dispose()
        pending.append(out.data())
        out.dispose()                                     # disposed with the read in flight
        if len(pending) > 1:
            got.append(pending.pop(0).result())
    got += [p.result() for p in pending]
    w.dispose()
    assert len(got) == steps
    for i, g in enumerate(got):
        np.testing.assert_array_equal(g, want[i % 4], err_msg="step %d" % i)


def test_overwrite_of_a_tensor_that_queued_kernels_still_read(tf):
    rng = np.random.default_rng(23)
    a = rng.standard_normal((512, 512)).astype(np.float32)
    b = rng.standard_normal((512, 512)).astype(np.float32)
    w_np = (rng.standard_normal((512, 512)) / 22).astype(np.float32)
    with tf.tidy():
        w = tf.tensor(w_np)
        t = tf.tensor(a)
        ya = _chain(tf, t, w)
        tf.backend().write(t.data_id, b)     # large write into a buffer with readers queued
        yb = _chain(tf, t, w)
        small = tf.tensor(np.zeros(8, np.float32))
        s1 = tf.add(small, small)
        tf.backend().write(small.data_id, np.arange(8, dtype=np.float32))  # ring-slot path
        s2 = tf.add(small, small)
        got_a, got_b = ya.data_sync(), yb.data_sync()
        assert s1.data_sync().tolist() == [0] * 8
        assert s2.data_sync().tolist() == [2 * i for i in range(8)]
        t2 = tf.tensor(a)
        want_a = _chain(tf, t2, w).data_sync()
        t3 = tf.tensor(b)
        want_b = _chain(tf, t3, w).data_sync()
    np.testing.assert_array_equal(got_a, want_a)
    np.testing.assert_array_equal(got_b, want_b)


def test_many_small_writes_wrap_the_staging_ring(tf):
    with tf.tidy():
        ts = [tf.tensor(np.full(100, i, np.float32)) for i in range(200)]
        total = ts[0]
        for t in ts[1:]:
            total = tf.add(total, t)
        assert total.data_sync().tolist() == [sum(range(200))] * 100


def test_async_read_returns_what_sync_read_returns(tf):
    rng = np.random.default_rng(24)
    with tf.tidy():
        for dtype, vals in (("float32", rng.standard_normal(70000).astype(np.float32)),
                            ("int32", rng.integers(-9, 9, 333).astype(np.int32)),
                            ("bool", rng.integers(0, 2, 50) != 0)):
            t = tf.tensor(vals)
            p = t.data()
            np.testing.assert_array_equal(p.result(), t.data_sync())
        empty = tf.tensor(np.zeros((0, 4), np.float32))
        assert empty.data().result().shape == (0, 4)
    be = tf.backend()
    ticket = C.c_void_p()
    assert be.lib.tfhip_read_begin(be.ctx, 10 ** 9 + 7, C.byref(ticket)) != 0   # unknown id
    assert b"unknown data id" in be.lib.tfhip_last_error(be.ctx)


def test_dispose_during_an_async_read_keeps_the_block_out_of_reach(tf):
    """A tensor disposed while its asynchronous read is still copying: the block neither goes to
    the next tensor of that size before the copy is done (the pool holds it back until the read
    is finished), nor is it lost (afterwards the pool hands it out again), and tf.memory() counts
    it as pooled, not in use, from the dispose on."""
    rng = np.random.default_rng(25)
    n = 3 * 1000 * 1000 + 17                 # a size class no other test of this module uses
    vals = [rng.standard_normal(n).astype(np.float32) for _ in range(4)]
    be = tf.backend()
    two = tf.tensor(np.float32(2.0))
    base = tf.memory()["numBytesInGPU"]
    reads = []
    for i, v in enumerate(vals):
        t = tf.tensor(v)
        u = tf.mul(t, two)                     # queued work in front of the read
        reads.append(u.data())
        tf.dispose([t, u])                    # while the copy of u is (most likely) still running
        # the next tensor of the same size must not land in u's block before the copy is over
        w = tf.tensor(np.full(n, -7.0, np.float32))
        tf.dispose(tf.add(w, w))
        w.dispose()
    assert tf.memory()["numBytesInGPU"] == base
    for v, r in zip(vals, reads):
        np.testing.assert_array_equal(r.result(), v * np.float32(2.0))
    pooled = tf.memory()["numBytesInGPUPool"]
    t = tf.tensor(vals[0])                    # comes out of the pool: no new device memory
    assert tf.memory()["numBytesInGPUPool"] < pooled
    np.testing.assert_array_equal(t.data_sync(), vals[0])
    tf.dispose([t, two])


def test_time_reports_every_kernel_and_nests(tf):
    """KernelBackend.time with the per-kernel figures behind getExtraProfileInfo
    (backend.ts:27-31): one entry per launch, in order, each the execution time of its kernel."""
    rng = np.random.default_rng(25)
    with tf.tidy():
        a = tf.tensor(rng.standard_normal((512, 512)).astype(np.float32))
        x = tf.tensor(rng.standard_normal((2, 32, 32, 16)).astype(np.float32))
        f = tf.tensor(rng.standard_normal((3, 3, 16, 1)).astype(np.float32))
        inner = {}

        def work():
            tf.matmul(a, a)
            inner.update(tf.time(lambda: tf.relu(a)))
            tf.depthwise_conv2d(x, f, 1, "same")
            tf.softmax(a)

        tf.matmul(a, a)
        info = tf.time(work)
    names = [k[0] for k in info["kernelTimes"]]
    if names[0].endswith("_splitk"):   # a product cut along K is two launches, each with its own line
        assert names[1] == "splitk_finish", names
        del names[1]
    assert len(names) == 4, names
    assert names[0].startswith("gemm_") and names[2].startswith("depthwise")
    assert names[1] == "tfhip_unary" and names[3] == "tfhip_softmax_rows", names
    assert all(ms > 0 for _, ms in info["kernelTimes"])
    total = sum(ms for _, ms in info["kernelTimes"])
    assert 0 < total <= info["kernelMs"] * 1.001   # idle time between kernels is in the total only
    assert [k[0] for k in inner["kernelTimes"]] == ["tfhip_unary"]
    assert 0 < inner["kernelMs"] < info["kernelMs"]
    assert info["getExtraProfileInfo"]().count(":") == len(info["kernelTimes"])
    be = tf.backend()
    ms = C.c_float()
    assert be.lib.tfhip_time_end(be.ctx, C.byref(ms)) != 0      # no region is open
    be.lib.tfhip_time_per_kernel(be.ctx, 0)
    try:
        with tf.tidy():
            a = tf.tensor(np.ones((64, 64), np.float32))
            quiet = tf.time(lambda: tf.matmul(a, a))
        assert quiet["kernelTimes"] == [] and quiet["kernelMs"] > 0
    finally:
        be.lib.tfhip_time_per_kernel(be.ctx, 1)


# ------------------------------------------------------- two compute streams ----
def _small_net(tf, x, w1, dw, w2):
    """conv 3x3 -> depthwise 3x3 -> global mean -> matMul: enough kernels, pool blocks and
    scratch memory (the product is cut along K) to notice a block handed to the wrong stream."""
    def run():
        h = tf.fused.conv2d(x, w1, 1, "same", activation="relu6")
        h = tf.fused.depthwise_conv2d(h, dw, 1, "same", activation="relu6")
        h = tf.mean(h, [1, 2])
        return tf.matmul(h, w2)
    return tf.tidy(run)


def test_two_streams_give_the_results_of_one(tf):
    """Independent passes queued alternately under the two compute streams (select_stream)
    overlap on the device; every result equals the one the same pass gives alone, the pools give
    back what they took, and a read follows the stream its tensor was produced on."""
    be = tf.backend()
    rng = np.random.default_rng(31)
    w1 = tf.tensor((rng.standard_normal((3, 3, 16, 64)) * 0.1).astype(np.float32))
    dw = tf.tensor((rng.standard_normal((3, 3, 64, 1)) * 0.3).astype(np.float32))
    w2 = tf.tensor((rng.standard_normal((64, 4096)) * 0.1).astype(np.float32))
    xs = [rng.uniform(0, 1, (8, 48 + 8 * (i % 3), 40, 16)).astype(np.float32) for i in range(6)]
    want = []
    for x in xs:                                   # one stream
        t = tf.tensor(x)
        y = _small_net(tf, t, w1, dw, w2)
        want.append(y.data_sync().copy())
        tf.dispose([t, y])
    base = tf.memory()
    for rounds in range(3):
        outs = []
        for i, x in enumerate(xs):                 # two streams, nothing awaited in between
            be.select_stream(i % 2)
            t = tf.tensor(x)
            outs.append(_small_net(tf, t, w1, dw, w2))
            t.dispose()
        be.select_stream(0)                        # (reads below are issued under index 0)
        for i, y in enumerate(outs):
            got = y.data().result() if i % 2 else y.data_sync()
            assert np.array_equal(got, want[i]), (rounds, i)
            y.dispose()
    after = tf.memory()
    assert after["numTensors"] == base["numTensors"]
    assert after["numBytesInGPU"] == base["numBytesInGPU"]
    tf.dispose([w1, dw, w2])


def test_select_stream_rejects_what_it_cannot_do(tf):
    be = tf.backend()
    with pytest.raises(RuntimeError, match="2 compute streams"):
        be.select_stream(2)
    with pytest.raises(RuntimeError, match="2 compute streams"):
        be.select_stream(-1)
    a = tf.tensor(np.ones((4, 4), np.float32))
    with pytest.raises(RuntimeError, match="timed region"):
        tf.time(lambda: be.select_stream(1))
    be.select_stream(1)
    b = tf.relu(a)                                  # produced under index 1 ...
    be.select_stream(0)
    assert b.data_sync().tolist() == a.data_sync().tolist()   # ... read under index 0
    tf.dispose([a, b])                              # ... and disposed under index 0


def test_tensor_handed_from_one_stream_to_the_other(tf):
    """A tensor produced under one stream index and used under the other right away: the second
    stream waits for the first one's work (no host wait in between), so the result is the one a
    single stream gives.  The pool blocks are filled with other values first, so that a kernel
    that ran ahead of its input would read those."""
    be = tf.backend()
    rng = np.random.default_rng(33)
    n = 3072
    a = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.05)
    w = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.05)
    with tf.tidy():
        want = tf.relu(tf.matmul(tf.matmul(a, w), w)).data_sync().copy()
    for rounds in range(2):
        tf.dispose([tf.fill((n, n), -1.0) for _ in range(3)])
        be.select_stream(0)
        p = tf.matmul(a, w)                         # a chain of long kernels under index 0 ...
        q = tf.matmul(p, w)
        be.select_stream(1)
        r = tf.relu(q)                              # ... and their result used under index 1
        be.select_stream(0)
        got = r.data_sync()
        assert np.array_equal(got, want), rounds
        tf.dispose([p, q, r])
    tf.dispose([a, w])


def test_block_used_under_both_streams_returns_behind_both(tf):
    """A tensor that work under both stream indices reads is disposed and its block taken again
    at once under the index that used it last: the new owner is ordered behind the other stream's
    readers too."""
    be = tf.backend()
    rng = np.random.default_rng(34)
    n = 3072
    a = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.05)
    w = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.05)
    with tf.tidy():
        want = tf.matmul(tf.relu(a), w).data_sync().copy()
    for rounds in range(2):
        be.select_stream(0)
        b = tf.relu(a)
        be.select_stream(1)
        busy = tf.tidy(lambda: tf.matmul(tf.matmul(a, w), w))   # keeps index 1 busy: b is read late
        c = tf.matmul(b, w)                         # reads b under index 1
        be.select_stream(0)
        d = tf.neg(b)                               # b's last use is under index 0
        b.dispose()
        e = tf.fill((n, n), 7.0)                    # takes b's block from the pool of index 0
        assert np.array_equal(c.data_sync(), want), rounds
        assert float(e.data_sync().flat[0]) == 7.0
        tf.dispose([busy, c, d, e])
    be.select_stream(0)
    tf.dispose([a, w])


def test_graph_captured_under_one_stream_reads_what_the_other_wrote(tf):
    """A graph recorded under stream index 0 whose kernels read a tensor produced under index 1
    just before: the producer is waited for before the recording (a captured stream cannot wait
    for an event from outside), the graph replays on the stream of its capture whichever index is
    selected, and its result read under either index is the eager one."""
    be = tf.backend()
    rng = np.random.default_rng(35)
    n = 1024
    a = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.05)
    w = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.05)
    be.select_stream(1)
    b = tf.tidy(lambda: tf.matmul(tf.matmul(a, w), w))   # under index 1, still running
    be.select_stream(0)
    net = lambda: tf.relu(tf.matmul(b, w))
    g = tf.capture_graph(net)
    with tf.tidy():
        want = net().data_sync().copy()
    for k in range(3):
        be.select_stream(k % 2)                            # replays ignore the selected index
        g.replay()
        assert np.array_equal(g.outputs.data_sync(), want), k
    be.select_stream(0)
    g.dispose()
    tf.dispose([a, w, b])


def test_graph_replays_are_ordered_against_the_other_stream(tf):
    """A replayed graph writes its tensors every time, so the rule "tensors are written once"
    cannot order it.  Recorded under index 0; five replays, each fed by a small write (copied by
    the selected stream, index 1) and each consumed by kernels under index 1 that are still
    running when the next replay would overwrite what they read.  No host wait in between."""
    be = tf.backend()
    rng = np.random.default_rng(36)
    n = 2048
    u = tf.tensor(rng.standard_normal((n, 64)).astype(np.float32) * 0.2)
    w1 = tf.tensor(rng.standard_normal((64, n)).astype(np.float32) * 0.2)
    w2 = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.03)
    w3 = tf.tensor(rng.standard_normal((n, 64)).astype(np.float32) * 0.03)
    x = tf.tensor(np.zeros((64, 64), np.float32))            # 16 KiB: written through the ring
    net = lambda: tf.matmul(tf.relu(tf.matmul(tf.matmul(u, x), w1)), w2)      # [n, n]
    consume = lambda y: tf.tidy(lambda: tf.matmul(tf.relu(tf.matmul(tf.matmul(y, w2), w2)), w3))
    inputs = [rng.standard_normal((64, 64)).astype(np.float32) for _ in range(5)]
    want = []
    for xi in inputs:
        be.write(x.data_id, xi)
        with tf.tidy():
            want.append(consume(net()).data_sync().copy())
    g = tf.capture_graph(net)                                 # recorded under index 0
    pending = []
    for xi in inputs:
        be.select_stream(1)
        be.write(x.data_id, xi)                               # a copy queued on stream 1
        g.replay()                                            # on stream 0
        z = consume(g.outputs)                                # on stream 1
        pending.append(z.data())
        z.dispose()
    got = [p.result() for p in pending]
    # and the other way round: index 0 selected, the consumer runs on the replay's own stream
    be.select_stream(0)
    be.write(x.data_id, inputs[0])
    g.replay()
    with tf.tidy():
        got.append(consume(g.outputs).data_sync().copy())
    # an asynchronous read of the graph's own result, still copying when the next replay comes
    be.write(x.data_id, inputs[1])
    g.replay()
    first = g.outputs.data()
    be.write(x.data_id, inputs[2])
    g.replay()
    second = g.outputs.data_sync().copy()
    first = first.result()
    g.dispose()
    for i, (a, e) in enumerate(zip(got, want + [want[0]])):
        assert np.array_equal(a, e), i
    for xi, y in ((inputs[1], first), (inputs[2], second)):
        be.write(x.data_id, xi)
        with tf.tidy():
            assert np.array_equal(net().data_sync(), y)
    tf.dispose([u, w1, w2, w3, x])


def test_block_held_by_a_read_goes_to_the_other_stream_behind_its_last_use(tf):
    """A tensor is read asynchronously, used again by kernels queued under index 0 and disposed
    while the copy runs; under index 1 a tensor of the same size then takes that very block (the
    pool of stream 1 has none of the size) and a kernel overwrites it.  The overwrite has to wait
    for stream 0's kernels, not only for the copy."""
    be = tf.backend()
    rng = np.random.default_rng(37)
    m, n = 2056, 2048                                         # a capacity no other test leaves behind
    a = tf.tensor(rng.standard_normal((m, n)).astype(np.float32) * 0.03)
    w = tf.tensor(rng.standard_normal((n, n)).astype(np.float32) * 0.03)

    def chain(y):
        def f():
            tf.matmul(tf.matmul(tf.matmul(w, w), w), w)       # long work queued ahead of y's reader
            return tf.matmul(y, w)
        return tf.tidy(f)

    with tf.tidy():
        y = tf.matmul(a, w)
        want_y = y.data_sync().copy()
        want_z = chain(y).data_sync().copy()
    be.sync()
    y = tf.matmul(a, w)
    p = y.data()                                              # copying on the download stream
    z = chain(y)                                              # long work under index 0 that reads y last
    pooled0 = tf.memory()["numBytesInGPUPool"]
    y.dispose()                                               # held: the read is still copying
    held = tf.memory()["numBytesInGPUPool"] - pooled0
    be.select_stream(1)
    t = tf.fill((m, n), 7.0)                                  # stream 1 writes into the block
    took = pooled0 + held - tf.memory()["numBytesInGPUPool"]
    tv = t.data_sync()
    be.select_stream(0)
    assert np.array_equal(p.result(), want_y)
    assert np.array_equal(z.data_sync(), want_z)
    assert np.all(tv == 7.0)
    assert held >= m * n * 4 and took == held, (held, took)   # the held block was the one handed out
    tf.dispose([a, w, z, t])


def test_pipelined_uploads_with_two_batches_in_flight(tf):
    """The serving loop of the benchmark in small: every step uploads its input from page-locked
    memory, runs under the stream of its parity and is read back asynchronously two steps late.
    The next upload never has to take the block whose readers are still queued."""
    be = tf.backend()
    rng = np.random.default_rng(32)
    w1 = tf.tensor((rng.standard_normal((3, 3, 16, 64)) * 0.1).astype(np.float32))
    dw = tf.tensor((rng.standard_normal((3, 3, 64, 1)) * 0.3).astype(np.float32))
    w2 = tf.tensor((rng.standard_normal((64, 4096)) * 0.1).astype(np.float32))
    shape = (32, 64, 64, 16)                       # 8 MiB per batch: an upload on the copy stream
    slots = [tf.pinned_array("float32", shape) for _ in range(3)]
    want = []
    for k, s in enumerate(slots):
        s[...] = rng.uniform(0, 1, shape).astype(np.float32)
        t = tf.tensor(s)
        y = _small_net(tf, t, w1, dw, w2)
        want.append(y.data_sync().copy())
        tf.dispose([t, y])
    pending, got = [], []
    nxt = tf.tensor(slots[0])
    n = 24
    for i in range(n):
        be.select_stream(i % 2)
        cur = nxt
        if i + 1 < n:
            nxt = tf.tensor(slots[(i + 1) % 3])
        y = _small_net(tf, cur, w1, dw, w2)
        pending.append(y.data())
        tf.dispose([cur, y])
        if len(pending) > 2:
            got.append(pending.pop(0).result())
    got += [p.result() for p in pending]
    be.select_stream(0)
    for i, g in enumerate(got):
        assert np.array_equal(g, want[i % 3]), i
    tf.dispose([w1, dw, w2])
