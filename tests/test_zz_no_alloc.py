"""tfhip_matmul_noalloc, the entry point for callers that cannot allocate device memory:
through the C ABI, against tfhip_matmul on the same operands (bit-equal: same kernels, the
partial tiles of a product cut along K in the library's static scratch array instead of a pool
block), on calls in a row that share the scratch array, the later ones smaller."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tfhip
    tfhip.set_backend("hip")
    return tfhip


def _both(tf, a, b, bias=None, act=0, ta=0, tb=0):
    """(result of tfhip_matmul, result of tfhip_matmul_noalloc, kernel variant, pool bytes
    before and after the no-alloc call) on freshly uploaded operands."""
    be = tf.backend()
    lib, ctx = be.lib, be.ctx
    batch = a.shape[0]
    m = a.shape[2] if ta else a.shape[1]
    k = a.shape[1] if ta else a.shape[2]
    n = b.shape[1] if tb else b.shape[2]
    with tf.tidy():
        ta_, tb_ = tf.tensor(a), tf.tensor(b)
        tbias = tf.tensor(bias) if bias is not None else None
        out1 = tf.tensor(np.full((batch, m, n), np.nan, np.float32))
        out2 = tf.tensor(np.full((batch, m, n), np.nan, np.float32))
        h = lambda t: be.data[t.data_id][0]
        args = (batch, m, n, k, ta, tb, h(tbias) if tbias is not None else -1,
                2 if tbias is not None else 0, act, -1, 0, None)
        be._ck(lib.tfhip_matmul(ctx, h(ta_), h(tb_), h(out1), *args))
        be.sync()
        mem0 = tf.memory()
        rc = lib.tfhip_matmul_noalloc(ctx, h(ta_), h(tb_), h(out2), *args)
        mem1 = tf.memory()
        if rc != 0:
            return None, lib.tfhip_last_error(ctx).decode(), None, None
        kernel = lib.tfhip_last_kernel(ctx).decode()
        r1, r2 = out1.data_sync(), out2.data_sync()
    foot = lambda mm: (mm["numBytesInGPU"], mm["numBytesInGPUPool"])
    return r1, r2, kernel, (foot(mem0), foot(mem1))


def test_noalloc_matches_matmul_on_calls_in_a_row(tf):
    rng = np.random.default_rng(70)
    seen_split = 0
    # a product that is cut along K over workgroups (too few tiles for 256 CUs, a contraction
    # too long for the single-launch kernel of small products); then smaller and differently
    # shaped ones that reuse the same scratch bytes; then some that need no scratch memory
    for (m, k, n) in [(128, 4096, 128), (128, 2304, 64), (64, 8192, 64), (32, 300, 20),
                      (128, 4096, 128), (256, 512, 256), (2048, 256, 2048)]:
        print("noalloc matmul", m, k, n, flush=True)
        a = rng.uniform(-1, 1, (1, m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (1, k, n)).astype(np.float32)
        bias = rng.standard_normal(n).astype(np.float32)
        r1, r2, kernel, mem = _both(tf, a, b, bias, act=1)
        assert r1 is not None, r2
        seen_split += "splitk" in kernel or "tailk" in kernel
        assert np.array_equal(r1, r2), (m, k, n, kernel)
        assert not np.isnan(r2).any()
        assert mem[0] == mem[1], "the pool changed during a no-alloc call: %s" % (mem,)
        want = np.maximum(a[0].astype(np.float64) @ b[0].astype(np.float64) + bias, 0)
        assert np.abs(r2[0] - want).max() < 1e-3
    assert seen_split >= 3, "the scratch path was not exercised"


def test_noalloc_rejects_what_would_need_memory(tf):
    be = tf.backend()
    rng = np.random.default_rng(71)
    # an int32 operand needs a converted copy
    with tf.tidy():
        a = tf.tensor(np.arange(6, dtype=np.int32).reshape(1, 2, 3))
        b = tf.tensor(np.ones((1, 3, 2), np.float32))
        out = tf.tensor(np.zeros((1, 2, 2), np.float32))
        h = lambda t: be.data[t.data_id][0]
        rc = be.lib.tfhip_matmul_noalloc(be.ctx, h(a), h(b), h(out), 1, 2, 2, 3, 0, 0, -1, 0, 0, -1, 0, None)
        assert rc != 0 and b"not stored as float32" in be.lib.tfhip_last_error(be.ctx)
        assert be.lib.tfhip_matmul(be.ctx, h(a), h(b), h(out), 1, 2, 2, 3, 0, 0, -1, 0, 0, -1, 0, None) == 0
    # partial tiles beyond the static array: among products with a long contraction and few
    # tiles at least one is cut so that its partial tiles exceed 8 MiB
    refused = 0
    for (m, k, n) in [(1024, 16384, 1024), (1536, 8192, 1536), (2048, 8192, 1024), (1280, 32768, 1280)]:
        a = rng.uniform(-1, 1, (1, m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (1, k, n)).astype(np.float32)
        r1, r2, kernel, _ = _both(tf, a, b)
        print("large", m, k, n, kernel if r1 is not None else r2, flush=True)
        if r1 is None:
            assert "static scratch" in r2
            refused += 1
        else:
            assert np.array_equal(r1, r2)
    assert refused >= 1


def test_noalloc_under_both_stream_indices_takes_turns_on_the_array(tf):
    """One scratch array per device, two compute streams per context: products cut along K that
    are queued under alternating stream indices, without a host wait between them, must not
    write their partial tiles into the array at the same time."""
    be = tf.backend()
    lib, ctx = be.lib, be.ctx
    rng = np.random.default_rng(72)
    shapes = [(128, 4096, 128), (64, 8192, 64)]
    h = lambda t: be.data[t.data_id][0]
    with tf.tidy():
        ops, want = [], []
        for (m, k, n) in shapes:
            a = tf.tensor(rng.uniform(-1, 1, (1, m, k)).astype(np.float32))
            b = tf.tensor(rng.uniform(-1, 1, (1, k, n)).astype(np.float32))
            ref = tf.tensor(np.zeros((1, m, n), np.float32))
            args = (1, m, n, k, 0, 0, -1, 0, 0, -1, 0, None)
            be._ck(lib.tfhip_matmul(ctx, h(a), h(b), h(ref), *args))
            assert "splitk" in lib.tfhip_last_kernel(ctx).decode()
            want.append(ref.data_sync().copy())
            ops.append((a, b, args))
        outs = []
        for i in range(12):
            a, b, args = ops[i % 2]
            be.select_stream(i % 2)
            out = tf.tensor(np.full((1,) + want[i % 2].shape[1:], np.nan, np.float32))
            be._ck(lib.tfhip_matmul_noalloc(ctx, h(a), h(b), h(out), *args))
            outs.append(out)
        # (and the same product under both indices back to back)
        for i in range(4):
            a, b, args = ops[0]
            be.select_stream(i % 2)
            out = tf.tensor(np.full(want[0].shape, np.nan, np.float32))
            be._ck(lib.tfhip_matmul_noalloc(ctx, h(a), h(b), h(out), *args))
            outs.append(out)
        be.select_stream(0)
        for i, out in enumerate(outs):
            assert np.array_equal(out.data_sync(), want[i % 2 if i < 12 else 0]), i
