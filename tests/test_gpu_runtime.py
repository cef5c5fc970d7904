"""The runtime half of the C ABI on a real MI355X: the caching allocator behind agh_malloc / agh_free
(the reference allocates one output per op, src/tensor.rs:1377-1389), the library's workspace under live
graphs, and the branch stream's bookkeeping around waits and copies."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ag():
    import autograph_amd as ag
    ag.Device(0)
    return ag


def cache_stats(ag):
    a, b, c = C.c_size_t(), C.c_size_t(), C.c_size_t()
    ag._ffi.check(ag.lib.agh_cache_stats(C.byref(a), C.byref(b), C.byref(c)))
    return a.value, b.value, c.value


def test_malloc_free_reuses_blocks_in_stream_order(ag):
    """alloc -> launch -> free -> alloc -> launch: the second allocation gets the first one's block back while
    the first launch may still be queued, and every result equals the one computed on fresh memory."""
    rng = np.random.default_rng(31)
    a = rng.uniform(-1, 1, (512, 384)).astype(np.float32)
    b = rng.uniform(-1, 1, (384, 256)).astype(np.float32)
    ta, tb = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
    first = ta.dot(tb)
    want = first.into_array()
    ptr0 = first.buffer.ptr
    del first
    _, blocks, live = cache_stats(ag)
    assert blocks >= 1
    ptrs = set()
    for _ in range(20):  # no wait between the iterations: free and reuse race only with queued work
        out = ta.dot(tb)
        ptrs.add(out.buffer.ptr)
        del out
    # every allocation was served from the cache: the driver was not asked for a single new block
    assert cache_stats(ag)[1:] == (blocks, live)
    assert len(ptrs) <= blocks and (blocks > 1 or ptrs == {ptr0})
    out = ta.dot(tb)
    assert np.array_equal(out.into_array(), want)
    # a chain whose intermediates are dropped as soon as the next op is queued (what `Tensor::dot(..)?.relu()` does)
    x = ta
    for _ in range(4):
        x = x.dot(tb).relu().dot(tb.t())
    got = x.into_array()
    h = a
    for _ in range(4):
        h = np.maximum(h @ b, 0) @ b.T
    assert np.allclose(got, h, rtol=2e-3, atol=2e-3 * np.abs(h).max())


def test_free_of_a_buffer_a_queued_kernel_still_reads(ag):
    """agh_free returns at once; a kernel queued before it still reads the right bytes even though the block
    is handed out again and overwritten by a later upload (which is ordered after the kernel)."""
    rng = np.random.default_rng(32)
    n = 2048
    a = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    ta = ag.Tensor.from_array(a)
    ident = ag.Tensor.from_array(np.eye(n, dtype=np.float32))
    outs = []
    for i in range(6):
        src = ag.Tensor.from_array(a + np.float32(i))      # upload i
        outs.append(src.dot(ident))                          # queued GEMM reads `src`
        del src                                              # freed while the GEMM may not have started
    for i, o in enumerate(outs):
        assert np.array_equal(o.into_array(), a + np.float32(i)), i
    del ta


def test_cache_release_and_stats(ag):
    t = ag.Tensor.zeros((1 << 20,), "f32")
    del t
    cached, blocks, _ = cache_stats(ag)
    assert cached >= 4 << 20 and blocks >= 1
    ag._ffi.check(ag.lib.agh_cache_release())
    assert cache_stats(ag)[:2] == (0, 0)
    # zero-length and odd sizes still work
    p = C.c_void_p()
    ag._ffi.check(ag.lib.agh_malloc(C.byref(p), 0))
    assert p.value
    ag._ffi.check(ag.lib.agh_free(p))
    ag._ffi.check(ag.lib.agh_free(None))


def test_graph_replay_survives_workspace_growth(ag, monkeypatch):
    """A captured split-K GEMM names the library's workspace in its nodes.  A much larger split-K GEMM run
    eagerly afterwards needs a bigger workspace: the old block must stay alive for the graph's replays."""
    rng = np.random.default_rng(33)
    ag._ffi.check(ag.lib.agh_cache_release())   # earlier tests may have grown the workspace: start from none
    m, k, n = 6, 57600, 25                      # dW of LeNet5's first convolution: 256 k-groups
    dy = rng.normal(0, 1, (k, m)).astype(np.float32)
    cols = rng.normal(0, 1, (k, n)).astype(np.float32)
    tdy, tcols = ag.Tensor.from_array(dy), ag.Tensor.from_array(cols)
    out = ag.Tensor.uninit((m, n), "f32")
    ag.gemm(1.0, tdy.t(), tcols, 0.0, out)      # eager: sizes the workspace
    want = out.into_array()
    ag._ffi.check(ag.lib.agh_graph_begin())
    try:
        ag.gemm(1.0, tdy.t(), tcols, 0.0, out)
    finally:
        g = C.c_void_p()
        ag._ffi.check(ag.lib.agh_graph_end(C.byref(g)))
    try:
        # 16 k-groups x 512 x 512 f32 partials = 16 MiB > the 8 MiB first block
        big_a = ag.Tensor.from_array(rng.uniform(-1, 1, (512, 2048)).astype(np.float32))
        big_b = ag.Tensor.from_array(rng.uniform(-1, 1, (2048, 512)).astype(np.float32))
        big = big_a.dot(big_b)
        for _ in range(3):
            ag._ffi.check(ag.lib.agh_memset(out._ptr(), 0xFF, m * n * 4))
            ag._ffi.check(ag.lib.agh_graph_launch(g))
            # the large GEMM again, between replays: it now owns the new workspace
            big2 = big_a.dot(big_b)
            assert np.array_equal(out.into_array(), want)
            assert np.array_equal(big2.into_array(), big.into_array())
        # growth is refused while capturing (nothing may allocate or wait inside a capture)
        # (allocated before the capture starts; 32 k-groups forced: 128 MiB of partials)
        huge_a, huge_b = ag.Tensor.uninit((1024, 32768), "f32"), ag.Tensor.uninit((32768, 1024), "f32")
        huge_c = ag.Tensor.uninit((1024, 1024), "f32")
        monkeypatch.setenv("AGH_GEMM_SPLITS", "32")
        ag._ffi.check(ag.lib.agh_graph_begin())
        try:
            with pytest.raises(ag.AghError, match="capturing"):
                ag.gemm(1.0, huge_a, huge_b, 0.0, huge_c)
        finally:
            monkeypatch.delenv("AGH_GEMM_SPLITS")
            g2 = C.c_void_p()
            rc = ag.lib.agh_graph_end(C.byref(g2))
            if rc == 0 and g2.value:
                ag._ffi.check(ag.lib.agh_graph_destroy(g2))
    finally:
        ag._ffi.check(ag.lib.agh_graph_destroy(g))
    ag._ffi.check(ag.lib.agh_sync())


def test_sync_and_copies_inside_a_branch(ag):
    """Tensor.from_array (upload + agh_sync) and into_array inside `with branch():` must neither lose the
    branch's later launches nor read a result before its producer has run."""
    rng = np.random.default_rng(34)
    a = rng.uniform(-1, 1, (300, 200)).astype(np.float32)
    b = rng.uniform(-1, 1, (200, 100)).astype(np.float32)
    ta = ag.Tensor.from_array(a)
    with ag.branch():
        tb = ag.Tensor.from_array(b)            # upload on the branch stream, then a sync inside the branch
        side = ta.dot(tb)                        # launched on the branch stream after that sync
        inside = side.into_array()               # copy inside the branch: waits for the producer
    main = ta.relu()                             # main stream, beside the branch
    outside = side.into_array()                  # no join yet: the copy itself must wait for the branch
    ag.join()
    want = orc.gemm_f64acc(a, b)
    assert np.allclose(inside, want, atol=1e-4) and np.array_equal(inside, outside)
    assert np.array_equal(main.into_array(), np.maximum(a, 0))
    # a capture with a sync-free branch still closes (the arm is joined by agh_graph_end)
    out = ag.Tensor.uninit((300, 100), "f32")
    ag.gemm(1.0, ta, tb, 0.0, out)
    ag._ffi.check(ag.lib.agh_sync())
    ag._ffi.check(ag.lib.agh_graph_begin())
    try:
        with ag.branch():
            ag.gemm(1.0, ta, tb, 0.0, out)
    finally:
        g = C.c_void_p()
        ag._ffi.check(ag.lib.agh_graph_end(C.byref(g)))
    ag._ffi.check(ag.lib.agh_memset(out._ptr(), 0, 300 * 100 * 4))
    ag._ffi.check(ag.lib.agh_graph_launch(g))
    assert np.array_equal(out.into_array(), inside)
    ag._ffi.check(ag.lib.agh_graph_destroy(g))


def test_block_freed_under_an_unjoined_branch_is_reused_safely(ag):
    """A block last used on the branch stream and freed before the join: the main stream's next user of that
    block waits for the branch."""
    rng = np.random.default_rng(35)
    n = 1536
    a = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    ta = ag.Tensor.from_array(a)
    ident = ag.Tensor.from_array(np.eye(n, dtype=np.float32))
    for i in range(4):
        with ag.branch():
            tmp = ta.dot(ident)                  # branch stream writes `tmp`
            res = tmp.dot(ident)                 # and reads it
        del tmp                                  # freed, branch not joined
        again = ta.relu()                        # main stream: same size class -> may get tmp's block
        ag.join()
        assert np.array_equal(res.into_array(), a), i
        assert np.array_equal(again.into_array(), np.maximum(a, 0)), i
        del res, again


def test_free_during_capture_is_deferred_not_lost(ag):
    """A host-side temporary may be dropped at any moment, also while a graph is being captured (the garbage collector
    does not ask).  agh_free then sets the block aside: it is neither handed to the driver nor reused inside the
    capture, and agh_graph_end files it with the cached blocks, so nothing leaks."""
    rng = np.random.default_rng(61)
    a = ag.Tensor.from_array(rng.uniform(-1, 1, (64, 64)).astype(np.float32))
    out = ag.Tensor.uninit((64, 64), "f32")
    victim = ag.Tensor.uninit((12345,), "f32")          # a size class of its own
    ag.gemm(1.0, a, a, 0.0, out)                          # eager run first
    ag._ffi.check(ag.lib.agh_sync())
    cached0, blocks0, live0 = cache_stats(ag)
    ag._ffi.check(ag.lib.agh_graph_begin())
    try:
        ag.gemm(1.0, a, a, 0.0, out)
        ptr = victim.buffer.ptr
        rc = ag.lib.agh_free(ptr)                         # what Buffer.__del__ does
        victim.buffer.ptr = None
        assert rc == 0
        # not reusable yet, but no longer counted as handed out
        assert cache_stats(ag)[2] == live0 - 1 and cache_stats(ag)[1] == blocks0
    finally:
        g = C.c_void_p()
        ag._ffi.check(ag.lib.agh_graph_end(C.byref(g)))
    try:
        cached1, blocks1, live1 = cache_stats(ag)
        assert live1 == live0 - 1 and blocks1 == blocks0 + 1 and cached1 > cached0
        again = ag.Tensor.uninit((12345,), "f32")         # the same size class: the deferred block comes back
        assert again.buffer.ptr == ptr
        ag._ffi.check(ag.lib.agh_graph_launch(g))
        ag._ffi.check(ag.lib.agh_sync())
    finally:
        ag._ffi.check(ag.lib.agh_graph_destroy(g))


def test_graph_replay_joins_an_open_branch_first(ag, monkeypatch):
    """A graph captured with a branch names the second stream's split-K workspace in its fork arm.  Eager split-K work
    inside a branch that has not been joined may still be using that block when the graph is replayed: agh_graph_launch
    orders the replay behind it.  Both products must come out as they do alone, on every repetition."""
    rng = np.random.default_rng(62)
    dy1, c1 = rng.normal(0, 1, (57600, 6)).astype(np.float32), rng.normal(0, 1, (57600, 25)).astype(np.float32)
    dy2, c2 = rng.normal(0, 1, (36864, 48)).astype(np.float32), rng.normal(0, 1, (36864, 40)).astype(np.float32)
    t1a, t1b, t2a, t2b = (ag.Tensor.from_array(v) for v in (dy1, c1, dy2, c2))
    out1, out2 = ag.Tensor.uninit((6, 25), "f32"), ag.Tensor.uninit((48, 40), "f32")
    # serial results; the second product also sizes the second stream's workspace for both
    with ag.branch():
        ag.gemm(1.0, t2a.t(), t2b, 0.0, out2)
        ag.gemm(1.0, t1a.t(), t1b, 0.0, out1)
    ag.join()
    want1, want2 = out1.into_array(), out2.into_array()
    ag._ffi.check(ag.lib.agh_graph_begin())
    try:
        with ag.branch():
            ag.gemm(1.0, t1a.t(), t1b, 0.0, out1)
        ag.join()
    finally:
        g = C.c_void_p()
        ag._ffi.check(ag.lib.agh_graph_end(C.byref(g)))
    try:
        for i in range(6):
            ag._ffi.check(ag.lib.agh_memset(out1._ptr(), 0xFF, 6 * 25 * 4))
            ag._ffi.check(ag.lib.agh_memset(out2._ptr(), 0xFF, 48 * 40 * 4))
            with ag.branch():                              # eager split-K product on the second stream, not joined
                ag.gemm(1.0, t2a.t(), t2b, 0.0, out2)
            ag._ffi.check(ag.lib.agh_graph_launch(g))      # the captured arm uses the same workspace
            ag.join()
            assert np.array_equal(out1.into_array(), want1), i
            assert np.array_equal(out2.into_array(), want2), i
        # a replay is refused inside a branch
        ag._ffi.check(ag.lib.agh_branch_begin())
        rc = ag.lib.agh_graph_launch(g)
        ag._ffi.check(ag.lib.agh_branch_end())
        ag.join()
        assert rc == -1
    finally:
        ag._ffi.check(ag.lib.agh_graph_destroy(g))


def test_calibration_launches(ag):
    """The measurement-only launches behind `bench.py --calib` (benchlib/, a library of its own): the copy and the read:write mix move exactly the bytes
    they claim (checked bit for bit on a small buffer), the MFMA loops run in both instruction shapes with and without
    direct loads, and arguments that would leave the buffers are refused before anything is launched."""
    import benchlib as cal
    check, lib = cal.check, cal.lib
    st = ag.lib.agh_stream()  # the product library's stream, as bench.py passes it
    rng = np.random.default_rng(5)
    n = 1 << 18  # 1 MiB of u32
    src = rng.integers(0, 2**32, 3 * n, dtype=np.uint32)
    tsrc = ag.Tensor.from_array(src.view(np.float32))
    tdst = ag.Tensor.zeros((n,), "f32")
    check(lib.calib_copy(st, tsrc._ptr(), tdst._ptr(), 4 * n, 64))
    assert np.array_equal(tdst.into_array().view(np.uint32), src[:n])
    sink = ag.Tensor.zeros((256,), "f32")
    check(lib.calib_read(st, tsrc._ptr(), sink._ptr(), 4 * n, 64))
    # every 16 bytes of dst: xor of the 16 bytes at the same offset of the streams, the first word also with the slot index
    for reads in (1, 2, 3):
        check(lib.calib_mix(st, tsrc._ptr(), tdst._ptr(), 4 * n, reads, 37))
        want = np.zeros(n, np.uint32)
        for r in range(reads):
            want ^= src[r * n:(r + 1) * n]
        want[0::4] ^= np.arange(n // 4, dtype=np.uint32)
        assert np.array_equal(tdst.into_array().view(np.uint32), want), reads
    for shape in (0, 1):
        for zero in (0, 1):
            check(lib.calib_mfma_bf16(st, sink._ptr(), zero, 4, 8, shape))
    for nld in (0, 2, 4, 8, 16):
        window = 4096 * nld * 2 if nld else 0
        check(lib.calib_mfma_dma(st, tsrc._ptr(), 12 * n, sink._ptr(), nld, window, 8, 4))
    ag._ffi.check(ag.lib.agh_sync())
    assert not np.any(sink.into_array())  # the sinks are never written
    # AGH_EINVAL is -1, AGH_ERANGE -4
    assert lib.calib_mfma_bf16(st, sink._ptr(), 0, 4, 8, 2) == -1
    assert lib.calib_mfma_dma(st, tsrc._ptr(), 12 * n, sink._ptr(), 3, 4096 * 3, 8, 4) == -1
    assert lib.calib_mfma_dma(st, tsrc._ptr(), 12 * n, sink._ptr(), 4, 4096 * 4 + 16, 8, 4) == -1
    assert lib.calib_mfma_dma(st, tsrc._ptr(), 65536, sink._ptr(), 4, 65536, 8, 4) == -4
    assert lib.calib_mix(st, tsrc._ptr(), tdst._ptr(), 4 * n + 4, 2, 8) == -1
    assert lib.calib_copy(st, tsrc._ptr(), tdst._ptr(), 4 * n, 0) == -1
