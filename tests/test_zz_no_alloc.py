"""agh_gemm_bf16_noalloc: the GEMM for callers that cannot allocate.  Same kernels as agh_gemm_bf16 with the
split-K partial sums in a fixed buffer inside the library image; checked bit for bit against agh_gemm_bf16
through the C ABI, on calls in a row that share that buffer (the second smaller than the first)."""
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


def run(ag, fn, a_t, b_t, out):
    (m, k), (_, n) = a_t.shape, b_t.shape
    ag._ffi.check(fn(m, k, n, 1.0, a_t._ptr(), a_t.offset, a_t.strides[0], a_t.strides[1], b_t._ptr(), b_t.offset,
                     b_t.strides[0], b_t.strides[1], 0.0, out._ptr(), out.offset, out.strides[0], out.strides[1]))


def cache_stats(ag):
    a, b, c = C.c_size_t(), C.c_size_t(), C.c_size_t()
    ag._ffi.check(ag.lib.agh_cache_stats(C.byref(a), C.byref(b), C.byref(c)))
    return a.value, b.value, c.value


def workspace_stats(ag):
    a, b = C.c_size_t(), C.c_size_t()
    ag._ffi.check(ag.lib.agh_workspace_stats(C.byref(a), C.byref(b)))
    return a.value, b.value


def test_noalloc_gemm_equals_gemm_on_calls_that_share_the_scratch(ag, monkeypatch):
    rng = np.random.default_rng(41)
    # k >> m*n: the split-K shapes of the LeNet5 weight gradients (256 and 25 k-groups), then smaller ones;
    # the last two take no split at all (no scratch)
    shapes = [(6, 57600, 25), (16, 6400, 150), (5, 1024, 7), (64, 16384, 64), (3, 4100, 5), (256, 128, 256), (33, 17, 65)]
    cases = []
    for m, k, n in shapes:
        dy = orc.f32_to_bf16(rng.normal(0, 1, (k, m)).astype(np.float32))
        cols = orc.f32_to_bf16(rng.normal(0, 1, (k, n)).astype(np.float32))
        ta, tb = ag.Tensor.from_array(dy).t(), ag.Tensor.from_array(cols)
        want_t = ag.Tensor.uninit((m, n), "bf16")
        run(ag, ag.lib.agh_gemm_bf16, ta, tb, want_t)
        cases.append((ta, tb, want_t.into_array(), dy, cols))
    outs = [ag.Tensor.zeros((m, n), "bf16") for m, _, n in shapes]
    # The library's own workspace, which the agh_gemm_bf16 calls above have grown, is handed back (unless a graph of
    # an earlier test still names it): a no-alloc call that fell back to it would have to grow it again.
    ag._ffi.check(ag.lib.agh_cache_release())
    before, ws_before = cache_stats(ag), workspace_stats(ag)
    # all calls queued back to back: each reuses the scratch the previous one has just read
    for (ta, tb, _, _, _), out in zip(cases, outs):
        run(ag, ag.lib.agh_gemm_bf16_noalloc, ta, tb, out)
    assert cache_stats(ag) == before, "no buffer was taken from or returned to the allocator"
    assert workspace_stats(ag) == ws_before, "the library's workspace (hipMalloc) was not touched"
    for (ta, tb, want, dy, cols), out, shape in zip(cases, outs, shapes):
        got = out.into_array()
        assert np.array_equal(got, want), shape
        # and the shared result is right: within one bf16 step of the f32-accumulated oracle product
        ref = orc.bf16_to_f32(orc.gemm_bf16_f32acc(np.ascontiguousarray(dy.T), cols)).astype(np.float64)
        g = orc.bf16_to_f32(got).astype(np.float64)
        scale = np.abs(orc.bf16_to_f32(dy)).astype(np.float64).T @ np.abs(orc.bf16_to_f32(cols)).astype(np.float64)
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref), 2.0**-126))) - 7)
        assert np.all(np.abs(g - ref) <= ulp + 1e-2 * np.abs(ref) + 8 * np.sqrt(shape[1]) * 2.0**-24 * scale), shape
    # first large, then small, then large again, with the results read in between
    for idx in (0, 2, 0, 4, 1):
        ta, tb, want, _, _ = cases[idx]
        out = outs[idx]
        ag._ffi.check(ag.lib.agh_memset(out._ptr(), 0xFF, want.size * 2))
        run(ag, ag.lib.agh_gemm_bf16_noalloc, ta, tb, out)
        assert np.array_equal(out.into_array(), want), idx

    # a plan that needs more scratch than the fixed buffer holds is refused and nothing is launched
    monkeypatch.setenv("AGH_GEMM_SPLITS", "64")
    big_a, big_b = ag.Tensor.uninit((1024, 32768), "bf16"), ag.Tensor.uninit((32768, 1024), "bf16")
    sentinel = np.full((1024, 1024), 0x3F80, dtype=np.uint16)
    big_c = ag.Tensor.from_array(sentinel)
    rc = ag.lib.agh_gemm_bf16_noalloc(1024, 32768, 1024, 1.0, big_a._ptr(), 0, 32768, 1, big_b._ptr(), 0, 1024, 1, 0.0,
                                      big_c._ptr(), 0, 1024, 1)
    assert rc == -4 and b"scratch" in ag.lib.agh_last_error_string()
    monkeypatch.delenv("AGH_GEMM_SPLITS")
    assert np.array_equal(big_c.into_array(), sentinel)
    # inside a branch a call that needs the scratch is refused (it would overlap the main stream's calls)
    ta, tb, want, _, _ = cases[0]
    with ag.branch():
        rc = ag.lib.agh_gemm_bf16_noalloc(6, 57600, 25, 1.0, ta._ptr(), 0, ta.strides[0], ta.strides[1], tb._ptr(), 0,
                                          tb.strides[0], tb.strides[1], 0.0, outs[0]._ptr(), 0, 25, 1)
    ag.join()
    assert rc == -1


def test_noalloc_gemm_under_graph_capture(ag):
    """The call this entry point exists for: captured without any eager run of that shape before (agh_gemm_bf16
    would have to grow its workspace and is refused there), replayed several times."""
    rng = np.random.default_rng(42)
    m, k, n = 10, 20480, 12
    dy = orc.f32_to_bf16(rng.normal(0, 1, (k, m)).astype(np.float32))
    cols = orc.f32_to_bf16(rng.normal(0, 1, (k, n)).astype(np.float32))
    ta, tb = ag.Tensor.from_array(dy).t(), ag.Tensor.from_array(cols)
    out = ag.Tensor.zeros((m, n), "bf16")
    ag._ffi.check(ag.lib.agh_sync())
    ag._ffi.check(ag.lib.agh_graph_begin())
    try:
        run(ag, ag.lib.agh_gemm_bf16_noalloc, ta, tb, out)
    finally:
        g = C.c_void_p()
        ag._ffi.check(ag.lib.agh_graph_end(C.byref(g)))
    want_t = ag.Tensor.uninit((m, n), "bf16")
    run(ag, ag.lib.agh_gemm_bf16, ta, tb, want_t)
    want = want_t.into_array()
    for i in range(3):
        ag._ffi.check(ag.lib.agh_memset(out._ptr(), 0xFF, m * n * 2))
        ag._ffi.check(ag.lib.agh_graph_launch(g))
        # eager work between the replays that uses the same scratch
        other = ag.Tensor.uninit((6, 25), "bf16")
        run(ag, ag.lib.agh_gemm_bf16_noalloc, ag.Tensor.from_array(dy[:, :6]).t(), ag.Tensor.from_array(cols[:, :1].repeat(25, 1)), other)
        assert np.array_equal(out.into_array(), want), i
    ag._ffi.check(ag.lib.agh_graph_destroy(g))
