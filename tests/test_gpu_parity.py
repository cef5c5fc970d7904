"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X.

Modelled on the reference's own device tests (tests/integration_tests.rs): the same
generators (ramps, cycles), the same parameter grids, host result vs device result.
Bars: im2col / col2im / pooling / relu bit-exact; f32 gemm within 1e-5*sqrt(K) relative;
bf16 gemm within 1 bf16 ulp + 1e-2 relative of an f32-accumulated reference.
"""
import ctypes as C  # noqa: F401

import numpy as np
import pytest

import oracle as orc
from refgrid import DOT_SIZES, POOL_SHAPES, cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ag():
    import autograph_amd as ag
    ag.Device(0)
    return ag


def to_dtype(x, dtype):
    return orc.f32_to_bf16(x) if dtype == "bf16" else np.ascontiguousarray(x, dtype=np.float32)


def as_f32(x):
    return orc.bf16_to_f32(x) if x.dtype == np.uint16 else x


# ------------------------------------------------------------------ tolerances ----
def assert_f32_gemm_close(got, a, b, want64=None, k=None):
    """|got - want| <= 1e-5*sqrt(K) * scale, with scale = max|want| (norm-wise) and, element-wise,
    sum_k |a||b| (the quantity a rounding-error bound of a dot product is relative to)."""
    k = k or a.shape[1]
    want64 = orc.gemm_f64acc(a, b) if want64 is None else want64
    absprod = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    err = np.abs(got.astype(np.float64) - want64)
    tol = 1e-5 * np.sqrt(max(k, 1))
    assert err.max() <= tol * max(np.abs(want64).max(), 1e-30), (err.max(), np.abs(want64).max())
    assert np.all(err <= tol * absprod + 1e-30)


def bf16_ulp(x):
    x = np.abs(x.astype(np.float64))
    e = np.floor(np.log2(np.maximum(x, 2.0**-126)))
    return 2.0 ** (e - 7)


def assert_bf16_gemm_close(got_bits, ref_bits, a_bits, b_bits):
    """got within 1 bf16 ulp + 1e-2 relative of the f32-accumulated reference.  Two f32
    accumulation orders can themselves differ by about sqrt(K)*2^-24*sum|a||b|, which matters
    only where the true result cancels to ~0; that floor is added so such entries do not
    decide the test."""
    got, ref = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(ref_bits).astype(np.float64)
    a, b = orc.bf16_to_f32(a_bits).astype(np.float64), orc.bf16_to_f32(b_bits).astype(np.float64)
    k = a.shape[1]
    floor = 8 * np.sqrt(k) * 2.0**-24 * (np.abs(a) @ np.abs(b))
    tol = bf16_ulp(ref) + 1e-2 * np.abs(ref) + floor
    bad = np.abs(got - ref) > tol
    assert not bad.any(), (np.argwhere(bad)[:5], got[bad][:5], ref[bad][:5])


# ------------------------------------------------------------------------ dot ----
def gen_array(shape):  # 1..9 cycling, integration_tests.rs:291-305
    return ((np.arange(shape[0] * shape[1]) % 9) + 1).astype(np.float32).reshape(shape)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("n", DOT_SIZES)
def test_tensor_dot_reference_cases(ag, dtype, n):
    """tensor_dot_<T>_m{n}_k{n}_n{n}_{nn,tn,nt,tt} (integration_tests.rs:272-376): exact data."""
    for ta in (False, True):
        for tb in (False, True):
            a1, a2 = to_dtype(gen_array((n, n)), dtype), to_dtype(gen_array((n, n)), dtype)
            t1, t2 = ag.Tensor.from_array(a1), ag.Tensor.from_array(a2)
            if ta:
                a1, t1 = a1.T, t1.t()
            if tb:
                a2, t2 = a2.T, t2.t()
            out = t1.dot(t2).into_array()
            want = orc.gemm_f64acc(a1, a2)
            if dtype == "f32":
                assert np.array_equal(out.astype(np.float64), want), (n, ta, tb)
            else:
                assert np.array_equal(out, orc.gemm_bf16_f32acc(a1, a2)), (n, ta, tb)
                assert np.all(np.abs(orc.bf16_to_f32(out) - want) <= n)  # the reference's own epsilon = k


SHAPES = [(1, 1, 1), (3, 7, 5), (33, 17, 65), (100, 77, 53), (64, 64, 64), (129, 256, 130), (256, 512, 384),
          (300, 1000, 20), (17, 2048, 9), (1000, 256, 128), (1000, 84, 10), (6400, 150, 16), (100, 25, 6),
          # k-tile counts 2, 3 and 5 with every dimension a multiple of 8: the direct-to-LDS bf16 kernel's
          # prologue, odd tail and two-share load order, for all four operand layouts
          (256, 128, 256), (136, 192, 264), (128, 320, 128)]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("mkn", SHAPES)
def test_dot_seeded_all_transposes(ag, dtype, mkn):
    m, k, n = mkn
    rng = np.random.default_rng(hash((m, k, n)) % 2**32)
    for ta in (False, True):
        for tb in (False, True):
            a = to_dtype(rng.uniform(-1, 1, (k, m) if ta else (m, k)), dtype)
            b = to_dtype(rng.uniform(-1, 1, (n, k) if tb else (k, n)), dtype)
            ta_, tb_ = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
            av, bv = (a.T if ta else a), (b.T if tb else b)
            tav, tbv = (ta_.t() if ta else ta_), (tb_.t() if tb else tb_)
            out = tav.dot(tbv).into_array()
            if dtype == "f32":
                assert_f32_gemm_close(out, av, bv)
            else:
                assert_bf16_gemm_close(out, orc.gemm_bf16_f32acc(av, bv), av, bv)


@pytest.fixture(params=["tiled", "default"])
def f32_small_kernel(request, monkeypatch):
    """f32 products of few tiles and short k have a kernel of their own, which by default takes most shapes of the
    view / stride / broadcast tests below: each of those runs once with it switched off (the tiled kernels and their
    loaders) and once as the library chooses."""
    if request.param == "tiled":
        monkeypatch.setenv("AGH_GEMM_SMALL", "0")
    return request.param


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gemm_strides_offsets_alpha_beta(ag, dtype, f32_small_kernel):
    """fn gemm with the full (offset, rs, cs) tuple for all three operands (linalg.rs:281-299):
    sub-views with offsets, negative strides, a column-major C, alpha and beta."""
    rng = np.random.default_rng(11)
    big_a = to_dtype(rng.uniform(-1, 1, (90, 150)), dtype)
    big_b = to_dtype(rng.uniform(-1, 1, (140, 120)), dtype)
    big_c = to_dtype(rng.uniform(-1, 1, (80, 100)), dtype)
    cases_ = [
        (big_a[3:67:2, 5:125:3], big_b[100:20:-2, 110:2:-3], big_c[2:34, 10:46]),         # 32x40 @ 40x36
        (big_a[10:74, 8:72], big_b[4:68, 16:80], big_c[0:64, 4:68]),                      # aligned 64^3 views
        (big_a[0:80, 0:96].T[0:96:1, 0:80][:, ::-1], big_b[0:80, 0:40], big_c.T[0:96, 0:40]),  # A transposed + reversed, C col-major
    ]
    for av, bv, cv in cases_:
        m, k = av.shape
        k2, n = bv.shape
        assert k == k2 and cv.shape == (m, n)
        for alpha, beta in [(1.0, 0.0), (0.5, 2.0), (-1.25, 1.0)]:
            ta, tb, tc = ag.Tensor.from_array(big_a), ag.Tensor.from_array(big_b), ag.Tensor.from_array(big_c)

            def view(t, base, v):
                _, off, rs, cs = orc._view(v)
                return ag.Tensor(t.buffer, v.shape, (rs, cs), off, t.dtype)

            tcv = view(tc, big_c, cv)
            ag.gemm(alpha, view(ta, big_a, av), view(tb, big_b, bv), beta, tcv)
            full = tc.into_array()
            got = np.lib.stride_tricks.as_strided(full.reshape(-1)[orc._view(cv)[1]:], shape=cv.shape,
                                                  strides=tuple(s * full.itemsize for s in orc._view(cv)[2:]))
            want = orc.gemm_f64acc(av, bv, alpha, beta, cv)
            # everything outside the C view is untouched
            mask = np.ones(big_c.size, bool)
            idx = (orc._view(cv)[1] + np.arange(m)[:, None] * orc._view(cv)[2] + np.arange(n)[None, :] * orc._view(cv)[3])
            mask[idx.reshape(-1)] = False
            assert np.array_equal(full.reshape(-1)[mask], big_c.reshape(-1)[mask])
            if dtype == "f32":
                absprod = abs(alpha) * (np.abs(av).astype(np.float64) @ np.abs(bv)) + abs(beta) * np.abs(cv)
                assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * absprod)
            else:
                gotf = orc.bf16_to_f32(np.ascontiguousarray(got)).astype(np.float64)
                absprod = abs(alpha) * (np.abs(as_f32(np.ascontiguousarray(av))).astype(np.float64) @ np.abs(as_f32(np.ascontiguousarray(bv)))) + abs(beta) * np.abs(as_f32(np.ascontiguousarray(cv)))
                assert np.all(np.abs(gotf - want) <= bf16_ulp(want) + 1e-2 * np.abs(want) + 1e-5 * absprod)


def test_gemm_random_views(ag):
    """150 seeded products over random views of larger buffers, as `fn gemm` receives them (linalg.rs:281-299): row and
    column steps of 1 to 3 elements, either sign, transposed or not, any offset, for A, B and C independently, both
    element types, alpha in {1, 0.5, -1.25} and beta in {0, 1, 2}.  The result against the f64 product under the
    element type's bound, and every element of C's buffer outside the view unchanged."""
    rng = np.random.default_rng(1618)

    def rand_view(big, r, c):
        rows, cols = big.shape
        for _ in range(100):
            tr = rng.random() < 0.5
            rr, cc = (c, r) if tr else (r, c)
            sr, sc = int(rng.integers(1, 4)), int(rng.integers(1, 4))
            if (rr - 1) * sr + 1 > rows or (cc - 1) * sc + 1 > cols:
                continue
            r0, c0 = int(rng.integers(0, rows - (rr - 1) * sr)), int(rng.integers(0, cols - (cc - 1) * sc))
            v = big[r0:r0 + (rr - 1) * sr + 1:sr, c0:c0 + (cc - 1) * sc + 1:sc]
            if rng.random() < 0.3:
                v = v[::-1]
            if rng.random() < 0.3:
                v = v[:, ::-1]
            return v.T if tr else v
        return None

    done = 0
    for _ in range(150):
        dtype = "bf16" if rng.random() < 0.5 else "f32"
        m, k, n = int(rng.integers(1, 150)), int(rng.integers(1, 200)), int(rng.integers(1, 150))
        if rng.random() < 0.4:
            m, k, n = 8 * max(1, m // 8), 8 * max(1, k // 8), 8 * max(1, n // 8)
        big_a = to_dtype(rng.uniform(-1, 1, (460, 620)), dtype)
        big_b = to_dtype(rng.uniform(-1, 1, (620, 460)), dtype)
        big_c = to_dtype(rng.uniform(-1, 1, (460, 460)), dtype)
        av, bv, cv = rand_view(big_a, m, k), rand_view(big_b, k, n), rand_view(big_c, m, n)
        if av is None or bv is None or cv is None:
            continue
        alpha, beta = float(rng.choice([1.0, 0.5, -1.25])), float(rng.choice([0.0, 0.0, 1.0, 2.0]))
        ta, tb, tc = ag.Tensor.from_array(big_a), ag.Tensor.from_array(big_b), ag.Tensor.from_array(big_c)

        def view(t, v):
            _, off, rs, cs = orc._view(v)
            return ag.Tensor(t.buffer, v.shape, (rs, cs), off, t.dtype)

        ag.gemm(alpha, view(ta, av), view(tb, bv), beta, view(tc, cv))
        full = tc.into_array().reshape(-1)
        _, off, rs, cs = orc._view(cv)
        idx = off + np.arange(m)[:, None] * rs + np.arange(n)[None, :] * cs
        mask = np.ones(big_c.size, bool)
        mask[idx.reshape(-1)] = False
        tag = (dtype, m, k, n, orc._view(av)[1:], orc._view(bv)[1:], orc._view(cv)[1:], alpha, beta)
        assert np.array_equal(full[mask], big_c.reshape(-1)[mask]), tag
        want = orc.gemm_f64acc(av, bv, alpha, beta, cv)
        f64 = lambda v: as_f32(np.ascontiguousarray(v)).astype(np.float64)  # noqa: E731
        absprod = abs(alpha) * (np.abs(f64(av)) @ np.abs(f64(bv))) + abs(beta) * np.abs(f64(cv))
        got = f64(full[idx])
        if dtype == "f32":
            assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * absprod + 1e-30), tag
        else:
            assert np.all(np.abs(got - want) <= bf16_ulp(want) + 1e-2 * np.abs(want) + 1e-5 * absprod), tag
        done += 1
    assert done >= 120


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gemm_zero_stride_operands(ag, dtype, f32_small_kernel):
    """Broadcast views as operands of `fn gemm` (strides are taken as they come, src/tensor/linalg.rs:285-299; ndarray's
    `broadcast` gives stride 0): every row of A the same vector, every column of B the same vector, an operand that is
    one scalar, k broadcast.  Against the f64 product of the materialised arrays, at sizes that take the small and the
    large tiles and split-K."""
    rng = np.random.default_rng(271)

    def check_case(av, bv, tag):
        m, k = av.shape
        n = bv.shape[1]
        ta_base, oa, rsa, csa = orc._view(av)
        tb_base, ob, rsb, csb = orc._view(bv)
        ta, tb = ag.Tensor.from_array(ta_base), ag.Tensor.from_array(tb_base)
        a = ag.Tensor(ta.buffer, (m, k), (rsa, csa), oa, dtype)
        b = ag.Tensor(tb.buffer, (k, n), (rsb, csb), ob, dtype)
        got = as_f32(a.dot(b).into_array()).astype(np.float64)
        am, bm = np.ascontiguousarray(av), np.ascontiguousarray(bv)
        want = orc.gemm_f64acc(am, bm)
        absprod = np.abs(as_f32(am)).astype(np.float64) @ np.abs(as_f32(bm)).astype(np.float64)
        if dtype == "f32":
            assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * absprod + 1e-30), tag
        else:
            assert np.all(np.abs(got - want) <= bf16_ulp(want) + 1e-2 * np.abs(want) + 1e-5 * absprod), tag

    for m, k, n in [(5, 7, 3), (64, 96, 80), (300, 1024, 260), (16, 8192, 24), (1024, 256, 1024)]:
        arow = to_dtype(rng.uniform(-1, 1, (1, k)), dtype)
        acol = to_dtype(rng.uniform(-1, 1, (m, 1)), dtype)
        a = to_dtype(rng.uniform(-1, 1, (m, k)), dtype)
        b = to_dtype(rng.uniform(-1, 1, (k, n)), dtype)
        bcol = to_dtype(rng.uniform(-1, 1, (k, 1)), dtype)
        brow = to_dtype(rng.uniform(-1, 1, (1, n)), dtype)
        one = to_dtype(rng.uniform(0.5, 1, (1, 1)), dtype)
        check_case(np.broadcast_to(arow, (m, k)), b, ("A rows stride 0", m, k, n))
        check_case(a, np.broadcast_to(bcol, (k, n)), ("B columns stride 0", m, k, n))
        check_case(np.broadcast_to(acol, (m, k)), b, ("A along k stride 0", m, k, n))
        check_case(a, np.broadcast_to(brow, (k, n)), ("B along k stride 0", m, k, n))
        check_case(np.broadcast_to(one, (m, k)), b, ("A scalar", m, k, n))
        check_case(a, np.broadcast_to(one, (k, n)), ("B scalar", m, k, n))
        check_case(np.broadcast_to(arow, (m, k)), np.broadcast_to(bcol, (k, n)), ("both", m, k, n))


def test_entry_points_from_two_threads(ag):
    """Tensors are `Send + Sync` in the reference (autograd.rs:97) and the C ABI says any thread may call any entry
    point: two host threads allocate, multiply and free concurrently (split-K shapes included, which share the
    library's workspace); every product must equal the one a single thread gets, bit for bit."""
    import threading
    rng = np.random.default_rng(272)
    shapes = [(128, 256, 64), (16, 8192, 24), (300, 200, 100), (6, 57600, 25), (1024, 512, 768), (64, 64, 64)]
    data = {}
    for dtype in ("f32", "bf16"):
        for s in shapes:
            data[(dtype, s)] = (to_dtype(rng.uniform(-1, 1, s[:2]), dtype), to_dtype(rng.uniform(-1, 1, s[1:]), dtype))
    serial = {key: ag.Tensor.from_array(a).dot(ag.Tensor.from_array(b)).into_array() for key, (a, b) in data.items()}
    errors = []

    def worker(order):
        try:
            for _ in range(6):
                for key in order:
                    a, b = data[key]
                    ta, tb = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
                    got = ta.dot(tb).into_array()
                    if not np.array_equal(got, serial[key]):
                        errors.append(key)
                    del ta, tb
        except Exception as e:  # noqa: BLE001
            errors.append(repr(e))

    keys = list(data)
    threads = [threading.Thread(target=worker, args=(keys,)), threading.Thread(target=worker, args=(keys[::-1],))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gemm_beta_zero_never_reads_c_and_k_zero(ag, dtype):
    rng = np.random.default_rng(12)
    a, b = to_dtype(rng.uniform(-1, 1, (40, 24)), dtype), to_dtype(rng.uniform(-1, 1, (24, 48)), dtype)
    poison = np.full((40, 48), np.nan, dtype=np.float32)
    c = ag.Tensor.from_array(to_dtype(poison, dtype))
    ag.gemm(1.0, ag.Tensor.from_array(a), ag.Tensor.from_array(b), 0.0, c)  # linalg.rs:215
    assert np.isfinite(as_f32(c.into_array())).all()
    # k == 0: C = beta*C
    c0 = to_dtype(rng.uniform(-1, 1, (8, 12)), dtype)
    c = ag.Tensor.from_array(c0)
    ag.gemm(1.0, ag.Tensor.uninit((8, 0), dtype), ag.Tensor.uninit((0, 12), dtype), 2.0, c)
    assert np.array_equal(as_f32(c.into_array()), as_f32(to_dtype(2.0 * as_f32(c0), dtype)))
    # empty outputs are a no-op
    assert ag.Tensor.uninit((0, 5), dtype).dot(ag.Tensor.uninit((5, 3), dtype)).shape == (0, 3)


def test_split_k_shapes(ag):
    """The weight-gradient shapes of the LeNet5 step (k >> m*n), which the reference splits along k
    (linalg.rs:306-340): dW1 = dY^T * im2col (6 x 57600 x 25), dW2 (16 x 6400 x 150)."""
    rng = np.random.default_rng(13)
    # the further shapes vary the number of k-groups (8 ... 256, ragged last group) and of threads that share an
    # output element in the reduction (1 ... 16), and cover an output of several tiles
    for (m, k, n) in [(6, 57600, 25), (16, 6400, 150), (64, 16384, 64), (5, 1000, 7), (3, 4100, 5), (20, 20001, 30),
                      (100, 9000, 100)]:
        for dtype in ("f32", "bf16"):
            dy = to_dtype(rng.normal(0, 1, (k, m)), dtype)
            cols = to_dtype(rng.normal(0, 1, (k, n)), dtype)
            out = ag.Tensor.from_array(dy).t().dot(ag.Tensor.from_array(cols)).into_array()
            again = ag.Tensor.from_array(dy).t().dot(ag.Tensor.from_array(cols)).into_array()
            assert np.array_equal(out, again), "the reduction order is fixed: same bits on every run"
            if dtype == "f32":
                assert_f32_gemm_close(out, dy.T, cols)
            else:
                assert_bf16_gemm_close(out, orc.gemm_bf16_f32acc(dy.T, cols), dy.T, cols)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dense_fused_bias_relu(ag, dtype):
    """Dense::forward + Relu (layer.rs:1134-1143, :1254-1267) in one launch equals dot -> add_assign(bias)
    -> relu done as three ops."""
    # exact data: small integers, so the f32 dot is exact and the fused result must be bit-identical
    x = ((np.arange(37 * 48) % 7) - 3).astype(np.float32).reshape(37, 48)
    w = ((np.arange(48 * 20) % 5) - 2).astype(np.float32).reshape(48, 20)
    bias = (np.arange(20) % 9 - 4).astype(np.float32) * 0.5
    xd, wd, bd = to_dtype(x, dtype), to_dtype(w, dtype), to_dtype(bias, dtype)
    got = ag.Tensor.from_array(xd).dot(ag.Tensor.from_array(wd), bias=ag.Tensor.from_array(bd), relu=True).into_array()
    dot = orc.gemm_bf16_f32acc(xd, wd) if dtype == "bf16" else orc.gemm_f64acc(xd, wd).astype(np.float32)
    want = orc.relu(orc.bias_add_rows(dot, bd))
    assert np.array_equal(got, want)
    # bias only (dense3 of LeNet5), relu only
    got = ag.Tensor.from_array(xd).dot(ag.Tensor.from_array(wd), bias=ag.Tensor.from_array(bd)).into_array()
    assert np.array_equal(got, orc.bias_add_rows(dot, bd))
    got = ag.Tensor.from_array(xd).dot(ag.Tensor.from_array(wd), relu=True).into_array()
    assert np.array_equal(got, orc.relu(dot))
    # seeded real data at a Dense-like shape, tolerance of the unfused sequence
    rng = np.random.default_rng(14)
    x = to_dtype(rng.normal(0, 0.02, (512, 256)), dtype)
    w = to_dtype(rng.normal(0, 0.02, (256, 384)), dtype)
    b = to_dtype(rng.normal(0, 0.02, (384,)), dtype)
    got = ag.Tensor.from_array(x).dot(ag.Tensor.from_array(w), bias=ag.Tensor.from_array(b), relu=True).into_array()
    if dtype == "f32":
        want = np.maximum(orc.gemm_f64acc(x, w) + b, 0)
        assert np.all(np.abs(got - want) <= 1e-5 * 16 * (np.abs(x).astype(np.float64) @ np.abs(w) + np.abs(b)))
    else:
        ref = orc.relu(orc.bias_add_rows(orc.gemm_bf16_f32acc(x, w), b))
        g, r = orc.bf16_to_f32(got).astype(np.float64), orc.bf16_to_f32(ref).astype(np.float64)
        scale = np.abs(orc.bf16_to_f32(x)).astype(np.float64) @ np.abs(orc.bf16_to_f32(w)) + np.abs(orc.bf16_to_f32(b))
        assert np.all(np.abs(g - r) <= 2 * bf16_ulp(np.maximum(np.abs(r), np.abs(g))) + 1e-2 * np.abs(r) + 1e-5 * scale)


def test_dot_error_behaviour(ag):
    a = ag.Tensor.from_array(np.zeros((4, 5), np.float32))
    with pytest.raises(ag.AghError, match="different types"):
        a.dot(ag.Tensor.from_array(np.zeros((5, 3), np.uint16)))
    with pytest.raises(ag.AghError, match="a_cols != b_rows"):
        a.dot(ag.Tensor.from_array(np.zeros((4, 3), np.float32)))
    with pytest.raises(ag.AghError, match="a_rows != c_rows"):
        ag.gemm(1.0, a, ag.Tensor.from_array(np.zeros((5, 3), np.float32)), 0.0, ag.Tensor.uninit((5, 3), "f32"))
    # the C ABI itself rejects bad arguments with a status
    assert ag.lib.agh_gemm_f32(-1, 1, 1, 1.0, None, 0, 1, 1, None, 0, 1, 1, 0.0, None, 0, 1, 1) == -1
    assert ag.lib.agh_gemm_f32(2, 2, 2, 1.0, None, 0, 1, 1, None, 0, 1, 1, 0.0, None, 0, 1, 1) == -3
    assert ag.lib.agh_im2col_conv2_f32(None, None, 1, 1, 2, 2, 3, 3, 0, 0, 1, 1, 1, 1) == -1  # filter > input
    assert ag.lib.agh_max_pool2_f32(None, None, 1, 2, 2, 3, 3, 1, 1) == -1


def test_bf16_output_rounding_matches_reference_rule(ag):
    """The device rounds f32 sums to bf16 with its conversion instruction; the reference's rule is the
    `half` crate's (round to nearest even, ties included).  A k = 2 product a*1 + b*1 with bf16 a, b
    builds f32 sums whose discarded half sits on, just above and just below a tie, over every binade."""
    rng = np.random.default_rng(26)
    hi = (rng.integers(0x0080, 0x7F00, 8192, dtype=np.uint32) | (rng.integers(0, 2, 8192, dtype=np.uint32) << 15)).astype(np.uint16)
    hf = orc.bf16_to_f32(hi)
    ulp = np.float32(2.0) ** (np.floor(np.log2(np.abs(hf))).astype(np.float32) - 7)
    rows = []
    for frac in (0.5, -0.5, 0.25, -0.25, 0.75, -0.75, 0.5 + 1 / 64, 0.5 - 1 / 64, -0.5 - 1 / 64, 1 / 128, 0.0):
        lo = orc.f32_to_bf16((ulp * np.float32(frac)).astype(np.float32))  # an exact power-of-two multiple: itself bf16
        rows.append(np.stack([hi, lo], axis=1))
    a = np.concatenate(rows)
    want = orc.f32_to_bf16(orc.bf16_to_f32(a[:, 0]) + orc.bf16_to_f32(a[:, 1]))
    ones = orc.f32_to_bf16(np.ones((2, 1), dtype=np.float32))
    got = ag.Tensor.from_array(a).dot(ag.Tensor.from_array(ones)).into_array()[:, 0]
    assert np.array_equal(got, want)
    # the large-tile kernels share the conversion: the same sums as columns of a 256 x 64 x 256 product
    n = 256
    big_a = np.zeros((n, 64), dtype=np.uint16)
    big_a[:, :2] = a[:n]
    big_b = np.zeros((64, n), dtype=np.uint16)
    big_b[:2, :] = ones[0, 0]
    got2 = ag.Tensor.from_array(big_a).dot(ag.Tensor.from_array(big_b)).into_array()
    assert np.array_equal(got2, np.repeat(want[:n, None], n, axis=1))


@pytest.mark.parametrize("dtype,shape", [("f32", (4096, 4096, 4096)), ("bf16", (8192, 8192, 8192)),
                                         ("f32", (8192, 8192, 8192))])
def test_gemm_full_size_sampled_entries_and_identity(ag, dtype, shape):
    """Benchmark-size GEMMs: the oracle cannot run 10^12 flops, so check (1) 4096 sampled output
    entries against f64 dot products of the corresponding row and column, for A*B, A^T*B and
    A*B^T, and (2) A*I == A bit for bit."""
    m, k, n = shape
    rng = np.random.default_rng(15)
    if dtype == "f32":
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    else:
        a = orc.f32_to_bf16(rng.normal(0, 0.02, (m, k)).astype(np.float32))
        b = orc.f32_to_bf16(rng.normal(0, 0.02, (k, n)).astype(np.float32))
    ta, tb = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
    ii, jj = rng.integers(0, m, 4096), rng.integers(0, n, 4096)
    af, bf = as_f32(a), as_f32(b)

    def check(out, av, bv):
        want = np.einsum("ik,ki->i", av[ii].astype(np.float64), bv[:, jj].astype(np.float64))
        scale = np.einsum("ik,ki->i", np.abs(av[ii]).astype(np.float64), np.abs(bv[:, jj]).astype(np.float64))
        got = as_f32(out[ii, jj]).astype(np.float64)
        if dtype == "f32":
            assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * scale)
            assert np.abs(got - want).max() <= 1e-5 * np.sqrt(k) * np.abs(want).max()
        else:
            assert np.all(np.abs(got - want) <= bf16_ulp(want) + 1e-2 * np.abs(want) + 8 * np.sqrt(k) * 2.0**-24 * scale)

    check(ta.dot(tb).into_array(), af, bf)
    if m == k == n:
        check(ta.t().dot(tb).into_array(), af.T, bf)
        check(ta.dot(tb.t()).into_array(), af, bf.T)
    eye = np.eye(k, n, dtype=np.float32)
    out = ta.dot(ag.Tensor.from_array(to_dtype(eye, dtype))).into_array()
    assert np.array_equal(out[:, :min(k, n)], a[:, :min(k, n)])


def test_gemm_f32_1024_cubed_all_layouts(ag):
    """The smallest standalone f32 GEMM of the benchmark list, M = N = K = 1024 (the one square shape on which
    the tile chooser leaves the 256x256 tile): every entry against the f64 product, all four operand layouts."""
    rng = np.random.default_rng(27)
    a = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    b = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    ta, tb = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
    assert_f32_gemm_close(ta.dot(tb).into_array(), a, b)
    assert_f32_gemm_close(ta.t().dot(tb).into_array(), a.T, b)
    assert_f32_gemm_close(ta.dot(tb.t()).into_array(), a, b.T)
    assert_f32_gemm_close(ta.t().dot(tb.t()).into_array(), a.T, b.T)
    eye = ag.Tensor.from_array(np.eye(1024, dtype=np.float32))
    assert np.array_equal(ta.dot(eye).into_array(), a)


def test_gemm_f32_direct_small_tiles(ag, monkeypatch):
    """The f32 kernel that loads 64 x 64 tiles straight into LDS (both operands vector-loadable, k a multiple of
    32): one to five k-tiles (its ring holds four), tile rows and columns cut off by the matrix edge, all four operand
    layouts, a batch, split-K partials, alpha / beta / bias / ReLU, integer data exactly, and the register-staged
    kernel on the same inputs."""
    rng = np.random.default_rng(31)
    for (m, k, n) in [(64, 32, 64), (64, 64, 64), (100, 96, 76), (132, 128, 200), (60, 160, 68), (256, 1024, 192)]:
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        at, bt = np.ascontiguousarray(a.T), np.ascontiguousarray(b.T)
        ta, tb, tat, tbt = (ag.Tensor.from_array(x) for x in (a, b, at, bt))
        outs = [ta.dot(tb).into_array(), tat.t().dot(tb).into_array(), ta.dot(tbt.t()).into_array(),
                tat.t().dot(tbt.t()).into_array()]
        for out in outs:
            assert_f32_gemm_close(out, a, b)
        monkeypatch.setenv("AGH_GEMM_DIRECT", "0")
        staged = ta.dot(tb).into_array()
        monkeypatch.delenv("AGH_GEMM_DIRECT")
        assert np.abs(outs[0] - staged).max() <= 1e-5 * np.sqrt(k) * np.abs(staged).max()
        # small integers: every product and partial sum is exact in f32, whatever the order
        ai = rng.integers(-8, 9, (m, k)).astype(np.float32)
        bi = rng.integers(-8, 9, (k, n)).astype(np.float32)
        assert np.array_equal(ag.Tensor.from_array(ai).dot(ag.Tensor.from_array(bi)).into_array(), ai @ bi)
    # alpha, beta, bias and ReLU through the shared epilogue
    m, k, n = 96, 64, 80
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    c = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    tc = ag.Tensor.from_array(c)
    ag.gemm(0.5, ag.Tensor.from_array(a), ag.Tensor.from_array(b), -2.0, tc)
    want = 0.5 * (a.astype(np.float64) @ b.astype(np.float64)) - 2.0 * c
    assert np.abs(tc.into_array() - want).max() <= 1e-5 * np.sqrt(k) * np.abs(want).max()
    bias = rng.uniform(-1, 1, n).astype(np.float32)
    got = ag.Dense(ag.Tensor.from_array(b), ag.Tensor.from_array(bias)).forward(ag.Tensor.from_array(a), relu=True).into_array()
    want = np.maximum(a.astype(np.float64) @ b.astype(np.float64) + bias, 0.0)
    assert np.abs(got - want).max() <= 1e-5 * np.sqrt(k) * max(np.abs(want).max(), 1.0)
    # split-K partials (forced) and the result's independence of the run
    monkeypatch.setenv("AGH_GEMM_CFG", "4")
    monkeypatch.setenv("AGH_GEMM_SPLITS", "3")
    a = rng.uniform(-1, 1, (70, 320)).astype(np.float32)
    b = rng.uniform(-1, 1, (320, 90)).astype(np.float32)
    out = ag.Tensor.from_array(a).dot(ag.Tensor.from_array(b)).into_array()
    again = ag.Tensor.from_array(a).dot(ag.Tensor.from_array(b)).into_array()
    monkeypatch.delenv("AGH_GEMM_CFG")
    monkeypatch.delenv("AGH_GEMM_SPLITS")
    assert np.array_equal(out, again)
    assert_f32_gemm_close(out, a, b)


def test_gemm_bf16_ring_of_four_stages(ag, monkeypatch):
    """The 128 x 128 bf16 direct-to-LDS kernel on four LDS stages, the form a launch of at most one workgroup per CU
    and 20 k-tiles or more takes: k-tile counts 20 to 23 (every length of the ring's tail) by the launch rule, counts
    1 to 5 forced (fewer tiles than stages: the requests beyond the last tile repeat it), tile rows and columns cut
    off by the matrix edge, all four operand layouts, bias and ReLU.  Against the oracle, and bit for bit against the
    same kernel on two stages (the order of every sum is the same)."""
    rng = np.random.default_rng(77)
    monkeypatch.setenv("AGH_GEMM_CFG", "3")
    cases = [(200, 1280, 264, None), (128, 1344, 128, None), (256, 1408, 136, None), (136, 1472, 384, None),
             (128, 64, 128, "4"), (136, 128, 200, "4"), (128, 192, 128, "4"), (264, 256, 128, "4"), (128, 320, 136, "4")]
    for (m, k, n, force) in cases:
        for ta in (False, True):
            for tb in (False, True):
                a = to_dtype(rng.uniform(-1, 1, (k, m) if ta else (m, k)), "bf16")
                b = to_dtype(rng.uniform(-1, 1, (n, k) if tb else (k, n)), "bf16")
                ta_, tb_ = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
                av, bv = (a.T if ta else a), (b.T if tb else b)
                tav, tbv = (ta_.t() if ta else ta_), (tb_.t() if tb else tb_)
                if force:
                    monkeypatch.setenv("AGH_GEMM_RING", force)
                out = tav.dot(tbv).into_array()
                monkeypatch.setenv("AGH_GEMM_RING", "2")
                two = tav.dot(tbv).into_array()
                monkeypatch.delenv("AGH_GEMM_RING")
                assert_bf16_gemm_close(out, orc.gemm_bf16_f32acc(av, bv), av, bv)
                assert np.array_equal(out, two), (m, k, n, ta, tb)
    # a batch of three products with a shared B in one launch (agh_gemm_bf16_batched), 22 k-tiles
    nb, m, k, n = 3, 136, 1408, 128
    a = to_dtype(rng.uniform(-1, 1, (nb, m, k)), "bf16")
    b = to_dtype(rng.uniform(-1, 1, (k, n)), "bf16")
    A, B, Cb = ag.Tensor.from_array(a), ag.Tensor.from_array(b), ag.Tensor.zeros((nb, m, n), "bf16")
    ag._ffi.check(ag.lib.agh_gemm_bf16_batched(nb, m, k, n, 1.0, A._ptr(), 0, k, 1, m * k, B._ptr(), 0, n, 1, 0, 0.0,
                                               Cb._ptr(), 0, n, 1, m * n, None, 0, 0, 0))
    got = Cb.into_array()
    for i in range(nb):
        assert_bf16_gemm_close(got[i], orc.gemm_bf16_f32acc(a[i], b), a[i], b)
        assert np.array_equal(got[i], ag.Tensor.from_array(a[i]).dot(B).into_array())
    m, k, n = 192, 1536, 256
    a = to_dtype(rng.uniform(-1, 1, (m, k)), "bf16")
    w = to_dtype(rng.uniform(-1, 1, (k, n)), "bf16")
    bias = to_dtype(rng.uniform(-1, 1, n), "bf16")
    layer = ag.Dense(ag.Tensor.from_array(w), ag.Tensor.from_array(bias))
    got = layer.forward(ag.Tensor.from_array(a), relu=True).into_array()
    monkeypatch.setenv("AGH_GEMM_RING", "2")
    two = layer.forward(ag.Tensor.from_array(a), relu=True).into_array()
    monkeypatch.delenv("AGH_GEMM_RING")
    assert np.array_equal(got, two)
    dot = orc.bf16_to_f32(orc.gemm_bf16_f32acc(a, w))
    want = np.maximum(orc.bf16_to_f32(orc.f32_to_bf16(dot + orc.bf16_to_f32(bias))), 0.0)
    gotf = orc.bf16_to_f32(got).astype(np.float64)
    assert np.all(np.abs(gotf - want) <= 2 * bf16_ulp(want) + 1e-2 * np.abs(want) + 0.05)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_gemm_split_k_second_pass_four_outputs_a_thread(ag, monkeypatch, dtype):
    """Split-K with fewer than 16 splits into a C whose rows are contiguous and whole groups of four: the second pass
    that reads the partials 16 bytes at a time.  2 to 15 forced splits (the last one shorter than the others), alpha
    and beta, a column bias and a row bias with ReLU, against the oracle; and against the one-output-a-thread pass,
    which a C of 6 more columns takes, on the shared columns of integer data (exact in any order)."""
    rng = np.random.default_rng(91)
    m, k, n = 96, 1920, 136
    a = to_dtype(rng.uniform(-1, 1, (m, k)), dtype)
    b = to_dtype(rng.uniform(-1, 1, (k, n)), dtype)
    c0 = to_dtype(rng.uniform(-1, 1, (m, n)), dtype)
    A, B = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
    for splits in (2, 3, 4, 5, 7, 15):
        monkeypatch.setenv("AGH_GEMM_SPLITS", str(splits))
        for alpha, beta in ((1.0, 0.0), (0.5, -1.0)):
            C = ag.Tensor.from_array(c0)
            ag.gemm(alpha, A, B, beta, C)
            got = C.into_array()
            if dtype == "f32":
                want = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0
                assert np.abs(got - want).max() <= 1e-5 * np.sqrt(k) * np.abs(want).max()
            else:
                want = orc.bf16_to_f32(orc.gemm_bf16_f32acc(a, b, alpha, beta, c0)).astype(np.float64)
                gf = orc.bf16_to_f32(got).astype(np.float64)
                assert np.all(np.abs(gf - want) <= bf16_ulp(want) + 1e-2 * np.abs(want) + 1e-3)
        bias = to_dtype(rng.uniform(-1, 1, n), dtype)
        got = ag.Dense(B, ag.Tensor.from_array(bias)).forward(A, relu=True).into_array()
        monkeypatch.delenv("AGH_GEMM_SPLITS")
        one = ag.Dense(B, ag.Tensor.from_array(bias)).forward(A, relu=True).into_array()
        gf, of = as_f32(got).astype(np.float64), as_f32(one).astype(np.float64)
        tol = 1e-5 * np.sqrt(k) * max(np.abs(of).max(), 1.0) if dtype == "f32" else bf16_ulp(of) + 1e-2 * np.abs(of) + 1e-3
        assert np.all(np.abs(gf - of) <= tol)
    ai = to_dtype(rng.integers(-4, 5, (m, k)).astype(np.float32), dtype)
    bi = to_dtype(rng.integers(-4, 5, (k, n + 6)).astype(np.float32), dtype)
    monkeypatch.setenv("AGH_GEMM_SPLITS", "6")
    wide = ag.Tensor.from_array(ai).dot(ag.Tensor.from_array(bi)).into_array()
    narrow = ag.Tensor.from_array(ai).dot(ag.Tensor.from_array(np.ascontiguousarray(bi[:, :n]))).into_array()
    monkeypatch.delenv("AGH_GEMM_SPLITS")
    assert np.array_equal(wide[:, :n], narrow)
    if dtype == "f32":
        assert np.array_equal(narrow, ai @ bi[:, :n])


def test_gemm_bf16_last_k_tile_shorter_than_64(ag, monkeypatch):
    """The bf16 direct-to-LDS kernels with k not a multiple of their 64-deep k-tile: the last tile is loaded with zeros
    behind k = K (both operands), outside the pipeline.  k below one tile, one tile and a rest, a rest of at most and of
    more than 32 (one or both halves of the tile multiplied), 20 tiles and a rest (the four-stage ring), all four
    layouts, every tile forced; odd k (operands stored k-major, the only vector-loadable form then); forced split-K,
    whose last split alone has the shorter tile; the register-staged kernel on the same inputs."""
    rng = np.random.default_rng(99)
    cases = [(128, k, 128) for k in (8, 24, 40, 56, 72, 104, 200, 1000, 1288)] + [(264, 120, 136), (136, 1096, 264)]
    for (m, k, n) in cases:
        for ta in (False, True):
            for tb in (False, True):
                a = to_dtype(rng.uniform(-1, 1, (k, m) if ta else (m, k)), "bf16")
                b = to_dtype(rng.uniform(-1, 1, (n, k) if tb else (k, n)), "bf16")
                A, B = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
                av, bv = (a.T if ta else a), (b.T if tb else b)
                want = orc.gemm_bf16_f32acc(av, bv)
                outs = []
                for cfg in (None, "0", "1", "2", "3"):
                    if cfg is None:
                        monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
                    else:
                        monkeypatch.setenv("AGH_GEMM_CFG", cfg)
                    out = (A.t() if ta else A).dot(B.t() if tb else B).into_array()
                    assert_bf16_gemm_close(out, want, av, bv)
                    outs.append(out)
                monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
                for other in outs[2:]:
                    assert np.array_equal(outs[1], other), (m, k, n, ta, tb)  # one f32 sum in k order, rounded once
    for (m, k, n) in ((96, 77, 200), (96, 3, 200), (104, 1001, 96)):
        a = to_dtype(rng.uniform(-1, 1, (k, m)), "bf16")
        b = to_dtype(rng.uniform(-1, 1, (k, n)), "bf16")
        out = ag.Tensor.from_array(a).t().dot(ag.Tensor.from_array(b)).into_array()
        assert_bf16_gemm_close(out, orc.gemm_bf16_f32acc(a.T, b), a.T, b)
        monkeypatch.setenv("AGH_GEMM_DIRECT", "0")
        staged = ag.Tensor.from_array(a).t().dot(ag.Tensor.from_array(b)).into_array()
        monkeypatch.delenv("AGH_GEMM_DIRECT")
        assert_bf16_gemm_close(staged, orc.gemm_bf16_f32acc(a.T, b), a.T, b)
    m, k, n = 136, 1000, 128
    a = to_dtype(rng.uniform(-1, 1, (m, k)), "bf16")
    b = to_dtype(rng.uniform(-1, 1, (k, n)), "bf16")
    for splits in ("3", "16"):
        monkeypatch.setenv("AGH_GEMM_SPLITS", splits)
        out = ag.Tensor.from_array(a).dot(ag.Tensor.from_array(b)).into_array()
        assert_bf16_gemm_close(out, orc.gemm_bf16_f32acc(a, b), a, b)
    monkeypatch.delenv("AGH_GEMM_SPLITS")
    # integer data: exact whatever the order, so any element dropped or counted twice at the tile's edge shows
    ai = to_dtype(rng.integers(-3, 4, (136, 1016)).astype(np.float32), "bf16")
    bi = to_dtype(rng.integers(-3, 4, (1016, 264)).astype(np.float32), "bf16")
    got = orc.bf16_to_f32(ag.Tensor.from_array(ai).dot(ag.Tensor.from_array(bi)).into_array())
    exact = orc.bf16_to_f32(ai).astype(np.float64) @ orc.bf16_to_f32(bi).astype(np.float64)
    assert np.array_equal(got, orc.bf16_to_f32(orc.f32_to_bf16(exact.astype(np.float32))))


def test_gemm_f32_last_k_tile_shorter_than_32(ag, monkeypatch):
    """The f32 direct-to-LDS kernels with k not a multiple of their 32-deep k-tile: the last tile is loaded with zeros
    behind k = K and multiplied after the pipelined loop.  k below one tile, whole tiles and a rest, all four layouts,
    the 256 x 256, 128 x 128 and 64 x 64 tiles forced, eight waves sharing every k-tile forced on and off, odd k
    (operands stored k-major), forced split-K (the last split alone has the shorter tile), integer data exactly."""
    rng = np.random.default_rng(98)
    cases = [(128, k, 128) for k in (4, 12, 28, 36, 60, 100, 1000)] + [(200, 44, 72), (72, 1028, 264)]
    for (m, k, n) in cases:
        for ta in (False, True):
            for tb in (False, True):
                a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
                b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
                A, B = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
                av, bv = (a.T if ta else a), (b.T if tb else b)
                for cfg in (None, "0", "3", "4"):
                    for ks in (None, "0", "1"):
                        if cfg is None and ks is not None:
                            continue
                        if cfg is None:
                            monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
                        else:
                            monkeypatch.setenv("AGH_GEMM_CFG", cfg)
                        if ks is None:
                            monkeypatch.delenv("AGH_GEMM_KSPLIT", raising=False)
                        else:
                            monkeypatch.setenv("AGH_GEMM_KSPLIT", ks)
                        out = (A.t() if ta else A).dot(B.t() if tb else B).into_array()
                        assert_f32_gemm_close(out, av, bv)
    monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
    monkeypatch.delenv("AGH_GEMM_KSPLIT", raising=False)
    for (m, k, n) in ((96, 77, 200), (96, 3, 200), (104, 1001, 96)):
        a = rng.uniform(-1, 1, (k, m)).astype(np.float32)
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        assert_f32_gemm_close(ag.Tensor.from_array(a).t().dot(ag.Tensor.from_array(b)).into_array(), a.T, b)
    a = rng.uniform(-1, 1, (136, 1000)).astype(np.float32)
    b = rng.uniform(-1, 1, (1000, 128)).astype(np.float32)
    for splits in ("3", "16"):
        monkeypatch.setenv("AGH_GEMM_SPLITS", splits)
        assert_f32_gemm_close(ag.Tensor.from_array(a).dot(ag.Tensor.from_array(b)).into_array(), a, b)
    monkeypatch.delenv("AGH_GEMM_SPLITS")
    ai = rng.integers(-8, 9, (136, 1012)).astype(np.float32)
    bi = rng.integers(-8, 9, (1012, 264)).astype(np.float32)
    assert np.array_equal(ag.Tensor.from_array(ai).dot(ag.Tensor.from_array(bi)).into_array(), ai @ bi)


def test_gemm_f32_seeded_shapes_in_every_tile_configuration(ag, monkeypatch):
    """150 seeded f32 products with k a multiple of 32 (so that the direct-to-LDS kernels apply wherever the operands
    are vector-loadable), odd and even m and n, all four layouts, alpha and beta, each in the chooser's tile
    configuration and forced into the 256 x 256, 128 x 128 and 64 x 64 ones (a forced configuration that has no
    kernel for the operands' loaders is refused, not miscomputed)."""
    rng = np.random.default_rng(123)
    ran = {None: 0, "0": 0, "3": 0, "4": 0}
    for _ in range(150):
        m, n, k = int(rng.integers(1, 400)), int(rng.integers(1, 400)), 32 * int(rng.integers(1, 12))
        if rng.random() < 0.5:
            m = 4 * max(1, m // 4)
        if rng.random() < 0.5:
            n = 4 * max(1, n // 4)
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
        c0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
        alpha, beta = float(rng.choice([1.0, 0.5])), float(rng.choice([0.0, 0.0, 1.0, -0.5]))
        A, B = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
        av, bv = (a.T if ta else a), (b.T if tb else b)
        want = alpha * (av.astype(np.float64) @ bv.astype(np.float64)) + beta * c0
        tol = 1e-5 * np.sqrt(k) * max(np.abs(want).max(), 1e-3) + 1e-6
        for cfg in ran:
            if cfg is None:
                monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
            else:
                monkeypatch.setenv("AGH_GEMM_CFG", cfg)
            C = ag.Tensor.from_array(c0)
            try:
                ag.gemm(alpha, A.t() if ta else A, B.t() if tb else B, beta, C)
            except ag.AghError as e:
                assert cfg is not None and e.code == -4
                continue
            ran[cfg] += 1
            assert np.abs(C.into_array() - want).max() <= tol, (m, k, n, ta, tb, alpha, beta, cfg)
    monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
    assert ran[None] == 150 and min(ran.values()) >= 30, ran


def test_gemm_f32_few_tiles_short_k_kernel(ag, monkeypatch):
    """Products of a few hundred 16 x 16 tiles with k <= 512 and both operands k-contiguous go to a kernel of their own
    (one tile per workgroup, k split over its four waves).  AGH_GEMM_SMALL=1 sends every eligible product there,
    =0 none: both against the f64 product, bias / ReLU epilogues bit for bit against the separate ops on the plain
    result, exact on integers.  Shapes: the LeNet5 Dense layers at batch 1000 and 100, k not a multiple of 16 or 64,
    k = 4, n = 10 (no 16-byte stores), one row, beta and alpha."""
    rng = np.random.default_rng(321)
    shapes = [(1000, 256, 128), (1000, 128, 84), (1000, 84, 10), (100, 256, 128), (7, 4, 3), (1, 40, 50), (33, 20, 1),
              (130, 500, 36), (16, 16, 16), (250, 1028, 20)]
    for (m, k, n) in shapes:
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        w = rng.uniform(-1, 1, (n, k)).astype(np.float32)     # Dense weight [out, in]: the product is a . w^T
        bias = rng.uniform(-1, 1, n).astype(np.float32)
        c0 = rng.uniform(-1, 1, (m, n)).astype(np.float32)
        A, W, Bv = ag.Tensor.from_array(a), ag.Tensor.from_array(w), ag.Tensor.from_array(bias)
        got = {}
        for small in ("1", "0"):
            monkeypatch.setenv("AGH_GEMM_SMALL", small)
            for alpha, beta in ((1.0, 0.0), (0.5, -0.5)):
                C = ag.Tensor.from_array(c0)
                ag.gemm(alpha, A, W.t(), beta, C)
                want = alpha * (a.astype(np.float64) @ w.T.astype(np.float64)) + beta * c0
                tol = 1e-5 * np.sqrt(k) * max(np.abs(want).max(), 1e-3) + 1e-6
                assert np.abs(C.into_array() - want).max() <= tol, (m, k, n, small, alpha, beta)
                got[small, alpha] = C.into_array()
            plain = got[small, 1.0]
            fused = ag.Tensor.from_array(a).dot(W.t(), bias=Bv, relu=True).into_array()
            assert np.array_equal(fused, orc.relu(orc.bias_add_rows(plain, bias))), (m, k, n, small)
            # c = a^T-free column-major output: p runs along m, the bias along q
            Ct = ag.Tensor.uninit((n, m), "f32")
            ag.gemm(1.0, A, W.t(), 0.0, Ct.t(), bias=Bv, relu=False)
            assert np.array_equal(Ct.into_array().T, orc.bias_add_rows(plain, bias)), (m, k, n, small)
        assert np.abs(got["1", 1.0] - got["0", 1.0]).max() <= 2e-5 * np.sqrt(k), (m, k, n)
        ai = rng.integers(-8, 9, (m, k)).astype(np.float32)
        wi = rng.integers(-8, 9, (n, k)).astype(np.float32)
        monkeypatch.setenv("AGH_GEMM_SMALL", "1")
        assert np.array_equal(ag.Tensor.from_array(ai).dot(ag.Tensor.from_array(wi).t()).into_array(), ai @ wi.T)
    monkeypatch.delenv("AGH_GEMM_SMALL")


def test_gemm_bf16_seeded_shapes_in_every_tile_configuration(ag, monkeypatch):
    """120 seeded bf16 products with k a multiple of 64 (so that the direct-to-LDS kernels apply wherever the operands
    are vector-loadable), m and n mostly multiples of 8, all four layouts, beta 0 or 1, each in the chooser's tile
    configuration and forced into the 256 x 256, 128 x 256, 256 x 128, 128 x 128 and 64 x 64 ones (two, three, three, two or
    four and four LDS stages; a forced large configuration that has no kernel for the operands' loaders is refused, not
    miscomputed; the 64 x 64 one then takes the register-staged kernel).  The forced configurations must agree bit for
    bit wherever they take the direct-to-LDS kernel: one f32 sum per output in k order, rounded once."""
    rng = np.random.default_rng(321)
    ran = {None: 0, "0": 0, "1": 0, "2": 0, "3": 0, "4": 0}
    for _ in range(120):
        m, n, k = int(rng.integers(1, 700)), int(rng.integers(1, 700)), 64 * int(rng.integers(1, 14))
        if rng.random() < 0.8:
            m = 8 * max(1, m // 8)
        if rng.random() < 0.8:
            n = 8 * max(1, n // 8)
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        a = to_dtype(rng.uniform(-1, 1, (k, m) if ta else (m, k)), "bf16")
        b = to_dtype(rng.uniform(-1, 1, (n, k) if tb else (k, n)), "bf16")
        c0 = to_dtype(rng.uniform(-1, 1, (m, n)), "bf16")
        beta = float(rng.choice([0.0, 0.0, 1.0]))
        A, B = ag.Tensor.from_array(a), ag.Tensor.from_array(b)
        av, bv = (a.T if ta else a), (b.T if tb else b)
        want = orc.gemm_bf16_f32acc(av, bv, 1.0, beta, c0)
        forced = []
        for cfg in ran:
            if cfg is None:
                monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
            else:
                monkeypatch.setenv("AGH_GEMM_CFG", cfg)
            C = ag.Tensor.from_array(c0)
            try:
                ag.gemm(1.0, A.t() if ta else A, B.t() if tb else B, beta, C)
            except ag.AghError as e:
                assert cfg is not None and e.code == -4
                continue
            ran[cfg] += 1
            got = C.into_array()
            if beta == 0.0:
                assert_bf16_gemm_close(got, want, av, bv)
            else:
                gf, wf = orc.bf16_to_f32(got).astype(np.float64), orc.bf16_to_f32(want).astype(np.float64)
                assert np.all(np.abs(gf - wf) <= bf16_ulp(wf) + 1e-2 * np.abs(wf) + 1e-3), (m, k, n, ta, tb, cfg)
            # (the 64 x 64 configuration takes the direct-to-LDS kernel exactly when the larger ones are not refused)
            if cfg is not None and (cfg != "4" or forced):
                forced.append(got)
        for other in forced[1:]:
            assert np.array_equal(forced[0], other), (m, k, n, ta, tb, beta)
    monkeypatch.delenv("AGH_GEMM_CFG", raising=False)
    assert ran[None] == 120 and min(ran.values()) >= 40, ran


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_dense_full_size_bias_relu(ag, dtype):
    """The Dense-shaped GEMM of the benchmark list at full size: M = 16384 (batch), K = 4096, N = 4096 with the
    fused bias + ReLU epilogue (layer.rs:1134-1143, :1254-1267).  4096 sampled entries against f64 dot + bias
    + relu for the fused launch and for its bias-only and relu-only forms; the three are consistent with the
    plain product bit for bit (epilogue = the separate ops on the rounded dot); A*I through the same epilogue
    is relu(a + bias) exactly."""
    m, k, n = 16384, 4096, 4096
    rng = np.random.default_rng(28)
    a = to_dtype(rng.normal(0, 0.02, (m, k)).astype(np.float32), dtype)
    b = to_dtype(rng.normal(0, 0.02, (k, n)).astype(np.float32), dtype)
    bias = to_dtype(rng.normal(0, 0.02, (n,)).astype(np.float32), dtype)
    ta, tb, tbias = ag.Tensor.from_array(a), ag.Tensor.from_array(b), ag.Tensor.from_array(bias)
    ii, jj = rng.integers(0, m, 4096), rng.integers(0, n, 4096)
    ii[:8], jj[:8] = [0, 0, m - 1, m - 1, 255, 256, 8191, 8192], [0, n - 1, 0, n - 1, 255, 256, 2047, 2048]
    af, bf, biasf = as_f32(a), as_f32(b), as_f32(bias).astype(np.float64)
    dot64 = np.einsum("ik,ki->i", af[ii].astype(np.float64), bf[:, jj].astype(np.float64))
    scale = np.einsum("ik,ki->i", np.abs(af[ii]).astype(np.float64), np.abs(bf[:, jj]).astype(np.float64))

    def close(got, want):
        got = as_f32(np.ascontiguousarray(got)).astype(np.float64)
        if dtype == "f32":
            assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * (scale + np.abs(biasf[jj])))
        else:  # two roundings, T(dot) then T(bias + .): a bf16 step of the dot and one of the result
            assert np.all(np.abs(got - want) <= bf16_ulp(dot64) + bf16_ulp(want) + 1e-2 * np.abs(want) +
                          8 * np.sqrt(k) * 2.0**-24 * scale)

    plain = ta.dot(tb).into_array()
    close(plain[ii, jj], dot64)
    fused = ta.dot(tb, bias=tbias, relu=True).into_array()
    close(fused[ii, jj], np.maximum(dot64 + biasf[jj], 0))
    assert (fused.view(np.uint32 if dtype == "f32" else np.uint16) == 0).mean() > 0.3  # the relu did cut
    # the epilogue is the separate ops applied to the rounded product: bit for bit on whole row blocks
    rows = np.r_[0:256, 8064:8320, m - 256:m]
    assert np.array_equal(fused[rows], orc.relu(orc.bias_add_rows(np.ascontiguousarray(plain[rows]), bias)))
    only_bias = ta.dot(tb, bias=tbias).into_array()
    assert np.array_equal(only_bias[rows], orc.bias_add_rows(np.ascontiguousarray(plain[rows]), bias))
    close(only_bias[ii, jj], dot64 + biasf[jj])
    del only_bias
    only_relu = ta.dot(tb, relu=True).into_array()
    assert np.array_equal(only_relu[rows], orc.relu(np.ascontiguousarray(plain[rows])))
    del only_relu, plain, fused
    # A * I + bias, relu: exact products, so the result is relu(T(a + bias)) for every entry
    eye = ag.Tensor.from_array(to_dtype(np.eye(k, n, dtype=np.float32), dtype))
    out = ta.dot(eye, bias=tbias, relu=True).into_array()
    assert np.array_equal(out, orc.relu(orc.bias_add_rows(a, bias)))


# ------------------------------------------------------------- im2col / col2im ----
# col2im has a streaming (ring) form for large patch matrices and a gathering form for small ones; the
# library picks by size, AGH_COL2IM_RING forces either, and the small reference cases must pass on both
@pytest.mark.parametrize("ring", ["1", "0"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_im2col_col2im_reference_grid(ag, dtype, ring, monkeypatch):
    """im2col_conv2_<T>_<opts> and col2im_conv2_<T>_<opts> (integration_tests.rs:946-981, :1499-1552):
    ramp inputs over the whole filter/padding/stride/dilation grid; host vs device, bit for bit."""
    monkeypatch.setenv("AGH_COL2IM_RING", ring)
    count = 0
    for bs, c, ih, iw, f, p, s, d in cases():
        x = to_dtype(np.arange(1, bs * c * ih * iw + 1, dtype=np.float32).reshape(bs, c, ih, iw), dtype)
        opts = ag.Im2ColConv2Options(filter=f, padding=p, stride=s, dilation=d)
        y = ag.Tensor.from_array(x).im2col_conv2(opts).into_array()
        want = orc.im2col_conv2(x, f, p, s, d)
        assert np.array_equal(y, want), ("im2col", bs, c, ih, iw, f, p, s, d)
        oh, ow = opts.output_shape((ih, iw))
        dy = to_dtype(np.arange(1, want.size + 1, dtype=np.float32).reshape(want.shape), dtype)
        copts = ag.Col2ImConv2Options(shape=(oh, ow), filter=f, padding=p, stride=s, dilation=d)
        dx = ag.Tensor.from_array(dy).col2im_conv2(copts).into_array()
        assert np.array_equal(dx, orc.col2im_conv2(dy, (oh, ow), f, p, s, d)), ("col2im", bs, c, ih, iw, f, p, s, d)
        count += 1
    assert count > 1000


IM2COL_SEEDED = [
    # bs, c, ih, iw, filter, padding, stride, dilation
    (4, 16, 28, 28, (3, 3), (1, 1), (1, 1), (1, 1)),      # vector-store path, all channels in one workgroup
    (100, 1, 28, 28, (5, 5), (0, 0), (1, 1), (1, 1)),     # LeNet5 conv1 (25-wide rows, scalar stores)
    (100, 6, 12, 12, (5, 5), (0, 0), (1, 1), (1, 1)),     # LeNet5 conv2
    (2, 512, 14, 14, (3, 3), (1, 1), (1, 1), (1, 1)),     # channels split over several workgroups
    (3, 8, 17, 23, (3, 5), (2, 1), (2, 3), (2, 1)),       # everything non-default at once
    (1, 4, 6, 9000, (1, 3), (0, 1), (1, 1), (1, 1)),      # rows too wide for LDS: direct kernel
    (2, 24, 9, 9, (2, 2), (0, 0), (2, 2), (1, 1)),
]


@pytest.mark.parametrize("ring", ["1", "0", None])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", IM2COL_SEEDED)
def test_im2col_col2im_seeded(ag, dtype, case, ring, monkeypatch):
    if ring is None:
        monkeypatch.delenv("AGH_COL2IM_RING", raising=False)
    else:
        monkeypatch.setenv("AGH_COL2IM_RING", ring)
    bs, c, ih, iw, f, p, s, d = case
    rng = np.random.default_rng(16)
    x = to_dtype(rng.standard_normal((bs, c, ih, iw)), dtype)
    opts = ag.Im2ColConv2Options(filter=f, padding=p, stride=s, dilation=d)
    y = ag.Tensor.from_array(x).im2col_conv2(opts).into_array()
    assert np.array_equal(y, orc.im2col_conv2(x, f, p, s, d))
    oh, ow = opts.output_shape((ih, iw))
    g = to_dtype(rng.standard_normal(y.shape), dtype)
    dx = ag.Tensor.from_array(g).col2im_conv2(ag.Col2ImConv2Options((oh, ow), f, p, s, d)).into_array()
    want = orc.col2im_conv2(g, (oh, ow), f, p, s, d)
    assert np.array_equal(dx, want)  # bit-exact incl. bf16's per-add rounding in host order


def test_col2im_bf16_rounding_order_case(ag):
    f, p = (1, 3), (0, 1)
    cols = np.zeros((3, 3), dtype=np.float32)
    cols[0, 2], cols[1, 1], cols[2, 0] = 256.0, 1.0, 1.0
    y = ag.Tensor.from_array(orc.f32_to_bf16(cols)).col2im_conv2(ag.Col2ImConv2Options((1, 3), f, p)).into_array()
    assert orc.bf16_to_f32(y)[0, 0, 0, 1] == 256.0  # an f32 accumulator would give 258


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_im2col_col2im_config3_full_size(ag, dtype):
    """Conv2 config: batch 256, 64 channels, 56x56, 3x3, stride 1, pad 1 - bit-exact against the
    oracle at full size (the oracle is a threaded copy loop, it finishes in seconds)."""
    rng = np.random.default_rng(17)
    bs, c, ih, iw, f, p = 256, 64, 56, 56, (3, 3), (1, 1)
    x = to_dtype(rng.standard_normal((bs, c, ih, iw), dtype=np.float32), dtype)
    t = ag.Tensor.from_array(x).im2col_conv2(ag.Im2ColConv2Options(filter=f, padding=p))
    y = t.into_array()
    want = orc.im2col_conv2(x, f, p)
    assert y.shape == (802816, 576)
    assert np.array_equal(y, want)
    del want
    # col2im of the patch matrix itself (values repeat, sums still round): bit-exact vs the host order
    dx = t.col2im_conv2(ag.Col2ImConv2Options((56, 56), f, p)).into_array()
    assert np.array_equal(dx, orc.col2im_conv2(y, (56, 56), f, p))


# ------------------------------------------------------------------- max pool ----
def cyc(shape):
    return (np.arange(int(np.prod(shape))) % 10).astype(np.float32).reshape(shape)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_max_pool2_reference_cases(ag, dtype):
    """max_pool2_<T> / max_pool2_backward_<T> (integration_tests.rs:1038-1061, :1554-1628)."""
    opts = ag.MaxPool2Options((2, 2), (2, 2))
    for shape in POOL_SHAPES:
        x = to_dtype(cyc(shape), dtype)
        tx = ag.Tensor.from_array(x)
        y = tx.max_pool2(opts).into_array()
        assert np.array_equal(y, orc.max_pool2(x, (2, 2)))
        dy = to_dtype(np.arange(y.size, dtype=np.float32).reshape(y.shape), dtype)
        dx = tx.clone()
        dx.max_pool2_backward(ag.Tensor.from_array(dy), opts)
        assert np.array_equal(dx.into_array(), orc.max_pool2_backward(x, dy, (2, 2)))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape,size,strides", [
    ((1000, 6, 24, 24), (2, 2), (2, 2)), ((1000, 16, 8, 8), (2, 2), (2, 2)), ((100, 6, 24, 24), (2, 2), (2, 2)),
    ((3, 5, 17, 23), (3, 2), (3, 2)), ((2, 4, 19, 21), (2, 3), (4, 5)), ((2, 3, 15, 15), (3, 3), (2, 2)),
    ((1, 2, 9, 11), (3, 3), (1, 1)), ((7, 3, 10, 33), (2, 2), (2, 1)),
])
def test_max_pool2_seeded(ag, dtype, shape, size, strides):
    rng = np.random.default_rng(18)
    # values drawn from a small set so windows contain ties; the first maximum must win
    x = to_dtype(rng.integers(-4, 5, shape).astype(np.float32) * 0.5, dtype)
    opts = ag.MaxPool2Options(size, strides)
    tx = ag.Tensor.from_array(x)
    y = tx.max_pool2(opts).into_array()
    assert np.array_equal(y, orc.max_pool2(x, size, strides))
    dy = to_dtype(rng.standard_normal(y.shape), dtype)
    dx = tx.clone()
    dx.max_pool2_backward(ag.Tensor.from_array(dy), opts)
    assert np.array_equal(dx.into_array(), orc.max_pool2_backward(x, dy, size, strides))


def test_max_pool2_special_values(ag):
    nan = np.nan
    x = np.array([[[[nan, 3, 1, nan], [4, 5, 4, 2], [-0.0, 0.0, 0.0, -0.0], [0.0, -0.0, -0.0, 0.0]]]], dtype=np.float32)
    for dtype in ("f32", "bf16"):
        xd = to_dtype(x, dtype)
        opts = ag.MaxPool2Options((2, 2), (2, 2))
        y = ag.Tensor.from_array(xd).max_pool2(opts).into_array()
        assert np.array_equal(y.view(np.uint32 if dtype == "f32" else np.uint16),
                              orc.max_pool2(xd, (2, 2)).view(np.uint32 if dtype == "f32" else np.uint16))
        dy = to_dtype(np.array([[[[1.0, -0.0], [-0.0, 2.0]]]], dtype=np.float32), dtype)
        dx = ag.Tensor.from_array(xd)
        dx.max_pool2_backward(ag.Tensor.from_array(dy), opts)
        got, want = dx.into_array(), orc.max_pool2_backward(xd, dy, (2, 2))
        assert np.array_equal(got.view(np.uint32 if dtype == "f32" else np.uint16),
                              want.view(np.uint32 if dtype == "f32" else np.uint16))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_fused_entry_points_empty_and_invalid(ag, dtype):
    """Empty batches are a no-op (the reference allows zero-length tensors); invalid geometry is an error code,
    never a launch."""
    buf = ag.Tensor.zeros((4, 4), dtype)
    ptr = buf._ptr()
    lib, check = ag.lib, ag._ffi.check
    check(getattr(lib, f"agh_relu_max_pool2_{dtype}")(ptr, ptr, 0, 4, 4, 2, 2, 2, 2))
    check(getattr(lib, f"agh_max_pool2_relu_backward_{dtype}")(ptr, ptr, None, 0, 3, 4, 4, 2, 2, 2, 2, 0))
    check(getattr(lib, f"agh_conv2_backward_input_{dtype}")(ptr, ptr, None, 0, 3, 4, 4, 8, 3, 3, 0, 0, 1, 1, 1, 1))
    with pytest.raises(ag.AghError):  # window larger than the image
        check(getattr(lib, f"agh_relu_max_pool2_{dtype}")(ptr, ptr, 1, 2, 2, 3, 3, 1, 1))
    with pytest.raises(ag.AghError):  # null output with work to do
        check(getattr(lib, f"agh_max_pool2_relu_backward_{dtype}")(ptr, ptr, None, 1, 1, 4, 4, 2, 2, 2, 2, 0))
    with pytest.raises(ag.AghError):  # zero stride
        check(getattr(lib, f"agh_conv2_backward_input_{dtype}")(ptr, ptr, ptr, 1, 1, 2, 2, 1, 3, 3, 0, 0, 0, 1, 1, 1))
    with pytest.raises(ag.AghError):  # padding swallows the image
        check(getattr(lib, f"agh_conv2_backward_input_{dtype}")(ptr, ptr, ptr, 1, 1, 1, 1, 1, 1, 1, 2, 2, 1, 1, 1, 1))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("bs,c,gh,gw,oc,f,p,s,d", [
    (100, 6, 8, 8, 16, (5, 5), (0, 0), (1, 1), (1, 1)),      # conv2 of LeNet5 (its input gradient)
    (3, 5, 7, 9, 7, (3, 2), (1, 0), (1, 1), (1, 1)),          # odd channel counts: element loads
    (2, 4, 6, 5, 8, (3, 3), (1, 1), (2, 2), (1, 1)),          # stride 2: image cells no patch reaches
    (2, 3, 5, 6, 4, (2, 3), (0, 1), (1, 2), (2, 1)),          # dilation
    (2, 4, 6, 5, 8, (3, 3), (1, 1), (1, 1), (1, 1)),          # 3x3, stride 1: a filter row at a time, one chunk
    (2, 3, 6, 7, 32, (3, 3), (1, 1), (1, 1), (2, 2)),         # the same with four / eight channel chunks, dilated
    (2, 2, 5, 5, 24, (2, 5), (0, 2), (1, 1), (1, 1)),         # 5 wide, three (f32: six) chunks
    (3, 8, 8, 8, 8, (3, 3), (1, 1), (1, 1), (1, 1)),          # images of >= 256 pixels: gradient rows staged in LDS
    (2, 16, 5, 6, 12, (3, 3), (0, 0), (1, 1), (1, 1)),        # the same, three chunks of four channels (f32 only)
    (5, 6, 9, 7, 16, (4, 5), (2, 1), (1, 1), (1, 2)),         # the same, 5 wide, padded and dilated
])
def test_conv2_backward_input_fused(ag, dtype, bs, c, gh, gw, oc, f, p, s, d):
    """agh_conv2_backward_input_<T> = dot with the weight matrix, then col2im (layer.rs:976-988).  On small
    integers every dot and every sum is exact in f32 and in bf16, so the result must equal the oracle's
    col2im of the exact product bit for bit (this pins indexing and order); on seeded real data it must be as
    close to the oracle's chain as the rounding of one dot product allows."""
    rng = np.random.default_rng(22)
    fn = getattr(ag.lib, f"agh_conv2_backward_input_{dtype}")
    k = c * f[0] * f[1]
    oh = (gh - 1) * s[0] + d[0] * (f[0] - 1) + 1 - 2 * p[0]
    ow = (gw - 1) * s[1] + d[1] * (f[1] - 1) + 1 - 2 * p[1]
    for exact in (True, False):
        if exact:
            gy = rng.integers(-2, 3, (bs * gh * gw, oc)).astype(np.float32)
            w = rng.integers(-2, 3, (oc, k)).astype(np.float32)
        else:
            gy = rng.standard_normal((bs * gh * gw, oc)).astype(np.float32)
            w = (rng.standard_normal((oc, k)) * 0.1).astype(np.float32)
        gyd, wd = to_dtype(gy, dtype), to_dtype(w, dtype)
        dx = ag.Tensor.uninit((bs, c, oh, ow), dtype)
        tgy, tw = ag.Tensor.from_array(gyd), ag.Tensor.from_array(wd)
        ag._ffi.check(fn(tgy._ptr(), tw._ptr(), dx._ptr(), bs, c, gh, gw, oc, *f, *p, *s, *d))
        got = dx.into_array()
        cols = orc.gemm_bf16_f32acc(gyd, wd) if dtype == "bf16" else orc.gemm_f64acc(gyd, wd).astype(np.float32)
        want = orc.col2im_conv2(cols, (gh, gw), f, p, s, d)
        if exact:
            assert np.array_equal(got, want)
        else:
            # each of the <= fh*fw entries of a pixel may differ by the rounding of one dot product
            scale = np.abs(as_f32(cols)).max()
            tol = f[0] * f[1] * scale * (2.0 ** -7 if dtype == "bf16" else 1e-5 * np.sqrt(oc))
            assert np.abs(as_f32(got).astype(np.float64) - as_f32(want)).max() <= tol
    big = getattr(ag.lib, f"agh_conv2_backward_input_{dtype}")
    with pytest.raises(ag.AghError):  # a filter bank that does not fit in LDS is refused, not mis-computed
        ag._ffi.check(big(dx._ptr(), dx._ptr(), dx._ptr(), 1, 64, 4, 4, 128, 3, 3, 1, 1, 1, 1, 1, 1))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("shape,size,strides", [
    ((100, 6, 24, 24), (2, 2), (2, 2)), ((100, 16, 8, 8), (2, 2), (2, 2)), ((3, 5, 17, 23), (3, 2), (3, 2)),
    ((2, 4, 19, 21), (2, 3), (4, 5)), ((1, 1, 4, 4), (2, 2), (2, 2)),
])
def test_relu_pool_fused_equals_the_separate_ops(ag, dtype, shape, size, strides):
    """agh_relu_max_pool2_<T> and agh_max_pool2_relu_backward_<T> against relu -> max_pool2 and
    max_pool2_backward -> relu_backward of the oracle, bit for bit, including cells no window covers,
    ties, signed zeros and NaN; the backward in both output layouts."""
    rng = np.random.default_rng(19)
    xf = rng.integers(-4, 5, shape).astype(np.float32) * 0.5
    if shape == (1, 1, 4, 4):
        nan = np.nan
        xf = np.array([[[[nan, 3, -1, nan], [-4, 5, -4, -2], [-0.0, 0.0, 0.0, -0.0], [0.0, -0.0, -0.0, 0.0]]]], np.float32)
    x = to_dtype(xf, dtype)
    bits = np.uint32 if dtype == "f32" else np.uint16
    bs, c, ih, iw = shape
    r = orc.relu(x)
    want_y = orc.max_pool2(r, size, strides)
    tx = ag.Tensor.from_array(x)
    y = ag.Tensor.uninit(want_y.shape, dtype)
    fwd = getattr(ag.lib, f"agh_relu_max_pool2_{dtype}")
    ag._ffi.check(fwd(tx._ptr(), y._ptr(), bs * c, ih, iw, *size, *strides))
    assert np.array_equal(y.into_array().view(bits), want_y.view(bits))
    dy = to_dtype(rng.standard_normal(want_y.shape), dtype)
    want_dx = orc.relu_backward(x, orc.max_pool2_backward(r, dy, size, strides))
    bwd = getattr(ag.lib, f"agh_max_pool2_relu_backward_{dtype}")
    tdy = ag.Tensor.from_array(dy)
    for nhwc in (0, 1):
        dx = ag.Tensor.uninit((bs, ih, iw, c) if nhwc else shape, dtype)
        ag._ffi.check(bwd(tx._ptr(), tdy._ptr(), dx._ptr(), bs, c, ih, iw, *size, *strides, nhwc))
        want = np.ascontiguousarray(want_dx.transpose(0, 2, 3, 1)) if nhwc else want_dx
        assert np.array_equal(dx.into_array().view(bits), want.view(bits)), nhwc
    # overlapping windows are refused, and so is an output on top of the input
    with pytest.raises(ag.AghError):
        ag._ffi.check(bwd(tx._ptr(), tdy._ptr(), dx._ptr(), bs, c, ih, iw, 3, 3, 2, 2, 0))
    with pytest.raises(ag.AghError):
        ag._ffi.check(bwd(tx._ptr(), tdy._ptr(), tx._ptr(), bs, c, ih, iw, *size, *strides, 0))


# ----------------------------------------------------------------------- relu ----
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_relu_reference_cases(ag, dtype):
    """relu_<T>, relu_backward_<T> (integration_tests.rs:1062-1078, :1630-1695)."""
    for shape in [(1, 8), (15, 20)]:
        n = shape[0] * shape[1]
        x = to_dtype(((np.arange(n) % 20) - 10).astype(np.float32).reshape(shape), dtype)
        assert np.array_equal(ag.Tensor.from_array(x).relu().into_array(), orc.relu(x))
        yv = to_dtype(((np.arange(n) % 2) - 1).astype(np.float32).reshape(shape), dtype)
        dy = to_dtype(np.arange(n, dtype=np.float32).reshape(shape), dtype)
        got = ag.Tensor.from_array(yv).relu_backward(ag.Tensor.from_array(dy)).into_array()
        assert np.array_equal(got, orc.relu_backward(yv, dy))
    sp = to_dtype(np.array([[-0.0, np.nan, np.inf, -np.inf, 1e-30, -1e-30]], dtype=np.float32), dtype)
    got = ag.Tensor.from_array(sp).relu().into_array()
    assert np.array_equal(got.view(np.uint8), orc.relu(sp).view(np.uint8))
