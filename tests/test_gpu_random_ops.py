"""Randomised sweeps of the operators either side of the sampler (seeded): LM head / MatMul shapes, element-wise
broadcasting, transposes, convolution and pooling shapes, argmax / softmax rows, per-row sampling configurations.
Each case is checked against the CPU oracle to the bar of the operator's own test module."""
import numpy as np
import pytest

from test_gpu_linear import _bound, _gpu_linear, _gpu_matmul

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rocm():
    from born_amd import sampler as S
    assert S.DeviceCount() >= 1, "no HIP device visible"
    return S


@pytest.fixture(scope="module")
def lin():
    from born_amd import linear as L
    return L


@pytest.fixture(scope="module")
def be():
    from born_amd import backend as B
    return B


@pytest.mark.parametrize("chunk", range(6))
def test_random_linear_and_matmul_shapes(oracle, rocm, lin, chunk):
    rng = np.random.default_rng(555 + chunk)
    for i in range(8):
        M = int(rng.choice([1, 2, 15, 16, 17, 31, 33, 64, 65, 100, 128, 129, 200]))
        K = int(rng.choice([1, 3, 8, 31, 32, 33, 64, 96, 100, 256, 260, 777, 1024, 2050]))    # (from 256 on a [K,N] product of few tiles splits K)
        N = int(rng.choice([1, 2, 4, 7, 127, 128, 129, 130, 255, 300, 512, 1001]))
        x = rng.standard_normal((M, K)).astype(np.float32)
        w = rng.standard_normal((N, K)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32) if rng.random() < 0.7 else None
        got = _gpu_linear(rocm, lin, x, w, bias)
        exact = x.astype(np.float64) @ w.astype(np.float64).T + (0 if bias is None else bias.astype(np.float64)[None, :])
        assert np.all(np.abs(got - exact) <= _bound(x, w, bias, K)), ("linear", chunk, i, M, K, N)
        b = np.ascontiguousarray(w.T)
        got = _gpu_matmul(rocm, lin, x, b)
        assert np.all(np.abs(got - x.astype(np.float64) @ b.astype(np.float64)) <= _bound(x, w, None, K)), ("matmul", chunk, i, M, K, N)
        # integer-valued operands: every partial sum is exact, so the result equals the oracle bit for bit
        xi = rng.integers(-4, 5, (M, K)).astype(np.float32)
        wi = rng.integers(-4, 5, (N, K)).astype(np.float32)
        assert np.array_equal(_gpu_linear(rocm, lin, xi, wi, None), oracle.linear_ref(xi, wi)), ("exact", chunk, i, M, K, N)


def _random_broadcast_pair(rng):
    nd = int(rng.integers(0, 6))
    full = [int(rng.choice([1, 2, 3, 5, 8, 33])) for _ in range(nd)]
    def side():
        keep = int(rng.integers(0, nd + 1))
        s = full[nd - keep:]
        return tuple(1 if rng.random() < 0.35 else d for d in s)
    return side(), side()


@pytest.mark.parametrize("chunk", range(4))
def test_random_broadcasts_transposes_reshapes(oracle, be, chunk):
    rocm = be.New()
    rng = np.random.default_rng(999 + chunk)
    for i in range(25):
        sa, sb = _random_broadcast_pair(rng)
        a = rng.standard_normal(sa).astype(np.float32)
        b = (rng.standard_normal(sb) + 3.0).astype(np.float32)
        op = str(rng.choice(["add", "sub", "mul", "div"]))
        fn = {"add": rocm.Add, "sub": rocm.Sub, "mul": rocm.Mul, "div": rocm.Div}[op]
        got = fn(be.DeviceTensor.from_numpy(a), be.DeviceTensor.from_numpy(b))
        want = oracle.binary_ref(op, a, b)
        assert tuple(got.Shape()) == want.shape and np.array_equal(got.numpy().view(np.uint32), want.view(np.uint32)), (op, sa, sb)
    for i in range(25):
        nd = int(rng.integers(1, 6))
        shape = tuple(int(rng.choice([1, 2, 3, 4, 7, 16, 65])) for _ in range(nd))
        x = rng.standard_normal(shape).astype(np.float32)
        axes = tuple(int(v) for v in rng.permutation(nd))
        got = rocm.Transpose(be.DeviceTensor.from_numpy(x), *axes)
        want = oracle.transpose_ref(x, axes)
        assert tuple(got.Shape()) == want.shape and np.array_equal(got.numpy(), want), (shape, axes)
        got = rocm.Reshape(be.DeviceTensor.from_numpy(x), (x.size,))
        assert np.array_equal(got.numpy(), x.ravel())


@pytest.mark.parametrize("chunk", range(3))
def test_random_conv2d_and_maxpool2d(oracle, be, chunk):
    rocm = be.New()
    rng = np.random.default_rng(321 + chunk)
    for i in range(10):
        N, C, CO = int(rng.integers(1, 4)), int(rng.integers(1, 6)), int(rng.integers(1, 7))
        H, W = int(rng.integers(3, 20)), int(rng.integers(3, 20))
        KH, KW = int(rng.integers(1, min(H, 5) + 1)), int(rng.integers(1, min(W, 5) + 1))
        stride, pad = int(rng.integers(1, 4)), int(rng.integers(0, 3))
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        k = rng.standard_normal((CO, C, KH, KW)).astype(np.float32)
        got = rocm.Conv2D(be.DeviceTensor.from_numpy(x), be.DeviceTensor.from_numpy(k), stride, pad)
        want = oracle.conv2d_ref(x, k, stride, pad)
        assert tuple(got.Shape()) == want.shape and np.array_equal(got.numpy().view(np.uint32), want.view(np.uint32)), (x.shape, k.shape, stride, pad)
        ks = int(rng.integers(1, min(H, W, 4) + 1))
        st = int(rng.integers(1, 4))
        got = rocm.MaxPool2D(be.DeviceTensor.from_numpy(x), ks, st)
        want = oracle.maxpool2d_ref(x, ks, st)
        assert tuple(got.Shape()) == want.shape and np.array_equal(got.numpy(), want), (x.shape, ks, st)


@pytest.mark.parametrize("chunk", range(3))
def test_random_argmax_and_softmax_rows(oracle, rocm, chunk):
    rng = np.random.default_rng(808 + chunk)
    for i in range(10):
        B = int(rng.integers(1, 9))
        V = int(rng.choice([1, 2, 63, 64, 65, 1000, 4097, 8192, 8193, 32000, 70001]))
        x = (rng.standard_normal((B, V)) * rng.choice([0.5, 3.0])).astype(np.float32)
        if rng.random() < 0.4:
            x = np.round(x).astype(np.float32)                            # ties
        if rng.random() < 0.3:
            x[rng.random((B, V)) < 0.05] = np.nan
        s = rocm.NewSampler(max_batch=B, max_vocab=V)
        dx = rocm.DeviceBuffer.from_numpy(x)
        tok = rocm.DeviceBuffer(4 * B)
        s.Argmax(dx, B, V, tok)
        assert np.array_equal(tok.to_numpy(np.int32, (B,)), oracle.argmax_ref(x)), (chunk, i, B, V)
        y = np.nan_to_num(x, nan=0.0)
        out = rocm.DeviceBuffer(4 * B * V)
        s.Softmax(rocm.DeviceBuffer.from_numpy(y), B, V, out)
        got = out.to_numpy(np.float32, (B, V))
        assert np.allclose(got, oracle.softmax_f64(y), rtol=1e-5, atol=1e-30), (chunk, i, B, V)
        s.Close()


@pytest.mark.parametrize("path", [0, 1, 2])
@pytest.mark.parametrize("chunk", range(4))
def test_random_per_row_configurations(oracle, rocm, chunk, path):
    from test_gpu_parity import _sample_rows
    rng = np.random.default_rng(2024 + chunk)
    for i in range(4):
        B = int(rng.integers(1, 17))
        V = int(rng.choice([3, 64, 130, 1001, 4100, 9000, 32000]))
        H = int(rng.choice([1, 8, 300, 1100]))
        x = (rng.standard_normal((B, V)) * 2.0).astype(np.float32)
        u = rng.random(B, dtype=np.float32)
        hist = ((rng.zipf(1.3, size=(B, H)) - 1) % V).astype(np.int32)
        Ts = rng.choice([0.5, 0.7, 1.0, 1.3], B).astype(np.float32)
        ks = rng.choice([0, 1, 5, 40, 64, 65, 300, V, V + 5, -3], B).astype(np.int32)
        ps = rng.choice([1.0, 0.9, 0.5, 0.99], B).astype(np.float32)
        reps = rng.choice([1.0, 1.15, 2.0, 0.8], B).astype(np.float32)
        extras = [dict(), dict(MinP=0.05), dict(FrequencyPenalty=0.2, PresencePenalty=0.1)][int(rng.integers(0, 3))]
        mps = frs = prs = None                                             # per-row arrays of the three, now and then
        if rng.random() < 0.5:
            mps = rng.choice([0.0, 0.02, 0.3], B).astype(np.float32)
        if rng.random() < 0.5:
            frs = rng.choice([0.0, 0.3, -0.2], B).astype(np.float32)
            prs = rng.choice([0.0, 0.5], B).astype(np.float32)
        s, tok, pr = _sample_rows(rocm, x, u, hist, Ts, ks, ps, reps, path, min_ps=mps, freqs=frs, press=prs, **extras)
        s.Status()
        s.Close()
        for b in range(B):
            want = oracle.sample(x[b:b + 1], u[b:b + 1], float(Ts[b]), int(ks[b]), float(ps[b]), float(reps[b]), hist[b:b + 1], None,
                                 mode=oracle.MODE_FIXED, min_p=extras.get("MinP", 0.0) if mps is None else float(mps[b]),
                                 freq=extras.get("FrequencyPenalty", 0.0) if frs is None else float(frs[b]),
                                 pres=extras.get("PresencePenalty", 0.0) if prs is None else float(prs[b]))
            assert tok[b] == want["tokens"][0], (chunk, i, b, V, H, Ts[b], ks[b], ps[b], reps[b], extras)
            assert pr[b:b + 1].view(np.uint32)[0] == want["probs"].view(np.uint32)[0], (chunk, i, b)


@pytest.mark.parametrize("chunk", range(4))
def test_random_gemm_pitches_and_alignments(rocm, chunk):
    # random shapes, row pitches (multiples of four and not) and base offsets, so that every load path of the GEMM
    # (direct-to-LDS, register-staged vector, scalar) and every tile height is met; nothing outside the output's
    # rows and columns may be written, nothing outside the operands' rows may influence the result (NaN padding)
    from born_amd import _capi
    rng = np.random.default_rng(31337 + chunk)
    for i in range(10):
        M = int(rng.choice([1, 7, 16, 24, 32, 33, 64, 100, 128, 130, 260]))
        K = int(rng.choice([1, 5, 32, 64, 96, 128, 160, 250, 512]))
        N = int(rng.choice([1, 3, 128, 129, 256, 300, 640, 1000]))
        lda = K + int(rng.choice([0, 0, 1, 4, 8]))
        ldw = K + int(rng.choice([0, 0, 3, 4, 32]))
        ldc = N + int(rng.choice([0, 0, 1, 4]))
        off = int(rng.choice([0, 0, 1, 2, 4]))
        xa = np.full((M, lda), np.nan, np.float32)
        wa = np.full((N, ldw), np.nan, np.float32)
        xa[:, :K] = rng.standard_normal((M, K))
        wa[:, :K] = rng.standard_normal((N, K))
        bias = rng.standard_normal(N).astype(np.float32) if rng.random() < 0.6 else None
        pad = np.full(off, np.nan, np.float32)
        dx = rocm.DeviceBuffer.from_numpy(np.concatenate([pad, xa.ravel(), pad, np.zeros(1, np.float32)]))
        dw = rocm.DeviceBuffer.from_numpy(np.concatenate([pad, wa.ravel(), pad, np.zeros(1, np.float32)]))
        db = None if bias is None else rocm.DeviceBuffer.from_numpy(np.concatenate([pad, bias, np.zeros(1, np.float32)]))
        sentinel = np.full(off + M * ldc + 1, -777.0, np.float32)
        dc = rocm.DeviceBuffer.from_numpy(sentinel)
        _capi.check(_capi.lib().born_rocm_linear(dx.ptr + 4 * off, M, K, lda, dw.ptr + 4 * off, N, ldw, None if db is None else db.ptr + 4 * off,
                                                 dc.ptr + 4 * off, ldc, None))
        out = dc.to_numpy(np.float32, sentinel.shape)
        got = out[off:off + M * ldc].reshape(M, ldc)
        tag = (chunk, i, M, K, N, lda, ldw, ldc, off, bias is not None)
        assert np.all(out[:off] == -777.0) and out[-1] == -777.0 and np.all(got[:, N:] == -777.0), tag
        x, w = xa[:, :K], wa[:, :K]
        exact = x.astype(np.float64) @ w.astype(np.float64).T + (0 if bias is None else bias.astype(np.float64)[None, :])
        assert np.all(np.abs(got[:, :N] - exact) <= _bound(x, w, bias, K)), tag
        # the same product through matmul, b = w^T stored [K, N] with its own pitch
        ldb = N + int(rng.choice([0, 0, 2, 4]))
        ba = np.full((K, ldb), np.nan, np.float32)
        ba[:, :N] = w.T
        dbm = rocm.DeviceBuffer.from_numpy(np.concatenate([pad, ba.ravel(), np.zeros(1, np.float32)]))
        dc2 = rocm.DeviceBuffer.from_numpy(sentinel)
        _capi.check(_capi.lib().born_rocm_matmul(dx.ptr + 4 * off, dbm.ptr + 4 * off, dc2.ptr + 4 * off, M, K, N, lda, ldb, ldc, None))
        out2 = dc2.to_numpy(np.float32, sentinel.shape)
        got2 = out2[off:off + M * ldc].reshape(M, ldc)
        assert np.all(out2[:off] == -777.0) and out2[-1] == -777.0 and np.all(got2[:, N:] == -777.0), tag
        assert np.all(np.abs(got2[:, :N] - x.astype(np.float64) @ w.astype(np.float64).T) <= _bound(x, w, None, K)), tag
