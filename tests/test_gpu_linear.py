"""GPU parity tests of the logits producer (born_rocm_linear / born_rocm_matmul, through the C ABI and its
Python mirror) against the CPU oracle's restatement of the reference's MatMul and Linear.Forward.

Tolerance (floating point; the order of the k-sum differs between the matrix-core kernel and the
reference's sequential loop, so agreement is to rounding):
    |gpu - exact| <= (4 * sqrt(K) + 2) * 2^-24 * (sum_k |a_k| |b_k| + |bias|)
against an fp64 product, and twice the reference loop's own worst-case bound plus that against the
oracle.  Integer-valued operands, whose partial sums are all exact in fp32, must match bit for bit.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

EPS = 2.0 ** -24


@pytest.fixture(scope="module")
def rocm():
    from born_amd import sampler as S
    assert S.DeviceCount() >= 1, "no HIP device visible"
    return S


@pytest.fixture(scope="module")
def lin():
    from born_amd import linear as L
    return L


def _bound(a, bt, bias, K):
    mag = np.abs(a).astype(np.float64) @ np.abs(bt).astype(np.float64).T
    if bias is not None:
        mag = mag + np.abs(bias).astype(np.float64)[None, :]
    return (4.0 * np.sqrt(K) + 2.0) * EPS * mag + 1e-37


def _gpu_linear(rocm, lin, x, w, bias):
    M, K = x.shape
    N = w.shape[0]
    layer = lin.Linear(K, N, rocm.DeviceBuffer.from_numpy(w), None if bias is None else rocm.DeviceBuffer.from_numpy(bias))
    dx = rocm.DeviceBuffer.from_numpy(x)
    out = rocm.DeviceBuffer(M * N * 4)
    layer.Forward(dx, (M, K), out)
    return out.to_numpy(np.float32, (M, N))


def _gpu_matmul(rocm, lin, a, b):
    M, K = a.shape
    N = b.shape[1]
    out = rocm.DeviceBuffer(M * N * 4)
    lin.MatMul(rocm.DeviceBuffer.from_numpy(a), rocm.DeviceBuffer.from_numpy(b), M, K, N, out, k_b=b.shape[0])
    return out.to_numpy(np.float32, (M, N))


def test_reference_kats(rocm, lin):
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_kats.json")) as f:
        kats = json.load(f)
    for case in kats["matmul"]:
        got = _gpu_matmul(rocm, lin, np.array(case["a"], np.float32), np.array(case["b"], np.float32))
        assert np.max(np.abs(got.astype(np.float64) - np.array(case["expected"]))) <= case["tol_abs"], case["source"]
    for case in kats["linear"]:
        bias = None if case["bias"] is None else np.array(case["bias"], np.float32)
        got = _gpu_linear(rocm, lin, np.array(case["x"], np.float32), np.array(case["weight"], np.float32), bias)
        assert np.max(np.abs(got.astype(np.float64) - np.array(case["expected"]))) <= case["tol_abs"], case["source"]


SHAPES = [(1, 1, 1), (1, 3, 2), (2, 2, 2), (3, 5, 7), (7, 16, 5), (33, 17, 65), (64, 64, 64), (127, 100, 129),
          (128, 128, 128), (129, 15, 127), (130, 257, 300), (256, 512, 1000), (5, 1000, 1), (300, 33, 31),
          # every tile height (16, 32, 64, 128 rows) on the unguarded-load route (K a multiple of 32)
          (1, 64, 300), (16, 128, 260), (17, 96, 132), (32, 256, 100), (48, 64, 256), (65, 32, 128), (12, 4096, 520),
          # few tiles and a long K: the [K,N] product splits K over workgroups (ragged last slice, unaligned K, one row)
          (64, 784, 128), (64, 790, 10), (512, 4096, 512), (100, 1000, 260), (1, 5000, 7), (33, 257, 129), (200, 2048, 300)]


@pytest.mark.parametrize("shape", SHAPES)
def test_linear_matches_oracle(oracle, rocm, lin, shape):
    M, K, N = shape
    rng = np.random.default_rng(M * 1000003 + K * 1009 + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.standard_normal((N, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    for b in (bias, None):
        got = _gpu_linear(rocm, lin, x, w, b)
        exact = x.astype(np.float64) @ w.astype(np.float64).T + (0.0 if b is None else b.astype(np.float64)[None, :])
        bound = _bound(x, w, b, K)
        assert np.all(np.abs(got - exact) <= bound), f"{shape}: off the fp64 product by {np.max(np.abs(got - exact) / bound):.2f} bounds"
        ref = oracle.linear_ref(x, w, b)
        ref_bound = (K + 2) * EPS * (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T + (0 if b is None else np.abs(b)[None, :]))
        assert np.all(np.abs(got.astype(np.float64) - ref) <= bound + ref_bound), shape


@pytest.mark.parametrize("shape", SHAPES)
def test_matmul_matches_oracle(oracle, rocm, lin, shape):
    M, K, N = shape
    rng = np.random.default_rng(M * 7919 + K * 104729 + N)
    a = rng.standard_normal((M, K)).astype(np.float32)
    b = rng.standard_normal((K, N)).astype(np.float32)
    got = _gpu_matmul(rocm, lin, a, b)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    bound = _bound(a, np.ascontiguousarray(b.T), None, K)
    assert np.all(np.abs(got - exact) <= bound), f"{shape}: off the fp64 product by {np.max(np.abs(got - exact) / bound):.2f} bounds"
    ref = oracle.matmul_ref(a, b)
    ref_bound = (K + 2) * EPS * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64))
    assert np.all(np.abs(got.astype(np.float64) - ref) <= bound + ref_bound), shape


@pytest.mark.parametrize("shape", [(3, 5, 7), (130, 257, 300), (256, 64, 129)])
def test_integer_valued_operands_are_bit_exact(oracle, rocm, lin, shape):
    # every product and partial sum is an integer below 2^24: exact in fp32 whatever the order of the sum
    M, K, N = shape
    rng = np.random.default_rng(11)
    x = rng.integers(-8, 9, (M, K)).astype(np.float32)
    w = rng.integers(-8, 9, (N, K)).astype(np.float32)
    bias = rng.integers(-100, 101, N).astype(np.float32)
    assert np.array_equal(_gpu_linear(rocm, lin, x, w, bias), oracle.linear_ref(x, w, bias))
    b = np.ascontiguousarray(w.T)
    assert np.array_equal(_gpu_matmul(rocm, lin, x, b), oracle.matmul_ref(x, b))


def test_pitches_and_unaligned_operands(oracle, rocm):
    # rows wider than the matrix, pitches that are not multiples of 4 elements, bases off 16-byte alignment:
    # the kernel must take its scalar loads, never read or write outside the rows
    import ctypes as C
    from born_amd import _capi
    rng = np.random.default_rng(5)
    M, K, N = 70, 37, 150
    lda, ldw, ldc = 41, 39, 153
    xa = rng.standard_normal((M, lda)).astype(np.float32)
    wa = rng.standard_normal((N, ldw)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    for off in (0, 1):                                   # element offset of every base pointer
        dx = rocm.DeviceBuffer.from_numpy(np.concatenate([np.zeros(off, np.float32), xa.ravel()]))
        dw = rocm.DeviceBuffer.from_numpy(np.concatenate([np.zeros(off, np.float32), wa.ravel()]))
        db = rocm.DeviceBuffer.from_numpy(np.concatenate([np.zeros(off, np.float32), bias]))
        sentinel = np.full(off + M * ldc, -777.0, np.float32)
        dc = rocm.DeviceBuffer.from_numpy(sentinel)
        _capi.check(_capi.lib().born_rocm_linear(dx.ptr + 4 * off, M, K, lda, dw.ptr + 4 * off, N, ldw, db.ptr + 4 * off,
                                                 dc.ptr + 4 * off, ldc, None))
        out = dc.to_numpy(np.float32, (off + M * ldc,))
        assert np.all(out[:off] == -777.0)
        got = out[off:].reshape(M, ldc)
        assert np.all(got[:, N:] == -777.0), "wrote outside the rows of the output"
        x, w = xa[:, :K], wa[:, :K]
        exact = x.astype(np.float64) @ w.astype(np.float64).T + bias[None, :]
        assert np.all(np.abs(got[:, :N] - exact) <= _bound(x, w, bias, K))
        # the same operands through matmul: b = w^T stored [K, N] with pitch ldb
        ldb = N + 3
        ba = np.zeros((K, ldb), np.float32)
        ba[:, :N] = w.T
        dbm = rocm.DeviceBuffer.from_numpy(np.concatenate([np.zeros(off, np.float32), ba.ravel()]))
        dc2 = rocm.DeviceBuffer.from_numpy(sentinel)
        _capi.check(_capi.lib().born_rocm_matmul(dx.ptr + 4 * off, dbm.ptr + 4 * off, dc2.ptr + 4 * off, M, K, N, lda, ldb, ldc, None))
        got2 = dc2.to_numpy(np.float32, (off + M * ldc,))[off:].reshape(M, ldc)
        assert np.all(got2[:, N:] == -777.0)
        assert np.all(np.abs(got2[:, :N] - (exact - bias[None, :])) <= _bound(x, w, None, K))


def test_argument_errors(rocm, lin):
    w = rocm.DeviceBuffer(64)
    layer = lin.Linear(4, 4, w, None)
    with pytest.raises(lin.LinearPanic, match="expected input with 4 features, got 3"):
        layer.Forward(w, (1, 3), w)
    with pytest.raises(lin.LinearPanic, match="expected 2D input"):
        layer.Forward(w, (4,), w)
    with pytest.raises(lin.LinearPanic, match="shape mismatch"):
        lin.MatMul(w, w, 2, 2, 2, w, k_b=3)
    from born_amd import _capi
    assert _capi.lib().born_rocm_linear(None, 1, 1, 1, None, 1, 1, None, None, 1, None) == _capi.ERR_ARGUMENT
    assert _capi.lib().born_rocm_matmul(w.ptr, w.ptr, w.ptr, 2, 2, 2, 1, 2, 2, None) == _capi.ERR_ARGUMENT   # pitch < row


def test_lm_head_then_sample_without_leaving_the_device(oracle, rocm, lin):
    # hidden states -> LM head -> sampler, all on the device; the sampler's tokens are bit-exact against the
    # oracle run on the logits the device produced, and those logits agree with the oracle's Linear to rounding
    rng = np.random.default_rng(2025)
    B, K, V = 48, 256, 32000
    hidden = rng.standard_normal((B, K)).astype(np.float32)
    w = (rng.standard_normal((V, K)) * (2.0 / np.sqrt(K))).astype(np.float32)
    bias = (rng.standard_normal(V) * 0.1).astype(np.float32)
    u = rng.random(B, dtype=np.float32)
    hist = rng.integers(0, V, (B, 64)).astype(np.int32)
    layer = lin.Linear(K, V, rocm.DeviceBuffer.from_numpy(w), rocm.DeviceBuffer.from_numpy(bias))
    logits = rocm.DeviceBuffer(B * V * 4)
    layer.Forward(rocm.DeviceBuffer.from_numpy(hidden), (B, K), logits)
    s = rocm.NewSampler(rocm.SamplerConfig(Temperature=0.7, TopK=50, TopP=0.9, RepetitionPenalty=1.15), max_batch=B, max_vocab=V)
    tokens = rocm.DeviceBuffer(B * 4)
    probs = rocm.DeviceBuffer(B * 4)
    s.Sample(logits, B, V, rocm.DeviceBuffer.from_numpy(hist), None, rocm.DeviceBuffer.from_numpy(u), tokens, probs, hist_stride=64)
    s.Status()
    got_tokens = tokens.to_numpy(np.int32, (B,))
    x = logits.to_numpy(np.float32, (B, V))
    exact = hidden.astype(np.float64) @ w.astype(np.float64).T + bias[None, :]
    assert np.all(np.abs(x - exact) <= _bound(hidden, w, bias, K))
    fx = oracle.sample(x, u, 0.7, 50, 0.9, 1.15, hist, None, mode=oracle.MODE_FIXED)
    assert np.array_equal(got_tokens, fx["tokens"])
    s.Close()


def test_lm_head_full_size_spot_check(rocm, lin):
    # batch 256 x hidden 2048 -> vocabulary 128256 (1 GB of weights): 4000 random entries and two whole
    # columns of tiles against fp64 dot products; every workgroup id mapping (XCD-aware order) is exercised
    rng = np.random.default_rng(99)
    M, K, N = 256, 2048, 128256
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.standard_normal((N, K), dtype=np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    got = _gpu_linear(rocm, lin, x, w, bias)
    rows = rng.integers(0, M, 4000)
    cols = rng.integers(0, N, 4000)
    exact = np.einsum("ik,ik->i", x[rows].astype(np.float64), w[cols].astype(np.float64)) + bias[cols]
    mag = np.einsum("ik,ik->i", np.abs(x[rows]).astype(np.float64), np.abs(w[cols]).astype(np.float64)) + np.abs(bias[cols])
    assert np.all(np.abs(got[rows, cols] - exact) <= (4 * np.sqrt(K) + 2) * EPS * mag)
    for c0 in (0, N - 300):                                # first tiles and the ragged last ones, all rows
        sl = slice(c0, c0 + 300)
        ex = x.astype(np.float64) @ w[sl].astype(np.float64).T + bias[sl][None, :]
        assert np.all(np.abs(got[:, sl] - ex) <= _bound(x, w[sl], bias[sl], K))
    # every output element was written: a checksum of all rows against the fp64 product with the column sum of W
    colsum = w.astype(np.float64).sum(axis=0)
    want = x.astype(np.float64) @ colsum + bias.astype(np.float64).sum()
    scale = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).sum(axis=0)
    assert np.all(np.abs(got.astype(np.float64).sum(axis=1) - want) <= (4 * np.sqrt(K) + 2) * EPS * scale)


@pytest.mark.parametrize("shape", [(1, 64, 300), (5, 1000, 77), (16, 128, 260), (17, 96, 132), (48, 64, 256), (65, 32, 128),
                                   (130, 257, 300), (256, 512, 1000), (12, 4096, 32000)])
def test_lm_head_argmax_fused_equals_linear_then_argmax(oracle, rocm, lin, shape):
    # tokens of the fused call == argmax kernel over the materialised logits of the same GEMM (bit-identical
    # arithmetic), == the oracle's argmax over those logits
    M, K, N = shape
    rng = np.random.default_rng(M * 31 + K * 7 + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.standard_normal((N, K)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    s = rocm.NewSampler(max_batch=M, max_vocab=N)
    for b in (bias, None):
        layer = lin.Linear(K, N, rocm.DeviceBuffer.from_numpy(w), None if b is None else rocm.DeviceBuffer.from_numpy(b))
        dx = rocm.DeviceBuffer.from_numpy(x)
        logits = rocm.DeviceBuffer(M * N * 4)
        layer.Forward(dx, (M, K), logits)
        tok_ref = rocm.DeviceBuffer(4 * M)
        s.Argmax(logits, M, N, tok_ref)
        tok = rocm.DeviceBuffer(4 * M)
        lin.ForwardArgmax(s, layer, dx, (M, K), tok)
        got = tok.to_numpy(np.int32, (M,))
        assert np.array_equal(got, tok_ref.to_numpy(np.int32, (M,))), shape
        assert np.array_equal(got, oracle.argmax_ref(logits.to_numpy(np.float32, (M, N)))), shape
    s.Close()


def test_lm_head_argmax_tie_and_nan_rules(oracle, rocm, lin):
    # integer-valued operands make exact ties; NaN never wins except at column 0; -0 equals +0; an all -inf row
    M, K, N = 6, 32, 300
    x = np.zeros((M, K), np.float32)
    w = np.zeros((N, K), np.float32)
    x[:, 0] = 1.0
    w[:, 0] = -5.0
    w[[7, 150, 299], 0] = 3.0                      # rows 0..: three equal maxima -> lowest column 7
    bias = np.zeros((M, N), np.float32)
    cases = []
    b0 = np.zeros(N, np.float32); cases.append(b0)                                    # tie -> 7
    b1 = b0.copy(); b1[200] = np.nan; cases.append(b1)                                # NaN elsewhere ignored -> 7
    b2 = b0.copy(); b2[0] = np.nan; cases.append(b2)                                  # NaN at column 0 -> 0
    b3 = np.full(N, -np.inf, np.float32); cases.append(b3)                            # all -inf -> 0
    b4 = b3.copy(); b4[[40, 41]] = [5.0 - 0.0, 5.0]; cases.append(b4)                 # two finite: w*x + b = 0 at both? no: -5+5 = 0 vs 0 -> tie -> 40
    b5 = np.full(N, np.nan, np.float32); cases.append(b5)                             # all NaN -> 0
    s = rocm.NewSampler(max_batch=M, max_vocab=N)
    for b in cases:
        layer = lin.Linear(K, N, rocm.DeviceBuffer.from_numpy(w), rocm.DeviceBuffer.from_numpy(b))
        dx = rocm.DeviceBuffer.from_numpy(x)
        tok = rocm.DeviceBuffer(4 * M)
        lin.ForwardArgmax(s, layer, dx, (M, K), tok)
        with np.errstate(all="ignore"):
            logits = oracle.linear_ref(x, w, b)
        want = oracle.argmax_ref(logits)
        assert np.array_equal(tok.to_numpy(np.int32, (M,)), want), (b[:3], want)
    s.Close()


@pytest.mark.parametrize("extras", [{}, dict(MinP=0.02, FrequencyPenalty=0.3, PresencePenalty=0.2)])
def test_lm_head_and_sampling_step_replay_from_a_hip_graph(oracle, rocm, lin, extras):
    # the decode step (LM head -> sampler -> log-probability of the sampled token; with the frequency / presence
    # penalties also the launches that raise and clear the table of counts) captured once into a HIP graph and
    # replayed with new activations, uniforms and histories in the same buffers; every replay is checked against
    # the eager calls and the oracle, with eager work and synchronisations between the replays.  The HIP runtime is
    # driven through ctypes (the library itself exports no graph calls).
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    def ok(rc):
        assert rc == 0, f"HIP error {rc}"
    rng = np.random.default_rng(404)
    B, K, V = 4, 256, 32000
    w = rocm.DeviceBuffer.from_numpy((rng.standard_normal((V, K)) * (2.0 / np.sqrt(K))).astype(np.float32))
    bias = rocm.DeviceBuffer.from_numpy((0.1 * rng.standard_normal(V)).astype(np.float32))
    hist_h = rng.integers(0, V, (B, 32)).astype(np.int32)
    hist = rocm.DeviceBuffer.from_numpy(hist_h)
    x, u = rocm.DeviceBuffer(B * K * 4), rocm.DeviceBuffer(B * 4)
    logits, tokens, probs = rocm.DeviceBuffer(B * V * 4), rocm.DeviceBuffer(B * 4), rocm.DeviceBuffer(B * 4)
    logprobs = rocm.DeviceBuffer(B * 4)
    layer = lin.Linear(K, V, w, bias)
    smp = rocm.NewSampler(rocm.SamplerConfig(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1, **extras), max_batch=B, max_vocab=V)
    okw = dict(min_p=extras.get("MinP", 0.0), freq=extras.get("FrequencyPenalty", 0.0), pres=extras.get("PresencePenalty", 0.0))

    def step(stream):
        layer.Forward(x, (B, K), logits, stream=stream)
        smp.Sample(logits, B, V, hist, None, u, tokens, probs, hist_stride=32, stream=stream)
        smp.TokenLogprobs(logits, B, V, hist, None, tokens, logprobs, hist_stride=32, stream=stream)

    def upload(buf, a):
        from born_amd import _capi
        _capi.check(_capi.lib().born_rocm_h2d(buf.ptr, a.ctypes.data, a.nbytes, None))

    stream = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(stream)))
    upload(x, np.zeros((B, K), np.float32))
    upload(u, np.zeros(B, np.float32))
    step(stream)                                                  # warm-up outside the capture
    ok(hip.hipStreamSynchronize(stream))
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(stream, 0))                      # hipStreamCaptureModeGlobal
    step(stream)
    ok(hip.hipStreamEndCapture(stream, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)))
    for it in range(4):
        xh = rng.standard_normal((B, K)).astype(np.float32)
        uh = rng.random(B, dtype=np.float32)
        hist_h = ((rng.zipf(1.3, size=(B, 32)) - 1) % V).astype(np.int32)
        upload(x, xh)
        upload(u, uh)
        upload(hist, hist_h)
        ok(hip.hipGraphLaunch(gexec, stream))
        ok(hip.hipStreamSynchronize(stream))
        got_tok, got_logits = tokens.to_numpy(np.int32, (B,)), logits.to_numpy(np.float32, (B, V))
        got_lp = logprobs.to_numpy(np.float32, (B,))
        upload(tokens, np.full(B, -1, np.int32))
        step(None)                                                # the same step, eagerly, on the null stream
        ok(hip.hipDeviceSynchronize())
        assert np.array_equal(got_tok, tokens.to_numpy(np.int32, (B,))), it
        assert np.array_equal(got_logits, logits.to_numpy(np.float32, (B, V))), it
        assert np.array_equal(got_lp, logprobs.to_numpy(np.float32, (B,))), it
        want = oracle.sample(got_logits, uh, 0.8, 40, 0.95, 1.1, hist_h, None, mode=oracle.MODE_FIXED, **okw)
        assert np.array_equal(got_tok, want["tokens"]), it
        want_lp, _ = oracle.token_logprobs(got_logits, got_tok, temperature=0.8, rep=1.1, history=hist_h, freq=okw["freq"], pres=okw["pres"])
        assert np.all(np.abs(got_lp - want_lp) <= 1e-5 + 1e-6 * np.abs(want_lp)), it
    ok(hip.hipGraphExecDestroy(gexec))
    ok(hip.hipGraphDestroy(graph))
    ok(hip.hipStreamDestroy(stream))
    smp.Status()
    smp.Close()


def _fused_vs_unfused(rocm, lin, x, w, bias, cfg, hist=None, expect_settled=True):
    """Tokens and probabilities of born_rocm_linear_sample against born_rocm_linear + born_rocm_sample on the same
    operands: the candidates the epilogue lists are the values the plain GEMM would write, so the two must agree bit
    for bit.  Returns what the fused call gave."""
    M, K = x.shape
    N = w.shape[0]
    rng = np.random.default_rng(M + 3 * N)
    u = rng.random(M, dtype=np.float32)
    s = rocm.NewSampler(cfg, max_batch=M, max_vocab=N)
    layer = lin.Linear(K, N, rocm.DeviceBuffer.from_numpy(w), None if bias is None else rocm.DeviceBuffer.from_numpy(bias))
    dx, du = rocm.DeviceBuffer.from_numpy(x), rocm.DeviceBuffer.from_numpy(u)
    dh = None if hist is None else rocm.DeviceBuffer.from_numpy(hist)
    H = 0 if hist is None else hist.shape[1]
    logits = rocm.DeviceBuffer(M * N * 4)
    layer.Forward(dx, (M, K), logits)
    tok_ref, pr_ref = rocm.DeviceBuffer(4 * M), rocm.DeviceBuffer(4 * M)
    s.Sample(logits, M, N, dh, None, du, tok_ref, pr_ref, hist_stride=H)
    s.Status()
    tok, pr = rocm.DeviceBuffer(4 * M), rocm.DeviceBuffer(4 * M)
    lin.ForwardSample(s, layer, dx, (M, K), dh, None, du, tok, pr, hist_stride=H)
    got, gp = tok.to_numpy(np.int32, (M,)), pr.to_numpy(np.float32, (M,))
    want, wp = tok_ref.to_numpy(np.int32, (M,)), pr_ref.to_numpy(np.float32, (M,))
    settled = got >= 0
    if expect_settled:
        s.Status()
        assert settled.all(), np.nonzero(~settled)[0][:8]
    assert np.array_equal(got[settled], want[settled])
    assert np.array_equal(gp[settled].view(np.uint32), wp[settled].view(np.uint32))
    # the host-side wrapper owes the caller the unsettled rows: it repeats the call unfused
    t2, p2, fell_back = lin.ForwardSampleHost(s, layer, dx, (M, K), dh, None, du, hist_stride=H)
    assert fell_back == (not settled.all())
    assert np.array_equal(t2, want) and np.array_equal(p2.view(np.uint32), wp.view(np.uint32))
    s.Close()
    return got, settled


@pytest.mark.parametrize("shape", [(1, 64, 300), (5, 1000, 777), (16, 128, 2600), (17, 96, 1320), (48, 64, 4096), (65, 32, 5000),
                                   (130, 257, 9000), (256, 512, 33000), (12, 4096, 32000)])
def test_lm_head_sampling_fused_equals_linear_then_sample(rocm, lin, shape):
    M, K, N = shape
    rng = np.random.default_rng(M * 31 + K * 7 + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * (1.5 / np.sqrt(K))).astype(np.float32)
    bias = (0.3 * rng.standard_normal(N)).astype(np.float32)
    hist = rng.integers(0, N, size=(M, 40)).astype(np.int32)
    cfg = rocm.SamplerConfig(Temperature=0.7, TopK=min(50, N - 1), TopP=0.9, RepetitionPenalty=1.15)
    for b in (bias, None):
        _fused_vs_unfused(rocm, lin, x, w, b, cfg, hist)
    _fused_vs_unfused(rocm, lin, x, w, bias, rocm.SamplerConfig(Temperature=1.0, TopK=min(128, N - 1)), None)


def test_lm_head_sampling_fused_penalised_favourites_and_unsettled_rows(rocm, lin):
    """Histories that hold the very tokens a row favours (the penalty moves candidates across the cut), then rows the
    fused step must hand back: every logit equal (the list overflows) and a history longer than the workgroup."""
    M, K, N = 24, 128, 6000
    rng = np.random.default_rng(99)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * (2.0 / np.sqrt(K))).astype(np.float32)
    logits = x.astype(np.float64) @ w.astype(np.float64).T
    hist = np.argsort(-logits, axis=1)[:, :60].astype(np.int32)      # the sixty largest of every row
    cfg = rocm.SamplerConfig(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.3)
    _fused_vs_unfused(rocm, lin, x, w, None, cfg, hist, expect_settled=False)
    # all logits equal: every column reaches the threshold
    got, settled = _fused_vs_unfused(rocm, lin, np.zeros((3, K), np.float32), w, None, rocm.SamplerConfig(TopK=5), None, expect_settled=False)
    assert not settled.any()
    long_hist = rng.integers(0, N, size=(M, 1500)).astype(np.int32)
    got, settled = _fused_vs_unfused(rocm, lin, x, w, None, cfg, long_hist, expect_settled=False)
    assert not settled.any()


def test_lm_head_sampling_fused_built_in_stream_survives_a_fallback(rocm, lin):
    """With the built-in uniform stream (uniforms = None) a seeded generation must not depend on whether a fused call
    fell back: the wrapper sets the draw counter back before it repeats the call unfused, so that call and every later
    one draw what a twin handle that never used the fused call draws."""
    M, K, N = 6, 128, 6000
    rng = np.random.default_rng(4242)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * (2.0 / np.sqrt(K))).astype(np.float32)
    cfg = rocm.SamplerConfig(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.3, Seed=777)
    dw = rocm.DeviceBuffer.from_numpy(w)
    layer = lin.Linear(K, N, dw, None)
    fused = rocm.NewSampler(cfg, max_batch=M, max_vocab=N)
    twin = rocm.NewSampler(cfg, max_batch=M, max_vocab=N)
    long_hist = rocm.DeviceBuffer.from_numpy(rng.integers(0, N, size=(M, 1500)).astype(np.int32))   # no row can settle
    short_hist = rocm.DeviceBuffer.from_numpy(rng.integers(0, N, size=(M, 40)).astype(np.int32))
    dx = rocm.DeviceBuffer.from_numpy(x)
    logits = rocm.DeviceBuffer(4 * M * N)
    layer.Forward(dx, (M, K), logits)
    tok = rocm.DeviceBuffer(4 * M)
    fell = []
    for step, (hist, H) in enumerate([(short_hist, 40), (long_hist, 1500), (short_hist, 40), (long_hist, 1500), (short_hist, 40)]):
        assert fused.Step() == step == twin.Step()
        got, _, fell_back = lin.ForwardSampleHost(fused, layer, dx, (M, K), hist, None, None, hist_stride=H)
        fell.append(fell_back)
        twin.Sample(logits, M, N, hist, None, None, tok, None, hist_stride=H)
        want = tok.to_numpy(np.int32, (M,))
        assert np.array_equal(got, want), (step, got, want)
    assert fell == [False, True, False, True, False]
    assert fused.Step() == 5 == twin.Step()
    with pytest.raises(rocm.SamplerPanic):
        fused.SetStep(-1)
    fused.Close()
    twin.Close()


def test_lm_head_sampling_fused_argument_errors(rocm, lin):
    from born_amd import _capi
    M, K, N = 4, 64, 500
    x = rocm.DeviceBuffer.from_numpy(np.zeros((M, K), np.float32))
    layer = lin.Linear(K, N, rocm.DeviceBuffer.from_numpy(np.zeros((N, K), np.float32)), None)
    u = rocm.DeviceBuffer.from_numpy(np.zeros(M, np.float32))
    tok = rocm.DeviceBuffer(4 * M)
    for cfg in (rocm.SamplerConfig(TopP=0.9), rocm.SamplerConfig(TopK=200), rocm.SamplerConfig(TopK=5, FrequencyPenalty=0.5)):
        s = rocm.NewSampler(cfg, max_batch=M, max_vocab=N)
        with pytest.raises(_capi.BornRocmError) as e:
            lin.ForwardSample(s, layer, x, (M, K), None, None, u, tok)
        assert e.value.code == _capi.ERR_UNSUPPORTED
        s.Close()
    s = rocm.NewSampler(rocm.SamplerConfig(TopK=5), max_batch=M, max_vocab=N)
    with pytest.raises(rocm.SamplerPanic):
        lin.ForwardSample(s, layer, x, (M + 1, K), None, None, u, tok)        # beyond the handle's batch
    s.Close()


def test_calls_that_would_allocate_are_refused_inside_a_capture_and_leave_it_valid(oracle, rocm, lin):
    # Three calls allocate on first use: per-row frequency penalties on a handle configured without any, a speculative
    # step larger than any before it, the first fused LM-head sampling call.  Inside a stream capture each is refused
    # with BORN_ROCM_ERR_UNSUPPORTED before it touches the stream, so the capture goes on: an ordinary sampling step
    # recorded after the refusals replays correctly.
    import ctypes as C
    from born_amd import _capi
    hip = C.CDLL("libamdhip64.so")
    def ok(rc):
        assert rc == 0, f"HIP error {rc}"
    rng = np.random.default_rng(405)
    B, K, V, G = 4, 128, 8000, 3
    xh = rng.standard_normal((B, V)).astype(np.float32)
    uh = rng.random(B, dtype=np.float32)
    hist_h = rng.integers(0, V, (B, 16)).astype(np.int32)
    logits, u, hist = rocm.DeviceBuffer.from_numpy(xh), rocm.DeviceBuffer.from_numpy(uh), rocm.DeviceBuffer.from_numpy(hist_h)
    tokens, probs = rocm.DeviceBuffer(B * 4), rocm.DeviceBuffer(B * 4)
    freqs = rocm.DeviceBuffer.from_numpy(np.full(B, 0.2, np.float32))
    w = rocm.DeviceBuffer.from_numpy((rng.standard_normal((V, K)) * 0.1).astype(np.float32))
    layer = lin.Linear(K, V, w, None)
    xin = rocm.DeviceBuffer.from_numpy(rng.standard_normal((B, K)).astype(np.float32))
    tgt = rocm.DeviceBuffer.from_numpy(rng.standard_normal((B, G, V)).astype(np.float32))
    dtok = rocm.DeviceBuffer.from_numpy(rng.integers(0, V, (B, G)).astype(np.int32))
    ua = rocm.DeviceBuffer.from_numpy(rng.random((B, G), dtype=np.float32))
    nacc, nxt = rocm.DeviceBuffer(B * 4), rocm.DeviceBuffer(B * 4)
    smp = rocm.NewSampler(rocm.SamplerConfig(Temperature=0.8, TopK=40, TopP=0.95, RepetitionPenalty=1.1), max_batch=B, max_vocab=V)

    stream = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(stream)))
    smp.Sample(logits, B, V, hist, None, u, tokens, probs, hist_stride=16, stream=stream)       # warm-up outside the capture
    ok(hip.hipStreamSynchronize(stream))
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(stream, 0))
    for call in (lambda: smp.SampleRows(logits, B, V, hist, None, u, None, None, None, None, tokens, probs, hist_stride=16, stream=stream,
                                        frequencyPenalties=freqs),
                 lambda: smp.Verify(tgt, tgt, B, G, V, dtok, ua, u, nacc, nxt, stream=stream),
                 lambda: lin.ForwardSample(smp, layer, xin, (B, K), hist, None, u, tokens, probs, hist_stride=16, stream=stream)):
        with pytest.raises(_capi.BornRocmError) as e:
            call()
        assert e.value.code == _capi.ERR_UNSUPPORTED and "capture" in str(e.value)
    smp.Sample(logits, B, V, hist, None, u, tokens, probs, hist_stride=16, stream=stream)
    ok(hip.hipStreamEndCapture(stream, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)))
    want = oracle.sample(xh, uh, 0.8, 40, 0.95, 1.1, hist_h, None, mode=oracle.MODE_FIXED)
    for it in range(2):
        _capi.check(_capi.lib().born_rocm_h2d(tokens.ptr, np.full(B, -1, np.int32).ctypes.data, 4 * B, None))
        ok(hip.hipDeviceSynchronize())
        ok(hip.hipGraphLaunch(gexec, stream))
        ok(hip.hipStreamSynchronize(stream))
        assert np.array_equal(tokens.to_numpy(np.int32, (B,)), want["tokens"]), it
    ok(hip.hipGraphExecDestroy(gexec))
    ok(hip.hipGraphDestroy(graph))
    ok(hip.hipStreamDestroy(stream))
    # outside a capture the same calls allocate and work
    smp.Verify(tgt, tgt, B, G, V, dtok, ua, u, nacc, nxt)
    assert nacc.to_numpy(np.int32, (B,)).tolist() == [G] * B                                # identical models accept everything
    smp.Status()
    smp.Close()
