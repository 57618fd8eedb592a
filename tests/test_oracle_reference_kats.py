"""Pins the reference-following part of the oracle against the known-answer vectors the
reference's own tests hold (tests/golden/reference_kats.json: data only)."""
import json
import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_kats.json")) as f:
    KATS = json.load(f)


def _expected(case):
    if "expected" in case:
        return np.array(case["expected"], dtype=np.float64)
    expr = case["expected_expr"]
    if expr in ("exp_ratio", "exp_ratio_of_1_2_3"):
        e = [math.exp(1.0), math.exp(2.0), math.exp(3.0)]
        s = sum(e)
        return np.array([[np.float32(v / s) for v in e]], dtype=np.float64)
    if expr == "1,e,e*e":
        return np.array([1.0, np.float32(math.e), np.float32(math.e * math.e)], dtype=np.float64)
    raise KeyError(expr)


def test_softmax_kats(oracle):
    for case in KATS["softmax"]:
        x = np.array(case["input"], dtype=np.float32)
        # ops_test.go exercises softmaxFloat32; cross_entropy_test.go exercises the exp(logSoftmax) form
        fns = (oracle.softmax_ref, oracle.softmax_f64)
        if "cross_entropy_test.go" in case["source"]:
            fns = (oracle.softmax_via_log_ref,) + fns
        for fn in fns:
            out = np.asarray(fn(x), dtype=np.float64)
            if "expected" in case or "expected_expr" in case:
                assert np.max(np.abs(out - _expected(case))) <= case["tol_abs"], (case["source"], fn.__name__)
            if "sum_tol" in case:
                assert abs(out.sum() - 1.0) <= case["sum_tol"]
            if case.get("finite"):
                assert np.all(np.isfinite(out))


def test_log_softmax_kats(oracle):
    for case in KATS["log_softmax"]:
        x = np.array(case["input"], dtype=np.float32)
        out = oracle.log_softmax_ref(x).astype(np.float64)
        if "expected" in case:
            assert np.max(np.abs(out - np.array(case["expected"]))) <= case["tol_abs"], case["source"]
        if case.get("finite"):
            assert np.all(np.isfinite(out))
            loss = -out[0, case["target"]]
            assert 0.0 <= loss <= case["max_loss"]


def check_cross_entropy_case(case, loss_of):
    """Asserts what the reference's test asserts; `loss_of(x, targets)` raises ValueError where the reference panics."""
    import pytest
    x = np.array(case["input"], dtype=np.float32)
    t = np.array(case["targets"], dtype=np.int32)
    if case.get("panics"):
        with pytest.raises(ValueError, match="target index out of bounds"):
            loss_of(x, t)
        return
    loss = float(loss_of(x, t))
    if "expected" in case:
        assert abs(loss - case["expected"]) < case["tol_abs"], case["source"]
    if case.get("finite"):
        assert math.isfinite(loss), case["source"]
    if "min" in case:
        assert loss >= case["min"], case["source"]
    if "min_exclusive" in case:
        assert loss > case["min_exclusive"], case["source"]
    if "max" in case:
        assert loss <= case["max"], case["source"]
    if "equals_first_row_alone_within" in case:
        assert abs(loss - float(loss_of(x[:1], t[:1]))) <= case["equals_first_row_alone_within"], case["source"]


def test_cross_entropy_kats(oracle):
    for case in KATS["cross_entropy"]:
        check_cross_entropy_case(case, oracle.cross_entropy_ref)


def test_cross_entropy_and_token_logprobs_against_what_the_mathematics_fixes(oracle):
    from scipy.special import logsumexp
    rng = np.random.default_rng(41)
    B, V = 40, 777
    x = (rng.standard_normal((B, V)) * 3.0).astype(np.float32)
    t = rng.integers(0, V, B).astype(np.int32)
    want = x.astype(np.float64)[np.arange(B), t] - logsumexp(x.astype(np.float64), axis=1)      # an independent routine
    # the reference arithmetic: the gather of its own logSoftmax, bit for bit, and its mean
    ref = oracle.log_softmax_ref(x)[np.arange(B), t]
    lp2, bad = oracle.token_logprobs(x, t, mode=oracle.MODE_REF32)
    assert bad == 0 and np.array_equal(lp2.view(np.uint32), ref.view(np.uint32))
    total = np.float32(0.0)
    for v in ref:
        total = np.float32(total + np.float32(-v))
    assert oracle.cross_entropy_ref(x, t) == float(np.float32(total / np.float32(B)))
    assert abs(oracle.cross_entropy_ref(x, t) - float(-want.mean())) < 1e-5
    # closed forms: uniform rows give -log V; a two-class row gives -log(1 + e^-gap)
    assert abs(oracle.cross_entropy_ref(np.zeros((3, 50), np.float32), np.array([0, 7, 49], np.int32)) - math.log(50.0)) < 1e-6
    assert abs(oracle.cross_entropy_ref(np.array([[0.5, -1.0]], np.float32), np.array([0], np.int32)) - math.log1p(math.exp(-1.5))) < 1e-6
    # the three layers agree with the independent routine
    for mode, tol in ((oracle.MODE_TRUTH, 2e-6), (oracle.MODE_FIXED, 2e-6), (oracle.MODE_REF32, 2e-5)):
        lp, _ = oracle.token_logprobs(x, t, mode=mode)
        assert np.max(np.abs(lp - want)) < tol, mode
    # temperature and penalties: z is what the sampling pipeline ranks, so exp(logprob) of a sampled token is the
    # probability the untruncated sampler reports for it
    hist = ((rng.zipf(1.3, size=(B, 60)) - 1) % V).astype(np.int32)
    u = rng.random(B, dtype=np.float32)
    kw = dict(temperature=0.7, rep=1.2, history=hist, freq=0.3, pres=0.2)
    for mode in (oracle.MODE_TRUTH, oracle.MODE_FIXED):
        smp = oracle.sample(x, u, mode=mode, **kw)
        lp, _ = oracle.token_logprobs(x, smp["tokens"], mode=mode, **kw)
        assert np.allclose(np.exp(lp.astype(np.float64)), smp["probs"], rtol=2e-6)
    # an explicit hand case: logits [2, 1, 0], history [0, 0]: rep 2 -> 1; minus 0.25 * 2 -> 0.5; minus 0.5 -> 0; T = 0.5 -> z = [0, 2, 0]
    lp, _ = oracle.token_logprobs(np.array([[2.0, 1.0, 0.0]], np.float32), np.array([0], np.int32), temperature=0.5, rep=2.0,
                                  history=np.array([[0, 0]], np.int32), freq=0.25, pres=0.5)
    assert abs(lp[0] - (0.0 - math.log(2.0 + math.exp(2.0)))) < 1e-6
    # special rows: nothing finite -> every token ties (-log V); a masked token -> -inf; a token outside the vocabulary -> NaN, counted
    y = np.full((3, 8), -np.inf, dtype=np.float32)
    y[1, 2] = 0.0
    y[2, :] = 1.0
    for mode in (oracle.MODE_TRUTH, oracle.MODE_FIXED, oracle.MODE_REF32):
        lp, bad = oracle.token_logprobs(y, np.array([3, 5, 8], np.int32), mode=mode)
        assert abs(lp[0] + math.log(8.0)) < 1e-6 and lp[1] == -np.inf and np.isnan(lp[2]) and bad == 1, mode
        lp, _ = oracle.token_logprobs(y, np.array([0, 2, 0], np.int32), mode=mode)
        assert lp[1] == 0.0 and abs(lp[2] + math.log(8.0)) < 1e-6


def test_argmax_kats(oracle):
    for case in KATS["argmax"]:
        x = np.array(case["input"], dtype=np.float32)
        assert oracle.argmax_ref(x).tolist() == case["expected"], case["source"]


def test_argmax_tie_rule_and_nan(oracle):
    # internal/nn/cross_entropy.go:245 uses strict '>' scanning upward: lowest index wins ties,
    # NaN never wins unless it is at index 0.
    x = np.array([[5, 5, 5], [1, 7, 7], [np.nan, 9, 1], [1, np.nan, 0], [-np.inf, -np.inf, -np.inf]], dtype=np.float32)
    assert oracle.argmax_ref(x).tolist() == [0, 1, 0, 0, 0]


def test_exp_kats(oracle):
    for case in KATS["exp"]:
        x = np.array(case["input"], dtype=np.float32)
        out = oracle.exp_ref(x).astype(np.float64)
        assert np.max(np.abs(out - _expected(case))) <= case["tol_abs"]


def test_extreme_logits(oracle):
    for case in KATS["cross_entropy_extremes"]:
        x = np.array(case["input"], dtype=np.float32)
        p = oracle.softmax_ref(x)
        assert oracle.argmax_ref(x)[0] == case["argmax"]
        assert p[0, case["argmax"]] >= case["p_argmax_min"]
        ls = oracle.log_softmax_ref(x)
        assert -ls[0, case["argmax"]] < 0.1          # PerfectPrediction: loss near 0
        assert -ls[0, 2] > 10.0                      # WorstPrediction: loss high


def test_row_independence(oracle):
    # internal/autodiff/ops/cross_entropy_test.go:168-195: a batch of identical rows gives the single-row result
    x1 = np.array([[1.0, 2.0, 3.0]], dtype=np.float32)
    x2 = np.repeat(x1, 2, axis=0)
    assert np.array_equal(oracle.softmax_ref(x2)[0], oracle.softmax_ref(x1)[0])
    assert np.array_equal(oracle.softmax_ref(x2)[1], oracle.softmax_ref(x1)[0])


def test_expneg_accuracy_and_edges(oracle):
    d = np.concatenate([np.linspace(0, 80, 4001), np.random.default_rng(1).uniform(0, 40, 4000)]).astype(np.float32)
    got = oracle.expneg(d).astype(np.float64)
    want = np.exp(-d.astype(np.float64))
    rel = np.abs(got - want) / want
    assert rel.max() < 4e-7, rel.max()
    assert oracle.expneg(np.float32(0.0))[0] == 1.0
    assert oracle.expneg(np.float32(80.5))[0] == 0.0
    assert oracle.expneg(np.float32(np.inf))[0] == 0.0
    # monotone non-increasing on a dense grid (a sign slip in the range reduction breaks this)
    g = oracle.expneg(np.linspace(0, 30, 20001).astype(np.float32))
    assert np.all(np.diff(g) <= 0)


def test_matmul_kats(oracle):
    for case in KATS["matmul"]:
        a = np.array(case["a"], dtype=np.float32)
        b = np.array(case["b"], dtype=np.float32)
        out = oracle.matmul_ref(a, b).astype(np.float64)
        assert out.shape == (a.shape[0], b.shape[1])
        assert np.max(np.abs(out - np.array(case["expected"], dtype=np.float64))) <= case["tol_abs"], case["source"]


def test_linear_kats(oracle):
    for case in KATS["linear"]:
        x = np.array(case["x"], dtype=np.float32)
        w = np.array(case["weight"], dtype=np.float32)
        bias = None if case["bias"] is None else np.array(case["bias"], dtype=np.float32)
        out = oracle.linear_ref(x, w, bias).astype(np.float64)
        assert out.shape == (x.shape[0], w.shape[0])
        assert np.max(np.abs(out - np.array(case["expected"], dtype=np.float64))) <= case["tol_abs"], case["source"]


def test_matmul_and_linear_against_what_the_mathematics_fixes(oracle):
    # Checks a transposed operand, a dropped bias, a wrong pitch or a dropped k-term would fail:
    # non-square shapes against an fp64 product, the transposition identity, bias as a rank-1 update.
    rng = np.random.default_rng(7)
    for (m, k, n) in [(1, 1, 1), (3, 5, 7), (7, 3, 5), (16, 33, 9), (5, 257, 11)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        c = oracle.matmul_ref(a, b)
        c64 = a.astype(np.float64) @ b.astype(np.float64)
        bound = (k + 1) * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64))
        assert np.all(np.abs(c - c64) <= bound), (m, k, n)
        # integer-valued operands: every partial sum is exact in fp32
        ai = rng.integers(-8, 9, (m, k)).astype(np.float32)
        bi = rng.integers(-8, 9, (k, n)).astype(np.float32)
        assert np.array_equal(oracle.matmul_ref(ai, bi), (ai.astype(np.int64) @ bi.astype(np.int64)).astype(np.float32))
        # Linear.Forward is MatMul with the transposed weight (same k order, so bit for bit), plus the bias
        w = np.ascontiguousarray(b.T)
        bias = rng.standard_normal(n).astype(np.float32)
        assert np.array_equal(oracle.linear_ref(a, w, None), c)
        assert np.array_equal(oracle.linear_ref(a, w, bias), c + bias[None, :])


def test_binary_reshape_transpose_kats(oracle):
    for case in KATS["binary"]:
        a = np.array(case["a"], dtype=np.float32).reshape(case["a_shape"])
        b = np.array(case["b"], dtype=np.float32).reshape(case["b_shape"])
        out = oracle.binary_ref(case["op"], a, b)
        assert list(out.shape) == case["shape"], case["source"]
        assert out.ravel().tolist() == case["expected"], case["source"]
    for case in KATS["transpose"]:
        x = np.array(case["data"], dtype=np.float32).reshape(case["shape"])
        out = oracle.transpose_ref(x, case["axes"])
        assert list(out.shape) == case["out_shape"] and out.ravel().tolist() == case["expected"], case["source"]
    for case in KATS["reshape"]:          # a reshape keeps the row-major element order: nothing to restate beyond the copy
        x = np.array(case["data"], dtype=np.float32).reshape(case["shape"])
        assert x.reshape(case["new_shape"]).ravel().tolist() == case["expected"], case["source"]


def test_binary_and_transpose_against_numpy(oracle):
    # NumPy's broadcasting and transpose are the library routines these operations reduce to; a wrong stride,
    # a swapped operand or an inverted permutation fails on non-square, non-commutative cases
    import pytest
    rng = np.random.default_rng(3)
    shapes = [((4, 5), (4, 5)), ((4, 5), (5,)), ((4, 1), (5,)), ((1,), (3, 2)), ((2, 3, 4), (3, 1)), ((2, 1, 4), (5, 1)),
              ((3, 1, 2, 1), (4, 1, 5)), ((), (2, 3)), ((2, 3), ()), ((6,), (1, 1, 6))]
    fns = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    for sa, sb in shapes:
        a = rng.standard_normal(sa).astype(np.float32)
        b = (rng.standard_normal(sb) + 3.0).astype(np.float32)
        for op, fn in fns.items():
            want = fn(a, b)
            got = oracle.binary_ref(op, a, b)
            assert got.shape == want.shape and np.array_equal(got.view(np.uint32), want.view(np.uint32)), (op, sa, sb)
    with pytest.raises(ValueError):
        oracle.binary_ref("add", np.zeros((2, 3), np.float32), np.zeros((4,), np.float32))
    for shape, axes in [((2, 3), None), ((2, 3, 4), None), ((2, 3, 4), (0, 2, 1)), ((2, 3, 4), (1, 0, 2)), ((2, 3, 4, 5), (3, 1, 0, 2)),
                        ((7,), None), ((1, 5), (1, 0))]:
        x = rng.standard_normal(shape).astype(np.float32)
        assert np.array_equal(oracle.transpose_ref(x, axes), np.transpose(x, axes)), (shape, axes)
    with pytest.raises(ValueError):
        oracle.transpose_ref(np.zeros((2, 3), np.float32), (0, 0))


def test_conv2d_and_maxpool2d_kats(oracle):
    for case in KATS["conv2d"]:
        x = np.array(case["x"], dtype=np.float32).reshape(case["x_shape"])
        k = np.array(case["k"], dtype=np.float32).reshape(case["k_shape"])
        out = oracle.conv2d_ref(x, k, case["stride"], case["padding"])
        assert list(out.shape) == case["shape"] and out.ravel().tolist() == case["expected"], case["source"]
    for case in KATS["maxpool2d"]:
        x = np.array(case["x"], dtype=np.float32).reshape(case["x_shape"])
        out = oracle.maxpool2d_ref(x, case["kernel"], case["stride"])
        assert list(out.shape) == case["shape"], case["source"]
        if "expected" in case:
            assert out.ravel().tolist() == case["expected"], case["source"]
        else:
            assert out.ravel()[0] == case["expected_first"], case["source"]


def test_conv2d_and_maxpool2d_against_independent_restatements(oracle):
    # conv2d as an explicit cross-correlation sum in fp64 over padded input (numpy), maxpool as a windowed max:
    # a swapped kernel axis, a flipped kernel, a wrong stride or padding offset fails on asymmetric cases
    rng = np.random.default_rng(17)
    for (N, C, H, W, CO, KH, KW, stride, pad) in [(2, 3, 7, 9, 4, 3, 2, 1, 0), (1, 2, 8, 8, 3, 3, 3, 2, 1), (3, 1, 5, 6, 2, 2, 4, 1, 2),
                                                  (1, 4, 6, 5, 5, 1, 1, 1, 0), (2, 2, 9, 7, 1, 5, 3, 3, 2)]:
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        k = rng.standard_normal((CO, C, KH, KW)).astype(np.float32)
        got = oracle.conv2d_ref(x, k, stride, pad)
        xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pad, pad), (pad, pad)))
        HO, WO = (H + 2 * pad - KH) // stride + 1, (W + 2 * pad - KW) // stride + 1
        want = np.zeros((N, CO, HO, WO))
        for oh in range(HO):
            for ow in range(WO):
                patch = xp[:, :, oh * stride:oh * stride + KH, ow * stride:ow * stride + KW]
                want[:, :, oh, ow] = np.einsum("nchw,ochw->no", patch, k.astype(np.float64))
        assert got.shape == want.shape
        assert np.max(np.abs(got - want)) <= 1e-5 * max(1.0, np.max(np.abs(want))), (N, C, H, W, CO, KH, KW, stride, pad)
    for (N, C, H, W, ks, stride) in [(2, 3, 8, 8, 2, 2), (1, 2, 7, 9, 3, 1), (2, 1, 6, 5, 2, 3), (1, 1, 4, 4, 4, 1)]:
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        got = oracle.maxpool2d_ref(x, ks, stride)
        HO, WO = (H - ks) // stride + 1, (W - ks) // stride + 1
        want = np.empty((N, C, HO, WO), np.float32)
        for oh in range(HO):
            for ow in range(WO):
                want[:, :, oh, ow] = x[:, :, oh * stride:oh * stride + ks, ow * stride:ow * stride + ks].max(axis=(2, 3))
        assert np.array_equal(got, want)
    # the reference's floor of -1e38 and its treatment of NaN (never greater)
    x = np.full((1, 1, 2, 2), -np.inf, np.float32)
    assert oracle.maxpool2d_ref(x, 2, 1).ravel()[0] == np.float32(-1e38)
    x = np.array([[[[np.nan, 1.0], [2.0, np.nan]]]], np.float32)
    assert oracle.maxpool2d_ref(x, 2, 1).ravel()[0] == 2.0
