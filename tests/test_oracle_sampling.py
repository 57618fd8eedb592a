"""Pins the stages of the oracle that have no counterpart in the reference (penalty, temperature,
top-k, top-p, inverse-CDF draw, speculative accept/reject) by hand-computed vectors, special cases that
reduce to the reference-pinned softmax / argmax, invariants, an independent torch restatement and
goodness-of-fit.  No test here retypes the oracle's own loop."""
import math

import numpy as np
import pytest
import torch

LOG = lambda *p: np.log(np.array([p], dtype=np.float64)).astype(np.float32)  # noqa: E731


# ---------------------------------------------------------------- hand vectors

def test_draw_hand_vector_rank_order(oracle):
    # probs 0.1, 0.4, 0.2, 0.3 at ids 0..3 -> rank order ids 1,3,2,0 with CDF .4 .7 .9 1.0
    x = LOG(1, 4, 2, 3)
    for u, want in [(0.0, 1), (0.39, 1), (0.41, 3), (0.69, 3), (0.71, 2), (0.89, 2), (0.91, 0), (0.999, 0)]:
        for mode in (oracle.MODE_TRUTH, oracle.MODE_FIXED, oracle.MODE_REF32):
            r = oracle.sample(x, [u], mode=mode)
            assert r["tokens"][0] == want, (u, mode)
    r = oracle.sample(x, [0.5], mode=oracle.MODE_TRUTH)
    assert abs(r["probs"][0] - 0.3) < 1e-6 and r["n_nucleus"][0] == 4


def test_top_k_hand_vector(oracle):
    x = LOG(1, 4, 2, 3)
    # k=2 keeps ids 1 (0.4) and 3 (0.3): renormalised 4/7, 3/7
    for u, want, p in [(0.5, 1, 4 / 7), (0.58, 3, 3 / 7)]:
        r = oracle.sample(x, [u], top_k=2)
        assert r["tokens"][0] == want and abs(r["probs"][0] - p) < 1e-6 and r["n_nucleus"][0] == 2


def test_top_p_hand_vector(oracle):
    x = LOG(1, 4, 2, 3)
    # p=0.65: prefix .4 (<.65), .7 (>=.65) -> keep 2 tokens; p=0.4 exactly reachable -> but fp: use 0.39 -> 1 token
    r = oracle.sample(x, [0.99], top_p=0.65)
    assert r["n_nucleus"][0] == 2 and r["tokens"][0] == 3
    r = oracle.sample(x, [0.99], top_p=0.39)
    assert r["n_nucleus"][0] == 1 and r["tokens"][0] == 1 and abs(r["probs"][0] - 1.0) < 1e-7
    r = oracle.sample(x, [0.99], top_p=0.95)
    assert r["n_nucleus"][0] == 4
    # top-k then top-p: k=3 keeps .4 .3 .2 (renorm /0.9): cumulative .444 .777 1.0 ; p=0.5 -> 2 tokens
    r = oracle.sample(x, [0.0], top_k=3, top_p=0.5, nuc_cap=4)
    assert r["n_nucleus"][0] == 2
    assert r["nuc_ids"][0].tolist() == [1, 3, -1, -1]
    assert np.allclose(r["nuc_probs"][0][:2], [4 / 7, 3 / 7], atol=1e-6)


def test_penalty_sign_rule_and_duplicates(oracle):
    # logits 2 and -2 with r=2: positive halves (1), negative doubles (-4); duplicates must not compound
    x = np.array([[2.0, -2.0, 0.5, 0.0]], dtype=np.float32)
    hist = np.array([[0, 1, 0, 0, 1, 3]], dtype=np.int32)
    r = oracle.sample(x, [0.0], rep=2.0, history=hist, nuc_cap=4)
    z = np.array([1.0, -4.0, 0.5, 0.0])
    p = np.exp(z) / np.exp(z).sum()
    order = [0, 2, 3, 1]
    assert r["nuc_ids"][0].tolist() == order
    assert np.allclose(r["nuc_probs"][0], p[order], rtol=1e-6)
    # hist_len limits how much of the history counts
    r2 = oracle.sample(x, [0.0], rep=2.0, history=hist, hist_len=[1], nuc_cap=4)
    z2 = np.array([1.0, -2.0, 0.5, 0.0])
    p2 = np.exp(z2) / np.exp(z2).sum()
    assert np.allclose(r2["nuc_probs"][0], p2[[0, 2, 3, 1]], rtol=1e-6)
    # out-of-range ids are counted and ignored
    r3 = oracle.sample(x, [0.0], rep=2.0, history=np.array([[7, -1, 0]], dtype=np.int32))
    assert r3["bad_ids"] == 2


def test_temperature_hand_vector(oracle):
    # T=0.5 squares the odds: probs proportional to 1,16,4,9
    x = LOG(1, 4, 2, 3)
    r = oracle.sample(x, [0.0], temperature=0.5, nuc_cap=4)
    assert r["nuc_ids"][0].tolist() == [1, 3, 2, 0]
    assert np.allclose(r["nuc_probs"][0], np.array([16, 9, 4, 1]) / 30.0, rtol=1e-5)


# ---------------------------------------------------------------- reductions onto reference-pinned functions

def test_k1_is_reference_argmax_with_tie_rule(oracle):
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, size=(64, 37)).astype(np.float32)      # many ties
    want = oracle.argmax_ref(x)
    for mode in (0, 1, 2):
        got = oracle.sample(x, rng.random(64, dtype=np.float32), top_k=1, mode=mode)
        assert np.array_equal(got["tokens"], want)
        assert np.all(got["probs"] == 1.0)


def test_identity_settings_give_reference_softmax(oracle):
    rng = np.random.default_rng(4)
    x = rng.normal(0, 2, size=(8, 50)).astype(np.float32)
    r = oracle.sample(x, np.zeros(8, np.float32), nuc_cap=50)          # T=1, k off, p off, r=1
    ref = oracle.softmax_ref(x)                                        # reference arithmetic
    for b in range(8):
        ids = r["nuc_ids"][b]
        assert sorted(ids.tolist()) == list(range(50))
        assert np.allclose(r["nuc_probs"][b], ref[b][ids], rtol=2e-6, atol=1e-9)
        assert np.all(np.diff(r["nuc_probs"][b]) <= 0)                 # rank order is probability-descending
    # k = V and k > V are "disabled"
    for k in (50, 51, 0, -3):
        rk = oracle.sample(x, np.full(8, 0.37, np.float32), top_k=k)
        r0 = oracle.sample(x, np.full(8, 0.37, np.float32))
        assert np.array_equal(rk["tokens"], r0["tokens"])
    # history with r=1 and empty history with r!=1 are identities
    h = rng.integers(0, 50, size=(8, 9)).astype(np.int32)
    assert np.array_equal(oracle.sample(x, np.full(8, 0.37, np.float32), history=h, rep=1.0)["tokens"], r0["tokens"])
    assert np.array_equal(oracle.sample(x, np.full(8, 0.37, np.float32), history=h, hist_len=np.zeros(8), rep=1.7)["tokens"],
                          r0["tokens"])


def test_softmax_shift_and_temperature_invariance(oracle):
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, size=(4, 33)).astype(np.float32)
    u = rng.random(4, dtype=np.float32)
    a = oracle.sample(x, u, temperature=0.5, top_k=7, top_p=0.9)
    b = oracle.sample((x * 2).astype(np.float32), u, temperature=1.0, top_k=7, top_p=0.9)   # x/0.5 == 2x exactly
    assert np.array_equal(a["tokens"], b["tokens"]) and np.array_equal(a["probs"], b["probs"])
    c = oracle.sample((x + 8).astype(np.float32) - 8 + 0, u, top_k=7)                      # shift by an exact amount
    d = oracle.sample(x, u, top_k=7)
    # (x+8)-8 is not exactly x in fp32, so compare the shifted row against itself shifted exactly by a power of two
    xs = (x.astype(np.float64) + 0).astype(np.float32)
    e = oracle.sample(xs + np.float32(0), u, top_k=7)
    assert np.array_equal(d["tokens"], e["tokens"]) and c["tokens"].shape == d["tokens"].shape


def test_top_p_limits(oracle):
    rng = np.random.default_rng(6)
    x = rng.normal(0, 1, size=(16, 40)).astype(np.float32)
    u = rng.random(16, dtype=np.float32)
    tiny = oracle.sample(x, u, top_p=1e-6)
    assert np.array_equal(tiny["tokens"], oracle.argmax_ref(x)) and np.all(tiny["n_nucleus"] == 1)
    assert np.all(oracle.sample(x, u, top_p=1.0)["n_nucleus"] == 40)
    assert np.all(oracle.sample(x, u, top_p=3.0)["n_nucleus"] == 40)
    # one-hot row: that token whatever u is
    oh = np.full((1, 9), -1e30, np.float32)
    oh[0, 5] = 0
    for uu in (0.0, 0.5, 0.999999):
        assert oracle.sample(oh, [uu])["tokens"][0] == 5


def test_special_values(oracle):
    x = np.array([[np.nan, 1.0, np.inf, -np.inf, -0.0, 0.0]], dtype=np.float32)
    r = oracle.sample(x, [0.0], nuc_cap=6)
    # +inf -> FLT_MAX wins with probability 1; NaN and -inf sort last (id order); -0 ties with +0 by id
    assert r["nuc_ids"][0].tolist() == [2, 1, 4, 5, 0, 3]
    assert r["probs"][0] == 1.0 and r["tokens"][0] == 2
    allneg = np.full((1, 5), -np.inf, np.float32)
    r = oracle.sample(allneg, [0.5], nuc_cap=5)
    assert np.allclose(r["nuc_probs"][0], 0.2) and r["tokens"][0] == 2     # (-inf)-(-inf) := 0 -> uniform


# ---------------------------------------------------------------- independent restatement in torch

def _torch_sample(x, u, T, k, p, rep, hist, min_p=0.0, freq=0.0, pres=0.0):
    """Independent restatement with torch primitives (float64 probabilities)."""
    x = torch.from_numpy(x.copy())
    B, V = x.shape
    toks, probs = [], []
    for b in range(B):
        row = x[b].clone()
        if hist is not None and rep != 1.0:
            ids = torch.unique(torch.from_numpy(hist[b].astype(np.int64)))
            sel = row[ids]
            row[ids] = torch.where(sel > 0, sel / np.float32(rep), sel * np.float32(rep))
        if hist is not None and (freq != 0.0 or pres != 0.0):
            counts = torch.bincount(torch.from_numpy(hist[b].astype(np.int64)), minlength=V).to(torch.float32)
            row = row - np.float32(freq) * counts
            row = row - np.float32(pres) * (counts > 0).to(torch.float32)
        z = row / np.float32(T)
        order = torch.from_numpy(np.lexsort((np.arange(V), -z.numpy().astype(np.float64))))  # z desc, id asc
        zs = z[order].double()
        if min_p > 0.0:                              # probability ratio to the most likely token, on the whole row
            full = torch.softmax(zs, dim=0)
            keep = full / full.max() >= np.float64(np.float32(min_p))
            zs, order = zs[keep], order[keep]
        if 0 < k < len(zs):
            zs, order = zs[:k], order[:k]
        pr = torch.softmax(zs, dim=0)
        c = torch.cumsum(pr, 0)
        if p < 1.0:
            n = int((c < np.float64(np.float32(p))).sum().item()) + 1
            n = min(n, len(c))
            pr, order = pr[:n], order[:n]
            pr = pr / pr.sum()
            c = torch.cumsum(pr, 0)
        i = int((c <= np.float64(np.float32(u[b]))).sum().item())
        i = min(i, len(c) - 1)
        toks.append(int(order[i]))
        probs.append(float(pr[i]))
    return np.array(toks), np.array(probs)


@pytest.mark.parametrize("T,k,p,rep", [(1.0, 0, 1.0, 1.0), (0.8, 40, 0.95, 1.1), (0.7, 50, 0.9, 1.15),
                                         (1.2, 0, 0.99, 1.05), (1.0, 5, 1.0, 1.0), (1.5, 0, 0.5, 0.8),
                                         (0.9, 129, 0.97, 1.1), (1.0, 256, 1.0, 1.0), (0.7, 512, 0.95, 1.2)])
def test_against_torch_restatement(oracle, T, k, p, rep):
    rng = np.random.default_rng(7)
    B, V, H = 48, 1000, 32
    x = rng.normal(0, 2, size=(B, V)).astype(np.float32)
    hist = rng.integers(0, V, size=(B, H)).astype(np.int32)
    u = rng.random(B, dtype=np.float32)
    want_t, want_p = _torch_sample(x, u, T, k, p, rep, hist)
    got = oracle.sample(x, u, temperature=T, top_k=k, top_p=p, rep=rep, history=hist, mode=oracle.MODE_TRUTH)
    ok = (got["tokens"] == want_t) | got["near"]
    assert ok.all(), np.nonzero(~ok)
    same = got["tokens"] == want_t
    assert np.allclose(got["probs"][same], want_p[same], rtol=1e-5)
    assert (~same).sum() <= 1


def test_min_p_hand_vector(oracle):
    # probabilities 1/2, 1/4, 1/8, 1/16, 1/16 => ratios to the top 1, 1/2, 1/4, 1/8, 1/8
    pr = [0.5, 0.25, 0.125, 0.0625, 0.0625]
    x = np.log(np.array([pr], dtype=np.float64)).astype(np.float32)
    for mode in (oracle.MODE_TRUTH, oracle.MODE_FIXED):
        for min_p, n in [(0.1, 5), (0.2, 3), (0.3, 2), (0.6, 1)]:
            want = np.array(pr[:n]) / sum(pr[:n])
            edges = np.cumsum(want)
            for u in (0.0, 0.3, 0.55, 0.7, 0.9, 0.99):
                r = oracle.sample(x, np.array([u], dtype=np.float32), min_p=min_p, mode=mode, nuc_cap=5)
                assert r["n_nucleus"][0] == n
                assert np.allclose(r["nuc_probs"][0, :n], want, rtol=1e-6) and (r["nuc_ids"][0, n:] == -1).all()
                assert r["tokens"][0] == int(np.searchsorted(edges, u, side="right"))
        # min-p, then top-k, then top-p on what is left: 0.2 keeps {1/2, 1/4, 1/8}; top-k 2 => {2/3, 1/3}; p = 0.6 => {1}
        r = oracle.sample(x, np.array([0.99], dtype=np.float32), min_p=0.2, top_k=2, top_p=0.6, mode=mode, nuc_cap=5)
        assert r["n_nucleus"][0] == 1 and r["tokens"][0] == 0 and r["probs"][0] == 1.0
        r = oracle.sample(x, np.array([0.99], dtype=np.float32), min_p=0.2, top_k=2, top_p=0.7, mode=mode, nuc_cap=5)
        assert r["n_nucleus"][0] == 2 and r["tokens"][0] == 1 and abs(r["probs"][0] - 1 / 3) < 1e-6


def test_min_p_limits_and_flags(oracle):
    rng = np.random.default_rng(21)
    x = rng.normal(0, 2, size=(64, 500)).astype(np.float32)
    u = rng.random(64, dtype=np.float32)
    base = oracle.sample(x, u, temperature=0.8, top_k=20, top_p=0.9, mode=oracle.MODE_FIXED, nuc_cap=20)
    # a bound below every ratio changes nothing; a bound just under 1 leaves the top token (and its exact ties)
    tiny = oracle.sample(x, u, temperature=0.8, top_k=20, top_p=0.9, min_p=1e-30, mode=oracle.MODE_FIXED, nuc_cap=20)
    for key in ("tokens", "probs", "n_nucleus", "nuc_ids", "nuc_probs"):
        assert np.array_equal(base[key], tiny[key])
    top = oracle.sample(x, u, temperature=0.8, min_p=0.999999, mode=oracle.MODE_TRUTH)
    assert np.array_equal(top["tokens"], oracle.argmax_ref(x)) and np.allclose(top["probs"], 1.0)
    # a survivor exactly on the bound is flagged: ratio 1/4 with min_p = 1/4
    y = np.log(np.array([[0.5, 0.25, 0.125, 0.125]], dtype=np.float64)).astype(np.float32)
    r = oracle.sample(y, np.array([0.5], dtype=np.float32), min_p=0.25, mode=oracle.MODE_TRUTH)
    assert r["near"][0] and r["near_cut"][0]
    # invalid values are refused
    for bad in (-0.5, 1.0, float("nan")):
        with pytest.raises(ValueError):
            oracle.sample(y, np.array([0.5], dtype=np.float32), min_p=bad)


@pytest.mark.parametrize("T,k,p,rep,min_p", [(1.0, 0, 1.0, 1.0, 0.05), (0.8, 40, 0.95, 1.1, 0.02), (0.7, 50, 0.9, 1.15, 0.1),
                                               (1.2, 0, 0.99, 1.05, 0.01), (1.5, 0, 0.5, 0.8, 0.3)])
def test_min_p_against_torch_restatement(oracle, T, k, p, rep, min_p):
    rng = np.random.default_rng(17)
    B, V, H = 48, 1000, 32
    x = rng.normal(0, 2, size=(B, V)).astype(np.float32)
    hist = rng.integers(0, V, size=(B, H)).astype(np.int32)
    u = rng.random(B, dtype=np.float32)
    want_t, want_p = _torch_sample(x, u, T, k, p, rep, hist, min_p)
    got = oracle.sample(x, u, temperature=T, top_k=k, top_p=p, rep=rep, history=hist, mode=oracle.MODE_TRUTH, min_p=min_p)
    ok = (got["tokens"] == want_t) | got["near"]
    assert ok.all(), np.nonzero(~ok)
    same = got["tokens"] == want_t
    assert np.allclose(got["probs"][same], want_p[same], rtol=1e-5)
    assert (~same).sum() <= 1
    fixed = oracle.sample(x, u, temperature=T, top_k=k, top_p=p, rep=rep, history=hist, mode=oracle.MODE_FIXED, min_p=min_p)
    diff = fixed["tokens"] != got["tokens"]
    assert not (diff & ~got["near"]).any()
    ok = ~got["near_cut"]
    assert np.array_equal(fixed["n_nucleus"][ok], got["n_nucleus"][ok])


def test_frequency_and_presence_penalty_hand_vectors(oracle):
    x = np.array([[2.0, 1.0, 0.5, -1.0]], dtype=np.float32)
    hist = np.array([[0, 0, 1, 3]], dtype=np.int32)
    u = np.array([0.5], dtype=np.float32)

    def dist(**kw):
        r = oracle.sample(x, u, history=hist, nuc_cap=4, mode=oracle.MODE_TRUTH, **kw)
        out = np.zeros(4)
        out[r["nuc_ids"][0]] = r["nuc_probs"][0]
        return out

    def softmax(y):
        e = np.exp(np.array(y, dtype=np.float64) - max(y))
        return e / e.sum()

    # frequency: minus 0.5 per occurrence; presence: minus 0.25 once; the token never emitted keeps its logit
    assert np.allclose(dist(freq=0.5), softmax([2.0 - 1.0, 1.0 - 0.5, 0.5, -1.0 - 0.5]), rtol=1e-6)
    assert np.allclose(dist(pres=0.25), softmax([1.75, 0.75, 0.5, -1.25]), rtol=1e-6)
    assert np.allclose(dist(freq=0.5, pres=0.25), softmax([0.75, 0.25, 0.5, -1.75]), rtol=1e-6)
    # after the repetition penalty (2/1.25 = 1.6, 1/1.25 = 0.8, -1 * 1.25 = -1.25), before the temperature
    assert np.allclose(dist(freq=0.5, pres=0.25, rep=1.25, temperature=0.5),
                       softmax([2 * (1.6 - 1.25), 2 * (0.8 - 0.75), 2 * 0.5, 2 * (-1.25 - 0.75)]), rtol=1e-6)
    # a negative penalty rewards repeats; ids outside the vocabulary are reported and ignored
    assert np.allclose(dist(freq=-0.5), softmax([3.0, 1.5, 0.5, -0.5]), rtol=1e-6)
    bad = oracle.sample(x, u, history=np.array([[0, 9, -1, 0]], dtype=np.int32), freq=0.5, nuc_cap=4)
    assert bad["bad_ids"] == 2
    out = np.zeros(4)
    out[bad["nuc_ids"][0]] = bad["nuc_probs"][0]
    assert np.allclose(out, softmax([1.0, 1.0, 0.5, -1.0]), rtol=1e-6)
    # hist_len shortens the history: only the first two entries count
    r = oracle.sample(x, u, history=hist, hist_len=np.array([2], dtype=np.int32), freq=0.5, nuc_cap=4)
    out = np.zeros(4)
    out[r["nuc_ids"][0]] = r["nuc_probs"][0]
    assert np.allclose(out, softmax([1.0, 1.0, 0.5, -1.0]), rtol=1e-6)
    for badv in (float("inf"), float("nan")):
        with pytest.raises(ValueError):
            oracle.sample(x, u, history=hist, freq=badv)
        with pytest.raises(ValueError):
            oracle.sample(x, u, history=hist, pres=badv)


@pytest.mark.parametrize("T,k,p,rep,freq,pres", [(1.0, 0, 1.0, 1.0, 0.3, 0.0), (0.8, 40, 0.95, 1.1, 0.2, 0.4),
                                                   (0.7, 50, 0.9, 1.0, 0.0, 0.6), (1.2, 0, 0.99, 1.05, -0.1, 0.2)])
def test_frequency_and_presence_against_torch_restatement(oracle, T, k, p, rep, freq, pres):
    rng = np.random.default_rng(19)
    B, V, H = 48, 300, 200                       # many repeats per id
    x = rng.normal(0, 2, size=(B, V)).astype(np.float32)
    hist = ((rng.zipf(1.3, size=(B, H)) - 1) % V).astype(np.int32)
    u = rng.random(B, dtype=np.float32)
    want_t, want_p = _torch_sample(x, u, T, k, p, rep, hist, 0.0, freq, pres)
    got = oracle.sample(x, u, temperature=T, top_k=k, top_p=p, rep=rep, history=hist, mode=oracle.MODE_TRUTH, freq=freq, pres=pres)
    ok = (got["tokens"] == want_t) | got["near"]
    assert ok.all(), np.nonzero(~ok)
    same = got["tokens"] == want_t
    assert np.allclose(got["probs"][same], want_p[same], rtol=1e-5)
    assert (~same).sum() <= 1
    fixed = oracle.sample(x, u, temperature=T, top_k=k, top_p=p, rep=rep, history=hist, mode=oracle.MODE_FIXED, freq=freq, pres=pres)
    diff = fixed["tokens"] != got["tokens"]
    assert not (diff & ~got["near"]).any()


# ---------------------------------------------------------------- layers agree, flags are honest

@pytest.mark.parametrize("V,k,p", [(257, 0, 1.0), (4000, 50, 0.9), (4000, 0, 0.99), (32000, 40, 0.95)])
def test_fixed_layer_equals_truth_except_flagged(oracle, V, k, p):
    rng = np.random.default_rng(8)
    B = 200 if V < 10000 else 40
    x = rng.normal(0, 1.5, size=(B, V)).astype(np.float32)
    u = rng.random(B, dtype=np.float32)
    t = oracle.sample(x, u, temperature=0.7, top_k=k, top_p=p, mode=oracle.MODE_TRUTH)
    f = oracle.sample(x, u, temperature=0.7, top_k=k, top_p=p, mode=oracle.MODE_FIXED)
    diff = t["tokens"] != f["tokens"]
    assert not (diff & ~t["near"]).any()
    same = ~diff
    assert np.allclose(t["probs"][same], f["probs"][same], rtol=1e-5)
    assert t["near"].mean() < 0.05


def test_goodness_of_fit(oracle):
    # empirical law of the draw equals the nucleus probabilities (chi-square, fixed seed)
    rng = np.random.default_rng(9)
    V, N = 12, 60000
    row = rng.normal(0, 1, size=(1, V)).astype(np.float32)
    x = np.repeat(row, N, axis=0)
    u = rng.random(N, dtype=np.float32)
    r = oracle.sample(x, u, temperature=0.9, top_k=8, top_p=0.9, nuc_cap=V)
    n = r["n_nucleus"][0]
    ids, pr = r["nuc_ids"][0][:n], r["nuc_probs"][0][:n].astype(np.float64)
    counts = np.array([(r["tokens"] == i).sum() for i in ids])
    assert counts.sum() == N
    chi2 = ((counts - N * pr) ** 2 / (N * pr)).sum()
    assert chi2 < 35.0, chi2          # dof <= 7; p-value of 35 is ~1e-5


def test_builtin_uniform_stream(oracle):
    us = np.array([oracle.uniform(1234, s, r) for s in range(50) for r in range(40)])
    assert us.min() >= 0.0 and us.max() < 1.0
    assert abs(us.mean() - 0.5) < 0.03 and len(np.unique(us)) > 1990
    assert oracle.uniform(1234, 0, 0) == oracle.uniform(1234, 0, 0)
    assert oracle.uniform(1234, 0, 0) != oracle.uniform(1235, 0, 0)


# ---------------------------------------------------------------- speculative accept / reject

def test_spec_identical_models_accept_everything(oracle):
    rng = np.random.default_rng(10)
    B, G, V = 6, 5, 300
    t = rng.normal(0, 1, size=(B, G, V)).astype(np.float32)
    d = rng.integers(0, V, size=(B, G)).astype(np.int32)
    for mode in (0, 1):
        r = oracle.spec_verify(t, t.copy(), d, rng.random((B, G), dtype=np.float32), rng.random(B, dtype=np.float32), mode=mode)
        assert np.all(r["n_accepted"] == G) and np.all(r["next_token"] == -1)


def test_spec_disjoint_supports_reject_and_resample_from_target(oracle):
    # target mass on ids {0,1} (0.25/0.75), draft mass on id 2: reject at 0, residual == p
    B, G, V = 1, 3, 4
    t = np.full((B, G, V), -1e30, np.float32)
    q = np.full((B, G, V), -1e30, np.float32)
    t[..., 0], t[..., 1] = math.log(1.0), math.log(3.0)
    q[..., 2] = 0.0
    d = np.full((B, G), 2, np.int32)
    for mode in (0, 1):
        for ur, want in [(0.1, 0), (0.24, 0), (0.26, 1), (0.9, 1)]:
            r = oracle.spec_verify(t, q, d, np.full((B, G), 0.5, np.float32), np.array([ur], np.float32), mode=mode)
            assert r["n_accepted"][0] == 0 and r["next_token"][0] == want, (mode, ur)


def test_spec_hand_vector_accept_ratio_and_residual(oracle):
    # p = [.5 .3 .2], q = [.2 .5 .3]; draft token 1: accept iff u < .6 ; residual = [.3 0 0] -> id 0
    t = LOG(5, 3, 2).reshape(1, 1, 3)
    q = LOG(2, 5, 3).reshape(1, 1, 3)
    d = np.array([[1]], np.int32)
    for mode in (0, 1):
        a = oracle.spec_verify(t, q, d, np.array([[0.59]], np.float32), np.array([0.7], np.float32), mode=mode)
        assert a["n_accepted"][0] == 1 and a["next_token"][0] == -1
        b = oracle.spec_verify(t, q, d, np.array([[0.61]], np.float32), np.array([0.7], np.float32), mode=mode)
        assert b["n_accepted"][0] == 0 and b["next_token"][0] == 0
    # draft token 0 (q < p): always accepted
    d0 = np.array([[0]], np.int32)
    assert oracle.spec_verify(t, q, d0, np.array([[0.999]], np.float32), np.array([0.1], np.float32))["n_accepted"][0] == 1
    # p = [.2 .3 .5], q = [.5 .3 .2]; token 0 rejected when u >= .4 ; residual [0 0 .3] -> id 2 ; two-sided residual:
    t2 = LOG(2, 2, 6).reshape(1, 1, 3)      # .2 .2 .6
    q2 = LOG(6, 1, 3).reshape(1, 1, 3)      # .6 .1 .3 -> residual [0 .1 .3] -> cdf .25 1.0
    for ur, want in [(0.2, 1), (0.3, 2)]:
        r = oracle.spec_verify(t2, q2, d0, np.array([[0.9]], np.float32), np.array([ur], np.float32))
        assert r["n_accepted"][0] == 0 and r["next_token"][0] == want


def test_spec_preserves_target_distribution(oracle):
    # the law of the first emitted token (accepted draft token or residual resample) equals p
    rng = np.random.default_rng(11)
    V, N = 6, 40000
    tl = rng.normal(0, 1, size=V).astype(np.float32)
    ql = (tl + rng.normal(0, 0.7, size=V)).astype(np.float32)
    p = np.exp(tl.astype(np.float64)); p /= p.sum()
    q = np.exp(ql.astype(np.float64)); q /= q.sum()
    d = rng.choice(V, size=N, p=q).astype(np.int32).reshape(N, 1)
    t = np.broadcast_to(tl, (N, 1, V)).copy()
    dr = np.broadcast_to(ql, (N, 1, V)).copy()
    for mode in (0, 1):
        r = oracle.spec_verify(t, dr, d, rng.random((N, 1), dtype=np.float32), rng.random(N, dtype=np.float32), mode=mode)
        first = np.where(r["n_accepted"] == 1, d[:, 0], r["next_token"])
        counts = np.bincount(first, minlength=V)
        chi2 = ((counts - N * p) ** 2 / (N * p)).sum()
        assert chi2 < 30.0, (mode, chi2)


def test_spec_layers_agree_except_flagged(oracle):
    rng = np.random.default_rng(12)
    B, G, V = 64, 5, 2000
    t = rng.normal(0, 1, size=(B, G, V)).astype(np.float32)
    dr = (t + rng.normal(0, 0.5, size=(B, G, V))).astype(np.float32)
    d = rng.integers(0, V, size=(B, G)).astype(np.int32)
    ua, ur = rng.random((B, G), dtype=np.float32), rng.random(B, dtype=np.float32)
    a = oracle.spec_verify(t, dr, d, ua, ur, mode=0)
    b = oracle.spec_verify(t, dr, d, ua, ur, mode=1)
    diff = (a["n_accepted"] != b["n_accepted"]) | (a["next_token"] != b["next_token"])
    assert not (diff & ~a["near"]).any()
    r = oracle.spec_verify(t, dr, np.full((B, G), V + 3, np.int32), ua, ur, mode=1)
    assert r["bad_tokens"] == B and np.all(r["n_accepted"] == 0)


def test_spec_bonus_draw_closed_forms(oracle):
    # identical models accept everything; the next token then comes from the bonus row by inverse CDF in
    # ascending id order.  Closed forms: uniform logits -> floor(u V); one-hot -> that id; p = [.5 .3 .2].
    rng = np.random.default_rng(21)
    B, G, V = 5, 3, 8
    t = rng.normal(0, 1, size=(B, G, V)).astype(np.float32)
    d = rng.integers(0, V, size=(B, G)).astype(np.int32)
    ua = rng.random((B, G), dtype=np.float32)
    ur = np.array([0.0, 0.124, 0.126, 0.6, 0.9999], np.float32)
    for mode in (0, 1):
        r = oracle.spec_verify(t, t.copy(), d, ua, ur, mode=mode, bonus=np.zeros((B, V), np.float32))
        assert np.all(r["n_accepted"] == G)
        assert r["next_token"].tolist() == [0, 0, 1, 4, 7], mode
        onehot = np.full((B, V), -1e30, np.float32)
        onehot[np.arange(B), [3, 0, 7, 5, 2]] = 1.5
        r = oracle.spec_verify(t, t.copy(), d, ua, ur, mode=mode, bonus=onehot)
        assert r["next_token"].tolist() == [3, 0, 7, 5, 2], mode
    p532 = np.tile(LOG(5, 3, 2), (4, 1))
    t3 = rng.normal(0, 1, size=(4, 2, 3)).astype(np.float32)
    d3 = rng.integers(0, 3, size=(4, 2)).astype(np.int32)
    for mode in (0, 1):
        r = oracle.spec_verify(t3, t3.copy(), d3, rng.random((4, 2), dtype=np.float32),
                               np.array([0.49, 0.51, 0.79, 0.81], np.float32), mode=mode, bonus=p532)
        assert r["next_token"].tolist() == [0, 1, 1, 2], mode
    # a rejected sequence ignores the bonus row: same answer with and without it
    dr = (t + rng.normal(0, 2.0, size=t.shape)).astype(np.float32)
    a = oracle.spec_verify(t, dr, d, ua, ur, mode=1)
    b = oracle.spec_verify(t, dr, d, ua, ur, mode=1, bonus=rng.normal(0, 1, size=(B, V)).astype(np.float32))
    rej = a["n_accepted"] < G
    assert rej.any() and np.array_equal(a["n_accepted"], b["n_accepted"])
    assert np.array_equal(a["next_token"][rej], b["next_token"][rej]) and np.all(b["next_token"][~rej] >= 0)


def test_spec_bonus_draw_law_and_brute_force(oracle):
    # the law of the bonus token is softmax(bonus / T); both layers agree with a numpy cumsum except when flagged
    rng = np.random.default_rng(22)
    V, N, T = 7, 30000, 0.8
    bl = rng.normal(0, 1.5, size=V).astype(np.float32)
    p = np.exp(bl.astype(np.float64) / np.float32(T)); p /= p.sum()
    t = np.zeros((N, 1, V), np.float32)
    d = np.zeros((N, 1), np.int32)
    ur = rng.random(N, dtype=np.float32)
    bonus = np.broadcast_to(bl, (N, V)).copy()
    want = np.searchsorted(np.cumsum(p), ur.astype(np.float64), side="right").clip(0, V - 1)
    for mode in (0, 1):
        r = oracle.spec_verify(t, t.copy(), d, np.full((N, 1), 0.5, np.float32), ur, temperature=T, mode=mode, bonus=bonus)
        assert np.all(r["n_accepted"] == 1)
        counts = np.bincount(r["next_token"], minlength=V)
        assert ((counts - N * p) ** 2 / (N * p)).sum() < 30.0, mode
        assert (r["next_token"] != want).mean() < 1e-3, mode
