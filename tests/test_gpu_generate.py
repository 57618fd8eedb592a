"""The generation loop (born_amd/generate.py) against a host loop built from the oracle: embedding lookup, LM head,
sampling with the built-in uniform stream, history append.  Embedding and head hold small integers, so every logit
is exact in fp32 whatever the order of the k-sum, and the device's token sequences must equal the oracle's."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rocm():
    from born_amd import sampler as S
    assert S.DeviceCount() >= 1, "no HIP device visible"
    return S


def _host_loop(oracle, E, W, bias, prompts, steps, seed, cfg):
    seqs = [list(p) for p in prompts]
    B = len(seqs)
    for t in range(steps):
        cur = np.array([s[-1] for s in seqs], dtype=np.int32)
        logits = oracle.linear_ref(E[cur], W, bias)
        H = max(len(s) for s in seqs)
        hist = np.zeros((B, H), dtype=np.int32)
        for b, s in enumerate(seqs):
            hist[b, :len(s)] = s
        lens = np.array([len(s) for s in seqs], dtype=np.int32)
        u = np.array([oracle.uniform(seed, t, b) for b in range(B)], dtype=np.float32)
        r = oracle.sample(logits, u, cfg["T"], cfg["k"], cfg["p"], cfg["rep"], hist, lens, mode=oracle.MODE_FIXED, min_p=cfg["min_p"],
                          freq=cfg["freq"], pres=cfg["pres"])
        for b in range(B):
            seqs[b].append(int(r["tokens"][b]))
    return seqs


@pytest.mark.parametrize("cfg", [
    dict(T=0.8, k=40, p=0.95, rep=1.1, min_p=0.0, freq=0.0, pres=0.0),
    dict(T=1.0, k=0, p=0.9, rep=1.0, min_p=0.02, freq=0.3, pres=0.2),
    dict(T=0.7, k=200, p=1.0, rep=1.3, min_p=0.0, freq=0.0, pres=0.5),
    dict(T=1.0, k=1, p=1.0, rep=1.5, min_p=0.0, freq=0.0, pres=0.0),              # greedy with a penalty: no repeats while it bites
])
def test_generation_loop_equals_the_host_loop(oracle, rocm, cfg):
    from born_amd import linear as L
    from born_amd.generate import Generator
    rng = np.random.default_rng(11)
    V, K, B, steps, seed = 5003, 64, 6, 24, 99
    E = rng.integers(-2, 3, (V, K)).astype(np.float32)
    W = rng.integers(-2, 3, (V, K)).astype(np.float32)
    bias = rng.integers(-3, 4, V).astype(np.float32)
    prompts = [list(rng.integers(0, V, int(rng.integers(1, 9)))) for _ in range(B)]
    smp = rocm.NewSampler(rocm.SamplerConfig(Temperature=cfg["T"], TopK=cfg["k"], TopP=cfg["p"], RepetitionPenalty=cfg["rep"], Seed=seed,
                                             MinP=cfg["min_p"], FrequencyPenalty=cfg["freq"], PresencePenalty=cfg["pres"]),
                          max_batch=B, max_vocab=V)
    head = L.Linear(K, V, rocm.DeviceBuffer.from_numpy(W), rocm.DeviceBuffer.from_numpy(bias))
    gen = Generator(rocm.DeviceBuffer.from_numpy(E), V, K, head, smp, max_batch=B, max_len=64)
    got = gen.Generate(prompts, steps)
    want = _host_loop(oracle, E, W, bias, prompts, steps, seed, cfg)
    for b in range(B):
        assert got[b].tolist() == want[b], (b, got[b].tolist(), want[b])
    smp.Close()


def test_history_append_and_gather_rows(rocm):
    rng = np.random.default_rng(12)
    s = rocm.NewSampler(max_batch=8, max_vocab=100)
    B, S = 5, 4
    hist = rng.integers(0, 100, (B, S)).astype(np.int32)
    lens = np.array([0, 1, 3, 4, 2], np.int32)
    tok = np.array([7, 8, 9, 10, 100], np.int32)                          # row 3 is full, row 4's token is outside the vocabulary
    d_h, d_l, d_t = (rocm.DeviceBuffer.from_numpy(a) for a in (hist, lens, tok))
    s.HistoryAppend(d_h, d_l, S, d_t, B, 100)
    h2, l2 = d_h.to_numpy(np.int32, (B, S)), d_l.to_numpy(np.int32, (B,))
    want = hist.copy()
    want[0, 0], want[1, 1], want[2, 3] = 7, 8, 9
    assert np.array_equal(h2, want) and l2.tolist() == [1, 2, 4, 4, 2]
    with pytest.raises(rocm.BornRocmError, match="full history row"):
        s.Status()
    # gather: aligned and unaligned widths, strided tables, an id outside the table
    for cols, ld in [(64, 64), (63, 70), (4, 8), (1, 1)]:
        table = rng.standard_normal((50, ld)).astype(np.float32)
        ids = np.array([0, 49, 7, 7, 50, -1], np.int32)
        out = rocm.DeviceBuffer(4 * len(ids) * cols)
        s.GatherRows(rocm.DeviceBuffer.from_numpy(table), 50, cols, rocm.DeviceBuffer.from_numpy(ids), len(ids), out, row_stride=ld)
        got = out.to_numpy(np.float32, (len(ids), cols))
        assert np.array_equal(got[:4], table[[0, 49, 7, 7], :cols]) and not got[4:].any()
        with pytest.raises(rocm.BornRocmError):
            s.Status()
    with pytest.raises(rocm.SamplerPanic, match="gather_rows"):
        s.GatherRows(None, 5, 5, d_t, 1, d_h)
    with pytest.raises(rocm.SamplerPanic, match="history_append"):
        s.HistoryAppend(d_h, d_l, 0, d_t, B, 100)
    s.Close()
