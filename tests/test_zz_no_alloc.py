"""born_rocm_sample_static (the sampling step for callers that cannot allocate) against born_rocm_sample, through the
C ABI: tokens and probabilities must be equal bit for bit, on two calls in a row that share the library's fixed
workspace, the second over a smaller batch and vocabulary; then the limits it states."""
import numpy as np
import pytest

from born_amd import _capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rocm():
    from born_amd import sampler as S
    assert S.DeviceCount() >= 1, "no HIP device visible"
    return S


def _rows(seed, B, V, H):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((B, V)) * 1.5).astype(np.float32)
    for b in range(B):
        x[b, rng.choice(V, 8, replace=False)] += rng.uniform(6, 12, 8).astype(np.float32)
    u = rng.random(B, dtype=np.float32)
    h = rng.integers(0, V, size=(B, H)).astype(np.int32) if H else None
    if h is not None:
        top = np.argsort(-x, axis=1)[:, :H // 2]                   # half the history are tokens the row would favour
        h[:, :H // 2] = top
    return x, u, h


def _both(rocm, cfg, x, u, h):
    S = rocm
    B, V = x.shape
    H = 0 if h is None else h.shape[1]
    dx, du = S.DeviceBuffer.from_numpy(x), S.DeviceBuffer.from_numpy(u)
    dh = S.DeviceBuffer.from_numpy(h) if h is not None else None
    tok_a, pr_a, tok_b, pr_b = (S.DeviceBuffer(4 * B) for _ in range(4))
    st = S.DeviceBuffer.from_numpy(np.zeros(1, np.int32))
    smp = S.NewSampler(cfg, max_batch=B, max_vocab=V)
    smp.Sample(dx, B, V, dh, None, du, tok_a, pr_a, hist_stride=H)
    try:
        smp.Status()
        handle_status = 0
    except _capi.BornRocmError as e:
        assert e.code == _capi.ERR_DATA
        handle_status = 1
    S.SampleStatic(cfg, dx, B, V, dh, None, du, tok_b, pr_b, status_out=st, hist_stride=H)
    got = (tok_a.to_numpy(np.int32, (B,)), pr_a.to_numpy(np.float32, (B,)), tok_b.to_numpy(np.int32, (B,)),
           pr_b.to_numpy(np.float32, (B,)), int(st.to_numpy(np.int32, (1,))[0]))
    assert (got[4] != 0) == (handle_status != 0), "the two entry points disagree about the data error"
    smp.Close()
    return got


@pytest.mark.parametrize("cfg_kw", [
    dict(Temperature=0.7, TopK=50, TopP=0.9, RepetitionPenalty=1.15),                       # the single-pass kernel
    dict(Temperature=1.2, TopP=0.95, RepetitionPenalty=1.05),                               # no top-k cut: the three-sweep kernel
    dict(Temperature=0.9, TopK=300, TopP=0.9),                                              # the general kernel
    dict(Temperature=0.8, TopK=40, TopP=0.95, FrequencyPenalty=0.3, PresencePenalty=0.2),   # occurrences counted in the kernel
])
def test_static_entry_point_equals_the_handle_one_on_two_calls_in_a_row(rocm, oracle, cfg_kw):
    cfg = rocm.SamplerConfig(**cfg_kw)
    for seed, (B, V, H) in enumerate([(48, 20000, 96), (5, 4102, 32)]):      # the second call: smaller, ragged vocabulary
        x, u, h = _rows(100 + seed, B, V, H)
        tok_a, pr_a, tok_b, pr_b, status = _both(rocm, cfg, x, u, h)
        assert np.array_equal(tok_a, tok_b), (B, V, np.nonzero(tok_a != tok_b)[0][:8])
        assert np.array_equal(pr_a.view(np.uint32), pr_b.view(np.uint32))
        assert status == 0
        # and both equal the oracle's fixed-point layer
        fx = oracle.sample(x, u, cfg_kw.get("Temperature", 1.0), cfg_kw.get("TopK", 0), cfg_kw.get("TopP", 1.0),
                           cfg_kw.get("RepetitionPenalty", 1.0), h, None, mode=oracle.MODE_FIXED,
                           freq=cfg_kw.get("FrequencyPenalty", 0.0), pres=cfg_kw.get("PresencePenalty", 0.0))
        assert np.array_equal(tok_b, fx["tokens"])
        assert np.array_equal(pr_b.view(np.uint32), fx["probs"].view(np.uint32))


def test_static_entry_point_reports_bad_history_ids_in_the_callers_word(rocm):
    cfg = rocm.SamplerConfig(Temperature=0.7, TopK=50, TopP=0.9, RepetitionPenalty=1.15)
    x, u, h = _rows(7, 4, 5000, 16)
    h[2, 3] = 5000                                                           # one id outside the vocabulary
    *_, status = _both(rocm, cfg, x, u, h.copy())
    assert status & 1
    h[2, 3] = 0
    *_, status = _both(rocm, cfg, x, u, h)
    assert status == 0


def test_static_entry_point_limits(rocm):
    S = rocm
    x, u, _ = _rows(3, 2, 1000, 0)
    dx, du, tok = S.DeviceBuffer.from_numpy(x), S.DeviceBuffer.from_numpy(u), S.DeviceBuffer(8)
    with pytest.raises(_capi.BornRocmError) as e:                            # more rows than the fixed workspace holds
        S.SampleStatic(S.SamplerConfig(TopK=5), dx, 4097, 1000, None, None, du, tok)
    assert e.value.code == _capi.ERR_UNSUPPORTED and "4096" in str(e.value)
    with pytest.raises(S.SamplerPanic):                                      # the built-in uniform stream needs a handle
        S.SampleStatic(S.SamplerConfig(TopK=5), dx, 2, 1000, None, None, None, tok)
    h = S.DeviceBuffer.from_numpy(np.zeros((2, 5000), np.int32))
    with pytest.raises(_capi.BornRocmError) as e:                            # counting a 5000-token history needs the table
        S.SampleStatic(S.SamplerConfig(TopK=5, FrequencyPenalty=0.5), dx, 2, 1000, h, None, du, tok, hist_stride=5000)
    assert e.value.code == _capi.ERR_UNSUPPORTED


@pytest.mark.parametrize("cfg_kw", [
    dict(Temperature=0.7, TopK=50, TopP=0.9, RepetitionPenalty=1.15),                       # the single-pass kernel
    dict(Temperature=1.2, TopP=0.95, RepetitionPenalty=1.05),                               # the three-sweep kernel
    dict(Temperature=0.9, TopK=300, TopP=0.9),                                              # the general kernel
])
def test_static_entry_point_allocates_nothing_and_can_be_captured(rocm, cfg_kw):
    """The property the entry point exists for.  (a) The device's free memory (hipMemGetInfo, read through torch) is the
    same before and after two calls.  (b) A call is recorded into a HIP graph after one warm call: an allocation, a free
    or a synchronisation inside the capture would invalidate it.  The graph is then replayed three times, with eager
    work (new uniforms uploaded, the handle-based call, synchronisations) between the replays, and every replay must
    equal the eager handle-based result for the uniforms it saw."""
    import torch
    S = rocm
    cfg = S.SamplerConfig(**cfg_kw)
    B, V, H = 40, 12000, 64
    x, u, h = _rows(11, B, V, H)
    dev = torch.device("cuda:0")
    tx, th = torch.from_numpy(x).to(dev), torch.from_numpy(h).to(dev)
    tu = torch.from_numpy(u).to(dev)
    tok_s = torch.full((B,), -7, dtype=torch.int32, device=dev)
    pr_s = torch.zeros(B, device=dev)
    tok_h = torch.empty(B, dtype=torch.int32, device=dev)
    pr_h = torch.empty(B, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    smp = S.NewSampler(cfg, max_batch=B, max_vocab=V)
    cur = lambda: torch.cuda.current_stream().cuda_stream

    def static_call():
        S.SampleStatic(cfg, tx, B, V, th, None, tu, tok_s, pr_s, status_out=status, hist_stride=H, stream=cur())

    static_call()                                                            # the warm call: looks up the array's address
    torch.cuda.synchronize()
    # (a) nothing allocated, nothing freed
    free_before = torch.cuda.mem_get_info()[0]
    static_call()
    static_call()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    # (b) under stream capture
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.graph(graph, stream=side):
        static_call()
    rng = np.random.default_rng(5)
    for replay in range(3):
        u_new = rng.random(B, dtype=np.float32)
        tu.copy_(torch.from_numpy(u_new))                                    # eager work between the replays
        tok_s.fill_(-7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        smp.Sample(tx, B, V, th, None, tu, tok_h, pr_h, hist_stride=H, stream=cur())
        torch.cuda.synchronize()
        assert torch.equal(tok_s, tok_h), (replay, (tok_s != tok_h).nonzero().flatten()[:8].tolist())
        assert torch.equal(pr_s.view(torch.int32), pr_h.view(torch.int32)), replay
    assert int(status.item()) == 0
    smp.Close()
