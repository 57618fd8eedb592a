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
    dict(Temperature=0.9, TopK=300, TopP=0.9),                                              # the single-pass kernel's larger sizes
    dict(Temperature=0.9, TopK=700, TopP=0.9),                                              # the general kernel
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


def _hip():
    """The HIP runtime the library itself is linked against (already mapped into this process), through ctypes."""
    import ctypes as C
    _capi.lib()
    with open("/proc/self/maps") as f:
        paths = sorted({line.split()[-1] for line in f if "libamdhip64" in line})
    assert paths, "the HIP runtime is not mapped"
    hip = C.CDLL(paths[0])
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_char_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    return hip


@pytest.mark.parametrize("cfg_kw", [
    dict(Temperature=0.7, TopK=50, TopP=0.9, RepetitionPenalty=1.15),                       # the single-pass kernel
    dict(Temperature=1.2, TopP=0.95, RepetitionPenalty=1.05),                               # the three-sweep kernel
    dict(Temperature=0.9, TopK=600, TopP=0.9),                                              # the general kernel
])
def test_static_entry_point_allocates_nothing_and_can_be_captured(rocm, cfg_kw):
    """The property the entry point exists for.  (a) The device's free memory (hipMemGetInfo) is the same before and
    after two calls.  (b) After one warm call, a call is recorded into a HIP graph: an allocation, a free or a
    synchronisation inside the capture would invalidate it.  The graph is then replayed three times, with eager work
    (new uniforms uploaded, the handle-based call, synchronisations) between the replays, and every replay must equal
    the eager handle-based result for the uniforms it saw."""
    import ctypes as C
    S = rocm
    hip = _hip()
    cfg = S.SamplerConfig(**cfg_kw)
    B, V, H = 40, 12000, 64
    x, u, h = _rows(11, B, V, H)
    dx, dh, du = S.DeviceBuffer.from_numpy(x), S.DeviceBuffer.from_numpy(h), S.DeviceBuffer.from_numpy(u)
    tok_s, pr_s, tok_h, pr_h = (S.DeviceBuffer(4 * B) for _ in range(4))
    status = S.DeviceBuffer.from_numpy(np.zeros(1, np.int32))
    smp = S.NewSampler(cfg, max_batch=B, max_vocab=V)
    stream = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0                         # (default priority)

    def static_call(st):
        S.SampleStatic(cfg, dx, B, V, dh, None, du, tok_s, pr_s, status_out=status, hist_stride=H, stream=st)

    def free_bytes():
        free, total = C.c_size_t(), C.c_size_t()
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    static_call(stream)                                                      # the warm call: looks up the array's address
    assert hip.hipStreamSynchronize(stream) == 0
    # (a) nothing allocated, nothing freed
    before = free_bytes()
    static_call(stream)
    static_call(stream)
    assert hip.hipStreamSynchronize(stream) == 0
    assert free_bytes() == before
    # (b) under stream capture (mode 0 = global: an allocation by any thread invalidates the capture)
    graph, graph_exec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 0) == 0
    try:
        static_call(stream)
    finally:
        rc = hip.hipStreamEndCapture(stream, C.byref(graph))
    assert rc == 0 and graph.value, "the capture was invalidated"
    assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, 0) == 0
    rng = np.random.default_rng(5)
    poison = np.full(B, -7, np.int32)
    for replay in range(3):
        u_new = rng.random(B, dtype=np.float32)
        _capi.check(_capi.lib().born_rocm_h2d(du.ptr, u_new.ctypes.data, u_new.nbytes, None))      # eager work between the replays
        _capi.check(_capi.lib().born_rocm_h2d(tok_s.ptr, poison.ctypes.data, poison.nbytes, None))
        assert hip.hipGraphLaunch(graph_exec, stream) == 0
        assert hip.hipStreamSynchronize(stream) == 0
        smp.Sample(dx, B, V, dh, None, du, tok_h, pr_h, hist_stride=H)
        smp.Status()
        got, want = tok_s.to_numpy(np.int32, (B,)), tok_h.to_numpy(np.int32, (B,))
        assert np.array_equal(got, want), (replay, np.nonzero(got != want)[0][:8])
        assert np.array_equal(pr_s.to_numpy(np.uint32, (B,)), pr_h.to_numpy(np.uint32, (B,))), replay
    assert int(status.to_numpy(np.int32, (1,))[0]) == 0
    hip.hipGraphExecDestroy(graph_exec)
    hip.hipGraphDestroy(graph)
    hip.hipStreamDestroy(stream)
    smp.Close()
