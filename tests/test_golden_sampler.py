"""The committed sampler vectors (tests/golden/sampler_fixtures.json, written by tests/golden/make_sampler_fixtures.py
from the CPU oracle's fixed-point and fp64 layers): the CPU test checks that the oracle still reproduces them, the GPU
test that the HIP path (through the C ABI) reproduces the fixed-point layer bit for bit and agrees with the fp64 layer
except on rows that layer flags as drawn within 1e-6 of a CDF step."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _load():
    with open(os.path.join(HERE, "golden", "sampler_fixtures.json")) as f:
        return json.load(f)


FIX = _load()
CASES = FIX["cases"]


def _f32(bits, shape=None):
    a = np.array(bits, dtype=np.uint32).view(np.float32)
    return a.reshape(shape) if shape is not None else a


def _tensor(name, shape):
    return _f32(FIX["tensors"][name], shape)


def _sample_inputs(c):
    x = _tensor(c["logits"], c["shape"])
    u = _f32(c["uniforms_bits"])
    h = None if c["history"] is None else np.array(c["history"], dtype=np.int32)
    hl = None if c["hist_len"] is None else np.array(c["hist_len"], dtype=np.int32)
    return x, u, h, hl


@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "sample"], ids=lambda c: c["name"])
def test_oracle_reproduces_the_sampling_vectors(oracle, c):
    x, u, h, hl = _sample_inputs(c)
    kw = dict(temperature=c["temperature"], top_k=c["top_k"], top_p=c["top_p"], rep=c["repetition_penalty"], history=h, hist_len=hl,
              min_p=c["min_p"], freq=c["frequency_penalty"], pres=c["presence_penalty"], nuc_cap=c["nucleus_cap"])
    fx = oracle.sample(x, u, mode=oracle.MODE_FIXED, **kw)
    tr = oracle.sample(x, u, mode=oracle.MODE_TRUTH, **kw)
    assert fx["tokens"].tolist() == c["fixed"]["tokens"]
    assert fx["probs"].view(np.uint32).tolist() == c["fixed"]["probs_bits"]
    assert fx["n_nucleus"].tolist() == c["fixed"]["n_nucleus"]
    assert tr["tokens"].tolist() == c["truth"]["tokens"]
    assert tr["probs"].view(np.uint32).tolist() == c["truth"]["probs_bits"]
    if c["nucleus_cap"]:
        assert fx["nuc_ids"].tolist() == c["fixed"]["nuc_ids"]
        assert fx["nuc_probs"].ravel().view(np.uint32).tolist() == c["fixed"]["nuc_probs_bits"]


@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "spec"], ids=lambda c: c["name"])
def test_oracle_reproduces_the_speculative_vectors(oracle, c):
    B, G, V = c["shape"]
    t, d = _tensor(c["target"], (B, G, V)), _tensor(c["draft"], (B, G, V))
    bonus = None if c["bonus"] is None else _tensor(c["bonus"], (B, V))
    dt = np.array(c["draft_tokens"], dtype=np.int32)
    ua, ur = _f32(c["u_accept_bits"], (B, G)), _f32(c["u_residual_bits"])
    for layer, mode in (("fixed", oracle.MODE_FIXED), ("truth", oracle.MODE_TRUTH)):
        got = oracle.spec_verify(t, d, dt, ua, ur, c["temperature"], mode=mode, bonus=bonus)
        assert got["n_accepted"].tolist() == c[layer]["n_accepted"]
        assert got["next_token"].tolist() == c[layer]["next_token"]


@pytest.mark.gpu
@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "sample"], ids=lambda c: c["name"])
def test_hip_path_reproduces_the_sampling_vectors(c):
    from born_amd import sampler as S
    x, u, h, hl = _sample_inputs(c)
    B, V = x.shape
    smp = S.NewSampler(S.SamplerConfig(Temperature=c["temperature"], TopK=c["top_k"], TopP=c["top_p"],
                                       RepetitionPenalty=c["repetition_penalty"], MinP=c["min_p"],
                                       FrequencyPenalty=c["frequency_penalty"], PresencePenalty=c["presence_penalty"]),
                       max_batch=B, max_vocab=V)
    listed = c["nucleus_cap"] if 1 <= c["top_k"] <= 4096 else 0
    for path in (0, 1):                                             # the configuration's own kernel, then the general one
        smp.SetPath(path)
        got = S.sample_host(smp, x, u, h, hl, nucleus_cap=listed)
        smp.Status()
        assert got["tokens"].tolist() == c["fixed"]["tokens"], path
        assert got["probs"].view(np.uint32).tolist() == c["fixed"]["probs_bits"], path
        if listed:
            assert got["n_nucleus"].tolist() == c["fixed"]["n_nucleus"]
            assert got["nuc_ids"].tolist() == c["fixed"]["nuc_ids"]
            assert got["nuc_probs"].ravel().view(np.uint32).tolist() == c["fixed"]["nuc_probs_bits"]
        near = np.array(c["truth"]["near"], dtype=bool)
        diff = got["tokens"] != np.array(c["truth"]["tokens"])
        assert not (diff & ~near).any(), "token differs from the fp64 layer on a row it does not flag"
        same = ~diff
        want = _f32(c["truth"]["probs_bits"])
        assert np.allclose(got["probs"][same], want[same], rtol=1e-5, atol=0)
    smp.Close()


@pytest.mark.gpu
@pytest.mark.parametrize("c", [c for c in CASES if c["kind"] == "spec"], ids=lambda c: c["name"])
def test_hip_path_reproduces_the_speculative_vectors(c):
    from born_amd import sampler as S
    B, G, V = c["shape"]
    t, d = _tensor(c["target"], (B, G, V)), _tensor(c["draft"], (B, G, V))
    dt = np.array(c["draft_tokens"], dtype=np.int32)
    ua, ur = _f32(c["u_accept_bits"], (B, G)), _f32(c["u_residual_bits"])
    smp = S.NewSampler(S.SamplerConfig(Temperature=c["temperature"]), max_batch=B, max_vocab=V)
    if c["bonus"] is None:
        got = S.verify_host(smp, t, d, dt, ua, ur)
    else:                                                           # the target scored one more position: the bonus rows
        t1 = np.concatenate([t, _tensor(c["bonus"], (B, 1, V))], axis=1)
        got = S.verify_host(smp, t1, d, dt, ua, ur, bonus=True)
    smp.Status()
    smp.Close()
    assert got["n_accepted"].tolist() == c["fixed"]["n_accepted"]
    assert got["next_token"].tolist() == c["fixed"]["next_token"]
