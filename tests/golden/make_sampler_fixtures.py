#!/usr/bin/env python3
"""Writes tests/golden/sampler_fixtures.json: small sampling and speculative-verify cases (inputs and expected
outputs) produced by the CPU oracle's two layers (fp64 truth, fixed point).  The file is committed, so that the
GPU box checks the HIP path against vectors that were not produced by a fresh CPU run there, and the CPU suite
checks that the oracle still reproduces them.

Usage: python tests/golden/make_sampler_fixtures.py      (from the repository root; rewrites the JSON)

Floats are stored as their fp32 bit patterns (uint32), so that the comparison is exact."""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import pyoracle as O  # noqa: E402


TENSORS = {}                                  # large inputs are stored once and referred to by name


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).tolist()


def tensor_ref(a):
    b = bits(np.ravel(a))
    for name, have in TENSORS.items():
        if have == b:
            return name
    name = f"t{len(TENSORS)}"
    TENSORS[name] = b
    return name


def sampling_case(name, x, u, T=1.0, k=0, p=1.0, rep=1.0, hist=None, hist_len=None, min_p=0.0, freq=0.0, pres=0.0, nuc=0):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = np.ascontiguousarray(u, dtype=np.float32)
    kw = dict(temperature=T, top_k=k, top_p=p, rep=rep, history=hist, hist_len=hist_len, min_p=min_p, freq=freq, pres=pres, nuc_cap=nuc)
    fx = O.sample(x, u, mode=O.MODE_FIXED, **kw)
    tr = O.sample(x, u, mode=O.MODE_TRUTH, **kw)
    case = {"name": name, "kind": "sample", "shape": list(x.shape), "logits": tensor_ref(x), "uniforms_bits": bits(u),
            "temperature": T, "top_k": k, "top_p": p, "repetition_penalty": rep, "min_p": min_p, "frequency_penalty": freq,
            "presence_penalty": pres, "nucleus_cap": nuc,
            "history": None if hist is None else np.asarray(hist, dtype=np.int32).tolist(),
            "hist_len": None if hist_len is None else np.asarray(hist_len, dtype=np.int32).tolist(),
            "fixed": {"tokens": fx["tokens"].tolist(), "probs_bits": bits(fx["probs"]), "n_nucleus": fx["n_nucleus"].tolist()},
            "truth": {"tokens": tr["tokens"].tolist(), "probs_bits": bits(tr["probs"]), "near": tr["near"].astype(int).tolist()}}
    if nuc:
        case["fixed"]["nuc_ids"] = fx["nuc_ids"].tolist()
        case["fixed"]["nuc_probs_bits"] = bits(fx["nuc_probs"].ravel())
    return case


def spec_case(name, target, draft, dt, ua, ur, T=1.0, bonus=None):
    fx = O.spec_verify(target, draft, dt, ua, ur, T, mode=O.MODE_FIXED, bonus=bonus)
    tr = O.spec_verify(target, draft, dt, ua, ur, T, mode=O.MODE_TRUTH, bonus=bonus)
    return {"name": name, "kind": "spec", "shape": list(target.shape), "target": tensor_ref(target), "draft": tensor_ref(draft),
            "bonus": None if bonus is None else tensor_ref(bonus),
            "draft_tokens": np.asarray(dt, dtype=np.int32).tolist(), "u_accept_bits": bits(np.ravel(ua)), "u_residual_bits": bits(ur),
            "temperature": T,
            "fixed": {"n_accepted": fx["n_accepted"].tolist(), "next_token": fx["next_token"].tolist()},
            "truth": {"n_accepted": tr["n_accepted"].tolist(), "next_token": tr["next_token"].tolist(), "near": tr["near"].astype(int).tolist()}}


def main():
    rng = np.random.default_rng(20251125)
    cases = []
    V = 37
    x = (rng.standard_normal((6, V)) * 2.0).astype(np.float32)
    u = rng.random(6, dtype=np.float32)
    hist = rng.integers(0, V, size=(6, 9)).astype(np.int32)
    cases.append(sampling_case("temperature alone", x, u, T=0.7))
    cases.append(sampling_case("top-k alone", x, u, k=5))
    cases.append(sampling_case("top-p alone", x, u, p=0.8))
    cases.append(sampling_case("repetition penalty alone, ragged histories", x, u, rep=1.3, hist=hist, hist_len=np.array([0, 1, 9, 4, 9, 2], np.int32)))
    cases.append(sampling_case("every stage, nucleus listed", x, u, T=0.8, k=12, p=0.9, rep=1.15, hist=hist, nuc=12))
    cases.append(sampling_case("min-p with frequency and presence penalties", x, u, T=0.9, k=20, p=0.95, min_p=0.05, freq=0.3, pres=0.2, hist=hist))
    # ties: equal logits across the top-k cut and inside the nucleus (lowest id first)
    t = np.full((4, V), -1.0, dtype=np.float32)
    t[:, [3, 7, 11, 19, 23]] = 2.0
    t[:, [5, 6]] = 2.5
    cases.append(sampling_case("ties across the cuts", t, np.array([0.0, 0.35, 0.7, 0.999], np.float32), k=4, p=0.9, nuc=8))
    # masked rows: -inf logits, a row with one finite logit, a row with nothing finite (uniform by definition), NaN as -inf
    m = (rng.standard_normal((4, V))).astype(np.float32)
    m[0, ::2] = -np.inf
    m[1, :] = -np.inf
    m[1, 17] = 0.25
    m[2, :] = -np.inf
    m[3, 5] = np.nan
    cases.append(sampling_case("masked rows", m, np.array([0.5, 0.9, 0.5, 0.1], np.float32), T=1.1, k=8, p=0.9))
    cases.append(sampling_case("masked rows, no top-k cut", m, np.array([0.5, 0.9, 0.5, 0.1], np.float32), T=1.1, p=0.9))
    cases.append(sampling_case("greedy limit: top-k 1", x, u, k=1))
    wide = (rng.standard_normal((2, 4102)) * 1.5).astype(np.float32)          # a ragged vocabulary, several waves wide
    wh = rng.integers(0, 4102, size=(2, 40)).astype(np.int32)
    cases.append(sampling_case("ragged vocabulary, top-k 50 + top-p", wide, rng.random(2, dtype=np.float32), T=0.7, k=50, p=0.9, rep=1.15, hist=wh))
    cases.append(sampling_case("ragged vocabulary, top-p without a top-k cut", wide, rng.random(2, dtype=np.float32), T=1.2, p=0.99, rep=1.05, hist=wh))
    cases.append(sampling_case("ragged vocabulary, top-k 300 (the general kernel)", wide, rng.random(2, dtype=np.float32), T=0.9, k=300, p=0.9))
    # speculative accept / reject
    B, G, Vs = 5, 4, 53
    tg = rng.standard_normal((B, G, Vs)).astype(np.float32)
    dr = (tg + 0.5 * rng.standard_normal((B, G, Vs))).astype(np.float32)
    dt = rng.integers(0, Vs, size=(B, G)).astype(np.int32)
    dt[0] = np.argmax(tg[0], axis=1)                                          # likely accepted
    ua = rng.random((B, G), dtype=np.float32)
    ua[0] = 0.01
    ur = rng.random(B, dtype=np.float32)
    cases.append(spec_case("speculative step", tg, dr, dt, ua, ur, T=1.0))
    cases.append(spec_case("speculative step, temperature 0.8, bonus rows", tg, dr, dt, ua, ur, T=0.8,
                           bonus=rng.standard_normal((B, Vs)).astype(np.float32)))
    cases.append(spec_case("identical models accept everything", tg, tg.copy(), dt, ua, ur, T=1.0))
    out = {"_comment": "Written by tests/golden/make_sampler_fixtures.py from the CPU oracle (layers: fixed point, fp64 truth). "
                       "Floats are fp32 bit patterns. No upstream Born sampler exists to compare with: these vectors freeze "
                       "docs/SAMPLING_SPEC.md as the oracle implements it.",
           "tensors": TENSORS, "cases": cases}
    path = os.path.join(HERE, "sampler_fixtures.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
        f.write("\n")
    print(f"wrote {path}: {len(cases)} cases, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
