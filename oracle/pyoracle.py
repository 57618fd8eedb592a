"""ctypes loader for the CPU oracle (oracle/libborn_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  The product package (born_amd/) never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libborn_oracle.so")

MODE_TRUTH = 0      # layer T: fp64
MODE_FIXED = 1      # layer F: fixed-point realisation (bit-exact target of the HIP kernels)
MODE_REF32 = 2      # reference arithmetic (timed CPU baseline only)


def build(force=False):
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "born_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libborn_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        f32p, i32p, u8p, f64p, u64p = (C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_uint8),
                                      C.POINTER(C.c_double), C.POINTER(C.c_uint64))
        i64p = C.POINTER(C.c_int64)
        L.born_oracle_expneg.restype = C.c_float
        L.born_oracle_expneg.argtypes = [C.c_float]
        L.born_oracle_mass_shift.restype = C.c_int
        L.born_oracle_mass_shift.argtypes = [C.c_int64]
        L.born_oracle_uniform.restype = C.c_float
        L.born_oracle_uniform.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
        for name in ("born_oracle_softmax_f32", "born_oracle_log_softmax_f32", "born_oracle_softmax_via_log"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [f32p, f32p, C.c_int64, C.c_int64]
        L.born_oracle_argmax.restype = None
        L.born_oracle_argmax.argtypes = [f32p, C.c_int64, C.c_int64, C.c_int64, i32p]
        L.born_oracle_exp_f32.restype = None
        L.born_oracle_exp_f32.argtypes = [f32p, f32p, C.c_int64]
        L.born_oracle_matmul_f32.restype = None
        L.born_oracle_matmul_f32.argtypes = [f32p, f32p, f32p, C.c_int64, C.c_int64, C.c_int64]
        L.born_oracle_linear_f32.restype = None
        L.born_oracle_linear_f32.argtypes = [f32p, f32p, f32p, f32p, C.c_int64, C.c_int64, C.c_int64]
        L.born_oracle_binary_f32.restype = C.c_int
        L.born_oracle_binary_f32.argtypes = [C.c_int, f32p, i64p, C.c_int, f32p, i64p, C.c_int, f32p, i64p]
        L.born_oracle_transpose_f32.restype = C.c_int
        L.born_oracle_transpose_f32.argtypes = [f32p, i64p, C.c_int, i32p, f32p]
        L.born_oracle_conv2d_f32.restype = C.c_int
        L.born_oracle_conv2d_f32.argtypes = [f32p] + [C.c_int64] * 4 + [f32p] + [C.c_int64] * 6 + [f32p]
        L.born_oracle_maxpool2d_f32.restype = C.c_int
        L.born_oracle_maxpool2d_f32.argtypes = [f32p] + [C.c_int64] * 6 + [f32p]
        L.born_oracle_softmax_f64.restype = None
        L.born_oracle_softmax_f64.argtypes = [f32p, f64p, C.c_int64, C.c_int64, C.c_int64]
        L.born_oracle_sample.restype = C.c_int64
        L.born_oracle_sample.argtypes = [f32p, C.c_int64, C.c_int64, C.c_int64, i32p, i32p, C.c_int64, f32p,
                                         C.c_float, C.c_int32, C.c_float, C.c_float, C.c_int32,
                                         i32p, f32p, u8p, i32p, C.c_int64, i32p, f32p]
        L.born_oracle_sample_ex.restype = C.c_int64
        L.born_oracle_sample_ex.argtypes = [f32p, C.c_int64, C.c_int64, C.c_int64, i32p, i32p, C.c_int64, f32p,
                                               C.c_float, C.c_int32, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int32,
                                            i32p, f32p, u8p, i32p, C.c_int64, i32p, f32p]
        L.born_oracle_token_logprobs.restype = C.c_int64
        L.born_oracle_token_logprobs.argtypes = [f32p, C.c_int64, C.c_int64, C.c_int64, i32p, i32p, C.c_int64, i32p,
                                                 C.c_float, C.c_float, C.c_float, C.c_float, C.c_int32, f32p]
        L.born_oracle_cross_entropy_f32.restype = C.c_int
        L.born_oracle_cross_entropy_f32.argtypes = [f32p, C.c_int64, C.c_int64, i32p, f32p]
        L.born_oracle_spec_verify.restype = C.c_int64
        L.born_oracle_spec_verify.argtypes = [f32p, f32p, C.c_int64, C.c_int64, C.c_int64, i32p, f32p, f32p,
                                              C.c_float, C.c_int32, i32p, i32p, u8p]
        L.born_oracle_spec_bonus_draw.restype = None
        L.born_oracle_spec_bonus_draw.argtypes = [f32p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, f32p, C.c_float,
                                                  C.c_int32, i32p, i32p, u8p]
        L.born_oracle_row_stats.restype = None
        L.born_oracle_row_stats.argtypes = [f32p, C.c_int64, C.c_int64, C.c_int64, C.c_float, f32p, u64p]
        _lib = L
    return _lib


def _p(a, ct):
    return None if a is None else a.ctypes.data_as(C.POINTER(ct))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def expneg(d):
    d = _f32(np.atleast_1d(d))
    out = np.empty_like(d)
    L = lib()
    for i, v in enumerate(d.ravel()):
        out.ravel()[i] = L.born_oracle_expneg(float(v))
    return out


def uniform(seed, step, row):
    return lib().born_oracle_uniform(int(seed) & (2**64 - 1), int(step), int(row))


def softmax_ref(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().born_oracle_softmax_f32(_p(x, C.c_float), _p(out, C.c_float), x.shape[0], x.shape[1])
    return out


def log_softmax_ref(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().born_oracle_log_softmax_f32(_p(x, C.c_float), _p(out, C.c_float), x.shape[0], x.shape[1])
    return out


def softmax_via_log_ref(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().born_oracle_softmax_via_log(_p(x, C.c_float), _p(out, C.c_float), x.shape[0], x.shape[1])
    return out


def softmax_f64(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.float64)
    lib().born_oracle_softmax_f64(_p(x, C.c_float), _p(out, C.c_double), x.shape[0], x.shape[1], x.shape[1])
    return out


def argmax_ref(x):
    x = _f32(x)
    out = np.empty(x.shape[0], dtype=np.int32)
    lib().born_oracle_argmax(_p(x, C.c_float), x.shape[0], x.shape[1], x.shape[1], _p(out, C.c_int32))
    return out


def exp_ref(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().born_oracle_exp_f32(_p(x, C.c_float), _p(out, C.c_float), x.size)
    return out


def matmul_ref(a, b):
    """The reference's naive fp32 MatMul: [m,k] @ [k,n], sequential k-sum per element."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2, "matmul: shape mismatch"
    c = np.empty((m, n), dtype=np.float32)
    lib().born_oracle_matmul_f32(_p(c, C.c_float), _p(a, C.c_float), _p(b, C.c_float), m, k, n)
    return c


def linear_ref(x, w, bias=None):
    """The reference's Linear.Forward: x[batch,in] @ w[out,in]^T + bias[out]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    batch, fin = x.shape
    fout, fin2 = w.shape
    assert fin == fin2, "linear: shape mismatch"
    bp = None
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
        assert bias.shape == (fout,)
        bp = _p(bias, C.c_float)
    y = np.empty((batch, fout), dtype=np.float32)
    lib().born_oracle_linear_f32(_p(y, C.c_float), _p(x, C.c_float), _p(w, C.c_float), bp, batch, fin, fout)
    return y


def binary_ref(op, a, b):
    """The reference's Add/Sub/Mul/Div ("add", "sub", "mul", "div") with broadcasting; raises ValueError when
    the shapes do not broadcast (where the reference panics)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    nd = max(a.ndim, b.ndim)
    ash = np.array(a.shape if a.ndim else [], dtype=np.int64)
    bsh = np.array(b.shape if b.ndim else [], dtype=np.int64)
    osh = np.zeros(max(nd, 1), dtype=np.int64)
    # the result is allocated at the largest size the rule can produce, then cut to the shape returned
    cap = 1
    for i in range(nd):
        ad = a.shape[a.ndim - 1 - i] if i < a.ndim else 1
        bd = b.shape[b.ndim - 1 - i] if i < b.ndim else 1
        cap *= max(ad, bd)
    out = np.empty(cap, dtype=np.float32)
    rc = lib().born_oracle_binary_f32(["add", "sub", "mul", "div"].index(op), _p(a, C.c_float), _p(ash, C.c_int64), a.ndim,
                                      _p(b, C.c_float), _p(bsh, C.c_int64), b.ndim, _p(out, C.c_float), _p(osh, C.c_int64))
    if rc != 0:
        raise ValueError(f"{op}: shapes not compatible for broadcasting: {list(a.shape)} vs {list(b.shape)}")
    shape = tuple(int(d) for d in osh[:nd])
    return out[:int(np.prod(shape, dtype=np.int64)) if nd else 1].reshape(shape)


def transpose_ref(x, axes=None):
    """The reference's Transpose (axes None: reverse all dimensions); raises ValueError on a bad permutation."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    sh = np.array(x.shape if x.ndim else [], dtype=np.int64)
    ax = None if axes is None else np.array(list(axes), dtype=np.int32)
    if ax is not None and len(ax) != x.ndim:
        raise ValueError(f"transpose: axes length {len(ax)} != ndim {x.ndim}")
    out = np.empty(x.size, dtype=np.float32)
    rc = lib().born_oracle_transpose_f32(_p(x, C.c_float), _p(sh, C.c_int64), x.ndim, None if ax is None else _p(ax, C.c_int32),
                                         _p(out, C.c_float))
    if rc != 0:
        raise ValueError("transpose: invalid permutation")
    order = list(range(x.ndim - 1, -1, -1)) if axes is None else list(axes)
    return out.reshape(tuple(x.shape[i] for i in order))


def conv2d_ref(x, k, stride=1, padding=0):
    """The reference's Conv2D: x [N,C,H,W], k [CO,C,KH,KW]; raises ValueError where the reference panics."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    if x.ndim != 4 or k.ndim != 4:
        raise ValueError("conv2d: input and kernel must be 4D")
    N, Cc, H, W = x.shape
    CO, CK, KH, KW = k.shape
    HO, WO = (H + 2 * padding - KH) // stride + 1, (W + 2 * padding - KW) // stride + 1
    out = np.empty((N, CO, max(HO, 1), max(WO, 1)), dtype=np.float32)
    rc = lib().born_oracle_conv2d_f32(_p(x, C.c_float), N, Cc, H, W, _p(k, C.c_float), CO, CK, KH, KW, stride, padding, _p(out, C.c_float))
    if rc != 0:
        raise ValueError("conv2d: invalid arguments")
    return out.reshape(N, CO, HO, WO)


def maxpool2d_ref(x, kernel_size, stride):
    """The reference's MaxPool2D over [N,C,H,W]; raises ValueError where the reference panics."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if x.ndim != 4:
        raise ValueError("maxpool2d: expected 4D input")
    N, Cc, H, W = x.shape
    if kernel_size <= 0 or stride <= 0 or kernel_size > H or kernel_size > W:
        raise ValueError("maxpool2d: invalid arguments")
    HO, WO = (H - kernel_size) // stride + 1, (W - kernel_size) // stride + 1
    out = np.empty((N, Cc, HO, WO), dtype=np.float32)
    rc = lib().born_oracle_maxpool2d_f32(_p(x, C.c_float), N, Cc, H, W, kernel_size, stride, _p(out, C.c_float))
    if rc != 0:
        raise ValueError("maxpool2d: invalid arguments")
    return out


def row_stats(x, T=1.0):
    x = _f32(x)
    m = np.empty(x.shape[0], dtype=np.float32)
    Z = np.empty(x.shape[0], dtype=np.uint64)
    lib().born_oracle_row_stats(_p(x, C.c_float), x.shape[0], x.shape[1], x.shape[1], float(T),
                                _p(m, C.c_float), _p(Z, C.c_uint64))
    return m, Z


def sample(logits, uniforms, temperature=1.0, top_k=0, top_p=1.0, rep=1.0, history=None, hist_len=None,
           mode=MODE_TRUTH, nuc_cap=0, min_p=0.0, freq=0.0, pres=0.0):
    """Returns dict(tokens, probs, near, n_nucleus[, nuc_ids, nuc_probs], bad_ids)."""
    x = _f32(logits)
    B, V = x.shape
    u = _f32(uniforms)
    assert u.shape == (B,)
    h = hl = None
    hs = 0
    if history is not None:
        h = np.ascontiguousarray(history, dtype=np.int32)
        assert h.ndim == 2 and h.shape[0] == B
        hs = h.shape[1]
        if hist_len is not None:
            hl = np.ascontiguousarray(hist_len, dtype=np.int32)
    tokens = np.empty(B, dtype=np.int32)
    probs = np.empty(B, dtype=np.float32)
    near = np.zeros(B, dtype=np.uint8)
    nn = np.empty(B, dtype=np.int32)
    nid = npr = None
    if nuc_cap > 0:
        nid = np.empty((B, nuc_cap), dtype=np.int32)
        npr = np.empty((B, nuc_cap), dtype=np.float32)
    bad = lib().born_oracle_sample_ex(_p(x, C.c_float), B, V, V, _p(h, C.c_int32), _p(hl, C.c_int32), hs,
                                   _p(u, C.c_float), float(temperature), int(top_k), float(top_p), float(min_p),
                                   float(rep), float(freq), float(pres), int(mode), _p(tokens, C.c_int32), _p(probs, C.c_float), _p(near, C.c_uint8),
                                   _p(nn, C.c_int32), int(nuc_cap), _p(nid, C.c_int32), _p(npr, C.c_float))
    if bad < 0:
        raise ValueError("born_oracle_sample: bad arguments")
    out = dict(tokens=tokens, probs=probs, near=(near & 1).astype(bool), near_cut=(near & 2).astype(bool),
               n_nucleus=nn, bad_ids=int(bad))
    if nuc_cap > 0:
        out["nuc_ids"] = nid
        out["nuc_probs"] = npr
    return out


def token_logprobs(logits, tokens, temperature=1.0, rep=1.0, history=None, hist_len=None, mode=MODE_TRUTH, freq=0.0, pres=0.0):
    """log_softmax of each row (after penalties and temperature) at the row's given token; returns (values, bad ids)."""
    x = _f32(logits)
    B, V = x.shape
    t = np.ascontiguousarray(tokens, dtype=np.int32)
    assert t.shape == (B,)
    h = hl = None
    hs = 0
    if history is not None:
        h = np.ascontiguousarray(history, dtype=np.int32)
        hs = h.shape[1]
        if hist_len is not None:
            hl = np.ascontiguousarray(hist_len, dtype=np.int32)
    out = np.empty(B, dtype=np.float32)
    bad = lib().born_oracle_token_logprobs(_p(x, C.c_float), B, V, V, _p(h, C.c_int32), _p(hl, C.c_int32), hs, _p(t, C.c_int32),
                                           float(temperature), float(rep), float(freq), float(pres), int(mode), _p(out, C.c_float))
    if bad < 0:
        raise ValueError("born_oracle_token_logprobs: bad arguments")
    return out, int(bad)


def cross_entropy_ref(logits, targets):
    """The reference's CrossEntropyLoss.Forward: mean over the batch of -logSoftmax(x)[target], fp32."""
    x = _f32(logits)
    t = np.ascontiguousarray(targets, dtype=np.int32)
    loss = np.zeros(1, dtype=np.float32)
    if lib().born_oracle_cross_entropy_f32(_p(x, C.c_float), x.shape[0], x.shape[1], _p(t, C.c_int32), _p(loss, C.c_float)) != 0:
        raise ValueError("CrossEntropyLoss: target index out of bounds")
    return float(loss[0])


def spec_verify(target, draft, draft_tokens, u_acc, u_res, temperature=1.0, mode=MODE_TRUTH, bonus=None):
    """bonus: fp32 [B, V], the target's logits one position past the draft (drawn from when nothing is rejected)."""
    t = _f32(target)
    d = _f32(draft)
    B, G, V = t.shape
    dt = np.ascontiguousarray(draft_tokens, dtype=np.int32)
    ua = _f32(u_acc)
    ur = _f32(u_res)
    nacc = np.empty(B, dtype=np.int32)
    nxt = np.empty(B, dtype=np.int32)
    near = np.zeros(B, dtype=np.uint8)
    bad = lib().born_oracle_spec_verify(_p(t, C.c_float), _p(d, C.c_float), B, G, V, _p(dt, C.c_int32),
                                        _p(ua, C.c_float), _p(ur, C.c_float), float(temperature), int(mode),
                                        _p(nacc, C.c_int32), _p(nxt, C.c_int32), _p(near, C.c_uint8))
    if bad < 0:
        raise ValueError("born_oracle_spec_verify: bad arguments")
    if bonus is not None:
        bn = _f32(bonus)
        assert bn.shape == (B, V)
        lib().born_oracle_spec_bonus_draw(_p(bn, C.c_float), B, V, V, G, _p(ur, C.c_float), float(temperature), int(mode),
                                          _p(nacc, C.c_int32), _p(nxt, C.c_int32), _p(near, C.c_uint8))
    return dict(n_accepted=nacc, next_token=nxt, near=near.astype(bool), bad_tokens=int(bad))
