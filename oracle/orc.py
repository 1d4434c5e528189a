"""ctypes front end of the CPU oracle (oracle/aeon_oracle.c) and, where it was built, of the
reference's own host oracle (oracle/_ref/libaeon_ref.so).

Test infrastructure: only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py import this module, and only as the checker. Nothing shipped depends on it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libaeon_oracle.so")
_REF = os.path.join(_HERE, "_ref", "libaeon_ref.so")


def build(force=False):
    """Compile the oracle (and oracle/_ref when /root/reference is present)."""
    if force or not os.path.exists(_LIB) or (
            os.path.isdir("/root/reference/src") and not os.path.exists(_REF)):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True)


def _ptr(a, ctype):
    return a.ctypes.data_as(C.POINTER(ctype)) if a is not None else None


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = C.CDLL(_LIB)
        _lib.orc_half_bits_to_double.restype = C.c_double
        _lib.orc_half_bits_to_double.argtypes = [C.c_uint16]
        _lib.orc_double_to_half_bits.restype = C.c_uint16
        _lib.orc_double_to_half_bits.argtypes = [C.c_double]
        _lib.orc_float_to_half_bits.restype = C.c_uint16
        _lib.orc_float_to_half_bits.argtypes = [C.c_float]
        _lib.orc_clamped_swiglu.restype = C.c_double
        _lib.orc_clamped_swiglu.argtypes = [C.c_double, C.c_double, C.c_double, C.c_int]
        _lib.orc_rng_next_u64.restype = C.c_uint64
        _lib.orc_rng_uniform01.restype = C.c_double
        _lib.orc_rng_symmetric.restype = C.c_double
        _lib.orc_rng_symmetric.argtypes = [C.c_void_p, C.c_double]
    return _lib


_ref = None


def ref():
    """The reference's own oracle, or None where oracle/_ref was not built."""
    global _ref
    if _ref is None:
        if not os.path.exists(_REF):
            return None
        _ref = C.CDLL(_REF)
        _ref.ref_half_bits_to_double.restype = C.c_double
        _ref.ref_half_bits_to_double.argtypes = [C.c_uint16]
        _ref.ref_clamped_swiglu.restype = C.c_double
        _ref.ref_clamped_swiglu.argtypes = [C.c_double, C.c_double, C.c_double, C.c_int]
        _ref.ref_sigmoid.restype = C.c_double
        _ref.ref_sigmoid.argtypes = [C.c_double]
        _ref.ref_rng_draws.restype = C.c_uint64
    return _ref


# ---- scalar helpers ---------------------------------------------------------------------

def half_bits_to_double(bits):
    b = np.ascontiguousarray(bits, dtype=np.uint16).ravel()
    out = np.empty(b.size, dtype=np.float64)
    f = lib().orc_half_bits_to_double
    for i, v in enumerate(b):
        out[i] = f(int(v))
    return out.reshape(np.shape(bits))


def half_to_double(h):
    """fp16 array -> float64, exact (numpy's widening is exact as well; this goes through the
    oracle's own decoder only in the pin tests)."""
    return np.asarray(h, dtype=np.float16).astype(np.float64)


def double_to_half_bits(x):
    f = lib().orc_double_to_half_bits
    a = np.asarray(x, dtype=np.float64)
    out = np.empty(a.size, dtype=np.uint16)
    for i, v in enumerate(a.ravel()):
        out[i] = f(float(v))
    return out.reshape(a.shape)


def rng_u64(seed, count):
    state = C.c_uint64(0)
    lib().orc_rng_seed(C.byref(state), C.c_uint64(seed))
    return np.array([lib().orc_rng_next_u64(C.byref(state)) for _ in range(count)], dtype=np.uint64)


def rng_uniform01(seed, count):
    state = C.c_uint64(0)
    lib().orc_rng_seed(C.byref(state), C.c_uint64(seed))
    return np.array([lib().orc_rng_uniform01(C.byref(state)) for _ in range(count)])


# ---- layout -----------------------------------------------------------------------------

def swizzle(src_packed, src_scale, N, K, rpw, lpr):
    sp = np.ascontiguousarray(src_packed, dtype=np.uint32)
    ss = np.ascontiguousarray(src_scale).view(np.uint16)
    dp = np.empty_like(sp)
    ds = np.empty_like(ss)
    rc = lib().orc_swizzle_w4a16(_ptr(sp, C.c_uint32), _ptr(ss, C.c_uint16), _ptr(dp, C.c_uint32),
                                 _ptr(ds, C.c_uint16), N, K, rpw, lpr)
    if rc != 0:
        raise ValueError("orc_swizzle_w4a16: bad shape")
    return dp, ds


def unswizzle(sw_packed, sw_scale, N, K, rpw, lpr):
    sp = np.ascontiguousarray(sw_packed, dtype=np.uint32)
    ss = np.ascontiguousarray(sw_scale).view(np.uint16)
    dp = np.empty_like(sp)
    ds = np.empty_like(ss)
    rc = lib().orc_unswizzle_w4a16(_ptr(sp, C.c_uint32), _ptr(ss, C.c_uint16),
                                   _ptr(dp, C.c_uint32), _ptr(ds, C.c_uint16), N, K, rpw, lpr)
    if rc != 0:
        raise ValueError("orc_unswizzle_w4a16: bad shape")
    return dp, ds


class _Addr(C.Structure):
    _fields_ = [("storage_slot", C.c_size_t), ("packed_word", C.c_size_t), ("nibble", C.c_int)]


class _A64Addr(C.Structure):
    _fields_ = [("packed_word", C.c_size_t), ("nibble", C.c_int), ("scale_index", C.c_size_t)]


def swizzled_address(columns, rpw, lpr, row, column):
    f = lib().orc_swizzled_address
    f.restype = _Addr
    a = f(columns, rpw, lpr, row, column)
    return a.storage_slot, a.packed_word, a.nibble


def a64_address(columns, row, column, scale_group=128):
    f = lib().orc_a64_address_g
    f.restype = _A64Addr
    a = f(columns, row, column, scale_group)
    return a.packed_word, a.nibble, a.scale_index


def swizzled_decode(packed, scale, rows, columns, rpw, lpr, signed_zp=True, permute=True):
    p = np.ascontiguousarray(packed, dtype=np.uint32)
    s = np.ascontiguousarray(scale).view(np.uint16)
    out = np.empty((rows, columns), dtype=np.float64)
    lib().orc_swizzled_decode(_ptr(p, C.c_uint32), _ptr(s, C.c_uint16), rows, columns, rpw, lpr,
                              int(signed_zp), int(permute), _ptr(out, C.c_double))
    return out


def swizzled_encode(w, rows, columns, rpw, lpr):
    w = np.ascontiguousarray(w, dtype=np.float64)
    p = np.empty(rows * columns // 8, dtype=np.uint32)
    s = np.empty(rows * columns // 32, dtype=np.uint16)
    lib().orc_swizzled_encode(_ptr(p, C.c_uint32), _ptr(s, C.c_uint16), rows, columns, rpw, lpr,
                              _ptr(w, C.c_double))
    return p, s


def a64_pack(src_packed, src_scale32, rows, columns, scale_group=128):
    sp = np.ascontiguousarray(src_packed, dtype=np.uint32)
    ss = np.ascontiguousarray(src_scale32).view(np.uint16)
    p = np.empty(rows * columns // 8, dtype=np.uint32)
    s = np.empty(rows * columns // scale_group, dtype=np.uint16)
    rc = lib().orc_a64_pack_g(_ptr(sp, C.c_uint32), _ptr(ss, C.c_uint16), rows, columns,
                              scale_group, _ptr(p, C.c_uint32), _ptr(s, C.c_uint16))
    if rc != 0:
        raise ValueError("orc_a64_pack failed with %d" % rc)
    return p, s


def a64_decode(a64_packed, a64_scale, rows, columns, scale_group=128):
    p = np.ascontiguousarray(a64_packed, dtype=np.uint32)
    s = np.ascontiguousarray(a64_scale).view(np.uint16)
    out = np.empty((rows, columns), dtype=np.float64)
    lib().orc_a64_decode_g(_ptr(p, C.c_uint32), _ptr(s, C.c_uint16), rows, columns, scale_group,
                           _ptr(out, C.c_double))
    return out


# ---- arithmetic -------------------------------------------------------------------------

def matvec(w, x):
    w = np.ascontiguousarray(w, dtype=np.float64)
    x = np.ascontiguousarray(x, dtype=np.float64)
    y = np.empty(w.shape[0], dtype=np.float64)
    lib().orc_matvec(C.c_size_t(w.shape[0]), C.c_size_t(w.shape[1]), _ptr(w, C.c_double),
                     _ptr(x, C.c_double), _ptr(y, C.c_double))
    return y


def swizzled_matvec(packed, scale, rows, columns, rpw, lpr, x):
    """x [tokens][columns] (or [columns]) float64 -> [tokens][rows]."""
    p = np.ascontiguousarray(packed, dtype=np.uint32)
    s = np.ascontiguousarray(scale).view(np.uint16)
    x2 = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float64)
    y = np.empty((x2.shape[0], rows), dtype=np.float64)
    lib().orc_swizzled_matvec(_ptr(p, C.c_uint32), _ptr(s, C.c_uint16), rows, columns, rpw, lpr,
                              _ptr(x2, C.c_double), x2.shape[0], _ptr(y, C.c_double))
    return y if np.ndim(x) == 2 else y[0]


def clamped_swiglu(gate, up, limit, mode=0):
    return lib().orc_clamped_swiglu(float(gate), float(up), float(limit), int(mode))


def expert_ffn(w1, w3, w2, H, I, x, limit, clamp_mode=0, round_hidden=False, cfg13=(4, 8),
               cfg2=(8, 4), want_hidden=False):
    """w1/w3/w2 are (packed, scale) pairs in the swizzled storage; x [tokens][H] float64."""
    x2 = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float64)
    t = x2.shape[0]
    arrs = []
    for p, s in (w1, w3, w2):
        arrs.append(np.ascontiguousarray(p, dtype=np.uint32))
        arrs.append(np.ascontiguousarray(s).view(np.uint16))
    out = np.empty((t, H), dtype=np.float64)
    hidden = np.empty((t, I), dtype=np.float64) if want_hidden else None
    lib().orc_expert_ffn(_ptr(arrs[0], C.c_uint32), _ptr(arrs[1], C.c_uint16),
                         _ptr(arrs[2], C.c_uint32), _ptr(arrs[3], C.c_uint16),
                         _ptr(arrs[4], C.c_uint32), _ptr(arrs[5], C.c_uint16),
                         H, I, cfg13[0], cfg13[1], cfg2[0], cfg2[1], _ptr(x2, C.c_double), t,
                         C.c_double(limit), int(clamp_mode), int(round_hidden),
                         _ptr(hidden, C.c_double), _ptr(out, C.c_double))
    if np.ndim(x) == 1:
        out = out[0]
        hidden = hidden[0] if hidden is not None else None
    return (out, hidden) if want_hidden else out


def dense_ffn(w1, w3, w2, x, limit, clamp_mode=0, round_stages=False, want_hidden=False):
    """The unquantised shared expert: w1, w3 [I][H], w2 [H][I] (row-major), x [tokens][H]."""
    w1, w3, w2 = (np.ascontiguousarray(w, dtype=np.float64) for w in (w1, w3, w2))
    I, H = w1.shape
    x2 = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float64)
    t = x2.shape[0]
    out = np.empty((t, H), dtype=np.float64)
    hidden = np.empty((t, I), dtype=np.float64) if want_hidden else None
    lib().orc_dense_ffn(C.c_size_t(I), C.c_size_t(H), _ptr(x2, C.c_double), C.c_size_t(t),
                        _ptr(w1, C.c_double), _ptr(w3, C.c_double), _ptr(w2, C.c_double),
                        C.c_double(limit), int(clamp_mode), int(round_stages),
                        _ptr(hidden, C.c_double), _ptr(out, C.c_double))
    if np.ndim(x) == 1:
        out = out[0]
        hidden = hidden[0] if hidden is not None else None
    return (out, hidden) if want_hidden else out


def topk_indices(scores, k):
    s = np.ascontiguousarray(scores, dtype=np.float64)
    ids = np.empty(min(k, s.size), dtype=np.int32)
    lib().orc_topk_indices(_ptr(s, C.c_double), C.c_size_t(s.size), C.c_size_t(k),
                           _ptr(ids, C.c_int32))
    return ids


def router_scores(logits, score_kind):
    """The fp64 scores router_topk compares (before any bias)."""
    l = np.ascontiguousarray(logits, dtype=np.float64)
    out = np.empty(l.size, dtype=np.float64)
    lib().orc_router_scores(_ptr(l, C.c_double), C.c_size_t(l.size), int(score_kind),
                            _ptr(out, C.c_double))
    return out.reshape(l.shape)


def router_topk(logits, bias, top_k, scaling, score_kind, bias_before=False):
    l = np.ascontiguousarray(logits, dtype=np.float64)
    b = np.ascontiguousarray(bias, dtype=np.float64) if bias is not None else None
    ids = np.empty(top_k, dtype=np.int32)
    w = np.empty(top_k, dtype=np.float64)
    lib().orc_router_topk(_ptr(l, C.c_double), _ptr(b, C.c_double), C.c_size_t(l.size),
                          C.c_size_t(top_k), C.c_double(scaling), int(score_kind),
                          int(bias_before), _ptr(ids, C.c_int32), _ptr(w, C.c_double))
    return ids, w


def expert_permutation(ids, tokens, slots, experts):
    i = np.ascontiguousarray(ids, dtype=np.int32).ravel()
    offsets = np.zeros(experts + 1, dtype=np.int32)
    tok = np.full(max(tokens * slots, 1), -1, dtype=np.int32)
    drw = np.full(max(tokens * slots, 1), -1, dtype=np.int32)
    lib().orc_expert_permutation(_ptr(i, C.c_int32), tokens, slots, experts,
                                 _ptr(offsets, C.c_int32), _ptr(tok, C.c_int32),
                                 _ptr(drw, C.c_int32))
    return offsets, tok[:tokens * slots], drw[:tokens * slots]


def moe_combine(contrib, shared):
    c = np.ascontiguousarray(contrib, dtype=np.float64)
    s = np.ascontiguousarray(shared, dtype=np.float64) if shared is not None else None
    out = np.empty(c.shape[1], dtype=np.float64)
    lib().orc_moe_combine(_ptr(c, C.c_double), c.shape[0], _ptr(s, C.c_double), c.shape[1],
                          _ptr(out, C.c_double))
    return out


class HcParams(C.Structure):
    _fields_ = [("rms_eps", C.c_double), ("pre_eps", C.c_double), ("sinkhorn_eps", C.c_double),
                ("post_mult", C.c_double), ("sinkhorn_iters", C.c_int)]


def hc_params(**kw):
    p = HcParams()
    lib().orc_hc_default_params(C.byref(p))
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def hc_sinkhorn(mixes, hc_scale, hc_base, hc_mult=4, params=None):
    p = params or hc_params()
    m = np.ascontiguousarray(mixes, dtype=np.float64)
    sc = np.ascontiguousarray(hc_scale, dtype=np.float64)
    ba = np.ascontiguousarray(hc_base, dtype=np.float64)
    pre = np.empty(hc_mult)
    post = np.empty(hc_mult)
    comb = np.empty(hc_mult * hc_mult)
    lib().orc_hc_sinkhorn(_ptr(m, C.c_double), _ptr(sc, C.c_double), _ptr(ba, C.c_double), hc_mult,
                          C.byref(p), _ptr(pre, C.c_double), _ptr(post, C.c_double),
                          _ptr(comb, C.c_double))
    return pre, post, comb


def hc_pre_combine(residual, pre_mix, hidden):
    r = np.ascontiguousarray(residual, dtype=np.float64)
    pm = np.ascontiguousarray(pre_mix, dtype=np.float64)
    out = np.empty(hidden)
    lib().orc_hc_pre_combine(_ptr(r, C.c_double), _ptr(pm, C.c_double), pm.size,
                             C.c_size_t(hidden), _ptr(out, C.c_double))
    return out


def hc_mixes(residual, fn, rms_eps=1e-6):
    """residual [hc_mult*hidden] flattened, fn [mixes][hc_mult*hidden] -> mixes [mixes]."""
    r = np.ascontiguousarray(residual, dtype=np.float64).ravel()
    f = np.ascontiguousarray(fn, dtype=np.float64)
    out = np.empty(f.shape[0])
    lib().orc_hc_mixes(_ptr(r, C.c_double), _ptr(f, C.c_double), C.c_size_t(f.shape[0]),
                       C.c_size_t(r.size), C.c_double(rms_eps), _ptr(out, C.c_double))
    return out


def rmsnorm(x, weight=None, eps=1e-6):
    xv = np.ascontiguousarray(x, dtype=np.float64)
    wv = None if weight is None else np.ascontiguousarray(weight, dtype=np.float64)
    out = np.empty(xv.size)
    lib().orc_rmsnorm(_ptr(xv, C.c_double), None if wv is None else _ptr(wv, C.c_double),
                      C.c_size_t(xv.size), C.c_double(eps), _ptr(out, C.c_double))
    return out


def hc_post(layer_out, residual, post_mix, comb, hidden, transpose_comb=False):
    lo = np.ascontiguousarray(layer_out, dtype=np.float64)
    r = np.ascontiguousarray(residual, dtype=np.float64)
    pm = np.ascontiguousarray(post_mix, dtype=np.float64)
    cm = np.ascontiguousarray(comb, dtype=np.float64)
    out = np.empty((pm.size, hidden))
    lib().orc_hc_post(_ptr(lo, C.c_double), _ptr(r, C.c_double), _ptr(pm, C.c_double),
                      _ptr(cm, C.c_double), pm.size, C.c_size_t(hidden), int(transpose_comb),
                      _ptr(out, C.c_double))
    return out
