"""Pins the C restatement (oracle/aeon_oracle.c) against the reference's own host oracle
compiled from /root/reference into oracle/_ref, on the reference's fixed shapes
(hidden 4096, intermediate 2048, quant group 32). Skipped where oracle/_ref is absent."""
import ctypes as C

import numpy as np
import pytest

P = lambda a, t: a.ctypes.data_as(C.POINTER(t))

SHAPES = {0: (2048, 4096, 4, 8), 1: (4096, 2048, 8, 4), 2: (2048, 4096, 4, 8)}
PAYLOAD_BYTES = 14155776


def _ref_shape(ref, kind):
    po, so = C.c_size_t(), C.c_size_t()
    rows, cols, rpw, lpr = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    ref.ref_shape(kind, C.byref(po), C.byref(so), C.byref(rows), C.byref(cols), C.byref(rpw),
                  C.byref(lpr))
    return po.value, so.value, rows.value, cols.value, rpw.value, lpr.value


def _payload(seed):
    """A full reference-layout expert payload: random nibbles, scales 2^-6..2^-3 (the scale
    family tests/test_moe_grouped_batch_parity.cpp:83-90 uses) plus a few arbitrary fp16s."""
    rng = np.random.default_rng(seed)
    payload = rng.integers(0, 256, PAYLOAD_BYTES, dtype=np.uint8)
    return payload


def _fix_scales(ref, payload, arbitrary):
    rng = np.random.default_rng(99)
    for kind in range(3):
        po, so, rows, cols, _, _ = _ref_shape(ref, kind)
        n = rows * cols // 32
        if arbitrary:
            s = rng.uniform(0.005, 0.02, n).astype(np.float16)
        else:
            s = np.ldexp(1.0, -6 + (np.arange(n) % 4)).astype(np.float16)
        payload[so:so + 2 * n] = s.view(np.uint8)
    return payload


def test_shapes_match_reference(ref):
    for kind, want in SHAPES.items():
        _, _, rows, cols, rpw, lpr = _ref_shape(ref, kind)
        assert (rows, cols, rpw, lpr) == want


def test_rng_matches_reference(orc, ref):
    for seed in (0, 1, 0x0E7E1217, 0xC0FFEE):
        n = 64
        u = np.empty(n, dtype=np.uint64)
        f = np.empty(n)
        ref.ref_rng_draws(C.c_uint64(seed), n, P(u, C.c_uint64), P(f, C.c_double), None,
                          C.c_double(1.0))
        assert np.array_equal(orc.rng_u64(seed, n), u)
        assert np.array_equal(orc.rng_uniform01(seed, n), f)


def test_half_bits_to_double_all_patterns(orc, ref):
    bits = np.arange(65536, dtype=np.uint16)
    mine = orc.half_bits_to_double(bits)
    theirs = np.array([ref.ref_half_bits_to_double(int(b)) for b in bits])
    finite = np.isfinite(theirs)
    assert np.array_equal(mine[finite], theirs[finite])
    assert np.array_equal(np.isnan(mine), np.isnan(theirs))
    # and it is the IEEE value (numpy's own widening), except that the reference maps the
    # infinities' exponent to NaN as well (dsv4_oracle.hpp:1380-1383)
    ieee = bits.view(np.float16).astype(np.float64)
    ok = np.isfinite(ieee)
    assert np.array_equal(mine[ok], ieee[ok])


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_swizzle_roundtrip_matches_reference(orc, ref, kind):
    rows, cols, rpw, lpr = SHAPES[kind]
    rng = np.random.default_rng(kind)
    sp = rng.integers(0, 2**32, rows * cols // 8, dtype=np.uint32)
    ss = rng.integers(0, 2**16, rows * cols // 32, dtype=np.uint16)
    dp, ds = orc.swizzle(sp, ss, rows, cols, rpw, lpr)
    rdp, rds = np.empty_like(sp), np.empty_like(ss)
    ref.ref_swizzle_u16(P(sp, C.c_uint32), P(ss, C.c_uint16), P(rdp, C.c_uint32),
                        P(rds, C.c_uint16), rows, cols, rpw, lpr)
    assert np.array_equal(dp, rdp) and np.array_equal(ds, rds)
    bp, bs = orc.unswizzle(dp, ds, rows, cols, rpw, lpr)
    assert np.array_equal(bp, sp) and np.array_equal(bs, ss)
    rbp, rbs = np.empty_like(sp), np.empty_like(ss)
    ref.ref_unswizzle_u16(P(dp, C.c_uint32), P(ds, C.c_uint16), P(rbp, C.c_uint32),
                          P(rbs, C.c_uint16), rows, cols, rpw, lpr)
    assert np.array_equal(rbp, sp) and np.array_equal(rbs, ss)


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_swizzled_address_matches_reference(orc, ref, kind):
    rows, cols, rpw, lpr = SHAPES[kind]
    rng = np.random.default_rng(5 + kind)
    for _ in range(2000):
        r, c = int(rng.integers(rows)), int(rng.integers(cols))
        a, b, n = C.c_size_t(), C.c_size_t(), C.c_int()
        ref.ref_swizzled_address(kind, r, c, C.byref(a), C.byref(b), C.byref(n))
        assert orc.swizzled_address(cols, rpw, lpr, r, c) == (a.value, b.value, n.value)


@pytest.mark.parametrize("arbitrary_scales", [False, True])
def test_swizzled_decode_matches_reference(orc, ref, arbitrary_scales):
    payload = _fix_scales(ref, _payload(3), arbitrary_scales)
    for kind in range(3):
        po, so, rows, cols, rpw, lpr = _ref_shape(ref, kind)
        want = np.empty((rows, cols))
        packed = payload[po:po + rows * cols // 2].view(np.uint32)
        scale = payload[so:so + rows * cols // 16].view(np.uint16)
        for szp, perm in ((1, 1), (0, 1), (1, 0)):
            ref.ref_swizzled_decode(P(payload, C.c_uint8), kind, szp, perm, P(want, C.c_double))
            got = orc.swizzled_decode(packed, scale, rows, cols, rpw, lpr, szp, perm)
            assert np.array_equal(got, want), (kind, szp, perm)


def test_swizzled_encode_matches_reference(orc, ref):
    rng = np.random.default_rng(11)
    for kind in (0, 1):
        po, so, rows, cols, rpw, lpr = _ref_shape(ref, kind)
        w = rng.normal(0, 0.05, (rows, cols))
        w[3, :64] = 0.0  # an all-zero group takes the exponent floor (dsv4_oracle.hpp:1545-1547)
        payload = np.zeros(PAYLOAD_BYTES, dtype=np.uint8)
        ref.ref_swizzled_encode(P(payload, C.c_uint8), kind, P(w, C.c_double))
        p, s = orc.swizzled_encode(w, rows, cols, rpw, lpr)
        assert np.array_equal(p, payload[po:po + rows * cols // 2].view(np.uint32))
        assert np.array_equal(s, payload[so:so + rows * cols // 16].view(np.uint16))


def test_matvec_bit_identical_to_reference(orc, ref):
    rng = np.random.default_rng(2)
    w = rng.normal(size=(257, 1031))
    x = rng.normal(size=1031)
    want = np.empty(257)
    ref.ref_matvec(C.c_size_t(257), C.c_size_t(1031), P(w, C.c_double), P(x, C.c_double),
                   P(want, C.c_double))
    assert np.array_equal(orc.matvec(w, x), want)


def test_clamped_swiglu_matches_reference(orc, ref):
    probes = [-40.0, -12.0, -5.0, 0.0, 5.0, 12.0, 40.0, 3.0]  # tests/test_v4_expert_oracle.cpp
    for limit in (7.0, 10.0):
        for mode in (0, 1, 2):
            for g in probes:
                for u in probes:
                    assert orc.clamped_swiglu(g, u, limit, mode) == \
                        ref.ref_clamped_swiglu(g, u, limit, mode)


@pytest.mark.parametrize("mode,limit", [(0, 10.0), (0, 0.5), (1, 0.5)])
def test_expert_ffn_bit_identical_to_reference(orc, ref, mode, limit):
    payload = _fix_scales(ref, _payload(8), arbitrary=True)
    rng = np.random.default_rng(4)
    x = rng.normal(size=4096)
    want = np.empty(4096)
    ref.ref_expert_ffn(P(payload, C.c_uint8), P(x, C.c_double), C.c_double(limit), mode,
                       P(want, C.c_double))
    mats = []
    for kind in (0, 2, 1):
        po, so, rows, cols, _, _ = _ref_shape(ref, kind)
        mats.append((payload[po:po + rows * cols // 2].view(np.uint32),
                     payload[so:so + rows * cols // 16].view(np.uint16)))
    got = orc.expert_ffn(mats[0], mats[1], mats[2], 4096, 2048, x, limit, clamp_mode=mode)
    assert np.array_equal(got, want)
    assert np.abs(want).max() > 1e-3


@pytest.mark.parametrize("mode,limit", [(0, 10.0), (0, 0.25), (1, 0.25), (2, 10.0)])
def test_dense_ffn_bit_identical_to_reference(orc, ref, mode, limit):
    """dense_ffn (dsv4_oracle.hpp:1708-1753), the unquantised shared expert: same bits, and the
    closed form of tests/test_v4_shared_expert_oracle.cpp:180-194 (w1 = w3 = w2 = e_0, x0 = 0.5
    gives silu(0.5) * 0.5 in out[0] and zeros elsewhere)."""
    rng = np.random.default_rng(8)
    I, H = 96, 160
    w1, w3 = rng.normal(0, 0.2, (I, H)), rng.normal(0, 0.2, (I, H))
    w2 = rng.normal(0, 0.2, (H, I))
    x = rng.normal(size=H)
    want = np.empty(H)
    ref.ref_dense_ffn(C.c_size_t(I), C.c_size_t(H), P(x, C.c_double), P(w1, C.c_double),
                      P(w3, C.c_double), P(w2, C.c_double), C.c_double(limit), mode,
                      P(want, C.c_double))
    got = orc.dense_ffn(w1, w3, w2, x, limit, clamp_mode=mode)
    assert np.array_equal(got, want)
    assert np.abs(want).max() > 1e-3
    e1, e3, e2 = np.zeros((2, 3)), np.zeros((2, 3)), np.zeros((3, 2))
    e1[0, 0] = e3[0, 0] = e2[0, 0] = 1.0
    out = orc.dense_ffn(e1, e3, e2, np.array([0.5, 0.0, 0.0]), 10.0)
    assert abs(out[0] - (0.5 / (1.0 + np.exp(-0.5))) * 0.5) < 1e-15 and out[1] == 0.0 and out[2] == 0.0
    # the device's view rounds gate, up and the activation to fp16: a different, nearby result
    rounded = orc.dense_ffn(w1, w3, w2, x, limit, clamp_mode=mode, round_stages=True)
    assert 0 < np.abs(rounded - got).max() <= 2e-2 * np.abs(got).max()


def test_topk_and_router_match_reference(orc, ref):
    rng = np.random.default_rng(6)
    for trial in range(50):
        logits = rng.normal(0, 2.0, 256)
        bias = rng.normal(0, 0.1, 256)
        if trial % 5 == 0:  # constructed ties, tests/test_v4_router_oracle.cpp:389-400
            logits[[7, 40, 41, 200]] = logits.max() + 1.0
            bias[[7, 40, 41, 200]] = 0.25
        for k in (6, 8):
            ids = np.empty(k, dtype=np.int32)
            ref.ref_topk_indices(P(logits, C.c_double), C.c_size_t(256), C.c_size_t(k),
                                 P(ids, C.c_int32))
            assert np.array_equal(orc.topk_indices(logits, k), ids)
            for bb in (0, 1):
                w = np.empty(k)
                ref.ref_router_topk(P(logits, C.c_double), P(bias, C.c_double), C.c_size_t(256),
                                    C.c_size_t(k), C.c_double(1.5), bb, P(ids, C.c_int32),
                                    P(w, C.c_double))
                gi, gw = orc.router_topk(logits, bias, k, 1.5, score_kind=0, bias_before=bool(bb))
                assert np.array_equal(gi, ids) and np.array_equal(gw, w)
            ref.ref_router_topk(P(logits, C.c_double), None, C.c_size_t(256), C.c_size_t(k),
                                C.c_double(1.5), 0, P(ids, C.c_int32), P(w, C.c_double))
            gi, gw = orc.router_topk(logits, None, k, 1.5, score_kind=0)
            assert np.array_equal(gi, ids) and np.array_equal(gw, w)


def test_sigmoid_matches_reference(orc, ref):
    # the sigmoid score of orc_router_topk is the reference's own sigmoid (dsv4_oracle.hpp:485)
    for x in np.linspace(-30, 30, 601):
        ids, w = orc.router_topk(np.array([x, -50.0]), None, 1, 1.0, score_kind=1)
        assert ids[0] == 0 and w[0] == 1.0
    xs = np.linspace(-12, 12, 97)
    ids, w = orc.router_topk(xs, None, 97, 1.0, score_kind=1)
    s = np.array([ref.ref_sigmoid(float(v)) for v in xs])
    assert np.array_equal(ids, np.argsort(-s, kind="stable").astype(np.int32))
    assert np.allclose(w, s[ids] / s[ids].sum(), rtol=1e-15, atol=0)


def test_hc_matches_reference(orc, ref):
    rng = np.random.default_rng(7)
    for iters in (1, 2, 20):
        mixes = rng.normal(size=24)
        scale = rng.normal(size=3)
        base = rng.normal(size=24)
        pre, post, comb = np.empty(4), np.empty(4), np.empty(16)
        ref.ref_hc_sinkhorn(P(mixes, C.c_double), P(scale, C.c_double), P(base, C.c_double), 4,
                            C.c_double(1e-6), C.c_double(1e-6), C.c_double(2.0), iters,
                            P(pre, C.c_double), P(post, C.c_double), P(comb, C.c_double))
        gp, gq, gc = orc.hc_sinkhorn(mixes, scale, base, 4, orc.hc_params(sinkhorn_iters=iters))
        assert np.array_equal(gp, pre) and np.array_equal(gq, post) and np.array_equal(gc, comb)
    hidden = 96
    res = rng.normal(size=(4, hidden))
    lo = rng.normal(size=hidden)
    want = np.empty(hidden)
    ref.ref_hc_pre_combine(P(res, C.c_double), P(pre, C.c_double), 4, C.c_size_t(hidden),
                           P(want, C.c_double))
    assert np.array_equal(orc.hc_pre_combine(res, pre, hidden), want)
    for tr in (0, 1):
        want = np.empty((4, hidden))
        ref.ref_hc_post(P(lo, C.c_double), P(res, C.c_double), P(post, C.c_double),
                        P(comb, C.c_double), 4, C.c_size_t(hidden), tr, P(want, C.c_double))
        assert np.array_equal(orc.hc_post(lo, res, post, comb, hidden, bool(tr)), want)


def test_hc_mixes_and_rmsnorm_match_reference(orc, ref):
    """hc_mixes (dsv4_oracle.hpp:509-524) and rmsnorm / rmsnorm_unit (:146-169), bit for bit."""
    rng = np.random.default_rng(11)
    for hc_hidden, rows in ((4 * 96, 24), (4 * 33, 5)):
        res = rng.normal(size=hc_hidden)
        fn = rng.normal(size=(rows, hc_hidden))
        for eps in (1e-6, 0.5):
            want = np.empty(rows)
            ref.ref_hc_mixes(P(res, C.c_double), P(fn, C.c_double), C.c_size_t(rows),
                             C.c_size_t(hc_hidden), C.c_double(eps), P(want, C.c_double))
            assert np.array_equal(orc.hc_mixes(res, fn, eps), want)
    for dim in (1, 7, 640):
        x, w = rng.normal(size=dim), rng.normal(size=dim)
        want = np.empty(dim)
        ref.ref_rmsnorm(P(x, C.c_double), P(w, C.c_double), C.c_size_t(dim), C.c_double(1e-6),
                        P(want, C.c_double))
        assert np.array_equal(orc.rmsnorm(x, w, 1e-6), want)
        ref.ref_rmsnorm(P(x, C.c_double), None, C.c_size_t(dim), C.c_double(1e-3), P(want, C.c_double))
        assert np.array_equal(orc.rmsnorm(x, None, 1e-3), want)
