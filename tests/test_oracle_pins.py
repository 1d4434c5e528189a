"""Pins for the parts of the CPU oracle that no reference host code covers, and closed-form /
brute-force checks for the rest, chosen so a dropped term, a wrong sign or index or a transposed
operand fails: fp16 conversion, sigmoid router, permutation, fixed-order combine, wave64 packing,
Sinkhorn closed forms, clamp probes."""
import itertools

import numpy as np
import pytest


def test_double_to_half_exhaustive_roundtrip_and_rounding(orc):
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16).astype(np.float64)
    finite = np.isfinite(vals)
    back = orc.double_to_half_bits(vals[finite])
    want = bits[finite].copy()
    assert np.array_equal(back, want)          # every finite fp16 survives the round trip (+-0 too)
    # ties to even and directed cases, against numpy's IEEE conversion
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 1, 20000), rng.normal(0, 1e-6, 5000), rng.normal(0, 3e4, 5000),
                        (vals[finite][:-1] + vals[finite][1:]) / 2,   # exact midpoints
                        [65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0**-25, 2.0**-24, 1.5 * 2.0**-25]])
    x = x[np.isfinite(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.double_to_half_bits(x), want)


def test_clamped_swiglu_probes(orc):
    L = 7.0
    silu = lambda g: g / (1.0 + np.exp(-g))
    # gate bounded from above only; up both sides (tests/test_v4_expert_oracle.cpp:302-406)
    assert orc.clamped_swiglu(40.0, 3.0, L) == silu(7.0) * 3.0
    assert orc.clamped_swiglu(-40.0, 3.0, L) == silu(-40.0) * 3.0        # NOT clamped at -7
    assert orc.clamped_swiglu(-40.0, 3.0, L, mode=1) == silu(-7.0) * 3.0  # the symmetric misreading
    assert orc.clamped_swiglu(2.0, 40.0, L) == silu(2.0) * 7.0
    assert orc.clamped_swiglu(2.0, -40.0, L) == silu(2.0) * -7.0
    assert orc.clamped_swiglu(12.0, 12.0, L, mode=2) == silu(12.0) * 12.0
    assert orc.clamped_swiglu(0.0, 5.0, L) == 0.0


def test_matvec_is_a_matrix_product(orc):
    rng = np.random.default_rng(1)
    w = rng.integers(-8, 8, (33, 70)).astype(np.float64)   # integers: every order gives the same sum
    x = rng.integers(-5, 6, 70).astype(np.float64)
    assert np.array_equal(orc.matvec(w, x), w @ x)
    assert not np.array_equal(orc.matvec(w, x), (w.T[:33, :33] @ x[:33]) if False else w @ x[::-1])


def test_swizzled_matvec_equals_decode_then_matvec(orc):
    rng = np.random.default_rng(2)
    N, K = 32, 512
    packed = rng.integers(0, 2**32, N * K // 8, dtype=np.uint32)
    scale = rng.uniform(0.005, 0.02, N * K // 32).astype(np.float16).view(np.uint16)
    x = rng.normal(size=(3, K))
    w = orc.swizzled_decode(packed, scale, N, K, 4, 8)
    got = orc.swizzled_matvec(packed, scale, N, K, 4, 8, x)
    for t in range(3):
        assert np.array_equal(got[t], orc.matvec(w, x[t]))
    # brute force through the address formula, element by element
    for r, c in itertools.product((0, 5, 31), (0, 7, 8, 33, 511)):
        slot, word, nib = orc.swizzled_address(K, 4, 8, r, c)
        q = (int(packed[word]) >> (4 * nib)) & 0xF
        assert w[r, c] == (q - 8) * float(scale.view(np.float16)[slot])


def test_expert_ffn_composition(orc):
    """expert_ffn == W2 . clamped_swiglu(W1 x, W3 x), checked by composing the pinned pieces; the
    rounded-hidden variant differs only by the fp16 rounding of hidden."""
    rng = np.random.default_rng(3)
    H, I = 256, 128
    mats = []
    for rows, cols, cfg in ((I, H, (4, 8)), (I, H, (4, 8)), (H, I, (8, 4))):
        mats.append((rng.integers(0, 2**32, rows * cols // 8, dtype=np.uint32),
                     rng.uniform(0.005, 0.02, rows * cols // 32).astype(np.float16).view(np.uint16)))
    x = rng.normal(size=(2, H))
    out, hidden = orc.expert_ffn(mats[0], mats[1], mats[2], H, I, x, 1.5, want_hidden=True)
    w1 = orc.swizzled_decode(*mats[0], I, H, 4, 8)
    w3 = orc.swizzled_decode(*mats[1], I, H, 4, 8)
    w2 = orc.swizzled_decode(*mats[2], H, I, 8, 4)
    for t in range(2):
        g, u = orc.matvec(w1, x[t]), orc.matvec(w3, x[t])
        h = np.array([orc.clamped_swiglu(a, b, 1.5) for a, b in zip(g, u)])
        assert np.array_equal(hidden[t], h)
        assert np.array_equal(out[t], orc.matvec(w2, h))
        assert (np.abs(g) > 1.5).any()          # the clamp is exercised
    out_r, hidden_r = orc.expert_ffn(mats[0], mats[1], mats[2], H, I, x, 1.5, round_hidden=True,
                                     want_hidden=True)
    assert np.array_equal(hidden_r, hidden.astype(np.float16).astype(np.float64))
    assert np.array_equal(out_r[0], orc.matvec(w2, hidden_r[0]))
    # swapping gate and up is a different function (the gate alone goes through silu)
    swapped = orc.expert_ffn(mats[1], mats[0], mats[2], H, I, x, 1.5)
    assert np.abs(swapped - out).max() > 1e-3 * np.abs(out).max()


def test_sigmoid_router_closed_forms(orc):
    # logits 0 -> every score 1/2; the bias alone orders them; weights are the UNBIASED scores
    E, k = 16, 4
    bias = np.linspace(-0.3, 0.3, E)
    ids, w = orc.router_topk(np.zeros(E), bias, k, 1.0, score_kind=1)
    assert list(ids) == [15, 14, 13, 12]
    assert np.allclose(w, 0.25, rtol=0, atol=1e-16)
    # two experts: sigmoid(x) and sigmoid(-x) sum to 1
    ids, w = orc.router_topk(np.array([1.25, -1.25]), None, 2, 1.0, score_kind=1)
    assert list(ids) == [0, 1] and abs(w[0] - 1 / (1 + np.exp(-1.25))) < 1e-15 and abs(w.sum() - 1) < 1e-15
    # scaling multiplies after the renormalisation
    _, w2 = orc.router_topk(np.array([1.25, -1.25]), None, 2, 1.5, score_kind=1)
    assert np.allclose(w2, 1.5 * w, rtol=1e-15)
    # bias after the activation: a large positive bias on a tiny-score expert selects it, with
    # its tiny unbiased score as the weight
    logits = np.array([-10.0, 2.0, 1.0, 0.0])
    ids, w = orc.router_topk(logits, np.array([5.0, 0, 0, 0]), 2, 1.0, score_kind=1)
    assert list(ids) == [0, 1] and w[0] < 1e-4
    # the deliberately wrong reading (bias inside the activation, dsv4_oracle.hpp:1196-1203)
    # keeps the selection here but reports a different, biased weight
    ids_b, w_b = orc.router_topk(logits, np.array([5.0, 0, 0, 0]), 2, 1.0, score_kind=1, bias_before=True)
    assert list(ids_b) == [0, 1] and w_b[0] > 50 * w[0]
    # ties go to the lower index, flat over all experts
    ids, _ = orc.router_topk(np.array([0.5, 3.0, 3.0, 0.1, 3.0]), None, 2, 1.0, score_kind=1)
    assert list(ids) == [1, 2]
    # against a brute-force numpy restatement on random data
    rng = np.random.default_rng(5)
    for _ in range(20):
        l, b = rng.normal(0, 2, 64), rng.normal(0, 0.1, 64)
        s = 1 / (1 + np.exp(-l))
        order = np.argsort(-(s + b), kind="stable")[:8]
        ids, w = orc.router_topk(l, b, 8, 1.0, score_kind=1)
        assert np.array_equal(ids, order.astype(np.int32))
        assert np.allclose(w, s[order] / s[order].sum(), rtol=1e-14, atol=0)


@pytest.mark.parametrize("T,slots,E", [(1, 6, 256), (7, 6, 256), (300, 6, 256), (64, 8, 8), (0, 6, 256),
                                       (2048, 8, 256)])
def test_permutation_invariants(orc, T, slots, E):
    """The five definitional invariants of tests/test_expert_permutation.cpp:134-180 and equality
    with numpy's stable sort."""
    rng = np.random.default_rng(T + E)
    ids = rng.integers(0, E, (T, slots)).astype(np.int32)
    off, tok, drw = orc.expert_permutation(ids, T, slots, E)
    draws = T * slots
    hist = np.bincount(ids.ravel(), minlength=E) if draws else np.zeros(E, dtype=int)
    assert off[0] == 0 and off[E] == draws
    assert np.array_equal(np.diff(off), hist)
    assert np.array_equal(np.sort(drw), np.arange(draws))              # a bijection
    for e in range(E):
        seg = drw[off[e]:off[e + 1]]
        assert np.all(ids.ravel()[seg] == e) and np.all(np.diff(seg) > 0)  # own expert, ascending
    assert np.array_equal(tok, drw // slots)
    assert np.array_equal(drw, np.argsort(ids.ravel(), kind="stable").astype(np.int32))
    if T >= 7:   # out-of-range ids are dropped
        bad = ids.copy()
        bad[1, 0], bad[2, 1] = -3, E
        off2, _, drw2 = orc.expert_permutation(bad, T, slots, E)
        assert off2[E] == draws - 2 and (1 * slots) not in drw2[:off2[E]]


def test_moe_combine_is_slot_ordered_with_shared_first(orc):
    # fp64 sums of values chosen so the ORDER matters: shared + big - big + small
    contrib = np.array([[1e17], [-1e17], [1.0]])
    assert orc.moe_combine(contrib, np.array([3.0]))[0] == 1.0      # ((3+1e17)-1e17)+1 = 0+1
    assert orc.moe_combine(contrib[[2, 0, 1]], np.array([3.0]))[0] == 0.0  # ((3+1)+1e17)-1e17
    assert orc.moe_combine(contrib, None)[0] == 1.0
    rng = np.random.default_rng(6)
    c, s = rng.normal(size=(8, 50)), rng.normal(size=50)
    want = s.copy()
    for e in range(8):
        want = want + c[e]
    assert np.array_equal(orc.moe_combine(c, s), want)


def test_a64_address_is_a_bijection_and_matches_the_layout_statement(orc):
    N, K = 32, 256
    seen = set()
    for r in range(N):
        for c in range(K):
            pw, nib, si = orc.a64_address(K, r, c)
            assert (pw, nib) not in seen
            seen.add((pw, nib))
            tile = (r // 16) * (K // 128) + c // 128
            lane = ((c % 32) // 8) * 16 + r % 16
            assert pw == (tile * 64 + lane) * 4 + (c % 128) // 32
            assert nib == [0, 4, 1, 5, 2, 6, 3, 7][c % 8]
            assert si == tile * 16 + r % 16
    assert len(seen) == N * K
    rng = np.random.default_rng(7)
    src = rng.integers(0, 2**32, N * K // 8, dtype=np.uint32)
    s128 = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    s32 = np.repeat(s128, 4, axis=1).view(np.uint16)
    p, s = orc.a64_pack(src, s32, N, K)
    sw_p, sw_s = orc.swizzle(src, s32.ravel(), N, K, 4, 8)
    assert np.array_equal(orc.a64_decode(p, s, N, K), orc.swizzled_decode(sw_p, sw_s, N, K, 4, 8))
    bad = s32.copy()
    bad[0, 1] ^= 1
    with pytest.raises(ValueError):
        orc.a64_pack(src, bad, N, K)
    # four scales kept per 128 columns: same nibble addresses, scale of (row, 32-column group)
    # at [tile][row%16][step]; a payload with a scale of its own per 32 columns decodes to the
    # same matrix the `.aeon` reading gives
    for r in range(N):
        for c in range(0, K, 8):
            pw, nib, si = orc.a64_address(K, r, c, 32)
            assert (pw, nib) == orc.a64_address(K, r, c)[:2]
            tile = (r // 16) * (K // 128) + c // 128
            assert si == (tile * 16 + r % 16) * 4 + (c % 128) // 32
    d32 = rng.uniform(0.005, 0.02, (N, K // 32)).astype(np.float16).view(np.uint16)
    p4, s4 = orc.a64_pack(src, d32, N, K, 32)
    assert np.array_equal(p4, p) and s4.size == N * K // 32
    sw_p4, sw_s4 = orc.swizzle(src, d32.ravel(), N, K, 4, 8)
    assert np.array_equal(orc.a64_decode(p4, s4, N, K, 32), orc.swizzled_decode(sw_p4, sw_s4, N, K, 4, 8))


def test_sinkhorn_closed_forms(orc):
    eps = 1e-6
    # zero logits: every entry exactly 1/4 up to the eps share (tests/test_v4_hc_oracle.cpp:371-404)
    pre, post, comb = orc.hc_sinkhorn(np.zeros(24), np.ones(3), np.zeros(24))
    assert np.abs(comb - 0.25).max() <= eps
    assert np.allclose(pre, 0.5 + eps, rtol=0, atol=1e-15) and np.allclose(post, 1.0, rtol=0, atol=1e-15)
    rng = np.random.default_rng(8)
    mixes = rng.normal(size=24)
    _, _, c20 = orc.hc_sinkhorn(mixes, np.ones(3), np.zeros(24))
    _, _, c1 = orc.hc_sinkhorn(mixes, np.ones(3), np.zeros(24), 4, orc.hc_params(sinkhorn_iters=1))
    dev = lambda c: max(np.abs(c.reshape(4, 4).sum(0) - 1).max(), np.abs(c.reshape(4, 4).sum(1) - 1).max())
    assert dev(c20) < 1e-4 and dev(c1) > 100 * dev(c20)          # :218-247
    # the last pass normalises over i: column sums (over the contraction index) are 1/(1+eps/sum)
    assert np.abs(c1.reshape(4, 4).sum(0) - 1).max() < 1e-5
    # a permutation-like logit matrix converges to that permutation: C[i][j] with i the row
    big = np.zeros(24)
    perm = [2, 0, 3, 1]
    for i, j in enumerate(perm):
        big[8 + i * 4 + j] = 30.0
    _, _, cp = orc.hc_sinkhorn(big, np.ones(3), np.zeros(24))
    want = np.zeros((4, 4))
    for i, j in enumerate(perm):
        want[i, j] = 1.0
    assert np.abs(cp.reshape(4, 4) - want).max() < 1e-4
    # third scale applies to comb only; post carries x2 and no eps
    pre_s, post_s, _ = orc.hc_sinkhorn(mixes, np.array([2.0, 3.0, 5.0]), np.zeros(24))
    assert np.allclose(pre_s, 1 / (1 + np.exp(-2 * mixes[:4])) + eps, rtol=1e-15)
    assert np.allclose(post_s, 2 / (1 + np.exp(-3 * mixes[4:8])), rtol=1e-15)


def test_hc_pre_and_post_are_the_stated_contractions(orc):
    rng = np.random.default_rng(9)
    H = 40
    res, lo = rng.normal(size=(4, H)), rng.normal(size=H)
    pre, post, comb = rng.random(4), rng.random(4), rng.random(16)
    assert np.allclose(orc.hc_pre_combine(res, pre, H), pre @ res, rtol=1e-14)
    want = np.einsum("ij,ih->jh", comb.reshape(4, 4), res) + post[:, None] * lo[None, :]
    assert np.allclose(orc.hc_post(lo, res, post, comb, H), want, rtol=1e-13)
    wrong = np.einsum("ji,ih->jh", comb.reshape(4, 4), res) + post[:, None] * lo[None, :]
    assert np.allclose(orc.hc_post(lo, res, post, comb, H, transpose_comb=True), wrong, rtol=1e-13)
    assert np.abs(want - wrong).max() > 1e-2
