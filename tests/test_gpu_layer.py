"""GPU parity for the device-resident MoE layer: synthetic experts generated and re-swizzled on
the device, router logits / top-k / permutation, and the full decode step of benchmark config 2
against the oracle."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _setup():
    import torch
    assert torch.cuda.is_available()
    import helpers
    from project_aeon_amd import capi, moe, synth
    return torch, helpers, capi, moe, synth


@pytest.mark.parametrize("scale_group", [128, 32])
def test_device_generator_and_repack_bit_exact(orc, scale_group):
    """The device generator equals the host one, and the device repack equals the host repack,
    for all three matrices of an expert at full size, in both scale groupings."""
    torch, h, capi, moe, synth = _setup()
    H, I = 7168, 2048
    pool = moe.ExpertPool(2, H, I, scale_group=scale_group)
    assert pool.fill_synthetic(seed=5, first_expert_id=40) == 0
    torch.cuda.synchronize()
    host = h.Expert(5, 41, H, I, scale_group)
    raw = pool.buffer.cpu().numpy()
    base = pool.slot_bytes
    for j, (m, which) in enumerate(((host.w1, "w1"), (host.w3, "w3"), (host.w2, "w2"))):
        po, so = base + pool.offsets[2 * j], base + pool.offsets[2 * j + 1]
        assert np.array_equal(raw[po:po + m.a64_packed.nbytes].view(np.uint32), m.a64_packed), which
        assert np.array_equal(raw[so:so + m.a64_scale.nbytes].view(np.uint16), m.a64_scale), which
    # the swizzled payload itself, for one matrix
    p = torch.empty(I * H // 2, dtype=torch.uint8, device="cuda")
    s = torch.empty(I * H // 32, dtype=torch.int16, device="cuda")
    capi.call("aeon_synth_matrix_swizzled", C.c_uint64(5), 41, 1, I, H, 4, 8, scale_group,
              capi.vp(p), capi.vp(s), h.stream_ptr())
    assert np.array_equal(p.cpu().numpy().view(np.uint32), host.w3.swz_packed)
    assert np.array_equal(s.cpu().numpy().view(np.uint16), host.w3.swz_scale)


def test_device_repack_flags_unequal_scales(orc):
    torch, h, capi, moe, synth = _setup()
    N, K = 32, 512
    p, s128 = synth.expert_matrix_source(0, 0, 0, N, K)
    s32 = np.ascontiguousarray(synth.scale32_from_scale128(s128)).view(np.uint16)
    s32[7, 2] ^= 1
    s32[9, 13] ^= 4
    swp, sws = orc.swizzle(p, s32.ravel(), N, K, 4, 8)
    out_p = torch.empty(N * K // 2, dtype=torch.uint8, device="cuda")
    out_s = torch.empty(N * K // 128, dtype=torch.int16, device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    d_swp, d_sws = h.dev_u32(swp), h.dev_u16(sws)
    capi.call("aeon_a64_repack_device", capi.vp(d_swp), capi.vp(d_sws), N, K, 4,
              8, 128, capi.vp(out_p), capi.vp(out_s), capi.vp(flag), h.stream_ptr())
    assert int(flag.item()) == 2
    # kept as they are, the same scales repack without a flag and equal the host repack
    out_s4 = torch.empty(N * K // 32, dtype=torch.int16, device="cuda")
    flag.zero_()
    capi.call("aeon_a64_repack_device", capi.vp(d_swp), capi.vp(d_sws), N, K, 4,
              8, 32, capi.vp(out_p), capi.vp(out_s4), capi.vp(flag), h.stream_ptr())
    assert int(flag.item()) == 0
    hp = np.empty(N * K // 8, dtype=np.uint32)
    hs = np.empty(N * K // 32, dtype=np.uint16)
    capi.call("aeon_a64_repack_host", h.u32p(swp), h.u16p(sws), N, K, 4, 8, 32, h.u32p(hp), h.u16p(hs))
    assert np.array_equal(out_p.cpu().numpy().view(np.uint32), hp)
    assert np.array_equal(out_s4.cpu().numpy().view(np.uint16), hs)


@pytest.mark.parametrize("score_kind,k,scaling", [(1, 8, 1.0), (0, 6, 1.5)])
def test_router_ids_bit_exact_on_identical_logits(orc, score_kind, k, scaling):
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(17)
    T, E = 96, 256
    logits = rng.normal(0, 2.0, (T, E)).astype(np.float32)
    bias = rng.normal(0, 0.1, E).astype(np.float32)
    # constructed ties: four experts share the top biased score (lowest index must win)
    logits[0, [7, 40, 41, 200]] = 6.0
    bias[[7, 40, 41, 200]] = 0.25
    logits[1, :] = 0.5  # all equal up to the bias
    d_ids = torch.zeros(T, k, dtype=torch.int32, device="cuda")
    d_w = torch.zeros(T, k, dtype=torch.float32, device="cuda")
    d_logits, d_bias = h.to_dev(logits), h.to_dev(bias)  # named: a temporary's memory is reused
    capi.call("aeon_moe_router", capi.vp(d_logits), capi.vp(d_bias), None, None,
              capi.vp(d_w), capi.vp(d_ids), T, E, k, C.c_float(scaling), 1, score_kind,
              h.stream_ptr())
    ids, w = d_ids.cpu().numpy(), d_w.cpu().numpy()
    for t in range(T):
        oi, ow = orc.router_topk(logits[t].astype(np.float64), bias.astype(np.float64), k, scaling,
                                 score_kind)
        assert np.array_equal(ids[t], oi), t
        assert np.abs(w[t] - ow).max() <= 1e-5 * np.abs(ow).max()
    assert list(ids[0][:4]) == [7, 40, 41, 200]
    # bias-before-activation is a different (wrong) rule and must give a different selection somewhere
    wrong = [orc.router_topk(logits[t].astype(np.float64), bias.astype(np.float64), k, scaling,
                             score_kind, bias_before=True)[0] for t in range(T)]
    assert any(not np.array_equal(ids[t], wrong[t]) for t in range(T))
    # no bias, hash branch
    table = rng.integers(0, E, (50, k)).astype(np.int64)
    tok = rng.integers(0, 50, T).astype(np.int32)
    d_table, d_tok = h.to_dev(table), h.to_dev(tok)
    capi.call("aeon_moe_router", capi.vp(d_logits), None, capi.vp(d_table),
              capi.vp(d_tok), capi.vp(d_w), capi.vp(d_ids), T, E, k, C.c_float(scaling), 1,
              score_kind, h.stream_ptr())
    ids = d_ids.cpu().numpy()
    assert np.array_equal(ids, table[tok].astype(np.int32))


@pytest.mark.parametrize("score_kind,exact_from", [(1, 8), (0, 16)])
def test_router_near_ties_order_like_the_oracle(orc, score_kind, exact_from, capsys):
    """How far "ids bit-exact" reaches. The device scores and selects in fp64 with its own exp /
    log1p / sqrt; the oracle with the host's. Two candidates whose biased scores differ by a few
    fp64 units in the last place (relative 1e-16) can therefore be ordered differently. The
    probes are built on the host: two live experts with random fp32 logits, the second's bias the
    fp32 nearest the score difference, the first's a tiny fp32 that closes the remaining gap to
    j units in the last place (a bias of magnitude 1e-9 has an fp32 spacing far below one fp64
    unit at 1), j from -64 to 64; six other experts far below. From `exact_from` units on the
    device must pick what the oracle picks, for every probe; below that the agreement is
    printed (measured: 1 probe of 150 differs for sigmoid out to 4 units, 5 of 150 for
    sqrt(softplus) at 0..1 units, one run with other draws showed single ones out to 6)."""
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(3 + score_kind)
    E, js = 8, [-64, -32, -16, -8, -4, -3, -2, -1, 0, 1, 2, 3, 4, 8, 16, 32, 64]
    logits_rows, bias_rows, meta = [], [], []
    while len(meta) < 150 * len(js):
        la, lb = rng.normal(0, 2, 2).astype(np.float32)
        sa, sb = orc.router_scores(np.array([la, lb], dtype=np.float64), score_kind)
        bb = np.float32(sa - sb)
        if not 1e-3 < abs(float(bb)) < 0.5:
            continue
        ulp = np.spacing(max(sa, sb + float(bb)))
        pa, pb = (int(v) for v in rng.permutation(E)[:2])
        for j in js:
            logits = np.full(E, -30.0, dtype=np.float32)
            bias = np.zeros(E, dtype=np.float32)
            logits[pa], logits[pb] = la, lb
            bias[pa], bias[pb] = np.float32((sb + float(bb) - sa) + j * ulp), bb
            logits_rows.append(logits)
            bias_rows.append(bias)
            meta.append(j)
    agree = {j: [0, 0] for j in js}
    ids = torch.zeros(1, 1, dtype=torch.int32, device="cuda")
    w = torch.zeros(1, 1, dtype=torch.float32, device="cuda")
    for logits, bias, j in zip(logits_rows, bias_rows, meta):
        oi, _ = orc.router_topk(logits.astype(np.float64), bias.astype(np.float64), 1, 1.0, score_kind)
        d_l, d_b = h.to_dev(logits.reshape(1, E)), h.to_dev(bias)
        capi.call("aeon_moe_router", capi.vp(d_l), capi.vp(d_b), None, None, capi.vp(w), capi.vp(ids),
                  1, E, 1, C.c_float(1.0), 1, score_kind, h.stream_ptr())
        agree[j][0] += int(ids.item() == oi[0])
        agree[j][1] += 1
    with capsys.disabled():
        print("\n  near-tie agreement (units in the last place: agreed/probes), score kind %d: %s"
              % (score_kind, ", ".join("%+d: %d/%d" % (j, a, n) for j, (a, n) in sorted(agree.items()))))
    for j, (a, n) in agree.items():
        if abs(j) >= exact_from:
            assert a == n, (score_kind, j, a, n)
    assert sum(a for a, _ in agree.values()) >= 0.97 * sum(n for _, n in agree.values())


@pytest.mark.parametrize("T,H,E", [(5, 1024, 10), (33, 896, 6), (3, 7168, 258), (17, 200, 64)])
def test_router_logits_at_expert_counts_not_divisible_by_four(orc, T, H, E):
    """aeon_router_logits where a weight row is not a whole number of 16-byte vectors (E % 4 != 0)
    or the hidden size is not a whole number of chunks: the aligned fast path must step aside.
    Against the fp64 product; run twice for bit-reproducibility."""
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(T * 1000 + E)
    x = rng.normal(0, 1, (T, H)).astype(np.float16)
    wr = rng.normal(0, 0.05, (H, E)).astype(np.float32)
    d_x, d_wr = h.dev_half(x), h.to_dev(wr)
    n = capi.lib().aeon_router_logits_workspace_bytes(T, H, E)
    ws = torch.empty(max(n, 4), dtype=torch.uint8, device="cuda")
    outs = []
    for _ in range(2):
        out = torch.full((T, E), 7.0, dtype=torch.float32, device="cuda")
        capi.call("aeon_router_logits", capi.vp(d_x), H, capi.vp(d_wr), capi.vp(out), T, H, E,
                  capi.vp(ws), C.c_size_t(ws.numel()), h.stream_ptr())
        outs.append(out.cpu().numpy())
    want = x.astype(np.float64) @ wr.astype(np.float64)
    assert np.abs(outs[0] - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("T,slots,E", [(1, 8, 256), (7, 6, 256), (300, 6, 256), (64, 8, 8),
                                       (0, 8, 256), (2048, 8, 256), (64, 8, 1024),
                                       (128, 8, 256), (129, 8, 256), (1024, 1, 3), (171, 6, 1024),
                                       (8192, 8, 256), (5000, 3, 1000)])
def test_expert_permutation_bit_exact(orc, T, slots, E):
    """Cases of tests/test_expert_permutation.cpp (T=1,7,300,64 at E=8, 0) plus the prefill size
    and the sizes either side of 1024 draws, where the one-launch form hands over to the
    two-launch form: equality with the host stable counting sort, which implies the five
    invariants."""
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(T * 31 + E)
    ids = rng.integers(0, E, (T, slots)).astype(np.int32)
    if T >= 7:
        ids[3, slots - 1] = -1      # out-of-range ids are dropped, not trusted
        ids[5, 0] = E
    wts = rng.random((T, slots)).astype(np.float32)
    n = max(T * slots, 1)
    d_off = torch.full((E + 1,), -7, dtype=torch.int32, device="cuda")
    d_tok = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    d_drw = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    d_wp = torch.zeros(n, dtype=torch.float32, device="cuda")
    d_ids = h.to_dev(ids.reshape(-1)) if T else d_tok
    d_wd = h.to_dev(wts.reshape(-1)) if T else d_wp
    capi.call("aeon_expert_permutation", capi.vp(d_ids), T, slots, E, capi.vp(d_off),
              capi.vp(d_tok), capi.vp(d_drw), capi.vp(d_wd), capi.vp(d_wp), h.stream_ptr())
    off, tok, drw = orc.expert_permutation(ids, T, slots, E)
    assert np.array_equal(d_off.cpu().numpy(), off)
    placed = int(off[E])
    assert np.array_equal(d_tok.cpu().numpy()[:placed], tok[:placed])
    assert np.array_equal(d_drw.cpu().numpy()[:placed], drw[:placed])
    if placed:
        assert np.array_equal(d_wp.cpu().numpy()[:placed], wts.reshape(-1)[drw[:placed]])


# Chained results (gate/up -> fp16 hidden -> W2 -> reduce over nine experts) against the fp64
# oracle, printed by the full-size tests as relative errors with the denominator floored at a
# fraction f of the peak (helpers.error_report):
#   * f = 1: the largest error over the peak. This is what the reference's own expert gates call
#     max_rel and bound by 6e-3; the stated tolerance of 1e-2 is read the same way. Observed
#     4e-4 (decode kernels) and 9e-4 (grouped GEMM, which rounds every weight times its scale to
#     fp16 once, as the reference's grouped feed does).
#   * f = 0.1: outputs of a tenth of the peak and more are within 1e-2 of themselves.
#   * f = 1e-2 and 1e-3 (`compare`'s default): set by outputs where nine contributions of the
#     size of the peak cancel to a hundredth or a thousandth of it; the error there is still a
#     few 1e-4 of the peak, which is several per cent (decode) to tens of per cent (grouped) of
#     such an element. Printed with the element's size; not a pass criterion beyond "finite".
PEAK_BOUND = 6e-3
TENTH_OF_PEAK_REL_BOUND = 1e-2


def check_chained(report):
    assert report["rel_floor_1"] <= PEAK_BOUND, report
    assert report["rel_floor_1e-1"] <= TENTH_OF_PEAK_REL_BOUND, report
    assert np.isfinite(report["rel_floor_1e-3"]), report


def _oracle_layer(orc, h, experts, x, ids, weights, shared, limit):
    """out[t] = half-rounded-shared + sum_k w_k * FFN_{id_k}(x_t), per the fixed-order combine,
    with every FFN from the fp64 oracle (hidden rounded to fp16 as the device stores it)."""
    T, k = ids.shape
    H = x.shape[1]
    contrib = np.zeros((T, k, H))
    for e in np.unique(ids):
        rows, slots = np.nonzero(ids == e)
        o = experts[int(e)].ffn(x[rows], limit, round_hidden=True)
        for i, (t, s) in enumerate(zip(rows, slots)):
            contrib[t, s] = float(weights[t, s]) * o[i]
    out = np.empty((T, H))
    for t in range(T):
        sh = None
        if shared is not None:
            sh = shared.ffn(x[t:t + 1], limit, round_hidden=True)[0].astype(np.float16).astype(np.float64)
        out[t] = orc.moe_combine(contrib[t], sh)
    return out


def _oracle_layer_streamed(orc, make_expert, x, ids, weights, shared, limit):
    """_oracle_layer for samples that touch many full-size experts: every expert is made when its
    turn comes (make_expert(id)) and dropped afterwards, so only one is in host memory at a time."""
    T, k = ids.shape
    H = x.shape[1]
    contrib = np.zeros((T, k, H))
    for e in np.unique(ids):
        rows, slots = np.nonzero(ids == e)
        o = make_expert(int(e)).ffn(x[rows], limit, round_hidden=True)
        for i, (t, s) in enumerate(zip(rows, slots)):
            contrib[t, s] = float(weights[t, s]) * o[i]
    out = np.empty((T, H))
    sh = None
    if shared is not None:
        sh = shared.ffn(x, limit, round_hidden=True).astype(np.float16).astype(np.float64)
    for t in range(T):
        out[t] = orc.moe_combine(contrib[t], None if sh is None else sh[t])
    return out


@pytest.mark.parametrize("B", [1, 8, 32, 64])
def test_config2_moe_layer_decode_reduced_experts(orc, B):
    """benchmark config 2 at full hidden/intermediate with a 24-expert layer (so the oracle can
    regenerate every expert): fp32 router [7168 x E], sigmoid + bias, top-8, renormalised, one
    always-on shared expert, int4 group-128 experts."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, limit = 7168, 2048, 24, 8, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=2, first_expert_id=0) == 0
    wr = synth.router_weight(2, H, E)
    bias = synth.router_bias(2, E)
    layer = moe.MoeLayer(pool, E, k, True, limit, h.to_dev(wr), h.to_dev(bias), score_kind=1)
    x = synth.activations(2, B, H, unit=B)
    d_x = h.dev_half(x)
    out, ids, w = layer.decode(d_x)
    logits = layer.router_logits(d_x).cpu().numpy()
    torch.cuda.synchronize()
    ids, w, out = ids.cpu().numpy(), w.cpu().numpy(), out.cpu().numpy()
    # logits: fp32 device accumulation against the fp64 matvec
    want_logits = x.astype(np.float64) @ wr.astype(np.float64)
    assert np.abs(logits - want_logits).max() <= 1e-5 * np.abs(want_logits).max()
    # ids / weights: the oracle on the device's own fp32 logits, bit-exact ids
    for t in range(B):
        oi, ow = orc.router_topk(logits[t].astype(np.float64), bias.astype(np.float64), k, 1.0, 1)
        assert np.array_equal(ids[t], oi)
        assert np.abs(w[t] - ow).max() <= 1e-5
        assert abs(w[t].sum() - 1.0) < 1e-5
    experts = {int(e): h.Expert(2, int(e), H, I) for e in np.unique(ids)}
    shared = h.Expert(2, E, H, I)
    want = _oracle_layer(orc, h, experts, x, ids, w, shared, limit)
    assert np.abs(want).max() > 1.0
    assert np.abs(out - want).max() <= 6e-3 * np.abs(want).max()
    # routed-only entry point with the same routing gives the same bits
    d_ids, d_w = h.to_dev(ids), h.to_dev(w)
    again = layer.routed(d_x, d_ids, d_w)
    assert np.array_equal(again.cpu().numpy(), out)
    # and a run is bit-reproducible
    out2, _, _ = layer.decode(d_x)
    assert np.array_equal(out2.cpu().numpy(), out)


@pytest.mark.parametrize("H,I,E,k,T,shared", [
    (4096, 2048, 64, 6, 64, False),     # the checkpoint's own shape: wide decode segments
    (4096, 2048, 64, 6, 1, False),      # one token: slots read directly, K-split kernels
    (4096, 2048, 32, 6, 48, True),      # hot experts: two token tiles per segment (wide form)
    (4096, 2048, 64, 6, 300, False),    # a prefill chunk: grouped windows
    (7168, 2048, 24, 8, 64, True),      # K too long for the wide form's LDS: K-split at a batch
])
def test_group32_scales_on_the_resident_path(orc, H, I, E, k, T, shared):
    """Experts with a scale of their own per 32 columns (the `.aeon` format's grouping,
    swizzled_expert_format.hpp:18-23; the reference model is hidden 4096, intermediate 2048,
    top-6) through aeon_moe_layer_routed with the four-scale packing. Sampled tokens against the
    oracle to 6e-3 of the peak, every token finite, run twice for the same bits; the decode
    steps are also held to the `.aeon`-layout trio on the same payloads, which applies the same
    exact fp32 scale per 32 columns."""
    torch, h, capi, moe, synth = _setup()
    limit = 10.0
    pool = moe.ExpertPool(E + (1 if shared else 0), H, I, scale_group=32)
    assert pool.fill_synthetic(seed=90, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, shared, limit)
    rng = np.random.default_rng(T + E)
    hot = E if T != 48 else 3
    ids = np.stack([np.concatenate([rng.permutation(hot)[:min(k, hot)],
                                    hot + rng.permutation(E - hot)[:k - min(k, hot)]])
                    for _ in range(T)]).astype(np.int32)
    w = synth.route_weights(90, T * k).reshape(T, k).astype(np.float32)
    x = synth.activations(90, T, H)
    d_x, d_ids, d_w = h.dev_half(x), h.to_dev(ids), h.to_dev(w)
    out = layer.routed(d_x, d_ids, d_w).cpu().numpy()
    assert np.isfinite(out).all()
    assert np.array_equal(layer.routed(d_x, d_ids, d_w).cpu().numpy(), out)
    sample = sorted({0, T // 2, T - 1})
    needed = sorted({int(e) for t in sample for e in ids[t]})
    experts = {e: h.Expert(90, e, H, I, 32) for e in needed}
    always = h.Expert(90, E, H, I, 32) if shared else None
    want = _oracle_layer(orc, h, experts, x[sample], ids[sample], w[sample], always, limit)
    assert np.abs(want).max() > 0.5
    assert np.abs(out[sample] - want).max() <= 6e-3 * np.abs(want).max()
    # one-scale reading of the same experts is a different layer: the check is not vacuous
    wrong = {e: h.Expert(90, e, H, I, 128) for e in needed[:1]}
    assert np.abs(wrong[needed[0]].w1.decode() - experts[needed[0]].w1.decode()).max() > 1e-3
    if T <= 64 and not shared:
        # the `.aeon`-layout trio of one token on the same payloads
        t = sample[-1]
        w13, w2 = capi.W13Table(), capi.W2Table()
        keep = []
        for j in range(k):
            e = experts[int(ids[t, j])]
            dev = [h.dev_u32(e.w1.swz_packed), h.dev_u16(e.w1.swz_scale), h.dev_u32(e.w3.swz_packed),
                   h.dev_u16(e.w3.swz_scale), h.dev_u32(e.w2.swz_packed), h.dev_u16(e.w2.swz_scale)]
            keep.append(dev)
            w13.w1[j], w13.s1[j], w13.w3[j], w13.s3[j] = (dev[0].data_ptr(), dev[1].data_ptr(),
                                                          dev[2].data_ptr(), dev[3].data_ptr())
            w2.w2[j], w2.s2[j] = dev[4].data_ptr(), dev[5].data_ptr()
        hidden = torch.zeros(k, I, dtype=torch.float16, device="cuda")
        contrib = torch.zeros(k, H, dtype=torch.float32, device="cuda")
        trio = torch.zeros(H, dtype=torch.float16, device="cuda")
        xt = d_x[t].contiguous()
        wt = d_w[t].contiguous()
        capi.call("aeon_moe_gemv_w13_swiglu", capi.vp(xt), C.byref(w13), capi.vp(hidden), None, I, k,
                  I, H, 4, 8, C.c_float(limit), h.stream_ptr())
        capi.call("aeon_moe_fused_w2_contrib", capi.vp(hidden), C.byref(w2), capi.vp(wt),
                  capi.vp(contrib), k, H, I, 8, 4, h.stream_ptr())
        capi.call("aeon_moe_accumulate_fixed_order", capi.vp(contrib), k, None, capi.vp(trio), H,
                  h.stream_ptr())
        trio = trio.cpu().numpy().astype(np.float64)
        assert np.abs(trio - out[t]).max() <= 2e-3 * np.abs(trio).max()


def test_config2_full_size_sampled(orc):
    """benchmark config 2 as written: batch 64, top-8 of 256 experts + the always-on one, fp32
    router with sigmoid scores and bias, H=7168, I=2048. The oracle covers a sample of tokens
    (ids bit-exact on the device's logits for all of them); the rest is covered by properties
    that hold at any size: a token's output does not depend on the other tokens of the batch
    (same bits under a reversed batch, same values to summation order when it is run alone
    through the K-split kernels) and a second run gives the same bits."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, B, limit = 7168, 2048, 256, 8, 64, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=0, first_expert_id=0) == 0
    wr, bias = synth.router_weight(0, H, E), synth.router_bias(0, E)
    layer = moe.MoeLayer(pool, E, k, True, limit, h.to_dev(wr), h.to_dev(bias), score_kind=1)
    x = synth.activations(0, B, H, unit=1000 * B)
    d_x = h.dev_half(x)
    out_t, ids_t, w_t = layer.decode(d_x)
    logits = layer.router_logits(d_x).cpu().numpy()
    torch.cuda.synchronize()
    out, ids, w = out_t.cpu().numpy(), ids_t.cpu().numpy(), w_t.cpu().numpy()
    assert np.isfinite(out).all()
    for t in range(B):
        oi, ow = orc.router_topk(logits[t].astype(np.float64), bias.astype(np.float64), k, 1.0, 1)
        assert np.array_equal(ids[t], oi)
        assert np.abs(w[t] - ow).max() <= 1e-5
    assert 60 <= np.unique(ids).size <= 140   # the biased router concentrates the routing
    # eight tokens spread over the batch; the experts' payloads come back from the device
    # generator (held to the host generator bit for bit above), one expert at a time
    sample = [0, 9, 18, 27, 36, 45, 54, 63]
    want = _oracle_layer_streamed(orc, lambda e: h.GeneratedExpert(0, e, H, I), x[sample], ids[sample],
                                  w[sample], h.GeneratedExpert(0, E, H, I), limit)
    assert np.abs(want).max() > 1.0
    report = h.error_report(out[sample], want)
    print("config 2 full size, %d tokens against the oracle: %s" % (len(sample), report))
    check_chained(report)
    again, _, _ = layer.decode(d_x)
    assert np.array_equal(again.cpu().numpy(), out)
    rev = layer.routed(d_x.flip(0).contiguous(), ids_t.flip(0).contiguous(),
                       w_t.flip(0).contiguous()).flip(0).cpu().numpy()
    assert np.array_equal(rev, out)
    for t in (5, 40):
        alone = layer.routed(d_x[t:t + 1], ids_t[t:t + 1], w_t[t:t + 1]).cpu().numpy()
        assert np.abs(alone[0] - out[t]).max() <= 1e-3 * np.abs(out[t]).max()
    # two tokens: one segment per draw, the always-on expert over both, wide W2 launch
    pair = layer.routed(d_x[40:42], ids_t[40:42], w_t[40:42]).cpu().numpy()
    assert np.abs(pair - out[40:42]).max() <= 1e-3 * np.abs(out[40:42]).max()


@pytest.mark.parametrize("H,I,B", [(256, 128, 3), (256, 384, 5), (768, 256, 17), (256, 128, 70),
                                   (256, 128, 128), (256, 128, 129), (256, 128, 256),
                                   (256, 128, 257)])
def test_layer_on_minimal_shapes(orc, H, I, B):
    """Shapes with fewer 128-column groups than a workgroup has K-split waves (a wave with no
    group of its own must not fetch anything outside the matrix), odd group counts for the
    pipeline tails, and batches at and just over the grouped path's threshold (128 tokens; with
    five experts every larger batch has enough positions per expert for it) and around two full
    windows (256, 257) on a one-group K."""
    torch, h, capi, moe, synth = _setup()
    E, k, limit = 5, 2, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=21, first_expert_id=0) == 0
    wr, bias = synth.router_weight(21, H, E), synth.router_bias(21, E)
    layer = moe.MoeLayer(pool, E, k, True, limit, h.to_dev(wr), h.to_dev(bias), score_kind=1)
    x = synth.activations(21, B, H, unit=B)
    d_x = h.dev_half(x)
    out, ids, w = layer.decode(d_x)
    torch.cuda.synchronize()
    ids, w, out = ids.cpu().numpy(), w.cpu().numpy(), out.cpu().numpy()
    experts = {int(e): h.Expert(21, int(e), H, I) for e in np.unique(ids)}
    shared = h.Expert(21, E, H, I)
    want = _oracle_layer(orc, h, experts, x, ids, w, shared, limit)
    assert np.abs(out - want).max() <= 6e-3 * np.abs(want).max()


@pytest.mark.parametrize("T,E,k", [(300, 64, 2), (200, 256, 4), (383, 128, 4)])
def test_chunks_with_few_positions_per_expert_stay_on_the_decode_kernels(orc, T, E, k):
    """Above 128 tokens the grouped GEMM only takes over when the experts hold more than twelve
    draws each on average; a chunk of many tokens over many experts keeps the weight-streaming
    kernels (segments of up to 32 positions, several per expert where the routing concentrates).
    Sampled tokens against the oracle, and the same chunk cut into two calls of at most 128
    tokens -- which always run on those kernels -- has to give the same bits (a token's result
    does not depend on which other tokens share its segment; the shapes are such that whole and
    parts take the same form, K-split or wide, of each launch)."""
    torch, h, capi, moe, synth = _setup()
    H, I, limit = 512, 256, 7.0
    assert T > 128 and T * k <= 12 * E
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=71, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, True, limit)
    ids, w = synth.zipf_routing(71, T, E, k, s=1.1)
    x = synth.activations(71, T, H)
    d_x, d_ids, d_w = h.dev_half(x), h.to_dev(ids), h.to_dev(w)
    out = layer.routed(d_x, d_ids, d_w)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    cut = 128
    parts = [layer.routed(d_x[a:b].contiguous(), d_ids[a:b].contiguous(), d_w[a:b].contiguous()).cpu().numpy()
             for a, b in ((0, cut), (cut, min(2 * cut, T)), (min(2 * cut, T), T)) if b > a]
    assert np.array_equal(np.concatenate(parts), got)
    rows = sorted(set([0, T // 2, T - 1, 129 % T]))
    experts = {int(e): h.Expert(71, int(e), H, I) for e in np.unique(ids[rows])}
    shared = h.Expert(71, E, H, I)
    want = _oracle_layer(orc, h, experts, x[rows], ids[rows], w[rows], shared, limit)
    assert np.abs(got[rows] - want).max() <= 6e-3 * np.abs(want).max()


@pytest.mark.parametrize("T", [1, 6, 150, 300])
def test_out_of_range_ids_contribute_nothing(orc, T):
    """An id outside [0, experts) is dropped by the permutation (as the reference's does); the
    slot-ordered reduce must then leave that slot out instead of adding a row nobody wrote. Run
    on the single-token path (which reads the ids directly; all three of its slots are bad), on
    the decode (segment) path and on the grouped path, after a call that left other values in
    the workspace."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, limit = 256, 256, 12, 3, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=31, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, True, limit)
    rng = np.random.default_rng(31)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    w = synth.route_weights(31, T * k).reshape(T, k).astype(np.float32)
    x = synth.activations(31, T, H)
    d_x = h.dev_half(x)
    layer.routed(d_x, h.to_dev(ids), h.to_dev(w))          # fills every contribution row
    bad = ids.copy()
    bad[min(1, T - 1), 0], bad[T - 1, k - 1], bad[min(2, T - 1), 1] = -1, E, 1 << 20
    out = layer.routed(d_x, h.to_dev(bad), h.to_dev(w)).cpu().numpy()
    experts = {e: h.Expert(31, e, H, I) for e in range(E)}
    shared = h.Expert(31, E, H, I)
    check = sorted({0, min(1, T - 1), min(2, T - 1), T - 1})
    want = np.zeros((len(check), H))
    for n, t in enumerate(check):
        keep = [s for s in range(k) if 0 <= bad[t, s] < E]
        row = _oracle_layer(orc, h, experts, x[t:t + 1], bad[t:t + 1, keep], w[t:t + 1, keep], shared, limit)
        want[n] = row[0]
    assert np.isfinite(out).all()
    assert np.abs(out[check] - want).max() <= 6e-3 * np.abs(want).max()


@pytest.mark.parametrize("shared", [True, False])
def test_few_tokens_read_their_slots_directly(orc, shared):
    """One or two tokens take no permutation launch: the kernels read the ids and weights as they
    are, one segment per draw (tokens 0 and 1 share expert 2 here, which is then streamed twice).
    A token's result has to be the one it gets in a six-token batch, which goes through the
    permutation (to summation order: the two may pick different kernel forms), bit for bit the
    one it gets alone, and the oracle's; without an always-on expert the routed sum is added to
    what the output holds."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, limit = 512, 384, 10, 4, 7.0
    pool = moe.ExpertPool(E + (1 if shared else 0), H, I)
    assert pool.fill_synthetic(seed=33, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, shared, limit)
    ids = np.array([[7, 2, 9, 0], [1, 2, 3, 4], [5, 6, 7, 8], [9, 8, 1, 0], [3, 5, 7, 9], [0, 2, 4, 6]],
                   dtype=np.int32)
    T = ids.shape[0]
    w = synth.route_weights(33, T * k).reshape(T, k).astype(np.float32)
    x = synth.activations(33, T, H)
    d_x, d_ids, d_w = h.dev_half(x), h.to_dev(ids), h.to_dev(w)
    start = synth.activations(34, T, H).astype(np.float16)
    six = layer.routed(d_x, d_ids, d_w, out=h.to_dev(start.copy())).cpu().numpy()
    experts = {int(e): h.Expert(33, int(e), H, I) for e in np.unique(ids[:4])}
    sh = h.Expert(33, E, H, I) if shared else None
    want = _oracle_layer(orc, h, experts, x[:4], ids[:4], w[:4], sh, limit)
    if not shared:
        want = want + start[:4].astype(np.float64)
    alone = [layer.routed(d_x[t:t + 1], d_ids[t:t + 1], d_w[t:t + 1],
                          out=h.to_dev(start[t:t + 1].copy())).cpu().numpy()[0] for t in range(4)]
    for n in (1, 2, 3, 4):
        got = layer.routed(d_x[:n], d_ids[:n], d_w[:n], out=h.to_dev(start[:n].copy())).cpu().numpy()
        assert np.abs(got - want[:n]).max() <= 6e-3 * np.abs(want).max(), n
        assert np.abs(got - six[:n]).max() <= 1e-3 * np.abs(six).max(), n
        for t in range(n):
            assert np.array_equal(got[t], alone[t]), (n, t)


def test_decode_segments_of_two_token_tiles(orc):
    """A decode batch in which both launches take the wide form (many live experts) and single
    experts hold 40, 20, 17 and 16 positions: segments of 32+8, 20, 17 and 16 positions, i.e. the
    two-tile path with full, partial and barely-started second tiles next to one-tile segments.
    The always-on expert's 64 tokens make two full two-tile segments."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, T, limit = 1024, 2048, 80, 2, 64, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=13, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, True, limit)
    ids = np.empty((T, k), dtype=np.int32)
    ids[:40, 0] = 3                       # 40 positions
    ids[40:60, 0] = 7                     # 20
    ids[60:, 0] = 11                      # 4
    ids[:17, 1] = 5                       # 17
    ids[17:33, 1] = 9                     # 16
    ids[33:, 1] = 20 + np.arange(T - 33)  # one each: keeps the live-expert count high
    w = synth.route_weights(13, T * k).reshape(T, k).astype(np.float32)
    x = synth.activations(13, T, H)
    d_x, d_ids, d_w = h.dev_half(x), h.to_dev(ids), h.to_dev(w)
    out = layer.routed(d_x, d_ids, d_w).cpu().numpy()
    check = [0, 16, 31, 32, 39, 40, 59, 60, 63]
    needed = sorted(set(int(e) for t in check for e in ids[t]))
    experts = {e: h.Expert(13, e, H, I) for e in needed}
    shared = h.Expert(13, E, H, I)
    want = _oracle_layer(orc, h, experts, x[check], ids[check], w[check], shared, limit)
    assert np.abs(want).max() > 0.5
    assert np.abs(out[check] - want).max() <= 6e-3 * np.abs(want).max()
    # reversed token order: other positions share a segment, a token's own sums keep their order,
    # so its output keeps its bits
    rev = layer.routed(d_x.flip(0).contiguous(), d_ids.flip(0).contiguous(),
                       d_w.flip(0).contiguous()).flip(0).cpu().numpy()
    assert np.array_equal(rev, out)
    # the K-split kernels a small batch takes sum K in four interleaved parts: same values to
    # fp32 summation order
    small = layer.routed(d_x[:8], d_ids[:8], d_w[:8]).cpu().numpy()
    assert np.abs(small - out[:8]).max() <= 1e-3 * np.abs(out[:8]).max()


def test_prefill_grouped_small_full_oracle(orc):
    """The grouped path end to end on a shape small enough for the oracle to cover every token:
    ragged experts (empty, a few tokens, more than one 128-position tile), top-4 of 16, shared
    expert, strided activation rows."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, T, limit = 1024, 512, 16, 4, 300, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=9, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, True, limit)
    ids, w = synth.zipf_routing(9, T, E, k, s=1.1)
    ids[ids == 5] = 6                      # expert 5 gets no tokens at all
    ids[:, 1] = np.where(ids[:, 0] == 6, 7, 6)  # and expert 6 sees nearly every token (> 128)
    for t in range(T):                      # keep the k experts of a token distinct
        seen = set()
        for s in range(k):
            while int(ids[t, s]) in seen or int(ids[t, s]) == 5:
                ids[t, s] = (ids[t, s] + 1) % E
            seen.add(int(ids[t, s]))
    counts = np.bincount(ids.ravel(), minlength=E)
    assert counts[5] == 0 and counts.max() > 128 and (counts[counts > 0] < 16).any()
    x = synth.activations(9, T, H)
    pitch = H + 64
    xbuf = torch.zeros(T, pitch, dtype=torch.float16, device="cuda")
    xbuf[:, :H] = h.dev_half(x)
    d_ids, d_w = h.to_dev(ids), h.to_dev(w)
    out = layer.routed(xbuf[:, :H], d_ids, d_w)
    torch.cuda.synchronize()
    out = out.cpu().numpy()
    experts = {int(e): h.Expert(9, int(e), H, I) for e in np.unique(ids)}
    shared = h.Expert(9, E, H, I)
    want = _oracle_layer(orc, h, experts, x, ids, w, shared, limit)
    assert np.abs(want).max() > 0.5
    # fp16 scale multiply per weight + fp16 hidden store: the chained bound of the reference's
    # FFN gates, as a fraction of the peak
    assert np.abs(out - want).max() <= 6e-3 * np.abs(want).max()
    # grouped path vs the weight-streaming path on the same routing: a summation-order /
    # scale-rounding difference only (tests/test_moe_grouped_batch_parity.cpp:283-284 asks 1e-3)
    dec = layer.routed(xbuf[:64, :H], d_ids[:64], d_w[:64]).cpu().numpy()
    assert np.abs(out[:64] - dec).max() <= 2e-3 * np.abs(dec).max()
    # bit-reproducible
    again = layer.routed(xbuf[:, :H], d_ids, d_w).cpu().numpy()
    assert np.array_equal(again, out)


def test_prefill_window_bodies_at_every_live_count(orc):
    """One expert per window size class and its edges: the grouped kernel picks a body by the
    window's live token tiles (1, 2, 3, 4, 6 or 8 of 16 positions), so experts are given exactly
    1, 15, 16, 17, ... 128, 129 and 200 tokens (top-1 routing makes the counts exact) and every
    token is checked against the oracle."""
    torch, h, capi, moe, synth = _setup()
    H, I, limit = 512, 256, 7.0
    counts = [1, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65, 80, 95, 96, 97, 111, 112, 113, 127,
              128, 129, 200]
    E, T = len(counts), sum(counts)
    pool = moe.ExpertPool(E, H, I)
    assert pool.fill_synthetic(seed=21, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, 1, False, limit)
    rng = np.random.default_rng(21)
    ids = np.repeat(np.arange(E, dtype=np.int32), counts)
    rng.shuffle(ids)
    ids = ids.reshape(T, 1)
    w = (0.25 + rng.random((T, 1))).astype(np.float32)
    x = synth.activations(21, T, H)
    out = layer.routed(h.dev_half(x), h.to_dev(ids), h.to_dev(w))
    torch.cuda.synchronize()
    out = out.cpu().numpy()
    experts = {e: h.Expert(21, e, H, I) for e in range(E)}
    want = _oracle_layer(orc, h, experts, x, ids, w, None, limit)
    peak = np.abs(want).max()
    assert peak > 0.1
    for e in range(E):
        rows = np.nonzero(ids[:, 0] == e)[0]
        assert len(rows) == counts[e]
        assert np.abs(out[rows] - want[rows]).max() <= 6e-3 * peak, (e, counts[e])


def test_config3_prefill_full_size_sampled(orc):
    """benchmark config 3 at full size: 2048 tokens, top-8 of 256 experts with Zipf(1.1)
    popularity, H=7168, I=2048, + shared expert. The oracle covers a sample of tokens; the rest
    is covered by parity with the decode path on 64 tokens and by a token-permutation property
    (reversing the token order permutes the output rows and nothing else)."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, T, limit = 7168, 2048, 256, 8, 2048, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=0, first_expert_id=0) == 0
    layer = moe.MoeLayer(pool, E, k, True, limit)
    ids, w = synth.zipf_routing(0, T, E, k, s=1.1)
    counts = np.bincount(ids.ravel(), minlength=E)
    assert counts.max() > 500 and (counts < 16).sum() > 20
    x = synth.activations(0, T, H, unit=3)
    d_x, d_ids, d_w = h.dev_half(x), h.to_dev(ids), h.to_dev(w)
    out_t = layer.routed(d_x, d_ids, d_w)
    torch.cuda.synchronize()
    out = out_t.cpu().numpy()
    assert np.isfinite(out).all()
    # The sample is stratified over what the grouped kernel does differently: for every window
    # body (1, 2, 3, 4, 6 and 8 live token tiles) the first and the last position of a window of
    # that size, two positions deep in the hottest expert's list (beyond its 1024th), and three
    # fixed tokens. A sampled token's whole output is checked, i.e. all eight of its experts and
    # the always-on one, whatever windows those draws fall in.
    order = np.argsort(ids.ravel(), kind="stable")          # draws by expert, ascending draw
    start = np.concatenate([[0], np.cumsum(counts)])
    token_of = lambda e, rank: int(order[start[e] + rank] // k)
    sample = {0, 123, 555, 777, 1024, 1500, 2047}
    hottest = int(counts.argmax())
    assert counts[hottest] > 1700
    sample |= {token_of(hottest, 1100), token_of(hottest, 1700)}
    classes_seen = set()
    for live in (1, 2, 3, 4, 6, 8):
        for e in np.argsort(-counts):
            tail = int(counts[e]) % 128 or (128 if counts[e] else 0)
            tiles = (tail + 15) // 16
            body = 1 if tiles <= 1 else 2 if tiles == 2 else 3 if tiles == 3 else 4 if tiles == 4 else 6 if tiles <= 6 else 8
            if counts[e] and body == live:
                first_of_window = int(counts[e]) - tail
                sample |= {token_of(int(e), first_of_window), token_of(int(e), int(counts[e]) - 1)}
                classes_seen.add(live)
                break
    assert classes_seen == {1, 2, 3, 4, 6, 8}
    sample = sorted(sample)
    assert len(sample) >= 16
    want = _oracle_layer_streamed(orc, lambda e: h.GeneratedExpert(0, e, H, I), x[sample], ids[sample],
                                  w[sample], h.GeneratedExpert(0, E, H, I), limit)
    report = h.error_report(out[sample], want)
    print("config 3 full size, %d tokens against the oracle: %s" % (len(sample), report))
    check_chained(report)
    dec = layer.routed(d_x[:64], d_ids[:64], d_w[:64]).cpu().numpy()
    assert np.abs(out[:64] - dec).max() <= 2e-3 * np.abs(dec).max()
    # reversed token order: same rows, reversed (per-token results do not depend on the batch)
    rev = layer.routed(d_x.flip(0).contiguous(), d_ids.flip(0).contiguous(),
                       d_w.flip(0).contiguous()).flip(0).cpu().numpy()
    assert np.abs(rev - out).max() <= 2e-3 * np.abs(out).max()


def test_random_layer_steps_against_oracle(orc):
    """Forty seeded random layer steps (hidden, intermediate, expert count, top-k, token count
    from 1 to 300, with and without an always-on expert, two ids out of range each): every token
    count class of the step -- direct slots, decode segments, grouped windows -- lands here with
    shapes the other tests do not use. Odd cases keep a scale of their own per 32 columns (the
    `.aeon` format's grouping, four scales per 128 columns in the packing), even ones one per
    128. Three tokens of each against the oracle, to 6e-3 of the peak; without an always-on
    expert the routed sum is added to what the output held."""
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(2024)
    for case in range(40):
        H = int(rng.choice([256, 512, 768, 1024]))
        I = int(rng.choice([128, 256, 384, 512]))
        E = int(rng.integers(2, 40))
        k = int(rng.integers(1, min(E, 8) + 1))
        T = int(rng.choice([1, 2, 3, 5, 16, 17, 33, 64, 100, 128, 129, 200, 257, 300]))
        shared = bool(rng.integers(0, 2))
        seed = 500 + case
        scale_group = 32 if case % 2 else 128
        pool = moe.ExpertPool(E + (1 if shared else 0), H, I, scale_group=scale_group)
        assert pool.fill_synthetic(seed=seed, first_expert_id=0) == 0
        layer = moe.MoeLayer(pool, E, k, shared, 7.0)
        ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
        if T > 2 and k > 1:
            ids[rng.integers(0, T), rng.integers(0, k)] = -1
            ids[rng.integers(0, T), rng.integers(0, k)] = E + 3
        w = synth.route_weights(seed, T * k).reshape(T, k).astype(np.float32)
        x = synth.activations(seed, T, H)
        start = synth.activations(seed + 1, T, H).astype(np.float16)
        out = layer.routed(h.dev_half(x), h.to_dev(ids), h.to_dev(w),
                           out=h.to_dev(start.copy())).cpu().numpy()
        what = (case, H, I, E, k, T, shared, scale_group)
        assert np.isfinite(out).all(), what
        check = sorted({0, T // 2, T - 1})
        need = sorted({int(e) for t in check for e in ids[t] if 0 <= e < E})
        experts = {e: h.Expert(seed, e, H, I, scale_group) for e in need}
        always = h.Expert(seed, E, H, I, scale_group) if shared else None
        for t in check:
            keep = [s for s in range(k) if 0 <= ids[t, s] < E]
            contrib = np.zeros((len(keep), H))
            for j, s_ in enumerate(keep):
                contrib[j] = float(w[t, s_]) * experts[int(ids[t, s_])].ffn(x[t:t + 1], 7.0, round_hidden=True)[0]
            if shared:
                first = always.ffn(x[t:t + 1], 7.0, round_hidden=True)[0].astype(np.float16).astype(np.float64)
            else:
                first = start[t].astype(np.float64)
            want = orc.moe_combine(contrib, first) if keep else first.astype(np.float16).astype(np.float64)
            assert np.abs(out[t] - want).max() <= 6e-3 * max(np.abs(want).max(), 1e-6), (what, t)


@pytest.mark.parametrize("B", [1, 8, 150, 300])
def test_layer_step_replays_from_a_captured_graph(orc, B):
    """The step allocates nothing, clears nothing with a memset and never synchronises, so it can
    be recorded into a HIP graph: the graph is replayed four times with new activations copied
    into its input buffer and eager work between the replays, and every replay has to give the
    bits of the eager step on the same activations (direct slots, decode segments, grouped
    windows)."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, limit = 512, 256, 20, 4, 7.0
    pool = moe.ExpertPool(E + 1, H, I)
    assert pool.fill_synthetic(seed=61, first_expert_id=0) == 0
    wr, bias = synth.router_weight(61, H, E), synth.router_bias(61, E)
    layer = moe.MoeLayer(pool, E, k, True, limit, h.to_dev(wr), h.to_dev(bias), score_kind=1)
    xs = [h.dev_half(synth.activations(61, B, H, unit=10 + r)) for r in range(4)]
    eager = []
    for x in xs:
        out, ids, w = layer.decode(x)
        eager.append((out.clone(), ids.clone(), w.clone()))
    torch.cuda.synchronize()
    x_in = xs[0].clone()
    out = torch.empty(B, H, dtype=torch.float16, device="cuda")
    ids = torch.empty(B, k, dtype=torch.int32, device="cuda")
    w = torch.empty(B, k, dtype=torch.float32, device="cuda")
    layer.decode(x_in, out, ids, w)          # warm: the workspace exists before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.decode(x_in, out, ids, w)
    for r in (1, 0, 3, 2):
        x_in.copy_(xs[r])
        scratch = layer.routed(xs[(r + 1) % 4], eager[(r + 1) % 4][1], eager[(r + 1) % 4][2])  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[r][0]), (B, r)
        assert torch.equal(ids, eager[r][1]) and torch.equal(w, eager[r][2]), (B, r)
        del scratch
