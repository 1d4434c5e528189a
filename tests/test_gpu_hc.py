"""GPU parity for the hyper-connection kernels and the stacked-layer decode step (config 4)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _setup():
    import torch
    assert torch.cuda.is_available()
    import helpers
    from project_aeon_amd import capi, moe, synth
    return torch, helpers, capi, moe, synth


def test_sinkhorn_against_oracle_and_closed_forms(orc):
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(3)
    T = 33
    mixes = rng.normal(size=(T, 24)).astype(np.float32)
    mixes[0] = 0.0
    scale = rng.normal(size=3).astype(np.float32)
    base = rng.normal(size=24).astype(np.float32)
    base0 = np.zeros(24, dtype=np.float32)
    for iters, b in ((20, base), (1, base), (20, base0)):
        d_m, d_s, d_b = h.to_dev(mixes), h.to_dev(scale), h.to_dev(b)
        pre = torch.zeros(T, 4, device="cuda")
        post = torch.zeros(T, 4, device="cuda")
        comb = torch.zeros(T, 16, device="cuda")
        capi.call("aeon_hc_sinkhorn_normalize", capi.vp(d_m), capi.vp(d_s), capi.vp(d_b),
                  capi.vp(pre), capi.vp(post), capi.vp(comb), T, C.c_float(1e-6), C.c_float(1e-6),
                  C.c_float(2.0), iters, h.stream_ptr())
        pre, post, comb = pre.cpu().numpy(), post.cpu().numpy(), comb.cpu().numpy()
        for t in range(T):
            op, oq, oc = orc.hc_sinkhorn(mixes[t], scale, b, 4, orc.hc_params(sinkhorn_iters=iters))
            assert np.abs(pre[t] - op).max() <= 1e-5      # tests/test_hc_sinkhorn.cpp tolerances
            assert np.abs(post[t] - oq).max() <= 1e-5
            assert np.abs(comb[t] - oc).max() <= 1e-5
        if iters == 20:
            c = comb.reshape(T, 4, 4)
            # doubly stochastic up to the eps the fixed point carries (row/col sums 1 - eps)
            assert np.abs(c.sum(1) - 1).max() < 1e-4 and np.abs(c.sum(2) - 1).max() < 1e-4
        if b is base0:
            # zero logits: every entry 1/4, off by the eps share (tests/test_v4_hc_oracle.cpp:371-404)
            assert np.abs(comb[0] - 0.25).max() < 1e-6
            assert np.abs(pre[0] - (0.5 + 1e-6)).max() < 1e-6 and np.abs(post[0] - 1.0).max() < 1e-6


def test_pre_combine_and_post_against_oracle(orc):
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(4)
    T, H = 5, 1024
    res = rng.normal(size=(4, T, H)).astype(np.float16)     # stream-major, as config 4 lays it out
    lo = rng.normal(size=(T, H)).astype(np.float16)
    mixes = rng.normal(size=24).astype(np.float32)
    hc = moe.HyperConnection(mixes)
    pre, post, comb = orc.hc_sinkhorn(mixes, np.ones(3), np.zeros(24), 4)
    assert np.abs(hc.pre.cpu().numpy()[0] - pre).max() <= 1e-5
    d_res, d_lo = h.dev_half(res), h.dev_half(lo)
    x = torch.zeros(T, H, dtype=torch.float16, device="cuda")
    hc.pre_combine(d_res, x)
    out = torch.zeros_like(d_res)
    hc.post_mix(d_lo, d_res, out)
    x, out = x.cpu().numpy().astype(np.float64), out.cpu().numpy().astype(np.float64)
    dpre = hc.pre.cpu().numpy()[0].astype(np.float64)
    dpost = hc.post.cpu().numpy()[0].astype(np.float64)
    dcomb = hc.comb.cpu().numpy()[0].astype(np.float64)
    for t in range(T):
        r = res[:, t, :].astype(np.float64)
        want_x = orc.hc_pre_combine(r, dpre, H)
        assert np.abs(x[t] - want_x).max() <= 1e-4 + 1e-3 * np.abs(want_x).max()
        want = orc.hc_post(lo[t].astype(np.float64), r, dpost, dcomb, H)
        assert np.abs(out[:, t, :] - want).max() <= 1e-4 + 1e-3 * np.abs(want).max()
        # the transposed reading of comb is a different function, and the kernel is not on it
        wrong = orc.hc_post(lo[t].astype(np.float64), r, dpost, dcomb, H, transpose_comb=True)
        assert np.abs(wrong - want).max() > 1e-2
        assert np.abs(out[:, t, :] - wrong).max() > 1e-2
    # fp32 residual form of the pre-combine (the reference kernel's input type), per-token mixes
    res32 = rng.normal(size=(T, 4, H)).astype(np.float32)
    pre_t = rng.random((T, 4)).astype(np.float32)
    x2 = torch.zeros(T, H, dtype=torch.float16, device="cuda")
    d_res32, d_pre = h.to_dev(res32), h.to_dev(pre_t)
    capi.call("aeon_hc_pre_combine", capi.vp(d_res32), 1, C.c_long(4 * H), C.c_long(H),
              capi.vp(d_pre), 4, capi.vp(x2), C.c_long(H), T, H, h.stream_ptr())
    want2 = np.einsum("tj,tjh->th", pre_t.astype(np.float64), res32.astype(np.float64))
    assert np.abs(x2.cpu().numpy() - want2).max() <= 1e-4 + 1e-3 * np.abs(want2).max()
    with pytest.raises(ValueError):
        hc.post_mix(d_lo, d_res, d_res)


@pytest.mark.parametrize("tokens,H", [(1, 256), (5, 1024), (64, 7168)])
def test_dynamic_mix_projection_norm_and_post(orc, tokens, H):
    """The per-token mix: projection (rms-scaled dots with 24 fn rows), per-token Sinkhorn,
    pre-combine with the token's own pre-mix, RMSNorm (weighted and weightless), and the post
    expansion with the token's post/comb -- each stage against the oracle fed the stage's own
    device input."""
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(tokens * 1000 + H)
    res = (rng.standard_normal((4, tokens, H)) * 1.5).astype(np.float16)
    fn = (rng.standard_normal((24, 4 * H)) * 0.05).astype(np.float32)
    scale = rng.standard_normal(3).astype(np.float32)
    base = rng.standard_normal(24).astype(np.float32)
    weight = (1.0 + 0.1 * rng.standard_normal(H)).astype(np.float16)
    hc = moe.DynamicHyperConnection(fn, scale, base, weight)
    d_res = h.to_dev(res)
    x_pre = torch.empty(tokens, H, dtype=torch.float16, device="cuda")
    x_norm = torch.empty(tokens, H, dtype=torch.float16, device="cuda")
    hc.pre_mix(d_res, x_pre, x_norm)
    torch.cuda.synchronize()
    mixes, pre = hc.mixes.cpu().numpy(), hc.pre.cpu().numpy()
    post, comb = hc.post.cpu().numpy(), hc.comb.cpu().numpy()
    check = range(tokens) if tokens <= 8 else (0, 17, tokens - 1)
    for t in check:
        flat = res[:, t, :].astype(np.float64).ravel()
        want = orc.hc_mixes(flat, fn.astype(np.float64), 1e-6)
        # fp32 accumulation of 4H products: a few ulps of the largest term, measured on the
        # scale the dot products themselves have
        assert np.abs(mixes[t] - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
        wp, wq, wc = orc.hc_sinkhorn(mixes[t].astype(np.float64), scale, base, 4)
        assert np.abs(pre[t] - wp).max() <= 1e-5 and np.abs(post[t] - wq).max() <= 1e-5
        assert np.abs(comb[t] - wc).max() <= 1e-5
        want_x = orc.hc_pre_combine(res[:, t, :].astype(np.float64), pre[t].astype(np.float64), H)
        got_x = x_pre[t].cpu().numpy()
        assert np.abs(got_x - want_x).max() <= 2e-3 * np.abs(want_x).max()
        want_n = orc.rmsnorm(got_x.astype(np.float64), weight.astype(np.float64), 1e-6)
        assert h.rel_err(x_norm[t].cpu().numpy(), want_n) <= 2e-3
    # the fp32 residual the reference keeps gives the same mixes as its fp16 rounding here
    mixes32 = torch.empty(tokens, 24, dtype=torch.float32, device="cuda")
    d_res32 = h.to_dev(res.astype(np.float32))
    capi.call("aeon_hc_project", capi.vp(d_res32), 1, C.c_long(d_res32.stride(1)),
              C.c_long(d_res32.stride(0)), capi.vp(hc.fn), capi.vp(mixes32), tokens, H,
              C.c_float(1e-6), h.stream_ptr())
    assert torch.equal(mixes32, hc.mixes)
    # weightless norm
    unit = torch.empty_like(x_norm)
    capi.call("aeon_rmsnorm", capi.vp(x_pre), C.c_long(H), None, capi.vp(unit), C.c_long(H), tokens, H,
              C.c_float(1e-6), h.stream_ptr())
    t = check[-1] if not isinstance(check, range) else tokens - 1
    want_u = orc.rmsnorm(x_pre[t].cpu().numpy().astype(np.float64), None, 1e-6)
    assert h.rel_err(unit[t].cpu().numpy(), want_u) <= 2e-3
    # post expansion with per-token post/comb
    y = h.dev_half((rng.standard_normal((tokens, H)) * 2).astype(np.float16))
    d_out = torch.empty_like(d_res)
    hc.post_mix(y, d_res, d_out)
    torch.cuda.synchronize()
    for t in check:
        want_r = orc.hc_post(y[t].cpu().numpy().astype(np.float64), res[:, t, :].astype(np.float64),
                             post[t].astype(np.float64), comb[t].astype(np.float64), H)
        assert np.abs(d_out[:, t, :].cpu().numpy() - want_r).max() <= 2e-3 * np.abs(want_r).max()
    # reproducible bit for bit
    first = hc.mixes.clone()
    hc.pre_mix(d_res, x_pre, x_norm)
    assert torch.equal(first, hc.mixes)


@pytest.mark.parametrize("B,H,I,E,normed", [(64, 1024, 512, 16, False), (4, 7168, 2048, 12, False),
                                             (64, 7168, 2048, 256, False), (64, 1024, 512, 16, True),
                                             (64, 7168, 2048, 256, True)])
def test_config4_stacked_layers(orc, B, H, I, E, normed):
    """Four MoE layers with independent seeded weights and the HC mix between them. Each layer is
    checked against the oracle on the device's own input to that layer and the device's routed
    ids (the way a composed gate isolates one stage from the rounding of the ones before it).
    The third case is benchmark config 4 as written: 4 x (256 + 1) resident experts (23 GB), batch
    64; there the oracle takes three tokens of every layer and its experts' payloads come back
    from the device generator. `normed` puts the FFN RMSNorm (seeded weight) between the
    pre-combine and the router/experts, where the reference's layer body has it
    (layer/v4_layer_body_attention.hpp:113-115): without it the residual grows from layer to
    layer, the sigmoid scores saturate and layers 2-4 route every token to the same few
    experts. The stack runs fused (reduce + post-mix + the next layer's pre-combine in one
    launch) and has to give the bits of the launch-by-launch sequence."""
    torch, h, capi, moe, synth = _setup()
    k, limit, L = 8, 7.0, 4
    layers, mixes, host, norm_w = [], [], [], []
    for l in range(L):
        pool = moe.ExpertPool(E + 1, H, I)
        assert pool.fill_synthetic(seed=11, first_expert_id=1000 * l) == 0
        wr, bias = synth.router_weight(11, H, E, unit=l), synth.router_bias(11, E, unit=l)
        d_wr, d_bias = h.to_dev(wr), h.to_dev(bias)
        layers.append(moe.MoeLayer(pool, E, k, True, limit, d_wr, d_bias, score_kind=1))
        mix = synth.normal(synth.stream_key(11, synth.STREAM_HC, l), 24).astype(np.float32)
        mixes.append(moe.HyperConnection(mix))
        nw = (1.0 + 0.1 * synth.normal(synth.stream_key(11, synth.STREAM_HC, 100 + l), H)).astype(np.float16)
        norm_w.append(nw)
        host.append((wr, bias, mix))
    d_norm = [h.dev_half(nw) for nw in norm_w] if normed else None
    stack = moe.LayerStack(layers, mixes, norm_weights=d_norm, fused=True)
    res0 = synth.activations(11, 4 * B, H).reshape(4, B, H)
    trace = []
    final = stack.step(h.dev_half(res0), trace=trace)
    torch.cuda.synchronize()
    assert np.isfinite(final.cpu().numpy()).all()
    import test_gpu_layer as tl
    distinct = []
    for l, (res_in, x_pre, x, ids, w, y, res_out) in enumerate(trace):
        wr, bias, mix = host[l]
        res_in, x_pre, x, y = res_in.cpu().numpy(), x_pre.cpu().numpy(), x.cpu().numpy(), y.cpu().numpy()
        ids, w, res_out = ids.cpu().numpy(), w.cpu().numpy(), res_out.cpu().numpy()
        distinct.append(int(np.unique(ids).size))
        pre, post, comb = orc.hc_sinkhorn(mix, np.ones(3), np.zeros(24), 4)
        check = range(B) if H <= 1024 else (range(min(B, 2)) if E < 256 else (0, B // 2, B - 1))
        make = h.GeneratedExpert if E >= 256 else h.Expert
        experts = {int(e): make(11, 1000 * l + int(e), H, I) for t in check for e in ids[t]}
        shared = make(11, 1000 * l + E, H, I)
        for t in check:
            r = res_in[:, t, :].astype(np.float64)
            want_x = orc.hc_pre_combine(r, pre, H)
            assert np.abs(x_pre[t] - want_x).max() <= 2e-3 * np.abs(want_x).max()
            if normed:
                want_n = orc.rmsnorm(x_pre[t].astype(np.float64), norm_w[l].astype(np.float64), 1e-6)
                assert h.rel_err(x[t], want_n) <= 2e-3
            else:
                assert np.array_equal(x[t], x_pre[t])
            logits = x[t].astype(np.float64) @ wr.astype(np.float64)
            oi, ow = orc.router_topk(logits, bias.astype(np.float64), k, 1.0, 1)
            # the device selects on its own fp32 logits; where the sets differ, the 8th and 9th
            # biased scores (what the selection compares) must be closer than that rounding
            choice = np.sort(1.0 / (1.0 + np.exp(-np.clip(logits, -700.0, 700.0))) + bias.astype(np.float64))
            assert set(oi) == set(ids[t]) or choice[-8] - choice[-9] < 1e-6
        rows = list(check)
        want_y = tl._oracle_layer(orc, h, experts, x[rows], ids[rows], w[rows], shared, limit)
        report = h.error_report(y[rows], want_y)
        print("config 4 layer %d (B=%d H=%d E=%d normed=%s), %d tokens against the oracle: %s"
              % (l, B, H, E, normed, len(rows), report))
        tl.check_chained(report)
        for t in check:
            want_r = orc.hc_post(y[t].astype(np.float64), res_in[:, t, :].astype(np.float64), post,
                                 comb, H)
            assert np.abs(res_out[:, t, :] - want_r).max() <= 2e-3 * np.abs(want_r).max()
    print("distinct routed experts per layer:", distinct)
    if normed and E >= 256:
        # every layer sees a unit-scale input: the routing spreads as in the one-layer config
        assert min(distinct) >= 60
    # the step is bit-reproducible, and the fused last launch gives the launch-by-launch bits
    again = stack.step(h.dev_half(res0))
    assert torch.equal(again, final)
    unfused = moe.LayerStack(layers, mixes, norm_weights=d_norm, fused=False).step(h.dev_half(res0))
    assert torch.equal(unfused, final)


@pytest.mark.parametrize("tokens,shared", [(1, False), (7, False), (7, True), (150, False)])
def test_fused_reduce_post_and_next_pre_combine_equal_the_three_launches(orc, tokens, shared):
    """aeon_moe_layer_decode_hc_post against aeon_moe_layer_decode + aeon_hc_post +
    aeon_hc_pre_combine on the same inputs, with per-token mixes (the reference's dynamic form)
    and with a layer that has no always-on expert (the routed sum is then added to what the
    output rows hold): layer output, expanded residual and next layer input bit for bit, for
    direct slots, decode segments and grouped windows."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k = 512, 256, 12, 4
    pool = moe.ExpertPool(E + (1 if shared else 0), H, I)
    assert pool.fill_synthetic(seed=71, first_expert_id=0) == 0
    wr, bias = synth.router_weight(71, H, E), synth.router_bias(71, E)
    layer = moe.MoeLayer(pool, E, k, shared, 7.0, h.to_dev(wr), h.to_dev(bias), score_kind=1)
    rng = np.random.default_rng(tokens)

    class Mix:
        pass
    this, nxt = Mix(), Mix()
    this.post = h.to_dev(rng.uniform(0.2, 2.0, (tokens, 4)).astype(np.float32))
    this.comb = h.to_dev(rng.uniform(0.0, 0.5, (tokens, 16)).astype(np.float32))
    nxt.pre = h.to_dev(rng.uniform(0.1, 1.0, (tokens, 4)).astype(np.float32))
    res = h.dev_half(synth.activations(71, 4 * tokens, H).reshape(4, tokens, H))
    x = h.dev_half(synth.activations(72, tokens, H))
    start = h.dev_half(synth.activations(73, tokens, H))   # what the output rows hold beforehand

    out_a, ids_a, w_a = layer.decode(x, out=start.clone())
    res_a = torch.empty_like(res)
    capi.call("aeon_hc_post", capi.vp(out_a), C.c_long(H), capi.vp(res), C.c_long(res.stride(1)),
              C.c_long(res.stride(0)), capi.vp(this.post), capi.vp(this.comb), 1, capi.vp(res_a),
              tokens, H, h.stream_ptr())
    next_a = torch.empty(tokens, H, dtype=torch.float16, device="cuda")
    capi.call("aeon_hc_pre_combine", capi.vp(res_a), 0, C.c_long(res_a.stride(1)),
              C.c_long(res_a.stride(0)), capi.vp(nxt.pre), 4, capi.vp(next_a), C.c_long(H), tokens, H,
              h.stream_ptr())

    res_b = torch.empty_like(res)
    next_b = torch.empty(tokens, H, dtype=torch.float16, device="cuda")
    out_b, ids_b, w_b = layer.decode_hc_post(x, res, res_b, this, nxt, next_b, out=start.clone())
    torch.cuda.synchronize()
    assert torch.equal(ids_a, ids_b) and torch.equal(w_a, w_b)
    assert torch.equal(out_a, out_b)
    assert torch.equal(res_a, res_b)
    assert torch.equal(next_a, next_b)
    # without a next layer the next-input buffer is left alone
    untouched = torch.full_like(next_b, 3.0)
    layer.decode_hc_post(x, res, res_b, this, None, untouched, out=start.clone())
    torch.cuda.synchronize()
    assert torch.all(untouched == 3.0) and torch.equal(res_a, res_b)
    # in-place expansion is refused
    with pytest.raises(ValueError, match="not aliased"):
        layer.decode_hc_post(x, res, res, this, None, None, out=start.clone())
