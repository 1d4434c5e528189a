"""GPU parity of the real model's dense fp16 pieces beside the int4 experts: the fp16 router
gate (gemv_fp16_vec8_kernel + widening, src/platform/ops/gemv.hpp:72-110 and
layer/v4_layer_body_moe.hpp:135-142) and the dense shared expert
(run_layer_body_moe_shared_expert, :216-256; oracle dense_ffn, dsv4_oracle.hpp:1708-1753),
alone and inside the layer step. Tolerances: an fp16 result of an fp32 accumulation is held to
one fp16 rounding of the fp64 value (neighbouring values allowed where the fp32 sum sits on a
rounding boundary); composed results to 6e-3 of the peak, the reference's FFN bound
(tests/test_v4_expert_oracle.cpp:75-77)."""
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


def _one_rounding(got16, want64):
    """(exact, near): got16 is fp16(want64) exactly, or within one fp16 rounding of want64 plus
    what an fp32 accumulation of this length cannot resolve (2e-6 of the peak: it matters only
    for results that cancel to nearly zero, whose fp16 spacing is finer than that)."""
    want16 = want64.astype(np.float16)
    exact = got16 == want16
    spacing = np.spacing(np.abs(want16).astype(np.float16)).astype(np.float64)
    near = np.abs(got16.astype(np.float64) - want64) <= spacing + 2e-6 * np.abs(want64).max()
    return exact, near


@pytest.mark.parametrize("tokens", [1, 5, 16, 33, 100])
@pytest.mark.parametrize("in_dim,out_dim", [(4096, 2048), (2048, 4096), (7168, 256), (128, 16)])
def test_dense_gemv_against_fp64(orc, tokens, in_dim, out_dim):
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(tokens * 7 + in_dim)
    w = rng.normal(0, 0.03, (out_dim, in_dim)).astype(np.float16)
    x = rng.normal(0, 1, (tokens, in_dim)).astype(np.float16)
    d_w, d_x = h.dev_half(w), h.dev_half(x)
    y = torch.full((tokens + 1, out_dim), 9.0, dtype=torch.float16, device="cuda")
    capi.call("aeon_dense_gemv_f16", capi.vp(d_x), in_dim, capi.vp(d_w), capi.vp(y), out_dim, tokens,
              in_dim, out_dim, h.stream_ptr())
    got = y.cpu().numpy()
    assert np.all(got[tokens] == np.float16(9.0))           # nothing past the last token
    want = x.astype(np.float64) @ w.astype(np.float64).T
    exact, near = _one_rounding(got[:tokens], want)
    assert np.all(exact | near)
    assert exact.mean() > 0.97
    assert h.rel_err(got[:tokens], want) <= 2e-3
    again = torch.zeros_like(y)
    capi.call("aeon_dense_gemv_f16", capi.vp(d_x), in_dim, capi.vp(d_w), capi.vp(again), out_dim, tokens,
              in_dim, out_dim, h.stream_ptr())
    assert torch.equal(again[:tokens], y[:tokens])          # fixed summation order


@pytest.mark.parametrize("tokens,in_dim,out_dim,x_pitch,y_pitch", [(3, 384, 48, 392, 52), (20, 640, 32, 768, 40),
                                                                    (64, 1152, 80, 1160, 96), (130, 384, 16, 512, 20)])
def test_dense_gemv_with_row_pitches_and_uneven_k_shares(orc, tokens, in_dim, out_dim, x_pitch, y_pitch):
    """Rows wider than the matrices (x_stride > in_dim, y_stride > out_dim) and a K whose 128-column
    groups do not divide among the four waves: the columns between rows stay untouched and the
    result is the compact call's, bit for bit."""
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(tokens * 11 + in_dim)
    w = rng.normal(0, 0.05, (out_dim, in_dim)).astype(np.float16)
    x = rng.normal(0, 1, (tokens, in_dim)).astype(np.float16)
    wide = np.full((tokens, x_pitch), np.float16(777.0))
    wide[:, :in_dim] = x
    d_w, d_x, d_wide = h.dev_half(w), h.dev_half(x), h.dev_half(wide)
    compact = torch.zeros((tokens, out_dim), dtype=torch.float16, device="cuda")
    capi.call("aeon_dense_gemv_f16", capi.vp(d_x), in_dim, capi.vp(d_w), capi.vp(compact), out_dim, tokens,
              in_dim, out_dim, h.stream_ptr())
    pitched = torch.full((tokens, y_pitch), 9.0, dtype=torch.float16, device="cuda")
    capi.call("aeon_dense_gemv_f16", capi.vp(d_wide), x_pitch, capi.vp(d_w), capi.vp(pitched), y_pitch, tokens,
              in_dim, out_dim, h.stream_ptr())
    assert torch.equal(pitched[:, :out_dim], compact)
    assert torch.all(pitched[:, out_dim:] == 9.0)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    exact, near = _one_rounding(compact.cpu().numpy(), want)
    assert np.all(exact | near)


@pytest.mark.parametrize("tokens,hidden,inter,limit", [(1, 4096, 2048, 10.0), (7, 4096, 2048, 10.0),
                                                       (40, 1024, 512, 0.5), (70, 512, 256, 10.0)])
def test_dense_shared_expert_against_the_oracle(orc, tokens, hidden, inter, limit):
    torch, h, capi, moe, synth = _setup()
    rng = np.random.default_rng(tokens + hidden)
    w1 = rng.normal(0, 0.03, (inter, hidden)).astype(np.float16)
    w3 = rng.normal(0, 0.03, (inter, hidden)).astype(np.float16)
    w2 = rng.normal(0, 0.03, (hidden, inter)).astype(np.float16)
    x = rng.normal(0, 1, (tokens, hidden)).astype(np.float16)
    dev = [h.dev_half(a) for a in (x, w1, w3, w2)]
    gate = torch.zeros(tokens, inter, dtype=torch.float16, device="cuda")
    up = torch.zeros_like(gate)
    act = torch.zeros_like(gate)
    out = torch.full((tokens, hidden), 5.0, dtype=torch.float16, device="cuda")   # stale accumulator
    capi.call("aeon_dense_shared_expert_f16", capi.vp(dev[0]), hidden, tokens, capi.vp(dev[1]),
              capi.vp(dev[2]), capi.vp(dev[3]), capi.vp(gate), capi.vp(up), capi.vp(act), capi.vp(out),
              hidden, hidden, inter, C.c_float(limit), h.stream_ptr())
    got = out.cpu().numpy().astype(np.float64)
    w64 = [a.astype(np.float64) for a in (w1, w3, w2)]
    # stage by stage: gate and up are single GEMVs
    ex, near = _one_rounding(gate.cpu().numpy(), x.astype(np.float64) @ w64[0].T)
    assert np.all(ex | near)
    ex, near = _one_rounding(up.cpu().numpy(), x.astype(np.float64) @ w64[1].T)
    assert np.all(ex | near)
    # the activation stage on the device's own gate and up: one rounding of the fp64 value
    g16, u16 = gate.cpu().numpy().astype(np.float64).ravel(), up.cpu().numpy().astype(np.float64).ravel()
    pick = rng.choice(g16.size, size=min(4000, g16.size), replace=False)
    want = np.array([orc.clamped_swiglu(g16[i], u16[i], limit) for i in pick])
    ex, near = _one_rounding(act.cpu().numpy().ravel()[pick], want)
    assert np.all(ex | near)
    # the composed FFN: the device's view (stages stored as fp16) and the oracle's own (no
    # rounding between stages, dense_ffn as the reference states it)
    staged = orc.dense_ffn(*w64, x.astype(np.float64), limit, round_stages=True)
    plain = orc.dense_ffn(*w64, x.astype(np.float64), limit)
    peak = np.abs(plain).max()
    assert peak > 1e-2
    assert np.abs(got - staged).max() <= 2e-3 * peak
    assert np.abs(got - plain).max() <= 6e-3 * peak
    # the symmetric-clamp misreading is farther away than the tolerance when the clamp bites
    if limit < 1.0:
        wrong = orc.dense_ffn(*w64, x.astype(np.float64), limit, clamp_mode=1)
        assert np.abs(wrong - plain).max() > 5 * 6e-3 * peak


def test_fp16_gate_logits_and_routing(orc):
    """The checkpoint's gate: logits rounded to fp16 then widened, so many logits tie exactly and
    the lowest index has to win; ids bit-exact against the oracle on the device's own logits,
    sqrt(softplus) score, bias after the activation, weights scaled by 1.5 (the reference's
    constants, layer/v4_layer_body_moe.hpp:150-158)."""
    torch, h, capi, moe, synth = _setup()
    T, H, E, k = 37, 4096, 256, 6
    rng = np.random.default_rng(12)
    gate_w = rng.normal(0, 0.02, (E, H)).astype(np.float16)
    gate_w[17] = gate_w[5]          # two experts with the same logit for every token
    bias = rng.normal(0, 0.05, E).astype(np.float32)
    bias[17] = bias[5]
    x = rng.normal(0, 1, (T, H)).astype(np.float16)
    d_x, d_w, d_b = h.dev_half(x), h.dev_half(gate_w), h.to_dev(bias)
    half = torch.zeros(T, E, dtype=torch.float16, device="cuda")
    wide = torch.zeros(T, E, dtype=torch.float32, device="cuda")
    capi.call("aeon_router_logits_f16", capi.vp(d_x), H, capi.vp(d_w), capi.vp(half), capi.vp(wide), T, H, E,
              h.stream_ptr())
    lh, lw = half.cpu().numpy(), wide.cpu().numpy()
    assert np.array_equal(lw, lh.astype(np.float32))
    want = x.astype(np.float64) @ gate_w.astype(np.float64).T
    exact, near = _one_rounding(lh, want)
    assert np.all(exact | near) and exact.mean() > 0.97
    assert np.array_equal(lh[:, 17], lh[:, 5])
    ids = torch.zeros(T, k, dtype=torch.int32, device="cuda")
    w = torch.zeros(T, k, dtype=torch.float32, device="cuda")
    capi.call("aeon_moe_router", capi.vp(wide), capi.vp(d_b), None, None, capi.vp(w), capi.vp(ids), T, E, k,
              C.c_float(1.5), 1, 0, h.stream_ptr())
    ids, w = ids.cpu().numpy(), w.cpu().numpy()
    both = 0
    for t in range(T):
        oi, ow = orc.router_topk(lw[t].astype(np.float64), bias.astype(np.float64), k, 1.5, 0)
        assert np.array_equal(ids[t], oi)
        assert np.abs(w[t] - ow).max() <= 1e-5 * np.abs(ow).max()
        if 5 in ids[t] and 17 in ids[t]:
            both += 1
            assert list(ids[t]).index(5) < list(ids[t]).index(17)   # the tie goes to the lower index
        assert 17 not in ids[t] or 5 in ids[t]


@pytest.mark.parametrize("T", [1, 9, 64, 200, 300])
def test_layer_step_with_the_checkpoint_pieces(orc, T):
    """The layer step as the real model composes it: fp16 gate, sqrt(softplus) score with bias
    after it, top-6 scaled by 1.5, group-32 int4 routed experts, the dense fp16 shared expert
    written first and the routed sum added to it in slot order (hidden 4096, intermediate 2048,
    32 experts here). Sampled tokens against the oracle composed the same way."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, limit = 4096, 2048, 32, 6, 10.0
    pool = moe.ExpertPool(E, H, I, scale_group=32)
    assert pool.fill_synthetic(seed=44, first_expert_id=0) == 0
    rng = np.random.default_rng(44)
    gate_w = rng.normal(0, 0.02, (E, H)).astype(np.float16)
    bias = rng.normal(0, 0.05, E).astype(np.float32)
    sw = [rng.normal(0, 0.06, s).astype(np.float16) for s in ((I, H), (I, H), (H, I))]
    d_sw = [h.dev_half(a) for a in sw]
    d_gate, d_bias = h.dev_half(gate_w), h.to_dev(bias)
    layer = moe.MoeLayer(pool, E, k, False, limit, None, d_bias, score_kind=0, routed_scaling_factor=1.5,
                         router_weight_f16=d_gate, dense_shared=tuple(d_sw))
    x = synth.activations(44, T, H)
    d_x = h.dev_half(x)
    out = torch.full((T, H), 3.0, dtype=torch.float16, device="cuda")     # stale rows: must be overwritten
    out, ids, w = layer.decode(d_x, out=out)
    logits = layer.router_logits(d_x).cpu().numpy()
    ids, w, got = ids.cpu().numpy(), w.cpu().numpy(), out.cpu().numpy().astype(np.float64)
    for t in range(T):
        oi, ow = orc.router_topk(logits[t].astype(np.float64), bias.astype(np.float64), k, 1.5, 0)
        assert np.array_equal(ids[t], oi)
        assert np.abs(w[t] - ow).max() <= 1e-5 * np.abs(ow).max()
    sample = sorted({0, T // 2, T - 1})
    experts = {int(e): h.GeneratedExpert(44, int(e), H, I, 32) for t in sample for e in ids[t]}
    w64 = [a.astype(np.float64) for a in sw]
    for t in sample:
        shared = orc.dense_ffn(*w64, x[t].astype(np.float64), limit, round_stages=True)
        shared = shared.astype(np.float16).astype(np.float64)
        contrib = np.stack([float(w[t, s]) * experts[int(ids[t, s])].ffn(x[t:t + 1], limit)[0] for s in range(k)])
        want = orc.moe_combine(contrib, shared)
        assert np.abs(got[t] - want).max() <= 6e-3 * np.abs(want).max()
        assert np.abs(contrib.sum(0)).max() > 0.05 * np.abs(want).max()     # both parts matter
        assert np.abs(shared).max() > 0.05 * np.abs(want).max()
    out2, _, _ = layer.decode(d_x)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("T", [1, 6, 40, 150])
def test_checkpoint_step_equals_its_routed_half_and_replays_from_a_graph(orc, T):
    """With the fp16 gate and the dense shared expert the full step and the routed entry point
    (given the step's own ids and weights) run the same expert kernels: same bits. The step is
    also captured into a graph and replayed with new activations and eager steps in between;
    every replay has to give the eager bits."""
    torch, h, capi, moe, synth = _setup()
    H, I, E, k, limit = 1024, 512, 32, 4, 10.0
    pool = moe.ExpertPool(E, H, I, scale_group=32)
    assert pool.fill_synthetic(seed=52, first_expert_id=0) == 0
    rng = np.random.default_rng(52)
    gate_w = rng.normal(0, 0.03, (E, H)).astype(np.float16)
    bias = rng.normal(0, 0.05, E).astype(np.float32)
    d_sw = [h.dev_half(rng.normal(0, 0.06, s).astype(np.float16)) for s in ((I, H), (I, H), (H, I))]
    layer = moe.MoeLayer(pool, E, k, False, limit, None, h.to_dev(bias), score_kind=0, routed_scaling_factor=1.5,
                         router_weight_f16=h.dev_half(gate_w), dense_shared=tuple(d_sw))
    xs = [h.dev_half(synth.activations(52, T, H, unit=r)) for r in range(3)]
    eager = []
    for x in xs:
        out, ids, w = layer.decode(x)
        alone = layer.routed(x, ids, w)
        torch.cuda.synchronize()
        assert torch.equal(out, alone)
        assert float(out.float().abs().max()) > 0.0
        eager.append((out.clone(), ids.clone(), w.clone()))
    x_in = xs[0].clone()
    out = torch.full((T, H), 5.0, dtype=torch.float16, device="cuda")
    ids = torch.empty(T, k, dtype=torch.int32, device="cuda")
    w = torch.empty(T, k, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.decode(x_in, out, ids, w)
    for r in (2, 0, 1, 2):
        x_in.copy_(xs[r])
        out.fill_(5.0)
        between = layer.decode(xs[(r + 1) % 3])      # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[r][0]), (T, r)
        assert torch.equal(ids, eager[r][1]) and torch.equal(w, eager[r][2]), (T, r)
        assert torch.equal(between[0], eager[(r + 1) % 3][0])
