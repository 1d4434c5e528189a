"""GPU parity: W4A16 GEMV / dual-GEMV (both layouts), the fused gate/up + SwiGLU, the W2
contribution and the fixed-order reduce, against the fp64 oracle on the same seeded inputs.
Tolerance: max relative error 1e-2 (denominator floored at 1e-3 of the peak), the bar for
fp32-accumulate outputs; the reference's own GEMV gate allows 0.05 absolute
(tests/test_w4a16_swizzled_gemv.cpp:122)."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _setup():
    import torch
    assert torch.cuda.is_available()
    import helpers
    from project_aeon_amd import capi
    return torch, helpers, capi


def _reference_fixture(N, K):
    """The closed-form fixture of tests/test_w4a16_swizzled_gemv.cpp:36-43,61-70, regenerated:
    nibble j of word i = (3i + 5j + 1) % 16, scale i = 2^-8 * (1 + i % 29),
    x[k] = ((k % 19) - 9) / 32."""
    idx = np.arange(N * K // 8, dtype=np.uint64)
    words = np.zeros(N * K // 8, dtype=np.uint32)
    for j in range(8):
        words |= (((idx * 3 + j * 5 + 1) % 16).astype(np.uint32)) << np.uint32(4 * j)
    scale = (0.00390625 * (1 + np.arange(N * K // 32) % 29)).astype(np.float16)
    x = (((np.arange(K) % 19) - 9) * 0.03125).astype(np.float16)
    return words, scale, x


@pytest.mark.parametrize("N,K,cfg", [(2048, 4096, (4, 8)), (4096, 2048, (8, 4))])
def test_swizzled_gemv_reference_fixture(orc, N, K, cfg):
    torch, h, capi = _setup()
    words, scale, x = _reference_fixture(N, K)
    swp, sws = orc.swizzle(words, scale.view(np.uint16), N, K, *cfg)
    want = orc.swizzled_matvec(swp, sws, N, K, cfg[0], cfg[1], x.astype(np.float64))
    d_x, d_p, d_s = h.dev_half(x), h.dev_u32(swp), h.dev_u16(sws)
    out = torch.zeros(N, dtype=torch.float16, device="cuda")
    capi.call("aeon_w4a16_swizzled_gemv", capi.vp(d_x), capi.vp(d_p), capi.vp(d_s), capi.vp(out),
              N, K, cfg[0], cfg[1], h.stream_ptr())
    got = out.cpu().numpy().astype(np.float64)
    assert np.abs(got - want).max() < 0.05
    assert h.rel_err(got, want) <= TOL
    # a deliberately wrong reading (unsigned zero point) must be far away: the check is not vacuous
    wrong = orc.swizzled_decode(swp, sws, N, K, cfg[0], cfg[1], signed_zp=False) @ x.astype(np.float64)
    assert h.rel_err(wrong, want) > 10 * TOL


def test_config0_single_gemv_both_layouts(orc):
    """benchmark config 0: x [1x7168] ~N(0,1), W int4 [7168->2048], group-128 scales, seed 0."""
    torch, h, capi = _setup()
    from project_aeon_amd import synth
    N, K = 2048, 7168
    m = h.synth_matrix(0, 0, synth.STREAM_W1, N, K)
    x = synth.activations(0, 1, K)
    want = orc.swizzled_matvec(m.swz_packed, m.swz_scale, N, K, 4, 8, x.astype(np.float64))[0]
    d_x = h.dev_half(x)
    out_swz = torch.zeros(N, dtype=torch.float16, device="cuda")
    d_p, d_s = h.dev_u32(m.swz_packed), h.dev_u16(m.swz_scale)
    capi.call("aeon_w4a16_swizzled_gemv", capi.vp(d_x), capi.vp(d_p), capi.vp(d_s),
              capi.vp(out_swz), N, K, 4, 8, h.stream_ptr())
    out_a64 = torch.zeros(N, dtype=torch.float16, device="cuda")
    d_ap, d_as = h.dev_u32(m.a64_packed), h.dev_u16(m.a64_scale)
    capi.call("aeon_a64_gemv", capi.vp(d_x), K, capi.vp(d_ap), capi.vp(d_as), 128, capi.vp(out_a64),
              N, 1, N, K, h.stream_ptr())
    for got in (out_swz, out_a64):
        g = got.cpu().numpy().astype(np.float64)
        assert np.abs(want).max() > 1.0
        assert h.rel_err(g, want) <= TOL


@pytest.mark.parametrize("scale_group", [128, 32])
@pytest.mark.parametrize("tokens", [1, 2, 3, 8])
@pytest.mark.parametrize("N,K,matrix", [(2048, 7168, 0), (7168, 2048, 2), (64, 256, 0)])
def test_a64_gemv_and_dual(orc, tokens, N, K, matrix, scale_group):
    """scale_group 32: every (row, 32-column group) has a scale of its own, as in a real
    `.aeon` payload (swizzled_expert_format.hpp:18-23)."""
    torch, h, capi = _setup()
    from project_aeon_amd import synth
    ma = h.synth_matrix(3, 1, matrix, N, K, scale_group)
    mb = h.synth_matrix(3, 2, matrix, N, K, scale_group)
    x = synth.activations(7, tokens, K)
    want_a = orc.swizzled_matvec(ma.swz_packed, ma.swz_scale, N, K, *ma.cfg, x.astype(np.float64))
    want_b = orc.swizzled_matvec(mb.swz_packed, mb.swz_scale, N, K, *mb.cfg, x.astype(np.float64))
    d_x = h.dev_half(x)
    pa, sa, pb, sb = (h.dev_u32(ma.a64_packed), h.dev_u16(ma.a64_scale), h.dev_u32(mb.a64_packed),
                      h.dev_u16(mb.a64_scale))
    single = torch.zeros(tokens, N, dtype=torch.float16, device="cuda")
    capi.call("aeon_a64_gemv", capi.vp(d_x), K, capi.vp(pa), capi.vp(sa), scale_group,
              capi.vp(single), N, tokens, N, K, h.stream_ptr())
    oa = torch.zeros(tokens, N, dtype=torch.float16, device="cuda")
    ob = torch.zeros(tokens, N, dtype=torch.float16, device="cuda")
    capi.call("aeon_a64_dual_gemv", capi.vp(d_x), K, capi.vp(pa), capi.vp(sa), capi.vp(pb),
              capi.vp(sb), scale_group, capi.vp(oa), capi.vp(ob), N, tokens, N, K, h.stream_ptr())
    assert h.rel_err(single.cpu().numpy(), want_a) <= TOL
    assert h.rel_err(oa.cpu().numpy(), want_a) <= TOL
    assert h.rel_err(ob.cpu().numpy(), want_b) <= TOL
    # the dual kernel is two single launches sharing one activation read: bit-equal
    # (tests/test_w4a16_swizzled_dual_gemv.cpp)
    assert torch.equal(single, oa)


@pytest.mark.parametrize("tokens,N,K", [(5, 2048, 7168), (8, 7168, 2048), (8, 64, 16384)])
def test_a64_gemv_batch_rows_staged_or_fetched(orc, tokens, N, K):
    """From four tokens on the batch's activation rows are copied to LDS once per workgroup where
    they fit (8 x 7168 halves do, 8 x 16384 do not and are fetched per lane as before): both
    forms against the oracle, and a batch whose rows sit in a wider buffer gives the bits of the
    packed one."""
    torch, h, capi = _setup()
    from project_aeon_amd import synth
    m = h.synth_matrix(5, 1, 0, N, K, 128)
    x = synth.activations(11, tokens, K)
    want = orc.swizzled_matvec(m.swz_packed, m.swz_scale, N, K, *m.cfg, x.astype(np.float64))
    pa, sa = h.dev_u32(m.a64_packed), h.dev_u16(m.a64_scale)
    packed = h.dev_half(x)
    wide = torch.full((tokens, K + 72), 3.0, dtype=torch.float16, device="cuda")
    wide[:, :K] = packed
    outs = []
    for buf, pitch in ((packed, K), (wide, K + 72)):
        out = torch.zeros(tokens, N, dtype=torch.float16, device="cuda")
        capi.call("aeon_a64_gemv", capi.vp(buf), pitch, capi.vp(pa), capi.vp(sa), 128, capi.vp(out), N,
                  tokens, N, K, h.stream_ptr())
        outs.append(out)
    assert h.rel_err(outs[0].cpu().numpy(), want) <= TOL
    assert torch.equal(outs[0], outs[1])


def test_swizzled_dual_equals_two_singles(orc):
    torch, h, capi = _setup()
    from project_aeon_amd import synth
    N, K = 2048, 4096
    ma = h.synth_matrix(1, 0, 0, N, K)
    mb = h.synth_matrix(7, 0, 1, N, K)
    x = synth.activations(1, 1, K)
    d_x = h.dev_half(x)
    pa, sa, pb, sb = (h.dev_u32(ma.swz_packed), h.dev_u16(ma.swz_scale), h.dev_u32(mb.swz_packed),
                      h.dev_u16(mb.swz_scale))
    outs = [torch.zeros(N, dtype=torch.float16, device="cuda") for _ in range(4)]
    capi.call("aeon_w4a16_swizzled_gemv", capi.vp(d_x), capi.vp(pa), capi.vp(sa), capi.vp(outs[0]),
              N, K, 4, 8, h.stream_ptr())
    capi.call("aeon_w4a16_swizzled_gemv", capi.vp(d_x), capi.vp(pb), capi.vp(sb), capi.vp(outs[1]),
              N, K, 4, 8, h.stream_ptr())
    capi.call("aeon_w4a16_swizzled_dual_gemv", capi.vp(d_x), capi.vp(pa), capi.vp(sa), capi.vp(pb),
              capi.vp(sb), capi.vp(outs[2]), capi.vp(outs[3]), N, K, 4, 8, h.stream_ptr())
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[3])
    want = orc.swizzled_matvec(ma.swz_packed, ma.swz_scale, N, K, 4, 8, x.astype(np.float64))[0]
    assert h.rel_err(outs[2].cpu().numpy(), want) <= TOL


def test_gemv_rejects_bad_shapes():
    torch, h, capi = _setup()
    t = torch.zeros(4096, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):  # K != iters*lpr*32
        capi.call("aeon_w4a16_swizzled_gemv", capi.vp(t), capi.vp(t), capi.vp(t), capi.vp(t), 64,
                  100, 4, 8, None)
    with pytest.raises(ValueError):  # N % rpw
        capi.call("aeon_w4a16_swizzled_gemv", capi.vp(t), capi.vp(t), capi.vp(t), capi.vp(t), 6,
                  256, 4, 8, None)
    with pytest.raises(ValueError):  # null
        capi.call("aeon_w4a16_swizzled_gemv", None, capi.vp(t), capi.vp(t), capi.vp(t), 64, 256,
                  4, 8, None)
    with pytest.raises(ValueError):
        capi.call("aeon_a64_gemv", capi.vp(t), 256, capi.vp(t), capi.vp(t), 128, capi.vp(t), 64, 9,
                  64, 256, None)
    with pytest.raises(ValueError, match="scale_group"):
        capi.call("aeon_a64_gemv", capi.vp(t), 256, capi.vp(t), capi.vp(t), 64, capi.vp(t), 64, 1,
                  64, 256, None)


@pytest.mark.parametrize("experts", [1, 6, 8])
def test_swizzled_expert_trio_reference_shapes(orc, experts):
    """The per-token trio of v4_expert_executor.hpp:340-369 on the reference's own shapes
    (hidden 4096, intermediate 2048, group 32) and the payload family of
    tests/test_moe_grouped_batch_parity.cpp:73-91 (byte pattern, power-of-two scales)."""
    torch, h, capi = _setup()
    H, I, limit = 4096, 2048, 10.0
    rng = np.random.default_rng(0xC0FFEE)
    x = (rng.random(H) - 0.5).astype(np.float16)
    weights = (0.6 / (np.arange(experts) + 1) + 0.02).astype(np.float32)
    w13, w2 = capi.W13Table(), capi.W2Table()
    keep, mats = [], []
    for e in range(experts):
        def payload(n_words, seed):
            i = np.arange(n_words * 4, dtype=np.uint64)
            return ((i * 37 + seed * 11) & 0xFF).astype(np.uint8).view(np.uint32)
        def scales(n):
            return np.ldexp(1.0, -6 + (np.arange(n) % 4)).astype(np.float16).view(np.uint16)
        m = {}
        for name, rows, cols in (("w1", I, H), ("w3", I, H), ("w2", H, I)):
            m[name] = (payload(rows * cols // 8, e * 3 + len(m)), scales(rows * cols // 32))
        mats.append(m)
        dev = {k: (h.dev_u32(v[0]), h.dev_u16(v[1])) for k, v in m.items()}
        keep.append(dev)
        w13.w1[e], w13.s1[e] = dev["w1"][0].data_ptr(), dev["w1"][1].data_ptr()
        w13.w3[e], w13.s3[e] = dev["w3"][0].data_ptr(), dev["w3"][1].data_ptr()
        w2.w2[e], w2.s2[e] = dev["w2"][0].data_ptr(), dev["w2"][1].data_ptr()
    d_x = h.dev_half(x)
    hidden = torch.zeros(8, I, dtype=torch.float16, device="cuda")
    contrib = torch.zeros(experts, H, dtype=torch.float32, device="cuda")
    shared = h.dev_half((rng.random(H) - 0.5).astype(np.float16))
    out = shared.clone()
    d_w = h.to_dev(weights)
    capi.call("aeon_moe_gemv_w13_swiglu", capi.vp(d_x), C.byref(w13), capi.vp(hidden), None, I,
              experts, I, H, 4, 8, C.c_float(limit), h.stream_ptr())
    capi.call("aeon_moe_fused_w2_contrib", capi.vp(hidden), C.byref(w2), capi.vp(d_w),
              capi.vp(contrib), experts, H, I, 8, 4, h.stream_ptr())
    capi.call("aeon_moe_accumulate_fixed_order", capi.vp(contrib), experts, capi.vp(out),
              capi.vp(out), H, h.stream_ptr())
    got_hidden = hidden.cpu().numpy()[:experts].astype(np.float64)
    got_contrib = contrib.cpu().numpy().astype(np.float64)
    want_contrib = np.empty((experts, H))
    for e, m in enumerate(mats):
        o, hid = orc.expert_ffn(m["w1"], m["w3"], m["w2"], H, I, x.astype(np.float64), limit,
                                round_hidden=True, want_hidden=True)
        assert h.rel_err(got_hidden[e], hid) <= TOL
        want_contrib[e] = float(weights[e]) * o
    assert h.rel_err(got_contrib, want_contrib) <= TOL
    # contrib == weight x unit-weight contribution, bit for bit (tests/test_v4_moe_accum_oracle.cpp)
    unit = torch.zeros_like(contrib)
    ones = torch.ones(experts, device="cuda")
    capi.call("aeon_moe_fused_w2_contrib", capi.vp(hidden), C.byref(w2),
              capi.vp(ones), capi.vp(unit), experts, H, I, 8, 4,
              h.stream_ptr())
    assert torch.equal(contrib, unit * d_w[:, None])
    # fixed-order reduce: fp32 slot-order sum with the shared value as the initial term, one rounding
    acc = shared.float()
    for e in range(experts):
        acc = acc + contrib[e]
    assert torch.equal(out, acc.half())
    want_out = orc.moe_combine(want_contrib, shared.cpu().numpy().astype(np.float64))
    assert h.rel_err(out.cpu().numpy(), want_out) <= TOL
    # the one-launch accumulation control (aeon_moe_fused_w2.hpp:73-174): the same slot-order
    # sum from a zeroed row, so bit-identical to contrib + reduce without an initial row, and
    # within tolerance of the oracle with the shared row entering beside the first expert
    acc32 = torch.zeros(H, dtype=torch.float32, device="cuda")
    acc16 = torch.zeros(H, dtype=torch.float16, device="cuda")
    capi.call("aeon_moe_fused_w2_accum", capi.vp(hidden), C.byref(w2), capi.vp(d_w), None,
              capi.vp(acc32), capi.vp(acc16), experts, H, I, 8, 4, h.stream_ptr())
    plain = torch.zeros(H, dtype=torch.float32, device="cuda")
    for e in range(experts):
        plain = plain + contrib[e]
    assert torch.equal(acc32, plain) and torch.equal(acc16, plain.half())
    acc32.zero_()
    capi.call("aeon_moe_fused_w2_accum", capi.vp(hidden), C.byref(w2), capi.vp(d_w),
              capi.vp(shared), capi.vp(acc32), capi.vp(acc16), experts, H, I, 8, 4,
              h.stream_ptr())
    assert h.rel_err(acc16.cpu().numpy(), want_out) <= TOL
    # it adds to what the row holds: a second call doubles the routed part
    capi.call("aeon_moe_fused_w2_accum", capi.vp(hidden), C.byref(w2), capi.vp(d_w), None,
              capi.vp(acc32), capi.vp(acc16), experts, H, I, 8, 4, h.stream_ptr())
    twice = orc.moe_combine(np.concatenate([want_contrib, want_contrib]),
                            shared.cpu().numpy().astype(np.float64))
    assert h.rel_err(acc32.cpu().numpy(), twice) <= TOL


@pytest.mark.parametrize("scale_group", [128, 32])
@pytest.mark.parametrize("use_mfma", [0, 1])
@pytest.mark.parametrize("tokens", [1, 4, 8])
def test_config1_one_expert_decode(orc, tokens, use_mfma, scale_group):
    """benchmark config 1: one routed expert, batch 1/4/8, H=7168, I=2048, clamp 7, output scaled
    by a router weight in (0,1]; with one scale per 128 columns (the config) and with a scale
    of its own per 32 columns (the `.aeon` format's grouping)."""
    torch, h, capi = _setup()
    from project_aeon_amd import synth
    H, I, limit = 7168, 2048, 7.0
    e = h.Expert(0, 0, H, I, scale_group)
    de = h.DevExpert(e)
    x = synth.activations(0, tokens, H)
    w = synth.route_weights(0, tokens)
    d_x, d_w = h.dev_half(x), h.to_dev(w)
    hidden = torch.zeros(tokens, I, dtype=torch.float16, device="cuda")
    contrib = torch.zeros(tokens, H, dtype=torch.float32, device="cuda")
    out = torch.zeros(tokens, H, dtype=torch.float16, device="cuda")
    capi.call("aeon_a64_expert_decode", capi.vp(d_x), tokens, C.byref(de.c), scale_group, capi.vp(d_w),
              capi.vp(hidden), capi.vp(contrib), None, capi.vp(out), H, I, C.c_float(limit),
              use_mfma, h.stream_ptr())
    want, want_hidden = e.ffn(x, limit, round_hidden=True, want_hidden=True)
    want = want * w.astype(np.float64)[:, None]
    assert np.abs(want).max() > 1.0
    # stage by stage at 1e-2: gate/up+SwiGLU against the oracle, then W2 against the oracle fed
    # the device's own fp16 hidden (one flipped fp16 rounding of a hidden value moves near-zero
    # outputs by more than 1e-2 of themselves, so the chained comparison is made on the peak)
    assert h.rel_err(hidden.cpu().numpy(), want_hidden) <= TOL
    staged = e.down(hidden.cpu().numpy()) * w.astype(np.float64)[:, None]
    assert h.rel_err(contrib.cpu().numpy(), staged) <= TOL
    assert h.rel_err(out.cpu().numpy(), staged) <= TOL
    assert np.abs(out.cpu().numpy() - want).max() <= 6e-3 * np.abs(want).max()
    assert torch.equal(out, contrib.half())
    # with a starting row (the accumulator the shared expert has already written), also in place:
    # out = half(float(start) + contrib), fp32 add, one rounding, no fused multiply-add
    start = h.dev_half(synth.activations(5, tokens, H))
    out2 = torch.zeros_like(out)
    capi.call("aeon_a64_expert_decode", capi.vp(d_x), tokens, C.byref(de.c), scale_group, capi.vp(d_w),
              capi.vp(hidden), capi.vp(contrib), capi.vp(start), capi.vp(out2), H, I,
              C.c_float(limit), use_mfma, h.stream_ptr())
    assert torch.equal(out2, (start.float() + contrib).half())
    inplace = start.clone()
    capi.call("aeon_a64_expert_decode", capi.vp(d_x), tokens, C.byref(de.c), scale_group, capi.vp(d_w),
              capi.vp(hidden), capi.vp(contrib), capi.vp(inplace), capi.vp(inplace), H, I,
              C.c_float(limit), use_mfma, h.stream_ptr())
    assert torch.equal(inplace, out2)
    # against the oracle that keeps hidden in fp64 (dsv4_oracle.hpp:1633-1671) the fp16 store of
    # hidden shows up on near-zero outputs, so that comparison is the reference's own: a fraction
    # of the peak (6e-3, tests/test_v4_expert_oracle.cpp:75-77)
    unrounded = e.ffn(x, limit, round_hidden=False) * w.astype(np.float64)[:, None]
    assert np.abs(out.cpu().numpy() - unrounded).max() <= 6e-3 * np.abs(unrounded).max()


def test_mfma_calibration_loop_runs_and_counts_its_flops():
    """The benchmark's measurement aid (calibration/libaeon_calibrate.so, not the product library):
    constant operands of 1.0 make every accumulator entry iterations*32, so the sink is checkable
    in closed form; random operands and the instruction-mix loop only have to stay finite."""
    torch, _, capi = _setup()
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "calibration",
                        "libaeon_calibrate.so")
    assert os.path.exists(path), "calibration/libaeon_calibrate.so is not built (make -C calibration)"
    cal = C.CDLL(path)
    wgs, iters = 8, 50
    sink = torch.zeros(wgs * 256, dtype=torch.float32, device="cuda")
    flop = C.c_double(0.0)
    assert cal.aeon_calibrate_mfma_f16(0, iters, wgs, capi.vp(sink), C.c_size_t(sink.numel()),
                                       C.byref(flop), None) == 0
    torch.cuda.synchronize()
    assert flop.value == wgs * 4 * iters * 16 * 16384.0
    # 16 tiles x 4 entries per lane, each the sum of `iters` MFMAs of 32 products of 1.0
    assert torch.all(sink == 16 * 4 * iters * 32.0)
    assert cal.aeon_calibrate_mfma_f16(1, iters, wgs, capi.vp(sink), C.c_size_t(sink.numel()),
                                       None, None) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(sink).all()
    for shape, waves in ((16, 2), (32, 2), (16, 1)):
        assert cal.aeon_calibrate_mfma_mix(shape, 2, 4, waves, iters, wgs, capi.vp(sink),
                                           C.c_size_t(sink.numel()), C.byref(flop), None) == 0
        torch.cuda.synchronize()
        assert flop.value == wgs * 4 * iters * 32 * 16384.0
        assert torch.isfinite(sink).all()


def test_swizzled_grouped_windows_against_oracle(orc):
    """The grouped entry points over the `.aeon` layout (distinct group-32 scales) on experts that
    own 0, 1, 16, 17, 63, 64, 65 and 130 positions: every window size of the kernel, windows that
    end inside a token tile, an expert split over three windows, an empty expert. Hidden and
    contributions against the fp64 oracle per position (to 2e-3 of the peak: the feed rounds each
    scaled weight to fp16); a strided activation buffer gives the
    same bits as a compact one (tests/test_v4_grouped_wmma_oracle.cpp checks the same)."""
    torch, h, capi = _setup()
    from project_aeon_amd import synth
    H, I, limit = 512, 256, 7.0
    counts = [0, 1, 16, 17, 63, 64, 65, 130]
    E, T = len(counts), 140
    # slot s of token t -> expert: expert e takes its first counts[e] tokens in slot e
    k = E
    ids = np.full((T, k), -1, dtype=np.int32)
    for e, c in enumerate(counts):
        ids[:c, e] = e
    weights = synth.route_weights(41, T * k).reshape(T, k).astype(np.float32)
    x = synth.activations(41, T, H)
    experts = []
    rng = np.random.default_rng(41)
    w13, w2 = capi.W13Table(), capi.W2Table()
    keep = []
    for e in range(E):
        m = {}
        for name, rows, cols in (("w1", I, H), ("w3", I, H), ("w2", H, I)):
            packed = rng.integers(0, 2**32, rows * cols // 8, dtype=np.uint64).astype(np.uint32)
            scale = (0.004 + 0.02 * rng.random(rows * cols // 32)).astype(np.float16).view(np.uint16)
            m[name] = (packed, scale)
        experts.append(m)
        dev = {n: (h.dev_u32(v[0]), h.dev_u16(v[1])) for n, v in m.items()}
        keep.append(dev)
        w13.w1[e], w13.s1[e] = dev["w1"][0].data_ptr(), dev["w1"][1].data_ptr()
        w13.w3[e], w13.s3[e] = dev["w3"][0].data_ptr(), dev["w3"][1].data_ptr()
        w2.w2[e], w2.s2[e] = dev["w2"][0].data_ptr(), dev["w2"][1].data_ptr()
    draws = T * k
    d_ids, d_w = h.to_dev(ids), h.to_dev(weights)
    off = torch.zeros(E + 1, dtype=torch.int32, device="cuda")
    tok = torch.zeros(draws, dtype=torch.int32, device="cuda")
    drw = torch.zeros_like(tok)
    wp = torch.zeros(draws, device="cuda")
    capi.call("aeon_expert_permutation", capi.vp(d_ids), T, k, E, capi.vp(off), capi.vp(tok),
              capi.vp(drw), capi.vp(d_w), capi.vp(wp), h.stream_ptr())
    widest = max(counts)
    results = []
    for stride in (H, H + 64):
        xin = torch.zeros(T, stride, dtype=torch.float16, device="cuda")
        xin[:, :H] = h.dev_half(x)
        hidden = torch.zeros(E * widest * I, dtype=torch.float16, device="cuda")
        contrib = torch.zeros(draws, H, dtype=torch.float32, device="cuda")
        capi.call("aeon_moe_grouped_w13_swiglu", capi.vp(xin), capi.vp(off), capi.vp(tok),
                  C.byref(w13), capi.vp(hidden), E, widest, I, H, 4, 8, C.c_float(limit), stride,
                  h.stream_ptr())
        capi.call("aeon_moe_grouped_w2", capi.vp(hidden), capi.vp(off), capi.vp(drw), capi.vp(wp),
                  C.byref(w2), capi.vp(contrib), E, widest, H, I, 8, 4, h.stream_ptr())
        torch.cuda.synchronize()
        results.append((hidden.cpu().numpy().reshape(E, widest, I), contrib.cpu().numpy()))
    assert np.array_equal(results[0][0], results[1][0]) and np.array_equal(results[0][1], results[1][1])
    got_hidden, got_contrib = results[0]
    assert np.array_equal(off.cpu().numpy(), np.concatenate([[0], np.cumsum(counts)]))
    xf = x.astype(np.float64)
    for e, c in enumerate(counts):
        if c == 0:
            continue
        m = experts[e]
        o, hid = orc.expert_ffn(m["w1"], m["w3"], m["w2"], H, I, xf[:c], limit, round_hidden=True,
                                want_hidden=True)
        # the grouped feed rounds every weight x scale product to fp16 (the reference's rule,
        # swizzled_w4a16_feed.hpp:86), so outputs near zero carry errors that are small against
        # the data's scale and large against themselves: bound |delta| by a fraction of the peak
        got_h = got_hidden[e, :c].astype(np.float64)
        assert np.abs(got_h - hid).max() <= 2e-3 * np.abs(hid).max(), (e, c)
        rows = np.arange(c) * k + e                   # draw index of (token, slot e)
        want = weights[:c, e].astype(np.float64)[:, None] * o
        got_c = got_contrib[rows].astype(np.float64)
        assert np.abs(got_c - want).max() <= 2e-3 * np.abs(want).max(), (e, c)


def test_swizzled_gemv_random_shapes_all_geometries(orc):
    """Forty-eight seeded shapes through the `.aeon`-layout GEMV and dual GEMV: the four storage
    geometries, 1..40 iterations (odd counts, more steps than one lane keeps in flight), row block
    counts that leave waves of the last workgroup without a block. Against the oracle's matvec at
    1e-2; the dual call's first output equals the single call's bit for bit."""
    torch, h, capi = _setup()
    rng = np.random.default_rng(3)
    for case in range(48):
        rpw, lpr = [(4, 8), (8, 4), (2, 16), (16, 2)][case % 4]
        K = int(rng.integers(1, 41)) * lpr * 32
        N = rpw * int(rng.integers(1, 40))
        mats = []
        for _ in range(2):
            packed = rng.integers(0, 2**32, N * K // 8, dtype=np.uint64).astype(np.uint32)
            scale = (0.004 + 0.02 * rng.random(N * K // 32)).astype(np.float16).view(np.uint16)
            mats.append((packed, scale))
        x = rng.standard_normal(K).astype(np.float16)
        d_x = h.dev_half(x)
        dev = [(h.dev_u32(p), h.dev_u16(s_)) for p, s_ in mats]
        y1 = torch.zeros(N, dtype=torch.float16, device="cuda")
        ya, yb = torch.zeros_like(y1), torch.zeros_like(y1)
        capi.call("aeon_w4a16_swizzled_gemv", capi.vp(d_x), capi.vp(dev[0][0]), capi.vp(dev[0][1]),
                  capi.vp(y1), N, K, rpw, lpr, h.stream_ptr())
        capi.call("aeon_w4a16_swizzled_dual_gemv", capi.vp(d_x), capi.vp(dev[0][0]), capi.vp(dev[0][1]),
                  capi.vp(dev[1][0]), capi.vp(dev[1][1]), capi.vp(ya), capi.vp(yb), N, K, rpw, lpr,
                  h.stream_ptr())
        torch.cuda.synchronize()
        what = (case, rpw, lpr, N, K)
        assert torch.equal(y1, ya), what
        for got, (p, s_) in ((ya, mats[0]), (yb, mats[1])):
            want = orc.swizzled_matvec(p, s_, N, K, rpw, lpr, x.astype(np.float64)[None, :])[0]
            assert h.rel_err(got.cpu().numpy(), want) <= TOL, what


def test_standalone_swiglu_clamp_against_the_oracle(orc):
    """aeon_swiglu_clamp (v4_swiglu_clamp_kernel, kernels/v4_swiglu_clamp.hpp:18-34) against
    orc.clamped_swiglu: every pair of the reference's probes {-40,-12,-5,0,5,12,40,3}
    (tests/test_v4_expert_oracle.cpp:302-406: gate < -limit and |up| > limit included) at limits
    7 and 10, then a seeded sweep whose length is not a multiple of the block size. The output
    is one fp16 rounding of an fp32 evaluation: it must equal the fp16 rounding of the oracle's
    fp64 value or its neighbour. The symmetric-clamp misreading (mode 1) must be far off on the
    gate < -limit probes, so the comparison can tell the two rules apart."""
    torch, h, capi = _setup()
    probes = np.array([-40, -12, -5, 0, 5, 12, 40, 3], dtype=np.float16)
    g, u = [a.ravel() for a in np.meshgrid(probes, probes, indexing="ij")]
    rng = np.random.default_rng(77)
    g = np.concatenate([g, rng.uniform(-15, 15, 5003).astype(np.float16)])
    u = np.concatenate([u, rng.uniform(-15, 15, 5003).astype(np.float16)])
    d_g, d_u = h.dev_half(g), h.dev_half(u)
    for limit in (7.0, 10.0):
        out = torch.full((g.size + 16,), 123.0, dtype=torch.float16, device="cuda")
        capi.call("aeon_swiglu_clamp", capi.vp(d_g), capi.vp(d_u), capi.vp(out), g.size,
                  C.c_float(limit), h.stream_ptr())
        got = out.cpu().numpy()
        assert np.all(got[g.size:] == np.float16(123.0))        # nothing written past the end
        got = got[:g.size]
        want = np.array([orc.clamped_swiglu(float(a), float(b), limit) for a, b in zip(g, u)])
        want16 = want.astype(np.float16)
        lo = np.nextafter(want16, np.float16(-np.inf))
        hi = np.nextafter(want16, np.float16(np.inf))
        assert np.all((got == want16) | (got == lo) | (got == hi))
        assert np.mean(got == want16) > 0.97
        wrong = np.array([orc.clamped_swiglu(float(a), float(b), limit, 1) for a, b in zip(g, u)])
        edge = (g.astype(np.float64) <= -limit - 3) & (np.abs(u.astype(np.float64)) >= 3)
        assert edge.sum() >= 10
        assert np.all(np.abs(got[edge].astype(np.float64) - wrong[edge]) >
                      0.5 * np.abs(wrong[edge]))
