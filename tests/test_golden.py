"""The C oracle against tests/golden/ref_vectors.npz, vectors the reference's own host code
produced (see tests/golden/make_golden.py). Runs where the reference tree is not mounted."""
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def test_rng(orc, gold):
    for seed in (0, 0x0E7E1217, 0xC0FFEE):
        assert np.array_equal(orc.rng_u64(seed, 16), gold["rng_u64_%x" % seed])
        assert np.array_equal(orc.rng_uniform01(seed, 16), gold["rng_uniform_%x" % seed])


def test_addresses_and_swizzle(orc, gold):
    for kind, (cols, rpw, lpr) in enumerate(((4096, 4, 8), (2048, 8, 4), (4096, 4, 8))):
        for (r, c), want in zip(gold["addr_in_%d" % kind], gold["addr_out_%d" % kind]):
            assert orc.swizzled_address(cols, rpw, lpr, int(r), int(c)) == tuple(int(v) for v in want)
    for name, (N, K, rpw, lpr) in (("w13", (8, 512, 4, 8)), ("w2", (16, 256, 8, 4))):
        dp, ds = orc.swizzle(gold["swz_%s_src_packed" % name], gold["swz_%s_src_scale" % name], N, K, rpw, lpr)
        assert np.array_equal(dp, gold["swz_%s_dst_packed" % name])
        assert np.array_equal(ds, gold["swz_%s_dst_scale" % name])


def _payload(gold):
    a, b = (int(v) for v in gold["payload_seed"])
    payload = np.random.default_rng(a).integers(0, 256, 14155776, dtype=np.uint8)
    srng = np.random.default_rng(b)
    for so, n in ((4194304, 2048 * 128), (8912896, 4096 * 64), (13631488, 2048 * 128)):
        payload[so:so + 2 * n] = srng.uniform(0.005, 0.02, n).astype(np.float16).view(np.uint8)
    return payload


def test_decode_and_expert_ffn(orc, gold):
    p = _payload(gold)
    view = lambda po, so, rows, cols: (p[po:po + rows * cols // 2].view(np.uint32),
                                       p[so:so + rows * cols // 16].view(np.uint16))
    w1, w2, w3 = view(0, 4194304, 2048, 4096), view(4718592, 8912896, 4096, 2048), view(9437184, 13631488, 2048, 4096)
    dec = orc.swizzled_decode(w1[0], w1[1], 2048, 4096, 4, 8)
    assert np.array_equal(dec[[0, 1, 777, 2047]], gold["decode_w1_rows"])
    for key, limit in (("ffn_out_limit10", 10.0), ("ffn_out_limit0p5", 0.5)):
        got = orc.expert_ffn(w1, w3, w2, 4096, 2048, gold["ffn_x"], limit)
        assert np.array_equal(got, gold[key])


def test_swiglu_router_hc(orc, gold):
    probes = gold["swiglu_probes"]
    for m in range(3):
        for i, g in enumerate(probes):
            for j, u in enumerate(probes):
                assert orc.clamped_swiglu(g, u, 7.0, m) == gold["swiglu_limit7"][m, i, j]
    for t in range(6):
        ids, w = orc.router_topk(gold["router_logits"][t], gold["router_bias"], 6, 1.5, score_kind=0)
        assert np.array_equal(ids, gold["router_ids"][t]) and np.array_equal(w, gold["router_weights"][t])
    assert list(gold["router_ids"][0][:4]) == [7, 40, 41, 200]
    pre, post, comb = orc.hc_sinkhorn(gold["hc_mixes"], gold["hc_scale"], gold["hc_base"])
    assert np.array_equal(pre, gold["hc_pre"]) and np.array_equal(post, gold["hc_post"])
    assert np.array_equal(comb, gold["hc_comb"])
    assert np.array_equal(orc.hc_pre_combine(gold["hc_res"], pre, 64), gold["hc_pre_combine"])
    assert np.array_equal(orc.hc_post(gold["hc_layer_out"], gold["hc_res"], post, comb, 64), gold["hc_post_out"])
    assert np.array_equal(orc.hc_mixes(gold["dyn_mix_res"], gold["dyn_mix_fn"]), gold["dyn_mix_out"])
    assert np.array_equal(orc.rmsnorm(gold["dyn_norm_x"], gold["dyn_norm_w"]), gold["dyn_norm_out"])
    assert np.array_equal(orc.rmsnorm(gold["dyn_norm_x"]), gold["dyn_norm_unit"])


def test_dense_ffn(orc, gold):
    for key, limit, mode in (("dense_out_limit10", 10.0, 0), ("dense_out_limit0p25", 0.25, 0),
                             ("dense_out_symmetric0p25", 0.25, 1)):
        got = orc.dense_ffn(gold["dense_w1"], gold["dense_w3"], gold["dense_w2"], gold["dense_x"], limit,
                            clamp_mode=mode)
        assert np.array_equal(got, gold[key])
    assert not np.array_equal(gold["dense_out_limit0p25"], gold["dense_out_symmetric0p25"])
