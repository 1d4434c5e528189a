#!/usr/bin/env python3
"""Writes tests/golden/ref_vectors.npz: small input/output vectors produced by the reference's
OWN host code (its dsv4_oracle.hpp and aeon_w4a16_swizzle.hpp, compiled from /root/reference
into oracle/_ref by oracle/Makefile). The fixture is data only; it lets the C oracle be checked
against the reference where the reference tree is not mounted. Run from the repo root:
    python tests/golden/make_golden.py
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import orc  # noqa: E402

P = lambda a, t: a.ctypes.data_as(C.POINTER(t))
PAYLOAD_BYTES = 14155776


def main():
    ref = orc.ref()
    assert ref is not None, "oracle/_ref is not built (needs /root/reference)"
    out = {}
    rng = np.random.default_rng(20250101)

    # SplitMix64 draws (dsv4_oracle.hpp:42-74)
    for seed in (0, 0x0E7E1217, 0xC0FFEE):
        u = np.empty(16, dtype=np.uint64)
        f = np.empty(16)
        ref.ref_rng_draws(C.c_uint64(seed), 16, P(u, C.c_uint64), P(f, C.c_double), None, C.c_double(1.0))
        out["rng_u64_%x" % seed] = u
        out["rng_uniform_%x" % seed] = f

    # swizzled addresses (dsv4_oracle.hpp:1313-1331) at sampled (row, column)
    for kind, (rows, cols) in enumerate(((2048, 4096), (4096, 2048), (2048, 4096))):
        rc = np.stack([rng.integers(0, rows, 200), rng.integers(0, cols, 200)], axis=1).astype(np.int32)
        res = np.empty((200, 3), dtype=np.int64)
        for i, (r, c) in enumerate(rc):
            a, b, n = C.c_size_t(), C.c_size_t(), C.c_int()
            ref.ref_swizzled_address(kind, int(r), int(c), C.byref(a), C.byref(b), C.byref(n))
            res[i] = (a.value, b.value, n.value)
        out["addr_in_%d" % kind] = rc
        out["addr_out_%d" % kind] = res

    # swizzle of a small matrix (aeon_w4a16_swizzle.hpp:45-85)
    for name, (N, K, rpw, lpr) in (("w13", (8, 512, 4, 8)), ("w2", (16, 256, 8, 4))):
        sp = rng.integers(0, 2**32, N * K // 8, dtype=np.uint32)
        ss = rng.integers(0, 2**16, N * K // 32, dtype=np.uint16)
        dp, ds = np.empty_like(sp), np.empty_like(ss)
        ref.ref_swizzle_u16(P(sp, C.c_uint32), P(ss, C.c_uint16), P(dp, C.c_uint32), P(ds, C.c_uint16),
                            N, K, rpw, lpr)
        out["swz_%s_src_packed" % name], out["swz_%s_src_scale" % name] = sp, ss
        out["swz_%s_dst_packed" % name], out["swz_%s_dst_scale" % name] = dp, ds

    # a seeded payload: decoded samples, one expert FFN (dsv4_oracle.hpp:1442-1488, 1633-1682)
    payload = np.random.default_rng(8).integers(0, 256, PAYLOAD_BYTES, dtype=np.uint8)
    srng = np.random.default_rng(99)
    for so, n in ((4194304, 2048 * 128), (8912896, 4096 * 64), (13631488, 2048 * 128)):
        payload[so:so + 2 * n] = srng.uniform(0.005, 0.02, n).astype(np.float16).view(np.uint8)
    out["payload_seed"] = np.array([8, 99])
    x = np.random.default_rng(4).normal(size=4096)
    y = np.empty(4096)
    ref.ref_expert_ffn(P(payload, C.c_uint8), P(x, C.c_double), C.c_double(10.0), 0, P(y, C.c_double))
    out["ffn_x"], out["ffn_out_limit10"] = x, y
    y2 = np.empty(4096)
    ref.ref_expert_ffn(P(payload, C.c_uint8), P(x, C.c_double), C.c_double(0.5), 0, P(y2, C.c_double))
    out["ffn_out_limit0p5"] = y2
    w1 = np.empty((2048, 4096))
    ref.ref_swizzled_decode(P(payload, C.c_uint8), 0, 1, 1, P(w1, C.c_double))
    out["decode_w1_rows"] = w1[[0, 1, 777, 2047]]

    # clamped SwiGLU (dsv4_oracle.hpp:1591-1606)
    probes = np.array([-40.0, -12.0, -5.0, 0.0, 5.0, 12.0, 40.0, 3.0])
    table = np.empty((3, 8, 8))
    for m in range(3):
        for i, g in enumerate(probes):
            for j, u in enumerate(probes):
                table[m, i, j] = ref.ref_clamped_swiglu(float(g), float(u), 7.0, m)
    out["swiglu_probes"], out["swiglu_limit7"] = probes, table

    # router (dsv4_oracle.hpp:1186-1223) incl. a constructed tie
    logits = rng.normal(0, 2.0, (6, 256))
    bias = rng.normal(0, 0.1, 256)
    logits[0, [7, 40, 41, 200]] = logits[0].max() + 1.0
    bias[[7, 40, 41, 200]] = 0.25
    ids = np.empty((6, 6), dtype=np.int32)
    wts = np.empty((6, 6))
    for t in range(6):
        ref.ref_router_topk(P(logits[t], C.c_double), P(bias, C.c_double), C.c_size_t(256), C.c_size_t(6),
                            C.c_double(1.5), 0, P(ids[t], C.c_int32), P(wts[t], C.c_double))
    out["router_logits"], out["router_bias"], out["router_ids"], out["router_weights"] = logits, bias, ids, wts

    # hyper-connections (dsv4_oracle.hpp:529-632)
    mixes, scale, base = rng.normal(size=24), rng.normal(size=3), rng.normal(size=24)
    pre, post, comb = np.empty(4), np.empty(4), np.empty(16)
    ref.ref_hc_sinkhorn(P(mixes, C.c_double), P(scale, C.c_double), P(base, C.c_double), 4, C.c_double(1e-6),
                        C.c_double(1e-6), C.c_double(2.0), 20, P(pre, C.c_double), P(post, C.c_double),
                        P(comb, C.c_double))
    res, lo = rng.normal(size=(4, 64)), rng.normal(size=64)
    xin, rout = np.empty(64), np.empty((4, 64))
    ref.ref_hc_pre_combine(P(res, C.c_double), P(pre, C.c_double), 4, C.c_size_t(64), P(xin, C.c_double))
    ref.ref_hc_post(P(lo, C.c_double), P(res, C.c_double), P(post, C.c_double), P(comb, C.c_double), 4,
                    C.c_size_t(64), 0, P(rout, C.c_double))
    for k, v in (("mixes", mixes), ("scale", scale), ("base", base), ("pre", pre), ("post", post),
                 ("comb", comb), ("res", res), ("layer_out", lo), ("pre_combine", xin), ("post_out", rout)):
        out["hc_" + k] = v

    # dynamic mixes and RMSNorm (dsv4_oracle.hpp:509-524, :146-169)
    mres, mfn = rng.normal(size=4 * 48), rng.normal(size=(24, 4 * 48))
    mout = np.empty(24)
    ref.ref_hc_mixes(P(mres, C.c_double), P(mfn, C.c_double), C.c_size_t(24), C.c_size_t(4 * 48),
                     C.c_double(1e-6), P(mout, C.c_double))
    nx, nw = rng.normal(size=80), rng.normal(size=80)
    nout, nunit = np.empty(80), np.empty(80)
    ref.ref_rmsnorm(P(nx, C.c_double), P(nw, C.c_double), C.c_size_t(80), C.c_double(1e-6), P(nout, C.c_double))
    ref.ref_rmsnorm(P(nx, C.c_double), None, C.c_size_t(80), C.c_double(1e-6), P(nunit, C.c_double))
    for k, v in (("mix_res", mres), ("mix_fn", mfn), ("mix_out", mout), ("norm_x", nx), ("norm_w", nw),
                 ("norm_out", nout), ("norm_unit", nunit)):
        out["dyn_" + k] = v

    # dense (unquantised) FFN, the shared expert (dsv4_oracle.hpp:1708-1753); its own generator so
    # the vectors above keep their values
    drng = np.random.default_rng(77)
    DI, DH = 48, 80
    dw1, dw3, dw2 = drng.normal(0, 0.3, (DI, DH)), drng.normal(0, 0.3, (DI, DH)), drng.normal(0, 0.3, (DH, DI))
    dx = drng.normal(size=DH)
    for key, limit, mode in (("dense_out_limit10", 10.0, 0), ("dense_out_limit0p25", 0.25, 0),
                             ("dense_out_symmetric0p25", 0.25, 1)):
        dy = np.empty(DH)
        ref.ref_dense_ffn(C.c_size_t(DI), C.c_size_t(DH), P(dx, C.c_double), P(dw1, C.c_double),
                          P(dw3, C.c_double), P(dw2, C.c_double), C.c_double(limit), mode, P(dy, C.c_double))
        out[key] = dy
    out["dense_w1"], out["dense_w3"], out["dense_w2"], out["dense_x"] = dw1, dw3, dw2, dx

    path = os.path.join(ROOT, "tests", "golden", "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
