"""The weight layouts on the host: the library's swizzle against the oracle's, and the wave64
repack checked bit-exact (round trip, address closed form, dequantised values)."""
import ctypes as C

import numpy as np
import pytest

from helpers import CFG13, CFG2, Matrix, synth_matrix, u16p, u32p
from project_aeon_amd import capi, synth


@pytest.mark.parametrize("N,K,cfg", [(2048, 7168, CFG13), (7168, 2048, CFG2), (16, 256, CFG13),
                                     (32, 128, CFG2), (2048, 4096, CFG13), (4096, 2048, CFG2)])
def test_swizzle_matches_oracle_and_roundtrips(orc, N, K, cfg):
    rng = np.random.default_rng(N + K)
    sp = rng.integers(0, 2**32, N * K // 8, dtype=np.uint32)
    ss = rng.integers(0, 2**16, N * K // 32, dtype=np.uint16)
    dp, ds = np.empty_like(sp), np.empty_like(ss)
    capi.call("aeon_swizzle_w4a16", u32p(sp), u16p(ss), u32p(dp), u16p(ds), N, K, *cfg)
    op, os_ = orc.swizzle(sp, ss, N, K, *cfg)
    assert np.array_equal(dp, op) and np.array_equal(ds, os_)
    bp, bs = np.empty_like(sp), np.empty_like(ss)
    capi.call("aeon_unswizzle_w4a16", u32p(dp), u16p(ds), u32p(bp), u16p(bs), N, K, *cfg)
    assert np.array_equal(bp, sp) and np.array_equal(bs, ss)


def test_swizzle_rejects_bad_shapes():
    a = np.zeros(64, dtype=np.uint32)
    s = np.zeros(64, dtype=np.uint16)
    for N, K, rpw, lpr in [(6, 256, 4, 8), (8, 100, 4, 8), (8, 256, 4, 4), (8, 128, 4, 8), (0, 256, 4, 8)]:
        with pytest.raises(ValueError):
            capi.call("aeon_swizzle_w4a16", u32p(a), u16p(s), u32p(a), u16p(s), N, K, rpw, lpr)


@pytest.mark.parametrize("scale_group", [128, 32])
@pytest.mark.parametrize("N,K,matrix", [(2048, 7168, synth.STREAM_W1), (7168, 2048, synth.STREAM_W2),
                                        (16, 256, synth.STREAM_W1), (48, 384, synth.STREAM_W2),
                                        (2048, 4096, synth.STREAM_W1), (4096, 2048, synth.STREAM_W2)])
def test_a64_repack_bit_exact(orc, N, K, matrix, scale_group):
    """Both scale groupings: 128 (one scale kept of four bit-equal ones) and 32 (the `.aeon`
    format's own, swizzled_expert_format.hpp:18-23, every group-32 scale distinct here)."""
    m = synth_matrix(0, 5, matrix, N, K, scale_group)
    if scale_group == 32:   # the fixture is not a replicated one in disguise
        s = m.scale32.view(np.uint16).reshape(N, K // 128, 4)
        assert np.mean(s[:, :, 0] != s[:, :, 1]) > 0.9
    # the oracle packs straight from the source layout; the library repacks the swizzled payload
    op, os_ = orc.a64_pack(m.src_packed, m.scale32.view(np.uint16), N, K, scale_group)
    assert np.array_equal(m.a64_packed, op)
    assert np.array_equal(m.a64_scale, os_)
    # round trip back to the `.aeon` payload
    bp, bs = np.empty_like(m.swz_packed), np.empty_like(m.swz_scale)
    capi.call("aeon_a64_unrepack_host", u32p(m.a64_packed), u16p(m.a64_scale), N, K, m.cfg[0],
              m.cfg[1], scale_group, u32p(bp), u16p(bs))
    assert np.array_equal(bp, m.swz_packed) and np.array_equal(bs, m.swz_scale)
    assert capi.lib().aeon_a64_packed_bytes(N, K) == m.a64_packed.nbytes
    assert capi.lib().aeon_a64_scale_bytes(N, K, scale_group) == m.a64_scale.nbytes
    assert capi.lib().aeon_a64_scale_bytes(N, K, 64) == 0


@pytest.mark.parametrize("scale_group", [128, 32])
def test_a64_dequantised_weights_bit_exact(orc, scale_group):
    # every element of a small matrix, through both layouts' decoders
    m = synth_matrix(1, 2, synth.STREAM_W1, 64, 512, scale_group)
    want = m.decode()
    got = orc.a64_decode(m.a64_packed, m.a64_scale, 64, 512, scale_group)
    assert np.array_equal(got, want)
    # and through the source layout by hand: (q-8)*scale with q at nibble k%8
    q = (m.src_packed.reshape(64, 64)[:, :, None] >> (4 * np.arange(8, dtype=np.uint32))) & 0xF
    w = (q.reshape(64, 512).astype(np.float64) - 8.0) * np.repeat(m.scale32.astype(np.float64), 32, axis=1)
    assert np.array_equal(w, want)
    assert np.array_equal(np.float32(w).astype(np.float64), w)  # exact in fp32 as well
    if scale_group == 32:
        # reading a four-scale packing as if it held one scale per 128 columns is a different
        # matrix: the two forms cannot be confused silently
        wrong = orc.a64_decode(m.a64_packed, m.a64_scale[: 64 * 512 // 128], 64, 512, 128)
        assert np.abs(wrong - want).max() > 1e-3


@pytest.mark.parametrize("scale_group", [128, 32])
def test_a64_full_size_checksum(orc, scale_group):
    # full-size matrix: sampled elements + a checksum of checksums instead of 14.7M decodes
    N, K = 2048, 7168
    m = synth_matrix(0, 0, synth.STREAM_W1, N, K, scale_group)
    rng = np.random.default_rng(0)
    for _ in range(4000):
        r, c = int(rng.integers(N)), int(rng.integers(K))
        pw, nib, si = orc.a64_address(K, r, c, scale_group)
        q = (int(m.a64_packed[pw]) >> (4 * nib)) & 0xF
        qs = (int(m.src_packed[r * (K // 8) + c // 8]) >> (4 * (c % 8))) & 0xF
        assert q == qs and m.a64_scale[si] == m.scale32.view(np.uint16)[r, c // 32]
    assert int(m.a64_packed.astype(np.uint64).sum()) == int(m.swz_packed.astype(np.uint64).sum())
    assert int(m.a64_scale.astype(np.uint64).sum()) * (4 if scale_group == 128 else 1) == \
        int(m.swz_scale.astype(np.uint64).sum())


def test_a64_repack_rejects_unequal_group32_scales(orc):
    N, K = 16, 256
    p, s128 = synth.expert_matrix_source(0, 0, synth.STREAM_W1, N, K)
    s32 = np.ascontiguousarray(synth.scale32_from_scale128(s128)).view(np.uint16)
    s32[3, 5] ^= 1
    swp, sws = orc.swizzle(p, s32.ravel(), N, K, *CFG13)
    out_p = np.empty(N * K // 8, dtype=np.uint32)
    out_s = np.empty(N * K // 128, dtype=np.uint16)
    with pytest.raises(ValueError, match="group-32"):
        capi.call("aeon_a64_repack_host", u32p(swp), u16p(sws), N, K, 4, 8, 128, u32p(out_p), u16p(out_s))
    with pytest.raises(ValueError):
        capi.call("aeon_a64_repack_host", u32p(swp), u16p(sws), 8, 256, 4, 8, 128, u32p(out_p), u16p(out_s))
    with pytest.raises(ValueError, match="scale_group"):
        capi.call("aeon_a64_repack_host", u32p(swp), u16p(sws), N, K, 4, 8, 64, u32p(out_p), u16p(out_s))
    # the same payload keeps all its scales with scale_group 32, and comes back bit for bit
    out_s4 = np.empty(N * K // 32, dtype=np.uint16)
    capi.call("aeon_a64_repack_host", u32p(swp), u16p(sws), N, K, 4, 8, 32, u32p(out_p), u16p(out_s4))
    bp, bs = np.empty_like(swp), np.empty_like(sws)
    capi.call("aeon_a64_unrepack_host", u32p(out_p), u16p(out_s4), N, K, 4, 8, 32, u32p(bp), u16p(bs))
    assert np.array_equal(bp, swp) and np.array_equal(bs, sws)


def test_host_layout_functions_under_host_sanitizers(tmp_path):
    """Swizzle / unswizzle and the wave64 repack / unrepack on exact-size heap buffers, with the
    layout source file rebuilt under the host-side address and undefined-behaviour sanitizers
    (device code untouched): an access one element past an end, or an overflowing index, ends the
    driver; it also checks both round trips."""
    import os
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    csrc = os.path.join(root, "project-aeon_amd", "csrc")
    lib_dir = os.path.join(root, "project-aeon_amd")
    if not os.path.exists(hipcc) or not os.path.exists(os.path.join(lib_dir, "libaeon_mi355.so")):
        pytest.skip("hipcc or the library is not available")
    inc = ["-I", os.path.join(root, "include"), "-I", csrc]
    dev = ["--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops"]
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined"]
    objs = []
    for src, extra in ((os.path.join(csrc, "layout.hip"), []), (os.path.join(csrc, "errors.cpp"), ["-x", "hip"]),
                       (os.path.join(root, "tests", "cpp", "layout_asan.cpp"), ["-x", "hip"])):
        obj = str(tmp_path / (os.path.basename(src) + ".o"))
        subprocess.run([hipcc] + dev + san + extra + inc + ["-c", src, "-o", obj], check=True,
                       capture_output=True)
        objs.append(obj)
    exe = str(tmp_path / "layout_asan")
    subprocess.run([hipcc, "--offload-arch=gfx950", "-fsanitize=address,undefined", "-fno-gpu-sanitize"]
                   + objs + ["-L", lib_dir, "-laeon_mi355", "-Wl,-rpath," + lib_dir, "-o", exe],
                   check=True, capture_output=True)
    run = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout[-1000:] + run.stderr[-2000:]
