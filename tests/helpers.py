"""Helpers shared by the tests: synthetic experts in every layout, device upload, comparison."""
import ctypes as C

import numpy as np

import orc
from project_aeon_amd import capi, synth

CFG13 = (4, 8)   # aeon::kCfgW13, aeon_w4a16_swizzle.hpp:14
CFG2 = (8, 4)    # aeon::kCfgW2,  aeon_w4a16_swizzle.hpp:15


def u32p(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint32))


def u16p(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint16))


class Matrix:
    """One int4 matrix in the three layouts: source, `.aeon` swizzled (group-32 scales) and the
    wave64 packing (via the library's own host repack). `scale` is fp16 [N][K/scale_group]:
    with scale_group 128 each scale is replicated over its four group-32 slots of the `.aeon`
    payload and the packing stores one; with 32 every slot has its own and the packing keeps
    all four."""

    def __init__(self, packed_src, scale, N, K, cfg, scale_group=128):
        self.N, self.K, self.cfg, self.scale_group = N, K, cfg, scale_group
        self.src_packed = packed_src
        assert scale.shape == (N, K // scale_group)
        scale32 = np.ascontiguousarray(synth.scale32_from_scale128(scale) if scale_group == 128 else scale)
        self.scale32 = scale32
        self.swz_packed, self.swz_scale = orc.swizzle(packed_src, scale32.view(np.uint16).ravel(),
                                                      N, K, *cfg)
        self.a64_packed = np.empty(N * K // 8, dtype=np.uint32)
        self.a64_scale = np.empty(N * K // scale_group, dtype=np.uint16)
        capi.call("aeon_a64_repack_host", u32p(self.swz_packed), u16p(self.swz_scale), N, K,
                  cfg[0], cfg[1], scale_group, u32p(self.a64_packed), u16p(self.a64_scale))

    def decode(self):
        return orc.swizzled_decode(self.swz_packed, self.swz_scale, self.N, self.K, *self.cfg)


def synth_matrix(seed, expert, matrix, N, K, scale_group=128):
    cfg = CFG2 if matrix == synth.STREAM_W2 else CFG13
    p, s = synth.expert_matrix_source(seed, expert, matrix, N, K, scale_group)
    return Matrix(p, s, N, K, cfg, scale_group)


class Expert:
    def __init__(self, seed, expert, H, I, scale_group=128):
        self.H, self.I, self.scale_group = H, I, scale_group
        self.w1 = synth_matrix(seed, expert, synth.STREAM_W1, I, H, scale_group)
        self.w3 = synth_matrix(seed, expert, synth.STREAM_W3, I, H, scale_group)
        self.w2 = synth_matrix(seed, expert, synth.STREAM_W2, H, I, scale_group)

    def ffn(self, x, limit, round_hidden=True, want_hidden=False):
        """Oracle FFN of fp16 activations x [tokens][H] -> float64 [tokens][H]."""
        return orc.expert_ffn((self.w1.swz_packed, self.w1.swz_scale),
                              (self.w3.swz_packed, self.w3.swz_scale),
                              (self.w2.swz_packed, self.w2.swz_scale), self.H, self.I,
                              np.asarray(x, dtype=np.float64), limit, round_hidden=round_hidden,
                              want_hidden=want_hidden)

    def down(self, hidden):
        """Oracle W2 over given hidden rows [tokens][I] -> float64 [tokens][H]."""
        return orc.swizzled_matvec(self.w2.swz_packed, self.w2.swz_scale, self.H, self.I,
                                   *self.w2.cfg, np.asarray(hidden, dtype=np.float64))


class GeneratedExpert:
    """The oracle's view of synthetic expert (seed, expert): its `.aeon` payload produced by the
    device generator and copied back (the generator is held to the host one bit for bit by the
    GPU suite), for tests that need many full-size experts and cannot afford the host generator.
    Same ffn()/down() as Expert."""

    def __init__(self, seed, expert, H, I, scale_group=128):
        import torch
        self.H, self.I = H, I
        self.mats = []
        for m, (n, k, cfg) in enumerate(((I, H, CFG13), (I, H, CFG13), (H, I, CFG2))):
            p = torch.empty(n * k // 2, dtype=torch.uint8, device="cuda")
            sc = torch.empty(n * k // 32, dtype=torch.int16, device="cuda")
            capi.call("aeon_synth_matrix_swizzled", C.c_uint64(seed), expert, m, n, k, cfg[0], cfg[1],
                      scale_group, capi.vp(p), capi.vp(sc), stream_ptr())
            self.mats.append((p.cpu().numpy().view(np.uint32), sc.cpu().numpy().view(np.uint16)))

    def ffn(self, x, limit, round_hidden=True, want_hidden=False):
        w1, w3, w2 = self.mats
        return orc.expert_ffn(w1, w3, w2, self.H, self.I, np.asarray(x, dtype=np.float64), limit,
                              round_hidden=round_hidden, want_hidden=want_hidden)

    def down(self, hidden):
        p, sc = self.mats[2]
        return orc.swizzled_matvec(p, sc, self.H, self.I, *CFG2, np.asarray(hidden, dtype=np.float64))


def to_dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def dev_u32(a):
    """uint32 numpy -> device tensor (stored as int32 bits)."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int32)).cuda()


def dev_u16(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda()


def dev_half(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float16)).cuda()


class DevExpert:
    """Device copies of an Expert in the wave64 packing plus the ctypes view of them."""

    def __init__(self, e):
        self.t = [dev_u32(e.w1.a64_packed), dev_u16(e.w1.a64_scale), dev_u32(e.w3.a64_packed),
                  dev_u16(e.w3.a64_scale), dev_u32(e.w2.a64_packed), dev_u16(e.w2.a64_scale)]
        self.c = capi.A64Expert(*[t.data_ptr() for t in self.t])


def rel_err(got, want, floor_fraction=1e-3):
    """max |got-want| / max(|want|, floor_fraction*max|want|): the relative error of
    dsv4_oracle.hpp:96-129 (denominator floored at a fraction of the data's scale)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.abs(want).max()
    denom = np.maximum(np.abs(want), floor_fraction * scale)
    return float((np.abs(got - want) / denom).max())


def error_report(got, want):
    """A comparison read the way the reference's `compare` reports it (dsv4_oracle.hpp:96-129):
    the largest |got-want| / max(|want|, f * peak) for four floor fractions f. f = 1.0 is the
    largest error as a fraction of the data's peak -- what the reference's expert gates call
    max_rel (they pass that floor, tests/test_v4_expert_oracle.cpp:86-98) and bound by 6e-3;
    f = 1e-3 is the function's default. For the default floor the element the maximum occurs at
    is reported too: its index, how large the wanted value there is against the peak, and the
    error there against the peak."""
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    peak = np.abs(want).max()
    diff = np.abs(got - want)
    out = {"peak": float(peak)}
    for name, f in (("rel_floor_1", 1.0), ("rel_floor_1e-1", 1e-1), ("rel_floor_1e-2", 1e-2),
                    ("rel_floor_1e-3", 1e-3)):
        rel = diff / np.maximum(np.abs(want), f * peak)
        out[name] = float(rel.max())
    at = int(rel.argmax())
    out.update({"floor_1e-3_at": at, "want_over_peak_there": float(abs(want[at]) / peak),
                "abs_over_peak_there": float(diff[at] / peak)})
    return out


def stream_ptr():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
