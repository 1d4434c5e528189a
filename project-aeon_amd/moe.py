"""Host-side view of the HBM-resident expert pool and of one MoE layer, over the C ABI.

ExpertPool plays the part of the reference's UnifiedVRAMExpertPool
(src/backend/swizzled_w4a16/core/vram_expert_pool.hpp:22-82): one device allocation cut into
per-expert slots, each slot the six sub-tensors of an expert -- here in the wave64 packing, with
every expert of the layer resident. torch is used for device memory and streams only.
"""
import ctypes as C

import numpy as np
import torch

from . import capi, synth

CFG13 = (4, 8)
CFG2 = (8, 4)


class MoeLayerStruct(C.Structure):
    _fields_ = [("hidden", C.c_int), ("intermediate", C.c_int), ("experts", C.c_int),
                ("top_k", C.c_int), ("has_shared", C.c_int), ("swiglu_limit", C.c_float),
                ("score_kind", C.c_int), ("routed_scaling_factor", C.c_float),
                ("renormalize", C.c_int), ("d_router_weight", C.c_void_p),
                ("d_router_bias", C.c_void_p), ("d_experts", C.c_void_p),
                ("scale_group", C.c_int), ("d_router_weight_f16", C.c_void_p),
                ("d_shared_w1_f16", C.c_void_p), ("d_shared_w3_f16", C.c_void_p),
                ("d_shared_w2_f16", C.c_void_p)]


class HcPostArgs(C.Structure):
    """aeon_hc_post_args of the C ABI."""
    _fields_ = [("d_residual_in", C.c_void_p), ("token_stride", C.c_long), ("stream_stride", C.c_long),
                ("d_post_mix", C.c_void_p), ("d_comb_mix", C.c_void_p), ("mix_per_token", C.c_int),
                ("d_residual_out", C.c_void_p), ("d_next_pre_mix", C.c_void_p),
                ("next_pre_token_stride", C.c_int), ("d_next_layer_input", C.c_void_p),
                ("next_input_stride", C.c_long)]


def stream_ptr():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class ExpertPool:
    """`slots` experts of shape (H, I) in the wave64 packing, 4096-byte aligned slots laid out
    [W1 packed | W1 scale | W3 packed | W3 scale | W2 packed | W2 scale]. `scale_group` = columns
    per fp16 scale: 128 (payloads whose group-32 scales repeat in fours) or 32 (all kept)."""

    def __init__(self, slots, hidden, intermediate, device="cuda", scale_group=128):
        self.slots, self.H, self.I = slots, hidden, intermediate
        self.scale_group = scale_group
        lib = capi.lib()
        self.pb13 = lib.aeon_a64_packed_bytes(intermediate, hidden)
        self.sb13 = lib.aeon_a64_scale_bytes(intermediate, hidden, scale_group)
        self.pb2 = lib.aeon_a64_packed_bytes(hidden, intermediate)
        self.sb2 = lib.aeon_a64_scale_bytes(hidden, intermediate, scale_group)
        self.slot_bytes = lib.aeon_a64_slot_bytes(hidden, intermediate, scale_group)
        assert self.slot_bytes > 0
        self.payload_bytes = 2 * (self.pb13 + self.sb13) + self.pb2 + self.sb2
        self.buffer = torch.empty(slots * self.slot_bytes, dtype=torch.uint8, device=device)
        base = self.buffer.data_ptr()
        table = np.empty((slots, 6), dtype=np.int64)
        view = capi.A64Expert()
        for s in range(slots):
            capi.call("aeon_a64_slot_views", C.c_void_p(base + s * self.slot_bytes), hidden,
                      intermediate, scale_group, C.byref(view))
            table[s] = [view.w1_packed, view.w1_scale, view.w3_packed, view.w3_scale,
                        view.w2_packed, view.w2_scale]
        self.host_table = table
        self.offsets = [int(v) - base for v in table[0]]  # of the six sub-tensors inside a slot
        self.table = torch.from_numpy(table).to(device)

    def load_catalog(self, catalog, layer, first=0, count=None, first_slot=0):
        """Experts [first, first+count) of `layer` of an opened `.aeon` expert catalog -> slots
        first_slot.. of this pool (payload -> device staging -> wave64 repack). A pool with
        scale_group 128 raises ValueError for a payload whose group-32 scales differ inside 128
        columns."""
        count = self.slots - first_slot if count is None else count
        table = (capi.A64Expert * count)()
        capi.call("aeon_resident_load_layer", catalog, layer, first, count, self.H, self.I,
                  self.scale_group,
                  C.c_void_p(self.buffer.data_ptr() + first_slot * self.slot_bytes),
                  C.c_size_t((self.slots - first_slot) * self.slot_bytes), table)
        for i in range(count):
            got = [table[i].w1_packed, table[i].w1_scale, table[i].w3_packed, table[i].w3_scale,
                   table[i].w2_packed, table[i].w2_scale]
            assert got == [int(v) for v in self.host_table[first_slot + i]]

    def expert_struct(self, slot):
        return capi.A64Expert(*[int(v) for v in self.host_table[slot]])

    def load_swizzled(self, slot, mats, mismatch=None):
        """Load-time re-swizzle of one expert: `mats` = ((w1p, w1s), (w3p, w3s), (w2p, w2s)) device
        tensors in the `.aeon` swizzled layout -> this slot's wave64 packing (device repack)."""
        H, I = self.H, self.I
        shapes = ((I, H, CFG13), (I, H, CFG13), (H, I, CFG2))
        for j, ((p, s), (n, k, cfg)) in enumerate(zip(mats, shapes)):
            capi.call("aeon_a64_repack_device", capi.vp(p), capi.vp(s), n, k, cfg[0], cfg[1],
                      self.scale_group, C.c_void_p(int(self.host_table[slot, 2 * j])),
                      C.c_void_p(int(self.host_table[slot, 2 * j + 1])), capi.vp(mismatch),
                      stream_ptr())

    def fill_synthetic(self, seed, first_expert_id=0):
        """Generate every slot on the device (`.aeon` layout, then the repack), expert id of slot
        s = first_expert_id + s. Returns the number of 128-groups whose four group-32 scales
        differed (must be 0)."""
        H, I = self.H, self.I
        dev = self.buffer.device
        tmp = [(torch.empty(I * H // 2, dtype=torch.uint8, device=dev),
                torch.empty(I * H // 32, dtype=torch.int16, device=dev)) for _ in range(2)]
        tmp.append((torch.empty(H * I // 2, dtype=torch.uint8, device=dev),
                    torch.empty(H * I // 32, dtype=torch.int16, device=dev)))
        shapes = ((I, H, CFG13), (I, H, CFG13), (H, I, CFG2))
        mismatch = torch.zeros(1, dtype=torch.int32, device=dev)
        for s in range(self.slots):
            for m, ((p, sc), (n, k, cfg)) in enumerate(zip(tmp, shapes)):
                capi.call("aeon_synth_matrix_swizzled", C.c_uint64(seed), first_expert_id + s, m, n,
                          k, cfg[0], cfg[1], self.scale_group, capi.vp(p), capi.vp(sc), stream_ptr())
            self.load_swizzled(s, tmp, mismatch)
        return int(mismatch.item())


class MoeLayer:
    """One MoE layer: router + `experts` routed experts (+ an always-on shared expert held in
    the pool's last slot)."""

    def __init__(self, pool, experts, top_k, has_shared, swiglu_limit, router_weight=None,
                 router_bias=None, score_kind=1, routed_scaling_factor=1.0, renormalize=True,
                 router_weight_f16=None, dense_shared=None):
        """router_weight: fp32 [hidden][experts]; router_weight_f16: the checkpoint's form, fp16
        [experts][hidden] (one of the two for decode()). dense_shared: (w1, w3, w2) fp16
        row-major device tensors of an unquantised shared expert (then has_shared is False)."""
        assert pool.slots == experts + (1 if has_shared else 0)
        assert dense_shared is None or not has_shared
        self.pool = pool
        self.router_weight = router_weight
        self.router_weight_f16 = router_weight_f16
        self.dense_shared = dense_shared
        self.router_bias = router_bias
        self.cfg = MoeLayerStruct(pool.H, pool.I, experts, top_k, int(has_shared), swiglu_limit,
                                  score_kind, routed_scaling_factor, int(renormalize),
                                  router_weight.data_ptr() if router_weight is not None else None,
                                  router_bias.data_ptr() if router_bias is not None else None,
                                  pool.table.data_ptr(), pool.scale_group,
                                  router_weight_f16.data_ptr() if router_weight_f16 is not None else None,
                                  *[(t.data_ptr() if dense_shared is not None else None)
                                    for t in (dense_shared or (None, None, None))])
        self.workspace = None
        self.workspace_tokens = 0

    def _workspace(self, tokens):
        if self.workspace is None or tokens > self.workspace_tokens:
            n = capi.lib().aeon_moe_layer_workspace_bytes(C.byref(self.cfg), tokens)
            self.workspace = torch.empty(n, dtype=torch.uint8, device=self.pool.buffer.device)
            self.workspace_tokens = tokens
        return self.workspace

    def _new_out(self, x):
        # with an always-on expert (int4 or dense) every output row is overwritten; without one
        # the routed sum is added to the row, which therefore has to start at zero
        overwritten = self.cfg.has_shared or self.dense_shared is not None
        return torch.empty_like(x) if overwritten else torch.zeros_like(x)

    def decode(self, x, out=None, ids=None, weights=None):
        """x fp16 [tokens][hidden] -> (out fp16 [tokens][hidden], ids int32, weights fp32).
        Without an always-on expert the routed sum is added to what `out` holds, so an `out`
        allocated here starts at zero."""
        tokens = x.shape[0]
        ws = self._workspace(tokens)
        k = self.cfg.top_k
        out = self._new_out(x) if out is None else out
        ids = torch.empty(tokens, k, dtype=torch.int32, device=x.device) if ids is None else ids
        weights = (torch.empty(tokens, k, dtype=torch.float32, device=x.device)
                   if weights is None else weights)
        capi.call("aeon_moe_layer_decode", C.byref(self.cfg), capi.vp(x), x.stride(0), tokens,
                  capi.vp(out), out.stride(0), capi.vp(ids), capi.vp(weights), capi.vp(ws),
                  C.c_size_t(ws.numel()), stream_ptr())
        return out, ids, weights

    def decode_hc_post(self, x, residual_in, residual_out, hc, next_hc=None, next_x=None, out=None,
                       ids=None, weights=None):
        """decode() with the fixed-order reduce, the hyper-connection expansion of `hc` (post and
        comb of a HyperConnection; residuals fp16 [4][tokens][hidden]) and, when `next_hc` is
        given, the next layer's pre-combine into `next_x`, in one launch
        (aeon_moe_layer_decode_hc_post). Returns (out, ids, weights)."""
        tokens = x.shape[0]
        ws = self._workspace(tokens)
        k = self.cfg.top_k
        out = self._new_out(x) if out is None else out
        ids = torch.empty(tokens, k, dtype=torch.int32, device=x.device) if ids is None else ids
        weights = (torch.empty(tokens, k, dtype=torch.float32, device=x.device)
                   if weights is None else weights)
        per_token = int(hc.post.shape[0] > 1)
        args = HcPostArgs(residual_in.data_ptr(), residual_in.stride(1), residual_in.stride(0),
                          hc.post.data_ptr(), hc.comb.data_ptr(), per_token, residual_out.data_ptr(),
                          next_hc.pre.data_ptr() if next_hc is not None else None,
                          (4 if next_hc is not None and next_hc.pre.shape[0] > 1 else 0),
                          next_x.data_ptr() if next_hc is not None else None,
                          next_x.stride(0) if next_hc is not None else 0)
        capi.call("aeon_moe_layer_decode_hc_post", C.byref(self.cfg), capi.vp(x), x.stride(0), tokens,
                  capi.vp(out), out.stride(0), capi.vp(ids), capi.vp(weights), C.byref(args),
                  capi.vp(ws), C.c_size_t(ws.numel()), stream_ptr())
        return out, ids, weights

    def routed(self, x, ids, weights, out=None):
        """The expert part only, for given routing (ids int32 / weights fp32 [tokens][top_k]).
        A layer without an always-on expert adds the routed sum to what `out` holds (the
        reference's in-place accumulator); an `out` allocated here therefore starts at zero."""
        tokens = x.shape[0]
        ws = self._workspace(tokens)
        out = self._new_out(x) if out is None else out
        capi.call("aeon_moe_layer_routed", C.byref(self.cfg), capi.vp(x), x.stride(0), tokens,
                  capi.vp(ids), capi.vp(weights), capi.vp(out), out.stride(0), capi.vp(ws),
                  C.c_size_t(ws.numel()), stream_ptr())
        return out

    def router_logits(self, x):
        """fp32 logits [tokens][experts] of x, by the same kernel (and so the same bits) the
        decode step selects from."""
        tokens = x.shape[0]
        E = self.cfg.experts
        lib = capi.lib()
        if self.router_weight is None:
            half = torch.empty(tokens, E, dtype=torch.float16, device=x.device)
            out = torch.empty(tokens, E, dtype=torch.float32, device=x.device)
            capi.call("aeon_router_logits_f16", capi.vp(x), x.stride(0), capi.vp(self.router_weight_f16),
                      capi.vp(half), capi.vp(out), tokens, self.cfg.hidden, E, stream_ptr())
            return out
        n = lib.aeon_router_logits_workspace_bytes(tokens, self.cfg.hidden, E)
        ws = torch.empty(max(n, 4), dtype=torch.uint8, device=x.device)
        out = torch.empty(tokens, E, dtype=torch.float32, device=x.device)
        capi.call("aeon_router_logits", capi.vp(x), x.stride(0), capi.vp(self.router_weight),
                  capi.vp(out), tokens, self.cfg.hidden, E, capi.vp(ws), C.c_size_t(ws.numel()),
                  stream_ptr())
        return out


class HyperConnection:
    """The static 4-stream mix of one layer boundary: mixes [24] -> (pre [4], post [4], comb [16])
    by the Sinkhorn kernel (20 iterations), shared by every token."""

    def __init__(self, mixes, hc_scale=(1.0, 1.0, 1.0), hc_base=None, pre_eps=1e-6,
                 sinkhorn_eps=1e-6, post_alpha=2.0, iters=20, device="cuda"):
        self.mixes = torch.as_tensor(np.asarray(mixes, dtype=np.float32)).reshape(1, 24).to(device)
        self.scale = torch.as_tensor(np.asarray(hc_scale, dtype=np.float32)).to(device)
        base = np.zeros(24, dtype=np.float32) if hc_base is None else np.asarray(hc_base, np.float32)
        self.base = torch.as_tensor(base).to(device)
        self.pre = torch.empty(1, 4, dtype=torch.float32, device=device)
        self.post = torch.empty(1, 4, dtype=torch.float32, device=device)
        self.comb = torch.empty(1, 16, dtype=torch.float32, device=device)
        capi.call("aeon_hc_sinkhorn_normalize", capi.vp(self.mixes), capi.vp(self.scale),
                  capi.vp(self.base), capi.vp(self.pre), capi.vp(self.post), capi.vp(self.comb), 1,
                  C.c_float(pre_eps), C.c_float(sinkhorn_eps), C.c_float(post_alpha), iters,
                  stream_ptr())

    def pre_combine(self, residual, out):
        """residual fp16 [4][tokens][hidden] -> out fp16 [tokens][hidden]."""
        streams, tokens, hidden = residual.shape
        capi.call("aeon_hc_pre_combine", capi.vp(residual), 0, C.c_long(residual.stride(1)),
                  C.c_long(residual.stride(0)), capi.vp(self.pre), 0, capi.vp(out),
                  C.c_long(out.stride(0)), tokens, hidden, stream_ptr())
        return out

    def post_mix(self, layer_out, residual_in, residual_out):
        streams, tokens, hidden = residual_in.shape
        capi.call("aeon_hc_post", capi.vp(layer_out), C.c_long(layer_out.stride(0)),
                  capi.vp(residual_in), C.c_long(residual_in.stride(1)),
                  C.c_long(residual_in.stride(0)), capi.vp(self.post), capi.vp(self.comb), 0,
                  capi.vp(residual_out), tokens, hidden, stream_ptr())
        return residual_out


class DynamicHyperConnection:
    """The per-token form of the mix (the reference's layer body, v4_layer_body_attention.hpp:
    99-115): mixes = project(residual) per token, Sinkhorn per token, pre-combine with the
    token's own pre-mix, then the FFN RMSNorm; the post expansion uses the token's post/comb."""

    def __init__(self, fn, hc_scale, hc_base, norm_weight=None, rms_eps=1e-6, pre_eps=1e-6,
                 sinkhorn_eps=1e-6, post_alpha=2.0, iters=20, device="cuda"):
        self.fn = torch.as_tensor(np.asarray(fn, dtype=np.float32)).contiguous().to(device)
        self.scale = torch.as_tensor(np.asarray(hc_scale, dtype=np.float32)).to(device)
        self.base = torch.as_tensor(np.asarray(hc_base, dtype=np.float32)).to(device)
        self.norm_weight = None if norm_weight is None else \
            torch.as_tensor(np.asarray(norm_weight, dtype=np.float16)).to(device)
        self.eps = (rms_eps, pre_eps, sinkhorn_eps, post_alpha, iters)
        self.mixes = self.pre = self.post = self.comb = None

    def pre_mix(self, residual, x_pre, x_norm):
        """residual fp16 [4][tokens][hidden] -> x_pre (pre-combined) and x_norm (normed), fp16
        [tokens][hidden]; keeps the per-token mixes for post_mix."""
        streams, tokens, hidden = residual.shape
        rms_eps, pre_eps, sinkhorn_eps, post_alpha, iters = self.eps
        dev = residual.device
        self.mixes = torch.empty(tokens, 24, dtype=torch.float32, device=dev)
        self.pre = torch.empty(tokens, 4, dtype=torch.float32, device=dev)
        self.post = torch.empty(tokens, 4, dtype=torch.float32, device=dev)
        self.comb = torch.empty(tokens, 16, dtype=torch.float32, device=dev)
        capi.call("aeon_hc_project", capi.vp(residual), 0, C.c_long(residual.stride(1)),
                  C.c_long(residual.stride(0)), capi.vp(self.fn), capi.vp(self.mixes), tokens, hidden,
                  C.c_float(rms_eps), stream_ptr())
        capi.call("aeon_hc_sinkhorn_normalize", capi.vp(self.mixes), capi.vp(self.scale),
                  capi.vp(self.base), capi.vp(self.pre), capi.vp(self.post), capi.vp(self.comb),
                  tokens, C.c_float(pre_eps), C.c_float(sinkhorn_eps), C.c_float(post_alpha), iters,
                  stream_ptr())
        capi.call("aeon_hc_pre_combine", capi.vp(residual), 0, C.c_long(residual.stride(1)),
                  C.c_long(residual.stride(0)), capi.vp(self.pre), 4, capi.vp(x_pre),
                  C.c_long(x_pre.stride(0)), tokens, hidden, stream_ptr())
        capi.call("aeon_rmsnorm", capi.vp(x_pre), C.c_long(x_pre.stride(0)),
                  capi.vp(self.norm_weight), capi.vp(x_norm), C.c_long(x_norm.stride(0)), tokens,
                  hidden, C.c_float(rms_eps), stream_ptr())
        return x_norm

    def post_mix(self, layer_out, residual_in, residual_out):
        streams, tokens, hidden = residual_in.shape
        capi.call("aeon_hc_post", capi.vp(layer_out), C.c_long(layer_out.stride(0)),
                  capi.vp(residual_in), C.c_long(residual_in.stride(1)),
                  C.c_long(residual_in.stride(0)), capi.vp(self.post), capi.vp(self.comb), 1,
                  capi.vp(residual_out), tokens, hidden, stream_ptr())
        return residual_out


class LayerStack:
    """benchmark config 4: stacked MoE layers with the hyper-connection residual mix between them.
    Per layer: x = pre-combine(residual); [x = RMSNorm(x) * norm_weight]; y = MoE(x);
    residual = post-mix(y, residual). `norm_weights`: None = no norm (the configuration as
    written); a list with one entry per layer, each a device fp16 [hidden] weight or None for the
    weightless norm = the FFN norm the reference's layer body applies to the layer input
    (layer/v4_layer_body_attention.hpp:113-115). `fused` runs the reduce, the post-mix and the
    next layer's pre-combine in the expert step's last launch instead of three launches of
    their own; same bits."""

    def __init__(self, layers, mixes, norm_weights=None, fused=True, rms_eps=1e-6):
        assert len(layers) == len(mixes)
        assert norm_weights is None or len(norm_weights) == len(layers)
        self.layers = layers
        self.mixes = mixes
        self.norm_weights = norm_weights
        self.fused = fused
        self.rms_eps = rms_eps

    def _norm(self, l, x, out):
        capi.call("aeon_rmsnorm", capi.vp(x), C.c_long(x.stride(0)), capi.vp(self.norm_weights[l]),
                  capi.vp(out), C.c_long(out.stride(0)), x.shape[0], x.shape[1],
                  C.c_float(self.rms_eps), stream_ptr())
        return out

    def step(self, residual, scratch=None, trace=None):
        """residual fp16 [4][tokens][hidden]; returns the new residual (a different buffer).
        `scratch` = (residual-shaped buffer, x [tokens][hidden]) and optionally the layer output,
        ids and weights buffers every layer reuses. A trace entry is (residual in, the
        pre-combined layer input, the input as the router and experts saw it (normed, if the stack
        norms), ids, weights, layer output, residual out)."""
        streams, tokens, hidden = residual.shape
        if scratch is None:
            scratch = (torch.empty_like(residual), torch.empty(tokens, hidden, dtype=torch.float16,
                                                               device=residual.device))
        other, x = scratch[:2]
        bufs = scratch[2:] if len(scratch) > 2 else (None, None, None)
        normed = self.norm_weights is not None
        if normed and getattr(self, "_x_norm", None) is None or (normed and self._x_norm.shape != x.shape):
            self._x_norm = torch.empty_like(x)
        last = len(self.layers) - 1
        for l, (layer, hc) in enumerate(zip(self.layers, self.mixes)):
            if l == 0 or not self.fused:
                hc.pre_combine(residual, x)
            x_in = self._norm(l, x, self._x_norm) if normed else x
            if trace is not None:
                x_pre, x_seen = x.clone(), x_in.clone()
            if bufs[0] is not None and not layer.cfg.has_shared:
                bufs[0].zero_()
            if self.fused:
                nxt = self.mixes[l + 1] if l < last else None
                y, ids, w = layer.decode_hc_post(x_in, residual, other, hc, nxt, x, *bufs)
            else:
                y, ids, w = layer.decode(x_in, *bufs)
                hc.post_mix(y, residual, other)
            if trace is not None:
                trace.append((residual.clone(), x_pre, x_seen, ids.clone(), w.clone(), y.clone(),
                              other.clone()))
            residual, other = other, residual
        return residual
