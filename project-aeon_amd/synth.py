"""Seeded, counter-based synthetic inputs for the routed-expert path (host side, numpy).

Every value is a pure function of (seed, stream, index) through the SplitMix64 finaliser
(the generator the reference's gates use, src/architecture/deepseek_v4/reference/
dsv4_oracle.hpp:42-74): draw i of stream s is SplitMix64 seeded with key(seed, s), i-th output.
The device generator in csrc/synth.hip evaluates the same function, so tens of gigabytes of int4
experts can be produced in HBM and any one of them regenerated here for checking.

Weights are defined in the *source* layout of aeon_w4a16_swizzle.hpp:45-85: packed [N][K/8]
u32 with column k in nibble k%8 (value q in 0..15, weight q-8), one fp16 scale per
(row, 128-column group) uniform in [0.005, 0.02] -- replicated over the four group-32 slots
of the `.aeon` payload -- or, with scale_group 32, one per (row, 32-column group) as the
reference's format stores them (swizzled_expert_format.hpp:18-23).
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_STREAM = np.uint64(0xD6E8FEB86659FD93)

# stream ids
STREAM_W1, STREAM_W3, STREAM_W2 = 0, 1, 2
STREAM_SCALE = 8          # + matrix stream
STREAM_ACTIVATION = 32
STREAM_ROUTER_W = 33
STREAM_ROUTER_BIAS = 34
STREAM_ROUTE_WEIGHT = 35
STREAM_ZIPF = 36
STREAM_HC = 37


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def stream_key(seed, stream, unit=0):
    """Key of one stream: (seed, stream id, unit such as the expert index)."""
    with np.errstate(over="ignore"):
        k = _mix(np.uint64(seed) ^ (np.uint64(stream + 1) * _STREAM))
        k = _mix(k ^ (np.uint64(unit + 1) * _GOLDEN))
    return k if k != 0 else _GOLDEN


def draws(key, start, count):
    """SplitMix64 outputs number start..start+count-1 of the stream `key` (uint64)."""
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + count + 1, dtype=np.uint64)
        return _mix(np.uint64(key) + i * _GOLDEN)


def uniform01(u64):
    return (u64 >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def normal(key, count):
    """N(0,1) by Box-Muller in fp64: draws 2i, 2i+1 give value i."""
    u = draws(key, 0, 2 * count)
    u1 = ((u[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
    u2 = uniform01(u[1::2])
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def expert_matrix_source(seed, expert, matrix, N, K, scale_group=128):
    """(packed [N*K/8] u32, scale [N][K/scale_group] fp16) of one matrix in the source layout.
    Word w takes the low or high 32 bits of draw w//2; the scale of (row, g) is draw
    row*(K/scale_group)+g of the matrix's scale stream mapped to [0.005, 0.02] and rounded to
    fp16."""
    words = N * K // 8
    u = draws(stream_key(seed, matrix, expert), 0, (words + 1) // 2)
    packed = np.empty(2 * u.size, dtype=np.uint32)
    packed[0::2] = (u & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    packed[1::2] = (u >> np.uint64(32)).astype(np.uint32)
    packed = packed[:words]
    s = uniform01(draws(stream_key(seed, STREAM_SCALE + matrix, expert), 0, N * (K // scale_group)))
    scale = (0.005 + 0.015 * s).astype(np.float16).reshape(N, K // scale_group)
    return packed, scale


def scale32_from_scale128(scale128):
    """[N][K/128] -> [N][K/32]: each scale replicated over its four group-32 slots."""
    return np.repeat(scale128, 4, axis=1)


def activations(seed, tokens, hidden, unit=0):
    return normal(stream_key(seed, STREAM_ACTIVATION, unit), tokens * hidden).astype(
        np.float16).reshape(tokens, hidden)


def router_weight(seed, hidden, experts, unit=0, std=0.02):
    """fp32 [hidden][experts] ~ N(0, std)."""
    return (normal(stream_key(seed, STREAM_ROUTER_W, unit), hidden * experts) * std).astype(
        np.float32).reshape(hidden, experts)


def router_bias(seed, experts, unit=0, std=0.1):
    return (normal(stream_key(seed, STREAM_ROUTER_BIAS, unit), experts) * std).astype(np.float32)


def route_weights(seed, count, unit=0):
    """Uniform in (0, 1]."""
    u = draws(stream_key(seed, STREAM_ROUTE_WEIGHT, unit), 0, count)
    return (((u >> np.uint64(11)).astype(np.float64) + 1.0) *
            (1.0 / 9007199254740992.0)).astype(np.float32)


def zipf_routing(seed, tokens, experts, top_k, s=1.1, unit=0):
    """ids [tokens][top_k] int32: per token, top_k distinct experts drawn without replacement
    with probability proportional to rank^-s (expert e has rank e+1), by the Gumbel top-k trick
    so the draw is one vectorised pass; ids within a token are in descending key order.
    weights [tokens][top_k] fp32: uniform (0,1], renormalised to sum 1 per token."""
    u = uniform01(draws(stream_key(seed, STREAM_ZIPF, unit), 0, tokens * experts))
    u = np.clip(u, 1e-300, 1.0 - 1e-16).reshape(tokens, experts)
    logp = -s * np.log(np.arange(1, experts + 1, dtype=np.float64))
    keys = logp[None, :] - np.log(-np.log(u))
    ids = np.argsort(-keys, axis=1, kind="stable")[:, :top_k].astype(np.int32)
    w = route_weights(seed, tokens * top_k, unit=unit + 1000).astype(np.float64).reshape(
        tokens, top_k)
    w = (w / w.sum(axis=1, keepdims=True)).astype(np.float32)
    return ids, w
