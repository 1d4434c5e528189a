"""The `.aeon` expert container reader and the load-time repack into the resident pool.
The container is written here with the writer's own format statement
(scripts/convert_safetensors_to_aeon.py:463-486: "<12sIIIQ" header, "<QQ" entries); the reader's
checks are the ones AeonModelLoader::open_experts makes (aeon_loader.hpp:345-405)."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

import helpers as h
from project_aeon_amd import capi

H, I = 256, 256
LAYERS, EXPERTS = 2, 3
SECTOR = 4096


def payload_of(expert):
    """One expert's container payload [W1p|W1s|W2p|W2s|W3p|W3s] from its swizzled matrices."""
    parts = [expert.w1.swz_packed, expert.w1.swz_scale, expert.w2.swz_packed, expert.w2.swz_scale,
             expert.w3.swz_packed, expert.w3.swz_scale]
    return b"".join(np.ascontiguousarray(p).tobytes() for p in parts)


def write_container(tmp_path, payloads, layers, experts, version=2, order=None, pad=0,
                    magic=b"AEON_EXPERTS", length_override=None, truncate_entries=0):
    """Payloads land in the file in `order` (default: catalog order) with `pad` sectors of
    filler between them, so the reader has to go by the index, not by position."""
    size = len(payloads[0])
    order = list(range(len(payloads))) if order is None else order
    offsets = [0] * len(payloads)
    blob = bytearray()
    for slot in order:
        blob += b"\xAB" * (pad * SECTOR)
        offsets[slot] = len(blob)
        blob += payloads[slot]
    experts_path = os.path.join(tmp_path, "model_experts_swizzled.aeon")
    index_path = os.path.join(tmp_path, "model_experts_swizzled.index")
    with open(experts_path, "wb") as f:
        f.write(bytes(blob))
    with open(index_path, "wb") as f:
        f.write(struct.pack("<12sIIIQ", magic, version, layers, experts, size))
        entries = [(offsets[i], size if length_override is None else length_override)
                   for i in range(len(payloads))]
        for off, ln in entries[:len(entries) - truncate_entries]:
            f.write(struct.pack("<QQ", off, ln))
    return index_path, experts_path


def open_catalog(index_path, experts_path, version=2, sector=SECTOR):
    cat = C.c_void_p()
    capi.call("aeon_expert_catalog_open", index_path.encode(), experts_path.encode(), version, sector,
              C.byref(cat))
    return cat


@pytest.fixture(scope="module")
def experts():
    return [h.Expert(5, 100 * l + e, H, I) for l in range(LAYERS) for e in range(EXPERTS)]


@pytest.fixture(scope="module")
def experts32():
    """The same experts with a scale of their own per 32 columns: what a real checkpoint holds."""
    return [h.Expert(5, 100 * l + e, H, I, 32) for l in range(LAYERS) for e in range(EXPERTS)]


def test_payload_layout_is_the_reference_constants():
    """At (4096, 2048) the offsets are the reference's hard-coded ones
    (swizzled_expert_format.hpp:11-30)."""
    lay = capi.PayloadLayout()
    capi.call("aeon_payload_layout_for", 4096, 2048, C.byref(lay))
    assert (lay.w1_packed, lay.w1_scale, lay.w2_packed, lay.w2_scale, lay.w3_packed, lay.w3_scale,
            lay.total) == (0, 4194304, 4718592, 8912896, 9437184, 13631488, 14155776)
    capi.call("aeon_payload_layout_for", 7168, 2048, C.byref(lay))
    assert lay.total == 3 * (7168 * 2048 // 2 + 7168 * 2048 // 32 * 2)
    with pytest.raises(ValueError):
        capi.call("aeon_payload_layout_for", 7168, 100, C.byref(lay))


def test_catalog_round_trip(tmp_path, experts):
    payloads = [payload_of(e) for e in experts]
    lay = capi.PayloadLayout()
    capi.call("aeon_payload_layout_for", H, I, C.byref(lay))
    assert lay.total == len(payloads[0]) and lay.total % SECTOR == 0
    order = [4, 0, 5, 2, 1, 3]
    index_path, experts_path = write_container(str(tmp_path), payloads, LAYERS, EXPERTS, order=order,
                                               pad=1)
    cat = open_catalog(index_path, experts_path)
    try:
        layers, per_layer, version = C.c_uint32(), C.c_uint32(), C.c_uint32()
        size = C.c_uint64()
        capi.call("aeon_expert_catalog_info", cat, C.byref(layers), C.byref(per_layer), C.byref(size),
                  C.byref(version))
        assert (layers.value, per_layer.value, size.value, version.value) == (LAYERS, EXPERTS,
                                                                              lay.total, 2)
        for l in range(LAYERS):
            for e in range(EXPERTS):
                ptr, n = C.c_void_p(), C.c_uint64()
                capi.call("aeon_expert_catalog_payload", cat, l, e, C.byref(ptr), C.byref(n))
                assert n.value == lay.total
                assert C.string_at(ptr.value, n.value) == payloads[l * EXPERTS + e]
        with pytest.raises(IndexError):
            capi.call("aeon_expert_catalog_payload", cat, LAYERS, 0, C.byref(ptr), C.byref(n))
        with pytest.raises(IndexError):
            capi.call("aeon_expert_catalog_payload", cat, 0, EXPERTS, C.byref(ptr), C.byref(n))
    finally:
        capi.lib().aeon_expert_catalog_close(cat)


@pytest.mark.parametrize("fault", ["magic", "version", "short_header", "missing_entries",
                                   "bad_length", "misaligned", "past_end", "no_file", "bad_spec"])
def test_catalog_rejects_what_the_reference_rejects(tmp_path, experts, fault):
    payloads = [payload_of(e) for e in experts]
    kw = {}
    if fault == "magic":
        kw["magic"] = b"AEON_EXPERTZ"
    elif fault == "missing_entries":
        kw["truncate_entries"] = 1
    elif fault == "bad_length":
        kw["length_override"] = len(payloads[0]) - 16
    index_path, experts_path = write_container(str(tmp_path), payloads, LAYERS, EXPERTS, **kw)
    version, sector = 2, SECTOR
    expected = OSError
    if fault == "version":
        version = 3
    elif fault == "short_header":
        with open(index_path, "r+b") as f:
            f.truncate(20)
    elif fault == "misaligned":
        sector = 1 << 20          # the payload offsets are multiples of 4096 only
    elif fault == "past_end":
        with open(experts_path, "r+b") as f:
            f.truncate(len(payloads[0]) * 5 + 100)
    elif fault == "no_file":
        os.remove(experts_path)
    elif fault == "bad_spec":
        sector, expected = 3000, ValueError
    with pytest.raises(expected):
        open_catalog(index_path, experts_path, version, sector)


@pytest.mark.gpu
@pytest.mark.parametrize("scale_group", [128, 32])
def test_resident_load_matches_direct_repack(tmp_path, experts, experts32, orc, scale_group):
    """Container -> device staging -> wave64 repack gives, bit for bit, the slots the
    host repack of the same matrices gives; a layer decode through the loaded pool is the one
    through a pool uploaded directly. With one scale per 128 columns (replicated in the payload)
    and with every group-32 scale distinct and kept."""
    import torch
    from project_aeon_amd import moe, synth
    experts = experts32 if scale_group == 32 else experts
    ExpertPool = lambda slots, hh, ii: moe.ExpertPool(slots, hh, ii, scale_group=scale_group)
    payloads = [payload_of(e) for e in experts]
    index_path, experts_path = write_container(str(tmp_path), payloads, LAYERS, EXPERTS,
                                               order=[5, 3, 1, 0, 2, 4], pad=2)
    cat = open_catalog(index_path, experts_path)
    try:
        for layer in range(LAYERS):
            pool = ExpertPool(EXPERTS, H, I)
            pool.buffer.fill_(0x5A)
            pool.load_catalog(cat, layer)
            torch.cuda.synchronize()
            raw = pool.buffer.cpu().numpy()
            base = pool.buffer.data_ptr()
            for s in range(EXPERTS):
                e = experts[layer * EXPERTS + s]
                want = [e.w1.a64_packed, e.w1.a64_scale, e.w3.a64_packed, e.w3.a64_scale,
                        e.w2.a64_packed, e.w2.a64_scale]
                for j, w in enumerate(want):
                    at = int(pool.host_table[s, j]) - base
                    got = raw[at:at + w.nbytes]
                    assert got.tobytes() == w.tobytes(), (layer, s, j)
        # a partial range into the middle of a pool
        pool = ExpertPool(EXPERTS, H, I)
        pool.load_catalog(cat, 1, first=1, count=2, first_slot=1)
        torch.cuda.synchronize()
        e = experts[EXPERTS + 2]
        at = int(pool.host_table[2, 4]) - pool.buffer.data_ptr()
        assert pool.buffer.cpu().numpy()[at:at + e.w2.a64_packed.nbytes].tobytes() == \
            e.w2.a64_packed.tobytes()
        with pytest.raises(IndexError):
            pool.load_catalog(cat, 1, first=2, count=2)
        with pytest.raises(ValueError):
            ExpertPool(EXPERTS, 512, I).load_catalog(cat, 0)   # shape does not match payloads
        # decode through the loaded pool
        pool = ExpertPool(EXPERTS, H, I)
        pool.load_catalog(cat, 0)
        layer0 = moe.MoeLayer(pool, EXPERTS - 1, 2, True, 7.0)
        x = h.dev_half(synth.activations(5, 6, H))
        ids = h.to_dev(np.array([[0, 1], [1, 0], [0, 1], [1, 0], [0, 1], [1, 0]], dtype=np.int32))
        w = h.to_dev(np.full((6, 2), 0.5, dtype=np.float32))
        out = layer0.routed(x, ids, w).cpu().numpy()
        ex = {i: experts[i] for i in range(EXPERTS - 1)}
        import test_gpu_layer as tl
        want = tl._oracle_layer(orc, h, ex, x.cpu().numpy(), ids.cpu().numpy(), w.cpu().numpy(),
                                experts[EXPERTS - 1], 7.0)
        assert np.abs(out - want).max() <= 6e-3 * np.abs(want).max()
    finally:
        capi.lib().aeon_expert_catalog_close(cat)


@pytest.mark.gpu
def test_resident_load_refuses_unequal_scales_in_a_one_scale_pool(tmp_path, experts):
    """A payload whose four group-32 scales of one 128-column group differ cannot be stored with
    one scale per 128 columns: the load fails (it does not return a pool that computes with
    other weights), and the same container loads into a pool that keeps every scale."""
    from project_aeon_amd import moe
    payloads = [bytearray(payload_of(e)) for e in experts]
    lay = capi.PayloadLayout()
    capi.call("aeon_payload_layout_for", H, I, C.byref(lay))
    payloads[1][lay.w2_scale + 6] ^= 0x01          # one fp16 scale bit of expert 1's W2
    index_path, experts_path = write_container(str(tmp_path), [bytes(p) for p in payloads], LAYERS,
                                               EXPERTS)
    cat = open_catalog(index_path, experts_path)
    try:
        pool = moe.ExpertPool(EXPERTS, H, I)
        with pytest.raises(ValueError, match="scale_group 32"):
            pool.load_catalog(cat, 0)
        pool.load_catalog(cat, 1)                     # layer 1 is untouched
        keep = moe.ExpertPool(EXPERTS, H, I, scale_group=32)
        keep.buffer.fill_(0)                          # padding between sub-tensors compares equal
        keep.load_catalog(cat, 0)
        import torch
        torch.cuda.synchronize()
        # the flipped bit is in the pool: slot 1's W2 scales differ from a pool of the clean payload
        clean = moe.ExpertPool(EXPERTS, H, I, scale_group=32)
        clean.buffer.fill_(0)
        os.makedirs(str(tmp_path / "clean"))
        index2, experts2 = write_container(str(tmp_path / "clean"), [payload_of(x) for x in experts],
                                           LAYERS, EXPERTS)
        cat2 = open_catalog(index2, experts2)
        try:
            clean.load_catalog(cat2, 0)
        finally:
            capi.lib().aeon_expert_catalog_close(cat2)
        torch.cuda.synchronize()
        a, b = keep.buffer.cpu().numpy(), clean.buffer.cpu().numpy()
        differing = np.flatnonzero(a != b)
        assert differing.size == 1
        at = int(keep.host_table[1, 5]) - keep.buffer.data_ptr()
        assert at <= differing[0] < at + H * I // 16
    finally:
        capi.lib().aeon_expert_catalog_close(cat)


def test_catalog_reader_survives_mutated_indexes_under_host_sanitizers(tmp_path):
    """The reader parses a file it has no reason to trust. Its source file is rebuilt with the
    host-side address and undefined-behaviour sanitizers (device code untouched), linked into a
    driver that feeds it mutated index files, and the driver has to end normally: every mutation
    either rejected or opened, read and closed without a sanitizer finding."""
    import shutil
    import subprocess
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    csrc = os.path.join(root, "project-aeon_amd", "csrc")
    lib_dir = os.path.join(root, "project-aeon_amd")
    if not os.path.exists(os.path.join(lib_dir, "libaeon_mi355.so")):
        pytest.skip("library not built")
    inc = ["-I", os.path.join(root, "include"), "-I", csrc]
    dev = ["--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops"]
    san = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined"]
    objs = []
    for src, extra in (("artifact.hip", []), ("errors.cpp", ["-x", "hip"])):
        obj = str(tmp_path / (src + ".o"))
        subprocess.run([hipcc] + dev + san + extra + inc + ["-c", os.path.join(csrc, src), "-o", obj],
                       check=True, capture_output=True)
        objs.append(obj)
    driver = str(tmp_path / "fuzz.o")
    subprocess.run([hipcc] + dev + san + ["-x", "hip"] + inc + ["-c",
                    os.path.join(root, "tests", "cpp", "fuzz_catalog.cpp"), "-o", driver],
                   check=True, capture_output=True)
    exe = str(tmp_path / "fuzz_catalog")
    subprocess.run([hipcc, "--offload-arch=gfx950", "-fsanitize=address,undefined", "-fno-gpu-sanitize",
                    driver] + objs + ["-L", lib_dir, "-laeon_mi355", "-Wl,-rpath," + lib_dir, "-o", exe],
                   check=True, capture_output=True)
    run = subprocess.run([exe, "4000"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "opened" in run.stdout and "rejected" in run.stdout
