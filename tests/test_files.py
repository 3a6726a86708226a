"""Checkpoint files (.hgn / GGUF): the library's parser against the reference's own readers
(hgn::Checkpoint, gguf::File — built into oracle/_ref) on files written by gfx1151_engine_amd.files,
and, on the GPU, layers loaded from a file against the same layers registered directly."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

from gfx1151_engine_amd import capi, files
from oracle import oracle as O
from tests.helpers import HostLayer

D, MID, E, K = 256, 256, 8, 3


def _layers(fmt, n=2, seed=5, router_dtype="f32"):
    rng = np.random.default_rng(seed)
    return [HostLayer(rng, D, MID, E, K, fmt=fmt, router_dtype=router_dtype, shared=(i == 0 or fmt == "q4k"))
            for i in range(n)]


def _hgn(tmp_path, layers, first=3):
    ts = []
    for i, hl in enumerate(layers):
        ts += files.hgn_layer_tensors(first + i, hl)
    ts.append(("model.norm.weight", files.HGN_BF16, [D], np.arange(D, dtype=np.uint16)))
    p = tmp_path / "m.hgn"
    files.write_hgn(p, ts)
    return p, ts


def _gguf(tmp_path, layers, first=0, version_kv=True):
    ts = []
    for i, hl in enumerate(layers):
        ts += files.gguf_layer_tensors(first + i, hl)
    ts.append(("output_norm.weight", files.GGML_F32, [D], np.arange(D, dtype=np.float32)))
    kv = {"general.architecture": "synthmoe", "synthmoe.expert_used_count": K, "synthmoe.expert_count": E,
          "synthmoe.rope.freq_base": 10000.0, "tokenizer.ggml.tokens": ["a", "bc", "def"], "general.alignment": 64}
    p = tmp_path / "m.gguf"
    files.write_gguf(p, ts, kv=kv, align=64)
    return p, ts


HAVE_REF = O.ref() is not None   # the reference readers are an extra witness where oracle/_ref is built


def test_hgn_parser_matches_reference_reader(tmp_path):
    p, ts = _hgn(tmp_path, _layers("q4cp", router_dtype="bf16"))
    f = capi.ModelFile(p)
    assert f.format == capi.FILE_HGN and len(f) == len(ts)
    for name, dt, dims, data in ts:
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        for got in [f.find(name)] + ([O.ref_hgn_tensor(p, name)] if HAVE_REF else []):
            assert got[0] == dt and got[1][:len(dims)] == tuple(dims) and np.array_equal(got[2], raw), name
    assert f.find("layers.0.mlp.gate.weight") is None
    assert not HAVE_REF or O.ref_hgn_tensor(p, "layers.0.mlp.gate.weight") is None
    cfg = f.config(3)
    assert (cfg.d, cfg.mid, cfg.experts, cfg.layers) == (D, MID, E, 2)
    assert f.config(4).layers == 1
    f.close()


def test_gguf_parser_matches_reference_reader(tmp_path):
    p, ts = _gguf(tmp_path, _layers("q4k"))
    f = capi.ModelFile(p)
    assert f.format == capi.FILE_GGUF and len(f) == len(ts)
    for name, dt, ne, data in ts:
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        for got in [f.find(name)] + ([O.ref_gguf_tensor(p, name)] if HAVE_REF else []):
            assert got[0] == dt and got[1][:len(ne)] == tuple(ne) and np.array_equal(got[2], raw), name
    cfg = f.config(0)
    assert (cfg.d, cfg.mid, cfg.experts, cfg.topk, cfg.layers) == (D, MID, E, K, 2)
    if HAVE_REF:
        assert O.ref_gguf_kv_i(p, "synthmoe.expert_used_count") == K
        assert O.ref_gguf_kv_i(p, "general.alignment") == 64
    f.close()


def test_split_gguf_opens_every_shard(tmp_path):
    """<stem>-0000i-of-0000n.gguf: naming any shard opens all of them (src/gguf.h:133-150); metadata of the first
    shard wins.  Checked against the reference's own reader where it is built."""
    layers = _layers("q4k")
    ts = []
    for i, hl in enumerate(layers):
        ts += files.gguf_layer_tensors(i, hl)
    kv0 = {"general.architecture": "synthmoe", "synthmoe.expert_used_count": K, "general.alignment": 64}
    kv1 = {"general.architecture": "synthmoe", "synthmoe.expert_used_count": K + 1, "synthmoe.only_in_shard_2": 7}
    cut = len(ts) // 2 + 1
    p1, p2 = tmp_path / "m-00001-of-00002.gguf", tmp_path / "m-00002-of-00002.gguf"
    files.write_gguf(p1, ts[:cut], kv=kv0, align=64)
    files.write_gguf(p2, ts[cut:], kv=kv1, align=32)
    for path in (p2, p1):
        f = capi.ModelFile(path)
        assert len(f) == len(ts)
        for name, dt, ne, data in ts:
            raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
            for got in [f.find(name)] + ([O.ref_gguf_tensor(path, name)] if HAVE_REF else []):
                assert got[0] == dt and got[1][:len(ne)] == tuple(ne) and np.array_equal(got[2], raw), name
        assert f.config(0).topk == K  # the first shard's value, not the second's
        f.close()
    if HAVE_REF:
        assert O.ref_gguf_kv_i(p2, "synthmoe.expert_used_count") == K
        assert O.ref_gguf_kv_i(p2, "synthmoe.only_in_shard_2") == 7
    # a missing shard is an error, and so is a tensor name that two shards both carry
    os.rename(p2, tmp_path / "gone.gguf")
    with pytest.raises(capi.MoeError):
        capi.ModelFile(p1)
    files.write_gguf(p2, ts[cut - 1:], kv=kv1, align=32)
    with pytest.raises(capi.MoeError):
        capi.ModelFile(p1)


def test_hgn_overlay_replaces_tensors_by_name(tmp_path):
    """hgn::Checkpoint::add_overlay (src/hgn.h:108-121,348-362): tensors of the overlay file replace the base file's;
    the file is left out as a whole if it is already mapped or would replace an hgn v2 tensor."""
    rng = np.random.default_rng(31)
    base_l = HostLayer(rng, D, MID, E, K)
    p, _ = _hgn(tmp_path, [base_l], first=0)
    over = HostLayer(rng, D, MID, E, K, shared_dense="bf16")
    ots = [t for t in files.hgn_layer_tensors(0, over) if "shared_expert." in t[0]]
    po = tmp_path / "overlay.hgn"
    files.write_hgn(po, ots + [("extra.tensor", files.HGN_F32, [4], np.arange(4, dtype=np.float32))])
    f = capi.ModelFile(p)
    n0 = len(f)
    assert f.find("layers.0.mlp.shared_expert.up_proj.weight")[0] == files.HGN_Q4CP
    assert f.add_overlay(po) is True
    assert len(f) == n0 + 1
    got = f.find("layers.0.mlp.shared_expert.up_proj.weight")
    assert got[0] == files.HGN_BF16 and np.array_equal(got[2], np.ascontiguousarray(over.shared[1]).view(np.uint8).reshape(-1))
    assert f.find("layers.0.mlp.gate.weight")[0] in (files.HGN_F32, files.HGN_BF16)  # untouched
    assert f.add_overlay(po) is False and f.add_overlay(p) is False  # already mapped
    f.close()
    # an overlay that would replace an hgn v2 tensor (dtype 23) is left out as a whole
    pv2 = tmp_path / "v2.hgn"
    files.write_hgn(pv2, [("a", 23, [2, 64], np.zeros(64, np.uint8)), ("b", files.HGN_F32, [4], np.zeros(4, np.float32))])
    pov = tmp_path / "ov2.hgn"
    files.write_hgn(pov, [("b", files.HGN_F32, [4], np.ones(4, np.float32)), ("a", files.HGN_F32, [4], np.ones(4, np.float32))])
    f = capi.ModelFile(pv2)
    assert f.add_overlay(pov) is False
    assert f.find("a")[0] == 23 and not f.find("b")[2].any()
    f.close()
    # GGUF files take no overlay; a file that is not HGN1 is refused
    pg, _ = _gguf(tmp_path, _layers("q4k"))
    f = capi.ModelFile(pg)
    with pytest.raises(capi.MoeError):
        f.add_overlay(po)
    f.close()
    f = capi.ModelFile(p)
    with pytest.raises(capi.MoeError):
        f.add_overlay(pg)
    f.close()


@pytest.mark.gpu
def test_layer_loaded_through_an_overlay(tmp_path):
    """Base file with a q4cp shared expert, overlay file with the same tensors in q8g32: the loaded layer computes
    with the overlay's."""
    import torch
    rng = np.random.default_rng(33)
    base_l = HostLayer(rng, D, MID, E, K)
    p, _ = _hgn(tmp_path, [base_l], first=0)
    over = HostLayer(rng, D, MID, E, K, shared_dense="q8g32")  # (the quality overlay's dtype for dense tensors)
    po = tmp_path / "overlay.hgn"
    files.write_hgn(po, [t for t in files.hgn_layer_tensors(0, over) if "shared_expert." in t[0]])
    f = capi.ModelFile(p)
    assert f.add_overlay(po)
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=64)
    w = f.load_layers(m, 0, 0, 1)
    f.close()
    base_l.shared[:3] = over.shared[:3]
    base_l.shared_dense = "q8g32"
    for T in (1, 7, 64):
        x = _x(T, seed=T)
        want, io, _ = O.moe_layer(base_l.oracle_layer(), x)
        y = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :K] == io[:, :K]).all()
        assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), T
    del m
    w.free()


def test_malformed_files_are_rejected(tmp_path):
    lib = capi.lib()

    def rc_of(path):
        h = C.c_void_p()
        rc = lib.moe_file_open(str(path).encode(), C.byref(h))
        if rc == 0:
            lib.moe_file_close(h)
        return rc

    assert rc_of(tmp_path / "absent.hgn") == -2
    (tmp_path / "tiny").write_bytes(b"HGN1")
    assert rc_of(tmp_path / "tiny") == -2
    (tmp_path / "other").write_bytes(b"SAFETENSORS_____")
    assert rc_of(tmp_path / "other") == -1
    p, _ = _hgn(tmp_path, _layers("q4cp", n=1))
    raw = p.read_bytes()
    (tmp_path / "cut.hgn").write_bytes(raw[:-64])            # file_size field no longer matches
    assert rc_of(tmp_path / "cut.hgn") == -2
    bad = bytearray(raw)
    struct.pack_into("<Q", bad, 104 + 96 + 8 + 32, len(raw) + 1)  # first record: data offset past the end
    (tmp_path / "off.hgn").write_bytes(bytes(bad))
    assert rc_of(tmp_path / "off.hgn") == -2
    g, _ = _gguf(tmp_path, _layers("q4k", n=1))
    graw = g.read_bytes()
    (tmp_path / "cut.gguf").write_bytes(graw[:len(graw) // 2])  # tensor data past the end
    assert rc_of(tmp_path / "cut.gguf") == -2
    (tmp_path / "hdr.gguf").write_bytes(graw[:40])              # key-value section cut
    assert rc_of(tmp_path / "hdr.gguf") == -2
    v1 = bytearray(graw)
    struct.pack_into("<I", v1, 4, 1)
    (tmp_path / "v1.gguf").write_bytes(bytes(v1))
    assert rc_of(tmp_path / "v1.gguf") == -1


def test_gguf_dims_that_wrap_around_are_rejected(tmp_path):
    # ne = [2^33, 2^33, 1]: the element count wraps to 4 in 64 bits; the parser must not accept 16 bytes for it
    name = b"blk.0.ffn_down_exps.weight"
    hdr = b"GGUF" + struct.pack("<IQQ", 3, 1, 0)
    hdr += struct.pack("<Q", len(name)) + name + struct.pack("<I", 3) + struct.pack("<3Q", 1 << 33, 1 << 33, 1)
    hdr += struct.pack("<IQ", files.GGML_F32, 0)
    pad = (-len(hdr)) % 32
    p = tmp_path / "wrap.gguf"
    p.write_bytes(hdr + b"\0" * pad + b"\0" * 64)
    h = C.c_void_p()
    assert capi.lib().moe_file_open(str(p).encode(), C.byref(h)) == -2


def test_gguf_offsets_alignment_and_array_sizes_that_wrap_are_rejected(tmp_path):
    """Crafted headers: a tensor offset near 2^64 (data start + offset wraps to a small number that points into
    the header), general.alignment that is no power of two or is huge, and an array whose byte count wraps."""
    lib = capi.lib()

    def rc_of(blob, name):
        p = tmp_path / name
        p.write_bytes(blob)
        h = C.c_void_p()
        rc = lib.moe_file_open(str(p).encode(), C.byref(h))
        if rc == 0:
            lib.moe_file_close(h)
        return rc

    def s(b):
        return struct.pack("<Q", len(b)) + b

    def tensor(name, off):
        return s(name) + struct.pack("<I", 1) + struct.pack("<Q", 8) + struct.pack("<IQ", files.GGML_F32, off)

    def kv_u32(key, v):
        return s(key) + struct.pack("<II", 4, v)

    def pad32(b):
        return b + b"\0" * ((-len(b)) % 32)

    good = pad32(b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + tensor(b"t", 0)) + b"\0" * 64
    assert rc_of(good, "good.gguf") == 0
    hdr = b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + tensor(b"t", (1 << 64) - 32)
    assert rc_of(pad32(hdr) + b"\0" * 64, "wrapoff.gguf") == -2
    for i, al in enumerate((48, 0, 1 << 20)):
        hdr = b"GGUF" + struct.pack("<IQQ", 3, 1, 1) + kv_u32(b"general.alignment", al) + tensor(b"t", 0)
        assert rc_of(hdr + b"\0" * 4096, f"align{i}.gguf") == -2, al
    # array of 2^61 + 1 u64 values: the byte count wraps to 8
    arr = s(b"a") + struct.pack("<IIQ", 9, 10, (1 << 61) + 1)
    hdr = b"GGUF" + struct.pack("<IQQ", 3, 1, 1) + arr + b"\0" * 8 + tensor(b"t", 0)
    assert rc_of(pad32(hdr) + b"\0" * 64, "wraparr.gguf") == -2
    # a GGUF cut in the middle of a tensor-info record
    assert rc_of(good[:len(b"GGUF") + 20 + 12], "cutinfo.gguf") == -2


def _x(T, seed=11):
    return np.random.default_rng(seed).standard_normal((T, D), dtype=np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["q4cp", "q4k"])
def test_layers_loaded_from_file_equal_direct_registration(tmp_path, fmt):
    import torch
    layers = _layers(fmt, n=2, seed=9)
    first = 2
    p, _ = (_hgn if fmt == "q4cp" else _gguf)(tmp_path, layers, first=first)
    f = capi.ModelFile(p)
    cfg = f.config(first)
    m = capi.Moe(cfg.d, cfg.mid, cfg.experts, K, layers=cfg.layers, max_tokens=64)
    f.set_option(capi.FILE_OPT_GGUF_F32_ROUTER, 1)  # bytes unchanged (by default a GGUF's F32 router goes to bf16)
    w = f.load_layers(m, first, 0, cfg.layers)
    f.close()                                  # the device copies do not depend on the mapping
    assert w.nbytes > 0
    for T in (1, 7, 48):
        x = torch.from_numpy(_x(T)).cuda()
        for l, hl in enumerate(layers):
            direct, keep = hl.to_gpu(max_tokens=64)
            y0 = direct.forward(0, x).cpu().numpy()
            y1 = m.forward(l, x).cpu().numpy()
            assert np.array_equal(y0, y1), (fmt, T, l)
            want = O.moe_layer(hl.oracle_layer(), _x(T))[0]
            assert np.abs(y1 - want).max() <= 2e-3 * np.abs(want).max()
            del direct, keep
    # clearing a layer makes forward refuse it; the other layer still runs
    capi.check(capi.lib().moe_clear_layer(m.h, 0), "moe_clear_layer")
    x = torch.from_numpy(_x(1)).cuda()
    y = torch.empty_like(x)
    assert capi.lib().moe_forward(m.h, 0, capi.ptr(x), 1, capi.ptr(y), capi.stream()) == -3
    m.forward(1, x)
    torch.cuda.synchronize()
    del m
    w.free()


@pytest.mark.gpu
def test_hgn_file_with_a_codebook_per_shared_tensor(tmp_path):
    """A standard .hgn file: the routed experts share one codebook, gate_proj / up_proj / down_proj of the shared
    expert each carry their own (tools/flashnext2hgn.py:164-187).  Decode, small batch and grouped-GEMM batch."""
    import torch
    rng = np.random.default_rng(21)
    cbs = [np.sort(rng.standard_normal(16)).astype(np.float32) * (i + 1) for i in range(3)]
    hl = HostLayer(rng, D, MID, E, K, codebook=np.sort(rng.uniform(-2, 2, 16)).astype(np.float32), shared_codebooks=cbs)
    p, _ = _hgn(tmp_path, [hl], first=0)
    f = capi.ModelFile(p)
    cfg = f.config(0)
    m = capi.Moe(cfg.d, cfg.mid, cfg.experts, K, layers=1, max_tokens=80)
    w = f.load_layers(m, 0, 0, 1)
    f.close()
    for T in (1, 9, 80):
        x = _x(T, seed=T)
        want, io, _ = O.moe_layer(hl.oracle_layer(), x)
        y = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :K] == io[:, :K]).all()
        assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), T
    del m
    w.free()


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["bf16", "q8g64", "q8g32"])
def test_hgn_file_with_a_densely_stored_shared_expert(tmp_path, kind):
    """The shared expert as bf16 (an unquantised checkpoint) or q8g64 (the overlay files' storage, src/hgn.h:10):
    the reference runs these through its generic matvec (src/ref.cpp:68-109,623-636)."""
    import torch
    rng = np.random.default_rng(23)
    hl = HostLayer(rng, D, MID, E, K, shared_dense=kind)
    p, _ = _hgn(tmp_path, [hl], first=0)
    f = capi.ModelFile(p)
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=80)
    w = f.load_layers(m, 0, 0, 1)
    f.close()
    for T in (1, 9, 80):
        x = _x(T, seed=T)
        want, io, _ = O.moe_layer(hl.oracle_layer(), x)
        y = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), T
    del m
    w.free()


@pytest.mark.gpu
def test_gguf_router_tensors_are_rounded_to_bf16_like_the_reference(tmp_path):
    """The reference maps a GGUF's F32 ffn_gate_inp / ffn_gate_inp_shexp to bf16 tensors (src/gguf_map.h:210-211), so
    its router multiplies the rounded values.  A loaded layer must route like the oracle fed those bf16 values, and
    like the oracle fed the F32 values only when the file object is told to keep them."""
    import torch
    from gfx1151_engine_amd import synth as S
    rng = np.random.default_rng(33)
    hl = HostLayer(rng, D, MID, E, K, fmt="q4k", router_std=1.0)
    # two pairs of rows that differ by less than a bf16 step: the rounding decides their order for many tokens
    hl.router[1] = hl.router[0] * (1 + 1e-4 * rng.standard_normal(D).astype(np.float32))
    hl.router[5] = hl.router[4] * (1 + 1e-4 * rng.standard_normal(D).astype(np.float32))
    p, _ = _gguf(tmp_path, [hl], first=0)
    T = 64
    x = _x(T, seed=3)
    l32 = hl.oracle_layer()
    y32, i32, w32 = O.moe_layer(l32, x)
    rb = S.f32_to_bf16_bits(hl.router)
    sgb = S.f32_to_bf16_bits(hl.shared[3])
    assert (S.bf16_round(hl.router) != hl.router).any()
    l16 = O.Layer(D, MID, E, K, O.Mat(O.BF16, rb, E, D), O.Mat(hl.tdn, hl.down, E * D, MID),
                  gate=O.Mat(hl.tgu, hl.gate, E * MID, D), up=O.Mat(hl.tgu, hl.up, E * MID, D),
                  shared=[O.Mat(hl.tsh, hl.shared[0], MID, D), O.Mat(hl.tsh, hl.shared[1], MID, D),
                          O.Mat(hl.tsh, hl.shared[2], D, MID), O.Mat(O.BF16, sgb, 1, D)])
    y16, i16, w16 = O.moe_layer(l16, x)
    assert (i16[:, :K] != i32[:, :K]).any(), "the test needs tokens whose routing the rounding changes"
    for keep_f32, (yo, io) in ((0, (y16, i16)), (1, (y32, i32))):
        f = capi.ModelFile(p)
        f.set_option(capi.FILE_OPT_GGUF_F32_ROUTER, keep_f32)
        m = capi.Moe(D, MID, E, K, layers=1, max_tokens=T)
        w = f.load_layers(m, 0, 0, 1)
        f.close()
        y = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :K] == io[:, :K]).all(), keep_f32
        assert np.abs(y - yo).max() <= 2e-3 * np.abs(yo).max(), keep_f32
        del m
        w.free()


@pytest.mark.gpu
def test_mtp_layer_from_a_file(tmp_path):
    """The MTP draft layer's MoE (mtp_moe / mtp_moe_b in the reference): the tensors mtp.layers.0.mlp.* of a .hgn file
    go into one more layer slot behind the trunk's layers; one token, a verify-size batch and a prefill-size batch
    through that slot against the oracle, and the trunk layer next to it is untouched."""
    import torch
    rng = np.random.default_rng(58)
    trunk = HostLayer(rng, D, MID, E, K)
    mtp = HostLayer(rng, D, MID, E, K, router_dtype="bf16")
    ts = files.hgn_layer_tensors(0, trunk)
    ts += [("mtp." + n, dt, dims, a) for n, dt, dims, a in files.hgn_layer_tensors(0, mtp)]
    p = tmp_path / "with_mtp.hgn"
    files.write_hgn(p, ts)
    f = capi.ModelFile(p)
    cfg = f.config(0)
    assert cfg.layers == 1
    m = capi.Moe(cfg.d, cfg.mid, cfg.experts, K, layers=2, max_tokens=70)
    w0 = f.load_layers(m, 0, 0, 1)
    w1 = f.load_mtp_layers(m, 0, 1, 1)
    f.close()
    for T in (1, 5, 70):
        x = _x(T, seed=40 + T)
        xt = torch.from_numpy(x).cuda()
        for slot, hl in ((1, mtp), (0, trunk)):
            want, io, _ = O.moe_layer(hl.oracle_layer(), x)
            y = m.forward(slot, xt).cpu().numpy()
            ids, _ = m.last_routing(T)
            assert (ids.cpu().numpy()[:, :K] == io[:, :K]).all(), (T, slot)
            assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), (T, slot)
    # a file without MTP tensors: nothing to load
    p2, _ = _hgn(tmp_path, [trunk], first=0)
    f2 = capi.ModelFile(p2)
    wv = C.c_void_p()
    assert capi.lib().moe_load_mtp_layers(m.h, f2.h, 0, 1, 1, C.byref(wv), capi.stream()) == -3
    f2.close()
    del m
    w0.free()
    w1.free()


def test_hgn_v2_records_match_reference_reader(tmp_path):
    """An hgn v2 layer's records (dtype 23 expert tensors, dtype 2 planes under the reference's names): the library's
    parser and the reference's own Checkpoint reader agree on dtype, dims and bytes."""
    rng = np.random.default_rng(31)
    hl = HostLayer(rng, D, MID, E, K, fmt="i4r")
    p, ts = _hgn(tmp_path, [hl], first=0)
    f = capi.ModelFile(p)
    names = {t[0] for t in ts}
    assert {"layers.0.mlp.experts.su", "layers.0.mlp.experts.gate_up_proj.svh", "layers.0.mlp.experts.down_proj.suh",
            "layers.0.mlp.experts.down_proj.svh"} <= names
    for name, dt, dims, data in ts:
        raw = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        for got in [f.find(name)] + ([O.ref_hgn_tensor(p, name)] if HAVE_REF else []):
            assert got[0] == dt and got[1][:len(dims)] == tuple(dims) and np.array_equal(got[2], raw), name
    cfg = f.config(0)
    assert (cfg.d, cfg.mid, cfg.experts, cfg.layers) == (D, MID, E, 1)
    f.close()


@pytest.mark.gpu
def test_hgn_v2_layer_loaded_from_a_file(tmp_path):
    """moe_load_layers on an hgn v2 layer: i4r expert tensors copied as they are, the four f16 planes uploaded as f32
    (src/gpu/parts/30_host_util.inc:818-861); decode, small batch and grouped-GEMM batch against the oracle.  A
    file without one of the planes is refused."""
    import torch
    rng = np.random.default_rng(32)
    hl = HostLayer(rng, D, MID, E, K, fmt="i4r")
    p, ts = _hgn(tmp_path, [hl], first=0)
    f = capi.ModelFile(p)
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=80)
    w = f.load_layers(m, 0, 0, 1)
    f.close()
    for T in (1, 9, 80):
        x = _x(T, seed=T)
        want, io, _ = O.moe_layer(hl.oracle_layer(), x)
        y = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :K] == io[:, :K]).all()
        assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), T
    del m
    w.free()
    p2 = tmp_path / "noplane.hgn"
    files.write_hgn(p2, [t for t in ts if not t[0].endswith("down_proj.suh")])
    f = capi.ModelFile(p2)
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=8)
    wh = C.c_void_p()
    assert capi.lib().moe_load_layers(m.h, f.h, 0, 0, 1, C.byref(wh), capi.stream()) == -3
    f.close()


@pytest.mark.gpu
def test_load_rejects_types_outside_the_path(tmp_path):
    # a GGUF whose experts are Q6_K: moe_load_layers reports unsupported and leaves no layer registered
    import torch
    rng = np.random.default_rng(1)
    ts = [("blk.0.ffn_gate_inp.weight", files.GGML_F32, [D, E], rng.standard_normal((E, D), dtype=np.float32))]
    files._GGML_BLOCK[14] = (256, 210)
    for n, ne in (("gate", [D, MID, E]), ("up", [D, MID, E]), ("down", [MID, D, E])):
        ts.append((f"blk.0.ffn_{n}_exps.weight", 14, ne, np.zeros(int(np.prod(ne)) // 256 * 210, np.uint8)))
    p = tmp_path / "q6.gguf"
    files.write_gguf(p, ts, kv={"general.architecture": "x"})
    f = capi.ModelFile(p)
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=8)
    w = C.c_void_p()
    assert capi.lib().moe_load_layers(m.h, f.h, 0, 0, 1, C.byref(w), capi.stream()) == -1
    x = torch.zeros(1, D, device="cuda")
    y = torch.empty_like(x)
    assert capi.lib().moe_forward(m.h, 0, capi.ptr(x), 1, capi.ptr(y), capi.stream()) == -3


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["q4cp", "q4k"])
def test_load_rejects_shapes_that_differ_from_the_context(tmp_path, fmt):
    # the kernels read what the context's shapes say: a file whose tensors are smaller must not be registered
    import torch
    layers = _layers(fmt, n=1, seed=4)
    p, _ = (_hgn if fmt == "q4cp" else _gguf)(tmp_path, layers, first=0)
    f = capi.ModelFile(p)
    for d, mid, e in ((D, 2 * MID, E), (2 * D, MID, E), (D, MID, 2 * E)):
        m = capi.Moe(d, mid, e, K, layers=1, max_tokens=8)
        w = C.c_void_p()
        assert capi.lib().moe_load_layers(m.h, f.h, 0, 0, 1, C.byref(w), capi.stream()) == -2, (d, mid, e)
        x = torch.zeros(1, d, device="cuda")
        y = torch.empty_like(x)
        assert capi.lib().moe_forward(m.h, 0, capi.ptr(x), 1, capi.ptr(y), capi.stream()) == -3
        cfg = capi.Config()
        assert capi.lib().moe_get_config(m.h, C.byref(cfg)) == 0 and (cfg.d, cfg.mid, cfg.experts) == (d, mid, e)
        m.close()
    f.close()


@pytest.mark.gpu
def test_hgn_record_size_must_match_its_dims(tmp_path):
    # a q4cp record that claims more rows than its bytes hold
    layers = _layers("q4cp", n=1, seed=6)
    ts = files.hgn_layer_tensors(0, layers[0])
    name, dt, dims, data = ts[1]
    ts[1] = (name, dt, [dims[0] * 2, dims[1], dims[2]], data)   # experts doubled, bytes unchanged
    p = tmp_path / "short.hgn"
    files.write_hgn(p, ts)
    f = capi.ModelFile(p)
    m = capi.Moe(D, MID, 2 * E, K, layers=1, max_tokens=8)
    w = C.c_void_p()
    assert capi.lib().moe_load_layers(m.h, f.h, 0, 0, 1, C.byref(w), capi.stream()) == -2
    m.close()
    f.close()


@pytest.mark.gpu
def test_large_tensor_takes_the_staged_copy_and_arrives_intact(tmp_path):
    # tensors of 64 MiB and more go through the pinned double-buffered staging (several chunks, worker
    # threads); the layer must still equal the directly registered one bit for bit
    import torch
    d, mid, e, k = 1024, 1024, 72, 4
    rng = np.random.default_rng(31)
    hl = HostLayer(rng, d, mid, e, k, fmt="q4cp", shared=False)
    assert hl.gate_up.nbytes > (64 << 20) > hl.down.nbytes
    p = tmp_path / "big.hgn"
    files.write_hgn(p, files.hgn_layer_tensors(0, hl))
    f = capi.ModelFile(p)
    m = capi.Moe(d, mid, e, k, layers=1, max_tokens=8)
    w = f.load_layers(m, 0, 0, 1)
    f.close()
    x = torch.from_numpy(np.random.default_rng(2).standard_normal((5, d), dtype=np.float32)).cuda()
    direct, keep = hl.to_gpu(max_tokens=8)
    assert torch.equal(direct.forward(0, x), m.forward(0, x))
    torch.cuda.synchronize()
    del m, direct, keep
    w.free()


@pytest.mark.gpu
def test_load_gguf_mixed_types(tmp_path):
    """A GGUF layer in the reference checkpoints' type mix (Q5_K gate/up, Q8_0 down, Q4_K shared expert):
    loaded from the file it gives the same output, bit for bit, as the same bytes registered directly, and
    stays within the GEMV bar of the oracle."""
    import torch
    from helpers import HostLayer, max_abs_rel
    rng = np.random.default_rng(23)
    d, mid, E, k = 512, 256, 8, 3
    hl = HostLayer(rng, d, mid, E, k, fmt="q4k", gg_types=(13, 8, 12))
    ts = files.gguf_layer_tensors(0, hl)
    p = tmp_path / "mixed.gguf"
    files.write_gguf(p, ts, kv={"general.architecture": "x"})
    f = capi.ModelFile(p)
    f.set_option(capi.FILE_OPT_GGUF_F32_ROUTER, 1)  # the comparison below is with the F32 router registered directly
    m = capi.Moe(d, mid, E, k, layers=1, max_tokens=8)
    w = f.load_layers(m, 0, 0, 1)
    x = rng.standard_normal((5, d), dtype=np.float32)
    xt = torch.from_numpy(x).cuda()
    y = m.forward(0, xt).cpu().numpy()
    m2, dev = hl.to_gpu(max_tokens=8)
    y2 = m2.forward(0, xt).cpu().numpy()
    assert (y == y2).all()
    yo, io, wo = O.moe_layer(hl.oracle_layer(), x)
    assert max_abs_rel(y, yo) <= 1e-4
    m.close()
    m2.close()
    w.free()


@pytest.mark.gpu
def test_hgn_v2_file_with_ht_and_q6g64_dense_tensors(tmp_path):
    """An hgn v2 file whose router and shared expert are "ht" tensors (dtype 16, with their .suh / .svh planes) and whose
    shared-expert gate is q6g64 (dtype 24): moe_load_layers turns them into the bf16 matrices of the reference's
    v2_deq_bf16 (src/gpu/parts/30_host_util.inc:1019-1031), so the loaded layer equals, bit for bit, the same layer
    registered with those bf16 matrices, and stays within the layer tolerance of the oracle.  A file without one of the
    planes is refused."""
    import torch
    d, mid, ne, k = 256, 128, 128, 3
    rng = np.random.default_rng(52)
    hl = HostLayer(rng, d, mid, ne, k, fmt="i4r", router_dtype="bf16", shared_dense="bf16")
    raw, extra = {}, []

    def ht(leaf, rows, cols, scale):
        codes = rng.integers(0, 256, rows * cols // 2, dtype=np.uint8)
        pl = [(rng.uniform(0.5, 1.5, n) * rng.choice([-1, 1], n) * s).astype(np.float16) for n, s in ((cols, scale), (rows, 1.0))]
        raw[f"layers.0.mlp.{leaf}.weight"] = (files.HGN_HT, codes)
        extra.extend([(f"layers.0.mlp.{leaf}.suh", files.HGN_F16, [cols], pl[0]), (f"layers.0.mlp.{leaf}.svh", files.HGN_F16, [rows], pl[1])])
        return O.v2_dense_bf16(16, codes, rows, cols, pl[0].astype(np.float32), pl[1].astype(np.float32))

    hl.router = ht("gate", ne, d, 0.02)
    hl.shared[0] = ht("shared_expert.gate_proj", mid, d, 0.05)
    hl.shared[1] = ht("shared_expert.up_proj", mid, d, 0.05)
    hl.shared[2] = ht("shared_expert.down_proj", d, mid, 0.05)
    st = (13 * d // 16 + 15) & ~15
    q6 = rng.integers(0, 256, (1, st), dtype=np.uint8)
    q6[0, 3 * d // 4: 3 * d // 4 + d // 64 * 4] = np.stack([rng.uniform(5e-4, 2e-3, d // 64), rng.uniform(-0.03, -0.01, d // 64)],
                                                          -1).astype(np.float16).view(np.uint8).reshape(-1)
    raw["layers.0.mlp.shared_expert_gate.weight"] = (files.HGN_Q6G64, q6)
    sx_bits = O.v2_dense_bf16(24, q6, 1, d)
    hl.shared[3] = (sx_bits.astype(np.uint32) << 16).view(np.float32)  # the gate as exact f32 for the direct registration
    ts = [(n, raw[n][0], dims, raw[n][1]) if n in raw else (n, dt, dims, a) for n, dt, dims, a in files.hgn_layer_tensors(0, hl)] + extra
    p = tmp_path / "v2dense.hgn"
    files.write_hgn(p, ts)
    f = capi.ModelFile(p)
    m = capi.Moe(d, mid, ne, k, layers=1, max_tokens=80)
    w = f.load_layers(m, 0, 0, 1)
    f.close()
    m2, keep = hl.to_gpu(max_tokens=80)
    for T in (1, 9, 80):
        x = np.random.default_rng(T).standard_normal((T, d), dtype=np.float32)
        want, io, _ = O.moe_layer(hl.oracle_layer(), x)
        xg = torch.from_numpy(x).cuda()
        y = m.forward(0, xg).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
        assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), T
        assert (y == m2.forward(0, xg).cpu().numpy()).all(), T
    del m, m2
    w.free()
    p2 = tmp_path / "noplane.hgn"
    files.write_hgn(p2, [t for t in ts if not t[0].endswith("mlp.gate.svh")])
    f = capi.ModelFile(p2)
    m = capi.Moe(d, mid, ne, k, layers=1, max_tokens=8)
    wh = C.c_void_p()
    assert capi.lib().moe_load_layers(m.h, f.h, 0, 0, 1, C.byref(wh), capi.stream()) == -3
    f.close()
