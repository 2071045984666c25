"""GGUF container reader (bpk_gguf_*): the library against files whose contents
are known by construction, against the oracle's restatement of the reference
parser, and against the reference's own parser where oracle/_ref was built.
CPU only: no device call is made here."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

import gguf_writer as gw
from backpack_amd import capi, synth
from backpack_amd.gguf import GGUFFile
from oracle import gguf_oracle as go

Q4_K, Q6_K = 12, 14


def _model_file(tmp_path, version=3, alignment=32, declare=False, name="m.gguf"):
    """A small file with every metadata kind and a mix of tensor types."""
    rng = np.random.default_rng(5)
    q4 = synth.make_raw(Q4_K, 6, 512, seed=1)
    q6 = synth.make_raw(Q6_K, 3, 256, seed=2)
    f32 = rng.standard_normal(7).astype(np.float32)
    f16 = rng.standard_normal((2, 5)).astype(np.float16)
    metadata = [
        ("general.architecture", gw.STRING, "qwen3"),
        ("general.name", gw.STRING, "tiny é中"),
        ("qwen3.block_count", gw.U32, 36),
        ("qwen3.embedding_length", gw.U64, 4096),
        ("qwen3.context_length", gw.I32, 40960),
        ("qwen3.neg", gw.I64, -2),
        ("small.u8", gw.U8, 200), ("small.i8", gw.I8, -5), ("small.u16", gw.U16, 65000), ("small.i16", gw.I16, -300),
        ("qwen3.rope.freq_base", gw.F32, 1000000.0),
        ("qwen3.attention.layer_norm_rms_epsilon", gw.F64, 1e-6),
        ("flag.on", gw.BOOL, 1), ("flag.off", gw.BOOL, 0),
        ("tokenizer.ggml.tokens", gw.ARRAY, (gw.STRING, ["<pad>", "a", "", "hello world", "中"])),
        ("tokenizer.ggml.token_type", gw.ARRAY, (gw.I32, [1, 3, 3, 1, 6])),
        ("gemma.feed_forward_length", gw.ARRAY, (gw.U32, [6144, 12288, 1228])),
        ("empty.ints", gw.ARRAY, (gw.I32, [])),
        ("scores", gw.ARRAY, (gw.F32, [0.5, -1.25, 3.0])),
        ("mask", gw.ARRAY, (gw.BOOL, [1, 0, 1, 1])),
        ("bytes", gw.ARRAY, (gw.U8, [1, 2, 3, 250])),
        ("wide", gw.ARRAY, (gw.U64, [1 << 40, 7])),
        ("nested", gw.ARRAY, (gw.ARRAY, [(gw.I32, [1, 2]), (gw.STRING, ["x"])])),
        ("empty.string", gw.STRING, ""),
    ]
    tensors = [
        ("blk.0.ffn_gate.weight", (512, 6), Q4_K, q4.tobytes()),
        ("output_norm.weight", (7,), 0, f32.tobytes()),
        ("blk.0.attn_v.weight", (256, 3), Q6_K, q6.tobytes()),
        ("tiny.f16", (5, 2), 1, f16.tobytes()),
        ("odd.type", (32, 2), 16, b"\x11" * 20),    # IQ2_XXS: a type whose size the reader does not know
    ]
    path = str(tmp_path / name)
    offsets, data_offset = gw.write(path, metadata, tensors, version=version, alignment=alignment,
                                    declare_alignment=declare)
    return path, metadata, tensors, offsets, data_offset


def test_reads_what_was_written(tmp_path):
    path, metadata, tensors, offsets, data_offset = _model_file(tmp_path)
    with GGUFFile(path) as g:
        assert (g.version, g.n_tensors, g.n_kv, g.data_offset) == (3, len(tensors), len(metadata), data_offset)
        blob = open(path, "rb").read()
        infos = g.tensors
        assert [t.name for t in infos] == [t[0] for t in tensors]          # file order kept
        for info, (name, dims, type_, data) in zip(infos, tensors):
            assert (info.type, info.shape, info.offset) == (type_, dims, offsets[name])
            by_name = g.tensor(name)
            assert by_name == info
            if type_ == 16:
                assert info.nbytes == 0
                first = (C.c_uint8 * 20).from_address(info.address)
                assert bytes(first) == data
            else:
                assert info.nbytes == len(data)
                assert g.tensor_bytes(name).tobytes() == data
                assert blob[data_offset + info.offset:][:len(data)] == data
        # scalars, with the widening rules of the reference's getters
        assert g.get_string("general.architecture") == "qwen3"
        assert g.get_string("general.name") == "tiny é中"
        assert g.get_string("empty.string", "dflt") == ""
        assert g.get_string("missing", "dflt") == "dflt"
        assert g.get_string("qwen3.block_count", "dflt") == "dflt"
        assert g.get_u32("qwen3.block_count") == 36
        assert g.get_u32("qwen3.embedding_length") == 4096
        assert g.get_u32("qwen3.context_length") == 40960
        assert g.get_u32("qwen3.neg") == 0xFFFFFFFE
        assert (g.get_u32("small.u8"), g.get_u32("small.u16")) == (200, 65000)
        assert (g.get_u32("small.i8"), g.get_u32("small.i16")) == ((-5) & 0xFFFFFFFF, (-300) & 0xFFFFFFFF)
        assert g.get_u32("missing", 17) == 17
        assert g.get_u32("general.name", 17) == 17
        assert g.get_u32("qwen3.rope.freq_base", 17) == 17
        assert g.get_u32("gemma.feed_forward_length") == 12288              # largest element of an int array
        assert g.get_u32("tokenizer.ggml.token_type") == 6
        assert g.get_u32("empty.ints", 9) == 9
        assert g.get_float("qwen3.rope.freq_base") == 1000000.0
        assert g.get_float("qwen3.attention.layer_norm_rms_epsilon") == np.float32(1e-6)
        assert g.get_float("qwen3.block_count", 2.5) == 2.5
        assert g.get_bool("flag.on") is True and g.get_bool("flag.off", True) is False
        assert g.get_bool("missing", True) is True and g.get_bool("qwen3.block_count", True) is True
        assert g.has_key("flag.off") and not g.has_key("flag")
        assert (g.key_type("scores"), g.key_type("flag.on"), g.key_type("nope")) == (gw.ARRAY, gw.BOOL, -1)
        # arrays
        assert g.get_string_array("tokenizer.ggml.tokens") == ["<pad>", "a", "", "hello world", "中"]
        assert g.get_string_array("scores") == [] and g.get_string_array("missing") == []
        assert g.get_array("tokenizer.ggml.token_type").tolist() == [1, 3, 3, 1, 6]
        assert g.get_array("scores").tolist() == [0.5, -1.25, 3.0]
        assert g.get_array("mask").tolist() == [1, 0, 1, 1]
        assert g.get_array("bytes").tolist() == [1, 2, 3, 250]
        assert g.get_array("wide").tolist() == [1 << 40, 7]
        assert g.array_len("nested") == (0, gw.ARRAY) and g.get_array("nested").size == 0
        assert g.array_len("tokenizer.ggml.tokens") == (5, gw.STRING)
        with pytest.raises(capi.BpkError) as e:
            g.tensor("no.such.tensor")
        assert e.value.code == -10
        with pytest.raises(capi.BpkError):
            g.tensor_at(len(tensors))


@pytest.mark.parametrize("version,alignment,declare", [(2, 32, False), (3, 64, True), (3, 4096, True), (3, 8, True)])
def test_versions_and_declared_alignment(tmp_path, version, alignment, declare):
    path, _, tensors, offsets, data_offset = _model_file(tmp_path, version, alignment, declare)
    with GGUFFile(path) as g:
        assert g.version == version and g.data_offset == data_offset
        assert g.tensor_bytes("blk.0.attn_v.weight").tobytes() == tensors[2][3]
        assert g.tensor("blk.0.attn_v.weight").offset % alignment == 0


def _ref_dump(kqref, path):
    r = kqref.ref()
    r.bpref_gguf_open.restype = C.c_void_p
    r.bpref_gguf_open.argtypes = [C.c_char_p]
    h = r.bpref_gguf_open(path.encode())
    assert h, "the reference parser refused the file"
    return r, C.c_void_p(h)


def test_oracle_restatement_against_known_contents_and_reference(tmp_path, request):
    path, metadata, tensors, offsets, data_offset = _model_file(tmp_path)
    p = go.parse(open(path, "rb").read())
    assert (p.version, p.n_tensors, p.data_offset) == (3, len(tensors), data_offset)
    assert p.tensors == [(n.encode(), d, t, offsets[n]) for n, d, t, _ in tensors]
    assert go.get_u32(p, b"gemma.feed_forward_length") == 12288
    assert go.get_u32(p, b"qwen3.neg") == 0xFFFFFFFE and go.get_u32(p, b"empty.ints", 9) == 9
    assert go.get_float(p, b"qwen3.attention.layer_norm_rms_epsilon") == np.float32(1e-6)
    assert go.get_string(p, b"general.architecture") == b"qwen3"
    assert p.metadata[b"tokenizer.ggml.tokens"] == ("strs", [b"<pad>", b"a", b"", b"hello world", "中".encode()])
    assert p.metadata[b"mask"] == ("bools", [True, False, True, True])
    assert p.metadata[b"bytes"][0] == "skipped" and p.metadata[b"nested"][0] == "skipped"
    kqref = request.getfixturevalue("kqref")     # skips from here on where the reference did not build
    r, h = _ref_dump(kqref, path)
    try:
        v, nt, off = C.c_uint32(), C.c_uint64(), C.c_uint64()
        r.bpref_gguf_info(h, C.byref(v), C.byref(nt), C.byref(off))
        assert (v.value, nt.value, off.value) == (p.version, p.n_tensors, p.data_offset)
        r.bpref_gguf_u32.restype = C.c_uint32
        r.bpref_gguf_u32.argtypes = [C.c_void_p, C.c_char_p, C.c_uint32]
        r.bpref_gguf_f32.restype = C.c_float
        r.bpref_gguf_f32.argtypes = [C.c_void_p, C.c_char_p, C.c_float]
        r.bpref_gguf_bool.argtypes = [C.c_void_p, C.c_char_p, C.c_int]
        r.bpref_gguf_has_key.argtypes = [C.c_void_p, C.c_char_p]
        r.bpref_gguf_string.restype = C.c_size_t
        r.bpref_gguf_string.argtypes = [C.c_void_p, C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t]
        keys = [k.encode() for k, _, _ in metadata] + [b"missing"]
        buf = C.create_string_buffer(256)
        for k in keys:
            assert r.bpref_gguf_u32(h, k, 77) == go.get_u32(p, k, 77), k
            assert r.bpref_gguf_f32(h, k, 1.5) == go.get_float(p, k, 1.5), k
            assert bool(r.bpref_gguf_bool(h, k, 1)) == go.get_bool(p, k, True), k
            assert bool(r.bpref_gguf_bool(h, k, 0)) == go.get_bool(p, k, False), k
            assert bool(r.bpref_gguf_has_key(h, k)) == (k in p.metadata)
            n = r.bpref_gguf_string(h, k, b"dflt", buf, 256)
            assert buf.raw[:n] == go.get_string(p, k, b"dflt"), k
        r.bpref_gguf_tensor.argtypes = [C.c_void_p, C.c_uint64, C.POINTER(C.c_char_p), C.POINTER(C.c_uint32),
                                        C.POINTER(C.c_uint32), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        r.bpref_gguf_find.restype = C.c_int64
        r.bpref_gguf_find.argtypes = [C.c_void_p, C.c_char_p]
        for i, (name, shape, type_, offset) in enumerate(p.tensors):
            nm, ty, nd, dims, of = C.c_char_p(), C.c_uint32(), C.c_uint32(), (C.c_uint64 * 8)(), C.c_uint64()
            assert r.bpref_gguf_tensor(h, i, C.byref(nm), C.byref(ty), C.byref(nd), dims, C.byref(of)) == 0
            assert (nm.value, ty.value, tuple(dims[:nd.value]), of.value) == (name, type_, shape, offset)
            assert r.bpref_gguf_find(h, name) == i
        assert r.bpref_gguf_find(h, b"nope") == -1
        r.bpref_gguf_string_array_len.restype = C.c_int64
        r.bpref_gguf_string_array_len.argtypes = [C.c_void_p, C.c_char_p]
        r.bpref_gguf_string_array_at.restype = C.c_size_t
        r.bpref_gguf_string_array_at.argtypes = [C.c_void_p, C.c_char_p, C.c_uint64, C.c_char_p, C.c_size_t]
        toks = p.metadata[b"tokenizer.ggml.tokens"][1]
        assert r.bpref_gguf_string_array_len(h, b"tokenizer.ggml.tokens") == len(toks)
        for i, t in enumerate(toks):
            n = r.bpref_gguf_string_array_at(h, b"tokenizer.ggml.tokens", i, buf, 256)
            assert buf.raw[:n] == t
        r.bpref_gguf_i32_array.restype = C.c_int64
        r.bpref_gguf_i32_array.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_int32), C.c_uint64]
        out = (C.c_int32 * 8)()
        assert r.bpref_gguf_i32_array(h, b"tokenizer.ggml.token_type", out, 8) == 5
        assert list(out[:5]) == p.metadata[b"tokenizer.ggml.token_type"][1]
        assert r.bpref_gguf_i32_array(h, b"scores", out, 8) == -1
    finally:
        r.bpref_gguf_close.argtypes = [C.c_void_p]
        r.bpref_gguf_close(h)


def test_library_agrees_with_oracle_on_every_key(tmp_path):
    """Same getters, same defaults — except where the library keeps what the reference drops:
    an array the reference skips reads there as an empty string; here it is an array and
    get_string returns the default."""
    path, metadata, tensors, _, _ = _model_file(tmp_path)
    p = go.parse(open(path, "rb").read())
    with GGUFFile(path) as g:
        assert (g.version, g.n_tensors, g.data_offset) == (p.version, p.n_tensors, p.data_offset)
        for k, _, _ in metadata + [("missing", 0, 0)]:
            kb = k.encode()
            assert g.get_u32(k, 77) == go.get_u32(p, kb, 77), k
            assert g.get_float(k, 1.5) == go.get_float(p, kb, 1.5), k
            assert g.get_bool(k, True) == go.get_bool(p, kb, True) and g.get_bool(k, False) == go.get_bool(p, kb, False)
            assert g.has_key(k) == (kb in p.metadata)
            if p.metadata.get(kb, ("", 0))[0] != "skipped":
                assert g.get_string(k, "dflt").encode() == go.get_string(p, kb, b"dflt"), k
            else:
                assert g.get_string(k, "dflt") == "dflt"
        for t, (name, shape, type_, offset) in zip(g.tensors, p.tensors):
            assert (t.name.encode(), t.shape, t.type, t.offset) == (name, shape, type_, offset)


def test_truncated_and_corrupt_files_are_refused(tmp_path):
    path, _, _, offsets, data_offset = _model_file(tmp_path)
    blob = open(path, "rb").read()
    cut = str(tmp_path / "cut.gguf")
    in_last_sized = data_offset + offsets["tiny.f16"] + 19     # one byte short of the last tensor of known size
    h = C.c_void_p()
    L = capi.lib()
    # every prefix of the header region, and a few inside the data section: refused, never read past the end
    for n in list(range(0, data_offset + 1, 3)) + [data_offset + 5, in_last_sized]:
        open(cut, "wb").write(blob[:n])
        rc = L.bpk_gguf_open(cut.encode(), C.byref(h))
        assert rc in (-8, -9), (n, rc)
        assert not h.value and L.bpk_last_error()
    open(cut, "wb").write(blob)
    assert L.bpk_gguf_open(cut.encode(), C.byref(h)) == 0
    L.bpk_gguf_close(h)

    def patched(at, fmt, v):
        b = bytearray(blob)
        struct.pack_into(fmt, b, at, v)
        open(cut, "wb").write(bytes(b))
        return L.bpk_gguf_open(cut.encode(), C.byref(h))

    assert patched(0, "<I", 0x46554746) == -9           # magic
    assert patched(4, "<I", 1) == -9 and patched(4, "<I", 4) == -9   # version
    assert patched(8, "<Q", 1 << 60) == -9             # tensor count
    assert patched(16, "<Q", 1 << 60) == -9            # kv count
    assert patched(24, "<Q", 1 << 62) == -9            # first key's length
    assert L.bpk_gguf_open(str(tmp_path / "absent.gguf").encode(), C.byref(h)) == -8
    # a tensor whose data would end past the file
    p2 = str(tmp_path / "short.gguf")
    gw.write(p2, [], [("w", (256, 4), Q4_K, b"\0" * (144 * 4 - 1))])
    assert L.bpk_gguf_open(p2.encode(), C.byref(h)) == -9
    # row length that is not whole blocks
    gw.write(p2, [], [("w", (200, 4), Q4_K, b"\0" * 576)])
    assert L.bpk_gguf_open(p2.encode(), C.byref(h)) == -9
    # five dimensions
    gw.write(p2, [], [("w", (2, 2, 2, 2, 2), 0, b"\0" * 128)])
    assert L.bpk_gguf_open(p2.encode(), C.byref(h)) == -9
    # an empty file with no tensors is fine
    gw.write(p2, [("k", gw.U32, 1)], [])
    assert L.bpk_gguf_open(p2.encode(), C.byref(h)) == 0
    L.bpk_gguf_close(h)


def test_hostile_counts_offsets_and_unsigned_arrays(tmp_path):
    """Files assembled by hand: a string array that claims more strings than the rest of the file could hold
    (refused before anything is reserved for them), a tensor of a type the reader does not know whose data
    would start past the end of the file (refused: the pointer handed out always lies inside the mapping),
    and a uint32 array with an element beyond 2^31 (the largest element, compared as unsigned)."""
    L = capi.lib()
    h = C.c_void_p()

    def s(b):
        return struct.pack("<Q", len(b)) + b
    path = str(tmp_path / "hostile.gguf")
    # 1. one key: array of strings, count = one more than eight bytes apiece would allow
    tail = b"\0" * 4096
    head = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + s(b"tok") + struct.pack("<II", 9, 8)
    count = (len(tail)) // 8 + 1
    open(path, "wb").write(head + struct.pack("<Q", count) + tail)
    assert L.bpk_gguf_open(path.encode(), C.byref(h)) == -9 and not h.value
    open(path, "wb").write(head + struct.pack("<Q", 1 << 40) + tail)
    assert L.bpk_gguf_open(path.encode(), C.byref(h)) == -9 and not h.value
    # ... while as many empty strings as do fit are read
    open(path, "wb").write(head + struct.pack("<Q", 512) + tail)
    assert L.bpk_gguf_open(path.encode(), C.byref(h)) == 0
    n, et = C.c_uint64(), C.c_uint32()
    assert L.bpk_gguf_array_len(h, b"tok", C.byref(n), C.byref(et)) == 0 and (n.value, et.value) == (512, 8)
    L.bpk_gguf_close(h)
    # 2. a tensor of an unknown type (IQ2_XXS = 16) at an offset past the end of the file
    for offset, want in ((0, 0), (64, 0), (1 << 20, -9), (1 << 62, -9)):
        blob = struct.pack("<IIQQ", 0x46554747, 3, 1, 0) + s(b"odd") + struct.pack("<IQQIQ", 2, 32, 2, 16, offset)
        blob += b"\0" * ((-len(blob)) % 32) + b"\x11" * 96
        open(path, "wb").write(blob)
        h = C.c_void_p()
        assert L.bpk_gguf_open(path.encode(), C.byref(h)) == want, offset
        if want == 0:
            t = capi.GgufTensor()
            assert L.bpk_gguf_find_tensor(h, b"odd", C.byref(t)) == 0 and t.bytes == 0 and t.offset == offset
            L.bpk_gguf_close(h)
    # 3. uint32 elements are compared as unsigned, int32 elements as signed
    kv = s(b"u") + struct.pack("<IIQ", 9, 4, 3) + struct.pack("<III", 7, 0x90000000, 12)
    kv += s(b"i") + struct.pack("<IIQ", 9, 5, 3) + struct.pack("<iii", 7, -5, 12)
    open(path, "wb").write(struct.pack("<IIQQ", 0x46554747, 3, 0, 2) + kv)
    h = C.c_void_p()
    assert L.bpk_gguf_open(path.encode(), C.byref(h)) == 0
    out = C.c_uint32()
    assert L.bpk_gguf_get_u32(h, b"u", 1, C.byref(out)) == 0 and out.value == 0x90000000
    assert L.bpk_gguf_get_u32(h, b"i", 1, C.byref(out)) == 0 and out.value == 12
    L.bpk_gguf_close(h)


def test_weight_create_argument_checks(tmp_path):
    """The checks that precede any device call (type, shape, names)."""
    path, *_ = _model_file(tmp_path)
    L = capi.lib()
    with GGUFFile(path) as g:
        w = C.c_void_p()

        def create(*names):
            arr = (C.c_char_p * len(names))(*[n.encode() for n in names])
            return L.bpk_gguf_weight_create(g.handle, arr, len(names), C.byref(w))

        assert create("output_norm.weight") == -1                                   # F32 is not a k-quant
        assert create("nope") == -10
        assert create("blk.0.ffn_gate.weight", "blk.0.attn_v.weight") == -2       # mixed type / K
        assert L.bpk_gguf_weight_create(g.handle, None, 1, C.byref(w)) == -3
        arr = (C.c_char_p * 1)(b"blk.0.ffn_gate.weight")
        assert L.bpk_gguf_weight_create(g.handle, arr, 0, C.byref(w)) == -2


# ---- model hyper-parameters (extractModelConfig, runtime/gguf_loader.cpp:184-317) --------------------
def _cfg_file(tmp_path, name, metadata, tensor_names=(), embd_dims=None):
    tensors = [(n, (4,), 0, np.zeros(4, np.float32).tobytes()) for n in tensor_names]
    if embd_dims:
        n = int(np.prod(embd_dims))
        tensors.append(("token_embd.weight", embd_dims, 0, np.zeros(n, np.float32).tobytes()))
    path = os.path.join(tmp_path, name)
    gw.write(path, metadata, tensors)
    return path


def test_model_config_llama_defaults_and_probes(tmp_path):
    """A plain Llama file: keys under 'llama.', the reference's defaults for what the file leaves out."""
    md = [("general.architecture", gw.STRING, "llama"), ("llama.block_count", gw.U32, 32),
          ("llama.embedding_length", gw.U32, 4096), ("llama.feed_forward_length", gw.U32, 14336),
          ("llama.attention.head_count", gw.U32, 32), ("llama.attention.head_count_kv", gw.U32, 8),
          ("llama.attention.layer_norm_rms_epsilon", gw.F32, 1e-5), ("llama.rope.freq_base", gw.F32, 500000.0)]
    with GGUFFile(_cfg_file(str(tmp_path), "llama.gguf", md, embd_dims=(64, 1000))) as f:
        c = f.model_config()
    assert c["arch"] == "llama"
    assert (c["n_layer"], c["n_embd"], c["intermediate_size"], c["n_head"], c["n_kv_heads"]) == (32, 4096, 14336, 32, 8)
    assert (c["head_dim"], c["kv_head_dim"]) == (128, 128)                       # n_embd / n_head
    assert c["n_vocab"] == 1000                                                  # GGUF shape is (columns, rows)
    assert c["rms_norm_eps"] == np.float32(1e-5) and c["rope_theta"] == 500000.0
    assert c["tie_word_embeddings"] == 1 and c["has_qk_norm"] == 0
    assert c["activation"] == 0 and c["embedding_scale"] == 0.0 and c["logit_softcap"] == 0.0
    assert c["sliding_window"] == 0 and c["layer_attn_types"] == []
    assert (c["num_experts"], c["num_experts_per_tok"], c["moe_intermediate_size"]) == (0, 0, 0)
    assert c["has_mtp"] == 0 and c["has_sandwich_norm"] == 0
    assert c["rope_sections"] == [11, 11, 10, 0]


def test_model_config_missing_architecture_and_fallbacks(tmp_path):
    """No architecture key: 'llama'; kv heads default to heads, eps 1e-6, theta 1e6; a 1-D embedding."""
    md = [("llama.block_count", gw.U32, 2), ("llama.embedding_length", gw.U32, 512),
          ("llama.attention.head_count", gw.U32, 8), ("output.weight", gw.BOOL, 1)]
    path = os.path.join(str(tmp_path), "bare.gguf")
    gw.write(path, md, [("token_embd.weight", (77,), 0, np.zeros(77, np.float32).tobytes())])
    with GGUFFile(path) as f:
        c = f.model_config()
    assert c["arch"] == "llama" and c["n_kv_heads"] == 8 and c["head_dim"] == 64
    assert c["rms_norm_eps"] == np.float32(1e-6) and c["rope_theta"] == 1000000.0
    assert c["n_vocab"] == 77
    assert c["tie_word_embeddings"] == 0          # the reference asks for a metadata key of that name


def test_model_config_qwen3_moe_with_hybrid_probes(tmp_path):
    md = [("general.architecture", gw.STRING, "qwen35moe"), ("qwen35moe.block_count", gw.U32, 6),
          ("qwen35moe.embedding_length", gw.U32, 2048), ("qwen35moe.feed_forward_length", gw.U32, 6144),
          ("qwen35moe.attention.head_count", gw.U32, 32), ("qwen35moe.attention.head_count_kv", gw.U32, 4),
          ("qwen35moe.attention.key_length", gw.U32, 256),
          ("qwen35moe.expert_count", gw.U32, 128), ("qwen35moe.expert_used_count", gw.U32, 8),
          ("qwen35moe.expert_feed_forward_length", gw.U32, 768),
          ("qwen35moe.ssm.inner_size", gw.U32, 4096), ("qwen35moe.ssm.state_size", gw.U32, 128),
          ("qwen35moe.ssm.conv_kernel", gw.U32, 4), ("qwen35moe.ssm.group_count", gw.U32, 16),
          ("qwen35moe.ssm.time_step_rank", gw.U32, 32), ("qwen35moe.full_attention_interval", gw.U32, 4),
          ("qwen35moe.nextn_predict_layers", gw.U32, 1),
          ("qwen35moe.rope.dimension_sections", gw.ARRAY, (gw.I32, [24, 20, 20, 0, 9]))]
    # QK norm only on the attention layers of a hybrid: layer 3, not layer 0
    with GGUFFile(_cfg_file(str(tmp_path), "moe.gguf", md, ["blk.3.attn_q_norm.weight"], embd_dims=(2048, 300))) as f:
        c = f.model_config()
    assert c["arch"] == "qwen35moe"
    assert (c["head_dim"], c["kv_head_dim"]) == (256, 256)                        # key_length, not n_embd / n_head = 64
    assert c["has_qk_norm"] == 1
    assert (c["num_experts"], c["num_experts_per_tok"], c["moe_intermediate_size"]) == (128, 8, 768)
    assert c["moe_shared_intermediate_size"] == 768                              # defaults to the routed size
    assert (c["ssm_inner_size"], c["ssm_state_size"], c["ssm_conv_kernel"], c["ssm_group_count"],
            c["ssm_time_step_rank"], c["full_attention_interval"]) == (4096, 128, 4, 16, 32, 4)
    assert c["has_mtp"] == 1 and c["mtp_num_layers"] == 1
    assert c["rope_sections"] == [24, 20, 20, 0]
    assert c["n_vocab"] == 300


@pytest.mark.parametrize("arch,expect", [
    ("gemma2", [1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0]),            # even layers slide
    ("gemma3", [1, 1, 1, 1, 1, 0, 1, 1, 1, 1, 1, 0]),            # five sliding, one global
    ("gemma4", [1, 1, 1, 1, 1, 0, 1, 1, 1, 1, 1, 0]),            # no pattern in the file: the same default
    ("gemma", [0] * 12),                                         # a window but no pattern rule: all global
])
def test_model_config_gemma_family(tmp_path, arch, expect):
    md = [("general.architecture", gw.STRING, arch), (f"{arch}.block_count", gw.U32, 12),
          (f"{arch}.embedding_length", gw.U32, 2304), (f"{arch}.attention.head_count", gw.U32, 8),
          (f"{arch}.attention.sliding_window", gw.U32, 4096), (f"{arch}.final_logit_softcapping", gw.F32, 30.0),
          # per-layer feed-forward lengths: the largest sizes the buffers
          (f"{arch}.feed_forward_length", gw.ARRAY, (gw.I32, [6144, 12288, 1228])),
          (f"{arch}.attention.shared_kv_layers", gw.U32, 3), (f"{arch}.embedding_length_per_layer_input", gw.U32, 256)]
    with GGUFFile(_cfg_file(str(tmp_path), "g.gguf", md, ["blk.0.post_attention_norm.weight", "mtp.0.enorm.weight"])) as f:
        c = f.model_config()
    assert c["activation"] == 1 and c["embedding_scale"] == np.float32(np.sqrt(np.float32(2304)))
    assert c["logit_softcap"] == 30.0 and c["sliding_window"] == 4096
    assert c["intermediate_size"] == 12288
    assert c["layer_attn_types"] == expect
    assert c["has_sandwich_norm"] == 1 and c["has_mtp"] == 1 and c["mtp_num_layers"] == 0
    assert (c["shared_kv_layers"], c["ple_size"]) == (3, 256)
    assert c["n_vocab"] == 0                                     # no embedding tensor in the file


def test_model_config_gemma4_pattern_from_the_file(tmp_path):
    pat = [1, 1, 0, 1, 0, 0]
    md = [("general.architecture", gw.STRING, "gemma4"), ("gemma4.block_count", gw.U32, 6),
          ("gemma4.embedding_length", gw.U32, 1024), ("gemma4.attention.head_count", gw.U32, 4),
          ("gemma4.attention.sliding_window", gw.U32, 512),
          ("gemma4.attention.sliding_window_pattern", gw.ARRAY, (gw.BOOL, pat))]
    with GGUFFile(_cfg_file(str(tmp_path), "g4.gguf", md)) as f:
        assert f.model_config()["layer_attn_types"] == pat
    # a pattern of the wrong length is ignored
    md[-1] = ("gemma4.attention.sliding_window_pattern", gw.ARRAY, (gw.BOOL, pat[:4]))
    with GGUFFile(_cfg_file(str(tmp_path), "g4b.gguf", md)) as f:
        c = f.model_config()
    assert c["layer_attn_types"] == [1, 1, 1, 1, 1, 0]
    # the buffer for the per-layer kinds must hold every layer
    with GGUFFile(_cfg_file(str(tmp_path), "g4c.gguf", md)) as f:
        out = capi.ModelConfig()
        small = (C.c_uint8 * 2)()
        assert capi.lib().bpk_gguf_model_config(f.handle, C.byref(out), small, 2) == -2
        assert capi.lib().bpk_gguf_model_config(None, C.byref(out), None, 0) == -3


_CFG_U = ["n_layer", "n_head", "n_kv_heads", "n_embd", "intermediate_size", "n_vocab", "head_dim", "kv_head_dim",
          "tie_word_embeddings", "has_qk_norm", "activation", "sliding_window", "n_layer_attn_types", "has_sandwich_norm",
          "ple_size", "shared_kv_layers", "has_mtp", "mtp_num_layers", "num_experts", "num_experts_per_tok",
          "moe_intermediate_size", "moe_shared_intermediate_size", "ssm_inner_size", "ssm_state_size", "ssm_conv_kernel",
          "ssm_group_count", "ssm_time_step_rank", "full_attention_interval"]
_CFG_F = ["rms_norm_eps", "rope_theta", "embedding_scale", "logit_softcap"]


def test_model_config_against_the_compiled_reference(tmp_path, kqref):
    """Every field, on files of each architecture family, against extractModelConfig itself
    (runtime/gguf_loader.cpp:184-317, compiled from the reference's sources into oracle/_ref)."""
    r = kqref.ref()
    r.bpref_gguf_open.restype = C.c_void_p
    r.bpref_gguf_open.argtypes = [C.c_char_p]
    r.bpref_model_config.restype = C.c_uint32
    r.bpref_model_config.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_char_p,
                                     C.c_size_t]
    rng = np.random.default_rng(11)
    files = []
    for i, arch in enumerate(["llama", "qwen3", "qwen35moe", "gemma", "gemma2", "gemma3", "gemma4", "gemma4", "mixtral", None]):
        a = arch or "llama"
        n_layer = int(rng.integers(2, 20))
        md = [] if arch is None else [("general.architecture", gw.STRING, arch)]
        md += [(f"{a}.block_count", gw.U32, n_layer), (f"{a}.embedding_length", gw.U32, int(rng.integers(1, 64)) * 64),
               (f"{a}.attention.head_count", gw.U32, int(rng.choice([0, 4, 8, 16])))]
        opt = [(f"{a}.feed_forward_length", gw.ARRAY, (gw.I32, [int(x) for x in rng.integers(100, 9000, 3)])),
               (f"{a}.attention.head_count_kv", gw.U32, 2), (f"{a}.attention.key_length", gw.U32, 256),
               (f"{a}.attention.layer_norm_rms_epsilon", gw.F64, 1e-5), (f"{a}.rope.freq_base", gw.F32, 10000.0),
               (f"{a}.final_logit_softcapping", gw.F32, 30.0), (f"{a}.attention.sliding_window", gw.U32, 1024),
               (f"{a}.attention.shared_kv_layers", gw.U32, 2), (f"{a}.embedding_length_per_layer_input", gw.U16, 128),
               (f"{a}.nextn_predict_layers", gw.U32, 2), (f"{a}.expert_count", gw.U32, 64),
               (f"{a}.expert_used_count", gw.U8, 6), (f"{a}.expert_feed_forward_length", gw.U32, 512),
               (f"{a}.expert_shared_feed_forward_length", gw.U32, 1024), (f"{a}.ssm.inner_size", gw.U32, 2048),
               (f"{a}.ssm.state_size", gw.U32, 64), (f"{a}.ssm.conv_kernel", gw.U32, 4), (f"{a}.ssm.group_count", gw.U32, 8),
               (f"{a}.ssm.time_step_rank", gw.U32, 16), (f"{a}.full_attention_interval", gw.U32, 4),
               (f"{a}.rope.dimension_sections", gw.ARRAY, (gw.I32, [16, 24, 24, 0])), ("output.weight", gw.U32, 1),
               (f"{a}.attention.sliding_window_pattern", gw.ARRAY, (gw.BOOL, [int(x) for x in rng.integers(0, 2, n_layer)]))]
        md += [o for o in opt if rng.random() < (0.6 if i != 7 else 1.0)]
        names = [n for n in ["blk.0.attn_q_norm.weight", f"blk.{n_layer - 1}.attn_q_norm.weight", "blk.0.post_norm.weight",
                             "blk.0.attn_post_norm.weight", "mtp.0.blk.0.attn_q.weight", "mtp.0.enorm.weight"]
                 if rng.random() < 0.4]
        files.append(_cfg_file(str(tmp_path), f"c{i}.gguf", md, names, embd_dims=(32, 50 + i) if i % 3 else None))
    for path in files:
        with GGUFFile(path) as f:
            mine = f.model_config()
        h = C.c_void_p(r.bpref_gguf_open(path.encode()))
        assert h.value
        u, fl, sec = (C.c_uint32 * 28)(), (C.c_float * 4)(), (C.c_int32 * 4)()
        types, arch = (C.c_uint8 * 64)(), C.create_string_buffer(64)
        n_types = r.bpref_model_config(h, u, fl, sec, types, 64, arch, 64)
        r.bpref_gguf_close(h)
        assert mine["arch"] == arch.value.decode()
        assert [mine[k] for k in _CFG_U] == list(u), path
        assert [np.float32(mine[k]) for k in _CFG_F] == [np.float32(x) for x in fl], path
        assert mine["rope_sections"] == list(sec)
        assert mine["layer_attn_types"] == list(types)[:n_types]
