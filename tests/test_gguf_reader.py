"""GGUF container reader of the library (host code, no device) against the plain-Python checker, the reference's
own reader tests and a byte string assembled by hand from the published layout."""
import struct

import numpy as np
import pytest

from kalosm_amd import _lib
from kalosm_amd.gguf import GgufMetadata, VarBuilder
from kalosm_amd._lib import FusorHipError
from oracle import gguf_ref as R


def status_of(data: bytes) -> int:
    with pytest.raises(FusorHipError) as e:
        GgufMetadata.read_bytes(data)
    return e.value.status


# One key/value (general.alignment = u32 64), one string value with trailing NULs, one 2-D Q8_0 tensor and one
# 1-D f32 tensor; every field written out by hand.
HAND = b"".join([
    b"GGUF", b"\x03\x00\x00\x00",                      # magic, version 3
    b"\x02\x00\x00\x00\x00\x00\x00\x00",              # 2 tensors
    b"\x03\x00\x00\x00\x00\x00\x00\x00",              # 3 key/values
    b"\x11\x00\x00\x00\x00\x00\x00\x00", b"general.alignment", b"\x04\x00\x00\x00", b"\x40\x00\x00\x00",
    b"\x04\x00\x00\x00\x00\x00\x00\x00", b"name", b"\x08\x00\x00\x00",
    b"\x05\x00\x00\x00\x00\x00\x00\x00", b"abc\x00\x00",
    b"\x04\x00\x00\x00\x00\x00\x00\x00", b"nums", b"\x09\x00\x00\x00", b"\x03\x00\x00\x00",   # array of i16
    b"\x03\x00\x00\x00\x00\x00\x00\x00", b"\xff\xff", b"\x02\x00", b"\x00\x80",              # -1, 2, -32768
    b"\x01\x00\x00\x00\x00\x00\x00\x00", b"w", b"\x02\x00\x00\x00",                          # tensor "w", 2 dims
    b"\x40\x00\x00\x00\x00\x00\x00\x00", b"\x03\x00\x00\x00\x00\x00\x00\x00",                # innermost 64, then 3
    b"\x08\x00\x00\x00", b"\x00\x00\x00\x00\x00\x00\x00\x00",                                # Q8_0, offset 0
    b"\x01\x00\x00\x00\x00\x00\x00\x00", b"b", b"\x01\x00\x00\x00",                          # tensor "b", 1 dim
    b"\x02\x00\x00\x00\x00\x00\x00\x00", b"\x00\x00\x00\x00", b"\x00\x01\x00\x00\x00\x00\x00\x00",  # 2 x f32 at 256
])
HAND_HEADER = len(HAND)                                    # 194 bytes -> payload starts at 256
HAND += b"\0" * (256 - HAND_HEADER) + bytes(range(204)) + b"\0" * 52 + struct.pack("<2f", 1.5, -2.0)


def test_hand_assembled_file():
    assert HAND_HEADER == 194
    for g in (GgufMetadata.read_bytes(HAND),):
        assert (g.version, g.alignment, g.tensor_data_offset) == (3, 64, 256)
        assert g.keys() == ["general.alignment", "name", "nums"]
        assert g.get_value("general.alignment") == 64
        assert g.get_value("name") == "abc"                                  # trailing NULs dropped
        assert g.get_value("nums").tolist() == [-1, 2, -32768]
        assert g.get_value("absent") is None
        infos = g.tensor_infos
        assert list(infos) == ["w", "b"]
        assert (infos["w"].ty, infos["w"].shape, infos["w"].offset) == (8, (3, 64), 0)   # dims reversed
        assert (infos["b"].ty, infos["b"].shape, infos["b"].offset) == (0, (2,), 256)
        assert g.read_tensor_bytes("w").tobytes() == bytes(range(204))       # 3 x 64 / 32 blocks of 34 bytes
        assert g.read_tensor_bytes("b").view(np.float32).tolist() == [1.5, -2.0]
    r = R.GgufRef(HAND)
    assert (r.version, r.alignment, r.data_offset) == (3, 64, 256)
    assert r.metadata[b"name"] == (R.STRING, b"abc") and r.metadata[b"nums"] == (R.ARRAY, [-1, 2, -32768])
    assert r.tensors == {b"w": (8, (3, 64), 0), b"b": (0, (2,), 256)}
    assert r.tensor_bytes(b"w").tobytes() == bytes(range(204))


def test_reference_round_trip_empty():
    """fusor-ml/gguf/src/lib.rs:2509-2536: an empty version-3 file; the payload offset reads back as 32."""
    data = R.write_gguf({}, [], version=3)
    assert data == b"GGUF" + struct.pack("<IQQ", 3, 0, 0) and len(data) == 24
    g = GgufMetadata.read_bytes(data)
    assert (g.tensor_data_offset, len(g.tensor_infos), g.version, g.keys()) == (32, 0, 3, [])
    assert R.GgufRef(data).data_offset == 32


@pytest.mark.parametrize("version", [1, 2, 3])
def test_reference_version_round_trip(version):
    """fusor-ml/gguf/src/lib.rs:144-155, and the 32-bit counts of version 1 (:201-209)."""
    data = R.write_gguf({}, [], version=version)
    assert len(data) == (16 if version == 1 else 24)
    assert GgufMetadata.read_bytes(data).version == version
    assert GgufMetadata.read_bytes(b"FUGG" + data[4:]).version == version   # reversed magic is accepted (:16-31)


def random_file(seed: int, version: int, alignment):
    rng = np.random.default_rng(seed)
    T = R.Typed
    md = {
        "general.architecture": "llama",
        "llama.attention.head_count": T(R.U32, 32),
        "x.llama.attention.head_count": T(R.U32, 99),
        "some.u8": T(R.U8, 200), "some.i8": T(R.I8, -100), "some.u16": T(R.U16, 60000), "some.i16": T(R.I16, -30000),
        "some.i32": T(R.I32, -2 ** 31), "some.u64": T(R.U64, 2 ** 64 - 1), "some.i64": T(R.I64, -2 ** 63),
        "some.f32": T(R.F32, 1e-5), "some.f64": T(R.F64, 0.1), "some.true": True, "some.false": False,
        "tokenizer.ggml.tokens": ["<s>", "", "café", "tail\0\0", "x" * 300],
        "floats": T(R.ARRAY, [float(np.float32(v)) for v in rng.normal(size=7)], R.F32),
        "bools": [True, False, True],
        "nested": T(R.ARRAY, [T(R.ARRAY, [1, 2], R.U8), T(R.ARRAY, [3], R.U8)], R.ARRAY),
        "after.nested": T(R.I64, -5),
    }
    tensors = []
    for i, (ty, shape) in enumerate([(12, (4, 512)), (14, (2, 256)), (0, (16,)), (1, (3, 5)), (2, (8, 64)), (8, (1, 32)),
                                     (6, (2, 64)), (13, (1, 256)), (0, (2, 3, 4))]):
        be, bb = R.BLOCK[ty]
        n = int(np.prod(shape)) // be * bb
        tensors.append((f"t{i}.weight", ty, shape, rng.integers(0, 256, n, dtype=np.uint8)))
    return md, tensors, R.write_gguf(md, tensors, version=version, alignment=alignment)


@pytest.mark.parametrize("version,alignment", [(3, None), (2, 64), (1, None), (3, 4096), (3, 1)])
def test_reader_matches_checker_on_random_files(version, alignment, tmp_path):
    md, tensors, data = random_file(7 + version, version, alignment)
    path = tmp_path / "m.gguf"
    path.write_bytes(data)
    r = R.GgufRef(data)
    for g in (GgufMetadata.read_bytes(data), GgufMetadata.read(str(path))):
        assert (g.version, g.alignment, g.tensor_data_offset) == (r.version, r.alignment, r.data_offset)
        assert g.alignment == (alignment or 32) and g.tensor_data_offset % g.alignment == 0
        assert [k.encode() for k in g.keys()] == list(r.metadata)
        for key, (t, v) in r.metadata.items():
            k = key.decode()
            if k == "nested":
                with pytest.raises(FusorHipError):
                    g.get_value(k)
                continue
            got = g.get_value(k)
            if t == R.STRING:
                assert got.encode() == v
            elif t == R.ARRAY and v and isinstance(v[0], bytes):
                assert [s.encode() for s in got] == v
            elif t == R.ARRAY:
                assert np.array_equal(np.asarray(got), np.asarray(v, dtype=np.asarray(got).dtype))
            elif t == R.F32:
                assert np.float32(got) == np.float32(v)
            else:
                assert got == v and type(got) is type(v)
        assert g.get_value("tokenizer.ggml.tokens")[3] == "tail"
        # suffix lookup: the shortest key that ends with the suffix (gguf/src/lib.rs:301-311)
        assert g.get_value(".attention.head_count") == 32
        assert g.get_value(".no.such.suffix") is None
        assert g.architecture() == "llama"
        assert {k.encode(): (m.ty, m.shape, m.offset) for k, m in g.tensor_infos.items()} == r.tensors
        for name, ty, shape, raw in tensors:
            assert np.array_equal(g.read_tensor_bytes(name), raw)
            assert np.array_equal(r.tensor_bytes(name.encode()), raw)
        vb = VarBuilder(g)
        assert vb.pp("t0").contains_key("weight") and not vb.pp("t0").contains_key("bias")
        assert sorted(vb.list_all_keys()) == sorted(n for n, *_ in tensors)
        g.close()


def test_alignment_value_types():
    """gguf/src/lib.rs:597-606: u8/u16/u32 and non-negative i8/i16/i32 are honoured, anything else means 32."""
    T = R.Typed
    for val, want in [(T(R.U8, 16), 16), (T(R.U16, 128), 128), (T(R.I8, 8), 8), (T(R.I16, 256), 256), (T(R.I32, 64), 64),
                      (T(R.I32, -64), 32), (T(R.U64, 64), 32), (T(R.I64, 64), 32), (T(R.F32, 64.0), 32), ("64", 32)]:
        data = R.write_gguf({"general.alignment": val}, [("a", 0, (1,), np.zeros(4, np.uint8))])
        g = GgufMetadata.read_bytes(data)
        assert g.alignment == want == R.GgufRef(data).alignment
        assert g.tensor_data_offset == R.GgufRef(data).data_offset and g.tensor_data_offset % want == 0


def test_duplicate_keys_keep_the_last_value():
    """The reference inserts into a map (gguf/src/lib.rs:566-572): a repeated key is overwritten."""
    one = R.write_gguf({"k": R.Typed(R.U32, 1)}, [])
    kv = one[24:]
    data = b"GGUF" + struct.pack("<IQQ", 3, 0, 2) + kv + kv[:-4] + struct.pack("<I", 2)
    g = GgufMetadata.read_bytes(data)
    assert g.keys() == ["k"] and g.get_value("k") == 2 == R.GgufRef(data).metadata[b"k"][1]


def test_value_conversions():
    """to_u32 & co accept every integer type, to_f32 only floats (gguf/src/lib.rs:544-556)."""
    import ctypes as C
    T = R.Typed
    data = R.write_gguf({"i": T(R.I8, -3), "f": T(R.F64, 2.5), "s": "x", "b": True, "a": [1, 2]}, [])
    g = GgufMetadata.read_bytes(data)
    L = _lib.load()
    v, d = C.c_int64(), C.c_double()
    assert L.fh_gguf_meta_int(g._h, b"i", C.byref(v)) == 0 and v.value == -3
    assert L.fh_gguf_meta_float(g._h, b"f", C.byref(d)) == 0 and d.value == 2.5
    assert L.fh_gguf_meta_int(g._h, b"f", C.byref(v)) == _lib.FH_ERR_INVALID
    assert L.fh_gguf_meta_float(g._h, b"i", C.byref(d)) == _lib.FH_ERR_INVALID
    assert L.fh_gguf_meta_int(g._h, b"s", C.byref(v)) == _lib.FH_ERR_INVALID
    assert L.fh_gguf_meta_int(g._h, b"b", C.byref(v)) == _lib.FH_ERR_INVALID
    assert L.fh_gguf_meta_int(g._h, b"zz", C.byref(v)) == _lib.FH_ERR_NOT_FOUND
    assert L.fh_gguf_meta_array_int(g._h, b"a", 1, C.byref(v)) == 0 and v.value == 2
    assert L.fh_gguf_meta_array_int(g._h, b"a", 2, C.byref(v)) == _lib.FH_ERR_INVALID
    assert b"not found" in L.fh_last_error() or b"out of range" in L.fh_last_error()


def test_errors():
    """GgufReadError variants (gguf/src/lib.rs:222-241) as status codes."""
    md, tensors, good = random_file(3, 3, None)
    assert status_of(b"GGML" + good[4:]) == _lib.FH_ERR_INVALID                       # MagicBytesMismatch
    assert status_of(good[:4] + struct.pack("<I", 4) + good[8:]) == _lib.FH_ERR_UNSUPPORTED   # UnsupportedVersion
    assert status_of(good[:4] + struct.pack("<I", 0) + good[8:]) == _lib.FH_ERR_UNSUPPORTED
    for cut in (0, 3, 7, 20, 40, 200, 700):                                          # Io: unexpected end of file
        assert status_of(good[:cut]) == _lib.FH_ERR_IO
        with pytest.raises(R.GgufError):
            R.GgufRef(good[:cut])
    bad_bool = R.write_gguf({"b": True}, [])
    assert status_of(bad_bool[:-1] + b"\x02") == _lib.FH_ERR_INVALID                  # InvalidBool
    bad_type = R.write_gguf({"b": R.Typed(R.U32, 1)}, [])
    assert status_of(bad_type[:-8] + struct.pack("<II", 13, 1)) == _lib.FH_ERR_INVALID   # InvalidValueType
    for ty in (4, 5, 16, 30):                                                        # UnsupportedDType (e.g. bf16 = 30)
        data = bytearray(R.write_gguf({}, [("a", 0, (1,), np.zeros(4, np.uint8))]))
        data[24 + 8 + 1 + 4 + 8:24 + 8 + 1 + 4 + 8 + 4] = struct.pack("<I", ty)
        assert status_of(bytes(data)) == _lib.FH_ERR_UNSUPPORTED
        with pytest.raises(R.GgufError):
            R.GgufRef(bytes(data))
    # known type ids without a block layout in the reference (its block_allocation_size is a todo!()): the
    # directory parses, asking for the bytes is refused
    g = GgufMetadata.read_bytes(R.write_gguf({}, [("a", 3, (32,), np.zeros(20, np.uint8))]))
    assert g.tensor_infos["a"].ty == 3
    with pytest.raises(FusorHipError) as e:
        g.read_tensor_bytes("a")
    assert e.value.status == _lib.FH_ERR_UNSUPPORTED
    # InvalidTensorSize: 48 elements of a 32-element block type
    g = GgufMetadata.read_bytes(R.write_gguf({}, [("a", 2, (48,), np.zeros(36, np.uint8))]))
    with pytest.raises(FusorHipError) as e:
        g.read_tensor_bytes("a")
    assert e.value.status == _lib.FH_ERR_INVALID and "multiple of the block size" in str(e.value)
    # payload beyond the end of the file
    whole = R.write_gguf({}, [("a", 0, (64,), np.zeros(256, np.uint8))])
    g = GgufMetadata.read_bytes(whole[:-1])
    with pytest.raises(FusorHipError) as e:
        g.read_tensor_bytes("a")
    assert e.value.status == _lib.FH_ERR_IO
    with pytest.raises(FusorHipError) as e:
        g.read_tensor_bytes("nope")
    assert e.value.status == _lib.FH_ERR_NOT_FOUND
    with pytest.raises(FusorHipError) as e:
        GgufMetadata.read("/nonexistent/file.gguf")
    assert e.value.status == _lib.FH_ERR_IO


def llama_file(cfg, seed=0, arch="llama", extra_md=None, extra_tensors=(), rope_freqs=True, mixed=True, five_bit=False):
    """A small random-init decoder file in the tensor naming of models/kalosm-llama/src/raw/mod.rs:473-604."""
    from kalosm_amd import synth
    rng = np.random.default_rng(seed)
    D, F, V = cfg["d_model"], cfg["ffn"], cfg["vocab"]
    QD, KD = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    tensors, weights, types = [], {}, {}

    def q(name, ty, n, k, s):
        raw = synth.random_weight(ty, n, k, seed=s, sigma=4e-4)
        tensors.append((name, ty, (n, k), raw))
        weights[name], types[name] = raw, ty

    def f(name, n, f16=False):
        v = (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)
        if f16:
            h = v.astype(np.float16)
            tensors.append((name, 1, (n,), h.view(np.uint8)))
            weights[name] = h.astype(np.float32)
        else:
            tensors.append((name, 0, (n,), v.view(np.uint8)))
            weights[name] = v

    if five_bit:  # the 5-bit formats and dense f16 rows, as Q5_K_M / Q5_0 files and f16 output heads hold them
        t_embd, t_o, t_down, t_out = 6, 13, 6, 1
    else:
        t_embd, t_o, t_down, t_out = 12, 12, None, 14
    q("token_embd.weight", t_embd, V, D, 1)
    for l in range(cfg["n_layers"]):
        p = f"blk.{l}."
        f(p + "attn_norm.weight", D)
        q(p + "attn_q.weight", 12, QD, D, 10 * l + 2)
        q(p + "attn_k.weight", 12, KD, D, 10 * l + 3)
        q(p + "attn_v.weight", 14 if mixed and l % 2 == 0 else 12, KD, D, 10 * l + 4)   # as Q4_K_M files do
        q(p + "attn_output.weight", t_o, D, QD, 10 * l + 5)
        f(p + "ffn_norm.weight", D, f16=(l == 1))
        q(p + "ffn_gate.weight", 12, F, D, 10 * l + 6)
        q(p + "ffn_up.weight", 8 if mixed and l == 1 else 12, F, D, 10 * l + 7)
        q(p + "ffn_down.weight", t_down or (14 if l % 2 == 0 else 12), D, F, 10 * l + 8)
    f("output_norm.weight", D)
    q("output.weight", t_out, V, D, 9)
    if rope_freqs:
        w = np.linspace(1.0, 0.125, cfg["head_dim"] // 2).astype(np.float32)
        tensors.append(("rope_freqs.weight", 0, (cfg["head_dim"] // 2,), w.view(np.uint8)))
        weights["rope_freqs.weight"] = w
    tensors.extend(extra_tensors)
    T = R.Typed
    md = {
        "general.architecture": arch, "general.name": "tiny random decoder",
        f"{arch}.attention.head_count": T(R.U32, cfg["n_heads"]),
        f"{arch}.attention.head_count_kv": T(R.U64, cfg["n_kv_heads"]),     # any integer type converts (:544-551)
        f"{arch}.block_count": T(R.I32, cfg["n_layers"]),
        f"{arch}.embedding_length": T(R.U32, D),
        f"{arch}.feed_forward_length": T(R.U32, F),
        f"{arch}.context_length": T(R.U32, cfg["ctx"]),
        f"{arch}.attention.layer_norm_rms_epsilon": T(R.F32, cfg["eps"]),
        f"{arch}.rope.freq_base": T(R.F32, cfg["theta"]),
        "tokenizer.ggml.tokens": [f"t{i}" for i in range(V)],
        "tokenizer.ggml.eos_token_id": T(R.U32, 2),
    }
    md.update(extra_md or {})
    return R.write_gguf(md, tensors), weights, types


TINY = dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, head_dim=64, ffn=512, vocab=320, ctx=96, eps=1e-5,
            theta=500000.0)


def test_decoder_config_from_metadata():
    """Parameter extraction of models/kalosm-llama/src/raw/mod.rs:377-416 (no device needed)."""
    import ctypes as C
    L = _lib.load()
    data, _, _ = llama_file(TINY)
    g = GgufMetadata.read_bytes(data)
    c = _lib.LlamaConfig()
    assert L.fh_llama_config_from_gguf(g._h, C.byref(c)) == 0, L.fh_last_error()
    got = {n: getattr(c, n) for n in TINY}
    assert got == {**TINY, "eps": np.float32(1e-5), "theta": 500000.0}
    assert (c.kv_dtype, c.fuse_qkv, c.fuse_gate_up, c.use_graph) == (0, 1, 1, 1)
    # head_dim from attention.key_length when present, rope base defaults to 1e6 (raw/mod.rs:104, :385-416)
    data, _, _ = llama_file(TINY, extra_md={"llama.attention.key_length": R.Typed(R.U32, 128),
                                            "llama.rope.freq_base": "oops"})
    g = GgufMetadata.read_bytes(data)
    assert L.fh_llama_config_from_gguf(g._h, C.byref(c)) == 0
    assert c.head_dim == 128 and c.theta == 1000000.0
    # other architectures and sliding windows are refused, missing keys are reported by name
    g = GgufMetadata.read_bytes(llama_file(TINY, arch="qwen2")[0])
    assert L.fh_llama_config_from_gguf(g._h, C.byref(c)) == _lib.FH_ERR_UNSUPPORTED
    g = GgufMetadata.read_bytes(llama_file(TINY, extra_md={"llama.attention.sliding_window": 64})[0])
    assert L.fh_llama_config_from_gguf(g._h, C.byref(c)) == _lib.FH_ERR_UNSUPPORTED
    g = GgufMetadata.read_bytes(R.write_gguf({"general.architecture": "llama"}, []))
    assert L.fh_llama_config_from_gguf(g._h, C.byref(c)) == _lib.FH_ERR_NOT_FOUND
    assert b".attention.head_count" in L.fh_last_error()


def test_corrupted_files_are_rejected_like_the_checker_does():
    """Random byte damage and truncation of a valid file: the library must answer with a status (never crash), and
    accept or reject exactly the inputs the plain-Python reader accepts or rejects."""
    rng = np.random.default_rng(0)
    _, _, good = random_file(3, 3, None)
    accepted = 0
    for it in range(600):
        data = bytearray(good)
        mode = it % 3
        if mode == 0:
            for _ in range(int(rng.integers(1, 4))):
                data[int(rng.integers(0, 1400))] = int(rng.integers(0, 256))
        elif mode == 1:
            data = data[:int(rng.integers(0, len(data)))]
        else:
            p = int(rng.integers(0, 1400))
            data[p:p + 8] = rng.integers(0, 256, 8, dtype=np.uint8).tobytes()
        data = bytes(data)
        try:
            g = GgufMetadata.read_bytes(data)
            for k in g.keys():
                try:
                    g.get_value(k)
                except FusorHipError:
                    pass
            for name in g.tensor_infos:
                try:
                    g.read_tensor_bytes(name)
                except FusorHipError:
                    pass
            lib_ok = True
        except FusorHipError:
            lib_ok = False
        try:
            R.GgufRef(data)
            ref_ok = True
        except Exception:
            ref_ok = False
        assert lib_ok == ref_ok, (it, mode)
        accepted += lib_ok
    assert 100 < accepted < 500
