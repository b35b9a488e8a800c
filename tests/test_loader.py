"""The loader side on the CPU: the memory-mapped safetensors reader against files written by the `safetensors`
package and against the cases the reference's reader is tested with (tests/unit/safetensors_test.cpp:47-234:
the round trip fixture, header lengths outside the file, numbers with leading zeros, invalid data_offsets and
shapes, byte-count mismatches and overflows, scalar / empty tensors, dtype aliases with a padded header), and
the matrix views' contracts (src/models/quant_matrix.hpp:55-96, :144-164)."""
import ctypes as C
import json
import os
import struct

import numpy as np
import pytest

from dgpp_amd import _lib, loader as LD


def write_raw(path, header: str, payload: bytes = b"", length=None):
    h = header.encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h) if length is None else length))
        f.write(h)
        f.write(payload)
    return str(path)


def tensor_header(shape: str, offsets: str, dtype: str = "U8") -> str:
    return '{"x":{"dtype":"%s","shape":%s,"data_offsets":%s}}' % (dtype, shape, offsets)


def expect_rejected(tmp_path, header, payload_bytes, diagnostic, length=None):
    p = write_raw(tmp_path / "bad.safetensors", header, bytes(i % 251 for i in range(payload_bytes)), length)
    with pytest.raises(LD.LoaderError) as e:
        LD.SafetensorsFile(p)
    assert diagnostic in str(e.value), str(e.value)


def test_reference_fixture_round_trip(tmp_path):
    header = ('{"a_f32":{"dtype":"F32","shape":[2,3],"data_offsets":[0,24]},'
              '"b_bf16":{"dtype":"BF16","shape":[4],"data_offsets":[24,32]},'
              '"c_fp8":{"dtype":"F8_E4M3","shape":[2,2],"data_offsets":[32,36]}}')
    f32 = np.array([1.0, -2.5, 3.25, 4.0, -5.0, 0.125], np.float32)
    bf16 = (np.array([0.0, 0.5, 1.0, 1.5], np.float32).view(np.uint32) >> 16).astype(np.uint16)
    fp8 = np.array([0x38, 0x40, 0x7E, 0x00], np.uint8)
    p = write_raw(tmp_path / "fixture.safetensors", header, f32.tobytes() + bf16.tobytes() + fp8.tobytes())
    with LD.SafetensorsFile(p) as f:
        assert len(f) == 3 and f.names() == ["a_f32", "b_bf16", "c_fp8"]
        a = f.find("a_f32")
        assert (a.dtype, a.dims(), a.numel, a.nbytes) == (LD.DT_F32, (2, 3), 6, 24)
        assert a.file_offset == 8 + len(header)
        assert np.array_equal(f.array("a_f32"), f32.reshape(2, 3))
        assert np.array_equal(f.array("b_bf16"), bf16)
        assert np.array_equal(f.array("c_fp8"), fp8.reshape(2, 2))
        assert "missing" not in f
        with pytest.raises(ValueError):
            f.find("missing")
        fold = 1469598103934665603
        for c in header.encode():
            fold = ((fold ^ c) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
        assert f.header_fold() == fold
        assert f.metadata_json() == ""
        f.prefetch(a)
        f.discard(a)
        assert np.array_equal(f.array("a_f32"), f32.reshape(2, 3)), "discarded pages are read again from the file"


def test_files_written_by_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.numpy")
    rng = np.random.default_rng(5)
    tensors = {
        "model.layers.0.mlp.experts.3.gate_proj.weight": rng.integers(0, 256, (64, 48), dtype=np.uint8),
        "model.layers.0.mlp.experts.3.gate_proj.weight_scale": rng.random((1, 1), dtype=np.float32),
        "ids": rng.integers(-5, 5, (7,), dtype=np.int64),
        "half": rng.random((3, 5)).astype(np.float16),
        "i32": rng.integers(-9, 9, (2, 2, 2), dtype=np.int32),
        "i8": rng.integers(-9, 9, (5,), dtype=np.int8),
        "scalar": np.array(3.5, dtype=np.float32),
    }
    path = str(tmp_path / "pkg.safetensors")
    st.save_file(tensors, path, metadata={"format": "pt", "note": 'a "quoted" value'})
    with LD.SafetensorsFile(path) as f:
        assert sorted(tensors) == f.names()
        for name, want in tensors.items():
            got = f.array(name)
            assert got.dtype == want.dtype and got.shape == want.shape and np.array_equal(got, want), name
        meta = json.loads(f.metadata_json())
        assert meta == {"format": "pt", "note": 'a "quoted" value'}


def test_rejects_header_lengths_outside_file(tmp_path):
    expect_rejected(tmp_path, "", 0, "header length", 2**64 - 1)
    expect_rejected(tmp_path, "{}", 0, "header length", 3)
    p = tmp_path / "tiny.safetensors"
    p.write_bytes(b"\x00\x00")
    with pytest.raises(LD.LoaderError, match="too small"):
        LD.SafetensorsFile(str(p))
    with pytest.raises(LD.LoaderError, match="cannot open"):
        LD.SafetensorsFile(str(tmp_path / "absent.safetensors"))


def test_rejects_leading_zero_numbers(tmp_path):
    expect_rejected(tmp_path, tensor_header("[01]", "[0,1]"), 1, "malformed number")
    expect_rejected(tmp_path, tensor_header("[1]", "[00,1]"), 1, "malformed number")


@pytest.mark.parametrize("offsets", ["[-1,0]", "[-8,-4]", "[0,-1]", "[1,0]", "[1048576,0]", "[0,2]",
                                     "[9223372036854775807,0]", "[18446744073709551615,0]", "[0.5,1]", '["0",1]',
                                     "[false,1]", "[0,1,2]", "[0]", "[]", "{}"])
def test_rejects_invalid_data_offsets(tmp_path, offsets):
    expect_rejected(tmp_path, tensor_header("[1]", offsets), 1, "data_offsets")


@pytest.mark.parametrize("shape", ["{}", "[-1]", "[0,-1]", "[1.5]", '["1"]', "[true]", "[18446744073709551615]"])
def test_rejects_invalid_shapes(tmp_path, shape):
    expect_rejected(tmp_path, tensor_header(shape, "[0,0]"), 0, "shape")


def test_rejects_size_mismatch_and_overflow(tmp_path):
    expect_rejected(tmp_path, tensor_header("[2]", "[0,4]", "F32"), 4, "shape/dtype")
    expect_rejected(tmp_path, tensor_header("[1]", "[0,8]", "F32"), 8, "shape/dtype")
    expect_rejected(tmp_path, tensor_header("[4294967296,4294967296]", "[0,0]"), 0, "element count")
    wide = str((2**64 - 1) // 4 + 1)
    expect_rejected(tmp_path, tensor_header("[" + wide + "]", "[0,0]", "F32"), 0, "shape/dtype")
    # the ordered checked product: a later zero does not undo an earlier overflowing multiply
    expect_rejected(tmp_path, tensor_header("[9223372036854775807,9223372036854775807,0]", "[0,0]"), 0, "element count")
    expect_rejected(tmp_path, tensor_header("[1]", "[0,1]", "F4"), 1, "unknown dtype")
    expect_rejected(tmp_path, "[1,2]", 0, "not an object")
    expect_rejected(tmp_path, '{"x":{"dtype":"U8","shape":[1]}}', 1, "data_offsets")
    expect_rejected(tmp_path, tensor_header("[1,1,1,1,1,1,1,1,1]", "[0,1]"), 1, "dimensions")


def test_scalar_empty_and_payload_end_views(tmp_path):
    header = ('{"scalar":{"dtype":"F32","shape":[],"data_offsets":[0,4]},'
              '"empty":{"dtype":"BF16","shape":[2,0,3],"data_offsets":[4,4]},'
              '"zero_first":{"dtype":"U8","shape":[0,5],"data_offsets":[4,4]}}')
    p = write_raw(tmp_path / "s.safetensors", header, bytes([0, 1, 2, 3]))
    with LD.SafetensorsFile(p) as f:
        assert len(f) == 3
        s = f.find("scalar")
        assert (s.rank, s.numel, s.nbytes) == (0, 1, 4)
        assert bytes((C.c_uint8 * 4).from_address(s.data)) == bytes([0, 1, 2, 3])
        for name in ("empty", "zero_first"):
            t = f.find(name)
            assert t.numel == 0 and t.nbytes == 0 and t.file_offset == 8 + len(header) + 4   # the end of the file
            assert f.array(name).size == 0
    # a zero reached before any overflowing product remains a valid empty tensor
    large = str((2**64 - 1) // 2)
    p = write_raw(tmp_path / "e.safetensors", tensor_header("[0," + large + "," + large + "]", "[0,0]"))
    with LD.SafetensorsFile(p) as f:
        assert f.find("x").numel == 0


@pytest.mark.parametrize("name,code,width", [("F32", LD.DT_F32, 4), ("F16", LD.DT_F16, 2), ("BF16", LD.DT_BF16, 2),
                                             ("F8_E4M3", LD.DT_F8_E4M3, 1), ("F8", LD.DT_F8_E4M3, 1),
                                             ("FP8", LD.DT_F8_E4M3, 1), ("I64", LD.DT_I64, 8), ("I32", LD.DT_I32, 4),
                                             ("U8", LD.DT_U8, 1), ("I8", LD.DT_I8, 1), ("F8_E8M0", LD.DT_F8_E8M0, 1),
                                             ("BOOL", LD.DT_U8, 1), ("U32", LD.DT_U32, 4), ("I16", LD.DT_I16, 2)])
def test_dtype_aliases_and_padded_header(tmp_path, name, code, width):
    header = tensor_header("[3]", "[0,%d]" % (3 * width), name)
    while (8 + len(header)) % 8:
        header += " "
    payload = bytes(i % 251 for i in range(3 * width))
    p = write_raw(tmp_path / "d.safetensors", header, payload)
    with LD.SafetensorsFile(p) as f:
        t = f.find("x")
        assert (t.dtype, t.numel, t.nbytes) == (code, 3, 3 * width)
        assert LD.lib().dgpp_dtype_size(code) == width
        assert bytes((C.c_uint8 * t.nbytes).from_address(t.data)) == payload


def test_duplicate_names_nested_metadata_and_escapes(tmp_path):
    header = ('{"__metadata__":{"a":{"b":[1,2.5e3,null,true]},"k":"v"},'
              '"t\\u0065nsor\\n":{"dtype":"U8","shape":[2],"data_offsets":[0,2],"extra":[{"x":1}]},'
              '"dup":{"dtype":"U8","shape":[1],"data_offsets":[0,1]},'
              '"dup":{"dtype":"U8","shape":[2],"data_offsets":[0,2]}}')
    p = write_raw(tmp_path / "m.safetensors", header, b"\x07\x09")
    with LD.SafetensorsFile(p) as f:
        assert f.names() == ["dup", "tensor\n"]
        assert f.find("dup").numel == 2, "the later descriptor of a repeated name stands"
        assert list(f.array("tensor\n")) == [7, 9]
        assert json.loads(f.metadata_json()) == {"a": {"b": [1, 2500.0, None, True]}, "k": "v"}
    expect_rejected(tmp_path, '{"x":{"dtype":"U8","shape":[1],"data_offsets":[0,1]}} trailing', 1, "trailing")


def test_quant_matrix_views_follow_the_scale_grid_contract():
    rows, cols = 512, 384
    payload = np.arange(rows * cols, dtype=np.uint32).astype(np.uint8)
    scales = np.arange(4 * 3, dtype=np.float32)
    m = LD.QuantMatrix(payload.ctypes.data, scales.ctypes.data, None, rows, cols, 128, 128)
    assert LD.quant_scale_shifts(m) == (True, 7, 7)
    v = LD.quant_rows_view(m, 256, 128)
    assert v.payload == payload.ctypes.data + 256 * cols and v.scales == scales.ctypes.data + 2 * 3 * 4
    assert (v.rows, v.cols, v.scale_block_rows, v.scale_block_cols) == (128, cols, 128, 128)
    assert LD.quant_rows_view(m, 0, rows).payload == payload.ctypes.data
    assert LD.quant_rows_view(m, 512, 0).rows == 0
    for start, n in ((200, 100), (64, 64), (-128, 128), (384, 256), (0, 513), (0, -1)):
        with pytest.raises(ValueError):
            LD.quant_rows_view(m, start, n)
    # the byte grid moves with the view too
    e8 = np.zeros(rows * (cols // 32), np.uint8)
    mx = LD.QuantMatrix(payload.ctypes.data, None, e8.ctypes.data, rows, cols, 1, 32)
    assert LD.quant_scale_shifts(mx) == (True, 0, 5)
    assert LD.quant_rows_view(mx, 7, 5).scales_e8m0 == e8.ctypes.data + 7 * (cols // 32)
    # a channel grid and grids no launcher takes
    assert LD.quant_scale_shifts(LD.QuantMatrix(None, None, None, 8, 4096, 1, 4096)) == (True, 0, 12)
    assert LD.quant_scale_shifts(LD.QuantMatrix(None, None, None, 8, 64, 96, 128))[0] is False
    assert LD.quant_scale_shifts(LD.QuantMatrix(None, None, None, 8, 64, 128, 8))[0] is False
    view = LD.expert_view_from_quant(m)
    assert (view.payload, view.scales, view.scale_shift_rows, view.scale_shift_cols) == (m.payload, m.scales, 7, 7)
    with pytest.raises(ValueError):
        LD.expert_view_from_quant(mx)


def test_fp4_matrix_views():
    rows, cols = 96, 256
    payload, scales = np.zeros(rows * cols // 2, np.uint8), np.zeros(rows * cols // 16, np.uint8)
    glob = np.ones(1, np.float32)
    m = _lib.Fp4Matrix(payload.ctypes.data, scales.ctypes.data, glob.ctypes.data, rows, cols, 16, 0, None)
    v = LD.fp4_rows_view(m, 33, 20)
    assert v.payload == payload.ctypes.data + 33 * cols // 2 and v.scales == scales.ctypes.data + 33 * cols // 16
    assert (v.rows, v.cols, v.scale_group, v.global_scale) == (20, cols, 16, glob.ctypes.data)
    mx = _lib.Fp4Matrix(payload.ctypes.data, scales.ctypes.data, None, rows, cols, 32, 0, None)
    assert LD.fp4_rows_view(mx, 95, 1).scales == scales.ctypes.data + 95 * cols // 32
    for start, n in ((90, 7), (-1, 1), (0, 97)):
        with pytest.raises(ValueError):
            LD.fp4_rows_view(m, start, n)
    with pytest.raises(ValueError):
        LD.fp4_rows_view(_lib.Fp4Matrix(payload.ctypes.data, scales.ctypes.data, None, rows, 250, 16, 0, None), 0, 1)
    with pytest.raises(ValueError):
        LD.fp4_rows_view(_lib.Fp4Matrix(payload.ctypes.data, scales.ctypes.data, None, rows, cols, 64, 0, None), 0, 1)
    e = LD.expert_view_from_fp4(m)
    assert (e.payload, e.fp4_scales, e.fp4_global, e.fp4_group) == (m.payload, m.scales, glob.ctypes.data, 16)
    e = LD.expert_view_from_fp4(mx)
    assert (e.fp4_global, e.fp4_group) == (None, 32)
    with pytest.raises(ValueError):
        LD.expert_view_from_fp4(_lib.Fp4Matrix(payload.ctypes.data, scales.ctypes.data, None, rows, cols, 16, 0, None))


@pytest.mark.parametrize("axis,start,count", [(0, 96, 96), (0, 64, 192), (0, 32, 32), (0, 128, 256), (1, 96, 96),
                                              (1, 192, 192), (1, 32, 160), (1, 0, 384), (0, 0, 512)])
def test_quant_slices_reblock_the_grid_and_keep_every_dequantized_value(axis, start, count):
    """A slice that starts inside a scale block is re-blocked at gcd(block, start, count) with the parent block's
    scale replicated (src/models/quant_matrix.hpp:28-34): each element dequantizes to exactly its parent value."""
    import np_ref
    from dgpp_amd import hostgen as hg
    rows, cols = 512, 384
    w = hg.f32_to_bf16(hg.normal_f32(0x5EED + axis, (rows, cols), 0.05))
    payload, scales = hg.encode_fp8_blocks(w, 128, 128)
    m = LD.QuantMatrix(payload.ctypes.data, scales.ctypes.data, None, rows, cols, 128, 128)
    sp, ss, v = LD.quant_slice(m, axis, start, count)
    g = int(np.gcd(128, np.gcd(start, count)))
    want_blocks = (g, 128) if axis == 0 else (128, g)
    assert (v.scale_block_rows, v.scale_block_cols) == want_blocks
    assert (v.rows, v.cols) == ((count, cols) if axis == 0 else (rows, count))
    ok, rs, cs = LD.quant_scale_shifts(v)
    assert ok and (1 << rs, 1 << cs) == want_blocks
    parent = np_ref.dequant_fp8(payload, scales, 7, 7)
    part = np_ref.dequant_fp8(sp, ss, rs, cs)
    sl = (slice(start, start + count), slice(None)) if axis == 0 else (slice(None), slice(start, start + count))
    assert np.array_equal(part, parent[sl])


def test_quant_slice_and_fp4_cols_slice_contracts():
    import np_ref
    from dgpp_amd import hostgen as hg
    rows, cols = 256, 256
    payload, scales = hg.encode_fp8_blocks(hg.f32_to_bf16(hg.normal_f32(77, (rows, cols), 0.05)), 128, 128)
    m = LD.QuantMatrix(payload.ctypes.data, scales.ctypes.data, None, rows, cols, 128, 128)
    for axis, start, count in ((1, 16, 16), (1, 24, 24), (0, 100, 60), (0, 48, 48), (0, -1, 4), (1, 200, 100), (2, 0, 32),
                               (0, 0, 0)):
        with pytest.raises(ValueError):
            LD.quant_slice(m, axis, start, count)   # blocks under 32 or not a power of two / outside the matrix
    assert LD.lib().dgpp_quant_slice_scale_count(C.byref(m), 1, 64, 64) == 2 * 1
    e8 = np.zeros((rows, cols // 32), np.uint8)
    with pytest.raises(ValueError):
        LD.quant_slice(LD.QuantMatrix(payload.ctypes.data, None, e8.ctypes.data, rows, cols, 1, 32), 1, 0, 64)

    for group, enc in ((16, hg.encode_nvfp4), (32, hg.encode_mxfp4)):
        res = enc(hg.normal_f32(78 + group, (rows, cols), 0.05))
        p4, s4 = res[0], res[1]
        glob = np.ones(1, np.float32)
        m4 = _lib.Fp4Matrix(p4.ctypes.data, s4.ctypes.data, glob.ctypes.data if group == 16 else None, rows, cols, group, 0, None)
        sp, ss, v = LD.fp4_cols_slice(m4, 64, 96)
        assert (v.rows, v.cols, v.scale_group, v.global_scale) == (rows, 96, group, m4.global_scale)
        assert np.array_equal(np_ref.dequant_fp4(sp, ss, group), np_ref.dequant_fp4(p4, s4, group)[:, 64:160])
        for start, n in ((8, 32), (0, 40), (224, 64), (-32, 32), (0, 0)):
            with pytest.raises(ValueError):
                LD.fp4_cols_slice(m4, start, n)


# ---- tensor names of a GLM-family MoE layer (src/models/glm/binding.cpp:32-54, :163-206) ---------------------------

def _glm_layer_tensors(prefix, E, H, I, fmt, shared_inter, rng):
    tensors, dtypes = {}, {}

    def fp8(name, rows, cols):
        tensors[name] = rng.integers(0, 120, size=(rows, cols), dtype=np.uint8)
        dtypes[name] = "F8_E4M3"
        tensors[name + "_scale_inv"] = rng.random((-(-rows // 128), -(-cols // 128)), dtype=np.float32)

    def nvfp4(name, rows, cols):
        tensors[name + "_packed"] = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
        tensors[name + "_scale"] = rng.integers(0, 120, size=(rows, cols // 16), dtype=np.uint8)
        dtypes[name + "_scale"] = "F8_E4M3"
        tensors[name + "_global_scale"] = np.array([2688.0], dtype=np.float32)

    tensors[prefix + "mlp.gate.weight"] = rng.integers(0, 2 ** 15, size=(E, H), dtype=np.uint16)
    dtypes[prefix + "mlp.gate.weight"] = "BF16"
    tensors[prefix + "mlp.gate.e_score_correction_bias"] = rng.random(E, dtype=np.float32)
    for proj, (r, c) in (("gate_proj", (shared_inter, H)), ("up_proj", (shared_inter, H)), ("down_proj", (H, shared_inter))):
        if shared_inter:
            fp8(f"{prefix}mlp.shared_experts.{proj}.weight", r, c)
    for e in range(E):
        for proj, (r, c) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            (nvfp4 if fmt == LD.BIND_NVFP4 else fp8)(f"{prefix}mlp.experts.{e}.{proj}.weight", r, c)
    return tensors, dtypes


def _write_named(path, tensors, dtypes):
    names = {np.dtype(np.uint8): "U8", np.dtype(np.float32): "F32", np.dtype(np.uint16): "BF16"}
    header, blobs, at = {}, [], 0
    for name, a in tensors.items():
        a = np.asarray(a, order="C")                       # keeps a scalar's empty shape
        header[name] = {"dtype": dtypes.get(name, names[a.dtype]), "shape": list(a.shape), "data_offsets": [at, at + a.nbytes]}
        blobs.append(a.tobytes())
        at += a.nbytes
    text = json.dumps(header, separators=(",", ":"))
    text += " " * (-(8 + len(text)) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text.encode() + b"".join(blobs))


@pytest.mark.parametrize("fmt", [LD.BIND_FP8, LD.BIND_NVFP4])
def test_glm_moe_layer_binding_finds_every_tensor_across_shards(tmp_path, fmt):
    rng = np.random.default_rng(17)
    E, H, I, S = 5, 256, 160, 160
    prefix = "model.layers.3."
    tensors, dtypes = _glm_layer_tensors(prefix, E, H, I, fmt, S, rng)
    names = list(tensors)
    shards = [dict((n, tensors[n]) for n in names[i::2]) for i in range(2)]      # spread over two shards
    paths = []
    for i, sh in enumerate(shards):
        paths.append(str(tmp_path / f"model-{i}.safetensors"))
        _write_named(paths[-1], sh, dtypes)
    files = [LD.SafetensorsFile(p) for p in paths]
    try:
        rw, rb, shared, routed = LD.glm_moe_bind_layer(files, prefix, E, H, I, fmt, S)
        assert rw.dims() == (E, H) and rw.dtype == LD.DT_BF16 and rb.dims() == (E,)
        assert np.array_equal(files[0].array(prefix + "mlp.gate.weight") if (prefix + "mlp.gate.weight") in files[0]
                              else files[1].array(prefix + "mlp.gate.weight"), tensors[prefix + "mlp.gate.weight"])
        assert [m.payload.dims() for m in shared] == [(S, H), (S, H), (H, S)] and all(m.format == LD.BIND_FP8 for m in shared)
        for e in range(E):
            for m, proj, (r, c) in zip(routed[e], ("gate_proj", "up_proj", "down_proj"), ((I, H), (I, H), (H, I))):
                base = f"{prefix}mlp.experts.{e}.{proj}.weight"
                pay_name = base + ("_packed" if fmt == LD.BIND_NVFP4 else "")
                assert m.format == fmt and pay_name in files[m.file_index]
                want = tensors[pay_name]
                got = np.frombuffer((C.c_uint8 * m.payload.nbytes).from_address(m.payload.data), dtype=np.uint8)
                assert np.array_equal(got.reshape(want.shape), want)
                if fmt == LD.BIND_NVFP4:
                    assert m.payload.dims() == (r, c // 2) and m.scales.dims() == (r, c // 16) and m.global_.dims() == (1,)
                    assert m.scales.dtype == LD.DT_F8_E4M3 and m.global_.dtype == LD.DT_F32
                else:
                    assert m.payload.dims() == (r, c) and m.scales.dims() == (-(-r // 128), -(-c // 128))
                    assert m.payload.dtype == LD.DT_F8_E4M3 and m.scales.dtype == LD.DT_F32
        # no shared expert, no bias: nothing of them is looked up
        rw2, rb2, sh2, routed2 = LD.glm_moe_bind_layer(files, prefix, E, H, I, fmt, 0, with_bias=False)
        assert rb2 is None and sh2 is None and len(routed2) == E
        # the resident build refuses what it cannot slice before it touches a device
        from dgpp_amd import launch as L, moe_layer as ML
        cfg = L.make_config(H, I, E, 2, n_shared_experts=1)
        for kw, text in ((dict(rank=2, world=2), "rank must lie"), (dict(rank=0, world=3), "must divide by world"),
                         (dict(rank=0, world=32), "re-block" if fmt == LD.BIND_FP8 else "whole scale groups")):
            with pytest.raises(L.InvalidArgument, match=text):
                ML.ResidentMoeLayer(cfg, 4, routed, shared=shared, shared_inter=S, router_weight=rw, router_bias=rb, **kw)
        with pytest.raises(L.InvalidArgument, match="does not have the layer's geometry"):
            ML.ResidentMoeLayer(L.make_config(H, I * 2, E, 2), 4, routed)
    finally:
        for f in files:
            f.close()


def test_glm_moe_layer_binding_names_what_is_wrong(tmp_path):
    rng = np.random.default_rng(18)
    E, H, I = 3, 128, 64
    prefix = "model.layers.0."
    tensors, dtypes = _glm_layer_tensors(prefix, E, H, I, LD.BIND_FP8, 0, rng)

    def bind(t, d, **kw):
        path = str(tmp_path / f"m{len(list(tmp_path.iterdir()))}.safetensors")
        _write_named(path, t, d)
        with LD.SafetensorsFile(path) as f:
            return LD.glm_moe_bind_layer([f], prefix, kw.get("E", E), H, I, kw.get("fmt", LD.BIND_FP8), kw.get("S", 0))

    bind(tensors, dtypes)
    missing = dict(tensors)
    del missing[prefix + "mlp.experts.2.up_proj.weight_scale_inv"]
    with pytest.raises(ValueError, match=r"missing tensor 'model\.layers\.0\.mlp\.experts\.2\.up_proj\.weight_scale_inv'"):
        bind(missing, dtypes)
    wrong_dtype = dict(dtypes)
    wrong_dtype[prefix + "mlp.experts.1.down_proj.weight"] = "U8"
    with pytest.raises(ValueError, match=r"experts\.1\.down_proj\.weight' is dtype"):
        bind(tensors, wrong_dtype)
    wrong_shape = dict(tensors)
    wrong_shape[prefix + "mlp.experts.0.gate_proj.weight_scale_inv"] = np.zeros((2, 1), dtype=np.float32)
    with pytest.raises(ValueError, match=r"gate_proj\.weight_scale_inv' is dtype .* expected"):
        bind(wrong_shape, dtypes)
    with pytest.raises(ValueError, match=r"mlp\.gate\.weight' is dtype .*\[3, 128\], expected .*\[4, 128\]"):
        bind(tensors, dtypes, E=4)                       # the router of this file serves three experts
    with pytest.raises(ValueError, match="missing tensor"):
        bind(tensors, dtypes, fmt=LD.BIND_NVFP4)         # the NVFP4 spelling is not there
    with pytest.raises(ValueError, match="shared_experts"):
        bind(tensors, dtypes, S=64)


# ---- tensor names of a Qwen-family MoE block (src/models/qwen/binding.cpp:26-66, :158-215) -------------------------

def _qwen_block_tensors(p, E, H, I, S, routed_fmt, shared_fmt, rng):
    tensors, dtypes = {}, {}

    def put(name, rows, cols, fmt):
        stem = name[:-len(".weight")]
        if fmt == LD.BIND_NVFP4_MODELOPT:
            tensors[name] = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
            tensors[stem + ".weight_scale"] = rng.integers(0, 120, size=(rows, cols // 16), dtype=np.uint8)
            dtypes[stem + ".weight_scale"] = "F8_E4M3"
            tensors[stem + ".weight_scale_2"] = np.array(3.5e-4, dtype=np.float32)
            tensors[stem + ".input_scale"] = np.array(1.0, dtype=np.float32)       # shipped, never looked up
        elif fmt == LD.BIND_MXFP8:
            tensors[name] = rng.integers(0, 120, size=(rows, cols), dtype=np.uint8)
            dtypes[name] = "F8_E4M3"
            tensors[stem + ".weight_scale"] = rng.integers(110, 130, size=(rows, cols // 32), dtype=np.uint8)
        else:
            tensors[name] = rng.integers(0, 120, size=(rows, cols), dtype=np.uint8)
            dtypes[name] = "F8_E4M3"
            grid = (-(-rows // 128), -(-cols // 128))
            if fmt == LD.BIND_FP8_BF16_SCALES:
                tensors[name + "_scale_inv"] = rng.integers(0x3000, 0x3F00, size=grid, dtype=np.uint16)
                dtypes[name + "_scale_inv"] = "BF16"
            else:
                tensors[name + "_scale_inv"] = rng.random(grid, dtype=np.float32)

    tensors[p + "gate.weight"] = rng.integers(0, 2 ** 15, size=(E, H), dtype=np.uint16)
    dtypes[p + "gate.weight"] = "BF16"
    if S:
        tensors[p + "shared_expert_gate.weight"] = rng.integers(0, 2 ** 15, size=(1, H), dtype=np.uint16)
        dtypes[p + "shared_expert_gate.weight"] = "BF16"
        for proj, (r, c) in (("gate_proj", (S, H)), ("up_proj", (S, H)), ("down_proj", (H, S))):
            put(f"{p}shared_expert.{proj}.weight", r, c, shared_fmt)
    for e in range(E):
        for proj, (r, c) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            put(f"{p}experts.{e}.{proj}.weight", r, c, routed_fmt)
    return tensors, dtypes


@pytest.mark.parametrize("routed_fmt,shared_fmt", [(LD.BIND_FP8_BF16_SCALES, LD.BIND_FP8), (LD.BIND_NVFP4_MODELOPT, LD.BIND_MXFP8),
                                                   (LD.BIND_FP8, LD.BIND_FP8)])
def test_qwen_moe_block_binding(tmp_path, routed_fmt, shared_fmt):
    rng = np.random.default_rng(23)
    E, H, I, S = 4, 256, 128, 192
    p = "model.layers.5.mlp."
    tensors, dtypes = _qwen_block_tensors(p, E, H, I, S, routed_fmt, shared_fmt, rng)
    path = str(tmp_path / "qwen.safetensors")
    _write_named(path, tensors, dtypes)
    with LD.SafetensorsFile(path) as f:
        rw, sg, shared, routed = LD.qwen_moe_bind_layer([f], p, E, H, I, routed_fmt, S, shared_fmt)
        assert rw.dims() == (E, H) and sg.dims() == (1, H) and sg.dtype == LD.DT_BF16
        assert [m.format for m in shared] == [shared_fmt] * 3
        assert shared[2].payload.dims() == (H, S)
        if shared_fmt == LD.BIND_MXFP8:
            assert shared[0].scales.dims() == (S, H // 32) and shared[0].scales.dtype == LD.DT_U8
        for e in range(E):
            g, u, d = routed[e]
            if routed_fmt == LD.BIND_NVFP4_MODELOPT:
                assert g.payload.dims() == (I, H // 2) and g.scales.dims() == (I, H // 16) and g.global_.dims() == ()
                assert d.payload.dims() == (H, I // 2)
                got = np.frombuffer((C.c_uint8 * 4).from_address(g.global_.data), dtype=np.float32)[0]
                assert got == np.float32(3.5e-4)
            else:
                want_dt = LD.DT_BF16 if routed_fmt == LD.BIND_FP8_BF16_SCALES else LD.DT_F32
                assert g.payload.dims() == (I, H) and g.scales.dims() == (1, 2) and g.scales.dtype == want_dt
                assert d.scales.dims() == (2, 1)
        rw2, sg2, sh2, routed2 = LD.qwen_moe_bind_layer([f], p, E, H, I, routed_fmt)
        assert sg2 is None and sh2 is None and len(routed2) == E
        with pytest.raises(ValueError, match="missing tensor|is dtype"):
            LD.qwen_moe_bind_layer([f], p, E, H, I, LD.BIND_MXFP8 if routed_fmt != LD.BIND_MXFP8 else LD.BIND_FP8)
        with pytest.raises(ValueError, match=r"shared_expert\.gate_proj\.weight' is dtype"):
            LD.qwen_moe_bind_layer([f], p, E, H, I, routed_fmt, S + 64, shared_fmt)
        with pytest.raises(ValueError, match="unknown expert format"):
            LD.qwen_moe_bind_layer([f], p, E, H, I, 9)


def test_checkpoint_directory_follows_the_index_when_there_is_one(tmp_path):
    """The shard set of a checkpoint directory (reference: src/loaders/resident_stream.hpp:257-296): the index's
    weight_map is authoritative (sub-directories included, files it does not name ignored), else every shard of the
    directory; a layer binds across the set by name."""
    rng = np.random.default_rng(23)
    E, H, I = 3, 256, 128
    prefix = "model.layers.0."
    tensors, dtypes = _glm_layer_tensors(prefix, E, H, I, LD.BIND_FP8, 0, rng)
    names = list(tensors)
    (tmp_path / "tensors").mkdir()
    rel = ["model-00002-of-00002.safetensors", "tensors/model-00001-of-00002.safetensors"]
    for i, r in enumerate(rel):
        _write_named(str(tmp_path / r), dict((n, tensors[n]) for n in names[i::2]), dtypes)
    # a stray shard that repeats a tensor: ignored under an index, a duplicate without one
    _write_named(str(tmp_path / "stray.safetensors"), {names[0]: tensors[names[0]]}, dtypes)
    index = {"metadata": {"total_size": 1, "nested": {"a": [1, 2, {"b": None}]}},
             "weight_map": {n: rel[i % 2] for i, n in enumerate(names)}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with LD.Checkpoint(str(tmp_path)) as ck:
        assert [os.path.relpath(p, tmp_path) for p in ck.shard_paths()] == sorted(rel)     # ascending path order
        assert ck.tensor_count() == len(names)
        for n in names[:7]:
            info, at = ck.find(n)
            assert rel[names.index(n) % 2] == os.path.relpath(ck.shard_paths()[at], tmp_path)
            assert np.array_equal(ck.array(n), np.asarray(tensors[n]))
        with pytest.raises(ValueError, match="missing tensor 'nope'"):
            ck.find("nope")
        rw, rb, shared, routed = LD.glm_moe_bind_layer(ck.files, prefix, E, H, I, LD.BIND_FP8, 0)
        assert len(routed) == E and shared is None
        assert routed[2][1].payload.dims() == (I, H)
    # a shard the index names but the directory lacks
    index["weight_map"]["extra.weight"] = "model-00003-of-00003.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(LD.LoaderError, match="named by the index is missing"):
        LD.Checkpoint(str(tmp_path))
    # an index without a weight_map, and one that is not JSON
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}}))
    with pytest.raises(LD.LoaderError, match="no weight_map"):
        LD.Checkpoint(str(tmp_path))
    (tmp_path / "model.safetensors.index.json").write_text('{"weight_map": {"a": 3}}')
    with pytest.raises(LD.LoaderError):
        LD.Checkpoint(str(tmp_path))


def test_checkpoint_directory_without_an_index(tmp_path):
    rng = np.random.default_rng(29)
    a = rng.integers(0, 255, size=(4, 32), dtype=np.uint8)
    b = rng.random((3,), dtype=np.float32)
    with pytest.raises(LD.LoaderError, match="no .safetensors shards"):
        LD.Checkpoint(str(tmp_path))
    with pytest.raises(LD.LoaderError, match="not a directory"):
        LD.Checkpoint(str(tmp_path / "absent"))
    _write_named(str(tmp_path / "b.safetensors"), {"w.b": b}, {})
    _write_named(str(tmp_path / "a.safetensors"), {"w.a": a}, {})
    (tmp_path / "notes.txt").write_text("not a shard")
    (tmp_path / "sub").mkdir()
    _write_named(str(tmp_path / "sub" / "c.safetensors"), {"w.a": a}, {})          # only the directory itself is scanned
    with LD.Checkpoint(str(tmp_path)) as ck:
        assert [os.path.basename(p) for p in ck.shard_paths()] == ["a.safetensors", "b.safetensors"]
        assert ck.find("w.a")[1] == 0 and ck.find("w.b")[1] == 1
        assert np.array_equal(ck.array("w.b"), b)
    _write_named(str(tmp_path / "c.safetensors"), {"w.a": a}, {})                  # the same name in two shards
    with pytest.raises(LD.LoaderError, match="duplicate tensor 'w.a'"):
        LD.Checkpoint(str(tmp_path))


def test_mimo_and_minimax_moe_block_bindings(tmp_path):
    """The MXFP4 block of a MiMo-family export (reference: src/models/mimo/binding.cpp:38-71) and the NVFP4 + MXFP8
    block of a MiniMax-family export (src/models/minimax/binding.cpp:15-71: w1 / w3 / w2 are gate / up / down)."""
    rng = np.random.default_rng(31)
    E, H, I, S = 3, 256, 128, 192
    tensors, dtypes = {}, {}

    def u8(name, shape, dt=None):
        tensors[name] = rng.integers(0, 120, size=shape, dtype=np.uint8)
        if dt:
            dtypes[name] = dt

    p = "model.layers.2.mlp."
    tensors[p + "gate.weight"] = rng.integers(0, 2 ** 15, size=(E, H), dtype=np.uint16)
    dtypes[p + "gate.weight"] = "BF16"
    tensors[p + "gate.e_score_correction_bias"] = rng.random(E, dtype=np.float32)
    q = "language_model.model.layers.4.block_sparse_moe."
    tensors[q + "gate.weight"] = rng.random((E, H), dtype=np.float32)
    tensors[q + "e_score_correction_bias"] = rng.random(E, dtype=np.float32)
    for proj, (r, c) in (("gate_proj", (S, H)), ("up_proj", (S, H)), ("down_proj", (H, S))):
        u8(f"{q}shared_experts.{proj}.weight", (r, c), "F8_E4M3")
        u8(f"{q}shared_experts.{proj}.weight_scale_inv", (r, c // 32))
    for e in range(E):
        for proj, (r, c) in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
            u8(f"{p}experts.{e}.{proj}.weight", (r, c // 2))
            u8(f"{p}experts.{e}.{proj}.weight_scale", (r, c // 32))
        for w, (r, c) in (("w1", (I, H)), ("w3", (I, H)), ("w2", (H, I))):
            u8(f"{q}experts.{e}.{w}.weight_packed", (r, c // 2))
            u8(f"{q}experts.{e}.{w}.weight_scale", (r, c // 16), "F8_E4M3")
            tensors[f"{q}experts.{e}.{w}.weight_global_scale"] = np.float32(2688.0 + e)
            tensors[f"{q}experts.{e}.{w}.input_global_scale"] = np.float32(1.0)
    path = str(tmp_path / "blocks.safetensors")
    _write_named(path, tensors, dtypes)
    with LD.SafetensorsFile(path) as f:
        rw, rb, routed = LD.mimo_moe_bind_layer([f], p, E, H, I)
        assert rw.dims() == (E, H) and rw.dtype == LD.DT_BF16 and rb.dims() == (E,)
        for e in range(E):
            g, u, d = routed[e]
            assert [m.format for m in (g, u, d)] == [LD.BIND_MXFP4] * 3
            assert g.payload.dims() == (I, H // 2) and g.scales.dims() == (I, H // 32) and g.scales.dtype == LD.DT_U8
            assert d.payload.dims() == (H, I // 2) and d.scales.dims() == (H, I // 32)
            assert np.array_equal(np.frombuffer((C.c_uint8 * u.payload.nbytes).from_address(u.payload.data), dtype=np.uint8),
                                  tensors[f"{p}experts.{e}.up_proj.weight"].ravel())
        with pytest.raises(ValueError, match=r"experts\.0\.gate_proj\.weight' is dtype"):
            LD.mimo_moe_bind_layer([f], p, E, H, I * 2)
        with pytest.raises(ValueError, match=r"gate\.weight' is dtype 2 \[3, 256\], expected dtype 2 \[4, 256\]"):
            LD.mimo_moe_bind_layer([f], p, E + 1, H, I)
        with pytest.raises(ValueError, match="missing tensor 'model.layers.9"):
            LD.mimo_moe_bind_layer([f], "model.layers.9.mlp.", E, H, I)

        rw, rb, shared, routed = LD.minimax_moe_bind_layer([f], q, E, H, I, S)
        assert rw.dims() == (E, H) and rw.dtype == LD.DT_F32 and rb.dims() == (E,)
        assert [m.format for m in shared] == [LD.BIND_MXFP8_SCALE_INV] * 3
        assert shared[0].scales.dims() == (S, H // 32) and shared[2].payload.dims() == (H, S)
        for e in range(E):
            g, u, d = routed[e]
            assert g.payload.dims() == (I, H // 2) and g.scales.dims() == (I, H // 16) and g.global_.dims() == ()
            assert d.payload.dims() == (H, I // 2) and d.scales.dims() == (H, I // 16)
            # w3 is the up projection, w2 the down projection
            assert np.array_equal(np.frombuffer((C.c_uint8 * u.payload.nbytes).from_address(u.payload.data), dtype=np.uint8),
                                  tensors[f"{q}experts.{e}.w3.weight_packed"].ravel())
            assert np.array_equal(np.frombuffer((C.c_uint8 * d.payload.nbytes).from_address(d.payload.data), dtype=np.uint8),
                                  tensors[f"{q}experts.{e}.w2.weight_packed"].ravel())
            assert np.frombuffer((C.c_uint8 * 4).from_address(g.global_.data), dtype=np.float32)[0] == np.float32(2688.0 + e)
        assert LD.minimax_moe_bind_layer([f], q, E, H, I)[2] is None
        with pytest.raises(ValueError, match=r"shared_experts\.gate_proj\.weight' is dtype"):
            LD.minimax_moe_bind_layer([f], q, E, H, I, S + 32)

