"""A checkpoint on disk drives the layer: per-expert tensors are written as a safetensors file (the names a
compressed-tensors MoE export uses), read back through the memory-mapped reader, uploaded as they are, turned
into expert-table entries by the loader's view helpers, and the layer's output equals — bit for bit — the
output of the same weights handed over directly. Row slices of a resident matrix (the tensor-parallel split of
gate / up) give the rows of the unsliced launch."""
import struct

import numpy as np
import pytest

import moe_data
from dgpp_amd import _lib, launch as L, loader as LD, moe_layer as ML
from gpu_util import DeviceMoe, dev, dev_empty, host, sync, view_table
from test_gpu_moe_layer import make_layer

pytestmark = pytest.mark.gpu

_DT = {np.dtype(np.uint8): "U8", np.dtype(np.float32): "F32", np.dtype(np.uint16): "BF16"}
PROJ = ("gate_proj", "up_proj", "down_proj")


def write_checkpoint(path, tensors, dtypes=None):
    """A safetensors file from numpy arrays (header JSON + payload, 8-byte padded header)."""
    header, payload, at = {}, [], 0
    for name, a in tensors.items():
        a = np.ascontiguousarray(a)
        dt = (dtypes or {}).get(name, _DT[a.dtype])
        header[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [at, at + a.nbytes]}
        payload.append(a.tobytes())
        at += a.nbytes
    import json
    h = json.dumps(header, separators=(",", ":"))
    while (8 + len(h)) % 8:
        h += " "
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)))
        f.write(h.encode())
        for b in payload:
            f.write(b)


@pytest.mark.parametrize("kind", ["fp8", "nvfp4", "mxfp4"])
def test_layer_from_a_checkpoint_file_is_bitwise_the_layer_from_the_arrays(gpu, tmp_path, kind):
    E, H, I, K, T = 6, 512, 128, 3, 5
    p = moe_data.make_problem(E, H, I, K, T, kind, 8800, shared_kind=None, limit=float("inf"), std=0.05)
    tensors, dtypes = {}, {}
    for e, mats in enumerate(p.experts):
        for m, proj in zip(mats, PROJ):
            base = f"model.layers.3.mlp.experts.{e}.{proj}"
            tensors[base + ".weight"] = m.payload
            tensors[base + ".weight_scale"] = m.scales
            if kind == "fp8":
                dtypes[base + ".weight"] = "F8_E4M3"
            elif kind == "nvfp4":
                dtypes[base + ".weight_scale"] = "F8_E4M3"
                tensors[base + ".weight_global"] = m.glob          # the device-side divisor, F32 [1]
            else:
                dtypes[base + ".weight_scale"] = "F8_E8M0"
    path = str(tmp_path / "layer3.safetensors")
    write_checkpoint(path, tensors, dtypes)

    keep, entries = [], []
    with LD.SafetensorsFile(path) as f:
        assert len(f) == len(tensors)
        for e in range(E):
            for proj in PROJ:
                base = f"model.layers.3.mlp.experts.{e}.{proj}"
                w, s = f.find(base + ".weight"), f.find(base + ".weight_scale")
                f.prefetch(w)
                wd, sd = dev(np.array(f.array(base + ".weight"))), dev(np.array(f.array(base + ".weight_scale")))
                f.discard(w)
                keep += [wd, sd]
                rows = w.dims()[0]
                if kind == "fp8":
                    assert w.dtype == LD.DT_F8_E4M3 and s.dtype == LD.DT_F32
                    m = LD.QuantMatrix(wd.data_ptr(), sd.data_ptr(), None, rows, w.dims()[1], 128, 128)
                    entries.append(LD.expert_view_from_quant(m))
                else:
                    group = 16 if kind == "nvfp4" else 32
                    assert s.dtype == (LD.DT_F8_E4M3 if kind == "nvfp4" else LD.DT_F8_E8M0)
                    gd = None
                    if kind == "nvfp4":
                        gd = dev(np.array(f.array(base + ".weight_global")))
                        keep.append(gd)
                    m = _lib.Fp4Matrix(wd.data_ptr(), sd.data_ptr(), gd.data_ptr() if gd is not None else None, rows,
                                       w.dims()[1] * 2, group, 0, None)
                    entries.append(LD.expert_view_from_fp4(m))
    # the mapping is gone; the layer runs from the uploaded bytes alone
    d = DeviceMoe(p)
    ref_layer = make_layer(p, d, 1, 1.0, T)
    d2 = DeviceMoe.__new__(DeviceMoe)
    d2.p, d2.keep, d2.views, d2.x, d2.shared_view_base, d2.sh = p, keep, view_table(entries), d.x, -1, None
    d2.fp4_group = d.fp4_group
    got_layer = make_layer(p, d2, 1, 1.0, T)
    want, got = dev_empty((T, H), np.uint16), dev_empty((T, H), np.uint16)
    ref_layer.enqueue_decode(d.x, H, want, T)
    got_layer.enqueue_decode(d.x, H, got, T)
    sync()
    assert np.array_equal(host(got, np.uint16), host(want, np.uint16))
    assert host(want, np.uint16).any()
    ref_layer.close()
    got_layer.close()


def test_row_slices_of_resident_matrices_give_the_rows_of_the_whole(gpu):
    """The tensor-parallel split of gate / up is a row range of the resident matrix: a pointer view
    (src/models/quant_matrix.hpp:78-96, :152-164) whose GEMV equals the rows of the unsliced launch."""
    n, k, m = 512, 1024, 3
    fp8 = moe_data.make_mat("fp8", n, k, 9100, 0.05)
    nv = moe_data.make_mat("nvfp4", n, k, 9101, 0.05)
    act = dev(moe_data.hg.normal_bf16(9102, (m, k)))
    pd, sd = dev(fp8.payload), dev(fp8.scales)
    whole = LD.QuantMatrix(pd.data_ptr(), sd.data_ptr(), None, n, k, 128, 128)
    full, part = dev_empty((m, n), np.uint16), dev_empty((m, 256), np.uint16)
    L.launch_scale_gemm_bf16(act, k, pd, sd, full, m, n, k, None)
    v = LD.quant_rows_view(whole, 256, 256)
    ok, rs, cs = LD.quant_scale_shifts(v)
    assert ok and (rs, cs) == (7, 7)
    L.launch_scale_gemm_bf16(act, k, v.payload, v.scales, part, m, 256, k, None)
    sync()
    assert np.array_equal(host(part, np.uint16), host(full, np.uint16)[:, 256:512])

    p4, s4, g4 = dev(nv.payload), dev(nv.scales), dev(nv.glob)
    whole4 = _lib.Fp4Matrix(p4.data_ptr(), s4.data_ptr(), g4.data_ptr(), n, k, 16, 0, None)
    full4, part4 = dev_empty((m, n), np.uint16), dev_empty((m, 100), np.uint16)
    L.launch_fp4_gemv_bf16(act, k, whole4, full4, m, n, k, None)
    v4 = LD.fp4_rows_view(whole4, 37, 100)
    L.launch_fp4_gemv_bf16(act, k, v4, part4, m, 100, k, None)
    sync()
    assert np.array_equal(host(part4, np.uint16), host(full4, np.uint16)[:, 37:137])


def test_column_slices_feed_the_grid_launchers(gpu):
    """The tensor-parallel split of the down projection: each rank's column slice (grid re-blocked at 64) against
    its slice of the activations matches the oracle on the sliced problem, and the ranks' partial rows add up to
    the unsliced product (to fp32 summation order)."""
    import oracle_lib as orc
    from dgpp_amd import hostgen as hg
    from test_gpu_dense_gemv import check
    n, k, m, world = 256, 384, 2, 2
    w = hg.f32_to_bf16(hg.normal_f32(9200, (n, k), 0.05))
    payload, scales = hg.encode_fp8_blocks(w, 128, 128)
    act = hg.normal_bf16(9201, (m, k))
    whole = LD.QuantMatrix(payload.ctypes.data, scales.ctypes.data, None, n, k, 128, 128)
    full = dev_empty((m, n), np.float32)
    L.launch_scale_gemm_f32(dev(act), k, dev(payload), dev(scales), full, m, n, k, None)
    total = np.zeros((m, n), np.float64)
    for r in range(world):
        c0, cn = r * k // world, k // world
        sp, ss, v = LD.quant_slice(whole, 1, c0, cn)
        ok, rs, cs = LD.quant_scale_shifts(v)
        assert ok and (rs, cs) == (7, 6)
        a_r = np.ascontiguousarray(act[:, c0:c0 + cn])
        out = dev_empty((m, n), np.float32)
        L.launch_scale_gemm_grid_f32(dev(a_r), cn, dev(sp), dev(ss), out, m, n, cn, None, 0, rs, cs)
        sync()
        got = host(out)
        raw = orc.gemv_fp8(a_r, sp, ss, m, n, cn, rs, cs, True)
        check(hg.f32_to_bf16(got), raw, f"down slice of rank {r}")
        total += got
    sync()
    ref = host(full).astype(np.float64)
    assert np.max(np.abs(total - ref)) <= 1e-4 * max(1.0, np.max(np.abs(ref)))


@pytest.mark.parametrize("kind", ["fp8", "nvfp4"])
def test_layer_bound_by_the_glm_tensor_names_is_bitwise_the_layer_from_the_arrays(gpu, tmp_path, kind):
    """The checkpoint spells its tensors as a GLM-family export does (src/models/glm/binding.cpp:32-54, :163-206);
    the loader's binding finds and checks them across two shards, and the layer built from what it found gives the
    bits of the layer built from the arrays."""
    import ctypes as C

    E, H, I, K, T = 6, 512, 128, 3, 5
    p = moe_data.make_problem(E, H, I, K, T, kind, 8900, shared_kind=None, limit=float("inf"), std=0.05)
    prefix = "model.layers.7."
    tensors, dtypes = {prefix + "mlp.gate.weight": p.router_gate,
                       prefix + "mlp.gate.e_score_correction_bias": p.router_bias}, {}
    for e, mats in enumerate(p.experts):
        for m, proj in zip(mats, PROJ):
            base = f"{prefix}mlp.experts.{e}.{proj}.weight"
            if kind == "fp8":
                tensors[base], dtypes[base] = m.payload, "F8_E4M3"
                tensors[base + "_scale_inv"] = m.scales
            else:
                tensors[base + "_packed"] = m.payload
                tensors[base + "_scale"], dtypes[base + "_scale"] = m.scales, "F8_E4M3"
                tensors[base + "_global_scale"] = m.glob
    names = sorted(tensors)
    paths = []
    for i in range(2):
        paths.append(str(tmp_path / f"model-0000{i + 1}-of-00002.safetensors"))
        write_checkpoint(paths[-1], {n: tensors[n] for n in names[i::2]}, dtypes)

    def upload(info):
        a = np.frombuffer((C.c_uint8 * info.nbytes).from_address(info.data), dtype=np.uint8)
        return dev(np.array(a))

    # the directory opens as one shard set through its index
    import json
    import os
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"metadata": {}, "weight_map": {n: os.path.basename(paths[i % 2]) for i, n in enumerate(names)}}))
    ck = LD.Checkpoint(str(tmp_path))
    files = ck.files
    assert ck.tensor_count() == len(names) and len(files) == 2
    keep, entries = [], []
    try:
        rw, rb, shared, routed = LD.glm_moe_bind_layer(files, prefix, E, H, I, LD.BIND_FP8 if kind == "fp8" else LD.BIND_NVFP4)
        assert shared is None and rw.dims() == (E, H) and rb.dims() == (E,)
        for e in range(E):
            for m in routed[e]:
                wd, sd = upload(m.payload), upload(m.scales)
                keep += [wd, sd]
                rows = m.payload.dims()[0]
                if kind == "fp8":
                    q = LD.QuantMatrix(wd.data_ptr(), sd.data_ptr(), None, rows, m.payload.dims()[1], 128, 128)
                    entries.append(LD.expert_view_from_quant(q))
                else:
                    gd = upload(m.global_)
                    keep.append(gd)
                    q = _lib.Fp4Matrix(wd.data_ptr(), sd.data_ptr(), gd.data_ptr(), rows, m.payload.dims()[1] * 2, 16, 0, None)
                    entries.append(LD.expert_view_from_fp4(q))
    finally:
        ck.close()
    d = DeviceMoe(p)
    ref_layer = make_layer(p, d, 1, 1.0, T)
    d2 = DeviceMoe.__new__(DeviceMoe)
    d2.p, d2.keep, d2.views, d2.x, d2.shared_view_base, d2.sh = p, keep, view_table(entries), d.x, -1, None
    d2.fp4_group = d.fp4_group
    got_layer = make_layer(p, d2, 1, 1.0, T)
    want, got = dev_empty((T, H), np.uint16), dev_empty((T, H), np.uint16)
    ref_layer.enqueue_decode(d.x, H, want, T)
    got_layer.enqueue_decode(d.x, H, got, T)
    sync()
    assert np.array_equal(host(got, np.uint16), host(want, np.uint16))
    assert host(want, np.uint16).any()
    ref_layer.close()
    got_layer.close()
