"""A checkpoint on disk drives the layer: per-expert tensors are written as a safetensors file (the names a
compressed-tensors MoE export uses), read back through the memory-mapped reader, uploaded as they are, turned
into expert-table entries by the loader's view helpers, and the layer's output equals — bit for bit — the
output of the same weights handed over directly. Row slices of a resident matrix (the tensor-parallel split of
gate / up) give the rows of the unsliced launch."""
import struct

import numpy as np
import pytest

import moe_data
from dgpp_amd import _lib, hostgen as hg, launch as L, loader as LD, moe_layer as ML
from gpu_util import DeviceMoe, dev, dev_empty, host, sync, view_table
from test_gpu_moe_layer import make_layer

pytestmark = pytest.mark.gpu

_DT = {np.dtype(np.uint8): "U8", np.dtype(np.float32): "F32", np.dtype(np.uint16): "BF16"}
PROJ = ("gate_proj", "up_proj", "down_proj")


def write_checkpoint(path, tensors, dtypes=None):
    """A safetensors file from numpy arrays (header JSON + payload, 8-byte padded header)."""
    header, payload, at = {}, [], 0
    for name, a in tensors.items():
        a = np.asarray(a, order="C")   # keeps a scalar tensor's empty shape
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


def _checkpoint_tensors(p, family):
    """The problem's tensors under a model family's names: 'glm' (block FP8 or NVFP4 in the engine's own spelling, the
    shared expert block FP8), 'mimo' (MXFP4), 'minimax' (compressed-tensors NVFP4, MXFP8 shared expert)."""
    tensors, dtypes = {}, {}
    if family == "glm":
        pre = "model.layers.3."
        tensors[pre + "mlp.gate.weight"], dtypes[pre + "mlp.gate.weight"] = p.router_gate, "BF16"
        tensors[pre + "mlp.gate.e_score_correction_bias"] = p.router_bias

        def put(base, m):
            if m.kind == "fp8":
                tensors[base], dtypes[base] = m.payload, "F8_E4M3"
                tensors[base + "_scale_inv"] = m.scales
            else:
                tensors[base + "_packed"] = m.payload
                tensors[base + "_scale"], dtypes[base + "_scale"] = m.scales, "F8_E4M3"
                tensors[base + "_global_scale"] = m.glob
        for e, mats in enumerate(p.experts):
            for m, proj in zip(mats, PROJ):
                put(f"{pre}mlp.experts.{e}.{proj}.weight", m)
        if p.shared:
            for m, proj in zip(p.shared, PROJ):
                put(f"{pre}mlp.shared_experts.{proj}.weight", m)
        return pre, tensors, dtypes
    if family == "mimo":
        pre = "model.layers.2.mlp."
        tensors[pre + "gate.weight"], dtypes[pre + "gate.weight"] = p.router_gate, "BF16"
        tensors[pre + "gate.e_score_correction_bias"] = p.router_bias
        for e, mats in enumerate(p.experts):
            for m, proj in zip(mats, PROJ):
                tensors[f"{pre}experts.{e}.{proj}.weight"] = m.payload
                tensors[f"{pre}experts.{e}.{proj}.weight_scale"] = m.scales
        return pre, tensors, dtypes
    pre = "language_model.model.layers.4.block_sparse_moe."
    tensors[pre + "gate.weight"] = hg.bf16_to_f32(p.router_gate)
    tensors[pre + "e_score_correction_bias"] = p.router_bias
    for e, mats in enumerate(p.experts):
        for m, w in zip(mats, ("w1", "w3", "w2")):
            tensors[f"{pre}experts.{e}.{w}.weight_packed"] = m.payload
            tensors[f"{pre}experts.{e}.{w}.weight_scale"], dtypes[f"{pre}experts.{e}.{w}.weight_scale"] = m.scales, "F8_E4M3"
            tensors[f"{pre}experts.{e}.{w}.weight_global_scale"] = np.float32(m.glob[0])
    if p.shared:
        for m, proj in zip(p.shared, PROJ):
            base = f"{pre}shared_experts.{proj}.weight"
            tensors[base], dtypes[base] = m.payload, "F8_E4M3"
            tensors[base + "_scale_inv"] = m.scales
    return pre, tensors, dtypes


RESIDENT_CASES = [
    # family, kind, shared kind, E, H, I, shared I, K, T, world
    ("glm", "fp8", "fp8", 8, 512, 128, 256, 2, 3, 1),
    ("glm", "fp8", "fp8", 6, 512, 256, 256, 2, 4, 2),       # slices of 128: views of the grid as it is
    ("glm", "fp8", None, 8, 512, 384, 0, 2, 3, 2),          # slices of 192: rank 1's grids re-blocked at 64
    ("glm", "nvfp4", None, 8, 512, 256, 0, 4, 5, 2),
    ("mimo", "mxfp4", None, 12, 1024, 512, 0, 8, 6, 4),
    ("minimax", "nvfp4", "mxfp8", 6, 512, 128, 192, 2, 5, 1),
    ("minimax", "nvfp4", "mxfp8", 6, 512, 128, 192, 2, 5, 2),
]


@pytest.mark.parametrize("family,kind,shared,E,H,I,sI,K,T,world", RESIDENT_CASES)
def test_resident_layer_from_a_bound_checkpoint_is_bitwise_the_hand_sliced_layer(gpu, tmp_path, family, kind, shared, E, H, I, sI,
                                                                                 K, T, world):
    """One call from a family's binding to a layer on the device (the reference's resident build of a MoE layer,
    src/models/glm/loader.cpp:418-471): every rank's layer gives the bits of the layer built by hand from the same
    slices (rows of gate / up, columns of down, cut with the loader's slice functions and uploaded one by one)."""
    from test_gpu_moe_tp_slices import cols_slice, rows_slice
    p = moe_data.make_problem(E, H, I, K, T, kind, 7100 + E + world, shared_kind=shared, shared_I=sI or None, limit=7.0, std=0.05)
    pre, tensors, dtypes = _checkpoint_tensors(p, family)
    names = sorted(tensors)
    paths = []
    for i in range(2):
        paths.append(str(tmp_path / f"model-0000{i + 1}-of-00002.safetensors"))
        write_checkpoint(paths[-1], {n: np.asarray(tensors[n]) for n in names[i::2]}, dtypes)
    mode = 0
    cfg = L.make_config(H, I, E, K, n_shared_experts=1 if shared else 0, routed_scaling_factor=2.5, swiglu_limit=p.limit, router_mode=mode)
    files = [LD.SafetensorsFile(x) for x in paths]
    layers = []
    try:
        if family == "glm":
            rw, rb, sh, routed = LD.glm_moe_bind_layer(files, pre, E, H, I, LD.BIND_FP8 if kind == "fp8" else LD.BIND_NVFP4, sI)
        elif family == "mimo":
            (rw, rb, routed), sh = LD.mimo_moe_bind_layer(files, pre, E, H, I), None
        else:
            rw, rb, sh, routed = LD.minimax_moe_bind_layer(files, pre, E, H, I, sI)
            rw = None   # this family's router weight is F32: the scores come from the caller
        for r in range(world):
            layers.append(ML.ResidentMoeLayer(cfg, T, routed, shared=sh, shared_inter=sI, router_weight=rw, router_bias=rb,
                                              rank=r, world=world))
        with pytest.raises(L.InvalidArgument):
            ML.ResidentMoeLayer(cfg, T, routed, shared=sh, shared_inter=sI, router_weight=rw, router_bias=rb, rank=world, world=world)
        with pytest.raises(L.InvalidArgument):
            ML.ResidentMoeLayer(cfg, T, routed, shared=sh, shared_inter=sI, rank=0, world=7)
        # a description whose byte counts do not cover the matrix its shape describes is refused before any copy
        for field in ("scales", "payload"):
            info = getattr(routed[1][0], field)
            kept = info.nbytes
            info.nbytes = kept - 1
            try:
                with pytest.raises(L.InvalidArgument, match="byte count"):
                    ML.ResidentMoeLayer(cfg, T, routed, shared=sh, shared_inter=sI, router_weight=rw, router_bias=rb, rank=0, world=world)
            finally:
                info.nbytes = kept
    finally:
        for f in files:
            f.close()   # the resident layers own device copies: the shards may go
    ids, w, _, _ = moe_data.orc_router(p, mode, 2.5, True)
    ids_d, w_d, x_d = dev(ids), dev(w), dev(p.x)
    M, SM = I // world, (sI // world if shared else 0)
    for r, layer in enumerate(layers):
        assert layer.inter == M and layer.weight_bytes > 0
        q = moe_data.MoeProblem(E, H, M, K, T, kind, shared, SM, limit=p.limit)
        q.x, q.router_gate, q.router_bias = p.x, p.router_gate, p.router_bias

        def rows(m, width):
            if world == 1:
                return m
            if m.kind == "fp8" and (r * width) % 128 != 0:
                whole = LD.QuantMatrix(m.payload.ctypes.data, m.scales.ctypes.data, None, m.rows, m.cols, 128, 128)
                payload, scales, v = LD.quant_slice(whole, 0, r * width, width)
                ok, rs, cs = LD.quant_scale_shifts(v)
                assert ok
                return moe_data.Mat("fp8", width, m.cols, payload, scales, rs=rs, cs=cs)
            if m.kind == "mxfp8":
                return moe_data.Mat("mxfp8", width, m.cols, np.ascontiguousarray(m.payload[r * width:(r + 1) * width]),
                                    np.ascontiguousarray(m.scales[r * width:(r + 1) * width]), rs=0, cs=5)
            return rows_slice(m, r * width, width)

        def cols(m, width):
            if world == 1:
                return m
            if m.kind == "mxfp8":
                c0 = r * width
                return moe_data.Mat("mxfp8", m.rows, width, np.ascontiguousarray(m.payload[:, c0:c0 + width]),
                                    np.ascontiguousarray(m.scales[:, c0 // 32:(c0 + width) // 32]), rs=0, cs=5)
            return cols_slice(m, r * width, width)
        for g, u, dn in p.experts:
            q.experts.append([rows(g, M), rows(u, M), cols(dn, M)])
        out_r, out_h = dev_empty((T, H), np.uint16), dev_empty((T, H), np.uint16)
        if shared == "mxfp8":
            q.shared = [rows(p.shared[0], SM), rows(p.shared[1], SM), cols(p.shared[2], SM)]
            d = DeviceMoe(moe_data.MoeProblem(E, H, M, K, T, kind, None, M, experts=q.experts, x=p.x, limit=p.limit))
            views = list((L.MoeExpertView * (d.views.numel() // 96)).from_buffer_copy(bytes(host(d.views))))
            shd = [(dev(m.payload), dev(m.scales)) for m in q.shared]
            cfg_r = L.make_config(H, M, E, K, n_shared_experts=1, routed_scaling_factor=2.5, swiglu_limit=p.limit, router_mode=mode)
            hand = ML.MoeLayer(cfg_r, ML.EXPERTS_NVFP4, views, T, shared_inter=SM, sh_payload=[t[0] for t in shd],
                               sh_scales_e8m0=[t[1] for t in shd])
        else:
            if shared:
                q.shared = [rows(p.shared[0], SM), rows(p.shared[1], SM), cols(p.shared[2], SM)]
            d = DeviceMoe(q)
            hand = make_layer(q, d, mode, 2.5, T)
        hand.enqueue_decode_routed(x_d, H, ids_d, w_d, out_h, T)
        layer.enqueue_decode_routed(x_d, H, ids_d, w_d, out_r, T)
        sync()
        assert np.array_equal(host(out_r, np.uint16), host(out_h, np.uint16)), f"rank {r}"
        assert host(out_h, np.uint16).any()
        if family != "minimax":   # the router came along: the whole step from the hidden rows
            out_r.zero_()
            hand.enqueue_decode(x_d, H, out_h, T)
            layer.enqueue_decode(x_d, H, out_r, T)
            sync()
            assert np.array_equal(host(out_r, np.uint16), host(out_h, np.uint16)), f"rank {r}: with the router"
        hand.close()
        layer.close()
