"""The C ABI library loads without a GPU and exports every symbol include/dgpp_amd.h declares."""
import ctypes
import re
from pathlib import Path
import pytest

from dgpp_amd import _lib

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols(header="dgpp_amd.h"):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dgpp_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 50
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/dgpp_amd.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)
    bench = declared_symbols("dgpp_amd_bench.h")
    assert set(bench) == set(_lib.BENCH_SIGNATURES) and not set(bench) & set(names)
    for n in bench:
        assert hasattr(lib, n), f"{n} is declared in include/dgpp_amd_bench.h but not exported"
    layer = declared_symbols("dgpp_amd_layer.h")
    assert set(layer) == set(_lib.LAYER_SIGNATURES)
    for n in layer:
        assert hasattr(lib, n), f"{n} is declared in include/dgpp_amd_layer.h but not exported"
    from dgpp_amd import loader
    loader_names = declared_symbols("dgpp_amd_loader.h")
    assert set(loader_names) == set(loader.SIGNATURES)
    for n in loader_names:
        assert hasattr(lib, n), f"{n} is declared in include/dgpp_amd_loader.h but not exported"
    assert lib.dgpp_target_arch() == b"gfx950"


def test_struct_layouts_match_the_reference_abi():
    V = _lib.MoeExpertView
    assert ctypes.sizeof(V) == 96
    offs = {f: getattr(V, f).offset for f in ("payload", "scales", "fp4_scales", "fp4_global", "scale_shift_rows",
                                              "scale_shift_cols", "fp4_group")}
    assert offs == {"payload": 0, "scales": 8, "fp4_scales": 16, "fp4_global": 24, "scale_shift_rows": 32,
                    "scale_shift_cols": 36, "fp4_group": 40}
    assert ctypes.sizeof(_lib.MoeSegment) == 12 and ctypes.sizeof(_lib.MoeTile) == 8
    assert ctypes.sizeof(_lib.Fp4Matrix) == 56 and _lib.Fp4Matrix.scale_group.offset == 40


def test_host_side_argument_checks_need_no_gpu():
    from dgpp_amd import launch as L
    import pytest
    cfg = L.make_config(64, 64, 8, 9)            # top_k > n_experts
    with pytest.raises(L.InvalidArgument):
        L.validate_config(cfg)
    with pytest.raises(L.InvalidArgument):
        L.validate_config(L.make_config(64, 64, 8, 17))
    L.validate_config(L.make_config(4096, 1024, 256, 8, n_shared_experts=0, router_mode=L.ROUTER_SOFTMAX_TOPK))
    assert L.moe_tile_list_capacity(5, 33, 16) == 5 + 3 and L.moe_run_groups_max(72) == 72 // 17 + 1
    w = L.Fp4Matrix(0x1000, 0x2000, None, 8, 1024, 16, 0, None)
    assert not L.fp4_gemv_accepts(w)            # NVFP4 without a global
    w.scale_group = 32
    assert L.fp4_gemv_accepts(w)
    w.cols = 3072
    assert not L.fp4_gemv_accepts(w)            # not in the MXFP4 set
    assert L.fp8_gemv_can_stage(0x1000, 4096) and not L.fp8_gemv_can_stage(0x1001, 4096)
    with pytest.raises(L.InvalidArgument):      # null pointers are refused before any launch
        L.launch_moe_segment(None, 4, 8, 16, None, None, None)
    L.launch_moe_segment(None, 0, 8, 16, None, None, None)      # tokens <= 0 returns silently


def test_headers_compile_as_c_and_the_shim_as_cpp(tmp_path):
    """include/dgpp_amd.h and dgpp_amd_layer.h are plain C; dgpp_amd.hpp (the reference's names) is C++17
    and links against the library without running anything."""
    import shutil
    import subprocess
    root = Path(__file__).resolve().parent.parent
    inc = root / "include"
    c_src = tmp_path / "c_check.c"
    c_src.write_text('#include "dgpp_amd.h"\n#include "dgpp_amd_layer.h"\n#include "dgpp_amd_loader.h"\n#include "dgpp_amd_bench.h"\n'
                     "int main(void) { return sizeof(DgppMoeExpertView) == 96 && sizeof(DgppTensorInfo) == 104 ? 0 : 1; }\n")
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-I", str(inc), "-c", str(c_src), "-o", str(tmp_path / "c.o")],
                   check=True)
    rocm_inc = Path("/opt/rocm/include")
    if not (shutil.which("g++") and rocm_inc.exists()):
        pytest.skip("no g++ / ROCm headers")
    cpp_src = tmp_path / "shim_check.cpp"
    cpp_src.write_text('#include "dgpp_amd.hpp"\n#include "dgpp_amd_layer.h"\n'
                       "int main() { return dgpp::moe_tile_list_capacity(1, 1, 16) > 0 ? 0 : 1; }\n")
    subprocess.run(["g++", "-std=c++17", "-Wall", "-I", str(inc), "-I", str(rocm_inc), "-D__HIP_PLATFORM_AMD__",
                    str(cpp_src), "-L", str(root / "dgpp_amd" / "lib"), "-ldgpp_amd", "-L/opt/rocm/lib", "-lamdhip64",
                    "-o", str(tmp_path / "shim_check")], check=True)


def test_layer_scratch_bytes_covers_what_the_layer_stages():
    """dgpp_moe_layer_scratch_bytes (reference: GlmMoeLayer::scratch_bytes, src/models/glm/moe_layer.cpp:72-129) is a
    host computation: at least the expert table, the slot activations and the unrounded slot outputs, and it grows
    with the token count and with a shared expert."""
    from dgpp_amd import launch as L, moe_layer as ML
    E, H, I, K = 256, 4096, 1024, 8
    cfg = L.make_config(H, I, E, K, n_shared_experts=0, router_mode=L.ROUTER_SOFTMAX_TOPK)
    sizes = [ML.scratch_bytes(cfg, t) for t in (1, 8, 64)]
    assert sizes[0] < sizes[1] < sizes[2]
    for t, s in zip((1, 8, 64), sizes):
        floor = E * 3 * 96 + t * (K + 1) * I * 2 + t * (K + 1) * H * 4 + t * K * 8
        assert floor <= s < 64 * floor
    cfg_sh = L.make_config(H, I, E, K, n_shared_experts=1, router_mode=L.ROUTER_SOFTMAX_TOPK)
    assert ML.scratch_bytes(cfg_sh, 8, 2048) > ML.scratch_bytes(cfg_sh, 8, 1024) >= sizes[1]


def test_slot_ex_launchers_refuse_what_they_cannot_honour():
    """The *_ex decode-slot launchers never drop a request silently: a pass selector outside 1..3, the shared pass
    alone without a shared expert, an accumulation target without both of its arguments or without the shared pass
    that would write it are all invalid arguments, raised before anything is launched (no GPU needed)."""
    from dgpp_amd import launch as L
    fake = 0x10000      # non-null, 16-byte aligned; never dereferenced: every call below is refused on the host
    base = dict(n_routed=128, k_routed=256, slots=9, top_k=8)

    def gate_up(n_shared, passes):
        L.launch_moe_slot_gate_up_swiglu_ex(fake, 256, fake, None, fake, base["n_routed"], base["k_routed"], n_shared,
                                            256 if n_shared else 0, fake, fake, fake, fake, fake, 128, base["slots"],
                                            base["top_k"], 10.0, None, 7, 7, passes)

    def down(n_shared, passes, acc_w, acc_o, fp4=False):
        if fp4:
            L.launch_moe_slot_down_fp4_ex(fake, 128, fake, None, fake, 256, 128, n_shared, 128 if n_shared else 0, fake, fake,
                                          fake, 256, base["slots"], base["top_k"], None, -1, 32, 7, 7, fake, passes, acc_w, acc_o)
        else:
            L.launch_moe_slot_down_ex(fake, 128, fake, None, fake, 256, 128, n_shared, 128 if n_shared else 0, fake, fake, fake,
                                      256, base["slots"], base["top_k"], None, 7, 7, passes, acc_w, acc_o)

    for bad in (0, 4, -1):
        with pytest.raises(L.InvalidArgument):
            gate_up(128, bad)
        with pytest.raises(L.InvalidArgument):
            down(256, bad, None, None)
    with pytest.raises(L.InvalidArgument):
        gate_up(0, 2)                                # the shared pass alone, no shared expert
    for fp4 in (False, True):
        with pytest.raises(L.InvalidArgument):
            down(0, 2, None, None, fp4)
        with pytest.raises(L.InvalidArgument):
            down(256, 3, fake, None, fp4)            # weights without an output row
        with pytest.raises(L.InvalidArgument):
            down(256, 3, None, fake, fp4)
        with pytest.raises(L.InvalidArgument):
            down(256, 1, fake, fake, fp4)            # the accumulation rides the shared pass, which is not run
        with pytest.raises(L.InvalidArgument):
            down(0, 3, fake, fake, fp4)              # ... or does not exist


def test_measurement_switches_are_inert_unless_the_process_opted_in():
    """dgpp_tune_set steers launcher choices for the benchmark and the form-comparison tests. A process that did not
    ask for that (no DGPP_AMD_BENCH=1 in its environment when the library is first asked) keeps every switch at 0
    whatever is called; one that did gets what it sets."""
    import os
    import subprocess
    import sys
    code = ("import ctypes, sys; lib = ctypes.CDLL(sys.argv[1]); lib.dgpp_tune_set(12, 2); lib.dgpp_tune_set(5, 1); "
            "print(lib.dgpp_tune_enabled(), lib.dgpp_tune_get(12), lib.dgpp_tune_get(5))")
    path = str(_lib.LIB_PATH)
    env = {k: v for k, v in os.environ.items() if k != "DGPP_AMD_BENCH"}
    off = subprocess.run([sys.executable, "-c", code, path], env=env, capture_output=True, text=True, check=True)
    assert off.stdout.split() == ["0", "0", "0"]
    env["DGPP_AMD_BENCH"] = "1"
    on = subprocess.run([sys.executable, "-c", code, path], env=env, capture_output=True, text=True, check=True)
    assert on.stdout.split() == ["1", "2", "1"]
