"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares."""
import ctypes
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol(cf):
    assert len(cf.decls) >= 25
    dll = ctypes.CDLL(str(ROOT / "canopy-foundry_amd" / "libcf_fp8.so"))
    for name in cf.decls:
        assert getattr(dll, name) is not None
    assert b"gfx950" in cf.cf_version()


def test_every_declaration_cites_the_reference():
    text = (ROOT / "include" / "cf_fp8.h").read_text()
    # each exported function is preceded (within its comment block) by a reference file:line or an explicit note
    for m in re.finditer(r"\n(?:int|const char\*) (cf_\w+)\(", text):
        head = text[: m.start()]
        block = head[head.rfind("/*"):]
        assert re.search(r"\w+\.(cu|hpp|cpp):\d+", block) or "no counterpart" in block or "identification" in block, m.group(1)


def test_missing_library_fails_loudly(tmp_path):
    import __graft_entry__ as entry
    import pytest
    pkg = entry.load_package()
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pkg.Lib(tmp_path / "libcf_fp8.so")


def test_argument_errors_do_not_need_a_gpu(cf):
    # argument validation happens before any launch
    assert cf.raw_cf_swiglu_forward(None, None, None, -1, None) == -1
    assert cf.raw_cf_swiglu_forward(None, None, None, 4, None) == -1
    assert cf.raw_cf_swiglu_forward(None, None, None, 0, None) == 0
    assert cf.raw_cf_fp8_quantize_e4m3(None, None, None, 0, None) == 0
    assert cf.raw_cf_fp8_quantize_e4m3(None, None, None, 8, None) == -1
    assert cf.raw_cf_fp8_quantize_rows(None, -1, 4, 0, None, None, None, None) == -1
    # the workspace forms of the expert bank: sizes are host arithmetic, argument checks come before any launch
    import ctypes
    n = ctypes.c_size_t(7)
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_workspace(16384, 98304, 64, 2048, 1408, None, ctypes.byref(n)) == 0
    assert 1_700_000_000 < n.value < 1_900_000_000 and n.value % 256 == 0
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_workspace(100, 200, 4, 96, 72, None, ctypes.byref(n)) == 0 and n.value == 0
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_workspace(-1, 0, 0, 0, 0, None, ctypes.byref(n)) == -1
    assert cf.raw_cf_moe_grouped_expert_forward_bf16_workspace(16384, 98304, 64, 2048, 1408, None, ctypes.byref(n)) == 0
    assert 1_500_000_000 < n.value < 1_700_000_000      # bf16 form: the GELU output travels as one bf16 term
    # the bank of per-expert delayed-scaling slots: argument checks before any launch
    assert cf.raw_cf_moe_grouped_quantize_delayed(None, None, 256, 4, None, None, 100, None, 32, 8, 0, 1, 0, None, None) == -1
    assert cf.raw_cf_moe_grouped_quantize_delayed(None, None, 256, 4, None, None, 0, None, 32, 8, 0, 1, 0, None, None) == 0
    assert cf.raw_cf_moe_grouped_quantize_delayed(None, None, -1, 4, None, None, 0, None, 32, 8, 0, 1, 0, None, None) == -1
    nul = [None] * 12
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_ws(None, None, 0, *nul[:9], 4, 256, 128, 2, 8, None, 0, None) == -1
    assert cf.raw_cf_moe_grouped_expert_forward_fp8_ws(None, None, 0, *nul[:9], 0, 256, 128, 2, 0, None, 0, None) == 0
    assert cf.raw_cf_moe_grouped_expert_forward_bf16_ws(*nul[:8], 4, 256, 128, 2, 8, None, 0, None) == -1
    assert cf.raw_cf_moe_grouped_expert_forward_bf16_ws(*nul[:8], -4, 256, 128, 2, 8, None, 0, None) == -1


def test_cpp_shim_compiles_links_and_maps_errors(tmp_path):
    """The header-only C++ shim keeps the reference's ida_native:: signatures over HIP types."""
    import subprocess
    exe = tmp_path / "shim_check"
    lib_dir = ROOT / "canopy-foundry_amd"
    cmd = ["g++", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", f"-I{ROOT / 'include'}",
           str(ROOT / "tests" / "shim_compile_check.cpp"), "-o", str(exe), f"-L{lib_dir}", "-lcf_fp8",
           f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True, capture_output=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and "shim ok 2" in out.stdout, out.stderr
