"""The C-ABI library loads without a GPU and exports every symbol that
include/offload_adam_hip.h declares; the ctypes table covers the same set.
No compute entry point is called here.
"""

import ctypes
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "offload_adam_hip.h"


def declared_symbols():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)  # drop comments
    return sorted(set(re.findall(r"\b(oa_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    syms = declared_symbols()
    assert "oa_adam_fp32_master" in syms and "oa_abi_version" in syms
    assert len(syms) >= 17


def test_library_exports_every_declared_symbol():
    from offload_adam_amd import _lib

    assert _lib.LIB_PATH.exists(), "build with `python -m offload_adam_amd._build`"
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_ctypes_table_matches_header():
    from offload_adam_amd import _lib

    assert sorted(_lib.SIGNATURES) == declared_symbols()


def test_version_and_error_strings():
    from offload_adam_amd import _lib

    lib = _lib.load()
    assert lib.oa_abi_version() == 1
    assert "success" in _lib.error_string(0)
    for code in (-1, -2, -3, -4):
        assert "offload_adam_hip" in _lib.error_string(code)
    assert _lib.error_string(1)  # a hipError_t gets the runtime's text
    assert lib.oa_norm_workspace_bytes() >= 4096 + 64


def test_argument_validation_needs_no_gpu():
    """Rejected arguments return an OA_E* code before anything is launched."""
    from offload_adam_amd import _lib

    lib = _lib.load()
    assert lib.oa_adam_fp32_master(None, None, None, None, None, 8, 0, 0, 0, 0, 0, 0, None, None) == -1
    assert lib.oa_adam_stochastic_rounding(None, None, None, None, 8, 0, 0, 0, 0, 0, 0, 0, 7, None,
                                           None, None) == -1  # bad rng enum
    assert lib.oa_adam_fp31_master(None, None, None, None, None, -5, 0, 0, 0, 0, 0, 0, None, None) == -1
    buf = (ctypes.c_char * 64)()
    base = ctypes.addressof(buf)
    odd = ctypes.c_void_p(base + 1)
    ok = ctypes.c_void_p(base)
    assert lib.oa_adam_fp32_master(odd, ok, ok, ok, ok, 8, 0, 0, 0, 0, 0, 0, None, None) == -2
    assert lib.oa_grad_norm_bf16(ok, 4, None, None, None, None) == -1
    assert lib.oa_quant_int4(ok, 0, 128, 1, 128, 100, ok, ok, 1, None) == -1  # group % 8
    assert lib.oa_quant_nvfp4(ok, 0, 24, 1, 24, ok, ok, ok, ok, None) == -1  # cols % 16
    assert lib.oa_dequant_int8(ok, ok, 9, 1, 8, ok, 1, 8, None) == -1  # bad dtype enum


def test_the_product_never_reaches_the_oracle():
    """The CPU restatement is test infrastructure: nothing in the package, and no
    benchmark program outside its CPU-baseline leg, imports it."""
    import ast

    def oracle_imports(path):
        found = []
        tree = ast.parse(path.read_text())
        for node in ast.walk(tree):
            names = []
            if isinstance(node, ast.Import):
                names = [a.name for a in node.names]
            elif isinstance(node, ast.ImportFrom) and node.level == 0:
                names = [node.module or ""]
            found += [(n, node.lineno) for n in names if n.split(".")[0] == "oracle"]
        return found

    for path in sorted((ROOT / "offload_adam_amd").rglob("*.py")):
        assert oracle_imports(path) == [], path
    assert oracle_imports(ROOT / "bench_e2e.py") == []
    assert oracle_imports(ROOT / "bench_kernels.py") == []
    # bench.py: only inside the functions of its CPU-baseline leg
    tree = ast.parse((ROOT / "bench.py").read_text())
    allowed = {"cpu_baseline", "cpu_baselines_of_the_other_kernels", "cpu_adam_inputs"}
    for fn in [n for n in tree.body if isinstance(n, ast.FunctionDef)]:
        uses = [n for n in ast.walk(fn)
                if isinstance(n, (ast.Import, ast.ImportFrom))
                and any((getattr(n, "module", None) or a.name).split(".")[0] == "oracle"
                        for a in n.names)]
        assert not uses or fn.name in allowed, fn.name
    top = [n for n in tree.body if isinstance(n, (ast.Import, ast.ImportFrom))]
    assert all((getattr(n, "module", None) or n.names[0].name).split(".")[0] != "oracle"
               for n in top)


def test_a_missing_library_fails_loudly(tmp_path):
    """No fallback: with the kernel library absent every operator raises."""
    import subprocess
    import sys

    code = (
        "import offload_adam_amd._lib as L\n"
        "try:\n"
        "    L.load()\n"
        "except L.LibraryNotBuiltError as e:\n"
        "    print('raised', type(e).__name__)\n"
    )
    import os

    env = dict(os.environ, OFFLOAD_ADAM_HIP_LIB=str(tmp_path / "absent.so"),
               OFFLOAD_ADAM_COPY_ENGINES="off")
    r = subprocess.run([sys.executable, "-c", code], cwd=str(ROOT), env=env,
                       capture_output=True, text=True, timeout=300)
    assert "raised LibraryNotBuiltError" in r.stdout, r.stdout + r.stderr
