"""The HSA tools library that fixes the SDMA engine per copy direction
(include/offload_adam_copy_engines.h, csrc/hsa_tool/copy_engine_pin.cpp)."""

import ctypes
import os
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "offload_adam_copy_engines.h"


def declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(oa_copy_engines_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_header_symbols_and_tool_entry_points():
    from offload_adam_amd import _copy_engines

    assert _copy_engines.LIB_PATH.exists(), "build with `python -m offload_adam_amd._build`"
    lib = ctypes.CDLL(str(_copy_engines.LIB_PATH))
    names = declared()
    assert names == ["oa_copy_engines_active", "oa_copy_engines_config", "oa_copy_engines_loaded",
                     "oa_copy_engines_passed_by", "oa_copy_engines_register_range",
                     "oa_copy_engines_scoped", "oa_copy_engines_stats",
                     "oa_copy_engines_unpinned_calls", "oa_copy_engines_unregister_range"]
    for name in names + ["OnLoad", "OnUnload"]:
        assert hasattr(lib, name), name


def test_status_without_runtime_reports_not_loaded():
    from offload_adam_amd import _copy_engines

    st = _copy_engines.status()
    if st["loaded"]:
        pytest.skip("a GPU runtime is up in this process")
    assert st["active"] is False
    assert (st["h2d_engine"], st["d2h_engine"]) == (1, 2)
    assert st["h2d_copies"] == st["d2h_copies"] == st["rejected"] == 0


def test_range_registry_in_a_process_of_its_own():
    """Registering switches the library to its scoped mode; bases are unique keys."""
    code = (
        "import ctypes; from offload_adam_amd import _copy_engines as c\n"
        "lib = c._lib(); lib.oa_copy_engines_scoped.restype = ctypes.c_int\n"
        "a = lib.oa_copy_engines_scoped()\n"
        "r = [lib.oa_copy_engines_register_range(ctypes.c_void_p(0x10000), 4096),\n"
        "     lib.oa_copy_engines_register_range(ctypes.c_void_p(0x10000), 8192),\n"
        "     lib.oa_copy_engines_register_range(ctypes.c_void_p(0x40000), 4096),\n"
        "     lib.oa_copy_engines_register_range(None, 4096),\n"
        "     lib.oa_copy_engines_register_range(ctypes.c_void_p(0x50000), 0)]\n"
        "u = [lib.oa_copy_engines_unregister_range(ctypes.c_void_p(0x10000)),\n"
        "     lib.oa_copy_engines_unregister_range(ctypes.c_void_p(0x10000)),\n"
        "     lib.oa_copy_engines_unregister_range(ctypes.c_void_p(0x40000))]\n"
        "print(a, r, u, lib.oa_copy_engines_scoped())")
    assert _run(code) == "0 [0, 0, 0, -1, -1] [0, -1, 0] 1"


def test_a_path_with_whitespace_is_reported_not_installed(monkeypatch, tmp_path):
    from offload_adam_amd import _copy_engines

    spaced = tmp_path / "with space" / "liboffload_adam_copy_engines.so"
    spaced.parent.mkdir()
    spaced.write_bytes(b"")
    monkeypatch.setattr(_copy_engines, "LIB_PATH", spaced)
    monkeypatch.setattr(_copy_engines, "_install_result", None)
    monkeypatch.delenv("OFFLOAD_ADAM_COPY_ENGINES", raising=False)
    before = os.environ.get("HSA_TOOLS_LIB")
    assert _copy_engines.install() == "unusable_path"
    assert os.environ.get("HSA_TOOLS_LIB") == before


def _run(code, **env):
    full = dict(os.environ)
    full.pop("HSA_TOOLS_LIB", None)
    full.pop("OFFLOAD_ADAM_COPY_ENGINES", None)
    full.update(env)
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=full,
                         cwd=str(ROOT), timeout=300)
    assert res.returncode == 0, res.stderr
    return res.stdout.strip().splitlines()[-1]


def test_import_puts_library_on_hsa_tools_lib():
    code = ("import os, offload_adam_amd; from offload_adam_amd import _copy_engines as c; "
            "print(c._install_result, os.environ.get('HSA_TOOLS_LIB'))")
    result, value = _run(code).split(" ", 1)
    assert result == "installed" and value.endswith("liboffload_adam_copy_engines.so")
    # an existing entry is kept, ours goes first
    result, value = _run(code, HSA_TOOLS_LIB="/some/other/tool.so").split(" ", 1)
    assert result == "installed"
    assert value.split()[0].endswith("liboffload_adam_copy_engines.so")
    assert value.split()[1] == "/some/other/tool.so"


def test_off_leaves_environment_alone():
    code = ("import os, offload_adam_amd; from offload_adam_amd import _copy_engines as c; "
            "print(c._install_result, os.environ.get('HSA_TOOLS_LIB'))")
    assert _run(code, OFFLOAD_ADAM_COPY_ENGINES="off") == "off None"


@pytest.mark.gpu
def test_copies_run_on_the_fixed_engines_and_move_the_right_bytes():
    import torch

    from offload_adam_amd import _copy_engines, _lib
    from offload_adam_amd.offload_adam import _copy_async
    from offload_adam_amd.pinned_alloc import zeros_pinned

    torch.cuda.init()
    st0 = _copy_engines.status()
    assert st0["loaded"] and st0["active"], st0
    n = 4 << 20
    host_in = zeros_pinned((n,), torch.int32, numa_node=None)
    host_out = zeros_pinned((n,), torch.int32, numa_node=None)
    host_in.copy_(torch.arange(n, dtype=torch.int32))
    h2d, d2h = torch.cuda.Stream(), torch.cuda.Stream()
    main = torch.cuda.current_stream()
    for rep in range(4):
        dev = torch.empty(n, dtype=torch.int32, device="cuda")
        h2d.wait_stream(main)
        _copy_async(dev, host_in, _lib.OA_COPY_H2D, h2d)
        main.wait_stream(h2d)
        dev.add_(rep)
        d2h.wait_stream(main)
        _copy_async(host_out, dev, _lib.OA_COPY_D2H, d2h)
        dev.record_stream(d2h)
        d2h.synchronize()
        assert torch.equal(host_out, host_in + rep)
    st1 = _copy_engines.status()
    assert st1["h2d_copies"] - st0["h2d_copies"] >= 4
    assert st1["d2h_copies"] - st0["d2h_copies"] >= 4
    assert st1["rejected"] == 0 and st1["active"]
    # the package's pinned buffers are registered, so the rewrite is scoped to them:
    # copies of torch's own pinned tensors keep the engine the runtime picks
    assert st1["scoped"]
    other = torch.empty(n, dtype=torch.int32).pin_memory()
    other.copy_(host_in)
    for _ in range(3):
        dev = other.to("cuda", non_blocking=True)
        back = dev.to("cpu", non_blocking=True)
        torch.cuda.synchronize()
        assert torch.equal(back, host_in)
    st2 = _copy_engines.status()
    assert st2["passed_by"] - st1["passed_by"] >= 3
    assert st2["h2d_copies"] == st1["h2d_copies"]


_LATE = (
    "import sys, warnings, torch\n"
    "torch.zeros(1, device='cuda')  # the GPU runtime starts before the package is imported\n"
    "import offload_adam_amd\n"
    "from offload_adam_amd import OffloadAdam, _copy_engines, _runtime_env\n"
    "model = torch.nn.Sequential(torch.nn.Linear(64, 64, bias=False)).to(device='cuda', dtype=torch.bfloat16)\n"
    "with warnings.catch_warnings(record=True) as caught:\n"
    "    warnings.simplefilter('always')\n"
    "    opt = OffloadAdam(model, inplace_param_threshold=0)\n"
    "    opt.ready_for_optimizer_step = True\n"
    "    model(torch.ones(4, 64, device='cuda', dtype=torch.bfloat16)).sum().backward()\n"
    "    torch.cuda.synchronize()\n"
    "st = _copy_engines.status()\n"
    "late = [w for w in caught if 'not pinned to fixed SDMA engines' in str(w.message)]\n"
    "print(st['install'], st['loaded'], st['direct'], st['direct_h2d_copies'] > 0,\n"
    "      st['direct_d2h_copies'] > 0, len(late), _runtime_env.prepare()['copy_engines'])"
)


@pytest.mark.gpu
def test_an_import_after_the_first_gpu_call_still_gets_fixed_engines():
    """``model.cuda()`` above the import - what a user of the reference writes: the
    environment edit comes too late for the tools library (``status()`` says so), but
    the optimizer's copies are put on their engines by the kernel library itself, so
    nothing is lost and nothing warns, also with OFFLOAD_ADAM_REQUIRE_COPY_ENGINES."""
    assert _run(_LATE) == "late False True True True 0 late"
    assert _run(_LATE, OFFLOAD_ADAM_REQUIRE_COPY_ENGINES="1") == "late False True True True 0 late"
    # neither way in effect and not asked to be silent about it: one warning, or an error
    neither = _LATE.replace("import offload_adam_amd\n",
                            "import offload_adam_amd\n"
                            "from offload_adam_amd import offload_adam as m\n"
                            "m._FIXED_ENGINE_COPIES = False\n"
                            "real = m._copy_engines.status\n"
                            "m._copy_engines.status = lambda: dict(real(), direct=False, "
                            "direct_reason='switched off for this test')\n")
    assert _run(neither).split()[5] == "1"
    full = dict(os.environ, OFFLOAD_ADAM_REQUIRE_COPY_ENGINES="1")
    full.pop("HSA_TOOLS_LIB", None)
    res = subprocess.run([sys.executable, "-c", neither], capture_output=True, text=True, env=full,
                         cwd=str(ROOT), timeout=300)
    assert res.returncode != 0
    assert "OFFLOAD_ADAM_REQUIRE_COPY_ENGINES is set" in res.stderr
    assert "switched off for this test" in res.stderr


@pytest.mark.gpu
def test_the_launcher_takes_the_import_order_out_of_the_script(tmp_path):
    """The same script started through ``python -m offload_adam_amd.launch``: the
    library is in effect although the script touches the GPU before its import."""
    script = tmp_path / "late_import.py"
    script.write_text(_LATE.replace("print(st['install']", "print(sys.argv[1:], st['install']"))
    full = dict(os.environ)
    full.pop("HSA_TOOLS_LIB", None)
    res = subprocess.run([sys.executable, "-m", "offload_adam_amd.launch", str(script), "--flag", "7"],
                         capture_output=True, text=True, env=full, cwd=str(ROOT), timeout=300)
    assert res.returncode == 0, res.stderr
    # (with the tools library in effect the copies are hipMemcpyAsync calls whose engine it
    # rewrites: the kernel library's own copies are available but idle)
    assert res.stdout.strip().splitlines()[-1] == "['--flag', '7'] installed True True False False 0 installed"


def test_the_launcher_prints_the_environment_for_a_shell():
    from offload_adam_amd import _copy_engines

    full = dict(os.environ, HSA_TOOLS_LIB="/some/other/tool.so")
    full.pop("GPU_MAX_HW_QUEUES", None)
    res = subprocess.run([sys.executable, "-m", "offload_adam_amd.launch", "--print-env"],
                         capture_output=True, text=True, env=full, cwd=str(ROOT), timeout=300)
    assert res.returncode == 0, res.stderr
    lines = res.stdout.strip().splitlines()
    assert lines == [f"export HSA_TOOLS_LIB='{_copy_engines.LIB_PATH} /some/other/tool.so'",
                     "export GPU_MAX_HW_QUEUES='8'"]
    # a value the user exported stands
    res = subprocess.run([sys.executable, "-m", "offload_adam_amd.launch", "--print-env"],
                         capture_output=True, text=True, env=dict(full, GPU_MAX_HW_QUEUES="6"),
                         cwd=str(ROOT), timeout=300)
    assert res.stdout.strip().splitlines()[-1] == "export GPU_MAX_HW_QUEUES='6'"


def test_roctx_ranges_are_off_by_default_and_load_on_request():
    from offload_adam_amd import _trace

    if not _trace.ENABLED:
        with _trace.range("nothing"):  # a null context
            pass
    code = ("from offload_adam_amd import _trace\n"
            "with _trace.range('outer'):\n"
            "    with _trace.range('inner'):\n"
            "        pass\n"
            "print(_trace.ENABLED)")
    assert _run(code, OFFLOAD_ADAM_ROCTX="1") == "True"
    assert _run(code) == "False"
