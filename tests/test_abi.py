"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every symbol include/spamm.h declares, and reports errors instead of computing."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "spamm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(spamm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = _declared_symbols()
    for must in ("spamm_create", "spamm_destroy", "spamm_multiply", "spamm_normmap_f32", "spamm_gate",
                 "spamm_gemm_gated", "spamm_get_mask", "spamm_get_counts", "spamm_get_klist",
                 "spamm_get_normmap", "spamm_strerror", "spamm_multiply_noalloc"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    import cuspamm_amd as sp
    L = sp.load_library()
    for name in _declared_symbols():
        assert hasattr(L, name), name
    assert L.spamm_version() >= 100


def test_dev_library_is_separate_from_the_engine():
    # measurement aids live in a library of their own: the engine exports no probe, and the aid's
    # header declares exactly what its library exports
    import cuspamm_amd as sp
    from cuspamm_amd import dev
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "spamm_dev.h")).read(), flags=re.S)
    syms = sorted(set(re.findall(r"\b(spamm_dev_[a-z0-9_]+)\s*\(", text)))
    assert syms == ["spamm_dev_mfma_ceiling", "spamm_dev_read_reference"]
    D = dev.load_dev_library()
    for name in syms:
        assert hasattr(D, name), name
    L = sp.load_library()
    assert not hasattr(L, "spamm_mfma_ceiling") and not hasattr(L, "spamm_dev_mfma_ceiling")
    assert D.spamm_dev_read_reference(0, 9, None) == -1
    assert D.spamm_dev_mfma_ceiling(0, 0, 0, None, None) == -1        # bad arguments: refused before any device call


def test_option_values_match_header():
    from cuspamm_amd import api
    text = open(os.path.join(ROOT, "include", "spamm.h")).read()
    opts = dict(re.findall(r"#define\s+SPAMM_(OPT_[A-Z_]+)\s+(\d+)", text))
    assert set(opts) == {"OPT_NUM_XCD", "OPT_GATE_CHUNK_WORDS", "OPT_GEMM_RING", "OPT_GEMM_SHAPE"}
    for name, value in opts.items():
        assert getattr(api, name) == int(value), name
    L = api.load_library()
    assert L.spamm_set_option(None, 1, 8) == -1


def test_engine_reads_no_environment_variables():
    # tuning goes through spamm_set_option on a context, never through process-wide state
    csrc = os.path.join(ROOT, "cuspamm_amd", "csrc")
    for f in os.listdir(csrc):
        if f.endswith((".hip", ".h")):
            assert "getenv" not in open(os.path.join(csrc, f)).read(), f


class _RecordingLib:
    """Stands in for the loaded library: any entry point called is recorded (and none should be)."""
    def __init__(self):
        self.calls = []

    def __getattr__(self, name):
        def f(*a):
            self.calls.append(name)
            return 0
        return f


def test_wrapper_refuses_a_short_c_before_any_launch():
    # the GEMM writes M x N floats through C's pointer: a smaller C must never reach the library
    import torch
    from cuspamm_amd import api
    ctx = object.__new__(api.SpammContext)
    ctx._lib, ctx._h, ctx._shape = _RecordingLib(), ctypes.c_void_p(1), None
    A, B = torch.zeros((128, 64)), torch.zeros((64, 256))
    for bad_c in (torch.zeros((128, 128)), torch.zeros((64, 256)), torch.zeros(128 * 256), torch.zeros((1, 128, 256))):
        with pytest.raises(ValueError):
            ctx.multiply(A, B, 64, 0.0, C=bad_c)
        with pytest.raises(ValueError):
            ctx.multiply_noalloc(A, B, 64, 0.0, bad_c)
    with pytest.raises(ValueError):
        ctx.multiply_noalloc(torch.zeros(128), B, 64, 0.0, torch.zeros((128, 256)))
    with pytest.raises(ValueError):
        ctx.multiply(A, torch.zeros((32, 256)), 64, 0.0)
    assert ctx._lib.calls == []
    ctx._h = ctypes.c_void_p()            # nothing to destroy


def test_struct_layout_matches_header():
    import cuspamm_amd as sp
    assert ctypes.sizeof(sp.SpammParams) == 40
    assert sp.SpammParams.tile.offset == 24 and sp.SpammParams.tau.offset == 28
    assert ctypes.sizeof(sp.SpammStats) == 40


def test_flag_values_match_header():
    from cuspamm_amd import api
    text = open(os.path.join(ROOT, "include", "spamm.h")).read()
    flags = dict(re.findall(r"#define\s+SPAMM_(FLAG_[A-Z_]+)\s+(\d+)u", text))
    assert set(flags) == {"FLAG_A_EQ_B", "FLAG_TIMING", "FLAG_REUSE_A", "FLAG_REUSE_B", "FLAG_PRUNE"}
    for name, value in flags.items():
        assert getattr(api, name) == int(value), name


def test_noalloc_workspace_size_matches_header():
    from cuspamm_amd import api
    text = open(os.path.join(ROOT, "include", "spamm.h")).read()
    m = re.search(r"#define\s+SPAMM_NOALLOC_WORKSPACE_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", text)
    assert m and (int(m.group(1)) << int(m.group(2))) == api.NOALLOC_WORKSPACE_BYTES
    assert api.ELIMIT == int(re.search(r"#define\s+SPAMM_ELIMIT\s+\((-\d+)\)", text).group(1))


def test_error_strings():
    import cuspamm_amd as sp
    L = sp.load_library()
    seen = set()
    for code in (0, -1, -2, -3, -4, -5, -6):
        s = L.spamm_strerror(code).decode()
        assert s and s != "unknown error"
        seen.add(s)
    assert len(seen) == 7
    assert L.spamm_strerror(-99).decode() == "unknown error"


def test_null_arguments_are_rejected_without_a_device():
    import cuspamm_amd as sp
    L = sp.load_library()
    assert L.spamm_create(None, 0) == -1
    assert L.spamm_destroy(None) == -1
    assert L.spamm_gate(None, 0.0) == -1
    assert L.spamm_multiply(None, None, None, None, None) == -1
    assert L.spamm_multiply_noalloc(None, None, None, None, None) == -1


def test_create_without_gpu_reports_no_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    import cuspamm_amd as sp
    with pytest.raises(sp.SpammError) as ei:
        sp.SpammContext(0)
    assert ei.value.code == -5


def test_command_line_driver_is_built_and_checks_its_arguments():
    # argument errors are reported before any device call, so this runs without a GPU
    import subprocess
    main = os.path.join(ROOT, "cuspamm_amd", "spamm_main")
    assert os.path.exists(main), "build it with `python -m cuspamm_amd.build`"
    for args, msg in ((["--tile", "48"], "tile must be"), (["--nonsense"], "unknown option"),
                      (["--testtime", "3", "--warmup", "5"], "bad sizes"),
                      (["--check", "--prune"], "complete fp16 copy")):
        proc = subprocess.run([main] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
        assert proc.returncode == 2 and msg in proc.stdout, proc.stdout


def test_missing_library_fails_loudly():
    # no CPU or PyTorch fallback: without the built HIP library the package refuses to work
    import subprocess
    import sys
    code = ("import cuspamm_amd as sp\n"
            "try:\n    sp.load_library()\nexcept ImportError as e:\n    print('refused:', e)\n")
    env = dict(os.environ, SPAMM_LIBRARY_PATH="/nonexistent/libspamm_gfx950.so")
    proc = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and "refused:" in proc.stdout and "no CPU or PyTorch fallback" in proc.stdout, proc.stdout


def test_product_package_never_imports_the_oracle():
    # the checker is test infrastructure: nothing under cuspamm_amd/ may reference it
    pkg = os.path.join(ROOT, "cuspamm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
