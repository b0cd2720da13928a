"""Host-side checks that need no GPU: the shared library loads and exports every symbol the
header declares, argument validation returns error codes instead of aborting, and the getp hook
file compiles inside the reference's translation unit where that tree is present."""
import ctypes as C
import os
import re
import subprocess

import pytest

from conftest import ROOT, load_pkg

HEADER = os.path.join(ROOT, "include", "gptoss_mi355.h")
REF = "/root/reference"


@pytest.fixture(scope="module")
def lib():
    return load_pkg("lib")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gptoss_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    L = C.CDLL(lib.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    # and the ctypes table binds exactly the declared set
    assert sorted(lib.SIGNATURES) == names


def test_no_oracle_or_cpu_fallback_in_product(lib):
    """The shipped package must not reach into oracle/ and must fail loudly without its library."""
    pkg_dir = os.path.dirname(lib.LIB_PATH)
    for root, _, files in os.walk(pkg_dir):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                src = open(os.path.join(root, f)).read()
                assert "oracle" not in src.lower(), f"{f} mentions the oracle"
    import importlib
    import unittest.mock as mock
    with mock.patch.object(lib, "LIB_PATH", "/nonexistent/libgptoss_mi355.so"), \
            mock.patch.object(lib, "_lib", None):
        with pytest.raises(ImportError):
            lib.load()


def test_argument_validation_without_gpu(lib):
    L = lib.load()
    assert L.gptoss_abi_version() == 101
    # null pointers and bad dimensions are rejected before anything touches a device
    assert L.gptoss_router_gemm(None, None, None, None, 4, 256, 8, None) == 1
    assert "null" in lib.last_error()
    buf = (C.c_char * 4096)()
    p = C.cast(buf, C.c_void_p)
    assert L.gptoss_router_gemm(p, p, None, p, 4, 250, 8, None) == 2          # H % 32
    assert L.gptoss_moe_route(p, 4, 300, 4, p, p, p, p, p, None, 0, None) == 2  # E > 256
    assert L.gptoss_moe_route(p, 4, 32, 9, p, p, p, p, p, None, 0, None) == 2   # k > 8
    assert L.gptoss_moe_route(p, 4, 32, 4, p, p, p, p, p, p, 100, None) == 2     # odd tile size
    assert L.gptoss_pack_weight(p, p, 1, 48, 64, 0, None) == 2                # n_out % 32
    assert L.gptoss_pack_weight(p, p, 1, 32, 100, lib.PACK_GLU, None) == 2    # n_in % 64
    assert L.gptoss_kv_cache_write(p, p, p, 1, 2, 48, 64, 0, 1, None) == 2  # head_dim
    assert L.gptoss_attn_decode(p, p, p, None, p, 1, 8, 3, 64, 64, 0, 10, p, 1 << 20, None) == 2
    w = lib.MoeWeights(32, 4, 2880, 2880, 7.0, p.value, p.value, p.value, p.value, p.value, p.value)
    assert L.gptoss_moe_forward(C.byref(w), p, 8, p, 0, None, 0, None) == 4   # no workspace
    assert "workspace" in lib.last_error()
    w.hidden = 100
    assert L.gptoss_moe_forward(C.byref(w), p, 8, p, 0, p, 1 << 30, None) == 2
    # size queries are pure functions
    assert L.gptoss_packed_weight_bytes(32, 5760, 2880) == 32 * 5760 * 2880 * 2
    assert L.gptoss_kv_cache_bytes(256, 8, 64, 4096) == 256 * 8 * 64 * 4096 * 2 * 2
    assert L.gptoss_moe_max_tiles(1024, 4, 32, 256) == 16 + 32
    assert L.gptoss_moe_workspace_bytes(1024, 32, 4, 2880, 2880) > 4096 * 2880 * 6
    assert L.gptoss_attn_workspace_bytes(256, 64, 8, 64, 4096) > 0
    cfg = lib.Config(4096, 256, 8, 4, 256, 4, 48, 8, 2, 64, 4096, 150000.0, 32.0, 128, 7.0)
    h = C.c_void_p()
    assert L.gptoss_engine_create(C.byref(cfg), p, 2, 16, 0, 0, C.byref(h)) == 2   # head_dim 48
    assert L.gptoss_engine_create(None, p, 2, 16, 0, 0, C.byref(h)) == 1


def test_getp_hooks_compile_inside_the_reference_tu():
    if not os.path.exists(os.path.join(REF, "run.cpp")):
        pytest.skip("reference tree absent")
    hooks = os.path.join(ROOT, "gpt-oss-team01_amd", "hooks", "getp_run.cpp")
    # run.cpp with its line 1072 (#include "getp-csrc/getp_run.cpp") replaced by our hook file
    include = '#include "%s"' % hooks
    cmd = ("( head -n 1071 %s/run.cpp; echo '%s'; tail -n +1073 %s/run.cpp ) | "
           "g++ -std=c++17 -fsyntax-only -w -x c++ - -I%s -I%s/include" % (REF, include, REF, REF, ROOT))
    r = subprocess.run(["bash", "-c", cmd], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]


def test_bench_refuses_more_than_one_gpu():
    """bench.py is a one-GPU benchmark: --gpus N with N > 1 (or a multi-rank launch) exits with a
    message instead of running, before anything touches a device."""
    import sys
    for extra_env, args in (({}, ["--gpus", "2"]), ({"WORLD_SIZE": "2"}, [])):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + args, capture_output=True, text=True,
                           env=dict(os.environ, **extra_env), timeout=120)
        assert r.returncode == 2, (r.returncode, r.stderr[-300:])
        assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_engine_entry_points_validate_before_touching_a_device(lib):
    L = lib.load()
    buf = (C.c_char * 256)()
    p = C.cast(buf, C.c_void_p)
    # null engine / null buffers
    assert L.gptoss_engine_step(None, p, 0, 1, p) == 1
    assert L.gptoss_engine_step_ragged(None, p, p, 1, p) == 1
    assert L.gptoss_engine_step_rows(None, 1, p, p, p, 1, p, p) == 1
    assert L.gptoss_engine_prefill(None, p, 1, 1, p) == 1
    n = C.c_longlong(0)
    assert L.gptoss_engine_generate(None, p, p, 1, 1, 8, p, C.byref(n)) == 1
    assert L.gptoss_engine_generate_ragged(None, p, p, 1, 1, 8, None, p, C.byref(n)) == 1
    # prompt attention: shape checks come before any launch
    assert L.gptoss_attn_prefill(p, p, None, p, 0, 4, 0, 8, 2, 32, 64, 0, p, 1 << 20, None) == 2      # B = 0
    assert L.gptoss_attn_prefill(p, p, None, p, 1, 200, 0, 8, 2, 32, 128, 128, p, 1 << 20, None) == 2  # ring too short
    assert "windowed cache" in lib.last_error()
    assert L.gptoss_attn_prefill_workspace_bytes(0, 4, 8, 2, 32, 64) == 0
    assert L.gptoss_attn_prefill_workspace_bytes(2, 64, 8, 2, 32, 64) > 2 * 64 * 4
    # flags that exclude each other
    cfg = lib.Config(4096, 256, 8, 4, 256, 4, 32, 8, 2, 64, 4096, 150000.0, 32.0, 128, 7.0)
    h = C.c_void_p()
    assert L.gptoss_engine_create(C.byref(cfg), p, 2, 16, lib.ENGINE_PRECISE | lib.ENGINE_SYNTHETIC, 0, C.byref(h)) == 6
    # 32-bit element offsets inside the GEMM kernels: a logits buffer of 2^32 floats or more is refused
    big = lib.Config(201088, 2880, 32, 4, 2880, 24, 64, 64, 8, 64, 4096, 150000.0, 32.0, 128, 7.0)
    assert L.gptoss_engine_create(C.byref(big), None, 21400, 16, lib.ENGINE_SYNTHETIC | lib.ENGINE_LOGITS, 0, C.byref(h)) == 2
    assert "2^32" in lib.last_error()
    assert L.gptoss_engine_create(C.byref(cfg), p, 2, 16, lib.ENGINE_PRECISE | lib.ENGINE_MXFP4_EXPERTS, 0, C.byref(h)) == 6
