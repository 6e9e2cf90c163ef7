"""The C-ABI library loads without a GPU and exports every function that
include/xattn_hip.h declares; the ctypes binding covers the same set."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "xattn_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xattn_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for must in ("xattn_estimate_block_sums", "xattn_select_blocks", "xattn_block_sparse_fwd",
                 "xattn_estimate_workspace_bytes", "xattn_abi_version", "xattn_error_string"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from xattn.src import hip_backend as hb

    if not os.path.exists(hb.LIB_PATH):
        pytest.fail(f"{hb.LIB_PATH} has not been built (python x-attention_amd/csrc/build.py)")
    lib = ctypes.CDLL(hb.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert sorted(hb.exported_symbols()) == declared_functions()


def test_host_side_calls_need_no_gpu():
    from xattn.src import hip_backend as hb

    lib = hb.lib()
    assert lib.xattn_abi_version() >= 1
    assert lib.xattn_error_string(0) == b"ok"
    assert b"128" in lib.xattn_error_string(-2)
    # geometry helper: pure host arithmetic
    assert lib.xattn_estimate_workspace_bytes(32, 131072, 131072, 16, 128, 16384, 0) == 32 * 8192 * (1024 + 2 * 64) * 4
    assert lib.xattn_estimate_workspace_bytes(32, 131072, 131072, 3, 128, 16384, 0) == 0     # bad stride
    assert lib.xattn_estimate_workspace_bytes(32, 4096, 2048, 8, 128, 2048, 0) == 0          # k shorter than q


def test_attention_entry_points_validate_strides_and_scale_before_launching():
    """Host-side validation only: the calls return before anything is enqueued,
    so dummy (aligned, non-null) addresses are enough."""
    from xattn.src import hip_backend as hb

    lib = hb.lib()
    a = 0x10000
    ok_strides = [128 * 256, 128, 128 * 256, 128, 128 * 256, 128, 128, 128 * 4]

    def fwd(strides, scale=0.1, heads=4, kv=2):
        return lib.xattn_block_sparse_fwd(a, a, a, a, None, None, 0, 0, 0, heads, kv, 256, 256, 128, *strides, 0, -1, 1,
                                          scale, None)

    big = 1 << 23
    assert fwd([ok_strides[0], 128, ok_strides[2], big] + ok_strides[4:]) == -4        # K token stride beyond 2^22
    assert fwd(ok_strides[:5] + [big] + ok_strides[6:]) == -4                          # V token stride
    assert fwd([ok_strides[0], big] + ok_strides[2:]) == -4                            # Q token stride (a tile like K)
    assert fwd(ok_strides[:3] + [64] + ok_strides[4:]) == -4                           # rows would overlap
    assert fwd(ok_strides, scale=0.0) == -4 and fwd(ok_strides, scale=-1.0) == -4
    assert fwd(ok_strides, scale=float("nan")) == -4
    assert fwd(ok_strides, heads=3, kv=2) == -3
    mass = lambda ksn, scale=0.1: lib.xattn_block_mass(a, a, a, 4, 2, 256, 256, 128, 128 * 256, 128, 128 * 256, ksn, 1,
                                                       scale, None)
    assert mass(big) == -4 and mass(64) == -4 and mass(128, scale=0.0) == -4
    # the allocation-free decode form refuses what its built-in array cannot hold, before touching anything
    assert lib.xattn_decode_fwd_static(a, a, a, a, 512 * 32, 512, 64, 128, 128, 8192, 128, 8192, 128, 128, 0.1, None) == -7


def test_operator_refuses_cpu_tensors_and_wrong_dtypes():
    import torch

    from xattn.src import hip_backend as hb
    from xattn.src.Xattention import Xattention_prefill, default_chunk_size, xattn_estimate

    q = torch.zeros(1, 2, 256, 128, dtype=torch.bfloat16)
    with pytest.raises(hb.XattnHipError):
        Xattention_prefill(q, q, q, 8)
    with pytest.raises(ValueError):
        xattn_estimate(q, q, 128, 8, select_mode="diagonal")     # not one of the reference's modes
    with pytest.raises(ValueError):
        xattn_estimate(q, q, 128, 8, kdb=2)
    with pytest.raises(hb.XattnHipError):
        xattn_estimate(q, q, 128, 8, select_mode="slash", softmax=False)   # valid request, CPU tensors
    table = {1024: 2048, 4096: 4096, 16384: 16384, 32768: 8192, 65536: 4096, 131072: 2048, 119056: 2048}
    for L, want in table.items():
        assert default_chunk_size(L) == want


def test_product_path_never_touches_the_oracle():
    """The oracle is a checker: nothing under the package may import or run it."""
    pkg = os.path.join(ROOT, "x-attention_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "import oracle" not in text and "from oracle" not in text and "xattn_oracle" not in text, f


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr
