"""CPU: the (workgroup id -> head, q-block) map of the attention-shaped kernels
covers every (head, q-block) exactly once, also when a KV head has more than 64
query heads.  The map is compiled for the host from the kernels' own header and
enumerated there; nothing runs on a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_head_and_q_block_is_dispatched_exactly_once(tmp_path):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not (os.path.exists(hipcc) or shutil.which(hipcc)):
        pytest.skip("hipcc not available")
    exe = str(tmp_path / "dispatch_map_check")
    src = os.path.join(ROOT, "tests", "host", "dispatch_map_check.cpp")
    cmd = [hipcc, "-x", "hip", "--offload-arch=gfx950", "-O1", "-std=c++17",
           "-I" + os.path.join(ROOT, "x-attention_amd", "csrc"), "-I" + os.path.join(ROOT, "include"), src, "-o", exe]
    build = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert build.returncode == 0, build.stdout
    run = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    print(run.stdout)
    assert run.returncode == 0, run.stdout
    assert run.stdout.count("missing 0 twice 0 stray 0 mixed-units 0") >= 16
