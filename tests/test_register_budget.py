"""Generated kernels must fit the register file of their workgroup size: a
kernel that spills still computes the right values, only two or three times
slower, so no numerics test notices.  A few kernels that once spilled (an LDS
join unrolled as a whole in 8-wide cooperative kernels; rows of 64 tiles
unrolled three sweeps over) and the benchmark's resident-row kernels are
compiled for gfx950 with hipcc's resource-usage remarks and checked for
scratch use.  Needs no GPU."""
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from neon_amd.backends import bfloat16
from neon_amd.backends.hip import prebuild

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")


def _usage(source, tmp_path):
    src = tmp_path / "k.hip"
    src.write_text('#include <hip/hip_runtime.h>\n#include "device/neon_device.h"\n' + source)
    cmd = ["hipcc", "-O3", "-std=c++17", "--offload-arch=gfx950", "-ffp-contract=off",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I" + os.path.join(ROOT, "neon_amd", "csrc"), "-c", str(src), "-o", os.devnull,
           "-Rpass-analysis=kernel-resource-usage", "--offload-device-only"]
    out = subprocess.run(cmd, capture_output=True, text=True)
    assert out.returncode == 0, out.stderr[-2000:]
    vgprs = int(re.search(r"\sVGPRs: (\d+)", out.stderr).group(1))
    spill = int(re.search(r"VGPRs Spill: (\d+)", out.stderr).group(1))
    scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", out.stderr).group(1))
    return vgprs, spill, scratch


def _softmax(be, x, axis):
    e = be.exp(x - be.max(x, axis=axis))
    return e / be.sum(e, axis=axis)


def _norm(be, x, axis):
    return (x - be.mean(x, axis=axis)) / be.sqrt(be.var(x, axis=axis) + 1e-5)


CASES = [
    ("cooperating columns, 8 values per lane, two levels", (32000, 512), np.float16, _norm, 0, "colcoop"),
    ("cooperating columns, softmax, fp16", (4096, 4096), np.float16, _softmax, 0, "colcoop"),
    ("cooperating rows of 64 tiles, mostly streamed", (64, 1048576), np.float32, _softmax, 1, "rowcoop"),
    ("cooperating rows of 64 tiles, three sweeps", (64, 1048576), np.float32, _norm, 1, "rowcoop"),
    ("resident fp16 rows, 1024 lanes, 13 tiles", (256, 100352), np.float16, _norm, 1, "row"),
    ("resident bf16 rows with the exponentials kept", (4096, 4096), bfloat16, _softmax, 1, "row"),
    ("column strips of 1024 lanes, fp16", (1000, 4096), np.float16, _softmax, 0, "col"),
]


@pytest.mark.parametrize("what,shape,dtype,tree,axis,family", CASES, ids=[c[0] for c in CASES])
def test_generated_kernels_do_not_spill(tmp_path, what, shape, dtype, tree, axis, family):
    be = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"), compile_kernels=False)
    x, out = be.empty(shape, dtype), be.empty(shape, dtype)
    out[:] = tree(be, x, axis)
    spec = be.choices[-1].spec
    assert spec.family == family
    vgprs, spill, scratch = _usage(spec.source, tmp_path)
    # 512 registers per lane of a SIMD, shared by the waves of the workgroups resident on it
    budget = 128 if spec.block == 1024 else 256 if spec.block == 512 else 512
    assert spill == 0 and scratch == 0 and vgprs <= budget, (what, vgprs, spill, scratch)


def test_benchmark_kernels_do_not_spill(tmp_path):
    """every kernel of the benchmark op-trees (the ones the build step pre-compiles)"""
    be = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"), compile_kernels=False)
    prebuild.benchmark_statements(be)
    seen = set()
    for ch in be.choices:
        if ch.spec.name in seen:
            continue
        seen.add(ch.spec.name)
        vgprs, spill, scratch = _usage(ch.spec.source, tmp_path)
        budget = 128 if ch.spec.block == 1024 else 256 if ch.spec.block == 512 else 512
        assert spill == 0 and scratch == 0 and vgprs <= budget, (ch.spec.family, ch.spec.params, vgprs, spill, scratch)
    assert len(seen) >= 8
