"""The C++ launch* shims (the reference's own entry-point names over the C ABI).

GPU part: runs build/bin/test_launch_api, whose cases construct TensorWrapper / weight structs the
way the reference's unit-test programs do and check the launchers against the oracle.
CPU part: the shim library exports an instantiation of every launcher for float and half."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "build", "bin", "test_launch_api")
LAUNCH_LIB = os.path.join(ROOT, "inferspore_amd", "lib", "libinferspore_launch.so")


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["embedding", "padding", "norm", "rmsnorm", "qkv", "act", "bias_modes", "errors"])
def test_launch_api_case(case):
    assert os.path.exists(EXE), "build/bin/test_launch_api is missing: run python -m inferspore_amd.build"
    print("[case] test_launch_api " + case, flush=True)
    p = subprocess.run([EXE, case], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert p.returncode == 0, p.stdout[-3000:]
    assert "passed" in p.stdout


NEIGHBOURS = os.path.join(ROOT, "build", "bin", "test_launch_neighbours")


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["rope", "transpose", "kvcache"])
def test_launch_neighbours_case(case):
    assert os.path.exists(NEIGHBOURS), "build/bin/test_launch_neighbours is missing: run python -m inferspore_amd.build"
    print("[case] test_launch_neighbours " + case, flush=True)
    p = subprocess.run([NEIGHBOURS, case], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert p.returncode == 0, p.stdout[-3000:]
    assert "passed" in p.stdout


def test_launch_library_exports_all_instantiations():
    assert os.path.exists(LAUNCH_LIB), "libinferspore_launch.so is missing: run python -m inferspore_amd.build"
    syms = subprocess.run(["nm", "-D", "--defined-only", "-C", LAUNCH_LIB], stdout=subprocess.PIPE, text=True,
                          check=True).stdout
    for name in ("launchInputEmbedding", "launchFusedAddBiasResidualRMSNorm", "launchRMSNorm",
                 "launchAddFusedQKVBiasTransposeAndRoPE", "launchAct", "launchRoPE",
                 "launchTransposeOutRemovePadding", "launchConcatKVCache", "launchRepeatKVCache"):
        for t in ("float", "__half"):
            assert any(name + "<" + t + ">" in line for line in syms.splitlines()), (name, t)
    assert "launchCalPaddingoffset(" in syms
