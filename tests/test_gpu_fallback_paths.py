"""The alternative kernel paths behind the environment switches, held to the same parity bars.

The kernel library reads its switches once per process, so every case runs a selection of the other GPU
test files in a child process with the switch set: the register-staged fp16 convolution kernels, the
direct (one output per lane) convolutions, the table-driven fp32 convolutions, batch-norm backward with
the relu mask read from y, and the engine without relu bit masks / position codes / arena / batched
filter transposes / batch-norm backward link / reordering of fan-in writers / row-resident convolution and pooling
kernels / pooled batch norm."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CONV = "test_conv_fwd_bwd or test_conv_golden or test_transposed_conv or test_conv_fp16_nhwc_network_shapes"
CASES = [
    ("SAGA_HIP_CONV_STAGES", "0", ["tests/test_gpu_ops.py", "-k", CONV]),
    # (without the pipelined kernels there is no batch-norm backward link to count)
    ("SAGA_HIP_CONV_STAGES", "0", ["tests/test_gpu_networks.py", "-k", "not link"]),
    ("SAGA_HIP_FORCE_DIRECT", "1", ["tests/test_gpu_ops.py", "-k", CONV]),
    ("SAGA_HIP_F32_NO_UNIFORM", "1", ["tests/test_gpu_ops.py", "-k", CONV]),
    ("SAGA_HIP_BN_MASK_FROM_Y", "1", ["tests/test_gpu_networks.py"]),
    ("SAGA_HIP_NO_RELU_MASK", "1", ["tests/test_gpu_networks.py"]),
    ("SAGA_HIP_NO_POOL_CODES", "1", ["tests/test_gpu_networks.py", "-k", "resnet50 or unet"]),
    ("SAGA_HIP_NO_ARENA", "1", ["tests/test_gpu_networks.py", "-k", "training"]),
    ("SAGA_HIP_NO_BATCHED_TRANSPOSE", "1", ["tests/test_gpu_networks.py", "-k", "training and not links"]),
    ("SAGA_HIP_NO_BNBWD_LINK", "1", ["tests/test_gpu_networks.py", "-k", "training and not links"]),
    ("SAGA_HIP_NO_WRITER_REORDER", "1", ["tests/test_gpu_networks.py", "-k", "training"]),
    # the stem and the 3x3 64 -> 64 layers through the gather kernel instead of the row-resident ones
    ("SAGA_HIP_THIN_ROWS", "0", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd or folded_bn or bnstats"]),
    ("SAGA_HIP_ROWS64", "0", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd or folded_bn or bnstats"]),
    ("SAGA_HIP_ROWS64_WGM", "2", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd or folded_bn or bnstats"]),
    # the 3x3 64 -> 64 layers with two wavefronts per SIMD (half the filter each) instead of one with all of it
    ("SAGA_HIP_ROWS64_WIDE", "0", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd or folded_bn or bnstats"]),
    # backward filter of those layers through the generic kernel
    ("SAGA_HIP_FILTER_ROWS64", "0", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd"]),
    # batch norm and max pooling as separate operations (forward and backward; backward only)
    ("SAGA_HIP_NO_BN_POOL_FUSE", "1", ["tests/test_gpu_networks.py", "-k", "resnet50"]),
    ("SAGA_HIP_NO_BN_POOL_BWD_FUSE", "1", ["tests/test_gpu_networks.py", "-k", "resnet50"]),
    # 1x1 64 -> 256: through the gather kernel; through the streaming kernel also where the tensor is small
    ("SAGA_HIP_C64_WIDE", "0", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd or folded_bn or bnstats"]),
    ("SAGA_HIP_C64_WIDE", "2", ["tests/test_gpu_ops.py", "-k", "test_conv_fwd_bwd or folded_bn or bnstats"]),
    # 3x3 / stride 2 max pooling with one thread per window instead of whole image rows in LDS
    ("SAGA_HIP_POOL_ROWS", "0", ["tests/test_gpu_ops.py", "-k", "pool"]),
]


@pytest.mark.parametrize("var,value,selection", CASES, ids=[f"{c[0]}={c[1]}:{c[2][0].split('/')[-1]}" for c in CASES])
def test_switch(var, value, selection):
    env = dict(os.environ)
    env[var] = value
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", *selection, "-x", "-q", "-m", "gpu", "--timeout", "120",
                        "--timeout-method", "thread", "-p", "no:cacheprovider"],
                       cwd=ROOT, env=env, capture_output=True, text=True, timeout=600)
    tail = "\n".join(r.stdout.strip().splitlines()[-15:])
    print(tail)
    assert r.returncode == 0, tail + "\n" + r.stderr[-1500:]
    assert " passed" in tail and "failed" not in tail
