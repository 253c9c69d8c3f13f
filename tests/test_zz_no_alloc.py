"""saga_hip_bias_bwd_noalloc (the entry point that allocates nothing) against saga_hip_bias_bwd with a
caller-provided workspace: same kernels, so the results must be identical bit for bit, on two calls in a
row that share the library's fixed scratch array, the second on a smaller tensor."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref
from saga_amd import kernels as K
from tests.gpu_util import dev, host, rnd

pytestmark = pytest.mark.gpu


def S():
    return K.stream_ptr()


def _both(y, dtype, padc, beta):
    """(with workspace, without allocation) results of db = beta*db + sum dy."""
    c = y.shape[1]
    dyd = dev(y, dtype, "nhwc", padc)
    vdy = K.view(dyd)
    need = K.lib().saga_hip_bias_bwd_workspace_size(C.byref(vdy))
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    out = []
    for noalloc in (False, True):
        db = dev(np.full(c, 0.5, np.float32), torch.float32)
        vdb = K.view(db.view(1, c, 1, 1))
        if noalloc:
            K.check(K.lib().saga_hip_bias_bwd_noalloc(C.byref(vdy), C.byref(vdb), beta, S()))
        else:
            K.check(K.lib().saga_hip_bias_bwd(C.byref(vdy), C.byref(vdb), beta, K.ptr(ws), need, S()))
        torch.cuda.synchronize()
        out.append(host(db))
    return need, out[0], out[1]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_noalloc_matches_workspace_twice(dtype):
    rng = np.random.default_rng(71)
    # first call: two-pass reduction over 1024 row blocks; second call: fewer blocks and channels, so the
    # scratch still holds the first call's partials beyond what the second one writes
    shapes = [((4, 64, 96, 96), 0), ((2, 24, 200, 150), 8), ((3, 16, 5, 5), 0)]
    needs = []
    for shape, padc in shapes:
        y = rnd(rng, *shape, dtype=dtype)
        need, with_ws, without = _both(y, dtype, padc, 1.0)
        needs.append(need)
        assert np.array_equal(with_ws, without), f"{shape}: no-alloc result differs from the workspace result"
        want = ref.bias_bwd(y) + 0.5
        scale = np.abs(y.astype(np.float64)).sum(axis=(0, 2, 3)).max()
        assert np.abs(without - want).max() <= 2e-6 * scale, f"{shape}: against the oracle"
    assert needs[0] > needs[1] > 0 and needs[2] == 0


def test_noalloc_rejects_beyond_scratch():
    """A tensor whose partial sums need more than the fixed array is refused and db is left alone."""
    c = 2056
    dyd = torch.zeros((8, 64, 64, c), dtype=torch.float16, device="cuda").permute(0, 3, 1, 2)
    vdy = K.view(dyd)
    assert K.lib().saga_hip_bias_bwd_workspace_size(C.byref(vdy)) > (4 << 20)
    db = dev(np.full(c, 3.0, np.float32), torch.float32)
    rc = K.lib().saga_hip_bias_bwd_noalloc(C.byref(vdy), C.byref(K.view(db.view(1, c, 1, 1))), 0.0, S())
    assert rc == -5
    assert b"scratch" in K.lib().saga_hip_error_string(rc)
    torch.cuda.synchronize()
    assert np.all(host(db) == 3.0)
