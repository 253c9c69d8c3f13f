"""Helpers shared by the GPU parity tests: device tensors with a chosen physical layout,
and the per-tensor relative max-abs error the parity bar is stated in."""
import numpy as np
import torch

TOL = {torch.float32: 1e-4, torch.float16: 2e-2}


def dev(a, dtype=torch.float32, layout="nchw", pad_c=0):
    """numpy array in logical order -> cuda tensor of the same logical shape.
    layout 'nhwc' gives channels-last strides; pad_c > 0 makes it a channel slice of a wider
    tensor (row pitch C + pad_c), which is how concat outputs look to a kernel."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if t.dtype.is_floating_point:
        t = t.to(dtype)
    t = t.cuda()
    if t.dim() == 4 and layout == "nhwc":
        N, C, H, W = t.shape
        wide = torch.zeros((N, H, W, C + pad_c), dtype=t.dtype, device="cuda")
        wide[..., :C] = t.permute(0, 2, 3, 1)
        t = wide[..., :C].permute(0, 3, 1, 2)
        assert t.stride(1) == 1
    return t


def empty_like_layout(shape, dtype, layout="nchw", pad_c=0, fill=None):
    a = np.zeros(shape, np.float32) if fill is None else np.full(shape, fill, np.float32)
    return dev(a, dtype, layout, pad_c)


def host(t):
    return t.detach().float().cpu().numpy()


def rel_err(got, want):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    scale = max(float(np.abs(want).max()), 1e-30)
    return float(np.abs(got - want).max()) / scale


def assert_close(got, want, dtype, what="", tol=None):
    tol = TOL[dtype] if tol is None else tol
    e = rel_err(got, want)
    assert e <= tol, f"{what}: relative max-abs error {e:.3e} > {tol:.1e}"
    return e


def rnd(rng, *shape, dtype=torch.float32, scale=1.0):
    a = (rng.standard_normal(shape) * scale).astype(np.float32)
    if dtype == torch.float16:
        a = a.astype(np.float16).astype(np.float32)
    return a
