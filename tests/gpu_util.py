"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

# Tolerance of the fp32 path, stated by the task: max |a - b| / max |b| <= 1e-4 against the CPU path.
FP32_REL_TOL = 1e-4


def rel_err(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    denom = np.max(np.abs(ref))
    if denom == 0:
        return float(np.max(np.abs(got)))
    return float(np.max(np.abs(got - ref)) / denom)


def assert_close(got, ref, tol=FP32_REL_TOL, what=""):
    err = rel_err(got, ref)
    assert err <= tol, f"{what}: max rel err {err:.3e} > {tol:.1e}"
    return err


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def announce(*args):
    """Print and flush the case about to run, so that a faulting kernel can be named from the log."""
    print("[case]", *args, flush=True)
