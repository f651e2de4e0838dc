"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def max_rel_err(got, want):
    """max |got - want| / max |want|: the error measure of the 1e-2 parity bar."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    scale = np.abs(want).max()
    if scale == 0:
        return float(np.abs(got).max())
    return float(np.abs(got - want).max() / scale)


# north-star bar for SpMM results (fp16 in, fp32 accumulate) against the host fp32 reference
PARITY_TOL = 1e-2
# what a correct fp32-accumulating kernel actually achieves; a wrong index or a dropped term
# shows up as an O(1) error, re-association of fp32 sums stays below this
TIGHT_F32 = 2e-5
TIGHT_F16 = 2e-3
