"""Shared checks for the parity tests."""
import numpy as np
import torch

# tolerances of the parity bar: relative 1e-4 for fp32, 2e-2 for bf16, with an absolute floor of
# rtol * rms(reference) so that results near zero (signed operands cancel) are judged at the
# scale of the output
RTOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


def assert_close(got, ref, dtype, what=""):
    """got: torch tensor (any device); ref: numpy float64 array of the same shape."""
    g = got.detach().to("cpu", torch.float64).numpy()
    assert g.shape == ref.shape, f"{what}: shape {g.shape} vs {ref.shape}"
    assert np.isfinite(g).all(), f"{what}: non-finite values"
    rtol = RTOL[dtype]
    rms = float(np.sqrt(np.mean(ref * ref))) if ref.size else 0.0
    atol = rtol * rms
    err = np.abs(g - ref)
    bad = err > atol + rtol * np.abs(ref)
    if bad.any():
        idx = np.unravel_index(np.argmax(err), err.shape)
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.size} elements off; max |err|={err.max():.3e} at {idx} "
            f"(got {g[idx]:.6e}, ref {ref[idx]:.6e}), rms(ref)={rms:.3e}, rtol={rtol}"
        )


def to64(t):
    return t.detach().to("cpu", torch.float64).numpy()


def load_golden():
    """The index-array vectors the reference's own tests hold (tests/golden/reference_index_vectors.json)."""
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_index_vectors.json")) as f:
        return json.load(f)
