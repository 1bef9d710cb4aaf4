"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch

from any_precision_amd import synth

# GEMV/GEMM tolerance of the path: 1e-2 relative (fp32 accumulate, fp16 out), taken normwise
# and against the largest reference magnitude (elementwise relative error is ill-posed near 0).
REL_TOL = 1e-2


def layer_to_gpu(layer, planes=None, device="cuda"):
    qw = layer.qweight if planes is None else np.ascontiguousarray(layer.qweight[:planes])
    q = torch.from_numpy(qw).to(device)
    luts = {b: torch.from_numpy(t).to(device) for b, t in layer.luts.items()}
    return q, luts


def assert_bit_exact(got: torch.Tensor, want: np.ndarray, what=""):
    g = got.detach().cpu().contiguous().view(torch.int16).numpy()
    w = np.ascontiguousarray(want).view(np.int16)
    assert g.shape == w.shape, (what, g.shape, w.shape)
    if not np.array_equal(g, w):
        bad = np.argwhere(g != w)
        raise AssertionError(f"{what}: {len(bad)} of {g.size} halves differ, first at {bad[0].tolist()}")


def assert_close_gemv(got: torch.Tensor, want64: np.ndarray, what=""):
    g = got.detach().float().cpu().numpy().astype(np.float64).reshape(want64.shape)
    assert np.isfinite(g).all(), what
    num = np.linalg.norm(g - want64)
    den = np.linalg.norm(want64)
    assert num <= REL_TOL * den, f"{what}: normwise rel err {num / max(den, 1e-30):.3e}"
    assert np.abs(g - want64).max() <= REL_TOL * np.abs(want64).max(), f"{what}: max abs err {np.abs(g - want64).max():.3e}"


def make(N, K, seed):
    return synth.make_layer(N, K, seed=seed)
