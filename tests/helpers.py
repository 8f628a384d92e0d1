"""Shared helpers of the GPU parity tests."""
import numpy as np


def to_np(t):
    import torch
    if isinstance(t, torch.Tensor):
        if t.dtype == torch.bfloat16:
            return t.detach().float().cpu().numpy()
        return t.detach().cpu().numpy()
    return np.asarray(t)


def code_stats(c_gpu, c_ref):
    """(fraction of unequal codes, largest absolute code difference)."""
    d = c_gpu.astype(np.int32) - c_ref.astype(np.int32)
    return float(np.mean(d != 0)), int(np.abs(d).max()) if d.size else 0


def recon_error(W, Q, X):
    """||X W - X Q|| / ||X W|| in fp64 (layer reconstruction error)."""
    W = W.astype(np.float64)
    Q = Q.astype(np.float64)
    X = X.astype(np.float64)
    return float(np.linalg.norm(X @ (W - Q)) / np.linalg.norm(X @ W))
