"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch


def to_layout(arr, canon, layout, device='cuda'):
    """canonical-order numpy array -> contiguous fp16 tensor in `layout` order."""
    perm = [canon.index(d) for d in layout]
    return torch.from_numpy(np.ascontiguousarray(np.transpose(arr, perm))).to(torch.float16).to(device)


def from_layout(t, canon, layout):
    """fp16 tensor in `layout` order -> canonical-order float64 numpy array."""
    a = t.detach().float().cpu().numpy().astype(np.float64)
    perm = [layout.index(d) for d in canon]
    return np.transpose(a, perm)


def h16(a):
    """Round to fp16 and back (the values the device actually sees)."""
    return np.asarray(a, dtype=np.float64).astype(np.float16).astype(np.float64)


def assert_close(got, want, tol=1e-2, name='', outliers=0.0):
    """The acceptance test of the build: |got-want| <= tol*(|want| + rms(want))
    elementwise and max|got-want| <= tol*max|want|.  ``outliers``: the fraction of
    elements that may miss the elementwise bound (they are still held to the bound
    on the maximum); for tensors whose rms says little about the size of the
    terms behind an element."""
    got = np.asarray(got, dtype=np.float64); want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (name, got.shape, want.shape)
    assert np.isfinite(got).all(), name + ': non-finite values'
    rms = np.sqrt(np.mean(want ** 2)) if want.size else 0.0
    err = np.abs(got - want)
    bound = tol * (np.abs(want) + rms) + 1e-6
    bad = err > bound
    assert bad.sum() <= outliers * bad.size, (f'{name}: {bad.sum()} of {bad.size} elements off; worst |err|='
                           f'{err.max():.4g} at want={want.flat[err.argmax()]:.4g}, rms={rms:.4g}')
    mx = np.abs(want).max() if want.size else 0.0
    assert err.max() <= tol * mx + 1e-6, f'{name}: max err {err.max():.4g} vs max|want| {mx:.4g}'
