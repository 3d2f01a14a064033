"""Kernel provider.  `load_hip_ops(device)` is the only one the product has."""

from __future__ import annotations

_OPS = {}


def load_hip_ops(device):
    """The HIP kernels for `device`; raises if there is no GPU or no built library."""
    import torch
    from tokensprint_amd.kernels.hip_ops import HipOps
    device = torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", torch.cuda.current_device() if torch.cuda.is_available() else 0)
    if device not in _OPS:
        _OPS[device] = HipOps(device)
    return _OPS[device]
