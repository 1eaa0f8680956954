"""Host-built rotary table.  cos/sin are evaluated once in float64 on the host and
rounded to float32, so the GPU cache writer and the CPU oracle read the same bytes
(device libm and host libm differ in the last ulp, which would break bit-exact
cache bytes)."""
import numpy as np
import torch


def rope_table(max_pos, head_dim, theta=500000.0, device=None):
    """Returns (cos, sin), each float32 [max_pos, head_dim // 2]:
    angle[pos, j] = pos * theta ** (-2 j / head_dim)."""
    j = np.arange(head_dim // 2, dtype=np.float64)
    inv_freq = np.power(float(theta), -2.0 * j / head_dim)
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv_freq[None, :]
    cos = torch.from_numpy(np.cos(ang).astype(np.float32))
    sin = torch.from_numpy(np.sin(ang).astype(np.float32))
    if device is not None:
        cos, sin = cos.to(device), sin.to(device)
    return cos, sin
