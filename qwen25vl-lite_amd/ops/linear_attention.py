"""Dispatch to the linear-attention kernels (``csrc/linear_attention.hip``, compiled per key size).

``S_t = diag(a_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` per head, with the state of every
request in its slot's row of a float32 tensor ``[slots, heads, dim, vdim]``.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _dev, _fn, _need, _ptr, _stream, dtype_code

__all__ = ["decayed_scan", "scan_groups", "MAX_KEY_SIZE"]

_c_int, _c_float, _c_ptr, _c_ll = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_longlong
MAX_KEY_SIZE = 256
LONG_RUN = 64
BLOCKS_PER_CU = 2
MIN_ROWS = 4


def decayed_scan(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, num_heads: int, dim: int, vdim: int,
                 state: torch.Tensor, cu_q: torch.Tensor, req_slots: torch.Tensor, *,
                 head_decay: Optional[torch.Tensor] = None, z: Optional[torch.Tensor] = None, tau: float = 1.0,
                 silu: bool = False, q_scale: float = 1.0, groups: int = 1) -> torch.Tensor:
    """Run every request's tokens of the step through the recurrence, from and into ``state``.

    ``proj [N, cols]`` (float32 or bfloat16) holds, per token, ``heads * dim`` query columns from
    ``q_off``, as many key columns from ``k_off`` and ``heads * vdim`` value columns from ``v_off``;
    ``silu`` applies the activation to all three as they are read, ``q_scale`` scales the queries.
    The decay is ``head_decay [heads]`` (float32, one constant per head) or, per token and key
    channel, ``sigmoid(z)^(1/tau)`` for float32 ``z [N, heads * dim]``.  ``cu_q [R + 1]`` bounds each
    request's run of tokens, ``req_slots [R]`` names its row of ``state``.  Returns float32
    ``[groups, N, heads * vdim]``: with ``groups`` above 1 (2, 4 or 8; the key size must be a multiple
    of four times it) the key channels are cut into that many groups with blocks of their own, and the
    output is the sum of the slabs (see :func:`scan_groups`)."""
    _dev(proj, state, cu_q, req_slots, head_decay, z)
    h, d, v = int(num_heads), int(dim), int(vdim)
    n = proj.shape[0]
    _need(d % 4 == 0 and 4 <= d <= MAX_KEY_SIZE, f"key sizes in steps of 4 up to {MAX_KEY_SIZE} are built")
    _need(proj.dim() == 2 and proj.stride(1) == 1, "proj must be [N, cols] with contiguous rows")
    for off, width in ((q_off, h * d), (k_off, h * d), (v_off, h * v)):
        _need(0 <= off and off + width <= proj.shape[1], "q, k or v columns lie outside proj")
    _need(state.dtype == torch.float32 and state.dim() == 4 and tuple(state.shape[1:]) == (h, d, v)
          and state.is_contiguous(), "state must be contiguous float32 [slots, heads, dim, vdim]")
    for t in (cu_q, req_slots):
        _need(t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous(), "cu_q and req_slots must be int32")
    r = req_slots.shape[0]
    _need(cu_q.shape[0] == r + 1, "cu_q must have one more entry than there are requests")
    _need((head_decay is None) != (z is None), "exactly one of head_decay and z is needed")
    zstride = 0
    if head_decay is not None:
        _need(head_decay.dtype == torch.float32 and head_decay.shape == (h,) and head_decay.is_contiguous(),
              "head_decay must be float32 [heads]")
    else:
        _need(z.dtype == torch.float32 and z.shape == (n, h * d) and z.stride(1) == 1, "z must be float32 [N, heads dim]")
        _need(tau > 0, "tau must be positive")
        zstride = z.stride(0)
    _need(groups in (1, 2, 4, 8) and d % (4 * groups) == 0, "groups must be 1, 2, 4 or 8 and divide a quarter of the key size")
    out = torch.empty((groups, n, h * v), dtype=torch.float32, device=proj.device)
    fn = _fn("linear_attention", "qvl_la_scan",
             [_c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ll, _c_float, _c_ptr, _c_ptr, _c_ptr,
              _c_ptr, _c_ll, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr], {"LA_DIM": d})
    _check(fn(_ptr(proj), proj.stride(0), int(q_off), int(k_off), int(v_off), dtype_code(proj.dtype),
              _ptr(head_decay), _ptr(z), zstride, 1.0 / float(tau), _ptr(state), _ptr(cu_q), _ptr(req_slots),
              _ptr(out), out.stride(0), int(groups), r, h, d, v, int(silu), float(q_scale), _stream()), "decayed_scan")
    return out


def scan_groups(num_reqs: int, max_run: int, num_heads: int, dim: int, vdim: int, device=None) -> int:
    """Into how many groups of key channels :func:`decayed_scan` is cut for a step.  A block walks its
    request's tokens one after the other, so the blocks, not the tokens, have to fill the device: runs
    of ``LONG_RUN`` tokens or more are cut until there are ``BLOCKS_PER_CU`` blocks a compute unit or
    a wave is down to ``MIN_ROWS`` rows of the state."""
    if max_run < LONG_RUN:
        return 1
    from .attention_mfma import _compute_units
    blocks = num_reqs * num_heads * ((vdim + 63) // 64)
    groups = 1
    while (groups < 8 and blocks * groups < BLOCKS_PER_CU * _compute_units(device)
           and dim % (8 * groups) == 0 and dim // (8 * groups) >= MIN_ROWS):
        groups *= 2
    return groups
