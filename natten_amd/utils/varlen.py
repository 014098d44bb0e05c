"""Parameters of variable-length (sequence-packed) attention.

Mirrors the reference's src/natten/utils/varlen.py:33-132 (`generate_varlen_parameters`) and
src/natten/utils/checks.py:569-726 (`varlen_tensor_checks`): same argument rules, same exception
classes, same return convention `(cumulative_seqlen_Q, cumulative_seqlen_KV, max_seqlen_Q,
max_seqlen_KV)` with `(None, None, 0, 0)` for "not variable-length".
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor


def generate_varlen_parameters(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    seqlens_Q: Optional[Tensor] = None,
    seqlens_KV: Optional[Tensor] = None,
) -> Tuple[Optional[Tensor], Optional[Tensor], int, int]:
    """Cumulative (leading 0, int32, on the tensors' device) and maximum sequence lengths from
    per-sequence lengths.  The maxima are Python ints, which costs one device-to-host
    synchronisation: call this ahead of a compiled region, not inside one."""
    if torch.compiler.is_compiling():
        raise RuntimeError(
            "'generate_varlen_parameters' synchronises with the device and cannot run inside a compiled "
            "region; call it ahead of time and pass cumulative_seqlen_{Q,KV} and max_seqlen_{Q,KV} to 'attention'."
        )
    if query.shape[0] != key.shape[0] or query.shape[0] != value.shape[0]:
        raise ValueError(
            f"Q, K, and V must match in batch size, got {query.shape[0]=}, {key.shape[0]=}, {value.shape[0]=}."
        )
    if (seqlens_Q is None) != (seqlens_KV is None):
        raise ValueError("Variable length Attention requires both of seqlens_Q and seqlens_KV to be set.")
    if seqlens_Q is None:
        return None, None, 0, 0
    if not isinstance(seqlens_Q, Tensor) or not isinstance(seqlens_KV, Tensor):
        raise ValueError("seqlens_Q and seqlens_KV must both be tensors.")
    if seqlens_Q.device != query.device or seqlens_KV.device != query.device:
        raise ValueError(
            f"seqlens_Q and seqlens_KV must be on the same device as QKV, but {seqlens_Q.device=}, "
            f"{seqlens_KV.device=}, {query.device=}."
        )
    if seqlens_Q.dtype != torch.int32 or seqlens_KV.dtype != torch.int32:
        raise ValueError(
            f"seqlens_Q and seqlens_KV must both be torch.int32 tensors, got {seqlens_Q.dtype=}, {seqlens_KV.dtype=}."
        )
    if seqlens_Q.dim() != 1 or seqlens_KV.dim() != 1:
        raise ValueError(f"seqlens_Q and seqlens_KV must both be 1-D tensors, got {seqlens_Q.dim()=}, {seqlens_KV.dim()=}.")
    if seqlens_Q.shape[0] != seqlens_KV.shape[0]:
        raise ValueError(f"seqlens_Q and seqlens_KV must match in size, got {seqlens_Q.shape=}, {seqlens_KV.shape=}.")
    if seqlens_Q.shape[0] < 1:
        raise ValueError("seqlens_Q and seqlens_KV must contain at least one element.")
    if query.shape[0] != 1:
        raise ValueError(
            f"Variable length attention only supports sequence-packed memory layout (batch = 1), got {query.shape[0]=}."
        )
    max_q = int(seqlens_Q.max().item())
    max_kv = int(seqlens_KV.max().item())
    zero = torch.zeros(1, dtype=torch.int32, device=seqlens_Q.device)
    cu_q = torch.cat([zero, seqlens_Q.cumsum(0).to(torch.int32)], dim=0)
    cu_kv = torch.cat([zero, seqlens_KV.cumsum(0).to(torch.int32)], dim=0)
    return cu_q, cu_kv, max_q, max_kv


def varlen_tensor_checks(
    query: Tensor,
    key: Tensor,
    value: Tensor,
    seqlens_Q: Optional[Tensor] = None,
    seqlens_KV: Optional[Tensor] = None,
    cumulative_seqlen_Q: Optional[Tensor] = None,
    cumulative_seqlen_KV: Optional[Tensor] = None,
    max_seqlen_Q: Optional[int] = None,
    max_seqlen_KV: Optional[int] = None,
) -> Tuple[Optional[Tensor], Optional[Tensor], int, int]:
    if query.shape[0] != key.shape[0] or query.shape[0] != value.shape[0]:
        raise ValueError(
            f"Q, K, and V must match in batch size, got {query.shape[0]=}, {key.shape[0]=}, {value.shape[0]=}."
        )
    if all(x is None for x in (seqlens_Q, seqlens_KV, cumulative_seqlen_Q, cumulative_seqlen_KV)) and all(
        x is None or x == 0 for x in (max_seqlen_Q, max_seqlen_KV)
    ):
        return None, None, 0, 0
    if seqlens_Q is not None or seqlens_KV is not None:
        return generate_varlen_parameters(query, key, value, seqlens_Q, seqlens_KV)
    if any(x is None for x in (cumulative_seqlen_Q, cumulative_seqlen_KV, max_seqlen_Q, max_seqlen_KV)):
        raise ValueError(
            "Variable length Attention requires all of cumulative_seqlen_{Q,KV} and max_seqlen_{Q,KV} to be set."
        )
    if query.shape[0] != 1:
        raise ValueError(
            f"Variable length Attention only supports sequence-packed memory layout (batch = 1), got {query.shape[0]=}."
        )
    if not isinstance(max_seqlen_Q, int) or not isinstance(max_seqlen_KV, int):
        raise ValueError(
            f"max_seqlen_Q and max_seqlen_KV must be ints, got {type(max_seqlen_Q)=}, {type(max_seqlen_KV)=}."
        )
    if max_seqlen_Q > query.shape[1]:
        raise ValueError(f"Maximum sequence length cannot exceed total, got {max_seqlen_Q=}, {query.shape[1]=}.")
    if max_seqlen_KV > key.shape[1]:
        raise ValueError(f"Maximum sequence length cannot exceed total, got {max_seqlen_KV=}, {key.shape[1]=}.")
    if not torch.compiler.is_compiling() and (max_seqlen_Q == 0) != (max_seqlen_KV == 0):
        raise ValueError(
            f"max_seqlen_Q and max_seqlen_KV must both be zero or both be non-zero, got {max_seqlen_Q=}, {max_seqlen_KV=}."
        )
    if max_seqlen_Q < 0 or max_seqlen_KV < 0:
        raise ValueError(f"Maximum sequence length cannot be negative, got {max_seqlen_Q=}, {max_seqlen_KV=}.")
    if not isinstance(cumulative_seqlen_Q, Tensor) or not isinstance(cumulative_seqlen_KV, Tensor):
        raise ValueError("cumulative_seqlen_Q and cumulative_seqlen_KV must both be tensors.")
    if cumulative_seqlen_Q.device != query.device or cumulative_seqlen_KV.device != query.device:
        raise ValueError(
            f"cumulative_seqlen_Q and cumulative_seqlen_KV must be on the same device as QKV, but "
            f"{cumulative_seqlen_Q.device=}, {cumulative_seqlen_KV.device=}, {query.device=}."
        )
    if cumulative_seqlen_Q.dtype != torch.int32 or cumulative_seqlen_KV.dtype != torch.int32:
        raise ValueError(
            f"cumulative_seqlen_Q and cumulative_seqlen_KV must both be torch.int32 tensors, got "
            f"{cumulative_seqlen_Q.dtype=}, {cumulative_seqlen_KV.dtype=}."
        )
    if cumulative_seqlen_Q.dim() != 1 or cumulative_seqlen_KV.dim() != 1:
        raise ValueError(
            f"cumulative_seqlen_Q and cumulative_seqlen_KV must both be 1-D tensors, got "
            f"{cumulative_seqlen_Q.dim()=}, {cumulative_seqlen_KV.dim()=}."
        )
    if cumulative_seqlen_Q.shape[0] != cumulative_seqlen_KV.shape[0]:
        raise ValueError(
            f"cumulative_seqlen_Q and cumulative_seqlen_KV must match in size, got "
            f"{cumulative_seqlen_Q.shape=}, {cumulative_seqlen_KV.shape=}."
        )
    if cumulative_seqlen_Q.shape[0] < 2:
        raise ValueError("cumulative_seqlen_Q and cumulative_seqlen_KV must contain at least 2 elements.")
    return cumulative_seqlen_Q, cumulative_seqlen_KV, max_seqlen_Q, max_seqlen_KV
