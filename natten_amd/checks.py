"""Argument and tensor validation of the public ops.

Same rules and exception classes as the reference's src/natten/utils/checks.py
(na_tensor_checks :85-182, fmha_tensor_checks :185-275, additional_kv_tensor_checks :278-370,
check_*_arg :373-470, check_args_against_input :486-508, is_self_attention :511-526).
"""

from __future__ import annotations

from collections.abc import Sequence
from typing import Any, Optional, Tuple

from torch import Tensor

DimensionType = Tuple[int, ...]
CausalArgType = Tuple[bool, ...]


def _same_kind_checks(query: Tensor, key: Tensor, value: Tensor):
    if query.is_sparse or key.is_sparse or value.is_sparse:
        raise NotImplementedError("Sparse tensors are not supported.")
    if query.is_nested or key.is_nested or value.is_nested:
        raise NotImplementedError("Nested tensors are not supported.")
    if query.device != key.device or query.device != value.device:
        raise ValueError(
            f"Query, key, and value must be on the same device, got {query.device}, {key.device}, {value.device}."
        )
    if query.dtype != key.dtype or query.dtype != value.dtype:
        raise ValueError(
            f"Query, key, and value must have the same data type, got {query.dtype}, {key.dtype}, {value.dtype}."
        )


def _head_checks(query: Tensor, key: Tensor, value: Tensor):
    if key.shape[-2] != value.shape[-2]:
        raise ValueError(
            f"Key and value must have the same number of heads, got {key.shape[-2]} and {value.shape[-2]}."
        )
    heads_q, heads_kv = query.shape[-2], key.shape[-2]
    if heads_q < heads_kv or heads_q % heads_kv != 0:
        raise ValueError(f"Key/value heads must evenly divide query heads, got {heads_q=}, {heads_kv=}.")


def na_tensor_checks(query: Tensor, key: Tensor, value: Tensor, must_match_head_dims: bool = False):
    _same_kind_checks(query, key, value)
    if query.dim() != key.dim() or query.dim() != value.dim():
        raise ValueError(
            f"Query, key, and value must have the same rank, got {query.dim()}, {key.dim()}, {value.dim()}."
        )
    if query.dim() not in (4, 5, 6):
        raise ValueError(
            f"Expected 4-D, 5-D, or 6-D tensors (NA1D, NA2D, NA3D: [batch, *tokens, heads, head_dim]), got {query.dim()}-D."
        )
    na_dim = query.dim() - 3
    if query.shape[-1] != key.shape[-1]:
        raise ValueError(f"Q and K head dims must match, got {query.shape[-1]} and {key.shape[-1]}.")
    if query.shape[0] != key.shape[0] or query.shape[0] != value.shape[0]:
        raise ValueError(
            f"Q, K, and V must match in batch size, got {query.shape[0]}, {key.shape[0]}, {value.shape[0]}."
        )
    if must_match_head_dims and query.shape[-1] != value.shape[-1]:
        raise ValueError(
            f"Different head dims for QK and V are not supported, got {query.shape[-1]} and {value.shape[-1]}."
        )
    lay = query.shape[1 : na_dim + 1]
    if lay != key.shape[1 : na_dim + 1] or lay != value.shape[1 : na_dim + 1]:
        raise ValueError(
            "Neighborhood attention requires Q, K, and V to match in their token layouts, got "
            f"{tuple(lay)}, {tuple(key.shape[1:na_dim + 1])}, {tuple(value.shape[1:na_dim + 1])}."
        )
    _head_checks(query, key, value)


def fmha_tensor_checks(query: Tensor, key: Tensor, value: Tensor, must_match_head_dims: bool = False):
    _same_kind_checks(query, key, value)
    if query.dim() != key.dim() or query.dim() != value.dim():
        raise ValueError(
            f"Query, key, and value must have the same rank, got {query.dim()}, {key.dim()}, {value.dim()}."
        )
    if query.dim() != 4:
        raise ValueError(f"Expected 4-D tensors [batch, seqlen, heads, head_dim], got {query.dim()}-D.")
    if query.shape[-1] != key.shape[-1]:
        raise ValueError(f"Q and K head dims must match, got {query.shape[-1]} and {key.shape[-1]}.")
    if must_match_head_dims and query.shape[-1] != value.shape[-1]:
        raise ValueError(
            f"Different head dims for QK and V are not supported, got {query.shape[-1]} and {value.shape[-1]}."
        )
    if query.shape[0] != key.shape[0] or query.shape[0] != value.shape[0]:
        raise ValueError(
            f"Q, K, and V must match in batch size, got {query.shape[0]}, {key.shape[0]}, {value.shape[0]}."
        )
    if key.shape[1] != value.shape[1]:
        raise ValueError(f"K and V must match in sequence length, got {key.shape[1]} and {value.shape[1]}.")
    _head_checks(query, key, value)


def additional_kv_tensor_checks(
    query: Tensor, key: Tensor, value: Tensor, add_key: Optional[Tensor], add_value: Optional[Tensor]
):
    if (add_key is None) != (add_value is None):
        raise ValueError("`additional_keys` and `additional_values` must be either both Tensors or both None.")
    if add_key is None or add_value is None:
        return
    _same_kind_checks(query, add_key, add_value)
    if add_key.dim() != 4 or add_value.dim() != 4:
        raise ValueError("Additional keys/values must be 4-D tensors [batch, seqlen, heads, head_dim].")
    if query.shape[-1] != add_key.shape[-1]:
        raise ValueError(f"Q and additional K head dims must match, got {query.shape[-1]} and {add_key.shape[-1]}.")
    if query.shape[0] != add_key.shape[0] or query.shape[0] != add_value.shape[0]:
        raise ValueError("Q, additional K, and additional V must match in batch size.")
    if add_key.shape[1] != add_value.shape[1]:
        raise ValueError(
            f"Additional K and V must match in sequence length, got {add_key.shape[1]} and {add_value.shape[1]}."
        )
    if key.shape[-2] != add_key.shape[-2] or value.shape[-2] != add_value.shape[-2]:
        raise ValueError("Additional key/value tokens must match the self attention key/value in number of heads.")
    if key.shape[-1] != add_key.shape[-1] or value.shape[-1] != add_value.shape[-1]:
        raise ValueError("Additional key/value tokens must match the self attention key/value in head dim.")
    _head_checks(query, key, value)


def _dim_arg(name: str, na_dim: int, value: Any, minimum: int, default: Optional[int]) -> DimensionType:
    if value is None and default is not None:
        return tuple([default] * na_dim)
    if (
        isinstance(value, Sequence)
        and len(value) == na_dim
        and all(isinstance(x, int) and not isinstance(x, bool) and x >= minimum for x in value)
    ):
        return tuple(int(x) for x in value)
    if isinstance(value, int) and not isinstance(value, bool) and value >= minimum:
        return tuple([int(value)] * na_dim)
    raise ValueError(
        f"Invalid value for `{name}`; expected an integer or a tuple of {na_dim} integers, all >= {minimum}, "
        f"got {type(value)=}, {value=}."
    )


def check_kernel_size_arg(na_dim: int, kernel_size: Any) -> DimensionType:
    return _dim_arg("kernel_size", na_dim, kernel_size, 2, None)


def check_stride_arg(na_dim: int, stride: Any) -> DimensionType:
    return _dim_arg("stride", na_dim, stride, 1, 1)


def check_dilation_arg(na_dim: int, dilation: Any) -> DimensionType:
    return _dim_arg("dilation", na_dim, dilation, 1, 1)


def check_causal_arg(na_dim: int, is_causal: Any) -> CausalArgType:
    if is_causal is None:
        return tuple([False] * na_dim)
    if isinstance(is_causal, Sequence) and len(is_causal) == na_dim and all(isinstance(c, bool) for c in is_causal):
        return tuple(bool(c) for c in is_causal)
    if isinstance(is_causal, bool):
        return tuple([is_causal] * na_dim)
    raise ValueError(
        f"Invalid value for `is_causal`; expected a boolean or a tuple of {na_dim} booleans, "
        f"got {type(is_causal)=}, {is_causal=}."
    )


def check_all_args(na_dim: int, kernel_size: Any, stride: Any, dilation: Any, is_causal: Any):
    assert 0 < na_dim < 4
    return (
        check_kernel_size_arg(na_dim, kernel_size),
        check_stride_arg(na_dim, stride),
        check_dilation_arg(na_dim, dilation),
        check_causal_arg(na_dim, is_causal),
    )


def check_args_against_input(input_tensor: Tensor, kernel_size, stride, dilation, is_causal):
    na_dim = input_tensor.dim() - 3
    input_size = tuple(input_tensor.shape[1 : 1 + na_dim])
    if any(k * d > x for x, k, d in zip(input_size, kernel_size, dilation)):
        raise ValueError(
            "The product of kernel size and dilation cannot be larger than input size along any dimension, "
            f"got {input_size=}, {kernel_size=}, {dilation=}."
        )
    if any(s > k for k, s in zip(kernel_size, stride)):
        raise ValueError(f"Stride cannot be larger than kernel size along any dimension, got {kernel_size=}, {stride=}.")


def is_self_attention(input_tensor: Tensor, kernel_size, is_causal, has_additional_attention: bool) -> bool:
    na_dim = input_tensor.dim() - 3
    input_size = tuple(input_tensor.shape[1 : 1 + na_dim])
    # 1-D with a full window is standard (causal or not) attention, unless extra non-causal context follows.
    if na_dim == 1 and not has_additional_attention:
        return kernel_size[0] == input_size[0]
    return all(k == x and not c for x, k, c in zip(input_size, kernel_size, is_causal))


def check_tile_shape(tile_shape: Any, na_dim: int, name: str) -> DimensionType:
    if (
        isinstance(tile_shape, Sequence)
        and len(tile_shape) == na_dim
        and all(isinstance(x, int) and not isinstance(x, bool) and x > 0 for x in tile_shape)
    ):
        return tuple(int(x) for x in tile_shape)
    raise ValueError(f"Invalid `{name}`; expected a tuple of {na_dim} positive integers, got {tile_shape!r}.")
