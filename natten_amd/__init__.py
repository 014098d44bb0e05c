"""natten_amd: MI355X (gfx950) fused neighborhood attention forward with the NATTEN API."""

from .attn_merge import merge_attentions
from .functional import attention, na1d, na2d, na3d, neighborhood_attention_generic
from .modules import NeighborhoodAttention1D, NeighborhoodAttention2D, NeighborhoodAttention3D
from .tile_config import check_fna_forward_config, get_all_tile_shapes
from .token_permute import token_permute_operation, token_unpermute_operation

__version__ = "0.1.0"

__all__ = [
    "NeighborhoodAttention1D",
    "NeighborhoodAttention2D",
    "NeighborhoodAttention3D",
    "attention",
    "na1d",
    "na2d",
    "na3d",
    "neighborhood_attention_generic",
    "merge_attentions",
    "token_permute_operation",
    "token_unpermute_operation",
    "check_fna_forward_config",
    "get_all_tile_shapes",
]
