from .attention import Attention
from .base import KVRequest, StateRequest, StepContext, Workspace
from .block import PreNormBlock
from .linear import Linear
from .mlp import GatedMLP
from .norm import RMSNorm
from .registry import (lookup, register_block, register_feed_forward, register_mixer,
                       register_norm, register_position, unregister)
from .rope import NoPosition, RotaryTable

register_mixer("attention", Attention)
register_feed_forward("gated_mlp", GatedMLP)
register_norm("rmsnorm", RMSNorm)
register_position("rope", RotaryTable)
register_position("none", NoPosition)
register_block("prenorm", PreNormBlock)

__all__ = ["Attention", "KVRequest", "StateRequest", "StepContext", "Workspace", "PreNormBlock",
           "Linear", "GatedMLP", "RMSNorm", "lookup", "register_block", "register_feed_forward",
           "register_mixer", "register_norm", "register_position", "unregister", "NoPosition",
           "RotaryTable"]
