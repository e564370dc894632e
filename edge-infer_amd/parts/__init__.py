from .attention import Attention
from .base import KVRequest, StateRequest, StepContext, Workspace
from .block import OutputNormBlock, PreNormBlock, SandwichBlock
from .delta import GatedDelta
from .latent import LatentAttention
from .linear_attention import LinearAttention
from .linear import Linear
from .mlp import DenseMLP, GatedMLP
from .mlstm import MatrixMemory
from .norm import LayerNorm, RMSNorm
from .parallel import ParallelMixer
from .registry import (lookup, register_block, register_feed_forward, register_mixer,
                       register_norm, register_position, unregister)
from .moe import RoutedMLP
from .rope import NoPosition, RotaryFrequencies, RotaryHalfFrequencies, RotaryTable
from .ssm import StateSpace

register_mixer("attention", Attention)
register_mixer("gated_delta", GatedDelta)
register_mixer("latent_attention", LatentAttention)
register_mixer("mlstm", MatrixMemory)
register_mixer("mamba2", StateSpace)
register_mixer("linear_attention", LinearAttention)
register_mixer("parallel", ParallelMixer)
register_feed_forward("gated_mlp", GatedMLP)
register_feed_forward("dense_mlp", DenseMLP)
register_feed_forward("routed_mlp", RoutedMLP)
register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
register_position("rope", RotaryTable)
register_position("none", NoPosition)
register_position("rope_pairs", RotaryFrequencies)
register_position("rope_half", RotaryHalfFrequencies)
register_block("prenorm", PreNormBlock)
register_block("outnorm", OutputNormBlock)
register_block("sandwich", SandwichBlock)

__all__ = ["Attention", "KVRequest", "StateRequest", "StepContext", "Workspace", "PreNormBlock",
           "OutputNormBlock", "SandwichBlock", "GatedDelta", "LatentAttention", "MatrixMemory", "RotaryFrequencies",
           "RotaryHalfFrequencies", "RoutedMLP", "LayerNorm", "LinearAttention", "ParallelMixer", "StateSpace", "DenseMLP", "Linear", "GatedMLP", "RMSNorm", "lookup", "register_block", "register_feed_forward",
           "register_mixer", "register_norm", "register_position", "unregister", "NoPosition",
           "RotaryTable"]
