from .registry import register_part, part_class, ROLES
from .base import StepContext, Residual, Workspace, Declared
from .linear import Linear, place_matrix, place_projection, place_vector
from . import (norm, position, attention, short_conv, ffn, embedding, block, token_shift, diff_attention,   # registers
               selective_scan, moe, latent_attention, hgrn2, gate, mamba2, gated_delta, retention, mixer_pair)                                                                          # the built-in parts
