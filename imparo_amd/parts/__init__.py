from .registry import register_part, part_class, ROLES
from .base import StepContext, Residual, Workspace, Declared
from .linear import Linear, place_matrix, place_vector
from . import norm, position, attention, short_conv, ffn, embedding, block   # registers the built-in parts
