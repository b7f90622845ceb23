from .chunk import chunk_simple_gla
from .fused_recurrent import fused_recurrent_simple_gla

__all__ = ['chunk_simple_gla', 'fused_recurrent_simple_gla']
