from .chunk import chunk_gla
from .fused_recurrent import fused_recurrent_gla

__all__ = ['chunk_gla', 'fused_recurrent_gla']
