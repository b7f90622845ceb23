from .chunk import chunk_delta_rule

__all__ = ['chunk_delta_rule']
