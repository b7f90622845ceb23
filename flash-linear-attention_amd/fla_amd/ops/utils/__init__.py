from .cumsum import chunk_local_cumsum

__all__ = ['chunk_local_cumsum']
