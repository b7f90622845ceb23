from .cumsum import chunk_global_cumsum, chunk_local_cumsum

__all__ = ['chunk_global_cumsum', 'chunk_local_cumsum']
