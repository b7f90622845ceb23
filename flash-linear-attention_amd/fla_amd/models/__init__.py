"""Only the state carrier of ``fla.models``: the ``Cache`` type that hands a layer's recurrent
state from one call to the next (``fla/models/utils.py:11-143``).  The model classes themselves
are unchanged callers and are not part of this package."""
from .utils import Cache

__all__ = ['Cache']
