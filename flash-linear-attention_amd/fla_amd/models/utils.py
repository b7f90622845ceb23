"""``Cache``: per-layer states between calls, with the interface of the reference's
``fla.models.utils.Cache`` (``fla/models/utils.py:11-143``): a list of per-layer dicts with the
keys ``recurrent_state``, ``attn_state``, ``conv_state``, ``ffn_state``; ``update`` swaps in what a
layer returns and counts tokens on layer 0.

What differs is where the state lives.  The reference's operators allocate a fresh final state on
every call and ``update`` replaces the pointer (``:94-95``), which rewrites 2 x [N,H,K,V] fp32 of
HBM per layer and decode step and changes addresses under a captured HIP graph.  The decode kernels
here update a state in place (``inplace_state=True``), so ``update`` receives the tensor it already
holds and the buffer (and its address) persists for the whole generation.  With ``persistent=True``
a state of the same shape that arrives in other storage is copied into the held buffer instead of
replacing it, for callers that need stable addresses but cannot run in place.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch


def _same_storage(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.data_ptr() == b.data_ptr() and a.shape == b.shape and a.dtype == b.dtype


# The reference's Cache subclasses transformers' (fla/models/utils.py:11), whose `generate` checks
# `isinstance(past_key_values, Cache)`; do the same wherever transformers is importable.
try:
    from transformers.cache_utils import Cache as _CacheBase
except Exception:   # transformers absent or broken: a plain class serves callers that drive the operators directly
    _CacheBase = object


class Cache(_CacheBase):

    def __init__(self, seen_tokens: int = 0, persistent: bool = False):
        # like the reference, the base class's own constructor is not run: nothing of its per-layer
        # key/value bookkeeping applies; `layers` is left empty for the base class's helpers that walk it
        if _CacheBase is not object:
            try:
                self.layers = []
            except AttributeError:
                pass
        self.states: List[Dict[str, Any]] = []
        self._seen_tokens = seen_tokens  # `generate` reads this to place new tokens
        self.persistent = persistent

    def __getitem__(self, layer_idx: int) -> Dict[str, Any]:
        if layer_idx < len(self):
            return self.states[layer_idx]
        raise KeyError(f"Cache only has {len(self)} layers, attempted to access layer with index {layer_idx}")

    def __iter__(self):
        yield from self.states

    def __len__(self):
        return len(self.states)

    def _keep(self, held: Optional[torch.Tensor], new: torch.Tensor) -> torch.Tensor:
        """The tensor a layer's slot holds after an update with ``new``."""
        if (self.persistent and isinstance(held, torch.Tensor) and isinstance(new, torch.Tensor)
                and held.shape == new.shape and held.dtype == new.dtype and held.device == new.device):
            if not _same_storage(held, new):
                held.copy_(new)
            return held
        return new

    def update(
        self,
        recurrent_state: torch.Tensor = None,
        attn_state: Tuple[torch.Tensor, torch.Tensor] = None,
        conv_state: Tuple[torch.Tensor] = None,
        ffn_state: torch.Tensor = None,
        layer_idx: int = 0,
        offset: Optional[int] = 1,
        cache_kwargs: Optional[Dict[str, Any]] = None,
    ) -> Dict[str, Any]:
        """Store the new states of layer ``layer_idx``; ``offset`` = number of new tokens.
        Returns the layer's dict."""
        if layer_idx == 0:
            self._seen_tokens += offset
        if attn_state is not None:
            if not isinstance(attn_state, (tuple, list)) or len(attn_state) != 2:
                raise ValueError("`attn_state` must be a tuple of two tensors for key/value states")
            # key/value states of softmax-attention layers in hybrid models (outside the linear-attention path;
            # kept for interface parity, fla/models/utils.py:75-111)
            window_size = (cache_kwargs or {}).get('window_size', None)
            input_size = attn_state[0].shape[-2]
            held = self.states[layer_idx].get('attn_state') if layer_idx < len(self.states) else None
            if held is None:
                # first entry of the layer: only the newest `window_size` tokens are kept (in a buffer of the
                # cache's own: it is shifted in place later, which must not reach into the caller's tensor)
                if window_size is not None and input_size >= window_size:
                    attn_state = tuple(x[..., -window_size:, :].clone() for x in attn_state)
            elif window_size is not None and held[0].shape[-2] == window_size and input_size <= window_size:
                # a full window: shift the held buffers left by the new tokens and write those at the end,
                # in the buffers the cache already holds (same addresses from step to step)
                for h, n in zip(held, attn_state):
                    if input_size < window_size:
                        h.copy_(h.roll(-input_size, -2))
                    h[..., -input_size:, :] = n
                attn_state = tuple(held)
            else:
                # a window that is not full yet grows by the new tokens and is not cut
                attn_state = tuple(torch.cat([h, n], -2) for h, n in zip(held, attn_state))
        if len(self.states) <= layer_idx:
            state = dict(recurrent_state=recurrent_state, attn_state=attn_state, conv_state=conv_state,
                         ffn_state=ffn_state)
            self.states.append(state)
            return state
        state = self.states[layer_idx]
        if recurrent_state is not None:
            state['recurrent_state'] = self._keep(state.get('recurrent_state'), recurrent_state)
        if attn_state is not None:
            state['attn_state'] = attn_state
        if conv_state is not None:
            held = state.get('conv_state')
            if isinstance(conv_state, (tuple, list)) and isinstance(held, (tuple, list)) and len(held) == len(conv_state):
                state['conv_state'] = type(conv_state)(
                    None if n is None else self._keep(h, n) for h, n in zip(held, conv_state))
            elif isinstance(conv_state, torch.Tensor):
                state['conv_state'] = self._keep(held, conv_state)
            else:
                state['conv_state'] = conv_state
        if ffn_state is not None:
            state['ffn_state'] = self._keep(state.get('ffn_state'), ffn_state)
        return state

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        """Tokens seen so far (0 while the layer has no entry)."""
        if len(self.states) <= layer_idx:
            return 0
        return self._seen_tokens

    def get_max_length(self) -> Optional[int]:
        """Recurrent states have no maximum length."""
        return None

    def to_legacy_cache(self) -> Tuple:
        return tuple(self.states)

    @classmethod
    def from_legacy_cache(cls, past_key_values: Optional[Tuple] = None, seen_tokens: int = 0) -> 'Cache':
        cache = cls(seen_tokens)
        if past_key_values is not None:
            for layer_state in past_key_values:
                cache.states.append(layer_state)
        return cache
