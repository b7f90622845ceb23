from .delta_rule import chunk_delta_rule
from .gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
from .gla import chunk_gla, fused_recurrent_gla
from .simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
from .utils import chunk_global_cumsum, chunk_local_cumsum

__all__ = ['chunk_gla', 'fused_recurrent_gla', 'chunk_gated_delta_rule', 'fused_recurrent_gated_delta_rule',
           'chunk_delta_rule', 'chunk_simple_gla', 'fused_recurrent_simple_gla', 'chunk_local_cumsum', 'chunk_global_cumsum']
