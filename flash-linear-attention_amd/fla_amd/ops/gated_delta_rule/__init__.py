from .fused_recurrent import fused_recurrent_gated_delta_rule

__all__ = ['fused_recurrent_gated_delta_rule']
