"""Mirror of the parts of ``fla.modules`` that sit either side of the chunk operators in the
layers: l2 normalisation of q/k, the gated output norms and the short causal convolution."""
from .convolution import ShortConvolution, causal_conv1d, causal_conv1d_update
from .fused_norm_gate import (FusedLayerNormSwishGate, FusedRMSNormSwishGate, LayerNormSwishGateFn,
                              layer_norm_swish_gate_fn, rms_norm_swish_gate_fn)
from .gate_activations import gdn_gate, gdn_gate_bwd, gdn_gate_fwd, gla_gate, gla_gate_bwd, gla_gate_fwd
from .l2norm import L2NormFunction, l2_norm, l2norm_bwd, l2norm_fwd

__all__ = [
    "ShortConvolution", "causal_conv1d", "causal_conv1d_update",
    "FusedLayerNormSwishGate", "FusedRMSNormSwishGate", "LayerNormSwishGateFn",
    "layer_norm_swish_gate_fn", "rms_norm_swish_gate_fn",
    "L2NormFunction", "l2_norm", "l2norm_fwd", "l2norm_bwd",
    "gla_gate", "gla_gate_fwd", "gla_gate_bwd", "gdn_gate", "gdn_gate_fwd", "gdn_gate_bwd",
]
