"""fla_amd: MI355X (gfx950) kernels behind the ``fla.ops`` call surface for the
chunked linear-attention hot path (``chunk_gla``, ``chunk_gated_delta_rule``,
``fused_recurrent_*``).  The module tree mirrors ``fla.ops`` so callers swap
``from fla.ops.gla import chunk_gla`` for ``from fla_amd.ops.gla import chunk_gla``,
or call :func:`install` to rebind the names inside an importable upstream ``fla``.
"""
from . import models, modules, ops  # noqa: F401
from ._backend import lib, lib_path  # noqa: F401

__version__ = '0.1.0'


def install() -> list:
    """Rebind the operators inside an importable upstream ``fla`` package.

    The upstream layers bind the operators by name at import time
    (``fla/layers/gla.py:16``, ``fla/layers/gated_deltanet.py:16-17``), so both
    the ``fla.ops`` packages and the layer modules' globals are patched.
    Returns the list of ``module.attribute`` names that were rebound.
    """
    import importlib
    patched = []
    table = {name: getattr(ops, name) for name in ops.__all__}
    # the steps either side of the operators: fla/modules/l2norm.py, fused_norm_gate.py, convolution.py
    table.update({name: getattr(modules, name) for name in (
        'l2_norm', 'l2norm_fwd', 'l2norm_bwd', 'L2NormFunction', 'FusedRMSNormSwishGate', 'FusedLayerNormSwishGate',
        'rms_norm_swish_gate_fn', 'layer_norm_swish_gate_fn', 'LayerNormSwishGateFn', 'ShortConvolution')})
    targets = ['fla.ops.gla', 'fla.ops.gated_delta_rule', 'fla.ops.delta_rule', 'fla.ops.simple_gla', 'fla.ops.utils',
               'fla.ops', 'fla.layers.gla', 'fla.layers.gated_deltanet', 'fla.layers.hgrn2', 'fla.layers.delta_net',
               'fla.layers.simple_gla', 'fla.modules', 'fla.modules.l2norm', 'fla.modules.fused_norm_gate',
               'fla.modules.convolution']
    for modname in targets:
        try:
            mod = importlib.import_module(modname)
        except Exception:
            continue
        for name, fn in table.items():
            if hasattr(mod, name):
                setattr(mod, name, fn)
                patched.append(f'{modname}.{name}')
    # fla.models.utils.Cache is left alone: the upstream models subclass-check it against
    # transformers' Cache; fla_amd.models.Cache is for callers that drive the operators directly
    return patched
