"""CPU: ``fla_amd.install()`` rebinds the operators inside an importable upstream ``fla`` — exercised on
stub ``fla.*`` modules placed in ``sys.modules`` (the reference itself is not imported)."""
import sys
import types

import pytest


def _stub(name, **attrs):
    mod = types.ModuleType(name)
    for k, v in attrs.items():
        setattr(mod, k, v)
    return mod


@pytest.fixture
def stub_fla(monkeypatch):
    sentinel = lambda name: (lambda *a, **k: name)      # what the upstream Triton entry points stand for
    mods = {
        'fla': _stub('fla'),
        'fla.ops': _stub('fla.ops', chunk_gla=sentinel('ops.chunk_gla'), unrelated_op=sentinel('ops.unrelated')),
        'fla.ops.gla': _stub('fla.ops.gla', chunk_gla=sentinel('gla.chunk_gla'),
                             fused_recurrent_gla=sentinel('gla.fused_recurrent_gla'),
                             fused_chunk_gla=sentinel('gla.fused_chunk_gla')),
        'fla.ops.gated_delta_rule': _stub('fla.ops.gated_delta_rule',
                                          chunk_gated_delta_rule=sentinel('gdr.chunk'),
                                          fused_recurrent_gated_delta_rule=sentinel('gdr.recurrent')),
        'fla.ops.utils': _stub('fla.ops.utils', chunk_local_cumsum=sentinel('utils.cumsum'), softmax_fwd=sentinel('x')),
        'fla.layers': _stub('fla.layers'),
        # the layers bind the operators by name at import time (fla/layers/gla.py:16, gated_deltanet.py:13-17)
        'fla.layers.gla': _stub('fla.layers.gla', chunk_gla=sentinel('layer.chunk_gla'),
                                fused_recurrent_gla=sentinel('layer.fused_recurrent_gla'),
                                fused_chunk_gla=sentinel('layer.fused_chunk_gla'),
                                FusedRMSNormSwishGate=object, ShortConvolution=object),
        'fla.layers.gated_deltanet': _stub('fla.layers.gated_deltanet',
                                           chunk_gated_delta_rule=sentinel('layer.gdr.chunk'),
                                           fused_recurrent_gated_delta_rule=sentinel('layer.gdr.recurrent'),
                                           l2_norm=sentinel('layer.l2'), ShortConvolution=object,
                                           FusedRMSNormSwishGate=object),
        'fla.modules': _stub('fla.modules', ShortConvolution=object, FusedRMSNormSwishGate=object, RMSNorm=object),
        'fla.modules.l2norm': _stub('fla.modules.l2norm', l2_norm=sentinel('mod.l2'), l2norm_fwd=sentinel('mod.l2f')),
    }
    for name, mod in mods.items():
        monkeypatch.setitem(sys.modules, name, mod)
    for name, mod in mods.items():           # parent packages expose their children as attributes
        parent, _, child = name.rpartition('.')
        if parent:
            setattr(mods[parent], child, mod)
    # modules install() looks for but this stub tree does not have must fail to import, not resolve elsewhere
    for missing in ('fla.ops.delta_rule', 'fla.ops.simple_gla', 'fla.layers.hgrn2', 'fla.layers.delta_net',
                    'fla.layers.simple_gla', 'fla.modules.fused_norm_gate', 'fla.modules.convolution'):
        monkeypatch.setitem(sys.modules, missing, None)
    return mods


def test_install_rebinds_ops_layers_and_modules(stub_fla):
    import fla_amd
    from fla_amd import modules, ops
    untouched = (stub_fla['fla.ops.gla'].fused_chunk_gla, stub_fla['fla.ops'].unrelated_op,
                 stub_fla['fla.ops.utils'].softmax_fwd, stub_fla['fla.modules'].RMSNorm)
    patched = fla_amd.install()
    assert stub_fla['fla.ops.gla'].chunk_gla is ops.chunk_gla
    assert stub_fla['fla.ops.gla'].fused_recurrent_gla is ops.fused_recurrent_gla
    assert stub_fla['fla.ops'].chunk_gla is ops.chunk_gla
    assert stub_fla['fla.ops.gated_delta_rule'].chunk_gated_delta_rule is ops.chunk_gated_delta_rule
    assert stub_fla['fla.ops.gated_delta_rule'].fused_recurrent_gated_delta_rule is ops.fused_recurrent_gated_delta_rule
    assert stub_fla['fla.ops.utils'].chunk_local_cumsum is ops.chunk_local_cumsum
    # the names the layer modules imported are rebound inside those modules as well
    assert stub_fla['fla.layers.gla'].chunk_gla is ops.chunk_gla
    assert stub_fla['fla.layers.gla'].fused_recurrent_gla is ops.fused_recurrent_gla
    assert stub_fla['fla.layers.gated_deltanet'].chunk_gated_delta_rule is ops.chunk_gated_delta_rule
    assert stub_fla['fla.layers.gated_deltanet'].l2_norm is modules.l2_norm
    assert stub_fla['fla.layers.gated_deltanet'].ShortConvolution is modules.ShortConvolution
    assert stub_fla['fla.layers.gla'].FusedRMSNormSwishGate is modules.FusedRMSNormSwishGate
    assert stub_fla['fla.modules'].ShortConvolution is modules.ShortConvolution
    assert stub_fla['fla.modules.l2norm'].l2_norm is modules.l2_norm
    # what this library does not provide stays as it was
    assert untouched == (stub_fla['fla.ops.gla'].fused_chunk_gla, stub_fla['fla.ops'].unrelated_op,
                         stub_fla['fla.ops.utils'].softmax_fwd, stub_fla['fla.modules'].RMSNorm)
    assert stub_fla['fla.layers.gla'].fused_chunk_gla() == 'layer.fused_chunk_gla'
    assert 'fla.ops.gla.chunk_gla' in patched and 'fla.layers.gla.chunk_gla' in patched
    assert all(not p.startswith('fla.layers.hgrn2') for p in patched)          # absent modules are skipped
    assert sorted(set(patched)) == sorted(patched)


def test_install_without_upstream_is_a_no_op(monkeypatch):
    import fla_amd
    for name in [m for m in sys.modules if m == 'fla' or m.startswith('fla.')]:
        monkeypatch.delitem(sys.modules, name)
    monkeypatch.setitem(sys.modules, 'fla', None)      # importing fla fails
    assert fla_amd.install() == []
