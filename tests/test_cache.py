"""CPU: the state carrier between calls (interface of fla/models/utils.py:11-143)."""
import sys
import os

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), '..', 'flash-linear-attention_amd'))


def _cache(**kw):
    from fla_amd.models import Cache
    return Cache(**kw)


def test_update_appends_then_swaps_pointer():
    c = _cache()
    assert len(c) == 0 and c.get_seq_length() == 0 and c.get_max_length() is None
    with pytest.raises(KeyError):
        c[0]
    s0, s1 = torch.zeros(2, 3), torch.ones(2, 3)
    st = c.update(recurrent_state=s0, conv_state=(torch.zeros(1),), layer_idx=0, offset=7)
    assert st is c[0] and st['recurrent_state'] is s0 and st['attn_state'] is None and st['ffn_state'] is None
    c.update(recurrent_state=s1, layer_idx=1, offset=7)       # only layer 0 counts tokens
    assert len(c) == 2 and c.get_seq_length() == 7 and c.get_seq_length(5) == 0
    s2 = torch.full((2, 3), 2.0)
    c.update(recurrent_state=s2, layer_idx=0, offset=1)
    assert c[0]['recurrent_state'] is s2 and c.get_seq_length() == 8     # pointer swap, as in the reference
    assert [s is t for s, t in zip(c, c.states)] == [True, True]
    legacy = c.to_legacy_cache()
    d = type(c).from_legacy_cache(legacy, seen_tokens=8)
    assert len(d) == 2 and d[1]['recurrent_state'] is s1 and d.get_seq_length() == 8


def test_persistent_keeps_the_buffer():
    c = _cache(persistent=True)
    buf = torch.zeros(2, 3)
    c.update(recurrent_state=buf, conv_state=(torch.zeros(4), None), layer_idx=0, offset=3)
    conv0 = c[0]['conv_state'][0]
    c.update(recurrent_state=torch.ones(2, 3), conv_state=(torch.ones(4), None), layer_idx=0)
    assert c[0]['recurrent_state'] is buf and torch.equal(buf, torch.ones(2, 3))      # copied in, same storage
    assert c[0]['conv_state'][0] is conv0 and torch.equal(conv0, torch.ones(4)) and c[0]['conv_state'][1] is None
    c.update(recurrent_state=buf, layer_idx=0)                                         # in-place caller: no copy needed
    assert c[0]['recurrent_state'] is buf
    other = torch.ones(4, 3)
    c.update(recurrent_state=other, layer_idx=0)                                       # another shape replaces
    assert c[0]['recurrent_state'] is other


def test_attention_window():
    c = _cache()
    k, v = torch.arange(12.).view(1, 1, 6, 2), -torch.arange(12.).view(1, 1, 6, 2)
    c.update(attn_state=(k, v), layer_idx=0, offset=6, cache_kwargs=dict(window_size=4))
    assert c[0]['attn_state'][0].shape[-2] == 4 and torch.equal(c[0]['attn_state'][0], k[..., -4:, :])
    nk, nv = torch.full((1, 1, 1, 2), 99.), torch.full((1, 1, 1, 2), -99.)
    c.update(attn_state=(nk, nv), layer_idx=0, offset=1, cache_kwargs=dict(window_size=4))
    ks, vs = c[0]['attn_state']
    assert ks.shape[-2] == 4 and torch.equal(ks[..., -1, :], nk[..., 0, :]) and torch.equal(ks[..., :3, :], k[..., -3:, :])
    assert torch.equal(vs[..., -1, :], nv[..., 0, :])
    with pytest.raises(ValueError):
        c.update(attn_state=k, layer_idx=0)
    d = _cache()
    d.update(attn_state=(k, v), layer_idx=0, offset=6, cache_kwargs={})
    d.update(attn_state=(nk, nv), layer_idx=0, offset=1, cache_kwargs={})
    assert d[0]['attn_state'][0].shape[-2] == 7


def test_attention_window_follows_the_reference_lengths():
    """The length rules of fla/models/utils.py:75-111, case by case: the first entry is cut to the window; a window
    that is not full grows by the new tokens and is never cut (a multi-token update may overshoot it); a full
    window is shifted in place in the buffers the cache holds."""
    kw = dict(cache_kwargs=dict(window_size=4))
    tok = lambda a, b: (torch.arange(a, b, dtype=torch.float32).view(1, 1, -1, 1).expand(1, 1, b - a, 2).contiguous(),
                        -torch.arange(a, b, dtype=torch.float32).view(1, 1, -1, 1).expand(1, 1, b - a, 2).contiguous())
    c = _cache()
    c.update(attn_state=tok(0, 3), layer_idx=0, offset=3, **kw)          # prefill shorter than the window
    assert c[0]['attn_state'][0].shape[-2] == 3
    c.update(attn_state=tok(3, 5), layer_idx=0, offset=2, **kw)          # crosses the window boundary: 5, not cut
    assert c[0]['attn_state'][0].shape[-2] == 5
    c.update(attn_state=tok(5, 6), layer_idx=0, offset=1, **kw)          # 5 != window: keeps growing, as the reference does
    assert c[0]['attn_state'][0].shape[-2] == 6
    d = _cache()
    d.update(attn_state=tok(0, 9), layer_idx=0, offset=9, **kw)          # first entry longer than the window: newest 4
    ks, vs = d[0]['attn_state']
    assert ks.shape[-2] == 4 and ks[0, 0, :, 0].tolist() == [5., 6., 7., 8.]
    ptrs = (ks.data_ptr(), vs.data_ptr())
    d.update(attn_state=tok(9, 11), layer_idx=0, offset=2, **kw)         # full window: shifted in place
    ks2, vs2 = d[0]['attn_state']
    assert (ks2.data_ptr(), vs2.data_ptr()) == ptrs
    assert ks2[0, 0, :, 0].tolist() == [7., 8., 9., 10.] and vs2[0, 0, :, 1].tolist() == [-7., -8., -9., -10.]
    d.update(attn_state=tok(11, 15), layer_idx=0, offset=4, **kw)        # a whole window of new tokens
    assert d[0]['attn_state'][0].data_ptr() == ptrs[0] and d[0]['attn_state'][0][0, 0, :, 0].tolist() == [11., 12., 13., 14.]


def test_is_a_transformers_cache_when_transformers_is_there():
    try:
        from transformers.cache_utils import Cache as HFCache
    except Exception:
        pytest.skip("transformers not importable")
    assert isinstance(_cache(), HFCache)
