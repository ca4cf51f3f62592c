"""Host-side tests of the layer-list model family: config reader, checkpoint reader, scheduler sessions, and the oracle's own
mechanisms against hand-computed cases (no GPU)."""
import ctypes as C
import math

import numpy as np
import pytest

from lmdeploy_amd import _ffi
from lmdeploy_amd.turbomind import layered
from tests import layered_oracle as lo


def _layer(**kw):
    d = dict(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.25, softcap=12.0, qtemp_coef=0.2, qtemp_every=5, sink=True, ff=48, weights_of=-1)
    d.update(kw)
    return d


def test_config_reader_and_tensor_names(tmp_path):
    cfg = lo.make_config(40, 70, [_layer(), _layer(weights_of=0), _layer(ff=0, heads=3, kv_heads=3, dim=8, vdim=24)])
    w = lo.make_weights(cfg, 1)
    lo.write_checkpoint(str(tmp_path), cfg, w)
    assert layered.is_layered(str(tmp_path))
    c = layered.read_layered_config(str(tmp_path))
    assert (c.width, c.vocab, len(c.layers), c.norm_offset) == (40, 70, 3, 1.0)
    assert c.layers[1].weights_of == 0 and c.layers[0].weights_of == -1
    assert c.layers[2].mlp == layered.MLP_NONE and c.layers[2].ff == 0 and c.layers[0].ff == 48
    assert c.layers[0].softcap == 12.0 and c.layers[0].qtemp_every == 5.0 and abs(c.layers[0].qtemp_coef - 0.2) < 1e-12
    shapes = c.tensor_shapes()
    assert set(shapes) == set(w) and all(tuple(shapes[k]) == w[k].shape for k in w)      # a weight-sharing layer has no tensors
    t = layered.read_safetensors(str(tmp_path / 'model.safetensors'))
    for k in w:
        dt, shp, data = t[k]
        assert dt == 'BF16' and tuple(shp) == w[k].shape
        assert np.array_equal(lo.from_bf16_bits(np.frombuffer(data, '<u2')).reshape(w[k].shape), w[k])
    native, keep = c.native('float32')
    assert native.n_layers == 3 and native.dtype == 1 and native.layers[2].heads == 3


def test_unknown_family_is_refused(tmp_path):
    (tmp_path / 'config.json').write_text('{"architecture": "Nope"}')
    assert not layered.is_layered(str(tmp_path))
    with pytest.raises(NotImplementedError):
        layered.read_layered_config(str(tmp_path))


def test_scheduler_sessions_take_blocks_as_they_grow_and_give_them_back(tm):
    s = C.c_void_p()
    _ffi.check(tm.tm_sched_create(C.byref(s), 2, 5, 64 * 5))
    free = lambda: (lambda a, w, f: (tm.tm_sched_counts(s, C.byref(a), C.byref(w), C.byref(f)), f.value)[1])(C.c_int(), C.c_int(), C.c_int())
    a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
    _ffi.check(tm.tm_sched_session_open(s, C.byref(a)))
    _ffi.check(tm.tm_sched_session_open(s, C.byref(b)))
    assert tm.tm_sched_session_open(s, C.byref(c)) == 2            # both slots taken
    assert free() == 5                                             # nothing is reserved at admission
    _ffi.check(tm.tm_sched_session_grow(s, a, 64))
    assert free() == 4
    _ffi.check(tm.tm_sched_session_grow(s, a, 65))                 # crossing a block border takes one more
    _ffi.check(tm.tm_sched_session_grow(s, a, 128))                # ... and stays inside it up to the next border
    assert free() == 3
    _ffi.check(tm.tm_sched_session_grow(s, b, 129))
    assert free() == 0
    assert tm.tm_sched_session_grow(s, a, 129) == 11               # pool exhausted: nothing taken
    assert free() == 0
    _ffi.check(tm.tm_sched_session_close(s, b))
    assert free() == 3
    _ffi.check(tm.tm_sched_session_open(s, C.byref(c)))            # the slot is free again
    _ffi.check(tm.tm_sched_session_grow(s, c, 64 * 3))
    assert free() == 0
    assert tm.tm_sched_session_grow(s, c, 64 * 5 + 1) == 1         # beyond session_len
    assert tm.tm_sched_session_close(s, b) == 1                    # closed twice
    _ffi.check(tm.tm_sched_session_close(s, a))
    _ffi.check(tm.tm_sched_session_close(s, c))
    assert free() == 5
    _ffi.check(tm.tm_sched_destroy(s))


def test_oracle_mechanisms_on_hand_cases():
    # temperature: steps of `every` positions, counted from position `every - 1`
    assert lo.query_temperature(0, 0.5, 4) == 1.0 and lo.query_temperature(2, 0.5, 4) == 1.0
    assert lo.query_temperature(3, 0.5, 4) == pytest.approx(1 + 0.5 * math.log(2)) and lo.query_temperature(7, 0.5, 4) == pytest.approx(1 + 0.5 * math.log(3))
    assert lo.soft_cap(np.array([1e9]), 5.0)[0] == pytest.approx(5.0) and lo.soft_cap(np.array([0.01]), 5.0)[0] == pytest.approx(0.01, rel=1e-5)
    # sink: counts once in the denominator, has no value
    w = lo.sink_softmax(np.array([0.0, 0.0]), 0.0)
    assert np.allclose(w, [1 / 3, 1 / 3])
    assert np.allclose(lo.sink_softmax(np.array([1.0, 2.0]), None).sum(), 1.0)
    assert np.allclose(lo.sink_softmax(np.array([1.0, 2.0]), -1e9), lo.sink_softmax(np.array([1.0, 2.0]), None))
    x = np.array([[3.0, 4.0]])
    assert np.allclose(lo.rms_norm(x, np.array([0.0, 1.0]), 0.0, 1.0), [[3 / math.sqrt(12.5), 8 / math.sqrt(12.5)]])
    assert np.allclose(lo.relu2_mlp(np.array([[1.0, -1.0]]), np.array([[1.0, 0.0], [0.0, 1.0]]), np.array([[1.0, 1.0]])), [[1.0]])
    # bf16 helper: round to nearest even on the 16 dropped bits
    assert lo.to_bf16_bits(np.array([1.0, 1.00390625, 1.01171875], np.float32)).tolist() == [0x3f80, 0x3f80, 0x3f82]


def test_oracle_prefill_equals_token_by_token():
    cfg = lo.make_config(24, 30, [_layer(heads=2, kv_heads=1, dim=8, vdim=4, ff=16, qtemp_every=3)])
    w = lo.make_weights(cfg, 3)
    toks = [1, 5, 9, 2, 7, 7, 3]
    full = lo.forward(cfg, w, toks)[0]
    for n in range(1, len(toks) + 1):
        assert np.allclose(lo.forward(cfg, w, toks[:n])[0][-1], full[n - 1], atol=1e-10)
