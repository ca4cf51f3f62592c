"""Host tests of the Bedenex design: the config reader (loop expansion, tensor names and shapes) against the tests' own checkpoints, and hand
cases of the float64 model the GPU tests compare the engine with."""
import numpy as np

from lmdeploy_amd.turbomind import layered
from tests import bedenex_oracle as bo


def _cfg():
    return bo.make_config(48, 61, [bo.attention_layer(4, 2, 8, 16, 0.3, 10, bo.dense(40)),
                                   bo.latent_layer(3, 8, 4, 8, 16, 0.2, mlp=bo.moe(4, 2, 24)),
                                   bo.attention_layer(2, 2, 8, 8, 0.4, 0),
                                   bo.latent_layer(2, 4, 8, 4, 24, 0.25, 500.0, bo.dense(32))], loop=(1, 3, 3))


def test_reader_expands_the_loop_into_layer_runs():
    mc = layered.FAMILIES['Bedenex'](_cfg())
    assert [bo.layer_runs(_cfg())[i][0] for i in range(8)] == [0, 1, 2, 1, 2, 1, 2, 3]
    assert mc.names == ['l0.', 'l1.', 'l2.', 'l1.', 'l2.', 'l1.', 'l2.', 'l3.'] and mc.loop_times == 3
    assert [s.weights_of for s in mc.layers] == [-1, -1, -1, 1, 2, 1, 2, -1]
    assert [s.loop_pass for s in mc.layers] == [-1, 0, -1, 1, -1, 2, -1, -1]
    a, l = mc.layers[0], mc.layers[1]
    assert (a.mixer, a.chunk, a.qk_unit_norm, a.v_unit_norm, a.dist_bias, a.out_gate, a.sink) == (layered.MIXER_ATTENTION, 10, True, True, True, True, False)
    assert (l.mixer, l.kv_heads, l.kv_rank, l.rot_dim, l.sink, l.mlp, l.experts, l.top, l.act) == (layered.MIXER_LATENT, 1, 16, 4, True, layered.MLP_MOE, 4, 2,
                                                                                                layered.ACT_SILU)
    assert mc.layers[2].chunk == 0 and mc.layers[2].mlp == layered.MLP_NONE and a.act == layered.ACT_GELU_TANH
    assert all(s.one_norm and s.resid_gate for s in mc.layers)


def test_reader_without_a_loop_and_with_a_loop_over_everything():
    c = _cfg()
    del c['loop']
    mc = layered.FAMILIES['Bedenex'](c)
    assert mc.loop_times == 0 and all(s.loop_pass < 0 and s.weights_of < 0 for s in mc.layers) and 'loop.in' not in mc.tensor_shapes()
    c['loop'] = {'start': 0, 'stop': 4, 'times': 1}
    mc = layered.FAMILIES['Bedenex'](c)
    assert [s.loop_pass for s in mc.layers] == [0, -1, -1, -1] and mc.tensor_shapes()['loop.step'] == (1, 48)


def test_tensor_shapes_are_the_checkpoint_s():
    cfg = _cfg()
    w = bo.make_weights(cfg, 0)
    mc = layered.FAMILIES['Bedenex'](cfg)
    want = {}
    for name, shape in mc.tensor_shapes().items():
        if name[0] == 'l' and name[1].isdigit():
            run, leaf = name[1:].split('.', 1)
            name = mc.tensor_name(int(run), leaf)
        want[name] = tuple(shape)
    assert want == {k: tuple(np.shape(v)) for k, v in w.items()}


def test_safetensors_round_trip(tmp_path):
    cfg = _cfg()
    w = bo.make_weights(cfg, 1)
    bo.write_checkpoint(str(tmp_path), cfg, w)
    t = layered.read_safetensors(str(tmp_path / 'model.safetensors'))
    assert layered.is_layered(str(tmp_path)) and set(t) == set(w)
    dt, shp, data = t['l1.mix.uk']
    assert dt == 'BF16' and shp == (24, 16) and np.array_equal(np.frombuffer(data, np.uint16).reshape(shp), bo.bf16_bits(w['l1.mix.uk']))


# ---- the oracle's hand cases ---------------------------------------------------------------------------------------------------------
def test_rotation_turns_pairs_and_depends_on_distance_only():
    rng = np.random.default_rng(0)
    x, y = rng.normal(0, 1, (1, 8)), rng.normal(0, 1, (1, 8))
    assert np.allclose(bo.rotate_half(x, [0], 100.0), x)
    r = bo.rotate_half(np.array([[1.0, 0, 0, 0, 0, 0, 0, 0]]), [3], 100.0)[0]           # channel 0 pairs with channel 4, frequency 1
    assert np.allclose(r, [np.cos(3.0), 0, 0, 0, np.sin(3.0), 0, 0, 0])
    r = bo.rotate_half(np.array([[0, 1.0, 0, 0, 0, 0, 0, 0]]), [5], 100.0)[0]           # channel 1: frequency 100^(-2/8)
    assert np.allclose(r[[1, 5]], [np.cos(5 * 100 ** -0.25), np.sin(5 * 100 ** -0.25)])
    d = [(bo.rotate_half(x, [p], 50.0) @ bo.rotate_half(y, [p - 4], 50.0).T).item() for p in (4, 9, 300)]
    assert np.allclose(d, d[0])


def test_chunks_hide_everything_before_the_query_s_own():
    rng = np.random.default_rng(1)
    T, W = 12, 16
    m = {'heads': 2, 'kv_heads': 1, 'dim': 4, 'vdim': 4, 'scale': 1.0, 'mask': {'size': 5}}
    t = {k: rng.normal(0, 1, s) for k, s in (('q', (8, W)), ('k', (4, W)), ('v', (4, W)), ('g', (2, W)), ('o', (W, 8)))}
    t['r1'], t['r2'] = np.array([0.5, 0.0]), np.array([0.3, 0.3])
    h = rng.normal(0, 1, (T, W))
    out = bo.chunk_attention(h, t, m, 1e-6)
    h2 = h.copy()
    h2[:5] = rng.normal(0, 1, (5, W))                         # another first chunk ...
    out2 = bo.chunk_attention(h2, t, m, 1e-6)
    assert np.allclose(out[5:], out2[5:]) and not np.allclose(out[:5], out2[:5])      # ... changes nothing behind it
    v = bo.unit_rms((h @ t['v'].T).reshape(T, 1, 4), 1e-6)[:, 0]
    first = (np.concatenate([v[5], v[5]]) * np.repeat(bo.sigmoid(h[5] @ t['g'].T), 4)) @ t['o'].T
    assert np.allclose(out[5], first)                           # the first row of a chunk sees itself only


def test_distance_penalty_and_sink_lower_the_weights():
    s = np.zeros((3, 3))
    vis = np.tril(np.ones((3, 3), bool))
    p = bo.softmax_rows(s, vis)
    assert np.allclose(p[2], [1 / 3] * 3)
    p = bo.softmax_rows(s, vis, sink=np.log(3.0))               # the sink counts like three more keys without a value
    assert np.allclose(p[2], [1 / 6] * 3) and np.isclose(p[0, 0], 0.25)
    pen = -1.0 * np.log(1.0 + 1.0 * np.array([2.0, 1.0, 0.0]))  # r1 = r2 = 1: weights 1/3 : 1/2 : 1
    p = bo.softmax_rows(pen[None, :].repeat(3, 0), vis)
    assert np.allclose(p[2], np.array([1 / 3, 1 / 2, 1]) / (11 / 6))


def test_experts_are_chosen_by_score_and_scale_their_input():
    rng = np.random.default_rng(2)
    W, F = 6, 5
    t = {'router': np.array([[1.0] + [0] * 5, [2.0] + [0] * 5, [-1.0] + [0] * 5])}
    for e in range(3):
        t[f'e{e}.gate'], t[f'e{e}.up'], t[f'e{e}.down'] = rng.normal(0, 1, (F, W)), rng.normal(0, 1, (F, W)), rng.normal(0, 1, (W, F))
    h = rng.normal(0, 1, (2, W))
    h[0, 0], h[1, 0] = 1.0, -1.0                               # logits (1, 2, -1) and (-1, -2, 1): experts {1, 0} and {2, 0}

    def expert(e, z):
        return (bo.silu(z @ t[f'e{e}.gate'].T) * (z @ t[f'e{e}.up'].T)) @ t[f'e{e}.down'].T
    out = bo.moe_ff(h, t, {'router': {'experts': 3, 'top': 2}})
    assert np.allclose(out[0], expert(1, bo.sigmoid(2.0) * h[0]) + expert(0, bo.sigmoid(1.0) * h[0]))
    assert np.allclose(out[1], expert(2, bo.sigmoid(1.0) * h[1]) + expert(0, bo.sigmoid(-1.0) * h[1]))
    out1 = bo.moe_ff(h, t, {'router': {'experts': 3, 'top': 1}})
    assert np.allclose(out1[0], expert(1, bo.sigmoid(2.0) * h[0]))


def test_a_loop_pass_starts_from_the_stream_and_the_embedding_output():
    cfg = _cfg()
    w = bo.make_weights(cfg, 3)
    toks = [3, 9, 27, 20]
    _, trail = bo.forward(cfg, w, toks, True)
    x0 = w['embed'][toks]
    x = np.concatenate([trail[2], x0], -1) @ w['loop.in'].T + w['loop.step'][1]      # what pass 1 (the fourth layer run) starts from
    assert np.allclose(bo.block(x, w, 1, cfg['layers'][1], cfg['norm']['eps']), trail[3])
