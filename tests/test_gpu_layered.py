"""GPU tests of the layer-list model family against the plain float64 oracle (tests/layered_oracle.py): the new operators alone
(fp32 RMSNorm pair, dense linears, general paged attention: row and tile kernels), then the engine -- whole prompts, token-by-token
decoding, portions, unequal batches, reused blocks and slots, long decoding, and greedy generation through the static batch, the
scheduler and the pipeline.  Configurations and weights are the tests' own."""
import ctypes as C
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from lmdeploy_amd import _ffi
from lmdeploy_amd.turbomind import layered
from tests import layered_oracle as lo
from tests.gpu_helpers import dev, host, release_all, st

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _release():
    yield
    release_all()


def bits(x):
    return lo.to_bf16_bits(np.asarray(x, np.float32)).view(np.int16)


def act(x, dtype):
    """float64 values -> device buffer in the activation type (bf16 bits as int16, or fp32)"""
    return dev(bits(x)) if dtype == 0 else dev(np.asarray(x, np.float32))


def read(t, dtype):
    return lo.from_bf16_bits(host(t).view(np.uint16)) if dtype == 0 else host(t).astype(np.float64)


# ---- operators ----------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize('dtype', [0, 1])
def test_rmsnorm_f32_pair(tm, cuda, dtype):
    rng = np.random.default_rng(0)
    for M, H in ((1, 40), (7, 256), (3, 1000)):
        x = rng.normal(0, 3, (M + 2, H)).astype(np.float32)
        w0, w1 = rng.normal(0, 0.2, H).astype(np.float32), rng.normal(0, 0.2, H).astype(np.float32)
        rows = rng.permutation(M + 2)[:M].astype(np.int32)
        ld = (H + 31) // 32 * 32
        y0, y1 = act(np.zeros((M, ld)), dtype), act(np.zeros((M, ld)), dtype)
        _ffi.check(tm.tm_rmsnorm_f32(y0.data_ptr(), y1.data_ptr(), ld, 2 if dtype == 0 else 4, dev(x).data_ptr(), dev(rows).data_ptr(),
                                     dev(w0).data_ptr(), dev(w1).data_ptr(), 1.0, 1e-5, M, H, st()))
        tol = 1e-2 if dtype == 0 else 2e-6
        for y, w in ((y0, w0), (y1, w1)):
            ref = lo.rms_norm(x[rows].astype(np.float64), w.astype(np.float64), 1e-5, 1.0)
            assert np.abs(read(y, dtype)[:, :H] - ref).max() <= tol * np.abs(ref).max()


@pytest.mark.parametrize('dtype', [0, 1])
def test_dense_linear_every_row_count_and_epilogue(tm, cuda, dtype):
    rng = np.random.default_rng(1)
    for K, N in ((72, 50), (256, 384), (40, 200)):
        w = lo.bf16(rng.normal(0, 1 / math.sqrt(K), (N, K)))
        h = C.c_void_p()
        _ffi.check(tm.tm_dense_create(C.byref(h), K, N, dtype, dev(bits(w)).data_ptr(), st()))
        ldx = (K + 31) // 32 * 32 + 32
        for M in (1, 5, 16, 17, 32, 33, 100, 130):
            xv = rng.normal(0, 1, (M, K))
            xv = lo.bf16(xv) if dtype == 0 else xv.astype(np.float32).astype(np.float64)
            xp = np.full((M, ldx), 7.0)        # pad columns hold finite junk: they meet zero weights
            xp[:, :K] = xv
            ref = xv @ w.T
            tol = (2e-2 if dtype == 0 else 3e-6) * np.abs(ref).max()
            y = act(np.zeros((M, N + 3)), dtype)
            _ffi.check(tm.tm_dense_forward(h, act(xp, dtype).data_ptr(), ldx, y.data_ptr(), N + 3, M, 0, 1.0, st()))
            got = read(y, dtype)
            assert np.abs(got[:, :N] - ref).max() <= tol and np.all(got[:, N:] == 0)      # nothing is written beyond column N
            _ffi.check(tm.tm_dense_forward(h, act(xp, dtype).data_ptr(), ldx, y.data_ptr(), N + 3, M, 1, 1.0, st()))
            r2 = np.maximum(ref, 0) ** 2
            assert np.abs(read(y, dtype)[:, :N] - r2).max() <= (4e-2 if dtype == 0 else 1e-5) * max(1.0, np.abs(r2).max())
            res = rng.normal(0, 1, (M, N)).astype(np.float32)
            yr = dev(res.copy())
            _ffi.check(tm.tm_dense_forward(h, act(xp, dtype).data_ptr(), ldx, yr.data_ptr(), N, M, 2, 0.25, st()))
            assert np.abs(host(yr) - (res + 0.25 * ref)).max() <= tol
            _ffi.check(tm.tm_dense_forward(h, act(xp, dtype).data_ptr(), ldx, yr.data_ptr(), N, M, 3, 3.0, st()))
            assert np.abs(host(yr) - 3.0 * ref).max() <= 3 * tol
        _ffi.check(tm.tm_dense_destroy(h))


class Cache:
    """a paged cache in the general layout (per block: keys [G][64][D], then values transposed [G][V][64]) with shuffled blocks; the
    tests only fix a block's size and where its values start -- every entry is written by the store path under test"""

    def __init__(self, dtype, G, D, V, lens, rng, extra_blocks=3):
        self.dtype, self.G, self.D, self.V, self.lens = dtype, G, D, V, lens
        per = [(n + 63) // 64 for n in lens]
        self.stride = max(per) + 1
        nb = sum(per) + extra_blocks
        self.block_elems = G * 64 * (D + V)
        pool = rng.normal(0, 50, (nb, self.block_elems))       # stale junk everywhere: what is not written must not be read
        order = rng.permutation(nb)
        self.tables, k = [], 0
        for n in per:
            self.tables.append(order[k:k + n].tolist())
            k += n
        self.pool = act(pool, dtype)
        eb = 2 if dtype == 0 else 4
        ptrs = np.zeros((len(lens), self.stride), np.uint64)
        for s, t in enumerate(self.tables):
            for i, b in enumerate(t):
                ptrs[s, i] = self.pool.data_ptr() + b * self.block_elems * eb
        self.ptrs = dev(ptrs.view(np.int64))
        self.v_offset = G * 64 * D * eb
        self.eb = eb


def run_attention(tm, cache, q, k_new, v_new, row_seq, row_pos, cu_q, k_len, spec, sink, kernel, splits=1, prefill=1):
    """store the new rows' keys / values, then attention; q [rows, H * D], k_new [rows, G * D], v_new [rows, G * V] (float64)"""
    dtype, H, G, D, V = cache.dtype, spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    rows = q.shape[0]
    ld = (H * D + G * D + G * V + 31) // 32 * 32
    qkv = np.zeros((rows, ld))
    qkv[:, :H * D], qkv[:, H * D:H * D + G * D], qkv[:, H * D + G * D:H * D + G * D + G * V] = q, k_new, v_new
    qkv_d = act(qkv, dtype)
    out = act(np.zeros((rows, H * V + 5)), dtype)
    ws = torch.zeros(max(1, tm.tm_general_attention_workspace(rows, H, V, splits) // 4), dtype=torch.float32, device='cuda')
    a = _ffi.GeneralAttn(qkv_d.data_ptr(), out.data_ptr(), ld, H * V + 5, rows, dev(np.asarray(row_seq, np.int32)).data_ptr(),
                         dev(np.asarray(row_pos, np.int32)).data_ptr(), cache.ptrs.data_ptr(), cache.stride, 0, cache.v_offset, cache.eb,
                         H, G, D, V, spec['scale'], spec['softcap'], spec['qtemp_coef'], spec['qtemp_every'],
                         dev(np.asarray(sink, np.float32)).data_ptr() if sink is not None else None, splits, ws.data_ptr(),
                         qkv_d.data_ptr(), ld, H * D, H * D + G * D, 1, kernel, prefill, len(cu_q) - 1, int(np.diff(cu_q).max()),
                         dev(np.asarray(cu_q, np.int32)).data_ptr(), dev(np.asarray(k_len, np.int32)).data_ptr())
    _ffi.check(tm.tm_general_attention(C.byref(a), st()))
    return read(out, dtype)[:, :H * V]


def oracle_attention(q, keys, vals, pos, spec, sink):
    """one query row [H * D] at position pos over keys / values [pos + 1, G, .]"""
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    out = np.zeros((H, V))
    t = lo.query_temperature(pos, spec['qtemp_coef'], spec['qtemp_every']) if spec['qtemp_coef'] else 1.0
    for h in range(H):
        g = h // (H // G)
        s = lo.soft_cap((keys[:pos + 1, g] @ q[h * D:(h + 1) * D]) * t * spec['scale'], spec['softcap'])
        out[h] = lo.sink_softmax(s, float(sink[h]) if sink is not None else None) @ vals[:pos + 1, g]
    return out.reshape(-1)


SPECS = {
    'plain': dict(heads=4, kv_heads=2, dim=32, vdim=16, scale=0.2, softcap=0.0, qtemp_coef=0.0, qtemp_every=1.0),
    'cap': dict(heads=4, kv_heads=2, dim=32, vdim=16, scale=0.9, softcap=3.0, qtemp_coef=0.0, qtemp_every=1.0),
    'temp': dict(heads=4, kv_heads=2, dim=32, vdim=16, scale=0.2, softcap=0.0, qtemp_coef=0.7, qtemp_every=3.0),
    'all_odd': dict(heads=6, kv_heads=2, dim=40, vdim=24, scale=0.15, softcap=8.0, qtemp_coef=0.4, qtemp_every=64.0),
    'one_group': dict(heads=3, kv_heads=3, dim=72, vdim=136, scale=0.1, softcap=30.0, qtemp_coef=0.25, qtemp_every=100.0),
    'unaligned': dict(heads=2, kv_heads=1, dim=20, vdim=12, scale=0.2, softcap=5.0, qtemp_coef=0.1, qtemp_every=7.0),
}


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('name', list(SPECS))
@pytest.mark.parametrize('use_sink', [False, True])
def test_general_attention_portions_and_decode_rows(tm, cuda, dtype, name, use_sink):
    """three sequences with history: a portion that starts and ends inside blocks, a portion from position 0 that crosses a block border,
    a single decoded row just behind a border -- row kernel (1 and 4 key splits) and, in bf16 with aligned sizes, the tile kernel"""
    spec, rng = SPECS[name], np.random.default_rng(hash(name) % 1000 + dtype)
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    hist, new = [130, 0, 64], [70, 67, 1]
    lens = [a + b for a, b in zip(hist, new)]
    rnd = (lambda *s: lo.bf16(rng.normal(0, 1, s))) if dtype == 0 else (lambda *s: rng.normal(0, 1, s).astype(np.float32).astype(np.float64))
    keys, vals = [rnd(n, G, D) for n in lens], [rnd(n, G, V) for n in lens]
    sink = rng.normal(0, 1, H).astype(np.float32) if use_sink else None
    cache = Cache(dtype, G, D, V, lens, rng)
    # history goes in through the store path as well: one "prefill" launch per sequence prefix
    for s, n in enumerate(hist):
        if n:
            run_attention(tm, cache, rnd(n, H * D), keys[s][:n].reshape(n, -1), vals[s][:n].reshape(n, -1), [s] * n, list(range(n)),
                          [0] * s + [0, n] + [n] * (len(lens) - s - 1), [0] * s + [n] + [0] * (len(lens) - s - 1), spec, sink, 1)
    row_seq = sum(([s] * n for s, n in enumerate(new)), [])
    row_pos = sum((list(range(h, h + n)) for h, n in zip(hist, new)), [])
    cu_q = np.concatenate([[0], np.cumsum(new)])
    q = rnd(len(row_seq), H * D)
    k_new = np.concatenate([keys[s][h:h + n].reshape(n, -1) for s, (h, n) in enumerate(zip(hist, new))])
    v_new = np.concatenate([vals[s][h:h + n].reshape(n, -1) for s, (h, n) in enumerate(zip(hist, new))])
    ref = np.stack([oracle_attention(q[t], keys[s], vals[s], p, spec, sink) for t, (s, p) in enumerate(zip(row_seq, row_pos))])
    tol = (2e-2 if dtype == 0 else 2e-5) * np.abs(ref).max()
    kernels = [(1, 1), (1, 4)] + ([(2, 1)] if dtype == 0 and D % 8 == 0 and V % 8 == 0 else [])
    for kernel, splits in kernels:
        got = run_attention(tm, cache, q, k_new, v_new, row_seq, row_pos, cu_q, lens, spec, sink, kernel, splits)
        assert np.abs(got - ref).max() <= tol, (kernel, splits, np.abs(got - ref).max(), tol)


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('kernel', [1, 2])
def test_attention_finds_one_far_key_and_respects_the_causal_edge(tm, cuda, dtype, kernel):
    """one key among hundreds carries the whole soft-max (scaled so that its score stands out): at a block border, far back, and as the
    newest key; a key ONE position ahead of the query must stay invisible however large its score"""
    if kernel == 2 and dtype == 1:
        pytest.skip('the tile kernel is bf16')
    spec = dict(heads=2, kv_heads=1, dim=32, vdim=16, scale=1.0, softcap=0.0, qtemp_coef=0.0, qtemp_every=1.0)
    rng, n = np.random.default_rng(5), 400
    for hot in (0, 63, 64, 127, 128, 300, 398):
        keys, vals = lo.bf16(rng.normal(0, 0.05, (n, 1, 32))), lo.bf16(rng.normal(0, 1, (n, 1, 16)))
        q = lo.bf16(rng.normal(0, 0.05, (n, 64)))
        keys[hot, 0, :] = 0
        keys[hot, 0, 3] = 8.0
        q[:, 3], q[:, 32 + 3] = 8.0, 8.0                  # score 64 at the hot key, ~0 elsewhere
        cache = Cache(dtype, 1, 32, 16, [n], rng)
        got = run_attention(tm, cache, q, keys.reshape(n, -1), vals.reshape(n, -1), [0] * n, list(range(n)), [0, n], [n], spec, None, kernel)
        after = got[hot:].reshape(-1, 2, 16)
        assert np.abs(after - vals[hot, 0]).max() <= 2e-2, hot                                  # every row from `hot` on returns its value
        if hot > 0:                                                                             # the row just before must not see it
            ref = oracle_attention(q[hot - 1], keys, vals, hot - 1, spec, None)
            assert np.abs(got[hot - 1] - ref).max() <= 3e-2 and np.abs(got[hot - 1].reshape(2, 16) - vals[hot, 0]).max() > 0.2


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('heads,kv_heads,D,V', [(4, 4, 32, 16), (6, 2, 40, 24), (40, 2, 72, 40), (8, 1, 128, 128), (2, 1, 20, 12)])
def test_attention_decode_rows_of_unequal_sequences(tm, cuda, dtype, heads, kv_heads, D, V):
    """one new row per sequence, contexts from 1 token to several blocks (one ends exactly at a block border, one just behind it): the
    row kernel with and without key splits, and in bf16 the matrix-core decode kernel (query heads as rows: groups of 1, 3, 8 and 20)"""
    spec = dict(heads=heads, kv_heads=kv_heads, dim=D, vdim=V, scale=0.2, softcap=6.0, qtemp_coef=0.5, qtemp_every=60.0)
    rng = np.random.default_rng(heads * 7 + D + dtype)
    hist = [0, 63, 64, 200, 330, 5]
    lens = [n + 1 for n in hist]
    rnd = (lambda *s: lo.bf16(rng.normal(0, 1, s))) if dtype == 0 else (lambda *s: rng.normal(0, 1, s).astype(np.float32).astype(np.float64))
    keys, vals = [rnd(n, kv_heads, D) for n in lens], [rnd(n, kv_heads, V) for n in lens]
    sink = rng.normal(0, 1, heads).astype(np.float32)
    cache = Cache(dtype, kv_heads, D, V, lens, rng)
    for s, n in enumerate(hist):
        if n:
            run_attention(tm, cache, rnd(n, heads * D), keys[s][:n].reshape(n, -1), vals[s][:n].reshape(n, -1), [s] * n, list(range(n)),
                          [0] * s + [0, n] + [n] * (len(lens) - s - 1), [0] * s + [n] + [0] * (len(lens) - s - 1), spec, sink, 1)
    q = rnd(len(lens), heads * D)
    k_new = np.stack([keys[s][-1].reshape(-1) for s in range(len(lens))])
    v_new = np.stack([vals[s][-1].reshape(-1) for s in range(len(lens))])
    ref = np.stack([oracle_attention(q[s], keys[s], vals[s], hist[s], spec, sink) for s in range(len(lens))])
    tol = (2e-2 if dtype == 0 else 2e-5) * np.abs(ref).max()
    kernels = [(1, 1), (1, 3)] + ([(3, 1), (3, 2), (3, 8), (0, 1)] if dtype == 0 and D % 8 == 0 and V % 8 == 0 else [])
    for kernel, splits in kernels:
        got = run_attention(tm, cache, q, k_new, v_new, list(range(len(lens))), hist, list(range(len(lens) + 1)), lens, spec, sink, kernel, splits, prefill=0)
        assert np.abs(got - ref).max() <= tol, (kernel, splits, np.abs(got - ref).max(), tol)


# ---- engine -------------------------------------------------------------------------------------------------------------------------
def _layer(**kw):
    d = dict(heads=4, kv_heads=2, dim=40, vdim=24, scale=0.16, softcap=9.0, qtemp_coef=0.35, qtemp_every=7, sink=True, ff=136, weights_of=-1)
    d.update(kw)
    return d


def small_model(seed=0):
    """four layer runs over two weight sets; the third layer has other sizes, one query head per key head and no feed-forward"""
    cfg = lo.make_config(88, 203, [_layer(), _layer(weights_of=0), _layer(heads=3, kv_heads=3, dim=16, vdim=48, ff=0, softcap=4.0, qtemp_every=64),
                                   _layer(weights_of=0)], mult=0.4, logit_scale=1.7)
    return cfg, lo.make_weights(cfg, seed)


def engine_for(cfg, w, dtype, **kw):
    specs = [layered.LayerSpec(weights_of=L['weights_of'], heads=L['heads'], kv_heads=L['kv_heads'], dim=L['dim'], vdim=L['vdim'],
                               scale=L['scale'], softcap=L['softcap'], qtemp_coef=L['qtemp_coef'], qtemp_every=L['qtemp_every'], sink=L['sink'],
                               mlp=layered.MLP_DENSE if L['ff'] else layered.MLP_NONE, ff=L['ff']) for L in cfg['layers']]
    mc = layered.LayeredConfig('test', cfg['width'], cfg['vocab'], specs, cfg['eps'], cfg['offset'], cfg['mult'], cfg['logit_scale'])
    args = dict(max_batch_size=4, session_len=512, cache_blocks=12, max_prefill_token_num=512, use_graph=0)
    args.update(kw)
    eng = layered.LayeredEngine(mc, dtype=dtype, **args)
    eng.load_weights({k: lo.to_bf16_bits(v) for k, v in w.items()})
    eng.start()
    return eng


TOL = {'float32': 3e-5, 'bfloat16': 4e-2}


def rel_err(got, ref):
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)).max() / ref.std()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_layers_and_whole_prompt(cuda, dtype):
    cfg, w = small_model()
    eng = engine_for(cfg, w, dtype)
    toks = np.random.default_rng(1).integers(0, cfg['vocab'], 150).tolist()
    for n in range(1, len(cfg['layers']) + 1):                    # the residual stream behind every layer run
        eng.stop_after(n)
        s = eng.open_session()
        eng.step_tokens([(s, toks[:70], [])])
        got = eng.fetch_residual(70)
        eng.close_session(s)
        ref = lo.forward(cfg, w, toks[:70], n)[1]
        assert np.abs(got - ref).max() <= TOL[dtype] * 3 * np.abs(ref).max(), n
    eng.stop_after(-1)
    ref = lo.forward(cfg, w, toks)[0]
    s = eng.open_session()
    got = eng.step_tokens([(s, toks, list(range(len(toks))))])
    eng.close_session(s)
    assert rel_err(got, ref) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_portions_decoding_batches_and_reuse(cuda, dtype):
    """every way of cutting the same requests gives the oracle's logits: token by token from the first token on, portions down to two
    tokens that start and end inside blocks, unequal requests in one forward, and sessions that come and go in a pool that holds
    only what is live (blocks and slots are used again, with other requests' keys still in them)"""
    cfg, w = small_model(1)
    rng = np.random.default_rng(2)
    reqs = [rng.integers(0, cfg['vocab'], n).tolist() for n in (200, 131, 65, 1, 23)]
    refs = [lo.forward(cfg, w, t)[0] for t in reqs]
    eng = engine_for(cfg, w, dtype, cache_blocks=9)               # 8 blocks for sessions: 512 tokens live at most
    tol = TOL[dtype]
    # token by token, the first tokens of a sequence included, across two block borders
    s = eng.open_session()
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in reqs[1]])
    eng.close_session(s)
    assert rel_err(got, refs[1]) <= tol
    # portions of changing size, the last tokens one by one
    s, at, rows = eng.open_session(), 0, []
    for n in [2, 61, 2, 64, 3, 30, 2] + [1] * 36:
        rows.append(eng.step_tokens([(s, reqs[0][at:at + n], list(range(n)))]))
        at += n
    eng.close_session(s)
    assert at == 200 and rel_err(np.concatenate(rows), refs[0]) <= tol
    # unequal requests together: portions beside single tokens, requests that join late, pause, and end while others go on
    plan = [[(0, 60)], [(0, 4), (1, 64), (3, 1)], [(0, 1), (1, 2), (2, 33)], [(1, 1), (2, 2), (4, 23)], [(0, 64), (2, 30)],
            [(0, 1), (1, 64)], [(0, 70)]]
    sess, at, got = {}, [0] * 5, [[] for _ in reqs]
    for step in plan:
        entries = []
        for r, n in step:
            if r not in sess:
                sess[r] = eng.open_session()
            entries.append((sess[r], reqs[r][at[r]:at[r] + n], list(range(n))))
        out, k = eng.step_tokens(entries), 0
        for r, n in step:
            got[r].append(out[k:k + n])
            k += n
            at[r] += n
            if at[r] == len(reqs[r]):
                eng.close_session(sess.pop(r))
    assert at == [200, 131, 65, 1, 23] and not sess
    for r in range(5):
        assert rel_err(np.concatenate(got[r]), refs[r]) <= tol, r
    # the pool is bounded: a step that cannot fit is refused and changes nothing
    a, b = eng.open_session(), eng.open_session()
    eng.step_tokens([(a, reqs[0][:200], []), (b, reqs[1][:131], [])])          # 4 + 3 blocks of 8
    with pytest.raises(_ffi.TmError) as ei:
        eng.step_tokens([(b, reqs[1][:131], [])])
    assert ei.value.status == 11
    eng.close_session(a)
    out = eng.step_tokens([(b, [5], [0])])                                     # b is intact and goes on
    assert rel_err(out, lo.forward(cfg, w, reqs[1] + [5])[0][-1:]) <= tol
    eng.close_session(b)
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_long_decoding_with_key_splits(cuda, dtype):
    """a long session decoded one token at a time with the decode rows' keys split over several workgroups (session_len 1024 -> 4 splits)"""
    cfg = lo.make_config(64, 97, [_layer(heads=2, kv_heads=1, dim=24, vdim=8, ff=72, qtemp_every=50), _layer(heads=2, kv_heads=1, dim=24, vdim=8, ff=72,
                                                                                                       qtemp_every=50, weights_of=0)])
    w = lo.make_weights(cfg, 4)
    toks = np.random.default_rng(3).integers(0, 97, 420).tolist()
    ref = lo.forward(cfg, w, toks)[0]
    eng = engine_for(cfg, w, dtype, session_len=1024, cache_blocks=17, max_prefill_token_num=256)
    s = eng.open_session()
    eng.step_tokens([(s, toks[:100], [])])
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in toks[100:]])
    eng.close_session(s)
    assert rel_err(got, ref[100:]) <= TOL[dtype]
    eng.close()


def _check_greedy(cfg, w, prompt, toks, min_margin=2e-2):     # (the sampler reads fp16 logits rows)
    """the engine's greedy tokens equal the oracle's as long as the oracle's own top-2 gap is not a rounding matter"""
    ref, margins = lo.greedy(cfg, w, prompt, len(toks))
    for i, (a, b, m) in enumerate(zip(toks, ref, margins)):
        if m < min_margin:
            return          # a near-tie: from here on the two may legitimately part
        assert int(a) == b, (i, toks, ref)


def test_greedy_generation_static_batch_and_scheduler(cuda):
    cfg, w = small_model(2)
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, cfg['vocab'], n).tolist() for n in (70, 3, 129, 40, 64, 9)]
    eng = engine_for(cfg, w, 'float32', max_batch_size=3, session_len=256, cache_blocks=13, max_prefill_token_num=128, use_graph=1)
    eng.prefill(prompts[:3], max_new_tokens=12)                   # static batch: chunked prefill (129 > ... 128 per forward) + graph decode
    eng.decode(11)
    toks = eng.fetch()
    eng.release()
    for p, t in zip(prompts[:3], toks):
        _check_greedy(cfg, w, p, t.tolist())
    ids = [eng.submit(p, 10) for p in prompts]                    # continuous batching: six requests through three slots
    for _ in range(200):
        na, nw = eng.step()
        if na == 0 and nw == 0:
            break
    for p, rid in zip(prompts, ids):
        status, out = eng.poll(rid)
        assert status == 7 and len(out) == 10
        _check_greedy(cfg, w, p, out.tolist())
    eng.release()
    s = eng.open_session()                                        # sessions work again once the requests are gone
    assert eng.step_tokens([(s, prompts[1], [2])]).shape == (1, cfg['vocab'])
    with pytest.raises(_ffi.TmError):
        eng.submit(prompts[0], 4)                                 # ... and the two do not mix
    eng.close_session(s)
    eng.close()


def test_pipeline_serves_a_checkpoint_folder(cuda, tmp_path):
    from lmdeploy_amd import GenerationConfig, TurbomindEngineConfig, pipeline
    cfg, w = small_model(3)
    lo.write_checkpoint(str(tmp_path), cfg, w)
    prompts = [np.random.default_rng(7).integers(0, cfg['vocab'], n).tolist() for n in (33, 5)]
    with pipeline(str(tmp_path), backend_config=TurbomindEngineConfig(dtype='float32', session_len=128, max_batch_size=2)) as pipe:
        outs = pipe(prompts, gen_config=GenerationConfig(max_new_tokens=8, ignore_eos=True))
        for p, r in zip(prompts, outs):
            assert len(r.token_ids) == 8
            _check_greedy(cfg, w, p, r.token_ids)
        sampled = pipe(prompts, gen_config=GenerationConfig(max_new_tokens=6, ignore_eos=True, do_sample=True, top_k=5, temperature=0.8,
                                                            random_seed=11))
        assert all(len(r.token_ids) == 6 and all(0 <= t < cfg['vocab'] for t in r.token_ids) for r in sampled)


def test_trace_run_replays_a_schedule_on_awkward_sizes(cuda, tmp_path):
    """bin/trace_run end to end, both number formats: a checkpoint folder with a width off the 8 grid, key / value sizes off it too, a group of
    17 query heads per key head, a non-integer temperature period, a layer without cap and temperature keys, weight sharing through a chain;
    five requests in shared steps, pool of 640 tokens"""
    def L(**kw):
        d = dict(heads=5, kv_heads=1, dim=24, vdim=40, scale=0.21, softcap=11.0, qtemp_coef=0.45, qtemp_every=33, sink=True, ff=72, weights_of=-1)
        d.update(kw)
        return d
    B = dict(heads=6, kv_heads=3, dim=20, vdim=12, ff=0, softcap=0.0, qtemp_coef=0.0)
    Cc = dict(heads=34, kv_heads=2, dim=8, vdim=8, ff=200, qtemp_every=2.5)
    cfg = lo.make_config(100, 333, [L(), L(**B), L(weights_of=0), L(weights_of=1, **B), L(**Cc), L(weights_of=4, **Cc), L(weights_of=0)], mult=0.2,
                         logit_scale=3.0)
    w = lo.make_weights(cfg, 11)
    folder = str(tmp_path / 'model')
    lo.write_checkpoint(folder, cfg, w)
    c = json.load(open(folder + '/config.json'))
    c['layers'][6]['weights_of'] = 2                      # a chain: 6 -> 2 -> 0
    del c['layers'][1]['mixer']['q_temp'], c['layers'][1]['mixer']['softcap']
    json.dump(c, open(folder + '/config.json', 'w'))
    rng = np.random.default_rng(0)
    reqs = {n: rng.integers(0, 333, k).tolist() for n, k in (('a', 300), ('b', 70), ('c', 1), ('d', 129), ('e', 40))}
    ref = {n: lo.forward(cfg, w, t)[0] for n, t in reqs.items()}
    plan = [[('a', 100)], [('a', 3), ('b', 64), ('c', 1)], [('a', 1), ('b', 2), ('d', 65)], [('a', 64), ('b', 1), ('d', 1), ('e', 2)],
            [('a', 2), ('b', 3), ('d', 63), ('e', 38)], [('a', 130)]]
    at, steps, rows = {n: 0 for n in reqs}, [], []
    for i, st_ in enumerate(plan):
        ent, end, rr = [], [], []
        for n, k in st_:
            ent.append({'id': n, 'tokens': reqs[n][at[n]:at[n] + k], 'want': list(range(0, k, 2))})
            rr += [(n, at[n] + j) for j in range(0, k, 2)]
            at[n] += k
            if at[n] == len(reqs[n]):
                end.append(n)
        steps.append(json.dumps({'step': i, 'entries': ent, 'end': end}))
        rows.append(rr)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype, tol in (('float32', 5e-5), ('bfloat16', 5e-2)):
        out = str(tmp_path / dtype)
        p = subprocess.run([sys.executable, os.path.join(root, 'bin', 'trace_run'), '--model', folder, '--dtype', dtype, '--out', out,
                            '--max-tokens', '640'], input='\n'.join(steps) + '\n', text=True, capture_output=True, timeout=100)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.split('\n') if l.startswith('done')] == ['done %d' % i for i in range(len(plan))]
        for i, rr in enumerate(rows):
            got = np.fromfile(os.path.join(out, '%d.f32' % i), '<f4').reshape(len(rr), -1)
            assert rel_err(got, np.stack([ref[n][j] for n, j in rr])) <= tol, (dtype, i)
