"""GPU tests of the Bedenex design on the layer-list engine against the plain float64 model in tests/bedenex_oracle.py: the attention
kernels' chunked visibility, distance penalty and output gate alone (every kernel, keys just inside and just outside a chunk, one key
that dominates); every block form alone in a one-layer model; then the engine -- the residual stream behind every layer run, whole
prompts, token-by-token decoding from the first token, portions down to two tokens, unequal batches, reused blocks and slots, long
decoding over many chunk edges, greedy generation through the static batch, the scheduler and the pipeline, and bin/trace_run.
Configurations and weights are the tests' own."""
import ctypes as C
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from lmdeploy_amd import _ffi
from lmdeploy_amd.turbomind import layered
from tests import bedenex_oracle as bo
from tests.gpu_helpers import dev, host, release_all, st

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _release():
    yield
    release_all()


def act(x, dtype):
    return dev(bo.bf16_bits(x).view(np.int16)) if dtype == 0 else dev(np.asarray(x, np.float32))


def read(t, dtype):
    if dtype == 0:
        return (host(t).view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return host(t).astype(np.float64)


# ---- the attention kernels with chunks, distance penalty and output gate ------------------------------------------------------------
class Paged:
    """keys [G][64][D] and transposed values [G][V][64] per block, blocks shuffled, junk where nothing was stored"""

    def __init__(self, dtype, G, D, V, lens, rng):
        per = [(n + 63) // 64 for n in lens]
        self.stride, nb = max(per) + 1, sum(per) + 2
        self.elems, self.eb = G * 64 * (D + V), 2 if dtype == 0 else 4
        self.pool = act(rng.normal(0, 30, (nb, self.elems)), dtype)
        order, ptrs, k = rng.permutation(nb), np.zeros((len(lens), self.stride), np.uint64), 0
        for s, n in enumerate(per):
            for i in range(n):
                ptrs[s, i] = self.pool.data_ptr() + int(order[k]) * self.elems * self.eb
                k += 1
        self.ptrs, self.v_offset = dev(ptrs.view(np.int64)), G * 64 * D * self.eb


def attend(tm, dtype, spec, cache, q, k_new, v_new, gate, row_seq, row_pos, cu_q, k_len, kernel, splits=1, prefill=1, head_stride=0):
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    rows = q.shape[0]
    ld = (H * D + G * D + G * V + 31) // 32 * 32
    qkv = np.zeros((rows, ld))
    qkv[:, :H * D], qkv[:, H * D:H * D + G * D], qkv[:, H * D + G * D:H * D + G * D + G * V] = q, k_new, v_new
    qkv_d = act(qkv, dtype)
    hs = head_stride or V
    out = act(np.zeros((rows, H * hs + 3)), dtype)
    ws = torch.zeros(max(1, tm.tm_general_attention_workspace(rows, H, V, splits) // 4), dtype=torch.float32, device='cuda')
    a = _ffi.GeneralAttn(qkv_d.data_ptr(), out.data_ptr(), ld, H * hs + 3, rows, dev(np.asarray(row_seq, np.int32)).data_ptr(),
                         dev(np.asarray(row_pos, np.int32)).data_ptr(), cache.ptrs.data_ptr(), cache.stride, 0, cache.v_offset, cache.eb,
                         H, G, D, V, spec['scale'], 0.0, 0.0, 1.0, None, splits, ws.data_ptr(), qkv_d.data_ptr(), ld, H * D, H * D + G * D, 1,
                         kernel, prefill, len(cu_q) - 1, int(np.diff(cu_q).max()), dev(np.asarray(cu_q, np.int32)).data_ptr(),
                         dev(np.asarray(k_len, np.int32)).data_ptr(),
                         dev(np.asarray(spec['r1'], np.float32)).data_ptr() if spec.get('r1') is not None else None,
                         dev(np.asarray(spec['r2'], np.float32)).data_ptr() if spec.get('r1') is not None else None, spec.get('chunk', 0),
                         dev(np.asarray(gate, np.float32)).data_ptr() if gate is not None else None, H + 2, head_stride)
    _ffi.check(tm.tm_general_attention(C.byref(a), st()))
    got = read(out, dtype)[:, :H * hs].reshape(rows, H, hs)[:, :, :V]
    return got.reshape(rows, H * V)


def attend_oracle(spec, q, keys, vals, gate, pos):
    """one row at position pos; keys / vals [pos + 1, G, .] -> [H * V]"""
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    j = np.arange(pos + 1)
    vis = j // spec['chunk'] == pos // spec['chunk'] if spec.get('chunk') else np.ones(pos + 1, bool)
    out = np.zeros((H, V))
    for h in range(H):
        g = h // (H // G)
        s = (keys[:, g] @ q[h * D:(h + 1) * D]) * spec['scale']
        if spec.get('r1') is not None:
            s = s - spec['r1'][h] * np.log(1.0 + spec['r2'][h] * (pos - j))
        s = np.where(vis, s, -np.inf)
        e = np.exp(s - s.max())
        out[h] = (e / e.sum()) @ vals[:, g]
        if gate is not None:
            out[h] *= bo.sigmoid(gate[h])
    return out.reshape(-1)


def _rounded(x, dtype):
    return bo.bf16_round(x) if dtype == 0 else np.asarray(x, np.float32).astype(np.float64)


ATT = {
    'edge_off_block': dict(heads=4, kv_heads=2, dim=32, vdim=16, scale=0.3, chunk=50, r1=[1.0, 0.2, 2.0, 0.0], r2=[0.3, 0.05, 0.5, 0.7]),
    'block_sized': dict(heads=6, kv_heads=2, dim=40, vdim=24, scale=0.2, chunk=64, r1=[0.5] * 6, r2=[0.25] * 6),
    'tiny_chunks': dict(heads=3, kv_heads=3, dim=72, vdim=136, scale=0.1, chunk=7, r1=None),
    'one_chunk': dict(heads=2, kv_heads=1, dim=20, vdim=12, scale=0.2, chunk=1000, r1=[1.5, 0.7], r2=[0.4, 0.1]),
    'no_chunk': dict(heads=16, kv_heads=1, dim=48, vdim=32, scale=0.15, chunk=0, r1=[0.1 * i for i in range(16)], r2=[0.2] * 16),
    'latent_sized': dict(heads=5, kv_heads=1, dim=256, vdim=192, scale=0.06, chunk=0, r1=None),     # one shared key head, the largest tile kernel
}


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('name', list(ATT))
def test_attention_chunks_distance_gate_in_every_kernel(tm, cuda, dtype, name):
    """portions that start and end inside chunks and blocks, then one decoded row per sequence, each kernel that serves the format"""
    spec, rng = ATT[name], np.random.default_rng(5)
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    lens, first = [203, 77, 1, 130], [0, 30, 0, 51]          # the sequences' lengths and where the portion under test starts
    cache = Paged(dtype, G, D, V, [n + 1 for n in lens], rng)
    K = [_rounded(rng.normal(0, 1, (n + 1, G, D)), dtype) for n in lens]
    Vv = [_rounded(rng.normal(0, 1, (n + 1, G, V)), dtype) for n in lens]
    tol = 3e-2 if dtype == 0 else 2e-5
    mfma = dtype == 0 and D % 8 == 0 and V % 8 == 0

    def run(lo_, hi_, kernels, prefill, splits=1, stride=0):
        rs, rp, cu, kl = [], [], [0], []
        for s in range(len(lens)):
            rs += [s] * (hi_[s] - lo_[s])
            rp += list(range(lo_[s], hi_[s]))
            cu.append(len(rs))
            kl.append(hi_[s])
        q = _rounded(rng.normal(0, 1, (len(rs), H * D)), dtype)
        gate = rng.normal(0, 1.5, (len(rs), H + 2)).astype(np.float32)
        kn = np.stack([K[s][p].reshape(-1) for s, p in zip(rs, rp)])
        vn = np.stack([Vv[s][p].reshape(-1) for s, p in zip(rs, rp)])
        ref = np.stack([attend_oracle(spec, q[i], K[s][:p + 1], Vv[s][:p + 1], gate[i].astype(np.float64), p) for i, (s, p) in enumerate(zip(rs, rp))])
        for kern in kernels:
            got = attend(tm, dtype, spec, cache, q, kn, vn, gate, rs, rp, cu, kl, kern, splits, prefill, stride)
            assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max()), (name, kern, splits)

    if first != [0, 0, 0, 0]:   # what precedes the portions
        run([0] * 4, first, [1], 1)
    run(first, lens, [1, 2] if mfma else [1], 1)
    run(first, lens, [0], 1, stride=V + 8)                                      # heads of the output spaced apart
    dec = [n + 1 for n in lens]
    run(lens, dec, [1, 3] if mfma else [1], 0)                                  # one more token each: decode rows
    run(lens, dec, [1, 3] if mfma else [1], 0, splits=3)                        # (re-stores the same keys) with split keys


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('kernel', [1, 2, 3])
def test_attention_sees_the_first_key_of_its_chunk_and_not_the_one_before(tm, cuda, dtype, kernel):
    """one key far louder than all others, planted at the first position of the query's chunk (seen: the output is its value) or one before
    it (unseen: the output must not move towards it); chunk edges inside a block, on a block border and far back"""
    if kernel != 1 and dtype == 1:
        pytest.skip('the matrix-core kernels are bf16')
    spec = dict(heads=2, kv_heads=1, dim=32, vdim=16, scale=1.0, chunk=96, r1=[0.3, 0.0], r2=[0.2, 0.5])
    rng = np.random.default_rng(9)
    n = 400
    for pos in (95, 96, 191, 192, 287, 399):                 # last / first position of a chunk, prompt rows and the decode kernel alike
        start = pos // 96 * 96
        for hot, seen in ((start, True), (start - 1, False)):
            if hot < 0:
                continue
            K = _rounded(rng.normal(0, 0.05, (n, 1, 32)), dtype)
            Vv = _rounded(rng.normal(0, 1, (n, 1, 16)), dtype)
            q = _rounded(np.tile(rng.normal(0, 1, 32), 2)[None, :], dtype)
            K[hot, 0] = _rounded(q[0, :32] * 1.5, dtype)       # score ~ 1.5 |q|^2 ~ 48 against ~0 elsewhere
            cache = Paged(dtype, 1, 32, 16, [n], rng)
            # the history first (row kernel), then the row under test
            attend(tm, dtype, spec, cache, _rounded(rng.normal(0, 1, (pos, 64)), dtype), K[:pos].reshape(pos, -1), Vv[:pos].reshape(pos, -1),
                   None, [0] * pos, list(range(pos)), [0, pos], [pos], 1)
            got = attend(tm, dtype, spec, cache, q, K[pos:pos + 1].reshape(1, -1), Vv[pos:pos + 1].reshape(1, -1), None, [0], [pos], [0, 1],
                         [pos + 1], kernel, 1, 1 if kernel == 2 else 0)
            ref = attend_oracle(spec, q[0], K[:pos + 1], Vv[:pos + 1], None, pos)
            assert np.abs(got[0] - ref).max() <= (4e-2 if dtype == 0 else 1e-4), (pos, hot)
            near = np.abs(got[0, :16] - Vv[hot, 0]).max()
            assert (near < 0.1) == seen, (pos, hot, near)


# ---- engine -------------------------------------------------------------------------------------------------------------------------
def model_folder(tmp_path, cfg, seed, name='m'):
    w = bo.make_weights(cfg, seed)
    folder = str(tmp_path / name)
    bo.write_checkpoint(folder, cfg, w)
    return folder, w


def engine(folder, dtype, **kw):
    args = dict(max_batch_size=4, session_len=512, cache_blocks=12, max_prefill_token_num=512, use_graph=0)
    args.update(kw)
    return layered.build_engine(folder, dtype=dtype, **args)


def chosen(dtype, k, experts):
    """experts per token of the many-layer models: k in float32.  In bfloat16 all of them: hundreds of routing decisions always hold one
    that rounding may turn, and the token it turns for is then simply another function -- top-k routing in bfloat16 is tested on the
    one-layer models, whose routers' closest calls are checked to be clear"""
    return k if dtype == 'float32' else experts


def looped_model(dtype='float32'):
    """eight layer runs over four weight sets: grouped and ungrouped attention with chunks that cut blocks, key sizes on and off the
    matrix-core grid, latent attention with rotated parts smaller and larger than the unrotated ones, a dense and an expert feed-forward
    (two experts per token) and a block without feed-forward; the middle two layers run three times"""
    return bo.make_config(72, 211, [bo.attention_layer(4, 2, 24, 40, 0.3, 50, bo.dense(88)),
                                    bo.latent_layer(3, 16, 8, 24, 40, 0.2, mlp=bo.moe(5, chosen(dtype, 2, 5), 48)),
                                    bo.attention_layer(3, 3, 20, 12, 0.4, 7),
                                    bo.latent_layer(5, 8, 16, 8, 72, 0.25, 500.0, bo.dense(40))], loop=(1, 3, 3))


TOL = {'float32': 3e-5, 'bfloat16': 8e-2}      # (eight layer runs deep: bf16 rounding alone reaches 6e-2 on single rows)


def rel_err(got, ref):
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)).max() / ref.std()


ALONE = {
    'attention': lambda: bo.make_config(64, 97, [bo.attention_layer(4, 1, 16, 32, 0.5, 33)]),
    'attention_plain_causal': lambda: bo.make_config(48, 97, [bo.attention_layer(2, 2, 40, 8, 0.2, 0)]),
    'latent': lambda: bo.make_config(64, 97, [bo.latent_layer(4, 24, 8, 16, 48, 0.3)]),
    'latent_part_turns': lambda: bo.make_config(64, 97, [bo.latent_layer(3, 8, 24, 16, 42, 0.3, 300.0, dims=10)]),      # latent size off the 8 grid
    'latent_wide': lambda: bo.make_config(40, 97, [bo.latent_layer(2, 12, 36, 20, 280, 0.1, 77.0)]),       # key size 316: beyond the tile kernels
    'gated_gelu': lambda: bo.make_config(64, 97, [bo.attention_layer(2, 1, 8, 8, 0.3, 16, bo.dense(100))]),
    'experts_top1': lambda: bo.make_config(64, 97, [bo.attention_layer(2, 1, 8, 8, 0.3, 16, bo.moe(3, 1, 24))]),
    'experts_top2': lambda: bo.make_config(64, 97, [bo.latent_layer(2, 8, 8, 8, 16, 0.3, mlp=bo.moe(6, 2, 24))]),
    'experts_all': lambda: bo.make_config(64, 97, [bo.attention_layer(2, 1, 8, 8, 0.3, 16, bo.moe(4, 4, 40))]),
    'loop_once': lambda: bo.make_config(64, 97, [bo.attention_layer(2, 1, 8, 8, 0.3, 16)], loop=(0, 1, 1)),
}


ALONE_SEED = {'experts_top1': 5, 'experts_top2': 24}     # weights whose routers make no close call on the test's tokens


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('name', list(ALONE))
def test_each_block_form_alone(cuda, tmp_path, dtype, name):
    cfg = ALONE[name]()
    folder, w = model_folder(tmp_path, cfg, ALONE_SEED.get(name, 3))
    toks = np.random.default_rng(1).integers(0, 97, 150).tolist()
    assert dtype == 'float32' or bo.router_gap(cfg, w, [toks]) >= 0.1      # no routing decision that bf16 rounding could turn
    ref_logits, trail = bo.forward(cfg, w, toks, True)
    eng = engine(folder, dtype)
    eng.stop_after(1)
    s = eng.open_session()
    eng.step_tokens([(s, toks, [])])
    got = eng.fetch_residual(len(toks))
    eng.close_session(s)
    assert np.abs(got - trail[0]).max() <= TOL[dtype] * 3 * np.abs(trail[0]).max()
    eng.stop_after(-1)
    s = eng.open_session()                                        # the same through the cache: a portion, then token by token
    rows = [eng.step_tokens([(s, toks[:70], list(range(70)))])] + [eng.step_tokens([(s, [t], [0])]) for t in toks[70:]]
    eng.close_session(s)
    assert rel_err(np.concatenate(rows), ref_logits) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_layer_runs_and_whole_prompt(cuda, tmp_path, dtype):
    cfg = looped_model(dtype)
    folder, w = model_folder(tmp_path, cfg, 0)
    eng = engine(folder, dtype)
    toks = np.random.default_rng(1).integers(0, cfg['vocab'], 150).tolist()
    ref, trail = bo.forward(cfg, w, toks[:70], True)
    assert len(trail) == 8
    for n in range(1, 9):                                         # the residual stream behind every layer run
        eng.stop_after(n)
        s = eng.open_session()
        eng.step_tokens([(s, toks[:70], [])])
        got = eng.fetch_residual(70)
        eng.close_session(s)
        assert np.abs(got - trail[n - 1]).max() <= TOL[dtype] * 3 * np.abs(trail[n - 1]).max(), n
    eng.stop_after(-1)
    ref = bo.forward(cfg, w, toks)
    s = eng.open_session()
    got = eng.step_tokens([(s, toks, list(range(len(toks))))])
    eng.close_session(s)
    assert rel_err(got, ref) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_portions_decoding_batches_and_reuse(cuda, tmp_path, dtype):
    """every way of cutting the same requests gives the oracle's logits: token by token from the first token on, portions down to two
    tokens that start and end inside blocks and chunks, unequal requests in one forward, and sessions that come and go in a pool that
    holds only what is live (blocks and slots are used again, with other requests' keys still in them)"""
    cfg = looped_model(dtype)
    folder, w = model_folder(tmp_path, cfg, 1)
    rng = np.random.default_rng(2)
    reqs = [rng.integers(0, cfg['vocab'], n).tolist() for n in (200, 131, 65, 1, 23)]
    refs = [bo.forward(cfg, w, t) for t in reqs]
    eng = engine(folder, dtype, cache_blocks=9)                   # 8 blocks for sessions: 512 tokens live at most
    tol = TOL[dtype]
    s = eng.open_session()
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in reqs[1]])
    eng.close_session(s)
    assert rel_err(got, refs[1]) <= tol
    s, at, rows = eng.open_session(), 0, []
    for n in [2, 61, 2, 64, 3, 30, 2] + [1] * 36:
        rows.append(eng.step_tokens([(s, reqs[0][at:at + n], list(range(n)))]))
        at += n
    eng.close_session(s)
    assert at == 200 and rel_err(np.concatenate(rows), refs[0]) <= tol
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
    a, b = eng.open_session(), eng.open_session()                 # the pool is bounded: a step that cannot fit is refused and changes nothing
    eng.step_tokens([(a, reqs[0][:200], []), (b, reqs[1][:131], [])])
    with pytest.raises(_ffi.TmError):
        eng.step_tokens([(b, reqs[1][:131], [])])
    eng.close_session(a)
    out = eng.step_tokens([(b, [5], [0])])
    assert rel_err(out, bo.forward(cfg, w, reqs[1] + [5])[-1:]) <= tol
    eng.close_session(b)
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_long_decoding_over_chunk_edges_with_key_splits(cuda, tmp_path, dtype):
    """420 tokens, the last 320 one at a time, with the decode rows' keys split over several workgroups (session_len 1024 -> 4 splits);
    chunks of 100 positions (edges inside blocks) beside a latent layer that looks all the way back"""
    cfg = bo.make_config(64, 97, [bo.attention_layer(4, 2, 16, 8, 0.4, 100, bo.moe(6, chosen(dtype, 2, 6), 32)), bo.latent_layer(2, 8, 8, 16, 32, 0.3, mlp=bo.dense(72))],
                         loop=(0, 2, 2))
    folder, w = model_folder(tmp_path, cfg, 4)
    toks = np.random.default_rng(3).integers(0, 97, 420).tolist()
    ref = bo.forward(cfg, w, toks)
    eng = engine(folder, dtype, session_len=1024, cache_blocks=17, max_prefill_token_num=256)
    s = eng.open_session()
    eng.step_tokens([(s, toks[:100], [])])
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in toks[100:]])
    eng.close_session(s)
    assert rel_err(got, ref[100:]) <= TOL[dtype]
    eng.close()


def _check_greedy(cfg, w, prompt, toks, min_margin=2e-2):     # (the sampler reads fp16 logits rows)
    ref, margins = bo.greedy(cfg, w, prompt, len(toks))
    for i, (a, b, m) in enumerate(zip(toks, ref, margins)):
        if m < min_margin:
            return          # a near-tie: from here on the two may legitimately part
        assert int(a) == b, (i, toks, ref)


def test_greedy_generation_static_batch_and_scheduler(cuda, tmp_path):
    cfg = looped_model()
    folder, w = model_folder(tmp_path, cfg, 2)
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, cfg['vocab'], n).tolist() for n in (70, 3, 129, 40, 64, 9)]
    eng = engine(folder, 'float32', max_batch_size=3, session_len=256, cache_blocks=13, max_prefill_token_num=128, use_graph=1)
    eng.prefill(prompts[:3], max_new_tokens=12)                   # static batch: chunked prefill + the captured decode step
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
    eng.close()


def test_pipeline_serves_a_checkpoint_folder(cuda, tmp_path):
    from lmdeploy_amd import GenerationConfig, TurbomindEngineConfig, pipeline
    cfg = looped_model('bfloat16')
    folder, w = model_folder(tmp_path, cfg, 3)
    prompts = [np.random.default_rng(7).integers(0, cfg['vocab'], n).tolist() for n in (33, 5)]
    with pipeline(folder, backend_config=TurbomindEngineConfig(dtype='bfloat16', session_len=128, max_batch_size=2)) as pipe:
        outs = pipe(prompts, gen_config=GenerationConfig(max_new_tokens=8, ignore_eos=True))
        for p, r in zip(prompts, outs):
            assert len(r.token_ids) == 8
            _check_greedy(cfg, w, p, r.token_ids, min_margin=0.15)
        sampled = pipe(prompts, gen_config=GenerationConfig(max_new_tokens=6, ignore_eos=True, do_sample=True, top_k=5, temperature=0.8,
                                                            random_seed=11))
        assert all(len(r.token_ids) == 6 and all(0 <= t < cfg['vocab'] for t in r.token_ids) for r in sampled)


def test_trace_run_replays_a_schedule(cuda, tmp_path):
    """bin/trace_run end to end, both number formats: a width off the 8 grid, a loop from the first layer to the last that runs once, one
    expert per token, a chunk as long as a cache block, a layer without chunks; five requests in shared steps, pool of 640 tokens"""
    rng = np.random.default_rng(0)
    reqs = {n: rng.integers(0, 333, k).tolist() for n, k in (('a', 300), ('b', 70), ('c', 1), ('d', 129), ('e', 40))}
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
        cfg = bo.make_config(100, 333, [bo.latent_layer(6, 20, 4, 12, 24, 0.2, 3000.0, bo.moe(7, chosen(dtype, 1, 7), 40)),
                                        bo.attention_layer(10, 2, 8, 24, 0.35, 64, bo.dense(72)),
                                        bo.attention_layer(5, 5, 24, 8, 0.3, 0)], loop=(0, 3, 1))
        folder, w = model_folder(tmp_path, cfg, 11, 'model_' + dtype)
        ref = {n: bo.forward(cfg, w, t) for n, t in reqs.items()}
        out = str(tmp_path / dtype)
        p = subprocess.run([sys.executable, os.path.join(root, 'bin', 'trace_run'), '--model', folder, '--dtype', dtype, '--out', out,
                            '--max-tokens', '640'], input='\n'.join(steps) + '\n', text=True, capture_output=True, timeout=100)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.split('\n') if l.startswith('done')] == ['done %d' % i for i in range(len(plan))]
        for i, rr in enumerate(rows):
            got = np.fromfile(os.path.join(out, '%d.f32' % i), '<f4').reshape(len(rr), -1)
            assert rel_err(got, np.stack([ref[n][j] for n, j in rr])) <= tol, (dtype, i)
