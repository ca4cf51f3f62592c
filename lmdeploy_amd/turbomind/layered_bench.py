"""`bench.py --layered`: prefill and decode throughput of a layer-list model (Fokonex blocks, bf16) at layer shapes of real decoders,
beside the closest model the engine already serves -- a Llama-family decoder with fp16 weights and fp16 KV -- at EQUAL size: same width,
heads, head size 128, layer count and vocabulary, and a feed-forward of the same parameter count (two matrices of 1.5 x the gated
feed-forward's three).  Random weights; both engines run their own static-batch entry points (chunked prefill, hipGraph decode).

Per kernel category of an eager decode step the table also gives the fraction of the HBM roofline (bytes the category must move /
8 TB/s / measured time) for both, and their ratio: the figure the two designs' like kernels are compared by.
"""
from __future__ import annotations

import time
from types import SimpleNamespace

import numpy as np

HBM_BYTES_PER_S = 8.0e12
MFMA_BF16_FLOPS = 2.5e15

SIZES = {
    'w2048': dict(width=2048, heads=16, kv_heads=8, inter=5632, layers=8, vocab=32000),
    'w4096': dict(width=4096, heads=32, kv_heads=8, inter=14336, layers=8, vocab=32000),
}


def _fokonex_engine(s, batch, session_len, max_prefill):
    from . import layered
    spec = layered.LayerSpec(heads=s['heads'], kv_heads=s['kv_heads'], dim=128, vdim=128, scale=128 ** -0.5, softcap=30.0, qtemp_coef=0.1,
                             qtemp_every=512.0, sink=True, mlp=layered.MLP_DENSE, ff=s['inter'] * 3 // 2)
    cfg = layered.LayeredConfig('Fokonex', s['width'], s['vocab'], [spec] * s['layers'], 1e-5, 1.0, 0.5, 1.0)
    eng = layered.LayeredEngine(cfg, dtype='bfloat16', max_batch_size=batch, session_len=session_len, max_prefill_token_num=max_prefill)
    eng.init_synthetic(seed=1)
    eng.start()
    return eng


def _llama_engine(s, batch, session_len, max_prefill):
    from .engine import Engine
    rope = SimpleNamespace(dim=128, base=10000.0, type='default', factor=1.0, low_freq_factor=1.0, high_freq_factor=4.0,
                           original_max_position_embeddings=8192)
    cfg = SimpleNamespace(hidden=s['width'], layers=s['layers'], q_heads=s['heads'], kv_heads=s['kv_heads'], head_dim=128, inter=s['inter'],
                          vocab=s['vocab'], rms_eps=1e-5, rope=rope, group=128)
    eng = Engine.from_model_config(cfg, weight_type=1, max_batch_size=batch, session_len=session_len, quant_policy=0,
                                   max_prefill_token_num=max_prefill)
    eng.init_synthetic(seed=1)
    eng.start()
    return eng


def _measure(eng, vocab, batch, prompt_len, steps, warmup, prefill_seqs):
    rng = np.random.default_rng(0)
    out = {}
    # prefill: `prefill_seqs` prompts in one admission (chunked to max_prefill_token_num tokens per forward)
    prompts = [rng.integers(0, vocab, prompt_len).astype(np.int32) for _ in range(prefill_seqs)]
    for rep in range(2):        # the first pass loads code objects
        t0 = time.perf_counter()
        eng.prefill(prompts, max_new_tokens=2)
        eng.sync()
        dt = time.perf_counter() - t0
        eng.release()
    out['prefill_tokens_per_s'] = prefill_seqs * prompt_len / dt
    out['prefill_ms'] = dt * 1e3
    # decode: `batch` sequences with `prompt_len` tokens of context
    prompts = [rng.integers(0, vocab, prompt_len).astype(np.int32) for _ in range(batch)]
    eng.prefill(prompts, max_new_tokens=warmup + steps + 24)
    eng.decode(warmup)
    eng.sync()
    t0 = time.perf_counter()
    eng.decode(steps)
    eng.sync()
    dt = time.perf_counter() - t0
    out['decode_tokens_per_s'] = batch * steps / dt
    out['decode_ms_per_step'] = dt / steps * 1e3
    prof = eng.profile_decode(8)
    out['decode_categories_ms'] = {k: round(v[0], 4) for k, v in prof.items() if v[1] > 0}
    eng.release()
    return out


def _decode_bytes(s, batch, ctx, fokonex: bool):
    """bytes each category of ONE decode step must move (weights once, KV of the context once; activations are noise beside them)"""
    W, H, G, L, I, D = s['width'], s['heads'], s['kv_heads'], s['layers'], s['inter'], 128
    b = {'gemm_qkv': 2 * W * (H + 2 * G) * D * L, 'attention': 2 * 2 * G * D * ctx * batch * L, 'lm_head': 2 * W * s['vocab']}
    if fokonex:     # up; [o | down] fused in one GEMM
        b['gemm_gate_up'] = 2 * W * (I * 3 // 2) * L
        b['gemm_o'] = 2 * W * (H * D + I * 3 // 2) * L
    else:
        b['gemm_gate_up'] = 2 * W * 2 * I * L
        b['gemm_o'] = 2 * W * H * D * L
        b['gemm_down'] = 2 * W * I * L
    return b


def run(steps: int, warmup: int, batch: int, prompt_len: int, sizes=None) -> dict:
    res = {}
    for name in (sizes or SIZES):
        s = SIZES[name]
        session_len = prompt_len + steps + warmup + 64
        prefill_seqs = max(1, 8192 // prompt_len)
        row = {}
        for kind, make in (('fokonex_bf16', _fokonex_engine), ('llama_f16', _llama_engine)):
            eng = make(s, batch, session_len, 8192)
            m = _measure(eng, s['vocab'], batch, prompt_len, steps, warmup, prefill_seqs)
            need = _decode_bytes(s, batch, prompt_len + warmup + steps // 2, kind == 'fokonex_bf16')
            m['decode_hbm_roofline_fraction'] = {k: round(need[k] / HBM_BYTES_PER_S / (m['decode_categories_ms'][k] * 1e-3), 4)
                                                 for k in need if m['decode_categories_ms'].get(k)}
            eng.close()
            row[kind] = m
        f, l = row['fokonex_bf16'], row['llama_f16']
        row['prefill_ratio'] = round(f['prefill_tokens_per_s'] / l['prefill_tokens_per_s'], 3)
        row['decode_ratio'] = round(f['decode_tokens_per_s'] / l['decode_tokens_per_s'], 3)
        res[name] = row
    return res
