"""Plain, slow float64 implementation of the layer-list decoder family, one function per mechanism, written from the equations:

    norm(x)      = x / sqrt(mean(x^2) + eps) * (offset + w)
    temp(p)      = 1 + coef * ln(floor((p + 1) / every) + 1)                      query temperature at position p
    cap(s)       = c * tanh(s / c)                                                 soft cap (c <= 0: identity)
    weights_i    = exp(s_i) / (sum_j exp(s_j) + exp(sink))                         soft-max with a sink logit (sink None: plain)
    attention    : s_ij = cap(temp(i) * (q_i . k_j) * scale) for j <= i, grouped heads (query head h -> kv head h // (H / G))
    feed-forward : down(relu(up(h))^2)
    block        : x + mult * (attention(norm1(x)) + ff(norm2(x)))
    logits       = head(norm_final(x)) * logit_scale

Shares no code with the engine or its loaders; tests build their own small configurations and random weights on top of it.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ---- bf16 <-> numpy ---------------------------------------------------------------------------------------------------------------
def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float -> bf16 bit patterns (uint16), round to nearest even"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7fff + ((u >> 16) & 1)) >> 16) & 0xffff).astype(np.uint16)


def from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def bf16(x: np.ndarray) -> np.ndarray:
    """values rounded to bf16, as float64"""
    return from_bf16_bits(to_bf16_bits(x))


# ---- mechanisms -------------------------------------------------------------------------------------------------------------------
def rms_norm(x, w, eps, offset):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * (offset + w)


def query_temperature(pos, coef, every):
    return 1.0 + coef * math.log(math.floor((pos + 1) / every) + 1.0)


def soft_cap(s, cap):
    return cap * np.tanh(s / cap) if cap > 0 else s


def sink_softmax(scores, sink):
    """scores: 1-d visible scores of one query; sink: float or None -> weights over the keys (they sum to < 1 with a sink)"""
    m = max(scores.max(), sink) if sink is not None else scores.max()
    e = np.exp(scores - m)
    return e / (e.sum() + (math.exp(sink - m) if sink is not None else 0.0))


def attention(h, wq, wk, wv, wo, sink, spec, k_hist=None, v_hist=None):
    """h [n, W] = normed rows of positions len(hist) .. len(hist) + n - 1; returns ([n, W], keys, values incl. history)"""
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    n = h.shape[0]
    q = (h @ wq.T).reshape(n, H, D)
    k = (h @ wk.T).reshape(n, G, D)
    v = (h @ wv.T).reshape(n, G, V)
    if k_hist is not None:
        k, v = np.concatenate([k_hist, k]), np.concatenate([v_hist, v])
    p0 = k.shape[0] - n
    out = np.zeros((n, H, V))
    for i in range(n):
        pos = p0 + i
        t = query_temperature(pos, spec['qtemp_coef'], spec['qtemp_every']) if spec['qtemp_coef'] else 1.0
        for hh in range(H):
            g = hh // (H // G)
            s = soft_cap((k[:pos + 1, g] @ (q[i, hh] * t)) * spec['scale'], spec['softcap'])
            w = sink_softmax(s, float(sink[hh]) if sink is not None else None)
            out[i, hh] = w @ v[:pos + 1, g]
    return out.reshape(n, H * V) @ wo.T, k, v


def relu2_mlp(h, up, down):
    return (np.maximum(h @ up.T, 0.0) ** 2) @ down.T


# ---- model ------------------------------------------------------------------------------------------------------------------------
def make_config(width, vocab, layers, eps=1e-5, mult=0.5, logit_scale=1.5, offset=1.0):
    """layers: list of dicts(heads, kv_heads, dim, vdim, scale, softcap, qtemp_coef, qtemp_every, sink, ff (0: no ff), weights_of (-1))"""
    return dict(width=width, vocab=vocab, layers=layers, eps=eps, mult=mult, logit_scale=logit_scale, offset=offset)


def make_weights(cfg, seed, spread=1.0):
    """{tensor name: float64 array of bf16-representable values}, checkpoint orientation [out, in]"""
    rng, W = np.random.default_rng(seed), cfg['width']
    w = {'embed': bf16(rng.normal(0, 1, (cfg['vocab'], W))), 'final.norm': bf16(rng.normal(0, 0.1, W)),
         'head': bf16(rng.normal(0, 1 / math.sqrt(W), (cfg['vocab'], W)))}
    for i, L in enumerate(cfg['layers']):
        if L['weights_of'] >= 0:
            continue
        p, H, G, D, V = f'l{i}.', L['heads'], L['kv_heads'], L['dim'], L['vdim']
        w[p + 'norm1'] = bf16(rng.normal(0, 0.1, W))
        w[p + 'mix.q'] = bf16(rng.normal(0, spread / math.sqrt(W), (H * D, W)))
        w[p + 'mix.k'] = bf16(rng.normal(0, spread / math.sqrt(W), (G * D, W)))
        w[p + 'mix.v'] = bf16(rng.normal(0, 1 / math.sqrt(W), (G * V, W)))
        w[p + 'mix.o'] = bf16(rng.normal(0, 1 / math.sqrt(H * V), (W, H * V)))
        if L['sink']:
            w[p + 'mix.sink'] = bf16(rng.normal(0, 1, H))
        if L['ff']:
            w[p + 'norm2'] = bf16(rng.normal(0, 0.1, W))
            w[p + 'mlp.up'] = bf16(rng.normal(0, 1 / math.sqrt(W), (L['ff'], W)))
            w[p + 'mlp.down'] = bf16(rng.normal(0, 1 / math.sqrt(L['ff']), (W, L['ff'])))
    return w


def forward(cfg, w, tokens, n_layers=None):
    """-> (logits [n, vocab], residual stream behind the last layer run [n, W])"""
    x = w['embed'][np.asarray(tokens)]
    for i, L in enumerate(cfg['layers'][:n_layers]):
        p = f'l{L["weights_of"] if L["weights_of"] >= 0 else i}.'
        y, _, _ = attention(rms_norm(x, w[p + 'norm1'], cfg['eps'], cfg['offset']), w[p + 'mix.q'], w[p + 'mix.k'], w[p + 'mix.v'],
                            w[p + 'mix.o'], w.get(p + 'mix.sink') if L['sink'] else None, L)
        if L['ff']:
            y = y + relu2_mlp(rms_norm(x, w[p + 'norm2'], cfg['eps'], cfg['offset']), w[p + 'mlp.up'], w[p + 'mlp.down'])
        x = x + cfg['mult'] * y
    return rms_norm(x, w['final.norm'], cfg['eps'], cfg['offset']) @ w['head'].T * cfg['logit_scale'], x


def greedy(cfg, w, prompt, n_new):
    """-> (tokens, margins): arg-max continuation and the top-1 / top-2 logit gap of every step"""
    toks, out, margins = list(prompt), [], []
    for _ in range(n_new):
        lg = forward(cfg, w, toks)[0][-1]
        top = np.sort(lg)[-2:]
        out.append(int(lg.argmax()))
        margins.append(float(top[1] - top[0]))
        toks.append(out[-1])
    return out, margins


# ---- checkpoint folder ------------------------------------------------------------------------------------------------------------
def config_json(cfg, arch='Fokonex'):
    layers = []
    for L in cfg['layers']:
        e = {'type': 'attention',
             'mixer': {'heads': L['heads'], 'kv_heads': L['kv_heads'], 'dim': L['dim'], 'vdim': L['vdim'], 'scale': L['scale'],
                       'softcap': L['softcap'], 'q_temp': {'coef': L['qtemp_coef'], 'every': L['qtemp_every']}},
             'mlp': {'kind': 'dense', 'ff': L['ff']} if L['ff'] else None}
        if L['weights_of'] >= 0:
            e['weights_of'] = L['weights_of']
        layers.append(e)
    return {'architecture': arch, 'width': cfg['width'], 'vocab': cfg['vocab'], 'layers': layers, 'norm': {'eps': cfg['eps']},
            'residual_mult': cfg['mult'], 'logit_scale': cfg['logit_scale']}


def write_checkpoint(folder, cfg, w):
    """config.json + model.safetensors (8-byte length, JSON header, bf16 data) written by hand"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, 'config.json'), 'w') as f:
        json.dump(config_json(cfg), f)
    header, blobs, off = {}, [], 0
    for name in sorted(w):
        b = to_bf16_bits(w[name]).astype('<u2').tobytes()
        header[name] = {'dtype': 'BF16', 'shape': list(w[name].shape), 'data_offsets': [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    with open(os.path.join(folder, 'model.safetensors'), 'wb') as f:
        f.write(struct.pack('<Q', len(hj)) + hj + b''.join(blobs))
