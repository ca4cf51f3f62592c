"""Slow float64 model of the Bedenex design, written from its equations: one function per mechanism, whole sequences only (no cache, no
batch, no portions).  The GPU tests compare the engine with it; it shares nothing with the product path.

Notation: T tokens, W width, x the residual stream [T, W], h = norm(x) the input of both sublayers of a block, p the position of a token
in its sequence (from 0).  Weights are stored [out, in] and applied as h @ w.T.
"""
from __future__ import annotations

import json
import os
import struct

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x scaled to root mean square 1 over its last axis (eps inside the root)"""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def rotate_half(x, pos, base, dims=None):
    """x [T, ..., n]: of the first d = dims channels (all when None) channel i pairs with i + d/2 and the pair turns by the angle
    pos * base^(-2i/d); channels from d on pass unchanged"""
    if dims is not None and dims < x.shape[-1]:
        return np.concatenate([rotate_half(x[..., :dims], pos, base), x[..., dims:]], axis=-1) if dims else x
    d = x.shape[-1]
    half = d // 2
    freq = base ** (-2.0 * np.arange(half) / d)
    ang = np.asarray(pos, np.float64)[:, None] * freq[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:]
    return np.concatenate([u * c - v * s, v * c + u * s], axis=-1)


def softmax_rows(scores, visible, sink=None):
    """scores [T, T] (query, key), visible boolean; sink: one more term exp(sink) in the denominator that has no value"""
    s = np.where(visible, scores, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink)
    e = np.where(visible, np.exp(s - m), 0.0)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink - m)
    return e / den


def chunk_attention(h, t, m, eps):
    """grouped-query attention without rotation: unit-RMS queries, keys and values per head, a logarithmic distance penalty
    r1 * ln(1 + r2 * (i - j)) per head, keys visible inside the query's own chunk of positions only, a sigmoid gate per head on the output.
    t: tensors q, k, v, r1, r2, g, o; m: heads, kv_heads, dim, vdim, scale, mask.size (absent: plain causal)"""
    T = h.shape[0]
    H, G, D, V = m['heads'], m['kv_heads'], m['dim'], m['vdim']
    q = unit_rms((h @ t['q'].T).reshape(T, H, D), eps)
    k = unit_rms((h @ t['k'].T).reshape(T, G, D), eps)
    v = unit_rms((h @ t['v'].T).reshape(T, G, V), eps)
    gate = sigmoid(h @ t['g'].T)  # [T, H]
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    visible = j <= i
    size = (m.get('mask') or {}).get('size')
    if size:
        visible = visible & (i // size == j // size)
    dist = np.where(visible, i - j, 0).astype(np.float64)
    out = np.zeros((T, H, V))
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m['scale'] - t['r1'][a] * np.log(1.0 + t['r2'][a] * dist)
        out[:, a] = softmax_rows(s, visible) @ v[:, g]
    out = out * gate[:, :, None]
    return out.reshape(T, H * V) @ t['o'].T


def latent_attention(h, t, m, eps):
    """keys and values of all heads expanded from one normed latent vector per token plus one rotated key part shared by the heads; plain
    causal; the soft-max denominator holds exp(sink) per head.  t: q, dkv, dkv.norm, uk, uv, sink, o; m: heads, dim, rot_dim, vdim, kv_rank,
    rot.base, scale"""
    T = h.shape[0]
    H, D, R, V, C = m['heads'], m['dim'], m['rot_dim'], m['vdim'], m['kv_rank']
    pos = np.arange(T)
    q = (h @ t['q'].T).reshape(T, H, D + R)
    dims = m['rot'].get('dims', R)
    q_plain, q_rot = q[..., :D], rotate_half(q[..., D:], pos, m['rot']['base'], dims)
    dkv = h @ t['dkv'].T
    c = rms_norm(dkv[:, :C], t['dkv.norm'], eps)
    k_rot = rotate_half(dkv[:, C:], pos, m['rot']['base'], dims)  # [T, R]
    k_plain = (c @ t['uk'].T).reshape(T, H, D)
    v = (c @ t['uv'].T).reshape(T, H, V)
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    visible = j <= i
    out = np.zeros((T, H, V))
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m['scale']
        out[:, a] = softmax_rows(s, visible, sink=t['sink'][a]) @ v[:, a]
    return out.reshape(T, H * V) @ t['o'].T


def dense_ff(h, t):
    return (gelu_tanh(h @ t['gate'].T) * (h @ t['up'].T)) @ t['down'].T


ROUTER_GAPS = []      # smallest gap between the last chosen and the first rejected router logit of every moe_ff call since it was cleared


def moe_ff(h, t, mlp):
    """sigmoid router; the `top` best experts of a token (ties: the lower index); the score scales the expert's INPUT"""
    E, top = mlp['router']['experts'], mlp['router']['top']
    z = h @ t['router'].T
    score = sigmoid(z)
    if top < E:
        zs = np.sort(z, axis=-1)
        ROUTER_GAPS.append(float((zs[:, E - top] - zs[:, E - top - 1]).min()))
    out = np.zeros((h.shape[0], t['e0.down'].shape[0]))
    for n in range(h.shape[0]):
        for e in np.argsort(-score[n], kind='stable')[:top]:
            z = score[n, e] * h[n]
            out[n] += (silu(z @ t[f'e{e}.gate'].T) * (z @ t[f'e{e}.up'].T)) @ t[f'e{e}.down'].T
    return out


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def block(x, tensors, i, layer, eps):
    """x + gate1 * mixer(h) + gate2 * ff(h), h = norm1(x), gate_i = sigmoid(rg_i h + b_i) element by element"""
    p = f'l{i}.'
    h = rms_norm(x, tensors[p + 'norm1'], eps)
    mix = sub(tensors, p + 'mix.')
    if layer['type'] == 'attention':
        y = chunk_attention(h, mix, layer['mixer'], eps)
    elif layer['type'] == 'latent_attention':
        y = latent_attention(h, mix, layer['mixer'], eps)
    else:
        raise NotImplementedError(layer['type'])
    out = x + sigmoid(h @ tensors[p + 'rg1'].T + tensors[p + 'rg1.b']) * y
    mlp = layer.get('mlp')
    if mlp is not None:
        t = sub(tensors, p + 'mlp.')
        f = dense_ff(h, t) if mlp['kind'] == 'dense' else moe_ff(h, t, mlp)
        out = out + sigmoid(h @ tensors[p + 'rg2'].T + tensors[p + 'rg2.b']) * f
    return out


def layer_runs(cfg):
    """[(layer index, pass number or None)]: the pass number stands at the first layer of every pass of the loop"""
    n = len(cfg['layers'])
    loop = cfg.get('loop')
    if not loop or loop['stop'] <= loop['start']:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop['start'])]
    for t in range(loop['times']):
        runs += [(i, t if i == loop['start'] else None) for i in range(loop['start'], loop['stop'])]
    return runs + [(i, None) for i in range(loop['stop'], n)]


def router_gap(cfg, tensors, requests):
    """the closest call any router makes over these token lists (logit units): reduced-precision runs may route a closer one differently"""
    ROUTER_GAPS.clear()
    for t in requests:
        forward(cfg, tensors, t)
    return min(ROUTER_GAPS) if ROUTER_GAPS else np.inf


def forward(cfg, tensors, tokens, want_layers=False):
    """tensors: {name: float64 array}; -> logits [T, vocab] (and the residual stream behind every layer run)"""
    eps = cfg['norm']['eps']
    x0 = tensors['embed'][np.asarray(tokens)]
    x, trail = x0, []
    for i, t in layer_runs(cfg):
        if t is not None:  # a pass of the loop begins: mix the stream with the embedding output, add the pass's vector
            x = np.concatenate([x, x0], axis=-1) @ tensors['loop.in'].T + tensors['loop.step'][t]
        x = block(x, tensors, i, cfg['layers'][i], eps)
        trail.append(x)
    logits = rms_norm(x, tensors['final.norm'], eps) @ tensors['head'].T
    return (logits, np.stack(trail)) if want_layers else logits


# ---- the tests' own models -----------------------------------------------------------------------------------------------------------
def bf16_round(x):
    """float64 values rounded to the nearest bfloat16 (ties to even), as float64"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def bf16_bits(x):
    return (np.ascontiguousarray(bf16_round(x), np.float32).view(np.uint32) >> 16).astype(np.uint16)


def attention_layer(heads, kv_heads, dim, vdim, scale, chunk, mlp=None):
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'scale': scale}
    if chunk:
        m['mask'] = {'size': chunk}
    return {'type': 'attention', 'mixer': m, 'mlp': mlp}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, mlp=None, dims=None):
    return {'type': 'latent_attention', 'mlp': mlp,
            'mixer': {'heads': heads, 'dim': dim, 'rot_dim': rot_dim, 'vdim': vdim, 'kv_rank': kv_rank, 'scale': scale,
                      'rot': {'base': base, 'dims': rot_dim if dims is None else dims}}}


def dense(ff):
    return {'kind': 'dense', 'ff': ff}


def moe(experts, top, ff):
    return {'kind': 'moe', 'expert': {'ff': ff}, 'router': {'experts': experts, 'top': top}}


def make_config(width, vocab, layers, loop=None, eps=1e-5):
    c = {'architecture': 'Bedenex', 'width': width, 'vocab': vocab, 'layers': layers, 'norm': {'eps': eps}}
    if loop:
        c['loop'] = {'start': loop[0], 'stop': loop[1], 'times': loop[2]}
    return c


def make_weights(cfg, seed, sink=3.0):
    """bf16-representable float64 tensors under the checkpoint's names.  Projections N(0, 1 / inputs); sinks around `sink` so that a
    forgotten sink moves every latent layer's output; distance numbers positive; gate biases around zero"""
    rng = np.random.default_rng(seed)
    W, w = cfg['width'], {}

    def mat(n_out, n_in, gain=1.0):
        return bf16_round(rng.normal(0, gain / np.sqrt(n_in), (n_out, n_in)))

    def vec(n, mean, std):
        return bf16_round(rng.normal(mean, std, n))

    w['embed'] = bf16_round(rng.normal(0, 1, (cfg['vocab'], W)))
    w['head'], w['final.norm'] = mat(cfg['vocab'], W), vec(W, 1.0, 0.2)
    loop = cfg.get('loop')
    if loop:
        w['loop.in'], w['loop.step'] = mat(W, 2 * W), bf16_round(rng.normal(0, 0.3, (loop['times'], W)))
    for i, L in enumerate(cfg['layers']):
        p, m = f'l{i}.', L['mixer']
        H, D, V = m['heads'], m['dim'], m['vdim']
        w[p + 'norm1'] = vec(W, 1.0, 0.2)
        w[p + 'rg1'], w[p + 'rg1.b'] = mat(W, W), vec(W, 0.0, 0.5)
        w[p + 'mix.o'] = mat(W, H * V)
        if L['type'] == 'attention':
            G = m['kv_heads']
            w[p + 'mix.q'], w[p + 'mix.k'], w[p + 'mix.v'] = mat(H * D, W), mat(G * D, W), mat(G * V, W)
            w[p + 'mix.g'] = mat(H, W)
            w[p + 'mix.r1'], w[p + 'mix.r2'] = np.abs(vec(H, 1.0, 0.6)), np.abs(vec(H, 0.3, 0.15))
        else:
            R, C = m['rot_dim'], m['kv_rank']
            w[p + 'mix.q'], w[p + 'mix.dkv'] = mat(H * (D + R), W, 2.0), mat(C + R, W, 2.0)
            w[p + 'mix.dkv.norm'] = vec(C, 1.0, 0.2)
            w[p + 'mix.uk'], w[p + 'mix.uv'] = mat(H * D, C, 2.0), mat(H * V, C)
            w[p + 'mix.sink'] = vec(H, sink, 1.0)
        mlp = L.get('mlp')
        if mlp is None:
            continue
        w[p + 'rg2'], w[p + 'rg2.b'] = mat(W, W), vec(W, 0.0, 0.5)
        if mlp['kind'] == 'dense':
            w[p + 'mlp.gate'], w[p + 'mlp.up'], w[p + 'mlp.down'] = mat(mlp['ff'], W, 2.0), mat(mlp['ff'], W), mat(W, mlp['ff'])
        else:
            w[p + 'mlp.router'] = mat(mlp['router']['experts'], W, 6.0)
            ff = mlp['expert']['ff']
            for e in range(mlp['router']['experts']):
                w[p + f'mlp.e{e}.gate'], w[p + f'mlp.e{e}.up'], w[p + f'mlp.e{e}.down'] = mat(ff, W, 3.0), mat(ff, W, 2.0), mat(W, ff)
    return w


def write_checkpoint(folder, cfg, w):
    """config.json + model.safetensors (8-byte length, JSON header, bf16 data), written by hand"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, 'config.json'), 'w') as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name in sorted(w):
        b = bf16_bits(w[name]).astype('<u2').tobytes()
        header[name] = {'dtype': 'BF16', 'shape': list(np.shape(w[name])), 'data_offsets': [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    with open(os.path.join(folder, 'model.safetensors'), 'wb') as f:
        f.write(struct.pack('<Q', len(hj)) + hj + b''.join(blobs))


def greedy(cfg, w, prompt, n_new):
    """-> (tokens, margins): arg-max continuation and the top-1 / top-2 logit gap of every step"""
    toks, out, margins = list(prompt), [], []
    for _ in range(n_new):
        lg = forward(cfg, w, toks)[-1]
        top = np.sort(lg)[-2:]
        out.append(int(lg.argmax()))
        margins.append(float(top[1] - top[0]))
        toks.append(out[-1])
    return out, margins
