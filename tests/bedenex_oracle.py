"""Slow float64 model of the Bedenex design, written from its equations: one function per mechanism, whole sequences only (no cache, no
batch, no portions).  The GPU tests compare the engine with it; it shares nothing with the product path.

Notation: T tokens, W width, x the residual stream [T, W], h = norm(x) the input of both sublayers of a block, p the position of a token
in its sequence (from 0).  Weights are stored [out, in] and applied as h @ w.T.
"""
from __future__ import annotations

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


def rotate_half(x, pos, base):
    """x [T, ..., d]: channel i pairs with i + d/2; the pair turns by the angle pos * base^(-2i/d)"""
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
    q_plain, q_rot = q[..., :D], rotate_half(q[..., D:], pos, m['rot']['base'])
    dkv = h @ t['dkv'].T
    c = rms_norm(dkv[:, :C], t['dkv.norm'], eps)
    k_rot = rotate_half(dkv[:, C:], pos, m['rot']['base'])  # [T, R]
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


def moe_ff(h, t, mlp):
    """sigmoid router; the `top` best experts of a token (ties: the lower index); the score scales the expert's INPUT"""
    E, top = mlp['router']['experts'], mlp['router']['top']
    score = sigmoid(h @ t['router'].T)
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
