"""Plain float64 model of the Mededra design, written from its equations: one function per mechanism, whole sequences, no cache, no
batching -- nothing here is shared with the engine.  `cfg` is the parsed config.json, `w` maps tensor names to float64 arrays.

A block adds the group-normed RESULT of each sublayer to the stream: x += GN1(mixer(x)); x += GN2(ff(x)); the sublayers read x as it
is.  GN splits the row into `groups` equal parts, scales every part to unit RMS and multiplies the whole by a weight.
Mixers: `attention` -- differential attention: two score maps per head over the same values, each query / key map RMS-normed with a
shared weight and rotated pairwise (interleaved pairs, YaRN-scaled frequencies), capped scores, a sliding window, the second map
subtracted with a learned factor, the head's result scaled to unit RMS; every projection passes a short causal convolution first.
`parallel` -- two mixers on the same input whose RMS-normed results are averaged: a windowed attention whose values are its unnormed
keys, with a bucketed distance bias, scores mixed between heads, one added to the soft-max denominator and a sigmoid gate on the output;
and a gated delta rule (convolved, silu'd, unit-normed queries and keys, a decay per head and key channel, a write strength per head).
Feed-forward: gated silu.  Logits are capped."""
import json
import math
import os
import struct

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms(x, eps):
    """x divided by its root mean square over the last axis"""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def group_norm(x, w, groups, eps):
    """[T, n]: `groups` consecutive equal parts, each to unit RMS; then the whole times w"""
    T, n = x.shape
    return rms(x.reshape(T, groups, n // groups), eps).reshape(T, n) * w


def short_conv(u, wc, before=None):
    """u [T, C], wc [C, taps]: y_t = sum_j wc[:, j] u_(t - taps + 1 + j); `before` [taps - 1, C] are the inputs ahead of u (zeros if None)"""
    T, C = u.shape
    taps = wc.shape[1]
    pad = np.zeros((taps - 1, C)) if before is None else np.asarray(before, np.float64)
    full = np.concatenate([pad, u], 0)
    y = np.zeros((T, C))
    for j in range(taps):
        y += full[j:j + T] * wc[:, j]
    return y


def yarn_frequencies(dims, base, scaling):
    """(frequencies [dims / 2], factor on cos and sin)"""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling['factor']), float(scaling['original'])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(dim_of(float(scaling['fast']))), 0)
    hi = min(math.ceil(dim_of(float(scaling['slow']))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, pos, dims, base, scaling):
    """x [T, ..., dim]: channels (2i, 2i + 1), i < dims / 2, turn by pos * f_i; the rest pass"""
    if dims <= 0:
        return x
    f, mult = yarn_frequencies(dims, base, scaling)
    ang = np.asarray(pos, np.float64).reshape((-1,) + (1,) * (x.ndim - 1)) * f
    c, s = np.cos(ang) * mult, np.sin(ang) * mult
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def window_mask(T, window, pos0=0):
    """[T, T] bool: row i sees column j iff 0 <= i - j < window (window <= 0: every earlier token)"""
    d = np.arange(T)[:, None] - np.arange(T)[None, :]
    return (d >= 0) & ((d < window) if window > 0 else True)


def softmax_rows(s, mask, plus_one=False):
    """soft-max over the visible columns; plus_one: a sink with score 0 and no value joins the denominator"""
    s = np.where(mask, s, -np.inf)
    m = s.max(-1, keepdims=True)
    if plus_one:
        m = np.maximum(m, 0.0)
    e = np.exp(s - m)
    den = e.sum(-1, keepdims=True) + (np.exp(-m) if plus_one else 0.0)
    return e / den


def diff_lambda(w, p, diff):
    return math.exp(float(w[p + 'lq1'] @ w[p + 'lk1'])) - math.exp(float(w[p + 'lq2'] @ w[p + 'lk2'])) + diff


def diff_attention_mixer(h, m, w, p, eps, pos0=0):
    """h [T, W] -> [T, W]"""
    T = h.shape[0]
    H, G, d, dv = int(m['heads']), int(m['kv_heads']), int(m['dim']), int(m['vdim'])
    q, k, v = h @ w[p + 'q'].T, h @ w[p + 'k'].T, h @ w[p + 'v'].T
    q, k, v = short_conv(q, w[p + 'q.conv']), short_conv(k, w[p + 'k.conv']), short_conv(v, w[p + 'v.conv'])
    q, k, v = q.reshape(T, H, 2, d), k.reshape(T, G, 2, d), v.reshape(T, G, dv)
    q, k = rms(q, eps) * w[p + 'q.norm'], rms(k, eps) * w[p + 'k.norm']
    rot = m.get('rot') or {}
    pos = np.arange(T) + pos0
    if rot:
        dims = int(rot.get('dims', d))
        q = rotate_pairs(q, pos, dims, float(rot['base']), rot.get('scaling'))
        k = rotate_pairs(k, pos, dims, float(rot['base']), rot.get('scaling'))
    mask = window_mask(T, int((m.get('mask') or {}).get('size', 0)))
    cap, diff = float(m.get('softcap') or 0.0), float(m['diff'])
    lam = diff_lambda(w, p, diff)
    out = np.zeros((T, H, dv))
    for hh in range(H):
        g = hh // (H // G)
        a = []
        for mp in range(2):
            s = (q[:, hh, mp] @ k[:, g, mp].T) * float(m['scale'])
            if cap > 0:
                s = cap * np.tanh(s / cap)
            a.append(softmax_rows(s, mask) @ v[:, g])
        out[:, hh] = rms(a[0] - lam * a[1], eps) * (1.0 - diff)
    return out.reshape(T, H * dv) @ w[p + 'o'].T


def distance_bucket(n, B, D):
    """bucket of the distance n >= 0 among B buckets: one per distance below B / 2, logarithmic up to D above"""
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(D / half) * (B - half))))


def biased_attention_mixer(h, m, w, p, eps):
    """the left mixer of a parallel block"""
    T = h.shape[0]
    H, G, d, dv = int(m['heads']), int(m['kv_heads']), int(m['dim']), int(m['vdim'])
    q, k = h @ w[p + 'q'].T, h @ w[p + 'k'].T
    v = k.reshape(T, G, dv)                              # the values are the keys as projected
    q = (rms(q, eps) * w[p + 'q.norm']).reshape(T, H, d)
    k = (rms(k, eps) * w[p + 'k.norm']).reshape(T, G, d)
    rel, talk = w[p + 'rel'], w[p + 'talk']
    B, D = rel.shape[0], float(m['bias_max'])
    dist = np.arange(T)[:, None] - np.arange(T)[None, :]
    bucket = np.vectorize(lambda n: distance_bucket(n, B, D) if n >= 0 else 0)(dist)
    s = np.zeros((H, T, T))
    for hh in range(H):
        s[hh] = (q[:, hh] @ k[:, hh // (H // G)].T) * float(m['scale']) + rel[bucket, hh]
    s = np.einsum('hg,gij->hij', talk, s)
    mask = window_mask(T, int((m.get('mask') or {}).get('size', 0)))
    out = np.zeros((T, H, dv))
    for hh in range(H):
        out[:, hh] = softmax_rows(s[hh], mask, plus_one=True) @ v[:, hh // (H // G)]
    return (out.reshape(T, H * dv) * sigmoid(h @ w[p + 'g'].T)) @ w[p + 'o'].T


def gated_delta_recurrence(q, k, v, g, beta, state=None):
    """q, k, g [T, d], v [T, dv], beta [T]: S <- g S (rows); u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  Returns (o [T, dv], S)"""
    T, d = q.shape
    S = np.zeros((d, v.shape[1])) if state is None else state.copy()
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def gated_delta_mixer(h, m, w, p, eps):
    """the right mixer of a parallel block"""
    T = h.shape[0]
    H, G, d, dv = int(m['heads']), int(m['kv_heads']), int(m['dim']), int(m['vdim'])
    q = silu(short_conv(h @ w[p + 'q'].T, w[p + 'q.conv'])).reshape(T, G, d)
    k = silu(short_conv(h @ w[p + 'k'].T, w[p + 'k.conv'])).reshape(T, G, d)
    v = silu(short_conv(h @ w[p + 'v'].T, w[p + 'v.conv'])).reshape(T, H, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ w[p + 'b'].T)                                                   # [T, H]
    dt = softplus((h @ w[p + 'a1'].T) @ w[p + 'a2'].T + w[p + 'dt_bias']).reshape(T, H, d)
    g = np.exp(-np.exp(w[p + 'A_log'])[None, :, None] * dt)
    gate = sigmoid((h @ w[p + 'g1'].T) @ w[p + 'g2'].T).reshape(T, H, dv)
    out = np.zeros((T, H, dv))
    for hh in range(H):
        c = hh // (H // G)
        o, _ = gated_delta_recurrence(q[:, c], k[:, c], v[:, hh], g[:, hh], beta[:, hh])
        out[:, hh] = rms(o, eps) * w[p + 'norm'] * gate[:, hh]
    return out.reshape(T, H * dv) @ w[p + 'o'].T


def parallel_mixer(h, m, w, p, eps):
    left = biased_attention_mixer(h, m['left'], w, p + 'left.', eps)
    right = gated_delta_mixer(h, m['right'], w, p + 'right.', eps)
    return 0.5 * (rms(left, eps) * w[p + 'left.out'] + rms(right, eps) * w[p + 'right.out'])


def gated_ff(h, w, p):
    return (silu(h @ w[p + 'gate'].T) * (h @ w[p + 'up'].T)) @ w[p + 'down'].T


def forward(cfg, w, tokens, return_layers=False):
    """logits [T, vocab] of one sequence (and the stream behind every layer)"""
    eps, groups = float(cfg['norm']['eps']), int(cfg['norm'].get('groups', 1))
    x = w['embed'][np.asarray(tokens)] * float((cfg.get('embedding') or {}).get('scale', 1.0))
    layers = []
    for i, L in enumerate(cfg['layers']):
        p = f'l{i}.'
        if L['type'] == 'attention':
            y = diff_attention_mixer(x, L['mixer'], w, p + 'mix.', eps)
        elif L['type'] == 'parallel':
            y = parallel_mixer(x, L['mixer'], w, p + 'mix.', eps)
        else:
            raise NotImplementedError(L['type'])
        x = x + group_norm(y, w[p + 'norm1'], groups, eps)
        if L.get('mlp') is not None:
            x = x + group_norm(gated_ff(x, w, p + 'mlp.'), w[p + 'norm2'], groups, eps)
        layers.append(x.copy())
    logits = group_norm(x, w['final.norm'], groups, eps) @ w['head'].T
    cap = float(cfg.get('logit_softcap') or 0.0)
    if cap > 0:
        logits = cap * np.tanh(logits / cap)
    return (logits, np.stack(layers)) if return_layers else logits


# ---- configurations, random weights, checkpoints ------------------------------------------------------------------------------------
def attention_layer(heads, kv_heads, dim, vdim, scale=None, window=0, rot_dims=None, base=10000.0, scaling=None, softcap=0.0, diff=0.5, conv=3,
                    mlp=None):
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'scale': dim ** -0.5 if scale is None else scale, 'diff': diff,
         'conv': conv, 'softcap': softcap}
    if window:
        m['mask'] = {'size': window}
    if rot_dims is None or rot_dims > 0:
        m['rot'] = {'base': base, 'dims': dim if rot_dims is None else rot_dims}
        if scaling:
            m['rot']['scaling'] = scaling
    return {'type': 'attention', 'mixer': m, 'mlp': mlp}


def parallel_layer(left, right, mlp=None):
    return {'type': 'parallel', 'mixer': {'left': left, 'right': right}, 'mlp': mlp}


def left_mixer(heads, kv_heads, dim, window, bias_max, scale=None):
    return {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': dim, 'scale': dim ** -0.5 if scale is None else scale,
            'mask': {'size': window}, 'bias_max': bias_max}


def right_mixer(heads, kv_heads, dim, vdim, conv=3):
    return {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'conv': conv}


def dense(ff):
    return {'kind': 'dense', 'ff': ff}


def make_config(width, vocab, layers, eps=1e-5, groups=1, embed_scale=1.0, logit_softcap=0.0):
    return {'architecture': 'Mededra', 'width': width, 'vocab': vocab, 'norm': {'eps': eps, 'groups': groups},
            'embedding': {'scale': embed_scale}, 'logit_softcap': logit_softcap, 'layers': layers}


def tensor_shapes(cfg, buckets=16, a_rank=8, g_rank=8):
    W, V = int(cfg['width']), int(cfg['vocab'])
    out = {'embed': (V, W), 'final.norm': (W,), 'head': (V, W)}
    for i, L in enumerate(cfg['layers']):
        p, m = f'l{i}.', L['mixer']
        out[p + 'norm1'] = (W,)
        if L['type'] == 'attention':
            H, G, d, dv, taps = m['heads'], m['kv_heads'], m['dim'], m['vdim'], m['conv']
            for t, n in (('q', H * 2 * d), ('k', G * 2 * d), ('v', G * dv)):
                out[p + 'mix.' + t], out[p + f'mix.{t}.conv'] = (n, W), (n, taps)
            for t in ('q.norm', 'k.norm', 'lq1', 'lk1', 'lq2', 'lk2'):
                out[p + 'mix.' + t] = (d,)
            out[p + 'mix.o'] = (W, H * dv)
        else:
            a, b = m['left'], m['right']
            H, G, d = a['heads'], a['kv_heads'], a['dim']
            out.update({p + 'mix.left.q': (H * d, W), p + 'mix.left.k': (G * d, W), p + 'mix.left.q.norm': (H * d,),
                        p + 'mix.left.k.norm': (G * d,), p + 'mix.left.rel': (buckets, H), p + 'mix.left.talk': (H, H),
                        p + 'mix.left.g': (H * a['vdim'], W), p + 'mix.left.o': (W, H * a['vdim']), p + 'mix.left.out': (W,),
                        p + 'mix.right.out': (W,)})
            H, G, d, dv, taps = b['heads'], b['kv_heads'], b['dim'], b['vdim'], b['conv']
            for t, n in (('q', G * d), ('k', G * d), ('v', H * dv)):
                out[p + 'mix.right.' + t], out[p + f'mix.right.{t}.conv'] = (n, W), (n, taps)
            out.update({p + 'mix.right.b': (H, W), p + 'mix.right.A_log': (H,), p + 'mix.right.norm': (dv,),
                        p + 'mix.right.a1': (a_rank, W), p + 'mix.right.a2': (H * d, a_rank), p + 'mix.right.dt_bias': (H * d,),
                        p + 'mix.right.g1': (g_rank, W), p + 'mix.right.g2': (H * dv, g_rank), p + 'mix.right.o': (W, H * dv)})
        if L.get('mlp') is not None:
            ff = L['mlp']['ff']
            out.update({p + 'norm2': (W,), p + 'mlp.gate': (ff, W), p + 'mlp.up': (ff, W), p + 'mlp.down': (W, ff)})
    return out


def bf16_round(x):
    b = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).astype(np.float64)


def random_weights(cfg, seed=0, **ranks):
    """bf16-representable float64 weights: matrices N(0, 1 / inputs), norm weights around 1, small vectors elsewhere"""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_shapes(cfg, **ranks).items():
        leaf = name.split('.')[-1]
        if name == 'embed':
            a = rng.standard_normal(shape)
        elif leaf in ('norm', 'norm1', 'norm2', 'out') and len(shape) == 1:
            a = 1.0 + 0.1 * rng.standard_normal(shape)
        elif leaf == 'conv':
            a = rng.standard_normal(shape) * 0.5 + (np.arange(shape[1]) == shape[1] - 1) * 0.5
        elif leaf == 'talk':
            a = np.eye(shape[0]) + 0.3 * rng.standard_normal(shape)
        elif leaf in ('rel', 'dt_bias', 'A_log'):
            a = rng.standard_normal(shape) * 0.5
        elif leaf in ('lq1', 'lk1', 'lq2', 'lk2'):
            a = rng.standard_normal(shape) * 0.3
        else:
            a = rng.standard_normal(shape) / math.sqrt(shape[-1])
        w[name] = bf16_round(a)
    return w


def bf16_bits(x):
    b = np.asarray(x, np.float32).view(np.uint32)
    return (b >> 16).astype(np.uint16)


def write_checkpoint(folder, cfg, w):
    """config.json + model.safetensors (bf16) in `folder`"""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, 'config.json'), 'w') as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name, a in w.items():
        raw = bf16_bits(a).tobytes()
        header[name] = {'dtype': 'BF16', 'shape': list(np.shape(a)), 'data_offsets': [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    hj = json.dumps(header).encode()
    hj += b' ' * (-len(hj) % 8)
    with open(os.path.join(folder, 'model.safetensors'), 'wb') as f:
        f.write(struct.pack('<Q', len(hj)) + hj + b''.join(blobs))


def greedy(cfg, w, prompt, n_new):
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(np.argmax(forward(cfg, w, toks)[-1])))
    return toks[len(prompt):]
