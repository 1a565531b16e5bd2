"""Plain float64 model of the Febivik design, written from its equations: one function per mechanism, whole sequences, no cache, no
batching -- nothing here is shared with the engine.  `cfg` is the parsed config.json, `w` maps tensor names to float64 arrays.

A block adds the layer-normed RESULT of each sublayer to the stream: x += LN1(mixer(x)); x += LN2(ff(x)); the sublayers read x as it is.
Mixers: `lightning` (linear attention with one decay per head), `attention` (grouped-query soft-max attention with biases, per-head
query / key RMS norm, partial rotation, a sliding window that also keeps the first tokens), `general_delta` (a delta-rule recurrence
with a decay and a removal rate per key channel).  Feed-forwards: dense with the xIELU activation, or routed experts (soft-max router,
squared-ReLU experts, a shared expert)."""
import numpy as np


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def rms_norm(x, w, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z) + z / 2"""
    pos = softplus(p) * z * z + 0.5 * z
    neg = (0.5 + softplus(q)) * (np.expm1(np.minimum(z, 0.0)) - z) + 0.5 * z
    return np.where(z > 0, pos, neg)


def rotate(x, pos, dims, base, factor):
    """x [T, heads, dim]: channel i < dims/2 turns with channel i + dims/2 by the angle pos * base^(-2i/dims) / factor"""
    if dims <= 0:
        return x
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims) / factor
    ang = np.asarray(pos, np.float64)[:, None, None] * f[None, None, :]
    c, s = np.cos(ang), np.sin(ang)
    u, v = x[..., :half], x[..., half:dims]
    out = x.copy()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def visible(i, j, window, keep_first):
    """may position i read position j?  inside the window, or one of the first tokens (window <= 0: no window)"""
    if j > i:
        return False
    if window <= 0:
        return True
    return i - j < window or j < keep_first


def windowed_attention(q, k, v, scale, window, keep_first, pos0=0):
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; query head h reads key head h // (H / G)"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            js = [j for j in range(T) if visible(i + pos0, j + pos0, window, keep_first)]
            s = (k[js, g] @ q[i, h]) * scale
            p = np.exp(s - s.max())
            out[i, h] = (p / p.sum()) @ v[js, g]
    return out


def attention_mixer(h, m, w, p, eps):
    T = h.shape[0]
    H, d = m['heads'], m['dim']
    G, dv = m.get('kv_heads', H), m.get('vdim', d)
    q = (h @ w[p + 'q'].T + w[p + 'q.b']).reshape(T, H, d)
    k = (h @ w[p + 'k'].T + w[p + 'k.b']).reshape(T, G, d)
    v = (h @ w[p + 'v'].T + w[p + 'v.b']).reshape(T, G, dv)
    q, k = rms_norm(q, w[p + 'q.norm'], eps), rms_norm(k, w[p + 'k.norm'], eps)
    rot, mask = m.get('rot') or {}, m.get('mask') or {}
    factor = float((rot.get('scaling') or {}).get('factor', 1.0))
    pos = np.arange(T)
    dims = int(rot.get('dims', d)) if rot else 0
    q = rotate(q, pos, dims, float(rot.get('base', 10000.0)), factor)
    k = rotate(k, pos, dims, float(rot.get('base', 10000.0)), factor)
    o = windowed_attention(q, k, v, m.get('scale', d ** -0.5), int(mask.get('size', 0)), int(mask.get('keep_first', 0)))
    return o.reshape(T, H * dv) @ w[p + 'o'].T


def lightning_recurrence(q, k, v, decay, state=None):
    """per head S <- decay S + k v^T, o = S^T q.  q, k [T, H, d], v [T, H, dv]; returns (o [T, H, dv], final state [H, d, dv])"""
    T, H, d = q.shape
    S = np.zeros((H, d, v.shape[2])) if state is None else state.copy()
    o = np.zeros((T, H, v.shape[2]))
    for t in range(T):
        for h in range(H):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    return o, S


def lightning_mixer(h, m, w, p, eps):
    T = h.shape[0]
    H, d, dv = m['heads'], m['dim'], m['vdim']
    q = silu(h @ w[p + 'q'].T).reshape(T, H, d)
    k = silu(h @ w[p + 'k'].T).reshape(T, H, d)
    v = silu(h @ w[p + 'v'].T).reshape(T, H, dv)
    o, _ = lightning_recurrence(q, k, v, np.asarray(m['decay'], np.float64))
    o = rms_norm(o.reshape(T, H * dv), w[p + 'norm'], eps) * sigmoid(h @ w[p + 'g'].T)
    return o @ w[p + 'o'].T


def delta_recurrence(r, k, v, decay, rate, state=None):
    """per head, with the unit key u = k / sqrt(|k|^2 + 1e-6):  S <- diag(decay) S - (rate * u)(u^T S) + k v^T, both from the old S;
    o = S^T r.  All inputs [T, H, d]."""
    T, H, d = r.shape
    S = np.zeros((H, d, d)) if state is None else state.copy()
    o = np.zeros((T, H, d))
    for t in range(T):
        for h in range(H):
            u = k[t, h] / np.sqrt((k[t, h] ** 2).sum() + 1e-6)
            S[h] = decay[t, h][:, None] * S[h] - np.outer(rate[t, h] * u, u @ S[h]) + np.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ r[t, h]
    return o, S


def delta_mixer(h, m, w, p, eps):
    T = h.shape[0]
    H, d = m['heads'], m['dim']
    r = (h @ w[p + 'r'].T).reshape(T, H, d)
    k = (h @ w[p + 'k'].T).reshape(T, H, d)
    v = (h @ w[p + 'v'].T).reshape(T, H, d)
    decay = np.exp(-np.exp(-0.5) * sigmoid(np.tanh(h @ w[p + 'w1'].T) @ w[p + 'w2'].T + w[p + 'w0'])).reshape(T, H, d)
    rate = sigmoid(h @ w[p + 'a'].T + w[p + 'a.b']).reshape(T, H, d)
    o, _ = delta_recurrence(r, k, v, decay, rate)
    o = o / np.sqrt((o * o).mean(-1, keepdims=True) + eps)
    o = o.reshape(T, H * d) * w[p + 'norm'] * sigmoid(h @ w[p + 'g'].T)
    return o @ w[p + 'o'].T


def dense_ff(h, w, p):
    a = w[p + 'act']
    return xielu(h @ w[p + 'up'].T, a[0], a[1]) @ w[p + 'down'].T


def relu2_expert(h, w, p):
    z = np.maximum(h @ w[p + 'up'].T, 0.0)
    return (z * z) @ w[p + 'down'].T


def route(h, w_router, top):
    """soft-max scores over all experts; the `top` largest per token (ties: lower index) -> (indices [T, top], scores [T, top])"""
    z = h @ w_router.T
    s = np.exp(z - z.max(-1, keepdims=True))
    s /= s.sum(-1, keepdims=True)
    idx = np.argsort(-s, axis=-1, kind='stable')[:, :top]
    return idx, np.take_along_axis(s, idx, -1)


def moe_ff(h, f, w, p):
    idx, sc = route(h, w[p + 'router'], int(f['router']['top']))
    out = np.zeros((h.shape[0], w[p + 'e0.down'].shape[0]))
    for t in range(h.shape[0]):
        for e, s in zip(idx[t], sc[t]):
            out[t] += float(f['router'].get('scale', 1.0)) * s * relu2_expert(h[t:t + 1], w, p + f'e{e}.')[0]
    if f.get('shared'):
        out += relu2_expert(h, w, p + 'shared.')
    return out


MIXERS = {'lightning': lightning_mixer, 'attention': attention_mixer, 'general_delta': delta_mixer}


def forward(cfg, w, tokens, return_layers=False):
    """logits [T, vocab] of one whole sequence (and the stream behind every layer)"""
    eps = float(cfg['norm']['eps'])
    x = w['embed'][np.asarray(tokens)]
    stream = []
    for i, L in enumerate(cfg['layers']):
        p = f'l{i}.'
        y = MIXERS[L['type']](x, L['mixer'], w, p + 'mix.', eps)
        x = x + layer_norm(y, w[p + 'norm1'], w[p + 'norm1.b'], eps)
        f = L.get('mlp')
        if f is not None:
            y = dense_ff(x, w, p + 'mlp.') if f['kind'] == 'dense' else moe_ff(x, f, w, p + 'mlp.')
            x = x + layer_norm(y, w[p + 'norm2'], w[p + 'norm2.b'], eps)
        stream.append(x.copy())
    logits = layer_norm(x, w['final.norm'], w['final.norm.b'], eps) @ w['head'].T
    return (logits, np.stack(stream)) if return_layers else logits


def router_gap(cfg, w, tokens):
    """smallest difference between the router logits of the last chosen and the first rejected expert over all tokens and routed layers: a
    model whose gap is tiny holds a decision that rounding can turn"""
    eps = float(cfg['norm']['eps'])
    x = w['embed'][np.asarray(tokens)]
    gap = np.inf
    for i, L in enumerate(cfg['layers']):
        p = f'l{i}.'
        x = x + layer_norm(MIXERS[L['type']](x, L['mixer'], w, p + 'mix.', eps), w[p + 'norm1'], w[p + 'norm1.b'], eps)
        f = L.get('mlp')
        if f is None:
            continue
        if f['kind'] == 'moe' and int(f['router']['top']) < int(f['router']['experts']):
            z = np.sort(x @ w[p + 'mlp.router'].T, -1)[:, ::-1]
            k = int(f['router']['top'])
            gap = min(gap, float((z[:, k - 1] - z[:, k]).min()))
        y = dense_ff(x, w, p + 'mlp.') if f['kind'] == 'dense' else moe_ff(x, f, w, p + 'mlp.')
        x = x + layer_norm(y, w[p + 'norm2'], w[p + 'norm2.b'], eps)
    return gap


def random_weights(cfg, seed=0, scale=1.0):
    """{name: float64 array of bf16-representable values} for a config; matrices N(0, 1/in), vectors small"""
    rng = np.random.default_rng(seed)
    W, out = int(cfg['width']), {}

    def bf16(a):
        b = np.asarray(a, np.float32).view(np.uint32)
        b = ((b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
        return b.view(np.float32).astype(np.float64)

    def mat(n, k, s=1.0):
        return bf16(rng.standard_normal((n, k)) * s * scale / np.sqrt(k))

    def vec(n, mean=0.0, s=0.1):
        return bf16(mean + s * rng.standard_normal(n))

    out['embed'] = bf16(rng.standard_normal((int(cfg['vocab']), W)))
    out['head'] = mat(int(cfg['vocab']), W)
    out['final.norm'], out['final.norm.b'] = vec(W, 1.0), vec(W)
    for i, L in enumerate(cfg['layers']):
        p, m = f'l{i}.', L['mixer']
        out[p + 'norm1'], out[p + 'norm1.b'] = vec(W, 1.0), vec(W)
        q = p + 'mix.'
        if L['type'] == 'lightning':
            H, d, dv = m['heads'], m['dim'], m['vdim']
            out[q + 'q'], out[q + 'k'], out[q + 'v'], out[q + 'g'] = mat(H * d, W), mat(H * d, W), mat(H * dv, W), mat(H * dv, W)
            out[q + 'norm'], out[q + 'o'] = vec(H * dv, 1.0), mat(W, H * dv)
        elif L['type'] == 'attention':
            H, G, d, dv = m['heads'], m['kv_heads'], m['dim'], m['vdim']
            out[q + 'q'], out[q + 'k'], out[q + 'v'] = mat(H * d, W, 2.0), mat(G * d, W, 2.0), mat(G * dv, W)
            out[q + 'q.b'], out[q + 'k.b'], out[q + 'v.b'] = vec(H * d), vec(G * d), vec(G * dv)
            out[q + 'q.norm'], out[q + 'k.norm'] = vec(d, 1.0), vec(d, 1.0)
            out[q + 'o'] = mat(W, H * dv)
        else:
            H, d = m['heads'], m['dim']
            lo = max(1, min(16, W // 4))
            for t in 'rkvga':
                out[q + t] = mat(H * d, W)
            out[q + 'a.b'], out[q + 'w0'] = vec(H * d), vec(H * d, 0.0, 1.0)
            out[q + 'w1'], out[q + 'w2'] = mat(int(m.get('decay_rank', lo)), W), mat(H * d, int(m.get('decay_rank', lo)))
            out[q + 'norm'], out[q + 'o'] = vec(H * d, 1.0), mat(W, H * d)
        f = L.get('mlp')
        if f is None:
            continue
        out[p + 'norm2'], out[p + 'norm2.b'] = vec(W, 1.0), vec(W)
        q = p + 'mlp.'
        if f['kind'] == 'dense':
            out[q + 'up'], out[q + 'down'], out[q + 'act'] = mat(f['ff'], W), mat(W, f['ff']), vec(2, 0.3, 0.5)
        else:
            out[q + 'router'] = mat(f['router']['experts'], W, 2.0)
            for e in range(f['router']['experts']):
                out[q + f'e{e}.up'], out[q + f'e{e}.down'] = mat(f['expert']['ff'], W), mat(W, f['expert']['ff'])
            if f.get('shared'):
                out[q + 'shared.up'], out[q + 'shared.down'] = mat(f['shared']['ff'], W), mat(W, f['shared']['ff'])
    return out


# ---- configurations, checkpoints, generation (test plumbing) ---------------------------------------------------------------------------
def lightning_layer(heads, dim, vdim, decay, mlp=None):
    return {'type': 'lightning', 'mixer': {'heads': heads, 'dim': dim, 'vdim': vdim, 'decay': list(decay)}, 'mlp': mlp}


def attention_layer(heads, kv_heads, dim, vdim, scale, window=0, keep_first=0, rot_dims=0, base=10000.0, factor=1.0, mlp=None):
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'scale': scale}
    if window:
        m['mask'] = {'size': window, 'keep_first': keep_first}
    if rot_dims:
        m['rot'] = {'dims': rot_dims, 'base': base, 'scaling': {'factor': factor}}
    return {'type': 'attention', 'mixer': m, 'mlp': mlp}


def delta_layer(heads, dim, rank=None, mlp=None):
    m = {'heads': heads, 'dim': dim}
    if rank:
        m['decay_rank'] = rank
    return {'type': 'general_delta', 'mixer': m, 'mlp': mlp}


def dense(ff):
    return {'kind': 'dense', 'ff': ff}


def moe(experts, top, ff, scale=1.0, shared=0):
    f = {'kind': 'moe', 'expert': {'ff': ff}, 'router': {'experts': experts, 'top': top, 'scale': scale}}
    if shared:
        f['shared'] = {'ff': shared}
    return f


def make_config(width, vocab, layers, eps=1e-5):
    return {'architecture': 'Febivik', 'width': width, 'vocab': vocab, 'norm': {'eps': eps}, 'layers': layers}


def bf16_bits(x):
    b = np.ascontiguousarray(np.asarray(x, np.float32)).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def write_checkpoint(folder, cfg, w):
    """config.json + model.safetensors (8-byte length, JSON header, bf16 data), written by hand"""
    import json
    import os
    import struct
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
