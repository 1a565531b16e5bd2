"""Layer-list model family: decoders described layer by layer in their config.json.

    {"architecture": NAME, "width", "vocab", "norm": {"eps"}, "residual_mult", "logit_scale",
     "layers": [{"type": MIXER, "mixer": {...sizes and constants...}, "mlp": {"kind", "ff"} | null, "weights_of": j}, ...],
     "loop": {"start", "stop", "times"}}

`FAMILIES` maps an architecture name to the reader that turns such a config into a `LayeredConfig` (the native engine's
tm_layered_config).  Weights are one `model.safetensors` of bf16 tensors, stored [out, in] under the names the engine's slots carry
("embed", "l<i>.norm1", "l<i>.mix.q", ..., "final.norm", "head"); they are handed over as the file's own bytes -- the engine builds
its images (fused projections, fp32 copies for dtype float32) on the device.  No torch in this module: a command-line tool that
only replays tokens starts in a fraction of a second.
"""
from __future__ import annotations

import ctypes as C
import json
import mmap
import os
import struct
from dataclasses import dataclass, field
from typing import Sequence

import numpy as np

from .. import _ffi
from .engine import Engine

MIXER_ATTENTION, MIXER_LATENT, MIXER_LIGHTNING, MIXER_DELTA, MIXER_PARALLEL = 1, 2, 3, 4, 5
MLP_NONE, MLP_DENSE, MLP_GATED, MLP_MOE = 0, 1, 2, 3
ACT_RELU2, ACT_GELU_TANH, ACT_SILU, ACT_XIELU = 0, 1, 2, 3
DTYPES = {'bfloat16': 0, 'bf16': 0, 'float32': 1, 'f32': 1}


@dataclass
class LayerSpec:
    mixer: int = MIXER_ATTENTION
    weights_of: int = -1
    heads: int = 1
    kv_heads: int = 1
    dim: int = 64
    vdim: int = 64
    scale: float = 1.0
    softcap: float = 0.0          # <= 0: scores are not capped
    qtemp_coef: float = 0.0       # 0: no query temperature
    qtemp_every: float = 1.0
    sink: bool = False
    mlp: int = MLP_NONE
    ff: int = 0
    act: int = ACT_RELU2
    one_norm: bool = False        # both sublayers read norm1(x)
    resid_gate: bool = False      # each sublayer's result times sigmoid(rg_i h + b_i)
    loop_pass: int = -1           # >= 0: this layer run opens that pass of the loop
    qk_unit_norm: bool = False    # queries and keys scaled to unit RMS per head
    v_unit_norm: bool = False
    dist_bias: bool = False       # score -= r1 * ln(1 + r2 * distance)
    out_gate: bool = False        # a sigmoid gate per head on the attention output
    chunk: int = 0                # > 0: keys are visible inside the query's chunk of positions only
    kv_rank: int = 0              # latent attention: size of the cached latent vector
    rot_dim: int = 0              # ... and of the rotated query / key part
    rot_base: float = 10000.0
    experts: int = 0
    top: int = 0
    rot_dims: int = 0             # how many channels of the rotated part turn (0: all of them)
    post_norm: bool = False       # x += LN(sublayer(x)): the sublayers read the stream, a layer norm with bias follows them
    qkv_bias: bool = False
    qk_norm_w: bool = False       # per-head RMS norm of queries and keys with a weight of size dim
    rot_scale: float = 1.0        # divides every rotation frequency
    window: int = 0               # > 0: position i sees j only if i - j < window or j < keep_first
    keep_first: int = 0
    decay: tuple = ()             # lightning: one decay per head
    decay_rank: int = 0           # delta rule: inner size of the decay's two-matrix projection
    expert_plain: bool = False    # experts down(act(up x)) instead of gated ones
    router_softmax: bool = False  # soft-max scores weight the experts' outputs (times router_scale)
    router_scale: float = 1.0
    shared_ff: int = 0            # > 0: an expert of this size runs for every token
    norm_groups: int = 0          # > 0 (post_norm blocks): the norm behind a sublayer is an RMS norm in that many groups, no bias
    conv_taps: int = 0            # > 0: q, k, v pass a short causal convolution over time
    diff_maps: bool = False       # differential attention: two score maps per head over the same values
    diff_init: float = 0.0
    rot_pairs: bool = False       # the rotation pairs channel 2i with 2i + 1
    yarn_factor: float = 0.0      # > 0: slow rotation frequencies are divided by it (ramp between yarn_fast and yarn_slow turns over
    yarn_original: float = 0.0    # yarn_original positions), cos and sin times 0.1 ln(factor) + 1
    yarn_fast: float = 0.0
    yarn_slow: float = 0.0
    dist_buckets: int = 0         # parallel, left mixer: rows of the distance-bias table
    dist_max: float = 0.0         # ... and the distance at which its logarithmic buckets end
    r_heads: int = 0              # parallel, right mixer (gated delta rule): sizes
    r_kv_heads: int = 0
    r_dim: int = 0
    r_vdim: int = 0
    r_conv: int = 0
    a_rank: int = 0               # inner sizes of the decay's and the gate's two-matrix projections
    g_rank: int = 0


@dataclass
class LayeredConfig:
    arch: str
    width: int
    vocab: int
    layers: list = field(default_factory=list)
    norm_eps: float = 1e-5
    norm_offset: float = 0.0      # weights stored around zero: 1.0
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    eos_token_id: int | None = None
    max_position_embeddings: int = 8192
    loop_times: int = 0           # > 0: tensors loop.in / loop.step exist
    final_layer_norm: bool = False  # the last norm is a layer norm with bias
    embed_scale: float = 1.0      # multiplies the embedding output
    logit_softcap: float = 0.0    # > 0: logits <- cap * tanh(logits / cap)
    norm_groups: int = 0          # > 0: the last norm is an RMS norm in that many groups
    names: list = field(default_factory=list)   # tensor prefix of every layer run with tensors of its own ('' -> 'l<index>.')

    def native(self, dtype: str):
        """(tm_layered_config, keep-alive array)"""
        keep = []

        def decays(s):
            if not s.decay:
                return None
            keep.append((C.c_float * len(s.decay))(*s.decay))
            return keep[-1]

        arr = (_ffi.LayerSpec * len(self.layers))(*[
            _ffi.LayerSpec(s.mixer, s.weights_of, s.heads, s.kv_heads, s.dim, s.vdim, s.scale, s.softcap, s.qtemp_coef, s.qtemp_every,
                           int(s.sink), s.mlp, s.ff, s.act, int(s.one_norm), int(s.resid_gate), s.loop_pass, int(s.qk_unit_norm),
                           int(s.v_unit_norm), int(s.dist_bias), int(s.out_gate), s.chunk, s.kv_rank, s.rot_dim, s.rot_base, s.experts, s.top, s.rot_dims,
                           int(s.post_norm), int(s.qkv_bias), int(s.qk_norm_w), s.rot_scale, s.window, s.keep_first, decays(s), s.decay_rank,
                           int(s.expert_plain), int(s.router_softmax), s.router_scale, s.shared_ff,
                           s.norm_groups, s.conv_taps, int(s.diff_maps), s.diff_init, int(s.rot_pairs), s.yarn_factor, s.yarn_original, s.yarn_fast,
                           s.yarn_slow, s.dist_buckets, s.dist_max, s.r_heads, s.r_kv_heads, s.r_dim, s.r_vdim, s.r_conv, s.a_rank, s.g_rank)
            for s in self.layers])
        return _ffi.LayeredConfig(self.width, self.vocab, len(self.layers), arr, self.norm_eps, self.norm_offset, self.residual_mult,
                                  self.logit_scale, DTYPES[dtype], self.loop_times, int(self.final_layer_norm), self.embed_scale,
                                  self.logit_softcap, self.norm_groups), (arr, keep)

    def tensor_name(self, run: int, leaf: str) -> str:
        """checkpoint name of tensor `leaf` of layer run `run` (the engine's slots count layer RUNS; a looped model's file counts layers)"""
        return (self.names[run] if self.names else f'l{run}.') + leaf

    def tensor_shapes(self) -> dict:
        """{tensor name: shape} a checkpoint of this config holds"""
        W, out = self.width, {'embed': (self.vocab, self.width), 'final.norm': (self.width,), 'head': (self.vocab, self.width)}
        if self.final_layer_norm and not self.norm_groups:
            out['final.norm.b'] = (W,)
        if self.loop_times > 0:
            out['loop.in'], out['loop.step'] = (W, 2 * W), (self.loop_times, W)
        for i, s in enumerate(self.layers):
            if s.weights_of >= 0:
                continue
            p = f'l{i}.'
            out[p + 'norm1'] = (W,)
            if s.post_norm and s.norm_groups:
                out.update(_group_shapes(p, s, W))
                continue
            if s.post_norm:
                out.update(_post_shapes(p, s, W))
                continue
            if s.mixer == MIXER_LATENT or s.one_norm:
                out.update(_wide_shapes(p, s, W))
                continue
            out[p + 'mix.q'], out[p + 'mix.k'] = (s.heads * s.dim, W), (s.kv_heads * s.dim, W)
            out[p + 'mix.v'], out[p + 'mix.o'] = (s.kv_heads * s.vdim, W), (W, s.heads * s.vdim)
            if s.sink:
                out[p + 'mix.sink'] = (s.heads,)
            if s.mlp:
                out[p + 'norm2'], out[p + 'mlp.up'], out[p + 'mlp.down'] = (W,), (s.ff, W), (W, s.ff)
        return out


def _wide_shapes(p: str, s: LayerSpec, W: int) -> dict:
    """tensors of a block with one norm: the mixer's, the residual gates', the feed-forward's"""
    out = {p + 'mix.o': (W, s.heads * s.vdim)}
    if s.mixer == MIXER_LATENT:
        out[p + 'mix.q'] = (s.heads * (s.dim + s.rot_dim), W)
        out[p + 'mix.dkv'], out[p + 'mix.dkv.norm'] = (s.kv_rank + s.rot_dim, W), (s.kv_rank,)
        out[p + 'mix.uk'], out[p + 'mix.uv'] = (s.heads * s.dim, s.kv_rank), (s.heads * s.vdim, s.kv_rank)
    else:
        out[p + 'mix.q'], out[p + 'mix.k'], out[p + 'mix.v'] = (s.heads * s.dim, W), (s.kv_heads * s.dim, W), (s.kv_heads * s.vdim, W)
        if s.out_gate:
            out[p + 'mix.g'] = (s.heads, W)
    if s.dist_bias:
        out[p + 'mix.r1'], out[p + 'mix.r2'] = (s.heads,), (s.heads,)
    if s.sink:
        out[p + 'mix.sink'] = (s.heads,)
    if s.resid_gate:
        out[p + 'rg1'], out[p + 'rg1.b'] = (W, W), (W,)
        if s.mlp:
            out[p + 'rg2'], out[p + 'rg2.b'] = (W, W), (W,)
    if s.mlp == MLP_GATED:
        out[p + 'mlp.gate'], out[p + 'mlp.up'], out[p + 'mlp.down'] = (s.ff, W), (s.ff, W), (W, s.ff)
    elif s.mlp == MLP_MOE:
        out[p + 'mlp.router'] = (s.experts, W)
        for e in range(s.experts):
            out[p + f'mlp.e{e}.gate'], out[p + f'mlp.e{e}.up'], out[p + f'mlp.e{e}.down'] = (s.ff, W), (s.ff, W), (W, s.ff)
    return out


def _post_shapes(p: str, s: LayerSpec, W: int) -> dict:
    """tensors of a block whose sublayers read the stream and are followed by a layer norm with bias"""
    H, d, dv = s.heads, s.dim, s.vdim
    out = {p + 'norm1.b': (W,), p + 'mix.o': (W, H * dv)}
    if s.mixer == MIXER_ATTENTION:
        out[p + 'mix.q'], out[p + 'mix.k'], out[p + 'mix.v'] = (H * d, W), (s.kv_heads * d, W), (s.kv_heads * dv, W)
        if s.qkv_bias:
            out[p + 'mix.q.b'], out[p + 'mix.k.b'], out[p + 'mix.v.b'] = (H * d,), (s.kv_heads * d,), (s.kv_heads * dv,)
        if s.qk_norm_w:
            out[p + 'mix.q.norm'], out[p + 'mix.k.norm'] = (d,), (d,)
    elif s.mixer == MIXER_LIGHTNING:
        out[p + 'mix.q'], out[p + 'mix.k'], out[p + 'mix.v'], out[p + 'mix.g'] = (H * d, W), (H * d, W), (H * dv, W), (H * dv, W)
        out[p + 'mix.norm'] = (H * dv,)
    elif s.mixer == MIXER_DELTA:
        for t in 'rkvga':
            out[p + 'mix.' + t] = (H * d, W)
        out[p + 'mix.a.b'], out[p + 'mix.w0'], out[p + 'mix.norm'] = (H * d,), (H * d,), (H * d,)
        out[p + 'mix.w1'], out[p + 'mix.w2'] = (s.decay_rank, W), (H * d, s.decay_rank)
    else:
        raise NotImplementedError(f'{p}: mixer {s.mixer} in a post-norm block')
    if s.mlp:
        out[p + 'norm2'], out[p + 'norm2.b'] = (W,), (W,)
    if s.mlp == MLP_DENSE:
        out[p + 'mlp.up'], out[p + 'mlp.down'] = (s.ff, W), (W, s.ff)
        if s.act == ACT_XIELU:
            out[p + 'mlp.act'] = (2,)
    elif s.mlp == MLP_MOE:
        out[p + 'mlp.router'] = (s.experts, W)
        for e in range(s.experts):
            out[p + f'mlp.e{e}.up'], out[p + f'mlp.e{e}.down'] = (s.ff, W), (W, s.ff)
        if s.shared_ff:
            out[p + 'mlp.shared.up'], out[p + 'mlp.shared.down'] = (s.shared_ff, W), (W, s.shared_ff)
    return out


def _group_shapes(p: str, s: LayerSpec, W: int) -> dict:
    """tensors of a post-norm block with RMS group norms: differential attention with convolved projections, or the parallel pair of a
    biased attention and a gated delta rule; gated feed-forward"""
    H, G, d, dv = s.heads, s.kv_heads, s.dim, s.vdim
    out = {}
    if s.mixer == MIXER_ATTENTION:
        maps = 2 if s.diff_maps else 1
        for t, n in (('q', H * maps * d), ('k', G * maps * d), ('v', G * dv)):
            out[p + 'mix.' + t] = (n, W)
            if s.conv_taps:
                out[p + f'mix.{t}.conv'] = (n, s.conv_taps)
        if s.qk_norm_w:
            out[p + 'mix.q.norm'], out[p + 'mix.k.norm'] = (d,), (d,)
        if s.diff_maps:
            for t in ('lq1', 'lk1', 'lq2', 'lk2'):
                out[p + 'mix.' + t] = (d,)
        out[p + 'mix.o'] = (W, H * dv)
    elif s.mixer == MIXER_PARALLEL:
        a, b = p + 'mix.left.', p + 'mix.right.'
        out.update({a + 'q': (H * d, W), a + 'k': (G * d, W), a + 'q.norm': (H * d,), a + 'k.norm': (G * d,), a + 'rel': (s.dist_buckets, H),
                    a + 'talk': (H, H), a + 'g': (H * dv, W), a + 'o': (W, H * dv), a + 'out': (W,), b + 'out': (W,)})
        Hr, Gr, dr, dvr = s.r_heads, s.r_kv_heads, s.r_dim, s.r_vdim
        for t, n in (('q', Gr * dr), ('k', Gr * dr), ('v', Hr * dvr)):
            out[b + t], out[b + t + '.conv'] = (n, W), (n, s.r_conv)
        out.update({b + 'b': (Hr, W), b + 'A_log': (Hr,), b + 'norm': (dvr,), b + 'a1': (s.a_rank, W), b + 'a2': (Hr * dr, s.a_rank),
                    b + 'dt_bias': (Hr * dr,), b + 'g1': (s.g_rank, W), b + 'g2': (Hr * dvr, s.g_rank), b + 'o': (W, Hr * dvr)})
    else:
        raise NotImplementedError(f'{p}: mixer {s.mixer} in a block with group norms')
    if s.mlp:
        out[p + 'norm2'] = (W,)
        out[p + 'mlp.gate'], out[p + 'mlp.up'], out[p + 'mlp.down'] = (s.ff, W), (s.ff, W), (W, s.ff)
    return out


def _mededra_layer(i: int, L: dict, shapes: dict, groups: int) -> LayerSpec:
    m, mlp, kind = L['mixer'], L.get('mlp'), L['type']
    s = LayerSpec(post_norm=True, norm_groups=groups)
    if kind == 'attention':
        s.mixer, s.heads, s.dim = MIXER_ATTENTION, int(m['heads']), int(m['dim'])
        s.kv_heads, s.vdim = int(m.get('kv_heads', s.heads)), int(m.get('vdim', s.dim))
        s.scale = float(m['scale']) if 'scale' in m else s.dim ** -0.5
        s.softcap = float(m.get('softcap') or 0.0)
        s.qk_norm_w, s.diff_maps, s.diff_init = True, True, float(m['diff'])
        s.conv_taps = int(m.get('conv') or 0)
        s.window = int((m.get('mask') or {}).get('size') or 0)
        rot = m.get('rot') or {}
        if rot:
            s.rot_pairs, s.rot_dims, s.rot_base = True, int(rot.get('dims', s.dim)), float(rot['base'])
            sc = rot.get('scaling') or {}
            if sc:
                s.yarn_factor, s.yarn_original = float(sc['factor']), float(sc['original'])
                s.yarn_fast, s.yarn_slow = float(sc['fast']), float(sc['slow'])
            if s.rot_dims % 2 or not 0 <= s.rot_dims <= s.dim:
                raise ValueError(f'layer {i}: rot.dims must be even and at most dim')
    elif kind == 'parallel':
        a, b = m['left'], m['right']
        s.mixer, s.heads, s.dim = MIXER_PARALLEL, int(a['heads']), int(a['dim'])
        s.kv_heads, s.vdim = int(a.get('kv_heads', s.heads)), int(a.get('vdim', s.dim))
        s.scale = float(a['scale']) if 'scale' in a else s.dim ** -0.5
        s.window = int((a.get('mask') or {}).get('size') or 0)
        s.dist_max = float(a['bias_max'])
        rel = shapes.get(f'l{i}.mix.left.rel')          # the number of buckets, and the inner sizes below, are the tensors' own
        s.dist_buckets = int(rel[0]) if rel else int(a.get('buckets', 0))
        if s.vdim != s.dim:
            raise ValueError(f'layer {i}: the left mixer\'s values are its keys: vdim = dim')
        s.r_heads, s.r_dim = int(b['heads']), int(b['dim'])
        s.r_kv_heads, s.r_vdim, s.r_conv = int(b.get('kv_heads', s.r_heads)), int(b.get('vdim', s.r_dim)), int(b.get('conv') or 1)
        a1, g1 = shapes.get(f'l{i}.mix.right.a1'), shapes.get(f'l{i}.mix.right.g1')
        s.a_rank = int(a1[0]) if a1 else int(b.get('a_rank', 0))
        s.g_rank = int(g1[0]) if g1 else int(b.get('g_rank', 0))
    else:
        raise NotImplementedError(f'layer {i}: mixer {kind!r}')
    if mlp is None:
        return s
    if mlp.get('kind') != 'dense':
        raise NotImplementedError(f'layer {i}: feed-forward kind {mlp.get("kind")!r}')
    s.mlp, s.ff, s.act = MLP_GATED, int(mlp['ff']), ACT_SILU
    return s


def _mededra(c: dict, shapes: dict | None = None) -> LayeredConfig:
    """Mededra: blocks x += GN1(mixer(x)); x += GN2(ff(x)) with RMS norms in groups on the sublayers' results.  Mixers: differential
    attention (two score maps per head, q / k / v through a short causal convolution, a weighted norm per map, pairwise rotation with
    scaled frequencies, capped scores, a sliding window), or a parallel pair -- windowed attention whose values are its keys, with a
    bucketed distance bias, scores mixed between heads, one added to the soft-max denominator and a gated output, beside a gated delta
    rule -- whose normed results are averaged.  Gated silu feed-forward, scaled embedding, capped logits.  `shapes` ({tensor name: shape}
    of the checkpoint) settles the sizes the config leaves to the tensors (distance buckets, inner sizes of two-matrix projections)."""
    groups = int(c['norm'].get('groups', 1))
    layers = [_mededra_layer(i, L, shapes or {}, groups) for i, L in enumerate(c['layers'])]
    return LayeredConfig(arch='Mededra', width=int(c['width']), vocab=int(c['vocab']), layers=layers, norm_eps=float(c['norm']['eps']),
                         norm_offset=0.0, residual_mult=1.0, logit_scale=1.0, eos_token_id=c.get('eos_token_id'),
                         embed_scale=float((c.get('embedding') or {}).get('scale', 1.0)), logit_softcap=float(c.get('logit_softcap') or 0.0),
                         norm_groups=groups)


def _febivik_layer(i: int, L: dict, shapes: dict) -> LayerSpec:
    m, mlp, kind = L['mixer'], L.get('mlp'), L['type']
    s = LayerSpec(heads=int(m['heads']), dim=int(m['dim']), post_norm=True)
    if kind == 'attention':
        s.mixer, s.kv_heads, s.vdim = MIXER_ATTENTION, int(m.get('kv_heads', s.heads)), int(m.get('vdim', s.dim))
        s.scale = float(m['scale']) if 'scale' in m else s.dim ** -0.5
        s.qkv_bias = s.qk_norm_w = True
        rot, mask = m.get('rot') or {}, m.get('mask') or {}
        s.rot_dims, s.rot_base = int(rot.get('dims', s.dim)) if rot else 0, float(rot.get('base', 10000.0))      # (a rotation without 'dims' turns the whole head)
        s.rot_scale = float((rot.get('scaling') or {}).get('factor', 1.0))
        s.window, s.keep_first = int(mask.get('size', 0)), int(mask.get('keep_first', 0))
        if s.rot_dims % 2 or not 0 <= s.rot_dims <= s.dim or s.rot_scale <= 0:
            raise ValueError(f'layer {i}: rot.dims must be even and at most dim, the scaling factor positive')
    elif kind == 'lightning':
        s.mixer, s.kv_heads, s.vdim = MIXER_LIGHTNING, s.heads, int(m.get('vdim', s.dim))
        d = m['decay']
        s.decay = tuple(float(v) for v in d) if isinstance(d, (list, tuple)) else (float(d),) * s.heads
        if len(s.decay) != s.heads:
            raise ValueError(f'layer {i}: one decay per head')
    elif kind == 'general_delta':
        s.mixer, s.kv_heads, s.vdim = MIXER_DELTA, s.heads, s.dim
        w1 = shapes.get(f'l{i}.mix.w1')     # the inner size of the decay projection is the tensor's own
        s.decay_rank = int(w1[0]) if w1 else int(m.get('decay_rank', 0) or max(1, min(64, s.dim // 2)))
    else:
        raise NotImplementedError(f'layer {i}: mixer {kind!r}')
    if mlp is None:
        return s
    if mlp.get('kind') == 'dense':
        s.mlp, s.ff, s.act = MLP_DENSE, int(mlp['ff']), ACT_XIELU
    elif mlp.get('kind') == 'moe':
        r = mlp['router']
        s.mlp, s.ff, s.act, s.expert_plain, s.router_softmax = MLP_MOE, int(mlp['expert']['ff']), ACT_RELU2, True, True
        s.experts, s.top, s.router_scale = int(r['experts']), int(r['top']), float(r.get('scale', 1.0))
        s.shared_ff = int((mlp.get('shared') or {}).get('ff', 0))
    else:
        raise NotImplementedError(f'layer {i}: feed-forward kind {mlp.get("kind")!r}')
    return s


def _febivik(c: dict, shapes: dict | None = None) -> LayeredConfig:
    """Febivik: blocks x += LN1(mixer(x)); x += LN2(ff(x)) -- the sublayers read the stream itself and a layer norm with bias follows
    them.  Mixers: lightning (linear attention, one decay per head, a state per head), grouped-query soft-max attention with biases,
    weighted per-head query / key norms, partial rotation with scaled frequencies and a sliding window that keeps the first tokens, and a
    generalized delta rule (decay and removal rate per key channel).  Feed-forwards: dense with the xIELU activation, or soft-max-routed
    squared-ReLU experts plus a shared expert.  `shapes` ({tensor name: shape} of the checkpoint) settles sizes the config leaves to the
    tensors."""
    layers = [_febivik_layer(i, L, shapes or {}) for i, L in enumerate(c['layers'])]
    return LayeredConfig(arch='Febivik', width=int(c['width']), vocab=int(c['vocab']), layers=layers, norm_eps=float(c['norm']['eps']),
                         norm_offset=0.0, residual_mult=1.0, logit_scale=1.0, eos_token_id=c.get('eos_token_id'), final_layer_norm=True)


def _bedenex_layer(i: int, L: dict) -> LayerSpec:
    m, mlp = L['mixer'], L.get('mlp')
    s = LayerSpec(heads=int(m['heads']), dim=int(m['dim']), vdim=int(m['vdim']), scale=float(m['scale']), one_norm=True, resid_gate=True)
    if L['type'] == 'attention':
        s.mixer, s.kv_heads = MIXER_ATTENTION, int(m['kv_heads'])
        s.qk_unit_norm = s.v_unit_norm = s.dist_bias = s.out_gate = True
        s.chunk = int((m.get('mask') or {}).get('size') or 0)
    elif L['type'] == 'latent_attention':
        s.mixer, s.kv_heads, s.sink = MIXER_LATENT, 1, True
        s.kv_rank, s.rot_dim, s.rot_base = int(m['kv_rank']), int(m['rot_dim']), float(m['rot']['base'])
        s.rot_dims = int(m['rot'].get('dims', s.rot_dim))
        if not 0 <= s.rot_dims <= s.rot_dim or s.rot_dims % 2:
            raise ValueError(f'layer {i}: rot.dims must be even and at most rot_dim')
    else:
        raise NotImplementedError(f'layer {i}: mixer {L["type"]!r}')
    if mlp is None:
        return s
    if mlp.get('kind') == 'dense':
        s.mlp, s.ff, s.act = MLP_GATED, int(mlp['ff']), ACT_GELU_TANH
    elif mlp.get('kind') == 'moe':
        s.mlp, s.ff, s.act = MLP_MOE, int(mlp['expert']['ff']), ACT_SILU
        s.experts, s.top = int(mlp['router']['experts']), int(mlp['router']['top'])
    else:
        raise NotImplementedError(f'layer {i}: feed-forward kind {mlp.get("kind")!r}')
    return s


def _bedenex(c: dict) -> LayeredConfig:
    """Bedenex: blocks x += sigmoid(rg1 h + b1) * mixer(h) + sigmoid(rg2 h + b2) * ff(h) with ONE norm h of the stream.  Mixers: grouped-query
    attention without rotation (unit-RMS queries, keys and values per head, a logarithmic distance penalty, keys visible inside the
    query's chunk of positions, a sigmoid gate per head on the output) and latent attention (one normed latent vector and one rotated key
    part cached per token, a sink logit per head).  Feed-forwards: gated GELU, or a sigmoid-routed mixture of gated SiLU experts whose
    scores scale the experts' inputs.  A range of layers may run several times in a row on the same weights (every run has its own cache);
    each pass starts from loop.in [x | embedding output] + loop.step[pass]."""
    import copy
    own = [_bedenex_layer(i, L) for i, L in enumerate(c['layers'])]
    loop = c.get('loop') or {}
    start, stop, times = int(loop.get('start', 0)), int(loop.get('stop', 0)), int(loop.get('times', 0))
    if stop <= start or times < 1:
        start = stop = times = 0
    runs, names = [], []
    first_run = {}      # layer -> its first run (the one that owns the tensors)
    order = list(range(start)) + [i for _ in range(times) for i in range(start, stop)] + list(range(stop, len(own)))
    seen_pass = 0
    for i in order:
        s = copy.copy(own[i])
        if times and i == start:
            s.loop_pass, seen_pass = seen_pass, seen_pass + 1
        if i in first_run:
            s.weights_of = first_run[i]
        else:
            first_run[i] = len(runs)
        runs.append(s)
        names.append(f'l{i}.')
    return LayeredConfig(arch='Bedenex', width=int(c['width']), vocab=int(c['vocab']), layers=runs, norm_eps=float(c['norm']['eps']),
                         norm_offset=0.0, residual_mult=1.0, logit_scale=1.0, eos_token_id=c.get('eos_token_id'), loop_times=times,
                         names=names)


def _fokonex(c: dict) -> LayeredConfig:
    """Fokonex: parallel residual blocks with two norms of the same input (weights stored around zero), attention without rotation --
    positions enter through a logarithmic query temperature -- with capped scores and a per-head sink logit, squared-ReLU
    feed-forward, scaled logits.  Layers may run on an earlier layer's weights."""
    layers = []
    for i, L in enumerate(c['layers']):
        if L['type'] != 'attention':
            raise NotImplementedError(f'layer {i}: mixer {L["type"]!r}')
        m, mlp = L['mixer'], L.get('mlp')
        if mlp is not None and mlp.get('kind') != 'dense':
            raise NotImplementedError(f'layer {i}: feed-forward kind {mlp.get("kind")!r}')
        qt = m.get('q_temp') or {}
        layers.append(LayerSpec(mixer=MIXER_ATTENTION, weights_of=int(L.get('weights_of', -1)), heads=int(m['heads']),
                                kv_heads=int(m['kv_heads']), dim=int(m['dim']), vdim=int(m['vdim']), scale=float(m['scale']),
                                softcap=float(m.get('softcap') or 0.0), qtemp_coef=float(qt.get('coef') or 0.0),
                                qtemp_every=float(qt.get('every') or 1.0), sink=True, mlp=MLP_DENSE if mlp is not None else MLP_NONE,
                                ff=int(mlp['ff']) if mlp is not None else 0, act=ACT_RELU2))
    for s in layers:        # a layer may name a layer that itself runs on another's weights: the tensors are the root's
        seen = set()
        while s.weights_of >= 0 and layers[s.weights_of].weights_of >= 0 and s.weights_of not in seen:
            seen.add(s.weights_of)
            s.weights_of = layers[s.weights_of].weights_of
    return LayeredConfig(arch='Fokonex', width=int(c['width']), vocab=int(c['vocab']), layers=layers,
                         norm_eps=float(c['norm']['eps']), norm_offset=1.0, residual_mult=float(c['residual_mult']),
                         logit_scale=float(c['logit_scale']), eos_token_id=c.get('eos_token_id'))


FAMILIES = {'Fokonex': _fokonex, 'Bedenex': _bedenex, 'Febivik': _febivik, 'Mededra': _mededra}
NEEDS_SHAPES = {'Febivik', 'Mededra'}     # readers that take the checkpoint's tensor shapes as a second argument


def is_layered(model_path: str) -> bool:
    try:
        with open(os.path.join(model_path, 'config.json')) as f:
            return json.load(f).get('architecture') in FAMILIES
    except (OSError, ValueError):
        return False


def read_layered_config(model_path: str) -> LayeredConfig:
    with open(os.path.join(model_path, 'config.json')) as f:
        c = json.load(f)
    arch = c.get('architecture')
    if arch not in FAMILIES:
        raise NotImplementedError(f'architecture {arch!r}: known layer-list families are {sorted(FAMILIES)}')
    if arch in NEEDS_SHAPES:
        st = os.path.join(model_path, 'model.safetensors')
        return FAMILIES[arch](c, safetensors_shapes(st) if os.path.exists(st) else {})
    return FAMILIES[arch](c)


def safetensors_shapes(path: str) -> dict:
    """{name: shape} from the header of a safetensors file"""
    with open(path, 'rb') as f:
        n, = struct.unpack('<Q', f.read(8))
        header = json.loads(f.read(n).decode('utf-8'))
    return {k: tuple(v['shape']) for k, v in header.items() if k != '__metadata__'}


def read_safetensors(path: str) -> dict:
    """{name: (dtype string, shape, bytes view)} of one safetensors file: 8-byte little-endian header length, JSON header
    (name -> dtype, shape, data_offsets), then the data.  The views point into a read-only mapping of the file."""
    f = open(path, 'rb')
    mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
    n, = struct.unpack('<Q', mm[:8])
    header = json.loads(mm[8:8 + n].decode('utf-8'))
    view = memoryview(mm)
    out = {}
    for name, t in header.items():
        if name == '__metadata__':
            continue
        lo, hi = t['data_offsets']
        out[name] = (t['dtype'], tuple(t['shape']), view[8 + n + lo:8 + n + hi])
    return out


class LayeredEngine(Engine):
    """The native engine running a layer-list model.  Static batch, continuous batching, sampling and the engine thread are the
    base class's; this adds the checkpoint hand-off and the sessions (caller-fed tokens -> logits)."""

    def __init__(self, model: LayeredConfig, *, dtype: str = 'bfloat16', device: int = 0, max_batch_size: int = 64,
                 session_len: int = 2048, cache_max_entry_count: float = 0.8, cache_blocks: int = 0,
                 max_prefill_token_num: int = 8192, use_graph: int = 1):
        self._lib = _ffi.load()
        self.model = model
        self.dtype = dtype
        self.cfg = _ffi.EngineConfig(_ffi.ModelConfig(), 1, 0, device, max_batch_size, session_len, 0, 64, cache_max_entry_count,
                                     cache_blocks, max_prefill_token_num, 0, use_graph)
        self.cfg.model.vocab, self.cfg.model.hidden, self.cfg.model.layers = model.vocab, model.width, len(model.layers)
        native, self._keep = model.native(dtype)
        self._h = C.c_void_p()
        _ffi.check(self._lib.tm_engine_create_layered(C.byref(self._h), C.byref(self.cfg), C.byref(native)))
        self.batch = 0
        self.max_new = 0

    def load_checkpoint(self, model_path: str):
        tensors = read_safetensors(os.path.join(model_path, 'model.safetensors'))
        for name, shape in self.model.tensor_shapes().items():
            slot = name
            if self.model.names and name[0] == 'l' and name[1].isdigit():   # the engine's slot counts layer runs, the file counts layers
                run, leaf = name[1:].split('.', 1)
                name = self.model.tensor_name(int(run), leaf)
            if name not in tensors:
                raise KeyError(f'{model_path}: tensor {name} is missing')
            dt, shp, data = tensors[name]
            if dt != 'BF16' or tuple(shp) != tuple(shape):
                raise ValueError(f'{name}: {dt} {shp} in the file, the config says BF16 {shape}')
            name = slot
            buf = np.frombuffer(data, np.uint8)
            _ffi.check(self._lib.tm_engine_weight_copy(self._h, name.encode(), buf.ctypes.data, buf.nbytes))
        _ffi.check(self._lib.tm_engine_process_weights(self._h))

    def load_weights(self, slots: dict):
        """slots: {tensor name: uint16 array holding bf16 bits}"""
        for name, arr in slots.items():
            arr = np.ascontiguousarray(arr)
            _ffi.check(self._lib.tm_engine_weight_copy(self._h, name.encode(), arr.ctypes.data, arr.nbytes))
        _ffi.check(self._lib.tm_engine_process_weights(self._h))

    # ---- sessions ---------------------------------------------------------------------------------
    def open_session(self) -> int:
        sid = C.c_int64(0)
        _ffi.check(self._lib.tm_engine_session_open(self._h, C.byref(sid)))
        return sid.value

    def close_session(self, session: int):
        _ffi.check(self._lib.tm_engine_session_close(self._h, session))

    def step_tokens(self, entries: Sequence) -> np.ndarray:
        """entries: (session, tokens, want) triples -- ONE forward over the next tokens of these sessions; returns the fp32 logits of
        the wanted places (indices into an entry's tokens), in entry order: [sum(len(want)), vocab]."""
        keep, arr = [], (_ffi.StepEntry * len(entries))()
        n_want = 0
        for i, (sid, toks, want) in enumerate(entries):
            t = np.ascontiguousarray(np.asarray(toks, np.int32))
            w = np.ascontiguousarray(np.asarray(want if want is not None else [], np.int32))
            keep += [t, w]
            arr[i] = _ffi.StepEntry(int(sid), t.ctypes.data, int(t.size), w.ctypes.data if w.size else None, int(w.size))
            n_want += int(w.size)
        out = np.zeros((n_want, self.model.vocab), np.float32)
        _ffi.check(self._lib.tm_engine_step_tokens(self._h, arr, len(entries), out.ctypes.data if n_want else None))
        return out

    def stop_after(self, layers: int):
        """parity tests: the next forwards stop behind `layers` layers (< 0: all)"""
        _ffi.check(self._lib.tm_engine_debug_stop_after(self._h, int(layers)))

    def fetch_residual(self, rows: int) -> np.ndarray:
        """the fp32 residual stream of the last forward, [rows][width]"""
        out = np.zeros((rows, self.model.width), np.float32)
        _ffi.check(self._lib.tm_engine_debug_read(self._h, 0, rows, 0, out.ctypes.data, out.nbytes))
        return out

    def fetch_logits(self) -> np.ndarray:
        ld = (self.model.vocab + 7) // 8 * 8
        out = np.zeros((self.batch, ld), np.float16)
        _ffi.check(self._lib.tm_engine_fetch_logits(self._h, out.ctypes.data))
        return out[:, :self.model.vocab]


def build_engine(model_path: str, *, dtype: str = 'bfloat16', **kw) -> LayeredEngine:
    """config.json + model.safetensors of a layer-list model -> a started engine"""
    eng = LayeredEngine(read_layered_config(model_path), dtype=dtype, **kw)
    eng.load_checkpoint(model_path)
    eng.start()
    return eng
