"""`bench.py --layered`: prefill and decode throughput of a layer-list model (Fokonex blocks, bf16) at layer shapes of real decoders,
beside the closest model the engine already serves -- a Llama-family decoder with fp16 weights and fp16 KV -- at EQUAL size: same width,
heads, head size 128, layer count and vocabulary, and a feed-forward of the same parameter count (two matrices of 1.5 x the gated
feed-forward's three).  Random weights; both engines run their own static-batch entry points (chunked prefill, hipGraph decode).

Per kernel category of an eager decode step the table also gives the fraction of the HBM roofline (bytes the category must move /
8 TB/s / measured time) for both, and their ratio: the figure the two designs' like kernels are compared by.

`bench.py --layered --layered-design bedenex`: the same for Bedenex blocks (chunked attention with unit norms, distance penalty and output
gate; latent attention; gated residuals; gated-GELU and routed-expert feed-forwards; a looped range of layers) beside the closest
model the engine serves, the Fokonex blocks above, at equal width, heads, layer count, vocabulary and active feed-forward parameters.

`bench.py --layered --layered-design febivik`: Febivik blocks (lightning and delta-rule state mixers, windowed attention with kept first
tokens, xIELU and soft-max-routed squared-ReLU experts with a shared expert, layer norms behind the sublayers) beside the closest model
the engine serves -- the Bedenex blocks above (routed experts, fused fp32 projections) -- at equal width, heads, layer count, vocabulary
and active feed-forward parameters.

`bench.py --layered --layered-design mededra`: Mededra blocks (differential attention with convolved projections, the parallel pair of a
biased attention with mixed heads and a gated delta rule, RMS group norms behind the sublayers, gated silu feed-forward) beside the
closest model the engine serves -- the Febivik blocks above (post-norm blocks, windowed attention, a delta-rule state mixer) -- at equal
width, heads, layer count and vocabulary.
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


BEDENEX = dict(chunk=2048, latent_dim=64, rot_dim=64, kv_rank=192, experts=8, top=2)


def bedenex_config(s) -> dict:
    """config.json of the benchmark model: [attention + dense, attention + experts, latent + dense, latent + experts] repeated, the middle
    layers inside a loop that runs once.  Experts of half the dense size, two per token: the active parameters equal the dense block's"""
    b = BEDENEX
    att = {'heads': s['heads'], 'kv_heads': s['kv_heads'], 'dim': 128, 'vdim': 128, 'scale': 128 ** -0.5, 'mask': {'size': b['chunk']}}
    lat = {'heads': s['heads'], 'dim': b['latent_dim'], 'rot_dim': b['rot_dim'], 'vdim': 128, 'kv_rank': b['kv_rank'], 'scale': 128 ** -0.5,
           'rot': {'base': 10000.0, 'dims': b['rot_dim']}}
    dense = {'kind': 'dense', 'ff': s['inter']}
    moe = {'kind': 'moe', 'expert': {'ff': s['inter'] // 2}, 'router': {'experts': b['experts'], 'top': b['top']}}
    four = [{'type': 'attention', 'mixer': att, 'mlp': dense}, {'type': 'attention', 'mixer': att, 'mlp': moe},
            {'type': 'latent_attention', 'mixer': lat, 'mlp': dense}, {'type': 'latent_attention', 'mixer': lat, 'mlp': moe}]
    n = s['layers']
    return {'architecture': 'Bedenex', 'width': s['width'], 'vocab': s['vocab'], 'norm': {'eps': 1e-5},
            'layers': [four[i % 4] for i in range(n)], 'loop': {'start': n // 4, 'stop': n - n // 4, 'times': 1}}


def _bedenex_engine(s, batch, session_len, max_prefill):
    from . import layered
    cfg = layered.FAMILIES['Bedenex'](bedenex_config(s))
    eng = layered.LayeredEngine(cfg, dtype='bfloat16', max_batch_size=batch, session_len=session_len, max_prefill_token_num=max_prefill)
    eng.init_synthetic(seed=1)
    eng.start()
    return eng


def _bedenex_decode_bytes(s, batch, ctx):
    """bytes each category of ONE decode step must move: every weight that takes part once (all experts: batch x top pairs reach each of
    them), the cache entries a row sees once per sequence; activations are noise beside them"""
    b, W, H, G, I, V = BEDENEX, s['width'], s['heads'], s['kv_heads'], s['inter'], s['vocab']
    C, R, D = b['kv_rank'], b['rot_dim'], b['latent_dim']
    out = dict(gemm_qkv=0, attention=0, gemm_o=2 * W * 2 * W, gemm_gate_up=0, gemm_down=0, lm_head=2 * W * V)
    for i in range(s['layers']):
        latent, moe = i % 4 >= 2, i % 2 == 1
        n_proj = (H * (D + R) + C + R if latent else (H + 2 * G) * 128 + H) + 2 * W + (b['experts'] if moe else 0)
        out['gemm_qkv'] += 2 * W * n_proj + (2 * H * D * C if latent else 0)
        # the latent cache holds the latent vector twice: inside the key rows and, transposed, as the value rows
        out['attention'] += 2 * batch * ((C + R + C) * ctx if latent else 2 * G * 128 * min(ctx, b['chunk'] // 2 if ctx > b['chunk'] else ctx))
        out['gemm_o'] += 2 * W * H * 128 + (2 * H * 128 * C if latent else 0)
        ff = b['experts'] * (I // 2) if moe else I
        out['gemm_gate_up'] += 2 * W * 2 * ff
        out['gemm_down'] += 2 * W * ff
    return out


FEBIVIK = dict(window=2048, keep_first=4, rot_dims=64, decay_rank=64, experts=8, top=2)


def febivik_config(s) -> dict:
    """config.json of the benchmark model: [lightning + dense, attention + experts, lightning + experts, delta rule + experts] repeated.
    The dense feed-forward has two matrices of 1.5 x the gated size (equal parameters); experts and the shared expert have a third of
    it, two experts per token: the active parameters equal the dense block's"""
    b, H = FEBIVIK, s['heads']
    ff = s['inter'] * 3 // 2
    lig = {'heads': H, 'dim': 128, 'vdim': 128, 'decay': [1.0 - 2.0 ** -(5 + 5 * h / max(1, H - 1)) for h in range(H)]}
    att = {'heads': H, 'kv_heads': s['kv_heads'], 'dim': 128, 'vdim': 128, 'scale': 128 ** -0.5,
           'mask': {'size': b['window'], 'keep_first': b['keep_first']}, 'rot': {'base': 10000.0, 'dims': b['rot_dims'], 'scaling': {'factor': 4.0}}}
    dlt = {'heads': H, 'dim': 128, 'decay_rank': b['decay_rank']}
    dense = {'kind': 'dense', 'ff': ff}
    moe = {'kind': 'moe', 'expert': {'ff': ff // 3}, 'router': {'experts': b['experts'], 'top': b['top'], 'scale': 1.0}, 'shared': {'ff': ff // 3}}
    four = [{'type': 'lightning', 'mixer': lig, 'mlp': dense}, {'type': 'attention', 'mixer': att, 'mlp': moe},
            {'type': 'lightning', 'mixer': lig, 'mlp': moe}, {'type': 'general_delta', 'mixer': dlt, 'mlp': moe}]
    return {'architecture': 'Febivik', 'width': s['width'], 'vocab': s['vocab'], 'norm': {'eps': 1e-5},
            'layers': [four[i % 4] for i in range(s['layers'])]}


def _febivik_engine(s, batch, session_len, max_prefill):
    from . import layered
    cfg = layered.FAMILIES['Febivik'](febivik_config(s))
    eng = layered.LayeredEngine(cfg, dtype='bfloat16', max_batch_size=batch, session_len=session_len, max_prefill_token_num=max_prefill)
    eng.init_synthetic(seed=1)
    eng.start()
    return eng


def _febivik_decode_bytes(s, batch, ctx):
    """bytes each category of ONE decode step must move: every weight that takes part once (all experts), the cache entries inside the
    window once per sequence, and every recurrent state read and written once (fp32)"""
    b, W, H, G, V = FEBIVIK, s['width'], s['heads'], s['kv_heads'], s['vocab']
    ff = s['inter'] * 3 // 2
    out = dict(gemm_qkv=0, attention=0, gemm_o=0, gemm_gate_up=0, gemm_down=0, lm_head=2 * W * V)
    for i in range(s['layers']):
        kind, moe = ('lightning', 'attention', 'lightning', 'delta')[i % 4], i % 4 != 0
        if kind == 'attention':
            out['gemm_qkv'] += 2 * W * (H + 2 * G) * 128
            out['attention'] += 2 * batch * 2 * G * 128 * min(ctx, b['window'] + b['keep_first'])
        else:
            out['gemm_qkv'] += 2 * W * H * 128 * (4 if kind == 'lightning' else 5) + (2 * b['decay_rank'] * (W + H * 128) if kind == 'delta' else 0)
            out['attention'] += batch * H * 128 * 128 * 4 * 2
        out['gemm_o'] += 2 * W * H * 128
        n = (b['experts'] + 1) * (ff // 3) if moe else ff
        out['gemm_gate_up'] += 2 * W * n + (2 * W * b['experts'] if moe else 0)
        out['gemm_down'] += 2 * W * n
    return out


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


MEDEDRA = dict(window=2048, map_dim=64, rot_dims=64, conv=4, left_kv=2, buckets=32, bias_max=4096, rank=64)


def mededra_config(s) -> dict:
    """config.json of the benchmark model: [differential attention x 3, parallel pair] repeated, every block with the gated feed-forward of
    the size's own `inter`.  Differential attention: two maps of 64 channels per head (the projections are as wide as heads of 128), values
    of 128, window 2048, scaled pairwise rotation, 4-tap convolutions.  Parallel pair: left = windowed attention over 2 key heads of 128
    (a wide key of 256) with the bucketed distance bias and mixed heads; right = gated delta rule with heads of 128 x 128"""
    b, H, G = MEDEDRA, s['heads'], s['kv_heads']
    att = {'heads': H, 'kv_heads': G, 'dim': b['map_dim'], 'vdim': 128, 'scale': b['map_dim'] ** -0.5, 'softcap': 50.0, 'diff': 0.8, 'conv': b['conv'],
           'mask': {'size': b['window']},
           'rot': {'base': 1000000.0, 'dims': b['rot_dims'], 'scaling': {'factor': 4.0, 'original': 1024, 'fast': 16.0, 'slow': 2.0}}}
    left = {'heads': H, 'kv_heads': b['left_kv'], 'dim': 128, 'vdim': 128, 'scale': 128 ** -0.5, 'mask': {'size': b['window']},
            'bias_max': b['bias_max'], 'buckets': b['buckets']}
    right = {'heads': H, 'kv_heads': G, 'dim': 128, 'vdim': 128, 'conv': b['conv'], 'a_rank': b['rank'], 'g_rank': b['rank']}
    dense = {'kind': 'dense', 'ff': s['inter']}
    four = [{'type': 'attention', 'mixer': att, 'mlp': dense}] * 3 + [{'type': 'parallel', 'mixer': {'left': left, 'right': right}, 'mlp': dense}]
    return {'architecture': 'Mededra', 'width': s['width'], 'vocab': s['vocab'], 'norm': {'eps': 1e-5, 'groups': 8}, 'embedding': {'scale': 1.0},
            'logit_softcap': 30.0, 'layers': [four[i % 4] for i in range(s['layers'])]}


def _mededra_engine(s, batch, session_len, max_prefill):
    from . import layered
    cfg = layered.FAMILIES['Mededra'](mededra_config(s))
    eng = layered.LayeredEngine(cfg, dtype='bfloat16', max_batch_size=batch, session_len=session_len, max_prefill_token_num=max_prefill)
    eng.init_synthetic(seed=1)
    eng.start()
    return eng


def _mededra_decode_bytes(s, batch, ctx):
    """bytes each category of ONE decode step must move: every weight once, the cache entries inside the windows once per sequence, the
    delta rule's state read and written once (fp32)"""
    b, W, H, G, V = MEDEDRA, s['width'], s['heads'], s['kv_heads'], s['vocab']
    out = dict(gemm_qkv=0, attention=0, gemm_o=0, gemm_gate_up=0, gemm_down=0, lm_head=2 * W * V)
    seen = min(ctx, b['window'])
    for i in range(s['layers']):
        if i % 4 != 3:
            out['gemm_qkv'] += 2 * W * (H * 2 * b['map_dim'] + G * 2 * b['map_dim'] + G * 128)
            out['attention'] += 2 * batch * (G * 2 * b['map_dim'] + G * 128) * seen
            out['gemm_o'] += 2 * W * H * 128
        else:
            lk = b['left_kv']
            out['gemm_qkv'] += 2 * W * (H * 128 + lk * 128 + H * 128 + 2 * G * 128 + H * 128 + H + 2 * b['rank']) + 2 * b['rank'] * 2 * H * 128
            out['attention'] += 2 * batch * 2 * lk * 128 * seen + batch * H * 128 * 128 * 4 * 2
            out['gemm_o'] += 2 * 2 * W * H * 128
        out['gemm_gate_up'] += 2 * W * 2 * s['inter']
        out['gemm_down'] += 2 * W * s['inter']
    return out


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


def run(steps: int, warmup: int, batch: int, prompt_len: int, sizes=None, design: str = 'fokonex', only_first: bool = False) -> dict:
    res = {}
    pair = {'fokonex': (('fokonex_bf16', _fokonex_engine), ('llama_f16', _llama_engine)),
            'bedenex': (('bedenex_bf16', _bedenex_engine), ('fokonex_bf16', _fokonex_engine)),
            'febivik': (('febivik_bf16', _febivik_engine), ('bedenex_bf16', _bedenex_engine)),
            'mededra': (('mededra_bf16', _mededra_engine), ('febivik_bf16', _febivik_engine))}[design]
    if only_first:
        pair = pair[:1]
    for name in (sizes or SIZES):
        s = SIZES[name]
        session_len = prompt_len + steps + warmup + 64
        prefill_seqs = max(1, 8192 // prompt_len)
        row = {}
        for kind, make in pair:
            eng = make(s, batch, session_len, 8192)
            m = _measure(eng, s['vocab'], batch, prompt_len, steps, warmup, prefill_seqs)
            ctx = prompt_len + warmup + steps // 2
            need = _mededra_decode_bytes(s, batch, ctx) if kind == 'mededra_bf16' else _febivik_decode_bytes(s, batch, ctx) if kind == 'febivik_bf16' else \
                _bedenex_decode_bytes(s, batch, ctx) if kind == 'bedenex_bf16' else _decode_bytes(s, batch, ctx, kind == 'fokonex_bf16')
            m['decode_hbm_roofline_fraction'] = {k: round(need[k] / HBM_BYTES_PER_S / (m['decode_categories_ms'][k] * 1e-3), 4)
                                                 for k in need if m['decode_categories_ms'].get(k)}
            eng.close()
            row[kind] = m
        if only_first:
            res[name] = row
            continue
        f, l = row[pair[0][0]], row[pair[1][0]]
        if design != 'fokonex':   # how much farther from its roofline each category of the new design runs than the like one beside it
            fa, fb = f['decode_hbm_roofline_fraction'], l['decode_hbm_roofline_fraction']
            fb = dict(fb, gemm_down=fb.get('gemm_down', fb.get('gemm_o')))      # (Fokonex closes a block with ONE [o | down] product)
            row['roofline_distance_ratio'] = {k: round(fb[k] / fa[k], 2) for k in fa if fb.get(k) and fa[k] > 0}
        row['prefill_ratio'] = round(f['prefill_tokens_per_s'] / l['prefill_tokens_per_s'], 3)
        row['decode_ratio'] = round(f['decode_tokens_per_s'] / l['decode_tokens_per_s'], 3)
        res[name] = row
    return res
