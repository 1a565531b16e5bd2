"""GPU tests of the Mededra design on the layer-list engine against the plain float64 model in tests/mededra_oracle.py: the attention
kernels with key and value head counts of their own, a distance table, a zero sink and fp32 output (every kernel; one loud key just inside
and just outside the window, a sink that outweighs every key); every mixer form alone in a one-layer model through a portion and
token-by-token decoding; then a model of all of them -- the stream behind every layer, whole prompts, decoding from the first token,
portions down to two tokens (shorter than the convolutions), unequal batches, state slots and cache blocks that are used again, long
decoding far beyond the windows, a far token held by the delta rule's state, greedy generation through the static batch, the scheduler
and the pipeline, and bin/trace_run.  Configurations and weights are the tests' own."""
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
from tests import mededra_oracle as mo
from tests.gpu_helpers import dev, host, release_all, st

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _release():
    yield
    release_all()


def act(x, dtype):
    return dev(mo.bf16_bits(x).view(np.int16)) if dtype == 0 else dev(np.asarray(x, np.float32))


def _rounded(x, dtype):
    return mo.bf16_round(x) if dtype == 0 else np.asarray(x, np.float32).astype(np.float64)


# ---- the attention kernels with the new parameters ---------------------------------------------------------------------------------
class Paged:
    """keys [KH][64][D] and transposed values [VH][V][64] per block, blocks shuffled, junk where nothing was stored"""

    def __init__(self, dtype, KH, VH, D, V, lens, rng):
        per = [(n + 63) // 64 for n in lens]
        self.stride, nb = max(per) + 1, sum(per) + 2
        self.elems, self.eb = 64 * (KH * D + VH * V), 2 if dtype == 0 else 4
        self.pool = act(rng.normal(0, 30, (nb, self.elems)), dtype)
        order, ptrs, k = rng.permutation(nb), np.zeros((len(lens), self.stride), np.uint64), 0
        for s, n in enumerate(per):
            for i in range(n):
                ptrs[s, i] = self.pool.data_ptr() + int(order[k]) * self.elems * self.eb
                k += 1
        self.ptrs, self.v_offset = dev(ptrs.view(np.int64)), KH * 64 * D * self.eb


def attend(tm, dtype, spec, cache, q, k_new, v_new, row_seq, row_pos, cu_q, k_len, kernel, splits=1, prefill=1):
    H, G, KH, VH, D, V = spec['heads'], spec['groups'], spec['k_heads'], spec['v_heads'], spec['dim'], spec['vdim']
    rows = q.shape[0]
    ld = (H * D + KH * D + VH * V + 31) // 32 * 32
    qkv = np.zeros((rows, ld))
    qkv[:, :H * D], qkv[:, H * D:H * D + KH * D], qkv[:, H * D + KH * D:H * D + KH * D + VH * V] = q, k_new, v_new
    qkv_d = act(qkv, dtype)
    out = torch.zeros((rows, H * V + 3), dtype=torch.float32, device='cuda')
    ws = torch.zeros(max(1, tm.tm_general_attention_workspace(rows, H, V, splits) // 4), dtype=torch.float32, device='cuda')
    tab = spec.get('table')
    tab_d = dev(np.asarray(tab, np.float32)) if tab is not None else None
    sink_d = dev(np.zeros(H, np.float32)) if spec.get('zero_sink') else None
    a = _ffi.GeneralAttn(qkv_d.data_ptr(), out.data_ptr(), ld, H * V + 3, rows, dev(np.asarray(row_seq, np.int32)).data_ptr(),
                         dev(np.asarray(row_pos, np.int32)).data_ptr(), cache.ptrs.data_ptr(), cache.stride, 0, cache.v_offset, cache.eb,
                         H, G, D, V, spec['scale'], spec.get('softcap', 0.0), 0.0, 1.0, sink_d.data_ptr() if sink_d is not None else None, splits,
                         ws.data_ptr(), qkv_d.data_ptr(), ld, H * D, H * D + KH * D, 1,
                         kernel, prefill, len(cu_q) - 1, int(np.diff(cu_q).max()), dev(np.asarray(cu_q, np.int32)).data_ptr(),
                         dev(np.asarray(k_len, np.int32)).data_ptr(), None, None, 0, None, 0, 0, spec['window'], 0, KH, VH,
                         tab_d.data_ptr() if tab_d is not None else None, tab.shape[1] if tab is not None else 0, 1)
    _ffi.check(tm.tm_general_attention(C.byref(a), st()))
    return host(out).astype(np.float64)[:, :H * V]


def row_oracle(spec, q, keys, vals, pos):
    """one row at position pos; keys [pos + 1, KH, D], vals [pos + 1, VH, V] -> [H * V]; group g reads key head g % KH, value head g % VH"""
    H, G, KH, VH, D, V = spec['heads'], spec['groups'], spec['k_heads'], spec['v_heads'], spec['dim'], spec['vdim']
    W, cap, tab = spec['window'], spec.get('softcap', 0.0), spec.get('table')
    js = [j for j in range(pos + 1) if W <= 0 or pos - j < W]
    out = np.zeros((H, V))
    for h in range(H):
        g = h // (H // G)
        s = (keys[js, g % KH] @ q[h * D:(h + 1) * D]) * spec['scale']
        if cap > 0:
            s = cap * np.tanh(s / cap)
        if tab is not None:
            s = s + np.array([tab[h, min(pos - j, tab.shape[1] - 1)] for j in js])
        m = max(s.max(), 0.0) if spec.get('zero_sink') else s.max()
        e = np.exp(s - m)
        out[h] = (e / (e.sum() + (np.exp(-m) if spec.get('zero_sink') else 0.0))) @ vals[js, g % VH]
    return out.reshape(-1)


def _table(heads, n, seed):
    return np.asarray(np.random.default_rng(seed).normal(0, 1.0, (heads, n)), np.float32).astype(np.float64)


ATT = {
    'two_maps_over_one_value_set': dict(heads=8, groups=4, k_heads=4, v_heads=2, dim=32, vdim=48, scale=0.3, window=50, softcap=5.0),
    'two_maps_ungrouped_odd_sizes': dict(heads=6, groups=6, k_heads=6, v_heads=3, dim=20, vdim=12, scale=0.2, window=0),
    'wide_key_value_head_per_group': dict(heads=6, groups=2, k_heads=1, v_heads=2, dim=64, vdim=32, scale=0.15, window=70, zero_sink=True,
                                          table=_table(6, 70, 1)),
    'wide_key_one_group_short_table': dict(heads=3, groups=1, k_heads=1, v_heads=1, dim=40, vdim=40, scale=0.2, window=0, zero_sink=True,
                                           table=_table(3, 33, 2)),
    'wide_key_beyond_the_tiles': dict(heads=4, groups=4, k_heads=1, v_heads=4, dim=320, vdim=80, scale=0.05, window=64, zero_sink=True,
                                      table=_table(4, 64, 3)),
}


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('name', list(ATT))
def test_attention_head_counts_table_sink_in_every_kernel(tm, cuda, dtype, name):
    """portions that start and end inside windows and blocks, then one decoded row per sequence, each kernel that serves the format"""
    spec, rng = ATT[name], np.random.default_rng(5)
    H, KH, VH, D, V = spec['heads'], spec['k_heads'], spec['v_heads'], spec['dim'], spec['vdim']
    lens, first = [203, 77, 1, 130], [0, 30, 0, 51]
    cache = Paged(dtype, KH, VH, D, V, [n + 1 for n in lens], rng)
    K = [_rounded(rng.normal(0, 1, (n + 1, KH, D)), dtype) for n in lens]
    Vv = [_rounded(rng.normal(0, 1, (n + 1, VH, V)), dtype) for n in lens]
    tol = 3e-2 if dtype == 0 else 2e-5
    mfma = dtype == 0 and D % 8 == 0 and V % 8 == 0 and D <= 256

    def run(lo_, hi_, kernels, prefill, splits=1):
        rs, rp, cu, kl = [], [], [0], []
        for s in range(len(lens)):
            rs += [s] * (hi_[s] - lo_[s])
            rp += list(range(lo_[s], hi_[s]))
            cu.append(len(rs))
            kl.append(hi_[s])
        q = _rounded(rng.normal(0, 1, (len(rs), H * D)), dtype)
        kn = np.stack([K[s][p].reshape(-1) for s, p in zip(rs, rp)])
        vn = np.stack([Vv[s][p].reshape(-1) for s, p in zip(rs, rp)])
        ref = np.stack([row_oracle(spec, q[i], K[s][:p + 1], Vv[s][:p + 1], p) for i, (s, p) in enumerate(zip(rs, rp))])
        for kern in kernels:
            got = attend(tm, dtype, spec, cache, q, kn, vn, rs, rp, cu, kl, kern, splits, prefill)
            assert np.abs(got - ref).max() <= tol * max(1.0, np.abs(ref).max()), (name, kern, splits)

    run([0] * 4, first, [1], 1)
    run(first, lens, [1, 2] if mfma else [1], 1)
    dec = [n + 1 for n in lens]
    run(lens, dec, [1, 3] if mfma else [1], 0)
    run(lens, dec, [1, 3] if mfma else [1], 0, splits=3)


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('kernel', [1, 2, 3])
def test_window_edges_and_sink_with_one_loud_key(tm, cuda, dtype, kernel):
    """one key far louder than all others at the window's last position (seen: the output is its value) or one before it (unseen), inside
    a block, on a block border and hundreds of tokens back, in the second map's key head; and a zero sink that outweighs every key when
    all scores are far below zero (the output vanishes)"""
    if kernel != 1 and dtype == 1:
        pytest.skip('the matrix-core kernels are bf16')
    spec = dict(heads=4, groups=2, k_heads=2, v_heads=1, dim=32, vdim=16, scale=1.0, window=96)
    rng = np.random.default_rng(9)
    n = 400
    for pos in (95, 96, 159, 160, 191, 399):
        for hot in sorted({pos - 95, pos - 96, 0, pos}):
            if hot < 0 or hot > pos:
                continue
            seen = pos - hot < 96
            K = _rounded(rng.normal(0, 0.05, (n, 2, 32)), dtype)
            Vv = _rounded(rng.normal(0, 1, (n, 1, 16)), dtype)
            q = _rounded(np.tile(rng.normal(0, 1, 32), 4)[None, :], dtype)
            K[hot, 1] = _rounded(q[0, :32] * 1.5, dtype)          # only the second key head holds the loud key: heads 2 and 3 hear it
            cache = Paged(dtype, 2, 1, 32, 16, [n], rng)
            if pos:
                attend(tm, dtype, spec, cache, _rounded(rng.normal(0, 1, (pos, 128)), dtype), K[:pos].reshape(pos, -1), Vv[:pos].reshape(pos, -1),
                       [0] * pos, list(range(pos)), [0, pos], [pos], 1)
            got = attend(tm, dtype, spec, cache, q, K[pos:pos + 1].reshape(1, -1), Vv[pos:pos + 1].reshape(1, -1), [0], [pos], [0, 1],
                         [pos + 1], kernel, 1, 1 if kernel == 2 else 0)
            ref = row_oracle(spec, q[0], K[:pos + 1], Vv[:pos + 1], pos)
            assert np.abs(got[0] - ref).max() <= (4e-2 if dtype == 0 else 1e-4), (pos, hot)
            near = np.abs(got[0, 32:48] - Vv[hot, 0]).max()
            assert (near < 0.1) == seen, (pos, hot, near)
            assert np.abs(got[0, :16] - Vv[hot, 0]).max() > 0.1 or pos == hot == 0              # the first key head's query heads do not hear it
    sink = dict(heads=2, groups=1, k_heads=1, v_heads=1, dim=32, vdim=16, scale=1.0, window=0, zero_sink=True)
    q = _rounded(rng.normal(0, 1, (1, 32)), dtype)
    K = _rounded(-q[0][None, None, :] * np.ones((130, 1, 1)), dtype)                               # every score is -|q|^2, about -32
    Vv = _rounded(rng.normal(0, 1, (130, 1, 16)), dtype)
    cache = Paged(dtype, 1, 1, 32, 16, [130], rng)
    attend(tm, dtype, sink, cache, _rounded(rng.normal(0, 1, (129, 64)), dtype), K[:129].reshape(129, -1), Vv[:129].reshape(129, -1), [0] * 129,
           list(range(129)), [0, 129], [129], 1)
    got = attend(tm, dtype, sink, cache, np.tile(q, (1, 2)), K[129:].reshape(1, -1), Vv[129:].reshape(1, -1), [0], [129], [0, 1], [130], kernel, 1,
                 1 if kernel == 2 else 0)
    assert np.abs(got).max() < 1e-6
    assert np.abs(got - row_oracle(sink, np.tile(q, (1, 2))[0], K, Vv, 129)).max() < 1e-6


# ---- engine -------------------------------------------------------------------------------------------------------------------------
YARN = {'factor': 4.0, 'original': 64, 'fast': 8.0, 'slow': 1.0}


def model_folder(tmp_path, cfg, seed, name='m', **kw):
    w = mo.random_weights(cfg, seed, **kw)
    folder = str(tmp_path / name)
    mo.write_checkpoint(folder, cfg, w)
    return folder, w


def engine(folder, dtype, **kw):
    args = dict(max_batch_size=4, session_len=512, cache_blocks=12, max_prefill_token_num=512, use_graph=0)
    args.update(kw)
    return layered.build_engine(folder, dtype=dtype, **args)


def full_model():
    """both mixers in several forms: grouped and ungrouped heads, key sizes on and off the 8 grid, value sizes that differ from the key
    sizes, windows that cut cache blocks, rotation of a part of the head with and without frequency scaling, convolutions of 2, 3 and 4
    taps, a block without feed-forward, norms in 3 groups"""
    return mo.make_config(72, 211, [
        mo.attention_layer(4, 2, 16, 24, 0.3, 50, 8, 3000.0, YARN, 10.0, 0.35, 4, mo.dense(88)),
        mo.parallel_layer(mo.left_mixer(6, 2, 24, 40, 100, 0.25), mo.right_mixer(4, 2, 20, 24, 2), mo.dense(40)),
        mo.attention_layer(3, 3, 20, 12, 0.4, 7, 20, 100.0, None, 0.0, 0.8, 2),
        mo.parallel_layer(mo.left_mixer(2, 2, 16, 33, 64), mo.right_mixer(2, 2, 16, 48, 4), mo.dense(56)),
        mo.attention_layer(6, 2, 8, 16, 0.5, 0, 0, diff=0.2, conv=3, mlp=mo.dense(40)),
    ], groups=3, embed_scale=2.0, logit_softcap=12.0)


TOL = {'float32': 3e-5, 'bfloat16': 8e-2}
RANKS = dict(buckets=12, a_rank=5, g_rank=9)


def rel_err(got, ref):
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)).max() / ref.std()


ALONE = {
    'diff_attention_window_rotation_scaled': lambda: mo.make_config(64, 97, [mo.attention_layer(4, 1, 16, 32, 0.5, 33, 8, 500.0, YARN, 20.0)], groups=2),
    'diff_attention_plain_causal_full_rotation': lambda: mo.make_config(48, 97, [mo.attention_layer(2, 2, 40, 8, 0.2, 0, None, 10000.0)]),
    'diff_attention_no_rotation_window_1_one_tap': lambda: mo.make_config(48, 97, [mo.attention_layer(2, 1, 24, 24, 0.2, 1, 0, conv=1)], groups=4),
    'diff_attention_head_128_taps_8': lambda: mo.make_config(64, 97, [mo.attention_layer(2, 1, 128, 128, 0.09, 100, 64, 1e6, YARN, 30.0, conv=8)]),
    'diff_attention_three_heads_per_key_head': lambda: mo.make_config(60, 97, [mo.attention_layer(6, 2, 12, 20, 0.3, 64, 12, conv=2, diff=0.7)], groups=5),
    'parallel_small': lambda: mo.make_config(64, 97, [mo.parallel_layer(mo.left_mixer(4, 2, 16, 40, 120), mo.right_mixer(4, 2, 16, 32))], groups=2),
    'parallel_one_key_head_one_state_head': lambda: mo.make_config(48, 97, [mo.parallel_layer(mo.left_mixer(3, 1, 20, 64, 70), mo.right_mixer(1, 1, 50, 70, 2))]),
    'parallel_ungrouped_large_heads': lambda: mo.make_config(64, 97, [mo.parallel_layer(mo.left_mixer(2, 2, 128, 150, 128), mo.right_mixer(2, 1, 128, 128, 4))]),
    'parallel_wide_key_beyond_the_tiles': lambda: mo.make_config(64, 97, [mo.parallel_layer(mo.left_mixer(8, 8, 40, 20, 30), mo.right_mixer(3, 3, 32, 8, 1))]),
    'parallel_state_head_256': lambda: mo.make_config(48, 97, [mo.parallel_layer(mo.left_mixer(2, 1, 8, 5, 40), mo.right_mixer(2, 1, 256, 40, 3))]),
    'gated_feed_forward': lambda: mo.make_config(64, 97, [mo.attention_layer(2, 2, 8, 8, 0.3, 16, 4, mlp=mo.dense(100))], groups=8, embed_scale=0.5,
                                                 logit_softcap=5.0),
}


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('name', list(ALONE))
def test_each_mechanism_alone(cuda, tmp_path, dtype, name):
    cfg = ALONE[name]()
    toks = np.random.default_rng(1).integers(0, 97, 150).tolist()
    cut = len(toks) // 2
    folder, w = model_folder(tmp_path, cfg, 3, buckets=8 if 'small' in name else 32, a_rank=3, g_rank=40)
    ref_logits, trail = mo.forward(cfg, w, toks, True)
    eng = engine(folder, dtype)
    eng.stop_after(1)
    s = eng.open_session()
    eng.step_tokens([(s, toks, [])])
    got = eng.fetch_residual(len(toks))
    eng.close_session(s)
    assert np.abs(got - trail[0]).max() <= TOL[dtype] * 3 * np.abs(trail[0]).max()
    eng.stop_after(-1)
    s = eng.open_session()                                        # the same through cache and state: a portion, then token by token
    rows = [eng.step_tokens([(s, toks[:cut], list(range(cut)))])] + [eng.step_tokens([(s, [t], [0])]) for t in toks[cut:]]
    eng.close_session(s)
    assert rel_err(np.concatenate(rows), ref_logits) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_layers_and_whole_prompt(cuda, tmp_path, dtype):
    cfg = full_model()
    folder, w = model_folder(tmp_path, cfg, 0, **RANKS)
    eng = engine(folder, dtype)
    toks = np.random.default_rng(1).integers(0, cfg['vocab'], 150).tolist()
    ref, trail = mo.forward(cfg, w, toks[:70], True)
    for n in range(1, len(cfg['layers']) + 1):                    # the residual stream behind every layer
        eng.stop_after(n)
        s = eng.open_session()
        eng.step_tokens([(s, toks[:70], [])])
        got = eng.fetch_residual(70)
        eng.close_session(s)
        assert np.abs(got - trail[n - 1]).max() <= TOL[dtype] * 3 * np.abs(trail[n - 1]).max(), n
    eng.stop_after(-1)
    ref = mo.forward(cfg, w, toks)
    s = eng.open_session()
    got = eng.step_tokens([(s, toks, list(range(len(toks))))])
    eng.close_session(s)
    assert rel_err(got, ref) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_portions_decoding_batches_and_reuse(cuda, tmp_path, dtype):
    """every way of cutting the same requests gives the oracle's logits: token by token from the first token on, portions down to one and
    two tokens (shorter than the convolutions' reach) that start and end inside blocks and windows, unequal requests in one forward, and
    sessions that come and go in a pool that holds only what is live -- cache blocks and state slots are used again with other requests'
    keys, convolution inputs and states still in them"""
    cfg = full_model()
    folder, w = model_folder(tmp_path, cfg, 1, **RANKS)
    rng = np.random.default_rng(2)
    reqs = [rng.integers(0, cfg['vocab'], n).tolist() for n in (200, 131, 65, 1, 23)]
    refs = [mo.forward(cfg, w, t) for t in reqs]
    eng = engine(folder, dtype, cache_blocks=9)
    tol = TOL[dtype]
    s = eng.open_session()
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in reqs[1]])
    eng.close_session(s)
    assert rel_err(got, refs[1]) <= tol
    s, at, rows = eng.open_session(), 0, []
    for n in [2, 1, 2, 58, 2, 64, 3, 30, 2] + [1] * 36:
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
    assert rel_err(out, mo.forward(cfg, w, reqs[1] + [5])[-1:]) <= tol
    eng.close_session(b)
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_long_decoding_far_beyond_the_windows(cuda, tmp_path, dtype):
    """420 tokens, the last 320 one at a time with the decode rows' keys split over several workgroups (session_len 1024 -> 4 splits):
    windows of 100 and 130 positions (edges inside blocks) pass over decoded tokens, the delta rule's state lives through hundreds of steps"""
    cfg = mo.make_config(64, 97, [mo.attention_layer(4, 2, 16, 8, 0.4, 100, 8, 1000.0, YARN, 15.0, mlp=mo.dense(72)),
                                  mo.parallel_layer(mo.left_mixer(4, 2, 16, 130, 200), mo.right_mixer(2, 1, 12, 24)),
                                  mo.attention_layer(2, 2, 8, 16, 0.4, 64, 0, conv=2)], groups=2)
    folder, w = model_folder(tmp_path, cfg, 4, **RANKS)
    toks = np.random.default_rng(3).integers(0, 97, 420).tolist()
    ref = mo.forward(cfg, w, toks)
    eng = engine(folder, dtype, session_len=1024, cache_blocks=17, max_prefill_token_num=256)
    s = eng.open_session()
    eng.step_tokens([(s, toks[:100], [])])
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in toks[100:]])
    eng.close_session(s)
    assert rel_err(got, ref[100:]) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('kind', ['differential', 'left'])
def test_window_edges_through_the_engine(cuda, tmp_path, dtype, kind):
    """one-layer models whose only way back in time is the window (one-tap convolutions; the delta rule's branch weighs zero): another
    token just outside a row's window leaves the row's logits as they are, another token at the window's last position moves them --
    windows that end inside a block and on a block border, prompt rows and decoded rows"""
    for W in (37, 64):
        if kind == 'differential':
            cfg = mo.make_config(48, 61, [mo.attention_layer(2, 1, 16, 16, 0.4, W, 8, 1000.0, None, 0.0, 0.4, 1)], groups=2)
            w = mo.random_weights(cfg, 21)
        else:
            cfg = mo.make_config(48, 61, [mo.parallel_layer(mo.left_mixer(4, 2, 16, W, 50, 0.4), mo.right_mixer(2, 1, 8, 8, 2))], groups=2)
            w = mo.random_weights(cfg, 21, buckets=8, a_rank=4, g_rank=4)
            w['l0.mix.right.out'] = np.zeros_like(w['l0.mix.right.out'])
        folder = str(tmp_path / f'{kind}{W}')
        mo.write_checkpoint(folder, cfg, w)
        eng = engine(folder, dtype)
        toks = np.random.default_rng(W).integers(0, 61, 150).tolist()
        rows = [W, 100, 128, 149]

        def logits(t, decode_from):
            s = eng.open_session()
            out = eng.step_tokens([(s, t[:decode_from], [r for r in rows if r < decode_from])])
            rest = [eng.step_tokens([(s, [x], [0])]) for x in t[decode_from:]]
            eng.close_session(s)
            return np.concatenate([out] + [rest[r - decode_from] for r in rows if r >= decode_from])

        for decode_from in (150, 90):
            base = logits(toks, decode_from)
            assert rel_err(base, mo.forward(cfg, w, toks)[rows]) <= TOL[dtype]
            for k, r in enumerate(rows):
                for j, seen in ((r - W, False), (r - W + 1, True)):
                    other = list(toks)
                    other[j] = (toks[j] + 7) % 61
                    moved = np.abs(logits(other, decode_from)[k] - base[k]).max() / base.std()
                    assert (moved > 1e-3) == seen and (seen or moved <= 1e-6), (W, decode_from, r, j, moved)
        eng.close()


def test_state_of_a_far_token_survives_hundreds_of_steps(cuda, tmp_path):
    """a delta-rule state that barely decays (A_log far below zero) and writes weakly keeps a token from 300 positions back, far outside
    the left mixer's window: moving that one token moves the last logits, in one portion and when everything after the first portion is
    decoded token by token"""
    cfg = mo.make_config(32, 53, [mo.parallel_layer(mo.left_mixer(2, 1, 8, 16, 32), mo.right_mixer(1, 1, 16, 16, 2))])
    folder = str(tmp_path / 'm')
    w = mo.random_weights(cfg, 6, buckets=8, a_rank=4, g_rank=4)
    w['l0.mix.right.A_log'] = mo.bf16_round(np.full(1, -9.0))
    w['l0.mix.right.b'] = mo.bf16_round(w['l0.mix.right.b'] * 0.0 - 0.0)
    w['l0.mix.right.out'] = mo.bf16_round(w['l0.mix.right.out'] * 4.0)
    mo.write_checkpoint(folder, cfg, w)
    rng = np.random.default_rng(8)
    a = rng.integers(0, 53, 330).tolist()
    b = list(a)
    b[20] = (a[20] + 17) % 53
    ra, rb = mo.forward(cfg, w, a)[-1], mo.forward(cfg, w, b)[-1]
    assert np.abs(ra - rb).max() > 50 * 3e-5 * ra.std()           # the far token matters far more than the tolerance
    eng = engine(folder, 'float32')
    for toks, ref in ((a, ra), (b, rb)):
        s = eng.open_session()
        whole = eng.step_tokens([(s, toks, [len(toks) - 1])])
        eng.close_session(s)
        s = eng.open_session()
        eng.step_tokens([(s, toks[:25], [])])
        for t in toks[25:-1]:
            eng.step_tokens([(s, [t], [])])
        last = eng.step_tokens([(s, toks[-1:], [0])])
        eng.close_session(s)
        assert rel_err(whole, ref[None]) <= 3e-5 and rel_err(last, ref[None]) <= 3e-5
    eng.close()


def _greedy(cfg, w, prompt, n_new):
    toks, margins = list(prompt), []
    for _ in range(n_new):
        lg = mo.forward(cfg, w, toks)[-1]
        top = np.sort(lg)[-2:]
        margins.append((top[1] - top[0]) / lg.std())
        toks.append(int(np.argmax(lg)))
    return toks[len(prompt):], margins


def _check_greedy(cfg, w, prompt, toks, min_margin=2e-2):     # (the sampler reads fp16 logits rows)
    ref, margins = _greedy(cfg, w, prompt, len(toks))
    for i, (a, b, m) in enumerate(zip(toks, ref, margins)):
        if m < min_margin:
            return          # a near-tie: from here on the two may legitimately part
        assert int(a) == b, (i, toks, ref)


def test_greedy_generation_static_batch_and_scheduler(cuda, tmp_path):
    cfg = full_model()
    folder, w = model_folder(tmp_path, cfg, 2, **RANKS)
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
    cfg = full_model()
    folder, w = model_folder(tmp_path, cfg, 3, **RANKS)
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
    """bin/trace_run end to end, both number formats: a width off the 8 grid, windows as long as a cache block and longer than a
    request, five requests in shared steps, pool of 640 tokens"""
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
    cfg = mo.make_config(100, 333, [mo.parallel_layer(mo.left_mixer(10, 2, 8, 64, 90), mo.right_mixer(3, 3, 20, 24), mo.dense(72)),
                                    mo.attention_layer(10, 2, 8, 24, 0.35, 64, 8, 20000.0, YARN, 25.0, mlp=mo.dense(72)),
                                    mo.attention_layer(5, 5, 24, 8, 0.3, 1000, 0)], groups=5, embed_scale=1.5, logit_softcap=20.0)
    folder, w = model_folder(tmp_path, cfg, 11, 'model', **RANKS)
    ref = {n: mo.forward(cfg, w, t) for n, t in reqs.items()}
    for dtype, tol in (('float32', 5e-5), ('bfloat16', 5e-2)):
        out = str(tmp_path / dtype)
        p = subprocess.run([sys.executable, os.path.join(root, 'bin', 'trace_run'), '--model', folder, '--dtype', dtype, '--out', out,
                            '--max-tokens', '640'], input='\n'.join(steps) + '\n', text=True, capture_output=True, timeout=100)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.split('\n') if l.startswith('done')] == ['done %d' % i for i in range(len(plan))]
        for i, rr in enumerate(rows):
            got = np.fromfile(os.path.join(out, '%d.f32' % i), '<f4').reshape(len(rr), -1)
            assert rel_err(got, np.stack([ref[n][j] for n, j in rr])) <= tol, (dtype, i)
