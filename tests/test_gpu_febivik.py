"""GPU tests of the Febivik design on the layer-list engine against the plain float64 model in tests/febivik_oracle.py: the attention
kernels' sliding window with kept first tokens alone (every kernel; one loud key just inside and just outside the window, among the kept
tokens and just behind them, at block borders and far back); every mixer and feed-forward alone in a one-layer model through a portion
and token-by-token decoding; then a model of all of them -- the stream behind every layer, whole prompts, decoding from the first token,
portions down to two tokens, unequal batches, state slots and cache blocks that are used again, long decoding far beyond the window,
greedy generation through the static batch, the scheduler and the pipeline, and bin/trace_run.  Configurations and weights are the
tests' own."""
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
from tests import febivik_oracle as fo
from tests.gpu_helpers import dev, host, release_all, st

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _release():
    yield
    release_all()


def bf16_round(x):
    return (fo.bf16_bits(x).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def act(x, dtype):
    return dev(fo.bf16_bits(x).view(np.int16)) if dtype == 0 else dev(np.asarray(x, np.float32))


def read(t, dtype):
    if dtype == 0:
        return (host(t).view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return host(t).astype(np.float64)


def _rounded(x, dtype):
    return bf16_round(x) if dtype == 0 else np.asarray(x, np.float32).astype(np.float64)


# ---- the attention kernels with a window and kept first tokens ---------------------------------------------------------------------
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


def attend(tm, dtype, spec, cache, q, k_new, v_new, row_seq, row_pos, cu_q, k_len, kernel, splits=1, prefill=1):
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    rows = q.shape[0]
    ld = (H * D + G * D + G * V + 31) // 32 * 32
    qkv = np.zeros((rows, ld))
    qkv[:, :H * D], qkv[:, H * D:H * D + G * D], qkv[:, H * D + G * D:H * D + G * D + G * V] = q, k_new, v_new
    qkv_d = act(qkv, dtype)
    out = act(np.zeros((rows, H * V + 3)), dtype)
    ws = torch.zeros(max(1, tm.tm_general_attention_workspace(rows, H, V, splits) // 4), dtype=torch.float32, device='cuda')
    a = _ffi.GeneralAttn(qkv_d.data_ptr(), out.data_ptr(), ld, H * V + 3, rows, dev(np.asarray(row_seq, np.int32)).data_ptr(),
                         dev(np.asarray(row_pos, np.int32)).data_ptr(), cache.ptrs.data_ptr(), cache.stride, 0, cache.v_offset, cache.eb,
                         H, G, D, V, spec['scale'], 0.0, 0.0, 1.0, None, splits, ws.data_ptr(), qkv_d.data_ptr(), ld, H * D, H * D + G * D, 1,
                         kernel, prefill, len(cu_q) - 1, int(np.diff(cu_q).max()), dev(np.asarray(cu_q, np.int32)).data_ptr(),
                         dev(np.asarray(k_len, np.int32)).data_ptr(), None, None, 0, None, 0, 0, spec['window'], spec['keep'])
    _ffi.check(tm.tm_general_attention(C.byref(a), st()))
    return read(out, dtype)[:, :H * V]


def row_oracle(spec, q, keys, vals, pos):
    """one row at position pos; keys / vals [pos + 1, G, .] -> [H * V]"""
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    js = [j for j in range(pos + 1) if fo.visible(pos, j, spec['window'], spec['keep'])]
    out = np.zeros((H, V))
    for h in range(H):
        g = h // (H // G)
        s = (keys[js, g] @ q[h * D:(h + 1) * D]) * spec['scale']
        e = np.exp(s - s.max())
        out[h] = (e / e.sum()) @ vals[js, g]
    return out.reshape(-1)


ATT = {
    'window_off_block': dict(heads=4, kv_heads=2, dim=32, vdim=16, scale=0.3, window=50, keep=3),
    'block_sized': dict(heads=6, kv_heads=1, dim=40, vdim=24, scale=0.2, window=64, keep=64),
    'tiny_window': dict(heads=3, kv_heads=3, dim=72, vdim=136, scale=0.1, window=1, keep=1),
    'kept_beyond_a_block': dict(heads=2, kv_heads=1, dim=20, vdim=12, scale=0.2, window=33, keep=70),
    'no_kept_tokens': dict(heads=16, kv_heads=1, dim=48, vdim=32, scale=0.15, window=100, keep=0),
    'window_longer_than_all': dict(heads=2, kv_heads=2, dim=64, vdim=64, scale=0.12, window=1000, keep=4),
}


@pytest.mark.parametrize('dtype', [0, 1])
@pytest.mark.parametrize('name', list(ATT))
def test_attention_window_and_kept_tokens_in_every_kernel(tm, cuda, dtype, name):
    """portions that start and end inside windows and blocks, then one decoded row per sequence, each kernel that serves the format"""
    spec, rng = ATT[name], np.random.default_rng(5)
    H, G, D, V = spec['heads'], spec['kv_heads'], spec['dim'], spec['vdim']
    lens, first = [203, 77, 1, 130], [0, 30, 0, 51]
    cache = Paged(dtype, G, D, V, [n + 1 for n in lens], rng)
    K = [_rounded(rng.normal(0, 1, (n + 1, G, D)), dtype) for n in lens]
    Vv = [_rounded(rng.normal(0, 1, (n + 1, G, V)), dtype) for n in lens]
    tol = 3e-2 if dtype == 0 else 2e-5
    mfma = dtype == 0 and D % 8 == 0 and V % 8 == 0

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
def test_attention_window_edges_with_one_loud_key(tm, cuda, dtype, kernel):
    """one key far louder than all others: at the window's last position (seen: the output is its value) or one before it (unseen), among
    the kept first tokens (seen) or right behind them (unseen); edges inside a block, on a block border and hundreds of tokens back"""
    if kernel != 1 and dtype == 1:
        pytest.skip('the matrix-core kernels are bf16')
    spec = dict(heads=2, kv_heads=1, dim=32, vdim=16, scale=1.0, window=96, keep=5)
    rng = np.random.default_rng(9)
    n = 400
    for pos in (95, 96, 159, 160, 191, 399):
        for hot in sorted({pos - 95, pos - 96, 4, 5, 0, pos}):
            if hot < 0 or hot > pos:
                continue
            seen = hot < 5 or pos - hot < 96
            K = _rounded(rng.normal(0, 0.05, (n, 1, 32)), dtype)
            Vv = _rounded(rng.normal(0, 1, (n, 1, 16)), dtype)
            q = _rounded(np.tile(rng.normal(0, 1, 32), 2)[None, :], dtype)
            K[hot, 0] = _rounded(q[0, :32] * 1.5, dtype)
            cache = Paged(dtype, 1, 32, 16, [n], rng)
            if pos:
                attend(tm, dtype, spec, cache, _rounded(rng.normal(0, 1, (pos, 64)), dtype), K[:pos].reshape(pos, -1), Vv[:pos].reshape(pos, -1),
                       [0] * pos, list(range(pos)), [0, pos], [pos], 1)
            got = attend(tm, dtype, spec, cache, q, K[pos:pos + 1].reshape(1, -1), Vv[pos:pos + 1].reshape(1, -1), [0], [pos], [0, 1],
                         [pos + 1], kernel, 1, 1 if kernel == 2 else 0)
            ref = row_oracle(spec, q[0], K[:pos + 1], Vv[:pos + 1], pos)
            assert np.abs(got[0] - ref).max() <= (4e-2 if dtype == 0 else 1e-4), (pos, hot)
            near = np.abs(got[0, :16] - Vv[hot, 0]).max()
            assert (near < 0.1) == seen, (pos, hot, near)


# ---- engine -------------------------------------------------------------------------------------------------------------------------
def model_folder(tmp_path, cfg, seed, name='m'):
    w = fo.random_weights(cfg, seed)
    folder = str(tmp_path / name)
    fo.write_checkpoint(folder, cfg, w)
    return folder, w


def engine(folder, dtype, **kw):
    args = dict(max_batch_size=4, session_len=512, cache_blocks=12, max_prefill_token_num=512, use_graph=0)
    args.update(kw)
    return layered.build_engine(folder, dtype=dtype, **args)


def chosen(dtype, k, experts):
    """experts per token of the many-layer models: k in float32; all of them in bfloat16, where one of hundreds of routing decisions can
    always be turned by rounding (top-k routing in bfloat16 is tested on one-layer models whose closest call is checked to be clear)"""
    return k if dtype == 'float32' else experts


def full_model(dtype='float32'):
    """all three mixers and both feed-forwards: key sizes on and off the 4 / 8 / 16 grids, value sizes that differ from the key sizes,
    a window that cuts cache blocks with three kept tokens, rotation of a part of the head, a block without feed-forward"""
    return fo.make_config(72, 211, [
        fo.lightning_layer(3, 20, 24, [0.5, 0.93, 0.999], fo.moe(5, chosen(dtype, 2, 5), 48, 1.7, 40)),
        fo.attention_layer(6, 2, 24, 40, 0.3, 50, 3, 16, 3000.0, 4.0, fo.dense(88)),
        fo.delta_layer(2, 18, 5, fo.moe(4, chosen(dtype, 1, 4), 24, 0.8)),
        fo.lightning_layer(2, 64, 16, [0.8, 0.97]),
        fo.attention_layer(3, 3, 20, 12, 0.4, 7, 0, 20, 100.0, 1.0, fo.dense(40)),
    ])


TOL = {'float32': 3e-5, 'bfloat16': 8e-2}


def rel_err(got, ref):
    d = got - ref
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)).max() / ref.std()


ALONE = {
    'lightning': lambda: fo.make_config(64, 97, [fo.lightning_layer(4, 16, 32, [0.55, 0.85, 0.95, 0.9975])]),
    'lightning_one_head_odd_sizes': lambda: fo.make_config(48, 97, [fo.lightning_layer(1, 30, 70, [0.95])]),
    'lightning_large_head': lambda: fo.make_config(64, 97, [fo.lightning_layer(2, 128, 128, [0.99, 0.9])]),
    'lightning_head_256': lambda: fo.make_config(48, 97, [fo.lightning_layer(1, 256, 40, [0.98])]),
    'lightning_head_32': lambda: fo.make_config(48, 97, [fo.lightning_layer(3, 32, 32, [0.7, 0.9, 0.99])]),
    'delta_head_256': lambda: fo.make_config(48, 97, [fo.delta_layer(1, 256, 6)]),
    'delta_head_32': lambda: fo.make_config(48, 97, [fo.delta_layer(2, 32, 2)]),
    'attention_window': lambda: fo.make_config(64, 97, [fo.attention_layer(4, 1, 16, 32, 0.5, 33, 2, 8, 500.0, 8.0)]),
    'attention_plain_causal_full_rotation': lambda: fo.make_config(48, 97, [fo.attention_layer(2, 2, 40, 8, 0.2, 0, 0, 40)]),
    'attention_no_rotation_window_1': lambda: fo.make_config(48, 97, [fo.attention_layer(2, 1, 24, 24, 0.2, 1, 1)]),
    'delta': lambda: fo.make_config(64, 97, [fo.delta_layer(4, 16, 8)]),
    'delta_odd_sizes': lambda: fo.make_config(40, 97, [fo.delta_layer(1, 50, 3)]),
    'delta_large_head': lambda: fo.make_config(64, 97, [fo.delta_layer(2, 128, 16)]),
    'xielu': lambda: fo.make_config(64, 97, [fo.lightning_layer(2, 8, 8, [0.9, 0.9], fo.dense(100))]),
    'experts_top1_no_shared': lambda: fo.make_config(64, 97, [fo.lightning_layer(2, 8, 8, [0.9, 0.9], fo.moe(3, 1, 24, 2.0))]),
    'experts_top2_shared': lambda: fo.make_config(64, 97, [fo.delta_layer(2, 8, 4, fo.moe(6, 2, 24, 1.5, 56))]),
    'experts_all': lambda: fo.make_config(64, 97, [fo.attention_layer(2, 1, 8, 8, 0.3, 16, 1, 4, mlp=fo.moe(4, 4, 40, 1.0, 8))]),
}


def _clear_seed(cfg, toks, dtype):
    """weights whose routers make no close call on the test's tokens (bfloat16 rounding must not turn a routing decision)"""
    for seed in range(3, 40):
        w = fo.random_weights(cfg, seed)
        if dtype == 'float32' or fo.router_gap(cfg, w, toks) >= 0.1:
            return seed
    raise AssertionError('no clear routing found')


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('name', list(ALONE))
def test_each_mechanism_alone(cuda, tmp_path, dtype, name):
    cfg = ALONE[name]()
    routed = dtype == 'bfloat16' and 'experts_top' in name      # (the fewer routing decisions, the likelier a seed without a close call)
    toks = np.random.default_rng(1).integers(0, 97, 40 if routed else 150).tolist()
    cut = len(toks) // 2
    folder, w = model_folder(tmp_path, cfg, _clear_seed(cfg, toks, dtype))
    ref_logits, trail = fo.forward(cfg, w, toks, True)
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
    cfg = full_model(dtype)
    folder, w = model_folder(tmp_path, cfg, 0)
    eng = engine(folder, dtype)
    toks = np.random.default_rng(1).integers(0, cfg['vocab'], 150).tolist()
    ref, trail = fo.forward(cfg, w, toks[:70], True)
    for n in range(1, len(cfg['layers']) + 1):                    # the residual stream behind every layer
        eng.stop_after(n)
        s = eng.open_session()
        eng.step_tokens([(s, toks[:70], [])])
        got = eng.fetch_residual(70)
        eng.close_session(s)
        assert np.abs(got - trail[n - 1]).max() <= TOL[dtype] * 3 * np.abs(trail[n - 1]).max(), n
    eng.stop_after(-1)
    ref = fo.forward(cfg, w, toks)
    s = eng.open_session()
    got = eng.step_tokens([(s, toks, list(range(len(toks))))])
    eng.close_session(s)
    assert rel_err(got, ref) <= TOL[dtype]
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_portions_decoding_batches_and_reuse(cuda, tmp_path, dtype):
    """every way of cutting the same requests gives the oracle's logits: token by token from the first token on, portions down to two
    tokens that start and end inside blocks and windows, unequal requests in one forward, and sessions that come and go in a pool that
    holds only what is live -- cache blocks and state slots are used again with other requests' keys and states still in them"""
    cfg = full_model(dtype)
    folder, w = model_folder(tmp_path, cfg, 1)
    rng = np.random.default_rng(2)
    reqs = [rng.integers(0, cfg['vocab'], n).tolist() for n in (200, 131, 65, 1, 23)]
    refs = [fo.forward(cfg, w, t) for t in reqs]
    eng = engine(folder, dtype, cache_blocks=9)
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
    assert rel_err(out, fo.forward(cfg, w, reqs[1] + [5])[-1:]) <= tol
    eng.close_session(b)
    eng.close()


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_engine_long_decoding_far_beyond_the_window(cuda, tmp_path, dtype):
    """420 tokens, the last 320 one at a time with the decode rows' keys split over several workgroups (session_len 1024 -> 4 splits): a
    window of 100 positions (edges inside blocks) with 4 kept tokens passes over decoded tokens, the states decay over hundreds of steps"""
    cfg = fo.make_config(64, 97, [fo.attention_layer(4, 2, 16, 8, 0.4, 100, 4, 8, 1000.0, 2.0, fo.moe(6, chosen(dtype, 2, 6), 32, 1.2, 16)),
                                  fo.lightning_layer(2, 8, 24, [0.995, 0.9], fo.dense(72)), fo.delta_layer(2, 12, 4)])
    folder, w = model_folder(tmp_path, cfg, 4)
    toks = np.random.default_rng(3).integers(0, 97, 420).tolist()
    ref = fo.forward(cfg, w, toks)
    eng = engine(folder, dtype, session_len=1024, cache_blocks=17, max_prefill_token_num=256)
    s = eng.open_session()
    eng.step_tokens([(s, toks[:100], [])])
    got = np.concatenate([eng.step_tokens([(s, [t], [0])]) for t in toks[100:]])
    eng.close_session(s)
    assert rel_err(got, ref[100:]) <= TOL[dtype]
    eng.close()


def test_state_of_a_far_token_survives_hundreds_of_steps(cuda, tmp_path):
    """a lightning layer whose decay is 1 - 2^-10 keeps a token from 300 positions back: moving that one token moves the last logits, in
    one portion and when everything after the first portion is decoded token by token"""
    cfg = fo.make_config(32, 53, [fo.lightning_layer(1, 16, 16, [1.0 - 2.0 ** -10])])
    folder, w = model_folder(tmp_path, cfg, 6)
    rng = np.random.default_rng(8)
    a = rng.integers(0, 53, 330).tolist()
    b = list(a)
    b[20] = (a[20] + 17) % 53
    ra, rb = fo.forward(cfg, w, a)[-1], fo.forward(cfg, w, b)[-1]
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


def _check_greedy(cfg, w, prompt, toks, min_margin=2e-2):     # (the sampler reads fp16 logits rows)
    ref, margins = fo.greedy(cfg, w, prompt, len(toks))
    for i, (a, b, m) in enumerate(zip(toks, ref, margins)):
        if m < min_margin:
            return          # a near-tie: from here on the two may legitimately part
        assert int(a) == b, (i, toks, ref)


def test_greedy_generation_static_batch_and_scheduler(cuda, tmp_path):
    cfg = full_model()
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
    cfg = full_model('bfloat16')
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
    """bin/trace_run end to end, both number formats: a width off the 8 grid, one expert per token, a window as long as a cache block,
    an attention layer without window or rotation; five requests in shared steps, pool of 640 tokens"""
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
        cfg = fo.make_config(100, 333, [fo.delta_layer(3, 20, 6, fo.moe(7, chosen(dtype, 1, 7), 40, 1.3, 12)),
                                        fo.attention_layer(10, 2, 8, 24, 0.35, 64, 2, 8, 20000.0, 16.0, fo.dense(72)),
                                        fo.lightning_layer(5, 12, 8, [0.7, 0.8, 0.9, 0.95, 0.99]),
                                        fo.attention_layer(5, 5, 24, 8, 0.3)])
        folder, w = model_folder(tmp_path, cfg, 11, 'model_' + dtype)
        ref = {n: fo.forward(cfg, w, t) for n, t in reqs.items()}
        out = str(tmp_path / dtype)
        p = subprocess.run([sys.executable, os.path.join(root, 'bin', 'trace_run'), '--model', folder, '--dtype', dtype, '--out', out,
                            '--max-tokens', '640'], input='\n'.join(steps) + '\n', text=True, capture_output=True, timeout=100)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.split('\n') if l.startswith('done')] == ['done %d' % i for i in range(len(plan))]
        for i, rr in enumerate(rows):
            got = np.fromfile(os.path.join(out, '%d.f32' % i), '<f4').reshape(len(rr), -1)
            assert rel_err(got, np.stack([ref[n][j] for n, j in rr])) <= tol, (dtype, i)
