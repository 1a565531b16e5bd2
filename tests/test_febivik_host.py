"""Host tests of the Febivik design: the config reader (mixers, windows, rotation, routers, sizes taken from tensor shapes) against the
tests' own checkpoints, and hand cases of the float64 model the GPU tests compare the engine with."""
import numpy as np

from lmdeploy_amd.turbomind import layered
from tests import febivik_oracle as fo


def _cfg():
    return fo.make_config(48, 61, [fo.lightning_layer(3, 8, 12, [0.5, 0.9, 0.99], fo.dense(40)),
                                   fo.attention_layer(4, 2, 8, 16, 0.3, 10, 2, 4, 777.0, 4.0, fo.moe(4, 2, 24, 1.5, 32)),
                                   fo.delta_layer(2, 12, 5),
                                   fo.attention_layer(2, 2, 8, 8, 0.4, mlp=fo.moe(3, 3, 16))])


def test_reader_maps_every_constant():
    cfg = _cfg()
    mc = layered.FAMILIES['Febivik'](cfg, {'l2.mix.w1': (5, 48)})
    li, at, de, pl = mc.layers
    assert mc.final_layer_norm and all(s.post_norm and s.weights_of < 0 for s in mc.layers)
    assert (li.mixer, li.heads, li.kv_heads, li.dim, li.vdim, li.decay) == (layered.MIXER_LIGHTNING, 3, 3, 8, 12, (0.5, 0.9, 0.99))
    assert (li.mlp, li.ff, li.act) == (layered.MLP_DENSE, 40, layered.ACT_XIELU)
    assert (at.mixer, at.heads, at.kv_heads, at.dim, at.vdim, at.window, at.keep_first) == (layered.MIXER_ATTENTION, 4, 2, 8, 16, 10, 2)
    assert (at.rot_dims, at.rot_base, at.rot_scale, at.qkv_bias, at.qk_norm_w) == (4, 777.0, 4.0, True, True) and abs(at.scale - 0.3) < 1e-12
    assert (at.mlp, at.experts, at.top, at.ff, at.shared_ff, at.router_scale, at.expert_plain, at.router_softmax) == (layered.MLP_MOE, 4, 2, 24, 32, 1.5,
                                                                                                                   True, True)
    assert (de.mixer, de.heads, de.dim, de.vdim, de.decay_rank, de.mlp) == (layered.MIXER_DELTA, 2, 12, 12, 5, layered.MLP_NONE)
    assert (pl.window, pl.keep_first, pl.rot_dims, pl.rot_scale, pl.shared_ff, pl.router_scale) == (0, 0, 0, 1.0, 0, 1.0)


def test_decay_rank_is_the_tensor_s_own(tmp_path):
    cfg = _cfg()
    del cfg['layers'][2]['mixer']['decay_rank']
    w = fo.random_weights(cfg, 0)
    fo.write_checkpoint(str(tmp_path), cfg, w)
    mc = layered.read_layered_config(str(tmp_path))
    assert mc.layers[2].decay_rank == w['l2.mix.w1'].shape[0]
    assert {k: tuple(v) for k, v in mc.tensor_shapes().items()} == {k: tuple(np.shape(v)) for k, v in w.items()}
    assert layered.is_layered(str(tmp_path))


def test_visibility_is_window_or_first_tokens():
    assert [j for j in range(12) if fo.visible(11, j, 4, 2)] == [0, 1, 8, 9, 10, 11]
    assert [j for j in range(12) if fo.visible(3, j, 4, 2)] == [0, 1, 2, 3]
    assert [j for j in range(6) if fo.visible(5, j, 0, 3)] == [0, 1, 2, 3, 4, 5]
    assert not fo.visible(2, 3, 4, 2)


def test_xielu_hand_values():
    p, q = 0.3, -0.2
    a, b = np.log1p(np.exp(p)), 0.5 + np.log1p(np.exp(q))
    z = np.array([2.0, 0.0, -1.5])
    want = [a * 4 + 1.0, 0.0, b * (np.exp(-1.5) - 1 + 1.5) - 0.75]
    assert np.allclose(fo.xielu(z, p, q), want, atol=1e-12)


def test_rotation_pairs_channel_i_with_i_plus_half_and_leaves_the_rest():
    x = np.arange(1.0, 9.0).reshape(1, 1, 8)
    y = fo.rotate(x, [3], 4, 100.0, 2.0)
    f = np.array([1.0, 100.0 ** -0.5]) / 2.0
    c, s = np.cos(3 * f), np.sin(3 * f)
    assert np.allclose(y[0, 0, :2], x[0, 0, :2] * c - x[0, 0, 2:4] * s) and np.allclose(y[0, 0, 2:4], x[0, 0, 2:4] * c + x[0, 0, :2] * s)
    assert np.array_equal(y[0, 0, 4:], x[0, 0, 4:]) and np.array_equal(fo.rotate(x, [3], 0, 100.0, 1.0), x)


def test_lightning_recurrence_is_decayed_linear_attention():
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(9, 2, 3)), rng.normal(size=(9, 2, 3)), rng.normal(size=(9, 2, 5))
    lam = np.array([0.5, 0.9])
    o, S = fo.lightning_recurrence(q, k, v, lam)
    for h in range(2):
        for t in range(9):
            want = sum(lam[h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            assert np.allclose(o[t, h], want)
    o2a, S2 = fo.lightning_recurrence(q[:4], k[:4], v[:4], lam)
    o2b, S3 = fo.lightning_recurrence(q[4:], k[4:], v[4:], lam, S2)
    assert np.allclose(np.concatenate([o2a, o2b]), o) and np.allclose(S3, S)


def test_delta_recurrence_hand_cases():
    rng = np.random.default_rng(1)
    r, k, v = rng.normal(size=(6, 1, 4)), rng.normal(size=(6, 1, 4)), rng.normal(size=(6, 1, 4))
    one, zero = np.ones((6, 1, 4)), np.zeros((6, 1, 4))
    o, S = fo.delta_recurrence(r, k, v, one, zero)                      # no decay, nothing removed: a plain sum of outer products
    assert np.allclose(S[0], sum(np.outer(k[t, 0], v[t, 0]) for t in range(6)))
    # full removal along the unit key: what the old state answered to u is gone before the new pair is written
    o, S1 = fo.delta_recurrence(r[:1], k[:1], v[:1], one[:1], zero[:1])
    o, S2 = fo.delta_recurrence(r[1:2], k[1:2], v[1:2], one[:1], one[:1], S1)
    u = k[1, 0] / np.sqrt((k[1, 0] ** 2).sum() + 1e-6)
    assert np.allclose(u @ (S2[0] - np.outer(k[1, 0], v[1, 0])), 0.0, atol=1e-5)


def test_router_takes_the_largest_scores_unrenormalised():
    h = np.array([[1.0, 0.0], [0.0, 2.0]])
    wr = np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]])
    idx, sc = fo.route(h, wr, 2)
    z = h @ wr.T
    s = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    assert idx.tolist() == [[0, 2], [1, 2]] and np.allclose(sc, [[s[0, 0], s[0, 2]], [s[1, 1], s[1, 2]]]) and sc.sum(-1).max() < 1.0


def test_a_block_adds_the_normed_sublayer_result():
    cfg = fo.make_config(16, 11, [fo.lightning_layer(1, 4, 4, [0.9])])
    w = fo.random_weights(cfg, 0)
    toks = [1, 5, 3]
    _, trail = fo.forward(cfg, w, toks, True)
    x = w['embed'][toks]
    y = fo.lightning_mixer(x, cfg['layers'][0]['mixer'], w, 'l0.mix.', 1e-5)
    assert np.allclose(trail[0], x + fo.layer_norm(y, w['l0.norm1'], w['l0.norm1.b'], 1e-5))
