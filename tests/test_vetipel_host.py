"""Host-side pieces of the Vetipel design that need no GPU: the configuration reader and the registry, the random-weight maker's
tensor list, and the oracle's own mechanisms against closed forms and against a second way of computing them."""
import numpy as np
import pytest

from oracle import vetipel_oracle as O
from tolenex_cases import as_f64
from vetipel_cases import chunk_layer, latent_layer, make_config, random_weights, window_layer


def test_registry_picks_the_class_by_config():
    from tensorrt_llm.models import MODEL_REGISTRY, VetipelForCausalLM, model_class_for
    assert model_class_for({'architecture': 'Vetipel'}) is VetipelForCausalLM
    assert 'Vetipel' in MODEL_REGISTRY and 'Tolenex' in MODEL_REGISTRY


def test_config_reader_takes_every_size_from_the_file():
    from tensorrt_llm.models import VetipelConfig
    cfg = make_config([window_layer(heads=10, kv_heads=5, dim=12, vdim=20, size=77, ff=33),
                       latent_layer(heads=7, dim=10, rot_dim=6, vdim=14, kv_rank=50, base=123.0, dims=4, ff=0),
                       chunk_layer(heads=9, kv_heads=3, dim=18, vdim=22, size=41, ff=55)], width=140, vocab=1001, streams=4, eps=3e-6,
                      emb_scale=2.5)
    c = VetipelConfig(cfg).engine_config()
    assert (c['width'], c['vocab'], c['streams'], c['block'], c['residual']) == (140, 1001, 4, 'sequential', 'hyper')
    assert float(c['norm_eps']) == 3e-6 and float(c['embedding_scale']) == 2.5 and float(c['norm_offset']) == 1.0
    assert (c['layer.0.type'], c['layer.0.heads'], c['layer.0.kv_heads'], c['layer.0.dim'], c['layer.0.vdim']) == ('attention', 10, 5, 12, 20)
    assert (c['layer.0.mask'], c['layer.0.mask_size'], c['layer.0.weights'], c['layer.0.pos_bias'], c['layer.0.ff']) == ('window', 77, 'sigmoid', 'linear', 33)
    assert (c['layer.1.type'], c['layer.1.kv_rank'], c['layer.1.rot_dim'], c['layer.1.rot_dims'], c['layer.1.ff']) == ('latent_attention', 50, 6, 4, 0)
    assert float(c['layer.1.rot_base']) == 123.0
    assert (c['layer.2.mask'], c['layer.2.mask_size'], c['layer.2.sink'], c['layer.2.qk_norm'], c['layer.2.qkv_bias'], c['layer.2.pos_bias']) == ('chunk', 41, 1, 1, 1, 'log')
    assert all(c[f'layer.{i}.mlp'] == 'relu2' for i in range(3))
    assert VetipelConfig(make_config([window_layer()], streams=0)).engine_config()['streams'] == 1
    with pytest.raises(ValueError):
        VetipelConfig(make_config([{'type': 'hgrn2', 'mixer': {}, 'mlp': None}]))


def test_random_weight_maker_names_what_the_tests_generator_names():
    """Two generators written apart (the product's, for benchmarks; the tests') must agree on names and shapes."""
    from tensorrt_llm.models import VetipelForCausalLM
    for streams in (0, 1, 3):
        cfg = make_config([window_layer(), latent_layer(ff=0), chunk_layer(ff=24)], streams=streams)
        ours = random_weights(cfg, 1)
        theirs = VetipelForCausalLM.from_random(cfg, seed=2).tensors
        assert {k: v.shape for k, v in ours.items()} == {k: a.shape for k, (a, _) in theirs.items()}


def test_mask_shapes():
    assert O.visible(5, 'window', 2).sum(axis=1).tolist() == [1, 2, 2, 2, 2]
    assert O.visible(7, 'chunk', 3).sum(axis=1).tolist() == [1, 2, 3, 1, 2, 3, 1]
    assert O.visible(4, 'causal', 0).sum(axis=1).tolist() == [1, 2, 3, 4]
    assert not O.visible(9, 'window', 4)[8, 4] and O.visible(9, 'window', 4)[8, 5]
    assert not O.visible(9, 'chunk', 4)[8, 7] and O.visible(9, 'chunk', 4)[7, 4]


def test_a_sink_takes_its_share_and_brings_nothing():
    """One token: the only key is the token itself, so the head's output is v * e^s / (e^s + e^sink) * gate."""
    cfg = make_config([chunk_layer(heads=2, kv_heads=1, dim=4, vdim=3, size=5)], width=8, vocab=11)
    w = as_f64(random_weights(cfg, 3))
    m, eps, p = cfg['layers'][0]['mixer'], cfg['norm']['eps'], 'l0.mix.'
    h = np.random.default_rng(0).standard_normal((1, 8))
    q = O.unit_rms((h @ w[p + 'q'].T + w[p + 'q.b']).reshape(2, 4), eps)
    k = O.unit_rms((h @ w[p + 'k'].T + w[p + 'k.b']).reshape(1, 4), eps)
    v = (h @ w[p + 'v'].T + w[p + 'v.b']).reshape(3)
    heads = []
    for a in range(2):
        s = q[a] @ k[0] * m['scale'] * w[p + 'temp'][a]                      # distance 0: the penalty is r1 ln 1 = 0
        heads.append(v * np.exp(s) / (np.exp(s) + np.exp(w[p + 'sink'][a])) * O.sigmoid(h[0] @ w[p + 'g'][a]))
    want = np.concatenate(heads) @ w[p + 'o'].T
    assert np.allclose(O.sink_chunk_attention(h, w, p, m, eps)[0], want, rtol=1e-12, atol=1e-12)


def test_sigmoid_weights_are_not_normalised():
    """Equal tokens inside the window: every key has the same value, so the output grows with the number of visible keys."""
    cfg = make_config([window_layer(heads=1, kv_heads=1, dim=4, vdim=3, size=3, ff=0)], width=8, vocab=11)
    w = as_f64(random_weights(cfg, 4))
    m, p = cfg['layers'][0]['mixer'], 'l0.mix.'
    h = np.tile(np.random.default_rng(1).standard_normal((1, 8)), (5, 1))
    q, k, v = h[0] @ w[p + 'q'].T, h[0] @ w[p + 'k'].T, h[0] @ w[p + 'v'].T
    slope = 2.0 ** -8.0
    wt = [O.sigmoid(q @ k * m['scale'] - slope * d + w[p + 'pb'][0]) for d in range(3)]
    gate = O.sigmoid(h[0] @ w[p + 'g'][0])
    out = O.sigmoid_window_attention(h, w, p, m)
    for i, n_keys in enumerate([1, 2, 3, 3, 3]):
        assert np.allclose(out[i], (sum(wt[:n_keys]) * v * gate) @ w[p + 'o'].T, rtol=1e-12, atol=1e-12)


def test_latent_attention_equals_its_absorbed_form():
    """Scores through W_uk^T q against the latent, values expanded after the weighted sum of latents: the same function."""
    cfg = make_config([latent_layer(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=10, dims=2, ff=0)], width=16, vocab=11)
    w = as_f64(random_weights(cfg, 5))
    m, eps, p = cfg['layers'][0]['mixer'], cfg['norm']['eps'], 'l0.mix.'
    n, H, D, R, E, C = 9, 3, 6, 4, 5, 10
    h = np.random.default_rng(2).standard_normal((n, 16))
    pos = np.arange(n)
    q = (h @ w[p + 'q'].T).reshape(n, H, D + R)
    down = h @ w[p + 'dkv'].T
    c = O.offset_rms_norm(down[:, :C], w[p + 'dkv.norm'], eps, offset=0.0)
    k_rot = O.rotate_pairs(down[:, C:], pos, 2, m['rot']['base'])
    q_rot = O.rotate_pairs(q[..., D:], pos, 2, m['rot']['base'])
    out = np.zeros((n, H, E))
    for a in range(H):
        q_abs = q[:, a, :D] @ w[p + 'uk'][a * D:(a + 1) * D]                   # [n, C]
        s = (q_abs @ c.T + q_rot[:, a] @ k_rot.T) * m['scale']
        s = np.where(np.tril(np.ones((n, n), bool)), s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, a] = ((e / e.sum(axis=1, keepdims=True)) @ c) @ w[p + 'uv'][a * E:(a + 1) * E].T
    assert np.allclose(O.latent_attention(h, w, p, m, eps), out.reshape(n, H * E) @ w[p + 'o'].T, rtol=1e-10, atol=1e-12)


def test_hyper_connections_with_unit_weights_are_the_plain_residual():
    cfg = make_config([window_layer(ff=24), chunk_layer(ff=0)], streams=1)
    w = random_weights(cfg, 6)
    for k in list(w):
        if '.hc' in k:
            w[k] = np.ones_like(w[k])
    toks = [1, 5, 9, 2, 2, 7]
    plain = dict(cfg)
    del plain['streams']
    assert np.allclose(O.logits(toks, as_f64(w), cfg), O.logits(toks, as_f64(w), plain), rtol=1e-12, atol=1e-12)


def test_streams_mix_from_to():
    """mix[s, t] carries stream s into stream t: with out = 0 a sublayer only permutes and scales the streams."""
    xs = np.arange(6, dtype=np.float64).reshape(3, 1, 2) + 1.0
    w = {'hc.in': np.array([1.0, 0.0, 0.0]), 'hc.out': np.zeros(3), 'hc.mix': np.array([[0, 2.0, 0], [0, 0, 1.0], [1.0, 0, 0]])}
    new = O.hyper_sublayer(xs, lambda u: u * 100.0, w, 'hc.')
    assert np.allclose(new[1], 2.0 * xs[0]) and np.allclose(new[2], xs[1]) and np.allclose(new[0], xs[2])
