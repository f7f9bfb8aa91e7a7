"""Host-side pieces around the ragged stack engine that need no GPU: the configuration reader and the registry, the
safetensors reader, the page / slot managers, the scheduler's step composition, and the oracle's own mechanisms against
closed forms."""
import json
import struct

import numpy as np
import pytest

from oracle import tolenex_oracle as O
from tolenex_cases import as_f64, attention_layer, hgrn2_layer, make_config, random_weights


def test_registry_picks_the_class_by_config():
    from tensorrt_llm.models import MODEL_REGISTRY, model_class_for, TolenexForCausalLM, LLaMAForCausalLM
    assert model_class_for({'architecture': 'Tolenex'}) is TolenexForCausalLM
    assert model_class_for({'architectures': ['LlamaForCausalLM']}) is LLaMAForCausalLM
    with pytest.raises(KeyError):
        model_class_for({'architecture': 'nothing'})
    assert 'Tolenex' in MODEL_REGISTRY


def test_config_reader_takes_every_size_from_the_file():
    from tensorrt_llm.models import TolenexConfig
    cfg = make_config([attention_layer(heads=10, kv_heads=5, dim=12, vdim=20, rot_dims=6, diff=0.125), hgrn2_layer(heads=7, dim=9, vdim=11, ff=33)],
                      width=140, vocab=1001, groups=7, eps=3e-6, emb_scale=2.5, loop=(1, 2, 5))
    c = TolenexConfig(cfg).engine_config()
    assert (c['width'], c['vocab'], c['norm_groups'], c['loop_start'], c['loop_stop'], c['loop_times']) == (140, 1001, 7, 1, 2, 5)
    assert float(c['norm_eps']) == 3e-6 and float(c['embedding_scale']) == 2.5
    assert (c['layer.0.heads'], c['layer.0.kv_heads'], c['layer.0.dim'], c['layer.0.vdim'], c['layer.0.rot_dims']) == (10, 5, 12, 20, 6)
    assert c['layer.0.maps'] == 2 and float(c['layer.0.diff']) == 0.125 and float(c['layer.0.rot_factor']) == 4.0
    assert (c['layer.1.type'], c['layer.1.heads'], c['layer.1.dim'], c['layer.1.vdim'], c['layer.1.ff']) == ('hgrn2', 7, 9, 11, 33)
    assert c['layer.0.ff'] == 136
    with pytest.raises(ValueError):
        TolenexConfig(make_config([{'type': 'conv', 'mixer': {}, 'mlp': None}]))


def test_safetensors_reader(tmp_path):
    from tensorrt_llm._utils import read_safetensors
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    bits = (a.view(np.uint32) >> 16).astype('<u2')
    tab = np.array([5, -2, 7], '<i4')
    header = {'x': {'dtype': 'BF16', 'shape': [3, 4], 'data_offsets': [0, 24]}, 't': {'dtype': 'I32', 'shape': [3], 'data_offsets': [24, 36]},
              '__metadata__': {'format': 'pt'}}
    h = json.dumps(header).encode()
    (tmp_path / 'm.safetensors').write_bytes(struct.pack('<Q', len(h)) + h + bits.tobytes() + tab.tobytes())
    t = read_safetensors(str(tmp_path / 'm.safetensors'))
    assert t['x'][1] == 'bfloat16' and ((t['x'][0].astype(np.uint32) << 16).view(np.float32) == a).all()
    assert t['t'][1] == 'int32' and t['t'][0].tolist() == [5, -2, 7]


def test_pages_are_taken_as_portions_come_and_given_back():
    from tensorrt_llm.runtime import GenerationSequence, KVCacheManager, StateSlotManager
    m = KVCacheManager(None, blocks=5, tokens_per_block=64, max_blocks_per_seq=5)
    a, b = GenerationSequence(0, 0), GenerationSequence(1, 1)
    m.reserve(a, 3)
    m.reserve(b, 64)
    m.reserve(a, 65)
    assert m.blocks_manager.block_ids(a) == [[0, 2]] and m.blocks_manager.block_ids(b) == [[1]]
    m.reserve(a, 128)
    assert m.blocks_manager.get_number_blocks(a) == 2 and m.blocks_manager.num_free_blocks() == 2
    with pytest.raises(RuntimeError):
        m.reserve(b, 64 * 3 + 1)
    assert m.blocks_manager.block_table([b, a], 3).tolist() == [[1, 0, 0], [0, 2, 0]]
    m.release(a)
    assert m.blocks_manager.num_free_blocks() == 4
    m.reserve(b, 64 * 4 + 1)  # the pages a gave back are used again
    assert sorted(m.blocks_manager.block_ids(b)[0]) == [0, 1, 2, 3, 4]
    s = StateSlotManager(2)
    assert (s.acquire(a), s.acquire(b), s.acquire(a)) == (0, 1, 0)
    with pytest.raises(RuntimeError):
        s.acquire(GenerationSequence(2, 2))
    s.release(a)
    assert s.acquire(GenerationSequence(2, 2)) == 0


def test_scheduler_fills_the_token_budget_and_never_overcommits():
    from tensorrt_llm.runtime import RaggedScheduler, Request
    sch = RaggedScheduler(max_batch_tokens=10, max_sequences=2, page_size=4, num_blocks=8)
    reqs = [Request(i, list(range(1, n + 1)), new) for i, (n, new) in enumerate(((13, 5), (2, 3), (6, 3)))]
    for r in reqs:
        sch.add(r)
    with pytest.raises(ValueError):
        sch.add(Request(9, [1] * 40, 3))
    trace, guard = [], 0
    while sch.has_work():
        plan = sch.schedule()
        assert plan and sum(n for _, n in plan) <= 10 and len(sch.running) <= 2
        assert sum(sch._committed.values()) <= 8
        trace.append([(r.rid, n) for r, n in plan])
        for r, n in plan:
            last = r.fed + n == len(r.prompt) + len(r.output)
            sch.update(r, n, 100 + len(r.output) if last else None)
        guard += 1
        assert guard < 50
    assert trace[0] == [(0, 10)]                       # the first prompt is cut by the budget
    assert trace[1] == [(0, 3), (1, 2)]                # its rest, then the next request's prompt in the same step
    assert trace[2][:2] == [(0, 1), (1, 1)]            # both decode
    assert all(r.finished and r.output == list(range(100, 100 + r.max_new_tokens)) for r in reqs)
    assert any((2, 6) in step and len(step) > 1 for step in trace)  # request 2 was admitted beside decoding ones


def test_oracle_norm_rotation_and_recurrence_against_closed_forms():
    x = np.array([[3.0, 4.0, 0.0, 5.0, 12.0, 0.0]])
    y = O.grouped_rms_norm(x, np.ones(6), 2, 0.0)
    assert np.allclose(y[0, :3], x[0, :3] / np.sqrt(25 / 3)) and np.allclose(y[0, 3:], x[0, 3:] / np.sqrt(169 / 3))
    # rotation: norm preserving without scaling, pair (1, 0) at position p turns to (cos, sin)
    rot = {'dims': 4, 'base': 100.0}
    v = np.zeros((3, 1, 6))
    v[:, 0, 0] = v[:, 0, 2] = v[:, 0, 5] = 1.0
    r = O.rotate_pairs(v, np.array([0, 1, 7]), rot)
    assert np.allclose(r[2, 0, :2], [np.cos(7.0), np.sin(7.0)]) and np.allclose(r[2, 0, 2:4], [np.cos(0.7), np.sin(0.7)])
    assert np.allclose(r[:, 0, 4:], v[:, 0, 4:]) and np.allclose(r[0], v[0])
    f, mult = O.rotary_frequencies({'dims': 8, 'base': 10000.0, 'scaling': {'factor': 4.0, 'original': 64, 'fast': 8.0, 'slow': 1.0}})
    plain = 10000.0 ** (-2.0 * np.arange(4) / 8)
    assert np.isclose(mult, 0.1 * np.log(4.0) + 1) and np.isclose(f[0], plain[0]) and np.isclose(f[-1], plain[-1] / 4)
    # recurrence with a constant gate: S_t = sum_j f^(t-j) (1 - f) v_j
    cfg = make_config([hgrn2_layer(heads=1, dim=2, vdim=3)], width=6, groups=1)
    w = as_f64(random_weights(cfg, 0))
    w['l0.mix.f'][:] = 0
    w['l0.mix.f.b'][:] = 0
    w['l0.mix.lower'][:] = 0.5            # f = 0.5 + 0.5 * sigmoid(0) = 0.75
    w['l0.mix.norm'][:] = 1
    w['l0.mix.o'] = np.eye(6)[:, :3]
    h = np.random.default_rng(0).standard_normal((5, 6))
    out = O.hgrn2_mixer(h, w, 'l0.', cfg['layers'][0]['mixer'], 0.0)
    z = h @ w['l0.mix.q'].T
    q, v = z / (1 + np.exp(-z)), h @ w['l0.mix.v'].T
    S = sum(0.75 ** (4 - j) * 0.25 * np.outer(np.ones(2), v[j]) for j in range(5))
    o = S.T @ q[4]
    assert np.allclose(out[4, :3], o / np.sqrt(np.mean(o * o)))


def test_oracle_attention_is_causal_and_differential():
    cfg = make_config([attention_layer(heads=2, kv_heads=1, dim=4, vdim=6, rot_dims=2, ff=0)], width=12, groups=1)
    w = as_f64(random_weights(cfg, 1))
    toks = [5, 9, 3, 7, 7, 2]
    a = O.tolenex_logits(toks, w, cfg)
    b = O.tolenex_logits(toks[:4] + [1, 1], w, cfg)
    assert np.allclose(a[:4], b[:4]) and not np.allclose(a[4:], b[4:])
    # equal maps and lambda = 1 would cancel: with lq/lk = 0 lambda is the constant diff
    for n in ('lq1', 'lk1', 'lq2', 'lk2'):
        w['l0.mix.' + n][:] = 0
    h = np.random.default_rng(2).standard_normal((3, 12))
    m = dict(cfg['layers'][0]['mixer'])
    wq = w['l0.mix.q'].reshape(2, 2, 4, 12)
    wq[:, 1] = wq[:, 0]
    wk = w['l0.mix.k'].reshape(1, 2, 4, 12)
    wk[:, 1] = wk[:, 0]
    w['l0.mix.o'] = np.eye(12)
    out = O.differential_attention(h, w, 'l0.', m, 0.0).reshape(3, 2, 6)
    # a1 == a2, so o = (1 - diff) a1 and the unit-RMS step leaves (1 - diff) * a1 / rms(a1)
    assert np.allclose(np.sqrt((out ** 2).mean(-1)), 1 - m['diff'])
