"""Tolenex through the ragged stack engine against the plain float64 oracle (oracle/tolenex_oracle.py), on small
configurations and random weights made here.  fp32 engine: tight bound (what summation order can explain); bfloat16
engine: loose bound, and crafted weights where random ones would hide a fault."""
import json
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

from oracle import tolenex_oracle as O
from tolenex_cases import (as_f64, as_model, attention_layer, hgrn2_layer, make_config, random_weights, rel_err, replay)

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 3e-5, 5e-2


def session_for(cfg, w, dtype='float32', max_tokens=1024, max_sequences=4, **kw):
    from tensorrt_llm.runtime import RaggedGenerationSession
    return RaggedGenerationSession(as_model(cfg, w), dtype=dtype, max_tokens=max_tokens, max_sequences=max_sequences, **kw)


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg['vocab'], n).tolist()


def check(got, want, tol, what=''):
    e = rel_err(got, want)
    assert np.isfinite(got).all(), what
    assert e.max() < tol, f'{what}: worst row {int(e.argmax())} of {len(e)} has relative error {e.max():.3g} (bound {tol})'


FULL = [attention_layer(), hgrn2_layer(ff=72), attention_layer(heads=4, kv_heads=4, dim=24, vdim=16, rot_dims=24, ff=0),
        hgrn2_layer(heads=3, dim=16, vdim=32, ff=40), attention_layer(kv_heads=1, rot_dims=0, softcap=0.0)]

# shapes the MFMA tile kernel takes in bfloat16 (dim and vdim of 32 / 64 / 128); fp32 runs them on the general kernel
TILED = [attention_layer(heads=6, kv_heads=2, dim=32, vdim=32, rot_dims=16), hgrn2_layer(heads=2, dim=32, vdim=64, ff=72),
         attention_layer(heads=2, kv_heads=1, dim=64, vdim=128, rot_dims=64, ff=0), attention_layer(heads=3, kv_heads=3, dim=32, vdim=64, rot_dims=0)]
STACKS = {'general': FULL, 'tiled': TILED}

MECHANISMS = {
    'attention_alone_no_ff': make_config([attention_layer(ff=0)]),
    'attention_one_group': make_config([attention_layer()], groups=1),
    'attention_full_rotation_no_scaling': make_config([attention_layer(rot_dims=16, scaling=False)]),
    'attention_no_rotation_no_cap': make_config([attention_layer(rot_dims=0, softcap=0.0)]),
    'attention_every_head_its_own_kv': make_config([attention_layer(heads=4, kv_heads=4)]),
    'attention_one_kv_head_odd_sizes': make_config([attention_layer(heads=5, kv_heads=1, dim=12, vdim=20, rot_dims=4)], width=80, groups=5),
    'attention_tile_32_32': make_config([TILED[0]]),
    'attention_tile_64_128': make_config([TILED[2]]),
    'attention_tile_128_64_one_map_group': make_config([attention_layer(heads=2, kv_heads=2, dim=128, vdim=64, rot_dims=32, softcap=0.0)]),
    'tiled_stack_looped': make_config(TILED, loop=(1, 3, 2), groups=2),
    'attention_wide_values': make_config([attention_layer(heads=2, kv_heads=1, dim=8, vdim=160)]),
    'hgrn2_alone_no_ff': make_config([hgrn2_layer()]),
    'hgrn2_small_heads': make_config([hgrn2_layer(heads=4, dim=8, vdim=8, ff=48)], groups=2),
    'hgrn2_wide': make_config([hgrn2_layer(heads=1, dim=72, vdim=136)]),
    'hgrn2_wider_than_a_workgroup': make_config([hgrn2_layer(heads=1, dim=40, vdim=320)]),
    'hgrn2_long_keys': make_config([hgrn2_layer(heads=2, dim=200, vdim=48)]),
    'rows_that_are_not_16_byte_multiples': make_config([attention_layer(heads=3, kv_heads=1, dim=10, vdim=14, rot_dims=6, ff=50), hgrn2_layer(heads=3, dim=6, vdim=10, ff=34)],
                                                       width=76, vocab=131, groups=19),
    'loop_three_passes': make_config(FULL[:3], loop=(0, 2, 3)),
    'loop_one_pass': make_config(FULL[:3], loop=(1, 3, 1)),
    'loop_whole_stack': make_config(FULL[:2], loop=(0, 2, 2), emb_scale=1.0),
    'no_loop_five_layers': make_config(FULL),
    'loop_in_the_middle': make_config(FULL, loop=(1, 4, 2), groups=4),
}


@pytest.mark.parametrize('name', sorted(MECHANISMS))
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_each_mechanism_whole_prompt(name, dtype):
    cfg = MECHANISMS[name]
    w = random_weights(cfg, seed=len(name))
    toks = tokens_for(cfg, 70, 1)  # crosses a page border
    want = O.tolenex_logits(toks, as_f64(w), cfg)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', len(toks))]])['a']
    check(got, want, F32_TOL if dtype == 'float32' else BF16_TOL, name)


def test_residual_stream_behind_every_layer_run():
    cfg = MECHANISMS['loop_in_the_middle']
    w = random_weights(cfg, seed=3)
    toks = tokens_for(cfg, 19, 2)
    res = []
    O.tolenex_logits(toks, as_f64(w), cfg, residuals=res)
    s = session_for(cfg, w, 'float32', debug_mode=True)
    s.step([('a', toks, [0])])
    assert s.engine.layer_runs == len(res) == 1 + 3 * 2 + 1
    for j, x in enumerate(res):
        assert np.abs(s.engine.tap(j) - x).max() < 2e-4 * np.abs(x).max(), f'layer run {j}'


@pytest.mark.parametrize('stack', sorted(STACKS))
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_prefill_then_token_by_token(dtype, stack):
    cfg = make_config(STACKS[stack], loop=(1, 4, 2), groups=4)
    w = random_weights(cfg, seed=5)
    toks = tokens_for(cfg, 150, 3)
    want = O.tolenex_logits(toks, as_f64(w), cfg)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', 100)]] + [[('a', 1)]] * 50)['a']
    check(got, want, F32_TOL if dtype == 'float32' else BF16_TOL)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('sizes', [[2] * 40, [3, 61, 2, 64, 1, 5, 2, 58, 1, 1, 2], [63, 2, 63, 1, 1, 66], [1] * 9 + [120, 2]])
@pytest.mark.parametrize('stack', sorted(STACKS))
def test_portions_of_a_prompt(sizes, dtype, stack):
    cfg = make_config(STACKS[stack], loop=(0, 4, 2))
    w = random_weights(cfg, seed=7)
    toks = tokens_for(cfg, sum(sizes), 4)
    want = O.tolenex_logits(toks, as_f64(w), cfg)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', n)] for n in sizes])['a']
    check(got, want, F32_TOL if dtype == 'float32' else BF16_TOL)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('stack', sorted(STACKS))
def test_unequal_requests_in_one_batch_equal_each_alone(dtype, stack):
    cfg = make_config(STACKS[stack], loop=(1, 3, 2))
    w = random_weights(cfg, seed=9)
    reqs = {'a': tokens_for(cfg, 131, 5), 'b': tokens_for(cfg, 9, 6), 'c': tokens_for(cfg, 66, 7), 'd': tokens_for(cfg, 2, 8)}
    schedule = [[('a', 60), ('b', 2)], [('b', 1), ('a', 5), ('c', 64)], [('c', 1), ('b', 1), ('a', 1), ('d', 2)],
                [('a', 63), ('b', 5), ('c', 1)], [('a', 1)], [('a', 1)]]
    s = session_for(cfg, w, dtype)
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check(got[rid], O.tolenex_logits(toks, as_f64(w), cfg), F32_TOL if dtype == 'float32' else BF16_TOL, rid)
    assert not s.live() and s.cache.blocks_manager.num_free_blocks() == s.num_blocks and s.slots.num_free_slots() == 4


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_requests_of_very_unequal_length_decode_side_by_side(dtype):
    """Steps of decoded tokens only, one request far ahead of the others: the keys of the long one are walked by several
    workgroups whose share of a short request is empty."""
    cfg = make_config([TILED[0], TILED[2], hgrn2_layer(heads=2, dim=32, vdim=64, ff=40)], loop=(0, 2, 2))
    w = random_weights(cfg, seed=21)
    reqs = {'long': tokens_for(cfg, 620, 90), 'mid': tokens_for(cfg, 75, 91), 'new': tokens_for(cfg, 12, 92)}
    schedule = [[('long', 600)], [('mid', 65), ('long', 1)]] + [[('long', 1), ('mid', 1), ('new', 1)]] * 10 + [[('long', 9), ('new', 2)]]
    s = session_for(cfg, w, dtype, max_tokens=1024)
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check(got[rid], O.tolenex_logits(toks, as_f64(w), cfg), F32_TOL if dtype == 'float32' else BF16_TOL, rid)


def test_pages_and_slots_that_are_used_again():
    """A pool of 4 pages and 2 slots serves six requests one after another and side by side: every page and slot is written by
    several requests, and a recurrent state must start from zero in a slot another request has left."""
    cfg = make_config([attention_layer(ff=0), hgrn2_layer(ff=40)], loop=(0, 2, 2))
    w = random_weights(cfg, seed=11)
    s = session_for(cfg, w, 'float32', max_tokens=256, max_sequences=2)
    assert s.num_blocks == 4
    used_blocks, used_slots = [], []
    for rnd in range(3):
        reqs = {f'x{rnd}': tokens_for(cfg, 100 + rnd, 20 + rnd), f'y{rnd}': tokens_for(cfg, 70 - rnd, 30 + rnd)}
        x, y = f'x{rnd}', f'y{rnd}'
        schedule = [[(x, 50), (y, 3)], [(y, len(reqs[y]) - 3), (x, 1)], [(x, len(reqs[x]) - 51)]]
        at = {}
        got = {r: [] for r in reqs}
        for step in schedule:
            entries = []
            for rid, n in step:
                lo = at.get(rid, 0)
                entries.append((rid, reqs[rid][lo:lo + n], list(range(n))))
                at[rid] = lo + n
            logits, _ = s.step(entries)
            k = 0
            for rid, n in step:
                got[rid].append(logits[k:k + n])
                k += n
        for rid in reqs:
            seq = s._seq[rid]
            used_blocks.append(tuple(s.cache.blocks_manager.block_ids(seq)[0]))
            used_slots.append(s.slots.slot_of(seq))
            check(np.concatenate(got[rid]), O.tolenex_logits(reqs[rid], as_f64(w), cfg), F32_TOL, rid)
            s.release(rid)
    assert len(set(used_slots)) == 2 and len(used_slots) == 6
    assert len({b for blocks in used_blocks for b in blocks}) == 4 and sum(len(b) for b in used_blocks) == 12


def test_pool_exhaustion_is_an_error_not_a_fault():
    cfg = make_config([attention_layer(ff=0)])
    s = session_for(cfg, random_weights(cfg, 1), 'float32', max_tokens=128, max_sequences=2)
    s.step([('a', tokens_for(cfg, 60, 1), [])])
    with pytest.raises(RuntimeError, match='block'):
        s.step([('b', tokens_for(cfg, 65, 2), [])])
    s.release('b')
    s.step([('c', tokens_for(cfg, 3, 2), [0])])
    with pytest.raises(RuntimeError, match='slot'):
        s.step([('d', [1], [0])])


def _far_key_case(p_far, n, seed, D=16):
    """One attention layer whose head 0, map 0 is rigged so that the LAST token's query meets the key of the token at p_far with
    a score far above all others (a bump on a dimension the rotation leaves alone): dropping, shifting or corrupting that one
    far key changes the logits at the last position by much more than bfloat16 rounding."""
    cfg = make_config([attention_layer(heads=2, kv_heads=1, dim=D, vdim=24 if D == 16 else 64, rot_dims=8, ff=0, softcap=60.0)], groups=2)
    w = random_weights(cfg, seed=seed)
    rng = np.random.default_rng(seed)
    far_tok, last_tok = 3, 4
    toks = [int(t) for t in rng.integers(5, cfg['vocab'], n)]
    toks[p_far], toks[-1] = far_tok, last_tok
    wf = as_f64(w)
    h = O.grouped_rms_norm(wf['embed'] * cfg['embedding']['scale'], wf['l0.norm1'], cfg['norm']['groups'], cfg['norm']['eps'])
    alpha = (30.0 / cfg['layers'][0]['mixer']['scale']) ** 0.5
    from tolenex_cases import bf16_round
    w['l0.mix.q'][0 * D + D - 1] = bf16_round((alpha * h[last_tok] / (h[last_tok] @ h[last_tok])).astype(np.float32))
    w['l0.mix.k'][0 * D + D - 1] = bf16_round((alpha * h[far_tok] / (h[far_tok] @ h[far_tok])).astype(np.float32))
    return cfg, w, toks


@pytest.mark.parametrize('p_far', [0, 1, 31, 32, 63, 64, 127, 128, 200])
@pytest.mark.parametrize('dtype,D', [('float32', 16), ('bfloat16', 16), ('bfloat16', 32)])
def test_a_far_key_that_decides_the_answer(p_far, dtype, D):
    n = 333
    cfg, w, toks = _far_key_case(p_far, n, seed=40 + p_far, D=D)
    wf = as_f64(w)
    want = O.tolenex_logits(toks, wf, cfg)
    other = list(toks)
    other[p_far] = 7
    moved = rel_err(O.tolenex_logits(other, wf, cfg)[-1:], want[-1:])[0]
    assert moved > 0.1, f'the rig does not bite: replacing the far token moves the last row by {moved:.3g} only'
    tol = F32_TOL if dtype == 'float32' else BF16_TOL
    s = session_for(cfg, w, dtype)
    # in a whole prompt, in a portion that starts behind the far key, and decoded alone
    check(replay(s, {'w': toks}, [[('w', n)]])['w'][-1:], want[-1:], tol, 'whole')
    check(replay(s, {'p': toks}, [[('p', p_far + 1)], [('p', n - p_far - 1)]])['p'][-1:], want[-1:], tol, 'portion')
    check(replay(s, {'d': toks}, [[('d', n - 1)], [('d', 1)]])['d'][-1:], want[-1:], tol, 'decoded')


def test_first_tokens_of_a_sequence():
    cfg = MECHANISMS['loop_in_the_middle']
    w = random_weights(cfg, seed=13)
    s = session_for(cfg, w, 'float32')
    for n in (1, 2, 3):
        toks = tokens_for(cfg, n, 50 + n)
        check(replay(s, {n: toks}, [[(n, n)]])[n], O.tolenex_logits(toks, as_f64(w), cfg), F32_TOL, f'{n} tokens at once')
        check(replay(s, {-n: toks}, [[(-n, 1)]] * n)[-n], O.tolenex_logits(toks, as_f64(w), cfg), F32_TOL, f'{n} tokens one by one')


@pytest.mark.parametrize('stack', sorted(STACKS))
def test_long_decoding(stack):
    cfg = make_config([STACKS[stack][0], hgrn2_layer(ff=40)], loop=(0, 2, 2))
    w = random_weights(cfg, seed=15)
    toks = tokens_for(cfg, 330, 9)
    want = O.tolenex_logits(toks, as_f64(w), cfg)
    for dtype, tol in (('float32', F32_TOL), ('bfloat16', BF16_TOL)):
        s = session_for(cfg, w, dtype)
        check(replay(s, {'a': toks}, [[('a', 2)]] + [[('a', 1)]] * 328)['a'], want, tol, dtype)


def test_greedy_generation_through_the_scheduler():
    """Six prompts, four state slots, 40 tokens per step: prompts are cut, requests queue, decoded tokens share steps with prompt
    portions.  fp32 engine against the oracle's greedy continuation (recomputed from scratch for every token)."""
    from tensorrt_llm.runtime import SamplingConfig
    cfg = make_config([attention_layer(ff=48), hgrn2_layer(heads=2, dim=16, vdim=16, ff=0)], width=64, vocab=97, groups=2, loop=(0, 2, 2))
    w = random_weights(cfg, seed=17)
    prompts = [tokens_for(cfg, n, 60 + n) for n in (70, 3, 45, 1, 90, 17)]
    s = session_for(cfg, w, 'float32', max_tokens=512, max_sequences=4, max_batch_tokens=40)
    outs = s.decode_batch(prompts, SamplingConfig(end_id=-1, pad_id=0), max_new_tokens=6)
    for p, o in zip(prompts, outs):
        assert o.tolist() == O.greedy(p, as_f64(w), cfg, 6)
    assert not s.live() and s.cache.blocks_manager.num_free_blocks() == s.num_blocks
    # the rectangular entry point, with an end token that stops one request early
    stop = int(outs[1][2])
    ids = np.zeros((2, 45), np.int32)
    ids[0, :3], ids[1, :45] = prompts[1], prompts[2]
    full = s.decode(ids, np.array([3, 45], np.int32), SamplingConfig(end_id=stop, pad_id=0), max_new_tokens=6)
    assert full.shape == (2, 1, 51) and full[0, 0, 45:48].tolist() == outs[1][:3].tolist() and (full[0, 0, 48:] == 0).all()


def write_checkpoint(path, cfg, w):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, 'config.json'), 'w') as f:
        json.dump(cfg, f)
    header, blobs, at = {}, [], 0
    for name, a in w.items():
        b = (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype('<u2').tobytes()
        header[name] = {'dtype': 'BF16', 'shape': list(a.shape), 'data_offsets': [at, at + len(b)]}
        blobs.append(b)
        at += len(b)
    h = json.dumps(header).encode()
    with open(os.path.join(path, 'model.safetensors'), 'wb') as f:
        f.write(struct.pack('<Q', len(h)) + h + b''.join(blobs))


def test_command_lines(tmp_path):
    """examples/tolenex/run.py generates from a checkpoint directory; bin/trace_run replays a recorded schedule from it."""
    cfg = make_config([attention_layer(ff=48), hgrn2_layer(heads=2, dim=16, vdim=16, ff=0)], width=64, vocab=97, groups=2)
    w = random_weights(cfg, seed=19)
    ck = str(tmp_path / 'ck')
    write_checkpoint(ck, cfg, w)
    prompt = tokens_for(cfg, 21, 70)
    np.save(tmp_path / 'in.npy', np.asarray(prompt, np.int32))
    run = os.path.join(ROOT, 'trtllm-llama_amd', 'examples', 'tolenex', 'run.py')
    subprocess.run([sys.executable, run, '--model_dir', ck, '--dtype', 'float32', '--input_tokens', str(tmp_path / 'in.npy'),
                    '--max_output_len', '5', '--output_npy', str(tmp_path / 'out.npy')], check=True, timeout=300)
    assert np.load(tmp_path / 'out.npy').reshape(-1)[len(prompt):].tolist() == O.greedy(prompt, as_f64(w), cfg, 5)
    # the trace runner
    a, b = tokens_for(cfg, 70, 71), tokens_for(cfg, 5, 72)
    steps = [{'step': 0, 'entries': [{'id': 'a', 'tokens': a[:66], 'want': [0, 65]}, {'id': 'b', 'tokens': b[:2], 'want': []}], 'end': []},
             {'step': 1, 'entries': [{'id': 'b', 'tokens': b[2:], 'want': [2]}], 'end': ['b']},
             {'step': 2, 'entries': [{'id': 'a', 'tokens': a[66:], 'want': [3]}], 'end': ['a']}]
    out = tmp_path / 'logits'
    r = subprocess.run([os.path.join(ROOT, 'bin', 'trace_run'), '--model', ck, '--dtype', 'float32', '--out', str(out), '--max-tokens', '192'],
                       input='\n'.join(json.dumps(s) for s in steps) + '\n', capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith('done')] == ['done 0', 'done 1', 'done 2']
    la, lb = O.tolenex_logits(a, as_f64(w), cfg), O.tolenex_logits(b, as_f64(w), cfg)
    got0 = np.fromfile(out / '0.f32', '<f4').reshape(2, -1)
    check(got0, la[[0, 65]], F32_TOL)
    check(np.fromfile(out / '1.f32', '<f4').reshape(1, -1), lb[[4]], F32_TOL)
    check(np.fromfile(out / '2.f32', '<f4').reshape(1, -1), la[[69]], F32_TOL)
