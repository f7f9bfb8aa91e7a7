"""Vetipel through the ragged stack engine against the plain float64 oracle (oracle/vetipel_oracle.py), on small configurations and
random weights made here.  fp32 engine: tight bound (what summation order can explain); bfloat16 engine: loose bound, and crafted
weights where random ones would hide a fault (a key at a window's or a chunk's edge, one far key among hundreds)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from oracle import vetipel_oracle as O
from tolenex_cases import as_f64, bf16_round, rel_err, replay
from vetipel_cases import as_model, chunk_layer, latent_layer, make_config, random_weights, window_layer

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


def tol_of(dtype):
    return F32_TOL if dtype == 'float32' else BF16_TOL


FULL = [window_layer(), latent_layer(), chunk_layer(ff=40), chunk_layer(heads=3, kv_heads=3, dim=8, vdim=40, size=64, ff=0),
        window_layer(heads=2, kv_heads=1, dim=24, vdim=8, size=64, ff=0), latent_layer(heads=1, dim=8, rot_dim=12, vdim=16, kv_rank=24, dims=4)]
# shapes the MFMA tile kernels take in bfloat16; fp32 runs them on the general kernel
TILED = [window_layer(heads=4, kv_heads=2, dim=32, vdim=64, size=45), latent_layer(heads=2, dim=32, rot_dim=32, vdim=32, kv_rank=128),
         chunk_layer(heads=2, kv_heads=1, dim=64, vdim=32, size=50, ff=72), window_layer(heads=2, kv_heads=2, dim=128, vdim=128, size=130, ff=0)]
STACKS = {'general': FULL, 'tiled': TILED}

MECHANISMS = {
    'window_alone_no_ff': make_config([window_layer(ff=0)]),
    'window_of_one': make_config([window_layer(size=1)]),
    'window_two': make_config([window_layer(size=2, ff=0)], streams=1),
    'window_a_page': make_config([window_layer(size=64)]),
    'window_wider_than_the_prompt': make_config([window_layer(size=500)]),
    'window_every_head_its_own_kv': make_config([window_layer(heads=4, kv_heads=4)]),
    'window_one_kv_head_odd_sizes': make_config([window_layer(heads=5, kv_heads=1, dim=12, vdim=20, size=33)], width=80),
    'window_tile_32_64': make_config([TILED[0]]),
    'window_tile_128_128': make_config([TILED[3]]),
    'latent_alone_no_ff': make_config([latent_layer(ff=0)]),
    'latent_one_head_partly_rotated': make_config([FULL[5]]),
    'latent_no_rotated_part_turns': make_config([latent_layer(dims=0)]),
    'latent_many_heads': make_config([latent_layer(heads=7, dim=6, rot_dim=2, vdim=10, kv_rank=18)], width=72),
    'latent_tile_160_128': make_config([TILED[1]]),
    'latent_tile_320_256': make_config([latent_layer(heads=2, dim=16, rot_dim=64, vdim=16, kv_rank=256, ff=0)]),
    'chunk_alone': make_config([chunk_layer()]),
    'chunk_of_one': make_config([chunk_layer(size=1, ff=40)]),
    'chunk_a_page': make_config([chunk_layer(size=64)]),
    'chunk_wider_than_the_prompt': make_config([chunk_layer(size=1000)]),
    'chunk_one_kv_head': make_config([chunk_layer(heads=3, kv_heads=1, dim=10, vdim=14, size=13, ff=50)], width=76, vocab=131),
    'chunk_tile_64_32': make_config([TILED[2]]),
    'one_stream_with_connections': make_config(FULL[:3], streams=1),
    'plain_residual': make_config(FULL[:3], streams=0),
    'five_streams': make_config(FULL[:3], streams=5),
    'whole_stack': make_config(FULL, emb_scale=1.0, eps=3e-6),
    'tiled_stack': make_config(TILED, streams=2),
    'width_that_is_no_multiple_of_four': make_config([window_layer(ff=30), latent_layer(ff=0), chunk_layer(ff=22)], width=70, vocab=131, streams=2),
    'odd_head_sizes': make_config([window_layer(heads=3, kv_heads=1, dim=9, vdim=7, size=11, ff=30), chunk_layer(heads=2, kv_heads=2, dim=5, vdim=3, size=9),
                                   latent_layer(heads=2, dim=7, rot_dim=6, vdim=5, kv_rank=13, ff=0)], width=52, vocab=131, streams=2),
    'wide_values': make_config([window_layer(heads=2, kv_heads=1, dim=8, vdim=160, size=20)]),
}


@pytest.mark.parametrize('name', sorted(MECHANISMS))
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_each_mechanism_whole_prompt(name, dtype):
    cfg = MECHANISMS[name]
    w = random_weights(cfg, seed=len(name))
    toks = tokens_for(cfg, 150, 1)  # crosses page borders, windows and chunks
    want = O.logits(toks, as_f64(w), cfg)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', len(toks))]])['a']
    check(got, want, tol_of(dtype), name)


def test_residual_stream_behind_every_layer():
    cfg = MECHANISMS['whole_stack']
    w = random_weights(cfg, seed=3)
    toks = tokens_for(cfg, 19, 2)
    _, taps = O.forward(cfg, as_f64(w), toks)
    s = session_for(cfg, w, 'float32', debug_mode=True)
    s.step([('a', toks, [0])])
    assert s.engine.layer_runs == len(taps) == len(FULL)
    for j, x in enumerate(taps):
        assert np.abs(s.engine.tap(j) - x).max() < 2e-4 * np.abs(x).max(), f'layer {j}'


@pytest.mark.parametrize('stack', sorted(STACKS))
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_prefill_then_token_by_token(dtype, stack):
    cfg = make_config(STACKS[stack])
    w = random_weights(cfg, seed=5)
    toks = tokens_for(cfg, 170, 3)
    want = O.logits(toks, as_f64(w), cfg)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', 100)]] + [[('a', 1)]] * 70)['a']
    check(got, want, tol_of(dtype))


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('sizes', [[2] * 40, [3, 61, 2, 64, 1, 5, 2, 58, 1, 1, 2], [63, 2, 63, 1, 1, 66], [1] * 9 + [120, 2], [36, 1, 37, 29, 28, 2, 45]])
@pytest.mark.parametrize('stack', sorted(STACKS))
def test_portions_of_a_prompt(sizes, dtype, stack):
    cfg = make_config(STACKS[stack], streams=2)
    w = random_weights(cfg, seed=7)
    toks = tokens_for(cfg, sum(sizes), 4)
    want = O.logits(toks, as_f64(w), cfg)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', n)] for n in sizes])['a']
    check(got, want, tol_of(dtype))


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('stack', sorted(STACKS))
def test_unequal_requests_in_one_batch_equal_each_alone(dtype, stack):
    cfg = make_config(STACKS[stack])
    w = random_weights(cfg, seed=9)
    reqs = {'a': tokens_for(cfg, 131, 5), 'b': tokens_for(cfg, 9, 6), 'c': tokens_for(cfg, 66, 7), 'd': tokens_for(cfg, 2, 8)}
    schedule = [[('a', 60), ('b', 2)], [('b', 1), ('a', 5), ('c', 64)], [('c', 1), ('b', 1), ('a', 1), ('d', 2)],
                [('a', 63), ('b', 5), ('c', 1)], [('a', 1)], [('a', 1)]]
    s = session_for(cfg, w, dtype)
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check(got[rid], O.logits(toks, as_f64(w), cfg), tol_of(dtype), rid)
    assert not s.live() and s.cache.blocks_manager.num_free_blocks() == s.num_blocks and s.slots.num_free_slots() == 4


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_requests_of_very_unequal_length_decode_side_by_side(dtype):
    cfg = make_config(TILED[:3], streams=2)
    w = random_weights(cfg, seed=21)
    reqs = {'long': tokens_for(cfg, 620, 90), 'mid': tokens_for(cfg, 75, 91), 'new': tokens_for(cfg, 12, 92)}
    schedule = [[('long', 600)], [('mid', 65), ('long', 1)]] + [[('long', 1), ('mid', 1), ('new', 1)]] * 10 + [[('long', 9), ('new', 2)]]
    s = session_for(cfg, w, dtype, max_tokens=1024)
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check(got[rid], O.logits(toks, as_f64(w), cfg), tol_of(dtype), rid)


@pytest.mark.parametrize('heads', [8, 20, 32])
def test_decoding_where_many_heads_share_one_key_value_head(heads):
    """Latent attention with 8 and more heads, single decoded tokens: the tile kernel walks the shared keys once per 16 heads (a
    head count that is not a multiple of 16 leaves part of the last tile empty), beside a request that brings a prompt portion."""
    cfg = make_config([latent_layer(heads=heads, dim=32, rot_dim=32, vdim=32, kv_rank=128, ff=0), window_layer(ff=40)], streams=2)
    w = random_weights(cfg, seed=23)
    reqs = {'a': tokens_for(cfg, 140, 93), 'b': tokens_for(cfg, 45, 94)}
    schedule = [[('a', 70)]] + [[('a', 1)]] * 30 + [[('a', 1), ('b', 1)]] * 5 + [[('a', 1), ('b', 40)]] + [[('a', 1)]] * 34
    for dtype in ('bfloat16', 'float32'):
        s = session_for(cfg, w, dtype)
        got = replay(s, reqs, schedule)
        for rid, toks in reqs.items():
            check(got[rid], O.logits(toks, as_f64(w), cfg), tol_of(dtype), f'{dtype} {rid}')


@pytest.mark.parametrize('wide', ['0', '1'])
def test_both_prefill_forms_of_long_head_rows(wide, monkeypatch):
    """Heads of 160 and more dimensions have two staged prompt forms (64 or 128 rows per workgroup, chosen by how many workgroups
    the step makes); both are forced here, on whole prompts, portions that end inside a tile, and mixed steps."""
    monkeypatch.setenv('TLLM_STACK_WIDE_PREFILL', wide)
    cfg = make_config([latent_layer(heads=3, dim=32, rot_dim=32, vdim=32, kv_rank=128, ff=0),
                       latent_layer(heads=2, dim=16, rot_dim=64, vdim=16, kv_rank=256, ff=40)], streams=2)
    w = random_weights(cfg, seed=25)
    reqs = {'a': tokens_for(cfg, 300, 95), 'b': tokens_for(cfg, 171, 96)}
    schedule = [[('a', 129), ('b', 33)], [('a', 1), ('b', 130)], [('a', 150), ('b', 1)], [('a', 20), ('b', 7)]]
    s = session_for(cfg, w, 'bfloat16')
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check(got[rid], O.logits(toks, as_f64(w), cfg), BF16_TOL, rid)


def test_pages_and_slots_that_are_used_again():
    """A pool of 4 pages and 2 slots serves six requests one after another and side by side: every page is written by several
    requests, and what an earlier request left in a page must never be seen through a window, a chunk or the causal mask."""
    cfg = make_config(FULL[:3], streams=2)
    w = random_weights(cfg, seed=11)
    s = session_for(cfg, w, 'float32', max_tokens=256, max_sequences=2)
    assert s.num_blocks == 4
    used_blocks, used_slots = [], []
    for rnd in range(3):
        reqs = {f'x{rnd}': tokens_for(cfg, 100 + rnd, 20 + rnd), f'y{rnd}': tokens_for(cfg, 70 - rnd, 30 + rnd)}
        x, y = f'x{rnd}', f'y{rnd}'
        schedule = [[(x, 50), (y, 3)], [(y, len(reqs[y]) - 3), (x, 1)], [(x, len(reqs[x]) - 51)]]
        got = replay(s, reqs, schedule, end_when_done=False)
        for rid in reqs:
            seq = s._seq[rid]
            used_blocks.append(tuple(s.cache.blocks_manager.block_ids(seq)[0]))
            used_slots.append(s.slots.slot_of(seq))
            check(got[rid], O.logits(reqs[rid], as_f64(w), cfg), F32_TOL, rid)
            s.release(rid)
    assert len(set(used_slots)) == 2 and len(used_slots) == 6
    assert len({b for blocks in used_blocks for b in blocks}) == 4 and sum(len(b) for b in used_blocks) == 12


def rigged(kind, n, p_far, seed, size=37, D=16):
    """One layer whose head 0 is rigged so that the LAST token's query meets the key of the token at p_far with a score far above
    all others: if that key is visible it decides the answer, and dropping, shifting or corrupting it moves the logits at the last
    position by much more than bfloat16 rounding; if the mask hides it, letting it in by mistake does the same."""
    E = 24 if D == 16 else 64
    layer = {'window': window_layer(heads=4, kv_heads=2, dim=D, vdim=E, size=size, ff=0),
             'chunk': chunk_layer(heads=4, kv_heads=2, dim=D, vdim=E, size=size),
             'latent': latent_layer(heads=2, dim=D, rot_dim=D // 2, vdim=E, kv_rank=2 * D, ff=0)}[kind]
    cfg = make_config([layer], streams=2)
    w = random_weights(cfg, seed)
    rng = np.random.default_rng(seed)
    far_tok, last_tok = 3, 4
    toks = [int(t) for t in rng.integers(5, cfg['vocab'], n)]
    toks[p_far], toks[-1] = far_tok, last_tok
    wf = as_f64(w)
    h = O.offset_rms_norm(wf['l0.hc1.in'].sum() * wf['embed'] * cfg['embedding']['scale'], wf['l0.norm1'], cfg['norm']['eps'])
    m = layer['mixer']

    def toward(t, a):
        return bf16_round((a * h[t] / (h[t] @ h[t])).astype(np.float32))

    if kind == 'window':
        # the score has to stand above the distance penalty of head 0; values of its key/value head are made loud, its gate 1/2
        a = ((16.0 + 2.0 ** (-8.0 / m['heads']) * (n - 1 - p_far)) / m['scale']) ** 0.5
        w['l0.mix.q'][D - 1], w['l0.mix.k'][D - 1] = toward(last_tok, a), toward(far_tok, a)
        w['l0.mix.pb'][:] = -4.0
        w['l0.mix.v'][:E] *= 4.0
        w['l0.mix.g'][0] = 0.0
    elif kind == 'chunk':
        w['l0.mix.q'][D - 1], w['l0.mix.k'][D - 1] = toward(last_tok, 24.0), toward(far_tok, 24.0)
        w['l0.mix.temp'][0], w['l0.mix.sink'][0], w['l0.mix.r1'][0] = 6.0, 0.5, 0.25
        w['l0.mix.v'][:E] *= 4.0
        w['l0.mix.g'][0] = 0.0
    else:
        w['l0.mix.dkv'][0] = toward(far_tok, 24.0)
        w['l0.mix.uk'][D - 1] = 0.0
        w['l0.mix.uk'][D - 1, 0] = 1.0
        w['l0.mix.q'][D - 1] = toward(last_tok, 32.0 / m['scale'] / (2 * D) ** 0.5)
    return cfg, w, toks


def run_rigged(kind, n, p_far, dtype, D, sees, size=37):
    cfg, w, toks = rigged(kind, n, p_far, seed=40 + p_far, size=size, D=D)
    wf = as_f64(w)
    want = O.logits(toks, wf, cfg)
    other = list(toks)
    other[p_far] = 7
    moved = rel_err(O.logits(other, wf, cfg)[-1:], want[-1:])[0]
    if sees:
        assert moved > 0.1, f'the rig does not bite: replacing the far token moves the last row by {moved:.3g} only'
    else:
        assert moved < 1e-9, f'the key at {p_far} should be hidden from the last row'
    s = session_for(cfg, w, dtype)
    cut = max(p_far + 1, 2) if p_far + 1 < n else n - 1
    # in a whole prompt, in a portion that starts behind the far key, and decoded alone
    check(replay(s, {'w': toks}, [[('w', n)]])['w'][-1:], want[-1:], tol_of(dtype), 'whole')
    check(replay(s, {'p': toks}, [[('p', cut)], [('p', n - cut)]])['p'][-1:], want[-1:], tol_of(dtype), 'portion')
    check(replay(s, {'d': toks}, [[('d', n - 1)], [('d', 1)]])['d'][-1:], want[-1:], tol_of(dtype), 'decoded')


KINDS = [('float32', 16), ('bfloat16', 16), ('bfloat16', 32)]


@pytest.mark.parametrize('p_far', [0, 1, 31, 32, 63, 64, 127, 128, 200, 331])
@pytest.mark.parametrize('dtype,D', KINDS)
def test_a_far_key_that_decides_the_answer(p_far, dtype, D):
    run_rigged('latent', 333, p_far, dtype, D, sees=True)


@pytest.mark.parametrize('n,size,back,sees', [(120, 37, 36, True), (120, 37, 37, False), (130, 64, 63, True), (130, 64, 64, False),
                                             (200, 65, 64, True), (200, 65, 65, False), (40, 2, 1, True), (40, 2, 2, False),
                                             (129, 128, 127, True), (300, 128, 128, False)])
@pytest.mark.parametrize('dtype,D', KINDS)
def test_keys_at_the_edge_of_a_window(n, size, back, sees, dtype, D):
    """The last row sits at position n - 1; the rigged key `back` tokens before it is the last one inside the window, or the first
    one outside."""
    run_rigged('window', n, n - 1 - back, dtype, D, sees, size=size)


@pytest.mark.parametrize('n,size,p_far,sees', [(120, 37, 111, True), (120, 37, 110, False), (130, 64, 128, True), (130, 64, 127, False),
                                              (197, 65, 195, True), (197, 65, 194, False), (129, 128, 128, True), (129, 128, 127, False),
                                              (128, 128, 0, True), (300, 150, 150, True), (300, 150, 149, False)])
@pytest.mark.parametrize('dtype,D', KINDS)
def test_keys_at_the_edge_of_a_chunk(n, size, p_far, sees, dtype, D):
    """The rigged key is the first one of the last row's chunk, or the last one of the chunk before it."""
    run_rigged('chunk', n, p_far, dtype, D, sees, size=size)


def test_first_tokens_of_a_sequence():
    cfg = MECHANISMS['whole_stack']
    w = random_weights(cfg, seed=13)
    s = session_for(cfg, w, 'float32')
    for n in (1, 2, 3):
        toks = tokens_for(cfg, n, 50 + n)
        check(replay(s, {n: toks}, [[(n, n)]])[n], O.logits(toks, as_f64(w), cfg), F32_TOL, f'{n} tokens at once')
        check(replay(s, {-n: toks}, [[(-n, 1)]] * n)[-n], O.logits(toks, as_f64(w), cfg), F32_TOL, f'{n} tokens one by one')


@pytest.mark.parametrize('stack', sorted(STACKS))
def test_long_decoding(stack):
    cfg = make_config(STACKS[stack][:3], streams=2)
    w = random_weights(cfg, seed=15)
    toks = tokens_for(cfg, 330, 9)
    want = O.logits(toks, as_f64(w), cfg)
    for dtype in ('float32', 'bfloat16'):
        s = session_for(cfg, w, dtype)
        check(replay(s, {'a': toks}, [[('a', 2)]] + [[('a', 1)]] * 328)['a'], want, tol_of(dtype), dtype)


def test_greedy_generation_through_the_scheduler():
    """Six prompts, four state slots, 40 tokens per step: prompts are cut, requests queue, decoded tokens share steps with prompt
    portions.  fp32 engine against the oracle's greedy continuation (recomputed from scratch for every token)."""
    from tensorrt_llm.runtime import SamplingConfig
    cfg = make_config([window_layer(heads=2, kv_heads=1, dim=16, vdim=16, size=23, ff=48), latent_layer(heads=2, ff=0),
                       chunk_layer(heads=2, kv_heads=2, dim=16, vdim=16, size=31, ff=48)], width=64, vocab=97, streams=2)
    w = random_weights(cfg, seed=17)
    prompts = [tokens_for(cfg, n, 60 + n) for n in (70, 3, 45, 1, 90, 17)]
    s = session_for(cfg, w, 'float32', max_tokens=512, max_sequences=4, max_batch_tokens=40)
    outs = s.decode_batch(prompts, SamplingConfig(end_id=-1, pad_id=0), max_new_tokens=6)
    for p, o in zip(prompts, outs):
        assert o.tolist() == O.greedy(p, as_f64(w), cfg, 6)
    assert not s.live() and s.cache.blocks_manager.num_free_blocks() == s.num_blocks


def test_command_lines(tmp_path):
    """examples/vetipel/run.py generates from a checkpoint directory; bin/trace_run replays a recorded schedule from it."""
    from test_gpu_tolenex import write_checkpoint
    cfg = make_config([window_layer(heads=2, kv_heads=1, dim=16, vdim=16, size=23, ff=48), latent_layer(heads=2, ff=0),
                       chunk_layer(heads=2, kv_heads=2, dim=16, vdim=16, size=31, ff=48)], width=64, vocab=97, streams=2)
    w = random_weights(cfg, seed=19)
    ck = str(tmp_path / 'ck')
    write_checkpoint(ck, cfg, w)
    prompt = tokens_for(cfg, 21, 70)
    np.save(tmp_path / 'in.npy', np.asarray(prompt, np.int32))
    run = os.path.join(ROOT, 'trtllm-llama_amd', 'examples', 'vetipel', 'run.py')
    subprocess.run([sys.executable, run, '--model_dir', ck, '--dtype', 'float32', '--input_tokens', str(tmp_path / 'in.npy'),
                    '--max_output_len', '5', '--output_npy', str(tmp_path / 'out.npy')], check=True, timeout=300)
    assert np.load(tmp_path / 'out.npy').reshape(-1)[len(prompt):].tolist() == O.greedy(prompt, as_f64(w), cfg, 5)
    a, b = tokens_for(cfg, 70, 71), tokens_for(cfg, 5, 72)
    steps = [{'step': 0, 'entries': [{'id': 'a', 'tokens': a[:66], 'want': [0, 65]}, {'id': 'b', 'tokens': b[:2], 'want': []}], 'end': []},
             {'step': 1, 'entries': [{'id': 'b', 'tokens': b[2:], 'want': [2]}], 'end': ['b']},
             {'step': 2, 'entries': [{'id': 'a', 'tokens': a[66:], 'want': [3]}], 'end': ['a']}]
    out = tmp_path / 'logits'
    r = subprocess.run([os.path.join(ROOT, 'bin', 'trace_run'), '--model', ck, '--dtype', 'float32', '--out', str(out), '--max-tokens', '192'],
                       input='\n'.join(json.dumps(s) for s in steps) + '\n', capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith('done')] == ['done 0', 'done 1', 'done 2']
    la, lb = O.logits(a, as_f64(w), cfg), O.logits(b, as_f64(w), cfg)
    check(np.fromfile(out / '0.f32', '<f4').reshape(2, -1), la[[0, 65]], F32_TOL)
    check(np.fromfile(out / '1.f32', '<f4').reshape(1, -1), lb[[4]], F32_TOL)
    check(np.fromfile(out / '2.f32', '<f4').reshape(1, -1), la[[69]], F32_TOL)
