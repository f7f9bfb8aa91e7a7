"""Small Tolenex configurations and random weights for the tests (own generator: nothing of the product's random-weight code),
plus the replay helper that drives RaggedGenerationSession.step by a hand-written schedule."""
import numpy as np


def bf16_round(a):
    """fp32 values that are exactly representable in bfloat16 (round to nearest even)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, diff=0.25, rot_dims=8, scaling=True, softcap=30.0, ff=136, base=5000.0):
    rot = None
    if rot_dims:
        rot = {'dims': rot_dims, 'base': base}
        if scaling:
            rot['scaling'] = {'factor': 4.0, 'original': 48, 'fast': 16.0, 'slow': 2.0}
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'diff': diff, 'scale': 1.7 / dim ** 0.5, 'softcap': softcap}
    if rot:
        m['rot'] = rot
    return {'type': 'attention', 'mixer': m, 'mlp': {'ff': ff, 'kind': 'dense'} if ff else None}


def hgrn2_layer(heads=2, dim=24, vdim=80, ff=0):
    return {'type': 'hgrn2', 'mixer': {'heads': heads, 'dim': dim, 'vdim': vdim}, 'mlp': {'ff': ff, 'kind': 'dense'} if ff else None}


def make_config(layers, width=96, vocab=211, groups=3, eps=1e-5, emb_scale=5.5, loop=None):
    cfg = {'architecture': 'Tolenex', 'vocab': vocab, 'width': width, 'embedding': {'scale': emb_scale},
           'norm': {'eps': eps, 'groups': groups}, 'layers': layers}
    if loop:
        cfg['loop'] = {'start': loop[0], 'stop': loop[1], 'times': loop[2]}
    return cfg


def random_weights(cfg, seed=0):
    """name -> fp32 array of bfloat16-representable values, sized by cfg; scaled so that scores, gates and logits are O(1)."""
    rng = np.random.default_rng(seed)
    W, w = cfg['width'], {}

    def put(name, *shape, std=1.0, mean=0.0):
        w[name] = bf16_round(rng.standard_normal(shape).astype(np.float32) * std + mean)

    put('embed', cfg['vocab'], W, std=1.0 / cfg['embedding']['scale'])
    put('head', cfg['vocab'], W, std=2.0 / W ** 0.5)
    put('final.norm', W, std=0.2, mean=1.0)
    loop = cfg.get('loop')
    if loop and loop['stop'] > loop['start']:
        put('loop.step', loop['times'], W, std=0.3)
    for i, layer in enumerate(cfg['layers']):
        p, m = f'l{i}.', layer['mixer']
        H, D, E = m['heads'], m['dim'], m.get('vdim', m['dim'])
        put(p + 'norm1', W, std=0.2, mean=1.0)
        put(p + 'rg1', W, W, std=1.0 / W ** 0.5)
        put(p + 'rg1.b', W, std=0.5)
        if layer['type'] == 'attention':
            G = m.get('kv_heads', H)
            put(p + 'mix.q', H * 2 * D, W, std=1.6 / W ** 0.5)
            put(p + 'mix.k', G * 2 * D, W, std=1.6 / W ** 0.5)
            put(p + 'mix.v', G * E, W, std=1.0 / W ** 0.5)
            for n in ('lq1', 'lk1', 'lq2', 'lk2'):
                put(p + 'mix.' + n, D, std=0.25)
        else:
            put(p + 'mix.q', H * D, W, std=1.0 / W ** 0.5)
            put(p + 'mix.f', H * D, W, std=1.5 / W ** 0.5)
            put(p + 'mix.f.b', H * D, std=1.0, mean=1.5)
            w[p + 'mix.lower'] = bf16_round(rng.uniform(0.0, 0.95, H * D).astype(np.float32))
            put(p + 'mix.v', H * E, W, std=1.0 / W ** 0.5)
            put(p + 'mix.norm', E, std=0.2, mean=1.0)
        put(p + 'mix.o', W, H * E, std=1.0 / (H * E) ** 0.5)
        if layer.get('mlp'):
            F = layer['mlp']['ff']
            put(p + 'norm2', W, std=0.2, mean=1.0)
            put(p + 'rg2', W, W, std=1.0 / W ** 0.5)
            put(p + 'rg2.b', W, std=0.5)
            put(p + 'mlp.gate', F, W, std=1.5 / W ** 0.5)
            put(p + 'mlp.up', F, W, std=1.0 / W ** 0.5)
            put(p + 'mlp.down', W, F, std=1.0 / F ** 0.5)
    return w


def as_model(cfg, w):
    """The product's model object over these weights (bfloat16 bit patterns, as a checkpoint reader would deliver them)."""
    from tensorrt_llm.models.tolenex.model import TolenexConfig, TolenexForCausalLM
    tensors = {k: ((np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(v.shape), 'bfloat16')
               for k, v in w.items()}
    return TolenexForCausalLM(TolenexConfig(cfg), tensors)


def as_f64(w):
    return {k: v.astype(np.float64) for k, v in w.items()}


def replay(session, requests, schedule, end_when_done=True):
    """requests: id -> token list; schedule: list of steps, a step = list of (id, count).  Every position's logits are asked for.
    Returns id -> [n, vocab] fp32 in position order."""
    at = {r: 0 for r in requests}
    rows = {r: [] for r in requests}
    for step in schedule:
        entries, end = [], []
        for rid, count in step:
            lo = at[rid]
            entries.append((rid, requests[rid][lo:lo + count], list(range(count))))
            at[rid] = lo + count
            if end_when_done and at[rid] == len(requests[rid]):
                end.append(rid)
        logits, _ = session.step(entries, end=end)
        k = 0
        for rid, count in step:
            rows[rid].append(logits[k:k + count])
            k += count
    return {r: np.concatenate(v) for r, v in rows.items() if v}


def rel_err(got, want):
    """per row: rms of the difference (mean over the vocabulary taken off) / rms of the expected row"""
    d = got - want
    d = d - d.mean(axis=1, keepdims=True)
    c = want - want.mean(axis=1, keepdims=True)
    return np.sqrt((d * d).mean(axis=1)) / np.sqrt((c * c).mean(axis=1))
