"""Small Vetipel configurations and random weights for the tests (own generator: nothing of the product's random-weight code)."""
import numpy as np

from tolenex_cases import bf16_round


def window_layer(heads=6, kv_heads=3, dim=16, vdim=24, size=37, ff=136):
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'scale': 1.3 / dim ** 0.5, 'mask': {'size': size}}
    return {'type': 'attention', 'mixer': m, 'mlp': {'ff': ff, 'kind': 'dense'} if ff else None}


def latent_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, base=5000.0, dims=None, ff=72):
    m = {'heads': heads, 'dim': dim, 'rot_dim': rot_dim, 'vdim': vdim, 'kv_rank': kv_rank, 'scale': 1.5 / (dim + rot_dim) ** 0.5,
         'rot': {'dims': rot_dim if dims is None else dims, 'base': base}}
    return {'type': 'latent_attention', 'mixer': m, 'mlp': {'ff': ff, 'kind': 'dense'} if ff else None}


def chunk_layer(heads=4, kv_heads=2, dim=24, vdim=16, size=29, ff=0):
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'scale': 1.0 / dim ** 0.5, 'mask': {'size': size}}
    return {'type': 'attention_2', 'mixer': m, 'mlp': {'ff': ff, 'kind': 'dense'} if ff else None}


def make_config(layers, width=96, vocab=211, streams=3, eps=1e-5, emb_scale=5.5):
    cfg = {'architecture': 'Vetipel', 'vocab': vocab, 'width': width, 'embedding': {'scale': emb_scale}, 'norm': {'eps': eps},
           'layers': layers}
    if streams:
        cfg['streams'] = streams
    return cfg


def random_weights(cfg, seed=0):
    """name -> fp32 array of bfloat16-representable values, sized by cfg; scaled so that scores, gates and logits are O(1)."""
    rng = np.random.default_rng(seed)
    W, S, w = cfg['width'], cfg.get('streams', 0), {}

    def put(name, *shape, std=1.0, mean=0.0):
        w[name] = bf16_round(rng.standard_normal(shape).astype(np.float32) * std + mean)

    put('embed', cfg['vocab'], W, std=1.0 / cfg['embedding']['scale'])
    put('head', cfg['vocab'], W, std=2.0 / W ** 0.5)
    put('final.norm', W, std=0.2)
    for i, layer in enumerate(cfg['layers']):
        p, m = f'l{i}.', layer['mixer']
        H, D, E = m['heads'], m['dim'], m['vdim']
        put(p + 'norm1', W, std=0.2)
        if layer['type'] == 'latent_attention':
            C, R = m['kv_rank'], m['rot_dim']
            put(p + 'mix.q', H * (D + R), W, std=1.5 / W ** 0.5)
            put(p + 'mix.dkv', C + R, W, std=1.5 / W ** 0.5)
            put(p + 'mix.dkv.norm', C, std=0.2, mean=1.0)
            put(p + 'mix.uk', H * D, C, std=1.5 / C ** 0.5)
            put(p + 'mix.uv', H * E, C, std=1.0 / C ** 0.5)
        else:
            G = m['kv_heads']
            put(p + 'mix.q', H * D, W, std=1.6 / W ** 0.5)
            put(p + 'mix.k', G * D, W, std=1.6 / W ** 0.5)
            put(p + 'mix.v', G * E, W, std=1.0 / W ** 0.5)
            put(p + 'mix.g', H, W, std=1.5 / W ** 0.5)
            if layer['type'] == 'attention':
                put(p + 'mix.pb', H, std=0.7, mean=-1.0)
            else:
                put(p + 'mix.q.b', H * D, std=0.3)
                put(p + 'mix.k.b', G * D, std=0.3)
                put(p + 'mix.v.b', G * E, std=0.3)
                put(p + 'mix.temp', H, std=0.5, mean=2.5)
                put(p + 'mix.sink', H, std=1.0, mean=1.0)
                w[p + 'mix.r1'] = bf16_round(rng.uniform(0.2, 1.5, H).astype(np.float32))
                w[p + 'mix.r2'] = bf16_round(rng.uniform(0.1, 2.0, H).astype(np.float32))
        put(p + 'mix.o', W, H * E, std=1.0 / (H * E) ** 0.5)
        if layer.get('mlp'):
            F = layer['mlp']['ff']
            put(p + 'norm2', W, std=0.2)
            put(p + 'mlp.up', F, W, std=1.5 / W ** 0.5)
            put(p + 'mlp.down', W, F, std=1.0 / F ** 0.5)
        for q in (1, 2):
            if S and (q == 1 or layer.get('mlp')):
                put(p + f'hc{q}.in', S, std=0.3, mean=0.6)
                put(p + f'hc{q}.out', S, std=0.4, mean=0.8)
                w[p + f'hc{q}.mix'] = bf16_round((np.eye(S) * 0.8 + rng.standard_normal((S, S)) * 0.2).astype(np.float32))
    return w


def as_model(cfg, w):
    """The product's model object over these weights (bfloat16 bit patterns, as a checkpoint reader would deliver them)."""
    from tensorrt_llm.models.vetipel.model import VetipelConfig, VetipelForCausalLM
    tensors = {k: ((np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(v.shape), 'bfloat16')
               for k, v in w.items()}
    return VetipelForCausalLM(VetipelConfig(cfg), tensors)
