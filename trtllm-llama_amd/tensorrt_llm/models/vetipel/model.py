"""Vetipel: a pre-norm decoder stack - x <- x + mixer(norm1(x)), x <- x + ff(norm2(x)) - whose residual is kept in `streams`
hyper-connected copies (a sublayer reads a weighted sum of the streams and its result is written back into all of them through a
mixing matrix), whose RMS-norm weights are stored as offsets from one, and whose mixers are three kinds of attention over the
paged cache:

  attention          grouped-query, no rotation; a linear distance penalty slope_h (i - j) with slope_h = 2^(-8 (h + 1) / H); a
                     sliding window; sigmoid weights with a per-head offset instead of a softmax; a per-head sigmoid output gate
  latent_attention   one RMS-normed latent per token from which every head's unrotated key and value are expanded, plus one
                     rotated key part shared by the heads (interleaved pairs); causal softmax.  The cache holds the latent and the
                     rotated part; the engine runs the absorbed form
  attention_2        grouped-query with projection biases, unit-RMS queries and keys, a per-head temperature, a logarithmic
                     distance penalty r1_h ln(1 + r2_h (i - j)), a chunked mask, a softmax with a per-head sink, the output gate

The feed-forward is W_down relu(W_up h)^2.  This class reads config.json and the safetensors file and describes the stack to the
ragged engine (runtime/stack.py).  Constants the design fixes live here (the slope base, the norm offset, which options each mixer
kind switches on); every size and every other constant is read from the configuration."""
import json
from typing import Dict

import numpy as np

from ..stack_model import PAGE_SIZE, StackModelForCausalLM, to_bf16_bits

SLOPE_BASE = 8.0       # attention: slope_h = 2^(-SLOPE_BASE (h + 1) / heads)
NORM_OFFSET = 1.0      # norm weights are stored around zero
MIXERS = ('attention', 'latent_attention', 'attention_2')


class VetipelConfig(object):
    """config.json: architecture, vocab, width, embedding.scale, norm.eps, streams (absent: one plain residual), layers[i].{type,
    mixer{...}, mlp{ff, kind} | null}."""

    def __init__(self, d: Dict):
        self.raw = d
        self.vocab, self.width = int(d['vocab']), int(d['width'])
        self.embedding_scale = float((d.get('embedding') or {}).get('scale', 1.0))
        self.norm_eps = float((d.get('norm') or {}).get('eps', 1e-6))
        self.streams = int(d.get('streams') or 0)
        self.layers = d['layers']
        for i, l in enumerate(self.layers):
            if l['type'] not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {l['type']!r} is not one this design has {MIXERS}")
            mlp = l.get('mlp')
            if mlp is not None and mlp.get('kind', 'dense') != 'dense':
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} (dense)")

    @staticmethod
    def from_json_file(path: str) -> 'VetipelConfig':
        with open(path) as f:
            return VetipelConfig(json.load(f))

    def engine_config(self) -> Dict:
        c = dict(width=self.width, vocab=self.vocab, num_layers=len(self.layers), norm_groups=1, norm_eps=repr(self.norm_eps),
                 norm_offset=repr(NORM_OFFSET), embedding_scale=repr(self.embedding_scale), page_size=PAGE_SIZE,
                 block='sequential', residual='hyper', streams=max(self.streams, 1))
        for i, l in enumerate(self.layers):
            p, m = f'layer.{i}.', l['mixer']
            c[p + 'heads'], c[p + 'dim'], c[p + 'vdim'] = int(m['heads']), int(m['dim']), int(m.get('vdim', m['dim']))
            c[p + 'ff'] = int(l['mlp']['ff']) if l.get('mlp') else 0
            c[p + 'mlp'] = 'relu2'
            if 'scale' in m:     # absent: the engine's default, 1 / sqrt(query size)
                c[p + 'scale'] = repr(float(m['scale']))
            if l['type'] == 'latent_attention':
                c[p + 'type'] = 'latent_attention'
                c[p + 'kv_rank'] = int(m['kv_rank'])
                rot = m.get('rot') or {}
                c[p + 'rot_dim'] = int(m.get('rot_dim', rot.get('dims', 0)))
                c[p + 'rot_dims'] = int(rot.get('dims', c[p + 'rot_dim']))
                c[p + 'rot_base'] = repr(float(rot.get('base', 10000.0)))
                continue
            c[p + 'type'] = 'attention'
            c[p + 'kv_heads'] = int(m.get('kv_heads', m['heads']))
            c[p + 'maps'], c[p + 'head_norm'], c[p + 'rot_dims'] = 1, 0, 0
            c[p + 'out_gate'] = 1
            size = int((m.get('mask') or {}).get('size', 0))   # no size: plain causal
            c[p + 'mask_size'] = size
            if l['type'] == 'attention':
                c[p + 'pos_bias'], c[p + 'slope_base'] = 'linear', repr(SLOPE_BASE)
                c[p + 'mask'], c[p + 'weights'] = ('window' if size else 'causal'), 'sigmoid'
            else:
                c[p + 'qkv_bias'], c[p + 'qk_norm'], c[p + 'head_temp'], c[p + 'sink'] = 1, 1, 1, 1
                c[p + 'pos_bias'], c[p + 'mask'], c[p + 'weights'] = 'log', ('chunk' if size else 'causal'), 'softmax'
        return c


class VetipelForCausalLM(StackModelForCausalLM):
    architecture = 'Vetipel'
    config_class = VetipelConfig

    @classmethod
    def from_random(cls, config: Dict, seed: int = 0) -> 'VetipelForCausalLM':
        """Random bfloat16-valued weights of the configuration's shapes (benchmarks, examples)."""
        cfg = config if isinstance(config, VetipelConfig) else VetipelConfig(config)
        rng = np.random.default_rng(seed)
        t = {}

        def mat(name, *shape, s=1.0, mean=0.0):
            a = (rng.standard_normal(shape, dtype=np.float32) * s + mean).astype(np.float32)
            t[name] = (to_bf16_bits(a), 'bfloat16')

        W, S = cfg.width, cfg.streams
        mat('embed', cfg.vocab, W, s=1.0 / max(cfg.embedding_scale, 1e-6))
        mat('head', cfg.vocab, W, s=W ** -0.5)
        mat('final.norm', W, s=0.1)
        for i, l in enumerate(cfg.layers):
            p, m = f'l{i}.', l['mixer']
            H, D, E = int(m['heads']), int(m['dim']), int(m.get('vdim', m['dim']))
            mat(p + 'norm1', W, s=0.1)
            if l['type'] == 'latent_attention':
                C, R = int(m['kv_rank']), int(m['rot_dim'])
                mat(p + 'mix.q', H * (D + R), W, s=W ** -0.5)
                mat(p + 'mix.dkv', C + R, W, s=W ** -0.5)
                mat(p + 'mix.dkv.norm', C, s=0.1, mean=1.0)
                mat(p + 'mix.uk', H * D, C, s=C ** -0.5)
                mat(p + 'mix.uv', H * E, C, s=C ** -0.5)
            else:
                G = int(m.get('kv_heads', H))
                mat(p + 'mix.q', H * D, W, s=W ** -0.5)
                mat(p + 'mix.k', G * D, W, s=W ** -0.5)
                mat(p + 'mix.v', G * E, W, s=W ** -0.5)
                mat(p + 'mix.g', H, W, s=W ** -0.5)
                if l['type'] == 'attention':
                    mat(p + 'mix.pb', H, s=0.5, mean=-2.0)
                else:
                    for n, k in (('q', H * D), ('k', G * D), ('v', G * E)):
                        mat(p + f'mix.{n}.b', k, s=0.1)
                    mat(p + 'mix.temp', H, s=0.2, mean=3.0)
                    mat(p + 'mix.sink', H, s=0.5)
                    t[p + 'mix.r1'] = (to_bf16_bits(rng.uniform(0.1, 1.0, H).astype(np.float32)), 'bfloat16')
                    t[p + 'mix.r2'] = (to_bf16_bits(rng.uniform(0.1, 1.0, H).astype(np.float32)), 'bfloat16')
            mat(p + 'mix.o', W, H * E, s=(H * E) ** -0.5)
            if l.get('mlp'):
                F = int(l['mlp']['ff'])
                mat(p + 'norm2', W, s=0.1)
                mat(p + 'mlp.up', F, W, s=W ** -0.5)
                mat(p + 'mlp.down', W, F, s=F ** -0.5)
            for q in (1, 2):
                if S and (q == 1 or l.get('mlp')):
                    mat(p + f'hc{q}.in', S, s=0.1, mean=1.0 / S)
                    mat(p + f'hc{q}.out', S, s=0.1, mean=1.0)
                    t[p + f'hc{q}.mix'] = (to_bf16_bits((np.eye(S) + rng.standard_normal((S, S)) * 0.05).astype(np.float32)), 'bfloat16')
        return cls(cfg, t)
