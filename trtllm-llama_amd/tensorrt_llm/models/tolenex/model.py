"""Tolenex: a decoder-only stack of parallel layers - x <- x + g1 * mixer(norm1(x)) + g2 * ff(norm2(x)) with sigmoid gates
g = sigmoid(W h + b) on both sublayers - whose mixers are differential attention (two attention maps per head over shared
values, o = a1 - lambda * a2, per-head RMS norm; interleaved rotary positions with YaRN frequency scaling; tanh soft cap;
grouped-query) or HGRN2 (gated linear recurrence with a lower-bounded forget gate).  Norms are RMS norms in groups; a range of
layers can be looped (every pass with its own cache, the embedding output re-added and a per-pass vector added at its entry).

This class reads the model's config.json and its safetensors file and describes the stack to the ragged engine
(runtime/stack.py); there is no Python forward pass.  Constants the design fixes live here (two maps per attention head, the
head norm, gelu-tanh in the feed-forward, the gated residual); everything else is read from the configuration."""
import json
from typing import Dict

import numpy as np

from ..stack_model import PAGE_SIZE, StackModelForCausalLM, bf16_bits_to_f32, to_bf16_bits  # noqa: F401


class TolenexConfig(object):
    """config.json: architecture, vocab, width, embedding.scale, norm.{eps, groups}, loop.{start, stop, times} (optional),
    layers[i].{type, mixer{...}, mlp{ff, kind} | null}."""

    def __init__(self, d: Dict):
        self.raw = d
        self.vocab, self.width = int(d['vocab']), int(d['width'])
        self.embedding_scale = float(d.get('embedding', {}).get('scale', 1.0))
        norm = d.get('norm', {})
        self.norm_eps, self.norm_groups = float(norm.get('eps', 1e-5)), int(norm.get('groups', 1))
        loop = d.get('loop') or {}
        self.loop_start, self.loop_stop = int(loop.get('start', 0)), int(loop.get('stop', 0))
        self.loop_times = int(loop.get('times', 1))
        self.layers = d['layers']
        for i, l in enumerate(self.layers):
            if l['type'] not in ('attention', 'hgrn2'):
                raise ValueError(f"layer {i}: mixer type {l['type']!r} is not one this design has (attention | hgrn2)")
            mlp = l.get('mlp')
            if mlp is not None and mlp.get('kind', 'dense') != 'dense':
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} (dense)")

    @staticmethod
    def from_json_file(path: str) -> 'TolenexConfig':
        with open(path) as f:
            return TolenexConfig(json.load(f))

    def engine_config(self) -> Dict:
        c = dict(width=self.width, vocab=self.vocab, num_layers=len(self.layers), norm_groups=self.norm_groups,
                 norm_eps=repr(self.norm_eps), embedding_scale=repr(self.embedding_scale), loop_start=self.loop_start,
                 loop_stop=self.loop_stop, loop_times=self.loop_times, page_size=PAGE_SIZE)
        for i, l in enumerate(self.layers):
            p, m = f'layer.{i}.', l['mixer']
            c[p + 'type'] = l['type']
            c[p + 'heads'], c[p + 'dim'], c[p + 'vdim'] = int(m['heads']), int(m['dim']), int(m.get('vdim', m['dim']))
            c[p + 'ff'] = int(l['mlp']['ff']) if l.get('mlp') else 0
            if l['type'] == 'attention':
                c[p + 'kv_heads'] = int(m.get('kv_heads', m['heads']))
                c[p + 'maps'] = 2          # differential attention
                c[p + 'head_norm'] = 1
                c[p + 'diff'] = repr(float(m['diff']))
                c[p + 'scale'] = repr(float(m['scale']))
                c[p + 'softcap'] = repr(float(m.get('softcap') or 0.0))
                rot = m.get('rot') or {}
                c[p + 'rot_dims'] = int(rot.get('dims', 0))
                c[p + 'rot_base'] = repr(float(rot.get('base', 10000.0)))
                sc = rot.get('scaling')
                if sc:
                    c[p + 'rot_factor'], c[p + 'rot_original'] = repr(float(sc['factor'])), repr(float(sc['original']))
                    c[p + 'rot_fast'], c[p + 'rot_slow'] = repr(float(sc['fast'])), repr(float(sc['slow']))
        return c


class TolenexForCausalLM(StackModelForCausalLM):
    architecture = 'Tolenex'
    config_class = TolenexConfig

    @classmethod
    def from_random(cls, config: Dict, seed: int = 0, std: float = 0.02) -> 'TolenexForCausalLM':
        """Random bfloat16-valued weights of the configuration's shapes (benchmarks, tests)."""
        cfg = config if isinstance(config, TolenexConfig) else TolenexConfig(config)
        rng = np.random.default_rng(seed)
        t = {}

        def mat(name, *shape, s=std, mean=0.0):
            a = (rng.standard_normal(shape, dtype=np.float32) * s + mean).astype(np.float32)
            t[name] = (to_bf16_bits(a), 'bfloat16')

        W = cfg.width
        mat('embed', cfg.vocab, W, s=1.0 / max(cfg.embedding_scale, 1e-6))
        mat('head', cfg.vocab, W, s=W ** -0.5)
        mat('final.norm', W, s=0.1, mean=1.0)
        if cfg.loop_stop > cfg.loop_start:
            mat('loop.step', cfg.loop_times, W, s=0.1)
        for i, l in enumerate(cfg.layers):
            p, m = f'l{i}.', l['mixer']
            H, D, V = int(m['heads']), int(m['dim']), int(m.get('vdim', m['dim']))
            mat(p + 'norm1', W, s=0.1, mean=1.0)
            mat(p + 'rg1', W, W, s=W ** -0.5)
            mat(p + 'rg1.b', W, s=0.5)
            if l['type'] == 'attention':
                G = int(m.get('kv_heads', H))
                mat(p + 'mix.q', H * 2 * D, W, s=W ** -0.5)
                mat(p + 'mix.k', G * 2 * D, W, s=W ** -0.5)
                mat(p + 'mix.v', G * V, W, s=W ** -0.5)
                for n in ('lq1', 'lk1', 'lq2', 'lk2'):
                    mat(p + 'mix.' + n, D, s=0.3)
            else:
                mat(p + 'mix.q', H * D, W, s=W ** -0.5)
                mat(p + 'mix.f', H * D, W, s=W ** -0.5)
                mat(p + 'mix.f.b', H * D, s=1.0, mean=1.0)
                t[p + 'mix.lower'] = (to_bf16_bits(rng.uniform(0.0, 0.9, H * D).astype(np.float32)), 'bfloat16')
                mat(p + 'mix.v', H * V, W, s=W ** -0.5)
                mat(p + 'mix.norm', V, s=0.1, mean=1.0)
            mat(p + 'mix.o', W, H * V, s=(H * V) ** -0.5)
            if l.get('mlp'):
                F = int(l['mlp']['ff'])
                mat(p + 'norm2', W, s=0.1, mean=1.0)
                mat(p + 'rg2', W, W, s=W ** -0.5)
                mat(p + 'rg2.b', W, s=0.5)
                mat(p + 'mlp.gate', F, W, s=W ** -0.5)
                mat(p + 'mlp.up', F, W, s=W ** -0.5)
                mat(p + 'mlp.down', W, F, s=F ** -0.5)
        return cls(cfg, t)
