"""Rofozen: a pre-norm decoder stack - x <- x + mixer(norm1(x)), x <- x + ff(norm2(x)) - with plain RMS norms, whose layers are
listed one by one in config.json (a layer may run on another layer's weights, with a cache / state of its own), two mixers

  mamba2             a selective state-space layer: one projection gives the gate z, the inputs x | B | C of the recurrence and a
                     step size per head; x | B | C pass a short causal convolution and silu; per head
                     S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x, dt = softplus(dt + dt_bias); y * silu(z) is RMS-normed
                     in equal parts of the row and projected back.  State and convolution tail live in a state slot
  latent_attention   queries expanded from a normed low-rank latent; keys and values from one normed latent per token plus one
                     rotated key part shared by the heads (half-split pairs, YaRN-blended frequencies, cos / sin scaled by
                     0.1 ln(factor) + 1); a sliding window; a softmax whose denominator holds a per-head sink.  The cache holds the
                     latent and the rotated part; the engine runs the absorbed form

and two feed-forwards: dense W_down (gelu_tanh(W_gate h) * W_up h), and a routed mixture of experts W_down (silu(W_gate h) * W_up h)
with a softmax router over experts in groups (the choice adds a stored correction to the score, the weight is the plain score times
a scale; only experts of the best groups can be chosen; the last router outputs are identity experts that return h).

This class reads config.json and the safetensors file and describes the stack to the ragged engine (runtime/stack.py).  What the
design fixes lives here (which options each mixer kind switches on, the activations); every size and every other constant is read
from the configuration."""
import json
from typing import Dict

import numpy as np

from ..stack_model import PAGE_SIZE, StackModelForCausalLM, to_bf16_bits

MIXERS = ('mamba2', 'latent_attention')
MLP_KINDS = ('dense', 'moe')


class RofozenConfig(object):
    """config.json: architecture, vocab, width, norm.eps, layers[i].{type, mixer{...}, mlp{kind, ...} | null, weights_of}."""

    def __init__(self, d: Dict):
        self.raw = d
        self.vocab, self.width = int(d['vocab']), int(d['width'])
        self.norm_eps = float((d.get('norm') or {}).get('eps', 1e-6))
        self.layers = d['layers']
        for i, l in enumerate(self.layers):
            if l['type'] not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {l['type']!r} is not one this design has {MIXERS}")
            mlp = l.get('mlp')
            if mlp is not None and mlp.get('kind', 'dense') not in MLP_KINDS:
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} {MLP_KINDS}")
            j = l.get('weights_of')
            if j is not None and not (0 <= int(j) < i and self.layers[int(j)].get('weights_of') is None):
                raise ValueError(f'layer {i}: weights_of {j} must name an earlier layer with weights of its own')

    @staticmethod
    def from_json_file(path: str) -> 'RofozenConfig':
        with open(path) as f:
            return RofozenConfig(json.load(f))

    def weight_layer(self, i: int) -> int:
        j = self.layers[i].get('weights_of')
        return i if j is None else int(j)

    def engine_config(self) -> Dict:
        c = dict(width=self.width, vocab=self.vocab, num_layers=len(self.layers), norm_groups=1, norm_eps=repr(self.norm_eps),
                 norm_offset=0, embedding_scale=1, page_size=PAGE_SIZE, block='sequential', residual='hyper', streams=1)
        for i, l in enumerate(self.layers):
            p, m = f'layer.{i}.', l['mixer']
            c[p + 'type'] = l['type']
            if l.get('weights_of') is not None:
                c[p + 'weights_of'] = int(l['weights_of'])
            c[p + 'heads'], c[p + 'vdim'] = int(m['heads']), int(m['vdim'])
            if l['type'] == 'mamba2':
                c[p + 'state'], c[p + 'groups'], c[p + 'conv'] = int(m['state']), int(m.get('groups', 1)), int(m['conv'])
                c[p + 'ssm_norm_groups'] = int(m.get('norm_groups', 1))
            else:
                rot = m.get('rot') or {}
                c[p + 'dim'], c[p + 'kv_rank'], c[p + 'q_rank'] = int(m['dim']), int(m['kv_rank']), int(m['q_rank'])
                c[p + 'rot_dim'] = int(m.get('rot_dim', rot.get('dims', 0)))
                c[p + 'rot_dims'] = int(rot.get('dims', 0))
                c[p + 'rot_base'] = repr(float(rot.get('base', 10000.0)))
                c[p + 'rot_pairing'] = 'halves'
                sc = rot.get('scaling')
                if sc:
                    c[p + 'rot_factor'], c[p + 'rot_original'] = repr(float(sc['factor'])), repr(float(sc['original']))
                    c[p + 'rot_fast'], c[p + 'rot_slow'] = repr(float(sc['fast'])), repr(float(sc['slow']))
                c[p + 'scale'] = repr(float(m['scale']))
                size = int((m.get('mask') or {}).get('size', 0))   # no size: plain causal
                c[p + 'mask'], c[p + 'mask_size'] = ('window' if size else 'causal'), size
                c[p + 'sink'] = 1
            mlp = l.get('mlp')
            if not mlp:
                c[p + 'ff'] = 0
            elif mlp.get('kind', 'dense') == 'dense':
                c[p + 'ff'], c[p + 'mlp'] = int(mlp['ff']), 'gelu_gate'
            else:
                r = mlp['router']
                g = r.get('groups') or {}
                c[p + 'ff'], c[p + 'mlp'] = int(mlp['expert']['ff']), 'moe'
                c[p + 'experts'], c[p + 'identity'], c[p + 'top'] = int(r['experts']), int(r.get('identity', 0)), int(r['top'])
                c[p + 'route_groups'] = int(g.get('count', 1))
                c[p + 'route_keep'] = int(g.get('keep', c[p + 'route_groups']))
                c[p + 'route_scale'] = repr(float(r.get('scale', 1.0)))
        return c


class RofozenForCausalLM(StackModelForCausalLM):
    architecture = 'Rofozen'
    config_class = RofozenConfig

    @classmethod
    def from_random(cls, config: Dict, seed: int = 0) -> 'RofozenForCausalLM':
        """Random bfloat16-valued weights of the configuration's shapes (benchmarks, examples)."""
        cfg = config if isinstance(config, RofozenConfig) else RofozenConfig(config)
        rng = np.random.default_rng(seed)
        t = {}

        def mat(name, *shape, s=1.0, mean=0.0):
            a = (rng.standard_normal(shape, dtype=np.float32) * s + mean).astype(np.float32)
            t[name] = (to_bf16_bits(a), 'bfloat16')

        W = cfg.width
        mat('embed', cfg.vocab, W)
        mat('head', cfg.vocab, W, s=W ** -0.5)
        mat('final.norm', W, s=0.1, mean=1.0)
        for i, l in enumerate(cfg.layers):
            if l.get('weights_of') is not None:
                continue
            p, m = f'l{i}.', l['mixer']
            H, E = int(m['heads']), int(m['vdim'])
            mat(p + 'norm1', W, s=0.1, mean=1.0)
            if l['type'] == 'mamba2':
                N, G, K = int(m['state']), int(m.get('groups', 1)), int(m['conv'])
                inner, ch = H * E, H * E + 2 * G * N
                mat(p + 'mix.in', inner + ch + H, W, s=W ** -0.5)
                mat(p + 'mix.conv', ch, K, s=K ** -0.5)
                mat(p + 'mix.conv.b', ch, s=0.1)
                mat(p + 'mix.dt_bias', H, s=0.5, mean=-1.0)
                t[p + 'mix.A_log'] = (to_bf16_bits(np.log(rng.uniform(0.5, 4.0, H)).astype(np.float32)), 'bfloat16')
                mat(p + 'mix.D', H, s=0.3, mean=1.0)
                mat(p + 'mix.norm', inner, s=0.1, mean=1.0)
                mat(p + 'mix.o', W, inner, s=inner ** -0.5)
            else:
                D, C, Q, R = int(m['dim']), int(m['kv_rank']), int(m['q_rank']), int(m['rot_dim'])
                mat(p + 'mix.dq', Q, W, s=W ** -0.5)
                mat(p + 'mix.dq.norm', Q, s=0.1, mean=1.0)
                mat(p + 'mix.uq', H * (D + R), Q, s=Q ** -0.5)
                mat(p + 'mix.dkv', C + R, W, s=W ** -0.5)
                mat(p + 'mix.dkv.norm', C, s=0.1, mean=1.0)
                mat(p + 'mix.uk', H * D, C, s=C ** -0.5)
                mat(p + 'mix.uv', H * E, C, s=C ** -0.5)
                mat(p + 'mix.sink', H, s=0.5)
                mat(p + 'mix.o', W, H * E, s=(H * E) ** -0.5)
            mlp = l.get('mlp')
            if not mlp:
                continue
            mat(p + 'norm2', W, s=0.1, mean=1.0)
            if mlp.get('kind', 'dense') == 'dense':
                F = int(mlp['ff'])
                mat(p + 'mlp.gate', F, W, s=W ** -0.5)
                mat(p + 'mlp.up', F, W, s=W ** -0.5)
                mat(p + 'mlp.down', W, F, s=F ** -0.5)
            else:
                r, F = mlp['router'], int(mlp['expert']['ff'])
                ne = int(r['experts']) + int(r.get('identity', 0))
                for e in range(int(r['experts'])):
                    mat(p + f'mlp.e{e}.gate', F, W, s=W ** -0.5)
                    mat(p + f'mlp.e{e}.up', F, W, s=W ** -0.5)
                    mat(p + f'mlp.e{e}.down', W, F, s=F ** -0.5)
                mat(p + 'mlp.router', ne, W, s=2.0 * W ** -0.5)
                mat(p + 'mlp.correction', ne, s=0.5 / ne)
        return cls(cfg, t)
