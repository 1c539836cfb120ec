"""Narurax: a pre-norm decoder stack - x <- x + mixer(shift(norm1(x))), x <- x + ff(norm2(x)) - with plain RMS norms, whose layers
are listed one by one in config.json.  The embedding adds a hashed row of a pair table per (previous token, token); every mixer
reads its normed input blended with the previous token's (token shift, a learned per-channel ratio).  Three mixers

  attention       grouped-query attention without a value projection (a token's value is its key as projected), neighbour-pair
                  rotation, a sliding window that also keeps the sequence's first tokens, a softmax whose denominator holds a
                  per-head sink, the normalised weights mixed across heads by a learned matrix, an elementwise sigmoid gate
  attention_2     grouped-query attention with biased projections, weighted RMS norm of q and k per head, rotation with
                  three-band frequency scaling, the same mask, a softmax whose denominator holds one more 1
  channel_delta   the gated delta rule with a decay per key channel: q | k | v through a short causal convolution and silu, unit
                  q and k, beta and the decay from the input (the decay through a low-rank pair), RMS norm per head, a low-rank
                  sigmoid gate.  State and convolution tail live in a state slot

and one feed-forward: a routed mixture of experts W_down (silu(W_gate a) * W_up a), a = s h, with sigmoid router scores s, the `top`
largest chosen and used as they are.

This class reads config.json and the safetensors file and describes the stack to the ragged engine (runtime/stack.py).  What the
design fixes lives here (which options each mixer kind switches on, the activations); every size and every other constant is read
from the configuration or, for the two low-rank pairs, from the tensors' shapes."""
import json
from typing import Dict, Optional

import numpy as np

from ..stack_model import PAGE_SIZE, StackModelForCausalLM, to_bf16_bits

MIXERS = ('attention', 'attention_2', 'channel_delta')


class NaruraxConfig(object):
    """config.json: architecture, vocab, width, norm.eps, embedding.bigram{buckets, mul_prev, mul_cur},
    layers[i].{type, mixer{...}, mlp{kind: moe, expert{ff}, router{experts, top}} | null}."""

    def __init__(self, d: Dict, ranks: Optional[Dict] = None):
        self.raw = d
        self.vocab, self.width = int(d['vocab']), int(d['width'])
        self.norm_eps = float((d.get('norm') or {}).get('eps', 1e-6))
        self.bigram = (d.get('embedding') or {}).get('bigram')
        self.layers = d['layers']
        self.ranks = dict(ranks or {})   # layer index -> (decay rank, gate rank) of a channel_delta layer
        for i, l in enumerate(self.layers):
            if l['type'] not in MIXERS:
                raise ValueError(f"layer {i}: mixer type {l['type']!r} is not one this design has {MIXERS}")
            mlp = l.get('mlp')
            if mlp is not None and mlp.get('kind', 'moe') != 'moe':
                raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} (moe)")

    @staticmethod
    def from_json_file(path: str) -> 'NaruraxConfig':
        with open(path) as f:
            return NaruraxConfig(json.load(f))

    def default_rank(self, i: int) -> int:
        return max(8, self.width // 8)

    def engine_config(self) -> Dict:
        c = dict(width=self.width, vocab=self.vocab, num_layers=len(self.layers), norm_groups=1, norm_eps=repr(self.norm_eps),
                 norm_offset=0, embedding_scale=1, page_size=PAGE_SIZE, block='sequential', residual='hyper', streams=1, token_shift=1)
        if self.bigram:
            c.update(pair_buckets=int(self.bigram['buckets']), pair_mul_prev=int(self.bigram['mul_prev']),
                     pair_mul_cur=int(self.bigram['mul_cur']))
        for i, l in enumerate(self.layers):
            p, m = f'layer.{i}.', l['mixer']
            c[p + 'heads'], c[p + 'kv_heads'] = int(m['heads']), int(m.get('kv_heads', m['heads']))
            # an 'attention' layer's values are its keys: their size is the key size
            c[p + 'dim'], c[p + 'vdim'] = int(m['dim']), int(m['dim'] if l['type'] == 'attention' else m.get('vdim', m['dim']))
            if l['type'] == 'channel_delta':
                c[p + 'type'], c[p + 'conv'] = 'delta_rule', int(m['conv'])
                ra, rg = self.ranks.get(i, (self.default_rank(i), self.default_rank(i)))
                c[p + 'decay_rank'], c[p + 'gate_rank'] = int(ra), int(rg)
            else:
                c[p + 'type'] = 'attention'
                rot, mask = m.get('rot') or {}, m.get('mask') or {}
                c[p + 'scale'] = repr(float(m['scale']))
                c[p + 'rot_dims'], c[p + 'rot_base'] = int(rot.get('dims', 0)), repr(float(rot.get('base', 10000.0)))
                sc = rot.get('scaling')
                if sc:
                    c[p + 'rot_scaling'] = 'banded'
                    c[p + 'rot_factor'], c[p + 'rot_original'] = repr(float(sc['factor'])), repr(float(sc['original']))
                    c[p + 'rot_low'], c[p + 'rot_high'] = repr(float(sc['low'])), repr(float(sc['high']))
                if 'size' in mask:
                    c[p + 'mask'], c[p + 'mask_size'] = 'window', int(mask['size'])
                    c[p + 'mask_keep'] = int(mask.get('keep_first', 0))
                else:
                    c[p + 'mask'] = 'causal'
                if l['type'] == 'attention':
                    # no value projection, a learned sink, head-mixed weights, a gate per output channel
                    c[p + 'values_are_keys'], c[p + 'sink'], c[p + 'talk'], c[p + 'out_gate'], c[p + 'gate_wide'] = 1, 1, 1, 1, 1
                else:
                    # biases, weighted q / k norm, a constant sink of logit 0
                    c[p + 'qkv_bias'], c[p + 'o_bias'], c[p + 'qk_norm'], c[p + 'qk_norm_weight'], c[p + 'sink'] = 1, 1, 1, 1, 2
            mlp = l.get('mlp')
            if not mlp:
                c[p + 'ff'] = 0
            else:
                r = mlp['router']
                c[p + 'ff'], c[p + 'mlp'] = int(mlp['expert']['ff']), 'moe'
                c[p + 'experts'], c[p + 'identity'], c[p + 'top'] = int(r['experts']), 0, int(r['top'])
                c[p + 'route_score'], c[p + 'route_weight'] = 'sigmoid', 'input'
        return c


class NaruraxForCausalLM(StackModelForCausalLM):
    architecture = 'Narurax'
    config_class = NaruraxConfig

    def __init__(self, config, tensors: Dict):
        super().__init__(config, tensors)
        # the ranks of a channel_delta layer's two low-rank pairs are the shapes of their first halves
        for i, l in enumerate(config.layers):
            if l['type'] == 'channel_delta' and f'l{i}.mix.a1' in tensors and f'l{i}.mix.g1' in tensors:
                config.ranks[i] = (int(tensors[f'l{i}.mix.a1'][0].shape[0]), int(tensors[f'l{i}.mix.g1'][0].shape[0]))

    @classmethod
    def from_random(cls, config: Dict, seed: int = 0, ranks: Optional[Dict] = None) -> 'NaruraxForCausalLM':
        """Random bfloat16-valued weights of the configuration's shapes (benchmarks, examples, tests)."""
        cfg = config if isinstance(config, NaruraxConfig) else NaruraxConfig(config, ranks)
        rng = np.random.default_rng(seed)
        t = {}

        def mat(name, *shape, s=1.0, mean=0.0):
            a = (rng.standard_normal(shape, dtype=np.float32) * s + mean).astype(np.float32)
            t[name] = (to_bf16_bits(a), 'bfloat16')

        W = cfg.width
        mat('embed', cfg.vocab, W)
        if cfg.bigram:
            mat('bigram', int(cfg.bigram['buckets']) + 1, W, s=0.5)
        mat('head', cfg.vocab, W, s=W ** -0.5)
        mat('final.norm', W, s=0.1, mean=1.0)
        for i, l in enumerate(cfg.layers):
            p, m = f'l{i}.', l['mixer']
            H, G, D = int(m['heads']), int(m.get('kv_heads', m['heads'])), int(m['dim'])
            E = int(m.get('vdim', D))
            mat(p + 'norm1', W, s=0.1, mean=1.0)
            t[p + 'shift'] = (to_bf16_bits(rng.uniform(0.0, 1.0, W).astype(np.float32)), 'bfloat16')
            if l['type'] == 'channel_delta':
                K = int(m['conv'])
                ra, rg = cfg.ranks.get(i, (cfg.default_rank(i), cfg.default_rank(i)))
                for n, rows in (('q', G * D), ('k', G * D), ('v', H * E)):
                    mat(p + 'mix.' + n, rows, W, s=W ** -0.5)
                    mat(p + f'mix.{n}.conv', rows, K, s=K ** -0.5)
                mat(p + 'mix.b', H, W, s=W ** -0.5)
                t[p + 'mix.A_log'] = (to_bf16_bits(np.log(rng.uniform(0.05, 1.0, H)).astype(np.float32)), 'bfloat16')
                mat(p + 'mix.norm', E, s=0.1, mean=1.0)
                mat(p + 'mix.a1', ra, W, s=W ** -0.5)
                mat(p + 'mix.a2', H * D, ra, s=ra ** -0.5)
                mat(p + 'mix.dt_bias', H * D, s=0.5, mean=-1.0)
                mat(p + 'mix.g1', rg, W, s=W ** -0.5)
                mat(p + 'mix.g2', H * E, rg, s=rg ** -0.5)
                mat(p + 'mix.o', W, H * E, s=(H * E) ** -0.5)
            else:
                mat(p + 'mix.q', H * D, W, s=W ** -0.5)
                mat(p + 'mix.k', G * D, W, s=W ** -0.5)
                mat(p + 'mix.o', W, H * E, s=(H * E) ** -0.5)
                if l['type'] == 'attention':
                    mat(p + 'mix.sink', H, s=0.5)
                    t[p + 'mix.talk'] = (to_bf16_bits((np.eye(H) + 0.3 * rng.standard_normal((H, H))).astype(np.float32)), 'bfloat16')
                    mat(p + 'mix.g', H * E, W, s=W ** -0.5)
                else:
                    mat(p + 'mix.v', G * E, W, s=W ** -0.5)
                    mat(p + 'mix.q.b', H * D, s=0.1)
                    mat(p + 'mix.k.b', G * D, s=0.1)
                    mat(p + 'mix.v.b', G * E, s=0.1)
                    mat(p + 'mix.o.b', W, s=0.1)
                    mat(p + 'mix.q.norm', D, s=0.1, mean=1.0)
                    mat(p + 'mix.k.norm', D, s=0.1, mean=1.0)
            mlp = l.get('mlp')
            if not mlp:
                continue
            mat(p + 'norm2', W, s=0.1, mean=1.0)
            F = int(mlp['expert']['ff'])
            for e in range(int(mlp['router']['experts'])):
                mat(p + f'mlp.e{e}.gate', F, W, s=W ** -0.5)
                mat(p + f'mlp.e{e}.up', F, W, s=W ** -0.5)
                mat(p + f'mlp.e{e}.down', W, F, s=F ** -0.5)
            mat(p + 'mlp.router', int(mlp['router']['experts']), W, s=2.0 * W ** -0.5)
        return cls(cfg, t)
