"""Small Narurax configurations and random weights for the tests (own generator: nothing of the product's random-weight code)."""
import numpy as np

from tolenex_cases import bf16_round


def moe(experts=6, top=2, ff=24):
    return {'kind': 'moe', 'expert': {'ff': ff}, 'router': {'experts': experts, 'top': top}}


def _mask(size, keep):
    return {'size': size, 'keep_first': keep} if size else None


def attn_layer(heads=6, kv_heads=3, dim=16, rot_dims=8, base=5000.0, size=37, keep=3, scale=None, mlp=None):
    """'attention': the values are the keys, sink, talking heads, gate per channel."""
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': dim, 'scale': scale or 1.6 / dim ** 0.5}
    if rot_dims:
        m['rot'] = {'dims': rot_dims, 'base': base}
    if size:
        m['mask'] = _mask(size, keep)
    return {'type': 'attention', 'mixer': m, 'mlp': mlp}


def attn2_layer(heads=4, kv_heads=2, dim=12, vdim=20, rot_dims=12, base=8000.0, scaling=True, size=29, keep=2, scale=None, mlp=None):
    """'attention_2': biases, weighted q / k norm, banded frequency scaling, one more 1 in the denominator."""
    m = {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'scale': scale or 3.0 / dim ** 0.5}
    if rot_dims:
        m['rot'] = {'dims': rot_dims, 'base': base}
        if scaling:
            m['rot']['scaling'] = {'factor': 8.0, 'low': 1.0, 'high': 3.0, 'original': 48}
    if size:
        m['mask'] = _mask(size, keep)
    return {'type': 'attention_2', 'mixer': m, 'mlp': mlp}


def delta_layer(heads=4, kv_heads=2, dim=10, vdim=12, conv=4, mlp=None):
    return {'type': 'channel_delta', 'mixer': {'heads': heads, 'kv_heads': kv_heads, 'dim': dim, 'vdim': vdim, 'conv': conv}, 'mlp': mlp}


def make_config(layers, width=96, vocab=211, eps=1e-5, bigram=(53, 31, 5)):
    cfg = {'architecture': 'Narurax', 'vocab': vocab, 'width': width, 'norm': {'eps': eps}, 'layers': layers}
    if bigram:
        cfg['embedding'] = {'bigram': {'buckets': bigram[0], 'mul_prev': bigram[1], 'mul_cur': bigram[2]}}
    return cfg


def random_weights(cfg, seed=0, ranks=(9, 11)):
    """name -> fp32 array of bfloat16-representable values, sized by cfg; scaled so that scores, gates, decays and logits are O(1)."""
    rng = np.random.default_rng(seed)
    W, w = cfg['width'], {}

    def put(name, *shape, std=1.0, mean=0.0):
        w[name] = bf16_round(rng.standard_normal(shape).astype(np.float32) * std + mean)

    put('embed', cfg['vocab'], W)
    bg = (cfg.get('embedding') or {}).get('bigram')
    if bg:
        put('bigram', bg['buckets'] + 1, W, std=0.7)
    put('head', cfg['vocab'], W, std=2.0 / W ** 0.5)
    put('final.norm', W, std=0.2, mean=1.0)
    for i, layer in enumerate(cfg['layers']):
        p, m = f'l{i}.', layer['mixer']
        H, G, D, E = m['heads'], m['kv_heads'], m['dim'], m['vdim']
        put(p + 'norm1', W, std=0.2, mean=1.0)
        w[p + 'shift'] = bf16_round(rng.uniform(0.0, 1.0, W).astype(np.float32))
        if layer['type'] == 'channel_delta':
            K = m['conv']
            for n, rows in (('q', G * D), ('k', G * D), ('v', H * E)):
                put(p + 'mix.' + n, rows, W, std=1.5 / W ** 0.5)
                put(p + f'mix.{n}.conv', rows, K, std=1.0 / K ** 0.5)
            put(p + 'mix.b', H, W, std=2.0 / W ** 0.5)
            w[p + 'mix.A_log'] = bf16_round(np.log(rng.uniform(0.02, 1.0, H)).astype(np.float32))
            put(p + 'mix.norm', E, std=0.2, mean=1.0)
            put(p + 'mix.a1', ranks[0], W, std=1.5 / W ** 0.5)
            put(p + 'mix.a2', H * D, ranks[0], std=1.5 / ranks[0] ** 0.5)
            put(p + 'mix.dt_bias', H * D, std=0.7, mean=-0.5)
            put(p + 'mix.g1', ranks[1], W, std=1.5 / W ** 0.5)
            put(p + 'mix.g2', H * E, ranks[1], std=1.5 / ranks[1] ** 0.5)
        else:
            put(p + 'mix.q', H * D, W, std=1.6 / W ** 0.5)
            put(p + 'mix.k', G * D, W, std=1.6 / W ** 0.5)
            if layer['type'] == 'attention':
                put(p + 'mix.sink', H, std=1.0, mean=0.5)
                w[p + 'mix.talk'] = bf16_round((np.eye(H) * 0.8 + 0.4 * rng.standard_normal((H, H))).astype(np.float32))
                put(p + 'mix.g', H * E, W, std=1.5 / W ** 0.5)
            else:
                put(p + 'mix.v', G * E, W, std=1.0 / W ** 0.5)
                put(p + 'mix.q.b', H * D, std=0.3)
                put(p + 'mix.k.b', G * D, std=0.3)
                put(p + 'mix.v.b', G * E, std=0.3)
                put(p + 'mix.o.b', W, std=0.3)
                put(p + 'mix.q.norm', D, std=0.3, mean=1.0)
                put(p + 'mix.k.norm', D, std=0.3, mean=1.0)
        put(p + 'mix.o', W, H * E, std=1.0 / (H * E) ** 0.5)
        mlp = layer.get('mlp')
        if not mlp:
            continue
        put(p + 'norm2', W, std=0.2, mean=1.0)
        F = mlp['expert']['ff']
        for e in range(mlp['router']['experts']):
            put(p + f'mlp.e{e}.gate', F, W, std=1.5 / W ** 0.5)
            put(p + f'mlp.e{e}.up', F, W, std=1.5 / W ** 0.5)
            put(p + f'mlp.e{e}.down', W, F, std=1.5 / F ** 0.5)
        put(p + 'mlp.router', mlp['router']['experts'], W, std=2.0 / W ** 0.5)
    return w


def as_model(cfg, w):
    """The product's model object over these weights (bfloat16 bit patterns, as a checkpoint reader would deliver them)."""
    from tensorrt_llm.models.narurax.model import NaruraxConfig, NaruraxForCausalLM
    tensors = {k: ((np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(v.shape), 'bfloat16')
               for k, v in w.items()}
    return NaruraxForCausalLM(NaruraxConfig(cfg), tensors)


def decisive_router(cfg, w, seed=0, gain=3.0):
    """Rewrites w so that no router decision is a close call (for the bfloat16 engine, whose rounding moves scores by a percent):
    the last channels of the residual are reserved - no mixer or feed-forward writes to them and the pair table is zero there, so
    they hold what the token's embedding put there, a per-token ranking of the experts - and every router reads nothing but its own
    channel of them.  Logits of neighbouring ranks then differ by gain * 4 / experts / rms(x)."""
    rng = np.random.default_rng(seed)
    ne = max([l['mlp']['router']['experts'] for l in cfg['layers'] if l.get('mlp')])
    for k in w:
        if k.endswith('mix.o') or k.endswith('.down'):
            w[k][-ne:, :] = 0.0
        if k.endswith('mix.o.b') or k == 'bigram':
            w[k][..., -ne:] = 0.0
        if k.endswith('norm2'):
            w[k][-ne:] = 1.0
    ranking = np.stack([rng.permutation(ne) for _ in range(cfg['vocab'])]).astype(np.float32) - (ne - 1) / 2.0
    w['embed'][:, -ne:] = bf16_round(ranking * np.float32(4.0 / ne))   # within +-2 whatever the number of experts: no score saturates
    for i, l in enumerate(cfg['layers']):
        if not l.get('mlp'):
            continue
        n = l['mlp']['router']['experts']
        r = np.zeros_like(w[f'l{i}.mlp.router'])
        r[np.arange(n), r.shape[1] - ne + np.arange(n)] = gain
        w[f'l{i}.mlp.router'] = r
    return w
