"""Small Rofozen configurations and random weights for the tests (own generator: nothing of the product's random-weight code)."""
import numpy as np

from tolenex_cases import bf16_round


def dense(ff=72):
    return {'kind': 'dense', 'ff': ff} if ff else None


def moe(experts=6, identity=2, top=2, count=2, keep=1, ff=24, scale=1.75):
    return {'kind': 'moe', 'expert': {'ff': ff},
            'router': {'experts': experts, 'identity': identity, 'top': top, 'scale': scale, 'groups': {'count': count, 'keep': keep}}}


def mamba_layer(heads=6, vdim=12, state=10, groups=3, conv=4, norm_groups=2, mlp=None):
    m = {'heads': heads, 'vdim': vdim, 'state': state, 'groups': groups, 'conv': conv, 'norm_groups': norm_groups}
    return {'type': 'mamba2', 'mixer': m, 'mlp': mlp}


def latent_layer(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, q_rank=28, size=37, base=5000.0, scaling=True, mlp=None):
    rot = {'dims': rot_dim, 'base': base}
    if scaling:
        rot['scaling'] = {'factor': 8.0, 'original': 64, 'fast': 16.0, 'slow': 2.0}
    m = {'heads': heads, 'dim': dim, 'rot_dim': rot_dim, 'vdim': vdim, 'kv_rank': kv_rank, 'q_rank': q_rank,
         'scale': 1.5 / (dim + rot_dim) ** 0.5, 'rot': rot}
    if size:
        m['mask'] = {'size': size}
    return {'type': 'latent_attention', 'mixer': m, 'mlp': mlp}


def shared(layer, j):
    """A layer that runs on layer j's weights: the same entry plus weights_of."""
    out = dict(layer)
    out['weights_of'] = j
    return out


def make_config(layers, width=96, vocab=211, eps=1e-5):
    return {'architecture': 'Rofozen', 'vocab': vocab, 'width': width, 'norm': {'eps': eps}, 'layers': layers}


def random_weights(cfg, seed=0):
    """name -> fp32 array of bfloat16-representable values, sized by cfg; scaled so that scores, gates, steps and logits are O(1)."""
    rng = np.random.default_rng(seed)
    W, w = cfg['width'], {}

    def put(name, *shape, std=1.0, mean=0.0):
        w[name] = bf16_round(rng.standard_normal(shape).astype(np.float32) * std + mean)

    put('embed', cfg['vocab'], W)
    put('head', cfg['vocab'], W, std=2.0 / W ** 0.5)
    put('final.norm', W, std=0.2, mean=1.0)
    for i, layer in enumerate(cfg['layers']):
        if layer.get('weights_of') is not None:
            continue
        p, m = f'l{i}.', layer['mixer']
        H, E = m['heads'], m['vdim']
        put(p + 'norm1', W, std=0.2, mean=1.0)
        if layer['type'] == 'mamba2':
            N, G, K = m['state'], m['groups'], m['conv']
            inner = H * E
            ch = inner + 2 * G * N
            put(p + 'mix.in', 2 * inner + 2 * G * N + H, W, std=1.5 / W ** 0.5)
            put(p + 'mix.conv', ch, K, std=1.0 / K ** 0.5)
            put(p + 'mix.conv.b', ch, std=0.2)
            put(p + 'mix.dt_bias', H, std=0.7, mean=-0.5)
            w[p + 'mix.A_log'] = bf16_round(np.log(rng.uniform(0.05, 3.0, H)).astype(np.float32))
            put(p + 'mix.D', H, std=0.5, mean=0.5)
            put(p + 'mix.norm', inner, std=0.2, mean=1.0)
            put(p + 'mix.o', W, inner, std=1.0 / inner ** 0.5)
        else:
            D, C, Q, R = m['dim'], m['kv_rank'], m['q_rank'], m['rot_dim']
            put(p + 'mix.dq', Q, W, std=1.5 / W ** 0.5)
            put(p + 'mix.dq.norm', Q, std=0.2, mean=1.0)
            put(p + 'mix.uq', H * (D + R), Q, std=1.5 / Q ** 0.5)
            put(p + 'mix.dkv', C + R, W, std=1.5 / W ** 0.5)
            put(p + 'mix.dkv.norm', C, std=0.2, mean=1.0)
            put(p + 'mix.uk', H * D, C, std=1.5 / C ** 0.5)
            put(p + 'mix.uv', H * E, C, std=1.0 / C ** 0.5)
            put(p + 'mix.sink', H, std=1.0, mean=1.0)
            put(p + 'mix.o', W, H * E, std=1.0 / (H * E) ** 0.5)
        mlp = layer.get('mlp')
        if not mlp:
            continue
        put(p + 'norm2', W, std=0.2, mean=1.0)
        if mlp['kind'] == 'dense':
            F = mlp['ff']
            put(p + 'mlp.gate', F, W, std=1.5 / W ** 0.5)
            put(p + 'mlp.up', F, W, std=1.5 / W ** 0.5)
            put(p + 'mlp.down', W, F, std=1.0 / F ** 0.5)
        else:
            r, F = mlp['router'], mlp['expert']['ff']
            ne = r['experts'] + r['identity']
            for e in range(r['experts']):
                put(p + f'mlp.e{e}.gate', F, W, std=1.5 / W ** 0.5)
                put(p + f'mlp.e{e}.up', F, W, std=1.5 / W ** 0.5)
                put(p + f'mlp.e{e}.down', W, F, std=1.0 / F ** 0.5)
            put(p + 'mlp.router', ne, W, std=3.0 / W ** 0.5)
            put(p + 'mlp.correction', ne, std=0.3 / ne)
    return w


def as_model(cfg, w):
    """The product's model object over these weights (bfloat16 bit patterns, as a checkpoint reader would deliver them)."""
    from tensorrt_llm.models.rofozen.model import RofozenConfig, RofozenForCausalLM
    tensors = {k: ((np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(v.shape), 'bfloat16')
               for k, v in w.items()}
    return RofozenForCausalLM(RofozenConfig(cfg), tensors)


def decisive_router(cfg, w, seed=0, gain=8.0):
    """Rewrites w so that no router decision is a close call (for the bfloat16 engine, whose rounding moves scores by a percent):
    the last channels of the residual are reserved - no mixer or feed-forward writes to them, so they hold what the embedding put
    there, a per-token ranking of the router's outputs - and every router reads nothing but its own channel of them.  Logits of
    neighbouring ranks then differ by gain / rms(x), so scores of neighbouring ranks differ by a factor; the correction is zero (with
    random weights it is at work in the float32 tests)."""
    rng = np.random.default_rng(seed)
    ne = max([l['mlp']['router']['experts'] + l['mlp']['router']['identity'] for l in cfg['layers'] if l.get('mlp') and l['mlp']['kind'] == 'moe'])
    for k in w:
        if k.endswith('mix.o') or k.endswith('.down'):
            w[k][-ne:, :] = 0.0
        if k.endswith('norm2'):
            w[k][-ne:] = 1.0
    w['embed'][:, -ne:] = np.stack([rng.permutation(ne) for _ in range(cfg['vocab'])]).astype(np.float32)
    for i, l in enumerate(cfg['layers']):
        mlp = l.get('mlp')
        if not mlp or mlp['kind'] != 'moe' or l.get('weights_of') is not None:
            continue
        n = mlp['router']['experts'] + mlp['router']['identity']
        r = np.zeros_like(w[f'l{i}.mlp.router'])
        r[np.arange(n), r.shape[1] - ne + np.arange(n)] = gain
        w[f'l{i}.mlp.router'] = r
        w[f'l{i}.mlp.correction'] = np.zeros(n, np.float32)
    return w


def routing_margin(cfg, w, toks):
    """The smallest relative gap (a - b) / (|a| + |b|), over tokens and routed layers, between a value that decides a router's
    choice and the next one (group values at the keep border, choice values at the top border) on the float64 oracle: a model whose
    margin is tiny would make a test rest on a close call."""
    from oracle import rofozen_oracle as O
    wf = {k: v.astype(np.float64) for k, v in w.items()}
    x = wf['embed'][np.asarray(toks)]
    eps = cfg['norm']['eps']
    worst = np.inf
    for i, l in enumerate(cfg['layers']):
        p = f"l{O.weight_layer(cfg, i)}."
        h = O.rms_norm(x, wf[p + 'norm1'], eps)
        x = x + (O.mamba2(h, wf, p + 'mix.', l['mixer'], eps) if l['type'] == 'mamba2' else O.latent_attention(h, wf, p + 'mix.', l['mixer'], eps))
        mlp = l.get('mlp')
        if not mlp:
            continue
        h = O.rms_norm(x, wf[p + 'norm2'], eps)
        if mlp['kind'] != 'moe':
            x = x + O.dense_ff(h, wf, p + 'mlp.')
            continue
        r = mlp['router']
        z = h @ wf[p + 'mlp.router'].T
        s = np.exp(z - z.max(-1, keepdims=True))
        s /= s.sum(-1, keepdims=True)
        c = s + wf[p + 'mlp.correction']
        cnt, keep = r['groups']['count'], r['groups']['keep']
        allowed = np.ones_like(c, bool)
        if keep < cnt:
            best = c.reshape(len(toks), cnt, -1).max(-1)
            g = np.sort(best, axis=-1)[:, ::-1]
            worst = min(worst, ((g[:, keep - 1] - g[:, keep]) / (np.abs(g[:, keep - 1]) + np.abs(g[:, keep]))).min())
            kept = np.argsort(-best, -1, kind='stable')[:, :keep]
            a = np.zeros((len(toks), cnt), bool)
            np.put_along_axis(a, kept, True, -1)
            allowed = np.repeat(a, c.shape[1] // cnt, axis=1)
        ranked = np.sort(np.where(allowed, c, -np.inf), axis=-1)[:, ::-1]
        if ranked.shape[1] > r['top']:
            a, b = ranked[:, r['top'] - 1], ranked[:, r['top']]
            ok = np.isfinite(b)
            if ok.any():
                worst = min(worst, ((a[ok] - b[ok]) / (np.abs(a[ok]) + np.abs(b[ok]))).min())
        x = x + O.moe_ff(h, wf, p + 'mlp.', mlp)
    return worst
