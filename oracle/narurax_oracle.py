"""Plain float64 numpy statement of the Narurax design, one function per mechanism.  Test infrastructure only: slow, whole
sequences, no cache, no batching - the product (the stack engine) never touches it and shares no code with it.

Narurax is a pre-norm decoder stack, x <- x + mixer(shift(n1(x))), x <- x + ff(n2(x)), with plain RMS norms.  The embedding adds a
hashed row per (previous token, token) pair.  The mixer's input is blended with the previous token's (token shift).  Mixers:
  'attention'      grouped-query, the values ARE the unrotated keys; neighbour-pair rotation; a sliding window that also keeps the
                   sequence's first tokens; a softmax whose denominator holds exp(sink_h); the normalised weights are then mixed
                   across heads by a matrix T ("talking heads": head h applies sum_g T[h, g] p_g to the values of its own key/value
                   head); an elementwise sigmoid gate on the concatenated heads;
  'attention_2'    grouped-query with biased projections, RMS-normed q and k per head (weighted), rotation with the three-band
                   frequency scaling, the same mask, a softmax whose denominator holds 1;
  'channel_delta'  gated delta rule with one decay per key channel: q, k, v through a short causal convolution and silu, q and k
                   made unit vectors, S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q; RMS norm per head, a low-rank
                   sigmoid gate.
Feed-forward: a routed mixture W_down (silu(W_gate a) * W_up a) with a = s_e h, s = sigmoid(router logits), the `top` largest.

Notation: n tokens, width W.  `w` is a dict name -> float64 array with the checkpoint's names; `cfg` is the parsed config.json."""
import math

import numpy as np

# inside `with rounding(fn):` every projection's output, norm output, convolution output, attention weight and hidden activation
# passes through fn (for instance a rounding to bfloat16): an estimate of a row's conditioning, not a model of any engine
_round = None


class rounding(object):
    def __init__(self, fn):
        self.fn = fn

    def __enter__(self):
        global _round
        self.old, _round = _round, self.fn

    def __exit__(self, *exc):
        global _round
        _round = self.old


def _r(x):
    return x if _round is None else _round(x)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_norm(x, weight, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * weight


# ------------------------------------------------------------------------------------------------ embedding, token shift
def bigram_rows(tokens, bg):
    """Row of the pair table for every token: (prev * mul_prev + cur * mul_cur) mod buckets, the extra last row for the first."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(int(bg['buckets']) if t == 0 else (int(tokens[t - 1]) * int(bg['mul_prev']) + int(tok) * int(bg['mul_cur'])) % int(bg['buckets']))
    return rows


def embed(tokens, w, cfg):
    x = w['embed'][np.asarray(tokens)]
    bg = (cfg.get('embedding') or {}).get('bigram')
    if bg:
        x = x + w['bigram'][np.asarray(bigram_rows(tokens, bg))]
    return x


def token_shift(h, mu):
    """h_t + (h_{t-1} - h_t) * mu, with h_{-1} = 0; the neighbour is the unshifted row."""
    prev = np.concatenate([np.zeros((1, h.shape[1])), h[:-1]], axis=0)
    return h + (prev - h) * mu[None, :]


# ------------------------------------------------------------------------------------------------ rotation
def plain_frequencies(dims, base):
    i = np.arange(dims // 2, dtype=np.float64)
    return base ** (-2.0 * i / dims)


def banded_frequencies(dims, base, sc):
    """Three bands by wavelength l = 2 pi / f against the original length L: short waves (l < L / high) keep f, long ones
    (l > L / low) get f / factor, between them a blend by s = (L / l - low) / (high - low)."""
    f = plain_frequencies(dims, base)
    if not sc:
        return f
    factor, lo, hi, L = float(sc['factor']), float(sc['low']), float(sc['high']), float(sc['original'])
    out = f.copy()
    for i, fi in enumerate(f):
        l = 2.0 * math.pi / fi
        if l < L / hi:
            out[i] = fi
        elif l > L / lo:
            out[i] = fi / factor
        else:
            s = (L / l - lo) / (hi - lo)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_pairs(x, positions, dims, freq):
    """x [n, heads, D]: dimensions (2i, 2i + 1), i < dims / 2, turn by positions * freq[i]; the rest pass."""
    if not dims:
        return x
    ang = positions.astype(np.float64)[:, None] * freq[None, :]
    cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cs - v * sn
    out[..., 1:dims:2] = v * cs + u * sn
    return out


# ------------------------------------------------------------------------------------------------ attention
def visible(n, size, keep_first):
    """[n, n] bool: row i sees key j <= i that lies within the last `size` positions or among the first `keep_first`."""
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def sink_softmax(scores, mask, sink):
    """scores [H, n, n], sink [H] logits that join the denominator only -> weights [H, n, n] (rows sum to less than one)."""
    s = np.where(mask[None], scores, -np.inf)
    m = np.maximum(s.max(axis=-1, keepdims=True), sink[:, None, None])
    e = np.exp(s - m)
    return e / (e.sum(axis=-1, keepdims=True) + np.exp(sink[:, None, None] - m))


def mask_of(m, n):
    mk = m.get('mask') or {}
    return visible(n, int(mk.get('size', n + 1)), int(mk.get('keep_first', 0)))


def attention(h, w, p, m, eps):
    """Mixer 'attention'.  h [n, W] -> [n, W]."""
    n = h.shape[0]
    H, G, D = int(m['heads']), int(m['kv_heads']), int(m['dim'])
    rot = m.get('rot') or {}
    pos = np.arange(n)
    q = _r(h @ w[p + 'q'].T).reshape(n, H, D)
    k = _r(h @ w[p + 'k'].T).reshape(n, G, D)
    v = k                                                              # the values are the keys as projected
    dims = int(rot.get('dims', 0))
    freq = banded_frequencies(dims, float(rot.get('base', 10000.0)), rot.get('scaling')) if dims else None
    qr, kr = rotate_pairs(q, pos, dims, freq), rotate_pairs(k, pos, dims, freq)
    kv_of = np.arange(H) // (H // G)
    scores = np.einsum('ihd,jhd->hij', qr, kr[:, kv_of]) * float(m['scale'])
    pw = _r(sink_softmax(scores, mask_of(m, n), w[p + 'sink']))
    pw = np.einsum('hg,gij->hij', w[p + 'talk'], pw)                   # weights of head g join head h with T[h, g]
    o = np.einsum('hij,jhe->ihe', pw, v[:, kv_of]).reshape(n, H * D)
    o = _r(o) * sigmoid(_r(h @ w[p + 'g'].T))
    return _r(o) @ w[p + 'o'].T


def attention_2(h, w, p, m, eps):
    """Mixer 'attention_2'.  h [n, W] -> [n, W]."""
    n = h.shape[0]
    H, G, D, E = int(m['heads']), int(m['kv_heads']), int(m['dim']), int(m['vdim'])
    rot = m.get('rot') or {}
    pos = np.arange(n)
    q = _r(h @ w[p + 'q'].T + w[p + 'q.b']).reshape(n, H, D)
    k = _r(h @ w[p + 'k'].T + w[p + 'k.b']).reshape(n, G, D)
    v = _r(h @ w[p + 'v'].T + w[p + 'v.b']).reshape(n, G, E)
    q, k = rms_norm(q, w[p + 'q.norm'], eps), rms_norm(k, w[p + 'k.norm'], eps)
    dims = int(rot.get('dims', 0))
    freq = banded_frequencies(dims, float(rot.get('base', 10000.0)), rot.get('scaling')) if dims else None
    q, k = _r(rotate_pairs(q, pos, dims, freq)), _r(rotate_pairs(k, pos, dims, freq))
    kv_of = np.arange(H) // (H // G)
    scores = np.einsum('ihd,jhd->hij', q, k[:, kv_of]) * float(m['scale'])
    pw = _r(sink_softmax(scores, mask_of(m, n), np.zeros(H)))         # exp(0) = 1 joins the denominator
    o = np.einsum('hij,jhe->ihe', pw, v[:, kv_of]).reshape(n, H * E)
    return _r(o) @ w[p + 'o'].T + w[p + 'o.b']


# ------------------------------------------------------------------------------------------------ channel_delta
def causal_conv(u, kernel):
    """u [n, C], kernel [C, taps] whose last column meets the current token, zeros ahead of the sequence, no bias."""
    n, taps = u.shape[0], kernel.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], axis=0)
    out = np.zeros((n, u.shape[1]))
    for t in range(taps):
        out += padded[t:t + n] * kernel[None, :, t]
    return out


def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def delta_scan(q, k, v, beta, g):
    """q, k, g [n, H, D]; v [n, H, E]; beta [n, H] -> o [n, H, E], with S [H, D, E] from zero:
    S <- g_t * S (rows); u = beta_t (v_t - S^T k_t); S <- S + k_t u^T; o_t = S^T q_t."""
    n, H, D = q.shape
    E = v.shape[-1]
    S = np.zeros((H, D, E))
    o = np.zeros((n, H, E))
    for t in range(n):
        S = g[t][:, :, None] * S
        u = beta[t][:, None] * (v[t] - np.einsum('hde,hd->he', S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        o[t] = np.einsum('hde,hd->he', S, q[t])
    return o


def channel_delta(h, w, p, m, eps):
    """Mixer 'channel_delta'.  h [n, W] -> [n, W]."""
    n = h.shape[0]
    H, G, D, E = int(m['heads']), int(m['kv_heads']), int(m['dim']), int(m['vdim'])
    q = _r(silu(causal_conv(_r(h @ w[p + 'q'].T), w[p + 'q.conv']))).reshape(n, G, D)
    k = _r(silu(causal_conv(_r(h @ w[p + 'k'].T), w[p + 'k.conv']))).reshape(n, G, D)
    v = _r(silu(causal_conv(_r(h @ w[p + 'v'].T), w[p + 'v.conv']))).reshape(n, H, E)
    q, k = unit(q) * D ** -0.5, unit(k)
    qk_of = np.arange(H) // (H // G)
    q, k = q[:, qk_of], k[:, qk_of]
    beta = sigmoid(_r(h @ w[p + 'b'].T))
    a = _r(_r(h @ w[p + 'a1'].T) @ w[p + 'a2'].T) + w[p + 'dt_bias']
    g = np.exp(-np.exp(np.repeat(w[p + 'A_log'], D))[None, :] * softplus(a)).reshape(n, H, D)
    o = delta_scan(q, k, v, beta, g)
    o = rms_norm(o, w[p + 'norm'], eps).reshape(n, H * E)
    o = o * sigmoid(_r(_r(h @ w[p + 'g1'].T) @ w[p + 'g2'].T))
    return _r(o) @ w[p + 'o'].T


# ------------------------------------------------------------------------------------------------ feed-forward
# a list here collects, per routed layer, the smallest relative gap between the last chosen logit and the first one left out
margins = None


def route(h, w, p, r):
    """-> (indices [n, top], weights [n, top]): the `top` largest sigmoid scores, lowest index among equals; the weights are those scores as they are."""
    z = h @ w[p + 'router'].T
    s = sigmoid(z)
    top = int(r['top'])
    idx = np.argsort(-s, axis=-1, kind='stable')[:, :top]
    if margins is not None and s.shape[1] > top:
        ranked = np.sort(z, axis=-1)[:, ::-1]   # the scores rise with the logits: the gap is measured where rounding acts
        margins.append(((ranked[:, top - 1] - ranked[:, top]) / (np.abs(ranked[:, top - 1]) + np.abs(ranked[:, top]) + 1e-30)).min())
    return idx, np.take_along_axis(s, idx, axis=-1)


def moe(h, w, p, mlp):
    idx, wt = route(h, w, p, mlp['router'])
    y = np.zeros((h.shape[0], w[p + 'e0.down'].shape[0]))
    for t in range(h.shape[0]):
        for e, s in zip(idx[t], wt[t]):
            a = _r(s * h[t])                                           # the weight scales the expert's input
            ep = p + 'e%d.' % e
            hid = _r(silu(_r(a @ w[ep + 'gate'].T)) * _r(a @ w[ep + 'up'].T))
            y[t] += hid @ w[ep + 'down'].T
    return y


# ------------------------------------------------------------------------------------------------ the stack
MIXERS = {'attention': attention, 'attention_2': attention_2, 'channel_delta': channel_delta}


def logits(tokens, w, cfg):
    return forward(tokens, w, cfg)


def greedy(prompt, w, cfg, n_new):
    """The greedy continuation, recomputed from scratch for every token."""
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(np.argmax(forward(toks, w, cfg)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out


def routing_margin(tokens, w, cfg):
    """The smallest relative gap, over routed layers and tokens, between the logit of a chosen expert and the next one's."""
    global margins
    margins = []
    try:
        forward(tokens, w, cfg)
        return min(margins) if margins else np.inf
    finally:
        margins = None


def forward(tokens, w, cfg, taps=None):
    """Logits [n, vocab] of a whole sequence.  taps: a list that receives the residual stream behind every layer."""
    eps = float((cfg.get('norm') or {}).get('eps', 1e-6))
    x = embed(tokens, w, cfg)
    for i, l in enumerate(cfg['layers']):
        p = 'l%d.' % i
        h = _r(token_shift(rms_norm(x, w[p + 'norm1'], eps), w[p + 'shift']))
        x = x + MIXERS[l['type']](h, w, p + 'mix.', l['mixer'], eps)
        if l.get('mlp'):
            x = x + moe(_r(rms_norm(x, w[p + 'norm2'], eps)), w, p + 'mlp.', l['mlp'])
        if taps is not None:
            taps.append(x.copy())
    return _r(rms_norm(x, w['final.norm'], eps)) @ w['head'].T
