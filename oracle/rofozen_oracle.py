"""Plain float64 numpy statement of the Rofozen design, one function per mechanism.  Test infrastructure only: slow, whole
sequences, no cache, no batching - the product (the stack engine) never touches it and shares no code with it.

Rofozen is a pre-norm decoder stack, x <- x + mixer(n1(x)), x <- x + ff(n2(x)), with plain RMS norms, two mixers and two
feed-forwards:
  'mamba2'            a selective state-space layer: one projection gives a gate z, the inputs x, B, C of the recurrence and a
                      step size per head; x, B, C pass a short causal convolution per channel and silu; per head the state
                      S [N, P] follows S <- exp(-exp(A_log) dt) S + dt B x^T and the output is S^T C + D x; the output is gated by
                      silu(z), RMS-normed in equal parts of the row and projected back;
  'latent_attention'  queries through a normed low-rank latent; keys and values expanded from one normed latent per token, plus
                      one rotated key part shared by the heads (half-split pairs, frequencies blended between a scaled and an
                      unscaled set); a sliding window; a softmax whose denominator holds a per-head sink;
  dense               W_down (gelu_tanh(W_gate h) * W_up h);
  moe                 a softmax router over experts in groups: only experts of the best groups can be chosen, the choice adds a
                      stored correction to the score while the weight does not, the last experts are identities (they return the
                      feed-forward's input); experts are W_down (silu(W_gate h) * W_up h).
A layer may use another layer's weights (its cache / state is its own).

Notation: n tokens, width W.  `w` is a dict name -> float64 array with the checkpoint's names; `cfg` is the parsed config.json."""
import math

import numpy as np

# A test may ask how much rounding of the activations moves a result: inside `with rounding(fn):` every projection's output, every
# norm's output, the convolution's output, attention weights and the feed-forwards' hidden activations pass through fn (for
# instance a rounding to bfloat16).  It is an estimate of a row's conditioning, not a model of any engine.
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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return _r(x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * weight)


def part_rms_norm(x, weight, parts, eps):
    """The last axis in `parts` equal consecutive pieces, each divided by its own root mean square; then times weight."""
    n, c = x.shape
    y = x.reshape(n, parts, c // parts)
    y = y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)
    return _r(y.reshape(n, c) * weight)


# ------------------------------------------------------------------------------------------------ mamba2
def causal_conv(u, kernel, bias):
    """u [n, C], kernel [C, taps] whose last column meets the current token, zeros ahead of the sequence."""
    n, taps = u.shape[0], kernel.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, u.shape[1])), u], axis=0)
    out = np.tile(bias[None, :], (n, 1)).astype(np.float64)
    for k in range(taps):
        out += padded[k:k + n] * kernel[None, :, k]
    return out


def selective_scan(x, dt, a, b, c, d):
    """x [n, H, P], dt [n, H], a [H] (negative rates), b and c [n, H, N] (already spread over the heads), d [H] -> y [n, H, P]."""
    n, H, P = x.shape
    N = b.shape[-1]
    state = np.zeros((H, N, P))
    y = np.zeros((n, H, P))
    for t in range(n):
        decay = np.exp(a * dt[t])                                      # [H]
        state = decay[:, None, None] * state + dt[t][:, None, None] * b[t][:, :, None] * x[t][:, None, :]
        y[t] = np.einsum('hnp,hn->hp', state, c[t]) + d[:, None] * x[t]
    return y


def mamba2(h, w, p, m, eps):
    """Mixer 'mamba2'.  h [n, W] -> [n, W]."""
    n = h.shape[0]
    H, P, N, G = m['heads'], m['vdim'], m['state'], m['groups']
    inner = H * P
    proj = _r(h @ w[p + 'in'].T)
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = _r(silu(causal_conv(xbc, w[p + 'conv'], w[p + 'conv.b'])))
    x = xbc[:, :inner].reshape(n, H, P)
    b = xbc[:, inner:inner + G * N].reshape(n, G, N)
    c = xbc[:, inner + G * N:].reshape(n, G, N)
    per = H // G
    b, c = np.repeat(b, per, axis=1), np.repeat(c, per, axis=1)       # head a reads group a // per
    dt = softplus(dt + w[p + 'dt_bias'][None, :])
    y = selective_scan(x, dt, -np.exp(w[p + 'A_log']), b, c, w[p + 'D']).reshape(n, inner)
    y = y * silu(z)
    y = part_rms_norm(y, w[p + 'norm'], m['norm_groups'], eps)
    return y @ w[p + 'o'].T


# ------------------------------------------------------------------------------------------------ latent attention
def blended_frequencies(dims, base, scaling):
    """f_i = base^(-2i / dims); with scaling, low frequencies are divided by `factor`, high ones kept, a linear ramp between the
    dimensions at which `fast` and `slow` turns fit into the original length.  Returns (frequencies, cos / sin multiplier)."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling['factor']), float(scaling['original'])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling['fast']))), 0)
    hi = min(math.ceil(dim_of(float(scaling['slow']))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_halves(x, positions, dims, freq, mult):
    """x [n, ..., D]: dimension i < dims / 2 pairs with i + dims / 2; the rest pass."""
    if not dims:
        return x
    half = dims // 2
    ang = positions.astype(np.float64)[:, None] * freq[None, :]
    shape = (x.shape[0], ) + (1, ) * (x.ndim - 2) + (half, )
    cs, sn = (np.cos(ang) * mult).reshape(shape), (np.sin(ang) * mult).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    out = x.copy()
    out[..., :half] = u * cs - v * sn
    out[..., half:dims] = v * cs + u * sn
    return out


def window_visible(n, size):
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    vis = j <= i
    if size:
        vis &= (i - j) < size
    return vis


def sink_softmax(scores, vis, sink):
    """Row-wise softmax over the visible columns whose denominator also holds exp(sink) (None: none)."""
    s = np.where(vis, scores, -np.inf)
    top = s.max(axis=-1, keepdims=True)
    if sink is not None:
        top = np.maximum(top, sink)
    e = np.where(vis, np.exp(s - top), 0.0)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink - top)
    return _r(e / den)


def latent_attention(h, w, p, m, eps, positions=None):
    """Mixer 'latent_attention'.  h [n, W] -> [n, W]."""
    n = h.shape[0]
    H, D, R, E, C = m['heads'], m['dim'], m['rot_dim'], m['vdim'], m['kv_rank']
    pos = np.arange(n) if positions is None else positions
    rot = m.get('rot') or {}
    dims = int(rot.get('dims', 0))
    freq, mult = blended_frequencies(dims, float(rot.get('base', 10000.0)), rot.get('scaling')) if dims else (None, 1.0)
    cq = rms_norm(_r(h @ w[p + 'dq'].T), w[p + 'dq.norm'], eps)
    q = _r(cq @ w[p + 'uq'].T).reshape(n, H, D + R)
    q_plain, q_rot = q[..., :D], _r(rotate_halves(q[..., D:], pos, dims, freq, mult))
    dkv = _r(h @ w[p + 'dkv'].T)
    c = rms_norm(dkv[:, :C], w[p + 'dkv.norm'], eps)
    k_rot = _r(rotate_halves(dkv[:, C:], pos, dims, freq, mult))       # one part for all heads
    k_plain = (c @ w[p + 'uk'].T).reshape(n, H, D)
    v = (c @ w[p + 'uv'].T).reshape(n, H, E)
    vis = window_visible(n, int((m.get('mask') or {}).get('size', 0)))
    out = np.zeros((n, H, E))
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m['scale']
        sink = float(w[p + 'sink'][a]) if (p + 'sink') in w else None
        out[:, a] = _r(sink_softmax(s, vis, sink) @ v[:, a])
    return out.reshape(n, H * E) @ w[p + 'o'].T


# ------------------------------------------------------------------------------------------------ feed-forwards
def dense_ff(h, w, p):
    return _r(_r(gelu_tanh(_r(h @ w[p + 'gate'].T))) * _r(h @ w[p + 'up'].T)) @ w[p + 'down'].T


def route(h, w, p, r):
    """-> (chosen [n, top] expert numbers, weights [n, top]).  Scores are a softmax over all router outputs; the choice is made on
    score + correction, among the experts of the `keep` groups whose best such value is largest; the weight is score * scale."""
    total, top = int(r['experts']) + int(r.get('identity', 0)), int(r['top'])
    z = h @ w[p + 'router'].T
    z = z - z.max(axis=-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(axis=-1, keepdims=True)
    choice = s + (w[p + 'correction'][None, :] if (p + 'correction') in w else 0.0)
    groups = r.get('groups') or {}
    count, keep = int(groups.get('count', 1)), int(groups.get('keep', groups.get('count', 1)))
    n = h.shape[0]
    if count > 1 and keep < count:
        best = choice.reshape(n, count, total // count).max(axis=-1)
        kept = np.argsort(-best, axis=-1, kind='stable')[:, :keep]
        allowed = np.zeros((n, count), bool)
        np.put_along_axis(allowed, kept, True, axis=-1)
        choice = np.where(np.repeat(allowed, total // count, axis=1), choice, -np.inf)
    chosen = np.argsort(-choice, axis=-1, kind='stable')[:, :top]
    return chosen, np.take_along_axis(s, chosen, axis=-1) * float(r.get('scale', 1.0))


def expert_ff(h, w, p):
    return _r(_r(silu(_r(h @ w[p + 'gate'].T))) * _r(h @ w[p + 'up'].T)) @ w[p + 'down'].T


def moe_ff(h, w, p, mlp):
    r = mlp['router']
    real = int(r['experts'])
    chosen, weights = route(h, w, p, r)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t], weights[t]):
            out[t] += g * (h[t] if e >= real else expert_ff(h[t:t + 1], w, f'{p}e{e}.')[0])
    return out


# ------------------------------------------------------------------------------------------------ the stack
def weight_layer(cfg, i):
    return int(cfg['layers'][i].get('weights_of', i))


def layer_forward(x, w, cfg, i):
    l, eps = cfg['layers'][i], float(cfg['norm']['eps'])
    p = f'l{weight_layer(cfg, i)}.'
    h = rms_norm(x, w[p + 'norm1'], eps)
    if l['type'] == 'mamba2':
        x = x + mamba2(h, w, p + 'mix.', l['mixer'], eps)
    elif l['type'] == 'latent_attention':
        x = x + latent_attention(h, w, p + 'mix.', l['mixer'], eps)
    else:
        raise ValueError(l['type'])
    mlp = l.get('mlp')
    if mlp:
        h = rms_norm(x, w[p + 'norm2'], eps)
        x = x + (moe_ff(h, w, p + 'mlp.', mlp) if mlp.get('kind', 'dense') == 'moe' else dense_ff(h, w, p + 'mlp.'))
    return x


def forward(tokens, w, cfg, return_layers=False):
    """tokens [n] -> logits [n, vocab] (and the residual stream behind every layer, [layers, n, W])."""
    x = w['embed'][np.asarray(tokens)]
    taps = []
    for i in range(len(cfg['layers'])):
        x = layer_forward(x, w, cfg, i)
        taps.append(x)
    logits = rms_norm(x, w['final.norm'], float(cfg['norm']['eps'])) @ w['head'].T
    return (logits, np.stack(taps)) if return_layers else logits


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
