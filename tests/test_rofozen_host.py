"""Host-side pieces of the Rofozen design that need no GPU: the configuration reader and the registry, the random-weight maker's
tensor list, and the oracle's own mechanisms against closed forms and against a second way of computing them."""
import math

import numpy as np
import pytest

from oracle import rofozen_oracle as O
from rofozen_cases import dense, latent_layer, make_config, mamba_layer, moe, random_weights, shared
from tolenex_cases import as_f64


def test_registry_picks_the_class_by_config():
    from tensorrt_llm.models import MODEL_REGISTRY, RofozenForCausalLM, model_class_for
    assert model_class_for({'architecture': 'Rofozen'}) is RofozenForCausalLM
    assert {'Rofozen', 'Vetipel', 'Tolenex'} <= set(MODEL_REGISTRY)


def test_config_reader_takes_every_size_from_the_file():
    from tensorrt_llm.models import RofozenConfig
    cfg = make_config([mamba_layer(heads=10, vdim=12, state=20, groups=5, conv=3, norm_groups=4, mlp=dense(33)),
                       latent_layer(heads=7, dim=10, rot_dim=6, vdim=14, kv_rank=50, q_rank=31, size=77, base=123.0,
                                    mlp=moe(experts=9, identity=3, top=4, count=6, keep=5, ff=17, scale=0.75)),
                       shared(mamba_layer(heads=10, vdim=12, state=20, groups=5, conv=3, norm_groups=4, mlp=dense(33)), 0),
                       latent_layer(size=0, scaling=False)], width=140, vocab=1001, eps=3e-6)
    c = RofozenConfig(cfg).engine_config()
    assert (c['width'], c['vocab'], c['num_layers'], c['streams'], c['block'], c['residual']) == (140, 1001, 4, 1, 'sequential', 'hyper')
    assert float(c['norm_eps']) == 3e-6 and float(c['norm_offset']) == 0.0
    assert (c['layer.0.type'], c['layer.0.heads'], c['layer.0.vdim'], c['layer.0.state'], c['layer.0.groups'], c['layer.0.conv'],
            c['layer.0.ssm_norm_groups'], c['layer.0.ff'], c['layer.0.mlp']) == ('mamba2', 10, 12, 20, 5, 3, 4, 33, 'gelu_gate')
    assert (c['layer.1.type'], c['layer.1.kv_rank'], c['layer.1.q_rank'], c['layer.1.rot_dim'], c['layer.1.rot_dims'], c['layer.1.rot_pairing'],
            c['layer.1.mask'], c['layer.1.mask_size'], c['layer.1.sink']) == ('latent_attention', 50, 31, 6, 6, 'halves', 'window', 77, 1)
    assert float(c['layer.1.rot_base']) == 123.0 and float(c['layer.1.rot_factor']) == 8.0 and float(c['layer.1.rot_original']) == 64.0
    assert (c['layer.1.mlp'], c['layer.1.ff'], c['layer.1.experts'], c['layer.1.identity'], c['layer.1.top'], c['layer.1.route_groups'],
            c['layer.1.route_keep']) == ('moe', 17, 9, 3, 4, 6, 5)
    assert float(c['layer.1.route_scale']) == 0.75
    assert c['layer.2.weights_of'] == 0 and 'layer.1.weights_of' not in c
    assert (c['layer.3.mask'], c['layer.3.ff']) == ('causal', 0) and 'layer.3.rot_factor' not in c
    with pytest.raises(ValueError):
        RofozenConfig(make_config([{'type': 'hgrn2', 'mixer': {}, 'mlp': None}]))
    with pytest.raises(ValueError):
        RofozenConfig(make_config([mamba_layer(), shared(mamba_layer(), 1)]))
    with pytest.raises(ValueError):
        RofozenConfig(make_config([mamba_layer(), shared(mamba_layer(), 0), shared(mamba_layer(), 1)]))


def test_random_weight_maker_names_what_the_tests_generator_names():
    """Two generators written apart (the product's, for benchmarks; the tests') must agree on names and shapes."""
    from tensorrt_llm.models import RofozenForCausalLM
    cfg = make_config([mamba_layer(mlp=moe()), latent_layer(mlp=dense()), shared(mamba_layer(mlp=moe()), 0), latent_layer(size=0)])
    ours = random_weights(cfg, 1)
    theirs = RofozenForCausalLM.from_random(cfg, seed=2).tensors
    assert {k: v.shape for k, v in ours.items()} == {k: a.shape for k, (a, _) in theirs.items()}
    assert not any(k.startswith('l2.') for k in ours)


def test_convolution_meets_the_current_token_with_its_last_tap():
    u = np.arange(1.0, 6.0)[:, None]
    out = O.causal_conv(u, np.array([[100.0, 10.0, 1.0]]), np.array([0.5]))
    assert out[:, 0].tolist() == [1.5, 12.5, 123.5, 234.5, 345.5]


def test_scan_against_its_closed_form():
    """y_t = sum_{s <= t} exp(a (dt_{s+1} + ... + dt_t)) dt_s (C_t . B_s) x_s + D x_t."""
    rng = np.random.default_rng(0)
    n, H, P, N = 7, 2, 3, 4
    x, dt = rng.standard_normal((n, H, P)), rng.uniform(0.1, 1.0, (n, H))
    a, d = -rng.uniform(0.2, 2.0, H), rng.standard_normal(H)
    b, c = rng.standard_normal((n, H, N)), rng.standard_normal((n, H, N))
    want = np.zeros((n, H, P))
    for t in range(n):
        for s in range(t + 1):
            want[t] += (np.exp(a * dt[s + 1:t + 1].sum(axis=0)) * dt[s] * (c[t] * b[s]).sum(-1))[:, None] * x[s]
        want[t] += d[:, None] * x[t]
    assert np.allclose(O.selective_scan(x, dt, a, b, c, d), want, rtol=1e-12, atol=1e-12)


def test_heads_read_the_group_of_their_neighbours():
    """4 heads in 2 groups: heads 0, 1 read B / C of group 0 and heads 2, 3 of group 1 - changing group 1's B moves heads 2, 3 only."""
    cfg = make_config([mamba_layer(heads=4, vdim=3, state=5, groups=2, conv=2, norm_groups=4)], width=16, vocab=11)
    w = as_f64(random_weights(cfg, 1))
    m, p = cfg['layers'][0]['mixer'], 'l0.mix.'
    h = np.random.default_rng(1).standard_normal((6, 16))
    w[p + 'o'] = np.eye(16)[:, :12]
    base = O.mamba2(h, w, p, m, 1e-5)
    w2 = dict(w)
    w2[p + 'in'] = w[p + 'in'].copy()
    w2[p + 'in'][2 * 12 + 5:2 * 12 + 10] *= 2.0   # rows of B, group 1
    moved = np.abs(O.mamba2(h, w2, p, m, 1e-5) - base)[:, :12].reshape(6, 4, 3).max(axis=(0, 2))
    assert moved[0] == 0 and moved[1] == 0 and moved[2] > 1e-3 and moved[3] > 1e-3


def test_blended_frequencies():
    f, mult = O.blended_frequencies(8, 100.0, None)
    assert mult == 1.0 and np.allclose(f, 100.0 ** (-np.arange(4) / 4.0))
    sc = {'factor': 4.0, 'original': 32, 'fast': 8.0, 'slow': 1.0}
    f2, mult2 = O.blended_frequencies(8, 100.0, sc)
    assert math.isclose(mult2, 0.1 * math.log(4.0) + 1.0)
    lo = max(math.floor(8 * math.log(32 / (2 * math.pi * 8.0)) / (2 * math.log(100.0))), 0)
    hi = min(math.ceil(8 * math.log(32 / (2 * math.pi * 1.0)) / (2 * math.log(100.0))), 7)
    assert (lo, hi) == (0, 2)
    assert np.allclose(f2, f * np.array([1.0, 0.625, 0.25, 0.25]))   # ramp 0, 1/2, 1, 1 between the full and the quartered frequency


def test_rotation_pairs_the_two_halves():
    x = np.zeros((1, 6))
    x[0, 0] = 1.0
    out = O.rotate_halves(x, np.array([1]), 4, np.array([math.pi / 2, 0.3]), 2.0)
    assert np.allclose(out[0], [0.0, 0.0, 2.0, 0.0, 0.0, 0.0], atol=1e-12)   # dimension 0 turns into its partner 2, times the multiplier


def test_a_sink_takes_its_share_and_brings_nothing():
    """One token: the only key is the token itself, so the head's output is v * e^s / (e^s + e^sink)."""
    cfg = make_config([latent_layer(heads=2, dim=4, rot_dim=2, vdim=3, kv_rank=6, q_rank=5, size=5)], width=8, vocab=11)
    w = as_f64(random_weights(cfg, 3))
    m, eps, p = cfg['layers'][0]['mixer'], cfg['norm']['eps'], 'l0.mix.'
    h = np.random.default_rng(0).standard_normal((1, 8))
    cq = O.rms_norm(h @ w[p + 'dq'].T, w[p + 'dq.norm'], eps)
    q = (cq @ w[p + 'uq'].T).reshape(2, 6)
    dkv = (h @ w[p + 'dkv'].T)[0]
    c = O.rms_norm(dkv[None, :6], w[p + 'dkv.norm'], eps)[0]
    mult = 0.1 * math.log(8.0) + 1.0   # position 0: cos = multiplier, sin = 0
    heads = []
    for a in range(2):
        k = w[p + 'uk'][a * 4:(a + 1) * 4] @ c
        s = (q[a, :4] @ k + (q[a, 4:] * mult) @ (dkv[6:] * mult)) * m['scale']
        heads.append((w[p + 'uv'][a * 3:(a + 1) * 3] @ c) * np.exp(s) / (np.exp(s) + np.exp(w[p + 'sink'][a])))
    assert np.allclose(O.latent_attention(h, w, p, m, eps)[0], np.concatenate(heads) @ w[p + 'o'].T, rtol=1e-12, atol=1e-12)


def test_latent_attention_equals_its_absorbed_form():
    """Scores through W_uk^T q against the latent, values expanded after the weighted sum of latents: the same function."""
    cfg = make_config([latent_layer(heads=3, dim=6, rot_dim=4, vdim=5, kv_rank=10, q_rank=7, size=4)], width=16, vocab=11)
    w = as_f64(random_weights(cfg, 5))
    m, eps, p = cfg['layers'][0]['mixer'], cfg['norm']['eps'], 'l0.mix.'
    n, H, D, R, E, C = 9, 3, 6, 4, 5, 10
    h = np.random.default_rng(2).standard_normal((n, 16))
    pos = np.arange(n)
    freq, mult = O.blended_frequencies(4, m['rot']['base'], m['rot']['scaling'])
    q = (O.rms_norm(h @ w[p + 'dq'].T, w[p + 'dq.norm'], eps) @ w[p + 'uq'].T).reshape(n, H, D + R)
    down = h @ w[p + 'dkv'].T
    c = O.rms_norm(down[:, :C], w[p + 'dkv.norm'], eps)
    k_rot, q_rot = O.rotate_halves(down[:, C:], pos, 4, freq, mult), O.rotate_halves(q[..., D:], pos, 4, freq, mult)
    vis = O.window_visible(n, 4)
    out = np.zeros((n, H, E))
    for a in range(H):
        q_abs = q[:, a, :D] @ w[p + 'uk'][a * D:(a + 1) * D]                   # [n, C]
        s = np.where(vis, (q_abs @ c.T + q_rot[:, a] @ k_rot.T) * m['scale'], -np.inf)
        e = np.exp(s)
        out[:, a] = ((e / (e.sum(axis=1, keepdims=True) + np.exp(w[p + 'sink'][a]))) @ c) @ w[p + 'uv'][a * E:(a + 1) * E].T
    assert np.allclose(O.latent_attention(h, w, p, m, eps), out.reshape(n, H * E) @ w[p + 'o'].T, rtol=1e-10, atol=1e-12)


def router_weights(scores, correction):
    """A router whose softmax scores on the input e_0 are `scores`: logits = ln scores in column 0."""
    ne = len(scores)
    r = np.zeros((ne, 4))
    r[:, 0] = np.log(scores)
    return {'router': r, 'correction': np.asarray(correction, np.float64)}


def test_choice_adds_the_correction_and_the_weight_does_not():
    h = np.array([[1.0, 0.0, 0.0, 0.0]])
    w = router_weights([0.4, 0.3, 0.2, 0.1], [0.0, 0.0, 0.15, 0.35])
    r = {'experts': 4, 'identity': 0, 'top': 2, 'scale': 2.0, 'groups': {'count': 1, 'keep': 1}}
    chosen, weights = O.route(h, w, '', r)
    assert chosen[0].tolist() == [3, 0]                      # 0.45, 0.4 beat 0.35, 0.3
    assert np.allclose(weights[0], [0.2, 0.8])               # the plain scores times the scale, not renormalised


def test_only_experts_of_the_best_groups_can_be_chosen():
    h = np.array([[1.0, 0.0, 0.0, 0.0]])
    # groups {0, 1}, {2, 3}, {4, 5}: their best choice values are 0.30, 0.32, 0.05: with one group kept the two largest scores (0.30
    # and 0.28 of group 0) lose to group 1's experts
    w = router_weights([0.30, 0.28, 0.32, 0.02, 0.05, 0.03], [0.0] * 6)
    r = {'experts': 5, 'identity': 1, 'top': 2, 'scale': 1.0, 'groups': {'count': 3, 'keep': 1}}
    assert O.route(h, w, '', r)[0][0].tolist() == [2, 3]
    r['groups']['keep'] = 2
    assert O.route(h, w, '', r)[0][0].tolist() == [2, 0]
    # a negative choice value inside a kept group still beats every expert outside it
    w = router_weights([0.30, 0.28, 0.32, 0.02, 0.05, 0.03], [0.0, 0.0, 0.0, -0.5, 0.0, 0.0])
    r['groups']['keep'] = 1
    assert O.route(h, w, '', r)[0][0].tolist() == [2, 3]


def test_identity_experts_return_their_input():
    cfg = make_config([mamba_layer(mlp=moe(experts=2, identity=2, top=2, count=1, keep=1, scale=1.5))], width=8, vocab=11)
    w = as_f64(random_weights(cfg, 7))
    w['l0.mlp.router'] = np.zeros((4, 8))
    w['l0.mlp.router'][:, 0] = np.log([0.1, 0.2, 0.3, 0.4])
    w['l0.mlp.correction'] = np.zeros(4)
    h = np.zeros((1, 8))
    h[0, 0], h[0, 3] = 1.0, -2.0
    out = O.moe_ff(h, w, 'l0.mlp.', cfg['layers'][0]['mlp'])
    assert np.allclose(out, 1.5 * (0.3 + 0.4) * h)           # both chosen outputs are identities
    w['l0.mlp.correction'] = np.array([0.0, 0.5, 0.0, 0.0])  # expert 1 is chosen instead of identity 2, at its plain score
    out = O.moe_ff(h, w, 'l0.mlp.', cfg['layers'][0]['mlp'])
    assert np.allclose(out, 1.5 * (0.4 * h + 0.2 * O.expert_ff(h, w, 'l0.mlp.e1.')))


def test_a_layer_on_shared_weights_is_the_same_function():
    """Two layers on one set of weights, applied to the same input, give the same update."""
    cfg = make_config([mamba_layer(mlp=dense()), shared(mamba_layer(mlp=dense()), 0)])
    w = as_f64(random_weights(cfg, 9))
    x = np.random.default_rng(3).standard_normal((5, 96))
    assert np.array_equal(O.layer_forward(x, w, cfg, 0), O.layer_forward(x, w, cfg, 1))
