"""Host-side pieces of the Narurax design that need no GPU: the configuration reader and the registry, the random-weight maker's
tensor list, and the oracle's own mechanisms against closed forms and against a second way of computing them."""
import math

import numpy as np
import pytest

from narurax_cases import attn2_layer, attn_layer, delta_layer, make_config, moe, random_weights
from oracle import narurax_oracle as O
from tolenex_cases import as_f64


def test_registry_picks_the_class_by_config():
    from tensorrt_llm.models import MODEL_REGISTRY, NaruraxForCausalLM, model_class_for
    assert model_class_for({'architecture': 'Narurax'}) is NaruraxForCausalLM
    assert {'Narurax', 'Rofozen', 'Vetipel', 'Tolenex'} <= set(MODEL_REGISTRY)


def test_config_reader_takes_every_size_from_the_file():
    from tensorrt_llm.models import NaruraxConfig
    cfg = make_config([attn_layer(heads=10, kv_heads=5, dim=12, rot_dims=6, base=123.0, size=77, keep=9, scale=0.3, mlp=moe(experts=9, top=4, ff=17)),
                       attn2_layer(heads=6, kv_heads=2, dim=10, vdim=14, rot_dims=10, base=77.0, size=31, keep=0, scale=0.7),
                       delta_layer(heads=8, kv_heads=4, dim=20, vdim=6, conv=3, mlp=moe(experts=3, top=1, ff=5)),
                       attn2_layer(size=0, scaling=False)], width=140, vocab=1001, eps=3e-6, bigram=(101, 17, 3))
    c = NaruraxConfig(cfg, ranks={2: (5, 7)}).engine_config()
    assert (c['width'], c['vocab'], c['num_layers'], c['streams'], c['block'], c['residual'], c['token_shift']) == (
        140, 1001, 4, 1, 'sequential', 'hyper', 1)
    assert (c['pair_buckets'], c['pair_mul_prev'], c['pair_mul_cur']) == (101, 17, 3) and float(c['norm_eps']) == 3e-6
    assert (c['layer.0.type'], c['layer.0.heads'], c['layer.0.kv_heads'], c['layer.0.dim'], c['layer.0.vdim'], c['layer.0.rot_dims'],
            c['layer.0.mask'], c['layer.0.mask_size'], c['layer.0.mask_keep'], c['layer.0.values_are_keys'], c['layer.0.talk'],
            c['layer.0.sink'], c['layer.0.out_gate'], c['layer.0.gate_wide']) == ('attention', 10, 5, 12, 12, 6, 'window', 77, 9, 1, 1, 1, 1, 1)
    assert float(c['layer.0.rot_base']) == 123.0 and float(c['layer.0.scale']) == 0.3 and 'layer.0.rot_scaling' not in c
    assert (c['layer.0.mlp'], c['layer.0.ff'], c['layer.0.experts'], c['layer.0.top'], c['layer.0.identity'], c['layer.0.route_score'],
            c['layer.0.route_weight']) == ('moe', 17, 9, 4, 0, 'sigmoid', 'input')
    assert (c['layer.1.type'], c['layer.1.vdim'], c['layer.1.qkv_bias'], c['layer.1.o_bias'], c['layer.1.qk_norm'], c['layer.1.qk_norm_weight'],
            c['layer.1.sink'], c['layer.1.rot_scaling'], c['layer.1.mask_keep'], c['layer.1.ff']) == ('attention', 14, 1, 1, 1, 1, 2, 'banded', 0, 0)
    assert (float(c['layer.1.rot_factor']), float(c['layer.1.rot_low']), float(c['layer.1.rot_high']), float(c['layer.1.rot_original'])) == (8.0, 1.0, 3.0, 48.0)
    assert 'layer.1.talk' not in c and 'layer.1.values_are_keys' not in c
    assert (c['layer.2.type'], c['layer.2.heads'], c['layer.2.kv_heads'], c['layer.2.dim'], c['layer.2.vdim'], c['layer.2.conv'],
            c['layer.2.decay_rank'], c['layer.2.gate_rank']) == ('delta_rule', 8, 4, 20, 6, 3, 5, 7)
    assert c['layer.3.mask'] == 'causal' and 'layer.3.rot_scaling' not in c
    with pytest.raises(ValueError):
        NaruraxConfig(make_config([{'type': 'mamba2', 'mixer': {}, 'mlp': None}]))
    with pytest.raises(ValueError):
        NaruraxConfig(make_config([attn_layer(mlp={'kind': 'dense', 'ff': 8})]))


def test_random_weight_maker_names_what_the_tests_generator_names():
    """Two generators written apart (the product's, for benchmarks; the tests') must agree on names and shapes; the model object
    takes the ranks of the low-rank pairs from the tensors."""
    from narurax_cases import as_model
    from tensorrt_llm.models import NaruraxForCausalLM
    cfg = make_config([attn_layer(mlp=moe()), delta_layer(mlp=moe(experts=3, top=1)), attn2_layer(), delta_layer()])
    ours = random_weights(cfg, 1, ranks=(9, 11))
    theirs = NaruraxForCausalLM.from_random(cfg, seed=2, ranks={1: (9, 11), 3: (9, 11)}).tensors
    assert {k: v.shape for k, v in ours.items()} == {k: a.shape for k, (a, _) in theirs.items()}
    c = as_model(cfg, ours).config.engine_config()
    assert (c['layer.1.decay_rank'], c['layer.1.gate_rank'], c['layer.3.decay_rank']) == (9, 11, 9)


def test_pair_rows():
    bg = {'buckets': 11, 'mul_prev': 7, 'mul_cur': 3}
    assert O.bigram_rows([5, 2, 9, 9], bg) == [11, (5 * 7 + 2 * 3) % 11, (2 * 7 + 9 * 3) % 11, (9 * 7 + 9 * 3) % 11]
    big = {'buckets': 1000003, 'mul_prev': 2 ** 31 - 1, 'mul_cur': 2 ** 31 - 19}
    assert O.bigram_rows([70000, 65000], big)[1] == (70000 * (2 ** 31 - 1) + 65000 * (2 ** 31 - 19)) % 1000003


def test_token_shift_blends_with_the_unshifted_neighbour():
    h = np.array([[1.0, 10.0], [2.0, 20.0], [4.0, 40.0]])
    out = O.token_shift(h, np.array([0.5, 1.0]))
    assert out.tolist() == [[0.5, 0.0], [1.5, 10.0], [3.0, 20.0]]


def test_visible_keys():
    m = O.visible(8, 3, 2)
    assert m[7].tolist() == [True, True, False, False, False, True, True, True]
    assert m[2].tolist() == [True, True, True, False, False, False, False, False]
    assert O.visible(5, 1, 0)[4].tolist() == [False, False, False, False, True]
    assert O.visible(4, 99, 0).tolist() == np.tril(np.ones((4, 4), bool)).tolist()


def test_sink_joins_the_denominator_only():
    scores = np.log(np.array([[[1.0, 3.0]]]))
    p = O.sink_softmax(scores, np.ones((1, 2), bool), np.array([math.log(4.0)]))
    assert np.allclose(p, [[[1 / 8, 3 / 8]]])
    p0 = O.sink_softmax(scores, np.ones((1, 2), bool), np.zeros(1))
    assert np.allclose(p0, [[[1 / 5, 3 / 5]]])


def test_banded_frequencies():
    sc = {'factor': 4.0, 'low': 1.0, 'high': 4.0, 'original': 64}
    f0, f = O.plain_frequencies(32, 10000.0), O.banded_frequencies(32, 10000.0, sc)
    wave = 2 * math.pi / f0
    assert np.allclose(f[wave < 16], f0[wave < 16]) and np.allclose(f[wave > 64], f0[wave > 64] / 4.0)
    mid = (wave >= 16) & (wave <= 64)
    assert mid.any() and ((f[mid] <= f0[mid] + 1e-15) & (f[mid] >= f0[mid] / 4.0 - 1e-15)).all()
    s = (64 / wave[mid] - 1.0) / 3.0
    assert np.allclose(f[mid], (1 - s) * f0[mid] / 4.0 + s * f0[mid])
    assert np.allclose(O.banded_frequencies(32, 10000.0, None), f0)


def test_rotation_turns_neighbouring_pairs_and_keeps_scores_relative():
    rng = np.random.default_rng(0)
    q, k = rng.standard_normal((1, 1, 8)), rng.standard_normal((1, 1, 8))
    f = O.plain_frequencies(4, 100.0)
    a = O.rotate_pairs(q, np.array([9]), 4, f)[0, 0] @ O.rotate_pairs(k, np.array([5]), 4, f)[0, 0]
    b = O.rotate_pairs(q, np.array([104]), 4, f)[0, 0] @ O.rotate_pairs(k, np.array([100]), 4, f)[0, 0]
    assert abs(a - b) < 1e-9
    one = O.rotate_pairs(np.array([[[1.0, 0.0, 0.0, 0.0, 5.0, 6.0]]]), np.array([1]), 4, np.array([math.pi / 2, 0.0]))[0, 0]
    assert np.allclose(one, [0.0, 1.0, 0.0, 0.0, 5.0, 6.0])


def test_talking_heads_against_a_loop():
    cfg = make_config([attn_layer(heads=4, kv_heads=2, dim=8, rot_dims=4, size=5, keep=1)], width=32)
    w = as_f64(random_weights(cfg, 3))
    m, p = cfg['layers'][0]['mixer'], 'l0.mix.'
    h = np.random.default_rng(1).standard_normal((9, 32))
    got = O.attention(h, w, p, m, 1e-5)
    n, H, G, D = 9, 4, 2, 8
    q, k = (h @ w[p + 'q'].T).reshape(n, H, D), (h @ w[p + 'k'].T).reshape(n, G, D)
    f = O.plain_frequencies(4, m['rot']['base'])
    qr, kr = O.rotate_pairs(q, np.arange(n), 4, f), O.rotate_pairs(k, np.arange(n), 4, f)
    out = np.zeros((n, H, D))
    for i in range(n):
        js = [j for j in range(i + 1) if i - j < 5 or j < 1]
        pw = np.zeros((H, len(js)))
        for g in range(H):
            e = np.exp([qr[i, g] @ kr[j, g // 2] * m['scale'] for j in js])
            pw[g] = e / (e.sum() + math.exp(w[p + 'sink'][g]))
        for hd in range(H):
            mixed = sum(w[p + 'talk'][hd, g] * pw[g] for g in range(H))
            out[i, hd] = sum(mixed[a] * k[j, hd // 2] for a, j in enumerate(js))
    want = (out.reshape(n, H * D) * O.sigmoid(h @ w[p + 'g'].T)) @ w[p + 'o'].T
    assert np.allclose(got, want, atol=1e-10)


def test_delta_rule_against_its_closed_form():
    """With beta = 1 and no decay, writing v under a unit key k and reading with q = k returns v; a second write under the same key
    replaces it; a decay of g on every key channel scales what is read by g per step."""
    k = np.zeros((3, 1, 4))
    k[:, 0, 1] = 1.0
    v = np.array([[[1.0, 2.0]], [[5.0, -1.0]], [[0.0, 0.0]]])
    one = np.ones((3, 1))
    o = O.delta_scan(k, k, v, one, np.ones((3, 1, 4)))
    assert np.allclose(o[:, 0], [[1.0, 2.0], [5.0, -1.0], [0.0, 0.0]])
    o = O.delta_scan(k, k, v, one * np.array([[1.0], [0.0], [0.0]]), np.full((3, 1, 4), 0.5))
    assert np.allclose(o[:, 0], [[1.0, 2.0], [0.5, 1.0], [0.25, 0.5]])


def test_convolution_meets_the_current_token_with_its_last_tap():
    u = np.arange(1.0, 6.0)[:, None]
    assert O.causal_conv(u, np.array([[100.0, 10.0, 1.0]]))[:, 0].tolist() == [1.0, 12.0, 123.0, 234.0, 345.0]


def test_router_takes_the_largest_scores_and_weights_the_input():
    w = {'r.router': np.array([[1.0, 0.0], [0.0, 1.0], [-1.0, 0.0], [0.5, 0.5]])}
    idx, wt = O.route(np.array([[2.0, 1.0]]), w, 'r.', {'top': 2})
    assert idx.tolist() == [[0, 3]] and np.allclose(wt, [[O.sigmoid(2.0), O.sigmoid(1.5)]])
    # one expert whose gate and up are the identity: the output is silu(s h) * (s h), not s * silu(h) * h
    e = {'r.router': np.array([[0.0, 0.0]]), 'r.e0.gate': np.eye(2), 'r.e0.up': np.eye(2), 'r.e0.down': np.eye(2)}
    y = O.moe(np.array([[2.0, -4.0]]), e, 'r.', {'router': {'top': 1}})
    a = 0.5 * np.array([2.0, -4.0])
    assert np.allclose(y, [O.silu(a) * a])
