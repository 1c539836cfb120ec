"""Narurax through the ragged stack engine against the plain float64 oracle (oracle/narurax_oracle.py), on small configurations and
random weights made here.  fp32 engine: tight bound (what summation order can explain), routers with random weights (their decisions
are checked on the oracle not to be close calls at that bound); bfloat16 engine: every row is held to what rounding the oracle's own
activations does to it, routers rigged so that no decision is close, and crafted weights where random ones would hide a fault (a key
at a window's edge or at the edge of the kept first tokens, one far key among hundreds, a sink, mixed heads, one far token whose
trace must survive in a recurrent state)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from narurax_cases import as_model, attn2_layer, attn_layer, decisive_router, delta_layer, make_config, moe, random_weights
from oracle import narurax_oracle as O
from tolenex_cases import as_f64, bf16_round, rel_err, replay

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 3e-5, 5e-2


def has_router(cfg):
    return any(l.get('mlp') for l in cfg['layers'])


def weights_for(cfg, seed, dtype, toks=None, ranks=(9, 11)):
    """Random weights; for the bfloat16 engine the routers are rigged.  With `toks`, the routers' decisions on them are checked on
    the oracle to stand clear of what the engine's rounding can move; a model with a close call is passed over for the next seed."""
    need = 0.02 if dtype == 'bfloat16' else 2e-4
    for attempt in range(10):
        w = random_weights(cfg, seed + 1000 * attempt, ranks)
        if not has_router(cfg):
            return w
        if dtype == 'bfloat16':
            w = decisive_router(cfg, w, seed)
        if toks is None or all(O.routing_margin(t, as_f64(w), cfg) > need for t in (toks.values() if isinstance(toks, dict) else [toks])):
            return w
    raise AssertionError('ten models in a row with a router decision that is a close call')


def session_for(cfg, w, dtype='float32', max_tokens=1024, max_sequences=4, **kw):
    from tensorrt_llm.runtime import RaggedGenerationSession
    return RaggedGenerationSession(as_model(cfg, w), dtype=dtype, max_tokens=max_tokens, max_sequences=max_sequences, **kw)


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg['vocab'], n).tolist()


def check(got, want, tol, what=''):
    e = rel_err(got, want)
    assert np.isfinite(got).all(), what
    assert e.max() < tol, f'{what}: worst row {int(e.argmax())} of {len(e)} has relative error {e.max():.3g} (bound {tol})'


def tol_of(dtype):
    return F32_TOL if dtype == 'float32' else BF16_TOL


def to_bf16(x):
    return bf16_round(np.asarray(x, np.float32)).astype(np.float64)


def check_rows(got, toks, w, cfg, dtype, what=''):
    """Every position of a request against the oracle.  fp32: the flat bound.  bfloat16: a row is held to 3 x what rounding the
    oracle's own activations to bfloat16 does to it (never less than the median row's); no row may pass 1.5 x that, and at most one
    row in fifty (or one) may pass it at all."""
    wf = as_f64(w)
    want = O.logits(toks, wf, cfg)
    if dtype == 'float32':
        return check(got, want, F32_TOL, what)
    with O.rounding(to_bf16):
        moved = rel_err(O.logits(toks, wf, cfg), want)
    limit = 3.0 * np.maximum(moved, np.median(moved))
    e = rel_err(got, want)
    assert np.isfinite(got).all(), what
    worst = int((e / limit).argmax())
    assert (e < 1.5 * limit).all(), f'{what}: row {worst} of {len(e)} has relative error {e[worst]:.3g}, its limit is {limit[worst]:.3g}'
    assert (e > limit).sum() <= max(1, len(e) // 50), f'{what}: {(e > limit).sum()} of {len(e)} rows are over their limits'
    assert np.median(e) < 3e-2, f'{what}: the median row is off by {np.median(e):.3g}'


FULL = [attn2_layer(mlp=moe()), delta_layer(mlp=moe(experts=5, top=1)), attn_layer(mlp=moe(experts=7, top=3, ff=10)),
        delta_layer(heads=3, kv_heads=3, dim=7, vdim=5, conv=3, mlp=None),
        attn2_layer(heads=3, kv_heads=1, dim=10, vdim=6, rot_dims=4, scaling=False, size=64, keep=0, mlp=moe(experts=4, top=4)),
        attn_layer(heads=2, kv_heads=2, dim=8, rot_dims=8, size=21, keep=9, mlp=None)]
# shapes the MFMA tile kernels and the LDS-staged products take in bfloat16; fp32 runs them on the general kernels
TILED = [attn2_layer(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=64, size=45, keep=5, mlp=moe(experts=4, top=2, ff=64)),
         delta_layer(heads=4, kv_heads=2, dim=32, vdim=64, conv=4, mlp=moe(experts=8, top=1, ff=64)),
         attn_layer(heads=4, kv_heads=2, dim=64, rot_dims=32, size=70, keep=33, mlp=None),
         attn2_layer(heads=2, kv_heads=1, dim=32, vdim=128, rot_dims=16, size=130, keep=1, mlp=moe(experts=2, top=1, ff=128)),
         delta_layer(heads=2, kv_heads=1, dim=128, vdim=32, conv=2, mlp=None)]
STACKS = {'general': (FULL, 96), 'tiled': (TILED, 128)}


def stack_config(name, layers=None):
    full, width = STACKS[name]
    return make_config(full if layers is None else full[:layers], width=width)


MECHANISMS = {
    'attention_alone_no_ff': make_config([attn_layer()]),
    'attention_no_pair_table': make_config([attn_layer()], bigram=None),
    'attention_one_head': make_config([attn_layer(heads=1, kv_heads=1, dim=20, rot_dims=20)]),
    'attention_one_kv_head': make_config([attn_layer(heads=5, kv_heads=1, dim=6, rot_dims=2)]),
    'attention_kv_per_head': make_config([attn_layer(heads=3, kv_heads=3)]),
    'attention_no_rotation': make_config([attn_layer(rot_dims=0)]),
    'attention_causal': make_config([attn_layer(size=0)]),
    'attention_window_of_one_keeps_four': make_config([attn_layer(size=1, keep=4)]),
    'attention_window_two_keeps_none': make_config([attn_layer(size=2, keep=0)]),
    'attention_window_a_page': make_config([attn_layer(size=64, keep=64)]),
    'attention_keeps_more_than_the_window': make_config([attn_layer(size=10, keep=80)]),
    'attention_window_wider_than_the_prompt': make_config([attn_layer(size=500, keep=2)]),
    'attention_many_heads': make_config([attn_layer(heads=16, kv_heads=4, dim=4, rot_dims=4)]),
    'attention_tile_64': make_config([TILED[2]], width=128),
    'attention_tile_32_one_kv_head': make_config([attn_layer(heads=4, kv_heads=1, dim=32, rot_dims=32, size=40, keep=2)], width=128),
    'attention_tile_128_kv_per_head': make_config([attn_layer(heads=2, kv_heads=2, dim=128, rot_dims=64, size=90, keep=35)], width=128),
    'attention_tile_64_eight_pairs_per_head': make_config([attn_layer(heads=8, kv_heads=8, dim=64, rot_dims=16, size=0)], width=128),
    'attention2_alone_no_ff': make_config([attn2_layer()]),
    'attention2_no_scaling': make_config([attn2_layer(scaling=False)]),
    'attention2_partly_rotated': make_config([attn2_layer(dim=14, rot_dims=6)]),
    'attention2_no_rotation': make_config([attn2_layer(rot_dims=0)]),
    'attention2_causal': make_config([attn2_layer(size=0)]),
    'attention2_one_head': make_config([attn2_layer(heads=1, kv_heads=1, dim=24, vdim=8, rot_dims=24)]),
    'attention2_window_of_one_keeps_one': make_config([attn2_layer(size=1, keep=1)]),
    'attention2_window_65_keeps_65': make_config([attn2_layer(size=65, keep=65)]),
    'attention2_tile_64_64': make_config([TILED[0]], width=128),
    'attention2_tile_32_128': make_config([TILED[3]], width=128),
    'delta_alone_no_ff': make_config([delta_layer()]),
    'delta_one_head': make_config([delta_layer(heads=1, kv_heads=1, dim=20, vdim=7)]),
    'delta_shared_qk_head': make_config([delta_layer(heads=6, kv_heads=1, dim=5, vdim=9)]),
    'delta_one_tap': make_config([delta_layer(conv=1)]),
    'delta_two_taps': make_config([delta_layer(conv=2)]),
    'delta_seven_taps': make_config([delta_layer(conv=7)]),
    'delta_dim_of_one': make_config([delta_layer(dim=1)]),
    'delta_large_dim_small_head': make_config([delta_layer(heads=2, kv_heads=2, dim=200, vdim=4)]),
    'delta_wide_head': make_config([delta_layer(heads=2, kv_heads=1, dim=24, vdim=96)]),
    'delta_tile_128_32': make_config([TILED[4]], width=128),
    'moe_top_one': make_config([delta_layer(mlp=moe(experts=4, top=1))]),
    'moe_every_expert': make_config([attn_layer(mlp=moe(experts=3, top=3))]),
    'moe_one_expert': make_config([attn2_layer(mlp=moe(experts=1, top=1))]),
    'moe_many_experts': make_config([delta_layer(mlp=moe(experts=40, top=5, ff=6))]),
    'moe_wide_experts': make_config([TILED[1]], width=128),
    'whole_stack': make_config(FULL, eps=3e-6),
    'tiled_stack': make_config(TILED, width=128),
    'width_that_is_no_multiple_of_four': make_config([attn_layer(heads=3, kv_heads=1, dim=6, rot_dims=4, size=9, keep=2, mlp=moe(ff=10)),
                                                      delta_layer(heads=3, kv_heads=1, dim=7, vdim=5, mlp=moe(experts=3, top=2, ff=9)),
                                                      attn2_layer(heads=2, kv_heads=2, dim=6, vdim=5, rot_dims=6, size=11, keep=3)],
                                                     width=70, vocab=131, bigram=(17, 1000003, 99998300017)),
}


@pytest.mark.parametrize('name', sorted(MECHANISMS))
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_each_mechanism_whole_prompt(name, dtype):
    cfg = MECHANISMS[name]
    toks = tokens_for(cfg, 150, 1)  # crosses page borders and windows
    w = weights_for(cfg, len(name), dtype, toks)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', len(toks))]])['a']
    check_rows(got, toks, w, cfg, dtype, name)


@pytest.mark.parametrize('ranks', [(8, 16), (1, 3), (40, 24)])
def test_ranks_of_the_low_rank_pairs_come_from_the_tensors(ranks):
    cfg = make_config([delta_layer(mlp=moe())])
    toks = tokens_for(cfg, 70, 2)
    for dtype in ('float32', 'bfloat16'):
        w = weights_for(cfg, 4, dtype, toks, ranks=ranks)
        check_rows(replay(session_for(cfg, w, dtype), {'a': toks}, [[('a', 70)]])['a'], toks, w, cfg, dtype)


def test_residual_stream_behind_every_layer():
    cfg = MECHANISMS['whole_stack']
    toks = tokens_for(cfg, 19, 2)
    w = weights_for(cfg, 3, 'float32', toks)
    taps = []
    O.forward(toks, as_f64(w), cfg, taps)
    s = session_for(cfg, w, 'float32', debug_mode=True)
    s.step([('a', toks, [0])])
    assert s.engine.layer_runs == len(taps) == len(FULL)
    for j, x in enumerate(taps):
        assert np.abs(s.engine.tap(j) - x).max() < 2e-4 * np.abs(x).max(), f'layer {j}'


@pytest.mark.parametrize('stack', sorted(STACKS))
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_prefill_then_token_by_token(dtype, stack):
    cfg = stack_config(stack)
    toks = tokens_for(cfg, 170, 3)
    w = weights_for(cfg, 5, dtype, toks)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', 100)]] + [[('a', 1)]] * 70)['a']
    check_rows(got, toks, w, cfg, dtype)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('sizes', [[2] * 40, [3, 61, 2, 64, 1, 5, 2, 58, 1, 1, 2], [63, 2, 63, 1, 1, 66], [1] * 9 + [120, 2], [36, 1, 37, 29, 28, 2, 45]])
@pytest.mark.parametrize('stack', sorted(STACKS))
def test_portions_of_a_prompt(sizes, dtype, stack):
    cfg = stack_config(stack)
    toks = tokens_for(cfg, sum(sizes), 4)
    w = weights_for(cfg, 8, dtype, toks)
    s = session_for(cfg, w, dtype)
    got = replay(s, {'a': toks}, [[('a', n)] for n in sizes])['a']
    check_rows(got, toks, w, cfg, dtype)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('stack', sorted(STACKS))
def test_unequal_requests_in_one_batch_equal_each_alone(dtype, stack):
    cfg = stack_config(stack)
    reqs = {'a': tokens_for(cfg, 131, 5), 'b': tokens_for(cfg, 9, 6), 'c': tokens_for(cfg, 66, 7), 'd': tokens_for(cfg, 2, 8)}
    w = weights_for(cfg, 9, dtype, reqs)
    schedule = [[('a', 60), ('b', 2)], [('b', 1), ('a', 5), ('c', 64)], [('c', 1), ('b', 1), ('a', 1), ('d', 2)],
                [('a', 63), ('b', 5), ('c', 1)], [('a', 1)], [('a', 1)]]
    s = session_for(cfg, w, dtype)
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check_rows(got[rid], toks, w, cfg, dtype, rid)
    assert not s.live() and s.cache.blocks_manager.num_free_blocks() == s.num_blocks and s.slots.num_free_slots() == 4


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_requests_of_very_unequal_length_decode_side_by_side(dtype):
    cfg = stack_config('tiled')
    reqs = {'long': tokens_for(cfg, 420, 90), 'mid': tokens_for(cfg, 75, 91), 'new': tokens_for(cfg, 12, 92)}
    w = weights_for(cfg, 21, dtype, reqs)
    schedule = [[('long', 400)], [('mid', 65), ('long', 1)]] + [[('long', 1), ('mid', 1), ('new', 1)]] * 10 + [[('long', 9), ('new', 2)]]
    s = session_for(cfg, w, dtype, max_tokens=1024)
    got = replay(s, reqs, schedule)
    for rid, toks in reqs.items():
        check_rows(got[rid], toks, w, cfg, dtype, rid)


def test_pages_and_slots_that_are_used_again():
    """A pool of 4 pages and 2 slots serves six requests one after another and side by side: every page and every state slot is
    written by several requests, and what an earlier request left there - keys behind a window, a recurrent state, a convolution's
    tail, the row a token shift carries, the previous token of the pair embedding - must never be seen by a later one."""
    cfg = stack_config('general', 4)
    s = None
    used_blocks, used_slots = [], []
    for rnd in range(3):
        reqs = {f'x{rnd}': tokens_for(cfg, 100 + rnd, 20 + rnd), f'y{rnd}': tokens_for(cfg, 70 - rnd, 30 + rnd)}
        if s is None:
            w = weights_for(cfg, 11, 'float32')
            s = session_for(cfg, w, 'float32', max_tokens=256, max_sequences=2)
            assert s.num_blocks == 4
        x, y = f'x{rnd}', f'y{rnd}'
        schedule = [[(x, 50), (y, 3)], [(y, len(reqs[y]) - 3), (x, 1)], [(x, len(reqs[x]) - 51)]]
        got = replay(s, reqs, schedule, end_when_done=False)
        for rid in reqs:
            seq = s._seq[rid]
            used_blocks.append(tuple(s.cache.blocks_manager.block_ids(seq)[0]))
            used_slots.append(s.slots.slot_of(seq))
            assert O.routing_margin(reqs[rid], as_f64(w), cfg) > 1e-4
            check(got[rid], O.logits(reqs[rid], as_f64(w), cfg), F32_TOL, rid)
            s.release(rid)
    assert len(set(used_slots)) == 2 and len(used_slots) == 6
    assert len({b for blocks in used_blocks for b in blocks}) == 4 and sum(len(b) for b in used_blocks) == 12


def rigged_attention(kind, n, p_far, seed, size, keep, D=16):
    """One attention layer whose head 0 is rigged so that the LAST token's query meets the key of the token at p_far with a score far
    above all others: if that key is visible it decides the answer, and dropping, shifting or corrupting it moves the logits at the
    last position by much more than bfloat16 rounding; if the mask hides it, letting it in by mistake does the same.  Channel 0 of the
    residual is loud for the far token only and channel 1 for the last token only (nothing else writes there; the pair table and the
    shift ratios are zero in this model); the last dimension of head 0 - which does not turn - reads nothing but channel 0
    on the key side and channel 1 on the query side."""
    if kind == 'attention':
        layer = attn_layer(heads=4, kv_heads=2, dim=D, rot_dims=D // 2, size=size, keep=keep)
    else:
        layer = attn2_layer(heads=4, kv_heads=2, dim=D, vdim=24 if D == 16 else D, rot_dims=D // 2, size=size, keep=keep)
    cfg = make_config([layer])
    w = random_weights(cfg, seed)
    rng = np.random.default_rng(seed)
    far_tok = 3
    last_tok = far_tok if p_far == n - 1 else 4  # (a window of one: the last token is its own only key)
    toks = [int(t) for t in rng.integers(5, cfg['vocab'], n)]
    toks[p_far], toks[-1] = far_tok, last_tok
    w['embed'][:, :2] = 0.0
    w['embed'][far_tok, 0] = w['embed'][last_tok, 1] = 8.0
    # a token reaches its neighbour neither through the pair table nor through the shift: what a hidden key changes stays hidden
    w['bigram'][:] = 0.0
    w['l0.norm1'][:2] = 1.0
    w['l0.shift'][:] = 0.0
    w['l0.mix.k'][D - 1] = 0.0
    w['l0.mix.k'][D - 1, 0] = 4.0
    w['l0.mix.q'][D - 1] = 0.0
    w['l0.mix.q'][D - 1, 1] = 2.0 if kind == 'attention' else 4.0
    if kind == 'attention':
        w['l0.mix.sink'][0] = 2.0
        w['l0.mix.talk'][:, 0] = np.array([1.0, 0.5, -0.5, 0.25], np.float32)  # what head 0 sees reaches every head
    else:
        w['l0.mix.q.b'][D - 1] = w['l0.mix.k.b'][D - 1] = 0.0
        w['l0.mix.q.norm'][D - 1] = w['l0.mix.k.norm'][D - 1] = 2.0
        w['l0.mix.v'] *= 4.0
    return cfg, w, toks


def rigged_delta(n, p_far, seed):
    """One delta-rule layer that forgets slowly (small rates, small steps) and whose first q / k head is rigged like the attention
    above: key channel 0 is loud at the far token (and, through the convolution, at the tokens right behind it), query channel 0 at
    the last token, and the far token's values are large - what it wrote into the state is most of what the last token reads, so a
    state that is lost, mixed up between slots or decayed wrongly on the way shows at the last position."""
    cfg = make_config([delta_layer(heads=4, kv_heads=2, dim=10, vdim=12, conv=4)])
    w = random_weights(cfg, seed)
    rng = np.random.default_rng(seed)
    far_tok, last_tok = 3, 4
    toks = [int(t) for t in rng.integers(5, cfg['vocab'], n)]
    toks[p_far] = far_tok
    if p_far != n - 1:
        toks[-1] = last_tok
    w['embed'][:, :2] = 0.0
    w['embed'][far_tok, 0] = w['embed'][last_tok, 1] = 8.0
    if p_far == n - 1:
        w['embed'][far_tok, 1] = 8.0
    w['bigram'][:, :2] = 0.0
    w['l0.norm1'][:2] = 1.0
    w['l0.shift'][:2] = 0.0
    w['l0.mix.k'][0] = 0.0
    w['l0.mix.k'][0, 0] = 4.0
    w['l0.mix.q'][0] = 0.0
    w['l0.mix.q'][0, 1] = 4.0
    w['l0.mix.q.conv'][0] = w['l0.mix.k.conv'][0] = np.array([0.0, 0.0, 0.0, 1.0], np.float32)
    w['l0.mix.v'][:, 0] = 1.0
    w['l0.mix.dt_bias'][:] = -6.0
    w['l0.mix.a2'] *= 0.25
    w['l0.mix.A_log'][:] = bf16_round(np.log(np.float32(0.05)))
    return cfg, w, toks


def run_rigged(cfg, w, toks, p_far, dtype, sees):
    n = len(toks)
    wf = as_f64(w)
    want = O.logits(toks, wf, cfg)
    other = list(toks)
    other[p_far] = 7
    moved = rel_err(O.logits(other, wf, cfg)[-1:], want[-1:])[0]
    if sees:
        assert moved > 0.1, f'the rig does not bite: replacing the far token moves the last row by {moved:.3g} only'
    else:
        assert moved < 1e-9, f'the key at {p_far} should be hidden from the last row'
    s = session_for(cfg, w, dtype)
    cut = max(p_far + 1, 2) if p_far + 1 < n else n - 1
    # in a whole prompt, in a portion that starts behind the far token, and decoded alone
    check(replay(s, {'w': toks}, [[('w', n)]])['w'][-1:], want[-1:], tol_of(dtype), 'whole')
    check(replay(s, {'p': toks}, [[('p', cut)], [('p', n - cut)]])['p'][-1:], want[-1:], tol_of(dtype), 'portion')
    check(replay(s, {'d': toks}, [[('d', n - 1)], [('d', 1)]])['d'][-1:], want[-1:], tol_of(dtype), 'decoded')


KINDS = [('float32', 16), ('bfloat16', 16), ('bfloat16', 64)]  # D = 64: a shape of the tile kernels


@pytest.mark.parametrize('p_far', [0, 1, 31, 32, 63, 64, 127, 128, 200, 331])
@pytest.mark.parametrize('dtype,D', KINDS)
@pytest.mark.parametrize('kind', ['attention', 'attention_2'])
def test_a_far_key_that_decides_the_answer(kind, p_far, dtype, D):
    cfg, w, toks = rigged_attention(kind, 333, p_far, seed=40 + p_far, size=0, keep=0, D=D)
    run_rigged(cfg, w, toks, p_far, dtype, sees=True)


@pytest.mark.parametrize('n,size,back,sees', [(120, 37, 36, True), (120, 37, 37, False), (130, 64, 63, True), (130, 64, 64, False),
                                             (200, 65, 64, True), (200, 65, 65, False), (40, 2, 1, True), (40, 2, 2, False),
                                             (129, 128, 127, True), (300, 128, 128, False), (30, 1, 0, True), (30, 1, 1, False)])
@pytest.mark.parametrize('dtype,D', KINDS)
@pytest.mark.parametrize('kind', ['attention', 'attention_2'])
def test_keys_at_the_edge_of_a_window(kind, n, size, back, sees, dtype, D):
    """The last row sits at position n - 1; the rigged key `back` tokens before it is the last one inside the window, or the first
    one outside (the kept first tokens end well before it)."""
    cfg, w, toks = rigged_attention(kind, n, n - 1 - back, seed=40 + back, size=size, keep=3 if n - 1 - back >= 3 else 0, D=D)
    run_rigged(cfg, w, toks, n - 1 - back, dtype, sees)


@pytest.mark.parametrize('n,size,keep,p_far,sees', [(150, 20, 1, 0, True), (150, 20, 1, 1, False), (150, 20, 7, 6, True), (150, 20, 7, 7, False),
                                                   (200, 37, 32, 31, True), (200, 37, 32, 32, False), (200, 10, 64, 63, True),
                                                   (200, 10, 64, 64, False), (300, 64, 65, 64, True), (300, 64, 65, 65, False),
                                                   (40, 1, 33, 32, True), (40, 1, 33, 33, False), (700, 320, 40, 39, True),
                                                   (700, 320, 40, 40, False)])
@pytest.mark.parametrize('dtype,D', KINDS)
@pytest.mark.parametrize('kind', ['attention', 'attention_2'])
def test_the_first_tokens_that_a_window_keeps(kind, n, size, keep, p_far, sees, dtype, D):
    """The rigged key is the last of the kept first tokens, or the first one behind them; the window is far away from both."""
    cfg, w, toks = rigged_attention(kind, n, p_far, seed=70 + p_far, size=size, keep=keep, D=D)
    run_rigged(cfg, w, toks, p_far, dtype, sees)


@pytest.mark.parametrize('p_far', [0, 1, 2, 3, 63, 64, 150, 298])
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_a_far_token_that_lives_on_in_the_state(p_far, dtype):
    cfg, w, toks = rigged_delta(300, p_far, seed=60 + p_far)
    run_rigged(cfg, w, toks, p_far, dtype, sees=True)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
@pytest.mark.parametrize('kind', ['attention', 'attention_2'])
def test_the_sink_takes_its_share(kind, dtype):
    """With the sink left out of the denominator every head's output would be too large by 1 / (1 - sink's share): the learned
    sinks are made larger than most scores; the constant one meets scores that are mostly negative."""
    cfg = make_config([attn_layer(size=20) if kind == 'attention' else attn2_layer(size=20, scale=0.2)])
    w = random_weights(cfg, 33)
    if kind == 'attention':
        w['l0.mix.sink'][:] = 8.0
    toks = tokens_for(cfg, 70, 34)
    wf = as_f64(w)
    want = O.logits(toks, wf, cfg)
    if kind == 'attention':
        no_sink = dict(wf)
        no_sink['l0.mix.sink'] = np.full_like(wf['l0.mix.sink'], -60.0)
        assert np.median(rel_err(O.logits(toks, no_sink, cfg), want)) > 0.1
    s = session_for(cfg, w, dtype)
    check_rows(replay(s, {'a': toks}, [[('a', 40)]] + [[('a', 1)]] * 30)['a'], toks, w, cfg, dtype)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_heads_whose_weights_are_swapped_by_the_mixing_matrix(dtype):
    """A mixing matrix that is a permutation plus a negative entry: every head applies ANOTHER head's weights to its own values, so
    leaving the mixing out, transposing it or applying it before the softmax all give a different answer."""
    cfg = make_config([attn_layer(heads=4, kv_heads=2, dim=16, rot_dims=8, size=50, keep=2)])
    w = random_weights(cfg, 35)
    w['l0.mix.talk'] = np.array([[0, 0, 1, 0], [1, 0, 0, -0.5], [0, 1, 0, 0], [0, 0.5, 0, 1]], np.float32)
    toks = tokens_for(cfg, 90, 36)
    wf = as_f64(w)
    want = O.logits(toks, wf, cfg)
    for wrong in (np.eye(4), wf['l0.mix.talk'].T):
        other = dict(wf)
        other['l0.mix.talk'] = wrong
        assert np.median(rel_err(O.logits(toks, other, cfg), want)) > 0.1
    s = session_for(cfg, w, dtype)
    check_rows(replay(s, {'a': toks}, [[('a', 50)], [('a', 7)]] + [[('a', 1)]] * 33)['a'], toks, w, cfg, dtype)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_the_shift_reads_the_token_before_across_steps(dtype):
    """Shift ratios of one: a mixer reads nothing but the PREVIOUS token's normed row, so a carried row that is lost, stale or taken
    from the shifted row instead of the plain one shows everywhere; every portion border and every decoded token needs the carry."""
    cfg = make_config([attn2_layer(), delta_layer(), attn_layer()])
    w = random_weights(cfg, 37)
    for i in range(3):
        w[f'l{i}.shift'][:] = 1.0
    toks = tokens_for(cfg, 80, 38)
    wf = as_f64(w)
    unshifted = dict(wf)
    for i in range(3):
        unshifted[f'l{i}.shift'] = np.zeros_like(wf[f'l{i}.shift'])
    assert np.median(rel_err(O.logits(toks, unshifted, cfg), O.logits(toks, wf, cfg))) > 0.1
    s = session_for(cfg, w, dtype)
    check_rows(replay(s, {'a': toks}, [[('a', 3)], [('a', 2)], [('a', 40)]] + [[('a', 1)]] * 35)['a'], toks, w, cfg, dtype)


def test_the_pair_embedding_knows_the_token_before_across_steps():
    """A model whose token embedding is zero: all it knows of its input is the pair table's rows, so the previous token of every
    step's first row, and the extra row of a sequence's first token, decide everything."""
    cfg = make_config([attn_layer(mlp=moe())], bigram=(97, 12345, 6789))
    w = random_weights(cfg, 39)
    w['embed'][:] = 0.0
    w['bigram'] *= 2.0
    toks = tokens_for(cfg, 70, 40)
    assert O.routing_margin(toks, as_f64(w), cfg) > 1e-4
    s = session_for(cfg, w, 'float32')
    want = O.logits(toks, as_f64(w), cfg)
    check(replay(s, {'a': toks}, [[('a', 1)], [('a', 2)], [('a', 30)]] + [[('a', 1)]] * 37)['a'], want, F32_TOL)
    other = {'b': tokens_for(cfg, 9, 41), 'c': toks}   # another request in the slot's place between c's steps
    got = replay(s, other, [[('c', 5), ('b', 4)], [('b', 5)], [('c', 65)]])
    check(got['c'], want, F32_TOL)


def test_first_tokens_of_a_sequence():
    cfg = MECHANISMS['whole_stack']
    w = weights_for(cfg, 13, 'float32')
    s = session_for(cfg, w, 'float32')
    for n in (1, 2, 3, 4, 5):
        toks = tokens_for(cfg, n, 50 + n)
        assert O.routing_margin(toks, as_f64(w), cfg) > 1e-4
        check(replay(s, {n: toks}, [[(n, n)]])[n], O.logits(toks, as_f64(w), cfg), F32_TOL, f'{n} tokens at once')
        check(replay(s, {-n: toks}, [[(-n, 1)]] * n)[-n], O.logits(toks, as_f64(w), cfg), F32_TOL, f'{n} tokens one by one')


@pytest.mark.parametrize('stack', sorted(STACKS))
def test_long_decoding(stack):
    cfg = stack_config(stack, 3)
    toks = tokens_for(cfg, 330, 9)
    for dtype in ('float32', 'bfloat16'):
        w = weights_for(cfg, 15, dtype, toks)
        s = session_for(cfg, w, dtype)
        check_rows(replay(s, {'a': toks}, [[('a', 2)]] + [[('a', 1)]] * 328)['a'], toks, w, cfg, dtype, dtype)


SMALL = make_config([attn2_layer(heads=2, kv_heads=1, dim=16, vdim=16, rot_dims=8, size=23, keep=2, mlp=moe(experts=4, top=2, ff=16)),
                     delta_layer(heads=2, kv_heads=1, dim=8, vdim=16, mlp=moe(experts=3, top=1, ff=16)),
                     attn_layer(heads=2, kv_heads=1, dim=16, rot_dims=16, size=19, keep=4, mlp=None)], width=64, vocab=97)


def test_greedy_generation_through_the_scheduler():
    """Six prompts, four state slots, 40 tokens per step: prompts are cut, requests queue, decoded tokens share steps with prompt
    portions.  fp32 engine against the oracle's greedy continuation (recomputed from scratch for every token)."""
    from tensorrt_llm.runtime import SamplingConfig
    cfg = SMALL
    w = random_weights(cfg, seed=17)
    prompts = [tokens_for(cfg, n, 60 + n) for n in (70, 3, 45, 1, 90, 17)]
    s = session_for(cfg, w, 'float32', max_tokens=512, max_sequences=4, max_batch_tokens=40)
    outs = s.decode_batch(prompts, SamplingConfig(end_id=-1, pad_id=0), max_new_tokens=6)
    for p, o in zip(prompts, outs):
        assert o.tolist() == O.greedy(p, as_f64(w), cfg, 6)
    assert not s.live() and s.cache.blocks_manager.num_free_blocks() == s.num_blocks


def test_command_lines(tmp_path):
    """examples/narurax/run.py generates from a checkpoint directory; bin/trace_run replays a recorded schedule from it."""
    from test_gpu_tolenex import write_checkpoint
    cfg = SMALL
    w = random_weights(cfg, seed=19)
    ck = str(tmp_path / 'ck')
    write_checkpoint(ck, cfg, w)
    prompt = tokens_for(cfg, 21, 70)
    np.save(tmp_path / 'in.npy', np.asarray(prompt, np.int32))
    run = os.path.join(ROOT, 'trtllm-llama_amd', 'examples', 'narurax', 'run.py')
    subprocess.run([sys.executable, run, '--model_dir', ck, '--dtype', 'float32', '--input_tokens', str(tmp_path / 'in.npy'),
                    '--max_output_len', '5', '--output_npy', str(tmp_path / 'out.npy')], check=True, timeout=300)
    assert np.load(tmp_path / 'out.npy').reshape(-1)[len(prompt):].tolist() == O.greedy(prompt, as_f64(w), cfg, 5)
    a, b = tokens_for(cfg, 70, 71), tokens_for(cfg, 5, 72)
    steps = [{'step': 0, 'entries': [{'id': 'a', 'tokens': a[:66], 'want': [0, 65]}, {'id': 'b', 'tokens': b[:2], 'want': []}], 'end': []},
             {'step': 1, 'entries': [{'id': 'b', 'tokens': b[2:], 'want': [2]}], 'end': ['b']},
             {'step': 2, 'entries': [{'id': 'a', 'tokens': a[66:], 'want': [3]}], 'end': ['a']}]
    out = tmp_path / 'logits'
    r = subprocess.run([os.path.join(ROOT, 'bin', 'trace_run'), '--model', ck, '--dtype', 'float32', '--out', str(out), '--max-tokens', '192'],
                       input='\n'.join(json.dumps(s) for s in steps) + '\n', capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith('done')] == ['done 0', 'done 1', 'done 2']
    la, lb = O.logits(a, as_f64(w), cfg), O.logits(b, as_f64(w), cfg)
    check(np.fromfile(out / '0.f32', '<f4').reshape(2, -1), la[[0, 65]], F32_TOL)
    check(np.fromfile(out / '1.f32', '<f4').reshape(1, -1), lb[[4]], F32_TOL)
    check(np.fromfile(out / '2.f32', '<f4').reshape(1, -1), la[[69]], F32_TOL)
