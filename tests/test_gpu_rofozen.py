"""Rofozen through the ragged stack engine against the plain float64 oracle (oracle/rofozen_oracle.py), on small configurations and
random weights made here.  fp32 engine: tight bound (what summation order can explain), routers with random weights (their decisions
are checked on the oracle not to be close calls at that bound); bfloat16 engine: loose bound, routers rigged so that no decision is
close, and crafted weights where random ones would hide a fault (a key at a window's edge, one far key among hundreds, a sink, one
far token whose trace must survive in a recurrent state)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from oracle import rofozen_oracle as O
from rofozen_cases import (as_model, decisive_router, dense, latent_layer, make_config, mamba_layer, moe, random_weights, routing_margin,
                           shared)
from tolenex_cases import as_f64, bf16_round, rel_err, replay

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F32_TOL, BF16_TOL = 3e-5, 5e-2


def has_router(cfg):
    return any(l.get('mlp') and l['mlp']['kind'] == 'moe' for l in cfg['layers'])


def weights_for(cfg, seed, dtype, toks=None):
    """Random weights; for the bfloat16 engine the routers are rigged.  With `toks`, the routers' decisions on them are checked on
    the oracle to stand clear of what the engine's rounding can move; a model with a close call is passed over for the next seed."""
    need = 0.2 if dtype == 'bfloat16' else 2e-4
    for attempt in range(10):
        w = random_weights(cfg, seed + 1000 * attempt)
        if not has_router(cfg):
            return w
        if dtype == 'bfloat16':
            w = decisive_router(cfg, w, seed)
        if toks is None or all(routing_margin(cfg, w, t) > need for t in (toks.values() if isinstance(toks, dict) else [toks])):
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
    """Every position of a request against the oracle.  fp32: the flat bound.  bfloat16: rows differ in how much rounding moves
    them - where a recurrence's output nearly cancels, the norm behind it magnifies what rounding left - so a row is held to 3 x
    what rounding the oracle's own activations to bfloat16 does to it (never less than the median row's), no row may pass 1.5 x
    that, and at most one row in fifty (or one) may pass it at all."""
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
    assert np.median(e) < 2e-2, f'{what}: the median row is off by {np.median(e):.3g}'


FULL = [mamba_layer(mlp=dense()), latent_layer(mlp=moe()), shared(mamba_layer(mlp=dense()), 0),
        mamba_layer(heads=4, vdim=8, state=16, groups=1, conv=3, norm_groups=1, mlp=moe(experts=8, identity=0, top=3, count=4, keep=2)),
        latent_layer(heads=1, dim=8, rot_dim=12, vdim=16, kv_rank=24, q_rank=10, size=64, scaling=False, mlp=None),
        shared(latent_layer(mlp=moe()), 1)]
# shapes the MFMA tile kernels and the LDS-staged products take in bfloat16; fp32 runs them on the general kernels
TILED = [mamba_layer(heads=4, vdim=32, state=64, groups=2, conv=4, norm_groups=4, mlp=moe(experts=4, identity=1, top=2, count=1, keep=1, ff=64)),
         latent_layer(heads=2, dim=32, rot_dim=32, vdim=32, kv_rank=128, q_rank=64, size=45, mlp=dense(128)),
         latent_layer(heads=3, dim=16, rot_dim=64, vdim=16, kv_rank=256, q_rank=64, size=130, mlp=None),
         mamba_layer(heads=2, vdim=64, state=128, groups=1, conv=4, norm_groups=1, mlp=dense(64))]
STACKS = {'general': (FULL, 96), 'tiled': (TILED, 128)}


def stack_config(name, layers=None):
    full, width = STACKS[name]
    return make_config(full if layers is None else full[:layers], width=width)


MECHANISMS = {
    'mamba_alone_no_ff': make_config([mamba_layer()]),
    'mamba_one_group_one_norm_part': make_config([mamba_layer(groups=1, norm_groups=1)]),
    'mamba_a_group_and_a_norm_part_per_head': make_config([mamba_layer(heads=4, groups=4, norm_groups=4)]),
    'mamba_one_head': make_config([mamba_layer(heads=1, vdim=20, state=7, groups=1, norm_groups=1)]),
    'mamba_one_tap': make_config([mamba_layer(conv=1)]),
    'mamba_two_taps': make_config([mamba_layer(conv=2)]),
    'mamba_seven_taps': make_config([mamba_layer(conv=7)]),
    'mamba_state_of_one': make_config([mamba_layer(state=1)]),
    'mamba_large_state_small_head': make_config([mamba_layer(heads=2, vdim=4, state=200, groups=2)]),
    'mamba_wide_head': make_config([mamba_layer(heads=2, vdim=96, state=24, groups=1)]),
    'mamba_tile_64_128': make_config([TILED[3]], width=128),
    'latent_alone_no_ff': make_config([latent_layer()]),
    'latent_window_of_one': make_config([latent_layer(size=1)]),
    'latent_window_two': make_config([latent_layer(size=2)]),
    'latent_window_a_page': make_config([latent_layer(size=64)]),
    'latent_window_wider_than_the_prompt': make_config([latent_layer(size=500)]),
    'latent_no_window': make_config([latent_layer(size=0)]),
    'latent_no_frequency_scaling': make_config([latent_layer(scaling=False)]),
    'latent_one_head': make_config([FULL[4]]),
    'latent_many_heads_odd_sizes': make_config([latent_layer(heads=7, dim=6, rot_dim=2, vdim=10, kv_rank=18, q_rank=9, size=33)], width=72),
    'latent_wide_query_latent': make_config([latent_layer(q_rank=150)]),
    'latent_tile_160_128': make_config([TILED[1]], width=128),
    'latent_tile_320_256': make_config([TILED[2]], width=128),
    'dense_ff': make_config([mamba_layer(mlp=dense(50))]),
    'moe_one_group': make_config([mamba_layer(mlp=moe(experts=5, identity=1, top=2, count=1, keep=1))]),
    'moe_all_groups_kept': make_config([mamba_layer(mlp=moe(experts=6, identity=2, top=3, count=4, keep=4))]),
    'moe_three_of_five_groups': make_config([mamba_layer(mlp=moe(experts=9, identity=1, top=2, count=5, keep=3))]),
    'moe_no_identity': make_config([latent_layer(mlp=moe(experts=6, identity=0, top=2, count=3, keep=1))]),
    'moe_top_one': make_config([mamba_layer(mlp=moe(experts=4, identity=2, top=1, count=2, keep=1, scale=1.0))]),
    'moe_every_expert_of_the_kept_group': make_config([mamba_layer(mlp=moe(experts=6, identity=2, top=4, count=2, keep=1))]),
    'moe_mostly_identities': make_config([mamba_layer(mlp=moe(experts=2, identity=6, top=3, count=2, keep=2))]),
    'moe_wide_experts': make_config([TILED[0]], width=128),
    'shared_weights': make_config([mamba_layer(mlp=moe()), latent_layer(mlp=dense()), shared(mamba_layer(mlp=moe()), 0),
                                   shared(latent_layer(mlp=dense()), 1), shared(mamba_layer(mlp=moe()), 0)]),
    'whole_stack': make_config(FULL, eps=3e-6),
    'tiled_stack': make_config(TILED, width=128),
    'width_that_is_no_multiple_of_four': make_config([mamba_layer(heads=3, vdim=7, state=5, groups=1, norm_groups=3, mlp=moe(ff=10)),
                                                      latent_layer(heads=2, dim=7, rot_dim=6, vdim=5, kv_rank=13, q_rank=11, size=9, mlp=dense(30))],
                                                     width=70, vocab=131),
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


def test_residual_stream_behind_every_layer():
    cfg = MECHANISMS['whole_stack']
    toks = tokens_for(cfg, 19, 2)
    w = weights_for(cfg, 3, 'float32', toks)
    _, taps = O.forward(toks, as_f64(w), cfg, return_layers=True)
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
    tail - must never be seen by a later one."""
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
            assert routing_margin(cfg, w, reqs[rid]) > 1e-4
            check(got[rid], O.logits(reqs[rid], as_f64(w), cfg), F32_TOL, rid)
            s.release(rid)
    assert len(set(used_slots)) == 2 and len(used_slots) == 6
    assert len({b for blocks in used_blocks for b in blocks}) == 4 and sum(len(b) for b in used_blocks) == 12


def rigged_latent(n, p_far, seed, size, D=16):
    """One latent layer whose head 0 is rigged so that the LAST token's query meets the key of the token at p_far with a score far
    above all others: if that key is visible it decides the answer, and dropping, shifting or corrupting it moves the logits at the
    last position by much more than bfloat16 rounding; if the window hides it, letting it in by mistake does the same.  The query
    goes through its latent: channel 0 of the query latent is loud for the last token only, and row D - 1 of head 0's expansion reads
    nothing else; channel 0 of the key latent is loud for the far token only, and row D - 1 of head 0's key expansion reads nothing else."""
    E = 24 if D == 16 else 64
    cfg = make_config([latent_layer(heads=2, dim=D, rot_dim=D // 2, vdim=E, kv_rank=2 * D, q_rank=D + 4, size=size)])
    w = random_weights(cfg, seed)
    rng = np.random.default_rng(seed)
    far_tok = 3
    last_tok = far_tok if p_far == n - 1 else 4  # (a window of one: the last token is its own only key)
    toks = [int(t) for t in rng.integers(5, cfg['vocab'], n)]
    toks[p_far], toks[-1] = far_tok, last_tok
    m = cfg['layers'][0]['mixer']
    # channel 0 of the residual belongs to the far token and channel 1 to the last one: no other embedding has anything there
    w['embed'][:, :2] = 0.0
    w['embed'][far_tok, 0] = w['embed'][last_tok, 1] = 8.0
    w['l0.norm1'][:2] = 1.0
    w['l0.mix.dkv'][0] = 0.0
    w['l0.mix.dkv'][0, 0] = 4.0
    w['l0.mix.uk'][D - 1] = 0.0
    w['l0.mix.uk'][D - 1, 0] = 1.0
    w['l0.mix.dkv.norm'][0] = 1.0
    w['l0.mix.dq'][0] = 0.0
    w['l0.mix.dq'][0, 1] = 4.0
    w['l0.mix.dq.norm'][0] = 1.0
    w['l0.mix.uq'][D - 1] = 0.0
    w['l0.mix.uq'][D - 1, 0] = bf16_round(np.float32(32.0 / m['scale'] / (2 * D) ** 0.5 / (D + 4) ** 0.5))
    w['l0.mix.sink'][0] = 2.0
    w['l0.mix.uv'][:E] *= 4.0
    return cfg, w, toks


def rigged_mamba(n, p_far, seed):
    """One mamba2 layer whose heads forget slowly and take a large step at one token only (the step size's projection points at that
    token's input, the bias keeps every other step small): what the far token wrote into the state is most of what the last token
    reads, so a state that is lost, mixed up between slots or decayed wrongly on the way shows at the last position."""
    cfg = make_config([mamba_layer(heads=4, vdim=12, state=10, groups=2, conv=4, norm_groups=2)])
    w = random_weights(cfg, seed)
    rng = np.random.default_rng(seed)
    far_tok = 3
    toks = [int(t) for t in rng.integers(5, cfg['vocab'], n)]
    toks[p_far] = far_tok
    w['embed'][:, 0] = 0.0  # channel 0 of the residual belongs to the far token
    w['embed'][far_tok, 0] = 8.0
    w['l0.norm1'][0] = 1.0
    H = 4
    w['l0.mix.in'][-H:] = 0.0
    w['l0.mix.in'][-H:, 0] = 1.5
    w['l0.mix.dt_bias'][:] = -5.0
    w['l0.mix.A_log'][:] = bf16_round(np.log(np.float32(0.02)))
    w['l0.mix.D'][:] = 0.0625
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


KINDS = [('float32', 16), ('bfloat16', 16), ('bfloat16', 64)]  # D = 64: 128 + 32 dimensions, a shape of the tile kernels


@pytest.mark.parametrize('p_far', [0, 1, 31, 32, 63, 64, 127, 128, 200, 331])
@pytest.mark.parametrize('dtype,D', KINDS)
def test_a_far_key_that_decides_the_answer(p_far, dtype, D):
    cfg, w, toks = rigged_latent(333, p_far, seed=40 + p_far, size=0, D=D)
    run_rigged(cfg, w, toks, p_far, dtype, sees=True)


@pytest.mark.parametrize('n,size,back,sees', [(120, 37, 36, True), (120, 37, 37, False), (130, 64, 63, True), (130, 64, 64, False),
                                             (200, 65, 64, True), (200, 65, 65, False), (40, 2, 1, True), (40, 2, 2, False),
                                             (129, 128, 127, True), (300, 128, 128, False), (30, 1, 0, True), (30, 1, 1, False)])
@pytest.mark.parametrize('dtype,D', KINDS)
def test_keys_at_the_edge_of_a_window(n, size, back, sees, dtype, D):
    """The last row sits at position n - 1; the rigged key `back` tokens before it is the last one inside the window, or the first
    one outside."""
    cfg, w, toks = rigged_latent(n, n - 1 - back, seed=40 + back, size=size, D=D)
    run_rigged(cfg, w, toks, n - 1 - back, dtype, sees)


@pytest.mark.parametrize('p_far', [0, 1, 2, 3, 63, 64, 150, 298])
@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_a_far_token_that_lives_on_in_the_state(p_far, dtype):
    cfg, w, toks = rigged_mamba(300, p_far, seed=60 + p_far)
    run_rigged(cfg, w, toks, p_far, dtype, sees=True)


@pytest.mark.parametrize('dtype', ['float32', 'bfloat16'])
def test_the_sink_takes_its_share(dtype):
    """With the sink left out of the denominator every head's output would be too large by 1 / (1 - sink's share): here the sinks
    are larger than most scores, so their share is a large part."""
    cfg = make_config([latent_layer(size=20)])
    w = random_weights(cfg, 33)
    w['l0.mix.sink'][:] = 8.0
    toks = tokens_for(cfg, 70, 34)
    wf = as_f64(w)
    want = O.logits(toks, wf, cfg)
    without = {k: v for k, v in wf.items() if k != 'l0.mix.sink'}
    assert np.median(rel_err(O.logits(toks, without, cfg), want)) > 0.1
    s = session_for(cfg, w, dtype)
    check_rows(replay(s, {'a': toks}, [[('a', 40)]] + [[('a', 1)]] * 30)['a'], toks, w, cfg, dtype)


def test_first_tokens_of_a_sequence():
    cfg = MECHANISMS['whole_stack']
    w = weights_for(cfg, 13, 'float32')
    s = session_for(cfg, w, 'float32')
    for n in (1, 2, 3, 4, 5):
        toks = tokens_for(cfg, n, 50 + n)
        assert routing_margin(cfg, w, toks) > 1e-4
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


SMALL = make_config([mamba_layer(heads=2, vdim=16, state=8, groups=1, norm_groups=2, mlp=moe(experts=4, identity=1, top=2, count=1, keep=1, ff=16)),
                     latent_layer(heads=2, size=23, mlp=dense(48)),
                     shared(mamba_layer(heads=2, vdim=16, state=8, groups=1, norm_groups=2, mlp=moe(experts=4, identity=1, top=2, count=1, keep=1, ff=16)), 0)],
                    width=64, vocab=97)


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
    """examples/rofozen/run.py generates from a checkpoint directory; bin/trace_run replays a recorded schedule from it."""
    from test_gpu_tolenex import write_checkpoint
    cfg = SMALL
    w = random_weights(cfg, seed=19)
    ck = str(tmp_path / 'ck')
    write_checkpoint(ck, cfg, w)
    prompt = tokens_for(cfg, 21, 70)
    np.save(tmp_path / 'in.npy', np.asarray(prompt, np.int32))
    run = os.path.join(ROOT, 'trtllm-llama_amd', 'examples', 'rofozen', 'run.py')
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
