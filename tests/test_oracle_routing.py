"""Pins the oracle's integer routing functions against closed forms, library routines and brute force.

Reference semantics under test: select_experts.cu:417-468 (slot walk and tie rule), :480-488 (softmax),
:535-580 (exclusive scan); build_expert_mapping.cu:18-103 (counting-sort scatter, inclusive post-state).
"""
import numpy as np
import pytest

import oracle_lib as O
from util import f32_to_bf16, bf16_to_f32, bf16_to_f64


def run_select(oracle, logits_f32, K):
    logits = f32_to_bf16(np.asarray(logits_f32, dtype=np.float32))
    return (logits,) + O.select_experts(oracle, logits, K)


def test_all_equal_logits_choose_first_k_in_order(oracle):
    # no later expert is STRICTLY greater than the running minimum, so the first K stay, in slot order
    for E, K in [(8, 2), (64, 8), (5, 5), (17, 3)]:
        _, w, chosen, counts, cumsum, host = run_select(oracle, np.full((3, E), 0.5), K)
        assert (chosen == np.arange(K, dtype=np.uint16)[None, :]).all()
        np.testing.assert_allclose(w, 1.0 / K, rtol=1e-6)
        assert counts[:K].tolist() == [3] * K and counts[K:E].sum() == 0 and counts[E] == 1


def test_strictly_increasing_logits_rotate_through_slots(oracle):
    # every expert beats the minimum; expert e lands in the slot of the current minimum, which cycles 0,1,..,K-1
    E, K = 16, 4
    _, w, chosen, *_ = run_select(oracle, np.arange(E, dtype=np.float32)[None, :] / 8.0, K)
    expect = np.zeros(K, dtype=np.uint16)
    for e in range(E):
        expect[e % K] = e
    assert chosen[0].tolist() == expect.tolist()
    assert set(chosen[0].tolist()) == set(range(E - K, E))


def test_strictly_decreasing_logits_keep_first_k(oracle):
    E, K = 12, 3
    _, _, chosen, *_ = run_select(oracle, -np.arange(E, dtype=np.float32)[None, :], K)
    assert chosen[0].tolist() == [0, 1, 2]


def test_ties_straddling_the_kth_value_prefer_lower_index(oracle):
    # values: two clear winners (idx 5, 2), then four experts tied for the last two places (idx 0,3,4,7)
    row = np.array([1.0, -3.0, 7.0, 1.0, 1.0, 9.0, -2.0, 1.0], dtype=np.float32)
    _, _, chosen, *_ = run_select(oracle, row[None, :], 4)
    assert set(chosen[0].tolist()) == {5, 2, 0, 3}
    # slot order by hand: 0,1,2,3 fill slots 0..3 (1,-3,7,1); e=4 (1.0): min is -3 at slot 1 -> slot1=4;
    # e=5 (9): min value 1.0 held by experts 0,3,4 -> evict the LARGEST id (4, slot 1) -> slot1=5;
    # e=6 (-2) no; e=7 (1.0): not strictly greater than min 1.0 -> no.
    assert chosen[0].tolist() == [0, 5, 2, 3]


def brute_force_set(row_f32, K):
    order = sorted(range(len(row_f32)), key=lambda e: (-float(row_f32[e]), e))
    return set(order[:K])


@pytest.mark.parametrize("E,K,seed", [(8, 2, 0), (32, 4, 1), (64, 8, 2), (7, 3, 3), (130, 6, 4), (64, 1, 5)])
def test_selected_set_is_topk_by_value_then_index(oracle, E, K, seed):
    rng = np.random.default_rng(seed)
    # coarse values -> many exact bf16 ties
    vals = np.round(rng.standard_normal((200, E)) * 4) / 4
    logits, w, chosen, counts, cumsum, host = run_select(oracle, vals, K)
    lf = bf16_to_f32(logits)
    for t in range(lf.shape[0]):
        assert set(chosen[t].tolist()) == brute_force_set(lf[t], K)
        assert len(set(chosen[t].tolist())) == K
    # counts / scan against numpy library routines
    bc = np.bincount(chosen.ravel(), minlength=E)
    assert (counts[:E] == bc).all() and (host == bc).all()
    assert (cumsum == np.concatenate([[0], np.cumsum(bc)[:-1]])).all()
    assert counts[:E].sum() == 200 * K


def test_slot_order_matches_an_independent_replay(oracle):
    # independent restatement with python tuples: worst slot = min by (value, -expert id)
    rng = np.random.default_rng(11)
    E, K = 24, 5
    vals = np.round(rng.standard_normal((100, E)) * 2) / 2
    logits, _, chosen, *_ = run_select(oracle, vals, K)
    lf = bf16_to_f32(logits)
    for t in range(lf.shape[0]):
        slots = [(-np.inf, 0xFFFF)] * K
        worst = 0
        worst_val = -np.inf
        for e in range(E):
            if lf[t, e] > worst_val:
                slots[worst] = (float(lf[t, e]), e)
                worst = min(range(K), key=lambda k: (slots[k][0], -slots[k][1]))
                worst_val = slots[worst][0]
        assert [s[1] for s in slots] == chosen[t].tolist()


def test_weights_are_softmax_over_selected_logits(oracle):
    rng = np.random.default_rng(5)
    E, K = 64, 8
    logits, w, chosen, *_ = run_select(oracle, rng.standard_normal((300, E)), K)
    lf = bf16_to_f64(logits)
    sel = np.take_along_axis(lf, chosen.astype(np.int64), axis=1)
    ref = np.exp(sel - sel.max(axis=1, keepdims=True))
    ref /= ref.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(w.sum(axis=1), 1.0, atol=1e-6)
    # the kernel rounds (v - max) to bf16 before exp: each exponent moves by at most 2^-9 * |v - max| relative,
    # and the normalising sum by at most the largest such move
    bound = 2.0 ** -9 * np.abs(sel - sel.max(axis=1, keepdims=True)).max(axis=1, keepdims=True)
    assert (np.abs(w - ref) / ref <= 2 * bound + 1e-5).all()


def test_softmax_difference_is_rounded_to_bf16(oracle):
    # 1.0 and 1.00390625*... choose values whose difference is not a bf16 number
    a, b = 3.0, 0.0078125 * 3  # both bf16-exact; a-b = 2.9765625 needs 8 mantissa bits -> rounds in bf16
    logits, w, chosen, *_ = run_select(oracle, np.array([[a, b]], dtype=np.float32), 2)
    d = bf16_to_f32(f32_to_bf16(np.array([b - a], dtype=np.float32)))[0]
    exact = np.exp(np.float64(b - a))
    rounded = np.exp(np.float64(d))
    assert d != np.float32(b - a)
    got_ratio = w[0, 1] / w[0, 0]
    assert abs(got_ratio - rounded) < abs(got_ratio - exact)


@pytest.mark.parametrize("T,E,K,seed", [(64, 8, 2, 0), (257, 32, 4, 1), (1000, 64, 8, 2), (5, 4, 4, 3), (1, 3, 1, 4)])
def test_build_expert_mapping_is_stable_counting_sort(oracle, T, E, K, seed):
    rng = np.random.default_rng(seed)
    chosen = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint16)
    bc = np.bincount(chosen.ravel(), minlength=E)
    excl = np.concatenate([[0], np.cumsum(bc)[:-1]]).astype(np.int32)
    emap, tmap, cumsum_after = O.build_expert_mapping(oracle, chosen, E, excl)
    # library routine: stable argsort of the flattened ids
    order = np.argsort(chosen.ravel(), kind="stable")
    assert (emap == (order // K)).all()
    inv = np.empty(T * K, dtype=np.int64)
    inv[order] = np.arange(T * K)
    assert (tmap.ravel() == inv).all()
    # invariants: bijection, segment membership, inclusive post-state
    assert sorted(tmap.ravel().tolist()) == list(range(T * K))
    assert (emap[tmap] == np.arange(T)[:, None]).all()
    seg = np.searchsorted(np.cumsum(bc), tmap.ravel(), side="right")
    assert (seg == chosen.ravel()).all()
    assert (cumsum_after == np.cumsum(bc)).all()


def test_empty_token_batch(oracle):
    logits = np.zeros((0, 8), dtype=np.uint16)
    w, chosen, counts, cumsum, host = O.select_experts(oracle, logits, 2)
    assert counts[:8].sum() == 0 and counts[8] == 1 and (cumsum == 0).all()


# ---- fp32 logits (select_experts.cu:3-295) ----

@pytest.mark.parametrize("E,K,seed", [(8, 2, 0), (64, 8, 2), (7, 3, 3), (130, 6, 4)])
def test_fp32_selection_set_slot_order_counts_and_unrounded_softmax(oracle, E, K, seed):
    rng = np.random.default_rng(seed)
    # half the rows coarse (many exact ties), half with full fp32 mantissas (values no bf16 could tell apart)
    vals = np.concatenate([np.round(rng.standard_normal((100, E)) * 4) / 4,
                           1.0 + rng.integers(0, 50, (100, E)) * 2.0 ** -20]).astype(np.float32)
    w, chosen, counts, cumsum, host = O.select_experts_fp32(oracle, vals, K)
    for t in range(vals.shape[0]):
        assert set(chosen[t].tolist()) == brute_force_set(vals[t], K)
        # independent replay of the slot walk: worst slot = min by (value, -expert id)
        slots, worst, worst_val = [(-np.inf, 0xFFFF)] * K, 0, -np.inf
        for e in range(E):
            if vals[t, e] > worst_val:
                slots[worst] = (float(vals[t, e]), e)
                worst = min(range(K), key=lambda k: (slots[k][0], -slots[k][1]))
                worst_val = slots[worst][0]
        assert [s_[1] for s_ in slots] == chosen[t].tolist()
    bc = np.bincount(chosen.ravel(), minlength=E)
    assert (counts[:E] == bc).all() and (host == bc).all() and counts[E] == 1
    assert (cumsum == np.concatenate([[0], np.cumsum(bc)[:-1]])).all()
    # softmax over the selected logits with the difference in fp32, not rounded to bf16: fp64 agrees to fp32 accuracy
    sel = np.take_along_axis(vals.astype(np.float64), chosen.astype(np.int64), axis=1)
    ref = np.exp(sel - sel.max(axis=1, keepdims=True))
    ref /= ref.sum(axis=1, keepdims=True)
    np.testing.assert_allclose(w, ref, rtol=3e-6)


def test_fp32_softmax_keeps_a_difference_bf16_would_round(oracle):
    a, b = 3.0, 0.0234375                              # a - b needs more mantissa bits than bf16 has
    w, *_ = O.select_experts_fp32(oracle, np.array([[a, b]], dtype=np.float32), 2)
    exact = np.exp(np.float64(b - a))
    rounded = np.exp(np.float64(bf16_to_f32(f32_to_bf16(np.array([b - a], dtype=np.float32)))[0]))
    ratio = w[0, 1] / w[0, 0]
    assert abs(ratio - exact) < abs(ratio - rounded)

