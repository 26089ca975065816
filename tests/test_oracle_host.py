"""Pins the oracle's routing, permutation, offsets and tile scheduler by brute force."""
import numpy as np

from oracle import mxmoe_oracle as O


def test_route_topk_textbook():
    rng = np.random.default_rng(0)
    logits = rng.standard_normal((50, 9)).astype(np.float32)
    ids, w = O.route_topk(logits, 3)
    p = np.exp(logits.astype(np.float64)); p /= p.sum(1, keepdims=True)
    for t in range(50):
        best = sorted(range(9), key=lambda e: -p[t, e])[:3]
        assert ids[t].tolist() == best
        assert np.allclose(w[t], p[t, best] / p[t, best].sum(), rtol=1e-5)
    assert np.allclose(w.sum(1), 1, atol=1e-6)


def test_route_topk_known_answers_ties_and_library_routine():
    import torch

    # probabilities 0.1, 0.4, 0.2, 0.3 by construction: logits = ln(1, 4, 2, 3) + any constant
    logits = (np.log(np.array([[1.0, 4.0, 2.0, 3.0]])) + 5.0).astype(np.float32)
    ids, w = O.route_topk(logits, 2, renormalise=False)
    assert ids.tolist() == [[1, 3]] and np.allclose(w, [[0.4, 0.3]], rtol=1e-6)
    ids, w = O.route_topk(logits, 2, renormalise=True)
    assert ids.tolist() == [[1, 3]] and np.allclose(w, [[4 / 7, 3 / 7]], rtol=1e-6)
    ids, w = O.route_topk(logits, 4, renormalise=False)
    assert ids.tolist() == [[1, 3, 2, 0]] and np.allclose(w.sum(), 1.0, rtol=1e-6)
    # equal logits: lower expert id first
    ids, w = O.route_topk(np.array([[0.5, 2.0, 2.0, -1.0, 2.0]], np.float32), 3, renormalise=True)
    assert ids.tolist() == [[1, 2, 4]] and np.allclose(w, 1 / 3, rtol=1e-6)
    # an independent library routine on logits without ties
    rng = np.random.default_rng(5)
    x = rng.standard_normal((200, 60)).astype(np.float32) * 3
    for renorm in (False, True):
        ids, w = O.route_topk(x, 4, renormalise=renorm)
        tw, ti = torch.topk(torch.softmax(torch.from_numpy(x), dim=1, dtype=torch.float32), 4, dim=-1)
        if renorm:
            tw = tw / tw.sum(dim=-1, keepdim=True)
        assert np.array_equal(ids, ti.numpy()) and np.allclose(w, tw.numpy(), rtol=1e-5)


def test_permutation_bruteforce_and_stability():
    rng = np.random.default_rng(1)
    E, T, k = 7, 40, 3
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    ids[ids == 4] = 5                                                      # leave expert 4 empty (may duplicate 5 in a row)
    dst, perm, slot, recv = O.permute_by_expert(ids, E)
    buckets = {e: [] for e in range(E)}
    for t in range(T):
        for s in range(k):
            buckets[int(ids[t, s])].append((t, t * k + s))
    exp_perm = [t for e in range(E) for t, _ in buckets[e]]
    exp_slot = [s for e in range(E) for _, s in buckets[e]]
    assert perm.tolist() == exp_perm and slot.tolist() == exp_slot         # stable order inside an expert
    assert recv.tolist() == [len(buckets[e]) for e in range(E)] and recv[4] == 0
    assert dst.tolist() == sorted(ids.reshape(-1).tolist())


def test_act_offsets_strides_and_shared():
    recv = np.array([3, 0, 2, 5])
    qp = [(16, 4, 128, False), (8, 8, -1, True), (4, 4, -1, True), (8, 8, -1, True), (4, 4, 128, True)]
    o = O.act_offsets(recv, num_tokens=6, qparams_per_exp=qp, k_dim=256, has_shared=True)
    assert o["tag"].tolist() == [0, 1, 2, 1, 3]
    assert o["start_row"].tolist() == [0, 3, 3, 5, 10]
    assert o["inp_size"].tolist() == [3 * 256, 0, 2 * 64, 5 * 128, 6 * 64]  # K, K/2, K/4 halves per row
    assert o["scale_size"].tolist() == [0, 0, 2, 5, 6 * 2]                  # 0 / 1 / 1 / K/128
    assert o["inp_off"].tolist() == [0, 768, 768, 896, 1536]
    assert o["scale_off"].tolist() == [0, 0, 0, 2, 7]
    assert [O.act_tag(2, -1), O.act_tag(8, 128)] == [-1, -1]


def test_tile_scheduler_visits_every_tile_once():
    rng = np.random.default_rng(2)
    for _ in range(20):
        p = int(rng.integers(1, 9))
        mn = [(int(rng.integers(1, 700)), int(rng.integers(1, 6)) * 128) for _ in range(p)]
        tiles = [(int(rng.choice([16, 32, 64, 128, 256])), int(rng.choice([64, 128, 256]))) for _ in range(p)]
        prefix = O.tile_prefix(mn, tiles)
        seen = set()
        for t in range(prefix[-1]):
            pi, tm, tn = O.tile_to_problem(t, prefix, mn, tiles)
            assert 0 <= pi < p
            bm, bn = tiles[pi]
            assert tm * bm < mn[pi][0] and tn * bn < mn[pi][1]
            assert (pi, tm, tn) not in seen
            seen.add((pi, tm, tn))
        assert len(seen) == sum(-(-m // bm) * -(-n // bn) for (m, n), (bm, bn) in zip(mn, tiles))
        assert O.tile_to_problem(prefix[-1], prefix, mn, tiles)[0] == -1


# ---- un-permute + top-k weighted combine ----

def _combine_case(seed, t=7, k=3, e=5, n=16, drop=False):
    rng = np.random.default_rng(seed)
    ids = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
    _, _, slot, recv = O.permute_by_expert(ids, e)
    rows = rng.standard_normal((int(recv.sum()), n)).astype(np.float16)
    w = rng.random((t, k)).astype(np.float32)
    w /= w.sum(1, keepdims=True)
    return ids, slot, rows, w


def test_combine_one_hot_weights_return_the_routed_row():
    ids, slot, rows, w = _combine_case(0)
    t, k = w.shape
    for j in range(k):
        onehot = np.zeros_like(w)
        onehot[:, j] = 1.0
        out = O.unpermute_combine(rows, slot, onehot)
        for tok in range(t):
            r = int(np.where(slot == tok * k + j)[0][0])
            assert np.array_equal(out[tok].view(np.uint16), rows[r].view(np.uint16))


def test_combine_matches_dense_float64_and_adds_shared():
    ids, slot, rows, w = _combine_case(1, t=33, k=4, e=9, n=64)
    t, k = w.shape
    shared = np.random.default_rng(2).standard_normal((t, 64)).astype(np.float16)
    dense = np.zeros((t, 64))
    for r, s in enumerate(slot):
        dense[s // k] += float(w[s // k, s % k]) * rows[r].astype(np.float64)
    out = O.unpermute_combine(rows, slot, w)
    assert np.abs(out.astype(np.float64) - dense).max() <= 2e-3 * np.abs(dense).max()
    out_s = O.unpermute_combine(rows, slot, w, shared)
    assert np.abs(out_s.astype(np.float64) - (dense + shared.astype(np.float64))).max() <= 2e-3 * np.abs(dense + shared).max()
    # a wrong sign, a dropped shared term or a transposed weight matrix would fail the two checks above; slot order is fixed:
    flipped = O.unpermute_combine(rows, slot, w[:, ::-1].copy())
    assert not np.array_equal(flipped, out)


def test_combine_does_not_depend_on_the_order_of_the_sorted_rows():
    ids, slot, rows, w = _combine_case(3, t=12, k=2, e=4, n=8)
    p = np.random.default_rng(4).permutation(len(slot))
    assert np.array_equal(O.unpermute_combine(rows, slot, w), O.unpermute_combine(rows[p], slot[p], w))


def test_combine_skips_dropped_slots():
    ids, slot, rows, w = _combine_case(5, t=6, k=2, e=3, n=8)
    keep = slot % 2 == 0                         # pretend every second slot's expert id was out of range
    out = O.unpermute_combine(rows[keep], slot[keep], w)
    w0 = w.copy()
    w0[:, 1] = 0.0
    assert np.array_equal(out, O.unpermute_combine(rows, slot, w0))
