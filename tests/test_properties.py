"""Property tests (hypothesis) of the oracle and the host-side packers over random shapes and values."""
import numpy as np
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from mxmoe_amd import pack
from oracle import mxmoe_oracle as O

F16 = np.float16
CFG = dict(max_examples=40, deadline=None)


@settings(**CFG)
@given(st.integers(1, 9), st.sampled_from([64, 128, 192, 1408]), st.sampled_from([3, 4, 8]), st.integers(0, 2**31 - 1))
def test_sym_quantiser_invariants(rows, k, bits, seed):
    x = (np.random.default_rng(seed).standard_normal((rows, k)) * 3).astype(F16)
    q, s, z = O.quant_minmax(x, bits, -1, True)
    upper = 2 ** (bits - 1) - 1
    assert np.all(np.abs(q) <= upper) and np.all(z == 0)
    amax = np.abs(x.astype(np.float64)).max(axis=1)
    hit = np.abs(q).max(axis=1)
    assert np.all((hit == upper) | (amax == 0))                      # the largest element lands on +-upper
    deq = O.dequant(q, s, z, -1).astype(np.float64)
    step = s.astype(np.float64).reshape(rows, 1)
    assert np.all(np.abs(deq - x.astype(np.float64)) <= step * 0.5 * (1 + 2e-3) + 2.0 ** -24 + np.abs(x.astype(np.float64)) * 2.0 ** -10)


@settings(**CFG)
@given(st.integers(1, 6), st.integers(1, 4), st.sampled_from([2, 3, 4]), st.integers(0, 2**31 - 1))
def test_asym_group_quantiser_invariants(rows, groups, bits, seed):
    k = 128 * groups
    x = np.random.default_rng(seed).standard_normal((rows, k)).astype(F16)
    q, s, z = O.quant_minmax(x, bits, 128, False)
    qg = q.reshape(rows, groups, 128)
    assert qg.min() >= 0 and qg.max() <= 2 ** bits - 1
    assert np.all(qg.min(axis=2) == 0) and np.all(qg.max(axis=2) == 2 ** bits - 1)   # group min -> 0, group max -> 2^b - 1
    xg = x.reshape(rows, groups, 128)
    assert np.array_equal(z.reshape(rows, groups), xg.min(axis=2))                    # float zero point = group minimum


@settings(**CFG)
@given(st.integers(1, 40), st.integers(1, 12), st.integers(1, 4), st.integers(0, 2**31 - 1))
def test_permutation_groups_every_slot_once_and_is_stable(tokens, experts, topk, seed):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, experts, size=(tokens, topk)).astype(np.int32)
    dst, perm, slot, recv = O.permute_by_expert(ids, experts)
    flat = ids.reshape(-1)
    assert sorted(slot.tolist()) == list(range(tokens * topk))
    assert np.array_equal(flat[slot], dst) and np.all(np.diff(dst) >= 0)
    assert np.array_equal(perm, slot // topk)
    assert np.array_equal(recv, np.bincount(flat, minlength=experts))
    for e in range(experts):
        s_e = slot[dst == e]
        assert np.all(np.diff(s_e) > 0)                               # stable: original order inside an expert


@settings(**CFG)
@given(st.integers(1, 5), st.integers(1, 6), st.integers(0, 2**31 - 1))
def test_packers_round_trip(nblk, kblk, seed):
    g = torch.Generator().manual_seed(seed)
    n, kb = 32 * nblk - (16 if nblk > 1 else 0), 64 * kblk           # channel counts that are not multiples of 32 too
    rows = torch.randint(0, 256, (n, kb), dtype=torch.uint8, generator=g)
    frag = pack.pack_wxax_fragments(rows)
    assert frag.numel() == -(-n // 32) * 32 * kb
    assert torch.equal(pack.unpack_wxax_fragments(frag, n, kb), rows)
    q = torch.randint(-8, 8, (n, 2 * kb), dtype=torch.int8, generator=g)
    assert torch.equal(pack.unpack_int4_k(pack.pack_int4_k(q)), q)


@settings(**CFG)
@given(st.sampled_from([64, 256, 1408, 1792, 3584]), st.integers(1, 3), st.integers(0, 2**31 - 1))
def test_online_rotation_preserves_norm_and_inverts(n, rows, seed):
    x = np.random.default_rng(seed).standard_normal((rows, n)).astype(F16)
    y = O.online_hadamard(x).astype(np.float64)
    nx, ny = np.linalg.norm(x.astype(np.float64), axis=1), np.linalg.norm(y, axis=1)
    assert np.all(np.abs(nx - ny) <= 2e-3 * nx)
    from mxmoe_amd.checkpoint import hadamard_matrix

    back = y @ hadamard_matrix(n).numpy()                              # Q^T y = x for the orthonormal Q
    assert np.abs(back - x.astype(np.float64)).max() <= 4e-3 * np.abs(x.astype(np.float64)).max() + 1e-3
