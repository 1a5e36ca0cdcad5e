"""Pins the oracle's MoE definition (the reference has no MoE code: routing,
sort and grouped forward are defined by this build) by brute force."""
import numpy as np

Q4_K = 12


def test_route_matches_stable_argsort_and_softmax(oracle):
    logits = oracle.randn(31, (64, 128))
    logits[3, 10] = logits[3, 90] = logits[3].max() + 1.0  # an exact tie at the top
    logits[5, :] = 0.25                                     # all equal
    ids, wts = oracle.moe_route(logits, 8)
    order = np.argsort(-logits, axis=1, kind="stable")[:, :8]
    assert np.array_equal(ids, order.astype(np.int32))
    assert ids[3, 0] == 10 and ids[3, 1] == 90
    assert np.array_equal(ids[5], np.arange(8))
    p = np.exp(logits.astype(np.float64) - logits.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    sel = np.take_along_axis(p, order, axis=1)
    sel /= sel.sum(axis=1, keepdims=True)
    assert np.allclose(wts, sel, rtol=1e-5, atol=1e-7)
    assert np.allclose(wts.sum(axis=1), 1.0, atol=1e-6)


def test_sort_is_stable_counting_sort(oracle):
    rng = np.random.default_rng(5)
    for T in (1, 16, 512):
        ids = np.stack([rng.permutation(128)[:8] for _ in range(T)]).astype(np.int32)
        perm, offsets = oracle.moe_sort(ids, 128)
        flat = ids.reshape(-1)
        assert np.array_equal(perm, np.argsort(flat, kind="stable").astype(np.int32))
        counts = np.bincount(flat, minlength=128)
        assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]).astype(np.int32))
        assert sorted(perm.tolist()) == list(range(T * 8))


def test_moe_forward_against_per_pair_composition(oracle):
    E, top_k, hidden, inter, T = 8, 2, 512, 256, 5
    gate = np.concatenate([oracle.quantize(Q4_K, oracle.randn(40 + e, (inter, hidden), std=0.02)) for e in range(E)])
    up = np.concatenate([oracle.quantize(Q4_K, oracle.randn(60 + e, (inter, hidden), std=0.02)) for e in range(E)])
    down = np.concatenate([oracle.quantize(Q4_K, oracle.randn(80 + e, (hidden, inter), std=0.02)) for e in range(E)])
    x = oracle.randn(99, (T, hidden))
    ids, wts = oracle.moe_route(oracle.randn(98, (T, E)), top_k)
    out = oracle.moe_forward(Q4_K, x, ids, wts, gate, up, down, E, inter)
    gu = oracle.storage_bytes(Q4_K, inter, hidden)
    dn = oracle.storage_bytes(Q4_K, hidden, inter)
    want = np.zeros((T, hidden), np.float32)
    for t in range(T):
        for s in range(top_k):
            e = int(ids[t, s])
            g = oracle.qmatmul(Q4_K, x[t:t + 1], gate[e * gu:(e + 1) * gu], inter)
            u = oracle.qmatmul(Q4_K, x[t:t + 1], up[e * gu:(e + 1) * gu], inter)
            h = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))) * u
            y = oracle.qmatmul(Q4_K, h.astype(np.float32), down[e * dn:(e + 1) * dn], hidden)
            want[t] += wts[t, s] * y[0]
    assert np.abs(out - want).max() <= 1e-3 * np.abs(want).max()


def test_moe_forward_with_a_down_stack_of_its_own_type(oracle):
    """Q4_K gate / up with a Q6_K down stack (the mix of a Q4_K_M file): the per-pair composition of
    per-type products; with one type on both sides the mixed entry is the plain one."""
    import sys
    import os
    sys.path.insert(0, os.path.dirname(__file__))
    import np_ref
    Q6_K = 14
    E, top_k, hidden, inter, T = 4, 2, 512, 256, 3
    gate = np.concatenate([oracle.quantize(Q4_K, oracle.randn(140 + e, (inter, hidden), std=0.02)) for e in range(E)])
    up = np.concatenate([oracle.quantize(Q4_K, oracle.randn(160 + e, (inter, hidden), std=0.02)) for e in range(E)])
    down6 = np_ref.random_q6_k_blocks(7, E * hidden, inter, d_scale=2e-3)
    down4 = np.concatenate([oracle.quantize(Q4_K, oracle.randn(180 + e, (hidden, inter), std=0.02)) for e in range(E)])
    x = oracle.randn(199, (T, hidden))
    ids, wts = oracle.moe_route(oracle.randn(198, (T, E)), top_k)
    assert np.array_equal(oracle.moe_forward(Q4_K, x, ids, wts, gate, up, down4, E, inter, down_dtype=Q4_K),
                          oracle.moe_forward(Q4_K, x, ids, wts, gate, up, down4, E, inter))
    out = oracle.moe_forward(Q4_K, x, ids, wts, gate, up, down6, E, inter, down_dtype=Q6_K)
    gu = oracle.storage_bytes(Q4_K, inter, hidden)
    dn = oracle.storage_bytes(Q6_K, hidden, inter)
    want = np.zeros((T, hidden), np.float32)
    for t in range(T):
        for s in range(top_k):
            e = int(ids[t, s])
            g = oracle.qmatmul(Q4_K, x[t:t + 1], gate[e * gu:(e + 1) * gu], inter)
            u = oracle.qmatmul(Q4_K, x[t:t + 1], up[e * gu:(e + 1) * gu], inter)
            h = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))) * u
            y = oracle.qmatmul(Q6_K, h.astype(np.float32), down6[e * dn:(e + 1) * dn], hidden)
            want[t] += wts[t, s] * y[0]
    assert np.abs(out - want).max() <= 1e-3 * np.abs(want).max()
