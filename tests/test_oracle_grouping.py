"""The oracle's integer grouping functions against brute-force numpy and permutation invariants."""
import numpy as np
import pytest

import oracle_lib as orc


def routes(rng, T, K, E):
    return np.stack([np.sort(rng.choice(E, K, replace=False)) for _ in range(T)]).astype(np.int32)


@pytest.mark.parametrize("T,K,E", [(1, 8, 256), (4, 8, 256), (32, 8, 128), (7, 3, 5), (64, 8, 256), (3, 1, 2)])
def test_segment_is_a_stable_counting_sort(T, K, E):
    rng = np.random.default_rng(T * 131 + K)
    ids = routes(rng, T, K, E)
    rows = np.empty(T * K + T, np.int32)
    slot_row = np.empty(T * K, np.int32)
    segs = np.empty((E + 1, 3), np.int32)
    orc.oracle().orc_moe_segment(orc.p(ids), T, K, E, orc.p(rows), orc.p(slot_row), orc.p(segs))
    flat = ids.ravel()
    order = np.argsort(flat, kind="stable")            # brute force: stable sort by expert
    assert np.array_equal(rows[:T * K], order // K)
    inv = np.empty(T * K, np.int64)
    inv[order] = np.arange(T * K)
    assert np.array_equal(slot_row, inv)
    counts = np.bincount(flat, minlength=E)
    assert np.array_equal(segs[:E, 1], counts) and np.array_equal(segs[:E, 0], np.cumsum(counts) - counts)
    assert np.array_equal(segs[:, 2], np.arange(E + 1))
    assert list(segs[E]) == [T * K, T, E] and np.array_equal(rows[T * K:], np.arange(T))
    assert np.array_equal(rows[slot_row], np.arange(T * K) // K)     # rows[slot_row[i]] == token of i


@pytest.mark.parametrize("T,K,E,early", [(1, 8, 256, 0), (4, 8, 256, 0), (8, 8, 64, 1), (5, 2, 3, 0), (5, 2, 3, 1),
                                         (30, 8, 16, 0)])
def test_slot_order_and_runs(T, K, E, early):
    rng = np.random.default_rng(T * 17 + K + early)
    ids = routes(rng, T, K, E)
    slots = T * (K + 1)
    order = np.empty(slots, np.int32)
    runs = np.empty(slots + slots // 17 + 1, np.int32)
    orc.oracle().orc_moe_slot_order(orc.p(ids), slots, K, E, early, orc.p(order), orc.p(runs))
    key = np.concatenate([ids, np.full((T, 1), E, np.int32)], axis=1).ravel()
    base = np.argsort(key, kind="stable")
    if not early:
        assert np.array_equal(order, base)
    else:
        routed, shared = base[:T * K], base[T * K:]
        want = []
        for i in range(T):
            want += [routed[i], shared[i]]
        want += list(routed[T:])
        assert np.array_equal(order, want)
    assert sorted(order) == list(range(slots))
    skey = key[order]
    p = 0
    groups = []
    while p < slots:
        q = p
        while q < slots and skey[q] == skey[p]:
            q += 1
        assert runs[p] == q - p and not runs[p + 1:q].any()
        if q - p > 16:
            groups += [(p + r0) | (min(64, q - p - r0) << 16) for r0 in range(0, q - p, 64)]
        p = q
    tail = runs[slots:]
    assert list(tail[:len(groups)]) == groups and np.all(tail[len(groups):] == -1)


def test_tile_list_and_compaction():
    rng = np.random.default_rng(9)
    E = 37
    counts = rng.integers(0, 40, E)
    counts[[3, 4, 20]] = 0
    segs = np.stack([np.cumsum(counts) - counts, counts, np.arange(E)], axis=1).astype(np.int32)
    for tile_rows in (1, 16, 64):
        tiles = np.full((E + int(counts.sum()), 2), -7, np.int32)
        n = orc.oracle().orc_moe_tile_list(orc.p(segs), E, tile_rows, orc.p(tiles))
        want = [(e, m0) for e in range(E) for m0 in range(0, counts[e], tile_rows)]
        assert n == len(want) and [tuple(t) for t in tiles[:n]] == want
        assert n <= E + (int(counts.sum()) + tile_rows - 1) // tile_rows          # the capacity bound
    for cap in (E, 30, 5):
        out = np.full((cap, 3), -1, np.int32)
        orc.oracle().orc_compact_segments(orc.p(segs), orc.p(out), E, cap)
        live = segs[counts > 0]
        k = min(cap, len(live))
        assert np.array_equal(out[:k], live[:k]) and not out[k:].any()


def test_accumulation_chains_are_fmaf_chains():
    """float32 fma emulated through float64: a*b is exact in fp64 for fp32 inputs and the sum is
    rounded once to fp32 (double rounding can differ only on exact halfway cases of the fp64 sum,
    which random data does not hit; the check also runs a deterministic exact case)."""
    rng = np.random.default_rng(2)
    T, H, K = 5, 33, 4
    contrib = rng.normal(size=(T * (K + 1), H)).astype(np.float32)
    w = rng.uniform(0, 1, (T, K)).astype(np.float32)
    out = np.empty((T, H), np.float32)
    bits = np.empty((T, H), np.uint16)
    orc.oracle().orc_slot_accum(orc.p(contrib), orc.p(w), T, H, K, 1, orc.p(out), orc.p(bits))
    for t in range(T):
        a = np.zeros(H, np.float32)
        for j in range(K):
            a = (w[t, j].astype(np.float64) * contrib[t * (K + 1) + j].astype(np.float64) + a.astype(np.float64)).astype(np.float32)
        a = (contrib[t * (K + 1) + K].astype(np.float64) + a.astype(np.float64)).astype(np.float32)
        assert np.array_equal(out[t], a)
    from dgpp_amd import hostgen as hg
    assert np.array_equal(bits, hg.f32_to_bf16(out))
    # ordered (grouped) layout visits slots in ascending expert id whatever order the router left
    ids = np.stack([rng.permutation(20)[:K] for _ in range(T)]).astype(np.int32)
    slot_row = rng.permutation(T * K).astype(np.int32)
    down = rng.normal(size=(T * K + T, H)).astype(np.float32)
    sw = rng.uniform(0, 1, T * K).astype(np.float32)
    orc.oracle().orc_accum_ordered(orc.p(down), H, orc.p(slot_row), orc.p(ids), orc.p(sw), T * K, T, K, H, orc.p(out), None)
    for t in range(T):
        a = np.zeros(H, np.float32)
        for j in np.argsort(ids[t], kind="stable"):
            s = t * K + j
            a = (sw[s].astype(np.float64) * down[slot_row[s]].astype(np.float64) + a.astype(np.float64)).astype(np.float32)
        a = (down[T * K + t].astype(np.float64) + a.astype(np.float64)).astype(np.float32)
        assert np.array_equal(out[t], a)
