"""Pins the CPU oracle (NumPy and plain C) with checks that do not restate its
formulas: closed-form answers, Python-level brute force, library routines
(sorted, np.unique, torch conv3d) and structural invariants."""
import itertools

import numpy as np
import pytest
import torch

import c_oracle
import minuet_oracle as orc
from helpers import random_cloud, sorted_unique


# ---------------------------------------------------------------- offsets ----

def test_offsets_known_answers():
    k3 = orc.generate_kernel_offsets(3, 3)
    assert k3.shape == (27, 3)
    assert k3[0].tolist() == [-1, -1, -1] and k3[1].tolist() == [-1, -1, 0]
    assert k3[13].tolist() == [0, 0, 0] and k3[26].tolist() == [1, 1, 1]
    k2 = orc.generate_kernel_offsets(3, 2)
    assert k2.tolist() == [list(p) for p in itertools.product([0, 1], repeat=3)]
    k5 = orc.generate_kernel_offsets(3, 5)
    assert k5.shape == (125, 3) and k5[62].tolist() == [0, 0, 0]
    assert k5.min() == -2 and k5.max() == 2
    k2s = orc.generate_kernel_offsets(3, 2, source_stride=2)
    assert sorted(set(k2s.ravel().tolist())) == [0, 2]
    k4 = orc.generate_kernel_offsets(1, 4)
    assert k4.ravel().tolist() == [-1, 0, 1, 2]
    mixed = orc.generate_kernel_offsets(3, (3, 1, 2), source_stride=(1, 2, 4), dilation=(2, 1, 1))
    assert mixed.tolist() == [[-2, 0, 0], [-2, 0, 4], [0, 0, 0], [0, 0, 4], [2, 0, 0], [2, 0, 4]]


def test_offsets_layouts():
    mk = orc.generate_kernel_offsets(3, 3, layout="minkowski")
    assert mk[1].tolist() == [0, -1, -1][::-1] or mk[1].tolist() == [0, -1, -1]
    # minkowski enumerates dimension 0 fastest
    assert mk[0].tolist() == [-1, -1, -1] and mk[1].tolist() == [0, -1, -1]
    ts_odd = orc.generate_kernel_offsets(3, 3, layout="torchsparse")
    np.testing.assert_array_equal(ts_odd, mk)
    ts_even = orc.generate_kernel_offsets(3, 2, layout="torchsparse")
    np.testing.assert_array_equal(ts_even, orc.generate_kernel_offsets(3, 2))
    # every layout is a permutation of the same offset set
    base = {tuple(r) for r in orc.generate_kernel_offsets(3, 3).tolist()}
    assert {tuple(r) for r in mk.tolist()} == base
    with pytest.raises(NotImplementedError):
        orc.generate_kernel_offsets(3, 3, layout="other")


def test_product_offsets_match_package_helper():
    from minuet_amd.utils.helpers import generate_kernel_offsets
    for ks, ss, dl, layout in [(3, 1, 1, "minuet"), (2, 2, 1, "minuet"), ((3, 2, 5), (1, 2, 4), (1, 1, 2), "minuet"),
                               (3, 1, 1, "minkowski"), (2, 1, 1, "torchsparse"), (3, 2, 1, "torchsparse")]:
        np.testing.assert_array_equal(generate_kernel_offsets(3, ks, ss, dl, layout),
                                      orc.generate_kernel_offsets(3, ks, ss, dl, layout))


# ------------------------------------------------------------------- sort ----

@pytest.mark.parametrize("ndim", [1, 2, 3, 4])
def test_arg_sort_against_python_sorted(ndim):
    c = random_cloud(400, 5, seed=ndim, ndim=ndim, lo=-2, duplicates=0.3)
    idx = orc.arg_sort_coordinates(c)
    expect = sorted(range(len(c)), key=lambda i: tuple(c[i].tolist()))   # sorted() is stable
    assert idx.tolist() == expect


def test_arg_sort_batched_against_python_sorted():
    bd = np.array([0, 100, 100, 260, 400])
    c = random_cloud(400, 4, seed=7, lo=-2, duplicates=0.3)
    idx = orc.arg_sort_coordinates(c, bd)
    batch = np.searchsorted(bd, np.arange(400), side="right") - 1
    expect = sorted(range(400), key=lambda i: (int(batch[i]),) + tuple(c[i].tolist()))
    assert idx.tolist() == expect
    # rows never leave their batch
    for g in range(4):
        seg = idx[bd[g]:bd[g + 1]]
        assert ((seg >= bd[g]) & (seg < bd[g + 1])).all()


def test_c_arg_sort_matches():
    for seed, extent, lo in [(1, 6, -3), (2, 3000, -1500), (3, 2 ** 20, -2 ** 19)]:
        c = random_cloud(5000, extent, seed=seed, lo=lo, duplicates=0.2)
        idx, out = c_oracle.arg_sort(c)
        np.testing.assert_array_equal(idx, orc.arg_sort_coordinates(c))
        np.testing.assert_array_equal(out, c[idx])


# ----------------------------------------------------------------- unique ----

def test_unique_against_np_unique():
    c = random_cloud(3000, 5, seed=3, lo=-2)
    c = c[orc.arg_sort_coordinates(c)]
    u, idx = orc.unique_coordinates(c)
    np.testing.assert_array_equal(u, np.unique(c, axis=0))
    assert idx[0] == 0 and idx[-1] == len(u) and (np.diff(idx) >= 0).all() and (np.diff(idx) <= 1).all()
    # idx[i] is the output row of sorted row i's run
    np.testing.assert_array_equal(u[np.minimum(idx[:-1], len(u) - 1)], c)


def test_unique_batched_keeps_cross_batch_duplicates():
    bd = np.array([0, 3, 5])
    c = np.array([[0, 0, 1], [0, 0, 1], [2, 2, 2], [0, 0, 1], [2, 2, 2]], dtype=np.int32)
    u, idx = orc.unique_coordinates(c, bd)
    assert u.tolist() == [[0, 0, 1], [2, 2, 2], [0, 0, 1], [2, 2, 2]]
    assert idx.tolist() == [0, 0, 1, 2, 3, 4]
    assert idx[bd].tolist() == [0, 2, 4]


def test_target_coordinates_against_python_sets():
    bd = np.array([0, 700, 1500], dtype=np.int32)
    c, bd = sorted_unique(random_cloud(1500, 21, seed=5, lo=-10), bd)
    for stride in [(2, 2, 2), (4, 1, 3)]:
        t, tbd = orc.target_coordinates(c, bd, stride)
        rows = []
        for g in range(2):
            cells = {tuple((int(v) // s) * s for v, s in zip(p, stride)) for p in c[bd[g]:bd[g + 1]].tolist()}
            rows.append(sorted(cells))      # Python // floors, also for negatives
        assert t.tolist() == [list(p) for p in rows[0] + rows[1]]
        assert tbd.tolist() == [0, len(rows[0]), len(rows[0]) + len(rows[1])]
    assert orc.target_coordinates(np.array([[-1, -2, -3]]), None, 2)[0].tolist() == [[-2, -2, -4]]


# ------------------------------------------------------------- kernel map ----

def brute_force_map(src, tgt, off, sbd=None, tbd=None):
    sb = np.zeros(len(src), int) if sbd is None else np.searchsorted(sbd, np.arange(len(src)), side="right") - 1
    tb = np.zeros(len(tgt), int) if tbd is None else np.searchsorted(tbd, np.arange(len(tgt)), side="right") - 1
    table = {(int(b),) + tuple(p): j for j, (b, p) in enumerate(zip(sb, src.tolist()))}
    out = np.full((len(off), len(tgt)), -1, dtype=np.int64)
    for o, d in enumerate(off.tolist()):
        for t, (b, q) in enumerate(zip(tb, tgt.tolist())):
            out[o, t] = table.get((int(b),) + tuple(a + e for a, e in zip(q, d)), -1)
    return out


@pytest.mark.parametrize("kernel,stride,batched", [(3, 1, False), (2, 2, False), (5, 1, False),
                                                   (3, 1, True), (2, 2, True), ((1, 3, 2), 1, False)])
def test_query_against_dict_brute_force(kernel, stride, batched):
    bd = np.array([0, 300, 300, 800], dtype=np.int32) if batched else None
    src, sbd = sorted_unique(random_cloud(800, 9, seed=11, lo=-4), bd)
    tgt, tbd = (src, sbd) if stride == 1 else orc.target_coordinates(src, sbd, stride)
    off = orc.generate_kernel_offsets(3, kernel)
    m = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd)
    np.testing.assert_array_equal(m, brute_force_map(src, tgt, off, sbd, tbd))
    if not batched:
        np.testing.assert_array_equal(c_oracle.query(src, tgt, off), m)


def test_query_no_aliasing_at_field_edges():
    # neighbours across the bounding box must not wrap into the next row
    src = np.array([[0, 0, 0], [0, 0, 3], [0, 1, 0], [0, 3, 3], [1, 0, 0], [3, 3, 3]], dtype=np.int32)
    off = orc.generate_kernel_offsets(3, 3)
    m = orc.query_sorted_index_with_offsets(src, src, off)
    np.testing.assert_array_equal(m, brute_force_map(src, src, off))
    np.testing.assert_array_equal(c_oracle.query(src, src, off), m)


def test_submanifold_invariants():
    src, _ = sorted_unique(random_cloud(2000, 12, seed=2))
    off = orc.generate_kernel_offsets(3, 3)
    m = orc.query_sorted_index_with_offsets(src, src, off)
    sizes = orc.compute_kernel_map_sizes(m)
    assert (m[13] == np.arange(len(src))).all()                  # zero offset is the identity
    assert (sizes == sizes[::-1]).all()                           # |hits(d)| == |hits(-d)|
    for o in range(27):
        t = np.nonzero(m[o] != -1)[0]
        assert (m[26 - o][m[o][t]] == t).all()                    # M[d,t]=j <=> M[-d,j]=t
        np.testing.assert_array_equal(src[m[o][t]], src[t] + off[o])


def test_sizes_masks_lists_by_loops():
    src, _ = sorted_unique(random_cloud(500, 7, seed=9))
    tgt, _ = orc.target_coordinates(src, None, 2)
    off = orc.generate_kernel_offsets(3, 2)
    m = orc.query_sorted_index_with_offsets(src, tgt, off)
    sizes = orc.compute_kernel_map_sizes(m)
    sm, tm = orc.compute_kernel_map_masks(len(src), m)
    ins, outs, _ = orc.kernel_map_pair_lists(m)
    pos = 0
    for o in range(len(off)):
        rank = 0
        for t in range(len(tgt)):
            if m[o, t] != -1:
                assert tm[o, t] == rank and sm[o, m[o, t]] == rank
                assert ins[pos] == m[o, t] and outs[pos] == t
                rank += 1
                pos += 1
            else:
                assert tm[o, t] == -1
        assert sizes[o] == rank
        assert (sm[o] != -1).sum() == rank
    assert pos == len(ins)
    csm, ctm = c_oracle.masks(m.astype(np.int32), len(src))
    np.testing.assert_array_equal(csm, sm)
    np.testing.assert_array_equal(ctm, tm)
    cin, cout = c_oracle.pair_lists(m.astype(np.int32))
    np.testing.assert_array_equal(cin, ins)
    np.testing.assert_array_equal(cout, outs)
    np.testing.assert_array_equal(c_oracle.sizes(m.astype(np.int32)), sizes)


def test_stable_size_order():
    assert orc.stable_size_order([3, 1, 3, 0, 1]).tolist() == [3, 1, 4, 0, 2]


# ---------------------------------------------------------------- buckets ----

def test_padding_buckets_hand_cases():
    sizes = [1, 1, 1, 10]
    assert orc.generate_padding_buckets(sizes, -1) == [0, 1, 2, 3, 4]
    assert orc.generate_padding_buckets(sizes, None) == [0, 4]
    assert orc.generate_padding_buckets(sizes, 0) == [0, 3, 4]      # 27/13 > 0 stops the first bucket
    assert orc.generate_padding_buckets(sizes, 2.5) == [0, 4]       # (40-13)/13 = 2.08 <= 2.5
    # zeros merge freely; adding 5 gives (15-5)/5 = 2 > .1 -> cut; then (12-11)/11 = .09 <= .1
    assert orc.generate_padding_buckets([0, 0, 5, 6], 0.1) == [0, 2, 4]
    assert orc.generate_padding_buckets([], 0.5) == [0]


def test_padding_buckets_zero_sizes_are_merged():
    # with an empty running sum the reference's ratio is NaN and never breaks
    assert orc.generate_padding_buckets([0, 0, 0], 0.0) == [0, 3]
    assert orc.generate_padding_buckets([0, 0, 7], 0.0) == [0, 2, 3]
    assert orc.cumsum_kernel_padded_sizes([0, 0, 7], [0, 2, 3]) == [0, 0, 0, 7]


def test_padding_bucket_invariants():
    rng = np.random.default_rng(0)
    for _ in range(50):
        sizes = np.sort(rng.integers(0, 50, size=rng.integers(1, 30))).tolist()
        for thr in (-1, 0.0, 0.2, 1.0, None):
            b = orc.generate_padding_buckets(sizes, thr)
            assert b[0] == 0 and b[-1] == len(sizes) and all(x < y for x, y in zip(b, b[1:]))
            cum = orc.cumsum_kernel_padded_sizes(sizes, b)
            slots = np.diff(cum)
            assert (slots >= np.asarray(sizes)).all()
            for lo, hi in zip(b, b[1:]):
                assert len(set(slots[lo:hi].tolist())) == 1 and slots[lo] == max(sizes[lo:hi])
                if thr is not None and thr >= 0 and hi - lo > 1 and sum(sizes[lo:hi]) > 0:
                    total = sum(sizes[lo:hi])
                    assert (max(sizes[lo:hi]) * (hi - lo) - total) / total <= thr


# --------------------------------------------------------------- features ----

def densify(coords, feats, lo, shape):
    grid = torch.zeros((1, feats.shape[1]) + tuple(shape), dtype=torch.float64)
    idx = coords - lo
    grid[0, :, idx[:, 0], idx[:, 1], idx[:, 2]] = torch.from_numpy(feats).T
    return grid


def test_submanifold_conv_against_dense_conv3d():
    rng = np.random.default_rng(1)
    c, _ = sorted_unique(random_cloud(300, 6, seed=4))
    feats = rng.normal(size=(len(c), 5))
    w = rng.normal(size=(27, 5, 7))
    out, oc, _, _ = orc.conv_layer(c, None, feats, w, 3)
    dense = densify(c, feats, 0, (6, 6, 6))
    # both are cross-correlations; offsets enumerate dimension 0 slowest
    weight = torch.from_numpy(w).reshape(3, 3, 3, 5, 7).permute(4, 3, 0, 1, 2)
    ref = torch.nn.functional.conv3d(dense, weight, padding=1)[0]
    got = ref[:, c[:, 0], c[:, 1], c[:, 2]].T.numpy()
    np.testing.assert_allclose(out, got, rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(oc, c)


def test_strided_and_transposed_conv_against_dense():
    rng = np.random.default_rng(2)
    c, _ = sorted_unique(random_cloud(250, 8, seed=6))
    feats = rng.normal(size=(len(c), 4))
    w = rng.normal(size=(8, 4, 6))
    out, oc, _, stride = orc.conv_layer(c, None, feats, w, 2, stride=2)
    assert stride == (2, 2, 2)
    dense = densify(c, feats, 0, (8, 8, 8))
    weight = torch.from_numpy(w).reshape(2, 2, 2, 4, 6).permute(4, 3, 0, 1, 2)
    ref = torch.nn.functional.conv3d(dense, weight, stride=2)[0]
    got = ref[:, oc[:, 0] // 2, oc[:, 1] // 2, oc[:, 2] // 2].T.numpy()
    np.testing.assert_allclose(out, got, rtol=1e-12, atol=1e-12)
    occupied = {tuple(p) for p in ((c // 2) * 2).tolist()}
    assert {tuple(p) for p in oc.tolist()} == occupied

    wt = rng.normal(size=(8, 6, 3))
    back, bc, _, bs = orc.conv_layer(oc, None, out, wt, 2, stride=2, source_stride=2,
                                     transposed_from=(c, None, 1))
    assert bs == (1, 1, 1)
    np.testing.assert_array_equal(bc, c)
    coarse = densify(oc // 2, out, 0, (4, 4, 4))
    tweight = torch.from_numpy(wt).reshape(2, 2, 2, 6, 3).permute(3, 4, 0, 1, 2)
    tref = torch.nn.functional.conv_transpose3d(coarse, tweight, stride=2)[0]
    got = tref[:, c[:, 0], c[:, 1], c[:, 2]].T.numpy()
    np.testing.assert_allclose(back, got, rtol=1e-12, atol=1e-12)


def test_conv_special_cases():
    rng = np.random.default_rng(3)
    c, _ = sorted_unique(random_cloud(200, 6, seed=8))
    feats = rng.normal(size=(len(c), 3))
    w1 = rng.normal(size=(1, 3, 4))
    out, _, _, _ = orc.conv_layer(c, None, feats, w1, 1, bias=np.ones(4))
    np.testing.assert_allclose(out, feats @ w1[0] + 1.0)
    lone = np.array([[5, 5, 5]], dtype=np.int32)
    w = rng.normal(size=(27, 3, 2))
    out, _, _, _ = orc.conv_layer(lone, None, feats[:1], w, 3)
    np.testing.assert_allclose(out, feats[:1] @ w[13])
    ones_out, _, _, _ = orc.conv_layer(c, None, np.ones((len(c), 3)), np.ones((27, 3, 1)), 3)
    m = orc.query_sorted_index_with_offsets(c, c, orc.generate_kernel_offsets(3, 3))
    np.testing.assert_allclose(ones_out[:, 0], 3.0 * (m != -1).sum(axis=0))


def test_c_conv_forward_matches_numpy_oracle():
    rng = np.random.default_rng(4)
    c, _ = sorted_unique(random_cloud(1500, 10, seed=10))
    off = orc.generate_kernel_offsets(3, 3)
    sm, tm, order, sizes, _ = orc.build_kernel_map(c, None, c, None, off)
    f = rng.normal(size=(len(c), 8)).astype(np.float32)
    w = rng.normal(size=(27, 8, 12)).astype(np.float32)
    ref = orc.sparse_convolution_forward(f, w, sm, tm, order, sizes)
    got = c_oracle.conv_forward(f, w, sm, tm, order, sizes)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-4)


def test_generators_are_seeded_and_unique():
    from minuet_amd.synthetic import make_cloud
    a = make_cloud(1, 0.1)["coords"]
    b = make_cloud(1, 0.1)["coords"]
    np.testing.assert_array_equal(a, b)
    assert a.dtype == np.int32 and len(np.unique(a, axis=0)) == len(a) == 2000
    s = make_cloud(2, 0.02)["coords"]
    assert len(np.unique(s, axis=0)) == len(s) == 4000
    batch = make_cloud(4, 0.02)
    assert batch["batch_dims"].tolist() == [0, 2000, 4000]
    room = make_cloud(3, 0.02)["coords"]
    assert room.min() >= 0 and len(room) == 3000
