"""GPU parity of the Map step against the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

import minuet_oracle as orc
from helpers import dev, host, random_cloud, sorted_unique
import minuet_amd as minuet
from minuet_amd.nn import functional as F
from minuet_amd.nn.functional import _C

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,extent,lo,cdtype", [
    (1, 5, 0, np.int32), (2, 1, 3, np.int32), (1000, 6, -3, np.int32), (5000, 300, -150, np.int32),
    (70000, 2000, -1000, np.int32), (3000, 50, -20, np.int64),
    (4000, 2 ** 30, -2 ** 29, np.int32), (4000, 2 ** 40, -2 ** 39, np.int64),
])
def test_arg_sort_single(n, extent, lo, cdtype):
    c = random_cloud(n, extent, seed=n, lo=lo, duplicates=0.2, dtype=cdtype)
    got = F.arg_sort_coordinates(dev(c))
    assert got.dtype == torch.int32
    np.testing.assert_array_equal(host(got).astype(np.int64), orc.arg_sort_coordinates(c))


def test_arg_sort_wide_range_multi_round():
    # 4 dims of int64 spanning ~2^62 each: keys cannot be packed in 64 bits
    rng = np.random.default_rng(5)
    c = rng.integers(-2 ** 61, 2 ** 61, size=(3000, 4)).astype(np.int64)
    c[rng.integers(0, 3000, 500)] = c[rng.integers(0, 3000, 500)]
    c[:, 0] = rng.integers(-2, 2, size=3000)          # many ties on the leading dimension
    got = F.arg_sort_coordinates(dev(c))
    np.testing.assert_array_equal(host(got).astype(np.int64), orc.arg_sort_coordinates(c))


@pytest.mark.parametrize("ndim", [1, 2, 3, 4])
@pytest.mark.parametrize("idtype", [np.int32, np.int64])
def test_arg_sort_batched(ndim, idtype):
    sizes = [700, 0, 1300, 1, 999]
    bd = np.concatenate([[0], np.cumsum(sizes)]).astype(idtype)
    c = random_cloud(int(bd[-1]), 9, seed=ndim, ndim=ndim, lo=-4, duplicates=0.3)
    got = F.arg_sort_coordinates(dev(c), batch_dims=dev(bd))
    assert got.dtype == (torch.int32 if idtype == np.int32 else torch.int64)
    np.testing.assert_array_equal(host(got).astype(np.int64), orc.arg_sort_coordinates(c, bd))
    got64 = F.build_sorted_index(dev(c), batch_dims=dev(bd))
    assert got64.dtype == torch.int64


def test_arg_sort_large_two_item_paths():
    c = random_cloud(1_300_000, 1500, seed=9, lo=-700)
    got = F.arg_sort_coordinates(dev(c))
    np.testing.assert_array_equal(host(got).astype(np.int64), orc.arg_sort_coordinates(c))


def test_arg_sort_beyond_the_bucket_sort_takes_the_radix_passes():
    # more rows than the bucket sort accepts: radix passes with 16 keys per thread
    c = random_cloud(2_200_000, 1200, seed=10, lo=-600)
    got = F.arg_sort_coordinates(dev(c))
    np.testing.assert_array_equal(host(got).astype(np.int64), orc.arg_sort_coordinates(c))


def _check_arg_sort(c, bd=None):
    got = F.arg_sort_coordinates(dev(c), batch_dims=None if bd is None else dev(bd))
    np.testing.assert_array_equal(host(got).astype(np.int64), orc.arg_sort_coordinates(c, bd))


@pytest.mark.parametrize("n", [2048, 4096, 4097, 40000])
def test_arg_sort_clustered_clouds(n):
    # a dense core and two far outliers: the buckets at the core hold hundreds
    # to thousands of rows (the largest in-LDS sorts), duplicates included
    rng = np.random.default_rng(n)
    c = np.rint(rng.normal(0.0, 30.0, size=(n, 3))).astype(np.int32)
    c[:, 1:] = rng.integers(-40, 40, size=(n, 2))
    c[0] = (-2000, 0, 0)
    c[1] = (2000, 0, 0)
    c[rng.integers(2, n, n // 5)] = c[rng.integers(2, n, n // 5)]
    _check_arg_sort(c)


@pytest.mark.parametrize("distinct,extent", [(3, 2), (1, 1), (40, 5000)])
def test_arg_sort_many_copies_of_few_rows(distinct, extent):
    # thousands of equal rows: the order among them is the input order
    rng = np.random.default_rng(distinct)
    points = rng.integers(-extent, extent, size=(distinct, 3)).astype(np.int32)
    c = points[rng.integers(0, distinct, 7000)]
    c[:500] = rng.integers(-extent, extent, size=(500, 3))
    _check_arg_sort(c)


@pytest.mark.parametrize("copies", [7600, 7680, 7681])
def test_arg_sort_bucket_at_the_lds_capacity(copies):
    # one bucket right at (and just past) the largest size the in-LDS ranking
    # takes; the rows around it are spread so thinly that they share no bucket
    rng = np.random.default_rng(copies)
    c = np.empty((copies + 400, 3), dtype=np.int32)
    c[:copies] = (5, 5, 5)
    c[copies:] = rng.integers(100000, 2000000, size=(400, 3))
    c = c[rng.permutation(len(c))]
    _check_arg_sort(c)


def test_arg_sort_one_overfull_bucket_takes_the_radix_passes():
    rng = np.random.default_rng(77)
    c = rng.integers(0, 40, size=(50000, 3)).astype(np.int32)
    c[123] = (10 ** 6, 5, 5)
    _check_arg_sort(c)


@pytest.mark.parametrize("width", [29, 30])
def test_arg_sort_key_and_row_fill_one_word(width):
    # 4096 rows (12 index bits), 6 bucket bits: with 2 x 29 key bits the rest of
    # the key and the row index fill 64 bits exactly; one bit more does not fit
    rng = np.random.default_rng(width)
    c = rng.integers(0, 2 ** width, size=(4096, 2)).astype(np.int64)
    c[0] = (0, 0)
    c[1] = (2 ** width - 1, 2 ** width - 1)
    c[rng.integers(2, 4096, 300)] = c[rng.integers(2, 4096, 300)]
    _check_arg_sort(c)


def test_arg_sort_batched_many_rows():
    sizes = [9000, 0, 20000, 1, 13000]
    bd = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    c = random_cloud(int(bd[-1]), 120, seed=3, lo=-50, duplicates=0.2)
    _check_arg_sort(c, bd)


@pytest.mark.parametrize("batched", [False, True])
def test_unique(batched):
    bd = np.array([0, 2500, 2500, 6000], dtype=np.int32) if batched else None
    c = random_cloud(6000, 7, seed=3, lo=-3, duplicates=0.1)
    c = c[orc.arg_sort_coordinates(c, bd)]
    u, idx = F.unique_coordinates(dev(c), batch_dims=dev(bd))
    eu, eidx = orc.unique_coordinates(c, bd)
    np.testing.assert_array_equal(host(u), eu)
    np.testing.assert_array_equal(host(idx).astype(np.int64), eidx)
    assert idx.dtype == (torch.int32 if batched else torch.int64)


def test_unique_empty_and_single():
    u, idx = F.unique_coordinates(dev(np.zeros((0, 3), dtype=np.int32)))
    assert u.shape == (0, 3) and host(idx).tolist() == [0]
    u, idx = F.unique_coordinates(dev(np.array([[1, 2, 3]], dtype=np.int32)))
    assert host(u).tolist() == [[1, 2, 3]] and host(idx).tolist() == [0, 1]


@pytest.mark.parametrize("stride", [(2, 2, 2), (4, 2, 1), (3, 3, 3)])
@pytest.mark.parametrize("batched", [False, True])
def test_target_coordinates(stride, batched):
    bd = np.array([0, 4000, 9000], dtype=np.int32) if batched else None
    c = random_cloud(9000, 40, seed=11, lo=-20)
    c, bd = sorted_unique(c, bd)
    got, got_bd = _C.target_coordinates(dev(c), dev(bd), stride)
    exp, exp_bd = orc.target_coordinates(c, bd, stride)
    np.testing.assert_array_equal(host(got), exp)
    if batched:
        np.testing.assert_array_equal(host(got_bd), exp_bd)
    else:
        assert got_bd is None


@pytest.mark.parametrize("extent,batches", [(3, 1), (40, 5), (1 << 11, 1), (1 << 13, 3), (1 << 20, 2)])
def test_target_coordinates_bitmap_and_sorted_forms(extent, batches):
    """Key ranges up to 2^28 take the bitmap form, wider ones the sorted one;
    both must equal the oracle, with empty batches and known bounds alike."""
    rng = np.random.default_rng(extent)
    n = 6000
    c = rng.integers(-extent, extent, size=(n, 3)).astype(np.int32)
    cuts = np.sort(rng.integers(0, n, size=batches - 1)) if batches > 1 else np.zeros(0, dtype=np.int64)
    bd = np.concatenate([[0], cuts, [n]]).astype(np.int32) if batches > 1 else None
    if batches > 2:
        bd[2] = bd[1]                                  # an empty cloud in the middle
    c, bd = sorted_unique(c, bd)
    for stride in ((2, 2, 2), (4, 4, 8)):
        exp, exp_bd = orc.target_coordinates(c, bd, stride)
        for known in (None, np.concatenate([c.min(0), [0], c.max(0), [0]]).astype(np.int64)):
            got, got_bd = _C.target_coordinates(dev(c), dev(bd), stride, source_bounds=known)
            np.testing.assert_array_equal(host(got), exp)
            if bd is not None:
                np.testing.assert_array_equal(host(got_bd), exp_bd)


def _target_coordinates_two_calls(c, bd, stride):
    """mnt_target_coordinates_count + _fill through the C-ABI (the library's
    one-call form is what ``_C.target_coordinates`` takes for n > 0)."""
    import ctypes
    n, ndim = c.shape
    lib = _C.load_library()
    strides = (ctypes.c_int64 * ndim)(*stride)
    count = ctypes.c_int64(0)
    with _C._on(c.device):
        _C._check(lib.mnt_target_coordinates_count(
            _C._ptr(c), n, ndim, 0, strides, _C._ptr(bd), bd.numel() - 1 if bd is not None else 1, 0,
            None, ctypes.byref(count), _C._stream(c.device)))
        out = torch.empty((count.value, ndim), dtype=c.dtype, device=c.device)
        out_bd = torch.empty_like(bd) if bd is not None else None
        _C._check(lib.mnt_target_coordinates_fill(_C._ptr(out), _C._ptr(out_bd), _C._stream(c.device)))
    return out, out_bd


@pytest.mark.parametrize("extent,batches", [(40, 3), (1 << 20, 2)])
def test_target_coordinates_one_call_equals_two_calls(extent, batches):
    """Bitmap form (narrow key range) and sorted form (wide): the one-call entry
    point writes, into room for n rows, what count + fill write."""
    rng = np.random.default_rng(7 + extent)
    n = 5000
    c = rng.integers(-extent, extent, size=(n, 3)).astype(np.int32)
    bd = np.concatenate([[0], np.sort(rng.integers(0, n, size=batches - 1)), [n]]).astype(np.int32)
    c, bd = sorted_unique(c, bd)
    for stride in ((2, 2, 2), (1, 4, 8)):
        one, one_bd = _C.target_coordinates(dev(c), dev(bd), stride)
        assert one.untyped_storage().nbytes() == c.shape[0] * 3 * 4          # the one-call form ran
        two, two_bd = _target_coordinates_two_calls(dev(c), dev(bd), stride)
        assert torch.equal(one, two) and torch.equal(one_bd, two_bd)
        exp, exp_bd = orc.target_coordinates(c, bd, stride)
        np.testing.assert_array_equal(host(one), exp)
        np.testing.assert_array_equal(host(one_bd), exp_bd)


def test_target_coordinates_builds_in_a_row():
    """The bitmap of one build is left zero for the next (no clearing launch):
    large, small, large again, the sorted-key form in between (it writes where
    the bitmap lives), a count whose fill never comes, clustered and spread
    clouds -- every build must equal the oracle."""
    import ctypes
    rng = np.random.default_rng(91)

    def cloud(n, extent, batches):
        c = rng.integers(-extent, extent, size=(n, 3)).astype(np.int32)
        bd = None
        if batches > 1:
            bd = np.concatenate([[0], np.sort(rng.integers(0, n, size=batches - 1)), [n]]).astype(np.int32)
        return sorted_unique(c, bd)

    def dense_slab(n_side):
        g = np.stack(np.meshgrid(np.arange(n_side), np.arange(n_side), np.arange(6), indexing="ij"), -1)
        return sorted_unique(g.reshape(-1, 3).astype(np.int32), None)

    def abandoned_count(c, bd, stride):
        lib = _C.load_library()
        count = ctypes.c_int64(0)
        c_dev, bd_dev = dev(c), dev(bd)
        with _C._on(c_dev.device):
            _C._check(lib.mnt_target_coordinates_count(
                _C._ptr(c_dev), c.shape[0], 3, 0, (ctypes.c_int64 * 3)(*stride), _C._ptr(bd_dev),
                bd.size - 1 if bd is not None else 1, 0, None, ctypes.byref(count), _C._stream(c_dev.device)))
        return count.value

    builds = [cloud(30000, 300, 1), cloud(2000, 20, 3), cloud(30000, 300, 2), cloud(4000, 1 << 20, 2),
              cloud(25000, 250, 1), dense_slab(60), cloud(500, 6, 1), cloud(30000, 400, 4), dense_slab(90)]
    for round_ in range(2):
        for i, (c, bd) in enumerate(builds):
            for stride in ((2, 2, 2), (4, 4, 2)):
                if round_ == 1 and i % 3 == 0:
                    assert abandoned_count(c, bd, stride) == orc.target_coordinates(c, bd, stride)[0].shape[0]
                exp, exp_bd = orc.target_coordinates(c, bd, stride)
                if (i + round_) % 2 == 0:
                    got, got_bd = _C.target_coordinates(dev(c), dev(bd), stride)
                else:
                    got, got_bd = _target_coordinates_two_calls(dev(c), dev(bd), stride)
                np.testing.assert_array_equal(host(got), exp)
                if bd is not None:
                    np.testing.assert_array_equal(host(got_bd), exp_bd)


def test_target_coordinates_one_call_rejects_short_room():
    import ctypes
    c = dev(sorted_unique(random_cloud(300, 12, seed=3), None)[0])
    n = c.shape[0]
    room = torch.empty((n - 1, 3), dtype=torch.int32, device=c.device)
    count = ctypes.c_int64(0)
    with _C._on(c.device):
        status = _C.load_library().mnt_target_coordinates(
            _C._ptr(c), n, 3, 0, (ctypes.c_int64 * 3)(2, 2, 2), None, 1, 0, None, _C._ptr(room), n - 1,
            None, ctypes.byref(count), _C._stream(c.device))
    assert status != 0
    with pytest.raises(RuntimeError, match="capacity"):
        _C._check(status)


def _query_case(seed, n, extent, lo, kernel, stride=1, batched=False, cdtype=np.int32, idtype=np.int32):
    bd = None
    if batched:
        bd = np.array([0, n // 3, n // 3, n], dtype=idtype)
    c = random_cloud(n, extent, seed=seed, lo=lo, dtype=cdtype)
    src, sbd = sorted_unique(c, bd)
    if stride == 1:
        tgt, tbd = src, sbd
    else:
        tgt, tbd = orc.target_coordinates(src, sbd, stride)
    off = orc.generate_kernel_offsets(3, kernel, 1, 1).astype(cdtype)
    return src, sbd, tgt, tbd, off


@pytest.mark.parametrize("kernel,stride,n,extent", [
    (3, 1, 1, 4), (3, 1, 600, 7), (3, 1, 30000, 60), (2, 2, 30000, 60), (5, 1, 20000, 40),
    (3, 1, 200000, 400), ((3, 1, 2), 1, 5000, 20),
])
def test_query_single(kernel, stride, n, extent):
    src, _, tgt, _, off = _query_case(1, n, extent, -extent // 2, kernel, stride)
    got = F.query_sorted_index_with_offsets(dev(src), dev(tgt), dev(off))
    assert got.dtype == torch.int32 and got.shape == (off.shape[0], tgt.shape[0])
    np.testing.assert_array_equal(host(got), orc.query_sorted_index_with_offsets(src, tgt, off))


def test_query_dense_block_many_chunks():
    # a fully occupied block: the source window of a tile spans several LDS chunks
    g = np.stack(np.meshgrid(np.arange(6), np.arange(40), np.arange(40), indexing="ij"), -1)
    src = g.reshape(-1, 3).astype(np.int32)
    off = orc.generate_kernel_offsets(3, 5, 1, 1).astype(np.int32)
    got = F.query_sorted_index_with_offsets(dev(src), dev(src), dev(off))
    np.testing.assert_array_equal(host(got), orc.query_sorted_index_with_offsets(src, src, off))


@pytest.mark.parametrize("cdtype,idtype", [(np.int32, np.int32), (np.int32, np.int64), (np.int64, np.int32)])
@pytest.mark.parametrize("stride", [1, 2])
def test_query_batched(cdtype, idtype, stride):
    src, sbd, tgt, tbd, off = _query_case(2, 20000, 30, -15, 3 if stride == 1 else 2, stride,
                                          batched=True, cdtype=cdtype, idtype=idtype)
    got = F.query_sorted_index_with_offsets(dev(src), dev(tgt), dev(off), dev(sbd), dev(tbd))
    exp = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd)
    assert got.dtype == (torch.int32 if idtype == np.int32 else torch.int64)
    np.testing.assert_array_equal(host(got), exp)


def test_query_empty_inputs():
    src = np.zeros((0, 3), dtype=np.int32)
    tgt = random_cloud(50, 4, seed=1)
    off = orc.generate_kernel_offsets(3, 3, 1, 1).astype(np.int32)
    got = F.query_sorted_index_with_offsets(dev(src), dev(tgt), dev(off))
    assert (host(got) == -1).all()
    got = F.query_sorted_index_with_offsets(dev(tgt), dev(src), dev(off))
    assert got.shape == (27, 0)


@pytest.mark.parametrize("idtype", [np.int32, np.int64])
def test_sizes_and_masks(idtype):
    src, _, tgt, _, off = _query_case(4, 25000, 50, 0, 2, 2)
    m = orc.query_sorted_index_with_offsets(src, tgt, off, dtype=idtype)
    sizes = F.compute_kernel_map_sizes(dev(m))
    np.testing.assert_array_equal(host(sizes), orc.compute_kernel_map_sizes(m))
    sm, tm = F.compute_kernel_map_masks(src.shape[0], dev(m), sizes)
    esm, etm = orc.compute_kernel_map_masks(src.shape[0], m)
    np.testing.assert_array_equal(host(sm), esm)
    np.testing.assert_array_equal(host(tm), etm)


@pytest.mark.parametrize("reorder", [True, False])
@pytest.mark.parametrize("kernel,stride,batched", [(3, 1, False), (2, 2, True), (5, 1, False)])
def test_kernel_map_build(reorder, kernel, stride, batched):
    src, sbd, tgt, tbd, off = _query_case(7, 30000, 45, -10, kernel, stride, batched=batched)
    built = _C.kernel_map_build(dev(src), dev(tgt), off.astype(np.int64), dev(sbd), dev(tbd),
                                reorder=reorder, want_masks=True, want_lists=True, want_dense=True)
    esm, etm, eorder, esizes, em = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=reorder)
    dense = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd, dtype=np.int32)
    np.testing.assert_array_equal(host(built["kernel_map"]), dense)
    np.testing.assert_array_equal(built["sizes_host"], esizes.astype(np.int64))
    np.testing.assert_array_equal(host(built["sizes"]), esizes)
    if reorder:
        np.testing.assert_array_equal(built["order_host"], eorder.astype(np.int64))
        np.testing.assert_array_equal(host(built["order"]), eorder)
    else:
        np.testing.assert_array_equal(built["order_host"], np.arange(off.shape[0]))
    np.testing.assert_array_equal(host(built["source_masks"]), esm)
    np.testing.assert_array_equal(host(built["target_masks"]), etm)
    ein, eout, _ = orc.kernel_map_pair_lists(em)
    np.testing.assert_array_equal(host(built["in_idx"]), ein)
    np.testing.assert_array_equal(host(built["out_idx"]), eout)
    # the stand-alone list builder agrees as well
    in2, out2 = _C.kernel_map_pair_lists(dev(dense), orc.compute_kernel_map_sizes(dense))
    e2in, e2out, _ = orc.kernel_map_pair_lists(dense)
    np.testing.assert_array_equal(host(in2), e2in)
    np.testing.assert_array_equal(host(out2), e2out)


def test_voxelize_matches_numpy_unique():
    """floor(p / voxel) -> distinct voxels in lexicographic order, and the
    reverse map sends every point to its voxel (checked with np.unique)."""
    rng = np.random.default_rng(31)
    points = rng.uniform(-3.0, 3.0, size=(20000, 3)).astype(np.float32)
    size = (0.25, 0.5, 0.125)
    expect, inverse = np.unique(np.floor(points / np.asarray(size, dtype=np.float32)).astype(np.int32),
                                axis=0, return_inverse=True)
    voxels, reverse = F.voxelize(dev(points), voxel_size=size, return_reverse_indices=True)
    assert voxels.dtype == torch.int32
    np.testing.assert_array_equal(host(voxels), expect)
    np.testing.assert_array_equal(host(reverse), inverse.reshape(-1))
    np.testing.assert_array_equal(host(F.voxelize(dev(points), voxel_size=size)), expect)
    only = F.voxelize(dev(points), voxel_size=100.0, dtype=torch.int64)
    assert only.dtype == torch.int64 and only.shape[0] <= 8
    with pytest.raises(NotImplementedError):
        F.voxelize(torch.zeros(4, 3))


def test_collate_sorts_each_cloud_and_carries_features():
    clouds = [sorted_unique(random_cloud(n, 12, seed=s, lo=-6))[0] for n, s in ((700, 1), (300, 2), (1, 3))]
    rng = np.random.default_rng(5)
    shuffled, feats = [], []
    for c in clouds:
        perm = rng.permutation(c.shape[0])
        shuffled.append(dev(c[perm]))
        # a feature row that names its coordinate, so that the pairing can be checked
        feats.append(dev(c[perm].astype(np.float32) * 2.0))
    coords, bd, f = F.collate(shuffled, feats)
    sizes = [c.shape[0] for c in clouds]
    np.testing.assert_array_equal(host(bd), np.concatenate([[0], np.cumsum(sizes)]))
    np.testing.assert_array_equal(host(coords), np.concatenate(clouds))
    np.testing.assert_array_equal(host(f), np.concatenate(clouds).astype(np.float32) * 2.0)
    x = minuet.SparseTensor(f, coords, batch_dims=bd)
    assert x.batch_dims is not None and x.C.shape[0] == sum(sizes)
    coords_only, bd2 = F.collate(shuffled)
    assert torch.equal(coords_only, coords) and torch.equal(bd2, bd)
    with pytest.raises(ValueError):
        F.collate([])


@pytest.mark.parametrize("reorder", [True, False])
@pytest.mark.parametrize("kernel,stride,batched", [(3, 1, True), (2, 2, False)])
def test_dense_then_tables_equals_full_build(reorder, kernel, stride, batched):
    """The query alone, and the rank tables made from its dense map later, give
    exactly what the one-call build gives (and what the oracle gives)."""
    src, sbd, tgt, tbd, off = _query_case(17, 20000, 40, -5, kernel, stride, batched=batched)
    dense, bounds = _C.kernel_map_dense(dev(src), dev(tgt), off.astype(np.int64), dev(sbd), dev(tbd))
    expect = orc.query_sorted_index_with_offsets(src, tgt, off, sbd, tbd, dtype=np.int32)
    np.testing.assert_array_equal(host(dense), expect)
    np.testing.assert_array_equal(bounds[:3], src.min(0))
    np.testing.assert_array_equal(bounds[4:7], src.max(0))
    np.testing.assert_array_equal(bounds[8:11], tgt.min(0))
    np.testing.assert_array_equal(bounds[12:15], tgt.max(0))
    # second call with the bounds known: same map, no reduction on the device
    again, _ = _C.kernel_map_dense(dev(src), dev(tgt), off.astype(np.int64), dev(sbd), dev(tbd),
                                   source_bounds=bounds[:8], target_bounds=bounds[8:])
    assert torch.equal(again, dense)
    tables = _C.kernel_map_tables(dense, src.shape[0], reorder=reorder, want_lists=True)
    esm, etm, eorder, esizes, em = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=reorder)
    np.testing.assert_array_equal(tables["sizes_host"], esizes.astype(np.int64))
    if reorder:
        np.testing.assert_array_equal(tables["order_host"], eorder.astype(np.int64))
    np.testing.assert_array_equal(host(tables["source_masks"]), esm)
    np.testing.assert_array_equal(host(tables["target_masks"]), etm)
    ein, eout, _ = orc.kernel_map_pair_lists(em)
    np.testing.assert_array_equal(host(tables["in_idx"]), ein)
    np.testing.assert_array_equal(host(tables["out_idx"]), eout)


@pytest.mark.parametrize("reorder", [True, False])
@pytest.mark.parametrize("kernel,stride,batched", [(3, 1, True), (2, 2, False)])
def test_one_call_build_equals_two_calls(monkeypatch, reorder, kernel, stride, batched):
    """mnt_kernel_map_build (lists sized for their worst case, tables written
    while the host waits) against mnt_kernel_map_query + _emit and the oracle."""
    src, sbd, tgt, tbd, off = _query_case(23, 20000, 40, -5, kernel, stride, batched=batched)
    args = (dev(src), dev(tgt), off.astype(np.int64), dev(sbd), dev(tbd), reorder)
    kw = dict(want_masks=True, want_lists=True, want_dense=True)
    one = _C.kernel_map_build(*args, **kw)
    assert one["in_idx"].untyped_storage().nbytes() >= 8 * off.shape[0] * tgt.shape[0]   # the one-call form ran
    monkeypatch.setattr(_C, "PAIR_LIST_SLACK_BYTES", 0)
    two = _C.kernel_map_build(*args, **kw)
    assert two["in_idx"].untyped_storage().nbytes() == 8 * int(two["sizes_host"].sum())
    for key in ("sizes_host", "order_host", "bounds"):
        np.testing.assert_array_equal(one[key], two[key])
    for key in ("sizes", "order", "source_masks", "target_masks", "in_idx", "out_idx", "kernel_map"):
        assert torch.equal(one[key], two[key]), key
    esm, etm, eorder, esizes, em = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=reorder)
    ein, eout, _ = orc.kernel_map_pair_lists(em)
    np.testing.assert_array_equal(host(one["in_idx"]), ein)
    np.testing.assert_array_equal(host(one["out_idx"]), eout)
    np.testing.assert_array_equal(host(one["source_masks"]), esm)


def test_one_call_build_rejects_short_lists():
    cloud = random_cloud(500, 16, seed=5)
    off = orc.generate_kernel_offsets(3, 3, 1, 1).astype(np.int64)
    c = dev(cloud)
    dense = torch.empty((27, 500), dtype=torch.int32, device=c.device)
    lists = torch.empty((2, 100), dtype=torch.int32, device=c.device)
    sizes = np.zeros(27, dtype=np.int64)
    order = np.zeros(27, dtype=np.int64)
    lib = _C.load_library()
    with _C._on(c.device):
        status = lib.mnt_kernel_map_build(
            _C._ptr(c), 500, _C._ptr(c), 500, off.ctypes.data_as(_C._pi64), 27, 3, 0, None, None, 1, 0, 1,
            None, None, None, _C._ptr(dense), None, None, _C._ptr(lists[0]), _C._ptr(lists[1]), 100,
            None, None, sizes.ctypes.data_as(_C._pi64), order.ctypes.data_as(_C._pi64), _C._stream(c.device))
    assert status != 0
    with pytest.raises(RuntimeError, match="list_capacity"):
        _C._check(status)


def test_dense_and_tables_empty_inputs():
    off = orc.generate_kernel_offsets(3, 3, 1, 1).astype(np.int64)
    cloud = random_cloud(40, 4, seed=2)
    none = np.zeros((0, 3), dtype=np.int32)
    dense, _ = _C.kernel_map_dense(dev(none), dev(cloud), off, None, None)
    assert dense.shape == (27, 40) and (host(dense) == -1).all()
    tables = _C.kernel_map_tables(dense, 0, reorder=True)
    assert tables["sizes_host"].sum() == 0 and tables["source_masks"].shape == (27, 0)
    assert (host(tables["target_masks"]) == -1).all() and tables["in_idx"].numel() == 0
    dense, _ = _C.kernel_map_dense(dev(cloud), dev(none), off, None, None)
    assert dense.shape == (27, 0)
    tables = _C.kernel_map_tables(dense, 40, reorder=False)
    assert tables["sizes_host"].sum() == 0 and (host(tables["source_masks"]) == -1).all()
    assert _C.kernel_map_invert(dense, 40).eq(-1).all()


def _check_lists_only(src, sbd, tgt, tbd, off, reorder):
    built = _C.kernel_map_build(dev(src), dev(tgt), off.astype(np.int64), dev(sbd), dev(tbd),
                                reorder=reorder, want_masks=False, want_lists=True)
    assert built["source_masks"] is None and "kernel_map" not in built          # the lists-only form ran
    _, _, eorder, esizes, em = orc.build_kernel_map(src, sbd, tgt, tbd, off, reorder=reorder)
    np.testing.assert_array_equal(built["sizes_host"], esizes.astype(np.int64))
    np.testing.assert_array_equal(host(built["sizes"]), esizes)
    expect_order = eorder.astype(np.int64) if reorder else np.arange(off.shape[0])
    np.testing.assert_array_equal(built["order_host"], expect_order)
    np.testing.assert_array_equal(host(built["order"]), expect_order)
    ein, eout, _ = orc.kernel_map_pair_lists(em)
    np.testing.assert_array_equal(host(built["in_idx"]), ein)
    np.testing.assert_array_equal(host(built["out_idx"]), eout)
    return built


@pytest.mark.parametrize("reorder", [True, False])
@pytest.mark.parametrize("kernel,stride,batched,n,extent", [
    (3, 1, False, 30000, 45), (2, 2, True, 30000, 45), (5, 1, False, 20000, 40), (3, 1, True, 70001, 64),
    (3, 1, False, 1, 4), (3, 1, False, 513, 9), (7, 1, False, 3000, 14), ((3, 1, 2), 1, False, 5000, 20),
])
def test_kernel_map_lists_only(reorder, kernel, stride, batched, n, extent):
    """Pair lists without the dense map (mnt_kernel_map_lists): compacted staging
    in the query kernel, placing kernel, sizes and order, against the oracle."""
    src, sbd, tgt, tbd, off = _query_case(29, n, extent, -extent // 3, kernel, stride, batched=batched)
    _check_lists_only(src, sbd, tgt, tbd, off, reorder)


def test_kernel_map_lists_only_many_chunks_and_int64():
    # a fully occupied block: the source window of a tile spans several LDS chunks,
    # so those tiles stage one slot per target instead of compacting
    g = np.stack(np.meshgrid(np.arange(6), np.arange(40), np.arange(40), indexing="ij"), -1)
    src = g.reshape(-1, 3).astype(np.int32)
    off = orc.generate_kernel_offsets(3, 5, 1, 1).astype(np.int32)
    _check_lists_only(src, None, src, None, off, True)
    src64, sbd, tgt, tbd, off64 = _query_case(31, 9000, 30, -7, 3, 1, batched=True, cdtype=np.int64,
                                              idtype=np.int64)
    _check_lists_only(src64, sbd, tgt, tbd, off64, True)
    # nothing matches: every size is zero and the lists are empty
    far = src + np.array([1000, 0, 0], dtype=np.int32)
    built = _check_lists_only(src, None, far, None, orc.generate_kernel_offsets(3, 3, 1, 1).astype(np.int32), True)
    assert built["in_idx"].numel() == 0


def test_repeated_offsets_fill_their_own_rows():
    """An offset table that names the same offset several times: every copy
    gets its own row of the map, sizes and lists (the reference resolves each
    row of the table on its own, query_sorted_index_with_offsets.cuh:36-77);
    seven copies of one offset overfill a group of the query's plan."""
    src, _, _, _, base = _query_case(37, 30000, 45, -10, 3)
    off = np.concatenate([base[:5], np.repeat(base[13:14], 7, axis=0), base[20:], base[4:6]]).astype(np.int32)
    dense = orc.query_sorted_index_with_offsets(src, src, off, dtype=np.int32)
    got = F.query_sorted_index_with_offsets(dev(src), dev(src), dev(off))
    np.testing.assert_array_equal(host(got), dense)
    for reorder in (True, False):
        _check_lists_only(src, None, src, None, off, reorder)
    cloud = src[np.random.default_rng(2).permutation(src.shape[0])]
    _check_sorted_lists(cloud, off.astype(np.int64))


def _wide_cloud(ndim, span_bits, dtype, clusters=60, per_cluster=60, seed=23):
    """Clusters of neighbouring voxels scattered over a range of 2^span_bits per
    dimension: neighbours exist, and a packed key of the frame would need
    ndim * span_bits bits."""
    rng = np.random.default_rng(seed)
    half = 1 << (span_bits - 1)
    centres = rng.integers(-half, half, size=(clusters, ndim))
    centres[0], centres[1] = -half, half - 4                    # the corners of the range
    rows = (centres[:, None, :] + rng.integers(0, 4, size=(clusters, per_cluster, ndim))).reshape(-1, ndim)
    return rows.astype(dtype)


def _brute_force_map(src, sbd, tgt, tbd, off):
    """Dict look-up of every shifted target, batch by batch."""
    nb = 1 if sbd is None else len(sbd) - 1
    sb = [0, src.shape[0]] if sbd is None else [int(v) for v in sbd]
    tb = [0, tgt.shape[0]] if tbd is None else [int(v) for v in tbd]
    out = np.full((off.shape[0], tgt.shape[0]), -1, dtype=np.int64)
    for b in range(nb):
        where = {tuple(int(v) for v in src[j]): j for j in range(sb[b], sb[b + 1])}
        for t in range(tb[b], tb[b + 1]):
            row = [int(v) for v in tgt[t]]
            for o in range(off.shape[0]):
                out[o, t] = where.get(tuple(c + int(d) for c, d in zip(row, off[o])), -1)
    return out


@pytest.mark.parametrize("ndim,span_bits,cdtype,batched", [
    (4, 40, np.int64, False), (4, 40, np.int64, True), (3, 30, np.int64, False),
    (4, 20, np.int32, False), (3, 31, np.int32, True), (4, 62, np.int64, False),
])
def test_query_on_frames_wider_than_a_packed_key(ndim, span_bits, cdtype, batched):
    """Coordinate ranges whose packed key would need more than 63 bits: the
    reference compares whole tuples (csrc/minuet/common/functions.h:94-105), so
    any range works there; here such frames take the tuple-comparing query.
    Dense map, sizes, rank tables, pair lists and the one-call Map step."""
    cloud = _wide_cloud(ndim, span_bits, cdtype)
    bd = np.array([0, cloud.shape[0] // 3, cloud.shape[0]], dtype=np.int32) if batched else None
    src, sbd = sorted_unique(cloud, bd)
    kernel = 3 if ndim == 3 else 2
    off = orc.generate_kernel_offsets(ndim, kernel, 1, 1).astype(cdtype)
    expect = _brute_force_map(src, sbd, src, sbd, off)
    assert (expect >= 0).sum() > 2 * src.shape[0]                 # neighbours were found
    np.testing.assert_array_equal(orc.query_sorted_index_with_offsets(src, src, off, sbd, sbd), expect)
    got = F.query_sorted_index_with_offsets(dev(src), dev(src), dev(off), dev(sbd), dev(sbd))
    np.testing.assert_array_equal(host(got), expect)
    for reorder in (True, False):
        built = _C.kernel_map_build(dev(src), dev(src), off.astype(np.int64), dev(sbd), dev(sbd),
                                    reorder=reorder, want_masks=True, want_lists=True, want_dense=True)
        esm, etm, eorder, esizes, em = orc.build_kernel_map(src, sbd, src, sbd, off, reorder=reorder)
        np.testing.assert_array_equal(host(built["kernel_map"]), expect)
        np.testing.assert_array_equal(built["sizes_host"], esizes.astype(np.int64))
        np.testing.assert_array_equal(host(built["source_masks"]), esm)
        np.testing.assert_array_equal(host(built["target_masks"]), etm)
        ein, eout, _ = orc.kernel_map_pair_lists(em)
        np.testing.assert_array_equal(host(built["in_idx"]), ein)
        np.testing.assert_array_equal(host(built["out_idx"]), eout)
        _check_lists_only(src, sbd, src, sbd, off, reorder)
    if not batched:
        shuffled = src[np.random.default_rng(1).permutation(src.shape[0])]
        _check_sorted_lists(shuffled, off.astype(np.int64))
        # ... and through a layer's cache
        cache = minuet.nn.KernelMapCache(ndim=ndim, dtype=torch.int32, device="cuda")
        dense = cache.get_dense_kernel_map(dev(src), 1, None, dev(src), 1, None, kernel, 1)
        np.testing.assert_array_equal(host(dense), expect)


def _check_sorted_lists(cloud, off, reorder=True):
    """mnt_sorted_kernel_map_lists against the oracle's sort and kernel map."""
    indices, sorted_dev, built = _C.sorted_kernel_map_lists(dev(cloud), off.astype(np.int64), reorder=reorder)
    order = orc.arg_sort_coordinates(cloud)
    ref = cloud[order]
    assert indices.dtype == torch.int32
    np.testing.assert_array_equal(host(indices).astype(np.int64), order)
    np.testing.assert_array_equal(host(sorted_dev), ref)
    np.testing.assert_array_equal(built["bounds"][:cloud.shape[1]], cloud.min(0))
    np.testing.assert_array_equal(built["bounds"][4:4 + cloud.shape[1]], cloud.max(0))
    _, _, eorder, esizes, em = orc.build_kernel_map(ref, None, ref, None, off.astype(cloud.dtype), reorder=reorder)
    np.testing.assert_array_equal(built["sizes_host"], esizes.astype(np.int64))
    np.testing.assert_array_equal(host(built["sizes"]), esizes)
    expect_order = eorder.astype(np.int64) if reorder else np.arange(off.shape[0])
    np.testing.assert_array_equal(built["order_host"], expect_order)
    np.testing.assert_array_equal(host(built["order"]), expect_order)
    ein, eout, _ = orc.kernel_map_pair_lists(em)
    np.testing.assert_array_equal(host(built["in_idx"]), ein)
    np.testing.assert_array_equal(host(built["out_idx"]), eout)
    # the result object alone: the same tensors, made when asked for
    alone = _C.sorted_kernel_map_lists(dev(cloud), off.astype(np.int64), reorder=reorder, result_only=True)
    for key in ("indices", "coordinates", "in_idx", "out_idx", "sizes", "order"):
        assert key in alone
        np.testing.assert_array_equal(host(alone[key]), host(indices if key == "indices" else
                                                             sorted_dev if key == "coordinates" else built[key]))
    np.testing.assert_array_equal(alone["sizes_host"], built["sizes_host"])
    np.testing.assert_array_equal(alone["order_host"], built["order_host"])


@pytest.mark.parametrize("reorder", [True, False])
@pytest.mark.parametrize("n,extent,kernel,cdtype", [
    (30000, 45, 3, np.int32), (2048, 20, 3, np.int32), (70001, 64, 2, np.int32), (50000, 300, 3, np.int64),
    (9000, 30, 4, np.int32), (40000, 50, (3, 1, 2), np.int32),
    # below the chain's smallest cloud and beyond its 64 offsets: the two separate calls inside
    (600, 9, 3, np.int32), (20000, 40, 5, np.int32),
])
def test_sorted_kernel_map_lists(reorder, n, extent, kernel, cdtype):
    cloud = np.unique(random_cloud(n, extent, seed=41, lo=-extent // 3, dtype=cdtype), axis=0)
    cloud = cloud[np.random.default_rng(5).permutation(cloud.shape[0])]
    off = orc.generate_kernel_offsets(3, kernel, 1, 1)
    _check_sorted_lists(cloud, off, reorder)


def test_sorted_kernel_map_lists_lidar_and_clustered():
    from minuet_amd.synthetic import make_cloud
    off = orc.generate_kernel_offsets(3, 3, 1, 1)
    # the generator of configuration 2 at a quarter of its size: planes of constant x make large buckets
    _check_sorted_lists(make_cloud(2, scale=0.25)["coords"], off)
    # one dense slab: a bucket far beyond what the chain ranks in LDS, so the chain declines on the device
    g = np.stack(np.meshgrid(np.arange(2), np.arange(120), np.arange(120), indexing="ij"), -1).reshape(-1, 3)
    far = np.array([[4000, 0, 0], [-4000, 5, 5]])
    cloud = np.concatenate([g, far]).astype(np.int32)
    cloud = cloud[np.random.default_rng(9).permutation(cloud.shape[0])]
    _check_sorted_lists(cloud, off)
    # rows that repeat (the sort is stable; the map is that of the rows as they are)
    dup = random_cloud(5000, 12, seed=3, duplicates=0.3)
    indices, sorted_dev, _ = _C.sorted_kernel_map_lists(dev(dup), off.astype(np.int64))
    order = orc.arg_sort_coordinates(dup)
    np.testing.assert_array_equal(host(indices).astype(np.int64), order)
    np.testing.assert_array_equal(host(sorted_dev), dup[order])


def test_sorted_kernel_map_lists_empty_cloud():
    off = orc.generate_kernel_offsets(3, 3, 1, 1).astype(np.int64)
    empty = np.zeros((0, 3), dtype=np.int32)
    indices, sorted_dev, built = _C.sorted_kernel_map_lists(dev(empty), off)
    assert indices.numel() == 0 and tuple(sorted_dev.shape) == (0, 3)
    assert built["in_idx"].numel() == 0 and int(np.asarray(built["sizes_host"]).sum()) == 0
    alone = _C.sorted_kernel_map_lists(dev(empty), off, result_only=True)
    assert alone["indices"].numel() == 0 and tuple(alone["coordinates"].shape) == (0, 3)
    assert alone["out_idx"].numel() == 0


def test_sorted_kernel_map_lists_2d_and_4d():
    rng = np.random.default_rng(11)
    for ndim, extent in ((2, 300), (4, 12)):
        cloud = np.unique(rng.integers(-5, extent, size=(20000, ndim)).astype(np.int32), axis=0)
        cloud = cloud[rng.permutation(cloud.shape[0])]
        off = orc.generate_kernel_offsets(ndim, 3 if ndim == 2 else 2, 1, 1)
        _check_sorted_lists(cloud, off)


@pytest.mark.parametrize("idtype", [np.int32, np.int64])
def test_target_coordinates_one_cloud_with_boundaries(idtype):
    """A single cloud that still carries batch_dims = [0, n] gets [0, count]
    back, as the reference's tensor expression gives (convolutions.py:92-96)."""
    c, _ = sorted_unique(random_cloud(6000, 30, seed=19, lo=-9))
    bd = np.array([0, c.shape[0]], dtype=idtype)
    got, got_bd = _C.target_coordinates(dev(c), dev(bd), (2, 2, 2))
    exp, _ = orc.target_coordinates(c, None, (2, 2, 2))
    np.testing.assert_array_equal(host(got), exp)
    assert got_bd.dtype == (torch.int32 if idtype == np.int32 else torch.int64)
    np.testing.assert_array_equal(host(got_bd), [0, exp.shape[0]])
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    coords, stride, dims = cache.get_target_coordinates(dev(c), dev(bd), 1, 2)
    np.testing.assert_array_equal(host(coords), exp)
    np.testing.assert_array_equal(host(dims), [0, exp.shape[0]])


def test_cache_bounds_survive_recycled_storage():
    """Bounds remembered for a temporary (the contiguous copy of a strided
    coordinate view) must not be picked up by a later tensor that lands on the
    recycled address: the cache keeps what it files bounds under alive."""
    cache = minuet.nn.KernelMapCache(ndim=3, dtype=torch.int32, device="cuda")
    a, _ = sorted_unique(random_cloud(4000, 20, seed=3, lo=0))
    wide = torch.zeros((a.shape[0], 6), dtype=torch.int32, device="cuda")
    wide[:, ::2] = dev(a)
    view = wide[:, ::2]                                    # not contiguous: the cache works on a copy
    assert not view.is_contiguous()
    dense_a = cache.get_dense_kernel_map(view, 1, None, view, 1, None, 3, 1)
    np.testing.assert_array_equal(host(dense_a), orc.query_sorted_index_with_offsets(
        a, a, orc.generate_kernel_offsets(3, 3, 1, 1)))
    # same row count, far larger coordinates, allocated right after the temporary went away
    b = a[: a.shape[0]].copy()
    b[:, 0] += 5000
    b_dev = dev(b)
    dense_b = cache.get_dense_kernel_map(b_dev, 2, None, b_dev, 2, None, 3, 1)
    np.testing.assert_array_equal(host(dense_b), orc.query_sorted_index_with_offsets(
        b, b, orc.generate_kernel_offsets(3, 3, 2, 1)))


def test_sorted_kernel_map_lists_wide_planes():
    """Planes of constant first coordinate with tens of thousands of rows: the
    one-call Map step's shortcut for a tile's source window (from the sort's
    bucket starts) would span more than one window chunk there, so the tiles
    fall back to their searches; and a cloud that is a single such plane."""
    rng = np.random.default_rng(23)
    off = orc.generate_kernel_offsets(3, 3, 1, 1)
    for planes, side, n in ((12, 220, 150000), (1, 300, 60000)):
        flat = rng.choice(planes * side * side, size=n, replace=False)
        cloud = np.stack([flat // (side * side) - 3, (flat // side) % side, flat % side - 100], 1).astype(np.int32)
        _check_sorted_lists(cloud, off)
