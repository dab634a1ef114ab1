"""Pins the CPU partition oracle: against the 16 golden .block4 files the
reference ships, against brute force, and its two formulations and the C
restatement against each other."""
import numpy as np
import pytest

import block4_codec
from oracle import c_oracle, partition_oracle as po


def test_slice_tables_known_answers():
    # values read off the golden files (every degree 1..384 occurs in them)
    w, r = po.slice_tables()
    for d, wn in {1: 1, 32: 32, 33: 17, 64: 32, 65: 22, 96: 32, 97: 25, 128: 32, 129: 22, 191: 32,
                  192: 32, 300: 32, 384: 32}.items():
        assert w[d] == wn, d
    for d, rows in {1: 12, 32: 12, 33: 6, 64: 6, 65: 4, 96: 4, 97: 3, 128: 3, 129: 2, 191: 2,
                    192: 1, 384: 1}.items():
        assert r[d] == rows, d
    # a block never exceeds 384 non-zeros or 12 slices
    d = np.arange(1, 385)
    assert np.all(r[1:] * d <= 384)
    assert np.all(r[1:] * -(-d // w[1:]) <= 12)


def test_golden_manifest_complete():
    assert len(block4_codec.names()) == 16
    for n in block4_codec.names():
        b = block4_codec.load(n)       # load() verifies the recorded SHA-256
        assert b.shape[1] == 4 and b.shape[0] == block4_codec.manifest()[n]["blocks"]


@pytest.mark.parametrize("name", block4_codec.names())
def test_closed_form_reproduces_golden(name):
    golden = block4_codec.load(name)
    indptr = po.indptr_from_degrees(po.degrees_from_block4(golden))
    assert po.block4_to_bytes(po.partition_closed_form(indptr)) == golden.tobytes()


@pytest.mark.parametrize("name", block4_codec.names())
def test_c_walk_reproduces_golden(name):
    golden = block4_codec.load(name)
    indptr = po.indptr_from_degrees(po.degrees_from_block4(golden))
    assert np.array_equal(c_oracle.partition_walk(indptr), golden)


@pytest.mark.parametrize("name", ["pubmed", "artist", "arxiv"])
def test_python_walk_reproduces_golden(name):
    golden = block4_codec.load(name)
    indptr = po.indptr_from_degrees(po.degrees_from_block4(golden))
    assert np.array_equal(po.partition_walk(indptr), golden)


def test_golden_covers_every_regime():
    degs = np.concatenate([po.degrees_from_block4(block4_codec.load(n)) for n in block4_codec.names()])
    u = np.unique(degs)
    assert set(range(0, 385)) <= set(u.tolist())
    assert (u > 384).sum() >= 1500
    for m in (768, 1152, 5376):            # exact multiples of 384: no empty tail segment
        assert m in u


def brute_force_blocks(deg):
    """Independent of the oracle's code: expand the rule literally."""
    out, loc, r, n = [], 0, 0, len(deg)
    while r < n:
        d = int(deg[r])
        if d == 0:
            r += 1
        elif d <= 384:
            split = 1 if d <= 32 else 2 if d <= 64 else 3 if d <= 96 else 4 if d <= 128 else 6 if d <= 191 else None
            cap, w = (12 // split, -(-d // split)) if split else (1, 32)
            j = r
            while j < n and j - r < cap and deg[j] == d:
                j += 1
            out.append((d, r, loc, (w << 16) + (j - r)))
            loc += (j - r) * d
            r = j
        else:
            left = d
            while left > 0:
                seg = min(384, left)
                out.append((d, r, loc, seg))
                loc += seg
                left -= seg
            r += 1
    return np.asarray(out, dtype=np.int32).reshape(-1, 4)


@pytest.mark.parametrize("seed", range(8))
def test_formulations_agree_on_unsorted_input(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 400))
    deg = rng.choice([0, 0, 1, 1, 2, 5, 32, 33, 64, 96, 97, 129, 191, 192, 384, 385, 768, 1000], size=n)
    # runs of equal degree, also zero-degree rows in the middle and at the end
    deg = np.repeat(deg, rng.integers(1, 20, size=n))
    indptr = po.indptr_from_degrees(deg)
    expect = brute_force_blocks(deg)
    assert np.array_equal(po.partition_walk(indptr), expect)
    assert np.array_equal(po.partition_closed_form(indptr), expect)
    assert np.array_equal(c_oracle.partition_walk(indptr), expect)


def test_edge_cases():
    for deg in ([], [0], [0, 0, 0], [1], [384], [385], [768], [0, 5, 0], [3] * 13, [40] * 7):
        indptr = po.indptr_from_degrees(np.asarray(deg, dtype=np.int64))
        e = brute_force_blocks(deg)
        assert np.array_equal(po.partition_closed_form(indptr), e), deg
        assert np.array_equal(po.partition_walk(indptr), e), deg
        assert np.array_equal(c_oracle.partition_walk(indptr), e), deg
    b = po.partition_walk(po.indptr_from_degrees([768]))
    assert b.tolist() == [[768, 0, 0, 384], [768, 0, 384, 384]]
    b = po.partition_walk(po.indptr_from_degrees([3] * 13))
    assert b.tolist() == [[3, 0, 0, (3 << 16) + 12], [3, 12, 36, (3 << 16) + 1]]


def test_blocks_tile_the_nonzeros():
    deg = np.sort(np.random.default_rng(3).integers(0, 900, size=3000))
    b = po.partition_closed_form(po.indptr_from_degrees(deg))
    row, n_rows, row_nz, loc, is_long = po.decode_block4(b)
    sizes = n_rows * row_nz
    assert np.all(sizes <= 384) and np.all(sizes > 0)
    assert loc[0] == 0 and np.array_equal(loc[1:], np.cumsum(sizes)[:-1])
    assert int(sizes.sum()) == int(deg.sum())
    assert np.array_equal(po.degrees_from_block4(b, deg.size), deg)


@pytest.mark.parametrize("seed", range(4))
def test_degree_sort_is_stable_ascending(seed):
    rng = np.random.default_rng(seed)
    deg = rng.integers(0, 50, size=2000)
    indptr = po.indptr_from_degrees(deg)
    perm = po.degree_sort(indptr)
    assert np.array_equal(np.sort(perm), np.arange(deg.size))
    sd = deg[perm]
    assert np.all(np.diff(sd) >= 0)
    same = sd[1:] == sd[:-1]
    assert np.all(perm[1:][same] > perm[:-1][same])       # ties keep original order
    assert np.array_equal(c_oracle.degree_sort(indptr), perm)


def test_permute_csr_moves_whole_rows():
    rng = np.random.default_rng(0)
    deg = rng.integers(0, 9, size=50)
    indptr = po.indptr_from_degrees(deg)
    idx = rng.integers(0, 100, size=int(indptr[-1])).astype(np.int32)
    val = rng.random(idx.size).astype(np.float32)
    perm = po.degree_sort(indptr)
    sip, six, sval = po.permute_csr(indptr, idx, val, perm)
    for new, old in enumerate(perm):
        assert np.array_equal(six[sip[new]:sip[new + 1]], idx[indptr[old]:indptr[old + 1]])
        assert np.array_equal(sval[sip[new]:sip[new + 1]], val[indptr[old]:indptr[old + 1]])


def test_group_long_rows_is_a_stable_partition():
    rng = np.random.default_rng(1)
    deg = np.array([5, 400, 384, 1000, 0, 385])
    indptr = po.indptr_from_degrees(deg)
    idx = rng.integers(0, 5000, size=int(indptr[-1])).astype(np.int32)
    val = rng.random(idx.size).astype(np.float32)
    gi, gv = po.group_long_rows(indptr, idx, val)
    for r, d in enumerate(deg):
        a, b = indptr[r], indptr[r + 1]
        if d <= 384:
            assert np.array_equal(gi[a:b], idx[a:b]) and np.array_equal(gv[a:b], val[a:b])
            continue
        grp = po.column_group(gi[a:b])
        assert np.all(np.diff(grp) >= 0)                          # grouped
        for g in range(8):                                        # original order inside a group
            assert np.array_equal(gi[a:b][grp == g], idx[a:b][po.column_group(idx[a:b]) == g])
        assert sorted(zip(gi[a:b].tolist(), gv[a:b].tolist())) == sorted(zip(idx[a:b].tolist(), val[a:b].tolist()))
    assert po.column_group(np.array([0, 7, 8, 15, 16, 63, 64])).tolist() == [0, 0, 1, 1, 2, 7, 0]
