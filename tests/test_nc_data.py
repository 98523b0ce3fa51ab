"""CPU-only: the .nc data path (NetCDF-3 reader + fraction builder) behind the C ABI against the numpy oracle,
which is itself pinned by a hand-computed case.  Files are written with scipy.io.netcdf_file, the writer the
reference's own tooling uses, in both the classic and the 64-bit-offset variant.  All comparisons are exact."""
import importlib.util
import os

import numpy as np
import pytest
from scipy.io import netcdf_file

from __graft_entry__ import ROOT, load_package

_spec = importlib.util.spec_from_file_location("nc_fraction", os.path.join(ROOT, "oracle", "nc_fraction.py"))
NF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(NF)


def write_nc(path, lengths, P, Q, version, classes=0, seed=0, extra_attr=True):
    rng = np.random.default_rng(seed)
    total = int(sum(lengths))
    f = netcdf_file(path, "w", version=version)
    if extra_attr:
        f.history = "written by the test"
    f.createDimension("numSeqs", len(lengths))
    f.createDimension("numTimesteps", total)
    f.createDimension("inputPattSize", P)
    f.createDimension("maxSeqTagLength", 12)
    tags = f.createVariable("seqTags", "c", ("numSeqs", "maxSeqTagLength"))
    for i in range(len(lengths)):
        t = ("utt%03d" % i).encode().ljust(12, b"\0")
        tags[i] = np.frombuffer(t, dtype="S1")
    ln = f.createVariable("seqLengths", "i", ("numSeqs",))
    ln[:] = np.asarray(lengths, np.int32)
    x = f.createVariable("inputs", "f", ("numTimesteps", "inputPattSize"))
    x.units = "none"
    x[:] = rng.standard_normal((total, P)).astype(np.float32)
    if classes:
        f.createDimension("numLabels", classes)
        c = f.createVariable("targetClasses", "i", ("numTimesteps",))
        c[:] = rng.integers(0, classes, total).astype(np.int32)
    else:
        f.createDimension("targetPattSize", Q)
        y = f.createVariable("targetPatterns", "f", ("numTimesteps", "targetPattSize"))
        y[:] = rng.standard_normal((total, Q)).astype(np.float32)
    f.close()


def test_oracle_fraction_hand_computed(tmp_path):
    # two sequences of lengths 3 and 1, one input, one target: inputs are 10,11,12 | 20
    p = str(tmp_path / "tiny.nc")
    f = netcdf_file(p, "w")
    for name, n in (("numSeqs", 2), ("numTimesteps", 4), ("inputPattSize", 1), ("targetPattSize", 1), ("maxSeqTagLength", 2)):
        f.createDimension(name, n)
    f.createVariable("seqTags", "c", ("numSeqs", "maxSeqTagLength"))[:] = np.array([[b"a", b"\0"], [b"b", b"\0"]])
    f.createVariable("seqLengths", "i", ("numSeqs",))[:] = np.array([3, 1], np.int32)
    f.createVariable("inputs", "f", ("numTimesteps", "inputPattSize"))[:] = np.array([[10], [11], [12], [20]], np.float32)
    f.createVariable("targetPatterns", "f", ("numTimesteps", "targetPattSize"))[:] = np.array([[1], [2], [3], [4]], np.float32)
    f.close()
    segs = NF.segments(p, training_mode=True)
    assert [(s["length"], s["tag"]) for s in segs] == [(1, "b"), (3, "a")]   # sorted by ascending length
    fr = NF.make_fraction(p, segs, 0, 2)
    # slot t*S+i: i=0 is "b" (length 1), i=1 is "a" (length 3)
    assert fr["max_len"] == 3 and fr["min_len"] == 1 and fr["total_length"] == 4
    assert fr["inputs"].tolist() == [20, 10, 0, 11, 0, 12]
    assert fr["targets"].tolist() == [4, 1, 0, 2, 0, 3]
    assert fr["patTypes"].tolist() == [1, 1, 0, 2, 0, 3]     # a length-1 sequence is FIRST, not LAST
    # truncation cuts only while more than 1.5 segments remain: 3 steps at truncate 2 stay whole (3 > 3 is false),
    # at truncate 1 they become 1 + 1 + 1
    segs = NF.segments(p, truncate_seq=2, training_mode=False)
    assert [s["length"] for s in segs] == [3, 1]
    segs = NF.segments(p, truncate_seq=1, training_mode=False)
    assert [s["length"] for s in segs] == [1, 1, 1, 1] and [s["original_seq_idx"] for s in segs] == [0, 1, 2, 0]
    assert [s["begin"] for s in segs] == [0, 1, 2, 3]


@pytest.mark.parametrize("version,classes,S,trunc,frac,train", [
    (1, 0, 4, 0, 1.0, True), (2, 0, 3, 0, 1.0, False), (2, 0, 5, 7, 1.0, True), (1, 5, 2, 0, 1.0, True),
    (1, 2, 4, 0, 0.5, True), (2, 0, 1, 0, 0.01, True),
])
def test_reader_matches_oracle(tmp_path, version, classes, S, trunc, frac, train):
    capi = load_package().capi
    lengths = [17, 5, 23, 9, 31, 12, 1, 40, 8]
    P, Q = 7, 3
    p = str(tmp_path / "data.nc")
    write_nc(p, lengths, P, Q, version, classes, seed=version + classes + S)
    segs = NF.segments(p, frac, trunc, train)
    ds = capi.Dataset(p, S, train, trunc, frac)
    try:
        assert ds.num_sequences == len(segs)
        assert ds.input_size == P and ds.output_size == ((1 if classes == 2 else classes) if classes else Q)
        assert ds.is_classification == bool(classes)
        take = max(int(len(lengths) * frac), 1)
        assert ds.total_timesteps == sum(lengths[:take])
        assert ds.min_len == min(s["length"] for s in segs) and ds.max_len == max(s["length"] for s in segs)
        got = [ds.sequence(i) for i in range(ds.num_sequences)]
        assert got == [(s["length"], s["original_seq_idx"], s["tag"]) for s in segs]
        for first in range(0, len(segs), S):
            a, b = ds.fraction(first), NF.make_fraction(p, segs, first, S)
            for key in ("num_seqs", "max_len", "min_len", "total_length"):
                assert a[key] == b[key], key
            for key in ("patTypes", "inputs", "targets", "target_classes"):
                if b[key] is None:
                    assert a[key] is None
                else:
                    assert np.array_equal(a[key], b[key]), (key, first)
    finally:
        ds.close()


def test_shuffling_permutes_sequences_and_fractions(tmp_path):
    """DataSet::_shuffleSequences / _shuffleFractions (data_sets/DataSet.cpp:491-514): a sequence shuffle is a
    permutation of the segment list, a fraction shuffle a permutation of the groups of S consecutive segments (the
    short last group included, each group's inner order kept); both are repeatable for a seed, go on to another
    permutation at the next epoch, and leave the fractions' contents those of the oracle for the new order."""
    capi = load_package().capi
    lengths = [5, 9, 3, 7, 11, 4, 8, 6, 10, 2, 12]
    S = 3
    p = str(tmp_path / "shuffle.nc")
    write_nc(p, lengths, 4, 2, 1, seed=3)

    def order(ds):
        return [ds.sequence(i)[2] for i in range(ds.num_sequences)]

    ds = capi.Dataset(p, S, training_mode=True)
    base = order(ds)
    groups = [tuple(base[i:i + S]) for i in range(0, len(base), S)]
    ds.shuffle(False, True, seed=7)
    after = order(ds)
    assert sorted(after) == sorted(base) and after != base
    # cut the new order back into the old groups: walk it group by group
    seen, i = [], 0
    while i < len(after):
        g = next(g for g in groups if g[0] == after[i])
        assert tuple(after[i:i + len(g)]) == g
        seen.append(g)
        i += len(g)
    assert sorted(seen) == sorted(groups)
    # the fractions of the new order are what the oracle builds for that order
    by_tag = {s["tag"]: s for s in NF.segments(p, training_mode=True)}
    new_segs = [by_tag[t] for t in after]
    for first in range(0, ds.num_sequences, S):
        got, want = ds.fraction(first), NF.make_fraction(p, new_segs, first, S)
        for k in ("num_seqs", "max_len", "min_len", "total_length"):
            assert got[k] == want[k], (first, k)
        for k in ("patTypes", "inputs", "targets"):
            assert np.array_equal(got[k], want[k]), (first, k)
    ds.shuffle(True, False)
    again = order(ds)
    assert sorted(again) == sorted(base) and again != after
    ds.close()
    # repeatable: the same seed gives the same two epochs
    twin = capi.Dataset(p, S, training_mode=True)
    twin.shuffle(False, True, seed=7)
    assert order(twin) == after
    twin.shuffle(True, False)
    assert order(twin) == again
    twin.close()
    other = capi.Dataset(p, S, training_mode=True)
    other.shuffle(True, True, seed=8)
    assert order(other) != after and sorted(order(other)) == sorted(base)
    other.close()


def test_reader_errors(tmp_path):
    capi = load_package().capi
    with pytest.raises(RuntimeError, match="Could not open"):
        capi.Dataset(str(tmp_path / "missing.nc"), 2)
    bad = tmp_path / "bad.nc"
    bad.write_bytes(b"\x89HDF\r\n\x1a\n" + b"\0" * 64)      # a NetCDF-4 (HDF5) file is not the classic format
    with pytest.raises(RuntimeError, match="CDF magic"):
        capi.Dataset(str(bad), 2)
    p = str(tmp_path / "ok.nc")
    write_nc(p, [4, 6], 2, 2, 1)
    with pytest.raises(RuntimeError, match="Invalid fraction"):
        capi.Dataset(p, 2, fraction=0.0)
    # a file without targets of either kind
    q = str(tmp_path / "notargets.nc")
    f = netcdf_file(q, "w")
    for name, n in (("numSeqs", 1), ("numTimesteps", 2), ("inputPattSize", 1), ("maxSeqTagLength", 2)):
        f.createDimension(name, n)
    f.createVariable("seqLengths", "i", ("numSeqs",))[:] = np.array([2], np.int32)
    f.close()
    with pytest.raises(RuntimeError, match="targetPattSize"):
        capi.Dataset(q, 1)
    # an unlimited (record) dimension is refused, not misread
    r = str(tmp_path / "record.nc")
    f = netcdf_file(r, "w")
    f.createDimension("numTimesteps", None); f.createDimension("numSeqs", 1); f.createDimension("inputPattSize", 1)
    f.createDimension("targetPattSize", 1); f.createDimension("maxSeqTagLength", 2)
    f.createVariable("seqTags", "c", ("numSeqs", "maxSeqTagLength"))[:] = np.array([[b"a", b"\0"]])
    f.createVariable("seqLengths", "i", ("numSeqs",))[:] = np.array([2], np.int32)
    f.createVariable("inputs", "f", ("numTimesteps", "inputPattSize"))[0:2] = np.zeros((2, 1), np.float32)
    f.createVariable("targetPatterns", "f", ("numTimesteps", "targetPattSize"))[0:2] = np.zeros((2, 1), np.float32)
    f.close()
    ds = capi.Dataset(r, 1)
    with pytest.raises(RuntimeError, match="unlimited"):
        ds.fraction(0)
    ds.close()


def test_damaged_header_is_rejected(tmp_path):
    """A dimension a damaged header claims (here inputPattSize = 2^32 - 1, read as a negative size) is refused, and
    a file cut anywhere in its header or data is an error, never a crash."""
    capi = load_package().capi
    p = str(tmp_path / "ok.nc")
    write_nc(p, [4, 6], 3, 2, 1)
    good = open(p, "rb").read()
    at = good.index(b"inputPattSize")
    pad = (4 - len(b"inputPattSize") % 4) % 4
    q = tmp_path / "dim.nc"
    q.write_bytes(good[:at + 13 + pad] + b"\xff\xff\xff\xff" + good[at + 13 + pad + 4:])
    with pytest.raises(RuntimeError, match="out of range|dimension"):
        capi.Dataset(str(q), 2)
    for cut in range(8, len(good), 37):
        c = tmp_path / "cut.nc"
        c.write_bytes(good[:cut])
        try:
            ds = capi.Dataset(str(c), 2)
        except RuntimeError:
            continue
        try:
            ds.fraction(0)
        except RuntimeError:
            pass
        ds.close()
