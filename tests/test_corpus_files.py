"""The file readers of the input pipeline without a GPU: LMDB cursor, Datum and mean-file decoding,
and the oracle's image transform.  Files come from the small writer in lmdb_util.py and, when the
reference checkout is present, from the LMDB and mean files its own tests hold."""
import os

import numpy as np
import pytest

import lmdb_util as W
from caffecontroll_amd import CctHipError, corpus

REF = "/root/reference/tests/imagenet_train"
needs_reference = pytest.mark.skipif(not os.path.isdir(REF), reason="reference checkout not present")


def _records(n, rng, sizes):
    recs = []
    for i in range(n):
        c, h, w = sizes[i % len(sizes)]
        px = rng.integers(0, 256, c * h * w, dtype=np.uint8)
        recs.append((b"%08d_img" % i, W.datum(c, h, w, px.tobytes(), i % 1000, extra_field=(i % 3 == 0)), px, (c, h, w)))
    return recs


@pytest.mark.parametrize("n,fanout,sizes", [
    (1, None, [(3, 40, 40)]),                       # one overflow value, one leaf
    (9, None, [(1, 28, 28)]),                       # inline values (MNIST-sized), several leaves -> a branch page
    (40, 3, [(1, 5, 5), (3, 40, 40), (1, 28, 28)]),  # mixed, three tree levels
    (300, None, [(1, 6, 6)]),
])
def test_lmdb_cursor_reads_what_was_written(tmp_path, n, fanout, sizes):
    rng = np.random.default_rng(n)
    recs = _records(n, rng, sizes)
    shuffled = [recs[i] for i in rng.permutation(n)]
    W.write_lmdb(str(tmp_path / "db"), [(k, v) for k, v, _, _ in shuffled], leaf_fanout=fanout, txnid=n)
    db = corpus.Lmdb(str(tmp_path / "db"))
    assert len(db) == n
    for _ in range(2):  # a second pass after rewind gives the same sequence
        got = list(db)
        assert [k for k, _ in got] == [k for k, _, _, _ in recs]
        for (k, v), (_, want, px, (c, h, w)) in zip(got, recs):
            assert v == want
            dc, dh, dw, label, pixels, nf = corpus.parse_datum(v)
            assert (dc, dh, dw) == (c, h, w) and label == int(k[:8]) % 1000 and nf == 0
            assert np.array_equal(pixels, px)
    db.close()
    # the data file itself is accepted as the path too
    assert len(corpus.Lmdb(str(tmp_path / "db" / "data.mdb"))) == n


def test_lmdb_rejects_what_it_cannot_read(tmp_path):
    with pytest.raises(CctHipError, match="cannot open"):
        corpus.Lmdb(str(tmp_path / "absent"))
    p = tmp_path / "junk"
    p.mkdir()
    (p / "data.mdb").write_bytes(b"\0" * 10000)
    with pytest.raises(CctHipError, match="bad magic"):
        corpus.Lmdb(str(p))
    # a truncated file: the last page is missing
    path = W.write_lmdb(str(tmp_path / "t"), [(b"k", W.datum(3, 40, 40, bytes(4800), 1))])
    data = open(path, "rb").read()
    open(path, "wb").write(data[:-4096])
    with pytest.raises(CctHipError, match="shorter"):
        corpus.Lmdb(str(tmp_path / "t"))
    # empty database
    W.write_lmdb(str(tmp_path / "e"), [])
    db = corpus.Lmdb(str(tmp_path / "e"))
    assert len(db) == 0 and list(db) == []
    with pytest.raises(CctHipError, match="malformed"):
        corpus.parse_datum(b"\x22\x7f\x00")


def test_mean_file_round_trip(tmp_path):
    vals = np.arange(2 * 3 * 4, dtype=np.float32) * 0.5 - 3
    (tmp_path / "m.binaryproto").write_bytes(W.cube(1, 2, 3, 4, vals.tolist()))
    m = corpus.read_mean(str(tmp_path / "m.binaryproto"))
    assert m.shape == (1, 2, 3, 4) and np.array_equal(m.reshape(-1), vals)
    with pytest.raises(CctHipError):
        corpus.read_mean(str(tmp_path / "none"))


@needs_reference
def test_reference_lmdb_and_mean_files():
    one = list(corpus.Lmdb(REF + "/ilsvrc12_train_1_lmdb"))
    five = list(corpus.Lmdb(REF + "/ilsvrc12_train_5_lmdb"))
    assert len(one) == 1 and len(five) == 5
    keys = [k for k, _ in five]
    assert keys == sorted(keys) and all(k[:8] == b"%08d" % i for i, k in enumerate(keys))
    assert all(k.endswith(b".JPEG") and b"n01440764" in k for k in keys)   # ILSVRC class 0 (tench)
    for k, v in one + five:
        c, h, w, label, px, nf = corpus.parse_datum(v)
        assert (c, h, w, label, nf) == (3, 256, 256, 0, 0) and px.size == 3 * 256 * 256
    # the single image of the first database is the last record of the second one
    assert one[0][0].split(b"_", 1)[1] == five[4][0].split(b"_", 1)[1] and one[0][1] == five[4][1]
    # the mean file is the well-known ILSVRC12 mean image: per-channel averages (B, G, R)
    m = corpus.read_mean(REF + "/imagenet_mean.binaryproto")
    assert m.shape == (1, 3, 256, 256)
    np.testing.assert_allclose(m.mean(axis=(0, 2, 3)), [104.00699, 116.66877, 122.67892], atol=2e-4)


@pytest.mark.parametrize("crop,mirror", [(0, 0), (7, 0), (7, 1), (12, 1)])
def test_oracle_transform_against_slicing(oracle, crop, mirror):
    rng = np.random.default_rng(crop * 2 + mirror)
    b, c, h, w = 5, 3, 12, 15
    if crop > min(h, w):
        crop = min(h, w)
    raw = rng.integers(0, 256, (b, c, h, w), dtype=np.uint8)
    mean = rng.uniform(90, 130, (c, h, w)).astype(np.float32)
    params = np.stack([rng.integers(0, h - crop + 1, b), rng.integers(0, w - crop + 1, b),
                       rng.integers(0, 2, b) * mirror], axis=1).astype(np.int32)
    scale = np.float32(0.0078125)
    for mn in (mean, None):
        got = oracle.transform_batch(raw, mn, crop, params, float(scale))
        for i in range(b):
            full = raw[i].astype(np.float32) - (mn if mn is not None else np.float32(0))
            if crop:
                ho, wo, mi = params[i]
                win = full[:, ho:ho + crop, wo:wo + crop]
                want = (win[:, :, ::-1] if mi else win) * scale
            else:
                want = full * scale
            assert np.array_equal(got[i], want.astype(np.float32))
