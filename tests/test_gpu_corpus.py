"""GPU parity of the input pipeline: the batch transform kernel against the oracle's
process_image (bit-exact: one subtraction and one multiplication per element), and the
double-buffered loader fed from memory and from LMDB files."""
import numpy as np
import pytest

import lmdb_util as W
from gpu_util import dev, driver, empty, host

pytestmark = pytest.mark.gpu


def _params(rng, b, h, w, crop, mirror):
    return np.stack([rng.integers(0, h - crop + 1, b), rng.integers(0, w - crop + 1, b),
                     rng.integers(0, 2, b) * mirror], axis=1).astype(np.int32)


@pytest.mark.parametrize("b,c,h,w,crop,mirror,use_mean", [
    (4, 3, 16, 16, 11, 1, True),
    (3, 1, 28, 28, 0, 0, False),      # MNIST: no crop, scale only
    (5, 3, 20, 33, 0, 0, True),       # rectangular, no crop
    (7, 2, 19, 23, 19, 1, True),      # crop as high as the image
    (2, 3, 256, 256, 227, 1, True),   # the ImageNet geometry
    (300, 1, 9, 9, 5, 1, False),
])
def test_transform_kernel_matches_oracle(oracle, b, c, h, w, crop, mirror, use_mean):
    from caffecontroll_amd import corpus
    driver()
    rng = np.random.default_rng(b * 131 + crop)
    raw = rng.integers(0, 256, (b, c, h, w), dtype=np.uint8)
    mean = rng.uniform(80, 140, (c, h, w)).astype(np.float32) if use_mean else None
    params = _params(rng, b, h, w, crop, mirror)
    scale = 0.00390625 if not use_mean else 0.017
    rows, cols = (crop, crop) if crop else (h, w)
    out = empty((b, c, rows, cols))
    corpus.transform_batch(out, dev(raw), None if mean is None else dev(mean), dev(params), b, c, h, w, crop, scale)
    want = oracle.transform_batch(raw, mean, crop, params, scale)
    assert np.array_equal(host(out), want)


def test_transform_rejects_bad_geometry():
    from caffecontroll_amd import CctHipError, corpus
    driver()
    raw, out = dev(np.zeros((1, 1, 8, 8), np.uint8)), empty((1, 1, 9, 9))
    with pytest.raises(CctHipError, match="does not fit"):
        corpus.transform_batch(out, raw, None, dev(np.zeros((1, 3), np.int32)), 1, 1, 8, 8, 9, 1.0)
    with pytest.raises(CctHipError, match="params"):
        corpus.transform_batch(out, raw, None, None, 1, 1, 8, 8, 4, 1.0)


def test_memory_fed_loader_double_buffering(oracle):
    """Seven batches through the two staging slots, uploads running ahead of the transforms."""
    from caffecontroll_amd import CctHipError, corpus
    driver()
    rng = np.random.default_rng(3)
    b, c, h, w, crop = 6, 3, 24, 30, 17
    mean = rng.uniform(90, 130, (c, h, w)).astype(np.float32)
    cp = corpus.Corpus.create(b, c, h, w, crop_size=crop, scale=0.5, mirror=True, phase=0, mean=mean, seed=11)
    assert (cp.info.out_rows, cp.info.out_cols, cp.info.n_images) == (crop, crop, 0)
    images, labels = empty((b, c, crop, crop)), empty((b,))
    batches = [(rng.integers(0, 256, (b, c, h, w), dtype=np.uint8), rng.integers(0, 1000, b).astype(np.float32))
               for _ in range(7)]

    def put(i):
        px, lb, _ = cp.stage()
        px[...] = batches[i][0]
        lb[...] = batches[i][1]
        cp.submit()

    put(0)
    put(1)
    with pytest.raises(CctHipError, match="in flight"):
        cp.stage()
    seen = []
    for i in range(7):
        params = cp.consume(images, labels, want_params=True)
        if i + 2 < 7:
            put(i + 2)   # the next upload overlaps the check below
        seen.append(params.copy())
        assert params[:, 0].min() >= 0 and params[:, 0].max() < h - crop
        assert params[:, 1].min() >= 0 and params[:, 1].max() < w - crop
        assert np.array_equal(host(images), oracle.transform_batch(batches[i][0], mean, crop, params, 0.5))
        assert np.array_equal(host(labels), batches[i][1])
    with pytest.raises(CctHipError, match="no batch in flight"):
        cp.consume(images, labels)
    allp = np.concatenate(seen)
    assert 8 <= allp[:, 2].sum() <= 34 and len({tuple(r) for r in allp}) > 30   # mirror ~ half, offsets vary
    cp.close()
    # TEST phase: centre crop, never mirrored; forced parameters are honoured
    cp = corpus.Corpus.create(b, c, h, w, crop_size=crop, scale=1.0, mirror=True, phase=1, seed=1)
    px, lb, pr = cp.stage()
    assert np.array_equal(pr, np.tile(np.array([(h - crop) // 2, (w - crop) // 2, 0], np.int32), (b, 1)))
    px[...] = batches[0][0]
    lb[...] = 0
    pr[0] = (0, 0, 1)
    cp.submit()
    params = cp.consume(images, labels, want_params=True)
    assert tuple(params[0]) == (0, 0, 1)
    assert np.array_equal(host(images), oracle.transform_batch(batches[0][0], None, crop, params, 1.0))
    px, lb, pr = cp.stage()
    pr[1] = (h - crop + 1, 0, 0)   # one row too far down: refused on the host, nothing is launched
    with pytest.raises(CctHipError, match="out of range"):
        cp.submit()
    pr[1] = (h - crop, w - crop, 0)
    cp.submit()
    cp.consume(images, labels)
    cp.close()


def test_lmdb_fed_loader_wraps_around(oracle, tmp_path):
    from caffecontroll_amd import CctHipError, corpus
    driver()
    rng = np.random.default_rng(8)
    c, h, w, n, b = 3, 40, 40, 7, 3
    px = rng.integers(0, 256, (n, c, h, w), dtype=np.uint8)
    W.write_lmdb(str(tmp_path / "db"), [(b"%08d" % i, W.datum(c, h, w, px[i].tobytes(), 10 + i)) for i in range(n)],
                 leaf_fanout=2)
    mean = rng.uniform(100, 120, (c, h, w)).astype(np.float32)
    (tmp_path / "mean.bin").write_bytes(W.cube(1, c, h, w, mean.reshape(-1).tolist()))
    cp = corpus.Corpus.open(str(tmp_path / "db"), b, crop_size=33, scale=0.25, mirror=True, phase=0,
                            mean_file=str(tmp_path / "mean.bin"), seed=5)
    i_ = cp.info
    assert (i_.n_images, i_.channels, i_.height, i_.width, i_.out_rows) == (n, c, h, w, 33)
    images, labels = empty((b, c, 33, 33)), empty((b,))
    order, epochs = [], []
    epochs.append(cp.load_next())
    for it in range(6):
        epochs.append(cp.load_next())      # one batch ahead
        params = cp.consume(images, labels, want_params=True)
        idx = [(it * b + j) % n for j in range(b)]
        order += idx
        assert np.array_equal(host(labels), np.array([10 + i for i in idx], np.float32))
        assert np.array_equal(host(images), oracle.transform_batch(px[idx], mean, 33, params, 0.25))
    # 7 records, batches of 3: the third batch wraps (epoch 1), the fifth wraps again (epoch 2); the
    # seventh ends exactly on the last record, and the wrap is only counted by the read after it
    assert epochs == [0, 0, 1, 1, 2, 2, 2]
    cp.close()
    # per-channel mean values instead of a file; channels beyond the list get 0
    cp = corpus.Corpus.open(str(tmp_path / "db"), b, crop_size=0, scale=1.0, mean_values=(100.0, 110.0), phase=1)
    cp.load_next()
    full = empty((b, c, h, w))
    cp.consume(full, labels)
    mv = np.zeros((c, h, w), np.float32)
    mv[0], mv[1] = 100.0, 110.0
    assert np.array_equal(host(full), oracle.transform_batch(px[:3], mv, 0, None, 1.0))
    cp.close()
    with pytest.raises(CctHipError, match="does not fit"):
        corpus.Corpus.open(str(tmp_path / "db"), b, crop_size=41)
    # a record of another size inside the database is reported, not read out of bounds
    W.write_lmdb(str(tmp_path / "bad"), [(b"0", W.datum(c, h, w, px[0].tobytes(), 1)), (b"1", W.datum(c, 8, 8, bytes(192), 2))])
    cp = corpus.Corpus.open(str(tmp_path / "bad"), 2)
    with pytest.raises(CctHipError, match="record 1"):
        cp.load_next()
    cp.close()


def test_training_loop_fed_from_lmdb(tmp_path):
    """solver prototxt + network prototxt + LMDB -> training: the loop of `caffe-ct train`."""
    from caffecontroll_amd import corpus, prototxt as P, solver as S
    driver()
    rng = np.random.default_rng(21)
    n, c, h = 40, 1, 14
    labels = rng.integers(0, 4, n)
    px = rng.integers(0, 40, (n, c, h, h), dtype=np.uint8)
    for i, y in enumerate(labels):   # the class decides the bright quadrant
        px[i, :, (y // 2) * 7:(y // 2) * 7 + 7, (y % 2) * 7:(y % 2) * 7 + 7] += 200
    W.write_lmdb(str(tmp_path / "train_lmdb"), [(b"%08d" % i, W.datum(c, h, h, px[i].tobytes(), int(labels[i])))
                                                for i in range(n)])
    (tmp_path / "net.prototxt").write_text("""
      name: "quadrants"
      layer { name: "data" type: "Data" top: "data" top: "label" include { phase: TRAIN }
              transform_param { scale: 0.00390625 crop_size: 12 mirror: false }
              data_param { source: "train_lmdb" batch_size: 8 backend: LMDB } }
      layer { name: "conv1" type: "Convolution" bottom: "data" top: "conv1"
              convolution_param { num_output: 4 kernel_size: 3 weight_filler { type: "xavier" } } }
      layer { name: "relu1" type: "ReLU" bottom: "conv1" top: "conv1" }
      layer { name: "pool1" type: "Pooling" bottom: "conv1" top: "pool1" pooling_param { kernel_size: 2 stride: 2 } }
      layer { name: "ip1" type: "InnerProduct" bottom: "pool1" top: "ip1"
              inner_product_param { num_output: 4 weight_filler { type: "xavier" } } }
      layer { name: "loss" type: "SoftmaxWithLoss" bottom: "ip1" bottom: "label" top: "loss" }
    """)
    (tmp_path / "solver.prototxt").write_text(
        'net: "net.prototxt"\nbase_lr: 0.1 momentum: 0.9 lr_policy: "fixed" max_iter: 30 display: 10 random_seed: 3\n')
    sp, ctl, nd = P.load_solver(str(tmp_path / "solver.prototxt"), root=str(tmp_path))
    cp = corpus.Corpus.open(str(tmp_path / nd.source), nd.batch_size, crop_size=nd.crop_size, scale=nd.scale,
                            mirror=nd.mirror, phase=0, seed=1)
    net = nd.build(depth=cp.info.channels, solver=sp)
    lines = []
    reports = S.train(net, sp, ctl, cp, log=lines.append)
    assert [r[0] for r in reports] == [9, 19, 29]
    assert reports[-1][1] < 0.5 * reports[0][1] and reports[-1][2] > 0.9
    # 40 records, batches of 8: iteration 29 reads records 232..239 -> epoch 5
    assert any(l.startswith("Training Status Report (Epoch 5 / Mini-batch iter 29)") for l in lines)
    net.close()
    cp.close()
