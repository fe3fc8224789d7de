"""The training loop of `caffe-ct train` over a device-resident `nets.Net`
(DeepNet::train_network / load_and_train_network, src/DeepNet.h:2030-2215, 2386-2445), driven by
the fields of a solver prototxt (`prototxt.solver_from_prototxt`).

Mini-batches come from a `corpus.Corpus` opened on an LMDB (raw bytes uploaded asynchronously and
transformed on the device, one batch ahead of the computation) or from any iterable of
(images, labels) host arrays -- float32 [b][d][n][n] and one float label per image, what
Corpus::LoadLmdbData leaves in its two cubes (src/parser/corpus.h:111-161); the iterable is
restarted when it runs out (the reference wraps around the training set and counts an epoch).
"""
import ctypes as C
import time

import numpy as np

from . import _lib, nets
from ._lib import check

__all__ = ["train", "test", "upload_batch", "batch_accuracy", "check_labels", "learning_rate"]


def check_labels(labels, num_classes):
    """The loss layer indexes the class scores with the label (src/kernels/softmax.hxx:49-52), so a
    label outside [0, num_classes) -- or a NaN -- is refused here, on the host, before it can reach
    the device.  Returns the labels as a flat float32 array."""
    labels = np.ascontiguousarray(labels, dtype=np.float32).reshape(-1)
    ok = (labels >= 0) & (labels < num_classes)   # False for NaN
    if not ok.all():
        i = int(np.flatnonzero(~ok)[0])
        raise ValueError("label %r of image %d is outside [0, %d)" % (float(labels[i]), i, num_classes))
    return labels


def _h2d(lib, dev_ptr, arr):
    check(lib.cct_hip_memcpy(C.c_void_p(dev_ptr), arr.ctypes.data_as(C.c_void_p), arr.nbytes, 0), "memcpy h2d")


def _d2h(lib, arr, dev_ptr):
    check(lib.cct_hip_memcpy(arr.ctypes.data_as(C.c_void_p), C.c_void_p(dev_ptr), arr.nbytes, 1), "memcpy d2h")


def upload_batch(net, images, labels):
    """Host mini-batch -> the network's input cube and label cube."""
    lib = _lib.load()
    images = np.ascontiguousarray(images, dtype=np.float32)
    labels = np.ascontiguousarray(labels, dtype=np.float32).reshape(-1)
    if net.num_classes():
        labels = check_labels(labels, net.num_classes())
    if images.shape != (net.batch, net.depth, net.size, net.size):
        raise ValueError("images have shape %r, the network takes %r"
                         % (images.shape, (net.batch, net.depth, net.size, net.size)))
    if labels.shape[0] != net.batch:
        raise ValueError("%d labels for a batch of %d" % (labels.shape[0], net.batch))
    _h2d(lib, net.input_ptr(), images)
    _h2d(lib, net.labels_ptr(), labels)


def batch_accuracy(net, labels):
    """DeepNet::find_accuracy (src/DeepNet.h:82-109): images whose largest class probability sits at
    the label's index."""
    lib = _lib.load()
    ptr, n = net.tensor(len(net.layers) - 1, nets.OUTPUT)
    prob = np.empty(n, np.float32)
    _d2h(lib, prob, ptr)
    prob = prob.reshape(net.batch, -1)
    return int(np.count_nonzero(prob.argmax(axis=1) == np.asarray(labels).reshape(-1).astype(np.int64)))


class _CorpusSource:
    """Feeds the network from a `corpus.Corpus` on an LMDB: one batch is always uploading while
    the previous one trains."""

    def __init__(self, net, cp):
        if (cp.info.batch, cp.info.channels, cp.info.out_rows, cp.info.out_cols) != (net.batch, net.depth, net.size, net.size):
            raise ValueError("the corpus produces %dx%dx%dx%d batches, the network takes %dx%dx%dx%d" % (
                cp.info.batch, cp.info.channels, cp.info.out_rows, cp.info.out_cols, net.batch, net.depth, net.size, net.size))
        self.net, self.cp = net, cp
        cp.set_num_classes(net.num_classes())
        self.epoch_of_next = cp.load_next()

    def next_into_network(self):
        """Transform the batch in flight into the input cube, start loading the one after it;
        returns (epoch, labels on the host)."""
        epoch = self.epoch_of_next
        self.cp.consume(self.net.input_ptr(), self.net.labels_ptr())
        self.epoch_of_next = self.cp.load_next()
        labels = np.empty(self.net.batch, np.float32)
        _d2h(_lib.load(), labels, self.net.labels_ptr())
        return epoch, labels


def _cycle(batches):
    """Yields (epoch, images, labels) forever, restarting `batches` when it is exhausted."""
    epoch = 0
    while True:
        empty = True
        for images, labels in batches:
            empty = False
            yield epoch, images, labels
        if empty:
            raise ValueError("the batch source is empty")
        epoch += 1


def learning_rate(solver, iteration):
    """Util::get_learning_rate (src/util.h:76-93) at `iteration`, for the status line: evaluated by
    the same C++ function the updaters on the device use (`cct_solver_learning_rate`)."""
    return nets.solver_learning_rate(solver, iteration)


def test(net, batches, log=print):
    """DeepNet::test_network (src/DeepNet.h:2262-2361): forward passes only, dropout off; returns
    (mean per-image loss, accuracy) over `batches`."""
    net.set_train(False)
    total_loss, correct, n = 0.0, 0, 0
    for images, labels in batches:
        upload_batch(net, images, labels)
        net.forward()
        total_loss += net.loss() / net.batch
        correct += batch_accuracy(net, labels)
        n += 1
    net.set_train(True)
    if n == 0:
        raise ValueError("the batch source is empty")
    loss, acc = total_loss / n, correct / float(n * net.batch)
    if log:
        log("Loss = %g, Accuracy %g" % (loss, acc))
    return loss, acc


def train(net, solver, control, batches, test_batches=None, output_model_file=None, start_iter=0, log=print):
    """Runs iterations start_iter .. max_iter-1: load, forward, loss/accuracy, backward (gradients
    and SGD update of every layer).  Every `display` iterations a status report with the averages
    of that window; every `test_interval` iterations a pass over `test_batches`; every `snapshot`
    iterations the model is written (file name `snapshot_prefix` or "trained_model.bin", plus a time
    stamp, as the reference does); at the end the model goes to `output_model_file` if given.
    Returns the list of (iteration, mean loss, mean accuracy) reports."""
    display, snapshot = control.get("display", 10), control.get("snapshot", 0)
    test_interval, max_iter = control.get("test_interval", 0), control["max_iter"]
    reports, loss, acc = [], 0.0, 0.0
    window = 0
    from .corpus import Corpus
    from_corpus = isinstance(batches, Corpus)
    source = _CorpusSource(net, batches) if from_corpus else _cycle(batches)
    net.set_train(True)
    if start_iter:
        net.set_iter(start_iter)
    t0 = time.time()
    for it in range(start_iter, max_iter):
        if from_corpus:
            epoch, labels = source.next_into_network()
        else:
            epoch, images, labels = next(source)
            upload_batch(net, images, labels)
        net.forward()
        loss += net.loss() / net.batch
        acc += batch_accuracy(net, labels) / float(net.batch)
        net.backward()
        window += 1
        if display > 0 and (it + 1) % display == 0:
            reports.append((it, loss / window, acc / window))
            if log:
                log("Training Status Report (Epoch %d / Mini-batch iter %d), LR = %g" % (epoch, it, learning_rate(solver, it + 1)))
                log("  Loss & Accuracy [Average of Past %d Iterations]\t%g\t%g" % (window, loss / window, acc / window))
            loss, acc, window = 0.0, 0.0, 0
        if test_interval > 0 and test_batches is not None and (it + 1) % test_interval == 0:
            if log:
                log("Validation/Test Status Report (Epoch %d / Mini-batch iter %d)" % (epoch, it))
            test(net, test_batches, log)
        if snapshot > 0 and (it + 1) % snapshot == 0:
            name = "%s.%s" % (control.get("snapshot_prefix") or "trained_model.bin", time.strftime("%d-%m-%Y-%I-%M-%S"))
            net.write_model(name)
            if log:
                log("======= Writing snapshot %s =======" % name)
    if log:
        log("Total Time (seconds): %g" % (time.time() - t0))
    if output_model_file:
        net.write_model(output_model_file)
    return reports
