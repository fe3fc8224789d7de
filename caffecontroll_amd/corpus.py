"""ctypes view of the input pipeline (``include/cct_corpus.h``): LMDB / Datum / mean-file readers
that need no device, the batch transform kernel, and the double-buffered `Corpus` loader."""
import ctypes as C
import os

import numpy as np

from . import _lib
from ._lib import check

_P, _I, _Z = C.c_void_p, C.c_int, C.c_size_t


class TransformArgs(C.Structure):
    _fields_ = [("batch", _I), ("channels", _I), ("height", _I), ("width", _I), ("crop_size", _I),
                ("scale", C.c_float)]


class CorpusInfo(C.Structure):
    _fields_ = [("n_images", _Z), ("batch", _I), ("channels", _I), ("height", _I), ("width", _I),
                ("out_rows", _I), ("out_cols", _I)]


_PP = C.POINTER(_P)
CORPUS_PROTOTYPES = {
    "cct_hip_transform_batch": ([_P, _P, _P, _P, C.POINTER(TransformArgs)], _I),
    "cct_corpus_open": ([_PP, C.c_char_p, _I, _I, C.c_float, _I, _I, C.c_char_p, C.POINTER(C.c_float), _I,
                         C.c_uint], _I),
    "cct_corpus_create": ([_PP, _I, _I, _I, _I, _I, C.c_float, _I, _I, _P, C.c_uint], _I),
    "cct_corpus_close": ([_P], _I),
    "cct_corpus_get_info": ([_P, C.POINTER(CorpusInfo)], _I),
    "cct_corpus_set_num_classes": ([_P, _I], _I),
    "cct_corpus_load_next": ([_P, C.POINTER(_I)], _I),
    "cct_corpus_stage": ([_P, _PP, _PP, _PP], _I),
    "cct_corpus_submit": ([_P], _I),
    "cct_corpus_consume": ([_P, _P, _P, _P], _I),
    "cct_lmdb_open": ([_PP, C.c_char_p], _I),
    "cct_lmdb_close": ([_P], _I),
    "cct_lmdb_entries": ([_P], _Z),
    "cct_lmdb_rewind": ([_P], _I),
    "cct_lmdb_next": ([_P, _PP, C.POINTER(_Z), _PP, C.POINTER(_Z)], _I),
    "cct_datum_parse": ([_P, _Z, C.POINTER(_I * 4), _PP, C.POINTER(_Z), C.POINTER(_Z)], _I),
    "cct_mean_read": ([C.c_char_p, C.POINTER(_I * 4), _P, _Z, C.POINTER(_Z)], _I),
}
_bound = False


def _bind():
    global _bound
    lib = _lib.load()
    if not _bound:
        for name, (argtypes, restype) in CORPUS_PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes, fn.restype = argtypes, restype
        _bound = True
    return lib


def _ptr(x):
    if x is None:
        return None
    return x.data_ptr() if hasattr(x, "data_ptr") else x


class Lmdb:
    """Read-only cursor over an LMDB environment (MDB_FIRST / MDB_NEXT order)."""

    def __init__(self, path):
        self.lib = _bind()
        h = _P()
        check(self.lib.cct_lmdb_open(C.byref(h), os.fsencode(path)), "lmdb_open")
        self.h = h

    def __len__(self):
        return self.lib.cct_lmdb_entries(self.h)

    def rewind(self):
        check(self.lib.cct_lmdb_rewind(self.h), "lmdb_rewind")

    def __iter__(self):
        self.rewind()
        k, v, kn, vn = _P(), _P(), _Z(), _Z()
        while True:
            r = self.lib.cct_lmdb_next(self.h, C.byref(k), C.byref(kn), C.byref(v), C.byref(vn))
            if r == 0:
                return
            if r < 0:
                check(1, "lmdb_next")
            yield C.string_at(k.value, kn.value), C.string_at(v.value, vn.value)

    def close(self):
        if self.h:
            self.lib.cct_lmdb_close(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def parse_datum(value):
    """Serialized Datum -> (channels, height, width, label, uint8 array or None, float_data count)."""
    lib = _bind()
    dims, data, n, nf = (_I * 4)(), _P(), _Z(), _Z()
    buf = C.create_string_buffer(value, len(value))
    check(lib.cct_datum_parse(buf, len(value), C.byref(dims), C.byref(data), C.byref(n), C.byref(nf)), "datum_parse")
    pixels = None
    if data.value:
        pixels = np.frombuffer(C.string_at(data.value, n.value), np.uint8)
    return dims[0], dims[1], dims[2], dims[3], pixels, nf.value


def read_mean(path):
    """Binary Cube message -> float32 array shaped (num, channels, height, width) when the counts agree."""
    lib = _bind()
    dims, n = (_I * 4)(), _Z()
    check(lib.cct_mean_read(os.fsencode(path), C.byref(dims), None, 0, C.byref(n)), "mean_read")
    out = np.empty(n.value, np.float32)
    check(lib.cct_mean_read(os.fsencode(path), C.byref(dims), out.ctypes.data_as(_P), n.value, C.byref(n)), "mean_read")
    shape = tuple(int(d) for d in dims)
    return out.reshape(shape) if int(np.prod(shape)) == out.size else out


def transform_batch(dst, raw, mean, params, batch, channels, height, width, crop_size, scale):
    """Corpus::process_image for a batch on the device (device tensors or addresses)."""
    lib = _bind()
    a = TransformArgs(batch, channels, height, width, crop_size, scale)
    check(lib.cct_hip_transform_batch(_ptr(dst), _ptr(raw), _ptr(mean), _ptr(params), C.byref(a)), "transform_batch")


class Corpus:
    """Double-buffered loader: host stage (`load_next`, or `stage` + `submit`) and device stage
    (`consume`).  TRAIN phase = 0, TEST = 1."""

    def __init__(self, handle):
        self.lib, self.h = _bind(), handle
        info = CorpusInfo()
        check(self.lib.cct_corpus_get_info(self.h, C.byref(info)), "corpus_get_info")
        self.info = info

    @classmethod
    def open(cls, lmdb_dir, batch, crop_size=0, scale=1.0, mirror=False, phase=0, mean_file=None, mean_values=(),
             seed=0):
        lib = _bind()
        h = _P()
        mv = (C.c_float * len(mean_values))(*mean_values) if len(mean_values) else None
        check(lib.cct_corpus_open(C.byref(h), os.fsencode(lmdb_dir), batch, crop_size, scale, int(mirror), phase,
                                  os.fsencode(mean_file) if mean_file else None, mv, len(mean_values), seed),
              "corpus_open")
        return cls(h)

    @classmethod
    def create(cls, batch, channels, height, width, crop_size=0, scale=1.0, mirror=False, phase=0, mean=None, seed=0):
        lib = _bind()
        h = _P()
        m = None
        if mean is not None:
            m = np.ascontiguousarray(mean, np.float32)
            assert m.size == channels * height * width
        check(lib.cct_corpus_create(C.byref(h), batch, channels, height, width, crop_size, scale, int(mirror), phase,
                                    m.ctypes.data_as(_P) if m is not None else None, seed), "corpus_create")
        return cls(h)

    def set_num_classes(self, num_classes):
        """Class count of the loss layer: batches with a label outside [0, num_classes) are refused on
        the host by `load_next` / `submit` (0 switches the check off)."""
        check(self.lib.cct_corpus_set_num_classes(self.h, int(num_classes)), "corpus_set_num_classes")

    def load_next(self):
        """Next LMDB mini-batch -> staging -> asynchronous upload; returns the epoch count."""
        e = _I()
        check(self.lib.cct_corpus_load_next(self.h, C.byref(e)), "corpus_load_next")
        return e.value

    def stage(self):
        """numpy views of the next pinned staging buffer: pixels uint8 [b][c][h][w], labels float32 [b],
        params int32 [b][3] (already drawn)."""
        p, l, q = _P(), _P(), _P()
        check(self.lib.cct_corpus_stage(self.h, C.byref(p), C.byref(l), C.byref(q)), "corpus_stage")
        i = self.info
        n = i.batch * i.channels * i.height * i.width
        pixels = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_ubyte)), (n,)).reshape(i.batch, i.channels, i.height, i.width)
        labels = np.ctypeslib.as_array(C.cast(l, C.POINTER(C.c_float)), (i.batch,))
        params = np.ctypeslib.as_array(C.cast(q, C.POINTER(C.c_int)), (i.batch * 3,)).reshape(i.batch, 3)
        return pixels, labels, params

    def submit(self):
        check(self.lib.cct_corpus_submit(self.h), "corpus_submit")

    def consume(self, images_dev, labels_dev, want_params=False):
        out = np.empty((self.info.batch, 3), np.int32) if want_params else None
        check(self.lib.cct_corpus_consume(self.h, _ptr(images_dev), _ptr(labels_dev),
                                          out.ctypes.data_as(_P) if want_params else None), "corpus_consume")
        return out

    def close(self):
        if self.h:
            self.lib.cct_corpus_close(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
