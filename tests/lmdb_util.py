"""Writes small LMDB data files and Datum / Cube messages for the tests, following LMDB's on-disk
layout (data format version 1) and the protobuf wire format.  Test data only: the product reads
such files, it never writes them."""
import os
import struct

PSIZE = 4096
HDR = 16
NODEMAX = (((PSIZE - HDR) // 2) & ~1) - 2
P_BRANCH, P_LEAF, P_OVERFLOW, P_META = 1, 2, 4, 8
F_BIGDATA = 1


def _varint(v):
    out = bytearray()
    v &= (1 << 64) - 1
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def datum(channels, height, width, pixels, label, extra_field=False):
    """Serialized Datum with `bytes data`; extra_field appends an unknown field a parser must skip."""
    body = b"\x08" + _varint(channels) + b"\x10" + _varint(height) + b"\x18" + _varint(width)
    body += b"\x22" + _varint(len(pixels)) + bytes(pixels) + b"\x28" + _varint(label)
    if extra_field:
        body += b"\x38\x01"  # field 7 (encoded), varint
    return body


def cube(num, channels, height, width, floats):
    data = struct.pack("<%df" % len(floats), *floats)
    return (b"\x08" + _varint(num) + b"\x10" + _varint(channels) + b"\x18" + _varint(height) + b"\x20" +
            _varint(width) + b"\x2a" + _varint(len(data)) + data)


def _page(pgno, flags, nodes):
    """nodes: list of serialized nodes in key order -> one page."""
    buf = bytearray(PSIZE)
    upper = PSIZE
    ptrs = []
    for n in nodes:
        size = (len(n) + 1) & ~1
        upper -= size
        buf[upper:upper + len(n)] = n
        ptrs.append(upper)
    lower = HDR + 2 * len(nodes)
    assert lower <= upper, "page overflow"
    struct.pack_into("<QHHHH", buf, 0, pgno, 0, flags, lower, upper)
    for i, p in enumerate(ptrs):
        struct.pack_into("<H", buf, HDR + 2 * i, p)
    return bytes(buf)


def _leaf_node(key, value, overflow_pgno=None):
    if overflow_pgno is None:
        return struct.pack("<HHHH", len(value) & 0xFFFF, len(value) >> 16, 0, len(key)) + key + value
    return struct.pack("<HHHH", len(value) & 0xFFFF, len(value) >> 16, F_BIGDATA, len(key)) + key + \
        struct.pack("<Q", overflow_pgno)


def _branch_node(key, child):
    return struct.pack("<HHHH", child & 0xFFFF, (child >> 16) & 0xFFFF, child >> 32, len(key)) + key


def write_lmdb(directory, records, leaf_fanout=None, txnid=7):
    """records: iterable of (key bytes, value bytes).  Keys are sorted as LMDB keeps them.  Values
    too large for a node go to overflow pages.  leaf_fanout caps the records per leaf page (to force
    several tree levels with few records)."""
    os.makedirs(directory, exist_ok=True)
    records = sorted(records)
    pages = {}
    next_pg = 2
    n_overflow = 0
    leaves = []  # (first key, pgno)
    cur, cur_size = [], HDR
    first_key = None

    def flush():
        nonlocal cur, cur_size, next_pg, first_key
        if cur:
            pages[next_pg] = _page(next_pg, P_LEAF, cur)
            leaves.append((first_key, next_pg))
            next_pg += 1
            cur, cur_size, first_key = [], HDR, None

    for key, value in records:
        if 8 + len(key) + len(value) > NODEMAX:
            npg = (HDR + len(value) + PSIZE - 1) // PSIZE
            opg = next_pg
            next_pg += npg
            blob = bytearray(npg * PSIZE)
            struct.pack_into("<QHHI", blob, 0, opg, 0, P_OVERFLOW, npg)
            blob[HDR:HDR + len(value)] = value
            for i in range(npg):
                pages[opg + i] = bytes(blob[i * PSIZE:(i + 1) * PSIZE])
            n_overflow += npg
            node = _leaf_node(key, value, opg)
        else:
            node = _leaf_node(key, value)
        need = ((len(node) + 1) & ~1) + 2
        if cur and (cur_size + need > PSIZE or (leaf_fanout and len(cur) >= leaf_fanout)):
            flush()
        if first_key is None:
            first_key = key
        cur.append(node)
        cur_size += need
    flush()
    n_leaf, n_branch, depth = len(leaves), 0, 1 if leaves else 0
    level = leaves
    while len(level) > 1:
        nxt = []
        fan = leaf_fanout or 64
        for i in range(0, len(level), fan):
            group = level[i:i + fan]
            nodes = [_branch_node(b"" if j == 0 else k, pg) for j, (k, pg) in enumerate(group)]
            pages[next_pg] = _page(next_pg, P_BRANCH, nodes)
            nxt.append((group[0][0], next_pg))
            next_pg += 1
            n_branch += 1
        level = nxt
        depth += 1
    root = level[0][1] if level else (1 << 64) - 1
    last_pg = next_pg - 1 if next_pg > 2 else 1

    def meta(pgno, txn, with_db):
        buf = bytearray(PSIZE)
        struct.pack_into("<QHHHH", buf, 0, pgno, 0, P_META, 0, 0)
        struct.pack_into("<IIQQ", buf, HDR, 0xBEEFC0DE, 1, 0, 1 << 30)
        struct.pack_into("<IHHQQQQQ", buf, HDR + 24, PSIZE, 8, 0, 0, 0, 0, 0, (1 << 64) - 1)
        if with_db:
            struct.pack_into("<IHHQQQQQ", buf, HDR + 24 + 48, 0, 0, depth, n_branch, n_leaf, n_overflow, len(records), root)
            struct.pack_into("<QQ", buf, HDR + 24 + 96, last_pg, txn)
        else:
            struct.pack_into("<IHHQQQQQ", buf, HDR + 24 + 48, 0, 0, 0, 0, 0, 0, 0, (1 << 64) - 1)
            struct.pack_into("<QQ", buf, HDR + 24 + 96, 1, 0)
        return bytes(buf)

    # the current meta page is the one with the larger transaction id; put it in slot txnid % 2
    metas = [meta(0, 0, False), meta(1, 0, False)]
    metas[txnid % 2] = meta(txnid % 2, txnid, True)
    path = os.path.join(directory, "data.mdb")
    with open(path, "wb") as f:
        f.write(metas[0])
        f.write(metas[1])
        for pg in range(2, next_pg):
            f.write(pages[pg])
    return path
