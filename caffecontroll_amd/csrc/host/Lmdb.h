// Read-only access to the files the reference's input pipeline reads
// (src/parser/corpus.h:62-108, 170-232): an LMDB environment of serialized `Datum` messages and a
// binary `Cube` message holding the mean image (src/parser/cnn.proto:3-19).
//
// The reference links liblmdb and libprotobuf; neither is used here.  LmdbReader walks the data file
// through a private read-only mapping using LMDB's published on-disk layout (data format version 1,
// `lmdb.h` / `mdb.c` of OpenLDAP LMDB 0.9.x):
//   page header   pgno u64 | pad u16 | flags u16 | lower u16, upper u16  (overflow pages: page count u32)
//                 then u16 node offsets; number of keys = (lower - 16) / 2
//   meta pages    0 and 1; after the header: magic 0xBEEFC0DE u32 | version u32 | address u64 |
//                 mapsize u64 | two 48-byte database records (free list, main) | last page u64 | txn id u64;
//                 the one with the larger txn id is current; record = pad u32 (page size in the free-list
//                 record) | flags u16 | depth u16 | branch, leaf, overflow page counts u64 x3 | entries u64 | root u64
//   node          lo u16 | hi u16 | flags u16 | key size u16 | key bytes | data
//                 branch: child page = lo | hi << 16 | flags << 32;  leaf: data size = lo | hi << 16,
//                 flag 0x01 = data is the u64 number of the first of a run of overflow pages whose
//                 payload starts 16 bytes into the first page and is contiguous
// Keys are visited in the tree's order, i.e. sorted, as an MDB_FIRST / MDB_NEXT cursor does.
// Named sub-databases and duplicate-key databases do not occur in Caffe-style datasets and are rejected.
#pragma once
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace cct {

class LmdbReader {
 public:
  struct Entry {
    const uint8_t *key = nullptr;
    size_t key_size = 0;
    const uint8_t *value = nullptr;
    size_t value_size = 0;
  };

  LmdbReader() {}
  ~LmdbReader() { close(); }
  LmdbReader(const LmdbReader &) = delete;
  LmdbReader &operator=(const LmdbReader &) = delete;

  const std::string &error() const { return error_; }
  size_t entries() const { return entries_; }
  size_t page_size() const { return psize_; }
  unsigned depth() const { return depth_; }

  // `path` is the environment directory (holding data.mdb) or the data file itself.
  bool open(const std::string &path) {
    close();
    std::string file = path;
    struct stat st;
    if (::stat(file.c_str(), &st) == 0 && S_ISDIR(st.st_mode)) file += "/data.mdb";
    fd_ = ::open(file.c_str(), O_RDONLY);
    if (fd_ < 0) return fail("cannot open " + file);
    if (::fstat(fd_, &st) != 0 || st.st_size < 2 * 4096) return fail(file + " is too small to be an LMDB data file");
    size_ = (size_t)st.st_size;
    void *p = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (p == MAP_FAILED) {
      base_ = nullptr;
      return fail("cannot map " + file);
    }
    base_ = (const uint8_t *)p;
    if (rd32(base_ + 16) != 0xBEEFC0DEu) return fail(file + ": not an LMDB data file (bad magic)");
    if (rd32(base_ + 20) != 1) return fail(file + ": unsupported LMDB data format version");
    psize_ = rd32(base_ + 16 + 24);  // pad field of the free-list record
    if (psize_ < 512 || (psize_ & (psize_ - 1)) || 2 * psize_ > size_) return fail(file + ": bad page size");
    const uint8_t *m0 = base_, *m1 = base_ + psize_;
    if (rd32(m1 + 16) != 0xBEEFC0DEu) return fail(file + ": second meta page is damaged");
    const uint8_t *meta = rd64(m1 + kMetaTxn) > rd64(m0 + kMetaTxn) ? m1 : m0;
    const uint8_t *main_db = meta + 16 + 24 + 48;
    const uint16_t flags = rd16(main_db + 4);
    if (flags & 0x04) return fail(file + ": duplicate-key databases are not supported");
    depth_ = rd16(main_db + 6);
    entries_ = (size_t)rd64(main_db + 32);
    root_ = rd64(main_db + 40);
    last_page_ = rd64(meta + kMetaTxn - 8);
    if ((last_page_ + 1) * psize_ > size_) return fail(file + ": file is shorter than its last page");
    if (entries_ == 0 || root_ == ~0ull) {
      entries_ = 0;
      root_ = ~0ull;
    }
    rewind();
    return true;
  }

  void close() {
    if (base_) ::munmap((void *)base_, size_);
    if (fd_ >= 0) ::close(fd_);
    base_ = nullptr;
    fd_ = -1;
    entries_ = 0;
    root_ = ~0ull;  // next() after close() reports the end instead of walking unmapped pages
    started_ = false;
    stack_.clear();
  }

  // MDB_FIRST on the next call of next()
  void rewind() {
    stack_.clear();
    started_ = false;
  }

  // MDB_FIRST / MDB_NEXT: false at the end of the database or on a damaged file (error() non-empty)
  bool next(Entry *out) {
    if (root_ == ~0ull) return false;
    if (!started_) {
      started_ = true;
      if (!descend(root_)) return false;
    } else {
      // advance in the leaf, climbing while pages are exhausted
      while (!stack_.empty()) {
        Frame &f = stack_.back();
        if (++f.index < f.nkeys) break;
        stack_.pop_back();
      }
      if (stack_.empty()) return false;
      if (!(flags_of(stack_.back().page) & kLeaf)) {
        const uint64_t child = branch_child(stack_.back().page, stack_.back().index);
        if (!descend(child)) return false;
      }
    }
    const Frame &f = stack_.back();
    return leaf_entry(f.page, f.index, out);
  }

 private:
  enum { kBranch = 0x01, kLeaf = 0x02, kOverflow = 0x04, kLeaf2 = 0x20, kBigData = 0x01, kSubData = 0x02, kDupData = 0x04 };
  static constexpr size_t kHeader = 16;
  static constexpr size_t kMetaTxn = 16 + 24 + 96 + 8;  // offset of the txn id inside a meta page

  struct Frame {
    const uint8_t *page;
    unsigned index, nkeys;
  };

  int fd_ = -1;
  const uint8_t *base_ = nullptr;
  size_t size_ = 0, psize_ = 0, entries_ = 0;
  uint64_t root_ = ~0ull, last_page_ = 0;
  unsigned depth_ = 0;
  bool started_ = false;
  std::vector<Frame> stack_;
  std::string error_;

  static uint16_t rd16(const uint8_t *p) { uint16_t v; std::memcpy(&v, p, 2); return v; }
  static uint32_t rd32(const uint8_t *p) { uint32_t v; std::memcpy(&v, p, 4); return v; }
  static uint64_t rd64(const uint8_t *p) { uint64_t v; std::memcpy(&v, p, 8); return v; }
  bool fail(const std::string &msg) {
    error_ = msg;
    if (base_) ::munmap((void *)base_, size_);
    if (fd_ >= 0) ::close(fd_);
    base_ = nullptr;
    fd_ = -1;
    root_ = ~0ull;
    entries_ = 0;
    stack_.clear();
    return false;
  }
  bool damaged(const char *what) {
    error_ = std::string("damaged LMDB file: ") + what;
    stack_.clear();
    root_ = ~0ull;
    return false;
  }
  const uint8_t *page(uint64_t pgno) const { return pgno <= last_page_ ? base_ + pgno * psize_ : nullptr; }
  static unsigned flags_of(const uint8_t *pg) { return rd16(pg + 10); }
  static unsigned nkeys_of(const uint8_t *pg) {
    const unsigned lower = rd16(pg + 12);
    return lower >= kHeader ? (lower - kHeader) >> 1 : 0;
  }
  const uint8_t *node(const uint8_t *pg, unsigned i) const {
    const unsigned off = rd16(pg + kHeader + 2 * i);
    return off + 8 <= psize_ ? pg + off : nullptr;
  }
  uint64_t branch_child(const uint8_t *pg, unsigned i) const {
    const uint8_t *n = node(pg, i);
    if (!n) return ~0ull;
    return (uint64_t)rd16(n) | ((uint64_t)rd16(n + 2) << 16) | ((uint64_t)rd16(n + 4) << 32);
  }
  // pushes the path from page `pgno` down to the first entry of its leftmost leaf
  bool descend(uint64_t pgno) {
    for (unsigned guard = 0; guard < 64; ++guard) {
      const uint8_t *pg = page(pgno);
      if (!pg) return damaged("page number out of range");
      const unsigned fl = flags_of(pg), nk = nkeys_of(pg);
      if (fl & kLeaf2) return damaged("fixed-size-key leaf pages are not supported");
      if (nk == 0 || kHeader + 2 * nk > psize_) return damaged("empty or oversized page");
      stack_.push_back(Frame{pg, 0u, nk});
      if (fl & kLeaf) return true;
      if (!(fl & kBranch)) return damaged("unexpected page type in the tree");
      pgno = branch_child(pg, 0);
    }
    return damaged("tree deeper than 64 levels");
  }
  bool leaf_entry(const uint8_t *pg, unsigned i, Entry *out) {
    const uint8_t *n = node(pg, i);
    if (!n) return damaged("node offset out of range");
    const size_t dsize = (size_t)rd16(n) | ((size_t)rd16(n + 2) << 16);
    const unsigned nflags = rd16(n + 4);
    const size_t ksize = rd16(n + 6);
    if (nflags & (kSubData | kDupData)) return damaged("sub-databases / duplicate keys are not supported");
    const size_t off = (size_t)(n - pg) + 8;
    if (off + ksize > psize_) return damaged("key runs past its page");
    out->key = n + 8;
    out->key_size = ksize;
    if (nflags & kBigData) {
      if (off + ksize + 8 > psize_) return damaged("overflow reference runs past its page");
      const uint64_t opg = rd64(n + 8 + ksize);
      const uint8_t *o = page(opg);
      if (!o || !(flags_of(o) & kOverflow)) return damaged("overflow page expected");
      const uint64_t npages = rd32(o + 12);
      if (npages == 0 || opg + npages - 1 > last_page_ || kHeader + dsize > npages * psize_)
        return damaged("overflow run does not hold its value");
      out->value = o + kHeader;
    } else {
      if (off + ksize + dsize > psize_) return damaged("value runs past its page");
      out->value = n + 8 + ksize;
    }
    out->value_size = dsize;
    return true;
  }
};

// ---- protobuf wire format, just enough for Datum and Cube -----------------------------------

struct DatumView {
  int channels = 0, height = 0, width = 0, label = 0;
  const uint8_t *data = nullptr;  // `bytes data = 4`
  size_t data_size = 0;
  size_t float_count = 0;  // number of `float_data = 6` values (not decoded)
};

namespace wire {
inline bool varint(const uint8_t *&p, const uint8_t *end, uint64_t *v) {
  uint64_t r = 0;
  for (unsigned shift = 0; shift < 64 && p < end; shift += 7) {
    const uint8_t b = *p++;
    r |= (uint64_t)(b & 0x7f) << shift;
    if (!(b & 0x80)) {
      *v = r;
      return true;
    }
  }
  return false;
}
// skips a field of wire type `wt`; false on malformed input
inline bool skip(const uint8_t *&p, const uint8_t *end, unsigned wt) {
  uint64_t v;
  switch (wt) {
    case 0: return varint(p, end, &v);
    case 1: if (end - p < 8) return false; p += 8; return true;
    case 2: if (!varint(p, end, &v) || (uint64_t)(end - p) < v) return false; p += v; return true;
    case 5: if (end - p < 4) return false; p += 4; return true;
    default: return false;
  }
}
}  // namespace wire

// message Datum { int32 channels=1, height=2, width=3; bytes data=4; int32 label=5; repeated float float_data=6 }
inline bool parse_datum(const uint8_t *p, size_t n, DatumView *d) {
  const uint8_t *end = p + n;
  *d = DatumView();
  while (p < end) {
    uint64_t tag, v;
    if (!wire::varint(p, end, &tag)) return false;
    const unsigned field = (unsigned)(tag >> 3), wt = (unsigned)(tag & 7);
    if (wt == 0 && (field == 1 || field == 2 || field == 3 || field == 5)) {
      if (!wire::varint(p, end, &v)) return false;
      (field == 1 ? d->channels : field == 2 ? d->height : field == 3 ? d->width : d->label) = (int)(int64_t)v;
    } else if (field == 4 && wt == 2) {
      if (!wire::varint(p, end, &v) || (uint64_t)(end - p) < v) return false;
      d->data = p;
      d->data_size = (size_t)v;
      p += v;
    } else if (field == 6 && wt == 2) {  // packed
      if (!wire::varint(p, end, &v) || (uint64_t)(end - p) < v) return false;
      d->float_count += (size_t)v / 4;
      p += v;
    } else if (field == 6 && wt == 5) {  // unpacked
      if (end - p < 4) return false;
      d->float_count += 1;
      p += 4;
    } else if (!wire::skip(p, end, wt)) {
      return false;
    }
  }
  return true;
}

// message Cube { int32 num=1, channels=2, height=3, width=4; repeated float data=5 [packed] }: the mean image
inline bool parse_cube(const uint8_t *p, size_t n, int dims[4], std::vector<float> *data) {
  const uint8_t *end = p + n;
  dims[0] = dims[1] = dims[2] = dims[3] = 0;
  data->clear();
  while (p < end) {
    uint64_t tag, v;
    if (!wire::varint(p, end, &tag)) return false;
    const unsigned field = (unsigned)(tag >> 3), wt = (unsigned)(tag & 7);
    if (wt == 0 && field >= 1 && field <= 4) {
      if (!wire::varint(p, end, &v)) return false;
      dims[field - 1] = (int)(int64_t)v;
    } else if (field == 5 && wt == 2) {
      if (!wire::varint(p, end, &v) || (uint64_t)(end - p) < v || (v & 3)) return false;
      const size_t old = data->size();
      data->resize(old + v / 4);
      std::memcpy(data->data() + old, p, v);
      p += v;
    } else if (field == 5 && wt == 5) {
      if (end - p < 4) return false;
      float f;
      std::memcpy(&f, p, 4);
      data->push_back(f);
      p += 4;
    } else if (!wire::skip(p, end, wt)) {
      return false;
    }
  }
  return true;
}

}  // namespace cct
