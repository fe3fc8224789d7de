// Input pipeline: raw Datum bytes -> pinned staging -> asynchronous upload on a copy stream ->
// one transform kernel into the network's input (include/cct_corpus.h).
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "../../include/cct_corpus.h"
#include "cct_common.h"
#include "host/Lmdb.h"

namespace cct {

// One lane per run of four output pixels of a row; blockIdx.y = image * channels + channel, so the
// crop parameters are wavefront-uniform.  Reads run along the source row (four bytes and one
// 16-byte mean load per lane), the four results leave in one 16-byte store (reversed for a
// mirrored image); all of them need dword alignment at most.
typedef float corpus_f4u __attribute__((ext_vector_type(4), aligned(4)));

__global__ void __launch_bounds__(256)
transform_kernel(float *__restrict__ dst, const unsigned char *__restrict__ raw, const float *__restrict__ mean,
                 const int *__restrict__ params, int channels, int height, int width, int out_rows, int out_cols,
                 int crop, float scale, int quads_per_row, FastDiv div_quads) {
  const uint32_t p = blockIdx.x * 256u + threadIdx.x;
  if (p >= (uint32_t)(out_rows * quads_per_row)) return;
  const uint32_t plane = blockIdx.y;  // image * channels + c
  const uint32_t img = plane / (uint32_t)channels, c = plane - img * (uint32_t)channels;
  const uint32_t h = fdiv(p, div_quads), w0 = (p - h * (uint32_t)quads_per_row) * 4u;
  int h_off = 0, w_off = 0, mirror = 0;
  if (crop > 0) {
    h_off = params[3 * img];
    w_off = params[3 * img + 1];
    mirror = params[3 * img + 2];
  }
  const size_t in_plane = (size_t)(c * (uint32_t)height + h + (uint32_t)h_off) * (uint32_t)width + w0 + (uint32_t)w_off;
  const unsigned char *src = raw + (size_t)img * channels * height * width + in_plane;
  float *drow = dst + ((size_t)plane * out_rows + h) * out_cols;
  const int n = min(4, out_cols - (int)w0);  // pixels of this run inside the row
  float v[4];
  if (n == 4) {
    const corpus_f4u m = mean ? *reinterpret_cast<const corpus_f4u *>(mean + in_plane) : corpus_f4u{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = ((float)src[j] - m[j]) * scale;
    if (mirror) {
      const corpus_f4u o = {v[3], v[2], v[1], v[0]};
      *reinterpret_cast<corpus_f4u *>(drow + (out_cols - 4 - (int)w0)) = o;
    } else {
      const corpus_f4u o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<corpus_f4u *>(drow + w0) = o;
    }
  } else {
    for (int j = 0; j < n; ++j) {
      const float x = ((float)src[j] - (mean ? mean[in_plane + j] : 0.f)) * scale;
      const int w = (int)w0 + j;
      drow[mirror ? out_cols - 1 - w : w] = x;
    }
  }
}

static int transform_batch(float *dst, const unsigned char *raw, const float *mean, const int *params,
                           const cct_transform_args &a, hipStream_t stream) {
  CCT_REQUIRE(dst && raw, "transform_batch: null pointer");
  CCT_REQUIRE(a.batch > 0 && a.channels > 0 && a.height > 0 && a.width > 0 && a.crop_size >= 0,
              "transform_batch: bad geometry");
  CCT_REQUIRE(a.crop_size == 0 || (a.crop_size <= a.height && a.crop_size <= a.width && params),
              "transform_batch: crop %d does not fit %dx%d (or params missing)", a.crop_size, a.height, a.width);
  const int rows = a.crop_size ? a.crop_size : a.height, cols = a.crop_size ? a.crop_size : a.width;
  CCT_REQUIRE(a.channels <= 65535 && (size_t)rows * cols < (1u << 30) && (size_t)a.height * a.width < (1u << 30),
              "transform_batch: image too large");
  CCT_REQUIRE((uintptr_t)dst % 4 == 0 && (!mean || (uintptr_t)mean % 4 == 0), "transform_batch: misaligned float pointer");
  const int quads = (cols + 3) / 4;
  // grid.y is limited to 65535: launch in slices of planes (whole images per slice)
  const size_t imgs_per_launch = std::max<size_t>(1, 65535u / (size_t)a.channels);
  for (size_t i0 = 0; i0 < (size_t)a.batch; i0 += imgs_per_launch) {
    const size_t ni = std::min(imgs_per_launch, (size_t)a.batch - i0);
    dim3 grid((unsigned)((rows * quads + 255) / 256), (unsigned)(ni * a.channels));
    transform_kernel<<<grid, 256, 0, stream>>>(dst + i0 * a.channels * rows * cols,
                                               raw + i0 * a.channels * a.height * a.width, mean,
                                               params ? params + 3 * i0 : nullptr, a.channels, a.height, a.width,
                                               rows, cols, a.crop_size, a.scale, quads, make_fastdiv((uint32_t)quads));
    CCT_LAUNCH_CHECK();
  }
  return 0;
}

// Two staging slots (pinned host + device raw buffer each), a copy stream and two events per slot.
class Corpus {
 public:
  cct_transform_args geo{};
  int mirror = 0, phase = 0;
  size_t n_images = 0;

  ~Corpus() { release(); }

  int init(int batch, int channels, int height, int width, int crop, float scale, int mirror_, int phase_,
           const float *mean_host, unsigned seed) {
    CCT_REQUIRE(batch > 0 && channels > 0 && height > 0 && width > 0, "corpus: bad geometry");
    CCT_REQUIRE(phase_ == 0 || phase_ == 1, "corpus: phase must be 0 (TRAIN) or 1 (TEST)");
    CCT_REQUIRE((double)batch * channels * height * width < 2147483648.0, "corpus: a batch of raw images must stay below 2 GiB");
    CCT_REQUIRE(crop >= 0 && crop <= height && crop <= width, "corpus: crop_size %d does not fit %dx%d images", crop,
                height, width);
    geo.batch = batch; geo.channels = channels; geo.height = height; geo.width = width;
    geo.crop_size = crop; geo.scale = scale;
    mirror = mirror_; phase = phase_;
    rng_.seed(seed);
    pixel_bytes_ = (size_t)batch * channels * height * width;
    labels_off_ = (pixel_bytes_ + 255) & ~(size_t)255;
    params_off_ = labels_off_ + (((size_t)batch * sizeof(float) + 255) & ~(size_t)255);
    slot_bytes_ = params_off_ + (size_t)batch * 3 * sizeof(int);
    CCT_HIP_CHECK(hipStreamCreateWithFlags(&copy_stream_, hipStreamNonBlocking));
    for (int s = 0; s < 2; ++s) {
      CCT_HIP_CHECK(hipHostMalloc(&host_[s], slot_bytes_, hipHostMallocDefault));
      CCT_HIP_CHECK(hipMalloc(&dev_[s], slot_bytes_));
      CCT_HIP_CHECK(hipEventCreateWithFlags(&uploaded_[s], hipEventDisableTiming));
      CCT_HIP_CHECK(hipEventCreateWithFlags(&consumed_[s], hipEventDisableTiming));
    }
    if (mean_host) {
      const size_t n = (size_t)channels * height * width;
      CCT_HIP_CHECK(hipMalloc((void **)&mean_dev_, n * sizeof(float)));
      CCT_HIP_CHECK(hipMemcpy(mean_dev_, mean_host, n * sizeof(float), hipMemcpyHostToDevice));
    }
    return 0;
  }

  int open_lmdb(const char *dir) {
    CCT_REQUIRE(db_.open(dir), "corpus: %s", db_.error().c_str());
    n_images = db_.entries();
    CCT_REQUIRE(n_images > 0, "corpus: %s holds no records", dir);
    return 0;
  }
  LmdbReader &db() { return db_; }

  // next free slot, its pinned buffer safe to overwrite
  int stage(unsigned char **pixels, float **labels, int **params) {
    CCT_REQUIRE(staged_ || in_flight_ < 2, "corpus: two batches are already in flight; consume one first");
    const int s = head_;
    if (!staged_) {
      if (upload_recorded_[s]) CCT_HIP_CHECK(hipEventSynchronize(uploaded_[s]));
      draw_params((int *)((char *)host_[s] + params_off_));
      staged_ = true;
    }
    if (pixels) *pixels = (unsigned char *)host_[s];
    if (labels) *labels = (float *)((char *)host_[s] + labels_off_);
    if (params) *params = (int *)((char *)host_[s] + params_off_);
    return 0;
  }

  // Labels index the class scores in the loss layer: with a class count set, a batch holding a
  // label outside [0, num_classes) (or a NaN) is refused on the host, before anything is uploaded.
  void set_num_classes(int n) { num_classes_ = n; }

  int submit() {
    CCT_REQUIRE(staged_, "corpus: nothing staged");
    const int s = head_;
    if (num_classes_ > 0) {
      const float *l = (const float *)((const char *)host_[s] + labels_off_);
      for (int b = 0; b < geo.batch; ++b)
        CCT_REQUIRE(l[b] >= 0.0f && l[b] < (float)num_classes_,
                    "corpus: label %g of image %d is outside [0, %d)", (double)l[b], b, num_classes_);
    }
    if (geo.crop_size > 0) {
      // a caller may have overwritten the drawn parameters: the kernel trusts them, so check here
      const int *p = (const int *)((const char *)host_[s] + params_off_);
      for (int b = 0; b < geo.batch; ++b)
        CCT_REQUIRE(p[3 * b] >= 0 && p[3 * b] <= geo.height - geo.crop_size && p[3 * b + 1] >= 0 &&
                        p[3 * b + 1] <= geo.width - geo.crop_size && (p[3 * b + 2] == 0 || p[3 * b + 2] == 1),
                    "corpus: crop parameters of image %d (%d, %d, %d) are out of range", b, p[3 * b], p[3 * b + 1],
                    p[3 * b + 2]);
    }
    // the device buffer of this slot may still be read by the transform of two batches ago
    if (consume_recorded_[s]) CCT_HIP_CHECK(hipStreamWaitEvent(copy_stream_, consumed_[s], 0));
    CCT_HIP_CHECK(hipMemcpyAsync(dev_[s], host_[s], slot_bytes_, hipMemcpyHostToDevice, copy_stream_));
    CCT_HIP_CHECK(hipEventRecord(uploaded_[s], copy_stream_));
    upload_recorded_[s] = true;
    staged_ = false;
    head_ ^= 1;
    ++in_flight_;
    return 0;
  }

  // LoadLmdbData over a whole batch with wrap-around; worker threads copy the Datum bytes
  int load_next(int *epoch) {
    CCT_REQUIRE(n_images > 0, "corpus: not opened on a database");
    unsigned char *pixels; float *labels; int *params;
    int rc = stage(&pixels, &labels, &params);
    if (rc) return rc;
    const size_t image_bytes = (size_t)geo.channels * geo.height * geo.width;
    records_.resize(geo.batch);
    for (int b = 0; b < geo.batch; ++b) {
      LmdbReader::Entry e;
      if (!db_.next(&e)) {
        CCT_REQUIRE(db_.error().empty(), "corpus: %s", db_.error().c_str());
        ++epoch_;          // end of the database: ResetCursor and continue filling the batch
        db_.rewind();
        CCT_REQUIRE(db_.next(&e), "corpus: %s", db_.error().empty() ? "empty database" : db_.error().c_str());
      }
      records_[b] = e;
    }
    const int workers = std::max(1, std::min<int>(geo.batch, std::min(16u, std::max(1u, std::thread::hardware_concurrency()))));
    std::vector<int> bad(workers, -1);
    auto work = [&](int t) {
      for (int b = t; b < geo.batch; b += workers) {
        DatumView d;
        if (!parse_datum(records_[b].value, records_[b].value_size, &d) || d.channels != geo.channels ||
            d.height != geo.height || d.width != geo.width || d.data_size != image_bytes) {
          bad[t] = b;
          return;
        }
        labels[b] = (float)d.label;
        std::memcpy(pixels + (size_t)b * image_bytes, d.data, image_bytes);
      }
    };
    std::vector<std::thread> pool;
    for (int t = 1; t < workers; ++t) pool.emplace_back(work, t);
    work(0);
    for (std::thread &t : pool) t.join();
    for (int t = 0; t < workers; ++t)
      CCT_REQUIRE(bad[t] < 0, "corpus: record %d of the batch is not a %dx%dx%d byte Datum (float_data records are not supported)",
                  bad[t], geo.channels, geo.height, geo.width);
    if (epoch) *epoch = epoch_;
    return submit();
  }

  int consume(float *images_dev, float *labels_dev, int *params_out) {
    CCT_REQUIRE(in_flight_ > 0, "corpus: no batch in flight");
    CCT_REQUIRE(images_dev && labels_dev, "corpus: null destination");
    const int s = tail_;
    hipStream_t st = ctx().stream;
    CCT_HIP_CHECK(hipStreamWaitEvent(st, uploaded_[s], 0));
    const char *d = (const char *)dev_[s];
    int rc = transform_batch(images_dev, (const unsigned char *)d, mean_dev_, (const int *)(d + params_off_), geo, st);
    if (rc) return rc;
    CCT_HIP_CHECK(hipMemcpyAsync(labels_dev, d + labels_off_, (size_t)geo.batch * sizeof(float), hipMemcpyDeviceToDevice, st));
    CCT_HIP_CHECK(hipEventRecord(consumed_[s], st));
    consume_recorded_[s] = true;
    if (params_out) {
      // the pinned copy is intact until this slot is staged again
      std::memcpy(params_out, (const char *)host_[s] + params_off_, (size_t)geo.batch * 3 * sizeof(int));
    }
    tail_ ^= 1;
    --in_flight_;
    return 0;
  }

 private:
  LmdbReader db_;
  std::vector<LmdbReader::Entry> records_;
  std::mt19937 rng_;
  hipStream_t copy_stream_ = nullptr;
  void *host_[2] = {nullptr, nullptr};
  void *dev_[2] = {nullptr, nullptr};
  hipEvent_t uploaded_[2] = {nullptr, nullptr}, consumed_[2] = {nullptr, nullptr};
  bool upload_recorded_[2] = {false, false}, consume_recorded_[2] = {false, false};
  float *mean_dev_ = nullptr;
  size_t pixel_bytes_ = 0, labels_off_ = 0, params_off_ = 0, slot_bytes_ = 0;
  int head_ = 0, tail_ = 0, in_flight_ = 0, epoch_ = 0, num_classes_ = 0;
  bool staged_ = false;

  // process_image's choices (src/parser/corpus.h:266-276): random offsets in [0, size - crop) and a
  // coin flip for the mirror while training, the centre crop otherwise.  An image exactly as large
  // as the crop gets offset 0 (the reference would take a remainder by zero there).
  void draw_params(int *p) {
    const int crop = geo.crop_size;
    for (int b = 0; b < geo.batch; ++b) {
      int h_off = 0, w_off = 0, flip = 0;
      if (crop > 0) {
        if (phase == 0) {
          h_off = geo.height > crop ? (int)(rng_() % (unsigned)(geo.height - crop)) : 0;
          w_off = geo.width > crop ? (int)(rng_() % (unsigned)(geo.width - crop)) : 0;
          flip = (mirror && (rng_() & 1u)) ? 1 : 0;
        } else {
          h_off = (geo.height - crop) / 2;
          w_off = (geo.width - crop) / 2;
        }
      }
      p[3 * b] = h_off; p[3 * b + 1] = w_off; p[3 * b + 2] = flip;
    }
  }

  void release() {
    if (copy_stream_) (void)hipStreamSynchronize(copy_stream_);
    (void)hipStreamSynchronize(ctx().stream);
    for (int s = 0; s < 2; ++s) {
      if (host_[s]) (void)hipHostFree(host_[s]);
      if (dev_[s]) (void)hipFree(dev_[s]);
      if (uploaded_[s]) (void)hipEventDestroy(uploaded_[s]);
      if (consumed_[s]) (void)hipEventDestroy(consumed_[s]);
    }
    if (mean_dev_) (void)hipFree(mean_dev_);
    if (copy_stream_) (void)hipStreamDestroy(copy_stream_);
  }
};

static bool read_file(const char *path, std::vector<uint8_t> *out) {
  FILE *f = std::fopen(path, "rb");
  if (!f) return false;
  std::fseek(f, 0, SEEK_END);
  const long n = std::ftell(f);
  std::fseek(f, 0, SEEK_SET);
  out->resize(n > 0 ? (size_t)n : 0);
  const bool ok = n >= 0 && std::fread(out->data(), 1, out->size(), f) == out->size();
  std::fclose(f);
  return ok;
}

}  // namespace cct

using namespace cct;

struct cct_corpus {
  Corpus impl;
};

struct cct_lmdb {
  LmdbReader reader;
};

extern "C" {

int cct_hip_transform_batch(float *dst, const unsigned char *raw, const float *mean, const int *params,
                            const cct_transform_args *args) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(args, "transform_batch: null args");
  return transform_batch(dst, raw, mean, params, *args, ctx().stream);
}

int cct_corpus_create(cct_corpus **out, int batch, int channels, int height, int width, int crop_size, float scale,
                      int mirror, int phase, const float *mean, unsigned int seed) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(out, "corpus_create: null handle");
  cct_corpus *c = new cct_corpus;
  int rc = c->impl.init(batch, channels, height, width, crop_size, scale, mirror, phase, mean, seed);
  if (rc) {
    delete c;
    return rc;
  }
  *out = c;
  return 0;
}

int cct_corpus_open(cct_corpus **out, const char *lmdb_dir, int batch, int crop_size, float scale, int mirror,
                    int phase, const char *mean_file, const float *mean_values, int n_mean_values,
                    unsigned int seed) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(out && lmdb_dir, "corpus_open: null argument");
  CCT_REQUIRE(!(mean_file && n_mean_values > 0), "corpus_open: mean_file and mean_value cannot both be given");
  cct_corpus *c = new cct_corpus;
  int rc = c->impl.open_lmdb(lmdb_dir);
  DatumView d;
  if (!rc) {
    // geometry from the first record (src/parser/corpus.h:192-224)
    LmdbReader::Entry e;
    if (!c->impl.db().next(&e) || !parse_datum(e.value, e.value_size, &d) || d.channels <= 0 || d.height <= 0 || d.width <= 0)
      rc = set_error(CCT_HIP_EINVAL, "corpus_open: the first record of %s is not a Datum", lmdb_dir);
    c->impl.db().rewind();
  }
  std::vector<float> mean;
  if (!rc) {
    const size_t plane = (size_t)d.height * d.width, n = plane * d.channels;
    if (mean_file) {
      std::vector<uint8_t> bytes;
      int dims[4];
      if (!read_file(mean_file, &bytes) || !parse_cube(bytes.data(), bytes.size(), dims, &mean))
        rc = set_error(CCT_HIP_EINVAL, "corpus_open: cannot read the mean image %s", mean_file);
      else if (mean.size() < n)
        rc = set_error(CCT_HIP_EINVAL, "corpus_open: mean image %s holds %zu values, the images have %zu", mean_file,
                       mean.size(), n);
      else
        mean.resize(n);
    } else if (n_mean_values > 0 && mean_values) {
      // one value per channel, channels beyond the list get 0 (src/parser/corpus.h:243-254)
      mean.assign(n, 0.f);
      for (int ch = 0; ch < d.channels && ch < n_mean_values; ++ch)
        std::fill(mean.begin() + ch * plane, mean.begin() + (ch + 1) * plane, mean_values[ch]);
    }
  }
  if (!rc)
    rc = c->impl.init(batch, d.channels, d.height, d.width, crop_size, scale, mirror, phase,
                      mean.empty() ? nullptr : mean.data(), seed);
  if (rc) {
    delete c;
    return rc;
  }
  *out = c;
  return 0;
}

int cct_corpus_close(cct_corpus *c) {
  if (!c) return 0;
  CCT_ENSURE_INIT();
  delete c;
  return 0;
}

int cct_corpus_get_info(cct_corpus *c, cct_corpus_info *info) {
  CCT_REQUIRE(c && info, "corpus_get_info: null argument");
  const cct_transform_args &g = c->impl.geo;
  info->n_images = c->impl.n_images;
  info->batch = g.batch; info->channels = g.channels; info->height = g.height; info->width = g.width;
  info->out_rows = g.crop_size ? g.crop_size : g.height;
  info->out_cols = g.crop_size ? g.crop_size : g.width;
  return 0;
}

int cct_corpus_set_num_classes(cct_corpus *c, int num_classes) {
  CCT_REQUIRE(c && num_classes >= 0, "corpus_set_num_classes: bad argument");
  c->impl.set_num_classes(num_classes);
  return 0;
}

int cct_corpus_load_next(cct_corpus *c, int *epoch) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(c, "corpus_load_next: null handle");
  return c->impl.load_next(epoch);
}

int cct_corpus_stage(cct_corpus *c, unsigned char **pixels, float **labels, int **params) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(c, "corpus_stage: null handle");
  return c->impl.stage(pixels, labels, params);
}

int cct_corpus_submit(cct_corpus *c) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(c, "corpus_submit: null handle");
  return c->impl.submit();
}

int cct_corpus_consume(cct_corpus *c, float *images_dev, float *labels_dev, int *params_out) {
  CCT_ENSURE_INIT();
  CCT_REQUIRE(c, "corpus_consume: null handle");
  return c->impl.consume(images_dev, labels_dev, params_out);
}

// ---- file readers on their own (no device) ----

int cct_lmdb_open(cct_lmdb **out, const char *path) {
  CCT_REQUIRE(out && path, "lmdb_open: null argument");
  cct_lmdb *db = new cct_lmdb;
  if (!db->reader.open(path)) {
    const int rc = set_error(CCT_HIP_EINVAL, "lmdb_open: %s", db->reader.error().c_str());
    delete db;
    return rc;
  }
  *out = db;
  return 0;
}

int cct_lmdb_close(cct_lmdb *db) {
  delete db;
  return 0;
}

size_t cct_lmdb_entries(cct_lmdb *db) { return db ? db->reader.entries() : 0; }

int cct_lmdb_rewind(cct_lmdb *db) {
  CCT_REQUIRE(db, "lmdb_rewind: null handle");
  db->reader.rewind();
  return 0;
}

int cct_lmdb_next(cct_lmdb *db, const void **key, size_t *key_size, const void **value, size_t *value_size) {
  if (!db) return -1;
  LmdbReader::Entry e;
  if (!db->reader.next(&e)) {
    if (db->reader.error().empty()) return 0;
    set_error(CCT_HIP_EINVAL, "lmdb_next: %s", db->reader.error().c_str());
    return -1;
  }
  if (key) *key = e.key;
  if (key_size) *key_size = e.key_size;
  if (value) *value = e.value;
  if (value_size) *value_size = e.value_size;
  return 1;
}

int cct_datum_parse(const void *value, size_t size, int dims[4], const void **data, size_t *data_size,
                    size_t *float_count) {
  CCT_REQUIRE(value && dims, "datum_parse: null argument");
  DatumView d;
  CCT_REQUIRE(parse_datum((const uint8_t *)value, size, &d), "datum_parse: malformed Datum");
  dims[0] = d.channels; dims[1] = d.height; dims[2] = d.width; dims[3] = d.label;
  if (data) *data = d.data;
  if (data_size) *data_size = d.data_size;
  if (float_count) *float_count = d.float_count;
  return 0;
}

int cct_mean_read(const char *file, int dims[4], float *data, size_t capacity, size_t *count) {
  CCT_REQUIRE(file && dims, "mean_read: null argument");
  std::vector<uint8_t> bytes;
  std::vector<float> values;
  CCT_REQUIRE(read_file(file, &bytes), "mean_read: cannot read %s", file);
  CCT_REQUIRE(parse_cube(bytes.data(), bytes.size(), dims, &values), "mean_read: %s is not a binary Cube message", file);
  if (count) *count = values.size();
  if (data) std::memcpy(data, values.data(), std::min(capacity, values.size()) * sizeof(float));
  return 0;
}

}  // extern "C"
