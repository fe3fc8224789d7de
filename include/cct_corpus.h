/*
 * cct_corpus.h -- the step before the training path: mini-batches from an LMDB of Datum records
 * to the network's input cube on the device.
 *
 * Stands for class Corpus of the reference (src/parser/corpus.h): the constructor's geometry and
 * mean set-up (:170-258), OpenLmdbReader / LoadLmdbData / ResetCursor (:62-161) and process_image
 * (:262-333).  The reference turns every Datum into floats on the host (one thread per image) and
 * the bridges then copy the float batch to the device.  Here the host stage only copies the raw
 * bytes of each Datum into pinned memory (worker threads), one asynchronous copy on a second
 * stream moves bytes + labels + per-image crop parameters to the device while the previous
 * iteration computes, and mean subtraction, crop, mirror and scaling run in one kernel that writes
 * the float batch straight into the network's input: a quarter of the bus traffic, no float copy
 * of the batch on the host.
 *
 * All functions return 0 on success; cct_hip_last_error() has the text otherwise.
 */
#ifndef CCT_CORPUS_H
#define CCT_CORPUS_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Geometry of one mini-batch of raw images and of what the transform produces. */
typedef struct cct_transform_args {
  int batch, channels, height, width; /* Datum geometry; raw is [batch][channels][height][width] bytes */
  int crop_size;                      /* 0: no crop and no mirror, output is height x width */
  float scale;                        /* applied after the mean is subtracted */
} cct_transform_args;

/* Corpus::process_image (src/parser/corpus.h:262-333) for a whole mini-batch, on the library's
 * stream:  dst[i][c][h][w'] = (float(raw[i][c][h+h_off][w+w_off]) - mean[c][h+h_off][w+w_off]) * scale
 * with w' = w, or crop_size-1-w for a mirrored image.  params holds (h_off, w_off, mirror) per
 * image as 3 ints (ignored when crop_size == 0); mean is [channels][height][width] or NULL (zero
 * mean).  All pointers are device pointers. */
int cct_hip_transform_batch(float *dst, const unsigned char *raw, const float *mean, const int *params,
                            const cct_transform_args *args);

typedef struct cct_corpus cct_corpus;

typedef struct cct_corpus_info {
  size_t n_images;                    /* entries of the database (0 for a memory-fed corpus) */
  int batch, channels, height, width; /* Datum geometry */
  int out_rows, out_cols;             /* crop_size if set, else height x width */
} cct_corpus_info;

/* Opens <lmdb_dir>/data.mdb read-only and reads the first Datum for the geometry, as the Corpus
 * constructor does.  phase 0 = TRAIN (random crop offsets, random mirror when `mirror` is set),
 * 1 = TEST (centre crop, no mirror).  The mean comes from `mean_file` (binary Cube message) or from
 * per-channel `mean_values` (n_mean_values may be 0: zero mean).  `seed` drives the crop/mirror
 * choices (the reference uses libc rand() from its image threads). */
int cct_corpus_open(cct_corpus **out, const char *lmdb_dir, int batch, int crop_size, float scale, int mirror,
                    int phase, const char *mean_file, const float *mean_values, int n_mean_values,
                    unsigned int seed);
/* The same pipeline without a database: the caller writes raw bytes and labels into the staging
 * buffers itself (cct_corpus_stage / cct_corpus_submit).  `mean` is a host array
 * [channels][height][width] or NULL. */
int cct_corpus_create(cct_corpus **out, int batch, int channels, int height, int width, int crop_size,
                      float scale, int mirror, int phase, const float *mean, unsigned int seed);
int cct_corpus_close(cct_corpus *c);
int cct_corpus_get_info(cct_corpus *c, cct_corpus_info *info);
/* Number of classes of the network's loss layer (0 = unknown, the default).  Once set, a batch that
 * holds a label outside [0, num_classes) is refused by cct_corpus_load_next / cct_corpus_submit on
 * the host and nothing of it is uploaded.  The reference indexes the class scores with the label
 * unchecked (src/kernels/softmax.hxx:49-52); on a device that would be an out-of-bounds read. */
int cct_corpus_set_num_classes(cct_corpus *c, int num_classes);

/* Host stage, LMDB-fed: reads the next `batch` records (LoadLmdbData; wraps to the first record at
 * the end of the database and counts an epoch, as DeepNet::train_network does, src/DeepNet.h:2083-2095),
 * draws the crop parameters and starts the asynchronous upload.  At most two batches can be in
 * flight; a third call before cct_corpus_consume fails.  *epoch receives the number of wraps so far. */
int cct_corpus_load_next(cct_corpus *c, int *epoch);
/* Host stage, memory-fed: pointers into the next free pinned staging buffer (pixels: batch*channels*
 * height*width bytes, labels: batch floats, params: 3*batch ints already drawn -- overwrite them
 * to force offsets), then cct_corpus_submit starts the upload. */
int cct_corpus_stage(cct_corpus *c, unsigned char **pixels, float **labels, int **params);
int cct_corpus_submit(cct_corpus *c);
/* Device stage: the library's stream waits for the oldest batch in flight, then the transform
 * kernel writes images [batch][channels][out_rows][out_cols] and the labels are copied to
 * labels_dev [batch].  params_out (host, 3*batch ints, may be NULL) receives the crop parameters
 * that were used. */
int cct_corpus_consume(cct_corpus *c, float *images_dev, float *labels_dev, int *params_out);

/* ---- the file readers on their own (host only, no device needed) ----------------------------
 * What the reference gets from liblmdb (mdb_env_open / mdb_cursor_get MDB_FIRST, MDB_NEXT / mdb_env_stat,
 * src/parser/corpus.h:62-108, 170-226) and from protobuf (Datum::ParseFromArray, the binary Cube of
 * the mean file, :120-123, :231-238). */
typedef struct cct_lmdb cct_lmdb;
int cct_lmdb_open(cct_lmdb **out, const char *path); /* environment directory or its data.mdb */
int cct_lmdb_close(cct_lmdb *db);
size_t cct_lmdb_entries(cct_lmdb *db);               /* MDB_stat.ms_entries */
int cct_lmdb_rewind(cct_lmdb *db);                   /* next read is MDB_FIRST */
/* Next record in key order: returns 1 and fills the pointers (valid until close), 0 at the end of
 * the database, a negative value for a damaged file. */
int cct_lmdb_next(cct_lmdb *db, const void **key, size_t *key_size, const void **value, size_t *value_size);
/* Decodes a serialized Datum: dims = channels, height, width, label; *data / *data_size = the
 * `bytes data` field inside `value` (NULL / 0 if absent); *float_count = number of float_data values. */
int cct_datum_parse(const void *value, size_t size, int dims[4], const void **data, size_t *data_size,
                    size_t *float_count);
/* Reads a binary Cube message (the mean image): dims = num, channels, height, width; up to
 * `capacity` floats are written to `data`, *count receives the number the file holds. */
int cct_mean_read(const char *file, int dims[4], float *data, size_t capacity, size_t *count);

#ifdef __cplusplus
}
#endif
#endif /* CCT_CORPUS_H */
