/* Seeded synthetic CSR workloads: the five benchmark shapes and scaled-down
 * versions of them for tests.  Everything is drawn from one counter-based
 * generator, so any element can be produced independently (parallel
 * generation, identical results on every machine and thread count):
 *
 *   r(seed, stream, i) = splitmix64_mix((seed ^ stream*GOLDEN) + i*GOLDEN)
 *   uniform(-1,1)      = (r >> 11) * 2^-53 * 2 - 1, then cast to the value type
 *
 * Streams: 1 structure, 2 matrix values, 3 x, 4 y / C, 5 B, 6 per-row R-MAT bits.
 * All routines are two-call: with the output arrays NULL they only size the
 * result (return nnz), so the caller allocates exactly.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GOLDEN 0x9E3779B97F4A7C15ull

static inline uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

static inline uint64_t draw(uint64_t seed, uint64_t stream, uint64_t i) {
  return mix64((seed ^ (stream * GOLDEN)) + (i + 1) * GOLDEN);
}

static inline double unit(uint64_t r) { return (double)(r >> 11) * 0x1.0p-53; } /* [0,1) */

uint64_t wl_draw(uint64_t seed, uint64_t stream, uint64_t i) { return draw(seed, stream, i); }

/* out[i] = lo + (hi-lo)*u_i for i in [0, n) */
void wl_fill_uniform_f32(float *out, int64_t n, uint64_t seed, uint64_t stream, double lo, double hi) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = (float)(lo + (hi - lo) * unit(draw(seed, stream, (uint64_t)i)));
}
void wl_fill_uniform_f64(double *out, int64_t n, uint64_t seed, uint64_t stream, double lo, double hi) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = lo + (hi - lo) * unit(draw(seed, stream, (uint64_t)i));
}

static int cmp_i32(const void *a, const void *b) {
  const int32_t x = *(const int32_t *)a, y = *(const int32_t *)b;
  return (x > y) - (x < y);
}

static void insertion_sort_i32(int32_t *a, int n) {
  for (int i = 1; i < n; ++i) {
    const int32_t v = a[i];
    int j = i - 1;
    while (j >= 0 && a[j] > v) {
      a[j + 1] = a[j];
      --j;
    }
    a[j + 1] = v;
  }
}

/* ---- exactly k distinct sorted uniform columns per row (configs 3 and 5) ----
 * Row r draws columns from stream 1 at counters r*2k, r*2k+1, ...; an in-row
 * repeat is skipped and the next counter is drawn.  Should 2k draws not yield k
 * distinct columns (only possible when k is close to cols), the row is topped
 * up with the smallest unused columns so that the count is always exact. */
int64_t wl_uniform_rows(int32_t rows, int32_t cols, int32_t k, uint64_t seed, int32_t base,
                        int32_t *row_ptr, int32_t *col_ind) {
  if (k > cols) k = cols;
  const int64_t nnz = (int64_t)rows * k;
  if (!row_ptr || !col_ind) return nnz;
#pragma omp parallel
  {
    int32_t *tmp = (int32_t *)malloc(sizeof(int32_t) * (size_t)(k > 0 ? k : 1));
#pragma omp for schedule(static)
    for (int32_t r = 0; r < rows; ++r) {
      int got = 0;
      for (int c = 0; c < 2 * k && got < k; ++c) {
        const int32_t col = (int32_t)(draw(seed, 1, (uint64_t)r * (uint64_t)(2 * k) + (uint64_t)c) % (uint64_t)cols);
        int dup = 0;
        for (int t = 0; t < got; ++t) dup |= tmp[t] == col;
        if (!dup) tmp[got++] = col;
      }
      if (k <= 64) insertion_sort_i32(tmp, got);
      else qsort(tmp, (size_t)got, sizeof(int32_t), cmp_i32);
      for (int32_t cand = 0; got < k; ++cand) { /* top-up, keeps the row sorted at the end */
        int dup = 0;
        for (int t = 0; t < got; ++t) dup |= tmp[t] == cand;
        if (!dup) {
          tmp[got++] = cand;
          qsort(tmp, (size_t)got, sizeof(int32_t), cmp_i32);
        }
      }
      int32_t *dst = col_ind + (int64_t)r * k;
      for (int t = 0; t < k; ++t) dst[t] = tmp[t] + base;
      row_ptr[r] = (int32_t)((int64_t)r * k) + base;
    }
    free(tmp);
  }
  row_ptr[rows] = (int32_t)nnz + base;
  return nnz;
}

/* ---- 2-D 5-point Laplacian on an nx x ny grid, natural ordering (config 2) --- */
int64_t wl_laplace2d(int32_t nx, int32_t ny, int32_t base, int32_t *row_ptr, int32_t *col_ind,
                     double *val_f64, float *val_f32) {
  const int64_t rows = (int64_t)nx * ny;
  const int64_t nnz = 5 * rows - 2 * (int64_t)nx - 2 * (int64_t)ny;
  if (!row_ptr || !col_ind) return nnz;
  /* entries before row (ix, iy): 5 per row minus the missing neighbours */
#pragma omp parallel for schedule(static)
  for (int64_t iy = 0; iy < ny; ++iy) {
    /* offset of the first row of grid line iy */
    int64_t off = 0;
    if (iy > 0) {
      /* line 0 has (5nx - 2 - nx) entries, middle lines (5nx - 2), counted directly: */
      off = (5 * (int64_t)nx - 2) * iy - (int64_t)nx; /* line 0 lacks its nx "up" neighbours */
    }
    for (int64_t ix = 0; ix < nx; ++ix) {
      const int64_t row = iy * nx + ix;
      row_ptr[row] = (int32_t)off + base;
      int64_t p = off;
#define WL_PUT(c, v)                                 \
  do {                                               \
    col_ind[p] = (int32_t)(c) + base;                \
    if (val_f64) val_f64[p] = (v);                   \
    if (val_f32) val_f32[p] = (float)(v);            \
    ++p;                                             \
  } while (0)
      if (iy > 0) WL_PUT(row - nx, -1.0);
      if (ix > 0) WL_PUT(row - 1, -1.0);
      WL_PUT(row, 4.0);
      if (ix < nx - 1) WL_PUT(row + 1, -1.0);
      if (iy < ny - 1) WL_PUT(row + nx, -1.0);
#undef WL_PUT
      off = p;
    }
  }
  row_ptr[rows] = (int32_t)nnz + base;
  return nnz;
}

/* ---- power-law rows with R-MAT columns (config 4) ------------------------------
 * Row length L = min(max_len, floor(1/u)), u uniform in (0,1]: P(L >= k) = 1/k.
 * Columns: `levels` bit levels (cols = 2^levels); at each level the column bit
 * is 0 with probability a/(a+b) = 0.75 when the row bit is 0 and c/(c+d) =
 * 19/24 when it is 1 (R-MAT a=.57 b=.19 c=.19 d=.05 conditioned on the row).
 * Each level consumes 16 random bits.  L columns are drawn, sorted and
 * de-duplicated, so the realised row length is <= L and >= 1. */
static inline int32_t zipf_len(uint64_t seed, int32_t row, int32_t max_len) {
  const double u = 1.0 - unit(draw(seed, 1, (uint64_t)row)); /* (0,1] */
  const double l = floor(1.0 / u);
  return l >= (double)max_len ? max_len : (int32_t)l;
}

static inline int32_t rmat_col(uint64_t row_seed, int32_t row, int32_t levels, uint64_t t) {
  int32_t col = 0;
  uint64_t bits = 0;
  for (int l = 0; l < levels; ++l) {
    if ((l & 3) == 0) bits = draw(row_seed, 6, t * 8 + (uint64_t)(l >> 2));
    const uint32_t chunk = (uint32_t)(bits & 0xFFFFu);
    bits >>= 16;
    const int rbit = (row >> (levels - 1 - l)) & 1;
    const uint32_t thresh = rbit ? 51883u /* 19/24 * 65536 */ : 49152u /* 0.75 * 65536 */;
    const int cbit = chunk < thresh ? 0 : 1;
    col = (col << 1) | cbit;
  }
  return col;
}

static int rmat_row(uint64_t seed, int32_t row, int32_t levels, int32_t max_len, int32_t *buf) {
  const int32_t L = zipf_len(seed, row, max_len);
  const uint64_t row_seed = draw(seed, 1, ((uint64_t)1 << 40) + (uint64_t)row);
  for (int32_t t = 0; t < L; ++t) buf[t] = rmat_col(row_seed, row, levels, (uint64_t)t);
  if (L <= 32) insertion_sort_i32(buf, L);
  else qsort(buf, (size_t)L, sizeof(int32_t), cmp_i32);
  int n = 0;
  for (int32_t t = 0; t < L; ++t)
    if (t == 0 || buf[t] != buf[t - 1]) buf[n++] = buf[t];
  return n;
}

/* First call (col_ind == NULL): fills row_ptr (rows+1 entries) and returns nnz.
 * Second call: fills col_ind using the row_ptr of the first call. */
int64_t wl_powerlaw_rmat(int32_t levels, int32_t max_len, uint64_t seed, int32_t base,
                         int32_t *row_ptr, int32_t *col_ind) {
  const int32_t rows = (int32_t)1 << levels;
  if (!row_ptr) return -1;
  if (!col_ind) {
    int32_t *len = (int32_t *)malloc(sizeof(int32_t) * (size_t)rows);
#pragma omp parallel
    {
      int32_t *buf = (int32_t *)malloc(sizeof(int32_t) * (size_t)max_len);
#pragma omp for schedule(dynamic, 4096)
      for (int32_t r = 0; r < rows; ++r) len[r] = rmat_row(seed, r, levels, max_len, buf);
      free(buf);
    }
    int64_t acc = 0;
    for (int32_t r = 0; r < rows; ++r) {
      row_ptr[r] = (int32_t)acc + base;
      acc += len[r];
    }
    row_ptr[rows] = (int32_t)acc + base;
    free(len);
    return acc;
  }
#pragma omp parallel
  {
    int32_t *buf = (int32_t *)malloc(sizeof(int32_t) * (size_t)max_len);
#pragma omp for schedule(dynamic, 4096)
    for (int32_t r = 0; r < rows; ++r) {
      const int n = rmat_row(seed, r, levels, max_len, buf);
      int32_t *dst = col_ind + (row_ptr[r] - base);
      for (int t = 0; t < n; ++t) dst[t] = buf[t] + base;
    }
    free(buf);
  }
  return (int64_t)row_ptr[rows] - base;
}

/* ---- `draws` uniformly random (row, col) points, duplicates merged (config 1) ---
 * Mirrors how the reference's generator builds its test matrices
 * (tools/sparse_gen.c:63-98: random points, sorted, repeated coordinates dropped).
 * Returns nnz; arrays may be NULL on the sizing call (row_ptr must then be NULL too). */
typedef struct { int32_t r, c; } wl_point;
static int cmp_point(const void *a, const void *b) {
  const wl_point *p = (const wl_point *)a, *q = (const wl_point *)b;
  if (p->r != q->r) return (p->r > q->r) - (p->r < q->r);
  return (p->c > q->c) - (p->c < q->c);
}
int64_t wl_random_points(int32_t rows, int32_t cols, int64_t draws, uint64_t seed, int32_t base,
                         int32_t *row_ptr, int32_t *col_ind) {
  wl_point *pts = (wl_point *)malloc(sizeof(wl_point) * (size_t)(draws > 0 ? draws : 1));
  for (int64_t i = 0; i < draws; ++i) {
    pts[i].r = (int32_t)(draw(seed, 1, 2 * (uint64_t)i) % (uint64_t)rows);
    pts[i].c = (int32_t)(draw(seed, 1, 2 * (uint64_t)i + 1) % (uint64_t)cols);
  }
  qsort(pts, (size_t)draws, sizeof(wl_point), cmp_point);
  int64_t n = 0;
  for (int64_t i = 0; i < draws; ++i)
    if (i == 0 || pts[i].r != pts[i - 1].r || pts[i].c != pts[i - 1].c) pts[n++] = pts[i];
  if (row_ptr && col_ind) {
    int64_t p = 0;
    for (int32_t r = 0; r < rows; ++r) {
      row_ptr[r] = (int32_t)p + base;
      while (p < n && pts[p].r == r) {
        col_ind[p] = pts[p].c + base;
        ++p;
      }
    }
    row_ptr[rows] = (int32_t)n + base;
  }
  free(pts);
  return n;
}

/* 64-bit order-sensitive checksum of a byte range (FNV-1a over 8-byte words,
 * tail bytes folded in); used to pin generated arrays in fixtures. */
uint64_t wl_checksum(const void *data, int64_t nbytes) {
  const unsigned char *p = (const unsigned char *)data;
  uint64_t h = 0xcbf29ce484222325ull;
  int64_t i = 0;
  for (; i + 8 <= nbytes; i += 8) {
    uint64_t w;
    memcpy(&w, p + i, 8);
    h = (h ^ w) * 0x100000001b3ull;
  }
  for (; i < nbytes; ++i) h = (h ^ p[i]) * 0x100000001b3ull;
  return h;
}
