/*
 * dgs_oracle.c -- CPU restatement of the reference's per-GPU hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is the checker the HIP
 * kernels are compared against (tests/, the smoke check) and the CPU baseline
 * timed by the benchmark.  Nothing in the shipped library links or calls it.
 *
 * Every function restates an algorithm of the upstream sources; citations are
 * file:line under the upstream tree.  What pins each function (beyond reading
 * the source) is listed next to it; the pins live in tests/test_oracle.py.
 *
 *   philox4x32_10        Random123 known-answer vectors (3 KATs)
 *   bounded draw         exhaustive check of the rejection rule on small n,
 *                        uniformity by counting
 *   store split          README demo ([100] int64, 200 B -> 25 device + 75 host)
 *                        and the invariants device+host == total, 0 -> all host
 *   gather               equals numpy fancy indexing for every split point
 *   split index          closed form row >= threshold/stride
 *   sample (deg <= k)    closed form: the CSC row itself
 *   sample (deg > k)     brute force on tiny rows: every k-subset equally often;
 *                        literal picks of the reference's cuRAND stream and of
 *                        DGL's CPU sampler: PARITY UNPINNED (neither can run here)
 *   unique / relabel     independent numpy computation (np.unique + first index)
 *   neg_log_u32          math.log on the same argument (<= 2 ulp), monotone
 *   weighted (deg > k)   brute force on tiny rows against the closed form of
 *                        successive sampling; equal weights -> uniform subsets;
 *                        zero weights lose every race
 *   weighted, replace    frequencies against w / sum(w); quanta and inclusive
 *                        sums against an independent numpy computation
 *                        (literal picks of the reference's cuRAND stream:
 *                        PARITY UNPINNED, as for the uniform sampler)
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -shared).
 */
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* Philox4x32-10 (Salmon et al., SC'11; constants as in Random123)           */
/* ------------------------------------------------------------------------ */

ORACLE_API void oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2],
                                     uint32_t out[4]) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  const uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)M0 * c0;
    uint64_t p1 = (uint64_t)M1 * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += W0; k1 += W1;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/*
 * Reduce a Philox block to [0, n), 1 <= n < 2^32: Lemire's multiply-shift with
 * rejection, consuming the four words in order; the last word is accepted
 * unconditionally (probability of getting there < (n / 2^32)^3).
 * Replaces `curand(&rng) % n` (src/cuda/rowwise_sampling.cu:81,128), which is
 * biased; documented deviation.
 */
ORACLE_API uint32_t oracle_bounded(const uint32_t w[4], uint32_t n) {
  uint64_t m = 0;
  for (int i = 0; i < 4; ++i) {
    m = (uint64_t)w[i] * n;
    uint32_t lo = (uint32_t)m;
    if (lo >= n) break;              /* cannot be in the rejection zone */
    uint32_t t = (uint32_t)(0u - n) % n; /* 2^32 mod n */
    if (lo >= t) break;
  }
  return (uint32_t)(m >> 32);
}

/* draw j of row r on (seed, stream): the "dgs-philox-1" contract */
static inline uint32_t draw_bounded(uint64_t seed, uint32_t stream, int64_t row,
                                    uint32_t j, uint32_t n) {
  uint32_t ctr[4] = {j, stream, (uint32_t)((uint64_t)row & 0xffffffffu),
                     (uint32_t)((uint64_t)row >> 32)};
  uint32_t key[2] = {(uint32_t)(seed & 0xffffffffu), (uint32_t)(seed >> 32)};
  uint32_t w[4];
  oracle_philox4x32_10(ctr, key, w);
  return oracle_bounded(w, n);
}

ORACLE_API uint32_t oracle_draw(uint64_t seed, uint32_t stream, int64_t row,
                                uint32_t j, uint32_t n) {
  return draw_bounded(seed, stream, row, j, n);
}

/* ------------------------------------------------------------------------ */
/* ChunkTensor split + element access                                        */
/* ------------------------------------------------------------------------ */

/*
 * src/chunk_tensor.cc:57-73 with num_partitions_ == world:
 *   device_elem_size = capacity / sizeof(dtype); threshold = device * world;
 *   if threshold > total: threshold = total, device = ceil(total / world);
 *   host = total - threshold.
 */
ORACLE_API void oracle_store_split(int64_t total, int64_t elem_bytes,
                                   int64_t capacity_bytes, int64_t world,
                                   int64_t* device_elems, int64_t* host_elems,
                                   int64_t* threshold) {
  int64_t dev = capacity_bytes / elem_bytes;
  int64_t thr = dev * world;
  if (thr > total) {
    thr = total;
    dev = (total + world - 1) / world;
  }
  *device_elems = dev;
  *host_elems = total - thr;
  *threshold = thr;
}

static inline int64_t load_int(const void* p, int64_t i, int bytes) {
  return bytes == 8 ? ((const int64_t*)p)[i] : (int64_t)((const int32_t*)p)[i];
}
static inline void store_int(void* p, int64_t i, int bytes, int64_t v) {
  if (bytes == 8) ((int64_t*)p)[i] = v; else ((int32_t*)p)[i] = (int32_t)v;
}

/* chunk_tensor_wrapper::At (src/chunk_tensor.h:33-42), one partition */
static inline const char* at_ptr(const char* dev, const char* host, int64_t thr,
                                 int64_t eb, int64_t i) {
  return i >= thr ? host + (i - thr) * eb : dev + i * eb;
}
static inline int64_t at_int(const void* dev, const void* host, int64_t thr,
                             int bytes, int64_t i) {
  return i >= thr ? load_int(host, i - thr, bytes) : load_int(dev, i, bytes);
}

/*
 * _IndexMemcpyKernel / _LocalIndexMemcpyKernel / _HostIndexMemcpyKernel
 * (src/cuda/index_with_chunk_tensor.cu:9-27, :110-128, :150-168):
 *   out[i*D + j] = At(index[i]*D + j)       tier 0
 *                  LocalAt(...) = dev[...]   tier 1 (src/chunk_tensor.h:44-47)
 *                  HostAt(...)  = host[e-thr] tier 2 (src/chunk_tensor.h:56-58)
 */
ORACLE_API void oracle_gather(const void* dev, const void* host, int64_t thr,
                              int64_t elem_bytes, int64_t row_elems,
                              const void* index, int index_bytes, int64_t n,
                              void* out, int tier) {
  const char* d = (const char*)dev;
  const char* h = (const char*)host;
  char* o = (char*)out;
#pragma omp parallel for schedule(static) if (n * row_elems > (1 << 16))
  for (int64_t i = 0; i < n; ++i) {
    int64_t pos = load_int(index, i, index_bytes);
    for (int64_t j = 0; j < row_elems; ++j) {
      int64_t e = pos * row_elems + j;
      const char* src;
      if (tier == 1) src = d + e * elem_bytes;
      else if (tier == 2) src = h + (e - thr) * elem_bytes;
      else src = at_ptr(d, h, thr, elem_bytes, e);
      memcpy(o + (i * row_elems + j) * elem_bytes, src, (size_t)elem_bytes);
    }
  }
}

/*
 * _GetSplitIndexMaskKernel + the three boolean-index compactions
 * (src/cuda/index_with_chunk_tensor.cu:55-108) at local_rank 0, one partition:
 * host iff id >= threshold/stride; local iff 0 <= id < device_elems/stride;
 * everything else "remote".  Order is preserved in each class.
 */
ORACLE_API void oracle_split_index(int64_t thr, int64_t device_elems,
                                   int64_t stride, const void* index,
                                   int index_bytes, int64_t n, void* out_local,
                                   void* out_remote, void* out_host,
                                   int64_t counts[3]) {
  int64_t nl = 0, nr = 0, nh = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t id = load_int(index, i, index_bytes);
    if (id >= thr / stride) store_int(out_host, nh++, index_bytes, id);
    else if (id >= 0 * device_elems / stride && id < 1 * device_elems / stride)
      store_int(out_local, nl++, index_bytes, id);
    else store_int(out_remote, nr++, index_bytes, id);
  }
  counts[0] = nl; counts[1] = nr; counts[2] = nh;
}

/* ------------------------------------------------------------------------ */
/* Row-wise uniform sampling                                                 */
/* ------------------------------------------------------------------------ */

/*
 * Per-seed pick counts and their exclusive scan
 * (src/cuda/rowwise_sampling_with_chunk_tensor.cu:136-153,
 *  src/cuda/rowwise_sampling.cu:13-40): replace ? (deg == 0 ? 0 : k) : min(deg, k).
 * sub_indptr has n_seeds + 1 entries; returns nnz = sub_indptr[n_seeds].
 */
ORACLE_API int64_t oracle_sample_counts(const void* seeds, int id_bytes,
                                        int64_t n_seeds, const void* ip_dev,
                                        const void* ip_host, int64_t ip_thr,
                                        int ptr_bytes, int64_t k, int replace,
                                        int64_t* sub_indptr) {
  int64_t acc = 0;
  for (int64_t i = 0; i < n_seeds; ++i) {
    int64_t row = load_int(seeds, i, id_bytes);
    int64_t b = at_int(ip_dev, ip_host, ip_thr, ptr_bytes, row);
    int64_t e = at_int(ip_dev, ip_host, ip_thr, ptr_bytes, row + 1);
    int64_t deg = e - b;
    int64_t c = replace ? (deg == 0 ? 0 : k) : (deg < k ? deg : k);
    sub_indptr[i] = acc;
    acc += c;
  }
  sub_indptr[n_seeds] = acc;
  return acc;
}

/*
 * COO fill (src/cuda/rowwise_sampling_with_chunk_tensor.cu:15-111):
 *   deg <= k, no replacement: the row in CSC order (:40-46) -- identical to the
 *     reference by construction;
 *   deg > k, no replacement: the reference runs a parallel Algorithm-R reservoir
 *     on a cuRAND stream (:48-69); restated here as the same DISTRIBUTION
 *     (uniform k-subset) drawn with Floyd's algorithm on the dgs-philox-1
 *     contract, which the HIP kernel reproduces bit for bit;
 *   replacement, deg > 0: k independent uniform picks (:100-108).
 */
ORACLE_API void oracle_sample_fill(const void* seeds, int id_bytes,
                                   int64_t n_seeds, const void* ip_dev,
                                   const void* ip_host, int64_t ip_thr,
                                   int ptr_bytes, const void* ix_dev,
                                   const void* ix_host, int64_t ix_thr,
                                   int64_t k, int replace, uint64_t rng_seed,
                                   uint32_t rng_stream,
                                   const int64_t* sub_indptr, void* out_rows,
                                   void* out_cols) {
#pragma omp parallel
  {
    uint32_t* picks = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)(k > 0 ? k : 1));
#pragma omp for schedule(dynamic, 64)
    for (int64_t i = 0; i < n_seeds; ++i) {
      int64_t row = load_int(seeds, i, id_bytes);
      int64_t b = at_int(ip_dev, ip_host, ip_thr, ptr_bytes, row);
      int64_t e = at_int(ip_dev, ip_host, ip_thr, ptr_bytes, row + 1);
      int64_t deg = e - b;
      int64_t off = sub_indptr[i];
      if (replace) {
        if (deg > 0) {
          for (int64_t j = 0; j < k; ++j) {
            uint32_t p = draw_bounded(rng_seed, rng_stream, row, (uint32_t)j,
                                      (uint32_t)deg);
            store_int(out_rows, off + j, id_bytes, row);
            store_int(out_cols, off + j, id_bytes,
                      at_int(ix_dev, ix_host, ix_thr, id_bytes, b + p));
          }
        }
      } else if (deg <= k) {
        for (int64_t j = 0; j < deg; ++j) {
          store_int(out_rows, off + j, id_bytes, row);
          store_int(out_cols, off + j, id_bytes,
                    at_int(ix_dev, ix_host, ix_thr, id_bytes, b + j));
        }
      } else {
        /* Floyd: step j considers position deg-k+j */
        for (int64_t j = 0; j < k; ++j) {
          uint32_t top = (uint32_t)(deg - k + j);
          uint32_t t = draw_bounded(rng_seed, rng_stream, row, (uint32_t)j, top + 1u);
          int dup = 0;
          for (int64_t q = 0; q < j; ++q) if (picks[q] == t) { dup = 1; break; }
          picks[j] = dup ? top : t;
        }
        for (int64_t j = 0; j < k; ++j) {
          store_int(out_rows, off + j, id_bytes, row);
          store_int(out_cols, off + j, id_bytes,
                    at_int(ix_dev, ix_host, ix_thr, id_bytes, b + picks[j]));
        }
      }
    }
    free(picks);
  }
}

/* ------------------------------------------------------------------------ */
/* Row-wise weighted sampling                                                */
/* ------------------------------------------------------------------------ */

/*
 * -ln((x + 0.5) / 2^32) from IEEE-754 basic operations only (exact integer
 * conversions, one division, explicitly fused multiply-adds), so that the HIP
 * kernel's copy of this routine returns the same bits.
 *   u = t / 2^33 with t = 2x + 1;  t = m * 2^e, m in [1, 2), folded to
 *   (sqrt(1/2), sqrt(2)];  ln m = 2 atanh(s), s = (m - 1) / (m + 1);
 *   atanh series to s^21 (|s| <= 0.1716: the next term is below 2^-60).
 */
ORACLE_API double oracle_neg_log_u32(uint32_t x) {
  static const double c[11] = {
      0x1.0000000000000p+0, 0x1.5555555555555p-2, 0x1.999999999999ap-3,
      0x1.2492492492492p-3, 0x1.c71c71c71c71cp-4, 0x1.745d1745d1746p-4,
      0x1.3b13b13b13b14p-4, 0x1.1111111111111p-4, 0x1.e1e1e1e1e1e1ep-5,
      0x1.af286bca1af28p-5, 0x1.8618618618618p-5};
  const double ln2 = 0x1.62e42fefa39efp-1, sqrt2 = 0x1.6a09e667f3bcdp+0;
  const uint64_t t = 2ull * x + 1ull;
  int e = 63 - __builtin_clzll(t);
  union { uint64_t u; double d; } scale;
  scale.u = (uint64_t)(1023 - e) << 52; /* 2^-e */
  double m = (double)t * scale.d;       /* exact */
  if (m > sqrt2) { m *= 0.5; ++e; }
  const double f = m - 1.0;             /* exact */
  const double s = f / (2.0 + f);
  const double z = s * s;
  double p = c[10];
  for (int i = 9; i >= 0; --i) p = __builtin_fma(p, z, c[i]);
  const double r = s * p;
  return __builtin_fma((double)(33 - e), ln2, -2.0 * r);
}

/* the four words of the Philox block that (row, j) names */
static inline void draw_words(uint64_t seed, uint32_t stream, int64_t row,
                              uint32_t j, uint32_t w[4]) {
  uint32_t ctr[4] = {j, stream, (uint32_t)((uint64_t)row & 0xffffffffu),
                     (uint32_t)((uint64_t)row >> 32)};
  uint32_t key[2] = {(uint32_t)(seed & 0xffffffffu), (uint32_t)(seed >> 32)};
  oracle_philox4x32_10(ctr, key, w);
}

/*
 * Race key of neighbour position p: E / w with E a unit exponential variate,
 * +inf for weights that are not > 0.  Keeping the k smallest keys is the
 * A-Res rule of the reference (k largest u^(1/w),
 * src/cuda/rowwise_sampling_probs.cu:102-118) in logarithms.
 * Position p uses word p & 3 of block 0x80000000 | (p >> 2).
 */
ORACLE_API double oracle_weighted_key(uint64_t seed, uint32_t stream, int64_t row,
                                      uint32_t p, float weight) {
  uint32_t w[4];
  draw_words(seed, stream, row, 0x80000000u | (p >> 2), w);
  const double e = oracle_neg_log_u32(w[p & 3]);
  const double wd = (double)weight;
  return wd > 0.0 ? e / wd : __builtin_inf();
}

/*
 * Integer share of a weight: floor(w * 2^(32 - E)) with 2^(E-1) <= row_max < 2^E,
 * so the largest weight of the row maps into [2^31, 2^32).  Scaling by a power
 * of two is exact: the shares, and with them every partial sum, are integers
 * that do not depend on the order of summation.  Weights that are not > 0 get
 * no share; when the largest weight is +inf only infinite weights get one.
 */
ORACLE_API uint64_t oracle_weight_quantum(float weight, float row_max) {
  if (!(weight > 0.0f) || !(row_max > 0.0f)) return 0;
  if (row_max > 3.4028234663852886e38f) return weight > 3.4028234663852886e38f ? 1 : 0;
  int e;
  (void)frexp((double)row_max, &e); /* row_max = f * 2^e, 0.5 <= f < 1 */
  return (uint64_t)ldexp((double)weight, 32 - e);
}

/* uniform in [0, n) from 64-bit words: Lemire's rule on (w0,w1), then (w2,w3)
 * accepted unconditionally */
ORACLE_API uint64_t oracle_bounded64(const uint32_t w[4], uint64_t n) {
  unsigned __int128 m = 0;
  for (int i = 0; i < 2; ++i) {
    const uint64_t x = (uint64_t)w[2 * i] | ((uint64_t)w[2 * i + 1] << 32);
    m = (unsigned __int128)x * n;
    const uint64_t lo = (uint64_t)m;
    if (lo >= n) break;
    if (lo >= (0ull - n) % n) break;
  }
  return (uint64_t)(m >> 64);
}

typedef struct { double key; uint32_t pos; } race_t;
static int race_cmp(const void* a, const void* b) {
  const race_t* x = (const race_t*)a; const race_t* y = (const race_t*)b;
  if (x->key < y->key) return -1;
  if (x->key > y->key) return 1;
  return x->pos < y->pos ? -1 : (x->pos > y->pos ? 1 : 0);
}

/*
 * Weighted COO fill (src/cuda/rowwise_sampling_probs.cu:54-216 and
 * rowwise_sampling_probs_with_chunk_tensor.cu:15-179); probs are float32, one
 * per edge, stored like `indices`.
 *   deg <= k, no replacement: the row in CSC order (:125-134);
 *   deg > k, no replacement: the k smallest race keys, ties by position, emitted
 *     in that order (the reference keeps the k largest u^(1/w) on a cuRAND
 *     stream: same distribution, different literal picks);
 *   replacement, deg > 0: k independent picks with P(i) = q_i / sum q, q_i the
 *     integer share floor(w_i * 2^(32-E)) for 2^(E-1) <= max w < 2^E (the
 *     reference scans float32 weights into a CDF and searches u * total,
 *     :176-206: same distribution up to 2^-31 of the largest weight); draw j is block 0x40000000 | j reduced to [0, sum q) and
 *     located with an upper bound on the inclusive sums; a row without any
 *     positive finite share picks its last neighbour, as the reference's
 *     clamped search does (:203-204).
 */
ORACLE_API void oracle_sample_fill_weighted(
    const void* seeds, int id_bytes, int64_t n_seeds, const void* ip_dev,
    const void* ip_host, int64_t ip_thr, int ptr_bytes, const void* ix_dev,
    const void* ix_host, int64_t ix_thr, const float* pr_dev, const float* pr_host,
    int64_t pr_thr, int64_t k, int replace, uint64_t rng_seed, uint32_t rng_stream,
    const int64_t* sub_indptr, void* out_rows, void* out_cols) {
#pragma omp parallel for schedule(dynamic, 16)
  for (int64_t i = 0; i < n_seeds; ++i) {
    int64_t row = load_int(seeds, i, id_bytes);
    int64_t b = at_int(ip_dev, ip_host, ip_thr, ptr_bytes, row);
    int64_t e = at_int(ip_dev, ip_host, ip_thr, ptr_bytes, row + 1);
    int64_t deg = e - b;
    int64_t off = sub_indptr[i];
#define PROB_AT(p) ((b + (p)) >= pr_thr ? pr_host[b + (p) - pr_thr] : pr_dev[b + (p)])
    if (replace) {
      if (deg == 0) continue;
      float wmax = 0.0f;
      for (int64_t p = 0; p < deg; ++p) { float w = PROB_AT(p); if (w > wmax) wmax = w; }
      uint64_t* cdf = (uint64_t*)malloc(sizeof(uint64_t) * (size_t)deg);
      uint64_t acc = 0;
      for (int64_t p = 0; p < deg; ++p) { acc += oracle_weight_quantum(PROB_AT(p), wmax); cdf[p] = acc; }
      for (int64_t j = 0; j < k; ++j) {
        int64_t pick = deg - 1;
        if (acc > 0) {
          uint32_t w[4];
          draw_words(rng_seed, rng_stream, row, 0x40000000u | (uint32_t)j, w);
          const uint64_t r = oracle_bounded64(w, acc);
          int64_t lo = 0, hi = deg - 1; /* first p with cdf[p] > r */
          while (lo < hi) { int64_t mid = (lo + hi) / 2; if (cdf[mid] > r) hi = mid; else lo = mid + 1; }
          pick = lo;
        }
        store_int(out_rows, off + j, id_bytes, row);
        store_int(out_cols, off + j, id_bytes, at_int(ix_dev, ix_host, ix_thr, id_bytes, b + pick));
      }
      free(cdf);
    } else if (deg <= k) {
      for (int64_t j = 0; j < deg; ++j) {
        store_int(out_rows, off + j, id_bytes, row);
        store_int(out_cols, off + j, id_bytes, at_int(ix_dev, ix_host, ix_thr, id_bytes, b + j));
      }
    } else {
      race_t* race = (race_t*)malloc(sizeof(race_t) * (size_t)deg);
      for (int64_t p = 0; p < deg; ++p) {
        race[p].key = oracle_weighted_key(rng_seed, rng_stream, row, (uint32_t)p, PROB_AT(p));
        race[p].pos = (uint32_t)p;
      }
      qsort(race, (size_t)deg, sizeof(race_t), race_cmp);
      for (int64_t j = 0; j < k; ++j) {
        store_int(out_rows, off + j, id_bytes, row);
        store_int(out_cols, off + j, id_bytes,
                  at_int(ix_dev, ix_host, ix_thr, id_bytes, b + race[j].pos));
      }
      free(race);
    }
#undef PROB_AT
  }
}

/* ------------------------------------------------------------------------ */
/* Unique + relabel                                                          */
/* ------------------------------------------------------------------------ */

/* _UpPower (src/cuda/tensor_reindex.cu:77-80), made safe for n == 0 */
static int64_t up_power(int64_t n) {
  int64_t c = 1;
  while (c <= n) c <<= 1; /* 1 << (floor(log2 n) + 1) for n >= 1 */
  return c;
}

/*
 * RelabelHashmap (src/cuda/tensor_reindex.cu:11-75) run sequentially:
 * identity hash key & (cap-1), probe pos = (pos + delta) & (cap-1) with
 * delta = 1, 2, 3, ...; key slot claimed once, stored value = min index.
 */
typedef struct { int64_t* key; int64_t* val; int64_t cap; } table_t;

static int64_t table_find_slot(const table_t* t, int64_t key, int claim) {
  uint64_t mask = (uint64_t)t->cap - 1;
  uint64_t pos = (uint64_t)key & mask;
  uint64_t delta = 1;
  for (;;) {
    if (t->key[pos] == key) return (int64_t)pos;
    if (t->key[pos] == -1) {
      if (!claim) return -1;
      t->key[pos] = key;
      return (int64_t)pos;
    }
    pos = (pos + delta) & mask;
    delta += 1;
  }
}

/*
 * Unique (src/cuda/tensor_reindex.cu:82-159) + Relabel (:161-180) +
 * TensorRelabelCUDA (:182-205) on already concatenated inputs:
 *   pass 1  insert key -> min index;
 *   pass 2  flag[i] = (stored index == i), exclusive scan;
 *   pass 3  unique[prefix[i]] = in[i], value[slot] = prefix[i] for flagged i;
 *   relabel out[i] = value[slot(in[i])], -1 when the key is absent.
 * Returns the number of unique ids.
 */
ORACLE_API int64_t oracle_unique_relabel(const void* mapping, int64_t n_map,
                                         const void* requiring, int64_t n_req,
                                         int id_bytes, void* unique_out,
                                         void* relabel_out) {
  table_t t;
  t.cap = up_power(n_map);
  t.key = (int64_t*)malloc(sizeof(int64_t) * (size_t)t.cap);
  t.val = (int64_t*)malloc(sizeof(int64_t) * (size_t)t.cap);
  int64_t* slot_local = (int64_t*)malloc(sizeof(int64_t) * (size_t)t.cap);
  for (int64_t i = 0; i < t.cap; ++i) { t.key[i] = -1; t.val[i] = INT64_MAX; slot_local[i] = -1; }
  for (int64_t i = 0; i < n_map; ++i) {
    int64_t s = table_find_slot(&t, load_int(mapping, i, id_bytes), 1);
    if (i < t.val[s]) t.val[s] = i;
  }
  int64_t tot = 0;
  for (int64_t i = 0; i < n_map; ++i) {
    int64_t key = load_int(mapping, i, id_bytes);
    int64_t s = table_find_slot(&t, key, 0);
    if (t.val[s] == i) {
      store_int(unique_out, tot, id_bytes, key);
      slot_local[s] = tot;
      ++tot;
    }
  }
  for (int64_t i = 0; i < n_req; ++i) {
    int64_t s = table_find_slot(&t, load_int(requiring, i, id_bytes), 0);
    store_int(relabel_out, i, id_bytes, s < 0 ? -1 : slot_local[s]);
  }
  free(t.key); free(t.val); free(slot_local);
  return tot;
}

/*
 * The same result on all host threads, for the TIMED CPU baseline only (the checker stays the
 * sequential restatement above, and tests/test_oracle.py holds this one against it): a fair
 * multi-core CPU figure needs all three legs on all cores, and upstream's table, an identity
 * hash filled by racing threads, has no sequential order a CPU port could keep to.
 * Keys are sharded by a mixing hash; thread t owns shard t, walks the whole mapping list in
 * order and inserts the keys of its shard into its own linear-probing table, so the first
 * insertion of a key carries its smallest index and no two threads write one table.  First
 * occurrences are flagged, counted per contiguous stretch of the list, and ranked in input
 * order, which makes the output independent of the sharding: it is the first-occurrence-ordered
 * unique list and its ranks, as above.
 */
static inline uint64_t mix64(uint64_t x) {
  x ^= x >> 33; x *= 0xff51afd7ed558ccdull; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ull; x ^= x >> 33;
  return x;
}

typedef struct { int64_t* key; int64_t* first; int64_t* rank; uint64_t mask; } shard_t;

static inline int64_t shard_find(const shard_t* sh, int64_t key, uint64_t h) {
  uint64_t pos = (h >> 8) & sh->mask;
  for (;;) {
    if (sh->key[pos] == key) return (int64_t)pos;
    if (sh->key[pos] == -1) return -1;
    pos = (pos + 1) & sh->mask;
  }
}

ORACLE_API int64_t oracle_unique_relabel_parallel(const void* mapping, int64_t n_map,
                                                  const void* requiring, int64_t n_req,
                                                  int id_bytes, void* unique_out,
                                                  void* relabel_out) {
  int n_threads = 1;
#pragma omp parallel
  {
#pragma omp single
    n_threads = omp_get_num_threads();
  }
  const int n_shards = n_threads;
  shard_t* shards = (shard_t*)malloc(sizeof(shard_t) * (size_t)n_shards);
  const int64_t cap = up_power(2 * (n_map / n_shards + 1) + 16);
  for (int t = 0; t < n_shards; ++t) {
    shards[t].key = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
    shards[t].first = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
    shards[t].rank = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap);
    shards[t].mask = (uint64_t)cap - 1;
  }
  unsigned char* flag = (unsigned char*)malloc((size_t)(n_map > 0 ? n_map : 1));
  int64_t* stretch_count = (int64_t*)calloc((size_t)n_threads + 1, sizeof(int64_t));
  int overfull = 0;
#pragma omp parallel num_threads(n_threads)
  {
    const int t = omp_get_thread_num();
    shard_t* mine = &shards[t];
    int64_t held = 0;
    for (int64_t i = 0; i < cap; ++i) { mine->key[i] = -1; mine->rank[i] = -1; }  /* (a lookup of -1 lands on an empty slot: rank -1) */
    /* pass 1: this thread's keys, in list order: the first insertion is the smallest index */
    for (int64_t i = 0; i < n_map; ++i) {
      const int64_t key = load_int(mapping, i, id_bytes);
      const uint64_t h = mix64((uint64_t)key);
      if ((int)(h % (uint64_t)n_shards) != t) continue;
      uint64_t pos = (h >> 8) & mine->mask;
      for (;;) {
        if (mine->key[pos] == key) break;
        if (mine->key[pos] == -1) {
          if (++held > cap - 1) { overfull = 1; break; }  /* cannot happen for a mixing hash; checked anyway */
          mine->key[pos] = key; mine->first[pos] = i; mine->rank[pos] = -1;
          break;
        }
        pos = (pos + 1) & mine->mask;
      }
      if (overfull) break;
    }
#pragma omp barrier
    /* pass 2: flags and counts per contiguous stretch of the list */
    const int64_t lo = n_map * t / n_threads, hi = n_map * (t + 1) / n_threads;
    int64_t c = 0;
    if (!overfull) {
      for (int64_t i = lo; i < hi; ++i) {
        const int64_t key = load_int(mapping, i, id_bytes);
        const uint64_t h = mix64((uint64_t)key);
        const shard_t* sh = &shards[h % (uint64_t)n_shards];
        const int64_t s = shard_find(sh, key, h);
        flag[i] = (unsigned char)(s >= 0 && sh->first[s] == i);
        c += flag[i];
      }
    }
    stretch_count[t + 1] = c;
#pragma omp barrier
#pragma omp single
    for (int q = 0; q < n_threads; ++q) stretch_count[q + 1] += stretch_count[q];
    /* pass 3: ranks in input order; every key is ranked by the one thread that holds its first index */
    int64_t r = stretch_count[t];
    if (!overfull) {
      for (int64_t i = lo; i < hi; ++i) {
        if (!flag[i]) continue;
        const int64_t key = load_int(mapping, i, id_bytes);
        const uint64_t h = mix64((uint64_t)key);
        shard_t* sh = &shards[h % (uint64_t)n_shards];
        sh->rank[shard_find(sh, key, h)] = r;
        store_int(unique_out, r, id_bytes, key);
        ++r;
      }
    }
#pragma omp barrier
    if (!overfull) {
#pragma omp for schedule(static)
      for (int64_t i = 0; i < n_req; ++i) {
        const int64_t key = load_int(requiring, i, id_bytes);
        const uint64_t h = mix64((uint64_t)key);
        const shard_t* sh = &shards[h % (uint64_t)n_shards];
        const int64_t s = shard_find(sh, key, h);
        store_int(relabel_out, i, id_bytes, s < 0 ? -1 : sh->rank[s]);
      }
    }
  }
  const int64_t tot = overfull ? -1 : stretch_count[n_threads];
  for (int t = 0; t < n_shards; ++t) { free(shards[t].key); free(shards[t].first); free(shards[t].rank); }
  free(shards); free(flag); free(stretch_count);
  return tot;
}
