/*
 * CPU oracle for the sparse_conv2d path.  TEST INFRASTRUCTURE ONLY: see the
 * header.  Plain C11; build with -ffp-contract=off so that every fused
 * multiply-add below is an explicit fmaf() and nothing else gets fused.
 */
#include "sparse_conv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* element helpers: dtype 0 = float, 1 = int8                               */
/* ------------------------------------------------------------------------ */
static inline size_t esize(int dtype) { return dtype == 0 ? 4u : 1u; }

static inline int is_nz(int dtype, const void* w, size_t i) {
  if (dtype == 0) return ((const float*)w)[i] != 0.0f;
  return ((const int8_t*)w)[i] != 0;
}

static inline void put(int dtype, void* dst, size_t di, const void* src,
                       size_t si) {
  if (dtype == 0)
    ((float*)dst)[di] = ((const float*)src)[si];
  else
    ((int8_t*)dst)[di] = ((const int8_t*)src)[si];
}

static inline void put_zero(int dtype, void* dst, size_t di) {
  if (dtype == 0)
    ((float*)dst)[di] = 0.0f;
  else
    ((int8_t*)dst)[di] = 0;
}

static inline int round_up4(int v) { return (v + 3) & ~3; }

/* ------------------------------------------------------------------------ */
/* counting passes                                                           */
/* ------------------------------------------------------------------------ */
int plo_count_zeros_pad4(int dtype, const void* w, int rows, int cols,
                         int* num_build_nonzeroes) {
  int padded = 0, real = 0;
  for (int r = 0; r < rows; ++r) {
    int n = 0;
    for (int c = 0; c < cols; ++c) n += is_nz(dtype, w, (size_t)r * cols + c);
    padded += round_up4(n);
    real += n;
  }
  *num_build_nonzeroes = padded;
  return rows * cols - real;
}

int plo_count_semi(int dtype, const void* w, int rows, int cols,
                   int need_rows_gt1, int* count_nonzeroes,
                   int* count_channels, int* count_blocks, int* flag_semi) {
  const int paired_rows = rows & ~1;
  long nnz_paired = 0, blocks2 = 0, nnz_tail = 0;
  /* The reference walks groups of four rows first and then a possible group
   * of two; the block-of-four count it also keeps is never used, so a walk
   * over row pairs yields the same three numbers. */
  for (int r = 0; r < paired_rows; r += 2) {
    for (int c = 0; c < cols; ++c) {
      int a = is_nz(dtype, w, (size_t)r * cols + c);
      int b = is_nz(dtype, w, (size_t)(r + 1) * cols + c);
      nnz_paired += a + b;
      blocks2 += (a | b);
    }
  }
  for (int r = paired_rows; r < rows; ++r)
    for (int c = 0; c < cols; ++c)
      nnz_tail += is_nz(dtype, w, (size_t)r * cols + c);

  *flag_semi = 0;
  *count_channels = rows;
  *count_nonzeroes = (int)(nnz_paired + nnz_tail);
  *count_blocks = (int)(nnz_paired + nnz_tail);
  int dense_enough = (nnz_paired * 5 >= blocks2 * 9);
  if (need_rows_gt1) dense_enough = dense_enough && (rows > 1);
  if (dense_enough) {
    *flag_semi = 1;
    *count_channels = rows / 2 + rows % 2;
    *count_nonzeroes = (int)(blocks2 * 2 + nnz_tail);
    *count_blocks = (int)(blocks2 + nnz_tail);
  }
  return rows * cols - *count_nonzeroes;
}

/* ------------------------------------------------------------------------ */
/* packers                                                                   */
/* ------------------------------------------------------------------------ */

/* Running-sum rewrite shared by the three layouts: entry (ends[r]-1) becomes
 * the sum of all raw entries up to and including itself, i.e. the byte
 * offset (from the start pointer) of the first entry of the next row.
 * `n_rows` row ends, indices are into diffs[]. */
static void rewrite_row_ends(int32_t* diffs, const uint32_t* ends,
                             int n_rows) {
  int32_t run = 0;
  uint32_t pos = 0;
  for (int r = 0; r < n_rows; ++r) {
    for (; pos < ends[r]; ++pos) run += diffs[pos];
    if (pos != 0) diffs[pos - 1] = run;
  }
}

int plo_pack_unpadded(int dtype, const void* w, int M, int K, int N,
                      void* nonzero_weights, uint32_t* oc_nonzeros,
                      int32_t* diffs) {
  const int step = (int)esize(dtype) * N; /* bytes between adjacent ICs */
  int first_ic = 0, last_ic = 0, seen = 0;
  uint32_t n = 0, d = 0;
  for (int r = 0; r < M; ++r) {
    for (int c = 0; c < K; ++c) {
      size_t i = (size_t)r * K + c;
      if (!is_nz(dtype, w, i)) continue;
      put(dtype, nonzero_weights, n, w, i);
      if (!seen)
        first_ic = c;
      else
        diffs[d++] = (c - last_ic) * step;
      seen = 1;
      last_ic = c;
      ++n;
    }
    oc_nonzeros[r] = n;
  }
  if (n) diffs[n - 1] = 0; /* the reference sums this slot before filling it */
  rewrite_row_ends(diffs, oc_nonzeros, M);
  if (seen) diffs[d] = (first_ic - last_ic) * step; /* wrap, written last */
  return first_ic;
}

int plo_pack_padded(int dtype, const void* w, int M, int K, int N,
                    void* nonzero_weights, uint32_t* oc_nonzeros,
                    int32_t* diffs) {
  const int step = (int)esize(dtype) * N;
  int first_ic = 0, last_ic = 0, seen = 0;
  uint32_t slot = 0; /* write position, always a multiple of 4 at row start */
  int32_t* pending = NULL; /* where the diff leading to the next nonzero goes */
  for (int r = 0; r < M; ++r) {
    uint32_t row_start = slot;
    for (int c = 0; c < K; ++c) {
      size_t i = (size_t)r * K + c;
      if (!is_nz(dtype, w, i)) continue;
      put(dtype, nonzero_weights, slot, w, i);
      if (!seen)
        first_ic = c;
      else
        *pending = (c - last_ic) * step;
      pending = &diffs[slot];
      seen = 1;
      last_ic = c;
      ++slot;
    }
    oc_nonzeros[r] = slot; /* end of the real entries of this row */
    uint32_t row_len = slot - row_start;
    for (uint32_t p = row_len; p < (uint32_t)round_up4((int)row_len); ++p) {
      put_zero(dtype, nonzero_weights, slot);
      diffs[slot] = 0;
      ++slot;
    }
  }
  /* here the wrap entry is part of the stream before the running sums */
  if (seen) *pending = (first_ic - last_ic) * step;
  rewrite_row_ends(diffs, oc_nonzeros, M);
  return first_ic;
}

int plo_pack_semi(int dtype, const void* w, int M, int K, int N,
                  void* nonzero_weights, uint32_t* oc_nonzeros,
                  int32_t* diffs) {
  const int step = (int)esize(dtype) * N;
  const int paired_rows = M & ~1;
  int first_ic = 0, last_ic = 0, seen = 0;
  uint32_t n = 0 /* weights */, e = 0 /* entries */, d = 0, g = 0 /* group */;
  for (int r = 0; r < paired_rows; r += 2) {
    for (int c = 0; c < K; ++c) {
      size_t i0 = (size_t)r * K + c, i1 = i0 + (size_t)K;
      if (!(is_nz(dtype, w, i0) | is_nz(dtype, w, i1))) continue;
      put(dtype, nonzero_weights, n++, w, i0);
      put(dtype, nonzero_weights, n++, w, i1);
      if (!seen)
        first_ic = c;
      else
        diffs[d++] = (c - last_ic) * step;
      seen = 1;
      last_ic = c;
      ++e;
    }
    oc_nonzeros[g++] = e;
  }
  for (int r = paired_rows; r < M; ++r) {
    for (int c = 0; c < K; ++c) {
      size_t i = (size_t)r * K + c;
      if (!is_nz(dtype, w, i)) continue;
      put(dtype, nonzero_weights, n++, w, i);
      if (!seen)
        first_ic = c;
      else
        diffs[d++] = (c - last_ic) * step;
      seen = 1;
      last_ic = c;
      ++e;
    }
    oc_nonzeros[g++] = e;
  }
  if (e) diffs[e - 1] = 0;
  rewrite_row_ends(diffs, oc_nonzeros, (int)g);
  if (seen) diffs[d] = (first_ic - last_ic) * step;
  return first_ic;
}

/* ------------------------------------------------------------------------ */
/* per-row start rules of the ARM math functions                             */
/* ------------------------------------------------------------------------ */
typedef struct row_span {
  uint32_t first; /* index of the first entry (weights and diffs)           */
  uint32_t count; /* number of real entries                                 */
  int64_t start;  /* byte offset of the first activation from the start ptr */
} row_span;

/* layout 0 unpadded / 2 semi groups: rows are back to back.
 * layout 1 padded: a row begins at the next multiple of four. */
static row_span span_of(int layout, const uint32_t* ends, const int32_t* diffs,
                        int g) {
  row_span s;
  if (g == 0) {
    s.first = 0;
    s.count = ends[0];
    s.start = 0;
    return s;
  }
  uint32_t prev = ends[g - 1];
  uint32_t pad = 0;
  if (layout == 1 && (prev & 3u)) pad = 4u - (prev & 3u);
  s.first = prev + pad;
  s.count = ends[g] - prev - pad;
  s.start = (prev == 0) ? 0 : diffs[prev - 1];
  return s;
}

int plo_decode(int dtype, int layout, const void* nonzero_weights,
               const uint32_t* oc_nonzeros, const int32_t* diffs,
               int first_ic, int M, int K, int N, void* dense_out) {
  const int64_t step = (int64_t)esize(dtype) * N;
  memset(dense_out, 0, (size_t)M * K * esize(dtype));
  const int pairs = (layout == 2) ? M / 2 : 0;
  const int groups = (layout == 2) ? pairs + (M & 1) : M;
  for (int g = 0; g < groups; ++g) {
    row_span s = span_of(layout, oc_nonzeros, diffs, g);
    int64_t off = s.start;
    const int is_pair = (layout == 2) && (g < pairs);
    for (uint32_t j = 0; j < s.count; ++j) {
      if (off % step) return -1;
      int64_t ic = first_ic + off / step;
      if (ic < 0 || ic >= K) return -1;
      if (layout == 2) {
        /* weights: 2 per entry for pairs; the odd tail row's weights start
         * at 2*ends[pairs-1] and are single */
        if (is_pair) {
          size_t wi = 2 * ((size_t)s.first + j);
          put(dtype, dense_out, (size_t)(2 * g) * K + ic, nonzero_weights, wi);
          put(dtype, dense_out, (size_t)(2 * g + 1) * K + ic, nonzero_weights,
              wi + 1);
        } else {
          size_t wi = 2 * (size_t)s.first + j;
          put(dtype, dense_out, (size_t)(2 * pairs) * K + ic, nonzero_weights,
              wi);
        }
      } else {
        put(dtype, dense_out, (size_t)g * K + ic, nonzero_weights,
            (size_t)s.first + j);
      }
      off += diffs[s.first + j];
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* epilogue                                                                  */
/* ------------------------------------------------------------------------ */
static inline float apply_act(float v, const plo_act* a, float hs_inv) {
  if (!a) return v;
  switch (a->type) {
    case PLO_ACT_RELU:
      return fmaxf(v, 0.0f);
    case PLO_ACT_RELU6:
      return fminf(fmaxf(v, 0.0f), a->relu6_coef);
    case PLO_ACT_LEAKY_RELU:
      return (v >= 0.0f) ? v : v * a->leaky_alpha;
    case PLO_ACT_HARD_SWISH: {
      float gate = fminf(fmaxf(v + a->hs_offset, 0.0f), a->hs_threshold);
      return (v * hs_inv) * gate;
    }
    default:
      return v;
  }
}

static inline float hs_inverse(const plo_act* a) {
  return (a && a->type == PLO_ACT_HARD_SWISH) ? (float)(1.0 / a->hs_scale)
                                              : 0.0f;
}

static inline int8_t to_int8_sat(float v) {
  v = fmaxf(v, -127.0f);
  float r = roundf(v); /* half away from zero */
  if (r > 127.0f) r = 127.0f;
  return (int8_t)(int)r;
}

/* ------------------------------------------------------------------------ */
/* SpMM walkers                                                              */
/* ------------------------------------------------------------------------ */
void plo_sparse_conv_fp32(const float* A, const float* x,
                          const int32_t* diffs, const uint32_t* ends,
                          const float* bias, float* out, int batch, int M,
                          int K, int N, int first_ic, int flag_semi,
                          const plo_act* act) {
  const float hs_inv = hs_inverse(act);
  const int layout = flag_semi ? 2 : 1;
  const int pairs = flag_semi ? M / 2 : 0;
  const int groups = flag_semi ? pairs + (M & 1) : M;
  for (int b = 0; b < batch; ++b) {
    const char* start = (const char*)(x + ((size_t)b * K + first_ic) * N);
    float* o = out + (size_t)b * M * N;
    for (int g = 0; g < groups; ++g) {
      row_span s = span_of(layout, ends, diffs, g);
      const int is_pair = flag_semi && g < pairs;
      const int row0 = flag_semi ? (is_pair ? 2 * g : 2 * pairs) : g;
      const float* w =
          flag_semi ? A + 2 * (size_t)s.first : A + (size_t)s.first;
      for (int p = 0; p < N; ++p) {
        float a0 = bias ? bias[row0] : 0.0f;
        float a1 = (is_pair && bias) ? bias[row0 + 1] : 0.0f;
        const char* ptr = start + s.start + (size_t)p * sizeof(float);
        for (uint32_t j = 0; j < s.count; ++j) {
          float xv = *(const float*)ptr;
          if (is_pair) {
            a0 = fmaf(xv, w[2 * j], a0);
            a1 = fmaf(xv, w[2 * j + 1], a1);
          } else {
            a0 = fmaf(xv, w[j], a0);
          }
          ptr += diffs[s.first + j];
        }
        o[(size_t)row0 * N + p] = apply_act(a0, act, hs_inv);
        if (is_pair) o[(size_t)(row0 + 1) * N + p] = apply_act(a1, act, hs_inv);
      }
    }
  }
}

/* ------------------------------------------------------------------------ */
/* fp16 path (IEEE binary16 on bit patterns; every operation rounds once,   */
/* to nearest even, like the NEON half-precision instructions)              */
/* ------------------------------------------------------------------------ */
static double h2d(uint16_t h) {
  const int sign = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  double v;
  if (e == 31)
    v = m ? NAN : INFINITY;
  else if (e == 0)
    v = ldexp((double)m, -24);
  else
    v = ldexp((double)(m + 1024), e - 25);
  return sign ? -v : v;
}

/* exact double -> binary16, round to nearest even */
static uint16_t d2h(double d) {
  uint16_t sign = signbit(d) ? 0x8000u : 0;
  if (isnan(d)) return (uint16_t)(sign | 0x7e00u);
  double a = fabs(d);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u); /* rounds to infinity */
  if (a < ldexp(1.0, -14)) {
    /* subnormal range: multiples of 2^-24; 1024 carries into the smallest
     * normal number by itself */
    return (uint16_t)(sign | (uint16_t)nearbyint(ldexp(a, 24)));
  }
  int e;
  double m = frexp(a, &e);               /* a = m * 2^e, m in [0.5, 1) */
  double q = nearbyint(ldexp(m, 11));    /* 1024 .. 2048 */
  if (q == 2048.0) {
    q = 1024.0;
    ++e;
  }
  /* value = q * 2^(e-11), biased exponent = e - 1 + 15 */
  return (uint16_t)(sign | (uint16_t)((e + 14) << 10) | ((uint16_t)q & 1023u));
}

uint16_t plo_f32_to_f16(float f) { return d2h((double)f); }
float plo_f16_to_f32(uint16_t h) { return (float)h2d(h); }

/* fused multiply-add: the product of two halves is exact in double; the sum
 * may not be, so it is rounded to odd first (error term from TwoSum), which
 * makes the final rounding to 11 bits the correctly rounded result */
static uint16_t h_fma(uint16_t a, uint16_t b, uint16_t c) {
  const double p = h2d(a) * h2d(b), cc = h2d(c);
  double s = p + cc;
  if (isfinite(s) && s != 0.0) {
    const double bb = s - p;
    const double err = (p - (s - bb)) + (cc - bb);
    if (err != 0.0) {
      uint64_t bits;
      memcpy(&bits, &s, 8);
      if ((bits & 1u) == 0) {
        /* one ulp towards the exact sum */
        if ((err > 0.0) == (s > 0.0))
          bits += 1;
        else
          bits -= 1;
        memcpy(&s, &bits, 8);
      }
    }
  }
  return d2h(s);
}
static uint16_t h_mul(uint16_t a, uint16_t b) { return d2h(h2d(a) * h2d(b)); }
static uint16_t h_add(uint16_t a, uint16_t b) { return d2h(h2d(a) + h2d(b)); }
static uint16_t h_max(uint16_t a, uint16_t b) { return h2d(a) >= h2d(b) ? a : b; }
static uint16_t h_min(uint16_t a, uint16_t b) { return h2d(a) <= h2d(b) ? a : b; }

void plo_fp32_to_fp16(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = plo_f32_to_f16(in[i]);
}
void plo_fp16_to_fp32(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = plo_f16_to_f32(in[i]);
}

typedef struct h_act {
  int type;
  uint16_t alpha; /* relu6 bound or leaky slope */
  uint16_t hs_offset, hs_inv_scale, hs_threshold;
} h_act;

/* reference: lite/backends/arm/math/fp16/sparse_conv_fp16.cc:1301-1325
 * (constants), :668-1173 (instruction order of the activations) */
static h_act make_h_act(const plo_act* act) {
  h_act a = {0, 0, 0, 0, 0};
  if (!act) return a;
  a.type = act->type;
  if (act->type == PLO_ACT_RELU6) a.alpha = plo_f32_to_f16(act->relu6_coef);
  if (act->type == PLO_ACT_LEAKY_RELU) a.alpha = plo_f32_to_f16(act->leaky_alpha);
  if (act->type == PLO_ACT_HARD_SWISH) {
    a.hs_offset = plo_f32_to_f16(act->hs_offset);
    a.hs_inv_scale = d2h(1.0 / (double)act->hs_scale);
    a.hs_threshold = plo_f32_to_f16(act->hs_threshold);
  }
  return a;
}

static uint16_t apply_h_act(uint16_t v, const h_act* a) {
  switch (a->type) {
    case PLO_ACT_RELU:
      return h_max(v, 0);
    case PLO_ACT_RELU6:
      return h_min(h_max(v, 0), a->alpha);
    case PLO_ACT_LEAKY_RELU:
      return h2d(v) >= 0.0 ? v : h_mul(v, a->alpha);
    case PLO_ACT_HARD_SWISH: {
      uint16_t t = h_add(v, a->hs_offset);
      uint16_t u = h_mul(v, a->hs_inv_scale);
      t = h_min(h_max(t, 0), a->hs_threshold);
      return h_mul(u, t);
    }
    default:
      return v;
  }
}

/* The three sparse tensors are those the pass makes for fp32 weights (rows
 * padded to four, or the semi layout); the kernel class converts weights and
 * bias to fp16 and halves the byte offsets
 * (lite/kernels/arm/sparse_conv_compute.cc:270-304); here the weights and the
 * bias arrive converted, the offsets as the pass wrote them. */
void plo_sparse_conv_fp16(const uint16_t* A, const uint16_t* x,
                          const int32_t* diffs, const uint32_t* ends,
                          const uint16_t* bias, uint16_t* out, int batch,
                          int M, int K, int N, int first_ic, int flag_semi,
                          const plo_act* act) {
  const h_act ha = make_h_act(act);
  const int layout = flag_semi ? 2 : 1;
  const int pairs = flag_semi ? M / 2 : 0;
  const int groups = flag_semi ? pairs + (M & 1) : M;
  for (int b = 0; b < batch; ++b) {
    const char* start = (const char*)(x + ((size_t)b * K + first_ic) * N);
    uint16_t* o = out + (size_t)b * M * N;
    for (int g = 0; g < groups; ++g) {
      row_span s = span_of(layout, ends, diffs, g);
      const int is_pair = flag_semi && g < pairs;
      const int row0 = flag_semi ? (is_pair ? 2 * g : 2 * pairs) : g;
      const uint16_t* w =
          flag_semi ? A + 2 * (size_t)s.first : A + (size_t)s.first;
      for (int p = 0; p < N; ++p) {
        uint16_t a0 = bias ? bias[row0] : 0;
        uint16_t a1 = (is_pair && bias) ? bias[row0 + 1] : 0;
        const char* ptr = start + s.start / 2 + (size_t)p * sizeof(uint16_t);
        for (uint32_t j = 0; j < s.count; ++j) {
          uint16_t xv;
          memcpy(&xv, ptr, 2);
          if (is_pair) {
            a0 = h_fma(xv, w[2 * j], a0);
            a1 = h_fma(xv, w[2 * j + 1], a1);
          } else {
            a0 = h_fma(xv, w[j], a0);
          }
          ptr += diffs[s.first + j] / 2;
        }
        o[(size_t)row0 * N + p] = apply_h_act(a0, &ha);
        if (is_pair) o[(size_t)(row0 + 1) * N + p] = apply_h_act(a1, &ha);
      }
    }
  }
}

/* int8 accumulation core: calls sink(row, p, acc) for every output */
typedef struct i8_sink {
  int kind; /* 0 raw acc, 1 fp32 out, 2 int8 out */
  void* out;
  const float* bias;
  const float* scale;
  const plo_act* act;
  float hs_inv;
  int N;
} i8_sink;

static inline void emit(const i8_sink* k, int row, int p, int32_t acc) {
  size_t idx = (size_t)row * k->N + p;
  if (k->kind == 0) {
    ((int32_t*)k->out)[idx] = acc;
    return;
  }
  float v = fmaf((float)acc, k->scale[row], k->bias ? k->bias[row] : 0.0f);
  v = apply_act(v, k->act, k->hs_inv);
  if (k->kind == 1)
    ((float*)k->out)[idx] = v;
  else
    ((int8_t*)k->out)[idx] = to_int8_sat(v);
}

static void walk_int8(const int8_t* A, const int8_t* x, const int32_t* diffs,
                      const uint32_t* ends, int batch, int M, int K, int N,
                      int first_ic, int flag_semi, i8_sink sink,
                      size_t out_elem) {
  const int layout = flag_semi ? 2 : 0;
  const int pairs = flag_semi ? M / 2 : 0;
  const int groups = flag_semi ? pairs + (M & 1) : M;
  char* out_base = (char*)sink.out;
  for (int b = 0; b < batch; ++b) {
    const int8_t* start = x + ((size_t)b * K + first_ic) * N;
    sink.out = out_base + (size_t)b * M * N * out_elem;
    for (int g = 0; g < groups; ++g) {
      row_span s = span_of(layout, ends, diffs, g);
      const int is_pair = flag_semi && g < pairs;
      const int row0 = flag_semi ? (is_pair ? 2 * g : 2 * pairs) : g;
      const int8_t* w =
          flag_semi ? A + 2 * (size_t)s.first : A + (size_t)s.first;
      for (int p = 0; p < N; ++p) {
        int32_t a0 = 0, a1 = 0;
        const int8_t* ptr = start + s.start + p;
        for (uint32_t j = 0; j < s.count; ++j) {
          int32_t xv = *ptr;
          if (is_pair) {
            a0 += xv * (int32_t)w[2 * j];
            a1 += xv * (int32_t)w[2 * j + 1];
          } else {
            a0 += xv * (int32_t)w[j];
          }
          ptr += diffs[s.first + j];
        }
        emit(&sink, row0, p, a0);
        if (is_pair) emit(&sink, row0 + 1, p, a1);
      }
    }
  }
}

void plo_sparse_conv_int8_fp32(const int8_t* A, const int8_t* x,
                               const int32_t* diffs, const uint32_t* ends,
                               const float* bias, const float* scale,
                               float* out, int batch, int M, int K, int N,
                               int first_ic, int flag_semi,
                               const plo_act* act) {
  i8_sink k = {1, out, bias, scale, act, hs_inverse(act), N};
  walk_int8(A, x, diffs, ends, batch, M, K, N, first_ic, flag_semi, k, 4);
}

void plo_sparse_conv_int8_int8(const int8_t* A, const int8_t* x,
                               const int32_t* diffs, const uint32_t* ends,
                               const float* bias, const float* scale,
                               int8_t* out, int batch, int M, int K, int N,
                               int first_ic, int flag_semi,
                               const plo_act* act) {
  i8_sink k = {2, out, bias, scale, act, hs_inverse(act), N};
  walk_int8(A, x, diffs, ends, batch, M, K, N, first_ic, flag_semi, k, 1);
}

void plo_sparse_conv_int8_acc(const int8_t* A, const int8_t* x,
                              const int32_t* diffs, const uint32_t* ends,
                              int32_t* acc_out, int batch, int M, int K,
                              int N, int first_ic, int flag_semi) {
  i8_sink k = {0, acc_out, NULL, NULL, NULL, 0.0f, N};
  walk_int8(A, x, diffs, ends, batch, M, K, N, first_ic, flag_semi, k, 4);
}

/* ------------------------------------------------------------------------ */
/* naive dense reference                                                     */
/* ------------------------------------------------------------------------ */
void plo_basic_gemm_f32(int m, int n, int k, const float* a, const float* b,
                        float* c, const float* bias, int flag_bias,
                        int flag_act, float six, float leaky_alpha,
                        float hs_scale, float hs_offset, float hs_threshold) {
  for (int i = 0; i < m; ++i) {
    const float bv = flag_bias ? bias[i] : 0.0f;
    for (int j = 0; j < n; ++j) {
      float sum = 0.0f;
      for (int l = 0; l < k; ++l) sum += a[(size_t)i * k + l] * b[(size_t)l * n + j];
      /* alpha = 1, beta = 0 with c pre-zeroed: 1*sum + 0*c + bias */
      float t = 1.0f * sum + 0.0f * 0.0f + bv;
      float r = t;
      if (flag_act == 1) {
        r = t > 0.0f ? t : 0.0f;
      } else if (flag_act == 2) {
        r = t > 0.0f ? t : 0.0f;
        r = r < six ? r : six;
      } else if (flag_act == 4) {
        r = t < 0.0f ? (float)(t * leaky_alpha) : t;
      } else if (flag_act == 10) {
        float t1 = t + hs_offset;
        if (t1 > 0.0f) {
          if (t1 < hs_threshold)
            r = (float)((double)(t1 * t) * 1.0 / (double)hs_scale);
          else
            r = (float)((double)(hs_threshold * t) * 1.0 / (double)hs_scale);
        } else {
          if (hs_threshold > 0.0f)
            r = 0.0f;
          else
            r = (float)((double)(hs_threshold * t) * 1.0 / (double)hs_scale);
        }
      }
      c[(size_t)i * n + j] = r;
    }
  }
}

void plo_fp32_to_int8(const float* in, int8_t* out, float scale, int64_t n) {
  const float inv = 1.0f / scale;
  for (int64_t i = 0; i < n; ++i) out[i] = to_int8_sat(in[i] * inv);
}

void plo_int8_to_fp32(const int8_t* in, float* out, float scale, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = (float)in[i] * scale;
}

/* ------------------------------------------------------------------------ */
/* kernel-class parameter merging                                            */
/* ------------------------------------------------------------------------ */
int plo_merge_params(int out_kind, int M, const float* weight_scale,
                     int n_scale, float input_scale, float output_scale,
                     const float* bias, float* merged_scale,
                     float* merged_bias, plo_act* act) {
  if (out_kind == 0) {
    if (bias && merged_bias) memcpy(merged_bias, bias, sizeof(float) * M);
    return 0;
  }
  if (n_scale != 1 && n_scale != M) return -1;
  for (int i = 0; i < M; ++i) {
    float ws = weight_scale[n_scale == 1 ? 0 : i];
    merged_scale[i] = (out_kind == 1) ? ws * input_scale
                                      : ws * input_scale / output_scale;
  }
  if (bias && merged_bias)
    for (int i = 0; i < M; ++i)
      merged_bias[i] = (out_kind == 2) ? bias[i] / output_scale : bias[i];
  if (out_kind == 2 && act) {
    if (act->type == PLO_ACT_RELU6) act->relu6_coef /= output_scale;
    if (act->type == PLO_ACT_LEAKY_RELU) act->leaky_alpha /= output_scale;
    if (act->type == PLO_ACT_HARD_SWISH) {
      act->hs_scale /= output_scale;
      act->hs_offset /= output_scale;
      act->hs_threshold /= output_scale;
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* dense per-image GEMM comparator                                           */
/* ------------------------------------------------------------------------ */
#define RB 8 /* output rows per register block */

static void dense_image_f32(const float* w, const float* x, const float* bias,
                            float* out, int M, int K, int N,
                            const plo_act* act, float hs_inv, int r0, int r1) {
  enum { NB = 256 };
  float acc[RB][NB];
  (void)M;
  for (int r = r0; r < r1; r += RB) {
    int rows = (r1 - r < RB) ? r1 - r : RB;
    for (int c0 = 0; c0 < N; c0 += NB) {
      int cols = (N - c0 < NB) ? N - c0 : NB;
      for (int i = 0; i < rows; ++i)
        for (int j = 0; j < cols; ++j) acc[i][j] = 0.0f;
      for (int l = 0; l < K; ++l) {
        const float* xr = x + (size_t)l * N + c0;
        for (int i = 0; i < rows; ++i) {
          float wv = w[(size_t)(r + i) * K + l];
#pragma omp simd
          for (int j = 0; j < cols; ++j) acc[i][j] += wv * xr[j];
        }
      }
      for (int i = 0; i < rows; ++i) {
        float bv = bias ? bias[r + i] : 0.0f;
        for (int j = 0; j < cols; ++j)
          out[(size_t)(r + i) * N + c0 + j] =
              apply_act(acc[i][j] + bv, act, hs_inv);
      }
    }
  }
}

static void dense_image_i8(const int8_t* w, const int8_t* x, const float* bias,
                           const float* scale, void* out, int out_int8, int M,
                           int K, int N, const plo_act* act, float hs_inv,
                           int r0, int r1) {
  enum { NB = 256 };
  int32_t acc[RB][NB];
  (void)M;
  for (int r = r0; r < r1; r += RB) {
    int rows = (r1 - r < RB) ? r1 - r : RB;
    for (int c0 = 0; c0 < N; c0 += NB) {
      int cols = (N - c0 < NB) ? N - c0 : NB;
      for (int i = 0; i < rows; ++i)
        for (int j = 0; j < cols; ++j) acc[i][j] = 0;
      for (int l = 0; l < K; ++l) {
        const int8_t* xr = x + (size_t)l * N + c0;
        for (int i = 0; i < rows; ++i) {
          int32_t wv = w[(size_t)(r + i) * K + l];
#pragma omp simd
          for (int j = 0; j < cols; ++j) acc[i][j] += wv * (int32_t)xr[j];
        }
      }
      for (int i = 0; i < rows; ++i) {
        float bv = bias ? bias[r + i] : 0.0f;
        float sv = scale[r + i];
        for (int j = 0; j < cols; ++j) {
          float v = apply_act(fmaf((float)acc[i][j], sv, bv), act, hs_inv);
          size_t idx = (size_t)(r + i) * N + c0 + j;
          if (out_int8)
            ((int8_t*)out)[idx] = to_int8_sat(v);
          else
            ((float*)out)[idx] = v;
        }
      }
    }
  }
}

int plo_dense_conv1x1(int out_kind, const void* w_dense, const void* x,
                      const float* bias, const float* scale, void* out,
                      int batch, int M, int K, int N, const plo_act* act,
                      int threads) {
  const float hs_inv = hs_inverse(act);
  /* split every image into row blocks so that small batches still use all
   * threads */
  const int blocks_per_image = (M + 63) / 64;
  const int tasks = batch * blocks_per_image;
  int used = 1;
#ifdef _OPENMP
  if (threads <= 0) threads = omp_get_max_threads();
  used = threads;
#else
  (void)threads;
#endif
#pragma omp parallel for schedule(dynamic) num_threads(used)
  for (int t = 0; t < tasks; ++t) {
    int b = t / blocks_per_image;
    int r0 = (t % blocks_per_image) * 64;
    int r1 = r0 + 64 < M ? r0 + 64 : M;
    if (out_kind == 0) {
      dense_image_f32((const float*)w_dense,
                      (const float*)x + (size_t)b * K * N, bias,
                      (float*)out + (size_t)b * M * N, M, K, N, act, hs_inv,
                      r0, r1);
    } else {
      size_t oe = (out_kind == 2) ? 1 : 4;
      dense_image_i8((const int8_t*)w_dense,
                     (const int8_t*)x + (size_t)b * K * N, bias, scale,
                     (char*)out + (size_t)b * M * N * oe, out_kind == 2, M, K,
                     N, act, hs_inv, r0, r1);
    }
  }
  return used;
}

/* ------------------------------------------------------------------------ */
/* int8 depthwise 3x3 convolution                                            */
/* ------------------------------------------------------------------------ */
/* Accumulators as the reference's naive conv_basic<int8_t, int> computes them
 * for group == channels (lite/tests/utils/naive_math_impl.h:395-519: zero
 * padding, out = (in + 2 pad - 3) / stride + 1), then the epilogue of the
 * ARM depthwise kernels (lite/backends/arm/math/conv_block_utils.h:3696-3753
 * cvt_kernel; the NEON bodies use fmla, :3888-3950): fmaf(acc, scale, bias),
 * activation - hard_swish there is (v * alpha) * min(max(v + offset, 0),
 * threshold) with alpha = hard_swish_scale, the scale MULTIPLIES - and for
 * int8 output max(v, -127), round half away from zero, saturate.
 * out_kind: 1 fp32, 2 int8, 3 raw int32 accumulators.
 * Pinned by tests/test_oracle_dwconv.py: accumulators against conv_basic from
 * the reference header (oracle/_ref) and against a numpy statement; the
 * epilogue pieces are those of the sparse convolution, pinned there. */
int plo_dwconv3x3_int8(const int8_t* x, const int8_t* w, const float* scale,
                       const float* bias, const plo_act* act, int out_kind,
                       int batch, int channels, int h, int wd, int stride,
                       int pad, void* out) {
  if (!x || !w || !out || batch < 0 || channels <= 0 || h <= 0 || wd <= 0)
    return -1;
  if ((stride != 1 && stride != 2) || (pad != 0 && pad != 1)) return -1;
  if (out_kind < 1 || out_kind > 3 || (out_kind != 3 && !scale)) return -1;
  if (h + 2 * pad < 3 || wd + 2 * pad < 3) return -1;
  const int oh = (h + 2 * pad - 3) / stride + 1;
  const int ow = (wd + 2 * pad - 3) / stride + 1;
  const float hs_mul = act ? act->hs_scale : 0.0f;
  for (int n = 0; n < batch; ++n)
    for (int c = 0; c < channels; ++c) {
      const int8_t* xp = x + ((size_t)n * channels + c) * h * wd;
      const int8_t* wp = w + (size_t)c * 9;
      const size_t obase = ((size_t)n * channels + c) * oh * ow;
      for (int oy = 0; oy < oh; ++oy)
        for (int ox = 0; ox < ow; ++ox) {
          int32_t acc = 0;
          for (int ky = 0; ky < 3; ++ky)
            for (int kx = 0; kx < 3; ++kx) {
              const int iy = oy * stride - pad + ky;
              const int ix = ox * stride - pad + kx;
              if (iy < 0 || iy >= h || ix < 0 || ix >= wd) continue;
              acc += (int32_t)xp[(size_t)iy * wd + ix] * (int32_t)wp[ky * 3 + kx];
            }
          const size_t o = obase + (size_t)oy * ow + ox;
          if (out_kind == 3) {
            ((int32_t*)out)[o] = acc;
            continue;
          }
          float v = fmaf((float)acc, scale[c], bias ? bias[c] : 0.0f);
          v = apply_act(v, act, hs_mul);
          if (out_kind == 1)
            ((float*)out)[o] = v;
          else
            ((int8_t*)out)[o] = to_int8_sat(v);
        }
    }
  return 0;
}
