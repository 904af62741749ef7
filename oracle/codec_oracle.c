/*
 * CPU oracle for the BCTX / PPCX static-rANS weight codec.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the
 * reference algorithm, written for clarity, and is only ever linked or loaded
 * by the test-suite, by the smoke check and by the CPU-baseline leg of the
 * benchmark.  Nothing in the shipped package may call it.
 *
 * Every function names the reference lines it restates (paths relative to the
 * reference tree, GCR = context-runtime/georefine_context_runtime):
 *
 *   orc_split / orc_join        GCR/bitexact_context_ans.cpp:9-12, GCR/bitexact_context_codec.py:426
 *   orc_normalize               GCR/bitexact_context_ans.cpp:17-67
 *   orc_bcx_encode              GCR/bitexact_context_ans.cpp:75-109, 235-266
 *   orc_bcx_decode              GCR/bitexact_context_ans.cpp:110-160, 291-308   (full 65536-slot lookup)
 *   orc_pack6 / orc_unpack6     GCR/bitexact_context_ans.cpp:328-359
 *   orc_bcx_checkpoint          GCR/bitexact_context_gpu_index.cpp:21-137
 *   orc_p_encode / orc_p_decode GCR/bitexact_predictive_ans.cpp:10-11
 *   orc_ppcx_checkpoint         GCR/bitexact_predictive_gpu_index.cpp:9-37
 *
 * Parity pins (see tests/test_oracle_*.py): every function here is compared
 * byte for byte against the reference C++ compiled into oracle/_ref/ when that
 * library is present, against committed golden vectors produced from it, and
 * against closed forms (all 65536 words, numpy packbits, an independent
 * pure-Python rANS step decoder, the checkpoint resume invariant).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_SCALE 16u
#define ORC_TOTAL (1u << ORC_SCALE)
#define ORC_LOW (1u << 23)

/* ---- symbol algebra (GCR/bitexact_context_ans.cpp:9-12) ---- */
static uint32_t main_of(uint16_t w) { return (((w >> 7) & 255u) << 2) | ((w & 127u) >> 5); }
static uint32_t resid_of(uint16_t w) { return ((uint32_t)(w >> 15) << 5) | (w & 31u); }

void orc_split(const uint16_t *w, uint64_t n, uint16_t *main_sym, uint16_t *res_sym) {
  for (uint64_t i = 0; i < n; i++) {
    main_sym[i] = (uint16_t)main_of(w[i]);
    res_sym[i] = (uint16_t)resid_of(w[i]);
  }
}

/* inverse: GCR/bitexact_context_codec.py:426 */
void orc_join(const uint16_t *main_sym, const uint16_t *res_sym, uint64_t n, uint16_t *w) {
  for (uint64_t i = 0; i < n; i++) {
    uint32_t s = main_sym[i], r = res_sym[i];
    w[i] = (uint16_t)(((s >> 2) << 7) | ((s & 3u) << 5) | (r & 31u) | ((r >> 5) << 15));
  }
}

/* ---- frequency normalisation (GCR/bitexact_context_ans.cpp:17-67) ---- */
typedef struct {
  uint32_t sym;
  uint64_t rem;
} rem_t;

static int cmp_grow(const void *pa, const void *pb) { /* remainder descending, symbol ascending */
  const rem_t *a = (const rem_t *)pa, *b = (const rem_t *)pb;
  if (a->rem != b->rem) return a->rem > b->rem ? -1 : 1;
  return a->sym < b->sym ? -1 : (a->sym > b->sym);
}
static int cmp_shrink(const void *pa, const void *pb) { /* remainder ascending, symbol descending */
  const rem_t *a = (const rem_t *)pa, *b = (const rem_t *)pb;
  if (a->rem != b->rem) return a->rem < b->rem ? -1 : 1;
  return a->sym > b->sym ? -1 : (a->sym < b->sym);
}

/* returns 1 when the histogram was non-empty (out written), 0 when empty (out untouched) */
int orc_normalize(const uint64_t *count, uint32_t vocab, uint32_t *out) {
  uint64_t total = 0;
  uint32_t present = 0;
  for (uint32_t s = 0; s < vocab; s++) {
    total += count[s];
    present += count[s] != 0;
  }
  if (!total) return 0;
  rem_t *order = (rem_t *)malloc(sizeof(rem_t) * present);
  if (!order) return -1;
  int64_t sum = 0;
  uint32_t k = 0;
  for (uint32_t s = 0; s < vocab; s++) {
    if (!count[s]) {
      out[s] = 0;
      continue;
    }
    uint64_t scaled = count[s] * (uint64_t)ORC_TOTAL;
    uint32_t f = (uint32_t)(scaled / total);
    if (!f) f = 1;
    out[s] = f;
    sum += f;
    order[k].sym = s;
    order[k].rem = scaled % total;
    k++;
  }
  qsort(order, present, sizeof(rem_t), cmp_grow);
  if (sum < (int64_t)ORC_TOTAL) {
    uint32_t deficit = ORC_TOTAL - (uint32_t)sum;
    for (uint32_t j = 0; j < deficit; j++) out[order[j % present].sym]++;
  } else if (sum > (int64_t)ORC_TOTAL) {
    qsort(order, present, sizeof(rem_t), cmp_shrink);
    uint32_t excess = (uint32_t)sum - ORC_TOTAL;
    for (uint32_t j = 0; excess; j = (j + 1) % present) {
      uint32_t s = order[j].sym;
      if (out[s] > 1) {
        out[s]--;
        excess--;
      }
    }
  }
  free(order);
  return 1;
}

/* ---- generic rANS over a precomputed (value, context) sequence ---- */
typedef struct {
  uint8_t *p;
  size_t n, cap;
} bytes_t;
static int push(bytes_t *b, uint8_t v) {
  if (b->n == b->cap) {
    size_t cap = b->cap ? b->cap * 2 : 4096;
    uint8_t *q = (uint8_t *)realloc(b->p, cap);
    if (!q) return 0;
    b->p = q;
    b->cap = cap;
  }
  b->p[b->n++] = v;
  return 1;
}

/* Encode backwards so the decoder reads forwards (GCR/bitexact_context_ans.cpp:84-108).
 * value(i)/context(i) are produced by callbacks so BCTX and PPCX share the loop. */
typedef uint32_t (*index_fn)(const void *env, uint64_t i);

static int encode_core(uint64_t n, uint32_t vocab, uint32_t nctx, const uint32_t *freq, index_fn value,
                       index_fn context, const void *env, uint8_t **stream, size_t *stream_n) {
  uint32_t *cum = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)nctx * vocab);
  if (!cum) return 2;
  for (uint32_t c = 0; c < nctx; c++) {
    uint32_t run = 0;
    for (uint32_t s = 0; s < vocab; s++) {
      cum[(size_t)c * vocab + s] = run;
      run += freq[(size_t)c * vocab + s];
    }
  }
  bytes_t ren = {0, 0, 0};
  uint32_t state = ORC_LOW;
  for (uint64_t z = n; z-- > 0;) {
    uint32_t s = value(env, z), c = context(env, z);
    uint32_t f = freq[(size_t)c * vocab + s], start = cum[(size_t)c * vocab + s];
    if (!f) {
      free(cum);
      free(ren.p);
      return 3;
    }
    uint64_t limit = ((uint64_t)(ORC_LOW >> ORC_SCALE) << 8) * f;
    while (state >= limit) {
      if (!push(&ren, (uint8_t)(state & 255u))) {
        free(cum);
        free(ren.p);
        return 2;
      }
      state >>= 8;
    }
    state = ((state / f) << ORC_SCALE) + (state % f) + start;
  }
  free(cum);
  uint8_t *out = (uint8_t *)malloc(4 + ren.n);
  if (!out) {
    free(ren.p);
    return 2;
  }
  out[0] = (uint8_t)state;
  out[1] = (uint8_t)(state >> 8);
  out[2] = (uint8_t)(state >> 16);
  out[3] = (uint8_t)(state >> 24);
  for (size_t i = 0; i < ren.n; i++) out[4 + i] = ren.p[ren.n - 1 - i];
  free(ren.p);
  *stream = out;
  *stream_n = 4 + ren.n;
  return 0;
}

/* ---- BCTX ---- */
typedef struct {
  const uint16_t *w;
  uint32_t cols, nc, kind;
  const uint8_t *rc, *cc;
} bcx_env;
static uint32_t bcx_value(const void *e, uint64_t i) {
  const bcx_env *x = (const bcx_env *)e;
  return x->kind ? resid_of(x->w[i]) : main_of(x->w[i]);
}
static uint32_t bcx_context(const void *e, uint64_t i) { /* GCR/bitexact_context_ans.cpp:13-16 */
  const bcx_env *x = (const bcx_env *)e;
  if (x->kind) return main_of(x->w[i]);
  return (uint32_t)x->rc[i / x->cols] * x->nc + x->cc[i % x->cols];
}

/* count, normalise every context, encode (GCR/bitexact_context_ans.cpp:235-266) */
int orc_bcx_encode(const uint16_t *w, uint64_t n, uint32_t rows, uint32_t cols, const uint8_t *rc,
                   const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind, uint32_t *freq,
                   uint8_t **stream, size_t *stream_n) {
  uint32_t vocab = kind ? 64u : 1024u, nctx = kind ? 1024u : nr * nc;
  if (!w || !rc || !cc || !freq || !stream || !stream_n || n != (uint64_t)rows * cols) return 1;
  uint64_t *count = (uint64_t *)calloc((size_t)nctx * vocab, sizeof(uint64_t));
  if (!count) return 2;
  bcx_env env = {w, cols, nc, kind, rc, cc};
  for (uint64_t i = 0; i < n; i++) count[(size_t)bcx_context(&env, i) * vocab + bcx_value(&env, i)]++;
  for (uint32_t c = 0; c < nctx; c++)
    orc_normalize(count + (size_t)c * vocab, vocab, freq + (size_t)c * vocab);
  free(count);
  return encode_core(n, vocab, nctx, freq, bcx_value, bcx_context, &env, stream, stream_n);
}

/* Full-lookup decoder: a 65536-slot symbol table per context, exactly as the
 * reference default path does (GCR/bitexact_context_ans.cpp:110-160). */
int orc_bcx_decode(const uint8_t *stream, size_t bytes, uint64_t n, uint32_t rows, uint32_t cols,
                   const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                   const uint16_t *resctx, const uint32_t *freq, uint16_t *out) {
  uint32_t vocab = kind ? 64u : 1024u, nctx = kind ? 1024u : nr * nc;
  if (!stream || !rc || !cc || !freq || !out || !cols || !rows || kind > 1 || !nr || !nc || nr > 64 ||
      nc > 16 || (kind && !resctx) || n != (uint64_t)rows * cols)
    return 1;
  if (bytes < 4) return 2;
  uint32_t state = stream[0] | (uint32_t)stream[1] << 8 | (uint32_t)stream[2] << 16 | (uint32_t)stream[3] << 24;
  if (state < ORC_LOW) return 2;
  size_t ip = 4;
  uint32_t *cum = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)nctx * vocab);
  uint16_t *lut = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)nctx * ORC_TOTAL);
  int status = 2;
  if (!cum || !lut) {
    status = 3;
    goto done;
  }
  for (uint32_t c = 0; c < nctx; c++) {
    uint32_t run = 0;
    for (uint32_t s = 0; s < vocab; s++) {
      uint32_t f = freq[(size_t)c * vocab + s];
      cum[(size_t)c * vocab + s] = run;
      if (f) {
        if (f > ORC_TOTAL - run) goto done;
        for (uint32_t k = 0; k < f; k++) lut[(size_t)c * ORC_TOTAL + run + k] = (uint16_t)s;
        run += f;
      }
    }
    if (run && run != ORC_TOTAL) goto done;
  }
  for (uint64_t i = 0; i < n; i++) {
    uint32_t c = kind ? resctx[i] : (uint32_t)rc[i / cols] * nc + cc[i % cols];
    if (c >= nctx) goto done;
    uint32_t slot = state & (ORC_TOTAL - 1);
    uint32_t s = lut[(size_t)c * ORC_TOTAL + slot];
    uint32_t f = freq[(size_t)c * vocab + s], start = cum[(size_t)c * vocab + s];
    if (!f) goto done;
    out[i] = (uint16_t)s;
    state = f * (state >> ORC_SCALE) + (slot - start);
    while (state < ORC_LOW) {
      if (ip >= bytes) goto done;
      state = (state << 8) | stream[ip++];
    }
  }
  status = (ip == bytes && state == ORC_LOW) ? 0 : 2;
done:
  free(cum);
  free(lut);
  return status;
}

/* MSB-first 6-bit residual packing (GCR/bitexact_context_ans.cpp:328-345) */
int orc_pack6(const uint16_t *w, uint64_t n, uint8_t **out, size_t *bytes) {
  if (!w || !out || !bytes) return 1;
  size_t z = (size_t)((n * 6 + 7) / 8);
  uint8_t *p = (uint8_t *)calloc(z ? z : 1, 1);
  if (!p) return 2;
  uint64_t bit = 0;
  for (uint64_t i = 0; i < n; i++) {
    uint32_t v = resid_of(w[i]);
    for (int j = 5; j >= 0; j--, bit++)
      if ((v >> j) & 1u) p[bit >> 3] |= (uint8_t)(0x80u >> (bit & 7));
  }
  *out = p;
  *bytes = z;
  return 0;
}

/* (GCR/bitexact_context_ans.cpp:346-359): exact length, zero padding bits */
int orc_unpack6(const uint8_t *in, size_t bytes, uint64_t n, uint16_t *out) {
  if (!in || !out || bytes != (n * 6 + 7) / 8) return 1;
  unsigned tail = (unsigned)(n * 6 % 8);
  if (tail && (in[bytes - 1] & ((1u << (8 - tail)) - 1))) return 2;
  uint64_t bit = 0;
  for (uint64_t i = 0; i < n; i++) {
    uint32_t v = 0;
    for (int j = 0; j < 6; j++, bit++) v = (v << 1) | ((in[bit >> 3] >> (7 - (bit & 7))) & 1u);
    out[i] = (uint16_t)v;
  }
  return 0;
}

/* Validated walk that records (state, byte offset) before every stride-th symbol
 * (GCR/bitexact_context_gpu_index.cpp:21-137).  Outputs are written only on success. */
int orc_bcx_checkpoint(const uint8_t *stream, size_t bytes, uint64_t n, uint32_t rows, uint32_t cols,
                       const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                       const uint16_t *resctx, const uint32_t *freq, uint32_t stride, uint32_t *states,
                       uint32_t *offsets, uint16_t *out) {
  if (!stream || !rc || !cc || !freq || !states || !offsets || !out || !rows || !cols || !nr || !nc ||
      nr > 64 || nc > 16 || !stride || kind > 1 || (kind == 1 && !resctx) || n != (uint64_t)rows * cols ||
      !n || bytes < 4 || bytes > UINT32_MAX)
    return 1;
  uint32_t vocab = kind ? 64u : 1024u, nctx = kind ? 1024u : nr * nc;
  uint64_t count = (n - 1) / stride + 1;
  for (uint32_t r = 0; r < rows; r++)
    if (rc[r] >= nr) return 1;
  for (uint32_t c = 0; c < cols; c++)
    if (cc[c] >= nc) return 1;
  if (kind)
    for (uint64_t i = 0; i < n; i++)
      if (resctx[i] >= nctx) return 1;

  int status = 5;
  uint32_t *cum = (uint32_t *)malloc(sizeof(uint32_t) * (size_t)nctx * vocab);
  uint16_t *lut = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)nctx * ORC_TOTAL);
  uint8_t *live = (uint8_t *)calloc(nctx, 1);
  uint32_t *st = (uint32_t *)malloc(sizeof(uint32_t) * count);
  uint32_t *of = (uint32_t *)malloc(sizeof(uint32_t) * count);
  uint16_t *sym = (uint16_t *)malloc(sizeof(uint16_t) * n);
  if (!cum || !lut || !live || !st || !of || !sym) goto done;

  status = 2;
  for (uint32_t c = 0; c < nctx; c++) {
    uint64_t run = 0;
    for (uint32_t s = 0; s < vocab; s++) {
      uint32_t f = freq[(size_t)c * vocab + s];
      if (f > ORC_TOTAL || run + f > ORC_TOTAL) goto done;
      cum[(size_t)c * vocab + s] = (uint32_t)run;
      for (uint32_t k = 0; k < f; k++) lut[(size_t)c * ORC_TOTAL + run + k] = (uint16_t)s;
      run += f;
    }
    if (run && run != ORC_TOTAL) goto done;
    live[c] = run == ORC_TOTAL;
  }
  status = 3;
  uint32_t state = stream[0] | (uint32_t)stream[1] << 8 | (uint32_t)stream[2] << 16 | (uint32_t)stream[3] << 24;
  if (state < ORC_LOW) goto done;
  size_t ip = 4, slot_i = 0;
  uint64_t next_mark = 0;
  uint32_t row = 0, col = 0;
  for (uint64_t i = 0; i < n; i++) {
    if (i == next_mark) {
      st[slot_i] = state;
      of[slot_i] = (uint32_t)ip;
      slot_i++;
      next_mark += stride;
    }
    uint32_t c = kind ? resctx[i] : (uint32_t)rc[row] * nc + cc[col];
    if (c >= nctx || !live[c]) {
      status = 2;
      goto done;
    }
    uint32_t slot = state & (ORC_TOTAL - 1);
    uint32_t s = lut[(size_t)c * ORC_TOTAL + slot];
    uint32_t f = freq[(size_t)c * vocab + s], start = cum[(size_t)c * vocab + s];
    if (s >= vocab || !f || slot < start || slot - start >= f) {
      status = 2;
      goto done;
    }
    sym[i] = (uint16_t)s;
    uint64_t next = (uint64_t)f * (state >> ORC_SCALE) + (slot - start);
    if (next > UINT32_MAX) goto done;
    state = (uint32_t)next;
    while (state < ORC_LOW) {
      if (ip >= bytes) goto done;
      state = (state << 8) | stream[ip++];
    }
    if (++col == cols) {
      col = 0;
      row++;
    }
  }
  if (ip != bytes || state != ORC_LOW) goto done;
  memcpy(states, st, sizeof(uint32_t) * count);
  memcpy(offsets, of, sizeof(uint32_t) * count);
  memcpy(out, sym, sizeof(uint16_t) * n);
  status = 0;
done:
  free(cum);
  free(lut);
  free(live);
  free(st);
  free(of);
  free(sym);
  return status;
}

/* ---- PPCX generic context coder (GCR/bitexact_predictive_ans.cpp:10-11) ---- */
typedef struct {
  const uint16_t *v, *cx;
} p_env;
static uint32_t p_value(const void *e, uint64_t i) { return ((const p_env *)e)->v[i]; }
static uint32_t p_context(const void *e, uint64_t i) { return ((const p_env *)e)->cx[i]; }

int orc_p_encode(const uint16_t *v, const uint16_t *cx, uint64_t n, uint32_t nctx, uint32_t vocab,
                 uint32_t **freq_out, uint8_t **stream, size_t *stream_n) {
  if (!v || !cx || !n || n > 100000000u || !nctx || !vocab || vocab > ORC_TOTAL || !freq_out || !stream ||
      !stream_n)
    return 1;
  *freq_out = 0;
  *stream = 0;
  *stream_n = 0;
  size_t cells = (size_t)nctx * vocab;
  uint64_t *count = (uint64_t *)calloc(cells, sizeof(uint64_t));
  uint32_t *freq = (uint32_t *)calloc(cells, sizeof(uint32_t));
  if (!count || !freq) {
    free(count);
    free(freq);
    return 4;
  }
  for (uint64_t i = 0; i < n; i++) {
    if (cx[i] >= nctx || v[i] >= vocab) {
      free(count);
      free(freq);
      return 2;
    }
    count[(size_t)cx[i] * vocab + v[i]]++;
  }
  for (uint32_t c = 0; c < nctx; c++)
    orc_normalize(count + (size_t)c * vocab, vocab, freq + (size_t)c * vocab);
  free(count);
  p_env env = {v, cx};
  int rc = encode_core(n, vocab, nctx, freq, p_value, p_context, &env, stream, stream_n);
  if (rc) {
    free(freq);
    return 4;
  }
  *freq_out = freq;
  return 0;
}

/* upper_bound over an inclusive prefix table; status codes follow the reference */
int orc_p_decode(const uint8_t *st, size_t bytes, uint64_t n, const uint16_t *cx, uint32_t nctx,
                 uint32_t vocab, const uint32_t *freq, uint16_t *out) {
  if (!st || bytes < 4 || !cx || !freq || !out || !n || n > 100000000u || !nctx || !vocab ||
      vocab > ORC_TOTAL)
    return 1;
  uint32_t state = st[0] | (uint32_t)st[1] << 8 | (uint32_t)st[2] << 16 | (uint32_t)st[3] << 24;
  if (state < ORC_LOW) return 2;
  size_t ip = 4, width = (size_t)vocab + 1;
  uint32_t *pref = (uint32_t *)calloc((size_t)nctx * width, sizeof(uint32_t));
  if (!pref) return 10;
  int status = 0;
  for (uint32_t c = 0; c < nctx && !status; c++) {
    uint32_t *p = pref + (size_t)c * width;
    for (uint32_t s = 0; s < vocab; s++) {
      uint32_t f = freq[(size_t)c * vocab + s];
      if (f > ORC_TOTAL - p[s]) {
        status = 3;
        break;
      }
      p[s + 1] = p[s] + f;
    }
  }
  for (uint64_t i = 0; i < n && !status; i++) {
    uint32_t c = cx[i];
    if (c >= nctx) {
      status = 5;
      break;
    }
    const uint32_t *p = pref + (size_t)c * width;
    if (p[vocab] != ORC_TOTAL) {
      status = 4;
      break;
    }
    uint32_t slot = state & (ORC_TOTAL - 1);
    /* first index j in [1, vocab] with p[j] > slot */
    uint32_t lo = 1, hi = vocab + 1;
    while (lo < hi) {
      uint32_t mid = lo + (hi - lo) / 2;
      if (p[mid] > slot) hi = mid;
      else lo = mid + 1;
    }
    if (lo == vocab + 1) {
      status = 6;
      break;
    }
    uint32_t s = lo - 1, f = freq[(size_t)c * vocab + s];
    if (!f) {
      status = 7;
      break;
    }
    out[i] = (uint16_t)s;
    state = f * (state >> ORC_SCALE) + (slot - p[s]);
    while (state < ORC_LOW) {
      if (ip >= bytes) {
        status = 8;
        break;
      }
      state = (state << 8) | st[ip++];
    }
  }
  if (!status && !(ip == bytes && state == ORC_LOW)) status = 9;
  free(pref);
  return status;
}

/* linear-scan checkpoint walk (GCR/bitexact_predictive_gpu_index.cpp:9-37) */
int orc_ppcx_checkpoint(const uint8_t *stream, size_t bytes, uint64_t n, const uint16_t *ctx, uint32_t nctx,
                        uint32_t vocab, const uint32_t *freq, uint32_t stride, uint32_t *states,
                        uint32_t *offsets, uint16_t *symbols) {
  if (!stream || bytes < 4 || bytes > UINT32_MAX || !n || !ctx || !nctx || !vocab || vocab > ORC_TOTAL ||
      !freq || !stride || !states || !offsets || !symbols || n > 100000000u)
    return 1;
  for (uint32_t c = 0; c < nctx; c++) {
    uint64_t sum = 0;
    for (uint32_t s = 0; s < vocab; s++) {
      uint32_t f = freq[(size_t)c * vocab + s];
      if (f > ORC_TOTAL || sum + f > ORC_TOTAL) return 2;
      sum += f;
    }
    if (sum && sum != ORC_TOTAL) return 2;
  }
  uint32_t state = stream[0] | (uint32_t)stream[1] << 8 | (uint32_t)stream[2] << 16 | (uint32_t)stream[3] << 24;
  if (state < ORC_LOW) return 3;
  size_t ip = 4, count = (size_t)((n + stride - 1) / stride), k = 0;
  uint32_t *st = (uint32_t *)malloc(sizeof(uint32_t) * count);
  uint32_t *of = (uint32_t *)malloc(sizeof(uint32_t) * count);
  if (!st || !of) {
    free(st);
    free(of);
    return 6;
  }
  int status = 0;
  uint64_t mark = 0;
  for (uint64_t i = 0; i < n; i++) {
    if (ctx[i] >= nctx) {
      status = 4;
      break;
    }
    if (i == mark) {
      st[k] = state;
      of[k] = (uint32_t)ip;
      k++;
      mark += stride;
    }
    const uint32_t *f = freq + (size_t)ctx[i] * vocab;
    uint32_t slot = state & 65535u, start = 0, s = 0;
    for (; s < vocab; s++) {
      if (slot < start + f[s]) break;
      start += f[s];
    }
    if (s == vocab) {
      status = 5;
      break;
    }
    symbols[i] = (uint16_t)s;
    uint64_t next = (uint64_t)f[s] * (state >> 16) + (slot - start);
    if (next > UINT32_MAX) {
      status = 3;
      break;
    }
    state = (uint32_t)next;
    while (state < ORC_LOW) {
      if (ip >= bytes) {
        status = 3;
        break;
      }
      state = (state << 8) | stream[ip++];
    }
    if (status) break;
  }
  if (!status && (ip != bytes || state != ORC_LOW)) status = 3;
  if (!status) {
    memcpy(states, st, sizeof(uint32_t) * count);
    memcpy(offsets, of, sizeof(uint32_t) * count);
  }
  free(st);
  free(of);
  return status;
}

void orc_free(void *p) { free(p); }
