// Host side of the BF16 context codec: encoder, decoder and rANS checkpoint
// (frame-index) builder.  Exports the C ABI the reference binds with ctypes:
//
//   bcx_encode bcx_frequencies bcx_decode bcx_decode_compact bcx_free
//   bcx_pack6 bcx_unpack6                  (GCR/bitexact_context_ans.cpp:235-359)
//   bcx_checkpoint                         (GCR/bitexact_context_gpu_index.cpp:21-26)
//   p_encode p_decode p_free               (GCR/bitexact_predictive_ans.cpp:10-12)
//   ppcx_checkpoint ppcx_checkpoint_binary (GCR/bitexact_predictive_gpu_index.cpp:9-12, 38-41)
//
// with the same argument meaning, ownership and status codes.  The
// implementation is organised differently from the reference: one table
// object (`SymbolTables`) validates the frequency rows once and answers
// slot -> symbol queries through a 4096-entry coarse index followed by a short
// forward scan of the inclusive prefix sums, and one templated walker serves
// plain decoding and checkpoint recording for both wire formats.  No function
// keeps state between calls, so all of them may run concurrently.
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <limits>
#include <new>
#include <vector>

namespace {

constexpr uint32_t kScaleBits = 16;
constexpr uint32_t kTotal = 1u << kScaleBits;
constexpr uint32_t kLow = 1u << 23;
constexpr uint32_t kCoarseShift = 4;  // 4096 coarse buckets per context
constexpr uint32_t kCoarse = kTotal >> kCoarseShift;

inline uint32_t main_symbol(uint16_t w) { return (w >> 5) & 0x3FFu; }
inline uint32_t residual_symbol(uint16_t w) { return ((uint32_t)(w >> 15) << 5) | (w & 31u); }

enum class Walk { ok, bad_context, dead_context, bad_symbol, overflow, overrun, bad_tail, bad_head };

// Validated frequency rows plus the lookup structures derived from them.
class SymbolTables {
 public:
  enum class Check { ok, overflow, bad_sum };
  // A row is usable ("live") when it sums to the total.  Rows that overflow the
  // total are always an error; rows with any other sum are an error unless
  // `partial_rows_are_dead` (then they only fail when a symbol selects them).
  Check build(const uint32_t *freq, uint32_t nctx, uint32_t vocab, bool partial_rows_are_dead = false) {
    nctx_ = nctx;
    vocab_ = vocab;
    freq_ = freq;
    prefix_.assign((size_t)nctx * (vocab + 1), 0);
    live_.assign(nctx, 0);
    for (uint32_t c = 0; c < nctx; ++c) {
      uint32_t *p = prefix_.data() + (size_t)c * (vocab + 1);
      const uint32_t *f = freq + (size_t)c * vocab;
      uint64_t run = 0;
      for (uint32_t s = 0; s < vocab; ++s) {
        if (f[s] > kTotal || run + f[s] > kTotal) return Check::overflow;
        run += f[s];
        p[s + 1] = (uint32_t)run;
      }
      if (run != 0 && run != kTotal && !partial_rows_are_dead) return Check::bad_sum;
      live_[c] = run == kTotal;
    }
    {
      coarse_.assign((size_t)nctx * kCoarse, 0);
      for (uint32_t c = 0; c < nctx; ++c) {
        if (!live_[c]) continue;
        const uint32_t *p = prefix_.data() + (size_t)c * (vocab + 1);
        uint16_t *q = coarse_.data() + (size_t)c * kCoarse;
        uint32_t s = 0;
        for (uint32_t b = 0; b < kCoarse; ++b) {
          const uint32_t first = b << kCoarseShift;
          while (p[s + 1] <= first) ++s;
          q[b] = (uint16_t)s;
        }
      }
    }
    return Check::ok;
  }
  bool live(uint32_t c) const { return live_[c] != 0; }
  uint32_t nctx() const { return nctx_; }
  uint32_t vocab() const { return vocab_; }
  // symbol whose half-open slot range contains `slot`; context must be live
  inline uint32_t find(uint32_t c, uint32_t slot, uint32_t &start, uint32_t &f) const {
    const uint32_t *p = prefix_.data() + (size_t)c * (vocab_ + 1);
    uint32_t s = coarse_[(size_t)c * kCoarse + (slot >> kCoarseShift)];
    while (p[s + 1] <= slot) ++s;
    start = p[s];
    f = p[s + 1] - p[s];
    return s;
  }
  inline uint32_t start_of(uint32_t c, uint32_t s) const { return prefix_[(size_t)c * (vocab_ + 1) + s]; }

 private:
  uint32_t nctx_ = 0, vocab_ = 0;
  const uint32_t *freq_ = nullptr;
  std::vector<uint32_t> prefix_;
  std::vector<uint16_t> coarse_;
  std::vector<uint8_t> live_;
};

inline bool read_head(const uint8_t *s, size_t bytes, uint32_t &state) {
  if (bytes < 4) return false;
  state = (uint32_t)s[0] | (uint32_t)s[1] << 8 | (uint32_t)s[2] << 16 | (uint32_t)s[3] << 24;
  return state >= kLow;
}

// One forward pass over a stream.  `context(i)` yields the model row of symbol i,
// `mark(i, state, ip)` is called before symbol i is decoded.
template <class ContextFn, class MarkFn>
Walk walk_stream(const uint8_t *stream, size_t bytes, uint64_t n, const SymbolTables &t, ContextFn context,
                 MarkFn mark, uint16_t *out) {
  uint32_t state;
  if (!read_head(stream, bytes, state)) return Walk::bad_head;
  size_t ip = 4;
  for (uint64_t i = 0; i < n; ++i) {
    mark(i, state, ip);
    const uint32_t c = context(i);
    if (c >= t.nctx()) return Walk::bad_context;
    if (!t.live(c)) return Walk::dead_context;
    const uint32_t slot = state & (kTotal - 1);
    uint32_t start, f;
    const uint32_t s = t.find(c, slot, start, f);
    out[i] = (uint16_t)s;
    const uint64_t next = (uint64_t)f * (state >> kScaleBits) + (slot - start);
    if (next > std::numeric_limits<uint32_t>::max()) return Walk::overflow;
    state = (uint32_t)next;
    while (state < kLow) {
      if (ip >= bytes) return Walk::overrun;
      state = (state << 8) | stream[ip++];
    }
  }
  return (ip == bytes && state == kLow) ? Walk::ok : Walk::bad_tail;
}

struct NoMark {
  void operator()(uint64_t, uint32_t, size_t) const {}
};

struct StrideMark {
  uint32_t stride;
  uint32_t *states, *offsets;
  uint64_t next = 0;
  size_t k = 0;
  void operator()(uint64_t i, uint32_t state, size_t ip) {
    if (i == next) {
      states[k] = state;
      offsets[k] = (uint32_t)ip;
      ++k;
      next += stride;
    }
  }
};

// Row-major (row class, column class) context without a division per symbol.
struct GridContext {
  const uint8_t *rc, *cc;
  uint32_t cols, nc, row = 0, col = 0;
  uint32_t operator()(uint64_t) {
    const uint32_t c = (uint32_t)rc[row] * nc + cc[col];
    if (++col == cols) {
      col = 0;
      ++row;
    }
    return c;
  }
};
struct ArrayContext {
  const uint16_t *ctx;
  uint32_t operator()(uint64_t i) const { return ctx[i]; }
};

// ---- frequency normalisation: largest remainders, deterministic ties ----
// (GCR/bitexact_context_ans.cpp:17-67)
bool normalize_row(const uint64_t *count, uint32_t vocab, uint32_t *out) {
  uint64_t total = 0;
  for (uint32_t s = 0; s < vocab; ++s) total += count[s];
  if (!total) return false;
  struct Item {
    uint64_t rem;
    uint32_t sym;
  };
  std::vector<Item> items;
  int64_t sum = 0;
  for (uint32_t s = 0; s < vocab; ++s) {
    if (!count[s]) {
      out[s] = 0;
      continue;
    }
    const uint64_t scaled = count[s] << kScaleBits;
    const uint32_t f = std::max<uint32_t>(1u, (uint32_t)(scaled / total));
    out[s] = f;
    sum += f;
    items.push_back({scaled % total, s});
  }
  if (sum < (int64_t)kTotal) {
    std::sort(items.begin(), items.end(),
              [](const Item &a, const Item &b) { return a.rem != b.rem ? a.rem > b.rem : a.sym < b.sym; });
    const uint32_t deficit = kTotal - (uint32_t)sum;
    for (uint32_t j = 0; j < deficit; ++j) ++out[items[j % items.size()].sym];
  } else if (sum > (int64_t)kTotal) {
    std::sort(items.begin(), items.end(),
              [](const Item &a, const Item &b) { return a.rem != b.rem ? a.rem < b.rem : a.sym > b.sym; });
    uint32_t excess = (uint32_t)sum - kTotal;
    for (size_t j = 0; excess; j = (j + 1) % items.size())
      if (out[items[j].sym] > 1) {
        --out[items[j].sym];
        --excess;
      }
  }
  return true;
}

// ---- encoder: symbols are pushed last-to-first so decoding runs forward ----
// (GCR/bitexact_context_ans.cpp:84-108)
template <class ValueFn, class ContextFn>
bool encode_stream(uint64_t n, const uint32_t *freq, uint32_t nctx, uint32_t vocab, ValueFn value,
                   ContextFn context, std::vector<uint8_t> &out) {
  // start | freq packed per (context, symbol); freq needs 17 bits
  std::vector<uint64_t> cell((size_t)nctx * vocab);
  for (uint32_t c = 0; c < nctx; ++c) {
    uint32_t run = 0;
    for (uint32_t s = 0; s < vocab; ++s) {
      const uint32_t f = freq[(size_t)c * vocab + s];
      cell[(size_t)c * vocab + s] = (uint64_t)run << 32 | f;
      run += f;
    }
  }
  std::vector<uint8_t> tail;
  tail.reserve((size_t)(n / 2) + 16);
  uint32_t state = kLow;
  for (uint64_t i = n; i-- > 0;) {
    const uint64_t e = cell[(size_t)context(i) * vocab + value(i)];
    const uint32_t f = (uint32_t)e, start = (uint32_t)(e >> 32);
    if (!f) return false;
    const uint64_t limit = (uint64_t)((kLow >> kScaleBits) << 8) * f;
    while (state >= limit) {
      tail.push_back((uint8_t)state);
      state >>= 8;
    }
    state = ((state / f) << kScaleBits) + state % f + start;
  }
  out.resize(4 + tail.size());
  out[0] = (uint8_t)state;
  out[1] = (uint8_t)(state >> 8);
  out[2] = (uint8_t)(state >> 16);
  out[3] = (uint8_t)(state >> 24);
  std::reverse_copy(tail.begin(), tail.end(), out.begin() + 4);
  return true;
}

struct BcxShape {
  uint32_t vocab, nctx;
};
inline BcxShape bcx_shape(uint32_t kind, uint32_t nr, uint32_t nc) {
  return kind ? BcxShape{64u, 1024u} : BcxShape{1024u, nr * nc};
}

// histogram + normalisation shared by bcx_encode and bcx_frequencies
void bcx_count_and_normalize(const uint16_t *w, uint64_t n, uint32_t cols, const uint8_t *rc, const uint8_t *cc,
                             uint32_t nc, uint32_t kind, BcxShape sh, uint32_t *freq) {
  std::vector<uint64_t> hist((size_t)sh.nctx * sh.vocab);
  if (kind) {
    for (uint64_t i = 0; i < n; ++i) ++hist[(size_t)main_symbol(w[i]) * 64 + residual_symbol(w[i])];
  } else {
    GridContext g{rc, cc, cols, nc};
    for (uint64_t i = 0; i < n; ++i) ++hist[(size_t)g(i) * 1024 + main_symbol(w[i])];
  }
  for (uint32_t c = 0; c < sh.nctx; ++c)
    normalize_row(hist.data() + (size_t)c * sh.vocab, sh.vocab, freq + (size_t)c * sh.vocab);
}

int bcx_decode_any(const uint8_t *stream, size_t bytes, uint64_t n, uint32_t rows, uint32_t cols,
                   const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                   const uint16_t *resctx, const uint32_t *freq, uint16_t *out) {
  if (!stream || !rc || !cc || !freq || !out || !cols || !rows || kind > 1 || !nr || !nc || nr > 64 ||
      nc > 16 || (kind && !resctx) || n != (uint64_t)rows * cols)
    return 1;
  const BcxShape sh = bcx_shape(kind, nr, nc);
  SymbolTables t;
  // the reference bounds each frequency by the room left in its row
  if (t.build(freq, sh.nctx, sh.vocab) != SymbolTables::Check::ok) return 2;
  Walk w = kind ? walk_stream(stream, bytes, n, t, ArrayContext{resctx}, NoMark{}, out)
                : walk_stream(stream, bytes, n, t, GridContext{rc, cc, cols, nc}, NoMark{}, out);
  return w == Walk::ok ? 0 : 2;
}

template <class Fn>
int guarded(Fn fn, int on_alloc, int on_other) {
  try {
    return fn();
  } catch (const std::bad_alloc &) {
    return on_alloc;
  } catch (...) {
    return on_other;
  }
}

}  // namespace

extern "C" {

int bcx_encode(const uint16_t *w, uint64_t n, uint32_t rows, uint32_t cols, const uint8_t *rc,
               const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind, uint32_t *freq, uint8_t **stream,
               size_t *stream_n) {
  return guarded(
      [&]() -> int {
        if (!w || !rc || !cc || !freq || !stream || !stream_n || n != (uint64_t)rows * cols) return 1;
        const BcxShape sh = bcx_shape(kind, nr, nc);
        bcx_count_and_normalize(w, n, cols, rc, cc, nc, kind, sh, freq);
        std::vector<uint8_t> bytes;
        bool ok;
        if (kind) {
          ok = encode_stream(
              n, freq, sh.nctx, sh.vocab, [&](uint64_t i) { return residual_symbol(w[i]); },
              [&](uint64_t i) { return main_symbol(w[i]); }, bytes);
        } else {
          ok = encode_stream(
              n, freq, sh.nctx, sh.vocab, [&](uint64_t i) { return main_symbol(w[i]); },
              [&](uint64_t i) { return (uint32_t)rc[i / cols] * nc + cc[i % cols]; }, bytes);
        }
        if (!ok) return 3;
        auto *p = (uint8_t *)std::malloc(bytes.size());
        if (!p) return 2;
        std::memcpy(p, bytes.data(), bytes.size());
        *stream = p;
        *stream_n = bytes.size();
        return 0;
      },
      3, 3);
}

int bcx_frequencies(const uint16_t *w, uint64_t n, uint32_t rows, uint32_t cols, const uint8_t *rc,
                    const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind, uint32_t *freq) {
  return guarded(
      [&]() -> int {
        if (!w || !rc || !cc || !freq || n != (uint64_t)rows * cols) return 1;
        bcx_count_and_normalize(w, n, cols, rc, cc, nc, kind, bcx_shape(kind, nr, nc), freq);
        return 0;
      },
      3, 3);
}

int bcx_decode(const uint8_t *stream, size_t bytes, uint64_t n, uint32_t rows, uint32_t cols,
               const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
               const uint16_t *resctx, const uint32_t *freq, uint16_t *out) {
  return guarded([&] { return bcx_decode_any(stream, bytes, n, rows, cols, rc, cc, nr, nc, kind, resctx, freq, out); },
                 3, 3);
}

// Same lookup structure serves both entry points; the reference keeps two
// decoders whose results are required to be identical.
int bcx_decode_compact(const uint8_t *stream, size_t bytes, uint64_t n, uint32_t rows, uint32_t cols,
                       const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                       const uint16_t *resctx, const uint32_t *freq, uint16_t *out) {
  return guarded([&] { return bcx_decode_any(stream, bytes, n, rows, cols, rc, cc, nr, nc, kind, resctx, freq, out); },
                 3, 3);
}

void bcx_free(void *p) { std::free(p); }

// 6-bit residuals, most significant bit first; four symbols fill three bytes.
int bcx_pack6(const uint16_t *w, uint64_t n, uint8_t **out, size_t *bytes) {
  if (!w || !out || !bytes) return 1;
  const size_t z = (size_t)((n * 6 + 7) / 8);
  auto *p = (uint8_t *)std::calloc(z ? z : 1, 1);
  if (!p) return 2;
  uint64_t i = 0;
  uint8_t *q = p;
  for (; i + 4 <= n; i += 4, q += 3) {
    const uint32_t v = residual_symbol(w[i]) << 18 | residual_symbol(w[i + 1]) << 12 |
                       residual_symbol(w[i + 2]) << 6 | residual_symbol(w[i + 3]);
    q[0] = (uint8_t)(v >> 16);
    q[1] = (uint8_t)(v >> 8);
    q[2] = (uint8_t)v;
  }
  if (i < n) {
    uint32_t v = 0;
    const unsigned left = (unsigned)(n - i);
    for (unsigned k = 0; k < left; ++k) v |= residual_symbol(w[i + k]) << (18 - 6 * k);
    const unsigned nb = (left * 6 + 7) / 8;
    for (unsigned k = 0; k < nb; ++k) q[k] = (uint8_t)(v >> (16 - 8 * k));
  }
  *out = p;
  *bytes = z;
  return 0;
}

int bcx_unpack6(const uint8_t *in, size_t bytes, uint64_t n, uint16_t *out) {
  if (!in || !out || bytes != (n * 6 + 7) / 8) return 1;
  const unsigned tail_bits = (unsigned)(n * 6 % 8);
  if (tail_bits && (in[bytes - 1] & ((1u << (8 - tail_bits)) - 1))) return 2;
  uint64_t i = 0;
  const uint8_t *q = in;
  for (; i + 4 <= n; i += 4, q += 3) {
    const uint32_t v = (uint32_t)q[0] << 16 | (uint32_t)q[1] << 8 | q[2];
    out[i] = (uint16_t)(v >> 18);
    out[i + 1] = (uint16_t)((v >> 12) & 63);
    out[i + 2] = (uint16_t)((v >> 6) & 63);
    out[i + 3] = (uint16_t)(v & 63);
  }
  if (i < n) {
    const unsigned left = (unsigned)(n - i), nb = (left * 6 + 7) / 8;
    uint32_t v = 0;
    for (unsigned k = 0; k < nb; ++k) v |= (uint32_t)q[k] << (16 - 8 * k);
    for (unsigned k = 0; k < left; ++k) out[i + k] = (uint16_t)((v >> (18 - 6 * k)) & 63);
  }
  return 0;
}

int bcx_checkpoint(const uint8_t *stream, size_t stream_bytes, uint64_t n, uint32_t rows, uint32_t cols,
                   const uint8_t *rc, const uint8_t *cc, uint32_t nr, uint32_t nc, uint32_t kind,
                   const uint16_t *resctx, const uint32_t *freq, uint32_t stride, uint32_t *states,
                   uint32_t *offsets, uint16_t *out) {
  return guarded(
      [&]() -> int {
        if (!stream || !rc || !cc || !freq || !states || !offsets || !out || !rows || !cols || !nr || !nc ||
            nr > 64 || nc > 16 || !stride || kind > 1 || (kind == 1 && !resctx) ||
            n != (uint64_t)rows * (uint64_t)cols || !n || stream_bytes < 4 ||
            stream_bytes > std::numeric_limits<uint32_t>::max())
          return 1;
        const BcxShape sh = bcx_shape(kind, nr, nc);
        if (std::any_of(rc, rc + rows, [&](uint8_t v) { return v >= nr; })) return 1;
        if (std::any_of(cc, cc + cols, [&](uint8_t v) { return v >= nc; })) return 1;
        if (kind)
          for (uint64_t i = 0; i < n; ++i)
            if (resctx[i] >= sh.nctx) return 1;
        SymbolTables t;
        if (t.build(freq, sh.nctx, sh.vocab) != SymbolTables::Check::ok) return 2;
        const size_t count = (size_t)((n - 1) / stride + 1);
        // Work on private buffers: the caller's arrays change only on success.
        std::vector<uint32_t> st(count), of(count);
        std::vector<uint16_t> sym((size_t)n);
        StrideMark mark{stride, st.data(), of.data()};
        Walk w = kind ? walk_stream(stream, stream_bytes, n, t, ArrayContext{resctx}, std::ref(mark), sym.data())
                      : walk_stream(stream, stream_bytes, n, t, GridContext{rc, cc, cols, nc}, std::ref(mark),
                                    sym.data());
        switch (w) {
          case Walk::ok:
            break;
          case Walk::bad_context:
          case Walk::dead_context:
          case Walk::bad_symbol:
            return 2;
          default:
            return 3;
        }
        std::copy(st.begin(), st.end(), states);
        std::copy(of.begin(), of.end(), offsets);
        std::copy(sym.begin(), sym.end(), out);
        return 0;
      },
      5, 6);
}

// 10-bit main symbols + 6-bit residuals -> BF16 words (no reference counterpart:
// the reference recombines in numpy, GCR/bitexact_context_codec.py:426).
int grf_bctx_join(const uint16_t *main_sym, const uint16_t *res_sym, uint64_t n, uint16_t *out) {
  if (!main_sym || !res_sym || !out) return 1;
  for (uint64_t i = 0; i < n; ++i) {
    const uint32_t m = main_sym[i], r = res_sym[i];
    if (m > 1023u || r > 63u) return 2;
    out[i] = (uint16_t)((m << 5) | (r & 31u) | ((r >> 5) << 15));
  }
  return 0;
}

// ---------------------------------------------------------------- PPCX
int p_encode(const uint16_t *v, const uint16_t *cx, uint64_t n, uint32_t nc, uint32_t vocab, uint32_t **freqp,
             uint8_t **streamp, size_t *sn) {
  return guarded(
      [&]() -> int {
        if (!v || !cx || !n || n > 100000000u || !nc || !vocab || vocab > kTotal || !freqp || !streamp || !sn)
          return 1;
        *freqp = nullptr;
        *streamp = nullptr;
        *sn = 0;
        const size_t cells = (size_t)nc * vocab;
        std::vector<uint64_t> hist(cells);
        for (uint64_t i = 0; i < n; ++i) {
          if (cx[i] >= nc || v[i] >= vocab) return 2;
          ++hist[(size_t)cx[i] * vocab + v[i]];
        }
        std::vector<uint32_t> freq(cells);
        for (uint32_t c = 0; c < nc; ++c) normalize_row(hist.data() + (size_t)c * vocab, vocab, freq.data() + (size_t)c * vocab);
        std::vector<uint8_t> bytes;
        if (!encode_stream(
                n, freq.data(), nc, vocab, [&](uint64_t i) { return (uint32_t)v[i]; },
                [&](uint64_t i) { return (uint32_t)cx[i]; }, bytes))
          return 3;
        auto *fp = (uint32_t *)std::malloc(cells * sizeof(uint32_t));
        auto *sp = (uint8_t *)std::malloc(bytes.size());
        if (!fp || !sp) {
          std::free(fp);
          std::free(sp);
          return 4;
        }
        std::memcpy(fp, freq.data(), cells * sizeof(uint32_t));
        std::memcpy(sp, bytes.data(), bytes.size());
        *freqp = fp;
        *streamp = sp;
        *sn = bytes.size();
        return 0;
      },
      5, 5);
}

// Status categories follow GCR/bitexact_predictive_ans.cpp:11 (1 arguments,
// 2 initial state, 3 table row overflow, 4 row does not sum to the total,
// 5 context out of range, 8 stream exhausted, 9 terminal state/length).
int p_decode(const uint8_t *st, size_t bytes, uint64_t n, const uint16_t *cx, uint32_t nc, uint32_t vocab,
             const uint32_t *f, uint16_t *out) {
  return guarded(
      [&]() -> int {
        if (!st || bytes < 4 || !cx || !f || !out || !n || n > 100000000u || !nc || !vocab || vocab > kTotal)
          return 1;
        uint32_t head;
        if (!read_head(st, bytes, head)) return 2;
        SymbolTables t;
        // a row whose sum is wrong only fails (4) when a symbol selects it
        if (t.build(f, nc, vocab, true) != SymbolTables::Check::ok) return 3;
        switch (walk_stream(st, bytes, n, t, ArrayContext{cx}, NoMark{}, out)) {
          case Walk::ok:
            return 0;
          case Walk::bad_context:
            return 5;
          case Walk::dead_context:
            return 4;
          case Walk::overrun:
            return 8;
          case Walk::bad_head:
            return 2;
          default:
            return 9;
        }
      },
      10, 10);
}

void p_free(void *p) { std::free(p); }

static int ppcx_checkpoint_impl(const uint8_t *stream, size_t bytes, uint64_t n, const uint16_t *ctx,
                                uint32_t nctx, uint32_t vocab, const uint32_t *freq, uint32_t stride,
                                uint32_t *states, uint32_t *offsets, uint16_t *symbols) {
  return guarded(
      [&]() -> int {
        if (!stream || bytes < 4 || bytes > std::numeric_limits<uint32_t>::max() || !n || !ctx || !nctx ||
            !vocab || vocab > kTotal || !freq || !stride || !states || !offsets || !symbols || n > 100000000u)
          return 1;
        SymbolTables t;
        if (t.build(freq, nctx, vocab) != SymbolTables::Check::ok) return 2;
        const size_t count = (size_t)((n + stride - 1) / stride);
        std::vector<uint32_t> st(count), of(count);
        StrideMark mark{stride, st.data(), of.data()};
        switch (walk_stream(stream, bytes, n, t, ArrayContext{ctx}, std::ref(mark), symbols)) {
          case Walk::ok:
            break;
          case Walk::bad_context:
            return 4;
          case Walk::dead_context:
          case Walk::bad_symbol:
            return 5;
          default:
            return 3;
        }
        std::copy(st.begin(), st.end(), states);
        std::copy(of.begin(), of.end(), offsets);
        return 0;
      },
      6, 6);
}

int ppcx_checkpoint(const uint8_t *stream, size_t bytes, uint64_t n, const uint16_t *ctx, uint32_t nctx,
                    uint32_t vocab, const uint32_t *freq, uint32_t stride, uint32_t *states, uint32_t *offsets,
                    uint16_t *symbols) {
  return ppcx_checkpoint_impl(stream, bytes, n, ctx, nctx, vocab, freq, stride, states, offsets, symbols);
}

// The reference offers a second entry point with a faster search; here both use
// the coarse-index lookup, so they are the same function.
int ppcx_checkpoint_binary(const uint8_t *stream, size_t bytes, uint64_t n, const uint16_t *ctx, uint32_t nctx,
                           uint32_t vocab, const uint32_t *freq, uint32_t stride, uint32_t *states,
                           uint32_t *offsets, uint16_t *symbols) {
  return ppcx_checkpoint_impl(stream, bytes, n, ctx, nctx, vocab, freq, stride, states, offsets, symbols);
}

}  // extern "C"
