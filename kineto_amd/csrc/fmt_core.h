/*
 * fmt_core.h — byte-exact formatting of one activity as ChromeTraceLogger would print it.
 *
 * Everything here is a pure function of its inputs and compiles both as HIP device code (the
 * size and emit kernels) and as plain host C++ (the host-side simulation used by the CPU tests).
 * The same template runs twice per record: once with CountWriter to get the exact byte length,
 * once with a tile writer to produce the bytes, so length and content cannot disagree.
 *
 * Reference being reproduced (paths relative to the pytorch/kineto tree):
 *   libkineto/src/output_json.cpp:237-259  writeCompleteEvent
 *   libkineto/src/output_json.cpp:318-345  writeFlowEvent
 *   libkineto/src/output_json.cpp:837-1021 handleActivity / handleGenericLink / handleLink
 *   libkineto/src/output_json.cpp:157-212  ArgsBuilder
 *   libkineto/include/TypedMetadataJson.h:38-205 JsonTypedMetadataVisitor
 *   libkineto/src/RocprofActivity_inl.h:98-299 ROCm metadata producers
 *   libkineto/src/CuptiActivity.h:682-713  memset metadata
 */
#ifndef KTJ_FMT_CORE_H_
#define KTJ_FMT_CORE_H_

#include "ktj_device.h"

/* The writer must live in registers: everything that touches it is inlined into the kernel. */
#define KTJ_FI __attribute__((always_inline))
#if defined(__clang__)
#define KTJ_NOUNROLL _Pragma("clang loop unroll(disable)")
#else
#define KTJ_NOUNROLL
#endif

#if defined(__HIP_DEVICE_COMPILE__)
#define KTJ_POW10_QUALIFIER __device__
#else
#define KTJ_POW10_QUALIFIER static
#endif
#include "pow10_table.h"

namespace ktj {

/* ---------------------------------------------------------------------------------------- */
/* integers                                                                                   */
/* ---------------------------------------------------------------------------------------- */
KTJ_HD KTJ_FI inline int ndigits_u64(uint64_t v) {
  int n = 1;
  if (v >= 10000000000ULL) { v /= 10000000000ULL; n += 10; }
  uint32_t x = (uint32_t)v; /* < 10^10 may exceed 32 bits */
  if (v >= 100000000ULL) { x = (uint32_t)(v / 100000000ULL); n += 8; }
  if (x >= 10000u) { x /= 10000u; n += 4; }
  if (x >= 100u) { x /= 100u; n += 2; }
  if (x >= 10u) { n += 1; }
  return n;
}

KTJ_HD KTJ_FI inline uint64_t mulhi64(uint64_t a, uint64_t b) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __umul64hi(a, b);
#else
  return (uint64_t)(((unsigned __int128)a * b) >> 64);
#endif
}

/* ---------------------------------------------------------------------------------------- */
/* shortest round-trip decimal of a finite positive double (Schubfach, R. Giulietti 2020):   */
/* returns digits (no trailing zeros) and decimal exponent so that v = digits * 10^exp10.     */
/* Reproduces what fmt's "{}" (Dragonbox) prints: shortest, closest, ties to even.            */
/* ---------------------------------------------------------------------------------------- */
KTJ_HD KTJ_FI inline int32_t floor_log2_pow10(int32_t e) { return (e * 1741647) >> 19; }
KTJ_HD KTJ_FI inline int32_t floor_log10_pow2(int32_t e) { return (e * 1262611) >> 22; }
KTJ_HD KTJ_FI inline int32_t floor_log10_3q_pow2(int32_t e) { return (e * 1262611 - 524031) >> 22; }

KTJ_HD KTJ_FI inline uint64_t round_to_odd(uint64_t ghi, uint64_t glo, uint64_t cp) {
  /* (cp * g) >> 128 with a sticky low bit; g = ghi:glo */
  uint64_t x_hi = mulhi64(cp, glo);
  uint64_t y_lo = cp * ghi;
  uint64_t y_hi = mulhi64(cp, ghi);
  uint64_t s_lo = y_lo + x_hi;
  uint64_t carry = s_lo < y_lo ? 1 : 0;
  uint64_t y1 = y_hi + carry;
  return y1 | (s_lo > 1 ? 1 : 0);
}

KTJ_HD KTJ_FI inline void shortest_decimal(uint64_t bits, uint64_t* digits, int32_t* exp10) {
  const uint64_t frac = bits & 0x000FFFFFFFFFFFFFULL;
  const uint32_t bexp = (uint32_t)((bits >> 52) & 0x7FF);
  uint64_t c;
  int32_t q;
  uint64_t sig;
  int32_t k;
  bool done = false;
  if (bexp != 0) {
    c = frac | 0x0010000000000000ULL;
    q = (int32_t)bexp - 1075;
    if (0 <= -q && -q < 53 && (c & ((1ULL << (-q)) - 1)) == 0) { /* integer below 2^53 */
      sig = c >> (-q);
      k = 0;
      done = true;
    }
  } else {
    c = frac;
    q = 1 - 1075;
  }
  if (!done) {
    const bool is_even = (c & 1) == 0;
    const bool lower_closer = frac == 0 && bexp > 1;
    const uint64_t cbl = 4 * c - 2 + (lower_closer ? 1 : 0);
    const uint64_t cb = 4 * c;
    const uint64_t cbr = 4 * c + 2;
    k = lower_closer ? floor_log10_3q_pow2(q) : floor_log10_pow2(q);
    const int32_t h = q + floor_log2_pow10(-k) + 1;
    const uint64_t ghi = ktj_pow10_table[-k - KTJ_POW10_KMIN][0];
    const uint64_t glo = ktj_pow10_table[-k - KTJ_POW10_KMIN][1];
    const uint64_t vbl = round_to_odd(ghi, glo, cbl << h);
    const uint64_t vb = round_to_odd(ghi, glo, cb << h);
    const uint64_t vbr = round_to_odd(ghi, glo, cbr << h);
    const uint64_t lower = vbl + (is_even ? 0 : 1);
    const uint64_t upper = vbr - (is_even ? 0 : 1);
    const uint64_t s = vb / 4;
    bool found = false;
    if (s >= 10) {
      const uint64_t sp = s / 10;
      const bool up_inside = lower <= 40 * sp;
      const bool wp_inside = 40 * sp + 40 <= upper;
      if (up_inside != wp_inside) {
        sig = sp + (wp_inside ? 1 : 0);
        k = k + 1;
        found = true;
      }
    }
    if (!found) {
      const bool u_inside = lower <= 4 * s;
      const bool w_inside = 4 * s + 4 <= upper;
      if (u_inside != w_inside) sig = s + (w_inside ? 1 : 0);
      else {
        const uint64_t mid = 4 * s + 2;
        const bool round_up = vb > mid || (vb == mid && (s & 1) != 0);
        sig = s + (round_up ? 1 : 0);
      }
    }
  }
  while (sig % 10 == 0 && sig != 0) { sig /= 10; ++k; }
  *digits = sig;
  *exp10 = k;
}

/* ---------------------------------------------------------------------------------------- */
/* clock conversion: (int64)((double)(t - t0_approx) * (long double)scale) + t0, exactly as    */
/* x87 extended precision computes it (libkineto/src/ApproximateClock.cpp:83-90): the exact    */
/* 106-bit product of two 53-bit significands is rounded to 64 bits (nearest even) and the     */
/* result truncated toward zero.                                                               */
/* ---------------------------------------------------------------------------------------- */
KTJ_HD KTJ_FI inline int64_t convert_timestamp(uint64_t t, uint64_t t0_approx, int64_t t0, uint64_t scale_bits) {
  const int64_t ta = (int64_t)t, t0a = (int64_t)t0_approx;
  if (!(ta > t0a)) return 0;
  const uint64_t dt = (uint64_t)(ta - t0a); /* > 0 */
  /* (double)dt: round to nearest even at 53 bits */
  int lz = 0; { uint64_t x = dt; while (!(x >> 63)) { x <<= 1; ++lz; } }
  uint64_t m1 = dt << lz;             /* normalised, bit 63 set */
  int e1 = 63 - lz;                   /* dt = m1 * 2^(e1-63) */
  { const uint64_t low = m1 & 0x7FF; m1 >>= 11; /* 53 bits */
    if (low > 0x400 || (low == 0x400 && (m1 & 1))) { ++m1; if (m1 >> 53) { m1 >>= 1; ++e1; } } }
  /* m1 in [2^52, 2^53), value = m1 * 2^(e1-52) */
  const uint32_t sexp = (uint32_t)((scale_bits >> 52) & 0x7FF);
  uint64_t m2 = scale_bits & 0x000FFFFFFFFFFFFFULL;
  const bool sneg = (scale_bits >> 63) != 0;
  if (sexp == 0x7FF) return (int64_t)0x8000000000000000ULL + t0; /* inf/nan → x87 "integer indefinite" */
  int e2;
  if (sexp == 0) { if (m2 == 0) return t0; e2 = -1074; while (!(m2 >> 52)) { m2 <<= 1; --e2; } }
  else { m2 |= 0x0010000000000000ULL; e2 = (int)sexp - 1075; }
  /* product P = m1*m2 in [2^104, 2^106), value = P * 2^(e1-52+e2) */
  const uint64_t phi = mulhi64(m1, m2), plo = m1 * m2;
  int top = (phi >> 41) ? 105 : 104;  /* index of the leading bit of P */
  /* keep 64 significant bits: drop `drop` low bits with round-to-nearest-even */
  const int drop = top - 63;          /* 41 or 42 */
  uint64_t kept = (phi << (64 - drop)) | (plo >> drop);
  const uint64_t rem = plo & ((1ULL << drop) - 1);
  const uint64_t half = 1ULL << (drop - 1);
  int ex = e1 - 52 + e2 + drop;       /* value = kept * 2^ex */
  if (rem > half || (rem == half && (kept & 1))) { ++kept; if (kept == 0) { kept = 1ULL << 63; ++ex; } }
  /* truncate toward zero to int64 */
  uint64_t mag;
  if (ex >= 0) { if (ex > 0 || (kept >> 63)) return (int64_t)0x8000000000000000ULL + t0; mag = kept; }
  else if (ex <= -64) mag = 0;
  else mag = kept >> (-ex);
  if (mag >> 63) return (int64_t)0x8000000000000000ULL + t0; /* out of int64 range */
  const int64_t r = sneg ? -(int64_t)mag : (int64_t)mag;
  return (int64_t)((uint64_t)r + (uint64_t)t0);
}

/* ---------------------------------------------------------------------------------------- */
/* constant strings: packed at compile time into 8-byte little-endian words so that the emit   */
/* kernel appends them as immediates (no loads) and the size pass adds a constant.             */
/* ---------------------------------------------------------------------------------------- */
template <unsigned N> struct PackedLit {
  uint64_t w[(N + 7) / 8 ? (N + 7) / 8 : 1];
};
template <unsigned M> constexpr PackedLit<M - 1> pack_lit(const char (&s)[M]) {
  PackedLit<M - 1> p{};
  for (unsigned i = 0; i < (M - 1 + 7) / 8; ++i) p.w[i] = 0;
  for (unsigned i = 0; i + 1 < M; ++i) p.w[i / 8] |= (uint64_t)(unsigned char)s[i] << (8 * (i % 8));
  return p;
}
#define KTJ_PUT(w, s)                                   \
  do {                                                  \
    constexpr auto ktj_lit_ = ::ktj::pack_lit(s);       \
    (w).lit(ktj_lit_);                                  \
  } while (0)

/* ---------------------------------------------------------------------------------------- */
/* decimal digits as packed ASCII                                                             */
/* ---------------------------------------------------------------------------------------- */
/* x < 10000 → its four digits as ASCII, most significant digit in the lowest byte */
KTJ_HD KTJ_FI inline uint32_t ascii4(uint32_t x) {
  const uint32_t hi = (x * 5243u) >> 19; /* x / 100 */
  const uint32_t lo = x - hi * 100u;
  const uint32_t h = (hi * 103u) >> 10, l = (lo * 103u) >> 10; /* / 10 */
  return (h | ((hi - h * 10u) << 8) | (l << 16) | ((lo - l * 10u) << 24)) + 0x30303030u;
}
/* x < 10^8 → eight ASCII digits, most significant first (lowest byte) */
KTJ_HD KTJ_FI inline uint64_t ascii8(uint32_t x) {
  const uint32_t hi = x / 10000u;
  const uint32_t lo = x - hi * 10000u;
  return (uint64_t)ascii4(hi) | ((uint64_t)ascii4(lo) << 32);
}
/* number of leading '0' characters of an ascii8 word, at most 7 */
KTJ_HD KTJ_FI inline uint32_t leading_zero_chars(uint64_t a) {
  const uint64_t d = a ^ 0x3030303030303030ULL;
  if (d == 0) return 7;
#if defined(__HIP_DEVICE_COMPILE__)
  return (uint32_t)(__ffsll((long long)d) - 1) >> 3;
#else
  return (uint32_t)__builtin_ctzll(d) >> 3;
#endif
}

/* ---------------------------------------------------------------------------------------- */
/* writers                                                                                     */
/* ---------------------------------------------------------------------------------------- */
/* Pass A: exact byte length. */
struct CountWriter {
  uint64_t n = 0;
  KTJ_HD KTJ_FI void ch(char) { ++n; }
  template <unsigned N> KTJ_HD KTJ_FI void lit(const PackedLit<N>&) { n += N; }
  KTJ_HD KTJ_FI void dec(uint64_t v) { n += (uint32_t)ndigits_u64(v); }
  KTJ_HD KTJ_FI void dec3(uint32_t) { n += 3; }
  KTJ_HD KTJ_FI void str(const char*, uint64_t len) { n += len; }
  KTJ_HD KTJ_FI void name(const char*, uint64_t len) { n += len; }
  /* a number that is printed more than once is prepared once */
  typedef uint32_t Prepared;
  KTJ_HD KTJ_FI static Prepared prepare(uint64_t v) { return (uint32_t)ndigits_u64(v); }
  KTJ_HD KTJ_FI void num(Prepared len) { n += len; }
  KTJ_HD KTJ_FI void relief() {}
};

/* A decimal number rendered once and appended several times (pid, tid and ts appear in the
 * complete event and again in the flow event). */
struct Num {
  uint64_t word;  /* up to 8 ASCII digits, first digit in the lowest byte */
  uint32_t len;   /* 1..8, or 0 when the value needs more than 8 digits */
  uint64_t value;
};
KTJ_HD KTJ_FI inline Num make_num(uint64_t v) {
  Num n;
  n.value = v;
  if (__builtin_expect(v < 100000000ULL, 1)) {
    const uint64_t a = ascii8((uint32_t)v);
    const uint32_t z = leading_zero_chars(a);
    n.word = a >> (8 * z);
    n.len = 8 - z;
  } else { n.word = 0; n.len = 0; }
  return n;
}

/* Pass B: bytes into one tile of the output, held in LDS.
 *
 * Coordinates are tile-local: byte L of the buffer is byte (tile origin + L) of the document and
 * the buffer covers L in [0, size); an activity that straddles a tile boundary is formatted by
 * both tiles and everything outside the buffer is dropped.  Bytes are gathered in a 64-bit
 * accumulator and leave as aligned 8-byte OR operations into the zero-filled tile: neighbouring
 * activities and strings share boundary words, and OR-ing zeros into their bytes leaves them
 * alone, so the writer needs no ownership bookkeeping.  Dictionary strings are not copied here
 * but queued as copy jobs that whole wavefronts execute afterwards. */
struct CopyJob { const char* src; int32_t dst; uint32_t len; };

struct TileWriter {
  char* buf;          /* 8-byte aligned, zero-filled, `size` bytes */
  uint32_t size;      /* multiple of 8 */
  CopyJob* jobs;
  uint32_t* n_jobs;
  uint32_t max_jobs;
  /* accumulator */
  uint64_t acc;
  int32_t wpos;       /* tile-local position of acc's byte 0; multiple of 8 */
  uint32_t fill;      /* bytes gathered in acc, 0..7 */

  KTJ_HD KTJ_FI void begin(int32_t pos) {
    wpos = pos & ~7;
    fill = (uint32_t)(pos - wpos);
    acc = 0;
  }
  KTJ_HD KTJ_FI int32_t position() const { return wpos + (int32_t)fill; }
  KTJ_HD KTJ_FI void or_word() {
    if ((uint32_t)wpos < size) {
#if defined(__HIP_DEVICE_COMPILE__)
      __hip_atomic_fetch_or(reinterpret_cast<unsigned long long*>(buf + wpos), (unsigned long long)acc, __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_WORKGROUP);
#else
      *reinterpret_cast<uint64_t*>(buf + wpos) |= acc;
#endif
    }
  }
  KTJ_HD KTJ_FI void end() { if (fill) or_word(); }
  /* append the n (0..8) low bytes of v; bytes above n must be zero */
  KTJ_HD KTJ_FI void append(uint64_t v, uint32_t n) {
    acc |= v << (8 * fill);
    const uint32_t total = fill + n;
    if (total >= 8) {
      or_word();
      wpos += 8;
      const uint32_t rest = total - 8;           /* bytes of v still unwritten: its top `rest` of n */
      acc = rest ? v >> (8 * (n - rest)) : 0;
      fill = rest;
    } else fill = total;
  }
  KTJ_HD KTJ_FI void ch(char c) { append((uint64_t)(unsigned char)c, 1); }
  KTJ_HD KTJ_FI void relief() {}
  template <unsigned N> KTJ_HD KTJ_FI void lit(const PackedLit<N>& l) {
    for (unsigned i = 0; i < N / 8; ++i) append(l.w[i], 8);
    if (N % 8) append(l.w[N / 8], N % 8);
  }
  KTJ_HD KTJ_FI void dec_wide(uint64_t v) { /* more than 8 digits: up to three 8-digit groups */
    const uint64_t top = v / 10000000000000000ULL;
    const uint64_t rest = v - top * 10000000000000000ULL;
    const uint64_t mid = rest / 100000000ULL;
    const uint32_t low = (uint32_t)(rest - mid * 100000000ULL);
    uint64_t a0 = 0, a1;
    uint32_t n0 = 0, n1;
    if (top) {
      a0 = ascii8((uint32_t)top);
      const uint32_t z = leading_zero_chars(a0);
      a0 >>= 8 * z; n0 = 8 - z;
      a1 = ascii8((uint32_t)mid); n1 = 8;
    } else {
      a1 = ascii8((uint32_t)mid);
      const uint32_t z = leading_zero_chars(a1);
      a1 >>= 8 * z; n1 = 8 - z;
    }
    append(a0, n0);
    append(a1, n1);
    append(ascii8(low), 8);
  }
  KTJ_HD KTJ_FI void dec(uint64_t v) {
    if (__builtin_expect(v < 100000000ULL, 1)) {
      const uint64_t a = ascii8((uint32_t)v);
      const uint32_t z = leading_zero_chars(a);
      append(a >> (8 * z), 8 - z);
    } else dec_wide(v);
  }
  typedef Num Prepared;
  KTJ_HD KTJ_FI static Prepared prepare(uint64_t v) { return make_num(v); }
  KTJ_HD KTJ_FI void num(const Num& n) {
    if (__builtin_expect(n.len != 0, 1)) append(n.word, n.len); else dec_wide(n.value);
  }
  KTJ_HD KTJ_FI void dec3(uint32_t x) { /* {:03} of 0..999 */
    append((uint64_t)(ascii4(x) >> 8), 3);
  }
  KTJ_HD KTJ_FI void name(const char* src, uint64_t len) { str(src, len); }
  KTJ_HD KTJ_FI void str(const char* src, uint64_t len) {
    if (len == 0) return;
    end(); /* bytes gathered so far */
    const int64_t pos = position();
    int64_t b = pos < 0 ? -pos : 0;
    int64_t e = (int64_t)size - pos;
    if (e > (int64_t)len) e = (int64_t)len;
    if (b < e) {
      uint32_t slot;
#if defined(__HIP_DEVICE_COMPILE__)
      slot = atomicAdd(n_jobs, 1u);
#else
      slot = (*n_jobs)++;
#endif
      if (slot < max_jobs) {
        jobs[slot].src = src + b;
        jobs[slot].dst = (int32_t)(pos + b);
        jobs[slot].len = (uint32_t)(e - b);
      } else { /* queue full: copy here (bytes of a zero-filled region nobody else writes) */
        KTJ_NOUNROLL
        for (int64_t i = b; i < e; ++i) buf[pos + i] = src[i];
      }
    }
    begin((int32_t)(pos + (int64_t)len));
  }
};

/* Long dictionary strings (templated C++ kernel names run to kilobytes) are not copied by the lane
 * that owns the activity but by all lanes that are active with it: for one owner at a time,
 * neighbouring lanes move neighbouring 16-byte blocks, so loads and stores are whole lines.  The
 * owner has already brought its output to a block boundary; `src` is the first byte that lands on
 * that boundary (any alignment: two aligned loads are funnel-shifted), `dst` the block, `n_words`
 * the 8-byte words of the whole blocks (0 for lanes that only help).  Works under any set of
 * active lanes. */
#define KTJ_COOP_MIN_BYTES 256u
#if defined(__HIP_DEVICE_COMPILE__)
static __device__ __attribute__((noinline)) void cooperative_word_copy(const char* src, uint64_t* dst, uint32_t n_words) {
  typedef unsigned long long v2u64 __attribute__((ext_vector_type(2)));
  typedef __attribute__((address_space(1))) v2u64* gblocks;            /* document and dictionary are */
  typedef const __attribute__((address_space(1))) uint64_t* gwords;    /* global memory: no flat accesses */
  const uint64_t active = __ballot(1);
  const uint32_t lane = (uint32_t)(threadIdx.x & 63u);
  const uint32_t n_active = (uint32_t)__popcll(active);
  const uint32_t rank = (uint32_t)__popcll(active & ((1ULL << lane) - 1ULL));
  uint64_t todo = __ballot(n_words != 0);
  while (todo) {
    const int owner = __ffsll((unsigned long long)todo) - 1;
    todo &= todo - 1;
    const uint32_t n = (uint32_t)__shfl((int)n_words, owner) >> 1; /* whole blocks: a lane moves sixteen bytes at a time */
    const uintptr_t sa = (uintptr_t)__shfl((unsigned long long)(uintptr_t)src, owner);
    gblocks d = reinterpret_cast<gblocks>((uintptr_t)__shfl((unsigned long long)(uintptr_t)dst, owner));
    const uint32_t sh = (uint32_t)(sa & 7u) * 8u;
    gwords sp = reinterpret_cast<gwords>(sa & ~(uintptr_t)7);
    KTJ_NOUNROLL
    for (uint32_t k = rank; k < n; k += n_active) {
      const uint64_t w0 = sp[2u * k], w1 = sp[2u * k + 1u];
      v2u64 v;
      v.x = w0; v.y = w1;
      if (sh) {
        const uint64_t w2 = sp[2u * k + 2u];
        v.x = (w0 >> sh) | (w1 << (64u - sh));
        v.y = (w1 >> sh) | (w2 << (64u - sh));
      }
      /* whole lines that nobody reads again: stored past the L2's usual replacement, so that the
       * dictionary the next strings come from stays in it (config 5: emit 3.64 -> 3.27 ms) */
      __builtin_nontemporal_store(v, &d[k]);
    }
  }
}
#endif

#if defined(__HIPCC__)
/* blocks per lane in the stage: one 128-byte line of the document and the first five blocks of the
 * next one; odd, so that the lanes' accesses to the same slot (lane stride 16 * KTJ_STAGE_BLOCKS
 * bytes) do not collide on LDS banks */
#define KTJ_STAGE_BLOCKS 13u
#define KTJ_LINE_BLOCKS 8u
/* a lane with this many slots used asks for a relief() at the next opportunity (11 and 13 measured
 * slower: more reliefs than needed, or too late for the blocks that follow) */
#define KTJ_RELIEF_AT 12u
extern __shared__ __attribute__((aligned(16))) char ktj_stage_lds[];
#endif

/* Pass B: one lane formats one activity straight into the document in device memory.  Bytes are
 * gathered in a 128-bit accumulator and leave as aligned 16-byte blocks (on the device through the
 * lane's stage in LDS, see below); literal text is appended sixteen bytes at a time, so that all
 * lanes of a wavefront complete a block at the same append, whatever their phases.  Dictionary strings are
 * appended inline through a funnel shift over aligned 8-byte loads (dictionary blobs are padded by
 * 16 bytes so that the last load stays inside the allocation).  Every block of the document has exactly one writer who knows all of
 * its bytes: a block that holds the end of activity A and the start of activity B is written
 *   - by B, if fewer than eight bytes of it are A's: they are one of the fixed tails (tail_kind);
 *   - by A otherwise: the at most eight bytes of B in it are the same for every activity
 *     ("\n  {\n    ", the start of each event of every kind).
 * The first activity reads what precedes it from the document, the last one merges with what
 * follows it; both were put in place by the host before the kernel runs. */
struct BlockWriter {
  uint64_t* wptr;     /* the 16-byte block being gathered (as two words) */
  uint64_t lo, hi;    /* its first `fill` bytes */
  uint32_t fill;      /* 0..15 */
  bool foreign;       /* the block belongs to the predecessor: gathered but not stored */
#if defined(__HIPCC__)
  /* Device: finished blocks do not go to the document one by one (64 lanes, 64 different lines per
   * store instruction, every line written sixteen bytes at a time over some microseconds) but wait
   * in LDS.  A lane's stage mirrors the document: slot q holds the block at line_base + 16 q, so
   * slots 0..7 are one 128-byte line and slots 8..12 the beginning of the next.  flush() and
   * relief() write the line out once it is complete, all of it at one moment (a line written in
   * pieces some microseconds apart leaves the L2 cache once per piece), and move the next line's
   * blocks down.  When the stage is full, and after a jump of wptr, blocks are stored directly
   * until the next flush(). */
  uint32_t stage_lds;   /* byte offset of this lane's stage in the workgroup's dynamic LDS */
  uint32_t q_first;     /* slot of the first waiting block (not 0 only in an activity's first line) */
  uint32_t q_end;       /* slot behind the last waiting block; nothing waits when q_end == q_first */
  uint32_t stage_cap;   /* KTJ_STAGE_BLOCKS, or 0 while the stage is closed */
  uintptr_t line_base;  /* 128-byte aligned address of the line in slots 0..7 */
#endif

  KTJ_HD KTJ_FI static uint64_t head_bytes() { constexpr auto h = pack_lit("\n  {\n   "); return h.w[0]; }
  KTJ_HD KTJ_FI void store_block() {
    if (!foreign) {
#if defined(__HIP_DEVICE_COMPILE__)
      typedef unsigned long long v2u64 __attribute__((ext_vector_type(2)));
      v2u64 v; v.x = lo; v.y = hi;
      if (q_end < stage_cap) { /* an open stage's slot q_end is the block at wptr */
        *reinterpret_cast<v2u64*>(ktj_stage_lds + stage_lds + q_end * 16u) = v;
        ++q_end;
      } else { stage_cap = 0; *reinterpret_cast<v2u64*>(wptr) = v; }
#else
      wptr[0] = lo; wptr[1] = hi;
#endif
    }
    foreign = false;
    wptr += 2;
  }
#if defined(__HIPCC__)
  __device__ KTJ_FI void stage_init(uint32_t lds_offset) {
    stage_lds = lds_offset; q_first = q_end = 0; stage_cap = KTJ_STAGE_BLOCKS; line_base = 0;
    wptr = nullptr; lo = hi = 0; fill = 0; foreign = false;
  }
  /* wptr is about to move by more than one block: what waits stays, nothing more is staged */
  __device__ KTJ_FI void stage_close() { stage_cap = 0; }
  /* an empty stage takes its place in the document from wptr: after begin(), and when a closed
   * stage opens again (a block that the predecessor writes is passed over) */
  __device__ KTJ_FI void stage_follow() {
    const uintptr_t a = (uintptr_t)(wptr + (foreign ? 2 : 0));
    line_base = a & ~(uintptr_t)127;
    q_first = q_end = (uint32_t)(a >> 4) & (KTJ_LINE_BLOCKS - 1u);
  }
  /* Blocks leave the stage.  Slots are read and written with constant offsets, and a lane touches
   * only its own stage: any set of lanes may come here.  stage_line: the line in slots 0..7 leaves
   * if it is complete, and what waits of the next line moves down. */
  __device__ KTJ_FI void stage_line() {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef unsigned long long v2u64 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2u64* gptr; /* the document is global memory: no flat stores */
    if (q_end < KTJ_LINE_BLOCKS) return;
    char* s = ktj_stage_lds + stage_lds;
    v2u64 x[KTJ_STAGE_BLOCKS];
    _Pragma("unroll")
    for (uint32_t p = 0; p < KTJ_STAGE_BLOCKS; ++p) x[p] = *reinterpret_cast<const v2u64*>(s + p * 16u); /* all reads first: one wait */
    gptr d = reinterpret_cast<gptr>(line_base);
    if (q_first == 0) { /* every line but an activity's first */
      _Pragma("unroll")
      for (uint32_t p = 0; p < KTJ_LINE_BLOCKS; ++p) d[p] = x[p];
    } else {
      _Pragma("unroll")
      for (uint32_t p = 1; p < KTJ_LINE_BLOCKS; ++p)
        if (p >= q_first) d[p] = x[p];
    }
    _Pragma("unroll")
    for (uint32_t p = KTJ_LINE_BLOCKS; p < KTJ_STAGE_BLOCKS; ++p)
      if (p < q_end) *reinterpret_cast<v2u64*>(s + (p - KTJ_LINE_BLOCKS) * 16u) = x[p];
    line_base += 128u;
    q_first = 0;
    q_end -= KTJ_LINE_BLOCKS;
#endif
  }
  /* every waiting block leaves (the lane's last flush, or a closed stage: the blocks behind them are
   * in the document already) */
  __device__ KTJ_FI void stage_all() {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef unsigned long long v2u64 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2u64* gptr;
    char* s = ktj_stage_lds + stage_lds;
    v2u64 x[KTJ_STAGE_BLOCKS];
    _Pragma("unroll")
    for (uint32_t p = 0; p < KTJ_STAGE_BLOCKS; ++p) x[p] = *reinterpret_cast<const v2u64*>(s + p * 16u);
    gptr d = reinterpret_cast<gptr>(line_base);
    _Pragma("unroll")
    for (uint32_t p = 0; p < KTJ_STAGE_BLOCKS; ++p)
      if (p >= q_first && p < q_end) d[p] = x[p];
#endif
  }
  /* The same for the stages of whole quads: the four lanes of a quad write each other's blocks, lane
   * k the slots k, k + 4, ... of every stage of its quad, so that a store instruction covers 64
   * contiguous bytes per quad.  All four lanes of a quad must be here together.  CAN_ALL: stages
   * that are closed, and every stage when `last`, are emptied (stage_all) instead. */
  template <bool CAN_ALL> __device__ KTJ_FI void quad_write(bool last) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef unsigned long long v2u64 __attribute__((ext_vector_type(2)));
    typedef __attribute__((address_space(1))) v2u64* gptr;
    const uint32_t k = (uint32_t)threadIdx.x & 3u;
    const bool all = CAN_ALL && (last || stage_cap == 0);
    const bool line = q_end >= KTJ_LINE_BLOCKS;
    const uint32_t lim = all ? q_end : (line ? KTJ_LINE_BLOCKS : 0u); /* slots [q_first, lim) leave */
    const uint32_t lb_lo = (uint32_t)line_base, lb_hi = (uint32_t)(line_base >> 32);
    const uint32_t quad_lds = stage_lds - k * (KTJ_STAGE_BLOCKS * 16u);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#define KTJ_QUAD_BCAST(v, t) ((uint32_t)__builtin_amdgcn_mov_dpp((int)(v), (t) * 0x55, 0xF, 0xF, true))
    constexpr uint32_t ROUNDS = CAN_ALL ? (KTJ_STAGE_BLOCKS + 3u) / 4u : KTJ_LINE_BLOCKS / 4u;
#define KTJ_FLUSH_FROM(t)                                                                                   \
    {                                                                                                       \
      const uint32_t first_t = KTJ_QUAD_BCAST(q_first, t), lim_t = KTJ_QUAD_BCAST(lim, t);                  \
      gptr d = reinterpret_cast<gptr>(((uintptr_t)KTJ_QUAD_BCAST(lb_hi, t) << 32) | (uintptr_t)KTJ_QUAD_BCAST(lb_lo, t)); \
      const char* s = ktj_stage_lds + quad_lds + (t) * (KTJ_STAGE_BLOCKS * 16u);                            \
      v2u64 x[ROUNDS];                                                                                      \
      _Pragma("unroll")                                                                                     \
      for (uint32_t m = 0; m < ROUNDS; ++m) {                                                               \
        const uint32_t p = k + 4u * m;                                                                      \
        x[m] = *reinterpret_cast<const v2u64*>(s + (p < KTJ_STAGE_BLOCKS ? p : 0u) * 16u);                  \
      }                                                                                                     \
      _Pragma("unroll")                                                                                     \
      for (uint32_t m = 0; m < ROUNDS; ++m) {                                                               \
        const uint32_t p = k + 4u * m;                                                                      \
        if (p >= first_t && p < lim_t) d[p] = x[m];                                                         \
      }                                                                                                     \
    }
    KTJ_FLUSH_FROM(0) KTJ_FLUSH_FROM(1) KTJ_FLUSH_FROM(2) KTJ_FLUSH_FROM(3)
#undef KTJ_FLUSH_FROM
#undef KTJ_QUAD_BCAST
    if (all) stage_follow();
    else if (line) { /* the next line's blocks move down; the wavefront's LDS accesses keep their order */
      char* s = ktj_stage_lds + stage_lds;
      v2u64 y[KTJ_STAGE_BLOCKS - KTJ_LINE_BLOCKS];
      _Pragma("unroll")
      for (uint32_t p = KTJ_LINE_BLOCKS; p < KTJ_STAGE_BLOCKS; ++p) y[p - KTJ_LINE_BLOCKS] = *reinterpret_cast<const v2u64*>(s + p * 16u);
      _Pragma("unroll")
      for (uint32_t p = KTJ_LINE_BLOCKS; p < KTJ_STAGE_BLOCKS; ++p)
        if (p < q_end) *reinterpret_cast<v2u64*>(s + (p - KTJ_LINE_BLOCKS) * 16u) = y[p - KTJ_LINE_BLOCKS];
      line_base += 128u;
      q_first = 0;
      q_end -= KTJ_LINE_BLOCKS;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
#endif
  }
  /* The three points of an activity where the whole wavefront meets (lanes without an activity
   * included): complete lines leave, closed stages are emptied and opened again; last: everything
   * leaves. */
  __device__ KTJ_FI void flush(bool last) {
#if defined(__HIP_DEVICE_COMPILE__)
    if (last || __any(stage_cap == 0)) quad_write<true>(last);
    else quad_write<false>(false);
    stage_cap = KTJ_STAGE_BLOCKS;
#endif
  }
  /* the same, but only if some lane's stage is full or closed: where the part that follows is short
   * enough for the stages of most wavefronts, the flush costs more than it saves */
  __device__ KTJ_FI void flush_if_full() {
#if defined(__HIP_DEVICE_COMPILE__)
    if (__any(stage_cap == 0 || q_end >= KTJ_STAGE_BLOCKS)) flush(false);
#endif
  }
  /* Between flushes, wherever the formatter calls it: when a lane's stage is nearly full, every lane
   * that is here with a complete line writes it out (whole quads together, other lanes each on its
   * own).  Without this a full stage sends the blocks that follow straight to the document one at a
   * time, and the lines around such a run reach memory in pieces. */
  __device__ KTJ_FI void relief() {
#if defined(__HIP_DEVICE_COMPILE__)
    if (__any(stage_cap != 0 && q_end >= KTJ_RELIEF_AT)) stage_line();
#endif
  }
#else
  KTJ_HD KTJ_FI void relief() {}
#endif
  /* pos: where the activity starts; tail_kind_before: kind of the activity before it */
  KTJ_HD KTJ_FI void begin(char* doc, uint64_t pos, uint32_t tail_kind_before, bool first);
  KTJ_HD KTJ_FI void end(bool last);
  /* bytes gathered so far count from the document start */
  KTJ_HD KTJ_FI uint64_t position(const char* doc) const { return (uint64_t)((const char*)wptr - doc) + fill; }

  /* append the n (0..8) low bytes of v; bytes above n must be zero */
  KTJ_HD KTJ_FI void append(uint64_t v, uint32_t n) {
    const uint32_t r = (fill & 7u) * 8u;
    const uint64_t t0 = v << r, t1 = (v >> 1) >> (63u - r); /* v >> (64 - r), 0 for r == 0 */
    if (fill < 8) { lo |= t0; hi |= t1; }
    else hi |= t0;
    const uint32_t total = fill + n;
    if (total >= 16) { /* only from the upper half: t1 starts the next block */
      store_block();
      lo = t1; hi = 0;
      fill = total - 16;
    } else fill = total;
  }
  /* sixteen bytes at once: completes exactly one block whatever the fill */
  KTJ_HD KTJ_FI void append16(uint64_t a, uint64_t b) {
    const uint32_t r = (fill & 7u) * 8u;
    const uint64_t t0 = a << r;
    const uint64_t t1 = (b << r) | ((a >> 1) >> (63u - r)); /* x >> (64 - r), 0 for r == 0 */
    const uint64_t t2 = (b >> 1) >> (63u - r);
    if (fill < 8) { lo |= t0; hi |= t1; store_block(); lo = t2; hi = 0; }
    else { hi |= t0; store_block(); lo = t1; hi = t2; }
  }
  KTJ_HD KTJ_FI void ch(char c) { append((uint64_t)(unsigned char)c, 1); }
  template <unsigned N> KTJ_HD KTJ_FI void lit(const PackedLit<N>& l) {
    for (unsigned i = 0; i < N / 16; ++i) append16(l.w[2 * i], l.w[2 * i + 1]);
    if ((N % 16) >= 8) append(l.w[(N / 16) * 2], 8);
    if (N % 8) append(l.w[N / 8], N % 8);
  }
  KTJ_HD KTJ_FI void dec_wide(uint64_t v) {
    const uint64_t top = v / 10000000000000000ULL;
    const uint64_t rest = v - top * 10000000000000000ULL;
    const uint64_t mid = rest / 100000000ULL;
    const uint32_t low = (uint32_t)(rest - mid * 100000000ULL);
    uint64_t a0 = 0, a1;
    uint32_t n0 = 0, n1;
    if (top) {
      a0 = ascii8((uint32_t)top);
      const uint32_t z = leading_zero_chars(a0);
      a0 >>= 8 * z; n0 = 8 - z;
      a1 = ascii8((uint32_t)mid); n1 = 8;
    } else {
      a1 = ascii8((uint32_t)mid);
      const uint32_t z = leading_zero_chars(a1);
      a1 >>= 8 * z; n1 = 8 - z;
    }
    append(a0, n0);
    append(a1, n1);
    append(ascii8(low), 8);
  }
  KTJ_HD KTJ_FI void dec(uint64_t v) {
    if (__builtin_expect(v < 100000000ULL, 1)) {
      const uint64_t a = ascii8((uint32_t)v);
      const uint32_t z = leading_zero_chars(a);
      append(a >> (8 * z), 8 - z);
    } else dec_wide(v);
  }
  typedef Num Prepared;
  KTJ_HD KTJ_FI static Prepared prepare(uint64_t v) { return make_num(v); }
  KTJ_HD KTJ_FI void num(const Num& n) {
    if (__builtin_expect(n.len != 0, 1)) append(n.word, n.len); else dec_wide(n.value);
  }
  KTJ_HD KTJ_FI void dec3(uint32_t x) { append((uint64_t)(ascii4(x) >> 8), 3); }
  /* a dictionary string copied by this lane: aligned 8-byte loads, funnel-shifted, sixteen bytes
   * per append while they last */
  KTJ_HD KTJ_FI void str_own(const char* src, uint64_t len) { str_own_t<false>(src, len); }
  /* RELIEF: with a relief() every 32 bytes, for the one string of an activity that is often longer
   * than the stage has room for (a kernel's name; everywhere else the call would only be code in the way) */
  template <bool RELIEF> KTJ_HD KTJ_FI void str_own_t(const char* src, uint64_t len) {
    if (len == 0) return;
    const uintptr_t sa = (uintptr_t)src;
    const uint32_t sh = (uint32_t)(sa & 7u) * 8u;
#if defined(__HIP_DEVICE_COMPILE__)
    /* every string lives in a dictionary blob in device memory: global loads, not flat ones */
    typedef const __attribute__((address_space(1))) uint64_t* words;
#else
    typedef const uint64_t* words;
#endif
    words sp = reinterpret_cast<words>(sa & ~(uintptr_t)7);
    uint64_t cur = sp[0];
    const uint64_t full = len >> 3;
    uint64_t k = 0;
    KTJ_NOUNROLL
    for (; k + 2 <= full; k += 2) {
      if (RELIEF && (k & 2u) != 0) relief();
      const uint64_t n1 = sp[k + 1], n2 = sp[k + 2];
      append16(sh ? (cur >> sh) | (n1 << (64u - sh)) : cur, sh ? (n1 >> sh) | (n2 << (64u - sh)) : n1);
      cur = n2;
    }
    if (k < full) {
      const uint64_t next = sp[k + 1];
      append(sh ? (cur >> sh) | (next << (64u - sh)) : cur, 8);
      cur = next;
    }
    const uint32_t rem = (uint32_t)(len & 7u);
    if (rem) {
      uint64_t v = cur >> sh;
      if (sh && rem * 8u > 64u - sh) v |= sp[full + 1] << (64u - sh);
      append(v & ((1ULL << (8 * rem)) - 1ULL), rem);
    }
  }
  KTJ_HD KTJ_FI void str(const char* src, uint64_t len) { str_t<false>(src, len); }
  /* an activity's name */
  KTJ_HD KTJ_FI void name(const char* src, uint64_t len) { str_t<true>(src, len); }
  template <bool RELIEF> KTJ_HD KTJ_FI void str_t(const char* src, uint64_t len) {
#if defined(__HIP_DEVICE_COMPILE__)
    const bool big = len >= KTJ_COOP_MIN_BYTES;
    if (__any(big)) { /* see cooperative_word_copy */
      const char* body = src;
      uint64_t* dst = nullptr;
      uint32_t n_words = 0;
      uint64_t tail = 0;
      if (big) {
        const uint32_t head = (16u - fill) & 15u;   /* bytes that complete the block being gathered */
        str_own(src, head);                          /* now fill == 0 and the accumulator is empty */
        body = src + head;
        n_words = (uint32_t)((len - head) >> 4) * 2u; /* whole blocks, as words */
        tail = (len - head) & 15u;
        dst = wptr;
        stage_close();
        wptr += n_words;
      } else str_own_t<RELIEF>(src, len);
      cooperative_word_copy(body, dst, n_words);
      if (big) str_own(body + (uint64_t)n_words * 8u, tail);
      return;
    }
#endif
    str_own_t<RELIEF>(src, len);
  }
};

/* The last seven bytes of a formatted activity, by kind (see format_activity):
 *   0: `  \n  },`   complete event without args, or a flow-start event
 *   1: ` }\n  },`   complete or instant event with args and no flow event, or a counter event
 *   2: `e"\n  },`   flow-end event */
KTJ_HD KTJ_FI inline uint32_t tail_kind(const MatRow& r, bool has_args) {
  if (r.meta & KTJ_M_FLOW) return (r.meta & KTJ_M_FLOW_START) ? 0u : 2u;
  if (((r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT) == KTJ_CLASS_GENERIC) { /* counter events always close an args object */
    const uint32_t type = r.meta & KTJ_M_TYPE_MASK;
    if (type == KTJ_TYPE_HARDWARE_COUNTERS || type == KTJ_TYPE_MTIA_COUNTERS || type == KTJ_TYPE_XPU_SCOPE_PROFILER) return 1u;
  }
  return has_args ? 1u : 0u;
}
KTJ_HD KTJ_FI inline uint64_t tail_bytes(uint32_t kind, uint32_t count) { /* last `count` (0..7) bytes, low-aligned */
  constexpr auto t0 = pack_lit("  \n  },");
  constexpr auto t1 = pack_lit(" }\n  },");
  constexpr auto t2 = pack_lit("e\"\n  },");
  const uint64_t t = kind == 0 ? t0.w[0] : (kind == 1 ? t1.w[0] : t2.w[0]);
  return t >> (8 * (7 - count));
}

KTJ_HD KTJ_FI inline void BlockWriter::begin(char* doc, uint64_t pos, uint32_t tail_kind_before, bool first) {
  wptr = reinterpret_cast<uint64_t*>(doc + (pos & ~15ULL));
  fill = (uint32_t)(pos & 15ULL);
  lo = 0; hi = 0;
  foreign = false;
  if (fill == 0) return;
  if (first) { /* what precedes the first activity is in the document already */
    lo = wptr[0]; hi = wptr[1];
    if (fill < 8) { lo &= (1ULL << (8 * fill)) - 1ULL; hi = 0; }
    else if (fill > 8) hi &= (1ULL << (8 * (fill - 8))) - 1ULL;
    else hi = 0;
  } else if (fill < 8) lo = tail_bytes(tail_kind_before, fill);
  else foreign = true; /* the predecessor wrote this block, my first bytes included */
}
KTJ_HD KTJ_FI inline void BlockWriter::end(bool last) {
  if (fill == 0) return;
  if (last) { /* merge with the bytes that follow the last activity */
    if (fill < 8) { const uint64_t m = (1ULL << (8 * fill)) - 1ULL; lo |= wptr[0] & ~m; hi = wptr[1]; }
    else if (fill > 8) { const uint64_t m = (1ULL << (8 * (fill - 8))) - 1ULL; hi |= wptr[1] & ~m; }
    else hi = wptr[1];
    store_block();
    return;
  }
  if (fill >= 8) { /* my block: the successor's first bytes complete it */
    const uint32_t n = 16u - fill;
    append(n == 8 ? head_bytes() : head_bytes() & ((1ULL << (8 * n)) - 1ULL), n);
  }
}

/* ---------------------------------------------------------------------------------------- */
/* pieces                                                                                      */
/* ---------------------------------------------------------------------------------------- */
template <class W> KTJ_HD KTJ_FI inline void put_i64(W& w, int64_t v) {
  if (v < 0) { w.ch('-'); w.dec(0ULL - (uint64_t)v); } else w.dec((uint64_t)v);
}
/* fmtTs: "{}.{:03}" of ns/1000, ns%1000 for ns >= 0 (libkineto/src/output_json.cpp:124-126) */
template <class W> KTJ_HD KTJ_FI inline void put_ts(W& w, int64_t ns) {
  const uint64_t u = (uint64_t)ns;
  if ((u >> 32) == 0) {
    const uint32_t x = (uint32_t)u, us = x / 1000u;
    w.dec(us);
    w.ch('.');
    w.dec3(x - us * 1000u);
  } else {
    const uint64_t us = u / 1000;
    w.dec(us);
    w.ch('.');
    w.dec3((uint32_t)(u - us * 1000));
  }
}
template <class W> KTJ_HD KTJ_FI inline void put_hex(W& w, uint64_t v) { /* fmt "{}" of a pointer, after "0x" */
  int nd = 1;
  { uint64_t t = v; while (t >>= 4) ++nd; }
  KTJ_NOUNROLL
  for (int i = nd - 1; i >= 0; --i) {
    const uint32_t d = (uint32_t)(v >> (4 * i)) & 15u;
    w.ch((char)(d < 10 ? '0' + d : 'a' + d - 10));
  }
}
/* fmt "{}" of a double (TypedMetadataJson.h:172-178): shortest digits; fixed notation iff the
 * scientific exponent is in [-4, 16), else d[.ddd]e±XX; non-finite values are quoted */
KTJ_HD KTJ_FI inline char digit_of(uint64_t p0, uint64_t p1, uint64_t p2, int j) {
  const uint64_t word = j < 8 ? p0 : (j < 16 ? p1 : p2);
  return (char)(word >> (8 * (j & 7)));
}
template <class W> KTJ_HD KTJ_FI inline void put_f64(W& w, uint64_t bits, bool quote_non_finite = true) {
  const bool neg = (bits >> 63) != 0;
  const uint64_t mag = bits & 0x7FFFFFFFFFFFFFFFULL;
  if (mag >= 0x7FF0000000000000ULL) {
    if (quote_non_finite) w.ch('"');
    if (neg) w.ch('-');
    if (mag > 0x7FF0000000000000ULL) KTJ_PUT(w, "nan"); else KTJ_PUT(w, "inf");
    if (quote_non_finite) w.ch('"');
    return;
  }
  if (neg) w.ch('-');
  if (mag == 0) { w.ch('0'); return; }
  uint64_t sig;
  int32_t k;
  shortest_decimal(mag, &sig, &k);
  const int nd = ndigits_u64(sig);
  const int E = k + nd - 1;
  /* digits as up to three ascii8 words, left-aligned: digit i (0 = most significant) */
  uint64_t p0, p1, p2;
  {
    const uint64_t top = sig / 10000000000000000ULL;            /* digits 17.. */
    const uint64_t rest = sig - top * 10000000000000000ULL;
    const uint64_t mid = rest / 100000000ULL;
    p0 = ascii8((uint32_t)top); p1 = ascii8((uint32_t)mid); p2 = ascii8((uint32_t)(rest - mid * 100000000ULL));
  }
  const int lead = 24 - nd; /* leading zero characters of the 24-character string p0 p1 p2 */
#define digit(i) ::ktj::digit_of(p0, p1, p2, (i) + lead)
  if (E >= -4 && E < 16) {
    if (E >= 0) {
      int i = 0;
      KTJ_NOUNROLL
      for (; i <= E; ++i) w.ch(i < nd ? digit(i) : '0');
      if (nd > E + 1) {
        w.ch('.');
        KTJ_NOUNROLL
        for (; i < nd; ++i) w.ch(digit(i));
      }
    } else {
      w.ch('0'); w.ch('.');
      KTJ_NOUNROLL
      for (int i = 0; i < -E - 1; ++i) w.ch('0');
      KTJ_NOUNROLL
      for (int i = 0; i < nd; ++i) w.ch(digit(i));
    }
  } else {
    w.ch(digit(0));
    if (nd > 1) {
      w.ch('.');
      KTJ_NOUNROLL
      for (int i = 1; i < nd; ++i) w.ch(digit(i));
    }
    w.ch('e');
    int a = E;
    if (a < 0) { w.ch('-'); a = -a; } else w.ch('+');
    if (a >= 100) { w.ch((char)('0' + a / 100)); a %= 100; }
    w.ch((char)('0' + a / 10));
    w.ch((char)('0' + a % 10));
  }
#undef digit
}
/* same text into a caller buffer (>= 32 bytes); used by host-side checks */
struct BufferWriter {
  char* p; int n = 0;
  KTJ_HD KTJ_FI void ch(char c) { p[n++] = c; }
  template <unsigned N> KTJ_HD KTJ_FI void lit(const PackedLit<N>& l) { for (unsigned i = 0; i < N; ++i) p[n++] = (char)(l.w[i / 8] >> (8 * (i % 8))); }
};
KTJ_HD KTJ_FI inline int format_double(uint64_t bits, char* out) {
  BufferWriter b{out};
  put_f64(b, bits, false);
  return b.n;
}

template <class W> KTJ_HD KTJ_FI inline void put_arg_string(W& w, const DictViews& d, uint32_t id, bool raw = false) {
  if (id >= d.n) return;
  if (raw) w.str(d.raw_blob + d.raw_off[id], d.raw_off[id + 1] - d.raw_off[id]);
  else w.str(d.arg_blob + d.arg_off[id], d.arg_off[id + 1] - d.arg_off[id]);
}
template <class W> KTJ_HD KTJ_FI inline void put_array3(W& w, uint64_t a, uint64_t b, uint64_t c) {
  w.ch('['); put_i64(w, (int64_t)a); KTJ_PUT(w, ", "); put_i64(w, (int64_t)b); KTJ_PUT(w, ", ");
  put_i64(w, (int64_t)c); w.ch(']');
}

KTJ_HD KTJ_FI inline int64_t sanitize_tid(int64_t tid) { /* output_json.cpp:114-121 */
  if (tid == (int64_t)0x8000000000000000ULL) return 0;
  return tid < 0 ? -tid : tid;
}

/* libkineto/include/ActivityType.h:80-111 */
template <class W> KTJ_HD KTJ_FI inline void put_category(W& w, uint32_t type) {
  switch (type) {
    case 0: KTJ_PUT(w, "cpu_op"); break;
    case 1: KTJ_PUT(w, "user_annotation"); break;
    case 2: KTJ_PUT(w, "gpu_user_annotation"); break;
    case 3: KTJ_PUT(w, "gpu_memcpy"); break;
    case 4: KTJ_PUT(w, "gpu_memset"); break;
    case 5: KTJ_PUT(w, "kernel"); break;
    case 6: KTJ_PUT(w, "external_correlation"); break;
    case 7: KTJ_PUT(w, "cuda_runtime"); break;
    case 8: KTJ_PUT(w, "cuda_driver"); break;
    case 9: KTJ_PUT(w, "cpu_instant_event"); break;
    case 10: KTJ_PUT(w, "python_function"); break;
    case 11: KTJ_PUT(w, "overhead"); break;
    case 12: KTJ_PUT(w, "mtia_runtime"); break;
    case 13: KTJ_PUT(w, "mtia_ccp_events"); break;
    case 14: KTJ_PUT(w, "mtia_insight"); break;
    case 15: KTJ_PUT(w, "cuda_sync"); break;
    case 16: KTJ_PUT(w, "cuda_event"); break;
    case 17: KTJ_PUT(w, "mtia_counters"); break;
    case 18: KTJ_PUT(w, "glow_runtime"); break;
    case 19: KTJ_PUT(w, "cuda_profiler_range"); break;
    case 20: KTJ_PUT(w, "hpu_op"); break;
    case 21: KTJ_PUT(w, "xpu_runtime"); break;
    case 22: KTJ_PUT(w, "xpu_driver"); break;
    case 23: KTJ_PUT(w, "collective_comm"); break;
    case 24: KTJ_PUT(w, "privateuse1_runtime"); break;
    case 25: KTJ_PUT(w, "privateuse1_driver"); break;
    case 26: KTJ_PUT(w, "xpu_scope_profiler"); break;
    case 27: KTJ_PUT(w, "xpu_sync"); break;
    case 28: KTJ_PUT(w, "hardware_counters"); break;
    default: KTJ_PUT(w, "ENUM_COUNT"); break;
  }
}
/* libkineto/src/RocprofActivity_inl.h:50-94, 98-127 */
template <class W> KTJ_HD KTJ_FI inline void put_memcpy_name(W& w, uint32_t op) {
  switch (op) {
    case KTJ_COPY_H2H: KTJ_PUT(w, "Memcpy HtoH (Host -> Host)"); break;
    case KTJ_COPY_H2D: KTJ_PUT(w, "Memcpy HtoD (Host -> Device)"); break;
    case KTJ_COPY_D2H: KTJ_PUT(w, "Memcpy DtoH (Device -> Host)"); break;
    case KTJ_COPY_D2D: KTJ_PUT(w, "Memcpy DtoD (Device -> Device)"); break;
    default: KTJ_PUT(w, "Memcpy <unknown> (? -> ?)"); break;
  }
}
template <class W> KTJ_HD KTJ_FI inline void put_copy_kind(W& w, uint32_t op) {
  switch (op) {
    case KTJ_COPY_H2H: KTJ_PUT(w, "HtoH"); break;
    case KTJ_COPY_H2D: KTJ_PUT(w, "HtoD"); break;
    case KTJ_COPY_D2H: KTJ_PUT(w, "DtoH"); break;
    case KTJ_COPY_D2D: KTJ_PUT(w, "DtoD"); break;
    default: KTJ_PUT(w, "<unknown>"); break;
  }
}

/* a leading KTJ_F_COLLECTIVE field refers to collective metadata and is no part of the fragment */
KTJ_HD KTJ_FI inline uint32_t leading_collective(const ktj_schema_desc& sd, const EmitCtx& c) {
  return sd.n_fields != 0 && c.fields[sd.first_field].type == KTJ_F_COLLECTIVE ? 1u : 0u;
}
/* does this row print a metadata fragment?  (ArgsBuilder::appendFragment, output_json.cpp:173-181) */
KTJ_HD KTJ_FI inline bool has_fragment(const MatRow& r, const EmitCtx& c) {
  const uint32_t cls = (r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
  if (cls != KTJ_CLASS_GENERIC) return true;
  if (r.aux >= c.n_schemas) return false;
  const ktj_schema_desc sd = c.schemas[r.aux];
  const uint32_t skip = leading_collective(sd, c);
  if (sd.n_fields == skip) return false;
  if (sd.n_fields == skip + 1 && c.fields[sd.first_field + skip].key_id == KTJ_NONE &&
      c.fields[sd.first_field + skip].type == KTJ_F_RAW) { /* a whole pre-rendered fragment */
    if (r.p[0] + skip >= c.n_args) return false;
    const uint32_t id = (uint32_t)c.args[r.p[0] + skip];
    return id < c.dict.n && (c.dict.flags[id] & KTJ_SF_ARG_BLANK) == 0;
  }
  return true;
}
/* 1 + index of the collective metadata this row carries (appendCollectiveMetadata,
 * output_json.cpp:899-908), 0 = none */
KTJ_HD KTJ_FI inline uint32_t collective_of(const MatRow& r) {
  const uint32_t cls = (r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
  if (cls == KTJ_CLASS_GENERIC) return (uint32_t)r.p[1];
  if (cls == KTJ_CLASS_DEVICE && (r.meta & KTJ_M_TYPE_MASK) == KTJ_TYPE_CONCURRENT_KERNEL) return (uint32_t)r.p[4];
  return 0;
}
/* does the row append collective arguments?  An op without any of the keys appends nothing. */
KTJ_HD KTJ_FI inline bool has_collective_args(const MatRow& r, const EmitCtx& c) {
  const uint32_t k = collective_of(r);
  return k != 0 && k <= c.n_coll && c.coll_off[k] != c.coll_off[k - 1];
}
/* does the complete event of this row print an args object? */
KTJ_HD KTJ_FI inline bool has_args(const MatRow& r, const EmitCtx& c) {
  return r.ext != 0 || has_fragment(r, c) || has_collective_args(r, c);
}
/* Generic rows: a record with a linked op and a leading KTJ_F_COLLECTIVE field prints that
 * collective metadata itself if it is a kernel, or an MTIA event named "hccl::..."
 * (output_json.cpp:899-908). */
KTJ_HD KTJ_FI inline void attach_own_collective(MatRow& m, const ktj_generic_rec& g, const EmitCtx& c) {
  if (c.n_coll == 0 || !(g.flags & KTJ_GF_LINKED)) return;
  if (g.type == KTJ_TYPE_MTIA_CCP_EVENTS) {
    if (g.name_id >= c.dict.n || c.dict.raw_off[g.name_id + 1] - c.dict.raw_off[g.name_id] < 6) return;
    const char* nm = c.dict.raw_blob + c.dict.raw_off[g.name_id];
    if (nm[0] != 'h' || nm[1] != 'c' || nm[2] != 'c' || nm[3] != 'l' || nm[4] != ':' || nm[5] != ':') return;
  } else if (g.type != KTJ_TYPE_CONCURRENT_KERNEL) return;
  if (g.schema_id >= c.n_schemas || !leading_collective(c.schemas[g.schema_id], c) || g.args_off >= c.n_args) return;
  const uint64_t k = c.args[g.args_off];
  if (k < c.n_coll) m.p[1] = k + 1;
}
/* Generic rows other than those: the collective metadata handed to the kernels linked to them. */
KTJ_HD KTJ_FI inline uint32_t collective_for_linked(const ktj_generic_rec& g, const EmitCtx& c) {
  if (c.n_coll == 0 || g.type == KTJ_TYPE_CONCURRENT_KERNEL || g.type == KTJ_TYPE_MTIA_CCP_EVENTS) return 0;
  if (g.schema_id >= c.n_schemas || !leading_collective(c.schemas[g.schema_id], c) || g.args_off >= c.n_args) return 0;
  const uint64_t k = c.args[g.args_off];
  return k < c.n_coll ? (uint32_t)k + 1u : 0u;
}

/* one shape of `rank` dims at slot p: [d0, d1] */
template <class W> KTJ_HD KTJ_FI inline uint64_t put_shape(W& w, const EmitCtx& c, uint64_t p, uint64_t rank) {
  w.ch('[');
  KTJ_NOUNROLL
  for (uint64_t k = 0; k < rank; ++k) {
    if (k) KTJ_PUT(w, ", ");
    put_i64(w, (int64_t)(p + k < c.n_args ? c.args[p + k] : 0));
  }
  w.ch(']');
  return p + rank;
}
/* InputShapes through appendArray (TypedMetadataJson.h:52-64, 186-201); the encoding is described
 * at KTJ_F_SHAPES.  Counts are clipped to the blob, so a damaged encoding cannot run away. */
template <class W> KTJ_HD KTJ_FI inline void put_shapes(W& w, const EmitCtx& c, uint64_t p) {
  const uint64_t n = p < c.n_args ? c.args[p] : 0;
  ++p;
  w.ch('[');
  KTJ_NOUNROLL
  for (uint64_t e = 0; e < n && p < c.n_args; ++e) {
    if (e) KTJ_PUT(w, ", ");
    const uint64_t head = c.args[p++];
    const uint64_t m = head & 0xFFFFFFFFull;
    if (head & KTJ_SHAPE_LIST) {
      w.ch('[');
      KTJ_NOUNROLL
      for (uint64_t t = 0; t < m && p < c.n_args; ++t) {
        if (t) KTJ_PUT(w, ", ");
        const uint64_t rank = c.args[p++] & 0xFFFFFFFFull;
        p = put_shape(w, c, p, rank);
      }
      w.ch(']');
    } else p = put_shape(w, c, p, m);
  }
  w.ch(']');
}

/* the metadataJson() fragment, after sanitizeStrForJSON (raw: as metadataJson() returned it) */
template <class W> KTJ_HD KTJ_FI inline void put_fragment(W& w, const MatRow& r, const EmitCtx& c, bool raw = false) {
  const uint32_t cls = (r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
  const uint32_t kind = (r.meta & KTJ_M_KIND_MASK) >> KTJ_M_KIND_SHIFT;
  if (cls == KTJ_CLASS_GENERIC) { /* GenericTraceActivity.cpp:60-64 + TypedMetadataJson.h */
    const ktj_schema_desc sd = c.schemas[r.aux];
    uint64_t slot = r.p[0];
    bool first = true;
    for (uint32_t f = 0; f < sd.n_fields; ++f) {
      const ktj_field fd = c.fields[sd.first_field + f];
      if (fd.type == KTJ_F_COLLECTIVE) { slot += fd.count; continue; }
      if (fd.key_id != KTJ_NONE) { /* appendKey, TypedMetadataJson.h:145-152 */
        if (!first) KTJ_PUT(w, ", ");
        first = false;
        w.ch('"'); put_arg_string(w, c.dict, fd.key_id, raw); KTJ_PUT(w, "\": ");
      }
      const uint64_t v = slot < c.n_args ? c.args[slot] : 0;
      switch (fd.type) {
        case KTJ_F_DICT_BEGIN: w.ch('{'); first = true; break;   /* beginDict :128-132 */
        case KTJ_F_DICT_END: w.ch('}'); first = false; break;    /* endDict :134-137 */
        case KTJ_F_UNSUPPORTED: KTJ_PUT(w, "\"<unsupported metadata type>\""); break;
        case KTJ_F_STR_ARRAY:
          w.ch('[');
          for (uint32_t k = 0; k < fd.count; ++k) {
            if (k) KTJ_PUT(w, ", ");
            w.ch('"'); put_arg_string(w, c.dict, (uint32_t)(slot + k < c.n_args ? c.args[slot + k] : KTJ_NONE), raw); w.ch('"');
          }
          w.ch(']');
          break;
        case KTJ_F_SHAPES: put_shapes(w, c, v); break;
        case KTJ_F_I64: put_i64(w, (int64_t)v); break;
        case KTJ_F_U64: w.dec(v); break;
        case KTJ_F_F64: put_f64(w, v); break;
        case KTJ_F_BOOL: if (v) KTJ_PUT(w, "true"); else KTJ_PUT(w, "false"); break;
        case KTJ_F_STR: w.ch('"'); put_arg_string(w, c.dict, (uint32_t)v, raw); w.ch('"'); break;
        case KTJ_F_RAW: put_arg_string(w, c.dict, (uint32_t)v, raw); break;
        case KTJ_F_I64_ARRAY:
          w.ch('[');
          for (uint32_t k = 0; k < fd.count; ++k) {
            if (k) KTJ_PUT(w, ", ");
            put_i64(w, (int64_t)(slot + k < c.n_args ? c.args[slot + k] : 0));
          }
          w.ch(']');
          break;
        default: break;
      }
      slot += fd.count;
      w.relief();
    }
    return;
  }
  if (cls == KTJ_CLASS_RUNTIME) {
    switch (kind) {
      case KTJ_RT_KERNEL: /* RocprofActivity_inl.h:208-232 */
        if (r.meta & KTJ_M_HAS_KERNEL_ARG) {
          KTJ_PUT(w, "\"kernel\": \""); put_arg_string(w, c.dict, (uint32_t)r.p[4]); KTJ_PUT(w, "\", ");
        }
        KTJ_PUT(w, "\"cid\": "); w.dec(r.aux);
        KTJ_PUT(w, ", \"correlation\": "); w.dec((uint64_t)r.flow_id);
        w.relief();
        KTJ_PUT(w, ", \"grid\": "); put_array3(w, r.p[0] & 0xFFFFFFFFu, r.p[0] >> 32, r.p[1] & 0xFFFFFFFFu);
        KTJ_PUT(w, ", \"block\": "); put_array3(w, r.p[1] >> 32, r.p[2] & 0xFFFFFFFFu, r.p[2] >> 32);
        KTJ_PUT(w, ", \"shared memory\": "); w.dec(r.p[3]);
        break;
      case KTJ_RT_COPY: /* RocprofActivity_inl.h:243-255 */
        KTJ_PUT(w, "\"cid\": "); w.dec(r.aux);
        KTJ_PUT(w, ", \"correlation\": "); w.dec((uint64_t)r.flow_id);
        KTJ_PUT(w, ", \"src\": \"0x"); put_hex(w, r.p[0]);
        KTJ_PUT(w, "\", \"dst\": \"0x"); put_hex(w, r.p[1]);
        w.relief();
        KTJ_PUT(w, "\", \"bytes\": "); w.dec(r.p[2]);
        KTJ_PUT(w, ", \"kind\": \""); put_i64(w, (int64_t)(int32_t)(uint32_t)r.p[3]); w.ch('"');
        break;
      case KTJ_RT_MALLOC: /* RocprofActivity_inl.h:265-277 */
        if (r.meta & KTJ_M_MALLOC_BYTES) { KTJ_PUT(w, "\"bytes\": "); w.dec(r.p[1]); KTJ_PUT(w, ", "); }
        KTJ_PUT(w, "\"cid\": "); w.dec(r.aux);
        KTJ_PUT(w, ", \"correlation\": "); w.dec((uint64_t)r.flow_id);
        KTJ_PUT(w, ", \"ptr\": \"0x"); put_hex(w, r.p[0]); w.ch('"');
        break;
      default: /* RocprofActivity_inl.h:294-299 */
        KTJ_PUT(w, "\"cid\": "); w.dec(r.aux);
        KTJ_PUT(w, ", \"correlation\": "); w.dec((uint64_t)r.flow_id);
        break;
    }
    return;
  }
  /* device rows */
  if (kind == KTJ_DOM_MEMSET) { /* CuptiActivity.h:682-719, 460-470 */
    KTJ_PUT(w, "\"device\": "); put_i64(w, r.dev);
    KTJ_PUT(w, ", \"context\": "); w.dec(r.p[3]);
    KTJ_PUT(w, ", \"stream\": "); put_i64(w, r.res);
    KTJ_PUT(w, ", \"correlation\": "); w.dec((uint64_t)r.flow_id);
    KTJ_PUT(w, ", \"bytes\": "); w.dec(r.p[0]);
    w.relief();
    if (r.dur != 0) {
      const double bw = (double)r.p[0] / (double)r.dur;
      uint64_t bits; __builtin_memcpy(&bits, &bw, 8);
      KTJ_PUT(w, ", \"memory bandwidth (GB/s)\": "); put_f64(w, bits);
    }
    if (c.create_flags & KTJ_CREATE_CUDA12_ARGS) { /* CUDA_VERSION >= 12000: CuptiActivity.h:424-458 */
      KTJ_PUT(w, ", \"graph id\": "); w.dec(r.p[2] & 0xFFFFFFFFu);
      KTJ_PUT(w, ", \"graph node id\": "); w.dec(r.p[1]);
      KTJ_PUT(w, ", \"channel\": "); w.dec(r.p[2] >> 32);
      KTJ_PUT(w, ", \"channel_type\": "); w.dec(r.aux & 0xFFu);
    }
    return;
  }
  /* GpuActivity::visitTypedMetadata: RocprofActivity_inl.h:147-180 */
  KTJ_PUT(w, "\"device\": "); put_i64(w, r.dev);
  KTJ_PUT(w, ", \"stream\": "); put_i64(w, r.res);
  KTJ_PUT(w, ", \"hsa_queue\": "); w.dec(r.p[3]);
  KTJ_PUT(w, ", \"correlation\": "); w.dec((uint64_t)r.flow_id);
  w.relief();
  if (kind == KTJ_DOM_MEMORY_COPY) { KTJ_PUT(w, ", \"kind\": \""); put_copy_kind(w, r.aux); w.ch('"'); }
  else KTJ_PUT(w, ", \"kind\": \"Dispatch Kernel\"");
  if (r.meta & KTJ_M_HAS_SIZE) {
    KTJ_PUT(w, ", \"bytes\": "); w.dec(r.p[0]);
    const uint64_t raw_dur = (uint64_t)r.dur + 1; /* end - begin; duration() is end - (begin + 1) */
    if (raw_dur != 0) { /* RocprofActivity_inl.h:129-139 */
      const double bw = (double)r.p[0] / (double)raw_dur;
      uint64_t bits; __builtin_memcpy(&bits, &bw, 8);
      KTJ_PUT(w, ", \"memory bandwidth (GB/s)\": "); put_f64(w, bits);
    }
  } else if (r.meta & KTJ_M_HAS_GRID) {
    KTJ_PUT(w, ", \"grid\": "); put_array3(w, r.p[0] & 0xFFFFFFFFu, r.p[0] >> 32, r.p[1] & 0xFFFFFFFFu);
    KTJ_PUT(w, ", \"block\": "); put_array3(w, r.p[1] >> 32, r.p[2] & 0xFFFFFFFFu, r.p[2] >> 32);
  }
}

/* name after the logger's pipeline (output_json.cpp:946-949) */
template <class W> KTJ_HD KTJ_FI inline void put_name(W& w, const MatRow& r, const EmitCtx& c) {
  if (r.meta & KTJ_M_NAME_BUILTIN) {
    if (r.name_id <= 4) put_memcpy_name(w, r.name_id);
    else if (r.name_id == KTJ_NAME_MEMSET) { /* "Memset ({})" of memoryKindString, cupti_strings.cpp:42-66 */
      KTJ_PUT(w, "Memset (");
      switch ((r.aux >> 8) & 0xFFu) {
        case KTJ_MEMKIND_UNKNOWN: KTJ_PUT(w, "Unknown)"); break;
        case KTJ_MEMKIND_PAGEABLE: KTJ_PUT(w, "Pageable)"); break;
        case KTJ_MEMKIND_PINNED: KTJ_PUT(w, "Pinned)"); break;
        case KTJ_MEMKIND_DEVICE: KTJ_PUT(w, "Device)"); break;
        case KTJ_MEMKIND_ARRAY: KTJ_PUT(w, "Array)"); break;
        case KTJ_MEMKIND_MANAGED: KTJ_PUT(w, "Managed)"); break;
        case KTJ_MEMKIND_DEVICE_STATIC: KTJ_PUT(w, "Device Static)"); break;
        case KTJ_MEMKIND_MANAGED_STATIC: KTJ_PUT(w, "Managed Static)"); break;
        default: KTJ_PUT(w, "Unrecognized)"); break;
      }
    }
    else if (r.name_id == KTJ_NAME_UNKNOWN_OP) { KTJ_PUT(w, "<unknown operation:"); w.dec(r.aux); w.ch('>'); }
    return;
  }
  if (r.name_id < c.dict.n)
    w.name(c.dict.name_blob + c.dict.name_off[r.name_id], c.dict.name_off[r.name_id + 1] - c.dict.name_off[r.name_id]);
}

/* Generic rows only: marks a CUDA_SYNC activity named "Stream Sync" (output_json.cpp:915) and
 * whether it is the first of its (device, row) in emission order. */
KTJ_HD KTJ_FI inline void mark_stream_sync(MatRow& m, const EmitCtx& c, bool first_of_row) {
  if ((m.meta & KTJ_M_TYPE_MASK) != KTJ_TYPE_CUDA_SYNC || (m.meta & KTJ_M_NAME_BUILTIN) || m.name_id >= c.dict.n) return;
  if (!(c.dict.flags[m.name_id] & KTJ_SF_STREAM_SYNC)) return;
  m.meta |= KTJ_M_SYNC;
  if (first_of_row) m.meta |= KTJ_M_SYNC_FIRST;
}
/* resource + kSyncStreamTidOffset (output_json.cpp:916); a resource id near INT64_MAX wraps, as the
 * logger's own addition does on the machines it runs on */
KTJ_HD KTJ_FI inline int64_t sync_row_tid(int64_t resource) {
  return (int64_t)((uint64_t)resource + (uint64_t)KTJ_SYNC_TID_OFFSET);
}
/* (device << 32) | virtual tid, the key of syncStreamMetadataEmitted_ (output_json.cpp:917) */
KTJ_HD KTJ_FI inline uint64_t stream_sync_key(int64_t device, int64_t resource) {
  return ((uint64_t)device << 32) | (uint64_t)sync_row_tid(resource);
}

/* handleGenericInstantEvent + writeInstantEvent (output_json.cpp:660-677, 261-292): name and
 * metadata are printed as they were handed over, no flow event follows. */
template <class W> KTJ_HD KTJ_FI inline void format_instant(W& w, const MatRow& r, const EmitCtx& c) {
  int64_t rel = r.ts - c.base_time_ns;
  if (rel < 0) rel = 0;
  KTJ_PUT(w, "\n  {\n    \"ph\": \"i\",\n    \n    \"cat\": \"cpu_instant_event\",\n    \"s\": \"t\",\n    \"name\": \"");
  if (!(r.meta & KTJ_M_NAME_BUILTIN)) put_arg_string(w, c.dict, r.name_id, true);
  KTJ_PUT(w, "\",\n    \"pid\": "); put_i64(w, r.dev);
  KTJ_PUT(w, ",\n    \"tid\": "); w.dec((uint64_t)sanitize_tid(r.res));
  KTJ_PUT(w, ",\n    \"ts\": "); put_ts(w, rel);
  if (has_fragment(r, c)) {
    KTJ_PUT(w, "\n    ,\n    \"args\": {\n      ");
    put_fragment(w, r, c, true);
    KTJ_PUT(w, "\n    }\n  },");
  } else KTJ_PUT(w, "\n    \n  },");
}

KTJ_HD KTJ_FI inline bool is_counter_type(uint32_t type) { /* output_json.cpp:847-856 */
  return type == KTJ_TYPE_HARDWARE_COUNTERS || type == KTJ_TYPE_MTIA_COUNTERS || type == KTJ_TYPE_XPU_SCOPE_PROFILER;
}
/* A hardware-counter record prints one event per value (output_json.cpp:687-701): without values
 * it prints nothing and takes no place in the document.  Every other record prints something. */
KTJ_HD KTJ_FI inline bool generic_record_prints(const ktj_generic_rec& g, const EmitCtx& c) {
  if (g.type != KTJ_TYPE_HARDWARE_COUNTERS) return true;
  if (g.schema_id >= c.n_schemas) return false;
  const ktj_schema_desc sd = c.schemas[g.schema_id];
  for (uint32_t f = 0; f < sd.n_fields; ++f) {
    const ktj_field fd = c.fields[sd.first_field + f];
    if (fd.type == KTJ_F_F64 && fd.key_id != KTJ_NONE) return true;
  }
  return false;
}
/* handleCounterEvent + writeCounterEvent (output_json.cpp:679-716, 294-316).  The counter values
 * of a record are the keyed double fields of its schema.  Hardware counters give one event per
 * value on the device's "GPU <n> Counters" track; the other kinds one event holding all values.
 * Names are printed as they were handed over, non-finite values bare; no flow event follows. */
template <class W> KTJ_HD KTJ_FI inline void put_counter_head(W& w, uint32_t type) {
  KTJ_PUT(w, "\n  {\n    \"ph\": \"C\",\n    \"cat\": \""); put_category(w, type); KTJ_PUT(w, "\",\n    \"name\": \"");
}
template <class W> KTJ_HD KTJ_FI inline void format_counter(W& w, const MatRow& r, const EmitCtx& c) {
  const uint32_t type = r.meta & KTJ_M_TYPE_MASK;
  const bool hw = type == KTJ_TYPE_HARDWARE_COUNTERS;
  int64_t rel = r.ts - c.base_time_ns;
  if (rel < 0) rel = 0;
  const uint64_t tid = (uint64_t)sanitize_tid(r.res);
  ktj_schema_desc sd;
  sd.first_field = 0; sd.n_fields = 0;
  if (r.aux < c.n_schemas) sd = c.schemas[r.aux];
  if (!hw) {
    put_counter_head(w, type);
    if (!(r.meta & KTJ_M_NAME_BUILTIN)) put_arg_string(w, c.dict, r.name_id, true);
    KTJ_PUT(w, "\",\n    \"pid\": "); put_i64(w, r.dev);
    KTJ_PUT(w, ",\n    \"tid\": "); w.dec(tid);
    KTJ_PUT(w, ",\n    \"ts\": "); put_ts(w, rel);
    KTJ_PUT(w, ",\n    \"args\": {\n      ");
  }
  uint64_t slot = r.p[0];
  bool first = true;
  for (uint32_t f = 0; f < sd.n_fields; ++f) {
    const ktj_field fd = c.fields[sd.first_field + f];
    if (fd.type == KTJ_F_F64 && fd.key_id != KTJ_NONE) {
      const uint64_t v = slot < c.n_args ? c.args[slot] : 0;
      if (hw) {
        put_counter_head(w, type);
        put_arg_string(w, c.dict, fd.key_id, true);
        KTJ_PUT(w, "\",\n    \"pid\": \"GPU "); put_i64(w, r.dev); KTJ_PUT(w, " Counters\"");
        KTJ_PUT(w, ",\n    \"tid\": "); w.dec(tid);
        KTJ_PUT(w, ",\n    \"ts\": "); put_ts(w, rel);
        KTJ_PUT(w, ",\n    \"args\": {\n      \"\": "); put_f64(w, v, false);
        KTJ_PUT(w, "\n    }\n  },");
      } else {
        if (!first) w.ch(',');
        first = false;
        w.ch('"'); put_arg_string(w, c.dict, fd.key_id, true); KTJ_PUT(w, "\": "); put_f64(w, v, false);
      }
    }
    slot += fd.count;
  }
  if (!hw) KTJ_PUT(w, "\n    }\n  },");
}

/* One activity: the complete event and, if it takes part in a flow, the flow event after it.
 * Formatting comes in three parts that run one after the other — head (everything up to "dur", or
 * the whole event for instant and counter events), args, flow event — so that the emit kernel can
 * let the wavefront hand over finished blocks between them (BlockWriter::flush). */
template <class W> struct ActivityParts {
  typename W::Prepared pid, tidn;  /* printed by the complete event and again by the flow event */
  bool pid_neg;
  bool complete;                   /* a complete event: args and flow parts follow the head */
};
template <class W> KTJ_HD KTJ_FI inline void format_head(W& w, const MatRow& r, const EmitCtx& c, ActivityParts<W>& st) {
  const uint32_t type = r.meta & KTJ_M_TYPE_MASK;
  st.complete = false;
  st.pid_neg = false;
  st.pid = W::prepare(0);
  st.tidn = st.pid;
  if (((r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT) == KTJ_CLASS_GENERIC) {
    if (type == KTJ_TYPE_CPU_INSTANT_EVENT) { format_instant(w, r, c); return; }
    if (is_counter_type(type)) { format_counter(w, r, c); return; }
  }
  st.complete = true;
  int64_t ts = r.ts;
  int64_t dur = r.dur < 0 ? 0 : r.dur;                       /* output_json.cpp:860 */
  if (type == KTJ_TYPE_GPU_USER_ANNOTATION) { ts -= 1; dur += 2; } /* :862-869 */
  int64_t rel = ts - c.base_time_ns;                         /* transToRelativeTime :144-153 */
  if (rel < 0) rel = 0;
  /* Stream Sync activities sit on a row of their own (output_json.cpp:913-943, 1008-1013) */
  const int64_t tid = sanitize_tid((r.meta & KTJ_M_SYNC) ? sync_row_tid(r.res) : r.res);
  st.pid_neg = r.dev < 0;
  st.pid = W::prepare(st.pid_neg ? 0ULL - (uint64_t)r.dev : (uint64_t)r.dev);
  st.tidn = W::prepare((uint64_t)tid);
  if (r.meta & KTJ_M_SYNC_FIRST) { /* the row is announced once, before its first activity */
    KTJ_PUT(w, "\n  {\n    \"name\": \"thread_name\", \"ph\": \"M\", \"ts\": "); put_ts(w, rel);
    KTJ_PUT(w, ", \"pid\": "); put_i64(w, r.dev); KTJ_PUT(w, ", \"tid\": "); put_i64(w, sync_row_tid(r.res));
    KTJ_PUT(w, ",\n    \"args\": {\n      \"name\": \"stream "); put_i64(w, r.res); KTJ_PUT(w, " (sync)\"\n    }\n  },");
    KTJ_PUT(w, "\n  {\n    \"name\": \"thread_sort_index\", \"ph\": \"M\", \"ts\": "); put_ts(w, rel);
    KTJ_PUT(w, ", \"pid\": "); put_i64(w, r.dev); KTJ_PUT(w, ", \"tid\": "); put_i64(w, sync_row_tid(r.res));
    KTJ_PUT(w, ",\n    \"args\": {\n      \"sort_index\": "); put_i64(w, r.res); KTJ_PUT(w, "\n    }\n  },");
  }
  KTJ_PUT(w, "\n  {\n    \"ph\": \"X\",\n    \"cat\": \"");
  put_category(w, type);
  KTJ_PUT(w, "\",\n    \"name\": \"");
  put_name(w, r, c);
  w.relief();
  KTJ_PUT(w, "\",\n    \"pid\": "); if (st.pid_neg) w.ch('-'); w.num(st.pid);
  KTJ_PUT(w, ",\n    \"tid\": "); w.num(st.tidn);
  KTJ_PUT(w, ",\n    \"ts\": "); put_ts(w, rel);
  KTJ_PUT(w, ",\n    \"dur\": "); put_ts(w, dur);
}
template <class W> KTJ_HD KTJ_FI inline void format_args(W& w, const MatRow& r, const EmitCtx& c, const ActivityParts<W>& st) {
  if (!st.complete) return;
  const bool frag = has_fragment(r, c);
  const bool coll = has_collective_args(r, c);
  if (r.ext != 0 || frag || coll) {                          /* ArgsBuilder :157-212 */
    KTJ_PUT(w, "\n    ,\n    \"args\": {\n      ");
    if (r.ext != 0) { KTJ_PUT(w, "\"External id\": "); put_i64(w, r.ext); }
    if (frag) { if (r.ext != 0) w.ch(','); put_fragment(w, r, c); }
    if (coll) { /* appendCollectiveMetadata :899-908: printed as the op's values were handed over */
      if (r.ext != 0 || frag) w.ch(',');
      const uint32_t k = collective_of(r);
      w.str(c.coll_blob + c.coll_off[k - 1], c.coll_off[k] - c.coll_off[k - 1]);
    }
    KTJ_PUT(w, "\n    }\n  },");
  } else KTJ_PUT(w, "\n    \n  },");
}
template <class W> KTJ_HD KTJ_FI inline void format_flow(W& w, const MatRow& r, const EmitCtx& c, const ActivityParts<W>& st) {
  if (!st.complete || !(r.meta & KTJ_M_FLOW)) return;       /* :960-1021, writeFlowEvent :318-345 */
  int64_t frel = r.ts - c.base_time_ns;
  if (frel < 0) frel = 0;
  if (r.meta & KTJ_M_FLOW_START) KTJ_PUT(w, "\n  {\n    \"ph\": \"s\",\n    \"id\": ");
  else KTJ_PUT(w, "\n  {\n    \"ph\": \"f\",\n    \"id\": ");
  put_i64(w, r.flow_id);
  KTJ_PUT(w, ",\n    \"pid\": "); if (st.pid_neg) w.ch('-'); w.num(st.pid);
  KTJ_PUT(w, ",\n    \"tid\": "); w.num(st.tidn);
  w.relief();
  KTJ_PUT(w, ",\n    \"ts\": "); put_ts(w, frel);
  if (r.meta & KTJ_M_FLOW_FWDBWD) KTJ_PUT(w, ",\n    \"cat\": \"fwdbwd\",\n    \"name\": \"fwdbwd\"\n    ");
  else KTJ_PUT(w, ",\n    \"cat\": \"ac2g\",\n    \"name\": \"ac2g\"\n    ");
  if (r.meta & KTJ_M_FLOW_START) KTJ_PUT(w, "\n  },"); else KTJ_PUT(w, ", \"bp\": \"e\"\n  },");
}
template <class W> KTJ_HD KTJ_FI inline void format_activity(W& w, const MatRow& r, const EmitCtx& c) {
  ActivityParts<W> st;
  format_head(w, r, c, st);
  format_args(w, r, c, st);
  format_flow(w, r, c, st);
}

}  // namespace ktj
#endif
