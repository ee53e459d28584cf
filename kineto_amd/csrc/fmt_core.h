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
KTJ_HD inline int ndigits_u64(uint64_t v) {
  int n = 1;
  if (v >= 10000000000ULL) { v /= 10000000000ULL; n += 10; }
  uint32_t x = (uint32_t)v; /* < 10^10 may exceed 32 bits */
  if (v >= 100000000ULL) { x = (uint32_t)(v / 100000000ULL); n += 8; }
  if (x >= 10000u) { x /= 10000u; n += 4; }
  if (x >= 100u) { x /= 100u; n += 2; }
  if (x >= 10u) { n += 1; }
  return n;
}

KTJ_HD inline uint64_t mulhi64(uint64_t a, uint64_t b) {
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
KTJ_HD inline int32_t floor_log2_pow10(int32_t e) { return (e * 1741647) >> 19; }
KTJ_HD inline int32_t floor_log10_pow2(int32_t e) { return (e * 1262611) >> 22; }
KTJ_HD inline int32_t floor_log10_3q_pow2(int32_t e) { return (e * 1262611 - 524031) >> 22; }

KTJ_HD inline uint64_t round_to_odd(uint64_t ghi, uint64_t glo, uint64_t cp) {
  /* (cp * g) >> 128 with a sticky low bit; g = ghi:glo */
  uint64_t x_hi = mulhi64(cp, glo);
  uint64_t y_lo = cp * ghi;
  uint64_t y_hi = mulhi64(cp, ghi);
  uint64_t s_lo = y_lo + x_hi;
  uint64_t carry = s_lo < y_lo ? 1 : 0;
  uint64_t y1 = y_hi + carry;
  return y1 | (s_lo > 1 ? 1 : 0);
}

KTJ_HD inline void shortest_decimal(uint64_t bits, uint64_t* digits, int32_t* exp10) {
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

/* fmt "{}" of a double into out (>= 32 bytes); returns the length.
 * Layout rule of fmt's write_float with default specs: fixed notation iff the scientific
 * exponent is in [-4, 16), else d[.ddd]e±XX with at least two exponent digits. */
KTJ_HD inline int format_double(uint64_t bits, char* out) {
  int n = 0;
  const bool neg = (bits >> 63) != 0;
  const uint64_t mag = bits & 0x7FFFFFFFFFFFFFFFULL;
  if (neg) out[n++] = '-';
  if (mag >= 0x7FF0000000000000ULL) { /* fmt prints "inf" / "nan" */
    const bool is_nan = mag > 0x7FF0000000000000ULL;
    out[n++] = is_nan ? 'n' : 'i';
    out[n++] = is_nan ? 'a' : 'n';
    out[n++] = is_nan ? 'n' : 'f';
    return n;
  }
  if (mag == 0) { out[n++] = '0'; return n; }
  uint64_t sig;
  int32_t k;
  shortest_decimal(mag, &sig, &k);
  const int nd = ndigits_u64(sig);
  const int E = k + nd - 1;
  char d[20];
  { uint64_t t = sig; for (int i = nd - 1; i >= 0; --i) { d[i] = (char)('0' + (int)(t % 10)); t /= 10; } }
  if (E >= -4 && E < 16) {
    if (E >= 0) {
      int i = 0;
      for (; i <= E; ++i) out[n++] = i < nd ? d[i] : '0';
      if (nd > E + 1) { out[n++] = '.'; for (; i < nd; ++i) out[n++] = d[i]; }
    } else {
      out[n++] = '0'; out[n++] = '.';
      for (int i = 0; i < -E - 1; ++i) out[n++] = '0';
      for (int i = 0; i < nd; ++i) out[n++] = d[i];
    }
  } else {
    out[n++] = d[0];
    if (nd > 1) { out[n++] = '.'; for (int i = 1; i < nd; ++i) out[n++] = d[i]; }
    out[n++] = 'e';
    int a = E;
    if (a < 0) { out[n++] = '-'; a = -a; } else out[n++] = '+';
    if (a >= 100) { out[n++] = (char)('0' + a / 100); a %= 100; }
    out[n++] = (char)('0' + a / 10);
    out[n++] = (char)('0' + a % 10);
  }
  return n;
}

/* ---------------------------------------------------------------------------------------- */
/* clock conversion: (int64)((double)(t - t0_approx) * (long double)scale) + t0, exactly as    */
/* x87 extended precision computes it (libkineto/src/ApproximateClock.cpp:83-90): the exact    */
/* 106-bit product of two 53-bit significands is rounded to 64 bits (nearest even) and the     */
/* result truncated toward zero.                                                               */
/* ---------------------------------------------------------------------------------------- */
KTJ_HD inline int64_t convert_timestamp(uint64_t t, uint64_t t0_approx, int64_t t0, uint64_t scale_bits) {
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
/* constant strings                                                                            */
/* ---------------------------------------------------------------------------------------- */
struct Lit { const char* p; uint32_t n; };
#define KTJ_LIT(s) ::ktj::Lit{s, (uint32_t)(sizeof(s) - 1)}

/* libkineto/include/ActivityType.h:80-111 */
KTJ_HD inline Lit category_name(uint32_t type) {
  switch (type) {
    case 0: return KTJ_LIT("cpu_op");
    case 1: return KTJ_LIT("user_annotation");
    case 2: return KTJ_LIT("gpu_user_annotation");
    case 3: return KTJ_LIT("gpu_memcpy");
    case 4: return KTJ_LIT("gpu_memset");
    case 5: return KTJ_LIT("kernel");
    case 6: return KTJ_LIT("external_correlation");
    case 7: return KTJ_LIT("cuda_runtime");
    case 8: return KTJ_LIT("cuda_driver");
    case 9: return KTJ_LIT("cpu_instant_event");
    case 10: return KTJ_LIT("python_function");
    case 11: return KTJ_LIT("overhead");
    case 12: return KTJ_LIT("mtia_runtime");
    case 13: return KTJ_LIT("mtia_ccp_events");
    case 14: return KTJ_LIT("mtia_insight");
    case 15: return KTJ_LIT("cuda_sync");
    case 16: return KTJ_LIT("cuda_event");
    case 17: return KTJ_LIT("mtia_counters");
    case 18: return KTJ_LIT("glow_runtime");
    case 19: return KTJ_LIT("cuda_profiler_range");
    case 20: return KTJ_LIT("hpu_op");
    case 21: return KTJ_LIT("xpu_runtime");
    case 22: return KTJ_LIT("xpu_driver");
    case 23: return KTJ_LIT("collective_comm");
    case 24: return KTJ_LIT("privateuse1_runtime");
    case 25: return KTJ_LIT("privateuse1_driver");
    case 26: return KTJ_LIT("xpu_scope_profiler");
    case 27: return KTJ_LIT("xpu_sync");
    case 28: return KTJ_LIT("hardware_counters");
    default: return KTJ_LIT("ENUM_COUNT");
  }
}

/* libkineto/src/RocprofActivity_inl.h:50-94, 98-127 */
KTJ_HD inline Lit memcpy_name(uint32_t op) {
  switch (op) {
    case KTJ_COPY_H2H: return KTJ_LIT("Memcpy HtoH (Host -> Host)");
    case KTJ_COPY_H2D: return KTJ_LIT("Memcpy HtoD (Host -> Device)");
    case KTJ_COPY_D2H: return KTJ_LIT("Memcpy DtoH (Device -> Host)");
    case KTJ_COPY_D2D: return KTJ_LIT("Memcpy DtoD (Device -> Device)");
    default: return KTJ_LIT("Memcpy <unknown> (? -> ?)");
  }
}
KTJ_HD inline Lit copy_kind_string(uint32_t op) {
  switch (op) {
    case KTJ_COPY_H2H: return KTJ_LIT("HtoH");
    case KTJ_COPY_H2D: return KTJ_LIT("HtoD");
    case KTJ_COPY_D2H: return KTJ_LIT("DtoH");
    case KTJ_COPY_D2D: return KTJ_LIT("DtoD");
    default: return KTJ_LIT("<unknown>");
  }
}

/* ---------------------------------------------------------------------------------------- */
/* writers                                                                                     */
/* ---------------------------------------------------------------------------------------- */
/* Pass A: exact byte length. */
struct CountWriter {
  uint64_t n = 0;
  KTJ_HD void ch(char) { ++n; }
  KTJ_HD void lit(Lit l) { n += l.n; }
  KTJ_HD void local(const char*, int len) { n += (uint32_t)len; }
  KTJ_HD void dec(uint64_t v) { n += (uint32_t)ndigits_u64(v); }
  KTJ_HD void dec3(uint32_t) { n += 3; }
  KTJ_HD void hex(uint64_t v) { int d = 1; while (v >>= 4) ++d; n += (uint32_t)d; }
  KTJ_HD void str(const char*, uint64_t len) { n += len; }
};

/* Pass B: bytes into one tile of the output.  `pos` is relative to the tile's first byte and may
 * lie outside [0, tile): everything is clipped.  Dictionary strings are not copied here but
 * queued as copy jobs that the whole workgroup executes afterwards with wide lanes. */
struct CopyJob { const char* src; int32_t dst; uint32_t len; };

struct TileWriter {
  char* buf;
  int32_t pos;
  int32_t tile;
  CopyJob* jobs;
  uint32_t* n_jobs;
  uint32_t max_jobs;

  KTJ_HD void put(int32_t p, char c) { if ((uint32_t)p < (uint32_t)tile) buf[p] = c; }
  KTJ_HD void ch(char c) { put(pos, c); ++pos; }
  KTJ_HD void copy_clipped(const char* s, uint32_t n) {
    int32_t b = pos < 0 ? -pos : 0;
    int64_t room = (int64_t)tile - pos;
    int32_t e = (int64_t)n < room ? (int32_t)n : (int32_t)(room < 0 ? 0 : room);
    for (int32_t i = b; i < e; ++i) buf[pos + i] = s[i];
  }
  KTJ_HD void lit(Lit l) { copy_clipped(l.p, l.n); pos += (int32_t)l.n; }
  KTJ_HD void local(const char* s, int len) { copy_clipped(s, (uint32_t)len); pos += len; }
  KTJ_HD void dec(uint64_t v) {
    const int nd = ndigits_u64(v);
    int32_t p = pos + nd - 1;
    if (v >> 32) {
      for (int i = 0; i < nd; ++i, --p) { const uint64_t q = v / 10; put(p, (char)('0' + (int)(v - q * 10))); v = q; }
    } else {
      uint32_t x = (uint32_t)v;
      for (int i = 0; i < nd; ++i, --p) { const uint32_t q = x / 10; put(p, (char)('0' + (int)(x - q * 10))); x = q; }
    }
    pos += nd;
  }
  KTJ_HD void dec3(uint32_t x) { /* {:03} of 0..999 */
    put(pos + 2, (char)('0' + x % 10)); x /= 10;
    put(pos + 1, (char)('0' + x % 10)); x /= 10;
    put(pos, (char)('0' + x));
    pos += 3;
  }
  KTJ_HD void hex(uint64_t v) {
    int nd = 1; { uint64_t t = v; while (t >>= 4) ++nd; }
    int32_t p = pos + nd - 1;
    for (int i = 0; i < nd; ++i, --p) { const uint32_t d = (uint32_t)(v & 15); put(p, (char)(d < 10 ? '0' + d : 'a' + d - 10)); v >>= 4; }
    pos += nd;
  }
  KTJ_HD void str(const char* src, uint64_t len) {
    if (len == 0) return;
    int64_t b = pos < 0 ? -(int64_t)pos : 0;
    int64_t room = (int64_t)tile - pos;
    int64_t e = (int64_t)len < room ? (int64_t)len : (room < 0 ? 0 : room);
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
      } else { /* queue full: copy here */
        for (int64_t i = b; i < e; ++i) buf[pos + i] = src[i];
      }
    }
    pos += (int32_t)len;
  }
};

/* ---------------------------------------------------------------------------------------- */
/* pieces                                                                                      */
/* ---------------------------------------------------------------------------------------- */
template <class W> KTJ_HD inline void put_i64(W& w, int64_t v) {
  if (v < 0) { w.ch('-'); w.dec(0ULL - (uint64_t)v); } else w.dec((uint64_t)v);
}
/* fmtTs: "{}.{:03}" of ns/1000, ns%1000 for ns >= 0 (libkineto/src/output_json.cpp:124-126) */
template <class W> KTJ_HD inline void put_ts(W& w, int64_t ns) {
  const uint64_t u = (uint64_t)ns;
  const uint64_t us = u / 1000;
  w.dec(us);
  w.ch('.');
  w.dec3((uint32_t)(u - us * 1000));
}
template <class W> KTJ_HD inline void put_f64(W& w, uint64_t bits) { /* TypedMetadataJson.h:172-178 */
  char tmp[32];
  const int n = format_double(bits, tmp);
  const bool finite = (bits & 0x7FF0000000000000ULL) != 0x7FF0000000000000ULL;
  if (!finite) w.ch('"');
  w.local(tmp, n);
  if (!finite) w.ch('"');
}
template <class W> KTJ_HD inline void put_arg_string(W& w, const DictViews& d, uint32_t id) {
  if (id < d.n) w.str(d.arg_blob + d.arg_off[id], d.arg_off[id + 1] - d.arg_off[id]);
}
template <class W> KTJ_HD inline void put_array3(W& w, uint64_t a, uint64_t b, uint64_t c) {
  w.ch('['); put_i64(w, (int64_t)a); w.lit(KTJ_LIT(", ")); put_i64(w, (int64_t)b); w.lit(KTJ_LIT(", "));
  put_i64(w, (int64_t)c); w.ch(']');
}

KTJ_HD inline int64_t sanitize_tid(int64_t tid) { /* output_json.cpp:114-121 */
  if (tid == (int64_t)0x8000000000000000ULL) return 0;
  return tid < 0 ? -tid : tid;
}

/* does this row print a metadata fragment?  (ArgsBuilder::appendFragment, output_json.cpp:173-181) */
KTJ_HD inline bool has_fragment(const MatRow& r, const EmitCtx& c) {
  const uint32_t cls = (r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
  if (cls != KTJ_CLASS_GENERIC) return true;
  if (r.aux >= c.n_schemas) return false;
  const ktj_schema_desc sd = c.schemas[r.aux];
  if (sd.n_fields == 0) return false;
  if (sd.n_fields == 1 && c.fields[sd.first_field].key_id == KTJ_NONE &&
      c.fields[sd.first_field].type == KTJ_F_RAW) { /* a whole pre-rendered fragment */
    if (r.p[0] >= c.n_args) return false;
    const uint32_t id = (uint32_t)c.args[r.p[0]];
    return id < c.dict.n && (c.dict.flags[id] & KTJ_SF_ARG_BLANK) == 0;
  }
  return true;
}

/* the metadataJson() fragment, after sanitizeStrForJSON */
template <class W> KTJ_HD inline void put_fragment(W& w, const MatRow& r, const EmitCtx& c) {
  const uint32_t cls = (r.meta & KTJ_M_CLASS_MASK) >> KTJ_M_CLASS_SHIFT;
  const uint32_t kind = (r.meta & KTJ_M_KIND_MASK) >> KTJ_M_KIND_SHIFT;
  if (cls == KTJ_CLASS_GENERIC) { /* GenericTraceActivity.cpp:60-64 + TypedMetadataJson.h */
    const ktj_schema_desc sd = c.schemas[r.aux];
    uint64_t slot = r.p[0];
    bool first = true;
    for (uint32_t f = 0; f < sd.n_fields; ++f) {
      const ktj_field fd = c.fields[sd.first_field + f];
      if (fd.key_id != KTJ_NONE) {
        if (!first) w.lit(KTJ_LIT(", "));
        first = false;
        w.ch('"'); put_arg_string(w, c.dict, fd.key_id); w.lit(KTJ_LIT("\": "));
      }
      const uint64_t v = slot < c.n_args ? c.args[slot] : 0;
      switch (fd.type) {
        case KTJ_F_I64: put_i64(w, (int64_t)v); break;
        case KTJ_F_U64: w.dec(v); break;
        case KTJ_F_F64: put_f64(w, v); break;
        case KTJ_F_BOOL: if (v) w.lit(KTJ_LIT("true")); else w.lit(KTJ_LIT("false")); break;
        case KTJ_F_STR: w.ch('"'); put_arg_string(w, c.dict, (uint32_t)v); w.ch('"'); break;
        case KTJ_F_RAW: put_arg_string(w, c.dict, (uint32_t)v); break;
        case KTJ_F_I64_ARRAY:
          w.ch('[');
          for (uint32_t k = 0; k < fd.count; ++k) {
            if (k) w.lit(KTJ_LIT(", "));
            put_i64(w, (int64_t)(slot + k < c.n_args ? c.args[slot + k] : 0));
          }
          w.ch(']');
          break;
        default: break;
      }
      slot += fd.count;
    }
    return;
  }
  if (cls == KTJ_CLASS_RUNTIME) {
    switch (kind) {
      case KTJ_RT_KERNEL: /* RocprofActivity_inl.h:208-232 */
        if (r.meta & KTJ_M_HAS_KERNEL_ARG) {
          w.lit(KTJ_LIT("\"kernel\": \"")); put_arg_string(w, c.dict, (uint32_t)r.p[4]); w.lit(KTJ_LIT("\", "));
        }
        w.lit(KTJ_LIT("\"cid\": ")); w.dec(r.aux);
        w.lit(KTJ_LIT(", \"correlation\": ")); w.dec((uint64_t)r.flow_id);
        w.lit(KTJ_LIT(", \"grid\": ")); put_array3(w, r.p[0] & 0xFFFFFFFFu, r.p[0] >> 32, r.p[1] & 0xFFFFFFFFu);
        w.lit(KTJ_LIT(", \"block\": ")); put_array3(w, r.p[1] >> 32, r.p[2] & 0xFFFFFFFFu, r.p[2] >> 32);
        w.lit(KTJ_LIT(", \"shared memory\": ")); w.dec(r.p[3]);
        break;
      case KTJ_RT_COPY: /* RocprofActivity_inl.h:243-255 */
        w.lit(KTJ_LIT("\"cid\": ")); w.dec(r.aux);
        w.lit(KTJ_LIT(", \"correlation\": ")); w.dec((uint64_t)r.flow_id);
        w.lit(KTJ_LIT(", \"src\": \"0x")); w.hex(r.p[0]);
        w.lit(KTJ_LIT("\", \"dst\": \"0x")); w.hex(r.p[1]);
        w.lit(KTJ_LIT("\", \"bytes\": ")); w.dec(r.p[2]);
        w.lit(KTJ_LIT(", \"kind\": \"")); put_i64(w, (int64_t)(int32_t)(uint32_t)r.p[3]); w.ch('"');
        break;
      case KTJ_RT_MALLOC: /* RocprofActivity_inl.h:265-277 */
        if (r.meta & KTJ_M_MALLOC_BYTES) { w.lit(KTJ_LIT("\"bytes\": ")); w.dec(r.p[1]); w.lit(KTJ_LIT(", ")); }
        w.lit(KTJ_LIT("\"cid\": ")); w.dec(r.aux);
        w.lit(KTJ_LIT(", \"correlation\": ")); w.dec((uint64_t)r.flow_id);
        w.lit(KTJ_LIT(", \"ptr\": \"0x")); w.hex(r.p[0]); w.ch('"');
        break;
      default: /* RocprofActivity_inl.h:294-299 */
        w.lit(KTJ_LIT("\"cid\": ")); w.dec(r.aux);
        w.lit(KTJ_LIT(", \"correlation\": ")); w.dec((uint64_t)r.flow_id);
        break;
    }
    return;
  }
  /* device rows */
  if (kind == KTJ_DOM_MEMSET) { /* CuptiActivity.h:682-713, 460-470 */
    w.lit(KTJ_LIT("\"device\": ")); put_i64(w, r.dev);
    w.lit(KTJ_LIT(", \"context\": ")); w.dec(r.p[3]);
    w.lit(KTJ_LIT(", \"stream\": ")); put_i64(w, r.res);
    w.lit(KTJ_LIT(", \"correlation\": ")); w.dec((uint64_t)r.flow_id);
    w.lit(KTJ_LIT(", \"bytes\": ")); w.dec(r.p[0]);
    if (r.dur != 0) {
      const double bw = (double)r.p[0] / (double)r.dur;
      uint64_t bits; __builtin_memcpy(&bits, &bw, 8);
      w.lit(KTJ_LIT(", \"memory bandwidth (GB/s)\": ")); put_f64(w, bits);
    }
    return;
  }
  /* GpuActivity::visitTypedMetadata: RocprofActivity_inl.h:147-180 */
  w.lit(KTJ_LIT("\"device\": ")); put_i64(w, r.dev);
  w.lit(KTJ_LIT(", \"stream\": ")); put_i64(w, r.res);
  w.lit(KTJ_LIT(", \"hsa_queue\": ")); w.dec(r.p[3]);
  w.lit(KTJ_LIT(", \"correlation\": ")); w.dec((uint64_t)r.flow_id);
  w.lit(KTJ_LIT(", \"kind\": \""));
  if (kind == KTJ_DOM_MEMORY_COPY) w.lit(copy_kind_string(r.aux)); else w.lit(KTJ_LIT("Dispatch Kernel"));
  w.ch('"');
  if (r.meta & KTJ_M_HAS_SIZE) {
    w.lit(KTJ_LIT(", \"bytes\": ")); w.dec(r.p[0]);
    const uint64_t raw_dur = (uint64_t)r.dur + 1; /* end - begin; duration() is end - (begin + 1) */
    if (raw_dur != 0) { /* RocprofActivity_inl.h:129-139 */
      const double bw = (double)r.p[0] / (double)raw_dur;
      uint64_t bits; __builtin_memcpy(&bits, &bw, 8);
      w.lit(KTJ_LIT(", \"memory bandwidth (GB/s)\": ")); put_f64(w, bits);
    }
  } else if (r.meta & KTJ_M_HAS_GRID) {
    w.lit(KTJ_LIT(", \"grid\": ")); put_array3(w, r.p[0] & 0xFFFFFFFFu, r.p[0] >> 32, r.p[1] & 0xFFFFFFFFu);
    w.lit(KTJ_LIT(", \"block\": ")); put_array3(w, r.p[1] >> 32, r.p[2] & 0xFFFFFFFFu, r.p[2] >> 32);
  }
}

/* name after the logger's pipeline (output_json.cpp:946-949) */
template <class W> KTJ_HD inline void put_name(W& w, const MatRow& r, const EmitCtx& c) {
  if (r.meta & KTJ_M_NAME_BUILTIN) {
    if (r.name_id <= 4) w.lit(memcpy_name(r.name_id));
    else if (r.name_id == KTJ_NAME_MEMSET) w.lit(KTJ_LIT("Memset (Device)"));
    else if (r.name_id == KTJ_NAME_UNKNOWN_OP) { w.lit(KTJ_LIT("<unknown operation:")); w.dec(r.aux); w.ch('>'); }
    return;
  }
  if (r.name_id < c.dict.n)
    w.str(c.dict.name_blob + c.dict.name_off[r.name_id], c.dict.name_off[r.name_id + 1] - c.dict.name_off[r.name_id]);
}

/* One activity: the complete event and, if it takes part in a flow, the flow event after it. */
template <class W> KTJ_HD inline void format_activity(W& w, const MatRow& r, const EmitCtx& c) {
  const uint32_t type = r.meta & KTJ_M_TYPE_MASK;
  int64_t ts = r.ts;
  int64_t dur = r.dur < 0 ? 0 : r.dur;                       /* output_json.cpp:860 */
  if (type == KTJ_TYPE_GPU_USER_ANNOTATION) { ts -= 1; dur += 2; } /* :862-869 */
  int64_t rel = ts - c.base_time_ns;                         /* transToRelativeTime :144-153 */
  if (rel < 0) rel = 0;
  const int64_t tid = sanitize_tid(r.res);
  w.lit(KTJ_LIT("\n  {\n    \"ph\": \"X\",\n    \"cat\": \""));
  w.lit(category_name(type));
  w.lit(KTJ_LIT("\",\n    \"name\": \""));
  put_name(w, r, c);
  w.lit(KTJ_LIT("\",\n    \"pid\": ")); put_i64(w, r.dev);
  w.lit(KTJ_LIT(",\n    \"tid\": ")); put_i64(w, tid);
  w.lit(KTJ_LIT(",\n    \"ts\": ")); put_ts(w, rel);
  w.lit(KTJ_LIT(",\n    \"dur\": ")); put_ts(w, dur);
  w.lit(KTJ_LIT("\n    "));
  const bool frag = has_fragment(r, c);
  if (r.ext != 0 || frag) {                                  /* ArgsBuilder :157-212 */
    w.lit(KTJ_LIT(",\n    \"args\": {\n      "));
    if (r.ext != 0) { w.lit(KTJ_LIT("\"External id\": ")); put_i64(w, r.ext); }
    if (frag) { if (r.ext != 0) w.ch(','); put_fragment(w, r, c); }
    w.lit(KTJ_LIT("\n    }"));
  }
  w.lit(KTJ_LIT("\n  },"));
  if (r.meta & KTJ_M_FLOW) {                                 /* :960-1021, writeFlowEvent :318-345 */
    int64_t frel = r.ts - c.base_time_ns;
    if (frel < 0) frel = 0;
    w.lit(KTJ_LIT("\n  {\n    \"ph\": \"")); w.ch((r.meta & KTJ_M_FLOW_START) ? 's' : 'f');
    w.lit(KTJ_LIT("\",\n    \"id\": ")); put_i64(w, r.flow_id);
    w.lit(KTJ_LIT(",\n    \"pid\": ")); put_i64(w, r.dev);
    w.lit(KTJ_LIT(",\n    \"tid\": ")); put_i64(w, tid);
    w.lit(KTJ_LIT(",\n    \"ts\": ")); put_ts(w, frel);
    if (r.meta & KTJ_M_FLOW_FWDBWD) w.lit(KTJ_LIT(",\n    \"cat\": \"fwdbwd\",\n    \"name\": \"fwdbwd\"\n    "));
    else w.lit(KTJ_LIT(",\n    \"cat\": \"ac2g\",\n    \"name\": \"ac2g\"\n    "));
    if (!(r.meta & KTJ_M_FLOW_START)) w.lit(KTJ_LIT(", \"bp\": \"e\""));
    w.lit(KTJ_LIT("\n  },"));
  }
}

}  // namespace ktj
#endif
