/*
 * TEST INFRASTRUCTURE - not part of the product.  CPU restatement, in plain C, of the byte work
 * the reference's redistribute path does per chunk and per bucket.  Only tests/, the smoke check
 * and the cpu_baseline leg of bench.py may load this; the product path never does.
 *
 * Each function names the reference code it restates (paths relative to the reference tree).
 * The arithmetic the reference delegates to third-party libraries (ATen copies and casts,
 * NCCL/gloo sums; torch 2.10/2.11, NCCL 2.28/2.30 per its pixi.lock) is restated from the
 * published definitions: a copy is a byte move, a cast to a narrower float is IEEE
 * round-to-nearest-even, and the Partial collapse is the fp32 sum of the partials in rank order
 * followed by one cast.
 *
 * Pinning (tests/test_oracle_*.py): casts against known-answer bit patterns, exhaustive
 * round trips and torch's CPU casts; gather/scatter against numpy slicing; the reduce against
 * order-sensitive closed forms; the self-copy cases against the reference's own vectors
 * (tests/test_self_copy_bucket.py:51-63).
 * Parity unpinned: the bit pattern a NaN gets in a narrowing cast (ATen's vectorised CPU cast, its
 * scalar c10 rule and the CUDA intrinsic write 0xFFFF, 0x7FC0 and 0x7FFF for bf16; fp16 depends on
 * F16C hardware vs software) - NaN-ness is pinned, the payload is not - and NaN handling of
 * max/min (backend-defined).
 */
#include <stdint.h>
#include <string.h>

enum { OR_F16 = 0, OR_BF16 = 1, OR_F32 = 2, OR_F64 = 3, OR_B8 = 4, OR_B16 = 5, OR_B32 = 6, OR_B64 = 7,
       OR_I8 = 8, OR_U8 = 9, OR_I16 = 10, OR_I32 = 11, OR_I64 = 12, OR_BOOL = 13, OR_F8E4M3 = 14, OR_F8E5M2 = 15 };
enum { OR_SUM = 0, OR_AVG = 1, OR_MAX = 2, OR_MIN = 3, OR_PRODUCT = 4 };
#define OR_MAX_NDIM 8

typedef struct {
  const void* tensor;        /* element [0,..,0] of the parent tensor */
  int64_t start[OR_MAX_NDIM];
  int64_t shape[OR_MAX_NDIM];
  int64_t stride[OR_MAX_NDIM]; /* elements */
  int32_t ndim;
  int32_t tensor_dtype;
  int32_t wire_dtype;
  int32_t n_partials;        /* >0: tensor ignored, peers[] used */
  const void* const* peers;
  int32_t reduce_op;
  int32_t pad;
  int64_t bucket_off;        /* Bucket.offsets[i] */
} OracleChunk;

int oracle_dtype_size(int dt) {
  switch (dt) {
    case OR_F16: case OR_BF16: case OR_B16: case OR_I16: return 2;
    case OR_F32: case OR_B32: case OR_I32: return 4;
    case OR_F64: case OR_B64: case OR_I64: return 8;
    case OR_B8: case OR_I8: case OR_U8: case OR_BOOL: case OR_F8E4M3: case OR_F8E5M2: return 1;
    default: return 0;
  }
}

/* ---- casts: what buffer.to(dtype) computes (ir.py:125-126,138-139) --------------------------- */

static float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* IEEE binary32 -> bfloat16, round to nearest even; NaN -> 0x7FC0 (c10::BFloat16's CPU rule) */
uint16_t oracle_f32_to_bf16(uint32_t u) {
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}
uint32_t oracle_bf16_to_f32(uint16_t h) { return (uint32_t)h << 16; }

/* IEEE binary32 -> binary16, round to nearest even, gradual underflow, overflow to infinity */
uint16_t oracle_f32_to_f16(uint32_t u) {
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t mag = u & 0x7fffffffu;
  if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);       /* NaN (payload not pinned) */
  if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);      /* >= 65536 or inf -> inf */
  int32_t e = (int32_t)(mag >> 23) - 127;                         /* unbiased exponent */
  uint32_t man = mag & 0x7fffffu;
  if (e < -25) return (uint16_t)sign;                             /* below half of the smallest subnormal */
  uint32_t q, rem, half;
  if (e >= -14) {                                                 /* normal result */
    q = ((uint32_t)(e + 15) << 10) | (man >> 13);
    rem = man & 0x1fffu;
    half = 0x1000u;
  } else {                                                        /* subnormal result: shift the full significand */
    uint32_t sig = man | 0x800000u;                               /* 24-bit significand */
    int shift = 13 + (-14 - e);                                   /* 14..24 */
    q = sig >> shift;
    rem = sig & ((1u << shift) - 1u);
    half = 1u << (shift - 1);
  }
  if (rem > half || (rem == half && (q & 1u))) q++;               /* carries propagate into the exponent correctly */
  return (uint16_t)(sign | q);
}
uint32_t oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  if (e == 0x1f) return sign | 0x7f800000u | (man << 13) | (man ? 0x00400000u : 0u);  /* a signalling NaN comes out quiet */
  if (e == 0) {
    if (man == 0) return sign;
    int shift = 0;
    while (!(man & 0x400u)) { man <<= 1; shift++; }
    man &= 0x3ffu;
    return sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
  }
  return sign | ((e + 127 - 15) << 23) | (man << 13);
}

static float load_as_f32(const void* p, int dt) {
  switch (dt) {
    case OR_F16: { uint16_t h; memcpy(&h, p, 2); return bits_to_f32(oracle_f16_to_f32(h)); }
    case OR_BF16: { uint16_t h; memcpy(&h, p, 2); return bits_to_f32(oracle_bf16_to_f32(h)); }
    case OR_F32: { float f; memcpy(&f, p, 4); return f; }
    default: { double d; memcpy(&d, p, 8); return (float)d; }     /* c10: narrower floats are built from float(value) */
  }
}
static void store_from_f32(void* p, int dt, float f) {
  switch (dt) {
    case OR_F16: { uint16_t h = oracle_f32_to_f16(f32_to_bits(f)); memcpy(p, &h, 2); break; }
    case OR_BF16: { uint16_t h = oracle_f32_to_bf16(f32_to_bits(f)); memcpy(p, &h, 2); break; }
    case OR_F32: memcpy(p, &f, 4); break;
    default: { double d = (double)f; memcpy(p, &d, 8); break; }
  }
}

/* ---- 8-bit floats (OCP e4m3fn: no infinities, S.1111.111 is NaN; e5m2: IEEE-like) ----------------
 * Restated from the published c10 conversion routines (c10/util/Float8_e4m3fn.h, Float8_e5m2.h): round to
 * nearest even on the fp32 bit pattern; e4m3fn maps everything from 480 up (and NaN) to NaN 0x7F, e5m2 maps
 * overflow to infinity 0x7C and NaN to 0x7F. */
uint8_t oracle_f32_to_e4m3(uint32_t u) {
  const uint32_t sign = u & 0x80000000u;
  uint32_t mag = u ^ sign;
  uint8_t r;
  if (mag >= (1087u << 20)) {
    r = 0x7f;
  } else if (mag < (121u << 23)) {               /* below 2^-6: subnormal result, rounded by a float addition */
    const uint32_t denorm = 141u << 23;
    r = (uint8_t)(f32_to_bits(bits_to_f32(mag) + bits_to_f32(denorm)) - denorm);
  } else {
    const uint32_t odd = (mag >> 20) & 1u;
    mag += ((uint32_t)(7 - 127) << 23) + 0x7ffffu + odd;
    r = (uint8_t)(mag >> 20);
  }
  return (uint8_t)(r | (sign >> 24));
}
uint8_t oracle_f32_to_e5m2(uint32_t u) {
  const uint32_t sign = u & 0x80000000u;
  uint32_t mag = u ^ sign;
  uint8_t r;
  if (mag >= (143u << 23)) {
    r = mag > (255u << 23) ? 0x7f : 0x7c;
  } else if (mag < (113u << 23)) {               /* below 2^-14 */
    const uint32_t denorm = 134u << 23;
    r = (uint8_t)(f32_to_bits(bits_to_f32(mag) + bits_to_f32(denorm)) - denorm);
  } else {
    const uint32_t odd = (mag >> 21) & 1u;
    mag += ((uint32_t)(15 - 127) << 23) + 0xfffffu + odd;
    r = (uint8_t)(mag >> 21);
  }
  return (uint8_t)(r | (sign >> 24));
}
uint32_t oracle_e5m2_to_f32(uint8_t b) { return oracle_f16_to_f32((uint16_t)((uint16_t)b << 8)); }
uint32_t oracle_e4m3_to_f32(uint8_t b) {
  const uint32_t sign = ((uint32_t)b & 0x80u) << 24, e = (b >> 3) & 0xfu, man = b & 7u;
  if (e == 0xf && man == 7) return sign | 0x7fc00000u;
  if (e == 0) {
    if (man == 0) return sign;
    float v = (float)man * 0.001953125f;          /* man * 2^-9, exact */
    return sign | f32_to_bits(v);
  }
  return sign | ((e + 127 - 7) << 23) | (man << 20);
}

/* ---- integers and bool: buffer.to(dtype) between any two of the types above is static_cast
 * (c10::convert).  A float becomes an integer by truncation toward zero; for values that do not fit,
 * and for NaN, the C++ cast is undefined and ATen's x86 CPU kernels return what cvttss2si / cvttsd2si
 * return: INT32_MIN for a 32-bit (or narrower: the low bits of that) result, INT64_MIN for a 64-bit one.
 * A uint8 result is taken from the 64-bit conversion (c10's static_cast_with_inter_type<uint8_t, T> casts
 * through int64_t).  Narrow floats (f16, bf16, fp8) go through float in both directions. */
static int is_float_dt(int dt) { return dt <= OR_F64 || dt == OR_F8E4M3 || dt == OR_F8E5M2; }
static int is_int_dt(int dt) { return dt >= OR_I8 && dt <= OR_BOOL; }

static int32_t trunc_i32_f32(float f) { return (f >= -2147483648.0f && f < 2147483648.0f) ? (int32_t)f : INT32_MIN; }
static int64_t trunc_i64_f32(float f) { return (f >= -9223372036854775808.0f && f < 9223372036854775808.0f) ? (int64_t)f : INT64_MIN; }
static int32_t trunc_i32_f64(double f) { return (f > -2147483649.0 && f < 2147483648.0) ? (int32_t)f : INT32_MIN; }
static int64_t trunc_i64_f64(double f) { return (f >= -9223372036854775808.0 && f < 9223372036854775808.0) ? (int64_t)f : INT64_MIN; }

static int64_t load_int(const void* p, int dt) {
  switch (dt) {
    case OR_I8: { int8_t v; memcpy(&v, p, 1); return v; }
    case OR_U8: { uint8_t v; memcpy(&v, p, 1); return v; }
    case OR_BOOL: { uint8_t v; memcpy(&v, p, 1); return v != 0; }
    case OR_I16: { int16_t v; memcpy(&v, p, 2); return v; }
    case OR_I32: { int32_t v; memcpy(&v, p, 4); return v; }
    default: { int64_t v; memcpy(&v, p, 8); return v; }
  }
}
static void store_int(void* p, int dt, int64_t v) {
  switch (dt) {
    case OR_I8: case OR_U8: { uint8_t b = (uint8_t)v; memcpy(p, &b, 1); break; }
    case OR_BOOL: { uint8_t b = v != 0; memcpy(p, &b, 1); break; }
    case OR_I16: { uint16_t b = (uint16_t)v; memcpy(p, &b, 2); break; }
    case OR_I32: { uint32_t b = (uint32_t)v; memcpy(p, &b, 4); break; }
    default: memcpy(p, &v, 8);
  }
}
static float load_float_as_f32(const void* p, int dt) {
  if (dt == OR_F8E4M3) { uint8_t b; memcpy(&b, p, 1); return bits_to_f32(oracle_e4m3_to_f32(b)); }
  if (dt == OR_F8E5M2) { uint8_t b; memcpy(&b, p, 1); return bits_to_f32(oracle_e5m2_to_f32(b)); }
  return load_as_f32(p, dt);
}
static void store_float_from_f32(void* p, int dt, float f) {
  if (dt == OR_F8E4M3) { uint8_t b = oracle_f32_to_e4m3(f32_to_bits(f)); memcpy(p, &b, 1); return; }
  if (dt == OR_F8E5M2) { uint8_t b = oracle_f32_to_e5m2(f32_to_bits(f)); memcpy(p, &b, 1); return; }
  store_from_f32(p, dt, f);
}

static void cast_one(const void* src, int sdt, void* dst, int ddt) {
  if (is_int_dt(sdt)) {
    const int64_t v = load_int(src, sdt);
    if (is_int_dt(ddt)) { store_int(dst, ddt, v); return; }
    if (ddt == OR_F64) { double d = (double)v; memcpy(dst, &d, 8); return; }
    store_float_from_f32(dst, ddt, (float)v);           /* narrower floats are built from float(value) */
    return;
  }
  if (sdt == OR_F64 && is_int_dt(ddt)) {
    double d; memcpy(&d, src, 8);
    if (ddt == OR_BOOL) store_int(dst, ddt, d != 0.0);
    else if (ddt == OR_I64 || ddt == OR_U8) store_int(dst, ddt, trunc_i64_f64(d));
    else store_int(dst, ddt, trunc_i32_f64(d));
    return;
  }
  const float f = load_float_as_f32(src, sdt);            /* f64 -> narrow float: two roundings, through float */
  if (is_int_dt(ddt)) {
    if (ddt == OR_BOOL) store_int(dst, ddt, f != 0.0f);
    else if (ddt == OR_I64 || ddt == OR_U8) store_int(dst, ddt, trunc_i64_f32(f));
    else store_int(dst, ddt, trunc_i32_f32(f));
    return;
  }
  store_float_from_f32(dst, ddt, f);
}

/* n elements src_dt -> dst_dt.  Same dtype: byte move.  Returns 0, or -1 if unsupported. */
int oracle_cast(const void* src, int src_dt, void* dst, int dst_dt, int64_t n) {
  int ss = oracle_dtype_size(src_dt), ds = oracle_dtype_size(dst_dt);
  if (!ss || !ds) return -1;
  if (src_dt == dst_dt) { memmove(dst, src, (size_t)(n * ss)); return 0; }
  if (!(is_float_dt(src_dt) || is_int_dt(src_dt)) || !(is_float_dt(dst_dt) || is_int_dt(dst_dt))) return -1;
  if (src_dt <= OR_F64 && dst_dt <= OR_F64) {
    for (int64_t i = 0; i < n; i++)
      store_from_f32((char*)dst + i * ds, dst_dt, load_as_f32((const char*)src + i * ss, src_dt));
    return 0;
  }
  for (int64_t i = 0; i < n; i++) cast_one((const char*)src + i * ss, src_dt, (char*)dst + i * ds, dst_dt);
  return 0;
}

/* ---- slicing: tensor[slice].contiguous() (ir.py:113-115) and tensor[slice].copy_(buf) (ir.py:140) */

static int64_t chunk_numel(const OracleChunk* c) {
  int64_t n = 1;
  for (int i = 0; i < c->ndim; i++) n *= c->shape[i];
  return n;
}

/* visit the chunk's elements in row-major order; dir 0: tensor -> out, dir 1: in -> tensor */
static void walk(const OracleChunk* c, const void* base, int es, char* contig, int dir) {
  int64_t idx[OR_MAX_NDIM] = {0};
  int64_t n = chunk_numel(c);
  for (int64_t k = 0; k < n; k++) {
    int64_t off = 0;
    for (int d = 0; d < c->ndim; d++) off += (c->start[d] + idx[d]) * c->stride[d];
    char* t = (char*)base + off * es;
    if (dir == 0) memcpy(contig + k * es, t, (size_t)es); else memcpy(t, contig + k * es, (size_t)es);
    for (int d = c->ndim - 1; d >= 0; d--) { if (++idx[d] < c->shape[d]) break; idx[d] = 0; }
  }
}

void oracle_gather(const OracleChunk* c, void* out) { walk(c, c->tensor, oracle_dtype_size(c->tensor_dtype), (char*)out, 0); }
void oracle_scatter(const OracleChunk* c, const void* in) { walk(c, c->tensor, oracle_dtype_size(c->tensor_dtype), (char*)in, 1); }

/* ---- Partial collapse (ir.py:116-124), as the fp32 rank-order combination, then one cast ------ */
int oracle_reduce(const OracleChunk* c, void* out /* wire dtype, contiguous */, void* scratch /* numel * tensor es */) {
  int es = oracle_dtype_size(c->tensor_dtype), ws = oracle_dtype_size(c->wire_dtype);
  if (c->tensor_dtype > OR_F64 || c->wire_dtype > OR_F64 || c->n_partials < 1) return -1;
  int64_t n = chunk_numel(c);
  if (c->tensor_dtype == OR_F64) {  /* f64 partials accumulate in f64 */
    double* acc = (double*)scratch;
    walk(c, c->peers[0], es, (char*)acc, 0);
    for (int p = 1; p < c->n_partials; p++) {
      int64_t idx[OR_MAX_NDIM] = {0};
      for (int64_t k = 0; k < n; k++) {
        int64_t off = 0;
        for (int d = 0; d < c->ndim; d++) off += (c->start[d] + idx[d]) * c->stride[d];
        double v; memcpy(&v, (const char*)c->peers[p] + off * 8, 8);
        double a = acc[k];
        switch (c->reduce_op) {
          case OR_MAX: a = a > v ? a : (v > a ? v : (a == a ? a : v)); break;
          case OR_MIN: a = a < v ? a : (v < a ? v : (a == a ? a : v)); break;
          case OR_PRODUCT: a = a * v; break;
          default: a = a + v;
        }
        acc[k] = a;
        for (int d = c->ndim - 1; d >= 0; d--) { if (++idx[d] < c->shape[d]) break; idx[d] = 0; }
      }
    }
    for (int64_t k = 0; k < n; k++) {
      double r = acc[k];
      if (c->reduce_op == OR_AVG) r = r / (double)c->n_partials;
      if (c->wire_dtype == OR_F64) memcpy((char*)out + k * 8, &r, 8);
      else store_from_f32((char*)out + k * ws, c->wire_dtype, (float)r);
    }
    return 0;
  }
  int64_t idx[OR_MAX_NDIM] = {0};
  for (int64_t k = 0; k < n; k++) {
    int64_t off = 0;
    for (int d = 0; d < c->ndim; d++) off += (c->start[d] + idx[d]) * c->stride[d];
    volatile float acc = load_as_f32((const char*)c->peers[0] + off * es, c->tensor_dtype);
    for (int p = 1; p < c->n_partials; p++) {
      float v = load_as_f32((const char*)c->peers[p] + off * es, c->tensor_dtype);
      float a = acc;
      switch (c->reduce_op) {
        case OR_MAX: a = a > v ? a : (v > a ? v : (a == a ? a : v)); break;
        case OR_MIN: a = a < v ? a : (v < a ? v : (a == a ? a : v)); break;
        case OR_PRODUCT: a = a * v; break;
        default: a = a + v;
      }
      acc = a;  /* volatile: one rounding per step, no reassociation or fusing */
    }
    float r = acc;
    if (c->reduce_op == OR_AVG) r = r / (float)c->n_partials;
    store_from_f32((char*)out + k * ws, c->wire_dtype, r);
    for (int d = c->ndim - 1; d >= 0; d--) { if (++idx[d] < c->shape[d]) break; idx[d] = 0; }
  }
  return 0;
}

/* ---- buckets -------------------------------------------------------------------------------- */

/* Bucket.prepare of a source bucket (ir.py:246-259 with Chunk.prepare ir.py:112-126): every chunk is
 * sliced, (reduced,) cast to the wire dtype and laid at its byte offset.  scratch: max chunk bytes
 * in tensor dtype. */
int oracle_pack_bucket(const OracleChunk* chunks, int64_t n_chunks, void* bucket, void* scratch) {
  for (int64_t i = 0; i < n_chunks; i++) {
    const OracleChunk* c = &chunks[i];
    char* dst = (char*)bucket + c->bucket_off;
    if (c->n_partials > 0) {
      if (oracle_reduce(c, dst, scratch)) return -1;
    } else {
      oracle_gather(c, scratch);
      if (oracle_cast(scratch, c->tensor_dtype, dst, c->wire_dtype, chunk_numel(c))) return -1;
    }
  }
  return 0;
}

/* Bucket.finalize of a target bucket (ir.py:300-310 with Chunk.finalize ir.py:134-141) */
int oracle_unpack_bucket(const OracleChunk* chunks, int64_t n_chunks, const void* bucket, void* scratch) {
  for (int64_t i = 0; i < n_chunks; i++) {
    const OracleChunk* c = &chunks[i];
    if (oracle_cast((const char*)bucket + c->bucket_off, c->wire_dtype, scratch, c->tensor_dtype, chunk_numel(c)))
      return -1;
    oracle_scatter(c, scratch);
  }
  return 0;
}
