// MI355X (gfx950) redistribute hot path: pack / unpack / self-copy / Partial reduce-pack.
//
// Design.  These are HBM-bound byte movers.  On MI355X a plain copy runs fastest when every
// work-item moves exactly one 16-byte vector, workgroups are one wavefront (64 work-items = 1 KiB),
// the grid is huge and ordered by address, and both sides use nontemporal accesses; loops and
// several vectors per work-item lose 10-30 %.  So all chunk geometry (slices, strides, bucket
// offsets, dtype pairs, alignment classes) is resolved once on the host into a flat
// device-resident *tile program*: one entry per 16 workgroups holding absolute addresses.  A
// workgroup does one scalar table load, each work-item one vector load and one vector store.  Only
// chunks whose contiguous dim differs between the two sides (transposes) are staged through LDS.
//
// What it replaces in the reference: the per-chunk ATen launches of Chunk.prepare /
// Bucket.prepare / Chunk.finalize / Bucket.finalize (src/etha/comm/ir.py:101-141, 229-264,
// 300-310) - slice, contiguous(), all_reduce, to(dtype), narrow/view/copy_.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdio>
#include <algorithm>
#include <array>
#include <atomic>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "etha_reshard.h"

namespace {

#ifndef ETHA_TILE_UNITS
#define ETHA_TILE_UNITS 1024
#endif
#ifndef ETHA_BLOCK_THREADS
#define ETHA_BLOCK_THREADS 64
#endif
#ifndef ETHA_CVT_WIDE_BYTES
#define ETHA_CVT_WIDE_BYTES 16
#endif
#ifndef ETHA_SKEW_PEEL_MIN_BYTES
#define ETHA_SKEW_PEEL_MIN_BYTES (256 * 1024)
#endif
// One table entry (tile) describes kTileThreads units; it is executed by kBlocksPerTile workgroups of
// kBlockThreads work-items (one wavefront each).  Wave-sized workgroups schedule best; the coarser
// table granularity keeps the tile program small.
constexpr uint32_t kTileThreads = ETHA_TILE_UNITS;     // units per tile
constexpr uint32_t kBlockThreads = ETHA_BLOCK_THREADS; // work-items per workgroup
constexpr uint32_t kBlocksPerTile = kTileThreads / kBlockThreads;
static_assert(kTileThreads % kBlockThreads == 0 && kBlocksPerTile >= 1, "tile must be a multiple of the workgroup");

// Elements one work-item converts at once: the narrow side moves up to 16 bytes, the wide side up to
// kCvtWideBytes (one or two 16-byte accesses).
constexpr int kCvtWideBytes = ETHA_CVT_WIDE_BYTES;
constexpr int cvt_elems_per_unit(int es_a, int es_b) {
  const int lo = es_a < es_b ? es_a : es_b, hi = es_a < es_b ? es_b : es_a;
  const int by_narrow = 16 / lo, by_wide = kCvtWideBytes / hi;
  return by_narrow < by_wide ? by_narrow : by_wide;
}

// ---- tile program entries (device-visible, also read back by host-side checkers) -------------
// A "unit" is what one work-item moves: 2^ua bytes on the a side and 2^ub bytes on the b side
// (equal for byte moves; different for converting moves).  a = tensor side, b = bucket side
// (for self-copy tables a = source region, b = destination region).
struct RunTile {  // one contiguous run on both sides
  uint64_t a;     // address of the tile's first unit, a side
  uint64_t b;     // address of the tile's first unit, b side
  uint32_t n;     // active units (<= kTileThreads)
  uint32_t meta;
};
static_assert(sizeof(RunTile) == 24, "RunTile layout");

struct RowTile {     // walks rows of `run` units; covers units [c0, c0+n) counted from row r0
  uint64_t a;        // address of (row r0, unit 0) on the a side; for reduce tiles: byte offset from each peer base
  uint64_t b;        // address of (row r0, unit 0) on the b side
  int64_t a_pitch;   // bytes between consecutive rows
  int64_t b_pitch;
  uint32_t n;        // active units (<= kTileThreads)
  uint32_t meta;
  uint32_t run;      // units per row
  uint32_t c0;       // first unit's column inside row r0 (< run)
  uint32_t peer_first;  // reduce tiles: index of the first peer base in the peers array
  uint32_t n_peers;     // 0 = plain tile
  uint32_t reduce_op;
  uint32_t via;         // reduce tiles: 0, or 1 + ETHA_* dtype the result is rounded to before the b-side dtype;
                        // gather tiles: units per piece
};
static_assert(sizeof(RowTile) == 64, "RowTile layout");

struct TransTile {   // a 2-D block whose contiguous dim differs between the two sides (a transposing chunk)
  uint64_t a;        // address of element (j0, k0) on the a side, contiguous along j
  uint64_t b;        // address of element (j0, k0) on the b side, contiguous along k
  int64_t a_pitch;   // bytes between consecutive k on the a side
  int64_t b_pitch;   // bytes between consecutive j on the b side
  uint32_t nj, nk;   // extent of the block: a wide block, a block of trans_dim_a x trans_dim_b elements, or less at an edge
  uint32_t es_log2;  // log2 of the element size in bytes (of the b side, when the block converts)
  uint32_t cvt;      // 0: same element type on both sides; else (dtype of a << 4) | dtype of b, plus kTransTyped for the
                     // blocks of the typed kernel (without it: a holds f32, b f16 or bf16, converted by the plain kernel)
  uint32_t peer_first;  // typed blocks of a Partial source: index of the first peer base (a is then an offset from each base)
  uint32_t n_peers;     // 0 = not a reduction
  uint32_t reduce_op;   // one ETHA_* op (nested levels keep their row tiles)
  uint32_t via;         // as in RowTile
};
static_assert(sizeof(TransTile) == 64, "TransTile layout");
// Blocks of the typed transposing kernel: any pair of value types (converted element by element while the block is
// parked in LDS) and Partial sources (the members' blocks are combined in registers first).  Full blocks are
// trans_typed_dim x trans_typed_dim elements.
constexpr uint32_t kTransTyped = 1u << 8;
__host__ __device__ constexpr uint32_t trans_typed_dim(uint32_t esa, uint32_t esb) { return (esa == 8 || esb == 8) ? 64u : 128u; }
// Full blocks of a Partial source whose members hold 2-byte elements (the straight-line reduce path): j x k elements.
constexpr uint32_t kRedDimJ2 = 128, kRedDimK2 = 128;
// A transposing block is D x D elements, handled by one workgroup of kTransThreads work-items.  D is chosen
// per element size so that a row of the block is at least 128 bytes on both sides and a full block is a
// few 16-byte vectors per work-item.  LDS rows are padded to an odd number of 32-bit words.
#ifndef ETHA_TRANS_THREADS
#define ETHA_TRANS_THREADS 1024
#endif
#ifndef ETHA_TRANS_DIM_A
#define ETHA_TRANS_DIM_A 128
#endif
#ifndef ETHA_TRANS_DIM_B
#define ETHA_TRANS_DIM_B 128
#endif
#ifndef ETHA_TRANS_SUPER
#define ETHA_TRANS_SUPER 4
#endif
constexpr uint32_t kTransThreads = ETHA_TRANS_THREADS;
// block extent in elements along j (the a side's contiguous dim) and along k (the b side's); half of it for
// 8-byte elements, which keeps the LDS footprint of a block at 16-66 KB
__host__ __device__ constexpr uint32_t trans_dim_a(uint32_t es) { return es == 8 ? ETHA_TRANS_DIM_A / 2u : (uint32_t)ETHA_TRANS_DIM_A; }
__host__ __device__ constexpr uint32_t trans_dim_b(uint32_t es) { return es == 8 ? ETHA_TRANS_DIM_B / 2u : (uint32_t)ETHA_TRANS_DIM_B; }
// Where a chunk is large enough, blocks are trans_wide(es) times that extent on both sides ("wide" blocks): a
// 128-element side of 1- or 2-byte elements is a run of only 128 or 256 bytes, and longer runs move faster
// (2-byte elements 5.9 -> 6.1-6.7 TB/s, 1-byte elements 5.1 -> 6.0-6.2).  A wide block is loaded whole into
// registers and goes through LDS in trans_panels(es) panels of columns, so LDS holds a panel, not the block.
__host__ __device__ constexpr uint32_t trans_wide(uint32_t es) { return es <= 2 ? 2u : 1u; }
__host__ __device__ constexpr uint32_t trans_panels(uint32_t es) { return es == 2 ? 2u : 1u; }
// wide blocks of chunks that convert between f32 (a side) and a 16-bit wire type: j x k elements
constexpr uint32_t kTransCvtWideJ = ETHA_TRANS_DIM_A, kTransCvtWideK = 2 * ETHA_TRANS_DIM_B;
__host__ __device__ constexpr uint32_t trans_pitch(uint32_t dim, uint32_t es) {  // LDS row pitch in elements: an odd number of words
  return dim + (es >= 4 ? 1u : 4u / es);
}
__host__ __device__ constexpr uint32_t trans_typed_lds_bytes(uint32_t esa, uint32_t esb) {  // rows of the destination's elements
  const uint32_t d = trans_typed_dim(esa, esb), m = esa > esb ? esa : esb;
  const uint32_t typed = d * (d + (m >= 4 ? 1u : 4u / m)) * m;
  const uint32_t red = esa == 2 ? kRedDimK2 * (kRedDimJ2 + (esb >= 4 ? 1u : 4u / esb)) * esb : 0u;
  return typed > red ? typed : red;
}
__host__ __device__ constexpr uint32_t trans_lds_bytes(uint32_t es) {  // either direction: rows of one side (one panel of a wide block), one row per element of the other
  const uint32_t w = trans_wide(es), p = trans_panels(es);
  const uint32_t fwd = w * trans_dim_b(es) * trans_pitch(w * trans_dim_a(es) / p, es) * es, rev = w * trans_dim_a(es) * trans_pitch(w * trans_dim_b(es) / p, es) * es;
  return fwd > rev ? fwd : rev;
}

// meta bits
constexpr uint32_t kMetaUaShift = 0;    // 4 bits: log2 bytes per unit, a side
constexpr uint32_t kMetaUbShift = 4;    // 4 bits: log2 bytes per unit, b side
constexpr uint32_t kMetaDtaShift = 8;   // 4 bits: ETHA_* dtype, a side
constexpr uint32_t kMetaDtbShift = 12;  // 4 bits: ETHA_* dtype, b side
constexpr uint32_t kMetaCvt = 1u << 16; // converting move (else byte move)
constexpr uint32_t kMetaVec = 1u << 17; // converting move handles the full vector (else 1 element)
constexpr uint32_t kMetaSkew = 1u << 18;  // a-side addresses are not all multiples of the a-side unit size
constexpr uint32_t kMetaSkewB = 1u << 19; // same for the b side (both are bookkeeping for checkers: the kernel's
                                          // accesses are legal at any element-aligned address)
constexpr uint32_t kMetaGeneric = 1u << 20;  // converting move with an integer, bool or 8-bit float side: one element per unit
// Row tile of a write-ordered range whose rows are assembled from several chunks (unpack only): a row of `run`
// units is n_peers pieces of `via` units each, piece p read at gather[peer_first + p] + row * b_pitch.  The a
// side is addressed as in any row tile, so one wavefront writes whole destination lines.
constexpr uint32_t kMetaGather = 1u << 21;
// converting and reducing moves: log2 of the elements one unit holds (2 bits).  kMetaVec marks the full vector of a
// dtype pair; a row's remainder moves in narrower vectors of 4 or 2 elements before single elements are used.
constexpr uint32_t kMetaElemsShift = 22;
constexpr uint32_t kGatherMaxPieces = 8;       // the kernel reads this many piece addresses per tile (the list is padded)

// ---- typed vector access ----------------------------------------------------------------------
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Addresses come out of the tile program as integers; the global address space is stated
// explicitly so that the accesses are global_load/global_store and not generic (flat) ones.
#define ETHA_GLOBAL __attribute__((address_space(1)))
template <typename V>
__device__ __forceinline__ V ld_stream(uint64_t addr) {
  return __builtin_nontemporal_load(reinterpret_cast<const ETHA_GLOBAL V*>(addr));
}
template <typename V>
__device__ __forceinline__ void st_stream(uint64_t addr, V v) {
  __builtin_nontemporal_store(v, reinterpret_cast<ETHA_GLOBAL V*>(addr));
}
// The device runs in unaligned-access mode: a 4/8/16-byte access may sit at any byte address and is still
// one instruction, so vector types are declared with the weakest alignment their use can meet.  The
// host decides per tile whether addresses are in fact aligned (the fast case) and records it in the
// meta bits; consecutive work-items cover one contiguous byte range either way.
typedef u32x4 u32x4_any __attribute__((aligned(1)));
typedef u32x2 u32x2_any __attribute__((aligned(1)));
typedef uint32_t u32_any __attribute__((aligned(1)));
typedef uint16_t u16_any __attribute__((aligned(1)));
template <typename V>
__device__ __forceinline__ void copy_as(uint64_t src, uint64_t dst) {
  st_stream<V>(dst, ld_stream<V>(src));
}

// N elements of storage type T as one vector that is only element-aligned.
template <typename T, int N>
struct Pack {
  typedef T vec __attribute__((ext_vector_type(N)));
  typedef vec vec_mem __attribute__((aligned(sizeof(T))));
  vec v;
  __device__ __forceinline__ void load(uint64_t addr) { v = ld_stream<vec_mem>(addr); }
  __device__ __forceinline__ void store(uint64_t addr) const { st_stream<vec_mem>(addr, v); }
  __device__ __forceinline__ T get(int i) const { return v[i]; }
  __device__ __forceinline__ void set(int i, T x) { v[i] = x; }
};
template <typename T>
struct Pack<T, 1> {
  T v;
  __device__ __forceinline__ void load(uint64_t addr) { v = ld_stream<T>(addr); }
  __device__ __forceinline__ void store(uint64_t addr) const { st_stream<T>(addr, v); }
  __device__ __forceinline__ T get(int) const { return v; }
  __device__ __forceinline__ void set(int, T x) { v = x; }
};

// ---- element conversions (all go through fp32, as c10::Half/BFloat16 constructors do) ----------
struct TagF16 { typedef uint16_t bits; };
struct TagBF16 { typedef uint16_t bits; };
struct TagF32 { typedef uint32_t bits; };
struct TagF64 { typedef uint64_t bits; };

__device__ __forceinline__ float to_f32(TagF16, uint16_t x) { return (float)__builtin_bit_cast(_Float16, x); }
__device__ __forceinline__ float to_f32(TagBF16, uint16_t x) { return __builtin_bit_cast(float, (uint32_t)x << 16); }
__device__ __forceinline__ float to_f32(TagF32, uint32_t x) { return __builtin_bit_cast(float, x); }
// f64 -> narrower float is two roundings (f64 -> f32 -> target), as c10::Half(double) and
// c10::BFloat16(double) do; the empty asm keeps the compiler from fusing them into one rounding.
__device__ __forceinline__ float to_f32(TagF64, uint64_t x) {
  float f = (float)__builtin_bit_cast(double, x);
  asm volatile("" : "+v"(f));
  return f;
}

__device__ __forceinline__ uint16_t from_f32(TagF16, float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
// round-to-nearest-even on the bit pattern; every NaN becomes the canonical quiet NaN 0x7FC0
__device__ __forceinline__ uint16_t from_f32(TagBF16, float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ uint32_t from_f32(TagF32, float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ uint64_t from_f32(TagF64, float f) { return __builtin_bit_cast(uint64_t, (double)f); }

template <typename S, typename D, int N>
__device__ __forceinline__ void cvt_n(uint64_t src, uint64_t dst) {
  Pack<typename S::bits, N> in;
  Pack<typename D::bits, N> out;
  in.load(src);
#pragma unroll
  for (int i = 0; i < N; i++) out.set(i, from_f32(D(), to_f32(S(), in.get(i))));
  out.store(dst);
}

// nl = log2 of the elements in this unit (at most those of the pair's full vector)
template <typename S, typename D>
__device__ __forceinline__ void cvt_pair(uint32_t nl, uint64_t src, uint64_t dst) {
  constexpr int kN = cvt_elems_per_unit(sizeof(typename S::bits), sizeof(typename D::bits));
  if constexpr (kN >= 8) {
    if (nl == 3) return cvt_n<S, D, 8>(src, dst);
  }
  if constexpr (kN >= 4) {
    if (nl == 2) return cvt_n<S, D, 4>(src, dst);
  }
  if constexpr (kN >= 2) {
    if (nl == 1) return cvt_n<S, D, 2>(src, dst);
  }
  cvt_n<S, D, 1>(src, dst);
}

template <typename S>
__device__ __forceinline__ void cvt_from(uint32_t dd, uint32_t nl, uint64_t src, uint64_t dst) {
  switch (dd) {
    case ETHA_F16: cvt_pair<S, TagF16>(nl, src, dst); break;
    case ETHA_BF16: cvt_pair<S, TagBF16>(nl, src, dst); break;
    case ETHA_F32: cvt_pair<S, TagF32>(nl, src, dst); break;
    default: cvt_pair<S, TagF64>(nl, src, dst); break;
  }
}

// ---- conversions with an integer, bool or 8-bit float side (Tensor.to(dtype) = static_cast, c10::convert) ----
// 8-bit floats as the published c10 routines define them: round to nearest even on the fp32 bit pattern;
// e4m3fn has no infinities (everything from 480 up and NaN become NaN 0x7F), e5m2 overflows to infinity.
__device__ __forceinline__ uint8_t f32_to_e4m3(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = u & 0x80000000u;
  uint32_t mag = u ^ sign;
  uint32_t r;
  if (mag >= (1087u << 20)) {
    r = 0x7f;
  } else if (mag < (121u << 23)) {  // below 2^-6: a subnormal result, rounded by a float addition
    const uint32_t denorm = 141u << 23;
    float t = __builtin_bit_cast(float, mag) + __builtin_bit_cast(float, denorm);
    r = (__builtin_bit_cast(uint32_t, t) - denorm) & 0xffu;
  } else {
    const uint32_t odd = (mag >> 20) & 1u;
    mag += ((uint32_t)(7 - 127) << 23) + 0x7ffffu + odd;
    r = (mag >> 20) & 0xffu;
  }
  return (uint8_t)(r | (sign >> 24));
}
__device__ __forceinline__ uint8_t f32_to_e5m2(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = u & 0x80000000u;
  uint32_t mag = u ^ sign;
  uint32_t r;
  if (mag >= (143u << 23)) {
    r = mag > (255u << 23) ? 0x7fu : 0x7cu;
  } else if (mag < (113u << 23)) {  // below 2^-14
    const uint32_t denorm = 134u << 23;
    float t = __builtin_bit_cast(float, mag) + __builtin_bit_cast(float, denorm);
    r = (__builtin_bit_cast(uint32_t, t) - denorm) & 0xffu;
  } else {
    const uint32_t odd = (mag >> 21) & 1u;
    mag += ((uint32_t)(15 - 127) << 23) + 0xfffffu + odd;
    r = (mag >> 21) & 0xffu;
  }
  return (uint8_t)(r | (sign >> 24));
}
__device__ __forceinline__ float e4m3_to_f32(uint8_t b) {
  const uint32_t sign = ((uint32_t)b & 0x80u) << 24, e = (b >> 3) & 0xfu, man = b & 7u;
  if (e == 0xf && man == 7) return __builtin_bit_cast(float, sign | 0x7fc00000u);
  if (e == 0) return __builtin_bit_cast(float, sign | __builtin_bit_cast(uint32_t, (float)man * 0.001953125f));
  return __builtin_bit_cast(float, sign | ((e + 127 - 7) << 23) | (man << 20));
}
__device__ __forceinline__ float e5m2_to_f32(uint8_t b) { return to_f32(TagF16(), (uint16_t)((uint16_t)b << 8)); }

// float -> integer: truncation toward zero.  Values that do not fit, and NaN, are undefined in C++; ATen's x86
// kernels return what cvttss2si / cvttsd2si return for them (INT32_MIN, or INT64_MIN for a 64-bit result), and a
// result narrower than 32 bits is the low bits of the 32-bit one.  A uint8 result is taken from the 64-bit
// conversion (c10 casts through int64_t for it).  The device's own conversions saturate, hence the range checks.
__device__ __forceinline__ int64_t trunc_i32(float f) { return (f >= -2147483648.0f && f < 2147483648.0f) ? (int64_t)(int32_t)f : (int64_t)INT32_MIN; }
__device__ __forceinline__ int64_t trunc_i64(float f) { return (f >= -9223372036854775808.0f && f < 9223372036854775808.0f) ? (int64_t)f : INT64_MIN; }
__device__ __forceinline__ int64_t trunc_i32(double f) { return (f > -2147483649.0 && f < 2147483648.0) ? (int64_t)(int32_t)f : (int64_t)INT32_MIN; }
__device__ __forceinline__ int64_t trunc_i64(double f) { return (f >= -9223372036854775808.0 && f < 9223372036854775808.0) ? (int64_t)f : INT64_MIN; }

__device__ __forceinline__ bool is_int_code(uint32_t dt) { return dt >= ETHA_I8 && dt <= ETHA_BOOL; }

// ---- one element as raw bits (zero-extended into 64) --------------------------------------------
__device__ __forceinline__ uint32_t dtype_bytes(uint32_t dt) {
  switch (dt) {
    case ETHA_F16: case ETHA_BF16: case ETHA_B16: case ETHA_I16: return 2;
    case ETHA_F32: case ETHA_B32: case ETHA_I32: return 4;
    case ETHA_F64: case ETHA_B64: case ETHA_I64: return 8;
    default: return 1;
  }
}
__device__ __forceinline__ uint64_t load_bits(uint32_t bytes, uint64_t addr) {
  switch (bytes) {
    case 1: return ld_stream<uint8_t>(addr);
    case 2: return ld_stream<uint16_t>(addr);
    case 4: return ld_stream<uint32_t>(addr);
    default: return ld_stream<uint64_t>(addr);
  }
}
__device__ __forceinline__ void store_bits(uint32_t bytes, uint64_t addr, uint64_t v) {
  switch (bytes) {
    case 1: st_stream<uint8_t>(addr, (uint8_t)v); break;
    case 2: st_stream<uint16_t>(addr, (uint16_t)v); break;
    case 4: st_stream<uint32_t>(addr, (uint32_t)v); break;
    default: st_stream<uint64_t>(addr, v); break;
  }
}
__device__ __forceinline__ int64_t int_value(uint32_t dt, uint64_t bits) {
  switch (dt) {
    case ETHA_I8: return (int8_t)(uint8_t)bits;
    case ETHA_U8: return (uint8_t)bits;
    case ETHA_BOOL: return (uint8_t)bits != 0;
    case ETHA_I16: return (int16_t)(uint16_t)bits;
    case ETHA_I32: return (int32_t)(uint32_t)bits;
    default: return (int64_t)bits;
  }
}
__device__ __forceinline__ uint64_t int_bits(uint32_t dt, int64_t v) {
  switch (dt) {
    case ETHA_I8: case ETHA_U8: return (uint8_t)v;
    case ETHA_BOOL: return v != 0 ? 1u : 0u;
    case ETHA_I16: return (uint16_t)v;
    case ETHA_I32: return (uint32_t)v;
    default: return (uint64_t)v;
  }
}
__device__ __forceinline__ float float_value(uint32_t dt, uint64_t bits) {  // every float type but f64 -> exact; f64 rounds
  switch (dt) {
    case ETHA_F16: return to_f32(TagF16(), (uint16_t)bits);
    case ETHA_BF16: return to_f32(TagBF16(), (uint16_t)bits);
    case ETHA_F32: return to_f32(TagF32(), (uint32_t)bits);
    case ETHA_F8E4M3: return e4m3_to_f32((uint8_t)bits);
    case ETHA_F8E5M2: return e5m2_to_f32((uint8_t)bits);
    default: return to_f32(TagF64(), bits);
  }
}
__device__ __forceinline__ uint64_t float_bits(uint32_t dt, float f) {
  switch (dt) {
    case ETHA_F16: return from_f32(TagF16(), f);
    case ETHA_BF16: return from_f32(TagBF16(), f);
    case ETHA_F32: return from_f32(TagF32(), f);
    case ETHA_F8E4M3: return f32_to_e4m3(f);
    case ETHA_F8E5M2: return f32_to_e5m2(f);
    default: return from_f32(TagF64(), f);
  }
}

// Tensor.to(dtype) on one element, for every pair of value types: the element-by-element moves of the tile kernels
// and the typed transposing blocks both go through this.
__device__ __forceinline__ uint64_t convert_bits(uint32_t sd, uint32_t dd, uint64_t bits) {
  if (is_int_code(sd)) {
    const int64_t v = int_value(sd, bits);
    if (is_int_code(dd)) return int_bits(dd, v);
    if (dd == ETHA_F64) return __builtin_bit_cast(uint64_t, (double)v);
    return float_bits(dd, (float)v);  // narrower floats are built from float(value)
  }
  if (sd == ETHA_F64 && is_int_code(dd)) {
    const double d = __builtin_bit_cast(double, bits);
    return int_bits(dd, dd == ETHA_BOOL ? (int64_t)(d != 0.0) : (dd == ETHA_I64 || dd == ETHA_U8) ? trunc_i64(d) : trunc_i32(d));
  }
  const float f = float_value(sd, bits);
  if (is_int_code(dd))
    return int_bits(dd, dd == ETHA_BOOL ? (int64_t)(f != 0.0f) : (dd == ETHA_I64 || dd == ETHA_U8) ? trunc_i64(f) : trunc_i32(f));
  return float_bits(dd, f);
}

__device__ __forceinline__ void convert_generic(uint32_t sd, uint32_t dd, uint64_t src, uint64_t dst) {
  store_bits(dtype_bytes(dd), dst, convert_bits(sd, dd, load_bits(dtype_bytes(sd), src)));
}

template <bool REV>
__device__ __forceinline__ void move_unit(uint32_t meta, uint64_t a, uint64_t b) {
  const uint64_t src = REV ? b : a, dst = REV ? a : b;
  if (!(meta & kMetaCvt)) {
    switch (meta & 15u) {
      case 4: copy_as<u32x4_any>(src, dst); break;
      case 3: copy_as<u32x2_any>(src, dst); break;
      case 2: copy_as<u32_any>(src, dst); break;
      case 1: copy_as<u16_any>(src, dst); break;
      default: copy_as<uint8_t>(src, dst); break;
    }
    return;
  }
  // The usual converting pairs first - f32 on the a side, bf16 or f16 in the bucket, whole vectors - found with one
  // compare each and handled by straight-line code: a workgroup lives a few microseconds, and the chain of
  // dtype switches below (with the jumps across this kernel's code that it takes) sits in front of its load.
  {
    constexpr uint32_t kPairMask = (15u << kMetaDtaShift) | (15u << kMetaDtbShift) | kMetaVec | kMetaGeneric;
    const uint32_t pair = meta & kPairMask;
    if (pair == (((uint32_t)ETHA_F32 << kMetaDtaShift) | ((uint32_t)ETHA_BF16 << kMetaDtbShift) | kMetaVec)) {
      constexpr int kN = cvt_elems_per_unit(4, 2);
      if (REV) cvt_n<TagBF16, TagF32, kN>(src, dst); else cvt_n<TagF32, TagBF16, kN>(src, dst);
      return;
    }
    if (pair == (((uint32_t)ETHA_F32 << kMetaDtaShift) | ((uint32_t)ETHA_F16 << kMetaDtbShift) | kMetaVec)) {
      constexpr int kN = cvt_elems_per_unit(4, 2);
      if (REV) cvt_n<TagF16, TagF32, kN>(src, dst); else cvt_n<TagF32, TagF16, kN>(src, dst);
      return;
    }
  }
  const uint32_t dta = (meta >> kMetaDtaShift) & 15u, dtb = (meta >> kMetaDtbShift) & 15u;
  const uint32_t sd = REV ? dtb : dta, dd = REV ? dta : dtb;
  if (meta & kMetaGeneric) {
    convert_generic(sd, dd, src, dst);
    return;
  }
  const uint32_t nl = (meta >> kMetaElemsShift) & 3u;
  switch (sd) {
    case ETHA_F16: cvt_from<TagF16>(dd, nl, src, dst); break;
    case ETHA_BF16: cvt_from<TagBF16>(dd, nl, src, dst); break;
    case ETHA_F32: cvt_from<TagF32>(dd, nl, src, dst); break;
    default: cvt_from<TagF64>(dd, nl, src, dst); break;
  }
}

__device__ __forceinline__ void row_position(const RowTile& t, uint32_t tid, uint32_t& r, uint32_t& c) {
  const uint32_t q = t.c0 + tid;  // c0 < run and tid < kTileThreads, so q < 2*run whenever run >= kTileThreads
  if (t.run >= kTileThreads) {
    r = q >= t.run ? 1u : 0u;
    c = q - (r ? t.run : 0u);
  } else {
    r = q / t.run;
    c = q - r * t.run;
  }
}

// pack (REV = false): a -> b.   unpack (REV = true): b -> a.
template <bool REV, bool GATHER = false>
__device__ __forceinline__ void tile_body(const RunTile* __restrict__ run_tiles, uint32_t n_run,
                                          const RowTile* __restrict__ row_tiles, const uint64_t* __restrict__ gather,
                                          uint32_t bid, uint32_t tid) {
  uint64_t a, b;
  uint32_t n, meta;
  if (bid < n_run) {
    const RunTile t = run_tiles[bid];
    n = t.n;
    meta = t.meta;
    a = t.a + ((uint64_t)tid << ((meta >> kMetaUaShift) & 15u));
    b = t.b + ((uint64_t)tid << ((meta >> kMetaUbShift) & 15u));
  } else {
    const RowTile t = row_tiles[bid - n_run];
    n = t.n;
    meta = t.meta;
    uint32_t r, c;
    row_position(t, tid, r, c);
    a = t.a + (uint64_t)((int64_t)r * t.a_pitch) + ((uint64_t)c << ((meta >> kMetaUaShift) & 15u));
    if (GATHER && (meta & kMetaGather)) {
      if (tid >= n) return;
      const uint32_t p = c / t.via;
      // the tile's piece addresses are the same for every lane: fetched through the scalar path, picked per lane
      const uint64_t* pieces = gather + t.peer_first;
      uint64_t base = 0;
#pragma unroll
      for (uint32_t j = 0; j < kGatherMaxPieces; j++) {
        const uint64_t v = pieces[j];  // readfirstlane keeps each of these a scalar load of its own
        // (the builtin returns a signed int: go through uint32_t, or the low word would be sign-extended)
        const uint64_t u = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32)) << 32) |
                           (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
        base = p == j ? u : base;
      }
      b = base + (uint64_t)((int64_t)r * t.b_pitch) + ((uint64_t)(c - p * t.via) << ((meta >> kMetaUbShift) & 15u));
    } else {
      b = t.b + (uint64_t)((int64_t)r * t.b_pitch) + ((uint64_t)c << ((meta >> kMetaUbShift) & 15u));
    }
  }
  if (tid >= n) return;
  move_unit<REV>(meta, a, b);
}

// A wave fetches its tile entry before it can do anything else, and an entry that has to come from HBM doubles the
// wave's life.  The entries are read once, in order, so a few waves fetch ahead for all the others: of every 4096
// workgroups (256 tiles) the first eight - one per XCD, as workgroups are dealt to the XCDs in turn - touch, after
// their own work, the lines that hold the entries of the 256 tiles kPrefetchGroups groups further on, each lane one
// line per step, so that those are in the XCD's L2 when their workgroups start (more than the 512 tiles in flight at
// a time lie between).  The eight of the first group also touch what lies before that.  Only these eight waves wait
// for what they fetch.
// Measured: converting packs, whose workgroups are issued faster than a copy's, gain 3 points of the HBM peak
// (fp32 -> bf16 of the Llama shapes: 79.2 -> 82.3 %), plain copies half a point.  The plain tile kernels only: in the
// gather and mixed kernels the same step cost 1.5 points, in the reduce kernel it changed nothing.
#ifndef ETHA_PREFETCH_GROUPS
#define ETHA_PREFETCH_GROUPS 4
#endif
constexpr uint32_t kPrefetchGroups = ETHA_PREFETCH_GROUPS, kPrefetchTiles = 4096u / kBlocksPerTile;
// every 128-byte line that holds bytes of [lo, hi), one line per lane and step.  Ordinary loads, so that the compiler
// knows which registers they write and when (a load issued from inline asm returns into a register the compiler
// already considers free); the values are folded into `seen`, which the caller keeps alive to the end.
__device__ __forceinline__ void touch_lines(uint64_t lo, uint64_t hi, uint32_t& seen) {
  for (uint64_t line = (lo & ~(uint64_t)127) + (uint64_t)threadIdx.x * 128u; line < hi; line += kBlockThreads * 128u)
    seen ^= *reinterpret_cast<const ETHA_GLOBAL uint32_t*>(line);
}
// tiles are counted run tiles first, then row tiles, as tile_body takes them
__device__ __forceinline__ void prefetch_entries(const RunTile* run_tiles, uint32_t n_run, const RowTile* row_tiles,
                                                 uint32_t n_tiles) {
  if (kPrefetchGroups == 0 || (blockIdx.x & 4095u) >= 8u) return;
  const uint32_t group = blockIdx.x >> 12;
  uint32_t first = group == 0 ? kPrefetchTiles : (group + kPrefetchGroups) * kPrefetchTiles;
  uint32_t last = (group + kPrefetchGroups + 1) * kPrefetchTiles;
  first = first < n_tiles ? first : n_tiles;
  last = last < n_tiles ? last : n_tiles;
  uint32_t seen = 0;
  if (first < n_run) touch_lines((uint64_t)(run_tiles + first), (uint64_t)(run_tiles + (last < n_run ? last : n_run)), seen);
  if (last > n_run)
    touch_lines((uint64_t)(row_tiles + ((first > n_run ? first : n_run) - n_run)), (uint64_t)(row_tiles + (last - n_run)), seen);
  asm volatile("" ::"v"(seen));  // the loads are performed although nothing uses what they return
}

template <bool REV>
__global__ __launch_bounds__(ETHA_BLOCK_THREADS) void etha_tile_kernel(const RunTile* __restrict__ run_tiles, uint32_t n_run,
                                                                        const RowTile* __restrict__ row_tiles,
                                                                        const uint64_t* __restrict__ gather) {
  tile_body<REV>(run_tiles, n_run, row_tiles, gather, blockIdx.x / kBlocksPerTile,
                 (blockIdx.x % kBlocksPerTile) * kBlockThreads + threadIdx.x);
  prefetch_entries(run_tiles, n_run, row_tiles, gridDim.x / kBlocksPerTile);
}

// Several chunk ranges of one direction in one launch: blockIdx.y picks the range, blockIdx.x walks its tiles
// (workgroups past the end of a shorter range leave at once).  The ranges run one after the other in dispatch
// order, as their own launches would, without the gap between launches.
struct alignas(32) Seg2D {
  const RunTile* run;
  const RowTile* row;
  const uint64_t* gather;
  uint32_t n_run;
  uint32_t n_tiles;
};
struct Args2D {
  Seg2D seg[ETHA_MAX_SEGMENTS];
};

template <bool REV>
__global__ __launch_bounds__(ETHA_BLOCK_THREADS) void etha_tile_kernel_2d(const Args2D args) {
  typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
  const u32x8 raw = *reinterpret_cast<const u32x8*>(&args.seg[blockIdx.y]);  // the whole entry in one scalar load
  const uint32_t bid = blockIdx.x / kBlocksPerTile;
  if (bid >= raw[7]) return;
  // (pointers rebuilt from integers must be told that they point to device memory, or they are dereferenced
  // with per-lane generic loads instead of scalar loads: measured 7 % slower)
  typedef const __attribute__((address_space(1))) RunTile* GlobalRun;
  typedef const __attribute__((address_space(1))) RowTile* GlobalRow;
  typedef const __attribute__((address_space(1))) uint64_t* GlobalU64;
  const RunTile* run = (const RunTile*)(GlobalRun)(((uint64_t)raw[1] << 32) | raw[0]);
  const RowTile* row = (const RowTile*)(GlobalRow)(((uint64_t)raw[3] << 32) | raw[2]);
  const uint64_t* gather = (const uint64_t*)(GlobalU64)(((uint64_t)raw[5] << 32) | raw[4]);
  tile_body<REV>(run, raw[6], row, gather, bid, (blockIdx.x % kBlocksPerTile) * kBlockThreads + threadIdx.x);
  prefetch_entries(run, raw[6], row, raw[7]);
}

// The gather tiles of write-ordered unpack ranges (see kMetaGather).  Consecutive 1 KiB pieces of such a tile read
// source lines that they share with their neighbours (a piece of 96 bytes does not end on a line), so the
// workgroups of one tile should share an L2: workgroups are dealt to the eight XCDs in turn, and this kernel lets
// workgroup w of every 128 handle piece w / 8 of tile w % 8 - the sixteen pieces of a tile then run on one XCD,
// close in time.  Measured on 96- to 480-byte pieces: 5.1-5.3 -> 6.25-6.3 TB/s.  (The same mapping costs plain
// copies 8 %: it is used for gather tiles only.)
static_assert(kBlocksPerTile == 16, "the XCD mapping below deals 8 tiles x 16 pieces to 128 workgroups");
__global__ __launch_bounds__(ETHA_BLOCK_THREADS) void etha_gather_kernel(const Args2D args) {
  typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
  const u32x8 raw = *reinterpret_cast<const u32x8*>(&args.seg[blockIdx.y]);
  const uint32_t w = blockIdx.x, tile = ((w >> 7) << 3) + (w & 7u), piece = (w & 127u) >> 3;
  if (tile >= raw[7]) return;
  typedef const __attribute__((address_space(1))) RowTile* GlobalRow;
  typedef const __attribute__((address_space(1))) uint64_t* GlobalU64;
  const RowTile* row = (const RowTile*)(GlobalRow)(((uint64_t)raw[3] << 32) | raw[2]);
  const uint64_t* gather = (const uint64_t*)(GlobalU64)(((uint64_t)raw[5] << 32) | raw[4]);
  tile_body<true, true>(nullptr, 0u, row, gather, tile, piece * kBlockThreads + threadIdx.x);
}

// An unpack range with both kinds of tile in one launch: the plain tiles first, then (from the next multiple of
// 128 workgroups on, which keeps the dealing above) the gather tiles.  One launch instead of two that run side by
// side: two kernels in flight interleave their address streams, and the gather part of a range is short.
__global__ __launch_bounds__(ETHA_BLOCK_THREADS) void etha_unpack_mixed_kernel(const RunTile* __restrict__ run_tiles,
                                                                                const RowTile* __restrict__ row_tiles,
                                                                                const uint64_t* __restrict__ gather,
                                                                                uint32_t n_run, uint32_t n_plain,
                                                                                uint32_t n_gather) {
  const uint32_t w = blockIdx.x, plain_groups = n_plain * kBlocksPerTile;
  if (w < plain_groups) {
    tile_body<true>(run_tiles, n_run, row_tiles, gather, w / kBlocksPerTile, (w % kBlocksPerTile) * kBlockThreads + threadIdx.x);
    return;
  }
  const uint32_t base = (plain_groups + 127u) & ~127u;
  if (w < base) return;
  const uint32_t g = w - base, tile = ((g >> 7) << 3) + (g & 7u), piece = (g & 127u) >> 3;
  if (tile >= n_gather) return;
  tile_body<true, true>(nullptr, 0u, row_tiles + (n_plain - n_run), gather, tile, piece * kBlockThreads + threadIdx.x);
}

// ---- transposing chunks: staged through LDS -----------------------------------------------------
// The a side is contiguous along j, the b side along k.  A full block of D x D elements is read with 16-byte
// vectors along the source's contiguous dim (consecutive work-items cover one row, then the next row),
// parked in LDS row by row, and written with 16-byte vectors along the destination's contiguous dim, each
// vector gathered element by element from LDS.  Both global sides therefore move whole 16-byte vectors in
// runs of at least 128 bytes; without the staging one side would touch a different line per element.
// Blocks at the edge of a chunk (fewer than D elements on a side) take the element-wise path.
// The steps of one block of DY source rows of DX elements: work-item tid handles vectors q = tid + i * kTransThreads,
// counted row by row.
template <typename E, uint32_t DX, uint32_t DY>
struct TransBlock {
  static constexpr uint32_t kEs = sizeof(E), kV = 16 / kEs, kVecPerRow = DX / kV, kOutPerRow = DY / kV;
  static constexpr uint32_t kPitchBytes = trans_pitch(DX, kEs) * kEs;  // a multiple of 4
  static constexpr uint32_t kVecs = DY * kVecPerRow, kPerThread = (kVecs + kTransThreads - 1) / kTransThreads;
  static constexpr bool kExact = kVecs % kTransThreads == 0;

  static __device__ __forceinline__ void load(u32x4 (&v)[kPerThread], uint64_t src, int64_t src_pitch) {
    const uint32_t tid = threadIdx.x;
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; i++) {
      const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
      if (kExact || q < kVecs) v[i] = ld_stream<u32x4_any>(src + (uint64_t)((int64_t)y * src_pitch) + xv * 16u);
    }
  }
  static __device__ __forceinline__ void park(const u32x4 (&v)[kPerThread], uint8_t* __restrict__ lds) {
    const uint32_t tid = threadIdx.x;
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; i++) {
      const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
      if (!kExact && q >= kVecs) break;
      uint32_t* row = reinterpret_cast<uint32_t*>(lds + y * kPitchBytes + xv * 16u);
      row[0] = v[i][0];
      row[1] = v[i][1];
      row[2] = v[i][2];
      row[3] = v[i][3];
    }
  }
  // writes the DX destination rows (index x) of DY elements out of the parked rows
  static __device__ __forceinline__ void emit(const uint8_t* __restrict__ lds, uint64_t dst, int64_t dst_pitch) {
    const uint32_t tid = threadIdx.x;
    if constexpr (kEs == 2) {
      // two destination rows at a time: the 32-bit words of 8 source rows hold the elements of columns x and x + 1
      constexpr uint32_t kPairs = kVecs / 2, kPairsPerThread = (kPairs + kTransThreads - 1) / kTransThreads;
#pragma unroll
      for (uint32_t i = 0; i < kPairsPerThread; i++) {
        const uint32_t q = tid + i * kTransThreads, xp = q / kOutPerRow, yv = q % kOutPerRow;
        if (kPairs % kTransThreads != 0 && q >= kPairs) break;
        uint32_t w[8];
#pragma unroll
        for (uint32_t e = 0; e < 8; e++) w[e] = *reinterpret_cast<const uint32_t*>(lds + (yv * 8 + e) * kPitchBytes + xp * 4u);
        u32x4 lo, hi;
#pragma unroll
        for (uint32_t p = 0; p < 4; p++) {
          lo[p] = (w[2 * p] & 0xffffu) | (w[2 * p + 1] << 16);
          hi[p] = (w[2 * p] >> 16) | (w[2 * p + 1] & 0xffff0000u);
        }
        const uint64_t d0 = dst + (uint64_t)((int64_t)(2 * xp) * dst_pitch) + yv * 16u;
        st_stream<u32x4_any>(d0, lo);
        st_stream<u32x4_any>(d0 + (uint64_t)dst_pitch, hi);
      }
      return;
    }
    if constexpr (kEs == 1) {
      // four destination rows at a time: the 32-bit words of 16 source rows hold the bytes of columns x .. x + 3
      constexpr uint32_t kQuads = kVecs / 4, kQuadsPerThread = (kQuads + kTransThreads - 1) / kTransThreads;
#pragma unroll
      for (uint32_t i = 0; i < kQuadsPerThread; i++) {
        const uint32_t q = tid + i * kTransThreads, xq = q / kOutPerRow, yv = q % kOutPerRow;
        if (kQuads % kTransThreads != 0 && q >= kQuads) break;
        u32x4 col[4];
#pragma unroll
        for (uint32_t p = 0; p < 4; p++) {
          uint32_t w[4];
#pragma unroll
          for (uint32_t e = 0; e < 4; e++) w[e] = *reinterpret_cast<const uint32_t*>(lds + (yv * 16 + p * 4 + e) * kPitchBytes + xq * 4u);
          // 4 x 4 byte transposition; selector bytes 0-3 pick from the second operand, 4-7 from the first
          const uint32_t a = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u), b = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);
          const uint32_t c = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u), d = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
          col[0][p] = __builtin_amdgcn_perm(c, a, 0x05040100u);
          col[1][p] = __builtin_amdgcn_perm(c, a, 0x07060302u);
          col[2][p] = __builtin_amdgcn_perm(d, b, 0x05040100u);
          col[3][p] = __builtin_amdgcn_perm(d, b, 0x07060302u);
        }
        const uint64_t d0 = dst + (uint64_t)((int64_t)(4 * xq) * dst_pitch) + yv * 16u;
#pragma unroll
        for (uint32_t c = 0; c < 4; c++) st_stream<u32x4_any>(d0 + (uint64_t)((int64_t)c * dst_pitch), col[c]);
      }
      return;
    }
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; i++) {
      const uint32_t q = tid + i * kTransThreads, x = q / kOutPerRow, yv = q % kOutPerRow;
      if (!kExact && q >= kVecs) break;
      Pack<E, kV> out;
#pragma unroll
      for (uint32_t e = 0; e < kV; e++)
        out.set(e, *reinterpret_cast<const E*>(lds + (yv * kV + e) * kPitchBytes + x * kEs));
      out.store(dst + (uint64_t)((int64_t)x * dst_pitch) + yv * 16u);
    }
  }
};

template <typename E, uint32_t DX, uint32_t DY>
__device__ __forceinline__ void transpose_full(uint64_t src, int64_t src_pitch, uint64_t dst, int64_t dst_pitch,
                                               uint8_t* __restrict__ lds) {
  // src: DY rows (index y) of DX elements contiguous along x.  dst: DX rows (index x) of DY elements along y.
  typedef TransBlock<E, DX, DY> B;
  u32x4 v[B::kPerThread];
  B::load(v, src, src_pitch);
  B::park(v, lds);
  __syncthreads();
  B::emit(lds, dst, dst_pitch);
}

// A block of P * DX x DY elements: every load is issued first, then the P column panels of DX elements go
// through LDS one after the other.  Both global sides then move runs of P * DX and DY elements while LDS holds
// one panel only.
template <typename E, uint32_t DX, uint32_t DY, uint32_t P>
__device__ __forceinline__ void transpose_panels(uint64_t src, int64_t src_pitch, uint64_t dst, int64_t dst_pitch,
                                                 uint8_t* __restrict__ lds) {
  typedef TransBlock<E, DX, DY> B;
  static_assert(B::kExact, "a panel is a whole number of vectors per work-item");
  u32x4 v[P][B::kPerThread];
#pragma unroll
  for (uint32_t h = 0; h < P; h++) B::load(v[h], src + h * DX * sizeof(E), src_pitch);
#pragma unroll
  for (uint32_t h = 0; h < P; h++) {
    if (h) __syncthreads();
    B::park(v[h], lds);
    __syncthreads();
    B::emit(lds, dst + (uint64_t)((int64_t)(h * DX) * dst_pitch), dst_pitch);
  }
}

template <typename E, uint32_t DX>
__device__ __forceinline__ void transpose_edge(uint64_t src, int64_t src_pitch, uint32_t nx, uint64_t dst,
                                               int64_t dst_pitch, uint32_t ny, uint8_t* __restrict__ lds) {
  // same roles as above with nx <= DX elements per source row and ny <= DY source rows; one element per access
  constexpr uint32_t kEs = sizeof(E), kPitchBytes = trans_pitch(DX, kEs) * kEs;
  const uint32_t n = nx * ny;
  for (uint32_t q = threadIdx.x; q < n; q += kTransThreads) {
    const uint32_t y = q / nx, x = q - y * nx;
    *reinterpret_cast<E*>(lds + y * kPitchBytes + x * kEs) =
        ld_stream<E>(src + (uint64_t)((int64_t)y * src_pitch) + (uint64_t)x * kEs);
  }
  __syncthreads();
  for (uint32_t q = threadIdx.x; q < n; q += kTransThreads) {
    const uint32_t x = q / ny, y = q - x * ny;
    st_stream<E>(dst + (uint64_t)((int64_t)x * dst_pitch) + (uint64_t)y * kEs,
                 *reinterpret_cast<const E*>(lds + y * kPitchBytes + x * kEs));
  }
}

// Transposing blocks that also convert: the a side holds f32, the b side (the bucket) f16 or bf16.  LDS holds the
// 16-bit elements, so the staging is that of a 2-byte block: a pack converts while it parks (four f32 of a source
// row become two words), an unpack while it emits (the eight elements of a gathered vector become two vectors).
template <typename TB, uint32_t DX, uint32_t DY>
__device__ __forceinline__ void transpose_cvt_pack(uint64_t src, int64_t src_pitch, uint64_t dst, int64_t dst_pitch,
                                                   uint8_t* __restrict__ lds) {
  // src: DY rows of DX f32 contiguous along x.  dst: DX rows of DY 16-bit elements.
  typedef TransBlock<uint16_t, DX, DY> B;
  constexpr uint32_t kVecPerRow = DX / 4, kVecs = DY * kVecPerRow, kPerThread = kVecs / kTransThreads;
  static_assert(kVecs % kTransThreads == 0, "a whole number of f32 vectors per work-item");
  const uint32_t tid = threadIdx.x;
  u32x4 v[kPerThread];
#pragma unroll
  for (uint32_t i = 0; i < kPerThread; i++) {
    const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
    v[i] = ld_stream<u32x4_any>(src + (uint64_t)((int64_t)y * src_pitch) + xv * 16u);
  }
#pragma unroll
  for (uint32_t i = 0; i < kPerThread; i++) {
    const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
    uint32_t h[4];
#pragma unroll
    for (uint32_t e = 0; e < 4; e++) h[e] = from_f32(TB(), to_f32(TagF32(), v[i][e]));
    uint32_t* row = reinterpret_cast<uint32_t*>(lds + y * B::kPitchBytes + xv * 8u);
    row[0] = h[0] | (h[1] << 16);
    row[1] = h[2] | (h[3] << 16);
  }
  __syncthreads();
  B::emit(lds, dst, dst_pitch);
}

template <typename TB, uint32_t DX, uint32_t DY>
__device__ __forceinline__ void transpose_cvt_unpack(uint64_t src, int64_t src_pitch, uint64_t dst, int64_t dst_pitch,
                                                     uint8_t* __restrict__ lds) {
  // src: DY rows of DX 16-bit elements contiguous along x.  dst: DX rows of DY f32.
  typedef TransBlock<uint16_t, DX, DY> B;
  u32x4 v[B::kPerThread];
  B::load(v, src, src_pitch);
  B::park(v, lds);
  __syncthreads();
  // two destination rows per work-item, four f32 (one vector) of each: the words of 4 source rows hold the elements
  // of columns x and x + 1, and consecutive work-items write consecutive vectors of a destination row
  constexpr uint32_t kQuadsPerRow = DY / 4, kItems = (DX / 2) * kQuadsPerRow, kItemsPerThread = (kItems + kTransThreads - 1) / kTransThreads;
  const uint32_t tid = threadIdx.x;
#pragma unroll
  for (uint32_t i = 0; i < kItemsPerThread; i++) {
    const uint32_t q = tid + i * kTransThreads, xp = q / kQuadsPerRow, y4 = q % kQuadsPerRow;
    if (kItems % kTransThreads != 0 && q >= kItems) break;
    u32x4 lo, hi;
#pragma unroll
    for (uint32_t e = 0; e < 4; e++) {
      const uint32_t w = *reinterpret_cast<const uint32_t*>(lds + (y4 * 4 + e) * B::kPitchBytes + xp * 4u);
      lo[e] = from_f32(TagF32(), to_f32(TB(), (uint16_t)(w & 0xffffu)));
      hi[e] = from_f32(TagF32(), to_f32(TB(), (uint16_t)(w >> 16)));
    }
    const uint64_t d0 = dst + (uint64_t)((int64_t)(2 * xp) * dst_pitch) + y4 * 16u;
    st_stream<u32x4_any>(d0, lo);
    st_stream<u32x4_any>(d0 + (uint64_t)dst_pitch, hi);
  }
}

template <typename TB, bool REV, uint32_t DX>
__device__ __forceinline__ void transpose_cvt_edge(uint64_t src, int64_t src_pitch, uint32_t nx, uint64_t dst,
                                                   int64_t dst_pitch, uint32_t ny, uint8_t* __restrict__ lds) {
  // nx <= DX elements per source row, ny source rows; one element per access, 16-bit elements in LDS
  constexpr uint32_t kPitchBytes = trans_pitch(DX, 2) * 2;
  const uint32_t n = nx * ny;
  for (uint32_t q = threadIdx.x; q < n; q += kTransThreads) {
    const uint32_t y = q / nx, x = q - y * nx;
    const uint64_t at = src + (uint64_t)((int64_t)y * src_pitch);
    *reinterpret_cast<uint16_t*>(lds + y * kPitchBytes + x * 2u) =
        REV ? ld_stream<uint16_t>(at + (uint64_t)x * 2u) : from_f32(TB(), to_f32(TagF32(), ld_stream<uint32_t>(at + (uint64_t)x * 4u)));
  }
  __syncthreads();
  for (uint32_t q = threadIdx.x; q < n; q += kTransThreads) {
    const uint32_t x = q / ny, y = q - x * ny;
    const uint16_t h = *reinterpret_cast<const uint16_t*>(lds + y * kPitchBytes + x * 2u);
    const uint64_t at = dst + (uint64_t)((int64_t)x * dst_pitch);
    if (REV)
      st_stream<uint32_t>(at + (uint64_t)y * 4u, from_f32(TagF32(), to_f32(TB(), h)));
    else
      st_stream<uint16_t>(at + (uint64_t)y * 2u, h);
  }
}

template <typename TB, bool REV>
__device__ __forceinline__ void transpose_block_cvt(const TransTile& t, uint8_t* __restrict__ lds) {
  constexpr uint32_t kDX = REV ? trans_dim_b(2) : trans_dim_a(2), kDY = REV ? trans_dim_a(2) : trans_dim_b(2);
  const uint64_t src = REV ? t.b : t.a, dst = REV ? t.a : t.b;
  const int64_t src_pitch = REV ? t.b_pitch : t.a_pitch, dst_pitch = REV ? t.a_pitch : t.b_pitch;
  const uint32_t nx = REV ? t.nk : t.nj, ny = REV ? t.nj : t.nk;
  if (t.nj == kTransCvtWideJ && t.nk == kTransCvtWideK) {  // runs of 512 bytes on both sides: 128 f32, 256 16-bit elements
    if constexpr (REV)
      transpose_cvt_unpack<TB, kTransCvtWideK, kTransCvtWideJ>(src, src_pitch, dst, dst_pitch, lds);
    else
      transpose_cvt_pack<TB, kTransCvtWideJ, kTransCvtWideK>(src, src_pitch, dst, dst_pitch, lds);
  } else if (nx == kDX && ny == kDY) {
    if constexpr (REV)
      transpose_cvt_unpack<TB, kDX, kDY>(src, src_pitch, dst, dst_pitch, lds);
    else
      transpose_cvt_pack<TB, kDX, kDY>(src, src_pitch, dst, dst_pitch, lds);
  } else {
    transpose_cvt_edge<TB, REV, kDX>(src, src_pitch, nx, dst, dst_pitch, ny, lds);
  }
}

template <typename E, bool REV>
__device__ __forceinline__ void transpose_block(const TransTile& t, uint8_t* __restrict__ lds) {
  // pack (a -> b): source rows run along j (one row per k); unpack (b -> a): source rows run along k (one per j)
  constexpr uint32_t kDX = REV ? trans_dim_b(sizeof(E)) : trans_dim_a(sizeof(E));
  constexpr uint32_t kDY = REV ? trans_dim_a(sizeof(E)) : trans_dim_b(sizeof(E));
  const uint64_t src = REV ? t.b : t.a, dst = REV ? t.a : t.b;
  const int64_t src_pitch = REV ? t.b_pitch : t.a_pitch, dst_pitch = REV ? t.a_pitch : t.b_pitch;
  const uint32_t nx = REV ? t.nk : t.nj, ny = REV ? t.nj : t.nk;
  constexpr uint32_t kW = trans_wide(sizeof(E)), kP = trans_panels(sizeof(E));
  if constexpr (kW > 1) {
    if (nx == kDX * kW && ny == kDY * kW) {  // a wide block
      transpose_panels<E, kDX * kW / kP, kDY * kW, kP>(src, src_pitch, dst, dst_pitch, lds);
      return;
    }
  }
  if (nx == kDX && ny == kDY)
    transpose_full<E, kDX, kDY>(src, src_pitch, dst, dst_pitch, lds);
  else
    transpose_edge<E, kDX>(src, src_pitch, nx, dst, dst_pitch, ny, lds);
}

template <bool REV>
__device__ __forceinline__ void transpose_tile(const TransTile& t, uint8_t* __restrict__ lds) {
  if (t.cvt & kTransTyped) return;  // a block of the typed kernel (uniform over the workgroup: no barrier is skipped)
  if (t.cvt) {  // f32 on the a side, f16 or bf16 on the b side
    if ((t.cvt & 15u) == ETHA_F16)
      transpose_block_cvt<TagF16, REV>(t, lds);
    else
      transpose_block_cvt<TagBF16, REV>(t, lds);
    return;
  }
  switch (t.es_log2) {
    case 0: transpose_block<uint8_t, REV>(t, lds); break;
    case 1: transpose_block<uint16_t, REV>(t, lds); break;
    case 2: transpose_block<uint32_t, REV>(t, lds); break;
    default: transpose_block<uint64_t, REV>(t, lds); break;
  }
}

template <bool REV>
__global__ __launch_bounds__(ETHA_TRANS_THREADS) void etha_transpose_kernel(const TransTile* __restrict__ tiles) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];  // trans_lds_bytes(largest element size)
  const TransTile t = tiles[blockIdx.x];
  transpose_tile<REV>(t, lds_bytes);
}

// several tables' transposing tiles in one launch: blockIdx.y picks the list, as in etha_tile_kernel_2d
struct alignas(16) TransSeg {
  const TransTile* tiles;
  uint32_t n;
  uint32_t reserved;
};
struct TransArgs {
  TransSeg seg[ETHA_MAX_SEGMENTS];
};

template <bool REV>
__global__ __launch_bounds__(ETHA_TRANS_THREADS) void etha_transpose_kernel_2d(const TransArgs args) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];
  const u32x4 raw = *reinterpret_cast<const u32x4*>(&args.seg[blockIdx.y]);
  if (blockIdx.x >= raw[2]) return;  // the whole workgroup leaves: no barrier is skipped by part of it
  typedef const __attribute__((address_space(1))) TransTile* GlobalTrans;
  const TransTile* tiles = (const TransTile*)(GlobalTrans)(((uint64_t)raw[1] << 32) | raw[0]);
  const TransTile t = tiles[blockIdx.x];
  transpose_tile<REV>(t, lds_bytes);
}

// ---- Partial reduce-pack ------------------------------------------------------------------------
template <typename ACC>
__device__ __forceinline__ ACC combine(uint32_t op, ACC x, ACC y) {
  switch (op) {
    case ETHA_MAX: return x > y ? x : (y > x ? y : (x == x ? x : y));
    case ETHA_MIN: return x < y ? x : (y < x ? y : (x == x ? x : y));
    case ETHA_PRODUCT: return x * y;
    default: return x + y;  // SUM, AVG
  }
}

template <typename S, int N>
struct LoadF32 {
  __device__ static __forceinline__ void run(uint64_t addr, float* out) {
    Pack<typename S::bits, N> in;
    in.load(addr);
#pragma unroll
    for (int i = 0; i < N; i++) out[i] = to_f32(S(), in.get(i));
  }
};

// A reduction that writes a tensor directly (no bucket in between) still rounds the way the bucket path
// does: accumulator -> wire dtype -> tensor dtype.  `via` names the wire dtype when it differs from the
// b-side dtype (0 = no intermediate rounding).
__device__ __forceinline__ float round_via(uint32_t via, float r) {
  switch (via) {
    case 1 + ETHA_F16: return to_f32(TagF16(), from_f32(TagF16(), r));
    case 1 + ETHA_BF16: return to_f32(TagBF16(), from_f32(TagBF16(), r));
    default: return r;
  }
}

// Reduce-op word of a reduce tile: bits 0-2 the op of the innermost level, 3-5 and 6-8 the ops of the next
// levels, bits 16-23 / 24-31 the member counts g0 / g1 of the two inner levels (0 = one level over all peers).
// Peers are listed innermost level fastest.  Level l combines, in list order, the results of level l - 1;
// an AVG level divides by its own member count.  One level is the common case (one Partial mesh dim, or
// several with the same op, combined in rank order); several levels are Partial mesh dims with different
// ops, applied in mesh-dim order as the reference's per-group all-reduces are (ir.py:123-124).
__device__ __forceinline__ uint32_t level_op(uint32_t word, int level) { return (word >> (3 * level)) & 7u; }

template <typename ACC, typename LOAD, int N>
__device__ __forceinline__ void reduce_levels(const uint64_t* __restrict__ peers, uint32_t np, uint32_t word,
                                              uint64_t a_off, ACC* acc) {
  const uint32_t g0 = (word >> 16) & 255u, g1raw = (word >> 24) & 255u, g1 = g1raw ? g1raw : 1u;
  const uint32_t g2 = np / (g0 * g1);
  const uint32_t op0 = level_op(word, 0), op1 = level_op(word, 1), op2 = level_op(word, 2);
  uint32_t p = 0;
  ACC mid[N];
  for (uint32_t i2 = 0; i2 < g2; i2++) {
    for (uint32_t i1 = 0; i1 < g1; i1++) {
      ACC inner[N];
      LOAD::run(peers[p++] + a_off, inner);
      for (uint32_t i0 = 1; i0 < g0; i0++) {
        ACC v[N];
        LOAD::run(peers[p++] + a_off, v);
#pragma unroll
        for (int i = 0; i < N; i++) inner[i] = combine(op0, inner[i], v[i]);
      }
#pragma unroll
      for (int i = 0; i < N; i++) {
        if (op0 == ETHA_AVG) inner[i] = inner[i] / (ACC)g0;
        mid[i] = i1 == 0 ? inner[i] : combine(op1, mid[i], inner[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < N; i++) {
      if (op1 == ETHA_AVG) mid[i] = mid[i] / (ACC)g1;
      acc[i] = i2 == 0 ? mid[i] : combine(op2, acc[i], mid[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < N; i++)
    if (op2 == ETHA_AVG) acc[i] = acc[i] / (ACC)g2;
}

// f16/bf16/f32 partials: fp32 accumulation, peers combined strictly in list (= rank) order.
template <typename S, typename D, int N>
__device__ __forceinline__ void reduce_f32(const uint64_t* __restrict__ peers, uint32_t np, uint32_t op, uint32_t via,
                                           uint64_t a_off, uint64_t dst) {
  float acc[N];
  if (op >> 16) {  // several levels
    reduce_levels<float, LoadF32<S, N>, N>(peers, np, op, a_off, acc);
    Pack<typename D::bits, N> out;
#pragma unroll
    for (int i = 0; i < N; i++) out.set(i, from_f32(D(), round_via(via, acc[i])));
    out.store(dst);
    return;
  }
  LoadF32<S, N>::run(peers[0] + a_off, acc);
  uint32_t p = 1;
  for (; p + 3 <= np; p += 3) {  // three peers' loads in flight, then combine in order
    float v0[N], v1[N], v2[N];
    LoadF32<S, N>::run(peers[p] + a_off, v0);
    LoadF32<S, N>::run(peers[p + 1] + a_off, v1);
    LoadF32<S, N>::run(peers[p + 2] + a_off, v2);
#pragma unroll
    for (int i = 0; i < N; i++) acc[i] = combine(op, combine(op, combine(op, acc[i], v0[i]), v1[i]), v2[i]);
  }
  for (; p < np; p++) {
    float v[N];
    LoadF32<S, N>::run(peers[p] + a_off, v);
#pragma unroll
    for (int i = 0; i < N; i++) acc[i] = combine(op, acc[i], v[i]);
  }
  Pack<typename D::bits, N> out;
  const float cnt = (float)np;
#pragma unroll
  for (int i = 0; i < N; i++) {
    float r = acc[i];
    if (op == ETHA_AVG) r = r / cnt;
    out.set(i, from_f32(D(), round_via(via, r)));
  }
  out.store(dst);
}

template <int N>
struct LoadF64 {
  __device__ static __forceinline__ void run(uint64_t addr, double* out) {
    Pack<uint64_t, N> in;
    in.load(addr);
#pragma unroll
    for (int i = 0; i < N; i++) out[i] = __builtin_bit_cast(double, in.get(i));
  }
};

// f64 partials: f64 accumulation; result converted like a plain f64 -> D move.
template <typename D, int N>
__device__ __forceinline__ void reduce_f64(const uint64_t* __restrict__ peers, uint32_t np, uint32_t op, uint32_t via,
                                           uint64_t a_off, uint64_t dst) {
  double acc[N];
  const bool levels = (op >> 16) != 0;
  if (levels) {
    reduce_levels<double, LoadF64<N>, N>(peers, np, op, a_off, acc);
  } else {
    LoadF64<N>::run(peers[0] + a_off, acc);
    for (uint32_t p = 1; p < np; p++) {
      double v[N];
      LoadF64<N>::run(peers[p] + a_off, v);
#pragma unroll
      for (int i = 0; i < N; i++) acc[i] = combine(op, acc[i], v[i]);
    }
  }
  Pack<typename D::bits, N> out;
#pragma unroll
  for (int i = 0; i < N; i++) {
    double r = acc[i];
    if (!levels && op == ETHA_AVG) r = r / (double)np;
    if (sizeof(typename D::bits) == 8 && via == 0)
      out.set(i, (typename D::bits)__builtin_bit_cast(uint64_t, r));
    else {
      float rf = (float)r;
      asm volatile("" : "+v"(rf));  // two roundings, as in the plain f64 -> D move
      out.set(i, from_f32(D(), round_via(via, rf)));
    }
  }
  out.store(dst);
}

template <typename S, typename D, int N>
__device__ __forceinline__ void reduce_n(const uint64_t* peers, uint32_t np, uint32_t op, uint32_t via, uint64_t a_off,
                                         uint64_t dst) {
  if constexpr (sizeof(typename S::bits) == 8)
    reduce_f64<D, N>(peers, np, op, via, a_off, dst);
  else
    reduce_f32<S, D, N>(peers, np, op, via, a_off, dst);
}

// nl = log2 of the elements in this unit (at most 16 bytes on the wider side)
template <typename S, typename D>
__device__ __forceinline__ void reduce_pair(uint32_t nl, const uint64_t* peers, uint32_t np, uint32_t op, uint32_t via,
                                            uint64_t a_off, uint64_t dst) {
  constexpr int kMaxBytes = sizeof(typename S::bits) > sizeof(typename D::bits) ? sizeof(typename S::bits)
                                                                                  : sizeof(typename D::bits);
  constexpr int kN = 16 / kMaxBytes;
  if constexpr (kN >= 8) {
    if (nl == 3) return reduce_n<S, D, 8>(peers, np, op, via, a_off, dst);
  }
  if constexpr (kN >= 4) {
    if (nl == 2) return reduce_n<S, D, 4>(peers, np, op, via, a_off, dst);
  }
  if constexpr (kN >= 2) {
    if (nl == 1) return reduce_n<S, D, 2>(peers, np, op, via, a_off, dst);
  }
  reduce_n<S, D, 1>(peers, np, op, via, a_off, dst);
}

template <typename S>
__device__ __forceinline__ void reduce_from(uint32_t dd, uint32_t nl, const uint64_t* peers, uint32_t np, uint32_t op,
                                            uint32_t via, uint64_t a_off, uint64_t dst) {
  switch (dd) {
    case ETHA_F16: reduce_pair<S, TagF16>(nl, peers, np, op, via, a_off, dst); break;
    case ETHA_BF16: reduce_pair<S, TagBF16>(nl, peers, np, op, via, a_off, dst); break;
    case ETHA_F32: reduce_pair<S, TagF32>(nl, peers, np, op, via, a_off, dst); break;
    default: reduce_pair<S, TagF64>(nl, peers, np, op, via, a_off, dst); break;
  }
}

__global__ __launch_bounds__(ETHA_BLOCK_THREADS) void etha_reduce_kernel(const RowTile* __restrict__ row_tiles,
                                                           const uint64_t* __restrict__ peer_bases) {
  const uint32_t tid = (blockIdx.x % kBlocksPerTile) * kBlockThreads + threadIdx.x;
  const RowTile t = row_tiles[blockIdx.x / kBlocksPerTile];
  if (tid >= t.n) return;
  uint32_t r, c;
  row_position(t, tid, r, c);
  const uint32_t meta = t.meta;
  const uint64_t a_off = t.a + (uint64_t)((int64_t)r * t.a_pitch) + ((uint64_t)c << ((meta >> kMetaUaShift) & 15u));
  const uint64_t dst = t.b + (uint64_t)((int64_t)r * t.b_pitch) + ((uint64_t)c << ((meta >> kMetaUbShift) & 15u));
  const uint64_t* peers = peer_bases + t.peer_first;
  const uint32_t nl = (meta >> kMetaElemsShift) & 3u;
  const uint32_t dd = (meta >> kMetaDtbShift) & 15u;
  switch ((meta >> kMetaDtaShift) & 15u) {
    case ETHA_F16: reduce_from<TagF16>(dd, nl, peers, t.n_peers, t.reduce_op, t.via, a_off, dst); break;
    case ETHA_BF16: reduce_from<TagBF16>(dd, nl, peers, t.n_peers, t.reduce_op, t.via, a_off, dst); break;
    case ETHA_F32: reduce_from<TagF32>(dd, nl, peers, t.n_peers, t.reduce_op, t.via, a_off, dst); break;
    default: reduce_from<TagF64>(dd, nl, peers, t.n_peers, t.reduce_op, t.via, a_off, dst); break;
  }
}

// ---- typed transposing blocks -------------------------------------------------------------------
// Transposing chunks that the plain transposing kernel does not take: any pair of value types, and Partial sources
// (the N members' blocks are combined in registers, strictly in list order, as the reduce kernel combines rows).
// The source side is read with 16-byte vectors along its contiguous dim, every element is converted to the
// destination's type (reduced first, for a Partial source) and parked in LDS, and the destination side is written
// by the same gather-from-LDS step the plain blocks use.  Edge blocks move element by element.
template <typename ES, int N, bool RED>
__device__ __forceinline__ void typed_values(uint32_t sd, uint32_t dd, uint64_t src, const uint64_t* __restrict__ peers,
                                             uint32_t np, uint32_t op, uint32_t via, uint64_t (&out)[N]) {
  Pack<ES, N> in;
  if constexpr (!RED) {
    in.load(src);
#pragma unroll
    for (int e = 0; e < N; e++) out[e] = convert_bits(sd, dd, (uint64_t)in.get(e));
    return;
  }
  // Partial source: src is an offset from each member's base; f16/bf16/f32 accumulate in fp32, f64 in f64
  if (sd == ETHA_F64) {
    double acc[N];
    in.load(peers[0] + src);
#pragma unroll
    for (int e = 0; e < N; e++) acc[e] = __builtin_bit_cast(double, (uint64_t)in.get(e));
    for (uint32_t p = 1; p < np; p++) {
      in.load(peers[p] + src);
#pragma unroll
      for (int e = 0; e < N; e++) acc[e] = combine(op, acc[e], __builtin_bit_cast(double, (uint64_t)in.get(e)));
    }
#pragma unroll
    for (int e = 0; e < N; e++) {
      double r = acc[e];
      if (op == ETHA_AVG) r = r / (double)np;
      if (dd == ETHA_F64 && via == 0) {
        out[e] = __builtin_bit_cast(uint64_t, r);
      } else {
        float rf = (float)r;
        asm volatile("" : "+v"(rf));  // two roundings, as in the plain f64 -> narrower move
        out[e] = float_bits(dd, round_via(via, rf));
      }
    }
    return;
  }
  float acc[N];
  in.load(peers[0] + src);
#pragma unroll
  for (int e = 0; e < N; e++) acc[e] = float_value(sd, (uint64_t)in.get(e));
  for (uint32_t p = 1; p < np; p++) {
    in.load(peers[p] + src);
#pragma unroll
    for (int e = 0; e < N; e++) acc[e] = combine(op, acc[e], float_value(sd, (uint64_t)in.get(e)));
  }
  const float cnt = (float)np;
#pragma unroll
  for (int e = 0; e < N; e++) {
    float r = acc[e];
    if (op == ETHA_AVG) r = r / cnt;
    out[e] = float_bits(dd, round_via(via, r));
  }
}

// Full block of a Partial source whose members hold f16, bf16 or f32: the loads of up to four members are in flight
// together (a member's vectors only meet the accumulators once all of the batch have been requested), members are
// still combined strictly in list order, and all conversions are straight-line code.
// SUM: true when the op is a sum or an average - the usual case, for which the combine step is straight-line code;
// with a run-time op every element of the unrolled loops would go through the op's switch.
template <typename S, typename D, uint32_t DX, uint32_t DY, bool SUM>
__device__ __forceinline__ void reduce_block_full(const TransTile& t, const uint64_t* __restrict__ peers, uint8_t* __restrict__ lds) {
  typedef typename S::bits ES;
  typedef typename D::bits ED;
  constexpr uint32_t kVs = 16 / sizeof(ES), kVecPerRow = DX / kVs, kVecs = DY * kVecPerRow, kPer = kVecs / kTransThreads;
  static_assert(kVecs % kTransThreads == 0 && kPer >= 1, "a whole number of vectors per work-item");
  constexpr uint32_t kPitchBytes = trans_pitch(DX, sizeof(ED)) * sizeof(ED);
  constexpr uint32_t kBatch = 2;  // members whose loads are in flight together
  const uint32_t tid = threadIdx.x, np = t.n_peers, op = t.reduce_op, via = t.via;
  uint64_t off[kPer];
#pragma unroll
  for (uint32_t i = 0; i < kPer; i++) {
    const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
    off[i] = t.a + (uint64_t)((int64_t)y * t.a_pitch) + xv * 16u;
  }
  float acc[kPer][kVs];
  for (uint32_t p = 0; p < np; p += kBatch) {
    Pack<ES, kVs> raw[kBatch][kPer];
#pragma unroll
    for (uint32_t j = 0; j < kBatch; j++)
      if (p + j < np) {
        const uint64_t base = peers[p + j];
#pragma unroll
        for (uint32_t i = 0; i < kPer; i++) raw[j][i].load(base + off[i]);
      }
    if (p == 0) {  // the first member starts the accumulators
#pragma unroll
      for (uint32_t i = 0; i < kPer; i++)
#pragma unroll
        for (uint32_t e = 0; e < kVs; e++) acc[i][e] = to_f32(S(), raw[0][i].get(e));
    }
#pragma unroll
    for (uint32_t j = 0; j < kBatch; j++)
      if (p + j < np && (j || p)) {
#pragma unroll
        for (uint32_t i = 0; i < kPer; i++)
#pragma unroll
          for (uint32_t e = 0; e < kVs; e++) {
            const float v = to_f32(S(), raw[j][i].get(e));
            acc[i][e] = SUM ? acc[i][e] + v : combine(op, acc[i][e], v);
          }
      }
  }
  const float cnt = (float)np;
#pragma unroll
  for (uint32_t i = 0; i < kPer; i++) {
    const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
    ED* row = reinterpret_cast<ED*>(lds + y * kPitchBytes) + xv * kVs;
#pragma unroll
    for (uint32_t e = 0; e < kVs; e++) {
      float r = acc[i][e];
      if (op == ETHA_AVG) r = r / cnt;
      row[e] = from_f32(D(), via ? round_via(via, r) : r);
    }
  }
  __syncthreads();
  TransBlock<ED, DX, DY>::emit(lds, t.b, t.b_pitch);
}

template <typename S, typename D, uint32_t DX, uint32_t DY>
__device__ __forceinline__ void reduce_block_any_op(const TransTile& t, const uint64_t* __restrict__ peers, uint8_t* __restrict__ lds) {
  if (t.reduce_op == ETHA_SUM || t.reduce_op == ETHA_AVG)
    reduce_block_full<S, D, DX, DY, true>(t, peers, lds);
  else
    reduce_block_full<S, D, DX, DY, false>(t, peers, lds);
}

template <typename S, typename ED, uint32_t DX, uint32_t DY>
__device__ __forceinline__ bool reduce_block_to(uint32_t dd, const TransTile& t, const uint64_t* __restrict__ peers, uint8_t* __restrict__ lds) {
  if constexpr (sizeof(ED) == 2) {
    if (dd == ETHA_F16) {
      reduce_block_any_op<S, TagF16, DX, DY>(t, peers, lds);
      return true;
    }
    if (dd == ETHA_BF16) {
      reduce_block_any_op<S, TagBF16, DX, DY>(t, peers, lds);
      return true;
    }
  }
  if constexpr (sizeof(ED) == 4) {
    if (dd == ETHA_F32) {
      reduce_block_any_op<S, TagF32, DX, DY>(t, peers, lds);
      return true;
    }
  }
  return false;
}

template <typename ES, typename ED, bool RED>
__device__ __forceinline__ void typed_block(const TransTile& t, bool rev, const uint64_t* __restrict__ peer_bases, uint8_t* __restrict__ lds) {
  constexpr uint32_t kD = trans_typed_dim(sizeof(ES), sizeof(ED));
  constexpr uint32_t kPitchBytes = trans_pitch(kD, sizeof(ED)) * sizeof(ED);
  const uint32_t dta = (t.cvt >> 4) & 15u, dtb = t.cvt & 15u;
  const uint32_t sd = rev ? dtb : dta, dd = rev ? dta : dtb;
  const uint64_t src = rev ? t.b : t.a, dst = rev ? t.a : t.b;
  const int64_t src_pitch = rev ? t.b_pitch : t.a_pitch, dst_pitch = rev ? t.a_pitch : t.b_pitch;
  const uint32_t nx = rev ? t.nk : t.nj, ny = rev ? t.nj : t.nk;  // elements per source row, source rows
  const uint64_t* peers = peer_bases + t.peer_first;
  const uint32_t np = t.n_peers, op = t.reduce_op, via = t.via, tid = threadIdx.x;
  if constexpr (RED && sizeof(ES) == 2 && sizeof(ED) <= 4) {  // f16 / bf16 members: the straight-line path, its own block shape
    if (nx == kRedDimJ2 && ny == kRedDimK2) {
      bool done = false;
      if (sd == ETHA_F16) done = reduce_block_to<TagF16, ED, kRedDimJ2, kRedDimK2>(dd, t, peers, lds);
      if (sd == ETHA_BF16) done = reduce_block_to<TagBF16, ED, kRedDimJ2, kRedDimK2>(dd, t, peers, lds);
      if (done) return;
    }
  }
  if (nx == kD && ny == kD) {
    if constexpr (RED && sizeof(ES) == 4 && sizeof(ED) <= 4) {  // f32 members
      if (sd == ETHA_F32 && reduce_block_to<TagF32, ED, kD, kD>(dd, t, peers, lds)) return;
    }
    constexpr uint32_t kVs = 16 / sizeof(ES), kVecPerRow = kD / kVs, kVecs = kD * kVecPerRow;
    constexpr uint32_t kPerThread = (kVecs + kTransThreads - 1) / kTransThreads;
#pragma unroll
    for (uint32_t i = 0; i < kPerThread; i++) {
      const uint32_t q = tid + i * kTransThreads, y = q / kVecPerRow, xv = q % kVecPerRow;
      if (kVecs % kTransThreads == 0 || q < kVecs) {
        uint64_t v[kVs];
        typed_values<ES, (int)kVs, RED>(sd, dd, src + (uint64_t)((int64_t)y * src_pitch) + xv * 16u, peers, np, op, via, v);
        ED* row = reinterpret_cast<ED*>(lds + y * kPitchBytes) + xv * kVs;
#pragma unroll
        for (uint32_t e = 0; e < kVs; e++) row[e] = (ED)v[e];
      }
    }
    __syncthreads();
    TransBlock<ED, kD, kD>::emit(lds, dst, dst_pitch);
    return;
  }
  const uint32_t n = nx * ny;
  for (uint32_t q = tid; q < n; q += kTransThreads) {
    const uint32_t y = q / nx, x = q - y * nx;
    uint64_t v[1];
    typed_values<ES, 1, RED>(sd, dd, src + (uint64_t)((int64_t)y * src_pitch) + (uint64_t)x * sizeof(ES), peers, np, op, via, v);
    *reinterpret_cast<ED*>(lds + y * kPitchBytes + x * sizeof(ED)) = (ED)v[0];
  }
  __syncthreads();
  for (uint32_t q = tid; q < n; q += kTransThreads) {
    const uint32_t x = q / ny, y = q - x * ny;
    st_stream<ED>(dst + (uint64_t)((int64_t)x * dst_pitch) + (uint64_t)y * sizeof(ED),
                  *reinterpret_cast<const ED*>(lds + y * kPitchBytes + x * sizeof(ED)));
  }
}

template <typename ES, bool RED>
__device__ __forceinline__ void typed_block_to(uint32_t dst_bytes, const TransTile& t, bool rev, const uint64_t* __restrict__ peers,
                                               uint8_t* __restrict__ lds) {
  switch (dst_bytes) {
    case 1:
      if constexpr (!RED) typed_block<ES, uint8_t, RED>(t, rev, peers, lds);  // no 1-byte float takes part in a reduction
      break;
    case 2: typed_block<ES, uint16_t, RED>(t, rev, peers, lds); break;
    case 4: typed_block<ES, uint32_t, RED>(t, rev, peers, lds); break;
    default: typed_block<ES, uint64_t, RED>(t, rev, peers, lds); break;
  }
}

// blocks that convert between two value types (no Partial source); rev = unpack direction
__global__ __launch_bounds__(ETHA_TRANS_THREADS) void etha_transpose_typed_kernel(const TransTile* __restrict__ tiles, uint32_t rev) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];
  const TransTile t = tiles[blockIdx.x];
  if (!(t.cvt & kTransTyped) || t.n_peers) return;  // another kernel's block (the whole workgroup leaves)
  const uint32_t dta = (t.cvt >> 4) & 15u, dtb = t.cvt & 15u;
  const uint32_t src_bytes = dtype_bytes(rev ? dtb : dta), dst_bytes = dtype_bytes(rev ? dta : dtb);
  switch (src_bytes) {
    case 1: typed_block_to<uint8_t, false>(dst_bytes, t, rev != 0, nullptr, lds_bytes); break;
    case 2: typed_block_to<uint16_t, false>(dst_bytes, t, rev != 0, nullptr, lds_bytes); break;
    case 4: typed_block_to<uint32_t, false>(dst_bytes, t, rev != 0, nullptr, lds_bytes); break;
    default: typed_block_to<uint64_t, false>(dst_bytes, t, rev != 0, nullptr, lds_bytes); break;
  }
}

// blocks of a Partial source whose members are stored transposed (pack direction only)
// (eight waves per SIMD, i.e. two workgroups per CU: with 64 registers the two-member batches fit without spills)
__global__ __launch_bounds__(ETHA_TRANS_THREADS, 8) void etha_transpose_reduce_kernel(const TransTile* __restrict__ tiles,
                                                                                    const uint64_t* __restrict__ peer_bases) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_bytes[];
  const TransTile t = tiles[blockIdx.x];
  if (!(t.cvt & kTransTyped) || !t.n_peers) return;
  const uint32_t dta = (t.cvt >> 4) & 15u, dtb = t.cvt & 15u;
  switch (dtype_bytes(dta)) {
    case 2: typed_block_to<uint16_t, true>(dtype_bytes(dtb), t, false, peer_bases, lds_bytes); break;
    case 4: typed_block_to<uint32_t, true>(dtype_bytes(dtb), t, false, peer_bases, lds_bytes); break;
    default: typed_block_to<uint64_t, true>(dtype_bytes(dtb), t, false, peer_bases, lds_bytes); break;
  }
}

// =================================================================================================
// Host side: validation and the tile compiler.
// =================================================================================================
// message of the calling thread's last failure; a fixed buffer, so that reporting a failure (out of host memory
// among them) allocates nothing
thread_local char g_err[512] = "";
// An allocation may be opened once per process; several tensors usually share one allocation, so
// mappings are cached per handle and reference-counted.
struct IpcMapping {
  void* base = nullptr;
  int refs = 0;
};
typedef std::array<uint8_t, 64> IpcKey;
std::mutex g_ipc_mutex;
std::map<IpcKey, IpcMapping> g_ipc_open;
std::map<void*, IpcKey> g_ipc_ptrs;  // pointer handed out by etha_ipc_open -> its handle (multimap not needed:
                                     // equal pointers come from equal handles and share the count)
std::map<void*, int> g_ipc_ptr_refs;

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Body of an entry point that builds host-side containers: no C++ exception leaves the library (the ABI is
// plain C); running out of host memory becomes ETHA_ERR_NOMEM.
template <typename F>
int guarded(const char* what, F&& body) {
  try {
    return body();
  } catch (const std::bad_alloc&) {
    return fail(ETHA_ERR_NOMEM, "%s: out of host memory", what);
  } catch (const std::exception& e) {
    return fail(ETHA_ERR_INVALID, "%s: %s", what, e.what());
  } catch (...) {
    return fail(ETHA_ERR_INVALID, "%s: unexpected exception", what);
  }
}

#define HIP_TRY(expr)                                                                      \
  do {                                                                                     \
    hipError_t e_ = (expr);                                                                \
    if (e_ != hipSuccess) return fail(ETHA_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

int dtype_size(uint32_t dt) {
  switch (dt) {
    case ETHA_F16: case ETHA_BF16: case ETHA_B16: case ETHA_I16: return 2;
    case ETHA_F32: case ETHA_B32: case ETHA_I32: return 4;
    case ETHA_F64: case ETHA_B64: case ETHA_I64: return 8;
    case ETHA_B8: case ETHA_I8: case ETHA_U8: case ETHA_BOOL: case ETHA_F8E4M3: case ETHA_F8E5M2: return 1;
    default: return 0;
  }
}
bool is_float(uint32_t dt) { return dt <= ETHA_F64; }                       // the four IEEE-style floats (vector conversions, reductions)
bool is_typed(uint32_t dt) { return dt <= ETHA_F64 || (dt >= ETHA_I8 && dt <= ETHA_F8E5M2); }  // has a value, can be converted
int log2u(uint64_t x) {
  int l = 0;
  while ((1ull << (l + 1)) <= x) l++;
  return l;
}

// reduce_op of a descriptor: a plain ETHA_* op, or ETHA_REDUCE_LEVELS(...) for Partial mesh dims with different ops
int check_reduce_op(uint32_t word, uint32_t n_partials, uint32_t idx) {
  const uint32_t g0 = (word >> 16) & 255u, g1 = (word >> 24) & 255u;
  if (!g0 && !g1) {
    if (word > ETHA_PRODUCT) return fail(ETHA_ERR_INVALID, "chunk %u: unknown reduce_op %u", idx, word);
    return ETHA_OK;
  }
  if ((word & 0xfe00u) || !g0) return fail(ETHA_ERR_INVALID, "chunk %u: malformed reduce_op 0x%x", idx, word);
  for (int l = 0; l < 3; l++)
    if (((word >> (3 * l)) & 7u) > ETHA_PRODUCT) return fail(ETHA_ERR_INVALID, "chunk %u: unknown reduce_op in level %d", idx, l);
  const uint32_t inner = g0 * (g1 ? g1 : 1u);
  if (n_partials == 0 || n_partials % inner != 0)
    return fail(ETHA_ERR_INVALID, "chunk %u: %u Partial members are not a whole number of groups of %u", idx, n_partials, inner);
  return ETHA_OK;
}

struct Region {  // strided region; strides in bytes
  uint64_t base = 0;
  int nd = 0;
  int64_t shape[ETHA_MAX_NDIM];
  int64_t stride[ETHA_MAX_NDIM];
};

// region of the tensor side of a descriptor + byte range check
int tensor_region(const EthaChunkDesc& d, uint32_t idx, uint64_t base_ptr, bool relative, Region* out) {
  const int es = dtype_size(d.tensor_dtype);
  if (es == 0) return fail(ETHA_ERR_INVALID, "chunk %u: unknown tensor_dtype %u", idx, d.tensor_dtype);
  if (d.ndim > ETHA_MAX_NDIM) return fail(ETHA_ERR_INVALID, "chunk %u: ndim %u > %d", idx, d.ndim, ETHA_MAX_NDIM);
  Region r;
  r.nd = (int)d.ndim;
  __int128 off = 0, lo = 0, hi = 0;
  bool empty = false;
  for (int i = 0; i < r.nd; i++) {
    if (d.shape[i] < 0 || d.start[i] < 0)
      return fail(ETHA_ERR_INVALID, "chunk %u: negative shape/start in dim %d", idx, i);
    r.shape[i] = d.shape[i];
    r.stride[i] = d.stride[i] * es;
    off += (__int128)d.start[i] * d.stride[i] * es;
    if (d.shape[i] == 0) empty = true;
    const __int128 ext = (__int128)(d.shape[i] - 1) * d.stride[i] * es;
    if (d.shape[i] > 0) (ext < 0 ? lo : hi) += ext;
  }
  // an empty tensor has no storage and a null data pointer; it also produces no tiles
  if (base_ptr == 0 && !relative && !empty) return fail(ETHA_ERR_INVALID, "chunk %u: null tensor pointer", idx);
  const __int128 first = (__int128)base_ptr + off;
  if (first < 0 || first > (__int128)UINT64_MAX) return fail(ETHA_ERR_INVALID, "chunk %u: address overflow", idx);
  r.base = (uint64_t)first;
  if (!empty && (d.tensor_lo || d.tensor_hi)) {
    if (first + lo < (__int128)d.tensor_lo || first + hi + es > (__int128)d.tensor_hi)
      return fail(ETHA_ERR_INVALID, "chunk %u: tensor region [%llx,%llx) leaves the allowed range [%llx,%llx)", idx,
                  (unsigned long long)(first + lo), (unsigned long long)(first + hi + es),
                  (unsigned long long)d.tensor_lo, (unsigned long long)d.tensor_hi);
  }
  *out = r;
  return ETHA_OK;
}

uint64_t region_numel(const Region& r) {
  uint64_t n = 1;
  for (int i = 0; i < r.nd; i++) n *= (uint64_t)r.shape[i];
  return n;
}

struct Builder {
  std::vector<RunTile> run;
  std::vector<RowTile> row;
  std::vector<TransTile> trans;
  std::vector<uint32_t> run_begin, row_begin, trans_begin;
  std::vector<uint8_t> is_reduce;
  uint64_t payload_bytes = 0;
  uint64_t max_bytes = 0;  // 0: no limit.  Else the tile program may take at most this many bytes (tiles only)
};

constexpr uint64_t kMaxTiles = 0x7fff0000ull / kBlocksPerTile;  // grid.x limit with margin

// Called before tiles are appended: refuses a program that would outgrow the grid limit or the builder's byte
// budget before the host vectors grow, not after.
int room_for(const Builder& b, uint32_t idx, uint64_t more_run, uint64_t more_row, uint64_t more_trans) {
  const uint64_t n_run = b.run.size() + more_run, n_row = b.row.size() + more_row, n_trans = b.trans.size() + more_trans;
#ifdef ETHA_TEST_THROW_AT_TILE
  // test builds only: stands in for a host allocation that fails while a program is being compiled
  if (n_run + n_row + n_trans > (uint64_t)(ETHA_TEST_THROW_AT_TILE)) throw std::bad_alloc();
#endif
  if (n_run + n_row > kMaxTiles || n_trans > kMaxTiles)
    return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: tile program too large (> %llu tiles)", idx, (unsigned long long)kMaxTiles);
  if (b.max_bytes) {
    const uint64_t bytes = n_run * sizeof(RunTile) + n_row * sizeof(RowTile) + n_trans * sizeof(TransTile);
    if (bytes > b.max_bytes)
      return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: the tile program would take more than %llu bytes; this entry point holds at most %llu",
                  idx, (unsigned long long)bytes, (unsigned long long)b.max_bytes);
  }
  return ETHA_OK;
}

struct ReduceSpec {
  uint32_t n_peers = 0, peer_first = 0, op = 0, via = 0;
};

// Compiles one chunk: emits the tiles that move region A (dtype dta) to/from region B (dtype dtb); both
// regions have the same shape.  For reduce chunks A.base is 0 and tile addresses on the a side are offsets
// from the peer bases; `align_bases` then lists the peers' real bases for the alignment bookkeeping.
class PairCompiler {
 public:
  PairCompiler(Builder& bld, uint32_t idx, const Region& A, const Region& B, uint32_t dta, uint32_t dtb,
               const ReduceSpec& red, const std::vector<uint64_t>& align_bases)
      : bld_(bld), idx_(idx), A_(A), B_(B), dta_(dta), dtb_(dtb), esa_(dtype_size(dta)), esb_(dtype_size(dtb)),
        red_(red), align_bases_(align_bases), cvt_(dta != dtb), plain_(dta == dtb && red.n_peers == 0),
        dt_bits_((dta << kMetaDtaShift) | (dtb << kMetaDtbShift)) {}

  int compile() {
    if (A_.nd != B_.nd) return fail(ETHA_ERR_INVALID, "chunk %u: rank mismatch", idx_);
    for (int i = 0; i < A_.nd; i++)
      if (A_.shape[i] != B_.shape[i]) return fail(ETHA_ERR_INVALID, "chunk %u: shape mismatch in dim %d", idx_, i);
    if (cvt_ && !(is_typed(dta_) && is_typed(dtb_)))
      return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: conversion %u -> %u: opaque element types can only be moved, not converted",
                  idx_, dta_, dtb_);
    if (red_.n_peers && !(is_float(dta_) && is_float(dtb_)))
      return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: Partial reduce needs f16/bf16/f32/f64 on both sides", idx_);
    if (region_numel(A_) == 0) return ETHA_OK;
    collapse_dims();
    bool done = false;
    int rc = try_transposing(&done);
    if (rc != ETHA_OK || done) return rc;
    collect_alignment();
    if (!plain_ && (mask_a_ % (uint64_t)esa_ || mask_b_ % (uint64_t)esb_))
      return fail(ETHA_ERR_INVALID, "chunk %u: element address not aligned to its dtype", idx_);
    return plain_ ? compile_byte_move() : compile_typed_move();
  }

 private:
  // 1. drop size-1 dims, 2. merge dims that are contiguous on both sides, 3. split off the innermost
  //    contiguous run (in elements).  Afterwards dims [0, k_) are the outer dims, strides in bytes.
  void collapse_dims() {
    k_ = 0;
    for (int i = 0; i < A_.nd; i++) {
      if (A_.shape[i] == 1) continue;
      if (k_ > 0 && sa_[k_ - 1] == A_.shape[i] * A_.stride[i] && sb_[k_ - 1] == A_.shape[i] * B_.stride[i]) {
        n_[k_ - 1] *= A_.shape[i];
        sa_[k_ - 1] = A_.stride[i];
        sb_[k_ - 1] = B_.stride[i];
      } else {
        n_[k_] = A_.shape[i];
        sa_[k_] = A_.stride[i];
        sb_[k_] = B_.stride[i];
        k_++;
      }
    }
    run_elems_ = 1;
    if (k_ > 0 && sa_[k_ - 1] == esa_ && sb_[k_ - 1] == esb_) {
      run_elems_ = (uint64_t)n_[k_ - 1];
      k_--;
    }
  }

  // Odometer over dims [0, dims) except `skip0` / `skip1`: advances pos and the two byte offsets; false at the end.
  bool next_position(int dims, int64_t* pos, uint64_t* off_a, uint64_t* off_b, int skip0 = -1, int skip1 = -1) const {
    for (int d = dims - 1; d >= 0; d--) {
      if (d == skip0 || d == skip1) continue;
      pos[d]++;
      *off_a += (uint64_t)sa_[d];  // wraps mod 2^64 for negative strides, which is fine
      *off_b += (uint64_t)sb_[d];
      if (pos[d] < n_[d]) return true;
      *off_a -= (uint64_t)(sa_[d] * n_[d]);
      *off_b -= (uint64_t)(sb_[d] * n_[d]);
      pos[d] = 0;
    }
    return false;
  }

  // Transposing chunk: no common contiguous dim, but the a side is contiguous along some other dim j while
  // the b side is contiguous along the innermost one.  Such chunks go through the LDS-staged transposing
  // kernel in blocks of trans_dim_a x trans_dim_b elements; all other dims are unrolled here.
  int try_transposing(bool* done) {
    *done = false;
    // same element type on both sides, or f32 on the a side with f16 / bf16 in the bucket (converted on the way):
    // blocks of the plain transposing kernel.  Every other pair of value types, and Partial sources reduced with one
    // op, take the blocks of the typed kernel (a Partial source with nested levels keeps its row tiles).
    const bool converting = cvt_ && red_.n_peers == 0 && dta_ == ETHA_F32 && (dtb_ == ETHA_F16 || dtb_ == ETHA_BF16);
    const bool typed = !plain_ && !converting && is_typed(dta_) && is_typed(dtb_) && (red_.op >> 16) == 0;
    if (!(run_elems_ == 1 && (plain_ || converting || typed) && k_ >= 2 && sb_[k_ - 1] == esb_ && sa_[k_ - 1] != esa_)) return ETHA_OK;
    int j = -1;
    for (int i = 0; i < k_ - 1; i++)
      if (sa_[i] == esa_ && n_[i] >= 8) j = i;
    const int kk = k_ - 1;
    if (j < 0 || n_[kk] < 8 || (A_.base % (uint64_t)esa_) != 0 || (B_.base % (uint64_t)esb_) != 0) return ETHA_OK;
    for (uint64_t p : align_bases_)
      if (p % (uint64_t)esa_) return ETHA_OK;  // the row tiles report the misaligned member
    for (int i = 0; i < k_; i++)
      if (sa_[i] % esa_ || sb_[i] % esb_) return ETHA_OK;
    int64_t pos[ETHA_MAX_NDIM] = {0};
    uint64_t off_a = 0, off_b = 0;
    // blocks are sized by the element that goes through LDS: the b side's (typed blocks: by the wider side)
    const int64_t kDimJ = typed ? (int64_t)trans_typed_dim((uint32_t)esa_, (uint32_t)esb_) : (int64_t)trans_dim_a((uint32_t)esb_);
    const int64_t kDimK = typed ? kDimJ : (int64_t)trans_dim_b((uint32_t)esb_);
    // the part of the chunk that whole wide blocks cover; blocks of the plain extent (and edge blocks) cover the rest
    const int64_t kP = typed ? 1 : (int64_t)trans_wide((uint32_t)esb_);
    // Partial members of 2-byte elements have a block shape of their own
    const bool red_shape = typed && red_.n_peers && esa_ == 2 && esb_ <= 4 && (dta_ == ETHA_F16 || dta_ == ETHA_BF16) && dtb_ <= ETHA_F32;
    const int64_t wide_dim_j = red_shape ? (int64_t)kRedDimJ2 : converting ? (int64_t)kTransCvtWideJ : kDimJ * kP;
    const int64_t wide_dim_k = red_shape ? (int64_t)kRedDimK2 : converting ? (int64_t)kTransCvtWideK : kDimK * kP;
    const bool has_wide = wide_dim_j != kDimJ || wide_dim_k != kDimK;
    // the region the wide blocks cover ends where blocks of the plain extent can take over
    const auto lcm = [](int64_t x, int64_t y) { int64_t a = x, b = y; while (b) { const int64_t r = a % b; a = b; b = r; } return x / a * y; };
    const int64_t step_j = lcm(wide_dim_j, kDimJ), step_k = lcm(wide_dim_k, kDimK);
    const int64_t wide_j = has_wide ? n_[j] / step_j * step_j : 0, wide_k = has_wide ? n_[kk] / step_k * step_k : 0;
    const bool wide = wide_j > 0 && wide_k > 0;
    do {
      // Launch order.  Blocks are grouped into super-blocks of S x S blocks that are emitted together: blocks
      // that are neighbours along j read neighbouring pieces of the same source rows, neighbours along k write
      // neighbouring pieces of the same destination rows, so running them at the same time keeps DRAM pages
      // open on both sides.  Super-blocks follow diagonals of their grid: row-major order would make everything
      // in flight read (or write) one narrow column stripe of rows that lie a power of two apart, i.e. the same
      // few memory channels.
      auto emit = [&](int64_t dim_j, int64_t dim_k, int64_t j_end, int64_t k_end, int64_t skip_j, int64_t skip_k) -> int {
        // blocks of dim_j x dim_k over [0, j_end) x [0, k_end), except those inside [0, skip_j) x [0, skip_k)
        const int64_t S = ETHA_TRANS_SUPER;
        const int64_t nbj = (j_end + dim_j - 1) / dim_j, nbk = (k_end + dim_k - 1) / dim_k;
        const int64_t nsj = (nbj + S - 1) / S, nsk = (nbk + S - 1) / S;
        const int rc_room = room_for(bld_, idx_, 0, 0, (uint64_t)nbj * (uint64_t)nbk);
        if (rc_room != ETHA_OK) return rc_room;
        for (int64_t d = 0; d < nsk; d++)
          for (int64_t sj = 0; sj < nsj; sj++)
            for (int64_t ij = 0; ij < S; ij++)
              for (int64_t ik = 0; ik < S; ik++) {
                const int64_t bj = sj * S + ij, bk = ((sj + d) % nsk) * S + ik;
                if (bj >= nbj || bk >= nbk) continue;
                const int64_t j0 = bj * dim_j, k0 = bk * dim_k;
                if (j0 < skip_j && k0 < skip_k) continue;
                TransTile t;
                memset(&t, 0, sizeof(t));
                t.a = A_.base + off_a + (uint64_t)(j0 * sa_[j]) + (uint64_t)(k0 * sa_[kk]);
                t.b = B_.base + off_b + (uint64_t)(j0 * sb_[j]) + (uint64_t)(k0 * sb_[kk]);
                t.a_pitch = sa_[kk];
                t.b_pitch = sb_[j];
                t.nj = (uint32_t)(j_end - j0 < dim_j ? j_end - j0 : dim_j);
                t.nk = (uint32_t)(k_end - k0 < dim_k ? k_end - k0 : dim_k);
                t.es_log2 = (uint32_t)log2u((uint64_t)esb_);
                t.cvt = converting ? (dta_ << 4) | dtb_ : typed ? ((dta_ << 4) | dtb_ | kTransTyped) : 0u;
                t.peer_first = red_.peer_first;
                t.n_peers = red_.n_peers;
                t.reduce_op = red_.op;
                t.via = red_.via;
                bld_.trans.push_back(t);
              }
        return ETHA_OK;
      };
      int rc = wide ? emit(wide_dim_j, wide_dim_k, wide_j, wide_k, 0, 0) : ETHA_OK;
      if (rc == ETHA_OK && (!wide || wide_j < n_[j] || wide_k < n_[kk]))
        rc = emit(kDimJ, kDimK, n_[j], n_[kk], wide ? wide_j : 0, wide ? wide_k : 0);
      if (rc != ETHA_OK) return rc;
    } while (next_position(k_, pos, &off_a, &off_b, j, kk));
    *done = true;
    return ETHA_OK;
  }

  // OR of every row start (base and outer strides) per side.  Lengths decide unit sizes, not addresses: the
  // kernel's accesses are legal at any (element-aligned) address, so a misaligned side only sets a meta flag.
  void collect_alignment() {
    mask_a_ = red_.n_peers ? 0 : A_.base;
    mask_b_ = B_.base;
    for (uint64_t p : align_bases_) mask_a_ |= p + A_.base;  // reduce: A_.base is an offset from each peer base
    for (int i = 0; i < k_; i++) {
      mask_a_ |= (uint64_t)(sa_[i] < 0 ? -sa_[i] : sa_[i]);
      mask_b_ |= (uint64_t)(sb_[i] < 0 ? -sb_[i] : sb_[i]);
    }
  }
  uint32_t skew_bits(int ua_log2, int ub_log2) const {
    return ((mask_a_ & ((1ull << ua_log2) - 1)) ? kMetaSkew : 0u) | ((mask_b_ & ((1ull << ub_log2) - 1)) ? kMetaSkewB : 0u);
  }
  static uint32_t unit_bits(int ua_log2, int ub_log2) {
    return ((uint32_t)ua_log2 << kMetaUaShift) | ((uint32_t)ub_log2 << kMetaUbShift);
  }
  static int widest_unit_log2(uint64_t bytes, int cap_log2) {  // widest power of two (<= 2^cap) dividing `bytes`
    int v = cap_log2;
    while (v > 0 && (bytes & ((1ull << v) - 1))) v--;
    return v;
  }

  // Byte moves (same dtype, no reduce): the widest power of two <= 16 bytes that divides the run.
  int compile_byte_move() {
    const uint64_t run_bytes = run_elems_ * (uint64_t)esa_;
    // Skewed byte moves: the two sides disagree on their position inside a 16-byte vector (typically a chunk
    // that follows an odd-sized one in an un-padded bucket).  Very long runs are peeled per run so that the
    // b side is 16-byte aligned: a head and a tail of < 16 bytes go through narrow tiles, the body moves in
    // 16-byte units whose a-side access is unaligned.  Peeling costs three tile sets per run, so it only
    // pays for runs of many tiles (measured: +5 % from 256 KiB up, 20x slower than the row split below at
    // 512-byte runs); shorter runs take the row split, unaligned on both sides.
    if (((mask_a_ | mask_b_) & 15) && run_bytes >= (uint64_t)ETHA_SKEW_PEEL_MIN_BYTES) return peel_runs(run_bytes);
    const int v = widest_unit_log2(run_bytes, 4);
    if (v == 4 || run_bytes < 32)
      return emit(A_.base, B_.base, run_bytes >> v, 1ull << v, 1ull << v, dt_bits_ | unit_bits(v, v) | skew_bits(v, v));
    // Rows that are not a whole number of 16-byte units: a body of 16-byte units and a remainder of < 16
    // bytes in narrow units, both ordinary, densely packed tile sets over the same rows.
    const uint64_t body_units = run_bytes / 16, rem_bytes = run_bytes % 16;
    int rc = emit(A_.base, B_.base, body_units, 16, 16, dt_bits_ | unit_bits(4, 4) | skew_bits(4, 4));
    if (rc != ETHA_OK) return rc;
    const int r = widest_unit_log2(rem_bytes, 3);
    // the remainder starts body_units * 16 bytes into each row: same position modulo 16 as the row start
    return emit(A_.base + body_units * 16, B_.base + body_units * 16, rem_bytes >> r, 1ull << r, 1ull << r,
                dt_bits_ | unit_bits(r, r) | skew_bits(r, r));
  }

  int peel_runs(uint64_t run_bytes) {
    const uint32_t body_meta = dt_bits_ | unit_bits(4, 4) | kMetaSkew;
    auto narrow = [&](uint64_t a, uint64_t b, uint64_t bytes) {  // bytes < 16
      if (!bytes) return;
      const int v = widest_unit_log2(bytes, 3);
      const uint64_t low = (1ull << v) - 1;
      RunTile t;
      t.a = a;
      t.b = b;
      t.n = (uint32_t)(bytes >> v);
      t.meta = dt_bits_ | unit_bits(v, v) | ((a & low) ? kMetaSkew : 0u) | ((b & low) ? kMetaSkewB : 0u);
      bld_.run.push_back(t);
    };
    int64_t pos[ETHA_MAX_NDIM] = {0};
    uint64_t off_a = 0, off_b = 0;
    do {
      const uint64_t a0 = A_.base + off_a, b0 = B_.base + off_b;
      const uint64_t head = (16 - (b0 & 15)) & 15;
      const uint64_t body_units = (run_bytes - head) / 16;
      const uint64_t tail = run_bytes - head - body_units * 16;
      const int rc = room_for(bld_, idx_, 2 + (body_units + kTileThreads - 1) / kTileThreads, 0, 0);
      if (rc != ETHA_OK) return rc;
      narrow(a0, b0, head);
      for (uint64_t q = 0; q < body_units; q += kTileThreads) {
        RunTile t;
        t.a = a0 + head + q * 16;
        t.b = b0 + head + q * 16;
        t.n = (uint32_t)(body_units - q < kTileThreads ? body_units - q : kTileThreads);
        t.meta = body_meta;
        bld_.run.push_back(t);
      }
      narrow(a0 + head + body_units * 16, b0 + head + body_units * 16, tail);
    } while (next_position(k_, pos, &off_a, &off_b));
    return ETHA_OK;
  }

  // Converting and reducing moves: a row is cut into whole vectors of `epv` elements (the narrow side moves up to 16
  // bytes; converting moves may use two accesses on the wide side, reductions one) and a remainder, which moves in
  // narrower vectors of 4 or 2 elements before single elements are used: each width is an ordinary, densely
  // packed tile set over the same rows.
  int compile_typed_move() {
    if (!(is_float(dta_) && is_float(dtb_)))  // an integer, bool or 8-bit float side: element by element
      return emit(A_.base, B_.base, run_elems_, (uint64_t)esa_, (uint64_t)esb_,
                  dt_bits_ | kMetaCvt | kMetaGeneric | unit_bits(log2u((uint64_t)esa_), log2u((uint64_t)esb_)));
    const int epv = red_.n_peers ? 16 / (esa_ > esb_ ? esa_ : esb_) : cvt_elems_per_unit(esa_, esb_);
    uint64_t done = 0, left = run_elems_;
    int v = epv;  // elements per unit: a power of two
    while (left) {
      while ((uint64_t)v > left) v >>= 1;
      const uint64_t units = left / (uint64_t)v, off_a = done * (uint64_t)esa_, off_b = done * (uint64_t)esb_;
      const int va = log2u((uint64_t)(v * esa_)), vb = log2u((uint64_t)(v * esb_));
      // single elements are always aligned (checked by the caller); wider units may sit at any element boundary
      const uint32_t skew = v == 1 ? 0u
                                   : ((((mask_a_ | off_a) & ((1ull << va) - 1)) ? kMetaSkew : 0u) |
                                      (((mask_b_ | off_b) & ((1ull << vb) - 1)) ? kMetaSkewB : 0u));
      const uint32_t meta = dt_bits_ | kMetaCvt | (v == epv && epv > 1 ? kMetaVec : 0u) |
                            ((uint32_t)log2u((uint64_t)v) << kMetaElemsShift) | unit_bits(va, vb) | skew;
      const int rc = emit(A_.base + off_a, B_.base + off_b, units, 1ull << va, 1ull << vb, meta);
      if (rc != ETHA_OK) return rc;
      done += units * (uint64_t)v;
      left -= units * (uint64_t)v;
    }
    return ETHA_OK;
  }

  // Tiles for rows of `run_units` units starting at base_a / base_b.  Long or tile-multiple rows (and
  // single runs) become run tiles; other shapes become row tiles over the innermost remaining dim; dims
  // further out are unrolled here.  Reduce chunks always use row tiles (they carry the peer list).
  int emit(uint64_t base_a, uint64_t base_b, uint64_t run_units, uint64_t ua, uint64_t ub, uint32_t meta) {
    const bool use_rows = red_.n_peers != 0 || (k_ > 0 && run_units % kTileThreads != 0 && run_units < 4 * kTileThreads);
    if (run_units > 0xffffffffull && use_rows && k_ > 0)
      return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: row longer than 2^32 units", idx_);
    const int outer = use_rows && k_ > 0 ? k_ - 1 : k_;  // dims unrolled on the host
    int64_t pos[ETHA_MAX_NDIM] = {0};
    uint64_t off_a = 0, off_b = 0;
    do {
      const uint64_t a0 = base_a + off_a, b0 = base_b + off_b;
      if (!use_rows) {
        const int rc = room_for(bld_, idx_, (run_units + kTileThreads - 1) / kTileThreads, 0, 0);
        if (rc != ETHA_OK) return rc;
        for (uint64_t q = 0; q < run_units; q += kTileThreads) {
          RunTile t;
          t.a = a0 + q * ua;
          t.b = b0 + q * ub;
          t.n = (uint32_t)(run_units - q < kTileThreads ? run_units - q : kTileThreads);
          t.meta = meta;
          bld_.run.push_back(t);
        }
      } else {
        const uint64_t rows = k_ > 0 ? (uint64_t)n_[k_ - 1] : 1;
        const int64_t pa = k_ > 0 ? sa_[k_ - 1] : 0, pb = k_ > 0 ? sb_[k_ - 1] : 0;
        const uint64_t total = rows * run_units;
        const uint64_t step = kTileThreads;
        const int rc = room_for(bld_, idx_, 0, (total + step - 1) / step, 0);
        if (rc != ETHA_OK) return rc;
        for (uint64_t q = 0; q < total; q += step) {
          RowTile t;
          memset(&t, 0, sizeof(t));
          const uint64_t left = total - q;
          t.n = (uint32_t)(left < step ? left : step);
          t.meta = meta;
          if (rows == 1) {  // one (possibly very long) run: address the tile directly
            t.a = a0 + q * ua;
            t.b = b0 + q * ub;
            t.run = kTileThreads;
            t.c0 = 0;
          } else {
            const uint64_t r0 = q / run_units, c0 = q % run_units;
            t.a = a0 + (uint64_t)((int64_t)r0 * pa);
            t.b = b0 + (uint64_t)((int64_t)r0 * pb);
            t.a_pitch = pa;
            t.b_pitch = pb;
            t.run = (uint32_t)run_units;
            t.c0 = (uint32_t)c0;
          }
          t.peer_first = red_.peer_first;
          t.n_peers = red_.n_peers;
          t.reduce_op = red_.op;
          t.via = red_.via;
          bld_.row.push_back(t);
        }
      }
    } while (next_position(outer, pos, &off_a, &off_b));
    return ETHA_OK;
  }

  Builder& bld_;
  const uint32_t idx_;
  const Region& A_;
  const Region& B_;
  const uint32_t dta_, dtb_;
  const int esa_, esb_;
  const ReduceSpec& red_;
  const std::vector<uint64_t>& align_bases_;
  const bool cvt_, plain_;
  const uint32_t dt_bits_;
  int k_ = 0;                                              // outer dims left after collapsing
  int64_t n_[ETHA_MAX_NDIM], sa_[ETHA_MAX_NDIM], sb_[ETHA_MAX_NDIM];  // their extents and byte strides
  uint64_t run_elems_ = 1;                                 // innermost contiguous run, in elements
  uint64_t mask_a_ = 0, mask_b_ = 0;
};

int compile_pair(Builder& bld, uint32_t idx, const Region& A, const Region& B, uint32_t dta, uint32_t dtb,
                 const ReduceSpec& red, const std::vector<uint64_t>& align_bases) {
  return PairCompiler(bld, idx, A, B, dta, dtb, red, align_bases).compile();
}

}  // namespace

struct EthaTable {
  int kind = 0;  // 0 = pack/unpack table, 1 = self-copy table
  std::vector<RunTile> h_run;
  std::vector<RowTile> h_row;
  std::vector<TransTile> h_trans;
  std::vector<uint32_t> run_begin, row_begin, trans_begin;
  std::vector<uint32_t> typed_begin;    // number of typed transposing tiles before chunk i's
  std::vector<uint32_t> reduce_prefix;  // number of reduce chunks before chunk i
  std::vector<uint64_t> h_peers;
  RunTile* d_run = nullptr;
  RowTile* d_row = nullptr;
  TransTile* d_trans = nullptr;
  uint32_t trans_lds = 0;  // LDS bytes the transposing tiles need (largest over their element sizes)
  uint64_t* d_peers = nullptr;
  uint32_t n_chunks = 0;
  uint64_t payload_bytes = 0;
  uint64_t device_bytes = 0;
  bool uploaded = false;
  // identity for schedules that hold launches of this table: `serial` is unique per table ever created in the
  // process, `version` changes when the launches of a chunk range change (a range gains a write-ordered copy)
  uint64_t serial = 0;
  uint32_t version = 0;
  // write-ordered copies of the tiles of ranges that are always launched as one unit
  struct Ordered {
    std::vector<RunTile> h_run;
    std::vector<RowTile> h_row;      // plain row tiles, then the gather tiles
    uint32_t n_plain_rows = 0;
    std::vector<uint64_t> h_gather;  // piece addresses of the gather tiles
    RunTile* d_run = nullptr;
    RowTile* d_row = nullptr;
    uint64_t* d_gather = nullptr;
  };
  std::map<std::pair<uint32_t, uint32_t>, Ordered> ordered;
};

namespace {

// LDS bytes a transposing tile needs
uint32_t trans_tile_lds(const TransTile& tt) {
  if (tt.cvt & kTransTyped) return trans_typed_lds_bytes((uint32_t)dtype_size((tt.cvt >> 4) & 15u), (uint32_t)dtype_size(tt.cvt & 15u));
  return trans_lds_bytes(1u << tt.es_log2);
}

// tables that exist, by address -> serial; a schedule checks its tables against this before it launches
std::mutex g_tables_mutex;
std::map<const EthaTable*, uint64_t> g_live_tables;
uint64_t g_next_table_serial = 1;

int upload_table(EthaTable* t) {
  if (!t->h_run.empty()) {
    const size_t bytes = t->h_run.size() * sizeof(RunTile);
    HIP_TRY(hipMalloc(&t->d_run, bytes));
    HIP_TRY(hipMemcpy(t->d_run, t->h_run.data(), bytes, hipMemcpyHostToDevice));
    t->device_bytes += bytes;
  }
  if (!t->h_row.empty()) {
    const size_t bytes = t->h_row.size() * sizeof(RowTile);
    HIP_TRY(hipMalloc(&t->d_row, bytes));
    HIP_TRY(hipMemcpy(t->d_row, t->h_row.data(), bytes, hipMemcpyHostToDevice));
    t->device_bytes += bytes;
  }
  if (!t->h_trans.empty()) {
    const size_t bytes = t->h_trans.size() * sizeof(TransTile);
    HIP_TRY(hipMalloc(&t->d_trans, bytes));
    HIP_TRY(hipMemcpy(t->d_trans, t->h_trans.data(), bytes, hipMemcpyHostToDevice));
    t->device_bytes += bytes;
  }
  if (!t->h_peers.empty()) {
    const size_t bytes = t->h_peers.size() * sizeof(uint64_t);
    HIP_TRY(hipMalloc(&t->d_peers, bytes));
    HIP_TRY(hipMemcpy(t->d_peers, t->h_peers.data(), bytes, hipMemcpyHostToDevice));
    t->device_bytes += bytes;
  }
  t->uploaded = true;
  return ETHA_OK;
}

void free_table(EthaTable* t) {
  if (!t) return;
  {
    std::lock_guard<std::mutex> lock(g_tables_mutex);
    g_live_tables.erase(t);
  }
  if (t->d_run) (void)hipFree(t->d_run);
  if (t->d_row) (void)hipFree(t->d_row);
  if (t->d_peers) (void)hipFree(t->d_peers);
  if (t->d_trans) (void)hipFree(t->d_trans);
  for (auto& kv : t->ordered) {
    if (kv.second.d_run) (void)hipFree(kv.second.d_run);
    if (kv.second.d_row) (void)hipFree(kv.second.d_row);
    if (kv.second.d_gather) (void)hipFree(kv.second.d_gather);
  }
  delete t;
}

// Takes ownership of t: on any failure (an exception included) the table is freed.
int finish_table(Builder& bld, EthaTable* t, const uint64_t* partial_ptrs, uint32_t n_partial_ptrs, int upload, EthaTable** out) {
  try {
    if (partial_ptrs && n_partial_ptrs) t->h_peers.assign(partial_ptrs, partial_ptrs + n_partial_ptrs);
    t->h_run.swap(bld.run);
    t->h_row.swap(bld.row);
    t->h_trans.swap(bld.trans);
    t->run_begin.swap(bld.run_begin);
    t->row_begin.swap(bld.row_begin);
    t->trans_begin.swap(bld.trans_begin);
    for (const TransTile& tt : t->h_trans)
      if (trans_tile_lds(tt) > t->trans_lds) t->trans_lds = trans_tile_lds(tt);
    t->typed_begin.assign(t->n_chunks + 1, 0);
    for (uint32_t i = 0; i < t->n_chunks; i++) {
      uint32_t typed = 0;
      for (uint32_t k = t->trans_begin[i]; k < t->trans_begin[i + 1]; k++) typed += (t->h_trans[k].cvt & kTransTyped) ? 1u : 0u;
      t->typed_begin[i + 1] = t->typed_begin[i] + typed;
    }
    t->reduce_prefix.assign(t->n_chunks + 1, 0);
    for (uint32_t i = 0; i < t->n_chunks; i++) t->reduce_prefix[i + 1] = t->reduce_prefix[i] + bld.is_reduce[i];
    t->payload_bytes = bld.payload_bytes;
    if (upload) {
      const int rc = upload_table(t);
      if (rc != ETHA_OK) {
        free_table(t);
        return rc;
      }
    }
    std::lock_guard<std::mutex> lock(g_tables_mutex);
    t->serial = g_next_table_serial++;
    g_live_tables[t] = t->serial;
  } catch (...) {
    free_table(t);
    throw;
  }
  *out = t;
  return ETHA_OK;
}

int check_range(const EthaTable* t, uint32_t first, uint32_t count, int kind) {
  if (!t) return fail(ETHA_ERR_INVALID, "null table");
  if (t->kind != kind) return fail(ETHA_ERR_INVALID, "wrong table kind for this entry point");
  if ((uint64_t)first + count > t->n_chunks)
    return fail(ETHA_ERR_INVALID, "chunk range [%u,%u) exceeds table of %u chunks", first, first + count, t->n_chunks);
  if (!t->uploaded) return fail(ETHA_ERR_INVALID, "table was created without upload; it cannot be launched");
  return ETHA_OK;
}

// Launch with or without ordering against the launches already on the stream.  An ordinary launch waits
// for every earlier packet of its queue (that is how a stream stays in order).  ETHA_LAUNCH_UNORDERED
// clears that wait for this one dispatch: the kernel may start while earlier launches are still running,
// which removes the drain/ramp bubble between launches that do not depend on each other.  The next
// ordinary launch on the stream again waits for everything before it, unordered launches included.
std::atomic<uint64_t> g_kernel_launches{0};

template <typename... Args, typename F>
void launch_kernel(F kernel, dim3 grid, dim3 block, size_t lds, void* stream, uint32_t flags, Args... args) {
  g_kernel_launches.fetch_add(1, std::memory_order_relaxed);
  if (flags & ETHA_LAUNCH_UNORDERED)
    hipExtLaunchKernelGGL(kernel, grid, block, (uint32_t)lds, (hipStream_t)stream, nullptr, nullptr, hipExtAnyOrderLaunch,
                          args...);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds, (hipStream_t)stream, args...);
}

// One kernel launch with everything resolved: which kernel, its grid and its arguments.  Every entry point
// first plans its launches into a list of these and then issues the list; a schedule (etha_schedule_create)
// keeps such lists, so that re-issuing a whole transfer is a loop over ready-made launches.
enum : uint32_t { kKernelTile = 0, kKernelTile2D, kKernelGather, kKernelMixed, kKernelTrans, kKernelTrans2D, kKernelReduce,
                  kKernelTransTyped, kKernelTransReduce };
const char* const kKernelNames[] = {"etha_tile_kernel", "etha_tile_kernel_2d", "etha_gather_kernel", "etha_unpack_mixed_kernel",
                                    "etha_transpose_kernel", "etha_transpose_kernel_2d", "etha_reduce_kernel",
                                    "etha_transpose_typed_kernel", "etha_transpose_reduce_kernel"};

struct PreparedLaunch {
  uint32_t kernel;  // kKernel*
  uint32_t rev;     // direction of the tile and transposing kernels (unpack = 1)
  uint32_t flags;   // ETHA_LAUNCH_UNORDERED or 0
  uint32_t gx, gy, block, lds;
  union Args {
    struct {  // kKernelTile, kKernelMixed
      const RunTile* run;
      const RowTile* row;
      const uint64_t* gather;
      uint32_t n_run, n_plain, n_gather;
    } tile;
    struct {  // kKernelTrans, kKernelTransTyped
      const TransTile* tiles;
      const uint64_t* peers;
    } trans;
    struct {
      const RowTile* row;
      const uint64_t* peers;
    } reduce;
    Args2D a2d;     // kKernelTile2D, kKernelGather
    TransArgs t2d;  // kKernelTrans2D
  } u;
};

PreparedLaunch new_launch(uint32_t kernel, bool rev, uint32_t flags, uint32_t gx, uint32_t gy, uint32_t block, uint32_t lds) {
  PreparedLaunch p;
  memset(&p, 0, sizeof(p));
  p.kernel = kernel;
  p.rev = rev ? 1u : 0u;
  p.flags = flags;
  p.gx = gx;
  p.gy = gy;
  p.block = block;
  p.lds = lds;
  return p;
}

void issue_one(const PreparedLaunch& p, void* stream, uint32_t flags) {
  const dim3 grid(p.gx, p.gy), block(p.block);
  switch (p.kernel) {
    case kKernelTile:
      if (p.rev)
        launch_kernel(etha_tile_kernel<true>, grid, block, 0, stream, flags, p.u.tile.run, p.u.tile.n_run, p.u.tile.row, p.u.tile.gather);
      else
        launch_kernel(etha_tile_kernel<false>, grid, block, 0, stream, flags, p.u.tile.run, p.u.tile.n_run, p.u.tile.row, p.u.tile.gather);
      break;
    case kKernelTile2D:
      if (p.rev)
        launch_kernel(etha_tile_kernel_2d<true>, grid, block, 0, stream, flags, p.u.a2d);
      else
        launch_kernel(etha_tile_kernel_2d<false>, grid, block, 0, stream, flags, p.u.a2d);
      break;
    case kKernelGather:
      launch_kernel(etha_gather_kernel, grid, block, 0, stream, flags, p.u.a2d);
      break;
    case kKernelMixed:
      launch_kernel(etha_unpack_mixed_kernel, grid, block, 0, stream, flags, p.u.tile.run, p.u.tile.row, p.u.tile.gather,
                    p.u.tile.n_run, p.u.tile.n_plain, p.u.tile.n_gather);
      break;
    case kKernelTrans:
      if (p.rev)
        launch_kernel(etha_transpose_kernel<true>, grid, block, p.lds, stream, flags, p.u.trans.tiles);
      else
        launch_kernel(etha_transpose_kernel<false>, grid, block, p.lds, stream, flags, p.u.trans.tiles);
      break;
    case kKernelTrans2D:
      if (p.rev)
        launch_kernel(etha_transpose_kernel_2d<true>, grid, block, p.lds, stream, flags, p.u.t2d);
      else
        launch_kernel(etha_transpose_kernel_2d<false>, grid, block, p.lds, stream, flags, p.u.t2d);
      break;
    case kKernelTransTyped:
      launch_kernel(etha_transpose_typed_kernel, grid, block, p.lds, stream, flags, p.u.trans.tiles, p.rev);
      break;
    case kKernelTransReduce:
      launch_kernel(etha_transpose_reduce_kernel, grid, block, p.lds, stream, flags, p.u.trans.tiles, p.u.trans.peers);
      break;
    default:
      launch_kernel(etha_reduce_kernel, grid, block, 0, stream, flags, p.u.reduce.row, p.u.reduce.peers);
      break;
  }
}

// Issues the launches in list order; each one is checked, so that a failure names the launch it belongs to.
// A stream under capture records its kernels as a chain: the unordered flag has no meaning there and is dropped.
int issue_all(const PreparedLaunch* list, size_t n, void* stream) {
  bool capturing = false;
  for (size_t i = 0; i < n; i++)
    if (list[i].flags & ETHA_LAUNCH_UNORDERED) {
      hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
      capturing = hipStreamIsCapturing((hipStream_t)stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone;
      break;
    }
  for (size_t i = 0; i < n; i++) {
    issue_one(list[i], stream, capturing ? 0u : list[i].flags);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess)
      return fail(ETHA_ERR_HIP, "launch %zu of %zu (%s, grid %u x %u): %s", i + 1, n, kKernelNames[list[i].kernel], list[i].gx,
                  list[i].gy, hipGetErrorString(e));
  }
  return ETHA_OK;
}

typedef std::vector<PreparedLaunch> LaunchList;

// the plain (run and row) tiles of a chunk range, as the tile kernels take them
Seg2D tile_range(const EthaTable* t, uint32_t first, uint32_t count, bool rev) {
  const uint32_t r0 = t->run_begin[first], w0 = t->row_begin[first];
  Seg2D g{t->d_run + r0, t->d_row + w0, nullptr, t->run_begin[first + count] - r0, 0};
  g.n_tiles = g.n_run + (t->row_begin[first + count] - w0);
  if (rev == (t->kind == 0)) {  // the direction that writes the a side (unpack) / b side (self-copy) of an ordered range
    auto it = t->ordered.find(std::make_pair(first, count));
    if (it != t->ordered.end()) {
      g.run = it->second.d_run;
      g.row = it->second.d_row;
      g.gather = it->second.d_gather;
      g.n_run = (uint32_t)it->second.h_run.size();
      g.n_tiles = g.n_run + it->second.n_plain_rows;  // chunks covered by gather tiles have no plain tiles here
    }
  }
  return g;
}

// the gather tiles of an unpack range that has a write-ordered copy (n_tiles == 0: none)
Seg2D gather_range(const EthaTable* t, uint32_t first, uint32_t count, bool rev) {
  Seg2D g{nullptr, nullptr, nullptr, 0, 0};
  if (!rev || t->kind != 0) return g;
  auto it = t->ordered.find(std::make_pair(first, count));
  if (it == t->ordered.end()) return g;
  g.row = it->second.d_row + it->second.n_plain_rows;
  g.gather = it->second.d_gather;
  g.n_tiles = (uint32_t)it->second.h_row.size() - it->second.n_plain_rows;
  return g;
}

// workgroups of a gather launch over `tiles` tiles: 8 tiles x 16 pieces per 128 workgroups
uint32_t gather_grid(uint32_t tiles) { return ((tiles + 7u) / 8u) * 128u; }

void plan_gather(const Seg2D* segs, uint32_t n, uint32_t top, uint32_t flags, LaunchList& out) {
  PreparedLaunch p = new_launch(kKernelGather, true, flags, gather_grid(top), n, kBlockThreads, 0);
  for (uint32_t k = 0; k < n; k++) p.u.a2d.seg[k] = segs[k];
  out.push_back(p);
}

void plan_plain(const Seg2D& g, bool rev, uint32_t flags, LaunchList& out) {
  PreparedLaunch p = new_launch(kKernelTile, rev, flags, g.n_tiles * kBlocksPerTile, 1, kBlockThreads, 0);
  p.u.tile.run = g.run;
  p.u.tile.row = g.row;
  p.u.tile.gather = g.gather;
  p.u.tile.n_run = g.n_run;
  out.push_back(p);
}

void plan_trans(const TransTile* tiles, uint32_t n, bool rev, uint32_t lds, uint32_t flags, LaunchList& out) {
  PreparedLaunch p = new_launch(kKernelTrans, rev, flags, n, 1, kTransThreads, lds);
  p.u.trans.tiles = tiles;
  out.push_back(p);
}

// One chunk range as the single-range entry points run it: the transposing tiles in their kernel, then the
// plain tiles - and, for an unpack range with a write-ordered copy, its gather tiles in the same launch.
// The typed transposing tiles of a chunk range.  Plain and typed tiles share one list in chunk order; a range that
// holds both is walked by both kernels, each leaving the other's blocks alone.
bool plan_typed(const EthaTable* t, uint32_t first, uint32_t count, bool rev, uint32_t flags, LaunchList& out) {
  const uint32_t x0 = t->trans_begin[first], n_trans = t->trans_begin[first + count] - x0;
  if (t->typed_begin[first + count] == t->typed_begin[first]) return false;
  // a chunk range is all Partial chunks or none (the entry points check): its typed tiles are all of one kind
  const bool reduce = t->reduce_prefix[first + count] != t->reduce_prefix[first];
  PreparedLaunch p = new_launch(reduce ? kKernelTransReduce : kKernelTransTyped, rev, flags, n_trans, 1, kTransThreads, t->trans_lds);
  p.u.trans.tiles = t->d_trans + x0;
  p.u.trans.peers = t->d_peers;
  out.push_back(p);
  return true;
}
uint32_t plain_trans_tiles(const EthaTable* t, uint32_t first, uint32_t count) {  // 0: none of the range's tiles is a plain one
  const uint32_t n_trans = t->trans_begin[first + count] - t->trans_begin[first];
  return n_trans - (t->typed_begin[first + count] - t->typed_begin[first]) ? n_trans : 0u;
}

void plan_tiles(const EthaTable* t, uint32_t first, uint32_t count, bool rev, uint32_t flags, LaunchList& out) {
  const uint32_t x0 = t->trans_begin[first], n_trans = plain_trans_tiles(t, first, count);
  if (n_trans) {
    plan_trans(t->d_trans + x0, n_trans, rev, t->trans_lds, flags, out);
    flags |= ETHA_LAUNCH_UNORDERED;  // the kernels of one call touch different chunks
  }
  if (plan_typed(t, first, count, rev, flags, out)) flags |= ETHA_LAUNCH_UNORDERED;
  const Seg2D g = tile_range(t, first, count, rev);
  const Seg2D gathered = gather_range(t, first, count, rev);
  if (g.n_tiles && gathered.n_tiles) {  // the gather tiles follow the plain row tiles in the ordered copy
    const uint32_t groups = ((g.n_tiles * kBlocksPerTile + 127u) & ~127u) + gather_grid(gathered.n_tiles);
    PreparedLaunch p = new_launch(kKernelMixed, true, flags, groups, 1, kBlockThreads, 0);
    p.u.tile.run = g.run;
    p.u.tile.row = g.row;
    p.u.tile.gather = g.gather;
    p.u.tile.n_run = g.n_run;
    p.u.tile.n_plain = g.n_tiles;
    p.u.tile.n_gather = gathered.n_tiles;
    out.push_back(p);
  } else if (g.n_tiles) {
    plan_plain(g, rev, flags, out);
  } else if (gathered.n_tiles) {
    plan_gather(&gathered, 1, gathered.n_tiles, flags, out);
  }
}

void plan_reduce(const EthaTable* t, uint32_t first, uint32_t count, uint32_t flags, LaunchList& out) {
  if (plan_typed(t, first, count, false, flags, out)) flags |= ETHA_LAUNCH_UNORDERED;  // members stored transposed
  const uint32_t w0 = t->row_begin[first], w1 = t->row_begin[first + count];
  if (w1 == w0) return;
  PreparedLaunch p = new_launch(kKernelReduce, false, flags, (w1 - w0) * kBlocksPerTile, 1, kBlockThreads, 0);
  p.u.reduce.row = t->d_row + w0;
  p.u.reduce.peers = t->d_peers;
  out.push_back(p);
}

// Segments of one direction, largest first: those of (nearly) the same size share a launch.  A workgroup that a
// shorter segment leaves unused is not free - with no limit on them the config-2 step took 6.0 instead of 4.9 ms -
// while a launch of its own costs about 1.8 us: a segment joins the open launch only while the unused
// workgroups it adds stay below a few thousand.  Equal-sized buckets, the usual case, add none.
constexpr uint64_t kJoinMaxIdleTiles = 6000 / kBlocksPerTile;

template <typename SEG, typename COUNT, typename LAUNCH>
void plan_neighbours(std::vector<SEG>& segs, uint64_t max_idle, COUNT count_of, LAUNCH launch, uint32_t& flags) {
  std::stable_sort(segs.begin(), segs.end(), [&](const SEG& x, const SEG& y) { return count_of(x) > count_of(y); });
  size_t i = 0;
  while (i < segs.size()) {
    uint64_t top = count_of(segs[i]), sum = top;
    size_t j = i + 1;
    while (j < segs.size() && j - i < ETHA_MAX_SEGMENTS) {
      const uint64_t n = count_of(segs[j]), new_top = n > top ? n : top;
      const uint64_t idle_now = top * (j - i) - sum, idle_then = new_top * (j - i + 1) - (sum + n);
      if (idle_then - idle_now > max_idle) break;
      top = new_top;
      sum += n;
      j++;
    }
    launch(i, j, (uint32_t)top, flags);
    flags |= ETHA_LAUNCH_UNORDERED;  // what follows belongs to the same set of independent segments
    i = j;
  }
}

void plan_group(std::vector<Seg2D>& segs, bool rev, uint32_t& flags, LaunchList& out) {
  plan_neighbours(
      segs, kJoinMaxIdleTiles, [](const Seg2D& g) { return (uint64_t)g.n_tiles; },
      [&](size_t i, size_t j, uint32_t top, uint32_t fl) {
        if (j - i == 1) return plan_plain(segs[i], rev, fl, out);
        PreparedLaunch p = new_launch(kKernelTile2D, rev, fl, top * kBlocksPerTile, (uint32_t)(j - i), kBlockThreads, 0);
        for (size_t k = i; k < j; k++) p.u.a2d.seg[k - i] = segs[k];
        out.push_back(p);
      },
      flags);
}

// the same for transposing tiles (one workgroup of kTransThreads work-items per tile)
constexpr uint64_t kTransJoinMaxIdleTiles = 64;

void plan_trans_group(std::vector<TransSeg>& segs, bool rev, uint32_t lds, uint32_t& flags, LaunchList& out) {
  plan_neighbours(
      segs, kTransJoinMaxIdleTiles, [](const TransSeg& g) { return (uint64_t)g.n; },
      [&](size_t i, size_t j, uint32_t top, uint32_t fl) {
        if (j - i == 1) return plan_trans(segs[i].tiles, segs[i].n, rev, lds, fl, out);
        PreparedLaunch p = new_launch(kKernelTrans2D, rev, fl, top, (uint32_t)(j - i), kTransThreads, lds);
        for (size_t k = i; k < j; k++) p.u.t2d.seg[k - i] = segs[k];
        out.push_back(p);
      },
      flags);
}

// Pieces of one destination row that arrive through different chunks (a target row assembled from several source
// ranks' column blocks).  When a piece is not a whole number of 128-byte lines, every line at a piece boundary is
// written in parts by different workgroups, which costs up to two thirds of the bandwidth (2.2 instead of 6.5 TB/s
// at 32-byte pieces, 5.3 at 352 bytes).  In a write-ordered unpack range such sibling chunks - same rows, same
// shape, adjacent columns - are taken out of the plain tiles and covered by gather tiles instead: row tiles whose
// row is all P pieces, so that one wavefront writes whole lines and reads P short streams.
constexpr uint32_t kGatherLineBytes = 128;
// Pieces above 1 KiB are left to the plain tiles: on the short-row workload (256 tensors, pieces of 32 B - 2 KiB)
// gathering every size measured 77.2 % of peak, gathering up to 256 B / 512 B / 1 KiB 77.8 / 77.9 / 77.8 %, and a
// lone scatter of 992-byte pieces still gains (5.5 -> 6.5 TB/s); at 2016 bytes the plain tiles already reach 5.9.
constexpr uint64_t kGatherMaxPieceBytes = 1024;

struct PieceRows {  // a chunk that is a plain 2-D block of rows: rows x run units at the two pitches
  uint32_t chunk;
  uint64_t a, b;
  int64_t a_pitch, b_pitch;
  uint32_t run, meta;
  uint64_t rows;
};

// the chunk as PieceRows when its tiles are exactly one such block (no run tiles, no transposing tiles, one tile
// sequence that walks the rows in order)
bool piece_rows_of(const EthaTable* t, uint32_t c, PieceRows* out) {
  const uint32_t w0 = t->row_begin[c], w1 = t->row_begin[c + 1];
  if (w1 == w0 || t->run_begin[c + 1] != t->run_begin[c] || t->trans_begin[c + 1] != t->trans_begin[c]) return false;
  const RowTile& t0 = t->h_row[w0];
  if (t0.n_peers != 0 || t0.c0 != 0 || t0.run >= kTileThreads || t0.a_pitch <= 0) return false;
  uint64_t units = 0;
  for (uint32_t k = w0; k < w1; k++) {
    const RowTile& y = t->h_row[k];
    const uint64_t r = units / t0.run, c0 = units % t0.run;
    if (y.n_peers != 0 || y.run != t0.run || y.meta != t0.meta || y.a_pitch != t0.a_pitch || y.b_pitch != t0.b_pitch ||
        y.c0 != c0 || y.a != t0.a + r * (uint64_t)t0.a_pitch || y.b != (uint64_t)((int64_t)t0.b + (int64_t)r * t0.b_pitch))
      return false;
    units += y.n;
  }
  if (units % t0.run != 0) return false;
  *out = PieceRows{c, t0.a, t0.b, t0.a_pitch, t0.b_pitch, t0.run, t0.meta, units / t0.run};
  return true;
}

// Finds the sibling groups among chunks [first, first + count), appends their gather tiles and piece addresses,
// and marks the chunks they replace.
void gather_sibling_chunks(const EthaTable* t, uint32_t first, uint32_t count, std::vector<RowTile>& tiles,
                           std::vector<uint64_t>& gather, std::vector<char>& replaced) {
  std::vector<PieceRows> cand;
  for (uint32_t c = first; c < first + count; c++) {
    PieceRows p;
    if (piece_rows_of(t, c, &p)) cand.push_back(p);
  }
  std::stable_sort(cand.begin(), cand.end(), [](const PieceRows& x, const PieceRows& y) { return x.a < y.a; });
  size_t i = 0;
  while (i < cand.size()) {
    const PieceRows& x = cand[i];
    const uint64_t piece = (uint64_t)x.run << ((x.meta >> kMetaUaShift) & 15u);
    uint32_t pieces = 1;
    if (piece % kGatherLineBytes != 0 && piece <= kGatherMaxPieceBytes) {
      while (pieces < kGatherMaxPieces && i + pieces < cand.size()) {
        const PieceRows& y = cand[i + pieces];
        if (y.run != x.run || y.meta != x.meta || y.a_pitch != x.a_pitch || y.b_pitch != x.b_pitch || y.rows != x.rows ||
            y.a != x.a + pieces * piece || (uint64_t)(pieces + 1) * piece > (uint64_t)x.a_pitch ||
            (uint64_t)(pieces + 1) * x.run > kTileThreads)
          break;
        pieces++;
      }
    }
    if (pieces < 2) {
      i++;
      continue;
    }
    // the rows of all pieces, `width` units each, are cut into tiles of kTileThreads units like any other rows
    const uint64_t width = (uint64_t)x.run * pieces, total = x.rows * width;
    for (uint64_t q = 0; q < total; q += kTileThreads) {
      const uint64_t row0 = q / width;
      RowTile g;
      memset(&g, 0, sizeof(g));
      g.a = x.a + row0 * (uint64_t)x.a_pitch;
      g.b = (uint64_t)((int64_t)x.b + (int64_t)row0 * x.b_pitch);  // piece 0, for inspection only
      g.a_pitch = x.a_pitch;
      g.b_pitch = x.b_pitch;
      g.meta = x.meta | kMetaGather;
      g.run = (uint32_t)width;
      g.c0 = (uint32_t)(q % width);
      g.n = (uint32_t)(total - q < kTileThreads ? total - q : kTileThreads);
      g.peer_first = (uint32_t)gather.size();
      g.n_peers = pieces;
      g.via = x.run;
      for (uint32_t p2 = 0; p2 < pieces; p2++)
        gather.push_back((uint64_t)((int64_t)cand[i + p2].b + (int64_t)row0 * x.b_pitch));
      tiles.push_back(g);
    }
    for (uint32_t p2 = 0; p2 < pieces; p2++) replaced[cand[i + p2].chunk - first] = 1;
    i += pieces;
  }
  if (!gather.empty()) gather.insert(gather.end(), kGatherMaxPieces, 0);  // a tile's fetch may run past its own pieces
}

int check_flags(uint32_t flags) {
  if (flags & ~(uint32_t)ETHA_LAUNCH_UNORDERED) return fail(ETHA_ERR_INVALID, "unknown launch flags 0x%x", flags);
  return ETHA_OK;
}

int check_segment(const EthaSegment& g, uint32_t i) {
  if (g.kind > ETHA_SEG_SELFCOPY) return fail(ETHA_ERR_INVALID, "segment %u: unknown kind %u", i, g.kind);
  const int rc = check_range(g.table, g.first, g.count, g.kind == ETHA_SEG_SELFCOPY ? 1 : 0);
  if (rc != ETHA_OK) return rc;
  const uint32_t n_reduce = g.table->reduce_prefix[g.first + g.count] - g.table->reduce_prefix[g.first];
  if ((g.kind == ETHA_SEG_PACK || g.kind == ETHA_SEG_UNPACK) && n_reduce)
    return fail(ETHA_ERR_INVALID, "segment %u: range holds Partial chunks", i);
  if (g.kind == ETHA_SEG_REDUCE_PACK && n_reduce != g.count)
    return fail(ETHA_ERR_INVALID, "segment %u: range holds chunks that are not Partial chunks", i);
  if (g.kind == ETHA_SEG_SELFCOPY && n_reduce && n_reduce != g.count)
    return fail(ETHA_ERR_INVALID, "segment %u: range mixes Partial and plain chunks; launch them separately", i);
  return ETHA_OK;
}

// The launches of one chunk range run by itself, as the entry point named by g.kind would run it.
void plan_single(const EthaSegment& g, uint32_t flags, LaunchList& out) {
  const EthaTable* t = g.table;
  if (t->reduce_prefix[g.first + g.count] != t->reduce_prefix[g.first])
    plan_reduce(t, g.first, g.count, flags, out);
  else
    plan_tiles(t, g.first, g.count, g.kind == ETHA_SEG_UNPACK, flags, out);
}

// The launches of a set of segments that do not depend on each other (validated by the caller).
void plan_segments(const EthaSegment* segs, uint32_t n_segments, uint32_t flags, LaunchList& out) {
  std::vector<Seg2D> forward, reverse, gathered;
  std::vector<TransSeg> trans_forward, trans_reverse;
  uint32_t trans_lds = 0;
  for (uint32_t i = 0; i < n_segments; i++) {
    const EthaSegment& g = segs[i];
    const EthaTable* t = g.table;
    if (t->reduce_prefix[g.first + g.count] != t->reduce_prefix[g.first]) {
      const size_t before = out.size();
      plan_reduce(t, g.first, g.count, flags, out);
      if (out.size() != before) flags |= ETHA_LAUNCH_UNORDERED;
      continue;
    }
    const bool rev = g.kind == ETHA_SEG_UNPACK;
    const uint32_t x0 = t->trans_begin[g.first], n_trans = plain_trans_tiles(t, g.first, g.count);
    if (n_trans) {
      (rev ? trans_reverse : trans_forward).push_back(TransSeg{t->d_trans + x0, n_trans, 0});
      if (t->trans_lds > trans_lds) trans_lds = t->trans_lds;
    }
    if (plan_typed(t, g.first, g.count, rev, flags, out)) flags |= ETHA_LAUNCH_UNORDERED;
    const Seg2D r = tile_range(t, g.first, g.count, rev);
    if (r.n_tiles) (rev ? reverse : forward).push_back(r);
    const Seg2D gr = gather_range(t, g.first, g.count, rev);
    if (gr.n_tiles) gathered.push_back(gr);
  }
  plan_trans_group(trans_forward, false, trans_lds, flags, out);
  plan_trans_group(trans_reverse, true, trans_lds, flags, out);
  plan_group(forward, false, flags, out);
  plan_group(reverse, true, flags, out);
  plan_neighbours(
      gathered, kJoinMaxIdleTiles, [](const Seg2D& x) { return (uint64_t)x.n_tiles; },
      [&](size_t i, size_t j, uint32_t top, uint32_t fl) { plan_gather(&gathered[i], (uint32_t)(j - i), top, fl, out); }, flags);
}

// launches of the calling thread's current entry-point call; kept between calls so that a transfer's launch calls
// do not allocate once the list has reached its size
LaunchList& scratch_launches() {
  thread_local LaunchList list;
  list.clear();
  return list;
}

int launch_single(const EthaTable* t, uint32_t kind, uint32_t first, uint32_t count, void* stream, uint32_t flags) {
  return guarded("launch", [&]() -> int {
    LaunchList& list = scratch_launches();
    plan_single(EthaSegment{t, kind, first, count, 0}, flags, list);
    return issue_all(list.data(), list.size(), stream);
  });
}

}  // namespace

// A recorded sequence of launch calls, planned once: see etha_schedule_create.
struct EthaSchedule {
  LaunchList launches;
  struct Dep {
    const EthaTable* table;
    uint64_t serial;
    uint32_t version;
  };
  std::vector<Dep> deps;
  uint32_t n_calls = 0;
};

extern "C" {

#ifndef ETHA_SOURCE_HASH
#define ETHA_SOURCE_HASH "unknown"
#endif
int etha_abi_version(void) { return ETHA_ABI_VERSION; }
uint64_t etha_kernel_launches(void) { return g_kernel_launches.load(std::memory_order_relaxed); }
// the marker lets a build script find the digest in the file without loading the library
static const char kSourceDigest[] = "etha-source-digest:" ETHA_SOURCE_HASH;
const char* etha_source_hash(void) { return kSourceDigest + sizeof("etha-source-digest:") - 1; }
const char* etha_last_error(void) { return g_err; }

int etha_table_create(const EthaChunkDesc* descs, uint32_t n_chunks, const uint64_t* partial_ptrs,
                      uint32_t n_partial_ptrs, int upload, EthaTable** out) {
  if (!out) return fail(ETHA_ERR_INVALID, "null out");
  *out = nullptr;
  if (n_chunks && !descs) return fail(ETHA_ERR_INVALID, "null descriptor array");
  return guarded("etha_table_create", [&]() -> int {
    Builder bld;
    bld.run_begin.reserve(n_chunks + 1);
    bld.row_begin.reserve(n_chunks + 1);
    bld.is_reduce.assign(n_chunks, 0);
    for (uint32_t i = 0; i < n_chunks; i++) {
      const EthaChunkDesc& d = descs[i];
      bld.run_begin.push_back((uint32_t)bld.run.size());
      bld.row_begin.push_back((uint32_t)bld.row.size());
      bld.trans_begin.push_back((uint32_t)bld.trans.size());
      const int esw = dtype_size(d.wire_dtype);
      if (esw == 0) return fail(ETHA_ERR_INVALID, "chunk %u: unknown wire_dtype %u", i, d.wire_dtype);
      ReduceSpec red;
      std::vector<uint64_t> peer_bases;
      Region A;
      if (d.n_partials) {
        { const int rc_op = check_reduce_op(d.reduce_op, d.n_partials, i); if (rc_op != ETHA_OK) return rc_op; }
        if (!partial_ptrs || (uint64_t)d.partial_first + d.n_partials > n_partial_ptrs)
          return fail(ETHA_ERR_INVALID, "chunk %u: partial pointer range outside partial_ptrs", i);
        // every peer shares the chunk geometry; validate each peer's range with its own base
        for (uint32_t p = 0; p < d.n_partials; p++) {
          Region tmp;
          EthaChunkDesc dp = d;
          dp.tensor_lo = dp.tensor_hi = 0;  // the single lo/hi pair cannot describe several peers
          const int rc = tensor_region(dp, i, partial_ptrs[d.partial_first + p], false, &tmp);
          if (rc != ETHA_OK) return rc;
          peer_bases.push_back(partial_ptrs[d.partial_first + p]);
        }
        EthaChunkDesc dz = d;
        dz.tensor_lo = dz.tensor_hi = 0;
        const int rc = tensor_region(dz, i, 0, true, &A);  // offsets relative to a peer base
        if (rc != ETHA_OK) return rc;
        red.n_peers = d.n_partials;
        red.peer_first = d.partial_first;
        red.op = d.reduce_op;
        bld.is_reduce[i] = 1;
      } else {
        const int rc = tensor_region(d, i, d.tensor_ptr, false, &A);
        if (rc != ETHA_OK) return rc;
      }
      // bucket side: contiguous, row-major, wire dtype
      Region B;
      B.nd = A.nd;
      B.base = d.bucket_ptr;
      int64_t acc = esw;
      for (int j = A.nd - 1; j >= 0; j--) {
        B.shape[j] = A.shape[j];
        B.stride[j] = acc;
        acc *= A.shape[j];
      }
      const uint64_t nbytes = region_numel(A) * (uint64_t)esw;
      if (nbytes) {
        if (d.bucket_ptr == 0) return fail(ETHA_ERR_INVALID, "chunk %u: null bucket pointer", i);
        if ((d.bucket_lo || d.bucket_hi) &&
            (d.bucket_ptr < d.bucket_lo || d.bucket_ptr + nbytes > d.bucket_hi || d.bucket_ptr + nbytes < d.bucket_ptr))
          return fail(ETHA_ERR_INVALID, "chunk %u: bucket bytes [%llx,%llx) leave the bucket buffer [%llx,%llx)", i,
                      (unsigned long long)d.bucket_ptr, (unsigned long long)(d.bucket_ptr + nbytes),
                      (unsigned long long)d.bucket_lo, (unsigned long long)d.bucket_hi);
      }
      bld.payload_bytes += nbytes;
      const int rc = compile_pair(bld, i, A, B, d.tensor_dtype, d.wire_dtype, red, peer_bases);
      if (rc != ETHA_OK) return rc;
    }
    bld.run_begin.push_back((uint32_t)bld.run.size());
    bld.row_begin.push_back((uint32_t)bld.row.size());
    bld.trans_begin.push_back((uint32_t)bld.trans.size());
    EthaTable* t = new (std::nothrow) EthaTable();
    if (!t) return fail(ETHA_ERR_NOMEM, "out of host memory");
    t->kind = 0;
    t->n_chunks = n_chunks;
    return finish_table(bld, t, partial_ptrs, n_partial_ptrs, upload, out);
  });
}

int etha_direct_table_create(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks,
                             const uint64_t* partial_ptrs, uint32_t n_partial_ptrs, int upload, EthaTable** out) {
  if (!out) return fail(ETHA_ERR_INVALID, "null out");
  *out = nullptr;
  if (n_chunks && (!src || !dst)) return fail(ETHA_ERR_INVALID, "null descriptor array");
  return guarded("etha_direct_table_create", [&]() -> int {
    Builder bld;
    bld.is_reduce.assign(n_chunks, 0);
    for (uint32_t i = 0; i < n_chunks; i++) {
      bld.run_begin.push_back((uint32_t)bld.run.size());
      bld.row_begin.push_back((uint32_t)bld.row.size());
      bld.trans_begin.push_back((uint32_t)bld.trans.size());
      if (dst[i].n_partials) return fail(ETHA_ERR_INVALID, "chunk %u: a destination cannot be Partial", i);
      Region A, B;
      ReduceSpec red;
      std::vector<uint64_t> peer_bases;
      const EthaChunkDesc& d = src[i];
      int rc;
      if (d.n_partials) {
        { const int rc_op = check_reduce_op(d.reduce_op, d.n_partials, i); if (rc_op != ETHA_OK) return rc_op; }
        if (!partial_ptrs || (uint64_t)d.partial_first + d.n_partials > n_partial_ptrs)
          return fail(ETHA_ERR_INVALID, "chunk %u: partial pointer range outside partial_ptrs", i);
        if (dtype_size(d.wire_dtype) == 0) return fail(ETHA_ERR_INVALID, "chunk %u: unknown wire_dtype %u", i, d.wire_dtype);
        EthaChunkDesc dz = d;
        dz.tensor_lo = dz.tensor_hi = 0;  // the single lo/hi pair cannot describe several peers
        for (uint32_t p = 0; p < d.n_partials; p++) {
          Region tmp;
          rc = tensor_region(dz, i, partial_ptrs[d.partial_first + p], false, &tmp);
          if (rc != ETHA_OK) return rc;
          peer_bases.push_back(partial_ptrs[d.partial_first + p]);
        }
        rc = tensor_region(dz, i, 0, true, &A);  // offsets relative to a peer base
        if (rc != ETHA_OK) return rc;
        red.n_peers = d.n_partials;
        red.peer_first = d.partial_first;
        red.op = d.reduce_op;
        // the bucket path rounds the accumulator to the wire dtype first; keep that rounding when it is not the last one
        if (d.wire_dtype != dst[i].tensor_dtype) {
          if (!is_float(d.wire_dtype))
            return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: Partial reduce needs a floating wire dtype", i);
          red.via = 1 + d.wire_dtype;
        }
        bld.is_reduce[i] = 1;
      } else {
        rc = tensor_region(d, i, d.tensor_ptr, false, &A);
        if (rc != ETHA_OK) return rc;
      }
      rc = tensor_region(dst[i], i, dst[i].tensor_ptr, false, &B);
      if (rc != ETHA_OK) return rc;
      bld.payload_bytes += region_numel(A) * (uint64_t)dtype_size(dst[i].tensor_dtype);
      rc = compile_pair(bld, i, A, B, d.tensor_dtype, dst[i].tensor_dtype, red, peer_bases);
      if (rc != ETHA_OK) return rc;
    }
    bld.run_begin.push_back((uint32_t)bld.run.size());
    bld.row_begin.push_back((uint32_t)bld.row.size());
    bld.trans_begin.push_back((uint32_t)bld.trans.size());
    EthaTable* t = new (std::nothrow) EthaTable();
    if (!t) return fail(ETHA_ERR_NOMEM, "out of host memory");
    t->kind = 1;
    t->n_chunks = n_chunks;
    return finish_table(bld, t, partial_ptrs, n_partial_ptrs, upload, out);
  });
}

int etha_selfcopy_table_create(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks, int upload,
                               EthaTable** out) {
  for (uint32_t i = 0; src && i < n_chunks; i++)
    if (src[i].n_partials) return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: a same-rank copy has no Partial source", i);
  return etha_direct_table_create(src, dst, n_chunks, nullptr, 0, upload, out);
}

int etha_table_destroy(EthaTable* table) {
  free_table(table);
  return ETHA_OK;
}

int etha_table_info(const EthaTable* t, EthaTableInfo* out) {
  if (!t || !out) return fail(ETHA_ERR_INVALID, "null argument");
  out->n_chunks = t->n_chunks;
  out->n_run_tiles = (uint32_t)t->h_run.size();
  out->n_row_tiles = (uint32_t)t->h_row.size();
  out->n_trans_tiles = (uint32_t)t->h_trans.size();
  out->tile_threads = kTileThreads;
  out->device_bytes = t->device_bytes;
  out->payload_bytes = t->payload_bytes;
  return ETHA_OK;
}

int etha_table_read_tiles(const EthaTable* t, int which, void* out, uint64_t cap_bytes, uint64_t* need_bytes) {
  if (!t || !need_bytes) return fail(ETHA_ERR_INVALID, "null argument");
  const void* src;
  uint64_t bytes;
  if (which == 0) {
    src = t->h_run.data();
    bytes = t->h_run.size() * sizeof(RunTile);
  } else if (which == 1) {
    src = t->h_row.data();
    bytes = t->h_row.size() * sizeof(RowTile);
  } else if (which == 2) {
    src = t->h_trans.data();
    bytes = t->h_trans.size() * sizeof(TransTile);
  } else {
    return fail(ETHA_ERR_INVALID, "which must be 0, 1 or 2");
  }
  *need_bytes = bytes;
  if (out && bytes) memcpy(out, src, bytes < cap_bytes ? bytes : cap_bytes);
  return ETHA_OK;
}

int etha_table_read_ranges(const EthaTable* t, uint32_t* run_begin, uint32_t* row_begin) {
  if (!t || !run_begin || !row_begin) return fail(ETHA_ERR_INVALID, "null argument");
  memcpy(run_begin, t->run_begin.data(), t->run_begin.size() * sizeof(uint32_t));
  memcpy(row_begin, t->row_begin.data(), t->row_begin.size() * sizeof(uint32_t));
  return ETHA_OK;
}

int etha_table_read_trans_ranges(const EthaTable* t, uint32_t* trans_begin) {
  if (!t || !trans_begin) return fail(ETHA_ERR_INVALID, "null argument");
  memcpy(trans_begin, t->trans_begin.data(), t->trans_begin.size() * sizeof(uint32_t));
  return ETHA_OK;
}

int etha_table_optimize_range(EthaTable* t, uint32_t first, uint32_t count) {
  if (!t) return fail(ETHA_ERR_INVALID, "null table");
  if ((uint64_t)first + count > t->n_chunks)
    return fail(ETHA_ERR_INVALID, "chunk range [%u,%u) exceeds table of %u chunks", first, first + count, t->n_chunks);
  return guarded("etha_table_optimize_range", [&]() -> int {
    if (t->reduce_prefix[first + count] != t->reduce_prefix[first]) return ETHA_OK;  // reduce-pack writes buckets: already ordered
    const auto key = std::make_pair(first, count);
    if (t->ordered.count(key)) return ETHA_OK;
    EthaTable::Ordered o;
    const bool by_a = t->kind == 0;  // unpack writes the tensor (a) side; a self-copy writes its b side
    std::vector<RowTile> gather_tiles;
    std::vector<char> replaced(count, 0);
    if (by_a) gather_sibling_chunks(t, first, count, gather_tiles, o.h_gather, replaced);
    o.h_run.assign(t->h_run.begin() + t->run_begin[first], t->h_run.begin() + t->run_begin[first + count]);
    for (uint32_t c = first; c < first + count; c++)
      if (!replaced[c - first]) o.h_row.insert(o.h_row.end(), t->h_row.begin() + t->row_begin[c], t->h_row.begin() + t->row_begin[c + 1]);
    const auto unit = [](uint32_t meta, bool a_side) { return 1ull << ((meta >> (a_side ? kMetaUaShift : kMetaUbShift)) & 15u); };
    std::stable_sort(o.h_run.begin(), o.h_run.end(),
                     [by_a](const RunTile& x, const RunTile& y) { return by_a ? x.a < y.a : x.b < y.b; });
    std::stable_sort(o.h_row.begin(), o.h_row.end(), [by_a, unit](const RowTile& x, const RowTile& y) {
      const uint64_t px = (by_a ? x.a : x.b) + x.c0 * unit(x.meta, by_a), py = (by_a ? y.a : y.b) + y.c0 * unit(y.meta, by_a);
      return px < py;
    });
    o.n_plain_rows = (uint32_t)o.h_row.size();
    o.h_row.insert(o.h_row.end(), gather_tiles.begin(), gather_tiles.end());  // in address order already
    if (t->uploaded) {
      const size_t run_bytes = o.h_run.size() * sizeof(RunTile), row_bytes = o.h_row.size() * sizeof(RowTile);
      const size_t gather_bytes = o.h_gather.size() * sizeof(uint64_t);
      hipError_t e = hipSuccess;
      if (run_bytes) e = hipMalloc(&o.d_run, run_bytes);
      if (e == hipSuccess && run_bytes) e = hipMemcpy(o.d_run, o.h_run.data(), run_bytes, hipMemcpyHostToDevice);
      if (e == hipSuccess && row_bytes) e = hipMalloc(&o.d_row, row_bytes);
      if (e == hipSuccess && row_bytes) e = hipMemcpy(o.d_row, o.h_row.data(), row_bytes, hipMemcpyHostToDevice);
      if (e == hipSuccess && gather_bytes) e = hipMalloc(&o.d_gather, gather_bytes);
      if (e == hipSuccess && gather_bytes) e = hipMemcpy(o.d_gather, o.h_gather.data(), gather_bytes, hipMemcpyHostToDevice);
      if (e != hipSuccess) {
        if (o.d_run) (void)hipFree(o.d_run);
        if (o.d_row) (void)hipFree(o.d_row);
        if (o.d_gather) (void)hipFree(o.d_gather);
        return fail(ETHA_ERR_HIP, "uploading the ordered range: %s", hipGetErrorString(e));
      }
      t->device_bytes += run_bytes + row_bytes + gather_bytes;
    }
    t->ordered.emplace(key, std::move(o));
    t->version++;  // launches of this range planned earlier (schedules) no longer describe what a launch does now
    return ETHA_OK;
  });
}

int etha_table_read_ordered(const EthaTable* t, uint32_t first, uint32_t count, int which, void* out, uint64_t cap_bytes,
                            uint64_t* need_bytes) {
  if (!t || !need_bytes) return fail(ETHA_ERR_INVALID, "null argument");
  auto it = t->ordered.find(std::make_pair(first, count));
  if (it == t->ordered.end()) return fail(ETHA_ERR_INVALID, "range [%u,+%u) has not been optimized", first, count);
  if (which != 0 && which != 1 && which != 3) return fail(ETHA_ERR_INVALID, "which must be 0, 1 or 3");
  const void* src = which == 0   ? (const void*)it->second.h_run.data()
                    : which == 1 ? (const void*)it->second.h_row.data()
                                 : (const void*)it->second.h_gather.data();
  const uint64_t bytes = which == 0   ? it->second.h_run.size() * sizeof(RunTile)
                         : which == 1 ? it->second.h_row.size() * sizeof(RowTile)
                                      : it->second.h_gather.size() * sizeof(uint64_t);
  *need_bytes = bytes;
  if (out && bytes) memcpy(out, src, bytes < cap_bytes ? bytes : cap_bytes);
  return ETHA_OK;
}

int etha_pack_bucket(const EthaTable* t, uint32_t first, uint32_t count, void* stream, uint32_t flags) {
  int rc = check_range(t, first, count, 0);
  if (rc == ETHA_OK) rc = check_flags(flags);
  if (rc != ETHA_OK) return rc;
  if (t->reduce_prefix[first + count] != t->reduce_prefix[first])
    return fail(ETHA_ERR_INVALID, "range holds Partial chunks; use etha_reduce_pack_bucket");
  return launch_single(t, ETHA_SEG_PACK, first, count, stream, flags);
}

int etha_unpack_bucket(const EthaTable* t, uint32_t first, uint32_t count, void* stream, uint32_t flags) {
  int rc = check_range(t, first, count, 0);
  if (rc == ETHA_OK) rc = check_flags(flags);
  if (rc != ETHA_OK) return rc;
  if (t->reduce_prefix[first + count] != t->reduce_prefix[first])
    return fail(ETHA_ERR_INVALID, "range holds Partial chunks; a Partial placement cannot be a target");
  return launch_single(t, ETHA_SEG_UNPACK, first, count, stream, flags);
}

int etha_reduce_pack_bucket(const EthaTable* t, uint32_t first, uint32_t count, void* stream, uint32_t flags) {
  int rc = check_range(t, first, count, 0);
  if (rc == ETHA_OK) rc = check_flags(flags);
  if (rc != ETHA_OK) return rc;
  if (t->reduce_prefix[first + count] - t->reduce_prefix[first] != count)
    return fail(ETHA_ERR_INVALID, "range holds chunks that are not Partial chunks");
  return launch_single(t, ETHA_SEG_REDUCE_PACK, first, count, stream, flags);
}

int etha_selfcopy_bucket(const EthaTable* t, uint32_t first, uint32_t count, void* stream, uint32_t flags) {
  int rc = check_range(t, first, count, 1);
  if (rc == ETHA_OK) rc = check_flags(flags);
  if (rc != ETHA_OK) return rc;
  const uint32_t n_reduce = t->reduce_prefix[first + count] - t->reduce_prefix[first];
  if (n_reduce && n_reduce != count) return fail(ETHA_ERR_INVALID, "range mixes Partial and plain chunks; launch them separately");
  return launch_single(t, ETHA_SEG_SELFCOPY, first, count, stream, flags);
}

int etha_launch_segments(const EthaSegment* segs, uint32_t n_segments, void* stream, uint32_t flags) {
  int rc = check_flags(flags);
  if (rc != ETHA_OK) return rc;
  if (n_segments == 0) return ETHA_OK;
  if (!segs) return fail(ETHA_ERR_INVALID, "null segment list");
  for (uint32_t i = 0; i < n_segments; i++) {  // validate everything before the first launch
    rc = check_segment(segs[i], i);
    if (rc != ETHA_OK) return rc;
  }
  return guarded("etha_launch_segments", [&]() -> int {
    LaunchList& list = scratch_launches();
    plan_segments(segs, n_segments, flags, list);
    return issue_all(list.data(), list.size(), stream);
  });
}

int etha_schedule_create(const EthaSegment* segments, uint32_t n_segments, const EthaScheduleCall* calls, uint32_t n_calls,
                         EthaSchedule** out) {
  if (!out) return fail(ETHA_ERR_INVALID, "null out");
  *out = nullptr;
  if ((n_segments && !segments) || (n_calls && !calls)) return fail(ETHA_ERR_INVALID, "null argument");
  return guarded("etha_schedule_create", [&]() -> int {
    std::unique_ptr<EthaSchedule> s(new EthaSchedule());
    std::map<const EthaTable*, int> seen;
    for (uint32_t c = 0; c < n_calls; c++) {
      const EthaScheduleCall& call = calls[c];
      int rc = check_flags(call.flags);
      if (rc != ETHA_OK) return rc;
      if ((uint64_t)call.first_segment + call.n_segments > n_segments)
        return fail(ETHA_ERR_INVALID, "call %u: segments [%u,+%u) outside the segment array of %u", c, call.first_segment,
                    call.n_segments, n_segments);
      if (call.single > 1 || (call.single && call.n_segments != 1))
        return fail(ETHA_ERR_INVALID, "call %u: a single-range call names exactly one segment", c);
      const EthaSegment* segs = segments + call.first_segment;
      for (uint32_t i = 0; i < call.n_segments; i++) {
        rc = check_segment(segs[i], call.first_segment + i);
        if (rc != ETHA_OK) return rc;
        if (seen.emplace(segs[i].table, 1).second) s->deps.push_back(EthaSchedule::Dep{segs[i].table, segs[i].table->serial, segs[i].table->version});
      }
      if (call.single)
        plan_single(segs[0], call.flags, s->launches);
      else if (call.n_segments)
        plan_segments(segs, call.n_segments, call.flags, s->launches);
    }
    s->n_calls = n_calls;
    *out = s.release();
    return ETHA_OK;
  });
}

int etha_schedule_launch(const EthaSchedule* s, void* stream) {
  if (!s) return fail(ETHA_ERR_INVALID, "null schedule");
  {
    // the launches hold device addresses of the tables' tile programs: every table must still exist, unchanged
    std::lock_guard<std::mutex> lock(g_tables_mutex);
    for (const EthaSchedule::Dep& d : s->deps) {
      auto it = g_live_tables.find(d.table);
      if (it == g_live_tables.end() || it->second != d.serial)
        return fail(ETHA_ERR_INVALID, "stale schedule: a table it launches has been destroyed");
      if (d.table->version != d.version)
        return fail(ETHA_ERR_INVALID, "stale schedule: a table it launches has changed since the schedule was created");
    }
  }
  return issue_all(s->launches.data(), s->launches.size(), stream);
}

int etha_schedule_info(const EthaSchedule* s, EthaScheduleInfo* out) {
  if (!s || !out) return fail(ETHA_ERR_INVALID, "null argument");
  out->n_calls = s->n_calls;
  out->n_kernel_launches = (uint32_t)s->launches.size();
  out->n_tables = (uint32_t)s->deps.size();
  out->reserved = 0;
  return ETHA_OK;
}

int etha_schedule_destroy(EthaSchedule* s) {
  delete s;
  return ETHA_OK;
}

// ---- region copies for callers that cannot allocate --------------------------------------------
// The tile program of etha_copy_regions_noalloc lives in this array instead of in memory from hipMalloc.
// Each GPU the library runs on holds its own copy until the process ends.  In host code the name is only
// a stand-in for the symbol: its device address comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) unsigned char scratch[ETHA_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
struct NoAllocState {
  void* scratch_ptr = nullptr;  // device address of `scratch` on this device
  void* staging = nullptr;      // pinned host buffer the tile program is assembled in
  hipEvent_t copied = nullptr;  // the last call's upload has left the staging buffer
  bool copy_pending = false;
};
NoAllocState g_noalloc[kMaxDevices];
std::mutex g_noalloc_mutex;

int copy_regions_compile(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks, Builder& bld) {
  bld.run.clear();
  bld.row.clear();
  bld.trans.clear();
  bld.payload_bytes = 0;
  // the compiled program must fit the array (the three tile lists start on 64-byte boundaries): compilation stops
  // as soon as it cannot, before the host vectors grow past it
  bld.max_bytes = ETHA_NOALLOC_SCRATCH_BYTES - 128;
  const ReduceSpec none;
  static const std::vector<uint64_t> no_peers;
  for (uint32_t i = 0; i < n_chunks; i++) {
    if (src[i].n_partials || dst[i].n_partials) return fail(ETHA_ERR_UNSUPPORTED, "chunk %u: a region copy has no Partial side", i);
    Region A, B;
    int rc = tensor_region(src[i], i, src[i].tensor_ptr, false, &A);
    if (rc == ETHA_OK) rc = tensor_region(dst[i], i, dst[i].tensor_ptr, false, &B);
    if (rc == ETHA_OK) rc = compile_pair(bld, i, A, B, src[i].tensor_dtype, dst[i].tensor_dtype, none, no_peers);
    if (rc != ETHA_OK) return rc;
  }
  return ETHA_OK;
}
}  // namespace

int etha_noalloc_setup(void) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(ETHA_ERR_UNSUPPORTED, "device index %d is beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_noalloc_mutex);
  NoAllocState& st = g_noalloc[dev];
  if (st.scratch_ptr) return ETHA_OK;
  void* ptr = nullptr;
  HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return fail(ETHA_ERR_HIP, "hipGetSymbolAddress returned a null address");
  void* staging = nullptr;
  HIP_TRY(hipHostMalloc(&staging, ETHA_NOALLOC_SCRATCH_BYTES, hipHostMallocDefault));
  hipEvent_t ev = nullptr;
  hipError_t e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
  if (e != hipSuccess) {
    (void)hipHostFree(staging);
    return fail(ETHA_ERR_HIP, "hipEventCreateWithFlags: %s", hipGetErrorString(e));
  }
  st.staging = staging;
  st.copied = ev;
  st.scratch_ptr = ptr;
  return ETHA_OK;
}

int etha_copy_regions_noalloc(const EthaChunkDesc* src, const EthaChunkDesc* dst, uint32_t n_chunks, void* stream) {
  if (n_chunks && (!src || !dst)) return fail(ETHA_ERR_INVALID, "null descriptor array");
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(ETHA_ERR_INVALID, "call etha_noalloc_setup() with this device current first");
  // Not for a stream under capture: the upload of the tile program would become a graph node that reads the
  // shared staging buffer at every replay, after later calls have overwritten it.
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  HIP_TRY(hipStreamIsCapturing((hipStream_t)stream, &capture));
  if (capture != hipStreamCaptureStatusNone)
    return fail(ETHA_ERR_UNSUPPORTED, "etha_copy_regions_noalloc cannot be recorded into a graph: the stream is capturing");
  return guarded("etha_copy_regions_noalloc", [&]() -> int {
    // host-side compilation reuses this thread's vectors: they grow to at most the array's size
    thread_local Builder bld;
    const int rc = copy_regions_compile(src, dst, n_chunks, bld);
    if (rc != ETHA_OK) {
      if (bld.run.capacity() * sizeof(RunTile) + bld.row.capacity() * sizeof(RowTile) + bld.trans.capacity() * sizeof(TransTile) >
          2ull * ETHA_NOALLOC_SCRATCH_BYTES) {  // a refused request does not leave its memory with the thread
        std::vector<RunTile>().swap(bld.run);
        std::vector<RowTile>().swap(bld.row);
        std::vector<TransTile>().swap(bld.trans);
      }
      return rc;
    }
    const size_t run_bytes = bld.run.size() * sizeof(RunTile);
    const size_t row_off = (run_bytes + 63) & ~(size_t)63, row_bytes = bld.row.size() * sizeof(RowTile);
    const size_t trans_off = (row_off + row_bytes + 63) & ~(size_t)63, trans_bytes = bld.trans.size() * sizeof(TransTile);
    const size_t total = trans_off + trans_bytes;
    if (total > (size_t)ETHA_NOALLOC_SCRATCH_BYTES)
      return fail(ETHA_ERR_UNSUPPORTED,
                  "these regions need a tile program of %llu bytes; etha_copy_regions_noalloc holds at most %llu "
                  "(use etha_selfcopy_table_create for larger copies)",
                  (unsigned long long)total, (unsigned long long)ETHA_NOALLOC_SCRATCH_BYTES);
    if (run_bytes + row_bytes + trans_bytes == 0) return ETHA_OK;
    // one call at a time per process from here on: the staging buffer and the array are shared
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    NoAllocState& st = g_noalloc[dev];
    if (!st.scratch_ptr) return fail(ETHA_ERR_INVALID, "call etha_noalloc_setup() with this device current first");
    if (st.copy_pending) HIP_TRY(hipEventSynchronize(st.copied));  // the previous call's upload still reads the staging buffer
    uint8_t* stage = static_cast<uint8_t*>(st.staging);
    if (run_bytes) memcpy(stage, bld.run.data(), run_bytes);
    if (row_bytes) memcpy(stage + row_off, bld.row.data(), row_bytes);
    if (trans_bytes) memcpy(stage + trans_off, bld.trans.data(), trans_bytes);
    uint8_t* base = static_cast<uint8_t*>(st.scratch_ptr);  // the array's memory on this device: never the symbol's name
    HIP_TRY(hipMemcpyAsync(base, stage, total, hipMemcpyHostToDevice, (hipStream_t)stream));
    HIP_TRY(hipEventRecord(st.copied, (hipStream_t)stream));
    st.copy_pending = true;
    uint32_t lds = 0;
    bool typed_tiles = false, plain_tiles = false;
    for (const TransTile& tt : bld.trans) {
      if (trans_tile_lds(tt) > lds) lds = trans_tile_lds(tt);
      ((tt.cvt & kTransTyped) ? typed_tiles : plain_tiles) = true;
    }
    PreparedLaunch launches[3];
    size_t n_launches = 0;
    if (plain_tiles) {
      launches[n_launches] = new_launch(kKernelTrans, false, 0, (uint32_t)bld.trans.size(), 1, kTransThreads, lds);
      launches[n_launches++].u.trans.tiles = (const TransTile*)(base + trans_off);
    }
    if (typed_tiles) {  // both kernels walk the whole list; each leaves the other's blocks alone
      launches[n_launches] = new_launch(kKernelTransTyped, false, 0, (uint32_t)bld.trans.size(), 1, kTransThreads, lds);
      launches[n_launches++].u.trans.tiles = (const TransTile*)(base + trans_off);
    }
    const uint32_t n_run = (uint32_t)bld.run.size(), n_row = (uint32_t)bld.row.size();
    if (n_run + n_row) {
      PreparedLaunch& p = launches[n_launches++];
      p = new_launch(kKernelTile, false, 0, (n_run + n_row) * kBlocksPerTile, 1, kBlockThreads, 0);
      p.u.tile.run = (const RunTile*)base;
      p.u.tile.n_run = n_run;
      p.u.tile.row = (const RowTile*)(base + row_off);
    }
    return issue_all(launches, n_launches, stream);
  });
}

int etha_arena_create(uint64_t nbytes, void** out_ptr) {
  if (!out_ptr || nbytes == 0) return fail(ETHA_ERR_INVALID, "bad arena request");
  *out_ptr = nullptr;
  HIP_TRY(hipMalloc(out_ptr, nbytes));
  return ETHA_OK;
}

int etha_arena_destroy(void* ptr) {
  if (ptr) HIP_TRY(hipFree(ptr));
  return ETHA_OK;
}

int etha_ipc_export(const void* dev_ptr, EthaIpcHandle* out) {
  if (!dev_ptr || !out) return fail(ETHA_ERR_INVALID, "null argument");
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  HIP_TRY(hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)dev_ptr));
  hipIpcMemHandle_t h;
  HIP_TRY(hipIpcGetMemHandle(&h, base));
  static_assert(sizeof(h) == 64, "hipIpcMemHandle_t size");
  memcpy(out->handle, &h, 64);
  out->offset = (uint64_t)((const char*)dev_ptr - (const char*)base);
  out->size = (uint64_t)size;
  return ETHA_OK;
}

int etha_ipc_open(const EthaIpcHandle* handle, void** out_ptr) {
  if (!handle || !out_ptr) return fail(ETHA_ERR_INVALID, "null argument");
  *out_ptr = nullptr;
  return guarded("etha_ipc_open", [&]() -> int {
    // shared allocations of 2 GiB and more have not opened reliably on this platform
    if (handle->size >= (2ull << 30))
      return fail(ETHA_ERR_UNSUPPORTED, "IPC allocation of %llu bytes: keep shared allocations under 2 GiB",
                  (unsigned long long)handle->size);
    IpcKey key;
    memcpy(key.data(), handle->handle, 64);
    std::lock_guard<std::mutex> lock(g_ipc_mutex);
    IpcMapping& m = g_ipc_open[key];
    if (m.refs == 0) {
      hipIpcMemHandle_t h;
      memcpy(&h, handle->handle, 64);
      void* base = nullptr;
      hipError_t e = hipIpcOpenMemHandle(&base, h, hipIpcMemLazyEnablePeerAccess);
      if (e != hipSuccess) {
        g_ipc_open.erase(key);
        return fail(ETHA_ERR_HIP, "hipIpcOpenMemHandle: %s", hipGetErrorString(e));
      }
      m.base = base;
    }
    m.refs++;
    void* p = (char*)m.base + handle->offset;
    g_ipc_ptrs[p] = key;
    g_ipc_ptr_refs[p]++;
    *out_ptr = p;
    return ETHA_OK;
  });
}

int etha_ipc_close(void* opened_ptr) {
  if (!opened_ptr) return ETHA_OK;
  return guarded("etha_ipc_close", [&]() -> int {
    std::lock_guard<std::mutex> lock(g_ipc_mutex);
    auto it = g_ipc_ptrs.find(opened_ptr);
    if (it == g_ipc_ptrs.end()) return fail(ETHA_ERR_INVALID, "pointer was not returned by etha_ipc_open");
    const IpcKey key = it->second;
    if (--g_ipc_ptr_refs[opened_ptr] == 0) {
      g_ipc_ptr_refs.erase(opened_ptr);
      g_ipc_ptrs.erase(it);
    }
    IpcMapping& m = g_ipc_open[key];
    if (--m.refs == 0) {
      void* base = m.base;
      g_ipc_open.erase(key);
      HIP_TRY(hipIpcCloseMemHandle(base));
    }
    return ETHA_OK;
  });
}

}  // extern "C"
