// Shared device helpers for the row-streaming distillation-loss kernels (gfx950).
//
// Execution model used by every kernel in this directory: one workgroup owns one
// token row of the [rows x vocab] logits.  The row is fetched with 16-byte
// non-temporal loads into registers (it is read from HBM exactly once), reduced
// with wave64 butterflies plus a cross-wave combine in LDS, and the gradient is
// written from the same registers with 16-byte non-temporal stores.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dl {

constexpr int WAVE = 64;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// dtype tags mirrored from the C header
enum : int { F32 = 0, BF16 = 1, F16 = 2 };
enum : int { I32 = 0, I64 = 1 };

struct TagF32 { static constexpr int id = F32; static constexpr int bytes = 4; static constexpr int epc = 4; };
struct TagBF16 { static constexpr int id = BF16; static constexpr int bytes = 2; static constexpr int epc = 8; };
struct TagF16 { static constexpr int id = F16; static constexpr int bytes = 2; static constexpr int epc = 8; };

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// ---- 16-byte chunk <-> floats -------------------------------------------------
template <class Tag> struct Chunk;

// eight floats <-> eight fp16 in 16 bytes (round to nearest even)
__device__ __forceinline__ void unpack_f16x8(const u32x4& c, float* f) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned u = c[i];   // copy first: bit_cast straight from a vector element reads element 0
    f16x2 h = __builtin_bit_cast(f16x2, u);
    f[2 * i] = (float)h[0];
    f[2 * i + 1] = (float)h[1];
  }
}
__device__ __forceinline__ u32x4 pack_f16x8(const float* f) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f16x2 h = __builtin_convertvector(f32x2{f[2 * i], f[2 * i + 1]}, f16x2);
    r[i] = __builtin_bit_cast(unsigned, h);
  }
  return r;
}

// Chunk<Tag>: a 16-byte piece of a row.  unpack/pack convert to and from floats in the row's
// dtype.  stash/unstash keep intermediate values in (0, 2^stash_bias] in the chunk's own 16 bytes
// between two sweeps: exactly for fp32 rows, as fp16 (11-bit significand, values pre-scaled by
// 2^15 so that 44 binades stay normal) for 16-bit rows.

template <> struct Chunk<TagF32> {
  static constexpr int N = 4;
  __device__ static __forceinline__ u32x4 neg_inf() { return u32x4{0xff800000u, 0xff800000u, 0xff800000u, 0xff800000u}; }
  __device__ static __forceinline__ void unpack(const u32x4& c, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(c[i]);
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {
    return u32x4{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
  }
  static constexpr float stash_bias = 0.f;
  __device__ static __forceinline__ u32x4 stash(const float* f) { return pack(f); }
  __device__ static __forceinline__ void unstash(const u32x4& c, float* f) { unpack(c, f); }
};

template <> struct Chunk<TagBF16> {
  static constexpr int N = 8;
  __device__ static __forceinline__ u32x4 neg_inf() { return u32x4{0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u}; }
  __device__ static __forceinline__ void unpack(const u32x4& c, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(c[i] << 16);
      f[2 * i + 1] = __uint_as_float(c[i] & 0xffff0000u);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float* f) {
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      bf16x2 b = __builtin_convertvector(f32x2{f[2 * i], f[2 * i + 1]}, bf16x2);   // v_cvt_pk_bf16_f32, RNE
      r[i] = __builtin_bit_cast(unsigned, b);
    }
    return r;
  }
  static constexpr float stash_bias = 15.f;
  __device__ static __forceinline__ u32x4 stash(const float* f) { return pack_f16x8(f); }
  __device__ static __forceinline__ void unstash(const u32x4& c, float* f) { unpack_f16x8(c, f); }
};

template <> struct Chunk<TagF16> {
  static constexpr int N = 8;
  __device__ static __forceinline__ u32x4 neg_inf() { return u32x4{0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u, 0xfc00fc00u}; }
  __device__ static __forceinline__ void unpack(const u32x4& c, float* f) { unpack_f16x8(c, f); }
  __device__ static __forceinline__ u32x4 pack(const float* f) { return pack_f16x8(f); }
  static constexpr float stash_bias = 15.f;
  __device__ static __forceinline__ u32x4 stash(const float* f) { return pack_f16x8(f); }
  __device__ static __forceinline__ void unstash(const u32x4& c, float* f) { unpack_f16x8(c, f); }
};

// ---- scalar element access by runtime dtype (K-wide side arrays only) ----------
__device__ __forceinline__ float load_as_float(const void* base, int dtype, int64_t i) {
  if (dtype == F32) return reinterpret_cast<const float*>(base)[i];
  unsigned short u = reinterpret_cast<const unsigned short*>(base)[i];
  if (dtype == BF16) return __uint_as_float(((unsigned)u) << 16);
  return (float)__builtin_bit_cast(_Float16, u);
}

__device__ __forceinline__ void store_from_float(void* base, int dtype, int64_t i, float v) {
  if (dtype == F32) {
    reinterpret_cast<float*>(base)[i] = v;
  } else if (dtype == BF16) {
    __bf16 b = (__bf16)v;
    reinterpret_cast<unsigned short*>(base)[i] = __builtin_bit_cast(unsigned short, b);
  } else {
    _Float16 h = (_Float16)v;
    reinterpret_cast<unsigned short*>(base)[i] = __builtin_bit_cast(unsigned short, h);
  }
}

__device__ __forceinline__ int64_t load_index(const void* base, int itype, int64_t i) {
  if (itype == I32) return (int64_t)reinterpret_cast<const int32_t*>(base)[i];
  return reinterpret_cast<const int64_t*>(base)[i];
}

// ---- streaming 16-byte accesses ------------------------------------------------
__device__ __forceinline__ u32x4 load16_stream(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
// 16 bytes from any address: the compiler lowers the copy to one unaligned 16-byte load, which global
// memory accesses of this target allow.
__device__ __forceinline__ u32x4 load16_unaligned(const void* p) {
  u32x4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}
__device__ __forceinline__ void store16_unaligned(void* p, const u32x4& v) { __builtin_memcpy(p, &v, 16); }
// Non-temporal stores: a bare copy kernel runs ~4 % faster with the default policy, but in the
// loss kernels (sparse corrections follow the dense row) the non-temporal hint measured faster.
__device__ __forceinline__ void store16_stream(void* p, const u32x4& v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// ---- sparse corrections of a row (part) held in registers -------------------------------------------
// A few columns of a row get a value other than the dense formula's.  Writing them with 2-byte stores
// after the dense 16-byte stores costs the memory system a read-modify-write of every touched line
// and the workgroup a wait for its dense stores to land; instead the thread that holds a column's
// chunk in its registers replaces the value before it stores the chunk.  Which register of which
// thread holds chunk c of the part (column offset / Chunk::N) is ChunkMap<NT, NCH>'s business.
//   correction_link:  called by whoever staged entry k: links k into the list of its chunk
//                     (head[slot] -> k -> next[k] ...) and marks the chunk in own[owner].  There are
//                     CORRECTION_HEADS list heads per workgroup, CORRECTION_HEADS / NT per thread:
//                     chunks i and i + CORRECTION_HEADS / NT of a thread share a list.
//   correction_apply: called by the owner for its chunk i when bit i % 32 of own[] is set: one walk
//                     over the chunk's list puts finish(k, term(k)) in place of the element of every
//                     entry k that falls into chunk i; returns true if an element was named more
//                     than once (ids repeat inside the row).
//   correction_repeats: called by the owner after its sweep for the chunks where correction_apply
//                     said so: every such element gets finish(k, sum of term over all its entries),
//                     written by an element-sized store behind the owner's own chunk store (same
//                     thread, same address: ordered).  The sum is taken in fixed point
//                     (correction_exact_sum), so it is the same whatever order the atomics gave the
//                     list.  Kept out of the sweep so that the sweep's registers do not pay for it.
// correction_clear (all threads) and a barrier come before the first link; a barrier separates the
// links from the applies.
constexpr int CORRECTION_HEADS = 2048;

// Where the 16-byte chunks of a row (part) sit while a workgroup of NT threads holds them in registers.
//   NCH == 0: striped over the workgroup: chunk c in register c / NT of thread c % NT (any number of
//             registers per thread; every load instruction of the workgroup covers NT consecutive chunks).
//   NCH > 0:  wave-major: every wave holds 64 * NCH consecutive chunks, chunk c in register
//             (c % (64 * NCH)) / 64 of lane c % 64 of wave c / (64 * NCH).  A wave's NCH loads then walk
//             through one contiguous stretch of NCH KiB instead of touching every NT * 16 bytes of the
//             part: with many waves in flight the memory system sees fewer, longer streams (a bare copy
//             of 256 threads x 16 chunks: 74.6 % of the HBM peak instead of 70.3 %).
template <int NT, int NCH>
struct ChunkMap {
  static constexpr bool WAVE_MAJOR = NCH > 0;
  static constexpr int SPAN = WAVE * (NCH > 0 ? NCH : 1);      // chunks per wave
  __device__ __forceinline__ static int chunk(int reg, int tid) {
    return WAVE_MAJOR ? (tid / WAVE) * SPAN + reg * WAVE + (tid % WAVE) : reg * NT + tid;
  }
  __device__ __forceinline__ static int owner(int c) { return WAVE_MAJOR ? (c / SPAN) * WAVE + c % WAVE : c % NT; }
  __device__ __forceinline__ static int reg(int c) { return WAVE_MAJOR ? (c % SPAN) / WAVE : c / NT; }
};

template <int NT>
__device__ __forceinline__ void correction_clear(int* head, unsigned* own) {
#pragma unroll
  for (int j = 0; j < CORRECTION_HEADS / NT; ++j) head[j * NT + threadIdx.x] = -1;
  own[threadIdx.x] = 0u;
}

// Index of the list head that serves the chunk holding column `offset` of the part.
template <class Tag, int NT, int NCH = 0>
__device__ __forceinline__ int correction_head_slot(int offset) {
  using M = ChunkMap<NT, NCH>;
  const int c = offset / Chunk<Tag>::N;
  return (M::reg(c) % (CORRECTION_HEADS / NT)) * NT + M::owner(c);
}

template <class Tag, int NT, int NCH = 0>
__device__ __forceinline__ void correction_link(int* head, unsigned* own, int* next, int k, int offset) {
  using M = ChunkMap<NT, NCH>;
  const int c = offset / Chunk<Tag>::N;
  next[k] = atomicExch(&head[correction_head_slot<Tag, NT, NCH>(offset)], k);
  atomicOr(&own[M::owner(c)], 1u << (M::reg(c) & 31));
}

// Sum of term(k) over the entries of a list that name column `want`: order-independent and exact to
// 2^-40 of the largest term.  Every term is scaled by a power of two chosen from the largest
// magnitude (an exact operation), cut to an integer and added as such; a single term comes back
// bit for bit.
template <class Term>
__device__ __forceinline__ float correction_exact_sum(const int* next, const int* col, int first, int want, Term term) {
  float big = 0.f;
  bool odd = false;                                   // NaN or infinity among the terms
  for (int k = first; k >= 0; k = next[k])
    if (col[k] == want) {
      const float t = term(k);
      odd = odd || !(fabsf(t) <= 3.0e38f);
      big = fmaxf(big, fabsf(t));
    }
  if (odd || big == 0.f) {                            // nothing to scale by: plain sum (its value is NaN, an infinity or 0)
    float sum = 0.f;
    for (int k = first; k >= 0; k = next[k]) sum += col[k] == want ? term(k) : 0.f;
    return sum;
  }
  int e;
  (void)frexpf(big, &e);                              // big = m * 2^e, 0.5 <= m < 1
  long long acc = 0;
  for (int k = first; k >= 0; k = next[k])
    if (col[k] == want) acc += (long long)ldexp((double)term(k), 40 - e);      // |.| < 2^40; up to 2048 of them: < 2^52
  return (float)ldexp((double)acc, e - 40);
}

template <class Tag, int NT, int NCH = 0, class Term, class Finish>
__device__ __forceinline__ bool correction_apply(const int* head, const int* next, const int* col, int lo, int i,
                                                 float (&f)[Chunk<Tag>::N], Term term, Finish finish) {
  using C = Chunk<Tag>;
  unsigned seen = 0u, again = 0u;
  for (int k = head[(i % (CORRECTION_HEADS / NT)) * NT + threadIdx.x]; k >= 0; k = next[k]) {
    const int off = col[k] - lo;
    if (ChunkMap<NT, NCH>::reg(off / C::N) != i) continue;
    const int e = off % C::N;
    again |= seen & (1u << e);
    seen |= 1u << e;
    const float v = finish(k, term(k));
#pragma unroll
    for (int j = 0; j < C::N; ++j) f[j] = (j == e) ? v : f[j];
  }
  return again != 0u;
}

// `chunks`: bit i % 32 set for the chunks i whose correction_apply returned true; n_chunks: chunks
// per thread; store(column, value) writes one element of the row.
template <class Tag, int NT, int NCH = 0, class Term, class Finish, class Store>
__device__ __forceinline__ void correction_repeats(const int* head, const int* next, const int* col, int lo,
                                                   unsigned chunks, int n_chunks, Term term, Finish finish, Store store) {
  using C = Chunk<Tag>;
  for (int i = 0; i < n_chunks; ++i) {
    if (!(chunks & (1u << (i & 31)))) continue;
    const int first = head[(i % (CORRECTION_HEADS / NT)) * NT + threadIdx.x];
    unsigned seen = 0u, again = 0u;
    for (int k = first; k >= 0; k = next[k]) {
      const int off = col[k] - lo;
      if (ChunkMap<NT, NCH>::reg(off / C::N) != i) continue;
      again |= seen & (1u << (off % C::N));
      seen |= 1u << (off % C::N);
    }
    while (again) {
      const int e = __ffs(again) - 1;
      again &= again - 1u;
      const int want = lo + ChunkMap<NT, NCH>::chunk(i, (int)threadIdx.x) * C::N + e;
      int any = -1;
      for (int k = first; k >= 0 && any < 0; k = next[k]) any = col[k] == want ? k : -1;
      store(want, finish(any, correction_exact_sum(next, col, first, want, term)));
    }
  }
}

// ---- workgroup id -> row ---------------------------------------------------------------------------
// Consecutive workgroup ids are dealt round-robin to the 8 XCDs.  For kernels that give a whole row to
// one workgroup this mapping makes every XCD work on 8 consecutive rows (one contiguous stretch of the
// gradient buffer per XCD instead of every eighth row): within a group of 64 ids, id b serves row
// (b % 8) * 8 + b / 8 of the group.  Measured: 4-5 % on the row-writing kernels.  The grid must be
// xcd_banded_grid(n_rows) workgroups; ids that map beyond the last row leave at once.
__device__ __forceinline__ int64_t xcd_banded_row(unsigned b) {
  return (int64_t)(b >> 6) * 64 + (b & 7u) * 8 + ((b & 63u) >> 3);
}
static inline unsigned xcd_banded_grid(int64_t n_rows) { return (unsigned)((n_rows + 63) / 64 * 64); }

// ---- reductions: fixed order => bit-reproducible ---------------------------------
// Over the 64 lanes of a wave (all of them active), result in every lane.  Data-parallel-primitive moves
// instead of lane exchanges through the LDS crossbar (six round trips of ~100 cycles each for a butterfly): the
// operand of each step comes through the ALU's own lane permutation -- neighbours inside a quad, quads inside
// half a row of 16, halves, then lane 15 of a row into the next row and lane 31 into the upper half -- after
// which lane 63 holds the total, read out as a scalar.  The order of the additions is fixed by the pattern.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_move(float old, float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
constexpr int DPP_QUAD_XOR1 = 0xB1, DPP_QUAD_XOR2 = 0x4E, DPP_ROW_HALF_MIRROR = 0x141, DPP_ROW_MIRROR = 0x140,
              DPP_ROW_BCAST15 = 0x142, DPP_ROW_BCAST31 = 0x143;
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_move<DPP_QUAD_XOR1>(v, v));
  v = fmaxf(v, dpp_move<DPP_QUAD_XOR2>(v, v));
  v = fmaxf(v, dpp_move<DPP_ROW_HALF_MIRROR>(v, v));
  v = fmaxf(v, dpp_move<DPP_ROW_MIRROR>(v, v));
  v = fmaxf(v, dpp_move<DPP_ROW_BCAST15, 0xa>(v, v));      // rows 1 and 3 take in rows 0 and 2 (the others keep their own)
  v = fmaxf(v, dpp_move<DPP_ROW_BCAST31, 0xc>(v, v));      // rows 2 and 3 take in rows 0-1
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), WAVE - 1));
}
// The same moves for other types: `from(old, v)` = v of the lane the step reads, or `old` where the step leaves the lane out.
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ int dpp_move(int old, int v) { return __builtin_amdgcn_update_dpp(old, v, CTRL, ROW_MASK, 0xf, false); }
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ double dpp_move(double old, double v) {
  const unsigned long long o = __builtin_bit_cast(unsigned long long, old), x = __builtin_bit_cast(unsigned long long, v);
  const unsigned lo = (unsigned)__builtin_amdgcn_update_dpp((int)(unsigned)o, (int)(unsigned)x, CTRL, ROW_MASK, 0xf, false);
  const unsigned hi = (unsigned)__builtin_amdgcn_update_dpp((int)(unsigned)(o >> 32), (int)(unsigned)(x >> 32), CTRL, ROW_MASK, 0xf, false);
  return __builtin_bit_cast(double, ((unsigned long long)hi << 32) | lo);
}
// The six steps with any commutative op; lanes that a step leaves out combine with their own value (`self`: min,
// max) or with `neutral` (sums).
template <class T, class Op>
__device__ __forceinline__ T wave_reduce_lane63(T v, T neutral, bool self, Op op) {
  v = op(v, dpp_move<DPP_QUAD_XOR1>(self ? v : neutral, v));
  v = op(v, dpp_move<DPP_QUAD_XOR2>(self ? v : neutral, v));
  v = op(v, dpp_move<DPP_ROW_HALF_MIRROR>(self ? v : neutral, v));
  v = op(v, dpp_move<DPP_ROW_MIRROR>(self ? v : neutral, v));
  v = op(v, dpp_move<DPP_ROW_BCAST15, 0xa>(self ? v : neutral, v));
  v = op(v, dpp_move<DPP_ROW_BCAST31, 0xc>(self ? v : neutral, v));
  return v;                                    // lane 63 holds the result
}
__device__ __forceinline__ int wave_min(int v) {
  v = wave_reduce_lane63(v, 0, true, [](int a, int b) { return a < b ? a : b; });
  return __builtin_amdgcn_readlane(v, WAVE - 1);
}
__device__ __forceinline__ int wave_max(int v) {
  v = wave_reduce_lane63(v, 0, true, [](int a, int b) { return a > b ? a : b; });
  return __builtin_amdgcn_readlane(v, WAVE - 1);
}
__device__ __forceinline__ unsigned wave_max(unsigned v) {
  int x = (int)v;
  x = wave_reduce_lane63(x, 0, true, [](int a, int b) { return (unsigned)a > (unsigned)b ? a : b; });
  return (unsigned)__builtin_amdgcn_readlane(x, WAVE - 1);
}
__device__ __forceinline__ unsigned wave_min(unsigned v) {
  int x = (int)v;
  x = wave_reduce_lane63(x, 0, true, [](int a, int b) { return (unsigned)a < (unsigned)b ? a : b; });
  return (unsigned)__builtin_amdgcn_readlane(x, WAVE - 1);
}
__device__ __forceinline__ int wave_sum(int v) {
  v = wave_reduce_lane63(v, 0, false, [](int a, int b) { return a + b; });
  return __builtin_amdgcn_readlane(v, WAVE - 1);
}
__device__ __forceinline__ double wave_sum(double v) {
  v = wave_reduce_lane63(v, 0.0, false, [](double a, double b) { return a + b; });
  const unsigned long long x = __builtin_bit_cast(unsigned long long, v);
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)x, WAVE - 1), hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(x >> 32), WAVE - 1);
  return __builtin_bit_cast(double, ((unsigned long long)hi << 32) | lo);
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<DPP_QUAD_XOR1>(0.f, v);
  v += dpp_move<DPP_QUAD_XOR2>(0.f, v);
  v += dpp_move<DPP_ROW_HALF_MIRROR>(0.f, v);
  v += dpp_move<DPP_ROW_MIRROR>(0.f, v);
  v += dpp_move<DPP_ROW_BCAST15, 0xa>(0.f, v);
  v += dpp_move<DPP_ROW_BCAST31, 0xc>(0.f, v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), WAVE - 1));
}

// All threads of the workgroup receive the result.  `scratch` holds NT/64 floats;
// two barriers per call so it can be reused immediately.
template <int NT, bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* scratch) {
  constexpr int NW = NT / WAVE;
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  if constexpr (NW == 1) return v;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = IS_MAX ? fmaxf(r, scratch[i]) : (r + scratch[i]);
  __syncthreads();
  return r;
}
template <int NT> __device__ __forceinline__ float block_max(float v, float* s) { return block_reduce<NT, true>(v, s); }
template <int NT> __device__ __forceinline__ float block_sum(float v, float* s) { return block_reduce<NT, false>(v, s); }

// Two maxima in one pair of barriers.
template <int NT>
__device__ __forceinline__ void block_max2(float& a, float& b, float* scratch) {
  constexpr int NW = NT / WAVE;
  a = wave_max(a);
  b = wave_max(b);
  if constexpr (NW == 1) return;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) { scratch[w] = a; scratch[NW + w] = b; }
  __syncthreads();
  float ra = scratch[0], rb = scratch[NW];
#pragma unroll
  for (int i = 1; i < NW; ++i) { ra = fmaxf(ra, scratch[i]); rb = fmaxf(rb, scratch[NW + i]); }
  __syncthreads();
  a = ra; b = rb;
}

// Two sums in one pair of barriers.
template <int NT>
__device__ __forceinline__ void block_sum2(float& a, float& b, float* scratch) {
  constexpr int NW = NT / WAVE;
  a = wave_sum(a);
  b = wave_sum(b);
  if constexpr (NW == 1) return;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) { scratch[w] = a; scratch[NW + w] = b; }
  __syncthreads();
  float ra = scratch[0], rb = scratch[NW];
#pragma unroll
  for (int i = 1; i < NW; ++i) { ra += scratch[i]; rb += scratch[NW + i]; }
  __syncthreads();
  a = ra; b = rb;
}

// Three sums in one pair of barriers (scratch: 3 * NT / 64 floats).
template <int NT>
__device__ __forceinline__ void block_sum3(float& a, float& b, float& c, float* scratch) {
  constexpr int NW = NT / WAVE;
  a = wave_sum(a);
  b = wave_sum(b);
  c = wave_sum(c);
  if constexpr (NW == 1) return;
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) { scratch[w] = a; scratch[NW + w] = b; scratch[2 * NW + w] = c; }
  __syncthreads();
  float ra = scratch[0], rb = scratch[NW], rc = scratch[2 * NW];
#pragma unroll
  for (int i = 1; i < NW; ++i) { ra += scratch[i]; rb += scratch[NW + i]; rc += scratch[2 * NW + i]; }
  __syncthreads();
  a = ra; b = rb; c = rc;
}

// Teacher row feeding logits row r: row_map[r] (identity without a map); anything outside
// [0, n_trows) means "masked row".
__device__ __forceinline__ int64_t teacher_row(const int32_t* row_map, int64_t r, int64_t n_trows) {
  const int64_t t = row_map ? (int64_t)row_map[r] : r;
  return (t >= 0 && t < n_trows) ? t : -1;
}

// Makes the compiler forget what it knows about a chunk held in registers.  Placed at
// the head of every sweep over a register-resident row so that the unpacked fp32 copies of
// one sweep are not kept alive for the next (that would double the register footprint).
__device__ __forceinline__ void forget(u32x4& c) {
  asm volatile("" : "+v"(c));
}

// ---- bitonic sort in registers ------------------------------------------------------------------
__device__ __forceinline__ unsigned lane_xor(unsigned v, int m) { return (unsigned)__shfl_xor((int)v, m, WAVE); }
__device__ __forceinline__ unsigned long long lane_xor(unsigned long long v, int m) {
  const unsigned l = (unsigned)__shfl_xor((int)(unsigned)v, m, WAVE), h = (unsigned)__shfl_xor((int)(unsigned)(v >> 32), m, WAVE);
  return ((unsigned long long)h << 32) | l;
}

template <class W, int EPL, int STRIDE>
__device__ __forceinline__ void sort_stage_in_lane(W (&c)[EPL], int first, int size) {
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    if ((j & STRIDE) == 0 && j + STRIDE < EPL) {
      const bool up = ((first + j) & size) == 0;
      const W a = c[j], b = c[j + STRIDE];
      const W mn = a < b ? a : b, mx = a < b ? b : a;
      c[j] = up ? mn : mx;
      c[j + STRIDE] = up ? mx : mn;
    }
  }
}

// The workgroup sorts NT * EPL words ascending; thread t holds elements t * EPL .. t * EPL + EPL - 1.
// Strides below EPL are exchanged inside a thread, strides inside a wave through lane exchanges,
// only the strides that cross waves through LDS (`xch`, NT * EPL words, free to reuse before and
// after; two barriers per such stage).  Far less LDS traffic than sorting in LDS: a 1024-word sort
// has 55 stages, of which 3 cross waves.
template <class W, int NT, int EPL>
__device__ __forceinline__ void block_sort(W (&c)[EPL], W* xch) {
  static_assert(EPL == 1 || EPL == 2 || EPL == 4 || EPL == 8 || EPL == 16, "elements per thread");
  const int tid = threadIdx.x;
  const int first = tid * EPL;
#pragma unroll 1
  for (int size = 2; size <= NT * EPL; size <<= 1) {
#pragma unroll 1
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride < EPL) {
        switch (stride) {
          case 1: sort_stage_in_lane<W, EPL, 1>(c, first, size); break;
          case 2: sort_stage_in_lane<W, EPL, 2>(c, first, size); break;
          case 4: sort_stage_in_lane<W, EPL, 4>(c, first, size); break;
          default: sort_stage_in_lane<W, EPL, 8>(c, first, size); break;
        }
      } else {
        const int tm = stride / EPL;                 // partner thread = tid ^ tm, same element slot
        const bool lower = (tid & tm) == 0;
        if (tm < WAVE) {
#pragma unroll
          for (int j = 0; j < EPL; ++j) {
            const bool up = ((first + j) & size) == 0;
            const W o = lane_xor(c[j], tm);
            const W mn = c[j] < o ? c[j] : o, mx = c[j] < o ? o : c[j];
            c[j] = (lower == up) ? mn : mx;
          }
        } else {
          __syncthreads();
#pragma unroll
          for (int j = 0; j < EPL; ++j) xch[j * NT + tid] = c[j];
          __syncthreads();
#pragma unroll
          for (int j = 0; j < EPL; ++j) {
            const bool up = ((first + j) & size) == 0;
            const W o = xch[j * NT + (tid ^ tm)];
            const W mn = c[j] < o ? c[j] : o, mx = c[j] < o ? o : c[j];
            c[j] = (lower == up) ? mn : mx;
          }
        }
      }
    }
  }
}

// A row that starts or ends off the 16-byte grid, seen as head | body | tail: the body is made of the
// 16-byte chunks that lie wholly inside the row (vector loads and stores), head and tail are the at
// most N - 1 elements on either side (element-wise).  peel == false: the row is on the grid and a whole
// number of chunks long; everything is body.
template <class Tag>
struct RowSplit {
  int head; int64_t nbody; int tail;
  __device__ __forceinline__ RowSplit(const void* row, int64_t V, bool peel) {
    constexpr int N = 16 / Tag::bytes;
    const int mis = peel ? (int)(reinterpret_cast<uintptr_t>(row) & 15) : 0;
    int64_t h = mis ? (16 - mis) / Tag::bytes : 0;
    if (h > V) h = V;
    head = (int)h;
    nbody = (V - h) / N;
    tail = (int)(V - h - nbody * N);
  }
  __device__ __forceinline__ int leftovers() const { return head + tail; }
  // column of leftover i, 0 <= i < leftovers()
  __device__ __forceinline__ int64_t column(int i) const { return i < head ? i : head + nbody * (16 / Tag::bytes) + (i - head); }
};

// One 16-byte chunk of a row that keeps no alignment promise and may end inside the chunk: assembled
// from element-sized loads, columns at or beyond n_cols read as -inf.
template <class Tag>
__device__ __forceinline__ u32x4 load_chunk_elementwise(const char* part, int chunk, int n_cols) {
  u32x4 v = Chunk<Tag>::neg_inf();
  const int col0 = chunk * Chunk<Tag>::N;
  if constexpr (Tag::bytes == 4) {
    const unsigned* e = reinterpret_cast<const unsigned*>(part) + col0;
#pragma unroll
    for (int d = 0; d < 4; ++d) if (col0 + d < n_cols) v[d] = e[d];
  } else {
    const unsigned short* e = reinterpret_cast<const unsigned short*>(part) + col0;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const unsigned lo = col0 + 2 * d < n_cols ? (unsigned)e[2 * d] : (v[d] & 0xffffu);
      const unsigned hi = col0 + 2 * d + 1 < n_cols ? (unsigned)e[2 * d + 1] : (v[d] >> 16);
      v[d] = lo | (hi << 16);
    }
  }
  return v;
}
// The counterpart for stores: the elements of chunk `chunk` that lie before column n_cols.
// The chunk with -inf in place of its elements n .. N-1 (the columns behind a row's end).
template <class Tag>
__device__ __forceinline__ u32x4 chunk_keep_first(u32x4 v, int n) {
  const u32x4 ninf = Chunk<Tag>::neg_inf();
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    if constexpr (Tag::bytes == 4) {
      v[d] = d < n ? v[d] : ninf[d];
    } else {
      const unsigned keep = (2 * d < n ? 0xffffu : 0u) | (2 * d + 1 < n ? 0xffff0000u : 0u);
      v[d] = (v[d] & keep) | (ninf[d] & ~keep);
    }
  }
  return v;
}

template <class Tag>
__device__ __forceinline__ void store_chunk_elementwise(char* part, int chunk, int n_cols, const u32x4& v) {
  const int col0 = chunk * Chunk<Tag>::N;
  if constexpr (Tag::bytes == 4) {
    unsigned* e = reinterpret_cast<unsigned*>(part) + col0;
#pragma unroll
    for (int d = 0; d < 4; ++d) if (col0 + d < n_cols) e[d] = v[d];
  } else {
    unsigned short* e = reinterpret_cast<unsigned short*>(part) + col0;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      if (col0 + 2 * d < n_cols) e[2 * d] = (unsigned short)(v[d] & 0xffffu);
      if (col0 + 2 * d + 1 < n_cols) e[2 * d + 1] = (unsigned short)(v[d] >> 16);
    }
  }
}

// zero-fill one gradient row (masked / padded token positions)
template <class Tag, int NT>
__device__ __forceinline__ void zero_row(void* grad_row, int64_t nchunks) {
  const u32x4 z{0u, 0u, 0u, 0u};
  for (int64_t c = threadIdx.x; c < nchunks; c += NT)
    store16_stream(reinterpret_cast<char*>(grad_row) + c * 16, z);
}

}  // namespace dl
