// Teacher-side producer: full-vocabulary log-softmax and the K largest entries per token row,
// emitted in the dataset's storage layout (log-probs fp16 or fp32, ids int32 or int64, descending).
//
// Two launches.  (1) One workgroup per column part of a row (512 threads x 8 chunks of 16 bytes,
// the part read from HBM once into registers; at 64 VGPRs four workgroups share a CU so that one
// part's loads overlap another's arithmetic).  After the max / sum-exp sweeps the registers are
// rewritten in place as order-preserving unsigned keys and the largest key of every chunk group is
// kept.  The K-th largest of those group maxima is a lower bound L of the part's K-th largest key
// (K distinct entries reach it), and with 1024 groups per part only ~K..1.5K entries lie at or above
// it: they are collected into LDS and written to a per-part record together with the part's
// (max, sum-exp) (sorted and cut to the best K only when the record cannot hold them all).
// (2) One workgroup per row merges the part records and the statistics into the row's log-sum-exp.
// The part kernel is bound by vector-ALU issue, not by memory: counters show the vector ALU busy
// ~95 % of the kernel's time at ~16 instructions per element (softmax sweeps ~8, key encoding and
// group maxima ~2, collection ~6).  Counting each thread's entries first and reserving their slots
// with one atomic per thread (instead of one wave-wide vote per entry position) was measured: more
// vector instructions, 9 % slower.  So was a region of candidates per wave with the count in a scalar
// register and every branch taken by whole waves (votes instead of atomics): no LDS atomics left, but
// 12 % more vector instructions (each vote costs a select and a compare) and 10 % more time.
// Ties go to the smaller id, deterministically; torch.topk, which the reference calls, leaves tie
// order open.  (Values are ordered by their bit patterns: -0 ranks just below +0, not level with it.)  Rows with more than 2048 entries at or above L (constant or coarsely quantised rows)
// take an exact but slow select by bisection over key bits and then over columns.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

constexpr int PROD_MAX_K = 1024;
constexpr int PROD_NT = 512, PROD_NCH = 8;
constexpr int PROD_G_SMALL = 1024 / PROD_NT, PROD_G_LARGE = PROD_NCH;    // chunk groups per thread: 1024 or 4096 groups per part
constexpr int PROD_CAP = 2048;              // candidates of a part held in LDS
constexpr int PROD_MAX_PARTS = 8;

typedef unsigned long long u64;
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));

struct PartHeader { float mx; float sm; int cnt; int pad; };     // 16 bytes, then cnt u64 entries

struct ProducerParams {
  const void* logits; int64_t row_stride; int64_t n_rows; int64_t V;
  const int32_t* row_list; int64_t n_out;
  int K; int parts;
  char* ws; int64_t part_stride;            // bytes per (row, part) record
  void* out_val; int out_dtype; void* out_idx; int out_itype;
  unsigned* redo_count; int32_t* redo_rows; // behind the records: output rows the row-level selection hands back
};

// Entries a part record can hold: a part with no more candidates than this hands all of them,
// unsorted, to the merge (which runs at far higher occupancy than the part kernel); a part with more
// sorts and keeps its best K.  parts * capacity <= 4096 (K <= 1024, parts <= 8 give at most 8192)
// keeps the merge inside 64 KiB of LDS together with its list of selected words.
__host__ __device__ inline int producer_record_cap(int K, int parts) {
  int want = 2 * K > 256 ? 2 * K : 256;
  if (want > PROD_CAP) want = PROD_CAP;
  const int fit = (4096 / parts) & ~1;
  if (want > fit) want = fit;
  return want > K ? want : K;
}
// Selected words (K plus ties) the merge can sort apart from the rest.
__host__ __device__ inline int producer_sel_cap(int K) {
  int c = 512;
  while (c < 2 * K && c < PROD_CAP) c <<= 1;
  return c;
}
// Candidate slots of the merge: the records of all parts, rounded up to a power of two.
__host__ __device__ inline int producer_merge_slots(int K, int parts) {
  int n2 = 64;
  while (n2 < parts * producer_record_cap(K, parts)) n2 <<= 1;
  return n2;
}
// Chunk groups per thread of the part kernel: 1024 groups per part for K <= 256, else one per chunk (4096).
__host__ __device__ inline int producer_groups(int K) { return K <= 256 ? PROD_G_SMALL : PROD_G_LARGE; }
// A (row, part) record: 16-byte header, then either the part's candidates (8 bytes each) or the largest key of
// each of its chunk groups (key_bytes each).
__host__ __device__ inline int64_t producer_part_stride(int K, int parts, int key_bytes) {
  const int64_t cands = (int64_t)producer_record_cap(K, parts) * 8, maxima = (int64_t)producer_groups(K) * PROD_NT * key_bytes;
  return 16 + (((cands > maxima ? cands : maxima) + 15) & ~15LL);
}

// ---- order-preserving keys ---------------------------------------------------------------------
// 16-bit storage types are handled as packed pairs of 16-bit keys, fp32 as 32-bit keys.
template <class Tag> struct Keys;

template <> struct Keys<TagF32> {
  typedef unsigned Stored;
  static constexpr int BITS = 32;
  static constexpr int PER_DWORD = 1;
  __device__ static __forceinline__ unsigned encode(unsigned u) {      // dword of raw bits -> dword of keys
    return u ^ ((unsigned)((int)u >> 31) | 0x80000000u);
  }
  __device__ static __forceinline__ unsigned key(unsigned kd, int) { return kd; }
  __device__ static __forceinline__ unsigned above(unsigned kd, unsigned lm1) { return kd > lm1 ? 1u : 0u; }
  __device__ static __forceinline__ unsigned dword_max(unsigned a, unsigned b) { return a > b ? a : b; }
  __device__ static __forceinline__ unsigned top_key(unsigned m) { return m; }
  __device__ static __forceinline__ float value(unsigned k) {
    const unsigned u = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
    return __uint_as_float(u);
  }
};

template <bool IS_BF16> struct Keys16 {
  typedef unsigned short Stored;
  static constexpr int BITS = 16;
  static constexpr int PER_DWORD = 2;
  __device__ static __forceinline__ unsigned encode(unsigned u) {
    const i16x2 neg = __builtin_bit_cast(i16x2, u) >> (short)15;              // 0xffff per negative half
    return u ^ (__builtin_bit_cast(unsigned, neg) | 0x80008000u);             // negative: flip all 16 bits; else the sign bit
  }
  // nonzero iff a half of kd exceeds the matching half of lm1x2 (= (L - 1) in both halves, L >= 1)
  __device__ static __forceinline__ unsigned above(unsigned kd, unsigned lm1x2) {
    const u16x2 d = __builtin_elementwise_sub_sat(__builtin_bit_cast(u16x2, kd), __builtin_bit_cast(u16x2, lm1x2));
    return __builtin_bit_cast(unsigned, d);
  }
  __device__ static __forceinline__ unsigned key(unsigned kd, int half) { return half ? (kd >> 16) : (kd & 0xffffu); }
  __device__ static __forceinline__ unsigned dword_max(unsigned a, unsigned b) {     // per 16-bit half
    const u16x2 m = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(unsigned, m);
  }
  __device__ static __forceinline__ unsigned top_key(unsigned m) { const unsigned l = m & 0xffffu, h = m >> 16; return l > h ? l : h; }
  __device__ static __forceinline__ float value(unsigned k) {
    const unsigned h = (k & 0x8000u) ? (k ^ 0x8000u) : (~k & 0xffffu);
    if (IS_BF16) return __uint_as_float(h << 16);
    return (float)__builtin_bit_cast(_Float16, (unsigned short)h);
  }
};
template <> struct Keys<TagBF16> : Keys16<true> {};
template <> struct Keys<TagF16> : Keys16<false> {};

// Sum of a per-thread integer over the workgroup; two barriers, scratch reusable at once.
template <int NT>
__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
  constexpr int NW = NT / WAVE;
  v = wave_sum(v);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  int r = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) r += scratch[i];
  __syncthreads();
  return r;
}

// Largest of a per-thread integer over the workgroup; two barriers, scratch reusable at once.
template <int NT>
__device__ __forceinline__ int block_max_int(int v, int* scratch) {
  constexpr int NW = NT / WAVE;
  v = wave_max(v);
  const int lane = threadIdx.x & (WAVE - 1), w = threadIdx.x / WAVE;
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  int r = scratch[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = max(r, scratch[i]);
  __syncthreads();
  return r;
}

// ---- candidate words -----------------------------------------------------------------------------
// A candidate is one word that sorts ascending = key descending, column ascending.  Inside a part
// the column needs 15 bits, so 16-bit keys give 31-bit words; fp32 keys need 64 bits.  The part
// record and the merge use the 64-bit form (~key in the high word, row-wide column in the low).
template <class Tag> struct Cand {
  typedef unsigned W;
  static constexpr W PAD = 0xffffffffu;
  __device__ static __forceinline__ W make(unsigned k, int col) { return ((~k & 0xffffu) << 15) | (unsigned)col; }
  __device__ static __forceinline__ u64 wide(W c, int lo) {
    return ((u64)(0xffff0000u | (c >> 15)) << 32) | (unsigned)(lo + (int)(c & 0x7fffu));
  }
};
template <> struct Cand<TagF32> {
  typedef u64 W;
  static constexpr W PAD = ~0ull;
  __device__ static __forceinline__ W make(unsigned k, int col) { return ((u64)(~k) << 32) | (unsigned)col; }
  __device__ static __forceinline__ u64 wide(W c, int lo) { return c + (unsigned)lo; }
};

// Number of entries of the part for which pred(key, column inside the part) holds.
template <class Tag, int NT, int NCH, class Pred>
__device__ __forceinline__ int count_entries(u32x4 (&reg)[NCH], int my_chunks, int* scratch, Pred pred) {
  using KY = Keys<Tag>;
  int c = 0;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    forget(reg[i]);       // the sweep is repeated in bisection loops: keep its unpacked keys from being hoisted out of them
    if (i < my_chunks) {
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int h = 0; h < KY::PER_DWORD; ++h) {
          const int col = (i * NT + (int)threadIdx.x) * Chunk<Tag>::N + d * KY::PER_DWORD + h;
          c += pred(KY::key(reg[i][d], h), col) ? 1 : 0;
        }
    }
  }
  return block_sum_int<NT>(c, scratch);
}

// Appends the entries of chunk i for which pred holds to cand (LDS); slots beyond PROD_CAP are counted, not written.
template <class Tag, int NT, int NCH, class Pred>
__device__ __forceinline__ void collect_entries(const u32x4 (&reg)[NCH], int i, typename Cand<Tag>::W* cand, int* n_cand,
                                                Pred pred) {
  using KY = Keys<Tag>;
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int h = 0; h < KY::PER_DWORD; ++h) {
      const unsigned k = KY::key(reg[i][d], h);
      const int col = (i * NT + (int)threadIdx.x) * Chunk<Tag>::N + d * KY::PER_DWORD + h;
      if (pred(k, col)) {
        const int slot = atomicAdd(n_cand, 1);
        if (slot < PROD_CAP) cand[slot] = Cand<Tag>::make(k, col);
      }
    }
}

// One wave sorts 64 * EPL words held in registers, element e = lane * EPL + j, ascending, with a
// bitonic network: strides below EPL inside a lane, the others through lane exchanges.  No barriers.
template <class W, int EPL>
__device__ __forceinline__ void wave_sort(W (&c)[EPL]) {
  const int lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int size = 2; size <= WAVE * EPL; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride < EPL) {
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
          if ((j & stride) == 0) {
            const bool up = ((lane * EPL + j) & size) == 0;
            const W a = c[j], b = c[j + stride];
            const W mn = a < b ? a : b, mx = a < b ? b : a;
            c[j] = up ? mn : mx;
            c[j + stride] = up ? mx : mn;
          }
        }
      } else {
        const int lm = stride / EPL;
        const bool lower = (lane & lm) == 0;
#pragma unroll
        for (int j = 0; j < EPL; ++j) {
          const bool up = ((lane * EPL + j) & size) == 0;
          const W o = lane_xor(c[j], lm);
          const W mn = c[j] < o ? c[j] : o, mx = c[j] < o ? o : c[j];
          c[j] = (lower == up) ? mn : mx;
        }
      }
    }
  }
}

// One wave sorts the n <= 64 * EPL candidate words of a part (LDS) and writes the best n_out to
// the part record in the 64-bit form.
template <class Tag, int EPL>
__device__ __forceinline__ void wave_sort_emit(const typename Cand<Tag>::W* cand, int n, int n_out, int lo, u64* lst) {
  typedef typename Cand<Tag>::W W;
  const int lane = threadIdx.x & (WAVE - 1);
  W c[EPL];
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane * EPL + j;
    c[j] = e < n ? cand[e] : Cand<Tag>::PAD;
  }
  wave_sort<W, EPL>(c);
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int e = lane * EPL + j;
    if (e < n_out) lst[e] = Cand<Tag>::wide(c[j], lo);
  }
}

// Logits row behind output row ro, or -1 when the caller's row list names a row outside the logits
// (negative padding entries, stale positions): such an output row is masked -- no logits are touched,
// the merge kernel fills it with -inf log-probs and id -1.
__device__ __forceinline__ int64_t producer_row(const ProducerParams& p, int64_t ro) {
  const int64_t r = p.row_list ? (int64_t)p.row_list[ro] : ro;
  return (r >= 0 && r < p.n_rows) ? r : -1;
}

// Chunk c of a part that starts at rpart and holds n_elems columns in nch chunks (beyond them: -inf).  ALIGNED: rows
// on the 16-byte grid that hold a whole number of chunks.  Otherwise only a last chunk that the row does not fill is put
// together element by element; the others come by 16-byte loads, from rows off the grid (`on_grid` false) by unaligned
// ones (which the device takes).
template <class Tag, bool ALIGNED>
__device__ __forceinline__ u32x4 producer_load_chunk(const char* rpart, int c, int nch, int n_elems, bool on_grid) {
  using C = Chunk<Tag>;
  if constexpr (ALIGNED) {
    return c < nch ? load16_stream(rpart + (int64_t)c * 16) : C::neg_inf();
  } else {
    const bool whole = (c + 1) * C::N <= n_elems;
    return c >= nch ? C::neg_inf()
           : !whole ? load_chunk_elementwise<Tag>(rpart, c, n_elems)
           : on_grid ? load16_stream(rpart + (int64_t)c * 16) : load16_unaligned(rpart + (int64_t)c * 16);
  }
}

constexpr int PART_FULL = 0;    // threshold, candidates and record of the part: all the part kernel's stages
constexpr int PART_LIGHT = 1;   // statistics and chunk-group maxima only: the candidates are picked per row (topk_select_kernel)
constexpr int PART_REDO = 2;    // PART_FULL for the rows the row-level selection handed back

// G = chunk groups per thread whose maxima feed the threshold search: 256 * G groups per part must
// be a few times K for the candidate set to stay close to K (4 for K <= 256, else 16).
// ALIGNED: rows start on 16-byte boundaries and hold a whole number of chunks (16-byte loads);
// otherwise the chunks are assembled element by element and the last one is padded with -inf,
// which the collection leaves out (a padding entry has the lowest key and the highest columns of
// its part, so the threshold searches, which only count, need no such test).
template <class Tag, int G, bool ALIGNED, int MODE>
__device__ __forceinline__ void topk_part(const ProducerParams& p, int64_t ro, int h_part) {
  constexpr int NT = PROD_NT, NCH = PROD_NCH, NW = NT / WAVE, CPG = NCH / G;
  using C = Chunk<Tag>;
  using KY = Keys<Tag>;
  typedef typename Cand<Tag>::W W;
  __shared__ float red[64];
  __shared__ int ired[NW];
  __shared__ int slots[2 * NW];
  __shared__ int s_n;
  __shared__ unsigned s_L;
  __shared__ __align__(16) W cand[PROD_CAP];      // before the collection: the group maxima (G == 4)

  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), w = tid / WAVE;
  const int P = p.parts;
  const int64_t r = producer_row(p, ro);
  if (r < 0) return;                                                 // masked output row: the merge kernel fills it
  const int64_t c0 = (int64_t)h_part * NT * NCH;
  const int lo = (int)(c0 * C::N);
  const int n_elems = (int)min((int64_t)NT * NCH * C::N, p.V - lo);  // columns of this part, >= 1
  const int nch = (n_elems + C::N - 1) / C::N;                       // its chunks (the last one padded unless ALIGNED)
  const int Kp = min(p.K, n_elems);
  const char* rpart = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes + c0 * 16;
  char* rec = p.ws + (ro * P + h_part) * p.part_stride;
  // single-wave stages rotate over the waves (and so over the SIMDs) from workgroup to workgroup
  const int select_wave = (int)((blockIdx.x >> 3) & (NW - 1));

  u32x4 reg[NCH];
  const bool on_grid = (reinterpret_cast<uintptr_t>(rpart) & 15) == 0;      // the same for the whole workgroup
#pragma unroll
  for (int i = 0; i < NCH; ++i) reg[i] = producer_load_chunk<Tag, ALIGNED>(rpart, i * NT + tid, nch, n_elems, on_grid);
  if (tid == 0) s_n = 0;

  if constexpr (MODE == PART_LIGHT) {
    // Statistics and the largest key of every chunk group, nothing else, and no barrier before the end: every
    // thread sums its exponentials against the largest of its own 64 entries, which it knows from the chunk keys it
    // makes anyway; the workgroup's maximum and the rescaled sums are combined once at the end.
    // A group is what the selection reads again: with four chunks per group, the chunks that four neighbouring
    // threads hold in the same register (64 contiguous bytes of the row: one access); the group's maximum is taken
    // across the quad.  One chunk per group: the thread's own.
    typedef typename KY::Stored KS;
    KS* gout = reinterpret_cast<KS*>(rec + 16);
    const int mine = (nch - tid + NT - 1) / NT;                       // chunks i < mine are inside the part
    unsigned tk = 0u;                                                 // largest key of the thread (0: none)
    unsigned gk[NCH];                                                 // group maxima; stored at the end: a store between the
                                                                      // loads' waits would make each of them a wait for everything
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      unsigned e[4];
#pragma unroll
      for (int d = 0; d < 4; ++d) e[d] = KY::encode(reg[i][d]);
      unsigned k = i < mine ? KY::top_key(KY::dword_max(KY::dword_max(e[0], e[1]), KY::dword_max(e[2], e[3]))) : 0u;
      tk = max(tk, k);
      if constexpr (CPG == 4) {
        k = max(k, (unsigned)dpp_move<DPP_QUAD_XOR1>((int)k, (int)k));
        k = max(k, (unsigned)dpp_move<DPP_QUAD_XOR2>((int)k, (int)k));
      } else {
        static_assert(CPG == 1 || CPG == 4, "chunk groups: a thread's chunk, or a quad's four");
      }
      gk[i] = k;
    }
    const float mt = tk ? KY::value(tk) : -INFINITY;
    const float mbt = (mt == -INFINITY) ? 0.f : mt * LOG2E;
    float st = 0.f;
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      float f[C::N];
      forget(reg[i]);
      C::unpack(reg[i], f);
#pragma unroll
      for (int e = 0; e < C::N; ++e) st += fast_exp2(fmaf(f[e], LOG2E, -mbt));
    }
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if constexpr (CPG == 4) {
        if ((tid & 3) == (i & 3)) gout[i * (NT / 4) + (tid >> 2)] = (KS)gk[i];
      } else {
        gout[i * NT + tid] = (KS)gk[i];
      }
    }
    const float M = block_max<NT>(mt, red);
    st = (mt == -INFINITY) ? 0.f : st * fast_exp2((mt - M) * LOG2E);
    st = block_sum<NT>(st, red);
    if (tid == 0) {
      PartHeader hd{M, st, -1, 0};
      *reinterpret_cast<PartHeader*>(rec) = hd;
    }
    return;
  }
  // max and sum-exp of the part (natural log-softmax; no temperature at collection time)
  float mx = -INFINITY;
  bool have_max = false;
  if constexpr (Tag::bytes == 2) {
    // Non-negative 16-bit floats order like their bit patterns read as signed integers, and every
    // negative one reads as a negative integer: the packed integer maximum of the raw pairs is the
    // row maximum whenever that is not negative (half an instruction per element instead of two).
    i16x2 pm = {(short)-32768, (short)-32768};
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      forget(reg[i]);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned w16 = reg[i][d];      // by value: a bit cast straight from a vector element reads element 0
        pm = __builtin_elementwise_max(pm, __builtin_bit_cast(i16x2, w16));
      }
    }
    const int top = block_max_int<NT>(max((int)pm.x, (int)pm.y), ired);
    if (top >= 0) {
      mx = Tag::id == BF16 ? __uint_as_float((unsigned)top << 16) : (float)__builtin_bit_cast(_Float16, (unsigned short)top);
      have_max = true;
    }
  }
  if (!have_max) {                        // the same for every thread
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      float f[C::N];
      forget(reg[i]);
      C::unpack(reg[i], f);
#pragma unroll
      for (int e = 0; e < C::N; ++e) mx = fmaxf(mx, f[e]);
    }
    mx = block_max<NT>(mx, red);
  }
  const float mb = (mx == -INFINITY) ? 0.f : mx * LOG2E;
  float sm = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    float f[C::N];
    forget(reg[i]);
    C::unpack(reg[i], f);
#pragma unroll
    for (int e = 0; e < C::N; ++e) sm += fast_exp2(fmaf(f[e], LOG2E, -mb));
  }
  sm = block_sum<NT>(sm, red);

  const int my_chunks = (nch - tid + NT - 1) / NT;                  // chunks i < my_chunks are inside the part
  // raw bits -> ordered keys, in place; largest key of every chunk group
  unsigned gm[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    unsigned m = 0u;
#pragma unroll
    for (int j = 0; j < CPG; ++j) {
      const int i = g * CPG + j;
      forget(reg[i]);
#pragma unroll
      for (int d = 0; d < 4; ++d) reg[i][d] = KY::encode(reg[i][d]);
      const unsigned mc = KY::dword_max(KY::dword_max(reg[i][0], reg[i][1]), KY::dword_max(reg[i][2], reg[i][3]));
      m = KY::dword_max(m, i < my_chunks ? mc : 0u);
    }
    gm[g] = KY::top_key(m);
  }
  // groups that hold at least one chunk of the part: thread tid's group g starts at chunk (g * CPG) * NT + tid
  int n_groups = 0;
#pragma unroll
  for (int g = 0; g < G; ++g) n_groups += max(0, min(NT, nch - g * CPG * NT));

  // L = Kp-th largest group maximum, found bit by bit (0 when the part has fewer groups than Kp)
  unsigned L = 0;
  if (n_groups >= Kp) {
    if constexpr (G * NT == 1024) {
      // one wave searches all 1024 maxima from its registers: no barrier per bit
      unsigned* gms = reinterpret_cast<unsigned*>(cand);
#pragma unroll
      for (int g = 0; g < G; ++g) gms[g * NT + tid] = gm[g];
      __syncthreads();
      if (w == select_wave) {
        unsigned v[G * NW];
#pragma unroll
        for (int j = 0; j < G * NW; ++j) v[j] = gms[j * WAVE + lane];
        // the answer nearly always shares the top 6 bits of the largest key: try that prefix first
        unsigned top = 0u;
#pragma unroll
        for (int j = 0; j < G * NW; ++j) top = max(top, v[j]);
        top = wave_max(top);
        const unsigned pre = top & ~((1u << (KY::BITS - 6)) - 1u);
        int cpre = 0;
#pragma unroll
        for (int j = 0; j < G * NW; ++j) cpre += __popcll(__ballot(v[j] >= pre));
        unsigned Lw = cpre >= Kp ? pre : 0u;
        int b = cpre >= Kp ? KY::BITS - 7 : KY::BITS - 1;
#pragma unroll 1
        for (; b >= 0; --b) {
          const unsigned t = Lw | (1u << b);
          int c = 0;
#pragma unroll
          for (int j = 0; j < G * NW; ++j) c += __popcll(__ballot(v[j] >= t));
          if (c >= Kp) Lw = t;
        }
        if (lane == 0) s_L = Lw;
      }
      __syncthreads();
      L = s_L;
    } else {
#pragma unroll 1
      for (int b = KY::BITS - 1; b >= 0; --b) {
        const unsigned t = L | (1u << b);
        int c = 0;
#pragma unroll
        for (int g = 0; g < G; ++g) c += __popcll(__ballot(gm[g] >= t));
        int* sl = slots + (b & 1) * NW;
        if (lane == 0) sl[w] = c;
        __syncthreads();
        int tot = 0;
#pragma unroll
        for (int j = 0; j < NW; ++j) tot += sl[j];
        if (tot >= Kp) L = t;
      }
      __syncthreads();
    }
  }

  // entries at or above L; the group maxima tell which groups hold any, a packed test which dwords
  if (L == 0) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (i < my_chunks)
        collect_entries<Tag, NT, NCH>(reg, i, cand, &s_n, [n_elems](unsigned, int col) { return ALIGNED || col < n_elems; });
    }
  } else {
    const unsigned lm1 = KY::PER_DWORD == 2 ? (L - 1) * 0x00010001u : L - 1;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (gm[g] >= L) {
#pragma unroll
        for (int j = 0; j < CPG; ++j) {
          const int i = g * CPG + j;
          if (i < my_chunks) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              if (KY::above(reg[i][d], lm1)) {
#pragma unroll
                for (int h = 0; h < KY::PER_DWORD; ++h) {
                  const unsigned k = KY::key(reg[i][d], h);
                  const int col = (i * NT + tid) * C::N + d * KY::PER_DWORD + h;
                  if (k >= L && (ALIGNED || col < n_elems)) {
                    const int slot = atomicAdd(&s_n, 1);
                    if (slot < PROD_CAP) cand[slot] = Cand<Tag>::make(k, col);
                  }
                }
              }
            }
          }
        }
      }
    }
  }
  __syncthreads();
  int n = s_n;

  if (n > PROD_CAP) {
    // exact select: T = Kp-th largest key by bisection over key bits, then the smallest columns among its ties
    unsigned T = 0;
#pragma unroll 1
    for (int b = KY::BITS - 1; b >= 0; --b) {
      const unsigned t = T | (1u << b);
      if (count_entries<Tag, NT, NCH>(reg, my_chunks, ired, [t](unsigned k, int) { return k >= t; }) >= Kp) T = t;
    }
    const int n_gt = count_entries<Tag, NT, NCH>(reg, my_chunks, ired, [T](unsigned k, int) { return k > T; });
    const int need = Kp - n_gt;                                     // >= 1 ties to take
    int clo = 0, chi = n_elems - 1;                                 // smallest column bound with `need` ties at or below it
    while (clo < chi) {
      const int mid = clo + (chi - clo) / 2;
      const int cnt = count_entries<Tag, NT, NCH>(reg, my_chunks, ired,
                                                  [T, mid](unsigned k, int col) { return k == T && col <= mid; });
      if (cnt >= need) chi = mid; else clo = mid + 1;
    }
    if (tid == 0) s_n = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (i < my_chunks)
        collect_entries<Tag, NT, NCH>(reg, i, cand, &s_n,
                                      [T, clo, n_elems](unsigned k, int col) {
                                        return (k > T || (k == T && col <= clo)) && (ALIGNED || col < n_elems);
                                      });
    }
    __syncthreads();
    n = s_n;                                                        // == Kp
  }

  // ---- hand the candidates over; sort and cut to the best Kp only if the record cannot hold them all
  const int capw = producer_record_cap(p.K, P);
  const int n_keep = n <= capw ? n : Kp;
  if (tid == 0) {
    PartHeader hd{mx, sm, n_keep, 0};
    *reinterpret_cast<PartHeader*>(rec) = hd;
  }
  u64* lst = reinterpret_cast<u64*>(rec + 16);
  if (n <= capw) {
    for (int a = tid; a < n; a += NT) lst[a] = Cand<Tag>::wide(cand[a], lo);
  } else if (n <= WAVE * 8) {
    if (w == select_wave) wave_sort_emit<Tag, 8>(cand, n, Kp, lo, lst);
  } else {
    int n2 = 1024;
    while (n2 < n) n2 <<= 1;
    for (int a = n + tid; a < n2; a += NT) cand[a] = Cand<Tag>::PAD;
    __syncthreads();
    for (int size = 2; size <= n2; size <<= 1) {
      for (int stride = size >> 1; stride > 0; stride >>= 1) {
        for (int t = tid; t < n2 / 2; t += NT) {
          const int lo_i = 2 * t - (t & (stride - 1)), hi_i = lo_i + stride;
          const bool up = (lo_i & size) == 0;
          const W a = cand[lo_i], b = cand[hi_i];
          if ((a > b) == up) { cand[lo_i] = b; cand[hi_i] = a; }
        }
        __syncthreads();
      }
    }
    for (int k = tid; k < Kp; k += NT) lst[k] = Cand<Tag>::wide(cand[k], lo);
  }
}

// Workgroup ids are dealt round-robin to the 8 XCDs: within a group of 8 * P ids, id t serves row (or, PART_REDO,
// entry of the list of rows handed back) 8 * group + t % 8, part t / 8, so the parts of a row run on one XCD back to
// back.  PART_REDO: a small grid whose workgroups walk the list, which is empty as a rule.
template <class Tag, int G, bool ALIGNED, int MODE>
__global__ __launch_bounds__(PROD_NT) __attribute__((amdgpu_waves_per_eu(PROD_NT / 64, 8)))
void topk_part_kernel(const ProducerParams p) {
  const unsigned P = (unsigned)p.parts;
  const unsigned grp = blockIdx.x / (8u * P), t_in = blockIdx.x % (8u * P);
  const int64_t slot = (int64_t)grp * 8 + (t_in & 7u);
  const int h_part = (int)(t_in >> 3);
  if constexpr (MODE == PART_REDO) {
    const int64_t n = min((int64_t)*p.redo_count, p.n_out), step = (int64_t)(gridDim.x / (8u * P)) * 8;
    for (int64_t e = slot; e < n; e += step) {
      topk_part<Tag, G, ALIGNED, MODE>(p, p.redo_rows[e], h_part);
      __syncthreads();                                               // the next row reuses the workgroup's LDS
    }
  } else {
    if (slot >= p.n_out) return;
    if (MODE == PART_LIGHT && blockIdx.x == 0 && threadIdx.x == 0) *p.redo_count = 0u;      // the selection, the next launch, appends to the list
    topk_part<Tag, G, ALIGNED, MODE>(p, slot, h_part);
  }
}

// Emits sorted words [0, K) held as element e = lane * EPL + j of one wave.
template <class Tag, int EPL>
__device__ __forceinline__ void emit_sorted(const ProducerParams& p, int64_t ro, float lse, const u64 (&c)[EPL]) {
  const int lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int k = lane * EPL + j;
    if (k < p.K) {
      const float logp = Keys<Tag>::value(~(unsigned)(c[j] >> 32)) - lse;
      const int col = (int)(unsigned)c[j];
      store_from_float(p.out_val, p.out_dtype, ro * p.K + k, logp);
      if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * p.K + k] = col;
      else reinterpret_cast<int64_t*>(p.out_idx)[ro * p.K + k] = col;
    }
  }
}

// The same for narrow words (16-bit keys that share their leading bits `prefix`): the complement of the key's low
// TAIL bits above CB bits of column.
template <class Tag, int EPL>
__device__ __forceinline__ void emit_sorted_narrow(const ProducerParams& p, int64_t ro, float lse, const unsigned (&c)[EPL],
                                                   unsigned prefix, int tail, int cb) {
  const int lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int j = 0; j < EPL; ++j) {
    const int k = lane * EPL + j;
    if (k < p.K) {
      const unsigned key = prefix | (~(c[j] >> cb) & ((1u << tail) - 1u));
      const float logp = Keys<Tag>::value(key) - lse;
      const int col = (int)(c[j] & ((1u << cb) - 1u));
      store_from_float(p.out_val, p.out_dtype, ro * p.K + k, logp);
      if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * p.K + k] = col;
      else reinterpret_cast<int64_t*>(p.out_idx)[ro * p.K + k] = col;
    }
  }
}

// The K best of `total` candidate words (LDS) to the output row.  Words sort ascending = key descending, column
// ascending, and no two are equal (the column is part of the word).  The K-th smallest high word (= K-th
// largest key) is found bit by bit; the words at or below it (K plus ties) are compacted and sorted by one wave in
// registers.  More than 512 of them (a tie plateau): everything is sorted in LDS instead.  256 threads, all of
// them; s_nsel zero and `all` complete behind a barrier on entry.
struct SelectLds { int slots[2 * 4]; unsigned best[4]; int nsel; };
template <class Tag>
__device__ __forceinline__ void select_and_emit(const ProducerParams& p, int64_t ro, float lse, u64* all, u64* sel, int total,
                                                int sel_cap, SelectLds& sh) {
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), w = tid / WAVE;
  const int K = p.K;
  int* slots = sh.slots;
  unsigned* s_best = sh.best;
  int& s_nsel = sh.nsel;
  if (total <= 512) {            // few enough for one wave's registers: sorted as they are (the same for every thread)
    if (w == 0) {
      if (total <= 256) {
        u64 c[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = lane * 4 + j < total ? all[lane * 4 + j] : ~0ull;
        wave_sort<u64, 4>(c);
        emit_sorted<Tag, 4>(p, ro, lse, c);
      } else {
        u64 c[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) c[j] = lane * 8 + j < total ? all[lane * 8 + j] : ~0ull;
        wave_sort<u64, 8>(c);
        emit_sorted<Tag, 8>(p, ro, lse, c);
      }
    }
    return;
  }
  // U = smallest high word with at least K words at or below it; only the low Keys::BITS bits vary.
  // Counting is ballot + popcount per wave, one barrier per probe; the first probe tries the six
  // leading bits of the best word, which the K-th almost always shares.
  constexpr int BITS = Keys<Tag>::BITS;
  const int trips = (total + 255) / 256;
  int probe = 0;
  auto count_le = [&](unsigned bound) {
    int c = 0;
    for (int it = 0; it < trips; ++it) {
      const int a = it * 256 + tid;
      c += __popcll(__ballot(a < total && (unsigned)(all[a < total ? a : 0] >> 32) <= bound));
    }
    int* sl = slots + (probe++ & 1) * 4;
    if (lane == 0) sl[w] = c;
    __syncthreads();
    return sl[0] + sl[1] + sl[2] + sl[3];
  };
  unsigned best = 0xffffffffu;
  for (int a = tid; a < total; a += 256) best = min(best, (unsigned)(all[a] >> 32));
  best = wave_min(best);
  if (lane == 0) s_best[w] = best;
  __syncthreads();
  best = min(min(s_best[0], s_best[1]), min(s_best[2], s_best[3]));
  const unsigned low = (1u << (BITS - 6)) - 1u;
  unsigned U = BITS == 32 ? 0u : 0xffff0000u;
  int b = BITS - 1;
  if (count_le(best | low) >= K) { U = best & ~low; b = BITS - 7; }
#pragma unroll 1
  for (; b >= 0; --b) {
    if (count_le(U | ((1u << b) - 1u)) < K) U |= 1u << b;          // probe with bit b left at zero
  }
  for (int a = tid; a < total; a += 256) {
    const u64 v = all[a];
    if ((unsigned)(v >> 32) <= U) {
      const int slot = atomicAdd(&s_nsel, 1);
      if (slot < sel_cap) sel[slot] = v;
    }
  }
  __syncthreads();
  const int n_sel = s_nsel;                                         // >= K when the parts delivered K or more
  if (n_sel <= 256) {
    if (w == 0) {
      u64 c[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) c[j] = lane * 4 + j < n_sel ? sel[lane * 4 + j] : ~0ull;
      wave_sort<u64, 4>(c);
      emit_sorted<Tag, 4>(p, ro, lse, c);
    }
    return;
  }
  if (n_sel <= 512) {
    if (w == 0) {
      u64 c[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) c[j] = lane * 8 + j < n_sel ? sel[lane * 8 + j] : ~0ull;
      wave_sort<u64, 8>(c);
      emit_sorted<Tag, 8>(p, ro, lse, c);
    }
    return;
  }
  // LDS bitonic sort: of the selected words if they fit their list, else (a tie plateau) of everything
  u64* arr = n_sel <= sel_cap ? sel : all;
  const int n_arr = n_sel <= sel_cap ? n_sel : total;
  int n2 = 64;
  while (n2 < n_arr) n2 <<= 1;
  for (int a = n_arr + tid; a < n2; a += 256) arr[a] = ~0ull;
  __syncthreads();
  for (int size = 2; size <= n2; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = tid; t < n2 / 2; t += 256) {
        const int lo_i = 2 * t - (t & (stride - 1)), hi_i = lo_i + stride;
        const bool up = (lo_i & size) == 0;
        const u64 a = arr[lo_i], b = arr[hi_i];
        if ((a > b) == up) { arr[lo_i] = b; arr[hi_i] = a; }
      }
      __syncthreads();
    }
  }
  for (int k = tid; k < K; k += 256) {
    const u64 a = arr[k];
    const float logp = Keys<Tag>::value(~(unsigned)(a >> 32)) - lse;
    const int col = (int)(unsigned)a;
    store_from_float(p.out_val, p.out_dtype, ro * K + k, logp);
    if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * K + k] = col;
    else reinterpret_cast<int64_t*>(p.out_idx)[ro * K + k] = col;
  }
}

// Merge of the parts of one row: log-sum-exp from the part statistics, and the K best of the parts'
// candidates (select_and_emit).  REDO: only the rows on the list of rows handed back.
template <class Tag, bool REDO>
__device__ __forceinline__ void topk_merge_row(const ProducerParams& p, int64_t redo_entry) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  u64* all = reinterpret_cast<u64*>(smem_raw);                      // the parts' records; producer_merge_slots words
  __shared__ SelectLds sh;
  const int tid = threadIdx.x;
  const int P = p.parts, K = p.K;
  int64_t ro = blockIdx.x;
  if constexpr (REDO) {                       // launched as workgroups of one round; see topk_merge_redo_kernel
    ro = p.redo_rows[redo_entry];
  }
  const int capw = producer_record_cap(K, P);
  const int sel_cap = producer_sel_cap(K);
  u64* sel = all + producer_merge_slots(K, P);                      // the selected words; sel_cap words
  const char* rec0 = p.ws + ro * P * p.part_stride;
  if (producer_row(p, ro) < 0) {                                    // the row list names no logits row: masked output row
    for (int k = tid; k < K; k += 256) {
      store_from_float(p.out_val, p.out_dtype, ro * K + k, -INFINITY);
      if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * K + k] = -1;
      else reinterpret_cast<int64_t*>(p.out_idx)[ro * K + k] = -1;
    }
    return;
  }

  float M = -INFINITY;
  for (int q = 0; q < P; ++q) M = fmaxf(M, reinterpret_cast<const PartHeader*>(rec0 + q * p.part_stride)->mx);
  float S = 0.f;
  int total = 0;
  for (int q = 0; q < P; ++q) {
    const PartHeader hd = *reinterpret_cast<const PartHeader*>(rec0 + q * p.part_stride);
    if (hd.mx != -INFINITY) S += hd.sm * fast_exp2((hd.mx - M) * LOG2E);
    const int cnt = min(max(hd.cnt, 0), capw);
    const u64* lst = reinterpret_cast<const u64*>(rec0 + q * p.part_stride + 16);
    for (int j = tid; j < cnt; j += 256) all[total + j] = lst[j];
    total += cnt;
  }
  const float lse = (M * LOG2E + fast_log2(S)) * LN2;
  if (tid == 0) sh.nsel = 0;
  __syncthreads();
  select_and_emit<Tag>(p, ro, lse, all, sel, total, sel_cap, sh);
}

template <class Tag>
__global__ __launch_bounds__(256) void topk_merge_kernel(const ProducerParams p) { topk_merge_row<Tag, false>(p, 0); }
// The rows handed back: a small grid whose workgroups walk the list.
template <class Tag>
__global__ __launch_bounds__(256) void topk_merge_redo_kernel(const ProducerParams p) {
  const int64_t n = min((int64_t)*p.redo_count, p.n_out);
  for (int64_t e = blockIdx.x; e < n; e += gridDim.x) {
    topk_merge_row<Tag, true>(p, e);
    __syncthreads();
  }
}

// ---- row-level selection behind the light part kernel ----------------------------------------------
// Candidate words the selection keeps in LDS, and chunk groups it opens, for a given K; a row with more (a tie
// plateau, a constant row) is handed back to the part kernel's own, exact selection.
__host__ __device__ inline int producer_select_cands(int K) {
  int c = 1024;
  while (c < 4 * K) c <<= 1;
  return c;
}
__host__ __device__ inline int producer_select_groups(int K) { return 2 * K > 512 ? 2 * K : 512; }
// Dynamic LDS of topk_select_kernel: the group maxima of all parts, later the candidate words; the selected
// words; the list of groups to open.
__host__ __device__ inline size_t producer_select_lds(int K, int parts, int key_bytes) {
  const size_t maxima = (size_t)parts * producer_groups(K) * PROD_NT * key_bytes, cands = (size_t)producer_select_cands(K) * 8;
  return ((maxima > cands ? maxima : cands) + 15) / 16 * 16 + (size_t)producer_sel_cap(K) * 8 + (size_t)producer_select_groups(K) * 4;
}

// One workgroup per output row.  The K-th largest of the row's chunk-group maxima, L, is a lower bound of the
// row's K-th largest key (K groups reach it, so K entries do), so every entry of the best K -- ties at the K-th
// key included -- lies in a group whose maximum reaches L.  Those groups (about K of them, out of thousands) are read
// again from the logits, the entries at or above L become the candidate words, and select_and_emit picks the best K.
// Against thresholds per part this opens a quarter of the groups when a row has four parts, and the part kernel,
// bound by vector-ALU issue, sheds its collection stage (a third of its instructions) for 20 % more bytes fetched.
// MAXR > 0: the group maxima stay in the threads' registers (MAXR rounds of 16 bytes per thread: every pass over them
// then costs no LDS access and no address arithmetic); MAXR == 0: any number of them, in LDS.
template <class Tag, int G, bool ALIGNED, int MAXR>
__global__ __launch_bounds__(256) void topk_select_kernel(const ProducerParams p) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  using KY = Keys<Tag>;
  using C = Chunk<Tag>;
  typedef typename KY::Stored KS;
  constexpr int NT = PROD_NT, NCH = PROD_NCH, CPG = NCH / G, GPP = G * NT;      // chunks per group, groups per part
  __shared__ SelectLds sh;
  __shared__ int s_sum[2 * 4];
  __shared__ int s_nq, s_total;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1), w = tid / WAVE;
  const int64_t ro = blockIdx.x;
  const int P = p.parts, K = p.K;
  const int n_g = P * GPP;
  const int acap = producer_select_cands(K), qcap = producer_select_groups(K), sel_cap = producer_sel_cap(K);
  const size_t region = (((size_t)n_g * sizeof(KS) > (size_t)acap * 8 ? (size_t)n_g * sizeof(KS) : (size_t)acap * 8) + 15) / 16 * 16;
  KS* gmax = reinterpret_cast<KS*>(smem_raw);
  u64* all = reinterpret_cast<u64*>(smem_raw);                      // takes the place of the maxima
  unsigned* all32 = reinterpret_cast<unsigned*>(smem_raw);          // the same list in narrow words
  u64* sel = reinterpret_cast<u64*>(smem_raw + region);
  int* glist = reinterpret_cast<int*>(smem_raw + region + (size_t)sel_cap * 8);
  const int64_t r = producer_row(p, ro);
  if (r < 0) {                                                      // the row list names no logits row: masked output row
    for (int k = tid; k < K; k += 256) {
      store_from_float(p.out_val, p.out_dtype, ro * K + k, -INFINITY);
      if (p.out_itype == I32) reinterpret_cast<int32_t*>(p.out_idx)[ro * K + k] = -1;
      else reinterpret_cast<int64_t*>(p.out_idx)[ro * K + k] = -1;
    }
    return;
  }
  const char* rec0 = p.ws + ro * P * p.part_stride;
  // all loads of the row's records first: the headers of the parts, then the group maxima
  PartHeader hd[PROD_MAX_PARTS];
#pragma unroll
  for (int q = 0; q < PROD_MAX_PARTS; ++q)
    hd[q] = *reinterpret_cast<const PartHeader*>(rec0 + (q < P ? q : 0) * p.part_stride);
  constexpr int KPL = 16 / (int)sizeof(KS), DW = KY::PER_DWORD;      // maxima per 16 bytes, per dword
  u32x4 mreg[MAXR > 0 ? MAXR : 1];
  if constexpr (MAXR > 0) {
#pragma unroll
    for (int rr = 0; rr < MAXR; ++rr) {
      const int a0 = (rr * 256 + tid) * KPL;                          // groups a0 .. a0 + KPL - 1: one part's (GPP is a multiple of KPL)
      mreg[rr] = u32x4{0u, 0u, 0u, 0u};                               // key 0: below every threshold but 0, which hands the row back
      if (a0 < n_g)
        mreg[rr] = *reinterpret_cast<const u32x4*>(rec0 + (int64_t)(a0 / GPP) * p.part_stride + 16 + (size_t)(a0 % GPP) * sizeof(KS));
    }
  } else {
    constexpr int RND = 16;
    for (int a0 = 0; a0 < n_g; a0 += RND * 256) {
      KS v[RND];
#pragma unroll
      for (int j = 0; j < RND; ++j) {
        const int a = a0 + j * 256 + tid, aa = a < n_g ? a : 0;
        v[j] = reinterpret_cast<const KS*>(rec0 + (aa / GPP) * p.part_stride + 16)[aa % GPP];
      }
#pragma unroll
      for (int j = 0; j < RND; ++j) {
        const int a = a0 + j * 256 + tid;
        if (a < n_g) gmax[a] = v[j];
      }
    }
  }
  // the row's log-sum-exp from the parts' statistics: worked out where it is used, by the threads that emit
  const auto row_lse = [&]() {
    float M = -INFINITY;
#pragma unroll
    for (int q = 0; q < PROD_MAX_PARTS; ++q) M = fmaxf(M, q < P ? hd[q].mx : -INFINITY);
    float S = 0.f;
#pragma unroll
    for (int q = 0; q < PROD_MAX_PARTS; ++q)
      if (q < P && hd[q].mx != -INFINITY) S += hd[q].sm * fast_exp2((hd[q].mx - M) * LOG2E);
    return (M * LOG2E + fast_log2(S)) * LN2;
  };
  int* hist = reinterpret_cast<int*>(sel);                          // 256 counters, in the list of selected words (unused so far)
  if (tid == 0) { s_nq = 0; s_total = 0; sh.nsel = 0; }
  hist[tid] = 0;
  __syncthreads();

  // Candidate words of 32 bits where the keys have 16 and the bound comes from the histogram step: every candidate then
  // shares the six leading bits of the largest maximum, so 10 key bits and 22 bits of column tell the words apart,
  // and the wave that sorts them moves and compares half as many registers.
  constexpr int TAIL_BITS = KY::BITS - 6, COL_BITS = 32 - TAIL_BITS;
  bool narrow = false;
  unsigned key_prefix = 0u;
  unsigned L = 0;
  if constexpr (MAXR > 0) {
    // every thread's maxima: `visit(key, group)` for each of them
    const auto for_keys = [&](auto visit) {
#pragma unroll
      for (int rr = 0; rr < MAXR; ++rr)
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int h = 0; h < DW; ++h) visit(KY::key(mreg[rr][d], h), (rr * 256 + tid) * KPL + d * DW + h);
    };
    int probe = 0;
    const auto count_ge = [&](unsigned t) {
      int c = 0;
      for_keys([&](unsigned k, int) { c += k >= t ? 1 : 0; });
      c = wave_sum(c);
      int* sl = s_sum + (probe++ & 1) * 4;
      if (lane == 0) sl[w] = c;
      __syncthreads();
      return sl[0] + sl[1] + sl[2] + sl[3];
    };
    unsigned dm = 0u;
#pragma unroll
    for (int rr = 0; rr < MAXR; ++rr)
#pragma unroll
      for (int d = 0; d < 4; ++d) dm = KY::dword_max(dm, mreg[rr][d]);
    unsigned top = wave_max(KY::top_key(dm));
    if (lane == 0) sh.best[w] = top;
    __syncthreads();
    top = max(max(sh.best[0], sh.best[1]), max(sh.best[2], sh.best[3]));
    constexpr int TAIL = KY::BITS - 6;                                // bits below the prefix
    const unsigned prefix = top & ~((1u << TAIL) - 1u);
    // histogram of the next eight bits of the maxima that share the prefix (prefix 0: the padding keys would count);
    // should fewer than K of them share it, no bin is found and the bisection below takes over
    bool found = false;
    if (prefix != 0u) {
      constexpr int SH = TAIL - 8;
      for_keys([&](unsigned k, int) { if (k >= prefix) atomicAdd(&hist[(k >> SH) & 255u], 1); });
      __syncthreads();
      if (w == 0) {
        int c[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = hist[lane * 4 + j];
        const int mine = c[0] + c[1] + c[2] + c[3];
        int incl = mine;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
          const int t = __shfl_up(incl, o, WAVE);
          incl += lane >= o ? t : 0;
        }
        const int sharing = __shfl(incl, WAVE - 1, WAVE);
        const int above = sharing - incl;
        int run = above, bin = -1;
#pragma unroll
        for (int j = 3; j >= 0; --j) {
          if (bin < 0 && run + c[j] >= K && run < K) bin = lane * 4 + j;
          run += c[j];
        }
        if (lane == 0 && sharing < K) s_sum[0] = -1;
        if (bin >= 0) s_sum[0] = bin;                                 // exactly one lane finds it when K or more share the prefix
      }
      __syncthreads();
      const int bin = s_sum[0];
      __syncthreads();
      if (bin >= 0) {
        L = prefix | ((unsigned)bin << SH);
        narrow = KY::BITS == 16 && p.V <= (1ll << COL_BITS);
        key_prefix = prefix;
        found = true;
      }
    }
    if (!found) {
#pragma unroll 1
      for (int b = KY::BITS - 1; b >= 0; --b) {
        const unsigned t = L | (1u << b);
        if (count_ge(t) >= K) L = t;
      }
    }
    if (L != 0u)
      for_keys([&](unsigned k, int a) {
        if (k >= L) {
          const int slot = atomicAdd(&s_nq, 1);
          if (slot < qcap) glist[slot] = a;
        }
      });
  } else {
    // L: a lower bound of the K-th largest group maximum, as tight as a few steps make it.  (Any bound at or below the
    // K-th largest key of the row gives the same result; a looser one costs candidates.)
    int probe = 0;
    const auto count_ge = [&](unsigned t) {
      int c = 0;
      for (int a = tid; a < n_g; a += 256) c += (unsigned)gmax[a] >= t ? 1 : 0;
      c = wave_sum(c);
      int* sl = s_sum + (probe++ & 1) * 4;
      if (lane == 0) sl[w] = c;
      __syncthreads();
      return sl[0] + sl[1] + sl[2] + sl[3];
    };
    // the answer nearly always shares the six leading bits of the largest maximum
    unsigned top = 0u;
    for (int a = tid; a < n_g; a += 256) top = max(top, (unsigned)gmax[a]);
    top = wave_max(top);
    if (lane == 0) sh.best[w] = top;
    __syncthreads();
    top = max(max(sh.best[0], sh.best[1]), max(sh.best[2], sh.best[3]));
    constexpr int TAIL = KY::BITS - 6;                                // bits below the prefix
    const unsigned prefix = top & ~((1u << TAIL) - 1u);
    if (count_ge(prefix) >= K) {
      // histogram of the next eight bits of the maxima that share the prefix; the bin that holds the K-th largest,
      // counted from the top, gives eight more bits of L (its lowest key: at most the bins' width below the true one)
      constexpr int SH = TAIL - 8;
      for (int a = tid; a < n_g; a += 256) {
        const unsigned v = (unsigned)gmax[a];
        if (v >= prefix) atomicAdd(&hist[(v >> SH) & 255u], 1);
      }
      __syncthreads();
      if (w == 0) {
        // lane l holds bins 4l .. 4l + 3; suffix sums from the top bin down
        int c[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) c[j] = hist[lane * 4 + j];
        const int mine = c[0] + c[1] + c[2] + c[3];
        int incl = mine;                                               // inclusive scan over the lanes
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
          const int t = __shfl_up(incl, o, WAVE);
          incl += lane >= o ? t : 0;
        }
        const int above = __shfl(incl, WAVE - 1, WAVE) - incl;         // entries in the bins of the lanes above this one
        int run = above, bin = -1;
#pragma unroll
        for (int j = 3; j >= 0; --j) {
          if (bin < 0 && run + c[j] >= K && run < K) bin = lane * 4 + j;
          run += c[j];
        }
        if (bin >= 0) s_sum[0] = bin;                                 // exactly one lane finds it
      }
      __syncthreads();
      L = prefix | ((unsigned)s_sum[0] << SH);
      narrow = KY::BITS == 16 && p.V <= (1ll << COL_BITS);
      key_prefix = prefix;
      __syncthreads();
    } else {
#pragma unroll 1
      for (int b = KY::BITS - 1; b >= 0; --b) {
        const unsigned t = L | (1u << b);
        if (count_ge(t) >= K) L = t;
      }
    }
    // the groups to open
    for (int a = tid; a < n_g; a += 256) {
      if ((unsigned)gmax[a] >= L) {
        const int slot = atomicAdd(&s_nq, 1);
        if (slot < qcap) glist[slot] = a;
      }
    }
  }
  __syncthreads();                                                  // the maxima are done with: their LDS takes the candidates
  const int n_q = s_nq;
  bool redo = n_q > qcap || L == 0;                                 // L == 0: fewer than K groups hold anything; the part kernel's own selection takes every entry then
  if (!redo) {
    const char* row = reinterpret_cast<const char*>(p.logits) + r * p.row_stride * Tag::bytes;
    // four chunks per thread and round: their loads are in flight together
    constexpr int U = 4;
    for (int idx0 = 0; idx0 < n_q * CPG; idx0 += U * 256) {
      u32x4 v[U];
      int base[U], left[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int idx = idx0 + u * 256 + tid;
        base[u] = 0;
        left[u] = 0;                                                // columns of the part from the chunk's first on: 0 = nothing to test
        v[u] = C::neg_inf();
        if constexpr (ALIGNED) {
          // whole chunks on the grid: the chunk's number in the row gives address and column; a chunk that is not
          // there reads as keys of 0, below every L
          v[u] = u32x4{~0u, ~0u, ~0u, ~0u};
          left[u] = C::N;
          if (idx < n_q * CPG) {
            const int a = glist[idx / CPG], j = idx % CPG;
            const int q = a / GPP, gi = a % GPP;
            const unsigned c = (unsigned)q * (NT * NCH) + (CPG == 4 ? (gi / (NT / 4)) * NT + 4 * (gi % (NT / 4)) + j : gi);
            base[u] = (int)(c * C::N);
            if ((int64_t)base[u] < p.V) v[u] = load16_stream(row + (uint64_t)c * 16);
          }
        } else if (idx < n_q * CPG) {
          const int a = glist[idx / CPG], j = idx % CPG;
          const int q = a / GPP, gi = a % GPP;
          // chunk of the part: the j-th of the quad's four neighbours, or the thread's own
          const int c = CPG == 4 ? (gi / (NT / 4)) * NT + 4 * (gi % (NT / 4)) + j : gi;
          const int64_t c0 = (int64_t)q * NT * NCH;
          const int lo = (int)(c0 * C::N);
          const int n_elems = (int)min((int64_t)NT * NCH * C::N, p.V - lo);
          const int nch = (n_elems + C::N - 1) / C::N;
          const char* rpart = row + c0 * 16;
          v[u] = producer_load_chunk<Tag, ALIGNED>(rpart, c, nch, n_elems, (reinterpret_cast<uintptr_t>(rpart) & 15) == 0);
          base[u] = lo + c * C::N;
          left[u] = n_elems - c * C::N;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const unsigned kd = KY::encode(v[u][d]);
#pragma unroll
          for (int h = 0; h < KY::PER_DWORD; ++h) {
            const unsigned k = KY::key(kd, h);
            const int e = d * KY::PER_DWORD + h;
            if (k >= L && (ALIGNED || e < left[u])) {
              const int slot = atomicAdd(&s_total, 1);
              if (slot < acap) {
                if (narrow) all32[slot] = ((~k & ((1u << TAIL_BITS) - 1u)) << COL_BITS) | (unsigned)(base[u] + e);
                else all[slot] = ((u64)(KY::BITS == 32 ? ~k : (0xffff0000u | (~k & 0xffffu))) << 32) | (unsigned)(base[u] + e);
              }
            }
          }
        }
      }
    }
    __syncthreads();
    redo = s_total > acap;
  }
  if (redo) {                                                       // the same for every thread
    if (tid == 0) p.redo_rows[atomicAdd(p.redo_count, 1u)] = (int32_t)ro;
    return;
  }
  const int total = s_total;
  if (KY::BITS == 16 && narrow) {
    if (total <= 512) {                                             // the rule: one wave sorts the narrow words as they are
      if (w == 0) {
        const float lse = row_lse();
        if (total <= 256) {
          unsigned c[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) c[j] = lane * 4 + j < total ? all32[lane * 4 + j] : ~0u;
          wave_sort<unsigned, 4>(c);
          emit_sorted_narrow<Tag, 4>(p, ro, lse, c, key_prefix, TAIL_BITS, COL_BITS);
        } else {
          unsigned c[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) c[j] = lane * 8 + j < total ? all32[lane * 8 + j] : ~0u;
          wave_sort<unsigned, 8>(c);
          emit_sorted_narrow<Tag, 8>(p, ro, lse, c, key_prefix, TAIL_BITS, COL_BITS);
        }
      }
      return;
    }
    // more of them (a tie plateau): widened in place, through registers, for the general selection
    constexpr int PER = (4 * PROD_MAX_K + 255) / 256;                // acap <= 4 * PROD_MAX_K
    unsigned wv[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) wv[j] = j * 256 + tid < total ? all32[j * 256 + tid] : 0u;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (j * 256 + tid < total) {
        const unsigned key = key_prefix | (~(wv[j] >> COL_BITS) & ((1u << TAIL_BITS) - 1u));
        all[j * 256 + tid] = ((u64)(0xffff0000u | (~key & 0xffffu)) << 32) | (wv[j] & ((1u << COL_BITS) - 1u));
      }
    __syncthreads();
  }
  select_and_emit<Tag>(p, ro, row_lse(), all, sel, total, sel_cap, sh);
}

static int producer_parts(int64_t V, int logits_dtype) {
  const int epc = logits_dtype == DL_F32 ? 4 : 8;
  const int64_t nch = (V + epc - 1) / epc;
  return (int)((nch + PROD_NT * PROD_NCH - 1) / (PROD_NT * PROD_NCH));
}

template <class Tag, int G, bool ALIGNED>
static void launch_producer_shape(const ProducerParams& p, hipStream_t st) {
  const dim3 grid((unsigned)((p.n_out + 7) / 8 * 8 * p.parts));
  const size_t lds_merge = (size_t)(producer_merge_slots(p.K, p.parts) + producer_sel_cap(p.K)) * 8;      // <= 48 KiB
  const size_t lds_select = producer_select_lds(p.K, p.parts, Tag::bytes == 4 ? 4 : 2);
  // chunk groups of a row that hold anything: with fewer than 4 K of them the group maxima bound the K-th key too
  // loosely (or not at all) for opening groups a second time to pay
  const int64_t chunks = (p.V + Chunk<Tag>::N - 1) / Chunk<Tag>::N, groups = (chunks + (PROD_NCH / G) - 1) / (PROD_NCH / G);
  if (lds_select > 64 * 1024 || groups < 4 * (int64_t)p.K) {      // (or too many groups for the selection's LDS): thresholds per part
    hipLaunchKernelGGL((topk_part_kernel<Tag, G, ALIGNED, PART_FULL>), grid, dim3(PROD_NT), 0, st, p);
    hipLaunchKernelGGL((topk_merge_kernel<Tag>), dim3((unsigned)p.n_out), dim3(256), lds_merge, st, p);
    return;
  }
  hipLaunchKernelGGL((topk_part_kernel<Tag, G, ALIGNED, PART_LIGHT>), grid, dim3(PROD_NT), 0, st, p);
  // the maxima of a row in the selection's registers where four rounds of 16 bytes per thread hold them
  if ((size_t)p.parts * G * PROD_NT * sizeof(typename Keys<Tag>::Stored) <= (size_t)4 * 256 * 16)
    hipLaunchKernelGGL((topk_select_kernel<Tag, G, ALIGNED, 4>), dim3((unsigned)p.n_out), dim3(256), lds_select, st, p);
  else
    hipLaunchKernelGGL((topk_select_kernel<Tag, G, ALIGNED, 0>), dim3((unsigned)p.n_out), dim3(256), lds_select, st, p);
  // the rows handed back (none, as a rule: the workgroups then leave at once)
  const unsigned redo_rows = (unsigned)std::min<int64_t>((p.n_out + 7) / 8 * 8, 256);
  hipLaunchKernelGGL((topk_part_kernel<Tag, G, ALIGNED, PART_REDO>), dim3(redo_rows * p.parts), dim3(PROD_NT), 0, st, p);
  hipLaunchKernelGGL((topk_merge_redo_kernel<Tag>), dim3(redo_rows), dim3(256), lds_merge, st, p);
}

template <class Tag>
static int launch_producer(const ProducerParams& p, bool aligned, hipStream_t st) {
  static bool lds_allowed = false;
  if (!lds_allowed) {
    // (up to 64 KiB of dynamic LDS for the selection: above the default limit of a launch)
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&topk_select_kernel<Tag, PROD_G_SMALL, true, 0>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&topk_select_kernel<Tag, PROD_G_SMALL, false, 0>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&topk_select_kernel<Tag, PROD_G_LARGE, true, 0>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&topk_select_kernel<Tag, PROD_G_LARGE, false, 0>), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    lds_allowed = true;
  }
  if (aligned) {
    if (p.K <= 256) launch_producer_shape<Tag, PROD_G_SMALL, true>(p, st);
    else launch_producer_shape<Tag, PROD_G_LARGE, true>(p, st);
  } else {
    if (p.K <= 256) launch_producer_shape<Tag, PROD_G_SMALL, false>(p, st);
    else launch_producer_shape<Tag, PROD_G_LARGE, false>(p, st);
  }
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

}  // namespace dl

extern "C" int64_t dl_teacher_topk_workspace_bytes(int logits_dtype, int64_t n_out, int64_t V, int K) {
  if (n_out <= 0 || V <= 0 || K <= 0) return 0;
  const int parts = dl::producer_parts(V, logits_dtype);
  if (parts > dl::PROD_MAX_PARTS || K > dl::PROD_MAX_K || (int64_t)parts * K > 4096) return 0;
  const int64_t records = n_out * parts * dl::producer_part_stride(K, parts, logits_dtype == DL_F32 ? 4 : 2);
  return records + 16 + ((n_out * 4 + 15) & ~15LL);                 // then the counter and the list of rows handed back
}

extern "C" int dl_teacher_topk(const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows, int64_t V,
                               const int32_t* row_list, int64_t n_out, int K, void* out_val, int out_dtype,
                               void* out_idx, int out_itype, void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace dl;
  if (!logits || !out_val || !out_idx) return DL_ERR_NULL;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || (out_dtype != DL_F32 && out_dtype != DL_F16) ||
      (out_itype != DL_I32 && out_itype != DL_I64))
    return DL_ERR_DTYPE;
  if (n_rows < 0 || n_out < 0 || V <= 0 || K <= 0 || K > V || row_stride < V || (!row_list && n_out > n_rows))
    return DL_ERR_SHAPE;
  const int parts = producer_parts(V, logits_dtype);
  if (K > PROD_MAX_K || parts > PROD_MAX_PARTS || (int64_t)parts * K > 4096 || V > 0x7fffffffLL ||
      n_out * parts > 0x7fffffffLL)
    return DL_ERR_LIMIT;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(logits) % eb != 0) return DL_ERR_ALIGN;
  const bool aligned = V % (16 / eb) == 0 && reinterpret_cast<uintptr_t>(logits) % 16 == 0 && (row_stride * eb) % 16 == 0;
  if (n_out == 0) return DL_OK;
  if (!workspace) return DL_ERR_NULL;
  if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0) return DL_ERR_ALIGN;
  if (workspace_bytes < dl_teacher_topk_workspace_bytes(logits_dtype, n_out, V, K)) return DL_ERR_WORKSPACE;
  const int64_t stride = producer_part_stride(K, parts, eb == 4 ? 4 : 2);
  char* redo = reinterpret_cast<char*>(workspace) + n_out * parts * stride;
  ProducerParams p{logits, row_stride, n_rows, V, row_list, n_out, K, parts, reinterpret_cast<char*>(workspace),
                   stride, out_val, out_dtype, out_idx, out_itype, reinterpret_cast<unsigned*>(redo),
                   reinterpret_cast<int32_t*>(redo + 16)};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  return logits_dtype == DL_F32 ? launch_producer<TagF32>(p, aligned, st)
         : logits_dtype == DL_BF16 ? launch_producer<TagBF16>(p, aligned, st)
                                   : launch_producer<TagF16>(p, aligned, st);
}
