// Stage 1, streaming kernels for the interleaved layouts.
//
// A row of n elements with b interleaved buckets is the row-major matrix
// [L = n / b sub-rows][b columns] plus a last partial sub-row of n mod b
// elements; bucket c is column c.  The job is a column-wise top-J.
//
// Mapping.  Every lane owns V adjacent columns (V*sizeof(T) = 16 bytes when the
// addresses allow it, else V = 1), so one wave64 load instruction reads 64*V
// adjacent elements of one sub-row (1 KiB with 16-byte loads) and the wave walks
// down the sub-rows.  The J-entry queue of each owned column lives in
// registers: values in compare form plus the sub-row number they came from; the
// position in the row, c + p*b, is formed only when results are written.
//
// Work split.  A workgroup of W waves owns one column tile (64*V columns) over
// one slab of sub-rows; each wave scans 1/W of the slab and waves 1..W-1 hand
// their queues to wave 0 through LDS.  Many short-lived waves keep far more of
// the HBM bandwidth than few long-lived ones on this part, and the merge is a
// handful of register operations.  Very long rows are additionally cut into
// `slabs` along the grid; then the per-slab queues go to a workspace and
// `stream_merge_kernel` folds them.
//
// Few buckets.  When the buckets do not fill one column tile, `fold`
// consecutive sub-rows are scanned side by side as one sub-row of a matrix with
// b*fold columns, so that every lane loads; a bucket then owns `fold` columns,
// whose queues are merged under the full order (value, then lower index) by
// the scanning workgroup (`fold_columns`) or by the merge kernel.
//
// Queues.  `CmpQueue` holds values in compare form and sub-row numbers;
// `PackedQueue` (16-bit element types) and `ByteQueue` (8-bit ones) pack an
// entry into one 32-bit word, order key above inverted sub-row number, so that
// unsigned max/min/med3 insert it with the right tie rule.  Register arrays are indexed by compile-time
// constants only (ATK_STATIC_FOR): run-time indices make the compiler keep the
// queues in scratch memory.
//
// Order.  Sub-rows are visited in increasing position and a newcomer displaces
// an entry only when it compares strictly greater, so equal values keep the
// lowest index.  Floating-point columns compare with the hardware's IEEE `>`
// (-0.0 == +0.0); a NaN makes that compare meaningless, so every load is also
// tested for NaN and a wave (or workgroup) that saw one recomputes its tile
// with the exact integer order keys of atk_device.h.
#pragma once

#include <type_traits>
#include <utility>

#include "atk_device.h"
#include "atk_launch.h"
#include "atk_trace.h"
#include "stage2_select.h"

namespace atk {
namespace stream {

constexpr int kWave = 64;

// Columns per lane with vector loads: 16 bytes' worth, but at most 8 columns so
// that the queues of one lane stay in registers.
__host__ __device__ constexpr int full_vec(int elem_size) { return elem_size == 1 ? 8 : 16 / elem_size; }

// LDS a workgroup of `waves` needs to hand the queues of waves 1.. to wave 0,
// and the most the planner lets it use.
// `entry_bytes`: a queue entry as handed over (the packed queues: one 32-bit word;
// else the value in compare form and the sub-row number).
__host__ __device__ constexpr size_t merge_lds_bytes(int vec, int j, int waves, int entry_bytes) {
  return (size_t)(waves - 1) * vec * j * kWave * entry_bytes;
}
constexpr size_t kMergeLdsLimit = 48 * 1024;
// Packed 16-bit queues may take more: eight waves of four entries over eight
// columns a lane (56 KiB; two workgroups per CU, which is what their registers
// allow anyway).
constexpr size_t kMergeLdsLimitPacked = 56 * 1024;
__host__ __device__ constexpr size_t merge_lds_limit(int entry_bytes) {
  return entry_bytes == 4 ? kMergeLdsLimitPacked : kMergeLdsLimit;
}

// Compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// `ATK_STATIC_FOR(i, N) { body };` runs body with i = 0..N-1 as compile-time
// constants.  Register-resident arrays are only ever indexed this way: an index
// that is a loop variable until late unrolling keeps the arrays in scratch.
#define ATK_STATIC_FOR(i, N) \
  ::atk::stream::static_for<(N)>([&](auto i##_c) __attribute__((always_inline)) { \
    constexpr int i = decltype(i##_c)::value;
#define ATK_STATIC_END })

// ---------------------------------------------------------------------------
// Compare form of an element type: what the queues hold in the hot loop.
// ---------------------------------------------------------------------------
template <typename E> struct Cmp;

template <> struct Cmp<Elem<ATK_F32>> {
  using cmp_t = float; static constexpr bool has_nan = true;
  __device__ static __forceinline__ cmp_t from_raw(uint32_t u) { return __uint_as_float(u); }
  __device__ static __forceinline__ uint32_t to_raw(cmp_t v) { return __float_as_uint(v); }
};
template <> struct Cmp<Elem<ATK_F16>> {
  using cmp_t = float; static constexpr bool has_nan = true;
  __device__ static __forceinline__ cmp_t from_raw(uint16_t u) {
    _Float16 h; __builtin_memcpy(&h, &u, 2); return (float)h;
  }
  __device__ static __forceinline__ uint16_t to_raw(cmp_t v) {
    _Float16 h = (_Float16)v; uint16_t u; __builtin_memcpy(&u, &h, 2); return u;
  }
};
template <> struct Cmp<Elem<ATK_BF16>> {
  using cmp_t = float; static constexpr bool has_nan = true;
  __device__ static __forceinline__ cmp_t from_raw(uint16_t u) { return __uint_as_float((uint32_t)u << 16); }
  __device__ static __forceinline__ uint16_t to_raw(cmp_t v) { return (uint16_t)(__float_as_uint(v) >> 16); }
};
template <> struct Cmp<Elem<ATK_F64>> {
  using cmp_t = double; static constexpr bool has_nan = true;
  __device__ static __forceinline__ cmp_t from_raw(uint64_t u) { return __longlong_as_double((long long)u); }
  __device__ static __forceinline__ uint64_t to_raw(cmp_t v) { return (uint64_t)__double_as_longlong(v); }
};
template <> struct Cmp<Elem<ATK_U8>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static __forceinline__ cmp_t from_raw(uint8_t u) { return (int)u; }
  __device__ static __forceinline__ uint8_t to_raw(cmp_t v) { return (uint8_t)v; }
};
template <> struct Cmp<Elem<ATK_I8>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static __forceinline__ cmp_t from_raw(uint8_t u) { return (int)(int8_t)u; }
  __device__ static __forceinline__ uint8_t to_raw(cmp_t v) { return (uint8_t)v; }
};
template <> struct Cmp<Elem<ATK_I16>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static __forceinline__ cmp_t from_raw(uint16_t u) { return (int)(int16_t)u; }
  __device__ static __forceinline__ uint16_t to_raw(cmp_t v) { return (uint16_t)v; }
};
template <> struct Cmp<Elem<ATK_I32>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static __forceinline__ cmp_t from_raw(uint32_t u) { return (int)u; }
  __device__ static __forceinline__ uint32_t to_raw(cmp_t v) { return (uint32_t)v; }
};
template <> struct Cmp<Elem<ATK_I64>> {
  using cmp_t = long long; static constexpr bool has_nan = false;
  __device__ static __forceinline__ cmp_t from_raw(uint64_t u) { return (long long)u; }
  __device__ static __forceinline__ uint64_t to_raw(cmp_t v) { return (uint64_t)v; }
};

// V elements moved by one load instruction.
template <typename raw_t, int V> struct alignas(sizeof(raw_t) * V) Pack { raw_t e[V]; };

template <typename raw_t, int V>
__device__ __forceinline__ Pack<raw_t, V> load_pack(const raw_t* p) {
  return *reinterpret_cast<const Pack<raw_t, V>*>(p);
}

// ---------------------------------------------------------------------------
// Queue of J entries per column, ascending (slot 0 weakest).  FILLED top slots
// are valid; the lower ones count as beaten by anything.
// ---------------------------------------------------------------------------
template <typename T, int J, int FILLED = J>
__device__ __forceinline__ void push(T (&q)[J], uint32_t (&pos)[J], T v, uint32_t p) {
  bool beats[J + 1];
  ATK_STATIC_FOR(s, J) { beats[s] = (s < J - FILLED) ? true : (v > q[s]); } ATK_STATIC_END;
  beats[J] = false;
  ATK_STATIC_FOR(s, J) {
    constexpr int up = (s + 1 < J) ? s + 1 : s;
    q[s] = beats[s + 1] ? q[up] : (beats[s] ? v : q[s]);
    pos[s] = beats[s + 1] ? pos[up] : (beats[s] ? p : pos[s]);
  } ATK_STATIC_END;
}

// The same under the full order (value, then lower sub-row number), for
// newcomers that do not arrive in increasing sub-row order.
template <typename T, int J>
__device__ __forceinline__ void push_ordered(T (&q)[J], uint32_t (&pos)[J], T v, uint32_t p) {
  bool beats[J + 1];
  ATK_STATIC_FOR(s, J) { beats[s] = v > q[s] || (v == q[s] && p < pos[s]); } ATK_STATIC_END;
  beats[J] = false;
  ATK_STATIC_FOR(s, J) {
    constexpr int up = (s + 1 < J) ? s + 1 : s;
    q[s] = beats[s + 1] ? q[up] : (beats[s] ? v : q[s]);
    pos[s] = beats[s + 1] ? pos[up] : (beats[s] ? p : pos[s]);
  } ATK_STATIC_END;
}

// Exact (order-key) push used off the hot path; entries hold raw elements and
// an entry whose sub-row number is kEmptySlot is empty (beaten by anything).
constexpr uint32_t kEmptySlot = 0xffffffffu;

template <typename E, int J>
__device__ __forceinline__ void clear_exact(typename E::raw_t (&q)[J], uint32_t (&pos)[J]) {
  ATK_STATIC_FOR(s, J) { q[s] = 0; pos[s] = kEmptySlot; } ATK_STATIC_END;
}

template <typename E, int J>
__device__ __forceinline__ void push_exact(typename E::raw_t (&q)[J], uint32_t (&pos)[J], typename E::raw_t v,
                                  uint32_t p) {
  const typename E::key_t kv = E::key(v);
  bool beats[J + 1];
  ATK_STATIC_FOR(s, J) { beats[s] = pos[s] == kEmptySlot || kv > E::key(q[s]); } ATK_STATIC_END;
  beats[J] = false;
  ATK_STATIC_FOR(s, J) {
    constexpr int up = (s + 1 < J) ? s + 1 : s;
    q[s] = beats[s + 1] ? q[up] : (beats[s] ? v : q[s]);
    pos[s] = beats[s + 1] ? pos[up] : (beats[s] ? p : pos[s]);
  } ATK_STATIC_END;
}

// ---------------------------------------------------------------------------
// Queue policies: the per-lane state of V columns x J entries and how a loaded
// pack of V elements is folded into it.
// ---------------------------------------------------------------------------

// General form: values in compare form plus the sub-row number of each entry.
template <typename E, int J, int V> struct CmpQueue {
  using raw_t = typename E::raw_t;
  using C = Cmp<E>;
  using cmp_t = typename C::cmp_t;
  // LDS one wave needs to hand its queues to another: [V*J][64] values, then positions
  static constexpr size_t kHandBytes = (size_t)V * J * kWave * (sizeof(cmp_t) + 4);

  cmp_t q[V][J];
  uint32_t pos[V][J];
  uint64_t nan_mask;  // lanes that loaded a NaN; wave-uniform

  __device__ __forceinline__ void reset() { nan_mask = 0; }
  __device__ __forceinline__ void set_position_shift(uint32_t) {}
  // low bits of sel_key that are the same in every entry
  __device__ __forceinline__ int sel_constant_bits() const { return 0; }

  // FILLED: how many entries every column already holds (the first J sub-rows fill the queues)
  template <int FILLED> __device__ __forceinline__ void take(const Pack<raw_t, V>& pk, uint32_t p) {
    cmp_t c[V];
    ATK_STATIC_FOR(v, V) { c[v] = C::from_raw(pk.e[v]); } ATK_STATIC_END;
    if constexpr (C::has_nan) {
      ATK_STATIC_FOR(h, V / 2) { nan_mask |= __ballot(__builtin_isunordered(c[2 * h], c[2 * h + 1])); } ATK_STATIC_END;
      if constexpr (V % 2 != 0) nan_mask |= __ballot(__builtin_isunordered(c[V - 1], c[V - 1]));
    }
    ATK_STATIC_FOR(v, V) { push<cmp_t, J, FILLED>(q[v], pos[v], c[v], p); } ATK_STATIC_END;
  }
  // elements of sub-rows p and p + 1 of column VI
  template <int VI, int FILLED> __device__ __forceinline__ void take_two(raw_t a, raw_t b, uint32_t p) {
    const cmp_t ca = C::from_raw(a), cb = C::from_raw(b);
    if constexpr (C::has_nan) nan_mask |= __ballot(__builtin_isunordered(ca, cb));
    push<cmp_t, J, FILLED>(q[VI], pos[VI], ca, p);
    push<cmp_t, J, (FILLED < J ? FILLED + 1 : J)>(q[VI], pos[VI], cb, p + 1);
  }
  // one more element for column VI of a full queue, when `valid`
  template <int VI> __device__ __forceinline__ void take_one(raw_t raw, uint32_t p, bool valid) {
    const cmp_t c = C::from_raw(raw);
    if constexpr (C::has_nan) nan_mask |= __ballot(valid && __builtin_isunordered(c, c));
    bool beats[J + 1];
    ATK_STATIC_FOR(s, J) { beats[s] = valid && (c > q[VI][s]); } ATK_STATIC_END;
    beats[J] = false;
    ATK_STATIC_FOR(s, J) {
      constexpr int up = (s + 1 < J) ? s + 1 : s;
      q[VI][s] = beats[s + 1] ? q[VI][up] : (beats[s] ? c : q[VI][s]);
      pos[VI][s] = beats[s + 1] ? pos[VI][up] : (beats[s] ? p : pos[VI][s]);
    } ATK_STATIC_END;
  }
  // a NaN was loaded: the queues are meaningless (wave-uniform)
  __device__ __forceinline__ bool poisoned() const { return C::has_nan && nan_mask != 0; }

  __device__ __forceinline__ void hand_over(unsigned char* area, uint32_t lane) const {
    cmp_t* hq = reinterpret_cast<cmp_t*>(area);
    uint32_t* hp = reinterpret_cast<uint32_t*>(area + (size_t)V * J * kWave * sizeof(cmp_t));
    ATK_STATIC_FOR(e, V * J) {
      hq[e * kWave + lane] = q[e / J][e % J];
      hp[e * kWave + lane] = pos[e / J][e % J];
    } ATK_STATIC_END;
  }
  // Folds in the queues a later wave (higher sub-rows) handed over, best entry
  // first, so that equal values keep the lowest index.
  __device__ __forceinline__ void fold_in(const unsigned char* area, uint32_t lane) {
    const cmp_t* hq = reinterpret_cast<const cmp_t*>(area);
    const uint32_t* hp = reinterpret_cast<const uint32_t*>(area + (size_t)V * J * kWave * sizeof(cmp_t));
    ATK_STATIC_FOR(v, V) {
      ATK_STATIC_FOR(r, J) {
        constexpr int s = J - 1 - r;
        push<cmp_t, J, J>(q[v], pos[v], hq[(v * J + s) * kWave + lane], hp[(v * J + s) * kWave + lane]);
      } ATK_STATIC_END;
    } ATK_STATIC_END;
  }
  // The same for queues of a wave whose sub-rows interleave with this wave's
  // (both hold J entries of distinct sub-rows): the full order decides.
  __device__ __forceinline__ void fold_in_interleaved(const unsigned char* area, uint32_t lane) {
    const cmp_t* hq = reinterpret_cast<const cmp_t*>(area);
    const uint32_t* hp = reinterpret_cast<const uint32_t*>(area + (size_t)V * J * kWave * sizeof(cmp_t));
    ATK_STATIC_FOR(v, V) {
      ATK_STATIC_FOR(sl, J) {
        push_ordered<cmp_t, J>(q[v], pos[v], hq[(v * J + sl) * kWave + lane], hp[(v * J + sl) * kWave + lane]);
      } ATK_STATIC_END;
    } ATK_STATIC_END;
  }
  __device__ __forceinline__ void fix_zeros(const raw_t* __restrict__, int64_t, int64_t, int64_t = 1) {}
  // exact order key of an entry (the queues are not poisoned)
  template <int VI, int SI> __device__ __forceinline__ typename E::key_t key() const { return E::key(C::to_raw(q[VI][SI])); }
  // A key cheap to get from an entry whose order is the selection order as far
  // as it goes: entries with different sel_key rank by it, entries with equal
  // sel_key by their index (lower first).
  using sel_t = typename E::key_t;
  static constexpr int sel_bits = E::key_bits;
  template <int VI, int SI> __device__ __forceinline__ sel_t sel_key() const { return key<VI, SI>(); }
  // An entry as two 32-bit words for a hand-over that is undone elsewhere
  // (elements of at most four bytes, sub-row numbers and columns below 65536):
  // what `unstage` needs to give back the element and where it came from.
  template <int VI, int SI> __device__ __forceinline__ uint2 staged(uint32_t column) const {
    return make_uint2((uint32_t)C::to_raw(q[VI][SI]), (pos[VI][SI] << 16) | column);
  }
  struct Unstaged { raw_t raw; uint32_t sub_row, column; bool reread; };  // reread: take the element from the row
  __device__ __forceinline__ Unstaged unstage(uint2 w) const {
    return Unstaged{(raw_t)w.x, w.y >> 16, w.y & 0xffffu, false};
  }
  template <int VI, int SI> __device__ __forceinline__ raw_t raw() const { return C::to_raw(q[VI][SI]); }
  template <int VI, int SI> __device__ __forceinline__ uint32_t position() const { return pos[VI][SI]; }
};

// Packed form for 16-bit element types and rows of fewer than 65535 sub-rows:
// one 32-bit word per entry, the element's 16-bit order key in the high half
// and 0xFFFF - sub-row in the low half.  Words of one column are distinct and
// their unsigned order is the selection order (equal values: lower sub-row =
// larger word), so a push is J-1 v_med3_u32 and one v_max_u32, two halves are
// keyed per instruction, and 0 serves as the empty entry.
//
// Floating-point keys: a non-negative half h keys as h | 0x8000, a negative
// one as -h (16-bit), which orders all non-NaN values and gives -0.0 the key of
// +0.0, as the exact order key does.  Two things are handled on the side: the
// key of a zero no longer tells -0.0 from +0.0, so entries that end up in the
// result with a zero key are re-read from the input (`fix_zeros`); and a NaN
// would key low, so loads are screened for NaN (max |h| per half) and a tile
// that saw one is recomputed exactly.
template <typename E> struct PackedKey { static constexpr bool available = false; };

typedef short atk_short2 __attribute__((ext_vector_type(2)));
typedef unsigned short atk_ushort2 __attribute__((ext_vector_type(2)));

template <uint16_t INF> struct PackedKeyFloat16 {
  static constexpr bool available = true;
  static constexpr bool zero_is_ambiguous = true;
  static constexpr uint32_t kZeroKey = 0x8000u;
  // two raw halves -> two keys; `screen` accumulates max |h| per half
  __device__ static __forceinline__ uint32_t keys2(uint32_t x, uint32_t& screen) {
    const atk_ushort2 xv = __builtin_bit_cast(atk_ushort2, x);
    const uint32_t sign = __builtin_bit_cast(uint32_t, __builtin_bit_cast(atk_short2, x) >> 15);  // 0xFFFF per negative half
    const uint32_t negated = __builtin_bit_cast(uint32_t, (atk_ushort2)(0) - xv);
    screen = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(
                 __builtin_bit_cast(atk_ushort2, screen), __builtin_bit_cast(atk_ushort2, x & 0x7fff7fffu)));
    return (sign & negated) | (~sign & (x ^ 0x80008000u));
  }
  __device__ static __forceinline__ bool special(uint32_t screen) {
    return (screen & 0xffffu) > INF || (screen >> 16) > INF;
  }
  // The same keys in three operations instead of four, with a screen of one
  // operation instead of two: `screen` accumulates the unsigned max of the raw
  // halves, which finds the NaNs with the sign bit set (they would key below
  // -inf and vanish); a NaN without it keys above +inf, stays at the head of its
  // column's queue whatever else arrives, and is looked for there when the scan
  // is over (nan_key).  (In the one-kernel path, which is held to 64 registers,
  // this form was measured slower: it keeps the four-operation one.)
  __device__ static __forceinline__ uint32_t keys2_lean(uint32_t x, uint32_t& screen) {
    const uint32_t sign = __builtin_bit_cast(uint32_t, __builtin_bit_cast(atk_short2, x) >> 15);  // 0xFFFF per negative half
    screen = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(
                 __builtin_bit_cast(atk_ushort2, screen), __builtin_bit_cast(atk_ushort2, x)));
    // h ^ 0x8000, or ~h + 1 = -h under the sign: one three-input bit operation, one packed subtract of -1 per negative half
    const uint32_t flipped = x ^ (sign | 0x80008000u);
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(atk_ushort2, flipped) - __builtin_bit_cast(atk_ushort2, sign));
  }
  __device__ static __forceinline__ bool special_lean(uint32_t screen) {
    return (screen & 0xffffu) > (0x8000u | INF) || (screen >> 16) > (0x8000u | INF);
  }
  __device__ static __forceinline__ bool nan_key(uint32_t key) { return key > (0x8000u | INF); }
  // the raw half of a key; a zero key gives +0.0
  __device__ static __forceinline__ uint16_t unkey(uint32_t key) {
    return (uint16_t)((key & 0x8000u) ? (key ^ 0x8000u) : (0u - key));
  }
  // the element's order key as atk_device.h defines it: negative values key one
  // lower there (-h - 1: the complement), which leaves a gap below the zeros
  __device__ static __forceinline__ uint32_t exact(uint32_t key) { return key - ((key >> 15) ^ 1u); }
};
template <> struct PackedKey<Elem<ATK_F16>> : PackedKeyFloat16<0x7c00u> {};
template <> struct PackedKey<Elem<ATK_BF16>> : PackedKeyFloat16<0x7f80u> {};
template <> struct PackedKey<Elem<ATK_I16>> {
  static constexpr bool available = true;
  static constexpr bool zero_is_ambiguous = false;
  static constexpr uint32_t kZeroKey = 0x8000u;
  __device__ static __forceinline__ uint32_t keys2(uint32_t x, uint32_t&) { return x ^ 0x80008000u; }
  __device__ static __forceinline__ bool special(uint32_t) { return false; }
  __device__ static __forceinline__ uint32_t keys2_lean(uint32_t x, uint32_t&) { return x ^ 0x80008000u; }
  __device__ static __forceinline__ bool special_lean(uint32_t) { return false; }
  __device__ static __forceinline__ bool nan_key(uint32_t) { return false; }
  __device__ static __forceinline__ uint16_t unkey(uint32_t key) { return (uint16_t)(key ^ 0x8000u); }
  __device__ static __forceinline__ uint32_t exact(uint32_t key) { return key; }
};

// largest sub-row number (the partial sub-row included) a packed entry can hold
constexpr uint32_t kPackedMaxSubRow = 0xfffeu;

// Inserts an entry word into a column's ascending words: the median of
// (col[s], word, col[s+1]) is the new col[s].
__device__ __forceinline__ uint32_t med3_u32(uint32_t a, uint32_t b, uint32_t c) {
  uint32_t r;
  asm("v_med3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
// FILLED: entries the column is known to hold already (they are its last ones,
// the others are the empty word 0, below every entry): the slots below them
// need no work.
template <int J, int FILLED = J> __device__ __forceinline__ void insert_word(uint32_t (&col)[J], uint32_t word) {
  ATK_STATIC_FOR(s, J - 1) {
    if constexpr (s + 1 + FILLED >= J) {
      if constexpr (s + 1 + FILLED == J) col[s] = col[s + 1] < word ? col[s + 1] : word;  // med3 with an empty col[s]
      else col[s] = med3_u32(col[s], word, col[s + 1]);
    }
  } ATK_STATIC_END;
  if constexpr (FILLED == 0) col[J - 1] = word;
  else col[J - 1] = col[J - 1] > word ? col[J - 1] : word;
}

// LEAN: the three-operation keys and the shorter first inserts (see keys2_lean).
template <typename E, int J, int V, bool SHIFTED = false, bool LEAN = !SHIFTED> struct PackedQueue {
  using raw_t = typename E::raw_t;
  using K = PackedKey<E>;
  static_assert(sizeof(raw_t) == 2 && (V % 2 == 0 || V == 1), "packed queues hold 16-bit elements");
  static constexpr size_t kHandBytes = (size_t)V * J * kWave * 4;

  uint32_t q[V][J];
  uint32_t screen;     // NaN screen, two halves
  uint32_t neg_zeros;  // bit v*J+s: entry (v, s) is a -0.0 (set by fix_zeros)
  // The low half of an entry holds 0xffff - sub-row, or, SHIFTED, that value
  // shifted left by `pshift` within the half: when sub-row numbers need only
  // 16 - pshift bits, this puts every bit in which the entries of a run differ
  // at the top of the word (wave-uniform; SHIFTED = false keeps no such member).
  struct None {};
  [[no_unique_address]] std::conditional_t<SHIFTED, uint32_t, None> pshift;

  __device__ __forceinline__ void set_position_shift(uint32_t shift) {
    if constexpr (SHIFTED) pshift = shift;
  }
  __device__ __forceinline__ int sel_constant_bits() const {
    if constexpr (SHIFTED) return (int)pshift;
    return 0;
  }
  __device__ __forceinline__ uint32_t low_half(uint32_t p) const {
    if constexpr (SHIFTED) return ((0xffffu - p) << pshift) & 0xffffu;
    return 0xffffu - p;
  }
  __device__ __forceinline__ uint32_t sub_row(uint32_t word) const {
    if constexpr (SHIFTED) return (0xffffu >> pshift) - ((word & 0xffffu) >> pshift);
    return 0xffffu - (word & 0xffffu);
  }
  __device__ __forceinline__ void reset() {
    ATK_STATIC_FOR(e, V * J) { q[e / J][e % J] = 0; } ATK_STATIC_END;
    screen = 0;
    neg_zeros = 0;
  }
  __device__ static __forceinline__ void insert(uint32_t (&col)[J], uint32_t word) { insert_word<J>(col, word); }
  template <int FILLED> __device__ __forceinline__ void take(const Pack<raw_t, V>& pk, uint32_t p) {
    const uint32_t pinv = low_half(p);
    constexpr int F = LEAN ? FILLED : J;
    if constexpr (V == 1) {
      const uint32_t keys = LEAN ? K::keys2_lean(pk.e[0], screen) : K::keys2(pk.e[0], screen);
      insert_word<J, F>(q[0], (keys << 16) | pinv);
    } else {
      ATK_STATIC_FOR(d, V / 2) {
        uint32_t x;  // elements 2d (low half) and 2d+1 (high half) as loaded
        __builtin_memcpy(&x, &pk.e[2 * d], 4);
        const uint32_t keys = LEAN ? K::keys2_lean(x, screen) : K::keys2(x, screen);
        insert_word<J, F>(q[2 * d], (keys << 16) | pinv);
        insert_word<J, F>(q[2 * d + 1], (keys & 0xffff0000u) | pinv);
      } ATK_STATIC_END;
    }
  }
  // two elements of column VI as loaded in one dword: sub-row p (low half) and p + 1
  template <int VI, int FILLED> __device__ __forceinline__ void take_two(uint32_t x, uint32_t p) {
    constexpr int F = LEAN ? FILLED : J;
    constexpr int F1 = F < J ? F + 1 : J;
    const uint32_t keys = LEAN ? K::keys2_lean(x, screen) : K::keys2(x, screen);
    insert_word<J, F>(q[VI], (keys << 16) | low_half(p));
    insert_word<J, F1>(q[VI], (keys & 0xffff0000u) | low_half(p + 1));
  }
  // one more element for column VI, when `valid` (the word 0 changes nothing)
  template <int VI> __device__ __forceinline__ void take_one(raw_t raw, uint32_t p, bool valid) {
    uint32_t scr = screen;
    const uint32_t keys = LEAN ? K::keys2_lean((uint32_t)raw, scr) : K::keys2((uint32_t)raw, scr);  // the empty high half screens as +0
    if (valid) screen = scr;
    insert(q[VI], valid ? ((keys << 16) | low_half(p)) : 0u);
  }
  __device__ __forceinline__ bool poisoned() const {
    if constexpr (!LEAN) {
      return __ballot(K::special(screen)) != 0;
    } else {
      bool nan = K::special_lean(screen);
      ATK_STATIC_FOR(v, V) { nan |= K::nan_key(q[v][J - 1] >> 16); } ATK_STATIC_END;
      return __ballot(nan) != 0;
    }
  }

  __device__ __forceinline__ void hand_over(unsigned char* area, uint32_t lane) const {
    uint32_t* h = reinterpret_cast<uint32_t*>(area);
    ATK_STATIC_FOR(e, V * J) { h[e * kWave + lane] = q[e / J][e % J]; } ATK_STATIC_END;
  }
  __device__ __forceinline__ void fold_in(const unsigned char* area, uint32_t lane) {
    const uint32_t* h = reinterpret_cast<const uint32_t*>(area);
    ATK_STATIC_FOR(e, V * J) { insert(q[e / J], h[e * kWave + lane]); } ATK_STATIC_END;
  }
  // (entry words carry their whole order: any arrival order gives the same queue)
  __device__ __forceinline__ void fold_in_interleaved(const unsigned char* area, uint32_t lane) { fold_in(area, lane); }
  // Final entries with a zero key are re-read from the row to learn their sign.
  // The element of sub-row p of the lane's v-th column is xr[p * b + col + v * step]
  // (`col` is the lane's first column); call once, after the last fold, by live lanes.
  __device__ __forceinline__ void fix_zeros(const raw_t* __restrict__ xr, int64_t b, int64_t col, int64_t step = 1) {
    if constexpr (K::zero_is_ambiguous) {
      bool any = false;
      ATK_STATIC_FOR(e, V * J) { any |= (q[e / J][e % J] >> 16) == K::kZeroKey; } ATK_STATIC_END;
      if (__ballot(any) == 0) return;
      ATK_STATIC_FOR(e, V * J) {
        const uint32_t word = q[e / J][e % J];
        if ((word >> 16) == K::kZeroKey) {
          const uint32_t p = sub_row(word);
          if (xr[(int64_t)p * b + col + (e / J) * step] == (raw_t)0x8000u) neg_zeros |= 1u << e;
        }
      } ATK_STATIC_END;
    }
  }
  // exact order key of an entry (the queues are not poisoned)
  template <int VI, int SI> __device__ __forceinline__ typename E::key_t key() const { return K::exact(q[VI][SI] >> 16); }
  // the entry's word as it is: packed key, then lower sub-row first -- the
  // selection order up to the column, which is what the index decides last
  using sel_t = uint32_t;
  static constexpr int sel_bits = 32;
  template <int VI, int SI> __device__ __forceinline__ sel_t sel_key() const { return q[VI][SI]; }
  template <int VI, int SI> __device__ __forceinline__ uint2 staged(uint32_t column) const {
    return make_uint2(q[VI][SI], column);
  }
  struct Unstaged { raw_t raw; uint32_t sub_row, column; bool reread; };
  __device__ __forceinline__ Unstaged unstage(uint2 w) const {
    bool zero = false;
    if constexpr (K::zero_is_ambiguous) zero = (w.x >> 16) == K::kZeroKey;
    return Unstaged{K::unkey(w.x >> 16), sub_row(w.x), w.y, zero};
  }
  template <int VI, int SI> __device__ __forceinline__ raw_t raw() const {
    const raw_t r = K::unkey(q[VI][SI] >> 16);
    if constexpr (K::zero_is_ambiguous) return (neg_zeros >> (VI * J + SI)) & 1u ? (raw_t)0x8000u : r;
    return r;
  }
  template <int VI, int SI> __device__ __forceinline__ uint32_t position() const { return sub_row(q[VI][SI]); }
};

// The same for 8-bit element types and rows of fewer than 2^24 - 1 sub-rows:
// the 8-bit order key in the top byte of the word, 0xFFFFFF - sub-row below it.
// Integers have no NaN and no signed zero, so nothing is handled on the side;
// one v_perm_b32 forms the word of an element from the loaded dword.
template <> struct PackedKey<Elem<ATK_U8>> { static constexpr bool available = true; static constexpr uint32_t kFlip = 0u; };
template <> struct PackedKey<Elem<ATK_I8>> { static constexpr bool available = true; static constexpr uint32_t kFlip = 0x80808080u; };

// largest sub-row number (the partial sub-row included) a byte entry can hold
constexpr uint32_t kByteMaxSubRow = 0xfffffeu;

template <typename E, int J, int V> struct ByteQueue {
  using raw_t = typename E::raw_t;
  using K = PackedKey<E>;
  static_assert(sizeof(raw_t) == 1 && (V % 4 == 0 || V == 1), "byte queues hold 8-bit elements");
  static constexpr size_t kHandBytes = (size_t)V * J * kWave * 4;

  uint32_t q[V][J];

  __device__ __forceinline__ void reset() {
    ATK_STATIC_FOR(e, V * J) { q[e / J][e % J] = 0; } ATK_STATIC_END;
  }
  __device__ __forceinline__ void set_position_shift(uint32_t) {}
  __device__ __forceinline__ int sel_constant_bits() const { return 0; }
  __device__ static __forceinline__ void insert(uint32_t (&col)[J], uint32_t word) { insert_word<J>(col, word); }
  template <int FILLED> __device__ __forceinline__ void take(const Pack<raw_t, V>& pk, uint32_t p) {
    const uint32_t pinv = 0xffffffu - p;
    if constexpr (V == 1) {
      insert(q[0], (E::key(pk.e[0]) << 24) | pinv);
    } else {
      ATK_STATIC_FOR(d, V / 4) {
        uint32_t x;  // elements 4d .. 4d+3 as loaded, lowest byte first
        __builtin_memcpy(&x, &pk.e[4 * d], 4);
        x ^= K::kFlip;
        // byte 3 of the word: byte i of x; bytes 2..0: those of pinv
        insert(q[4 * d], __builtin_amdgcn_perm(x, pinv, 0x04020100u));
        insert(q[4 * d + 1], __builtin_amdgcn_perm(x, pinv, 0x05020100u));
        insert(q[4 * d + 2], __builtin_amdgcn_perm(x, pinv, 0x06020100u));
        insert(q[4 * d + 3], __builtin_amdgcn_perm(x, pinv, 0x07020100u));
      } ATK_STATIC_END;
    }
  }
  // one more element for column VI, when `valid` (the word 0 changes nothing)
  template <int VI> __device__ __forceinline__ void take_one(raw_t raw, uint32_t p, bool valid) {
    insert(q[VI], valid ? ((E::key(raw) << 24) | (0xffffffu - p)) : 0u);
  }
  __device__ __forceinline__ bool poisoned() const { return false; }

  __device__ __forceinline__ void hand_over(unsigned char* area, uint32_t lane) const {
    uint32_t* h = reinterpret_cast<uint32_t*>(area);
    ATK_STATIC_FOR(e, V * J) { h[e * kWave + lane] = q[e / J][e % J]; } ATK_STATIC_END;
  }
  __device__ __forceinline__ void fold_in(const unsigned char* area, uint32_t lane) {
    const uint32_t* h = reinterpret_cast<const uint32_t*>(area);
    ATK_STATIC_FOR(e, V * J) { insert(q[e / J], h[e * kWave + lane]); } ATK_STATIC_END;
  }
  // (entry words carry their whole order: any arrival order gives the same queue)
  __device__ __forceinline__ void fold_in_interleaved(const unsigned char* area, uint32_t lane) { fold_in(area, lane); }
  __device__ __forceinline__ void fix_zeros(const raw_t* __restrict__, int64_t, int64_t, int64_t = 1) {}
  template <int VI, int SI> __device__ __forceinline__ typename E::key_t key() const { return q[VI][SI] >> 24; }
  using sel_t = uint32_t;
  static constexpr int sel_bits = 32;
  template <int VI, int SI> __device__ __forceinline__ sel_t sel_key() const { return q[VI][SI]; }
  template <int VI, int SI> __device__ __forceinline__ uint2 staged(uint32_t column) const {
    return make_uint2(q[VI][SI], column);
  }
  struct Unstaged { raw_t raw; uint32_t sub_row, column; bool reread; };
  __device__ __forceinline__ Unstaged unstage(uint2 w) const {
    return Unstaged{(raw_t)((w.x >> 24) ^ (K::kFlip & 0xffu)), 0xffffffu - (w.x & 0xffffffu), w.y, false};
  }
  template <int VI, int SI> __device__ __forceinline__ raw_t raw() const {
    return (raw_t)((q[VI][SI] >> 24) ^ (K::kFlip & 0xffu));
  }
  template <int VI, int SI> __device__ __forceinline__ uint32_t position() const { return 0xffffffu - (q[VI][SI] & 0xffffffu); }
};

// Wide form for fp32 with two or more entries per column: an entry is one
// 64-bit word read as a double, the element's bits in the high half and the
// sub-row number below it, so that a push is J v_max_f64 and J-1 v_min_f64
// (both issue at the rate of 32-bit operations on this part) where the general
// form takes J compares and about 4 J selects.
//
// Why the order is right: a non-NaN float's bits, taken as the high word of a
// double (sign, then 8 + 3 bits as exponent, then mantissa), order as the float
// does, and the exponent field is all ones only for some NaNs, so that every
// word is a finite double.  Among equal elements the lower sub-row must win:
// the low word holds ~sub-row under a positive element and sub-row under a
// negative one (where a larger magnitude is the smaller double).  -0.0 is read
// as +0.0 first (x + 0.0f), as the order has them equal; entries with a zero
// element are re-read from the row at the end to learn their sign
// (`fix_zeros`).  Loads are screened for NaN as in the general form.  The empty
// entry is the double -inf, below every word.  Words under a zero or a tiny
// element are subnormal doubles: the kernels run with double-precision
// subnormals kept (the compiler's default for this target, whatever the fp32
// mode), and v_max_f64 / v_min_f64 hand back one of their operands unchanged.
__device__ __forceinline__ double max_f64(double a, double b) {
  double r;
  asm("v_max_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ double min_f64(double a, double b) {
  double r;
  asm("v_min_f64 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

template <typename E, int J, int V> struct WideQueue {
  using raw_t = typename E::raw_t;
  static_assert(std::is_same<E, Elem<ATK_F32>>::value && J >= 2, "wide queues hold fp32 elements");
  static constexpr size_t kHandBytes = (size_t)V * J * kWave * 8;

  double q[V][J];
  uint64_t nan_mask;   // lanes that loaded a NaN; wave-uniform
  uint32_t neg_zeros;  // bit v*J+s: entry (v, s) is a -0.0 (set by fix_zeros)

  __device__ static __forceinline__ double empty() { return __longlong_as_double((long long)0xfff0000000000000ull); }
  __device__ static __forceinline__ uint32_t high(double w) { return (uint32_t)((uint64_t)__double_as_longlong(w) >> 32); }
  __device__ static __forceinline__ uint32_t low(double w) { return (uint32_t)(uint64_t)__double_as_longlong(w); }
  // `c`: the element with -0.0 already read as +0.0; np: ~sub-row
  __device__ static __forceinline__ double word(float c, uint32_t np) {
    const uint32_t hi = __float_as_uint(c);
    const uint32_t lo = np ^ (uint32_t)((int32_t)hi >> 31);
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
  }
  // FILLED: entries the column is known to hold already (its last ones; the others are empty)
  template <int FILLED = J> __device__ static __forceinline__ void insert(double (&col)[J], double w) {
    ATK_STATIC_FOR(s, J - 1) {
      if constexpr (s + 1 + FILLED == J) col[s] = min_f64(w, col[s + 1]);
      else if constexpr (s + 1 + FILLED > J) col[s] = max_f64(col[s], min_f64(w, col[s + 1]));
    } ATK_STATIC_END;
    if constexpr (FILLED == 0) col[J - 1] = w;
    else col[J - 1] = max_f64(col[J - 1], w);
  }

  __device__ __forceinline__ void reset() {
    ATK_STATIC_FOR(e, V * J) { q[e / J][e % J] = empty(); } ATK_STATIC_END;
    nan_mask = 0;
    neg_zeros = 0;
  }
  __device__ __forceinline__ void set_position_shift(uint32_t) {}
  __device__ __forceinline__ int sel_constant_bits() const { return 0; }

  template <int FILLED> __device__ __forceinline__ void take(const Pack<raw_t, V>& pk, uint32_t p) {
    const uint32_t np = ~p;
    float c[V];
    ATK_STATIC_FOR(v, V) { c[v] = __uint_as_float(pk.e[v]) + 0.0f; } ATK_STATIC_END;
    ATK_STATIC_FOR(h, V / 2) { nan_mask |= __ballot(__builtin_isunordered(c[2 * h], c[2 * h + 1])); } ATK_STATIC_END;
    if constexpr (V % 2 != 0) nan_mask |= __ballot(__builtin_isunordered(c[V - 1], c[V - 1]));
    ATK_STATIC_FOR(v, V) { insert<FILLED>(q[v], word(c[v], np)); } ATK_STATIC_END;
  }
  // elements of sub-rows p and p + 1 of column VI
  template <int VI, int FILLED> __device__ __forceinline__ void take_two(raw_t a, raw_t b, uint32_t p) {
    const float ca = __uint_as_float(a) + 0.0f, cb = __uint_as_float(b) + 0.0f;
    nan_mask |= __ballot(__builtin_isunordered(ca, cb));
    insert<FILLED>(q[VI], word(ca, ~p));
    insert<(FILLED < J ? FILLED + 1 : J)>(q[VI], word(cb, ~(p + 1)));
  }
  template <int VI> __device__ __forceinline__ void take_one(raw_t raw, uint32_t p, bool valid) {
    const float c = __uint_as_float(raw) + 0.0f;
    nan_mask |= __ballot(valid && __builtin_isunordered(c, c));
    insert(q[VI], valid ? word(c, ~p) : empty());
  }
  __device__ __forceinline__ bool poisoned() const { return nan_mask != 0; }

  __device__ __forceinline__ void hand_over(unsigned char* area, uint32_t lane) const {
    double* h = reinterpret_cast<double*>(area);
    ATK_STATIC_FOR(e, V * J) { h[e * kWave + lane] = q[e / J][e % J]; } ATK_STATIC_END;
  }
  // (entry words carry their whole order: any arrival order gives the same queue)
  __device__ __forceinline__ void fold_in(const unsigned char* area, uint32_t lane) {
    const double* h = reinterpret_cast<const double*>(area);
    ATK_STATIC_FOR(e, V * J) { insert(q[e / J], h[e * kWave + lane]); } ATK_STATIC_END;
  }
  __device__ __forceinline__ void fold_in_interleaved(const unsigned char* area, uint32_t lane) { fold_in(area, lane); }
  // Final entries with a zero element are re-read from the row to learn their
  // sign (sub-row p of the lane's v-th column is xr[p * b + col + v * step]); call once,
  // after the last fold, by live lanes.
  __device__ __forceinline__ void fix_zeros(const raw_t* __restrict__ xr, int64_t b, int64_t col, int64_t step = 1) {
    bool any = false;
    ATK_STATIC_FOR(e, V * J) { any |= high(q[e / J][e % J]) == 0u; } ATK_STATIC_END;
    if (__ballot(any) == 0) return;
    ATK_STATIC_FOR(e, V * J) {
      if (high(q[e / J][e % J]) == 0u) {
        const uint32_t p = ~low(q[e / J][e % J]);
        if (xr[(int64_t)p * b + col + (e / J) * step] == 0x80000000u) neg_zeros |= 1u << e;
      }
    } ATK_STATIC_END;
  }
  template <int VI, int SI> __device__ __forceinline__ typename E::key_t key() const { return E::key(high(q[VI][SI])); }
  using sel_t = typename E::key_t;
  static constexpr int sel_bits = E::key_bits;
  template <int VI, int SI> __device__ __forceinline__ sel_t sel_key() const { return key<VI, SI>(); }
  template <int VI, int SI> __device__ __forceinline__ uint2 staged(uint32_t column) const {
    return make_uint2(high(q[VI][SI]), (position<VI, SI>() << 16) | column);
  }
  struct Unstaged { raw_t raw; uint32_t sub_row, column; bool reread; };
  __device__ __forceinline__ Unstaged unstage(uint2 w) const {
    return Unstaged{w.x, w.y >> 16, w.y & 0xffffu, w.x == 0u};
  }
  template <int VI, int SI> __device__ __forceinline__ raw_t raw() const {
    return (neg_zeros >> (VI * J + SI)) & 1u ? 0x80000000u : high(q[VI][SI]);
  }
  template <int VI, int SI> __device__ __forceinline__ uint32_t position() const {
    const uint32_t hi = high(q[VI][SI]);
    return ~(low(q[VI][SI]) ^ (uint32_t)((int32_t)hi >> 31));
  }
};

// fewest entries per column from which fp32 queues take the wide form
constexpr int kWideFromJ = 2;

// Loads a lane keeps in flight (the kernels' U).  Packed queues: bytes load 8
// per lane and keep few registers per entry.  General queues of J >= 3 leave
// registers for four; the wide fp32 queues cost half the instructions, so
// that their scan waits on memory and eight pay (fp32 [1, 2^26], 8192 buckets,
// J = 4: 50.6 -> 48.2 us; sixteen: 66.8 us).
__host__ __device__ constexpr int loads_in_flight(int dtype, int j, int vec, bool packed) {
  if (packed) return elem_bytes(dtype) == 1 ? 8 : (vec * j <= 8 ? 8 : 4);
  return (j <= 2 || (dtype == ATK_F32 && j >= kWideFromJ)) ? 8 : 4;
}

// Packed 16-bit queues of two or four entries over columns of at most
// kShortColumn sub-rows, scanned by the general loop (run == 0: columns of 33-64
// sub-rows), keep eight loads in flight instead of four: fp16 [256, 2^20]
// k=65536 j=4 166 -> 149 us, [128, 2^20] k=32768 j=2 65.5 -> 60.5 us, [16, 2^22]
// k=2^18 j=4 47.8 -> 45.3 us.  The exact short runs (columns of up to 32) gain
// nothing from it, and with long columns eight lose (fp16 [1, 2^26] j=4 k_mult=2
// 53.9 -> 62.1 us, [128, 2^20] k=16384 j=4 62.7 -> 74.8 us).
constexpr uint32_t kShortColumn = 64;
__host__ __device__ constexpr bool deep_loads_for_short_columns(int dtype, int j, int vec, bool packed, int run,
                                                                uint32_t full_rows) {
  return packed && elem_bytes(dtype) == 2 && vec == 8 && (j == 2 || j == 4) && run == 0 &&
         full_rows <= kShortColumn;
}

template <typename E, int J, int V, bool PACKED, bool SHIFTED = false>
using QueueFor = std::conditional_t<
    !PACKED,
    std::conditional_t<std::is_same<E, Elem<ATK_F32>>::value && (J >= kWideFromJ), WideQueue<E, (J >= 2 ? J : 2), V>,
                       CmpQueue<E, J, V>>,
    std::conditional_t<sizeof(typename E::raw_t) == 1, ByteQueue<E, J, V>, PackedQueue<E, J, V, SHIFTED>>>;

// Shape of one launch; passed to the kernels by value.  With few buckets the
// planner folds the row: `fold` consecutive sub-rows of the true [L][b] matrix
// form one sub-row of a matrix with b * fold columns, which is what the kernel
// scans; column f*b + c of it holds every fold-th element of bucket c, the flat
// index of an element is the same in both views, and the scanning workgroup
// folds the `fold` columns of a bucket back together.  `b` below is the scanned
// width.
struct Geom {
  int64_t row_stride;     // elements between rows
  int64_t b;              // columns per row as scanned
  uint32_t full_rows;     // L = n / b
  uint32_t rem;           // n mod b: columns that have one more element
  uint32_t pad_tail;      // padded row: the other columns hold the pad value there
  uint32_t slabs;         // sub-row slabs per row
  uint32_t slab_len;      // sub-rows per slab (the last slab takes the rest)
  uint32_t col_tiles;     // workgroup column tiles per row
  uint32_t fold;          // scanned columns per bucket (1: not folded)
};

// Where results go: final values/indices[rows][buckets*J], or, when the merge
// kernel follows (several slabs; part_values != nullptr), per-slab queues
// [rows][slabs][buckets*J] (raw values and the entries' numbers within their
// buckets).
template <typename raw_t> struct Sink {
  raw_t* values;
  IndexOut indices;
  raw_t* part_values;
  uint32_t* part_pos;
};

// Writes the queues of this lane's V columns, either as final results or as a
// slab's partial result.
template <typename E, int J, int V, typename Queue>
__device__ __forceinline__ void emit(const Geom& g, const Sink<typename E::raw_t>& out, int64_t row,
                                     uint32_t slab, int64_t col, const Queue& queue) {
  using raw_t = typename E::raw_t;
  if (out.part_values == nullptr) {
    const int64_t o = (row * g.b + col) * J;
    raw_t* ov = out.values + o;
    if constexpr (V > 1) {
      // V*J values = J stores of V elements; V*J int64 = V*J/2 16-byte stores
      // (int32: 16-byte stores when V*J is a multiple of 4, else 8-byte ones)
      if (out.values != nullptr) {
        ATK_STATIC_FOR(t, J) {
          Pack<raw_t, V> pv;
          ATK_STATIC_FOR(e, V) { pv.e[e] = queue.template raw<(t * V + e) / J, (t * V + e) % J>(); } ATK_STATIC_END;
          reinterpret_cast<Pack<raw_t, V>*>(ov)[t] = pv;
        } ATK_STATIC_END;
      }
      if (out.indices.narrow) {
        constexpr int kPer = (V * J) % 4 == 0 ? 4 : 2;
        int32_t* oi = static_cast<int32_t*>(out.indices.base) + o;
        ATK_STATIC_FOR(t, V * J / kPer) {
          Pack<int32_t, kPer> pi;
          ATK_STATIC_FOR(e, kPer) {
            constexpr int v = (t * kPer + e) / J, sl = (t * kPer + e) % J;
            pi.e[e] = (int32_t)(col + v + (int64_t)queue.template position<v, sl>() * g.b);
          } ATK_STATIC_END;
          reinterpret_cast<Pack<int32_t, kPer>*>(oi)[t] = pi;
        } ATK_STATIC_END;
      } else {
        int64_t* oi = static_cast<int64_t*>(out.indices.base) + o;
        ATK_STATIC_FOR(t, V * J / 2) {
          Pack<int64_t, 2> pi;
          ATK_STATIC_FOR(e, 2) {
            constexpr int v = (t * 2 + e) / J, sl = (t * 2 + e) % J;
            pi.e[e] = col + v + (int64_t)queue.template position<v, sl>() * g.b;
          } ATK_STATIC_END;
          reinterpret_cast<Pack<int64_t, 2>*>(oi)[t] = pi;
        } ATK_STATIC_END;
      }
    } else {
      ATK_STATIC_FOR(sl, J) {
        if (out.values != nullptr) ov[sl] = queue.template raw<0, sl>();
        out.indices.put(o + sl, col + (int64_t)queue.template position<0, sl>() * g.b);
      } ATK_STATIC_END;
    }
  } else {
    const int64_t o = ((row * g.slabs + slab) * g.b + col) * J;
    raw_t* ov = out.part_values + o;
    uint32_t* op = out.part_pos + o;
    ATK_STATIC_FOR(e, V * J) {
      ov[e] = queue.template raw<e / J, e % J>();
      op[e] = queue.template position<e / J, e % J>();
    } ATK_STATIC_END;
  }
}

// The same for final results, by the one wave that holds a tile's queues, with
// every store instruction covering 1 KiB of adjacent bytes.  Written as above, a
// store instruction sends 64 separate 16-byte pieces to L2, a lane's stretch of
// output (V * J entries) apart: fp16 [128, 2^20] k=262144 j=4, 32 entries a lane,
// took 188 us that way and takes 109 us this way, [256, 2^20] k=65536 j=4 147 -> 135 us
// and j=2 132 -> 118 us, uint8 [128, 2^20] k=65536 j=2 50 -> 42 us, fp32 k=262144 j=4
// 177 -> 165 us; with eight 4-byte entries a lane (fp32, j=2) it makes no difference.
// The lanes park their entries in LDS -- the elements in one array, the sub-row
// numbers in another, a lane's stretch 16 bytes further on than a power of two
// from the next lane's for the banks -- and read them back in the order of the
// output.  `col0`: the tile's first column; lanes beyond the row's last column
// hold nothing that is read.  One wave: its LDS accesses complete in program
// order, so nothing waits on a barrier.  The trip through LDS is a few hundred
// cycles at the end of every workgroup, which a launch of few workgroups, or one
// whose output is small beside its input, does not get back: fp16 [256, 65536]
// k=4096 j=4 (512 workgroups) 14.2 -> 15.5 us; the planner decides (Plan::wave_stores).
template <typename E, int J, int V>
struct Transposed {
  using raw_t = typename E::raw_t;
  static constexpr int NC = V * J;                           // entries of a lane
  static constexpr int kPerStore = 16 / (int)sizeof(raw_t);  // elements in 16 bytes
  // whole 16-byte pieces on both sides, elements of up to four bytes; not for eight 4-byte
  // entries a lane (fp32 [128, 2^20] k=65536 j=2: 108.6-109.6 us either way)
  static constexpr bool available = V > 1 && sizeof(raw_t) <= 4 && NC % 4 == 0 && NC % kPerStore == 0 &&
                                    (NC * 8 >= 128 || sizeof(raw_t) < 4) && J != 3;  // (j = 3: not built)
  static constexpr size_t kRawPitch = (size_t)NC * sizeof(raw_t) + 16;  // bytes from lane to lane
  static constexpr size_t kPosPitch = (size_t)NC * 4 + 16;
  static constexpr size_t kPosArea = kWave * kRawPitch;                 // where the sub-row numbers start
  static constexpr size_t kBytes = kPosArea + kWave * kPosPitch;
};

template <typename E, int J, int V, typename Queue>
__device__ __forceinline__ void emit_transposed(const Geom& g, const Sink<typename E::raw_t>& out, int64_t row,
                                                int64_t col0, uint32_t lane, const Queue& queue,
                                                unsigned char* lds) {
  using raw_t = typename E::raw_t;
  using T = Transposed<E, J, V>;
  constexpr int NC = T::NC, kPerStore = T::kPerStore;
  static_assert(T::available, "see Transposed");
  unsigned char* raws = lds;
  unsigned char* poss = lds + T::kPosArea;
  if (out.values != nullptr) {
    ATK_STATIC_FOR(t, NC / kPerStore) {
      Pack<raw_t, kPerStore> pv;
      ATK_STATIC_FOR(u, kPerStore) {
        constexpr int e = t * kPerStore + u;
        pv.e[u] = queue.template raw<e / J, e % J>();
      } ATK_STATIC_END;
      *reinterpret_cast<Pack<raw_t, kPerStore>*>(raws + lane * T::kRawPitch + 16 * t) = pv;
    } ATK_STATIC_END;
  }
  ATK_STATIC_FOR(t, NC / 4) {
    uint32_t w[4];
    ATK_STATIC_FOR(u, 4) {
      constexpr int e = t * 4 + u;
      w[u] = queue.template position<e / J, e % J>();
    } ATK_STATIC_END;
    *reinterpret_cast<uint4*>(poss + lane * T::kPosPitch + 16 * t) = make_uint4(w[0], w[1], w[2], w[3]);
  } ATK_STATIC_END;

  const int64_t left = (g.b - col0) * J;  // entries from this tile's first to the row's last
  const uint32_t valid = left < (int64_t)(kWave * NC) ? (uint32_t)left : (uint32_t)(kWave * NC);
  const int64_t o = (row * g.b + col0) * J;
  if (out.values != nullptr) {
    ATK_STATIC_FOR(t, NC / kPerStore) {
      const uint32_t i = t * (kWave * kPerStore) + lane * kPerStore;  // (valid is a multiple of kPerStore)
      if (i < valid) {
        const Pack<raw_t, kPerStore> pv = *reinterpret_cast<const Pack<raw_t, kPerStore>*>(
            raws + (i / NC) * T::kRawPitch + (i % NC) * sizeof(raw_t));
        *reinterpret_cast<Pack<raw_t, kPerStore>*>(out.values + o + i) = pv;
      }
    } ATK_STATIC_END;
  }
  auto pos_at = [&](uint32_t i) __attribute__((always_inline)) -> const unsigned char* {
    return poss + (i / NC) * T::kPosPitch + (i % NC) * 4;
  };
  auto index_of = [&](uint32_t i, uint32_t sub_row) __attribute__((always_inline)) -> int64_t {
    return col0 + (int64_t)(i / J) + (int64_t)sub_row * g.b;
  };
  if (out.indices.narrow) {
    int32_t* oi = static_cast<int32_t*>(out.indices.base) + o;
    ATK_STATIC_FOR(t, NC / 4) {
      const uint32_t i = t * (kWave * 4) + lane * 4;
      if (i < valid) {
        const uint4 a = *reinterpret_cast<const uint4*>(pos_at(i));
        Pack<int32_t, 4> pi;
        pi.e[0] = (int32_t)index_of(i, a.x); pi.e[1] = (int32_t)index_of(i + 1, a.y);
        pi.e[2] = (int32_t)index_of(i + 2, a.z); pi.e[3] = (int32_t)index_of(i + 3, a.w);
        *reinterpret_cast<Pack<int32_t, 4>*>(oi + i) = pi;
      }
    } ATK_STATIC_END;
  } else {
    int64_t* oi = static_cast<int64_t*>(out.indices.base) + o;
    ATK_STATIC_FOR(t, NC / 2) {
      const uint32_t i = t * (kWave * 2) + lane * 2;
      if (i < valid) {
        const uint2 a = *reinterpret_cast<const uint2*>(pos_at(i));
        Pack<int64_t, 2> pi;
        pi.e[0] = index_of(i, a.x);
        pi.e[1] = index_of(i + 1, a.y);
        *reinterpret_cast<Pack<int64_t, 2>*>(oi + i) = pi;
      }
    } ATK_STATIC_END;
  }
}

// Exact recomputation of one lane's V columns over sub-rows [p0, p1) (plus the
// partial sub-row when `with_rem`), through order keys, one column at a time.
// Off the hot path: kept small in registers rather than fast.
template <typename E, int J, int V>
__device__ __forceinline__ void exact_columns(const typename E::raw_t* __restrict__ xr, const Geom& g,
                                     const Sink<typename E::raw_t>& out, int64_t row, uint32_t slab,
                                     int64_t col, uint32_t p0, uint32_t p1, bool with_rem) {
  using raw_t = typename E::raw_t;
#pragma nounroll
  for (int v = 0; v < V; ++v) {
    const int64_t c = col + v;
    raw_t val[J];
    uint32_t pos[J];
    clear_exact<E, J>(val, pos);
    uint32_t p = p0;
    for (; p + 8 <= p1; p += 8) {  // eight loads in flight
      raw_t got[8];
      ATK_STATIC_FOR(u, 8) { got[u] = xr[(int64_t)(p + u) * g.b + c]; } ATK_STATIC_END;
      ATK_STATIC_FOR(u, 8) { push_exact<E, J>(val, pos, got[u], p + u); } ATK_STATIC_END;
    }
    for (; p < p1; ++p) push_exact<E, J>(val, pos, xr[(int64_t)p * g.b + c], p);
    if (with_rem && g.rem != 0) {
      if (c < (int64_t)g.rem)
        push_exact<E, J>(val, pos, xr[(int64_t)g.full_rows * g.b + c], g.full_rows);
      else if (g.pad_tail)
        push_exact<E, J>(val, pos, E::pad_raw, g.full_rows);
    }
    if (out.part_values == nullptr) {
      const int64_t o = (row * g.b + c) * J;
#pragma unroll
      for (int s = 0; s < J; ++s) {
        if (out.values != nullptr) out.values[o + s] = val[s];
        out.indices.put(o + s, c + (int64_t)pos[s] * g.b);
      }
    } else {
      const int64_t o = ((row * g.slabs + slab) * g.b + c) * J;
#pragma unroll
      for (int s = 0; s < J; ++s) { out.part_values[o + s] = val[s]; out.part_pos[o + s] = pos[s]; }
    }
  }
}

// The rest of a wave's scan once its queues are full: sub-rows [p, p1) of this
// lane's columns, `next` pointing at sub-row p, U loads in flight: an odd batch
// of fewer than U, then batches of U that are refilled while they are consumed.
// Loads and their uses are kept in the same basic block wherever a load is
// outstanding across them, so that the wait counts are exact.
template <typename E, int J, int V, int U, typename Queue>
__device__ __forceinline__ void scan_rest(const typename E::raw_t* next, int64_t b, uint32_t p, uint32_t p1,
                                          Queue& queue) {
  using raw_t = typename E::raw_t;
  auto load_next = [&]() __attribute__((always_inline)) {
    const Pack<raw_t, V> pk = load_pack<raw_t, V>(next);
    next += b;
    return pk;
  };
  const uint32_t odd = (p1 - p) % U;
  if (odd != 0) {  // fewer than U sub-rows, so that whole batches remain
    Pack<raw_t, V> buf[U];
#pragma unroll
    for (int u = 0; u < U - 1; ++u) {
      if ((uint32_t)u < odd) buf[u] = load_next();
    }
#pragma unroll
    for (int u = 0; u < U - 1; ++u) {
      if ((uint32_t)u < odd) queue.template take<J>(buf[u], p + u);
    }
    p += odd;
  }
  uint32_t batches = (p1 - p) / U;
  if (batches != 0) {
    Pack<raw_t, V> buf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) buf[u] = load_next();
    for (; batches > 1; --batches) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const Pack<raw_t, V> cur = buf[u];
        buf[u] = load_next();
        queue.template take<J>(cur, p + u);
      }
      p += U;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) queue.template take<J>(buf[u], p + u);
  }
}

// The row's partial sub-row: column c has one more element when c < rem (with a
// padded row the other columns see the pad value there).  Its number is above
// all others, so it comes last.
template <typename E, int V, typename Queue>
__device__ __forceinline__ void scan_partial_sub_row(const typename E::raw_t* __restrict__ xr, const Geom& g,
                                                     int64_t col, bool live, Queue& queue) {
  using raw_t = typename E::raw_t;
  if (g.rem != 0) {
    ATK_STATIC_FOR(v, V) {
      const bool real = live && col + v < (int64_t)g.rem;
      const raw_t* at = real ? xr + (int64_t)g.full_rows * g.b + col + v : xr;  // xr[0] always exists
      const raw_t value = *at;
      queue.template take_one<v>(real ? value : E::pad_raw, g.full_rows, real || (live && g.pad_tail != 0));
    } ATK_STATIC_END;
  }
}

// One wave's scan: folds sub-rows [p0, p1) (p1 - p0 >= J) of this lane's V
// columns starting at `col` into `queue`, plus the row's partial sub-row when
// `with_rem`.  `xr` is the row; lanes that are not `live` load column 0 and are
// ignored by the caller.  RUN > 0 promises p1 - p0 == RUN (J <= RUN): all loads
// are issued at once and the code is one straight line.  RUN == 0 takes any
// length: the first J sub-rows, then the rest as scan_rest does.
template <typename E, int J, int V, int U, int RUN, typename Queue>
__device__ __forceinline__ void scan_run(const typename E::raw_t* __restrict__ xr, const Geom& g, int64_t col,
                                bool live, uint32_t p0, uint32_t p1, bool with_rem, Queue& queue) {
  using raw_t = typename E::raw_t;
  static_assert(RUN == 0 || RUN >= J, "a run holds at least J sub-rows");
  // `next` walks down this lane's columns one sub-row per load
  const raw_t* next = xr + (live ? col : 0) + (int64_t)p0 * g.b;
  auto load_next = [&]() __attribute__((always_inline)) {
    const Pack<raw_t, V> pk = load_pack<raw_t, V>(next);
    next += g.b;
    return pk;
  };
  queue.reset();

  if constexpr (RUN > 0) {
    Pack<raw_t, V> buf[RUN];
#pragma unroll
    for (int u = 0; u < RUN; ++u) buf[u] = load_next();
    ATK_STATIC_FOR(u, RUN) { queue.template take<(u < J ? u : J)>(buf[u], p0 + u); } ATK_STATIC_END;
  } else {
    {  // the first J sub-rows fill the queues
      Pack<raw_t, V> buf[J];
#pragma unroll
      for (int u = 0; u < J; ++u) buf[u] = load_next();
      ATK_STATIC_FOR(u, J) { queue.template take<u>(buf[u], p0 + u); } ATK_STATIC_END;
    }
    scan_rest<E, J, V, U>(next, g.b, p0 + J, p1, queue);
  }
  if (with_rem) scan_partial_sub_row<E, V>(xr, g, col, live, queue);
}

// The same scan for a wave that shares its column tile with `split` - 1 others
// in windows: the full sub-rows are cut into windows of U, and the wave with
// number `part` takes windows part, part + split, ...  At any time the waves of
// a tile then read one stretch of split * U adjacent sub-rows together instead
// of `split` streams far apart, which keeps the DRAM pages they open in use
// (measured on fp32 [256, 131072] with 512 buckets, four waves per tile:
// 29 -> 25 us for the scan).  Every wave must own at least one whole window
// (full_rows >= split * U; U >= J).  With `with_rem` the wave also takes the
// row's partial sub-row (one wave of the tile should).  U loads stay in flight:
// a window is consumed while the next one is loaded, in one basic block.  The
// waves' sub-rows interleave, so their queues are put together under the full
// order (fold_in_interleaved).
template <typename E, int J, int V, int U, typename Queue>
__device__ __forceinline__ void scan_windows(const typename E::raw_t* __restrict__ xr, const Geom& g, int64_t col,
                                             bool live, uint32_t part, uint32_t split, bool with_rem,
                                             Queue& queue) {
  using raw_t = typename E::raw_t;
  static_assert(U >= J, "the first window fills the queues");
  const uint32_t whole = g.full_rows / U;  // whole windows in the row
  const uint32_t tail = g.full_rows % U;   // sub-rows of the window after them
  const uint32_t mine = (whole - part + split - 1) / split;      // whole windows of this wave (>= 1)
  const bool has_tail = tail != 0 && whole % split == part;      // the last, shorter window is this wave's
  const raw_t* base = xr + (live ? col : 0);
  const int64_t window_step = (int64_t)g.b * U * split;          // elements from a window to this wave's next
  const raw_t* next = base + (int64_t)part * U * g.b;            // the window being loaded
  queue.reset();

  Pack<raw_t, V> buf[U];
#pragma unroll
  for (int u = 0; u < U; ++u) buf[u] = load_pack<raw_t, V>(next + (int64_t)u * g.b);
  next += window_step;
  uint32_t p = part * U;  // first sub-row of the window in `buf`
  const uint32_t p_step = U * split;
  if (mine > 1) {
    // the first window fills the queues while the second is loaded
    ATK_STATIC_FOR(u, U) {
      const Pack<raw_t, V> cur = buf[u];
      buf[u] = load_pack<raw_t, V>(next + (int64_t)u * g.b);
      queue.template take<(u < J ? u : J)>(cur, p + u);
    } ATK_STATIC_END;
    next += window_step;
    p += p_step;
    for (uint32_t left = mine - 2; left != 0; --left) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const Pack<raw_t, V> cur = buf[u];
        buf[u] = load_pack<raw_t, V>(next + (int64_t)u * g.b);
        queue.template take<J>(cur, p + u);
      }
      next += window_step;
      p += p_step;
    }
    // the last whole window; the shorter one behind it, if it is this wave's, is loaded meanwhile
    if (has_tail) {
      Pack<raw_t, V> last[U - 1 > 0 ? U - 1 : 1];
#pragma unroll
      for (int u = 0; u < U - 1; ++u) {
        if ((uint32_t)u < tail) last[u] = load_pack<raw_t, V>(next + (int64_t)u * g.b);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) queue.template take<J>(buf[u], p + u);
      p += p_step;
#pragma unroll
      for (int u = 0; u < U - 1; ++u) {
        if ((uint32_t)u < tail) queue.template take<J>(last[u], p + u);
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) queue.template take<J>(buf[u], p + u);
    }
  } else {
    // one whole window only
    if (has_tail) {
      Pack<raw_t, V> last[U - 1 > 0 ? U - 1 : 1];
#pragma unroll
      for (int u = 0; u < U - 1; ++u) {
        if ((uint32_t)u < tail) last[u] = load_pack<raw_t, V>(next + (int64_t)u * g.b);
      }
      ATK_STATIC_FOR(u, U) { queue.template take<(u < J ? u : J)>(buf[u], p + u); } ATK_STATIC_END;
      p += p_step;
#pragma unroll
      for (int u = 0; u < U - 1; ++u) {
        if ((uint32_t)u < tail) queue.template take<J>(last[u], p + u);
      }
    } else {
      ATK_STATIC_FOR(u, U) { queue.template take<(u < J ? u : J)>(buf[u], p + u); } ATK_STATIC_END;
    }
  }
  // the partial sub-row: its number is above all others, so it comes last
  if (with_rem && g.rem != 0) {
    ATK_STATIC_FOR(v, V) {
      const bool real = live && col + v < (int64_t)g.rem;
      const raw_t* at = real ? xr + (int64_t)g.full_rows * g.b + col + v : xr;  // xr[0] always exists
      const raw_t value = *at;
      queue.template take_one<v>(real ? value : E::pad_raw, g.full_rows, real || (live && g.pad_tail != 0));
    } ATK_STATIC_END;
  }
}

// An entry while partial queues are merged: order key and sub-row number in one comparable
// word (a larger word is a better entry; the all-zero word is an empty slot,
// which no entry equals because sub-row numbers stay below 0xfffffffe).
template <typename E, bool WIDE = (E::key_bits > 32)> struct MergeWord {
  using word_t = uint64_t;
  __device__ static __forceinline__ word_t make(typename E::raw_t raw, uint32_t p) {
    return ((uint64_t)E::key(raw) << 32) | (uint64_t)(0xffffffffu - p);
  }
  __device__ static __forceinline__ word_t from_key(typename E::key_t key, uint32_t p) {
    return ((uint64_t)key << 32) | (uint64_t)(0xffffffffu - p);
  }
  __device__ static __forceinline__ word_t empty() { return 0; }
  __device__ static __forceinline__ bool better(word_t a, word_t b) { return a > b; }
  __device__ static __forceinline__ uint32_t pos(word_t w) { return 0xffffffffu - (uint32_t)w; }
  __device__ static __forceinline__ typename E::key_t key(word_t w) { return (typename E::key_t)(w >> 32); }
  __device__ static __forceinline__ word_t from_lane(word_t w, int lane) { return __shfl(w, lane); }
};
template <typename E> struct MergeWord<E, true> {
  struct word_t { uint64_t key; uint32_t npos; uint32_t unused; };
  __device__ static __forceinline__ word_t make(typename E::raw_t raw, uint32_t p) {
    return word_t{E::key(raw), 0xffffffffu - p, 0u};
  }
  __device__ static __forceinline__ word_t from_key(uint64_t key, uint32_t p) {
    return word_t{key, 0xffffffffu - p, 0u};
  }
  __device__ static __forceinline__ word_t empty() { return word_t{0, 0, 0}; }
  __device__ static __forceinline__ bool better(const word_t& a, const word_t& b) {
    return a.key > b.key || (a.key == b.key && a.npos > b.npos);
  }
  __device__ static __forceinline__ uint32_t pos(const word_t& w) { return 0xffffffffu - w.npos; }
  __device__ static __forceinline__ uint64_t key(const word_t& w) { return w.key; }
  __device__ static __forceinline__ word_t from_lane(const word_t& w, int lane) {
    return word_t{__shfl(w.key, lane), __shfl(w.npos, lane), 0u};
  }
};

// The element a merge word stands for, as the input holds it: worked out from
// the key, or read from the row at `index` when the key does not say (a zero's
// sign, a NaN's payload), which saves the round trip to memory in most calls.
template <typename E>
__device__ __forceinline__ typename E::raw_t element_of(const typename MergeWord<E>::word_t& w,
                                                        const typename E::raw_t* __restrict__ xr,
                                                        int64_t index) {
  const typename E::key_t key = MergeWord<E>::key(w);
  typename E::raw_t value = E::unkey(key);
  if (!E::key_is_exact(key)) value = xr[index];
  return value;
}

// acc and in are ascending lists of N entries (N a power of two); acc becomes
// the N best of both, ascending: the element-wise better of acc and reversed
// `in` is a bitonic sequence holding exactly those, which half-cleaners sort.
template <typename M, int N>
__device__ __forceinline__ void merge_best(typename M::word_t (&acc)[N], const typename M::word_t (&in)[N]) {
  ATK_STATIC_FOR(i, N) { if (M::better(in[N - 1 - i], acc[i])) acc[i] = in[N - 1 - i]; } ATK_STATIC_END;
  auto order = [&](auto lo, auto hi) __attribute__((always_inline)) {
    const bool swap = M::better(acc[lo], acc[hi]);
    const typename M::word_t a = acc[lo], b = acc[hi];
    acc[lo] = swap ? b : a;
    acc[hi] = swap ? a : b;
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  static_assert(N == 1 || N == 2 || N == 4, "queues hold at most four entries");
  if constexpr (N == 4) { order(I0{}, I2{}); order(I1{}, I3{}); order(I0{}, I1{}); order(I2{}, I3{}); }
  if constexpr (N == 2) { order(I0{}, I1{}); }
}

// The last step of a workgroup that scanned a folded row or slab (wave 0, all
// 64 lanes, after the waves' queues are folded): the `fold` scanned columns of
// every bucket are merged and the bucket's entries written, as the final
// result or as the slab's partial queue.  The queues go to LDS as merge words;
// cb lanes (a power of two) then cover cb buckets at a time with 64/cb lanes
// per bucket, which share out the bucket's columns and combine pairwise by
// lane shuffles.
template <typename E, int J, int V, typename Queue>
__device__ __forceinline__ void fold_columns(const typename E::raw_t* __restrict__ xr, const Geom& g,
                                             const Sink<typename E::raw_t>& out, int64_t row, uint32_t slab,
                                             int64_t col, bool live, uint32_t lane, const Queue& queue,
                                             unsigned char* lds) {
  using M = MergeWord<E>;
  using word_t = typename M::word_t;
  constexpr int N = J == 3 ? 4 : J;
  word_t* words = reinterpret_cast<word_t*>(lds);  // [scanned column][J]
  const uint32_t b = (uint32_t)g.b / g.fold;       // buckets
  if (live) {
    ATK_STATIC_FOR(v, V) {
      const uint32_t cw = (uint32_t)col + v;
      const uint32_t f = cw / b;
      ATK_STATIC_FOR(sl, J) {
        words[cw * J + sl] = M::make(queue.template raw<v, sl>(), queue.template position<v, sl>() * g.fold + f);
      } ATK_STATIC_END;
    } ATK_STATIC_END;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  uint32_t cb = kWave;
  while (cb > 1 && cb / 2 >= b) cb /= 2;
  const uint32_t share = lane / cb, shares = kWave / cb;
  for (uint32_t c0 = 0; c0 < b; c0 += cb) {  // the same trips for every lane
    const uint32_t c = c0 + lane % cb;
    word_t acc[N], in[N];
    ATK_STATIC_FOR(sl, N) { acc[sl] = M::empty(); in[sl] = M::empty(); } ATK_STATIC_END;
    if (c < b) {
      for (uint32_t f = share; f < g.fold; f += shares) {
        ATK_STATIC_FOR(sl, J) { in[N - J + sl] = words[(f * b + c) * J + sl]; } ATK_STATIC_END;
        merge_best<M, N>(acc, in);
      }
    }
    for (uint32_t half = shares / 2; half >= 1; half /= 2) {
      ATK_STATIC_FOR(sl, N) { in[sl] = M::from_lane(acc[sl], (int)(lane + half * cb)); } ATK_STATIC_END;
      merge_best<M, N>(acc, in);  // meaningful in the lanes with share < half, which are the ones read next
    }
    if (share == 0 && c < b) {
      ATK_STATIC_FOR(sl, J) {
        const uint32_t p = M::pos(acc[N - J + sl]);  // the entry's number within its bucket
        const int64_t index = c + (int64_t)p * b;
        const typename E::raw_t value = element_of<E>(acc[N - J + sl], xr, index);
        if (out.part_values == nullptr) {
          const int64_t o = (row * b + c) * J + sl;
          if (out.values != nullptr) out.values[o] = value;
          out.indices.put(o, index);
        } else {
          const int64_t o = ((row * g.slabs + slab) * b + c) * J + sl;
          out.part_values[o] = value;
          out.part_pos[o] = p;
        }
      } ATK_STATIC_END;
    }
  }
}

// The same result through order keys, one lane per bucket walking the bucket's
// part of the scanned sub-rows [s0, s1) (and, with `tail`, what follows the
// last full scanned sub-row): taken when the workgroup met a value the fast
// queues cannot order.
template <typename E, int J>
__device__ __forceinline__ void fold_columns_exact(const typename E::raw_t* __restrict__ xr, const Geom& g,
                                                   const Sink<typename E::raw_t>& out, int64_t row,
                                                   uint32_t slab, uint32_t s0, uint32_t s1, bool tail,
                                                   uint32_t lane) {
  using raw_t = typename E::raw_t;
  const uint32_t b = (uint32_t)g.b / g.fold;
  const uint32_t first = s0 * g.fold;
  const uint32_t length = s1 * g.fold + (tail ? g.rem / b : 0u), rem = tail ? g.rem % b : 0u;
  for (uint32_t c = lane; c < b; c += kWave) {
    raw_t val[J];
    uint32_t pos[J];
    clear_exact<E, J>(val, pos);
    for (uint32_t p = first; p < length; ++p) push_exact<E, J>(val, pos, xr[(int64_t)p * b + c], p);
    if (rem != 0) {
      if (c < rem) push_exact<E, J>(val, pos, xr[(int64_t)length * b + c], length);
      else if (g.pad_tail) push_exact<E, J>(val, pos, E::pad_raw, length);
    }
    if (out.part_values == nullptr) {
      const int64_t o = (row * b + c) * J;
#pragma unroll
      for (int s = 0; s < J; ++s) {
        if (out.values != nullptr) out.values[o + s] = val[s];
        out.indices.put(o + s, c + (int64_t)pos[s] * b);
      }
    } else {
      const int64_t o = ((row * g.slabs + slab) * b + c) * J;
#pragma unroll
      for (int s = 0; s < J; ++s) { out.part_values[o + s] = val[s]; out.part_pos[o + s] = pos[s]; }
    }
  }
}

// E: element traits; J: entries kept per bucket; V: columns per lane; W: waves
// per workgroup, sharing one column tile and splitting its sub-rows; U: loads
// kept in flight per lane; RUN: exact sub-rows per wave when known (else 0);
// PACKED: packed 16-bit queues; WAVE_STORES: final results leave through LDS
// (emit_transposed; a kernel of its own rather than a branch: with both ways
// out in one kernel, fp16 [256, 2^20] k=4096 j=2 took 117 instead of 110 us the
// usual way).
template <typename E, int J, int V, int W, int U, int RUN, bool PACKED, bool WAVE_STORES = false>
__global__ __launch_bounds__(kWave * W) __attribute__((amdgpu_waves_per_eu(4))) void stream_kernel(
    const typename E::raw_t* __restrict__ x, const Sink<typename E::raw_t> out, const Geom g,
    const KeyRangeOut ranges) {
  using raw_t = typename E::raw_t;
  using Queue = QueueFor<E, J, V, PACKED>;
  constexpr int kTileCols = kWave * V;

  const uint32_t lane = threadIdx.x % kWave;
  // Everything that decides control flow is wave-uniform; say so, so that it
  // lives in scalar registers.
  const uint32_t wave = W > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) : 0;
  uint32_t blk = blockIdx.x;
  const uint32_t col_tile = __builtin_amdgcn_readfirstlane(blk % g.col_tiles);
  blk /= g.col_tiles;
  const uint32_t slab = __builtin_amdgcn_readfirstlane(blk % g.slabs);
  const int64_t row = __builtin_amdgcn_readfirstlane(blk / g.slabs);

  const int64_t col = (int64_t)col_tile * kTileCols + lane * V;
  const bool live = col < g.b;  // b is a multiple of V whenever V > 1

  // sub-rows of this slab [s0, s1), then of this wave [p0, p1)
  const uint32_t s0 = slab * g.slab_len;
  const uint32_t s1 = (slab + 1 == g.slabs) ? g.full_rows : s0 + g.slab_len;
  const uint32_t p0 = __builtin_amdgcn_readfirstlane(s0 + (uint32_t)(((uint64_t)(s1 - s0) * wave) / W));
  const uint32_t p1 = __builtin_amdgcn_readfirstlane(s0 + (uint32_t)(((uint64_t)(s1 - s0) * (wave + 1)) / W));
  const bool last_slab = slab + 1 == g.slabs;

  const raw_t* xr = x + row * g.row_stride;
  Queue queue;
  ATK_TRACE_WAVE((int)wave * 2);  // slots 2w, 2w + 1: wave w's scan; 16: the workgroup's end
  scan_run<E, J, V, U, RUN>(xr, g, col, live, p0, p1, last_slab && wave == W - 1, queue);
  ATK_TRACE_WAVE((int)wave * 2 + 1);

  bool redo = queue.poisoned();
  // LDS: the hand-over area of waves 1.., later the merge words of a folded row
  using word_t = typename MergeWord<E>::word_t;
  constexpr size_t kHandArea = (size_t)(W - 1) * Queue::kHandBytes;
  constexpr size_t kWordArea = (size_t)kTileCols * J * sizeof(word_t);
  // final results leave through LDS, in whole-wave stores of adjacent bytes
  constexpr bool kTransposed = WAVE_STORES;
  static_assert(!WAVE_STORES || Transposed<E, J, V>::available, "see Transposed");
  constexpr size_t kOutArea = kTransposed ? Transposed<E, J, V>::kBytes : 0;
  constexpr size_t kLdsArea = kHandArea > kWordArea ? (kHandArea > kOutArea ? kHandArea : kOutArea)
                                                    : (kWordArea > kOutArea ? kWordArea : kOutArea);
  __shared__ __align__(16) unsigned char lds[kLdsArea];
  if constexpr (W > 1) {
    // waves 1.. hand their queues to wave 0 through LDS
    if (wave > 0) queue.hand_over(lds + (size_t)(wave - 1) * Queue::kHandBytes, lane);
    redo = __syncthreads_or(redo);
    if (wave > 0) return;
    if (!redo) {
#pragma nounroll
      for (int w = 0; w < W - 1; ++w) queue.fold_in(lds + (size_t)w * Queue::kHandBytes, lane);
    }
  }
  // order keys of what this workgroup leaves, smallest and largest (all keys
  // when that is not worked out: any range that holds them will do)
  uint32_t low = 0u, high = ~0u;
  if (g.fold > 1) {
    if (redo) {
      fold_columns_exact<E, J>(xr, g, out, row, slab, s0, s1, last_slab, lane);
    } else {
      if (live) queue.fix_zeros(xr, g.b, col);
      fold_columns<E, J, V>(xr, g, out, row, slab, col, live, lane, queue, lds);
    }
  } else if (!live) {
    low = ~0u; high = 0u;
  } else if (redo) {
    exact_columns<E, J, V>(xr, g, out, row, slab, col, s0, W > 1 ? s1 : p1, last_slab);
  } else {
    queue.fix_zeros(xr, g.b, col);
    if constexpr (!kTransposed) emit<E, J, V>(g, out, row, slab, col, queue);
    if constexpr (E::key_bits <= 32) {
      if (ranges.range != nullptr) {
        low = ~0u; high = 0u;
        ATK_STATIC_FOR(e, V * J) {
          const uint32_t key = (uint32_t)queue.template key<e / J, e % J>();
          low = key < low ? key : low;
          high = key > high ? key : high;
        } ATK_STATIC_END;
      }
    }
  }
  if constexpr (kTransposed) {
    // (wave-uniform: whole waves get here, the lanes beyond the row's last column included)
    if (!redo) emit_transposed<E, J, V>(g, out, row, (int64_t)col_tile * kTileCols, lane, queue, lds);
  }
  if constexpr (E::key_bits <= 32) {
    if (ranges.range != nullptr) {
      // For the chained select that follows the merge of the slabs
      // (stage2_chain_select.hip): the key range of this workgroup's queues, and
      // this workgroup's share of that select's histogram and row state cleared.
      namespace regs = select::regs;
      low = regs::wave_min(low);
      high = regs::wave_max(high);
      const uint32_t blocks_per_row = g.slabs * g.col_tiles;
      const uint32_t block = slab * g.col_tiles + col_tile;
      if (lane == 0) ranges.range[(size_t)row * blocks_per_row + block] = make_uint2(low, high);
      uint32_t* h = ranges.hist + (size_t)row * ranges.hist_words;
      for (uint32_t i = block * kWave + lane; i < ranges.hist_words; i += blocks_per_row * kWave) h[i] = 0;
      if (block == 0 && lane < ranges.state_words) ranges.state[(size_t)row * ranges.state_words + lane] = 0;
    }
  }
  ATK_TRACE_WAVE(16);
}

// Folds the slabs' partial queues of every bucket into the final result under
// the full order (order key, then lower index); an entry's position is its
// number within the bucket.  A workgroup of 256 threads covers `cb` buckets (a
// power of two up to 64) with 256/cb threads per bucket, which share the slabs
// out and then combine pairwise through LDS.  Every partial queue arrives
// ascending, so combining two is a merge network, not J insertions.  The
// winners' values are the input's bit patterns (`element_of`).
constexpr int kMergeThreads = 256;

template <typename E, int J>
__global__ __launch_bounds__(kMergeThreads) void stream_merge_kernel(
    const typename E::raw_t* __restrict__ x, int64_t row_stride,
    const typename E::raw_t* __restrict__ part_values, const uint32_t* __restrict__ part_pos,
    int64_t b, uint32_t slabs, uint32_t cb, uint32_t blocks_per_row,
    typename E::raw_t* __restrict__ values, const IndexOut indices, const KeyRangeOut ranges) {
  using M = MergeWord<E>;
  using word_t = typename M::word_t;
  constexpr int N = J == 3 ? 4 : J;  // list length of the merge network
  __shared__ word_t lds[N][kMergeThreads];
  const uint32_t t = threadIdx.x;
  const uint32_t share = t / cb, shares = kMergeThreads / cb;
  const uint32_t row32 = blockIdx.x / blocks_per_row;
  const int64_t row = row32;
  const int64_t c = (int64_t)(blockIdx.x - row32 * blocks_per_row) * cb + t % cb;
  const bool live = c < b;
  word_t acc[N], in[N];
  ATK_STATIC_FOR(s, N) { acc[s] = M::empty(); in[s] = M::empty(); } ATK_STATIC_END;
  if (live) {
    // four slabs per round, their loads issued together
    constexpr int kBatch = 4;
    for (uint32_t slab0 = share; slab0 < slabs; slab0 += shares * kBatch) {
      typename E::raw_t got[kBatch][J];
      uint32_t at[kBatch][J];
      bool real[kBatch];
      ATK_STATIC_FOR(u, kBatch) {
        const uint32_t slab = slab0 + u * shares;
        real[u] = slab < slabs;
        const int64_t o = ((row * slabs + (real[u] ? slab : share)) * b + c) * J;  // a slab that exists
        ATK_STATIC_FOR(s, J) { got[u][s] = part_values[o + s]; at[u][s] = part_pos[o + s]; } ATK_STATIC_END;
      } ATK_STATIC_END;
      ATK_STATIC_FOR(u, kBatch) {
        if (real[u]) {
          ATK_STATIC_FOR(s, J) { in[N - J + s] = M::make(got[u][s], at[u][s]); } ATK_STATIC_END;
          merge_best<M, N>(acc, in);
        }
      } ATK_STATIC_END;
    }
  }
  for (uint32_t half = shares / 2; half >= 1; half /= 2) {
    if (share >= half && share < 2 * half) {
      ATK_STATIC_FOR(s, N) { lds[s][t] = acc[s]; } ATK_STATIC_END;
    }
    __syncthreads();
    if (share < half) {
      ATK_STATIC_FOR(s, N) { in[s] = lds[s][t + half * cb]; } ATK_STATIC_END;
      merge_best<M, N>(acc, in);
    }
  }
  const bool writer = share == 0 && live;
  if (writer) {
    const typename E::raw_t* xr = x + row * row_stride;
    const int64_t o = (row * b + c) * J;
    ATK_STATIC_FOR(s, J) {
      const int64_t index = c + (int64_t)M::pos(acc[N - J + s]) * b;
      if (values != nullptr) values[o + s] = element_of<E>(acc[N - J + s], xr, index);
      indices.put(o + s, index);
    } ATK_STATIC_END;
  }
  if constexpr (E::key_bits <= 32) {
    if (ranges.range != nullptr) {
      // For the chained select that follows (stage2_chain_select.hip): the
      // digits of this workgroup's results added to the row's histogram, which
      // the scanning kernel cleared; the digit's place comes from the key ranges
      // that kernel left of its queues, which hold every result.
      // (Added up in LDS first: thousands of atomic adds to the few words of
      // the crowded digits, straight to memory, take hundreds of microseconds.)
      namespace regs = select::regs;
      __shared__ uint32_t red[2 * kMergeThreads / kWave];
      __shared__ uint32_t local[regs::kHistWords];
      for (uint32_t i = t; i < (uint32_t)regs::kHistWords; i += kMergeThreads) local[i] = 0;
      uint32_t low, shift;
      regs::digit_of_row<kMergeThreads>(ranges.range + (size_t)row32 * ranges.entries, ranges.entries, red, low, shift);
      if (writer) {  // (the barrier in digit_of_row also covers the clearing)
        ATK_STATIC_FOR(s, J) {
          const uint32_t key = (uint32_t)M::key(acc[N - J + s]);
          atomicAdd(&local[regs::hist_slot((key - low) >> shift)], 1u);
        } ATK_STATIC_END;
      }
      __syncthreads();
      uint32_t* h = ranges.hist + (size_t)row32 * ranges.hist_words;
      for (uint32_t i = t; i < (uint32_t)regs::kHistWords; i += kMergeThreads) {
        const uint32_t c = local[i];
        if (c != 0) atomicAdd(&h[i], c);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Host side: the plan (pure arithmetic, shared with the workspace query) and
// the launch.
// ---------------------------------------------------------------------------
struct Plan {
  bool ok;            // the streaming kernels accept this shape
  int vec;            // V: elements per load (16 bytes' worth, or 1)
  int waves;          // W: waves per workgroup (1, 2, 4 or 8)
  bool packed;        // packed 16-bit queues (16-bit element type, short enough rows)
  int run;            // sub-rows per wave when every wave gets exactly 4 or 8, else 0
  uint32_t fold;      // sub-rows of the true matrix per scanned sub-row (1: not folded)
  int64_t width;      // scanned columns per row: buckets * fold
  uint32_t full_rows, rem, pad_tail;  // of the scanned matrix
  uint32_t slabs, slab_len, col_tiles;
  bool merge;         // the merge kernel follows (several slabs)
  bool wave_stores;   // final results leave through LDS in whole-wave stores
  size_t part_values_off, part_pos_off, ws_bytes;
};

// `aligned`: base pointers and row stride allow 16-byte accesses.
Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype, bool aligned);

// One instance per element type, each in its own translation unit.
// `ranges`: see KeyRangeOut; may be nullptr.
template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int j, void* values,
                 IndexOut indices, void* ws, hipStream_t stream, KeyRangeOut* ranges);

}  // namespace stream
}  // namespace atk
