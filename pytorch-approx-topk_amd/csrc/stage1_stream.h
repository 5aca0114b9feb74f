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

namespace atk {
namespace stream {

constexpr int kWave = 64;

// Columns per lane with vector loads: 16 bytes' worth, but at most 8 columns so
// that the queues of one lane stay in registers.
__host__ __device__ constexpr int full_vec(int elem_size) { return elem_size == 1 ? 8 : 16 / elem_size; }

// LDS a workgroup of `waves` needs to hand the queues of waves 1.. to wave 0,
// and the most the planner lets it use.
__host__ __device__ constexpr size_t merge_lds_bytes(int vec, int j, int waves, int cmp_size) {
  return (size_t)(waves - 1) * vec * j * kWave * (cmp_size + 4);
}
constexpr size_t kMergeLdsLimit = 48 * 1024;

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
  __device__ __forceinline__ void fix_zeros(const raw_t* __restrict__, int64_t, int64_t) {}
  // exact order key of an entry (the queues are not poisoned)
  template <int VI, int SI> __device__ __forceinline__ typename E::key_t key() const { return E::key(C::to_raw(q[VI][SI])); }
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
  // the raw half of a key; a zero key gives +0.0
  __device__ static __forceinline__ uint16_t unkey(uint32_t key) {
    return (uint16_t)((key & 0x8000u) ? (key ^ 0x8000u) : (0u - key));
  }
};
template <> struct PackedKey<Elem<ATK_F16>> : PackedKeyFloat16<0x7c00u> {};
template <> struct PackedKey<Elem<ATK_BF16>> : PackedKeyFloat16<0x7f80u> {};
template <> struct PackedKey<Elem<ATK_I16>> {
  static constexpr bool available = true;
  static constexpr bool zero_is_ambiguous = false;
  static constexpr uint32_t kZeroKey = 0x8000u;
  __device__ static __forceinline__ uint32_t keys2(uint32_t x, uint32_t&) { return x ^ 0x80008000u; }
  __device__ static __forceinline__ bool special(uint32_t) { return false; }
  __device__ static __forceinline__ uint16_t unkey(uint32_t key) { return (uint16_t)(key ^ 0x8000u); }
};

// largest sub-row number (the partial sub-row included) a packed entry can hold
constexpr uint32_t kPackedMaxSubRow = 0xfffeu;

template <typename E, int J, int V> struct PackedQueue {
  using raw_t = typename E::raw_t;
  using K = PackedKey<E>;
  static_assert(sizeof(raw_t) == 2 && (V % 2 == 0 || V == 1), "packed queues hold 16-bit elements");
  static constexpr size_t kHandBytes = (size_t)V * J * kWave * 4;

  uint32_t q[V][J];
  uint32_t screen;     // NaN screen, two halves
  uint32_t neg_zeros;  // bit v*J+s: entry (v, s) is a -0.0 (set by fix_zeros)

  __device__ __forceinline__ void reset() {
    ATK_STATIC_FOR(e, V * J) { q[e / J][e % J] = 0; } ATK_STATIC_END;
    screen = 0;
    neg_zeros = 0;
  }
  __device__ static __forceinline__ uint32_t med3(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r;
    asm("v_med3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
  }
  // col is ascending; the median of (col[s], word, col[s+1]) is the new col[s]
  __device__ static __forceinline__ void insert(uint32_t (&col)[J], uint32_t word) {
    ATK_STATIC_FOR(s, J - 1) { col[s] = med3(col[s], word, col[s + 1]); } ATK_STATIC_END;
    col[J - 1] = col[J - 1] > word ? col[J - 1] : word;
  }
  template <int FILLED> __device__ __forceinline__ void take(const Pack<raw_t, V>& pk, uint32_t p) {
    const uint32_t pinv = 0xffffu - p;
    if constexpr (V == 1) {
      const uint32_t keys = K::keys2(pk.e[0], screen);
      insert(q[0], (keys << 16) | pinv);
    } else {
      ATK_STATIC_FOR(d, V / 2) {
        uint32_t x;  // elements 2d (low half) and 2d+1 (high half) as loaded
        __builtin_memcpy(&x, &pk.e[2 * d], 4);
        const uint32_t keys = K::keys2(x, screen);
        insert(q[2 * d], (keys << 16) | pinv);
        insert(q[2 * d + 1], (keys & 0xffff0000u) | pinv);
      } ATK_STATIC_END;
    }
  }
  // one more element for column VI, when `valid` (the word 0 changes nothing)
  template <int VI> __device__ __forceinline__ void take_one(raw_t raw, uint32_t p, bool valid) {
    uint32_t scr = screen;
    const uint32_t keys = K::keys2((uint32_t)raw, scr);  // the empty high half screens as +0
    if (valid) screen = scr;
    insert(q[VI], valid ? ((keys << 16) | (0xffffu - p)) : 0u);
  }
  __device__ __forceinline__ bool poisoned() const { return __ballot(K::special(screen)) != 0; }

  __device__ __forceinline__ void hand_over(unsigned char* area, uint32_t lane) const {
    uint32_t* h = reinterpret_cast<uint32_t*>(area);
    ATK_STATIC_FOR(e, V * J) { h[e * kWave + lane] = q[e / J][e % J]; } ATK_STATIC_END;
  }
  __device__ __forceinline__ void fold_in(const unsigned char* area, uint32_t lane) {
    const uint32_t* h = reinterpret_cast<const uint32_t*>(area);
    ATK_STATIC_FOR(e, V * J) { insert(q[e / J], h[e * kWave + lane]); } ATK_STATIC_END;
  }
  // Final entries with a zero key are re-read from the row to learn their sign.
  // `col` is the lane's first column; call once, after the last fold, by live lanes.
  __device__ __forceinline__ void fix_zeros(const raw_t* __restrict__ xr, int64_t b, int64_t col) {
    if constexpr (K::zero_is_ambiguous) {
      bool any = false;
      ATK_STATIC_FOR(e, V * J) { any |= (q[e / J][e % J] >> 16) == K::kZeroKey; } ATK_STATIC_END;
      if (__ballot(any) == 0) return;
      ATK_STATIC_FOR(e, V * J) {
        const uint32_t word = q[e / J][e % J];
        if ((word >> 16) == K::kZeroKey) {
          const uint32_t p = 0xffffu - (word & 0xffffu);
          if (xr[(int64_t)p * b + col + e / J] == (raw_t)0x8000u) neg_zeros |= 1u << e;
        }
      } ATK_STATIC_END;
    }
  }
  // exact order key of an entry: without NaN the packed key is the exact key
  template <int VI, int SI> __device__ __forceinline__ typename E::key_t key() const { return q[VI][SI] >> 16; }
  template <int VI, int SI> __device__ __forceinline__ raw_t raw() const {
    const raw_t r = K::unkey(q[VI][SI] >> 16);
    if constexpr (K::zero_is_ambiguous) return (neg_zeros >> (VI * J + SI)) & 1u ? (raw_t)0x8000u : r;
    return r;
  }
  template <int VI, int SI> __device__ __forceinline__ uint32_t position() const { return 0xffffu - (q[VI][SI] & 0xffffu); }
};

template <typename E, int J, int V, bool PACKED>
using QueueFor = std::conditional_t<PACKED, PackedQueue<E, J, V>, CmpQueue<E, J, V>>;

// Shape of one launch; passed to the kernels by value.
struct Geom {
  int64_t row_stride;     // elements between rows
  int64_t b;              // buckets (columns) per row
  uint32_t full_rows;     // L = n / b
  uint32_t rem;           // n mod b: columns that have one more element
  uint32_t pad_tail;      // padded row: the other columns hold the pad value there
  uint32_t slabs;         // sub-row slabs per row
  uint32_t slab_len;      // sub-rows per slab (the last slab takes the rest)
  uint32_t col_tiles;     // workgroup column tiles per row
};

// Where results go: final values/indices[rows][b*J] when there is one slab,
// else per-slab queues [rows][slabs][b*J] (raw values and sub-row numbers).
template <typename raw_t> struct Sink {
  raw_t* values;
  int64_t* indices;
  raw_t* part_values;
  uint32_t* part_pos;
};

// Writes the queues of this lane's V columns, either as final results or as a
// slab's partial result.
template <typename E, int J, int V, typename Queue>
__device__ __forceinline__ void emit(const Geom& g, const Sink<typename E::raw_t>& out, int64_t row,
                                     uint32_t slab, int64_t col, const Queue& queue) {
  using raw_t = typename E::raw_t;
  if (g.slabs == 1) {
    const int64_t o = (row * g.b + col) * J;
    raw_t* ov = out.values + o;
    int64_t* oi = out.indices + o;
    if constexpr (V > 1) {
      // V*J values = J stores of V elements; V*J int64 = V*J/2 16-byte stores
      ATK_STATIC_FOR(t, J) {
        Pack<raw_t, V> pv;
        ATK_STATIC_FOR(e, V) { pv.e[e] = queue.template raw<(t * V + e) / J, (t * V + e) % J>(); } ATK_STATIC_END;
        reinterpret_cast<Pack<raw_t, V>*>(ov)[t] = pv;
      } ATK_STATIC_END;
      ATK_STATIC_FOR(t, V * J / 2) {
        Pack<int64_t, 2> pi;
        ATK_STATIC_FOR(e, 2) {
          constexpr int v = (t * 2 + e) / J, sl = (t * 2 + e) % J;
          pi.e[e] = col + v + (int64_t)queue.template position<v, sl>() * g.b;
        } ATK_STATIC_END;
        reinterpret_cast<Pack<int64_t, 2>*>(oi)[t] = pi;
      } ATK_STATIC_END;
    } else {
      ATK_STATIC_FOR(sl, J) {
        ov[sl] = queue.template raw<0, sl>();
        oi[sl] = col + (int64_t)queue.template position<0, sl>() * g.b;
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
    if (g.slabs == 1) {
      const int64_t o = (row * g.b + c) * J;
#pragma unroll
      for (int s = 0; s < J; ++s) { out.values[o + s] = val[s]; out.indices[o + s] = c + (int64_t)pos[s] * g.b; }
    } else {
      const int64_t o = ((row * g.slabs + slab) * g.b + c) * J;
#pragma unroll
      for (int s = 0; s < J; ++s) { out.part_values[o + s] = val[s]; out.part_pos[o + s] = pos[s]; }
    }
  }
}

// One wave's scan: folds sub-rows [p0, p1) (p1 - p0 >= J) of this lane's V
// columns starting at `col` into `queue`, plus the row's partial sub-row when
// `with_rem`.  `xr` is the row; lanes that are not `live` load column 0 and are
// ignored by the caller.  RUN > 0 promises p1 - p0 == RUN (J <= RUN): all loads
// are issued at once and the code is one straight line.  RUN == 0 takes any
// length: the first J sub-rows, then an odd batch of fewer than U, then batches
// of U that are refilled while they are consumed.  Loads and their uses are
// kept in the same basic block wherever a load is outstanding across them, so
// that the wait counts are exact.
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
    uint32_t p = p0;
    {  // the first J sub-rows fill the queues
      Pack<raw_t, V> buf[J];
#pragma unroll
      for (int u = 0; u < J; ++u) buf[u] = load_next();
      ATK_STATIC_FOR(u, J) { queue.template take<u>(buf[u], p0 + u); } ATK_STATIC_END;
      p += J;
    }
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
  // the partial sub-row: column c has one more element when c < rem
  // (with a padded row the other columns see the pad value there)
  if (with_rem && g.rem != 0) {
    ATK_STATIC_FOR(v, V) {
      const bool real = live && col + v < (int64_t)g.rem;
      const raw_t* at = real ? xr + (int64_t)g.full_rows * g.b + col + v : xr;  // xr[0] always exists
      const raw_t value = *at;
      queue.template take_one<v>(real ? value : E::pad_raw, g.full_rows, real || (live && g.pad_tail != 0));
    } ATK_STATIC_END;
  }
}

// E: element traits; J: entries kept per bucket; V: columns per lane; W: waves
// per workgroup, sharing one column tile and splitting its sub-rows; U: loads
// kept in flight per lane; RUN: exact sub-rows per wave when known (else 0);
// PACKED: packed 16-bit queues.
template <typename E, int J, int V, int W, int U, int RUN, bool PACKED>
__global__ __launch_bounds__(kWave * W) __attribute__((amdgpu_waves_per_eu(4))) void stream_kernel(
    const typename E::raw_t* __restrict__ x, const Sink<typename E::raw_t> out, const Geom g) {
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
  scan_run<E, J, V, U, RUN>(xr, g, col, live, p0, p1, last_slab && wave == W - 1, queue);

  bool redo = queue.poisoned();
  if constexpr (W > 1) {
    // waves 1.. hand their queues to wave 0 through LDS
    __shared__ __align__(16) unsigned char hand[(W - 1) * Queue::kHandBytes];
    if (wave > 0) queue.hand_over(hand + (size_t)(wave - 1) * Queue::kHandBytes, lane);
    redo = __syncthreads_or(redo);
    if (wave > 0) return;
    if (!redo) {
#pragma nounroll
      for (int w = 0; w < W - 1; ++w) queue.fold_in(hand + (size_t)w * Queue::kHandBytes, lane);
    }
  }
  if (!live) return;
  if (redo) {
    exact_columns<E, J, V>(xr, g, out, row, slab, col, s0, W > 1 ? s1 : p1, last_slab);
    return;
  }
  queue.fix_zeros(xr, g.b, col);
  emit<E, J, V>(g, out, row, slab, col, queue);
}

// Folds the per-slab queues of every bucket into the final result with exact
// order keys.  A workgroup of 4 waves covers 64 buckets (one per lane); wave w
// folds a contiguous quarter of the slabs, then waves 1..3 hand their queues to
// wave 0 through LDS.  Slabs are visited in sub-row order and each queue's
// entries best first, so equal values keep the lowest index.
constexpr int kMergeWaves = 4;

template <typename E, int J>
__global__ __launch_bounds__(kWave * kMergeWaves) void stream_merge_kernel(
    const typename E::raw_t* __restrict__ part_values, const uint32_t* __restrict__ part_pos,
    int64_t b, uint32_t slabs, int64_t blocks_per_row, typename E::raw_t* __restrict__ values,
    int64_t* __restrict__ indices) {
  using raw_t = typename E::raw_t;
  __shared__ raw_t lds_q[kMergeWaves - 1][J][kWave];
  __shared__ uint32_t lds_p[kMergeWaves - 1][J][kWave];
  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int64_t row = blockIdx.x / blocks_per_row;
  const int64_t c = (blockIdx.x - row * blocks_per_row) * kWave + lane;
  const bool live = c < b;
  raw_t q[J];
  uint32_t pos[J];
  clear_exact<E, J>(q, pos);
  const uint32_t lo = (uint32_t)(((uint64_t)slabs * wave) / kMergeWaves);
  const uint32_t hi = (uint32_t)(((uint64_t)slabs * (wave + 1)) / kMergeWaves);
  if (live) {
    for (uint32_t slab = lo; slab < hi; ++slab) {
      const int64_t o = ((row * slabs + slab) * b + c) * J;
#pragma unroll
      for (int s = J - 1; s >= 0; --s) push_exact<E, J>(q, pos, part_values[o + s], part_pos[o + s]);
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int s = 0; s < J; ++s) { lds_q[wave - 1][s][lane] = q[s]; lds_p[wave - 1][s][lane] = pos[s]; }
  }
  __syncthreads();
  if (wave > 0 || !live) return;
  for (int w = 1; w < kMergeWaves; ++w) {
    const uint32_t wlo = (uint32_t)(((uint64_t)slabs * w) / kMergeWaves);
    const uint32_t whi = (uint32_t)(((uint64_t)slabs * (w + 1)) / kMergeWaves);
    if (whi == wlo) continue;  // that wave had no slab
#pragma unroll
    for (int s = J - 1; s >= 0; --s) push_exact<E, J>(q, pos, lds_q[w - 1][s][lane], lds_p[w - 1][s][lane]);
  }
  const int64_t o = (row * b + c) * J;
#pragma unroll
  for (int s = 0; s < J; ++s) { values[o + s] = q[s]; indices[o + s] = c + (int64_t)pos[s] * b; }
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
  uint32_t full_rows, rem, pad_tail;
  uint32_t slabs, slab_len, col_tiles;
  size_t part_values_off, part_pos_off, ws_bytes;
};

// `aligned`: base pointers and row stride allow 16-byte accesses.
Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype, bool aligned);

// One instance per element type, each in its own translation unit.
template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int64_t b, int j,
                 void* values, int64_t* indices, void* ws, hipStream_t stream);

}  // namespace stream
}  // namespace atk
