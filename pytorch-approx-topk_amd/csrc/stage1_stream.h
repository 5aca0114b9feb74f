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

// ---------------------------------------------------------------------------
// Compare form of an element type: what the queues hold in the hot loop.
// ---------------------------------------------------------------------------
template <typename E> struct Cmp;

template <> struct Cmp<Elem<ATK_F32>> {
  using cmp_t = float; static constexpr bool has_nan = true;
  __device__ static inline cmp_t from_raw(uint32_t u) { return __uint_as_float(u); }
  __device__ static inline uint32_t to_raw(cmp_t v) { return __float_as_uint(v); }
};
template <> struct Cmp<Elem<ATK_F16>> {
  using cmp_t = float; static constexpr bool has_nan = true;
  __device__ static inline cmp_t from_raw(uint16_t u) {
    _Float16 h; __builtin_memcpy(&h, &u, 2); return (float)h;
  }
  __device__ static inline uint16_t to_raw(cmp_t v) {
    _Float16 h = (_Float16)v; uint16_t u; __builtin_memcpy(&u, &h, 2); return u;
  }
};
template <> struct Cmp<Elem<ATK_BF16>> {
  using cmp_t = float; static constexpr bool has_nan = true;
  __device__ static inline cmp_t from_raw(uint16_t u) { return __uint_as_float((uint32_t)u << 16); }
  __device__ static inline uint16_t to_raw(cmp_t v) { return (uint16_t)(__float_as_uint(v) >> 16); }
};
template <> struct Cmp<Elem<ATK_F64>> {
  using cmp_t = double; static constexpr bool has_nan = true;
  __device__ static inline cmp_t from_raw(uint64_t u) { return __longlong_as_double((long long)u); }
  __device__ static inline uint64_t to_raw(cmp_t v) { return (uint64_t)__double_as_longlong(v); }
};
template <> struct Cmp<Elem<ATK_U8>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static inline cmp_t from_raw(uint8_t u) { return (int)u; }
  __device__ static inline uint8_t to_raw(cmp_t v) { return (uint8_t)v; }
};
template <> struct Cmp<Elem<ATK_I8>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static inline cmp_t from_raw(uint8_t u) { return (int)(int8_t)u; }
  __device__ static inline uint8_t to_raw(cmp_t v) { return (uint8_t)v; }
};
template <> struct Cmp<Elem<ATK_I16>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static inline cmp_t from_raw(uint16_t u) { return (int)(int16_t)u; }
  __device__ static inline uint16_t to_raw(cmp_t v) { return (uint16_t)v; }
};
template <> struct Cmp<Elem<ATK_I32>> {
  using cmp_t = int; static constexpr bool has_nan = false;
  __device__ static inline cmp_t from_raw(uint32_t u) { return (int)u; }
  __device__ static inline uint32_t to_raw(cmp_t v) { return (uint32_t)v; }
};
template <> struct Cmp<Elem<ATK_I64>> {
  using cmp_t = long long; static constexpr bool has_nan = false;
  __device__ static inline cmp_t from_raw(uint64_t u) { return (long long)u; }
  __device__ static inline uint64_t to_raw(cmp_t v) { return (uint64_t)v; }
};

// Compile-time loop: f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>).
template <typename F, int... I>
__device__ inline void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ inline void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// V elements moved by one load instruction.
template <typename raw_t, int V> struct alignas(sizeof(raw_t) * V) Pack { raw_t e[V]; };

template <typename raw_t, int V>
__device__ inline Pack<raw_t, V> load_pack(const raw_t* p) {
  return *reinterpret_cast<const Pack<raw_t, V>*>(p);
}

// ---------------------------------------------------------------------------
// Queue of J entries per column, ascending (slot 0 weakest).  FILLED top slots
// are valid; the lower ones count as beaten by anything.
// ---------------------------------------------------------------------------
template <typename T, int J, int FILLED = J>
__device__ inline void push(T (&q)[J], uint32_t (&pos)[J], T v, uint32_t p) {
  bool beats[J + 1];
#pragma unroll
  for (int s = 0; s < J; ++s) beats[s] = (s < J - FILLED) ? true : (v > q[s]);
  beats[J] = false;
#pragma unroll
  for (int s = 0; s < J; ++s) {
    q[s] = beats[s + 1] ? q[(s + 1 < J) ? s + 1 : s] : (beats[s] ? v : q[s]);
    pos[s] = beats[s + 1] ? pos[(s + 1 < J) ? s + 1 : s] : (beats[s] ? p : pos[s]);
  }
}

// Exact (order-key) push used off the hot path; entries hold raw elements.
template <typename E, int J>
__device__ inline void push_exact(typename E::raw_t (&q)[J], uint32_t (&pos)[J], int& filled,
                                  typename E::raw_t v, uint32_t p) {
  const typename E::key_t kv = E::key(v);
  bool beats[J + 1];
#pragma unroll
  for (int s = 0; s < J; ++s) beats[s] = (s < J - filled) ? true : (kv > E::key(q[s]));
  beats[J] = false;
#pragma unroll
  for (int s = 0; s < J; ++s) {
    q[s] = beats[s + 1] ? q[(s + 1 < J) ? s + 1 : s] : (beats[s] ? v : q[s]);
    pos[s] = beats[s + 1] ? pos[(s + 1 < J) ? s + 1 : s] : (beats[s] ? p : pos[s]);
  }
  if (filled < J) ++filled;
}

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
template <typename E, int J, int V>
__device__ inline void emit(const Geom& g, const Sink<typename E::raw_t>& out, int64_t row,
                            uint32_t slab, int64_t col, const typename E::raw_t (&val)[V][J],
                            const uint32_t (&pos)[V][J]) {
  using raw_t = typename E::raw_t;
  if (g.slabs == 1) {
    const int64_t o = (row * g.b + col) * J;
    raw_t* ov = out.values + o;
    int64_t* oi = out.indices + o;
    if constexpr (V > 1) {
      // V*J values = J 16-byte stores; V*J int64 = V*J/2 16-byte stores
      Pack<raw_t, V> pv[J];
      Pack<int64_t, 2> pi[V * J / 2];
#pragma unroll
      for (int v = 0; v < V; ++v)
#pragma unroll
        for (int s = 0; s < J; ++s) {
          pv[(v * J + s) / V].e[(v * J + s) % V] = val[v][s];
          pi[(v * J + s) / 2].e[(v * J + s) % 2] = col + v + (int64_t)pos[v][s] * g.b;
        }
#pragma unroll
      for (int t = 0; t < J; ++t) reinterpret_cast<Pack<raw_t, V>*>(ov)[t] = pv[t];
#pragma unroll
      for (int t = 0; t < V * J / 2; ++t) reinterpret_cast<Pack<int64_t, 2>*>(oi)[t] = pi[t];
    } else {
#pragma unroll
      for (int s = 0; s < J; ++s) { ov[s] = val[0][s]; oi[s] = col + (int64_t)pos[0][s] * g.b; }
    }
  } else {
    const int64_t o = ((row * g.slabs + slab) * g.b + col) * J;
    raw_t* ov = out.part_values + o;
    uint32_t* op = out.part_pos + o;
#pragma unroll
    for (int v = 0; v < V; ++v)
#pragma unroll
      for (int s = 0; s < J; ++s) { ov[v * J + s] = val[v][s]; op[v * J + s] = pos[v][s]; }
  }
}

// Exact recomputation of one lane's V columns over sub-rows [p0, p1) (plus the
// partial sub-row when `with_rem`), through order keys.  Off the hot path.
template <typename E, int J, int V>
__device__ inline void exact_columns(const typename E::raw_t* __restrict__ xr, const Geom& g,
                                     const Sink<typename E::raw_t>& out, int64_t row, uint32_t slab,
                                     int64_t col, uint32_t p0, uint32_t p1, bool with_rem) {
  using raw_t = typename E::raw_t;
  raw_t val[V][J];
  uint32_t pos[V][J];
#pragma unroll
  for (int v = 0; v < V; ++v)
#pragma unroll
    for (int s = 0; s < J; ++s) { val[v][s] = 0; pos[v][s] = 0; }
  int filled = 0;  // the V columns fill in step
  for (uint32_t p = p0; p < p1; ++p) {
    int f = filled;
#pragma unroll
    for (int v = 0; v < V; ++v) {
      f = filled;
      push_exact<E, J>(val[v], pos[v], f, xr[(int64_t)p * g.b + col + v], p);
    }
    filled = f;
  }
  if (with_rem && g.rem != 0) {
#pragma unroll
    for (int v = 0; v < V; ++v) {
      int f = filled;
      if (col + v < (int64_t)g.rem)
        push_exact<E, J>(val[v], pos[v], f, xr[(int64_t)g.full_rows * g.b + col + v], g.full_rows);
      else if (g.pad_tail)
        push_exact<E, J>(val[v], pos[v], f, E::pad_raw, g.full_rows);
    }
  }
  emit<E, J, V>(g, out, row, slab, col, val, pos);
}

// One wave's scan: the top J of sub-rows [p0, p1) (p1 - p0 >= J) for this lane's V
// columns starting at `col`, plus the row's partial sub-row when `with_rem`.
// `xr` is the row; lanes that are not `live` load column 0 and are ignored by
// the caller.  U loads stay in flight per lane.  Sets bits in `nan_mask`
// (wave-uniform) for lanes that loaded a NaN; the queues are meaningless then.
template <typename E, int J, int V, int U>
__device__ inline void scan_run(const typename E::raw_t* __restrict__ xr, const Geom& g, int64_t col,
                                bool live, uint32_t p0, uint32_t p1, bool with_rem,
                                typename Cmp<E>::cmp_t (&q)[V][J], uint32_t (&pos)[V][J],
                                uint64_t& nan_mask) {
  using raw_t = typename E::raw_t;
  using C = Cmp<E>;
  using cmp_t = typename C::cmp_t;
  static_assert(U >= J, "the first U loads must cover the J sub-rows that fill the queues");
  // `next` walks down this lane's columns one sub-row per load
  const raw_t* next = xr + (live ? col : 0) + (int64_t)p0 * g.b;
  auto load_next = [&]() {
    const Pack<raw_t, V> pk = load_pack<raw_t, V>(next);
    next += g.b;
    return pk;
  };
  auto take = [&](const Pack<raw_t, V>& pk, uint32_t p, auto filled_tag) {
    constexpr int FILLED = decltype(filled_tag)::value;
    cmp_t c[V];
#pragma unroll
    for (int v = 0; v < V; ++v) c[v] = C::from_raw(pk.e[v]);
    if constexpr (C::has_nan) {
#pragma unroll
      for (int v = 0; v + 1 < V; v += 2) nan_mask |= __ballot(__builtin_isunordered(c[v], c[v + 1]));
      if constexpr (V % 2 != 0) nan_mask |= __ballot(__builtin_isunordered(c[V - 1], c[V - 1]));
    }
#pragma unroll
    for (int v = 0; v < V; ++v) push<cmp_t, J, FILLED>(q[v], pos[v], c[v], p);
  };

  // Slot u of `buf` holds sub-row p + u; consuming it frees the slot for
  // sub-row p + U + u.  `ld` is the next sub-row to load.
  Pack<raw_t, V> buf[U];
  uint32_t ld = p0;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (ld < p1) { buf[u] = load_next(); ++ld; }
  }
  uint32_t p = p0;
  // first group: also fills the queues
  static_for<U>([&](auto uc) {
    constexpr int u = decltype(uc)::value;
    if (p0 + u < p1) {
      const Pack<raw_t, V> cur = buf[u];
      if (ld < p1) { buf[u] = load_next(); ++ld; }
      take(cur, p0 + u, std::integral_constant<int, (u < J ? u : J)>{});
    }
  });
  p += U;
  // steady state: every slot is consumed and refilled
  while (ld + U <= p1) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const Pack<raw_t, V> cur = buf[u];
      buf[u] = load_next();
      take(cur, p + u, std::integral_constant<int, J>{});
    }
    p += U;
    ld += U;
  }
  // drain: at most two partly valid groups
  for (; p < p1; p += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (p + u < p1) {
        const Pack<raw_t, V> cur = buf[u];
        if (ld < p1) { buf[u] = load_next(); ++ld; }
        take(cur, p + u, std::integral_constant<int, J>{});
      }
    }
  }
  // the partial sub-row: column c has one more element when c < rem
  // (with a padded row the other columns see the pad value there)
  if (with_rem && g.rem != 0) {
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const bool real = col + v < (int64_t)g.rem;
      if (live && (real || g.pad_tail)) {
        const cmp_t c = C::from_raw(real ? xr[(int64_t)g.full_rows * g.b + col + v] : E::pad_raw);
        if constexpr (C::has_nan) nan_mask |= __ballot(__builtin_isunordered(c, c));
        push<cmp_t, J, J>(q[v], pos[v], c, g.full_rows);
      }
    }
  }
}

// E: element traits; J: entries kept per bucket; V: columns per lane; W: waves
// per workgroup, sharing one column tile and splitting its sub-rows; U: loads
// kept in flight per lane.
template <typename E, int J, int V, int W, int U>
__global__ __launch_bounds__(kWave * W) void stream_kernel(
    const typename E::raw_t* __restrict__ x, const Sink<typename E::raw_t> out, const Geom g) {
  using raw_t = typename E::raw_t;
  using C = Cmp<E>;
  using cmp_t = typename C::cmp_t;
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
  cmp_t q[V][J];
  uint32_t pos[V][J];
  uint64_t nan_mask = 0;
  scan_run<E, J, V, U>(xr, g, col, live, p0, p1, last_slab && wave == W - 1, q, pos, nan_mask);

  bool any_nan = C::has_nan && nan_mask != 0;
  if constexpr (W > 1) {
    // waves 1.. hand their queues to wave 0 through LDS
    __shared__ cmp_t lds_q[W - 1][V * J][kWave];
    __shared__ uint32_t lds_p[W - 1][V * J][kWave];
    if (wave > 0) {
#pragma unroll
      for (int v = 0; v < V; ++v)
#pragma unroll
        for (int s = 0; s < J; ++s) {
          lds_q[wave - 1][v * J + s][lane] = q[v][s];
          lds_p[wave - 1][v * J + s][lane] = pos[v][s];
        }
    }
    if constexpr (C::has_nan) {
      any_nan = __syncthreads_or(any_nan);
    } else {
      __syncthreads();
    }
    if (wave > 0) return;
    if (!any_nan) {
      // fold in sub-row order, each wave's entries best first, so that equal
      // values keep the lowest index
#pragma nounroll
      for (int w = 0; w < W - 1; ++w)
#pragma unroll
        for (int v = 0; v < V; ++v)
#pragma unroll
          for (int s = J - 1; s >= 0; --s)
            push<cmp_t, J, J>(q[v], pos[v], lds_q[w][v * J + s][lane], lds_p[w][v * J + s][lane]);
    }
  }
  if (!live) return;
  if (any_nan) {
    exact_columns<E, J, V>(xr, g, out, row, slab, col, s0, W > 1 ? s1 : p1, last_slab);
    return;
  }
  raw_t val[V][J];
#pragma unroll
  for (int v = 0; v < V; ++v)
#pragma unroll
    for (int s = 0; s < J; ++s) val[v][s] = C::to_raw(q[v][s]);
  emit<E, J, V>(g, out, row, slab, col, val, pos);
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
  int filled = 0;
#pragma unroll
  for (int s = 0; s < J; ++s) { q[s] = 0; pos[s] = 0; }
  const uint32_t lo = (uint32_t)(((uint64_t)slabs * wave) / kMergeWaves);
  const uint32_t hi = (uint32_t)(((uint64_t)slabs * (wave + 1)) / kMergeWaves);
  if (live) {
    for (uint32_t slab = lo; slab < hi; ++slab) {
      const int64_t o = ((row * slabs + slab) * b + c) * J;
#pragma unroll
      for (int s = J - 1; s >= 0; --s) push_exact<E, J>(q, pos, filled, part_values[o + s], part_pos[o + s]);
    }
  }
  // a wave whose quarter is empty hands over nothing; all lanes of a wave agree on `filled`
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
    for (int s = J - 1; s >= 0; --s) push_exact<E, J>(q, pos, filled, lds_q[w - 1][s][lane], lds_p[w - 1][s][lane]);
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
