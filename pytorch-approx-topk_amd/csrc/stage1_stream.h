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
// Work split.  Sub-rows are cut into `slabs` (grid dimension) so that short,
// wide batches and long single rows both fill the machine.  Inside a workgroup
// of 4 waves either every wave takes its own column tile (SPLIT_WG = false) or
// the four waves share one column tile and each scans a quarter of the slab,
// merging through LDS (SPLIT_WG = true).  With more than one slab the per-slab
// queues go to a workspace and `stream_merge_kernel` folds them.
//
// Order.  Sub-rows are visited in increasing position and a newcomer displaces
// an entry only when it compares strictly greater, so equal values keep the
// lowest index.  Floating-point columns compare with the hardware's IEEE `>`
// (-0.0 == +0.0); a NaN makes that compare meaningless, so every load is also
// tested for NaN and a wave (or workgroup) that saw one recomputes its tile
// with the exact integer order keys of atk_device.h.
#pragma once

#include <type_traits>

#include "atk_device.h"
#include "atk_launch.h"

namespace atk {
namespace stream {

constexpr int kWave = 64;
constexpr int kWavesPerGroup = 4;
constexpr int kGroup = kWave * kWavesPerGroup;

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

struct Args {
  const void* x;          // input rows
  int64_t row_stride;     // elements between rows
  int64_t b;              // buckets (columns) per row
  uint32_t full_rows;     // L = n / b
  uint32_t rem;           // n mod b: columns that have one more element
  uint32_t pad_tail;      // padded row: the other columns hold the pad value there
  uint32_t slabs;         // sub-row slabs per row
  uint32_t slab_len;      // sub-rows per slab (the last slab takes the rest)
  uint32_t col_tiles;     // workgroup column tiles per row
  void* values;           // slabs == 1: final values[rows][b*J]
  int64_t* indices;       //             final indices
  void* part_values;      // slabs > 1: [rows][slabs][b*J] raw values
  uint32_t* part_pos;     //            and their sub-row numbers
};

// Writes the queues of this lane's V columns, either as final results or as a
// slab's partial result.
template <typename E, int J, int V>
__device__ inline void emit(const Args& a, int64_t row, uint32_t slab, int64_t col,
                            const typename E::raw_t (&val)[V][J], const uint32_t (&pos)[V][J]) {
  using raw_t = typename E::raw_t;
  if (a.slabs == 1) {
    const int64_t o = (row * a.b + col) * J;
    raw_t* ov = static_cast<raw_t*>(a.values) + o;
    int64_t* oi = a.indices + o;
    if constexpr (V > 1) {
      // V*J values = J 16-byte stores; V*J int64 = V*J/2 16-byte stores
      Pack<raw_t, V> pv[J];
      Pack<int64_t, 2> pi[V * J / 2];
#pragma unroll
      for (int v = 0; v < V; ++v)
#pragma unroll
        for (int s = 0; s < J; ++s) {
          pv[(v * J + s) / V].e[(v * J + s) % V] = val[v][s];
          pi[(v * J + s) / 2].e[(v * J + s) % 2] = col + v + (int64_t)pos[v][s] * a.b;
        }
#pragma unroll
      for (int t = 0; t < J; ++t) reinterpret_cast<Pack<raw_t, V>*>(ov)[t] = pv[t];
#pragma unroll
      for (int t = 0; t < V * J / 2; ++t) reinterpret_cast<Pack<int64_t, 2>*>(oi)[t] = pi[t];
    } else {
#pragma unroll
      for (int s = 0; s < J; ++s) { ov[s] = val[0][s]; oi[s] = col + (int64_t)pos[0][s] * a.b; }
    }
  } else {
    const int64_t o = ((row * a.slabs + slab) * a.b + col) * J;
    raw_t* ov = static_cast<raw_t*>(a.part_values) + o;
    uint32_t* op = a.part_pos + o;
#pragma unroll
    for (int v = 0; v < V; ++v)
#pragma unroll
      for (int s = 0; s < J; ++s) { ov[v * J + s] = val[v][s]; op[v * J + s] = pos[v][s]; }
  }
}

// Exact recomputation of one lane's V columns over sub-rows [p0, p1) (plus the
// partial sub-row when `with_rem`), through order keys.  Off the hot path.
template <typename E, int J, int V>
__device__ __noinline__ void exact_columns(const Args& a, int64_t row, uint32_t slab, int64_t col,
                                           uint32_t p0, uint32_t p1, bool with_rem) {
  using raw_t = typename E::raw_t;
  const raw_t* xr = static_cast<const raw_t*>(a.x) + row * a.row_stride;
  raw_t val[V][J];
  uint32_t pos[V][J];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    int filled = 0;
#pragma unroll
    for (int s = 0; s < J; ++s) { val[v][s] = 0; pos[v][s] = 0; }
    for (uint32_t p = p0; p < p1; ++p)
      push_exact<E, J>(val[v], pos[v], filled, xr[(int64_t)p * a.b + col + v], p);
    if (with_rem && a.rem != 0) {
      if (col + v < (int64_t)a.rem)
        push_exact<E, J>(val[v], pos[v], filled, xr[(int64_t)a.full_rows * a.b + col + v], a.full_rows);
      else if (a.pad_tail)
        push_exact<E, J>(val[v], pos[v], filled, E::pad_raw, a.full_rows);
    }
  }
  emit<E, J, V>(a, row, slab, col, val, pos);
}

template <typename E, int J, int V, bool SPLIT_WG, int U>
__global__ __launch_bounds__(kGroup) void stream_kernel(const Args a) {
  using raw_t = typename E::raw_t;
  using C = Cmp<E>;
  using cmp_t = typename C::cmp_t;
  constexpr int kTileCols = kWave * V;                                  // columns per wave
  constexpr int kGroupCols = SPLIT_WG ? kTileCols : kTileCols * kWavesPerGroup;

  const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  uint32_t blk = blockIdx.x;
  const uint32_t col_tile = blk % a.col_tiles; blk /= a.col_tiles;
  const uint32_t slab = blk % a.slabs;
  const int64_t row = blk / a.slabs;

  const int64_t col = (int64_t)col_tile * kGroupCols + (SPLIT_WG ? 0 : wave * kTileCols) + lane * V;
  const bool live = col < a.b;  // b is a multiple of V whenever V > 1

  // sub-rows of this slab, then of this wave
  uint32_t p0 = slab * a.slab_len;
  uint32_t p1 = (slab + 1 == a.slabs) ? a.full_rows : p0 + a.slab_len;
  const uint32_t s0 = p0, s1 = p1;
  if (SPLIT_WG) {
    const uint32_t len = p1 - p0;
    p1 = p0 + (uint32_t)(((uint64_t)len * (wave + 1)) / kWavesPerGroup);
    p0 = p0 + (uint32_t)(((uint64_t)len * wave) / kWavesPerGroup);
  }
  const bool last_run = (slab + 1 == a.slabs) && (!SPLIT_WG || wave == kWavesPerGroup - 1);

  const raw_t* xr = static_cast<const raw_t*>(a.x) + row * a.row_stride;
  const raw_t* src = xr + (live ? col : 0);

  cmp_t q[V][J];
  uint32_t pos[V][J];
  bool nan_seen = false;

  auto take = [&](const Pack<raw_t, V>& pk, uint32_t p, auto filled_tag) {
    constexpr int FILLED = decltype(filled_tag)::value;
    cmp_t c[V];
#pragma unroll
    for (int v = 0; v < V; ++v) c[v] = C::from_raw(pk.e[v]);
    if constexpr (C::has_nan) {
#pragma unroll
      for (int v = 0; v + 1 < V; v += 2) nan_seen |= __builtin_isunordered(c[v], c[v + 1]);
      if constexpr (V % 2 != 0) nan_seen |= __builtin_isunordered(c[V - 1], c[V - 1]);
    }
#pragma unroll
    for (int v = 0; v < V; ++v) push<cmp_t, J, FILLED>(q[v], pos[v], c[v], p);
  };

  // first J sub-rows fill the queues
  {
    Pack<raw_t, V> first[J];
#pragma unroll
    for (int t = 0; t < J; ++t) first[t] = load_pack<raw_t, V>(src + (int64_t)(p0 + t) * a.b);
    take(first[0], p0, std::integral_constant<int, 0>{});
    if constexpr (J > 1) take(first[1], p0 + 1, std::integral_constant<int, 1>{});
    if constexpr (J > 2) take(first[2], p0 + 2, std::integral_constant<int, 2>{});
    if constexpr (J > 3) take(first[3], p0 + 3, std::integral_constant<int, 3>{});
  }
  uint32_t p = p0 + J;
  const raw_t* cur = src + (int64_t)p * a.b;
  for (; p + U <= p1; p += U) {
    Pack<raw_t, V> buf[U];
#pragma unroll
    for (int u = 0; u < U; ++u) buf[u] = load_pack<raw_t, V>(cur + (int64_t)u * a.b);
    cur += (int64_t)U * a.b;
#pragma unroll
    for (int u = 0; u < U; ++u) take(buf[u], p + u, std::integral_constant<int, J>{});
  }
  for (; p < p1; ++p) {
    const Pack<raw_t, V> one = load_pack<raw_t, V>(cur);
    cur += a.b;
    take(one, p, std::integral_constant<int, J>{});
  }
  // the partial sub-row: column c has one more element when c < rem
  // (with a padded row the other columns see the pad value there)
  if (last_run && a.rem != 0) {
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const bool real = col + v < (int64_t)a.rem;
      if (live && (real || a.pad_tail)) {
        const cmp_t c = C::from_raw(real ? xr[(int64_t)a.full_rows * a.b + col + v] : E::pad_raw);
        if constexpr (C::has_nan) nan_seen |= __builtin_isunordered(c, c);
        push<cmp_t, J, J>(q[v], pos[v], c, a.full_rows);
      }
    }
  }

  raw_t val[V][J];
  if constexpr (!SPLIT_WG) {
    if (C::has_nan && __any(nan_seen)) {
      if (live) exact_columns<E, J, V>(a, row, slab, col, p0, p1, last_run);
      return;
    }
  } else {
    // waves 1..3 hand their queues to wave 0 through LDS, in sub-row order
    __shared__ cmp_t lds_q[kWavesPerGroup - 1][V * J][kWave];
    __shared__ uint32_t lds_p[kWavesPerGroup - 1][V * J][kWave];
    if (wave > 0) {
#pragma unroll
      for (int v = 0; v < V; ++v)
#pragma unroll
        for (int s = 0; s < J; ++s) {
          lds_q[wave - 1][v * J + s][lane] = q[v][s];
          lds_p[wave - 1][v * J + s][lane] = pos[v][s];
        }
    }
    const int any_nan = __syncthreads_or(C::has_nan && nan_seen);
    if (wave > 0) return;
    if (any_nan) {
      if (live) exact_columns<E, J, V>(a, row, slab, col, s0, s1, slab + 1 == a.slabs);
      return;
    }
#pragma unroll
    for (int w = 0; w < kWavesPerGroup - 1; ++w)
#pragma unroll
      for (int v = 0; v < V; ++v)
#pragma unroll
        for (int s = J - 1; s >= 0; --s)  // best entry first keeps equal values in index order
          push<cmp_t, J, J>(q[v], pos[v], lds_q[w][v * J + s][lane], lds_p[w][v * J + s][lane]);
  }
  if (!live) return;
#pragma unroll
  for (int v = 0; v < V; ++v)
#pragma unroll
    for (int s = 0; s < J; ++s) val[v][s] = C::to_raw(q[v][s]);
  emit<E, J, V>(a, row, slab, col, val, pos);
}

// Folds the per-slab queues of every bucket into the final result, one lane per
// bucket, with exact order keys.  Slabs are visited in sub-row order and each
// slab's entries best first, so equal values keep the lowest index.
template <typename E, int J>
__global__ __launch_bounds__(256) void stream_merge_kernel(
    const typename E::raw_t* __restrict__ part_values, const uint32_t* __restrict__ part_pos,
    int64_t b, uint32_t slabs, int64_t blocks_per_row, typename E::raw_t* __restrict__ values,
    int64_t* __restrict__ indices) {
  using raw_t = typename E::raw_t;
  const int64_t row = blockIdx.x / blocks_per_row;
  const int64_t c = (blockIdx.x - row * blocks_per_row) * 256 + threadIdx.x;
  if (c >= b) return;
  raw_t q[J];
  uint32_t pos[J];
  int filled = 0;
#pragma unroll
  for (int s = 0; s < J; ++s) { q[s] = 0; pos[s] = 0; }
  for (uint32_t slab = 0; slab < slabs; ++slab) {
    const int64_t o = ((row * slabs + slab) * b + c) * J;
#pragma unroll
    for (int s = J - 1; s >= 0; --s) push_exact<E, J>(q, pos, filled, part_values[o + s], part_pos[o + s]);
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
  bool split_wg;
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
