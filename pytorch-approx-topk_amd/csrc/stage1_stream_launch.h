// Launch code of the streaming stage-1 kernels for one element type.  Included
// by one translation unit per type so that the types compile in parallel.
#pragma once

#include "stage1_stream.h"

namespace atk {
namespace stream {

// WS: results through LDS in whole-wave stores (Plan::wave_stores)
template <typename E, int J, int V, int W, int RUN, bool WS>
static int launch_out(const Plan& pl, const typename E::raw_t* x, const Sink<typename E::raw_t>& out,
                      const Geom& g, dim3 grid, hipStream_t stream, const KeyRangeOut& left) {
  constexpr int U = loads_in_flight(DtypeOf<E>::value, J, V, false);
  if constexpr (PackedKey<E>::available) {
    if (pl.packed) {
      constexpr int UP = loads_in_flight(DtypeOf<E>::value, J, V, true);
      if constexpr (deep_loads_for_short_columns(DtypeOf<E>::value, J, V, true, RUN, 0) && UP != 8) {
        if (deep_loads_for_short_columns(DtypeOf<E>::value, J, V, true, RUN, g.full_rows)) {
          hipLaunchKernelGGL((stream_kernel<E, J, V, W, 8, RUN, true, WS>), grid, dim3(kWave * W), 0, stream, x, out,
                             g, left);
          return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
        }
      }
      hipLaunchKernelGGL((stream_kernel<E, J, V, W, UP, RUN, true, WS>), grid, dim3(kWave * W), 0, stream, x, out, g,
                         left);
      return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
    }
  }
  // (the general queues hand over twice the bytes of the packed ones: combinations of theirs
  // beyond the LDS budget, which the planner never picks, are not compiled)
  if constexpr (merge_lds_bytes(V, J, W, (int)sizeof(typename Cmp<E>::cmp_t) + 4) <= merge_lds_limit(8)) {
    hipLaunchKernelGGL((stream_kernel<E, J, V, W, U, RUN, false, WS>), grid, dim3(kWave * W), 0, stream, x, out, g,
                       left);
    return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
  } else {
    return ATK_ERR_ARG;
  }
}

template <typename E, int J, int V, int W, int RUN>
static int launch_run(const Plan& pl, const typename E::raw_t* x, const Sink<typename E::raw_t>& out,
                      const Geom& g, dim3 grid, hipStream_t stream, const KeyRangeOut& left) {
  if constexpr (Transposed<E, J, V>::available) {
    if (pl.wave_stores) return launch_out<E, J, V, W, RUN, true>(pl, x, out, g, grid, stream, left);
  } else if (pl.wave_stores) {
    return ATK_ERR_ARG;  // the planner never asks for it
  }
  return launch_out<E, J, V, W, RUN, false>(pl, x, out, g, grid, stream, left);
}

template <typename E, int J, int V, int W>
static int launch_one(const Plan& pl, const typename E::raw_t* x, const Sink<typename E::raw_t>& out,
                      const Geom& g, int64_t rows, hipStream_t stream, const KeyRangeOut& left) {
  const int64_t groups = rows * (int64_t)pl.slabs * pl.col_tiles;
  if (groups > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  const dim3 grid((unsigned)groups);
  // combinations the planner never picks are not compiled
  constexpr int kEntryBytes = PackedKey<E>::available ? 4 : (int)sizeof(typename Cmp<E>::cmp_t) + 4;
  if constexpr (merge_lds_bytes(V, J, W, kEntryBytes) <= merge_lds_limit(kEntryBytes)) {
    if constexpr (V > 1) {  // exact short runs exist for the vector kernels only
      if (pl.run == 4) return launch_run<E, J, V, W, 4>(pl, x, out, g, grid, stream, left);
      if (pl.run == 8) return launch_run<E, J, V, W, 8>(pl, x, out, g, grid, stream, left);
    }
    return launch_run<E, J, V, W, 0>(pl, x, out, g, grid, stream, left);
  } else {
    (void)x; (void)out; (void)g; (void)stream; (void)left;
    return ATK_ERR_ARG;
  }
}

template <typename E, int J, int V>
static int launch_w(const Plan& pl, const typename E::raw_t* x, const Sink<typename E::raw_t>& out,
                    const Geom& g, int64_t rows, hipStream_t stream, const KeyRangeOut& left) {
  switch (pl.waves) {
    case 1: return launch_one<E, J, V, 1>(pl, x, out, g, rows, stream, left);
    case 2: return launch_one<E, J, V, 2>(pl, x, out, g, rows, stream, left);
    case 4: return launch_one<E, J, V, 4>(pl, x, out, g, rows, stream, left);
    case 8: return launch_one<E, J, V, 8>(pl, x, out, g, rows, stream, left);
  }
  return ATK_ERR_ARG;
}

template <typename E, int J>
static int launch_j(const Plan& pl, const typename E::raw_t* x, const Sink<typename E::raw_t>& out,
                    const Geom& g, int64_t rows, hipStream_t stream, KeyRangeOut* ranges) {
  using raw_t = typename E::raw_t;
  constexpr int VF = full_vec((int)sizeof(raw_t));
  // Kernels that end in the merge of slabs can leave a chained select its key
  // ranges (one per scanning workgroup) and its histogram.
  KeyRangeOut left{}, left_to_merge{};
  const int64_t scan_blocks = (int64_t)pl.slabs * pl.col_tiles;  // per row
  if (ranges != nullptr && ranges->range != nullptr && E::key_bits <= 32 && pl.merge &&
      scan_blocks <= (int64_t)ranges->capacity) {
    ranges->entries = (uint32_t)scan_blocks;
    left = *ranges;
    if (ranges->want_hist != 0) {
      ranges->hist_done = 1;
      left_to_merge = left;
    }
  }
  const int rc = pl.vec > 1 ? launch_w<E, J, VF>(pl, x, out, g, rows, stream, left)
                            : launch_w<E, J, 1>(pl, x, out, g, rows, stream, left);
  if (rc != ATK_OK || !pl.merge) return rc;
  const int64_t b = pl.width / pl.fold;  // buckets
  // buckets per workgroup: a power of two, no more than there are, and few
  // enough that a thread folds at most about 32 of a bucket's partial queues
  uint32_t cb = kWave;
  while (cb > 1 && ((int64_t)(cb / 2) >= b || (int64_t)pl.slabs * cb > 32 * kMergeThreads)) cb /= 2;
  const int64_t blocks_per_row = (b + cb - 1) / cb;
  if (blocks_per_row * rows > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  hipLaunchKernelGGL((stream_merge_kernel<E, J>), dim3((unsigned)(blocks_per_row * rows)),
                     dim3(kMergeThreads), 0,
                     stream, x, g.row_stride, (const raw_t*)out.part_values, (const uint32_t*)out.part_pos,
                     b, pl.slabs, cb, (uint32_t)blocks_per_row, out.values, out.indices, left_to_merge);
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int j,
                 void* values, IndexOut indices, void* ws, hipStream_t stream, KeyRangeOut* ranges) {
  using raw_t = typename E::raw_t;
  Geom g;
  g.row_stride = row_stride; g.b = pl.width;
  g.full_rows = pl.full_rows; g.rem = pl.rem; g.pad_tail = pl.pad_tail;
  g.slabs = pl.slabs; g.slab_len = pl.slab_len; g.col_tiles = pl.col_tiles;
  g.fold = pl.fold;
  Sink<raw_t> out;
  out.values = static_cast<raw_t*>(values); out.indices = indices;
  unsigned char* base = static_cast<unsigned char*>(ws);
  out.part_values = pl.merge ? reinterpret_cast<raw_t*>(base + pl.part_values_off) : nullptr;
  out.part_pos = pl.merge ? reinterpret_cast<uint32_t*>(base + pl.part_pos_off) : nullptr;
  const raw_t* xs = static_cast<const raw_t*>(x);
  switch (j) {
    case 1: return launch_j<E, 1>(pl, xs, out, g, rows, stream, ranges);
    case 2: return launch_j<E, 2>(pl, xs, out, g, rows, stream, ranges);
    case 3: return launch_j<E, 3>(pl, xs, out, g, rows, stream, ranges);
    case 4: return launch_j<E, 4>(pl, xs, out, g, rows, stream, ranges);
  }
  return ATK_ERR_J;
}

#define ATK_INSTANTIATE_STREAM(DT)                                                          \
  template int launch_typed<Elem<DT>>(const Plan&, const void*, int64_t, int64_t, int, void*, \
                                      IndexOut, void*, hipStream_t, KeyRangeOut*);

}  // namespace stream
}  // namespace atk
