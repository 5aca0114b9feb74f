// Launch code of the streaming stage-1 kernels for one element type.  Included
// by one translation unit per type so that the types compile in parallel.
#pragma once

#include "stage1_stream.h"

namespace atk {
namespace stream {

template <typename E, int J, int V, bool SPLIT_WG>
static int launch_one(const Plan& pl, const Args& a, int64_t rows, hipStream_t stream) {
  const int64_t groups = rows * (int64_t)pl.slabs * pl.col_tiles;
  if (groups > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  hipLaunchKernelGGL((stream_kernel<E, J, V, SPLIT_WG, 8>), dim3((unsigned)groups), dim3(kGroup), 0,
                     stream, a);
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

template <typename E, int J>
static int launch_j(const Plan& pl, const Args& a, int64_t rows, hipStream_t stream) {
  using raw_t = typename E::raw_t;
  constexpr int VF = 16 / (int)sizeof(raw_t);
  int rc;
  if (pl.vec > 1)
    rc = pl.split_wg ? launch_one<E, J, VF, true>(pl, a, rows, stream)
                     : launch_one<E, J, VF, false>(pl, a, rows, stream);
  else
    rc = pl.split_wg ? launch_one<E, J, 1, true>(pl, a, rows, stream)
                     : launch_one<E, J, 1, false>(pl, a, rows, stream);
  if (rc != ATK_OK || pl.slabs == 1) return rc;
  const int64_t blocks_per_row = (a.b + 255) / 256;
  if (blocks_per_row * rows > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  hipLaunchKernelGGL((stream_merge_kernel<E, J>), dim3((unsigned)(blocks_per_row * rows)), dim3(256), 0,
                     stream, (const raw_t*)a.part_values, (const uint32_t*)a.part_pos, a.b, pl.slabs,
                     blocks_per_row, (raw_t*)a.values, a.indices);
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int64_t b, int j,
                 void* values, int64_t* indices, void* ws, hipStream_t stream) {
  Args a;
  a.x = x; a.row_stride = row_stride; a.b = b;
  a.full_rows = pl.full_rows; a.rem = pl.rem; a.pad_tail = pl.pad_tail;
  a.slabs = pl.slabs; a.slab_len = pl.slab_len; a.col_tiles = pl.col_tiles;
  a.values = values; a.indices = indices;
  a.part_values = pl.slabs > 1 ? static_cast<unsigned char*>(ws) + pl.part_values_off : nullptr;
  a.part_pos = pl.slabs > 1
                   ? reinterpret_cast<uint32_t*>(static_cast<unsigned char*>(ws) + pl.part_pos_off)
                   : nullptr;
  switch (j) {
    case 1: return launch_j<E, 1>(pl, a, rows, stream);
    case 2: return launch_j<E, 2>(pl, a, rows, stream);
    case 3: return launch_j<E, 3>(pl, a, rows, stream);
    case 4: return launch_j<E, 4>(pl, a, rows, stream);
  }
  return ATK_ERR_J;
}

#define ATK_INSTANTIATE_STREAM(DT)                                                          \
  template int launch_typed<Elem<DT>>(const Plan&, const void*, int64_t, int64_t, int64_t, \
                                      int, void*, int64_t*, void*, hipStream_t);

}  // namespace stream
}  // namespace atk
