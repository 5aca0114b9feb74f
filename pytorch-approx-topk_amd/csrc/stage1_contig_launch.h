// Launch code of the contiguous-layout stage-1 kernel for one element type.
// Included by one translation unit per type so that the types compile in parallel.
#pragma once

#include "stage1_contig.h"

namespace atk {
namespace contig {

template <typename E, int J, int V>
static int launch_one(const Plan& pl, const Geom& g, const typename E::raw_t* x, int64_t rows,
                      typename E::raw_t* values, IndexOut indices, void* ws, hipStream_t stream) {
  const int64_t groups = rows * (int64_t)g.groups;
  if (groups > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  hipLaunchKernelGGL((contig_kernel<E, J, V>), dim3((unsigned)groups), dim3(kThreads), pl.lds_bytes, stream, x,
                     values, indices, ws, g);
  if (g.slabs > 1)
    hipLaunchKernelGGL((contig_merge_kernel<E, J>), dim3((unsigned)(rows * g.b)), dim3(64), 0, stream, x,
                       (const void*)ws, values, indices, g);
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

template <typename E, int J>
static int launch_j(const Plan& pl, const Geom& g, const typename E::raw_t* x, int64_t rows,
                    typename E::raw_t* values, IndexOut indices, void* ws, hipStream_t stream) {
  constexpr int VF = stream::full_vec((int)sizeof(typename E::raw_t));
  if (g.whole != 0) {
    constexpr int ES = (int)sizeof(typename E::raw_t);
    if constexpr (ES == 2 || ES == 4) {
      const int64_t buckets = rows * (int64_t)g.b;
      const int64_t groups = (buckets + kThreads - 1) / kThreads;
      if (groups > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
      constexpr bool kPacked = ES == 2 && stream::PackedKey<E>::available;
      hipLaunchKernelGGL((whole_bucket_kernel<E, J, kPacked>), dim3((unsigned)groups), dim3(kThreads), 0, stream, x,
                         values, indices, g, buckets);
      return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
    } else {
      return ATK_ERR_ARG;  // the planner never asks for it
    }
  }
  return pl.vec > 1 ? launch_one<E, J, VF>(pl, g, x, rows, values, indices, ws, stream)
                    : launch_one<E, J, 1>(pl, g, x, rows, values, indices, ws, stream);
}

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int j, void* values,
                 IndexOut indices, void* ws, hipStream_t stream) {
  using raw_t = typename E::raw_t;
  Geom g = pl.geom;
  g.row_stride = row_stride;
  // (whole_bucket_kernel stores a bucket's J values at once: J * sizeof(raw_t) bytes, at most 16)
  g.wide_out = ((uintptr_t)values % 16 == 0 && (uintptr_t)indices.base % 16 == 0) ? 1u : 0u;
  const raw_t* xs = static_cast<const raw_t*>(x);
  raw_t* vs = static_cast<raw_t*>(values);
  switch (j) {
    case 1: return launch_j<E, 1>(pl, g, xs, rows, vs, indices, ws, stream);
    case 2: return launch_j<E, 2>(pl, g, xs, rows, vs, indices, ws, stream);
    case 3: return launch_j<E, 3>(pl, g, xs, rows, vs, indices, ws, stream);
    case 4: return launch_j<E, 4>(pl, g, xs, rows, vs, indices, ws, stream);
  }
  return ATK_ERR_J;
}

#define ATK_INSTANTIATE_CONTIG(DT)                                                                \
  template int launch_typed<Elem<DT>>(const Plan&, const void*, int64_t, int64_t, int, void*, \
                                      IndexOut, void*, hipStream_t);

}  // namespace contig
}  // namespace atk
