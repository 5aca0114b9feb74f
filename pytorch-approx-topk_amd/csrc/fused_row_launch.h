// Launch code of the fused one-workgroup-per-row kernel for one element type.
#pragma once

#include "fused_row.h"

namespace atk {
namespace fused {

template <typename E, int J, int V, int MAXW, typename pos_t, bool PACKED>
static int launch_packed(const Plan& pl, const typename E::raw_t* x, int64_t rows, const Geom& g, uint32_t k0,
                         uint32_t k, typename E::raw_t* values, IndexOut indices, hipStream_t stream) {
  if constexpr (MAXW > 8) {
    if (pl.in_registers) return ATK_ERR_ARG;  // (the register kernel is built for eight waves)
  } else if (pl.in_registers) {
    auto kern = fused_regs_kernel<E, J, V, MAXW, pos_t, PACKED>;
    // staged results leave four per thread when the outputs allow 16-byte stores, and then,
    // when the planner says so, past the cache
    const bool wide = k % 4 == 0 && (uintptr_t)values % 16 == 0 && (uintptr_t)indices.base % 16 == 0;
    [[maybe_unused]] const bool past_cache = pl.staged && pl.past_cache && wide;
    // contiguous short buckets: 16-bit positions, elements of two (packed queues) or four bytes
    constexpr int ES = (int)sizeof(typename E::raw_t);
    if constexpr (sizeof(pos_t) == 2 && ((ES == 2 && PACKED) || ES == 4) && V == 4) {
      if (pl.contig)
        kern = past_cache ? fused_regs_kernel<E, J, V, MAXW, pos_t, PACKED, true, true>
                          : fused_regs_kernel<E, J, V, MAXW, pos_t, PACKED, true>;
    } else if (pl.contig) {
      return ATK_ERR_ARG;  // the planner never asks for it
    }
    if constexpr (sizeof(pos_t) == 2 && ES <= 4) {  // (what staging asks for)
      if (!pl.contig && past_cache) kern = fused_regs_kernel<E, J, V, MAXW, pos_t, PACKED, false, true>;
    }
    if (pl.lds_bytes > 48 * 1024) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)pl.lds_bytes) != hipSuccess)
        return ATK_ERR_LAUNCH;
    }
    const int staged = pl.staged ? (wide ? 2 : 1) : 0;
    hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(kWave * pl.waves), pl.lds_bytes, stream, x, values,
                       indices, g, pl.tiles, pl.split, pl.hand_off, k0, k, pl.index_bits, staged);
    return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
  }
  auto kern = fused_row_kernel<E, J, V, MAXW, pos_t, PACKED>;
  if (pl.lds_bytes > 48 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)pl.lds_bytes) != hipSuccess)
      return ATK_ERR_LAUNCH;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)rows), dim3(kWave * pl.waves), pl.lds_bytes, stream, x, values,
                     indices, g, pl.tiles, pl.split, pl.hand_off, k0, k, pl.index_bits);
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

template <typename E, int J, int V, int MAXW, typename pos_t>
static int launch_one(const Plan& pl, const typename E::raw_t* x, int64_t rows, const Geom& g, uint32_t k0,
                      uint32_t k, typename E::raw_t* values, IndexOut indices, hipStream_t stream) {
  constexpr int VF = stream::full_vec((int)sizeof(typename E::raw_t));
  if constexpr (stream::PackedKey<E>::available && sizeof(typename E::raw_t) == 2 && V == VF / 2) {
    // Half the load width is the packed queues' (and only theirs: the planner halves it for
    // them alone); they need every sub-row number to fit 16 bits, as pos_t == uint16_t does.
    if constexpr (sizeof(pos_t) == 2) {
      if (pl.packed) return launch_packed<E, J, V, MAXW, pos_t, true>(pl, x, rows, g, k0, k, values, indices, stream);
    }
    return ATK_ERR_ARG;  // the planner never asks for it
  } else {
    if (pl.packed) return ATK_ERR_ARG;  // (packed queues at full load width: never planned)
    return launch_packed<E, J, V, MAXW, pos_t, false>(pl, x, rows, g, k0, k, values, indices, stream);
  }
}

template <typename E, int J, int VF>
static int launch_v(const Plan& pl, const typename E::raw_t* x, int64_t rows, const Geom& g, uint32_t k0,
                    uint32_t k, typename E::raw_t* values, IndexOut indices, hipStream_t stream) {
  if (pl.waves > 16) return ATK_ERR_ARG;  // the planner never asks for more
  if (pl.waves > 8)  // candidates beyond the usual LDS budget: one workgroup of sixteen waves per CU
    return pl.pos16 ? launch_one<E, J, VF, 16, uint16_t>(pl, x, rows, g, k0, k, values, indices, stream)
                    : launch_one<E, J, VF, 16, uint32_t>(pl, x, rows, g, k0, k, values, indices, stream);
  return pl.pos16 ? launch_one<E, J, VF, 8, uint16_t>(pl, x, rows, g, k0, k, values, indices, stream)
                  : launch_one<E, J, VF, 8, uint32_t>(pl, x, rows, g, k0, k, values, indices, stream);
}

template <typename E, int J>
static int launch_j(const Plan& pl, const typename E::raw_t* x, int64_t rows, const Geom& g, uint32_t k0,
                    uint32_t k, typename E::raw_t* values, IndexOut indices, hipStream_t stream) {
  constexpr int VF = stream::full_vec((int)sizeof(typename E::raw_t));
  if constexpr (stream::PackedKey<E>::available && sizeof(typename E::raw_t) == 2) {
    // packed queues may run at half the load width (fewer registers, more workgroups per CU)
    if (pl.vec == VF / 2) return launch_v<E, J, VF / 2>(pl, x, rows, g, k0, k, values, indices, stream);
  }
  return launch_v<E, J, VF>(pl, x, rows, g, k0, k, values, indices, stream);
}

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int64_t k0, int j,
                 int64_t k, void* values, IndexOut indices, hipStream_t stream) {
  using raw_t = typename E::raw_t;
  Geom g{};
  g.row_stride = row_stride; g.b = k0 / j;
  g.full_rows = pl.full_rows; g.rem = pl.rem; g.pad_tail = pl.pad_tail;
  g.slabs = 1; g.slab_len = pl.full_rows; g.col_tiles = pl.tiles; g.fold = 1;
  const raw_t* xs = static_cast<const raw_t*>(x);
  raw_t* ov = static_cast<raw_t*>(values);
  switch (j) {
    case 1: return launch_j<E, 1>(pl, xs, rows, g, (uint32_t)k0, (uint32_t)k, ov, indices, stream);
    case 2: return launch_j<E, 2>(pl, xs, rows, g, (uint32_t)k0, (uint32_t)k, ov, indices, stream);
    case 3: return launch_j<E, 3>(pl, xs, rows, g, (uint32_t)k0, (uint32_t)k, ov, indices, stream);
    case 4: return launch_j<E, 4>(pl, xs, rows, g, (uint32_t)k0, (uint32_t)k, ov, indices, stream);
  }
  return ATK_ERR_J;
}

#define ATK_INSTANTIATE_FUSED(DT)                                                                  \
  template int launch_typed<Elem<DT>>(const Plan&, const void*, int64_t, int64_t, int64_t, int,    \
                                      int64_t, void*, IndexOut, hipStream_t);

}  // namespace fused
}  // namespace atk
