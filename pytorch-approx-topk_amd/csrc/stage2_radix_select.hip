// Stage 2: exact top-k of a row's k0 candidates by radix select, one workgroup
// per row.
//
// The order key of every candidate is staged in LDS (or re-read from global
// memory when a row's keys do not fit); the selection itself is the block-wide
// radix select of stage2_select.h.
#include "atk_device.h"
#include "atk_launch.h"
#include "stage2_select.h"

namespace atk {

namespace {

template <typename raw_t> struct Candidate { raw_t value; int64_t index; };

template <typename E, bool KEYS_IN_LDS>
__global__ __launch_bounds__(1024) void select_kernel(
    const typename E::raw_t* __restrict__ cand_values,
    const int64_t* __restrict__ cand_indices, uint32_t k0, uint32_t k, int index_bits,
    typename E::raw_t* __restrict__ values, const IndexOut indices) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ select::Shared sh;
  key_t* keys = reinterpret_cast<key_t*>(dyn_lds);

  const int64_t row = blockIdx.x;
  const raw_t* cv = cand_values + row * (int64_t)k0;
  const int64_t* ci = cand_indices + row * (int64_t)k0;

  if (KEYS_IN_LDS) {
    // eight loads in flight per lane
    uint32_t i = threadIdx.x;
    for (; i + 7 * blockDim.x < k0; i += 8 * blockDim.x) {
      raw_t got[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) got[u] = cv[i + u * blockDim.x];
#pragma unroll
      for (int u = 0; u < 8; ++u) keys[i + u * blockDim.x] = E::key(got[u]);
    }
    for (; i < k0; i += blockDim.x) keys[i] = E::key(cv[i]);
  }
  auto key_at = [&](uint32_t i) -> key_t { return KEYS_IN_LDS ? keys[i] : E::key(cv[i]); };
  auto index_at = [&](uint32_t i) -> uint64_t { return (uint64_t)ci[i]; };

  const select::Cut<key_t> cut =
      select::find_cut<key_t, E::key_bits>(sh, k0, k, index_bits, key_at, index_at);

  raw_t* ov = values + row * (int64_t)k;
  const int64_t oi = row * (int64_t)k;  // this row's first output slot
  select::compact(
      sh, k0, k,
      [&](uint32_t i) -> bool {
        const key_t key = key_at(i);
        if (key != cut.T) return key > cut.T;
        return cut.index_cut == ~0ull || index_at(i) <= cut.index_cut;
      },
      [&](uint32_t i) { return Candidate<raw_t>{cv[i], ci[i]}; },
      [&](uint32_t, uint32_t o, const Candidate<raw_t>& c) { ov[o] = c.value; indices.put(oi + o, c.index); });
}

// LDS a workgroup may use for keys; the rest of the 160 KB of a gfx950 CU is
// left to the static block above and to a second resident workgroup's needs.
constexpr size_t kMaxKeyLds = 128 * 1024;

template <typename E>
int launch_select_typed(const void* cand_values, const int64_t* cand_indices, int64_t rows,
                        int64_t k0, int64_t k, int index_bits, void* values, IndexOut indices,
                        hipStream_t stream) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  const size_t key_bytes = (size_t)k0 * sizeof(key_t);
  const bool in_lds = key_bytes <= kMaxKeyLds;
  int nt = 1024;
  if (k0 <= 1024) nt = 256;
  if (k0 <= 128) nt = 64;
  const dim3 grid((unsigned)rows), block(nt);
  if (in_lds) {
    auto kern = select_kernel<E, true>;
    if (key_bytes > 48 * 1024) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)key_bytes) != hipSuccess)
        return ATK_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, grid, block, key_bytes, stream, (const raw_t*)cand_values,
                       cand_indices, (uint32_t)k0, (uint32_t)k, index_bits, (raw_t*)values,
                       indices);
  } else {
    hipLaunchKernelGGL((select_kernel<E, false>), grid, block, 0, stream,
                       (const raw_t*)cand_values, cand_indices, (uint32_t)k0, (uint32_t)k,
                       index_bits, (raw_t*)values, indices);
  }
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

}  // namespace

int launch_select(const void* cand_values, const int64_t* cand_indices, int64_t rows,
                  int64_t k0, int64_t k, int64_t index_bound, int dtype, void* values,
                  IndexOut indices, hipStream_t stream) {
  if (k0 > 0x7fffffffll || rows > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  int index_bits = 1;
  while (index_bits < 63 && (1ll << index_bits) < index_bound) ++index_bits;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = launch_select_typed<E>(cand_values, cand_indices, rows, k0, k,
                                               index_bits, values, indices, stream));
  return rc;
}

}  // namespace atk
