// Stage 1, general kernel: one lane owns one bucket and walks it front to back.
//
// This is the kernel that covers every element type, every bucket layout, every
// row length and alignment.  Consecutive lanes own consecutive buckets, so for
// the interleaved layouts a wave64 reads 64 adjacent elements per step; the
// contiguous layouts read with a stride of one bucket length between lanes.
// The streaming kernels in stage1_stream.hip take over the shapes where that
// matters; this one is the fallback for everything they do not accept.
//
// Selection follows the library-wide total order (value, then lowest index):
// members are visited in increasing position, so a newcomer only displaces a
// queue entry it beats strictly.
#include "atk_device.h"
#include "atk_launch.h"

namespace atk {

template <typename E, int J>
__global__ __launch_bounds__(256) void stage1_lane_per_bucket_kernel(
    const typename E::raw_t* __restrict__ x, int64_t n, int64_t row_stride,
    int64_t b, int layout, int64_t blocks_per_row,
    typename E::raw_t* __restrict__ values, const IndexOut indices) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  const int64_t row = blockIdx.x / blocks_per_row;
  const int64_t c = (blockIdx.x - row * blocks_per_row) * 256 + threadIdx.x;
  if (c >= b) return;
  const Bucket g = bucket_of(n, b, c, layout);
  const raw_t* xr = x + row * row_stride;
  const key_t pad_key = E::key(E::pad_raw);

  // q[0] is the weakest entry kept; pos[s] < 0 marks an empty slot.
  key_t q[J];
  int64_t pos[J];
#pragma unroll
  for (int s = 0; s < J; ++s) { q[s] = 0; pos[s] = -1; }

  for (int64_t t = 0; t < g.count; ++t) {
    const int64_t p = g.start + t * g.stride;
    const key_t key = p < n ? E::key(xr[p]) : pad_key;
    if (pos[0] < 0 || key > q[0]) {
      // Slide weaker entries down and drop the newcomer below the first entry
      // it does not beat.
      int at = 0;
#pragma unroll
      for (int s = 1; s < J; ++s) {
        if (at == s - 1 && (pos[s] < 0 || key > q[s])) {
          q[s - 1] = q[s]; pos[s - 1] = pos[s]; at = s;
        }
      }
#pragma unroll
      for (int s = 0; s < J; ++s) {
        if (s == at) { q[s] = key; pos[s] = p; }
      }
    }
  }

  const int64_t out = (row * b + c) * J;
#pragma unroll
  for (int s = 0; s < J; ++s) {
    const int64_t p = pos[s];
    if (values != nullptr) values[out + s] = (p >= 0 && p < n) ? xr[p] : E::pad_raw;
    indices.put(out + s, p);
  }
}

template <typename E>
static int launch_for_j(const void* x, int64_t rows, int64_t n, int64_t row_stride,
                        int64_t b, int j, int layout, void* values, IndexOut indices,
                        hipStream_t stream) {
  using raw_t = typename E::raw_t;
  const int64_t blocks_per_row = (b + 255) / 256;
  if (blocks_per_row * rows > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  const dim3 grid((unsigned)(blocks_per_row * rows)), block(256);
#define ATK_LAUNCH_J(J)                                                          \
  hipLaunchKernelGGL((stage1_lane_per_bucket_kernel<E, J>), grid, block, 0, stream, \
                     (const raw_t*)x, n, row_stride, b, layout, blocks_per_row,  \
                     (raw_t*)values, indices)
  switch (j) {
    case 1: ATK_LAUNCH_J(1); break;
    case 2: ATK_LAUNCH_J(2); break;
    case 3: ATK_LAUNCH_J(3); break;
    case 4: ATK_LAUNCH_J(4); break;
    default: return ATK_ERR_J;
  }
#undef ATK_LAUNCH_J
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

const char* dtype_name(int dtype) {
  switch (dtype) {
    case ATK_F32: return "f32"; case ATK_F16: return "f16"; case ATK_BF16: return "bf16";
    case ATK_F64: return "f64"; case ATK_U8: return "u8"; case ATK_I8: return "i8";
    case ATK_I16: return "i16"; case ATK_I32: return "i32"; case ATK_I64: return "i64";
  }
  return "?";
}

void describe_stage1_lane_per_bucket(int64_t rows, int64_t k0, int j, int dtype, std::string& out) {
  const int64_t b = j > 0 ? k0 / j : 0;
  out += "stage1_lane_per_bucket_kernel<" + std::string(dtype_name(dtype)) + ", J=" + std::to_string(j) +
         "> grid=" + std::to_string((b + 255) / 256 * rows) + " block=256";
}

int launch_stage1_lane_per_bucket(const void* x, int64_t rows, int64_t n,
                                  int64_t row_stride, int64_t k0, int j, int layout,
                                  int dtype, void* values, IndexOut indices,
                                  hipStream_t stream) {
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = launch_for_j<E>(x, rows, n, row_stride, k0 / j, j, layout,
                                        values, indices, stream));
  return rc;
}

}  // namespace atk
