// Stage 2: exact top-k of a row's k0 candidates by radix select, one workgroup
// per row.
//
// The order key of every candidate is staged in LDS (or re-read from global
// memory when a row's keys do not fit).  An MSB-first radix select with 8-bit
// digits finds the key T of the k-th best candidate and how many candidates
// with key == T belong to the result.  When only part of that tie group
// belongs, a second radix select over the candidates' original indices finds
// the cut so that the lowest indices win.  The survivors are then written in
// increasing candidate position with wave-level ballot/mbcnt compaction.
#include "atk_device.h"
#include "atk_launch.h"

namespace atk {

namespace {

constexpr int kWave = 64;
constexpr int kMaxWaves = 16;

// Histogram counters are kept in kCopies private copies (lane % kCopies picks
// one) so that the many candidates sharing a digit -- the top byte of a float
// key is nearly constant among top-k candidates -- do not serialise on one LDS
// address; the odd stride spreads equal digits of different copies over banks.
constexpr int kCopies = 16;
constexpr int kCopyStride = 257;

struct SelectShared {
  uint32_t copies[kCopies * kCopyStride];
  uint32_t hist[256];
  uint32_t wave_total[kMaxWaves];
  uint32_t digit;
  uint32_t need;
  uint32_t bin_count;
};

__device__ inline uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `m` below this lane.
__device__ inline uint32_t rank_in(uint64_t m) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
}

// Wave 0 scans the 256-bin histogram for the bin holding the `need`-th element,
// counting from the top bin (FROM_TOP) or from the bottom bin, and publishes
// the bin, the rank left within it and the bin's population.
template <bool FROM_TOP>
__device__ inline void find_bin(SelectShared& sh, uint32_t need) {
  if (threadIdx.x < kWave) {
    const uint32_t lane = threadIdx.x;
    // Lane l owns bins 4l..4l+3; `grp` is the lane's position in scan order.
    uint32_t h[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) h[i] = sh.hist[4 * lane + i];
    const uint32_t mine = h[0] + h[1] + h[2] + h[3];
    // Inclusive scan over lanes in scan order (descending lanes when FROM_TOP).
    uint32_t incl = mine;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t other = FROM_TOP ? __shfl_down(incl, d, kWave) : __shfl_up(incl, d, kWave);
      const bool has = FROM_TOP ? (lane + d < kWave) : (lane >= (uint32_t)d);
      if (has) incl += other;
    }
    uint32_t before = incl - mine;  // population of all bins scanned before this lane's
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int bin = FROM_TOP ? 3 - i : i;
      const uint32_t c = h[bin];
      if (before < need && need <= before + c) {
        sh.digit = 4 * lane + bin;
        sh.need = need - before;
        sh.bin_count = c;
      }
      before += c;
    }
  }
}

// hist[d] = sum of the private copies of bin d
__device__ inline void fold_copies(SelectShared& sh, uint32_t tid, uint32_t nt) {
  for (uint32_t d = tid; d < 256; d += nt) {
    uint32_t total = 0;
#pragma unroll
    for (int c = 0; c < kCopies; ++c) total += sh.copies[c * kCopyStride + d];
    sh.hist[d] = total;
  }
}

template <typename E, bool KEYS_IN_LDS>
__global__ __launch_bounds__(1024) void select_kernel(
    const typename E::raw_t* __restrict__ cand_values,
    const int64_t* __restrict__ cand_indices, uint32_t k0, uint32_t k, int index_bits,
    typename E::raw_t* __restrict__ values, int64_t* __restrict__ indices) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ SelectShared sh;
  key_t* keys = reinterpret_cast<key_t*>(dyn_lds);

  const uint32_t tid = threadIdx.x, nt = blockDim.x;
  const int64_t row = blockIdx.x;
  const raw_t* cv = cand_values + row * (int64_t)k0;
  const int64_t* ci = cand_indices + row * (int64_t)k0;

  if (KEYS_IN_LDS) {
    for (uint32_t i = tid; i < k0; i += nt) keys[i] = E::key(cv[i]);
  }
  auto key_at = [&](uint32_t i) -> key_t { return KEYS_IN_LDS ? keys[i] : E::key(cv[i]); };
  uint32_t* my_copy = &sh.copies[(tid % kCopies) * kCopyStride];  // this lane's histogram copy

  // ---- value select: T = key of the k-th best candidate --------------------
  key_t prefix = 0, mask = 0;
  uint32_t need = k;
  for (int shift = E::key_bits - 8; shift >= 0; shift -= 8) {
    for (uint32_t i = tid; i < kCopies * kCopyStride; i += nt) sh.copies[i] = 0;
    __syncthreads();
    for (uint32_t i = tid; i < k0; i += nt) {
      const key_t key = key_at(i);
      if ((key & mask) == prefix) atomicAdd(&my_copy[(uint32_t)(key >> shift) & 0xffu], 1u);
    }
    __syncthreads();
    fold_copies(sh, tid, nt);
    __syncthreads();
    find_bin<true>(sh, need);
    __syncthreads();
    prefix |= (key_t)sh.digit << shift;
    mask |= (key_t)0xff << shift;
    need = sh.need;
  }
  const key_t T = prefix;
  const uint32_t ties = sh.bin_count;  // candidates with key == T

  // ---- index select inside the tie group, only when it is cut --------------
  uint64_t index_cut = ~0ull;  // ties with index <= index_cut are kept
  if (need < ties) {
    uint64_t iprefix = 0, imask = 0;
    for (int shift = ((index_bits + 7) / 8 - 1) * 8; shift >= 0; shift -= 8) {
      __syncthreads();
      for (uint32_t i = tid; i < kCopies * kCopyStride; i += nt) sh.copies[i] = 0;
      __syncthreads();
      for (uint32_t i = tid; i < k0; i += nt) {
        if (key_at(i) == T) {
          const uint64_t idx = (uint64_t)ci[i];
          if ((idx & imask) == iprefix) atomicAdd(&my_copy[(uint32_t)(idx >> shift) & 0xffu], 1u);
        }
      }
      __syncthreads();
      fold_copies(sh, tid, nt);
      __syncthreads();
      find_bin<false>(sh, need);
      __syncthreads();
      iprefix |= (uint64_t)sh.digit << shift;
      imask |= (uint64_t)0xff << shift;
      need = sh.need;
    }
    index_cut = iprefix;
  }

  auto selected = [&](uint32_t i) -> bool {
    const key_t key = key_at(i);
    if (key > T) return true;
    if (key < T) return false;
    return index_cut == ~0ull || (uint64_t)ci[i] <= index_cut;
  };

  // ---- stable compaction: wave w owns a contiguous run of candidates -------
  const uint32_t waves = nt / kWave, wave = tid / kWave, lane = lane_id();
  uint32_t per_wave = (k0 + waves - 1) / waves;
  per_wave = (per_wave + kWave - 1) / kWave * kWave;
  const uint32_t lo = min(wave * per_wave, k0), hi = min(lo + per_wave, k0);

  uint32_t mine = 0;
  for (uint32_t base = lo; base < hi; base += kWave) {
    const uint32_t i = base + lane;
    const bool sel = i < hi && selected(i);
    mine += (uint32_t)__popcll(__ballot(sel));
  }
  if (lane == 0) sh.wave_total[wave] = mine;
  __syncthreads();
  uint32_t out = 0;
  for (uint32_t w = 0; w < wave; ++w) out += sh.wave_total[w];

  raw_t* ov = values + row * (int64_t)k;
  int64_t* oi = indices + row * (int64_t)k;
  for (uint32_t base = lo; base < hi; base += kWave) {
    const uint32_t i = base + lane;
    const bool sel = i < hi && selected(i);
    const uint64_t m = __ballot(sel);
    if (sel) {
      const uint32_t o = out + rank_in(m);
      if (o < k) { ov[o] = cv[i]; oi[o] = ci[i]; }
    }
    out += (uint32_t)__popcll(m);
  }
}

// LDS a workgroup may use for keys; the rest of the 160 KB of a gfx950 CU is
// left to the static block above and to a second resident workgroup's needs.
constexpr size_t kMaxKeyLds = 128 * 1024;

template <typename E>
int launch_select_typed(const void* cand_values, const int64_t* cand_indices, int64_t rows,
                        int64_t k0, int64_t k, int index_bits, void* values, int64_t* indices,
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
                  int64_t* indices, hipStream_t stream) {
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
