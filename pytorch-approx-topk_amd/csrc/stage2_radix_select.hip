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

template <typename E, bool KEYS_IN_LDS, int COPIES>
__global__ __launch_bounds__(COPIES == 8 ? 1024 : 256) void select_kernel(
    const typename E::raw_t* __restrict__ cand_values,
    const int64_t* __restrict__ cand_indices, uint32_t k0, uint32_t k, int index_bits,
    typename E::raw_t* __restrict__ values, const IndexOut indices, select::GlobalCut* cuts,
    uint32_t* __restrict__ counts, uint32_t seg, uint32_t groups) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ select::SharedT<COPIES> sh;
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

  auto survives = [&](uint32_t i) -> bool {
    const key_t key = key_at(i);
    if (key != cut.T) return key > cut.T;
    return cut.index_cut == ~0ull || index_at(i) <= cut.index_cut;
  };
  if (cuts != nullptr) {
    // Few long rows: one CU would spend as long again writing the survivors.
    // Store the cut and the survivors of every segment of `seg` candidates;
    // a second launch writes them with one workgroup per segment.
    if (threadIdx.x == 0) cuts[row] = select::GlobalCut{(uint64_t)cut.T, cut.index_cut};
    const uint32_t lane = threadIdx.x % select::kWave, wave = threadIdx.x / select::kWave;
    const uint32_t waves = blockDim.x / select::kWave;
    for (uint32_t g = wave; g < groups; g += waves) {
      const uint32_t lo = g * seg < k0 ? g * seg : k0, hi = lo + seg < k0 ? lo + seg : k0;
      uint32_t kept = 0;
      uint32_t base = lo;
      for (; base + 4 * select::kWave <= hi; base += 4 * select::kWave) {  // independent LDS reads
        bool sel[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) sel[u] = survives(base + u * select::kWave + lane);
#pragma unroll
        for (int u = 0; u < 4; ++u) kept += (uint32_t)__popcll(__ballot(sel[u]));
      }
      for (; base < hi; base += select::kWave) {
        const uint32_t i = base + lane;
        kept += (uint32_t)__popcll(__ballot(i < hi && survives(i)));
      }
      if (lane == 0) counts[row * groups + g] = kept;
    }
    return;
  }
  raw_t* ov = values + row * (int64_t)k;
  const int64_t oi = row * (int64_t)k;  // this row's first output slot
  select::compact(
      sh, k0, k, survives,
      [&](uint32_t i) { return Candidate<raw_t>{cv[i], ci[i]}; },
      [&](uint32_t, uint32_t o, const Candidate<raw_t>& c) {
        if (values != nullptr) ov[o] = c.value;
        indices.put(oi + o, c.index);
      });
}

// LDS a workgroup may use for keys; the rest of the 160 KB of a gfx950 CU is
// left to the static block above and to a second resident workgroup's needs.
constexpr size_t kMaxKeyLds = 128 * 1024;

// Few rows of many candidates each: the survivors are written by a second
// launch, kSegments workgroups per row (measured per call, 1-32 rows, k = k0/4:
// 8192 candidates 13 us in one launch, 18 us in two; 16384: 19 us either way;
// 32768: 31 us in one, 26 us in two).
constexpr int64_t kSplitMinCandidates = 24576;
constexpr int64_t kSplitMaxRows = 32;
constexpr uint32_t kSegments = 32;
// Rows from which the select is sized for throughput rather than for one row's latency.
constexpr int64_t kManyRows = 1024;

struct SplitPlan {
  bool use;
  uint32_t seg;
  size_t counts_off, total;
};

SplitPlan plan_split(int64_t rows, int64_t k0, int64_t k) {
  SplitPlan sp{};
  sp.use = rows > 0 && rows <= kSplitMaxRows && k0 >= kSplitMinCandidates && k > 0 && k < k0;
  if (!sp.use) return sp;
  sp.seg = (uint32_t)(((k0 + kSegments - 1) / kSegments + 255) / 256 * 256);
  sp.counts_off = ((size_t)rows * sizeof(select::GlobalCut) + 255) / 256 * 256;
  sp.total = sp.counts_off + ((size_t)rows * kSegments * sizeof(uint32_t) + 255) / 256 * 256;
  return sp;
}

template <typename E>
int launch_select_typed(const void* cand_values, const int64_t* cand_indices, int64_t rows,
                        int64_t k0, int64_t k, int index_bits, void* values, IndexOut indices,
                        select::GlobalCut* cuts, uint32_t* counts, uint32_t seg, hipStream_t stream) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  const size_t key_bytes = (size_t)k0 * sizeof(key_t);
  const bool in_lds = key_bytes <= kMaxKeyLds;
  // Few rows: as many threads as help one row finish early (256 with two
  // histogram copies up to 1024 candidates: 5.5-8.1 us where 512 threads with
  // eight copies take 6.1-9.1 us).  Many rows (four or more per CU): about four
  // candidates per thread, so that more rows are resident and in different
  // phases (measured on [4096 rows, 1024 candidates]: 38 -> 27 us; on
  // [16384, 256]: 512 threads 99 us, 64 threads 28 us).
  int nt = 1024;
  if (k0 <= 1024) nt = 256;
  if (rows >= kManyRows) {
    nt = 64;
    while (nt < 1024 && (int64_t)nt * 4 < k0) nt *= 2;
  }
  const dim3 grid((unsigned)rows), block(nt);
  if (in_lds && nt <= 256) {
    // small workgroups (many rows of few candidates): wave 0 spends longer
    // summing eight histogram copies than the copies save in LDS conflicts
    // (measured on [16384 rows, 256 candidates]: 65 -> 28 us with one copy)
    auto kern = nt <= 128 ? select_kernel<E, true, 1> : select_kernel<E, true, 2>;
    hipLaunchKernelGGL(kern, grid, block, key_bytes, stream, (const raw_t*)cand_values,
                       cand_indices, (uint32_t)k0, (uint32_t)k, index_bits, (raw_t*)values,
                       indices, cuts, counts, seg, kSegments);
  } else if (in_lds) {
    auto kern = select_kernel<E, true, 8>;
    if (key_bytes > 48 * 1024) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)key_bytes) != hipSuccess)
        return ATK_ERR_LAUNCH;
    }
    hipLaunchKernelGGL(kern, grid, block, key_bytes, stream, (const raw_t*)cand_values,
                       cand_indices, (uint32_t)k0, (uint32_t)k, index_bits, (raw_t*)values,
                       indices, cuts, counts, seg, kSegments);
  } else {
    hipLaunchKernelGGL((select_kernel<E, false, 8>), grid, block, 0, stream,
                       (const raw_t*)cand_values, cand_indices, (uint32_t)k0, (uint32_t)k,
                       index_bits, (raw_t*)values, indices, cuts, counts, seg, kSegments);
  }
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

}  // namespace

size_t select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int dtype) {
  (void)dtype;
  const SplitPlan sp = plan_split(rows, k0, k);
  return sp.use ? sp.total : 0;
}

void describe_select(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, bool with_workspace,
                     std::string& out) {
  (void)index_bound;
  const int kb = elem_bytes(dtype) == 8 ? 8 : 4;  // bytes of an order key
  const bool in_lds = (size_t)k0 * kb <= kMaxKeyLds;
  int nt = 1024;
  if (k0 <= 1024) nt = 256;
  if (rows >= kManyRows) {
    nt = 64;
    while (nt < 1024 && (int64_t)nt * 4 < k0) nt *= 2;
  }
  const int copies = (in_lds && nt <= 256) ? (nt <= 128 ? 1 : 2) : 8;
  const SplitPlan sp = plan_split(rows, k0, k);
  out += "select_kernel<" + std::string(dtype_name(dtype)) + ", KEYS_IN_LDS=" + (in_lds ? "1" : "0") +
         ", COPIES=" + std::to_string(copies) + "> grid=" + std::to_string(rows) + " block=" + std::to_string(nt);
  if (sp.use && with_workspace)
    out += " + ms_emit_kernel<" + std::string(dtype_name(dtype)) + "> grid=" + std::to_string(rows * kSegments);
}

int launch_select(const void* cand_values, const int64_t* cand_indices, int64_t rows,
                  int64_t k0, int64_t k, int64_t index_bound, int dtype, void* values,
                  IndexOut indices, void* ws, size_t ws_bytes, hipStream_t stream) {
  if (k0 > 0x7fffffffll || rows > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  int index_bits = 1;
  while (index_bits < 63 && (1ll << index_bits) < index_bound) ++index_bits;
  // without a workspace the one workgroup also writes the survivors
  const SplitPlan sp = plan_split(rows, k0, k);
  const bool split = sp.use && ws != nullptr && ws_bytes >= sp.total && (uintptr_t)ws % 16 == 0;
  select::GlobalCut* cuts = split ? static_cast<select::GlobalCut*>(ws) : nullptr;
  uint32_t* counts = split ? reinterpret_cast<uint32_t*>(static_cast<unsigned char*>(ws) + sp.counts_off) : nullptr;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = launch_select_typed<E>(cand_values, cand_indices, rows, k0, k, index_bits, values,
                                               indices, cuts, counts, sp.seg, stream));
  if (rc != ATK_OK || !split) return rc;
  return launch_emit_segments(cand_values, cand_indices, rows, k0, k, sp.seg, kSegments, cuts, counts, dtype,
                              values, indices, stream);
}

}  // namespace atk
