// Block-wide exact top-k selection over candidates held by one workgroup.
//
// An MSB-first radix select with 8-bit digits finds the order key T of the k-th
// best candidate and how many of the candidates with key == T belong to the
// result; when only part of that tie group belongs, a second radix select over
// the candidates' original indices finds the cut so that the lowest indices
// win.  Survivors are then emitted in increasing candidate position with
// wave-level ballot/mbcnt compaction.  Candidates are reached through
// accessors, so the same code serves keys staged in LDS, keys re-read from
// global memory, and candidates that never left the workgroup.
//
// Every function here must be called by all threads of the workgroup.
#pragma once

#include "atk_device.h"

namespace atk {
namespace select {

constexpr int kWave = 64;
constexpr int kMaxWaves = 16;

// Histogram counters are kept in COPIES private copies (lane % kCopies picks
// one) so that the many candidates sharing a digit -- the top byte of a float
// key is nearly constant among top-k candidates -- do not serialise on one LDS
// address; the odd stride spreads equal digits of different copies over banks.
constexpr int kCopyStride = 257;
// Tie groups up to this size are cut by ranking their listed indices in one
// wave instead of by radix passes over all candidates.
constexpr int kTieList = 64;

template <int COPIES> struct SharedT {
  static constexpr int kCopies = COPIES;
  uint32_t copies[COPIES * kCopyStride];  // all zero between passes
  uint32_t wave_total[kMaxWaves];
  uint32_t digit;
  uint32_t need;
  uint32_t bin_count;
  // a short tie group, listed: original indices of the candidates with key == T
  uint32_t tie_count;
  uint64_t tie_index[kTieList];
  uint64_t index_cut;
};
using Shared = SharedT<8>;  // the stand-alone select kernel; the fused kernel takes fewer copies to save LDS


__device__ __forceinline__ uint32_t lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

// Number of set bits of `m` below this lane.
__device__ __forceinline__ uint32_t rank_in(uint64_t m) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                   __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
}

// Wave 0 sums the private copies of the 256-bin histogram (and leaves them zero
// for the next pass), scans for the bin holding the `need`-th element, counting
// from the top bin (FROM_TOP) or from the bottom bin, and publishes the bin,
// the rank left within it and the bin's population.
template <bool FROM_TOP, typename Sh>
__device__ __forceinline__ void find_bin(Sh& sh, uint32_t need) {
  if (threadIdx.x < kWave) {
    const uint32_t lane = threadIdx.x;
    // Lane l owns bins 4l..4l+3.
    uint32_t h[4] = {0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < Sh::kCopies; ++c) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        h[i] += sh.copies[c * kCopyStride + 4 * lane + i];
        sh.copies[c * kCopyStride + 4 * lane + i] = 0;
      }
    }
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

// One radix pass: histogram digit `shift` of the values `digit_source(i)` over
// the candidates with `participates(i)`, then locate the bin of rank `need`.
template <bool FROM_TOP, typename Participates, typename Sh>
__device__ __forceinline__ void radix_pass(Sh& sh, uint32_t k0, uint32_t need, Participates digit_or_skip) {
  const uint32_t tid = threadIdx.x, nt = blockDim.x;
  uint32_t* my_copy = &sh.copies[(tid % Sh::kCopies) * kCopyStride];
  __syncthreads();  // the copies are zero (clear_copies, or the last pass's find_bin)
  // four candidates per trip, so that their LDS reads and adds overlap
  uint32_t i = tid;
  for (; i + 3 * nt < k0; i += 4 * nt) {
    int d[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) d[u] = digit_or_skip(i + u * nt);  // 0..255, or -1: out of the race
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (d[u] >= 0) atomicAdd(&my_copy[d[u]], 1u);
  }
  for (; i < k0; i += nt) {
    const int d = digit_or_skip(i);
    if (d >= 0) atomicAdd(&my_copy[d], 1u);
  }
  __syncthreads();
  find_bin<FROM_TOP>(sh, need);
  __syncthreads();
}

// Zeroes the histogram copies before the first pass (no barrier: radix_pass
// starts with one).
template <typename Sh> __device__ __forceinline__ void clear_copies(Sh& sh) {
  for (uint32_t i = threadIdx.x; i < Sh::kCopies * kCopyStride; i += blockDim.x) sh.copies[i] = 0;
}

// A row's cut as kernels hand it to one another through global memory:
// survivors have key > cut.key, or key == cut.key and index <= cut.index.
struct GlobalCut { uint64_t key, index; };

// The cut: candidate i survives iff key(i) > T, or key(i) == T and index(i) <= index_cut.
template <typename key_t> struct Cut {
  key_t T;
  uint64_t index_cut;  // ~0: every tie survives
};

// The largest index taken among the candidates with key == T when `need` of them
// (those with the lowest indices) belong to the result: radix passes over the
// indices, least index first.  The histogram copies must be zero on entry.
template <typename key_t, typename KeyAt, typename IndexAt, typename Sh>
__device__ __forceinline__ uint64_t index_cut_among_ties(Sh& sh, uint32_t k0, key_t T, uint32_t need, int index_bits,
                                                         KeyAt key_at, IndexAt index_at) {
  uint64_t iprefix = 0, imask = 0;
  for (int shift = ((index_bits + 7) / 8 - 1) * 8; shift >= 0; shift -= 8) {
    radix_pass<false>(sh, k0, need, [&](uint32_t i) -> int {
      if (key_at(i) != T) return -1;
      const uint64_t idx = index_at(i);
      return (idx & imask) == iprefix ? (int)((uint32_t)(idx >> shift) & 0xffu) : -1;
    });
    iprefix |= (uint64_t)sh.digit << shift;
    imask |= (uint64_t)0xff << shift;
    need = sh.need;
  }
  return iprefix;
}

// key_at(i): order key of candidate i; index_at(i): its original index (only
// read for candidates tied at T, and only when the tie group is cut).
template <typename key_t, int KEY_BITS, typename KeyAt, typename IndexAt, typename Sh>
__device__ __forceinline__ Cut<key_t> find_cut(Sh& sh, uint32_t k0, uint32_t k, int index_bits, KeyAt key_at,
                                      IndexAt index_at) {
  key_t prefix = 0, mask = 0;
  uint32_t need = k;
  clear_copies(sh);
  for (int shift = KEY_BITS - 8; shift >= 0; shift -= 8) {
    radix_pass<true>(sh, k0, need, [&](uint32_t i) -> int {
      const key_t key = key_at(i);
      return (key & mask) == prefix ? (int)((uint32_t)(key >> shift) & 0xffu) : -1;
    });
    prefix |= (key_t)sh.digit << shift;
    mask |= (key_t)0xff << shift;
    need = sh.need;
  }
  Cut<key_t> cut{prefix, ~0ull};
  const uint32_t ties = sh.bin_count;  // candidates with key == T
  if (need < ties && ties <= (uint32_t)kTieList) {  // uniform over the workgroup
    // list the tied candidates' indices (in any order), then one wave finds
    // the need-th smallest by counting, for every index, the smaller ones
    const uint32_t tid = threadIdx.x, nt = blockDim.x;
    if (tid == 0) sh.tie_count = 0;
    __syncthreads();
    for (uint32_t i = tid; i < k0; i += nt) {
      if (key_at(i) == cut.T) sh.tie_index[atomicAdd(&sh.tie_count, 1u)] = index_at(i);
    }
    __syncthreads();
    if (tid < (uint32_t)kWave) {
      const uint64_t mine = tid < ties ? sh.tie_index[tid] : ~0ull;
      uint32_t smaller = 0;
      for (uint32_t m = 0; m < ties; ++m) smaller += sh.tie_index[m] < mine ? 1u : 0u;
      if (tid < ties && smaller == need - 1) sh.index_cut = mine;
    }
    __syncthreads();
    cut.index_cut = sh.index_cut;
  } else if (need < ties) {
    cut.index_cut = index_cut_among_ties(sh, k0, cut.T, need, index_bits, key_at, index_at);
  }
  return cut;
}

// The same when the key T of the k-th best is already known, with more
// candidates of that key than belong to the result: `need` of them do, the ones
// with the lowest indices.
template <typename key_t, typename KeyAt, typename IndexAt, typename Sh>
__device__ __forceinline__ Cut<key_t> cut_among_ties(Sh& sh, uint32_t k0, key_t T, uint32_t need, int index_bits,
                                                     KeyAt key_at, IndexAt index_at) {
  clear_copies(sh);
  return Cut<key_t>{T, index_cut_among_ties(sh, k0, T, need, index_bits, key_at, index_at)};
}

// Stable compaction: wave w owns a contiguous run of candidates.  fetch(i) is
// called for every candidate of a group before any of them is tested, so that
// its loads (coalesced, independent of the outcome) overlap; emit(i, o, what
// fetch(i) returned) is called for every surviving candidate i with its output
// slot o < k.
template <typename Survives, typename Fetch, typename Emit, typename Sh>
__device__ __forceinline__ void compact(Sh& sh, uint32_t k0, uint32_t k, Survives survives, Fetch fetch,
                                        Emit emit) {
  const uint32_t tid = threadIdx.x, nt = blockDim.x;
  const uint32_t waves = nt / kWave, wave = tid / kWave, lane = lane_id();
  uint32_t per_wave = (k0 + waves - 1) / waves;
  per_wave = (per_wave + kWave - 1) / kWave * kWave;
  const uint32_t lo = min(wave * per_wave, k0), hi = min(lo + per_wave, k0);
  uint32_t mine = 0;
  uint32_t base = lo;
  for (; base + 4 * kWave <= hi; base += 4 * kWave) {  // four groups per trip: independent LDS reads
    bool sel[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) sel[u] = survives(base + u * kWave + lane);
#pragma unroll
    for (int u = 0; u < 4; ++u) mine += (uint32_t)__popcll(__ballot(sel[u]));
  }
  for (; base < hi; base += kWave) {
    const uint32_t i = base + lane;
    const bool sel = i < hi && survives(i);
    mine += (uint32_t)__popcll(__ballot(sel));
  }
  __syncthreads();
  if (lane == 0) sh.wave_total[wave] = mine;
  __syncthreads();
  uint32_t out = 0;
  for (uint32_t w = 0; w < wave; ++w) out += sh.wave_total[w];
  using Fetched = decltype(fetch(0u));
  base = lo;
  for (; base + 4 * kWave <= hi; base += 4 * kWave) {
    Fetched got[4];
    bool sel[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) got[u] = fetch(base + u * kWave + lane);
#pragma unroll
    for (int u = 0; u < 4; ++u) sel[u] = survives(base + u * kWave + lane);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint64_t m = __ballot(sel[u]);
      if (sel[u]) {
        const uint32_t o = out + rank_in(m);
        if (o < k) emit(base + u * kWave + lane, o, got[u]);
      }
      out += (uint32_t)__popcll(m);
    }
  }
  for (; base < hi; base += kWave) {
    const uint32_t i = base + lane;
    const bool sel = i < hi && survives(i);
    const uint64_t m = __ballot(sel);
    if (sel) {
      const uint32_t o = out + rank_in(m);
      if (o < k) emit(i, o, fetch(i));
    }
    out += (uint32_t)__popcll(m);
  }
}

// ---------------------------------------------------------------------------
// Pieces of a selection over candidates that stay in the registers of the
// threads that hold them: MSB-first radix passes with 11-bit digits whose
// histograms (LDS, one atomic add per candidate) one wave reads, and the
// wave-level scans they need.
// ---------------------------------------------------------------------------
namespace regs {

constexpr int kDigitBits = 11;
constexpr int kBins = 1 << kDigitBits;
constexpr uint32_t kListMax = 64;

// A histogram holds the count of digit d at word d + (d / 32) * 4, so that the
// 32 bins every lane of a wave sums (16-byte reads, 144 bytes apart) fall on
// different LDS banks.
constexpr uint32_t kHistWords = kBins + kBins / 32 * 4;
__device__ __forceinline__ uint32_t hist_slot(uint32_t digit) { return digit + ((digit >> 1) & ~15u) / 4u; }

// LDS of a selection over candidates held in registers: two histograms (passes
// alternate, so that two barriers per pass are enough), then the listed
// candidates.
constexpr size_t kListOff = 2 * (size_t)kHistWords * sizeof(uint32_t);
constexpr size_t kListWords = kListMax + 8;  // rounded up to whole groups of eight when ranking
constexpr size_t kLdsBytes = kListOff + 2 * kListWords * sizeof(uint64_t);

struct Shared {
  uint32_t wave_total[kMaxWaves];
  uint32_t wave_low[kMaxWaves], wave_high[kMaxWaves];  // per-wave smallest and largest key
  uint32_t list_count;
  uint32_t digit, need, count;       // what wave 0 found in the last pass
  uint64_t cut_key, cut_index;       // the cut, when wave 0 ranked a list
};

// Inclusive prefix sum over the 64 lanes of a wave, in registers.
__device__ __forceinline__ uint32_t wave_scan(uint32_t v) {
  // within rows of 16 lanes: shifts by 1, 2, 4, 8 (lanes without a source add 0)
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x111, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x112, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x114, 0xf, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x118, 0xf, 0xf, false);
  // lane 15 of a row into the next row (rows 1 and 3), then lane 31 into rows 2 and 3
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x142, 0xa, 0xf, false);
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x143, 0xc, 0xf, false);
  return v;
}

// Smallest and largest of a 32-bit value over the 64 lanes of a wave, in every
// lane: the steps of wave_scan with min / max in place of the sum (lanes without
// a source take the identity), then the last lane's result for all.
__device__ __forceinline__ uint32_t wave_min(uint32_t v) {
#define ATK_WAVE_STEP(ctrl, rows)                                                                      \
  {                                                                                                     \
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)~0u, (int)v, ctrl, rows, 0xf, false); \
    v = o < v ? o : v;                                                                                  \
  }
  ATK_WAVE_STEP(0x111, 0xf) ATK_WAVE_STEP(0x112, 0xf) ATK_WAVE_STEP(0x114, 0xf) ATK_WAVE_STEP(0x118, 0xf)
  ATK_WAVE_STEP(0x142, 0xa) ATK_WAVE_STEP(0x143, 0xc)
#undef ATK_WAVE_STEP
  return (uint32_t)__builtin_amdgcn_readlane((int)v, kWave - 1);
}
__device__ __forceinline__ uint32_t wave_max(uint32_t v) {
#define ATK_WAVE_STEP(ctrl, rows)                                                                  \
  {                                                                                                 \
    const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, ctrl, rows, 0xf, false);    \
    v = o > v ? o : v;                                                                              \
  }
  ATK_WAVE_STEP(0x111, 0xf) ATK_WAVE_STEP(0x112, 0xf) ATK_WAVE_STEP(0x114, 0xf) ATK_WAVE_STEP(0x118, 0xf)
  ATK_WAVE_STEP(0x142, 0xa) ATK_WAVE_STEP(0x143, 0xc)
#undef ATK_WAVE_STEP
  return (uint32_t)__builtin_amdgcn_readlane((int)v, kWave - 1);
}

struct Found { uint32_t digit, need, count; };  // wave-uniform

// One wave, all 64 lanes: the bin that holds the need-th entry (1-based) of
// `total` counted from the best digit down, the rank left within it (again from
// the best) and its population.  PADDED: the histogram has the layout of
// hist_slot; else digit d is word d, and the lanes start their 16-byte reads at
// different quarters of their 128 bytes to stay off each other's banks (two
// more operations per read and eight address registers for the one reader, for
// writers that have the registers to spare and many candidates to count).
template <bool PADDED = true>
__device__ __forceinline__ Found find_bin_wave(const uint32_t* hist, uint32_t need_from_top, uint32_t total,
                                               uint32_t lane) {
  const uint32_t need = total - need_from_top + 1u;  // counted from the weakest digit up
  constexpr uint32_t kStride = PADDED ? 36u : 32u;   // words between the chunks of neighbouring lanes
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t quarter = PADDED ? (uint32_t)i : ((lane + (uint32_t)i) & 7u);
    const uint4 h = *reinterpret_cast<const uint4*>(&hist[lane * kStride + 4u * quarter]);
    mine += h.x + h.y + h.z + h.w;
  }
  const uint32_t incl = wave_scan(mine);
  const uint64_t hit = __ballot(incl - mine < need && need <= incl);
  const int chunk = __builtin_amdgcn_readfirstlane((int)__ffsll((unsigned long long)hit) - 1);
  const uint32_t before = (uint32_t)__builtin_amdgcn_readlane((int)(incl - mine), chunk);
  // the 32 bins of that chunk, one per lane
  const uint32_t bin = lane < 32u ? hist[(uint32_t)chunk * kStride + lane] : 0u;
  const uint32_t incl2 = wave_scan(bin);
  const uint32_t left = need - before;
  const uint64_t hit2 = __ballot(incl2 - bin < left && left <= incl2);
  const int at = __builtin_amdgcn_readfirstlane((int)__ffsll((unsigned long long)hit2) - 1);
  Found f;
  f.digit = (uint32_t)chunk * 32u + (uint32_t)at;
  f.count = (uint32_t)__builtin_amdgcn_readlane((int)bin, at);
  // rank within the bin from its weakest member up, turned round
  f.need = f.count - (left - (uint32_t)__builtin_amdgcn_readlane((int)(incl2 - bin), at)) + 1u;
  return f;
}

// The digit of a key when all that is known of a row's candidates is the key
// range of every share of them (`range[0 .. entries)`: smallest and largest
// key; shares of a superset will do): with `low` the smallest key of the row
// and the row's keys spanning `width`, the digit is (key - low) >> shift, where
// shift leaves the kDigitBits leading bits of the span.  (Taking the digit from
// the offset rather than from the key's own bits keeps it fine-grained when
// the keys straddle a power of two, where most bits of the smallest and the
// largest key differ.)  Whole workgroup of THREADS threads; `red` is
// 2 * THREADS / 64 words of LDS; contains a barrier, after which every thread
// holds the result.
// The ranges this thread looks at, folded: the first half of digit_of_row, for
// callers that want the loads on their way before they wait for other data.
template <int THREADS>
__device__ __forceinline__ uint2 fold_ranges(const uint2* __restrict__ range, uint32_t entries) {
  uint32_t lo = ~0u, hi = 0;
  for (uint32_t g = threadIdx.x; g < entries; g += THREADS) {
    const uint2 r = range[g];
    lo = r.x < lo ? r.x : lo;
    hi = r.y > hi ? r.y : hi;
  }
  return make_uint2(lo, hi);
}

template <int THREADS>
__device__ __forceinline__ void digit_from_folded(uint2 folded, uint32_t* red, uint32_t& low, uint32_t& shift) {
  constexpr int kWaves = THREADS / kWave;
  const uint32_t tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  uint32_t lo = folded.x, hi = folded.y;
  lo = wave_min(lo);
  hi = wave_max(hi);
  if (lane == 0) { red[wave] = lo; red[kWaves + wave] = hi; }
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    lo = red[w] < lo ? red[w] : lo;
    hi = red[kWaves + w] > hi ? red[kWaves + w] : hi;
  }
  const uint32_t span = lo >= hi ? 0u : 32u - (uint32_t)__builtin_clz(hi - lo);  // bits of the largest offset
  low = lo >= hi ? hi : lo;
  shift = span > (uint32_t)kDigitBits ? span - (uint32_t)kDigitBits : 0u;
}

template <int THREADS>
__device__ __forceinline__ void digit_of_row(const uint2* __restrict__ range, uint32_t entries, uint32_t* red,
                                             uint32_t& low, uint32_t& shift) {
  digit_from_folded<THREADS>(fold_ranges<THREADS>(range, entries), red, low, shift);
}

}  // namespace regs

}  // namespace select
}  // namespace atk
