// Stage 2 for few rows of many candidates (thousands to tens of thousands per
// row): the exact top-k selection spread over several workgroups per row in a
// short chain of launches.
//
// One workgroup per row (stage2_radix_select.hip) pushes all of a row's
// candidates through one CU: about 0.8 us per thousand candidates, 25 us at
// 32768.  Here a row is cut into segments of 1024 or 4096 candidates, one workgroup
// each, and up to four small kernels follow one another on the stream:
//
//   range:   every workgroup finds the smallest and largest order key of its
//            segment (and clears its share of the row's histogram).
//   hist:    from the row's key range every workgroup works out the digit of
//            a key, the leading 11 bits of its offset from the row's smallest
//            key within the span of the row's keys, and adds its segment's
//            digit histogram to the row's.  (The candidates of a top-k lie
//            close together: their keys span a small part of the key space.)
//   refine:  every workgroup finds the digit B of the k-th best from the row's
//            histogram, counts its candidates above B and lists those in B
//            (order key, inverted index and candidate number) in the row's list.
//   emit:    every workgroup ranks the listed candidates (a few dozen, as a rule)
//            to find the weakest survivor, offsets by the survivors of the
//            segments before it and writes its own in candidate order.
//
// A candidate is the 64-bit word (order key, inverted index): a greater word is a
// better candidate and no two are equal, so that ties go to the lower index.
// When the digit B holds more candidates than a workgroup's LDS list takes
// (kListCap; keys that crowd into a small part of their span: heavy tails,
// outliers), the members of B are counted again by the next 11 bits of their
// offsets, and so on, through the bits of the key and then of the index, until
// the cut digit fits (every emit workgroup does this over the row's list in
// global memory, which holds all of B; the one-launch form narrows over the key
// bits of the keys in its registers and, in the forms built with TIES, over the
// index bits; without TIES it leaves a row with more than kListCap candidates
// of one key around the cut to its first workgroup, with radix passes over the
// indices of all candidates of that key).  When stage 1 ends in kernels that can leave key ranges and the
// histogram behind (KeyRangeOut: the streaming kernel's slabs and their merge),
// the range and hist launches are skipped.  Results are those of the
// one-workgroup kernel: same survivors, same order.
#include "atk_device.h"
#include "atk_launch.h"
#include "atk_trace.h"
#include "stage2_select.h"

namespace atk {
namespace {

namespace regs = select::regs;

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / select::kWave;
// Candidates per thread of the chain's kernels (PT): 4, so that a few rows spread over
// many CUs, or 16 when the rows are many enough for that anyway (a workgroup's fixed
// work -- the row's histogram, the ranges, the search -- is then shared by four times
// the candidates).  A segment is kThreads * PT candidates.
constexpr int kPerThreadFew = 4, kPerThreadMany = 16;
constexpr uint32_t kSoloSegment = 1024;  // the one-launch form's segments (one candidate per thread)
constexpr uint32_t kListCap = 2048;                   // listed candidates a row can hold
constexpr uint32_t kRankDirect = 256;                 // lists up to this size are ranked by counting

// Per-row words in the workspace.
struct RowState {
  uint32_t list_count;  // candidates appended to the row's list
  uint32_t digit;       // B
  uint32_t need;        // members of B that belong to the result
  uint32_t count;       // members of B
  uint32_t shift, low;  // the digit is (key - low) >> shift
  uint32_t unused[2];
};

// Shares per row whose key ranges the workspace has room for: the chain's own
// segments, or the workgroups of a stage-1 kernel that left them (KeyRangeOut).
constexpr uint32_t kRangeCapacity = 4096;

struct ChainPlan {
  bool use;
  bool solo;        // one launch does it (chain_solo_kernel)
  int per_thread;   // candidates per thread of the chain's kernels
  uint32_t groups;  // workgroups per row
  uint32_t range_capacity;
  size_t range_off, hist_off, state_off, above_off, list_word_off, list_at_off, total;
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Thread t of a workgroup holds candidates first + u * kThreads, u = 0..PT-1, of its row.
template <typename E, int PT>
__device__ __forceinline__ void load_keys(const typename E::raw_t* __restrict__ cv, uint32_t first, uint32_t k0,
                                          uint32_t (&key)[PT], bool (&valid)[PT]) {
  typename E::raw_t raw[PT];
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    valid[u] = first + u * kThreads < k0;
    raw[u] = valid[u] ? cv[first + u * kThreads] : (typename E::raw_t)0;
  }
#pragma unroll
  for (int u = 0; u < PT; ++u) key[u] = (uint32_t)E::key(raw[u]);
}

template <typename E, int PT>
__global__ __launch_bounds__(kThreads) void chain_range_kernel(const typename E::raw_t* __restrict__ cand_values,
                                                               uint32_t k0, uint32_t groups, uint2* __restrict__ range,
                                                               uint32_t* __restrict__ hist, RowState* __restrict__ state) {
  __shared__ uint32_t wave_low[kWaves], wave_high[kWaves];
  const uint32_t row = blockIdx.x / groups, g = blockIdx.x - row * groups;
  const uint32_t tid = threadIdx.x, lane = tid % select::kWave, wave = tid / select::kWave;
  uint32_t key[PT];
  bool valid[PT];
  load_keys<E, PT>(cand_values + (int64_t)row * k0, g * (kThreads * (uint32_t)PT) + tid, k0, key, valid);
  uint32_t low = ~0u, high = 0;
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    if (valid[u]) {
      low = key[u] < low ? key[u] : low;
      high = key[u] > high ? key[u] : high;
    }
  }
  low = regs::wave_min(low);
  high = regs::wave_max(high);
  if (lane == 0) { wave_low[wave] = low; wave_high[wave] = high; }
  // this workgroup's share of the row's histogram, and the row's state
  uint32_t* h = hist + (size_t)row * regs::kHistWords;
  for (uint32_t i = g * kThreads + tid; i < regs::kHistWords; i += groups * kThreads) h[i] = 0;
  if (g == 0 && tid == 0) state[row] = RowState{0, 0, 0, 0, 0, 0, {0, 0}};
  __syncthreads();
  if (tid == 0) {
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      low = wave_low[w] < low ? wave_low[w] : low;
      high = wave_high[w] > high ? wave_high[w] : high;
    }
    range[(size_t)row * groups + g] = make_uint2(low, high);
  }
}

template <typename E, int PT>
__global__ __launch_bounds__(kThreads) void chain_hist_kernel(const typename E::raw_t* __restrict__ cand_values,
                                                              uint32_t k0, uint32_t groups,
                                                              const uint2* __restrict__ range, uint32_t entries,
                                                              uint32_t* __restrict__ hist) {
  __shared__ uint32_t local[regs::kHistWords];
  __shared__ uint32_t red[2 * kWaves];
  const uint32_t row = blockIdx.x / groups, g = blockIdx.x - row * groups;
  const uint32_t tid = threadIdx.x;
  uint32_t key[PT];
  bool valid[PT];
  load_keys<E, PT>(cand_values + (int64_t)row * k0, g * (kThreads * (uint32_t)PT) + tid, k0, key, valid);
  for (uint32_t i = tid; i < regs::kHistWords; i += kThreads) local[i] = 0;
  uint32_t low, shift;
  regs::digit_of_row<kThreads>(range + (size_t)row * entries, entries, red, low, shift);  // (its barrier also covers the clearing)
#pragma unroll
  for (int u = 0; u < PT; ++u)
    if (valid[u]) atomicAdd(&local[regs::hist_slot((key[u] - low) >> shift)], 1u);
  __syncthreads();
  uint32_t* h = hist + (size_t)row * regs::kHistWords;
  for (uint32_t i = tid; i < regs::kHistWords; i += kThreads) {
    const uint32_t c = local[i];
    if (c != 0) atomicAdd(&h[i], c);
  }
}

template <typename E, int PT>
__global__ __launch_bounds__(kThreads) void chain_refine_kernel(
    const typename E::raw_t* __restrict__ cand_values, const int64_t* __restrict__ cand_indices, uint32_t k0,
    uint32_t k, uint32_t groups, const uint2* __restrict__ range, uint32_t entries,
    const uint32_t* __restrict__ hist, RowState* __restrict__ state, uint32_t* __restrict__ above,
    uint64_t* __restrict__ list_word, uint32_t* __restrict__ list_at) {
  __shared__ __align__(16) uint32_t local[regs::kHistWords];
  __shared__ regs::Found found;
  __shared__ uint32_t wave_above[kWaves], wave_listed[kWaves];
  __shared__ uint32_t list_base;
  __shared__ uint32_t red[2 * kWaves];
  const uint32_t row = blockIdx.x / groups, g = blockIdx.x - row * groups;
  const uint32_t tid = threadIdx.x, lane = tid % select::kWave, wave = tid / select::kWave;
  const uint32_t first = g * (kThreads * (uint32_t)PT) + tid;
  // everything this workgroup reads is asked for at once: keys, indices, the row's histogram and ranges
  uint32_t key[PT], inv[PT];
  bool valid[PT];
  load_keys<E, PT>(cand_values + (int64_t)row * k0, first, k0, key, valid);
  const int64_t* ci = cand_indices + (int64_t)row * k0;
#pragma unroll
  for (int u = 0; u < PT; ++u) inv[u] = valid[u] ? ~(uint32_t)ci[first + u * kThreads] : 0u;
  const uint32_t* h = hist + (size_t)row * regs::kHistWords;
  for (uint32_t i = tid; i < regs::kHistWords; i += kThreads) local[i] = h[i];
  uint32_t low, shift;
  regs::digit_of_row<kThreads>(range + (size_t)row * entries, entries, red, low, shift);  // (its barrier also publishes `local`)
  if (wave == 0) {
    const regs::Found f = regs::find_bin_wave(local, k, k0, lane);
    if (lane == 0) found = f;
  }
  __syncthreads();
  const regs::Found f = found;
  uint32_t mine = 0;
  bool member[PT];  // of a digit that is cut: ranked later, from the row's list
  uint32_t listed = 0;
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    const uint32_t d = (key[u] - low) >> shift;
    // survivors known now: above B, and all of B when none of it is cut
    mine += (valid[u] && (d > f.digit || (d == f.digit && f.need == f.count))) ? 1u : 0u;
    member[u] = valid[u] && d == f.digit && f.need != f.count;
    listed += member[u] ? 1u : 0u;
  }
  const uint32_t incl = regs::wave_scan(mine);
  const uint32_t listed_incl = regs::wave_scan(listed);
  if (lane == select::kWave - 1) { wave_above[wave] = incl; wave_listed[wave] = listed_incl; }
  __syncthreads();
  if (tid == 0) {
    uint32_t total = 0, total_listed = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) { total += wave_above[w]; total_listed += wave_listed[w]; }
    above[(size_t)row * groups + g] = total;
    // one reservation in the row's list for the whole workgroup (the row's list takes
    // all k0 candidates, so every member has a place)
    list_base = total_listed != 0 ? atomicAdd(&state[row].list_count, total_listed) : 0u;
    if (g == 0) {
      RowState* s = &state[row];
      s->digit = f.digit; s->need = f.need; s->count = f.count; s->shift = shift; s->low = low;
    }
  }
  if (f.need == f.count) return;  // (uniform) nothing is listed
  __syncthreads();
  uint32_t slot = list_base + listed_incl - listed;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) slot += (uint32_t)w < wave ? wave_listed[w] : 0u;
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    if (member[u]) {
      list_word[(size_t)row * k0 + slot] = ((uint64_t)key[u] << 32) | (uint64_t)inv[u];
      list_at[(size_t)row * k0 + slot] = first + u * kThreads;
      ++slot;
    }
  }
}

template <typename E, int PT>
__global__ __launch_bounds__(kThreads) void chain_emit_kernel(
    const typename E::raw_t* __restrict__ cand_values, const int64_t* __restrict__ cand_indices, uint32_t k0,
    uint32_t k, uint32_t groups, int index_bits, const RowState* __restrict__ state,
    const uint32_t* __restrict__ above, const uint64_t* __restrict__ list_word,
    const uint32_t* __restrict__ list_at, typename E::raw_t* __restrict__ values, const IndexOut indices) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ select::SharedT<2> sh;
  __shared__ uint64_t cut_word;
  __shared__ uint32_t listed_before;
  __shared__ uint32_t wave_kept[PT][kWaves];
  __shared__ regs::Found found;
  __shared__ uint32_t lds_count;
  const uint32_t row = blockIdx.x / groups, g = blockIdx.x - row * groups;
  const uint32_t tid = threadIdx.x, lane = tid % select::kWave, wave = tid / select::kWave;
  const uint64_t* lw = list_word + (size_t)row * k0;
  const uint32_t* la = list_at + (size_t)row * k0;
  // asked for before the row's state is known: the start of the list (most lists end within it) and
  // the survivors counted for the segments before this one
  const uint64_t early_word = lw[tid];
  const uint32_t early_at = la[tid];
  uint32_t counted = 0;
  for (uint32_t p = tid; p < g; p += kThreads) counted += above[(size_t)row * groups + p];
  const RowState s = state[row];
  // A candidate's word less the row's smallest key, (key - low, inverted index), is what the
  // digits are taken from: the first 32 bits are the key's offset, the rest the index, so that
  // candidates of one key are told apart by their indices when the digits reach that far.
  const uint64_t low_word = (uint64_t)s.low << 32;
  uint64_t digit = s.digit;  // of (word - low_word) >> shift
  uint32_t shift = s.shift + 32u, need = s.need, count = s.count;
  const uint32_t listed = need != count ? count : 0u;  // entries of the row's list: all members of B
  const bool narrowed = listed > kListCap;
  if (narrowed) {
    // More members than a workgroup ranks: they are counted again by the next bits of their
    // words, which narrows the digit that is cut, until its members fit (the histogram borrows
    // the memory of the LDS list, which is filled afterwards).  Every workgroup of the row goes
    // through the whole list once per level; even for a row of 131072 equal keys that is several
    // times faster than leaving the row to one workgroup (65536 equal keys: 460 us there).
    uint32_t* local = reinterpret_cast<uint32_t*>(dyn_lds);
    while (need != count && count > kListCap && shift != 0) {
      const uint32_t finer = shift > (uint32_t)regs::kDigitBits ? shift - (uint32_t)regs::kDigitBits : 0u;
      const uint32_t mask = (1u << (shift - finer)) - 1u;
      for (uint32_t i = tid; i < regs::kHistWords; i += kThreads) local[i] = 0;
      __syncthreads();
      for (uint32_t i = tid; i < listed; i += kThreads) {
        const uint64_t off = lw[i] - low_word;
        if ((off >> shift) == digit) atomicAdd(&local[regs::hist_slot((uint32_t)(off >> finer) & mask)], 1u);
      }
      __syncthreads();
      if (wave == 0) {
        const regs::Found f = regs::find_bin_wave(local, need, count, lane);
        if (lane == 0) found = f;
      }
      __syncthreads();
      const regs::Found f = found;
      digit = (digit << (shift - finer)) | (uint64_t)f.digit;
      shift = finer;
      need = f.need;
      count = f.count;
    }
  }
  if (need != count && count > kListCap) {
    // No bits left and still more than the list takes: thousands of candidates
    // with one key and one index, which only a caller of the stand-alone select
    // can hand over (stage 1 gives every candidate its own index).  The row's
    // first workgroup runs the block-wide radix select of stage2_select.h over
    // all of the row's candidates, read from global memory.
    if (g != 0) return;
    const raw_t* rv = cand_values + (int64_t)row * k0;
    const int64_t* ri = cand_indices + (int64_t)row * k0;
    auto key_at = [&](uint32_t i) -> key_t { return E::key(rv[i]); };
    auto index_at = [&](uint32_t i) -> uint64_t { return (uint64_t)ri[i]; };
    const select::Cut<key_t> whole = select::find_cut<key_t, E::key_bits>(sh, k0, k, index_bits, key_at, index_at);
    auto survives = [&](uint32_t i) -> bool {
      const key_t key = key_at(i);
      if (key != whole.T) return key > whole.T;
      return whole.index_cut == ~0ull || index_at(i) <= whole.index_cut;
    };
    struct Candidate { raw_t value; int64_t index; };
    raw_t* out_values = values + (int64_t)row * k;
    const int64_t out_first = (int64_t)row * k;
    select::compact(
        sh, k0, k, survives, [&](uint32_t i) { return Candidate{rv[i], ri[i]}; },
        [&](uint32_t, uint32_t o, const Candidate& c) {
          if (values != nullptr) out_values[o] = c.value;
          indices.put(out_first + o, c.index);
        });
    return;
  }
  const bool cut_digit = need != count;  // else every member of the digit survives
  const uint32_t n = cut_digit ? count : 0u;  // members ranked here, in LDS
  uint64_t* words = reinterpret_cast<uint64_t*>(dyn_lds);
  uint32_t* ats = reinterpret_cast<uint32_t*>(dyn_lds + (size_t)kListCap * sizeof(uint64_t));
  const uint32_t first = g * (kThreads * (uint32_t)PT) + tid;
  const raw_t* cv = cand_values + (int64_t)row * k0;
  const int64_t* ci = cand_indices + (int64_t)row * k0;
  // this thread's candidates: elements, keys and indices
  raw_t raw[PT];
  uint32_t inv[PT];
  bool valid[PT];
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    valid[u] = first + u * kThreads < k0;
    raw[u] = valid[u] ? cv[first + u * kThreads] : (raw_t)0;
    inv[u] = valid[u] ? ~(uint32_t)ci[first + u * kThreads] : 0u;
  }
  // entries past the list's end count as beating nothing (ranking reads the list in groups of eight)
  if (listed <= kListCap) {
    words[tid] = tid < n ? early_word : 0ull;
    ats[tid] = tid < n ? early_at : ~0u;
    for (uint32_t i = tid + kThreads; i < ((n + 7u) & ~7u); i += kThreads) {
      words[i] = i < n ? lw[i] : 0ull;
      ats[i] = i < n ? la[i] : ~0u;
    }
  } else {
    // of the row's list, the members of the narrowed digit are ranked; those above it survive
    if (tid == 0) lds_count = 0;
    __syncthreads();  // (also: the histogram in this memory has been read)
    for (uint32_t i = tid; i < listed; i += kThreads) {
      const uint64_t w = lw[i];
      const uint32_t at = la[i];
      const uint64_t d = (w - low_word) >> shift;
      if (d > digit || (d == digit && !cut_digit)) {
        counted += at < g * (kThreads * (uint32_t)PT) ? 1u : 0u;
      } else if (d == digit) {
        const uint32_t slot = atomicAdd(&lds_count, 1u);
        words[slot] = w;
        ats[slot] = at;
      }
    }
    if (tid < 8u && n + tid < ((n + 7u) & ~7u)) {
      words[n + tid] = 0ull;
      ats[n + tid] = ~0u;
    }
  }
  if (tid == 0) { cut_word = 0; listed_before = 0; }
  __syncthreads();
  uint64_t cut = 0;  // the weakest surviving member of B (0: all of them survive)
  if (n != 0) {
    if (n <= kRankDirect) {
      // thread t counts the entries better than entry t: the need-th best is the cut
      if (tid < n) {
        const uint64_t mine = words[tid];
        uint32_t better = 0;
        for (uint32_t m = 0; m < n; m += 8) {
          uint64_t got[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) got[e] = words[m + e];
#pragma unroll
          for (int e = 0; e < 8; ++e) better += got[e] > mine ? 1u : 0u;
        }
        if (better + 1 == need) cut_word = mine;
      }
      __syncthreads();
      cut = cut_word;
    } else {
      // a longer list: the block-wide radix select over its words (all distinct)
      auto key_at = [&](uint32_t i) -> uint64_t { return words[i]; };
      auto index_at = [&](uint32_t) -> uint64_t { return 0; };
      cut = select::find_cut<uint64_t, 64>(sh, n, need, 1, key_at, index_at).T;
    }
    // listed survivors of the segments before this one
    uint32_t before = 0;
    for (uint32_t i = tid; i < n; i += kThreads) before += (ats[i] < g * (kThreads * (uint32_t)PT) && words[i] >= cut) ? 1u : 0u;
    before = regs::wave_scan(before);
    if (lane == select::kWave - 1 && before != 0) atomicAdd(&listed_before, before);
  }
  // survivors of this thread, counted per u and wave (candidate order: u, then thread)
  bool sel[PT];
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    const uint32_t key = (uint32_t)E::key(raw[u]);
    const uint64_t word = ((uint64_t)key << 32) | inv[u];
    if (!narrowed) {  // the digit lies within the key
      const uint32_t d = (key - s.low) >> (shift - 32u);
      sel[u] = valid[u] && (d > (uint32_t)digit || (d == (uint32_t)digit && word >= cut));
    } else {
      const uint64_t d = (word - low_word) >> shift;
      sel[u] = valid[u] && (d > digit || (d == digit && word >= cut));
    }
    const uint64_t m = __ballot(sel[u]);
    if (lane == 0) wave_kept[u][wave] = (uint32_t)__popcll(m);
  }
  // survivors of the segments before this one that the refine step counted
  counted = regs::wave_scan(counted);
  if (lane == select::kWave - 1 && counted != 0) atomicAdd(&listed_before, counted);
  __syncthreads();
  uint32_t base = listed_before;
  raw_t* ov = values + (int64_t)row * k;
  const int64_t oi = (int64_t)row * k;
#pragma unroll
  for (int u = 0; u < PT; ++u) {
    uint32_t o = base;
    for (int w = 0; w < kWaves; ++w) {
      if ((uint32_t)w < wave) o += wave_kept[u][w];
    }
    const uint64_t m = __ballot(sel[u]);
    if (sel[u]) {
      const uint32_t at = o + select::rank_in(m);
      if (at < k) {
        if (values != nullptr) ov[at] = raw[u];
        indices.put(oi + at, (int64_t)(uint32_t)~inv[u]);
      }
    }
#pragma unroll
    for (int w = 0; w < kWaves; ++w) base += wave_kept[u][w];
  }
}


// ---------------------------------------------------------------------------
// The chain in one launch, for rows of up to kSoloMaxCandidates (32768) candidates.
//
// The launches of the chain cost more than their work (4-7 us each against
// 1-2 us), so for rows short enough every workgroup does the row-wide steps
// itself, redundantly, and only its own segment's write-out is its own: it
// reads all of the row's keys into registers (k0 / 1024 per thread: candidate
// u * 1024 + t is thread t's u-th, so that a thread's u-th key belongs to
// segment u), builds the digit histogram in LDS, finds the digit B of the k-th
// best, lists the members of B in LDS and ranks them, counts the survivors of
// the segments before its own from the keys it holds, and writes its segment.
// The row's keys are read groups-times over (32 x 128 KiB at fp32 [1, 32768]),
// from L2 for the most part.  The key ranges come from stage 1, or from the
// keys themselves when stage 1 left none.
// ---------------------------------------------------------------------------
constexpr int kSoloThreads = 1024;  // == kSoloSegment
constexpr int kSoloWaves = kSoloThreads / select::kWave;
constexpr uint32_t kSoloRankDirect = 512;
static_assert((uint32_t)kSoloThreads == kSoloSegment, "a thread's u-th candidate lies in segment u");

// FULL: the row has exactly NPT * 1024 candidates, so that every key a thread holds exists and
// nothing has to say which do (32 wave-wide masks otherwise, which the kernel with 32 keys per
// thread has no scalar registers for).
template <typename E, int NPT, bool OWN_RANGE, bool TIES = (sizeof(typename E::raw_t) == 1 || NPT <= 16),
          bool FULL = false>
__global__ __launch_bounds__(kSoloThreads) void chain_solo_kernel(
    const typename E::raw_t* __restrict__ cand_values, const int64_t* __restrict__ cand_indices, uint32_t k0,
    uint32_t k, uint32_t groups, int index_bits, const uint2* __restrict__ range, uint32_t entries,
    typename E::raw_t* __restrict__ values, const IndexOut indices, uint32_t tie_lds) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ __align__(16) uint32_t hist[regs::kBins];  // digit d at word d (find_bin_wave<false>)
  __shared__ select::SharedT<2> sh;
  __shared__ regs::Found found;
  __shared__ uint32_t red[2 * kSoloWaves];
  __shared__ uint32_t wave_before[kSoloWaves], wave_kept[kSoloWaves];
  __shared__ uint32_t list_count;
  __shared__ uint64_t cut_word;
  uint64_t* words = reinterpret_cast<uint64_t*>(dyn_lds);
  uint32_t* ats = reinterpret_cast<uint32_t*>(dyn_lds + (size_t)(kListCap + 8) * sizeof(uint64_t));
  const uint32_t row = blockIdx.x / groups, g = blockIdx.x - row * groups;
  const uint32_t tid = threadIdx.x, lane = tid % select::kWave, wave = tid / select::kWave;
  const raw_t* cv = cand_values + (int64_t)row * k0;
  const int64_t* ci = cand_indices + (int64_t)row * k0;

  ATK_TRACE_GROUP(0);
  // (the key ranges are asked for first, so that they travel with the keys; OWN_RANGE:
  // stage 1 left none, and the range is that of the keys read below)
  uint2 folded = make_uint2(~0u, 0u);
  if constexpr (!OWN_RANGE) folded = regs::fold_ranges<kSoloThreads>(range + (size_t)row * entries, entries);
  // all keys of the row, NPT per thread (0 past the row's end; `valid` says so)
  // (The kernel is bound by instruction issue -- sixteen waves on one CU go
  // through every key of the row -- and short of registers: the keys alone take
  // up to 64 of its 128.)
  uint32_t key[NPT];
  auto valid = [&](int u) -> bool { return FULL || (uint32_t)u * kSoloThreads + tid < k0; };
  {
    raw_t raw[NPT];
#pragma unroll
    for (int u = 0; u < NPT; ++u) raw[u] = valid(u) ? cv[(uint32_t)u * kSoloThreads + tid] : (raw_t)0;
#pragma unroll
    for (int u = 0; u < NPT; ++u) key[u] = (uint32_t)E::key(raw[u]);
  }
  for (uint32_t i = tid; i < (uint32_t)regs::kBins; i += kSoloThreads) hist[i] = 0;
  if (tid == 0) { list_count = 0; cut_word = 0; }
  if constexpr (OWN_RANGE) {
#pragma unroll
    for (int u = 0; u < NPT; ++u) {
      if (valid(u)) {
        folded.x = key[u] < folded.x ? key[u] : folded.x;
        folded.y = key[u] > folded.y ? key[u] : folded.y;
      }
    }
  }
  uint32_t low, shift;
  regs::digit_from_folded<kSoloThreads>(folded, red, low, shift);  // (its barrier covers the clearing)
  ATK_TRACE_GROUP(1);
#pragma unroll
  for (int u = 0; u < NPT; ++u)
    if (valid(u)) atomicAdd(&hist[(key[u] - low) >> shift], 1u);
  __syncthreads();
  ATK_TRACE_GROUP(2);
  if (wave == 0) {
    const regs::Found f = regs::find_bin_wave<false>(hist, k, k0, lane);
    if (lane == 0) found = f;
  }
  __syncthreads();
  ATK_TRACE_GROUP(3);
  regs::Found f = found;
  // The cut digit holds more candidates than the list: they are counted again by
  // the next bits of their offsets, which narrows the digit, until its members
  // fit or no bits are left.
  if (f.need != f.count && f.count > kListCap && shift != 0) {
    // Members of one and the same key (a ReLU's zeros) are not told apart by any further level,
    // and every level would add them up in one counter, a lane at a time (16384 of them: 20 us
    // a level).  Found out first: some member leaves its key in LDS, and every thread compares
    // its members with that one.  (`red` is free: the digit's place has been worked out.)
    __syncthreads();
    if (tid == 0) red[1] = 0;
#pragma unroll
    for (int u = 0; u < NPT; ++u)
      if (valid(u) && ((key[u] - low) >> shift) == f.digit) red[0] = key[u];  // (any of them will do)
    __syncthreads();
    const uint32_t one = (uint32_t)__builtin_amdgcn_readfirstlane((int)red[0]);
    bool other = false;
#pragma unroll
    for (int u = 0; u < NPT; ++u) other |= valid(u) && ((key[u] - low) >> shift) == f.digit && key[u] != one;
    if (__ballot(other) != 0 && lane == 0) red[1] = 1;
    __syncthreads();
    if (red[1] == 0) {  // the digit is the key's offset from here on
      f.digit = one - low;
      shift = 0;
    }
  }
  while (f.need != f.count && f.count > kListCap && shift != 0) {
    const uint32_t finer = shift > (uint32_t)regs::kDigitBits ? shift - (uint32_t)regs::kDigitBits : 0u;
    const uint32_t mask = (1u << (shift - finer)) - 1u;
    __syncthreads();  // everyone has read `found`, wave 0 the histogram
    for (uint32_t i = tid; i < (uint32_t)regs::kBins; i += kSoloThreads) hist[i] = 0;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NPT; ++u) {
      const uint32_t off = key[u] - low;
      if (valid(u) && (off >> shift) == f.digit) atomicAdd(&hist[(off >> finer) & mask], 1u);
    }
    __syncthreads();
    if (wave == 0) {
      const regs::Found f2 = regs::find_bin_wave<false>(hist, f.need, f.count, lane);
      if (lane == 0) found = f2;
    }
    __syncthreads();
    const regs::Found f2 = found;
    f.digit = (f.digit << (shift - finer)) | f2.digit;
    f.need = f2.need;
    f.count = f2.count;
    shift = finer;
  }
  const bool cut_digit = f.need != f.count;  // else every member of B survives
  // TIES: shift == 0 and still too many -- thousands of candidates of one key around the cut,
  // which is what stage 1 makes of saturated 8-bit data (the bucket maxima of uniform uint8 are
  // all 255) -- and their indices decide.  Built for the 1-byte types only: the code costs the
  // kernel 4-5 us whether it runs or not (it sits at its register limit).
  const bool tie_mode = TIES && cut_digit && f.count > kListCap;
  // The list in LDS holds kListCap entries: a cut digit with more members (which, without
  // TIES, no bits are left to narrow) is not listed at all; the row then goes to the
  // whole-row path below.
  const bool list_it = cut_digit && f.count <= kListCap;
  const uint32_t own = g * kSoloThreads + tid;  // this thread's candidate of segment g
  const bool own_valid = FULL || own < k0;
  // survivors above the cut digit (or in it, when it belongs whole) in the
  // segments before this one, and the members of a cut digit: listed, or flagged for the
  // look at their indices below
  uint32_t before = 0;
  uint32_t own_key = 0;
  [[maybe_unused]] uint32_t members = 0;
#pragma unroll
  for (int u = 0; u < NPT; ++u) {
    const uint32_t d = (key[u] - low) >> shift;
    const bool ok = valid(u);
    if ((uint32_t)u < g) before += (ok && (d > f.digit || (d == f.digit && !cut_digit))) ? 1u : 0u;
    if ((uint32_t)u == g) own_key = key[u];
    if (ok && cut_digit && d == f.digit) {
      if constexpr (TIES) members |= 1u << u;
      if (list_it) {
        const uint32_t at = (uint32_t)u * kSoloThreads + tid;
        const uint32_t slot = atomicAdd(&list_count, 1u);
        words[slot] = (uint64_t)key[u] << 32;  // (the index follows below, for all members in one trip to memory)
        ats[slot] = at;
      }
    }
  }
  uint32_t need = f.need, count = f.count;
  uint64_t floor_word = 0;  // tie mode, when a whole group of indices survives: its smallest word
  if constexpr (TIES) {
    if (tie_mode) {
      // The members (all of one key) are counted by the leading bits of their inverted indices,
      // 11 at a time, until the group that is cut fits the list.  Their indices are read eight
      // segments at a time (the low halves: the planner sends only indices below 2^31 here).
      const uint32_t* ci_low = reinterpret_cast<const uint32_t*>(ci);
      auto for_members = [&](auto&& fn) __attribute__((always_inline)) {
        constexpr int kChunk = NPT < 8 ? NPT : 8;
#pragma unroll
        for (int c0 = 0; c0 < NPT; c0 += kChunk) {
          uint32_t iv[kChunk];
#pragma unroll
          for (int e = 0; e < kChunk; ++e) {
            const uint32_t i = (uint32_t)(c0 + e) * kSoloThreads + tid;
            iv[e] = i < k0 ? ci_low[2u * i] : 0u;
          }
#pragma unroll
          for (int e = 0; e < kChunk; ++e)
            if ((members >> (c0 + e)) & 1u) fn((uint32_t)(c0 + e), ~iv[e]);
        }
      };
      uint32_t ishift = 32, iprefix = 0;  // the group: inverted indices whose bits from ishift up are iprefix
      while (need != count && count > kListCap && ishift != 0) {
        const uint32_t finer = ishift > (uint32_t)regs::kDigitBits ? ishift - (uint32_t)regs::kDigitBits : 0u;
        const uint32_t mask = (1u << (ishift - finer)) - 1u;
        __syncthreads();  // everyone has read `found`, wave 0 the histogram
        for (uint32_t i = tid; i < (uint32_t)regs::kBins; i += kSoloThreads) hist[i] = 0;
        __syncthreads();
        for_members([&](uint32_t, uint32_t inv) {
          if (ishift == 32u || (inv >> ishift) == iprefix) atomicAdd(&hist[(inv >> finer) & mask], 1u);
        });
        __syncthreads();
        if (wave == 0) {
          const regs::Found f2 = regs::find_bin_wave<false>(hist, need, count, lane);
          if (lane == 0) found = f2;
        }
        __syncthreads();
        const regs::Found f2 = found;
        iprefix = (iprefix << (ishift - finer)) | f2.digit;
        ishift = finer;
        need = f2.need;
        count = f2.count;
      }
      if (ishift != 32u && (need == count || count <= kListCap)) {
        const uint64_t key_word = (uint64_t)(low + f.digit) << 32;  // (shift == 0: the digit is the key's offset)
        for_members([&](uint32_t u, uint32_t inv) {
          const uint32_t group = inv >> ishift;
          if (group > iprefix || (group == iprefix && need == count)) {
            before += u < g ? 1u : 0u;  // survives whatever the list says
          } else if (group == iprefix) {
            const uint32_t slot = atomicAdd(&list_count, 1u);
            words[slot] = key_word | (uint64_t)inv;
            ats[slot] = u * kSoloThreads + tid;
          }
        });
        if (need == count) floor_word = key_word | ((uint64_t)iprefix << ishift);
      }
    }
  }
  if constexpr (!TIES) {
    if (cut_digit && f.count > kListCap && tie_lds) {
      // Thousands of candidates of one key around the cut (a ReLU's zeros), in the form that keeps
      // 32 keys per thread and has no registers to spare for the index levels above: the inverted
      // indices of all members (up to the whole row) are listed in LDS, which the launch sized for
      // it, the block-wide radix select of stage2_select.h finds the need-th largest among them,
      // and a second look at the members' indices counts the survivors of the segments before this
      // one.  Every workgroup of the row does all of it.  (shift == 0: the digit is the key's offset.)
      uint32_t* inv_list = reinterpret_cast<uint32_t*>(dyn_lds);
      const uint32_t* ci_low = reinterpret_cast<const uint32_t*>(ci);  // (indices below 2^31: the planner's rule)
      const uint32_t cut_key = low + f.digit;
      // an index's inverted bits, moved to the top of the word: the select's digits start where
      // the indices differ (their leading bits are all alike, and a histogram of one bin is slow)
      const uint32_t up = 32u - (uint32_t)(index_bits < 32 ? index_bits : 32);
      __syncthreads();  // the list's LDS may still be read as `words`
      constexpr int kChunk = 8;
#pragma unroll
      for (int c0 = 0; c0 < NPT; c0 += kChunk) {
        uint32_t iv[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          const uint32_t i = (uint32_t)(c0 + e) * kSoloThreads + tid;
          iv[e] = i < k0 ? ci_low[2u * i] : 0u;
        }
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          const bool member = valid(c0 + e) && key[c0 + e] == cut_key;
          const uint64_t m = __ballot(member);
          uint32_t base = 0;
          if (lane == 0 && m != 0) base = atomicAdd(&list_count, (uint32_t)__popcll(m));
          base = (uint32_t)__builtin_amdgcn_readfirstlane((int)base);
          if (member) inv_list[base + select::rank_in(m)] = ~iv[e] << up;
        }
      }
      // the need-th largest of the listed words (distinct values: no ties among them), by levels
      // of 11 bits over the list, from the top down to the last bit an index has
      uint32_t cut_inv = 0, level = 32, left_need = f.need, left_count = f.count;
      while (level > up) {
        const uint32_t finer = level - up > (uint32_t)regs::kDigitBits ? level - (uint32_t)regs::kDigitBits : up;
        const uint32_t mask = (1u << (level - finer)) - 1u;
        __syncthreads();  // the list is complete; everyone has read `found`, wave 0 the histogram
        for (uint32_t i = tid; i < (uint32_t)regs::kBins; i += kSoloThreads) hist[i] = 0;
        __syncthreads();
        for (uint32_t i = tid; i < f.count; i += kSoloThreads) {
          const uint32_t v = inv_list[i];
          if (level == 32u || (v >> level) == (cut_inv >> level)) atomicAdd(&hist[(v >> finer) & mask], 1u);
        }
        __syncthreads();
        if (wave == 0) {
          const regs::Found f2 = regs::find_bin_wave<false>(hist, left_need, left_count, lane);
          if (lane == 0) found = f2;
        }
        __syncthreads();
        const regs::Found f2 = found;
        cut_inv |= f2.digit << finer;
        left_need = f2.need;
        left_count = f2.count;
        level = finer;
      }
      // members that survive in the segments before this one
#pragma unroll
      for (int c0 = 0; c0 < NPT; c0 += kChunk) {
        uint32_t iv[kChunk];
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          const uint32_t i = (uint32_t)(c0 + e) * kSoloThreads + tid;
          iv[e] = i < k0 ? ci_low[2u * i] : 0u;
        }
#pragma unroll
        for (int e = 0; e < kChunk; ++e) {
          if ((uint32_t)(c0 + e) < g && valid(c0 + e) && key[c0 + e] == cut_key && (~iv[e] << up) >= cut_inv) ++before;
        }
      }
      need = count;  // settled: the members at or above the floor survive, nothing is listed
      floor_word = ((uint64_t)cut_key << 32) | (uint64_t)((cut_inv >> up) | ~(0xffffffffu >> up));
      __syncthreads();  // the list's LDS goes back to `words` (the padding entries below)
      if (tid == 0) list_count = 0;
    }
  }
  if (need != count && count > kListCap) {
    // More than kListCap candidates of one key around the cut (TIES: of one key and
    // one index, which only a caller of the stand-alone select can hand over): the
    // row's first workgroup runs the block-wide radix select of stage2_select.h over
    // all of the row's candidates, read from global memory.
    if (g != 0) return;
    auto key_at = [&](uint32_t i) -> key_t { return E::key(cv[i]); };
    auto index_at = [&](uint32_t i) -> uint64_t { return (uint64_t)ci[i]; };
    // (the key of the k-th best is known by now, shift == 0: the digit is its offset from `low`;
    // f.need of its candidates belong)
    const select::Cut<key_t> whole =
        select::cut_among_ties<key_t>(sh, k0, (key_t)(low + f.digit), f.need, index_bits, key_at, index_at);
    auto survives = [&](uint32_t i) -> bool {
      const key_t kk = key_at(i);
      if (kk != whole.T) return kk > whole.T;
      return whole.index_cut == ~0ull || index_at(i) <= whole.index_cut;
    };
    struct Candidate { raw_t value; int64_t index; };
    raw_t* out_values = values + (int64_t)row * k;
    const int64_t out_first = (int64_t)row * k;
    select::compact(
        sh, k0, k, survives, [&](uint32_t i) { return Candidate{cv[i], ci[i]}; },
        [&](uint32_t, uint32_t o, const Candidate& c) {
          if (values != nullptr) out_values[o] = c.value;
          indices.put(out_first + o, c.index);
        });
    return;
  }
  const uint32_t n = need != count ? count : 0u;  // (== list_count after the barrier)
  if (tid < 8u) {  // entries past the list's end beat nothing (ranking reads it in groups of eight)
    words[n + tid] = 0ull;
    ats[n + tid] = ~0u;
  }
  __syncthreads();
  ATK_TRACE_GROUP(4);
  // This thread's own candidate, asked for together with the listed members'
  // indices: one trip to memory for both.  (Asked for with the keys at the top,
  // the index load made the kernel 5 us slower, measured.)
  const raw_t own_raw = own_valid ? cv[own] : (raw_t)0;
  const uint32_t own_inv = own_valid ? ~(uint32_t)ci[own] : 0u;
  uint64_t cut = floor_word;  // the weakest surviving member of B (0: all of them survive)
  if (n != 0) {
    if (!tie_mode)
      for (uint32_t i = tid; i < n; i += kSoloThreads) words[i] |= (uint64_t)(~(uint32_t)ci[ats[i]]);
    __syncthreads();
    if (n <= kSoloRankDirect) {
      if (tid < n) {  // thread t counts the entries better than entry t: the need-th best is the cut
        const uint64_t mine = words[tid];
        uint32_t better = 0;
        for (uint32_t m = 0; m < n; m += 8) {
          uint64_t got[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) got[e] = words[m + e];
#pragma unroll
          for (int e = 0; e < 8; ++e) better += got[e] > mine ? 1u : 0u;
        }
        if (better + 1 == need) cut_word = mine;
      }
      __syncthreads();
      cut = cut_word;
    } else {  // a longer list: the block-wide radix select over its words (all distinct)
      auto key_at = [&](uint32_t i) -> uint64_t { return words[i]; };
      auto index_at = [&](uint32_t) -> uint64_t { return 0; };
      cut = select::find_cut<uint64_t, 64>(sh, n, need, 1, key_at, index_at).T;
    }
    for (uint32_t i = tid; i < n; i += kSoloThreads) before += (ats[i] < g * kSoloThreads && words[i] >= cut) ? 1u : 0u;
  }
  ATK_TRACE_GROUP(5);
  // this thread's own candidate
  const uint32_t own_d = (own_key - low) >> shift;
  const bool sel = own_valid && (own_d > f.digit ||
                                 (own_d == f.digit && (((uint64_t)own_key << 32) | own_inv) >= cut));
  const uint64_t m = __ballot(sel);
  before = regs::wave_scan(before);
  if (lane == select::kWave - 1) wave_before[wave] = before;
  if (lane == 0) wave_kept[wave] = (uint32_t)__popcll(m);
  __syncthreads();
  uint32_t at = 0;
#pragma unroll
  for (int w = 0; w < kSoloWaves; ++w) {
    at += wave_before[w];
    if ((uint32_t)w < wave) at += wave_kept[w];
  }
  if (sel) {
    at += select::rank_in(m);
    if (at < k) {
      if (values != nullptr) values[(int64_t)row * k + at] = own_raw;
      indices.put((int64_t)row * k + at, (int64_t)(uint32_t)~own_inv);
    }
  }
  ATK_TRACE_GROUP(6);
}

// Rows the one-launch form takes: short enough for the keys to sit in registers,
// and few enough that all workgroups run at once, one per CU (a second round
// doubles the time: 16 rows of 32768 fp16 candidates took 32.6 us in 512
// workgroups, 8 rows 18.4 us in 256).
// (With 64 keys per thread the kernel spills: rows of 40000-65536 candidates took
// 28-30 us against 18 us for the chain of launches.)
constexpr int64_t kSoloMaxCandidates = 32 * kSoloThreads;
constexpr int64_t kSoloMaxWorkgroups = 256;

// Rows for which the chain beats one workgroup per row: few rows (one workgroup
// per row already fills the GPU with many), enough candidates that a single CU
// is what bounds them, keys of at most 32 bits and indices below 2^31.  Measured,
// select alone, microseconds, fp16 / fp32, chain against one workgroup per row:
// 16 rows of 16384: 14.6 / 18.9 against 16.3 / 18.3; 32 rows of 16384: 21.7 / 35.2;
// 17-32 rows of 32768: 29 / 38 against 23 / 26; 16 rows of 65536: 34 / 33 against
// 70 / 73; 64 rows of 49152: 43 / 46 against 54 / 58, 96 rows 59 / 62 against 56 / 72;
// 64 rows of 65536: 49 / 53 against 72 / 74, 96 rows 79 / 84 against 74 / 75;
// 64 rows of 131072: 99 / 110 against 107 / 118, 96 rows 141 / 162 against 142 / 173.
// Segments of 4096 candidates from 1024 workgroups of the short ones on: 32 rows of
// 131072 took 120 / 127 us with segments of 1024, 33 rows 65 / 71 us with 4096.
constexpr int64_t kChainMinCandidates = 10240;  // (8192: 11.8 us against 10.5 for one workgroup)
constexpr int64_t kChainMaxCandidates = 1 << 17;
constexpr int64_t kChainMaxRows = 16;
constexpr int64_t kChainMaxRowsLong = 64;  // rows of more than kSoloMaxCandidates candidates
constexpr int64_t kChainShortSegmentGroups = 1024;

ChainPlan plan_chain(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype) {
  ChainPlan pl{};
  pl.use = false;
  const int es = elem_bytes(dtype);
  if (es == 0 || es > 4 || rows <= 0 || k <= 0 || k >= k0) return pl;
  if (k0 < kChainMinCandidates || k0 > kChainMaxCandidates || index_bound > 0x7fffffffll) return pl;
  if (rows > (k0 > kSoloMaxCandidates ? kChainMaxRowsLong : kChainMaxRows)) return pl;
  pl.groups = (uint32_t)((k0 + kSoloSegment - 1) / kSoloSegment);
  pl.per_thread = rows * (int64_t)pl.groups > kChainShortSegmentGroups ? kPerThreadMany : kPerThreadFew;
  pl.solo = k0 <= kSoloMaxCandidates && rows * (int64_t)pl.groups <= kSoloMaxWorkgroups;
  if (!pl.solo) {
    const int64_t segment = (int64_t)kThreads * pl.per_thread;
    pl.groups = (uint32_t)((k0 + segment - 1) / segment);
  }
  pl.range_off = 0;
  pl.range_capacity = pl.groups > kRangeCapacity ? pl.groups : kRangeCapacity;
  pl.hist_off = align_up((size_t)rows * pl.range_capacity * sizeof(uint2), 256);
  pl.state_off = pl.hist_off + align_up((size_t)rows * regs::kHistWords * sizeof(uint32_t), 256);
  pl.above_off = pl.state_off + align_up((size_t)rows * sizeof(RowState), 256);
  pl.list_word_off = pl.above_off + align_up((size_t)rows * pl.groups * sizeof(uint32_t), 256);
  // the row's list takes every candidate of the row (all may share the cut digit); the
  // one-launch form keeps its list in LDS
  const size_t listed = pl.solo ? 0 : (size_t)rows * (size_t)k0;
  pl.list_at_off = pl.list_word_off + align_up(listed * sizeof(uint64_t), 256);
  pl.total = pl.list_at_off + align_up(listed * sizeof(uint32_t), 256);
  pl.use = true;
  return pl;
}

template <typename E>
int launch_chain_typed(const ChainPlan& pl, const void* cand_values, const int64_t* cand_indices, int64_t rows,
                       int64_t k0, int64_t k, int index_bits, void* values, IndexOut indices, void* ws,
                       uint32_t range_entries, bool hist_done, hipStream_t stream) {
  using raw_t = typename E::raw_t;
  if constexpr (sizeof(typename E::key_t) == 4) {
    unsigned char* base = static_cast<unsigned char*>(ws);
    uint2* range = reinterpret_cast<uint2*>(base + pl.range_off);
    uint32_t* hist = reinterpret_cast<uint32_t*>(base + pl.hist_off);
    RowState* state = reinterpret_cast<RowState*>(base + pl.state_off);
    uint32_t* above = reinterpret_cast<uint32_t*>(base + pl.above_off);
    uint64_t* list_word = reinterpret_cast<uint64_t*>(base + pl.list_word_off);
    uint32_t* list_at = reinterpret_cast<uint32_t*>(base + pl.list_at_off);
    const raw_t* cv = static_cast<const raw_t*>(cand_values);
    const dim3 grid((unsigned)(rows * pl.groups)), block(kThreads);
    const size_t emit_lds = (size_t)kListCap * (sizeof(uint64_t) + sizeof(uint32_t));
    uint32_t entries = range_entries;
    const bool own_ranges = entries == 0 && !pl.solo;  // stage 1 left no key ranges
    if (own_ranges) entries = pl.groups;
    if (pl.solo) {
      size_t solo_lds = (size_t)(kListCap + 8) * (sizeof(uint64_t) + sizeof(uint32_t));
      // The form with 32 keys per thread of a 2- or 4-byte type lists the inverted indices of a
      // tied row's members in LDS: room for the whole row (up to 128 KiB; one workgroup per CU
      // is all that runs of this kernel anyway).
      uint32_t tie_lds = 0;
      if (sizeof(raw_t) > 1 && k0 > 16 * kSoloThreads) {
        const size_t tie_bytes = (size_t)k0 * sizeof(uint32_t);
        if (solo_lds < tie_bytes) solo_lds = tie_bytes;
        tie_lds = 1;
      }
      const dim3 solo_block(kSoloThreads);
      raw_t* out = static_cast<raw_t*>(values);
#define ATK_SOLO(NPT, OWN)                                                                                       \
  {                                                                                                              \
    constexpr bool kTies = sizeof(raw_t) == 1 || NPT <= 16;                                                      \
    auto kern = chain_solo_kernel<E, NPT, OWN>;                                                                  \
    if (k0 == (int64_t)NPT * kSoloThreads) kern = chain_solo_kernel<E, NPT, OWN, kTies, true>;                    \
    if (solo_lds > 48 * 1024 &&                                                                                  \
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,     \
                            (int)solo_lds) != hipSuccess)                                                        \
      return ATK_ERR_LAUNCH;                                                                                     \
    hipLaunchKernelGGL(kern, grid, solo_block, solo_lds, stream, cv, cand_indices, (uint32_t)k0, (uint32_t)k,    \
                       pl.groups, index_bits, (const uint2*)range, entries, out, indices, tie_lds);              \
  }
      if (entries != 0) {
        if (k0 <= 8 * kSoloThreads) ATK_SOLO(8, false)
        else if (k0 <= 16 * kSoloThreads) ATK_SOLO(16, false)
        else ATK_SOLO(32, false)
      } else {
        if (k0 <= 8 * kSoloThreads) ATK_SOLO(8, true)
        else if (k0 <= 16 * kSoloThreads) ATK_SOLO(16, true)
        else ATK_SOLO(32, true)
      }
#undef ATK_SOLO
      return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
    }
#define ATK_CHAIN(PT)                                                                                              \
  {                                                                                                                \
    if (own_ranges)                                                                                                \
      hipLaunchKernelGGL((chain_range_kernel<E, PT>), grid, block, 0, stream, cv, (uint32_t)k0, pl.groups, range,  \
                         hist, state);                                                                             \
    if (!hist_done || range_entries == 0)                                                                          \
      hipLaunchKernelGGL((chain_hist_kernel<E, PT>), grid, block, 0, stream, cv, (uint32_t)k0, pl.groups,          \
                         (const uint2*)range, entries, hist);                                                      \
    hipLaunchKernelGGL((chain_refine_kernel<E, PT>), grid, block, 0, stream, cv, cand_indices, (uint32_t)k0,       \
                       (uint32_t)k, pl.groups, (const uint2*)range, entries, (const uint32_t*)hist, state, above,  \
                       list_word, list_at);                                                                        \
    hipLaunchKernelGGL((chain_emit_kernel<E, PT>), grid, block, emit_lds, stream, cv, cand_indices, (uint32_t)k0,  \
                       (uint32_t)k, pl.groups, index_bits, (const RowState*)state, (const uint32_t*)above,         \
                       (const uint64_t*)list_word, (const uint32_t*)list_at, static_cast<raw_t*>(values),          \
                       indices);                                                                                   \
  }
    if (pl.per_thread == kPerThreadMany) ATK_CHAIN(kPerThreadMany) else ATK_CHAIN(kPerThreadFew)
#undef ATK_CHAIN
    return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
  } else {
    (void)pl; (void)cand_values; (void)cand_indices; (void)rows; (void)k0; (void)k; (void)index_bits; (void)values;
    (void)indices; (void)ws; (void)range_entries; (void)hist_done; (void)stream;
    return ATK_ERR_DTYPE;
  }
}

}  // namespace

size_t chain_select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype) {
  const ChainPlan pl = plan_chain(rows, k0, k, index_bound, dtype);
  return pl.use ? pl.total : 0;
}

bool describe_chain_select(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, std::string& out) {
  const ChainPlan pl = plan_chain(rows, k0, k, index_bound, dtype);
  if (!pl.use) return false;
  const std::string t = dtype_name(dtype);
  if (pl.solo) {
    out += "chain_solo_kernel<" + t + "> grid=" +
           std::to_string(rows * (int64_t)pl.groups) + " block=" + std::to_string(kSoloThreads);
    return true;
  }
  out += "[chain_range_kernel<" + t + "> + chain_hist_kernel<" + t +
         "> unless stage 1 left key ranges and histogram] + chain_refine_kernel<" + t +
         "> + chain_emit_kernel<" + t + "> grid=" + std::to_string(rows * (int64_t)pl.groups) + " block=" +
         std::to_string(kThreads) + " per_thread=" + std::to_string(pl.per_thread);
  return true;
}

KeyRangeOut chain_select_ranges(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, void* ws,
                                size_t ws_bytes) {
  KeyRangeOut out{};
  const ChainPlan pl = plan_chain(rows, k0, k, index_bound, dtype);
  if (!pl.use || !ws || ws_bytes < pl.total || (uintptr_t)ws % 16 != 0) return out;
  unsigned char* base = static_cast<unsigned char*>(ws);
  out.range = reinterpret_cast<uint2*>(base + pl.range_off);
  out.capacity = pl.range_capacity;
  out.hist = reinterpret_cast<uint32_t*>(base + pl.hist_off);
  out.hist_words = regs::kHistWords;
  out.state = reinterpret_cast<uint32_t*>(base + pl.state_off);
  out.state_words = (uint32_t)(sizeof(RowState) / sizeof(uint32_t));
  out.want_hist = pl.solo ? 0u : 1u;
  return out;
}

int launch_chain_select(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0, int64_t k,
                        int64_t index_bound, int dtype, void* values, IndexOut indices, void* ws, size_t ws_bytes,
                        uint32_t range_entries, bool hist_done, hipStream_t stream, bool* handled) {
  const ChainPlan pl = plan_chain(rows, k0, k, index_bound, dtype);
  *handled = pl.use;
  if (!pl.use) return ATK_OK;
  if (!ws || ws_bytes < pl.total || (uintptr_t)ws % 16 != 0) return ATK_ERR_WORKSPACE;
  int index_bits = 1;
  while (index_bits < 63 && (1ll << index_bits) < index_bound) ++index_bits;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = launch_chain_typed<E>(pl, cand_values, cand_indices, rows, k0, k, index_bits, values, indices,
                                              ws, range_entries, hist_done, stream));
  return rc;
}

}  // namespace atk

ATK_TRACE_READER(atk_trace_stage2_chain_select)  // (nothing, unless the library is built for the phase timelines)
