// Stage 2 for rows with very many candidates: the exact top-k selection of
// stage2_select.h spread over many workgroups per row.
//
// One workgroup per row reads its candidates through a single CU, which is
// what bounds it once a row holds more than a few tens of thousands of
// candidates.  Here every row is cut into segments, one workgroup each, and
// the MSB-first radix select runs as a chain of launches, one per 11-bit digit:
//
//   pass p:   every workgroup first advances the selection state by the
//             histogram of pass p-1 (all of a row's workgroups compute the same
//             state from the same global histogram; the row's first workgroup
//             also stores it for pass p+1), then adds the digit-p histogram of
//             its segment's participating candidates to the row's global
//             histogram of pass p.
//   count:    advances by the last histogram, stores the cut (the key T of the
//             k-th best and the largest index taken among the candidates with
//             key == T) and counts the survivors of each segment.
//   emit:     every workgroup offsets by the survivors of the segments before
//             it and writes its own in candidate order.
//
// Value digits come first; then, only if the group of candidates with key == T
// is cut, the digits of the candidates' original indices, so that the lowest
// indices win.  The index passes are launched either way (the host cannot know)
// and return at once when there is nothing to cut.  Results are those of the
// one-workgroup kernel: same survivors, same order.
#include "atk_device.h"
#include "atk_launch.h"
#include "stage2_select.h"

namespace atk {
namespace {

constexpr int kThreads = 256;
constexpr int kWave = 64;
constexpr int kWaves = kThreads / kWave;
constexpr int kDigitBits = 11;
constexpr int kBins = 1 << kDigitBits;
constexpr int kMaxIndexDigits = 6;  // 63 bits

// Digits of a `bits`-wide number, most significant first: the first takes what
// the others (11 bits each) leave.
__host__ __device__ inline int digit_count(int bits) { return (bits + kDigitBits - 1) / kDigitBits; }
__host__ __device__ inline int digit_shift(int count, int d) { return kDigitBits * (count - 1 - d); }
__host__ __device__ inline int digit_width(int bits, int count, int d) {
  return d == 0 ? bits - kDigitBits * (count - 1) : kDigitBits;
}

// Where the selection of one row stands before a pass.
struct State {
  uint64_t key;       // value digits chosen so far; after the value passes, the key T of the k-th best
  uint64_t index;     // index digits chosen so far
  uint32_t need;      // members of the current group that belong to the result
  uint32_t group;     // candidates that match every digit chosen so far
  uint32_t idigits;   // index digits chosen so far
  uint32_t unused;
};

using Cut = select::GlobalCut;

struct Passes {
  int key_bits, index_bits;
  int vc, ic;  // value and index digits
};

// State after pass q, from the state before it and the row's histogram of it.
// Called by the whole workgroup; `lh` is kBins words of LDS.
__device__ State advance(const State& before, const uint32_t* __restrict__ hist, int q, const Passes& ps,
                         uint32_t* lh) {
  const bool value_pass = q < ps.vc;
  // asked for before `before` is looked at, which may still be on its way from memory
  uint32_t mine[kBins / kThreads];
#pragma unroll
  for (int e = 0; e < kBins / kThreads; ++e) mine[e] = hist[e * kThreads + threadIdx.x];
  if (!value_pass && before.need == before.group) return before;  // nothing left to cut
  __shared__ State result;
#pragma unroll
  for (int e = 0; e < kBins / kThreads; ++e) lh[e * kThreads + threadIdx.x] = mine[e];
  __syncthreads();
  if (threadIdx.x < kWave) {
    // value digits are searched from the top (largest keys first), index digits from the bottom
    constexpr int kPer = kBins / kWave;
    const uint32_t lane = threadIdx.x;
    auto bin_at = [&](uint32_t r) -> uint32_t { return value_pass ? (uint32_t)kBins - 1 - r : r; };
    uint32_t part = 0;
    for (int e = 0; e < kPer; ++e) part += lh[bin_at(lane * kPer + e)];
    uint32_t incl = part;
    for (int d = 1; d < kWave; d *= 2) {
      const uint32_t up = __shfl_up(incl, d);
      if (lane >= (uint32_t)d) incl += up;
    }
    const uint32_t ahead = incl - part;
    if (ahead < before.need && before.need <= incl) {  // exactly one lane
      uint32_t run = ahead, bin = 0, count = 0;
      for (int e = 0; e < kPer; ++e) {
        bin = bin_at(lane * kPer + e);
        count = lh[bin];
        if (run + count >= before.need) break;
        run += count;
      }
      State after = before;
      after.need = before.need - run;
      after.group = count;
      if (value_pass) {
        after.key = (before.key << digit_width(ps.key_bits, ps.vc, q)) | bin;
      } else {
        after.index = (before.index << digit_width(ps.index_bits, ps.ic, q - ps.vc)) | bin;
        after.idigits = before.idigits + 1;
      }
      result = after;
    }
  }
  __syncthreads();
  const State after = result;
  __syncthreads();  // `result` and `lh` may be rewritten
  return after;
}

__device__ __forceinline__ State initial_state(uint32_t k0, uint32_t k) { return State{0, 0, k, k0, 0, 0}; }

// State before pass p (p >= 0), which the row's first workgroup also records.
__device__ State state_before(int p, int64_t row, int64_t rows, uint32_t k0, uint32_t k, bool record,
                              const Passes& ps, const uint32_t* __restrict__ hist, State* states, uint32_t* lh) {
  if (p == 0) return initial_state(k0, k);
  const State prev = p == 1 ? initial_state(k0, k) : states[(int64_t)(p - 1) * rows + row];
  const State now = advance(prev, hist + ((int64_t)(p - 1) * rows + row) * kBins, p - 1, ps, lh);
  if (record && threadIdx.x == 0) states[(int64_t)p * rows + row] = now;
  return now;
}

__global__ __launch_bounds__(kThreads) void ms_zero_kernel(uint32_t* words, size_t count) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < count) words[i] = 0;
}

// Candidates a thread loads ahead of testing them: the loop below is bound by
// the latency of its loads, not by their number.
constexpr int kBatch = 8;

template <typename E>
__global__ __launch_bounds__(kThreads) void ms_pass_kernel(
    const typename E::raw_t* __restrict__ cand_values, const int64_t* __restrict__ cand_indices, uint32_t k0,
    uint32_t k, uint32_t seg, uint32_t groups, int p, const Passes ps, uint32_t* __restrict__ hist,
    State* states) {
  using raw_t = typename E::raw_t;
  __shared__ uint32_t lh[kBins];
  const int64_t rows = gridDim.x / groups;
  const int64_t row = blockIdx.x / groups;
  const uint32_t g = blockIdx.x - (uint32_t)row * groups;
  const raw_t* cv = cand_values + row * (int64_t)k0;
  const int64_t* ci = cand_indices + row * (int64_t)k0;
  const uint32_t lo = g * seg < k0 ? g * seg : k0, hi = lo + seg < k0 ? lo + seg : k0;
  // the first batch is on its way while the state is worked out
  auto load = [&](uint32_t base, raw_t (&into)[kBatch]) {
#pragma unroll
    for (int e = 0; e < kBatch; ++e) {
      const uint32_t i = base + e * kThreads + threadIdx.x;
      into[e] = cv[i < hi ? i : lo < k0 ? lo : 0];
    }
  };
  raw_t ahead[kBatch];
  load(lo, ahead);

  const State st = state_before(p, row, rows, k0, k, g == 0, ps, hist, states, lh);
  const bool value_pass = p < ps.vc;
  if (!value_pass && st.need == st.group) return;

  for (uint32_t bin = threadIdx.x; bin < kBins; bin += kThreads) lh[bin] = 0;
  __syncthreads();
  const int d = value_pass ? p : p - ps.vc;
  const int shift = value_pass ? digit_shift(ps.vc, d) : digit_shift(ps.ic, d);
  const int width = value_pass ? digit_width(ps.key_bits, ps.vc, d) : digit_width(ps.index_bits, ps.ic, d);
  const uint32_t mask = (1u << width) - 1u;
  const uint64_t prefix = value_pass ? st.key : st.index;
  const uint32_t lane = threadIdx.x % kWave;
  constexpr uint32_t kStep = kBatch * kThreads;
  for (uint32_t base = lo; base < hi; base += kStep) {  // the same trips for every thread of a wave
    raw_t now[kBatch];
#pragma unroll
    for (int e = 0; e < kBatch; ++e) now[e] = ahead[e];
    if (base + kStep < hi) load(base + kStep, ahead);
    // the number the digit is taken from: the key, or the index of a candidate with key == T
    uint64_t from[kBatch];
    bool ok[kBatch];
#pragma unroll
    for (int e = 0; e < kBatch; ++e) {
      const uint32_t i = base + e * kThreads + threadIdx.x;
      const uint64_t key = E::key(now[e]);
      ok[e] = i < hi && (value_pass || key == st.key);
      from[e] = value_pass ? key : (ok[e] ? (uint64_t)ci[i] : 0ull);
    }
#pragma unroll
    for (int e = 0; e < kBatch; ++e) {
      const bool in = ok[e] && (d == 0 || (from[e] >> (shift + width)) == prefix);
      const uint32_t digit = (uint32_t)(from[e] >> shift) & mask;
      // the leading digits of neighbouring candidates are mostly equal: count
      // the lanes that share the first lane's digit with one atomic
      const uint64_t live = __ballot(in);
      if (live != 0) {
        const int first = __ffsll((unsigned long long)live) - 1;
        const uint32_t lead = __shfl(digit, first);
        const uint64_t same = __ballot(in && digit == lead);
        if (lane == (uint32_t)first) atomicAdd(&lh[lead], (uint32_t)__popcll(same));
        if (in && digit != lead) atomicAdd(&lh[digit], 1u);
      }
    }
  }
  __syncthreads();
  uint32_t* gh = hist + ((int64_t)p * rows + row) * kBins;
  for (uint32_t bin = threadIdx.x; bin < kBins; bin += kThreads) {
    const uint32_t count = lh[bin];
    if (count != 0) atomicAdd(&gh[bin], count);
  }
}

template <typename E>
__device__ __forceinline__ bool survives(const Cut& cut, typename E::raw_t value, const int64_t* index_at) {
  const uint64_t key = E::key(value);
  if (key != cut.key) return key > cut.key;
  return (uint64_t)*index_at <= cut.index;
}

template <typename E>
__global__ __launch_bounds__(kThreads) void ms_count_kernel(
    const typename E::raw_t* __restrict__ cand_values, const int64_t* __restrict__ cand_indices, uint32_t k0,
    uint32_t k, uint32_t seg, uint32_t groups, const Passes ps, const uint32_t* __restrict__ hist,
    State* states, Cut* cuts, uint32_t* __restrict__ counts) {
  __shared__ uint32_t lh[kBins];
  __shared__ uint32_t wave_total[kWaves];
  const int64_t rows = gridDim.x / groups;
  const int64_t row = blockIdx.x / groups;
  const uint32_t g = blockIdx.x - (uint32_t)row * groups;
  const State st = state_before(ps.vc + ps.ic, row, rows, k0, k, false, ps, hist, states, lh);
  // the whole current group is taken: every index that starts with the chosen digits
  const int open = st.idigits == 0 ? ps.index_bits : digit_shift(ps.ic, (int)st.idigits - 1);
  Cut cut;
  cut.key = st.key;
  cut.index = open >= 64 ? ~0ull : ((st.index << open) | ((1ull << open) - 1ull));
  if (g == 0 && threadIdx.x == 0) cuts[row] = cut;

  const typename E::raw_t* cv = cand_values + row * (int64_t)k0;
  const int64_t* ci = cand_indices + row * (int64_t)k0;
  const uint32_t lo = g * seg, hi = lo + seg < k0 ? lo + seg : k0;
  uint32_t mine = 0;
  for (uint32_t i = lo + threadIdx.x; i < hi; i += kThreads) mine += survives<E>(cut, cv[i], ci + i) ? 1u : 0u;
  for (int d = kWave / 2; d >= 1; d /= 2) mine += __shfl_down(mine, d);
  if (threadIdx.x % kWave == 0) wave_total[threadIdx.x / kWave] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t total = 0;
    for (int w = 0; w < kWaves; ++w) total += wave_total[w];
    counts[row * groups + g] = total;
  }
}

template <typename raw_t> struct Candidate { raw_t value; int64_t index; };
struct WaveTotals { uint32_t wave_total[select::kMaxWaves]; };

template <typename E>
__global__ __launch_bounds__(kThreads) void ms_emit_kernel(
    const typename E::raw_t* __restrict__ cand_values, const int64_t* __restrict__ cand_indices, uint32_t k0,
    uint32_t k, uint32_t seg, uint32_t groups, const Cut* __restrict__ cuts,
    const uint32_t* __restrict__ counts, typename E::raw_t* __restrict__ values,
    const IndexOut indices) {
  using raw_t = typename E::raw_t;
  __shared__ WaveTotals totals;
  __shared__ uint32_t start;
  const int64_t row = blockIdx.x / groups;
  const uint32_t g = blockIdx.x - (uint32_t)row * groups;
  const Cut cut = cuts[row];
  // survivors of the segments before this one
  uint32_t ahead = 0;
  for (uint32_t s = threadIdx.x; s < g; s += kThreads) ahead += counts[row * groups + s];
  for (int d = kWave / 2; d >= 1; d /= 2) ahead += __shfl_down(ahead, d);
  if (threadIdx.x % kWave == 0) totals.wave_total[threadIdx.x / kWave] = ahead;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t total = 0;
    for (int w = 0; w < kWaves; ++w) total += totals.wave_total[w];
    start = total;
  }
  __syncthreads();
  const uint32_t first = start;

  const uint32_t lo = g * seg < k0 ? g * seg : k0, hi = lo + seg < k0 ? lo + seg : k0;
  const raw_t* cv = cand_values + row * (int64_t)k0 + lo;
  const int64_t* ci = cand_indices + row * (int64_t)k0 + lo;
  raw_t* ov = values + row * (int64_t)k;
  const int64_t oi = row * (int64_t)k;  // this row's first output slot
  // the segment's survivors in candidate order, behind those of the segments before
  select::compact(
      totals, hi - lo, k,
      [&](uint32_t i) -> bool { return survives<E>(cut, cv[i], ci + i); },
      [&](uint32_t i) { return Candidate<raw_t>{cv[i], ci[i]}; },
      [&](uint32_t, uint32_t o, const Candidate<raw_t>& c) {
        if (first + o < k) {  // always true for consistent inputs; keeps a wrong cut from writing out of bounds
          if (values != nullptr) ov[first + o] = c.value;
          indices.put(oi + first + o, c.index);
        }
      });
}

struct MultiPlan {
  bool use;
  uint32_t groups, seg;
  int vc;
  size_t hist_words;  // with the most index digits
  size_t states_off, cuts_off, counts_off, total;
};

// The multi-workgroup select is taken when it is expected to be the faster one.
// Measured on an MI355X (fp32 and fp16, k = k0/4, 1 to 256 rows of 64K to 4M
// candidates): the chain of launches costs about 45 us plus 9.3 us per million
// candidates of the whole batch; one workgroup per row is bound by what one CU
// can read, 0.75 to 1 us per thousand candidates of a row, and slows down
// further once more than 16 rows run side by side.  The two meet at about one
// row per 1500 candidates of a row.  Rows of up to 48K candidates always stay
// with one workgroup (its keys then sit in LDS).
constexpr int64_t kMultiMinCandidates = 49152;
constexpr int64_t kMultiCandidatesPerRow = 1500;

bool multi_is_faster(int64_t rows, int64_t k0) { return rows * kMultiCandidatesPerRow <= k0; }

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int key_bits_of(int dtype) {
  int bits = 0;
  ATK_DTYPE_SWITCH(dtype, E, bits = 0, bits = E::key_bits);
  return bits;
}

MultiPlan plan_multi(int64_t rows, int64_t k0, int64_t k, int dtype) {
  MultiPlan pl{};
  pl.use = false;
  const int bits = key_bits_of(dtype);
  if (!bits || rows <= 0 || k0 <= kMultiMinCandidates || !multi_is_faster(rows, k0) || k <= 0 || k >= k0 || k0 > 0xfffffff0ll) return pl;
  int64_t groups = (k0 + 4095) / 4096;
  const int64_t most = rows >= 2048 ? 1 : 2048 / rows;
  if (groups > most) groups = most;
  int64_t seg = (k0 + groups - 1) / groups;
  seg = (seg + kThreads - 1) / kThreads * kThreads;
  groups = (k0 + seg - 1) / seg;
  if (rows * groups > 0x7fffffffll) return pl;
  pl.groups = (uint32_t)groups;
  pl.seg = (uint32_t)seg;
  pl.vc = digit_count(bits);
  const int passes = pl.vc + kMaxIndexDigits;
  pl.hist_words = (size_t)passes * (size_t)rows * kBins;
  pl.states_off = align_up(pl.hist_words * sizeof(uint32_t), 256);
  pl.cuts_off = pl.states_off + align_up((size_t)(passes + 1) * (size_t)rows * sizeof(State), 256);
  pl.counts_off = pl.cuts_off + align_up((size_t)rows * sizeof(Cut), 256);
  pl.total = pl.counts_off + align_up((size_t)rows * (size_t)groups * sizeof(uint32_t), 256);
  pl.use = true;
  return pl;
}

template <typename E>
int launch_multi_typed(const MultiPlan& pl, const void* cand_values, const int64_t* cand_indices, int64_t rows,
                       int64_t k0, int64_t k, int index_bits, void* values, IndexOut indices, void* ws,
                       hipStream_t stream) {
  using raw_t = typename E::raw_t;
  unsigned char* base = static_cast<unsigned char*>(ws);
  uint32_t* hist = reinterpret_cast<uint32_t*>(base);
  State* states = reinterpret_cast<State*>(base + pl.states_off);
  Cut* cuts = reinterpret_cast<Cut*>(base + pl.cuts_off);
  uint32_t* counts = reinterpret_cast<uint32_t*>(base + pl.counts_off);
  Passes ps;
  ps.key_bits = E::key_bits;
  ps.index_bits = index_bits;
  ps.vc = pl.vc;
  ps.ic = digit_count(index_bits);
  const int passes = ps.vc + ps.ic;
  const size_t words = (size_t)passes * (size_t)rows * kBins;
  const dim3 grid((unsigned)(rows * pl.groups)), block(kThreads);
  const raw_t* cv = static_cast<const raw_t*>(cand_values);
  // a fill kernel rather than a memset node, so that the chain can be captured in a graph
  hipLaunchKernelGGL(ms_zero_kernel, dim3((unsigned)((words + kThreads - 1) / kThreads)), block, 0, stream, hist,
                     words);
  for (int p = 0; p < passes; ++p)
    hipLaunchKernelGGL((ms_pass_kernel<E>), grid, block, 0, stream, cv, cand_indices, (uint32_t)k0, (uint32_t)k,
                       pl.seg, pl.groups, p, ps, hist, states);
  hipLaunchKernelGGL((ms_count_kernel<E>), grid, block, 0, stream, cv, cand_indices, (uint32_t)k0, (uint32_t)k,
                     pl.seg, pl.groups, ps, (const uint32_t*)hist, states, cuts, counts);
  hipLaunchKernelGGL((ms_emit_kernel<E>), grid, block, 0, stream, cv, cand_indices, (uint32_t)k0, (uint32_t)k,
                     pl.seg, pl.groups, (const Cut*)cuts, (const uint32_t*)counts, static_cast<raw_t*>(values),
                     indices);
  return hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
}

}  // namespace

int launch_emit_segments(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0,
                         int64_t k, uint32_t seg, uint32_t groups, const void* cuts, const uint32_t* counts,
                         int dtype, void* values, IndexOut indices, hipStream_t stream) {
  if (rows * (int64_t)groups > 0x7fffffffll) return ATK_ERR_TOO_LARGE;
  const dim3 grid((unsigned)(rows * groups)), block(kThreads);
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE, {
    using raw_t = typename E::raw_t;
    hipLaunchKernelGGL((ms_emit_kernel<E>), grid, block, 0, stream, static_cast<const raw_t*>(cand_values),
                       cand_indices, (uint32_t)k0, (uint32_t)k, seg, groups, static_cast<const Cut*>(cuts), counts,
                       static_cast<raw_t*>(values), indices);
    rc = hipGetLastError() == hipSuccess ? ATK_OK : ATK_ERR_LAUNCH;
  });
  return rc;
}

bool describe_multi_select(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, std::string& out) {
  const MultiPlan pl = plan_multi(rows, k0, k, dtype);
  if (!pl.use) return false;
  int index_bits = 1;
  while (index_bits < 63 && (1ll << index_bits) < index_bound) ++index_bits;
  const int passes = pl.vc + digit_count(index_bits);
  const std::string t = dtype_name(dtype);
  out += "ms_zero_kernel + " + std::to_string(passes) + " x ms_pass_kernel<" + t + "> + ms_count_kernel<" + t +
         "> + ms_emit_kernel<" + t + "> grid=" + std::to_string(rows * (int64_t)pl.groups) + " block=" +
         std::to_string(kThreads);
  return true;
}

size_t multi_select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int dtype) {
  const MultiPlan pl = plan_multi(rows, k0, k, dtype);
  return pl.use ? pl.total : 0;
}

int launch_multi_select(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0,
                        int64_t k, int64_t index_bound, int dtype, void* values, IndexOut indices, void* ws,
                        size_t ws_bytes, hipStream_t stream, bool* handled) {
  const MultiPlan pl = plan_multi(rows, k0, k, dtype);
  *handled = pl.use;
  if (!pl.use) return ATK_OK;
  if (!ws || ws_bytes < pl.total || (uintptr_t)ws % 16 != 0) return ATK_ERR_WORKSPACE;
  int index_bits = 1;
  while (index_bits < 63 && (1ll << index_bits) < index_bound) ++index_bits;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = launch_multi_typed<E>(pl, cand_values, cand_indices, rows, k0, k, index_bits, values,
                                              indices, ws, stream));
  return rc;
}

}  // namespace atk
