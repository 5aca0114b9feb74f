// Both stages in one kernel, one workgroup per row.
//
// For batches of many moderate rows (a row's candidates fit in LDS) the
// candidates never travel to HBM: the workgroup streams its row through the
// same register queues as the streaming stage-1 kernel (stage1_stream.h),
// parks the k0 candidates (order key + sub-row number) in LDS, runs the
// block-wide radix select of stage2_select.h over them and writes only the k
// survivors, whose values it works out from their keys (a zero or a NaN is
// read from the row, still in L2, so that outputs are the input's bit
// patterns).  HBM traffic is the input once plus the final
// k values and indices per row; the two-kernel path additionally writes and
// re-reads k0 * (sizeof(T) + 8) bytes per row.
//
// Work split inside the workgroup: the row's T column tiles (64*V columns each)
// are shared out over the waves; with few tiles, `split` waves share a tile,
// each scanning 1/split of the sub-rows, and fold through LDS as in the
// streaming kernel.  Results are identical to atk_stage1 followed by
// atk_select: same candidates in the same positions, same cut, same order.
#pragma once

#include "stage1_stream.h"
#include "stage2_select.h"
#include "atk_trace.h"

namespace atk {
namespace fused {

using stream::Cmp;
using stream::Geom;
using stream::kWave;

// A value the fast queues cannot order (NaN) was loaded somewhere in the row:
// stage 1 again with exact order keys, one thread per column, into the
// candidate arrays in LDS.  All threads of the workgroup call this.
// CONTIG: bucket c is the run of g.full_rows adjacent elements from c * g.full_rows
// on (no partial sub-row), not column c of the [full_rows][b] matrix.
template <typename E, int J, bool CONTIG, typename skey_t, typename pos_t>
__device__ __forceinline__ void redo_exact_into_lds(const typename E::raw_t* __restrict__ xr, const Geom& g,
                                                    skey_t* cand_key, pos_t* cand_pos) {
  using raw_t = typename E::raw_t;
  for (int64_t c = threadIdx.x; c < g.b; c += blockDim.x) {
    raw_t qv[J];
    uint32_t qp[J];
    stream::clear_exact<E, J>(qv, qp);
    for (uint32_t p = 0; p < g.full_rows; ++p)
      stream::push_exact<E, J>(qv, qp, xr[CONTIG ? c * (int64_t)g.full_rows + p : (int64_t)p * g.b + c], p);
    if (!CONTIG && g.rem != 0) {
      if (c < (int64_t)g.rem)
        stream::push_exact<E, J>(qv, qp, xr[(int64_t)g.full_rows * g.b + c], g.full_rows);
      else if (g.pad_tail)
        stream::push_exact<E, J>(qv, qp, E::pad_raw, g.full_rows);
    }
#pragma unroll
    for (int s = 0; s < J; ++s) { cand_key[c * J + s] = (skey_t)E::key(qv[s]); cand_pos[c * J + s] = (pos_t)qp[s]; }
  }
}

// Stage 2 over the candidates parked in LDS (exact order keys and sub-row
// numbers, candidate c*J + s belonging to column c): the block-wide radix
// select, then the survivors in candidate order.  Starts with a barrier.
template <typename E, int J, bool CONTIG, typename skey_t, typename pos_t, typename Sh>
__device__ __forceinline__ void select_from_lds(Sh& sh, const typename E::raw_t* __restrict__ xr, const Geom& g,
                                                const skey_t* cand_key, const pos_t* cand_pos, uint32_t k0,
                                                uint32_t k, int index_bits, int64_t row,
                                                typename E::raw_t* __restrict__ values, const IndexOut& indices) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  auto key_at = [&](uint32_t i) -> key_t { return cand_key[i]; };
  auto index_at = [&](uint32_t i) -> uint64_t {
    if constexpr (CONTIG) return (uint64_t)(i / J) * g.full_rows + cand_pos[i];
    return (uint64_t)cand_pos[i] * (uint64_t)g.b + i / J;
  };
  const select::Cut<key_t> cut =
      select::find_cut<key_t, E::key_bits>(sh, k0, k, index_bits, key_at, index_at);

  raw_t* ov = values + row * (int64_t)k;
  const int64_t oi = row * (int64_t)k;  // this row's first output slot
  auto survives = [&](uint32_t i) -> bool {
    const key_t key = key_at(i);
    if (key != cut.T) return key > cut.T;
    return cut.index_cut == ~0ull || index_at(i) <= cut.index_cut;
  };
  // The survivors' values are worked out from their keys; only a key that does
  // not name one bit pattern (a zero, a NaN) sends its lane to the row.
  struct Got { int64_t index; raw_t value; };
  select::compact(
      sh, k0, k, survives,
      [&](uint32_t i) {
        const int64_t index = (int64_t)index_at(i);
        const key_t key = key_at(i);
        raw_t value = E::unkey(key);
        if (!E::key_is_exact(key) && survives(i)) value = xr[index];
        return Got{index, value};
      },
      [&](uint32_t, uint32_t o, const Got& got) {
        if (values != nullptr) ov[o] = got.value;
        indices.put(oi + o, got.index);
      });
}

// pos_t: uint16_t when every sub-row number fits, else uint32_t.  PACKED: packed
// 16-bit queues (stage1_stream.h).
// The SGPR cap keeps eight waves per SIMD possible (beyond 96 scalar registers
// only seven fit, whatever the vector registers allow): for 1024 fp16 rows of
// 32768 with 8192 candidates that is a fourth workgroup per CU and every row
// resident at once.
template <typename E, int J, int V, int MAXW, typename pos_t, bool PACKED>
__global__ __launch_bounds__(kWave * MAXW) __attribute__((amdgpu_num_sgpr(80))) void fused_row_kernel(
    const typename E::raw_t* __restrict__ x, typename E::raw_t* __restrict__ values,
    const IndexOut indices, const Geom g, uint32_t tiles, uint32_t split, uint32_t hand_off,
    uint32_t k0, uint32_t k, int index_bits) {
  using raw_t = typename E::raw_t;
  using key_t = typename E::key_t;
  // keys are stored at their significant width
  using skey_t = std::conditional_t<E::key_bits <= 16, uint16_t, key_t>;
  using Queue = stream::QueueFor<E, J, V, PACKED>;
  constexpr int kTileCols = kWave * V;
  constexpr int U = PACKED ? (V * J <= 8 ? 8 : 4) : (J <= 2 ? 8 : 4);

  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ select::SharedT<4> sh;  // four histogram copies: four workgroups of C3's shape fit one CU's LDS
  // Candidates, and the hand-over area of the waves that share a tile: behind
  // the candidates, or (hand_off == 0, single round only) on top of them, in
  // which case a barrier separates the last fold from the first candidate.
  skey_t* cand_key = reinterpret_cast<skey_t*>(dyn_lds);
  const uint32_t pos_off = (k0 * (uint32_t)sizeof(skey_t) + 15u) & ~15u;
  pos_t* cand_pos = reinterpret_cast<pos_t*>(dyn_lds + pos_off);
  const uint32_t nwaves = blockDim.x / kWave;
  unsigned char* hand = dyn_lds + hand_off;  // one Queue::kHandBytes area per wave that is not a tile leader

  const uint32_t lane = threadIdx.x % kWave;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int64_t row = blockIdx.x;
  const raw_t* xr = x + row * g.row_stride;

  const uint32_t part = wave % split;            // which share of the sub-rows
  const uint32_t group = wave / split;           // tile slot of this wave
  const uint32_t groups = nwaves / split;        // tiles in flight per round
  const uint32_t p0 = __builtin_amdgcn_readfirstlane((uint32_t)(((uint64_t)g.full_rows * part) / split));
  const uint32_t p1 = __builtin_amdgcn_readfirstlane((uint32_t)(((uint64_t)g.full_rows * (part + 1)) / split));

  bool any_nan = false;
  for (uint32_t base = 0; base < tiles; base += groups) {  // same trip count for every wave
    const uint32_t tile = base + group;
    const bool has_tile = tile < tiles;
    const int64_t col = (int64_t)tile * kTileCols + lane * V;
    const bool live = has_tile && col < g.b;
    Queue queue;
    if (has_tile) {
      if (split > 1) stream::scan_windows<E, J, V, U>(xr, g, col, live, part, split, part == split - 1, queue);
      else stream::scan_run<E, J, V, U, 0>(xr, g, col, live, p0, p1, true, queue);
      any_nan |= queue.poisoned();
    }
    if (split > 1) {
      if (has_tile && part > 0)
        queue.hand_over(hand + (size_t)(group * (split - 1) + (part - 1)) * Queue::kHandBytes, lane);
      __syncthreads();
      if (has_tile && part == 0) {
        for (uint32_t w = 0; w + 1 < split; ++w)
          queue.fold_in_interleaved(hand + (size_t)(group * (split - 1) + w) * Queue::kHandBytes, lane);
      }
      if (hand_off == 0) __syncthreads();
    }
    if (live && part == 0) {
      ATK_STATIC_FOR(e, V * J) {
        cand_key[col * J + e] = (skey_t)queue.template key<e / J, e % J>();
        cand_pos[col * J + e] = (pos_t)queue.template position<e / J, e % J>();
      } ATK_STATIC_END;
    }
    if (split > 1 && hand_off != 0) __syncthreads();  // the hand-over area is reused by the next round
  }

  if (__syncthreads_or(any_nan)) redo_exact_into_lds<E, J, false>(xr, g, cand_key, cand_pos);
  // (the select's first pass starts with a barrier, which also publishes the candidates)
  select_from_lds<E, J, false>(sh, xr, g, cand_key, cand_pos, k0, k, index_bits, row, values, indices);
}

// ---------------------------------------------------------------------------
// The same with the candidates kept in registers through stage 2, for rows all
// of whose column tiles are scanned at once (tiles * split <= waves): when the
// scan ends, every lane of a tile's leading wave holds its V*J candidates, so
// nothing is parked in LDS.  The cut is found by an MSB-first radix select with
// 12-bit digits whose histograms (4096 bins in LDS, one atomic add per
// candidate straight from its register) are read by all threads; as soon as
// the bin that holds the k-th best has at most kListMax members, those are
// listed and ranked under the full order (key, then lower index), which gives
// the cut in one step whatever key bits are left.  Survivors are counted per
// lane, placed by a wave prefix sum and per-wave bases, and written from
// registers in candidate order.  Rows that met a NaN, or whose cut falls among
// more than kListMax candidates with one and the same key, take the LDS path
// of the kernel above.  Results are identical.
// ---------------------------------------------------------------------------
namespace regs = select::regs;

// Stage 1 of a row whose buckets are runs of `m` adjacent elements of 16 to 256
// bytes each (contiguous layout, every bucket as long).  A lane takes V buckets
// kWave apart, `first` the first of them, so that the lanes of a wave load from
// adjacent buckets, and loads a bucket whole (64 bytes of it at a time), 16
// bytes a load, before it feeds it to the bucket's queue with the place within the bucket as the sub-row
// number: the loads of a wave then cover a stretch of the row back to back.
// (With the lane's buckets side by side, lanes 128-256 bytes apart, and with one
// load per bucket at a time, so that the second 16 bytes of a cache line are
// asked for long after the first, fp32 [1024, 32768] with 2048 buckets took
// 72-75 us against 47 for the interleaved row.)  AHEAD: the next bucket is loaded
// before this one is fed.
template <typename E, int J, int V, bool PACKED, bool AHEAD, typename Queue>
__device__ __forceinline__ void scan_short_buckets(const typename E::raw_t* __restrict__ xr, uint32_t m,
                                                   int64_t first, Queue& queue) {
  using raw_t = typename E::raw_t;
  constexpr int EPL = 16 / (int)sizeof(raw_t);  // elements per load
  constexpr int kMaxLoads = 4;                  // loads of a bucket issued together
  static_assert(EPL >= J && EPL % 2 == 0, "the first load of a bucket fills its queue");
  using Load = stream::Pack<raw_t, EPL>;
  const raw_t* next = xr + first * (int64_t)m;
  const int64_t apart = (int64_t)kWave * m;
  const uint32_t loads = __builtin_amdgcn_readfirstlane(m / EPL);
  queue.reset();
  auto load_bucket = [&](Load (&buf)[kMaxLoads]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < kMaxLoads; ++c) {
      if (c == 0 || (uint32_t)c < loads) buf[c] = stream::load_pack<raw_t, EPL>(next + c * EPL);
    }
    next += apart;
  };
  // the loads `buf` of bucket v: elements at + c * EPL .. of the bucket, c = 0 .. kMaxLoads - 1
  auto feed_loads = [&](auto v_c, auto first_c, const Load (&buf)[kMaxLoads], uint32_t at, uint32_t count)
      __attribute__((always_inline)) {
    constexpr int v = decltype(v_c)::value;
    constexpr bool kFirst = decltype(first_c)::value;  // the bucket's first loads: its queue fills
    ATK_STATIC_FOR(c, kMaxLoads) {
      if (c == 0 || (uint32_t)c < count) {
        ATK_STATIC_FOR(d, EPL / 2) {
          constexpr int kFilled = (kFirst && c == 0 && 2 * d < J) ? 2 * d : J;
          if constexpr (PACKED) {
            uint32_t x;
            __builtin_memcpy(&x, &buf[c].e[2 * d], 4);
            queue.template take_two<v, kFilled>(x, at + c * EPL + 2 * d);
          } else {
            queue.template take_two<v, kFilled>(buf[c].e[2 * d], buf[c].e[2 * d + 1], at + c * EPL + 2 * d);
          }
        } ATK_STATIC_END;
      }
    } ATK_STATIC_END;
  };
  auto feed = [&](auto v_c, const Load (&buf)[kMaxLoads]) __attribute__((always_inline)) {
    constexpr int v = decltype(v_c)::value;
    feed_loads(v_c, std::true_type{}, buf, 0u, loads);
    // a bucket of more than 64 bytes: the rest of it, kMaxLoads loads at a time
    const raw_t* rest = xr + (first + (int64_t)v * kWave) * (int64_t)m;
#pragma nounroll
    for (uint32_t c0 = kMaxLoads; c0 < loads; c0 += kMaxLoads) {
      Load more[kMaxLoads];
#pragma unroll
      for (int c = 0; c < kMaxLoads; ++c) {
        if (c == 0 || c0 + (uint32_t)c < loads) more[c] = stream::load_pack<raw_t, EPL>(rest + (c0 + c) * EPL);
      }
      feed_loads(v_c, std::false_type{}, more, c0 * EPL, loads - c0);
    }
  };
  if constexpr (AHEAD) {
    Load buf[2][kMaxLoads];
    load_bucket(buf[0]);
    ATK_STATIC_FOR(v, V) {
      if constexpr (v + 1 < V) load_bucket(buf[(v + 1) % 2]);
      feed(std::integral_constant<int, v>{}, buf[v % 2]);
    } ATK_STATIC_END;
  } else {
    ATK_STATIC_FOR(v, V) {
      Load buf[kMaxLoads];
      load_bucket(buf);
      feed(std::integral_constant<int, v>{}, buf);
    } ATK_STATIC_END;
  }
}

// Packed queues of up to 16 entries per lane are held to 64 vector registers
// (eight waves per SIMD: four 8-wave workgroups per CU); what does not fit is
// spilled where the pressure peaks, in the rarely taken LDS path.  The scan of
// contiguous buckets with 16 entries per lane is left its 80 registers (six
// waves per SIMD): its loads of whole buckets spill in the scan itself
// otherwise (fp16 [1024, 32768] k=2048 j=4 k_mult=4 36 -> 31 us, [4096, 8192]
// k=512 45 -> 36 us; with 8 entries per lane the 64 registers win by a tenth).
// (No cap on the scalar registers here: the packed kernels' eight waves per SIMD already hold the
// compiler to 96, and the others, which cannot reach eight waves for their vector registers, spilled
// 46-107 scalar registers into vector lanes under a cap of 80: fp32 [256, 131072] k=64 j=1 k_mult=8
// 28.3 -> 28.0 us without it.)
// PAST_CACHE: staged results leave four per thread (staged == 2) in non-temporal stores; a
// kernel of its own, because as a branch it cost the usual way out 2 us of 36 (fp16 [4096, 8192]
// k=512 j=4 k_mult=4) through the registers it moved.
// CONTIG: the row's buckets are contiguous runs of g.full_rows elements of at
// most 256 bytes (no remainder, whole tiles, one wave per tile).  The scan differs,
// the way an index is put together, and which buckets a lane holds: V buckets
// kWave apart (bucket_of), so that a wave's candidates in their order are those
// of every lane's first bucket, then of every lane's second, ...
template <typename E, int J, int V, int MAXW, typename pos_t, bool PACKED, bool CONTIG = false, bool PAST_CACHE = false>
__global__ __launch_bounds__(kWave * MAXW)
__attribute__((amdgpu_waves_per_eu(PACKED && V * J <= 16 && !(CONTIG && V * J > 8) ? 8 : 1))) void fused_regs_kernel(
    const typename E::raw_t* __restrict__ x, typename E::raw_t* __restrict__ values,
    const IndexOut indices, const Geom g, uint32_t tiles, uint32_t split, uint32_t hand_off,
    uint32_t k0, uint32_t k, int index_bits, int staged) {
  using raw_t = typename E::raw_t;
  using skey_t = std::conditional_t<E::key_bits <= 16, uint16_t, typename E::key_t>;
  using Queue = stream::QueueFor<E, J, V, PACKED, true>;
  using sel_t = typename Queue::sel_t;
  // positions in the row fit 32 bits whenever sub-row numbers fit 16 (the candidates fit LDS)
  using idx_t = std::conditional_t<sizeof(pos_t) == 2, uint32_t, uint64_t>;
  constexpr int kTileCols = kWave * V;
  constexpr int NC = V * J;  // candidates per lane
  constexpr int U = PACKED ? (V * J <= 8 ? 8 : 4) : (J <= 2 ? 8 : 4);

  extern __shared__ __align__(16) unsigned char dyn_lds[];
  __shared__ select::SharedT<4> sh;  // the LDS path's
  __shared__ regs::Shared rs;
  skey_t* cand_key = reinterpret_cast<skey_t*>(dyn_lds);
  const uint32_t pos_off = (k0 * (uint32_t)sizeof(skey_t) + 15u) & ~15u;
  pos_t* cand_pos = reinterpret_cast<pos_t*>(dyn_lds + pos_off);
  unsigned char* hand = dyn_lds + hand_off;
  uint32_t* hist = reinterpret_cast<uint32_t*>(dyn_lds);  // on top of the candidates: they are parked only after it
  uint64_t* list_key = reinterpret_cast<uint64_t*>(dyn_lds + regs::kListOff);
  uint64_t* list_index = list_key + regs::kListWords;

  const uint32_t tid = threadIdx.x, nt = blockDim.x;
  const uint32_t lane = tid % kWave;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int64_t row = blockIdx.x;
  const raw_t* xr = x + row * g.row_stride;

  ATK_TRACE_GROUP(0);
  const uint32_t part = wave % split;   // which share of the sub-rows
  const uint32_t tile = wave / split;   // every tile has its waves: tiles * split == waves
  const uint32_t p0 = __builtin_amdgcn_readfirstlane((uint32_t)(((uint64_t)g.full_rows * part) / split));
  const uint32_t p1 = __builtin_amdgcn_readfirstlane((uint32_t)(((uint64_t)g.full_rows * (part + 1)) / split));
  const bool has_tile = tile < tiles;
  const int64_t col = (int64_t)tile * kTileCols + (CONTIG ? lane : lane * V);
  const bool live = has_tile && col < g.b;
  const bool mine = live && part == 0;  // this lane ends up holding candidates
  // the bucket (column) of the lane's v-th queue
  auto bucket_of = [&](int v) __attribute__((always_inline)) -> int64_t {
    return CONTIG ? col + (int64_t)v * kWave : col + v;
  };

  Queue queue;
  // packed entries: sub-row numbers 0..full_rows at the top of the low half, so
  // that the bits in which entries differ are the leading ones
  queue.set_position_shift(sizeof(pos_t) == 2 ? (uint32_t)__builtin_clz(g.full_rows | 1u) - 16u : 0u);
  // The first radix pass over sel_key (below) takes its leading `bits0` bits.  With a wave per
  // tile (split == 1) nothing else uses the LDS while the row is scanned, so the histograms are
  // cleared before the scan and a wave counts its candidates' digits as soon as its own scan is
  // done, rather than after the workgroup's slowest wave: one barrier phase less in the chain that
  // every workgroup goes through after its scan.
  constexpr bool kKeyHalf = CONTIG && PACKED;
  const int shift_end = kKeyHalf ? 16 : queue.sel_constant_bits();
  const int bits0 = Queue::sel_bits - shift_end < regs::kDigitBits ? Queue::sel_bits - shift_end : regs::kDigitBits;
  const bool early = (CONTIG || split == 1) && k != k0 && k0 > regs::kListMax && bits0 > 0;
  if (early) {
    for (uint32_t i = tid * 4; i < 2 * regs::kHistWords; i += nt * 4)
      *reinterpret_cast<uint4*>(&hist[i]) = make_uint4(0, 0, 0, 0);
    if (tid == 0) rs.list_count = 0;
    __syncthreads();
  }
  bool any_nan = false;
  if (has_tile) {
    if constexpr (CONTIG) scan_short_buckets<E, J, V, PACKED, !PACKED>(xr, g.full_rows, col, queue);
    else if (split > 1) stream::scan_windows<E, J, V, U>(xr, g, col, live, part, split, part == split - 1, queue);
    else stream::scan_run<E, J, V, U, 0>(xr, g, col, live, p0, p1, true, queue);
    any_nan = queue.poisoned();
  }
  if (early && mine) {  // (a wave that met a NaN counts keys that mean nothing: the row leaves the fast path anyway)
    const int shift0 = Queue::sel_bits - bits0;
    const uint32_t dmask0 = (1u << bits0) - 1u;
    ATK_STATIC_FOR(e, NC) {
      sel_t key = queue.template sel_key<e / J, e % J>();
      if constexpr (kKeyHalf) key &= (sel_t)0xffff0000u;
      atomicAdd(&hist[regs::hist_slot((uint32_t)(key >> shift0) & dmask0)], 1u);
    } ATK_STATIC_END;
  }
  if constexpr (!CONTIG) {
    if (split > 1) {
      if (has_tile && part > 0)
        queue.hand_over(hand + (size_t)(tile * (split - 1) + (part - 1)) * Queue::kHandBytes, lane);
      __syncthreads();
      if (has_tile && part == 0) {
        for (uint32_t w = 0; w + 1 < split; ++w)
          queue.fold_in_interleaved(hand + (size_t)(tile * (split - 1) + w) * Queue::kHandBytes, lane);
      }
    }
    // Both histograms start at zero.  Waves that shared a tile must first be done
    // with the hand-over area, which may lie in the same place.
    if (split > 1) __syncthreads();
  }
  ATK_TRACE_GROUP(1);
  if (!early) {
    for (uint32_t i = tid * 4; i < 2 * regs::kHistWords; i += nt * 4)
      *reinterpret_cast<uint4*>(&hist[i]) = make_uint4(0, 0, 0, 0);
    if (tid == 0) rs.list_count = 0;
  }
  const bool nan_row = __syncthreads_or(any_nan);
  ATK_TRACE_GROUP(2);

  // (keys are taken from the queues where they are used rather than kept: registers)
  // (Packed entries carry the sub-row number below the key, which is the order of the
  // indices of equal keys in the interleaved layout only: sub-row first, then column.)
  auto key_of = [&](auto e_c) __attribute__((always_inline)) -> sel_t {
    constexpr int e = decltype(e_c)::value;
    if constexpr (kKeyHalf) return queue.template sel_key<e / J, e % J>() & (sel_t)0xffff0000u;
    return queue.template sel_key<e / J, e % J>();
  };
  auto index_of = [&](auto e_c) __attribute__((always_inline)) -> idx_t {
    constexpr int e = decltype(e_c)::value;
    if constexpr (CONTIG) return (idx_t)bucket_of(e / J) * (idx_t)g.full_rows + (idx_t)queue.template position<e / J, e % J>();
    return (idx_t)queue.template position<e / J, e % J>() * (idx_t)g.b + (idx_t)bucket_of(e / J);
  };

  // MSB-first radix passes over sel_key.  After a pass the candidates still in
  // the race share `prefix` in the bits of `mask`; `need` of those `count` belong
  // to the result.  The race ends when all of them do (the cut is then the
  // prefix itself), when they are few enough to be listed and ranked, or, with
  // no bits left, when they are too many equal keys for that (the LDS path then
  // cuts them by index).  Pass p counts into histogram p % 2, which the pass
  // before last left cleared; wave 0 reads it.
  sel_t prefix = 0, mask = 0;
  uint32_t need = k, count = k0;
  enum { kByPrefix, kByList, kGiveUp } how = kGiveUp;
  if (!nan_row) {
    int shift = Queue::sel_bits;
    for (uint32_t pass = 0;; ++pass) {
      if (need == count) { how = kByPrefix; break; }
      if (count <= regs::kListMax) { how = kByList; break; }
      if (shift <= shift_end) break;
      const int bits = shift - shift_end < regs::kDigitBits ? shift - shift_end : regs::kDigitBits;
      shift -= bits;
      const uint32_t dmask = (1u << bits) - 1u;
      uint32_t* h = hist + (pass & 1u) * regs::kHistWords;
      if (pass == 0 && early) {
        // counted already, and the barrier that told of NaNs has published the counts
      } else {
        if (mine) {
          if (pass == 0) {  // every candidate counts
            ATK_STATIC_FOR(e, NC) {
              const sel_t key = key_of(std::integral_constant<int, e>{});
              atomicAdd(&h[regs::hist_slot((uint32_t)(key >> shift) & dmask)], 1u);
            } ATK_STATIC_END;
          } else {
            ATK_STATIC_FOR(e, NC) {
              const sel_t key = key_of(std::integral_constant<int, e>{});
              if ((key & mask) == prefix) atomicAdd(&h[regs::hist_slot((uint32_t)(key >> shift) & dmask)], 1u);
            } ATK_STATIC_END;
          }
        }
        __syncthreads();
      }
      if (wave == 0) {
        const regs::Found f = regs::find_bin_wave(h, need, count, lane);
        if (lane == 0) { rs.digit = f.digit; rs.need = f.need; rs.count = f.count; }
      }
      if (pass >= 1) {  // the other histogram, for the pass after this one
        uint32_t* other = hist + ((pass & 1u) ^ 1u) * regs::kHistWords;
        for (uint32_t i = tid * 4; i < regs::kHistWords; i += nt * 4)
          *reinterpret_cast<uint4*>(&other[i]) = make_uint4(0, 0, 0, 0);
      }
      __syncthreads();
      ATK_TRACE_GROUP(pass == 0 ? 3 : 4);
      prefix |= (sel_t)rs.digit << shift;
      mask |= (sel_t)dmask << shift;
      need = rs.need;
      count = rs.count;
    }
  }
  if (how == kGiveUp) {
    // Off the fast path, through the candidate arrays in LDS as in the kernel
    // above: a NaN in the row (stage 1 again, with exact keys), or more than
    // kListMax candidates equal to the cut key under sel_key (cut by index).
    __syncthreads();
    if (nan_row) {
      redo_exact_into_lds<E, J, CONTIG>(xr, g, cand_key, cand_pos);
    } else if (mine) {
      ATK_STATIC_FOR(e, NC) {
        cand_key[bucket_of(e / J) * J + e % J] = (skey_t)queue.template key<e / J, e % J>();
        cand_pos[bucket_of(e / J) * J + e % J] = (pos_t)queue.template position<e / J, e % J>();
      } ATK_STATIC_END;
    }
    select_from_lds<E, J, CONTIG>(sh, xr, g, cand_key, cand_pos, k0, k, index_bits, row, values, indices);
    return;
  }

  // The cut: a candidate survives when its key is above cut_key, or equal to it
  // with an index below cut_below.
  sel_t cut_key;
  idx_t cut_below;
  if (how == kByPrefix) {
    // everything at or above the prefix survives (prefix > 0: something is cut)
    cut_key = prefix - 1;
    cut_below = 0;
  } else {
    // List the candidates that share the prefix; wave 0 ranks them (lane t takes
    // entry t and counts the better ones): the need-th best is the cut.  An entry
    // is one 64-bit word when key and index fit 32 bits each (key above inverted
    // index: a larger word is a better candidate), else two.  The list is read
    // four entries at a time; its last group is filled up with entries that
    // beat nothing.
    constexpr bool kOneWord = sizeof(sel_t) == 4 && sizeof(idx_t) == 4;
    if (tid < 8u) {
      list_key[count + tid] = 0;
      list_index[count + tid] = ~0ull;
    }
    if (mine) {
      ATK_STATIC_FOR(e, NC) {
        const sel_t key = key_of(std::integral_constant<int, e>{});
        if ((key & mask) == prefix) {
          const uint32_t slot = atomicAdd(&rs.list_count, 1u);
          const idx_t index = index_of(std::integral_constant<int, e>{});
          if constexpr (kOneWord) {
            list_key[slot] = ((uint64_t)key << 32) | (uint64_t)(0xffffffffu - (uint32_t)index);
          } else {
            list_key[slot] = (uint64_t)key;
            list_index[slot] = (uint64_t)index;
          }
        }
      } ATK_STATIC_END;
    }
    __syncthreads();
    if (wave == 0) {
      const uint32_t t = lane < count ? lane : 0u;
      const uint64_t my_key = list_key[t];
      const uint64_t my_index = kOneWord ? 0ull : list_index[t];
      uint32_t better = 0;
      // (four entries per trip and no unrolling: with eight, the sixteen registers of a trip were
      // what made the compiler spill part of the lane's candidates to scratch memory in the
      // kernels held to 64 registers -- 9 to 24 registers, 13 to 35 MB of HBM traffic per launch
      // of fp16 [1024, 32768] k=2048 j=4 k_mult=4, which takes 24.2 us without them against 25.9)
      constexpr int kGroup = 4;
#pragma nounroll
      for (uint32_t m = 0; m < count; m += kGroup) {
        uint64_t key[kGroup], index[kGroup];
#pragma unroll
        for (int u = 0; u < kGroup; ++u) { key[u] = list_key[m + u]; index[u] = kOneWord ? 0ull : list_index[m + u]; }
#pragma unroll
        for (int u = 0; u < kGroup; ++u)
          better += (key[u] > my_key || (!kOneWord && key[u] == my_key && index[u] < my_index)) ? 1u : 0u;
      }
      if (lane < count && better + 1 == need) {  // one lane
        rs.cut_key = my_key;
        rs.cut_index = my_index;
      }
    }
    __syncthreads();
    if constexpr (kOneWord) {
      cut_key = (sel_t)(rs.cut_key >> 32);
      cut_below = (idx_t)(0xffffffffu - (uint32_t)rs.cut_key) + 1u;
    } else {
      cut_key = (sel_t)rs.cut_key;
      cut_below = (idx_t)rs.cut_index + 1u;
    }
  }

  ATK_TRACE_GROUP(5);
  // survivors among this lane's candidates
  uint32_t selected = 0;  // bit e: candidate e survives
  ATK_STATIC_FOR(e, NC) {
    const sel_t key = key_of(std::integral_constant<int, e>{});
    bool s = key > cut_key;
    if (key == cut_key) s = index_of(std::integral_constant<int, e>{}) < cut_below;
    selected |= (mine && s) ? (1u << e) : 0u;
  } ATK_STATIC_END;
  // Output slots follow the candidates' order: wave by wave, and within a wave lane by
  // lane with the lane's candidates in a row, or (CONTIG) the lanes' v-th buckets
  // together for one v after the other.  slot[r]: where the next survivor of run r goes.
  constexpr int kRuns = CONTIG ? V : 1, kRunLen = NC / kRuns;
  uint32_t slot[kRuns];
  {
    uint32_t before = 0;  // survivors of this wave in the runs so far
    ATK_STATIC_FOR(r, kRuns) {
      const uint32_t kept = (uint32_t)__popc((selected >> (r * kRunLen)) & (uint32_t)((1ull << kRunLen) - 1ull));
      const uint32_t incl = regs::wave_scan(kept);
      slot[r] = before + incl - kept;
      before += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
    } ATK_STATIC_END;
    if (lane == kWave - 1) rs.wave_total[wave] = before;
  }
  __syncthreads();
  ATK_TRACE_GROUP(6);
  {
    uint32_t waves_before = 0;
    for (uint32_t w = 0; w < wave; ++w) waves_before += rs.wave_total[w];
    ATK_STATIC_FOR(r, kRuns) { slot[r] += waves_before; } ATK_STATIC_END;
  }
  raw_t* ov = values + row * (int64_t)k;
  const int64_t oi = row * (int64_t)k;
  if constexpr (sizeof(idx_t) == 4 && sizeof(raw_t) <= 4) {
    if (staged != 0) {
      // Survivors go to LDS first, as their queue entries and columns at their
      // output slots (eight bytes each; exactly k of them), and the threads that
      // carry the row's results out in whole-wave stores turn them into elements
      // and indices: a quarter as many conversions as candidates.  The area
      // lies on top of the histograms and the list, which nobody reads any more
      // (the barrier above).
      uint2* stage = reinterpret_cast<uint2*>(dyn_lds);
      ATK_STATIC_FOR(e, NC) {
        uint32_t& o = slot[e / kRunLen];
        if ((selected >> e) & 1u) stage[o] = queue.template staged<e / J, e % J>((uint32_t)bucket_of(e / J));
        o += (selected >> e) & 1u;
      } ATK_STATIC_END;
      __syncthreads();
      ATK_TRACE_GROUP(7);
      auto result = [&](uint2 w, raw_t& value) __attribute__((always_inline)) -> uint32_t {
        const typename Queue::Unstaged u = queue.unstage(w);
        const uint32_t index = CONTIG ? u.column * g.full_rows + u.sub_row : u.sub_row * (uint32_t)g.b + u.column;
        value = u.raw;
        if (u.reread) value = xr[index];  // a zero: its sign is in the row
        return index;
      };
      if (staged == 2) {  // four results per thread: k is a multiple of four and the outputs are 16-byte aligned
        for (uint32_t at = tid * 4; at < k; at += nt * 4) {
          const uint4 e01 = *reinterpret_cast<const uint4*>(&stage[at]);
          const uint4 e23 = *reinterpret_cast<const uint4*>(&stage[at + 2]);
          stream::Pack<raw_t, 4> pv;
          uint32_t index[4];
          index[0] = result(make_uint2(e01.x, e01.y), pv.e[0]);
          index[1] = result(make_uint2(e01.z, e01.w), pv.e[1]);
          index[2] = result(make_uint2(e23.x, e23.y), pv.e[2]);
          index[3] = result(make_uint2(e23.z, e23.w), pv.e[3]);
          if constexpr (PAST_CACHE) {
            // (non-temporal stores: one round of workgroups with a sizeable output, see the planner)
            typedef uint32_t nt4 __attribute__((ext_vector_type(4)));
            typedef uint32_t nt2 __attribute__((ext_vector_type(2)));
            if (values != nullptr) {
              if constexpr (sizeof(raw_t) == 4) {
                nt4 w;
                __builtin_memcpy(&w, &pv, 16);
                __builtin_nontemporal_store(w, reinterpret_cast<nt4*>(ov + at));
              } else if constexpr (sizeof(raw_t) == 2) {
                nt2 w;
                __builtin_memcpy(&w, &pv, 8);
                __builtin_nontemporal_store(w, reinterpret_cast<nt2*>(ov + at));
              } else {
                uint32_t w;
                __builtin_memcpy(&w, &pv, 4);
                __builtin_nontemporal_store(w, reinterpret_cast<uint32_t*>(ov + at));
              }
            }
            if (indices.narrow) {
              const nt4 w = {index[0], index[1], index[2], index[3]};
              __builtin_nontemporal_store(w, reinterpret_cast<nt4*>(static_cast<int32_t*>(indices.base) + oi + at));
            } else {
              nt4* out = reinterpret_cast<nt4*>(static_cast<int64_t*>(indices.base) + oi + at);
              const nt4 lo = {index[0], 0u, index[1], 0u}, hi = {index[2], 0u, index[3], 0u};
              __builtin_nontemporal_store(lo, out);
              __builtin_nontemporal_store(hi, out + 1);
            }
            continue;
          }
          if (values != nullptr) *reinterpret_cast<stream::Pack<raw_t, 4>*>(ov + at) = pv;
          if (indices.narrow) {
            stream::Pack<int32_t, 4> pi;
#pragma unroll
            for (int u = 0; u < 4; ++u) pi.e[u] = (int32_t)index[u];
            *reinterpret_cast<stream::Pack<int32_t, 4>*>(static_cast<int32_t*>(indices.base) + oi + at) = pi;
          } else {
            int64_t* out = static_cast<int64_t*>(indices.base) + oi + at;
            stream::Pack<int64_t, 2> lo, hi;
            lo.e[0] = (int64_t)index[0]; lo.e[1] = (int64_t)index[1];
            hi.e[0] = (int64_t)index[2]; hi.e[1] = (int64_t)index[3];
            reinterpret_cast<stream::Pack<int64_t, 2>*>(out)[0] = lo;
            reinterpret_cast<stream::Pack<int64_t, 2>*>(out)[1] = hi;
          }
        }
      } else {
        for (uint32_t at = tid; at < k; at += nt) {
          raw_t value;
          const uint32_t index = result(stage[at], value);
          if (values != nullptr) ov[at] = value;
          indices.put(oi + at, (int64_t)index);
        }
      }
      ATK_TRACE_GROUP(8);
      return;
    }
  }
  if (mine) {
    if constexpr (CONTIG) queue.fix_zeros(xr, 1, col * (int64_t)g.full_rows, (int64_t)kWave * g.full_rows);
    else queue.fix_zeros(xr, g.b, col);
  }
  ATK_STATIC_FOR(e, NC) {
    uint32_t& o = slot[e / kRunLen];
    if ((selected >> e) & 1u) {
      if (o < k) {
        if (values != nullptr) ov[o] = queue.template raw<e / J, e % J>();
        indices.put(oi + o, (int64_t)index_of(std::integral_constant<int, e>{}));
      }
      ++o;
    }
  } ATK_STATIC_END;
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct Plan {
  bool ok;
  int vec;              // V
  uint32_t full_rows, rem, pad_tail;
  uint32_t tiles;       // column tiles per row
  uint32_t split;       // waves sharing a tile
  uint32_t waves;       // waves per workgroup
  bool pos16;           // sub-row numbers fit 16 bits
  bool packed;          // packed 16-bit queues
  int index_bits;
  uint32_t hand_off;    // byte offset of the hand-over area in dynamic LDS (0: on top of the candidates)
  size_t lds_bytes;     // dynamic LDS
  bool contig;          // contiguous buckets of a few elements each (in_registers only)
  bool in_registers;    // all tiles are scanned at once: the candidates stay in registers through stage 2
  bool staged;          // in_registers: the survivors are gathered in LDS and leave in whole-wave stores
  bool past_cache;      // staged: ... in non-temporal stores (one round of workgroups with a sizeable output)
};

Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int64_t k, int layout, int dtype, bool aligned);

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int64_t k0, int j,
                 int64_t k, void* values, IndexOut indices, hipStream_t stream);

}  // namespace fused
}  // namespace atk
