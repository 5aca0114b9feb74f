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

namespace atk {
namespace fused {

using stream::Cmp;
using stream::Geom;
using stream::kWave;

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
      stream::scan_run<E, J, V, U, 0>(xr, g, col, live, p0, p1, part == split - 1, queue);
      any_nan |= queue.poisoned();
    }
    if (split > 1) {
      if (has_tile && part > 0)
        queue.hand_over(hand + (size_t)(group * (split - 1) + (part - 1)) * Queue::kHandBytes, lane);
      __syncthreads();
      if (has_tile && part == 0) {
        for (uint32_t w = 0; w + 1 < split; ++w)
          queue.fold_in(hand + (size_t)(group * (split - 1) + w) * Queue::kHandBytes, lane);
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

  if (__syncthreads_or(any_nan)) {
    // a value the fast queues cannot order (NaN; -0.0 for packed queues) was
    // loaded somewhere in the row: redo stage 1 with exact order keys
    for (int64_t c = threadIdx.x; c < g.b; c += blockDim.x) {
      raw_t qv[J];
      uint32_t qp[J];
      stream::clear_exact<E, J>(qv, qp);
      for (uint32_t p = 0; p < g.full_rows; ++p) stream::push_exact<E, J>(qv, qp, xr[(int64_t)p * g.b + c], p);
      if (g.rem != 0) {
        if (c < (int64_t)g.rem)
          stream::push_exact<E, J>(qv, qp, xr[(int64_t)g.full_rows * g.b + c], g.full_rows);
        else if (g.pad_tail)
          stream::push_exact<E, J>(qv, qp, E::pad_raw, g.full_rows);
      }
#pragma unroll
      for (int s = 0; s < J; ++s) { cand_key[c * J + s] = (skey_t)E::key(qv[s]); cand_pos[c * J + s] = (pos_t)qp[s]; }
    }
  }
  // (the select's first pass starts with a barrier, which also publishes the candidates)

  auto key_at = [&](uint32_t i) -> key_t { return cand_key[i]; };
  auto index_at = [&](uint32_t i) -> uint64_t { return (uint64_t)cand_pos[i] * (uint64_t)g.b + i / J; };
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
        ov[o] = got.value;
        indices.put(oi + o, got.index);
      });
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
};

Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int64_t k, int layout, int dtype, bool aligned);

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int64_t k0, int j,
                 int64_t k, void* values, IndexOut indices, hipStream_t stream);

}  // namespace fused
}  // namespace atk
