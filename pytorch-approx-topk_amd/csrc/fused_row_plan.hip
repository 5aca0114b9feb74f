// Host-side planning and dispatch of the fused one-workgroup-per-row kernel.
#include "fused_row.h"

namespace atk {
namespace fused {

namespace {
// Rows below which one workgroup per row leaves most of the 256 CUs idle: taken
// then only for rows one workgroup reads in a few microseconds, where saving
// the second launch is what counts (1-96 rows in a HIP graph, bf16 up to 128K
// elements: 16-31 % faster; rows of 512 KiB: even to 13 % slower; of 1 MiB: 20-60 %
// slower).
constexpr int64_t kMinRows = 128;
constexpr size_t kSoloRow = 256 * 1024;
// Dynamic LDS a workgroup may use (candidates + hand-over); the select's own
// block adds about 9 KiB.
constexpr size_t kLdsBudget = 64 * 1024;
// The candidates may take twice that, one workgroup of sixteen waves per CU
// then: the alternative parks them in HBM and selects with one workgroup per
// row as well.  Measured against the two-kernel path: fp16 [256, 65536]
// k0=32768 71 -> 38 us, [1024, 65536] 312 -> 142 us, [512, 262144] 184 -> 113 us,
// [128, 2^20] 90 -> 85 us, fp32 [256, 65536] k0=16384 52 -> 35 us, [2048, 131072]
// 375 -> 336 us.  (With eight waves the larger budget lost for rows beyond
// 256 KiB: [128, 2^20] 87 -> 115 us.)
constexpr size_t kLdsBudgetLarge = 128 * 1024;
// Most waves per workgroup.  Measured over shapes from [4096, 4096] to
// [256, 65536]: 8 beats 16 (more workgroups per CU, in different phases, and
// cheaper barriers) and is never far behind 4.
constexpr uint32_t kMaxWaves = 8;
// Corners in which the two-kernel path may be the faster one (see make_plan).
constexpr int64_t kManyRows = 1024, kAllCus = 256;
// Longest contiguous bucket (bytes) the register kernel takes.
constexpr int64_t kShortBucket = 256;
constexpr size_t kShortRow = 128 * 1024, kLongRow = 512 * 1024;
}  // namespace

// Staged results leave in non-temporal stores when the launch is one round of workgroups
// (no more rows than the GPU holds at once) and a row's results are an eighth of its bytes
// or more.  What a kernel has written sits in the L2 of its XCD until the kernel ends and
// is written back then, with nothing left to hide it behind: first workgroup's start to
// last store 22.8 us of fp16 [1024, 32768] k=2048 j=4 k_mult=4's 27.1 us per call.  Sent
// past the cache the results travel while other workgroups still work: 27.6 -> 25.4 us
// there, fp16 [256, 131072] k=4096 j=4 k_mult=2 22.2 -> 20.1 us, fp32 [512, 32768] k=2048
// j=4 k_mult=4 24.4 -> 23.1 us.  With several rounds the write-back hides behind the
// later rounds by itself and the stores past the cache cost more than they save ([4096,
// 8192] k=512 35.6 -> 36.9 us, [2048, 32768] 46.3 -> 47.3 us), as they do with little
// output ([1024, 65536] k=512 44.0 -> 45.1 us).
static bool stores_past_cache(int64_t rows, int64_t n, int64_t k, int64_t es) {
  return rows <= kManyRows && k * (es + 8) * 8 >= n * es;
}

// Contiguous buckets, all of one length of 16 to kShortBucket bytes, elements of
// two or four bytes: a lane of the register kernel loads its four buckets whole.  The
// alternative is a stage-1 kernel that copies spans of buckets through LDS and
// parks the candidates in HBM for a stand-alone select: fp16 [1024, 32768]
// k=2048 j=4 k_mult=4 (buckets of 32 bytes) 68.6 us that way against 35; buckets of
// 128 bytes fp16 [256, 131072] k0=8192 39.2 against 33.3 us, fp32 [64, 32768] k0=2048
// 17.4 against 12.7 us; of 256 bytes fp16 [256, 262144] k0=8192 57.6 against 49.4 us,
// [1024, 131072] 109.9 against 110.3 us.
static Plan plan_short_buckets(int64_t rows, int64_t n, int64_t k0, int j, int64_t k, int dtype, bool aligned) {
  Plan pl{};
  pl.ok = false;
  if (!aligned || rows > 0x7fffffffll) return pl;
  if (k0 <= 0 || k <= 0 || k >= k0 || j < 1 || j > 4 || k0 % j) return pl;
  const int es = elem_bytes(dtype);
  if (es != 2 && es != 4) return pl;
  // fewer rows than CUs: only rows one workgroup reads in a few microseconds (fp32 [130, 131072]
  // with 2048 buckets of 256 bytes: 38.4 us here against 32.4 through two kernels, whose stage 1
  // has sixteen workgroups per row)
  if (rows < kAllCus && (size_t)n * es > kSoloRow) return pl;
  const int64_t b = k0 / j;
  if (n % b) return pl;
  const int64_t m = n / b;
  if ((m * es) % 16 || m * es > kShortBucket || m < j) return pl;
  pl.full_rows = (uint32_t)m;
  pl.pos16 = true;
  pl.packed = es == 2;
  pl.vec = 4;
  // whole tiles only: a lane's buckets lie a wave's width apart
  if (b % (stream::kWave * pl.vec)) return pl;
  pl.tiles = (uint32_t)(b / (stream::kWave * pl.vec));
  if (pl.tiles > kMaxWaves) return pl;
  pl.index_bits = 1;
  while (pl.index_bits < 63 && (1ll << pl.index_bits) < n) ++pl.index_bits;
  pl.split = 1;
  pl.waves = pl.tiles;
  pl.contig = pl.in_registers = true;
  const size_t cand_bytes = (((size_t)k0 * es + 15) & ~(size_t)15) + (((size_t)k0 * 2 + 15) & ~(size_t)15);
  pl.lds_bytes = cand_bytes > regs::kLdsBytes ? cand_bytes : regs::kLdsBytes;
  pl.staged = (size_t)k * 8 <= kLdsBudget;
  if (pl.staged && pl.lds_bytes < (size_t)k * 8) pl.lds_bytes = (size_t)k * 8;
  pl.past_cache = pl.staged && stores_past_cache(rows, n, k, es);
  pl.ok = true;
  return pl;
}

Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int64_t k, int layout, int dtype, bool aligned) {
  Plan pl{};
  pl.ok = false;
  if (layout == ATK_BALANCED) return plan_short_buckets(rows, n, k0, j, k, dtype, aligned);
  // (a padded row is never reduced further: its callers keep every bucket)
  if (layout != ATK_INTERLEAVED) return pl;
  if (!aligned || rows > 0x7fffffffll) return pl;
  if (k0 <= 0 || k <= 0 || k >= k0 || j < 1 || j > 4 || k0 % j) return pl;
  const int es = elem_bytes(dtype);
  if (!es) return pl;
  if (rows < kMinRows && (size_t)n * es > kSoloRow) return pl;
  const int64_t b = k0 / j;
  const int64_t full = n / b;
  if (full < j || full > 0x7fffffffll) return pl;
  pl.full_rows = (uint32_t)full;
  pl.rem = (uint32_t)(n - full * b);
  pl.pad_tail = 0;
  pl.pos16 = full + 1 <= 0xffff;
  pl.packed = (dtype == ATK_F16 || dtype == ATK_BF16 || dtype == ATK_I16) && full <= stream::kPackedMaxSubRow;
  pl.vec = stream::full_vec(es);
  // packed queues at half the load width need about 50 VGPRs instead of 127:
  // twice the workgroups per CU, which is worth more here than 16-byte loads
  if (pl.packed) pl.vec /= 2;
  if (b % pl.vec) return pl;
  const int64_t bound = (full + 1) * b;  // indices are < this
  pl.index_bits = 1;
  while (pl.index_bits < 63 && (1ll << pl.index_bits) < bound) ++pl.index_bits;

  const int64_t tile_cols = (int64_t)stream::kWave * pl.vec;
  pl.tiles = (uint32_t)((b + tile_cols - 1) / tile_cols);
  // Few buckets: a sub-row of b elements is all a wave loads at a time here
  // (this kernel does not fold sub-rows side by side as the streaming kernel
  // does), so with narrow sub-rows most lanes idle and the few that work walk
  // the whole row.  Measured against the two-kernel path (fp16 and fp32, 8-256
  // buckets, k_mult = 2): fp16 [256, 2^22] with 8 buckets 10.2 ms against
  // 0.36 ms, [2048, 8192] with 32 buckets 29 against 14 us, while rows of a few
  // KiB still gain from the saved launch (5.5 against 7.7 us).  The sub-row a
  // call needs grows with the row and with the number of rows.  Batches of up to
  // 1 MiB in all are bound by launches, not by bytes: there this kernel takes
  // 5 us + 11 ns per sub-row of the row ([4, 32768] with 4 buckets: 94-118 us)
  // against 8-15 us for the two kernels whatever the shape, and narrow sub-rows
  // are taken while the row has fewer than 256 of them.
  {
    const size_t sub_row_bytes = (size_t)b * es, row_bytes_ = (size_t)n * es;
    size_t least = 128;
    if (row_bytes_ > 16 * 1024) least = 256;
    if (row_bytes_ > 32 * 1024 || rows >= 2048) least = 512;
    const bool small_batch = (size_t)rows * row_bytes_ <= (1u << 20);
    if (sub_row_bytes < least && (!small_batch || full >= 256)) return pl;
  }
  // One launch instead of two, and no candidates parked in HBM: measured over
  // 128-4096 rows of 8192-262144 elements with 256-4096 candidates, this kernel
  // is 5-40 % faster than the two-kernel path for the packed 16-bit types
  // throughout and for wider types except in two corners: many short rows
  // (>= 1024 rows of < 128 KiB: +5-35 %; the stand-alone select runs more rows
  // per CU) and fewer rows than CUs with j >= 3 and rows of >= 512 KiB (+10-30 %;
  // the two-kernel path cuts such rows into slabs).  There, and for 1-byte
  // types (whose packed queues only the streaming kernel has), it is taken only
  // when parking the candidates would cost a good part of what reading the row
  // costs: written and re-read k0*(es+8) bytes against n*es.
  const size_t row_bytes = (size_t)n * es;
  const bool corner = es == 1 || (!pl.packed && ((rows >= kManyRows && row_bytes < kShortRow) ||
                                                 (rows < kAllCus && j >= 3 && row_bytes >= kLongRow)));
  if (corner && (size_t)k0 * (es + 8) * 4 < row_bytes) return pl;
  const int skey = (dtype == ATK_U8 || dtype == ATK_I8) ? 2 : es;  // stored key width
  const size_t cand_bytes = (((size_t)k0 * skey + 15) & ~(size_t)15) +
                            (((size_t)k0 * (pl.pos16 ? 2 : 4) + 15) & ~(size_t)15);
  const size_t lds_budget = kLdsBudgetLarge;
  if (cand_bytes > lds_budget) return pl;

  // With more than the usual LDS budget taken, or with no more rows than CUs, one
  // workgroup has the CU to itself: sixteen waves then, when eight would go through
  // the tiles in several rounds (the scan and the selection both gain: fp16
  // [256, 65536] k0=16384 32.8 -> 25.8 us, [200, 32768] k0=16384 30.3 -> 22.7 us; with
  // 300-512 rows eight waves stay ahead, 43 against 49 us at [512, 65536]).
  const uint32_t max_waves =
      (cand_bytes > kLdsBudget || (rows <= kAllCus && pl.tiles > kMaxWaves)) ? 2 * kMaxWaves : kMaxWaves;
  // Waves sharing a tile: as many as keep each share at least max(j, 8)
  // sub-rows long, the workgroup within its wave limit and LDS within budget.
  // When all tiles are in flight at once the hand-over area may lie on top of
  // the candidates.
  const int cmp_size = es > 4 ? 8 : 4;
  const int64_t min_run = j > 8 ? j : 8;
  auto hand_bytes = [&](uint32_t split) {
    const uint32_t waves = pl.tiles * split <= max_waves ? pl.tiles * split : max_waves;
    return (size_t)(waves - waves / split) * pl.vec * j * stream::kWave * (cmp_size + 4);
  };
  auto lds_need = [&](uint32_t split) {
    const bool one_round = pl.tiles * split <= max_waves;
    const size_t hand = hand_bytes(split);
    return one_round ? (hand > cand_bytes ? hand : cand_bytes) : cand_bytes + hand;
  };
  uint32_t split = 1;
  if (pl.tiles < max_waves) {
    for (uint32_t cand = 2; cand * pl.tiles <= max_waves; cand *= 2) {
      if (full / cand < min_run || lds_need(cand) > lds_budget) break;
      split = cand;
    }
  }
  pl.split = split;
  pl.waves = pl.tiles * split <= max_waves ? pl.tiles * split : max_waves;
  const bool one_round = pl.tiles * split <= max_waves;
  pl.hand_off = (split > 1 && !one_round) ? (uint32_t)cand_bytes : 0u;
  pl.lds_bytes = lds_need(split);
  // every tile has its waves: stage 2 runs on the candidates where they are, in
  // registers, and needs the histogram's room in LDS
  pl.in_registers = one_round && pl.waves <= kMaxWaves;  // (the register kernel is built for eight waves)
  if (pl.in_registers && pl.lds_bytes < regs::kLdsBytes) pl.lds_bytes = regs::kLdsBytes;
  // survivors staged in LDS, eight bytes each (element, 32-bit index), when that fits
  pl.staged = pl.in_registers && pl.pos16 && es <= 4 && (size_t)k * 8 <= kLdsBudget;
  if (pl.staged && pl.lds_bytes < (size_t)k * 8) pl.lds_bytes = (size_t)k * 8;
  pl.past_cache = pl.staged && stores_past_cache(rows, n, k, es);
  pl.ok = true;
  return pl;
}

}  // namespace fused

namespace {
fused::Plan plan_for(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
                     int layout, int dtype) {
  const int es = elem_bytes(dtype);
  const int vf = es ? stream::full_vec(es) : 1;
  const bool aligned = ((uintptr_t)x % 16 == 0) && (row_stride % vf == 0);
  return fused::make_plan(rows, n, k0, j, k, layout, dtype, aligned);
}
}  // namespace

bool fused_row_takes(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
                     int layout, int dtype) {
  return plan_for(x, rows, n, row_stride, k0, j, k, layout, dtype).ok;
}

bool describe_fused_row(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
                        int layout, int dtype, std::string& out) {
  const fused::Plan pl = plan_for(x, rows, n, row_stride, k0, j, k, layout, dtype);
  if (!pl.ok) return false;
  out += std::string(pl.in_registers ? "fused_regs_kernel<" : "fused_row_kernel<") + dtype_name(dtype) + ", J=" +
         std::to_string(j) + ", V=" + std::to_string(pl.vec) + ", pos" + (pl.pos16 ? "16" : "32") +
         ", PACKED=" + (pl.packed ? "1" : "0") + "> grid=" + std::to_string(rows) + " block=" +
         std::to_string(64 * pl.waves) + " tiles=" + std::to_string(pl.tiles) + " split=" + std::to_string(pl.split) +
         " lds=" + std::to_string(pl.lds_bytes) + (pl.in_registers && pl.staged ? (pl.past_cache ? " staged past-cache" : " staged") : "") +
         (pl.contig ? " short contiguous buckets" : "");
  return true;
}

int launch_fused_row(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                     int64_t k, int layout, int dtype, void* values, IndexOut indices, hipStream_t stream,
                     bool* handled) {
  const fused::Plan pl = plan_for(x, rows, n, row_stride, k0, j, k, layout, dtype);
  *handled = pl.ok;
  if (!pl.ok) return ATK_OK;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = fused::launch_typed<E>(pl, x, rows, row_stride, k0, j, k, values, indices, stream));
  return rc;
}

}  // namespace atk
