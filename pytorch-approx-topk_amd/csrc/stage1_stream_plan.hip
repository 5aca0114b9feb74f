// Host-side planning and dispatch of the streaming stage-1 kernels.
#include "stage1_stream.h"

namespace atk {
namespace stream {

namespace {
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Waves wanted in the grid before a row is cut into slabs: one per SIMD of the
// 256 CUs x 4 SIMDs (each keeps 8 KiB of loads in flight).
constexpr int64_t kTargetWaves = 1024;
// Sub-rows worth giving to one wave before a row is also cut into slabs.
constexpr int64_t kSlabRun = 16;
// Fewest workgroups of a launch whose results take the trip through LDS.
constexpr int64_t kTransposeGroups = 2048;
// Sub-rows a wave keeps when a row is cut only to put a second wave on every SIMD.
constexpr int64_t kLongRun = 64;
// Fewest sub-rows a wave scans when several share a tile: with runs of 2 the
// hand-over costs more than the scan (measured at 16 sub-rows: 4 waves x 4 beat
// 8 x 2 by 25-45 %).
constexpr int64_t kMinRun = 4;
// Fewest sub-rows per wave for which a workgroup may take more LDS than kMergeLdsLimit.
constexpr int64_t kLongWaveRun = 16;
// Buckets at least this long are folded when they do not fill a column tile
// (measured down to 8: fp32 [32768, 1024] with 16 buckets 104 -> 22 us, bf16
// 193 -> 32 us; [65536, 256] with 16 buckets 70 -> 31 us).
constexpr int64_t kFoldMinLength = 8;
// Buckets from this length on are folded whatever the fold.
constexpr int64_t kFoldAnyLength = 128;
}  // namespace

Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype, bool aligned) {
  Plan pl{};
  pl.ok = false;
  if (layout != ATK_INTERLEAVED && layout != ATK_INTERLEAVED_PADDED) return pl;
  if (rows <= 0 || k0 <= 0 || j < 1 || j > 4 || k0 % j) return pl;
  const int es = elem_bytes(dtype);
  if (!es) return pl;
  const int64_t b = k0 / j;
  const int64_t length = n / b;  // elements every bucket has
  if (length < j || length > 0xfffffffell || b > 0x7fffffffll) return pl;
  const int vf = full_vec(es);

  // Few buckets: scan `fold` sub-rows side by side so that the lanes of a wave
  // are all busy (the largest fold that fits one column tile, keeps 16-byte
  // loads possible and leaves every scanned column j elements); the scanning
  // workgroup puts each bucket back together.
  int64_t fold = 1;
  if (length >= kFoldMinLength) {
    const int v = aligned ? vf : 1;
    int64_t f = (int64_t)kWave * v / b;
    while (f > 1 && ((b * f) % v != 0 || n / (b * f) < j)) --f;
    // short buckets: only when at least three lanes in four would idle (a fold of
    // two costs more in the merge than it gains: [128, 4096] with 128 buckets, j = 4, +23 %)
    if (f > 1 && (length >= kFoldAnyLength || f >= 4)) fold = f;
  }
  pl.fold = (uint32_t)fold;
  const int64_t width = b * fold;
  pl.width = width;
  const int64_t full = n / width;
  pl.full_rows = (uint32_t)full;
  pl.rem = (uint32_t)(n - full * width);
  pl.pad_tail = layout == ATK_INTERLEAVED_PADDED ? 1u : 0u;
  pl.vec = (aligned && width % vf == 0) ? vf : 1;
  pl.packed = ((dtype == ATK_F16 || dtype == ATK_BF16 || dtype == ATK_I16) && full <= kPackedMaxSubRow) ||
              ((dtype == ATK_U8 || dtype == ATK_I8) && full <= kByteMaxSubRow);

  const int64_t tile_cols = (int64_t)kWave * pl.vec;
  pl.col_tiles = (uint32_t)((width + tile_cols - 1) / tile_cols);

  // Waves per workgroup.  Wave 0's serial work per column is its own run,
  // full/w pushes, plus (w-1)*j pushes to fold the other waves' queues.  Take
  // the largest w within 30 % of the cheapest (short-lived waves keep more of
  // the HBM bandwidth: measured, 8 waves x 4 sub-rows beats 4 x 8 at the
  // headline shape), with every run at least max(j, 4) long and the LDS
  // hand-over within its budget.
  const int entry_bytes = pl.packed ? 4 : (es > 4 ? 8 : 4) + 4;
  int64_t cost[4] = {full, 0, 0, 0};
  int cands = 1;
  for (int cand = 2; cand <= 8; cand *= 2, ++cands) {
    const size_t hand = merge_lds_bytes(pl.vec, j, cand, entry_bytes);
    if (full / cand < (j > kMinRun ? j : kMinRun) || hand > merge_lds_limit(entry_bytes)) break;
    // Beyond the usual budget (packed queues of four entries, eight waves: 56 KiB, two workgroups
    // per CU) only for long runs.  Measured, fp16 [256, 2^20], j = 4: columns of 256 sub-rows
    // 125 -> 117 us, [1, 2^26] k = 16384 k_mult = 2 63 -> 47 us, but columns of 64 (runs of 8) 150 -> 162 us.
    if (hand > kMergeLdsLimit && full / cand < kLongWaveRun) break;
    cost[cands] = full / cand + (int64_t)(cand - 1) * j;
  }
  int64_t best = cost[0];
  for (int i = 1; i < cands; ++i) best = cost[i] < best ? cost[i] : best;
  int w = 1;
  for (int i = 0; i < cands; ++i)
    if (cost[i] * 10 <= best * 13) w = 1 << i;
  pl.waves = w;

  // Slabs: only when the grid would still be small and the runs are long.
  // Once a row is cut at all (the merge launch is then paid for anyway), short
  // queues (j <= 2, whose merge is cheap) are cut for twice as many waves:
  // measured 41 -> 28 us on fp32 [2, 2^24] with 4096 buckets, 57 -> 52 us on
  // [1, 2^26] with 16384 buckets at j = 2; j = 4 loses a little.
  pl.slabs = 1;
  const int64_t waves = rows * pl.col_tiles * w;
  const int64_t most = full / (w * kSlabRun);
  if (waves < kTargetWaves && most > 1) {
    const int64_t target = j <= 2 ? 2 * kTargetWaves : kTargetWaves;
    int64_t slabs = (target + waves - 1) / waves;
    if (slabs > most) slabs = most;
    pl.slabs = (uint32_t)slabs;
  }
  // Elements of one or two bytes cost twice or more the instructions per byte
  // loaded; a second wave per SIMD hides them, while every wave still has a
  // long run (measured on fp16 [128, 2^20] with 16 to 256 buckets: 87 -> 56 us
  // at j = 1, 120 -> 89 us at j = 4; with shorter runs the merge eats the gain).
  if (es <= 2) {
    int64_t slabs = (2 * kTargetWaves + waves - 1) / waves;
    const int64_t longest = full / (w * kLongRun);
    if (slabs > longest) slabs = longest;
    if (slabs > (int64_t)pl.slabs) pl.slabs = (uint32_t)slabs;
  }
  pl.slab_len = (uint32_t)(full / pl.slabs);
  // every wave scans exactly 4 or 8 sub-rows: straight-line kernels exist for that
  pl.run = 0;
  if (pl.vec > 1 && pl.slabs == 1 && full % pl.waves == 0) {
    const int64_t run = full / pl.waves;
    if ((run == 4 || run == 8) && run >= j) pl.run = (int)run;
  }
  // the slabs' queues (one per bucket: a workgroup merges the folded columns of
  // its slab itself) go to the workspace and the merge kernel follows
  pl.merge = pl.slabs > 1;
  if (pl.merge) {
    const size_t entries = (size_t)rows * pl.slabs * (size_t)b * (size_t)j;
    pl.part_values_off = 0;
    pl.part_pos_off = align_up(entries * es, 256);
    pl.ws_bytes = pl.part_pos_off + align_up(entries * sizeof(uint32_t), 256);
  }
  // Results through LDS in whole-wave stores (emit_transposed): when a lane's stretch of
  // the output is long (its indices 128 bytes or more) or its elements short, the launch
  // has workgroups by the thousand, and a workgroup writes at least an eighth of what it reads
  // (at a twelfth, fp16 [256, 2^20] k=16384: j=2 112.6 -> 115.1 us, j=4 118.2 -> 115.2 us, j=1 104.9 -> 102.5 us).
  pl.wave_stores = false;
  if (pl.vec > 1 && es <= 4 && !pl.merge && pl.fold == 1) {
    const int64_t entries = (int64_t)pl.vec * j;  // of a lane
    const bool whole_pieces = entries % 4 == 0 && entries % (16 / es) == 0 && j != 3;  // (Transposed::available)
    const int64_t groups = rows * (int64_t)pl.col_tiles;
    const int64_t in_bytes = full * kWave * pl.vec * es, out_bytes = kWave * entries * (es + 8);
    pl.wave_stores = whole_pieces && (entries * 8 >= 128 || es < 4) && groups >= kTransposeGroups &&
                     out_bytes * 8 >= in_bytes;
  }
  pl.ok = true;
  return pl;
}

}  // namespace stream

size_t stage1_stream_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype) {
  const stream::Plan a = stream::make_plan(rows, n, k0, j, layout, dtype, true);
  const stream::Plan u = stream::make_plan(rows, n, k0, j, layout, dtype, false);
  size_t need = 0;
  if (a.ok && a.ws_bytes > need) need = a.ws_bytes;
  if (u.ok && u.ws_bytes > need) need = u.ws_bytes;
  return need;
}

bool describe_stage1_stream(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                            int layout, int dtype, const void* values, const void* indices, std::string& out) {
  const int es = elem_bytes(dtype);
  const int vf = es ? stream::full_vec(es) : 1;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)values % 16 == 0) &&
                       ((uintptr_t)indices % 16 == 0) && (row_stride % vf == 0);
  const stream::Plan pl = stream::make_plan(rows, n, k0, j, layout, dtype, aligned);
  if (!pl.ok) return false;
  const int loads = stream::deep_loads_for_short_columns(dtype, j, pl.vec, pl.packed, pl.run, pl.full_rows)
                        ? 8
                        : stream::loads_in_flight(dtype, j, pl.vec, pl.packed);
  out += "stream_kernel<" + std::string(dtype_name(dtype)) + ", J=" + std::to_string(j) +
         ", V=" + std::to_string(pl.vec) + ", W=" + std::to_string(pl.waves) + ", U=" + std::to_string(loads) +
         ", RUN=" + std::to_string(pl.run) + ", PACKED=" + (pl.packed ? "1" : "0") + "> grid=" +
         std::to_string(rows * (int64_t)pl.slabs * pl.col_tiles) + " block=" + std::to_string(64 * pl.waves) +
         " fold=" + std::to_string(pl.fold) + " slabs=" + std::to_string(pl.slabs) +
         (pl.wave_stores ? " wave-stores" : "");
  if (pl.merge) out += " + stream_merge_kernel<" + std::string(dtype_name(dtype)) + ", J=" + std::to_string(j) + ">";
  return true;
}

int launch_stage1_stream(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                         int layout, int dtype, void* values, IndexOut indices, void* ws,
                         size_t ws_bytes, hipStream_t stream, bool* handled, KeyRangeOut* ranges) {
  const int es = elem_bytes(dtype);
  const int vf = es ? stream::full_vec(es) : 1;
  const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)values % 16 == 0) &&
                       ((uintptr_t)indices.base % 16 == 0) && (row_stride % vf == 0);
  const stream::Plan pl = stream::make_plan(rows, n, k0, j, layout, dtype, aligned);
  *handled = pl.ok;
  if (!pl.ok) return ATK_OK;
  if (pl.ws_bytes && (!ws || ws_bytes < pl.ws_bytes || (uintptr_t)ws % 16 != 0)) return ATK_ERR_WORKSPACE;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = stream::launch_typed<E>(pl, x, rows, row_stride, j, values, indices, ws,
                                                stream, ranges));
  return rc;
}

}  // namespace atk
