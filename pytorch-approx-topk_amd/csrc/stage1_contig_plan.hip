// Host-side planning and dispatch of the contiguous-layout stage-1 kernel.
#include "stage1_contig.h"

namespace atk {
namespace contig {

namespace {
// Workgroups wanted in the grid before long buckets are left whole.
constexpr int64_t kTargetGroups = 1024;
}  // namespace

Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype, bool aligned) {
  Plan pl{};
  pl.ok = false;
  if (layout != ATK_BALANCED && layout != ATK_CEIL_CHUNK) return pl;
  if (rows <= 0 || n <= 0 || k0 <= 0 || j < 1 || j > 4 || k0 % j) return pl;
  const int es = elem_bytes(dtype);
  if (!es) return pl;
  const int64_t b = k0 / j;
  const int64_t m = layout == ATK_BALANCED ? n / b : (n + b - 1) / b;
  const int64_t r = layout == ATK_BALANCED ? n - m * b : 0;
  // every bucket holds at least j elements; positions fit 32 bits
  if (m < j || b > 0x7fffffffll || (double)b * (double)m + (double)r > 4294967294.0) return pl;
  const int64_t longest = m + (r > 0 ? 1 : 0);
  const int64_t piece = max_piece(es);

  Geom& g = pl.geom;
  g.n = n;
  g.b = (uint32_t)b;
  g.m = (uint32_t)m;
  g.r = (uint32_t)r;
  uint32_t lg = 0;
  while (lg < 8 && ((longest + (1ll << lg) - 1) >> lg) > piece) ++lg;
  // Few buckets: more threads per bucket (shorter pieces, more merge rounds)
  // as long as one workgroup still covers all of them and a piece keeps at
  // least four elements, so that the threads of the workgroup all scan.
  while (lg < 8 && (int64_t)(kThreads >> (lg + 1)) >= b && (m >> (lg + 1)) >= (j > 4 ? j : 4)) ++lg;
  g.pieces_log2 = lg;
  const int64_t per_thread = (longest + (1ll << lg) - 1) >> lg;
  if (per_thread > piece) {  // lg == 8: a workgroup per bucket, in chunks of 256 pieces
    g.chunks = (uint32_t)((longest + kThreads * piece - 1) / (kThreads * piece));
    g.trip = (uint32_t)piece;
  } else {
    g.chunks = 1;
    g.trip = (uint32_t)per_thread;
    g.sure = (uint32_t)(m >> lg);
  }
  const int64_t per_group = kThreads >> lg;
  g.groups = (uint32_t)((b + per_group - 1) / per_group);
  // Few rows of few very long buckets: share a bucket's chunks out over
  // workgroups (at least two chunks each, so that every workgroup starts on a
  // full chunk) until the grid has about kTargetGroups of them.
  g.slabs = 1;
  g.slab_chunks = g.chunks;
  if (g.chunks >= 4 && rows * b < kTargetGroups / 2) {
    int64_t slabs = (kTargetGroups + rows * b - 1) / (rows * b);
    if (slabs > g.chunks / 2) slabs = g.chunks / 2;
    if (slabs > 256) slabs = 256;
    g.slabs = (uint32_t)slabs;
    g.slab_chunks = g.chunks / g.slabs;
    g.groups = (uint32_t)(b * slabs);
    pl.ws_bytes = (size_t)rows * (size_t)b * (size_t)slabs * 4 * (es == 8 ? 16 : 8);
  }
  if (rows * (int64_t)g.groups > 0x7fffffffll) return pl;

  pl.vec = aligned ? stream::full_vec(es) : 1;
  // LDS: the longest span (whole packs, one element of slack) with its padding, or the queues
  const int64_t span = (g.chunks > 1 ? kThreads * piece : per_group * longest) + 2 * pl.vec + 2;
  const size_t data_bytes = (size_t)(span + ((span >> 5) + 1) * pad_elems(es)) * es;
  const size_t list_bytes = (size_t)4 * kThreads * (es == 8 ? 16 : 8);
  pl.lds_bytes = ((data_bytes > list_bytes ? data_bytes : list_bytes) + 15) / 16 * 16;
  // scan_even: buckets of one length, whole in the span, pieces of whole 16-byte packs, sub-row
  // numbers that fit the packed entries
  const int64_t per_pack = pl.vec;  // elements of a pack
  g.fast = 0;
  if (pl.vec > 1 && es <= 4 && r == 0 && g.chunks == 1 && (m >> lg) << lg == m && (m >> lg) % per_pack == 0 &&
      (m >> lg) >= per_pack && per_pack >= j && (es != 2 || m <= (int64_t)stream::kPackedMaxSubRow)) {
    const size_t packs = (size_t)(per_group * m) / per_pack;
    const size_t even_bytes = even_offset((uint32_t)packs, (uint32_t)(per_pack * es)) + 16;
    if (even_bytes <= 64 * 1024) {
      g.fast = 1;
      if (pl.lds_bytes < even_bytes) pl.lds_bytes = (even_bytes + 15) / 16 * 16;
    }
  }
  // whole_bucket_kernel: a lane per bucket, no LDS
  g.whole = 0;
  if (pl.vec > 1 && (es == 2 || es == 4) && r == 0 && (int64_t)b * m == n && (m * es) % 16 == 0 &&
      m * es <= (int64_t)kWholeBucket) {
    g.whole = 1;
    g.slabs = 1;
    pl.ws_bytes = 0;
    pl.lds_bytes = 0;
  }
  if (pl.lds_bytes > 64 * 1024) return pl;
  pl.ok = true;
  return pl;
}

}  // namespace contig

size_t stage1_contig_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype) {
  const contig::Plan a = contig::make_plan(rows, n, k0, j, layout, dtype, true);
  const contig::Plan u = contig::make_plan(rows, n, k0, j, layout, dtype, false);
  size_t need = 0;
  if (a.ok && a.ws_bytes > need) need = a.ws_bytes;
  if (u.ok && u.ws_bytes > need) need = u.ws_bytes;
  return need;
}

bool describe_stage1_contig(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                            int layout, int dtype, std::string& out) {
  const int es = elem_bytes(dtype);
  const int vf = es ? stream::full_vec(es) : 1;
  const bool aligned = ((uintptr_t)x % 16 == 0) && (row_stride % vf == 0);
  const contig::Plan pl = contig::make_plan(rows, n, k0, j, layout, dtype, aligned);
  if (!pl.ok) return false;
  if (pl.geom.whole) {
    out += "whole_bucket_kernel<" + std::string(dtype_name(dtype)) + ", J=" + std::to_string(j) + "> grid=" +
           std::to_string((rows * (int64_t)pl.geom.b + contig::kThreads - 1) / contig::kThreads) + " block=256";
    return true;
  }
  out += "contig_kernel<" + std::string(dtype_name(dtype)) + ", J=" + std::to_string(j) + ", V=" +
         std::to_string(pl.vec) + "> grid=" + std::to_string(rows * (int64_t)pl.geom.groups) + " block=256 chunks=" +
         std::to_string(pl.geom.chunks) + " slabs=" + std::to_string(pl.geom.slabs) +
         (pl.geom.fast ? " even" : "");
  if (pl.geom.slabs > 1) out += " + contig_merge_kernel<" + std::string(dtype_name(dtype)) + ", J=" + std::to_string(j) + ">";
  return true;
}

int launch_stage1_contig(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                         int layout, int dtype, void* values, IndexOut indices, void* ws, size_t ws_bytes,
                         hipStream_t stream, bool* handled) {
  const int es = elem_bytes(dtype);
  const int vf = es ? stream::full_vec(es) : 1;
  const bool aligned = ((uintptr_t)x % 16 == 0) && (row_stride % vf == 0);
  const contig::Plan pl = contig::make_plan(rows, n, k0, j, layout, dtype, aligned);
  *handled = pl.ok;
  if (!pl.ok) return ATK_OK;
  if (pl.ws_bytes && (!ws || ws_bytes < pl.ws_bytes || (uintptr_t)ws % 16 != 0)) return ATK_ERR_WORKSPACE;
  int rc = ATK_ERR_DTYPE;
  ATK_DTYPE_SWITCH(dtype, E, rc = ATK_ERR_DTYPE,
                   rc = contig::launch_typed<E>(pl, x, rows, row_stride, j, values, indices, ws, stream));
  return rc;
}

}  // namespace atk
