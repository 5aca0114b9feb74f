// extern "C" entry points of libapprox_topk_hip.so: argument checks and the
// choice of kernel.  Everything here runs on the host and only enqueues work.
#include <mutex>
#include <string>

#include "atk_device.h"
#include "atk_launch.h"

namespace {

constexpr int kAbiVersion = 3;

// Scratch memory of atk_topk_noalloc: one array per GPU, part of the loaded
// code object, held until the process ends.  In host code the array's name is
// only a handle for hipGetSymbolAddress; the device address it yields (one per
// device) is what kernels, through do_topk's workspace argument, are given.
constexpr size_t kScratchBytes = ATK_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// The current device's copy of `scratch`; looked up once per device.
int scratch_of_current_device(void** out) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return ATK_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return ATK_ERR_LAUNCH;
    g_scratch_ptr[device] = ptr;
  }
  *out = g_scratch_ptr[device];
  return ATK_OK;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Data pointers must be aligned to what they point at (elements, indices of
// the chosen width), a workspace to 16 bytes: the kernels carve 8-byte
// candidate indices and 16-byte vectors out of it.
constexpr uintptr_t kWorkspaceAlign = 16;
inline bool aligned_to(const void* p, size_t a) { return (uintptr_t)p % a == 0; }
int check_alignment(const void* x, const void* values, int dtype, atk::IndexOut indices, const void* ws) {
  const size_t es = (size_t)atk::elem_bytes(dtype);
  if (!aligned_to(x, es) || !aligned_to(values, es) || !aligned_to(indices.base, indices.narrow ? 4 : 8))
    return ATK_ERR_ALIGN;
  if (ws && !aligned_to(ws, kWorkspaceAlign)) return ATK_ERR_ALIGN;
  return ATK_OK;
}

int check_stage1(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0,
                 int j, int layout, int dtype, const void* values, const void* indices) {
  if (atk::elem_bytes(dtype) == 0) return ATK_ERR_DTYPE;
  if (layout < ATK_INTERLEAVED || layout > ATK_INTERLEAVED_PADDED) return ATK_ERR_LAYOUT;
  if (rows < 0 || n < 0 || k0 < 0) return ATK_ERR_K;
  if (k0 == 0 || rows == 0) return ATK_OK;
  if (j < 1 || j > 4 || k0 % j) return ATK_ERR_J;
  const bool padded = layout == ATK_CEIL_CHUNK || layout == ATK_INTERLEAVED_PADDED;
  if (padded && j != 1) return ATK_ERR_LAYOUT;
  if (padded ? n < 1 : k0 > n) return ATK_ERR_K;
  if (!x || !indices || row_stride < n) return ATK_ERR_ARG;  // (values may be NULL: indices only)
  return ATK_OK;
}

// Workspace of atk_topk: the stage-1 candidates, then stage 1's own scratch,
// then stage 2's.
struct TopkPlan {
  size_t cand_values_off, cand_indices_off, stage1_off, stage1_bytes, select_off, select_bytes, total;
};

TopkPlan plan_topk(int64_t rows, int64_t n, int64_t k0, int j, int64_t k, int layout, int dtype) {
  TopkPlan p{0, 0, 0, 0, 0, 0, 0};
  if (rows <= 0 || k0 <= 0) return p;
  p.stage1_bytes = atk_stage1_workspace_bytes(rows, n, k0, j, layout, dtype);
  if (k == k0) {
    p.total = p.stage1_bytes;
    return p;
  }
  const size_t vals = align_up((size_t)rows * (size_t)k0 * atk::elem_bytes(dtype), 256);
  p.cand_indices_off = vals;
  p.stage1_off = vals + align_up((size_t)rows * (size_t)k0 * sizeof(int64_t), 256);
  p.select_off = p.stage1_off + align_up(p.stage1_bytes, 256);
  p.select_bytes = atk_select_workspace_bytes(rows, k0, k, dtype);
  p.total = p.select_off + p.select_bytes;
  return p;
}

// Stage 1 through the streaming kernels when they take the shape, else the
// general kernel.
int run_stage1(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
               int layout, int dtype, void* values, atk::IndexOut indices, void* ws, size_t ws_bytes,
               hipStream_t stream, atk::KeyRangeOut* ranges = nullptr) {
  bool handled = false;
  const int rc = atk::launch_stage1_stream(x, rows, n, row_stride, k0, j, layout, dtype, values,
                                           indices, ws, ws_bytes, stream, &handled, ranges);
  if (handled || rc != ATK_OK) return rc;
  const int rc2 = atk::launch_stage1_contig(x, rows, n, row_stride, k0, j, layout, dtype, values, indices,
                                            ws, ws_bytes, stream, &handled);
  if (handled || rc2 != ATK_OK) return rc2;
  return atk::launch_stage1_lane_per_bucket(x, rows, n, row_stride, k0, j, layout, dtype, values,
                                            indices, stream);
}

// Stage 2 over many workgroups per row when a row holds very many candidates,
// else one workgroup per row.
int run_select(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0, int64_t k,
               int64_t index_bound, int dtype, void* values, atk::IndexOut indices, void* ws, size_t ws_bytes,
               hipStream_t stream, uint32_t range_entries = 0, bool hist_done = false) {
  bool handled = false;
  const int rcc = atk::launch_chain_select(cand_values, cand_indices, rows, k0, k, index_bound, dtype, values,
                                           indices, ws, ws_bytes, range_entries, hist_done, stream, &handled);
  if (handled || rcc != ATK_OK) return rcc;
  const int rc = atk::launch_multi_select(cand_values, cand_indices, rows, k0, k, index_bound, dtype, values,
                                          indices, ws, ws_bytes, stream, &handled);
  if (handled || rc != ATK_OK) return rc;
  return atk::launch_select(cand_values, cand_indices, rows, k0, k, index_bound, dtype, values, indices,
                            ws, ws_bytes, stream);
}

// Positions a layout can report: the row, or the padded row of the arg-max layouts.
int64_t index_bound_of(int64_t n, int64_t k0, int layout) {
  return (layout == ATK_CEIL_CHUNK || layout == ATK_INTERLEAVED_PADDED) ? ((n + k0 - 1) / k0) * k0 : n;
}

// int32 indices must be able to hold every position.
bool fits_narrow(int64_t n, int64_t k0, int layout) { return index_bound_of(n, k0, layout) <= 0x7fffffffll; }

int do_stage1(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int layout,
              int dtype, void* values, atk::IndexOut indices, void* ws, size_t ws_bytes, hipStream_t stream) {
  const int rc = check_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, indices.base);
  if (rc != ATK_OK || k0 == 0 || rows == 0) return rc;
  if (indices.narrow && !fits_narrow(n, k0, layout)) return ATK_ERR_TOO_LARGE;
  if (const int rca = check_alignment(x, values, dtype, indices, ws); rca != ATK_OK) return rca;
  const size_t need = atk_stage1_workspace_bytes(rows, n, k0, j, layout, dtype);
  if (need && (!ws || ws_bytes < need)) return ATK_ERR_WORKSPACE;
  return run_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, indices, ws, ws_bytes, stream);
}

int do_topk(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
            int layout, int dtype, void* values, atk::IndexOut indices, void* ws, size_t ws_bytes,
            hipStream_t stream) {
  if (k < 0 || k > k0) return ATK_ERR_K;
  const int rc = check_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, indices.base);
  if (rc != ATK_OK || k == 0 || rows == 0) return rc;
  if (k == k0) return do_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, indices, ws, ws_bytes, stream);
  if (indices.narrow && !fits_narrow(n, k0, layout)) return ATK_ERR_TOO_LARGE;
  if (const int rca = check_alignment(x, values, dtype, indices, ws); rca != ATK_OK) return rca;
  {
    bool handled = false;
    const int rcf = atk::launch_fused_row(x, rows, n, row_stride, k0, j, k, layout, dtype, values,
                                          indices, stream, &handled);
    if (handled || rcf != ATK_OK) return rcf;
  }
  const TopkPlan p = plan_topk(rows, n, k0, j, k, layout, dtype);
  if (!ws || ws_bytes < p.total) return ATK_ERR_WORKSPACE;
  unsigned char* base = static_cast<unsigned char*>(ws);
  void* cand_values = base + p.cand_values_off;
  int64_t* cand_indices = reinterpret_cast<int64_t*>(base + p.cand_indices_off);
  // a chained select can take the key ranges of the candidates from stage 1's last kernel
  atk::KeyRangeOut ranges = atk::chain_select_ranges(rows, k0, k, index_bound_of(n, k0, layout), dtype,
                                                      base + p.select_off, p.select_bytes);
  // the candidates keep int64 indices whatever the output's width
  const int rc1 = run_stage1(x, rows, n, row_stride, k0, j, layout, dtype, cand_values,
                             atk::IndexOut{cand_indices, 0}, base + p.stage1_off, p.stage1_bytes, stream, &ranges);
  if (rc1 != ATK_OK) return rc1;
  return run_select(cand_values, cand_indices, rows, k0, k, index_bound_of(n, k0, layout), dtype, values,
                    indices, base + p.select_off, p.select_bytes, stream, ranges.entries, ranges.hist_done != 0);
}

}  // namespace

extern "C" {

int atk_version(void) { return kAbiVersion; }

const char* atk_strerror(int status) {
  switch (status) {
    case ATK_OK: return "ok";
    case ATK_ERR_DTYPE: return "unsupported element type";
    case ATK_ERR_J: return "topk: j must satisfy 0 < j < 5 and j must divide k";
    case ATK_ERR_K: return "topk: k must not be larger than topk size";
    case ATK_ERR_LAYOUT: return "unknown bucket layout, or a padded layout with j != 1";
    case ATK_ERR_WORKSPACE: return "workspace missing or too small";
    case ATK_ERR_LAUNCH: return "HIP kernel launch failed";
    case ATK_ERR_ARG: return "invalid pointer or stride argument";
    case ATK_ERR_TOO_LARGE: return "topk: too many buckets or slices, or positions beyond 32-bit indices";
    case ATK_ERR_SCRATCH:
      return "atk_topk_noalloc: the call needs more scratch memory than the library holds "
             "(ATK_NOALLOC_SCRATCH_BYTES); use atk_topk with a caller workspace";
    case ATK_ERR_ALIGN:
      return "misaligned pointer: data needs its element size, indices their width, a workspace 16 bytes";
  }
  return "unknown status";
}

size_t atk_stage1_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype) {
  const size_t a = atk::stage1_stream_workspace_bytes(rows, n, k0, j, layout, dtype);
  const size_t c = atk::stage1_contig_workspace_bytes(rows, n, k0, j, layout, dtype);
  return a > c ? a : c;
}

int atk_stage1(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
               int layout, int dtype, void* values, int64_t* indices, void* ws,
               size_t ws_bytes, atk_stream_t stream) {
  return do_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, atk::IndexOut{indices, 0}, ws,
                   ws_bytes, (hipStream_t)stream);
}

int atk_stage1_i32(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                   int layout, int dtype, void* values, int32_t* indices, void* ws,
                   size_t ws_bytes, atk_stream_t stream) {
  return do_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, atk::IndexOut{indices, 1}, ws,
                   ws_bytes, (hipStream_t)stream);
}

size_t atk_select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int dtype) {
  const size_t a = atk::multi_select_workspace_bytes(rows, k0, k, dtype);
  const size_t b = atk::select_workspace_bytes(rows, k0, k, dtype);
  const size_t c = atk::chain_select_workspace_bytes(rows, k0, k, 0, dtype);
  return a > b ? (a > c ? a : c) : (b > c ? b : c);
}

int atk_select(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0,
               int64_t k, int64_t index_bound, int dtype, void* values, int64_t* indices,
               void* ws, size_t ws_bytes, atk_stream_t stream) {
  if (atk::elem_bytes(dtype) == 0) return ATK_ERR_DTYPE;
  if (rows < 0 || k0 < 0 || k < 0 || k > k0 || index_bound < 0) return ATK_ERR_K;
  if (rows == 0 || k == 0) return ATK_OK;
  if (!cand_values || !cand_indices || !indices) return ATK_ERR_ARG;  // (values may be NULL: indices only)
  if (!aligned_to(cand_indices, 8)) return ATK_ERR_ALIGN;
  if (const int rca = check_alignment(cand_values, values, dtype, atk::IndexOut{indices, 0}, ws); rca != ATK_OK)
    return rca;
  return run_select(cand_values, cand_indices, rows, k0, k, index_bound, dtype, values,
                    atk::IndexOut{indices, 0}, ws, ws_bytes, (hipStream_t)stream);
}

size_t atk_topk_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j, int64_t k,
                                int layout, int dtype) {
  return plan_topk(rows, n, k0, j, k, layout, dtype).total;
}

size_t atk_topk_workspace_bytes_at(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0,
                                   int j, int64_t k, int layout, int dtype) {
  if (rows > 0 && k > 0 && k < k0 && check_stage1(x, rows, n, row_stride, k0, j, layout, dtype, x, x) == ATK_OK &&
      atk::fused_row_takes(x, rows, n, row_stride, k0, j, k, layout, dtype))
    return 0;
  return plan_topk(rows, n, k0, j, k, layout, dtype).total;
}

int atk_topk(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
             int64_t k, int layout, int dtype, void* values, int64_t* indices, void* ws,
             size_t ws_bytes, atk_stream_t stream) {
  return do_topk(x, rows, n, row_stride, k0, j, k, layout, dtype, values, atk::IndexOut{indices, 0}, ws,
                 ws_bytes, (hipStream_t)stream);
}

int atk_topk_i32(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                 int64_t k, int layout, int dtype, void* values, int32_t* indices, void* ws,
                 size_t ws_bytes, atk_stream_t stream) {
  return do_topk(x, rows, n, row_stride, k0, j, k, layout, dtype, values, atk::IndexOut{indices, 1}, ws,
                 ws_bytes, (hipStream_t)stream);
}

int atk_describe(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
                 int layout, int dtype, const void* values, const void* indices, char* text,
                 size_t text_bytes) {
  if (k < 0 || k > k0) return ATK_ERR_K;
  const int rc = check_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, indices);
  if (rc != ATK_OK) return rc;
  if (!text || text_bytes == 0) return ATK_ERR_ARG;
  std::string out;
  if (rows != 0 && k != 0) {
    bool fused = false;
    if (k < k0) fused = atk::describe_fused_row(x, rows, n, row_stride, k0, j, k, layout, dtype, out);
    if (!fused) {
      // the candidates of a two-stage call are written to the (aligned) workspace
      const void* v1 = k < k0 ? nullptr : values;
      const void* i1 = k < k0 ? nullptr : indices;
      if (!atk::describe_stage1_stream(x, rows, n, row_stride, k0, j, layout, dtype, v1, i1, out) &&
          !atk::describe_stage1_contig(x, rows, n, row_stride, k0, j, layout, dtype, out))
        atk::describe_stage1_lane_per_bucket(rows, k0, j, dtype, out);
      if (k < k0) {
        out += " + ";
        if (!atk::describe_chain_select(rows, k0, k, index_bound_of(n, k0, layout), dtype, out) &&
            !atk::describe_multi_select(rows, k0, k, index_bound_of(n, k0, layout), dtype, out))
          atk::describe_select(rows, k0, k, index_bound_of(n, k0, layout), dtype, true, out);
      }
    }
  }
  const size_t len = out.size() < text_bytes - 1 ? out.size() : text_bytes - 1;
  __builtin_memcpy(text, out.data(), len);
  text[len] = 0;
  return ATK_OK;
}

int atk_topk_noalloc(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                     int64_t k, int layout, int dtype, void* values, int64_t* indices,
                     atk_stream_t stream) {
  // the checks of do_topk that decide whether any workspace is needed come first,
  // so that an invalid call reports its own error rather than a size
  if (k < 0 || k > k0) return ATK_ERR_K;
  const int rc = check_stage1(x, rows, n, row_stride, k0, j, layout, dtype, values, indices);
  if (rc != ATK_OK || k == 0 || rows == 0) return rc;
  const size_t need = atk_topk_workspace_bytes_at(x, rows, n, row_stride, k0, j, k, layout, dtype);
  if (need > kScratchBytes) return ATK_ERR_SCRATCH;
  void* ws = nullptr;
  if (need != 0) {
    const int rcs = scratch_of_current_device(&ws);
    if (rcs != ATK_OK) return rcs;
  }
  return do_topk(x, rows, n, row_stride, k0, j, k, layout, dtype, values, atk::IndexOut{indices, 0}, ws,
                 need ? kScratchBytes : 0, (hipStream_t)stream);
}

}  // extern "C"
