// Host-side launchers shared between the translation units of the library.
// Each returns an atk_status and only enqueues work on `stream`.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

#include "atk_device.h"

namespace atk {

// stage1_lane_per_bucket.hip: any dtype / layout / shape.
int launch_stage1_lane_per_bucket(const void* x, int64_t rows, int64_t n,
                                  int64_t row_stride, int64_t k0, int j, int layout,
                                  int dtype, void* values, IndexOut indices,
                                  hipStream_t stream);

// What stage 1 can leave behind for the chained select of stage2_chain_select.hip,
// which otherwise spends launches of its own on it: the smallest and largest
// order key of shares of every row's candidates (shares of a superset of them
// will do: the ranges only say which key bits all candidates have in common),
// that select's row states cleared, and its histogram either cleared or
// already filled with the candidates' digits (`want_hist`, set by the select's
// side: whether it has a use for that).  The stage-1 launcher sets `entries`:
// shares per row it wrote (0: it wrote nothing and cleared nothing), and
// `hist_done`: the histogram holds the candidates' digits.
struct KeyRangeOut {
  uint2* range;             // [rows][entries]
  uint32_t capacity;        // entries per row that fit
  uint32_t* hist;           // [rows][hist_words]
  uint32_t hist_words;
  uint32_t* state;          // [rows][state_words]
  uint32_t state_words;
  uint32_t want_hist;
  uint32_t entries;
  uint32_t hist_done;
};

// stage1_stream_plan.hip: interleaved layouts with at least j full sub-rows.
// `*handled` tells whether the shape was accepted; if not, nothing was enqueued.
size_t stage1_stream_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j, int layout,
                                     int dtype);
int launch_stage1_stream(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0,
                         int j, int layout, int dtype, void* values, IndexOut indices, void* ws,
                         size_t ws_bytes, hipStream_t stream, bool* handled, KeyRangeOut* ranges = nullptr);

// stage1_contig_plan.hip: the contiguous layouts, through LDS.  `*handled` as above.
size_t stage1_contig_workspace_bytes(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype);
int launch_stage1_contig(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                         int layout, int dtype, void* values, IndexOut indices, void* ws, size_t ws_bytes,
                         hipStream_t stream, bool* handled);

// Whether launch_fused_row takes this very call (the input's address and row
// stride decide with the shape).
bool fused_row_takes(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
                     int layout, int dtype);
// fused_row_plan.hip: both stages in one kernel, one workgroup per row, for
// batches of many rows whose candidates fit in LDS.  `*handled` as above.
int launch_fused_row(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                     int64_t k, int layout, int dtype, void* values, IndexOut indices,
                     hipStream_t stream, bool* handled);

// stage2_radix_select.hip: one workgroup per row.  With a workspace (see
// select_workspace_bytes) and few long rows, only the cut is found by that
// workgroup and the survivors are written by many (launch_emit_segments).
size_t select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int dtype);
int launch_select(const void* cand_values, const int64_t* cand_indices, int64_t rows,
                  int64_t k0, int64_t k, int64_t index_bound, int dtype, void* values,
                  IndexOut indices, void* ws, size_t ws_bytes, hipStream_t stream);

// stage2_chain_select.hip: few rows of thousands of candidates, several workgroups
// per row in a chain of three or four launches; needs a workspace.  `*handled` as above.
size_t chain_select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype);
// Where stage 1 may leave the key ranges for a chained select over workspace `ws`
// (range == nullptr when that select would not take the call).
KeyRangeOut chain_select_ranges(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, void* ws,
                                size_t ws_bytes);
// `range_entries`: shares per row stage 1 left in the workspace (see KeyRangeOut), or 0;
// `hist_done`: it also filled the histogram.
int launch_chain_select(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0, int64_t k,
                        int64_t index_bound, int dtype, void* values, IndexOut indices, void* ws, size_t ws_bytes,
                        uint32_t range_entries, bool hist_done, hipStream_t stream, bool* handled);

// stage2_multi_select.hip: writes the survivors of every segment of `seg`
// candidates (`groups` per row) in candidate order, given every row's cut
// (select::GlobalCut) and the survivors counted per segment.
int launch_emit_segments(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0,
                         int64_t k, uint32_t seg, uint32_t groups, const void* cuts, const uint32_t* counts,
                         int dtype, void* values, IndexOut indices, hipStream_t stream);

// stage2_multi_select.hip: many workgroups per row, for rows with very many
// candidates; needs a workspace.  `*handled` as above.
size_t multi_select_workspace_bytes(int64_t rows, int64_t k0, int64_t k, int dtype);
int launch_multi_select(const void* cand_values, const int64_t* cand_indices, int64_t rows, int64_t k0,
                        int64_t k, int64_t index_bound, int dtype, void* values, IndexOut indices, void* ws,
                        size_t ws_bytes, hipStream_t stream, bool* handled);

// The kernels each launcher above would enqueue for a call, as text appended to
// `out` ("name<parameters> grid=... block=..."; several kernels joined by " + ").
// The describe_* functions that return bool say whether their launcher takes
// the call; they enqueue nothing.
const char* dtype_name(int dtype);
bool describe_stage1_stream(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                            int layout, int dtype, const void* values, const void* indices, std::string& out);
bool describe_stage1_contig(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j,
                            int layout, int dtype, std::string& out);
void describe_stage1_lane_per_bucket(int64_t rows, int64_t k0, int j, int dtype, std::string& out);
bool describe_fused_row(const void* x, int64_t rows, int64_t n, int64_t row_stride, int64_t k0, int j, int64_t k,
                        int layout, int dtype, std::string& out);
bool describe_multi_select(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, std::string& out);
bool describe_chain_select(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, std::string& out);
void describe_select(int64_t rows, int64_t k0, int64_t k, int64_t index_bound, int dtype, bool with_workspace,
                     std::string& out);

}  // namespace atk
