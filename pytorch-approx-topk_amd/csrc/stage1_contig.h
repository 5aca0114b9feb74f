// Stage 1 for the contiguous layouts (every bucket a run of adjacent elements).
//
// Reading a bucket front to back with one lane per bucket puts a whole bucket
// length between the addresses of neighbouring lanes.  Here a workgroup instead
// copies a span of whole buckets from the row into LDS with coalesced 16-byte
// loads and scans it from there: each of its 256 threads walks one *piece* of a
// bucket (at most 32 adjacent elements; 16 for 8-byte types) with a J-entry
// queue in registers, the P = 2^k threads that share a bucket combine their
// queues through LDS with the merge network of stage1_stream.h under the full
// order (value, then lower index), and the first of them writes the bucket's J
// entries.  A workgroup covers 256 / P adjacent buckets.  A bucket longer than
// 256 pieces takes a workgroup of its own, which goes through it in chunks of
// 256 pieces; a thread's queue then lives across the chunks (its pieces come
// in increasing position, so a newcomer still only displaces what it beats
// strictly).  When that leaves too few workgroups for the GPU (few rows of few,
// very long buckets), a bucket's chunks are shared out over `slabs` workgroups,
// which park their J best as merge words in a workspace, and
// `contig_merge_kernel` (one wave per bucket) combines them.
//
// LDS placement.  Element i of the span sits at i + i/32 words' worth of
// elements (one 4-byte word of padding per 32 elements): the 4-byte writes of a
// 16-byte pack stay adjacent, and threads that read with a stride of one piece
// (any length, powers of two included) spread over the banks.
//
// Values.  Floating-point elements are compared in IEEE form, and the copy into
// LDS tests every element for NaN; a workgroup that finds one starts over with
// the integer order keys of atk_device.h (NaN above +inf, all NaN equal).
// Positions >= n (the padded arg-max layout) hold the pad element.
#pragma once

#include "stage1_stream.h"

namespace atk {
namespace contig {

using stream::Cmp;
using stream::MergeWord;
using stream::Pack;

constexpr int kThreads = 256;
constexpr int kLoads = 8;  // loads one thread keeps in flight while a span is copied

// Longest piece one thread scans.
__host__ __device__ constexpr int max_piece(int elem_size) { return elem_size == 8 ? 16 : 32; }
// LDS elements of padding per 32 elements: one 4-byte word's worth.
__host__ __device__ constexpr int pad_elems(int elem_size) { return elem_size >= 4 ? 1 : 4 / elem_size; }

struct Geom {
  int64_t row_stride;    // elements between rows
  int64_t n;             // real elements per row; positions beyond hold the pad element
  uint32_t b;            // buckets per row
  uint32_t m;            // elements per bucket (balanced layout: of the shorter buckets)
  uint32_t r;            // balanced layout: the first r buckets hold m + 1 elements
  uint32_t pieces_log2;  // log2 of P, the threads per bucket
  uint32_t trip;         // the longest piece of any thread
  uint32_t sure;         // the shortest piece of any thread (one chunk; chunks but the last are full)
  uint32_t chunks;       // > 1: one bucket per workgroup, scanned in that many chunks
  uint32_t groups;       // workgroups per row
  uint32_t slabs;        // > 1 (only with chunks > 1): workgroups sharing a bucket's chunks
  uint32_t slab_chunks;  // least chunks per slab: slab s takes chunks [s * chunks / slabs, (s + 1) * chunks / slabs)
  uint32_t fast;         // the shape allows scan_even (see there)
  uint32_t whole;        // the shape allows whole_bucket_kernel (see there)
  uint32_t wide_out;     // the outputs allow 16-byte stores (filled in at launch)
};

// How a thread's queue holds values: in compare form (fast; no NaN may be
// present) or as order keys (exact).
template <typename E> struct CmpForm {
  using T = typename Cmp<E>::cmp_t;
  using M = MergeWord<E>;
  __device__ static __forceinline__ T conv(typename E::raw_t raw) { return Cmp<E>::from_raw(raw); }
  __device__ static __forceinline__ typename M::word_t word(T v, uint32_t p) { return M::make(Cmp<E>::to_raw(v), p); }
};
template <typename E> struct KeyForm {
  using T = typename E::key_t;
  using M = MergeWord<E>;
  __device__ static __forceinline__ T conv(typename E::raw_t raw) { return E::key(raw); }
  __device__ static __forceinline__ typename M::word_t word(T v, uint32_t p) { return M::from_key(v, p); }
};

template <typename E> __device__ __forceinline__ uint32_t lds_slot(uint32_t i) {
  return i + (i >> 5) * (uint32_t)pad_elems((int)sizeof(typename E::raw_t));
}

// One pass over the workgroup's buckets in form F.  Returns false, having
// written nothing, when F cannot order the data (a NaN in compare form).
template <typename E, int J, int V, typename F>
__device__ __forceinline__ bool scan_buckets(const typename E::raw_t* __restrict__ xr,
                                             typename E::raw_t* __restrict__ values,
                                             const IndexOut& indices, void* __restrict__ partial,
                                             int64_t row, uint32_t group, const Geom& g, unsigned char* lds) {
  using raw_t = typename E::raw_t;
  using T = typename F::T;
  using M = typename F::M;
  using word_t = typename M::word_t;
  constexpr int N = J == 3 ? 4 : J;
  constexpr bool kScreen = Cmp<E>::has_nan && std::is_same<F, CmpForm<E>>::value;
  constexpr uint32_t kChunk = kThreads * max_piece((int)sizeof(raw_t));
  raw_t* data = reinterpret_cast<raw_t*>(lds);

  const uint32_t t = threadIdx.x;
  const uint32_t pieces = 1u << g.pieces_log2;
  const uint32_t per_group = kThreads >> g.pieces_log2;  // buckets per workgroup
  const uint32_t slab = g.slabs > 1 ? group % g.slabs : 0u;
  const uint32_t c0 = g.slabs > 1 ? group / g.slabs : group * per_group;
  // the chunks of this workgroup
  // (shared out evenly: with the remainder all on the last slab, 1024 chunks over
  // 171 slabs left one workgroup 174 chunks and the others 5)
  const uint32_t it0 = g.slabs == 1 ? 0u : (uint32_t)(((uint64_t)slab * g.chunks) / g.slabs);
  const uint32_t it1 = g.slabs == 1 ? g.chunks : (uint32_t)(((uint64_t)(slab + 1) * g.chunks) / g.slabs);
  const uint32_t c = c0 + (t >> g.pieces_log2);
  const uint32_t piece = t & (pieces - 1);
  const bool has = c < g.b;
  auto start_of = [&](uint32_t bucket) -> uint32_t { return bucket * g.m + (bucket < g.r ? bucket : g.r); };
  const uint32_t start = start_of(c);
  const uint32_t len = g.m + (c < g.r ? 1u : 0u);
  const uint32_t c1 = c0 + per_group < g.b ? c0 + per_group : g.b;

  T q[J];
  uint32_t pos[J];
  for (uint32_t it = it0; it < it1; ++it) {
    // the span of this trip: all the workgroup's buckets, or one chunk of its only bucket
    uint32_t e0, e1;
    if (g.chunks == 1) {
      e0 = start_of(c0);
      e1 = start_of(c1);
    } else {
      e0 = start_of(c0) + it * kChunk;
      const uint32_t end = start_of(c0) + g.m + (c0 < g.r ? 1u : 0u);
      e1 = e0 + kChunk < end ? e0 + kChunk : end;
    }
    const uint32_t a0 = e0 & ~(uint32_t)(V - 1);  // packs are aligned in the row
    if (it != it0) __syncthreads();               // the last round's reads are done

    bool nan = false;
    const uint32_t packs = (e1 - a0 + V - 1) / V;
    auto park = [&](uint32_t pk, const Pack<raw_t, V>& got) __attribute__((always_inline)) {
      if constexpr (kScreen) {
        ATK_STATIC_FOR(h, V / 2) {
          nan |= __builtin_isunordered(F::conv(got.e[2 * h]), F::conv(got.e[2 * h + 1]));
        } ATK_STATIC_END;
        if constexpr (V % 2 != 0) nan |= __builtin_isunordered(F::conv(got.e[V - 1]), F::conv(got.e[V - 1]));
      }
      const uint32_t slot = lds_slot<E>(pk * V);  // the V elements of a pack stay adjacent
      if constexpr (V * sizeof(raw_t) % 4 == 0) {
        uint32_t words[V * sizeof(raw_t) / 4];
        __builtin_memcpy(words, &got, sizeof(words));
        uint32_t* dst = reinterpret_cast<uint32_t*>(data + slot);
        ATK_STATIC_FOR(w, (int)(V * sizeof(raw_t) / 4)) { dst[w] = words[w]; } ATK_STATIC_END;
      } else {
        ATK_STATIC_FOR(e, V) { data[slot + e] = got.e[e]; } ATK_STATIC_END;
      }
    };
    // packs that lie inside the row: kLoads loads in flight per thread
    const int64_t inside = (g.n - (int64_t)a0) / V;
    const uint32_t whole = inside <= 0 ? 0u : (inside < (int64_t)packs ? (uint32_t)inside : packs);
    for (uint32_t base = 0; base < whole; base += kThreads * kLoads) {
      Pack<raw_t, V> got[kLoads];
      ATK_STATIC_FOR(u, kLoads) {
        const uint32_t pk = base + u * kThreads + t;
        got[u] = stream::load_pack<raw_t, V>(xr + a0 + (size_t)(pk < whole ? pk : whole - 1) * V);
      } ATK_STATIC_END;
      ATK_STATIC_FOR(u, kLoads) {
        const uint32_t pk = base + u * kThreads + t;
        if (pk < whole) park(pk, got[u]);
      } ATK_STATIC_END;
    }
    // packs that reach past the row's end: the pad element beyond it
    for (uint32_t pk = whole + t; pk < packs; pk += kThreads) {
      const uint32_t at = a0 + pk * V;
      Pack<raw_t, V> got;
      ATK_STATIC_FOR(e, V) { got.e[e] = (int64_t)at + e < g.n ? xr[at + e] : E::pad_raw; } ATK_STATIC_END;
      park(pk, got);
    }
    if constexpr (kScreen) {
      if (__syncthreads_or(nan)) return false;
    } else {
      __syncthreads();
    }

    // this thread's piece [lo, hi) of its bucket
    uint32_t lo, hi;
    if (g.chunks == 1) {
      lo = (uint32_t)(((uint64_t)len * piece) >> g.pieces_log2);
      hi = (uint32_t)(((uint64_t)len * (piece + 1)) >> g.pieces_log2);
    } else {
      lo = it * kChunk + piece * (uint32_t)max_piece((int)sizeof(raw_t));
      hi = lo + (uint32_t)max_piece((int)sizeof(raw_t));
      lo = lo < len ? lo : len;
      hi = hi < len ? hi : len;
    }
    if (has) {
      const uint32_t count = hi - lo;
      const uint32_t first = start + lo;  // position in the row
      const uint32_t li = first - a0;     // position in the span
      uint32_t s = 0;
      if (it == it0) {  // every piece of a workgroup's first round holds at least J elements
        ATK_STATIC_FOR(u, J) {
          stream::push<T, J, u>(q, pos, F::conv(data[lds_slot<E>(li + u)]), first + u);
        } ATK_STATIC_END;
        s = J;
      }
      // every piece holds `sure` elements; only the few after that need a check
      const uint32_t sure = g.chunks == 1 ? g.sure : (it + 1 < g.chunks ? g.trip : 0u);
#pragma unroll 4
      for (; s < sure; ++s) {
        stream::push<T, J, J>(q, pos, F::conv(data[lds_slot<E>(li + s)]), first + s);
      }
      for (; s < g.trip; ++s) {
        const bool valid = s < count;
        const T v = F::conv(data[lds_slot<E>(li + (valid ? s : 0u))]);
        stream::push<T, J, J>(q, pos, valid ? v : q[0], first + s);  // q[0] beats nothing
      }
    }
  }

  // combine the pieces of every bucket
  word_t acc[N], in[N];
  ATK_STATIC_FOR(sl, N) { acc[sl] = M::empty(); in[sl] = M::empty(); } ATK_STATIC_END;
  if (has) {
    ATK_STATIC_FOR(sl, J) { acc[N - J + sl] = F::word(q[sl], pos[sl]); } ATK_STATIC_END;
  }
  if (pieces > 1) {
    __syncthreads();  // the span is no longer read: its LDS now carries the queues
    word_t* lists = reinterpret_cast<word_t*>(lds);  // [N][kThreads]
    for (uint32_t half = pieces / 2; half >= 1; half /= 2) {
      if (piece >= half && piece < 2 * half) {
        ATK_STATIC_FOR(sl, N) { lists[sl * kThreads + t] = acc[sl]; } ATK_STATIC_END;
      }
      __syncthreads();
      if (piece < half) {
        ATK_STATIC_FOR(sl, N) { in[sl] = lists[sl * kThreads + t + half]; } ATK_STATIC_END;
        stream::merge_best<M, N>(acc, in);
      }
    }
  }
  if (has && piece == 0) {
    if (g.slabs > 1) {
      word_t* park = reinterpret_cast<word_t*>(partial) + ((row * g.b + c) * g.slabs + slab) * N;
      ATK_STATIC_FOR(sl, N) { park[sl] = acc[sl]; } ATK_STATIC_END;
    } else {
      const int64_t o = (row * g.b + c) * J;
      ATK_STATIC_FOR(sl, J) {
        const uint32_t p = M::pos(acc[N - J + sl]);
        if (values != nullptr) values[o + sl] = (int64_t)p < g.n ? stream::element_of<E>(acc[N - J + sl], xr, p) : E::pad_raw;
        indices.put(o + sl, p);
      } ATK_STATIC_END;
    }
  }
  return true;
}

// LDS placement of scan_even: the span as the packs it was loaded in, 16 bytes of
// padding per 128, so that the 16-byte reads of threads whose pieces lie a multiple of 32
// words apart fall on different banks.
// (`pack_bytes`: 16, or 8 for the 1-byte types, which load eight elements at a time)
__host__ __device__ constexpr uint32_t even_offset(uint32_t pack, uint32_t pack_bytes) {
  return pack * pack_bytes + ((pack * pack_bytes) >> 7) * 16u;
}

// The same pass for the shapes that allow it, with the register queues of the
// streaming kernel (stage1_stream.h: one 32-bit word per entry for 8- and 16-bit
// types, one 64-bit word for fp32 with J >= 2; about half the instructions per
// element of the general form) and 16-byte LDS accesses: buckets of one length
// (no remainder), whole within the span (no chunks), 16-byte loads from the
// row, element types of at most four bytes, and pieces that are whole 16-byte
// packs, so that every thread reads aligned packs only.  Positions are kept
// relative to the bucket (packed entries hold 16 or 24 bits of them).  Returns
// false, having written nothing, when a NaN was met (the caller then runs the
// exact pass).
template <typename E, int J, int V, bool PACKED>
__device__ __forceinline__ bool scan_even(const typename E::raw_t* __restrict__ xr,
                                          typename E::raw_t* __restrict__ values, const IndexOut& indices,
                                          int64_t row, uint32_t group, const Geom& g, unsigned char* lds) {
  using raw_t = typename E::raw_t;
  using M = MergeWord<E>;
  using word_t = typename M::word_t;
  using Queue = stream::QueueFor<E, J, 1, PACKED>;
  constexpr int N = J == 3 ? 4 : J;
  constexpr uint32_t kPer = V;                                   // elements of a pack
  constexpr uint32_t kPackBytes = V * (uint32_t)sizeof(raw_t);   // 16, or 8 for the 1-byte types
  static_assert(V > 1 && sizeof(raw_t) <= 4 && V >= J, "whole packs, queues filled by the first");

  const uint32_t t = threadIdx.x;
  const uint32_t pieces = 1u << g.pieces_log2;
  const uint32_t per_group = kThreads >> g.pieces_log2;  // buckets per workgroup
  const uint32_t c0 = group * per_group;
  const uint32_t c = c0 + (t >> g.pieces_log2);
  const uint32_t piece = t & (pieces - 1);
  const bool has = c < g.b;
  const uint32_t c1 = c0 + per_group < g.b ? c0 + per_group : g.b;
  const uint32_t e0 = c0 * g.m, e1 = c1 * g.m;  // the span (e0 is a multiple of a pack)

  // the span into LDS, a pack per thread and trip, kLoads loads in flight
  const uint32_t packs = (e1 - e0) / kPer;
  const int64_t inside = (g.n - (int64_t)e0) / kPer;
  const uint32_t whole = inside <= 0 ? 0u : (inside < (int64_t)packs ? (uint32_t)inside : packs);
  for (uint32_t base = 0; base < whole; base += kThreads * kLoads) {
    Pack<raw_t, V> got[kLoads];
    ATK_STATIC_FOR(u, kLoads) {
      const uint32_t pk = base + u * kThreads + t;
      got[u] = stream::load_pack<raw_t, V>(xr + e0 + (size_t)(pk < whole ? pk : whole - 1) * V);
    } ATK_STATIC_END;
    ATK_STATIC_FOR(u, kLoads) {
      const uint32_t pk = base + u * kThreads + t;
      if (pk < whole) *reinterpret_cast<Pack<raw_t, V>*>(lds + even_offset(pk, kPackBytes)) = got[u];
    } ATK_STATIC_END;
  }
  for (uint32_t pk = whole + t; pk < packs; pk += kThreads) {  // packs that reach past the row's end
    const uint32_t at = e0 + pk * V;
    Pack<raw_t, V> got;
    ATK_STATIC_FOR(e, V) { got.e[e] = (int64_t)at + e < g.n ? xr[at + e] : E::pad_raw; } ATK_STATIC_END;
    *reinterpret_cast<Pack<raw_t, V>*>(lds + even_offset(pk, kPackBytes)) = got;
  }
  __syncthreads();

  // this thread's piece: `count` elements from position `first` of its bucket on
  const uint32_t count = g.m >> g.pieces_log2;
  const uint32_t first = piece * count;
  const uint32_t pack0 = ((c - c0) * g.m + first) / kPer;
  Queue queue;
  queue.reset();
  if (has) {
    auto pack_at = [&](uint32_t i) __attribute__((always_inline)) {
      return *reinterpret_cast<const Pack<raw_t, V>*>(lds + even_offset(pack0 + i, kPackBytes));
    };
    Pack<raw_t, V> cur = pack_at(0);
    ATK_STATIC_FOR(e, V) {
      queue.template take<(e < J ? e : J)>(Pack<raw_t, 1>{{cur.e[e]}}, first + e);
    } ATK_STATIC_END;
    const uint32_t trips = count / kPer;
    for (uint32_t i = 1; i < trips; ++i) {
      cur = pack_at(i);
      ATK_STATIC_FOR(e, V) { queue.template take<J>(Pack<raw_t, 1>{{cur.e[e]}}, first + i * kPer + e); } ATK_STATIC_END;
    }
  }
  if (__syncthreads_or(queue.poisoned())) return false;  // (also: the span is no longer read)

  // combine the pieces of every bucket
  const uint32_t start = c * g.m;
  word_t acc[N], in[N];
  ATK_STATIC_FOR(sl, N) { acc[sl] = M::empty(); in[sl] = M::empty(); } ATK_STATIC_END;
  if (has) {
    ATK_STATIC_FOR(sl, J) {
      acc[N - J + sl] = M::from_key(queue.template key<0, sl>(), start + queue.template position<0, sl>());
    } ATK_STATIC_END;
  }
  if (pieces > 1) {
    word_t* lists = reinterpret_cast<word_t*>(lds);  // [N][kThreads]
    for (uint32_t half = pieces / 2; half >= 1; half /= 2) {
      if (piece >= half && piece < 2 * half) {
        ATK_STATIC_FOR(sl, N) { lists[sl * kThreads + t] = acc[sl]; } ATK_STATIC_END;
      }
      __syncthreads();
      if (piece < half) {
        ATK_STATIC_FOR(sl, N) { in[sl] = lists[sl * kThreads + t + half]; } ATK_STATIC_END;
        stream::merge_best<M, N>(acc, in);
      }
    }
  }
  if (has && piece == 0) {
    const int64_t o = (row * g.b + c) * J;
    if constexpr (J == 2 || J == 4) {
      if (g.wide_out != 0) {  // a bucket's entries in one store of values and 16-byte stores of indices
        Pack<raw_t, J> pv;
        uint32_t p[J];
        ATK_STATIC_FOR(sl, J) {
          p[sl] = M::pos(acc[N - J + sl]);
          pv.e[sl] = (int64_t)p[sl] < g.n ? stream::element_of<E>(acc[N - J + sl], xr, p[sl]) : E::pad_raw;
        } ATK_STATIC_END;
        if (values != nullptr) *reinterpret_cast<Pack<raw_t, J>*>(values + o) = pv;
        if (indices.narrow) {
          Pack<int32_t, J> pi;
          ATK_STATIC_FOR(sl, J) { pi.e[sl] = (int32_t)p[sl]; } ATK_STATIC_END;
          *reinterpret_cast<Pack<int32_t, J>*>(static_cast<int32_t*>(indices.base) + o) = pi;
        } else {
          ATK_STATIC_FOR(h, J / 2) {
            Pack<int64_t, 2> pi;
            pi.e[0] = (int64_t)p[2 * h];
            pi.e[1] = (int64_t)p[2 * h + 1];
            reinterpret_cast<Pack<int64_t, 2>*>(static_cast<int64_t*>(indices.base) + o)[h] = pi;
          } ATK_STATIC_END;
        }
        return true;
      }
    }
    ATK_STATIC_FOR(sl, J) {
      const uint32_t p = M::pos(acc[N - J + sl]);
      if (values != nullptr) values[o + sl] = (int64_t)p < g.n ? stream::element_of<E>(acc[N - J + sl], xr, p) : E::pad_raw;
      indices.put(o + sl, p);
    } ATK_STATIC_END;
  }
  return true;
}

// E: element traits; J: entries kept per bucket; V: elements per load (16
// bytes' worth when the row allows it, else 1).
template <typename E, int J, int V>
__global__ __launch_bounds__(kThreads) void contig_kernel(const typename E::raw_t* __restrict__ x,
                                                          typename E::raw_t* __restrict__ values,
                                                          const IndexOut indices,
                                                          void* __restrict__ partial, const Geom g) {
  extern __shared__ __align__(16) unsigned char contig_lds[];
  const uint32_t row32 = blockIdx.x / g.groups;
  const uint32_t group = blockIdx.x - row32 * g.groups;
  const int64_t row = row32;
  const typename E::raw_t* xr = x + row * g.row_stride;
  bool done = false;
  if constexpr (V > 1 && sizeof(typename E::raw_t) <= 4) {
    if (g.fast != 0) {
      constexpr bool kPackable = stream::PackedKey<E>::available;
      done = scan_even<E, J, V, kPackable>(xr, values, indices, row, group, g, contig_lds);
      if (done) return;
      if constexpr (Cmp<E>::has_nan) {
        __syncthreads();
        scan_buckets<E, J, V, KeyForm<E>>(xr, values, indices, partial, row, group, g, contig_lds);
      }
      return;
    }
  }
  if (scan_buckets<E, J, V, CmpForm<E>>(xr, values, indices, partial, row, group, g, contig_lds)) return;
  if constexpr (Cmp<E>::has_nan) {
    __syncthreads();
    scan_buckets<E, J, V, KeyForm<E>>(xr, values, indices, partial, row, group, g, contig_lds);
  }
}

// Buckets of one length of 16 to kWholeBucket bytes (no remainder, rows that allow
// 16-byte loads, elements of two or four bytes): a lane per bucket.  The lane loads
// its bucket whole, 64 bytes of it at a time, 16 bytes a load -- neighbouring lanes
// hold neighbouring buckets, so the loads of a wave cover a stretch of the row back
// to back -- feeds it to a one-column register queue of the streaming kernel with
// the place within the bucket as the sub-row number, and writes the bucket's J
// entries; nothing goes through LDS and a row needs no workgroup of its own.  A NaN
// (a wave that met one) sends the wave's lanes through their buckets again with
// order keys.  Buckets are numbered row after row: lane t of workgroup w takes
// bucket w * kThreads + t of the rows * b there are.
constexpr uint32_t kWholeBucket = 64;

template <typename E, int J, bool PACKED>
__global__ __launch_bounds__(kThreads) void whole_bucket_kernel(const typename E::raw_t* __restrict__ x,
                                                                typename E::raw_t* __restrict__ values,
                                                                const IndexOut indices, const Geom g,
                                                                int64_t buckets) {
  using raw_t = typename E::raw_t;
  using Queue = stream::QueueFor<E, J, 1, PACKED>;
  constexpr int EPL = 16 / (int)sizeof(raw_t);  // elements per load
  constexpr int kMaxLoads = 4;                  // loads of a bucket issued together
  static_assert(EPL >= J && EPL % 2 == 0, "the first load of a bucket fills its queue");
  using Load = Pack<raw_t, EPL>;

  const int64_t at = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  const bool has = at < buckets;
  const int64_t mine = has ? at : buckets - 1;  // idle lanes go through the last bucket and write nothing
  int64_t row;
  uint32_t c;
  if (buckets <= 0xffffffffll) {
    const uint32_t row32 = (uint32_t)mine / g.b;
    row = row32;
    c = (uint32_t)mine - row32 * g.b;
  } else {
    row = mine / g.b;
    c = (uint32_t)(mine - row * g.b);
  }
  const raw_t* xr = x + row * g.row_stride;
  const raw_t* bucket = xr + (int64_t)c * g.m;
  const uint32_t loads = __builtin_amdgcn_readfirstlane(g.m / EPL);

  Queue queue;
  queue.reset();
  auto feed = [&](auto first_c, const Load (&buf)[kMaxLoads], uint32_t from, uint32_t count)
      __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(first_c)::value;  // the bucket's first loads: its queue fills
    ATK_STATIC_FOR(l, kMaxLoads) {
      if (l == 0 || (uint32_t)l < count) {
        ATK_STATIC_FOR(d, EPL / 2) {
          constexpr int kFilled = (kFirst && l == 0 && 2 * d < J) ? 2 * d : J;
          if constexpr (PACKED) {
            uint32_t pair;
            __builtin_memcpy(&pair, &buf[l].e[2 * d], 4);
            queue.template take_two<0, kFilled>(pair, from + l * EPL + 2 * d);
          } else {
            queue.template take_two<0, kFilled>(buf[l].e[2 * d], buf[l].e[2 * d + 1], from + l * EPL + 2 * d);
          }
        } ATK_STATIC_END;
      }
    } ATK_STATIC_END;
  };
  {
    Load buf[kMaxLoads];
#pragma unroll
    for (int l = 0; l < kMaxLoads; ++l) {
      if (l == 0 || (uint32_t)l < loads) buf[l] = stream::load_pack<raw_t, EPL>(bucket + l * EPL);
    }
    feed(std::true_type{}, buf, 0u, loads);
  }
#pragma nounroll
  for (uint32_t l0 = kMaxLoads; l0 < loads; l0 += kMaxLoads) {
    Load buf[kMaxLoads];
#pragma unroll
    for (int l = 0; l < kMaxLoads; ++l) {
      if (l == 0 || l0 + (uint32_t)l < loads) buf[l] = stream::load_pack<raw_t, EPL>(bucket + (l0 + l) * EPL);
    }
    feed(std::false_type{}, buf, l0 * EPL, loads - l0);
  }

  const int64_t o = (row * g.b + c) * J;
  const int64_t first_index = (int64_t)c * g.m;
  if (queue.poisoned()) {  // (wave-uniform)
    raw_t qv[J];
    uint32_t qp[J];
    stream::clear_exact<E, J>(qv, qp);
    for (uint32_t p = 0; p < g.m; ++p) stream::push_exact<E, J>(qv, qp, bucket[p], p);
    if (!has) return;
#pragma unroll
    for (int sl = 0; sl < J; ++sl) {
      if (values != nullptr) values[o + sl] = qv[sl];
      indices.put(o + sl, first_index + qp[sl]);
    }
    return;
  }
  queue.fix_zeros(xr, 1, first_index, 0);
  if (!has) return;
  if constexpr (J == 2 || J == 4) {
    if (g.wide_out != 0) {  // the outputs allow whole-bucket stores
      if (values != nullptr) {
        Pack<raw_t, J> pv;
        ATK_STATIC_FOR(sl, J) { pv.e[sl] = queue.template raw<0, sl>(); } ATK_STATIC_END;
        *reinterpret_cast<Pack<raw_t, J>*>(values + o) = pv;
      }
      if (indices.narrow) {
        Pack<int32_t, J> pi;
        ATK_STATIC_FOR(sl, J) { pi.e[sl] = (int32_t)(first_index + queue.template position<0, sl>()); } ATK_STATIC_END;
        *reinterpret_cast<Pack<int32_t, J>*>(static_cast<int32_t*>(indices.base) + o) = pi;
      } else {
        ATK_STATIC_FOR(t, J / 2) {
          Pack<int64_t, 2> pi;
          pi.e[0] = first_index + queue.template position<0, 2 * t>();
          pi.e[1] = first_index + queue.template position<0, 2 * t + 1>();
          reinterpret_cast<Pack<int64_t, 2>*>(static_cast<int64_t*>(indices.base) + o)[t] = pi;
        } ATK_STATIC_END;
      }
      return;
    }
  }
  ATK_STATIC_FOR(sl, J) {
    if (values != nullptr) values[o + sl] = queue.template raw<0, sl>();
    indices.put(o + sl, first_index + queue.template position<0, sl>());
  } ATK_STATIC_END;
}

// Combines the `slabs` partial results of every bucket: one wave per bucket,
// lane l folding slabs l, l + 64, ..., then pairwise by lane shuffles.
template <typename E, int J>
__global__ __launch_bounds__(64) void contig_merge_kernel(const typename E::raw_t* __restrict__ x,
                                                         const void* __restrict__ partial,
                                                         typename E::raw_t* __restrict__ values,
                                                         const IndexOut indices, const Geom g) {
  using M = MergeWord<E>;
  using word_t = typename M::word_t;
  constexpr int N = J == 3 ? 4 : J;
  const int64_t bucket = blockIdx.x;  // row * b + c
  const int64_t row = bucket / g.b;
  const uint32_t c = (uint32_t)(bucket - row * g.b);
  const uint32_t lane = threadIdx.x;
  const word_t* lists = reinterpret_cast<const word_t*>(partial) + bucket * g.slabs * N;
  word_t acc[N], in[N];
  ATK_STATIC_FOR(sl, N) { acc[sl] = M::empty(); } ATK_STATIC_END;
  for (uint32_t s = lane; s < g.slabs; s += 64) {
    ATK_STATIC_FOR(sl, N) { in[sl] = lists[(int64_t)s * N + sl]; } ATK_STATIC_END;
    stream::merge_best<M, N>(acc, in);
  }
  for (int half = 32; half >= 1; half /= 2) {
    ATK_STATIC_FOR(sl, N) { in[sl] = M::from_lane(acc[sl], (int)lane + half); } ATK_STATIC_END;
    stream::merge_best<M, N>(acc, in);  // meaningful in the lanes below `half`, which are the ones read next
  }
  if (lane != 0) return;
  const typename E::raw_t* xr = x + row * g.row_stride;
  const int64_t o = (row * g.b + c) * J;
  ATK_STATIC_FOR(sl, J) {
    const uint32_t p = M::pos(acc[N - J + sl]);
    if (values != nullptr) values[o + sl] = (int64_t)p < g.n ? stream::element_of<E>(acc[N - J + sl], xr, p) : E::pad_raw;
    indices.put(o + sl, p);
  } ATK_STATIC_END;
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
struct Plan {
  bool ok;
  int vec;           // V
  Geom geom;         // row_stride is filled in at launch
  size_t lds_bytes;  // dynamic LDS per workgroup
  size_t ws_bytes;   // workspace for the slabs' partial results
};

// `aligned`: base pointer and row stride allow 16-byte loads.
Plan make_plan(int64_t rows, int64_t n, int64_t k0, int j, int layout, int dtype, bool aligned);

template <typename E>
int launch_typed(const Plan& pl, const void* x, int64_t rows, int64_t row_stride, int j, void* values,
                 IndexOut indices, void* ws, hipStream_t stream);

}  // namespace contig
}  // namespace atk
