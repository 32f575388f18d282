// Device-side helpers shared by the attention forward and backward kernels.
//
// Register layouts used throughout (wave64, gfx950), verified on hardware:
//   v_mfma_f32_32x32x16 A (32 x 16): lane l holds row l%32, k = 8*(l/32) .. +7
//                       B (16 x 32): lane l holds col l%32, k = 8*(l/32) .. +7
//                       C (32 x 32): lane l holds col l%32, reg i is row
//                                    8*(i/4) + 4*(l/32) + i%4
//   ds_read_b64_tr_b16: within each group of 16 lanes, lane i supplies the
//                       address of 4 consecutive 16-bit elements; it receives
//                       element i%4 of lanes (i/4), 4+(i/4), 8+(i/4), 12+(i/4),
//                       i.e. column i of the 4 x 16 block whose row r is the
//                       concatenation of lanes 4r .. 4r+3.
#pragma once

#include "rswa_common.h"

#include <type_traits>
#include <utility>

namespace rswa {

constexpr float kLog2e = 1.4426950408889634f;

// Kernel-side view of rswa_attn_params (strides in elements).
struct AttnArgs {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  float* delta;   // fp32 [heads_q, rows_q] packed: -sum_d dO * O         (workspace)
  float* lse2;    // fp32 [heads_q, rows_q] packed: -lse * log2(e); empty rows -inf (workspace)
  // dK/dV kernel with the q heads of a GQA group split over `nsplit` blocks per key tile:
  // fp32 partial sums [tile unit][part] and one arrival counter per tile unit (workspace)
  float* dkv_part;
  int32_t* dkv_count;
  int32_t nsplit;     // 1: one block per (key tile, kv head) walks the whole group
  int32_t n_count;    // arrival counters in the workspace
  const int32_t* cu_q;
  const int32_t* cu_k;
  int64_t q_st[3], k_st[3], v_st[3], o_st[3], do_st[3], dq_st[3], dk_st[3], dv_st[3], lse_st[3];
  int64_t rows_q;  // batch * seqlen_q (dense) or total_q (packed)
  int64_t rows_k;  // batch * seqlen_k (dense) or total_k (packed)
  int32_t batch, heads_q, heads_kv, group;  // group = heads_q / heads_kv
  int32_t seqlen_q, seqlen_k;
  int32_t wl, wr, n_sink;  // wl/wr < 0: unbounded
  int32_t shift_explicit, shift_val;
  int32_t dq_accumulate;  // backward: add to dq instead of overwriting it
  int32_t out_accumulate;  // forward: merge the block into what out / lse hold
  // fp32 / fp64 accumulators of the ring loops in place of 16-bit / fp32 results (RSWA_WIDE_*):
  // forward out fp32 + lse fp64; backward dq fp32; backward dk, dv fp32 (+ add to them)
  int32_t wide_out, wide_dq, wide_dkv, dkv_accumulate;
  int32_t n_tile;          // tiles per sequence (dense) / total tile slots (packed)
  int32_t n_work;          // logical blocks
  // Blocks are dispatched in logical order; these flags reverse the order of the query
  // tiles (forward, dQ) or key tiles (dK/dV) so that the tiles with the most visible
  // pairs start first and the short ones fill the tail of the launch.
  int32_t rev_q, rev_k;
  // backward with sink keys and a bounded window: workspace of the sink kernel -- fp32 sums
  // [sequence x kv head][chunk of rows][sink][dK, dV][D] and one arrival counter per
  // (sequence, kv head); null when that kernel does not run
  float* sink_part;
  int32_t* sink_count;
  int32_t sink_chunks;  // row chunks per (sequence, kv head)
  // keys in two row ranges: key rows [0, seg) of k / v / dk / dv, the rest in k2 / v2 / dk2 / dv2
  // (same strides); seg = INT32_MAX when all keys lie in k / v
  const void* k2;
  const void* v2;
  void* dk2;
  void* dv2;
  int32_t seg;
  int32_t avg_keys;  // keys a query row sees on average (host estimate; block shapes hang on it)
  int32_t far;  // a sequence of some streamed tensor spans 2 GiB or more: FAR kernels
  // dS hand-off (backward): the dK/dV kernel stores its packed 16-bit dS tiles and the dQ
  // kernel of that route only multiplies them with K.  Unit = 32 query rows x 64 keys (one
  // wave's step), 4 KiB, at ds + (((q head * ds_slots + row-tile slot) * ds_nkb + key block %
  // ds_nkb) * 4 + 64-key group) * 4096; a row tile sees at most ds_nkb consecutive 256-key
  // blocks.  Null: the dQ kernel recomputes S and dP.
  char* ds;
  int32_t ds_nkb;
  int32_t ds_slots;  // 32-row tile slots per q head (dense: batch * tiles; packed: rows / 32 + batch)
  float scale, scale_log2;
};

struct SeqInfo {
  int64_t q_row0, k_row0;  // first row of the sequence in the (batch-strided or packed) tensor
  int64_t q_base, k_base;  // element offset of the batch (dense) — 0 in packed mode
  int32_t len_q, len_k;
  int32_t batch_idx;
};

// XCD-aware block id: consecutive logical ids land on the same XCD (8 XCDs,
// hardware deals physical block ids round-robin), so that blocks sharing K/V
// tiles share an L2.  The grid is padded to a multiple of 8; returns -1 for pad.
__device__ __forceinline__ int logical_block_id(int n_work) {
  const int per_xcd = (int)gridDim.x >> 3;
  const int id = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
  return id < n_work ? id : -1;
}

static inline unsigned padded_grid(int64_t n_work) { return (unsigned)(ceil_div(n_work, 8) * 8); }

// Mask bounds of one query row i (local index): visible keys are
//   j <= hi  and  (j >= lo or j < n_sink);   hi already clipped to len_k - 1.
struct RowBounds {
  int lo, hi;
};

__device__ __forceinline__ RowBounds row_bounds(const AttnArgs& a, int i, int len_q, int len_k) {
  RowBounds r;
  const int shift = a.shift_explicit ? a.shift_val : len_k - len_q;
  r.hi = (a.wr >= 0) ? min(len_k - 1, i + shift + a.wr) : len_k - 1;
  r.lo = (a.wl >= 0) ? max(0, i + shift - a.wl) : 0;
  if (i >= len_q) r.hi = -1;  // rows past the end see nothing
  return r;
}

// Packed mode: which sequence, and which of its tiles of `tile` = 2^tile_log2 rows, does
// tile slot `t` along the q or k axis stand for?  Sequence b owns the slots from
// cu[b] / tile + b on -- strictly increasing in b, so a binary search over cu finds b in
// log2(batch) dependent loads, where a running count of tiles would have to walk every
// sequence before it.  ceil(len_b / tile) of its slots are its tiles; at most one more, before
// the next sequence's first, stays unused (false is returned for it), which is why a packed
// grid has ceil(rows / tile) + batch slots.
__device__ __forceinline__ bool locate_packed(const AttnArgs& a, int t, int tile_log2, bool along_k,
                                              SeqInfo& s, int& tile_in_seq) {
  const int32_t* cu = along_k ? a.cu_k : a.cu_q;
  int lo = 0, hi = a.batch;  // first slot of lo <= t; hi == batch or first slot of hi > t
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((cu[mid] >> tile_log2) + mid <= t) lo = mid;
    else hi = mid;
  }
  const int b = lo;
  const int first = cu[b];
  tile_in_seq = t - ((first >> tile_log2) + b);
  if ((tile_in_seq << tile_log2) >= cu[b + 1] - first) return false;
  s.batch_idx = b;
  s.q_row0 = a.cu_q[b];
  s.k_row0 = a.cu_k[b];
  s.len_q = a.cu_q[b + 1] - a.cu_q[b];
  s.len_k = a.cu_k[b + 1] - a.cu_k[b];
  s.q_base = 0;
  s.k_base = 0;
  return true;
}

template <typename T>
struct Mma;

template <>
struct Mma<__bf16> {
  using V8 = bf16x8;
  using V4 = bf16x4;
  static __device__ __forceinline__ f32x16 mfma32(V8 a, V8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(V8 a, V8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // The same instruction as inline assembly with the accumulator kept in vector registers
  // (for accumulators the vector ALU reads next; the builtin's accumulators live in
  // accumulation registers), and a zero-initialising form (early clobber: the destination
  // of a 32x32 MFMA must not overlap its A / B operands).  The compiler sees opaque
  // statements and inserts no wait states after them: the caller keeps at least two later
  // MFMAs (or 32 idle cycles) between one of these and any other instruction that reads
  // its result, copies added by the register allocator included -- accumulators that live
  // across control flow are therefore better served by the builtin.  Volatile: they keep
  // their order among themselves and the empty volatile statements that pin vector work.
  // RSWA_MFMA_BUILTIN_ONLY builds the same three through the builtin instead: the compiler then
  // pads every hazard itself (and is free to place the accumulators badly).  The build makes a
  // second library that way, and a GPU test holds the two to the same output bits -- a
  // scheduler change in a later compiler that broke the distance kept by hand would show there.
#ifndef RSWA_MFMA_BUILTIN_ONLY
  static __device__ __forceinline__ void mfma32_vec(V8 a, V8 b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma32_vec0(V8 a, V8 b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
  // first MFMA of a chain that starts from `init` instead of zero
  static __device__ __forceinline__ void mfma32_vec_init(V8 a, V8 b, const f32x16& init, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(c) : "v"(a), "v"(b), "v"(init));
  }
#else
  static __device__ __forceinline__ void mfma32_vec(V8 a, V8 b, f32x16& c) { c = mfma32(a, b, c); }
  static __device__ __forceinline__ void mfma32_vec0(V8 a, V8 b, f32x16& c) {
    c = mfma32(a, b, f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0});
  }
  static __device__ __forceinline__ void mfma32_vec_init(V8 a, V8 b, const f32x16& init, f32x16& c) {
    c = mfma32(a, b, init);
  }
#endif
  static __device__ __forceinline__ V8 pack(const float* x) {
    f32x8 f = {x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7]};
    return __builtin_convertvector(f, V8);
  }
  static __device__ __forceinline__ V4 pack4(float a, float b, float c, float d) {
    f32x4 f = {a, b, c, d};
    return __builtin_convertvector(f, V4);
  }
};

template <>
struct Mma<_Float16> {
  using V8 = f16x8;
  using V4 = f16x4;
  static __device__ __forceinline__ f32x16 mfma32(V8 a, V8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(V8 a, V8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
#ifndef RSWA_MFMA_BUILTIN_ONLY
  static __device__ __forceinline__ void mfma32_vec(V8 a, V8 b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma32_vec0(V8 a, V8 b, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(c) : "v"(a), "v"(b));
  }
  // first MFMA of a chain that starts from `init` instead of zero
  static __device__ __forceinline__ void mfma32_vec_init(V8 a, V8 b, const f32x16& init, f32x16& c) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(c) : "v"(a), "v"(b), "v"(init));
  }
#else
  static __device__ __forceinline__ void mfma32_vec(V8 a, V8 b, f32x16& c) { c = mfma32(a, b, c); }
  static __device__ __forceinline__ void mfma32_vec0(V8 a, V8 b, f32x16& c) {
    c = mfma32(a, b, f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0});
  }
  static __device__ __forceinline__ void mfma32_vec_init(V8 a, V8 b, const f32x16& init, f32x16& c) {
    c = mfma32(a, b, init);
  }
#endif
  static __device__ __forceinline__ V8 pack(const float* x) {
    f32x8 f = {x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7]};
    return __builtin_convertvector(f, V8);
  }
  static __device__ __forceinline__ V4 pack4(float a, float b, float c, float d) {
    f32x4 f = {a, b, c, d};
    return __builtin_convertvector(f, V4);
  }
};

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// XOR swizzle of 16-byte chunks inside an LDS tile whose rows hold CH chunks (8 or 16):
// chunk c of row r is stored at chunk position c ^ swz_f<CH>(r).  It makes both access
// patterns used by the kernels bank-conflict free: 16 consecutive rows at one logical
// chunk (MFMA row fragments, 16-byte reads) and 4 consecutive rows x 4 consecutive chunks
// (one phase of the transposing 8-byte reads).  swz_f only looks at the low 4 bits of the
// row, so offsets of 16 rows (and of 32-row blocks) fold into immediate offsets.
template <int CH>
__device__ __forceinline__ int swz_f(int row) {
  if constexpr (CH == 16) {
    return ((row & 3) << 2) | ((row >> 2) & 3);
  } else {
    static_assert(CH == 8, "rows of 8 or 16 chunks");
    return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  }
}
template <int CH>
__device__ __forceinline__ int swz(int row, int chunk) {
  return chunk ^ swz_f<CH>(row);
}
// The swizzle of the kernels built on 16x16x32 MFMAs (A / B: lane = row or column l % 16,
// 8 consecutive k at 8 (l / 16); C: lane = column l % 16, rows 4 (l / 16) + i).  Their access
// patterns: 16 consecutive rows x 4 consecutive chunks (row fragments, 16-byte reads: lane =
// row l % 16, chunk 4 ks + l / 16) and 16 consecutive rows x 2 consecutive chunks (transposing
// 8-byte reads: row 4 (l / 16) + (l % 16) / 4).  The functions are GF(2)-linear in the row and
// were picked by measurement: of all linear maps, run through both patterns on the hardware,
// these are among those that reach the full LDS rate in both (an obvious candidate, the row's
// low three bits shifted up by one with bit 3 as the lowest bit, runs the 16-byte pattern at
// half rate).  They look at the row's low three bits only.
template <int CH>
__device__ __forceinline__ int swz16_f(int row) {
  if constexpr (CH == 16) {
    return ((row & 1) ? 0xc : 0) ^ ((row & 2) ? 0x8 : 0) ^ ((row & 4) ? 0x2 : 0);
  } else {
    static_assert(CH == 8, "rows of 8 or 16 chunks");
    return ((row & 1) ? 0x6 : 0) ^ ((row & 2) ? 0x7 : 0) ^ ((row & 4) ? 0x2 : 0);
  }
}
template <int CH, bool W16>
__device__ __forceinline__ int swz_sel(int row) {
  if constexpr (W16) return swz16_f<CH>(row);
  else return swz_f<CH>(row);
}

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;

// Two transposing reads -> one 8-element MFMA fragment.
template <typename V8>
__device__ __forceinline__ V8 tr_pair(const char* p0, const char* p1) {
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p0);
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p1);
  const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  V8 out;
  __builtin_memcpy(&out, &both, 16);
  return out;
}

typedef __attribute__((address_space(3))) void lds_void_t;

// Buffer resource over the rows of one (sequence, head) slice: `rows` rows of `row_bytes`
// useful bytes, `stride_bytes` apart.  Loads past the last row return zero, in registers
// and in LDS alike, so partial tiles need no clamping.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rows_rsrc(const void* base, int rows,
                                                                 int64_t stride_bytes,
                                                                 int row_bytes) {
  const int64_t bytes = rows > 0 ? (int64_t)(rows - 1) * stride_bytes + row_bytes : 0;
  return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)bytes, 0x00020000);
}

// Where the ROWS-row tile that starts at row `row0` of a slice of `rows` rows is fetched from:
// a resource and the byte offset of the tile's first row inside it (rows past the slice's
// last read as zero).
//   FAR = false: the resource covers the whole slice (loop-invariant) and the offset selects the
//                tile; the slice must span less than 2 GiB.
//   FAR = true:  the resource is based at the tile's first row (64-bit pointer arithmetic, all
//                else 32-bit scalar arithmetic) and covers the tile only, so that a slice may
//                span any number of bytes as long as one tile spans less than 2 GiB.  Costs a
//                dozen scalar instructions per tile (2 % of the dK/dV kernel, whose single wave
//                per SIMD hides nothing), which is why the host picks it only when needed.
struct TileSrc {
  __amdgpu_buffer_rsrc_t rsrc;
  int soff;
};
template <int ROWS, bool FAR>
__device__ __forceinline__ TileSrc tile_src(const void* base, int row0, int rows, int stride_bytes,
                                            int row_bytes) {
  if constexpr (FAR) {
    const int n = min(rows - row0, ROWS);  // rows of the tile that exist
    const int bytes = n > 0 ? (n - 1) * stride_bytes + row_bytes : 0;
    const uint64_t off = (uint64_t)(uint32_t)row0 * (uint64_t)(uint32_t)stride_bytes;
    return {__builtin_amdgcn_make_buffer_rsrc((void*)((const char*)base + off), 0, bytes, 0x00020000),
            0};
  } else {
    return {make_rows_rsrc(base, rows, stride_bytes, row_bytes), row0 * stride_bytes};
  }
}

// Key rows in two ranges (AttnArgs::seg): where the tile of key rows starting at `row0` (never
// straddling the boundary: seg is a multiple of every tile size) is fetched from.
template <typename T>
struct KeySeg {
  const T* base;
  int row0, rows;  // first row of the tile inside its range, rows of the range
};
template <typename T>
__device__ __forceinline__ KeySeg<T> key_seg(const T* first, const T* second, int seg, int row0,
                                             int len_k) {
  const bool s2 = row0 >= seg;
  return {s2 ? second : first, s2 ? row0 - seg : row0, s2 ? len_k - seg : min(len_k, seg)};
}

// Cooperative copy of a [ROWS x D] tile into a swizzled LDS tile with buffer loads that
// land directly in LDS (buffer_load_dwordx4 ... lds: lane L of a wave writes
// wave_base + 16 L).  The per-lane byte offsets are computed once (init); a tile load is
// then N instructions with one scalar offset and no vector arithmetic at all.
template <int D, int ROWS, int THREADS, bool W16 = false>
struct TileDma {
  static constexpr int CPR = D / 8;
  static constexpr int RPI = 64 / CPR;  // rows per wave instruction
  static constexpr int NW = THREADS / 64;
  static constexpr int N = ROWS * CPR / THREADS;
  static_assert(N >= 1 && N * THREADS == ROWS * CPR, "tile must divide evenly");
  // Instruction n of a wave covers rows (n NW + wave) RPI + lane / CPR: NW RPI (a multiple
  // of 16) rows further per n, which leaves the swizzle unchanged, so one per-lane offset
  // serves all N instructions and the step goes into the scalar offset.
  static_assert((NW * RPI) % 16 == 0, "row step must preserve the swizzle");
  int voff;
  int step_bytes;
  int wave;
  __device__ __forceinline__ void init(int64_t stride_elems, int tid) {
    const int lane = tid & 63;
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row = wave * RPI + lane / CPR;
    voff = (int)(row * stride_elems * 2) + (((lane % CPR) ^ swz_sel<CPR, W16>(row)) << 4);
    step_bytes = (int)(NW * RPI * stride_elems * 2);
  }
  // `soff` = byte offset of the tile's first row inside the resource (wave-uniform)
  __device__ __forceinline__ void load_one(__amdgpu_buffer_rsrc_t rsrc, int soff, char* lds_tile,
                                           int n) const {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc, (lds_void_t*)(lds_tile + (n * NW + wave) * 1024), 16, voff, soff + n * step_bytes, 0,
        0);
  }
  __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t rsrc, int soff, char* lds_tile) const {
#pragma unroll
    for (int n = 0; n < N; n++) load_one(rsrc, soff, lds_tile, n);
  }
  __device__ __forceinline__ void load(const TileSrc& t, char* lds_tile) const {
    load(t.rsrc, t.soff, lds_tile);
  }
};

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose
// index is a compile-time constant in every iteration (register arrays indexed by it never
// fall back to dynamic indexing, whatever the unroller thinks of the body's size).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Block barrier that waits for this wave's LDS traffic only: loads still in flight from
// global memory into LDS (vmcnt) are NOT drained, unlike __syncthreads().  A wave that
// issued such loads calls wait_dma() before the barrier that publishes them.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ void wait_dma() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Wait until at most N of this wave's vector memory operations (loads, loads into LDS, stores:
// they complete in issue order) are outstanding.  Through the builtin, so that the compiler's own
// bookkeeping of what is in flight sees the wait (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// the other counters left at their "no wait" values).
template <int N>
__device__ __forceinline__ void wait_vmem_but() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");
}

// max / sum across the two half-waves (lane l <-> lane l ^ 32).
__device__ __forceinline__ float halfwave_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halfwave_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Keys per block of the dK/dV kernel, and how a launch of it is laid out: with so few key
// tiles that one block per (tile, kv head) would leave half of the 256 compute units without
// work, the q heads of each GQA group are dealt to `nsplit` blocks, whose fp32 partial sums
// meet in the workspace.  Measured on the rank share (8192-token chunk, window 4096, 32 / 8
// heads): the previous-chunk corner (128 blocks) 0.75 -> 0.30 ms; the own-chunk block (256
// blocks of 32..544 steps) gains 4 % alone and loses 8 % beside the corner launch -- more
// compute units busy lowers the shader clock (1.92 -> 1.77 GHz), and every part pays its own
// prologue, partial store and share of the final sum -- so launches that already give every
// compute unit a block are left alone.
constexpr int kDkvKeysPerBlock = 256;
// dS hand-off: bytes one dK/dV block leaves per 32-row query tile (32 x 256 16-bit values) and
// per wave of it (32 x 64: the unit the dQ kernel of that route fetches)
constexpr int kDsBlockBytes = 32 * kDkvKeysPerBlock * 2;
constexpr int kDsUnitBytes = kDsBlockBytes / 4;
constexpr int kMaxTileRows = 256;  // bound on the rows fetched as one tile that the stride checks assume
                                   // (today's largest tile has 64 rows: K / V in the forward and dQ kernels)
constexpr int kComputeUnits = 256;  // MI355X
#ifndef RSWA_DKDV_SPLIT_BELOW
#define RSWA_DKDV_SPLIT_BELOW (kComputeUnits / 2 + 1)
#endif
constexpr int kDkvSplitBelow = RSWA_DKDV_SPLIT_BELOW;  // split launches of fewer blocks
struct BwdLayout {
  uint64_t stats_bytes;    // each of the two statistics arrays
  int nsplit;
  int n_tile_k;            // key tile slots per kv head (dense: per batch entry)
  int n_count;             // arrival counters (one per key tile unit)
  uint64_t count_off, part_off, total_bytes;
  int sink_chunks;         // row chunks of the sink kernel per (sequence, kv head); 0: no sink kernel
  int sink_count_index;    // its first arrival counter
  uint64_t sink_off;       // its fp32 sums
  // dS hand-off (ds_bytes == 0: not used for this call)
  uint64_t ds_off, ds_bytes;
  int ds_nkb, ds_slots;
};
BwdLayout bwd_layout(const rswa_attn_params* p, bool allow_split, bool allow_handoff = false);

// Fill an AttnArgs from the public struct; validates what both directions share.
// `allow_split` = false keeps the dK/dV kernel at one block per key tile, whatever the shape
// (workspace holds the statistics only).
int fill_args(const rswa_attn_params* p, bool backward, AttnArgs& a, bool allow_split = true,
              bool allow_handoff = false);

}  // namespace rswa
