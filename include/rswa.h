/*
 * rswa.h — C ABI of the MI355X (gfx950) kernels behind ring_swa's single-GPU
 * attention path.
 *
 * Plain C: raw device pointers, element strides, sizes.  No torch types.  Every
 * call only enqueues work on `stream` (a hipStream_t passed as void*); nothing
 * synchronises the device and nothing allocates or frees device memory — the
 * caller owns all buffers, scratch included.  Functions return 0 on success and
 * a negative rswa_status otherwise; rswa_last_error() gives the message of the
 * calling thread's last failure.
 *
 * Each entry point replaces one interface of the upstream Python package
 * (paths relative to its repository root):
 *
 *   rswa_merge_attn_out   ring_swa/ops/merge.py:150-193  (triton_merge_attn_out;
 *                         torch twin :16-50; selector :196-208)
 *   rswa_attn_fwd         ring_swa/ops/wrap_flash.py:168-200 (wrapped_flash_attn_fwd)
 *                         and :203-273 (wrapped_flash_attn_fwd_varlen); also the
 *                         forward half of flash_attn_func / flash_attn_varlen_func at
 *                         ring_swa/sliding_window/nonvarlen.py:379-386 and
 *                         ring_swa/sliding_window/varlen.py:406-417
 *   rswa_attn_bwd         ring_swa/ops/wrap_flash.py:276-327 (wrapped_flash_attn_bwd)
 *                         and :330-429 (wrapped_flash_attn_bwd_varlen)
 *   rswa_attn_bwd_phases  the same interface, one launch of the three at a time
 *   rswa_attn_bwd_static, rswa_attn_bwd_static_init  (no upstream counterpart:
 *                         rswa_attn_bwd for callers that cannot allocate; see their
 *                         declarations)
 *   rswa_attn_bwd_workspace_bytes, rswa_attn_bwd_handoff_active   (sizing helper for the
 *                         scratch rswa_attn_bwd needs -- upstream flash-attn allocates the
 *                         same internally -- and which route a backward call takes)
 *   rswa_stream_copy      (no upstream counterpart: the copy kernel the merge kernel's
 *                         rate is measured against)
 * The accumulating forms of the block operators, ring_swa/ops/attn.py:12-196 with the
 * fp32 / fp64 / fp32 accumulators of ring_swa/sliding_window/nonvarlen.py:53-59, 203-206,
 * are served by the fields out_accumulate, dq_accumulate, wide and dkv_accumulate of
 * rswa_attn_params.
 */
#ifndef RSWA_H
#define RSWA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RSWA_VERSION 3

typedef enum rswa_status {
  RSWA_OK = 0,
  RSWA_ERR_INVALID = -1,     /* bad argument / inconsistent shapes            */
  RSWA_ERR_UNSUPPORTED = -2, /* dtype / head_dim / stride the kernels lack    */
  RSWA_ERR_LAUNCH = -3       /* HIP reported an error at launch               */
} rswa_status;

typedef enum rswa_dtype {
  RSWA_BF16 = 0,
  RSWA_F16 = 1,
  RSWA_F32 = 2,
  RSWA_F64 = 3
} rswa_dtype;

/*
 * In-place log-sum-exp merge of a new partial into a running one:
 *   w_old = sigmoid(lse - lse_new), w_new = sigmoid(lse_new - lse)
 *   o   <- w_old * o + w_new * o_new
 *   lse <- max(lse, lse_new) + log1p(exp(-|lse_new - lse|))
 * lse = -inf is the identity element on either side; both -inf gives
 * (o = 0, lse = -inf).  Arithmetic is fp32 whatever the storage types
 * (ring_swa/ops/merge.py:134-135 down-casts fp64 LSE the same way).
 *
 * o, o_new: logical [batch, seqlen, heads, head_dim]; lse, lse_new: logical
 * [batch, heads, seqlen].  Strides are in ELEMENTS, arrays of 4 (b,s,h,d) and
 * 3 (b,h,s); the head_dim stride must be 1.  Sliced / expanded views are fine.
 * o_dtype, o_new_dtype in {BF16, F16, F32}; lse_dtype, lse_new_dtype in
 * {F32, F64}.  head_dim must be a multiple of 8, at most 256.
 */
int rswa_merge_attn_out(void* o, int o_dtype, const int64_t* o_stride,
                        void* lse, int lse_dtype, const int64_t* lse_stride,
                        const void* o_new, int o_new_dtype, const int64_t* o_new_stride,
                        const void* lse_new, int lse_new_dtype, const int64_t* lse_new_stride,
                        int64_t batch, int64_t seqlen, int64_t heads, int64_t head_dim,
                        void* stream);

/*
 * Plain device-to-device copy of `bytes` bytes (a multiple of 16; both pointers 16-byte
 * aligned, ranges not overlapping) by a kernel that does nothing else: 16 bytes a lane,
 * non-temporal.  No counterpart in the upstream package, whose merge harness
 * (ring_swa/ops/merge.py:257-302) only times the merge: this is the yardstick beside it -- the
 * rate a kernel that only moves memory reaches on the same device in the same run -- against
 * which rswa_merge_attn_out's rate is reported.
 */
int rswa_stream_copy(void* dst, const void* src, uint64_t bytes, void* stream);

/*
 * One attention block, forward or backward.
 *
 * Dense mode (cu_seqlens_q == NULL): q/out/dout/dq are [batch, seqlen_q,
 * heads_q, head_dim], k/v/dk/dv are [batch, seqlen_k, heads_kv, head_dim], lse
 * is fp32 [batch, heads_q, seqlen_q].
 * Packed mode (cu_seqlens_q and cu_seqlens_k given, int32 device arrays of
 * batch + 1 entries): tensors are [total, heads, head_dim], lse is fp32
 * [heads_q, total_q]; the batch strides are ignored; seqlen_q / seqlen_k are
 * upper bounds on the per-sequence lengths (they only size the launch) and
 * total_q / total_k are the packed row counts.
 *
 * Strides are in elements: *_stride[0] batch, [1] row (token), [2] head; the
 * head_dim stride must be 1 and every row must start 16-byte aligned.
 * lse_stride: [0] batch, [1] head, [2] row.
 *
 * Mask (flash-attn's local-window rule, bottom-right aligned): with
 * shift = len_k - len_q of the sequence, key j is visible from query i iff
 *   i + shift - window_left <= j <= i + shift + window_right
 * where a negative window bound means unbounded and causal != 0 forces
 * window_right = 0.  num_sink > 0 additionally makes keys j < num_sink visible
 * whenever they satisfy the right bound (attention sinks at the sequence head).
 * shift_explicit != 0 replaces the bottom-right shift by the caller's `shift`
 * (any sign) for every sequence: e.g. shift = 0 aligns the diagonals top-left,
 * and shift = -(w + 1) with window_left < 0, window_right = 0 selects the keys
 * that lie more than w positions behind the query.
 * Rows with no visible key produce out = 0, lse = -inf.
 *
 * lse is the natural-log sum of exp(softmax_scale * q.k) over visible keys.
 *
 * Backward takes the caller's out / lse — they may be the result of merging
 * several blocks, which is how the ring's "merge backward" is realised
 * (ring_swa/sliding_window/nonvarlen.py:242-253) — and OVERWRITES dq, dk, dv
 * (rows/keys that receive nothing are written as zero).  dk/dv are reduced over
 * the heads_q / heads_kv query heads that share a kv head.  No atomics are used:
 * results are run-to-run deterministic (upstream runs flash-attn with
 * deterministic=False, ring_swa/ops/wrap_flash.py:61).
 */
typedef struct rswa_attn_params {
  int32_t dtype;    /* RSWA_BF16 or RSWA_F16: type of q,k,v,out,dout,dq,dk,dv */
  int32_t head_dim; /* 64 or 128                                             */
  int32_t batch;
  int32_t heads_q;
  int32_t heads_kv;
  int32_t seqlen_q; /* dense: exact; packed: upper bound of per-sequence len  */
  int32_t seqlen_k;
  int64_t total_q;  /* packed mode only; sequences stay below 2^28 rows       */
  int64_t total_k;
  const int32_t* cu_seqlens_q; /* NULL => dense                               */
  const int32_t* cu_seqlens_k;

  float softmax_scale;
  int32_t window_left;  /* < 0 (or >= 2^28): unbounded */
  int32_t window_right; /* < 0 (or >= 2^28): unbounded */
  int32_t causal;
  int32_t num_sink;
  int32_t shift_explicit; /* 0: shift = len_k - len_q (flash-attn alignment) */
  int32_t shift;          /* used when shift_explicit != 0; |shift| < 2^28   */

  const void* q;
  const void* k;
  const void* v;
  int64_t q_stride[3];
  int64_t k_stride[3];
  int64_t v_stride[3];

  void* out;  /* fwd: written.  bwd: read (const) */
  int64_t out_stride[3];
  float* lse; /* fwd: written.  bwd: read (const) */
  int64_t lse_stride[3];

  /* backward only */
  const void* dout;
  int64_t dout_stride[3];
  void* dq;
  void* dk;
  void* dv;
  int64_t dq_stride[3];
  int64_t dk_stride[3];
  int64_t dv_stride[3];
  void* workspace;        /* >= rswa_attn_bwd_workspace_bytes(), 256-byte aligned */
  uint64_t workspace_bytes;
  /* != 0: dq += this call's dQ instead of dq = (the buffer's 16-bit values and the new
   * 16-bit values are added in fp32 and rounded once: what the reference's fp32 dq
   * accumulator over two ring blocks gives, ring_swa/sliding_window/nonvarlen.py:318-321,
   * without the extra passes over dq).  dk / dv are always overwritten. */
  int32_t dq_accumulate;
  /* RSWA_ADDR_AUTO (0): tiles are fetched through 32-bit offsets that count from a sequence's
   * first row when every sequence of q, k, v (and dout) spans less than 2 GiB (rows x row
   * stride), from each tile's first row otherwise -- a sequence may then span anything, only
   * one row stride must stay below 8 MiB.  RSWA_ADDR_FAR (1) selects the second form whatever
   * the sizes (same results; a few per cent slower). */
  int32_t addressing;
  /* Forward only.  != 0: out / lse already hold a running partial result for these rows (16-bit
   * out, fp32 lse, e.g. what an earlier rswa_attn_fwd over other keys wrote); this call's block is
   * merged into them in place instead of overwriting them -- the arithmetic of
   * rswa_merge_attn_out (ring_swa/ops/merge.py:16-50) applied to the block's 16-bit output, in
   * the kernel's epilogue: same bits as the two calls, one launch and one pass over out less
   * (what ring_swa/ops/attn.py:23-37 does with a temporary and a merge kernel). */
  int32_t out_accumulate;
  /* Dense mode only.  > 0: the keys of the block are two row ranges of different tensors -- a
   * ring rank's tail of the previous chunk followed by its own chunk -- taken as they lie,
   * without concatenating them: key rows [0, seg_rows) are rows 0 .. of k / v (gradients: dk /
   * dv), key rows [seg_rows, seqlen_k) are rows 0 .. of k2 / v2 (dk2 / dv2), which have the
   * strides of k / v (dk / dv).  One kernel pass then covers what the reference computes as
   * two blocks and a merge (ring_swa/sliding_window/nonvarlen.py:95-150: the own-chunk block
   * and the previous chunk's corner).  seg_rows must be a multiple of 256 below seqlen_k, and
   * num_sink 0.  0: one range, k2 .. dv2 ignored. */
  int32_t seg_rows;
  const void* k2;
  const void* v2;
  void* dk2;
  void* dv2;
  /* Backward only.  != 0: dS hand-off.  The dK/dV kernel, which computes P and dS for its own
   * sums anyway, also stores its 16-bit dS tiles in the workspace, and dq comes from a kernel
   * that only multiplies them with K (dQ = scale * dS K) instead of computing S = Q K^T and
   * dP = dO V^T a second time: 12 D multiply-adds per (query, key) pair instead of 14 D for the
   * whole backward, at the price of 2 bytes per pair written and read once.  The workspace
   * grows by rswa_attn_bwd_workspace_bytes' account of it (about 2.2 bytes per visible pair and
   * q head for a window of thousands of keys).  Honoured when the call has no sink keys under a
   * bounded window, every sequence spans less than 2 GiB (the first addressing form), one
   * q head's tiles stay below 2 GiB and, with the value 1, the launch is not one of the small
   * ones whose key tiles are split over several blocks (the value 2 prefers the hand-off to that
   * split); silently the recomputing route otherwise -- ask rswa_attn_bwd_handoff_active().  With rswa_attn_bwd_phases the DQ phase of this route reads
   * what the DKDV phase of the same call parameters left in the same workspace, so DKDV must
   * have run before it.  rswa_attn_bwd_static never uses it.  Same interface replaced:
   * ring_swa/ops/wrap_flash.py:276-429. */
  int32_t ds_handoff;
  /* Accumulators of the ring loops (ring_swa/sliding_window/nonvarlen.py:53-59, 203-206: fp32
   * running output, fp64 running LSE, fp32 dq and dkv that every block is added to) taken as
   * they are, so that a block needs no temporary, no merge launch and no elementwise passes
   * (ring_swa/ops/attn.py:23-37, ring_swa/sliding_window/nonvarlen.py:318-321).  Bit mask:
   *   RSWA_WIDE_OUT  forward: out is fp32 and lse is fp64 (strides in their own elements).  The
   *                  block's output is rounded to the 16-bit type of q first, as the reference's
   *                  block kernel returns it, then written as fp32 -- or, with out_accumulate,
   *                  merged into what out / lse hold: the bits of rswa_attn_fwd into 16-bit
   *                  temporaries followed by rswa_merge_attn_out on these accumulators.
   *   RSWA_WIDE_DQ   backward: dq is fp32: the block's dq, rounded to 16 bits, is written as
   *                  fp32 or, with dq_accumulate, added to what dq holds.
   *   RSWA_WIDE_DKV  backward: dk and dv (dk2 / dv2 too) are fp32, written likewise; with
   *                  dkv_accumulate != 0 the block's values are added to what they hold.  Not
   *                  with sink keys under a bounded window (RSWA_ERR_UNSUPPORTED).
   * The backward still reads out in the 16-bit type and lse as fp32 (the reference casts its
   * accumulators before the backward, ring_swa/sliding_window/nonvarlen.py:156-157). */
  int32_t wide;
  int32_t dkv_accumulate; /* only with RSWA_WIDE_DKV */
} rswa_attn_params;

#define RSWA_WIDE_OUT 1
#define RSWA_WIDE_DQ 2
#define RSWA_WIDE_DKV 4

#define RSWA_ADDR_AUTO 0
#define RSWA_ADDR_FAR 1

int rswa_attn_fwd(const rswa_attn_params* p, void* stream);
int rswa_attn_bwd(const rswa_attn_params* p, void* stream);

/*
 * rswa_attn_bwd is three launches: PREP (row statistics into the workspace), DKDV
 * (dk, dv written; reads the statistics) and DQ (dq written; reads the statistics).
 * This variant enqueues only the phases named in the bit mask, on the same
 * workspace: it lets a profiler or benchmark bracket one kernel alone, and lets a
 * caller that needs only some of the gradients skip the rest.  Same interface
 * replaced as rswa_attn_bwd (ring_swa/ops/wrap_flash.py:276-429).
 */
#define RSWA_BWD_PREP 1
#define RSWA_BWD_DKDV 2
#define RSWA_BWD_DQ 4
int rswa_attn_bwd_phases(const rswa_attn_params* p, void* stream, int phases);

/*
 * rswa_attn_bwd without a caller workspace and without any allocation: the row statistics
 * go to a buffer of RSWA_BWD_STATIC_MAX_BYTES that is part of the library's device image
 * (every GPU the library runs on holds it until the process ends); p->workspace and
 * p->workspace_bytes are ignored.  No counterpart in the upstream package: it is for
 * callers that cannot allocate device memory around the call - code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Shapes whose statistics
 * (8 bytes per (row, q head) pair) exceed the buffer -- more than 4 194 304 pairs -- are
 * refused with RSWA_ERR_UNSUPPORTED; the dK/dV kernel runs one block per key tile here,
 * whatever the shape (no partial sums).  The buffer's address is looked up on the
 * first call on each device (the device must be current, as for every other call); nothing
 * in it has to be cleared between calls, the statistics kernel rewrites what the others
 * read.  All calls on one GPU share the one buffer: calls that may overlap in time on the
 * same GPU (different streams, different threads) race and must be serialised by the caller.
 */
#define RSWA_BWD_STATIC_MAX_BYTES (32u << 20)
int rswa_attn_bwd_static(const rswa_attn_params* p, void* stream);

/* Looks up the address of that buffer on the current device, which the first
 * rswa_attn_bwd_static call on a device otherwise does itself (a symbol look-up that may load
 * the library's device image, under a host mutex).  A caller that captures rswa_attn_bwd_static
 * into a HIP graph calls this once per device BEFORE the capture begins: the look-up is no
 * stream operation and must not happen inside a capture.  Launches nothing, allocates nothing;
 * calling it again is free.  No counterpart in the upstream package (it serves the same callers
 * as rswa_attn_bwd_static: those that cannot allocate). */
int rswa_attn_bwd_static_init(void);

/* Scratch rswa_attn_bwd needs for these shapes: two fp32 values per (row, q head) -- the
 * row sum of dout * out and the LSE in base-2 units -- and, for launches with so few key
 * tiles (fewer than 129 blocks of 256 keys x kv head) that the q heads of each GQA group are
 * dealt to 2-4 blocks per tile, one arrival counter per tile and the fp32 partial dK / dV of
 * every part (256 keys x head_dim x 2 x 4 bytes each).  The call leaves the counters at zero;
 * nothing in the workspace has to be initialised by the caller. */
uint64_t rswa_attn_bwd_workspace_bytes(const rswa_attn_params* p);

/* 1 when a backward with these parameters takes the dS hand-off route (ds_handoff != 0 and the
 * shape is eligible), 0 otherwise. */
int rswa_attn_bwd_handoff_active(const rswa_attn_params* p);

/* Message of the calling thread's last failed call ("" if none). */
const char* rswa_last_error(void);

/* RSWA_VERSION the library was built from. */
int rswa_version(void);

/* sizeof(rswa_attn_params) the library was built with (binding self-check). */
uint64_t rswa_sizeof_attn_params(void);

#ifdef __cplusplus
}
#endif
#endif /* RSWA_H */
