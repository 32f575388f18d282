// Host-side validation of rswa_attn_params and translation to kernel arguments.
#include <algorithm>
#include "attn_common.h"

namespace rswa {

static uint64_t align_up(uint64_t x, uint64_t a) { return (x + a - 1) / a * a; }

static uint64_t delta_bytes(const rswa_attn_params* p) {
  const uint64_t rows = p->cu_seqlens_q ? (uint64_t)p->total_q
                                        : (uint64_t)p->batch * (uint64_t)p->seqlen_q;
  return align_up(rows * (uint64_t)p->heads_q * sizeof(float), 256);
}

// Can a backward with these parameters hand dS over?  Not with sink keys under a bounded window
// (a row tile's key blocks are no longer consecutive), and only in the first addressing form.
static bool handoff_eligible(const rswa_attn_params* p) {
  if (p->num_sink > 0 && p->window_left >= 0 && p->window_left < (1 << 28)) return false;
  if (p->addressing == RSWA_ADDR_FAR) return false;
  const bool packed = p->cu_seqlens_q != nullptr;
  const int64_t lim = (1ll << 31) - 65536;
  const int64_t rq = packed ? p->total_q : p->seqlen_q, rk = packed ? p->total_k : p->seqlen_k;
  if (rq * p->q_stride[1] * 2 >= lim || rk * p->k_stride[1] * 2 >= lim ||
      rk * p->v_stride[1] * 2 >= lim || rq * p->dout_stride[1] * 2 >= lim)
    return false;
  return true;
}

BwdLayout bwd_layout(const rswa_attn_params* p, bool allow_split, bool allow_handoff) {
  BwdLayout L{};
  L.nsplit = 1;
  if (!p || p->batch <= 0 || p->heads_q <= 0 || p->heads_kv <= 0 || p->head_dim <= 0) return L;
  L.stats_bytes = delta_bytes(p);
  const bool packed = p->cu_seqlens_q != nullptr;
  const int64_t rows_k = packed ? p->total_k : p->seqlen_k;
  L.n_tile_k = (int)((rows_k + kDkvKeysPerBlock - 1) / kDkvKeysPerBlock + (packed ? p->batch : 0));
  const int64_t blocks = (int64_t)L.n_tile_k * p->heads_kv * (packed ? 1 : p->batch);
  const int group = p->heads_q / p->heads_kv;
  // Splitting pays when one block per key tile leaves compute units without any work (see
  // kDkvSplitBelow).  The parts of a tile are summed in a fixed order.
  // (ds_handoff >= 2: the caller prefers the dS hand-off, which the split kernel does not do)
  const bool prefer_handoff = allow_handoff && p->ds_handoff >= 2 && handoff_eligible(p);
  if (allow_split && !prefer_handoff && group > 1 && blocks > 0 && blocks < kDkvSplitBelow) {
    for (int n : {4, 3, 2})
      if (group % n == 0) {
        L.nsplit = n;
        break;
      }
  }
  // Sink keys under a bounded window: the sink kernel, one chunk per ~512 rows of an average
  // sequence (at most 64), one arrival counter per (sequence, kv head).
  int64_t sink_units = 0;
  if (p->num_sink > 0 && p->window_left >= 0) {
    const int64_t rows_q = packed ? p->total_q / p->batch : p->seqlen_q;
    L.sink_chunks = (int)std::min<int64_t>(64, std::max<int64_t>(1, (rows_q + 511) / 512));
    sink_units = (int64_t)p->batch * p->heads_kv;
  }
  // workspace: statistics | arrival counters (split key tiles, then sink units) | partial
  // dK / dV of split key tiles | sums of the sink kernel
  const int64_t split_units = L.nsplit > 1 ? blocks : 0;
  L.n_count = (int)(split_units + sink_units);
  L.sink_count_index = (int)split_units;
  L.count_off = 2 * L.stats_bytes;
  L.part_off = L.count_off + align_up((uint64_t)L.n_count * sizeof(int32_t), 256);
  const uint64_t per_unit = (uint64_t)kDkvKeysPerBlock * p->head_dim * 2 * sizeof(float);
  L.sink_off = L.part_off + (uint64_t)split_units * L.nsplit * per_unit;
  L.total_bytes = L.sink_off + (uint64_t)sink_units * L.sink_chunks * p->num_sink * 2 * p->head_dim *
                                   sizeof(float);
  // dS hand-off: one 4 KiB unit per (q head, 32-row tile slot, 256-key block modulo nkb, 64-key
  // group).  A row tile sees keys [i0 + shift - left, i0 + 31 + shift + right]: left + right + 32
  // consecutive keys, which touch at most (left + right + 31) / 256 + 2 blocks of 256, and never
  // more than a sequence has.
  // (Launches whose key tiles are split over several blocks are small ones; they keep the
  // recomputing route: the split kernel has no registers left for the hand-off.)
  if (allow_handoff && p->ds_handoff && L.nsplit == 1 && handoff_eligible(p)) {
    const int64_t rows_q = packed ? p->total_q : (int64_t)p->batch * p->seqlen_q;
    const int64_t blocks_seq = (rows_k + kDkvKeysPerBlock - 1) / kDkvKeysPerBlock;  // rows_k: one sequence's bound
    int64_t nkb = blocks_seq;
    const bool causal = p->causal != 0;
    const int64_t wl = p->window_left, wr = causal ? 0 : p->window_right;
    if (wl >= 0 && wr >= 0 && wl < (1 << 28) && wr < (1 << 28))
      nkb = std::min<int64_t>(nkb, (wl + wr + 31) / kDkvKeysPerBlock + 2);
    nkb = std::max<int64_t>(nkb, 1);
    const int64_t slots = packed ? (rows_q + 31) / 32 + p->batch
                                 : (int64_t)p->batch * ((p->seqlen_q + 31) / 32);
    const uint64_t head_bytes = (uint64_t)slots * nkb * kDsBlockBytes;
    // (the dK/dV kernel addresses the units of a GQA group's heads through 32-bit offsets)
    if (rows_q > 0 && rows_k > 0 && head_bytes * (uint64_t)group < 0x7ff00000ull) {
      L.ds_nkb = (int)nkb;
      L.ds_slots = (int)slots;
      L.ds_off = align_up(L.total_bytes, 4096);
      L.ds_bytes = head_bytes * (uint64_t)p->heads_q;
      L.total_bytes = L.ds_off + L.ds_bytes;
    }
  }
  return L;
}

uint64_t bwd_workspace_bytes(const rswa_attn_params* p) { return bwd_layout(p, true, true).total_bytes; }

static bool rows_aligned(const void* ptr, const int64_t* st, int elem_bytes = 2) {
  if (((uintptr_t)ptr) % 16) return false;
  for (int i = 0; i < 3; i++)
    if (st[i] % (16 / elem_bytes)) return false;
  return true;
}

int fill_args(const rswa_attn_params* p, bool backward, AttnArgs& a, bool allow_split,
              bool allow_handoff) {
  RSWA_REQUIRE(p != nullptr, RSWA_ERR_INVALID, "attn: null params");
  RSWA_REQUIRE(p->dtype == RSWA_BF16 || p->dtype == RSWA_F16, RSWA_ERR_UNSUPPORTED,
               "attn: dtype %d (only bf16 and fp16)", p->dtype);
  RSWA_REQUIRE(p->head_dim == 64 || p->head_dim == 128, RSWA_ERR_UNSUPPORTED,
               "attn: head_dim %d (only 64 and 128)", p->head_dim);
  RSWA_REQUIRE(p->batch > 0 && p->heads_q > 0 && p->heads_kv > 0, RSWA_ERR_INVALID,
               "attn: batch/heads must be positive");
  RSWA_REQUIRE(p->heads_q % p->heads_kv == 0, RSWA_ERR_INVALID,
               "attn: heads_q %d not a multiple of heads_kv %d", p->heads_q, p->heads_kv);
  RSWA_REQUIRE(p->seqlen_q >= 0 && p->seqlen_k >= 0, RSWA_ERR_INVALID, "attn: negative seqlen");
  RSWA_REQUIRE(p->softmax_scale > 0.f && p->softmax_scale < 1e30f, RSWA_ERR_INVALID,
               "attn: softmax_scale must be positive and finite");
  RSWA_REQUIRE(p->num_sink >= 0, RSWA_ERR_INVALID, "attn: negative num_sink");
  const bool packed = p->cu_seqlens_q != nullptr || p->cu_seqlens_k != nullptr;
  if (packed) {
    RSWA_REQUIRE(p->cu_seqlens_q && p->cu_seqlens_k, RSWA_ERR_INVALID,
                 "attn: packed mode needs both cu_seqlens_q and cu_seqlens_k");
    RSWA_REQUIRE(p->total_q >= 0 && p->total_k >= 0, RSWA_ERR_INVALID, "attn: negative totals");
    RSWA_REQUIRE(p->total_q < (1ll << 31) && p->total_k < (1ll << 31), RSWA_ERR_INVALID,
                 "attn: totals out of range");
  }
  RSWA_REQUIRE(p->q && p->k && p->v && p->out && p->lse, RSWA_ERR_INVALID, "attn: null tensor");
  RSWA_REQUIRE((p->wide & ~(RSWA_WIDE_OUT | RSWA_WIDE_DQ | RSWA_WIDE_DKV)) == 0, RSWA_ERR_INVALID,
               "attn: unknown bits in wide (%d)", p->wide);
  const bool wide_out = !backward && (p->wide & RSWA_WIDE_OUT);
  RSWA_REQUIRE(rows_aligned(p->q, p->q_stride) && rows_aligned(p->k, p->k_stride) &&
                   rows_aligned(p->v, p->v_stride) &&
                   rows_aligned(p->out, p->out_stride, wide_out ? 4 : 2),
               RSWA_ERR_UNSUPPORTED, "attn: q/k/v/out rows must start 16-byte aligned");
  RSWA_REQUIRE(((uintptr_t)p->lse) % (wide_out ? 8 : 4) == 0, RSWA_ERR_UNSUPPORTED,
               "attn: lse misaligned");
  {
    // Tiles are fetched through 32-bit byte offsets.  The rows of one tile (at most
    // kMaxTileRows) must span less than 2 GiB; when a whole sequence does too, offsets count
    // from the sequence's first row, otherwise from each tile's (FAR kernels).
    const int64_t lim = (1ll << 31) - 65536;
    RSWA_REQUIRE(p->q_stride[1] >= 0 && p->k_stride[1] >= 0 && p->v_stride[1] >= 0 &&
                     p->q_stride[1] * 2 < lim / kMaxTileRows && p->k_stride[1] * 2 < lim / kMaxTileRows &&
                     p->v_stride[1] * 2 < lim / kMaxTileRows,
                 RSWA_ERR_UNSUPPORTED,
                 "attn: row stride of q, k or v is negative or %lld bytes or more",
                 (long long)(lim / kMaxTileRows));
    // packed: judged on the whole pack (no sequence is longer)
    const int64_t rq = packed ? p->total_q : p->seqlen_q, rk = packed ? p->total_k : p->seqlen_k;
    a.far = (p->addressing == RSWA_ADDR_FAR) || rq * p->q_stride[1] * 2 >= lim ||
            rk * p->k_stride[1] * 2 >= lim || rk * p->v_stride[1] * 2 >= lim ||
            (backward && rq * p->dout_stride[1] * 2 >= lim);
  }

  a.q = p->q;
  a.k = p->k;
  a.v = p->v;
  a.out = p->out;
  a.lse = p->lse;
  a.dout = p->dout;
  a.dq = p->dq;
  a.dk = p->dk;
  a.dv = p->dv;
  a.k2 = a.v2 = nullptr;
  a.dk2 = a.dv2 = nullptr;
  a.seg = INT32_MAX;
  if (p->seg_rows != 0) {
    RSWA_REQUIRE(!packed, RSWA_ERR_UNSUPPORTED, "attn: two key ranges (seg_rows) in dense mode only");
    RSWA_REQUIRE(p->num_sink == 0, RSWA_ERR_UNSUPPORTED, "attn: two key ranges (seg_rows) with sink keys");
    RSWA_REQUIRE(p->seg_rows > 0 && p->seg_rows % kDkvKeysPerBlock == 0 && p->seg_rows < p->seqlen_k,
                 RSWA_ERR_UNSUPPORTED,
                 "attn: seg_rows %d must be a positive multiple of %d below seqlen_k %d", p->seg_rows,
                 kDkvKeysPerBlock, p->seqlen_k);
    RSWA_REQUIRE(p->k2 && p->v2, RSWA_ERR_INVALID, "attn: seg_rows given but k2 / v2 null");
    RSWA_REQUIRE(((uintptr_t)p->k2) % 16 == 0 && ((uintptr_t)p->v2) % 16 == 0, RSWA_ERR_UNSUPPORTED,
                 "attn: k2 / v2 rows must start 16-byte aligned");
    if (backward) {
      RSWA_REQUIRE(p->dk2 && p->dv2, RSWA_ERR_INVALID, "attn_bwd: seg_rows given but dk2 / dv2 null");
      RSWA_REQUIRE(((uintptr_t)p->dk2) % 16 == 0 && ((uintptr_t)p->dv2) % 16 == 0,
                   RSWA_ERR_UNSUPPORTED, "attn_bwd: dk2 / dv2 rows must start 16-byte aligned");
    }
    a.k2 = p->k2;
    a.v2 = p->v2;
    a.dk2 = p->dk2;
    a.dv2 = p->dv2;
    a.seg = p->seg_rows;
  }
  a.delta = nullptr;
  a.lse2 = nullptr;
  a.dkv_part = nullptr;
  a.dkv_count = nullptr;
  a.nsplit = 1;
  a.n_count = 0;
  a.sink_part = nullptr;
  a.sink_count = nullptr;
  a.sink_chunks = 0;
  a.ds = nullptr;
  a.ds_nkb = 0;
  a.ds_slots = 0;
  a.cu_q = p->cu_seqlens_q;
  a.cu_k = p->cu_seqlens_k;
  for (int i = 0; i < 3; i++) {
    a.q_st[i] = p->q_stride[i];
    a.k_st[i] = p->k_stride[i];
    a.v_st[i] = p->v_stride[i];
    a.o_st[i] = p->out_stride[i];
    a.lse_st[i] = p->lse_stride[i];
    a.do_st[i] = p->dout_stride[i];
    a.dq_st[i] = p->dq_stride[i];
    a.dk_st[i] = p->dk_stride[i];
    a.dv_st[i] = p->dv_stride[i];
  }
  if (packed) {
    a.q_st[0] = a.k_st[0] = a.v_st[0] = a.o_st[0] = a.lse_st[0] = 0;
    a.do_st[0] = a.dq_st[0] = a.dk_st[0] = a.dv_st[0] = 0;
  }
  a.rows_q = packed ? p->total_q : (int64_t)p->batch * p->seqlen_q;
  a.rows_k = packed ? p->total_k : (int64_t)p->batch * p->seqlen_k;
  a.batch = p->batch;
  a.heads_q = p->heads_q;
  a.heads_kv = p->heads_kv;
  a.group = p->heads_q / p->heads_kv;
  a.seqlen_q = p->seqlen_q;
  a.seqlen_k = p->seqlen_k;
  // The kernels' mask arithmetic (row + shift +- window, key - row - shift) runs in 32 bits:
  // lengths and an explicit shift stay below 2^28, and a window that reaches that far is the
  // unbounded one.
  constexpr int64_t kMaskLim = 1ll << 28;
  RSWA_REQUIRE((packed ? std::max(p->total_q, p->total_k) : (int64_t)std::max(p->seqlen_q, p->seqlen_k)) < kMaskLim,
               RSWA_ERR_UNSUPPORTED, "attn: sequences of 2^28 rows or more");
  RSWA_REQUIRE(!p->shift_explicit || (p->shift > -kMaskLim && p->shift < kMaskLim), RSWA_ERR_UNSUPPORTED,
               "attn: explicit mask shift %lld out of range (|shift| < 2^28)", (long long)p->shift);
  a.wl = (p->window_left < 0 || p->window_left >= kMaskLim) ? -1 : p->window_left;
  a.wr = p->causal ? 0 : ((p->window_right < 0 || p->window_right >= kMaskLim) ? -1 : p->window_right);
  a.n_sink = p->num_sink;
  a.shift_explicit = p->shift_explicit != 0;
  a.shift_val = p->shift;
  a.dq_accumulate = backward && p->dq_accumulate != 0;
  a.out_accumulate = !backward && p->out_accumulate != 0;
  a.wide_out = wide_out;
  a.wide_dq = backward && (p->wide & RSWA_WIDE_DQ);
  a.wide_dkv = backward && (p->wide & RSWA_WIDE_DKV);
  a.dkv_accumulate = a.wide_dkv && p->dkv_accumulate != 0;
  RSWA_REQUIRE(!(backward && p->dkv_accumulate && !a.wide_dkv), RSWA_ERR_INVALID,
               "attn_bwd: dkv_accumulate needs fp32 dk / dv (RSWA_WIDE_DKV)");
  RSWA_REQUIRE(!(a.wide_dkv && p->num_sink > 0 && a.wl >= 0), RSWA_ERR_UNSUPPORTED,
               "attn_bwd: fp32 dk / dv (RSWA_WIDE_DKV) with sink keys under a bounded window");
  a.n_tile = 0;
  a.n_work = 0;
  {
    // Heaviest tiles first: compare the number of keys the first and the last query row
    // see, and the number of query rows that see the first and the last key (packed
    // batches: judged on the average sequence; the order affects speed only).
    const int64_t lq = packed ? std::max<int64_t>(1, p->total_q / std::max(1, p->batch)) : p->seqlen_q;
    const int64_t lk = packed ? std::max<int64_t>(1, p->total_k / std::max(1, p->batch)) : p->seqlen_k;
    const int64_t sh = a.shift_explicit ? a.shift_val : lk - lq;
    auto keys_of = [&](int64_t i) {
      const int64_t hi = a.wr >= 0 ? std::min(lk - 1, i + sh + a.wr) : lk - 1;
      const int64_t lo = a.wl >= 0 ? std::max<int64_t>(0, i + sh - a.wl) : 0;
      return std::max<int64_t>(0, hi - lo + 1) +
             std::max<int64_t>(0, std::min<int64_t>(a.n_sink, std::min(lo, hi + 1)));
    };
    auto rows_of = [&](int64_t j) {
      const int64_t i_lo = a.wr >= 0 ? std::max<int64_t>(0, j - sh - a.wr) : 0;
      const int64_t i_hi = (a.wl >= 0 && j >= a.n_sink) ? std::min(lq - 1, j - sh + a.wl) : lq - 1;
      return std::max<int64_t>(0, i_hi - i_lo + 1);
    };
    a.rev_q = keys_of(lq - 1) > keys_of(0);
    a.rev_k = rows_of(lk - 1) > rows_of(0);
    // keys a query row sees on average (keys_of is piecewise linear: 17 samples)
    int64_t sum = 0;
    for (int t = 0; t <= 16; t++) sum += keys_of((lq - 1) * t / 16);
    a.avg_keys = (int32_t)std::min<int64_t>(sum / 17, INT32_MAX);
  }
  a.scale = p->softmax_scale;
  a.scale_log2 = p->softmax_scale * kLog2e;

  if (backward) {
    RSWA_REQUIRE(p->dout && p->dq && p->dk && p->dv, RSWA_ERR_INVALID, "attn_bwd: null tensor");
    RSWA_REQUIRE(rows_aligned(p->dout, p->dout_stride) &&
                     rows_aligned(p->dq, p->dq_stride, a.wide_dq ? 4 : 2) &&
                     rows_aligned(p->dk, p->dk_stride, a.wide_dkv ? 4 : 2) &&
                     rows_aligned(p->dv, p->dv_stride, a.wide_dkv ? 4 : 2),
                 RSWA_ERR_UNSUPPORTED, "attn_bwd: dout/dq/dk/dv rows must start 16-byte aligned");
    RSWA_REQUIRE(p->dout_stride[1] >= 0 && p->dout_stride[1] * 2 < ((1ll << 31) - 65536) / kMaxTileRows,
                 RSWA_ERR_UNSUPPORTED, "attn_bwd: row stride of dout is negative or too large");
    const BwdLayout L = bwd_layout(p, allow_split, allow_handoff);
    const uint64_t need = L.total_bytes;
    RSWA_REQUIRE(p->workspace != nullptr || need == 0, RSWA_ERR_INVALID,
                 "attn_bwd: null workspace");
    RSWA_REQUIRE(p->workspace_bytes >= need, RSWA_ERR_INVALID,
                 "attn_bwd: workspace %llu bytes < required %llu",
                 (unsigned long long)p->workspace_bytes, (unsigned long long)need);
    RSWA_REQUIRE(((uintptr_t)p->workspace) % 256 == 0, RSWA_ERR_INVALID,
                 "attn_bwd: workspace must be 256-byte aligned");
    a.lse2 = (float*)p->workspace;
    a.delta = (float*)((char*)p->workspace + delta_bytes(p));
    a.nsplit = L.nsplit;
    a.n_count = L.n_count;
    a.dkv_count = (int32_t*)((char*)p->workspace + L.count_off);
    a.dkv_part = (float*)((char*)p->workspace + L.part_off);
    a.sink_chunks = L.sink_chunks;
    a.sink_part = L.sink_chunks ? (float*)((char*)p->workspace + L.sink_off) : nullptr;
    a.sink_count = a.dkv_count + L.sink_count_index;
    if (L.ds_bytes) {
      a.ds = (char*)p->workspace + L.ds_off;
      a.ds_nkb = L.ds_nkb;
      a.ds_slots = L.ds_slots;
    }
    // one load reaches from a row's lse2 to its delta, one array further on
    RSWA_REQUIRE(delta_bytes(p) < (1ull << 31) - 65536, RSWA_ERR_UNSUPPORTED,
                 "attn_bwd: rows * heads_q = %lld: each statistics array must stay below 2 GiB "
                 "(536 854 528 (row, q head) pairs)",
                 (long long)(delta_bytes(p) / 4));
  }
  return RSWA_OK;
}

}  // namespace rswa

extern "C" uint64_t rswa_attn_bwd_workspace_bytes(const rswa_attn_params* p) {
  return rswa::bwd_workspace_bytes(p);
}

extern "C" int rswa_attn_bwd_handoff_active(const rswa_attn_params* p) {
  return rswa::bwd_layout(p, true, true).ds_bytes != 0;
}
