// Band / sink attention forward for gfx950: bf16|fp16 MFMA, K/V tiles in LDS,
// online softmax, tiles outside the visible band never touched.
//
// Replaces flash-attn's forward as wrapped at ring_swa/ops/wrap_flash.py:168-273.
//
// One block = 4 waves x 32 query rows sharing every K/V tile it loads: either 64 rows of
// TWO q heads of one GQA group (group size even) or 128 rows of one q head; two blocks fit a
// compute unit (two waves per SIMD, from independent blocks).  Per 64-key
// tile a wave computes S^T = K Q^T (keys x queries) with v_mfma_f32_32x32x16, so each
// lane owns ONE query column: the row max / sum of the online softmax are in-lane
// reductions plus a single half-wave exchange, and P^T is already laid out as the B
// operand of O^T += V^T P^T.  V^T fragments come straight out of the row-major V tile
// with ds_read_b64_tr_b16.
//
// Pipeline.  K/V tiles are double-buffered in LDS and filled by buffer loads that land
// directly in LDS, issued one (V) and two (K) tiles ahead.  The buffers are SEPARATE
// static __shared__ arrays and the tile loop is unrolled by two, so that every access
// names its buffer statically: only then can the compiler tell that an in-flight load
// does not alias the LDS reads of the current tile, and not wait for it.  The waves of a
// block run in lock-step, one barrier per tile; the softmax of one block runs under the MFMAs
// of the compute unit's other block, and a block's prologue and epilogue under the other's
// tiles.  (An 8-wave block whose two halves ran half a tile apart -- the softmax of one half
// under the MFMAs of the other, two barriers per tile -- measured 5 % slower at window 4096
// and 24 % slower at head_dim 64 and window 1000: half the tile loads per row, but one
// block per compute unit and nothing to cover its prologue and epilogue.)
#include "attn_common.h"

namespace rswa {
namespace {

template <int D>
struct FwdCfg {
  static constexpr int BN = 64;
  static constexpr int THREADS = 256;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLK = D / 32;
  static constexpr int CPR = D / 8;   // 16-byte chunks per row
  static constexpr int ROWB = D * 2;  // bytes per row
  static constexpr int TILE = BN * ROWB;
  static constexpr int O_STRIDE = D * 2 + 16;
  static_assert(TILE >= 32 * O_STRIDE, "one wave's epilogue staging fits one tile buffer");
};

template <typename T, int D, bool SKIP, bool FAR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attn_fwd_kernel(const AttnArgs a) {
  using C = FwdCfg<D>;
  constexpr int NW = C::THREADS / 64;
  using M = Mma<T>;
  using V8 = typename M::V8;
  __shared__ __attribute__((aligned(1024))) char k_s0[C::TILE];
  __shared__ __attribute__((aligned(1024))) char k_s1[C::TILE];
  __shared__ __attribute__((aligned(1024))) char v_s0[C::TILE];
  __shared__ __attribute__((aligned(1024))) char v_s1[C::TILE];

  const int wid = logical_block_id(a.n_work);
  if (wid < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;
  const int i16 = lane & 15;
  const int u = lane >> 4;

  // ---- which (sequence, kv head, q tile, q head(s)) -------------------------
  // pair mode: waves 0-1 and 2-3 take the same 64 rows of two neighbouring q heads;
  // row mode: the 4 waves take 128 consecutive rows of one q head
  const bool pair = (a.group & 1) == 0;
  const int units = pair ? a.group >> 1 : a.group;  // blocks per (kv head, q tile)
  const int bm = pair ? 16 * NW : 32 * NW;          // query rows per block
  const int hu = wid % units;
  int rest = wid / units;
  const int slot = a.rev_q ? a.n_tile - 1 - rest % a.n_tile : rest % a.n_tile;
  rest /= a.n_tile;
  const int hk = rest % a.heads_kv;
  const int hq = hk * a.group + (pair ? 2 * hu + (wave >> 1) : hu);
  SeqInfo s;
  int qt;
  if (a.cu_q) {
    if (!locate_packed(a, slot, pair ? 6 : 7, false, s, qt)) return;
  } else {
    s.batch_idx = rest / a.heads_kv;
    s.q_row0 = s.k_row0 = 0;
    s.len_q = a.seqlen_q;
    s.len_k = a.seqlen_k;
    qt = slot;
  }
  const int b = s.batch_idx;
  const int len_q = s.len_q, len_k = s.len_k;
  const int i0 = qt * bm;
  if (i0 >= len_q) return;

  const T* q_ptr = (const T*)a.q + b * a.q_st[0] + s.q_row0 * a.q_st[1] + hq * a.q_st[2];
  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + s.k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + s.k_row0 * a.v_st[1] + hk * a.v_st[2];
  // (element offsets: out is T or, as a ring accumulator, fp32; lse is fp32 or fp64)
  const int64_t o_off = b * a.o_st[0] + s.q_row0 * a.o_st[1] + hq * a.o_st[2];
  const int64_t lse_off = b * a.lse_st[0] + hq * a.lse_st[1] + s.q_row0 * a.lse_st[2];

  // ---- key tiles this block visits -----------------------------------------
  const int i_last = min(i0 + bm, len_q) - 1;
  const int lo_blk = row_bounds(a, i0, len_q, len_k).lo;
  const int hi_blk = row_bounds(a, i_last, len_q, len_k).hi;
  const bool band = hi_blk >= lo_blk;
  const int t_lo = band ? lo_blk / C::BN : (1 << 29);
  const int n_band = band ? hi_blk / C::BN - t_lo + 1 : 0;
  const int sink_keys = max(0, min(min(a.n_sink, hi_blk + 1), lo_blk));
  const int n_sink_t = min((sink_keys + C::BN - 1) / C::BN, t_lo);
  const int n_tiles = n_sink_t + n_band;
  auto tile_of = [&](int it) { return it < n_sink_t ? it : t_lo + (it - n_sink_t); };

  // ---- this wave's rows ----------------------------------------------------
  const int r0 = i0 + (pair ? wave & 1 : wave) * 32;
  const int iq = r0 + l32;
  const RowBounds rb = row_bounds(a, iq, len_q, len_k);
  const bool wave_rows_full = r0 + 31 < len_q;
  const RowBounds wb_first = row_bounds(a, r0, len_q, len_k);
  const RowBounds wb_last = row_bounds(a, min(r0 + 31, len_q - 1), len_q, len_k);

  // Q fragments (B operand of K Q^T): lane = query column, 8 consecutive d per k-step.
  V8 qf[C::KSTEPS];
#pragma unroll
  for (int ks = 0; ks < C::KSTEPS; ks++) {
    if (iq < len_q) {
      qf[ks] = *(const V8*)(q_ptr + (int64_t)iq * a.q_st[1] + ks * 16 + g * 8);
    } else {
      qf[ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  f32x16 o_acc[C::DBLK];
#pragma unroll
  for (int d = 0; d < C::DBLK; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) o_acc[d][i] = 0.f;
  float m_run = -__builtin_inff();  // running max of raw scores (shared by the lane pair)
  float l_run = 0.f;                // this lane's share of the running sum

  // ---- lane-constant LDS offsets (swizzle folded into XOR / immediate parts) ----
  // K row fragments (16-byte reads): row = 32 t + l32, chunk = 2 ks + g
  //   offset = (a_row ^ (ks << 5)) + t * 32 * ROWB
  const int a_row = l32 * C::ROWB + ((g ^ swz_f<C::CPR>(l32)) << 4);
  // transposing reads of V: rows 16 s4 + 4 g + (i16 >> 2) and + 8, chunk = 4 d + lp
  //   offset = (t_row{0,1} ^ (d << 6)) + s4 * 16 * ROWB
  const int rl = 4 * g + (i16 >> 2);
  const int lp = 2 * (u & 1) + ((i16 & 3) >> 1);
  const int t_row0 = rl * C::ROWB + ((lp ^ swz_f<C::CPR>(rl)) << 4) + (i16 & 1) * 8;
  const int t_row1 = (rl + 8) * C::ROWB + ((lp ^ swz_f<C::CPR>(rl + 8)) << 4) + (i16 & 1) * 8;

  // ---- tile DMA: rows past len_k read as zero ---------------------------------
  TileDma<D, C::BN, C::THREADS> k_dma, v_dma;
  k_dma.init(a.k_st[1], tid);
  v_dma.init(a.v_st[1], tid);
  const int k_row_bytes = (int)(a.k_st[1] * 2), v_row_bytes = (int)(a.v_st[1] * 2);
  // (keys in two row ranges: the second range's tensors, at this batch entry and kv head)
  const T* k2_ptr = a.k2 ? (const T*)a.k2 + b * a.k_st[0] + hk * a.k_st[2] : k_ptr;
  const T* v2_ptr = a.v2 ? (const T*)a.v2 + b * a.v_st[0] + hk * a.v_st[2] : v_ptr;
  auto load_k = [&](int it, char* dst) __attribute__((always_inline)) {
    const KeySeg<T> g = key_seg(k_ptr, k2_ptr, a.seg, tile_of(it) * C::BN, len_k);
    k_dma.load(tile_src<C::BN, FAR>(g.base, g.row0, g.rows, k_row_bytes, C::ROWB), dst);
  };
  auto load_v = [&](int it, char* dst) __attribute__((always_inline)) {
    const KeySeg<T> g = key_seg(v_ptr, v2_ptr, a.seg, tile_of(it) * C::BN, len_k);
    v_dma.load(tile_src<C::BN, FAR>(g.base, g.row0, g.rows, v_row_bytes, C::ROWB), dst);
  };

  // ---- pieces of one tile ------------------------------------------------------
  // S^T[key, query] = K Q^T
  auto qk = [&](const char* kc, f32x16(&sacc)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) sacc[t][i] = 0.f;
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
      const int off = a_row ^ (ks << 5);
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const V8 kf = *(const V8*)(kc + off + t * 32 * C::ROWB);
        sacc[t] = M::mfma32(kf, qf[ks], sacc[t]);
      }
    }
  };
  // mask of an edge tile: visible iff j <= hi and (j >= lo or j < n_sink)
  auto mask = [&](int it, f32x16(&sacc)[2]) __attribute__((always_inline)) {
    const int j0 = tile_of(it) * C::BN;
    const int j1 = j0 + C::BN - 1;
    const bool full =
        wave_rows_full && j1 <= wb_first.hi && (j0 >= wb_last.lo || j1 < a.n_sink);
    if (!full) {
      const int hi_rel = rb.hi - j0;
      const int lo_rel = rb.lo - j0;
      const int sink_rel = a.n_sink - j0;
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int j = t * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          const bool ok = (j <= hi_rel) & ((j >= lo_rel) | (j < sink_rel));
          sacc[t][i] = ok ? sacc[t][i] : -__builtin_inff();
        }
    }
  };
  // online softmax of one tile (raw-score max, exponent in base 2); P^T packed for the
  // PV MFMAs; returns the factor the running output must be scaled by
  auto softmax = [&](f32x16(&sacc)[2], V8(&pb)[4]) __attribute__((always_inline)) -> float {
    float mx = sacc[0][0];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[t][i]);
    mx = halfwave_max(mx);
    // The reference point of the exponentials moves only when the maximum has grown by
    // more than 2^8: until then P <= 256, exact in fp32 sums and harmless in 16 bits, and
    // the rescale of the running output is skipped for almost every tile.
    const float m_new = fmaxf(m_run, mx);
    const bool bump = (m_new - m_run) * a.scale_log2 > 8.f;  // true from -inf, false for NaN
    const float m_keep = bump ? m_new : m_run;
    const float m_use = (m_keep == -__builtin_inff()) ? 0.f : m_keep;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * a.scale_log2);
    const float mc = m_use * a.scale_log2;
    m_run = m_keep;
    float psum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++) {
      float pv[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        pv[j] = __builtin_amdgcn_exp2f(
            __builtin_fmaf(sacc[s4 >> 1][8 * (s4 & 1) + j], a.scale_log2, -mc));
        psum[j & 3] += pv[j];
      }
      pb[s4] = M::pack(pv);
      // keep the vector work in the vector phase: the packed P is opaque from here on
      asm volatile("" : "+v"(pb[s4]));
    }
    float psum_all = (psum[0] + psum[1]) + (psum[2] + psum[3]);
    asm volatile("" : "+v"(psum_all));
    l_run = l_run * alpha + psum_all;
    return alpha;
  };
  // O^T[d, query] = alpha * O^T + V^T P^T, in two parts
  auto rescale = [&](float alpha) __attribute__((always_inline)) {
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
      for (int d = 0; d < C::DBLK; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) o_acc[d][i] *= alpha;
    }
  };
  auto pv_acc = [&](const char* vc, const V8(&pb)[4]) __attribute__((always_inline)) {
#pragma unroll
    for (int s4 = 0; s4 < 4; s4++) {
#pragma unroll
      for (int d = 0; d < C::DBLK; d++) {
        const int off0 = (t_row0 ^ (d << 6)) + s4 * 16 * C::ROWB;
        const int off1 = (t_row1 ^ (d << 6)) + s4 * 16 * C::ROWB;
        o_acc[d] = M::mfma32(tr_pair<V8>(vc + off0, vc + off1), pb[s4], o_acc[d]);
      }
    }
  };

  // ---- tile loop ------------------------------------------------------------------------
  // Per tile: a vector section (mask + softmax of tile t, rescale of O), the block barrier,
  // a matrix section (O += P(t) V(t), S(t+1) = K(t+1) Q^T).  The barrier publishes K(t+1) and
  // V(t), loaded during the previous matrix section, and releases the buffers of K(t) and
  // V(t-1), last read before it: the loads of K(t+2) and V(t+1) into them follow it.
  f32x16 s_cur[2];
  auto prefetch = [&](int it, char* kfree, char* vn) __attribute__((always_inline)) {
    if (it + 2 < n_tiles) load_k(it + 2, kfree);
    if (it + 1 < n_tiles) load_v(it + 1, vn);
  };
  // A tile the block visits may hold no key that this wave's 32 rows can see (the block's
  // key range is as wide as the window plus all its rows): the wave then skips the tile's
  // work and only keeps the barrier.  With a short window that is a sizeable share: at
  // window 256 and 128 rows per block a wave needs 5 of the block's 7 tiles.
  // (SKIP is chosen by the host for short windows only: with a long window the test costs
  // more than the rare skipped tile saves.)
  auto wave_needs = [&](int it) __attribute__((always_inline)) -> bool {
    if constexpr (!SKIP) return it < n_tiles;
    const int j0 = tile_of(it) * C::BN;
    return it < n_tiles && r0 < len_q && j0 <= wb_last.hi &&
           (j0 + C::BN - 1 >= wb_first.lo || j0 < a.n_sink);
  };
  auto iter = [&](int it, const char* kn, char* kfree, const char* vc,
                  char* vn) __attribute__((always_inline)) {
    // without SKIP both are compile-time true: one path, and after the last tile S(t+1) is
    // computed from stale LDS contents and never used
    const bool need_cur = SKIP ? wave_needs(it) : true;
    const bool need_next = SKIP ? wave_needs(it + 1) : true;
    V8 pb[4];
    if (need_cur) {
      mask(it, s_cur);
      const float alpha = softmax(s_cur, pb);
      rescale(alpha);
    }
    wait_dma();
    lds_barrier();
    if (!(need_cur && need_next)) prefetch(it, kfree, vn);
    if (need_cur && need_next) {
      // matrix section as ONE basic block, LDS reads scheduled four fragments ahead of their
      // MFMA.  The tile loads ride between the MFMAs, one every fourth: issued in a row they
      // hold the wave for about 50 cycles apiece before its first MFMA.  No branch may split
      // the block, so past the last tile the last one is fetched again, into a buffer nobody
      // reads.
      load_k(min(it + 2, n_tiles - 1), kfree);
      load_v(min(it + 1, n_tiles - 1), vn);
      pv_acc(vc, pb);
      qk(kn, s_cur);
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
      static_for<32>([&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (i < 12) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        else if constexpr (i < 28) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        if constexpr (i % 4 == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      });
    } else if (need_cur) {
      pv_acc(vc, pb);
    } else if (need_next) {
      qk(kn, s_cur);
    }
  };

  if (n_tiles > 0) {
    load_k(0, k_s0);
    load_v(0, v_s0);
  }
  if (n_tiles > 1) load_k(1, k_s1);
  __syncthreads();
  if (wave_needs(0)) qk(k_s0, s_cur);
  for (int it = 0; it < n_tiles; it += 2) {
    iter(it, k_s1, k_s0, v_s0, v_s1);
    if (it + 1 < n_tiles) iter(it + 1, k_s0, k_s1, v_s1, v_s0);
  }
  __syncthreads();

  // ---- epilogue --------------------------------------------------------------
  const float l_tot = halfwave_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  // transpose O^T through LDS for coalesced 16-byte stores, one tile buffer per wave
  char* stage = wave == 0 ? k_s0 : wave == 1 ? k_s1 : wave == 2 ? v_s0 : v_s1;
  // out_accumulate: out / lse hold a running partial result; the block is merged into it with
  // the arithmetic of the merge kernel (merge_lse.hip), applied to the block's output after
  // its rounding to 16 bits -- the same bits as a forward into a temporary plus a merge.  The
  // rows' two weights wait in LDS behind the staged tile for the lanes that store the rows.
  float* wgt = (float*)(stage + 32 * C::O_STRIDE);
  static_assert(C::TILE >= 32 * C::O_STRIDE + 32 * 2 * 4, "weights fit behind the staged tile");
  {
    const float ninf = -__builtin_inff();
    float lse_new = l_tot > 0.f ? m_run * a.scale + __logf(l_tot) : ninf;
    float w_old = 0.f, w_new = 1.f;
    const int64_t lse_at = lse_off + (int64_t)iq * a.lse_st[2];
    if (a.out_accumulate && iq < len_q) {
      // (an fp64 running LSE enters the arithmetic as fp32, as in the merge kernel)
      const float la = a.wide_out ? (float)((const double*)a.lse)[lse_at] : a.lse[lse_at];
      const float lb = lse_new;
      const bool both_empty = (la == ninf) && (lb == ninf);
      const float diff = both_empty ? 0.f : lb - la;
      w_old = both_empty ? 0.f : 1.f / (1.f + __expf(diff));
      w_new = both_empty ? 0.f : 1.f / (1.f + __expf(-diff));
      lse_new = both_empty ? ninf : fmaxf(la, lb) + log1pf(__expf(-fabsf(diff)));
    }
    if (g == 0 && iq < len_q) {
      if (a.wide_out) ((double*)a.lse)[lse_at] = (double)lse_new;
      else a.lse[lse_at] = lse_new;
    }
    // (the staging buffer is the wave's own: its writes only have to land before its reads)
#pragma unroll
    for (int d = 0; d < C::DBLK; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const auto h4 = M::pack4(o_acc[d][4 * i4] * inv, o_acc[d][4 * i4 + 1] * inv,
                                 o_acc[d][4 * i4 + 2] * inv, o_acc[d][4 * i4 + 3] * inv);
        *(typename M::V4*)(stage + l32 * C::O_STRIDE + (d * 32 + 8 * i4 + 4 * g) * 2) = h4;
      }
    if (g == 0) {
      wgt[2 * l32] = w_old;
      wgt[2 * l32 + 1] = w_new;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int n = 0; n < 32 * C::CPR / 64; n++) {
      const int c = lane + n * 64;
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      if (r0 + row < len_q) {
        V8 val = *(const V8*)(stage + row * C::O_STRIDE + col * 2);
        const int64_t at = o_off + (int64_t)(r0 + row) * a.o_st[1] + col;
        const float wo = a.out_accumulate ? wgt[2 * row] : 0.f;
        const float wn = a.out_accumulate ? wgt[2 * row + 1] : 1.f;
        if (a.wide_out) {
          // fp32 accumulator: the block's 16-bit values as fp32, or merged into what it holds
          float* dst = (float*)a.out + at;
          f32x4 y[2];
#pragma unroll
          for (int hh = 0; hh < 2; hh++) {
            f32x4 old = {0.f, 0.f, 0.f, 0.f};
            if (a.out_accumulate) old = *(const f32x4*)(dst + 4 * hh);
#pragma unroll
            for (int j = 0; j < 4; j++) {
              const float t0 = (wo == 0.f) ? 0.f : old[j] * wo;
              const float t1 = (wn == 0.f) ? 0.f : (float)val[4 * hh + j] * wn;
              y[hh][j] = t0 + t1;
            }
          }
          *(f32x4*)dst = y[0];
          *(f32x4*)(dst + 4) = y[1];
        } else {
          T* dst = (T*)a.out + at;
          if (a.out_accumulate) {
            const V8 old = *(const V8*)dst;
            float y[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
              // a zero weight must annihilate whatever the other side holds
              const float t0 = (wo == 0.f) ? 0.f : (float)old[j] * wo;
              const float t1 = (wn == 0.f) ? 0.f : (float)val[j] * wn;
              y[j] = t0 + t1;
            }
            val = M::pack(y);
          }
          *(V8*)dst = val;
        }
      }
    }
  }
}

// Explicit instantiations: with implicit instantiation alone this hipcc emits the host
// launch stubs of only some of the four variants.
#define RSWA_INSTANTIATE(T, D)                                                   \
  template __global__ void attn_fwd_kernel<T, D, false, false>(const AttnArgs); \
  template __global__ void attn_fwd_kernel<T, D, true, false>(const AttnArgs);  \
  template __global__ void attn_fwd_kernel<T, D, false, true>(const AttnArgs);  \
  template __global__ void attn_fwd_kernel<T, D, true, true>(const AttnArgs);
RSWA_INSTANTIATE(__bf16, 128)
RSWA_INSTANTIATE(__bf16, 64)
RSWA_INSTANTIATE(_Float16, 128)
RSWA_INSTANTIATE(_Float16, 64)
#undef RSWA_INSTANTIATE

template <typename T, int D>
int launch_fwd(AttnArgs& a, hipStream_t stream) {
  using C = FwdCfg<D>;
  const bool pair = (a.group & 1) == 0;
  const int bm = pair ? 64 : 128;
  const int units = (pair ? a.group / 2 : a.group) * a.heads_kv;  // blocks per q tile
  if (a.cu_q) {
    a.n_tile = (int)(ceil_div(a.rows_q, bm) + a.batch);
    a.n_work = a.n_tile * units;
  } else {
    a.n_tile = (int)ceil_div(a.seqlen_q, bm);
    a.n_work = a.n_tile * units * a.batch;
  }
  if (a.n_work == 0) return RSWA_OK;
  // keys a row sees at most; the per-wave tile skip pays when the rows of a block beyond one
  // wave's 32 add a tenth or more to that span
  const int64_t span = (a.wl < 0 || a.wr < 0) ? (int64_t)1 << 40 : (int64_t)a.wl + a.wr + 1;
  // (measured at window 1000 and 128-row blocks, where the skip would save a wave one tile in
  // eighteen: no difference either way, 0.435 against 0.431-0.441 ms)
  const bool skip = (bm - 32) * 10 >= span + bm;
  clear_launch_error();
  const dim3 grid(padded_grid(a.n_work)), block(C::THREADS);
  if (skip) {
    if (a.far) hipLaunchKernelGGL((attn_fwd_kernel<T, D, true, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((attn_fwd_kernel<T, D, true, false>), grid, block, 0, stream, a);
  } else {
    if (a.far) hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, false>), grid, block, 0, stream, a);
  }
  return check_launch("attn_fwd");
}

}  // namespace
}  // namespace rswa

extern "C" int rswa_attn_fwd(const rswa_attn_params* p, void* stream) {
  using namespace rswa;
  AttnArgs a;
  int rc = fill_args(p, false, a);
  if (rc != RSWA_OK) return rc;
  if (a.rows_q == 0) return RSWA_OK;
  hipStream_t st = (hipStream_t)stream;
  if (p->dtype == RSWA_BF16) {
    return p->head_dim == 128 ? launch_fwd<__bf16, 128>(a, st) : launch_fwd<__bf16, 64>(a, st);
  }
  return p->head_dim == 128 ? launch_fwd<_Float16, 128>(a, st) : launch_fwd<_Float16, 64>(a, st);
}
