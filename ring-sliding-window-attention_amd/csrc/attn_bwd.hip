// Band / sink attention backward for gfx950, without atomics.
//
// Replaces flash-attn's backward as wrapped at ring_swa/ops/wrap_flash.py:276-429.
// Three launches on the caller's stream:
//   PREP : delta[h][row] = sum_d dO * O   (fp32, in the caller's workspace)
//   DKDV : one block (8 waves) owns 128 keys of one (sequence, kv head), keeps their K and
//          V tiles in LDS and walks the query tiles (64 rows) that can see them, for every
//          q head of the GQA group; wave (wk, wq) handles key columns 32 wk.. of query rows
//          32 wq.. of each tile; dK^T / dV^T partials stay in registers for the whole walk,
//          the two query halves are added through LDS at the end and written once
//   DQ   : one block owns 128 queries of one (sequence, q head) and walks the key tiles
//          (64 keys) it can see, like the forward kernel; dQ^T stays in registers
// S and dP are computed in both main kernels (7 GEMM units instead of 5).  That costs
// less here than fp32 atomics on dQ: the L2 retires about one fp32 atomic per clock per
// channel, which caps an atomic dQ far below the MFMA rate.  It also makes the result
// run-to-run deterministic.
//
// DKDV per (query half-tile, wave) (C layout: lane = key):
//   S = Q K^T, dP = dO V^T      A = Q / dO row fragments, B = K / V row fragments (all LDS)
//   P = exp2(S*c - lse*log2e), dS = P * (dP - delta)
//   dV^T += dO^T P, dK^T += Q^T dS   A = transposing LDS reads of dO / Q, B = P / dS (regs)
// DQ per (key tile, wave); wave w owns query columns 32w..32w+31 (C layout: lane = query):
//   S^T = K Q^T, dP^T = V dO^T  A = K / V row fragments from LDS, B = Q / dO fragments (regs)
//   dS^T as above with per-lane lse / delta
//   dQ^T += K^T dS^T            A = transposing LDS reads of K, B = dS^T (regs)
#include "attn_common.h"

namespace rswa {
namespace {

// ============================================================================
// dK / dV
// ============================================================================
template <int D>
struct DkvCfg {
  static constexpr int BM = 64;   // query rows per step
  static constexpr int BN = 128;  // keys per block
  static constexpr int THREADS = 512;  // 8 waves: 4 key groups x 2 query halves
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLK = D / 32;
  static constexpr int CPR = D / 8;   // 16-byte chunks per row
  static constexpr int ROWB = D * 2;  // bytes per row
  static constexpr int Q_TILE = BM * ROWB;
  static constexpr int KV_TILE = BN * ROWB;
  static constexpr int OFF_K = 0;
  static constexpr int OFF_V = KV_TILE;
  static constexpr int OFF_Q = 2 * KV_TILE;            // 2 buffers
  static constexpr int OFF_DO = OFF_Q + 2 * Q_TILE;    // 2 buffers
  static constexpr int OFF_ST = OFF_DO + 2 * Q_TILE;   // lse2[2][BM], delta[2][BM] fp32
  static constexpr int SMEM = OFF_ST + 4 * BM * 4;
  // end-of-walk reduction of the two query halves: per key group 2 matrices of
  // DBLK x 16 registers x 64 lanes fp32
  static constexpr int RED_PER_WK = 2 * DBLK * 16 * 64 * 4;
  static_assert(4 * RED_PER_WK <= SMEM, "reduction staging must fit");
};

template <typename T, int D>
__global__ __launch_bounds__(512) void attn_bwd_dkdv_kernel(const AttnArgs a) {
  using C = DkvCfg<D>;
  using M = Mma<T>;
  using V8 = typename M::V8;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int wid = logical_block_id(a.n_work);
  if (wid < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wk = wave & 3;   // key group: columns 32 wk .. 32 wk + 31 of the block's 128 keys
  const int wq = wave >> 2;  // query half: rows 32 wq .. 32 wq + 31 of each 64-row tile
  const int l32 = lane & 31;
  const int g = lane >> 5;
  const int i16 = lane & 15;
  const int u = lane >> 4;

  // ---- which (sequence, kv head, key tile) ---------------------------------
  const int slot = wid % a.n_tile;
  int rest = wid / a.n_tile;
  const int hk = rest % a.heads_kv;
  SeqInfo s;
  int kt;
  if (a.cu_q) {
    if (!locate_packed(a, slot, C::BN, true, s, kt)) return;
  } else {
    s.batch_idx = rest / a.heads_kv;
    s.q_row0 = s.k_row0 = 0;
    s.len_q = a.seqlen_q;
    s.len_k = a.seqlen_k;
    kt = slot;
  }
  const int b = s.batch_idx;
  const int len_q = s.len_q, len_k = s.len_k;
  const int j0 = kt * C::BN;
  if (j0 >= len_k) return;
  const int j_last = min(j0 + C::BN, len_k) - 1;
  const int shift = a.shift_explicit ? a.shift_val : len_k - len_q;

  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + (s.k_row0 + j0) * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + (s.k_row0 + j0) * a.v_st[1] + hk * a.v_st[2];
  T* dk_ptr = (T*)a.dk + b * a.dk_st[0] + s.k_row0 * a.dk_st[1] + hk * a.dk_st[2];
  T* dv_ptr = (T*)a.dv + b * a.dv_st[0] + s.k_row0 * a.dv_st[1] + hk * a.dv_st[2];
  const int64_t ws_row0 = a.cu_q ? s.q_row0 : (int64_t)b * a.seqlen_q;

  // ---- query tiles that can see this key tile -------------------------------
  const int i_min = (a.wr >= 0) ? max(0, j0 - shift - a.wr) : 0;
  const int i_max =
      (a.wl >= 0 && j0 >= a.n_sink) ? min(len_q - 1, j_last - shift + a.wl) : len_q - 1;
  const int qt_lo = i_min / C::BM;
  const int n_qt = (i_max >= i_min) ? i_max / C::BM - qt_lo + 1 : 0;
  const int n_iter = n_qt * a.group;

  const int jw0 = j0 + wk * 32;  // first key column of this wave
  const int jc = jw0 + l32;      // this lane's key column

  f32x16 dk_acc[C::DBLK], dv_acc[C::DBLK];
#pragma unroll
  for (int d = 0; d < C::DBLK; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) {
      dk_acc[d][i] = 0.f;
      dv_acc[d][i] = 0.f;
    }

  // ---- lane-constant LDS offsets (swizzle folded: varying parts are XOR / immediates) ----
  // 16-byte row fragments: row = 32 blk + l32, chunk = 2 ks + g
  //   offset = (a_row ^ (ks << 5)) + blk * 32 * ROWB      (Q / dO: blk = wq; K / V: blk = wk)
  const int a_row = l32 * C::ROWB + ((g ^ swz_f<C::CPR>(l32)) << 4);
  // transposing reads of Q / dO: rows 16 ks + 4 g + (i16 >> 2) and + 8, chunk = 4 d + lp
  //   offset = (t_row{0,1} ^ (d << 6)) + ks * 16 * ROWB
  const int rl = 4 * g + (i16 >> 2);
  const int lp = 2 * (u & 1) + ((i16 & 3) >> 1);
  const int t_row0 = rl * C::ROWB + ((lp ^ swz_f<C::CPR>(rl)) << 4) + (i16 & 1) * 8;
  const int t_row1 = (rl + 8) * C::ROWB + ((lp ^ swz_f<C::CPR>(rl + 8)) << 4) + (i16 & 1) * 8;

  // ---- tile movement: everything lands in LDS directly; lse, delta via one register ----
  float streg = 0.f;
  auto iter_coords = [&](int it, int& hq, int& i0) {
    hq = hk * a.group + it / n_qt;
    i0 = (qt_lo + it % n_qt) * C::BM;
  };
  auto load_iter = [&](int it, int buf) {
    int hq, i0;
    iter_coords(it, hq, i0);
    const T* q_ptr = (const T*)a.q + b * a.q_st[0] + (s.q_row0 + i0) * a.q_st[1] + hq * a.q_st[2];
    const T* do_ptr =
        (const T*)a.dout + b * a.do_st[0] + (s.q_row0 + i0) * a.do_st[1] + hq * a.do_st[2];
    g2lds_tile<T, D, C::BM, C::THREADS>(q_ptr, a.q_st[1], len_q - i0,
                                         smem + C::OFF_Q + buf * C::Q_TILE, tid);
    g2lds_tile<T, D, C::BM, C::THREADS>(do_ptr, a.do_st[1], len_q - i0,
                                         smem + C::OFF_DO + buf * C::Q_TILE, tid);
    if (tid < C::BM) {
      // lse in base-2 units; rows that must contribute nothing get +inf (P = 0)
      const int i = i0 + tid;
      float l = __builtin_inff();
      if (i < len_q) {
        l = a.lse[b * a.lse_st[0] + hq * a.lse_st[1] + (s.q_row0 + i) * a.lse_st[2]];
        l = (l == -__builtin_inff()) ? __builtin_inff() : l * kLog2e;
      }
      streg = l;
    } else if (tid < 2 * C::BM) {
      const int i = i0 + tid - C::BM;
      streg = (i < len_q) ? a.delta[(int64_t)hq * a.rows_q + ws_row0 + i] : 0.f;
    }
  };
  auto store_stats = [&](int buf) {
    if (tid < 2 * C::BM) *(float*)(smem + C::OFF_ST + buf * 2 * C::BM * 4 + tid * 4) = streg;
  };

  if (n_iter > 0) {
    g2lds_tile<T, D, C::BN, C::THREADS>(k_ptr, a.k_st[1], len_k - j0, smem + C::OFF_K, tid);
    g2lds_tile<T, D, C::BN, C::THREADS>(v_ptr, a.v_st[1], len_k - j0, smem + C::OFF_V, tid);
    load_iter(0, 0);
    store_stats(0);
  }
  __syncthreads();

  const char* k_lds = smem + C::OFF_K + wk * 32 * C::ROWB;
  const char* v_lds = smem + C::OFF_V + wk * 32 * C::ROWB;

  for (int it = 0; it < n_iter; it++) {
    const int buf = it & 1;
    int hq, i0;
    iter_coords(it, hq, i0);
    if (it + 1 < n_iter) load_iter(it + 1, buf ^ 1);
    const char* q_lds = smem + C::OFF_Q + buf * C::Q_TILE;
    const char* do_lds = smem + C::OFF_DO + buf * C::Q_TILE;
    const float* lse_lds = (const float*)(smem + C::OFF_ST + buf * 2 * C::BM * 4) + wq * 32;
    const float* delta_lds = lse_lds + C::BM;

    // Does any (query of this wave's half-tile, key of this wave) pair survive the mask?
    const int iw0 = i0 + wq * 32;
    const int iw1 = min(iw0 + 32, len_q) - 1;
    const int jw1 = jw0 + 31;
    const bool needed = iw0 < len_q && jw0 < len_k &&
                        (a.wr < 0 || jw0 <= iw1 + shift + a.wr) &&
                        (a.wl < 0 || jw1 >= iw0 + shift - a.wl || jw0 < a.n_sink);
    if (needed) {
      // ---- S = Q K^T and dP = dO V^T (rows = queries, lane = key column) ------
      f32x16 sacc, pacc;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        sacc[i] = 0.f;
        pacc[i] = 0.f;
      }
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ks++) {
        const int off = a_row ^ (ks << 5);
        const V8 qa = *(const V8*)(q_lds + off + wq * 32 * C::ROWB);
        const V8 kb = *(const V8*)(k_lds + off);
        const V8 da = *(const V8*)(do_lds + off + wq * 32 * C::ROWB);
        const V8 vb = *(const V8*)(v_lds + off);
        sacc = M::mfma32(qa, kb, sacc);
        pacc = M::mfma32(da, vb, pacc);
      }

      // ---- P and dS -----------------------------------------------------------
      const bool full = iw0 + 31 < len_q && jw1 < len_k &&
                        (a.wr < 0 || jw1 <= iw0 + shift + a.wr) &&
                        (a.wl < 0 || jw0 >= iw0 + 31 + shift - a.wl || jw1 < a.n_sink);
      // key position relative to the aligned diagonal of row iw0: rel(i) = rel0 - (i - iw0)
      const int rel0 = jc - iw0 - shift;
      const int rel_hi = (a.wr < 0) ? (1 << 30) : a.wr;
      const int rel_lo = (a.wl < 0 || jc < a.n_sink) ? -(1 << 30) : -a.wl;
      const bool col_ok = jc < len_k;
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int rbase = 8 * i4 + 4 * g;
        const f32x4 l4 = *(const f32x4*)(lse_lds + rbase);
        const f32x4 d4 = *(const f32x4*)(delta_lds + rbase);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int i = 4 * i4 + e;
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[i], a.scale_log2, -l4[e]));
          if (!full) {
            const int rel = rel0 - (rbase + e);
            const bool ok = col_ok & (rel <= rel_hi) & (rel >= rel_lo);
            p = ok ? p : 0.f;  // rows past the end already have lse = +inf
          }
          sacc[i] = p;
          pacc[i] = p * (pacc[i] - d4[e]);
        }
      }

      // ---- dV^T += dO^T P ; dK^T += Q^T dS --------------------------------------
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        float pv[8], dsv[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
          pv[j] = sacc[8 * ks + j];
          dsv[j] = pacc[8 * ks + j];
        }
        const V8 pb = M::pack(pv);
        const V8 dsb = M::pack(dsv);
        const int rowoff = (wq * 32 + ks * 16) * C::ROWB;
#pragma unroll
        for (int d = 0; d < C::DBLK; d++) {
          const int off0 = (t_row0 ^ (d << 6)) + rowoff;
          const int off1 = (t_row1 ^ (d << 6)) + rowoff;
          dv_acc[d] = M::mfma32(tr_pair<V8>(do_lds + off0, do_lds + off1), pb, dv_acc[d]);
          dk_acc[d] = M::mfma32(tr_pair<V8>(q_lds + off0, q_lds + off1), dsb, dk_acc[d]);
        }
      }
    }

    if (it + 1 < n_iter) store_stats(buf ^ 1);
    __syncthreads();
  }

  // ---- add the two query halves (through LDS), then write dK, dV --------------------
  // (C layout: lane = key, regs = d)
  float* red = (float*)(smem + wk * C::RED_PER_WK);
  if (wq == 1) {
#pragma unroll
    for (int d = 0; d < C::DBLK; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const f32x4 kk = {dk_acc[d][4 * i4], dk_acc[d][4 * i4 + 1], dk_acc[d][4 * i4 + 2],
                          dk_acc[d][4 * i4 + 3]};
        const f32x4 vv = {dv_acc[d][4 * i4], dv_acc[d][4 * i4 + 1], dv_acc[d][4 * i4 + 2],
                          dv_acc[d][4 * i4 + 3]};
        *(f32x4*)(red + ((d * 4 + i4) * 64 + lane) * 4) = kk;
        *(f32x4*)(red + ((C::DBLK * 4 + d * 4 + i4) * 64 + lane) * 4) = vv;
      }
  }
  __syncthreads();
  if (wq == 0 && jc < len_k) {
#pragma unroll
    for (int d = 0; d < C::DBLK; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const f32x4 kk = *(const f32x4*)(red + ((d * 4 + i4) * 64 + lane) * 4);
        const f32x4 vv = *(const f32x4*)(red + ((C::DBLK * 4 + d * 4 + i4) * 64 + lane) * 4);
        const int col = d * 32 + 8 * i4 + 4 * g;
        const auto k4 = M::pack4((dk_acc[d][4 * i4] + kk[0]) * a.scale,
                                 (dk_acc[d][4 * i4 + 1] + kk[1]) * a.scale,
                                 (dk_acc[d][4 * i4 + 2] + kk[2]) * a.scale,
                                 (dk_acc[d][4 * i4 + 3] + kk[3]) * a.scale);
        const auto v4 = M::pack4(dv_acc[d][4 * i4] + vv[0], dv_acc[d][4 * i4 + 1] + vv[1],
                                 dv_acc[d][4 * i4 + 2] + vv[2], dv_acc[d][4 * i4 + 3] + vv[3]);
        *(typename M::V4*)(dk_ptr + (int64_t)jc * a.dk_st[1] + col) = k4;
        *(typename M::V4*)(dv_ptr + (int64_t)jc * a.dv_st[1] + col) = v4;
      }
  }
}

// ============================================================================
// dQ
// ============================================================================
template <int D>
struct DqCfg {
  static constexpr int BM = 128;  // query rows per block
  static constexpr int BN = 64;   // keys per step
  static constexpr int THREADS = 256;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLK = D / 32;
  static constexpr int CPR = D / 8;
  static constexpr int ROWB = D * 2;
  static constexpr int CH = BN * CPR / THREADS;
  static constexpr int TILE = BN * ROWB;
  static constexpr int OFF_K = 0;         // 2 buffers
  static constexpr int OFF_V = 2 * TILE;  // 2 buffers
  static constexpr int SMEM = 4 * TILE;
  static constexpr int O_STRIDE = D * 2 + 16;
  static_assert(SMEM >= 4 * 32 * O_STRIDE, "epilogue staging must fit");
};

template <typename T, int D>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_kernel(const AttnArgs a) {
  using C = DqCfg<D>;
  using M = Mma<T>;
  using V8 = typename M::V8;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int wid = logical_block_id(a.n_work);
  if (wid < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int g = lane >> 5;
  const int i16 = lane & 15;
  const int u = lane >> 4;

  const int hg = wid % a.group;
  int rest = wid / a.group;
  const int slot = rest % a.n_tile;
  rest /= a.n_tile;
  const int hk = rest % a.heads_kv;
  const int hq = hk * a.group + hg;
  SeqInfo s;
  int qt;
  if (a.cu_q) {
    if (!locate_packed(a, slot, C::BM, false, s, qt)) return;
  } else {
    s.batch_idx = rest / a.heads_kv;
    s.q_row0 = s.k_row0 = 0;
    s.len_q = a.seqlen_q;
    s.len_k = a.seqlen_k;
    qt = slot;
  }
  const int b = s.batch_idx;
  const int len_q = s.len_q, len_k = s.len_k;
  const int i0 = qt * C::BM;
  if (i0 >= len_q) return;

  const T* q_ptr = (const T*)a.q + b * a.q_st[0] + s.q_row0 * a.q_st[1] + hq * a.q_st[2];
  const T* do_ptr = (const T*)a.dout + b * a.do_st[0] + s.q_row0 * a.do_st[1] + hq * a.do_st[2];
  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + s.k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + s.k_row0 * a.v_st[1] + hk * a.v_st[2];
  T* dq_ptr = (T*)a.dq + b * a.dq_st[0] + s.q_row0 * a.dq_st[1] + hq * a.dq_st[2];
  const int64_t ws_row0 = a.cu_q ? s.q_row0 : (int64_t)b * a.seqlen_q;

  // ---- key tiles this block visits (same rule as the forward kernel) -----------
  const int i_last = min(i0 + C::BM, len_q) - 1;
  const int lo_blk = row_bounds(a, i0, len_q, len_k).lo;
  const int hi_blk = row_bounds(a, i_last, len_q, len_k).hi;
  const bool band = hi_blk >= lo_blk;
  const int t_lo = band ? lo_blk / C::BN : (1 << 29);
  const int n_band = band ? hi_blk / C::BN - t_lo + 1 : 0;
  const int sink_keys = max(0, min(min(a.n_sink, hi_blk + 1), lo_blk));
  const int n_sink_t = min((sink_keys + C::BN - 1) / C::BN, t_lo);
  const int n_tiles = n_sink_t + n_band;
  auto tile_of = [&](int it) { return it < n_sink_t ? it : t_lo + (it - n_sink_t); };

  const int r0 = i0 + wave * 32;
  const int iq = r0 + l32;
  const RowBounds rb = row_bounds(a, iq, len_q, len_k);
  const bool wave_valid = r0 < len_q;
  const bool wave_rows_full = r0 + 31 < len_q;
  const RowBounds wb_first = row_bounds(a, r0, len_q, len_k);
  const RowBounds wb_last = row_bounds(a, min(r0 + 31, len_q - 1), len_q, len_k);

  // Q / dO fragments (B operands): lane = query column, 8 consecutive d per k-step
  V8 qf[C::KSTEPS], dof[C::KSTEPS];
  float lse2 = __builtin_inff(), delta = 0.f;
  if (iq < len_q) {
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
      qf[ks] = *(const V8*)(q_ptr + (int64_t)iq * a.q_st[1] + ks * 16 + g * 8);
      dof[ks] = *(const V8*)(do_ptr + (int64_t)iq * a.do_st[1] + ks * 16 + g * 8);
    }
    const float l = a.lse[b * a.lse_st[0] + hq * a.lse_st[1] + (s.q_row0 + iq) * a.lse_st[2]];
    lse2 = (l == -__builtin_inff()) ? __builtin_inff() : l * kLog2e;
    delta = a.delta[(int64_t)hq * a.rows_q + ws_row0 + iq];
  } else {
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
      qf[ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
      dof[ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  f32x16 dq_acc[C::DBLK];
#pragma unroll
  for (int d = 0; d < C::DBLK; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) dq_acc[d][i] = 0.f;

  u32x4 kreg[C::CH], vreg[C::CH];
  auto load_tile = [&](int tile) {
    const int j0 = tile * C::BN;
#pragma unroll
    for (int n = 0; n < C::CH; n++) {
      const int c = tid + n * C::THREADS;
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      if (j0 + row < len_k) {
        kreg[n] = *(const u32x4*)(k_ptr + (int64_t)(j0 + row) * a.k_st[1] + col);
        vreg[n] = *(const u32x4*)(v_ptr + (int64_t)(j0 + row) * a.v_st[1] + col);
      } else {
        kreg[n] = u32x4{0, 0, 0, 0};
        vreg[n] = u32x4{0, 0, 0, 0};
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int n = 0; n < C::CH; n++) {
      const int c = tid + n * C::THREADS;
      const int row = c / C::CPR, ch = c % C::CPR;
      const int off = row * C::ROWB + swz<C::CPR>(row, ch) * 16;
      *(u32x4*)(smem + C::OFF_K + buf * C::TILE + off) = kreg[n];
      *(u32x4*)(smem + C::OFF_V + buf * C::TILE + off) = vreg[n];
    }
  };

  if (n_tiles > 0) {
    load_tile(tile_of(0));
    store_tile(0);
  }
  __syncthreads();

  for (int it = 0; it < n_tiles; it++) {
    const int buf = it & 1;
    const int j0 = tile_of(it) * C::BN;
    const int j1 = j0 + C::BN - 1;
    if (it + 1 < n_tiles) load_tile(tile_of(it + 1));

    const bool needed =
        wave_valid && j0 <= wb_last.hi && (j1 >= wb_first.lo || j0 < a.n_sink);
    if (needed) {
      const char* k_lds = smem + C::OFF_K + buf * C::TILE;
      const char* v_lds = smem + C::OFF_V + buf * C::TILE;
      // S^T = K Q^T and dP^T = V dO^T (rows = keys, lane = query column)
      f32x16 sacc[2], pacc[2];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          sacc[t][i] = 0.f;
          pacc[t][i] = 0.f;
        }
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ks++) {
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const int row = t * 32 + l32;
          const int off = row * C::ROWB + swz<C::CPR>(row, ks * 2 + g) * 16;
          sacc[t] = M::mfma32(*(const V8*)(k_lds + off), qf[ks], sacc[t]);
          pacc[t] = M::mfma32(*(const V8*)(v_lds + off), dof[ks], pacc[t]);
        }
      }
      const bool full = wave_rows_full && j1 <= wb_first.hi &&
                        (j0 >= wb_last.lo || j1 < a.n_sink);
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[t][i], a.scale_log2, -lse2));
          if (!full) {
            const int j = j0 + t * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
            const bool ok = j <= rb.hi && (j >= rb.lo || j < a.n_sink);
            p = ok ? p : 0.f;
          }
          pacc[t][i] = p * (pacc[t][i] - delta);
        }
      // dQ^T[d, query] += K^T dS^T
      const int rlane = 4 * g + (i16 >> 2);
      const int half = (i16 & 1) * 8;
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++) {
        float dsv[8];
#pragma unroll
        for (int j = 0; j < 8; j++) dsv[j] = pacc[s4 >> 1][8 * (s4 & 1) + j];
        const V8 dsb = M::pack(dsv);
        const int row = s4 * 16 + rlane;
#pragma unroll
        for (int d = 0; d < C::DBLK; d++) {
          const int ch = 4 * d + 2 * (u & 1) + ((i16 & 3) >> 1);
          const int off0 = row * C::ROWB + swz<C::CPR>(row, ch) * 16 + half;
          const int off1 = (row + 8) * C::ROWB + swz<C::CPR>(row + 8, ch) * 16 + half;
          dq_acc[d] = M::mfma32(tr_pair<V8>(k_lds + off0, k_lds + off1), dsb, dq_acc[d]);
        }
      }
    }
    if (it + 1 < n_tiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: dq = scale * acc, transposed through LDS for 16-byte stores ------
  char* stage = smem + wave * 32 * C::O_STRIDE;
#pragma unroll
  for (int d = 0; d < C::DBLK; d++)
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++) {
      const auto h4 = M::pack4(dq_acc[d][4 * i4] * a.scale, dq_acc[d][4 * i4 + 1] * a.scale,
                               dq_acc[d][4 * i4 + 2] * a.scale, dq_acc[d][4 * i4 + 3] * a.scale);
      *(typename M::V4*)(stage + l32 * C::O_STRIDE + (d * 32 + 8 * i4 + 4 * g) * 2) = h4;
    }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < 32 * C::CPR / 64; n++) {
    const int c = lane + n * 64;
    const int row = c / C::CPR, col = (c % C::CPR) * 8;
    if (r0 + row < len_q) {
      const u32x4 val = *(const u32x4*)(stage + row * C::O_STRIDE + col * 2);
      *(u32x4*)(dq_ptr + (int64_t)(r0 + row) * a.dq_st[1] + col) = val;
    }
  }
}

// ============================================================================
// delta[h][row] = sum_d dO * O.  One 16-lane (D=128) or 8-lane (D=64) group per (row, head).
// ============================================================================
template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_prep_kernel(const AttnArgs a) {
  constexpr int LPR = D / 8;
  const int64_t unit = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;  // (row, head)
  const int c = (threadIdx.x % LPR) * 8;
  if (unit >= a.rows_q * a.heads_q) return;
  const int h = (int)(unit % a.heads_q);
  const int64_t row = unit / a.heads_q;
  int64_t o_off, do_off;
  if (a.cu_q) {
    o_off = row * a.o_st[1];
    do_off = row * a.do_st[1];
  } else {
    const int64_t bb = row / a.seqlen_q, i = row % a.seqlen_q;
    o_off = bb * a.o_st[0] + i * a.o_st[1];
    do_off = bb * a.do_st[0] + i * a.do_st[1];
  }
  using V8 = typename Mma<T>::V8;
  const V8 o8 = *(const V8*)((const T*)a.out + o_off + h * a.o_st[2] + c);
  const V8 d8 = *(const V8*)((const T*)a.dout + do_off + h * a.do_st[2] + c);
  float acc = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) acc += (float)o8[j] * (float)d8[j];
#pragma unroll
  for (int m = LPR / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
  if (c == 0) a.delta[(int64_t)h * a.rows_q + row] = acc;
}

template <typename Kern>
int set_smem(Kern kern, int bytes, bool& configured, const char* what) {
  if (!configured) {  // benign race: the attribute call is idempotent
    hipError_t e =
        hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(RSWA_ERR_LAUNCH, "%s: set smem: %s", what, hipGetErrorString(e));
    configured = true;
  }
  return RSWA_OK;
}

template <typename T, int D>
int launch_bwd(AttnArgs& a, hipStream_t stream, int phases) {
  const int64_t units = a.rows_q * a.heads_q;
  if (units > 0 && (phases & RSWA_BWD_PREP)) {
    const unsigned blocks = (unsigned)ceil_div(units * (D / 8), 256);
    hipLaunchKernelGGL((attn_bwd_prep_kernel<T, D>), dim3(blocks), dim3(256), 0, stream, a);
    int rc = check_launch("attn_bwd prep");
    if (rc != RSWA_OK) return rc;
  }
  if (phases & RSWA_BWD_DKDV) {
    using C = DkvCfg<D>;
    if (a.cu_q) {
      a.n_tile = (int)(ceil_div(a.rows_k, C::BN) + a.batch);
      a.n_work = a.n_tile * a.heads_kv;
    } else {
      a.n_tile = (int)ceil_div(a.seqlen_k, C::BN);
      a.n_work = a.n_tile * a.heads_kv * a.batch;
    }
    if (a.n_work > 0) {
      auto kern = attn_bwd_dkdv_kernel<T, D>;
      static bool configured = false;
      int rc = set_smem(kern, C::SMEM, configured, "attn_bwd dkdv");
      if (rc != RSWA_OK) return rc;
      hipLaunchKernelGGL(kern, dim3(padded_grid(a.n_work)), dim3(C::THREADS), C::SMEM, stream, a);
      rc = check_launch("attn_bwd dkdv");
      if (rc != RSWA_OK) return rc;
    }
  }
  if (phases & RSWA_BWD_DQ) {
    using C = DqCfg<D>;
    if (a.cu_q) {
      a.n_tile = (int)(ceil_div(a.rows_q, C::BM) + a.batch);
      a.n_work = a.n_tile * a.heads_q;
    } else {
      a.n_tile = (int)ceil_div(a.seqlen_q, C::BM);
      a.n_work = a.n_tile * a.heads_q * a.batch;
    }
    if (a.n_work > 0) {
      auto kern = attn_bwd_dq_kernel<T, D>;
      static bool configured = false;
      int rc = set_smem(kern, C::SMEM, configured, "attn_bwd dq");
      if (rc != RSWA_OK) return rc;
      hipLaunchKernelGGL(kern, dim3(padded_grid(a.n_work)), dim3(C::THREADS), C::SMEM, stream, a);
      rc = check_launch("attn_bwd dq");
      if (rc != RSWA_OK) return rc;
    }
  }
  return RSWA_OK;
}

}  // namespace
}  // namespace rswa

extern "C" int rswa_attn_bwd_phases(const rswa_attn_params* p, void* stream, int phases) {
  using namespace rswa;
  AttnArgs a;
  int rc = fill_args(p, true, a);
  if (rc != RSWA_OK) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (p->dtype == RSWA_BF16) {
    return p->head_dim == 128 ? launch_bwd<__bf16, 128>(a, st, phases)
                              : launch_bwd<__bf16, 64>(a, st, phases);
  }
  return p->head_dim == 128 ? launch_bwd<_Float16, 128>(a, st, phases)
                            : launch_bwd<_Float16, 64>(a, st, phases);
}

extern "C" int rswa_attn_bwd(const rswa_attn_params* p, void* stream) {
  return rswa_attn_bwd_phases(p, stream, RSWA_BWD_PREP | RSWA_BWD_DKDV | RSWA_BWD_DQ);
}
