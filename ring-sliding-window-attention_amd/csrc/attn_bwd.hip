// Band / sink attention backward for gfx950.
//
// Replaces flash-attn's backward as wrapped at ring_swa/ops/wrap_flash.py:276-429.
// Three launches on the caller's stream:
//   1. prep : delta[h][row] = sum_d dO*O (fp32) and zero of the fp32 dQ accumulator
//   2. main : one block owns 128 keys of one (sequence, kv head) and walks the query
//             tiles (64 rows) that can see them, for every q head of the GQA group;
//             dK^T / dV^T stay in registers for the whole walk, dQ goes out through
//             fp32 atomics
//   3. post : dq = cast(scale * dq_acc)
//
// Main-kernel data flow per (query tile, wave); wave w owns key columns 32w..32w+31:
//   S  = Q K^T, dP = dO V^T     A = Q / dO rows from LDS, B = K / V fragments (registers)
//   P  = exp2(S*c - lse*log2e), dS = P * (dP - delta)           (C layout: lane = key)
//   dV^T += dO^T P, dK^T += Q^T dS   A = transposing LDS reads of dO / Q, B = P / dS regs
//   dS^T -> LDS; dQ[:, d-slice] = dS K   A = transposing reads of dS^T, B = K^T fragments
#include "attn_common.h"

namespace rswa {
namespace {

// XOR swizzle of 16-byte chunks inside an LDS tile whose rows hold CH chunks (8 or 16).
// It makes both access patterns used here bank-conflict free: 16 consecutive rows at one
// logical chunk (MFMA row fragments, 16-byte reads) and 4 consecutive rows x 4 consecutive
// chunks (one phase of the transposing 8-byte reads).
template <int CH>
__device__ __forceinline__ int swz(int row, int chunk) {
  if constexpr (CH == 16) {
    return chunk ^ (((row & 3) << 2) | ((row >> 2) & 3));
  } else {
    static_assert(CH == 8, "rows of 8 or 16 chunks");
    return chunk ^ ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
  }
}

template <int D>
struct BwdCfg {
  static constexpr int BM = 64;   // query rows per step
  static constexpr int BN = 128;  // keys per block
  static constexpr int THREADS = 256;
  static constexpr int MI = BM / 32;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLK = D / 32;
  static constexpr int CPR = D / 8;                      // chunks per row of a [*, D] tile
  static constexpr int ROWB = D * 2;                     // bytes per row
  static constexpr int QCH = BM * CPR / THREADS;         // chunks per thread per Q (or dO) tile
  static constexpr int KCH = BN * CPR / THREADS;
  static constexpr int DQ_TILES = MI * DBLK / 4;         // dQ 32x32 tiles per wave
  static constexpr int Q_TILE = BM * ROWB;
  static constexpr int DS_ROWB = BM * 2;                 // dS^T tile: [BN keys][BM queries]
  static constexpr int DS_TILE = BN * DS_ROWB;
  static constexpr int OFF_Q = 0;                        // 2 buffers
  static constexpr int OFF_DO = 2 * Q_TILE;              // 2 buffers
  static constexpr int OFF_DS = 4 * Q_TILE;
  static constexpr int OFF_ST = OFF_DS + DS_TILE;        // lse2[2][BM], delta[2][BM] fp32
  static constexpr int SMEM = OFF_ST + 4 * BM * 4;
  static_assert(BN * ROWB <= OFF_DS, "K staging aliases the Q/dO buffers");
  static_assert(BM == 64, "dS^T rows are 8 chunks");
};

template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_kernel(const AttnArgs a) {
  using C = BwdCfg<D>;
  using M = Mma<T>;
  using V8 = typename M::V8;
  typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
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

  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + s.k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + s.k_row0 * a.v_st[1] + hk * a.v_st[2];
  T* dk_ptr = (T*)a.dk + b * a.dk_st[0] + s.k_row0 * a.dk_st[1] + hk * a.dk_st[2];
  T* dv_ptr = (T*)a.dv + b * a.dv_st[0] + s.k_row0 * a.dv_st[1] + hk * a.dv_st[2];
  // packed row index of this sequence's first query (for the workspace arrays)
  const int64_t ws_row0 = a.cu_q ? s.q_row0 : (int64_t)b * a.seqlen_q;

  // ---- query tiles that can see this key tile -------------------------------
  int i_min = (a.wr >= 0) ? max(0, j0 - shift - a.wr) : 0;
  int i_max = (a.wl >= 0 && j0 >= a.n_sink) ? min(len_q - 1, j_last - shift + a.wl) : len_q - 1;
  const int qt_lo = i_min / C::BM;
  const int n_qt = (i_max >= i_min) ? i_max / C::BM - qt_lo + 1 : 0;
  const int n_iter = n_qt * a.group;

  // ---- K / V fragments -------------------------------------------------------
  const int jc = j0 + wave * 32 + l32;  // this lane's key column
  V8 kf[C::KSTEPS], vf[C::KSTEPS];
#pragma unroll
  for (int ks = 0; ks < C::KSTEPS; ks++) {
    if (jc < len_k) {
      kf[ks] = *(const V8*)(k_ptr + (int64_t)jc * a.k_st[1] + ks * 16 + g * 8);
      vf[ks] = *(const V8*)(v_ptr + (int64_t)jc * a.v_st[1] + ks * 16 + g * 8);
    } else {
      kf[ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
      vf[ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }
  // K^T fragments for dQ = dS K: B operand, lane = d column of this wave's d-block,
  // slots = 8 consecutive keys.  Staged through LDS for the transposing read.
  const int dq_db = wave % C::DBLK;
  V8 ktf[C::BN / 16];
  if (n_iter > 0) {
#pragma unroll
    for (int n = 0; n < C::KCH; n++) {
      const int c = tid + n * C::THREADS;
      const int row = c / C::CPR, ch = c % C::CPR;
      u32x4 val = u32x4{0, 0, 0, 0};
      if (j0 + row < len_k) val = *(const u32x4*)(k_ptr + (int64_t)(j0 + row) * a.k_st[1] + ch * 8);
      *(u32x4*)(smem + row * C::ROWB + swz<C::CPR>(row, ch) * 16) = val;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < C::BN / 16; ks++) {
      const int row = ks * 16 + 8 * g + (i16 >> 2);
      const int ch = 4 * dq_db + 2 * (u & 1) + ((i16 & 3) >> 1);
      const int half = (i16 & 1) * 8;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_s16x4*)(smem + row * C::ROWB + swz<C::CPR>(row, ch) * 16 + half));
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (lds_s16x4*)(smem + (row + 4) * C::ROWB + swz<C::CPR>(row + 4, ch) * 16 + half));
      const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      __builtin_memcpy(&ktf[ks], &both, 16);
    }
    __syncthreads();
  }

  f32x16 dk_acc[C::DBLK], dv_acc[C::DBLK];
#pragma unroll
  for (int d = 0; d < C::DBLK; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) {
      dk_acc[d][i] = 0.f;
      dv_acc[d][i] = 0.f;
    }

  // ---- tile movement: Q, dO, lse, delta of iteration `it` ---------------------
  u32x4 qreg[C::QCH], doreg[C::QCH];
  float streg = 0.f;
  auto iter_coords = [&](int it, int& hq, int& i0) {
    hq = hk * a.group + it / n_qt;
    i0 = (qt_lo + it % n_qt) * C::BM;
  };
  auto load_iter = [&](int it) {
    int hq, i0;
    iter_coords(it, hq, i0);
    const T* q_ptr = (const T*)a.q + b * a.q_st[0] + s.q_row0 * a.q_st[1] + hq * a.q_st[2];
    const T* do_ptr = (const T*)a.dout + b * a.do_st[0] + s.q_row0 * a.do_st[1] + hq * a.do_st[2];
#pragma unroll
    for (int n = 0; n < C::QCH; n++) {
      const int c = tid + n * C::THREADS;
      const int row = c / C::CPR, ch = c % C::CPR;
      if (i0 + row < len_q) {
        qreg[n] = *(const u32x4*)(q_ptr + (int64_t)(i0 + row) * a.q_st[1] + ch * 8);
        doreg[n] = *(const u32x4*)(do_ptr + (int64_t)(i0 + row) * a.do_st[1] + ch * 8);
      } else {
        qreg[n] = u32x4{0, 0, 0, 0};
        doreg[n] = u32x4{0, 0, 0, 0};
      }
    }
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
  auto store_iter = [&](int buf) {
#pragma unroll
    for (int n = 0; n < C::QCH; n++) {
      const int c = tid + n * C::THREADS;
      const int row = c / C::CPR, ch = c % C::CPR;
      const int off = row * C::ROWB + swz<C::CPR>(row, ch) * 16;
      *(u32x4*)(smem + C::OFF_Q + buf * C::Q_TILE + off) = qreg[n];
      *(u32x4*)(smem + C::OFF_DO + buf * C::Q_TILE + off) = doreg[n];
    }
    if (tid < 2 * C::BM) *(float*)(smem + C::OFF_ST + buf * 2 * C::BM * 4 + tid * 4) = streg;
  };

  if (n_iter > 0) {
    load_iter(0);
    store_iter(0);
  }
  __syncthreads();

  for (int it = 0; it < n_iter; it++) {
    const int buf = it & 1;
    int hq, i0;
    iter_coords(it, hq, i0);
    if (it + 1 < n_iter) load_iter(it + 1);
    const char* q_lds = smem + C::OFF_Q + buf * C::Q_TILE;
    const char* do_lds = smem + C::OFF_DO + buf * C::Q_TILE;
    const float* lse_lds = (const float*)(smem + C::OFF_ST + buf * 2 * C::BM * 4);
    const float* delta_lds = lse_lds + C::BM;

    // ---- S = Q K^T and dP = dO V^T (rows = queries, lane = key column) ------
    f32x16 sacc[C::MI], pacc[C::MI];
#pragma unroll
    for (int mi = 0; mi < C::MI; mi++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        sacc[mi][i] = 0.f;
        pacc[mi][i] = 0.f;
      }
#pragma unroll
    for (int ks = 0; ks < C::KSTEPS; ks++) {
#pragma unroll
      for (int mi = 0; mi < C::MI; mi++) {
        const int row = mi * 32 + l32;
        const int off = row * C::ROWB + swz<C::CPR>(row, ks * 2 + g) * 16;
        const V8 qa = *(const V8*)(q_lds + off);
        const V8 da = *(const V8*)(do_lds + off);
        sacc[mi] = M::mfma32(qa, kf[ks], sacc[mi]);
        pacc[mi] = M::mfma32(da, vf[ks], pacc[mi]);
      }
    }

    // ---- P and dS -----------------------------------------------------------
    // tile fully visible?  (every row valid, every key inside every row's band)
    const int i_end = i0 + C::BM - 1;
    const bool full = i_end < len_q && j0 + C::BN - 1 < len_k &&
                      (a.wr < 0 || j0 + C::BN - 1 <= i0 + shift + a.wr) &&
                      (a.wl < 0 || j0 >= i_end + shift - a.wl || j0 + C::BN - 1 < a.n_sink);
#pragma unroll
    for (int mi = 0; mi < C::MI; mi++) {
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int rbase = mi * 32 + 8 * i4 + 4 * g;
        const f32x4 l4 = *(const f32x4*)(lse_lds + rbase);
        const f32x4 d4 = *(const f32x4*)(delta_lds + rbase);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int i = 4 * i4 + e;
          float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[mi][i], a.scale_log2, -l4[e]));
          if (!full) {
            const int iq = i0 + rbase + e;
            const int rel = jc - iq - shift;  // key position relative to the aligned diagonal
            const bool ok = jc < len_k && (a.wr < 0 || rel <= a.wr) &&
                            (a.wl < 0 || rel >= -a.wl || jc < a.n_sink);
            p = ok ? p : 0.f;  // invalid rows already have lse = +inf
          }
          sacc[mi][i] = p;
          pacc[mi][i] = p * (pacc[mi][i] - d4[e]);
        }
      }
    }

    // ---- dV^T += dO^T P ; dK^T += Q^T dS --------------------------------------
#pragma unroll
    for (int ks = 0; ks < C::BM / 16; ks++) {
      const int mi = ks >> 1;
      float pv[8], dsv[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        pv[j] = sacc[mi][8 * (ks & 1) + j];
        dsv[j] = pacc[mi][8 * (ks & 1) + j];
      }
      const V8 pb = M::pack(pv);
      const V8 dsb = M::pack(dsv);
      const int row = ks * 16 + 4 * g + (i16 >> 2);
#pragma unroll
      for (int d = 0; d < C::DBLK; d++) {
        const int ch = 4 * d + 2 * (u & 1) + ((i16 & 3) >> 1);
        const int half = (i16 & 1) * 8;
        const int off0 = row * C::ROWB + swz<C::CPR>(row, ch) * 16 + half;
        const int off1 = (row + 8) * C::ROWB + swz<C::CPR>(row + 8, ch) * 16 + half;
        {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(do_lds + off0));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(do_lds + off1));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          V8 af;
          __builtin_memcpy(&af, &both, 16);
          dv_acc[d] = M::mfma32(af, pb, dv_acc[d]);
        }
        {
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q_lds + off0));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(q_lds + off1));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          V8 af;
          __builtin_memcpy(&af, &both, 16);
          dk_acc[d] = M::mfma32(af, dsb, dk_acc[d]);
        }
      }
    }

    // ---- dS^T -> LDS ([key][query], 8 chunks per row) --------------------------
    {
      char* ds_lds = smem + C::OFF_DS;
      const int row = wave * 32 + l32;
#pragma unroll
      for (int mi = 0; mi < C::MI; mi++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const auto h4 = M::pack4(pacc[mi][4 * i4], pacc[mi][4 * i4 + 1], pacc[mi][4 * i4 + 2],
                                   pacc[mi][4 * i4 + 3]);
          *(typename M::V4*)(ds_lds + row * C::DS_ROWB + swz<8>(row, 4 * mi + i4) * 16 + 8 * g) = h4;
        }
    }
    __syncthreads();

    // ---- dQ[:, d-block] = dS K, out through fp32 atomics ------------------------
    {
      const char* ds_lds = smem + C::OFF_DS;
      float* dq_row0 = a.dq_acc + ((ws_row0 + i0) * a.heads_q + hq) * D + dq_db * 32 + l32;
#pragma unroll
      for (int n = 0; n < C::DQ_TILES; n++) {
        const int mi = wave / C::DBLK + n * (4 / C::DBLK);
        f32x16 acc;
#pragma unroll
        for (int i = 0; i < 16; i++) acc[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < C::BN / 16; ks++) {
          const int row = ks * 16 + 8 * g + (i16 >> 2);
          const int ch = 4 * mi + 2 * (u & 1) + ((i16 & 3) >> 1);
          const int half = (i16 & 1) * 8;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (lds_s16x4*)(ds_lds + row * C::DS_ROWB + swz<8>(row, ch) * 16 + half));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (lds_s16x4*)(ds_lds + (row + 4) * C::DS_ROWB + swz<8>(row + 4, ch) * 16 + half));
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          V8 af;
          __builtin_memcpy(&af, &both, 16);
          acc = M::mfma32(af, ktf[ks], acc);
        }
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const int r = mi * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
          if (i0 + r < len_q) unsafeAtomicAdd(dq_row0 + (int64_t)r * a.heads_q * D, acc[i]);
        }
      }
    }

    if (it + 1 < n_iter) store_iter(buf ^ 1);
    __syncthreads();
  }

  // ---- write dK, dV (C layout: lane = key, regs = d) ------------------------------
  if (jc < len_k) {
#pragma unroll
    for (int d = 0; d < C::DBLK; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const int col = d * 32 + 8 * i4 + 4 * g;
        const auto k4 = M::pack4(dk_acc[d][4 * i4] * a.scale, dk_acc[d][4 * i4 + 1] * a.scale,
                                 dk_acc[d][4 * i4 + 2] * a.scale, dk_acc[d][4 * i4 + 3] * a.scale);
        const auto v4 = M::pack4(dv_acc[d][4 * i4], dv_acc[d][4 * i4 + 1], dv_acc[d][4 * i4 + 2],
                                 dv_acc[d][4 * i4 + 3]);
        *(typename M::V4*)(dk_ptr + (int64_t)jc * a.dk_st[1] + col) = k4;
        *(typename M::V4*)(dv_ptr + (int64_t)jc * a.dv_st[1] + col) = v4;
      }
  }
}

// delta[h][row] = sum_d dO * O ; zero the fp32 dQ accumulator.  One 16-lane (D=128) or
// 8-lane (D=64) group per (row, head).
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
  f32x4* z = (f32x4*)(a.dq_acc + unit * D + c);
  z[0] = f32x4{0.f, 0.f, 0.f, 0.f};
  z[1] = f32x4{0.f, 0.f, 0.f, 0.f};
}

template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_post_kernel(const AttnArgs a) {
  constexpr int LPR = D / 8;
  const int64_t unit = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int c = (threadIdx.x % LPR) * 8;
  if (unit >= a.rows_q * a.heads_q) return;
  const int h = (int)(unit % a.heads_q);
  const int64_t row = unit / a.heads_q;
  int64_t off;
  if (a.cu_q) {
    off = row * a.dq_st[1];
  } else {
    off = (row / a.seqlen_q) * a.dq_st[0] + (row % a.seqlen_q) * a.dq_st[1];
  }
  const f32x4* src = (const f32x4*)(a.dq_acc + unit * D + c);
  const f32x4 x = src[0], y = src[1];
  float f[8] = {x[0] * a.scale, x[1] * a.scale, x[2] * a.scale, x[3] * a.scale,
                y[0] * a.scale, y[1] * a.scale, y[2] * a.scale, y[3] * a.scale};
  *(typename Mma<T>::V8*)((T*)a.dq + off + h * a.dq_st[2] + c) = Mma<T>::pack(f);
}

template <typename T, int D>
int launch_bwd(AttnArgs& a, hipStream_t stream, int phases) {
  using C = BwdCfg<D>;
  const int64_t units = a.rows_q * a.heads_q;
  const unsigned ew_blocks = (unsigned)ceil_div(units * (D / 8), 256);
  if (units > 0 && (phases & RSWA_BWD_PREP)) {
    hipLaunchKernelGGL((attn_bwd_prep_kernel<T, D>), dim3(ew_blocks), dim3(256), 0, stream, a);
    int rc = check_launch("attn_bwd prep");
    if (rc != RSWA_OK) return rc;
  }
  if (a.cu_q) {
    a.n_tile = (int)(ceil_div(a.rows_k, C::BN) + a.batch);
    a.n_work = a.n_tile * a.heads_kv;
  } else {
    a.n_tile = (int)ceil_div(a.seqlen_k, C::BN);
    a.n_work = a.n_tile * a.heads_kv * a.batch;
  }
  if (a.n_work > 0 && (phases & RSWA_BWD_MAIN)) {
    auto kern = attn_bwd_kernel<T, D>;
    static bool configured = false;  // benign race: the attribute call is idempotent
    if (!configured) {
      hipError_t e = hipFuncSetAttribute((const void*)kern,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, C::SMEM);
      if (e != hipSuccess)
        return fail(RSWA_ERR_LAUNCH, "attn_bwd: set smem: %s", hipGetErrorString(e));
      configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(padded_grid(a.n_work)), dim3(C::THREADS), C::SMEM, stream, a);
    int rc = check_launch("attn_bwd main");
    if (rc != RSWA_OK) return rc;
  }
  if (units > 0 && (phases & RSWA_BWD_POST)) {
    hipLaunchKernelGGL((attn_bwd_post_kernel<T, D>), dim3(ew_blocks), dim3(256), 0, stream, a);
    return check_launch("attn_bwd post");
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
  return rswa_attn_bwd_phases(p, stream, RSWA_BWD_PREP | RSWA_BWD_MAIN | RSWA_BWD_POST);
}
