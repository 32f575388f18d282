// Band / sink attention forward for gfx950: bf16|fp16 MFMA, K/V tiles in LDS,
// online softmax, tiles outside the visible band never touched.
//
// Replaces flash-attn's forward as wrapped at ring_swa/ops/wrap_flash.py:168-273.
//
// One block = 128 query rows of one (sequence, q head); 4 waves x 32 rows.
// Per 64-key tile a wave computes S^T = K Q^T (keys x queries) with
// v_mfma_f32_32x32x16, so each lane owns ONE query column: the row max / sum of
// the online softmax are in-lane reductions plus a single half-wave exchange,
// and P^T is already laid out as the B operand of O^T += V^T P^T.  V^T fragments
// come straight out of the row-major V tile with ds_read_b64_tr_b16.
#include "attn_common.h"

namespace rswa {
namespace {

template <int D>
struct FwdCfg {
  static constexpr int BM = 128;
  static constexpr int BN = 64;
  static constexpr int THREADS = 256;
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLK = D / 32;
  static constexpr int CPR = D / 8;  // 16-byte chunks per row
  static constexpr int CH = BN * CPR / THREADS;
  // LDS row strides (bytes).  K: +16 B keeps the 16 rows of a b128 phase on distinct
  // banks.  V: stride = 16 dwords mod 32 so the 4 rows x 64 B of a transposing read
  // phase cover all 64 banks once.
  static constexpr int K_STRIDE = D * 2 + 16;
  static constexpr int V_STRIDE = (D == 128) ? 320 : 192;
  static constexpr int K_TILE = BN * K_STRIDE;
  static constexpr int V_TILE = BN * V_STRIDE;
  static constexpr int O_STRIDE = D * 2 + 16;
  static constexpr int SMEM = 2 * K_TILE + 2 * V_TILE;
  static_assert(SMEM >= 4 * 32 * O_STRIDE, "epilogue staging must fit");
};

template <typename T, int D>
// two blocks per CU (2 waves per SIMD): keeps everything in the 256 architectural VGPRs,
// so no accumulator-register copies, and lets one wave's softmax overlap another's MFMAs
__global__ __launch_bounds__(256, 2) void attn_fwd_kernel(const AttnArgs a) {
  using C = FwdCfg<D>;
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

  // ---- which (sequence, kv head, q tile, q head) ---------------------------
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
  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + s.k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + s.k_row0 * a.v_st[1] + hk * a.v_st[2];
  T* o_ptr = (T*)a.out + b * a.o_st[0] + s.q_row0 * a.o_st[1] + hq * a.o_st[2];
  float* lse_ptr = a.lse + b * a.lse_st[0] + hq * a.lse_st[1] + s.q_row0 * a.lse_st[2];

  // ---- key tiles this block visits -----------------------------------------
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

  // ---- this wave's rows ----------------------------------------------------
  const int r0 = i0 + wave * 32;
  const int iq = r0 + l32;
  const RowBounds rb = row_bounds(a, iq, len_q, len_k);
  const bool wave_valid = r0 < len_q;
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

  // ---- global -> register -> LDS tile movement ------------------------------
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
      const int row = c / C::CPR, col = (c % C::CPR) * 8;
      *(u32x4*)(smem + buf * C::K_TILE + row * C::K_STRIDE + col * 2) = kreg[n];
      *(u32x4*)(smem + 2 * C::K_TILE + buf * C::V_TILE + row * C::V_STRIDE + col * 2) = vreg[n];
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
      const char* kbuf = smem + buf * C::K_TILE;
      const char* vbuf = smem + 2 * C::K_TILE + buf * C::V_TILE;
      // S^T[key, query] = K Q^T
      f32x16 sacc[2];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) sacc[t][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < C::KSTEPS; ks++) {
#pragma unroll
        for (int t = 0; t < 2; t++) {
          const V8 kf = *(const V8*)(kbuf + (t * 32 + l32) * C::K_STRIDE + (ks * 16 + g * 8) * 2);
          sacc[t] = M::mfma32(kf, qf[ks], sacc[t]);
        }
      }
      const bool full = wave_rows_full && j1 <= wb_first.hi &&
                        (j0 >= wb_last.lo || j1 < a.n_sink);
      if (!full) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int j = j0 + t * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
            const bool ok = j <= rb.hi && (j >= rb.lo || j < a.n_sink);
            sacc[t][i] = ok ? sacc[t][i] : -__builtin_inff();
          }
      }
      // online softmax (raw-score max; exponent in base 2)
      float mx = sacc[0][0];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) mx = fmaxf(mx, sacc[t][i]);
      mx = halfwave_max(mx);
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == -__builtin_inff()) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * a.scale_log2);
      const float mc = m_use * a.scale_log2;
      m_run = m_new;
      float psum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[t][i], a.scale_log2, -mc));
          sacc[t][i] = p;
          psum += p;
        }
      l_run = l_run * alpha + psum;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
        for (int d = 0; d < C::DBLK; d++)
#pragma unroll
          for (int i = 0; i < 16; i++) o_acc[d][i] *= alpha;
      }
      // O^T[d, query] += V^T P^T
      const int i16 = lane & 15, u = lane >> 4;
      const char* vlane = vbuf + (4 * g + (i16 >> 2)) * C::V_STRIDE + (16 * (u & 1) + 4 * (i16 & 3)) * 2;
#pragma unroll
      for (int s4 = 0; s4 < 4; s4++) {
        float pv[8];
#pragma unroll
        for (int j = 0; j < 8; j++) pv[j] = sacc[s4 >> 1][8 * (s4 & 1) + j];
        const V8 pb = M::pack(pv);
#pragma unroll
        for (int d = 0; d < C::DBLK; d++) {
          const char* p0 = vlane + (s4 * 16) * C::V_STRIDE + d * 64;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p0);
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p0 + 8 * C::V_STRIDE));
          typedef __attribute__((__vector_size__(8 * sizeof(short)))) short s16x8;
          const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          V8 vf;
          __builtin_memcpy(&vf, &both, 16);
          o_acc[d] = M::mfma32(vf, pb, o_acc[d]);
        }
      }
    }
    if (it + 1 < n_tiles) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue --------------------------------------------------------------
  const float l_tot = halfwave_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (g == 0 && iq < len_q) {
    lse_ptr[(int64_t)iq * a.lse_st[2]] =
        l_tot > 0.f ? m_run * a.scale + __logf(l_tot) : -__builtin_inff();
  }
  // transpose O^T through LDS (per-wave region) for coalesced 16-byte stores
  char* stage = smem + wave * 32 * C::O_STRIDE;
#pragma unroll
  for (int d = 0; d < C::DBLK; d++)
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++) {
      const auto h4 = M::pack4(o_acc[d][4 * i4] * inv, o_acc[d][4 * i4 + 1] * inv,
                               o_acc[d][4 * i4 + 2] * inv, o_acc[d][4 * i4 + 3] * inv);
      *(typename M::V4*)(stage + l32 * C::O_STRIDE + (d * 32 + 8 * i4 + 4 * g) * 2) = h4;
    }
  __syncthreads();
#pragma unroll
  for (int n = 0; n < 32 * C::CPR / 64; n++) {
    const int c = lane + n * 64;
    const int row = c / C::CPR, col = (c % C::CPR) * 8;
    if (r0 + row < len_q) {
      const u32x4 val = *(const u32x4*)(stage + row * C::O_STRIDE + col * 2);
      *(u32x4*)(o_ptr + (int64_t)(r0 + row) * a.o_st[1] + col) = val;
    }
  }
}

template <typename T, int D>
int launch_fwd(AttnArgs& a, hipStream_t stream) {
  using C = FwdCfg<D>;
  if (a.cu_q) {
    a.n_tile = (int)(ceil_div(a.rows_q, C::BM) + a.batch);
    a.n_work = a.n_tile * a.heads_q;
  } else {
    a.n_tile = (int)ceil_div(a.seqlen_q, C::BM);
    a.n_work = a.n_tile * a.heads_q * a.batch;
  }
  if (a.n_work == 0) return RSWA_OK;
  auto kern = attn_fwd_kernel<T, D>;
  static bool configured = false;  // benign race: the attribute call is idempotent
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       C::SMEM);
    if (e != hipSuccess) return fail(RSWA_ERR_LAUNCH, "attn_fwd: set smem: %s", hipGetErrorString(e));
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3(padded_grid(a.n_work)), dim3(C::THREADS), C::SMEM, stream, a);
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
