// Band / sink attention backward for gfx950, without atomics.
//
// Replaces flash-attn's backward as wrapped at ring_swa/ops/wrap_flash.py:276-429.
// Three launches on the caller's stream:
//   PREP : per (row, q head): -delta = -sum_d dO * O and -lse2 = -lse * log2(e) (stored negated:
//          they enter the kernels as addends),
//          both fp32, into the caller's workspace
//   DKDV : one block (4 waves, one per SIMD, up to 512 registers each) owns 256 keys of one
//          (sequence, kv head) and walks the query tiles (32 rows) that can see them, for
//          every q head of the GQA group; a wave owns 64 keys: their K and V fragments stay
//          in registers, dK^T / dV^T accumulate in accumulation registers for the whole
//          walk and are written once
//   DQ   : one block (8 waves x 32 query rows: 128 rows of two q heads of a GQA group, or
//          256 rows of one head) walks the key tiles (64 keys) it can see, like the forward
//          kernel; dQ^T stays in registers
// S and dP are computed in both main kernels (7 GEMM units instead of 5).  That costs
// less here than fp32 atomics on dQ: hardware fp32 atomic adds retire at 340 G elements/s on
// the whole device (measured with 64 consecutive floats per wave instruction, the pattern a
// fused kernel would use), a dQ tile of 32 x 128 per 256-key block and step needs 700 G/s at
// the rate the dK/dV kernel walks.  It also makes the result run-to-run deterministic.
//
// DKDV per (query tile, wave) (C layout: lane = key; two 32-key blocks per wave, so every
// fragment read from LDS feeds two MFMAs):
//   S = Q K^T, dP = dO V^T      A = Q / dO row fragments (LDS), B = K / V (registers)
//   P = exp2(S*c - lse2), dS = P * (dP - delta); the dP chains start from -delta instead of zero.
//   (Folding c into 16-bit K fragments and starting the S chains from -lse2 would save the
//   multiply-add per score -- 1-2 % -- but the rounding of K c shifts the exponent by up to
//   2^-9 |S c|: with peaked scores, e.g. sink keys four times the usual size, it doubled the
//   error of dK / dV against the fp32 oracle, 4e-3 -> 7e-3.  The scale stays in fp32.)
//   dV^T += dO^T P, dK^T += Q^T dS   A = transposing LDS reads of dO / Q, B = P / dS (regs)
// The S and dP MFMAs are inline assembly so that their accumulators live in vector
// registers, where the vector ALU reads them next; left to the compiler they end up in
// accumulation registers like dK^T and dV^T and every element costs two copies.  The
// compiler does not know that these statements are MFMAs and pads nothing after them:
// the code keeps at least two later MFMAs between the last one that writes S or dP and
// the first read of the result.  The dK^T / dV^T MFMAs are compiler builtins (accumulation
// registers), so every copy or read the compiler adds around them is padded as required.
// DQ per (key tile, wave), on 16x16x32 MFMAs; wave owns 32 query columns (lane = query l % 16
// of two 16-query blocks):
//   S^T = K Q^T, dP^T = V dO^T  A = K / V row fragments from LDS, B = Q / dO fragments (regs);
//                               the dP^T chains start from -delta of the lane's queries
//   dS^T = exp2(S^T c - lse2) dP^T   (the scale is applied in fp32: see the note at DKDV)
//   dQ^T += K^T dS^T            A = transposing LDS reads of K, B = dS^T (regs)
//
// Streamed tiles are double-buffered in SEPARATE static __shared__ arrays, filled by buffer
// loads that land directly in LDS one tile ahead, and the tile loops are unrolled by two so
// that every access names its buffer statically (see attn_fwd.hip for why).
#include "attn_common.h"

#include <mutex>

namespace rswa {
namespace {

// One lane's 8 consecutive values of a gradient row, already rounded to the 16-bit type, into
// the caller's buffer at element offset `at`: as they are, as fp32 (a ring accumulator), and in
// either case added to what the buffer holds (fp32 sum, one rounding for a 16-bit buffer).
template <typename T>
__device__ __forceinline__ void put_grad8(void* buf, int64_t at, typename Mma<T>::V8 val, bool wide,
                                          bool accumulate) {
  using V8 = typename Mma<T>::V8;
  if (wide) {
    float* dst = (float*)buf + at;
    f32x4 y[2];
#pragma unroll
    for (int hh = 0; hh < 2; hh++) {
      f32x4 old = {0.f, 0.f, 0.f, 0.f};
      if (accumulate) old = *(const f32x4*)(dst + 4 * hh);
#pragma unroll
      for (int j = 0; j < 4; j++) y[hh][j] = old[j] + (float)val[4 * hh + j];
    }
    *(f32x4*)dst = y[0];
    *(f32x4*)(dst + 4) = y[1];
  } else {
    T* dst = (T*)buf + at;
    if (accumulate) {
      const V8 old = *(const V8*)dst;
      float sum[8];
#pragma unroll
      for (int j = 0; j < 8; j++) sum[j] = (float)old[j] + (float)val[j];
      val = Mma<T>::pack(sum);
    }
    *(V8*)dst = val;
  }
}

// ============================================================================
// dK / dV
// ============================================================================
template <int D>
struct DkvCfg {
  static constexpr int BM = 32;        // query rows per step
  static constexpr int KB = 2;         // 32-key blocks per wave
  static constexpr int BN = kDkvKeysPerBlock;  // keys per block: 4 waves x KB x 32
  static_assert(BN == 256, "4 waves x KB x 32 keys");
  static constexpr int THREADS = 256;  // one wave per SIMD, up to 512 registers each
  static constexpr int KSTEPS = D / 16;
  static constexpr int DBLK = D / 32;
  static constexpr int CPR = D / 8;   // 16-byte chunks per row
  static constexpr int ROWB = D * 2;  // bytes per row
  static constexpr int Q_TILE = BM * ROWB;
};

template <typename T, int D, bool SPLIT, bool FAR, bool HAND>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_kernel(const AttnArgs a) {
  static_assert(!(HAND && FAR), "dS hand-off in the first addressing form only");
  using C = DkvCfg<D>;
  using M = Mma<T>;
  using V8 = typename M::V8;
  constexpr int KB = C::KB, KS = C::KSTEPS, DB = C::DBLK;
  __shared__ __attribute__((aligned(1024))) char q_s0[C::Q_TILE];
  __shared__ __attribute__((aligned(1024))) char q_s1[C::Q_TILE];
  __shared__ __attribute__((aligned(1024))) char do_s0[C::Q_TILE];
  __shared__ __attribute__((aligned(1024))) char do_s1[C::Q_TILE];
  __shared__ __attribute__((aligned(1024))) float st_s0[2 * C::BM];  // -lse2[BM], -delta[BM]
  __shared__ __attribute__((aligned(1024))) float st_s1[2 * C::BM];
  __shared__ int arrived_s;

  const int wid = logical_block_id(a.n_work);
  if (wid < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // key group: 64 keys each
  const int l32 = lane & 31;
  const int g = lane >> 5;
  const int i16 = lane & 15;
  const int u = lane >> 4;

  // ---- which (sequence, kv head, key tile) and which part of the GQA group -----------
  // parts of a tile are neighbours in the launch order; tiles go heaviest first
  const int part = wid % a.nsplit;
  const int unit = wid / a.nsplit;
  const int hpu = a.group / a.nsplit;  // q heads this block walks
  const int slot = a.rev_k ? a.n_tile - 1 - unit % a.n_tile : unit % a.n_tile;
  int rest = unit / a.n_tile;
  const int hk = rest % a.heads_kv;
  SeqInfo s;
  int kt;
  if (a.cu_q) {
    static_assert(C::BN == 1 << 8, "tile size passed to locate_packed");
    if (!locate_packed(a, slot, 8, true, s, kt)) return;
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

  // Keys in two row ranges (dense mode; the boundary is a multiple of the block's keys): the
  // block's keys all lie in one of them, and its pointers are set so that a key's index in the
  // sequence selects its row.
  const bool seg2 = j0 >= a.seg;
  const int64_t seg_row0 = seg2 ? -(int64_t)a.seg : s.k_row0;
  const T* k_ptr = (const T*)(seg2 ? a.k2 : a.k) + b * a.k_st[0] + seg_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)(seg2 ? a.v2 : a.v) + b * a.v_st[0] + seg_row0 * a.v_st[1] + hk * a.v_st[2];
  // (gradient buffers: T or, as ring accumulators, fp32 -- element offsets)
  void* const dk_buf = seg2 ? a.dk2 : a.dk;
  void* const dv_buf = seg2 ? a.dv2 : a.dv;
  const int64_t dk_off = b * a.dk_st[0] + seg_row0 * a.dk_st[1] + hk * a.dk_st[2];
  const int64_t dv_off = b * a.dv_st[0] + seg_row0 * a.dv_st[1] + hk * a.dv_st[2];
  const int64_t ws_row0 = a.cu_q ? s.q_row0 : (int64_t)b * a.seqlen_q;

  // ---- query tiles that can see this key tile -------------------------------
  const int i_min = (a.wr >= 0) ? max(0, j0 - shift - a.wr) : 0;
  const int i_max =
      (a.wl >= 0) ? min(len_q - 1, j_last - shift + a.wl) : len_q - 1;
  const int qt_lo = i_min / C::BM;
  const int n_qt = (i_max >= i_min) ? i_max / C::BM - qt_lo + 1 : 0;
  const int n_iter = n_qt * hpu;

  const int jw0 = j0 + wave * (32 * KB);  // first key column of this wave
  const int jw1 = jw0 + 32 * KB - 1;

  // ---- lane-constant LDS offsets (swizzle folded: varying parts are XOR / immediates) ----
  // 16-byte row fragments: row = l32 (+ 32 per block), chunk = 2 ks + g
  //   offset = (a_row ^ (ks << 5)) + blk * 32 * ROWB
  const int a_row = l32 * C::ROWB + ((g ^ swz_f<C::CPR>(l32)) << 4);
  // transposing reads of Q / dO: rows 16 ks + 4 g + (i16 >> 2) and + 8, chunk = 4 d + lp
  //   offset = (t_row{0,1} ^ (d << 6)) + ks * 16 * ROWB
  const int rl = 4 * g + (i16 >> 2);
  const int lp = 2 * (u & 1) + ((i16 & 3) >> 1);
  const int t_row0 = rl * C::ROWB + ((lp ^ swz_f<C::CPR>(rl)) << 4) + (i16 & 1) * 8;
  const int t_row1 = (rl + 8) * C::ROWB + ((lp ^ swz_f<C::CPR>(rl + 8)) << 4) + (i16 & 1) * 8;

  // ---- this wave's K fragments stay in registers for the whole walk (B operand of
  // S = Q K^T: lane = key column, 8 consecutive d per k-step); keys past the end are zero
  V8 kf[KB][KS];
#pragma unroll
  for (int kb = 0; kb < KB; kb++) {
    const int jc = jw0 + kb * 32 + l32;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (jc < len_k) {
        kf[kb][ks] = *(const V8*)(k_ptr + (int64_t)jc * a.k_st[1] + ks * 16 + g * 8);
      } else {
        kf[kb][ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  }

  // ... and so do its V fragments (B operand of dP = dO V^T, same layout)
  V8 vf[KB][KS];
#pragma unroll
  for (int kb = 0; kb < KB; kb++) {
    const int jc = jw0 + kb * 32 + l32;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      if (jc < len_k) {
        vf[kb][ks] = *(const V8*)(v_ptr + (int64_t)jc * a.v_st[1] + ks * 16 + g * 8);
      } else {
        vf[kb][ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  }
  f32x16 dk_acc[KB][DB], dv_acc[KB][DB];
#pragma unroll
  for (int kb = 0; kb < KB; kb++)
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        dk_acc[kb][d][i] = 0.f;
        dv_acc[kb][d][i] = 0.f;
      }
  // ---- tile DMA (rows past the end of the sequence read as zero) ------------------
  TileDma<D, C::BM, C::THREADS> q_dma, do_dma;
  q_dma.init(a.q_st[1], tid);
  do_dma.init(a.do_st[1], tid);
  const T* q_base = (const T*)a.q + b * a.q_st[0] + s.q_row0 * a.q_st[1];
  const T* do_base = (const T*)a.dout + b * a.do_st[0] + s.q_row0 * a.do_st[1];
  // statistics: one load covers both workspace arrays (lse2, then delta `stat_elems` further
  // on) through a resource based at the tile's first row; rows past the sequence end read a
  // neighbour's finite values, which the row mask / zero Q, dO rows void
  // (element counts below 2^30: the host refuses larger statistics arrays)
  const int stat_elems = (int)(a.delta - a.lse2);  // elements between the two arrays
  const int stat_end = stat_elems + a.heads_q * (int)a.rows_q;  // end of delta
  const int q_row_bytes = (int)(a.q_st[1] * 2), do_row_bytes = (int)(a.do_st[1] * 2);
  // Cursor over the (q head of the group, query tile) pairs, advanced incrementally so
  // that a step costs a handful of scalar instructions: the tile's first row, the head's
  // Q / dO base pointers and the offset of its statistics.
  struct Cursor {
    int qt, i0;
    const T *q_head, *do_head;
    int stat_row;  // index of row 0 of this head in the statistics arrays
    int ds;        // HAND: byte offset of this wave's dS unit of the tile (from ds_first)
  };
  const int i_first = qt_lo * C::BM;
  // Every head's walk over the n_qt query tiles starts at tile qt_start and wraps around,
  // chosen so that at any step all blocks of a kv head whose walks are equally long are
  // on the same query tile modulo n_qt: neighbouring key tiles see almost the same query
  // rows, and walking them in step lets one L2 fill serve all of them.
  const int qt_start = n_qt > 0 ? (n_qt - qt_lo % n_qt) % n_qt : 0;
  Cursor nxt;  // the tile that the load parts fetch
  nxt.qt = qt_start;
  nxt.i0 = i_first + qt_start * C::BM;
  int nxt_left = n_qt;  // tiles left in the walk of nxt's head, nxt included
  const int h_first = hk * a.group + part * hpu;
  nxt.q_head = q_base + (int64_t)h_first * a.q_st[2];
  nxt.do_head = do_base + (int64_t)h_first * a.do_st[2];
  nxt.stat_row = (int)(h_first * a.rows_q + ws_row0);
  // dS hand-off: unit of (q head h, row tile qt of the sequence, this block's keys, this wave) at
  //   ds + (((h ds_slots + slot0 + qt) ds_nkb + kt % ds_nkb) 4 + wave) 4 KiB
  // -- per step one row of ds_nkb blocks further, per head ds_slots rows further.  The units
  // of the block's heads are addressed as 32-bit offsets from that of its first head's first
  // tile, through a buffer resource that ends with the last head's rows: an offset beyond it
  // (kDsNowhere) makes the hardware drop the store.
  const int ds_row_bytes = HAND ? a.ds_nkb * kDsBlockBytes : 0;
  const int ds_head_bytes = HAND ? a.ds_slots * ds_row_bytes : 0;  // (host: group x this < 2 GiB)
  constexpr int kDsNowhere = 0x7ff00000;
  const int64_t ds_slot0 = a.cu_q ? (s.q_row0 >> 5) + b : (int64_t)b * ((a.seqlen_q + 31) >> 5);
  const int64_t ds_first = HAND ? (int64_t)h_first * ds_head_bytes + (ds_slot0 + qt_lo) * ds_row_bytes +
                                      (kt % max(a.ds_nkb, 1)) * kDsBlockBytes + wave * kDsUnitBytes
                                : 0;
  const __amdgpu_buffer_rsrc_t ds_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      a.ds + ds_first, 0,
      HAND ? (int)min((int64_t)hpu * ds_head_bytes, (int64_t)a.heads_q * ds_head_bytes - ds_first) : 0,
      0x00020000);
  int ds_head_off = 0;  // of the head the cursor is on
  nxt.ds = qt_start * ds_row_bytes;
  [[maybe_unused]] int cur_ds = nxt.ds;  // the unit of the tile being computed
  // The next tile is fetched by NPART instructions per wave (statistics, Q, dO), issued
  // one at a time between the first MFMAs of a step; advance() then moves the cursor on.
  constexpr int NQD = TileDma<D, C::BM, C::THREADS>::N;
  constexpr int NPART = 1 + 2 * NQD;
  const int st_voff = ((lane & 31) << 2) + (lane >> 5) * (stat_elems * 4);
  auto load_part = [&](int part, char* qd, char* dod, float* std_) __attribute__((always_inline)) {
    if (part == 0) {
      if (wave == 0) {  // lanes 0-31: lse2 of the 32 rows, lanes 32-63: their delta
        const int first = nxt.stat_row + nxt.i0;
        const __amdgpu_buffer_rsrc_t st_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void*)(a.lse2 + first), 0, min(stat_end - first, stat_elems + C::BM) * 4, 0x00020000);
        // the per-lane offset is recomputed here (opaque to the optimiser): kept in a
        // register across the walk it could be spilled, and its reload would wait for
        // every tile load issued before it
        __builtin_amdgcn_raw_ptr_buffer_load_lds(st_rsrc, (lds_void_t*)std_, 4, st_voff, 0, 0, 0);
      }
    } else if (part <= NQD) {
      const TileSrc t = tile_src<C::BM, FAR>(nxt.q_head, nxt.i0, len_q, q_row_bytes, C::ROWB);
      q_dma.load_one(t.rsrc, t.soff, qd, part - 1);
    } else {
      const TileSrc t = tile_src<C::BM, FAR>(nxt.do_head, nxt.i0, len_q, do_row_bytes, C::ROWB);
      do_dma.load_one(t.rsrc, t.soff, dod, part - 1 - NQD);
    }
  };
  auto advance = [&]() __attribute__((always_inline)) {
    nxt.qt++;
    nxt.i0 += C::BM;
    if constexpr (HAND) nxt.ds += ds_row_bytes;
    if (nxt.qt == n_qt) {
      nxt.qt = 0;
      nxt.i0 = i_first;
      if constexpr (HAND) nxt.ds = ds_head_off;
    }
    if (--nxt_left == 0) {
      nxt_left = n_qt;
      nxt.qt = qt_start;
      nxt.i0 = i_first + qt_start * C::BM;
      nxt.q_head += a.q_st[2];
      nxt.do_head += a.do_st[2];
      nxt.stat_row += (int)a.rows_q;
      if constexpr (HAND) {
        ds_head_off += ds_head_bytes;
        nxt.ds = ds_head_off + qt_start * ds_row_bytes;
      }
    }
  };

  if (n_iter > 0) {
#pragma unroll
    for (int part = 0; part < NPART; part++) load_part(part, q_s0, do_s0, st_s0);
    if (n_iter > 1) advance();
  }
  __syncthreads();


  int cur_i0 = i_first + qt_start * C::BM;  // first row of the tile being computed
  // byte of a lane's 16 in a 1 KiB piece of a dS unit: [key l32][query group g]
  const int ds_lane = l32 * 32 + g * 16;
  // dS of a step, packed to 16 bits as the operand of its dK MFMAs.  HAND: the four groups also
  // go to the step's dS unit -- under the first MFMAs of the NEXT step (stores issued late in
  // their own step would still be on their way at its end, and the wait for the tile loads
  // there waits for every vector memory operation of the wave: that cost a fifth of the
  // kernel).  ds_pend = where they go: the unit of the last computed step, or nowhere.
  [[maybe_unused]] V8 ds_carry[KB][2];
  [[maybe_unused]] int ds_pend = kDsNowhere;
  auto store_ds = [&](int pc, int voff) __attribute__((always_inline)) {
    // piece [key block][query half] of the unit, 1 KiB per wave instruction: a key's 32 bytes
    // side by side ([query group g][rows 16 ks2 + 4 g .., 16 ks2 + 8 + 4 g ..])
    u32x4 bits;
    __builtin_memcpy(&bits, &ds_carry[pc >> 1][pc & 1], 16);
    // (aux 2 = non-temporal: the tiles are read once, by another kernel, much later; measured
    // 6 % faster than plain stores on a 2.4 GB hand-off)
    __builtin_amdgcn_raw_buffer_store_b128(bits, ds_rsrc, voff + pc * 1024, ds_pend, 2);
  };
  // (the lane's offset, opaque to the optimiser: or it keeps the four sums voff + pc * 1024 in
  // registers across the walk instead of using the instruction's immediate offset)
  auto ds_voff = [&]() __attribute__((always_inline)) {
    int v = ds_lane;
    asm volatile("" : "+v"(v));
    return v;
  };
  // For which first rows i0 of a 32-row tile does any (query, key of this wave) pair survive
  // the mask (need_*), and for which is no pair masked (full_*)?  With
  // i1 = min(i0 + 32, len_q) - 1 and the wave's keys jw0 .. jw1 the conditions
  //   needed: i0 < len_q, jw0 < len_k, jw0 <= i1 + shift + wr, jw1 >= i0 + shift - wl
  //   full:   i0 + 31 < len_q, jw1 < len_k, jw1 <= i0 + shift + wr, jw0 >= i0 + 31 + shift - wl
  // are intervals of i0 whose ends depend on the wave only: a step tests two of them.
  constexpr int kInf = 1 << 30;
  int need_lo = (a.wr < 0) ? -kInf : jw0 - shift - a.wr - 31;
  int need_hi = min(len_q - 1, (a.wl < 0) ? kInf : jw1 - shift + a.wl);
  if (jw0 >= len_k || (a.wr >= 0 && len_q - 1 < jw0 - shift - a.wr)) need_hi = -kInf - 1;
  int full_lo = (a.wr < 0) ? -kInf : jw1 - shift - a.wr;
  int full_hi = min(len_q - 32, (a.wl < 0) ? kInf : jw0 - 31 - shift + a.wl);
  if (jw1 >= len_k) full_hi = -kInf - 1;

  // one query tile: prefetch the next one into (qn, don, stn), compute on (qc, doc, stc)
  auto step = [&](int it, const char* qc, const char* doc, const float* stc, char* qn, char* don,
                  float* stn) __attribute__((always_inline)) {
    const int i0 = cur_i0;
    cur_i0 = nxt.i0;  // the tile fetched now is the next step's
    [[maybe_unused]] const int ds_unit = cur_ds;
    cur_ds = nxt.ds;
    const bool has_next = it + 1 < n_iter;
    const float* lse_lds = stc;
    const float* delta_lds = stc + C::BM;
    const bool needed = i0 >= need_lo && i0 <= need_hi;
    if (!needed && has_next) {
#pragma unroll
      for (int part = 0; part < NPART; part++) load_part(part, qn, don, stn);
      if (it + 2 < n_iter) advance();
    }
    if constexpr (HAND) {
      if (!needed) {
        const int voff = ds_voff();
#pragma unroll
        for (int pc = 0; pc < 2 * KB; pc++) store_ds(pc, voff);
        ds_pend = kDsNowhere;
      }
    }
    if (needed) {
      const bool full = i0 >= full_lo && i0 <= full_hi;
      // The four GEMMs of the (32 queries x 64 keys) sub-tile -- S = Q K^T, dP = dO V^T,
      // dV^T += dO^T P, dK^T += Q^T dS; KB KS MFMAs each, rows = queries, lane = key column
      // -- their LDS reads and the vector work are written out in issue order, one group
      // per MFMA, with scheduling fences between the groups.  Every fragment read from LDS
      // feeds the MFMAs of both key blocks; K and V come from registers; fragments are fetched
      // AH fragment slots ahead; P = exp2(S c - lse2) is computed under the dP MFMAs and
      // dS = P (dP - delta) under the dV MFMAs; dP - delta comes out of the MFMAs, whose
      // chains start from -delta in the accumulator layout.
      constexpr int NG = KB * KS;   // MFMAs per GEMM (KS = 2 DB)
      constexpr int NF = 4 * KS;    // fragment slots: Q, dO, dO^T, Q^T; KB MFMAs each
      constexpr int AH = 2;
      constexpr int GPC = NG / (4 * KB);  // MFMA groups per chunk of vector work
      static_assert(KS == 2 * DB && KB == 2, "GEMM shapes");
      auto fence = []() __attribute__((always_inline)) { __builtin_amdgcn_sched_barrier(0); };
      V8 fa[NF];
      auto fetch = [&](auto fc) __attribute__((always_inline)) {
        constexpr int f = decltype(fc)::value;
        if constexpr (f < KS) {
          fa[f] = *(const V8*)(qc + (a_row ^ (f << 5)));
        } else if constexpr (f < 2 * KS) {
          constexpr int ks = f - KS;
          fa[f] = *(const V8*)(doc + (a_row ^ (ks << 5)));
        } else if constexpr (f < NF) {
          constexpr int j = (f - 2 * KS) % KS, ks2 = j / DB, d = j % DB;
          const char* src = f < 3 * KS ? doc : qc;
          const int off0 = (t_row0 ^ (d << 6)) + ks2 * 16 * C::ROWB;
          const int off1 = (t_row1 ^ (d << 6)) + ks2 * 16 * C::ROWB;
          fa[f] = tr_pair<V8>(src + off0, src + off1);
        }
      };
      f32x16 sacc[KB], pacc[KB];
      // -delta of the 32 rows in the accumulator layout, from which the dP chains start, is read
      // into the second key block's accumulator: the first block's chain takes it as a separate
      // start operand, the second block's chain then accumulates in place
      f32x4 l4[4];   // -lse2 of the rows
      V8 pb[KB][2], ds_step[KB][2];
      V8(&dsb)[KB][2] = *[&]() __attribute__((always_inline)) {
        if constexpr (HAND) return &ds_carry;  // lives on into the next step
        else return &ds_step;
      }();
      // vector work in 2 KB chunks of four rows: chunk order lets the packed operands of
      // the first k-step be complete first
      auto chunk_of = [](int c, int& kb, int& i4) __attribute__((always_inline)) {
        kb = (c >> 1) & 1;
        i4 = (c & 1) | ((c >> 2) << 1);
      };
      // P stays in vector registers from here to dS (the S / dP accumulators live in
      // accumulation registers, which the vector ALU reaches only through copies)
      float pk[KB][16];
      auto p_chunk = [&](auto cc) __attribute__((always_inline)) {
        int kb, i4;
        chunk_of(decltype(cc)::value, kb, i4);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int i = 4 * i4 + e;
          pk[kb][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][i], a.scale_log2, l4[i4][e]));
        }
        if (i4 & 1) pb[kb][i4 >> 1] = M::pack(&pk[kb][8 * (i4 >> 1)]);
      };
      float dsk[KB][8];  // dS of the current pair of chunks
      auto ds_chunk = [&](auto cc) __attribute__((always_inline)) {
        int kb, i4;
        chunk_of(decltype(cc)::value, kb, i4);
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int i = 4 * i4 + e;
          dsk[kb][4 * (i4 & 1) + e] = pk[kb][i] * pacc[kb][i];  // zero where P is
        }
        if (i4 & 1) dsb[kb][i4 >> 1] = M::pack(dsk[kb]);
      };

      [[maybe_unused]] int ds_voff_step = 0;
      if constexpr (HAND) ds_voff_step = ds_voff();
      static_for<AH>([&](auto fc) __attribute__((always_inline)) { fetch(fc); });
      fence();
      static_for<4 * NG>([&](auto mc) __attribute__((always_inline)) {
        constexpr int m = decltype(mc)::value;
        constexpr int f = m / KB, kb = m % KB;  // fragment slot and key block of this MFMA
        if constexpr (kb == 0) fetch(std::integral_constant<int, f + AH>{});
        // (after the last tile the cursor still names it: its rows are fetched once more, into
        // the idle buffers, rather than branching around every load)
        if constexpr (m < NPART) load_part(m, qn, don, stn);
        if constexpr (HAND && m < 2 * KB) {
          store_ds(m, ds_voff_step);
          if constexpr (m == 2 * KB - 1) ds_pend = ds_unit;
        }
        // row statistics: -delta early in S (the dP chains start from it), -lse2 at its end
        if constexpr (m >= 4 && m < 8) {
          const f32x4 t4 = *(const f32x4*)(delta_lds + 8 * (m - 4) + 4 * g);
#pragma unroll
          for (int e = 0; e < 4; e++) pacc[KB - 1][4 * (m - 4) + e] = t4[e];
        }
        if constexpr (m >= NG - 4 && m < NG) l4[m - (NG - 4)] = *(const f32x4*)(lse_lds + 8 * (m - (NG - 4)) + 4 * g);
        if constexpr (m < NG) {
          if constexpr (f == 0) {
            if (full) {
              M::mfma32_vec0(fa[f], kf[kb][f], sacc[kb]);
            } else {
              // The mask enters as the start value of the S chain: 0 for a visible pair, -inf
              // otherwise (P = exp2(-inf) = 0, hence dS = 0).  Row r = c + 4 g of the tile, c
              // fixed per register, is visible from key jc iff rmin <= r <= rmax with
              //   rmin = t - rel_hi, rmax = min(t - rel_lo, rows_ok - 1), t = jc - i0 - shift:
              // one unsigned comparison of r - rmin against the width of that interval.
              constexpr int kBig = 1 << 29;  // |t| stays below it
              const int rel_lo = (a.wl < 0) ? -kBig : -a.wl;
              const int rel_up = (a.wr < 0) ? kBig : a.wr;
              const int jc = jw0 + kb * 32 + l32;
              const int t = jc - i0 - shift;
              const int rows_ok = (jc < len_k) ? len_q - i0 : 0;  // rows r < rows_ok are real
              const int rmin = t - rel_up;
              const int rmax = min(t - rel_lo, rows_ok - 1);
              const unsigned width = (unsigned)max(rmax - rmin + 1, 0);
              const int base = 4 * g - rmin;
#pragma unroll
              for (int i = 0; i < 16; i++) {
                const int c = 8 * (i >> 2) + (i & 3);
                sacc[kb][i] = ((unsigned)(base + c) < width) ? 0.f : -__builtin_inff();
              }
              M::mfma32_vec(fa[f], kf[kb][f], sacc[kb]);
            }
          } else {
            M::mfma32_vec(fa[f], kf[kb][f], sacc[kb]);
          }
        } else if constexpr (m < 2 * NG) {
          if constexpr (f == KS) {
            if constexpr (kb < KB - 1) {
              M::mfma32_vec_init(fa[f], vf[kb][f - KS], pacc[KB - 1], pacc[kb]);
            } else {
              M::mfma32_vec(fa[f], vf[kb][f - KS], pacc[kb]);
            }
          } else {
            M::mfma32_vec(fa[f], vf[kb][f - KS], pacc[kb]);
          }
          if constexpr ((m - NG + 1) % GPC == 0) p_chunk(std::integral_constant<int, (m - NG + 1) / GPC - 1>{});
        } else if constexpr (m < 3 * NG) {
          constexpr int j = f - 2 * KS, ks2 = j / DB, d = j % DB;
          dv_acc[kb][d] = M::mfma32(fa[f], pb[kb][ks2], dv_acc[kb][d]);
          if constexpr ((m - 2 * NG + 1) % GPC == 0)
            ds_chunk(std::integral_constant<int, (m - 2 * NG + 1) / GPC - 1>{});
        } else {
          constexpr int j = f - 3 * KS, ks2 = j / DB, d = j % DB;
          dk_acc[kb][d] = M::mfma32(fa[f], dsb[kb][ks2], dk_acc[kb][d]);
        }
        fence();
      });
      if (it + 2 < n_iter) advance();
    }
    __syncthreads();
  };

  for (int it = 0; it < n_iter; it += 2) {
    step(it, q_s0, do_s0, st_s0, q_s1, do_s1, st_s1);
    if (it + 1 < n_iter) step(it + 1, q_s1, do_s1, st_s1, q_s0, do_s0, st_s0);
  }
  if constexpr (HAND) {  // the last computed step's dS
    const int voff = ds_voff();
#pragma unroll
    for (int pc = 0; pc < 2 * KB; pc++) store_ds(pc, voff);
  }

  // ---- write dK, dV (C layout: lane = key, regs = d) -----------------------------------
  // The lane's position is taken afresh (opaque to the optimiser): addresses derived from
  // values computed before the walk would be kept in registers across it, and spilled.
  int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  asm volatile("" : "+v"(lane_e));
  const int l32_e = lane_e & 31, g_e = lane_e >> 5;
  // value group (mtx: 0 dK / 1 dV, key block, d block, four consecutive d) of this lane -> memory
  auto emit = [&](int mtx, int kb, int d, int i4, f32x4 val) __attribute__((always_inline)) {
    const int jc = jw0 + kb * 32 + l32_e;
    if (jc < len_k) {
      const float sc = mtx == 0 ? a.scale : 1.f;
      const int64_t at = (mtx == 0 ? dk_off + (int64_t)jc * a.dk_st[1] : dv_off + (int64_t)jc * a.dv_st[1]) +
                         d * 32 + 8 * i4 + 4 * g_e;
      const typename M::V4 h4 = M::pack4(val[0] * sc, val[1] * sc, val[2] * sc, val[3] * sc);
      if (a.wide_dkv) {
        float* dst = (float*)(mtx == 0 ? dk_buf : dv_buf) + at;
        f32x4 y = {(float)h4[0], (float)h4[1], (float)h4[2], (float)h4[3]};
        if (a.dkv_accumulate) y += *(const f32x4*)dst;
        *(f32x4*)dst = y;
      } else {
        *(typename M::V4*)((T*)(mtx == 0 ? dk_buf : dv_buf) + at) = h4;
      }
    }
  };
  // Without a split (SPLIT = false, nsplit = 1) the lane's sums go straight out.  Otherwise the
  // group's q heads were dealt to nsplit blocks: every block stores its fp32 partial sums (16
  // bytes per lane and value group, lanes contiguous), then counts itself in; the block that
  // arrives last adds the parts in part order -- the same order whichever block that is, so
  // the result does not depend on timing -- and writes dK, dV.  Nobody waits for anybody.
  constexpr int GROUPS = 2 * KB * DB * 4;  // value groups per lane
  f32x4* part_base = (f32x4*)a.dkv_part + (int64_t)unit * a.nsplit * (GROUPS * C::THREADS);
  if constexpr (!SPLIT) {
    // Through LDS, one 32-key block of one matrix at a time: in the accumulator layout a lane
    // holds 4 consecutive d of one key, so a direct store instruction would touch 32 rows with
    // 16 bytes each (256 such instructions per block; at short walks -- 40 steps per block at
    // window 1000 and one q head per kv head -- they took a tenth of the kernel).  Each wave
    // stages its block in the tile buffer nobody reads any more (rows of 16-byte chunks, chunk
    // c of row r at position c ^ (r % chunks-per-row)), and stores whole rows, 16 bytes a lane.
    char* stage = wave == 0 ? q_s0 : wave == 1 ? q_s1 : wave == 2 ? do_s0 : do_s1;
    static_assert(C::Q_TILE >= 32 * C::ROWB, "a 32-key block fits a tile buffer");
    const int wr_row = l32_e * C::ROWB + g_e * 8;
    const int wr_swz = l32_e & (C::CPR - 1);
#pragma unroll
    for (int mtx = 0; mtx < 2; mtx++)
#pragma unroll
      for (int kb = 0; kb < KB; kb++) {
        const float sc = mtx == 0 ? a.scale : 1.f;
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
          for (int i4 = 0; i4 < 4; i4++) {
            const f32x16& acc = mtx == 0 ? dk_acc[kb][d] : dv_acc[kb][d];
            *(typename M::V4*)(stage + wr_row + (((d * 4 + i4) ^ wr_swz) << 4)) =
                M::pack4(acc[4 * i4] * sc, acc[4 * i4 + 1] * sc, acc[4 * i4 + 2] * sc,
                         acc[4 * i4 + 3] * sc);
          }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave's own writes have landed
        void* const dst = mtx == 0 ? dk_buf : dv_buf;
        const int64_t dst_off = mtx == 0 ? dk_off : dv_off;
        const int64_t dst_st = mtx == 0 ? a.dk_st[1] : a.dv_st[1];
#pragma unroll
        for (int n = 0; n < 32 * C::CPR / 64; n++) {
          const int idx = n * 64 + lane_e;
          const int row = idx / C::CPR, c = idx % C::CPR;
          const V8 val = *(const V8*)(stage + row * C::ROWB + ((c ^ (row & (C::CPR - 1))) << 4));
          const int jc = jw0 + kb * 32 + row;
          if (jc < len_k)
            put_grad8<T>(dst, dst_off + (int64_t)jc * dst_st + c * 8, val, a.wide_dkv, a.dkv_accumulate);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // read before the next block overwrites
      }
    return;
  }
  {
    // one running pointer (opaque to the optimiser, or it would keep 64 addresses in registers)
    f32x4* mine = part_base + (int64_t)part * (GROUPS * C::THREADS) + (wave * 64 + lane_e);
#pragma unroll
    for (int mtx = 0; mtx < 2; mtx++)
#pragma unroll
      for (int kb = 0; kb < KB; kb++)
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
          for (int i4 = 0; i4 < 4; i4++) {
            const f32x16& acc = mtx == 0 ? dk_acc[kb][d] : dv_acc[kb][d];
            const f32x4 val = {acc[4 * i4], acc[4 * i4 + 1], acc[4 * i4 + 2], acc[4 * i4 + 3]};
            *mine = val;
            mine += C::THREADS;
            asm volatile("" : "+v"(mine));
          }
  }
  // Release: every wave waits for its own stores, then one thread makes the block's partial
  // sums visible device-wide and counts the block in.  Acquire on the other side: the block
  // that finds itself last drops what its compute unit and L2 may hold of those lines.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    __threadfence();
    arrived_s = atomicAdd(a.dkv_count + unit, 1);
  }
  __syncthreads();
  if (arrived_s != a.nsplit - 1) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  if (tid == 0) a.dkv_count[unit] = 0;  // the next launch on this workspace starts from zero
  // eight value groups at a time, all their loads in flight before the first sum
  const f32x4* parts = part_base + (wave * 64 + lane_e);
  constexpr int GB = 8;
  static_assert(GROUPS % GB == 0, "batches of value groups");
  for (int g0 = 0; g0 < GROUPS; g0 += GB) {  // group = ((mtx KB + kb) DB + d) 4 + i4
    // four loads per group whatever nsplit is (a part past the last reads the last one again
    // and is left out of the sum): no branch, so nothing waits between the loads
    f32x4 v[GB][4];
#pragma unroll
    for (int j = 0; j < GB; j++)
#pragma unroll
      for (int pp = 0; pp < 4; pp++)
        v[j][pp] = parts[(int64_t)min(pp, a.nsplit - 1) * (GROUPS * C::THREADS) + j * C::THREADS];
#pragma unroll
    for (int j = 0; j < GB; j++) {
      f32x4 sum = v[j][0];
#pragma unroll
      for (int pp = 1; pp < 4; pp++) {
        const float use = pp < a.nsplit ? 1.f : 0.f;
        sum += v[j][pp] * use;
      }
      const int grp = g0 + j;
      emit(grp / (KB * DB * 4), grp / (DB * 4) % KB, grp / 4 % DB, grp % 4, sum);
    }
    parts += GB * C::THREADS;
  }
}

// ============================================================================
// dK / dV of sink keys
// ============================================================================
// With sink keys and a bounded window, key j < n_sink is seen by every later row of its
// sequence: a few keys against all the rows, far too thin for MFMA tiles.  Left to the dK/dV
// kernel, the first key tile of every sequence walked every query tile with one wave of four
// at work and took several times as long as any other block (a pack of 65536 tokens in four
// sequences: 10.8 ms, a third of it that tail).  So the dK/dV kernel treats sink keys like any
// other key (band pairs only), and this kernel, which runs after it, computes the sink keys'
// complete dK / dV -- all the rows that see them, inside the window and beyond -- as plain
// fp32 vector work at memory speed, and overwrites those few rows of dk / dv:
//   s = q . k_j, P = exp2(s c - lse2), dP = dO . v_j, dS = P (dP - delta)
//   dV_j = sum P dO, dK_j = scale sum dS q
// One block per (sequence, kv head, chunk of rows); Q and dO are read once per pass of kSinkPass
// sink keys; a lane owns 8 consecutive d of one row at a time (D / 8 lanes per row), the dot
// products are summed across those lanes, and the block's sums -- added in a fixed order -- go
// to the workspace as fp32 [unit][chunk][sink][dK, dV][D].  The block of a unit that arrives
// last adds the chunks in chunk order and writes the rows (same protocol as the split dK/dV
// blocks: deterministic, nobody waits).
constexpr int kSinkPass = 4;

// sum over the aligned group of W = 8 or 16 lanes, in every lane of the group
template <int W>
__device__ __forceinline__ float lane_group_sum(float x) {
  auto dpp = [](float v, auto ctrl) __attribute__((always_inline)) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), decltype(ctrl)::value,
                                                       0xf, 0xf, true));
  };
  if constexpr (W == 16) x += dpp(x, std::integral_constant<int, 0x140>{});  // row_mirror
  x += dpp(x, std::integral_constant<int, 0x141>{});                          // row_half_mirror
  x += dpp(x, std::integral_constant<int, 0x1b>{});                           // quad_perm 3 2 1 0
  x += dpp(x, std::integral_constant<int, 0xb1>{});                           // quad_perm 1 0 3 2
  return x;
}

template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_sink_kernel(const AttnArgs a) {
  using V8 = typename Mma<T>::V8;
  constexpr int LPR = D / 8;     // lanes per row
  constexpr int RPW = 64 / LPR;  // rows per wave pass
  constexpr int NS = kSinkPass;
  constexpr int NSRC = 4 * RPW;  // (wave, row group) sources of the block's sums
  __shared__ float red_s[NSRC][NS * 2 * D];
  static_assert(sizeof(red_s) <= 65536, "staging buffer");

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int sub = lane % LPR, rg = lane / LPR;
  const int c = blockIdx.x % a.sink_chunks;
  const int unit = blockIdx.x / a.sink_chunks;  // (sequence, kv head)
  const int hk = unit % a.heads_kv, b = unit / a.heads_kv;
  int64_t q_row0 = 0, k_row0 = 0;
  int len_q = a.seqlen_q, len_k = a.seqlen_k;
  if (a.cu_q) {
    q_row0 = a.cu_q[b];
    k_row0 = a.cu_k[b];
    len_q = a.cu_q[b + 1] - a.cu_q[b];
    len_k = a.cu_k[b + 1] - a.cu_k[b];
  }
  const int ns_all = min(a.n_sink, len_k);
  // rows of the sequence in n_chunks chunks (at most a.sink_chunks)
  const int rows_per = (len_q + a.sink_chunks - 1) / a.sink_chunks;
  const int n_chunks = rows_per > 0 ? (len_q + rows_per - 1) / rows_per : 0;
  if (c >= n_chunks || ns_all == 0) return;
  const int shift = a.shift_explicit ? a.shift_val : len_k - len_q;
  const int r_begin = c * rows_per, r_end = min(len_q, r_begin + rows_per);

  const T* q_ptr = (const T*)a.q + b * a.q_st[0] + q_row0 * a.q_st[1];
  const T* do_ptr = (const T*)a.dout + b * a.do_st[0] + q_row0 * a.do_st[1];
  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + k_row0 * a.v_st[1] + hk * a.v_st[2];
  const int64_t ws_row0 = a.cu_q ? q_row0 : (int64_t)b * a.seqlen_q;
  float* out = a.sink_part + ((int64_t)unit * a.sink_chunks + c) * (a.n_sink * 2 * D);

  for (int j0 = 0; j0 < ns_all; j0 += NS) {
    float kf[NS][8], vf[NS][8], acck[NS][8], accv[NS][8];
#pragma unroll
    for (int jj = 0; jj < NS; jj++) {
      V8 k8 = V8{0, 0, 0, 0, 0, 0, 0, 0}, v8 = k8;
      if (j0 + jj < ns_all) {
        k8 = *(const V8*)(k_ptr + (int64_t)(j0 + jj) * a.k_st[1] + sub * 8);
        v8 = *(const V8*)(v_ptr + (int64_t)(j0 + jj) * a.v_st[1] + sub * 8);
      }
#pragma unroll
      for (int e = 0; e < 8; e++) {
        kf[jj][e] = (float)k8[e];
        vf[jj][e] = (float)v8[e];
        acck[jj][e] = 0.f;
        accv[jj][e] = 0.f;
      }
    }
    for (int h = 0; h < a.group; h++) {
      const int hq = hk * a.group + h;
      const T* qh = q_ptr + (int64_t)hq * a.q_st[2] + sub * 8;
      const T* doh = do_ptr + (int64_t)hq * a.do_st[2] + sub * 8;
      const float* lse_h = a.lse2 + (int64_t)hq * a.rows_q + ws_row0;
      const float* delta_h = a.delta + (int64_t)hq * a.rows_q + ws_row0;
      for (int base = r_begin + wave * RPW; base < r_end; base += 4 * RPW) {
        const int row = base + rg;
        const bool valid = row < r_end;
        V8 q8 = V8{0, 0, 0, 0, 0, 0, 0, 0}, d8 = q8;
        float nl = -__builtin_inff(), nd = 0.f;  // the statistics are stored negated
        if (valid) {
          q8 = *(const V8*)(qh + (int64_t)row * a.q_st[1]);
          d8 = *(const V8*)(doh + (int64_t)row * a.do_st[1]);
          nl = lse_h[row];
          nd = delta_h[row];
        }
        float qf[8], df[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
          qf[e] = (float)q8[e];
          df[e] = (float)d8[e];
        }
        const int hi = (a.wr >= 0) ? min(len_k - 1, row + shift + a.wr) : len_k - 1;
#pragma unroll
        for (int jj = 0; jj < NS; jj++) {
          float sdot = 0.f, pdot = 0.f;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            sdot = __builtin_fmaf(qf[e], kf[jj][e], sdot);
            pdot = __builtin_fmaf(df[e], vf[jj][e], pdot);
          }
          sdot = lane_group_sum<LPR>(sdot);
          pdot = lane_group_sum<LPR>(pdot);
          const int j = j0 + jj;
          const bool vis = valid && j < ns_all && j <= hi;  // a sink key: no lower bound
          const float p = vis ? __builtin_amdgcn_exp2f(__builtin_fmaf(sdot, a.scale_log2, nl)) : 0.f;
          const float ds = vis ? p * (pdot + nd) : 0.f;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            accv[jj][e] = __builtin_fmaf(p, df[e], accv[jj][e]);
            acck[jj][e] = __builtin_fmaf(ds, qf[e], acck[jj][e]);
          }
        }
      }
    }
    // the block's sums: every (wave, row group) source staged, then added in source order
    __syncthreads();  // the previous pass's readers are done
#pragma unroll
    for (int jj = 0; jj < NS; jj++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        red_s[wave * RPW + rg][(jj * 2 + 0) * D + sub * 8 + e] = acck[jj][e];
        red_s[wave * RPW + rg][(jj * 2 + 1) * D + sub * 8 + e] = accv[jj][e];
      }
    __syncthreads();
    for (int idx = tid; idx < NS * 2 * D; idx += 256) {
      float sum = 0.f;
#pragma unroll
      for (int src = 0; src < NSRC; src++) sum += red_s[src][idx];
      const int jj = idx / (2 * D);
      if (j0 + jj < ns_all) out[(int64_t)(j0 + jj) * (2 * D) + idx % (2 * D)] = sum;
    }
  }
  // count this chunk in; the last one of the unit adds them all up
  __shared__ int arrived_s;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    __threadfence();
    arrived_s = atomicAdd(a.sink_count + unit, 1);
  }
  __syncthreads();
  if (arrived_s != n_chunks - 1) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  if (tid == 0) a.sink_count[unit] = 0;  // the next launch on this workspace starts from zero
  T* dk_ptr = (T*)a.dk + b * a.dk_st[0] + k_row0 * a.dk_st[1] + hk * a.dk_st[2];
  T* dv_ptr = (T*)a.dv + b * a.dv_st[0] + k_row0 * a.dv_st[1] + hk * a.dv_st[2];
  const float* parts = a.sink_part + (int64_t)unit * a.sink_chunks * (a.n_sink * 2 * D);
  for (int idx = tid; idx < ns_all * 2 * D; idx += 256) {
    float sum = 0.f;
    for (int cc = 0; cc < n_chunks; cc++) sum += parts[(int64_t)cc * (a.n_sink * 2 * D) + idx];
    const int j = idx / (2 * D), dd = idx % D;
    if ((idx / D) & 1) {
      dv_ptr[(int64_t)j * a.dv_st[1] + dd] = (T)sum;
    } else {
      dk_ptr[(int64_t)j * a.dk_st[1] + dd] = (T)(sum * a.scale);
    }
  }
}

// ============================================================================
// dQ
// ============================================================================
// LDS read-ahead of the dQ kernel's two matrix sections, in fragments (measured: 7 / 4 and
// 6 / 4 are equal, 12 / 6 is 2-3 % slower; 8 / 4 spills at head_dim 128 -- all 256 registers of
// a lane are in use in the first section once S^T and dP^T are both live -- and is 5 % slower)
#ifndef RSWA_DQ_AH1
#define RSWA_DQ_AH1 7
#endif
#ifndef RSWA_DQ_AH2
#define RSWA_DQ_AH2 4
#endif
// dQ launches whose rows see at most this many keys on average use blocks of 4 waves, two per
// compute unit (measured, 32 / 8 heads, head_dim 128: window 256 -22 %, window 1000 -8 %, the rank
// step with its half-empty previous-chunk block -1.4 %; sequences of 16384 and more rows at
// window 4096 +1 %; 32 = 32 heads, window 1000: -2 %)
#ifndef RSWA_DQ_SMALL_AVG_KEYS
#define RSWA_DQ_SMALL_AVG_KEYS 3200
#endif
template <int D>
struct DqCfg {
  static constexpr int BN = 64;  // keys per step
  static constexpr int KS = D / 32;   // k-steps of the 16x16x32 MFMAs over the head dim
  static constexpr int DB = D / 16;   // 16-row blocks of dQ^T
  static constexpr int KBLK = BN / 16;  // 16-key blocks per tile
  static constexpr int CPR = D / 8;
  static constexpr int ROWB = D * 2;
  static constexpr int TILE = BN * ROWB;
  static constexpr int O_STRIDE = D * 2 + 16;
  static_assert(TILE >= 32 * O_STRIDE, "one wave's epilogue staging fits one tile buffer");
};

// Built on v_mfma_f32_16x16x32 (with random operands the matrix pipes sustain about 14 % more
// of these than of the 32x32x16 form before the power limit pulls the clock down).  A wave
// owns 32 query rows as two 16-column blocks: lane l holds query column l % 16 of each block;
// its 8-element fragments cover d = 32 ks + 8 (l / 16) ...; a 64-key tile is four 16-key
// blocks, and S^T / dP^T tiles hold keys 16 kb + 4 (l / 16) + i in element i.  Two such tiles
// of neighbouring key blocks, packed, are the B operand of dQ^T += K^T dS^T over a 32-key slab
// (k order: four keys of the first block, then four of the second); the A operand follows the
// same order: two transposing reads, one per key block.
//
// NW = 8: one block of 8 waves per compute unit (two waves per SIMD).  NW = 4: blocks of 4 waves,
// two of them per compute unit -- the same two waves per SIMD, but from independent blocks, so
// that one block's prologue (three dependent round trips to memory) and epilogue run under the
// other's tiles; the price is that a K / V tile serves half as many rows.
template <typename T, int D, bool FAR, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attn_bwd_dq_kernel(const AttnArgs a) {
  using C = DqCfg<D>;
  static_assert(NW == 8 || NW == 4, "waves per block");
  constexpr int HSH = NW == 8 ? 2 : 1;  // waves per q head in pair mode: 1 << HSH
  using M = Mma<T>;
  using V8 = typename M::V8;
  constexpr int KS = C::KS, DB = C::DB, KBLK = C::KBLK;
  __shared__ __attribute__((aligned(1024))) char k_s0[C::TILE];
  __shared__ __attribute__((aligned(1024))) char k_s1[C::TILE];
  __shared__ __attribute__((aligned(1024))) char v_s0[C::TILE];
  __shared__ __attribute__((aligned(1024))) char v_s1[C::TILE];

  const int wid = logical_block_id(a.n_work);
  if (wid < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;   // column (query) / row (key, d) inside a 16 block
  const int u = lane >> 4;   // k group

  // pair mode: waves 0-3 and 4-7 take the same 128 rows of two neighbouring q heads;
  // row mode: the 8 waves take 256 consecutive rows of one q head
  const bool pair = (a.group & 1) == 0;
  const int units = pair ? a.group >> 1 : a.group;
  const int bm = pair ? 16 * NW : 32 * NW;
  const int hu = wid % units;
  int rest = wid / units;
  const int slot = a.rev_q ? a.n_tile - 1 - rest % a.n_tile : rest % a.n_tile;
  rest /= a.n_tile;
  const int hk = rest % a.heads_kv;
  const int hq = hk * a.group + (pair ? 2 * hu + (wave >> HSH) : hu);
  SeqInfo s;
  int qt;
  if (a.cu_q) {
    if (!locate_packed(a, slot, (pair ? 4 : 5) + (NW == 8 ? 3 : 2), false, s, qt)) return;
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
  const T* do_ptr = (const T*)a.dout + b * a.do_st[0] + s.q_row0 * a.do_st[1] + hq * a.do_st[2];
  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + s.k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* v_ptr = (const T*)a.v + b * a.v_st[0] + s.k_row0 * a.v_st[1] + hk * a.v_st[2];
  const int64_t dq_off = b * a.dq_st[0] + s.q_row0 * a.dq_st[1] + hq * a.dq_st[2];  // (T or fp32)
  const int64_t ws_row0 = a.cu_q ? s.q_row0 : (int64_t)b * a.seqlen_q;

  // ---- key tiles this block visits (same rule as the forward kernel) -----------
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

  const int r0 = i0 + (pair ? wave & ((1 << HSH) - 1) : wave) * 32;
  const bool wave_valid = r0 < len_q;
  const bool wave_rows_full = r0 + 31 < len_q;
  const RowBounds wb_first = row_bounds(a, r0, len_q, len_k);
  const RowBounds wb_last = row_bounds(a, min(r0 + 31, len_q - 1), len_q, len_k);

  // Q / dO fragments (B operands) and the statistics of the lane's two query rows.  Q is
  // multiplied by scale * log2(e) here, once, and the (negated) statistics are the values the
  // S^T and dP^T accumulator chains start from: the MFMAs then deliver S c - lse2 and
  // dP - delta, and the vector ALU is left with one exponential, one product and the 16-bit
  // conversion per score.  Rounding the scaled Q to 16 bits moves a score by about 2^-9 of its
  // typical magnitude (P by about 0.1 %), a quarter of what rounding P itself to 16 bits does.
  V8 qf[2][KS], dof[2][KS];
  float lse2[2];   // -lse2 of the lane's two queries
  f32x4 delta[2];  // -delta of the same, in all four elements (start value of the dP^T chains)
#pragma unroll
  for (int qb = 0; qb < 2; qb++) {
    const int iq = r0 + 16 * qb + r;
    float l2 = -__builtin_inff(), dl = 0.f;
    if (iq < len_q) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        qf[qb][ks] = *(const V8*)(q_ptr + (int64_t)iq * a.q_st[1] + ks * 32 + u * 8);
        dof[qb][ks] = *(const V8*)(do_ptr + (int64_t)iq * a.do_st[1] + ks * 32 + u * 8);
      }
      l2 = a.lse2[(int64_t)hq * a.rows_q + ws_row0 + iq];
      dl = a.delta[(int64_t)hq * a.rows_q + ws_row0 + iq];
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        qf[qb][ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
        dof[qb][ks] = V8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    lse2[qb] = l2;
    delta[qb] = f32x4{dl, dl, dl, dl};
  }

  f32x4 dq_acc[DB][2];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int qb = 0; qb < 2; qb++) dq_acc[d][qb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // ---- lane-constant LDS offsets (swizzle folded: the varying parts are XOR / immediates) ----
  // row fragments of K / V (16-byte reads): row 16 kb + r, chunk 4 ks + u
  //   offset = (a_row ^ (ks << 6)) + kb * 16 * ROWB
  const int a_row = r * C::ROWB + ((u ^ swz16_f<C::CPR>(r)) << 4);
  // transposing reads of K: row 32 ks2 + 16 blk + 4 u + (r >> 2), chunk 2 db + ((r & 3) >> 1),
  // second half of the chunk for odd r
  //   offset = (t_row ^ (db << 5)) + (32 ks2 + 16 blk) * ROWB
  const int rl = 4 * u + (r >> 2);
  const int t_row = rl * C::ROWB + ((((r & 3) >> 1) ^ swz16_f<C::CPR>(rl)) << 4) + (r & 1) * 8;

  TileDma<D, C::BN, NW * 64, true> k_dma, v_dma;
  k_dma.init(a.k_st[1], tid);
  v_dma.init(a.v_st[1], tid);
  const int k_row_bytes = (int)(a.k_st[1] * 2), v_row_bytes = (int)(a.v_st[1] * 2);
  // (keys in two row ranges: the second range's tensors, at this batch entry and kv head)
  const T* k2_ptr = a.k2 ? (const T*)a.k2 + b * a.k_st[0] + hk * a.k_st[2] : k_ptr;
  const T* v2_ptr = a.v2 ? (const T*)a.v2 + b * a.v_st[0] + hk * a.v_st[2] : v_ptr;
  auto load_tile = [&](int it, char* kd, char* vd) __attribute__((always_inline)) {
    const int j = tile_of(it) * C::BN;
    const KeySeg<T> gk = key_seg(k_ptr, k2_ptr, a.seg, j, len_k);
    const KeySeg<T> gv = key_seg(v_ptr, v2_ptr, a.seg, j, len_k);
    k_dma.load(tile_src<C::BN, FAR>(gk.base, gk.row0, gk.rows, k_row_bytes, C::ROWB), kd);
    v_dma.load(tile_src<C::BN, FAR>(gv.base, gv.row0, gv.rows, v_row_bytes, C::ROWB), vd);
  };

  auto step = [&](int it, const char* kc, const char* vc, char* kn,
                  char* vn) __attribute__((always_inline)) {
    const int j0 = tile_of(it) * C::BN;
    const int j1 = j0 + C::BN - 1;
    if (it + 1 < n_tiles) load_tile(it + 1, kn, vn);
    const bool needed =
        wave_valid && j0 <= wb_last.hi && (j1 >= wb_first.lo || j0 < a.n_sink);
    if (needed) {
      const bool full = wave_rows_full && j1 <= wb_first.hi &&
                        (j0 >= wb_last.lo || j1 < a.n_sink);
      // S^T and dP^T (element i of tile [kb][qb]: key 16 kb + 4 u + i, query 16 qb + r); every
      // K / V fragment read feeds the MFMAs of both query blocks; the chains start from the
      // row statistics.  The two waves of a SIMD overlap best when each keeps its matrix and
      // its vector work apart: vector instructions placed between a wave's own MFMAs hold its
      // MFMAs back, the other wave's do not.
      f32x4 sacc[KBLK][2], pacc[KBLK][2];
      // (the lane offset is made opaque here: its XOR variants, times the buffers, would
      // otherwise be kept in registers across the whole loop)
      int a_off = a_row;
      asm volatile("" : "+v"(a_off));
#pragma unroll
      for (int ks = 0; ks < KS; ks++)
#pragma unroll
        for (int kb = 0; kb < KBLK; kb++) {
          const int off = (a_off ^ (ks << 6)) + kb * 16 * C::ROWB;
          const V8 kfrag = *(const V8*)(kc + off);
          const V8 vfrag = *(const V8*)(vc + off);
#pragma unroll
          for (int qb = 0; qb < 2; qb++) {
            sacc[kb][qb] = M::mfma16(kfrag, qf[qb][ks], ks == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : sacc[kb][qb]);
            pacc[kb][qb] = M::mfma16(vfrag, dof[qb][ks], ks == 0 ? delta[qb] : pacc[kb][qb]);
          }
        }
      {
        constexpr int NRD = 2 * KBLK * KS, AH = RSWA_DQ_AH1;  // LDS reads AH ahead, 2 MFMAs each
        __builtin_amdgcn_sched_group_barrier(0x100, AH, 0);
#pragma unroll
        for (int i = 0; i < NRD - AH; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * AH, 0);
      }
      // P = exp2(S c - lse2), dS^T = P (dP^T - delta), packed slab by slab (32 keys) as the B
      // operands of dQ^T += K^T dS^T
      V8 dsb[2][2];
      auto body = [&](auto full_c) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full_c)::value;
        int hi_rel[2], lo_rel[2], sink_rel = 0, u_m = 0;
        if constexpr (!FULL) {
          // edge tile: the lane's own mask bounds are recomputed here (only a few tiles per
          // block take this path; kept across the loop they would cost registers)
          int lane_m = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
          asm volatile("" : "+v"(lane_m));
          u_m = lane_m >> 4;
          sink_rel = a.n_sink - j0;
#pragma unroll
          for (int qb = 0; qb < 2; qb++) {
            const RowBounds rb = row_bounds(a, r0 + 16 * qb + (lane_m & 15), len_q, len_k);
            hi_rel[qb] = rb.hi - j0;
            lo_rel[qb] = rb.lo - j0;
          }
        }
#pragma unroll
        for (int ks2 = 0; ks2 < 2; ks2++)
#pragma unroll
          for (int qb = 0; qb < 2; qb++) {
            float dsv[8];
#pragma unroll
            for (int e = 0; e < 8; e++) {
              const int kb = 2 * ks2 + (e >> 2), i = e & 3;
              float ds = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][qb][i], a.scale_log2, lse2[qb])) *
                         pacc[kb][qb][i];
              if constexpr (!FULL) {
                const int j = 16 * kb + 4 * u_m + i;
                const bool ok = (j <= hi_rel[qb]) & ((j >= lo_rel[qb]) | (j < sink_rel));
                ds = ok ? ds : 0.f;
              }
              dsv[e] = ds;
            }
            dsb[ks2][qb] = M::pack(dsv);
            asm volatile("" : "+v"(dsb[ks2][qb]));
          }
      };
      if (full) {
        body(std::true_type{});
      } else {
        body(std::false_type{});
      }
      int t_off = t_row;
      asm volatile("" : "+v"(t_off));
#pragma unroll
      for (int ks2 = 0; ks2 < 2; ks2++)
#pragma unroll
        for (int d = 0; d < DB; d++) {
          const int off = (t_off ^ (d << 5)) + ks2 * 32 * C::ROWB;
          const V8 kt = tr_pair<V8>(kc + off, kc + off + 16 * C::ROWB);
#pragma unroll
          for (int qb = 0; qb < 2; qb++) dq_acc[d][qb] = M::mfma16(kt, dsb[ks2][qb], dq_acc[d][qb]);
        }
      {
        constexpr int NFR = 2 * DB, AH = RSWA_DQ_AH2;  // transposed fragments (2 reads, 2 MFMAs each)
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * AH, 0);
#pragma unroll
        for (int i = 0; i < NFR - AH; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 2 * AH, 0);
      }
    }
    __syncthreads();
  };

  if (n_tiles > 0) load_tile(0, k_s0, v_s0);
  __syncthreads();
  for (int it = 0; it < n_tiles; it += 2) {
    step(it, k_s0, v_s0, k_s1, v_s1);
    if (it + 1 < n_tiles) step(it + 1, k_s1, v_s1, k_s0, v_s0);
  }

  // ---- epilogue: dq = scale * acc, transposed through LDS for 16-byte stores ------
  // element i of dq_acc[d][qb] is dQ[query 16 qb + r][16 d + 4 u + i]
  char* stage = (wave & 3) == 0 ? k_s0 : (wave & 3) == 1 ? k_s1 : (wave & 3) == 2 ? v_s0 : v_s1;
  for (int half = 0; half < NW / 4; half++) {
    if ((wave >> 2) == half) {
#pragma unroll
      for (int d = 0; d < DB; d++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
          const auto h4 = M::pack4(dq_acc[d][qb][0] * a.scale, dq_acc[d][qb][1] * a.scale,
                                   dq_acc[d][qb][2] * a.scale, dq_acc[d][qb][3] * a.scale);
          *(typename M::V4*)(stage + (16 * qb + r) * C::O_STRIDE + (16 * d + 4 * u) * 2) = h4;
        }
    }
    __syncthreads();
    if ((wave >> 2) == half) {
#pragma unroll
      for (int n = 0; n < 32 * C::CPR / 64; n++) {
        const int c = lane + n * 64;
        const int row = c / C::CPR, col = (c % C::CPR) * 8;
        if (r0 + row < len_q) {
          const V8 val = *(const V8*)(stage + row * C::O_STRIDE + col * 2);
          put_grad8<T>(a.dq, dq_off + (int64_t)(r0 + row) * a.dq_st[1] + col, val, a.wide_dq,
                       a.dq_accumulate);
        }
      }
    }
    __syncthreads();
  }
}

// ============================================================================
// dQ from handed-over dS
// ============================================================================
// The dK/dV kernel of the hand-off route leaves, per (q head, 32-row query tile, 64-key group),
// the 16-bit dS values it computed (zero where the mask hides a pair): a 4 KiB unit of four
// 1 KiB pieces [32-key block kb][query half ks2], a piece holding for each of its 32 keys 32
// bytes: the key's dS for queries 16 ks2 + {0..3, 8..11} and then 16 ks2 + {4..7, 12..15}.  This
// kernel only computes dQ^T += K^T dS^T (2 D multiply-adds per pair, against the 6 D of the
// kernel that recomputes S and dP), so it is bound by reading those units once: it keeps two
// stages of them in flight while it works on a third.
//
// Block = 4 waves; a wave owns 64 query rows (two 32-row tiles) of one q head: the 4 waves are
// 4 / 2 / 1 q heads of a GQA group on the same 64 / 128 / 256 rows, sharing each 64-key K tile.
// Per 16 keys and wave: A = K^T (32 d x 16 keys, transposing reads of the K tile), B = dS^T
// (16 keys x 32 queries, transposing reads of the unit: the 16-lane groups of such a read take
// 4 keys x 16 queries, which is 128 consecutive bytes of a piece), C = dQ^T (lane = query).
template <int D>
struct DqDsCfg {
  static constexpr int BN = 64;   // keys per stage
  static constexpr int NST = 3;   // stages held in LDS
  static constexpr int ROWB = D * 2;
  static constexpr int CPR = D / 8;
  static constexpr int DBLK = D / 32;
  static constexpr int K_TILE = BN * ROWB;
  // LDS image of a unit: piece (kb, ks2) at kb KBLK + ks2 PIECE1 -- 128 bytes between the two
  // query halves, which the two halves of a half-wave read together, put them on different banks
  static constexpr int PIECE1 = 1024 + 128;
  static constexpr int KBLK = 2048 + 256;
  static constexpr int UNIT_LDS = 2 * KBLK;
  static constexpr int WAVE_LDS = 2 * UNIT_LDS;
  static constexpr int O_STRIDE = D * 2 + 16;
  static_assert(WAVE_LDS >= 32 * O_STRIDE, "a wave's epilogue staging fits its dS buffers of a stage");
  static constexpr int NKD = BN * CPR / 256;  // K tile load instructions per wave and stage
  static constexpr int NLD = NKD + 8;         // ... and all loads
};

template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_dq_ds_kernel(const AttnArgs a) {
  using C = DqDsCfg<D>;
  using M = Mma<T>;
  using V8 = typename M::V8;
  constexpr int DB = C::DBLK;
  __shared__ __attribute__((aligned(1024))) char k_s0[C::K_TILE];
  __shared__ __attribute__((aligned(1024))) char k_s1[C::K_TILE];
  __shared__ __attribute__((aligned(1024))) char k_s2[C::K_TILE];
  __shared__ __attribute__((aligned(1024))) char ds_s0[4 * C::WAVE_LDS];
  __shared__ __attribute__((aligned(1024))) char ds_s1[4 * C::WAVE_LDS];
  __shared__ __attribute__((aligned(1024))) char ds_s2[4 * C::WAVE_LDS];

  const int wid = logical_block_id(a.n_work);
  if (wid < 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c32 = lane & 31;  // query column of a tile
  const int gg = lane >> 5;   // k half
  const int i16 = lane & 15;

  // heads per block: 4, 2 or 1 (the rest of the waves go to further 64-row units)
  const int hsh = (a.group & 3) == 0 ? 2 : (a.group & 1) == 0 ? 1 : 0;
  const int units = a.group >> hsh;
  const int bm_log2 = 8 - hsh;  // 64 rows x (4 >> hsh) units
  const int bm = 1 << bm_log2;
  const int hu = wid % units;
  int rest = wid / units;
  const int slot = a.rev_q ? a.n_tile - 1 - rest % a.n_tile : rest % a.n_tile;
  rest /= a.n_tile;
  const int hk = rest % a.heads_kv;
  const int hq = hk * a.group + (hu << hsh) + (wave & ((1 << hsh) - 1));
  SeqInfo s;
  int qt;
  if (a.cu_q) {
    if (!locate_packed(a, slot, bm_log2, false, s, qt)) return;
  } else {
    s.batch_idx = rest / a.heads_kv;
    s.q_row0 = s.k_row0 = 0;
    s.len_q = a.seqlen_q;
    s.len_k = a.seqlen_k;
    qt = slot;
  }
  const int b = s.batch_idx;
  const int len_q = s.len_q, len_k = s.len_k;
  const int i0 = qt << bm_log2;
  if (i0 >= len_q) return;

  const T* k_ptr = (const T*)a.k + b * a.k_st[0] + s.k_row0 * a.k_st[1] + hk * a.k_st[2];
  const T* k2_ptr = a.k2 ? (const T*)a.k2 + b * a.k_st[0] + hk * a.k_st[2] : k_ptr;
  const int64_t dq_off = b * a.dq_st[0] + s.q_row0 * a.dq_st[1] + hq * a.dq_st[2];  // (T or fp32)

  // ---- key stages of the block (64 keys each): those any of its rows can see -------------
  const int i_last = min(i0 + bm, len_q) - 1;
  const int lo_blk = row_bounds(a, i0, len_q, len_k).lo;
  const int hi_blk = row_bounds(a, i_last, len_q, len_k).hi;
  const int t_lo = lo_blk / C::BN;
  const int n_st = hi_blk >= lo_blk ? hi_blk / C::BN - t_lo + 1 : 0;

  // ---- this wave's two row tiles, and for which stages j0 the dK/dV kernel wrote their unit:
  // its wave (keys j0 .. j0 + 63) computed tile i iff some pair of the two survives the mask,
  //   i < len_q, j0 < len_k, j0 <= min(i + 31, len_q - 1) + shift + right,
  //   min(j0 + 63, len_k - 1) >= i + shift - left
  const int r0 = i0 + ((wave >> hsh) << 6);
  const int shift = a.shift_explicit ? a.shift_val : len_k - len_q;
  constexpr int kInf = 1 << 30;
  int jmin[2], jmax[2];
#pragma unroll
  for (int t = 0; t < 2; t++) {
    const int it = r0 + 32 * t;
    jmax[t] = (a.wr < 0) ? len_k - 1 : min(len_k - 1, min(it + 31, len_q - 1) + shift + a.wr);
    jmin[t] = (a.wl < 0) ? -kInf : it + shift - a.wl - (C::BN - 1);
    if (it >= len_q || (a.wl >= 0 && it + shift - a.wl > len_k - 1)) jmax[t] = -kInf - 1;
  }

  // ---- the wave's dS units: rows of ds_nkb blocks of 4 units per (head, tile slot) ---------
  const int ds_row_bytes = a.ds_nkb * kDsBlockBytes;
  const int64_t ds_head_bytes = (int64_t)a.ds_slots * ds_row_bytes;
  const int64_t slot0 = a.cu_q ? (s.q_row0 >> 5) + b : (int64_t)b * ((a.seqlen_q + 31) >> 5);
  const int64_t ds_off = hq * ds_head_bytes + (slot0 + (r0 >> 5)) * ds_row_bytes;
  const int64_t ds_left = (int64_t)a.heads_q * ds_head_bytes - ds_off;  // bytes up to the buffer's end
  const int ds_span = r0 < len_q ? (int)min((int64_t)2 * ds_row_bytes, ds_left) : 0;
  const __amdgpu_buffer_rsrc_t ds_rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)(a.ds + (ds_span > 0 ? ds_off : 0)), 0, ds_span, 0x00020000);
  const int ds_voff = lane * 16;

  TileDma<D, C::BN, 256> k_dma;
  k_dma.init(a.k_st[1], tid);
  const int k_row_bytes = (int)(a.k_st[1] * 2);

  // load cursor: the stage fetched next
  int ld_j = t_lo * C::BN;
  int ld_kb = (ld_j >> 8) % a.ds_nkb;
  auto load_stage = [&](char* kd, char* dsd) __attribute__((always_inline)) {
    const KeySeg<T> gk = key_seg(k_ptr, k2_ptr, a.seg, ld_j, len_k);
    k_dma.load(tile_src<C::BN, false>(gk.base, gk.row0, gk.rows, k_row_bytes, C::ROWB), kd);
    const int soff = ld_kb * kDsBlockBytes + ((ld_j >> 6) & 3) * kDsUnitBytes;
    char* dst = dsd + wave * C::WAVE_LDS;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int pc = 0; pc < 4; pc++)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            ds_rsrc, (lds_void_t*)(dst + t * C::UNIT_LDS + (pc >> 1) * C::KBLK + (pc & 1) * C::PIECE1), 16,
            ds_voff, t * ds_row_bytes + soff + pc * 1024, 0, 0);
    ld_j += C::BN;
    if ((ld_j & 255) == 0) ld_kb = ld_kb + 1 == a.ds_nkb ? 0 : ld_kb + 1;
  };

  // ---- lane-constant LDS offsets ------------------------------------------------------------
  // transposing reads of K: rows 16 s + 8 gg + (i16 >> 2) (+ 4), chunk 4 db + 2 (c32 / 16) +
  // ((i16 & 3) >> 1), second half of the chunk for odd i16
  //   offset = (kt_row{0,1} ^ (db << 6)) + s * 16 * ROWB
  const int krow = 8 * gg + (i16 >> 2);
  const int kch = 2 * (c32 >> 4) + ((i16 & 3) >> 1);
  const int kt_row0 = krow * C::ROWB + ((kch ^ swz_f<C::CPR>(krow)) << 4) + (i16 & 1) * 8;
  const int kt_row1 = (krow + 4) * C::ROWB + ((kch ^ swz_f<C::CPR>(krow + 4)) << 4) + (i16 & 1) * 8;
  // transposing reads of a dS unit: key 16 (s & 1) + 8 gg + (i16 >> 2) (+ 4) of block s >> 1,
  // queries 16 (c32 / 16) + 4 (i16 & 3) ..: byte (i16 & 1) 16 + ((i16 >> 1) & 1) 8 of the key's 32
  const int ds_row = (c32 >> 4) * C::PIECE1 + krow * 32 + (i16 & 1) * 16 + ((i16 >> 1) & 1) * 8;

  f32x16 acc[2][DB];
#pragma unroll
  for (int t = 0; t < 2; t++)
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i = 0; i < 16; i++) acc[t][d][i] = 0.f;

  int cur_j = t_lo * C::BN;
  auto stage = [&](int it, const char* kc, const char* dsc, char* kn, char* dsn)
      __attribute__((always_inline)) {
    // this wave's loads of the stage have landed (those of the next one may still fly) ...
    if (it + 1 < n_st) {
      wait_vmem_but<C::NLD>();
    } else {
      wait_vmem_but<0>();
    }
    // ... and everybody's: the K tile is complete, and nobody reads the buffers of the stage
    // before this one any more, which the loads of the stage after the next now overwrite
    lds_barrier();
    if (it + 2 < n_st) load_stage(kn, dsn);
    const int j0 = cur_j;
    cur_j += C::BN;
    const bool n0 = j0 >= jmin[0] && j0 <= jmax[0];
    const bool n1 = j0 >= jmin[1] && j0 <= jmax[1];
    if (!(n0 || n1)) return;
    const char* dsw = dsc + wave * C::WAVE_LDS + ds_row;
    auto body = [&](auto c0, auto c1) __attribute__((always_inline)) {
      constexpr bool T0 = decltype(c0)::value, T1 = decltype(c1)::value;
#pragma unroll
      for (int sl = 0; sl < 4; sl++) {
        V8 kt[DB];
#pragma unroll
        for (int d = 0; d < DB; d++)
          kt[d] = tr_pair<V8>(kc + (kt_row0 ^ (d << 6)) + sl * 16 * C::ROWB,
                              kc + (kt_row1 ^ (d << 6)) + sl * 16 * C::ROWB);
        const int uo = (sl >> 1) * C::KBLK + (sl & 1) * 512;
        if constexpr (T0) {
          const V8 dsf = tr_pair<V8>(dsw + uo, dsw + uo + 128);
#pragma unroll
          for (int d = 0; d < DB; d++) acc[0][d] = M::mfma32(kt[d], dsf, acc[0][d]);
        }
        if constexpr (T1) {
          const V8 dsf = tr_pair<V8>(dsw + C::UNIT_LDS + uo, dsw + C::UNIT_LDS + uo + 128);
#pragma unroll
          for (int d = 0; d < DB; d++) acc[1][d] = M::mfma32(kt[d], dsf, acc[1][d]);
        }
      }
    };
    if (n0 && n1) body(std::true_type{}, std::true_type{});
    else if (n0) body(std::true_type{}, std::false_type{});
    else body(std::false_type{}, std::true_type{});
  };

  if (n_st > 0) load_stage(k_s0, ds_s0);
  if (n_st > 1) load_stage(k_s1, ds_s1);
  for (int it = 0; it < n_st; it += 3) {
    stage(it, k_s0, ds_s0, k_s2, ds_s2);
    if (it + 1 < n_st) stage(it + 1, k_s1, ds_s1, k_s0, ds_s0);
    if (it + 2 < n_st) stage(it + 2, k_s2, ds_s2, k_s1, ds_s1);
  }

  // ---- epilogue: dq = scale * acc, a tile at a time through the wave's own LDS ----------------
  // element i of acc[t][d] is dQ[query 32 t + c32][32 d + 8 (i / 4) + 4 gg + i % 4]
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  char* stg = ds_s0 + wave * C::WAVE_LDS;
#pragma unroll
  for (int t = 0; t < 2; t++) {
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++)
        *(typename M::V4*)(stg + c32 * C::O_STRIDE + (32 * d + 8 * i4 + 4 * gg) * 2) =
            M::pack4(acc[t][d][4 * i4] * a.scale, acc[t][d][4 * i4 + 1] * a.scale,
                     acc[t][d][4 * i4 + 2] * a.scale, acc[t][d][4 * i4 + 3] * a.scale);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int n = 0; n < 32 * C::CPR / 64; n++) {
      const int cc = lane + n * 64;
      const int row = cc / C::CPR, col = (cc % C::CPR) * 8;
      const V8 val = *(const V8*)(stg + row * C::O_STRIDE + col * 2);
      if (r0 + 32 * t + row < len_q)
        put_grad8<T>(a.dq, dq_off + (int64_t)(r0 + 32 * t + row) * a.dq_st[1] + col, val, a.wide_dq,
                     a.dq_accumulate);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

// ============================================================================
// row statistics, stored negated: -delta = -sum_d dO * O and -lse2 = -lse * log2(e) (empty
// rows: -inf, so that P = exp2(S*c - lse2) is zero).  One 16-lane (D=128) or 8-lane (D=64) group per
// (row, head).
// ============================================================================
// A block owns PrepCfg::ROWS consecutive rows of one q head -- the statistics, [head][row], are then
// written as whole cache lines -- and neighbouring blocks take neighbouring heads, so that the
// blocks in flight sweep out / dout as one dense front; all eight loads of a thread's four rows
// are issued before the first use (one row per thread and the heads innermost: 39 -> 27 us on
// 8192 rows x 32 heads, head_dim 128).
template <int D>
struct PrepCfg {
  static constexpr int LPR = D / 8;         // lanes per row
  static constexpr int RP = 256 / LPR;      // rows per pass
  static constexpr int NR = 4;              // passes
  static constexpr int ROWS = RP * NR;      // rows per block
};

template <typename T, int D>
__global__ __launch_bounds__(256) void attn_bwd_prep_kernel(const AttnArgs a) {
  using P = PrepCfg<D>;
  using V8 = typename Mma<T>::V8;
  // arrival counters of the dK/dV kernel's split blocks start from zero
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < a.n_count; i += (int64_t)gridDim.x * 256)
    a.dkv_count[i] = 0;
  // The delta array starts at the next 256-byte boundary after the lse2 array, and the tile
  // kernels read up to a tile of rows past the last one as statistics: the elements in between
  // get the neutral value (P exactly zero) rather than whatever the workspace held.
  if (blockIdx.x == 0) {
    const int64_t used = a.rows_q * a.heads_q;
    if (used + threadIdx.x < a.delta - a.lse2) a.lse2[used + threadIdx.x] = -__builtin_inff();
  }
  const int h = (int)(blockIdx.x % (unsigned)a.heads_q);
  const int64_t row0 = (int64_t)(blockIdx.x / (unsigned)a.heads_q) * P::ROWS + threadIdx.x / P::LPR;
  const int c = (threadIdx.x % P::LPR) * 8;
  // Packed rows past the last sequence belong to nobody: their out / dout may hold anything
  // (NaN included), and the tile kernels read the statistics of the rows that follow a
  // sequence's last tile.  They get the neutral pair, which keeps P and dS exactly zero.
  const int64_t rows_real = a.cu_q ? (int64_t)a.cu_q[a.batch] : a.rows_q;
  V8 o8[P::NR], d8[P::NR];
  float l[P::NR];
#pragma unroll
  for (int i = 0; i < P::NR; i++) {
    const int64_t row = row0 + i * P::RP;
    o8[i] = d8[i] = V8{0, 0, 0, 0, 0, 0, 0, 0};
    l[i] = -__builtin_inff();
    if (row < rows_real) {
      int64_t o_off, do_off, l_off;
      if (a.cu_q) {
        o_off = row * a.o_st[1];
        do_off = row * a.do_st[1];
        l_off = row * a.lse_st[2];
      } else {
        const int64_t bb = row / a.seqlen_q, ii = row % a.seqlen_q;
        o_off = bb * a.o_st[0] + ii * a.o_st[1];
        do_off = bb * a.do_st[0] + ii * a.do_st[1];
        l_off = bb * a.lse_st[0] + ii * a.lse_st[2];
      }
      o8[i] = *(const V8*)((const T*)a.out + o_off + h * a.o_st[2] + c);
      d8[i] = *(const V8*)((const T*)a.dout + do_off + h * a.do_st[2] + c);
      if (c == 0) l[i] = a.lse[l_off + h * a.lse_st[1]];
    }
  }
#pragma unroll
  for (int i = 0; i < P::NR; i++) {
    const int64_t row = row0 + i * P::RP;
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) acc += (float)o8[i][j] * (float)d8[i][j];
#pragma unroll
    for (int m = P::LPR / 2; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
    if (c == 0 && row < a.rows_q) {
      a.delta[(int64_t)h * a.rows_q + row] = -acc;  // (rows nobody owns: -0)
      a.lse2[(int64_t)h * a.rows_q + row] = (l[i] == -__builtin_inff()) ? l[i] : -l[i] * kLog2e;
    }
  }
}

// Explicit instantiations: with implicit instantiation alone this hipcc emits the host
// launch stubs of only some of the variants.
#define RSWA_INSTANTIATE(T, D)                                              \
  template __global__ void attn_bwd_dkdv_kernel<T, D, false, false, false>(const AttnArgs); \
  template __global__ void attn_bwd_dkdv_kernel<T, D, true, false, false>(const AttnArgs);  \
  template __global__ void attn_bwd_dkdv_kernel<T, D, false, true, false>(const AttnArgs);  \
  template __global__ void attn_bwd_dkdv_kernel<T, D, true, true, false>(const AttnArgs);   \
  template __global__ void attn_bwd_dkdv_kernel<T, D, false, false, true>(const AttnArgs);  \
  template __global__ void attn_bwd_dq_ds_kernel<T, D>(const AttnArgs);                     \
  template __global__ void attn_bwd_dq_kernel<T, D, false, 8>(const AttnArgs);       \
  template __global__ void attn_bwd_dq_kernel<T, D, true, 8>(const AttnArgs);        \
  template __global__ void attn_bwd_dq_kernel<T, D, false, 4>(const AttnArgs);       \
  template __global__ void attn_bwd_dq_kernel<T, D, true, 4>(const AttnArgs);        \
  template __global__ void attn_bwd_sink_kernel<T, D>(const AttnArgs);                  \
  template __global__ void attn_bwd_prep_kernel<T, D>(const AttnArgs);
RSWA_INSTANTIATE(__bf16, 128)
RSWA_INSTANTIATE(__bf16, 64)
RSWA_INSTANTIATE(_Float16, 128)
RSWA_INSTANTIATE(_Float16, 64)
#undef RSWA_INSTANTIATE

template <typename T, int D>
int launch_bwd(AttnArgs& a, hipStream_t stream, int phases) {
  const int64_t units = a.rows_q * a.heads_q;
  if (units > 0 && (phases & RSWA_BWD_PREP)) {
    const int64_t blocks = ceil_div(a.rows_q, PrepCfg<D>::ROWS) * a.heads_q;
    RSWA_REQUIRE(blocks < (1ll << 31), RSWA_ERR_UNSUPPORTED, "attn_bwd: too many (row, head) pairs");
    clear_launch_error();
    hipLaunchKernelGGL((attn_bwd_prep_kernel<T, D>), dim3((unsigned)blocks), dim3(256), 0, stream, a);
    int rc = check_launch("attn_bwd prep");
    if (rc != RSWA_OK) return rc;
  }
  if (phases & RSWA_BWD_DKDV) {
    using C = DkvCfg<D>;
    if (a.rows_q == 0) a.nsplit = 1;  // nothing to walk (and no statistics launch ran)
    if (a.cu_q) {
      a.n_tile = (int)(ceil_div(a.rows_k, C::BN) + a.batch);
      a.n_work = a.n_tile * a.heads_kv * a.nsplit;
    } else {
      a.n_tile = (int)ceil_div(a.seqlen_k, C::BN);
      a.n_work = a.n_tile * a.heads_kv * a.batch * a.nsplit;
    }
    if (a.n_work > 0) {
      clear_launch_error();
      const dim3 grid(padded_grid(a.n_work)), block(C::THREADS);
      if (a.ds) {  // (never with a.far or a.nsplit > 1: see bwd_layout)
        hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, false, false, true>), grid, block, 0, stream, a);
      } else if (a.nsplit > 1) {
        if (a.far) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, true, true, false>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, true, false, false>), grid, block, 0, stream, a);
      } else {
        if (a.far) hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, false, true, false>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((attn_bwd_dkdv_kernel<T, D, false, false, false>), grid, block, 0, stream, a);
      }
      int rc = check_launch("attn_bwd dkdv");
      if (rc != RSWA_OK) return rc;
    }
    if (a.n_work > 0 && a.sink_part && a.rows_q > 0) {
      clear_launch_error();
      hipLaunchKernelGGL((attn_bwd_sink_kernel<T, D>), dim3(a.batch * a.heads_kv * a.sink_chunks),
                         dim3(256), 0, stream, a);
      int rc = check_launch("attn_bwd sink");
      if (rc != RSWA_OK) return rc;
    }
  }
  if ((phases & RSWA_BWD_DQ) && a.ds) {
    const int hsh = (a.group & 3) == 0 ? 2 : (a.group & 1) == 0 ? 1 : 0;
    const int bm = 256 >> hsh;
    const int units_q = (a.group >> hsh) * a.heads_kv;
    if (a.cu_q) {
      a.n_tile = (int)(ceil_div(a.rows_q, bm) + a.batch);
      a.n_work = a.n_tile * units_q;
    } else {
      a.n_tile = (int)ceil_div(a.seqlen_q, bm);
      a.n_work = a.n_tile * units_q * a.batch;
    }
    if (a.n_work > 0) {
      clear_launch_error();
      hipLaunchKernelGGL((attn_bwd_dq_ds_kernel<T, D>), dim3(padded_grid(a.n_work)), dim3(256), 0,
                         stream, a);
      int rc = check_launch("attn_bwd dq (dS hand-off)");
      if (rc != RSWA_OK) return rc;
    }
  } else if (phases & RSWA_BWD_DQ) {
    const bool pair = (a.group & 1) == 0;
    const bool small = a.avg_keys <= RSWA_DQ_SMALL_AVG_KEYS;
    const int bm = (pair ? 16 : 32) * (small ? 4 : 8);
    const int units_q = (pair ? a.group / 2 : a.group) * a.heads_kv;  // blocks per q tile
    if (a.cu_q) {
      a.n_tile = (int)(ceil_div(a.rows_q, bm) + a.batch);
      a.n_work = a.n_tile * units_q;
    } else {
      a.n_tile = (int)ceil_div(a.seqlen_q, bm);
      a.n_work = a.n_tile * units_q * a.batch;
    }
    if (a.n_work > 0) {
      clear_launch_error();
      const dim3 grid(padded_grid(a.n_work)), block(small ? 256 : 512);
      if (small) {
        if (a.far) hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, true, 4>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, false, 4>), grid, block, 0, stream, a);
      } else {
        if (a.far) hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, true, 8>), grid, block, 0, stream, a);
        else hipLaunchKernelGGL((attn_bwd_dq_kernel<T, D, false, 8>), grid, block, 0, stream, a);
      }
      int rc = check_launch("attn_bwd dq");
      if (rc != RSWA_OK) return rc;
    }
  }
  return RSWA_OK;
}

}  // namespace
}  // namespace rswa

namespace rswa {
namespace {
int bwd_entry(const rswa_attn_params* p, void* stream, int phases, bool allow_split,
              bool allow_handoff) {
  AttnArgs a;
  int rc = fill_args(p, true, a, allow_split, allow_handoff);
  if (rc != RSWA_OK) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (p->dtype == RSWA_BF16) {
    return p->head_dim == 128 ? launch_bwd<__bf16, 128>(a, st, phases)
                              : launch_bwd<__bf16, 64>(a, st, phases);
  }
  return p->head_dim == 128 ? launch_bwd<_Float16, 128>(a, st, phases)
                            : launch_bwd<_Float16, 64>(a, st, phases);
}
}  // namespace
}  // namespace rswa

extern "C" int rswa_attn_bwd_phases(const rswa_attn_params* p, void* stream, int phases) {
  return rswa::bwd_entry(p, stream, phases, true, true);
}

extern "C" int rswa_attn_bwd(const rswa_attn_params* p, void* stream) {
  return rswa_attn_bwd_phases(p, stream, RSWA_BWD_PREP | RSWA_BWD_DKDV | RSWA_BWD_DQ);
}

// ---- backward on the library's own statistics buffer --------------------------------------
// The row statistics of rswa_attn_bwd_static live in this array instead of a caller
// workspace.  In host code the array's name is only a handle: its device address is looked
// up once per device (each GPU holds its own copy) and that pointer is what the kernels get.
static __device__ __align__(256) unsigned char scratch[RSWA_BWD_STATIC_MAX_BYTES];

namespace rswa {
namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices] = {nullptr};

// Device address of `scratch` on the current device (nullptr + error message on failure).
void* scratch_on_current_device() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(RSWA_ERR_LAUNCH, "attn_bwd_static: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      fail(RSWA_ERR_LAUNCH, "attn_bwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    scratch_ptr[dev] = ptr;
  }
  return scratch_ptr[dev];
}
}  // namespace
}  // namespace rswa

extern "C" int rswa_attn_bwd_static_init(void) {
  return rswa::scratch_on_current_device() ? RSWA_OK : RSWA_ERR_LAUNCH;
}

extern "C" int rswa_attn_bwd_static(const rswa_attn_params* p, void* stream) {
  using namespace rswa;
  RSWA_REQUIRE(p != nullptr, RSWA_ERR_INVALID, "attn_bwd_static: null params");
  // statistics only: on the built-in buffer the dK/dV kernel never splits its key tiles
  const uint64_t need = bwd_layout(p, false).total_bytes;
  RSWA_REQUIRE(need <= RSWA_BWD_STATIC_MAX_BYTES, RSWA_ERR_UNSUPPORTED,
               "attn_bwd_static: rows * heads_q needs %llu bytes of statistics, the built-in "
               "buffer holds %llu (use rswa_attn_bwd with a caller workspace)",
               (unsigned long long)need, (unsigned long long)RSWA_BWD_STATIC_MAX_BYTES);
  rswa_attn_params q = *p;
  // validate everything else before the device is touched (a placeholder keeps the
  // workspace checks quiet; the real address replaces it below)
  q.workspace = (void*)(uintptr_t)256;
  q.workspace_bytes = RSWA_BWD_STATIC_MAX_BYTES;
  {
    AttnArgs probe;
    int rc = fill_args(&q, true, probe, false);
    if (rc != RSWA_OK) return rc;
  }
  void* ptr = scratch_on_current_device();
  if (!ptr) return RSWA_ERR_LAUNCH;
  q.workspace = ptr;
  return bwd_entry(&q, stream, RSWA_BWD_PREP | RSWA_BWD_DKDV | RSWA_BWD_DQ, false, false);
}
