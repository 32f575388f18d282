// In-place log-sum-exp merge of two attention partials: an HBM-streaming kernel.
//
// Replaces the Triton kernel at ring_swa/ops/merge.py:68-147 (launch :150-193).
// Work unit = one row (b, s, h): head_dim outputs of `o`, `o_new` and one LSE of
// each.  A block owns 64 consecutive s of one (b, h) so the LSE accesses
// ([batch, heads, seq], seq fastest) coalesce, while neighbouring blocks take
// neighbouring heads so that the blocks in flight sweep `o` ([batch, seq, heads,
// dim]) as one dense front.  Each lane moves 8 elements of a row with 16-byte
// accesses; all loads of a thread's rows are issued before the first use.
#include "rswa_common.h"

#include <type_traits>

namespace rswa {
namespace {

struct MergeArgs {
  void* o;
  void* lse;
  const void* on;
  const void* lsen;
  int64_t o_st[3];   // b, s, h
  int64_t on_st[3];
  int64_t l_st[3];   // b, h, s
  int64_t ln_st[3];
  int32_t seqlen, heads, head_dim, n_stile;
  int32_t lse_f64, lsen_f64;
};

// E = 8 or 4 consecutive elements of a row, to / from fp32 registers, with non-temporal accesses
// of 16 bytes where the type allows (8 bytes for four 16-bit elements).
template <typename T, int E>
struct Vec;

template <>
struct Vec<float, 8> {
  static __device__ __forceinline__ void load(const float* p, float (&x)[8]) {
    f32x4 a = __builtin_nontemporal_load((const f32x4*)p);
    f32x4 b = __builtin_nontemporal_load((const f32x4*)p + 1);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      x[i] = a[i];
      x[4 + i] = b[i];
    }
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[8]) {
    f32x4 a = {x[0], x[1], x[2], x[3]};
    f32x4 b = {x[4], x[5], x[6], x[7]};
    __builtin_nontemporal_store(a, (f32x4*)p);
    __builtin_nontemporal_store(b, (f32x4*)p + 1);
  }
};

template <>
struct Vec<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float (&x)[4]) {
    f32x4 a = __builtin_nontemporal_load((const f32x4*)p);
#pragma unroll
    for (int i = 0; i < 4; i++) x[i] = a[i];
  }
  static __device__ __forceinline__ void store(float* p, const float (&x)[4]) {
    f32x4 a = {x[0], x[1], x[2], x[3]};
    __builtin_nontemporal_store(a, (f32x4*)p);
  }
};

template <>
struct Vec<__bf16, 8> {
  static __device__ __forceinline__ void load(const __bf16* p, float (&x)[8]) {
    u32x4 a = __builtin_nontemporal_load((const u32x4*)p);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      x[2 * i] = __uint_as_float(a[i] << 16);
      x[2 * i + 1] = __uint_as_float(a[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(__bf16* p, const float (&x)[8]) {
    f32x8 f = {x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7]};
    bf16x8 h = __builtin_convertvector(f, bf16x8);
    __builtin_nontemporal_store(h, (bf16x8*)p);
  }
};

template <>
struct Vec<__bf16, 4> {
  static __device__ __forceinline__ void load(const __bf16* p, float (&x)[4]) {
    u32x2 a = __builtin_nontemporal_load((const u32x2*)p);
#pragma unroll
    for (int i = 0; i < 2; i++) {
      x[2 * i] = __uint_as_float(a[i] << 16);
      x[2 * i + 1] = __uint_as_float(a[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(__bf16* p, const float (&x)[4]) {
    f32x4 f = {x[0], x[1], x[2], x[3]};
    bf16x4 h = __builtin_convertvector(f, bf16x4);
    __builtin_nontemporal_store(h, (bf16x4*)p);
  }
};

template <>
struct Vec<_Float16, 8> {
  static __device__ __forceinline__ void load(const _Float16* p, float (&x)[8]) {
    f16x8 a = __builtin_nontemporal_load((const f16x8*)p);
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = (float)a[i];
  }
  static __device__ __forceinline__ void store(_Float16* p, const float (&x)[8]) {
    f32x8 f = {x[0], x[1], x[2], x[3], x[4], x[5], x[6], x[7]};
    f16x8 h = __builtin_convertvector(f, f16x8);
    __builtin_nontemporal_store(h, (f16x8*)p);
  }
};

template <>
struct Vec<_Float16, 4> {
  static __device__ __forceinline__ void load(const _Float16* p, float (&x)[4]) {
    f16x4 a = __builtin_nontemporal_load((const f16x4*)p);
#pragma unroll
    for (int i = 0; i < 4; i++) x[i] = (float)a[i];
  }
  static __device__ __forceinline__ void store(_Float16* p, const float (&x)[4]) {
    f32x4 f = {x[0], x[1], x[2], x[3]};
    f16x4 h = __builtin_convertvector(f, f16x4);
    __builtin_nontemporal_store(h, (f16x4*)p);
  }
};

constexpr int kThreads = 256;

// A lane moves E consecutive elements of a row: 8 when the running output is a 16-bit type (16
// bytes of it a lane), 4 when it is fp32 -- 16 bytes a lane again, so that the 64 lanes of every
// access to it cover whole consecutive cache lines.  (With 8 fp32 elements a lane, two 16-byte
// accesses 32 bytes apart, each instruction touched every line half: 69.4 % of the HBM peak on
// 5.45 GB against 75.5 % this way; the library's plain copy kernel reaches 75.8 %.)  Rows per
// thread, all loaded before the first use: 4 and 2 -- with 4 elements a lane 1 to 4 rows were
// timed, 2 is never behind; more rows in flight per thread lose (8: 59 %).
template <typename TO>
struct MergeShape {
  static constexpr int E = sizeof(TO) == 4 ? 4 : 8;
  static constexpr int ROWS = sizeof(TO) == 4 ? 2 : 4;
};

// LPR = lanes per row (power of two, LPR * E >= head_dim).
template <typename TO, typename TN, int LPR>
__global__ __launch_bounds__(kThreads) void merge_kernel(const MergeArgs a) {
  constexpr int E = MergeShape<TO>::E;
  constexpr int kRowsPerThread = MergeShape<TO>::ROWS;
  constexpr int RP = kThreads / LPR;          // rows per pass
  constexpr int BS = RP * kRowsPerThread;     // rows per block
  const int bid = blockIdx.x;
  const int h = bid % a.heads;
  const int rest = bid / a.heads;
  const int st = rest % a.n_stile;
  const int b = rest / a.n_stile;
  const int r = threadIdx.x / LPR;
  const int c = (threadIdx.x % LPR) * E;
  const bool col_ok = c < a.head_dim;

  TO* o = (TO*)a.o + (int64_t)b * a.o_st[0] + (int64_t)h * a.o_st[2] + c;
  const TN* on = (const TN*)a.on + (int64_t)b * a.on_st[0] + (int64_t)h * a.on_st[2] + c;
  const int64_t l_base = (int64_t)b * a.l_st[0] + (int64_t)h * a.l_st[1];
  const int64_t ln_base = (int64_t)b * a.ln_st[0] + (int64_t)h * a.ln_st[1];

  float xo[kRowsPerThread][E], xn[kRowsPerThread][E];
  float la[kRowsPerThread], lb[kRowsPerThread];
  const int s0 = st * BS + r;

#pragma unroll
  for (int i = 0; i < kRowsPerThread; i++) {
    const int s = s0 + i * RP;
    if (s < a.seqlen) {
      la[i] = a.lse_f64 ? (float)((const double*)a.lse)[l_base + (int64_t)s * a.l_st[2]]
                        : ((const float*)a.lse)[l_base + (int64_t)s * a.l_st[2]];
      lb[i] = a.lsen_f64 ? (float)((const double*)a.lsen)[ln_base + (int64_t)s * a.ln_st[2]]
                         : ((const float*)a.lsen)[ln_base + (int64_t)s * a.ln_st[2]];
      if (col_ok) {
        Vec<TO, E>::load(o + (int64_t)s * a.o_st[1], xo[i]);
        Vec<TN, E>::load(on + (int64_t)s * a.on_st[1], xn[i]);
      }
    }
  }

#pragma unroll
  for (int i = 0; i < kRowsPerThread; i++) {
    const int s = s0 + i * RP;
    if (s < a.seqlen) {
      const float ninf = -__builtin_inff();
      const bool both_empty = (la[i] == ninf) && (lb[i] == ninf);
      const float diff = both_empty ? 0.f : lb[i] - la[i];
      // sigmoid(+-diff); exp overflow to +inf gives the exact limits 0 and 1
      // (both sides empty: no mass on either side, the row stays zero)
      const float w_old = both_empty ? 0.f : 1.f / (1.f + __expf(diff));
      const float w_new = both_empty ? 0.f : 1.f / (1.f + __expf(-diff));
      if (col_ok) {
        float y[E];
#pragma unroll
        for (int j = 0; j < E; j++) {
          // a zero weight must annihilate whatever garbage the other side holds
          const float t0 = (w_old == 0.f) ? 0.f : xo[i][j] * w_old;
          const float t1 = (w_new == 0.f) ? 0.f : xn[i][j] * w_new;
          y[j] = t0 + t1;
        }
        Vec<TO, E>::store(o + (int64_t)s * a.o_st[1], y);
      }
      if ((threadIdx.x % LPR) == 0) {
        const float m = fmaxf(la[i], lb[i]);
        const float merged = both_empty ? ninf : m + log1pf(__expf(-fabsf(diff)));
        if (a.lse_f64)
          ((double*)a.lse)[l_base + (int64_t)s * a.l_st[2]] = (double)merged;
        else
          ((float*)a.lse)[l_base + (int64_t)s * a.l_st[2]] = merged;
      }
    }
  }
}

template <typename TO, typename TN>
int launch_merge(const MergeArgs& a, int64_t batch, hipStream_t stream) {
  constexpr int E = MergeShape<TO>::E;
  const int chunks = (a.head_dim + E - 1) / E;
  int lpr = 1;
  while (lpr < chunks) lpr *= 2;
  MergeArgs args = a;
  auto go = [&](auto lpr_c) {
    constexpr int LPR = decltype(lpr_c)::value;
    constexpr int BS = (kThreads / LPR) * MergeShape<TO>::ROWS;
    args.n_stile = (int)ceil_div(a.seqlen, BS);
    const int64_t blocks = (int64_t)args.n_stile * a.heads * batch;
    if (blocks == 0) return;
    clear_launch_error();
    hipLaunchKernelGGL((merge_kernel<TO, TN, LPR>), dim3((unsigned)blocks), dim3(kThreads), 0,
                       stream, args);
  };
  switch (lpr) {
    case 1: go(std::integral_constant<int, 1>{}); break;
    case 2: go(std::integral_constant<int, 2>{}); break;
    case 4: go(std::integral_constant<int, 4>{}); break;
    case 8: go(std::integral_constant<int, 8>{}); break;
    case 16: go(std::integral_constant<int, 16>{}); break;
    case 32: go(std::integral_constant<int, 32>{}); break;
    default: go(std::integral_constant<int, 64>{}); break;
  }
  return check_launch("merge_attn_out");
}

// Plain streaming copy, 16 bytes a lane, four loads of a thread in flight before its first
// store, non-temporal both ways: the yardstick for what a kernel that only moves memory reaches
// on the device it runs on.
__global__ __launch_bounds__(kThreads) void stream_copy_kernel(u32x4* __restrict__ dst,
                                                               const u32x4* __restrict__ src,
                                                               int64_t n16) {
  const int64_t base = (int64_t)blockIdx.x * (kThreads * 4) + threadIdx.x;
  u32x4 v[4];
#pragma unroll
  for (int i = 0; i < 4; i++)
    if (base + i * kThreads < n16) v[i] = __builtin_nontemporal_load(src + base + i * kThreads);
#pragma unroll
  for (int i = 0; i < 4; i++)
    if (base + i * kThreads < n16) __builtin_nontemporal_store(v[i], dst + base + i * kThreads);
}

int elem_bytes(int dt) {
  switch (dt) {
    case RSWA_BF16:
    case RSWA_F16: return 2;
    case RSWA_F32: return 4;
    case RSWA_F64: return 8;
  }
  return 0;
}

}  // namespace
}  // namespace rswa

extern "C" int rswa_stream_copy(void* dst, const void* src, uint64_t bytes, void* stream) {
  using namespace rswa;
  RSWA_REQUIRE(dst && src, RSWA_ERR_INVALID, "stream_copy: null pointer");
  RSWA_REQUIRE(((uintptr_t)dst) % 16 == 0 && ((uintptr_t)src) % 16 == 0 && bytes % 16 == 0,
               RSWA_ERR_UNSUPPORTED, "stream_copy: pointers and size must be multiples of 16 bytes");
  const int64_t n16 = (int64_t)(bytes / 16);
  const int64_t blocks = ceil_div(n16, kThreads * 4);
  RSWA_REQUIRE(blocks < (1ll << 31), RSWA_ERR_UNSUPPORTED, "stream_copy: more than 32 TiB");
  if (blocks == 0) return RSWA_OK;
  clear_launch_error();
  hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)blocks), dim3(kThreads), 0,
                     (hipStream_t)stream, (u32x4*)dst, (const u32x4*)src, n16);
  return check_launch("stream_copy");
}

extern "C" int rswa_merge_attn_out(void* o, int o_dtype, const int64_t* o_stride, void* lse,
                                   int lse_dtype, const int64_t* lse_stride, const void* o_new,
                                   int o_new_dtype, const int64_t* o_new_stride,
                                   const void* lse_new, int lse_new_dtype,
                                   const int64_t* lse_new_stride, int64_t batch, int64_t seqlen,
                                   int64_t heads, int64_t head_dim, void* stream) {
  using namespace rswa;
  RSWA_REQUIRE(batch >= 0 && seqlen >= 0 && heads >= 0, RSWA_ERR_INVALID, "merge: negative size");
  if (batch == 0 || seqlen == 0 || heads == 0) return RSWA_OK;
  RSWA_REQUIRE(o && lse && o_new && lse_new, RSWA_ERR_INVALID, "merge: null tensor");
  RSWA_REQUIRE(o_stride && lse_stride && o_new_stride && lse_new_stride, RSWA_ERR_INVALID,
               "merge: null stride array");
  RSWA_REQUIRE(head_dim > 0 && head_dim % 8 == 0 && head_dim <= 256, RSWA_ERR_UNSUPPORTED,
               "merge: head_dim %lld must be a multiple of 8, at most 256", (long long)head_dim);
  RSWA_REQUIRE(o_stride[3] == 1 && o_new_stride[3] == 1, RSWA_ERR_UNSUPPORTED,
               "merge: head_dim stride must be 1");
  RSWA_REQUIRE(o_dtype == RSWA_BF16 || o_dtype == RSWA_F16 || o_dtype == RSWA_F32,
               RSWA_ERR_UNSUPPORTED, "merge: o dtype %d", o_dtype);
  RSWA_REQUIRE(o_new_dtype == RSWA_BF16 || o_new_dtype == RSWA_F16 || o_new_dtype == RSWA_F32,
               RSWA_ERR_UNSUPPORTED, "merge: o_new dtype %d", o_new_dtype);
  RSWA_REQUIRE(lse_dtype == RSWA_F32 || lse_dtype == RSWA_F64, RSWA_ERR_UNSUPPORTED,
               "merge: lse dtype %d", lse_dtype);
  RSWA_REQUIRE(lse_new_dtype == RSWA_F32 || lse_new_dtype == RSWA_F64, RSWA_ERR_UNSUPPORTED,
               "merge: lse_new dtype %d", lse_new_dtype);
  RSWA_REQUIRE(seqlen < (1ll << 31) && heads < (1 << 20) && batch < (1 << 20), RSWA_ERR_INVALID,
               "merge: size out of range");
  // 16-byte accesses: every row must start on a 16-byte boundary.
  auto aligned = [](const void* p, const int64_t* st, int dt) {
    const int64_t per16 = 16 / elem_bytes(dt);
    if (((uintptr_t)p) % 16) return false;
    for (int i = 0; i < 3; i++)
      if (st[i] % per16) return false;
    return true;
  };
  RSWA_REQUIRE(aligned(o, o_stride, o_dtype) && aligned(o_new, o_new_stride, o_new_dtype),
               RSWA_ERR_UNSUPPORTED, "merge: rows of o / o_new must be 16-byte aligned");

  MergeArgs a;
  a.o = o;
  a.lse = lse;
  a.on = o_new;
  a.lsen = lse_new;
  for (int i = 0; i < 3; i++) {
    a.o_st[i] = o_stride[i];
    a.on_st[i] = o_new_stride[i];
    a.l_st[i] = lse_stride[i];
    a.ln_st[i] = lse_new_stride[i];
  }
  a.seqlen = (int32_t)seqlen;
  a.heads = (int32_t)heads;
  a.head_dim = (int32_t)head_dim;
  a.n_stile = 0;
  a.lse_f64 = lse_dtype == RSWA_F64;
  a.lsen_f64 = lse_new_dtype == RSWA_F64;
  hipStream_t st = (hipStream_t)stream;

#define RSWA_MERGE_CASE(DO, TO, DN, TN) \
  if (o_dtype == DO && o_new_dtype == DN) return launch_merge<TO, TN>(a, batch, st);
  RSWA_MERGE_CASE(RSWA_F32, float, RSWA_BF16, __bf16)
  RSWA_MERGE_CASE(RSWA_BF16, __bf16, RSWA_BF16, __bf16)
  RSWA_MERGE_CASE(RSWA_F32, float, RSWA_F32, float)
  RSWA_MERGE_CASE(RSWA_F32, float, RSWA_F16, _Float16)
  RSWA_MERGE_CASE(RSWA_F16, _Float16, RSWA_F16, _Float16)
  RSWA_MERGE_CASE(RSWA_BF16, __bf16, RSWA_F32, float)
  RSWA_MERGE_CASE(RSWA_F16, _Float16, RSWA_F32, float)
#undef RSWA_MERGE_CASE
  return fail(RSWA_ERR_UNSUPPORTED, "merge: dtype pair o=%d o_new=%d", o_dtype, o_new_dtype);
}
