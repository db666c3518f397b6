// Rotary position embedding of the query and key projections, alone (prompt)
// and fused with the decode-step append into the circular KV cache.
//
// Replaces the step in front of the attention path in the reference's caller
// (MoA/models/llama/modeling_llama.py:238-262): apply_rotary_pos_emb(q, k,
// cos, sin) of transformers 4.44.2 (the reference's pinned dependency,
// requirements.txt:8) followed, in decode, by StaticCircularCache.update
// (MoA/attention/cache_utils.py:1020-1058).  The published formula is
//   x_embed = (x * cos) + (rotate_half(x) * sin),
//   rotate_half(x) = cat(-x[D/2:], x[:D/2]),
// evaluated by torch in the tensors' dtype, that is with one rounding after
// each of the two products and one after the sum.  The kernels round at the
// same three places, so their results are bit-identical to that evaluation.
//
// Both kernels are HBM/latency bound byte work: 128-bit accesses, no LDS.  One
// thread owns a PAIR of 16-byte chunks (elements e..e+7 and e+D/2..e+D/2+7 of
// one head row), reads both and writes both, which makes in-place use safe.
#include "moa_common.h"

// Every product and sum below is rounded on its own, as torch does.  This file must be compiled
// with -ffp-contract=off (the build does): otherwise the compiler contracts the rounded products
// and the sum into v_fma_f16 / v_pk_fma_f16, which rounds once.

namespace moa {

constexpr int kRopeThreads = 256;
constexpr int kRopeRowLanes = 16;   // lanes that share one head row in the fused kernel
constexpr int kRopeRowsPerBlock = kRopeThreads / kRopeRowLanes;

struct EF16 {
  static constexpr int kPerChunk = 8;
  static __device__ __forceinline__ float get(const u32x4& c, int i) {
    const uint32_t w = c[i >> 1];
    return (float)__builtin_bit_cast(_Float16, (uint16_t)((i & 1) ? (w >> 16) : (w & 0xffffu)));
  }
  static __device__ __forceinline__ uint32_t bits(float x) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
  }
  static __device__ __forceinline__ float round(float x) { return (float)(_Float16)x; }
};
struct EBF16 {
  static constexpr int kPerChunk = 8;
  static __device__ __forceinline__ float get(const u32x4& c, int i) {
    const uint32_t w = c[i >> 1];
    return __builtin_bit_cast(float, (i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  static __device__ __forceinline__ uint32_t bits(float x) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
  }
  static __device__ __forceinline__ float round(float x) { return (float)(__bf16)x; }
};
struct EF32 {
  static constexpr int kPerChunk = 4;
  static __device__ __forceinline__ float get(const u32x4& c, int i) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4 f = __builtin_bit_cast(f32x4, c);
    return f[i];
  }
  static __device__ __forceinline__ uint32_t bits(float x) { return __builtin_bit_cast(uint32_t, x); }
  static __device__ __forceinline__ float round(float x) { return x; }
};

// lo/hi: chunk e..e+k-1 of the first half of a row and the chunk D/2 further; cl/sl, ch/sh: the
// cos and sin chunks at the same places.  Three roundings per element, no fused multiply-add.
template <typename E>
__device__ __forceinline__ void rope_pair(const u32x4& lo, const u32x4& hi, const u32x4& cl, const u32x4& sl,
                                          const u32x4& ch, const u32x4& sh, u32x4& out_lo, u32x4& out_hi) {
  uint32_t ol[E::kPerChunk], oh[E::kPerChunk];
#pragma unroll
  for (int i = 0; i < E::kPerChunk; ++i) {
    const float x1 = E::get(lo, i), x2 = E::get(hi, i);
    // first half: x1*cos + (-x2)*sin = x1*cos - x2*sin (rounding is symmetric, so the sign may move
    // out of the product); second half: x2*cos + x1*sin
    const float a1 = E::round(__fmul_rn(x1, E::get(cl, i)));
    const float b1 = E::round(__fmul_rn(x2, E::get(sl, i)));
    const float a2 = E::round(__fmul_rn(x2, E::get(ch, i)));
    const float b2 = E::round(__fmul_rn(x1, E::get(sh, i)));
    ol[i] = E::bits(__fsub_rn(a1, b1));
    oh[i] = E::bits(__fadd_rn(a2, b2));
  }
  if constexpr (E::kPerChunk == 8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out_lo[i] = ol[2 * i] | (ol[2 * i + 1] << 16);
      out_hi[i] = oh[2 * i] | (oh[2 * i + 1] << 16);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out_lo[i] = ol[i];
      out_hi[i] = oh[i];
    }
  }
}

template <typename E>
__device__ __forceinline__ void rope_row_pair(const char* src, char* dst,
                                              const char* __restrict__ cos_row, const char* __restrict__ sin_row,
                                              int pair, int half_bytes) {
  const size_t o_lo = (size_t)pair * 16, o_hi = o_lo + half_bytes;
  const u32x4 lo = *reinterpret_cast<const u32x4*>(src + o_lo);
  const u32x4 hi = *reinterpret_cast<const u32x4*>(src + o_hi);
  const u32x4 cl = *reinterpret_cast<const u32x4*>(cos_row + o_lo);
  const u32x4 ch = *reinterpret_cast<const u32x4*>(cos_row + o_hi);
  const u32x4 sl = *reinterpret_cast<const u32x4*>(sin_row + o_lo);
  const u32x4 sh = *reinterpret_cast<const u32x4*>(sin_row + o_hi);
  u32x4 out_lo, out_hi;
  rope_pair<E>(lo, hi, cl, sl, ch, sh, out_lo, out_hi);
  *reinterpret_cast<u32x4*>(dst + o_lo) = out_lo;
  *reinterpret_cast<u32x4*>(dst + o_hi) = out_hi;
}

struct RopeTensor {
  const char* src;
  char* dst;
  int64_t sb, sh, sn;   // source byte strides (batch, head, token)
  int64_t db, dh, dn;   // destination byte strides
};

// q and k of a whole prompt (or of one step): one thread per chunk pair.  Consecutive threads walk a row,
// then the dimension in which the SOURCE rows lie closer together (heads for views of [B, N, H, D]
// projections, tokens for [B, H, N, D] tensors), so that a wave reads one consecutive piece of memory.
template <typename E>
__global__ __launch_bounds__(kRopeThreads) void rope_kernel(RopeTensor tq, RopeTensor tk,
                                                             const char* __restrict__ cos,
                                                             const char* __restrict__ sin, int64_t cs_sb,
                                                             int64_t cs_sn, int B, int Hq, int Hkv, int N,
                                                             int pairs_per_row, int half_bytes, bool heads_inner) {
  const int64_t idx = (int64_t)blockIdx.x * kRopeThreads + threadIdx.x;
  const int64_t total = (int64_t)B * (Hq + Hkv) * N * pairs_per_row;
  if (idx >= total) return;
  const int pair = (int)(idx % pairs_per_row);
  int64_t row = idx / pairs_per_row;
  int n, hh;
  if (heads_inner) {
    hh = (int)(row % (Hq + Hkv));
    row /= (Hq + Hkv);
    n = (int)(row % N);
    row /= N;
  } else {
    n = (int)(row % N);
    row /= N;
    hh = (int)(row % (Hq + Hkv));
    row /= (Hq + Hkv);
  }
  const int b = (int)row;
  const bool is_q = hh < Hq;
  const RopeTensor& t = is_q ? tq : tk;
  const int h = is_q ? hh : hh - Hq;
  rope_row_pair<E>(t.src + b * t.sb + h * t.sh + n * t.sn, t.dst + b * t.db + h * t.dh + n * t.dn,
                   cos + b * cs_sb + n * cs_sn, sin + b * cs_sb + n * cs_sn, pair, half_bytes);
}

// Decode step: rotate q into q_out, rotate k into its ring slot, copy v into its ring slot, and
// advance the ring bookkeeping exactly as cache_append_kernel does (cache_utils.py:1020-1058).
// One group of 16 lanes per (batch row, query head) and per (batch row, kv head).
template <typename E>
__global__ __launch_bounds__(kRopeThreads) void rope_append_kernel(
    const char* __restrict__ q_new, const char* __restrict__ k_new, const char* __restrict__ v_new,
    int64_t qn_sb, int64_t qn_sh, int64_t kn_sb, int64_t kn_sh, int64_t vn_sb, int64_t vn_sh,
    const char* __restrict__ cos, const char* __restrict__ sin, int64_t cs_sb, char* __restrict__ q_out,
    char* __restrict__ kc, char* __restrict__ vc, int64_t* __restrict__ mask_cache,
    int64_t* __restrict__ update_index, int64_t* __restrict__ valid_len,
    const int64_t* __restrict__ circ_head, const int64_t* __restrict__ circ_size,
    const int64_t* __restrict__ static_size, const int64_t* __restrict__ max_len, int64_t kv_len, int B,
    int Hq, int Hkv, int row_bytes, int64_t sumC) {
  const int lane = threadIdx.x % kRopeRowLanes;
  const int64_t unit = (int64_t)blockIdx.x * kRopeRowsPerBlock + threadIdx.x / kRopeRowLanes;
  if (unit >= (int64_t)B * (Hq + Hkv)) return;
  const int b = (int)(unit / (Hq + Hkv));
  const int r = (int)(unit % (Hq + Hkv));
  const int half_bytes = row_bytes / 2;
  const int pairs = half_bytes / 16;
  const char* cos_row = cos + b * cs_sb;
  const char* sin_row = sin + b * cs_sb;
  if (r < Hq) {
    const char* src = q_new + b * qn_sb + r * qn_sh;
    char* dst = q_out + ((size_t)b * Hq + r) * row_bytes;
    for (int p = lane; p < pairs; p += kRopeRowLanes) rope_row_pair<E>(src, dst, cos_row, sin_row, p, half_bytes);
    return;
  }
  const int h = r - Hq;
  const int64_t bh = (int64_t)b * Hkv + h;
  const int64_t idx = update_index[bh];
  const bool in_range = idx >= 0 && idx < sumC;
  if (in_range) {
    const size_t dst = ((size_t)b * sumC + idx) * row_bytes;
    for (int p = lane; p < pairs; p += kRopeRowLanes)
      rope_row_pair<E>(k_new + b * kn_sb + h * kn_sh, kc + dst, cos_row, sin_row, p, half_bytes);
    const char* vsrc = v_new + b * vn_sb + h * vn_sh;
    for (int u = lane; u < row_bytes / 16; u += kRopeRowLanes)
      *reinterpret_cast<u32x4*>(vc + dst + (size_t)u * 16) = *reinterpret_cast<const u32x4*>(vsrc + (size_t)u * 16);
  }
  if (lane == 0) {
    if (in_range && mask_cache != nullptr) mask_cache[(size_t)b * sumC + idx] = 1;
    const int64_t vl = valid_len[bh];
    valid_len[bh] = vl + (vl < max_len[h] ? 1 : 0);
    const bool is_circular = (kv_len + 1) > static_size[h];
    int64_t next = idx + 1;
    if (is_circular) {
      const int64_t chd = circ_head[h];
      next = py_mod(idx + 1 - chd, circ_size[h]) + chd;
    }
    update_index[bh] = next;
  }
}

static int check_rope_rows(const char* who, const char* name, int D, int eb, const int64_t* strides, int nstr,
                           const void* p) {
  if (!p) return fail(MOA_ERR_ARG, "%s: null %s", who, name);
  if (!strides) return fail(MOA_ERR_ARG, "%s: null %s strides", who, name);
  if (strides[nstr - 1] != 1) return fail(MOA_ERR_ARG, "%s: innermost %s stride must be 1", who, name);
  for (int i = 0; i < nstr - 1; ++i)
    if ((strides[i] * eb) % 16 != 0)
      return fail(MOA_ERR_ARG, "%s: %s stride %d (%lld elements) breaks 16-byte row alignment", who, name, i,
                  (long long)strides[i]);
  if (!aligned16(p)) return fail(MOA_ERR_ARG, "%s: %s must be 16-byte aligned", who, name);
  (void)D;
  return MOA_OK;
}

static int check_head_dim(const char* who, int D, int dtype, int* eb_out) {
  const int eb = elem_bytes(dtype);
  if (eb == 0) return fail(MOA_ERR_ARG, "%s: unknown dtype %d", who, dtype);
  if (D <= 0 || (D * eb) % 32 != 0)
    return fail(MOA_ERR_UNSUPPORTED, "%s: half a head row (head_dim %d, %d-byte elements) is not a multiple of 16 bytes",
                who, D, eb);
  *eb_out = eb;
  return MOA_OK;
}

}  // namespace moa

using namespace moa;

extern "C" int moa_rope_fwd(const void* q, const void* k, void* q_out, void* k_out, const int64_t* q_strides,
                            const int64_t* k_strides, const int64_t* qo_strides, const int64_t* ko_strides,
                            const void* cos, const void* sin, const int64_t* cs_strides, int B, int Hq, int Hkv,
                            int N, int D, int dtype, void* stream) {
  const char* who = "moa_rope_fwd";
  if (B <= 0 || Hq < 0 || Hkv < 0 || Hq + Hkv <= 0 || N <= 0) return fail(MOA_ERR_ARG, "%s: B, H, N must be positive", who);
  int eb = 0, rc;
  if ((rc = check_head_dim(who, D, dtype, &eb))) return rc;
  if (Hq > 0) {
    if ((rc = check_rope_rows(who, "q", D, eb, q_strides, 4, q))) return rc;
    if ((rc = check_rope_rows(who, "q_out", D, eb, qo_strides, 4, q_out))) return rc;
  }
  if (Hkv > 0) {
    if ((rc = check_rope_rows(who, "k", D, eb, k_strides, 4, k))) return rc;
    if ((rc = check_rope_rows(who, "k_out", D, eb, ko_strides, 4, k_out))) return rc;
  }
  if ((rc = check_rope_rows(who, "cos", D, eb, cs_strides, 3, cos))) return rc;
  if ((rc = check_rope_rows(who, "sin", D, eb, cs_strides, 3, sin))) return rc;
  RopeTensor tq = {}, tk = {};
  if (Hq > 0)
    tq = {(const char*)q, (char*)q_out, q_strides[0] * eb, q_strides[1] * eb, q_strides[2] * eb,
          qo_strides[0] * eb, qo_strides[1] * eb, qo_strides[2] * eb};
  if (Hkv > 0)
    tk = {(const char*)k, (char*)k_out, k_strides[0] * eb, k_strides[1] * eb, k_strides[2] * eb,
          ko_strides[0] * eb, ko_strides[1] * eb, ko_strides[2] * eb};
  const int half_bytes = D * eb / 2;
  const int pairs = half_bytes / 16;
  const int64_t total = (int64_t)B * (Hq + Hkv) * N * pairs;
  const int64_t blocks = (total + kRopeThreads - 1) / kRopeThreads;
  if (blocks > 0x7fffffffLL) return fail(MOA_ERR_UNSUPPORTED, "%s: too many rows", who);
  hipStream_t st = (hipStream_t)stream;
  const int64_t csb = cs_strides[0] * eb, csn = cs_strides[1] * eb;
  const RopeTensor& lead = Hq > 0 ? tq : tk;
  const bool heads_inner = lead.sh < lead.sn;
#define MOA_ROPE_LAUNCH(E)                                                                                  \
  hipLaunchKernelGGL(rope_kernel<E>, dim3((unsigned)blocks), dim3(kRopeThreads), 0, st, tq, tk,             \
                     (const char*)cos, (const char*)sin, csb, csn, B, Hq, Hkv, N, pairs, half_bytes, heads_inner)
  if (dtype == MOA_DTYPE_F16) MOA_ROPE_LAUNCH(EF16);
  else if (dtype == MOA_DTYPE_BF16) MOA_ROPE_LAUNCH(EBF16);
  else MOA_ROPE_LAUNCH(EF32);
#undef MOA_ROPE_LAUNCH
  return check_launch(who);
}

extern "C" int moa_rope_cache_append(const void* q_new, const void* k_new, const void* v_new,
                                     const int64_t* qn_strides, const int64_t* kn_strides,
                                     const int64_t* vn_strides, const void* cos, const void* sin,
                                     int64_t cs_stride_b, void* q_out, void* kc, void* vc, int64_t* mask_cache,
                                     int64_t* update_index, int64_t* valid_len, const int64_t* circ_head,
                                     const int64_t* circ_size, const int64_t* static_size, const int64_t* max_len,
                                     int64_t kv_len, int B, int Hq, int Hkv, int D, int64_t sumC, int dtype,
                                     void* stream) {
  const char* who = "moa_rope_cache_append";
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || sumC <= 0) return fail(MOA_ERR_ARG, "%s: B, Hq, Hkv, sumC must be positive", who);
  if (!update_index || !valid_len || !circ_head || !circ_size || !static_size || !max_len)
    return fail(MOA_ERR_ARG, "%s: null index array", who);
  if (!kc || !vc || !q_out) return fail(MOA_ERR_ARG, "%s: null kc, vc or q_out", who);
  int eb = 0, rc;
  if ((rc = check_head_dim(who, D, dtype, &eb))) return rc;
  if ((rc = check_rope_rows(who, "q_new", D, eb, qn_strides, 3, q_new))) return rc;
  if ((rc = check_rope_rows(who, "k_new", D, eb, kn_strides, 3, k_new))) return rc;
  if ((rc = check_rope_rows(who, "v_new", D, eb, vn_strides, 3, v_new))) return rc;
  if (!cos || !sin) return fail(MOA_ERR_ARG, "%s: null cos or sin", who);
  if ((cs_stride_b * eb) % 16 != 0 || !aligned16(cos) || !aligned16(sin) || !aligned16(q_out) || !aligned16(kc) ||
      !aligned16(vc))
    return fail(MOA_ERR_ARG, "%s: cos, sin, q_out, kc, vc must be 16-byte aligned rows", who);
  const int64_t units = (int64_t)B * (Hq + Hkv);
  dim3 grid((unsigned)((units + kRopeRowsPerBlock - 1) / kRopeRowsPerBlock));
  hipStream_t st = (hipStream_t)stream;
#define MOA_ROPE_APPEND_LAUNCH(E)                                                                            \
  hipLaunchKernelGGL(rope_append_kernel<E>, grid, dim3(kRopeThreads), 0, st, (const char*)q_new,             \
                     (const char*)k_new, (const char*)v_new, qn_strides[0] * eb, qn_strides[1] * eb,         \
                     kn_strides[0] * eb, kn_strides[1] * eb, vn_strides[0] * eb, vn_strides[1] * eb,         \
                     (const char*)cos, (const char*)sin, cs_stride_b * eb, (char*)q_out, (char*)kc,          \
                     (char*)vc, mask_cache, update_index, valid_len, circ_head, circ_size, static_size,      \
                     max_len, kv_len, B, Hq, Hkv, D * eb, sumC)
  if (dtype == MOA_DTYPE_F16) MOA_ROPE_APPEND_LAUNCH(EF16);
  else if (dtype == MOA_DTYPE_BF16) MOA_ROPE_APPEND_LAUNCH(EBF16);
  else MOA_ROPE_APPEND_LAUNCH(EF32);
#undef MOA_ROPE_APPEND_LAUNCH
  return check_launch(who);
}
