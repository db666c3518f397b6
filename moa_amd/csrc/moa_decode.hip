// Split-K flash-decoding over per-head segments of the packed circular cache.
//
// Replaces the external decode op the reference calls at
// MoA/kernels/mixture_of_attention.py:465-473.  Every (batch row b, head h)
// attends one query row to rows [start[b,h], start[b,h]+len[b,h]) of
// kc/vc [B, sumC, D].  The work is pure HBM streaming (each K and V byte is
// used once), so the kernel is built around wide coalesced loads:
//
//   * a K/V row of D 16-bit elements is read by D/8 adjacent lanes, 16 bytes
//     each, so one wave-wide load instruction covers 1 KiB of consecutive
//     cache memory (4 rows at D=128);
//   * every wave issues kBatch K loads and kBatch V loads before it consumes
//     any of them (16 KiB in flight per wave);
//   * q.k is a lane-local dot2 chain plus a 4-step DPP sum inside the D/8
//     lanes of a row; the softmax is the usual running (max, sum) in fp32,
//     base 2, rescaled once per batch of rows;
//   * segments differ in length by ~80x between heads, so the unit of work is
//     a fixed-size chunk of rows, not a head: block (x, b) walks the chunks
//     x, x+gridDim.x, ... of batch row b, locating (head, chunk) through a
//     prefix sum over the row's heads that it rebuilds in LDS from
//     head_valid_len (no host knowledge of the lengths, no host sync);
//   * a head with one chunk writes its output directly; otherwise chunks
//     write fp32 partial (acc, max, sum) triples and a small second kernel
//     merges them;
//   * grouped-query attention (G = Hq / Hkv query heads per ring, which the
//     reference does not have): the G query rows of a ring share every K/V
//     row that a wave loads, so the cache is still read once.
#include "moa_common.h"

#include <hip/hip_fp16.h>

namespace moa {

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kDecThreads = 256;
constexpr int kDecWaves = kDecThreads / 64;
#ifndef MOA_DEC_BATCH
#define MOA_DEC_BATCH 8
#endif
constexpr int kBatch = MOA_DEC_BATCH;   // wave-wide loads in flight per tensor
constexpr int kMaxHeads = 256;     // heads per batch row the LDS prefix covers
constexpr float kLog2e = 1.4426950408889634f;

struct F16 {};
struct BF16 {};

template <typename T>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c);
template <>
__device__ __forceinline__ float dot2<F16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}
template <>
__device__ __forceinline__ float dot2<BF16>(uint32_t a, uint32_t b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c,
                                         false);
}

template <typename T>
__device__ __forceinline__ void unpack2(uint32_t x, float& lo, float& hi);
template <>
__device__ __forceinline__ void unpack2<F16>(uint32_t x, float& lo, float& hi) {
  f16x2 h = __builtin_bit_cast(f16x2, x);
  lo = (float)h.x;
  hi = (float)h.y;
}
template <>
__device__ __forceinline__ void unpack2<BF16>(uint32_t x, float& lo, float& hi) {
  lo = __builtin_bit_cast(float, x << 16);
  hi = __builtin_bit_cast(float, x & 0xffff0000u);
}

template <typename T>
__device__ __forceinline__ uint16_t pack1(float x);
template <>
__device__ __forceinline__ uint16_t pack1<F16>(float x) {
  return __builtin_bit_cast(uint16_t, (_Float16)x);
}
template <>
__device__ __forceinline__ uint16_t pack1<BF16>(float x) {
  // round to nearest even
  uint32_t u = __builtin_bit_cast(uint32_t, x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Chunk table of one batch row: prefix[h] = number of chunks of heads < h.
// Built by all threads of the block; returns the row's total chunk count.
template <int CHUNK>
__device__ __forceinline__ int build_prefix(const int64_t* __restrict__ valid_row, int H,
                                            int* __restrict__ s_prefix /* [kMaxHeads + 1] */) {
  const int tid = threadIdx.x;
  // kDecThreads >= kMaxHeads: one thread per head, Hillis-Steele scan in LDS
  int n = 0;
  if (tid < H) {
    int64_t len = valid_row[tid];
    if (len < 0) len = 0;
    n = (int)((len + CHUNK - 1) / CHUNK);
  }
  s_prefix[tid + 1] = n;
  if (tid == 0) s_prefix[0] = 0;
  __syncthreads();
  for (int off = 1; off < kMaxHeads; off <<= 1) {
    int add = (tid >= off) ? s_prefix[tid + 1 - off] : 0;
    __syncthreads();
    s_prefix[tid + 1] += add;
    __syncthreads();
  }
  return s_prefix[H];
}

// Largest h with prefix[h] <= w  (w < prefix[H]).
__device__ __forceinline__ int find_head(const int* __restrict__ s_prefix, int H, int w) {
  int lo = 0, hi = H;  // invariant: prefix[lo] <= w < prefix[hi]
  while (hi - lo > 1) {
    int mid = (lo + hi) >> 1;
    if (s_prefix[mid] <= w) lo = mid; else hi = mid;
  }
  return lo;
}

// H: kv heads (rings) per batch row; query head hk*G + g reads ring hk.
template <typename T, int D, int CHUNK, int G>
__global__ __launch_bounds__(kDecThreads) void decode_split_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    uint16_t* __restrict__ o, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const int64_t* __restrict__ head_start, const int64_t* __restrict__ head_valid, int H,
    int64_t sumC, float scale_log2, int cap /* partial slots per batch row */) {
  constexpr int LPR = D / 8;          // lanes per row
  constexpr int RPL = 64 / LPR;       // rows per wave-wide load
  constexpr int KB = (G >= 8) ? kBatch / 2 : kBatch;   // loads in flight per tensor (registers bound it at G = 8)
  constexpr int ROWS = RPL * KB;      // rows per wave per batch of loads
  constexpr int WCHUNK = CHUNK / kDecWaves;
  static_assert(WCHUNK % ROWS == 0, "chunk must split evenly over waves and load batches");

  __shared__ int s_prefix[kMaxHeads + 1];
  __shared__ float s_acc[kDecWaves][G][D];
  __shared__ float s_m[kDecWaves][G];
  __shared__ float s_l[kDecWaves][G];

  const int b = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;   // which 8-element slice of the row
  const int sub = lane / LPR;   // which row of a wave-wide load

  // Disjoint segments give at most `cap` chunks per row; the clamp keeps partial
  // slots inside the workspace if a caller hands in overlapping segments.
  const int total = min(build_prefix<CHUNK>(head_valid + (int64_t)b * H, H, s_prefix), cap);

  for (int w = blockIdx.x; w < total; w += gridDim.x) {
    const int h = find_head(s_prefix, H, w);
    const int c = w - s_prefix[h];
    const int n_chunks = s_prefix[h + 1] - s_prefix[h];
    const int64_t bh = (int64_t)b * H + h;
    const int64_t seg0 = head_start[bh];
    int64_t len = head_valid[bh];
    // clamp the segment into the row so that a bad index cannot fault
    if (seg0 < 0 || seg0 >= sumC) len = 0;
    if (len > sumC - seg0) len = sumC - seg0;
    const int64_t r_begin = (int64_t)c * CHUNK + (int64_t)wave * WCHUNK;
    int64_t r_end = r_begin + WCHUNK;
    if (r_end > len) r_end = len;

    // this lane's 8 query elements of each of the G query heads, kept packed for dot2
    u32x4 qv[G];
#pragma unroll
    for (int g = 0; g < G; ++g) qv[g] = *reinterpret_cast<const u32x4*>(q + (bh * G + g) * D + col * 8);

    const uint16_t* kbase = kc + ((int64_t)b * sumC + seg0) * D + col * 8;
    const uint16_t* vbase = vc + ((int64_t)b * sumC + seg0) * D + col * 8;

    float m[G], l[G];
    float acc[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      m[g] = -INFINITY;
      l[g] = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[g][j] = 0.f;
    }

    for (int64_t r0 = r_begin; r0 < r_end; r0 += ROWS) {
      u32x4 kr[KB], vr[KB];
#pragma unroll
      for (int i = 0; i < KB; ++i) {
        const int64_t row = r0 + i * RPL + sub;
        const bool ok = row < r_end;
        const int64_t rr = ok ? row : r_begin;  // any valid row: keeps the load in bounds
        kr[i] = *reinterpret_cast<const u32x4*>(kbase + rr * D);
        vr[i] = *reinterpret_cast<const u32x4*>(vbase + rr * D);
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float s[KB];
        float bm = -INFINITY;
#pragma unroll
        for (int i = 0; i < KB; ++i) {
          float d = 0.f;
          d = dot2<T>(qv[g].x, kr[i].x, d);
          d = dot2<T>(qv[g].y, kr[i].y, d);
          d = dot2<T>(qv[g].z, kr[i].z, d);
          d = dot2<T>(qv[g].w, kr[i].w, d);
          d = group_sum<LPR>(d) * scale_log2;
          const bool ok = (r0 + i * RPL + sub) < r_end;
          s[i] = ok ? d : -INFINITY;
          bm = fmaxf(bm, s[i]);
        }
        const float m_new = fmaxf(m[g], bm);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(m[g] - m_use);
        l[g] *= alpha;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] *= alpha;
#pragma unroll
        for (int i = 0; i < KB; ++i) {
          const float p = fast_exp2(s[i] - m_use);
          l[g] += p;
          float lo, hi;
          unpack2<T>(vr[i].x, lo, hi); acc[g][0] = fmaf(p, lo, acc[g][0]); acc[g][1] = fmaf(p, hi, acc[g][1]);
          unpack2<T>(vr[i].y, lo, hi); acc[g][2] = fmaf(p, lo, acc[g][2]); acc[g][3] = fmaf(p, hi, acc[g][3]);
          unpack2<T>(vr[i].z, lo, hi); acc[g][4] = fmaf(p, lo, acc[g][4]); acc[g][5] = fmaf(p, hi, acc[g][5]);
          unpack2<T>(vr[i].w, lo, hi); acc[g][6] = fmaf(p, lo, acc[g][6]); acc[g][7] = fmaf(p, hi, acc[g][7]);
        }
        m[g] = m_new;
      }
    }

    // ---- combine the RPL row-groups of the wave ----
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mw = m[g];
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off, 64));
      {
        const float m_use = (mw == -INFINITY) ? 0.f : mw;
        const float f = fast_exp2(m[g] - m_use);
        l[g] *= f;
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] *= f;
      }
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) {
        l[g] += __shfl_xor(l[g], off, 64);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[g][j] += __shfl_xor(acc[g][j], off, 64);
      }
      if (lane < LPR) {
#pragma unroll
        for (int j = 0; j < 8; ++j) s_acc[wave][g][lane * 8 + j] = acc[g][j];
        if (lane == 0) {
          s_m[wave][g] = mw;
          s_l[wave][g] = l[g];
        }
      }
    }
    __syncthreads();

    // ---- combine the waves; thread d owns output column d of every query head of the ring ----
    if (tid < D) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float M = s_m[0][g];
#pragma unroll
        for (int i = 1; i < kDecWaves; ++i) M = fmaxf(M, s_m[i][g]);
        const float m_use = (M == -INFINITY) ? 0.f : M;
        float L = 0.f, a = 0.f;
#pragma unroll
        for (int i = 0; i < kDecWaves; ++i) {
          const float f = fast_exp2(s_m[i][g] - m_use);
          L += s_l[i][g] * f;
          a += s_acc[i][g][tid] * f;
        }
        if (n_chunks == 1) {
          const float out = (L > 0.f) ? a / L : 0.f;
          o[(bh * G + g) * D + tid] = pack1<T>(out);
        } else {
          const int64_t slot = ((int64_t)b * cap + w) * G + g;
          part_acc[slot * D + tid] = a;
          if (tid == 0) {
            part_ml[slot * 2 + 0] = M;
            part_ml[slot * 2 + 1] = L;
          }
        }
      }
    }
    __syncthreads();  // s_acc / s_m / s_l are reused by the next chunk
  }
}

// Merge of the per-chunk partials of heads with more than one chunk, and the
// zero output of empty heads.  One block of D threads per (h, b).
template <typename T, int D, int CHUNK, int G>
__global__ __launch_bounds__(kDecThreads) void decode_merge_kernel(
    uint16_t* __restrict__ o, const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const int64_t* __restrict__ head_valid, int H, int cap) {
  __shared__ int s_prefix[kMaxHeads + 1];
  const int b = blockIdx.y;
  const int tid = threadIdx.x;
  build_prefix<CHUNK>(head_valid + (int64_t)b * H, H, s_prefix);
  // each group of D threads takes query heads t, t + groups, ... (query head hq reads ring hq / G)
  constexpr int GROUPS = kDecThreads / D;
  const int grp = tid / D;
  const int d = tid % D;
  for (int hq = blockIdx.x * GROUPS + grp; hq < H * G; hq += gridDim.x * GROUPS) {
    const int h = hq / G, g = hq % G;
    const int w0 = s_prefix[h];
    const int n = s_prefix[h + 1] - w0;
    const int64_t bhq = (int64_t)b * H * G + hq;
    if (n == 1) continue;  // written by the split kernel
    if (n == 0) {
      o[bhq * D + d] = 0;
      continue;
    }
    const int64_t slot0 = (int64_t)b * cap + w0;
    float M = -INFINITY;
    for (int i = 0; i < n; ++i) M = fmaxf(M, part_ml[((slot0 + i) * G + g) * 2]);
    const float m_use = (M == -INFINITY) ? 0.f : M;
    float L = 0.f, a = 0.f;
    for (int i = 0; i < n; ++i) {
      const int64_t slot = (slot0 + i) * G + g;
      const float f = fast_exp2(part_ml[slot * 2] - m_use);
      L += part_ml[slot * 2 + 1] * f;
      a += part_acc[slot * D + d] * f;
    }
    o[bhq * D + d] = pack1<T>((L > 0.f) ? a / L : 0.f);
  }
}

#ifndef MOA_DEC_CHUNK
#define MOA_DEC_CHUNK 512
#endif
#ifndef MOA_DEC_BLOCKS
#define MOA_DEC_BLOCKS 16
#endif
constexpr int kChunk = MOA_DEC_CHUNK;

// partial slots per batch row: at most this many chunks exist when the rings do not overlap
static inline int64_t decode_cap(int64_t sumC, int H) { return (sumC + kChunk - 1) / kChunk + H; }
// every chunk keeps one partial per query head of its ring
static inline size_t decode_slots(int B, int Hq, int Hkv, int64_t sumC) {
  return (size_t)B * (size_t)decode_cap(sumC, Hkv) * (size_t)((Hq + Hkv - 1) / Hkv);
}

template <typename T, int D, int G>
static int launch_decode(const void* q, const void* kc, const void* vc, void* o, float* part_acc,
                         float* part_ml, const int64_t* head_start, const int64_t* head_valid, int B,
                         int H, int64_t sumC, float sm_scale, hipStream_t st) {
  const int cap = (int)decode_cap(sumC, H);
  // 16 work-groups per CU over the whole grid (measured: 8 leaves a visible tail, 32 is no better),
  // never more per batch row than chunks exist
  int bx = (int)((256 * MOA_DEC_BLOCKS + B - 1) / B);
  if (bx > cap) bx = cap;
  if (bx < 1) bx = 1;
  hipLaunchKernelGGL((decode_split_kernel<T, D, kChunk, G>), dim3(bx, B), dim3(kDecThreads), 0, st,
                     (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)o,
                     part_acc, part_ml, head_start, head_valid, H, sumC, sm_scale * kLog2e, cap);
  int rc = check_launch("moa_decode_fwd(split)");
  if (rc) return rc;
  constexpr int GROUPS = kDecThreads / D;
  int mx = (H * G + GROUPS - 1) / GROUPS;
  hipLaunchKernelGGL((decode_merge_kernel<T, D, kChunk, G>), dim3(mx, B), dim3(kDecThreads), 0, st,
                     (uint16_t*)o, part_acc, part_ml, head_valid, H, cap);
  return check_launch("moa_decode_fwd(merge)");
}

}  // namespace moa

using namespace moa;

extern "C" size_t moa_decode_workspace_bytes(int B, int Hq, int Hkv, int D, int64_t sumC) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || sumC <= 0) return 0;
  const size_t slots = decode_slots(B, Hq, Hkv, sumC);
  return ((slots * ((size_t)D + 2) * sizeof(float)) + 255) & ~(size_t)255;
}

extern "C" int moa_decode_fwd(const void* q, const void* kc, const void* vc, void* o, void* workspace,
                              size_t workspace_bytes, const int64_t* head_start,
                              const int64_t* head_valid_len, int B, int Hq, int Hkv, int D, int64_t sumC,
                              float sm_scale, int dtype, void* stream) {
  if (!q || !kc || !vc || !o || !head_start || !head_valid_len)
    return fail(MOA_ERR_ARG, "moa_decode_fwd: null pointer");
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || sumC <= 0) return fail(MOA_ERR_ARG, "moa_decode_fwd: B, H, sumC must be positive");
  if (B > 65535) return fail(MOA_ERR_UNSUPPORTED, "moa_decode_fwd: B <= 65535");
  if (Hq % Hkv != 0) return fail(MOA_ERR_ARG, "moa_decode_fwd: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  const int G = Hq / Hkv;
  if (G != 1 && G != 2 && G != 4 && G != 8)
    return fail(MOA_ERR_UNSUPPORTED, "moa_decode_fwd: %d query heads per kv head (1, 2, 4 or 8)", G);
  if (Hkv > kMaxHeads) return fail(MOA_ERR_UNSUPPORTED, "moa_decode_fwd: at most %d kv heads", kMaxHeads);
  if (D != 64 && D != 128) return fail(MOA_ERR_UNSUPPORTED, "moa_decode_fwd: head_dim %d (64 or 128)", D);
  if (dtype != MOA_DTYPE_F16 && dtype != MOA_DTYPE_BF16)
    return fail(MOA_ERR_UNSUPPORTED, "moa_decode_fwd: dtype %d (f16 or bf16)", dtype);
  if (!aligned16(q) || !aligned16(kc) || !aligned16(vc) || !aligned16(o))
    return fail(MOA_ERR_ARG, "moa_decode_fwd: pointers must be 16-byte aligned");
  const size_t need = moa_decode_workspace_bytes(B, Hq, Hkv, D, sumC);
  if (!workspace || workspace_bytes < need)
    return fail(MOA_ERR_WORKSPACE, "moa_decode_fwd: workspace %zu < %zu bytes", workspace_bytes, need);
  const size_t slots = decode_slots(B, Hq, Hkv, sumC);
  float* part_acc = reinterpret_cast<float*>(workspace);
  float* part_ml = part_acc + slots * (size_t)D;
  hipStream_t st = (hipStream_t)stream;
#define MOA_DEC_ARGS q, kc, vc, o, part_acc, part_ml, head_start, head_valid_len, B, Hkv, sumC, sm_scale, st
#define MOA_DEC_G(T, DD)                                        \
  switch (G) {                                                  \
    case 1: return launch_decode<T, DD, 1>(MOA_DEC_ARGS);       \
    case 2: return launch_decode<T, DD, 2>(MOA_DEC_ARGS);       \
    case 4: return launch_decode<T, DD, 4>(MOA_DEC_ARGS);       \
    default: return launch_decode<T, DD, 8>(MOA_DEC_ARGS);      \
  }
  if (dtype == MOA_DTYPE_F16) {
    if (D == 128) { MOA_DEC_G(F16, 128) }
    MOA_DEC_G(F16, 64)
  }
  if (D == 128) { MOA_DEC_G(BF16, 128) }
  MOA_DEC_G(BF16, 64)
#undef MOA_DEC_G
#undef MOA_DEC_ARGS
}
