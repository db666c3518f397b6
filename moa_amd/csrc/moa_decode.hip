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
//     row that a wave loads, so the cache is still read once.  This kernel is
//     written for any G but instantiated for G = 1 only; G = 2, 4, 8 run on the
//     matrix cores (decode_gqa_kernel below).
#include "moa_mfma.h"

#include <hip/hip_fp16.h>

#include <mutex>

namespace moa {

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kDecThreads = 256;
constexpr int kDecWaves = kDecThreads / 64;
constexpr int kBatch = 8;           // wave-wide loads in flight per tensor
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

template <int N>
struct DecInt {
  static constexpr int value = N;
};

// Chunk table of one batch row: prefix[h] = number of chunks of heads < h, and every head's segment
// (first row, length) clamped into the row, so that a bad index cannot fault and a work-group finds a
// chunk's segment in LDS instead of behind another memory latency.
// Built by all threads of the block (one thread per head: kDecThreads >= kMaxHeads): a shuffle
// scan inside each wave, then the wave totals through LDS.  Returns the row's total chunk count.
// Every entry is clamped to `cap`, the partial slots a batch row owns: with disjoint segments the clamp
// never acts; with overlapping ones (lengths that sum to more than the row holds) the chunks past the cap
// do not exist for any kernel that builds the table, so none of them is written, read or merged.
struct HeadTable {
  int prefix[kMaxHeads + 1];
  int seg0[kMaxHeads];   // first cache row of the head's segment (rows per batch row fit 31 bits: checked on the host)
  int len[kMaxHeads];    // valid rows, clamped to the end of the batch row
  int clen[kMaxHeads];   // rows per chunk of this head
};

template <int CHUNK, int NWAVES = kDecWaves>
__device__ __forceinline__ int build_prefix(const int64_t* __restrict__ valid_row, const int64_t* __restrict__ start_row,
                                            int H, int64_t sumC, int cap, HeadTable* __restrict__ tab) {
  __shared__ int s_wave_total[NWAVES];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  int n = 0;
  if (tid < H) {
    int64_t len = valid_row[tid];
    const int64_t seg0 = start_row[tid];
    if (len < 0 || seg0 < 0 || seg0 >= sumC) len = 0;
    if (len > sumC - seg0) len = sumC - seg0;
    tab->seg0[tid] = (int)(len > 0 ? seg0 : 0);
    tab->len[tid] = (int)len;
    tab->clen[tid] = CHUNK;
    n = (int)((len + CHUNK - 1) / CHUNK);
  }
  int incl = n;   // inclusive scan inside the wave
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) s_wave_total[wave] = incl;
  __syncthreads();
  int base = 0;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) base += (w < wave) ? s_wave_total[w] : 0;
  if (tid < kMaxHeads) tab->prefix[tid + 1] = min(base + incl, cap);
  if (tid == 0) tab->prefix[0] = 0;
  __syncthreads();
  return tab->prefix[H];
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

// The same table with chunks of about equal length over the whole batch row instead of a fixed chunk
// length.  With a fixed length the last chunk of every head is a remainder and the number of chunks is
// whatever it comes to; here the caller names the number of chunks (`target`) a batch row should not
// exceed, and the table takes the shortest chunk length c (whole steps of kEvenStep rows, at least
// kEvenMinChunk) for which sum_h ceil(len_h / c) <= target; head h is then split evenly into
// ceil(len_h / c) chunks.  The search starts at total / target and goes up step by step (the sum exceeds
// the target by at most the number of heads at the start, so a few steps do), and gives up after
// kEvenTries: the table is valid for any c, the target is a wish.  Integer arithmetic only: the split
// and the merge kernel build this table independently and must agree on every entry.
constexpr int kEvenMinChunk = 256;   // also the chunk length the partial slots of a batch row are sized for
constexpr int kEvenStep = 128;
constexpr int kEvenTries = 24;
template <int NWAVES>
__device__ __forceinline__ int build_prefix_even(const int64_t* __restrict__ valid_row, const int64_t* __restrict__ start_row,
                                                 int H, int64_t sumC, int cap, int target, HeadTable* __restrict__ tab) {
  __shared__ int s_wave_total[NWAVES];
  __shared__ int s_wave_sum[2][NWAVES];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  int len = 0;
  if (tid < H) {
    int64_t l = valid_row[tid];
    const int64_t seg0 = start_row[tid];
    if (l < 0 || seg0 < 0 || seg0 >= sumC) l = 0;
    if (l > sumC - seg0) l = sumC - seg0;
    tab->seg0[tid] = (int)(l > 0 ? seg0 : 0);
    tab->len[tid] = (int)l;
    len = (int)l;
  }
  // sum over the work-group of a per-thread count (every thread gets the sum); `buf` alternates so that
  // one barrier per call is enough
  auto block_sum = [&](int x, int buf) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    if (lane == 0) s_wave_sum[buf][wave] = x;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) t += s_wave_sum[buf][w];
    return t;
  };
  // rows of the batch row in steps (a sum of at most 256 heads of < 2^31 rows each fits 32 bits in steps)
  const int total_steps = block_sum((len + kEvenStep - 1) / kEvenStep, 0);
  int c = max(kEvenMinChunk, ((total_steps + target - 1) / max(target, 1)) * kEvenStep);
  int n = 0;
  for (int i = 0; i < kEvenTries; ++i) {
    n = (len + c - 1) / c;
    if (block_sum(n, (i + 1) & 1) <= target) break;   // the same for every thread
    c += kEvenStep;
    n = (len + c - 1) / c;   // what the table holds if this was the last try
  }
  int clen = kEvenStep;
  if (n > 0) {
    clen = (((len + n - 1) / n + kEvenStep - 1) / kEvenStep) * kEvenStep;   // even split, <= c
    n = (len + clen - 1) / clen;
  }
  if (tid < kMaxHeads) tab->clen[tid] = clen;
  int incl = n;   // inclusive scan inside the wave
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const int up = __shfl_up(incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) s_wave_total[wave] = incl;
  __syncthreads();
  int base = 0;
#pragma unroll
  for (int w = 0; w < NWAVES; ++w) base += (w < wave) ? s_wave_total[w] : 0;
  if (tid < kMaxHeads) tab->prefix[tid + 1] = min(base + incl, cap);
  if (tid == 0) tab->prefix[0] = 0;
  __syncthreads();
  return tab->prefix[H];
}

// H: kv heads (rings) per batch row; query head hk*G + g reads ring hk.
// PIPE: the wave keeps two half-batches of loads going (the next one is issued before the current
// one is consumed) instead of loading a full batch, waiting for it and consuming it.  Measured at
// the 7B decode shape: 8 % faster at batch 4, 2 % at 8-16, 0.7 % at 64; at batch 1-2 (about one
// work-group per CU, the call is launch-latency bound) the plain loop is 2-4 % faster.
template <typename T, int D, int CHUNK, int G, bool PIPE>
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

  __shared__ HeadTable s_tab;
  const int* const s_prefix = s_tab.prefix;
  __shared__ float s_acc[kDecWaves][G][D];
  __shared__ float s_m[kDecWaves][G];
  __shared__ float s_l[kDecWaves][G];

  const int b = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane % LPR;   // which 8-element slice of the row
  const int sub = lane / LPR;   // which row of a wave-wide load

  // Disjoint segments give at most `cap` chunks per row; the clamp inside keeps partial
  // slots inside the workspace if a caller hands in overlapping segments.
  const int total = build_prefix<CHUNK>(head_valid + (int64_t)b * H, head_start + (int64_t)b * H, H, sumC, cap, &s_tab);

  for (int w = blockIdx.x; w < total; w += gridDim.x) {
    const int h = find_head(s_prefix, H, w);
    const int c = w - s_prefix[h];
    const int n_chunks = s_prefix[h + 1] - s_prefix[h];
    const int64_t bh = (int64_t)b * H + h;
    const int64_t seg0 = s_tab.seg0[h];
    const int64_t len = s_tab.len[h];
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

    // n wave-wide loads of K and of V starting at row r0 of the wave's share
    auto load_rows = [&](auto N, u32x4* kr, u32x4* vr, int64_t r0) __attribute__((always_inline)) {
      constexpr int n = decltype(N)::value;
#pragma unroll
      for (int i = 0; i < n; ++i) {
        const int64_t row = r0 + i * RPL + sub;
        const bool ok = row < r_end;
        const int64_t rr = ok ? row : r_begin;  // any valid row: keeps the load in bounds
        kr[i] = *reinterpret_cast<const u32x4*>(kbase + rr * D);
        vr[i] = *reinterpret_cast<const u32x4*>(vbase + rr * D);
      }
    };
    // online-softmax update with those rows
    auto consume_rows = [&](auto N, const u32x4* kr, const u32x4* vr, int64_t r0) __attribute__((always_inline)) {
      constexpr int n = decltype(N)::value;
#pragma unroll
      for (int g = 0; g < G; ++g) {
        float s[n];
        float bm = -INFINITY;
#pragma unroll
        for (int i = 0; i < n; ++i) {
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
        for (int i = 0; i < n; ++i) {
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
    };
    if (!PIPE) {
      for (int64_t r0 = r_begin; r0 < r_end; r0 += ROWS) {
        u32x4 kr[KB], vr[KB];
        load_rows(DecInt<KB>{}, kr, vr, r0);
        consume_rows(DecInt<KB>{}, kr, vr, r0);
      }
    } else {
      constexpr int KH = KB / 2, HROWS = ROWS / 2;
      u32x4 ka[KH], va[KH], kb2[KH], vb2[KH];
      if (r_begin < r_end) load_rows(DecInt<KH>{}, ka, va, r_begin);
      for (int64_t r0 = r_begin; r0 < r_end; r0 += ROWS) {
        const bool second = r0 + HROWS < r_end;
        if (second) load_rows(DecInt<KH>{}, kb2, vb2, r0 + HROWS);
        consume_rows(DecInt<KH>{}, ka, va, r0);
        if (second) {
          if (r0 + ROWS < r_end) load_rows(DecInt<KH>{}, ka, va, r0 + ROWS);
          consume_rows(DecInt<KH>{}, kb2, vb2, r0 + HROWS);
        }
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
// zero output of empty heads.  A group of D threads takes one query head at a time: its lanes load
// the (max, sum) pairs of the chunks side by side, the factors go through LDS, then thread d sums
// column d of the partial accumulators with several loads in flight.
template <typename T, int D, int CHUNK>
__global__ __launch_bounds__(kDecThreads) void decode_merge_kernel(
    uint16_t* __restrict__ o, const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const int64_t* __restrict__ head_start, const int64_t* __restrict__ head_valid, int H,
    int G /* query heads per ring */, int64_t sumC, int cap,
    int even_target /* > 0: the split kernel used build_prefix_even with this target */) {
  constexpr int GROUPS = kDecThreads / D;
  constexpr int kFactors = 64;   // chunks whose factors are staged at a time
  __shared__ HeadTable s_tab;
  const int* const s_prefix = s_tab.prefix;
  __shared__ float s_f[GROUPS][kFactors];
  __shared__ int s_n[GROUPS];
  const int b = blockIdx.y;
  const int tid = threadIdx.x;
  if (even_target > 0)
    build_prefix_even<kDecWaves>(head_valid + (int64_t)b * H, head_start + (int64_t)b * H, H, sumC, cap, even_target, &s_tab);
  else
    build_prefix<CHUNK>(head_valid + (int64_t)b * H, head_start + (int64_t)b * H, H, sumC, cap, &s_tab);
  const int grp = tid / D;
  const int d = tid % D;
  // every group runs the same number of rounds so that the barriers below are uniform
  const int rounds = (H * G + gridDim.x * GROUPS - 1) / (gridDim.x * GROUPS);
  for (int r = 0; r < rounds; ++r) {
    const int hq = (r * gridDim.x + blockIdx.x) * GROUPS + grp;
    const bool on = hq < H * G;
    const int h = on ? hq / G : 0, g = on ? hq % G : 0;
    const int w0 = s_prefix[h];
    const int n = on ? s_prefix[h + 1] - w0 : 1;
    const int64_t bhq = (int64_t)b * H * G + hq;
    const int64_t slot0 = (int64_t)b * cap + w0;
    if (on && n == 0) o[bhq * D + d] = 0;
    // n == 1: written by the split kernel
    float M = -INFINITY;
    if (n > 1)
      for (int i = d; i < n; i += D) M = fmaxf(M, part_ml[((slot0 + i) * G + g) * 2]);
    // max over the group's lanes (D = 64: one wave; D = 128: two waves, through LDS)
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
    if (D > 64) {
      if ((tid & 63) == 0) s_f[grp][(d >> 6)] = M;
      __syncthreads();
      M = fmaxf(s_f[grp][0], s_f[grp][1]);
      __syncthreads();
    }
    const float m_use = (M == -INFINITY) ? 0.f : M;
    float L = 0.f, a = 0.f;
    // the groups of a block walk their chunks in lockstep (work-group barriers inside): as many
    // rounds as the longest of them needs
    const int n_eff = (n > 1) ? n : 0;
    if (d == 0) s_n[grp] = n_eff;
    __syncthreads();
    int n_loop = 0;
#pragma unroll
    for (int k = 0; k < GROUPS; ++k) n_loop = max(n_loop, s_n[k]);
    for (int i0 = 0; i0 < n_loop; i0 += kFactors) {
      const int cnt = max(0, min(kFactors, n_eff - i0));
      if (d < cnt) {
        const int64_t slot = (slot0 + i0 + d) * G + g;
        const float f = fast_exp2(part_ml[slot * 2] - m_use);
        s_f[grp][d] = f;
        L += part_ml[slot * 2 + 1] * f;
      }
      __syncthreads();
      const float* acc = part_acc + ((slot0 + i0) * G + g) * D + d;
      int i = 0;
      for (; i + 4 <= cnt; i += 4) {
        const float x0 = acc[(int64_t)(i + 0) * G * D], x1 = acc[(int64_t)(i + 1) * G * D];
        const float x2 = acc[(int64_t)(i + 2) * G * D], x3 = acc[(int64_t)(i + 3) * G * D];
        a += x0 * s_f[grp][i] + x1 * s_f[grp][i + 1] + x2 * s_f[grp][i + 2] + x3 * s_f[grp][i + 3];
      }
      for (; i < cnt; ++i) a += acc[(int64_t)i * G * D] * s_f[grp][i];
      __syncthreads();
    }
    // the sum of the group's partial L values
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) L += __shfl_xor(L, off, 64);
    if (D > 64) {
      if ((tid & 63) == 0) s_f[grp][(d >> 6)] = L;
      __syncthreads();
      L = s_f[grp][0] + s_f[grp][1];
      __syncthreads();
    }
    if (on && n > 1) o[bhq * D + d] = pack1<T>((L > 0.f) ? a / L : 0.f);
    __syncthreads();   // s_n and s_f are written again in the next round
  }
}

// ---- grouped-query decode on the matrix cores (G >= 2) ---------------------------------------
// With G query heads per ring the vector ALU version above does G times the arithmetic per cache
// byte and stops being HBM bound (measured: 65 % of peak at G = 2, 46 % at G = 8).  Here the G query rows of a ring are the
// columns of a 32-wide MFMA tile (columns >= G are zero padding; the matrix pipe has the room):
//   S^T[key][q] = sum_d K[key][d] Q[q][d]      A = K (LDS), B = Q^T (registers)
//   O^T[d][q]   = sum_key V[key][d] P[q][key]   A = V^T (LDS, transposing read), B = P^T
// the same transposed pair of products as the prefill kernel, 32 keys at a time, so the softmax
// state of a query head is lane-local.  Each wave streams its own share of the chunk through a
// private two-stage LDS ring with asynchronous copies (16-byte chunks XOR-permuted as in the
// prefill kernel), so no work-group barrier is needed inside the loop.  Chunks, partials and the
// merge kernel are those of the vector version, with a longer chunk.
// Work-groups per CU the grid may hold.  A CU runs one at a time (the LDS rings fill it), so the hardware
// dispatcher hands out chunks as CUs become free when every chunk is a work-group of its own: 602 us at
// batch 64 of the 70B shape against 612-628 us with 2-16 per CU, each walking several chunks in a fixed order.
constexpr int kGqaBlocksPerCu = 64;
// Largest number of cache rows per work-group step (a quarter per wave) the launch aims for; the actual
// chunk lengths come out of an even split of every batch row (build_prefix_even).  A chunk start costs a
// wave full memory latencies with nothing in flight, so long chunks win: with one fixed length, 2048 was
// the best of 512..4096 at batch 64 and at batch 4.
constexpr int kGqaChunk = 2048;
constexpr int kGqaTile = 32;      // keys per MFMA tile
constexpr int kGqaMaxG = 8;       // query heads per ring the per-wave result buffers are sized for
constexpr int kGqaWaves = 4;      // waves per work-group (8 waves with one stage each measure the same)
constexpr int kGqaThreads = 64 * kGqaWaves;
constexpr int kGqaStages = 2;     // LDS stages per wave (8 stages of 16 KiB at D = 128 in all)

template <typename T> struct MfmaElem;
template <> struct MfmaElem<F16> { typedef PF16 type; };
template <> struct MfmaElem<BF16> { typedef PBF16 type; };

template <int D>
constexpr size_t gqa_lds_bytes() { return (size_t)kGqaWaves * kGqaStages * 2 * kGqaTile * D * 2; }

template <typename T, int D>
__global__ __launch_bounds__(kGqaThreads) void decode_gqa_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
    uint16_t* __restrict__ o, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const int64_t* __restrict__ head_start, const int64_t* __restrict__ head_valid, int H,
    int G /* query heads per ring, <= kGqaMaxG */, int64_t sumC, float scale_log2_signed, int cap,
    int target /* > 0: chunks a batch row is split into (build_prefix_even); 0: chunks of kGqaChunk rows */) {
  typedef typename MfmaElem<T>::type M;
  // the row maximum is taken over unscaled scores: a negative softmax scale goes into Q (sign flip, exact)
  const float scale_log2 = __builtin_fabsf(scale_log2_signed);
  const uint32_t q_sign = scale_log2_signed < 0.f ? 0x80008000u : 0u;
  constexpr int KS = D / 16;                    // MFMA k-steps of Q.K^T
  constexpr int DT = D / 32;                    // 32-wide d tiles of the output
  constexpr int CPR = D / 8;                    // 16-byte chunks per cache row
  constexpr int ROW_B = D * 2;
  constexpr int RSH = 16 / CPR;                 // rows per 256 bytes of LDS
  constexpr int TILE_B = kGqaTile * ROW_B;      // bytes of one K or V tile
  constexpr int NCP = TILE_B / 1024;            // async copies per tile and tensor
  constexpr int STAGE_B = 2 * TILE_B;           // K tile, then V tile
  constexpr float kRescaleStep = 8.f;
  static_assert((kEvenStep / kGqaWaves) % kGqaTile == 0, "a wave's share of a chunk is whole tiles");

  extern __shared__ __attribute__((aligned(1024))) char s_mem[];
  __shared__ HeadTable s_tab;
  const int* const s_prefix = s_tab.prefix;
  // the per-wave results (m, l, O[d] per query head) go into the first 4.5 KiB of the wave's own ring
  // once its loop is over
  __shared__ float s_m[kGqaWaves][kGqaMaxG];
  __shared__ float s_l[kGqaWaves][kGqaMaxG];
  static_assert(kGqaMaxG * D * 4 <= kGqaStages * STAGE_B, "the result buffer fits the wave's ring");

  const int b = blockIdx.y;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mcol = lane & 31;   // query head inside the ring (the MFMA column); >= G: padding
  const int g = lane >> 5;      // half-wave
  const uint32_t ring0 = lds_address(s_mem) + wave * (kGqaStages * STAGE_B);   // this wave's stages

  // copy i of a tile moves chunks [64 i, 64 i + 64): chunk c = row * CPR + position
  uint32_t koff[NCP], voff[NCP];
  int crow[NCP];
#pragma unroll
  for (int i = 0; i < NCP; ++i) {
    const int L = i * 64 + lane;
    const int row = L / CPR, pos = L % CPR;
    crow[i] = row;
    koff[i] = (uint32_t)(row * ROW_B + (pos ^ ((row / RSH) % CPR)) * 16);
    voff[i] = (uint32_t)(row * ROW_B + (pos ^ (4 * ((row / RSH) % (CPR / 4)))) * 16);
  }
  // operand read addresses inside stage 0 (see the prefill kernel for the layout)
  uint32_t k_ad[KS], v_ad[DT];
  {
    const uint32_t k_rd = (uint32_t)(mcol * ROW_B) | (uint32_t)(((g ^ ((mcol / RSH) % CPR)) & (CPR - 1)) * 16);
#pragma unroll
    for (int s = 0; s < KS; ++s) k_ad[s] = ring0 + (k_rd ^ (uint32_t)(32 * s));
    const int grp16 = lane & 15, dhalf = (lane >> 4) & 1, v_row = 4 * g + (grp16 >> 2);
    const uint32_t v_rd = (uint32_t)(v_row * ROW_B) +
                          (uint32_t)(((2 * dhalf + ((grp16 & 3) >> 1)) ^ (4 * ((v_row / RSH) % (CPR / 4)))) * 16 +
                                     8 * (grp16 & 1));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) v_ad[dt] = ring0 + TILE_B + (v_rd ^ (uint32_t)(64 * dt));
  }

  const int total = target > 0
      ? build_prefix_even<kGqaWaves>(head_valid + (int64_t)b * H, head_start + (int64_t)b * H, H, sumC, cap, target, &s_tab)
      : build_prefix<kGqaChunk, kGqaWaves>(head_valid + (int64_t)b * H, head_start + (int64_t)b * H, H, sumC, cap, &s_tab);

  for (int w = blockIdx.x; w < total; w += gridDim.x) {
    const int h = find_head(s_prefix, H, w);
    const int c = w - s_prefix[h];
    const int n_chunks = s_prefix[h + 1] - s_prefix[h];
    const int64_t bh = (int64_t)b * H + h;
    const int64_t seg0 = s_tab.seg0[h];
    const int64_t len = s_tab.len[h];
    const int clen = s_tab.clen[h];            // rows of one chunk of this head
    const int wchunk = clen / kGqaWaves;       // a wave's share: whole tiles
    const int64_t r_begin = (int64_t)c * clen + (int64_t)wave * wchunk;
    int64_t r_end = r_begin + wchunk;
    if (r_end > len) r_end = len;
    const int n_rows = __builtin_amdgcn_readfirstlane(r_end > r_begin ? (int)(r_end - r_begin) : 0);
    const int n_t = (n_rows + kGqaTile - 1) / kGqaTile;
    const char* kbase = reinterpret_cast<const char*>(kc + ((int64_t)b * sumC + seg0 + r_begin) * D);
    const char* vbase = reinterpret_cast<const char*>(vc + ((int64_t)b * sumC + seg0 + r_begin) * D);

    // Q^T fragments: column mcol = query head, k-step s holds Q[mcol][16 s + 8 g .. +7]
    u32x4 qf[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      u32x4 z = {0, 0, 0, 0};
      qf[s] = (mcol < G) ? *reinterpret_cast<const u32x4*>(q + (bh * G + mcol) * D + 16 * s + 8 * g) : z;
      qf[s] ^= u32x4{q_sign, q_sign, q_sign, q_sign};
    }
    f32x16 oacc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[dt][i] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // tile t: rows [32 t, 32 t + 32) of the wave's share, into stage t % kGqaStages; rows past the
    // end repeat the last row (their scores are masked)
    auto issue = [&](int t) __attribute__((always_inline)) {
      const char* ksrc = kbase + (int64_t)t * TILE_B;
      const char* vsrc = vbase + (int64_t)t * TILE_B;
      const uint32_t dst = ring0 + (t % kGqaStages) * STAGE_B;
      const int last = n_rows - 1 - t * kGqaTile;   // last valid row of the tile, >= 0
      if (last >= kGqaTile - 1) {
#pragma unroll
        for (int i = 0; i < NCP; ++i) async_copy16(ksrc, koff[i], dst + i * 1024);
#pragma unroll
        for (int i = 0; i < NCP; ++i) async_copy16(vsrc, voff[i], dst + TILE_B + i * 1024);
      } else {
#pragma unroll
        for (int i = 0; i < NCP; ++i)
          async_copy16(ksrc, koff[i] - (uint32_t)(max(crow[i] - last, 0) * ROW_B), dst + i * 1024);
#pragma unroll
        for (int i = 0; i < NCP; ++i)
          async_copy16(vsrc, voff[i] - (uint32_t)(max(crow[i] - last, 0) * ROW_B), dst + TILE_B + i * 1024);
      }
    };
    if (n_t > 0) issue(0);
    if (kGqaStages > 1 && n_t > 1) issue(1);
    // the Q loads are older than every copy: pin their arrival here
    if (kGqaStages > 1 && n_t > 1) wait_vm(4 * NCP); else if (n_t > 0) wait_vm(2 * NCP);
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));

    for (int t = 0; t < n_t; ++t) {
      if (kGqaStages > 1 && t + 1 < n_t) wait_vm(2 * NCP); else wait_vm(0);   // tile t has landed; tile t+1 may be in flight
      const uint32_t so = (uint32_t)((t % kGqaStages) * STAGE_B);
      // ---- S^T = K . Q^T ----
      f32x16 st;
      {
        u32x4 kf[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) kf[s] = lds_load16(k_ad[s] + so, 0);
        f32x16 z;
#pragma unroll
        for (int i = 0; i < 16; ++i) z[i] = 0.f;
        st = M::mfma(kf[0], qf[0], z);
#pragma unroll
        for (int s = 1; s < KS; ++s) st = M::mfma(kf[s], qf[s], st);
      }
      // ---- softmax over the 32 keys (element i of a lane: key 8 (i / 4) + 4 g + i % 4) ----
      const int n_valid = n_rows - t * kGqaTile;
      if (n_valid < kGqaTile) {
        int thr = n_valid - 4 * g;
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (8 * (i >> 2) + (i & 3) >= thr) st[i] = -INFINITY;
      }
      float mx = st[0];
#pragma unroll
      for (int i = 1; i < 16; ++i) mx = fmaxf(mx, st[i]);
      mx = max_with_other_half(mx);
      const float m_cand = mx * scale_log2;   // finite: key 0 of the tile is valid
      if (__any(m_cand > m_run + kRescaleStep)) {
        // an integer reference exponent: the rounding of the weights below is then independent of it
        const float m_new = __builtin_ceilf(fmaxf(m_run, m_cand));
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[dt][i] *= alpha;
        m_run = m_new;
      }
      uint32_t pf[8];
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[i], scale_log2, -m_run));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[i + 1], scale_log2, -m_run));
        pf[i >> 1] = M::pack_rne(p0, p1);
        psum += p0 + p1;
      }
      l_run += psum;
      // ---- O^T += V^T . P^T ----
#pragma unroll
      for (int tk = 0; tk < 2; ++tk) {
        const u32x4 bfrag = {pf[4 * tk], pf[4 * tk + 1], pf[4 * tk + 2], pf[4 * tk + 3]};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const u32x2 lo = lds_load_tr16(v_ad[dt] + so, (16 * tk) * ROW_B);
          const u32x2 hi = lds_load_tr16(v_ad[dt] + so, (16 * tk + 8) * ROW_B);
          oacc[dt] = M::mfma(u32x4{lo.x, lo.y, hi.x, hi.y}, bfrag, oacc[dt]);
        }
      }
      if (t + kGqaStages < n_t) issue(t + kGqaStages);   // every read of this stage has returned
    }

    // ---- the wave's result per query head: (m, l, O[d]) ----
    {
      const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
      float* s_acc_w = reinterpret_cast<float*>(s_mem + wave * (kGqaStages * STAGE_B));
      if (mcol < G) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int i = 0; i < 16; ++i) s_acc_w[mcol * D + 32 * dt + 8 * (i >> 2) + 4 * g + (i & 3)] = oacc[dt][i];
        if (g == 0) {
          s_m[wave][mcol] = m_run;
          s_l[wave][mcol] = l_tot;
        }
      }
    }
    __syncthreads();

    // ---- combine the waves; thread d owns output column d of every query head of the ring ----
    if (tid < D) {
      for (int gq = 0; gq < G; ++gq) {
        float Mx = s_m[0][gq];
#pragma unroll
        for (int i = 1; i < kGqaWaves; ++i) Mx = fmaxf(Mx, s_m[i][gq]);
        const float m_use = (Mx == -INFINITY) ? 0.f : Mx;
        float L = 0.f, a = 0.f;
#pragma unroll
        for (int i = 0; i < kGqaWaves; ++i) {
          const float f = fast_exp2(s_m[i][gq] - m_use);
          L += s_l[i][gq] * f;
          a += reinterpret_cast<const float*>(s_mem + i * (kGqaStages * STAGE_B))[gq * D + tid] * f;
        }
        if (n_chunks == 1) {
          o[(bh * G + gq) * D + tid] = pack1<T>((L > 0.f) ? a / L : 0.f);
        } else {
          const int64_t slot = ((int64_t)b * cap + w) * G + gq;
          part_acc[slot * D + tid] = a;
          if (tid == 0) {
            part_ml[slot * 2 + 0] = Mx;
            part_ml[slot * 2 + 1] = L;
          }
        }
      }
    }
    __syncthreads();  // s_acc / s_m / s_l are reused by the next chunk
  }
}

constexpr int kChunk = 512;           // cache rows per work-group step of the one-query-head kernel
constexpr int kDecBlocksPerCu = 16;   // work-groups per CU over the whole grid
constexpr int kDecSmallBelow = 2;     // work-groups per CU below which the chunks are half as long
constexpr int kDecPipeFrom = 3;       // work-groups per CU from which the waves pipeline their own loads

constexpr int kSmallChunk = kChunk / 2;   // chunk length of the one-query-head kernel when the grid is small

// partial slots per batch row: at most this many chunks exist when the rings do not overlap (sized
// for the shortest chunk any of the kernels uses)
static inline int64_t decode_cap(int64_t sumC, int H) { return (sumC + kSmallChunk - 1) / kSmallChunk + H; }
// every chunk keeps one partial per query head of its ring
static inline size_t decode_slots(int B, int Hq, int Hkv, int64_t sumC) {
  return (size_t)B * (size_t)decode_cap(sumC, Hkv) * (size_t)((Hq + Hkv - 1) / Hkv);
}

template <typename T, int D, int G>
static int launch_decode(const void* q, const void* kc, const void* vc, void* o, float* part_acc,
                         float* part_ml, const int64_t* head_start, const int64_t* head_valid, int B,
                         int H, int64_t sumC, float sm_scale, hipStream_t st) {
  const int cap = (int)decode_cap(sumC, H);
  const int64_t chunks = (sumC + kChunk - 1) / kChunk + H;   // per batch row, at the normal chunk length
  // 16 work-groups per CU over the whole grid (measured: 8 leaves a visible tail, 32 is no better),
  // never more per batch row than chunks exist
  int bx = (int)((256 * kDecBlocksPerCu + B - 1) / B);
  if (bx > cap) bx = cap;
  if (bx < 1) bx = 1;
  const bool pipe = (int64_t)B * chunks >= (int64_t)256 * kDecPipeFrom;
  // fewer than two work-groups per CU: half-length chunks give every CU something to do
  const bool small = (int64_t)B * chunks < (int64_t)256 * kDecSmallBelow;
  constexpr int GROUPS = kDecThreads / D;
  const int mx = (H * G + GROUPS - 1) / GROUPS;
  if (small) {
    hipLaunchKernelGGL((decode_split_kernel<T, D, kSmallChunk, G, false>), dim3(bx, B), dim3(kDecThreads), 0, st,
                       (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)o,
                       part_acc, part_ml, head_start, head_valid, H, sumC, sm_scale * kLog2e, cap);
    int rc = check_launch("moa_decode_fwd(split)");
    if (rc) return rc;
    hipLaunchKernelGGL((decode_merge_kernel<T, D, kSmallChunk>), dim3(mx, B), dim3(kDecThreads), 0, st,
                       (uint16_t*)o, part_acc, part_ml, head_start, head_valid, H, G, sumC, cap, 0);
    return check_launch("moa_decode_fwd(merge)");
  }
  if (pipe)
    hipLaunchKernelGGL((decode_split_kernel<T, D, kChunk, G, true>), dim3(bx, B), dim3(kDecThreads), 0, st,
                       (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)o,
                       part_acc, part_ml, head_start, head_valid, H, sumC, sm_scale * kLog2e, cap);
  else
    hipLaunchKernelGGL((decode_split_kernel<T, D, kChunk, G, false>), dim3(bx, B), dim3(kDecThreads), 0, st,
                       (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)o,
                       part_acc, part_ml, head_start, head_valid, H, sumC, sm_scale * kLog2e, cap);
  int rc = check_launch("moa_decode_fwd(split)");
  if (rc) return rc;
  hipLaunchKernelGGL((decode_merge_kernel<T, D, kChunk>), dim3(mx, B), dim3(kDecThreads), 0, st,
                     (uint16_t*)o, part_acc, part_ml, head_start, head_valid, H, G, sumC, cap, 0);
  return check_launch("moa_decode_fwd(merge)");
}


template <typename T, int D>
static int launch_decode_gqa(const void* q, const void* kc, const void* vc, void* o, float* part_acc,
                             float* part_ml, const int64_t* head_start, const int64_t* head_valid, int B,
                             int H, int G, int64_t sumC, float sm_scale, hipStream_t st) {
  const int cap = (int)decode_cap(sumC, H);   // partial slots per batch row the workspace was sized for
  // Chunk policy.  Chunks of kGqaChunk rows when they give at least half of the CUs a chunk: measured at
  // the 70B shape (8 rings per batch row, 104 k rows) with one fixed length, 49.8 us per call at batch 4
  // with 2048-row chunks, 53.3 with 1024, 62.3 with 512 -- a chunk start costs three dependent memory
  // latencies (ring index, query rows, first tiles).  Below that (batch 1 and 2 at that shape: 54 and 108
  // chunks) every batch row is split evenly into its share of 256 chunks instead: 25.8 against 32.4 us at
  // batch 1, 33.5 against 36-39 us at batch 2.  From batch 3 on the even split gains nothing (one round of
  // 256 chunks of 1664 rows at batch 4: 50.6-52.2 us against 50.4-51.8 us with 213 chunks of 2048; whole
  // rounds of even chunks at batch 6 to 64: between 4 % faster and 7 % slower): those launches stream at
  // the rate of the large batches already.  The host does not know how full the rings are; it plans with
  // their capacity.
  const int64_t fixed_chunks = (int64_t)B * (sumC / kGqaChunk + (H + 1) / 2);
  int64_t target = 0;   // 0: chunks of kGqaChunk rows
  if (fixed_chunks <= 128) {
    target = (256 + B - 1) / B;
    if (target > cap) target = cap;
  }
  // at most this many chunks per batch row (a work-group without a chunk still holds a CU while it finds that out)
  const int64_t chunks = target > 0 ? target + H : (sumC + kGqaChunk - 1) / kGqaChunk + H;
  int64_t bx = (256 * kGqaBlocksPerCu + B - 1) / B;   // in practice one work-group per chunk (see kGqaBlocksPerCu)
  if (bx > chunks) bx = chunks;
  if (bx > cap) bx = cap;
  if (bx < 1) bx = 1;
  constexpr size_t lds = gqa_lds_bytes<D>();
  static bool lds_reserved[kMaxDevices] = {};   // per template instance
  if (int rc = reserve_lds(reinterpret_cast<const void*>(&decode_gqa_kernel<T, D>), lds, lds_reserved, "moa_decode_fwd"))
    return rc;
  hipLaunchKernelGGL((decode_gqa_kernel<T, D>), dim3((unsigned)bx, B), dim3(kGqaThreads), lds, st,
                     (const uint16_t*)q, (const uint16_t*)kc, (const uint16_t*)vc, (uint16_t*)o,
                     part_acc, part_ml, head_start, head_valid, H, G, sumC, mfma_softmax_scale(sm_scale), cap,
                     (int)target);
  int rc = check_launch("moa_decode_fwd(grouped split)");
  if (rc) return rc;
  constexpr int GROUPS = kDecThreads / D;
  int mx = (H * G + GROUPS - 1) / GROUPS;
  hipLaunchKernelGGL((decode_merge_kernel<T, D, kGqaChunk>), dim3(mx, B), dim3(kDecThreads), 0, st,
                     (uint16_t*)o, part_acc, part_ml, head_start, head_valid, H, G, sumC, cap, (int)target);
  return check_launch("moa_decode_fwd(merge)");
}

// Launches the decode kernels with their partials in `workspace` (at least
// moa_decode_workspace_bytes(...) bytes; arguments and size are checked by the entry points).
static int decode_dispatch(const void* q, const void* kc, const void* vc, void* o,
                           void* workspace, const int64_t* head_start, const int64_t* head_valid_len,
                           int B, int Hq, int Hkv, int D, int64_t sumC, float sm_scale, int dtype,
                           void* stream) {
  const int G = Hq / Hkv;
  const size_t slots = decode_slots(B, Hq, Hkv, sumC);
  float* part_acc = reinterpret_cast<float*>(workspace);
  float* part_ml = part_acc + slots * (size_t)D;
  hipStream_t st = (hipStream_t)stream;
#define MOA_DEC_ARGS q, kc, vc, o, part_acc, part_ml, head_start, head_valid_len, B, Hkv
#define MOA_DEC_TAIL sumC, sm_scale, st
  // one query head per ring: vector ALU kernel; more: matrix-core kernel
  if (dtype == MOA_DTYPE_F16) {
    if (D == 128) return G == 1 ? launch_decode<F16, 128, 1>(MOA_DEC_ARGS, MOA_DEC_TAIL) : launch_decode_gqa<F16, 128>(MOA_DEC_ARGS, G, MOA_DEC_TAIL);
    return G == 1 ? launch_decode<F16, 64, 1>(MOA_DEC_ARGS, MOA_DEC_TAIL) : launch_decode_gqa<F16, 64>(MOA_DEC_ARGS, G, MOA_DEC_TAIL);
  }
  if (D == 128) return G == 1 ? launch_decode<BF16, 128, 1>(MOA_DEC_ARGS, MOA_DEC_TAIL) : launch_decode_gqa<BF16, 128>(MOA_DEC_ARGS, G, MOA_DEC_TAIL);
  return G == 1 ? launch_decode<BF16, 64, 1>(MOA_DEC_ARGS, MOA_DEC_TAIL) : launch_decode_gqa<BF16, 64>(MOA_DEC_ARGS, G, MOA_DEC_TAIL);
#undef MOA_DEC_TAIL
#undef MOA_DEC_ARGS
}

static int decode_check_args(const char* who, const void* q, const void* kc, const void* vc, const void* o,
                             const int64_t* head_start, const int64_t* head_valid_len, int B, int Hq,
                             int Hkv, int D, int64_t sumC, int dtype) {
  if (!q || !kc || !vc || !o || !head_start || !head_valid_len) return fail(MOA_ERR_ARG, "%s: null pointer", who);
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || sumC <= 0) return fail(MOA_ERR_ARG, "%s: B, H, sumC must be positive", who);
  if (B > 65535) return fail(MOA_ERR_UNSUPPORTED, "%s: B <= 65535", who);
  if (sumC >= ((int64_t)1 << 31)) return fail(MOA_ERR_UNSUPPORTED, "%s: at most 2^31 - 1 cache rows per batch row", who);
  if (Hq % Hkv != 0) return fail(MOA_ERR_ARG, "%s: Hq=%d is not a multiple of Hkv=%d", who, Hq, Hkv);
  const int G = Hq / Hkv;
  if (G > kGqaMaxG) return fail(MOA_ERR_UNSUPPORTED, "%s: %d query heads per kv head (at most %d)", who, G, kGqaMaxG);
  if (Hkv > kMaxHeads) return fail(MOA_ERR_UNSUPPORTED, "%s: at most %d kv heads", who, kMaxHeads);
  if (D != 64 && D != 128) return fail(MOA_ERR_UNSUPPORTED, "%s: head_dim %d (64 or 128)", who, D);
  if (dtype != MOA_DTYPE_F16 && dtype != MOA_DTYPE_BF16) return fail(MOA_ERR_UNSUPPORTED, "%s: dtype %d (f16 or bf16)", who, dtype);
  if (!aligned16(q) || !aligned16(kc) || !aligned16(vc) || !aligned16(o))
    return fail(MOA_ERR_ARG, "%s: pointers must be 16-byte aligned", who);
  return MOA_OK;
}

// ---- scratch of the entry point that allocates nothing -------------------------------------------
// The split-K partials of moa_decode_fwd_noalloc live in this file-scope array instead of a caller's
// workspace.  Every GPU the library runs on holds its own copy at its own address until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the kernels get the
// device address looked up below, once per device.
static __device__ __align__(256) unsigned char scratch[MOA_DECODE_NOALLOC_MAX_BYTES];

static int noalloc_scratch(void** out) {
  static void* ptr_of_device[kMaxDevices] = {};
  static std::mutex mu;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MOA_ERR_LAUNCH, "moa_decode_fwd_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(MOA_ERR_UNSUPPORTED, "moa_decode_fwd_noalloc: device %d (at most %d devices)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr_of_device[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));   // the copy of the array on the current device
    if (e != hipSuccess || !p)
      return fail(MOA_ERR_LAUNCH, "moa_decode_fwd_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    ptr_of_device[dev] = p;
  }
  *out = ptr_of_device[dev];
  return MOA_OK;
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
  if (int rc = decode_check_args("moa_decode_fwd", q, kc, vc, o, head_start, head_valid_len, B, Hq, Hkv, D, sumC, dtype))
    return rc;
  const size_t need = moa_decode_workspace_bytes(B, Hq, Hkv, D, sumC);
  if (!workspace || workspace_bytes < need)
    return fail(MOA_ERR_WORKSPACE, "moa_decode_fwd: workspace %zu < %zu bytes", workspace_bytes, need);
  return decode_dispatch(q, kc, vc, o, workspace, head_start, head_valid_len, B, Hq, Hkv, D,
                         sumC, sm_scale, dtype, stream);
}

extern "C" int moa_decode_fwd_noalloc(const void* q, const void* kc, const void* vc, void* o,
                                      const int64_t* head_start, const int64_t* head_valid_len, int B,
                                      int Hq, int Hkv, int D, int64_t sumC, float sm_scale, int dtype,
                                      void* stream) {
  if (int rc = decode_check_args("moa_decode_fwd_noalloc", q, kc, vc, o, head_start, head_valid_len, B, Hq, Hkv, D, sumC, dtype))
    return rc;
  const size_t need = moa_decode_workspace_bytes(B, Hq, Hkv, D, sumC);
  if (need > (size_t)MOA_DECODE_NOALLOC_MAX_BYTES)
    return fail(MOA_ERR_WORKSPACE,
                "moa_decode_fwd_noalloc: these sizes need %zu bytes of partials, the built-in scratch holds %zu; "
                "use moa_decode_fwd with a workspace",
                need, (size_t)MOA_DECODE_NOALLOC_MAX_BYTES);
  void* ws = nullptr;
  if (int rc = noalloc_scratch(&ws)) return rc;
  return decode_dispatch(q, kc, vc, o, ws, head_start, head_valid_len, B, Hq, Hkv, D,
                         sumC, sm_scale, dtype, stream);
}
