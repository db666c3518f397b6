// Block-sparse causal prefill attention for per-head sink + sliding-window
// spans, on the gfx950 matrix cores.
//
// Replaces the reference's prefill kernels (Triton
// _sparse_attention_prefill_moa_fwd_kernel, MoA/kernels/block_sparse_attention_prefill.py:473-629,
// and the external moa_prefill op, MoA/kernels/mixture_of_attention.py:435-444).
// For query block m (64 rows) of a head with ns sink blocks and nl local
// blocks the live key blocks are {0..min(ns-1,m)} U {max(0,m+1-nl)..m}, with
// the causal test inside the diagonal block (:558-580).
//
// Work decomposition
//   * one work-group (4 waves) owns 128 consecutive query rows = two 64-row
//     query blocks of one (batch, head); each wave owns 32 rows;
//   * it walks the union of the live 64-key tiles of its two query blocks; a
//     wave skips the MFMA work of a tile that is dead for ITS query block;
//   * K and V tiles go global -> registers -> LDS (row-major, padded rows,
//     two buffers each): the next tile's global loads are issued one
//     iteration ahead and written to the other buffer after this tile's math,
//     so there is one work-group barrier per tile;
//   * the LDS reads of the MFMA operands are issued several MFMAs ahead of
//     their use.
//
// Matrix layout.  Both GEMMs are computed transposed so that every per-row
// softmax quantity lives in ONE lane:
//   S^T[n][m] = sum_d K[n][d] Q[m][d]      A = K (LDS), B = Q^T (registers)
//   O^T[d][m] = sum_n V[n][d] P[m][n]      A = V^T (LDS, transposing read), B = P^T
// v_mfma_f32_32x32x16 puts column m of the result in lane (m mod 32) of both
// half-waves, so row max / row sum / rescale are lane-local except for one
// exchange with lane+32, and the P tile that leaves the softmax is already in
// B-operand order (the contraction index n may be permuted freely as long as A
// and B agree; the V^T operand is fetched with that same permutation by
// ds_read_b64_tr_b16, which returns 4 consecutive rows of one column).
#include "moa_common.h"

namespace moa {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kPfThreads = 256;
constexpr int kQRows = 128;   // query rows per work-group
constexpr int kWRows = 32;    // query rows per wave
constexpr int kKV = 64;       // keys per tile (the sparsity block)
constexpr float kLog2eF = 1.4426950408889634f;

struct PF16 {
  static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
  static __device__ __forceinline__ uint32_t pack_rne(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 r = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, r);
  }
};
struct PBF16 {
  static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
    f32x2 x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2v));
  }
  static __device__ __forceinline__ uint32_t pack_rne(float lo, float hi) { return pack(lo, hi); }
};

// 4 consecutive rows of one 16-bit column out of a row-major LDS tile: within
// each group of 16 lanes, lane i must point at (row0 + i/4, col0 + 4*(i%4));
// it receives rows row0..row0+3 of column col0 + i.
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t* p) {
  typedef s16x4 __attribute__((address_space(3))) * lds_s16x4_ptr;
  s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p));
  return __builtin_bit_cast(u32x2, r);
}

struct Strides4 {
  int64_t b, h, n;
};

template <typename T, int D>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    uint16_t* __restrict__ o, Strides4 qs, Strides4 ks, Strides4 vs, Strides4 os, int BH, int Hq,
    int group, int N, int n_qtiles, const int64_t* __restrict__ sink_blocks,
    const int64_t* __restrict__ local_blocks, float scale_log2) {
  constexpr int KS = D / 16;          // MFMA k-steps of the QK^T product
  constexpr int DT = D / 32;          // 32-wide d tiles of the output
  constexpr int LDK = D + 8;          // K tile row stride (elements): rows shift 4 banks
  constexpr int LDV = D + 32;         // V tile row stride: rows shift 16 banks
  constexpr int CPR = D / 8;          // 16-byte chunks per row
  constexpr int RPP = kPfThreads / CPR;   // rows per pass of the cooperative tile load
  constexpr int PASSES = kKV / RPP;
  constexpr int KTILE = kKV * LDK;    // elements of one K buffer
  constexpr int VTILE = kKV * LDV;
  constexpr float kRescaleStep = 8.f; // rescale O only when a row max grew by more than 2^8

  // two K and two V buffers: tile j+1 is written while tile j is being read
  extern __shared__ __attribute__((aligned(16))) uint16_t s_mem[];
  uint16_t* const s_k = s_mem;
  uint16_t* const s_v = s_mem + 2 * KTILE;

  // ---- which (head, query tile) --------------------------------------------
  // Work-groups are dealt to the 8 XCDs round-robin by the hardware.  Group
  // idx goes to XCD idx%8 and is the (idx/8)-th one there; an XCD owns the heads
  // congruent to it mod 8 and walks them one after the other, late (long) query
  // tiles first, so that the groups resident on an XCD share one head's K/V in L2.
  const int xcd = blockIdx.x & 7;
  const int seq = blockIdx.x >> 3;
  const int heads_here = (BH - xcd + 7) >> 3;
  if (seq >= heads_here * n_qtiles) return;
  const int bh = (seq / n_qtiles) * 8 + xcd;
  const int qt = n_qtiles - 1 - (seq % n_qtiles);
  const int b = bh / Hq;
  const int hq = bh % Hq;
  const int hk = hq / group;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int mcol = lane & 31;   // query row inside the wave's 32 (the MFMA column)
  const int g = lane >> 5;      // half-wave

  const int nb = (N + kKV - 1) / kKV;
  const int ns = __builtin_amdgcn_readfirstlane((int)sink_blocks[hk]);
  const int nl = __builtin_amdgcn_readfirstlane((int)local_blocks[hk]);
  const int mb0 = 2 * qt;                                  // first query block of the group
  const int mb1 = min(2 * qt + 1, nb - 1);                 // last one that exists
  const int mbw = 2 * qt + (wave >> 1);                    // this wave's query block
  const bool wave_has_rows = mbw < nb;

  // tile ranges of the work-group: sinks [0, hi1], then band [lo2, mb1]
  const int hi1 = min(ns - 1, mb1);
  int lo2 = max(0, mb0 + 1 - nl);
  if (lo2 <= hi1) lo2 = hi1 + 1;
  // this wave's own live set
  const int w_hi1 = min(ns - 1, mbw);
  const int w_lo2 = max(0, mbw + 1 - nl);

  const int64_t m_glob = (int64_t)qt * kQRows + wave * kWRows + mcol;   // this lane's query row

  // ---- Q fragment (B operand): Q[m][16*ks + 8*g .. +7] ---------------------
  u32x4 qf[KS];
  {
    const uint16_t* qrow = q + b * qs.b + hq * qs.h + m_glob * qs.n + 8 * g;
    const bool ok = m_glob < N;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      u32x4 z = {0, 0, 0, 0};
      qf[s] = ok ? *reinterpret_cast<const u32x4*>(qrow + 16 * s) : z;
    }
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[t][i] = 0.f;
  float m_run = -INFINITY;   // reference max of scale_log2 * s used by exp2 (lags the true max by <= kRescaleStep)
  float l_run = 0.f;         // this lane's share of the running sum (the lane+32 twin holds the rest)

  // ---- cooperative tile load: thread -> (row, 16-byte chunk) ----------------
  const int ld_row = tid / CPR;
  const int ld_chk = tid % CPR;
  const uint16_t* kbase = k + b * ks.b + hk * ks.h;   // uniform
  const uint16_t* vbase = v + b * vs.b + hk * vs.h;
  uint32_t koff[PASSES], voff[PASSES];                // element offsets inside a tile
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    koff[p] = (uint32_t)((p * RPP + ld_row) * ks.n + ld_chk * 8);
    voff[p] = (uint32_t)((p * RPP + ld_row) * vs.n + ld_chk * 8);
  }
  u32x4 kreg[PASSES], vreg[PASSES];

  auto issue_loads = [&](int j) {
    const uint16_t* kt = kbase + (int64_t)j * kKV * ks.n;
    const uint16_t* vt = vbase + (int64_t)j * kKV * vs.n;
    if ((j + 1) * kKV <= N) {
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        kreg[p] = *reinterpret_cast<const u32x4*>(kt + koff[p]);
        vreg[p] = *reinterpret_cast<const u32x4*>(vt + voff[p]);
      }
    } else {   // the ragged last tile: rows >= N read as zero
#pragma unroll
      for (int p = 0; p < PASSES; ++p) {
        const bool ok = j * kKV + p * RPP + ld_row < N;
        u32x4 z = {0, 0, 0, 0};
        kreg[p] = ok ? *reinterpret_cast<const u32x4*>(kt + koff[p]) : z;
        vreg[p] = ok ? *reinterpret_cast<const u32x4*>(vt + voff[p]) : z;
      }
    }
  };
  auto store_tile = [&](int buf) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int r = p * RPP + ld_row;
      *reinterpret_cast<u32x4*>(s_k + buf * KTILE + r * LDK + ld_chk * 8) = kreg[p];
      *reinterpret_cast<u32x4*>(s_v + buf * VTILE + r * LDV + ld_chk * 8) = vreg[p];
    }
  };
  auto next_tile = [&](int j) { return (j == hi1) ? lo2 : j + 1; };

  // operand read positions inside a buffer
  const int k_rd_off = mcol * LDK + 8 * g;                               // + 32*nt*LDK + 16*ks
  const int grp16 = lane & 15;
  const int dhalf = (lane >> 4) & 1;
  const int v_rd_off = (4 * g + (grp16 >> 2)) * LDV + 16 * dhalf + 4 * (grp16 & 3);
                                                                         // + (16*t [+8])*LDV + 32*dt

  int j = (hi1 >= 0) ? 0 : lo2;
  if (j > mb1) {   // nothing is visible from this query tile: zeros
    if (wave_has_rows && m_glob < N) {
      uint16_t* orow = o + b * os.b + hq * os.h + m_glob * os.n;
      u32x2 z = {0, 0};
#pragma unroll
      for (int i = 0; i < D / 8; ++i) *reinterpret_cast<u32x2*>(orow + 8 * i + 4 * g) = z;
    }
    return;
  }
  issue_loads(j);
  store_tile(0);
  int jn = next_tile(j);
  if (jn <= mb1) issue_loads(jn);
  __syncthreads();

  int buf = 0;
  while (true) {
    const bool live = wave_has_rows && (j <= w_hi1 || (j >= w_lo2 && j <= mbw));
    if (live) {
      const uint16_t* k_rd = s_k + buf * KTILE + k_rd_off;
      const uint16_t* v_rd = s_v + buf * VTILE + v_rd_off;
      // ---- S^T = K Q^T : two 32-key tiles; the operand reads run kPre MFMAs ahead ----
      f32x16 st[2];
      {
        constexpr int kPre = 8;
        u32x4 a[2 * KS];
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int s = 0; s < KS; ++s)
            a[nt * KS + s] = *reinterpret_cast<const u32x4*>(k_rd + nt * 32 * LDK + 16 * s);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
          for (int i = 0; i < 16; ++i) st[nt][i] = 0.f;
#pragma unroll
          for (int s = 0; s < KS; ++s) st[nt] = T::mfma(a[nt * KS + s], qf[s], st[nt]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, kPre < 2 * KS ? kPre : 2 * KS, 0);
#pragma unroll
        for (int i = 0; i < 2 * KS - kPre; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kPre < 2 * KS ? kPre : 2 * KS, 0);
      }
      // ---- causal mask on the diagonal tile ----
      if (j == mbw) {
        const int m_in = (wave & 1) * kWRows + mcol;   // row inside the 64-row block
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int n_in = nt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
            if (n_in > m_in) st[nt][i] = -INFINITY;
          }
      }
      // ---- online softmax, base 2, with a lagging reference max ----
      float mx = st[0][0];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, st[nt][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_cand = mx * scale_log2;   // finite: a live tile has a visible key in every row
      // exp2 arguments stay <= kRescaleStep as long as no row max outgrew its reference by more
      // than that; only then are O and l rescaled (a wave-uniform, rare branch after the first tile)
      if (__any(m_cand > m_run + kRescaleStep)) {
        const float m_new = fmaxf(m_run, m_cand);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        l_run *= alpha;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) oacc[t][i] *= alpha;
        m_run = m_new;
      }
      float psum = 0.f;
      uint32_t pf[16];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[nt][i], scale_log2, -m_run));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[nt][i + 1], scale_log2, -m_run));
          psum += p0 + p1;
          pf[nt * 8 + (i >> 1)] = T::pack(p0, p1);
        }
      l_run += psum;
      // ---- O^T += V^T P^T ; operand reads run kPre MFMAs ahead ----
      {
        constexpr int kPre = 4;
        u32x4 a[4 * DT];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const u32x2 lo = lds_read_tr16(v_rd + (16 * t) * LDV + 32 * dt);
            const u32x2 hi = lds_read_tr16(v_rd + (16 * t + 8) * LDV + 32 * dt);
            a[t * DT + dt] = u32x4{lo.x, lo.y, hi.x, hi.y};
          }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const u32x4 bfrag = {pf[4 * t], pf[4 * t + 1], pf[4 * t + 2], pf[4 * t + 3]};
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) oacc[dt] = T::mfma(a[t * DT + dt], bfrag, oacc[dt]);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * kPre, 0);
#pragma unroll
        for (int i = 0; i < 4 * DT - kPre; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, kPre, 0);
      }
    }
    if (jn > mb1) break;
    // tile jn (in registers since the previous iteration) goes into the other buffer; every wave
    // left that buffer before the last barrier
    store_tile(buf ^ 1);
    j = jn;
    jn = next_tile(j);
    if (jn <= mb1) issue_loads(jn);
    __syncthreads();
    buf ^= 1;
  }

  // ---- epilogue: O[m][d] = O^T[d][m] / l ---------------------------------
  if (!wave_has_rows || m_glob >= N) return;
  const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
  uint16_t* orow = o + b * os.b + hq * os.h + m_glob * os.n;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int gi = 0; gi < 4; ++gi) {
      const int d = 32 * dt + 8 * gi + 4 * g;
      u32x2 w;
      w.x = T::pack_rne(oacc[dt][4 * gi + 0] * inv, oacc[dt][4 * gi + 1] * inv);
      w.y = T::pack_rne(oacc[dt][4 * gi + 2] * inv, oacc[dt][4 * gi + 3] * inv);
      *reinterpret_cast<u32x2*>(orow + d) = w;
    }
}

template <typename T, int D>
static size_t prefill_lds_bytes() {
  return (size_t)2 * kKV * ((D + 8) + (D + 32)) * sizeof(uint16_t);
}

template <typename T, int D>
static int launch_prefill(const void* q, const void* k, const void* v, void* o, const int64_t* qs,
                          const int64_t* ks, const int64_t* vs, const int64_t* os, int B, int Hq,
                          int Hkv, int N, const int64_t* sink_blocks, const int64_t* local_blocks,
                          float sm_scale, hipStream_t st) {
  const int n_qtiles = (N + kQRows - 1) / kQRows;
  const int BH = B * Hq;
  const int64_t groups = (int64_t)((BH + 7) / 8) * 8 * n_qtiles;
  if (groups > 0x7fffffffLL) return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: too many work-groups");
  Strides4 sq = {qs[0], qs[1], qs[2]}, sk = {ks[0], ks[1], ks[2]}, sv = {vs[0], vs[1], vs[2]},
           so = {os[0], os[1], os[2]};
  const size_t lds = prefill_lds_bytes<T, D>();
  static bool attr_set = false;   // per template instance
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_kernel<T, D>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess)
      return fail(MOA_ERR_LAUNCH, "moa_prefill_fwd: cannot reserve %zu bytes of LDS: %s", lds,
                  hipGetErrorString(e));
    attr_set = true;
  }
  hipLaunchKernelGGL((prefill_kernel<T, D>), dim3((unsigned)groups), dim3(kPfThreads), lds, st,
                     (const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (uint16_t*)o, sq, sk, sv,
                     so, BH, Hq, Hq / Hkv, N, n_qtiles, sink_blocks, local_blocks, sm_scale * kLog2eF);
  return check_launch("moa_prefill_fwd");
}

static int check_strides(const char* name, const int64_t* s, const void* p) {
  if (!s) return fail(MOA_ERR_ARG, "moa_prefill_fwd: null %s strides", name);
  if (s[3] != 1) return fail(MOA_ERR_ARG, "moa_prefill_fwd: %s must have unit stride along head_dim", name);
  for (int i = 0; i < 3; ++i)
    if (s[i] % 8 != 0)
      return fail(MOA_ERR_ARG, "moa_prefill_fwd: %s stride %d (%lld elements) breaks 16-byte row alignment",
                  name, i, (long long)s[i]);
  if (!aligned16(p)) return fail(MOA_ERR_ARG, "moa_prefill_fwd: %s must be 16-byte aligned", name);
  return MOA_OK;
}

}  // namespace moa

using namespace moa;

extern "C" int moa_prefill_fwd(const void* q, const void* k, const void* v, void* o,
                               const int64_t* q_strides, const int64_t* k_strides,
                               const int64_t* v_strides, const int64_t* o_strides, int B, int Hq,
                               int Hkv, int N, int D, const int64_t* sink_blocks,
                               const int64_t* local_blocks, float sm_scale, int dtype, void* stream) {
  if (!q || !k || !v || !o || !sink_blocks || !local_blocks)
    return fail(MOA_ERR_ARG, "moa_prefill_fwd: null pointer");
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || N <= 0) return fail(MOA_ERR_ARG, "moa_prefill_fwd: B, H, N must be positive");
  if (Hq % Hkv != 0) return fail(MOA_ERR_ARG, "moa_prefill_fwd: Hq=%d is not a multiple of Hkv=%d", Hq, Hkv);
  if (D != 64 && D != 128) return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: head_dim %d (64 or 128)", D);
  if (dtype != MOA_DTYPE_F16 && dtype != MOA_DTYPE_BF16)
    return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: dtype %d (f16 or bf16)", dtype);
  int rc;
  if ((rc = check_strides("q", q_strides, q))) return rc;
  if ((rc = check_strides("k", k_strides, k))) return rc;
  if ((rc = check_strides("v", v_strides, v))) return rc;
  if ((rc = check_strides("o", o_strides, o))) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MOA_DTYPE_F16) {
    if (D == 128) return launch_prefill<PF16, 128>(q, k, v, o, q_strides, k_strides, v_strides, o_strides, B, Hq, Hkv, N, sink_blocks, local_blocks, sm_scale, st);
    return launch_prefill<PF16, 64>(q, k, v, o, q_strides, k_strides, v_strides, o_strides, B, Hq, Hkv, N, sink_blocks, local_blocks, sm_scale, st);
  }
  if (D == 128) return launch_prefill<PBF16, 128>(q, k, v, o, q_strides, k_strides, v_strides, o_strides, B, Hq, Hkv, N, sink_blocks, local_blocks, sm_scale, st);
  return launch_prefill<PBF16, 64>(q, k, v, o, q_strides, k_strides, v_strides, o_strides, B, Hq, Hkv, N, sink_blocks, local_blocks, sm_scale, st);
}
