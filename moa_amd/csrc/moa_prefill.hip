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
//   * one work-group of 8 waves owns 256 consecutive query rows (four 64-row
//     query blocks) of one (batch, head); each wave owns 32 rows;
//   * it walks the union of the live 64-key tiles of its four query blocks; a
//     wave skips the math of a tile that is dead for ITS query block;
//   * K and V tiles are copied global -> LDS asynchronously (no registers),
//     four stages deep, rows unpadded with XOR-permuted 16-byte chunks so
//     that every operand read is bank-conflict free;
//   * the band of a work-group is walked circularly from the tile whose index is
//     a multiple of the band length, so that neighbouring query tiles of a head
//     (resident on one XCD at the same time) ask for the same tile at the same
//     step and share it in L2.
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
//
// Schedule.  A tile costs a wave 32 MFMAs (~1000 matrix-core cycles) and about
// as many cycles of softmax VALU work, and the two do not overlap inside one
// wave.  The 8 waves therefore run as two groups of four, one wave of each
// group per SIMD.  Between two work-group barriers (one per tile) group A runs
// its matrix phase (P.V of the previous tile, Q.K^T of the current one) and then
// its softmax; group B, one phase behind, runs the softmax of the previous tile
// and then its matrix phase, so each SIMD has one wave on the matrix pipe and
// one on the vector ALU most of the time.  The matrix phase is free of VALU
// instructions: operand addresses are kept per lane in registers, stage and row
// selection go into the instructions' immediate offsets.
#include "moa_mfma.h"

namespace moa {

constexpr int kWRows = 32;    // query rows per wave
constexpr int kKV = 64;       // keys per tile (the sparsity block)
// Two shapes of work-group (NW waves, S LDS stages per tensor):
//   8 waves, 4 stages: 256 query rows, one work-group per CU, the two halves of the work-group ping-pong
//                      between matrix and softmax phase under one barrier per tile;
//   4 waves, 2 stages: 128 query rows, two work-groups per CU (half the LDS and half the waves each), which
//                      share the SIMDs the way the two halves do but are not tied to each other: while one
//                      of them starts, ends or waits for the dispatcher the other has the CU to itself.
#ifndef MOA_PF_WAVES
#define MOA_PF_WAVES 8
#endif
constexpr int kMaxSortedHeads = 512;   // kv heads the span-sorted schedule handles (else: given order)

struct Strides4 {
  int64_t b, h, n;
};

template <typename T, int D, int NW, int S>
__global__ __launch_bounds__(NW * 64, 8 / NW) void prefill_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    uint16_t* __restrict__ o, Strides4 qs, Strides4 ks, Strides4 vs, Strides4 os, int BH, int Hq,
    int group, int N, int n_qtiles, const int64_t* __restrict__ sink_blocks,
    const int64_t* __restrict__ local_blocks, float scale_log2_signed) {
  constexpr int KS = D / 16;          // MFMA k-steps of the QK^T product
  constexpr int DT = D / 32;          // 32-wide d tiles of the output
  constexpr int CPR = D / 8;          // 16-byte chunks per K/V row
  constexpr int kPfThreads = NW * 64;
  constexpr int kQRows = NW * kWRows; // query rows per work-group
  constexpr int kQBlocks = kQRows / kKV;   // 64-row query blocks per work-group (two waves each)
  constexpr int kStages = S;          // LDS stages per tensor
  constexpr int LPW = CPR / NW;       // async copies per wave per tile and tensor (64 chunks each)
  static_assert(NW == 4 || NW == 8, "4 or 8 waves");
  static_assert(S == 2 || S == 4, "the stage ring is a power of two");
  constexpr int TILE_B = kKV * D * 2; // bytes of one K or V stage (rows unpadded)
  constexpr int ROW_B = D * 2;
  constexpr int RSH = 16 / CPR;       // rows per 256 bytes of LDS (1 at D=128, 2 at D=64)
  constexpr float kRescaleLimit = 256.f;   // the reference exponent is raised (and O rescaled) when a lane's 32 weights sum to more
  // The row maximum is taken over the unscaled scores, which needs a scale >= 0: a negative softmax
  // scale is moved into Q (sign bits of the packed 16-bit elements flipped, exact) and its magnitude kept.
  const float scale_log2 = __builtin_fabsf(scale_log2_signed);
  const uint32_t q_sign = scale_log2_signed < 0.f ? 0x80008000u : 0u;
  static_assert(4 * DT == 2 * KS, "P.V and Q.K^T have the same number of MFMAs per tile");

  // LDS: kStages K stages, then kStages V stages; tile t lives in stage t % kStages.  Rows are
  // unpadded (an async copy fills 1 KiB of consecutive LDS) with their 16-byte chunks XOR-permuted:
  //   K: chunk c of row n sits at position c ^ ((n / RSH) % CPR)           (16 rows x same chunk)
  //   V: chunk c of row n sits at position c ^ (4 * ((n / RSH) % (CPR/4)))  (4 rows x 4 chunks)
  extern __shared__ __attribute__((aligned(1024))) char s_mem[];
  char* const s_k = s_mem;
  char* const s_v = s_mem + kStages * TILE_B;

  // ---- which (head, query tile) --------------------------------------------
  // Work-groups are dealt to the 8 XCDs round-robin by the hardware: group idx goes to XCD idx%8
  // and is the (idx/8)-th one there.  An XCD walks (batch, head) pairs one after the other, late
  // (long) query tiles first, so that the groups resident on it share one head's K/V in L2.
  // Heads differ a lot in span, so the pairs are dealt to the XCDs from a list sorted by
  // decreasing span, in snake order (0..7, 7..0, ...): every XCD gets about the same work and
  // takes its long heads first, its short ones last.
  const int tid = threadIdx.x;
  const int Hkv = Hq / group;
  const int nb = (N + kKV - 1) / kKV;
  __shared__ int s_head_of_rank[kMaxSortedHeads], s_ns[kMaxSortedHeads], s_nl[kMaxSortedHeads];
  const bool sorted = Hkv <= kMaxSortedHeads;
  // block counts clamped to [0, nb]: beyond that range they select the same tiles
  auto clamp_blocks = [&](int64_t x) __attribute__((always_inline)) { return (int)max((int64_t)0, min((int64_t)nb, x)); };
  if (sorted) {
    for (int h = tid; h < Hkv; h += kPfThreads) {
      s_ns[h] = clamp_blocks(sink_blocks[h]);
      s_nl[h] = clamp_blocks(local_blocks[h]);
    }
    __syncthreads();
    for (int h = tid; h < Hkv; h += kPfThreads) {
      const int wh = min(nb, s_ns[h] + s_nl[h]);
      int rank = 0;
      for (int j = 0; j < Hkv; ++j) {
        const int wj = min(nb, s_ns[j] + s_nl[j]);
        rank += (wj > wh) || (wj == wh && j < h);
      }
      s_head_of_rank[rank] = h;
    }
    __syncthreads();
  }
  const int xcd = blockIdx.x & 7;
  const int seq = blockIdx.x >> 3;
  const int round = seq / n_qtiles;                                // this XCD's round-th pair
  const int pos = round * 8 + ((round & 1) ? 7 - xcd : xcd);      // position in the sorted list
  if (pos >= BH) return;
  // sorted list: kv heads by rank; per kv head, batch-major, then the query heads of its group
  const int per_head = (BH / Hq) * group;
  const int hk = __builtin_amdgcn_readfirstlane(sorted ? s_head_of_rank[pos / per_head] : pos / per_head);
  const int b = (pos % per_head) / group;
  const int hq = hk * group + pos % group;
  const int qt = n_qtiles - 1 - (seq % n_qtiles);

  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;    // 0: group A, 1: group B (one phase behind A); four waves: all A
  const int mcol = lane & 31;   // query row inside the wave's 32 (the MFMA column)
  const int g = lane >> 5;      // half-wave

  const int ns = __builtin_amdgcn_readfirstlane(sorted ? s_ns[hk] : clamp_blocks(sink_blocks[hk]));
  const int nl = __builtin_amdgcn_readfirstlane(sorted ? s_nl[hk] : clamp_blocks(local_blocks[hk]));
  const int mb0 = kQBlocks * qt;                           // first query block of the group
  const int mbl = min(kQBlocks * qt + kQBlocks - 1, nb - 1);   // last one that exists
  const int mbw = kQBlocks * qt + (wave >> 1);             // this wave's query block
  const bool wave_has_rows = mbw < nb;

  // tiles of the work-group: sinks [0, hi1], then band [lo2, mbl]
  const int hi1 = min(ns - 1, mbl);
  int lo2 = max(0, mb0 + 1 - nl);
  if (lo2 <= hi1) lo2 = hi1 + 1;
  const int n_sink = hi1 + 1;
  const int n_tiles = n_sink + max(0, mbl - lo2 + 1);
  // The band is walked circularly, starting at the tile whose index is a multiple of the band
  // length: step u visits the band tile congruent to u.  Work-groups of one head whose bands
  // overlap (neighbouring query tiles, resident on the same XCD at the same time) then ask for
  // the same K/V tile at the same step and share it in L2.  The order is free: online softmax
  // does not care, liveness and the causal mask go by tile index.
  const int n_band = n_tiles - n_sink;
  const int band_rot = n_band > 0 ? (n_band - lo2 % n_band) % n_band : 0;
  auto tile_at = [&](int t) __attribute__((always_inline)) {
    if (t < n_sink) return t;
    int u = t - n_sink + band_rot;
    if (u >= n_band) u -= n_band;
    return lo2 + u;
  };
  // this wave's own live set
  const int w_hi1 = min(ns - 1, mbw);
  const int w_lo2 = max(0, mbw + 1 - nl);
  auto live_tile = [&](int j) __attribute__((always_inline)) { return wave_has_rows && (j <= w_hi1 || (j >= w_lo2 && j <= mbw)); };

  const int64_t m_glob = (int64_t)qt * kQRows + wave * kWRows + mcol;   // this lane's query row

  if (n_tiles == 0) {   // nothing is visible from this query tile: zeros
    if (wave_has_rows && m_glob < N) {
      uint16_t* orow = o + b * os.b + hq * os.h + m_glob * os.n;
      u32x2 z = {0, 0};
#pragma unroll
      for (int i = 0; i < D / 8; ++i) *reinterpret_cast<u32x2*>(orow + 8 * i + 4 * g) = z;
    }
    return;
  }

  // ---- async tile copies: wave w, copy i fills chunks [(w*LPW+i)*64, +64) of a stage --------
  const uint16_t* kbase = k + b * ks.b + hk * ks.h;   // uniform
  const uint16_t* vbase = v + b * vs.b + hk * vs.h;
  uint32_t koff[LPW], voff[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int L = (wave * LPW + i) * 64 + lane;     // chunk position inside the stage
    const int row = L / CPR, pos = L % CPR;
    koff[i] = 2u * ((uint32_t)(row * ks.n) + (uint32_t)((pos ^ ((row / RSH) % CPR)) * 8));   // bytes
    voff[i] = 2u * ((uint32_t)(row * vs.n) + (uint32_t)((pos ^ (4 * ((row / RSH) % (CPR / 4)))) * 8));
  }
  // rows >= N of the ragged last tile repeat row N-1: their scores are masked, their softmax
  // weight is exactly 0, and a repeated real row is finite
  // a tile is 64 rows: its byte offset inside the head fits 32 bits (checked on the host)
  const uint32_t k_tile_bytes = (uint32_t)(2 * kKV * ks.n), v_tile_bytes = (uint32_t)(2 * kKV * vs.n);
  const int j_ragged = (N % kKV) ? nb - 1 : -1;    // the only tile with rows past N, if any
  auto issue_tile = [&](const uint16_t* base, uint32_t tile_bytes, int64_t stride_n, const uint32_t (&off)[LPW],
                        bool is_k, int j, uint32_t dst) __attribute__((always_inline)) {
    const char* src = reinterpret_cast<const char*>(base) + (uint64_t)(uint32_t)j * tile_bytes;
    if (j != j_ragged) {
#pragma unroll
      for (int i = 0; i < LPW; ++i) async_copy16(src, off[i], dst + i * 1024);
    } else {
      const int last = N - 1 - j * kKV;
#pragma unroll
      for (int i = 0; i < LPW; ++i) {
        const int L = (wave * LPW + i) * 64 + lane;
        const int row = L / CPR, pos = L % CPR;
        const int sw = is_k ? ((row / RSH) % CPR) : (4 * ((row / RSH) % (CPR / 4)));
        async_copy16(src, 2u * ((uint32_t)(min(row, last) * stride_n) + (uint32_t)((pos ^ sw) * 8)), dst + i * 1024);
      }
    }
  };
  // Scalar schedule state.  The tile order is piecewise consecutive (sinks, then the band from its
  // rotated start, wrapping once), so the tile of the next step follows from the current one with a
  // few scalar instructions; a step past the last tile repeats the last tile: its copy goes into a
  // stage that nobody reads any more, every iteration starts the same number of copies and the
  // wait before a barrier is a constant.
  const int band_last = lo2 + n_band - 1;
  const int band_first = lo2 + band_rot;
  auto next_tile = [&](int j, int t_next) __attribute__((always_inline)) {
    int jn = j + 1;
    jn = (jn > band_last) ? lo2 : jn;
    jn = (t_next == n_sink) ? band_first : jn;
    return (t_next >= n_tiles) ? j : jn;
  };
  constexpr uint32_t kRing = kStages * TILE_B;                       // bytes of one tensor's ring (a power of two)
  const uint32_t k_dst0 = lds_address(s_k) + wave * LPW * 1024;      // this wave's share of stage 0
  const uint32_t v_dst0 = lds_address(s_v) + wave * LPW * 1024;
  int jt[S];   // tiles of steps t .. t+S-1
  jt[0] = tile_at(0);
#pragma unroll
  for (int i = 1; i < S; ++i) jt[i] = next_tile(jt[i - 1], i);

  // The matrix phase of iteration t reads K(t) and V(t-1) and starts the copies of K(t+S-1) and
  // V(t+S-2), whose stages were last read in iteration t-1 by every wave.  Before the loop:
  // K(0..S-2), V(0..S-3).
#pragma unroll
  for (int i = 0; i + 1 < S; ++i) {
    issue_tile(kbase, k_tile_bytes, ks.n, koff, true, jt[i], k_dst0 + i * TILE_B);
    if (i + 2 < S) issue_tile(vbase, v_tile_bytes, vs.n, voff, false, jt[i], v_dst0 + i * TILE_B);
  }

  // ---- Q fragment (B operand): Q[m][16*ks + 8*g .. +7] ---------------------
  u32x4 qf[KS];
  {
    const uint16_t* qrow = q + b * qs.b + hq * qs.h + m_glob * qs.n + 8 * g;
    const bool ok = m_glob < N;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      u32x4 z = {0, 0, 0, 0};
      qf[s] = ok ? *reinterpret_cast<const u32x4*>(qrow + 16 * s) : z;
      qf[s] ^= u32x4{q_sign, q_sign, q_sign, q_sign};
    }
  }

  f32x16 oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[t][i] = 0.f;
  f32x16 st[2];              // S^T of the current tile
  uint32_t pf[16];           // P^T of the current tile, packed pairs, B-operand order
#pragma unroll
  for (int i = 0; i < 16; ++i) pf[i] = 0;
  float m_run = -INFINITY;   // reference exponent of exp2: an integer, ceil of the row max of scale_log2 * s when it was last set; a later max may pass it by < 8
  float l_run = 0.f;         // this lane's share of the running sum (the lane+32 twin holds the rest)

  // ---- operand read addresses: LDS byte address of stage 0, row 0 of this lane; stage, half and
  // k-step go into the instruction's immediate offset, so the matrix phase needs no VALU work ----
  uint32_t k_ad[KS];
  {
    const uint32_t k_rd = (uint32_t)(mcol * ROW_B) | (uint32_t)(((g ^ ((mcol / RSH) % CPR)) & (CPR - 1)) * 16);
#pragma unroll
    for (int s = 0; s < KS; ++s) k_ad[s] = lds_address(s_k) + (k_rd ^ (uint32_t)(32 * s));
  }
  uint32_t v_ad[DT];
  {
    const int grp16 = lane & 15;
    const int dhalf = (lane >> 4) & 1;
    const int v_row = 4 * g + (grp16 >> 2);
    const uint32_t v_rd = (uint32_t)(v_row * ROW_B) +
                          (uint32_t)(((2 * dhalf + ((grp16 & 3) >> 1)) ^ (4 * ((v_row / RSH) % (CPR / 4)))) * 16 +
                                     8 * (grp16 & 1));
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) v_ad[dt] = lds_address(s_v) + (v_rd ^ (uint32_t)(64 * dt));
  }

  // Matrix phase of one iteration: P.V of the previous tile and Q.K^T of the current one,
  // alternating, operands fetched kAhead MFMAs ahead.  k_ad / v_ad point at the stages to read.
  // Slot i: even -> P.V op i/2 (k-step (i/2)/DT, d tile (i/2)%DT), odd -> Q.K^T op i/2
  // (half (i/2)%2, k-step (i/2)/2).
  auto matrix_phase = [&]() __attribute__((always_inline)) {
    constexpr int kSlots = 4 * DT + 2 * KS;
    constexpr int kAhead = 6;
    u32x4 opnd[kSlots];
    auto fetch = [&](int i) __attribute__((always_inline)) {
      const int j = i >> 1;
      if (i & 1) {
        opnd[i] = lds_load16(k_ad[j >> 1], (j & 1) * 32 * ROW_B);
      } else {
        const int tk = j / DT, dt = j % DT;
        const u32x2 lo = lds_load_tr16(v_ad[dt], (16 * tk) * ROW_B);
        const u32x2 hi = lds_load_tr16(v_ad[dt], (16 * tk + 8) * ROW_B);
        opnd[i] = u32x4{lo.x, lo.y, hi.x, hi.y};
      }
    };
    auto op = [&](int i) __attribute__((always_inline)) {
      const int j = i >> 1;
      if (i & 1) {
        const int nt = j & 1, s = j >> 1;
        if (s == 0) {
          f32x16 z;
#pragma unroll
          for (int e = 0; e < 16; ++e) z[e] = 0.f;
          st[nt] = T::mfma(opnd[i], qf[0], z);
        } else {
          st[nt] = T::mfma(opnd[i], qf[s], st[nt]);
        }
      } else {
        const int tk = j / DT, dt = j % DT;
        const u32x4 bfrag = {pf[4 * tk], pf[4 * tk + 1], pf[4 * tk + 2], pf[4 * tk + 3]};
        oacc[dt] = T::mfma(opnd[i], bfrag, oacc[dt]);
      }
    };
#pragma unroll
    for (int i = 0; i < kAhead; ++i) fetch(i);
#pragma unroll
    for (int i = 0; i < kSlots; ++i) {
      if (i + kAhead < kSlots) fetch(i + kAhead);
      op(i);
      __builtin_amdgcn_sched_barrier(0);   // keeps the operand reads kAhead MFMAs ahead of their use
    }
  };
  // Q.K^T only (the first iteration)
  auto qk_phase = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      u32x4 kf[KS];
#pragma unroll
      for (int s = 0; s < KS; ++s) kf[s] = lds_load16(k_ad[s], nt * 32 * ROW_B);
#pragma unroll
      for (int i = 0; i < 16; ++i) st[nt][i] = 0.f;
#pragma unroll
      for (int s = 0; s < KS; ++s) st[nt] = T::mfma(kf[s], qf[s], st[nt]);
    }
  };
  // mask + online softmax of tile j: st -> pf, updates m_run, l_run (and rescales oacc when needed;
  // every P.V issued so far belongs to earlier tiles and has completed in this wave's matrix phase)
  auto softmax = [&](int j) __attribute__((always_inline)) {
    if (j == mbw) {   // causal mask on the diagonal tile
      int thr = (wave & 1) * kWRows + mcol - 4 * g;   // row inside the 64-row block, minus the lane's column base
      asm volatile("" : "+v"(thr));                  // keeps the 32 compares in this branch instead of 32 hoisted lane masks
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (nt * 32 + 8 * (i >> 2) + (i & 3) > thr) st[nt][i] = -INFINITY;
    }
    // Row sums are plain fp32 adds of the unrounded weights.  (v_dot2_f32_{f16,bf16} of the packed
    // pair with a pair of ones would halve the instruction count, but those instructions stall the
    // MFMA stream of the wave that shares the SIMD: measured 20 % slower per iteration.)
    float psum[2];
    auto weights = [&]() __attribute__((always_inline)) {
      psum[0] = psum[1] = 0.f;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[nt][i], scale_log2, -m_run));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(st[nt][i + 1], scale_log2, -m_run));
          pf[nt * 8 + (i >> 1)] = T::pack_rne(p0, p1);
          psum[0] += p0;
          psum[1] += p1;
        }
    };
    // The common case needs no row maximum: weights are formed against the reference exponent as it
    // stands, and their sum tells whether that was good enough.  A lane's 32 weights are >= 0, so a sum of
    // at most 2^8 bounds each of them by 2^8 (the 16-bit types hold that with room to spare); a larger
    // sum, or the first live tile (the reference is still -inf and the sum is inf or NaN; the file is
    // compiled without NaN semantics, so that case is asked for by name), takes the path below.
    weights();
    if (__builtin_expect(__any(m_run == -INFINITY || psum[0] + psum[1] > kRescaleLimit), 0)) {
      float mx = st[0][0];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = fmaxf(mx, st[nt][i]);
      mx = max_with_other_half(mx);
      const float m_cand = mx * scale_log2;   // finite: a live tile has a visible key in every row
      // The reference exponent stays an INTEGER: a weight is then 2^frac * 2^int, and its rounding to the
      // storage type does not depend on the power of two, so the rounded weights (relative to the row's
      // sum) do not depend on the tile order or on how far m_run lags behind the true maximum.
      const float m_new = __builtin_ceilf(fmaxf(m_run, m_cand));
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= alpha;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) oacc[t][i] *= alpha;
      m_run = m_new;
      weights();
    }
    l_run += psum[0] + psum[1];
  };

  wait_vm(0);
  // the Q loads have landed too; pin that fact here so that the compiler does not put its own
  // vmcnt(0) wait at their first use inside the loop, where it would also wait for the copies
#pragma unroll
  for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));
  phase_barrier();               // K(0..2) and V(0..1) are in LDS

  // Iteration t: matrix phase = P.V of tile t-1 and Q.K^T of tile t, then softmax phase = tile t.
  // There is one work-group barrier per iteration; group A meets it after its softmax phase, group
  // B after its matrix phase, so B's softmax of tile t runs beside A's matrix phase of tile t+1 and
  // each SIMD holds one wave in either phase.  A wave for which tile t-1 or t is not live still
  // runs the whole matrix phase (with P = 0, or ignoring S), which keeps the loop body a single
  // straight block; it skips the phase when neither is live.  The copies started in iteration t
  // overwrite the stages of K(t-1) and V(t-2), which every wave has finished reading before
  // barrier t-1; the copies started two iterations ago (K(t+1), V(t)) are first read after barrier
  // t, and every wave waits for its own before it.  Iteration n_tiles only finishes P.V of the
  // last tile.
  uint32_t cst = (S - 1) * TILE_B;   // ring offset of the stage K(t+S-1) is copied into; V(t+S-2) goes one stage below
  uint32_t rst = 0;            // ring offset of the stage K(t) is read from
  int kd_prev = 0;             // how far the K read addresses moved in the previous iteration
  bool lc_prev = false;        // was tile t-1 live for this wave
  auto iteration = [&](int t, auto FIRST) __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(FIRST)::value != 0;
    constexpr int n_wait = (S - 2) * 2 * LPW;   // copies started in the last S-2 iterations may still be in flight
    // ---------------- matrix phase ----------------
    issue_tile(kbase, k_tile_bytes, ks.n, koff, true, jt[S - 1], k_dst0 + cst);
    issue_tile(vbase, v_tile_bytes, vs.n, voff, false, jt[S - 2], v_dst0 + ((cst - TILE_B) & (kRing - 1)));
    const bool lp = lc_prev, lc = (t < n_tiles) && live_tile(jt[0]);
    if (kFirst) {
      if (lc) qk_phase();
    } else {
      if (lp || lc) matrix_phase();
    }
    if (NW == 8 && grp == 1) { wait_vm(n_wait); phase_barrier(); }
    // ---------------- softmax phase ----------------
    if (lc) {
      softmax(jt[0]);
    } else if (lp) {   // the next matrix phase this wave runs must add nothing for a dead tile
#pragma unroll
      for (int i = 0; i < 16; ++i) pf[i] = 0;
    }
    // advance the operand addresses to the next stages (K: t+1, V: t) and the schedule by one step
    {
      const int kd = (rst == (kStages - 1) * TILE_B) ? -(kStages - 1) * TILE_B : TILE_B;
#pragma unroll
      for (int s = 0; s < KS; ++s) k_ad[s] += kd;
      if (!kFirst) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) v_ad[dt] += kd_prev;   // V trails K by one step
      }
      kd_prev = kd;
      rst = (rst + TILE_B) & (kRing - 1);
      cst = (cst + TILE_B) & (kRing - 1);
      lc_prev = lc;
#pragma unroll
      for (int i = 0; i + 1 < S; ++i) jt[i] = jt[i + 1];
      jt[S - 1] = next_tile(jt[S - 1], t + S);
    }
    if (NW == 4 || grp == 0) { wait_vm(n_wait); phase_barrier(); }
  };
  iteration(0, IC<1>{});   // no P.V yet (and no V stage to read)
  for (int t = 1; t <= n_tiles; ++t) iteration(t, IC<0>{});

  wait_vm(0);   // the repeated copies of the last steps
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

template <int D, int S>
static size_t prefill_lds_bytes() {
  return (size_t)2 * S * kKV * D * sizeof(uint16_t);   // K stages + V stages
}

template <typename T, int D>
static int launch_prefill(const void* q, const void* k, const void* v, void* o, const int64_t* qs,
                          const int64_t* ks, const int64_t* vs, const int64_t* os, int B, int Hq,
                          int Hkv, int N, const int64_t* sink_blocks, const int64_t* local_blocks,
                          float sm_scale, hipStream_t st) {
  constexpr int NW = MOA_PF_WAVES, S = NW / 2;
  constexpr int kQRows = NW * kWRows;
  const int n_qtiles = (N + kQRows - 1) / kQRows;
  const int BH = B * Hq;
  const int64_t groups = (int64_t)((BH + 7) / 8) * 8 * n_qtiles;
  if (groups > 0x7fffffffLL) return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: too many work-groups");
  // the async copies address a tile row through a 32-bit element offset
  if (64 * ks[2] + D >= (1ll << 31) || 64 * vs[2] + D >= (1ll << 31))
    return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: k/v token stride too large");
  Strides4 sq = {qs[0], qs[1], qs[2]}, sk = {ks[0], ks[1], ks[2]}, sv = {vs[0], vs[1], vs[2]},
           so = {os[0], os[1], os[2]};
  const size_t lds = prefill_lds_bytes<D, S>();
  static bool lds_reserved[kMaxDevices] = {};   // per template instance
  if (int rc = reserve_lds(reinterpret_cast<const void*>(&prefill_kernel<T, D, NW, S>), lds, lds_reserved, "moa_prefill_fwd"))
    return rc;
  hipLaunchKernelGGL((prefill_kernel<T, D, NW, S>), dim3((unsigned)groups), dim3(NW * 64), lds, st,
                     (const uint16_t*)q, (const uint16_t*)k, (const uint16_t*)v, (uint16_t*)o, sq, sk, sv,
                     so, BH, Hq, Hq / Hkv, N, n_qtiles, sink_blocks, local_blocks, mfma_softmax_scale(sm_scale));
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
