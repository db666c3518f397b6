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
//   * a work item is 256 consecutive query rows (four 64-row query blocks) of
//     one (batch, head); a work-group of 8 waves takes one item at a time, each
//     wave 32 rows of it;
//   * one work-group per CU stays resident for the whole launch and takes items
//     from a queue (a few counters in device memory): the hardware dispatcher
//     hands work-groups to the XCDs strictly round-robin, so with one
//     work-group per item a CU that falls free waits until it is its XCD's turn
//     (measured: 7 % of CU time at the benchmark shape);
//   * thread 0 turns a queue ticket into an item descriptor (base pointers, tile
//     schedule) once and leaves it in LDS; it does so for item i+1 a few
//     iterations before item i ends, and item i's last iteration starts the
//     first copies of item i+1;
//   * a work-group walks the union of the live 64-key tiles of its four query
//     blocks; a wave skips the math of a tile that is dead for ITS query block;
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

#include <atomic>
#include <mutex>

namespace moa {

constexpr int kWRows = 32;    // query rows per wave
constexpr int kKV = 64;       // keys per tile (the sparsity block)

// Work queue of one launch: next[x] = items of XCD list x handed out so far, done = work-groups that have
// left.  The queues live in a file-scope device array (every GPU the library runs on holds its own copy; in
// host code the array's name is only a handle for hipGetSymbolAddress).  A launch takes the next of the
// kQueueSlots slots in turn, so launches that overlap on one GPU do not share counters unless more than
// kQueueSlots of them are under way at once.  A slot starts at zero and is left at zero: the last
// work-group to leave a launch clears it.
struct PrefillQueue {
  unsigned next[8];
  unsigned done;
  unsigned pad[7];
};
constexpr int kQueueSlots = 256;
static __device__ __align__(256) PrefillQueue g_prefill_queues[kQueueSlots];
constexpr int kMaxSortedHeads = 512;   // kv heads the span-sorted schedule handles (else: given order)

struct Strides4 {
  int64_t b, h, n;
};

// Everything the kernel is told, as ONE kernel argument: the kernel reads the fields it needs from the
// kernel-argument segment again for every work item (through a pointer the compiler cannot see through),
// so that none of them is held in a scalar register across the item loop.
struct PrefillArgs {
  const uint16_t *q, *k, *v;
  uint16_t* o;
  Strides4 qs, ks, vs, os;
  const int64_t *sink_blocks, *local_blocks;
  PrefillQueue* queue;
  int BH, Hq, group, N, n_qtiles;
  int per_head, Hkv;   // (BH / Hq) * group pairs per kv head in the sorted list; Hq / group
  float scale_log2_signed;
};
typedef const PrefillArgs __attribute__((address_space(4)))* PrefillArgsPtr;

// x / d and x % d for 0 <= x < 2^22, 0 < d < 2^22, through the float reciprocal and one correction step
// each way (the compiler's general 32-bit division is four times as many instructions, and thread 0 does
// a dozen of these per work item on the critical path).
struct DivMod {
  int q, r;
};
__device__ __forceinline__ DivMod divmod_small(int x, int d) {
  int q = (int)((float)x * __builtin_amdgcn_rcpf((float)d));
  int r = x - q * d;
  if (r < 0) { q -= 1; r += d; }
  if (r >= d) { q += 1; r -= d; }
  return {q, r};
}

template <typename T, int D>
__global__ __launch_bounds__(512, 1) void prefill_kernel(PrefillArgs args_in_kernarg) {
  const PrefillArgsPtr a0 = (PrefillArgsPtr)__builtin_amdgcn_kernarg_segment_ptr();   // the argument above
  constexpr int NW = 8, S = 4;
  constexpr int KS = D / 16;          // MFMA k-steps of the QK^T product
  constexpr int DT = D / 32;          // 32-wide d tiles of the output
  constexpr int CPR = D / 8;          // 16-byte chunks per K/V row
  constexpr int kPfThreads = NW * 64;
  constexpr int kQRows = NW * kWRows; // query rows per work-group
  constexpr int kQBlocks = kQRows / kKV;   // 64-row query blocks per work-group (two waves each)
  constexpr int kStages = S;          // LDS stages per tensor
  constexpr int LPW = CPR / NW;       // async copies per wave per tile and tensor (64 chunks each)
  constexpr int TILE_B = kKV * D * 2; // bytes of one K or V stage (rows unpadded)
  constexpr int ROW_B = D * 2;
  constexpr int RSH = 16 / CPR;       // rows per 256 bytes of LDS (1 at D=128, 2 at D=64)
  constexpr float kRescaleLimit = 256.f;   // the reference exponent is raised (and O rescaled) when a lane's 32 weights sum to more
  constexpr uint32_t kRing = kStages * TILE_B;   // bytes of one tensor's ring (a power of two)
  static_assert(4 * DT == 2 * KS, "P.V and Q.K^T have the same number of MFMAs per tile");

  extern __shared__ __attribute__((aligned(1024))) char s_mem[];
  char* const s_k = s_mem;
  char* const s_v = s_mem + kStages * TILE_B;

  // ---- once per work-group: heads sorted by span ------------------------------------------------
  __shared__ int s_head_of_rank[kMaxSortedHeads], s_ns[kMaxSortedHeads], s_nl[kMaxSortedHeads];
  {
    const int tid = threadIdx.x;
    const int Hkv = a0->Hq / a0->group;
    const int nb = (a0->N + kKV - 1) / kKV;
    const int64_t* sink_blocks = a0->sink_blocks;
    const int64_t* local_blocks = a0->local_blocks;
    if (Hkv <= kMaxSortedHeads) {
      for (int h = tid; h < Hkv; h += kPfThreads) {
        s_ns[h] = (int)max((int64_t)0, min((int64_t)nb, sink_blocks[h]));
        s_nl[h] = (int)max((int64_t)0, min((int64_t)nb, local_blocks[h]));
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
    }
  }

  // ---- the LDS ring keeps turning across items ----
  uint32_t cst = (S - 1) * TILE_B;   // ring offset of the stage K(t+S-1) is copied into; V(t+S-2) goes one stage below
  uint32_t rst = 0;                  // ring offset of the stage K(t) is read from
  bool prefetched = false;           // the previous item has started this item's first copies
  uint32_t q_touch = 0;              // landing place of the load that pulls the next item's Q rows into L2

  // ---- the work queue ---------------------------------------------------------------------------
  // Thread 0 takes a ticket for the item after the one under way (from the own XCD's list while that has
  // items, from the other lists then), turns it into an item descriptor once and leaves it in LDS; every wave
  // reads it from there.  The ticket is taken kTakeLead iterations before the item under way ends, not at its
  // start: a ticket held through a long item starts late, behind tickets handed out after it, and the items
  // of a head then run spread over the launch instead of side by side on their XCD (start order logged per
  // item and replayed through an LRU model of the L2: 37 % of the K/V tile reads miss with tickets taken at
  // the item's start, 22 % with late ones; measured HBM reads of the launch 2.2 GB against 1.2 GB).
  //   [0] n_tiles (-1: no more items)  [1] query tile  [2] ns  [3] nl  [4] lo2  [5] n_sink  [6] n_band  [7] band_rot
  //   [8,9] K base  [10,11] V base  [12,13] Q base (row 0 of the head)  [14,15] O base
  const int my_xcd = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 7;   // XCC_ID
  __shared__ __attribute__((aligned(16))) int s_item[2][16];
  bool own_alive = true;     // thread 0: the own list still had items when last asked
  auto take = [&](int slot) __attribute__((always_inline)) {
    PrefillArgsPtr ap = a0;
    asm volatile("" : "+s"(ap));
    const int BH = ap->BH, group = ap->group, N = ap->N, n_qtiles = ap->n_qtiles;
    const int per_head = ap->per_head, Hkv = ap->Hkv;
    const int full_rounds = BH >> 3, rem = BH & 7;
    auto list_items = [&](int x) __attribute__((always_inline)) {
      const int snake = (full_rounds & 1) ? 7 - x : x;
      return (unsigned)((full_rounds + (snake < rem ? 1 : 0)) * n_qtiles);
    };
    int list = -1;
    unsigned sq = 0;
    if (own_alive) {
      sq = atomicAdd(&ap->queue->next[my_xcd], 1u);
      if (sq < list_items(my_xcd)) list = my_xcd; else own_alive = false;
    }
    if (list < 0) {
      for (int a = 1; a < 8; ++a) {
        const int x = (my_xcd + a) & 7;
        sq = atomicAdd(&ap->queue->next[x], 1u);
        if (sq < list_items(x)) { list = x; break; }
      }
    }
    int* d = s_item[slot];
    if (list < 0) { d[0] = -1; return; }
    const int nb = (N + kKV - 1) / kKV;
    const bool sorted = Hkv <= kMaxSortedHeads;
    // A list walks its pairs one after the other, late (long) query tiles first.
    const DivMod rq = divmod_small((int)sq, n_qtiles);
    const int round = rq.q;
    const int qt = n_qtiles - 1 - rq.r;
    const int pos = round * 8 + ((round & 1) ? 7 - list : list);   // position in the sorted list
    // sorted list: kv heads by rank; per kv head, batch-major, then the query heads of its group
    const DivMod ph = divmod_small(pos, per_head);   // (kv head rank, place inside the head's pairs)
    const DivMod bg = divmod_small(ph.r, group);     // (batch row, query head inside the group)
    const int hk = sorted ? s_head_of_rank[ph.q] : ph.q;
    const int b = bg.q;
    const int hq = hk * group + bg.r;
    const int ns = sorted ? s_ns[hk] : (int)max((int64_t)0, min((int64_t)nb, ap->sink_blocks[hk]));
    const int nl = sorted ? s_nl[hk] : (int)max((int64_t)0, min((int64_t)nb, ap->local_blocks[hk]));
    const int mb0 = kQBlocks * qt;                              // first query block of the group
    const int mbl = min(kQBlocks * qt + kQBlocks - 1, nb - 1);  // last one that exists
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
    int band_rot = 0;
    if (n_band > 0) {
      band_rot = n_band - divmod_small(lo2, n_band).r;   // in [1, n_band]
      if (band_rot == n_band) band_rot = 0;
    }
    d[0] = n_tiles; d[1] = qt; d[2] = ns; d[3] = nl; d[4] = lo2; d[5] = n_sink; d[6] = n_band; d[7] = band_rot;
    const uint64_t kb = (uint64_t)(ap->k + b * ap->ks.b + hk * ap->ks.h);
    const uint64_t vb = (uint64_t)(ap->v + b * ap->vs.b + hk * ap->vs.h);
    const uint64_t qb = (uint64_t)(ap->q + b * ap->qs.b + hq * ap->qs.h);
    const uint64_t ob = (uint64_t)(ap->o + b * ap->os.b + hq * ap->os.h);
    d[8] = (int)(uint32_t)kb; d[9] = (int)(uint32_t)(kb >> 32); d[10] = (int)(uint32_t)vb; d[11] = (int)(uint32_t)(vb >> 32);
    d[12] = (int)(uint32_t)qb; d[13] = (int)(uint32_t)(qb >> 32); d[14] = (int)(uint32_t)ob; d[15] = (int)(uint32_t)(ob >> 32);
  };
  __syncthreads();   // the sorted heads
  if (threadIdx.x == 0) take(0);
  __syncthreads();

  // An item as the waves see it.
  struct Item {
    int n_tiles, qt, ns, nl, lo2, n_sink, n_band, band_rot;
    const uint16_t *kbase, *vbase, *qbase;
    uint16_t* obase;
  };
  auto read_item = [&](int slot) __attribute__((always_inline)) {
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    const i32x4* p = reinterpret_cast<const i32x4*>(s_item[slot]);
    const i32x4 a = p[0], b = p[1], c = p[2], e = p[3];
    auto u = [](int x) __attribute__((always_inline)) { return __builtin_amdgcn_readfirstlane(x); };
    Item it;
    it.n_tiles = u(a.x); it.qt = u(a.y); it.ns = u(a.z); it.nl = u(a.w);
    it.lo2 = u(b.x); it.n_sink = u(b.y); it.n_band = u(b.z); it.band_rot = u(b.w);
    auto ptr = [&](int lo, int hi) __attribute__((always_inline)) {
      return ((uint64_t)(uint32_t)u(hi) << 32) | (uint64_t)(uint32_t)u(lo);
    };
    it.kbase = (const uint16_t*)ptr(c.x, c.y);
    it.vbase = (const uint16_t*)ptr(c.z, c.w);
    it.qbase = (const uint16_t*)ptr(e.x, e.y);
    it.obase = (uint16_t*)ptr(e.z, e.w);
    return it;
  };
  // Scalar schedule.  The tile order is piecewise consecutive (sinks, then the band from its
  // rotated start, wrapping once), so the tile of the next step follows from the current one with a
  // few scalar instructions; a step past the last tile repeats the last tile.
  auto first_tile = [&](const Item& it) __attribute__((always_inline)) {
    return it.n_sink > 0 ? 0 : it.lo2 + it.band_rot;
  };
  auto next_tile_of = [&](const Item& it, int j, int t_next) __attribute__((always_inline)) {
    int jn = j + 1;
    jn = (jn > it.lo2 + it.n_band - 1) ? it.lo2 : jn;
    jn = (t_next == it.n_sink) ? it.lo2 + it.band_rot : jn;
    return (t_next >= it.n_tiles) ? j : jn;
  };
  for (int par = 0;; par ^= 1) {
  const Item it = read_item(par);
  const int n_tiles = it.n_tiles;
  if (n_tiles < 0) break;

  // what the waves need of the arguments, read again for every item (the pointer is opaque to the compiler)
  PrefillArgsPtr ap = a0;
  asm volatile("" : "+s"(ap));
  const int64_t qs_n = ap->qs.n, ks_n = ap->ks.n, vs_n = ap->vs.n, os_n = ap->os.n;
  const int N = ap->N;
  const float scale_log2_signed = ap->scale_log2_signed;
  // The row maximum is taken over the unscaled scores, which needs a scale >= 0: a negative softmax
  // scale is moved into Q (sign bits of the packed 16-bit elements flipped, exact) and its magnitude kept.
  const float scale_log2 = __builtin_fabsf(scale_log2_signed);
  const uint32_t q_sign = scale_log2_signed < 0.f ? 0x80008000u : 0u;
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));   // per-lane constants are formed again per item instead of living in registers across items
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int grp = wave >> 2;    // 0: group A, 1: group B (one phase behind A)
  const int mcol = lane & 31;   // query row inside the wave's 32 (the MFMA column)
  const int g = lane >> 5;      // half-wave
  const int nb = (N + kKV - 1) / kKV;

  const int mbw = kQBlocks * it.qt + (wave >> 1);             // this wave's query block
  const bool wave_has_rows = mbw < nb;
  // this wave's own live set
  const int w_hi1 = min(it.ns - 1, mbw);
  const int w_lo2 = max(0, mbw + 1 - it.nl);
  auto live_tile = [&](int j) __attribute__((always_inline)) { return wave_has_rows && (j <= w_hi1 || (j >= w_lo2 && j <= mbw)); };
  const int row0 = it.qt * kQRows + wave * kWRows;            // first query row of this wave
  const int64_t m_glob = row0 + mcol;                          // this lane's query row

  // the Q rows are asked for first: theirs is the longest way (the other loads of an item were started by
  // the item before it)
  u32x4 qf[KS];              // Q fragment (B operand): Q[m][16*ks + 8*g .. +7]
  if (n_tiles > 0) {
    const uint16_t* qrow = it.qbase + m_glob * qs_n + 8 * g;
    const bool ok = m_glob < N;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      u32x4 z = {0, 0, 0, 0};
      qf[s] = ok ? *reinterpret_cast<const u32x4*>(qrow + 16 * s) : z;
    }
  }

  // ---- async tile copies: wave w, copy i fills chunks [(w*LPW+i)*64, +64) of a stage --------
  const uint16_t* const kbase = it.kbase;   // uniform
  const uint16_t* const vbase = it.vbase;
  uint32_t koff[LPW], voff[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int L = (wave * LPW + i) * 64 + lane;     // chunk position inside the stage
    const int row = L / CPR, pos = L % CPR;
    koff[i] = 2u * ((uint32_t)(row * ks_n) + (uint32_t)((pos ^ ((row / RSH) % CPR)) * 8));   // bytes
    voff[i] = 2u * ((uint32_t)(row * vs_n) + (uint32_t)((pos ^ (4 * ((row / RSH) % (CPR / 4)))) * 8));
  }
  // rows >= N of the ragged last tile repeat row N-1: their scores are masked, their softmax
  // weight is exactly 0, and a repeated real row is finite
  // a tile is 64 rows: its byte offset inside the head fits 32 bits (checked on the host)
  const uint32_t k_tile_bytes = (uint32_t)(2 * kKV * ks_n), v_tile_bytes = (uint32_t)(2 * kKV * vs_n);
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
  const uint32_t k_dst0 = lds_address(s_k) + wave * LPW * 1024;      // this wave's share of stage 0
  const uint32_t v_dst0 = lds_address(s_v) + wave * LPW * 1024;
  // Starts the first copies, K(0..S-2) and V(0..S-3), of item ni into the stages from ring offset r0 on.
  auto start_copies = [&](const Item& ni, uint32_t r0) __attribute__((always_inline)) {
    int j = first_tile(ni);
#pragma unroll
    for (int i = 0; i + 1 < S; ++i) {
      issue_tile(ni.kbase, k_tile_bytes, ks_n, koff, true, j, k_dst0 + ((r0 + i * TILE_B) & (kRing - 1)));
      if (i + 2 < S) issue_tile(ni.vbase, v_tile_bytes, vs_n, voff, false, j, v_dst0 + ((r0 + i * TILE_B) & (kRing - 1)));
      j = next_tile_of(ni, j, i + 1);
    }
  };
  constexpr int kPrefetchOps = (2 * S - 3) * LPW + 1;   // vector memory operations prefetch_next starts
  // The item after this one (its descriptor is in the other slot): its first copies go out now, and one load per
  // lane touches both cache lines of each of its Q rows so that the real Q loads of the next pass hit in L2.
  // The touched word lands in q_touch, which is kept allocated until the next pass has waited for it.
  auto prefetch_next = [&](uint32_t r0) __attribute__((always_inline)) {
    const Item ni = read_item(par ^ 1);
    if (ni.n_tiles <= 0) return false;
    start_copies(ni, r0);
    const int64_t m_row = min((int64_t)ni.qt * kQRows + wave * kWRows + mcol, (int64_t)N - 1);
    const uint16_t* qrow = ni.qbase + m_row * qs_n + (D / 2) * g;
    asm volatile("global_load_dword %0, %1, off" : "=v"(q_touch) : "v"(qrow) : "memory");
    return true;
  };

  // operand read addresses of this lane: LDS byte address of its row in the stage at the ring position; stage,
  // half and k-step go into the instruction's immediate offset, so the matrix phase needs no VALU work
  uint32_t k_ad[KS], v_ad[DT];
  {
    const uint32_t k_rd = (uint32_t)(mcol * ROW_B) | (uint32_t)(((g ^ ((mcol / RSH) % CPR)) & (CPR - 1)) * 16);
#pragma unroll
    for (int s = 0; s < KS; ++s) k_ad[s] = lds_address(s_k) + rst + (k_rd ^ (uint32_t)(32 * s));
    const int grp16 = lane & 15;
    const int dhalf = (lane >> 4) & 1;
    const int v_row = 4 * g + (grp16 >> 2);
    const uint32_t v_rd = (uint32_t)(v_row * ROW_B) +
                          (uint32_t)(((2 * dhalf + ((grp16 & 3) >> 1)) ^ (4 * ((v_row / RSH) % (CPR / 4)))) * 16 +
                                     8 * (grp16 & 1));
    // V trails K by one step
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) v_ad[dt] = lds_address(s_v) + ((rst - TILE_B) & (kRing - 1)) + (v_rd ^ (uint32_t)(64 * dt));
  }
  int kd_prev = (rst == 0) ? -(kStages - 1) * TILE_B : TILE_B;   // how far the K read addresses moved in the previous step

  if (n_tiles == 0) {   // nothing is visible from this query tile: zeros (nobody prefetches for such an item)
    if (threadIdx.x == 0) take(par ^ 1);
    if (wave_has_rows && m_glob < N) {
      uint16_t* orow = it.obase + m_glob * os_n;
      u32x2 z = {0, 0};
#pragma unroll
      for (int i = 0; i < D / 8; ++i) *reinterpret_cast<u32x2*>(orow + 8 * i + 4 * g) = z;
    }
    __syncthreads();   // the next descriptor, written by thread 0 above
    prefetched = false;
    continue;
  }
  if (!prefetched) start_copies(it, rst);
  // the item after this one: thread 0 works its descriptor out kTakeLead iterations before this item's last
  // one (every wave sees it after the next barrier), or here when the item is that short
  constexpr int kTakeLead = 6;
  const int t_take = n_tiles - kTakeLead;
  if (threadIdx.x == 0 && t_take < 1) take(par ^ 1);

  int jt[S];   // tiles of steps t .. t+S-1
  jt[0] = first_tile(it);
#pragma unroll
  for (int i = 1; i < S; ++i) jt[i] = next_tile_of(it, jt[i - 1], i);

  // the zero the accumulators start from is formed per item (a register full of zeros that the compiler
  // keeps across items costs more than it saves)
  float zero = 0.f;
  asm volatile("" : "+v"(zero));
  f32x16 oacc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[t][i] = zero;
  f32x16 st[2];              // S^T of the current tile (defined on every path: an undefined one is carried from item to item)
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int i = 0; i < 16; ++i) st[nt][i] = zero;
  uint32_t pf[16];           // P^T of the current tile, packed pairs, B-operand order
#pragma unroll
  for (int i = 0; i < 16; ++i) pf[i] = __builtin_bit_cast(uint32_t, zero);
  float m_run = -INFINITY;   // reference exponent of exp2: an integer, ceil of the row max of scale_log2 * s when it was last set; a later max may pass it by < 8
  float l_run = 0.f;         // this lane's share of the running sum (the lane+32 twin holds the rest)

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
  // P.V only (the last iteration)
  auto pv_phase = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int tk = 0; tk < 4; ++tk) {
      u32x4 vf[DT];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const u32x2 lo = lds_load_tr16(v_ad[dt], (16 * tk) * ROW_B);
        const u32x2 hi = lds_load_tr16(v_ad[dt], (16 * tk + 8) * ROW_B);
        vf[dt] = u32x4{lo.x, lo.y, hi.x, hi.y};
      }
      const u32x4 bfrag = {pf[4 * tk], pf[4 * tk + 1], pf[4 * tk + 2], pf[4 * tk + 3]};
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) oacc[dt] = T::mfma(vf[dt], bfrag, oacc[dt]);
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

  // Iteration t: matrix phase = P.V of tile t-1 and Q.K^T of tile t, then softmax phase = tile t.
  // There is one work-group barrier per iteration; group A meets it after its softmax phase, group
  // B after its matrix phase, so B's softmax of tile t runs beside A's matrix phase of tile t+1 and
  // each SIMD holds one wave in either phase.  A wave for which tile t-1 or t is not live still
  // runs the whole matrix phase (with P = 0, or ignoring S), which keeps the loop body a single
  // straight block; it skips the phase when neither is live.  The copies started in iteration t
  // overwrite the stages of K(t-1) and V(t-2), which every wave has finished reading before
  // barrier t-1; the copies started two iterations ago (K(t+1), V(t)) are first read after barrier
  // t, and every wave waits for its own before it.  Iteration n_tiles only finishes P.V of the
  // last tile and starts the next item.
  bool lc_prev = false;        // was tile t-1 live for this wave
  constexpr int n_wait = (S - 2) * 2 * LPW;   // copies started in the last S-2 iterations may still be in flight
  auto advance = [&]() __attribute__((always_inline)) {
    // the operand addresses move to the next stages (K: t+1, V: t)
    const int kd = (rst == (kStages - 1) * TILE_B) ? -(kStages - 1) * TILE_B : TILE_B;
#pragma unroll
    for (int s = 0; s < KS; ++s) k_ad[s] += kd;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) v_ad[dt] += kd_prev;   // V trails K by one step
    kd_prev = kd;
    rst = (rst + TILE_B) & (kRing - 1);
    cst = (cst + TILE_B) & (kRing - 1);
  };
  auto iteration = [&](int t, auto FIRST) __attribute__((always_inline)) {
    constexpr bool kFirst = decltype(FIRST)::value != 0;
    // ---------------- matrix phase ----------------
    issue_tile(kbase, k_tile_bytes, ks_n, koff, true, jt[S - 1], k_dst0 + cst);
    issue_tile(vbase, v_tile_bytes, vs_n, voff, false, jt[S - 2], v_dst0 + ((cst - TILE_B) & (kRing - 1)));
    const bool lp = lc_prev, lc = live_tile(jt[0]);
    if (kFirst) {
      if (lc) qk_phase();
    } else {
      if (lp || lc) matrix_phase();
    }
    if (grp == 1) { wait_vm(n_wait); phase_barrier(); }
    // ---------------- softmax phase ----------------
    if (lc) {
      softmax(jt[0]);
    } else if (lp) {   // the next matrix phase this wave runs must add nothing for a dead tile
#pragma unroll
      for (int i = 0; i < 16; ++i) pf[i] = 0;
    }
    advance();
    lc_prev = lc;
#pragma unroll
    for (int i = 0; i + 1 < S; ++i) jt[i] = jt[i + 1];
    jt[S - 1] = next_tile_of(it, jt[S - 1], t + S);
    if (grp == 0) { wait_vm(n_wait); phase_barrier(); }
  };
  wait_vm(0);
  // the Q loads have landed too; pin that fact here so that the compiler does not put its own
  // vmcnt(0) wait at their first use inside the loop, where it would also wait for the copies
#pragma unroll
  for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));
#pragma unroll
  for (int s = 0; s < KS; ++s) qf[s] ^= u32x4{q_sign, q_sign, q_sign, q_sign};
  asm volatile("" : "+v"(q_touch));   // the touch of the previous pass has landed as well
  phase_barrier();               // K(0..2) and V(0..1) are in LDS
  iteration(0, IC<1>{});   // no P.V yet (and no V stage to read)
  {
    int t = 1;
    for (; t < t_take; ++t) iteration(t, IC<0>{});
    if (threadIdx.x == 0 && t_take >= 1) take(par ^ 1);
    for (; t < n_tiles; ++t) iteration(t, IC<0>{});
  }

  // ---- iteration n_tiles: P.V of the last tile; the next item's first copies start here.
  // Every K stage is free by now (K(n_tiles-1) was read before the last barrier) and so are the V
  // stages other than V(n_tiles-1)'s; the next item's tile u goes where this ring position + 1 + u
  // points, which is where its iterations will look for it.  The repeated copies of the last steps
  // may still be under way into those stages: a wave's copies land in the order they were started.
  prefetched = prefetch_next((rst + TILE_B) & (kRing - 1));
  if (lc_prev) pv_phase();
  if (grp == 1) phase_barrier();
  advance();
  if (grp == 0) phase_barrier();

  // ---- epilogue: O[m][d] = O^T[d][m] / l, written as whole rows ---------------------------------
  // A lane holds 8-byte pieces of one row; stored as they are, a wave's store touches 32 rows with 16 bytes
  // each.  The rows go through LDS instead, 16 at a time, into this wave's quarter of one of the two V
  // stages that are free now (V(n_tiles-1)'s, which every wave has finished reading at the barrier above, and
  // the one after it; the next item's V(0), V(1) are in the other two), 16-byte chunks XOR-permuted like the
  // K tiles; then 16 lanes store one row of 2 D bytes.  The repeated copies of the last two iterations may
  // still be under way into these stages: they are older than everything prefetch_next started.
  if (prefetched) wait_vm_exact<kPrefetchOps>(); else wait_vm(0);
  {
    const float l_tot = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = (l_tot > 0.f) ? 1.f / l_tot : 0.f;
    const uint32_t stage = (rst + (2 + (wave >> 2)) * TILE_B) & (kRing - 1);
    const uint32_t slice = lds_address(s_v) + stage + (wave & 3) * (TILE_B / 4);
    const int wrow = mcol & 15;
    const uint32_t wr = slice + wrow * ROW_B + 8 * g;
    const uint32_t wswz = (uint32_t)((wrow / RSH) % CPR);
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if ((mcol >> 4) == r) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int gi = 0; gi < 4; ++gi) {
            u32x2 w;
            w.x = T::pack_rne(oacc[dt][4 * gi + 0] * inv, oacc[dt][4 * gi + 1] * inv);
            w.y = T::pack_rne(oacc[dt][4 * gi + 2] * inv, oacc[dt][4 * gi + 3] * inv);
            lds_store8(wr + ((uint32_t)(4 * dt + gi) ^ wswz) * 16, w);
          }
      }
      constexpr int kReads = 16 * CPR / 64;   // 16 rows of CPR chunks, 64 lanes
      u32x4 rowv[kReads];
#pragma unroll
      for (int i = 0; i < kReads; ++i) {
        const int idx = i * 64 + lane;
        const int row = idx / CPR, c = idx % CPR;
        rowv[i] = lds_load16(slice + row * ROW_B + ((uint32_t)c ^ (uint32_t)((row / RSH) % CPR)) * 16, 0);
      }
#pragma unroll
      for (int i = 0; i < kReads; ++i) {
        const int idx = i * 64 + lane;
        const int row = idx / CPR, c = idx % CPR;
        const int64_t m_out = row0 + 16 * r + row;
        if (wave_has_rows && m_out < N) *reinterpret_cast<u32x4*>(it.obase + m_out * os_n + 8 * c) = rowv[i];
      }
    }
  }
  }   // item loop
  // the last work-group to leave clears the queue for the next launch that uses this slot
  if (threadIdx.x == 0) {
    PrefillQueue* queue = a0->queue;
    const unsigned d = atomicAdd(&queue->done, 1u);
    if (d == gridDim.x - 1) {
      for (int x = 0; x < 8; ++x) atomicExch(&queue->next[x], 0u);
      atomicExch(&queue->done, 0u);
    }
  }
}

template <int D, int S>
static size_t prefill_lds_bytes() {
  return (size_t)2 * S * kKV * D * sizeof(uint16_t);   // K stages + V stages
}

// A queue slot for one launch (round robin over the slots) and the number of CUs of the current device.
static int prefill_queue(PrefillQueue** out, int* cus) {
  static PrefillQueue* base_of_device[kMaxDevices] = {};
  static int cus_of_device[kMaxDevices] = {};
  static std::atomic<unsigned> turn{0};
  static std::mutex mu;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MOA_ERR_LAUNCH, "moa_prefill_fwd: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: device %d", dev);
  {
    std::lock_guard<std::mutex> lock(mu);
    if (!base_of_device[dev]) {
      void* p = nullptr;
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_prefill_queues));
      if (e != hipSuccess || !p) return fail(MOA_ERR_LAUNCH, "moa_prefill_fwd: hipGetSymbolAddress: %s", hipGetErrorString(e));
      int n = 0;
      e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
      if (e != hipSuccess || n <= 0) return fail(MOA_ERR_LAUNCH, "moa_prefill_fwd: cannot read the CU count");
      cus_of_device[dev] = n;
      base_of_device[dev] = reinterpret_cast<PrefillQueue*>(p);
    }
  }
  *out = base_of_device[dev] + (turn.fetch_add(1) % kQueueSlots);
  *cus = cus_of_device[dev];
  return MOA_OK;
}

template <typename T, int D>
static int launch_prefill(const void* q, const void* k, const void* v, void* o, const int64_t* qs,
                          const int64_t* ks, const int64_t* vs, const int64_t* os, int B, int Hq,
                          int Hkv, int N, const int64_t* sink_blocks, const int64_t* local_blocks,
                          float sm_scale, hipStream_t st) {
  constexpr int NW = 8, S = 4;
  constexpr int kQRows = NW * kWRows;
  const int n_qtiles = (N + kQRows - 1) / kQRows;
  const int64_t pairs = (int64_t)B * Hq;
  const int64_t items = pairs * n_qtiles;
  // the queue's ticket arithmetic (divmod_small) is exact below 2^22: tickets of one XCD's list (an eighth
  // of the items) and positions in the list of (batch, head) pairs
  if (items > (1LL << 25) || pairs > (1LL << 22) || N > (1 << 28))
    return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: too many work items");
  const int BH = (int)pairs;
  // the async copies address a tile row through a 32-bit element offset
  if (64 * ks[2] + D >= (1ll << 31) || 64 * vs[2] + D >= (1ll << 31))
    return fail(MOA_ERR_UNSUPPORTED, "moa_prefill_fwd: k/v token stride too large");
  Strides4 sq = {qs[0], qs[1], qs[2]}, sk = {ks[0], ks[1], ks[2]}, sv = {vs[0], vs[1], vs[2]},
           so = {os[0], os[1], os[2]};
  const size_t lds = prefill_lds_bytes<D, S>();
  static bool lds_reserved[kMaxDevices] = {};   // per template instance
  if (int rc = reserve_lds(reinterpret_cast<const void*>(&prefill_kernel<T, D>), lds, lds_reserved, "moa_prefill_fwd"))
    return rc;
  PrefillQueue* queue = nullptr;
  int cus = 0;
  if (int rc = prefill_queue(&queue, &cus)) return rc;
  const int64_t groups = items < cus ? items : cus;
  PrefillArgs args;
  args.q = (const uint16_t*)q; args.k = (const uint16_t*)k; args.v = (const uint16_t*)v; args.o = (uint16_t*)o;
  args.qs = sq; args.ks = sk; args.vs = sv; args.os = so;
  args.sink_blocks = sink_blocks; args.local_blocks = local_blocks; args.queue = queue;
  args.BH = BH; args.Hq = Hq; args.group = Hq / Hkv; args.N = N; args.n_qtiles = n_qtiles;
  args.per_head = B * (Hq / Hkv); args.Hkv = Hkv;
  args.scale_log2_signed = mfma_softmax_scale(sm_scale);
  hipLaunchKernelGGL((prefill_kernel<T, D>), dim3((unsigned)groups), dim3(NW * 64), lds, st, args);
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
