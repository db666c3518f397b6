// Circular KV-cache kernels: one-token append and prompt bulk insert.
//
// Both restate, per (batch row, head), the index arithmetic of the reference's
// StaticCircularCache.update (MoA/attention/cache_utils.py:1020-1058 decode
// branch, :1060-1164 prefill branch) and move the K/V rows with 128-bit
// accesses.  They are HBM/latency bound integer + byte work: no LDS, no MFMA.
//
// Layout: kc/vc are [B, sumC, D] contiguous; head h of row b owns rows
// [head_start, head_start + cache_size) of that row's sumC; the first
// static_size rows are the sink part, the rest is the ring that starts at
// circ_head[h] and has circ_size[h] rows.
#include "moa_common.h"

namespace moa {

constexpr int kRowLanes = 16;                    // lanes that move one K/V row
constexpr int kCacheThreads = 256;
constexpr int kRowsPerBlock = kCacheThreads / kRowLanes;

__device__ __forceinline__ void copy_row16(const char* __restrict__ src, char* __restrict__ dst,
                                           int units, int lane) {
  for (int u = lane; u < units; u += kRowLanes) {
    u32x4 x = *reinterpret_cast<const u32x4*>(src + (size_t)u * 16);
    *reinterpret_cast<u32x4*>(dst + (size_t)u * 16) = x;
  }
}

// ---------------------------------------------------------------------------
// Decode-step append (cache_utils.py:1020-1058)
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kCacheThreads) void cache_append_kernel(
    const char* __restrict__ k_new, const char* __restrict__ v_new,
    int64_t kn_sb, int64_t kn_sh, int64_t vn_sb, int64_t vn_sh,  // byte strides
    char* __restrict__ kc, char* __restrict__ vc, int64_t* __restrict__ mask_cache,
    int64_t* __restrict__ update_index, int64_t* __restrict__ valid_len,
    const int64_t* __restrict__ circ_head, const int64_t* __restrict__ circ_size,
    const int64_t* __restrict__ static_size, const int64_t* __restrict__ max_len,
    int64_t kv_len, int B, int H, int row_bytes, int64_t sumC) {
  const int lane = threadIdx.x % kRowLanes;
  const int64_t bh = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kRowLanes;
  if (bh >= (int64_t)B * H) return;
  const int b = (int)(bh / H);
  const int h = (int)(bh % H);

  const int64_t idx = update_index[bh];
  const bool in_range = idx >= 0 && idx < sumC;
  if (in_range && kc != nullptr) {
    const int units = row_bytes / 16;
    const size_t dst = ((size_t)b * sumC + idx) * row_bytes;
    copy_row16(k_new + b * kn_sb + h * kn_sh, kc + dst, units, lane);
    copy_row16(v_new + b * vn_sb + h * vn_sh, vc + dst, units, lane);
  }
  if (lane == 0) {
    if (in_range && mask_cache != nullptr) mask_cache[(size_t)b * sumC + idx] = 1;
    const int64_t vl = valid_len[bh];
    valid_len[bh] = vl + (vl < max_len[h] ? 1 : 0);
    const bool is_circular = (kv_len + 1) > static_size[h];
    int64_t next = idx + 1;
    if (is_circular) {
      const int64_t ch = circ_head[h];
      next = py_mod(idx + 1 - ch, circ_size[h]) + ch;
    }
    update_index[bh] = next;
  }
}

// ---------------------------------------------------------------------------
// Prompt bulk insert (cache_utils.py:1060-1164)
// ---------------------------------------------------------------------------
struct HeadRing {
  int64_t upd0;   // cache_update_index before the call
  int64_t ch;     // first ring row
  int64_t csz;    // ring rows
  int64_t s;      // static_cache_size
  int64_t kv0;    // _kv_len before the call
};

// Slot of the token whose advancing position is `a` (:1088-1107).
__device__ __forceinline__ int64_t slot_of(const HeadRing& g, int64_t a) {
  const bool circ = (g.kv0 + a) > g.s;
  return circ ? py_mod(g.upd0 + a - g.ch, g.csz) + g.ch : g.upd0 + a;
}

// Keep rule (:1122-1133) without the mask term.
__device__ __forceinline__ bool keep_of(const HeadRing& g, int64_t slot, int64_t rap) {
  return (rap <= g.csz) || (slot < g.ch);
}

// Candidate r -> the token with advancing position a (its index among the row's valid tokens; without a
// mask every token is valid and a is the token's position).  Only tokens that can be kept are
// enumerated: r < csz walks the valid tokens from the last one backwards (these have
// rap = r+1 <= csz); r >= csz walks the first ones (the only ones whose slot can lie in the static
// part); any other token is a ring token older than the last csz and is dropped by the keep rule.
// n_valid: valid tokens of the batch row.  Returns whether the candidate is kept, with a and its slot.
__device__ __forceinline__ bool candidate(const HeadRing& g, int64_t r, int64_t n_valid, int64_t& a, int64_t& slot) {
  if (r < g.csz) {
    a = n_valid - 1 - r;
    if (a < 0) return false;
  } else {
    a = r - g.csz;
    if (a >= n_valid - g.csz || a > g.s) return false;
  }
  const int64_t rap = n_valid - a;   // valid tokens at or after this one (:1081-1086)
  slot = slot_of(g, a);
  return keep_of(g, slot, rap);
}
// how many candidates a head has
__device__ __forceinline__ int64_t candidate_count(const HeadRing& g, int64_t n_valid) {
  return min(n_valid, g.csz + g.s + 1);
}

__device__ __forceinline__ HeadRing load_ring(const int64_t* update_index, const int64_t* circ_head,
                                              const int64_t* circ_size, const int64_t* static_size,
                                              int64_t kv_len, int64_t bh, int h) {
  HeadRing g;
  g.upd0 = update_index[bh];
  g.ch = circ_head[h];
  g.csz = circ_size[h];
  g.s = static_size[h];
  g.kv0 = kv_len;
  return g;
}

// With an attention mask: the positions of a batch row's valid tokens (mask == 1) in order,
// tok_of[b, a] = position of the a-th valid token, and their number n_valid[b].  This is the inverse of
// the reference's advancing_pos = cumsum(mask) - 1 (:1075-1080); its reversed_advancing_pos of a valid
// token is n_valid - a (:1081-1086).  One work-group per batch row; every wave owns a contiguous segment
// of the row and walks it twice, a lane looking at four consecutive tokens per step: first to count its
// valid tokens (independent loads, nothing waits on LDS), then, once the waves' totals have met in LDS
// (the only barrier), to write the positions from its offset on (ballots and population counts give a
// lane the number of valid tokens in front of its four).
constexpr int kScanThreads = 1024;
__global__ __launch_bounds__(kScanThreads) void mask_compact_kernel(const int64_t* __restrict__ am,
                                                                     int64_t am_stride, int S,
                                                                     int32_t* __restrict__ tok_of,
                                                                     int32_t* __restrict__ n_valid) {
  constexpr int kWaves = kScanThreads / 64;
  __shared__ int s_wave[kWaves];
  const int b = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t* row = am + (int64_t)b * am_stride;
  int32_t* out = tok_of + (int64_t)b * S;
  constexpr int kPerLane = 4;              // consecutive tokens a lane looks at per step
  constexpr int kStep = 64 * kPerLane;
  const int seg = ((S + kWaves - 1) / kWaves + kStep - 1) / kStep * kStep;   // tokens per wave, whole steps
  const int t_begin = min(S, wave * seg), t_end = min(S, t_begin + seg);
  int mine = 0;
#pragma unroll 4
  for (int t0 = t_begin; t0 < t_end; t0 += kStep) {
    const int t = t0 + kPerLane * lane;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) mine += (t + j < t_end && row[t + j] == 1) ? 1 : 0;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off, 64);
  if (lane == 0) s_wave[wave] = mine;
  __syncthreads();
  int base = 0, total = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const int c = s_wave[w];
    base += (w < wave) ? c : 0;
    total += c;
  }
  const unsigned long long below = (1ull << lane) - 1ull;
  for (int t0 = t_begin; t0 < t_end; t0 += kStep) {
    const int t = t0 + kPerLane * lane;
    bool valid[kPerLane];
    int before = 0, step_total = 0;   // valid tokens of lower lanes; of the whole step
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
      valid[j] = t + j < t_end && row[t + j] == 1;
      const unsigned long long bal = __ballot(valid[j]);
      before += __popcll(bal & below);
      step_total += __popcll(bal);
    }
    int at = base + before;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
      if (valid[j]) out[at] = t + j;
      at += valid[j] ? 1 : 0;
    }
    base += step_total;
  }
  if (tid == 0) n_valid[b] = total;
}

constexpr int kRowsPerThread = 4;   // rows a group of 16 lanes moves: all loads go out before the first store

__global__ __launch_bounds__(kCacheThreads) void cache_prefill_copy_kernel(
    const char* __restrict__ k, const char* __restrict__ v,
    int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,  // bytes
    char* __restrict__ kc, char* __restrict__ vc, int64_t* __restrict__ mask_cache,
    const int64_t* __restrict__ update_index, const int64_t* __restrict__ circ_head,
    const int64_t* __restrict__ circ_size, const int64_t* __restrict__ static_size,
    const int32_t* __restrict__ tok_of, const int32_t* __restrict__ n_valid, int64_t kv_len, int H, int S,
    int row_bytes, int64_t sumC) {
  const int lane = threadIdx.x % kRowLanes;
  const int h = blockIdx.y;
  const int b = blockIdx.z;
  const int64_t bh = (int64_t)b * H + h;
  const HeadRing g = load_ring(update_index, circ_head, circ_size, static_size, kv_len, bh, h);
  const int64_t nv = n_valid ? (int64_t)n_valid[b] : (int64_t)S;
  const int64_t r0 = (int64_t)blockIdx.x * (kRowsPerBlock * kRowsPerThread) + threadIdx.x / kRowLanes;
  if ((int64_t)blockIdx.x * (kRowsPerBlock * kRowsPerThread) >= candidate_count(g, nv)) return;
  const char* src_k[kRowsPerThread];
  const char* src_v[kRowsPerThread];
  size_t dst[kRowsPerThread];
  bool keep[kRowsPerThread];
#pragma unroll
  for (int j = 0; j < kRowsPerThread; ++j) {
    int64_t a, slot;
    keep[j] = candidate(g, r0 + j * kRowsPerBlock, nv, a, slot) && slot >= 0 && slot < sumC;
    const int64_t t = keep[j] ? (tok_of ? (int64_t)tok_of[(int64_t)b * S + a] : a) : 0;
    src_k[j] = k + b * k_sb + h * k_sh + t * k_ss;
    src_v[j] = v + b * v_sb + h * v_sh + t * v_ss;
    dst[j] = keep[j] ? ((size_t)b * sumC + slot) * row_bytes : 0;
    if (keep[j] && lane == 0 && mask_cache != nullptr) mask_cache[(size_t)b * sumC + slot] = 1;
  }
  if (kc == nullptr) return;
  const int units = row_bytes / 16;
  for (int u = lane; u < units; u += kRowLanes) {
    u32x4 xk[kRowsPerThread], xv[kRowsPerThread];
#pragma unroll
    for (int j = 0; j < kRowsPerThread; ++j)
      if (keep[j]) {
        xk[j] = *reinterpret_cast<const u32x4*>(src_k[j] + (size_t)u * 16);
        xv[j] = *reinterpret_cast<const u32x4*>(src_v[j] + (size_t)u * 16);
      }
#pragma unroll
    for (int j = 0; j < kRowsPerThread; ++j)
      if (keep[j]) {
        *reinterpret_cast<u32x4*>(kc + dst[j] + (size_t)u * 16) = xk[j];
        *reinterpret_cast<u32x4*>(vc + dst[j] + (size_t)u * 16) = xv[j];
      }
  }
}

// One thread per (b, h): add the number of kept tokens to the valid length, then move the pointer
// (:1110, :1136-1138).  Runs after the copy kernel on the same stream because it overwrites
// update_index, which the copy kernel reads.  The count has a closed form in the candidates' terms:
// the last min(csz, n_valid) valid tokens have rap <= csz and are all kept; of the earlier ones
// (a < n_valid - csz, so rap > csz) exactly those are kept whose slot lies in front of the ring, which
// needs a non-circular slot (kv0 + a <= s, then slot = upd0 + a) below the ring's first row.
__global__ __launch_bounds__(256) void cache_prefill_index_kernel(
    int64_t* __restrict__ update_index, int64_t* __restrict__ valid_len,
    const int64_t* __restrict__ circ_head, const int64_t* __restrict__ circ_size,
    const int64_t* __restrict__ static_size, const int32_t* __restrict__ n_valid, int64_t kv_len, int B, int H,
    int S) {
  const int64_t bh = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (bh >= (int64_t)B * H) return;
  const int b = (int)(bh / H);
  const int h = (int)(bh % H);
  const HeadRing g = load_ring(update_index, circ_head, circ_size, static_size, kv_len, bh, h);
  const int64_t nv = n_valid ? (int64_t)n_valid[b] : (int64_t)S;
  const int64_t recent = min(g.csz, nv);
  const int64_t early = max((int64_t)0, min(min(nv - g.csz, g.s + 1), min(g.s - g.kv0 + 1, g.ch - g.upd0)));
  update_index[bh] = slot_of(g, nv);   // the slot the token after the last valid one would take (:1110)
  valid_len[bh] += recent + early;
}

static int check_rows(const char* who, int D, int dtype, const int64_t* strides, int nstr,
                      const void* p0, const void* p1) {
  const int eb = elem_bytes(dtype);
  if (eb == 0) return fail(MOA_ERR_ARG, "%s: unknown dtype %d", who, dtype);
  if (D <= 0 || (D * eb) % 16 != 0)
    return fail(MOA_ERR_UNSUPPORTED, "%s: head_dim %d * %d bytes is not a multiple of 16", who, D, eb);
  if (strides) {
    if (strides[nstr - 1] != 1) return fail(MOA_ERR_ARG, "%s: innermost stride must be 1", who);
    for (int i = 0; i < nstr - 1; ++i)
      if ((strides[i] * eb) % 16 != 0)
        return fail(MOA_ERR_ARG, "%s: stride %d (%lld elements) breaks 16-byte row alignment", who, i,
                    (long long)strides[i]);
  }
  if (!aligned16(p0) || !aligned16(p1)) return fail(MOA_ERR_ARG, "%s: pointers must be 16-byte aligned", who);
  return MOA_OK;
}

}  // namespace moa

using namespace moa;

extern "C" int moa_cache_append(const void* k_new, const void* v_new, const int64_t* kn_strides,
                                const int64_t* vn_strides, void* kc, void* vc, int64_t* mask_cache,
                                int64_t* update_index, int64_t* valid_len, const int64_t* circ_head,
                                const int64_t* circ_size, const int64_t* static_size,
                                const int64_t* max_len, int64_t kv_len, int B, int H, int D,
                                int64_t sumC, int dtype, void* stream) {
  if (B <= 0 || H <= 0 || sumC <= 0) return fail(MOA_ERR_ARG, "moa_cache_append: B, H, sumC must be positive");
  if (!update_index || !valid_len || !circ_head || !circ_size || !static_size || !max_len)
    return fail(MOA_ERR_ARG, "moa_cache_append: null index array");
  if ((kc == nullptr) != (vc == nullptr))
    return fail(MOA_ERR_ARG, "moa_cache_append: kc and vc must both be set or both be NULL");
  int64_t ksb = 0, ksh = 0, vsb = 0, vsh = 0;
  const int eb = elem_bytes(dtype);
  if (kc != nullptr) {
    if (!k_new || !v_new || !kn_strides || !vn_strides)
      return fail(MOA_ERR_ARG, "moa_cache_append: null k_new/v_new/strides");
    int rc = check_rows("moa_cache_append(k_new)", D, dtype, kn_strides, 3, k_new, kc);
    if (rc) return rc;
    rc = check_rows("moa_cache_append(v_new)", D, dtype, vn_strides, 3, v_new, vc);
    if (rc) return rc;
    ksb = kn_strides[0] * eb; ksh = kn_strides[1] * eb;
    vsb = vn_strides[0] * eb; vsh = vn_strides[1] * eb;
  } else if (eb == 0) {
    return fail(MOA_ERR_ARG, "moa_cache_append: unknown dtype %d", dtype);
  }
  const int64_t n = (int64_t)B * H;
  dim3 grid((unsigned)((n + kRowsPerBlock - 1) / kRowsPerBlock));
  hipLaunchKernelGGL(cache_append_kernel, grid, dim3(kCacheThreads), 0, (hipStream_t)stream,
                     (const char*)k_new, (const char*)v_new, ksb, ksh, vsb, vsh, (char*)kc, (char*)vc,
                     mask_cache, update_index, valid_len, circ_head, circ_size, static_size, max_len,
                     kv_len, B, H, D * eb, sumC);
  return check_launch("moa_cache_append");
}

extern "C" size_t moa_cache_prefill_workspace_bytes(int B, int S) {
  if (B <= 0 || S <= 0) return 0;
  return ((size_t)B * (2 * (size_t)S + 1) * sizeof(int32_t) + 255) & ~(size_t)255;
}

extern "C" int moa_cache_prefill_insert(const void* k, const void* v, const int64_t* k_strides,
                                        const int64_t* v_strides, void* kc, void* vc,
                                        int64_t* mask_cache, int64_t* update_index, int64_t* valid_len,
                                        const int64_t* circ_head, const int64_t* circ_size,
                                        const int64_t* static_size, const int64_t* attention_mask,
                                        int64_t am_stride, void* workspace, size_t workspace_bytes,
                                        int64_t kv_len, int B, int H, int S, int D, int64_t sumC,
                                        int64_t max_cache_size, int dtype, void* stream) {
  if (B <= 0 || H <= 0 || S <= 0 || sumC <= 0)
    return fail(MOA_ERR_ARG, "moa_cache_prefill_insert: B, H, S, sumC must be positive");
  if (H > 65535 || B > 65535) return fail(MOA_ERR_UNSUPPORTED, "moa_cache_prefill_insert: B, H <= 65535");
  if (!update_index || !valid_len || !circ_head || !circ_size || !static_size)
    return fail(MOA_ERR_ARG, "moa_cache_prefill_insert: null index array");
  if ((kc == nullptr) != (vc == nullptr))
    return fail(MOA_ERR_ARG, "moa_cache_prefill_insert: kc and vc must both be set or both be NULL");
  const int eb = elem_bytes(dtype);
  if (eb == 0) return fail(MOA_ERR_ARG, "moa_cache_prefill_insert: unknown dtype %d", dtype);
  int64_t ks[3] = {0, 0, 0}, vs[3] = {0, 0, 0};
  if (kc != nullptr) {
    if (!k || !v || !k_strides || !v_strides)
      return fail(MOA_ERR_ARG, "moa_cache_prefill_insert: null k/v/strides");
    int rc = check_rows("moa_cache_prefill_insert(k)", D, dtype, k_strides, 4, k, kc);
    if (rc) return rc;
    rc = check_rows("moa_cache_prefill_insert(v)", D, dtype, v_strides, 4, v, vc);
    if (rc) return rc;
    for (int i = 0; i < 3; ++i) { ks[i] = k_strides[i] * eb; vs[i] = v_strides[i] * eb; }
  }
  hipStream_t st = (hipStream_t)stream;
  int32_t* tok_of = nullptr;
  int32_t* n_valid = nullptr;
  if (attention_mask != nullptr) {
    const size_t need = moa_cache_prefill_workspace_bytes(B, S);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(MOA_ERR_WORKSPACE, "moa_cache_prefill_insert: workspace %zu < %zu bytes", workspace_bytes, need);
    tok_of = reinterpret_cast<int32_t*>(workspace);
    n_valid = tok_of + (size_t)B * (size_t)S;
    hipLaunchKernelGGL(mask_compact_kernel, dim3(B), dim3(kScanThreads), 0, st, attention_mask, am_stride, S, tok_of,
                       n_valid);
    int rc = check_launch("moa_cache_prefill_insert(mask scan)");
    if (rc) return rc;
  }
  // candidates r >= S never name a token, nor do those past a head's cache size + 1 (see candidate())
  int64_t n_rows = S;
  if (max_cache_size > 0 && max_cache_size + 1 < n_rows) n_rows = max_cache_size + 1;
  if (kc != nullptr || mask_cache != nullptr) {
    constexpr int kPerBlock = kRowsPerBlock * kRowsPerThread;
    dim3 grid((unsigned)((n_rows + kPerBlock - 1) / kPerBlock), (unsigned)H, (unsigned)B);
    hipLaunchKernelGGL(cache_prefill_copy_kernel, grid, dim3(kCacheThreads), 0, st, (const char*)k,
                       (const char*)v, ks[0], ks[1], ks[2], vs[0], vs[1], vs[2], (char*)kc, (char*)vc,
                       mask_cache, (const int64_t*)update_index, circ_head, circ_size, static_size,
                       (const int32_t*)tok_of, (const int32_t*)n_valid, kv_len, H, S, D * eb, sumC);
    int rc = check_launch("moa_cache_prefill_insert(copy)");
    if (rc) return rc;
  }
  const int64_t n = (int64_t)B * H;
  hipLaunchKernelGGL(cache_prefill_index_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                     update_index, valid_len, circ_head, circ_size, static_size, (const int32_t*)n_valid, kv_len, B, H,
                     S);
  return check_launch("moa_cache_prefill_insert(index)");
}
