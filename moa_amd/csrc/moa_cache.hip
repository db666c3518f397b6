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

// Candidate r -> token t.  Without a mask only tokens that can be kept are
// enumerated: r < csz walks the prompt's tail backwards (these have
// rap = r+1 <= csz); r >= csz walks the first tokens (the only ones whose slot
// can lie in the static part); any other token is a ring token older than
// the last csz and is dropped by the keep rule.
__device__ __forceinline__ bool candidate(const HeadRing& g, int64_t r, int S,
                                          const int32_t* __restrict__ ap_row,
                                          const int32_t* __restrict__ rap_row,
                                          const int64_t* __restrict__ am_row,
                                          int64_t& t, int64_t& slot) {
  int64_t a, rap;
  if (ap_row == nullptr) {
    if (r < g.csz) {
      t = (int64_t)S - 1 - r;
      if (t < 0) return false;
    } else {
      t = r - g.csz;
      if (t >= (int64_t)S - g.csz || t > g.s) return false;
    }
    a = t;
    rap = (int64_t)S - t;
  } else {
    t = r;
    if (t >= S) return false;
    if (am_row[t] != 1) return false;
    a = ap_row[t];
    rap = rap_row[t];
  }
  slot = slot_of(g, a);
  return keep_of(g, slot, rap);
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

// ap[b, t] = (#ones in am[b, 0..t]) - 1 for t in [0, S), ap[b, S] = ap[b, S-1] + 1;
// rap[b, t] = #ones in am[b, t..S-1]   (:1075-1086)
__global__ __launch_bounds__(256) void mask_scan_kernel(const int64_t* __restrict__ am,
                                                         int64_t am_stride, int S,
                                                         int32_t* __restrict__ ap,
                                                         int32_t* __restrict__ rap) {
  __shared__ int32_t part[256];
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t* row = am + (int64_t)b * am_stride;
  const int per = (S + 255) / 256;
  const int t0 = tid * per;
  const int t1 = min(S, t0 + per);
  int32_t sum = 0;
  for (int t = t0; t < t1; ++t) sum += (int32_t)row[t];
  part[tid] = sum;
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0;
    for (int i = 0; i < 256; ++i) {
      int32_t x = part[i];
      part[i] = run;
      run += x;
    }
  }
  __syncthreads();
  int32_t total = part[255];
  {
    // total = exclusive prefix of the last thread + its own sum
    const int lt0 = 255 * per;
    for (int t = lt0; t < S; ++t) total += (int32_t)row[t];
  }
  int32_t run = part[tid];
  int32_t* ap_row = ap + (int64_t)b * (S + 1);
  int32_t* rap_row = rap + (int64_t)b * S;
  for (int t = t0; t < t1; ++t) {
    const int32_t x = (int32_t)row[t];
    run += x;
    ap_row[t] = run - 1;
    rap_row[t] = total - run + x;
  }
  if (tid == 0) ap_row[S] = total;  // ap[S-1] + 1 == total - 1 + 1
}

__global__ __launch_bounds__(kCacheThreads) void cache_prefill_copy_kernel(
    const char* __restrict__ k, const char* __restrict__ v,
    int64_t k_sb, int64_t k_sh, int64_t k_ss, int64_t v_sb, int64_t v_sh, int64_t v_ss,  // bytes
    char* __restrict__ kc, char* __restrict__ vc, int64_t* __restrict__ mask_cache,
    const int64_t* __restrict__ update_index, const int64_t* __restrict__ circ_head,
    const int64_t* __restrict__ circ_size, const int64_t* __restrict__ static_size,
    const int64_t* __restrict__ am, int64_t am_stride, const int32_t* __restrict__ ap,
    const int32_t* __restrict__ rap, int64_t kv_len, int H, int S, int row_bytes, int64_t sumC) {
  const int lane = threadIdx.x % kRowLanes;
  const int64_t r = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kRowLanes;
  const int h = blockIdx.y;
  const int b = blockIdx.z;
  const int64_t bh = (int64_t)b * H + h;
  const HeadRing g = load_ring(update_index, circ_head, circ_size, static_size, kv_len, bh, h);
  int64_t t, slot;
  const bool keep = candidate(g, r, S, ap ? ap + (int64_t)b * (S + 1) : nullptr,
                              rap ? rap + (int64_t)b * S : nullptr,
                              am ? am + (int64_t)b * am_stride : nullptr, t, slot);
  if (!keep || slot < 0 || slot >= sumC) return;
  if (kc != nullptr) {
    const int units = row_bytes / 16;
    const size_t dst = ((size_t)b * sumC + slot) * row_bytes;
    copy_row16(k + b * k_sb + h * k_sh + t * k_ss, kc + dst, units, lane);
    copy_row16(v + b * v_sb + h * v_sh + t * v_ss, vc + dst, units, lane);
  }
  if (lane == 0 && mask_cache != nullptr) mask_cache[(size_t)b * sumC + slot] = 1;
}

// One wavefront per (b, h): count the kept tokens, then move the pointers
// (:1110, :1136-1138).  Runs after the copy kernel on the same stream because
// it overwrites update_index, which the copy kernel reads.
__global__ __launch_bounds__(256) void cache_prefill_index_kernel(
    int64_t* __restrict__ update_index, int64_t* __restrict__ valid_len,
    const int64_t* __restrict__ circ_head, const int64_t* __restrict__ circ_size,
    const int64_t* __restrict__ static_size, const int64_t* __restrict__ am, int64_t am_stride,
    const int32_t* __restrict__ ap, const int32_t* __restrict__ rap, int64_t kv_len, int B, int H,
    int S) {
  const int lane = threadIdx.x & 63;
  const int64_t bh = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (bh >= (int64_t)B * H) return;
  const int b = (int)(bh / H);
  const int h = (int)(bh % H);
  const HeadRing g = load_ring(update_index, circ_head, circ_size, static_size, kv_len, bh, h);
  const int32_t* ap_row = ap ? ap + (int64_t)b * (S + 1) : nullptr;
  const int32_t* rap_row = rap ? rap + (int64_t)b * S : nullptr;
  const int64_t* am_row = am ? am + (int64_t)b * am_stride : nullptr;
  // number of candidates: all tokens with a mask; else tail (<= csz) + first s+1 tokens
  const int64_t n_cand = ap ? (int64_t)S : min((int64_t)S, g.csz + g.s + 1);
  int count = 0;
  for (int64_t r = lane; r < n_cand; r += 64) {
    int64_t t, slot;
    count += candidate(g, r, S, ap_row, rap_row, am_row, t, slot) ? 1 : 0;
  }
  for (int off = 32; off > 0; off >>= 1) count += __shfl_xor(count, off, 64);
  if (lane == 0) {
    const int64_t a_end = ap ? (int64_t)ap_row[S] : (int64_t)S;
    update_index[bh] = slot_of(g, a_end);
    valid_len[bh] += count;
  }
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
  int32_t* ap = nullptr;
  int32_t* rap = nullptr;
  int64_t n_rows;
  if (attention_mask != nullptr) {
    const size_t need = moa_cache_prefill_workspace_bytes(B, S);
    if (workspace == nullptr || workspace_bytes < need)
      return fail(MOA_ERR_WORKSPACE, "moa_cache_prefill_insert: workspace %zu < %zu bytes", workspace_bytes, need);
    ap = reinterpret_cast<int32_t*>(workspace);
    rap = ap + (size_t)B * ((size_t)S + 1);
    hipLaunchKernelGGL(mask_scan_kernel, dim3(B), dim3(256), 0, st, attention_mask, am_stride, S, ap, rap);
    int rc = check_launch("moa_cache_prefill_insert(mask scan)");
    if (rc) return rc;
    n_rows = S;
  } else {
    // candidates r >= S never name a token (see candidate())
    n_rows = S;
    if (max_cache_size > 0 && max_cache_size + 1 < n_rows) n_rows = max_cache_size + 1;
  }
  if (kc != nullptr || mask_cache != nullptr) {
    dim3 grid((unsigned)((n_rows + kRowsPerBlock - 1) / kRowsPerBlock), (unsigned)H, (unsigned)B);
    hipLaunchKernelGGL(cache_prefill_copy_kernel, grid, dim3(kCacheThreads), 0, st, (const char*)k,
                       (const char*)v, ks[0], ks[1], ks[2], vs[0], vs[1], vs[2], (char*)kc, (char*)vc,
                       mask_cache, (const int64_t*)update_index, circ_head, circ_size, static_size,
                       attention_mask, am_stride, (const int32_t*)ap, (const int32_t*)rap, kv_len, H, S,
                       D * eb, sumC);
    int rc = check_launch("moa_cache_prefill_insert(copy)");
    if (rc) return rc;
  }
  const int64_t n = (int64_t)B * H;
  hipLaunchKernelGGL(cache_prefill_index_kernel, dim3((unsigned)((n + 3) / 4)), dim3(256), 0, st,
                     update_index, valid_len, circ_head, circ_size, static_size, attention_mask,
                     am_stride, (const int32_t*)ap, (const int32_t*)rap, kv_len, B, H, S);
  return check_launch("moa_cache_prefill_insert(index)");
}
