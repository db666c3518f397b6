/*
 * moa_hip.h -- C ABI of libmoa_hip.so: the MoA sparse-attention hot path on
 * AMD MI355X (gfx950).
 *
 * The reference (thu-nics/MoA) has no native code of its own: its Python
 * dispatcher calls an external CUDA package (`from flashinfer import
 * moa_prefill, moa_decode`, MoA/kernels/mixture_of_attention.py:22-30) and
 * moves KV rows with torch indexing ops (MoA/attention/cache_utils.py:953-1164).
 * Each entry point below replaces one of those call sites; the citation says
 * which.  All pointers are DEVICE pointers unless marked "host".  Every call
 * only enqueues work on `stream` (a hipStream_t passed as void*; NULL = the
 * null stream): no allocation, no synchronisation, no host read-back, no
 * global state except a thread-local error string.
 *
 * Return value: MOA_OK (0) or a negative MOA_ERR_* code; moa_last_error()
 * then describes the failure.  Nothing throws.
 */
#ifndef MOA_HIP_H
#define MOA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOA_OK 0
#define MOA_ERR_ARG (-1)         /* bad shape / null pointer / misaligned    */
#define MOA_ERR_UNSUPPORTED (-2) /* valid request this build does not cover  */
#define MOA_ERR_LAUNCH (-3)      /* the HIP runtime refused a launch         */
#define MOA_ERR_WORKSPACE (-4)   /* workspace too small                      */

#define MOA_DTYPE_F16 0
#define MOA_DTYPE_BF16 1
#define MOA_DTYPE_F32 2 /* cache entry points only */

#define MOA_BLOCK 64 /* tokens per sparsity block: mixture_of_attention.py:32-33 */

/* ABI version of this header (bumped on any signature change). */
int moa_abi_version(void);

/* Human-readable description of the last failure on the calling thread. */
const char* moa_last_error(void);

/*
 * Block-sparse causal prefill attention.
 * Replaces: flashinfer.moa_prefill (call site mixture_of_attention.py:435-444)
 * and the Triton kernel _sparse_attention_prefill_moa_fwd_kernel
 * (MoA/kernels/block_sparse_attention_prefill.py:473-629, launched :677-690).
 *
 * For query block m (64 rows) of kv-head h the live key blocks are
 *   {0 .. min(sink_blocks[h]-1, m)}  U  {max(0, m+1-local_blocks[h]) .. m},
 * causal inside the diagonal block; rows with no live key produce 0.
 *
 * q, o: [B, Hq, N, D]; k, v: [B, Hkv, N, D]; each addressed through its own
 * strides (host array of 4 element strides, order B,H,N,D; the D stride must
 * be 1 and every row 16-byte aligned).  The reference's return layout
 * [B, N, H, D] is obtained by passing the strides of that layout for `o`.
 * Hq must be a multiple of Hkv; query head h reads kv-head h / (Hq/Hkv).
 * sink_blocks, local_blocks: int64 [Hkv] BLOCK counts (the reference passes
 * sink_size // 64 and local_size // 64, mixture_of_attention.py:441-442).
 * dtype: MOA_DTYPE_F16 or MOA_DTYPE_BF16.  D: 64 or 128.
 *
 * The launch hands its (head, query tile) work items to one resident work-group
 * per CU through a few counters in a small device array that is part of the
 * library's device image (64 bytes per launch, 256 slots used in turn; a slot is
 * left cleared by the launch that used it).  The call itself allocates nothing.
 * Launches may overlap on one GPU as long as fewer than 256 of them are under
 * way at once.  The first call on a device looks that array up and the first
 * call per (dtype, D) sets a kernel attribute: make one ordinary call per device
 * and (dtype, D) before recording the call into a HIP graph; a recorded call
 * keeps the slot it was recorded with, so replays of ONE graph that overlap each
 * other on a GPU are not supported.  Sizes beyond what the queue arithmetic
 * covers return MOA_ERR_UNSUPPORTED: B * Hq <= 2^22, B * Hq * ceil(N / 256) <=
 * 2^25, N <= 2^28.
 */
int moa_prefill_fwd(const void* q, const void* k, const void* v, void* o,
                    const int64_t* q_strides, const int64_t* k_strides,
                    const int64_t* v_strides, const int64_t* o_strides,
                    int B, int Hq, int Hkv, int N, int D,
                    const int64_t* sink_blocks, const int64_t* local_blocks,
                    float sm_scale, int dtype, void* stream);

/*
 * Bytes of scratch moa_decode_fwd needs for these sizes (split-K partials).
 */
size_t moa_decode_workspace_bytes(int B, int Hq, int Hkv, int D, int64_t sumC);

/*
 * Single-token decode attention over per-head segments of the packed cache.
 * Replaces: flashinfer.moa_decode (call site mixture_of_attention.py:465-473;
 * argument meaning :389-392).
 *
 * For each (b, h): o[b,h,:] = softmax(sm_scale * q[b,h,:] . K_seg^T) V_seg with
 * K_seg = kc[b, start : start+len, :], start = head_start[b, h/(Hq/Hkv)],
 * len = head_valid_len[b, h/(Hq/Hkv)].  No mask, no causality (every cached
 * token is in the past); row order inside a segment does not matter, so ring
 * wraparound needs no special handling.  len == 0 gives 0.
 *
 * q, o: contiguous [B, Hq, D] (the reference's [B,1,Hq,D]); kc, vc: contiguous
 * [B, sumC, D]; head_start, head_valid_len: int64 [B, Hkv].  The segments of
 * one batch row must not overlap (their lengths sum to at most sumC), as in
 * the packed cache; the workspace is sized for that.
 * Query head h reads ring h / (Hq/Hkv): grouped-query attention, which the
 * reference does not have (its caller asserts one kv group,
 * MoA/models/llama/modeling_llama.py:220-224), with Hq/Hkv in 1..8.
 * With one query head per ring the kernel works on the vector ALU in fp32;
 * with 2 to 8 it works on the matrix cores and rounds the softmax weights
 * to the input type before multiplying with V (like the prefill kernel).
 * D in {64,128}, f16/bf16, at most 256 kv heads.
 */
int moa_decode_fwd(const void* q, const void* kc, const void* vc, void* o,
                   void* workspace, size_t workspace_bytes,
                   const int64_t* head_start, const int64_t* head_valid_len,
                   int B, int Hq, int Hkv, int D, int64_t sumC,
                   float sm_scale, int dtype, void* stream);

/*
 * moa_decode_fwd without a workspace argument, for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.  Same
 * arguments, kernels and results as moa_decode_fwd; the split-K partials go
 * into a scratch array of MOA_DECODE_NOALLOC_MAX_BYTES that is part of the
 * library's device image (every GPU the library runs on holds it until the
 * process ends).  Sizes for which moa_decode_workspace_bytes(...) exceeds that
 * are rejected with MOA_ERR_WORKSPACE.  The call allocates and frees nothing.
 * All calls on one GPU share that GPU's array: calls that may overlap on one
 * GPU (different streams, different threads) race on it and must be
 * serialised by the caller.
 * The first call on a device looks the array's device address up and the first
 * call of a (dtype, head_dim, grouped or not) class sets a kernel attribute:
 * make one ordinary call per device and class before recording the call into a
 * HIP graph.
 */
#define MOA_DECODE_NOALLOC_MAX_BYTES (32u << 20)
int moa_decode_fwd_noalloc(const void* q, const void* kc, const void* vc, void* o,
                           const int64_t* head_start, const int64_t* head_valid_len,
                           int B, int Hq, int Hkv, int D, int64_t sumC,
                           float sm_scale, int dtype, void* stream);

/*
 * One decode-step append into every head's ring, with the index bookkeeping,
 * in one launch.
 * Replaces: the decode branch of StaticCircularCache.update
 * (MoA/attention/cache_utils.py:1020-1058): for every (b,h)
 *   idx = update_index[b,h]; mask_cache[b,idx] = 1; kc[b,idx,:] = k_new[b,h,:];
 *   vc likewise; valid_len += (valid_len < max_len[h]);
 *   update_index = (kv_len+1 > static_size[h])
 *                    ? (idx+1-circ_head[h]) mod circ_size[h] + circ_head[h]
 *                    : idx+1.
 * k_new, v_new: [B, H, D] through host strides (3 element strides, order
 * B,H,D; D stride 1).  kc/vc may both be NULL (bookkeeping only -- the
 * reference's update_cache_content=False, cache_utils.py:661,1032-1034);
 * mask_cache may be NULL.  update_index, valid_len: int64 [B,H], updated in
 * place (they must be materialised, not stride-0 views).  circ_head,
 * circ_size, static_size, max_len: int64 [H].  kv_len: tokens seen so far by
 * this layer (host value, the reference's python int _kv_len).
 */
int moa_cache_append(const void* k_new, const void* v_new,
                     const int64_t* kn_strides, const int64_t* vn_strides,
                     void* kc, void* vc, int64_t* mask_cache,
                     int64_t* update_index, int64_t* valid_len,
                     const int64_t* circ_head, const int64_t* circ_size,
                     const int64_t* static_size, const int64_t* max_len,
                     int64_t kv_len, int B, int H, int D, int64_t sumC,
                     int dtype, void* stream);

/*
 * Rotary position embedding of the query and key heads (prompt or single step).
 * Replaces: apply_rotary_pos_emb(query_states, key_states, cos, sin) in the
 * reference's caller (MoA/models/llama/modeling_llama.py:252; the function is
 * transformers 4.44.2's, requirements.txt:8):
 *   x_embed = (x * cos) + (rotate_half(x) * sin),  rotate_half(x) = cat(-x[D/2:], x[:D/2]),
 * rounded to the tensors' dtype after each product and after the sum, as torch
 * evaluates it (results are bit-identical to that evaluation).
 * q, k, q_out, k_out: [B, H, N, D] through host strides (4 element strides,
 * order B,H,N,D; D stride 1); q_out == q and k_out == k (in place) is allowed.
 * cos, sin: [B, N, D] through cs_strides (3 element strides; a batch stride of 0
 * broadcasts one position table).  Hq or Hkv may be 0 to rotate one tensor only.
 * head_dim * element size must be a multiple of 32 bytes.  f16, bf16, f32.
 */
int moa_rope_fwd(const void* q, const void* k, void* q_out, void* k_out,
                 const int64_t* q_strides, const int64_t* k_strides,
                 const int64_t* qo_strides, const int64_t* ko_strides,
                 const void* cos, const void* sin, const int64_t* cs_strides,
                 int B, int Hq, int Hkv, int N, int D, int dtype, void* stream);

/*
 * One decode step in front of the attention kernel, in one launch: rotary
 * embedding of q (written to q_out, contiguous [B, Hq, D] = the reference's
 * [B,1,Hq,D]) and of k, and the append of the rotated k and of v into every
 * head's ring with the index bookkeeping of moa_cache_append.
 * Replaces: modeling_llama.py:252 (apply_rotary_pos_emb) + :262
 * (past_key_value.update, decode branch cache_utils.py:1020-1058).
 * q_new, k_new, v_new: [B, H, D] through host strides (3 element strides,
 * order B,H,D; D stride 1); cos, sin: [B, D] rows cs_stride_b elements apart
 * (0 broadcasts).  The other arguments are those of moa_cache_append; kc and vc
 * are required.
 */
int moa_rope_cache_append(const void* q_new, const void* k_new, const void* v_new,
                          const int64_t* qn_strides, const int64_t* kn_strides,
                          const int64_t* vn_strides, const void* cos, const void* sin,
                          int64_t cs_stride_b, void* q_out, void* kc, void* vc,
                          int64_t* mask_cache, int64_t* update_index, int64_t* valid_len,
                          const int64_t* circ_head, const int64_t* circ_size,
                          const int64_t* static_size, const int64_t* max_len,
                          int64_t kv_len, int B, int Hq, int Hkv, int D, int64_t sumC,
                          int dtype, void* stream);

/* Scratch bytes for moa_cache_prefill_insert when an attention_mask is given
 * (0 otherwise). */
size_t moa_cache_prefill_workspace_bytes(int B, int S);

/*
 * Bulk insert of a prompt's K/V into the rings.
 * Replaces: the prefill branch of StaticCircularCache.update
 * (cache_utils.py:1060-1164), same slot / keep / pointer / valid-length
 * formulas, including the optional 0/1 attention_mask [B, S] (int64, row
 * stride am_stride; NULL = all ones) that left-pads shorter prompts.
 * k, v: [B, H, S, D] through host strides (order B,H,S,D; D stride 1).
 * max_cache_size: host upper bound of max_len over heads (bounds the launch;
 * pass 0 if unknown).
 */
int moa_cache_prefill_insert(const void* k, const void* v,
                             const int64_t* k_strides, const int64_t* v_strides,
                             void* kc, void* vc, int64_t* mask_cache,
                             int64_t* update_index, int64_t* valid_len,
                             const int64_t* circ_head, const int64_t* circ_size,
                             const int64_t* static_size,
                             const int64_t* attention_mask, int64_t am_stride,
                             void* workspace, size_t workspace_bytes,
                             int64_t kv_len, int B, int H, int S, int D,
                             int64_t sumC, int64_t max_cache_size, int dtype,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOA_HIP_H */
