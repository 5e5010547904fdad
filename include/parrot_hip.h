/*
 * parrot_hip.h -- C ABI of libparrot_hip.so: the attention hot path of
 * Parrot's builtin engine on AMD MI355X (gfx950).
 *
 * Conventions (they mirror the reference's native extension, which takes
 * tensors owned by the caller, launches on the caller's current stream and
 * neither synchronises nor allocates -- csrc/attention/attention_post_kernels.cu:416):
 *   - every pointer is a DEVICE pointer owned by the caller unless it says host;
 *   - strides and sizes are in ELEMENTS unless the name ends in _bytes;
 *   - all launches are asynchronous on `stream` (a hipStream_t passed as void*);
 *   - no entry point allocates, frees or synchronises; scratch comes in through
 *     a workspace argument whose size the matching *_workspace_bytes() reports;
 *   - return value: PH_OK or a PH_ERR_* code; ph_status_string() names it.
 *     The reference raises RuntimeError through TORCH_CHECK for unsupported
 *     head size / dtype (csrc/attention/attention_kernels.cu:482,535,568); the
 *     Python layer turns a non-zero status into the same exception class.
 *   - KV pools are token-granular: [slots, H, D], the reference's
 *     MemLayout.NORMAL (parrot/engine/builtin/mem.py:43-56); a "block table"
 *     of the reference with block_size 1 is a list of slot ids here.
 */
#ifndef PARROT_HIP_H
#define PARROT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types.  The reference's configuration offers float16 and float32 (parrot/engine/config.py:22-25), its CUDA
 * kernels also bfloat16.  PH_F32 is served by the per-request decode kernels (every attention entry point: a
 * shared prefix is then read once per request, a prefill runs row by row), the merge, RMSNorm, both rotary forms,
 * the token move, the KV append and the sampler; the matrix-core kernels and the fused per-layer ops are 16-bit. */
typedef enum { PH_F16 = 0, PH_BF16 = 1, PH_F32 = 2 } ph_dtype;
typedef enum { PH_IDX_I32 = 0, PH_IDX_I64 = 1 } ph_index_type;

enum {
  PH_OK = 0,
  PH_ERR_DTYPE = 1,     /* unsupported element type */
  PH_ERR_HEAD_DIM = 2,  /* unsupported head size */
  PH_ERR_ALIGN = 3,     /* pointer or stride not aligned as the kernel needs */
  PH_ERR_ARG = 4,       /* inconsistent sizes, null pointer, negative count */
  PH_ERR_WORKSPACE = 5, /* workspace too small */
  PH_ERR_LAUNCH = 6,    /* hipLaunchKernel reported an error */
  PH_ERR_SCRATCH = 7    /* the shape needs more scratch than the library's own fixed array holds */
};

const char* ph_status_string(int status);
/* Library ABI version; bumped whenever a signature changes. */
int ph_abi_version(void);

/* ------------------------------------------------------------------------ */
/* Token move: dest[dst_idx[i], :, :] = src[src_idx[i], :, :], i < n.
 * Replaces discontinuous_move_tokens and its Triton kernel
 * (parrot/engine/builtin/kernels/tokens_moving.py:25-100): rows are
 * [num_heads, head_dim] with free strides on all three axes.
 * src_idx == NULL means the identity (row i); same for dst_idx.
 * dst indices must be unique (the reference has the same requirement).
 * Bit-exact copy; elem_bytes in {1,2,4,8}. */
int ph_move_tokens(const void* src, void* dst,
                   const void* src_idx, const void* dst_idx, int index_type,
                   int64_t n, int64_t num_heads, int64_t head_dim, int elem_bytes,
                   int64_t src_stride_n, int64_t src_stride_h, int64_t src_stride_d,
                   int64_t dst_stride_n, int64_t dst_stride_h, int64_t dst_stride_d,
                   void* stream);

/* Gather of token rows out of the block-structured (vLLM) cache layouts into
 * token-granular rows dest[n, H, D]; slot = src_slots[i], b = slot / block_size,
 * o = slot % block_size:
 *   K [num_blocks, H, D/x, block_size, x]:
 *       dest[dest_idx[i], h, c*x + e] = k_cache[b, h, c, o, e]
 *   V [num_blocks, H, D, block_size]:
 *       dest[dest_idx[i], h, d]       = v_cache[b, h, d, o]
 * Replace move_tokens_from_blocked_k_cache / move_tokens_from_blocked_v_cache
 * and their Triton kernels (parrot/engine/builtin/kernels/tokens_moving.py:
 * 104-218 and 222-313).  All strides are in elements and free; the fast path
 * needs unit-stride x (K), contiguous destination head rows and 16-byte
 * aligned destination rows, anything else takes an element-wise path.
 * dest_idx entries must be unique; slots must lie inside the cache (not
 * checked, as in the reference).  Bit-exact copy; elem_bytes in {1,2,4,8}. */
int ph_gather_blocked_k(const void* k_cache, void* dest,
                        const void* src_slots, const void* dest_idx, int index_type,
                        int64_t n, int64_t num_heads, int64_t head_dim,
                        int64_t block_size, int64_t x, int elem_bytes,
                        int64_t stride_n, int64_t stride_h, int64_t stride_c,
                        int64_t stride_b, int64_t stride_x,
                        int64_t dst_stride_n, int64_t dst_stride_h, int64_t dst_stride_d,
                        void* stream);
int ph_gather_blocked_v(const void* v_cache, void* dest,
                        const void* src_slots, const void* dest_idx, int index_type,
                        int64_t n, int64_t num_heads, int64_t head_dim,
                        int64_t block_size, int elem_bytes,
                        int64_t stride_n, int64_t stride_h, int64_t stride_d, int64_t stride_b,
                        int64_t dst_stride_n, int64_t dst_stride_h, int64_t dst_stride_d,
                        void* stream);

/* KV append: k_cache[slot[t]] = k[t], v_cache[slot[t]] = v[t] in ONE launch.
 * Replaces vllm_reshape_and_cache -> cache_ops.reshape_and_cache
 * (parrot/engine/builtin/kernels/vllm/reshape_and_cache.py:9-22,
 * 3rdparty/vllm/csrc/cache_kernels.cu:142-224) on the token-granular layout,
 * and the arange-source token move of attn_func.py:143-155.
 * k, v: [T, H, D] with row stride k_stride_n / v_stride_n (heads contiguous);
 * caches: [slots, H, D] with row stride cache_stride_n. */
int ph_kv_append(const void* k, const void* v, void* k_cache, void* v_cache,
                 const void* slot_mapping, int index_type,
                 int64_t num_tokens, int64_t num_heads, int64_t head_dim, int dtype,
                 int64_t k_stride_n, int64_t v_stride_n, int64_t cache_stride_n,
                 void* stream);

/* ------------------------------------------------------------------------ */
/* RMSNorm: out = w * t(x * rsqrt(mean(x^2) + eps)).
 * Replaces layernorm_ops.rms_norm (3rdparty/vllm/csrc/layernorm_kernels.cu:9-63,
 * wrapper parrot/engine/builtin/kernels/vllm/rms_norm.py:9-16) when
 * round_before_weight != 0 (the normalised value is rounded to the element
 * type before the weight multiply, :32), and rmsnorm_forward
 * (parrot/engine/builtin/kernels/rms_norm.py:15-78) when it is 0 (one rounding).
 * x, out: [rows, n] with row strides; w: [n]. */
int ph_rms_norm(void* out, const void* x, const void* weight, float eps,
                int64_t rows, int64_t n, int64_t x_stride, int64_t out_stride,
                int dtype, int round_before_weight, void* stream);

/* NeoX RoPE on q and k in place, one launch, cos/sin looked up by position.
 * Replaces pos_encoding_ops.rotary_embedding_neox
 * (3rdparty/vllm/csrc/pos_encoding_kernels.cu:6-104, wrapper
 * parrot/engine/builtin/kernels/vllm/rotary_embed.py:10-25).
 * q: [T, num_q_heads*head_dim] row stride q_stride; k likewise (they are chunk
 * views of the fused qkv, models/llama.py:111-112); k may be NULL.
 * cos_sin_cache: [max_pos, rot_dim] = cat(cos, sin); positions: int64 [T].
 * Arithmetic follows the reference kernel: each product and the sum are rounded
 * to the element type (:36-42). */
int ph_rope_neox(const int64_t* positions, void* q, void* k, const void* cos_sin_cache,
                 int64_t num_tokens, int64_t num_q_heads, int64_t num_k_heads,
                 int64_t head_dim, int64_t rot_dim,
                 int64_t q_stride, int64_t k_stride, int dtype, void* stream);

/* NeoX RoPE in place with per-token cos / sin rows already gathered.
 * Replaces rotary_embedding(state, cos, sin)
 * (parrot/engine/builtin/kernels/rotary_embedding.py:24-143).
 * state: [T, H, D] strides (stride_n, stride_h, 1); cos, sin: [T, 1, D/2] with
 * row stride cs_stride. */
int ph_rotary_embedding(void* state, const void* cos, const void* sin,
                        int64_t num_tokens, int64_t num_heads, int64_t head_dim,
                        int64_t stride_n, int64_t stride_h, int64_t cs_stride,
                        int dtype, void* stream);

/* ------------------------------------------------------------------------ */
/* Decode attention (one query token per request) over slot tables.
 *
 * A request b attends over   prefix_slots[group(b)]  ||  suffix slots of b.
 * Partials are (O, m, l) in the exp2 domain: y = q.k*scale*log2(e),
 * m = max y, l = sum 2^(y-m), O = sum 2^(y-m) v / l
 * (parrot/engine/builtin/kernels/shared_flash_decoding.py:98-134); the merge
 * is M = max, L = sum 2^(m-M) l, O = sum 2^(m-M) l O / L
 * (csrc/attention/attention_post_kernels.cu:321-340).
 *
 * ph_decode_attention replaces, depending on its arguments:
 *   - flash_paged_attention / paged_flash_attention (shared prefix + suffix +
 *     merge; shared_flash_decoding.py:285-376 = triton_flash_attention :202-277
 *     + attention_ops.single_query_cached_kv_post_attention,
 *     csrc/attention.cpp:34-47), when num_groups >= 1;
 *   - vllm_paged_attention -> attention_ops.single_query_cached_kv_attention
 *     (parrot/engine/builtin/kernels/vllm/paged_attention.py:12-38,
 *     3rdparty/vllm/csrc/attention.cpp:4-15), when num_groups == 0.
 *
 * q, out: [B, H, D], row strides q_stride / out_stride (heads contiguous).
 * k_cache, v_cache: [slots, H, D], row stride cache_stride_n.
 * Prefix groups (num_groups may be 0):
 *   prefix_slots: int32, all groups' prefix slot lists back to back;
 *   prefix_cu:    int32 [num_groups+1] offsets into prefix_slots   (DEVICE);
 *   group_req_cu: int32 [num_groups+1]: requests group_req_cu[g] ..
 *                 group_req_cu[g+1]-1 belong to group g (requests of one group
 *                 are contiguous; requests outside every range have no
 *                 prefix).  Passed twice: a DEVICE copy for the kernels and a
 *                 HOST copy for the launch geometry;
 *   max_prefix_len: host upper bound of any group's prefix length.
 * Suffix (per request) slot table, two forms:
 *   suffix_offsets != NULL: int64 [B] start of request b's list inside
 *                 suffix_slots (ragged, back to back);
 *   suffix_offsets == NULL: suffix_slots is a padded 2-D table, request b's
 *                 list starts at b * suffix_table_stride (the reference's
 *                 paged_block_tables [B, max]).
 *   suffix_slots_count: number of int32 entries readable behind suffix_slots
 *                 (the kernel prefetches slot ids before it knows a list's
 *                 length and clamps those reads to this bound).  A padded
 *                 table must hold max_suffix_len entries in every row:
 *                 suffix_slots_count >= (B - 1) * suffix_table_stride +
 *                 max_suffix_len, else PH_ERR_ARG;
 *   suffix_lens:  int32 [B] (DEVICE); max_suffix_len: host upper bound -- the
 *                 kernels read a length as min(max(len, 0), max_suffix_len)
 *                 (and no further than the table's end), so a bad entry
 *                 cannot walk into another request's slots (for a padded
 *                 table pass at most its width).  This is a clamp, not only a
 *                 sizing hint: tokens beyond max_suffix_len are not attended
 *                 to.  A call captured into a graph and replayed while the
 *                 lists grow must therefore be captured with the largest
 *                 length a replay will see (the table's width, say) -- also
 *                 when the library builds the plan itself, whose arguments
 *                 are recorded with the call.
 * chunk_tokens: suffix split size of the plain (request, chunk) grid form
 *   (multiple of 16); 0 = leave the decomposition to the library.
 * plan (HOST struct of DEVICE pointers, may be NULL): a caller that knows the
 *   suffix lengths on the host (the reference builds them from Python lists,
 *   attn_func.py:523-531) cuts the batch's suffix token stream into num_lanes
 *   near-equal pieces; a piece is one or more items (request, first token,
 *   token count).  The suffix phase then runs one wave set per piece, every wave
 *   moving the same number of bytes, instead of one per fixed-size chunk.
 *   With plan == NULL and chunk_tokens == 0 the library builds the same plan
 *   itself, on the device, at the start of the call (ph_suffix_plan_build into
 *   the workspace; up to 8192 requests, a few microseconds per call) -- a
 *   caller that runs many layers per iteration saves that by building the plan
 *   once and passing it.  plan == NULL with chunk_tokens > 0, or more than
 *   8192 requests, runs the grid form.
 *   items:        int32 [num_items][4] = request, first token, count, 0, in
 *                 request order (a request's items are consecutive, its tokens
 *                 ascending and covered exactly once);
 *   lane_rec:     int32 [num_lanes][8], piece j = (first item, item count,
 *                 then a copy of its first item's request, first token, count,
 *                 0, 0, 0) -- one record read starts a piece;
 *   req_item_cu:  int32 [B+1], request b owns items [cu[b], cu[b+1]).
 *   num_items may be the capacity of the items array rather than the count
 *   in use (only items named by lane_rec / req_item_cu are touched, and at
 *   most num_lanes + B - 1 can be): it sizes the workspace only.  A caller
 *   that replays a captured graph while contexts grow keeps the pointers,
 *   num_items and num_lanes fixed and rewrites the arrays in place.
 * workspace: at least ph_decode_workspace_bytes(...) bytes, 256-byte aligned
 *   (num_items = plan->num_items, or 0 without a plan).
 * head_dim: 64, 80, 96, 112, 128 or 256 -- the sizes the reference's kernels
 *   dispatch (csrc/attention/attention_post_kernels.cu:420-446); anything else
 *   returns PH_ERR_HEAD_DIM.  The same set holds for every attention entry
 *   point below.
 */
typedef struct {
  const int32_t* items;
  int64_t num_items;
  const int32_t* lane_rec;
  int64_t num_lanes;
  const int32_t* req_item_cu;
} ph_suffix_plan;

size_t ph_decode_workspace_bytes(int64_t num_reqs, int64_t num_heads, int64_t head_dim,
                                 int64_t num_groups, int64_t max_prefix_len,
                                 int64_t max_suffix_len, int64_t chunk_tokens, int64_t num_items);

/* Number of pieces (num_lanes) a caller's balanced suffix plan should be cut
 * into for a ph_decode_attention call of this shape: one round of waves, two
 * per SIMD, on the compute units the suffix phase runs on.  That is every
 * compute unit of the device, except where the library runs the prefix and
 * suffix phases of a call in one launch with workgroups of their own (16-bit
 * elements, head size 128 or paired 64, and a shape for which the library's
 * cost estimate favours that form: most, except prefixes that want the whole
 * device): there the prefix keeps the compute units a
 * cost model gives it and the suffix takes the rest.  A plan cut into another
 * number of pieces stays correct: with more pieces than that (a plan cut for
 * the whole device) the call runs both phases in every workgroup
 * instead; with fewer, waves idle.  kv_group: 1 (or 0) for a plain call; G for
 * a ph_decode_attention_gqa call that will state kv_group = G -- the planner
 * then counts the K/V bytes and matrix rows of that call, and with G a power of
 * two from 4 on (head size 128, 16-bit elements) and lists long enough to gain
 * from it the suffix waves stream every token row for four query heads of its
 * KV head at once, so a piece occupies a quarter of the waves and the device
 * takes four times the pieces.  Host-only,
 * no launch.  The
 * reference has no counterpart (fixed (request, block) grids,
 * attention_post_kernels.cu:395-418). */
int64_t ph_decode_suffix_lanes(int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                               int64_t num_groups, int64_t max_prefix_len, int64_t max_suffix_len,
                               int64_t kv_group);

int ph_decode_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                        int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                        int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                        float scale,
                        int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                        const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                        int64_t max_prefix_len,
                        const int32_t* suffix_slots, const int64_t* suffix_offsets,
                        int64_t suffix_table_stride, int64_t suffix_slots_count,
                        const int32_t* suffix_lens,
                        int64_t max_suffix_len, int64_t chunk_tokens,
                        const ph_suffix_plan* plan,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ph_decode_attention for query heads that share KV heads (grouped / multi-query
 * attention): the reference's native kernels read the KV head
 * head_mapping[query head] (csrc/attention/attention_post_kernels.cu:79,101,
 * attention_prev_kernels.cu, 3rdparty/vllm/csrc/attention/attention_kernels.cu:
 * kv_head_idx = head_mapping[head_idx]).
 *   k_cache, v_cache: [slots, num_kv_heads, D];
 *   head_mapping: int32 [num_heads] (DEVICE), KV head of every query head, each
 *                 in [0, num_kv_heads);
 *   kv_group:     host statement about the mapping.  G > 0 asserts
 *                 head_mapping[h] == h / G with num_heads == G * num_kv_heads
 *                 (what repeat_interleave(arange(num_kv_heads), G) holds): for
 *                 G a power of two up to 64, head size 128 and 16-bit elements
 *                 the prefix phase then runs on the matrix cores with the G
 *                 query heads of a KV head as G rows per request of one tile,
 *                 so a group's prefix K/V is still read once -- and at G times
 *                 the arithmetic per byte; from G = 4 on, suffix lists of 200
 *                 tokens and more (about 8000 in all) are streamed for four
 *                 query heads of a KV head at once, one load of a token row
 *                 for the four (a suffix plan for such a call is cut for the
 *                 count ph_decode_suffix_lanes(.., kv_group = G) returns).
 *                 0 = any mapping: every phase runs per request.
 * Everything else as ph_decode_attention (workspace: the same
 * ph_decode_workspace_bytes). */
int ph_decode_attention_gqa(void* out, const void* q, const void* k_cache, const void* v_cache,
                            int64_t num_reqs, int64_t num_heads, int64_t num_kv_heads,
                            const int32_t* head_mapping, int64_t kv_group, int64_t head_dim, int dtype,
                            int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                            float scale,
                            int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                            const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                            int64_t max_prefix_len,
                            const int32_t* suffix_slots, const int64_t* suffix_offsets,
                            int64_t suffix_table_stride, int64_t suffix_slots_count,
                            const int32_t* suffix_lens, int64_t max_suffix_len,
                            int64_t chunk_tokens, const ph_suffix_plan* plan,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ph_decode_attention without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, serving loops with a
 * fixed memory plan, harnesses that forbid hipMalloc).  No counterpart in the
 * reference, whose launcher lets torch allocate its temporaries
 * (shared_flash_decoding.py:298-313).  Same arguments, same kernels, same
 * results; the partials live in an array of ph_decode_static_scratch_bytes()
 * (32 MiB) that the library holds on every device it runs on until the process
 * ends.  The call allocates and frees nothing.  A shape whose
 * ph_decode_workspace_bytes() exceeds the array returns PH_ERR_SCRATCH before
 * anything is launched (config 2, batch 64 x 32 x 128 with a 4096-token prefix,
 * needs 13.9 MB; config 5, 128 x 40 x 128 in four groups, 15 MB).  All calls on
 * one device share the array: calls that overlap on one device (two streams,
 * two threads) race on it -- serialise them, or use ph_decode_attention with a
 * workspace per stream.  The first call on a device asks the runtime for the
 * array's address (hipGetSymbolAddress, once per device): make that call
 * outside stream capture; later calls only launch kernels. */
size_t ph_decode_static_scratch_bytes(void);

int ph_decode_attention_static(void* out, const void* q, const void* k_cache, const void* v_cache,
                               int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                               int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                               float scale,
                               int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                               const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                               int64_t max_prefix_len,
                               const int32_t* suffix_slots, const int64_t* suffix_offsets,
                               int64_t suffix_table_stride, int64_t suffix_slots_count,
                               const int32_t* suffix_lens,
                               int64_t max_suffix_len, int64_t chunk_tokens,
                               const ph_suffix_plan* plan, void* stream);

/* The two halves of the shared-prefix op, exposed separately because the
 * reference's extension does (csrc/attention.cpp:19-47):
 *
 * ph_prefix_attention: prefix phase only -- writes the normalised O (element
 * type), and m / l as fp32 [B, H].  Replaces triton_flash_attention(...,
 * save_mid_results=True) (shared_flash_decoding.py:202-277).
 *
 * ph_suffix_post_attention: suffix phase, then merge with the partial that
 * already sits in out / prev_m / prev_l; out is in/out.  Replaces
 * attention_ops.single_query_cached_kv_post_attention
 * (csrc/attention/attention_post_kernels.cu:74-341). */
int ph_prefix_attention(void* out, float* m_out, float* l_out,
                        const void* q, const void* k_cache, const void* v_cache,
                        int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                        int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                        const int32_t* prefix_slots, int64_t prefix_len,
                        void* workspace, size_t workspace_bytes, void* stream);

int ph_suffix_post_attention(void* out, const float* prev_m, const float* prev_l,
                             const void* q, const void* k_cache, const void* v_cache,
                             int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                             int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                             const int32_t* suffix_slots, const int64_t* suffix_offsets,
                             int64_t suffix_table_stride, int64_t suffix_slots_count,
                             const int32_t* suffix_lens,
                             int64_t max_suffix_len, int64_t chunk_tokens,
                             void* workspace, size_t workspace_bytes, void* stream);

/* The other order, which the reference's extension exports as well
 * (csrc/attention.cpp:19-32, shared_flash_decoding.py:332-376): suffix phase
 * first, prefix phase second.
 *
 * ph_suffix_prev_attention: suffix phase only -- writes the normalised O
 * (element type) and m / l as fp32 [B, H] (m in the exp2 domain, l relative to
 * m; l == 0 where a request has no suffix).  Replaces
 * attention_ops.single_query_cached_kv_prev_attention
 * (csrc/attention/attention_prev_kernels.cu:74-338).
 *
 * ph_prefix_post_attention: prefix phase over one shared slot list, then
 * merge with the partial that already sits in out / prev_m / prev_l; out is
 * in/out.  Replaces triton_flash_attention(..., load_mid_results=True)
 * (shared_flash_decoding.py:202-277,332-376). */
int ph_suffix_prev_attention(void* out, float* m_out, float* l_out,
                             const void* q, const void* k_cache, const void* v_cache,
                             int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                             int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                             const int32_t* suffix_slots, const int64_t* suffix_offsets,
                             int64_t suffix_table_stride, int64_t suffix_slots_count,
                             const int32_t* suffix_lens,
                             int64_t max_suffix_len, int64_t chunk_tokens,
                             void* workspace, size_t workspace_bytes, void* stream);

int ph_prefix_post_attention(void* out, const float* prev_m, const float* prev_l,
                             const void* q, const void* k_cache, const void* v_cache,
                             int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                             int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                             const int32_t* prefix_slots, int64_t prefix_len,
                             void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Prefill with parent context: packed ragged chunks, each causal
 * (bottom-right aligned) over ancestors' + own KV read through a slot table.
 * Replaces the gather (move_tokens_from_blocked_{k,v}_cache) + xformers
 * memory_efficient_attention_forward with
 * BlockDiagonalCausalFromBottomRightMask of
 * parrot/engine/builtin/attn_func.py:635-674, i.e. the kernel declared and left
 * unimplemented in parrot/engine/builtin/kernels/flash_attention_with_context.py:37-56.
 * q, out: [T, H, D] packed chunk after chunk, row strides q_stride/out_stride.
 * q_cu:  int32 [num_chunks+1] query offsets (DEVICE);
 * kv_cu: int32 [num_chunks+1] offsets into ctx_slots (DEVICE);
 * ctx_slots: int32 [ctx_slots_count], every chunk's whole context (ancestors || own), in order.
 * Query r of chunk c sees key j iff j <= r + (kv_len_c - q_len_c).
 * The new tokens' K/V must already be in the cache (append first).
 * max_kv_len: host upper bound of any chunk's context length.
 * workspace: at least ph_prefill_workspace_bytes(...) bytes, 256-byte aligned. */
size_t ph_prefill_workspace_bytes(int64_t num_tokens, int64_t num_heads, int64_t head_dim, int dtype,
                                  int64_t max_kv_len);

int ph_prefill_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                         int64_t num_tokens, int64_t num_chunks, int64_t num_heads, int64_t head_dim,
                         int dtype, int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                         float scale, const int32_t* q_cu, const int32_t* kv_cu,
                         const int32_t* ctx_slots, int64_t ctx_slots_count, int64_t max_kv_len,
                         void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Fused forms of the small per-layer ops (same arithmetic as the unfused
 * sequences, one launch each).
 *
 * ph_add_rms_norm: residual += x (stored back, rounded to the element type),
 * out = RMSNorm(residual) * weight.  Replaces the torch residual add of
 * parrot/engine/builtin/models/llama.py:160-178 followed by rms_norm
 * (3rdparty/vllm/csrc/layernorm_kernels.cu:9-63 for round_before_weight = 1,
 * parrot/engine/builtin/kernels/rms_norm.py:15-78 for 0).  Strides in elements.
 *
 * ph_silu_mul: out = silu(gate) * up, silu in fp32 rounded to the element
 * type, then the product -- silu_and_mul of
 * 3rdparty/vllm/csrc/activation_kernels.cu:6-48 with gate and up given by
 * pointer and row stride (gate = input, up = input + d for its [T, 2d] form),
 * and the act_fn(gate) * up of the Hugging Face LlamaMLP the reference imports
 * (models/llama.py:36-39).
 *
 * ph_rope_append: NeoX rotation of q and k in place (as ph_rope_neox), then
 * the rotated k rows and the v rows go to their slots (as ph_kv_append) --
 * one pass over k instead of two.  Replaces rotary_embedding_neox +
 * reshape_and_cache (pos_encoding_kernels.cu:38-104, cache_kernels.cu:142-224)
 * as called back to back in models/llama.py:122-129 / attn_func.py:143-155.
 * k_in_place = 1: k holds the rotated rows afterwards, as after the reference's
 * two calls.  k_in_place = 0: the rotated k rows go to the cache only and the
 * contents of k after the call are unspecified -- for a caller whose attention
 * reads K from the cache (the model code does: attn_func.py:143-155 appends, then
 * every kernel gathers from the cache); the pass then skips the write-back of
 * the k rows. */
int ph_add_rms_norm(void* out, void* residual, const void* x, const void* weight, float eps,
                    int64_t rows, int64_t n, int64_t x_stride, int64_t residual_stride,
                    int64_t out_stride, int dtype, int round_before_weight, void* stream);

int ph_silu_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t d,
                int64_t gate_stride, int64_t up_stride, int64_t out_stride, int dtype, void* stream);

int ph_rope_append(const int64_t* positions, void* q, void* k, const void* v,
                   const void* cos_sin_cache, void* k_cache, void* v_cache,
                   const void* slot_mapping, int index_type, int64_t num_tokens,
                   int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim, int64_t rot_dim,
                   int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t cache_stride_n,
                   int dtype, int k_in_place, void* stream);

/* ------------------------------------------------------------------------ */
/* Incremental suffix tables.  The reference rebuilds paged_block_tables /
 * paged_context_lens from Python lists and uploads them every iteration
 * (parrot/engine/builtin/attn_func.py:523-531,553-569); between two decode
 * iterations of the same batch each request's list only gains the slot of the
 * token being generated, so the device tables are patched instead:
 *   table[rows[i] * table_stride + lens[rows[i]]] = new_slots[i];  lens[rows[i]] += 1
 * for i < n.  rows (DEVICE int32, unique; NULL = identity) maps the caller's
 * request order to table rows; a row that is already table_stride long is left
 * untouched (the caller widens the table first).  All pointers DEVICE. */
int ph_suffix_tables_append(int32_t* table, int64_t table_stride, int32_t* lens, const int32_t* rows,
                            const int32_t* new_slots, int64_t n, void* stream);

/* Balanced suffix plan built on the device from the length vector alone (the
 * three arrays of ph_suffix_plan; see ph_decode_attention): one small launch
 * per iteration in place of host-side list work and an upload.  items must
 * hold num_lanes + num_reqs entries of 4 ints, lane_rec num_lanes entries of
 * 8, req_item_cu num_reqs + 1.  The stream is cut into
 * min(num_lanes, ceil(total / 4)) pieces; records of the remaining lanes are
 * empty.  num_reqs <= 8192; the lengths must sum to less than 2^31; a length
 * is read as min(max(len, 0), max_suffix_len), the same clamp the attention
 * kernels apply (pass the max_suffix_len of the ph_decode_attention call).
 * The reference has no counterpart (its kernels take fixed-size blocks per
 * request, attention_post_kernels.cu:74-110). */
int ph_suffix_plan_build(const int32_t* suffix_lens, int64_t num_reqs, int64_t max_suffix_len,
                         int64_t num_lanes, int32_t* items, int32_t* lane_rec, int32_t* req_item_cu,
                         void* stream);

/* ------------------------------------------------------------------------ */
/* Token sampler: temperature, top-p filter and one draw per row, in one launch.
 * Replaces the body of Sampler.forward after the logits GEMM
 * (parrot/engine/builtin/models/sampler.py:33-64: division by the
 * temperature in the logits' element type, descending sort, soft-max,
 * cumulative sum, mask, gather back through an arg-sort, soft-max,
 * torch.multinomial).  Per row r:
 *   x = logits[r] / temperature[r]   (rounded to the element type; skipped at 1)
 *   token i survives iff the soft-max mass of the tokens sorted before it
 *   (descending x, equal values by ascending id) is <= top_p[r];
 *   out_ids[r] = the first id whose cumulative surviving mass, in ascending id
 *   order, exceeds uniform[r] * (surviving mass).
 * The filter is found by bisection over the element type's ordered bit
 * patterns instead of a sort.  uniform[r] in [0, 1) comes from the caller's
 * random generator, so the draw is reproducible from the inputs; the
 * distribution of the drawn token is that of the reference, the mapping from
 * a seed to a token is not (that one is torch.multinomial's).
 * temperature == NULL means 1 for every row, top_p == NULL means 1 (no
 * filter); a temperature <= 0 selects the most likely token.  logits
 * [rows, vocab] with row_stride elements between rows, dtype PH_F16, PH_BF16
 * or PH_F32; temperature, top_p, uniform: float32 [rows]; out_ids int64 [rows].
 * All pointers DEVICE. */
int ph_sample_top_p(const void* logits, int64_t row_stride, const float* temperature,
                    const float* top_p, const float* uniform, int64_t* out_ids, int64_t rows,
                    int64_t vocab, int dtype, void* stream);

/* The same temperature and top-p filter without the draw: probs[r, i] = the
 * renormalised soft-max probability of token i of row r, 0 for tokens the
 * filter drops -- the tensor the reference hands to torch.multinomial
 * (parrot/engine/builtin/models/sampler.py:58-64).  A caller that wants the
 * reference's own draw (the library's random stream: same seed, same kind of
 * call) runs torch.multinomial(probs, 1, replacement=True) on it.
 * probs: float32 [rows, vocab], probs_stride floats between rows. */
int ph_top_p_probs(const void* logits, int64_t row_stride, const float* temperature,
                   const float* top_p, float* probs, int64_t probs_stride, int64_t rows,
                   int64_t vocab, int dtype, void* stream);

/* ------------------------------------------------------------------------ */
/* Instrumentation (no counterpart in the reference, which times whole
 * iterations from Python, parrot/engine/builtin/builtin_runner.py:158-175).
 * ph_decode_attention with one more argument: events6, six hipEvent_t handles
 * created and owned by the caller.  The call's prefix, suffix and merge
 * kernels are launched with (start, stop) event pairs that carry each
 * dispatch's own begin and end timestamps: events6[0,1] prefix kernel,
 * events6[2,3] suffix kernel (or the kernel that runs both phases),
 * events6[4,5] merge kernel; read them with hipEventElapsedTime after
 * synchronising.  A pair whose kernel the call does not launch is left
 * untouched.  events6 == NULL is exactly ph_decode_attention.  The events
 * travel with the call: the library keeps no state between calls. */
int ph_decode_attention_timed(void* out, const void* q, const void* k_cache, const void* v_cache,
                              int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                              int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                              float scale,
                              int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                              const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                              int64_t max_prefix_len,
                              const int32_t* suffix_slots, const int64_t* suffix_offsets,
                              int64_t suffix_table_stride, int64_t suffix_slots_count,
                              const int32_t* suffix_lens,
                              int64_t max_suffix_len, int64_t chunk_tokens,
                              const ph_suffix_plan* plan,
                              void* workspace, size_t workspace_bytes, void* stream,
                              void* const* events6);

#ifdef __cplusplus
}
#endif
#endif /* PARROT_HIP_H */
