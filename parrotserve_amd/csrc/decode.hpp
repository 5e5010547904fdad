// Argument blocks shared by the decode-attention kernels and their host entry
// points.  Partials live in a caller-provided workspace:
//   opart [parts, B, H, D] fp32 (normalised O of each part)
//   ml    [parts, B, H, 2] fp32 (m in the exp2 domain, l; l == 0 marks an empty part)
#pragma once

#include "common.hpp"

namespace ph {

struct PartialArgs {
  const uint16_t* q;
  int64_t q_stride;
  const uint16_t* kc;
  const uint16_t* vc;
  int64_t row_stride;       // elements between consecutive slots
  const int32_t* slots;     // slot table base
  int64_t slots_total;      // entries readable behind `slots` (speculative reads are clamped to it)
  const int64_t* offsets;   // per-request start inside `slots`, or null
  int64_t table_stride;     // start = b * table_stride when offsets is null
  const int32_t* lens;      // per-request list length
  int max_len;              // host bound of any list's length: a length read from `lens` is clamped to [0, max_len]
  const int32_t* shared_cu; // if set: every request uses slots[cu[0] .. cu[1])
  int shared_len;           // if >= 0 (and shared_cu null): every request uses slots[0 .. shared_len)
  int chunk;                // tokens per part
  int n_chunks;             // parts per request in this launch (grid extent)
  int part_base;            // first part index written
  float* opart;
  float* ml;
  int B, H;                 // full batch size / head count (workspace extents)
  int req_begin, num_reqs;  // requests covered by this launch
  float scale_log2e;
  const int32_t* head_map;  // KV head of each query head (device, [H]); null = query head h reads KV head h
};

// Balanced (host-planned) suffix phase; partial rows are [item][H].
struct ItemArgs {
  const uint16_t* q;
  int64_t q_stride;
  const uint16_t* kc;
  const uint16_t* vc;
  int64_t row_stride;
  const int32_t* slots;
  const int64_t* offsets;      // per-request start inside `slots`, or null
  int64_t table_stride;
  const int4* items;           // (request, first token, token count, 0)
  const int4* lane_rec;        // [num_lanes][2]: (first item, item count, request, first token), (count, 0, 0, 0)
  int num_lanes;
  float* opart;                // already offset to the items' first row
  float* ml;
  int H;
  float scale_log2e;
  const int32_t* head_map;     // KV head of each query head (device, [H]); null = identity
  int nq;                      // > 1: runs of nq adjacent query heads are streamed together against the KV head they
                               // share, the waves dividing the H / nq runs (head size 128, 16-bit); else 0 / 1
  int kv_shift;                // nq > 1: run r reads KV head r >> kv_shift (query head h reads KV head h / (nq << kv_shift))
};

// Query heads streamed together in the balanced suffix form (ItemArgs.nq) where the form exists: 4 when the
// mapping is the plain h / G with G a power of two from 4 on (a KV head's heads are G / 4 runs of 4) at head size 128
// and 16-bit elements, else 1.  (Runs of 8 for G = 8 were measured slower than two runs of 4: 72 against 57 us at
// 64 requests x 64 / 8 heads, suffixes of up to 512 tokens over a 4096-token prefix.)
inline int grouped_stream_heads(int64_t kv_group, int D, int dtype) {
  const bool pow2 = kv_group >= 4 && kv_group <= 64 && (kv_group & (kv_group - 1)) == 0;
  return pow2 && D == 128 && (dtype == PH_F16 || dtype == PH_BF16) ? 4 : 1;
}

struct MergeArgs {
  const float* opart;
  const float* ml;
  // Head pairs (D = 64 only): parts [0, nA) were written by the 128-wide matrix-core kernel on a query set in which
  // request b, head 2p + s is row 2b + s, head p, with the other head's half of the query zeroed; they live in
  // their own buffers, rows of 128 floats [part][2B][H/2], of which dims [64 s, 64 s + 64) are this head's output.
  const float* opart_pairs;
  const float* ml_pairs;
  uint16_t* out;
  int64_t out_stride;
  int B, H;
  int gshift;               // log2 G when parts [0, nA) were written on G rows per request and H / G KV heads
                            // (grouped KV heads on the matrix-core kernel), 0 otherwise
  int nA;                   // parts [0, nA) are candidates for every request
  int baseB;                // parts [baseB, baseB + ceil(lens[b]/chunk)) likewise
  const int32_t* lens;      // may be null (no B range)
  int max_len;              // lengths read from `lens` are clamped to [0, max_len] ...
  const int64_t* offsets;   // ... and, when slots_total > 0, to the entries behind the request's list start
  int64_t table_stride;     //     (offsets[b], or b * table_stride): the clamp of the kernel that wrote the parts
  int64_t slots_total;
  int chunk;
  const int32_t* req_item_cu; // balanced form: request b owns items [cu[b], cu[b+1]) ...
  int64_t item_base;          // ... whose partial rows start at item_base (rows of H)
  const float* prev_m;      // optional partial already in out/prev_m/prev_l
  const float* prev_l;
  float* m_out;             // optional export of the merged m / l
  float* l_out;
};

// Length of request b's slot list as every kernel reads it: the device value clamped to [0, max_len] and to the
// entries the table holds behind the list's start (a corrupt length then reads a wrong token of the same table
// instead of unmapped memory, and the kernels that write parts and the one that merges them agree on the count).
__device__ __forceinline__ int clamped_list_len(const int32_t* lens, int b, int max_len, int64_t off,
                                                int64_t slots_total) {
  const int64_t len = min(max(lens[b], 0), max_len);
  const int64_t room = slots_total - off;
  return (int)max((int64_t)0, min(len, room));
}

struct PrefixArgs {
  const uint16_t* q;
  int64_t q_stride;
  const uint16_t* kc;
  const uint16_t* vc;
  int64_t row_stride;
  const int32_t* slots;        // all groups' prefix slots
  const int32_t* prefix_cu;    // [G+1] device
  const int32_t* group_req_cu; // [G+1] device
  int req_shift;               // rows per request = 1 << req_shift; B counts rows and H what a row's heads are:
                               //   gqa == 0, req_shift == 1: 64-wide heads on head pairs -- row 2b + s is request b,
                               //     half s, H head pairs, q is the real [B][2 H][64] tensor;
                               //   gqa == 1: G = 1 << req_shift query heads share each KV head -- row b G + j is
                               //     request b, query head (KV head) G + j; H counts KV heads, q is [B][H G][128]
  int gqa;
  int head_dim;                // 0 / 128, or 80 / 96 / 112: a short head on the 128-wide tile (set by launch_prefix_mfma)
  int fixed_prefix_len;        // used when prefix_cu is null: one group, all requests, slots[0 .. len)
  int split_tokens;            // tokens per split (multiple of the tile)
  int n_splits;                // parts [0, n_splits)
  float* opart;
  float* ml;
  int B, H;
  float scale_log2e;
};

struct PrefillArgs {
  const uint16_t* q;
  int64_t q_stride;
  const uint16_t* kc;
  const uint16_t* vc;
  int64_t row_stride;
  uint16_t* out;
  int64_t out_stride;
  const int32_t* q_cu;       // [C+1] device
  const int32_t* kv_cu;      // [C+1] device
  const int32_t* ctx_slots;
  int32_t* tile_cu;          // [C+1] scratch: 64-query tiles before each chunk
  int num_chunks;
  int H;
  float scale_log2e;
  int pair;                  // 1: heads are 64 wide and run as halves of 128-wide head pairs (q, out, caches [.., H, 64])
  int tile_row0;             // first tile row of this launch (grid.y covers rows tile_row0 ..)
  int head_dim;              // 0 / 128, or 80 / 96 / 112: a short head on the 128-wide tile (set by launch_prefill_mfma)
};

int launch_partial(const PartialArgs& a, int dtype, int D, hipStream_t st, const KernelEvents& ev = KernelEvents());
// MFMA prefill: grid (head, query tile); num_tokens = total query rows (bounds the tile count).
int launch_prefill_mfma(const PrefillArgs& a, int dtype, int D, int64_t num_tokens, hipStream_t st);
int launch_items(const ItemArgs& a, int dtype, int D, hipStream_t st, const KernelEvents& ev = KernelEvents());
int launch_merge(const MergeArgs& a, int dtype, int D, hipStream_t st, const KernelEvents& ev = KernelEvents());
int launch_clear_ml(float* ml, int64_t entries, hipStream_t st);
// balanced suffix plan written on the device from the length vector (tables.hip); arrays as in ph_suffix_plan
constexpr int kPlanMaxReqs = 8192;
// lengths are clamped to [0, max_len]
int launch_suffix_plan(const int32_t* lens, int B, int max_len, int lanes, int32_t* items, int32_t* lane_rec,
                       int32_t* req_item_cu, hipStream_t st);
// MFMA shared-prefix kernel: grid (split, head, group x m-tile).  internal_ml: the parts' (m, l) only feed the
// call's own merge (not exported to the caller), which frees the kernel to pre-scale and re-round the query.
int launch_prefix_mfma(const PrefixArgs& a, int dtype, int D, int num_groups, int max_group_reqs, bool internal_ml,
                       hipStream_t st, const KernelEvents& ev = KernelEvents());
bool prefix_mfma_supported(int dtype, int D);
// Prefix + suffix phases in one launch (see decode_fused_kernel); cus = compute units of the device;
// prefix_wgs > 0: that many workgroups run only prefix units and the others only suffix pieces, 0: every
// workgroup runs both.
bool decode_fused_supported(int dtype, int D);
int launch_decode_fused(const PrefixArgs& a, const ItemArgs& ia, int dtype, int num_groups, int max_group_reqs, int cus,
                        int prefix_wgs, hipStream_t st, const KernelEvents& ev = KernelEvents());

}  // namespace ph
