// Host entry points of the decode-attention family: launch geometry, workspace
// carving, argument checks.  No allocation, no synchronisation: everything is
// enqueued on the caller's stream.
#include "decode.hpp"

#include <algorithm>
#include <mutex>

namespace ph {

// Scratch of ph_decode_attention_static: the partials workspace of a decode call, held by the library for
// callers that cannot allocate.  Every device the library runs on holds its own copy until the process ends.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device.  The array's name is a host-side stand-in for the symbol,
// not an address a kernel can use: the address is asked for once per device and kept.
static int static_scratch_ptr(void** out) {
  static std::mutex mu;
  static void* ptrs[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return PH_ERR_ARG;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
      (void)hipGetLastError();
      return PH_ERR_LAUNCH;
    }
    ptrs[dev] = p;
  }
  *out = ptrs[dev];
  return PH_OK;
}

struct DecodePlan {
  int chunk;         // suffix tokens per part (grid form)
  int n_chunks;      // suffix parts per request (grid form)
  int split_tokens;  // prefix tokens per part
  int n_splits;      // prefix parts
  int64_t items;     // suffix items (balanced form), 0 in the grid form
  int dev_lanes;     // lanes of a plan the library builds on the device into the workspace (0: the caller's plan or none)
  bool paired;       // D == 64: the prefix phase runs on head pairs through the 128-wide matrix-core kernel
  int prefix_wgs;    // fused launch: workgroups that run only prefix units (0: every workgroup runs both phases)
  int parts() const { return n_chunks + n_splits; }
  // partial rows (one row = one head's (O, m, l)): [parts][B][H] then [items][H]
  size_t rows(int64_t B, int64_t H) const { return (size_t)parts() * B * H + (size_t)items * H; }
};

static int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
static int64_t cdiv(int64_t x, int64_t m) { return (x + m - 1) / m; }

constexpr int kPrefixTile = 64;        // tokens per LDS tile of the MFMA kernel
constexpr int kPrefixQueryTile = 64;   // queries per workgroup of the MFMA kernel

// compute units of the current device (cached per device id)
static int device_cus() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

// Query heads that share KV heads, as the planner sees them: mfma_group = G when the prefix phase runs the G query
// heads of a KV head as G rows per request on H / G heads (1: plain), stream_group = query heads the suffix waves
// stream together per KV head (grouped_stream_heads: G or 1).
struct HeadGrouping {
  int64_t mfma_group = 1;
  int stream_group = 1;
};

// waves that one suffix piece occupies: the streamed heads (KV heads when their query heads go together) over the
// heads a wave holds
static int64_t suffix_head_groups(int64_t H, int64_t D, int stream_group) {
  return cdiv(H / std::max(1, stream_group), std::max(1, 64 / lanes_per_head((int)D)));
}

// What the planner knows of a decode call's two phases.  The suffix volume is an estimate from what the host
// knows -- half the longest list per request.
struct FusedShape {
  int64_t units_per_split;  // prefix units (head x group x query tile) per split of the prefix
  int64_t reqs, head_groups;  // requests; waves that one suffix piece occupies (heads / heads per wave)
  int64_t group_rows, query_tile;  // query rows of a group as the matrix-core kernel sees them; its tile: 64 / 128 / 256
  double prefix_mb, suffix_mb;
  double stream_mb_per_us;  // what one compute unit of suffix waves streams
};
static FusedShape fused_shape(int64_t B, int64_t H, int64_t D, int64_t groups, int64_t max_prefix, int64_t max_suffix,
                              bool paired, const HeadGrouping& hg = HeadGrouping()) {
  FusedShape f{};
  if (groups <= 0 || max_prefix <= 0) return f;
  const int64_t G = std::max<int64_t>(1, hg.mfma_group);
  // what the matrix-core kernel sees
  const int64_t rows_b = paired ? 2 * B : B * G, rows_h = paired ? H / 2 : H / G;
  f.group_rows = cdiv(rows_b, groups);
  f.query_tile = f.group_rows <= 64 ? 64 : f.group_rows <= 128 ? 128 : 256;
  const int64_t mtiles = cdiv(f.group_rows, f.query_tile);
  f.units_per_split = groups * rows_h * (mtiles > 0 ? mtiles : 1);
  f.reqs = B;
  f.head_groups = suffix_head_groups(H, D, hg.stream_group);
  const double row_mb = (double)(H / G) * D * 4 / 1e6;  // K and V of one token, 16-bit elements
  // 40 GB/s when every load instruction brings rows of its own; query heads that share a KV head re-read its rows
  // (G loads per row), or, streamed together, meet each row with stream_group queries (bound by the vector ALUs)
  f.stream_mb_per_us = hg.stream_group > 1 ? 0.096 / hg.stream_group : 0.040 / (double)G;
  f.prefix_mb = (double)groups * max_prefix * row_mb;
  f.suffix_mb = (double)B * max_suffix / 2 * row_mb;
  return f;
}

constexpr double kHbmMbPerUs = 6.9;  // what the device sustains on this access mix

// Roles: the split count and the number of prefix-only workgroups.  A prefix workgroup is latency-bound next to
// the suffix stream -- one 128-token step (64 KB) in flight ahead of the one it multiplies, about 2.7 us per step
// with the memory system saturated, 12 us from launch to its first step -- so the prefix wants enough workgroups
// to be done a little before the stream, and the stream wants the rest (it holds about 40 GB/s per compute unit).
// A suffix wave spends about 4 us per piece before it streams (slot ids, then rows, then the partial's write), and
// a lane walks at least requests / lanes pieces: with many short lists on few lanes that, not the bytes, is what
// the suffix workgroups take (256 requests x 16 tokens on 32 lanes: 69 us; on 64 lanes: 54.5 us).
// Both end no earlier than the bytes of the launch take at the rate the device sustains.
struct RoleChoice {
  int splits, prefix_wgs;
  double cost_us;
};
static RoleChoice choose_roles(const FusedShape& f, int64_t max_prefix, int64_t cus) {
  constexpr double kHbm = kHbmMbPerUs;  // MB per us
  const double kCu = f.stream_mb_per_us;
  constexpr double kStep = 2.7, kFirst = 12.0, kFold = 2.0, kNext = 6.0, kMargin = 3.0, kPiece = 4.0;
  const double floor_us = 4.0 + (f.prefix_mb + f.suffix_mb) / kHbm;
  // a step of the 128- and 256-query tiles is twice and four times the matrix work of the 64-query tile's
  const double tile_mul = f.query_tile == 256 ? 1.5 : f.query_tile == 128 ? 1.1 : 1.0;
  RoleChoice best{1, 1, 0.0};
  double best_cost = -1.0;
  const int64_t max_splits = std::max<int64_t>(1, cdiv(max_prefix, 4 * kPrefixTile));
  for (int64_t s = 1; s <= 64 && s <= max_splits; ++s) {
    const int64_t tok = round_up(cdiv(max_prefix, s), 2 * kPrefixTile);
    if (cdiv(max_prefix, tok) != s) continue;  // rounding left a split empty: the same plan as a smaller s
    const double steps = (double)cdiv(tok, 2 * kPrefixTile);
    const int64_t units = f.units_per_split * s;
    for (int64_t r = 1; r <= 8; ++r) {
      const int64_t np = cdiv(units, r);
      if (np > cus - 1) continue;
      const double t_prefix = kFirst + r * (steps * kStep * tile_mul + kFold) + (r - 1) * kNext + kMargin;
      const int64_t lanes = std::max<int64_t>(1, (cus - np) * 8 / f.head_groups);
      const double t_suffix =
          6.0 + (double)cdiv(f.reqs, lanes) * kPiece + f.suffix_mb / std::min(kHbm, (double)(cus - np) * kCu);
      const double cost = std::max(std::max(t_prefix, t_suffix), floor_us) + 0.25 * s;
      if (best_cost < 0 || cost < best_cost) {
        best_cost = cost;
        best = RoleChoice{(int)s, (int)np, cost};
      }
    }
  }
  return best;
}

// The other form: every workgroup runs both phases, its suffix pieces first (groups of over 32 rows; smaller ones
// take a prefix launch on the four-wave tile, then the suffix launch) -- the phases one after the other, each on
// every compute unit.  Split count: one workgroup per compute unit at a time (the kernel uses most of the register
// file), so the count whose workgroup total wastes the least of a whole number of rounds over the device, at
// rounds x (tokens per split + a fixed prologue / epilogue worth ~96 tokens).  cost_us is on the scale of
// choose_roles' cost, which overstates a lightly loaded launch (its 12 us to the first step and 2.7 us per step are
// what a prefix workgroup sees next to a saturating stream): the estimate of this form's time plus 11.5 us, that
// offset fitted, with the step time of this form (3.1 us; x 1.44 on the 256-query tile, x 0.87 on the four-wave
// tile) and its 9.3 us of start and end, to 106 shapes measured in both forms --
// 1 .. 16 groups of 1 .. 256 requests, prefixes of 128 .. 16384 tokens, suffixes of up to 8 .. 4096 tokens, 32 and
// 40 heads of 128.  Choosing by the two costs is within 0.3 % of the better form on average over those shapes and
// 9 % at worst; the two phases in workgroups of their own win by 3 .. 25 % on most (small launches are chains of
// memory latencies, which then run side by side: 16 requests x 256 over 1024 tokens 19.3 against 25.6 us; the
// reference benchmark's 64 x 20 over 8192 at 40 heads 49.3 against 52.6 us) and lose by 3 .. 19 % where the prefix
// wants every compute unit: long prefixes under tiny suffixes, 256-query tiles under short suffixes, and many
// small groups whose units fill the device evenly (8 groups of 8 over 2000 tokens: 77 against 66 us).
struct SharedChoice {
  int splits;
  double cost_us;
};
static SharedChoice choose_shared(const FusedShape& f, int64_t max_prefix, int64_t cus) {
  const int64_t max_splits = std::max<int64_t>(1, cdiv(max_prefix, 4 * kPrefixTile));
  int64_t splits = 1, best = -1;
  for (int64_t s = 1; s <= 64 && s <= max_splits; ++s) {
    const int64_t tok = round_up(cdiv(max_prefix, s), 2 * kPrefixTile);
    const int64_t cost = cdiv(f.units_per_split * s, cus) * (tok + 96);
    if (best < 0 || cost < best) {
      best = cost;
      splits = s;
    }
  }
  const int64_t tok = round_up(cdiv(max_prefix, splits), 2 * kPrefixTile);
  const double steps = (double)cdiv(tok, 2 * kPrefixTile), rounds = (double)cdiv(f.units_per_split * cdiv(max_prefix, tok), cus);
  const double step_us = 3.1 * (f.query_tile == 256 ? 1.44 : 1.0) * (f.group_rows <= 32 ? 0.87 : 1.0);
  const double t = 9.3 + f.suffix_mb / kHbmMbPerUs + rounds * (steps * step_us + 2.0);
  constexpr double kRolesScale = 11.5;
  return SharedChoice{(int)splits, std::max(t, 4.0 + (f.prefix_mb + f.suffix_mb) / kHbmMbPerUs) + kRolesScale};
}

// plan_head_dim > 0: a caller without a plan of its own that leaves the chunk size to the library gets the
// balanced form from a plan built on the device (up to kPlanMaxReqs requests); an explicit chunk size keeps the
// plain (request, chunk) grid.  roles: the fused launch may give the two phases workgroups of their own.
static DecodePlan plan_decode(int64_t B, int64_t H, int64_t groups, int64_t max_prefix, int64_t max_suffix,
                              int64_t chunk_tokens, int64_t num_items = 0, int64_t plan_head_dim = 0,
                              bool paired = false, bool roles = false, const HeadGrouping& hg = HeadGrouping()) {
  DecodePlan p{};
  p.items = num_items;
  const int64_t cus = device_cus();
  if (groups > 0 && max_prefix > 0) {
    p.paired = paired;
    const FusedShape f =
        fused_shape(B, H, plan_head_dim > 0 ? plan_head_dim : 128, groups, max_prefix, max_suffix, paired, hg);
    const SharedChoice sc = choose_shared(f, max_prefix, cus);
    int64_t splits = sc.splits;
    if (roles && max_suffix > 0) {
      const RoleChoice rc = choose_roles(f, max_prefix, cus);
      if (rc.cost_us < sc.cost_us) {
        splits = rc.splits;
        p.prefix_wgs = rc.prefix_wgs;
      }
    }
    const int64_t st = round_up(cdiv(max_prefix, splits), 2 * kPrefixTile);
    p.split_tokens = (int)st;
    p.n_splits = (int)cdiv(max_prefix, st);
  }
  if (num_items > 0) {
    p.chunk = 32;
    p.n_chunks = 0;
  } else if (max_suffix > 0 && chunk_tokens <= 0 && plan_head_dim >= 8 && B <= kPlanMaxReqs) {
    // two waves per SIMD on the compute units the suffix phase has to itself
    const int64_t lanes = (cus - p.prefix_wgs) * 4 * 2 / suffix_head_groups(H, plan_head_dim, hg.stream_group);
    p.dev_lanes = (int)(lanes > 0 ? lanes : 1);
    p.items = p.dev_lanes + B;  // capacity: a cut at every lane mark and every request boundary
    p.chunk = 32;
    p.n_chunks = 0;
  } else if (max_suffix > 0) {
    int64_t chunk = chunk_tokens;
    if (chunk <= 0) {
      // Aim for about 2048 (request, chunk) items assuming mean length = max/2.
      const int64_t want = B * max_suffix / 2 / 2048;
      chunk = 32;
      while (chunk < want && chunk < 1024) chunk *= 2;
    }
    chunk = round_up(chunk, 16);
    p.chunk = (int)chunk;
    p.n_chunks = (int)cdiv(max_suffix, chunk);
  } else {
    p.chunk = 32;
    p.n_chunks = 0;
  }
  return p;
}

static size_t plan_bytes(const DecodePlan& p, int64_t B, int64_t H, int64_t D) {
  const size_t rows = p.rows(B, H);
  size_t n = round_up((int64_t)(rows * D * sizeof(float)), 256) + round_up((int64_t)(rows * 2 * sizeof(float)), 256);
  if (p.dev_lanes > 0)
    n += round_up(p.items * 16, 256) + round_up((int64_t)p.dev_lanes * 32, 256) + round_up((B + 1) * 4, 256);
  if (p.paired)  // the head-pair partials of the prefix parts
    n += round_up((int64_t)p.n_splits * B * H * 128 * 4, 256) + round_up((int64_t)p.n_splits * B * H * 2 * 4, 256);
  return n;
}

struct Carve {
  float* opart;
  float* ml;
  int32_t *items, *lane_rec, *req_item_cu;  // the device-built plan (dev_lanes > 0)
  float *opart_pairs, *ml_pairs;            // paired prefix phase: [n_splits][2B][H/2] partial rows of 128 floats / (m, l)
};
static Carve carve(void* ws, const DecodePlan& p, int64_t B, int64_t H, int64_t D) {
  const size_t rows = p.rows(B, H);
  Carve c{};
  char* at = (char*)ws;
  c.opart = (float*)at;
  at += round_up((int64_t)(rows * D * sizeof(float)), 256);
  c.ml = (float*)at;
  at += round_up((int64_t)(rows * 2 * sizeof(float)), 256);
  if (p.dev_lanes > 0) {
    c.items = (int32_t*)at;
    at += round_up(p.items * 16, 256);
    c.lane_rec = (int32_t*)at;
    at += round_up((int64_t)p.dev_lanes * 32, 256);
    c.req_item_cu = (int32_t*)at;
    at += round_up((B + 1) * 4, 256);
  }
  if (p.paired) {
    c.opart_pairs = (float*)at;
    at += round_up((int64_t)p.n_splits * B * H * 128 * 4, 256);
    c.ml_pairs = (float*)at;
  }
  return c;
}

// D == 64 with an even head count: two adjacent heads of a token row are one 128-wide row of the matrix-core
// kernel.  Request b, head 2p + s becomes row 2b + s, pseudo-head p, whose query (as the kernel loads it) is the
// head's 64 values in half s and zeros in the other half: the zeros cancel the neighbour's keys in the score, and half s of the
// 128-wide output is exactly the head's output (the other half, the neighbour's values under this head's
// weights, is ignored).  Twice the matrix work, the same K/V traffic -- read once per group, not once per request.
static bool pair_heads(int64_t D, int64_t H) { return D == 64 && H % 2 == 0; }

// How the query heads of a decode call map onto the KV heads of the pools (grouped / multi-query attention,
// csrc/attention/attention_post_kernels.cu:79,101).  map == null: query head h reads KV head h.
struct KvHeads {
  int64_t num_kv_heads = 0;       // 0: as many as query heads
  const int32_t* map = nullptr;   // device, [H]: KV head of each query head
  int64_t group = 0;              // host hint: > 0 asserts map[h] == h / group (H == group x num_kv_heads); 0: any map
};

static int check_common(const void* out, const void* q, const void* kc, const void* vc, int64_t B, int64_t H,
                        int64_t D, int dtype, int64_t q_stride, int64_t out_stride, int64_t row_stride,
                        int64_t kv_heads = 0) {
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (D != 64 && D != 80 && D != 96 && D != 112 && D != 128 && D != 256) return PH_ERR_HEAD_DIM;
  if (B < 0 || H <= 0 || B > (1 << 24) || H > 4096) return PH_ERR_ARG;
  if (B == 0) return PH_OK;
  if (!out || !q || !kc || !vc) return PH_ERR_ARG;
  if (q_stride < H * D || out_stride < H * D || row_stride < (kv_heads > 0 ? kv_heads : H) * D) return PH_ERR_ARG;
  if (!aligned16(out) || !aligned16(q) || !aligned16(kc) || !aligned16(vc) || q_stride % 8 || out_stride % 8 ||
      row_stride % 8)
    return PH_ERR_ALIGN;
  return PH_OK;
}

// Prefix phase: matrix-core kernel for head size 128; other head sizes run the
// per-request gather kernel once per group over the shared slot list.
// the prefix phase's arguments as the 128-wide kernel sees them when 64-wide heads run as head pairs
static PrefixArgs pair_args(const PrefixArgs& pa, const Carve& ws) {
  PrefixArgs w = pa;
  w.B = 2 * pa.B;
  w.H = pa.H / 2;
  w.req_shift = 1;
  w.opart = ws.opart_pairs;
  w.ml = ws.ml_pairs;
  return w;
}

// the prefix phase's arguments as the matrix-core kernel sees them when G = 1 << gshift query heads share each KV
// head: G rows per request, one "head" per KV head
static PrefixArgs gqa_args(const PrefixArgs& pa, int gshift) {
  PrefixArgs w = pa;
  w.B = pa.B << gshift;
  w.H = pa.H >> gshift;
  w.req_shift = gshift;
  w.gqa = 1;
  return w;
}

// log2 of the group size when the matrix-core kernel can take the query heads of a KV head as rows of one tile
// (a power of two up to 64, the plain h -> h / G map, head size 128, 16-bit elements); -1 otherwise
static int gqa_shift(const KvHeads& kv, int64_t H, int64_t D, int dtype) {
  if (!kv.map || kv.group < 2 || kv.group > 64 || (kv.group & (kv.group - 1)) || D != 128 ||
      !prefix_mfma_supported(dtype, 128) || kv.num_kv_heads * kv.group != H)
    return -1;
  int s = 0;
  while ((1 << s) < kv.group) ++s;
  return s;
}

// head_map != null with gshift < 0: any mapping, through the per-request kernel
static int run_prefix(PrefixArgs& pa, int dtype, int D, int num_groups, const int32_t* group_req_cu_host,
                      int max_group_reqs, bool internal_ml, hipStream_t st, const Carve* pairs = nullptr,
                      const KernelEvents& ev = KernelEvents(), const int32_t* head_map = nullptr, int gshift = -1) {
  if (pairs && pairs->opart_pairs)
    return launch_prefix_mfma(pair_args(pa, *pairs), dtype, 128, num_groups, 2 * max_group_reqs, internal_ml, st, ev);
  if (head_map && gshift > 0)
    return launch_prefix_mfma(gqa_args(pa, gshift), dtype, D, num_groups, max_group_reqs << gshift, internal_ml, st,
                              ev);
  if (!head_map && prefix_mfma_supported(dtype, D))
    return launch_prefix_mfma(pa, dtype, D, num_groups, max_group_reqs, internal_ml, st, ev);
  int rc = launch_clear_ml(pa.ml, (int64_t)pa.n_splits * pa.B * pa.H, st);
  if (rc != PH_OK) return rc;
  for (int g = 0; g < num_groups; ++g) {
    PartialArgs sa{};
    sa.q = pa.q;
    sa.q_stride = pa.q_stride;
    sa.kc = pa.kc;
    sa.vc = pa.vc;
    sa.row_stride = pa.row_stride;
    sa.slots = pa.slots;
    sa.shared_cu = pa.prefix_cu ? pa.prefix_cu + g : nullptr;
    sa.shared_len = pa.prefix_cu ? -1 : pa.fixed_prefix_len;
    sa.chunk = pa.split_tokens;
    sa.n_chunks = pa.n_splits;
    sa.part_base = 0;
    sa.opart = pa.opart;
    sa.ml = pa.ml;
    sa.B = pa.B;
    sa.H = pa.H;
    sa.req_begin = group_req_cu_host ? group_req_cu_host[g] : 0;
    sa.num_reqs = group_req_cu_host ? group_req_cu_host[g + 1] - group_req_cu_host[g] : pa.B;
    sa.scale_log2e = pa.scale_log2e;
    sa.head_map = head_map;
    rc = launch_partial(sa, dtype, D, st);
    if (rc != PH_OK) return rc;
  }
  return PH_OK;
}

// Per-token (offset, length) of the prefill-as-ragged-decode formulation.
__global__ __launch_bounds__(256) void prefill_rows_kernel(const int32_t* q_cu, const int32_t* kv_cu, int num_chunks,
                                                           int num_tokens, int64_t* offsets, int32_t* lens) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= num_tokens) return;
  int lo = 0, hi = num_chunks;  // last chunk with q_cu[c] <= i
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (q_cu[mid] <= i) lo = mid; else hi = mid;
  }
  const int qn = q_cu[lo + 1] - q_cu[lo];
  const int kvn = kv_cu[lo + 1] - kv_cu[lo];
  offsets[i] = kv_cu[lo];
  lens[i] = kvn - qn + (i - q_cu[lo]) + 1;
}

}  // namespace ph

using namespace ph;

extern "C" const char* ph_status_string(int status) {
  switch (status) {
    case PH_OK: return "ok";
    case PH_ERR_DTYPE: return "unsupported data type";
    case PH_ERR_HEAD_DIM: return "unsupported head size";
    case PH_ERR_ALIGN: return "pointer or stride not 16-byte aligned";
    case PH_ERR_ARG: return "invalid argument";
    case PH_ERR_WORKSPACE: return "workspace too small";
    case PH_ERR_LAUNCH: return "kernel launch failed";
    case PH_ERR_SCRATCH: return "shape needs more scratch than the library's static array holds (use the workspace form)";
    default: return "unknown status";
  }
}

extern "C" int ph_abi_version(void) { return 3; }

extern "C" size_t ph_decode_workspace_bytes(int64_t num_reqs, int64_t num_heads, int64_t head_dim,
                                            int64_t num_groups, int64_t max_prefix_len, int64_t max_suffix_len,
                                            int64_t chunk_tokens, int64_t num_items) {
  if (num_reqs <= 0 || num_heads <= 0 || head_dim <= 0) return 0;
  // the call picks one of two layouts (prefix and suffix workgroups of their own, or not) by what the element type
  // and the group sizes allow, and its split count and plan size follow how query heads share KV heads -- none of
  // which this query sees: large enough for every case
  size_t need = 0;
  for (int64_t group = 1; group <= 64 && group <= num_heads; group *= 2) {
    if (num_heads % group != 0) break;
    for (int stream = 0; stream < 2; ++stream) {
      HeadGrouping hg;
      hg.mfma_group = group;
      hg.stream_group = stream ? grouped_stream_heads(group, (int)head_dim, PH_F16) : 1;  // whatever the lengths
      if (stream && hg.stream_group == 1) continue;
      for (int roles = 0; roles < 2; ++roles) {
        const DecodePlan p = plan_decode(num_reqs, num_heads, num_groups, max_prefix_len, max_suffix_len, chunk_tokens,
                                         num_items, head_dim, pair_heads(head_dim, num_heads), roles != 0, hg);
        need = std::max(need, plan_bytes(p, num_reqs, num_heads, head_dim));
      }
    }
  }
  return need;
}

// How a call whose query heads share KV heads as h -> h / kv_group is planned: on the matrix cores with the group's
// heads as rows (a power of two up to 64, head size 128, 16-bit elements; gqa_shift() is the call's own test) and,
// where that form exists and the lists are long enough, with runs of the group streamed together in the suffix
// phase.  Long enough: the grouped form cuts the suffix into four times the pieces (a piece occupies a quarter of
// the waves), each with its ~4 us of start and its partial rows for the merge, so it wins from lists of ~100 tokens
// and ~8000 tokens in all on (64 requests x 32 / 8 heads, <= 512 tokens over 4096: 41.7 against 49.8 us; four
// groups of 32 x 64 / 8 heads, <= 1024 tokens over 6000: 134.5 against 195.6 us) and loses below (16 requests x
// <= 256 tokens: 28.4 against 23.4 us; 256 x <= 128 tokens: 67.1 against 64.5 us).  kv_group <= 1: plain.
static HeadGrouping head_grouping(int64_t kv_group, int64_t H, int64_t D, int dtype, int64_t B, int64_t max_suffix) {
  HeadGrouping hg;
  if (kv_group >= 2 && kv_group <= 64 && (kv_group & (kv_group - 1)) == 0 && D == 128 &&
      prefix_mfma_supported(dtype, 128) && H % kv_group == 0) {
    hg.mfma_group = kv_group;
    if (max_suffix >= 200 && B * max_suffix / 2 >= 8000) hg.stream_group = grouped_stream_heads(kv_group, (int)D, dtype);
  }
  return hg;
}

// can the prefix and suffix phases of this call share one launch with workgroups of their own?
static bool roles_possible(int64_t B, int64_t H, int64_t D, int dtype, bool has_prefix, bool has_suffix, bool planned,
                           int64_t chunk_tokens) {
  if (!has_prefix || !has_suffix) return false;
  if (!planned && !(chunk_tokens <= 0 && B <= kPlanMaxReqs)) return false;  // no balanced plan: the grid form
  return pair_heads(D, H) ? decode_fused_supported(dtype, 128) : decode_fused_supported(dtype, (int)D);
}

extern "C" int64_t ph_decode_suffix_lanes(int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                                          int64_t num_groups, int64_t max_prefix_len, int64_t max_suffix_len,
                                          int64_t kv_group) {
  if (num_reqs <= 0 || num_heads <= 0 || head_dim < 8) return 1;
  const bool has_prefix = num_groups > 0 && max_prefix_len > 0;
  const HeadGrouping hg = head_grouping(kv_group, num_heads, head_dim, dtype, num_reqs, max_suffix_len);
  const bool mfma_prefix = kv_group <= 1 || hg.mfma_group > 1;  // another mapping runs every phase per request
  const bool roles =
      mfma_prefix && roles_possible(num_reqs, num_heads, head_dim, dtype, has_prefix, max_suffix_len > 0, true, 0);
  const DecodePlan p = plan_decode(num_reqs, num_heads, has_prefix ? num_groups : 0, max_prefix_len, max_suffix_len, 0,
                                   1, head_dim, pair_heads(head_dim, num_heads), roles, hg);
  const int64_t lanes =
      ((int64_t)device_cus() - p.prefix_wgs) * 4 * 2 / suffix_head_groups(num_heads, head_dim, hg.stream_group);
  return lanes > 0 ? lanes : 1;
}

// events6: null, or (start, stop) event pairs for the prefix, suffix and merge kernels of this call
static int decode_attention_impl(void* out, const void* q, const void* k_cache, const void* v_cache,
                                 int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                                 int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                                 int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                                 const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                                 int64_t max_prefix_len, const int32_t* suffix_slots,
                                 const int64_t* suffix_offsets, int64_t suffix_table_stride,
                                 int64_t suffix_slots_count, const int32_t* suffix_lens, int64_t max_suffix_len,
                                 int64_t chunk_tokens, const ph_suffix_plan* plan, void* workspace,
                                 size_t workspace_bytes, void* stream, void* const* events6,
                                 const KvHeads& kv = KvHeads()) {
  const int B = (int)num_reqs, H = (int)num_heads, D = (int)head_dim;
  KernelEvents ev_prefix, ev_suffix, ev_merge;
  if (events6) {
    ev_prefix = KernelEvents{(hipEvent_t)events6[0], (hipEvent_t)events6[1]};
    ev_suffix = KernelEvents{(hipEvent_t)events6[2], (hipEvent_t)events6[3]};
    ev_merge = KernelEvents{(hipEvent_t)events6[4], (hipEvent_t)events6[5]};
  }
  if (kv.map && (kv.num_kv_heads <= 0 || kv.num_kv_heads > num_heads || kv.group < 0)) return PH_ERR_ARG;
  int rc = check_common(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                        cache_stride_n, kv.map ? kv.num_kv_heads : 0);
  if (rc != PH_OK || num_reqs == 0) return rc;
  if (num_groups < 0 || max_prefix_len < 0 || max_suffix_len < 0 || max_suffix_len > INT32_MAX) return PH_ERR_ARG;
  const bool has_prefix = num_groups > 0 && max_prefix_len > 0;
  const bool has_suffix = max_suffix_len > 0;
  if (has_prefix && (!prefix_slots || !prefix_cu || !group_req_cu || !group_req_cu_host)) return PH_ERR_ARG;
  const int gshift = gqa_shift(kv, num_heads, head_dim, dtype);  // > 0: the KV heads' query heads as matrix rows
  if (has_suffix && (!suffix_slots || !suffix_lens || suffix_slots_count <= 0)) return PH_ERR_ARG;
  // padded table: every row must hold max_suffix_len entries inside the table (the balanced form walks a row up to
  // its clamped length without knowing where the table ends)
  if (has_suffix && !suffix_offsets &&
      (suffix_table_stride < 0 || suffix_slots_count < (num_reqs - 1) * suffix_table_stride + max_suffix_len))
    return PH_ERR_ARG;
  bool planned = has_suffix && plan != nullptr && plan->num_items > 0;
  if (planned && (!plan->items || !plan->lane_rec || !plan->req_item_cu || plan->num_lanes <= 0 ||
                  plan->num_items > (int64_t)1 << 30))
    return PH_ERR_ARG;
  // a head mapping takes the 64-wide head pairs out (a pair's heads need not share anything); it runs on the
  // matrix cores as G rows per request when it is the plain h / G map at head size 128, else per request
  const bool paired = !kv.map && pair_heads(D, H) && prefix_mfma_supported(dtype, 128);
  const bool mfma_prefix = kv.map ? gshift > 0 : (paired || prefix_mfma_supported(dtype, D));
  const bool roles = mfma_prefix && roles_possible(num_reqs, num_heads, head_dim, dtype, has_prefix, has_suffix,
                                                   planned, chunk_tokens);
  // the planner's view of shared KV heads is the call's own: the same test as gqa_shift()
  const HeadGrouping hg =
      gshift > 0 ? head_grouping(kv.group, num_heads, head_dim, dtype, num_reqs, max_suffix_len) : HeadGrouping();
  DecodePlan p = plan_decode(num_reqs, num_heads, has_prefix ? num_groups : 0, max_prefix_len, max_suffix_len,
                             chunk_tokens, planned ? plan->num_items : 0, head_dim, pair_heads(D, H), roles, hg);
  if (planned && p.prefix_wgs > 0) {
    // A caller's plan cut into more pieces than the suffix-only workgroups have waves (a plan made for the whole
    // device: ph_decode_suffix_lanes was not asked, or for another shape) would take them a second round (config 2
    // with 170 pieces for 160 workgroups: 93 us against 66 us): such a plan gets the form it was cut for, every
    // workgroup running both phases (75 us).
    const int64_t fit = ((int64_t)device_cus() - p.prefix_wgs) * 8 / suffix_head_groups(H, D, hg.stream_group);
    if (plan->num_lanes > fit)
      p = plan_decode(num_reqs, num_heads, num_groups, max_prefix_len, max_suffix_len, chunk_tokens, plan->num_items,
                      head_dim, pair_heads(D, H), false, hg);
  }
  if (plan_bytes(p, B, H, D) > workspace_bytes || ((p.parts() > 0 || p.items > 0) && !workspace))
    return PH_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 255u) != 0) return PH_ERR_ALIGN;
  const Carve ws = carve(workspace, p, B, H, D);
  hipStream_t st = (hipStream_t)stream;
  ph_suffix_plan own_plan{};
  if (!planned && p.dev_lanes > 0) {  // no plan from the caller: one is built on the device first
    rc = launch_suffix_plan(suffix_lens, B, (int)max_suffix_len, p.dev_lanes, ws.items, ws.lane_rec, ws.req_item_cu, st);
    if (rc != PH_OK) return rc;
    own_plan = ph_suffix_plan{ws.items, p.items, ws.lane_rec, p.dev_lanes, ws.req_item_cu};
    plan = &own_plan;
    planned = true;
  }
  const float sl2 = scale * kLog2e;
  bool fuse = false;  // prefix and suffix phases in one launch
  PrefixArgs fused_pa{};
  int fused_groups = 0, fused_max_reqs = 0;
  if (has_prefix) {
    int covered = 0, max_group_reqs = 0;
    for (int g = 0; g < num_groups; ++g) {
      const int r0 = group_req_cu_host[g], r1 = group_req_cu_host[g + 1];
      if (r0 < 0 || r1 < r0 || r1 > B) return PH_ERR_ARG;
      covered += r1 - r0;
      if (r1 - r0 > max_group_reqs) max_group_reqs = r1 - r0;
    }
    if (covered != B) {  // requests outside every group: their prefix parts must read as empty
      rc = launch_clear_ml(paired ? ws.ml_pairs : ws.ml, (int64_t)p.n_splits * B * H, st);
      if (rc != PH_OK) return rc;
    }
    PrefixArgs pa{};
    pa.q = (const uint16_t*)q;
    pa.q_stride = q_stride;
    pa.kc = (const uint16_t*)k_cache;
    pa.vc = (const uint16_t*)v_cache;
    pa.row_stride = cache_stride_n;
    pa.slots = prefix_slots;
    pa.prefix_cu = prefix_cu;
    pa.group_req_cu = group_req_cu;
    pa.fixed_prefix_len = -1;
    pa.split_tokens = p.split_tokens;
    pa.n_splits = p.n_splits;
    pa.opart = ws.opart;
    pa.ml = ws.ml;
    pa.B = B;
    pa.H = H;
    pa.scale_log2e = sl2;
    // roles for groups of any size; the shared form only where its eight-wave tile is at least half full
    const int row_mult = paired ? 2 : gshift > 0 ? 1 << gshift : 1;  // rows of the matrix-core kernel per request
    fuse = planned && mfma_prefix && (paired ? decode_fused_supported(dtype, 128) : decode_fused_supported(dtype, D)) &&
           (p.prefix_wgs > 0 || row_mult * max_group_reqs > 32);
    if (fuse) {
      fused_pa = paired ? pair_args(pa, ws) : gshift > 0 ? gqa_args(pa, gshift) : pa;
      fused_groups = (int)num_groups;
      fused_max_reqs = row_mult * max_group_reqs;
    } else {
      rc = run_prefix(pa, dtype, D, (int)num_groups, group_req_cu_host, max_group_reqs, true, st,
                      paired ? &ws : nullptr, ev_prefix, kv.map, gshift);
      if (rc != PH_OK) return rc;
    }
  }
  const int64_t item_base = (int64_t)p.n_splits * B * H;  // first partial row of the balanced form's items
  if (planned) {
    ItemArgs ia{};
    ia.q = (const uint16_t*)q;
    ia.q_stride = q_stride;
    ia.kc = (const uint16_t*)k_cache;
    ia.vc = (const uint16_t*)v_cache;
    ia.row_stride = cache_stride_n;
    ia.slots = suffix_slots;
    ia.offsets = suffix_offsets;
    ia.table_stride = suffix_table_stride;
    ia.items = reinterpret_cast<const int4*>(plan->items);
    ia.lane_rec = reinterpret_cast<const int4*>(plan->lane_rec);
    ia.num_lanes = (int)plan->num_lanes;
    ia.opart = ws.opart + item_base * D;
    ia.ml = ws.ml + item_base * 2;
    ia.H = H;
    ia.scale_log2e = sl2;
    ia.head_map = kv.map;
    ia.nq = hg.stream_group;
    for (int64_t runs = hg.stream_group > 1 ? hg.mfma_group / hg.stream_group : 1; runs > 1; runs >>= 1) ++ia.kv_shift;
    rc = fuse ? launch_decode_fused(fused_pa, ia, dtype, fused_groups, fused_max_reqs, device_cus(), p.prefix_wgs, st,
                                      ev_suffix)
              : launch_items(ia, dtype, D, st, ev_suffix);
    if (rc != PH_OK) return rc;
  } else if (has_suffix) {
    PartialArgs sa{};
    sa.q = (const uint16_t*)q;
    sa.q_stride = q_stride;
    sa.kc = (const uint16_t*)k_cache;
    sa.vc = (const uint16_t*)v_cache;
    sa.row_stride = cache_stride_n;
    sa.slots = suffix_slots;
    sa.slots_total = suffix_slots_count;
    sa.offsets = suffix_offsets;
    sa.table_stride = suffix_table_stride;
    sa.lens = suffix_lens;
    sa.max_len = (int)max_suffix_len;
    sa.shared_cu = nullptr;
    sa.shared_len = -1;
    sa.chunk = p.chunk;
    sa.n_chunks = p.n_chunks;
    sa.part_base = p.n_splits;
    sa.opart = ws.opart;
    sa.ml = ws.ml;
    sa.B = B;
    sa.H = H;
    sa.req_begin = 0;
    sa.num_reqs = B;
    sa.scale_log2e = sl2;
    sa.head_map = kv.map;
    rc = launch_partial(sa, dtype, D, st, ev_suffix);
    if (rc != PH_OK) return rc;
  }
  MergeArgs ma{};
  ma.opart = ws.opart;
  ma.ml = ws.ml;
  ma.out = (uint16_t*)out;
  ma.out_stride = out_stride;
  ma.B = B;
  ma.H = H;
  ma.nA = has_prefix ? p.n_splits : 0;
  ma.gshift = has_prefix && gshift > 0 ? gshift : 0;
  if (has_prefix && paired) {
    ma.opart_pairs = ws.opart_pairs;
    ma.ml_pairs = ws.ml_pairs;
  }
  ma.baseB = p.n_splits;
  ma.lens = has_suffix ? suffix_lens : nullptr;
  ma.max_len = (int)max_suffix_len;
  ma.offsets = suffix_offsets;
  ma.table_stride = suffix_table_stride;
  ma.slots_total = suffix_slots_count;
  ma.chunk = p.chunk;
  ma.req_item_cu = planned ? plan->req_item_cu : nullptr;
  ma.item_base = item_base;
  return launch_merge(ma, dtype, D, st, ev_merge);
}

extern "C" int ph_decode_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                   int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                                   int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                                   int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                                   const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                                   int64_t max_prefix_len, const int32_t* suffix_slots,
                                   const int64_t* suffix_offsets, int64_t suffix_table_stride,
                                   int64_t suffix_slots_count, const int32_t* suffix_lens, int64_t max_suffix_len,
                                   int64_t chunk_tokens, const ph_suffix_plan* plan, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  return decode_attention_impl(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                               cache_stride_n, scale, num_groups, prefix_slots, prefix_cu, group_req_cu,
                               group_req_cu_host, max_prefix_len, suffix_slots, suffix_offsets, suffix_table_stride,
                               suffix_slots_count, suffix_lens, max_suffix_len, chunk_tokens, plan, workspace,
                               workspace_bytes, stream, nullptr);
}

extern "C" int ph_decode_attention_gqa(void* out, const void* q, const void* k_cache, const void* v_cache,
                                       int64_t num_reqs, int64_t num_heads, int64_t num_kv_heads,
                                       const int32_t* head_mapping, int64_t kv_group, int64_t head_dim, int dtype,
                                       int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                                       int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                                       const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                                       int64_t max_prefix_len, const int32_t* suffix_slots,
                                       const int64_t* suffix_offsets, int64_t suffix_table_stride,
                                       int64_t suffix_slots_count, const int32_t* suffix_lens,
                                       int64_t max_suffix_len, int64_t chunk_tokens, const ph_suffix_plan* plan,
                                       void* workspace, size_t workspace_bytes, void* stream) {
  if (!head_mapping) return PH_ERR_ARG;
  KvHeads kv;
  kv.num_kv_heads = num_kv_heads;
  kv.map = head_mapping;
  kv.group = kv_group;
  return decode_attention_impl(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                               cache_stride_n, scale, num_groups, prefix_slots, prefix_cu, group_req_cu,
                               group_req_cu_host, max_prefix_len, suffix_slots, suffix_offsets, suffix_table_stride,
                               suffix_slots_count, suffix_lens, max_suffix_len, chunk_tokens, plan, workspace,
                               workspace_bytes, stream, nullptr, kv);
}

extern "C" size_t ph_decode_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int ph_decode_attention_static(void* out, const void* q, const void* k_cache, const void* v_cache,
                                          int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                                          int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                                          int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                                          const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                                          int64_t max_prefix_len, const int32_t* suffix_slots,
                                          const int64_t* suffix_offsets, int64_t suffix_table_stride,
                                          int64_t suffix_slots_count, const int32_t* suffix_lens,
                                          int64_t max_suffix_len, int64_t chunk_tokens, const ph_suffix_plan* plan,
                                          void* stream) {
  // the same sizing as ph_decode_workspace_bytes; a shape whose partials do not fit the array is refused
  if (num_reqs > 0 && num_heads > 0 && head_dim > 0) {
    const size_t need = ph_decode_workspace_bytes(num_reqs, num_heads, head_dim, num_groups, max_prefix_len,
                                                  max_suffix_len, chunk_tokens, plan ? plan->num_items : 0);
    if (need > kStaticScratchBytes) return PH_ERR_SCRATCH;
  }
  void* ws = nullptr;
  const int rc = static_scratch_ptr(&ws);
  if (rc != PH_OK) return rc;
  return decode_attention_impl(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                               cache_stride_n, scale, num_groups, prefix_slots, prefix_cu, group_req_cu,
                               group_req_cu_host, max_prefix_len, suffix_slots, suffix_offsets, suffix_table_stride,
                               suffix_slots_count, suffix_lens, max_suffix_len, chunk_tokens, plan, ws,
                               kStaticScratchBytes, stream, nullptr);
}

extern "C" int ph_decode_attention_timed(void* out, const void* q, const void* k_cache, const void* v_cache,
                                         int64_t num_reqs, int64_t num_heads, int64_t head_dim, int dtype,
                                         int64_t q_stride, int64_t out_stride, int64_t cache_stride_n, float scale,
                                         int64_t num_groups, const int32_t* prefix_slots, const int32_t* prefix_cu,
                                         const int32_t* group_req_cu, const int32_t* group_req_cu_host,
                                         int64_t max_prefix_len, const int32_t* suffix_slots,
                                         const int64_t* suffix_offsets, int64_t suffix_table_stride,
                                         int64_t suffix_slots_count, const int32_t* suffix_lens,
                                         int64_t max_suffix_len, int64_t chunk_tokens, const ph_suffix_plan* plan,
                                         void* workspace, size_t workspace_bytes, void* stream,
                                         void* const* events6) {
  return decode_attention_impl(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                               cache_stride_n, scale, num_groups, prefix_slots, prefix_cu, group_req_cu,
                               group_req_cu_host, max_prefix_len, suffix_slots, suffix_offsets, suffix_table_stride,
                               suffix_slots_count, suffix_lens, max_suffix_len, chunk_tokens, plan, workspace,
                               workspace_bytes, stream, events6);
}

// Prefix phase over one shared slot list, merged with an optional partial already in out / prev_m / prev_l; the
// merged m / l are exported when asked for.
static int prefix_phase(void* out, const float* prev_m, const float* prev_l, float* m_out, float* l_out, const void* q,
                        const void* k_cache, const void* v_cache, int64_t num_reqs, int64_t num_heads,
                        int64_t head_dim, int dtype, int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                        float scale, const int32_t* prefix_slots, int64_t prefix_len, void* workspace,
                        size_t workspace_bytes, void* stream) {
  const int B = (int)num_reqs, H = (int)num_heads, D = (int)head_dim;
  int rc = check_common(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                        cache_stride_n);
  if (rc != PH_OK || num_reqs == 0) return rc;
  if (prefix_len < 0 || (prefix_len > 0 && !prefix_slots)) return PH_ERR_ARG;
  const bool paired = pair_heads(D, H) && prefix_mfma_supported(dtype, 128);
  const DecodePlan p = plan_decode(num_reqs, num_heads, prefix_len > 0 ? 1 : 0, prefix_len, 0, 0, 0, 0, pair_heads(D, H));
  if (plan_bytes(p, B, H, D) > workspace_bytes || (p.parts() > 0 && !workspace)) return PH_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 255u) != 0) return PH_ERR_ALIGN;
  const Carve ws = carve(workspace, p, B, H, D);
  hipStream_t st = (hipStream_t)stream;
  if (prefix_len > 0) {
    PrefixArgs pa{};
    pa.q = (const uint16_t*)q;
    pa.q_stride = q_stride;
    pa.kc = (const uint16_t*)k_cache;
    pa.vc = (const uint16_t*)v_cache;
    pa.row_stride = cache_stride_n;
    pa.slots = prefix_slots;
    pa.prefix_cu = nullptr;
    pa.group_req_cu = nullptr;
    pa.fixed_prefix_len = (int)prefix_len;
    pa.split_tokens = p.split_tokens;
    pa.n_splits = p.n_splits;
    pa.opart = ws.opart;
    pa.ml = ws.ml;
    pa.B = B;
    pa.H = H;
    pa.scale_log2e = scale * kLog2e;
    rc = run_prefix(pa, dtype, D, 1, nullptr, B, m_out == nullptr, st, paired ? &ws : nullptr);
    if (rc != PH_OK) return rc;
  }
  MergeArgs ma{};
  ma.opart = ws.opart;
  ma.ml = ws.ml;
  if (prefix_len > 0 && paired) {
    ma.opart_pairs = ws.opart_pairs;
    ma.ml_pairs = ws.ml_pairs;
  }
  ma.out = (uint16_t*)out;
  ma.out_stride = out_stride;
  ma.B = B;
  ma.H = H;
  ma.nA = p.n_splits;
  ma.baseB = p.n_splits;
  ma.lens = nullptr;
  ma.chunk = p.chunk;
  ma.prev_m = prev_m;
  ma.prev_l = prev_l;
  ma.m_out = m_out;
  ma.l_out = l_out;
  return launch_merge(ma, dtype, D, st);
}

extern "C" int ph_prefix_attention(void* out, float* m_out, float* l_out, const void* q, const void* k_cache,
                                   const void* v_cache, int64_t num_reqs, int64_t num_heads, int64_t head_dim,
                                   int dtype, int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                                   float scale, const int32_t* prefix_slots, int64_t prefix_len, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  if (num_reqs > 0 && (!m_out || !l_out)) return PH_ERR_ARG;
  return prefix_phase(out, nullptr, nullptr, m_out, l_out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype,
                      q_stride, out_stride, cache_stride_n, scale, prefix_slots, prefix_len, workspace,
                      workspace_bytes, stream);
}

extern "C" int ph_prefix_post_attention(void* out, const float* prev_m, const float* prev_l, const void* q,
                                        const void* k_cache, const void* v_cache, int64_t num_reqs,
                                        int64_t num_heads, int64_t head_dim, int dtype, int64_t q_stride,
                                        int64_t out_stride, int64_t cache_stride_n, float scale,
                                        const int32_t* prefix_slots, int64_t prefix_len, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  if (num_reqs > 0 && (!prev_m || !prev_l)) return PH_ERR_ARG;
  return prefix_phase(out, prev_m, prev_l, nullptr, nullptr, q, k_cache, v_cache, num_reqs, num_heads, head_dim,
                      dtype, q_stride, out_stride, cache_stride_n, scale, prefix_slots, prefix_len, workspace,
                      workspace_bytes, stream);
}

// Suffix phase, merged with an optional partial already in out / prev_m / prev_l; the merged m / l are exported
// when asked for.
static int suffix_phase(void* out, const float* prev_m, const float* prev_l, float* m_out, float* l_out, const void* q,
                        const void* k_cache, const void* v_cache, int64_t num_reqs, int64_t num_heads,
                        int64_t head_dim, int dtype, int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                        float scale, const int32_t* suffix_slots, const int64_t* suffix_offsets,
                        int64_t suffix_table_stride, int64_t suffix_slots_count, const int32_t* suffix_lens,
                        int64_t max_suffix_len, int64_t chunk_tokens, void* workspace, size_t workspace_bytes,
                        void* stream) {
  const int B = (int)num_reqs, H = (int)num_heads, D = (int)head_dim;
  int rc = check_common(out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype, q_stride, out_stride,
                        cache_stride_n);
  if (rc != PH_OK || num_reqs == 0) return rc;
  if (max_suffix_len < 0 || max_suffix_len > INT32_MAX) return PH_ERR_ARG;
  const bool has_suffix = max_suffix_len > 0;
  if (has_suffix && (!suffix_slots || !suffix_lens || suffix_slots_count <= 0)) return PH_ERR_ARG;
  // padded table: every row must hold max_suffix_len entries inside the table (the balanced form walks a row up to
  // its clamped length without knowing where the table ends)
  if (has_suffix && !suffix_offsets &&
      (suffix_table_stride < 0 || suffix_slots_count < (num_reqs - 1) * suffix_table_stride + max_suffix_len))
    return PH_ERR_ARG;
  const DecodePlan p = plan_decode(num_reqs, num_heads, 0, 0, max_suffix_len, chunk_tokens, 0, head_dim);
  if (plan_bytes(p, B, H, D) > workspace_bytes || ((p.parts() > 0 || p.items > 0) && !workspace))
    return PH_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 255u) != 0) return PH_ERR_ALIGN;
  const Carve ws = carve(workspace, p, B, H, D);
  hipStream_t st = (hipStream_t)stream;
  if (has_suffix && p.dev_lanes > 0) {  // balanced form on a plan built on the device
    rc = launch_suffix_plan(suffix_lens, B, (int)max_suffix_len, p.dev_lanes, ws.items, ws.lane_rec, ws.req_item_cu, st);
    if (rc != PH_OK) return rc;
    ItemArgs ia{};
    ia.q = (const uint16_t*)q;
    ia.q_stride = q_stride;
    ia.kc = (const uint16_t*)k_cache;
    ia.vc = (const uint16_t*)v_cache;
    ia.row_stride = cache_stride_n;
    ia.slots = suffix_slots;
    ia.offsets = suffix_offsets;
    ia.table_stride = suffix_table_stride;
    ia.items = reinterpret_cast<const int4*>(ws.items);
    ia.lane_rec = reinterpret_cast<const int4*>(ws.lane_rec);
    ia.num_lanes = p.dev_lanes;
    ia.opart = ws.opart;
    ia.ml = ws.ml;
    ia.H = H;
    ia.scale_log2e = scale * kLog2e;
    rc = launch_items(ia, dtype, D, st);
    if (rc != PH_OK) return rc;
  } else if (has_suffix) {
    PartialArgs sa{};
    sa.q = (const uint16_t*)q;
    sa.q_stride = q_stride;
    sa.kc = (const uint16_t*)k_cache;
    sa.vc = (const uint16_t*)v_cache;
    sa.row_stride = cache_stride_n;
    sa.slots = suffix_slots;
    sa.slots_total = suffix_slots_count;
    sa.offsets = suffix_offsets;
    sa.table_stride = suffix_table_stride;
    sa.lens = suffix_lens;
    sa.max_len = (int)max_suffix_len;
    sa.shared_cu = nullptr;
    sa.shared_len = -1;
    sa.chunk = p.chunk;
    sa.n_chunks = p.n_chunks;
    sa.part_base = 0;
    sa.opart = ws.opart;
    sa.ml = ws.ml;
    sa.B = B;
    sa.H = H;
    sa.req_begin = 0;
    sa.num_reqs = B;
    sa.scale_log2e = scale * kLog2e;
    rc = launch_partial(sa, dtype, D, st);
    if (rc != PH_OK) return rc;
  }
  MergeArgs ma{};
  ma.opart = ws.opart;
  ma.ml = ws.ml;
  ma.out = (uint16_t*)out;
  ma.out_stride = out_stride;
  ma.B = B;
  ma.H = H;
  ma.nA = 0;
  ma.baseB = 0;
  ma.lens = has_suffix ? suffix_lens : nullptr;
  ma.max_len = (int)max_suffix_len;
  ma.offsets = suffix_offsets;
  ma.table_stride = suffix_table_stride;
  ma.slots_total = suffix_slots_count;
  ma.chunk = p.chunk;
  ma.req_item_cu = has_suffix && p.dev_lanes > 0 ? ws.req_item_cu : nullptr;
  ma.item_base = 0;
  ma.prev_m = prev_m;
  ma.prev_l = prev_l;
  ma.m_out = m_out;
  ma.l_out = l_out;
  return launch_merge(ma, dtype, D, st);
}

extern "C" int ph_suffix_post_attention(void* out, const float* prev_m, const float* prev_l, const void* q,
                                        const void* k_cache, const void* v_cache, int64_t num_reqs,
                                        int64_t num_heads, int64_t head_dim, int dtype, int64_t q_stride,
                                        int64_t out_stride, int64_t cache_stride_n, float scale,
                                        const int32_t* suffix_slots, const int64_t* suffix_offsets,
                                        int64_t suffix_table_stride, int64_t suffix_slots_count,
                                        const int32_t* suffix_lens,
                                        int64_t max_suffix_len, int64_t chunk_tokens, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  if (num_reqs > 0 && (!prev_m || !prev_l)) return PH_ERR_ARG;
  return suffix_phase(out, prev_m, prev_l, nullptr, nullptr, q, k_cache, v_cache, num_reqs, num_heads, head_dim,
                      dtype, q_stride, out_stride, cache_stride_n, scale, suffix_slots, suffix_offsets,
                      suffix_table_stride, suffix_slots_count, suffix_lens, max_suffix_len, chunk_tokens, workspace,
                      workspace_bytes, stream);
}

extern "C" int ph_suffix_prev_attention(void* out, float* m_out, float* l_out, const void* q, const void* k_cache,
                                        const void* v_cache, int64_t num_reqs, int64_t num_heads, int64_t head_dim,
                                        int dtype, int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                                        float scale, const int32_t* suffix_slots, const int64_t* suffix_offsets,
                                        int64_t suffix_table_stride, int64_t suffix_slots_count,
                                        const int32_t* suffix_lens, int64_t max_suffix_len, int64_t chunk_tokens,
                                        void* workspace, size_t workspace_bytes, void* stream) {
  if (num_reqs > 0 && (!m_out || !l_out)) return PH_ERR_ARG;
  return suffix_phase(out, nullptr, nullptr, m_out, l_out, q, k_cache, v_cache, num_reqs, num_heads, head_dim, dtype,
                      q_stride, out_stride, cache_stride_n, scale, suffix_slots, suffix_offsets, suffix_table_stride,
                      suffix_slots_count, suffix_lens, max_suffix_len, chunk_tokens, workspace, workspace_bytes,
                      stream);
}

extern "C" size_t ph_prefill_workspace_bytes(int64_t num_tokens, int64_t num_heads, int64_t head_dim, int dtype,
                                             int64_t max_kv_len) {
  if (num_tokens <= 0 || num_heads <= 0 || head_dim <= 0) return 0;
  const DecodePlan p = plan_decode(num_tokens, num_heads, 0, 0, max_kv_len, 0);
  if (prefix_mfma_supported(dtype, (int)head_dim) || (pair_heads(head_dim, num_heads) && prefix_mfma_supported(dtype, 128)))
    return 256 + (size_t)round_up((num_tokens + 2) * 4, 256);
  return (size_t)round_up(num_tokens * 8, 256) + (size_t)round_up(num_tokens * 4, 256) +
         plan_bytes(p, num_tokens, num_heads, head_dim);
}

extern "C" int ph_prefill_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                    int64_t num_tokens, int64_t num_chunks, int64_t num_heads, int64_t head_dim,
                                    int dtype, int64_t q_stride, int64_t out_stride, int64_t cache_stride_n,
                                    float scale, const int32_t* q_cu, const int32_t* kv_cu,
                                    const int32_t* ctx_slots, int64_t ctx_slots_count, int64_t max_kv_len,
                                    void* workspace,
                                    size_t workspace_bytes, void* stream) {
  const int T = (int)num_tokens, H = (int)num_heads, D = (int)head_dim;
  int rc = check_common(out, q, k_cache, v_cache, num_tokens, num_heads, head_dim, dtype, q_stride, out_stride,
                        cache_stride_n);
  if (rc != PH_OK || num_tokens == 0) return rc;
  if (num_chunks <= 0 || max_kv_len <= 0 || max_kv_len > INT32_MAX || !q_cu || !kv_cu || !ctx_slots || ctx_slots_count <= 0) return PH_ERR_ARG;
  if (ph_prefill_workspace_bytes(num_tokens, num_heads, head_dim, dtype, max_kv_len) > workspace_bytes || !workspace)
    return PH_ERR_WORKSPACE;
  if (((uintptr_t)workspace & 255u) != 0) return PH_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const bool paired = pair_heads(D, H) && prefix_mfma_supported(dtype, 128);  // 64-wide heads as halves of head pairs
  if (prefix_mfma_supported(dtype, D) || paired) {
    if (num_chunks > num_tokens) return PH_ERR_ARG;  // every chunk holds at least one query (tile_cu fits the workspace)
    PrefillArgs pa{};
    pa.q = (const uint16_t*)q;
    pa.q_stride = q_stride;
    pa.kc = (const uint16_t*)k_cache;
    pa.vc = (const uint16_t*)v_cache;
    pa.row_stride = cache_stride_n;
    pa.out = (uint16_t*)out;
    pa.out_stride = out_stride;
    pa.q_cu = q_cu;
    pa.kv_cu = kv_cu;
    pa.ctx_slots = ctx_slots;
    pa.tile_cu = (int32_t*)workspace;
    pa.num_chunks = (int)num_chunks;
    pa.H = H;
    pa.scale_log2e = scale * kLog2e;
    pa.pair = paired ? 1 : 0;
    return launch_prefill_mfma(pa, dtype, paired ? 128 : D, num_tokens, st);
  }
  int64_t* offsets = (int64_t*)workspace;
  int32_t* lens = (int32_t*)((char*)workspace + round_up(num_tokens * 8, 256));
  void* dws = (char*)lens + round_up(num_tokens * 4, 256);
  hipLaunchKernelGGL(prefill_rows_kernel, dim3((T + 255) / 256), dim3(256), 0, st, q_cu, kv_cu, (int)num_chunks, T,
                     offsets, lens);
  if ((rc = launch_status()) != PH_OK) return rc;
  const DecodePlan p = plan_decode(num_tokens, num_heads, 0, 0, max_kv_len, 0);
  const Carve ws = carve(dws, p, T, H, D);
  PartialArgs sa{};
  sa.q = (const uint16_t*)q;
  sa.q_stride = q_stride;
  sa.kc = (const uint16_t*)k_cache;
  sa.vc = (const uint16_t*)v_cache;
  sa.row_stride = cache_stride_n;
  sa.slots = ctx_slots;
  sa.slots_total = ctx_slots_count;
  sa.offsets = offsets;
  sa.lens = lens;
  sa.max_len = (int)max_kv_len;
  sa.shared_len = -1;
  sa.chunk = p.chunk;
  sa.n_chunks = p.n_chunks;
  sa.part_base = 0;
  sa.opart = ws.opart;
  sa.ml = ws.ml;
  sa.B = T;
  sa.H = H;
  sa.req_begin = 0;
  sa.num_reqs = T;
  sa.scale_log2e = scale * kLog2e;
  if ((rc = launch_partial(sa, dtype, D, st)) != PH_OK) return rc;
  MergeArgs ma{};
  ma.opart = ws.opart;
  ma.ml = ws.ml;
  ma.out = (uint16_t*)out;
  ma.out_stride = out_stride;
  ma.B = T;
  ma.H = H;
  ma.nA = 0;
  ma.baseB = 0;
  ma.lens = lens;
  ma.max_len = (int)max_kv_len;
  ma.offsets = offsets;
  ma.slots_total = ctx_slots_count;
  ma.chunk = p.chunk;
  return launch_merge(ma, dtype, D, st);
}
