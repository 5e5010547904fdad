// Device side of the incremental slot tables: a decode iteration appends exactly one slot to the
// suffix list of every request of the batch, so the padded [B, width] table and the length vector
// that the reference rebuilds from Python lists every iteration
// (parrot/engine/builtin/attn_func.py:523-531,553-569) are patched in place instead.
#include "decode.hpp"

namespace ph {

__global__ __launch_bounds__(256) void append_slots_kernel(int32_t* __restrict__ table, int64_t stride,
                                                           int32_t* __restrict__ lens,
                                                           const int32_t* __restrict__ rows,
                                                           const int32_t* __restrict__ new_slots, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int r = rows ? rows[i] : i;
  const int l = lens[r];
  if (l < stride) {  // the host grows the table before a row fills up; never write past a row
    table[(int64_t)r * stride + l] = new_slots[i];
    lens[r] = l + 1;
  }
}

// ---------------------------------------------------------------------------------------------------------
// Balanced suffix plan on the device.  The token stream of all requests back to back (request b owns tokens
// [cu[b], cu[b+1]) of it) is cut at `lanes` near-equal marks cut(l) = floor(l * total / lanes); an item is a
// maximal run of one request's tokens between neighbouring marks or request boundaries.  One workgroup; the
// prefix sums live in LDS, every item and every lane record is then written independently:
//   - the first item of request b starts at cu[b];
//   - mark l that falls strictly inside a request starts another item of that request;
//   - lane l's record names the item that starts at cut(l) and counts the items up to cut(l + 1).
// lanes = min(lanes_cap, ceil(total / kMinPiece), total): no piece under kMinPiece tokens; records beyond `lanes`
// are empty.
constexpr int kPlanThreads = 1024;
// Smallest piece: one round of the streaming body's register pipeline.  A short total is a latency problem, not a
// bandwidth problem: spread over many lanes every wave walks the slot-id -> rows -> partial chain once, instead of
// a few waves walking it several times in a row while the rest of the launch waits for them.
constexpr int kMinPiece = 4;

struct PlanScratch {
  int cu[kPlanMaxReqs + 1];      // token prefix sums
  int icu[kPlanMaxReqs + 1];     // item prefix sums
  int part[kPlanThreads];
};

// exclusive prefix sums of v(0..n-1) into out[0..n] by the whole workgroup: each thread owns a run, the thread
// sums are scanned inside each wave with lane shuffles and across the sixteen waves by the first wave
template <typename F>
__device__ __forceinline__ void block_scan(F v, int n, int* out, int* part) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int per = (n + kPlanThreads - 1) / kPlanThreads;
  const int b0 = min(t * per, n), b1 = min(b0 + per, n);
  int s = 0;
  for (int i = b0; i < b1; ++i) s += v(i);
  int inc = s;  // inclusive scan over the wave
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(inc, d, kWave);
    if (lane >= d) inc += up;
  }
  if (lane == kWave - 1) part[w] = inc;
  __syncthreads();
  if (w == 0) {
    constexpr int NW = kPlanThreads / kWave;
    int ws = lane < NW ? part[lane] : 0;
#pragma unroll
    for (int d = 1; d < NW; d <<= 1) {
      const int up = __shfl_up(ws, d, kWave);
      if (lane >= d) ws += up;
    }
    if (lane < NW) part[lane] = ws;  // inclusive over the waves
  }
  __syncthreads();
  int run = inc - s + (w > 0 ? part[w - 1] : 0);
  for (int i = b0; i < b1; ++i) {
    out[i] = run;
    run += v(i);
  }
  if (t == kPlanThreads - 1) out[n] = run;
  __syncthreads();
}

__global__ __launch_bounds__(kPlanThreads) void suffix_plan_kernel(const int32_t* __restrict__ lens, int B, int max_len,
                                                                   int lanes_cap,
                                                                   int4* __restrict__ items,
                                                                   int4* __restrict__ lane_rec,
                                                                   int32_t* __restrict__ req_item_cu) {
  __shared__ PlanScratch sh;
  const int t = threadIdx.x;
  // a length beyond the host's bound would walk into the next request's row of the slot table
  block_scan([&](int i) { return min(max(lens[i], 0), max_len); }, B, sh.cu, sh.part);
  const int64_t total = sh.cu[B];
  const int lanes = (int)max((int64_t)1, min((int64_t)lanes_cap, min((total + kMinPiece - 1) / kMinPiece, total)));
  auto cut = [&](int l) { return (int)((int64_t)l * total / lanes); };
  // first mark strictly inside request b (cut(l) > cu[b]), and one past the last (cut(l) < cu[b+1])
  auto mark_lo = [&](int b) { return (int)((((int64_t)sh.cu[b] + 1) * lanes + total - 1) / total); };
  auto mark_hi = [&](int b) { return (int)(((int64_t)sh.cu[b + 1] * lanes + total - 1) / total); };
  auto n_items = [&](int b) {
    if (sh.cu[b + 1] == sh.cu[b] || total == 0) return 0;
    return 1 + max(0, mark_hi(b) - mark_lo(b));
  };
  block_scan(n_items, B, sh.icu, sh.part);
  const int total_items = sh.icu[B];
  for (int b = t; b <= B; b += kPlanThreads) req_item_cu[b] = sh.icu[b];
  // request owning global token g (the last b with cu[b] <= g; it has cu[b+1] > g)
  auto owner = [&](int g) {
    int lo = 0, hi = B;  // cu[lo] <= g < cu[hi]
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (sh.cu[mid] <= g) lo = mid; else hi = mid;
    }
    return lo;
  };
  // index of the item that starts at mark l (0 <= l < lanes)
  auto item_at_mark = [&](int l, int& b_out) {
    const int g = cut(l);
    const int b = owner(g);
    b_out = b;
    return g == sh.cu[b] ? sh.icu[b] : sh.icu[b] + (l - mark_lo(b) + 1);
  };
  if (total > 0) {
    for (int b = t; b < B; b += kPlanThreads) {
      if (sh.cu[b + 1] == sh.cu[b]) continue;
      const int lo = mark_lo(b);
      const int end = lo < mark_hi(b) ? cut(lo) : sh.cu[b + 1];
      items[sh.icu[b]] = int4{b, 0, end - sh.cu[b], 0};
    }
    for (int l = 1 + t; l < lanes; l += kPlanThreads) {
      const int g = cut(l);
      const int b = owner(g);
      if (g == sh.cu[b]) continue;  // the mark is a request boundary: that request's first item
      const int end = min(sh.cu[b + 1], cut(l + 1));
      items[sh.icu[b] + (l - mark_lo(b) + 1)] = int4{b, g - sh.cu[b], end - g, 0};
    }
  }
  for (int l = t; l < lanes_cap; l += kPlanThreads) {
    int4 r0 = {total_items, 0, 0, 0}, r1 = {0, 0, 0, 0};
    if (total > 0 && l < lanes) {
      int b, bn;
      const int first = item_at_mark(l, b);
      const int next = l + 1 < lanes ? item_at_mark(l + 1, bn) : total_items;
      const int g = cut(l);
      const int end = min(sh.cu[b + 1], cut(l + 1));
      r0 = int4{first, next - first, b, g - sh.cu[b]};
      r1 = int4{end - g, 0, 0, 0};
    }
    lane_rec[2 * l] = r0;
    lane_rec[2 * l + 1] = r1;
  }
}

int launch_suffix_plan(const int32_t* lens, int B, int max_len, int lanes, int32_t* items, int32_t* lane_rec,
                       int32_t* req_item_cu, hipStream_t st) {
  hipLaunchKernelGGL(suffix_plan_kernel, dim3(1), dim3(kPlanThreads), 0, st, lens, B, max_len, lanes,
                     reinterpret_cast<int4*>(items), reinterpret_cast<int4*>(lane_rec), req_item_cu);
  return launch_status();
}

}  // namespace ph

extern "C" int ph_suffix_plan_build(const int32_t* suffix_lens, int64_t num_reqs, int64_t max_suffix_len,
                                    int64_t num_lanes, int32_t* items, int32_t* lane_rec, int32_t* req_item_cu,
                                    void* stream) {
  if (num_reqs < 0 || num_lanes <= 0 || num_reqs > ph::kPlanMaxReqs || num_lanes > (1 << 20)) return PH_ERR_ARG;
  if (max_suffix_len < 0 || max_suffix_len > INT32_MAX) return PH_ERR_ARG;
  if (num_reqs == 0) return PH_OK;
  if (!suffix_lens || !items || !lane_rec || !req_item_cu) return PH_ERR_ARG;
  return ph::launch_suffix_plan(suffix_lens, (int)num_reqs, (int)max_suffix_len, (int)num_lanes, items, lane_rec,
                                req_item_cu, (hipStream_t)stream);
}

extern "C" int ph_suffix_tables_append(int32_t* table, int64_t table_stride, int32_t* lens, const int32_t* rows,
                                       const int32_t* new_slots, int64_t n, void* stream) {
  if (n < 0 || table_stride <= 0) return PH_ERR_ARG;
  if (n == 0) return PH_OK;
  if (!table || !lens || !new_slots) return PH_ERR_ARG;
  hipLaunchKernelGGL(ph::append_slots_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     table, table_stride, lens, rows, new_slots, (int)n);
  return ph::launch_status();
}
