// Decode attention over token-granular slot tables: per-request partial
// attention (suffix phase and the non-shared ragged decode), and the n-way
// log-sum-exp merge.  HBM-bound (1 FLOP per KV byte): no MFMA, no LDS.
//
// Mapping: in the [slot, H, D] pool all heads of a token are one contiguous
// row.  A wave owns HPW = 64 / LPH adjacent heads of one (request, chunk), LPH = D/8 lanes per head
// (rounded up to a power of two for D = 80, 96, 112, whose spare lanes idle):
// each lane loads 8 contiguous elements (one 128-bit load), so a wave reads a
// contiguous HPW*D*2-byte span of every token row.  The D/8 lanes of a head
// combine their partial dot products with a butterfly; softmax runs online in
// the exp2 domain; slot ids are fetched 64 at a time into one VGPR and
// broadcast through v_readlane.
//
// Math restated from csrc/attention/attention_post_kernels.cu:74-341 (suffix
// phase + merge), attention_prev_kernels.cu:147,223,332-337 (m / l export) and
// parrot/engine/builtin/kernels/shared_flash_decoding.py:137-199 (n-way reduce).
#include "stream_item.hpp"

namespace ph {

// Grid form: one wave per (request, fixed-size chunk, HPW heads); lengths are read on the device, waves
// of chunks past a request's end exit at once.  Used when the caller has no host copy of the lengths.
template <typename E, int D, int TB, int STAGES>
__global__ __launch_bounds__(256) void decode_partial_kernel(PartialArgs a) {
  constexpr int LPH = HeadLanes<D>::LPH;  // lanes per head
  constexpr int HPW = HeadLanes<D>::HPW;  // heads per wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int hgroups = (a.H + HPW - 1) / HPW;
  const int item = wave / hgroups;
  const int hg = wave - item * hgroups;
  const int rb = item / a.n_chunks;  // request index inside this launch
  const int c = item - rb * a.n_chunks;
  if (rb >= a.num_reqs) return;
  const int b = a.req_begin + rb;

  // The first block's slot ids are fetched before the length is known (clamped to the table's
  // end), so the chain of dependent loads in front of the K/V stream is two deep, not three.
  const int t0 = c * a.chunk;
  int64_t off, last;  // last = highest readable index behind this list's start
  int len;
  if (a.shared_cu) {
    off = a.shared_cu[0];
    len = a.shared_cu[1] - a.shared_cu[0];
    last = len - 1;
  } else if (a.shared_len >= 0) {
    off = 0;
    len = a.shared_len;
    last = len - 1;
  } else {
    off = a.offsets ? a.offsets[b] : (int64_t)b * a.table_stride;
    len = -1;
    last = a.slots_total - 1 - off;
  }
  if (last < 0) return;  // an empty shared list, or an offset at the very end of the table
  const int32_t* slots = a.slots + off;
  const int myslot = slots[min((int64_t)(t0 + lane), last)];
  // a length beyond the host's bound (or the table's end) would walk into other requests' slots
  if (len < 0) len = clamped_list_len(a.lens, b, a.max_len, off, a.slots_total);

  const int head = hg * HPW + lane / LPH;
  const bool head_ok = head < a.H;
  const int hclamp = head_ok ? head : a.H - 1;
  const uint32_t lane_off = (uint32_t)(hclamp * D + HeadLanes<D>::chunk(lane) * 8);  // elements inside a query row
  const uint32_t kv_off = kv_lane_off<D>(a.head_map, hclamp, lane);                  // ... inside a K/V token row
  if (t0 >= len) return;
  const int t1 = min(len, t0 + a.chunk);
  const int64_t pr = ((int64_t)(a.part_base + c) * a.B + b) * a.H + hclamp;
  stream_request<E, D, TB, STAGES>(a.q, (int64_t)b * a.q_stride, a.kc, a.vc, a.row_stride, slots, myslot, t0, t1,
                                   lane_off, kv_off, a.scale_log2e, head_ok, a.opart, a.ml, pr);
}

// Balanced form: the host cut the batch's token stream into `num_lanes` near-equal pieces; a piece is
// one or more items (request, first token, count) and is streamed by hgroups waves (one per HPW heads),
// so every wave of the launch moves the same number of bytes and the launch is a single round.
// NQ > 1 (a.nq): the NQ query heads of a KV head go through one wave's lanes together (stream_item)
template <typename E, int D, int TB, int STAGES, int NQ = 1>
__global__ __launch_bounds__(256) void decode_items_kernel(ItemArgs a) {
  constexpr int HPW = HeadLanes<D>::HPW;
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int hgroups = (a.H / NQ + HPW - 1) / HPW;
  const int piece = wave / hgroups;
  if (piece >= a.num_lanes) return;
  run_piece<E, D, TB, STAGES, NQ>(a, piece, wave - piece * hgroups);
}

// One workgroup per (request, HPW heads); its four waves fold every fourth part each
// (loads are unconditional and independent, so several parts are in flight per wave),
// then wave 0 folds the four running results through LDS and writes the output row.
template <typename E, int D>
__global__ __launch_bounds__(256) void merge_kernel(MergeArgs a) {
  constexpr int LPH = HeadLanes<D>::LPH;
  constexpr int HPW = HeadLanes<D>::HPW;
  __shared__ float sh[3][10][kWave];
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  const int hgroups = (a.H + HPW - 1) / HPW;
  const int b = blockIdx.x / hgroups;
  const int hg = blockIdx.x - b * hgroups;
  const int head_raw = hg * HPW + lane / LPH;
  const bool head_ok = head_raw < a.H;
  const int head = head_ok ? head_raw : a.H - 1;
  const int dl = HeadLanes<D>::chunk(lane) * 8;

  float M = -INFINITY, L = 0.f;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;

  if (a.prev_m && w == 0) {  // a partial already sitting in out / prev_m / prev_l
    const float lp = a.prev_l[(int64_t)b * a.H + head];
    if (lp > 0.f) {
      float ov[8];
      load8f<E>(a.out, (int64_t)b * a.out_stride + (int64_t)head * D + dl, ov);
      M = a.prev_m[(int64_t)b * a.H + head];
      L = lp;
#pragma unroll
      for (int k = 0; k < 8; ++k) acc[k] = lp * ov[k];
    }
  }

  // candidates: prefix parts [0, nA) laid out [part][B][H]; then either the request's suffix chunks
  // (same layout, parts baseB ..) or its items of the balanced form ([item][H], rows item_base ..)
  int nB, it0 = 0;
  if (a.req_item_cu) {
    it0 = a.req_item_cu[b];
    nB = a.req_item_cu[b + 1] - it0;
  } else {
    int len = 0;
    if (a.lens && a.slots_total > 0)
      len = clamped_list_len(a.lens, b, a.max_len, a.offsets ? a.offsets[b] : (int64_t)b * a.table_stride, a.slots_total);
    else if (a.lens)
      len = min(max(a.lens[b], 0), a.max_len);
    nB = (len + a.chunk - 1) / a.chunk;
  }
  const int total = a.nA + nB;
#pragma unroll 2
  for (int i = w; i < total; i += 4) {
    int64_t pr;
    const float* mlrow;
    const float* op;
    if (i < a.nA && a.opart_pairs) {  // D == 64: this head is one half of a 128-wide row
      pr = ((int64_t)i * (2 * a.B) + 2 * b + (head & 1)) * (a.H >> 1) + (head >> 1);
      mlrow = a.ml_pairs + pr * 2;
      op = a.opart_pairs + pr * (2 * D) + (head & 1) * D + dl;
    } else {
      if (i < a.nA && a.gshift > 0)  // grouped KV heads: the part of row b G + (head mod G), KV head head / G
        pr = ((int64_t)i * ((int64_t)a.B << a.gshift) + ((int64_t)b << a.gshift) + (head & ((1 << a.gshift) - 1))) *
                 (a.H >> a.gshift) + (head >> a.gshift);
      else if (i < a.nA)
        pr = ((int64_t)i * a.B + b) * a.H + head;
      else if (a.req_item_cu)
        pr = a.item_base + (int64_t)(it0 + i - a.nA) * a.H + head;
      else
        pr = ((int64_t)(a.baseB + i - a.nA) * a.B + b) * a.H + head;
      mlrow = a.ml + pr * 2;
      op = a.opart + pr * D + dl;
    }
    const float2 mlp = *reinterpret_cast<const float2*>(mlrow);
    const float4_t o0 = *reinterpret_cast<const float4_t*>(op);
    const float4_t o1 = *reinterpret_cast<const float4_t*>(op + 4);
    const bool live = mlp.y > 0.f;  // l == 0 marks an empty part (its O may be garbage)
    const float mp = live ? mlp.x : -INFINITY;
    const float Mn = fmaxf(M, mp);
    const float sc = (M == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(M - Mn);
    const float wgt = live ? __builtin_amdgcn_exp2f(mp - Mn) * mlp.y : 0.f;
    L = L * sc + wgt;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      acc[k] = acc[k] * sc + (live ? wgt * o0[k] : 0.f);
      acc[4 + k] = acc[4 + k] * sc + (live ? wgt * o1[k] : 0.f);
    }
    M = Mn;
  }

  if (w > 0) {
    sh[w - 1][0][lane] = M;
    sh[w - 1][1][lane] = L;
#pragma unroll
    for (int k = 0; k < 8; ++k) sh[w - 1][2 + k][lane] = acc[k];
  }
  __syncthreads();
  if (w != 0) return;
#pragma unroll
  for (int o = 0; o < 3; ++o) {
    const float mo = sh[o][0][lane], lo = sh[o][1][lane];
    const float Mn = fmaxf(M, mo);
    const float sa = (M == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(M - Mn);
    const float sb = (mo == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mo - Mn);
    L = L * sa + lo * sb;
#pragma unroll
    for (int k = 0; k < 8; ++k) acc[k] = acc[k] * sa + sh[o][2 + k][lane] * sb;
    M = Mn;
  }
  if (!head_ok || !HeadLanes<D>::active(lane)) return;
  const float inv = L > 0.f ? 1.f / L : 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) acc[k] *= inv;
  store8f<E>(a.out, (int64_t)b * a.out_stride + (int64_t)head * D + dl, acc);
  if (a.m_out && lane % LPH == 0) {
    a.m_out[(int64_t)b * a.H + head] = M;
    a.l_out[(int64_t)b * a.H + head] = L;
  }
}

// Marks parts [part0, part0+nparts) empty (l = 0) for every (request, head).
__global__ __launch_bounds__(256) void clear_ml_kernel(float* ml, int64_t n2) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n2) ml[i] = (i & 1) ? 0.f : -INFINITY;
}

template <typename E, int D>
static int launch_partial_t(const PartialArgs& a, hipStream_t st, const KernelEvents& ev) {
  constexpr int HPW = HeadLanes<D>::HPW;
  const int64_t hgroups = (a.H + HPW - 1) / HPW;
  const int64_t waves = (int64_t)a.num_reqs * a.n_chunks * hgroups;
  if (waves == 0) return PH_OK;
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  PH_LAUNCH_TIMED((decode_partial_kernel<E, D, 4, 2>), grid, block, 0, st, ev, a);
  return launch_status();
}

template <typename E, int D>
static int launch_items_t(const ItemArgs& a, hipStream_t st, const KernelEvents& ev) {
  constexpr int HPW = HeadLanes<D>::HPW;
  const int nq = a.nq > 1 ? a.nq : 1;
  const int64_t hgroups = (a.H / nq + HPW - 1) / HPW;
  const int64_t waves = (int64_t)a.num_lanes * hgroups;
  if (waves == 0) return PH_OK;
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  if constexpr (D == 128 && !is_f32<E>::value) {
    if (nq == 4) {
      PH_LAUNCH_TIMED((decode_items_kernel<E, D, 4, 2, 4>), grid, block, 0, st, ev, a);
      return launch_status();
    }
  }
  if (nq != 1) return PH_ERR_ARG;  // grouped_stream_heads() says which shapes have the grouped form
  PH_LAUNCH_TIMED((decode_items_kernel<E, D, 4, 2>), grid, block, 0, st, ev, a);
  return launch_status();
}

template <typename E, int D>
static int launch_merge_t(const MergeArgs& a, hipStream_t st, const KernelEvents& ev) {
  constexpr int HPW = HeadLanes<D>::HPW;
  const int64_t hgroups = (a.H + HPW - 1) / HPW;
  const int64_t groups = (int64_t)a.B * hgroups;
  if (groups == 0) return PH_OK;
  dim3 grid((unsigned)groups), block(256);
  PH_LAUNCH_TIMED((merge_kernel<E, D>), grid, block, 0, st, ev, a);
  return launch_status();
}

#define PH_DISPATCH(FN, dtype, D, ...)                                  \
  do {                                                                  \
    if ((dtype) == PH_F16) {                                            \
      if ((D) == 128) return FN<F16, 128>(__VA_ARGS__);                 \
      if ((D) == 64) return FN<F16, 64>(__VA_ARGS__);                   \
      if ((D) == 256) return FN<F16, 256>(__VA_ARGS__);                 \
      if ((D) == 80) return FN<F16, 80>(__VA_ARGS__);                   \
      if ((D) == 96) return FN<F16, 96>(__VA_ARGS__);                   \
      if ((D) == 112) return FN<F16, 112>(__VA_ARGS__);                 \
    } else if ((dtype) == PH_F32) {                                     \
      if ((D) == 128) return FN<F32, 128>(__VA_ARGS__);                 \
      if ((D) == 64) return FN<F32, 64>(__VA_ARGS__);                   \
      if ((D) == 256) return FN<F32, 256>(__VA_ARGS__);                 \
      if ((D) == 80) return FN<F32, 80>(__VA_ARGS__);                   \
      if ((D) == 96) return FN<F32, 96>(__VA_ARGS__);                   \
      if ((D) == 112) return FN<F32, 112>(__VA_ARGS__);                 \
    } else {                                                            \
      if ((D) == 128) return FN<BF16, 128>(__VA_ARGS__);                \
      if ((D) == 64) return FN<BF16, 64>(__VA_ARGS__);                  \
      if ((D) == 256) return FN<BF16, 256>(__VA_ARGS__);                \
      if ((D) == 80) return FN<BF16, 80>(__VA_ARGS__);                  \
      if ((D) == 96) return FN<BF16, 96>(__VA_ARGS__);                  \
      if ((D) == 112) return FN<BF16, 112>(__VA_ARGS__);                \
    }                                                                   \
    return PH_ERR_HEAD_DIM;                                             \
  } while (0)

int launch_partial(const PartialArgs& a, int dtype, int D, hipStream_t st, const KernelEvents& ev) {
  PH_DISPATCH(launch_partial_t, dtype, D, a, st, ev);
}
int launch_items(const ItemArgs& a, int dtype, int D, hipStream_t st, const KernelEvents& ev) {
  PH_DISPATCH(launch_items_t, dtype, D, a, st, ev);
}
int launch_merge(const MergeArgs& a, int dtype, int D, hipStream_t st, const KernelEvents& ev) {
  PH_DISPATCH(launch_merge_t, dtype, D, a, st, ev);
}
int launch_clear_ml(float* ml, int64_t entries, hipStream_t st) {
  if (entries == 0) return PH_OK;
  const int64_t n2 = entries * 2;
  hipLaunchKernelGGL(clear_ml_kernel, dim3((unsigned)((n2 + 255) / 256)), dim3(256), 0, st, ml, n2);
  return launch_status();
}

}  // namespace ph
