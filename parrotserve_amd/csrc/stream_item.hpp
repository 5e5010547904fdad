// The streaming body of the per-request decode kernels (suffix phase, ragged decode): one wave, HPW adjacent
// heads, token rows gathered by slot with 128-bit non-temporal loads, online softmax in the exp2 domain.
// Shared by the stand-alone kernels (decode.hip) and the fused prefix + suffix kernel (prefix_mfma.hip).
//
// Math restated from csrc/attention/attention_post_kernels.cu:74-341 and
// attention_prev_kernels.cu:147,223,332-337 (m / l export).
#pragma once

#include "decode.hpp"

namespace ph {

// Streams the token rows slots[t0 .. t1) of one request through one wave (HPW adjacent heads) and
// writes the (O, m, l) part at row `pr` of the partial buffers.  `myslot` holds the slot ids of the
// first 64 tokens (lane i: token t0 + i, clamped), already fetched by the caller.  `lane_off` = this lane's
// element offset inside a token row of the K/V pools (its KV head's row, see kv_lane_off).
// NQ > 1 (grouped KV heads): a wave's head slot holds a run of NQ adjacent query heads that share a KV head, and every
// token row meets the NQ queries at once -- one load of the row, NQ scores, NQ parts at rows pr .. pr + NQ - 1 --
// instead of being loaded once per query head.
template <typename E, int D, int TB, int STAGES, int NQ = 1>
__device__ __forceinline__ void stream_item(const uint16_t* __restrict__ kc, const uint16_t* __restrict__ vc,
                                            int64_t row_stride, const int32_t* __restrict__ slots, int myslot,
                                            int t0, int t1, const u32x4 (&qv)[NQ], uint32_t lane_off,
                                            float scale_log2e, bool head_ok, float* __restrict__ opart,
                                            float* __restrict__ ml, int64_t pr) {
  constexpr int LPH = HeadLanes<D>::LPH;
  const int lane = threadIdx.x & 63;
  float m[NQ], l[NQ];
  float o[NQ][8];
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    m[n] = -INFINITY;
    l[n] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) o[n][i] = 0.f;
  }

  u32x4 kb[STAGES][TB], vb[STAGES][TB];

  for (int tb = t0; tb < t1; tb += kWave) {
    if (tb > t0) myslot = slots[min(tb + lane, t1 - 1)];
    const int nb = min(kWave, t1 - tb);

    // TB token rows (K and V) in flight per stage; row bases are wave-uniform (SGPR)
    auto load = [&](u32x4(&kk)[TB], u32x4(&vv)[TB], int j0) {
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const int64_t slot = __builtin_amdgcn_readlane(myslot, min(j0 + j, nb - 1));
        const uint16_t* kr = kc + slot * row_stride;
        const uint16_t* vr = vc + slot * row_stride;
        kk[j] = ld16_nt(kr + lane_off);
        vv[j] = ld16_nt(vr + lane_off);
      }
    };
    auto compute = [&](const u32x4(&kk)[TB], const u32x4(&vv)[TB], int j0) {
#pragma unroll
      for (int n = 0; n < NQ; ++n) {
        float s[TB];
        float mb = -INFINITY;
#pragma unroll
        for (int j = 0; j < TB; ++j) {
          float d = 0.f;
#pragma unroll
          for (int w = 0; w < 4; ++w) d = Elem<E>::dot2(qv[n][w], kk[j][w], d);
          d = group_sum<LPH>(d) * scale_log2e;
          s[j] = (j0 + j < nb) ? d : -INFINITY;
          mb = fmaxf(mb, s[j]);
        }
        const float mn = fmaxf(m[n], mb);
        const float alpha = __builtin_amdgcn_exp2f(m[n] - mn);
        l[n] *= alpha;
#pragma unroll
        for (int i = 0; i < 8; ++i) o[n][i] *= alpha;
#pragma unroll
        for (int j = 0; j < TB; ++j) {
          const float p = __builtin_amdgcn_exp2f(s[j] - mn);
          l[n] += p;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            o[n][2 * w] = __builtin_fmaf(p, Elem<E>::lo(vv[j][w]), o[n][2 * w]);
            o[n][2 * w + 1] = __builtin_fmaf(p, Elem<E>::hi(vv[j][w]), o[n][2 * w + 1]);
          }
        }
        m[n] = mn;
      }
    };

    if (STAGES == 2) {
      // two-stage software pipeline: the next batch's rows are in flight while this one is reduced
      load(kb[0], vb[0], 0);
      for (int j0 = 0; j0 < nb; j0 += 2 * TB) {
        const bool more1 = j0 + TB < nb;
        if (more1) load(kb[STAGES - 1], vb[STAGES - 1], j0 + TB);
        compute(kb[0], vb[0], j0);
        if (j0 + 2 * TB < nb) load(kb[0], vb[0], j0 + 2 * TB);
        if (more1) compute(kb[STAGES - 1], vb[STAGES - 1], j0 + TB);
      }
    } else {
      for (int j0 = 0; j0 < nb; j0 += TB) {
        load(kb[0], vb[0], j0);
        compute(kb[0], vb[0], j0);
      }
    }
  }

  if (!head_ok || !HeadLanes<D>::active(lane)) return;
#pragma unroll
  for (int n = 0; n < NQ; ++n) {
    const float inv = 1.f / l[n];
    float* op = opart + (pr + n) * D + (lane % LPH) * 8;
    float4_t o0 = {o[n][0] * inv, o[n][1] * inv, o[n][2] * inv, o[n][3] * inv};
    float4_t o1 = {o[n][4] * inv, o[n][5] * inv, o[n][6] * inv, o[n][7] * inv};
    *reinterpret_cast<float4_t*>(op) = o0;
    *reinterpret_cast<float4_t*>(op + 4) = o1;
    if (lane % LPH == 0) {
      ml[(pr + n) * 2] = m[n];
      ml[(pr + n) * 2 + 1] = l[n];
    }
  }
}

// The same for 32-bit elements: a lane's eight elements of a token row are two 128-bit loads (the lanes of a head
// still cover the head's row contiguously), the dot product and P.V are plain fp32 FMAs.  One stage of TB token
// rows in flight; this element type is served for completeness of the reference's configuration (float32), the
// tuned path is the 16-bit one above.
template <int D, int TB>
__device__ __forceinline__ void stream_item_f32(const float* __restrict__ kc, const float* __restrict__ vc,
                                                int64_t row_stride, const int32_t* __restrict__ slots, int myslot,
                                                int t0, int t1, const float (&q)[8], uint32_t lane_off,
                                                float scale_log2e, bool head_ok, float* __restrict__ opart,
                                                float* __restrict__ ml, int64_t pr) {
  constexpr int LPH = HeadLanes<D>::LPH;
  const int lane = threadIdx.x & 63;
  float m = -INFINITY, l = 0.f;
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = 0.f;
  for (int tb = t0; tb < t1; tb += kWave) {
    if (tb > t0) myslot = slots[min(tb + lane, t1 - 1)];
    const int nb = min(kWave, t1 - tb);
    for (int j0 = 0; j0 < nb; j0 += TB) {
      float4_t k0[TB], k1[TB], v0[TB], v1[TB];
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const int64_t slot = __builtin_amdgcn_readlane(myslot, min(j0 + j, nb - 1));
        const float* kr = kc + slot * row_stride + lane_off;
        const float* vr = vc + slot * row_stride + lane_off;
        k0[j] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(kr));
        k1[j] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(kr + 4));
        v0[j] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(vr));
        v1[j] = __builtin_nontemporal_load(reinterpret_cast<const float4_t*>(vr + 4));
      }
      float s[TB];
      float mb = -INFINITY;
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          d = __builtin_fmaf(q[i], k0[j][i], d);
          d = __builtin_fmaf(q[4 + i], k1[j][i], d);
        }
        d = group_sum<LPH>(d) * scale_log2e;
        s[j] = (j0 + j < nb) ? d : -INFINITY;
        mb = fmaxf(mb, s[j]);
      }
      const float mn = fmaxf(m, mb);
      const float alpha = __builtin_amdgcn_exp2f(m - mn);
      l *= alpha;
#pragma unroll
      for (int i = 0; i < 8; ++i) o[i] *= alpha;
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const float p = __builtin_amdgcn_exp2f(s[j] - mn);
        l += p;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          o[i] = __builtin_fmaf(p, v0[j][i], o[i]);
          o[4 + i] = __builtin_fmaf(p, v1[j][i], o[4 + i]);
        }
      }
      m = mn;
    }
  }
  if (!head_ok || !HeadLanes<D>::active(lane)) return;
  const float inv = 1.f / l;
  float* op = opart + pr * D + (lane % LPH) * 8;
  *reinterpret_cast<float4_t*>(op) = float4_t{o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
  *reinterpret_cast<float4_t*>(op + 4) = float4_t{o[4] * inv, o[5] * inv, o[6] * inv, o[7] * inv};
  if (lane % LPH == 0) {
    ml[pr * 2] = m;
    ml[pr * 2 + 1] = l;
  }
}

// Element offset of this lane's 8 elements inside a token row of the K/V pools: the row of the lane's KV head --
// the query head itself, or head_map[query head] when query heads share KV heads (grouped / multi-query
// attention, csrc/attention/attention_post_kernels.cu:79,101: kv_head_idx = head_mapping[head_idx]).
template <int D>
__device__ __forceinline__ uint32_t kv_lane_off(const int32_t* head_map, int head, int lane) {
  const int kvh = head_map ? head_map[head] : head;
  return (uint32_t)(kvh * D + HeadLanes<D>::chunk(lane) * 8);
}

// One request's list [t0, t1) through one wave, whatever the element type: loads the query (at lane_off of the
// query row; NQ > 1: the NQ adjacent query heads from there on) and runs the streaming body (K/V at kv_off of every
// token row).
template <typename E, int D, int TB, int STAGES, int NQ = 1>
__device__ __forceinline__ void stream_request(const uint16_t* q, int64_t q_off, const uint16_t* kc, const uint16_t* vc,
                                               int64_t row_stride, const int32_t* slots, int myslot, int t0, int t1,
                                               uint32_t lane_off, uint32_t kv_off, float scale_log2e, bool head_ok,
                                               float* opart, float* ml, int64_t pr) {
  const int lane = threadIdx.x & 63;
  if constexpr (is_f32<E>::value) {
    static_assert(NQ == 1, "grouped streaming is built for 16-bit elements");
    float qf[8];
    load8f<F32>(q, q_off + lane_off, qf);
    if (!HeadLanes<D>::active(lane)) {
#pragma unroll
      for (int i = 0; i < 8; ++i) qf[i] = 0.f;
    }
    stream_item_f32<D, TB>(reinterpret_cast<const float*>(kc), reinterpret_cast<const float*>(vc), row_stride, slots,
                           myslot, t0, t1, qf, kv_off, scale_log2e, head_ok, opart, ml, pr);
  } else {
    u32x4 qv[NQ];
#pragma unroll
    for (int n = 0; n < NQ; ++n) {
      qv[n] = ld16(q + q_off + lane_off + n * D);
      if (!HeadLanes<D>::active(lane)) qv[n] = u32x4{0u, 0u, 0u, 0u};
    }
    stream_item<E, D, TB, STAGES, NQ>(kc, vc, row_stride, slots, myslot, t0, t1, qv, kv_off, scale_log2e, head_ok,
                                      opart, ml, pr);
  }
}

// One piece of the balanced form for one head group: the piece's items (request, first token, count) are
// streamed one after the other by this wave, one partial row per item.
// (rec0, rec1) = the piece's lane record, already loaded by the caller
// NQ > 1: the waves divide the a.H / NQ runs of NQ adjacent query heads; run r reads KV head r >> a.kv_shift (a KV
// head's query heads are one run, or 2, 4 .. adjacent runs).
template <typename E, int D, int TB, int STAGES, int NQ = 1>
__device__ __forceinline__ void run_piece_rec(const ItemArgs& a, int hg, int4 rec0, int4 rec1) {
  constexpr int LPH = HeadLanes<D>::LPH;
  constexpr int HPW = HeadLanes<D>::HPW;
  const int lane = threadIdx.x & 63;
  const int heads = NQ > 1 ? a.H / NQ : a.H;  // the heads the waves divide among themselves
  const int head = hg * HPW + lane / LPH;
  const bool head_ok = head < heads;
  const int hclamp = head_ok ? head : heads - 1;
  const uint32_t lane_off = (uint32_t)(hclamp * NQ * D + HeadLanes<D>::chunk(lane) * 8);  // the (first) query head
  const uint32_t kv_off = NQ > 1 ? (uint32_t)((hclamp >> a.kv_shift) * D + HeadLanes<D>::chunk(lane) * 8)
                                 : kv_lane_off<D>(a.head_map, hclamp, lane);
  const int i0 = rec0.x, i1 = rec0.x + rec0.y;
  for (int it = i0; it < i1; ++it) {
    int4 meta = {rec0.z, rec0.w, rec1.x, 0};
    if (it > i0) meta = a.items[it];  // request, first token, token count
    const int b = meta.x, t0 = meta.y, t1 = meta.y + meta.z;
    const int32_t* slots = a.slots + (a.offsets ? a.offsets[b] : (int64_t)b * a.table_stride);
    const int myslot = slots[min(t0 + lane, t1 - 1)];
    stream_request<E, D, TB, STAGES, NQ>(a.q, (int64_t)b * a.q_stride, a.kc, a.vc, a.row_stride, slots, myslot, t0, t1,
                                         lane_off, kv_off, a.scale_log2e, head_ok, a.opart, a.ml,
                                         (int64_t)it * a.H + hclamp * NQ);
  }
}

template <typename E, int D, int TB, int STAGES, int NQ = 1>
__device__ __forceinline__ void run_piece(const ItemArgs& a, int piece, int hg) {
  // lane record: (first item, item count, then the first item's request / first token / count inline,
  // so the first K/V rows are three dependent loads away from launch, not five)
  run_piece_rec<E, D, TB, STAGES, NQ>(a, hg, a.lane_rec[2 * piece], a.lane_rec[2 * piece + 1]);
}

}  // namespace ph
