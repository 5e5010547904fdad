// Decode attention over token-granular slot tables: per-request partial
// attention (suffix phase and the non-shared ragged decode), and the n-way
// log-sum-exp merge.  HBM-bound (1 FLOP per KV byte): no MFMA, no LDS.
//
// Mapping: in the [slot, H, D] pool all heads of a token are one contiguous
// row.  A wave owns HPW = 64 / (D/8) adjacent heads of one (request, chunk):
// each lane loads 8 contiguous elements (one 128-bit load), so a wave reads a
// contiguous HPW*D*2-byte span of every token row.  The D/8 lanes of a head
// combine their partial dot products with a butterfly; softmax runs online in
// the exp2 domain; slot ids are fetched 64 at a time into one VGPR and
// broadcast through v_readlane.
//
// Math restated from csrc/attention/attention_post_kernels.cu:74-341 (suffix
// phase + merge), attention_prev_kernels.cu:147,223,332-337 (m / l export) and
// parrot/engine/builtin/kernels/shared_flash_decoding.py:137-199 (n-way reduce).
#include "decode.hpp"

namespace ph {

template <typename E, int D, int TB>
__global__ __launch_bounds__(256) void decode_partial_kernel(PartialArgs a) {
  constexpr int LPH = D / 8;       // lanes per head
  constexpr int HPW = kWave / LPH;  // heads per wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int hgroups = (a.H + HPW - 1) / HPW;
  const int item = wave / hgroups;
  const int hg = wave - item * hgroups;
  const int rb = item / a.n_chunks;  // request index inside this launch
  const int c = item - rb * a.n_chunks;
  if (rb >= a.num_reqs) return;
  const int b = a.req_begin + rb;

  int64_t off;
  int len;
  if (a.shared_cu) {
    off = a.shared_cu[0];
    len = a.shared_cu[1] - a.shared_cu[0];
  } else if (a.shared_len >= 0) {
    off = 0;
    len = a.shared_len;
  } else {
    off = a.offsets ? a.offsets[b] : (int64_t)b * a.table_stride;
    len = a.lens[b];
  }
  const int t0 = c * a.chunk;
  if (t0 >= len) return;
  const int t1 = min(len, t0 + a.chunk);

  const int head = hg * HPW + lane / LPH;
  const bool head_ok = head < a.H;
  const int hclamp = head_ok ? head : a.H - 1;
  const int64_t lane_off = (int64_t)hclamp * D + (lane % LPH) * 8;

  const u32x4 qv = ld16(a.q + (int64_t)b * a.q_stride + lane_off);
  const int32_t* slots = a.slots + off;

  float m = -INFINITY, l = 0.f;
  float o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = 0.f;

  for (int tb = t0; tb < t1; tb += kWave) {
    const int mine = min(tb + lane, t1 - 1);
    const int myslot = slots[mine];
    const int nb = min(kWave, t1 - tb);
    for (int j0 = 0; j0 < nb; j0 += TB) {
      u32x4 kk[TB], vv[TB];
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        const int64_t slot = __builtin_amdgcn_readlane(myslot, j0 + j);
        const int64_t ro = slot * a.row_stride + lane_off;
        kk[j] = ld16(a.kc + ro);
        vv[j] = ld16(a.vc + ro);
      }
      float s[TB];
      float mb = -INFINITY;
#pragma unroll
      for (int j = 0; j < TB; ++j) {
        float d = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) d = Elem<E>::dot2(qv[w], kk[j][w], d);
        d = group_sum<LPH>(d) * a.scale_log2e;
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
        for (int w = 0; w < 4; ++w) {
          o[2 * w] += p * Elem<E>::lo(vv[j][w]);
          o[2 * w + 1] += p * Elem<E>::hi(vv[j][w]);
        }
      }
      m = mn;
    }
  }

  if (!head_ok) return;
  const float inv = 1.f / l;
  const int64_t pr = ((int64_t)(a.part_base + c) * a.B + b) * a.H + head;
  float* op = a.opart + pr * D + (lane % LPH) * 8;
  float4_t o0 = {o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
  float4_t o1 = {o[4] * inv, o[5] * inv, o[6] * inv, o[7] * inv};
  *reinterpret_cast<float4_t*>(op) = o0;
  *reinterpret_cast<float4_t*>(op + 4) = o1;
  if (lane % LPH == 0) {
    a.ml[pr * 2] = m;
    a.ml[pr * 2 + 1] = l;
  }
}

// One wave per (request, HPW heads): fold every valid partial.
template <typename E, int D>
__global__ __launch_bounds__(256) void merge_kernel(MergeArgs a) {
  constexpr int LPH = D / 8;
  constexpr int HPW = kWave / LPH;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4 + (threadIdx.x >> 6));
  const int hgroups = (a.H + HPW - 1) / HPW;
  const int b = wave / hgroups;
  const int hg = wave - b * hgroups;
  if (b >= a.B) return;
  const int head = hg * HPW + lane / LPH;
  if (head >= a.H) return;
  const int dl = (lane % LPH) * 8;

  float M = -INFINITY, L = 0.f;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;

  if (a.prev_m) {  // a partial already sitting in out / prev_m / prev_l
    const float lp = a.prev_l[(int64_t)b * a.H + head];
    if (lp > 0.f) {
      const u32x4 ov = ld16(a.out + (int64_t)b * a.out_stride + (int64_t)head * D + dl);
      M = a.prev_m[(int64_t)b * a.H + head];
      L = lp;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        acc[2 * w] = lp * Elem<E>::lo(ov[w]);
        acc[2 * w + 1] = lp * Elem<E>::hi(ov[w]);
      }
    }
  }

  const int nB = a.lens ? (a.lens[b] + a.chunk - 1) / a.chunk : 0;
  const int total = a.nA + nB;
  for (int i = 0; i < total; ++i) {
    const int part = i < a.nA ? i : a.baseB + (i - a.nA);
    const int64_t pr = ((int64_t)part * a.B + b) * a.H + head;
    const float lp = a.ml[pr * 2 + 1];
    if (lp > 0.f) {
      const float mp = a.ml[pr * 2];
      const float* op = a.opart + pr * D + dl;
      const float4_t o0 = *reinterpret_cast<const float4_t*>(op);
      const float4_t o1 = *reinterpret_cast<const float4_t*>(op + 4);
      const float Mn = fmaxf(M, mp);
      const float sc = __builtin_amdgcn_exp2f(M - Mn);
      const float w = __builtin_amdgcn_exp2f(mp - Mn) * lp;
      L = L * sc + w;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[k] = acc[k] * sc + w * o0[k];
        acc[4 + k] = acc[4 + k] * sc + w * o1[k];
      }
      M = Mn;
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  u32x4 r;
#pragma unroll
  for (int w = 0; w < 4; ++w) r[w] = pack2<E>(acc[2 * w] * inv, acc[2 * w + 1] * inv);
  st16(a.out + (int64_t)b * a.out_stride + (int64_t)head * D + dl, r);
  if (a.m_out && dl == 0) {
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
static int launch_partial_t(const PartialArgs& a, hipStream_t st) {
  constexpr int HPW = kWave / (D / 8);
  const int64_t hgroups = (a.H + HPW - 1) / HPW;
  const int64_t waves = (int64_t)a.num_reqs * a.n_chunks * hgroups;
  if (waves == 0) return PH_OK;
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  hipLaunchKernelGGL((decode_partial_kernel<E, D, 8>), grid, block, 0, st, a);
  return launch_status();
}

template <typename E, int D>
static int launch_merge_t(const MergeArgs& a, hipStream_t st) {
  constexpr int HPW = kWave / (D / 8);
  const int64_t hgroups = (a.H + HPW - 1) / HPW;
  const int64_t waves = (int64_t)a.B * hgroups;
  if (waves == 0) return PH_OK;
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  hipLaunchKernelGGL((merge_kernel<E, D>), grid, block, 0, st, a);
  return launch_status();
}

#define PH_DISPATCH(FN, dtype, D, ...)                                  \
  do {                                                                  \
    if ((dtype) == PH_F16) {                                            \
      if ((D) == 128) return FN<F16, 128>(__VA_ARGS__);                 \
      if ((D) == 64) return FN<F16, 64>(__VA_ARGS__);                   \
      if ((D) == 256) return FN<F16, 256>(__VA_ARGS__);                 \
    } else {                                                            \
      if ((D) == 128) return FN<BF16, 128>(__VA_ARGS__);                \
      if ((D) == 64) return FN<BF16, 64>(__VA_ARGS__);                  \
      if ((D) == 256) return FN<BF16, 256>(__VA_ARGS__);                \
    }                                                                   \
    return PH_ERR_HEAD_DIM;                                             \
  } while (0)

int launch_partial(const PartialArgs& a, int dtype, int D, hipStream_t st) {
  PH_DISPATCH(launch_partial_t, dtype, D, a, st);
}
int launch_merge(const MergeArgs& a, int dtype, int D, hipStream_t st) {
  PH_DISPATCH(launch_merge_t, dtype, D, a, st);
}
int launch_clear_ml(float* ml, int64_t entries, hipStream_t st) {
  if (entries == 0) return PH_OK;
  const int64_t n2 = entries * 2;
  hipLaunchKernelGGL(clear_ml_kernel, dim3((unsigned)((n2 + 255) / 256)), dim3(256), 0, st, ml, n2);
  return launch_status();
}

}  // namespace ph
