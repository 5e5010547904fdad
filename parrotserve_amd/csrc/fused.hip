// Fused forms of the small per-layer kernels around the attention op.  Decode batches make these
// launch-bound (a few microseconds each, a dozen per layer), so each fusion removes a launch and a pass:
//   residual += x; y = RMSNorm(residual) * w        (two torch adds + norm -> one kernel per norm)
//   out = silu(gate) * up                           (torch silu + mul -> one kernel)
//   RoPE(q, k) in place + K/V rows to their slots   (rotary kernel + cache append -> one kernel)
// Arithmetic is that of the unfused sequence, rounding step by step in the element type where the
// reference's kernels / torch ops do:
//   adds: parrot/engine/builtin/models/llama.py:160-178 (torch add in the element type)
//   norm: 3rdparty/vllm/csrc/layernorm_kernels.cu:9-35, parrot/engine/builtin/kernels/rms_norm.py:15-46
//   activation: 3rdparty/vllm/csrc/activation_kernels.cu:6-24 (silu in fp32, rounded, then the product)
//   rotary + append: 3rdparty/vllm/csrc/pos_encoding_kernels.cu:6-65, cache_kernels.cu:142-224
#include "common.hpp"

namespace ph {

constexpr int kFusedThreads = 256;

__device__ __forceinline__ float block_sum4(float v, float* red) {
  v = group_sum<64>(v);
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// One workgroup per row; ITERS 16-byte chunks per thread stay in registers between the sum and the write.
template <typename E, int ITERS, bool ROUND_FIRST>
__global__ __launch_bounds__(kFusedThreads) void add_rms_norm_vec(uint16_t* __restrict__ out, uint16_t* residual,
                                                                 const uint16_t* __restrict__ x,
                                                                 const uint16_t* __restrict__ w, float eps, int n,
                                                                 int64_t x_stride, int64_t r_stride,
                                                                 int64_t out_stride) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * x_stride;
  uint16_t* rr = residual + row * r_stride;
  uint16_t* orow = out + row * out_stride;
  const int chunks = n >> 3;
  u32x4 v[ITERS];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = threadIdx.x + i * kFusedThreads;
    if (c < chunks) {
      const u32x4 a = ld16(xr + c * 8), b = ld16(rr + c * 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // the sum is stored (rounded) as the new residual, and the norm runs on the stored value
        const uint32_t s = pack2<E>(Elem<E>::lo(a[j]) + Elem<E>::lo(b[j]), Elem<E>::hi(a[j]) + Elem<E>::hi(b[j]));
        v[i][j] = s;
        const float lo = Elem<E>::lo(s), hi = Elem<E>::hi(s);
        ss += lo * lo + hi * hi;
      }
      st16(rr + c * 8, v[i]);
    }
  }
  ss = block_sum4(ss, red);
  const float rstd = rsqrtf(ss / (float)n + eps);
#pragma unroll
  for (int i = 0; i < ITERS; ++i) {
    const int c = threadIdx.x + i * kFusedThreads;
    if (c < chunks) {
      const u32x4 wv = ld16(w + c * 8);
      u32x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float a = Elem<E>::lo(v[i][j]) * rstd, b = Elem<E>::hi(v[i][j]) * rstd;
        if (ROUND_FIRST) {
          a = rnd<E>(a);
          b = rnd<E>(b);
        }
        o[j] = pack2<E>(a * Elem<E>::lo(wv[j]), b * Elem<E>::hi(wv[j]));
      }
      st16(orow + c * 8, o);
    }
  }
}

// Any n / alignment: element accesses, the row is re-read after the reduction.
template <typename E, bool ROUND_FIRST>
__global__ __launch_bounds__(kFusedThreads) void add_rms_norm_generic(uint16_t* __restrict__ out, uint16_t* residual,
                                                                     const uint16_t* __restrict__ x,
                                                                     const uint16_t* __restrict__ w, float eps, int n,
                                                                     int64_t x_stride, int64_t r_stride,
                                                                     int64_t out_stride) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const uint16_t* xr = x + row * x_stride;
  uint16_t* rr = residual + row * r_stride;
  uint16_t* orow = out + row * out_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += kFusedThreads) {
    const uint16_t s = Elem<E>::bits(Elem<E>::one(xr[i]) + Elem<E>::one(rr[i]));
    rr[i] = s;
    const float a = Elem<E>::one(s);
    ss += a * a;
  }
  ss = block_sum4(ss, red);  // the barrier inside also orders each thread's own writes before its re-reads
  const float rstd = rsqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += kFusedThreads) {
    float a = Elem<E>::one(rr[i]) * rstd;
    if (ROUND_FIRST) a = rnd<E>(a);
    orow[i] = Elem<E>::bits(a * Elem<E>::one(w[i]));
  }
}

template <typename E, bool RF>
static int launch_add_rms(void* out, void* residual, const void* x, const void* w, float eps, int64_t rows, int64_t n,
                          int64_t xs, int64_t rs, int64_t os, hipStream_t st) {
  uint16_t* o = (uint16_t*)out;
  uint16_t* r = (uint16_t*)residual;
  const uint16_t* xi = (const uint16_t*)x;
  const uint16_t* wi = (const uint16_t*)w;
  const bool vec = n % 8 == 0 && xs % 8 == 0 && rs % 8 == 0 && os % 8 == 0 && aligned16(out) && aligned16(x) &&
                   aligned16(residual) && aligned16(w) && n <= 8 * kFusedThreads * 8;
  dim3 grid((unsigned)rows), block(kFusedThreads);
  if (vec) {
    const int iters = (int)((n / 8 + kFusedThreads - 1) / kFusedThreads);
#define PH_ARMS(I) \
  hipLaunchKernelGGL((add_rms_norm_vec<E, I, RF>), grid, block, 0, st, o, r, xi, wi, eps, (int)n, xs, rs, os)
    if (iters <= 1) PH_ARMS(1);
    else if (iters <= 2) PH_ARMS(2);
    else if (iters <= 3) PH_ARMS(3);
    else if (iters <= 4) PH_ARMS(4);
    else PH_ARMS(8);
#undef PH_ARMS
  } else {
    hipLaunchKernelGGL((add_rms_norm_generic<E, RF>), grid, block, 0, st, o, r, xi, wi, eps, (int)n, xs, rs, os);
  }
  return launch_status();
}

// silu(gate) * up: silu in fp32, rounded to the element type, then the product rounded again.
template <typename E>
__device__ __forceinline__ float silu_mul_one(float g, float u) {
  const float s = rnd<E>(g / (1.0f + __expf(-g)));
  return s * u;
}

template <typename E>
__global__ __launch_bounds__(256) void silu_mul_vec(uint16_t* __restrict__ out, const uint16_t* __restrict__ gate,
                                                    const uint16_t* __restrict__ up, int64_t rows, int chunks,
                                                    int64_t g_stride, int64_t u_stride, int64_t o_stride) {
  const int64_t total = rows * chunks;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / chunks;
    const int c = (int)(i - r * chunks) * 8;
    const u32x4 g = ld16(gate + r * g_stride + c), u = ld16(up + r * u_stride + c);
    u32x4 o;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j] = pack2<E>(silu_mul_one<E>(Elem<E>::lo(g[j]), Elem<E>::lo(u[j])),
                      silu_mul_one<E>(Elem<E>::hi(g[j]), Elem<E>::hi(u[j])));
    st16(out + r * o_stride + c, o);
  }
}

template <typename E>
__global__ __launch_bounds__(256) void silu_mul_generic(uint16_t* __restrict__ out, const uint16_t* __restrict__ gate,
                                                        const uint16_t* __restrict__ up, int64_t rows, int d,
                                                        int64_t g_stride, int64_t u_stride, int64_t o_stride) {
  const int64_t total = rows * d;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / d;
    const int c = (int)(i - r * d);
    out[r * o_stride + c] =
        Elem<E>::bits(silu_mul_one<E>(Elem<E>::one(gate[r * g_stride + c]), Elem<E>::one(up[r * u_stride + c])));
  }
}

template <typename E>
static int launch_silu_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t d, int64_t gs,
                           int64_t us, int64_t os, hipStream_t st) {
  const bool vec = d % 8 == 0 && gs % 8 == 0 && us % 8 == 0 && os % 8 == 0 && aligned16(out) && aligned16(gate) &&
                   aligned16(up);
  const int64_t work = vec ? rows * (d / 8) : rows * d;
  int64_t blocks = (work + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  dim3 grid((unsigned)blocks), block(256);
  if (vec)
    hipLaunchKernelGGL((silu_mul_vec<E>), grid, block, 0, st, (uint16_t*)out, (const uint16_t*)gate,
                       (const uint16_t*)up, rows, (int)(d / 8), gs, us, os);
  else
    hipLaunchKernelGGL((silu_mul_generic<E>), grid, block, 0, st, (uint16_t*)out, (const uint16_t*)gate,
                       (const uint16_t*)up, rows, (int)d, gs, us, os);
  return launch_status();
}

// One workgroup per token: rotate q and k heads (whole head rotated: rot_dim == head_dim), q in place, write the
// rotated k row and the v row to the token's slot; k itself is rewritten only when the caller wants it
// (k_in_place): a caller that reads K from the cache from here on saves the read-modify-write of the k rows,
// a quarter of the pass's time.
template <typename E, typename IDX>
__global__ __launch_bounds__(256) void rope_append_vec(const int64_t* __restrict__ positions, uint16_t* q, uint16_t* k,
                                                       const uint16_t* __restrict__ v,
                                                       const uint16_t* __restrict__ cos_sin, uint16_t* k_cache,
                                                       uint16_t* v_cache, const IDX* __restrict__ slot_mapping, int hq,
                                                       int hk, int D, int64_t q_stride, int64_t k_stride,
                                                       int64_t v_stride, int64_t cache_stride, int k_in_place) {
  const int64_t t = blockIdx.x;
  const int64_t p = positions[t];
  const int64_t slot = (int64_t)slot_mapping[t];
  const int half = D >> 1;
  const uint16_t* cr = cos_sin + p * D;
  const uint16_t* sr = cr + half;
  const int upd = half >> 3;  // rotation units (8 pairs) per head
  const int rot_units = (hq + hk) * upd;
  const int v_units = hk * (D >> 3);
  uint16_t* kc = k_cache + slot * cache_stride;
  uint16_t* vc = v_cache + slot * cache_stride;
  // UN units per thread and pass, every load of the pass issued before the first rotation or store (a thread
  // keeps up to 4 UN 16-byte loads in flight); rotation units first, then the v row's copy units
  constexpr int UN = 3;
  for (int u0 = threadIdx.x; u0 < rot_units; u0 += 256 * UN) {
    uint16_t* base[UN];
    int cc[UN], hh[UN];
    u32x4 x[UN], y[UN], cs[UN], sn[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int u = u0 + j * 256;
      if (u < rot_units) {
        const int h = u / upd;
        hh[j] = h;
        cc[j] = (u - h * upd) * 8;
        base[j] = h >= hq ? k + t * k_stride + (int64_t)(h - hq) * D : q + t * q_stride + (int64_t)h * D;
        x[j] = ld16_nt(base[j] + cc[j]);
        y[j] = ld16_nt(base[j] + half + cc[j]);
        cs[j] = ld16(cr + cc[j]);
        sn[j] = ld16(sr + cc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      if (u0 + j * 256 < rot_units) {
        rotate8<E>(x[j], y[j], cs[j], sn[j]);
        if (k_in_place || hh[j] < hq) {
          st16(base[j] + cc[j], x[j]);
          st16(base[j] + half + cc[j], y[j]);
        }
        if (hh[j] >= hq) {
          uint16_t* dst = kc + (int64_t)(hh[j] - hq) * D;
          st16(dst + cc[j], x[j]);
          st16(dst + half + cc[j], y[j]);
        }
      }
    }
  }
  for (int u0 = threadIdx.x; u0 < v_units; u0 += 256 * UN) {
    u32x4 w[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j)
      if (u0 + j * 256 < v_units) w[j] = ld16_nt(v + t * v_stride + (u0 + j * 256) * 8);
#pragma unroll
    for (int j = 0; j < UN; ++j)
      if (u0 + j * 256 < v_units) st16(vc + (u0 + j * 256) * 8, w[j]);
  }
}

}  // namespace ph

using namespace ph;

extern "C" int ph_add_rms_norm(void* out, void* residual, const void* x, const void* weight, float eps, int64_t rows,
                               int64_t n, int64_t x_stride, int64_t residual_stride, int64_t out_stride, int dtype,
                               int round_before_weight, void* stream) {
  if (rows < 0 || n <= 0 || x_stride < n || residual_stride < n || out_stride < n) return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16) return PH_ERR_DTYPE;
  if (rows == 0) return PH_OK;
  if (!out || !residual || !x || !weight) return PH_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
#define PH_GO(E, RF) launch_add_rms<E, RF>(out, residual, x, weight, eps, rows, n, x_stride, residual_stride, out_stride, st)
  if (dtype == PH_F16) return round_before_weight ? PH_GO(F16, true) : PH_GO(F16, false);
  return round_before_weight ? PH_GO(BF16, true) : PH_GO(BF16, false);
#undef PH_GO
}

extern "C" int ph_silu_mul(void* out, const void* gate, const void* up, int64_t rows, int64_t d, int64_t gate_stride,
                           int64_t up_stride, int64_t out_stride, int dtype, void* stream) {
  if (rows < 0 || d <= 0 || gate_stride < d || up_stride < d || out_stride < d) return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16) return PH_ERR_DTYPE;
  if (rows == 0) return PH_OK;
  if (!out || !gate || !up) return PH_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  return dtype == PH_F16 ? launch_silu_mul<F16>(out, gate, up, rows, d, gate_stride, up_stride, out_stride, st)
                         : launch_silu_mul<BF16>(out, gate, up, rows, d, gate_stride, up_stride, out_stride, st);
}

extern "C" int ph_rope_append(const int64_t* positions, void* q, void* k, const void* v, const void* cos_sin_cache,
                              void* k_cache, void* v_cache, const void* slot_mapping, int index_type,
                              int64_t num_tokens, int64_t num_q_heads, int64_t num_kv_heads, int64_t head_dim,
                              int64_t rot_dim, int64_t q_stride, int64_t k_stride, int64_t v_stride,
                              int64_t cache_stride_n, int dtype, int k_in_place, void* stream) {
  if (num_tokens < 0 || num_q_heads <= 0 || num_kv_heads <= 0 || head_dim <= 0 || rot_dim <= 0 || rot_dim % 2 ||
      rot_dim > head_dim)
    return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16) return PH_ERR_DTYPE;
  if (index_type != PH_IDX_I32 && index_type != PH_IDX_I64) return PH_ERR_ARG;
  if (num_tokens == 0) return PH_OK;
  if (!positions || !q || !k || !v || !cos_sin_cache || !k_cache || !v_cache || !slot_mapping) return PH_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  const bool fused = rot_dim == head_dim && head_dim % 16 == 0 && aligned16(q) && aligned16(k) && aligned16(v) &&
                     aligned16(cos_sin_cache) && aligned16(k_cache) && aligned16(v_cache) && q_stride % 8 == 0 &&
                     k_stride % 8 == 0 && v_stride % 8 == 0 && cache_stride_n % 8 == 0;
  if (!fused) {  // same result from the two separate kernels
    const int rc = ph_rope_neox(positions, q, k, cos_sin_cache, num_tokens, num_q_heads, num_kv_heads, head_dim,
                                rot_dim, q_stride, k_stride, dtype, stream);
    if (rc != PH_OK) return rc;
    return ph_kv_append(k, v, k_cache, v_cache, slot_mapping, index_type, num_tokens, num_kv_heads, head_dim, dtype,
                        k_stride, v_stride, cache_stride_n, stream);
  }
  dim3 grid((unsigned)num_tokens), block(256);
#define PH_GO(E, IDX)                                                                                              \
  hipLaunchKernelGGL((rope_append_vec<E, IDX>), grid, block, 0, st, positions, (uint16_t*)q, (uint16_t*)k,         \
                     (const uint16_t*)v, (const uint16_t*)cos_sin_cache, (uint16_t*)k_cache, (uint16_t*)v_cache,   \
                     (const IDX*)slot_mapping, (int)num_q_heads, (int)num_kv_heads, (int)head_dim, q_stride,       \
                     k_stride, v_stride, cache_stride_n, k_in_place)
  if (dtype == PH_F16) {
    if (index_type == PH_IDX_I64) PH_GO(F16, int64_t); else PH_GO(F16, int32_t);
  } else {
    if (index_type == PH_IDX_I64) PH_GO(BF16, int64_t); else PH_GO(BF16, int32_t);
  }
#undef PH_GO
  return launch_status();
}
