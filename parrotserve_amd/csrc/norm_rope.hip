// RMSNorm and NeoX rotary embedding.  Both are HBM-bound: 128-bit I/O, the row
// stays in registers between the reduction and the write (one HBM read), wave64
// shuffle reduction plus one LDS hop across the four waves.
//
// Arithmetic restated from 3rdparty/vllm/csrc/layernorm_kernels.cu:9-35,
// parrot/engine/builtin/kernels/rms_norm.py:15-46,
// 3rdparty/vllm/csrc/pos_encoding_kernels.cu:6-65 and
// parrot/engine/builtin/kernels/rotary_embedding.py:24-104.
#include "common.hpp"

namespace ph {

constexpr int kNormThreads = 256;

__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = group_sum<64>(v);
  const int w = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  return red[0] + red[1] + red[2] + red[3];
}

// One workgroup per ROWS consecutive rows; ITERS 16-byte chunks per thread and row are kept in registers.  The
// rows' loads and the weights' are all requested before the first reduction, so a workgroup has ROWS rows in
// flight and pays the load -> reduce -> store chain once per round.  Measured at 8192 x 5120 fp16: three rows per
// workgroup 29.6 us (71 % of HBM peak) against 31.4 us with one, 32 us with four; with one row per workgroup the
// weights are better read behind the reduction (31.4 against 35 us), with three ahead of it (29.6 against 31.4).
template <typename E, int ITERS, bool ROUND_FIRST, int ROWS>
__global__ __launch_bounds__(kNormThreads) void rms_norm_vec(uint16_t* __restrict__ out,
                                                             const uint16_t* __restrict__ x,
                                                             const uint16_t* __restrict__ w, float eps,
                                                             int n, int64_t rows, int64_t x_stride,
                                                             int64_t out_stride) {
  __shared__ float red[ROWS][4];
  const int64_t row0 = (int64_t)blockIdx.x * ROWS;
  const int chunks = n >> 3;
  u32x4 v[ROWS][ITERS], wv[ITERS];
  float ss[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    const uint16_t* xr = x + (row0 + r < rows ? row0 + r : rows - 1) * x_stride;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = threadIdx.x + i * kNormThreads;
      if (c < chunks) v[r][i] = ld16_nt(xr + c * 8);
    }
  }
  if (ROWS > 1) {
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = threadIdx.x + i * kNormThreads;
      if (c < chunks) wv[i] = ld16(w + c * 8);
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    ss[r] = 0.f;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = threadIdx.x + i * kNormThreads;
      if (c < chunks) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float a = Elem<E>::lo(v[r][i][j]), b = Elem<E>::hi(v[r][i][j]);
          ss[r] += a * a + b * b;
        }
      }
    }
    ss[r] = group_sum<64>(ss[r]);
    if ((threadIdx.x & 63) == 0) red[r][threadIdx.x >> 6] = ss[r];
  }
  __syncthreads();
  if (ROWS == 1) {
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = threadIdx.x + i * kNormThreads;
      if (c < chunks) wv[i] = ld16(w + c * 8);
    }
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    if (row0 + r >= rows) break;
    const float tot = red[r][0] + red[r][1] + red[r][2] + red[r][3];
    const float rstd = rsqrtf(tot / (float)n + eps);
    uint16_t* orow = out + (row0 + r) * out_stride;
#pragma unroll
    for (int i = 0; i < ITERS; ++i) {
      const int c = threadIdx.x + i * kNormThreads;
      if (c < chunks) {
        u32x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float a = Elem<E>::lo(v[r][i][j]) * rstd, b = Elem<E>::hi(v[r][i][j]) * rstd;
          if (ROUND_FIRST) {
            a = rnd<E>(a);
            b = rnd<E>(b);
          }
          o[j] = pack2<E>(a * Elem<E>::lo(wv[i][j]), b * Elem<E>::hi(wv[i][j]));
        }
        st16(orow + c * 8, o);
      }
    }
  }
}

// Any n / alignment: two passes over the row, scalar accesses.
template <typename E, bool ROUND_FIRST>
__global__ __launch_bounds__(kNormThreads) void rms_norm_generic(typename ElemStore<E>::T* __restrict__ out,
                                                                 const typename ElemStore<E>::T* __restrict__ x,
                                                                 const typename ElemStore<E>::T* __restrict__ w,
                                                                 float eps, int n, int64_t x_stride,
                                                                 int64_t out_stride) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const typename ElemStore<E>::T* xr = x + row * x_stride;
  typename ElemStore<E>::T* orow = out + row * out_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += kNormThreads) {
    const float a = Elem<E>::one(xr[i]);
    ss += a * a;
  }
  ss = block_sum_256(ss, red);
  const float rstd = rsqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += kNormThreads) {
    float a = Elem<E>::one(xr[i]) * rstd;
    if (ROUND_FIRST) a = rnd<E>(a);
    orow[i] = Elem<E>::bits(a * Elem<E>::one(w[i]));
  }
}

template <typename E, bool RF>
static int launch_rms(void* out, const void* x, const void* w, float eps, int64_t rows, int64_t n,
                      int64_t xs, int64_t os, hipStream_t st) {
  uint16_t* o = (uint16_t*)out;
  const uint16_t* xi = (const uint16_t*)x;
  const uint16_t* wi = (const uint16_t*)w;
  const bool vec = n % 8 == 0 && xs % 8 == 0 && os % 8 == 0 && aligned16(out) && aligned16(x) && aligned16(w) &&
                   n <= 8 * kNormThreads * 8;
  dim3 grid((unsigned)rows), block(kNormThreads);
  if (vec) {
    const int iters = (int)((n / 8 + kNormThreads - 1) / kNormThreads);
    // three rows per workgroup once there are rows enough to fill the device that way
    const bool multi = rows >= 2048 && iters <= 4;
    const dim3 vgrid((unsigned)(multi ? (rows + 2) / 3 : rows));
#define PH_RMS(I)                                                                                                \
  do {                                                                                                           \
    if (multi)                                                                                                   \
      hipLaunchKernelGGL((rms_norm_vec<E, I, RF, 3>), vgrid, block, 0, st, o, xi, wi, eps, (int)n, rows, xs, os); \
    else                                                                                                         \
      hipLaunchKernelGGL((rms_norm_vec<E, I, RF, 1>), vgrid, block, 0, st, o, xi, wi, eps, (int)n, rows, xs, os); \
  } while (0)
    if (iters <= 1) PH_RMS(1);
    else if (iters <= 2) PH_RMS(2);
    else if (iters <= 3) PH_RMS(3);
    else if (iters <= 4) PH_RMS(4);
    else PH_RMS(8);
#undef PH_RMS
  } else {
    hipLaunchKernelGGL((rms_norm_generic<E, RF>), grid, block, 0, st, o, xi, wi, eps, (int)n, xs, os);
  }
  return launch_status();
}

// 32-bit elements: the element-wise kernel (rounding to the element type is the identity, so both rounding orders
// of the 16-bit kernels coincide)
static int launch_rms_f32(void* out, const void* x, const void* w, float eps, int64_t rows, int64_t n, int64_t xs,
                          int64_t os, hipStream_t st) {
  hipLaunchKernelGGL((rms_norm_generic<F32, false>), dim3((unsigned)rows), dim3(kNormThreads), 0, st, (float*)out,
                     (const float*)x, (const float*)w, eps, (int)n, xs, os);
  return launch_status();
}

// ------------------------------------------------------------------------- //
// RoPE.  One workgroup per token; a work unit is 8 rotation pairs of one head:
// 8 x (first half), the matching 8 y (second half), 8 cos, 8 sin.
// Element-type arithmetic: every product and the final sum/difference is
// rounded to the element type, as the reference's CUDA kernel does.
template <typename E>
__global__ __launch_bounds__(256) void rope_vec(const int64_t* __restrict__ positions, uint16_t* q, uint16_t* k,
                                                const uint16_t* __restrict__ cos_base,
                                                const uint16_t* __restrict__ sin_base, int64_t cs_stride,
                                                int hq, int hk, int64_t q_stride_n, int64_t q_stride_h,
                                                int64_t k_stride_n, int64_t k_stride_h, int half_rot) {
  const int64_t t = blockIdx.x;
  const int64_t p = positions ? positions[t] : t;
  const uint16_t* cr = cos_base + p * cs_stride;
  const uint16_t* sr = sin_base + p * cs_stride;
  const int upd = half_rot >> 3;  // units per head
  const int units = (hq + hk) * upd;
  // four units per thread and pass: all their loads are issued before the first rotation, so a thread keeps
  // up to sixteen 16-byte loads in flight instead of four
  constexpr int UN = 4;
  for (int u0 = threadIdx.x; u0 < units; u0 += 256 * UN) {
    uint16_t* base[UN];
    int cc[UN];
    u32x4 x[UN], y[UN], cs[UN], sn[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      const int u = u0 + j * 256;
      const bool ok = u < units;
      const int uu = ok ? u : u0;
      const int h = uu / upd;
      cc[j] = (uu - h * upd) * 8;
      base[j] = h < hq ? q + t * q_stride_n + (int64_t)h * q_stride_h
                       : k + t * k_stride_n + (int64_t)(h - hq) * k_stride_h;
      x[j] = ld16(base[j] + cc[j]);
      y[j] = ld16(base[j] + half_rot + cc[j]);
      cs[j] = ld16(cr + cc[j]);
      sn[j] = ld16(sr + cc[j]);
    }
#pragma unroll
    for (int j = 0; j < UN; ++j) {
      if (u0 + j * 256 < units) {
        rotate8<E>(x[j], y[j], cs[j], sn[j]);
        st16(base[j] + cc[j], x[j]);
        st16(base[j] + half_rot + cc[j], y[j]);
      }
    }
  }
}

template <typename E>
__global__ __launch_bounds__(256) void rope_generic(const int64_t* __restrict__ positions,
                                                    typename ElemStore<E>::T* q, typename ElemStore<E>::T* k,
                                                    const typename ElemStore<E>::T* __restrict__ cos_base,
                                                    const typename ElemStore<E>::T* __restrict__ sin_base,
                                                    int64_t cs_stride,
                                                    int hq, int hk, int64_t q_stride_n, int64_t q_stride_h,
                                                    int64_t k_stride_n, int64_t k_stride_h, int half_rot) {
  const int64_t t = blockIdx.x;
  const int64_t p = positions ? positions[t] : t;
  const typename ElemStore<E>::T* cr = cos_base + p * cs_stride;
  const typename ElemStore<E>::T* sr = sin_base + p * cs_stride;
  const int units = (hq + hk) * half_rot;
  for (int u = threadIdx.x; u < units; u += 256) {
    const int h = u / half_rot;
    const int i = u - h * half_rot;
    typename ElemStore<E>::T* base = h < hq ? q + t * q_stride_n + (int64_t)h * q_stride_h
                            : k + t * k_stride_n + (int64_t)(h - hq) * k_stride_h;
    const float x = Elem<E>::one(base[i]), y = Elem<E>::one(base[half_rot + i]);
    const float c = Elem<E>::one(cr[i]), s = Elem<E>::one(sr[i]);
    base[i] = Elem<E>::bits(rnd<E>(x * c) - rnd<E>(y * s));
    base[half_rot + i] = Elem<E>::bits(rnd<E>(y * c) + rnd<E>(x * s));
  }
}

template <typename E>
static int launch_rope(const int64_t* pos, void* q, void* k, const void* cosb, const void* sinb, int64_t cs_stride,
                       int64_t T, int hq, int hk, int64_t qsn, int64_t qsh, int64_t ksn, int64_t ksh, int half_rot,
                       hipStream_t st) {
  const bool vec = half_rot % 8 == 0 && aligned16(q) && (hk == 0 || aligned16(k)) && aligned16(cosb) &&
                   aligned16(sinb) && cs_stride % 8 == 0 && qsn % 8 == 0 && qsh % 8 == 0 &&
                   (hk == 0 || (ksn % 8 == 0 && ksh % 8 == 0));
  dim3 grid((unsigned)T), block(256);
  if (vec)
    hipLaunchKernelGGL((rope_vec<E>), grid, block, 0, st, pos, (uint16_t*)q, (uint16_t*)k, (const uint16_t*)cosb,
                       (const uint16_t*)sinb, cs_stride, hq, hk, qsn, qsh, ksn, ksh, half_rot);
  else
    hipLaunchKernelGGL((rope_generic<E>), grid, block, 0, st, pos, (uint16_t*)q, (uint16_t*)k, (const uint16_t*)cosb,
                       (const uint16_t*)sinb, cs_stride, hq, hk, qsn, qsh, ksn, ksh, half_rot);
  return launch_status();
}

// 32-bit elements: the element-wise kernel (fp32 products and sums, as the reference's CUDA kernel computes in float)
static int launch_rope_f32(const int64_t* pos, void* q, void* k, const void* cosb, const void* sinb, int64_t cs_stride,
                           int64_t T, int hq, int hk, int64_t qsn, int64_t qsh, int64_t ksn, int64_t ksh, int half_rot,
                           hipStream_t st) {
  hipLaunchKernelGGL((rope_generic<F32>), dim3((unsigned)T), dim3(256), 0, st, pos, (float*)q, (float*)k,
                     (const float*)cosb, (const float*)sinb, cs_stride, hq, hk, qsn, qsh, ksn, ksh, half_rot);
  return launch_status();
}

}  // namespace ph

using namespace ph;

extern "C" int ph_rms_norm(void* out, const void* x, const void* weight, float eps, int64_t rows, int64_t n,
                           int64_t x_stride, int64_t out_stride, int dtype, int round_before_weight,
                           void* stream) {
  if (rows < 0 || n <= 0 || x_stride < n || out_stride < n) return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (rows == 0) return PH_OK;
  if (!out || !x || !weight) return PH_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == PH_F32) return launch_rms_f32(out, x, weight, eps, rows, n, x_stride, out_stride, st);
  if (dtype == PH_F16)
    return round_before_weight ? launch_rms<F16, true>(out, x, weight, eps, rows, n, x_stride, out_stride, st)
                               : launch_rms<F16, false>(out, x, weight, eps, rows, n, x_stride, out_stride, st);
  return round_before_weight ? launch_rms<BF16, true>(out, x, weight, eps, rows, n, x_stride, out_stride, st)
                             : launch_rms<BF16, false>(out, x, weight, eps, rows, n, x_stride, out_stride, st);
}

extern "C" int ph_rope_neox(const int64_t* positions, void* q, void* k, const void* cos_sin_cache,
                            int64_t num_tokens, int64_t num_q_heads, int64_t num_k_heads, int64_t head_dim,
                            int64_t rot_dim, int64_t q_stride, int64_t k_stride, int dtype, void* stream) {
  if (num_tokens < 0 || num_q_heads <= 0 || num_k_heads < 0 || head_dim <= 0 || rot_dim <= 0 || rot_dim % 2 ||
      rot_dim > head_dim)
    return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (num_tokens == 0) return PH_OK;
  if (!positions || !q || !cos_sin_cache || (num_k_heads > 0 && !k)) return PH_ERR_ARG;
  const int half = (int)(rot_dim / 2);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == PH_F32)
    return launch_rope_f32(positions, q, k, cos_sin_cache, (const float*)cos_sin_cache + half, rot_dim, num_tokens,
                           (int)num_q_heads, (int)num_k_heads, q_stride, head_dim, k_stride, head_dim, half, st);
  const uint16_t* cosb = (const uint16_t*)cos_sin_cache;
  const uint16_t* sinb = cosb + half;
  if (dtype == PH_F16)
    return launch_rope<F16>(positions, q, k, cosb, sinb, rot_dim, num_tokens, (int)num_q_heads, (int)num_k_heads,
                            q_stride, head_dim, k_stride, head_dim, half, st);
  return launch_rope<BF16>(positions, q, k, cosb, sinb, rot_dim, num_tokens, (int)num_q_heads, (int)num_k_heads,
                           q_stride, head_dim, k_stride, head_dim, half, st);
}

extern "C" int ph_rotary_embedding(void* state, const void* cos, const void* sin, int64_t num_tokens,
                                   int64_t num_heads, int64_t head_dim, int64_t stride_n, int64_t stride_h,
                                   int64_t cs_stride, int dtype, void* stream) {
  if (num_tokens < 0 || num_heads <= 0 || head_dim <= 0 || head_dim % 2) return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (num_tokens == 0) return PH_OK;
  if (!state || !cos || !sin) return PH_ERR_ARG;
  hipStream_t st = (hipStream_t)stream;
  const int half = (int)(head_dim / 2);
  if (dtype == PH_F32)
    return launch_rope_f32(nullptr, state, nullptr, cos, sin, cs_stride, num_tokens, (int)num_heads, 0, stride_n,
                           stride_h, 0, 0, half, st);
  if (dtype == PH_F16)
    return launch_rope<F16>(nullptr, state, nullptr, cos, sin, cs_stride, num_tokens, (int)num_heads, 0, stride_n,
                            stride_h, 0, 0, half, st);
  return launch_rope<BF16>(nullptr, state, nullptr, cos, sin, cs_stride, num_tokens, (int)num_heads, 0, stride_n,
                           stride_h, 0, 0, half, st);
}
