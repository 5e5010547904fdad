// Shared device helpers for the gfx950 kernels: 16-bit element traits,
// 128-bit vector I/O, wave64 reductions, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "../../include/parrot_hip.h"

namespace ph {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct F16 {};   // IEEE binary16
struct BF16 {};  // bfloat16
struct F32 {};   // IEEE binary32: the per-request decode, merge, norm, rotary and copy kernels only (no matrix cores)

template <typename E>
struct is_f32 {
  static constexpr bool value = false;
};
template <>
struct is_f32<F32> {
  static constexpr bool value = true;
};

template <typename E>
struct Elem;

template <>
struct Elem<F16> {
  static __device__ __forceinline__ float lo(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu));
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
  }
  static __device__ __forceinline__ float one(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
  static __device__ __forceinline__ uint16_t bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
  static constexpr uint32_t kOnes = 0x3C003C00u;  // (1.0, 1.0)
  // acc + a.lo*b.lo + a.hi*b.hi with fp32 accumulate (v_dot2_f32_f16)
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), acc, false);
  }
};

template <>
struct Elem<BF16> {
  static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
  static __device__ __forceinline__ float one(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
  static __device__ __forceinline__ uint16_t bits(float f) {  // round to nearest even
    return __builtin_bit_cast(uint16_t, (__bf16)f);
  }
  static constexpr uint32_t kOnes = 0x3F803F80u;  // (1.0, 1.0)
  static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc, false);
  }
};

// Two floats -> one packed pair of elements, round to nearest even (v_cvt_pk_{f16,bf16}_f32).
template <typename E>
__device__ __forceinline__ uint32_t pack2(float a, float b);
template <>
__device__ __forceinline__ uint32_t pack2<F16>(float a, float b) {
  typedef float float2_t __attribute__((ext_vector_type(2)));
  const float2_t f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, half2_t));
}
template <>
__device__ __forceinline__ uint32_t pack2<BF16>(float a, float b) {
  const bf16x2_t v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, v);
}

template <>
struct Elem<F32> {
  static __device__ __forceinline__ float one(float b) { return b; }
  static __device__ __forceinline__ float bits(float f) { return f; }
};

// storage type of one element
template <typename E>
struct ElemStore {
  typedef uint16_t T;
};
template <>
struct ElemStore<F32> {
  typedef float T;
};

// Round a float to the element type and back (the "t(.)" of the reference's
// element-type arithmetic).
template <typename E>
__device__ __forceinline__ float rnd(float f) {
  return Elem<E>::one(Elem<E>::bits(f));
}

__device__ __forceinline__ u32x4 ld16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void st16(void* p, u32x4 v) { *reinterpret_cast<u32x4*>(p) = v; }
__device__ __forceinline__ u32x4 ld16_nt(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void st16_nt(void* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// Eight consecutive elements at element offset `off` behind `base`, as floats / from floats rounded to the element type.
template <typename E>
__device__ __forceinline__ void load8f(const void* base, int64_t off, float (&f)[8]) {
  if constexpr (is_f32<E>::value) {
    const float4_t a = *reinterpret_cast<const float4_t*>(reinterpret_cast<const float*>(base) + off);
    const float4_t b = *reinterpret_cast<const float4_t*>(reinterpret_cast<const float*>(base) + off + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[i] = a[i];
      f[4 + i] = b[i];
    }
  } else {
    const u32x4 v = ld16(reinterpret_cast<const uint16_t*>(base) + off);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      f[2 * k] = Elem<E>::lo(v[k]);
      f[2 * k + 1] = Elem<E>::hi(v[k]);
    }
  }
}
template <typename E>
__device__ __forceinline__ void store8f(void* base, int64_t off, const float (&f)[8]) {
  if constexpr (is_f32<E>::value) {
    *reinterpret_cast<float4_t*>(reinterpret_cast<float*>(base) + off) = float4_t{f[0], f[1], f[2], f[3]};
    *reinterpret_cast<float4_t*>(reinterpret_cast<float*>(base) + off + 4) = float4_t{f[4], f[5], f[6], f[7]};
  } else {
    u32x4 r;
#pragma unroll
    for (int k = 0; k < 4; ++k) r[k] = pack2<E>(f[2 * k], f[2 * k + 1]);
    st16(reinterpret_cast<uint16_t*>(base) + off, r);
  }
}

// v + (v of the lane selected by a DPP control): one v_add_f32_dpp, no LDS round trip.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
  return v + __builtin_bit_cast(float, moved);
}

// Sum over aligned groups of W lanes (W a power of two <= 64); every lane of
// the group ends with the group's sum.  Up to 16 lanes the exchange stays inside
// a DPP row: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror,
// row_mirror (pairing lanes, not an xor butterfly, which is all a sum needs).
template <int W>
__device__ __forceinline__ float group_sum(float v) {
  if (W >= 2) v = dpp_add<0xB1>(v);
  if (W >= 4) v = dpp_add<0x4E>(v);
  if (W >= 8) v = dpp_add<0x141>(v);
  if (W >= 16) v = dpp_add<0x140>(v);
  if (W >= 32) v += __shfl_xor(v, 16, kWave);
  if (W >= 64) v += __shfl_xor(v, 32, kWave);
  return v;
}
template <int W>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int s = W / 2; s >= 1; s >>= 1) v = fmaxf(v, __shfl_xor(v, s, kWave));
  return v;
}

// NeoX rotation of 8 pairs in the element type: every product and the final sum / difference is rounded
// to the element type, as the reference's CUDA kernel does (3rdparty/vllm/csrc/pos_encoding_kernels.cu:6-36).
template <typename E>
__device__ __forceinline__ void rotate8(u32x4& x, u32x4& y, const u32x4 c, const u32x4 s) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float xl = Elem<E>::lo(x[j]), xh = Elem<E>::hi(x[j]);
    const float yl = Elem<E>::lo(y[j]), yh = Elem<E>::hi(y[j]);
    const float cl = Elem<E>::lo(c[j]), ch = Elem<E>::hi(c[j]);
    const float sl = Elem<E>::lo(s[j]), sh = Elem<E>::hi(s[j]);
    const float nxl = rnd<E>(xl * cl) - rnd<E>(yl * sl);
    const float nxh = rnd<E>(xh * ch) - rnd<E>(yh * sh);
    const float nyl = rnd<E>(yl * cl) + rnd<E>(xl * sl);
    const float nyh = rnd<E>(yh * ch) + rnd<E>(xh * sh);
    x[j] = pack2<E>(nxl, nxh);
    y[j] = pack2<E>(nyl, nyh);
  }
}

// Optional timing of one kernel's own dispatch: the three main kernels of the decode path (prefix, suffix,
// merge) can be launched through hipExtLaunchKernelGGL, which stamps a start and a stop event with the
// dispatch's begin and end timestamps.  The events come in per call (ph_decode_attention_timed); null events
// (the normal case) make it a plain launch.
struct KernelEvents {
  hipEvent_t start = nullptr, stop = nullptr;
};

// Launch with the optional event pair; without events this is the ordinary launch call (the one that
// stream capture and every tool expects), the extended call is only used when a caller asked for timing.
#define PH_LAUNCH_TIMED(kernel, grid, block, shmem, stream, ev, ...)                                     \
  do {                                                                                                   \
    if ((ev).start || (ev).stop)                                                                         \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, (ev).start, (ev).stop, 0, __VA_ARGS__);  \
    else                                                                                                 \
      hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                               \
  } while (0)

// Lane mapping of the per-request decode kernels: a head's D elements are spread over LPH lanes of 8 elements
// each, LPH the power of two >= D / 8, so that a wave holds 64 / LPH whole heads.  For D = 80, 96, 112 the lanes
// past the head's last 8-element chunk are idle: they point at chunk 0 (a duplicate of another lane's load, no
// extra traffic), carry a zero query and store nothing.
constexpr int lanes_per_head(int D) {
  int p = 1;
  while (p * 8 < D) p <<= 1;
  return p;
}
template <int D>
struct HeadLanes {
  static constexpr int LPH = lanes_per_head(D);
  static constexpr int HPW = kWave / LPH;
  static __device__ __forceinline__ bool active(int lane) { return LPH * 8 == D || (lane % LPH) * 8 < D; }
  static __device__ __forceinline__ int chunk(int lane) { return active(lane) ? lane % LPH : 0; }
};

// Timeline marks of the decode kernels: nothing unless a profiling build defines PH_TL(i) (it then records a
// timestamp per wave at mark i).
#ifndef PH_TL
#define PH_TL(i)
#endif

inline int launch_status() { return hipGetLastError() == hipSuccess ? PH_OK : PH_ERR_LAUNCH; }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace ph
