// Discontinuous token move and KV append: dest[dst[i]] = src[src[i]] for rows
// of [H, D] elements.  Pure bit copy, HBM-bound: 128-bit non-temporal loads,
// stores non-temporal or plain by entry point, one workgroup per row (rows are 8-10 KB at LLaMA head shapes), row
// indices read through the scalar unit (they are uniform per workgroup).
//
// Behaviour restated from parrot/engine/builtin/kernels/tokens_moving.py:25-100
// (free strides on all three axes, int64 indices) and
// 3rdparty/vllm/csrc/cache_kernels.cu:142-224 (append by slot_mapping).
#include "common.hpp"

namespace ph {

struct MoveSet {
  const char* src;
  char* dst;
  int64_t s_n, s_h, s_d;  // byte strides
  int64_t d_n, d_h, d_d;
};

struct MoveArgs {
  MoveSet set[2];  // gridDim.y selects (K, V share one launch on append)
  const void* sidx;
  const void* didx;
  int64_t n;
  int heads;
  int cph;         // 16-byte chunks per head (vector path)
  int head_dim;    // elements per head (generic path)
  int elem_bytes;  // generic path
};

template <typename IDX>
__device__ __forceinline__ int64_t row_of(const void* idx, int64_t i) {
  return idx ? (int64_t) reinterpret_cast<const IDX*>(idx)[i] : i;
}

// Vector path: innermost stride is one element and every head row is a whole
// number of aligned 16-byte chunks.  NT_STORE: non-temporal stores.  Measured: the pool-to-pool move of
// random rows is a little faster with them (61 % against 60 % of HBM peak), the append of freshly produced
// rows much faster without (81 % against 60 %), so the two entry points differ.
template <typename IDX, bool CONTIG, bool NT_STORE>
__global__ __launch_bounds__(256) void move_rows_vec16(MoveArgs a) {
  const MoveSet s = a.set[blockIdx.y];
  const int cpr = a.cph * a.heads;
  for (int64_t row = blockIdx.x; row < a.n; row += gridDim.x) {
    const int64_t si = row_of<IDX>(a.sidx, row);
    const int64_t di = row_of<IDX>(a.didx, row);
    const char* sp = s.src + si * s.s_n;
    char* dp = s.dst + di * s.d_n;
    for (int c0 = threadIdx.x; c0 < cpr; c0 += 256 * 4) {
      u32x4 buf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 256;
        if (c < cpr) {
          int64_t off;
          if (CONTIG) {
            off = (int64_t)c * 16;
          } else {
            const int h = c / a.cph;
            off = h * s.s_h + (int64_t)(c - h * a.cph) * 16;
          }
          buf[u] = ld16_nt(sp + off);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 256;
        if (c < cpr) {
          int64_t off;
          if (CONTIG) {
            off = (int64_t)c * 16;
          } else {
            const int h = c / a.cph;
            off = h * s.d_h + (int64_t)(c - h * a.cph) * 16;
          }
          if (NT_STORE) st16_nt(dp + off, buf[u]); else st16(dp + off, buf[u]);
        }
      }
    }
  }
}

// Generic path: any strides, any alignment, one element per thread step.
template <typename IDX, typename W>
__global__ __launch_bounds__(256) void move_rows_generic(MoveArgs a) {
  const MoveSet s = a.set[blockIdx.y];
  const int per_row = a.heads * a.head_dim;
  for (int64_t row = blockIdx.x; row < a.n; row += gridDim.x) {
    const int64_t si = row_of<IDX>(a.sidx, row);
    const int64_t di = row_of<IDX>(a.didx, row);
    for (int e = threadIdx.x; e < per_row; e += 256) {
      const int h = e / a.head_dim;
      const int d = e - h * a.head_dim;
      const W v = *reinterpret_cast<const W*>(s.src + si * s.s_n + h * s.s_h + d * s.s_d);
      *reinterpret_cast<W*>(s.dst + di * s.d_n + h * s.d_h + d * s.d_d) = v;
    }
  }
}

static bool set_vectorisable(const MoveSet& s, int64_t row_head_bytes, int elem_bytes) {
  return s.s_d == elem_bytes && s.d_d == elem_bytes && row_head_bytes % 16 == 0 && aligned16(s.src) &&
         aligned16(s.dst) && s.s_n % 16 == 0 && s.s_h % 16 == 0 && s.d_n % 16 == 0 && s.d_h % 16 == 0;
}

template <typename IDX, bool NT_STORE>
static int launch_move(MoveArgs& a, int nsets, hipStream_t st) {
  const int64_t head_bytes = (int64_t)a.head_dim * a.elem_bytes;
  bool vec = true, contig = true;
  for (int i = 0; i < nsets; ++i) {
    vec = vec && set_vectorisable(a.set[i], head_bytes, a.elem_bytes);
    contig = contig && a.set[i].s_h == head_bytes && a.set[i].d_h == head_bytes;
  }
  const int64_t max_grid = 1 << 20;
  dim3 grid((unsigned)(a.n < max_grid ? a.n : max_grid), nsets);
  if (vec) {
    a.cph = (int)(head_bytes / 16);
    if (contig)
      hipLaunchKernelGGL((move_rows_vec16<IDX, true, NT_STORE>), grid, dim3(256), 0, st, a);
    else
      hipLaunchKernelGGL((move_rows_vec16<IDX, false, NT_STORE>), grid, dim3(256), 0, st, a);
  } else {
    switch (a.elem_bytes) {
      case 1: hipLaunchKernelGGL((move_rows_generic<IDX, uint8_t>), grid, dim3(256), 0, st, a); break;
      case 2: hipLaunchKernelGGL((move_rows_generic<IDX, uint16_t>), grid, dim3(256), 0, st, a); break;
      case 4: hipLaunchKernelGGL((move_rows_generic<IDX, uint32_t>), grid, dim3(256), 0, st, a); break;
      case 8: hipLaunchKernelGGL((move_rows_generic<IDX, uint64_t>), grid, dim3(256), 0, st, a); break;
      default: return PH_ERR_DTYPE;
    }
  }
  return launch_status();
}

}  // namespace ph

using namespace ph;

extern "C" int ph_move_tokens(const void* src, void* dst, const void* src_idx, const void* dst_idx,
                              int index_type, int64_t n, int64_t num_heads, int64_t head_dim,
                              int elem_bytes, int64_t src_stride_n, int64_t src_stride_h,
                              int64_t src_stride_d, int64_t dst_stride_n, int64_t dst_stride_h,
                              int64_t dst_stride_d, void* stream) {
  if (n < 0 || num_heads <= 0 || head_dim <= 0 || num_heads * head_dim > (1 << 24)) return PH_ERR_ARG;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return PH_ERR_DTYPE;
  if (index_type != PH_IDX_I32 && index_type != PH_IDX_I64) return PH_ERR_ARG;
  if (n == 0) return PH_OK;
  if (!src || !dst) return PH_ERR_ARG;
  MoveArgs a{};
  a.set[0] = MoveSet{(const char*)src,          (char*)dst,
                     src_stride_n * elem_bytes, src_stride_h * elem_bytes, src_stride_d * elem_bytes,
                     dst_stride_n * elem_bytes, dst_stride_h * elem_bytes, dst_stride_d * elem_bytes};
  a.sidx = src_idx;
  a.didx = dst_idx;
  a.n = n;
  a.heads = (int)num_heads;
  a.head_dim = (int)head_dim;
  a.elem_bytes = elem_bytes;
  hipStream_t st = (hipStream_t)stream;
  return index_type == PH_IDX_I64 ? launch_move<int64_t, true>(a, 1, st) : launch_move<int32_t, true>(a, 1, st);
}

extern "C" int ph_kv_append(const void* k, const void* v, void* k_cache, void* v_cache,
                            const void* slot_mapping, int index_type, int64_t num_tokens,
                            int64_t num_heads, int64_t head_dim, int dtype, int64_t k_stride_n,
                            int64_t v_stride_n, int64_t cache_stride_n, void* stream) {
  if (num_tokens < 0 || num_heads <= 0 || head_dim <= 0) return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (index_type != PH_IDX_I32 && index_type != PH_IDX_I64) return PH_ERR_ARG;
  if (num_tokens == 0) return PH_OK;
  if (!k || !v || !k_cache || !v_cache || !slot_mapping) return PH_ERR_ARG;
  const int eb = dtype == PH_F32 ? 4 : 2;
  MoveArgs a{};
  a.set[0] = MoveSet{(const char*)k,  (char*)k_cache,      k_stride_n * eb, head_dim * eb, eb,
                     cache_stride_n * eb, head_dim * eb, eb};
  a.set[1] = MoveSet{(const char*)v,  (char*)v_cache,      v_stride_n * eb, head_dim * eb, eb,
                     cache_stride_n * eb, head_dim * eb, eb};
  a.sidx = nullptr;
  a.didx = slot_mapping;
  a.n = num_tokens;
  a.heads = (int)num_heads;
  a.head_dim = (int)head_dim;
  a.elem_bytes = eb;
  hipStream_t st = (hipStream_t)stream;
  return index_type == PH_IDX_I64 ? launch_move<int64_t, false>(a, 2, st) : launch_move<int32_t, false>(a, 2, st);
}
