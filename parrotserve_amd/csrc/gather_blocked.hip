// Gather of token rows out of block-structured KV caches (the vLLM layouts):
//   K  [num_blocks, H, D/x, block_size, x]     dest[di, h, c*x + e] = K[slot / bs, h, c, slot % bs, e]
//   V  [num_blocks, H, D,   block_size]        dest[di, h, d]       = V[slot / bs, h, d, slot % bs]
// into token-granular rows [n, H, D].  Pure bit copy, HBM-bound.  Both layouts are one strided source whose
// smallest contiguous piece belonging to a single token is a *unit* of x elements (K) or one element (V); a
// token row is H * D/x units, scattered with the block-offset stride between neighbouring tokens of a block.
//
// Fast path: a workgroup takes 16 consecutive list entries.  Reads put the entry index on the fastest lane
// axis, so entries that are neighbours in a block (the common case: a context occupies whole blocks) are
// read as one contiguous run of 16 units; the units go through a padded LDS tile and leave as 128-bit
// non-temporal stores along the destination rows (256 contiguous bytes per head row at D = 128, 16-bit).
// Generic path: any strides and element sizes, one workgroup per entry, one element per thread step.
//
// Behaviour restated from parrot/engine/builtin/kernels/tokens_moving.py:104-313
// (move_tokens_from_blocked_k_cache / move_tokens_from_blocked_v_cache and their Triton kernels).
#include "common.hpp"

namespace ph {

struct GatherArgs {
  const char* cache;
  char* dest;
  const void* src_slots;
  const void* dest_idx;
  int64_t n;
  int64_t block_size;
  int64_t sn, sh, sc, sb, sx;  // cache strides in bytes: block, head, unit column, block offset, element in unit
  int64_t dn, dh, dd;          // destination strides in bytes: row, head, element
  int heads;
  int head_dim;    // elements per head
  int x;           // elements per unit
  int elem_bytes;
  int ru_log2;     // fast path: log2(units per head row)
  int head_bytes;  // fast path: D * elem_bytes
  int runs_ok;     // fast path, units under 16 bytes: neighbouring block offsets are neighbours in memory and
                   // everything is 16-byte aligned, so 16 / unit-size consecutive slots can share one load
};

constexpr int kG = 16;    // list entries per workgroup
constexpr int kPad = 16;  // bytes appended to every LDS row (spreads the transposed accesses over the banks)

template <int UB>
struct UnitT;
template <>
struct UnitT<2> { using type = uint16_t; };
template <>
struct UnitT<4> { using type = uint32_t; };
template <>
struct UnitT<8> { using type = u32x2; };
template <>
struct UnitT<16> { using type = u32x4; };

template <int UB, int HB, typename IDX>
__global__ __launch_bounds__(256) void gather_units_kernel(GatherArgs a) {
  using U = typename UnitT<UB>::type;
  extern __shared__ __attribute__((aligned(16))) char tile[];  // [HB][kG][head_bytes + kPad]
  constexpr int UNR = UB >= 16 ? 4 : 8;
  const int tid = threadIdx.x;
  const int pitch = a.head_bytes + kPad;
  const int64_t i0 = (int64_t)blockIdx.x * kG;
  // read role: entry jr, unit columns tid >> 4, + 16, ...
  const int jr = tid & (kG - 1);
  const bool valid_r = i0 + jr < a.n;
  const char* sbase = a.cache;
  if (valid_r) {
    const int64_t slot = (int64_t) reinterpret_cast<const IDX*>(a.src_slots)[i0 + jr];
    const int64_t b = slot / a.block_size;
    sbase += b * a.sn + (slot - b * a.block_size) * a.sb;
  }
  // write role: entry jw, 16-byte chunks tid & 15, + 16, ...
  const int jw = tid >> 4, l16 = tid & 15;
  const bool valid_w = i0 + jw < a.n;
  char* dbase = a.dest;
  if (valid_w) dbase += (int64_t) reinterpret_cast<const IDX*>(a.dest_idx)[i0 + jw] * a.dn;
  const int ru_mask = (1 << a.ru_log2) - 1;
  const int units_round = HB << a.ru_log2;
  const int cpr = a.head_bytes >> 4;

  // Units under 16 bytes (the V layout: one element): when every aligned group of R = 16 / UB entries of this
  // workgroup is R consecutive slots starting at a multiple of R, one 128-bit load brings a unit column of all
  // R tokens, and the pieces are dealt to the tokens' LDS rows.
  bool runs = false;
  int g = 0, col0 = 0;
  const char* rbase = a.cache;
  if constexpr (UB < 16) {
    constexpr int R = 16 / UB, NG = kG / R;
    g = tid % NG;
    col0 = tid / NG;
    bool ok = a.runs_ok != 0 && i0 + kG <= a.n;
    if (ok) {
      const IDX* sl = reinterpret_cast<const IDX*>(a.src_slots) + i0 + g * R;
      const int64_t s0 = (int64_t)sl[0];
      ok = s0 % R == 0;
#pragma unroll
      for (int r = 1; r < R; ++r) ok = ok && (int64_t)sl[r] == s0 + r;
      const int64_t b = s0 / a.block_size;
      rbase += b * a.sn + (s0 - b * a.block_size) * a.sb;
    }
    runs = __syncthreads_and(ok);
  }

  for (int h0 = 0; h0 < a.heads; h0 += HB) {
    if constexpr (UB < 16) {
      if (runs) {
        constexpr int R = 16 / UB, NG = kG / R;
        const int cols_round = HB << a.ru_log2;  // unit columns of HB heads
        for (int k0 = col0; k0 < cols_round; k0 += (256 / NG) * 4) {
          u32x4 v[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int cu = k0 + (256 / NG) * u;
            const int hh = cu >> a.ru_log2, c = cu & ru_mask;
            if (cu < cols_round && h0 + hh < a.heads)
              v[u] = ld16(rbase + (int64_t)(h0 + hh) * a.sh + (int64_t)c * a.sc);
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int cu = k0 + (256 / NG) * u;
            const int hh = cu >> a.ru_log2, c = cu & ru_mask;
            if (cu < cols_round && h0 + hh < a.heads) {
              U piece[R];
              __builtin_memcpy(piece, &v[u], 16);
#pragma unroll
              for (int r = 0; r < R; ++r)
                *reinterpret_cast<U*>(tile + (hh * kG + g * R + r) * pitch + c * UB) = piece[r];
            }
          }
        }
      }
    }
    if (!runs)
    for (int k0 = tid >> 4; k0 < units_round; k0 += 16 * UNR) {
      U v[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int cu = k0 + 16 * u;
        const int hh = cu >> a.ru_log2, c = cu & ru_mask;
        if (cu < units_round && h0 + hh < a.heads && valid_r)
          v[u] = *reinterpret_cast<const U*>(sbase + (int64_t)(h0 + hh) * a.sh + (int64_t)c * a.sc);
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int cu = k0 + 16 * u;
        const int hh = cu >> a.ru_log2, c = cu & ru_mask;
        if (cu < units_round && h0 + hh < a.heads && valid_r)
          *reinterpret_cast<U*>(tile + (hh * kG + jr) * pitch + c * UB) = v[u];
      }
    }
    __syncthreads();
    if (valid_w) {
#pragma unroll
      for (int hh = 0; hh < HB; ++hh) {
        if (h0 + hh >= a.heads) break;
        for (int m = l16; m < cpr; m += 16) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(tile + (hh * kG + jw) * pitch + m * 16);
          st16_nt(dbase + (int64_t)(h0 + hh) * a.head_bytes + m * 16, v);
        }
      }
    }
    __syncthreads();
  }
}

template <typename IDX, typename W>
__global__ __launch_bounds__(256) void gather_generic_kernel(GatherArgs a) {
  const int per_row = a.heads * a.head_dim;
  for (int64_t i = blockIdx.x; i < a.n; i += gridDim.x) {
    const int64_t slot = (int64_t) reinterpret_cast<const IDX*>(a.src_slots)[i];
    const int64_t di = (int64_t) reinterpret_cast<const IDX*>(a.dest_idx)[i];
    const int64_t b = slot / a.block_size;
    const char* sp = a.cache + b * a.sn + (slot - b * a.block_size) * a.sb;
    char* dp = a.dest + di * a.dn;
    for (int e = threadIdx.x; e < per_row; e += 256) {
      const int h = e / a.head_dim;
      const int d = e - h * a.head_dim;
      const int c = d / a.x;
      const W v = *reinterpret_cast<const W*>(sp + h * a.sh + c * a.sc + (d - c * a.x) * a.sx);
      *reinterpret_cast<W*>(dp + h * a.dh + d * a.dd) = v;
    }
  }
}

namespace {

bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

template <int UB, typename IDX>
int launch_units(const GatherArgs& a, hipStream_t st) {
  const unsigned grid = (unsigned)((a.n + kG - 1) / kG);
  const int row = kG * (a.head_bytes + kPad);
  if (a.head_bytes <= 512) {
    hipLaunchKernelGGL((gather_units_kernel<UB, 4, IDX>), dim3(grid), dim3(256), 4 * row, st, a);
  } else {
    hipLaunchKernelGGL((gather_units_kernel<UB, 1, IDX>), dim3(grid), dim3(256), row, st, a);
  }
  return launch_status();
}

template <typename IDX>
int launch_gather(GatherArgs& a, hipStream_t st) {
  const int64_t ub = (int64_t)a.x * a.elem_bytes;
  const int64_t head_bytes = (int64_t)a.head_dim * a.elem_bytes;
  const int64_t ru = a.head_dim / a.x;
  const bool fast = (ub == 2 || ub == 4 || ub == 8 || ub == 16) && (a.x == 1 || a.sx == a.elem_bytes) &&
                    a.dd == a.elem_bytes && a.dh == head_bytes && head_bytes % 16 == 0 && head_bytes <= 2048 &&
                    is_pow2(ru) && a.sn % ub == 0 && a.sh % ub == 0 && a.sc % ub == 0 && a.sb % ub == 0 &&
                    reinterpret_cast<uintptr_t>(a.cache) % ub == 0 && aligned16(a.dest) && a.dn % 16 == 0 &&
                    a.n / kG < (int64_t)0x7fffffff;
  if (fast) {
    a.head_bytes = (int)head_bytes;
    a.runs_ok = ub < 16 && a.sb == ub && a.block_size % (16 / ub) == 0 && aligned16(a.cache) && a.sn % 16 == 0 &&
                a.sh % 16 == 0 && a.sc % 16 == 0;
    a.ru_log2 = 0;
    while ((1 << a.ru_log2) < ru) ++a.ru_log2;
    switch ((int)ub) {
      case 2: return launch_units<2, IDX>(a, st);
      case 4: return launch_units<4, IDX>(a, st);
      case 8: return launch_units<8, IDX>(a, st);
      default: return launch_units<16, IDX>(a, st);
    }
  }
  const int64_t max_grid = 1 << 20;
  const dim3 grid((unsigned)(a.n < max_grid ? a.n : max_grid));
  switch (a.elem_bytes) {
    case 1: hipLaunchKernelGGL((gather_generic_kernel<IDX, uint8_t>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((gather_generic_kernel<IDX, uint16_t>), grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL((gather_generic_kernel<IDX, uint32_t>), grid, dim3(256), 0, st, a); break;
    case 8: hipLaunchKernelGGL((gather_generic_kernel<IDX, uint64_t>), grid, dim3(256), 0, st, a); break;
    default: return PH_ERR_DTYPE;
  }
  return launch_status();
}

int gather_entry(const void* cache, void* dest, const void* src_slots, const void* dest_idx, int index_type, int64_t n,
                 int64_t num_heads, int64_t head_dim, int64_t block_size, int64_t x, int elem_bytes, int64_t sn,
                 int64_t sh, int64_t sc, int64_t sb, int64_t sx, int64_t dn, int64_t dh, int64_t dd, void* stream) {
  if (n < 0 || num_heads <= 0 || head_dim <= 0 || block_size <= 0 || x <= 0 || head_dim % x != 0 ||
      num_heads * head_dim > (1 << 24))
    return PH_ERR_ARG;
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return PH_ERR_DTYPE;
  if (index_type != PH_IDX_I32 && index_type != PH_IDX_I64) return PH_ERR_ARG;
  if (n == 0) return PH_OK;
  if (!cache || !dest || !src_slots || !dest_idx) return PH_ERR_ARG;
  GatherArgs a{};
  a.cache = (const char*)cache;
  a.dest = (char*)dest;
  a.src_slots = src_slots;
  a.dest_idx = dest_idx;
  a.n = n;
  a.block_size = block_size;
  a.sn = sn * elem_bytes;
  a.sh = sh * elem_bytes;
  a.sc = sc * elem_bytes;
  a.sb = sb * elem_bytes;
  a.sx = sx * elem_bytes;
  a.dn = dn * elem_bytes;
  a.dh = dh * elem_bytes;
  a.dd = dd * elem_bytes;
  a.heads = (int)num_heads;
  a.head_dim = (int)head_dim;
  a.x = (int)x;
  a.elem_bytes = elem_bytes;
  hipStream_t st = (hipStream_t)stream;
  return index_type == PH_IDX_I64 ? launch_gather<int64_t>(a, st) : launch_gather<int32_t>(a, st);
}

}  // namespace
}  // namespace ph

using namespace ph;

extern "C" int ph_gather_blocked_k(const void* k_cache, void* dest, const void* src_slots, const void* dest_idx,
                                   int index_type, int64_t n, int64_t num_heads, int64_t head_dim, int64_t block_size,
                                   int64_t x, int elem_bytes, int64_t stride_n, int64_t stride_h, int64_t stride_c,
                                   int64_t stride_b, int64_t stride_x, int64_t dst_stride_n, int64_t dst_stride_h,
                                   int64_t dst_stride_d, void* stream) {
  return gather_entry(k_cache, dest, src_slots, dest_idx, index_type, n, num_heads, head_dim, block_size, x, elem_bytes,
                      stride_n, stride_h, stride_c, stride_b, stride_x, dst_stride_n, dst_stride_h, dst_stride_d,
                      stream);
}

extern "C" int ph_gather_blocked_v(const void* v_cache, void* dest, const void* src_slots, const void* dest_idx,
                                   int index_type, int64_t n, int64_t num_heads, int64_t head_dim, int64_t block_size,
                                   int elem_bytes, int64_t stride_n, int64_t stride_h, int64_t stride_d,
                                   int64_t stride_b, int64_t dst_stride_n, int64_t dst_stride_h, int64_t dst_stride_d,
                                   void* stream) {
  return gather_entry(v_cache, dest, src_slots, dest_idx, index_type, n, num_heads, head_dim, block_size, 1, elem_bytes,
                      stride_n, stride_h, stride_d, stride_b, 0, dst_stride_n, dst_stride_h, dst_stride_d, stream);
}
