// Shared-prefix flash-decoding on CDNA4 matrix cores.
//
// All queries of a group attend over the SAME prefix slots, so per head the
// phase is a dense contraction: S^T = K Q^T (tokens x queries), O^T = V^T P^T.
// Workgroup = (split of the prefix, head, group x 64-query tile), 4 waves.
// Each wave owns every fourth 32-token tile of the split and ALL queries of
// the tile, so each K/V byte is fetched from HBM once per (group, query tile)
// and crosses LDS once: global -> wave-private LDS tile (coalesced 128-bit gathers by slot, written
// by the load itself, double-buffered) -> MFMA operand layout.  No workgroup barrier in
// the main loop.  Online softmax in the exp2 domain, fp32 accumulation in
// v_mfma_f32_32x32x16_{f16,bf16}.  The four waves' partials are folded through
// LDS at the end and one (O, m, l) part per (split, request, head) is written.
//
// Operand layouts (lane = 32*h + r):
//   A (32 x 16): lane holds row r, 8 contraction elements chosen by (h, step)
//   B (16 x 32): lane holds column r, the same 8 contraction elements
//   C (32 x 32): lane holds column r, rows 8*j + 4*h + i at register 4*j + i
// The contraction index is a free permutation as long as A and B agree, which
// lets the fp32 S^T registers feed the second product as its B operand with no
// cross-lane movement.  V stays row-major [token][dim] in LDS; its transposed A
// operand comes from ds_read_b64_tr_b16, which hands lane j of each 16-lane
// group column j of a 4-row x 16-column block whose row addresses the lanes
// supply (source lane s -> row s/4, columns 4*(s%4)..+3).  Both tiles are
// XOR-swizzled in 16-byte chunks so that the 128-bit K reads and the
// transposing V reads are free of bank conflicts.
//
// Math restated from parrot/engine/builtin/kernels/shared_flash_decoding.py:34-134.
#include "decode.hpp"

namespace ph {

template <typename E>
struct Mfma32;
template <>
struct Mfma32<F16> {
  static __device__ __forceinline__ float16_t run(u32x4 a, u32x4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c,
                                                  0, 0, 0);
  }
};
template <>
struct Mfma32<BF16> {
  static __device__ __forceinline__ float16_t run(u32x4 a, u32x4 b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                   c, 0, 0, 0);
  }
};

constexpr int kPD = 128;             // head size handled by this kernel
constexpr int kTile = 32;            // tokens per wave tile
constexpr int kStage = 16384;        // one staged tile: K 8 KB + V 8 KB
constexpr int kWaveLds = 2 * kStage; // two stages per wave
constexpr int kVtOff = 8192;

// 16 bytes per lane from global memory straight into LDS (no VGPR staging): lane i's data lands at
// lds_addr + 16 * i (an LDS byte address, wave-uniform).  Issued as inline assembly on purpose: the compiler then
// does not tie later LDS reads of the *other* stage to these loads, so a whole tile stays in flight
// under the matrix work; completion is awaited explicitly (vmcnt) before a stage is read.
__device__ __forceinline__ void lds_dma16(const void* gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "memory");
}
// LDS byte address of a generic pointer into shared memory, as a wave-uniform scalar
__device__ __forceinline__ uint32_t lds_addr_of(const char* p) {
  return __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p);
}

__device__ __forceinline__ u32x4 lds_ld16(const char* p) { return *reinterpret_cast<const u32x4*>(p); }

typedef short short4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x2 lds_tr16(const char* p) {
  const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (short4_t __attribute__((address_space(3)))*)(const_cast<char*>(p)));
  return __builtin_bit_cast(u32x2, v);
}

// One 64-query (NQB = 2) or 32-query (NQB = 1) tile against the slot list [s0, s1).
struct TileWork {
  const uint16_t* qrow0;  // first query row of the tile, already offset to the head
  int64_t q_stride;
  int nq;                 // live queries in the tile
  const int32_t* slots;   // slot list base
  int s0, s1;             // token range of this workgroup
  int causal_off;         // CAUSAL: query i sees token t iff t <= causal_off + i
};

// Runs the tile on all four waves.  On return wave w holds, for the 32 dims [32w, 32w+32) of every
// query, the accumulators folded over the four waves (unnormalised, C layout: register 4j+i = dim
// 32w + 8j + 4h + i of query 32nb + ql), plus each query's final maximum and softmax denominator.
template <typename E, int NQB, bool CAUSAL>
__device__ __forceinline__ void attn_tile(const TileWork& wk, const uint16_t* __restrict__ kc,
                                          const uint16_t* __restrict__ vc, int64_t row_stride, int head,
                                          float scale_log2e, char* smem, float16_t (&ofold)[NQB], float (&mfin)[NQB],
                                          float (&lfin)[NQB]) {
  float16_t oacc[4][NQB];
  float m[NQB], lsum[NQB], mtrue[NQB];  // exponent reference, denominator relative to it, true running maximum
  constexpr float kSlack = 8.f;
  const int lane = threadIdx.x & 63;
  const int w = threadIdx.x >> 6;
  const int h = lane >> 5, ql = lane & 31;
  char* wl = smem + w * kWaveLds;
  const int32_t* slots = wk.slots;
  const int s1 = wk.s1;

#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    m[nb] = -INFINITY;
    mtrue[nb] = -INFINITY;
    lsum[nb] = 0.f;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][nb][r] = 0.f;
  }

  // global -> LDS staging without registers: instruction r covers tokens 4r .. 4r+3, 16 lanes per
  // token row; LDS chunk position c of row t receives global chunk c ^ swizzle(t), so the tiles sit
  // XOR-swizzled in LDS while every lane's destination stays lane-linear as the DMA requires.
  const int tl = lane >> 4, c = lane & 15;
  // per-lane source bases (the row offset slot * row bytes is one 64-bit multiply-add per load)
  const uint32_t row_bytes = (uint32_t)(row_stride * 2);
  const char* kbase[8];
#pragma unroll
  for (int r = 0; r < 8; ++r)
    kbase[r] = reinterpret_cast<const char*>(kc + (int64_t)head * kPD + ((c ^ ((4 * r + tl) & 15)) * 8));
  const char* vbase_g = reinterpret_cast<const char*>(vc + (int64_t)head * kPD + ((c ^ (4 * tl)) * 8));
  const uint32_t wl_lds = lds_addr_of(wl);
  // the 32 slot ids of a tile sit in one VGPR (lane l: token l & 31), fetched one tile ahead of the
  // rows in flight; a lane picks the id of the row it loads with a cross-lane read
  int snext = 0;
  auto fetch_slots = [&](int t0) { snext = slots[min(t0 + (lane & 31), s1 - 1)]; };
  auto fetch_rows = [&](int stage) {
    const uint32_t kb = wl_lds + stage * kStage;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const uint32_t slot = (uint32_t)__shfl(snext, 4 * r + tl, kWave);
      const uint64_t ro = (uint64_t)slot * row_bytes;
      lds_dma16(kbase[r] + ro, kb + r * 1024);
      lds_dma16(vbase_g + ro, kb + kVtOff + r * 1024);
    }
  };
  int tb = wk.s0 + kTile * w;
  int stage = 0;
  if (tb < s1) {
    fetch_slots(tb);
    fetch_rows(0);
    if (tb + 4 * kTile < s1) fetch_slots(tb + 4 * kTile);
  }

  // (issued after the first K/V rows so the two latencies overlap)
  // Q as the B operand: column = query ql (+32 nb), contraction chunk (h, s) = dims 64h + 8s .. +8
  u32x4 qop[NQB][8];
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    const int q = 32 * nb + ql;
    const bool ok = q < wk.nq;
    const uint16_t* qp = wk.qrow0 + (int64_t)(ok ? q : 0) * wk.q_stride + 64 * h;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      u32x4 v = ld16(qp + 8 * s);
      if (!ok) v = u32x4{0, 0, 0, 0};
      qop[nb][s] = v;
    }
  }

  for (; tb < s1; tb += 4 * kTile, stage ^= 1) {
    // this tile's rows (and the slot ids fetched behind them) have landed
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_sched_barrier(0);
    // next tile's rows go in flight into the other stage (last read a full iteration ago);
    // then the slot ids of the tile after that
    if (tb + 4 * kTile < s1) {
      fetch_rows(stage ^ 1);
      if (tb + 8 * kTile < s1) fetch_slots(tb + 8 * kTile);
    }
    const char* st = wl + stage * kStage;

    // S^T = K Q^T
    float16_t sacc[NQB];
    // All LDS operand reads of the tile are issued ahead of their consumers and pinned there with
    // scheduling barriers (left alone, the scheduler sinks every read next to the matrix instruction
    // that uses it and the LDS latency is paid once per instruction): the eight K operands before the
    // score product, the V operands right behind it so that they arrive under the softmax arithmetic.
    u32x4 ka[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) ka[s] = lds_ld16(st + ql * 256 + (((8 * h + s) ^ (ql & 15)) * 16));
    __builtin_amdgcn_sched_barrier(0);
    {
      const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int nb = 0; nb < NQB; ++nb) sacc[nb] = Mfma32<E>::run(ka[0], qop[nb][0], zero);
#pragma unroll
      for (int s = 1; s < 8; ++s)
#pragma unroll
        for (int nb = 0; nb < NQB; ++nb) sacc[nb] = Mfma32<E>::run(ka[s], qop[nb][s], sacc[nb]);
    }
    u32x4 va[4][2];
    {
      // A operand of O^T += V^T P^T (row = dim 32db + ql, contraction = the 8 tokens of (h, u)): two
      // transposing reads, tokens 16u + 4h + {0..3} and 16u + 8 + 4h + {0..3}.
      const int sl = lane & 15, rh = (lane >> 4) & 1;
      const int trow = 4 * h + (sl >> 2);                       // + 16u + 8x
      const int tcol = 2 * rh + ((sl & 3) >> 1);                // + 4db, in 16-byte chunks
      const int tswz = 4 * (sl >> 2);                           // = 4 * (row & 3)
      const char* vbase = st + kVtOff + trow * 256 + (sl & 1) * 8;
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const int chunk = ((4 * db + tcol) ^ tswz) * 16;
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const u32x2 lo = lds_tr16(vbase + (16 * u) * 256 + chunk);
          const u32x2 hi = lds_tr16(vbase + (16 * u + 8) * 256 + chunk);
          va[db][u] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    // Online softmax in the exp2 domain, in two phases around the (rare) accumulator rescale, so that
    // the exponent work of one query block and the P.V matrix instructions of the other share a
    // scheduling region and can overlap.  Tokens need masking only in a split's last tile and, when
    // causal, in tiles that reach past what the tile's first query may see.
    const bool full = tb + kTile <= s1 && (!CAUSAL || tb + kTile - 1 <= wk.causal_off);
    float x[NQB][16], mref[NQB], alpha[NQB];
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
      if (full) {
#pragma unroll
        for (int r = 0; r < 16; ++r) x[nb][r] = sacc[nb][r];
      } else {
        const int tmax = CAUSAL ? min(s1 - 1, wk.causal_off + 32 * nb + ql) : s1 - 1;  // last visible token
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int t = 8 * (r >> 2) + 4 * h + (r & 3);
          x[nb][r] = (tb + t <= tmax) ? sacc[nb][r] : -INFINITY;
        }
      }
      float mloc = fmaxf(fmaxf(x[nb][0], x[nb][1]), fmaxf(x[nb][2], x[nb][3]));
#pragma unroll
      for (int r = 4; r < 16; r += 4)
        mloc = fmaxf(mloc, fmaxf(fmaxf(x[nb][r], x[nb][r + 1]), fmaxf(x[nb][r + 2], x[nb][r + 3])));
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, kWave)) * scale_log2e;  // scale > 0 keeps the order
      mtrue[nb] = fmaxf(mtrue[nb], mloc);
      // The exponent reference m[nb] follows the running maximum lazily: it moves only when the maximum
      // has outgrown it by more than kSlack (so P stays below 2^kSlack, well inside fp16/bf16 range).
      const bool move = mloc > m[nb] + kSlack;
      const float mnew = move ? mloc : m[nb];
      mref[nb] = (mnew == -INFINITY) ? 0.f : mnew;           // a row with nothing visible yet
      const bool had = m[nb] != -INFINITY;                   // accumulators are still zero otherwise
      alpha[nb] = (move && had) ? __builtin_amdgcn_exp2f(m[nb] - mref[nb]) : 1.f;
      m[nb] = mnew;
    }
    bool rescale = false;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) rescale = rescale || alpha[nb] != 1.f;
    if (__builtin_amdgcn_ballot_w64(rescale) != 0) {  // wave-uniform, rare
      // The accumulators live in accumulation registers, which the vector ALU cannot multiply in
      // place.  The round trip is written as assembly pinned inside this branch so that it is not
      // hoisted into the common path (where it would cost hundreds of register moves per tile).
      // Wait states: the matrix results are 16 passes deep before the reads, and the rewritten
      // registers are read as the C operand of the next matrix instruction after the writes.
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
      for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float t;
            asm volatile("v_accvgpr_read_b32 %0, %1\n\tv_mul_f32 %0, %0, %2\n\tv_accvgpr_write_b32 %1, %0"
                         : "=&v"(t), "+a"(oacc[db][nb][r])
                         : "v"(alpha[nb]));
          }
      asm volatile("s_nop 7" ::: "memory");
    }
    // exponentials, denominators, P^T packed straight into B-operand form, and O^T += V^T P^T
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb) {
      float ps = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        x[nb][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[nb][r], scale_log2e, -mref[nb]));
        ps += x[nb][r];
      }
      lsum[nb] = lsum[nb] * alpha[nb] + ps;
      u32x4 pop[2];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) pop[u][e] = pack2<E>(x[nb][8 * u + 2 * e], x[nb][8 * u + 2 * e + 1]);
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int u = 0; u < 2; ++u) oacc[db][nb] = Mfma32<E>::run(va[db][u], pop[u], oacc[db][nb]);
    }
  }

  // Fold the four waves.  Every wave parks the three 32-dim blocks it does not own, and its (m, l);
  // after one barrier wave w folds block w of all four waves, so the fold and the write-out that
  // follows run on the whole workgroup.
  constexpr int kBlk = NQB * 16 * 256;            // bytes of one (source wave, dim block): NQB x 16 floats x 64 lanes
  char* mlb = smem + 16 * kBlk;                    // [wave][m or l][nb][lane] floats
  __syncthreads();                                 // the staging tiles are dead from here on
#pragma unroll
  for (int db = 0; db < 4; ++db) {
    if (db == w) continue;
    char* base = smem + (w * 4 + db) * kBlk + lane * 16;
#pragma unroll
    for (int nb = 0; nb < NQB; ++nb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4_t v = {oacc[db][nb][4 * j], oacc[db][nb][4 * j + 1], oacc[db][nb][4 * j + 2],
                            oacc[db][nb][4 * j + 3]};
        *reinterpret_cast<float4_t*>(base + (nb * 4 + j) * 1024) = v;
      }
  }
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    *reinterpret_cast<float*>(mlb + ((w * 2 + 0) * NQB + nb) * 256 + lane * 4) = m[nb];
    *reinterpret_cast<float*>(mlb + ((w * 2 + 1) * NQB + nb) * 256 + lane * 4) = lsum[nb];
    *reinterpret_cast<float*>(mlb + ((8 + w) * NQB + nb) * 256 + lane * 4) = mtrue[nb];
  }
  __syncthreads();
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    float ms[4], ls[4];
    float M = -INFINITY;
#pragma unroll
    for (int src = 0; src < 4; ++src) {
      ms[src] = *reinterpret_cast<const float*>(mlb + ((src * 2 + 0) * NQB + nb) * 256 + lane * 4);
      ls[src] = *reinterpret_cast<const float*>(mlb + ((src * 2 + 1) * NQB + nb) * 256 + lane * 4);
      M = fmaxf(M, ms[src]);
    }
    float L = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) ofold[nb][r] = 0.f;
#pragma unroll
    for (int src = 0; src < 4; ++src) {
      const float sc = (ms[src] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ms[src] - M);
      L += ls[src] * sc;
      if (src == w) {
        // the block this wave kept in registers (static register index per candidate w)
#pragma unroll
        for (int db = 0; db < 4; ++db)
          if (db == w) {
#pragma unroll
            for (int r = 0; r < 16; ++r) ofold[nb][r] += oacc[db][nb][r] * sc;
          }
      } else {
        const char* base = smem + (src * 4 + w) * kBlk + lane * 16;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4_t v = *reinterpret_cast<const float4_t*>(base + (nb * 4 + j) * 1024);
#pragma unroll
          for (int i = 0; i < 4; ++i) ofold[nb][4 * j + i] += v[i] * sc;
        }
      }
    }
    // report the true maximum, with the denominator re-expressed relative to it
    float mt = mtrue[nb];
#pragma unroll
    for (int src = 0; src < 4; ++src)
      mt = fmaxf(mt, *reinterpret_cast<const float*>(mlb + ((8 + src) * NQB + nb) * 256 + lane * 4));
    const float Lall = L + __shfl_xor(L, 32, kWave);
    const float toTrue = (mt == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(M - mt);
    mfin[nb] = mt;
    lfin[nb] = Lall * toTrue;
#pragma unroll
    for (int r = 0; r < 16; ++r) ofold[nb][r] *= toTrue;
  }
}

template <int NQB>
constexpr int tile_lds_bytes() {
  constexpr int fold = 16 * NQB * 16 * 256 + 4 * 3 * NQB * 256;  // parked blocks + (m, l, true max) of four waves
  return 4 * kWaveLds > fold ? 4 * kWaveLds : fold;
}

// Shared-prefix phase: workgroup = (split, head, group x query tile); writes one (O, m, l) part.
template <typename E, int NQB>
__global__ __launch_bounds__(256, 1) void prefix_mfma_kernel(PrefixArgs a, int mtiles) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int split = blockIdx.x, head = blockIdx.y;
  const int g = blockIdx.z / mtiles, mt = blockIdx.z - g * mtiles;
  int r0 = 0, r1 = a.B, poff = 0, plen = a.fixed_prefix_len;
  if (a.prefix_cu) {
    r0 = a.group_req_cu[g];
    r1 = a.group_req_cu[g + 1];
    poff = a.prefix_cu[g];
    plen = a.prefix_cu[g + 1] - poff;
  }
  const int qbase = r0 + mt * 32 * NQB;
  const int nq = min(32 * NQB, r1 - qbase);
  if (nq <= 0) return;
  const int s0 = split * a.split_tokens;
  const int s1 = min(plen, s0 + a.split_tokens);
  if (s0 >= plen) {  // this group's prefix ends before the split: mark the part empty
    for (int q = threadIdx.x; q < nq; q += 256) {
      const int64_t pr = ((int64_t)split * a.B + qbase + q) * a.H + head;
      a.ml[pr * 2] = -INFINITY;
      a.ml[pr * 2 + 1] = 0.f;
    }
    return;
  }
  TileWork wk;
  wk.qrow0 = a.q + (int64_t)qbase * a.q_stride + head * kPD;
  wk.q_stride = a.q_stride;
  wk.nq = nq;
  wk.slots = a.slots + poff;
  wk.s0 = s0;
  wk.s1 = s1;
  wk.causal_off = 0;
  float16_t of[NQB];
  float m[NQB], l[NQB];
  attn_tile<E, NQB, false>(wk, a.kc, a.vc, a.row_stride, head, a.scale_log2e, smem, of, m, l);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, h = lane >> 5, ql = lane & 31;
#pragma unroll
  for (int nb = 0; nb < NQB; ++nb) {
    const int q = 32 * nb + ql;
    if (q < nq) {
      const float inv = 1.f / l[nb];
      const int64_t pr = ((int64_t)split * a.B + qbase + q) * a.H + head;
      float* op = a.opart + pr * kPD + 32 * w + 4 * h;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float4_t v = {of[nb][4 * j] * inv, of[nb][4 * j + 1] * inv, of[nb][4 * j + 2] * inv, of[nb][4 * j + 3] * inv};
        *reinterpret_cast<float4_t*>(op + 8 * j) = v;
      }
      if (h == 0 && w == 0) {
        a.ml[pr * 2] = m[nb];
        a.ml[pr * 2 + 1] = l[nb];
      }
    }
  }
}

// Prefill with parent context: workgroup = (head, 64-query tile of one chunk), all of the tile's
// visible keys (ancestors, then the chunk's own tokens up to the diagonal); writes the final rows.
// blockIdx.x is the head so that the query tiles of one (chunk, head), which stream the same K/V,
// land on the same XCD (workgroups go round-robin over the 8 XCDs in linear order) and share its L2.
template <typename E>
__global__ __launch_bounds__(256, 1) void prefill_mfma_kernel(PrefillArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int head = blockIdx.x;
  const int ti = blockIdx.y;
  if (head >= a.H) return;
  if (ti >= a.tile_cu[a.num_chunks]) return;
  int lo = 0, hi = a.num_chunks;  // chunk with tile_cu[c] <= ti < tile_cu[c+1]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.tile_cu[mid] <= ti) lo = mid; else hi = mid;
  }
  const int cq0 = a.q_cu[lo], n = a.q_cu[lo + 1] - cq0;
  const int kv0 = a.kv_cu[lo], kvn = a.kv_cu[lo + 1] - kv0;
  const int q0 = (ti - a.tile_cu[lo]) * 64;
  const int nq = min(64, n - q0);
  TileWork wk;
  wk.qrow0 = a.q + (int64_t)(cq0 + q0) * a.q_stride + head * kPD;
  wk.q_stride = a.q_stride;
  wk.nq = nq;
  wk.slots = a.ctx_slots + kv0;
  wk.s0 = 0;
  wk.causal_off = kvn - n + q0;
  wk.s1 = min(kvn, wk.causal_off + nq);  // the last live query sees tokens up to causal_off + nq - 1
  float16_t of[2];
  float m[2], l[2];
  attn_tile<E, 2, true>(wk, a.kc, a.vc, a.row_stride, head, a.scale_log2e, smem, of, m, l);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, h = lane >> 5, ql = lane & 31;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int q = 32 * nb + ql;
    if (q < nq) {
      const float inv = l[nb] > 0.f ? 1.f / l[nb] : 0.f;
      uint16_t* op = a.out + (int64_t)(cq0 + q0 + q) * a.out_stride + head * kPD + 32 * w + 4 * h;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x2 v = {pack2<E>(of[nb][4 * j] * inv, of[nb][4 * j + 1] * inv),
                   pack2<E>(of[nb][4 * j + 2] * inv, of[nb][4 * j + 3] * inv)};
        *reinterpret_cast<u32x2*>(op + 8 * j) = v;
      }
    }
  }
}

// tile_cu[c] = number of 64-query tiles before chunk c (serial scan; chunk counts are small)
__global__ void prefill_tiles_kernel(const int32_t* q_cu, int num_chunks, int32_t* tile_cu) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int acc = 0;
  for (int c = 0; c < num_chunks; ++c) {
    tile_cu[c] = acc;
    acc += (q_cu[c + 1] - q_cu[c] + 63) / 64;
  }
  tile_cu[num_chunks] = acc;
}

template <typename E>
static int launch_prefix_t(const PrefixArgs& a, int num_groups, int max_group_reqs, hipStream_t st) {
  const int nqb = max_group_reqs <= 32 ? 1 : 2;
  const int mtiles = (max_group_reqs + 32 * nqb - 1) / (32 * nqb);
  dim3 grid(a.n_splits, a.H, num_groups * mtiles), block(256);
  const KernelEvents ev = take_kernel_events(0);
  if (nqb == 1) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&prefix_mfma_kernel<E, 1>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, tile_lds_bytes<1>());
    hipExtLaunchKernelGGL((prefix_mfma_kernel<E, 1>), grid, block, tile_lds_bytes<1>(), st, ev.start, ev.stop, 0, a, mtiles);
  } else {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&prefix_mfma_kernel<E, 2>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, tile_lds_bytes<2>());
    hipExtLaunchKernelGGL((prefix_mfma_kernel<E, 2>), grid, block, tile_lds_bytes<2>(), st, ev.start, ev.stop, 0, a, mtiles);
  }
  return launch_status();
}

template <typename E>
static int launch_prefill_t(const PrefillArgs& a, int max_tiles, hipStream_t st) {
  hipLaunchKernelGGL(prefill_tiles_kernel, dim3(1), dim3(64), 0, st, a.q_cu, a.num_chunks, a.tile_cu);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_mfma_kernel<E>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, tile_lds_bytes<2>());
  const int hx = (a.H + 7) / 8 * 8;  // keeps head == linear id mod 8 for every tile row
  hipLaunchKernelGGL((prefill_mfma_kernel<E>), dim3(hx, max_tiles), dim3(256), tile_lds_bytes<2>(), st, a);
  return launch_status();
}

bool prefix_mfma_supported(int dtype, int D) { return D == kPD && (dtype == PH_F16 || dtype == PH_BF16); }

int launch_prefix_mfma(const PrefixArgs& a, int dtype, int D, int num_groups, int max_group_reqs, hipStream_t st) {
  if (D != kPD) return PH_ERR_HEAD_DIM;
  if (num_groups <= 0 || max_group_reqs <= 0 || a.n_splits <= 0) return PH_OK;
  return dtype == PH_F16 ? launch_prefix_t<F16>(a, num_groups, max_group_reqs, st)
                         : launch_prefix_t<BF16>(a, num_groups, max_group_reqs, st);
}

int launch_prefill_mfma(const PrefillArgs& a, int dtype, int D, int max_tiles, hipStream_t st) {
  if (D != kPD) return PH_ERR_HEAD_DIM;
  if (max_tiles <= 0) return PH_OK;
  return dtype == PH_F16 ? launch_prefill_t<F16>(a, max_tiles, st) : launch_prefill_t<BF16>(a, max_tiles, st);
}

}  // namespace ph
