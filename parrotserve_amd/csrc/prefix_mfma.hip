// Shared-prefix flash-decoding and prefill with parent context on CDNA4 matrix cores.
//
// All queries of a group attend over the SAME prefix slots (decode), and all query rows of a prefill
// chunk over the same parent + own slots, so per head the work is a dense contraction:
// S^T = K Q^T (tokens x queries), O^T = V^T P^T, online softmax in the exp2 domain between them, fp32
// accumulation in v_mfma_f32_32x32x16_{f16,bf16}.  K/V rows are gathered by slot straight from global
// memory into XOR-swizzled LDS tiles (the load writes LDS itself, no register staging) and read back in
// matrix-operand layout, so each K/V byte crosses LDS once.  Two forms of the tile loop:
//   * four waves, one 32-query block (groups of up to 32 requests): every wave owns every fourth
//     32-token tile in a private double-buffered LDS region, no workgroup barrier in the loop;
//   * eight waves (two per SIMD), 64 to 256 queries per workgroup: the waves of a token group share each
//     K/V tile through a ring of LDS stages, one barrier per step (attn_tile8 below).
// Partials of the waves that split the tokens are folded through LDS at the end.
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
#include "stream_item.hpp"

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
// NT: non-temporal (streaming) cache policy for rows that are read once per launch.
template <bool NT = false>
__device__ __forceinline__ void lds_dma16(const void* gptr, uint32_t lds_addr) {
  if (NT)
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(gptr), "s"(lds_addr) : "memory");
  else
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(lds_addr) : "memory");
}
// 4 bytes per lane the same way: used only to pull cache lines towards L2 ahead of the row loads (the data
// lands in an LDS area nobody reads, so no register waits for it)
__device__ __forceinline__ void lds_dma4(const void* gptr, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr), "s"(lds_addr) : "memory");
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
  int slots_len;          // entries of the list (reads beyond [s0, s1) are clamped to it)
  int s0, s1;             // token range of this workgroup
  int causal_off;         // CAUSAL: query i sees token t iff t <= causal_off + i
  // 64-wide heads as halves of 128-wide head pairs (the query's other half is zero):
  //   0 / 1: every row of the tile is that half, qrow0 points at the half's 64 values;
  //   2: rows alternate, row q = request q >> 1 (rows of q_stride from qrow0, the pair's first value), half q & 1
  int pair_half = -1;
  // Head sizes 80, 96 and 112 on the 128-wide tile: a head's row in the pools and in q is head_dim elements long;
  // the lanes that would load the chunks beyond it load the row's first chunk instead (valid memory, finite
  // values), the query's dims beyond it are zero (so those K values never reach a score) and the output's are not
  // written.  HBM traffic stays that of the real rows; LDS and the matrix pipe carry the padding.
  int head_dim = 128;
  // grouped KV heads: row q of the tile is request q >> gshift, member q & (G - 1) of the G = 1 << gshift query
  // heads that share this KV head; qrow0 points at the group's first query head of the tile's first request
  int gshift = 0;
  // decode form: shares at most two steps longer than the ring touch the lines beyond it during their first two
  // steps.  Off for the prefix-only workgroups of the fused launch: next to a suffix stream that saturates the
  // memory system the touches (at any distance, at every step) made the steps slower, not faster (cold K/V:
  // 70 us against 63 us per launch at config 2 with 64 prefix workgroups)
  bool touch_ahead = true;
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
      lds_dma16<!CAUSAL>(kbase[r] + ro, kb + r * 1024);
      lds_dma16<!CAUSAL>(vbase_g + ro, kb + kVtOff + r * 1024);
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
    r0 = a.group_req_cu[g] << a.req_shift;
    r1 = a.group_req_cu[g + 1] << a.req_shift;
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
  wk.slots_len = plen;
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

// ---------------------------------------------------------------------------------------------------------
// Eight-wave form of the tile.  The workgroup's eight waves are TQ token groups x QB = 8 / TQ query blocks:
// wave (g, qb) works on every TQ-th 32-token tile (those with index = g mod TQ) for queries 32 qb .. 32 qb + 31,
// so a workgroup covers 32 QB queries.  The QB waves of a token group share each K/V tile: every wave stages
// 16 / QB of the tile's sixteen 1 KB row groups into the group's ring of 8 / TQ LDS stages (7, 3 or 1 tiles
// in flight ahead of the one being multiplied), and one workgroup barrier per step publishes the parts to
// each other (all waves run the same trip count).  Two waves per SIMD: one wave's softmax arithmetic overlaps
// the other's matrix instructions, and at 256 registers per lane every matrix operand and result stays in
// ordinary vector registers.  Slot ids come from a 4096-token window of the slot list kept in LDS (refilled
// by the whole workgroup when the staging front crosses it), so the only vector-memory operations in the
// loop are the LDS-direct row loads and their completion can be counted exactly.
// On return wave (g, qb) holds 4 / TQ blocks of 32 dims, [32 (4/TQ) g, +32 (4/TQ)), of its queries, folded
// over the token groups (register 4j+i of block n = dim 32 ((4/TQ) g + n) + 8j + 4h + i of query 32 qb + ql).
constexpr int kWin = 4096;                        // tokens per slot window
constexpr int kWinOff = 8 * kStage;               // LDS offset of the window (behind the 128 KB of stages)
constexpr int kMlOff = kWinOff + kWin * 4;        // (m, l, true max) of eight waves for the fold
constexpr int kPfOff = kMlOff + 8 * 3 * 256;    // landing area of the cache-line touches (256 bytes per wave)
constexpr int kTile8Lds = kPfOff + 8 * 256;

// max over the two 32-lane halves of the wave: lane l gets max(x[l], x[l ^ 32]).  One lane-swap instruction
// (lanes 32..63 of the first register trade places with lanes 0..31 of the second) instead of a trip
// through LDS; written as assembly because the builtin's second result is mis-compiled by this toolchain.
__device__ __forceinline__ float half_swap_max(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
}

// LDS reads by byte address (the ring's stage offset then folds into the instruction's immediate)
__device__ __forceinline__ u32x4 lds_ld16_a(uint32_t addr) {
  return *reinterpret_cast<const u32x4 __attribute__((address_space(3)))*>((uintptr_t)addr);
}
__device__ __forceinline__ u32x2 lds_tr16_a(uint32_t addr) {
  const short4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      reinterpret_cast<short4_t __attribute__((address_space(3)))*>((uintptr_t)addr));
  return __builtin_bit_cast(u32x2, v);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {  // vmcnt <= N, other counters untouched (gfx9 encoding)
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// `mid` is called once by every wave between the prologue (slot window filled, first tiles in flight into
// LDS, Q loaded) and the main loop: work placed there runs while the first tiles land, and must leave LDS
// alone.  The default does nothing.
struct NoMid {
  __device__ __forceinline__ void operator()() const {}
};

template <typename E, bool CAUSAL, int TQ, typename Mid = NoMid, int SUB = 1, bool HALF = false, bool PRESC = false>
__device__ __forceinline__ void attn_tile8(const TileWork& wk, const uint16_t* __restrict__ kc,
                                           const uint16_t* __restrict__ vc, int64_t row_stride, int head,
                                           float scale_log2e, char* smem, float16_t (&ofold)[4 / TQ], float& mfin,
                                           float& lfin, Mid mid = Mid()) {
  // SUB: 32-token sub-tiles per step of a token group (a ring stage holds SUB of them back to back).  Two
  // halve the per-step costs (barrier, waits, staging bookkeeping, one softmax bookkeeping per 64 tokens) and
  // give the scheduler two independent score products to overlap with the vector work.
  constexpr int QB = 8 / TQ;            // query blocks = waves sharing a tile
  constexpr int STEP = kTile * SUB;     // tokens per step
  constexpr int SBYTES = kStage * SUB;  // bytes per ring stage
  constexpr int NST = 8 / (TQ * SUB);   // stages per token group
  constexpr int A = NST - 1;            // steps in flight ahead of the current one
  constexpr int LPT = 16 * SUB / QB;    // row-group loads per wave per step
  static_assert(NST >= 2 && LPT >= 1 && LPT <= 8, "unsupported tile split");
  constexpr int NDB = 4 / TQ;     // dim blocks a wave finishes
  // decode reads every prefix row once per launch (streaming policy); prefill tiles, and the tiles of a decode
  // group of more than 256 requests (the 256-query form), are re-read by the other query tiles and should stay
  // in L2 (batch 1024 over 8192 tokens: 158 -> 144 us)
  constexpr bool NTLOAD = !CAUSAL && TQ > 1;
  // Decode: the LDS ring holds one step beyond the one being multiplied, which is too little to cover the
  // memory latency (the ring cannot grow: it is all of LDS).  When the workgroup's share is at most two steps
  // longer than the ring, every thread also touches one 128-byte line of the step after the one being staged
  // (128 tokens x K and V x 2 lines = 512 lines) with a 4-byte load during the first two steps: the rows of
  // the steps beyond the ring are then on their way to L2 a whole step before the ring has room for them, and
  // the row loads that follow find them there.  Issued behind the step's row loads, so their completion is
  // still counted exactly (one younger load per step).  Longer shares run in a bandwidth-bound steady state
  // where the extra requests cost more than the earlier start gains (measured on cold K/V: 2 % slower with
  // them at 11 steps per workgroup, 1 % faster at 4), so they go without.
  constexpr bool PREFETCH = !CAUSAL && A == 1 && STEP * TQ == 128;
  constexpr int kPfSteps = 2;
  constexpr float kSlack = 8.f;
  // HALF: a 64-wide head as half wk.pair_half (0 / 1) of a head pair -- only that half's two 32-dim blocks of the
  // output are wanted, so only they are multiplied (accumulators 0 and 1 stand for blocks 2 half, 2 half + 1)
  static_assert(!HALF || TQ == 1, "the half-output form has no fold across token groups");
  constexpr int NDBV = HALF ? 2 : 4;
  float16_t oacc[4];
  float m = -INFINITY, lsum = 0.f, mtrue = -INFINITY;
  const int lane = threadIdx.x & 63;
  const int w8 = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), g = w8 / QB, qb = w8 % QB;
  const int h = lane >> 5, ql = lane & 31;
  char* gl = smem + g * NST * SBYTES;
  int32_t* win = reinterpret_cast<int32_t*>(smem + kWinOff);
  const int s0 = wk.s0, s1 = wk.s1;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;

  // slot window [win0, win0 + kWin) of the list, clamped to the list's end
  int win0 = s0;
  auto fill_window = [&]() {
    for (int i = threadIdx.x; i < kWin; i += 512) win[i] = wk.slots[min(win0 + i, wk.slots_len - 1)];
  };
  fill_window();

  // staging: row group L (0..7 K, 8..15 V) covers tokens 4 (L & 7) .. +3, 16 lanes per token row; this wave
  // brings row groups qb LPT .. + LPT - 1 (same swizzles as the four-wave form)
  const int tl = lane >> 4, c = lane & 15;
  const uint32_t row_bytes = (uint32_t)(row_stride * 2);
  const int sub0 = (qb * LPT) / 16;            // sub-tile, K or V half and first row group of this wave's loads
  const bool isv = ((qb * LPT) & 15) >= 8;
  const int r0 = (qb * LPT) & 7;
  const char* gbase[LPT];
#pragma unroll
  for (int i = 0; i < LPT; ++i)
  {
    const int cg = isv ? (c ^ (4 * tl)) : (c ^ ((4 * (r0 + i) + tl) & 15));  // the 16-byte chunk of the row this lane loads
    const int cl = cg * 8 < wk.head_dim ? cg : 0;                            // chunks beyond a short head: its first chunk
    gbase[i] = reinterpret_cast<const char*>((isv ? vc : kc) + (int64_t)head * wk.head_dim + cl * 8);
  }
  const uint32_t dst0 = lds_addr_of(gl) + sub0 * kStage + (isv ? kVtOff : 0) + r0 * 1024;
  const uint32_t pf_lds = lds_addr_of(smem + kPfOff) + w8 * 256;
  const int pf_steps =
      (PREFETCH && wk.touch_ahead && (s1 - s0 + STEP * TQ - 1) / (STEP * TQ) <= NST + kPfSteps) ? kPfSteps : 0;
  // rows of the group's tile that starts at token tb, into ring stage `stage`
  auto fetch_rows = [&](int tb, int stage) {
    uint32_t sl[LPT];
#pragma unroll
    for (int i = 0; i < LPT; ++i) sl[i] = (uint32_t)win[tb - win0 + kTile * sub0 + 4 * (r0 + i) + tl];
    const uint32_t kb = dst0 + stage * SBYTES;
#pragma unroll
    for (int i = 0; i < LPT; ++i) lds_dma16<NTLOAD>(gbase[i] + (uint64_t)sl[i] * row_bytes, kb + i * 1024);
  };
  const int ntile = (s1 - s0 + STEP - 1) / STEP;
  const int iters = (ntile + TQ - 1) / TQ;                 // same for all eight waves
  const int my_iters = ntile > g ? (ntile - g + TQ - 1) / TQ : 0;  // tiles of this token group
  __syncthreads();                                         // window visible
  PH_TL(1);
  // the whole ring is filled up front: tiles 0 .. A (the main loop issues tile it + A at step it >= 1)
#pragma unroll
  for (int j = 0; j < NST; ++j)
    if (j < my_iters) fetch_rows(s0 + STEP * (g + TQ * j), j);

  // Q as the B operand: column = query 32 qb + ql, contraction chunk (h, s) = dims 64h + 8s .. +8
  u32x4 qop[8];
  {
    const int q = 32 * qb + ql;
    const bool ok = q < wk.nq;
    const uint16_t* qp = wk.qrow0 + (int64_t)(ok ? q : 0) * wk.q_stride + 64 * h;
    // a 64-wide head as one half of a head pair: the other half of the query is zero, which cancels the
    // neighbouring head's keys in the score (the row pointer already points at this half's 64 values)
    int half = wk.pair_half;
    if (wk.pair_half == 2) {  // rows alternate between the two heads of the pair: row q = request q >> 1, half q & 1
      half = q & 1;
      qp = wk.qrow0 + (int64_t)(ok ? q >> 1 : 0) * wk.q_stride + 64 * half;
    } else if (wk.pair_half >= 0) {
      qp = wk.qrow0 + (int64_t)(ok ? q : 0) * wk.q_stride;
    }
    if (wk.gshift > 0)
      qp = wk.qrow0 + (int64_t)(ok ? q >> wk.gshift : 0) * wk.q_stride + (q & ((1 << wk.gshift) - 1)) * kPD + 64 * h;
    const bool mine = wk.pair_half < 0 || h == half;
    const bool padded = wk.head_dim < kPD;  // (never together with head pairs or grouped rows)
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const bool in = !padded || 64 * h + 8 * s < wk.head_dim;  // dims beyond a short head: read its first dims, use zero
      u32x4 v = ld16(in ? qp + 8 * s : qp - 64 * h);
      if (!ok || !mine || !in) v = u32x4{0, 0, 0, 0};
      if (PRESC) {
        // PRESC: q takes the factor scale * log2(e) here and is rounded to the element type again (what the
        // reference's own prefix kernel does, shared_flash_decoding.py:100), and the exponent reference enters
        // the score product as its initial accumulator: the product is the exponent's argument as it stands
#pragma unroll
        for (int j = 0; j < 4; ++j)
          v[j] = pack2<E>(Elem<E>::lo(v[j]) * scale_log2e, Elem<E>::hi(v[j]) * scale_log2e);
      }
      qop[s] = v;
    }
  }
  // PRESC: minus the exponent reference (0 while there is none) in all sixteen accumulator registers
  float16_t cinit = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // last token any query of this wave's block may see (none if the block has no live query)
  const int wave_last = 32 * qb >= wk.nq ? -1 : CAUSAL ? min(s1 - 1, wk.causal_off + 32 * qb + 31) : s1 - 1;

  PH_TL(2);
  mid();
  PH_TL(3);

  // Operand read addresses of ring stage 0 (and of stage 4, beyond the reach of the 16-bit immediate).
  // K: row ql, chunk (8h + s) swizzled by the row; V: the transposing read's row/column of this lane.
  constexpr int NHI = NST * SBYTES > 65536 ? 2 : 1;
  uint32_t kaddr[NHI][8], vaddr[NHI][4];
  {
    const uint32_t gl_a = lds_addr_of(gl);
    const int sl = lane & 15, rh = (lane >> 4) & 1;
    const int trow = 4 * h + (sl >> 2);                       // + 16u + 8x
    const int tcol = 2 * rh + ((sl & 3) >> 1);                // + 4db, in 16-byte chunks
    const int tswz = 4 * (sl >> 2);                           // = 4 * (row & 3)
#pragma unroll
    for (int hi = 0; hi < NHI; ++hi) {
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        kaddr[hi][s] = gl_a + hi * 65536 + ql * 256 + (((8 * h + s) ^ (ql & 15)) * 16);
        asm("" : "+v"(kaddr[hi][s]));  // keep the sum in one register (otherwise it is re-added at every read)
      }
#pragma unroll
      for (int db = 0; db < NDBV; ++db) {
        const int dbr = HALF ? 2 * wk.pair_half + db : db;  // 32-dim block of the 128-wide row
        vaddr[hi][db] = gl_a + hi * 65536 + kVtOff + trow * 256 + (sl & 1) * 8 + (((4 * dbr + tcol) ^ tswz) * 16);
        asm("" : "+v"(vaddr[hi][db]));
      }
    }
  }
  // the ring position is a compile-time constant in the unrolled inner loop, so every LDS address of a
  // step is a fixed register plus an immediate offset
  for (int it0 = 0; it0 < iters; it0 += NST) {
#pragma unroll
   for (int stage = 0; stage < NST; ++stage) {
    const int it = it0 + stage;
    if (it >= iters) break;
    const int tb = s0 + STEP * (g + TQ * it);
    // Tile `it` of this group has landed once at most the (A - 1) LPT loads issued after it are outstanding
    // (near the end fewer were issued, so everything is awaited); the barrier publishes all parts of the
    // tile and tells everyone that the stage read in the previous step is free again.
    if (it + A - 1 >= my_iters) {
      wait_vmcnt<0>();
    } else if (PREFETCH && pf_steps > 0 && it >= 1 && it <= pf_steps) {
      wait_vmcnt<(A - 1) * LPT + 1>();  // the line touches issued behind the last row loads may still be out
    } else {
      wait_vmcnt<(A - 1) * LPT>();
    }
    __syncthreads();
    if (it < 4) PH_TL(4 + it);
    {
      const int front = s0 + STEP * TQ * (it + A);           // first token of the step being staged
      if (front < s1 && front >= win0 + kWin) {              // workgroup-uniform: slide the slot window
        win0 += kWin;
        fill_window();
        __syncthreads();
      }
      if (it > 0 && it + A < my_iters) fetch_rows(front + STEP * g, (stage + A) % NST);
      if (PREFETCH && it < pf_steps) {
        // token (of all four groups) and line of the step after `front`, clamped into the list and the window
        const int pt = min(min(front + STEP * TQ + (int)(threadIdx.x >> 2), s1 - 1), win0 + kWin - 1);
        const uint32_t slot = (uint32_t)win[pt - win0];
        const char* base = reinterpret_cast<const char*>((threadIdx.x & 2) ? vc : kc) +
                           (int64_t)head * (wk.head_dim * 2) + (threadIdx.x & 1) * 128;
        lds_dma4(base + (uint64_t)slot * row_bytes, pf_lds);
      }
    }
    if (it >= my_iters || tb > wave_last) continue;           // wave-uniform
    float16_t sacc[SUB];
#pragma unroll
    for (int sb = 0; sb < SUB; ++sb) {
      const int off = stage * SBYTES + sb * kStage;
      const int shi = off >> 16, slo = off & 65535;
      u32x4 ka[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) ka[s] = lds_ld16_a(kaddr[shi][s] + slo);
      if (SUB == 1) __builtin_amdgcn_sched_barrier(0);
      const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      sacc[sb] = Mfma32<E>::run(ka[0], qop[0], PRESC ? cinit : zero);
#pragma unroll
      for (int s = 1; s < 8; ++s) sacc[sb] = Mfma32<E>::run(ka[s], qop[s], sacc[sb]);
    }
    // A operand of O^T += V^T P^T (row = dim 32db + ql, contraction = the 8 tokens of (h, u)): two
    // transposing reads, tokens 16u + 4h + {0..3} and 16u + 8 + 4h + {0..3}
    u32x4 va[SUB][4][2];
#pragma unroll
    for (int sb = 0; sb < SUB; ++sb) {
      const int off = stage * SBYTES + sb * kStage;
      const int shi = off >> 16, slo = off & 65535;
#pragma unroll
      for (int db = 0; db < NDBV; ++db)
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const u32x2 lo = lds_tr16_a(vaddr[shi][db] + slo + (16 * u) * 256);
          const u32x2 hi = lds_tr16_a(vaddr[shi][db] + slo + (16 * u + 8) * 256);
          va[sb][db][u] = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    }
    if (SUB == 1) __builtin_amdgcn_sched_barrier(0);

    const bool full = tb + STEP <= s1 && (!CAUSAL || tb + STEP - 1 <= wk.causal_off + 32 * qb);
    float x[SUB][16];
    if (full) {
#pragma unroll
      for (int sb = 0; sb < SUB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[sb][r] = sacc[sb][r];
    } else {
      const int tmax = CAUSAL ? min(s1 - 1, wk.causal_off + 32 * qb + ql) : s1 - 1;  // last visible token
#pragma unroll
      for (int sb = 0; sb < SUB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int t = kTile * sb + 8 * (r >> 2) + 4 * h + (r & 3);
          x[sb][r] = (tb + t <= tmax) ? sacc[sb][r] : -INFINITY;
        }
    }
    float mloc = -INFINITY;
#pragma unroll
    for (int sb = 0; sb < SUB; ++sb)
#pragma unroll
      for (int r = 0; r < 16; r += 4)
        mloc = fmaxf(mloc, fmaxf(fmaxf(x[sb][r], x[sb][r + 1]), fmaxf(x[sb][r + 2], x[sb][r + 3])));
    const bool had = m != -INFINITY;
    if (PRESC) mloc = half_swap_max(mloc) + (had ? m : 0.f);  // the scores are relative to the reference so far
    else mloc = half_swap_max(mloc) * scale_log2e;              // scale > 0 keeps the order
    mtrue = fmaxf(mtrue, mloc);
    // lazy exponent reference: moves only when the maximum has outgrown it by more than kSlack
    const bool move = mloc > m + kSlack;
    const float mnew = move ? mloc : m;
    const float mref = (mnew == -INFINITY) ? 0.f : mnew;
    const float alpha = (move && had) ? __builtin_amdgcn_exp2f(m - mref) : 1.f;
    if (PRESC && __builtin_amdgcn_ballot_w64(move) != 0) {  // wave-uniform, rare: re-base the scores and the seed
      const float delta = mref - (had ? m : 0.f);            // 0 on the lanes whose reference stays
#pragma unroll
      for (int sb = 0; sb < SUB; ++sb)
#pragma unroll
        for (int r = 0; r < 16; ++r) x[sb][r] -= delta;
#pragma unroll
      for (int r = 0; r < 16; ++r) cinit[r] = -mref;
    }
    m = mnew;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // wave-uniform, rare
      // pinned in assembly so that the multiply stays inside this branch; wait states cover the matrix
      // results being read by the vector ALU and the rewritten registers feeding the next C operand
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
      for (int db = 0; db < NDBV; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(oacc[db][r]) : "v"(alpha));
      asm volatile("s_nop 7" ::: "memory");
    }
    // P^T packed straight into B-operand form; the denominator sums the rounded values the product uses
    float ps = 0.f;
#pragma unroll
    for (int sb = 0; sb < SUB; ++sb) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        x[sb][r] = PRESC ? __builtin_amdgcn_exp2f(x[sb][r])
                         : __builtin_amdgcn_exp2f(__builtin_fmaf(x[sb][r], scale_log2e, -mref));
      u32x4 pop[2];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pop[u][e] = pack2<E>(x[sb][8 * u + 2 * e], x[sb][8 * u + 2 * e + 1]);
          ps = Elem<E>::dot2(pop[u][e], Elem<E>::kOnes, ps);
        }
#pragma unroll
      for (int db = 0; db < NDBV; ++db)
#pragma unroll
        for (int u = 0; u < 2; ++u) oacc[db] = Mfma32<E>::run(va[sb][db][u], pop[u], oacc[db]);
    }
    lsum = lsum * alpha + ps;
   }
  }

  PH_TL(8);
  if constexpr (TQ == 1) {
    // one token group: nothing to fold across waves
    const float Lall = lsum + __shfl_xor(lsum, 32, kWave);
    const float toTrue = (mtrue == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - mtrue);
    mfin = mtrue;
    lfin = Lall * toTrue;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) ofold[db][r] = oacc[db][r] * toTrue;
  } else {
    // Fold the token groups of each query block: every wave parks the dim blocks it does not finish, and
    // its (m, l, true max); after one barrier wave (g, qb) folds blocks [NDB g, NDB g + NDB) of its block.
    constexpr int kBlk = 16 * 256;                  // one parked block: 16 floats x 64 lanes
    char* fb = smem + qb * (TQ * 4) * kBlk;         // [source group][dim block]
    char* mlb = smem + kMlOff + qb * TQ * 3 * 256;  // [group][m, l, true max][lane] floats
    __syncthreads();                                // the staging tiles are dead from here on
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      if (db / NDB == g) continue;
      char* base = fb + (g * 4 + db) * kBlk + lane * 16;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float4_t v = {oacc[db][4 * j], oacc[db][4 * j + 1], oacc[db][4 * j + 2], oacc[db][4 * j + 3]};
        *reinterpret_cast<float4_t*>(base + j * 1024) = v;
      }
    }
    *reinterpret_cast<float*>(mlb + (g * 3 + 0) * 256 + lane * 4) = m;
    *reinterpret_cast<float*>(mlb + (g * 3 + 1) * 256 + lane * 4) = lsum;
    *reinterpret_cast<float*>(mlb + (g * 3 + 2) * 256 + lane * 4) = mtrue;
    __syncthreads();
    float ms[TQ], ls[TQ];
    float M = -INFINITY, mt = -INFINITY;
#pragma unroll
    for (int src = 0; src < TQ; ++src) {
      ms[src] = *reinterpret_cast<const float*>(mlb + (src * 3 + 0) * 256 + lane * 4);
      ls[src] = *reinterpret_cast<const float*>(mlb + (src * 3 + 1) * 256 + lane * 4);
      mt = fmaxf(mt, *reinterpret_cast<const float*>(mlb + (src * 3 + 2) * 256 + lane * 4));
      M = fmaxf(M, ms[src]);
    }
    float L = 0.f;
#pragma unroll
    for (int n = 0; n < NDB; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) ofold[n][r] = 0.f;
#pragma unroll
    for (int src = 0; src < TQ; ++src) {
      const float sc = (ms[src] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ms[src] - M);
      L += ls[src] * sc;
#pragma unroll
      for (int n = 0; n < NDB; ++n) {
        if (src == g) {
          // the blocks this wave kept in registers (static register index per candidate g)
#pragma unroll
          for (int db = 0; db < 4; ++db)
            if (db == NDB * g + n) {
#pragma unroll
              for (int r = 0; r < 16; ++r) ofold[n][r] += oacc[db][r] * sc;
            }
        } else {
          const char* base = fb + (src * 4 + NDB * g + n) * kBlk + lane * 16;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float4_t v = *reinterpret_cast<const float4_t*>(base + j * 1024);
#pragma unroll
            for (int i = 0; i < 4; ++i) ofold[n][4 * j + i] += v[i] * sc;
          }
        }
      }
    }
    // report the true maximum, with the denominator re-expressed relative to it
    const float Lall = L + __shfl_xor(L, 32, kWave);
    const float toTrue = (mt == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(M - mt);
    mfin = mt;
    lfin = Lall * toTrue;
#pragma unroll
    for (int n = 0; n < NDB; ++n)
#pragma unroll
      for (int r = 0; r < 16; ++r) ofold[n][r] *= toTrue;
  }
}

// Shared-prefix phase, eight waves: one unit of work = (split, head, group x 64-query tile z), run by the
// whole workgroup; writes one (O, m, l) part per request of the tile.
// SUB, PRESC: the tile loop's step length and pre-scaled query (see attn_tile8).  PRESC moves a part's (m, l) by the
// rounding of the scaled query (up to 9e-3 in bf16), inside the tolerance of the merged output but not of an
// exported (m, l): only calls that export neither use it.
template <typename E, int TQ, typename Mid = NoMid, int SUB = 1, bool PRESC = false>
__device__ __forceinline__ void prefix_unit8(const PrefixArgs& a, int split, int head, int z, int mtiles, char* smem,
                                             Mid mid = Mid(), bool touch_ahead = true) {
  constexpr int QB = 8 / TQ, QT = 32 * QB, NDB = 4 / TQ;  // query blocks, queries per tile, dim blocks per wave
  const int g = z / mtiles, mt = z - g * mtiles;
  int r0 = 0, r1 = a.B, poff = 0, plen = a.fixed_prefix_len;
  if (a.prefix_cu) {
    r0 = a.group_req_cu[g] << a.req_shift;
    r1 = a.group_req_cu[g + 1] << a.req_shift;
    poff = a.prefix_cu[g];
    plen = a.prefix_cu[g + 1] - poff;
  }
  const int qbase = r0 + mt * QT;
  const int nq = min(QT, r1 - qbase);
  if (nq <= 0) {
    mid();
    return;
  }
  const int s0 = split * a.split_tokens;
  const int s1 = min(plen, s0 + a.split_tokens);
  if (s0 >= plen) {  // this group's prefix ends before the split: mark the part empty
    for (int q = threadIdx.x; q < nq; q += 512) {
      const int64_t pr = ((int64_t)split * a.B + qbase + q) * a.H + head;
      a.ml[pr * 2] = -INFINITY;
      a.ml[pr * 2 + 1] = 0.f;
    }
    mid();
    return;
  }
  TileWork wk;
  // req_shift > 0: B counts rows (1 << req_shift per request).  Head pairs: H counts pairs, q is the real
  // [B][2 H][64] tensor (a pair is 128 values wide).  Grouped KV heads: H counts KV heads, `head` is one, and its
  // G query heads lie side by side in the query row.
  const int hd = a.head_dim ? a.head_dim : kPD;  // 80 / 96 / 112: a short head on the 128-wide tile
  wk.qrow0 = a.q + (int64_t)(qbase >> a.req_shift) * a.q_stride + (a.gqa ? (head << a.req_shift) : head) * hd;
  wk.head_dim = hd;
  wk.pair_half = (a.req_shift && !a.gqa) ? 2 : -1;
  wk.gshift = a.gqa ? a.req_shift : 0;
  wk.q_stride = a.q_stride;
  wk.nq = nq;
  wk.slots = a.slots + poff;
  wk.slots_len = plen;
  wk.s0 = s0;
  wk.s1 = s1;
  wk.causal_off = 0;
  wk.touch_ahead = touch_ahead;
  float16_t of[NDB];
  float m, l;
  attn_tile8<E, false, TQ, Mid, SUB, false, PRESC>(wk, a.kc, a.vc, a.row_stride, head, a.scale_log2e, smem, of, m, l,
                                                   mid);
  PH_TL(9);
  const int lane = threadIdx.x & 63, w8 = threadIdx.x >> 6, tq = w8 / QB, qh = w8 % QB, h = lane >> 5, ql = lane & 31;
  const int q = 32 * qh + ql;
  if (q < nq) {
    const float inv = 1.f / l;
    const int64_t pr = ((int64_t)split * a.B + qbase + q) * a.H + head;
#pragma unroll
    for (int nd = 0; nd < NDB; ++nd) {
      const int d0 = 32 * (NDB * tq + nd) + 4 * h;
      float* op = a.opart + pr * hd + d0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float4_t v = {of[nd][4 * j] * inv, of[nd][4 * j + 1] * inv, of[nd][4 * j + 2] * inv, of[nd][4 * j + 3] * inv};
        if (d0 + 8 * j < hd) *reinterpret_cast<float4_t*>(op + 8 * j) = v;  // (a short head's row is hd floats long)
      }
    }
    if (h == 0 && tq == 0) {
      a.ml[pr * 2] = m;
      a.ml[pr * 2 + 1] = l;
    }
  }
}

template <typename E, int TQ, int SUB = 1, bool PRESC = false>
__global__ __launch_bounds__(512) void prefix_mfma8_kernel(PrefixArgs a, int mtiles) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  prefix_unit8<E, TQ, NoMid, SUB, PRESC>(a, blockIdx.x, blockIdx.y, blockIdx.z, mtiles, smem);
}

// The decode tile forms that are bound by the matrix pipe, not by memory (128- and 256-query tiles), take the step
// length and the pre-scaled query of the prefill loop where the call exports no (m, l).
template <int TQ>
struct WideTile {
  static constexpr int SUB = TQ == 1 ? 2 : 1;
  static constexpr bool PRESC = TQ <= 2;
};

// Prefix and suffix phases of one decode step in one launch, in one of two forms.
//
// Roles (np > 0): workgroups [0, np) are prefix-only -- workgroup b walks the prefix units b, b + np, ... back to
// back -- and workgroups [np, grid) are suffix-only: their eight waves take one (piece, head group) of the balanced
// form each, the pieces cut for 8 (grid - np) waves.  Whole compute units belong to the matrix product for the
// whole launch while the others stream, so neither phase waits for the other inside a workgroup and the memory
// system sees both from the first microseconds to the last.  Consecutive workgroup ids land on different XCDs, so
// both kinds spread evenly over the chip.
//
// Shared (np == 0): workgroup b owns the prefix units b, b + grid, ... (normally at most one) and its eight waves one
// suffix piece each.  Order inside a workgroup: suffix records requested, prefix prologue (slot window, first K/V
// tiles sent on their way into LDS, Q), then the suffix stream (it needs no LDS), then the prefix main loop on tiles
// that landed long ago, then the fold.  Taken when the suffix is too short to keep separate workgroups busy.
//
// The merge stays a separate launch: it needs every part.
// DS = head size of the suffix phase: 128, or 64 when the prefix phase runs on head pairs (pa.req_shift == 1).
// NQ > 1 (grouped KV heads, ia.nq): the suffix waves divide runs of NQ query heads that share a KV head and stream a
// row for the run at once.
template <typename E, int TQ, int DS = kPD, int NQ = 1>
__global__ __launch_bounds__(512) void decode_fused_kernel(PrefixArgs pa, int mtiles, int n_units, int np,
                                                           ItemArgs ia) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr int SUB = WideTile<TQ>::SUB;
  constexpr bool PRESC = WideTile<TQ>::PRESC;
  PH_TL(0);
  constexpr int HPW = HeadLanes<DS>::HPW;
  const int hgroups = (ia.H / NQ + HPW - 1) / HPW;
  const int slots = ia.num_lanes * hgroups;
  if (np > 0) {
    if ((int)blockIdx.x < np) {
      for (int u = blockIdx.x; u < n_units; u += np) {
        if (u != (int)blockIdx.x) __syncthreads();  // the fold scratch of the last unit is the staging ring of the next
        const int split = u % pa.n_splits;
        const int rest = u / pa.n_splits;
        prefix_unit8<E, TQ, NoMid, SUB, PRESC>(pa, split, rest % pa.H, rest / pa.H, mtiles, smem, NoMid(), false);
      }
    } else {
      const int stride = ((int)gridDim.x - np) * 8;
      const int wave = __builtin_amdgcn_readfirstlane(((int)blockIdx.x - np) * 8 + (int)(threadIdx.x >> 6));
      for (int s = wave; s < slots; s += stride) {
        const int piece = s / hgroups;
        run_piece<E, DS, 4, 2, NQ>(ia, piece, s - piece * hgroups);
      }
    }
    PH_TL(11);
    return;
  }
  const int wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 8 + (threadIdx.x >> 6));
  // this wave's first suffix piece: its record is requested before anything else
  const int piece0 = wave < slots ? wave / hgroups : -1;
  int4 rec0 = {0, 0, 0, 0}, rec1 = {0, 0, 0, 0};
  if (piece0 >= 0) {
    rec0 = ia.lane_rec[2 * piece0];
    rec1 = ia.lane_rec[2 * piece0 + 1];
  }
  auto suffix = [&]() {
    if (piece0 >= 0) run_piece_rec<E, DS, 4, 2, NQ>(ia, wave - piece0 * hgroups, rec0, rec1);
    for (int s = wave + gridDim.x * 8; s < slots; s += gridDim.x * 8) {
      const int piece = s / hgroups;
      run_piece<E, DS, 4, 2, NQ>(ia, piece, s - piece * hgroups);
    }
  };
  if ((int)blockIdx.x < n_units) {
    // the suffix stream runs between the first unit's prologue and its main loop
    const int u = blockIdx.x;
    const int split = u % pa.n_splits;
    const int rest = u / pa.n_splits;
    prefix_unit8<E, TQ, decltype(suffix), SUB, PRESC>(pa, split, rest % pa.H, rest / pa.H, mtiles, smem, suffix);
    for (int v = u + gridDim.x; v < n_units; v += gridDim.x) {
      __syncthreads();  // the fold scratch of the last unit is the staging ring of the next
      const int sp = v % pa.n_splits;
      const int rs = v / pa.n_splits;
      prefix_unit8<E, TQ, NoMid, SUB, PRESC>(pa, sp, rs % pa.H, rs / pa.H, mtiles, smem);
    }
  } else {
    suffix();
  }
  PH_TL(11);
}

// Prefill with parent context, eight waves: workgroup = (head, tile of 32 * (8 / TQ) queries of one chunk)
// HALF (64-wide heads, 256-query tiles): only this head's half of the pair's output is computed
template <typename E, int TQ, int SUB, bool HALF = false>
__device__ __forceinline__ void prefill_tile8(const PrefillArgs& a, int tile_row, char* smem) {
  constexpr int QB = 8 / TQ, NDB = 4 / TQ, QT = 32 * QB;
  // 64-wide heads: workgroup x is head x = half (x & 1) of pair x >> 1, whose K/V rows are one 128-wide row
  const int head = a.pair ? blockIdx.x >> 1 : blockIdx.x;
  const int half = a.pair ? (int)(blockIdx.x & 1) : -1;
  // later tiles of a chunk see more keys: hand them out first so the launch does not end on the longest ones
  const int ti = a.tile_cu[a.num_chunks] - 1 - tile_row;
  int lo = 0, hi = a.num_chunks;  // chunk with tile_cu[c] <= ti < tile_cu[c+1]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a.tile_cu[mid] <= ti) lo = mid; else hi = mid;
  }
  const int cq0 = a.q_cu[lo], n = a.q_cu[lo + 1] - cq0;
  const int kv0 = a.kv_cu[lo], kvn = a.kv_cu[lo + 1] - kv0;
  const int q0 = (ti - a.tile_cu[lo]) * QT;
  const int nq = min(QT, n - q0);
  TileWork wk;
  const int hd = a.head_dim ? a.head_dim : kPD;  // 80 / 96 / 112: a short head on the 128-wide tile
  wk.qrow0 = a.q + (int64_t)(cq0 + q0) * a.q_stride + (a.pair ? (int)blockIdx.x * 64 : head * hd);
  wk.head_dim = a.pair ? kPD : hd;
  wk.pair_half = half;
  wk.q_stride = a.q_stride;
  wk.nq = nq;
  wk.slots = a.ctx_slots + kv0;
  wk.slots_len = kvn;
  wk.s0 = 0;
  wk.causal_off = kvn - n + q0;
  wk.s1 = min(kvn, wk.causal_off + nq);  // the last live query sees tokens up to causal_off + nq - 1
  float16_t of[NDB];
  float m, l;
  // the prefill loop is bound by instruction issue: the pre-scaled query saves it one multiply-add per score
  attn_tile8<E, true, TQ, NoMid, SUB, HALF, true>(wk, a.kc, a.vc, a.row_stride, head, a.scale_log2e, smem, of, m, l);
  const int lane = threadIdx.x & 63, w8 = threadIdx.x >> 6, g = w8 / QB, qb = w8 % QB, h = lane >> 5, ql = lane & 31;
  const int q = 32 * qb + ql;
  if (q < nq) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int nd = 0; nd < NDB; ++nd) {
      if (HALF && nd >= 2) continue;                      // accumulators 0, 1 hold this half's two blocks
      const int db = HALF ? 2 * half + nd : NDB * g + nd;  // 32-dim block of the 128-wide row
      if (a.pair && (db >> 1) != half) continue;  // the other half holds the neighbouring head's values: dropped
      // paired: head 2 * pair + half, dims 32 * (db & 1) ..; else head, dims 32 * db ..
      uint16_t* op = a.out + (int64_t)(cq0 + q0 + q) * a.out_stride +
                     (a.pair ? (int)blockIdx.x * 64 + 32 * (db & 1) : head * hd + 32 * db) + 4 * h;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        u32x2 v = {pack2<E>(of[nd][4 * j] * inv, of[nd][4 * j + 1] * inv),
                   pack2<E>(of[nd][4 * j + 2] * inv, of[nd][4 * j + 3] * inv)};
        if (a.pair || 32 * db + 4 * h + 8 * j < hd) *reinterpret_cast<u32x2*>(op + 8 * j) = v;
      }
    }
  }
}

// Prefill with parent context, eight waves: workgroup = (head, tile of 32 * (8 / TQ) queries of one chunk); grid.y
// covers the tile rows from a.tile_row0 on (more rows than a grid's y extent holds take several launches; a loop
// over rows inside the kernel cost the common single-launch case 6 %)
// HALF (64-wide heads, 256-query tiles): only this head's half of the pair's output is computed
template <typename E, int TQ, int SUB, bool HALF = false>
__global__ __launch_bounds__(512) void prefill_mfma8_kernel(PrefillArgs a) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  PH_TL(0);
  if ((int)blockIdx.x >= a.H) return;
  const int row = a.tile_row0 + (int)blockIdx.y;
  if (row >= a.tile_cu[a.num_chunks]) return;
  prefill_tile8<E, TQ, SUB, HALF>(a, row, smem);
  PH_TL(11);
}

// tile_cu[c] = number of 64-query tiles before chunk c (serial scan; chunk counts are small)
__global__ void prefill_tiles_kernel(const int32_t* q_cu, int num_chunks, int32_t* tile_cu, int tile_q) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  int acc = 0;
  for (int c = 0; c < num_chunks; ++c) {
    tile_cu[c] = acc;
    acc += (q_cu[c + 1] - q_cu[c] + tile_q - 1) / tile_q;
  }
  tile_cu[num_chunks] = acc;
}

template <typename E, int TQ, int SUB = 1, bool PRESC = false>
static void launch_prefix8(const PrefixArgs& a, int num_groups, int max_group_reqs, hipStream_t st,
                           const KernelEvents& ev) {
  constexpr int QT = 32 * (8 / TQ);
  const int mtiles = (max_group_reqs + QT - 1) / QT;
  dim3 grid(a.n_splits, a.H, num_groups * mtiles), block(512);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&prefix_mfma8_kernel<E, TQ, SUB, PRESC>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kTile8Lds);
  PH_LAUNCH_TIMED((prefix_mfma8_kernel<E, TQ, SUB, PRESC>), grid, block, kTile8Lds, st, ev, a, mtiles);
}

// internal_ml: the parts' (m, l) stay inside the call (they only feed its merge)
template <typename E>
static int launch_prefix_t(const PrefixArgs& a, int num_groups, int max_group_reqs, bool internal_ml, hipStream_t st,
                           const KernelEvents& ev) {
  if (max_group_reqs <= 32 && a.req_shift == 0 && (a.head_dim == 0 || a.head_dim == kPD)) {  // four waves, one 32-query block
    dim3 grid(a.n_splits, a.H, num_groups), block(256);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&prefix_mfma_kernel<E, 1>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, tile_lds_bytes<1>());
    PH_LAUNCH_TIMED((prefix_mfma_kernel<E, 1>), grid, block, tile_lds_bytes<1>(), st, ev, a, 1);
  } else if (max_group_reqs <= 64) {   // eight waves, 64-query tiles
    launch_prefix8<E, 4>(a, num_groups, max_group_reqs, st, ev);
  } else if (max_group_reqs <= 128) {  // 128-query tiles: the prefix is read once for up to 128 requests
    if (internal_ml) launch_prefix8<E, 2, WideTile<2>::SUB, WideTile<2>::PRESC>(a, num_groups, max_group_reqs, st, ev);
    else launch_prefix8<E, 2, WideTile<2>::SUB, false>(a, num_groups, max_group_reqs, st, ev);
  } else {                             // 256-query tiles
    if (internal_ml) launch_prefix8<E, 1, WideTile<1>::SUB, WideTile<1>::PRESC>(a, num_groups, max_group_reqs, st, ev);
    else launch_prefix8<E, 1, WideTile<1>::SUB, false>(a, num_groups, max_group_reqs, st, ev);
  }
  return launch_status();
}

constexpr int64_t kMaxGridY = 65535;  // grid extent in y and z

template <typename E, int TQ, int SUB, bool HALF = false>
static int launch_prefill_tq(const PrefillArgs& a, int64_t num_tokens, hipStream_t st) {
  constexpr int QT = 32 * (8 / TQ);  // queries per workgroup tile
  hipLaunchKernelGGL(prefill_tiles_kernel, dim3(1), dim3(64), 0, st, a.q_cu, a.num_chunks, a.tile_cu, QT);
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_mfma8_kernel<E, TQ, SUB, HALF>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kTile8Lds);
  const int hx = (a.H + 7) / 8 * 8;  // keeps head == linear id mod 8 for every tile row
  const int64_t max_tiles = num_tokens / QT + a.num_chunks;  // >= sum of ceil(n_c / QT)
  for (int64_t row0 = 0; row0 < max_tiles; row0 += kMaxGridY) {
    PrefillArgs part = a;
    part.tile_row0 = (int)row0;
    const int64_t rows = max_tiles - row0 < kMaxGridY ? max_tiles - row0 : kMaxGridY;
    hipLaunchKernelGGL((prefill_mfma8_kernel<E, TQ, SUB, HALF>), dim3(hx, (unsigned)rows), dim3(512), kTile8Lds, st,
                       part);
  }
  return launch_status();
}

// Query tile by the average chunk length: 256-query tiles share every K/V tile among all eight waves (least
// traffic, deepest staging ring) but idle whole waves on short chunks, which take 128- or 64-query tiles.
template <typename E>
static int launch_prefill_t(const PrefillArgs& a, int64_t num_tokens, hipStream_t st) {
  const int64_t avg = num_tokens / (a.num_chunks > 0 ? a.num_chunks : 1);
  if (avg >= 192 && a.pair) return launch_prefill_tq<E, 1, 2, true>(a, num_tokens, st);
  if (avg >= 192) return launch_prefill_tq<E, 1, 2>(a, num_tokens, st);  // 64-token steps (measured 4 % faster)
  if (avg >= 96) return launch_prefill_tq<E, 2, 1>(a, num_tokens, st);
  return launch_prefill_tq<E, 4, 1>(a, num_tokens, st);
}

template <typename E, int TQ, int DS, int NQ = 1>
static int launch_fused_tq(const PrefixArgs& a, const ItemArgs& ia, int num_groups, int max_group_reqs, int cus,
                           int np, hipStream_t st, const KernelEvents& ev) {
  constexpr int QT = 32 * (8 / TQ);
  constexpr int HPW = HeadLanes<DS>::HPW;
  const int mtiles = (max_group_reqs + QT - 1) / QT;
  const int n_units = a.n_splits * a.H * num_groups * mtiles;
  const int hgroups = (ia.H / NQ + HPW - 1) / HPW;
  const int wave_slots = ia.num_lanes * hgroups;
  int grid;
  if (np > 0) {
    // roles: np prefix-only workgroups, then one round of suffix-only workgroups on the other compute units
    if (np > n_units) np = n_units;
    int swg = (wave_slots + 7) / 8;
    const int room = cus - np > 1 ? cus - np : 1;
    if (swg > room) swg = room;
    grid = np + swg;
  } else {
    grid = (wave_slots + 7) / 8;
    const int unit_grid = n_units < cus ? n_units : cus;
    if (grid < unit_grid) grid = unit_grid;
  }
  if (grid <= 0) return PH_OK;
  (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&decode_fused_kernel<E, TQ, DS, NQ>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kTile8Lds);
  PH_LAUNCH_TIMED((decode_fused_kernel<E, TQ, DS, NQ>), dim3(grid), dim3(512), kTile8Lds, st, ev, a, mtiles,
                        n_units, np, ia);
  return launch_status();
}

// query tile by the largest group: 64, 128 or 256 requests share each K/V tile of the prefix
template <typename E, int DS, int NQ = 1>
static int launch_fused_t(const PrefixArgs& a, const ItemArgs& ia, int num_groups, int max_group_reqs, int cus, int np,
                          hipStream_t st, const KernelEvents& ev) {
  if (max_group_reqs <= 64) return launch_fused_tq<E, 4, DS, NQ>(a, ia, num_groups, max_group_reqs, cus, np, st, ev);
  if (max_group_reqs <= 128) return launch_fused_tq<E, 2, DS, NQ>(a, ia, num_groups, max_group_reqs, cus, np, st, ev);
  return launch_fused_tq<E, 1, DS, NQ>(a, ia, num_groups, max_group_reqs, cus, np, st, ev);
}

template <typename E>
static int launch_fused_e(const PrefixArgs& a, const ItemArgs& ia, int num_groups, int max_group_reqs, int cus, int np,
                          hipStream_t st, const KernelEvents& ev) {
  if (a.req_shift && !a.gqa)  // 64-wide heads: the prefix phase on head pairs, the suffix phase at its own width
    return launch_fused_t<E, 64>(a, ia, num_groups, max_group_reqs, cus, np, st, ev);
  if (ia.nq == 4) return launch_fused_t<E, kPD, 4>(a, ia, num_groups, max_group_reqs, cus, np, st, ev);
  if (ia.nq > 1) return PH_ERR_ARG;  // grouped_stream_heads() says which shapes have the grouped form
  return launch_fused_t<E, kPD>(a, ia, num_groups, max_group_reqs, cus, np, st, ev);
}

// One launch for the prefix and suffix phases: head size 128 (the eight-wave prefix form), balanced suffix plan present.
bool decode_fused_supported(int dtype, int D) { return D == kPD && (dtype == PH_F16 || dtype == PH_BF16); }

int launch_decode_fused(const PrefixArgs& a, const ItemArgs& ia, int dtype, int num_groups, int max_group_reqs, int cus,
                        int prefix_wgs, hipStream_t st, const KernelEvents& ev) {
  return dtype == PH_F16 ? launch_fused_e<F16>(a, ia, num_groups, max_group_reqs, cus, prefix_wgs, st, ev)
                         : launch_fused_e<BF16>(a, ia, num_groups, max_group_reqs, cus, prefix_wgs, st, ev);
}

// head size 128, and 80 / 96 / 112 as short heads on the 128-wide tile (TileWork::head_dim)
bool prefix_mfma_supported(int dtype, int D) {
  return (D == kPD || D == 112 || D == 96 || D == 80) && (dtype == PH_F16 || dtype == PH_BF16);
}

int launch_prefix_mfma(const PrefixArgs& a0, int dtype, int D, int num_groups, int max_group_reqs, bool internal_ml,
                       hipStream_t st, const KernelEvents& ev) {
  if (!prefix_mfma_supported(dtype, D)) return PH_ERR_HEAD_DIM;
  if (num_groups <= 0 || max_group_reqs <= 0 || a0.n_splits <= 0) return PH_OK;
  PrefixArgs a = a0;
  a.head_dim = D;
  return dtype == PH_F16 ? launch_prefix_t<F16>(a, num_groups, max_group_reqs, internal_ml, st, ev)
                         : launch_prefix_t<BF16>(a, num_groups, max_group_reqs, internal_ml, st, ev);
}

int launch_prefill_mfma(const PrefillArgs& a0, int dtype, int D, int64_t num_tokens, hipStream_t st) {
  if (!prefix_mfma_supported(dtype, D)) return PH_ERR_HEAD_DIM;
  if (num_tokens <= 0 || a0.num_chunks <= 0) return PH_OK;
  PrefillArgs a = a0;
  a.head_dim = a.pair ? kPD : D;
  return dtype == PH_F16 ? launch_prefill_t<F16>(a, num_tokens, st) : launch_prefill_t<BF16>(a, num_tokens, st);
}

}  // namespace ph
