// Token sampler: temperature, top-p filter and one draw per row in one launch, without sorting the row.
// Follows parrot/engine/builtin/models/sampler.py:19-66:
//   :33-40  logits / temperature, the quotient rounded to the logits' element type (in-place division);
//   :43-56  a token is dropped when the probability mass of the tokens sorted before it (descending) exceeds
//           top_p -- the most likely token always stays, and so does the token on which the mass crosses top_p;
//   :63-64  soft-max of the surviving logits, one token drawn from it.
// The reference sorts every row twice (sort, then arg-sort of the permutation) to apply the filter.  Here the
// filter is a threshold: with e_i = exp(x_i - max) and G(t) = sum of e_j over e_j > t, token i stays iff
// G(e_i) + (its rank among equal values) * e_i <= top_p * sum(e).  G is monotone, so the smallest surviving value
// is found by bisection over the ordered bit patterns of the element type (16 steps for bf16, 19 for fp16, 32
// for fp32), each step a compare-and-add over the row's e values (the exponential is taken once per token) and
// one block reduction.  Equal values are ranked by ascending token id.
// The draw is the inverse-CDF draw over ascending token ids from a uniform number the caller passes, so the
// result is a function of the inputs (the reference draws through torch.multinomial's own random stream).
//
// One workgroup of 1024 lanes per row.  Two kernels, same arithmetic:
//   sample_rows_kernel   rows on the 16-byte grid of up to 57,344 tokens: the row lives in registers;
//   sample_top_p_kernel  any other row: e values in LDS up to 36 K tokens, longer rows are re-read and
//                        re-exponentiated in every pass (they sit in L2; slower).
// Sums are taken in a fixed order (per-lane partial sums, a wave tree, then the sixteen wave sums in
// sequence): the same tokens on every run.
#include "common.hpp"

namespace ph {

constexpr int kSampThreads = 1024;
constexpr int kSampWaves = kSampThreads / kWave;
constexpr int kSampLdsFloats = 36 * 1024;

template <typename E>
struct Logit {  // 16-bit element types
  static constexpr int kBytes = 2;
  static __device__ __forceinline__ float load(const void* row, int i) {
    return Elem<E>::one(static_cast<const uint16_t*>(row)[i]);
  }
  static __device__ __forceinline__ float round(float f) { return rnd<E>(f); }
  static __device__ __forceinline__ void unpack(const u32x4 raw, float* x) {  // 8 elements
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      x[2 * j] = Elem<E>::lo(raw[j]);
      x[2 * j + 1] = Elem<E>::hi(raw[j]);
    }
  }
};
template <>
struct Logit<F32> {
  static constexpr int kBytes = 4;
  static __device__ __forceinline__ void unpack(const u32x4 raw, float* x) {  // 4 elements
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = raw[j];  // a copy: the cast below is applied to a plain scalar, not to a vector element
      x[j] = __builtin_bit_cast(float, w);
    }
  }
  static __device__ __forceinline__ float load(const void* row, int i) { return static_cast<const float*>(row)[i]; }
  static __device__ __forceinline__ float round(float f) { return f; }
};
// low bits of the fp32 pattern that are zero for every value of the element type
template <typename E> constexpr int key_shift();
template <> constexpr int key_shift<F16>() { return 13; }
template <> constexpr int key_shift<BF16>() { return 16; }
template <> constexpr int key_shift<F32>() { return 0; }

// order-preserving map float -> unsigned (shifted down by SH), and back to the float of a key
template <int SH>
__device__ __forceinline__ uint32_t to_key(float f) {
  uint32_t b = __builtin_bit_cast(uint32_t, f);
  b ^= (b >> 31) ? 0xffffffffu : 0x80000000u;
  return b >> SH;
}
template <int SH>
__device__ __forceinline__ float from_key(uint32_t ks) {
  const uint32_t k = ks << SH;
  const uint32_t b = (k >> 31) ? (k ^ 0x80000000u) : ~(k | ((1u << SH) - 1u));
  return __builtin_bit_cast(float, b);
}

struct SampShared {
  float red[2][kSampWaves];
  float fpart[kSampWaves];
  int ipart[kSampWaves];
  int found, found_after, last;
};

struct SampArgs {
  const void* logits;
  int64_t row_stride;  // elements
  const float* temperature;
  const float* top_p;
  const float* uniform;
  int64_t* out;
  int V;
  float* probs;          // set: no draw, the filtered and renormalised probabilities of every row go here
  int64_t probs_stride;  // floats between rows
};

template <typename E, bool LDSX>
__global__ __launch_bounds__(kSampThreads) void sample_top_p_kernel(const SampArgs a) {
  extern __shared__ __attribute__((aligned(16))) float xs[];
  __shared__ SampShared sh;
  constexpr int SH = key_shift<E>();
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int64_t row = blockIdx.x;
  const int V = a.V;
  const void* lrow = static_cast<const char*>(a.logits) + row * a.row_stride * Logit<E>::kBytes;
  float T = a.temperature ? a.temperature[row] : 1.f;
  float p = a.top_p ? a.top_p[row] : 1.f;
  if (!(T > 0.f)) {  // the limit of a vanishing temperature: the most likely token
    T = 1.f;
    p = 0.f;
  }
  if (t == 0) {
    sh.found = INT_MAX;
    sh.last = -1;
  }
  int par = 0;
  // block-wide reductions; the two buffers alternate so that one barrier per reduction is enough
  auto block_sum = [&](float v) {
    v = group_sum<64>(v);
    if (lane == 0) sh.red[par][w] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < kSampWaves; ++i) s += sh.red[par][i];
    par ^= 1;
    return s;
  };
  auto block_max = [&](float v) {
    v = group_max<64>(v);
    if (lane == 0) sh.red[par][w] = v;
    __syncthreads();
    float s = sh.red[par][0];
#pragma unroll
    for (int i = 1; i < kSampWaves; ++i) s = fmaxf(s, sh.red[par][i]);
    par ^= 1;
    return s;
  };
  auto fresh = [&](int i) {
    float l = Logit<E>::load(lrow, i);
    if (T != 1.f) l = Logit<E>::round(__fdiv_rn(l, T));
    return l;
  };

  float m = -INFINITY;
  for (int i = t; i < V; i += kSampThreads) {
    const float x = fresh(i);
    if (LDSX) xs[i] = x;
    m = fmaxf(m, x);
  }
  m = block_max(m);
  if (!(m > -INFINITY && m < INFINITY)) m = 0.f;
  // e_i = exp(x_i - max): computed once and kept in LDS (each lane rewrites the slots it filled itself); every
  // later pass, the equal-value ranking included, works on e alone
  float z = 0.f;
  for (int i = t; i < V; i += kSampThreads) {
    const float e = expf((LDSX ? xs[i] : fresh(i)) - m);
    if (LDSX) xs[i] = e;
    z += e;
  }
  z = block_sum(z);  // and its barrier publishes the e values
  auto e_at = [&](int i) { return LDSX ? xs[i] : expf(fresh(i) - m); };

  // smallest surviving e `thr`, the mass above it, and how many tokens equal to it survive
  float thr = -1.f;  // no filter: everything is above
  int n_equal = INT_MAX;
  if (p < 1.f) {
    const float target = fmaxf(p, 0.f) * z;
    uint32_t lo = to_key<SH>(-INFINITY), hi = to_key<SH>(m);
    float g_hi = 0.f;
    while (lo < hi) {  // lo, hi and g are the same in every lane
      const uint32_t mid = lo + ((hi - lo) >> 1);
      const float cut = expf(from_key<SH>(mid) - m);
      float g = 0.f;
      for (int i = t; i < V; i += kSampThreads) {
        const float e = e_at(i);
        g += e > cut ? e : 0.f;
      }
      g = block_sum(g);
      if (g <= target) {
        hi = mid;
        g_hi = g;
      } else {
        lo = mid + 1;
      }
    }
    thr = expf(from_key<SH>(hi) - m);
    if (thr > 0.f) {
      const float r = floorf((target - g_hi) / thr);
      n_equal = r >= 2.0e9f ? INT_MAX : max((int)r + 1, 1);
    }
  }

  // last pass: every lane owns a run of consecutive token ids (odd length: conflict-free in LDS)
  const int per = ((V + kSampThreads - 1) / kSampThreads) | 1;
  const int b0 = min(t * per, V), b1 = min(b0 + per, V);
  int eq = 0;
  for (int i = b0; i < b1; ++i) eq += e_at(i) == thr ? 1 : 0;
  int inc = eq;  // rank of this lane's first equal token = equal tokens in the lanes before
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int up = __shfl_up(inc, d, kWave);
    if (lane >= d) inc += up;
  }
  if (lane == kWave - 1) sh.ipart[w] = inc;
  __syncthreads();
  int rank0 = inc - eq;
  for (int i = 0; i < w; ++i) rank0 += sh.ipart[i];

  auto walk = [&](auto&& visit) {  // visit(i, e) for every surviving token of this lane's run, in id order
    int rank = rank0;
    for (int i = b0; i < b1; ++i) {
      const float e = e_at(i);
      const bool keep = e > thr || (e == thr && rank++ < n_equal);
      if (keep) visit(i, e);
    }
  };
  float s = 0.f;
  walk([&](int, float e) { s += e; });
  float finc = s;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const float up = __shfl_up(finc, d, kWave);
    if (lane >= d) finc += up;
  }
  if (lane == kWave - 1) sh.fpart[w] = finc;
  __syncthreads();
  float base = 0.f, kept = 0.f;
  for (int i = 0; i < kSampWaves; ++i) {
    if (i == w) base = kept;
    kept += sh.fpart[i];
  }
  base += finc - s;
  if (a.probs) {  // the distribution itself instead of a draw from it: zero for dropped tokens, e / (kept mass) else
    float* prow = a.probs + row * a.probs_stride;
    const float inv = 1.f / kept;
    for (int i = b0; i < b1; ++i) prow[i] = 0.f;
    walk([&](int i, float e) { prow[i] = e * inv; });
    return;
  }
  const float goal = a.uniform[row] * kept;
  int found = INT_MAX, last = -1;
  float running = base;
  walk([&](int i, float e) {
    running += e;
    if (e > 0.f) last = i;
    if (running > goal && found == INT_MAX) found = i;
  });
  if (found != INT_MAX) atomicMin(&sh.found, found);
  if (last >= 0) atomicMax(&sh.last, last);
  __syncthreads();
  if (t == 0) {
    // rounding can leave the goal a hair above the last partial sum: then the last surviving token
    const int id = sh.found != INT_MAX ? sh.found : max(sh.last, 0);
    a.out[row] = id;
  }
}

// Rows that fit the register file: 16-byte aligned rows of up to 1024 * kSampRegFloats tokens.  Lane t owns the
// 16-byte chunks t, t + 1024, t + 2048, ... of the row (K "rounds" of 1024 chunks); the row is read once, the
// exponentials are taken once, and every later pass is compares and adds on registers.  Token-id order is
// (round, lane, position in the chunk), so the two places that need it -- ranking equal values at the cut and
// the cumulative sum of the draw -- take one batched reduction over the rounds to find the round in which the
// count / the sum crosses, and one scan over the lanes inside that round.
constexpr int kSampRegFloats = 56;

template <typename E>
__global__ __launch_bounds__(kSampThreads) void sample_rows_kernel(const SampArgs a) {
  constexpr int N = 16 / Logit<E>::kBytes;  // tokens per chunk
  constexpr int K = kSampRegFloats / N;     // chunks per lane
  constexpr int SH = key_shift<E>();
  __shared__ SampShared sh;
  __shared__ float fred[K][kSampWaves];
  __shared__ int ired[K][kSampWaves];
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  const int64_t row = blockIdx.x;
  const int V = a.V;
  const char* lrow = static_cast<const char*>(a.logits) + row * a.row_stride * Logit<E>::kBytes;
  float T = a.temperature ? a.temperature[row] : 1.f;
  float p = a.top_p ? a.top_p[row] : 1.f;
  if (!(T > 0.f)) {
    T = 1.f;
    p = 0.f;
  }
  if (t == 0) {
    sh.found = INT_MAX;
    sh.found_after = INT_MAX;
    sh.last = -1;
  }
  int par = 0;
  auto block_sum = [&](float v) {
    v = group_sum<64>(v);
    if (lane == 0) sh.red[par][w] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < kSampWaves; ++i) s += sh.red[par][i];
    par ^= 1;
    return s;
  };

  float e[K][N];
  const int chunks = (V + N - 1) / N;
  const int rounds = (chunks + kSampThreads - 1) / kSampThreads;  // rounds that hold tokens; the rest stay zero
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int c = t + k * kSampThreads;
    if (k >= rounds) {
#pragma unroll
      for (int j = 0; j < N; ++j) e[k][j] = 0.f;
    } else if (c < chunks && (c + 1) * N <= V) {
      Logit<E>::unpack(ld16(lrow + (int64_t)c * 16), e[k]);
    } else {  // the row's last, partial chunk, and chunks past the row
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const int i = c * N + j;
        e[k][j] = i < V ? Logit<E>::load(lrow, i) : -INFINITY;
      }
    }
  }
  float m = -INFINITY;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (k >= rounds) break;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      if (T != 1.f) e[k][j] = Logit<E>::round(__fdiv_rn(e[k][j], T));
      m = fmaxf(m, e[k][j]);
    }
  }
  m = group_max<64>(m);
  if (lane == 0) sh.red[par][w] = m;
  __syncthreads();
  m = sh.red[par][0];
#pragma unroll
  for (int i = 1; i < kSampWaves; ++i) m = fmaxf(m, sh.red[par][i]);
  par ^= 1;
  if (!(m > -INFINITY && m < INFINITY)) m = 0.f;
  float z = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (k >= rounds) break;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      e[k][j] = expf(e[k][j] - m);
      z += e[k][j];
    }
  }
  z = block_sum(z);

  if (p < 1.f) {  // the filter: zero the e of every token that does not survive
    const float target = fmaxf(p, 0.f) * z;
    uint32_t lo = to_key<SH>(-INFINITY), hi = to_key<SH>(m);
    float g_hi = 0.f;
    while (lo < hi) {  // lo, hi and g are the same in every lane
      const uint32_t mid = lo + ((hi - lo) >> 1);
      const float cut = expf(from_key<SH>(mid) - m);
      float g = 0.f;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        if (k >= rounds) break;
#pragma unroll
        for (int j = 0; j < N; ++j) g += e[k][j] > cut ? e[k][j] : 0.f;
      }
      g = block_sum(g);
      if (g <= target) {
        hi = mid;
        g_hi = g;
      } else {
        lo = mid + 1;
      }
    }
    const float thr = expf(from_key<SH>(hi) - m);
    int n_equal = INT_MAX;
    if (thr > 0.f) {
      const float r = floorf((target - g_hi) / thr);
      n_equal = r >= 2.0e9f ? INT_MAX : max((int)r + 1, 1);
    }
    // tokens equal to thr, per round; they survive in id order until n_equal of them have
    int cnt[K], tot[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      cnt[k] = 0;
      if (k >= rounds) continue;
#pragma unroll
      for (int j = 0; j < N; ++j) cnt[k] += e[k][j] == thr ? 1 : 0;
      int v = cnt[k];
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
      if (lane == 0) ired[k][w] = v;
    }
    __syncthreads();
    int kc = K, before_kc = 0, run = 0;  // the round in which the count passes n_equal (K: it never does)
#pragma unroll
    for (int k = 0; k < K; ++k) {
      tot[k] = 0;
      if (k < rounds) {
#pragma unroll
        for (int i = 0; i < kSampWaves; ++i) tot[k] += ired[k][i];
      }
      if (kc == K && run + tot[k] > n_equal) {
        kc = k;
        before_kc = run;
      }
      run += tot[k];
    }
    int rank_kc = 0;  // rank of this lane's first equal token of round kc
    if (kc < K) {     // same in every lane
      int mine = 0;
#pragma unroll
      for (int k = 0; k < K; ++k) mine = k == kc ? cnt[k] : mine;
      int inc = mine;
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int up = __shfl_up(inc, d, kWave);
        if (lane >= d) inc += up;
      }
      if (lane == kWave - 1) sh.ipart[w] = inc;
      __syncthreads();
      rank_kc = before_kc + inc - mine;
      for (int i = 0; i < w; ++i) rank_kc += sh.ipart[i];
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      if (k >= rounds) break;
      int rank = rank_kc;
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const float v = e[k][j];
        bool keep = v > thr;
        if (v == thr) keep = k < kc || (k == kc && rank++ < n_equal);
        e[k][j] = keep ? v : 0.f;
      }
    }
  }

  // the draw: first token, in id order, at which the running sum of e passes uniform * (sum of e)
  float cs[K], tot[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    cs[k] = 0.f;
    if (k >= rounds) continue;
#pragma unroll
    for (int j = 0; j < N; ++j) cs[k] += e[k][j];
    const float v = group_sum<64>(cs[k]);
    if (lane == 0) fred[k][w] = v;
  }
  __syncthreads();
  float kept = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    tot[k] = 0.f;
    if (k < rounds) {
#pragma unroll
      for (int i = 0; i < kSampWaves; ++i) tot[k] += fred[k][i];
    }
    kept += tot[k];
  }
  const float goal = a.uniform[row] * kept;
  int kd = K;  // the round in which the running sum passes the goal
  float before_kd = 0.f, run = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (kd == K && run + tot[k] > goal) {
      kd = k;
      before_kd = run;
    }
    run += tot[k];
  }
  float mine = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) mine = k == kd ? cs[k] : mine;
  float finc = mine;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const float up = __shfl_up(finc, d, kWave);
    if (lane >= d) finc += up;
  }
  if (lane == kWave - 1) sh.fpart[w] = finc;
  __syncthreads();
  float running = before_kd;
  for (int i = 0; i < w; ++i) running += sh.fpart[i];
  running += finc - mine;
  int found = INT_MAX, found_after = INT_MAX, last = -1;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (k >= rounds) break;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float v = e[k][j];
      const int i = (t + k * kSampThreads) * N + j;
      if (v > 0.f) {
        last = i;
        if (k > kd && found_after == INT_MAX) found_after = i;
        if (k == kd) {
          running += v;
          if (running > goal && found == INT_MAX) found = i;
        }
      }
    }
  }
  if (found != INT_MAX) atomicMin(&sh.found, found);
  if (found_after != INT_MAX) atomicMin(&sh.found_after, found_after);
  if (last >= 0) atomicMax(&sh.last, last);
  __syncthreads();
  if (t == 0) {
    // rounding can leave the goal a hair above the sums of the round it was placed in: then the next surviving
    // token, or the last one of the row
    const int id = sh.found != INT_MAX ? sh.found : sh.found_after != INT_MAX ? sh.found_after : max(sh.last, 0);
    a.out[row] = id;
  }
}

template <typename E>
static int launch_sample(const SampArgs& a, int64_t rows, hipStream_t st) {
  dim3 grid((unsigned)rows), block(kSampThreads);
  const bool rows_aligned = aligned16(a.logits) && (a.row_stride * Logit<E>::kBytes) % 16 == 0;
  if (rows_aligned && a.V <= kSampThreads * kSampRegFloats) {
    hipLaunchKernelGGL((sample_rows_kernel<E>), grid, block, 0, st, a);
  } else if (a.V <= kSampLdsFloats) {
    const size_t lds = (size_t)a.V * sizeof(float);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_top_p_kernel<E, true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kSampLdsFloats * (int)sizeof(float));
    hipLaunchKernelGGL((sample_top_p_kernel<E, true>), grid, block, lds, st, a);
  } else {
    hipLaunchKernelGGL((sample_top_p_kernel<E, false>), grid, block, 0, st, a);
  }
  return launch_status();
}

}  // namespace ph

using namespace ph;

extern "C" int ph_sample_top_p(const void* logits, int64_t row_stride, const float* temperature, const float* top_p,
                               const float* uniform, int64_t* out_ids, int64_t rows, int64_t vocab, int dtype,
                               void* stream) {
  if (rows < 0 || vocab <= 0 || vocab >= ((int64_t)1 << 30) || row_stride < vocab) return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (rows == 0) return PH_OK;
  if (!logits || !uniform || !out_ids) return PH_ERR_ARG;
  if (rows > 0x7fffffff) return PH_ERR_ARG;
  const SampArgs a{logits, row_stride, temperature, top_p, uniform, out_ids, (int)vocab, nullptr, 0};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == PH_F16) return launch_sample<F16>(a, rows, st);
  if (dtype == PH_BF16) return launch_sample<BF16>(a, rows, st);
  return launch_sample<F32>(a, rows, st);
}

template <typename E>
static int launch_probs(const SampArgs& a, int64_t rows, hipStream_t st) {
  dim3 grid((unsigned)rows), block(kSampThreads);
  if (a.V <= kSampLdsFloats) {
    const size_t lds = (size_t)a.V * sizeof(float);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&sample_top_p_kernel<E, true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kSampLdsFloats * (int)sizeof(float));
    hipLaunchKernelGGL((sample_top_p_kernel<E, true>), grid, block, lds, st, a);
  } else {
    hipLaunchKernelGGL((sample_top_p_kernel<E, false>), grid, block, 0, st, a);
  }
  return launch_status();
}

extern "C" int ph_top_p_probs(const void* logits, int64_t row_stride, const float* temperature, const float* top_p,
                              float* probs, int64_t probs_stride, int64_t rows, int64_t vocab, int dtype,
                              void* stream) {
  if (rows < 0 || vocab <= 0 || vocab >= ((int64_t)1 << 30) || row_stride < vocab || probs_stride < vocab)
    return PH_ERR_ARG;
  if (dtype != PH_F16 && dtype != PH_BF16 && dtype != PH_F32) return PH_ERR_DTYPE;
  if (rows == 0) return PH_OK;
  if (!logits || !probs || rows > 0x7fffffff) return PH_ERR_ARG;
  const SampArgs a{logits, row_stride, temperature, top_p, nullptr, nullptr, (int)vocab, probs, probs_stride};
  hipStream_t st = (hipStream_t)stream;
  if (dtype == PH_F16) return launch_probs<F16>(a, rows, st);
  if (dtype == PH_BF16) return launch_probs<BF16>(a, rows, st);
  return launch_probs<F32>(a, rows, st);
}
