// On-GPU sampling and scheduler bookkeeping: greedy / categorical sampling with raw
// log-probabilities, temperature + top-k + nucleus sampling, the per-row record step of a
// generation session (stop automaton, finish codes, RNG positions) and the slot gather/scatter
// used by compact decode batches.  Nothing here synchronises with the host.
#include "lfm2_common.h"

#include <mutex>

namespace {

#define DISPATCH_DTYPE(dtype, name, ...)                                               \
  switch (dtype) {                                                                     \
    case LFM2_DTYPE_BF16: { typedef __bf16 T; __VA_ARGS__; } break;                    \
    case LFM2_DTYPE_F16: { typedef _Float16 T; __VA_ARGS__; } break;                   \
    case LFM2_DTYPE_F32: { typedef float T; __VA_ARGS__; } break;                      \
    default: LFM2_FAIL(LFM2_ERR_ARGUMENT, "%s: unknown dtype %d", name, dtype);        \
  }

constexpr uint64_t kGolden = 0x9E3779B97F4A7C15ull;
constexpr uint64_t kMask63 = 0x7FFFFFFFFFFFFFFFull;
constexpr int kTile = 4096;
constexpr int kNoIndex = 0x7fffffff;

// Philox4x32-10 (Salmon et al. 2011): 128-bit counter, 64-bit key -> four 32-bit words.
__device__ __forceinline__ void philox(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                       uint32_t* out) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    c0 = hi1 ^ c1 ^ k0; c1 = lo1; c2 = hi0 ^ c3 ^ k1; c3 = lo0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
// Standard Gumbel noise from a 32-bit word: u in [0,1) floored at 1e-30 (lfm25_sampling.py:21-27).
// The two logarithms run on the hardware log2 unit (about 1 ulp): this is noise, and the full-precision library
// routine made the sampler compute-bound (about a hundred instructions per logit).
__device__ __forceinline__ float gumbel(uint32_t bits) {
  const float u = fmaxf((float)(bits >> 8) * (1.0f / 16777216.0f), 1.0e-30f);
  return -__logf(-__logf(u));
}
__device__ __forceinline__ uint64_t row_key(int64_t seed, int64_t step) {
  return ((uint64_t)seed + (uint64_t)step * kGolden) & kMask63;
}

// ------------------------------------------------------------------------------------ full-support sampler
// Greedy rows take the first maximum.  Rows with a temperature draw from softmax(logits / T) by inverting the
// cumulative distribution with ONE uniform number per row (Philox keyed by the row's seed and step): the same
// categorical law as the reference's Gumbel-max (lfm25_sampling.py:9-58) without a random number, two logarithms and
// ten rounds of 32-bit multiplies per logit, which made the sampler compute-bound (30 us at 256 x 65536; the logits
// themselves stream in 8 us).  Exact draws were never comparable with the reference (its generator is Triton's);
// the distribution and the determinism in (seed, step) are what the tests hold.
//
// Pass 1: one workgroup per (row, 4096-column tile): the tile's maximum, sum exp(x - max) of the raw logits (for
// the log-probability) and of the tempered ones (the tile's probability mass).  About eight vector instructions per
// logit: with 16.8 M logits a step the arithmetic, not the 33 MB of traffic, is what the pass costs, hence the
// hardware exp2 with the scale folded into one multiply-add, and no second exponential at temperature 0 or 1.
// scratch[(row*parts+part)*4 + {tempered sum, unused, max, raw sum}].
constexpr float kLog2e = 1.4426950408889634f;
struct TileStat { float max, sum, mass; };
// Joins two partial softmax states (online normaliser, Milakov & Gimelshein 2018).
__device__ __forceinline__ TileStat join(const TileStat& a, const TileStat& b, float inv_temp) {
  TileStat r;
  r.max = fmaxf(a.max, b.max);
  const float da = a.max == r.max ? 0.f : a.max - r.max, db = b.max == r.max ? 0.f : b.max - r.max;  // no inf - inf
  r.sum = a.sum * __expf(da) + b.sum * __expf(db);
  r.mass = a.mass * __expf(da * inv_temp) + b.mass * __expf(db * inv_temp);
  return r;
}
// 16 bytes of consecutive columns, one load when the row stride allows it; columns beyond V read as -inf.
template <typename T>
__device__ __forceinline__ void load_columns(const T* src, int64_t col0, int64_t V, bool vector_ok, float* out) {
  constexpr int EPL = 16 / sizeof(T);
  typedef T vec __attribute__((ext_vector_type(EPL)));
  if (vector_ok && col0 < V) {
    const vec v = *reinterpret_cast<const vec*>(src + col0);
#pragma unroll
    for (int e = 0; e < EPL; ++e) out[e] = Elem<T>::load(v[e]);
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) out[e] = col0 + e < V ? Elem<T>::load(src[col0 + e]) : -INFINITY;
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
sample_partial_kernel(const T* logits, float* scratch, const float* temperatures, float temperature, int64_t V, int parts) {
  constexpr int EPL = 16 / sizeof(T), LOADS = 16 / EPL;
  __shared__ TileStat s_stat[4];
  const int64_t row = blockIdx.y;
  const int part = blockIdx.x;
  const float temp = temperatures ? temperatures[row] : temperature;
  const float inv_temp = temp > 0.f ? 1.0f / temp : 0.f;
  const T* src = logits + row * V;
  const bool vector_ok = V % EPL == 0;
  float vals[16];
#pragma unroll
  for (int i = 0; i < LOADS; ++i)
    load_columns(src, (int64_t)part * kTile + (i * 256 + threadIdx.x) * EPL, V, vector_ok, vals + i * EPL);
  float top = vals[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) top = fmaxf(top, vals[i]);
  top = wave_max(top);
  const float shift = top == -INFINITY ? 0.f : top;
  TileStat mine{top, 0.f, 0.f};
  const float bias = -shift * kLog2e;
#pragma unroll
  for (int i = 0; i < 16; ++i) mine.sum += __builtin_amdgcn_exp2f(fmaf(vals[i], kLog2e, bias));
  mine.sum = wave_sum(mine.sum);
  if (inv_temp == 1.f || inv_temp == 0.f) {
    mine.mass = mine.sum;   // greedy rows never read it
  } else {
    const float scale = kLog2e * inv_temp, tempered_bias = bias * inv_temp;
#pragma unroll
    for (int i = 0; i < 16; ++i) mine.mass += __builtin_amdgcn_exp2f(fmaf(vals[i], scale, tempered_bias));
    mine.mass = wave_sum(mine.mass);
  }
  if ((threadIdx.x & 63) == 0) s_stat[threadIdx.x >> 6] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    const TileStat t = join(join(s_stat[0], s_stat[1], inv_temp), join(s_stat[2], s_stat[3], inv_temp), inv_temp);
    float4 packed;
    packed.x = t.mass; packed.y = 0.f; packed.z = t.max; packed.w = t.sum;
    *reinterpret_cast<float4*>(scratch + (row * parts + part) * 4) = packed;
  }
}

// The per-row record step of lfm25_session.py:34-56 for one row and its freshly drawn token: token and raw
// log-probability into the row's buffers, stop automaton, finish code, flags, next input, random-stream position.
// `tokens == nullptr` means "no record": the sampler then only returns its draw.
struct RecordArgs {
  int64_t* tokens; float* logprobs; int32_t* lengths; const int32_t* limits; int8_t* reasons; uint8_t* alive;
  uint8_t* pending; int64_t* input; int64_t* stop_states; const int64_t* stop_offsets; const int32_t* stop_table;
  const uint8_t* ignore_eos; int64_t* rng_positions; int64_t eos, V, cap;
};
__device__ __forceinline__ void record_row(const RecordArgs& r, int64_t row, int64_t token, float logp) {
  if (!r.alive[row]) return;
  const int32_t length = r.lengths[row];
  r.tokens[row * r.cap + length] = token;
  r.logprobs[row * r.cap + length] = logp;
  const int32_t value = r.stop_table[r.stop_offsets[row] + r.stop_states[row] * r.V + token];
  r.stop_states[row] = value & 65535;
  int8_t reason = 0;
  if (token == r.eos && !r.ignore_eos[row]) reason = 1;
  else if (value >= 65536) reason = 2;
  else if (length + 1 >= r.limits[row]) reason = 3;
  r.lengths[row] = length + 1;
  r.rng_positions[row] += 1;
  r.reasons[row] = reason;
  r.alive[row] = reason == 0;
  r.pending[row] = reason == 0;
  r.input[row] = token;
}

// Pass 2, one workgroup per row: merge the tiles, then read one tile again.  Greedy rows take the first column
// that holds the maximum, in the first tile that has it.  The others pick the tile and then the column where the
// cumulative mass passes u * total (tiles and columns in index order; the last column with mass if rounding pushes
// the target past the end).  At most 256 tiles (a vocabulary of 2^20).
template <typename T>
__global__ void __launch_bounds__(256)
sample_finish_kernel(const T* logits, const float* scratch, int64_t* tokens, float* logprobs, float* sampling_logprobs,
                     const int64_t* seeds, const int64_t* steps, const float* temperatures, int64_t seed, int64_t step,
                     float temperature, int64_t V, int parts, RecordArgs record) {
  __shared__ TileStat s_stat[4];
  __shared__ float s_tile_mass[256];
  __shared__ float s_wave[4];
  __shared__ float s_target, s_log_mass;
  __shared__ double s_uniform;
  __shared__ int s_tile, s_pick;
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool per_row = seeds != nullptr;
  const float temp = per_row ? temperatures[row] : temperature;
  const float inv_temp = temp > 0.f ? 1.0f / temp : 0.f;
  TileStat own{-INFINITY, 0.f, 0.f};
  if (threadIdx.x < parts) {
    const float4 packed = *reinterpret_cast<const float4*>(scratch + (row * parts + threadIdx.x) * 4);
    own.mass = packed.x; own.max = packed.z; own.sum = packed.w;
  }
  if (threadIdx.x == 255) {  // a thread with no tile of its own draws the row's uniform number meanwhile
    const uint64_t key = per_row ? row_key(seeds[row], steps[row]) : row_key(seed, step);
    uint32_t rnd[4];
    // per-row streams use counter 0; the shared stream counts rows
    philox(per_row ? 0u : (uint32_t)row, per_row ? 0u : (uint32_t)(row >> 32), 0u, 0u, (uint32_t)key, (uint32_t)(key >> 32), rnd);
    s_uniform = (double)((((uint64_t)rnd[0] << 32) | rnd[1]) >> 11) * (1.0 / 9007199254740992.0);
    s_pick = kNoIndex;
  }
  const float wave_top = wave_max(own.max);
  if (lane == 0) s_wave[wave] = wave_top;
  __syncthreads();
  const float mx = fmaxf(fmaxf(s_wave[0], s_wave[1]), fmaxf(s_wave[2], s_wave[3]));
  const float gap = own.max == mx ? 0.f : own.max - mx;
  float total = own.sum * __expf(gap);
  if (threadIdx.x < parts) s_tile_mass[threadIdx.x] = temp > 0.f ? own.mass * __expf(gap * inv_temp) : (own.max == mx ? 1.f : 0.f);
  total = wave_sum(total);
  if (lane == 0) s_stat[wave].sum = total;
  __syncthreads();
  total = (s_stat[0].sum + s_stat[1].sum) + (s_stat[2].sum + s_stat[3].sum);
  if (threadIdx.x == 0) {
    int tile = 0;
    float inside = 0.f;
    if (temp > 0.f) {
      // 53 uniform bits and double sums across tiles: the resolution inside the chosen tile is then relative to
      // that tile's mass, not to the whole row's
      double z = 0.0;
      for (int p = 0; p < parts; ++p) z += (double)s_tile_mass[p];
      const double target = s_uniform * z;
      double before = 0.0;
      for (int p = 0; p < parts; ++p) {
        const double m = (double)s_tile_mass[p];
        if (m > 0.0) tile = p;                   // last tile with mass, in case rounding overshoots
        if (target < before + m) break;
        before += m;
      }
      inside = (float)(target - before);
      s_log_mass = (float)log(z);   // log sum exp((x - max) / T): the normaliser of the distribution the draw is from
    } else {
      while (tile < parts - 1 && s_tile_mass[tile] == 0.f) ++tile;   // first tile that holds the maximum
    }
    s_tile = tile;
    s_target = inside;
  }
  __syncthreads();
  const int tile = s_tile;
  const float target = s_target;
  // the tile again: each thread owns 16 consecutive columns, so column order = thread order
  constexpr int EPL = 16 / sizeof(T), LOADS = 16 / EPL;
  const int64_t col0 = (int64_t)tile * kTile + threadIdx.x * 16;
  const bool vector_ok = V % EPL == 0;
  float x[16];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) load_columns(logits + row * V, col0 + i * EPL, V, vector_ok, x + i * EPL);
  int pick = kNoIndex, last = -1;
  if (temp > 0.f) {
    float e[16], sum = 0.f;
    const float scale = kLog2e * inv_temp, bias = -mx * scale;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      e[i] = __builtin_amdgcn_exp2f(fmaf(x[i], scale, bias));   // -inf beyond V and for masked columns: 0
      sum += e[i];
    }
    // exclusive prefix of the threads' sums: wave scan, then the earlier waves' totals
    float incl = sum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float v = __shfl_up(incl, o, 64);
      if (lane >= o) incl += v;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    float run = incl - sum;
    for (int w = 0; w < wave; ++w) run += s_wave[w];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      if (e[i] > 0.f) {
        last = (int)(col0 + i);
        if (pick == kNoIndex && target < run + e[i]) pick = last;
      }
      run += e[i];
    }
  } else {
#pragma unroll
    for (int i = 15; i >= 0; --i)
      if (x[i] == mx && col0 + i < V) pick = (int)(col0 + i);
  }
  if (pick != kNoIndex) atomicMin(&s_pick, pick);
  __syncthreads();
  if (s_pick == kNoIndex) {  // the target lies past the tile's recomputed mass: the last column with mass
    __syncthreads();
    if (threadIdx.x == 0) s_pick = -1;
    __syncthreads();
    if (last >= 0) atomicMax(&s_pick, last);
    __syncthreads();
  }
  const int token = s_pick < 0 ? (int)((int64_t)tile * kTile) : s_pick;   // nothing comparable (NaN row): the tile's first column
  // the thread that holds the chosen column writes the row's result
  if (token >= col0 && token < col0 + 16) {
    tokens[row] = token;
    float chosen = x[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) chosen = token - col0 == i ? x[i] : chosen;
    const float logp = chosen - (mx + logf(total));
    if (logprobs) logprobs[row] = logp;
    // log-probability under softmax(logits / T), the distribution sampled from (lfm25_engine.py:1605-1608); greedy
    // rows report the raw one (lfm25_engine.py:1591-1596)
    if (sampling_logprobs) sampling_logprobs[row] = temp > 0.f ? (chosen - mx) * inv_temp - s_log_mass : logp;
    if (record.tokens) record_row(record, row, token, logp);
  }
}

// ------------------------------------------------------------------------------------ filtered sampler
// Order-preserving map float -> uint32 (larger float = larger key).
__device__ __forceinline__ uint32_t order_key(float x) {
  const uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
constexpr int kFT = 1024;  // threads of the filtered sampler

// One workgroup per row.  All decisions use integer histograms (counts, and 2^40 fixed-point
// softmax mass), so results do not depend on the order in which lanes reach the atomics.
// This form re-reads the row from memory in every pass and serves vocabularies beyond what a workgroup can hold in
// registers; the register form below makes the same decisions.
template <typename T>
__global__ void __launch_bounds__(kFT)
sample_filtered_stream_kernel(const T* logits, int64_t* tokens, float* logprobs, float* sampling_logprobs, int32_t* kept_count, const int64_t* seeds,
                       const int64_t* steps, const float* temperatures, const int32_t* top_ks, const float* top_ps, int64_t seed,
                       int64_t step, float temperature, int top_k, float top_p, int64_t V) {
  if (temperatures) {   // per-row parameters: rows that ask for no filter (or are greedy) keep what the outputs hold
    temperature = temperatures[blockIdx.x];
    top_k = top_ks[blockIdx.x];
    top_p = top_ps[blockIdx.x];
    if (!(temperature > 0.f) || (top_k <= 0 && !(top_p < 1.0f))) return;
  }
  __shared__ uint32_t h_cnt[256];
  __shared__ unsigned long long h_mass[256];
  __shared__ float s_f[kFT / 64], s_kept[kFT / 64];
  __shared__ int s_i[kFT / 64];
  __shared__ uint32_t s_digit, s_remaining, s_cnt_above;
  __shared__ unsigned long long s_mass_above, s_total;
  __shared__ int s_scan[kFT];
  __shared__ int s_cut, s_cross;
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* src = logits + row * V;
  const uint64_t key64 = seeds ? row_key(seeds[row], steps[row]) : row_key(seed, step);

  // raw max / normaliser (for the returned log-probability) -- identical for scaled logits' argmax
  float mx = -INFINITY;
  for (int64_t i = tid; i < V; i += kFT) mx = fmaxf(mx, Elem<T>::load(src[i]));
  mx = wave_max(mx);
  if (lane == 0) s_f[wave] = mx;
  __syncthreads();
  mx = s_f[0];
  for (int w = 1; w < kFT / 64; ++w) mx = fmaxf(mx, s_f[w]);
  __syncthreads();
  float raw_sum = 0.f;
  for (int64_t i = tid; i < V; i += kFT) raw_sum += expf(Elem<T>::load(src[i]) - mx);
  raw_sum = wave_sum(raw_sum);
  if (lane == 0) s_f[wave] = raw_sum;
  __syncthreads();
  raw_sum = 0.f;
  for (int w = 0; w < kFT / 64; ++w) raw_sum += s_f[w];
  const float xmax = mx / temperature;
  auto scaled = [&](int64_t i) { return Elem<T>::load(src[i]) / temperature; };
  auto mass_of = [&](float x) -> unsigned long long { return (unsigned long long)(exp2f((x - xmax) * LFM2_LOG2E) * 1099511627776.0f); };

  // ---- top-k: key of the k-th largest scaled logit
  uint32_t key_k = 0;
  if (top_k > 0 && top_k < V) {
    uint32_t prefix = 0, mask = 0;
    if (tid == 0) s_remaining = (uint32_t)top_k;
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      for (int i = tid; i < 256; i += kFT) h_cnt[i] = 0;
      __syncthreads();
      for (int64_t i = tid; i < V; i += kFT) {
        const uint32_t k = order_key(scaled(i));
        if ((k & mask) == prefix) atomicAdd(&h_cnt[(k >> shift) & 255], 1u);
      }
      __syncthreads();
      if (tid == 0) {
        uint32_t rem = s_remaining;
        int d = 255;
        for (; d > 0; --d) {
          if (h_cnt[d] >= rem) break;
          rem -= h_cnt[d];
        }
        s_digit = (uint32_t)d; s_remaining = rem;
      }
      __syncthreads();
      prefix |= s_digit << shift;
      mask |= 0xFFu << shift;
      __syncthreads();
    }
    key_k = prefix;
  }

  // ---- nucleus: walk keys downward until the inclusive cumulative mass exceeds top_p * Z
  uint32_t kp = key_k;
  int ties_kept = 0x7fffffff;
  uint32_t cnt_above = 0;
  if (top_p < 1.0f) {
    unsigned long long z = 0;
    for (int64_t i = tid; i < V; i += kFT) {
      const float x = scaled(i);
      if (order_key(x) >= key_k) z += mass_of(x);
    }
    if (tid == 0) s_total = 0;
    __syncthreads();
    atomicAdd(&s_total, z);
    __syncthreads();
    const unsigned long long limit = (unsigned long long)((double)top_p * (double)s_total);
    uint32_t prefix = 0, mask = 0;
    if (tid == 0) { s_mass_above = 0; s_cnt_above = 0; s_cross = 0; }
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      for (int i = tid; i < 256; i += kFT) { h_cnt[i] = 0; h_mass[i] = 0; }
      __syncthreads();
      for (int64_t i = tid; i < V; i += kFT) {
        const float x = scaled(i);
        const uint32_t k = order_key(x);
        if (k >= key_k && (k & mask) == prefix) {
          atomicAdd(&h_cnt[(k >> shift) & 255], 1u);
          atomicAdd(&h_mass[(k >> shift) & 255], mass_of(x));
        }
      }
      __syncthreads();
      if (tid == 0) {
        unsigned long long above = s_mass_above;
        uint32_t ca = s_cnt_above;
        int d = 255, crossed = 0;
        for (; d >= 0; --d) {
          if (h_cnt[d] == 0) continue;
          if (above + h_mass[d] > limit) { crossed = 1; break; }
          above += h_mass[d]; ca += h_cnt[d];
        }
        s_cross = crossed; s_digit = (uint32_t)(d < 0 ? 0 : d); s_mass_above = above; s_cnt_above = ca;
        s_remaining = crossed ? h_cnt[d] : 0;
      }
      __syncthreads();
      if (!s_cross) break;
      prefix |= s_digit << shift;
      mask |= 0xFFu << shift;
      __syncthreads();
    }
    if (s_cross) {
      kp = prefix;
      cnt_above = s_cnt_above;
      const unsigned long long w = mass_of(__uint_as_float((kp & 0x80000000u) ? (kp & 0x7fffffffu) : ~kp));
      unsigned long long fit = w ? (limit - s_mass_above) / w : 0;
      if (fit >= s_remaining) fit = s_remaining;
      ties_kept = (int)fit;
      if (cnt_above == 0 && ties_kept == 0) ties_kept = 1;  // rank 0 always survives
    }
    __syncthreads();
  }

  // ---- when only some of the ties at kp survive, keep the lowest-index ones: find the cut column
  int cut = 0x7fffffff;
  if (ties_kept != 0x7fffffff) {
    const int64_t strip = (V + kFT - 1) / kFT;
    const int64_t lo = tid * strip, hi = lo + strip < V ? lo + strip : V;
    int c = 0;
    for (int64_t i = lo; i < hi; ++i) c += order_key(scaled(i)) == kp;
    s_scan[tid] = c;
    __syncthreads();
    if (tid == 0) {
      int run = 0;
      s_cut = -1;
      for (int t = 0; t < kFT; ++t) { const int v = s_scan[t]; s_scan[t] = run; run += v; }
    }
    __syncthreads();
    const int before = s_scan[tid];
    if (ties_kept > before && ties_kept <= before + c) {
      int seen = before;
      for (int64_t i = lo; i < hi; ++i)
        if (order_key(scaled(i)) == kp && ++seen == ties_kept) { s_cut = (int)i; break; }
    }
    __syncthreads();
    cut = s_cut;
    if (kept_count && tid == 0) kept_count[row] = (int)cnt_above + ties_kept;
  } else if (kept_count) {
    int c = 0;
    for (int64_t i = tid; i < V; i += kFT) c += order_key(scaled(i)) >= kp;
    if (tid == 0) s_cut = 0;
    __syncthreads();
    atomicAdd(&s_cut, c);
    __syncthreads();
    if (tid == 0) kept_count[row] = s_cut;
  }

  // ---- Gumbel-max over the survivors
  float best = -INFINITY, kept_mass = 0.f;
  int best_i = 0x7fffffff;
  for (int64_t i = tid; i < V; i += kFT) {
    const float x = scaled(i);
    const uint32_t k = order_key(x);
    if (!(k > kp || (k == kp && i <= cut))) continue;
    kept_mass += exp2f((x - xmax) * LFM2_LOG2E);
    uint32_t rnd[4];
    // per-row streams depend on the row's own (seed, step) only; a shared seed also counts the row
    philox((uint32_t)(i >> 2), seeds ? 0u : (uint32_t)row, 0x5eed5eedu, seeds ? 0u : (uint32_t)((uint64_t)row >> 32),
           (uint32_t)key64, (uint32_t)(key64 >> 32), rnd);
    const float score = x + gumbel(rnd[i & 3]);
    if (best_i == 0x7fffffff || score > best) { best = score; best_i = (int)i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (oi != 0x7fffffff && (best_i == 0x7fffffff || ob > best || (ob == best && oi < best_i))) { best = ob; best_i = oi; }
  }
  __syncthreads();
  kept_mass = wave_sum(kept_mass);
  if (lane == 0) { s_f[wave] = best; s_i[wave] = best_i; s_kept[wave] = kept_mass; }
  __syncthreads();
  if (tid == 0) {
    float b = s_f[0];
    int bi = s_i[0];
    for (int w = 1; w < kFT / 64; ++w)
      if (s_i[w] != 0x7fffffff && (bi == 0x7fffffff || s_f[w] > b || (s_f[w] == b && s_i[w] < bi))) { b = s_f[w]; bi = s_i[w]; }
    if (bi == 0x7fffffff) bi = 0;
    tokens[row] = bi;
    if (logprobs) logprobs[row] = Elem<T>::load(src[bi]) - (mx + logf(raw_sum));
    if (sampling_logprobs) {   // under the tempered, filtered distribution (lfm25_engine.py:1605-1608)
      float kept = 0.f;
      for (int w = 0; w < kFT / 64; ++w) kept += s_kept[w];
      sampling_logprobs[row] = (scaled(bi) - xmax) - logf(kept);
    }
  }
}

// The same sampler for rows of at most kFT * kFV logits (65536): the row is read from memory ONCE, 16 bytes per load,
// and stays in registers (64 tempered logits per thread) for every later pass.  The selections are radix selections
// on the order keys with 12-bit digits: one pass is 4096-bin histograms of counts (and of 2^40 fixed-point masses for
// the nucleus) filled with LDS atomics, then every thread looks at its four bins with the totals of the bins above
// them (a wave scan and sixteen wave totals) and the highest bin that crosses the limit wins.  Three passes fix a
// 32-bit key; after the first one only the elements of one bin take part.  Same integer decisions as the streaming
// form, so results do not depend on the order of the atomics.
// What such a kernel costs is its instruction count: every pass over 64 registers per thread is a few hundred
// instructions whether or not an element takes part.  So the elements that can still matter are copied to a list
// in LDS as soon as they are few (at most kCand), and every later step walks the list.  With top_k <= 1024 that is
// right at the start: the k-th largest of the threads' own maxima is a lower bound of the k-th largest logit (k
// threads hold a value that large) and only a handful of logits lie above it; otherwise after the top-k selection.
// A nucleus without top-k keeps working on the registers.
constexpr int kFV = 64, kBins = 4096, kCand = 2048;

struct Crossed { int bin; uint32_t count_above, count_at; unsigned long long mass_above; };

template <typename T>
__global__ void __launch_bounds__(kFT)
sample_filtered_kernel(const T* logits, int64_t* tokens, float* logprobs, float* sampling_logprobs, int32_t* kept_count, const int64_t* seeds,
                       const int64_t* steps, const float* temperatures, const int32_t* top_ks, const float* top_ps, int64_t seed,
                       int64_t step, float temperature, int top_k, float top_p, int64_t V) {
  if (temperatures) {   // per-row parameters: rows that ask for no filter (or are greedy) keep what the outputs hold
    temperature = temperatures[blockIdx.x];
    top_k = top_ks[blockIdx.x];
    top_p = top_ps[blockIdx.x];
    if (!(temperature > 0.f) || (top_k <= 0 && !(top_p < 1.0f))) return;
  }
  constexpr int EPV = 16 / sizeof(T), CHUNKS = kFV / EPV, WAVES = kFT / 64;
  __shared__ uint32_t h_cnt[kBins];
  __shared__ unsigned long long h_mass[kBins];
  __shared__ uint32_t w_cnt[WAVES];
  __shared__ unsigned long long w_mass[WAVES];
  __shared__ float s_f[WAVES], s_kept[WAVES];
  __shared__ int s_i[WAVES];
  __shared__ int s_best;
  __shared__ Crossed s_crossed;
  __shared__ unsigned long long s_total;
  __shared__ uint32_t c_key[kCand];
  __shared__ int c_col[kCand];
  __shared__ int s_candidates;
  const int64_t row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* src = logits + row * V;
  const uint64_t key64 = seeds ? row_key(seeds[row], steps[row]) : row_key(seed, step);
  const bool vector_ok = V % EPV == 0;
  // element j of a thread is column tid * EPV + (j / EPV) * kFT * EPV + j % EPV; columns beyond V hold -inf, the
  // smallest key with no mass, so only the steps that count or pick elements need to look at the column
  const int V32 = (int)V, col0 = tid * EPV;
  auto column = [&](int j) { return col0 + (j / EPV) * (kFT * EPV) + j % EPV; };

  // ---- the row, once: raw maximum and normaliser (for the returned log-probability), then the tempered logits
  float xs[kFV];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) load_columns(src, (int64_t)(c * kFT + tid) * EPV, V, vector_ok, xs + c * EPV);
  float mx = xs[0];
#pragma unroll
  for (int j = 1; j < kFV; ++j) mx = fmaxf(mx, xs[j]);
  mx = wave_max(mx);
  if (lane == 0) s_f[wave] = mx;
  __syncthreads();
  mx = s_f[0];
  for (int w = 1; w < WAVES; ++w) mx = fmaxf(mx, s_f[w]);
  __syncthreads();
  float raw_sum = 0.f;
#pragma unroll
  for (int j = 0; j < kFV; ++j) {
    raw_sum += __expf(xs[j] - mx);
    __builtin_amdgcn_sched_barrier(0);   // one element at a time: interleaved, the unrolled bodies need more registers than there are
  }
  raw_sum = wave_sum(raw_sum);
  if (lane == 0) s_f[wave] = raw_sum;
  __syncthreads();
  raw_sum = 0.f;
  for (int w = 0; w < WAVES; ++w) raw_sum += s_f[w];
  __syncthreads();
  const float xmax = mx / temperature;
  // from here on the row lives in registers as the order keys of the tempered logits: every selection compares keys,
  // and the few places that need a value turn the key back into it
  uint32_t ks[kFV];
#pragma unroll
  for (int j = 0; j < kFV; ++j) ks[j] = order_key(xs[j] / temperature);
  auto value_of = [](uint32_t k) { return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k); };
  auto mass_of = [&](float x) -> unsigned long long { return (unsigned long long)(exp2f((x - xmax) * LFM2_LOG2E) * 1099511627776.0f); };
  // A mass is recomputed wherever it is used: kept from one pass to the next, sixty-four 64-bit masses per thread
  // would not fit in registers.  The empty statement hides the value's origin from common-subexpression elimination.
  auto fresh = [](uint32_t k) { asm volatile("" : "+v"(k)); return k; };

  // One selection pass over the histograms just filled: thread t owns bins 4t .. 4t+3.  Walking from the highest
  // bin down with the running totals (count, mass) of everything above, the first bin where the limit is crossed
  // (by_mass: above + mass > mass_limit; else: above + count >= count_limit) is reported in s_crossed; bin -1: none.
  auto select = [&](bool by_mass, uint32_t count_limit, unsigned long long mass_limit, uint32_t count_base,
                    unsigned long long mass_base) {
    uint32_t cnt[4], mine_c = 0;
    unsigned long long mass[4], mine_m = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      cnt[b] = h_cnt[4 * tid + b]; mass[b] = by_mass ? h_mass[4 * tid + b] : 0ull;
      mine_c += cnt[b]; mine_m += mass[b];
    }
    uint32_t c = mine_c;
    unsigned long long m = mine_m;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {   // totals of this lane and the lanes above it in the wave
      const uint32_t oc = __shfl_down(c, o, 64);
      const unsigned long long om = __shfl_down(m, o, 64);
      if (lane + o < 64) { c += oc; m += om; }
    }
    if (lane == 0) { w_cnt[wave] = c; w_mass[wave] = m; }
    if (tid == 0) s_best = -1;
    __syncthreads();
    uint32_t above_c = count_base + c - mine_c;
    unsigned long long above_m = mass_base + m - mine_m;
    for (int w = wave + 1; w < WAVES; ++w) { above_c += w_cnt[w]; above_m += w_mass[w]; }
    Crossed found{-1, 0, 0, 0};
#pragma unroll
    for (int b = 3; b >= 0; --b) {
      if (cnt[b] == 0) continue;
      const bool crosses = by_mass ? above_m + mass[b] > mass_limit : above_c + cnt[b] >= count_limit;
      if (crosses && found.bin < 0) found = Crossed{4 * tid + b, above_c, cnt[b], above_m};
      above_c += cnt[b]; above_m += mass[b];
    }
    if (found.bin >= 0) atomicMax(&s_best, found.bin);
    __syncthreads();
    if (found.bin >= 0 && found.bin == s_best) s_crossed = found;
    if (tid == 0 && s_best < 0) s_crossed = Crossed{-1, above_c, 0, above_m};   // thread 0 ends with the totals of all bins
    __syncthreads();
  };
  auto clear_bins = [&](bool with_mass) {
#pragma unroll
    for (int b = 0; b < 4; ++b) { h_cnt[4 * tid + b] = 0; if (with_mass) h_mass[4 * tid + b] = 0; }
    __syncthreads();
  };
  constexpr int kShift[3] = {20, 8, 0};
  constexpr uint32_t kDigit[3] = {0xFFFu, 0xFFFu, 0xFFu}, kDone[3] = {0xFFF00000u, 0xFFFFFF00u, 0xFFFFFFFFu};

  // ---- the elements that can still matter, as a list in LDS once they are few: (key, column) of every logit whose
  // key is at least `floor`.  All later steps then walk the list (a few entries per thread at most) instead of the
  // 64 registers of every thread.
  bool listed = false;
  int list_size = 0;
  auto try_list = [&](uint32_t floor) {
    if (tid == 0) s_candidates = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kFV; ++j) {
      if (ks[j] >= floor && column(j) < V32) {
        const int at = atomicAdd(&s_candidates, 1);
        if (at < kCand) { c_key[at] = ks[j]; c_col[at] = column(j); }
      }
    }
    __syncthreads();
    list_size = s_candidates;
    listed = list_size <= kCand;
    __syncthreads();
  };
  // visit(key, column) for the elements with key >= at_least that this thread is responsible for; without a list
  // that includes the -inf padding beyond the row's end when at_least is below every real key
  auto for_each = [&](uint32_t at_least, auto&& visit) {
    if (listed) {
      for (int e = tid; e < list_size; e += kFT) {
        const uint32_t k = c_key[e];
        if (k >= at_least) visit(k, c_col[e]);
      }
    } else {
#pragma unroll
      for (int j = 0; j < kFV; ++j) {
        if (ks[j] >= at_least) visit(fresh(ks[j]), column(j));
        __builtin_amdgcn_sched_barrier(0);   // one element at a time: interleaved, the unrolled bodies need more registers than there are
      }
    }
  };

  // ---- top-k: key of the k-th largest tempered logit
  uint32_t key_k = 0;
  if (top_k > 0 && top_k < V) {
    // the k-th largest of the keys that `keys` visits
    auto kth_largest = [&](auto&& keys) -> uint32_t {
      uint32_t prefix = 0, mask = 0, remaining = (uint32_t)top_k;
      for (int pass = 0; pass < 3; ++pass) {
        clear_bins(false);
        keys([&](uint32_t k, int) {
          if ((k & mask) == prefix) atomicAdd(&h_cnt[(k >> kShift[pass]) & kDigit[pass]], 1u);
        });
        __syncthreads();
        select(false, remaining, 0ull, 0u, 0ull);
        prefix |= (uint32_t)s_crossed.bin << kShift[pass];
        mask = kDone[pass];
        remaining -= s_crossed.count_above;
        __syncthreads();
      }
      return prefix;
    };
    uint32_t floor_key = 0;
    if (top_k <= kFT) {
      // k threads hold a logit at least as large as the k-th largest of the threads' maxima: a lower bound of the
      // k-th largest logit, above which only a handful of logits lie
      uint32_t top = ks[0];
#pragma unroll
      for (int j = 1; j < kFV; ++j) top = top > ks[j] ? top : ks[j];
      floor_key = kth_largest([&](auto&& visit) { visit(top, 0); });
      try_list(floor_key);
    }
    key_k = kth_largest([&](auto&& visit) { for_each(floor_key, visit); });
    if (!listed) try_list(key_k);
  }

  // ---- nucleus: walk keys downward until the inclusive cumulative mass exceeds top_p * Z
  uint32_t kp = key_k;
  int ties_kept = kNoIndex, ties_total = 0;
  uint32_t cnt_above = 0;
  bool crossed = false;
  if (top_p < 1.0f) {
    unsigned long long z = 0;
    for_each(key_k, [&](uint32_t k, int) { z += mass_of(value_of(k)); });
    if (tid == 0) s_total = 0;
    __syncthreads();
    if (z) atomicAdd(&s_total, z);
    __syncthreads();
    const unsigned long long limit = (unsigned long long)((double)top_p * (double)s_total);
    uint32_t prefix = 0, mask = 0;
    unsigned long long mass_above = 0;
    crossed = true;
    for (int pass = 0; pass < 3 && crossed; ++pass) {
      clear_bins(true);
      for_each(key_k, [&](uint32_t k, int) {
        if ((k & mask) == prefix) {
          const uint32_t bin = (k >> kShift[pass]) & kDigit[pass];
          atomicAdd(&h_cnt[bin], 1u);
          atomicAdd(&h_mass[bin], mass_of(value_of(k)));
        }
      });
      __syncthreads();
      select(true, 0u, limit, cnt_above, mass_above);
      crossed = s_crossed.bin >= 0;
      cnt_above = s_crossed.count_above;
      mass_above = s_crossed.mass_above;
      if (crossed) {
        prefix |= (uint32_t)s_crossed.bin << kShift[pass];
        mask = kDone[pass];
        ties_total = (int)s_crossed.count_at;
      }
      __syncthreads();
    }
    if (crossed) {
      kp = prefix;
      const unsigned long long w = mass_of(value_of(kp));
      unsigned long long fit = w ? (limit - mass_above) / w : 0;
      if (fit >= (unsigned long long)ties_total) fit = ties_total;
      ties_kept = (int)fit;
      if (cnt_above == 0 && ties_kept == 0) ties_kept = 1;  // rank 0 always survives
    }
  }

  // Number of elements of the row (padding excluded) with key >= at_least that a predicate holds for.
  auto block_count = [&](uint32_t at_least, auto&& holds) -> int {
    int c = 0;
    for_each(at_least, [&](uint32_t k, int col) { c += (col < V32 && holds(k, col)) ? 1 : 0; });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
    __syncthreads();
    if (lane == 0) s_i[wave] = c;
    __syncthreads();
    int total = 0;
    for (int w = 0; w < WAVES; ++w) total += s_i[w];
    return total;
  };

  // ---- when only some of the ties at kp survive, keep the lowest-index ones: find the cut column (rare: two
  // equal logits exactly on the nucleus boundary), by bisection on the column
  int cut = kNoIndex;
  if (crossed) {
    if (ties_kept == 0) {
      cut = -1;
    } else if (ties_kept < ties_total) {
      int lo = 0, hi = V32 - 1;
      while (lo < hi) {
        const int mid = lo + (hi - lo) / 2;
        if (block_count(kp, [&](uint32_t k, int col) { return k == kp && col <= mid; }) >= ties_kept) hi = mid;
        else lo = mid + 1;
      }
      cut = lo;
    }
    if (kept_count && tid == 0) kept_count[row] = (int)cnt_above + ties_kept;
  } else if (kept_count) {
    const int kept = block_count(kp, [&](uint32_t, int) { return true; });
    if (tid == 0) kept_count[row] = kept;
  }

  // ---- Gumbel-max over the survivors
  float best = -INFINITY, kept_mass = 0.f;
  int best_i = kNoIndex;
  auto consider = [&](float x, int i) {
    kept_mass += exp2f((x - xmax) * LFM2_LOG2E);
    uint32_t rnd[4];
    // per-row streams depend on the row's own (seed, step) only; a shared seed also counts the row
    philox((uint32_t)(i >> 2), seeds ? 0u : (uint32_t)row, 0x5eed5eedu, seeds ? 0u : (uint32_t)((uint64_t)row >> 32),
           (uint32_t)key64, (uint32_t)(key64 >> 32), rnd);
    const float score = x + gumbel(rnd[i & 3]);
    if (best_i == kNoIndex || score > best || (score == best && i < best_i)) { best = score; best_i = i; }
  };
  if (listed) {
    for (int e = tid; e < list_size; e += kFT) {
      const uint32_t k = c_key[e];
      const int i = c_col[e];
      if (k > kp || (k == kp && i <= cut)) consider(value_of(k), i);
    }
  } else {
    // a thread's survivors as a bit mask first, then a loop over the set bits that reads the survivor's logit again:
    // registers cannot be indexed by a loop variable, and sixty-four unrolled Philox blocks would not fit in them
    uint64_t survivors = 0;
#pragma unroll
    for (int j = 0; j < kFV; ++j) {
      const uint32_t k = ks[j];
      if (column(j) < V32 && (k > kp || (k == kp && column(j) <= cut))) survivors |= 1ull << j;
    }
    while (survivors) {
      const int j = __builtin_ctzll(survivors);
      survivors &= survivors - 1;
      const int i = col0 + (j / EPV) * (kFT * EPV) + j % EPV;
      consider(Elem<T>::load(src[i]) / temperature, i);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (oi != kNoIndex && (best_i == kNoIndex || ob > best || (ob == best && oi < best_i))) { best = ob; best_i = oi; }
  }
  __syncthreads();
  kept_mass = wave_sum(kept_mass);
  if (lane == 0) { s_f[wave] = best; s_i[wave] = best_i; s_kept[wave] = kept_mass; }
  __syncthreads();
  if (tid == 0) {
    float b = s_f[0];
    int bi = s_i[0];
    for (int w = 1; w < WAVES; ++w)
      if (s_i[w] != kNoIndex && (bi == kNoIndex || s_f[w] > b || (s_f[w] == b && s_i[w] < bi))) { b = s_f[w]; bi = s_i[w]; }
    if (bi == kNoIndex) bi = 0;
    tokens[row] = bi;
    const float chosen = Elem<T>::load(src[bi]);
    if (logprobs) logprobs[row] = chosen - (mx + logf(raw_sum));
    if (sampling_logprobs) {   // under the tempered, filtered distribution (lfm25_engine.py:1605-1608)
      float kept = 0.f;
      for (int w = 0; w < WAVES; ++w) kept += s_kept[w];
      sampling_logprobs[row] = (chosen / temperature - xmax) - logf(kept);
    }
  }
}

// ------------------------------------------------------------------------------------ small row kernels
template <typename T>
__global__ void head_logprobs_kernel(float* out, const T* logits, const int64_t* selected, const float* logprobs,
                                     const T* values, int64_t V, int K) {
  const int64_t row = blockIdx.x;
  const float log_z = Elem<T>::load(logits[row * V + selected[row]]) - logprobs[row];
  for (int c = threadIdx.x; c < K; c += blockDim.x) out[row * K + c] = Elem<T>::load(values[row * K + c]) - log_z;
}

__global__ void record_sample_kernel(const int64_t* sampled, const float* logp, int64_t* tokens, float* logprobs,
                                     int32_t* lengths, const int32_t* limits, int8_t* reasons, uint8_t* alive,
                                     uint8_t* pending, int64_t* input, int64_t* stop_states, const int64_t* stop_offsets,
                                     const int32_t* stop_table, const uint8_t* ignore_eos, int64_t* rng_positions,
                                     int64_t eos, int64_t V, int64_t cap, int64_t B) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= B || !alive[row]) return;
  const int64_t token = sampled[row];
  const int32_t length = lengths[row];
  tokens[row * cap + length] = token;
  logprobs[row * cap + length] = logp[row];
  const int32_t value = stop_table[stop_offsets[row] + stop_states[row] * V + token];
  stop_states[row] = value & 65535;
  int8_t reason = 0;
  if (token == eos && !ignore_eos[row]) reason = 1;
  else if (value >= 65536) reason = 2;
  else if (length + 1 >= limits[row]) reason = 3;
  lengths[row] = length + 1;
  rng_positions[row] += 1;
  reasons[row] = reason;
  alive[row] = reason == 0;
  pending[row] = reason == 0;
  input[row] = token;
}

// Per-row state of newly admitted requests (the state tensors of lfm25_session.py:150-165, set per request at
// :244-262), all columns in one launch.  A spec is eight int64 words: slot, length limit, seed, emitted-token count
// the random stream continues from, stop-automaton state, offset of the request's automaton in the flat stop table,
// flags (bit 0: ignore EOS; bits 8..39: top_k), and temperature | top_p as two float bit patterns (low, high word).
__global__ void configure_rows_kernel(const int64_t* specs, int64_t count, int64_t rows, int32_t* lengths, int32_t* limits,
                                      int8_t* reasons, uint8_t* alive, uint8_t* pending, uint8_t* ignore_eos,
                                      float* temperatures, int32_t* top_ks, float* top_ps, int64_t* seeds,
                                      int64_t* rng_positions, int64_t* stop_states, int64_t* stop_offsets) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const int64_t* spec = specs + i * 8;
  const int64_t slot = spec[0];
  if (slot < 0 || slot >= rows) return;
  lengths[slot] = 0;
  reasons[slot] = 0;
  alive[slot] = 1;
  pending[slot] = 0;
  limits[slot] = (int32_t)spec[1];
  seeds[slot] = spec[2];
  rng_positions[slot] = spec[3];
  stop_states[slot] = spec[4];
  stop_offsets[slot] = spec[5];
  ignore_eos[slot] = (uint8_t)(spec[6] & 1);
  top_ks[slot] = (int32_t)((spec[6] >> 8) & 0xffffffffll);
  temperatures[slot] = __uint_as_float((uint32_t)(spec[7] & 0xffffffffll));
  top_ps[slot] = __uint_as_float((uint32_t)((uint64_t)spec[7] >> 32));
}

__global__ void record_head_kernel(const int64_t* ids, const float* probs, int32_t* out_ids, float* out_probs,
                                   const int32_t* lengths, const uint8_t* alive, int K, int64_t cap) {
  const int64_t row = blockIdx.x;
  if (!alive[row]) return;
  const int64_t base = (row * cap + lengths[row]) * K;
  for (int c = threadIdx.x; c < K; c += blockDim.x) {
    out_ids[base + c] = (int32_t)ids[row * K + c];
    out_probs[base + c] = probs[row * K + c];
  }
}

__global__ void gather_inputs_kernel(int64_t* tokens, int32_t* positions, uint8_t* mask, const int64_t* input,
                                     const int32_t* lengths, const uint8_t* active, const int32_t* slots, int64_t B) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= B) return;
  const int32_t slot = slots[row];
  const bool valid = slot >= 0;
  tokens[row] = valid ? input[slot] : 0;
  positions[row] = valid ? lengths[slot] : 0;
  mask[row] = valid ? active[slot] : 0;
}

template <typename T>
__global__ void __launch_bounds__(256)
scatter_logits_kernel(T* saved, const T* logits, const int32_t* slots, const uint8_t* active, int64_t V) {
  const int64_t row = blockIdx.y;
  if (!active[row]) return;
  const int64_t slot = slots ? slots[row] : row;
  if (slot < 0) return;
  constexpr int N = 16 / sizeof(T);
  typedef T vec __attribute__((ext_vector_type(N)));
  const int64_t col = ((int64_t)blockIdx.x * 256 + threadIdx.x) * N;
  if (V % N == 0) {
    if (col < V) *reinterpret_cast<vec*>(saved + slot * V + col) = *reinterpret_cast<const vec*>(logits + row * V + col);
  } else {
    for (int e = 0; e < N; ++e)
      if (col + e < V) saved[slot * V + col + e] = logits[row * V + col + e];
  }
}

__global__ void advance_positions_kernel(int32_t* lengths, const int32_t* positions, const int32_t* slots,
                                         const uint8_t* active, int64_t B) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= B) return;
  const int32_t slot = slots ? slots[row] : (int32_t)row;
  if (slot >= 0 && (active == nullptr || active[row])) lengths[slot] = positions[row] + 1;
}

}  // namespace

extern "C" int lfm2_sample(int64_t* tokens, float* logprobs, float* sampling_logprobs, const void* logits, float* scratch,
                           const int64_t* seeds, const int64_t* steps, const float* temperatures, int64_t seed, int64_t step,
                           float temperature, int64_t B, int64_t V, int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0, "sample: empty logits");
  LFM2_REQUIRE(B <= 65535, "sample: more than 65535 rows");
  LFM2_REQUIRE(temperature >= 0.f, "sample: negative temperature");
  LFM2_REQUIRE((seeds == nullptr) == (steps == nullptr) && (seeds == nullptr) == (temperatures == nullptr),
               "sample: seeds, steps and temperatures go together");
  LFM2_REQUIRE(V <= 256ll * kTile, "sample: vocabulary above 1048576");
  const int parts = ceil_div(V, kTile);
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, "sample",
                 hipLaunchKernelGGL(sample_partial_kernel<T>, dim3(parts, B), dim3(256), 0, s, (const T*)logits, scratch,
                                    temperatures, temperature, V, parts);
                 hipLaunchKernelGGL(sample_finish_kernel<T>, dim3(B), dim3(256), 0, s, (const T*)logits, scratch, tokens,
                                    logprobs, sampling_logprobs, seeds, steps, temperatures, seed, step, temperature, V, parts,
                                    RecordArgs{}));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_sample_record(int64_t* sampled, float* logp, const void* logits, float* scratch, const int64_t* seeds,
                                  const int64_t* steps, const float* temperatures, int64_t* tokens, float* logprobs,
                                  int32_t* lengths, const int32_t* limits, int8_t* reasons, uint8_t* alive, uint8_t* pending,
                                  int64_t* input, int64_t* stop_states, const int64_t* stop_offsets,
                                  const int32_t* stop_table, const uint8_t* ignore_eos, int64_t* rng_positions, int64_t eos,
                                  int64_t cap, int64_t B, int64_t V, int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0 && cap > 0, "sample_record: bad shape");
  LFM2_REQUIRE(B <= 65535, "sample_record: more than 65535 rows");
  LFM2_REQUIRE(V <= 256ll * kTile, "sample_record: vocabulary above 1048576");
  LFM2_REQUIRE(sampled && logp && logits && scratch && seeds && steps && temperatures && tokens && logprobs && lengths &&
               limits && reasons && alive && pending && input && stop_states && stop_offsets && stop_table && ignore_eos &&
               rng_positions, "sample_record: a required pointer is null");
  const int parts = ceil_div(V, kTile);
  const RecordArgs record{tokens, logprobs, lengths, limits, reasons, alive, pending, input, stop_states, stop_offsets,
                          stop_table, ignore_eos, rng_positions, eos, V, cap};
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, "sample_record",
                 hipLaunchKernelGGL(sample_partial_kernel<T>, dim3(parts, B), dim3(256), 0, s, (const T*)logits, scratch,
                                    temperatures, 0.f, V, parts);
                 hipLaunchKernelGGL(sample_finish_kernel<T>, dim3(B), dim3(256), 0, s, (const T*)logits, scratch, sampled, logp,
                                    (float*)nullptr, seeds, steps, temperatures, 0, 0, 0.f, V, parts, record));
  LFM2_LAUNCH_CHECK();
}

// ---- the sampler for callers that cannot allocate: the tile statistics live in a file-scope device array ----------
// One array per GPU (each device that loads this code object holds its own copy at its own address, until the process
// ends).  Host code never passes the array's name to a kernel: the name is a host-side stand-in, the device address
// comes from hipGetSymbolAddress, looked up once per device with that device current.
constexpr int64_t kStaticTiles = 16384;                       // rows x 4096-column tiles one call may use
static __device__ __align__(256) float scratch[kStaticTiles * 4];   // 256 KiB
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
float* g_static_scratch[kMaxDevices] = {};
// Device address of `scratch` on the current device, or nullptr with the error text set.
float* static_scratch() {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    lfm2_set_error("sample_static: no current device, or a device index above %d", kMaxDevices - 1);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_scratch[device] == nullptr) {
    float* ptr = nullptr;
    const hipError_t status = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (status != hipSuccess || ptr == nullptr) {
      lfm2_set_error("sample_static: hipGetSymbolAddress failed: %s", hipGetErrorString(status));
      return nullptr;
    }
    g_static_scratch[device] = ptr;
  }
  return g_static_scratch[device];
}
}  // namespace

extern "C" int lfm2_sample_static(int64_t* tokens, float* logprobs, const void* logits, const int64_t* seeds,
                                  const int64_t* steps, const float* temperatures, int64_t seed, int64_t step,
                                  float temperature, int64_t B, int64_t V, int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0, "sample_static: empty logits");
  const int64_t tiles = B * ((V + kTile - 1) / kTile);
  LFM2_REQUIRE(tiles <= kStaticTiles,
               "sample_static: %ld rows x %ld tiles of 4096 columns = %ld tile records, the static scratch holds %ld "
               "(use lfm2_sample with a caller-provided scratch)", (long)B, (long)((V + kTile - 1) / kTile), (long)tiles,
               (long)kStaticTiles);
  float* ptr = static_scratch();
  if (ptr == nullptr) return LFM2_ERR_LAUNCH;
  // pass 1 writes every record pass 2 reads, so nothing of the previous call's contents needs clearing
  return lfm2_sample(tokens, logprobs, nullptr, logits, ptr, seeds, steps, temperatures, seed, step, temperature, B, V, dtype, stream);
}

extern "C" int lfm2_sample_filtered(int64_t* tokens, float* logprobs, float* sampling_logprobs, int32_t* kept_count, const void* logits,
                                    const int64_t* seeds, const int64_t* steps, const float* temperatures,
                                    const int32_t* top_ks, const float* top_ps, int64_t seed, int64_t step,
                                    float temperature, int top_k, float top_p, int64_t B, int64_t V, int dtype,
                                    void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0, "sample_filtered: empty logits");
  LFM2_REQUIRE((temperatures == nullptr) == (top_ks == nullptr) && (temperatures == nullptr) == (top_ps == nullptr),
               "sample_filtered: per-row temperatures, top_ks and top_ps go together");
  if (temperatures == nullptr) {
    LFM2_REQUIRE(temperature > 0.f, "sample_filtered: temperature must be positive");
    LFM2_REQUIRE(top_k >= 0 && top_p > 0.f && top_p <= 1.f, "sample_filtered: top_k >= 0 and top_p in (0,1] required");
  }
  LFM2_REQUIRE(V < (1ll << 31), "sample_filtered: vocabulary too large");
  LFM2_REQUIRE((seeds == nullptr) == (steps == nullptr), "sample_filtered: seeds and steps go together");
  DISPATCH_DTYPE(dtype, "sample_filtered",
                 if (V <= (int64_t)kFT * kFV)
                   hipLaunchKernelGGL(sample_filtered_kernel<T>, dim3(B), dim3(kFT), 0, (hipStream_t)stream, (const T*)logits,
                                      tokens, logprobs, sampling_logprobs, kept_count, seeds, steps, temperatures, top_ks, top_ps,
                                      seed, step, temperature, top_k, top_p, V);
                 else
                   hipLaunchKernelGGL(sample_filtered_stream_kernel<T>, dim3(B), dim3(kFT), 0, (hipStream_t)stream,
                                      (const T*)logits, tokens, logprobs, sampling_logprobs, kept_count, seeds, steps, temperatures,
                                      top_ks, top_ps, seed, step, temperature, top_k, top_p, V));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_configure_rows(const int64_t* specs, int64_t count, int64_t rows, int32_t* lengths, int32_t* limits,
                                   int8_t* reasons, uint8_t* alive, uint8_t* pending, uint8_t* ignore_eos,
                                   float* temperatures, int32_t* top_ks, float* top_ps, int64_t* seeds,
                                   int64_t* rng_positions, int64_t* stop_states, int64_t* stop_offsets, void* stream) {
  LFM2_REQUIRE(count > 0 && rows > 0, "configure_rows: empty request list");
  LFM2_REQUIRE(specs && lengths && limits && reasons && alive && pending && ignore_eos && temperatures && top_ks && top_ps &&
               seeds && rng_positions && stop_states && stop_offsets, "configure_rows: a state column is missing");
  hipLaunchKernelGGL(configure_rows_kernel, dim3(ceil_div(count, 128)), dim3(128), 0, (hipStream_t)stream, specs, count, rows,
                     lengths, limits, reasons, alive, pending, ignore_eos, temperatures, top_ks, top_ps, seeds, rng_positions,
                     stop_states, stop_offsets);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_head_logprobs(float* out, const void* logits, const int64_t* selected, const float* logprobs,
                                  const void* values, int64_t B, int64_t V, int K, int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0 && K > 0 && K <= 128, "head_logprobs: bad shape");
  DISPATCH_DTYPE(dtype, "head_logprobs",
                 hipLaunchKernelGGL(head_logprobs_kernel<T>, dim3(B), dim3(128), 0, (hipStream_t)stream, out, (const T*)logits,
                                    selected, logprobs, (const T*)values, V, K));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_record_sample(const int64_t* sampled, const float* logp, int64_t* tokens, float* logprobs,
                                  int32_t* lengths, const int32_t* limits, int8_t* reasons, uint8_t* alive,
                                  uint8_t* pending, int64_t* input, int64_t* stop_states, const int64_t* stop_offsets,
                                  const int32_t* stop_table, const uint8_t* ignore_eos, int64_t* rng_positions,
                                  int64_t eos, int64_t V, int64_t cap, int64_t B, void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0 && cap > 0, "record_sample: bad shape");
  hipLaunchKernelGGL(record_sample_kernel, dim3(ceil_div(B, 128)), dim3(128), 0, (hipStream_t)stream, sampled, logp, tokens,
                     logprobs, lengths, limits, reasons, alive, pending, input, stop_states, stop_offsets, stop_table,
                     ignore_eos, rng_positions, eos, V, cap, B);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_record_head(const int64_t* ids, const float* probs, int32_t* out_ids, float* out_probs,
                                const int32_t* lengths, const uint8_t* alive, int K, int64_t cap, int64_t B, void* stream) {
  LFM2_REQUIRE(B > 0 && K > 0 && cap > 0, "record_head: bad shape");
  hipLaunchKernelGGL(record_head_kernel, dim3(B), dim3(128), 0, (hipStream_t)stream, ids, probs, out_ids, out_probs, lengths,
                     alive, K, cap);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_gather_inputs(int64_t* tokens, int32_t* positions, uint8_t* mask, const int64_t* input,
                                  const int32_t* lengths, const uint8_t* active, const int32_t* slots, int64_t B,
                                  void* stream) {
  LFM2_REQUIRE(B > 0, "gather_inputs: empty batch");
  hipLaunchKernelGGL(gather_inputs_kernel, dim3(ceil_div(B, 128)), dim3(128), 0, (hipStream_t)stream, tokens, positions, mask,
                     input, lengths, active, slots, B);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_scatter_logits(void* saved, const void* logits, const int32_t* slots, const uint8_t* active, int64_t B,
                                   int64_t V, int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && V > 0 && active, "scatter_logits: bad arguments");
  LFM2_REQUIRE(B <= 65535, "scatter_logits: more than 65535 rows");
  DISPATCH_DTYPE(dtype, "scatter_logits",
                 hipLaunchKernelGGL(scatter_logits_kernel<T>, dim3(ceil_div(V, 256 * (16 / sizeof(T))), B), dim3(256), 0,
                                    (hipStream_t)stream, (T*)saved, (const T*)logits, slots, active, V));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_advance_positions(int32_t* lengths, const int32_t* positions, const int32_t* slots,
                                      const uint8_t* active, int64_t B, void* stream) {
  LFM2_REQUIRE(B > 0, "advance_positions: empty batch");
  hipLaunchKernelGGL(advance_positions_kernel, dim3(ceil_div(B, 128)), dim3(128), 0, (hipStream_t)stream, lengths, positions,
                     slots, active, B);
  LFM2_LAUNCH_CHECK();
}
