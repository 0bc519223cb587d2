// Row-wise fused kernels of the LFM2 decode step: embedding gather, residual+RMSNorm (with an
// optional per-token e4m3 epilogue), SwiGLU (same), row quantisation, the gated short-conv
// rolling-state update, QK-norm + RoPE + QKV split, and the packed-prefill short conv.
//
// All of them are HBM/launch bound: one 256-thread workgroup owns one row (or one row x 2048
// column slab), reads it once with 16-byte loads, keeps it in registers across the two
// reductions (sum of squares, abs-max) and writes each output once.
#include <stdarg.h>
#include <stdio.h>

#include <type_traits>

#include "lfm2_common.h"

// ------------------------------------------------------------------------------------ errors
static thread_local char g_error[512] = "";
void lfm2_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
extern "C" const char* lfm2_last_error(void) { return g_error; }
extern "C" int lfm2_abi_version(void) { return 1; }

#define DISPATCH_DTYPE(dtype, ...)                                         \
  switch (dtype) {                                                         \
    case LFM2_DTYPE_BF16: { typedef __bf16 T; __VA_ARGS__; } break;        \
    case LFM2_DTYPE_F16: { typedef _Float16 T; __VA_ARGS__; } break;       \
    case LFM2_DTYPE_F32: { typedef float T; __VA_ARGS__; } break;          \
    default: LFM2_FAIL(LFM2_ERR_ARGUMENT, "unknown dtype %d", dtype);      \
  }

#ifndef ROW_THREADS
#define ROW_THREADS 512
#endif
constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;
// The per-row kernels (RMSNorm, row quantisation): threads per row
constexpr int kRowThreads = ROW_THREADS;
constexpr int kRowWaves = kRowThreads / 64;

template <typename T> struct Vec {
  static constexpr int N = 16 / sizeof(T);
  typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};

template <typename T> __device__ __forceinline__ void load_vec(const T* p, float* out) {
  typename Vec<T>::type v = *reinterpret_cast<const typename Vec<T>::type*>(p);
#pragma unroll
  for (int i = 0; i < Vec<T>::N; ++i) out[i] = Elem<T>::load(v[i]);
}
template <typename T> __device__ __forceinline__ void store_vec(T* p, const float* in) {
  typename Vec<T>::type v;
#pragma unroll
  for (int i = 0; i < Vec<T>::N; ++i) v[i] = Elem<T>::store(in[i]);
  *reinterpret_cast<typename Vec<T>::type*>(p) = v;
}
// N consecutive e4m3 codes (N = 4 or 8).
template <int N> __device__ __forceinline__ void store_e4m3(uint8_t* p, const float* v, float scale) {
  int w0 = pack_e4m3x4(v[0] / scale, v[1] / scale, v[2] / scale, v[3] / scale);
  if (N == 4) {
    *reinterpret_cast<int*>(p) = w0;
  } else {
    int w1 = pack_e4m3x4(v[4] / scale, v[5] / scale, v[6] / scale, v[7] / scale);
    i32x2 w = {w0, w1};
    *reinterpret_cast<i32x2*>(p) = w;
  }
}

// ------------------------------------------------------------------------------------ embedding
template <typename T>
__global__ void __launch_bounds__(kThreads) embedding_kernel(T* out, const T* table, const int64_t* tokens,
                                                            int64_t H, int64_t V) {
  const int64_t row = blockIdx.x;
  int64_t tok = tokens[row];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  const T* src = table + tok * H;
  T* dst = out + row * H;
  constexpr int N = Vec<T>::N;
  if (H % N == 0) {
    for (int64_t i = threadIdx.x * N; i < H; i += kThreads * N)
      *reinterpret_cast<typename Vec<T>::type*>(dst + i) = *reinterpret_cast<const typename Vec<T>::type*>(src + i);
  } else {
    for (int64_t i = threadIdx.x; i < H; i += kThreads) dst[i] = src[i];
  }
}

extern "C" int lfm2_embedding(void* out, const void* table, const int64_t* tokens, int64_t M, int64_t H,
                              int64_t V, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0 && V > 0, "embedding: empty shape");
  DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(embedding_kernel<T>, dim3(M), dim3(kThreads), 0, (hipStream_t)stream,
                                           (T*)out, (const T*)table, tokens, H, V));
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ RMSNorm (+e4m3)
// NV = 16-byte vectors per thread held in registers; NV == 0 selects the scalar path that
// recomputes values from global memory in each pass (any H).
// With `split.partial` set the input row is not read from `x` but rebuilt from split-K partial products of an FP8
// projection, sum over splits in split order, times the row's activation scale, times the column's weight scale,
// rounded to T: the value the projection's own reduce pass would have stored.
struct SplitInput {
  const float* partial;   // [splits, M, H] or NULL
  const float* a_scales;  // [M]
  const float* w_scales;  // [H]
  int64_t stride;         // M * H
  int splits;
  // With `tokens` set (no residual) `x` is an embedding table [vocab, H]: the row's input is the table row of its token
  // (ids clamped into the table like lfm2_embedding), and that row is also written to `summed`, the residual stream.
  const int64_t* tokens = nullptr;
  int64_t vocab = 0;
};

template <typename T, int NV, bool ADD, bool FP8>
__global__ void __launch_bounds__(kRowThreads)
rms_norm_kernel(T* out, uint8_t* q, float* scales, T* summed, const T* x, const T* w, const T* res, int64_t H,
                float eps, SplitInput split) {
  __shared__ float red[kRowWaves];
  const int64_t row = blockIdx.x;
  constexpr int N = Vec<T>::N;
  const bool gather = !ADD && split.tokens != nullptr;
  if (gather) {
    int64_t tok = split.tokens[row];
    tok = tok < 0 ? 0 : (tok >= split.vocab ? split.vocab - 1 : tok);
    x += tok * H;
    summed += row * H;
  } else {
    x += row * H;
  }
  if (ADD) { res += row * H; summed += row * H; }
  if (FP8) q += row * H; else out += row * H;

  if constexpr (NV > 0) {
    float v[NV][N], g[NV][N];
    float ss = 0.f;
    // Every load of the row is issued before anything waits: the residual, the norm weights, the scales, and the fp32
    // planes of a product left as partial sums, whose count is spelled out for 1, 2 and 4 planes (a loop with a count
    // only known at run time waits for each plane before it asks for the next: one more memory round trip per plane,
    // in a kernel that is little else).  The planes are added in their order either way.
    const float sa = (split.partial && split.a_scales) ? split.a_scales[row] : 1.0f;   // a bf16 product has no scales
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t i = (int64_t)(j * kRowThreads + threadIdx.x) * N;
      if (i < H) {
        float r[N];
        if (ADD) load_vec<T>(res + i, r);
        load_vec<T>(w + i, g[j]);
        if (split.partial) {
          float cs[N];
          if (split.w_scales) {
#pragma unroll
            for (int e = 0; e < N; ++e) cs[e] = split.w_scales[i + e];
          }
          const float* p = split.partial + row * H + i;
          auto planes = [&](auto count) {
            constexpr int SP = decltype(count)::value;
            float part[SP][N];
#pragma unroll
            for (int sp = 0; sp < SP; ++sp)
#pragma unroll
              for (int e = 0; e < N; ++e) part[sp][e] = p[sp * split.stride + e];
#pragma unroll
            for (int e = 0; e < N; ++e) v[j][e] = 0.f;
#pragma unroll
            for (int sp = 0; sp < SP; ++sp)
#pragma unroll
              for (int e = 0; e < N; ++e) v[j][e] += part[sp][e];
          };
          if (split.splits == 1) planes(std::integral_constant<int, 1>{});
          else if (split.splits == 2) planes(std::integral_constant<int, 2>{});
          else if (split.splits == 4) planes(std::integral_constant<int, 4>{});
          else {
#pragma unroll
            for (int e = 0; e < N; ++e) v[j][e] = 0.f;
            for (int sp = 0; sp < split.splits; ++sp)
#pragma unroll
              for (int e = 0; e < N; ++e) v[j][e] += p[sp * split.stride + e];
          }
#pragma unroll
          for (int e = 0; e < N; ++e) v[j][e] = round_to<T>(split.w_scales ? (v[j][e] * sa) * cs[e] : v[j][e]);
        } else {
          load_vec<T>(x + i, v[j]);
          if (gather) store_vec<T>(summed + i, v[j]);
        }
        if (ADD) {
#pragma unroll
          for (int e = 0; e < N; ++e) v[j][e] = round_to<T>(v[j][e] + r[e]);
          store_vec<T>(summed + i, v[j]);
        }
#pragma unroll
        for (int e = 0; e < N; ++e) ss += v[j][e] * v[j][e];
      }
    }
    ss = block_sum<kRowWaves>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t i = (int64_t)(j * kRowThreads + threadIdx.x) * N;
      if (i < H) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
          v[j][e] = round_to<T>(v[j][e] * rstd) * g[j][e];
          if (FP8) { v[j][e] = round_to<T>(v[j][e]); amax = fmaxf(amax, fabsf(v[j][e])); }
        }
        if (!FP8) store_vec<T>(out + i, v[j]);
      }
    }
    if (FP8) {
      amax = block_max<kRowWaves>(amax, red);
      const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
      if (threadIdx.x == 0) scales[row] = scale;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int64_t i = (int64_t)(j * kRowThreads + threadIdx.x) * N;
        if (i < H) store_e4m3<N>(q + i, v[j], scale);
      }
    }
  } else {
    auto value = [&](int64_t i) {
      float a = Elem<T>::load(x[i]);
      if (ADD) a = round_to<T>(a + Elem<T>::load(res[i]));
      return a;
    };
    float ss = 0.f;
    for (int64_t i = threadIdx.x; i < H; i += kRowThreads) {
      const float a = value(i);
      if (ADD || gather) summed[i] = Elem<T>::store(a);
      ss += a * a;
    }
    ss = block_sum<kRowWaves>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    auto normed = [&](int64_t i) {
      float n = round_to<T>(value(i) * rstd) * Elem<T>::load(w[i]);
      return FP8 ? round_to<T>(n) : n;
    };
    if (!FP8) {
      for (int64_t i = threadIdx.x; i < H; i += kRowThreads) out[i] = Elem<T>::store(normed(i));
    } else {
      float amax = 0.f;
      for (int64_t i = threadIdx.x; i < H; i += kRowThreads) amax = fmaxf(amax, fabsf(normed(i)));
      amax = block_max<kRowWaves>(amax, red);
      const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
      if (threadIdx.x == 0) scales[row] = scale;
      for (int64_t i = threadIdx.x; i < H; i += kRowThreads) q[i] = to_e4m3(normed(i) / scale);
    }
  }
}

// Smallest register tile that covers a row of `width` elements, 0 when it must take the scalar path.
template <typename T> static int pick_nv(int64_t width) {
  constexpr int N = 16 / sizeof(T);
  if (width % N != 0) return 0;
  for (int nv = 1; nv <= 16; nv *= 2)
    if ((int64_t)nv * kRowThreads * N >= width) return nv;
  return 0;
}

#define LAUNCH_NV(nv, KERNEL_EXPR_1, KERNEL_EXPR_2, KERNEL_EXPR_4, KERNEL_EXPR_8, KERNEL_EXPR_16, KERNEL_EXPR_0) \
  switch (nv) {                                                                                                  \
    case 1: KERNEL_EXPR_1; break;                                                                                \
    case 2: KERNEL_EXPR_2; break;                                                                                \
    case 4: KERNEL_EXPR_4; break;                                                                                \
    case 8: KERNEL_EXPR_8; break;                                                                                \
    case 16: KERNEL_EXPR_16; break;                                                                              \
    default: KERNEL_EXPR_0; break;                                                                               \
  }

template <typename T, bool ADD, bool FP8>
static void launch_rms(void* out, uint8_t* q, float* scales, void* summed, const void* x, const void* w,
                       const void* res, int64_t M, int64_t H, float eps, hipStream_t s,
                       SplitInput split = SplitInput{nullptr, nullptr, nullptr, 0, 0}) {
  const int nv = pick_nv<T>(H);
#define RMS_(NVV)                                                                                            \
  hipLaunchKernelGGL((rms_norm_kernel<T, NVV, ADD, FP8>), dim3(M), dim3(kRowThreads), 0, s, (T*)out, q, scales, \
                     (T*)summed, (const T*)x, (const T*)w, (const T*)res, H, eps, split)
  LAUNCH_NV(nv, RMS_(1), RMS_(2), RMS_(4), RMS_(8), RMS_(16), RMS_(0));
#undef RMS_
}

extern "C" int lfm2_rms_norm(void* out, void* summed, const void* x, const void* weight, const void* residual,
                             int64_t M, int64_t H, float eps, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0, "rms_norm: empty shape");
  LFM2_REQUIRE(residual == nullptr || summed != nullptr, "rms_norm: residual given without a summed output");
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, if (residual) launch_rms<T, true, false>(out, nullptr, nullptr, summed, x, weight, residual, M, H, eps, s);
                 else launch_rms<T, false, false>(out, nullptr, nullptr, nullptr, x, weight, nullptr, M, H, eps, s));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_rms_norm_fp8(uint8_t* q, float* scales, void* summed, const void* x, const void* weight,
                                 const void* residual, int64_t M, int64_t H, float eps, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0, "rms_norm_fp8: empty shape");
  LFM2_REQUIRE(residual == nullptr || summed != nullptr, "rms_norm_fp8: residual given without a summed output");
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, if (residual) launch_rms<T, true, true>(nullptr, q, scales, summed, x, weight, residual, M, H, eps, s);
                 else launch_rms<T, false, true>(nullptr, q, scales, nullptr, x, weight, nullptr, M, H, eps, s));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_embedding_rms_norm(void* out, uint8_t* q, float* scales, void* hidden, const void* table,
                                       const int64_t* tokens, const void* weight, int64_t M, int64_t H, int64_t V, float eps,
                                       int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0 && V > 0, "embedding_rms_norm: empty shape");
  LFM2_REQUIRE(hidden && table && tokens && weight, "embedding_rms_norm: a required pointer is null");
  LFM2_REQUIRE((q == nullptr) == (scales == nullptr) && (q == nullptr) != (out == nullptr),
               "embedding_rms_norm: either out, or q with scales");
  SplitInput gather{nullptr, nullptr, nullptr, 0, 0};
  gather.tokens = tokens;
  gather.vocab = V;
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, if (q) launch_rms<T, false, true>(nullptr, q, scales, hidden, table, weight, nullptr, M, H, eps, s, gather);
                 else launch_rms<T, false, false>(out, nullptr, nullptr, hidden, table, weight, nullptr, M, H, eps, s, gather));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_rms_norm_fp8_split(uint8_t* q, float* scales, void* summed, const float* partial, int splits,
                                       const float* a_scales, const float* w_scales, const void* weight,
                                       const void* residual, int64_t M, int64_t H, float eps, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0, "rms_norm_fp8_split: empty shape");
  LFM2_REQUIRE(partial && splits >= 1, "rms_norm_fp8_split: partial products are required");
  LFM2_REQUIRE((a_scales == nullptr) == (w_scales == nullptr), "rms_norm_fp8_split: both scale vectors or neither");
  LFM2_REQUIRE(residual == nullptr || summed != nullptr, "rms_norm_fp8_split: residual given without a summed output");
  const int vec = dtype == LFM2_DTYPE_F32 ? 4 : 8;
  LFM2_REQUIRE(H % vec == 0 && H <= (int64_t)16 * kRowThreads * vec, "rms_norm_fp8_split: width %ld is not a multiple of %d or too wide", (long)H, vec);
  const SplitInput split{partial, a_scales, w_scales, M * H, splits};
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, if (residual) launch_rms<T, true, true>(nullptr, q, scales, summed, nullptr, weight, residual, M, H, eps, s, split);
                 else launch_rms<T, false, true>(nullptr, q, scales, nullptr, nullptr, weight, nullptr, M, H, eps, s, split));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_rms_norm_split(void* out, void* summed, const float* partial, int splits, const float* a_scales,
                                   const float* w_scales, const void* weight, const void* residual, int64_t M, int64_t H,
                                   float eps, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0, "rms_norm_split: empty shape");
  LFM2_REQUIRE(partial && splits >= 1, "rms_norm_split: partial products are required");
  LFM2_REQUIRE((a_scales == nullptr) == (w_scales == nullptr), "rms_norm_split: both scale vectors or neither");
  LFM2_REQUIRE(residual == nullptr || summed != nullptr, "rms_norm_split: residual given without a summed output");
  const int vec = dtype == LFM2_DTYPE_F32 ? 4 : 8;
  LFM2_REQUIRE(H % vec == 0 && H <= (int64_t)16 * kRowThreads * vec, "rms_norm_split: width %ld is not a multiple of %d or too wide", (long)H, vec);
  const SplitInput split{partial, a_scales, w_scales, M * H, splits};
  hipStream_t s = (hipStream_t)stream;
  DISPATCH_DTYPE(dtype, if (residual) launch_rms<T, true, false>(out, nullptr, nullptr, summed, nullptr, weight, residual, M, H, eps, s, split);
                 else launch_rms<T, false, false>(out, nullptr, nullptr, nullptr, nullptr, weight, nullptr, M, H, eps, s, split));
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ SwiGLU

template <typename T>
__global__ void __launch_bounds__(kThreads) swiglu_kernel(T* out, const T* x, int64_t I) {
  const int64_t row = blockIdx.y;
  constexpr int N = Vec<T>::N;
  const T* gate = x + row * 2 * I;
  const T* up = gate + I;
  out += row * I;
  if (I % N == 0) {
    const int64_t i = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * N;
    if (i < I) {
      float g[N], u[N];
      load_vec<T>(gate + i, g);
      load_vec<T>(up + i, u);
#pragma unroll
      for (int e = 0; e < N; ++e) g[e] = round_to<T>(silu_f(g[e])) * u[e];
      store_vec<T>(out + i, g);
    }
  } else {
    for (int e = 0; e < N; ++e) {
      const int64_t i = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * N + e;
      if (i < I) out[i] = Elem<T>::store(round_to<T>(silu_f(Elem<T>::load(gate[i]))) * Elem<T>::load(up[i]));
    }
  }
}

extern "C" int lfm2_swiglu(void* out, const void* x, int64_t M, int64_t I, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && I > 0, "swiglu: empty shape");
  LFM2_REQUIRE(M <= 65535, "swiglu: more than 65535 rows");
  DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(swiglu_kernel<T>, dim3(ceil_div(I, kThreads * Vec<T>::N), M), dim3(kThreads),
                                           0, (hipStream_t)stream, (T*)out, (const T*)x, I));
  LFM2_LAUNCH_CHECK();
}

// SWIGLU = false gives plain row quantisation of x[M,K].
template <typename T, int NV, bool SWIGLU>
__global__ void __launch_bounds__(kRowThreads) quantize_kernel(uint8_t* q, float* scales, const T* x, int64_t K) {
  __shared__ float red[kRowWaves];
  const int64_t row = blockIdx.x;
  constexpr int N = Vec<T>::N;
  const T* a = x + row * (SWIGLU ? 2 * K : K);
  const T* b = a + K;
  q += row * K;
  float amax = 0.f;
  if constexpr (NV > 0) {
    float v[NV][N];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t i = (int64_t)(j * kRowThreads + threadIdx.x) * N;
      if (i < K) {
        load_vec<T>(a + i, v[j]);
        if (SWIGLU) {
          float u[N];
          load_vec<T>(b + i, u);
#pragma unroll
          for (int e = 0; e < N; ++e) v[j][e] = round_to<T>(round_to<T>(silu_f(v[j][e])) * u[e]);
        }
#pragma unroll
        for (int e = 0; e < N; ++e) amax = fmaxf(amax, fabsf(v[j][e]));
      }
    }
    amax = block_max<kRowWaves>(amax, red);
    const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
    if (threadIdx.x == 0) scales[row] = scale;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t i = (int64_t)(j * kRowThreads + threadIdx.x) * N;
      if (i < K) store_e4m3<N>(q + i, v[j], scale);
    }
  } else {
    auto value = [&](int64_t i) {
      float g = Elem<T>::load(a[i]);
      return SWIGLU ? round_to<T>(round_to<T>(silu_f(g)) * Elem<T>::load(b[i])) : g;
    };
    for (int64_t i = threadIdx.x; i < K; i += kRowThreads) amax = fmaxf(amax, fabsf(value(i)));
    amax = block_max<kRowWaves>(amax, red);
    const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
    if (threadIdx.x == 0) scales[row] = scale;
    for (int64_t i = threadIdx.x; i < K; i += kRowThreads) q[i] = to_e4m3(value(i) / scale);
  }
}

template <typename T, bool SWIGLU>
static void launch_quantize(uint8_t* q, float* scales, const void* x, int64_t M, int64_t K, hipStream_t s) {
  const int nv = pick_nv<T>(K);
#define Q_(NVV) \
  hipLaunchKernelGGL((quantize_kernel<T, NVV, SWIGLU>), dim3(M), dim3(kRowThreads), 0, s, q, scales, (const T*)x, K)
  LAUNCH_NV(nv, Q_(1), Q_(2), Q_(4), Q_(8), Q_(16), Q_(0));
#undef Q_
}

extern "C" int lfm2_swiglu_fp8(uint8_t* q, float* scales, const void* x, int64_t M, int64_t I, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && I > 0, "swiglu_fp8: empty shape");
  DISPATCH_DTYPE(dtype, launch_quantize<T, true>(q, scales, x, M, I, (hipStream_t)stream));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_quantize_rows(uint8_t* q, float* scales, const void* x, int64_t M, int64_t K, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && K > 0, "quantize_rows: empty shape");
  DISPATCH_DTYPE(dtype, launch_quantize<T, false>(q, scales, x, M, K, (hipStream_t)stream));
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ short-conv update
// Eight consecutive channels of one row with 16-byte accesses (16-bit T): 3 loads of the (B, C, x) thirds, 3 of the
// weights [8][3], 3 loads and 3 stores of the state [8][3].
template <typename T>
__device__ __forceinline__ void conv_group8(const T* in, const T* w, T* st, int64_t H, int64_t col, bool on, float* y) {
  float b[8], c[8], x[8], wt[24], s[24];
  load_vec<T>(in + col, b);
  load_vec<T>(in + H + col, c);
  load_vec<T>(in + 2 * H + col, x);
#pragma unroll
  for (int v = 0; v < 3; ++v) { load_vec<T>(w + col * 3 + 8 * v, wt + 8 * v); load_vec<T>(st + col * 3 + 8 * v, s + 8 * v); }
  float ns[24];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float bx;
    y[e] = conv_channel<T>(b[e], c[e], x[e], s[3 * e + 1], s[3 * e + 2], wt[3 * e], wt[3 * e + 1], wt[3 * e + 2], &bx);
    ns[3 * e] = s[3 * e + 1]; ns[3 * e + 1] = s[3 * e + 2]; ns[3 * e + 2] = bx;
  }
  if (on) {
#pragma unroll
    for (int v = 0; v < 3; ++v) store_vec<T>(st + col * 3 + 8 * v, ns + 8 * v);
  }
}

template <typename T>
__global__ void __launch_bounds__(kThreads)
conv_update_kernel(T* out, const T* bcx, const T* w, T* state, const uint8_t* active, const int32_t* slot_ids, int64_t H) {
  const int64_t row = blockIdx.y;
  int64_t slot = row;
  if (slot_ids) { const int32_t s = slot_ids[row]; slot = s < 0 ? 0 : s; }
  const bool on = active ? active[row] != 0 : true;
  const T* in = bcx + row * 3 * H;
  T* st = state + slot * H * 3;
  if constexpr (sizeof(T) == 2) {
    if (H % 8 == 0) {
      const int64_t col = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 8;
      if (col >= H) return;
      float y[8];
      conv_group8<T>(in, w, st, H, col, on, y);
      store_vec<T>(out + row * H + col, y);
      return;
    }
  }
  for (int e = 0; e < 8; ++e) {
    const int64_t col = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 8 + e;
    if (col >= H) return;
    float bx;
    const T t1 = st[col * 3 + 1], t2 = st[col * 3 + 2];
    const float y = conv_channel<T>(Elem<T>::load(in[col]), Elem<T>::load(in[H + col]), Elem<T>::load(in[2 * H + col]),
                                    Elem<T>::load(t1), Elem<T>::load(t2), Elem<T>::load(w[col * 3]),
                                    Elem<T>::load(w[col * 3 + 1]), Elem<T>::load(w[col * 3 + 2]), &bx);
    if (on) { st[col * 3] = t1; st[col * 3 + 1] = t2; st[col * 3 + 2] = Elem<T>::store(bx); }
    out[row * H + col] = Elem<T>::store(y);
  }
}

extern "C" int lfm2_conv_update(void* out, const void* bcx, const void* weight, void* state, const uint8_t* active,
                                const int32_t* slot_ids, int64_t M, int64_t H, int64_t slots, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0 && slots > 0, "conv_update: empty shape");
  LFM2_REQUIRE(slot_ids != nullptr || M <= slots, "conv_update: %ld rows but only %ld state slots", (long)M, (long)slots);
  LFM2_REQUIRE(M <= 65535, "conv_update: more than 65535 rows");
  DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(conv_update_kernel<T>, dim3(ceil_div(H, kThreads * 8), M), dim3(kThreads), 0,
                                           (hipStream_t)stream, (T*)out, (const T*)bcx, (const T*)weight, (T*)state,
                                           active, slot_ids, H));
  LFM2_LAUNCH_CHECK();
}

// conv_update followed by per-row e4m3 quantisation of its (model-dtype rounded) output, in one launch: one
// workgroup per row keeps the row's outputs in registers between the amax reduction and the conversion.
// NG = groups of eight consecutive channels per thread (H <= NG * 2048, H a multiple of 8, 16-bit T).
template <typename T, int NG>
__global__ void __launch_bounds__(kThreads)
conv_update_fp8_kernel(uint8_t* q, float* scales, const T* bcx, const T* w, T* state, const uint8_t* active,
                       const int32_t* slot_ids, int64_t H) {
  __shared__ float red[kWaves];
  const int64_t row = blockIdx.x;
  int64_t slot = row;
  if (slot_ids) { const int32_t s = slot_ids[row]; slot = s < 0 ? 0 : s; }
  const bool on = active ? active[row] != 0 : true;
  const T* in = bcx + row * 3 * H;
  T* st = state + slot * H * 3;
  float y[NG][8];
  float amax = 0.f;
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int64_t col = ((int64_t)g * kThreads + threadIdx.x) * 8;
    if (col < H) {
      conv_group8<T>(in, w, st, H, col, on, y[g]);
#pragma unroll
      for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(y[g][e]));
    }
  }
  amax = block_max<kWaves>(amax, red);
  const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
  if (threadIdx.x == 0) scales[row] = scale;
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int64_t col = ((int64_t)g * kThreads + threadIdx.x) * 8;
    if (col < H) store_e4m3<8>(q + row * H + col, y[g], scale);
  }
}

extern "C" int lfm2_conv_update_fp8(uint8_t* q, float* scales, const void* bcx, const void* weight, void* state,
                                    const uint8_t* active, const int32_t* slot_ids, int64_t M, int64_t H, int64_t slots,
                                    int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && H > 0 && slots > 0, "conv_update_fp8: empty shape");
  LFM2_REQUIRE(slot_ids != nullptr || M <= slots, "conv_update_fp8: %ld rows but only %ld state slots", (long)M, (long)slots);
  LFM2_REQUIRE(H % 8 == 0 && H <= 2 * 8 * kThreads, "conv_update_fp8: width %ld is not a multiple of 8 or above %d", (long)H, 2 * 8 * kThreads);
  hipStream_t s = (hipStream_t)stream;
#define CU_(TT, NGG) hipLaunchKernelGGL((conv_update_fp8_kernel<TT, NGG>), dim3(M), dim3(kThreads), 0, s, q, scales, \
                                        (const TT*)bcx, (const TT*)weight, (TT*)state, active, slot_ids, H)
  switch (dtype) {
    case LFM2_DTYPE_BF16: if (H <= 8 * kThreads) CU_(__bf16, 1); else CU_(__bf16, 2); break;
    case LFM2_DTYPE_F16: if (H <= 8 * kThreads) CU_(_Float16, 1); else CU_(_Float16, 2); break;
    default: LFM2_FAIL(LFM2_ERR_UNSUPPORTED, "conv_update_fp8: dtype %d is not bf16/f16", dtype);
  }
#undef CU_
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ packed-prefill short conv
// One thread per (token, channel).  Taps that would reach before the start of the token's own
// sequence read zero, so sequences packed back to back do not leak into each other.
template <typename T>
__global__ void __launch_bounds__(kThreads)
conv_prefill_kernel(T* out, T* state, const T* bcx, const T* w, const int32_t* cu, const int32_t* seq_of_token,
                    const int32_t* slots, int64_t H) {
  const int64_t t = blockIdx.y;
  const int64_t col = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (col >= H) return;
  const int seq = seq_of_token[t];
  const int64_t begin = cu[seq], end = cu[seq + 1];
  auto bx_at = [&](int64_t tok) -> float {
    if (tok < begin) return 0.f;
    const T* in = bcx + tok * 3 * H;
    return round_to<T>(Elem<T>::load(in[col]) * Elem<T>::load(in[2 * H + col]));
  };
  const float x0 = bx_at(t - 2), x1 = bx_at(t - 1), x2 = bx_at(t);
  const float w0 = Elem<T>::load(w[col * 3]), w1 = Elem<T>::load(w[col * 3 + 1]), w2 = Elem<T>::load(w[col * 3 + 2]);
  const float conv = round_to<T>(fmaf(x2, w2, fmaf(x1, w1, x0 * w0)));
  const float c = Elem<T>::load(bcx[t * 3 * H + H + col]);
  out[t * H + col] = Elem<T>::store(c * conv);
  if (t == end - 1) {
    T* st = state + ((int64_t)slots[seq] * H + col) * 3;
    st[0] = Elem<T>::store(x0); st[1] = Elem<T>::store(x1); st[2] = Elem<T>::store(x2);
  }
}

// The same for H % 8 == 0 with 16-byte accesses: a thread owns 8 channels of 4 consecutive tokens, so the products
// B.x of the six tokens its window touches are formed once (the scalar form reads ten 2-byte values per output).
// FP8 (H <= 2048: one workgroup holds whole rows): the rows leave as e4m3 codes with one scale per token, the bits
// `quantize_rows` makes of the rows the plain form stores, for an out projection that takes quantised activations.
template <typename T, bool FP8>
__global__ void __launch_bounds__(256)
conv_prefill_vec_kernel(T* out, uint8_t* q, float* scales, T* state, const T* bcx, const T* w, const int32_t* cu,
                        const int32_t* seq_of_token, const int32_t* slots, int64_t H, int64_t T_) {
  typedef T vec8 __attribute__((ext_vector_type(8)));
  constexpr int TOK = 4;
  __shared__ float red[4][TOK];
  const int64_t t0 = (int64_t)blockIdx.y * TOK;
  const int64_t col = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  const bool owns = col < H;
  if (!FP8 && !owns) return;
  float y[TOK][8], amax[TOK];
#pragma unroll
  for (int j = 0; j < TOK; ++j) amax[j] = 0.f;
  if (owns) {
    float bx[TOK + 2][8];
#pragma unroll
    for (int i = 0; i < TOK + 2; ++i) {
      const int64_t tok = t0 - 2 + i;
      if (tok >= 0 && tok < T_) {
        const T* in = bcx + tok * 3 * H + col;
        const vec8 bv = *reinterpret_cast<const vec8*>(in), xv = *reinterpret_cast<const vec8*>(in + 2 * H);
#pragma unroll
        for (int e = 0; e < 8; ++e) bx[i][e] = round_to<T>(Elem<T>::load(bv[e]) * Elem<T>::load(xv[e]));
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) bx[i][e] = 0.f;
      }
    }
    float taps[24];   // w[col .. col+7][0..2]
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const vec8 wv = *reinterpret_cast<const vec8*>(w + col * 3 + 8 * i);
#pragma unroll
      for (int e = 0; e < 8; ++e) taps[8 * i + e] = Elem<T>::load(wv[e]);
    }
#pragma unroll
    for (int j = 0; j < TOK; ++j) {
      const int64_t t = t0 + j;
      if (t >= T_) break;
      const int seq = seq_of_token[t];
      const int64_t begin = cu[seq], end = cu[seq + 1];
      const bool has1 = t - 1 >= begin, has2 = t - 2 >= begin;
      const vec8 cv = *reinterpret_cast<const vec8*>(bcx + t * 3 * H + H + col);
      vec8 ov;
      float x0[8], x1[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x0[e] = has2 ? bx[j][e] : 0.f;
        x1[e] = has1 ? bx[j + 1][e] : 0.f;
        const float conv = round_to<T>(fmaf(bx[j + 2][e], taps[3 * e + 2], fmaf(x1[e], taps[3 * e + 1], x0[e] * taps[3 * e])));
        ov[e] = Elem<T>::store(Elem<T>::load(cv[e]) * conv);
        if (FP8) { y[j][e] = Elem<T>::load(ov[e]); amax[j] = fmaxf(amax[j], fabsf(y[j][e])); }
      }
      if (!FP8) *reinterpret_cast<vec8*>(out + t * H + col) = ov;
      if (t == end - 1) {
        T* st = state + ((int64_t)slots[seq] * H + col) * 3;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          st[3 * e] = Elem<T>::store(x0[e]); st[3 * e + 1] = Elem<T>::store(x1[e]); st[3 * e + 2] = Elem<T>::store(bx[j + 2][e]);
        }
      }
    }
  }
  if constexpr (FP8) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < TOK; ++j) {
      const float m = wave_max(amax[j]);
      if (lane == 0) red[wave][j] = m;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TOK; ++j) {
      const int64_t t = t0 + j;
      if (t >= T_) break;
      const float m = fmaxf(fmaxf(red[0][j], red[1][j]), fmaxf(red[2][j], red[3][j]));
      const float scale = fmaxf(m / LFM2_E4M3_MAX, 1.0e-12f);
      if (threadIdx.x == 0) scales[t] = scale;
      if (owns) store_e4m3<8>(q + t * H + col, y[j], scale);
    }
  }
}

extern "C" int lfm2_conv_prefill(void* out, void* state, const void* bcx, const void* weight, const int32_t* cu_seqlens,
                                 const int32_t* seq_of_token, const int32_t* slots, int64_t T_, int64_t nseq, int64_t H,
                                 int64_t nslots, int dtype, void* stream) {
  LFM2_REQUIRE(T_ > 0 && nseq > 0 && H > 0 && nslots > 0, "conv_prefill: empty shape");
  LFM2_REQUIRE(T_ <= 65535, "conv_prefill: more than 65535 packed tokens in one call");
  if (H % 8 == 0 && dtype != LFM2_DTYPE_F32 && (((uintptr_t)out | (uintptr_t)bcx | (uintptr_t)weight) & 15) == 0) {
    const dim3 grid(ceil_div(H, 2048), ceil_div(T_, 4));
    if (dtype == LFM2_DTYPE_BF16)
      hipLaunchKernelGGL((conv_prefill_vec_kernel<__bf16, false>), grid, dim3(256), 0, (hipStream_t)stream, (__bf16*)out, nullptr, nullptr, (__bf16*)state,
                         (const __bf16*)bcx, (const __bf16*)weight, cu_seqlens, seq_of_token, slots, H, T_);
    else
      hipLaunchKernelGGL((conv_prefill_vec_kernel<_Float16, false>), grid, dim3(256), 0, (hipStream_t)stream, (_Float16*)out,
                         nullptr, nullptr, (_Float16*)state, (const _Float16*)bcx, (const _Float16*)weight, cu_seqlens, seq_of_token, slots, H, T_);
    LFM2_LAUNCH_CHECK();
  }
  DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(conv_prefill_kernel<T>, dim3(ceil_div(H, kThreads), T_), dim3(kThreads), 0,
                                           (hipStream_t)stream, (T*)out, (T*)state, (const T*)bcx, (const T*)weight,
                                           cu_seqlens, seq_of_token, slots, H));
  LFM2_LAUNCH_CHECK();
}

// The packed-prefill short conv with its rows quantised for a W8A8 out projection: `lfm2_conv_prefill` followed by
// `lfm2_quantize_rows`, the same bits, in one launch.  A workgroup must hold whole rows: H <= 2048, H % 8 == 0, 16-bit dtype.
extern "C" int lfm2_conv_prefill_fp8(uint8_t* q, float* scales, void* state, const void* bcx, const void* weight,
                                     const int32_t* cu_seqlens, const int32_t* seq_of_token, const int32_t* slots, int64_t T_,
                                     int64_t nseq, int64_t H, int64_t nslots, int dtype, void* stream) {
  LFM2_REQUIRE(T_ > 0 && nseq > 0 && H > 0 && nslots > 0, "conv_prefill_fp8: empty shape");
  LFM2_REQUIRE(T_ <= 4 * 65535, "conv_prefill_fp8: more than 262140 packed tokens in one call");
  LFM2_REQUIRE(H % 8 == 0 && H <= 2048, "conv_prefill_fp8: width %ld is not a multiple of 8 up to 2048", (long)H);
  LFM2_REQUIRE(dtype == LFM2_DTYPE_BF16 || dtype == LFM2_DTYPE_F16, "conv_prefill_fp8: 16-bit activations only");
  LFM2_REQUIRE((((uintptr_t)q & 7) | (((uintptr_t)bcx | (uintptr_t)weight) & 15)) == 0, "conv_prefill_fp8: misaligned buffer");
  const dim3 grid(1, ceil_div(T_, 4));
  if (dtype == LFM2_DTYPE_BF16)
    hipLaunchKernelGGL((conv_prefill_vec_kernel<__bf16, true>), grid, dim3(256), 0, (hipStream_t)stream, (__bf16*)nullptr, q, scales,
                       (__bf16*)state, (const __bf16*)bcx, (const __bf16*)weight, cu_seqlens, seq_of_token, slots, H, T_);
  else
    hipLaunchKernelGGL((conv_prefill_vec_kernel<_Float16, true>), grid, dim3(256), 0, (hipStream_t)stream, (_Float16*)nullptr, q,
                       scales, (_Float16*)state, (const _Float16*)bcx, (const _Float16*)weight, cu_seqlens, seq_of_token, slots, H, T_);
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ QK-norm + RoPE + split
// One workgroup per row; each wave walks over heads.  A lane owns D/64 (or fewer) elements of a
// head and reaches its rotate-half partner through LDS.
template <typename T>
__global__ void __launch_bounds__(kThreads)
prepare_qkv_kernel(T* q, T* k, T* v, const T* x, const T* qw, const T* kw, const float* cosT, const float* sinT,
                   const int32_t* positions, int QH, int KH, int D, int64_t max_positions, float eps) {
  __shared__ float buf[kWaves][256];
  const int64_t row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t width = (int64_t)(QH + 2 * KH) * D;
  const T* in = x + row * width;
  int64_t pos = positions[row];
  pos = pos < 0 ? 0 : (pos >= max_positions ? max_positions - 1 : pos);
  const int half = D / 2;
  for (int head = wave; head < QH + KH; head += kWaves) {
    const T* src = in + (int64_t)head * D;
    const T* wgt = head < QH ? qw : kw;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) { const float a = Elem<T>::load(src[d]); ss += a * a; }
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)D + eps);
    for (int d = lane; d < D; d += 64) {
      float n = round_to<T>(Elem<T>::load(src[d]) * rstd);
      buf[wave][d] = round_to<T>(n * Elem<T>::load(wgt[d]));
    }
    __builtin_amdgcn_wave_barrier();
    T* dst = head < QH ? q + (row * QH + head) * D : k + (row * KH + (head - QH)) * D;
    for (int d = lane; d < D; d += 64) {
      const float c = round_to<T>(cosT[pos * half + d % half]);
      const float s = round_to<T>(sinT[pos * half + d % half]);
      const float left = round_to<T>(buf[wave][d] * c);
      const float right = round_to<T>(buf[wave][(d + half) % D] * s);
      dst[d] = Elem<T>::store(d < half ? left - right : left + right);
    }
    __builtin_amdgcn_wave_barrier();
    if (head >= QH) {
      const int kh = head - QH;
      const T* vs = in + (int64_t)(QH + KH + kh) * D;
      T* vd = v + (row * KH + kh) * D;
      for (int d = lane; d < D; d += 64) vd[d] = vs[d];
    }
  }
}

// One wave per (row, head) unit for the usual head sizes: units 0..QH-1 are query heads, QH..QH+KH-1 key heads (both
// normalised and rotated), the rest value heads (copied).  A lane holds elements lane, lane+64, ...; the rotate-half
// partner is the lane D/2 away (D <= 64) or another register of the same lane (D >= 128).  With STORE the key and
// value heads go straight into the cache row of the token (model dtype, or e4m3 with one scale per token and head,
// quantised from the value rounded to the model dtype exactly as a separate store of the rounded tensor would).
struct PrepArgs {
  void *q, *k, *v;
  const void *x, *qw, *kw;
  const float *cosT, *sinT;
  const int32_t *positions, *slot_ids;
  const uint8_t* active;
  void *kc, *vc;
  float *ks, *vs;
  int64_t M, max_positions, c0, c1, c2;
  int QH, KH;
  float eps;
};

template <typename T, int D, int STORE>  // STORE 0: q, k, v tensors; 1: cache in the model dtype; 2: e4m3 cache
__global__ void __launch_bounds__(kThreads) prepare_qkv_wave_kernel(PrepArgs a) {
  constexpr int R = (D + 63) / 64, half = D / 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int U = a.QH + 2 * a.KH;
  const int64_t unit = (int64_t)blockIdx.x * kWaves + wave;
  if (unit >= a.M * U) return;
  const int64_t row = unit / U;
  const int u = (int)(unit % U);
  const T* src = (const T*)a.x + row * U * D + (int64_t)u * D;
  const bool on = D >= 64 || lane < D;
  float val[R];
#pragma unroll
  for (int i = 0; i < R; ++i) val[i] = on ? Elem<T>::load(src[lane + 64 * i]) : 0.f;
  if (u < a.QH + a.KH) {
    // everything the head needs is requested before the reduction: norm weights, and the rotary factors behind the
    // row's position
    const T* wgt = u < a.QH ? (const T*)a.qw : (const T*)a.kw;
    int64_t pos = a.positions[row];
    pos = pos < 0 ? 0 : (pos >= a.max_positions ? a.max_positions - 1 : pos);
    float gw[R], c[R], sn[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int t = on ? (lane + 64 * i) % half : 0;
      gw[i] = on ? Elem<T>::load(wgt[lane + 64 * i]) : 0.f;
      c[i] = round_to<T>(a.cosT[pos * half + t]);
      sn[i] = round_to<T>(a.sinT[pos * half + t]);
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) ss += val[i] * val[i];
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)D + a.eps);
    float w[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const float n = round_to<T>(val[i] * rstd);
      w[i] = on ? round_to<T>(n * gw[i]) : 0.f;
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int d = lane + 64 * i;
      const float partner = D >= 128 ? w[i ^ (D / 128)] : __shfl_xor(w[i], half, 64);
      const float left = round_to<T>(w[i] * c[i]), right = round_to<T>(partner * sn[i]);
      val[i] = round_to<T>(d < half ? left - right : left + right);
    }
  }
  if (u < a.QH) {
    T* dst = (T*)a.q + (row * a.QH + u) * D;
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (on) dst[lane + 64 * i] = Elem<T>::store(val[i]);
    return;
  }
  const bool is_v = u >= a.QH + a.KH;
  const int h = is_v ? u - a.QH - a.KH : u - a.QH;
  if (STORE == 0) {
    T* dst = (T*)(is_v ? a.v : a.k) + (row * a.KH + h) * D;
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (on) dst[lane + 64 * i] = Elem<T>::store(val[i]);
    return;
  }
  if (a.active && !a.active[row]) return;
  const int64_t slot = a.slot_ids ? a.slot_ids[row] : row;
  const int64_t at = a.positions[row];
  if (slot < 0 || at < 0) return;
  const int64_t dst = slot * a.c0 + at * a.c1 + (int64_t)h * a.c2;
  if (STORE == 1) {
    T* out = (T*)(is_v ? a.vc : a.kc) + dst;
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (on) out[lane + 64 * i] = Elem<T>::store(val[i]);
  } else {
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) amax = fmaxf(amax, fabsf(val[i]));
    amax = wave_max(amax);
    const float sc = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
    uint8_t* out = (uint8_t*)(is_v ? a.vc : a.kc) + dst;
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (on) out[lane + 64 * i] = to_e4m3(val[i] / sc);
    if (lane == 0) (is_v ? a.vs : a.ks)[dst / D] = sc;
  }
}

// head_dim 64 into q, k, v tensors (prefill: thousands of rows), 16 bytes per access: eight lanes share a head
// unit, lane s of the eight owns elements 8s .. 8s+7, its rotate-half partner is the lane four away.  Same rounding
// points as the wave-per-unit form.
template <typename T>
__global__ void __launch_bounds__(kThreads) prepare_qkv_vec64_kernel(PrepArgs a) {
  typedef T vec8 __attribute__((ext_vector_type(8)));
  constexpr int D = 64, half = 32;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane & 7;
  const int U = a.QH + 2 * a.KH;
  const int64_t units = a.M * U;
  int64_t unit = ((int64_t)blockIdx.x * kWaves + wave) * 8 + (lane >> 3);
  const bool live = unit < units;
  unit = live ? unit : units - 1;
  const int64_t row = unit / U;
  const int u = (int)(unit % U);
  const vec8 raw = *reinterpret_cast<const vec8*>((const T*)a.x + row * U * D + (int64_t)u * D + 8 * sub);
  float val[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) val[e] = Elem<T>::load(raw[e]);
  if (u < a.QH + a.KH) {
    const vec8 gw = *reinterpret_cast<const vec8*>((u < a.QH ? (const T*)a.qw : (const T*)a.kw) + 8 * sub);
    int64_t pos = a.positions[row];
    pos = pos < 0 ? 0 : (pos >= a.max_positions ? a.max_positions - 1 : pos);
    const f32x4* cs = reinterpret_cast<const f32x4*>(a.cosT + pos * half + 8 * (sub & 3));
    const f32x4* sn = reinterpret_cast<const f32x4*>(a.sinT + pos * half + 8 * (sub & 3));
    const f32x4 c0 = cs[0], c1 = cs[1], s0 = sn[0], s1 = sn[1];
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += val[e] * val[e];
    ss += __shfl_xor(ss, 1, 64); ss += __shfl_xor(ss, 2, 64); ss += __shfl_xor(ss, 4, 64);
    const float rstd = 1.0f / sqrtf(ss / (float)D + a.eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float n = round_to<T>(val[e] * rstd);
      const float w = round_to<T>(n * Elem<T>::load(gw[e]));
      const float partner = __shfl_xor(w, 4, 64);
      const float c = round_to<T>(e < 4 ? c0[e & 3] : c1[e & 3]), s = round_to<T>(e < 4 ? s0[e & 3] : s1[e & 3]);
      const float left = round_to<T>(w * c), right = round_to<T>(partner * s);
      val[e] = round_to<T>(sub < 4 ? left - right : left + right);
    }
  }
  if (!live) return;
  vec8 outv;
#pragma unroll
  for (int e = 0; e < 8; ++e) outv[e] = Elem<T>::store(val[e]);
  T* dst = u < a.QH ? (T*)a.q + (row * a.QH + u) * D
                    : (u < a.QH + a.KH ? (T*)a.k + (row * a.KH + (u - a.QH)) * D : (T*)a.v + (row * a.KH + (u - a.QH - a.KH)) * D);
  *reinterpret_cast<vec8*>(dst + 8 * sub) = outv;
}

template <typename T, int STORE>
int launch_prepare(const PrepArgs& a, int D, hipStream_t s) {
  const int64_t units = a.M * (a.QH + 2 * a.KH);
  const dim3 grid(ceil_div(units, kWaves)), block(kThreads);
  switch (D) {
    case 32: hipLaunchKernelGGL((prepare_qkv_wave_kernel<T, 32, STORE>), grid, block, 0, s, a); break;
    case 64: hipLaunchKernelGGL((prepare_qkv_wave_kernel<T, 64, STORE>), grid, block, 0, s, a); break;
    case 128: hipLaunchKernelGGL((prepare_qkv_wave_kernel<T, 128, STORE>), grid, block, 0, s, a); break;
    case 256: hipLaunchKernelGGL((prepare_qkv_wave_kernel<T, 256, STORE>), grid, block, 0, s, a); break;
    default: return 1;
  }
  return 0;
}

extern "C" int lfm2_prepare_qkv(void* q, void* k, void* v, const void* x, const void* q_weight, const void* k_weight,
                                const float* cos, const float* sin, const int32_t* positions, int64_t M, int QH, int KH,
                                int D, int64_t max_positions, float eps, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && QH > 0 && KH > 0, "prepare_qkv: empty shape");
  LFM2_REQUIRE(D > 0 && D <= 256 && D % 2 == 0, "prepare_qkv: head_dim %d not in (0,256] or odd", D);
  LFM2_REQUIRE(max_positions > 0, "prepare_qkv: empty rotary table");
  if (D == 32 || D == 64 || D == 128 || D == 256) {
    const PrepArgs a{q, k, v, x, q_weight, k_weight, cos, sin, positions, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                     M, max_positions, 0, 0, 0, QH, KH, eps};
    const uintptr_t pointers = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)x | (uintptr_t)q_weight |
                               (uintptr_t)k_weight | (uintptr_t)cos | (uintptr_t)sin;
    if (D == 64 && dtype != LFM2_DTYPE_F32 && M >= 512 && (pointers & 15) == 0) {
      const dim3 grid(ceil_div(M * (QH + 2 * KH), kWaves * 8));
      if (dtype == LFM2_DTYPE_BF16) hipLaunchKernelGGL(prepare_qkv_vec64_kernel<__bf16>, grid, dim3(kThreads), 0, (hipStream_t)stream, a);
      else hipLaunchKernelGGL(prepare_qkv_vec64_kernel<_Float16>, grid, dim3(kThreads), 0, (hipStream_t)stream, a);
      LFM2_LAUNCH_CHECK();
    }
    DISPATCH_DTYPE(dtype, (launch_prepare<T, 0>(a, D, (hipStream_t)stream)));
    LFM2_LAUNCH_CHECK();
  }
  DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(prepare_qkv_kernel<T>, dim3(M), dim3(kThreads), 0, (hipStream_t)stream, (T*)q,
                                           (T*)k, (T*)v, (const T*)x, (const T*)q_weight, (const T*)k_weight, cos, sin,
                                           positions, QH, KH, D, max_positions, eps));
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_prepare_qkv_store(void* q, const void* x, const void* q_weight, const void* k_weight, const float* cos,
                                      const float* sin, const int32_t* positions, void* k_cache, void* v_cache,
                                      float* k_scales, float* v_scales, const uint8_t* active, const int32_t* slot_ids,
                                      int64_t M, int QH, int KH, int D, int64_t max_positions, float eps, int64_t c0,
                                      int64_t c1, int64_t c2, int kv_fp8, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && QH > 0 && KH > 0, "prepare_qkv_store: empty shape");
  LFM2_REQUIRE(D == 32 || D == 64 || D == 128 || D == 256, "prepare_qkv_store: head_dim %d not in {32,64,128,256}", D);
  LFM2_REQUIRE(max_positions > 0, "prepare_qkv_store: empty rotary table");
  LFM2_REQUIRE(k_cache && v_cache && positions, "prepare_qkv_store: caches and positions are required");
  LFM2_REQUIRE(!kv_fp8 || (k_scales && v_scales), "prepare_qkv_store: e4m3 cache without scale tensors");
  const PrepArgs a{q, nullptr, nullptr, x, q_weight, k_weight, cos, sin, positions, slot_ids, active, k_cache, v_cache,
                   k_scales, v_scales, M, max_positions, c0, c1, c2, QH, KH, eps};
  if (kv_fp8) { DISPATCH_DTYPE(dtype, (launch_prepare<T, 2>(a, D, (hipStream_t)stream))); }
  else { DISPATCH_DTYPE(dtype, (launch_prepare<T, 1>(a, D, (hipStream_t)stream))); }
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ HBM streaming read probe
// What the chip delivers when every CU only reads: the measured ceiling that the bandwidth-bound kernels of this
// library are held against next to the nominal 8 TB/s.  Each lane keeps UNROLL 16-byte loads in flight, folds what
// arrives into one word (so the loads cannot be dropped) and stores that word once at the end.
//   layout 0: every workgroup streams a private contiguous region (how the decode-attention kernel reads a history);
//   layout 1: the whole grid sweeps the buffer together, workgroup w taking 4 KiB blocks w, w + grid, ...
namespace {
template <int UNROLL, bool SWEEP>
__global__ void __launch_bounds__(256)
hbm_stream_kernel(const i32x4* __restrict__ src, int64_t vectors, int32_t* __restrict__ sink) {
  const int64_t grid = gridDim.x, block = blockIdx.x;
  // a block is 256 lanes x 16 bytes; blocks [first, first + count) with stride `step` belong to this workgroup
  const int64_t blocks = vectors / 256;
  const int64_t per = blocks / grid;                      // whole blocks per workgroup; the tail is not read
  const int64_t first = SWEEP ? block : block * per, step = SWEEP ? grid : 1;
  i32x4 acc = {0, 0, 0, 0};
  int64_t b = 0;
  for (; b + UNROLL <= per; b += UNROLL) {
    i32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
      v[u] = __builtin_nontemporal_load(src + (first + (b + u) * step) * 256 + threadIdx.x);
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
  }
  for (; b < per; ++b) acc ^= __builtin_nontemporal_load(src + (first + b * step) * 256 + threadIdx.x);
  sink[block * 256 + threadIdx.x] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
}
}  // namespace

extern "C" int lfm2_hbm_stream_read(const void* src, int64_t bytes, int32_t* sink, int workgroups, int layout, void* stream) {
  LFM2_REQUIRE(src && sink, "hbm_stream_read: null buffer");
  LFM2_REQUIRE(((uintptr_t)src & 15) == 0, "hbm_stream_read: source not 16-byte aligned");
  LFM2_REQUIRE(workgroups > 0 && workgroups <= 65536, "hbm_stream_read: workgroups %d not in [1, 65536]", workgroups);
  LFM2_REQUIRE(bytes >= (int64_t)workgroups * 4096, "hbm_stream_read: fewer than 4096 bytes per workgroup");
  LFM2_REQUIRE(layout == 0 || layout == 1, "hbm_stream_read: layout %d not 0 (private regions) or 1 (sweep)", layout);
  const int64_t vectors = bytes / 16;
  if (layout == 0)
    hipLaunchKernelGGL((hbm_stream_kernel<8, false>), dim3(workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const i32x4*)src, vectors, sink);
  else
    hipLaunchKernelGGL((hbm_stream_kernel<8, true>), dim3(workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const i32x4*)src, vectors, sink);
  LFM2_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------ device timestamps
// A one-lane kernel that stores the device's constant-rate wall clock.  Recorded into a graph in front of and behind
// a kernel, two of them bracket that kernel's time inside the replayed graph (stream order makes each run when its
// predecessor has finished); two adjacent ones measure the cost of the bracket itself.
namespace {
__global__ void timestamp_kernel(int64_t* out) {
  if (threadIdx.x == 0) *out = (int64_t)wall_clock64();
}
}  // namespace

extern "C" int lfm2_timestamp(int64_t* out, void* stream) {
  LFM2_REQUIRE(out != nullptr, "timestamp: null output");
  hipLaunchKernelGGL(timestamp_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, out);
  LFM2_LAUNCH_CHECK();
}

extern "C" int64_t lfm2_timestamp_rate_khz(void) {
  int device = 0, rate = 0;
  if (hipGetDevice(&device) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&rate, hipDeviceAttributeWallClockRate, device) != hipSuccess) return 0;
  return rate;
}
