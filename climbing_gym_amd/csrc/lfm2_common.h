// Shared device helpers for the LFM2 gfx950 kernels (wave64, CDNA4).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/lfm2_hip.h"

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

#define LFM2_E4M3_MAX 448.0f
#define LFM2_LOG2E 1.4426950408889634f

// ---- error reporting shared by every translation unit -------------------------------
void lfm2_set_error(const char* fmt, ...);
#define LFM2_FAIL(code, ...)       \
  do {                             \
    lfm2_set_error(__VA_ARGS__);   \
    return (code);                 \
  } while (0)
#define LFM2_REQUIRE(cond, ...) \
  do {                          \
    if (!(cond)) LFM2_FAIL(LFM2_ERR_ARGUMENT, __VA_ARGS__); \
  } while (0)
#define LFM2_LAUNCH_CHECK()                                                    \
  do {                                                                         \
    hipError_t e_ = hipGetLastError();                                         \
    if (e_ != hipSuccess) LFM2_FAIL(LFM2_ERR_LAUNCH, "%s", hipGetErrorString(e_)); \
    return LFM2_OK;                                                            \
  } while (0)

// ---- dtype traits -----------------------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  static __device__ __forceinline__ float load(__bf16 v) { return (float)v; }
  static __device__ __forceinline__ __bf16 store(float v) { return (__bf16)v; }
};
template <> struct Elem<_Float16> {
  static __device__ __forceinline__ float load(_Float16 v) { return (float)v; }
  static __device__ __forceinline__ _Float16 store(float v) { return (_Float16)v; }
};
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(float v) { return v; }
  static __device__ __forceinline__ float store(float v) { return v; }
};
// Round an fp32 value to the model dtype and return it as fp32 again.
template <typename T> __device__ __forceinline__ float round_to(float v) { return Elem<T>::load(Elem<T>::store(v)); }

// SiLU as the SwiGLU kernels compute it (one definition, so that a fused epilogue and the stand-alone kernels give the
// same bits): g / (1 + e^-g) on the hardware's base-2 exponential and reciprocal (v_exp_f32, v_rcp_f32: one unit in
// the last place each) instead of the library exponential and an IEEE division, which cost a 256x256 tile of the fused
// gate+up product a tenth of its time.  The relative error is bounded by (3 + max(-g, 0)) 2^-23: the argument g log2(e)
// is rounded once, which the exponential turns into max(-g, 0) 2^-24 of relative error where e^-g dominates and into
// nothing where 1 does.  A 16-bit result differs from the exactly rounded one in about one element in ten thousand.
// Limits: e^-g overflows to infinity for g < -88.7 and the result is -0 (the exact value is below the smallest normal
// number there); NaN stays NaN.
__device__ __forceinline__ float silu_f(float g) {
  return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -LFM2_LOG2E));
}

// One channel of the gated short conv: taps (state[1], state[2], b*x) with weights w[0..2]; returns c * conv and the
// new state entry b*x, every product and the tap sum rounded to T as the reference's kernel rounds them.
template <typename T>
__device__ __forceinline__ float conv_channel(float b, float c, float x, float s0, float s1, float w0, float w1, float w2,
                                              float* bx_out) {
  const float bx = round_to<T>(b * x);
  const float p0 = round_to<T>(s0 * w0), p1 = round_to<T>(s1 * w1), p2 = round_to<T>(bx * w2);
  const float conv = round_to<T>((p0 + p1) + p2);
  *bx_out = bx;
  return round_to<T>(c * conv);
}

// ---- wave / block reductions (64-lane wavefronts) ----------------------------------
// All-reduce butterflies that stay in the vector ALU: two quad permutes, the two row mirrors (lane i <-> 7-i, then
// i <-> 15-i: by then each half already holds one value, so a mirror pairs the halves), and gfx950's row and
// half-wave swaps.  Every lane ends with the same bits.  (__shfl_xor goes through the LDS crossbar instead:
// six dependent round trips of more than a hundred cycles each.)
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// v combined with the value of the same lane position in the neighbouring row of 16 lanes (lane ^ 16), or in the
// other half of the wave (lane ^ 32).  The swap returns {own | partner, partner | own} by row parity: a commutative
// combination of the two is the same on both sides.
struct AddOp { static __device__ __forceinline__ float apply(float a, float b) { return a + b; } };
struct MaxOp { static __device__ __forceinline__ float apply(float a, float b) { return fmaxf(a, b); } };
template <typename Op, bool HALVES> __device__ __forceinline__ float combine_swapped(float v) {
  const unsigned x = __builtin_bit_cast(unsigned, v);
  const auto r = HALVES ? __builtin_amdgcn_permlane32_swap(x, x, false, false) : __builtin_amdgcn_permlane16_swap(x, x, false, false);
  return Op::apply(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float add_lane_xor16(float v) { return combine_swapped<AddOp, false>(v); }
__device__ __forceinline__ float add_lane_xor32(float v) { return combine_swapped<AddOp, true>(v); }
__device__ __forceinline__ float max_lane_xor16(float v) { return combine_swapped<MaxOp, false>(v); }
__device__ __forceinline__ float max_lane_xor32(float v) { return combine_swapped<MaxOp, true>(v); }
template <typename Op> __device__ __forceinline__ float wave_all(float v) {
  v = Op::apply(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
  v = Op::apply(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
  v = Op::apply(v, dpp_move<0x141>(v));   // row_half_mirror
  v = Op::apply(v, dpp_move<0x140>(v));   // row_mirror
  v = combine_swapped<Op, false>(v);
  return combine_swapped<Op, true>(v);
}
__device__ __forceinline__ float wave_sum(float v) { return wave_all<AddOp>(v); }
__device__ __forceinline__ float wave_max(float v) { return wave_all<MaxOp>(v); }
// Block-wide reductions through a small LDS array; every thread gets the result.
template <int WAVES> __device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  if (WAVES == 1) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < WAVES; ++i) t += scratch[i];
  return t;
}
template <int WAVES> __device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  if (WAVES == 1) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
#pragma unroll
  for (int i = 1; i < WAVES; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

// ---- e4m3 (OCP, finite-only) conversions --------------------------------------------
// Saturating round-to-nearest-even of four fp32 values into one dword of e4m3 codes.
__device__ __forceinline__ int pack_e4m3x4(float a, float b, float c, float d) {
  a = fminf(fmaxf(a, -LFM2_E4M3_MAX), LFM2_E4M3_MAX);
  b = fminf(fmaxf(b, -LFM2_E4M3_MAX), LFM2_E4M3_MAX);
  c = fminf(fmaxf(c, -LFM2_E4M3_MAX), LFM2_E4M3_MAX);
  d = fminf(fmaxf(d, -LFM2_E4M3_MAX), LFM2_E4M3_MAX);
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  return __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
}
__device__ __forceinline__ uint8_t to_e4m3(float a) {
  a = fminf(fmaxf(a, -LFM2_E4M3_MAX), LFM2_E4M3_MAX);
  return (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(a, a, 0, false) & 0xff);
}
// Four e4m3 codes in a dword -> four floats.
__device__ __forceinline__ void unpack_e4m3x4(int w, float* out) {
  f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
  f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
  out[0] = lo[0]; out[1] = lo[1]; out[2] = hi[0]; out[3] = hi[1];
}

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }
