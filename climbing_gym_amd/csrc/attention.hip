// KV-cache writes, ragged GQA decode attention (split over the history) and varlen causal prefill
// attention for the LFM2 attention layers.
//
// Cache addressing follows the reference's strided views: element (slot, pos, head, d) of a layer
// lives at slot*c0 + pos*c1 + head*c2 + d, and the e4m3 scale of (slot, pos, head) at that offset
// divided by D.  With a block table, c0 is the page stride and pos is the in-page index.
#include "lfm2_common.h"

namespace {

#define DISPATCH_HALF(dtype, name, ...)                                                    \
  switch (dtype) {                                                                         \
    case LFM2_DTYPE_BF16: { typedef __bf16 T; __VA_ARGS__; } break;                        \
    case LFM2_DTYPE_F16: { typedef _Float16 T; __VA_ARGS__; } break;                       \
    default: LFM2_FAIL(LFM2_ERR_UNSUPPORTED, "%s: dtype %d is not bf16/f16", name, dtype); \
  }

// ===================================================================================== KV writes
struct StoreArgs {
  const void *k, *v;
  void *kc, *vc;
  float *ks, *vs;
  const int32_t *positions, *slot_ids, *cu, *seq_of_token;
  const uint8_t* active;
  int64_t T, ks0, ks1, ks2, vs0, vs1, vs2, c0, c1, c2;
  int KH, D;
};

// One workgroup per (batch, token) row; a head is covered by D/4 lanes holding 4 dims each.
template <typename T, bool FP8, bool PACKED>
__global__ void __launch_bounds__(256) store_kv_kernel(StoreArgs a) {
  const int64_t row = blockIdx.x;
  int64_t slot, pos, ksrc, vsrc;
  if (PACKED) {
    const int seq = a.seq_of_token[row];
    pos = row - a.cu[seq];
    slot = a.slot_ids ? a.slot_ids[seq] : seq;
    ksrc = vsrc = row * a.KH * a.D;
  } else {
    const int64_t batch = row / a.T, token = row % a.T;
    if (a.active && !a.active[batch]) return;
    slot = a.slot_ids ? a.slot_ids[batch] : batch;
    pos = a.positions ? a.positions[batch] : token;
    ksrc = batch * a.ks0 + token * a.ks1;
    vsrc = batch * a.vs0 + token * a.vs1;
  }
  if (slot < 0) return;
  const int lph = a.D / 4;                 // lanes per head (8..64)
  const int heads_per_pass = 256 / lph;
  const int sub = threadIdx.x % lph;
  const int64_t kstep = PACKED ? a.D : a.ks2, vstep = PACKED ? a.D : a.vs2;
  for (int h0 = 0; h0 < a.KH; h0 += heads_per_pass) {
    const int h = h0 + threadIdx.x / lph;
    const bool live = h < a.KH;
    const int hh = live ? h : a.KH - 1;
    const int64_t dst = slot * a.c0 + pos * a.c1 + (int64_t)hh * a.c2;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      const T* src = which ? (const T*)a.v + vsrc + hh * vstep : (const T*)a.k + ksrc + hh * kstep;
      float x[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = Elem<T>::load(src[sub * 4 + e]);
      if (FP8) {
        float amax = fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3])));
        for (int o = lph / 2; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
        const float s = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
        if (live) {
          uint8_t* out = (uint8_t*)(which ? a.vc : a.kc) + dst + sub * 4;
          *reinterpret_cast<int*>(out) = pack_e4m3x4(x[0] / s, x[1] / s, x[2] / s, x[3] / s);
          if (sub == 0) (which ? a.vs : a.ks)[dst / a.D] = s;
        }
      } else if (live) {
        T* out = (T*)(which ? a.vc : a.kc) + dst + sub * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = src[sub * 4 + e];
      }
    }
  }
}

int check_head_dim(const char* name, int D) {
  LFM2_REQUIRE(D == 32 || D == 64 || D == 128 || D == 256, "%s: head_dim %d not in {32,64,128,256}", name, D);
  return LFM2_OK;
}

// ===================================================================================== decode attention
constexpr int kChunk = 512;        // history tokens per workgroup
constexpr int kWaveTok = kChunk / 4;
constexpr int kGB = 4;             // query heads per workgroup (one GQA group, padded)

struct DecodeArgs {
  void* out;
  const void *q, *kc, *vc;
  const float *ks, *vs;
  const int32_t *positions, *slot_ids, *block_table;
  const uint8_t* active;
  float *ws_acc, *ws_m, *ws_l;
  const int32_t* schedule;  // [0] = number of (row, chunk) items, then the pairs
  int64_t max_blocks, c0, c1, c2;
  int page, QH, KH, D, G, nchunks, chunk;
  float scale_log2e;
};

template <bool FP8> struct KvLoad;
template <> struct KvLoad<true> {  // 16 e4m3 codes
  static __device__ __forceinline__ void run(const void* base, int64_t off, bool ok, float* out) {
    i32x4 w = {0, 0, 0, 0};
    if (ok) w = *reinterpret_cast<const i32x4*>((const uint8_t*)base + off);
#pragma unroll
    for (int i = 0; i < 4; ++i) unpack_e4m3x4(w[i], out + 4 * i);
  }
};
template <typename T> __device__ __forceinline__ void load16(const T* p, bool ok, float* out) {
  typedef T vec8 __attribute__((ext_vector_type(8)));
  vec8 a = {}, b = {};
  if (ok) { a = *reinterpret_cast<const vec8*>(p); b = *reinterpret_cast<const vec8*>(p + 8); }
#pragma unroll
  for (int i = 0; i < 8; ++i) { out[i] = (float)a[i]; out[8 + i] = (float)b[i]; }
}

// Generic path: every lane owns 16 dims of one history token per step (D/16 lanes per token), two
// tokens per lane per iteration.  The running maximum is kept wave-uniform so per-lane partial
// sums can simply be added at the end of the wave's range.
template <typename T, bool FP8, int D>
__global__ void __launch_bounds__(256) decode_attn_kernel(DecodeArgs a) {
  constexpr int LPT = D / 16, TPI = 64 / LPT;
  const int b = blockIdx.z, chunk = blockIdx.x;
  const int gblocks = (a.G + kGB - 1) / kGB;
  const int h = blockIdx.y / gblocks, g0 = (blockIdx.y % gblocks) * kGB;
  if (a.active && !a.active[b]) return;
  const int64_t slot = a.slot_ids ? a.slot_ids[b] : b;
  if (slot < 0) return;
  const int len = a.positions[b] + 1;
  const int start = chunk * kChunk;
  if (start >= len) return;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane % LPT, tg = lane / LPT;

  float qr[kGB][16];
#pragma unroll
  for (int g = 0; g < kGB; ++g) {
    const bool ok = g0 + g < a.G;
    const T* src = (const T*)a.q + ((int64_t)b * a.QH + h * a.G + (ok ? g0 + g : 0)) * D + sub * 16;
    load16<T>(src, ok, qr[g]);
  }
  float m[kGB], l[kGB], acc[kGB][16];
#pragma unroll
  for (int g = 0; g < kGB; ++g) {
    m[g] = -1.0e30f; l[g] = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[g][j] = 0.f;
  }

  auto token_offset = [&](int t) -> int64_t {
    if (a.block_table) {
      const int64_t blk = a.block_table[(int64_t)b * a.max_blocks + t / a.page];
      return blk * a.c0 + (int64_t)(t % a.page) * a.c1 + (int64_t)h * a.c2;
    }
    return slot * a.c0 + (int64_t)t * a.c1 + (int64_t)h * a.c2;
  };

  const int wbeg = start + wave * kWaveTok;
  int wend = wbeg + kWaveTok;
  wend = wend < len ? wend : len;
  for (int t0 = wbeg; t0 < wend; t0 += 2 * TPI) {
    float kf[2][16], vf[2][16], sk[2], sv[2];
    bool ok[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int t = t0 + u * TPI + tg;
      ok[u] = t < wend;
      const int64_t off = token_offset(ok[u] ? t : wbeg);
      if (FP8) {
        KvLoad<true>::run(a.kc, off + sub * 16, ok[u], kf[u]);
        KvLoad<true>::run(a.vc, off + sub * 16, ok[u], vf[u]);
        sk[u] = ok[u] ? a.ks[off / D] : 0.f;
        sv[u] = ok[u] ? a.vs[off / D] : 0.f;
      } else {
        load16<T>((const T*)a.kc + off + sub * 16, ok[u], kf[u]);
        load16<T>((const T*)a.vc + off + sub * 16, ok[u], vf[u]);
        sk[u] = 1.f; sv[u] = 1.f;
      }
    }
#pragma unroll
    for (int g = 0; g < kGB; ++g) {
      float s[2];
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        float d = 0.f;
#pragma unroll
        for (int j = 0; j < 16; ++j) d = fmaf(qr[g][j], kf[u][j], d);
#pragma unroll
        for (int o = LPT / 2; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
        s[u] = ok[u] ? d * (a.scale_log2e * sk[u]) : -1.0e30f;
      }
      float mx = fmaxf(s[0], s[1]);
#pragma unroll
      for (int o = 32; o >= LPT; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
      const float mnew = fmaxf(m[g], mx);
      const float alpha = exp2f(m[g] - mnew);
      const float p0 = ok[0] ? exp2f(s[0] - mnew) : 0.f, p1 = ok[1] ? exp2f(s[1] - mnew) : 0.f;
      l[g] = fmaf(l[g], alpha, p0 + p1);
      const float w0 = p0 * sv[0], w1 = p1 * sv[1];
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[g][j] = fmaf(w1, vf[1][j], fmaf(w0, vf[0][j], acc[g][j] * alpha));
      m[g] = mnew;
    }
  }

  // Add the per-lane partial sums of the TPI token groups (same maximum everywhere in the wave).
#pragma unroll
  for (int g = 0; g < kGB; ++g) {
#pragma unroll
    for (int o = 32; o >= LPT; o >>= 1) {
      l[g] += __shfl_xor(l[g], o, 64);
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[g][j] += __shfl_xor(acc[g][j], o, 64);
    }
  }
  __shared__ float sm[4][kGB], sl[4][kGB], sacc[4][kGB][D];
  if (tg == 0) {
#pragma unroll
    for (int g = 0; g < kGB; ++g) {
      if (sub == 0) { sm[wave][g] = m[g]; sl[wave][g] = l[g]; }
#pragma unroll
      for (int j = 0; j < 16; ++j) sacc[wave][g][sub * 16 + j] = acc[g][j];
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < kGB * D; idx += 256) {
    const int g = idx / D, d = idx % D;
    if (g0 + g >= a.G) continue;
    float mm = sm[0][g];
#pragma unroll
    for (int w = 1; w < 4; ++w) mm = fmaxf(mm, sm[w][g]);
    float lt = 0.f, ot = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(sm[w][g] - mm);
      lt = fmaf(sl[w][g], f, lt);
      ot = fmaf(sacc[w][g][d], f, ot);
    }
    const int64_t prow = ((int64_t)b * a.QH + h * a.G + g0 + g) * a.nchunks + chunk;
    a.ws_acc[prow * D + d] = ot;
    if (d == 0) { a.ws_m[prow] = mm; a.ws_l[prow] = lt; }
  }
}

// ----------------------------------------------------------------------------- e4m3 history on MFMA
// Specialisation for the headline shape: e4m3 history, head_dim 64, a GQA group of at most 4 query heads.
// A wave walks its token range in tiles of 64 tokens and never leaves registers except for a 512-byte P tile:
//
//   S = Q.K^T : sixteen v_mfma_f32_4x4x4_16B_bf16 (16 independent 4x4x4 blocks per instruction).  Block b
//               multiplies Q[4 heads][4 dims] by K[tokens 4b..4b+3][4 dims], so lane l owns token l of the tile:
//               it loads that token's 64-byte row with four 16-byte loads and ends with S[0..3][token l].
//   softmax   : running maxima are wave-uniform and only raised (with a rescale) when some lane exceeds them by
//               more than kMaxSlack (so p <= 2^kMaxSlack, harmless in fp32 and bf16: the softmax is invariant to
//               the reference point), so per-lane partial sums of l and O can simply be added at the end and the
//               wave-wide maximum is needed on a wave's first tile and rarely afterwards.
//   O += P.V  : lane (g16, q, i) loads V[token 4*g16+i (+16u)][dims 16q..16q+15]; every dword is a 4x4 byte block
//               over the quad (4 tokens x 4 dims) which two DPP quad permutes + two v_perm transpose in
//               registers, giving the B operand V[4 tokens][dim]; P comes back from LDS as the A operand.
//               Block (g16, q) accumulates O[4 heads][dims 16q+4w..] over its own tokens; the four g16 partials
//               are added once per wave.
//
// e4m3 -> bf16 conversion is v_cvt_scalef32_pk_bf16_fp8 (two values per instruction, scale 1).
constexpr int kMfmaChunk = 1024;  // history tokens per workgroup (4 waves x 256)
constexpr int kMfmaWaveTok = kMfmaChunk / 4;
constexpr float kMaxSlack = 8.0f;  // log2 units

typedef short s16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ s16x4 e4m3x4_to_bf16x4(int w) {
  const bf16x2 lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
  const bf16x2 hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
  const bf16x4 v = {lo[0], lo[1], hi[0], hi[1]};
  return __builtin_bit_cast(s16x4, v);
}
// 4x4 byte transpose across the four lanes of a quad: out.byte[k] of lane j = in.byte[j] of lane k.
__device__ __forceinline__ int quad_transpose_bytes(int x, int lane) {
  const int t = __builtin_amdgcn_mov_dpp(x, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  const int y = __builtin_amdgcn_perm(t, x, (lane & 1) ? 0x03070105 : 0x06020400);
  const int u = __builtin_amdgcn_mov_dpp(y, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  return __builtin_amdgcn_perm(u, y, (lane & 2) ? 0x03020706 : 0x05040100);
}

// The grid is persistent: workgroups stride over the (row, chunk, KV head) items of a schedule that a tiny kernel
// builds from the rows' current lengths, so a ragged batch in a large-capacity cache launches no empty workgroups.
template <bool PAGED>
__global__ void __launch_bounds__(256) decode_attn_mfma_kernel(DecodeArgs a) {
  constexpr int D = 64;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane & 3, vq = (lane >> 2) & 3, g16 = lane >> 4;
  __shared__ __bf16 lds_p[4][4][64];
  __shared__ float sm[4][4], sl[4][4], sacc[4][4][D];
  const int items = a.schedule[0] * a.KH;
  if (items <= 0) return;
  // An item's row, chunk, length and slot sit behind three dependent loads; the next item's are fetched while the
  // current one is processed so that chain is off the critical path of every item but a workgroup's first.
  struct Meta { int b, chunk, len; int64_t slot; };
  auto load_meta = [&](int item) {
    const int pair = (item < items ? item : items - 1) / a.KH;
    Meta mt;
    mt.b = a.schedule[2 + 2 * pair];
    mt.chunk = a.schedule[3 + 2 * pair];
    mt.slot = a.slot_ids ? a.slot_ids[mt.b] : mt.b;
    mt.len = a.positions[mt.b] + 1;
    return mt;
  };
  Meta next_meta = load_meta(blockIdx.x);
  for (int item = blockIdx.x; item < items; item += gridDim.x) {
  const Meta meta = next_meta;
  next_meta = load_meta(item + gridDim.x);
  const int h = item % a.KH;
  const int b = meta.b, chunk = meta.chunk, len = meta.len;
  const int64_t slot = meta.slot;
  const int start = chunk * kMfmaChunk;

  // A operand of S = Q.K^T: Q[head g][dims 4s..4s+3] for s = 0..15 (zero rows beyond the group)
  s16x4 qop[16];
  {
    const bool ok = g < a.G;
    const __bf16* src = (const __bf16*)a.q + ((int64_t)b * a.QH + h * a.G + (ok ? g : 0)) * D;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      i32x4 w = {0, 0, 0, 0};
      if (ok) w = *reinterpret_cast<const i32x4*>(src + 8 * c);
      const i32x2 lo = {w[0], w[1]}, hi = {w[2], w[3]};
      qop[2 * c] = __builtin_bit_cast(s16x4, lo);
      qop[2 * c + 1] = __builtin_bit_cast(s16x4, hi);
    }
  }
  auto token_offset = [&](int t) -> int64_t {
    if (PAGED) {
      const int64_t blk = a.block_table[(int64_t)b * a.max_blocks + t / a.page];
      return blk * a.c0 + (int64_t)(t % a.page) * a.c1 + (int64_t)h * a.c2;
    }
    return slot * a.c0 + (int64_t)t * a.c1 + (int64_t)h * a.c2;
  };

  float m[4], l[4];
  f32x4 acc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) { m[i] = -1.0e30f; l[i] = 0.f; acc[i] = f32x4{0.f, 0.f, 0.f, 0.f}; }

  const int wbeg = start + wave * kMfmaWaveTok;
  int wend = wbeg + kMfmaWaveTok;
  wend = wend < len ? wend : len;
  const uint8_t* kbase = (const uint8_t*)a.kc;
  const uint8_t* vbase = (const uint8_t*)a.vc;
  for (int T = wbeg; T < wend; T += 64) {
    // ---- loads: this lane's K row, its scales, and its four V slices
    const int tk = T + lane;
    const bool valid = tk < wend;
    const int64_t koff = token_offset(valid ? tk : wend - 1);
    i32x4 kreg[4], vreg[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) kreg[c] = *reinterpret_cast<const i32x4*>(kbase + koff + 16 * c);
    const float sk = a.ks[koff / D], sv = a.vs[koff / D];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      int tv = T + 16 * u + 4 * g16 + g;
      tv = tv < wend ? tv : wend - 1;
      vreg[u] = *reinterpret_cast<const i32x4*>(vbase + token_offset(tv) + 16 * vq);
    }
    // ---- S[0..3][token lane]
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int w = 0; w < 4; ++w)
        s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(qop[4 * c + w], e4m3x4_to_bf16x4(kreg[c][w]), s, 0, 0, 0);
    const float kscale = a.scale_log2e * sk;
    bool raise = false;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s[i] = valid ? s[i] * kscale : -1.0e30f;
      raise |= s[i] > m[i] + kMaxSlack;
    }
    if (__any(raise)) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float mnew = fmaxf(m[i], wave_max(s[i]));
        const float alpha = __builtin_amdgcn_exp2f(m[i] - mnew);
        m[i] = mnew;
        l[i] *= alpha;
#pragma unroll
        for (int w = 0; w < 4; ++w) acc[w][i] *= alpha;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = valid ? __builtin_amdgcn_exp2f(s[i] - m[i]) : 0.f;
      l[i] += p;
      lds_p[wave][i][lane] = (__bf16)(p * sv);
    }
    // ---- O[0..3][dims 16*vq + 4w + g] += P . V over this lane group's tokens
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const i32x2 praw = *reinterpret_cast<const i32x2*>(&lds_p[wave][g][16 * u + 4 * g16]);
      const s16x4 pop = __builtin_bit_cast(s16x4, praw);
#pragma unroll
      for (int w = 0; w < 4; ++w)
        acc[w] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(pop, e4m3x4_to_bf16x4(quad_transpose_bytes(vreg[u][w], lane)), acc[w], 0, 0, 0);
    }
  }
  // ---- wave totals: l over all lanes, O over the four token groups
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    l[i] = wave_sum(l[i]);
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float v = acc[w][i];
      v = add_lane_xor32(add_lane_xor16(v));
      acc[w][i] = v;
    }
  }
  if (g16 == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int w = 0; w < 4; ++w) sacc[wave][i][16 * vq + 4 * w + g] = acc[w][i];
    }
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { sm[wave][i] = m[i]; sl[wave][i] = l[i]; }
    }
  }
  __syncthreads();
  {
    const int gi = threadIdx.x >> 6, d = threadIdx.x & 63;  // 4 heads x 64 dims = 256 threads
    if (gi < a.G) {
      float mm = sm[0][gi];
#pragma unroll
      for (int w = 1; w < 4; ++w) mm = fmaxf(mm, sm[w][gi]);
      float lt = 0.f, ot = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float f = __builtin_amdgcn_exp2f(sm[w][gi] - mm);
        lt = fmaf(sl[w][gi], f, lt);
        ot = fmaf(sacc[w][gi][d], f, ot);
      }
      const int64_t prow = ((int64_t)b * a.QH + h * a.G + gi) * a.nchunks + chunk;
      a.ws_acc[prow * D + d] = ot;
      if (d == 0) { a.ws_m[prow] = mm; a.ws_l[prow] = lt; }
    }
  }
  __syncthreads();  // the LDS tiles are reused by the next item
  }
}

// One workgroup turns the rows' lengths into the item list of the persistent kernel: row b contributes
// ceil((positions[b]+1) / chunk) items unless it is inactive or padding.
__global__ void __launch_bounds__(1024)
decode_schedule_kernel(int32_t* schedule, const int32_t* positions, const uint8_t* active, const int32_t* slot_ids, int B,
                       int chunk) {
  __shared__ int scan[1024];
  __shared__ int carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < B; base += 1024) {
    const int b = base + threadIdx.x;
    int n = 0;
    if (b < B && (!active || active[b]) && (!slot_ids || slot_ids[b] >= 0)) n = (positions[b] + chunk) / chunk;
    scan[threadIdx.x] = n;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
      const int v = threadIdx.x >= o ? scan[threadIdx.x - o] : 0;
      __syncthreads();
      scan[threadIdx.x] += v;
      __syncthreads();
    }
    const int first = carry + scan[threadIdx.x] - n;
    for (int c = 0; c < n; ++c) { schedule[2 + 2 * (first + c)] = b; schedule[3 + 2 * (first + c)] = c; }
    __syncthreads();
    if (threadIdx.x == 1023) carry += scan[1023];
    __syncthreads();
  }
  if (threadIdx.x == 0) { schedule[0] = carry; schedule[1] = chunk; }
}

// Merge the chunk partials of one (row, query head); inactive or empty rows give zeros.
template <typename T>
__global__ void __launch_bounds__(64) decode_combine_kernel(DecodeArgs a) {
  const int b = blockIdx.x, qh = blockIdx.y;
  T* out = (T*)a.out + ((int64_t)b * a.QH + qh) * a.D;
  int len = a.positions[b] + 1;
  if (a.active && !a.active[b]) len = 0;
  if (a.slot_ids && a.slot_ids[b] < 0) len = 0;
  if (len <= 0) {
    for (int d = threadIdx.x; d < a.D; d += 64) out[d] = Elem<T>::store(0.f);
    return;
  }
  const int n = (len + a.chunk - 1) / a.chunk;
  const int64_t prow = ((int64_t)b * a.QH + qh) * a.nchunks;
  float mm = -1.0e30f;
  for (int c = 0; c < n; ++c) mm = fmaxf(mm, a.ws_m[prow + c]);
  float lt = 0.f;
  for (int c = 0; c < n; ++c) lt = fmaf(a.ws_l[prow + c], exp2f(a.ws_m[prow + c] - mm), lt);
  const float inv = 1.0f / fmaxf(lt, 1.0e-20f);
  for (int d = threadIdx.x; d < a.D; d += 64) {
    float o = 0.f;
    for (int c = 0; c < n; ++c) o = fmaf(a.ws_acc[(prow + c) * a.D + d], exp2f(a.ws_m[prow + c] - mm), o);
    out[d] = Elem<T>::store(o * inv);
  }
}

// The same merge for a whole row (all query heads) followed by the row's e4m3 quantisation, for callers whose next
// step is an FP8 projection: values are rounded to the model dtype first, exactly as the two separate launches do.
// Sixteen waves per row, wave w owning query heads w, w+16, ...; with NC > 0 the chunk loops are fully unrolled over
// NC predicated iterations so that all of a lane's partial loads are in flight together (the partials were written
// by other XCDs and come from beyond the local L2, so each dependent round costs a full memory latency).
template <typename T, int NC>
__global__ void __launch_bounds__(1024) decode_combine_fp8_kernel(DecodeArgs a, uint8_t* q_out, float* q_scales) {
  constexpr int kMaxPerLane = 4, kWavesPerRow = 16;
  __shared__ float red[kWavesPerRow];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int len = a.positions[b] + 1;
  if (a.active && !a.active[b]) len = 0;
  if (a.slot_ids && a.slot_ids[b] < 0) len = 0;
  const int n = len > 0 ? (len + a.chunk - 1) / a.chunk : 0;
  const int per_head = (a.D + 63) / 64;
  float y[kMaxPerLane];
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int qh = wave + kWavesPerRow * (i / per_head), d = lane + 64 * (i % per_head);
    y[i] = 0.f;
    if (qh < a.QH && d < a.D && n > 0) {
      const int64_t prow = ((int64_t)b * a.QH + qh) * a.nchunks;
      float mm = -1.0e30f, lt = 0.f, o = 0.f;
      if constexpr (NC > 0) {
        float m[NC], l[NC], acc[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const int cc = c < n ? c : 0;
          m[c] = a.ws_m[prow + cc]; l[c] = a.ws_l[prow + cc]; acc[c] = a.ws_acc[(prow + cc) * a.D + d];
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) if (c < n) mm = fmaxf(mm, m[c]);
#pragma unroll
        for (int c = 0; c < NC; ++c) if (c < n) lt = fmaf(l[c], exp2f(m[c] - mm), lt);
#pragma unroll
        for (int c = 0; c < NC; ++c) if (c < n) o = fmaf(acc[c], exp2f(m[c] - mm), o);
      } else {
        for (int c = 0; c < n; ++c) mm = fmaxf(mm, a.ws_m[prow + c]);
        for (int c = 0; c < n; ++c) lt = fmaf(a.ws_l[prow + c], exp2f(a.ws_m[prow + c] - mm), lt);
        for (int c = 0; c < n; ++c) o = fmaf(a.ws_acc[(prow + c) * a.D + d], exp2f(a.ws_m[prow + c] - mm), o);
      }
      y[i] = round_to<T>(o * (1.0f / fmaxf(lt, 1.0e-20f)));
      amax = fmaxf(amax, fabsf(y[i]));
    }
  }
  amax = block_max<kWavesPerRow>(amax, red);
  const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
  if (threadIdx.x == 0) q_scales[b] = scale;
  uint8_t* dst = q_out + (int64_t)b * a.QH * a.D;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int qh = wave + kWavesPerRow * (i / per_head), d = lane + 64 * (i % per_head);
    if (qh < a.QH && d < a.D) dst[qh * a.D + d] = to_e4m3(y[i] / scale);
  }
}

template <typename T>
void launch_combine_fp8(const DecodeArgs& a, int64_t B, uint8_t* out_q, float* out_scales, hipStream_t s) {
  if (a.nchunks <= 8) hipLaunchKernelGGL((decode_combine_fp8_kernel<T, 8>), dim3(B), dim3(1024), 0, s, a, out_q, out_scales);
  else hipLaunchKernelGGL((decode_combine_fp8_kernel<T, 0>), dim3(B), dim3(1024), 0, s, a, out_q, out_scales);
}

// ===================================================================================== prefill attention
template <typename T> struct HalfMfma;
template <> struct HalfMfma<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ f32x4 run(vec8 a, vec8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct HalfMfma<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ f32x4 run(vec8 a, vec8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

// Flash-style causal attention on a packed varlen batch.  A workgroup owns 64 query rows of one
// (sequence, query head); wave w owns rows 16w..16w+15 and lane%16 is the lane's row throughout:
//   S^T  = K . Q^T   (A = K rows from LDS, B = Q rows in registers)  -> lane has 4 tokens x 4 subtiles of its row
//   O^T += V^T . P^T (A = V^T from the transposed LDS tile, B = P straight from the S^T registers)
// so softmax statistics never cross rows and P needs no relayout; the contraction order over the
// 64 tokens of a tile is the same permutation on both operands.
template <typename T, int D>
__global__ void __launch_bounds__(256)
prefill_attn_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                    const int32_t* __restrict__ cu, int QH, int KH, float scale_log2e) {
  typedef typename HalfMfma<T>::vec8 vec8;
  typedef T vec4 __attribute__((ext_vector_type(4)));
  constexpr int KC = D / 8;          // 16-byte chunks per K row
  constexpr int VP = 64 + 8;         // padded token stride of the transposed V tile
  __shared__ vec8 ldsK[64 * KC];
  __shared__ T ldsVt[D * VP];

  const int seq = blockIdx.z, qh = blockIdx.y, kh = qh / (QH / KH);
  const int begin = cu[seq], len = cu[seq + 1] - begin;
  const int q0 = blockIdx.x * 64;
  if (q0 >= len) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, grp = lane >> 4;
  const int qpos = q0 + wave * 16 + r;
  const int qrow = qpos < len ? qpos : len - 1;

  vec8 qf[D / 32];
#pragma unroll
  for (int kk = 0; kk < D / 32; ++kk)
    qf[kk] = *reinterpret_cast<const vec8*>(q + ((int64_t)(begin + qrow) * QH + qh) * D + 32 * kk + 8 * grp);

  f32x4 o[D / 16];
#pragma unroll
  for (int dd = 0; dd < D / 16; ++dd) o[dd] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -1.0e30f, l = 0.f;

  int kv_end = q0 + 64;
  kv_end = kv_end < len ? kv_end : len;
  for (int t0 = 0; t0 < kv_end; t0 += 64) {
    __syncthreads();
    for (int idx = tid; idx < 64 * KC; idx += 256) {
      const int tok = idx / KC, c = idx % KC;
      int gt = t0 + tok;
      gt = gt < len ? gt : len - 1;
      const int64_t src = ((int64_t)(begin + gt) * KH + kh) * D + c * 8;
      ldsK[tok * KC + (c ^ (tok & (KC - 1)))] = *reinterpret_cast<const vec8*>(k + src);
      const vec8 vv = *reinterpret_cast<const vec8*>(v + src);
#pragma unroll
      for (int e = 0; e < 8; ++e) ldsVt[(c * 8 + e) * VP + tok] = vv[e];
    }
    __syncthreads();

    f32x4 st[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      st[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      const int tok = 16 * j + r;
#pragma unroll
      for (int kk = 0; kk < D / 32; ++kk) {
        const int c = 4 * kk + grp;
        st[j] = HalfMfma<T>::run(ldsK[tok * KC + (c ^ (tok & (KC - 1)))], qf[kk], st[j]);
      }
    }
    float mx = -1.0e30f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tk = t0 + 16 * j + 4 * grp + i;
        const bool ok = tk <= qpos && tk < len;
        st[j][i] = ok ? st[j][i] * scale_log2e : -1.0e30f;
        mx = fmaxf(mx, st[j][i]);
      }
    mx = max_lane_xor32(max_lane_xor16(mx));
    const float mnew = fmaxf(m, mx);
    const float alpha = exp2f(m - mnew);
    float rs = 0.f;
    vec8 pf[2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = st[j][i] > -0.9e30f ? exp2f(st[j][i] - mnew) : 0.f;
        rs += p;
        pf[j >> 1][(j & 1) * 4 + i] = (T)p;
      }
    rs = add_lane_xor32(add_lane_xor16(rs));
    l = fmaf(l, alpha, rs);
    m = mnew;
#pragma unroll
    for (int dd = 0; dd < D / 16; ++dd) {
#pragma unroll
      for (int i = 0; i < 4; ++i) o[dd][i] *= alpha;
      const T* vrow = ldsVt + (16 * dd + r) * VP + 4 * grp;
#pragma unroll
      for (int kk2 = 0; kk2 < 2; ++kk2) {
        const vec4 lo = *reinterpret_cast<const vec4*>(vrow + 16 * (2 * kk2));
        const vec4 hi = *reinterpret_cast<const vec4*>(vrow + 16 * (2 * kk2 + 1));
        const vec8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        o[dd] = HalfMfma<T>::run(vf, pf[kk2], o[dd]);
      }
    }
  }
  if (qpos < len) {
    const float inv = 1.0f / fmaxf(l, 1.0e-20f);
    T* dst = out + ((int64_t)(begin + qpos) * QH + qh) * D;
#pragma unroll
    for (int dd = 0; dd < D / 16; ++dd) {
      vec4 w = {(T)(o[dd][0] * inv), (T)(o[dd][1] * inv), (T)(o[dd][2] * inv), (T)(o[dd][3] * inv)};
      *reinterpret_cast<vec4*>(dst + 16 * dd + 4 * grp) = w;
    }
  }
}

// ===================================================================================== token map
__global__ void __launch_bounds__(256)
token_map_kernel(int32_t* seq_of_token, int32_t* pos_of_token, const int32_t* cu, int nseq, int64_t T) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= T) return;
  int lo = 0, hi = nseq - 1;  // last seq with cu[seq] <= t
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= t) lo = mid; else hi = mid - 1;
  }
  seq_of_token[t] = lo;
  pos_of_token[t] = (int32_t)(t - cu[lo]);
}

}  // namespace

extern "C" int lfm2_store_kv_fp8(const void* k, const void* v, uint8_t* k_cache, uint8_t* v_cache, float* k_scales,
                                 float* v_scales, const int32_t* positions, const uint8_t* active,
                                 const int32_t* slot_ids, int64_t B, int64_t T_, int KH, int D, int64_t ks0, int64_t ks1,
                                 int64_t ks2, int64_t vs0, int64_t vs1, int64_t vs2, int64_t c0, int64_t c1, int64_t c2,
                                 int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && T_ > 0 && KH > 0, "store_kv_fp8: empty shape");
  if (int e = check_head_dim("store_kv_fp8", D)) return e;
  LFM2_REQUIRE(c2 % 4 == 0 && c1 % 4 == 0 && c0 % 4 == 0, "store_kv_fp8: cache strides must be multiples of 4");
  StoreArgs a{k, v, k_cache, v_cache, k_scales, v_scales, positions, slot_ids, nullptr, nullptr, active,
              T_, ks0, ks1, ks2, vs0, vs1, vs2, c0, c1, c2, KH, D};
  switch (dtype) {
    case LFM2_DTYPE_BF16: hipLaunchKernelGGL((store_kv_kernel<__bf16, true, false>), dim3(B * T_), dim3(256), 0, (hipStream_t)stream, a); break;
    case LFM2_DTYPE_F16: hipLaunchKernelGGL((store_kv_kernel<_Float16, true, false>), dim3(B * T_), dim3(256), 0, (hipStream_t)stream, a); break;
    case LFM2_DTYPE_F32: hipLaunchKernelGGL((store_kv_kernel<float, true, false>), dim3(B * T_), dim3(256), 0, (hipStream_t)stream, a); break;
    default: LFM2_FAIL(LFM2_ERR_ARGUMENT, "store_kv_fp8: unknown dtype %d", dtype);
  }
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_append_kv(const void* k, const void* v, void* k_cache, void* v_cache, const int32_t* positions,
                              const int32_t* slot_ids, const uint8_t* active, int64_t B, int KH, int D, int64_t c0,
                              int64_t c1, int64_t c2, int dtype, void* stream) {
  LFM2_REQUIRE(B > 0 && KH > 0 && positions, "append_kv: empty shape or missing positions");
  if (int e = check_head_dim("append_kv", D)) return e;
  StoreArgs a{k, v, k_cache, v_cache, nullptr, nullptr, positions, slot_ids, nullptr, nullptr, active,
              1, (int64_t)KH * D, (int64_t)KH * D, D, (int64_t)KH * D, (int64_t)KH * D, D, c0, c1, c2, KH, D};
  switch (dtype) {
    case LFM2_DTYPE_BF16: hipLaunchKernelGGL((store_kv_kernel<__bf16, false, false>), dim3(B), dim3(256), 0, (hipStream_t)stream, a); break;
    case LFM2_DTYPE_F16: hipLaunchKernelGGL((store_kv_kernel<_Float16, false, false>), dim3(B), dim3(256), 0, (hipStream_t)stream, a); break;
    case LFM2_DTYPE_F32: hipLaunchKernelGGL((store_kv_kernel<float, false, false>), dim3(B), dim3(256), 0, (hipStream_t)stream, a); break;
    default: LFM2_FAIL(LFM2_ERR_ARGUMENT, "append_kv: unknown dtype %d", dtype);
  }
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_store_kv_packed(const void* k, const void* v, void* k_cache, void* v_cache, float* k_scales,
                                    float* v_scales, const int32_t* cu_seqlens, const int32_t* seq_of_token,
                                    const int32_t* slots, int64_t T_, int KH, int D, int64_t c0, int64_t c1, int64_t c2,
                                    int kv_fp8, int dtype, void* stream) {
  LFM2_REQUIRE(T_ > 0 && KH > 0 && cu_seqlens && seq_of_token, "store_kv_packed: empty shape or missing maps");
  if (int e = check_head_dim("store_kv_packed", D)) return e;
  LFM2_REQUIRE(!kv_fp8 || (k_scales && v_scales), "store_kv_packed: e4m3 cache without scale tensors");
  StoreArgs a{k, v, k_cache, v_cache, k_scales, v_scales, nullptr, slots, cu_seqlens, seq_of_token, nullptr,
              1, 0, 0, 0, 0, 0, 0, c0, c1, c2, KH, D};
  hipStream_t s = (hipStream_t)stream;
#define SKP_(TT)                                                                                          \
  if (kv_fp8) hipLaunchKernelGGL((store_kv_kernel<TT, true, true>), dim3(T_), dim3(256), 0, s, a);        \
  else hipLaunchKernelGGL((store_kv_kernel<TT, false, true>), dim3(T_), dim3(256), 0, s, a)
  switch (dtype) {
    case LFM2_DTYPE_BF16: SKP_(__bf16); break;
    case LFM2_DTYPE_F16: SKP_(_Float16); break;
    case LFM2_DTYPE_F32: SKP_(float); break;
    default: LFM2_FAIL(LFM2_ERR_ARGUMENT, "store_kv_packed: unknown dtype %d", dtype);
  }
#undef SKP_
  LFM2_LAUNCH_CHECK();
}

static int64_t schedule_ints(int64_t B, int64_t capacity) {
  return 2 + 2 * B * ((capacity + kMfmaChunk - 1) / kMfmaChunk);
}

extern "C" int64_t lfm2_decode_attention_workspace(int64_t B, int QH, int D, int64_t capacity) {
  const int64_t nch = (capacity + kChunk - 1) / kChunk;  // the smaller chunk of the two kernels bounds both
  return B * QH * nch * (D + 2) + schedule_ints(B, capacity);
}

extern "C" int64_t lfm2_decode_schedule_size(int64_t B, int64_t capacity) { return schedule_ints(B, capacity); }

extern "C" int lfm2_decode_schedule(int32_t* schedule, const int32_t* positions, const uint8_t* active,
                                    const int32_t* slot_ids, int64_t B, void* stream) {
  LFM2_REQUIRE(B > 0 && schedule && positions, "decode_schedule: bad arguments");
  hipLaunchKernelGGL(decode_schedule_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, schedule, positions, active,
                     slot_ids, (int)B, kMfmaChunk);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_decode_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                                     const float* k_scales, const float* v_scales, const int32_t* positions,
                                     const uint8_t* active, const int32_t* slot_ids, const int32_t* block_table,
                                     int64_t max_blocks, int page, const int32_t* schedule, float* workspace, int64_t B,
                                     int QH, int KH, int D,
                                     int64_t capacity, int64_t c0, int64_t c1, int64_t c2, float scale, int kv_fp8,
                                     int dtype, uint8_t* out_q, float* out_scales, void* stream) {
  LFM2_REQUIRE(B > 0 && QH > 0 && KH > 0 && capacity > 0, "decode_attention: empty shape");
  LFM2_REQUIRE((out_q == nullptr) == (out_scales == nullptr), "decode_attention: quantised output needs values and scales");
  LFM2_REQUIRE(out_q != nullptr || out != nullptr, "decode_attention: no output");
  LFM2_REQUIRE(out_q == nullptr || (int64_t)((QH + 15) / 16) * ((D + 63) / 64) <= 4, "decode_attention: quantised output supports at most 4096 values per row");
  LFM2_REQUIRE(QH % KH == 0, "decode_attention: %d query heads not divisible by %d KV heads", QH, KH);
  LFM2_REQUIRE(positions && workspace, "decode_attention: positions and workspace are required");
  LFM2_REQUIRE(!kv_fp8 || (k_scales && v_scales), "decode_attention: e4m3 history without scales");
  LFM2_REQUIRE(!block_table || (page > 0 && max_blocks > 0), "decode_attention: bad page geometry");
  LFM2_REQUIRE(B <= 65535, "decode_attention: more than 65535 rows");
  if (int e = check_head_dim("decode_attention", D)) return e;
  const int align = kv_fp8 ? 16 : 8;
  LFM2_REQUIRE(c0 % align == 0 && c1 % align == 0 && c2 % align == 0, "decode_attention: cache strides must be multiples of %d elements", align);
  const int G = QH / KH;
  const bool mfma = kv_fp8 && D == 64 && G <= 4 && dtype == LFM2_DTYPE_BF16;
  const int chunk = mfma ? kMfmaChunk : kChunk;
  const int nch = (int)((capacity + chunk - 1) / chunk);
  DecodeArgs a;
  a.out = out; a.q = q; a.kc = k_cache; a.vc = v_cache; a.ks = k_scales; a.vs = v_scales;
  a.positions = positions; a.slot_ids = slot_ids; a.block_table = block_table; a.active = active;
  a.ws_acc = workspace;
  a.ws_m = workspace + B * QH * nch * D;
  a.ws_l = a.ws_m + B * QH * nch;
  a.schedule = nullptr;
  a.max_blocks = max_blocks; a.c0 = c0; a.c1 = c1; a.c2 = c2;
  a.page = page; a.QH = QH; a.KH = KH; a.D = D; a.G = G; a.nchunks = nch; a.chunk = chunk;
  a.scale_log2e = scale * LFM2_LOG2E;
  hipStream_t s = (hipStream_t)stream;
  if (mfma) {
    if (schedule == nullptr) {  // no shared schedule from the caller: build one in the tail of the workspace
      int32_t* own = reinterpret_cast<int32_t*>(workspace + B * QH * ((capacity + kChunk - 1) / kChunk) * (D + 2));
      hipLaunchKernelGGL(decode_schedule_kernel, dim3(1), dim3(1024), 0, s, own, positions, active, slot_ids, (int)B, kMfmaChunk);
      schedule = own;
    }
    a.schedule = schedule;
    // 3 workgroups per CU is what the kernel's register use allows on the 256 CUs; never more than the worst case
    int64_t blocks = (int64_t)B * nch * KH;
    blocks = blocks < 768 ? blocks : 768;
    const dim3 mgrid((unsigned)blocks);
    if (block_table) hipLaunchKernelGGL(decode_attn_mfma_kernel<true>, mgrid, dim3(256), 0, s, a);
    else hipLaunchKernelGGL(decode_attn_mfma_kernel<false>, mgrid, dim3(256), 0, s, a);
    if (out_q) launch_combine_fp8<__bf16>(a, B, out_q, out_scales, s);
    else hipLaunchKernelGGL(decode_combine_kernel<__bf16>, dim3(B, QH), dim3(64), 0, s, a);
    LFM2_LAUNCH_CHECK();
  }
  const dim3 grid(nch, KH * ((G + kGB - 1) / kGB), B);
#define DEC_(DD)                                                                                     \
  if (kv_fp8) hipLaunchKernelGGL((decode_attn_kernel<T, true, DD>), grid, dim3(256), 0, s, a);       \
  else hipLaunchKernelGGL((decode_attn_kernel<T, false, DD>), grid, dim3(256), 0, s, a)
  DISPATCH_HALF(dtype, "decode_attention", switch (D) {
    case 32: DEC_(32); break;
    case 64: DEC_(64); break;
    case 128: DEC_(128); break;
    default: DEC_(256); break;
  } if (out_q) launch_combine_fp8<T>(a, B, out_q, out_scales, s);
    else hipLaunchKernelGGL(decode_combine_kernel<T>, dim3(B, QH), dim3(64), 0, s, a));
#undef DEC_
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_prefill_attention(void* out, const void* q, const void* k, const void* v, const int32_t* cu_seqlens,
                                      int64_t nseq, int64_t max_seqlen, int QH, int KH, int D, float scale, int dtype,
                                      void* stream) {
  LFM2_REQUIRE(nseq > 0 && max_seqlen > 0 && QH > 0 && KH > 0, "prefill_attention: empty shape");
  LFM2_REQUIRE(QH % KH == 0, "prefill_attention: %d query heads not divisible by %d KV heads", QH, KH);
  LFM2_REQUIRE(nseq <= 65535 && QH <= 65535, "prefill_attention: grid too large");
  LFM2_REQUIRE(D == 32 || D == 64 || D == 128, "prefill_attention: head_dim %d not in {32,64,128}", D);
  const dim3 grid(ceil_div(max_seqlen, 64), QH, nseq);
  hipStream_t s = (hipStream_t)stream;
  const float sl = scale * LFM2_LOG2E;
#define PRE_(DD) hipLaunchKernelGGL((prefill_attn_kernel<T, DD>), grid, dim3(256), 0, s, (T*)out, (const T*)q, (const T*)k, (const T*)v, cu_seqlens, QH, KH, sl)
  DISPATCH_HALF(dtype, "prefill_attention", switch (D) {
    case 32: PRE_(32); break;
    case 64: PRE_(64); break;
    default: PRE_(128); break;
  });
#undef PRE_
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_build_token_map(int32_t* seq_of_token, int32_t* pos_of_token, const int32_t* cu_seqlens, int64_t nseq,
                                    int64_t T_, void* stream) {
  LFM2_REQUIRE(nseq > 0 && T_ > 0, "build_token_map: empty shape");
  hipLaunchKernelGGL(token_map_kernel, dim3(ceil_div(T_, 256)), dim3(256), 0, (hipStream_t)stream, seq_of_token,
                     pos_of_token, cu_seqlens, (int)nseq, T_);
  LFM2_LAUNCH_CHECK();
}
