// KV-cache writes, ragged GQA decode attention (split over the history) and varlen causal prefill
// attention for the LFM2 attention layers.
//
// Cache addressing follows the reference's strided views: element (slot, pos, head, d) of a layer
// lives at slot*c0 + pos*c1 + head*c2 + d, and the e4m3 scale of (slot, pos, head) at that offset
// divided by D.  With a block table, c0 is the page stride and pos is the in-page index.
#include "lfm2_common.h"
#include <type_traits>

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

// Schedule layout (int32): [0] number of (row, chunk) pairs; [1] tokens per chunk (the kernel that builds the list
// picks 256 or 512 from the rows' lengths); from kSchedRows on one 16-byte record per row (index of
// the pair of its first full chunk, index of the pair of its partial chunk, its length or 0 when it sits out, 0);
// then one 16-byte record per pair (row, chunk, length, slot).
constexpr int kSchedRows = 4;
struct DecodeArgs {
  void* out;
  const void *q, *kc, *vc;
  const float *ks, *vs;
  const int32_t *positions, *slot_ids, *block_table;
  const uint8_t* active;
  float *ws_acc, *ws_m, *ws_l;
  const int32_t* schedule;  // work list of the scheduled kernel (layout above); null for the generic kernel
  int64_t max_blocks, c0, c1, c2;
  int page, QH, KH, D, G, nchunks, chunk, B;
  float scale_log2e;
};

// Row of the partial-result arrays that holds chunk c of (row b, query head qh).  The generic kernel's rows are dense,
// [b][qh][chunk]; the scheduled kernel's are [pair][qh], so that one item's heads are one contiguous block.
struct RowPairs { int full_first, partial, nfull, len, chunk; };
// The row's length (0: inactive, padding or empty) and, for the scheduled kernel, where its partial results are:
// one load of the row's record there, the rows' own arrays otherwise.
__device__ __forceinline__ RowPairs row_pairs(const DecodeArgs& a, int b) {
  RowPairs r{0, 0, 0, 0, a.chunk};
  if (a.schedule) {
    const i32x4 rec = *reinterpret_cast<const i32x4*>(a.schedule + kSchedRows + 4 * b);
    r.chunk = a.schedule[1];
    r.full_first = rec[0]; r.partial = rec[1]; r.len = rec[2]; r.nfull = rec[2] / r.chunk;
    return r;
  }
  r.len = a.positions[b] + 1;
  if (a.active && !a.active[b]) r.len = 0;
  if (a.slot_ids && a.slot_ids[b] < 0) r.len = 0;
  return r;
}
__device__ __forceinline__ int64_t partial_row(const DecodeArgs& a, const RowPairs& r, int b, int qh, int c) {
  if (!a.schedule) return ((int64_t)b * a.QH + qh) * a.nchunks + c;
  return (int64_t)(c < r.nfull ? r.full_first + c : r.partial) * a.QH + qh;
}

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
constexpr int kMfmaChunk = 256;      // history tokens per item (one wave) ...
constexpr int kMfmaLongChunk = 512;  // ... or this many, when the batch holds at least kLongPairs items of the short kind:
constexpr int kLongPairs = 3072;     // with enough items for every wave, longer ones halve the partial results and their merge
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

// The grid is persistent and its unit is the wave: every wave works on its own through (row, chunk, KV head) items of
// a schedule that a tiny kernel builds from the rows' current lengths, and writes its item's partial result itself.
// A ragged batch in a large-capacity cache therefore launches no empty work, and no wave ever waits at a barrier
// for a neighbour with a longer piece of history.
//
// What the kernel can draw from memory is bounded by the bytes its waves have in flight, so a wave treats its items
// as one stream of 64-token tiles and always has the next tile of the stream on its way while it multiplies the
// current one, across item boundaries too:
//   * a wave's items are its own index plus multiples of the number of waves; the schedule lists the items by
//     decreasing length (in tiles), so every wave gets the same work to within a tile or two without a work queue
//     (a counter's returned value would sit in a register that no wait protects across a whole item);
//   * an item's 16-byte record (row, chunk, length, slot) is read through the scalar cache one item ahead;
//   * the next item's first tile goes into the spare tile registers while the current item's last tile is
//     multiplied, and with every tile come eight bytes per lane of the queries of the item it belongs to, which
//     the wave puts into LDS when it starts that item (the query operands are read from there for every tile
//     rather than held in 32 registers).
// Loads are never issued under a condition (a branch around loads makes every later wait a wait for all of them),
// and nothing is loaded straight into LDS (with such a load in flight the compiler waits for all loads at once).
struct ItemRecord { int b, chunk, len, slot; };

template <bool PAGED, bool FP8, bool ROWHEAD = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) decode_attn_mfma_kernel(DecodeArgs a) {
  // ROWHEAD: a workgroup owns one (row, KV head): its four waves take the history's tiles round robin, merge their
  // four partial results through LDS and write the row's output themselves; no partial results leave the chip and no
  // merge launch follows.  Rows are taken by rank of length, longest first.
  constexpr int D = 64;
  constexpr int TT = FP8 ? 64 : 32;   // tokens per tile: 4 KiB of K rows and 4 KiB of V rows either way
  constexpr int ES = FP8 ? 1 : 2;     // bytes per element of the history
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // item state lives in scalar registers
  const int g = lane & 3, vq = (lane >> 2) & 3, g16 = lane >> 4;
  __shared__ __bf16 lds_p[4][4][64];   // one P tile per wave; nothing in LDS is shared between waves
  __shared__ __attribute__((aligned(16))) uint8_t lds_v[4][TT][D * ES];   // per wave: the tile's V rows, for the transposing read
  __shared__ __attribute__((aligned(16))) __bf16 lds_q[4][4][D];          // per wave: the item's query rows
  __shared__ float lds_merge[ROWHEAD ? 4 : 1][4][D + 2];   // per wave and head: O[dim], then the maximum and the sum
  const int32_t* const records = a.schedule + kSchedRows + 4 * a.B;
  const int items = ROWHEAD ? 1 : a.schedule[0] * a.KH;
  const int first = ROWHEAD ? 0 : blockIdx.x * 4 + wave, nwaves = gridDim.x * 4;
  if (first >= items) return;
  constexpr int kStride = ROWHEAD ? 4 * TT : TT;   // from one tile of a wave to its next

  // ---- the pieces of the pipeline
  // An item's record comes through the scalar cache (nothing writes the records while this kernel runs, so they are
  // read as constant memory): scalar loads have their own counter and do not queue behind the tile loads.
  auto read_record = [&](int idx) {
    const int pair = (idx < items ? idx : items - 1) / a.KH;
    const uint64_t address = (uint64_t)(records + 4 * (int64_t)pair);   // the same in every lane; say so to the compiler
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)address), hi = __builtin_amdgcn_readfirstlane((uint32_t)(address >> 32));
    return *reinterpret_cast<const __attribute__((address_space(4))) i32x4*>(((uint64_t)hi << 32) | lo);
  };
  auto token_offset = [&](int b, int64_t slot, int h, int t) -> int64_t {
    if (PAGED) {
      const int64_t blk = a.block_table[(int64_t)b * a.max_blocks + t / a.page];
      return blk * a.c0 + (int64_t)(t % a.page) * a.c1 + (int64_t)h * a.c2;
    }
    return slot * a.c0 + (int64_t)t * a.c1 + (int64_t)h * a.c2;
  };
  const uint8_t* kbase = (const uint8_t*)a.kc;
  const uint8_t* vbase = (const uint8_t*)a.vc;
  struct Tile { i32x4 k[4], v[4]; float sk, sv; i32x2 q; };
  // this lane's K row, its scales, and its four V slices of the tile at T (tokens clamped to the item's last).
  // e4m3 history: lane L owns token L of 64 (a 64-byte row) and the V slices of tokens 16u + L / 16 * 4 + L % 4.
  // 16-bit history: lane L owns dims 32 (L / 32) .. + 31 of token L % 32 (64 bytes of a 128-byte row) and 16 bytes
  // of the V rows of tokens 8u + L / 8.
  const int tl = FP8 ? lane : (lane & 31);              // this lane's token within a tile
  const int krow_byte = FP8 ? 0 : 64 * (lane >> 5);     // where its share of a K row starts
  const int vtok = FP8 ? 4 * g16 + g : (lane >> 3), vstep = FP8 ? 16 : 8, vbyte = FP8 ? 16 * vq : 16 * (lane & 7);
  auto fetch = [&](int b, int64_t slot, int h, int T, int wend, Tile& t) {
    int tk = T + tl;
    tk = tk < wend ? tk : wend - 1;
    if (PAGED) {
      const int64_t koff = token_offset(b, slot, h, tk);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if constexpr (FP8) {   // a quarter row of token 16c + lane / 4: see the dense form below
          int tc = T + 16 * c + (lane >> 2);
          tc = tc < wend ? tc : wend - 1;
          t.k[c] = *reinterpret_cast<const i32x4*>(kbase + token_offset(b, slot, h, tc) + 16 * (lane & 3));
        } else {
          int tc = T + 8 * c + (lane >> 3);
          tc = tc < wend ? tc : wend - 1;
          t.k[c] = *reinterpret_cast<const i32x4*>(kbase + token_offset(b, slot, h, tc) * ES + 16 * (lane & 7));
        }
      }
      if constexpr (FP8) {
        t.sk = a.ks[koff / D];
        t.sv = a.vs[koff / D];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        int tv = T + vstep * u + vtok;
        tv = tv < wend ? tv : wend - 1;
        t.v[u] = *reinterpret_cast<const i32x4*>(vbase + token_offset(b, slot, h, tv) * ES + vbyte);
      }
    } else {
      // the item's base is the same in every lane (scalar registers); a lane adds a 32-bit offset (the host checks
      // that a slot's history spans less than 2 GiB and that the strides are whole scale rows)
      const int64_t item_base = slot * a.c0 + (int64_t)h * a.c2;
      const uint8_t* kitem = kbase + item_base * ES;
      const uint8_t* vitem = vbase + item_base * ES;
      const uint32_t row_bytes = (uint32_t)a.c1 * ES;
      const uint32_t koff = (uint32_t)tk * row_bytes + krow_byte;
      // a history is read once per step and is far larger than the caches: non-temporal loads (streaming reads of
      // this size run at 6.6-6.9 TB/s with the hint against 5.9-6.1 without)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if constexpr (FP8) {
          // the K tile as 4 x 1 KiB of consecutive bytes: load c brings lane L the quarter row L % 4 of token
          // 16c + L / 4, so every instruction asks for whole cache lines; the rows are put back together through LDS
          int tc = T + 16 * c + (lane >> 2);
          tc = tc < wend ? tc : wend - 1;
          t.k[c] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(kitem + (uint32_t)tc * row_bytes + 16 * (lane & 3)));
        } else {   // 16-bit rows: load c brings lane L the eighth L % 8 of the 128-byte row of token 8c + L / 8
          int tc = T + 8 * c + (lane >> 3);
          tc = tc < wend ? tc : wend - 1;
          t.k[c] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(kitem + (uint32_t)tc * row_bytes + 16 * (lane & 7)));
        }
      }
      if constexpr (FP8) {
        const float* ks_item = a.ks + item_base / D;
        const float* vs_item = a.vs + item_base / D;
        const uint32_t soff = (uint32_t)tk * (uint32_t)(a.c1 / D);
        t.sk = __builtin_nontemporal_load(ks_item + soff);
        t.sv = __builtin_nontemporal_load(vs_item + soff);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        int tv = T + vstep * u + vtok;
        tv = tv < wend ? tv : wend - 1;
        t.v[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4*>(vitem + (uint32_t)tv * row_bytes + vbyte));
      }
    }
    if constexpr (!FP8) { t.sk = 1.f; t.sv = 1.f; }
    // this lane's share of the item's queries: head g (clamped into the tensor), dims 4 (lane / 4) .. + 3
    int row = h * a.G + g;
    row = row < a.QH ? row : a.QH - 1;
    t.q = *reinterpret_cast<const i32x2*>((const __bf16*)a.q + ((int64_t)b * a.QH + row) * D + 4 * (lane >> 2));
  };
  // Operand B of O += P.V needs, per lane, consecutive tokens of one dim, and V rows hold consecutive dims of one
  // token.  The tile's rows go to LDS as they are and come back through ds_read_b64_tr_b8: within 16 lanes, lane s
  // receives byte s % 8 of the eight 8-byte pieces that lanes 2j + s / 8 (j = 0..7) point at.  With lane p pointing
  // at row p / 2, bytes 8 (p % 2) .. + 7 of a 16-dim column block, lane s gets 8 tokens of dim s: lane L of the
  // wave owns dim L for the whole tile and the item.
  // The 16-bit form, ds_read_b64_tr_b16, gives lane s element s % 4 of the four 8-byte pieces that lanes
  // 4j + s / 4 (j = 0..3) point at: with lane p pointing at row p / 4, bytes 8 (p % 4) .. + 7 of a 16-dim column
  // block, lane s gets 4 tokens of dim s.
  const int s16 = lane & 15;
  const uint8_t* v_piece = FP8 ? &lds_v[wave][s16 >> 1][16 * g16 + 8 * (s16 & 1)]
                               : &lds_v[wave][s16 >> 2][32 * g16 + 8 * (s16 & 3)];

  // ---- prologue: the first item, the second item's record, the first tile
  int idx = first, idx_next = first + nwaves;
  int b, chunk, len, h;
  int64_t slot;
  i32x4 rec_next;
  int chunk_tokens, wbeg, wend;
  if constexpr (ROWHEAD) {
    // workgroup ids are dealt round robin over the 8 XCDs: the KV heads of one row go to one XCD, one after the other,
    // so that with token-major histories (a token's heads share cache lines) the heads meet in one L2
    const int stream = blockIdx.x / 8;
    const int rank = 8 * (stream / a.KH) + (int)(blockIdx.x % 8);
    h = stream % a.KH;
    if (rank >= a.B) return;
    b = a.schedule[kSchedRows + 4 * rank + 3];
    len = a.schedule[kSchedRows + 4 * b + 2];
    slot = a.slot_ids ? a.slot_ids[b] : b;
    chunk = 0; chunk_tokens = 0; rec_next = i32x4{0, 0, 0, 0};
    wbeg = wave * TT;
    wend = len;
    if (len <= 0) {   // a row that sits out: zeros, as the merge kernel writes them (the same for the whole workgroup)
      if (wave < a.G) ((__bf16*)a.out)[((int64_t)b * a.QH + h * a.G + wave) * D + lane] = (__bf16)0.f;
      return;
    }
  } else {
    const i32x4 rec = read_record(idx);
    b = rec[0]; chunk = rec[1]; len = rec[2]; slot = rec[3]; h = idx % a.KH;
    rec_next = read_record(idx_next);
    chunk_tokens = a.schedule[1];
    wbeg = chunk * chunk_tokens;
    wend = wbeg + chunk_tokens;
    wend = wend < len ? wend : len;
  }
  Tile tile, ahead;
  const bool has_tiles = !ROWHEAD || wbeg < wend;   // the same for the whole wave
  if (has_tiles) fetch(b, slot, h, wbeg, wend, tile);

  float m[4], l[4];
  f32x4 acc;   // O[head 0..3][dim lane]
  int T = wbeg;
  // One tile of the stream: `cur` holds it, the tile after it is fetched into `nxt`.  Returns false after the
  // wave's last item.  (Two calls with the tiles swapped make the loop body, so no tile is ever copied: a copy of
  // registers that a load is still filling would wait for the load.)
  auto step = [&](Tile& cur, Tile& nxt) __attribute__((always_inline)) -> bool {
    if (T == wbeg) {   // ---- item start: the queries that came with this tile
      *reinterpret_cast<i32x2*>(&lds_q[wave][g][4 * (lane >> 2)]) = cur.q;
#pragma unroll
      for (int i = 0; i < 4; ++i) { m[i] = -1.0e30f; l[i] = 0.f; }
      acc = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // ---- the next tile of the stream: this item's, or the first of the next item (its record was asked for one
    // item ago)
    const bool last = T + kStride >= wend;
    int nb = b, nlen = len, nh = h, nwbeg = wbeg, nwend = wend;
    int64_t nslot = slot;
    const bool have_next = !ROWHEAD && last && idx_next < items;
    if (have_next) {
      nb = rec_next[0]; nlen = rec_next[2]; nslot = rec_next[3]; nh = idx_next % a.KH;
      nwbeg = rec_next[1] * chunk_tokens;
      nwend = nwbeg + chunk_tokens;
      nwend = nwend < nlen ? nwend : nlen;
    }
    // (without a next item the fetch still has to be issued: every lane then asks for the item's last token, one
    // line per operand; the whole last tile again would be fetched from memory a second time, since non-temporal
    // loads leave nothing behind in the caches)
    const int fT = last ? (have_next ? nwbeg : nwend - 1) : T + kStride;
    fetch(nb, nslot, nh, fT, nwend, nxt);

    const bool valid = T + tl < wend;
    const float sk = cur.sk, sv = cur.sv;
    // ---- S[0..3][token lane].  A operand: Q[head g][dims 4s..4s+3] for s = 0..15, read from LDS for every tile
    // rather than held in 32 registers (rows beyond the group hold a neighbouring head's queries: their results are
    // computed and never stored).
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    if constexpr (!FP8) {
      // 16-bit history: a lane's K registers hold dims 32 (lane / 32) + 8c .. + 7; the two halves of the wave each
      // sum over their 32 dims and exchange the sums
      const __bf16* qrow = &lds_q[wave][g][32 * (lane >> 5)];
      // the K row eighths go to LDS as they arrived and come back as half rows (the wave's V buffer; the V rows are
      // stored after these reads).  The 16-byte column of a row is XORed with bits 1..3 of its token: the 16 stores
      // and the 16 loads that share a cycle then fall on distinct banks.
#pragma unroll
      for (int c = 0; c < 4; ++c)
        *reinterpret_cast<i32x4*>(&lds_v[wave][8 * c + (lane >> 3)][16 * ((lane & 7) ^ (((8 * c + (lane >> 3)) >> 1) & 7))]) = cur.k[c];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const i32x4 kr = *reinterpret_cast<const i32x4*>(&lds_v[wave][tl][16 * ((4 * (lane >> 5) + c) ^ ((tl >> 1) & 7))]);
        const i32x4 q8 = *reinterpret_cast<const i32x4*>(qrow + 8 * c);
        const i32x2 qa = {q8[0], q8[1]}, qb = {q8[2], q8[3]};
        const i32x2 ka = {kr[0], kr[1]}, kb = {kr[2], kr[3]};
        s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, qa), __builtin_bit_cast(s16x4, ka), s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, qb), __builtin_bit_cast(s16x4, kb), s, 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) s[i] = add_lane_xor32(s[i]);
    } else {
    // the K quarter rows go to LDS as they arrived and come back as rows: lane L owns token L.  The 16-byte column of
    // a row is XORed with bits 2..3 of its token, which spreads both the 16 stores and the 16 loads that share a cycle
    // over all banks.  The buffer is the wave's V buffer: the V rows are stored after these reads.
#pragma unroll
    for (int c = 0; c < 4; ++c)
      *reinterpret_cast<i32x4*>(&lds_v[wave][16 * c + (lane >> 2)][16 * ((lane & 3) ^ (g16 & 3))]) = cur.k[c];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const i32x4 kr = *reinterpret_cast<const i32x4*>(&lds_v[wave][lane][16 * (c ^ ((lane >> 2) & 3))]);
      const i32x4 q4 = *reinterpret_cast<const i32x4*>(&lds_q[wave][g][16 * c]);       // dims 16c .. 16c+7
      const i32x4 q5 = *reinterpret_cast<const i32x4*>(&lds_q[wave][g][16 * c + 8]);   // dims 16c+8 .. 16c+15
      const i32x2 qa = {q4[0], q4[1]}, qb = {q4[2], q4[3]}, qc = {q5[0], q5[1]}, qd = {q5[2], q5[3]};
      s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, qa), e4m3x4_to_bf16x4(kr[0]), s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, qb), e4m3x4_to_bf16x4(kr[1]), s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, qc), e4m3x4_to_bf16x4(kr[2]), s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, qd), e4m3x4_to_bf16x4(kr[3]), s, 0, 0, 0);
    }
    }
    // the tile's V rows to LDS, as they arrived (row = token, 16 bytes per lane)
#pragma unroll
    for (int u = 0; u < 4; ++u) *reinterpret_cast<i32x4*>(&lds_v[wave][vstep * u + vtok][vbyte]) = cur.v[u];
    const float kscale = FP8 ? a.scale_log2e * sk : a.scale_log2e;
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
        acc[i] *= alpha;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p = valid ? __builtin_amdgcn_exp2f(s[i] - m[i]) : 0.f;
      if constexpr (FP8) {
        l[i] += p;
        lds_p[wave][i][lane] = (__bf16)(p * sv);
      } else {   // both halves of the wave hold the tile's 32 probabilities: count them once
        l[i] += lane < 32 ? p : 0.f;
        lds_p[wave][i][tl] = (__bf16)p;
      }
    }
    // ---- O[0..3][dim lane] += P . V, eight (e4m3) or four (16-bit) tokens per transposing read
    if constexpr (!FP8) {
#pragma unroll
      for (int tb = 0; tb < 8; ++tb) {
        const s16x4 vt = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4*)(v_piece + tb * 4 * D * ES));
        const i32x2 praw = *reinterpret_cast<const i32x2*>(&lds_p[wave][g][4 * tb]);
        acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, praw), vt, acc, 0, 0, 0);
      }
    } else {
#pragma unroll
    for (int tb = 0; tb < 8; ++tb) {
      const i32x2 vt = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) i32x2*)(v_piece + tb * 8 * D));
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const i32x2 praw = *reinterpret_cast<const i32x2*>(&lds_p[wave][g][8 * tb + 4 * half]);
        acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, praw), e4m3x4_to_bf16x4(vt[half]), acc, 0, 0, 0);
      }
    }
    }
    T += kStride;
    if (!last) return true;

    // ---- item end.  Wave totals of l; lane L holds O[head 0..3][dim L], so a head's row leaves as 256 contiguous bytes
#pragma unroll
    for (int i = 0; i < 4; ++i) l[i] = wave_sum(l[i]);
    if constexpr (ROWHEAD) {   // this wave's share of the (row, KV head) is done: its partial result waits in LDS
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lds_merge[wave][i][lane] = acc[i];
        if (lane == 0) { lds_merge[wave][i][D] = m[i]; lds_merge[wave][i][D + 1] = l[i]; }
      }
      return false;
    }
    // The partial results leave through hand-written stores.  Reads and writes share one counter and complete out
    // of order with respect to each other, so with a store it knows of in flight the compiler turns every wait for
    // a load into a wait for everything, which would stop the stream at each item.  Unknown to it, a pending store
    // only makes a counted wait stricter: loads still complete in order among themselves.
    {
      const int64_t prow = (int64_t)(idx / a.KH) * a.QH + h * a.G;
      float* dst = a.ws_acc + prow * D + lane;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (i < a.G) asm volatile("global_store_dword %0, %1, off" : : "v"(dst + i * D), "v"(acc[i]) : "memory");
      if (lane < a.G) {   // the heads' maxima and sums are the same in every lane: lane i stores head i's
        const float mv = lane == 0 ? m[0] : lane == 1 ? m[1] : lane == 2 ? m[2] : m[3];
        const float lv = lane == 0 ? l[0] : lane == 1 ? l[1] : lane == 2 ? l[2] : l[3];
        asm volatile("global_store_dword %0, %1, off" : : "v"(a.ws_m + prow + lane), "v"(mv) : "memory");
        asm volatile("global_store_dword %0, %1, off" : : "v"(a.ws_l + prow + lane), "v"(lv) : "memory");
      }
    }
    // ---- step to the next item; ask for the record of the one after it
    if (!have_next) return false;
    idx = idx_next;
    b = nb; len = nlen; slot = nslot; h = nh; wbeg = nwbeg; wend = nwend;
    T = wbeg;
    idx_next = idx + nwaves;
    rec_next = read_record(idx_next);
    return true;
  };
  if (has_tiles) {
    while (step(tile, ahead) && step(ahead, tile)) {}
  }
  if constexpr (ROWHEAD) {
    if (!has_tiles) {   // a history shorter than this wave's first tile: a neutral partial result
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lds_merge[wave][i][lane] = 0.f;
        if (lane == 0) { lds_merge[wave][i][D] = -1.0e30f; lds_merge[wave][i][D + 1] = 0.f; }
      }
    }
    __syncthreads();
    // wave w merges query head w of the group over the four partial results: lane = dim, one 128-byte row out
    if (wave < a.G) {
      float mm = -1.0e30f;
#pragma unroll
      for (int p = 0; p < 4; ++p) mm = fmaxf(mm, lds_merge[p][wave][D]);
      float lt = 0.f, o = 0.f;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const float f = __builtin_amdgcn_exp2f(lds_merge[p][wave][D] - mm);
        lt = fmaf(lds_merge[p][wave][D + 1], f, lt);
        o = fmaf(lds_merge[p][wave][lane], f, o);
      }
      ((__bf16*)a.out)[((int64_t)b * a.QH + h * a.G + wave) * D + lane] = (__bf16)(o * (1.0f / fmaxf(lt, 1.0e-20f)));
    }
  }
}

// One workgroup turns the rows' lengths into the item list of the persistent kernel: row b contributes
// ceil((positions[b]+1) / chunk) items unless it is inactive or padding.  Items are listed by decreasing length in
// 64-token tiles: all full chunks first, then the rows' last, partial chunks of 4, 3, 2 and 1 tiles.  Waves take the
// items round robin, so the r-th items of all waves are (nearly) equally long and every wave gets the same work.
// One counting sweep over the rows gives the classes' sizes, a second one places the rows: in each, a thread's rank
// within its class comes from a wave scan and the waves' totals.
constexpr int kSchedClasses = 9;   // full chunks, then partial chunks of 8 (512-token chunks only), 7, ... 1 tiles
__device__ __forceinline__ void
schedule_rows(int32_t* schedule, const int32_t* positions, const uint8_t* active, const int32_t* slot_ids, int B) {
  __shared__ int wave_total[kSchedClasses][16];
  __shared__ int class_base[kSchedClasses + 1];   // where each class starts; running, during the second sweep
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pairs_at = kSchedRows + 4 * B;
  auto read_length = [&](int b) {
    int len = 0;
    if (b < B && (!active || active[b]) && (!slot_ids || slot_ids[b] >= 0)) len = positions[b] + 1;
    return len > 0 ? len : 0;
  };
  // every sweep below hands row base + threadIdx.x to this thread: the first 1024 rows (every decode batch) are read
  // from memory once, not once per sweep (each read is a round trip the next phase would wait for)
  const int first_length = read_length(threadIdx.x);
  auto row_length = [&](int b) { return b == (int)threadIdx.x ? first_length : read_length(b); };
  // sweep 0: the chunk size, from the number of items the rows would make at the short one
  int short_items = 0;
  for (int base = 0; base < B; base += 1024) short_items += (row_length(base + threadIdx.x) + kMfmaChunk - 1) / kMfmaChunk;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) short_items += __shfl_xor(short_items, o, 64);
  if (lane == 0) wave_total[0][wave] = short_items;
  __syncthreads();
  short_items = 0;
  for (int w = 0; w < 16; ++w) short_items += wave_total[0][w];
  __syncthreads();
  const int chunk = short_items >= kLongPairs ? kMfmaLongChunk : kMfmaChunk;
  const int tiles_per_chunk = chunk / 64;
  auto classify = [&](int len, int* n) {   // how many items of each class the row contributes
#pragma unroll
    for (int k = 0; k < kSchedClasses; ++k) n[k] = 0;
    n[0] = len / chunk;
    const int rest_tiles = (len % chunk + 63) / 64;
    if (rest_tiles > 0) {
      const int k = tiles_per_chunk + 1 - rest_tiles;   // 1 .. tiles_per_chunk
#pragma unroll
      for (int c = 1; c < kSchedClasses; ++c) n[c] = c == (k < kSchedClasses ? k : kSchedClasses - 1);
    }
  };
  // sweep 1: class sizes
  int mine[kSchedClasses] = {};
  for (int base = 0; base < B; base += 1024) {
    int n[kSchedClasses];
    classify(row_length(base + threadIdx.x), n);
#pragma unroll
    for (int k = 0; k < kSchedClasses; ++k) mine[k] += n[k];
  }
  // a row has at most one partial chunk, so with one row per thread (B <= 1024, every decode batch) the partial
  // classes are counted with ballots instead of shuffle trees; only the full-chunk counts need a sum
  const bool one_sweep = B <= 1024;
#pragma unroll
  for (int k = 0; k < kSchedClasses; ++k) {
    int v = mine[k];
    if (k > 0 && one_sweep) {
      v = __popcll(__ballot(v != 0));
    } else {
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    }
    if (lane == 0) wave_total[k][wave] = v;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int k = 0; k < kSchedClasses; ++k) {
      class_base[k] = at;
      for (int w = 0; w < 16; ++w) at += wave_total[k][w];
    }
    class_base[kSchedClasses] = at;
    schedule[0] = at;
    schedule[1] = chunk;
  }
  __syncthreads();
  // sweep 2: places
  for (int base = 0; base < B; base += 1024) {
    const int b = base + threadIdx.x;
    const int len = row_length(b);
    int n[kSchedClasses], before[kSchedClasses];
    classify(len, n);
    const unsigned long long below = (1ull << lane) - 1;
#pragma unroll
    for (int k = 0; k < kSchedClasses; ++k) {   // exclusive scan over the wave, and the wave's total
      if (k > 0) {                              // 0 or 1 per row: positions of the set lanes
        const unsigned long long set = __ballot(n[k] != 0);
        before[k] = __popcll(set & below);
        if (lane == 63) wave_total[k][wave] = __popcll(set);
      } else {
        int v = n[k];
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const int up = __shfl_up(v, o, 64);
          if (lane >= o) v += up;
        }
        before[k] = v - n[k];
        if (lane == 63) wave_total[k][wave] = v;
      }
    }
    __syncthreads();
    int first[kSchedClasses];
#pragma unroll
    for (int k = 0; k < kSchedClasses; ++k) {
      int at = class_base[k] + before[k];
      for (int w = 0; w < wave; ++w) at += wave_total[k][w];
      first[k] = at;
    }
    if (b < B) {
      const int full = n[0];
      int partial = 0;
#pragma unroll
      for (int k = 1; k < kSchedClasses; ++k) if (n[k]) partial = first[k];
      int32_t* row = schedule + kSchedRows + 4 * b;
      row[0] = first[0]; row[1] = partial; row[2] = len;
      if (B > 1024) row[3] = 0;   // up to 1024 rows the word names the row of this rank (below)
      const int slot = slot_ids ? slot_ids[b] : b;
      for (int c = 0; c < full; ++c) {   // the record the attention kernel reads: row, chunk, length, slot
        int32_t* rec = schedule + pairs_at + 4 * (first[0] + c);
        rec[0] = b; rec[1] = c; rec[2] = len; rec[3] = slot;
      }
      if (len % chunk) {
        int32_t* rec = schedule + pairs_at + 4 * partial;
        rec[0] = b; rec[1] = full; rec[2] = len; rec[3] = slot;
      }
    }
    __syncthreads();
    if (threadIdx.x < kSchedClasses) {
      int add = 0;
      for (int w = 0; w < 16; ++w) add += wave_total[threadIdx.x][w];
      class_base[threadIdx.x] += add;
    }
    __syncthreads();
  }
  // The rows by decreasing length, for the kernel that gives every (row, KV head) a workgroup of its own: the spare
  // word of record r names the row of rank r (ties: the lower row first).  Keys (length, row) are distinct, so a row's
  // rank is the number of larger keys: every thread counts them over the keys in LDS (four per read, the same
  // address for all lanes) and writes its row at its rank.  Batches of up to 1024 rows; larger ones keep the item list.
  if (B <= 1024) {
    __shared__ __attribute__((aligned(16))) unsigned keys[1024];
    const int t = threadIdx.x;
    const unsigned mine = t < B ? ((unsigned)first_length << 10) | (unsigned)(1023 - t) : 0u;
    keys[t] = mine;
    __syncthreads();
    if (t < B) {
      int rank = 0;
      typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
      const u32x4* quad = reinterpret_cast<const u32x4*>(keys);
      for (int i = 0; i < (B + 3) / 4; ++i) {
        const u32x4 k = quad[i];
        rank += (k[0] > mine) + (k[1] > mine) + (k[2] > mine) + (k[3] > mine);
      }
      schedule[kSchedRows + 4 * rank + 3] = t;
    }
  }
}

__global__ void __launch_bounds__(1024)
decode_schedule_kernel(int32_t* schedule, const int32_t* positions, const uint8_t* active, const int32_t* slot_ids, int B) {
  schedule_rows(schedule, positions, active, slot_ids, B);
}

// The head of a decode step in one launch: the rows' inputs (through the slot map of a compact batch when `slots` is
// given: _gather_inputs of lfm25_batching.py:11-22), the positions the step's layers use (a snapshot of the lengths),
// the lengths advanced for the rows that take part (lfm25_cuda.py:185-186, lfm25_batching.py:35-46: nothing else of the
// step reads the lengths, so advancing them first changes nothing), and the attention work list.  Row b is handled by
// thread b % 1024 in every sweep, so a thread only reads back what it wrote itself.
__global__ void __launch_bounds__(1024)
decode_begin_kernel(int32_t* schedule, int32_t* positions_out, int64_t* tokens_out, uint8_t* mask_out, int32_t* lengths,
                    const int64_t* input, const uint8_t* active, const int32_t* slots, int B) {
  for (int b = threadIdx.x; b < B; b += 1024) {
    int pos;
    if (slots) {
      const int slot = slots[b];
      const bool valid = slot >= 0;
      const bool on = valid && active[slot];
      pos = valid ? lengths[slot] : 0;
      tokens_out[b] = valid ? input[slot] : 0;
      mask_out[b] = on;
      if (on) lengths[slot] = pos + 1;
    } else {
      pos = lengths[b];
      if (!active || active[b]) lengths[b] = pos + 1;
    }
    positions_out[b] = pos;
  }
  schedule_rows(schedule, positions_out, slots ? mask_out : active, slots, B);
}

// Merge the chunk partials of one (row, query head); inactive or empty rows give zeros.
template <typename T>
__global__ void __launch_bounds__(64) decode_combine_kernel(DecodeArgs a) {
  const int b = blockIdx.x, qh = blockIdx.y;
  T* out = (T*)a.out + ((int64_t)b * a.QH + qh) * a.D;
  const RowPairs rp = row_pairs(a, b);
  const int len = rp.len;
  if (len <= 0) {
    for (int d = threadIdx.x; d < a.D; d += 64) out[d] = Elem<T>::store(0.f);
    return;
  }
  const int n = (len + rp.chunk - 1) / rp.chunk;
  auto prow = [&](int c) { return partial_row(a, rp, b, qh, c); };
  float mm = -1.0e30f;
  for (int c = 0; c < n; ++c) mm = fmaxf(mm, a.ws_m[prow(c)]);
  float lt = 0.f;
  for (int c = 0; c < n; ++c) lt = fmaf(a.ws_l[prow(c)], exp2f(a.ws_m[prow(c)] - mm), lt);
  const float inv = 1.0f / fmaxf(lt, 1.0e-20f);
  for (int d = threadIdx.x; d < a.D; d += 64) {
    float o = 0.f;
    for (int c = 0; c < n; ++c) o = fmaf(a.ws_acc[prow(c) * a.D + d], exp2f(a.ws_m[prow(c)] - mm), o);
    out[d] = Elem<T>::store(o * inv);
  }
}

// The same merge for a whole row (all query heads), for rows of at most 4096 values; with QUANT followed by the row's
// e4m3 quantisation, for callers whose next step is an FP8 projection: values are rounded to the model dtype first,
// exactly as a separate quantisation of the stored row would.
// Sixteen waves per row, wave w owning query heads w, w+16, ...; a lane owns one dim of a head.  The partials were
// written by other XCDs and come from beyond the local L2, so every dependent round of loads costs a full memory
// latency: a chunk's maximum and sum are loaded by the lane of the chunk's index (the chunks' weights
// exp2(m_c - max) are then one exp2 per lane, read back lane by lane as scalars), and the accumulator loads do not
// depend on them, so a row of up to NC chunks (all outputs of a lane together) or 32 chunks (half of them at a time) has every
// load of its merge in flight at once.
template <typename T, int NC, bool QUANT>
__global__ void __launch_bounds__(1024) decode_combine_row_kernel(DecodeArgs a, uint8_t* q_out, float* q_scales) {
  constexpr int kMaxPerLane = 4, kWavesPerRow = 16, kMidChunks = 32;
  __shared__ float red[kWavesPerRow];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const RowPairs rp = row_pairs(a, b);
  const int len = rp.len;
  const int n = len > 0 ? (len + rp.chunk - 1) / rp.chunk : 0;
  const int per_head = (a.D + 63) / 64;
  auto head_of = [&](int i) { return wave + kWavesPerRow * (i / per_head); };
  auto dim_of = [&](int i) { return lane + 64 * (i % per_head); };
  auto owned = [&](int i) { return head_of(i) < a.QH && dim_of(i) < a.D; };   // dim_of < D can differ per lane only when D % 64 != 0
  auto weight_of = [&](float f, int c) {   // lane c's value, the same for every lane
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, f), c));
  };
  float y[kMaxPerLane] = {0.f, 0.f, 0.f, 0.f};
  // outputs first .. first + COUNT - 1 of a row of at most CHUNKS chunks, with every load issued before the first use
  auto merge_at_once = [&](auto count, auto chunks, int first) {
    constexpr int COUNT = decltype(count)::value, CHUNKS = decltype(chunks)::value;
    float mv[COUNT], lv[COUNT], accv[COUNT][CHUNKS];
#pragma unroll
    for (int u = 0; u < COUNT; ++u) {
      const int i = first + u;
      const int qh = head_of(i) < a.QH ? head_of(i) : a.QH - 1, d = dim_of(i) < a.D ? dim_of(i) : a.D - 1;
      if (head_of(i) < a.QH) {   // the same for the whole wave
        const int64_t mine = partial_row(a, rp, b, qh, lane < n ? lane : 0);
        mv[u] = a.ws_m[mine];
        lv[u] = a.ws_l[mine];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) accv[u][c] = a.ws_acc[partial_row(a, rp, b, qh, c < n ? c : 0) * a.D + d];
      }
    }
#pragma unroll
    for (int u = 0; u < COUNT; ++u) {
      const int i = first + u;
      if (head_of(i) < a.QH) {
        const float mm = wave_max(lane < n ? mv[u] : -1.0e30f);
        const float f = lane < n ? exp2f(mv[u] - mm) : 0.f;
        const float lt = wave_sum(lv[u] * f);
        float o = 0.f;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) o = fmaf(accv[u][c], weight_of(f, c), o);   // chunks past the row's: weight 0
        y[i] = round_to<T>(o * (1.0f / fmaxf(lt, 1.0e-20f)));
      }
    }
  };
  typedef std::integral_constant<int, kMaxPerLane> AllOutputs;
  typedef std::integral_constant<int, kMaxPerLane / 2> HalfOutputs;
  if (n > 0 && n <= NC) {
    merge_at_once(AllOutputs{}, std::integral_constant<int, NC>{}, 0);
  } else if (n > 0 && n <= kMidChunks) {   // more chunks, half the outputs at a time: about the same registers
    merge_at_once(HalfOutputs{}, std::integral_constant<int, kMidChunks>{}, 0);
    merge_at_once(HalfOutputs{}, std::integral_constant<int, kMidChunks>{}, kMaxPerLane / 2);
  } else if (n > 0) {
    // longer rows: the chunks' maxima and sums in groups of 64 (one per lane), the accumulators in blocks of NC
    for (int i = 0; i < kMaxPerLane; ++i) {
      if (head_of(i) >= a.QH) break;
      const int qh = head_of(i), d = dim_of(i) < a.D ? dim_of(i) : a.D - 1;
      float mm = -1.0e30f;
      for (int c0 = 0; c0 < n; c0 += 64)
        if (c0 + lane < n) mm = fmaxf(mm, a.ws_m[partial_row(a, rp, b, qh, c0 + lane)]);
      mm = wave_max(mm);
      float lt = 0.f, o = 0.f;
      for (int c0 = 0; c0 < n; c0 += 64) {
        const bool mine = c0 + lane < n;
        const int64_t row = partial_row(a, rp, b, qh, mine ? c0 + lane : 0);
        const float f = mine ? exp2f(a.ws_m[row] - mm) : 0.f;
        lt = fmaf(a.ws_l[row], f, lt);
        const int group = n - c0 < 64 ? n - c0 : 64;
        for (int cb = 0; cb < group; cb += NC) {
          float accv[NC];
#pragma unroll
          for (int c = 0; c < NC; ++c) accv[c] = a.ws_acc[partial_row(a, rp, b, qh, c0 + cb + c < n ? c0 + cb + c : 0) * a.D + d];
#pragma unroll
          for (int c = 0; c < NC; ++c) o = fmaf(accv[c], cb + c < 64 ? weight_of(f, cb + c) : 0.f, o);
        }
      }
      lt = wave_sum(lt);
      y[i] = round_to<T>(o * (1.0f / fmaxf(lt, 1.0e-20f)));
    }
  }
  if constexpr (!QUANT) {
    T* out = (T*)a.out + (int64_t)b * a.QH * a.D;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i)
      if (owned(i)) out[head_of(i) * a.D + dim_of(i)] = Elem<T>::store(y[i]);
    return;
  }
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i)
    if (owned(i)) amax = fmaxf(amax, fabsf(y[i]));
  amax = block_max<kWavesPerRow>(amax, red);
  const float scale = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
  if (threadIdx.x == 0) q_scales[b] = scale;
  uint8_t* dst = q_out + (int64_t)b * a.QH * a.D;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i)
    if (owned(i)) dst[head_of(i) * a.D + dim_of(i)] = to_e4m3(y[i] / scale);
}

template <typename T>
void launch_combine_fp8(const DecodeArgs& a, int64_t B, uint8_t* out_q, float* out_scales, hipStream_t s) {
  hipLaunchKernelGGL((decode_combine_row_kernel<T, 12, true>), dim3(B), dim3(1024), 0, s, a, out_q, out_scales);
}
// The merge alone: a row per workgroup when the row fits the row kernel's registers, a (row, head) per wave otherwise.
template <typename T>
void launch_combine(const DecodeArgs& a, int64_t B, hipStream_t s) {
  if ((int64_t)((a.QH + 15) / 16) * ((a.D + 63) / 64) <= 4)
    hipLaunchKernelGGL((decode_combine_row_kernel<T, 12, false>), dim3(B), dim3(1024), 0, s, a, nullptr, nullptr);
  else
    hipLaunchKernelGGL(decode_combine_kernel<T>, dim3(B, a.QH), dim3(64), 0, s, a);
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
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2)))
prefill_attn_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                    const int32_t* __restrict__ cu, int QH, int KH, float scale_log2e) {
  typedef typename HalfMfma<T>::vec8 vec8;
  typedef T vec4 __attribute__((ext_vector_type(4)));
  constexpr int KC = D / 8;          // 16-byte chunks per K or V row
  constexpr int NCH = 64 * KC / 256; // chunks of a 64-token tile per thread, for K and for V
  // K and V tiles sit in LDS as they are in memory (row = token), 16-byte chunks XOR-swizzled by the token.  The
  // V^T operand comes out of the row-major tile through ds_read_b64_tr_b16: lane p of 16 points at token p / 4,
  // bytes 8 (p % 4) .. of a 16-dim block, and lane s receives 4 consecutive tokens of dim s.
  __shared__ vec8 ldsK[64 * KC];
  __shared__ vec8 ldsV[64 * KC];

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
  // the next tile's rows travel to registers while the current tile is multiplied (tokens clamped into the sequence)
  vec8 kreg[NCH], vreg[NCH];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int idx = tid + 256 * i, tok = idx / KC, c = idx % KC;
      int gt = t0 + tok;
      gt = gt < len ? gt : len - 1;
      const int64_t src = ((int64_t)(begin + gt) * KH + kh) * D + c * 8;
      kreg[i] = *reinterpret_cast<const vec8*>(k + src);
      vreg[i] = *reinterpret_cast<const vec8*>(v + src);
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < kv_end; t0 += 64) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int idx = tid + 256 * i, tok = idx / KC, c = idx % KC;
      ldsK[tok * KC + (c ^ (tok & (KC - 1)))] = kreg[i];
      ldsV[tok * KC + (c ^ (tok & (KC - 1)))] = vreg[i];
    }
    __syncthreads();
    fetch(t0 + 64 < kv_end ? t0 + 64 : t0);

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
    // Only a tile that reaches this wave's diagonal or the end of the sequence needs the causal mask (the test is
    // the same for the whole wave).  The softmax is the wave's arithmetic cost, several times the MFMAs': scores stay
    // unscaled and the scale goes into the one multiply-add in front of the hardware exp2.
    const bool edge = t0 + 63 > q0 + 16 * wave || t0 + 63 >= len;
    float mx = -3.0e38f;
    if (edge) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int tk = t0 + 16 * j + 4 * grp + i;
          st[j][i] = (tk <= qpos && tk < len) ? st[j][i] : -3.0e38f;
          mx = fmaxf(mx, st[j][i]);
        }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, st[j][i]);
    }
    mx = max_lane_xor32(max_lane_xor16(mx));
    const float mnew = fmaxf(m, fmaxf(mx * scale_log2e, -1.0e30f));   // a fully masked row keeps its old maximum
    const float alpha = __builtin_amdgcn_exp2f(m - mnew);
    float rs = 0.f;
    vec8 pf[2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(fmaf(st[j][i], scale_log2e, -mnew));   // masked: exp2(-inf) = 0
        rs += p;
        pf[j >> 1][(j & 1) * 4 + i] = (T)p;
      }
    rs = add_lane_xor32(add_lane_xor16(rs));
    l = fmaf(l, alpha, rs);
    m = mnew;
    // the running maximum rarely moves after the first tiles: a branch the whole wave takes or skips (the empty asm
    // keeps it a branch; as selects it costs twice the multiplies it saves)
    if (__any(alpha != 1.0f)) {
      asm volatile("" ::: "memory");
#pragma unroll
      for (int dd = 0; dd < D / 16; ++dd)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[dd][i] *= alpha;
    }
#pragma unroll
    for (int dd = 0; dd < D / 16; ++dd) {
#pragma unroll
      for (int kk2 = 0; kk2 < 2; ++kk2) {
        // tokens 32 kk2 + 4 grp + 0..3 and the same + 16 of dim 16 dd + r: the order P holds them in
        vec4 half[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int tok = 32 * kk2 + 16 * h + 4 * grp + (r >> 2), c = 2 * dd + ((r & 3) >> 1);
          const char* piece = reinterpret_cast<const char*>(&ldsV[tok * KC + (c ^ (tok & (KC - 1)))]) + 8 * (r & 1);
          typedef short s16x4_t __attribute__((ext_vector_type(4)));
          const s16x4_t raw = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4_t*)piece);
          half[h] = __builtin_bit_cast(vec4, raw);
        }
        const vec8 vf = {half[0][0], half[0][1], half[0][2], half[0][3], half[1][0], half[1][1], half[1][2], half[1][3]};
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

// (row, KV head) workgroups from which the row-head kernel is used.  Decode step of the 1.2B shape against the item
// list, prompts U[256, 2048] / U[6000, 7000]: 1 row 0.800 / 0.888 ms against 0.837 / 0.869, 8 rows 0.840 / 0.922 against
// 0.863 / 0.929, 16 rows 0.850 / 0.949 against 0.875 / 1.001, 64 rows 0.995 / 1.367 against 1.043 / 1.497.
constexpr int kRowHeadMinGroups = 64;
constexpr int kMinChunk = kMfmaChunk < kChunk ? kMfmaChunk : kChunk;
static int64_t schedule_ints(int64_t B, int64_t capacity) {
  return kSchedRows + 4 * B + 4 * B * ((capacity + kMfmaChunk - 1) / kMfmaChunk);
}

extern "C" int64_t lfm2_decode_attention_workspace(int64_t B, int QH, int D, int64_t capacity) {
  const int64_t nch = (capacity + kMinChunk - 1) / kMinChunk;  // the smaller chunk of the two kernels bounds both
  return B * QH * nch * (D + 2) + schedule_ints(B, capacity);
}

extern "C" int64_t lfm2_decode_schedule_size(int64_t B, int64_t capacity) { return schedule_ints(B, capacity); }

extern "C" int lfm2_decode_schedule(int32_t* schedule, const int32_t* positions, const uint8_t* active,
                                    const int32_t* slot_ids, int64_t B, void* stream) {
  LFM2_REQUIRE(B > 0 && schedule && positions, "decode_schedule: bad arguments");
  hipLaunchKernelGGL(decode_schedule_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, schedule, positions, active,
                     slot_ids, (int)B);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_decode_begin(int32_t* schedule, int32_t* positions_out, int64_t* tokens_out, uint8_t* mask_out,
                                 int32_t* lengths, const int64_t* input, const uint8_t* active, const int32_t* slots,
                                 int64_t B, void* stream) {
  LFM2_REQUIRE(B > 0 && schedule && positions_out && lengths, "decode_begin: bad arguments");
  LFM2_REQUIRE(slots == nullptr || (tokens_out && mask_out && input && active),
               "decode_begin: a slot map needs the input tokens, the slots' activity flags and the two row outputs");
  hipLaunchKernelGGL(decode_begin_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, schedule, positions_out, tokens_out,
                     mask_out, lengths, input, active, slots, (int)B);
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
  // The scheduled kernel: head_dim 64, a GQA group of at most 4, bf16 queries, and an e4m3 or bf16 history whose
  // rows it can address with 32-bit byte offsets within a slot (paged histories are addressed per token).
  const bool mfma = D == 64 && G <= 4 && dtype == LFM2_DTYPE_BF16 &&
                    (block_table || (kv_fp8 ? c0 % 64 == 0 && c1 % 64 == 0 && c2 % 64 == 0 && capacity * c1 < (1ll << 31)
                                            : capacity * c1 * 2 < (1ll << 31)));
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
  a.page = page; a.QH = QH; a.KH = KH; a.D = D; a.G = G; a.nchunks = nch; a.chunk = chunk; a.B = (int)B;
  a.scale_log2e = scale * LFM2_LOG2E;
  hipStream_t s = (hipStream_t)stream;
  if (mfma) {
    if (schedule == nullptr) {  // no shared schedule from the caller: build one in the tail of the workspace
      int32_t* own = reinterpret_cast<int32_t*>(workspace + B * QH * ((capacity + kMinChunk - 1) / kMinChunk) * (D + 2));
      hipLaunchKernelGGL(decode_schedule_kernel, dim3(1), dim3(1024), 0, s, own, positions, active, slot_ids, (int)B);
      schedule = own;
    }
    a.schedule = schedule;
    // From a few dozen (row, KV head) pairs on, each pair gets a workgroup of its own, longest rows first: the output is
    // written by the kernel itself (no partial results, no merge launch); rows quantised for a W8A8 out projection go
    // through the row quantiser.  A handful of rows keeps the item list, which spreads one long history over all the
    // waves; so do batches beyond the 1024 rows the work-list launch sorts.
    if ((int64_t)B * KH >= kRowHeadMinGroups && B <= 1024) {
      float* scratch = workspace;   // bf16 rows [B, QH * D] when the caller only wants the quantised rows
      a.out = out ? out : (void*)scratch;
      const dim3 rgrid((unsigned)(8 * KH * ((B + 7) / 8)));
      if (kv_fp8) {
        if (block_table) hipLaunchKernelGGL((decode_attn_mfma_kernel<true, true, true>), rgrid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((decode_attn_mfma_kernel<false, true, true>), rgrid, dim3(256), 0, s, a);
      } else {
        if (block_table) hipLaunchKernelGGL((decode_attn_mfma_kernel<true, false, true>), rgrid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL((decode_attn_mfma_kernel<false, false, true>), rgrid, dim3(256), 0, s, a);
      }
      if (out_q) return lfm2_quantize_rows(out_q, out_scales, a.out, B, (int64_t)QH * D, dtype, stream);
      LFM2_LAUNCH_CHECK();
    }
    // 3 workgroups per CU (the register budget of 128 would allow 4, but with a handful of items per wave more
    // waves only make the shares of work more unequal); never more than the worst case
    int64_t blocks = ((int64_t)B * nch * KH + 3) / 4;
    blocks = blocks < 768 ? blocks : 768;
    const dim3 mgrid((unsigned)blocks);
    if (kv_fp8) {
      if (block_table) hipLaunchKernelGGL((decode_attn_mfma_kernel<true, true>), mgrid, dim3(256), 0, s, a);
      else hipLaunchKernelGGL((decode_attn_mfma_kernel<false, true>), mgrid, dim3(256), 0, s, a);
    } else {
      if (block_table) hipLaunchKernelGGL((decode_attn_mfma_kernel<true, false>), mgrid, dim3(256), 0, s, a);
      else hipLaunchKernelGGL((decode_attn_mfma_kernel<false, false>), mgrid, dim3(256), 0, s, a);
    }
    if (out_q) launch_combine_fp8<__bf16>(a, B, out_q, out_scales, s);
    else launch_combine<__bf16>(a, B, s);
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
    else launch_combine<T>(a, B, s));
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
