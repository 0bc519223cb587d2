// "NT" GEMMs of the LFM2 linear layers on MFMA: out[M,N] = A[M,K] . W[N,K]^T.
//
//   fp8  : A, W are OCP e4m3 bytes, v_mfma_f32_16x16x128_f8f6f4 (unit block scales), epilogue * a_scale[m] * w_scale[n]
//   bf16 : v_mfma_f32_16x16x32_bf16, plain epilogue
//
// Both operands are K-contiguous, so the kernel works on 16-byte chunks of K for either type:
// a workgroup stages a BM x 128 B tile of A and a BN x 128 B tile of W per step through LDS
// (double buffered, one barrier per step, the next two tiles in flight in registers during the MFMAs).
// Chunks are XOR-swizzled by row so the 16-lane column reads of the MFMA operand layout spread
// over all banks.  A lane of lane-group g = lane/16 takes the same chunks of its row for both
// operands (2g, 2g+1 for e4m3; g, g+4 for bf16), so the contraction order inside a 128 B step is
// permuted identically on both sides and needs no shuffles.  W is the MFMA "A" operand, so a lane ends with four consecutive output
// columns of one row and stores 8 bytes at a time.
//
// Workgroup ids are remapped so that the M-tiles sharing one W tile run back to back on the same
// XCD (ids are dealt round-robin over the 8 XCDs, each with its own L2): W streams from HBM once.
#include "lfm2_common.h"
#ifndef LFM2_W_AUX
#define LFM2_W_AUX 0
#endif

namespace {

constexpr int kStepBytes = 128;          // K bytes one MFMA pass group consumes per row (and the default staging step)

// Slot of a row's 16-byte chunk in a staged tile.  The XOR pattern is chosen per operand type from a sweep of
// ds_read_b128 patterns on gfx950 (LDS reads peak at 256 B/clk): the e4m3 fragment read (16 rows x chunks 2g, 2g+1)
// runs at 240 B/clk with row&7 ^ bit 3 of the row and at 128 B/clk with row&7 alone; the bf16 fragment read
// (chunk g + 4*pass) is the other way round.  Staging writes (8 lanes per row) are indifferent (78 B/clk either way).
// CPR = chunks per staged row (8 for 128-byte K steps, 16 for 256-byte steps, where rows are a full bank sweep apart
// and the XOR must cover four chunk bits: row&15 reads at 241 B/clk, row&7 at 128).
template <int SW, int CPR> __device__ __forceinline__ int lds_slot(int row, int chunk) {
  const int x = CPR == 16 ? (row & 15) : SW == 1 ? ((row & 7) ^ ((row >> 3) & 1)) : (row & 7);
  return row * CPR + (chunk ^ x);
}

typedef int i32x8 __attribute__((ext_vector_type(8)));

// One K step (128 bytes per row) of a 16x16 output tile.  `lds_w`/`lds_a` point at the staged tiles, `wrow`/`arow`
// are the lane's rows.  Both operands take the same chunks per lane group, so the K order inside the step is
// permuted identically on both sides.
template <int EB> struct StepMfma;
template <> struct StepMfma<1> {
  // e4m3: lane group g owns chunks 2g, 2g+1 (32 bytes) -> one v_mfma_f32_16x16x128_f8f6f4 (unit scales)
  typedef i32x8 frag;
  static constexpr int PASSES = 1;
  template <int SW, int CPR> static __device__ __forceinline__ frag load(const i32x4* tile, int row, int lgrp, int, int sub) {
    const i32x4 lo = tile[lds_slot<SW, CPR>(row, 8 * sub + 2 * lgrp)], hi = tile[lds_slot<SW, CPR>(row, 8 * sub + 2 * lgrp + 1)];
    return frag{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  }
  static __device__ __forceinline__ f32x4 run(const frag& w, const frag& a, f32x4 acc) {
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, a, acc, 0, 0, 0, 0, 0, 0);
  }
};
template <> struct StepMfma<2> {
  // bf16: two passes; in pass h lane group g owns chunk g + 4h (8 values) -> v_mfma_f32_16x16x32_bf16
  typedef i32x4 frag;
  static constexpr int PASSES = 2;
  template <int SW, int CPR> static __device__ __forceinline__ frag load(const i32x4* tile, int row, int lgrp, int pass, int sub) {
    return tile[lds_slot<SW, CPR>(row, 8 * sub + lgrp + 4 * pass)];
  }
  static __device__ __forceinline__ f32x4 run(const frag& w, const frag& a, f32x4 acc) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, a), acc, 0, 0, 0);
  }
};

// Optional placement of output rows: row m goes to out row slots[m] (m when slots is null); rows whose slot is
// negative, not below `capacity` (the rows `out` holds), or whose `active` byte is 0 are not written.  This is the
// scatter of lfm25_batching.py:25-32 done by the producing GEMM instead of by a copy of the logits.
struct RowMap { const int32_t* slots; const uint8_t* active; int capacity; };
__device__ __forceinline__ int mapped_row(const RowMap& rows, int m) {
  if (rows.active && !rows.active[m]) return -1;
  const int slot = rows.slots ? rows.slots[m] : m;
  return slot < rows.capacity ? slot : -1;
}

__device__ __forceinline__ void store_out(void* out, int out_dtype, int64_t idx, float v) {
  if (out_dtype == LFM2_DTYPE_BF16) ((__bf16*)out)[idx] = (__bf16)v;
  else if (out_dtype == LFM2_DTYPE_F16) ((_Float16*)out)[idx] = (_Float16)v;
  else ((float*)out)[idx] = v;
}

// Epilogue of the fused QKV projection (EPI = 1; 64 x 64 tiles, head_dim 64, so a column tile is one head of 64 rows):
// what prepare_qkv with cache append does to the projection's bf16 output (lfm25_cuda_kernels.py:113-151 then the
// append of lfm25_fp8_kv.py:58-69 or lfm25_batching.py:49-69), with the same rounding points and the same
// summation tree for the head's mean square, so the results are bit for bit those of the two launches.
struct QkvEpilogue {
  void* q;                 // [M, QH, 64] model dtype
  const void *qw, *kw;     // q/k norm weights [64]
  const float *cosT, *sinT;
  const int32_t *positions, *slot_ids;
  const uint8_t* active;
  void *kc, *vc;           // caches addressed slot*c0 + pos*c1 + head*c2 + d
  float *ks, *vs;          // e4m3 cache scales (same offsets / 64) or NULL for a model-dtype cache
  int64_t max_positions, c0, c1, c2;
  int QH, KH;
  float eps;
};

// The fused gate+up projection (EPI = 2) walks the packed weight [gate rows; up rows] in an interleaved order: output
// column n of the product is gate row 8*(n/16) + n%8 when n%16 < 8 and the up row of the same index otherwise, so that
// every 16-column MFMA tile holds eight gate columns and the eight up columns that pair with them.  Only the addresses
// of the weight rows and of their scales change; the weight keeps the layout the unfused path reads.
__device__ __forceinline__ int swiglu_weight_row(int n, int N) {
  return ((n >> 4) << 3) + (n & 7) + ((n & 8) ? (N >> 1) : 0);
}

// The conv in-projection with the gated short-conv update as its epilogue (EPI = 3): the packed weight [B rows; C rows;
// x rows] (N = 3 H) is walked so that output columns 48g .. 48g+47 are the B, C and x rows of channels 16g .. 16g+15,
// 16 columns each: the three MFMA tiles of a wave (tile columns 96, two waves across) then hold B, C and x of the same
// channels in the same lanes.
__device__ __forceinline__ int conv_weight_row(int n, int N) {
  const int group = n / 48, within = n % 48;
  return (within >> 4) * (N / 3) + 16 * group + (within & 15);
}
struct ConvEpilogue {
  const void* weight;        // [H, 3] model dtype
  void* state;               // [slots, H, 3] model dtype, updated in place for rows that take part
  const uint8_t* active;     // per row, or NULL
  const int32_t* slot_ids;   // row -> state slot (negative: padding), or NULL for row = slot
};

// The kernel body; the two entry points below differ in their arguments only (the fused QKV projection carries its
// epilogue's arguments, the plain products do not pay for them in every launch's argument block).
template <int EB, int BM, int BN, int WM, int WN, int SW, int KS, bool KTAIL, int ST, int EPI>
__device__ __forceinline__ void
gemm_nt_body(void* __restrict__ out, float* __restrict__ partial, const uint8_t* __restrict__ A,
             const uint8_t* __restrict__ W, const float* __restrict__ a_scales, const float* __restrict__ w_scales,
             int M, int N, int64_t Kb, int steps_per_split, int out_dtype, const RowMap& rows, const QkvEpilogue& epi,
             const ConvEpilogue& conv = ConvEpilogue{}) {
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM, TN = BN / WN, MI = TM / 16, NI = TN / 16;
  constexpr int kChunksPerRow = KS / 16;  // KS = K bytes staged per step and row: 128, or 256 (two MFMA sub-steps per barrier)
  constexpr int A_CHUNKS = BM * kChunksPerRow, W_CHUNKS = BN * kChunksPerRow;
  constexpr int A_PER = (A_CHUNKS + NT - 1) / NT, W_PER = (W_CHUNKS + NT - 1) / NT;
  // ST = 0: tiles staged through registers into two LDS buffers; ST >= 2: a ring of ST LDS buffers filled by
  // direct global->LDS loads (no staging registers, no ds_write and no wait between load and LDS store)
  __shared__ i32x4 lds[ST > 0 ? ST : 2][A_CHUNKS + W_CHUNKS];

  // XCD-aware tile order: consecutive logical ids (same XCD, adjacent in time) share an N tile.
  const int mt = (M + BM - 1) / BM, nt = (N + BN - 1) / BN, tiles = mt * nt;
  const int per_xcd = gridDim.x / 8;
  const int lid = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (lid >= tiles) return;
  // Within an XCD the ids walk groups of kGroupM M-tiles across all N-tiles: the 64 or so tiles an XCD has in flight are
  // then about 8 x 8, whose operands (2 + 2 MB at K = 2048) stay in its 4 MB L2, instead of every M-tile of two
  // N-tiles (all of A: 8 MB at 4096 rows, re-streamed from beyond L2 for every N-tile).
  constexpr int kGroupM = 8;
  const int group = lid / (kGroupM * nt), in_group = lid % (kGroupM * nt);
  const int first_m = group * kGroupM, rows_m = mt - first_m < kGroupM ? mt - first_m : kGroupM;
  const int m_base = (first_m + in_group % rows_m) * BM, n_base = (in_group / rows_m) * BN;

  const int64_t total_steps = (Kb + KS - 1) / KS;
  const int64_t step0 = (int64_t)blockIdx.y * steps_per_split;
  int64_t nsteps = total_steps - step0;
  if (nsteps > steps_per_split) nsteps = steps_per_split;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;
  const int lrow = lane & 15, lgrp = lane >> 4;

  // Two register sets give a prefetch distance of two K steps with only two LDS buffers: while step s is
  // multiplied out of LDS buffer s&1, set (s+1)&1 holds step s+1 in flight and set s&1 is refilled with step s+2.
  i32x4 ra[2][A_PER], rw[2][W_PER];
  // Loads are unconditional (addresses clamped into the operand, out-of-range chunks zeroed by a select): with
  // no branch between issue and use the compiler keeps them in flight across the MFMAs of two K steps.
  auto fetch = [&](int64_t step, int set) {
    step = step < nsteps ? step : nsteps - 1;
    const int64_t kb = (step0 + step) * KS;
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      int idx = tid + i * NT;
      if (A_CHUNKS % NT != 0) idx = idx < A_CHUNKS ? idx : A_CHUNKS - 1;
      const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
      int gr = m_base + row;
      gr = gr < M ? gr : M - 1;
      const int64_t ko = kb + c * 16;
      if (KTAIL) {  // K bytes not a multiple of the step: chunks past the end read a valid address and become zero
        const bool ok = ko < Kb;
        const i32x4 v = *reinterpret_cast<const i32x4*>(A + (int64_t)gr * Kb + (ok ? ko : Kb - 16));
        const i32x4 zero = {0, 0, 0, 0};
        ra[set][i] = ok ? v : zero;
      } else {
        ra[set][i] = *reinterpret_cast<const i32x4*>(A + (int64_t)gr * Kb + ko);
      }
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      int idx = tid + i * NT;
      if (W_CHUNKS % NT != 0) idx = idx < W_CHUNKS ? idx : W_CHUNKS - 1;
      const int row = idx / kChunksPerRow, c = idx % kChunksPerRow;
      int gr = n_base + row;
      gr = gr < N ? gr : N - 1;
      const int64_t ko = kb + c * 16;
      if (KTAIL) {
        const bool ok = ko < Kb;
        const i32x4 v = *reinterpret_cast<const i32x4*>(W + (int64_t)gr * Kb + (ok ? ko : Kb - 16));
        const i32x4 zero = {0, 0, 0, 0};
        rw[set][i] = ok ? v : zero;
      } else {
        rw[set][i] = *reinterpret_cast<const i32x4*>(W + (int64_t)gr * Kb + ko);
      }
    }
  };
  auto stash = [&](int set, int buf) {
#pragma unroll
    for (int i = 0; i < A_PER; ++i) {
      const int idx = tid + i * NT;
      if (A_CHUNKS % NT == 0 || idx < A_CHUNKS) lds[buf][lds_slot<SW, kChunksPerRow>(idx / kChunksPerRow, idx % kChunksPerRow)] = ra[set][i];
    }
#pragma unroll
    for (int i = 0; i < W_PER; ++i) {
      const int idx = tid + i * NT;
      if (W_CHUNKS % NT == 0 || idx < W_CHUNKS)
        lds[buf][A_CHUNKS + lds_slot<SW, kChunksPerRow>(idx / kChunksPerRow, idx % kChunksPerRow)] = rw[set][i];
    }
  };

  f32x4 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto multiply = [&](int buf) {
    typedef typename StepMfma<EB>::frag frag;
#pragma unroll
    for (int sub = 0; sub < KS / kStepBytes; ++sub) {
#pragma unroll
      for (int pass = 0; pass < StepMfma<EB>::PASSES; ++pass) {
        frag fa[MI], fw[NI];
#pragma unroll
        for (int i = 0; i < MI; ++i)
          fa[i] = StepMfma<EB>::template load<SW, kChunksPerRow>(&lds[buf][0], wm * TM + i * 16 + lrow, lgrp, pass, sub);
#pragma unroll
        for (int j = 0; j < NI; ++j)
          fw[j] = StepMfma<EB>::template load<SW, kChunksPerRow>(&lds[buf][A_CHUNKS], wn * TN + j * 16 + lrow, lgrp, pass, sub);
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) acc[i][j] = StepMfma<EB>::run(fw[j], fa[i], acc[i][j]);
      }
    }
  };

  // Small wave tiles (the decode batch's tiles) fetch the scales their epilogue needs here, before the K loop: asked for
  // at the end they are a memory round trip (the weight's scales come from HBM) in which the workgroup does nothing.
  // Large wave tiles have no registers to spare for them across the loop and find theirs in L2 anyway.
  constexpr bool kEarlyScales = (EPI == 0 || EPI == 2) && MI * NI <= 6;
  constexpr int kColScales = EPI == 2 ? 8 * ((NI + 1) / 2) : 4 * NI;
  float early_cols[kEarlyScales ? kColScales : 1], early_rows[kEarlyScales ? MI : 1];
  if constexpr (kEarlyScales) {
    if (a_scales && partial == nullptr) {
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int m = m_base + wm * TM + i * 16 + lrow;
        early_rows[i] = a_scales[m < M ? m : M - 1];
      }
      if constexpr (EPI == 2) {
#pragma unroll
        for (int j = 0; j < NI; j += 2) {
          const int j1 = j + 1 < NI ? j + 1 : j;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int n0 = n_base + wn * TN + j * 16 + 4 * lgrp + r, n1 = n_base + wn * TN + j1 * 16 + 4 * lgrp + r;
            early_cols[8 * (j / 2) + r] = w_scales[swiglu_weight_row(n0 < N ? n0 : N - 1, N)];
            early_cols[8 * (j / 2) + 4 + r] = w_scales[swiglu_weight_row(n1 < N ? n1 : N - 1, N)];
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          const int n = n_base + wn * TN + j * 16 + 4 * lgrp;
#pragma unroll
          for (int r = 0; r < 4; ++r) early_cols[4 * j + r] = n + r < N ? w_scales[n + r] : 0.f;
        }
      }
    }
  }
  static_assert((EPI != 2 && EPI != 3) || ST > 0, "the fused SwiGLU and conv epilogues are built on the ring tiles");
  if constexpr (ST > 0) {
    static_assert(!KTAIL, "direct-to-LDS loads cannot zero-fill a partial K step");
    static_assert(A_CHUNKS % 64 == 0 && W_CHUNKS % 64 == 0, "a wave fills 64 consecutive slots per instruction");
    // Slot s of a staged tile holds (row s / CPR, chunk (s % CPR) ^ swizzle(row)); the instruction writes lane l's
    // 16 bytes to slot base + l, so each lane fetches the global chunk that belongs to its slot.
    auto issue = [&](int64_t step, int buf) {
      step = step < nsteps ? step : nsteps - 1;
      const int64_t kb = (step0 + step) * KS;
#pragma unroll
      for (int i = 0; i < A_PER; ++i) {
        const int slot = i * NT + tid;
        if (A_CHUNKS % NT == 0 || slot < A_CHUNKS) {
          const int row = slot / kChunksPerRow;
          const int c = lds_slot<SW, kChunksPerRow>(row, slot % kChunksPerRow) - row * kChunksPerRow;
          int gr = m_base + row;
          gr = gr < M ? gr : M - 1;
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(A + (int64_t)gr * Kb + kb + c * 16),
                                           (__attribute__((address_space(3))) void*)(&lds[buf][i * NT + wave * 64]), 16, 0, 0);
        }
      }
#pragma unroll
      for (int i = 0; i < W_PER; ++i) {
        const int slot = i * NT + tid;
        if (W_CHUNKS % NT == 0 || slot < W_CHUNKS) {
          const int row = slot / kChunksPerRow;
          const int c = lds_slot<SW, kChunksPerRow>(row, slot % kChunksPerRow) - row * kChunksPerRow;
          int gr = n_base + row;
          gr = gr < N ? gr : N - 1;
          if (EPI == 2) gr = swiglu_weight_row(gr, N);
          if (EPI == 3) gr = conv_weight_row(gr, N);
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(W + (int64_t)gr * Kb + kb + c * 16),
                                           (__attribute__((address_space(3))) void*)(&lds[buf][A_CHUNKS + i * NT + wave * 64]), 16, 0, LFM2_W_AUX);
        }
      }
    };
    // loads complete in order: with ST-1 steps in flight, step s has landed once at most ST-2 steps' loads remain.
    // Each wave counts its own loads, and when a tile has fewer chunks than threads the last waves issue fewer per
    // step (only the full passes).  The wait must use the wave's own count: waiting for the smallest count makes a
    // wave that issues more wait for loads of the NEXT step as well, which halves its prefetch distance (the 128x96
    // tile of 16 waves: 12.2 -> 10.6 us for its loads alone).  The immediate is a constant, so the (at most three)
    // possible counts are spelled out; the choice is wave-uniform.
    constexpr int kPerStep = A_CHUNKS / NT + W_CHUNKS / NT;   // loads of a wave that only takes part in full passes
    const int extra = ((A_CHUNKS % NT != 0 && (A_PER - 1) * NT + wave * 64 < A_CHUNKS) ? 1 : 0) +
                      ((W_CHUNKS % NT != 0 && (W_PER - 1) * NT + wave * 64 < W_CHUNKS) ? 1 : 0);
    auto wait_for_step = [&]() {
#define LFM2_VMCNT_(N) ((((N) & 0xF)) | (0x7 << 4) | (0xF << 8) | ((((N) >> 4) & 0x3) << 14))
      static_assert((ST - 2) * (kPerStep + 2) < 64, "vmcnt has six bits");
      if (extra == 0) __builtin_amdgcn_s_waitcnt(LFM2_VMCNT_((ST - 2) * kPerStep));
      else if (extra == 1) __builtin_amdgcn_s_waitcnt(LFM2_VMCNT_((ST - 2) * (kPerStep + 1)));
      else __builtin_amdgcn_s_waitcnt(LFM2_VMCNT_((ST - 2) * (kPerStep + 2)));
#undef LFM2_VMCNT_
    };
#pragma unroll
    for (int st = 0; st < ST - 1; ++st) issue(st, st);
    int buf = 0, fill = ST - 1;
    for (int64_t s = 0; s < nsteps; ++s) {
      wait_for_step();
      __builtin_amdgcn_s_barrier();  // (a bare barrier: __syncthreads would add a fence that drains the loads in flight)
      // step s is in LDS for every wave, and every wave is done reading the buffer refilled next
      issue(s + ST - 1, fill);
      multiply(buf);
      buf = buf + 1 == ST ? 0 : buf + 1;
      fill = fill + 1 == ST ? 0 : fill + 1;
    }
  } else {
  if (nsteps > 0) {
    fetch(0, 0);
    fetch(1, 1);
    stash(0, 0);
  }
  __syncthreads();
  // Steps beyond the last one are clamped re-reads whose data is never multiplied.
  // sched_barrier keeps the scheduler from sinking the prefetch loads down to their use after the MFMAs.
  for (int64_t s = 0; s < nsteps; s += 2) {
    fetch(s + 2, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(0);
    __builtin_amdgcn_sched_barrier(0);
    stash(1, 1);
    __syncthreads();
    if (s + 1 < nsteps) {
      fetch(s + 3, 1);
      __builtin_amdgcn_sched_barrier(0);
      multiply(1);
      __builtin_amdgcn_sched_barrier(0);
      stash(0, 0);
      __syncthreads();
    }
  }
  }

  if constexpr (EPI == 1) {
    static_assert(BM == 64 && BN == 64 && NT == 256 && EB == 1, "the QKV epilogue works on 64 x 64 tiles of 256 threads");
    typedef __bf16 T;
    constexpr int LD = 68;   // padded row of the fp32 tile
    // every load into LDS has landed and every wave is done with the staged operands: the ring becomes the tile
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    float* tile = reinterpret_cast<float*>(&lds[0][0]);
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const int ml = wm * TM + i * 16 + lrow;
      const int mg = m_base + ml < M ? m_base + ml : M - 1;
      const float sa = a_scales[mg];
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        const int nl = wn * TN + j * 16 + 4 * lgrp;
#pragma unroll
        for (int r = 0; r < 4; ++r) tile[ml * LD + nl + r] = round_to<T>((acc[i][j][r] * sa) * w_scales[n_base + nl + r]);
      }
    }
    __syncthreads();
    // four adjacent lanes own a row of the head: 16 consecutive dims each
    const int row = tid >> 2, part = tid & 3;
    const bool live = m_base + row < M;
    const int64_t m = live ? m_base + row : M - 1;
    const int u = n_base / 64;   // head unit: query heads, then key heads, then value heads
    float val[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) val[e] = tile[row * LD + 16 * part + e];
    if (u < epi.QH + epi.KH) {
      typedef T vec8 __attribute__((ext_vector_type(8)));
      const T* wgt = (u < epi.QH ? (const T*)epi.qw : (const T*)epi.kw) + 16 * part;
      const vec8 g0 = *reinterpret_cast<const vec8*>(wgt), g1 = *reinterpret_cast<const vec8*>(wgt + 8);
      int64_t pos = epi.positions[m];
      pos = pos < 0 ? 0 : (pos >= epi.max_positions ? epi.max_positions - 1 : pos);
      const f32x4* cs = reinterpret_cast<const f32x4*>(epi.cosT + pos * 32 + 16 * (part & 1));
      const f32x4* sn = reinterpret_cast<const f32x4*>(epi.sinT + pos * 32 + 16 * (part & 1));
      float c[16], sv[16];
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const f32x4 cv = cs[v4], xv = sn[v4];
#pragma unroll
        for (int e = 0; e < 4; ++e) { c[4 * v4 + e] = round_to<T>(cv[e]); sv[4 * v4 + e] = round_to<T>(xv[e]); }
      }
      // mean square by the pairwise tree of a wave's butterfly reduction over one dim per lane
      float sq[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) sq[e] = val[e] * val[e];
#pragma unroll
      for (int width = 1; width < 16; width *= 2)
#pragma unroll
        for (int e = 0; e < 16; e += 2 * width) sq[e] = sq[e] + sq[e + width];
      float ss = sq[0];
      ss = ss + __shfl_xor(ss, 1, 64);
      ss = ss + __shfl_xor(ss, 2, 64);
      const float rstd = 1.0f / sqrtf(ss / 64.0f + epi.eps);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float nrm = round_to<T>(val[e] * rstd);
        val[e] = round_to<T>(nrm * Elem<T>::load(e < 8 ? g0[e & 7] : g1[e & 7]));
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float partner = __shfl_xor(val[e], 2, 64);   // the dim 32 away
        const float left = round_to<T>(val[e] * c[e]), right = round_to<T>(partner * sv[e]);
        sq[e] = round_to<T>(part < 2 ? left - right : left + right);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) val[e] = sq[e];
    }
    typedef T vec8 __attribute__((ext_vector_type(8)));
    auto store_model = [&](T* dst) {
      vec8 lo, hi;
#pragma unroll
      for (int e = 0; e < 8; ++e) { lo[e] = Elem<T>::store(val[e]); hi[e] = Elem<T>::store(val[8 + e]); }
      *reinterpret_cast<vec8*>(dst) = lo;
      *reinterpret_cast<vec8*>(dst + 8) = hi;
    };
    if (u < epi.QH) {
      if (live) store_model((T*)epi.q + (m * epi.QH + u) * 64 + 16 * part);
      return;
    }
    const bool is_v = u >= epi.QH + epi.KH;
    const int h = is_v ? u - epi.QH - epi.KH : u - epi.QH;
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(val[e]));
    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
    const int64_t slot = epi.slot_ids ? epi.slot_ids[m] : m;
    const int64_t at = epi.positions[m];
    if (!live || (epi.active && !epi.active[m]) || slot < 0 || at < 0) return;
    const int64_t dst = slot * epi.c0 + at * epi.c1 + (int64_t)h * epi.c2;
    if (epi.ks == nullptr) {
      store_model((T*)(is_v ? epi.vc : epi.kc) + dst + 16 * part);
    } else {
      const float sc = fmaxf(amax / LFM2_E4M3_MAX, 1.0e-12f);
      i32x4 packed;
#pragma unroll
      for (int wd = 0; wd < 4; ++wd) {
        uint32_t bits = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) bits |= (uint32_t)to_e4m3(val[4 * wd + e] / sc) << (8 * e);
        packed[wd] = (int)bits;
      }
      *reinterpret_cast<i32x4*>((uint8_t*)(is_v ? epi.vc : epi.kc) + dst + 16 * part) = packed;
      if (part == 0) (is_v ? epi.vs : epi.ks)[dst / 64] = sc;
    }
    return;
  }

  if constexpr (EPI == 2) {
    // SwiGLU of lfm25_cuda_kernels.py:58-72 on the product's own tile: gate and up values are rounded to the model dtype
    // as the plain product stores them, then act = round(silu(gate)), out = round(act * up).  In a 16-column tile lane
    // groups 0, 1 hold gate columns 0-7 and groups 2, 3 the up columns that pair with them; one half-wave swap per value
    // of two neighbouring tiles leaves lanes 0-31 with gate and up of the first tile and lanes 32-63 with those of the
    // second, so every lane finishes four outputs.  out is [M, N / 2].
    auto finish_rows = [&](auto tag) {
      typedef decltype(tag) T;
      const int half = lane >> 5, I = N >> 1;
      // the column scales of this lane's values do not depend on the row: fetched once, before the rows
      float cs0[(NI + 1) / 2][4], cs1[(NI + 1) / 2][4];
      if (a_scales) {
#pragma unroll
        for (int j = 0; j < NI; j += 2) {
          const int j1 = j + 1 < NI ? j + 1 : j;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if constexpr (kEarlyScales) {
              cs0[j / 2][r] = early_cols[8 * (j / 2) + r];
              cs1[j / 2][r] = early_cols[8 * (j / 2) + 4 + r];
            } else {
              const int n0 = n_base + wn * TN + j * 16 + 4 * lgrp + r, n1 = n_base + wn * TN + j1 * 16 + 4 * lgrp + r;
              cs0[j / 2][r] = w_scales[swiglu_weight_row(n0 < N ? n0 : N - 1, N)];
              cs1[j / 2][r] = w_scales[swiglu_weight_row(n1 < N ? n1 : N - 1, N)];
            }
          }
        }
      }
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int m = m_base + wm * TM + i * 16 + lrow;
        float sa = 1.0f;
        if (a_scales) {
          if constexpr (kEarlyScales) sa = early_rows[i];
          else sa = a_scales[m < M ? m : M - 1];
        }
#pragma unroll
        for (int j = 0; j < NI; j += 2) {
          const int j1 = j + 1 < NI ? j + 1 : j;
          float first[4], second[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float y0 = acc[i][j][r], y1 = acc[i][j1][r];
            if (a_scales) {
              y0 = (y0 * sa) * cs0[j / 2][r];
              y1 = (y1 * sa) * cs1[j / 2][r];
            }
            const unsigned a = __builtin_bit_cast(unsigned, round_to<T>(y0)), b = __builtin_bit_cast(unsigned, round_to<T>(y1));
            const auto swapped = __builtin_amdgcn_permlane32_swap(a, b, false, false);
            first[r] = __builtin_bit_cast(float, (unsigned)swapped[0]);    // gate: tile j in lanes 0-31, tile j1 in lanes 32-63
            second[r] = __builtin_bit_cast(float, (unsigned)swapped[1]);   // up, same split
          }
          const int jj = half ? j1 : j;
          if (half && j1 == j) continue;          // an odd last tile is finished by the lower half alone
          const int tile_n = n_base + wn * TN + jj * 16;
          if (m >= M || tile_n >= N) continue;
          const int64_t at = (int64_t)m * I + (tile_n >> 1) + 4 * (lgrp & 1);
          float h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) h[r] = round_to<T>(round_to<T>(silu_f(first[r])) * second[r]);
          T* dst = (T*)out + at;
          if constexpr (sizeof(T) == 2) {
            typedef T vec4 __attribute__((ext_vector_type(4)));
            vec4 o = {Elem<T>::store(h[0]), Elem<T>::store(h[1]), Elem<T>::store(h[2]), Elem<T>::store(h[3])};
            *reinterpret_cast<vec4*>(dst) = o;
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) dst[r] = Elem<T>::store(h[r]);
          }
        }
      }
    };
    if (out_dtype == LFM2_DTYPE_BF16) finish_rows(__bf16{});
    else if (out_dtype == LFM2_DTYPE_F16) finish_rows(_Float16{});
    else finish_rows(float{});
    return;
  }

  if constexpr (EPI == 3) {
    // conv_update of lfm25_cuda_kernels.py:75-110 on the product's own tile: B, C and x are rounded to the model dtype as
    // the plain product stores them; a lane owns four channels of one row: their taps (12 values, contiguous in the
    // state), their weights, their outputs.  out is [M, N / 3].
    static_assert(NI == 3, "a wave's three MFMA tiles are B, C and x of the same channels");
    auto finish_rows = [&](auto tag) {
      typedef decltype(tag) T;
      const int H = N / 3;
      const int channel = ((n_base + wn * TN) / 48) * 16 + 4 * lgrp;
      if (n_base + wn * TN >= N) return;
      float wt[12];
      {
        const T* w = (const T*)conv.weight + (int64_t)channel * 3;
#pragma unroll
        for (int e = 0; e < 12; ++e) wt[e] = Elem<T>::load(w[e]);
      }
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        const int m = m_base + wm * TM + i * 16 + lrow;
        if (m >= M) continue;
        const float sa = a_scales ? a_scales[m] : 1.0f;
        float v[3][4];
#pragma unroll
        for (int t = 0; t < 3; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float y = acc[i][t][r];
            if (a_scales) y = (y * sa) * w_scales[t * H + channel + r];
            v[t][r] = round_to<T>(y);
          }
        int64_t slot = m;
        if (conv.slot_ids) { const int32_t sid = conv.slot_ids[m]; slot = sid < 0 ? 0 : sid; }
        const bool on = conv.active ? conv.active[m] != 0 : true;
        T* st = (T*)conv.state + (slot * H + channel) * 3;
        float taps[12], fresh[12], y[4];
#pragma unroll
        for (int e = 0; e < 12; ++e) taps[e] = Elem<T>::load(st[e]);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float bx;
          y[r] = conv_channel<T>(v[0][r], v[1][r], v[2][r], taps[3 * r + 1], taps[3 * r + 2], wt[3 * r], wt[3 * r + 1],
                                 wt[3 * r + 2], &bx);
          fresh[3 * r] = taps[3 * r + 1]; fresh[3 * r + 1] = taps[3 * r + 2]; fresh[3 * r + 2] = bx;
        }
        if (on) {
#pragma unroll
          for (int e = 0; e < 12; ++e) st[e] = Elem<T>::store(fresh[e]);
        }
        T* dst = (T*)out + (int64_t)m * H + channel;
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[r] = Elem<T>::store(y[r]);
      }
    };
    if (out_dtype == LFM2_DTYPE_BF16) finish_rows(__bf16{});
    else if (out_dtype == LFM2_DTYPE_F16) finish_rows(_Float16{});
    else finish_rows(float{});
    return;
  }

  // Epilogue: lane holds out[m = .. + lrow][n = .. + 4*lgrp + r], r = 0..3.
  const bool split = partial != nullptr;
  // the column scales of this lane's values do not depend on the row: fetched once, before the rows
  float cw[NI][4];
  if (a_scales && !split) {
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int n = n_base + wn * TN + j * 16 + 4 * lgrp;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if constexpr (kEarlyScales) cw[j][r] = early_cols[4 * j + r];
        else cw[j][r] = n + r < N ? w_scales[n + r] : 0.f;
      }
    }
  }
  auto finish = [&](f32x4 v, int m_out, int n, float sa, const float* cols) {  // scale (row then column) and store up to 4 columns
    if (a_scales)
      for (int r = 0; r < 4; ++r) v[r] = (v[r] * sa) * cols[r];
    const int64_t idx = (int64_t)m_out * N + n;
    if (out_dtype == LFM2_DTYPE_BF16 && n + 3 < N && (N & 3) == 0) {
      bf16x4 o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
      *reinterpret_cast<bf16x4*>((__bf16*)out + idx) = o;
    } else {
      for (int r = 0; r < 4 && n + r < N; ++r) store_out(out, out_dtype, idx + r, v[r]);
    }
  };
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    const int m = m_base + wm * TM + i * 16 + lrow;
    if (m >= M) continue;
    const int m_out = split ? m : mapped_row(rows, m);
    if (m_out < 0) continue;
    float sa = 1.0f;
    if (!split && a_scales) {
      if constexpr (kEarlyScales) sa = early_rows[i];
      else sa = a_scales[m];
    }
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int n = n_base + wn * TN + j * 16 + 4 * lgrp;
      if (n >= N) continue;
      if (split) {
        float* dst = partial + ((int64_t)blockIdx.y * M + m) * N + n;
        if (n + 3 < N && (N & 3) == 0) *reinterpret_cast<f32x4*>(dst) = acc[i][j];
        else for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = acc[i][j][r];
      } else {
        finish(acc[i][j], m_out, n, sa, cw[j]);
      }
    }
  }
}

template <int EB, int BM, int BN, int WM, int WN, int SW, int KS, bool KTAIL, int ST = 0>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_nt_kernel(void* __restrict__ out, float* __restrict__ partial, const uint8_t* __restrict__ A,
               const uint8_t* __restrict__ W, const float* __restrict__ a_scales, const float* __restrict__ w_scales,
               int M, int N, int64_t Kb, int steps_per_split, int out_dtype, RowMap rows) {
  gemm_nt_body<EB, BM, BN, WM, WN, SW, KS, KTAIL, ST, 0>(out, partial, A, W, a_scales, w_scales, M, N, Kb, steps_per_split,
                                                         out_dtype, rows, QkvEpilogue{});
}

template <int ST>
__global__ void __launch_bounds__(256)
gemm_qkv_kernel(const uint8_t* __restrict__ A, const uint8_t* __restrict__ W, const float* __restrict__ a_scales,
                const float* __restrict__ w_scales, int M, int N, int64_t Kb, QkvEpilogue epi) {
  gemm_nt_body<1, 64, 64, 2, 2, 1, 128, false, ST, 1>(nullptr, nullptr, A, W, a_scales, w_scales, M, N, Kb, (int)(Kb / 128),
                                                      LFM2_DTYPE_BF16, RowMap{nullptr, nullptr, 0x7fffffff}, epi);
}

// The gate+up projection with SwiGLU as its epilogue, on the tiles the default plan gives that projection: the 8-wave
// 128 x 128 ring tile at large M and the 16-wave 128 x 96 tile of the decode batch.
template <int EB, int BM, int BN, int WM, int WN, int ST>
__global__ void __launch_bounds__(WM * WN * 64)
gemm_swiglu_kernel(void* __restrict__ out, const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                   const float* __restrict__ a_scales, const float* __restrict__ w_scales, int M, int N, int64_t Kb,
                   int out_dtype) {
  gemm_nt_body<EB, BM, BN, WM, WN, EB == 1 ? 1 : 0, 128, false, ST, 2>(out, nullptr, A, W, a_scales, w_scales, M, N, Kb,
                                                                         (int)(Kb / 128), out_dtype,
                                                                         RowMap{nullptr, nullptr, 0x7fffffff}, QkvEpilogue{});
}

// The conv in-projection with the short-conv update as its epilogue, on the 64 x 96 tile of the decode batch.
template <int EB>
__global__ void __launch_bounds__(512)
gemm_conv_kernel(void* __restrict__ out, const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                 const float* __restrict__ a_scales, const float* __restrict__ w_scales, int M, int N, int64_t Kb,
                 int out_dtype, ConvEpilogue conv) {
  gemm_nt_body<EB, 64, 96, 4, 2, EB == 1 ? 1 : 0, 128, false, 4, 3>(out, nullptr, A, W, a_scales, w_scales, M, N, Kb,
                                                                     (int)(Kb / 128), out_dtype,
                                                                     RowMap{nullptr, nullptr, 0x7fffffff}, QkvEpilogue{}, conv);
}

// Sum split-K partials in split order, then scale (row scale, then column scale).  A separate launch on purpose:
// the eight XCDs have private L2s, so partials written by workgroups on other XCDs are only visible to a reader
// cheaply at a kernel boundary; an in-kernel "last workgroup reduces" scheme needs device-scope fences that write
// back and invalidate L2 and measured ten times slower.
__global__ void __launch_bounds__(256)
reduce_split_kernel(void* out, const float* partial, const float* a_scales, const float* w_scales, int64_t M, int64_t N,
                    int splits, int out_dtype) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * N) return;
  float t = 0.f;
  for (int s = 0; s < splits; ++s) t += partial[(int64_t)s * M * N + idx];
  if (a_scales) t = (t * a_scales[idx / N]) * w_scales[idx % N];
  store_out(out, out_dtype, idx, t);
}

// Any-shape fallback (K not a multiple of 16 bytes): one thread per output element.
template <int EB>
__global__ void __launch_bounds__(256)
gemm_naive_kernel(void* out, const uint8_t* A, const uint8_t* W, const float* a_scales, const float* w_scales, int64_t M,
                  int64_t N, int64_t K, int out_dtype, RowMap rows) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * N) return;
  const int64_t m = idx / N, n = idx % N;
  const int m_out = mapped_row(rows, (int)m);
  if (m_out < 0) return;
  float t = 0.f;
  if (EB == 1) {
    const uint8_t *a = A + m * K, *w = W + n * K;
    for (int64_t k = 0; k < K; ++k) {
      f32x2 x = __builtin_amdgcn_cvt_pk_f32_fp8((int)a[k], false), y = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[k], false);
      t = fmaf(x[0], y[0], t);
    }
  } else {
    const __bf16 *a = (const __bf16*)A + m * K, *w = (const __bf16*)W + n * K;
    for (int64_t k = 0; k < K; ++k) t = fmaf((float)a[k], (float)w[k], t);
  }
  if (a_scales) t = (t * a_scales[m]) * w_scales[n];
  store_out(out, out_dtype, (int64_t)m_out * N + n, t);
}

// ------------------------------------------------------------------------------------ few rows: everything in flight at once
// Up to 64 rows the tiled kernels are a serial chain: a workgroup walks its K loop step by step behind a ring a few
// steps deep, so a launch lasts several memory latencies whatever the shape (6.5-7.5 us for every K = 2048 projection
// at 1-16 rows, on 32-176 workgroups of a 256-CU chip).  This kernel has no K loop.  A workgroup owns 16 NI output
// columns (weight rows) and all rows of the batch; its waves split K among themselves, 128-byte steps dealt round
// robin, and every wave loads ALL of its operand fragments straight into registers in the MFMA's own layout (lane
// l: row l % 16, bytes 32 (l / 16) .. + 31 of a step: no staging through LDS, no barrier before the MFMAs), one memory
// latency deep.  The waves' partial tiles meet in LDS and are summed in wave order.  N / (16 NI) workgroups, times the
// parts of K when the product is left as partial sums for the norm that follows it.
//   EPI 0: out[m, n] = (acc * a_scale[m]) * w_scale[n] with optional row placement; EPI 2: SwiGLU over interleaved
//   gate/up weight rows as in the tiled kernel's epilogue, out [M, N / 2]; EPI 4: fp32 partial sums of this
//   workgroup's part of K, partial[blockIdx.y][m][n].
template <int MI, int NI, int WAVES, int MAXS, int EPI>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(void* __restrict__ out, const uint8_t* __restrict__ A, const uint8_t* __restrict__ W,
                   const float* __restrict__ a_scales, const float* __restrict__ w_scales, int M, int N, int64_t Kb,
                   int steps_per_part, int out_dtype, RowMap rows) {
  typedef StepMfma<1>::frag frag;
  __shared__ f32x4 red[WAVES][MI * NI][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, lgrp = lane >> 4;
  const int n_base = blockIdx.x * (16 * NI);
  const int step0 = blockIdx.y * steps_per_part;
  int nsteps = (int)(Kb / kStepBytes) - step0;
  nsteps = nsteps < steps_per_part ? nsteps : steps_per_part;
  const uint8_t* wp[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    int n = n_base + 16 * j + lrow;
    n = n < N ? n : N - 1;
    wp[j] = W + (int64_t)(EPI == 2 ? swiglu_weight_row(n, N) : n) * Kb + 32 * lgrp;
  }
  const uint8_t* ap[MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) {
    int m = i * 16 + lrow;
    m = m < M ? m : M - 1;
    ap[i] = A + (int64_t)m * Kb + 32 * lgrp;
  }
  // the scales of the output item this thread finishes (at most one when the items fit the workgroup), asked for with
  // the operands: at the end they would be one more memory round trip
  constexpr bool kOneItem = MI * NI <= WAVES && EPI != 4;
  float item_row_scale = 1.0f, item_cols[8];
  if constexpr (kOneItem) {
    if (tid < MI * NI * 64) {
      const int tile = tid >> 6, l = tid & 63, m = (tile / NI) * 16 + (l & 15), col = n_base + 16 * (tile % NI) + 4 * (l >> 4);
      if (m < M && col < N) {
        item_row_scale = a_scales[m];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if constexpr (EPI == 2) {
            item_cols[r] = w_scales[swiglu_weight_row(col + r, N)];
            item_cols[4 + r] = l < 32 ? w_scales[swiglu_weight_row(col + 8 + r, N)] : 0.f;
          } else {
            item_cols[r] = w_scales[col + r];
          }
        }
      }
    }
  }
  // every load of the wave, unconditionally (a step beyond the last is the last one again and is not multiplied)
  frag fw[MAXS][NI], fa[MAXS][MI];
#pragma unroll
  for (int t = 0; t < MAXS; ++t) {
    int step = wave + t * WAVES;
    step = step < nsteps ? step : nsteps - 1;
    const int64_t kb = (int64_t)(step0 + step) * kStepBytes;
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const i32x4 lo = *reinterpret_cast<const i32x4*>(wp[j] + kb), hi = *reinterpret_cast<const i32x4*>(wp[j] + kb + 16);
      fw[t][j] = frag{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int i = 0; i < MI; ++i) {
      const i32x4 lo = *reinterpret_cast<const i32x4*>(ap[i] + kb), hi = *reinterpret_cast<const i32x4*>(ap[i] + kb + 16);
      fa[t][i] = frag{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  }
  f32x4 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < MAXS; ++t) {
    if (wave + t * WAVES < nsteps) {   // the same for the whole wave
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = StepMfma<1>::run(fw[t][j], fa[t][i], acc[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) red[wave][i * NI + j][lane] = acc[i][j];
  __syncthreads();
  // item (i, j, l) finishes out[m = 16 i + l % 16][n = n_base + 16 j + 4 (l / 16) + r]: the waves' partial sums in wave order
  auto total = [&](int tile, int l) {
    f32x4 v = red[0][tile][l];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) v += red[w][tile][l];
    return v;
  };
  for (int item = tid; item < MI * NI * 64; item += WAVES * 64) {
    const int tile = item >> 6, l = item & 63, i = tile / NI, j = tile % NI;
    const int m = i * 16 + (l & 15), grp = l >> 4;
    if (m >= M) continue;
    const int col = n_base + 16 * j + 4 * grp;
    if (col >= N) continue;
    if constexpr (EPI == 4) {
      *reinterpret_cast<f32x4*>((float*)out + ((int64_t)blockIdx.y * M + m) * N + col) = total(tile, l);
      continue;
    }
    const float sa = kOneItem ? item_row_scale : a_scales[m];
    if constexpr (EPI == 2) {
      // lane groups 0, 1 hold gate columns 0-7 of a tile, groups 2, 3 (32 lanes on) the up columns that pair with them
      if (l >= 32) continue;
      const f32x4 gate = total(tile, l), up = total(tile, l + 32);
      auto finish = [&](auto tag) {
        typedef decltype(tag) T;
        float h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float gs = kOneItem ? item_cols[r] : w_scales[swiglu_weight_row(col + r, N)];
          const float us = kOneItem ? item_cols[4 + r] : w_scales[swiglu_weight_row(col + 8 + r, N)];
          const float g = round_to<T>((gate[r] * sa) * gs);
          const float u = round_to<T>((up[r] * sa) * us);
          h[r] = round_to<T>(round_to<T>(silu_f(g)) * u);
        }
        T* dst = (T*)out + (int64_t)m * (N >> 1) + ((n_base + 16 * j) >> 1) + 4 * grp;
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[r] = Elem<T>::store(h[r]);
      };
      if (out_dtype == LFM2_DTYPE_BF16) finish(__bf16{});
      else if (out_dtype == LFM2_DTYPE_F16) finish(_Float16{});
      else finish(float{});
      continue;
    }
    const int m_out = mapped_row(rows, m);
    if (m_out < 0) continue;
    f32x4 v = total(tile, l);
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = (v[r] * sa) * (kOneItem ? item_cols[r] : w_scales[col + r]);
    const int64_t idx = (int64_t)m_out * N + col;
    if (out_dtype == LFM2_DTYPE_BF16) {
      bf16x4 o = {(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]};
      *reinterpret_cast<bf16x4*>((__bf16*)out + idx) = o;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) store_out(out, out_dtype, idx + r, v[r]);
    }
  }
}

// Whether the few-row kernel serves an e4m3 product: whole 128-byte steps, whole 16-column tiles, at most 64 rows, and
// few enough steps per wave that all of a wave's fragments fit in its registers (16 waves share the steps of a long
// K).  `parts` > 1: the product is left as that many partial sums along K (one workgroup row per part).
constexpr int kSkinnyTile = 60;
struct SkinnyShape { int mi, ni, waves, maxs, per_part; };
bool skinny_shape(int64_t M, int64_t N, int64_t Kb, int parts, SkinnyShape* shape, bool wide = true) {
  if (M <= 0 || M > 64 || N <= 0 || N % 16 != 0 || Kb % kStepBytes != 0 || Kb < kStepBytes || parts < 1) return false;
  const int steps = (int)(Kb / kStepBytes), mi = (int)((M + 15) / 16);
  if (steps < parts) return false;
  const int per_part = (steps + parts - 1) / parts;
  if ((int64_t)per_part * (parts - 1) >= steps) return false;   // a part without a step
  const int waves = per_part > 16 ? 16 : 8;
  const int maxs = (per_part + waves - 1) / waves;
  if (maxs > 4) return false;
  // Where it wins (weights streamed from HBM, launches replayed in a graph, us per launch against the tiled plan):
  // N 2048 and 3072, K 2048: 4.1-4.8 against 6.2-6.4 at 1-16 rows, 5.8 against 7.2 at 32, level at 48-64; N 6144:
  // 5.6-6.4 against 7.0-7.2 at 1-16 rows, 7.2 against 7.9 at 32, behind from 48 on; N 11264: behind everywhere (the
  // tiled kernel is already at the 23 MB's streaming time); K 5632 whole: 6.9-7.5 against 8.1-8.3 at 1-8 rows, level at 16.
  const int64_t row_limit = steps <= 16 ? (N <= 4096 ? 48 : N <= 8192 ? 32 : 0) : (parts > 1 ? 32 : N <= 4096 ? 8 : 0);
  if (M > row_limit) return false;
  // wide outputs on few rows: several column tiles per workgroup, while at least 128 workgroups remain (every workgroup
  // reads all of the activations, so fewer of them re-read less)
  int ni = 1;
  if (wide && parts == 1 && waves == 8 && mi <= 2) ni = N % 64 == 0 && N / 64 >= 128 ? 4 : N % 32 == 0 && N / 32 >= 128 ? 2 : 1;
  // registers a lane holds in flight: 8 per weight fragment and 8 per activation fragment of every step
  if (maxs * (8 * ni + 8 * mi) + 4 * mi * ni > (waves == 16 ? 104 : 200)) return false;
  if (shape) *shape = SkinnyShape{mi, ni, waves, maxs, per_part};
  return true;
}

template <int EPI>
bool launch_skinny(void* out, const uint8_t* A, const uint8_t* W, const float* as, const float* ws, int64_t M, int64_t N,
                   int64_t Kb, int parts, int out_dtype, RowMap rows, hipStream_t s) {
  SkinnyShape shape;
  if (!skinny_shape(M, N, Kb, parts, &shape, EPI != 4)) return false;   // partial sums: one column tile per workgroup
  const dim3 grid((unsigned)(N / (16 * shape.ni)), (unsigned)parts);
#define SKINNY_(MI, NI, WAVES, MAXS)                                                                                    \
  if (shape.mi == MI && shape.ni == NI && shape.waves == WAVES && shape.maxs == MAXS) {                                 \
    hipLaunchKernelGGL((gemm_skinny_kernel<MI, NI, WAVES, MAXS, EPI>), grid, dim3(WAVES * 64), 0, s, out, A, W, as, ws, \
                       (int)M, (int)N, Kb, shape.per_part, out_dtype, rows);                                            \
    return true;                                                                                                        \
  }
#define SKINNY_ROWS_(WAVES, MAXS) SKINNY_(1, 1, WAVES, MAXS) SKINNY_(2, 1, WAVES, MAXS) SKINNY_(3, 1, WAVES, MAXS) SKINNY_(4, 1, WAVES, MAXS)
  SKINNY_ROWS_(8, 1) SKINNY_ROWS_(8, 2) SKINNY_ROWS_(16, 2) SKINNY_ROWS_(16, 3) SKINNY_ROWS_(16, 4)
  if constexpr (EPI != 4) {
    SKINNY_(1, 2, 8, 1) SKINNY_(2, 2, 8, 1) SKINNY_(1, 4, 8, 1) SKINNY_(2, 4, 8, 1)
    SKINNY_(1, 2, 8, 2) SKINNY_(2, 2, 8, 2) SKINNY_(1, 4, 8, 2) SKINNY_(2, 4, 8, 2)
  }
#undef SKINNY_ROWS_
#undef SKINNY_
  return false;
}

struct TileInfo { int bm, bn, ks; };
constexpr int kNumTiles = 62;
constexpr TileInfo kTiles[kNumTiles] = {{16, 64, 128}, {32, 64, 128}, {64, 64, 128}, {128, 64, 128}, {128, 128, 128},
                                        {64, 128, 128}, {128, 128, 128}, {64, 128, 128}, {128, 64, 128},
                                        {16, 64, 256}, {32, 64, 256}, {64, 64, 256},
                                        {32, 64, 128}, {64, 64, 128}, {128, 128, 128}, {32, 64, 256},
                                        {64, 64, 128}, {32, 64, 128}, {16, 64, 256}, {128, 64, 128}, {64, 128, 128},
                                        {16, 64, 128}, {128, 64, 128},
                                        {64, 176, 128}, {64, 176, 128}, {64, 96, 128}, {64, 96, 128}, {256, 128, 128},
                                        {256, 128, 128}, {64, 128, 128}, {128, 176, 128}, {128, 96, 128}, {64, 128, 128},
                                        {32, 128, 128},
                                        {64, 192, 128}, {64, 192, 128}, {128, 96, 128}, {64, 96, 128}, {64, 64, 128},
                                        {64, 96, 128}, {128, 96, 128},
                                        {128, 96, 256}, {64, 96, 256}, {128, 96, 128}, {128, 96, 256}, {64, 96, 256},
                                        {32, 64, 128}, {32, 64, 256}, {32, 64, 256}, {64, 64, 256},
                                        {256, 48, 128}, {256, 48, 128}, {256, 32, 128}, {256, 64, 128}, {256, 48, 128},
                                        {256, 32, 128},
                                        {256, 128, 128}, {128, 256, 128}, {256, 256, 128}, {128, 128, 128},
                                        {64, 16, 128},   // 60: the few-row kernel (all rows, 16 columns)
                                        {256, 192, 128}};
int64_t tile_steps(int tile, int64_t Kb) { return (Kb + kTiles[tile].ks - 1) / kTiles[tile].ks; }

struct Plan { int tile, splits; };

// Default tile/split choice, from sweeps on MI355X at M = 256 (decode, weights streaming from HBM inside a HIP graph)
// and M = 4096 (prefill).  Above 64 rows the direct-to-LDS ring variants win everywhere: the 8-wave 128x128 tile
// once it alone fills the 256 CUs (1.3-2.0 PFLOP/s at M = 4096; 42 us for the 65536-row head at M = 256), otherwise
// smaller tiles with deeper rings the fewer workgroups a CU gets (its K loop is then a serial chain that nothing
// overlaps).  With K bytes not a multiple of the step these indices run their register-staged twins.
Plan default_plan(int64_t M, int64_t N, int64_t Kb, bool deferred = false, int eb = 2) {
  if (eb == 1 && skinny_shape(M, N, Kb, 1, nullptr)) {
    // a long K on a narrow output whose partial sums the next norm adds up anyway (the down projection of a small decode
    // batch: 44 steps on 128 column tiles): two parts of K, 256 workgroups
    if (deferred && Kb / kStepBytes >= 32 && N / 16 <= 128 && skinny_shape(M, N, Kb, 2, nullptr)) return {kSkinnyTile, 2};
    return {kSkinnyTile, 1};
  }
  auto count = [&](int t) { return ((M + kTiles[t].bm - 1) / kTiles[t].bm) * ((N + kTiles[t].bn - 1) / kTiles[t].bn); };
  const int64_t steps = (Kb + kStepBytes - 1) / kStepBytes;
  // Few output tiles on a K loop of 32 steps or more: split K (2 or 4 ways) while every part keeps 8 steps and the
  // launch stays within about 256 workgroups.  Weights streamed from HBM, product + reduce launch, 16 rows: e4m3
  // N 2048 K 5632 7.9 us against 19.6 unsplit; bf16 N 2048 K 2048 6.4 against 14.6, N 6144 8.8 against 9.4,
  // K 5632 9.6 against 35.  K loops of 16 steps (e4m3, K 2048) gain nothing from a split.
  auto splits_for = [&](int64_t tiles) {
    if (steps < 32) return 1;
    const int64_t most = std::min<int64_t>(std::min<int64_t>(4, steps / 8), 256 / std::max<int64_t>(tiles, 1));
    return most >= 4 ? 4 : most >= 2 ? 2 : 1;
  };
  // up to 64 rows the direct-to-LDS rings win over register staging by 25-40 % once the weights come from HBM
  // (e4m3 N 3072: 6.2 / 7.2 / 7.1 us at 16 / 32 / 64 rows against 9.2 / 10.9 / 12.9)
  // A short K loop on few tiles whose partial sums the next norm adds up anyway (the out projection of a small decode
  // batch): four parts of K (16 rows, N 2048, K 2048: 3.3 us against 4.8 whole; the reduce launch would cost more)
  if (deferred && M <= 64 && steps >= 16 && steps < 32) {
    const int t = M <= 16 ? 18 : 17;
    if (count(t) * 4 <= 256) return {t, 4};
  }
  if (M <= 16) return {18, splits_for(count(18))};            // 16x64, 256-byte steps, ring of 3
  if (M <= 32) return {17, splits_for(count(17))};            // 32x64, ring of 5
  if (M <= 64 && count(1) <= 256) return {17, splits_for(count(17))};
  if (steps >= 64 && count(13) <= 256) {
    // a long K loop on few output tiles (the bf16 down projection at decode: 88 steps on 128 tiles): split K so that
    // about 512 workgroups share it.  M 256, N 2048, 11264 K bytes: 16.5 us against 24.3 (bf16), 21.1 against 22.4
    // (e4m3); M 128: 13.0 against 24.5
    // where 64x128 tiles of 8 waves on four parts of K make one workgroup per CU they pull fewer bytes into it: the
    // same shape 14.9 us alone against 17.5, the all-bf16 decode step 2.036 against 2.070 ms
    if (count(29) * 4 > 128 && count(29) * 4 <= 256) return {29, 4};
    const int splits = (int)(512 / count(13));
    return {13, splits > 4 ? 4 : splits};
  }
  // A product whose partial sums the next norm adds up (the e4m3 down projection of a decode step: 44 steps on a
  // 256 x 2048 output): 64x64 tiles on two halves of K, one workgroup per CU.  Alone 9.9 us against 13.1 for the
  // unsplit 32x64 tiles; the norm then reads two fp32 partials instead of one 16-bit product, which leaves 6 us of
  // the step's 1.48 ms (four-way splits on 64x128 tiles: 9.5 us alone, nothing left in the step).
  if (deferred && M > 128 && M <= 256 && steps >= 32 && steps < 64 && count(16) <= 128) return {16, 2};
  // One tile per CU, as square as the output allows, with many waves: the K loop moves about 50 B/ns into a CU
  // whatever the ring depth or step size, so the bytes a CU pulls decide (tile rows + columns, times K).
  // 256 rows: N 11264 on 128x96 tiles of 16 waves 15.4 us against 19.4 on 64x64; N 6144 on 64x96 tiles of 8 waves
  // 10.9 against 13.1; 512 rows, N 6144 on 128x96 tiles of 8 waves 15.2 against 17.7.
  // 65-128 rows of a wide output: 64x96 tiles of 8 waves, one per CU (N 11264: 11.0 us against 14.7 and more on 32x64 tiles)
  if (M > 64 && M <= 128 && steps <= 32 && N >= 8192 && count(37) <= 256 && count(37) > 128) return {37, 1};
  // and of a narrow one: 16x64 tiles with 256-byte steps, one per CU (128 rows, N 2048, K 2048: 4.9 us against 6.0)
  if (M > 64 && M <= 128 && steps <= 16 && count(18) <= 256 && count(18) > 128) return {18, 1};
  if (M > 128 && M <= 256 && steps <= 32) {
    if (N % 96 == 0 && count(37) <= 256 && count(37) > 128) return {37, 1};
    if (N >= 8192 && count(36) <= 256) return {36, 1};
  }
  // 257-512 rows: the same 128x96 tile of 16 waves (N 6144: 13.6 us against 15.0 with 8 waves), and for the widest
  // outputs 256x128 tiles of 16 waves, which halve the weight bytes a CU pulls (N 11264: 23.2 us against 26.2 on
  // 128x128 tiles)
  if (M > 256 && M <= 512 && steps <= 32 && N % 96 == 0 && count(36) <= 256 && count(36) > 128) return {36, 1};
  if (M > 256 && M <= 512 && steps <= 32 && N >= 8192 && count(56) <= 256) return {56, 1};
  // The vocabulary projection at a decode batch (N 65536): one 256x256 tile per CU instead of four 128x128 tiles
  // halves the activation bytes a CU pulls (M 256: 48.8 us against 60.0; M 512: 79.4 against 103.9; up to 128 rows the
  // 128x128 tile stays ahead, 37.6 against 43.9).
  if (M > 192 && M <= 512 && N >= 32768 && N % 256 == 0 && Kb % kStepBytes == 0 && steps <= 32) return {58, 1};
  // Prefill-sized e4m3 products (more than 512 rows, at least a round of 128x128 tiles): the 128x128 tile of 8 waves
  // (two workgroups per CU), the 256x128 tile of 16 waves or the 256x256 tile of 16 waves (one per CU), whichever
  // finishes its rounds over the 256 CUs first.  A round's time goes with the tile's area (times the workgroups that
  // share a CU); against the 128x128 tile at equal rounds the 256x128 tile is 7 % faster and the 256x256 tile 27 %
  // (its waves read a third fewer LDS bytes per MFMA: 64x64 wave tiles instead of 64x32).  Measured, weights streaming,
  // us at 4096 / 3400 / 2688 rows for the three tiles: N 11264 147 / 137 / 115, 123 / 115 / 108, 103 / 94 / 78; N 6144
  // 78 / 71 / 75, 67 / 68 / 70, 51 / 64 / 69; N 3072 45 / 45 / 37, 38 / 42 / 36, 26 / 41 / 36; N 2048 K 5632 58 / 49 / 70,
  // 53 / 48 / 70, 48 / 45 / 70: the model picks the fastest of each triple, and at 640-2304 rows the fastest or one within
  // 2 % of it (N 11264: 128x128 at 640 rows, 256x256 at 768-1280 and 2304, 256x128 at 1536-2048).
  if (eb == 1 && M > 512 && Kb % kStepBytes == 0 && count(6) >= 256) {
    auto cost = [&](int t, int per_cu, double speed) {
      const int64_t rounds = (count(t) + 256 * per_cu - 1) / (256 * per_cu);
      return (double)rounds * kTiles[t].bm * kTiles[t].bn * per_cu / speed;
    };
    // a last round of 128x128 tiles that leaves every CU at most one workgroup takes three quarters of a full one
    // (2048 rows, N 2048: 19.7 us for 256 tiles, 26.1 us for the 512 tiles of 4096 rows)
    const int64_t rest14 = count(14) % 512;
    const double c14 = cost(14, 2, 1.0) - (rest14 > 0 && rest14 <= 256 ? 0.5 * 128 * 128 : 0.0);
    const double c56 = cost(56, 1, 1.07), c58 = cost(58, 1, 1.27);
    // and a 256x192 tile of 16 waves (64x48 wave tiles, speed 1.15) for the widths it cuts into whole rounds: N 3072 at
    // 4096 rows is one round of 256 tiles (32 us against 37 on 192 tiles of 256x256), N 6144 two rounds (65 against 70
    // on three rounds of 256x128; N 11264 at 2048 rows two rounds of 472 tiles, 63 us against 71).
    const double c61 = cost(61, 1, 1.15);
    if (c61 < c14 && c61 < c56 && c61 < c58) return {61, 1};
    if (c58 < c14 && c58 <= c56) return {58, 1};
    if (c56 < c14) return {56, 1};
    return {14, 1};
  }
  if (count(6) >= 256) return {14, 1};                // 128x128, ring of 2
  if (count(2) >= 512) return {13, 1};                // 64x64, ring of 3
  // one round of 64x64 tiles over the 256 CUs beats two rounds of 32x64 (512 rows, N 2048: K 5632 16.8 us against
  // 21.0, K 2048 8.9 against 9.9)
  if (count(1) > 384 && count(2) <= 256) return {38, 1};   // sixteen waves (512 rows, N 2048: 8.1 us against 8.9 with four)
  if (count(1) > 384) return {15, 1};                 // 32x64, 256-byte steps, ring of 2
  if (count(1) > 256) return {38, 1};                 // 64x64, ring of 4, sixteen waves (128 rows, N 6144: 8.5 us against 9.2 with four)
  // 32x64, ring of 5 (a long K loop; above 128 rows a short one as well: the out projection of the 256-row decode step
  // gains 5-11 us per step over the ring of 4, which is level with it alone) or 4
  return {steps >= 32 || M > 128 ? 17 : 12, splits_for(count(1))};
}

template <int EB, int BM, int BN, int WM, int WN, int SW, int KS, int ST = 0>
void launch_tile(void* out, float* partial, const uint8_t* A, const uint8_t* W, const float* as, const float* ws, int M,
                 int N, int64_t Kb, int splits, int out_dtype, bool keep_partials, RowMap rows, hipStream_t s) {
  const int tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
  const int64_t steps = (Kb + KS - 1) / KS;
  const int per = (int)((steps + splits - 1) / splits);
  const dim3 grid((tiles + 7) / 8 * 8, splits), block(WM * WN * 64);
  if (Kb % KS == 0)
    hipLaunchKernelGGL((gemm_nt_kernel<EB, BM, BN, WM, WN, SW, KS, false, ST>), grid, block, 0, s, out, (splits > 1 || keep_partials) ? partial : nullptr, A, W,
                       as, ws, M, N, Kb, per, out_dtype, rows);
  else
    hipLaunchKernelGGL((gemm_nt_kernel<EB, BM, BN, WM, WN, SW, KS, true>), grid, block, 0, s, out, (splits > 1 || keep_partials) ? partial : nullptr, A, W,
                       as, ws, M, N, Kb, per, out_dtype, rows);
}

// The fused QKV projection on one of the 64 x 64 ring tiles (ST buffers).
template <int ST>
void launch_qkv(const uint8_t* A, const uint8_t* W, const float* as, const float* ws, int M, int N, int64_t Kb,
                const QkvEpilogue& epi, hipStream_t s) {
  const int tiles = ((M + 63) / 64) * (N / 64);
  const dim3 grid((tiles + 7) / 8 * 8, 1), block(256);
  hipLaunchKernelGGL(gemm_qkv_kernel<ST>, grid, block, 0, s, A, W, as, ws, M, N, Kb, epi);
}

template <int EB>
int gemm_entry(const char* name, void* out, const void* a, const float* as, const void* w, const float* ws,
               float* workspace, int64_t M, int64_t N, int64_t K, int out_dtype, int tile, int split_k, void* stream,
               bool reduce = true, RowMap rows = {nullptr, nullptr, 0x7fffffff}) {
  LFM2_REQUIRE(M > 0 && N > 0 && K > 0, "%s: empty shape", name);
  LFM2_REQUIRE(M < (1 << 30) && N < (1 << 30), "%s: M or N too large", name);
  LFM2_REQUIRE(out_dtype >= LFM2_DTYPE_BF16 && out_dtype <= LFM2_DTYPE_F32, "%s: bad output dtype", name);
  hipStream_t s = (hipStream_t)stream;
  const uint8_t *A = (const uint8_t*)a, *W = (const uint8_t*)w;
  const int64_t Kb = K * EB;
  if (Kb % 16 != 0 || ((uintptr_t)a | (uintptr_t)w) % 16 != 0) {
    LFM2_REQUIRE(reduce, "%s: partial products need K bytes and pointers aligned to 16", name);
    hipLaunchKernelGGL(gemm_naive_kernel<EB>, dim3(ceil_div(M * N, 256)), dim3(256), 0, s, out, A, W, as, ws, M, N, K, out_dtype, rows);
    LFM2_LAUNCH_CHECK();
  }
  // the few-row kernel finishes its product itself: it serves the default plan of a product that is neither split on
  // request nor left as partial sums
  // the few-row kernel finishes its product itself, or leaves it as the partial sums of its own plan: it serves the
  // default plan of a product that is not split on request
  Plan plan = default_plan(M, N, Kb, !reduce, (tile < 0 && (reduce ? split_k <= 1 : true)) ? EB : 2);
  if (!reduce && tile < 0 && plan.tile == kSkinnyTile && split_k > 0 && split_k != plan.splits)
    plan = default_plan(M, N, Kb, true, 2);   // another number of parts than the few-row plan's: the tiled kernels
  if (tile >= 0) {
    LFM2_REQUIRE(tile < kNumTiles, "%s: tile index %d out of range", name, tile);
    plan.tile = tile;
  }
  if (plan.tile == kSkinnyTile) {
    LFM2_REQUIRE(EB == 1, "%s: the few-row kernel takes e4m3 operands", name);
    const int parts = reduce ? 1 : (split_k > 0 ? split_k : plan.splits);
    LFM2_REQUIRE(!reduce || split_k <= 1, "%s: the few-row kernel splits K only for partial sums", name);
    const bool ok = reduce ? launch_skinny<0>(out, A, W, as, ws, M, N, Kb, 1, out_dtype, rows, s)
                           : launch_skinny<4>(workspace, A, W, as, ws, M, N, Kb, parts, LFM2_DTYPE_F32, rows, s);
    if (ok) LFM2_LAUNCH_CHECK();
    LFM2_FAIL(LFM2_ERR_UNSUPPORTED, "%s: the few-row kernel does not cover M %ld, N %ld, K bytes %ld in %d parts", name,
              (long)M, (long)N, (long)Kb, parts);
  }
  if (split_k > 0) plan.splits = split_k;
  else if (rows.slots || rows.active) plan.splits = 1;   // placed rows are written by the product itself
  LFM2_REQUIRE(plan.splits == 1 || (!rows.slots && !rows.active), "%s: placed output rows do not combine with split-K", name);
  const int64_t steps = tile_steps(plan.tile, Kb);
  if (plan.splits > steps) plan.splits = (int)steps;
  // every split must own at least one step
  while (plan.splits > 1 && (steps + plan.splits - 1) / plan.splits * (plan.splits - 1) >= steps) --plan.splits;
  LFM2_REQUIRE(plan.splits == 1 || workspace != nullptr, "%s: split-K needs a workspace", name);
  LFM2_REQUIRE(reduce || workspace != nullptr, "%s: partial products need a destination", name);
#define TILE_(ID, BM, BN, WM, WN, KS, ...) \
  case ID: launch_tile<EB, BM, BN, WM, WN, EB == 1 ? 1 : 0, KS, ##__VA_ARGS__>(out, workspace, A, W, as, ws, (int)M, (int)N, Kb, plan.splits, out_dtype, !reduce, rows, s); break
  switch (plan.tile) {
    TILE_(0, 16, 64, 1, 4, 128);
    TILE_(1, 32, 64, 2, 2, 128);
    TILE_(2, 64, 64, 2, 2, 128);
    TILE_(3, 128, 64, 2, 2, 128);
    TILE_(4, 128, 128, 2, 2, 128);
    TILE_(5, 64, 128, 2, 2, 128);
    TILE_(6, 128, 128, 2, 4, 128);
    TILE_(7, 64, 128, 2, 4, 128);
    TILE_(8, 128, 64, 4, 2, 128);
    TILE_(9, 16, 64, 1, 4, 256);
    TILE_(10, 32, 64, 2, 2, 256);
    TILE_(11, 64, 64, 2, 2, 256);
    TILE_(12, 32, 64, 2, 2, 128, 4);
    TILE_(13, 64, 64, 2, 2, 128, 3);
    TILE_(14, 128, 128, 2, 4, 128, 2);
    TILE_(15, 32, 64, 2, 2, 256, 2);
    TILE_(16, 64, 64, 2, 2, 128, 4);
    TILE_(17, 32, 64, 2, 2, 128, 5);
    TILE_(18, 16, 64, 1, 4, 256, 3);
    TILE_(19, 128, 64, 4, 2, 128, 2);
    TILE_(20, 64, 128, 2, 4, 128, 2);
    TILE_(21, 16, 64, 1, 4, 128, 4);
    TILE_(22, 128, 64, 2, 2, 128, 2);
    TILE_(23, 64, 176, 4, 1, 128, 3);
    TILE_(24, 64, 176, 4, 1, 128, 4);
    TILE_(25, 64, 96, 2, 2, 128, 4);
    TILE_(26, 64, 96, 2, 2, 128, 3);
    TILE_(27, 256, 128, 4, 2, 128, 2);
    TILE_(28, 256, 128, 4, 2, 128, 3);
    TILE_(29, 64, 128, 2, 4, 128, 4);
    TILE_(30, 128, 176, 4, 1, 128, 3);
    TILE_(31, 128, 96, 4, 2, 128, 3);
    TILE_(32, 64, 128, 2, 2, 128, 4);
    TILE_(33, 32, 128, 2, 2, 128, 4);
    TILE_(34, 64, 192, 2, 4, 128, 3);
    TILE_(35, 64, 192, 4, 4, 128, 3);
    TILE_(36, 128, 96, 8, 2, 128, 3);
    TILE_(37, 64, 96, 4, 2, 128, 4);
    TILE_(38, 64, 64, 4, 4, 128, 4);
    TILE_(39, 64, 96, 4, 2, 128, 6);
    TILE_(40, 128, 96, 4, 2, 128, 4);
    TILE_(41, 128, 96, 8, 2, 256, 2);
    TILE_(42, 64, 96, 4, 2, 256, 3);
    TILE_(43, 128, 96, 8, 2, 128, 5);
    TILE_(44, 128, 96, 4, 2, 256, 2);
    TILE_(45, 64, 96, 2, 2, 256, 3);
    TILE_(46, 32, 64, 2, 2, 128, 8);
    TILE_(47, 32, 64, 2, 2, 256, 4);
    TILE_(48, 32, 64, 2, 2, 256, 6);
    TILE_(49, 64, 64, 2, 2, 256, 4);
    TILE_(50, 256, 48, 8, 1, 128, 3);
    TILE_(51, 256, 48, 16, 1, 128, 3);
    TILE_(52, 256, 32, 8, 1, 128, 3);
    TILE_(53, 256, 64, 8, 1, 128, 3);
    TILE_(54, 256, 48, 8, 1, 128, 4);
    TILE_(55, 256, 32, 16, 1, 128, 4);
    TILE_(56, 256, 128, 4, 4, 128, 3);
    TILE_(57, 128, 256, 2, 4, 128, 3);
    TILE_(58, 256, 256, 4, 4, 128, 2);
    TILE_(59, 128, 128, 2, 4, 128, 3);
    TILE_(61, 256, 192, 4, 4, 128, 2);
  }
#undef TILE_
  if (plan.splits > 1 && reduce)
    hipLaunchKernelGGL(reduce_split_kernel, dim3(ceil_div(M * N, 256)), dim3(256), 0, s, out, workspace, as, ws, M, N,
                       plan.splits, out_dtype);
  LFM2_LAUNCH_CHECK();
}

}  // namespace

extern "C" int lfm2_fp8_gemm(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q,
                             const float* w_scales, float* workspace, int64_t M, int64_t N, int64_t K, int out_dtype,
                             int tile, int split_k, void* stream) {
  LFM2_REQUIRE(a_scales && w_scales, "fp8_gemm: scales are required");
  LFM2_REQUIRE(split_k <= 16, "fp8_gemm: split_k above 16");
  return gemm_entry<1>("fp8_gemm", out, a_q, a_scales, w_q, w_scales, workspace, M, N, K, out_dtype, tile, split_k, stream);
}

namespace {
// The fused form exists for the tile the default plan takes at large M; other shapes use the two launches.
bool swiglu_fits(int64_t M, int64_t N, int64_t Kb, int eb) {
  if (M <= 0 || N <= 0 || Kb <= 0 || N % 16 != 0 || Kb % kStepBytes != 0 || M >= (1 << 30) || N >= (1 << 30)) return false;
  const Plan plan = default_plan(M, N, Kb, false, eb);
  return (plan.tile == 14 || plan.tile == 36 || plan.tile == 56 || plan.tile == 58 || plan.tile == 61 || plan.tile == kSkinnyTile) &&
         plan.splits == 1;
}
template <int EB>
int swiglu_entry(const char* name, void* out, const void* a, const float* as, const void* w, const float* ws, int64_t M,
                 int64_t N, int64_t K, int out_dtype, void* stream) {
  LFM2_REQUIRE(out && a && w, "%s: a required pointer is null", name);
  LFM2_REQUIRE(out_dtype >= LFM2_DTYPE_BF16 && out_dtype <= LFM2_DTYPE_F32, "%s: bad output dtype", name);
  LFM2_REQUIRE(((uintptr_t)a | (uintptr_t)w | (uintptr_t)out) % 16 == 0, "%s: pointers must be aligned to 16 bytes", name);
  if (!swiglu_fits(M, N, K * EB, EB)) LFM2_FAIL(LFM2_ERR_UNSUPPORTED, "%s: no fused form for M %ld, N %ld, K %ld", name, (long)M, (long)N, (long)K);
  const int tile = default_plan(M, N, K * EB, false, EB).tile;
  if (tile == kSkinnyTile) {
    launch_skinny<2>(out, (const uint8_t*)a, (const uint8_t*)w, as, ws, M, N, K * EB, 1, out_dtype,
                     RowMap{nullptr, nullptr, 0x7fffffff}, (hipStream_t)stream);
    LFM2_LAUNCH_CHECK();
  }
  const int tiles = (int)(((M + kTiles[tile].bm - 1) / kTiles[tile].bm) * ((N + kTiles[tile].bn - 1) / kTiles[tile].bn));
  const dim3 grid((tiles + 7) / 8 * 8);
  if (tile == 14)
    hipLaunchKernelGGL((gemm_swiglu_kernel<EB, 128, 128, 2, 4, 2>), grid, dim3(512), 0, (hipStream_t)stream, out,
                       (const uint8_t*)a, (const uint8_t*)w, as, ws, (int)M, (int)N, K * EB, out_dtype);
  else if (tile == 56)
    hipLaunchKernelGGL((gemm_swiglu_kernel<EB, 256, 128, 4, 4, 3>), grid, dim3(1024), 0, (hipStream_t)stream, out,
                       (const uint8_t*)a, (const uint8_t*)w, as, ws, (int)M, (int)N, K * EB, out_dtype);
  else if (tile == 58)
    hipLaunchKernelGGL((gemm_swiglu_kernel<EB, 256, 256, 4, 4, 2>), grid, dim3(1024), 0, (hipStream_t)stream, out,
                       (const uint8_t*)a, (const uint8_t*)w, as, ws, (int)M, (int)N, K * EB, out_dtype);
  else if (tile == 61)
    hipLaunchKernelGGL((gemm_swiglu_kernel<EB, 256, 192, 4, 4, 2>), grid, dim3(1024), 0, (hipStream_t)stream, out,
                       (const uint8_t*)a, (const uint8_t*)w, as, ws, (int)M, (int)N, K * EB, out_dtype);
  else
    hipLaunchKernelGGL((gemm_swiglu_kernel<EB, 128, 96, 8, 2, 3>), grid, dim3(1024), 0, (hipStream_t)stream, out,
                       (const uint8_t*)a, (const uint8_t*)w, as, ws, (int)M, (int)N, K * EB, out_dtype);
  LFM2_LAUNCH_CHECK();
}
}  // namespace

namespace {
bool conv_fits(int64_t M, int64_t N, int64_t Kb) {
  if (M <= 0 || N <= 0 || Kb <= 0 || N % 48 != 0 || Kb % kStepBytes != 0 || M >= (1 << 30) || N >= (1 << 30)) return false;
  const Plan plan = default_plan(M, N, Kb);
  return plan.tile == 37 && plan.splits == 1;
}
template <int EB>
int conv_entry(const char* name, void* out, const void* a, const float* as, const void* w, const float* ws,
               const void* conv_weight, void* state, const uint8_t* active, const int32_t* slot_ids, int64_t M, int64_t N,
               int64_t K, int64_t slots, int out_dtype, void* stream) {
  LFM2_REQUIRE(out && a && w && conv_weight && state, "%s: a required pointer is null", name);
  LFM2_REQUIRE(out_dtype >= LFM2_DTYPE_BF16 && out_dtype <= LFM2_DTYPE_F32, "%s: bad output dtype", name);
  LFM2_REQUIRE(((uintptr_t)a | (uintptr_t)w) % 16 == 0, "%s: operands must be aligned to 16 bytes", name);
  LFM2_REQUIRE(slots > 0 && (slot_ids != nullptr || M <= slots), "%s: %ld rows but only %ld state slots", name, (long)M, (long)slots);
  if (!conv_fits(M, N, K * EB)) LFM2_FAIL(LFM2_ERR_UNSUPPORTED, "%s: no fused form for M %ld, N %ld, K %ld", name, (long)M, (long)N, (long)K);
  const int tiles = (int)(((M + 63) / 64) * (N / 96));
  hipLaunchKernelGGL(gemm_conv_kernel<EB>, dim3((tiles + 7) / 8 * 8), dim3(512), 0, (hipStream_t)stream, out,
                     (const uint8_t*)a, (const uint8_t*)w, as, ws, (int)M, (int)N, K * EB, out_dtype,
                     ConvEpilogue{conv_weight, state, active, slot_ids});
  LFM2_LAUNCH_CHECK();
}
}  // namespace

extern "C" int lfm2_gemm_conv_fits(int64_t M, int64_t N, int64_t K, int element_bytes) {
  return (element_bytes == 1 || element_bytes == 2) && conv_fits(M, N, K * element_bytes) ? 1 : 0;
}

extern "C" int lfm2_fp8_gemm_conv_update(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q,
                                         const float* w_scales, const void* conv_weight, void* state, const uint8_t* active,
                                         const int32_t* slot_ids, int64_t M, int64_t N, int64_t K, int64_t slots,
                                         int out_dtype, void* stream) {
  LFM2_REQUIRE(a_scales && w_scales, "fp8_gemm_conv_update: scales are required");
  return conv_entry<1>("fp8_gemm_conv_update", out, a_q, a_scales, w_q, w_scales, conv_weight, state, active, slot_ids, M, N,
                       K, slots, out_dtype, stream);
}

extern "C" int lfm2_bf16_gemm_conv_update(void* out, const void* x, const void* w, const void* conv_weight, void* state,
                                          const uint8_t* active, const int32_t* slot_ids, int64_t M, int64_t N, int64_t K,
                                          int64_t slots, void* stream) {
  return conv_entry<2>("bf16_gemm_conv_update", out, x, nullptr, w, nullptr, conv_weight, state, active, slot_ids, M, N, K,
                       slots, LFM2_DTYPE_BF16, stream);
}

extern "C" int lfm2_gemm_swiglu_fits(int64_t M, int64_t N, int64_t K, int element_bytes) {
  return (element_bytes == 1 || element_bytes == 2) && swiglu_fits(M, N, K * element_bytes, element_bytes) ? 1 : 0;
}

extern "C" int lfm2_fp8_gemm_swiglu(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q,
                                    const float* w_scales, int64_t M, int64_t N, int64_t K, int out_dtype, void* stream) {
  LFM2_REQUIRE(a_scales && w_scales, "fp8_gemm_swiglu: scales are required");
  return swiglu_entry<1>("fp8_gemm_swiglu", out, a_q, a_scales, w_q, w_scales, M, N, K, out_dtype, stream);
}

extern "C" int lfm2_bf16_gemm_swiglu(void* out, const void* x, const void* w, int64_t M, int64_t N, int64_t K, void* stream) {
  return swiglu_entry<2>("bf16_gemm_swiglu", out, x, nullptr, w, nullptr, M, N, K, LFM2_DTYPE_BF16, stream);
}

extern "C" int lfm2_fp8_gemm_qkv_store(void* q, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q,
                                        const float* w_scales, const void* q_weight, const void* k_weight, const float* cos,
                                        const float* sin, const int32_t* positions, void* k_cache, void* v_cache,
                                        float* k_scales, float* v_scales, const uint8_t* active, const int32_t* slot_ids,
                                        int64_t M, int QH, int KH, int D, int64_t K, int64_t max_positions, float eps,
                                        int64_t c0, int64_t c1, int64_t c2, int kv_fp8, int dtype, void* stream) {
  LFM2_REQUIRE(M > 0 && QH > 0 && KH > 0 && K > 0, "fp8_gemm_qkv_store: empty shape");
  LFM2_REQUIRE(M < (1 << 30), "fp8_gemm_qkv_store: too many rows");
  LFM2_REQUIRE(D == 64 && dtype == LFM2_DTYPE_BF16 && K % 128 == 0,
               "fp8_gemm_qkv_store: needs head_dim 64, bf16 and K a multiple of 128 (got %d, dtype %d, %ld)", D, dtype, (long)K);
  LFM2_REQUIRE(q && a_q && a_scales && w_q && w_scales && q_weight && k_weight && cos && sin && positions && k_cache && v_cache,
               "fp8_gemm_qkv_store: a required pointer is null");
  LFM2_REQUIRE(!kv_fp8 || (k_scales && v_scales), "fp8_gemm_qkv_store: e4m3 cache without scale tensors");
  LFM2_REQUIRE(max_positions > 0, "fp8_gemm_qkv_store: empty rotary table");
  LFM2_REQUIRE(c0 % 16 == 0 && c1 % 16 == 0 && c2 % 16 == 0, "fp8_gemm_qkv_store: cache strides must be multiples of 16 elements");
  LFM2_REQUIRE((((uintptr_t)q | (uintptr_t)a_q | (uintptr_t)w_q | (uintptr_t)q_weight | (uintptr_t)k_weight | (uintptr_t)cos |
                 (uintptr_t)sin | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0, "fp8_gemm_qkv_store: pointers must be 16-byte aligned");
  const QkvEpilogue epi{q, q_weight, k_weight, cos, sin, positions, slot_ids, active, k_cache, v_cache,
                        kv_fp8 ? k_scales : nullptr, kv_fp8 ? v_scales : nullptr, max_positions, c0, c1, c2, QH, KH, eps};
  const int N = (QH + 2 * KH) * 64;
  hipStream_t s = (hipStream_t)stream;
  // the 64 x 64 tile the plain product would take for the shape, else the ring of four
  const int tile = default_plan(M, N, K).tile;
  if (tile == 13) launch_qkv<3>(a_q, w_q, a_scales, w_scales, (int)M, N, K, epi, s);
  else launch_qkv<4>(a_q, w_q, a_scales, w_scales, (int)M, N, K, epi, s);
  LFM2_LAUNCH_CHECK();
}

extern "C" int lfm2_fp8_gemm_partials(float* partials, const uint8_t* a_q, const uint8_t* w_q, int64_t M, int64_t N,
                                      int64_t K, int tile, int split_k, void* stream) {
  LFM2_REQUIRE(split_k >= 1 && split_k <= 16, "fp8_gemm_partials: split_k %d not in [1,16]", split_k);
  LFM2_REQUIRE(tile < kNumTiles, "fp8_gemm_partials: tile index %d out of range", tile);
  const int64_t steps = tile_steps(tile >= 0 ? tile : default_plan(M, N, K, true, 1).tile, K);
  LFM2_REQUIRE(split_k <= steps && (steps + split_k - 1) / split_k * (split_k - 1) < steps,
               "fp8_gemm_partials: %d splits leave one without a K step", split_k);
  return gemm_entry<1>("fp8_gemm_partials", nullptr, a_q, nullptr, w_q, nullptr, partials, M, N, K, LFM2_DTYPE_F32, tile,
                       split_k, stream, false);
}

extern "C" int64_t lfm2_fp8_gemm_default_splits(int64_t M, int64_t N, int64_t K) {
  return K % 16 == 0 ? default_plan(M, N, K, true, 1).splits : 1;
}

extern "C" int64_t lfm2_fp8_gemm_workspace(int64_t M, int64_t N, int64_t K) {
  const Plan p = default_plan(M, N, K, false, 1);
  return (K % 16 == 0 && p.splits > 1) ? (int64_t)p.splits * M * N : 0;
}

extern "C" int lfm2_bf16_gemm(void* out, const void* x, const void* w, float* workspace, int64_t M, int64_t N, int64_t K,
                              int tile, int split_k, void* stream) {
  LFM2_REQUIRE(split_k <= 16, "bf16_gemm: split_k above 16");
  return gemm_entry<2>("bf16_gemm", out, x, nullptr, w, nullptr, workspace, M, N, K, LFM2_DTYPE_BF16, tile, split_k, stream);
}

extern "C" int lfm2_fp8_gemm_rows(void* out, const uint8_t* a_q, const float* a_scales, const uint8_t* w_q,
                                  const float* w_scales, const int32_t* out_rows, const uint8_t* row_active,
                                  int64_t out_capacity, int64_t M, int64_t N, int64_t K, int out_dtype, int tile,
                                  void* stream) {
  LFM2_REQUIRE(a_scales && w_scales, "fp8_gemm_rows: scales are required");
  LFM2_REQUIRE(out_capacity > 0 && out_capacity < (1ll << 31), "fp8_gemm_rows: bad output capacity");
  LFM2_REQUIRE(out_rows || M <= out_capacity, "fp8_gemm_rows: more rows than the output holds");
  return gemm_entry<1>("fp8_gemm_rows", out, a_q, a_scales, w_q, w_scales, nullptr, M, N, K, out_dtype, tile, 1, stream, true,
                       RowMap{out_rows, row_active, (int)out_capacity});
}

extern "C" int lfm2_bf16_gemm_rows(void* out, const void* x, const void* w, const int32_t* out_rows,
                                   const uint8_t* row_active, int64_t out_capacity, int64_t M, int64_t N, int64_t K, int tile,
                                   void* stream) {
  LFM2_REQUIRE(out_capacity > 0 && out_capacity < (1ll << 31), "bf16_gemm_rows: bad output capacity");
  LFM2_REQUIRE(out_rows || M <= out_capacity, "bf16_gemm_rows: more rows than the output holds");
  return gemm_entry<2>("bf16_gemm_rows", out, x, nullptr, w, nullptr, nullptr, M, N, K, LFM2_DTYPE_BF16, tile, 1, stream, true,
                       RowMap{out_rows, row_active, (int)out_capacity});
}

extern "C" int lfm2_bf16_gemm_partials(float* partials, const void* x, const void* w, int64_t M, int64_t N, int64_t K,
                                       int tile, int split_k, void* stream) {
  LFM2_REQUIRE(split_k >= 1 && split_k <= 16, "bf16_gemm_partials: split_k %d not in [1,16]", split_k);
  LFM2_REQUIRE(tile < kNumTiles, "bf16_gemm_partials: tile index %d out of range", tile);
  const int64_t steps = tile_steps(tile >= 0 ? tile : default_plan(M, N, K * 2, true).tile, K * 2);
  LFM2_REQUIRE(split_k <= steps && (steps + split_k - 1) / split_k * (split_k - 1) < steps,
               "bf16_gemm_partials: %d splits leave one without a K step", split_k);
  return gemm_entry<2>("bf16_gemm_partials", nullptr, x, nullptr, w, nullptr, partials, M, N, K, LFM2_DTYPE_F32, tile, split_k,
                       stream, false);
}

extern "C" int64_t lfm2_bf16_gemm_default_splits(int64_t M, int64_t N, int64_t K) {
  return (K * 2) % 16 == 0 ? default_plan(M, N, K * 2, true).splits : 1;
}

extern "C" int64_t lfm2_bf16_gemm_workspace(int64_t M, int64_t N, int64_t K) {
  const Plan p = default_plan(M, N, K * 2);
  return ((K * 2) % 16 == 0 && p.splits > 1) ? (int64_t)p.splits * M * N : 0;
}

// ------------------------------------------------------------------------------------ MFMA peak probe
// What the matrix units deliver when nothing else is in the way: every wave issues `iterations` rounds of eight
// independent v_mfma_f32_16x16x128_f8f6f4 (e4m3 operands held in registers, eight accumulators, so no instruction
// waits for the one before it).  No memory traffic inside the loop; the accumulators are folded into one store per
// lane at the end so the loop cannot be dropped.  The measured peak that the prefill products' MFMA utilisation is
// held against next to the nominal 5.0 PFLOP/s.  Also stores the core clock cycles and the 100 MHz wall clock ticks
// the loop took in the first wave of each workgroup (clock[2 * workgroup], clock[2 * workgroup + 1]): the clock the
// matrix units run at under this load.
namespace {
template <int WAVES>
__global__ void __launch_bounds__(WAVES * 64)
mfma_fp8_peak_kernel(float* __restrict__ sink, int64_t* __restrict__ clock, int iterations) {
  typedef StepMfma<1>::frag frag;
  const int lane = threadIdx.x & 63;
  frag a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {   // e4m3 codes of small finite values (exponent field 6 or 7): no infinities, no NaNs
    a[e] = 0x30303030 + 0x01010101 * ((lane + e) & 7);
    b[e] = 0x38383838 + 0x01010101 * ((lane * 3 + e) & 7);
  }
  f32x4 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int64_t c0 = (int64_t)clock64(), w0 = (int64_t)wall_clock64();
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = StepMfma<1>::run(a, b, acc[i]);
  }
  const int64_t c1 = (int64_t)clock64(), w1 = (int64_t)wall_clock64();
  f32x4 total = acc[0];
#pragma unroll
  for (int i = 1; i < 8; ++i) total += acc[i];
  sink[(int64_t)blockIdx.x * (WAVES * 64) + threadIdx.x] = total[0] + total[1] + total[2] + total[3];
  if (threadIdx.x == 0 && clock) { clock[2 * blockIdx.x] = c1 - c0; clock[2 * blockIdx.x + 1] = w1 - w0; }
}
}  // namespace

extern "C" int lfm2_mfma_fp8_peak(float* sink, int64_t* clock, int workgroups, int waves, int iterations, void* stream) {
  LFM2_REQUIRE(sink != nullptr, "mfma_fp8_peak: null sink");
  LFM2_REQUIRE(workgroups > 0 && workgroups <= 65536, "mfma_fp8_peak: workgroups %d not in [1, 65536]", workgroups);
  LFM2_REQUIRE(waves == 4 || waves == 8 || waves == 16, "mfma_fp8_peak: %d waves per workgroup, not 4, 8 or 16", waves);
  LFM2_REQUIRE(iterations > 0 && iterations <= (1 << 24), "mfma_fp8_peak: iterations %d not in [1, 2^24]", iterations);
  hipStream_t s = (hipStream_t)stream;
  if (waves == 4) hipLaunchKernelGGL(mfma_fp8_peak_kernel<4>, dim3(workgroups), dim3(256), 0, s, sink, clock, iterations);
  else if (waves == 8) hipLaunchKernelGGL(mfma_fp8_peak_kernel<8>, dim3(workgroups), dim3(512), 0, s, sink, clock, iterations);
  else hipLaunchKernelGGL(mfma_fp8_peak_kernel<16>, dim3(workgroups), dim3(1024), 0, s, sink, clock, iterations);
  LFM2_LAUNCH_CHECK();
}
