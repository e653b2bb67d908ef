// Token log-prob + entropy straight from the hidden states: the lm_head GEMM with the
// log-softmax statistics reduced in its epilogue, so the [rows, V] logits are never written.
//
// Replaces the forward of a replay chunk (unirl/models/qwen3/ar.py:82-99):
//   lf   = lm_head(h).float() / T          bf16 Linear: fp32 accumulation, result rounded to bf16
//   logp = lf[tok] - logsumexp(lf)
// for a bf16 head W [V, K] (nn.Linear's layout, K contiguous) and bf16 hidden states H [rows, K]
// (K contiguous): both operands are read along K, the layout MFMA fragments want.
//
// Kernel 1 (lmhead_tile_kernel): one workgroup of four wavefronts (2 x 2) per tile of the logits,
// 256 x 256 from 256 rows (one workgroup per compute unit, accumulators in AGPRs), 128 x 128 below
// (two per compute unit).  K is walked in steps of 64 through two LDS stages; each wavefront owns
// a quarter of the tile as blocks of v_mfma_f32_32x32x16_bf16, its fragments double-buffered in
// registers, and every memory instruction is issued between the step's MFMAs.  The operands reach
// LDS in one of two ways: from 512 rows straight from global memory (buffer loads with the LDS
// as destination, unpadded rows, bank conflicts avoided by an XOR swizzle applied on the global
// side), half a step's loads under the step's first slice and half under the previous step's
// last; below, through two register sets, loads two steps ahead and stores to LDS one step
// ahead.  Epilogue: accumulators (+ bias) are rounded to bf16 -- the values the reference's
// logits hold -- and passed through LDS transposed, so that a thread owns four rows over a part
// of the tile's columns; it reduces them to (m, s, t) per row: the maximum, sum 2^a and sum
// 2^a * a with a = (x - m) * log2(e)/T, and the parts of a row are merged.  One (m, s, t) per (row,
// column tile) goes to scratch memory (16 bytes for 256 or 512 bytes of logits) and the tile that
// holds a row's target column also stores that logit.
// Kernel 2 (lmhead_merge_kernel): one wavefront per row merges the row's tile states in fp64 and
// finishes logsumexp, log-prob and entropy.
//
// Tiles are dealt to the workgroups so that each XCD (workgroup id modulo 8) walks its own
// contiguous range of column groups, row block by row block: the group's slice of W stays in
// that XCD's L2 while the hidden states stream past it.

#include <type_traits>

#include "common_hip.h"
#include "unirl_internal.h"

namespace unirl {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int kHdThreads = 256;
constexpr int kBK = 64;
// LDS rows are padded by 16 bytes: the 16-byte fragment reads of 16 consecutive rows then
// cover all 64 banks exactly once
constexpr int kLdsRow = kBK + 8;  // bf16 elements per operand row
constexpr int kXcds = 8;
constexpr double kHdLn2 = 0.6931471805599453;

struct HeadArgs {
  const uint16_t* h;
  const uint16_t* w;
  const uint16_t* bias;
  const int64_t* ids;
  int64_t M, N, K, ldh, ldw;
  float c;  // log2(e) / T
  float4* state;  // [M][n_tiles]: (m, s, t, -)
  float* xid;     // [M]: the target's logit, written by the tile that holds its column
  uint16_t* logits_out;
  int64_t ld_logits;
  int n_tiles, m_blocks, group;
  float* logp;
  float* ent;
  float* lse;
  UNIRL_TRACE_FIELD
};

// Tile of workgroup `wg`: every XCD takes a contiguous range of the sequence
//   for column group g: for row block mb: for column tile n of the group: (mb, g*group + n)
__device__ __forceinline__ void head_tile_of(const HeadArgs& A, unsigned int wg, int& mb, int& nt) {
  const long long total = (long long)A.m_blocks * A.n_tiles;
  const long long per_xcd = (total + kXcds - 1) / kXcds;
  const long long pos = (long long)(wg % kXcds) * per_xcd + wg / kXcds;
  if (pos >= total) {
    mb = -1;
    nt = -1;
    return;
  }
  const long long per_group = (long long)A.m_blocks * A.group;
  const long long g = pos / per_group;
  // the last group may hold fewer column tiles
  const int g_cols = (int)((g + 1) * A.group <= A.n_tiles ? A.group : A.n_tiles - g * A.group);
  const long long in_group = pos - g * per_group;
  mb = (int)(in_group / g_cols);
  nt = (int)(g * A.group + in_group % g_cols);
}

__device__ __forceinline__ bf16x8_t lds_frag(const uint16_t* p) {
  return *reinterpret_cast<const bf16x8_t*>(p);
}

// Scheduling pattern of one slice of NM matrix instructions: before the m-th of them go its share
// of the slice's NR LDS reads, NW LDS writes and NL global loads.
template <int MASK, int N>
__device__ __forceinline__ void sched_group() {
  if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
}
template <int NM, int NR, int NW, int NL, int M = 0>
__device__ __forceinline__ void sched_slice() {
  if constexpr (M < NM) {
    sched_group<0x100, (M + 1) * NR / NM - M * NR / NM>();  // LDS reads
    sched_group<0x020, (M + 1) * NL / NM - M * NL / NM>();  // global loads
    sched_group<0x200, (M + 1) * NW / NM - M * NW / NM>();  // LDS writes
    sched_group<0x008, 1>();                                // one MFMA
    sched_slice<NM, NR, NW, NL, M + 1>();
  }
}

// BM x BN: the workgroup's tile of the logits; its four wavefronts sit 2 x 2, each on a
// (BM/2) x (BN/2) quarter of BI x BJ MFMA blocks.
template <int BM, int BN, bool HAS_BIAS, bool WRITE_LOGITS, bool DMA = false>
__global__ __launch_bounds__(kHdThreads, (BM * BN > 128 * 128) ? 1 : 2) void lmhead_tile_kernel(HeadArgs A) {
  constexpr int WM = BM / 2, WN = BN / 2, BI = WM / 32, BJ = WN / 32;
  constexpr int kAElems = BM * kLdsRow, kBElems = BN * kLdsRow, kStage = kAElems + kBElems;
  constexpr int CA = BM * 8 / kHdThreads, CB = BN * 8 / kHdThreads;  // 16-byte chunks per thread and step
  // epilogue: the tile's bf16 logits transposed, [BN][kOutPitch]; the pitch (BM * 2 + 8 bytes, 2 mod 32
  // words) spreads the 8-byte stores of 32 lanes on 32 columns over all banks
  constexpr int kOutPitch = BM + 4;
  static_assert(BN * kOutPitch * 2 + (kHdThreads / (BM / 4)) * BM * 12 <= 2 * kStage * 2,
                "the epilogue tile and the partial states reuse the operand stages");
  __shared__ __attribute__((aligned(16))) uint16_t lds[2 * kStage];  // [stage][A rows | B rows][kLdsRow]
  UNIRL_TRACE_T0();
#ifdef UNIRL_TRACE
  const long long trace_c0_ = clock64();  // shader clock: with the 100 MHz marks it gives the clock rate under load
#endif
  int mb, nt;
  head_tile_of(A, blockIdx.x, mb, nt);
  if (mb < 0) return;  // the padding of the last XCD's range (whole workgroup)
  const int64_t m0 = (int64_t)mb * BM, n0 = (int64_t)nt * BN;
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> LDS assignment: 16-byte chunk c = tid + 256*i covers row c/8, k-chunk c%8 of a tile.
  // The operands are read through buffer descriptors based at the tile's first row: a lane keeps
  // one 32-bit offset per operand (row and k-chunk; the K step travels in the scalar offset), and
  // rows past the end of the matrix fall outside the descriptor's range and read as zeros.
  const int kc = tid & 7, row0 = tid >> 3;
  auto tile_rsrc = [](const uint16_t* base, int64_t rows_left, int64_t ld, int64_t K) {
    const int64_t bytes = rows_left > 0 ? ((rows_left - 1) * ld + K) * 2 : 0;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(base), 0,
                                             bytes > 0xffffffffLL ? (int)0xffffffffu : (int)(uint32_t)bytes, 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t ra = tile_rsrc(A.h + m0 * A.ldh, A.M - m0, A.ldh, A.K);
  const __amdgpu_buffer_rsrc_t rb = tile_rsrc(A.w + n0 * A.ldw, A.N - n0, A.ldw, A.K);
  const int va0 = (int)((row0 * A.ldh + kc * 8) * 2), vb0 = (int)((row0 * A.ldw + kc * 8) * 2);
  const int va_step = (int)(32 * A.ldh * 2), vb_step = (int)(32 * A.ldw * 2);  // chunk i sits 32 rows further down
  const int lds_off0 = row0 * kLdsRow + kc * 8;
  // DMA: global -> LDS without registers.  One instruction of a wavefront fills 1 KB of LDS, lane by
  // lane: 8 operand rows of 128 bytes, unpadded.  Bank conflicts are avoided by an XOR swizzle on
  // the global side: the lane that fills slot (row r, chunk c) fetches chunk c ^ (r % 8).  Stage =
  // [BM + BN rows][64]; instruction i = 4 j + wave covers rows 8 i .. 8 i + 7 of (hidden rows, weight rows).
  constexpr int kStageD = (BM + BN) * kBK;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int dr = lane >> 3, dc = (lane & 7) ^ (lane >> 3);
  const int da0 = (int)((((int64_t)wave_u * 8 + dr) * A.ldh + dc * 8) * 2);
  const int db0 = (int)((((int64_t)wave_u * 8 + dr) * A.ldw + dc * 8) * 2);
  auto dma_range = [&](int stage, int64_t k0, int j0, int j1) {
    const int sk = (int)(k0 * 2);
#pragma unroll
    for (int j = j0; j < j1; ++j) {
      auto* dst = (__attribute__((address_space(3))) void*)(lds + stage * kStageD + (j * 4 + wave_u) * 512);
      if (j < CA) __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, dst, 16, da0 + j * va_step, sk, 0, 0);
      else __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, dst, 16, db0 + (j - CA) * vb_step, sk, 0, 0);
    }
  };
  // Two register sets stage the operands of two K steps between global memory and LDS.  A step's
  // CA + CB loads go out a quarter under each 16-wide slice of the multiplication and, a step
  // later, its stores to LDS a third under each of the first three slices.
  constexpr int NW = CA + CB, NQ = NW / 4;
  static_assert(NW % 4 == 0, "a quarter of a step's chunks per slice");
  constexpr int W0 = (NW + 2) / 3, W1 = (NW - W0 + 1) / 2;  // stores under slices 0 and 1; the rest under slice 2
  u32x4 gs[2][NW];  // [set][chunk]: chunks 0 .. CA-1 of the hidden states, CA .. of the weight
  auto load_range = [&](int set, int64_t k0, int j0, int j1) {
    const int sk = (int)(k0 * 2);
#pragma unroll
    for (int j = j0; j < j1; ++j)
      gs[set][j] = (j < CA) ? __builtin_amdgcn_raw_buffer_load_b128(ra, va0 + j * va_step, sk, 0)
                            : __builtin_amdgcn_raw_buffer_load_b128(rb, vb0 + (j - CA) * vb_step, sk, 0);
  };
  auto store_range = [&](int set, int stage, int j0, int j1) {
    uint16_t* sa = lds + stage * kStage;
    uint16_t* sb = sa + kAElems;
#pragma unroll
    for (int j = j0; j < j1; ++j)
      *reinterpret_cast<u32x4*>((j < CA ? sa + j * 32 * kLdsRow : sb + (j - CA) * 32 * kLdsRow) + lds_off0) = gs[set][j];
  };

  f32x16_t acc[BI][BJ];
#pragma unroll
  for (int bi = 0; bi < BI; ++bi)
#pragma unroll
    for (int bj = 0; bj < BJ; ++bj)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[bi][bj][i] = 0.0f;

  // fragment addresses inside a stage: lane l reads row (l % 32) of a 32-row block, k = 8 * (l / 32) ..
  const int frag_a = (wm * WM + (lane & 31)) * kLdsRow + 8 * (lane >> 5);
  const int frag_b = (wn * WN + (lane & 31)) * kLdsRow + 8 * (lane >> 5);
  bf16x8_t fa[2][BI], fb[2][BJ];  // the fragments of two consecutive 16-wide K slices
  // DMA layout: slot of (row, chunk kc) is chunk kc ^ (row % 8); row % 8 = lane % 8 for every block
  int fsw[kBK / 16];
#pragma unroll
  for (int ks = 0; ks < kBK / 16; ++ks) fsw[ks] = (lane & 31) * kBK + (((2 * ks + (lane >> 5)) ^ (lane & 7)) * 8);
  auto read_frags = [&](int stage, int ks, bf16x8_t(&a)[BI], bf16x8_t(&b)[BJ]) {
    if (DMA) {
      const uint16_t* sa = lds + stage * kStageD + (wm * WM) * kBK + fsw[ks];
      const uint16_t* sb = lds + stage * kStageD + (BM + wn * WN) * kBK + fsw[ks];
#pragma unroll
      for (int bi = 0; bi < BI; ++bi) a[bi] = lds_frag(sa + bi * 32 * kBK);
#pragma unroll
      for (int bj = 0; bj < BJ; ++bj) b[bj] = lds_frag(sb + bj * 32 * kBK);
      return;
    }
    const uint16_t* sa = lds + stage * kStage;
    const uint16_t* sb = sa + kAElems;
#pragma unroll
    for (int bi = 0; bi < BI; ++bi) a[bi] = lds_frag(sa + frag_a + bi * 32 * kLdsRow + ks * 16);
#pragma unroll
    for (int bj = 0; bj < BJ; ++bj) b[bj] = lds_frag(sb + frag_b + bj * 32 * kLdsRow + ks * 16);
  };
  // DMA mode, one fragment: index < BI of the hidden-state blocks, else of the weight blocks
  auto read_one = [&](int stage, int ks, int idx, bf16x8_t(&a)[BI], bf16x8_t(&b)[BJ]) {
    if (idx < BI) a[idx] = lds_frag(lds + stage * kStageD + (wm * WM + idx * 32) * kBK + fsw[ks]);
    else b[idx - BI] = lds_frag(lds + stage * kStageD + (BM + wn * WN + (idx - BI) * 32) * kBK + fsw[ks]);
  };
  constexpr int NR = BI + BJ, NM = BI * BJ;  // LDS reads and MFMAs per K slice
  // One K step out of LDS stage `stage`, as four slices of NM matrix instructions, each with the
  // fragment reads of the next slice under it.  The next step's operands travel under them too.
  // Register-staged: the loads of step k + 2 go into register set `stage` (which held this step's
  // operands until they were stored a step ago), a quarter per slice, and the stores of step
  // k + 1's operands (register set stage ^ 1, loaded a step ago) into the other LDS stage, under
  // slices 0 - 2.  DMA: the other stage is free from the previous step's barrier to this step's;
  // half of step k + 1's loads into it went out under the previous step's last slice, the other
  // half goes out under this step's first slice.
  // The step's barrier stands before its LAST slice: by then every wavefront has read this
  // stage's last fragments and the other stage is complete (stores issued, or loads into LDS
  // waited for), so the last slice already reads the next step's first fragments and no slice
  // waits for LDS behind a barrier.  (What the next step writes goes to this stage, which nobody
  // reads any more.)
  // Every memory instruction is issued between matrix instructions: a wavefront issues in order,
  // and a burst of sixteen loads or stores holds up the MFMAs behind it for as long as the memory
  // pipeline takes to accept them (measured: the bursts cost 0.9 us of a 1.8 us step).  The
  // scheduling fences keep each slice's instructions together; inside a slice sched_slice deals
  // them out among the MFMAs.
#ifdef UNIRL_TRACE
  long long trace_bar_ = 0;  // shader cycles this wavefront spent waiting at the step barriers
#define UNIRL_HEAD_STEP_BARRIER()              \
  do {                                         \
    const long long b0_ = clock64();           \
    __syncthreads();                           \
    trace_bar_ += clock64() - b0_;             \
  } while (0)
#else
#define UNIRL_HEAD_STEP_BARRIER() __syncthreads()
#endif
  // (With two workgroups on a compute unit -- the 128 x 128 tile -- the other workgroup fills such
  // waits, and the plain arrangement measures faster: barrier at the end of the step, the stores a
  // quarter under each slice, the step's first fragments read after the barrier.)
  constexpr bool kEarlyBarrier = DMA || BM * BN > 128 * 128;
  auto multiply = [&](int stage, int64_t k_load, int64_t k_load2) {
    if (!kEarlyBarrier) read_frags(stage, 0, fa[0], fb[0]);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      const int cur = ks & 1;
      if (DMA) {
        // the other stage is free from the previous step's barrier to this step's: the second half
        // of step k + 1 goes into it now, the first half went under the previous step's last slice;
        // after this step's barrier this stage is free and takes the first half of step k + 2.
        // Loads into LDS and reads of LDS keep their program order, so they alternate here.
        static_assert(NW / 2 <= NR, "at most one load per fragment read");
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          if (ks + 1 < kBK / 16) read_one(stage, ks + 1, i, fa[cur ^ 1], fb[cur ^ 1]);
          else read_one(stage ^ 1, 0, i, fa[cur ^ 1], fb[cur ^ 1]);
          if (ks == 0 && i < NW / 2) dma_range(stage ^ 1, k_load, NW / 2 + i, NW / 2 + i + 1);
          if (ks == 3 && i < NW / 2) dma_range(stage, k_load2, i, i + 1);
        }
      } else {
        if (ks + 1 < kBK / 16) read_frags(stage, ks + 1, fa[cur ^ 1], fb[cur ^ 1]);
        else if (kEarlyBarrier) read_frags(stage ^ 1, 0, fa[cur ^ 1], fb[cur ^ 1]);  // the next step's first slice
        load_range(stage, k_load, ks * NQ, (ks + 1) * NQ);
      }
      if (!DMA && kEarlyBarrier) {
        if (ks == 0) store_range(stage ^ 1, stage ^ 1, 0, W0);
        if (ks == 1) store_range(stage ^ 1, stage ^ 1, W0, W0 + W1);
        if (ks == 2) store_range(stage ^ 1, stage ^ 1, W0 + W1, NW);
      } else if (!DMA) {
        store_range(stage ^ 1, stage ^ 1, ks * NQ, (ks + 1) * NQ);
      }
#pragma unroll
      for (int bi = 0; bi < BI; ++bi)
#pragma unroll
        for (int bj = 0; bj < BJ; ++bj)
          acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][bi], fb[cur][bj], acc[bi][bj], 0, 0, 0);
      if (DMA) {
        if (ks == 0 || ks == 3) sched_slice<NM, NR, 0, NW / 2>();
        else sched_slice<NM, NR, 0, 0>();
      } else if (kEarlyBarrier) {
        if (ks == 0) sched_slice<NM, NR, W0, NQ>();
        if (ks == 1) sched_slice<NM, NR, W1, NQ>();
        if (ks == 2) sched_slice<NM, NR, NW - W0 - W1, NQ>();
        if (ks == 3) sched_slice<NM, NR, 0, NQ>();
      } else {
        if (ks + 1 < kBK / 16) sched_slice<NM, NR, NQ, NQ>();
        else sched_slice<NM, 0, NQ, NQ>();
      }
      __builtin_amdgcn_sched_barrier(0);
      if (ks == (kEarlyBarrier ? 2 : 3)) UNIRL_HEAD_STEP_BARRIER();
    }
  };

  // Step k sits in LDS stage k % 2 (and came through register set k % 2).  Every trip issues its
  // loads and stores unconditionally (past the last step the loads repeat the last step's
  // addresses and the stores fill a stage nobody multiplies any more): with a branch around them
  // the compiler can no longer count which loads are outstanding at the stores and waits for all
  // of them.
  const int nk = (int)(A.K / kBK);
  const int64_t k_last = (int64_t)(nk - 1) * kBK;
  auto k_of = [&](int step) { return step < nk ? (int64_t)step * kBK : k_last; };
  if (DMA) {
    dma_range(0, 0, 0, NW);
    __syncthreads();
    dma_range(1, k_of(1), 0, NW / 2);
  } else {
    load_range(0, 0, 0, NW);
    load_range(1, k_of(1), 0, NW);
    store_range(0, 0, 0, NW);
    __syncthreads();
  }
  if (kEarlyBarrier) read_frags(0, 0, fa[0], fb[0]);
  int kt = 0;
  for (; kt + 1 < nk; kt += 2) {
    multiply(0, DMA ? k_of(kt + 1) : k_of(kt + 2), k_of(kt + 2));
    multiply(1, DMA ? k_of(kt + 2) : k_of(kt + 3), k_of(kt + 3));
  }
  if (kt < nk) multiply(0, k_last, k_last);  // an odd number of steps: the last one sits in stage 0
#undef UNIRL_HEAD_STEP_BARRIER
  if (kEarlyBarrier) __syncthreads();  // the last slice's reads of the other stage are done before the epilogue writes over it
  UNIRL_TRACE_MARK1();
#ifdef UNIRL_TRACE
  // slot 2 of the record: shader cycles of the K loop (low half) and of its barrier waits (high half)
  trace_m2_ = ((unsigned long long)(clock64() - trace_c0_) & 0xffffffffull) | ((unsigned long long)trace_bar_ << 32);
#endif

  // ---- epilogue ----
  // The tile's logits -- accumulators (+ bias) rounded to bf16, the values the reference's logits
  // hold -- go through LDS transposed, tile column by tile column: a lane's four consecutive
  // accumulators are four consecutive rows of one column, 8 bytes.  Then thread (row quad q,
  // column part cq) reduces rows 4q .. 4q+3 over the COLS columns of its part: one 8-byte read
  // per column, consecutive lanes on consecutive row quads (one contiguous run of LDS per
  // wavefront read).  Per logit: unpack, max, fma, exp2, add, fma.
  uint16_t* out = lds;  // [BN][kOutPitch] bf16; the operand stages are free now
#pragma unroll
  for (int bj = 0; bj < BJ; ++bj) {
    const int col = wn * WN + bj * 32 + (lane & 31);
    float bv = 0.0f;
    if (HAS_BIAS) {
      const int64_t gc = n0 + col;
      bv = bf16_bits_to_f32(A.bias[gc < A.N ? gc : A.N - 1]);
    }
#pragma unroll
    for (int bi = 0; bi < BI; ++bi) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const int row = wm * WM + bi * 32 + 8 * g4 + 4 * (lane >> 5);
        float f[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) f[k] = HAS_BIAS ? acc[bi][bj][g4 * 4 + k] + bv : acc[bi][bj][g4 * 4 + k];
        u32x2 pk;  // two values per conversion instruction
        pk.x = f32x2_to_bf16x2_bits(f[0], f[1]);
        pk.y = f32x2_to_bf16x2_bits(f[2], f[3]);
        *reinterpret_cast<u32x2*>(out + col * kOutPitch + row) = pk;
      }
    }
  }
  __syncthreads();

  constexpr int NQUAD = BM / 4;              // row quads of the tile
  constexpr int PARTS = kHdThreads / NQUAD;  // column parts (4 or 8)
  constexpr int COLS = BN / PARTS;           // columns of a part (64 or 16)
  constexpr int PIECE = 16;                  // columns between two updates of the running maxima
  static_assert(COLS % PIECE == 0, "whole pieces");
  const int q = tid % NQUAD, cq = tid / NQUAD;
  const float c = A.c;
  float m[4], sum[4], tsum[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m[r] = -INFINITY;
    sum[r] = 0.0f;
    tsum[r] = 0.0f;
  }
  const int64_t gcol0 = n0 + (int64_t)cq * COLS;  // this thread's first column in the vocabulary
  auto reduce_columns = [&](auto full_tag, auto ent_tag) {
    constexpr bool FULL = decltype(full_tag)::value;  // every column of the tile lies inside the vocabulary
    constexpr bool ENT = decltype(ent_tag)::value;    // the entropy is asked for: sum 2^a * a is needed
    const uint16_t* src = out + (cq * COLS) * kOutPitch + 4 * q;
#pragma unroll 1
    for (int p0 = 0; p0 < COLS; p0 += PIECE) {
      float x[4][PIECE];
#pragma unroll
      for (int j = 0; j < PIECE; ++j) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(src + (p0 + j) * kOutPitch);
        const bool ok = FULL || (gcol0 + p0 + j < A.N);
        x[0][j] = ok ? __uint_as_float(v.x << 16) : -INFINITY;
        x[1][j] = ok ? __uint_as_float(v.x & 0xffff0000u) : -INFINITY;
        x[2][j] = ok ? __uint_as_float(v.y << 16) : -INFINITY;
        x[3][j] = ok ? __uint_as_float(v.y & 0xffff0000u) : -INFINITY;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float pm = x[r][0];
#pragma unroll
        for (int j = 1; j < PIECE; ++j) pm = fmaxf(pm, x[r][j]);
        const float mn = fmaxf(m[r], pm);
        // raise the reference of what has been summed so far (nothing yet: the sums are zero)
        const float d = (mn - m[r]) * c;
        const float f = __builtin_amdgcn_exp2f(-d);
        const bool had = m[r] != -INFINITY;
        if (ENT) tsum[r] = had ? f * fmaf(-d, sum[r], tsum[r]) : 0.0f;
        sum[r] = had ? f * sum[r] : 0.0f;
        m[r] = mn;
        // nothing but -inf so far (columns outside the vocabulary, or masked entries: a -inf bias)
        if (mn == -INFINITY) continue;
        const float mc = -mn * c;
#pragma unroll
        for (int j = 0; j < PIECE; ++j) {
          // a = (x - m) * c <= 0.  A -inf logit (outside the vocabulary, or masked) has e = 0 and must
          // add 0 to the entropy sum, not 0 * -inf: the product is taken with a held at a large finite value
          const float a = fmaf(x[r][j], c, mc);
          const float e = __builtin_amdgcn_exp2f(a);
          sum[r] += e;
          if (ENT) tsum[r] = fmaf(e, fmaxf(a, -65536.0f), tsum[r]);
        }
      }
    }
  };
  if (A.ent) {
    if (n0 + BN <= A.N) reduce_columns(std::true_type{}, std::true_type{});
    else reduce_columns(std::false_type{}, std::true_type{});
  } else {
    if (n0 + BN <= A.N) reduce_columns(std::true_type{}, std::false_type{});
    else reduce_columns(std::false_type{}, std::false_type{});
  }

  // the PARTS partial states of a row meet in LDS above the logits; thread `row` merges them in part order
  float* part_state = reinterpret_cast<float*>(lds + BN * kOutPitch);  // [PARTS][BM][3]
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float* ps = part_state + ((size_t)cq * BM + 4 * q + r) * 3;
    ps[0] = m[r];
    ps[1] = sum[r];
    ps[2] = tsum[r];
  }
  __syncthreads();
  if (tid < BM) {
    const int row = tid;
    const int64_t grow = m0 + row;
    float M = -INFINITY, S = 0.0f, T = 0.0f;
#pragma unroll
    for (int p = 0; p < PARTS; ++p) {
      const float* ps = part_state + ((size_t)p * BM + row) * 3;
      const float pm = ps[0], psum = ps[1], pt = ps[2];
      if (pm == -INFINITY) continue;  // a part wholly outside the vocabulary
      if (M == -INFINITY) {
        M = pm;
        S = psum;
        T = pt;
        continue;
      }
      const float mm = fmaxf(M, pm);
      const float d0 = (mm - M) * c, f0 = __builtin_amdgcn_exp2f(-d0);
      const float d1 = (mm - pm) * c, f1 = __builtin_amdgcn_exp2f(-d1);
      T = f0 * fmaf(-d0, S, T) + f1 * fmaf(-d1, psum, pt);
      S = f0 * S + f1 * psum;
      M = (M != M || pm != pm) ? (M + pm) : mm;
    }
    if (grow < A.M) {
      A.state[grow * A.n_tiles + nt] = make_float4(M, S, T, 0.0f);
      if (A.ids) {  // the tile that holds the row's target column stores that logit
        const int64_t id = A.ids[grow];
        if (id >= n0 && id < n0 + BN && id < A.N) A.xid[grow] = bf16_bits_to_f32(out[(id - n0) * kOutPitch + row]);
      }
    }
  }
  if (WRITE_LOGITS) {  // validation: the tile's logits, row by row
    for (int idx = tid; idx < BM * BN; idx += kHdThreads) {
      const int row = idx / BN, col = idx % BN;
      const int64_t grow = m0 + row, gcol = n0 + col;
      if (grow < A.M && gcol < A.N) A.logits_out[grow * A.ld_logits + gcol] = out[col * kOutPitch + row];
    }
  }
  UNIRL_TRACE_END(A.trace);
}

struct HeadState {
  double m, s, t;
};

// (m, s, t) of the union of two column sets; sums are relative to their own maximum
__device__ __forceinline__ HeadState head_merge(const HeadState& p, const HeadState& q, double c) {
  if (q.m == -INFINITY) return p;
  if (p.m == -INFINITY) return q;
  const double M = p.m > q.m ? p.m : q.m;
  const double dp = (M - p.m) * c, dq = (M - q.m) * c;
  const double fp = exp2(-dp), fq = exp2(-dq);
  HeadState r;
  r.m = (p.m != p.m || q.m != q.m) ? (p.m + q.m) : M;
  r.s = fp * p.s + fq * q.s;
  r.t = fp * (p.t - dp * p.s) + fq * (q.t - dq * q.s);
  return r;
}

__device__ __forceinline__ double shfl_xor_f64(double v, int mask) {
  const long long b = __double_as_longlong(v);
  const unsigned int lo = (unsigned int)__shfl_xor((int)(unsigned int)b, mask, kWave);
  const unsigned int hi = (unsigned int)__shfl_xor((int)(unsigned int)((unsigned long long)b >> 32), mask, kWave);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// One wavefront per row: merge the row's tile states (index order per lane, then a butterfly)
// and finish the three outputs.
__global__ __launch_bounds__(kHdThreads) void lmhead_merge_kernel(HeadArgs A) {
  const int64_t row = (int64_t)blockIdx.x * (kHdThreads / kWave) + threadIdx.x / kWave;
  if (row >= A.M) return;
  const int lane = threadIdx.x & (kWave - 1);
  const double c = (double)A.c;
  const float4* st = A.state + row * A.n_tiles;
  HeadState acc{-(double)INFINITY, 0.0, 0.0};
  for (int j = lane; j < A.n_tiles; j += kWave) {
    const float4 v = st[j];
    acc = head_merge(acc, HeadState{(double)v.x, (double)v.y, (double)v.z}, c);
  }
#pragma unroll
  for (int mask = 1; mask < kWave; mask <<= 1) {
    HeadState o{shfl_xor_f64(acc.m, mask), shfl_xor_f64(acc.s, mask), shfl_xor_f64(acc.t, mask)};
    acc = head_merge(acc, o, c);
  }
  if (lane != 0) return;
  // ln sum = ln2 * (m*c + log2 s);  H = ln s - ln2 * t / s;  logp = ln2 * (x_id - m) * c - ln s
  const double ln_s = log(acc.s);
  const double lse = kHdLn2 * (acc.m * c) + ln_s;
  if (A.lse) A.lse[row] = (float)lse;
  if (A.ent) {
    const double h = ln_s - kHdLn2 * acc.t / acc.s;
    A.ent[row] = (float)(h < 0.0 ? 0.0 : h);
  }
  if (A.logp) {
    float out = quiet_nan();
    const int64_t id = A.ids[row];
    if (id >= 0 && id < A.N) out = (float)(kHdLn2 * (((double)A.xid[row] - acc.m) * c) - ln_s);
    A.logp[row] = out;
  }
}


// ---- transposed copy of a 2-D matrix of 2- or 4-byte elements --------------------------------
// dst[c][r] = src[r][c].  One workgroup per 64 x 64 tile: 16-byte loads along the source rows,
// the tile through LDS as 32-bit words (rows padded by one word so that a walk down a column
// meets every bank once), 16-byte stores along the destination rows; eight (2-byte elements) or
// sixteen (4-byte) neighbouring lanes write one whole 128- or 256-byte run of a destination row.
constexpr int kTrTile = 64;
constexpr int kTrThreads = 256;

struct TransposeArgs {
  const void* src;
  void* dst;
  int64_t rows, cols, ld_src, ld_dst;
  int vec_src, vec_dst;  // 16-byte accesses allowed on that side (alignment of base and leading dimension)
};

template <typename T>
__global__ __launch_bounds__(kTrThreads) void transpose_tile_kernel(TransposeArgs A) {
  constexpr int VE = 16 / (int)sizeof(T);          // elements per 16-byte vector
  constexpr int WPR = kTrTile * (int)sizeof(T) / 4;  // 32-bit words per tile row
  constexpr int TPR = kTrTile / VE;                // threads covering a tile row with one vector each
  constexpr int RPP = kTrThreads / TPR;            // tile rows per pass
  __shared__ uint32_t lds[kTrTile][WPR + 1];
  const T* src = reinterpret_cast<const T*>(A.src);
  T* dst = reinterpret_cast<T*>(A.dst);
  const int64_t r0 = (int64_t)blockIdx.y * kTrTile, c0 = (int64_t)blockIdx.x * kTrTile;
  const int tid = threadIdx.x;

  // load: thread (row tid / TPR, vector tid % TPR) of each pass
#pragma unroll
  for (int p = 0; p < kTrTile / RPP; ++p) {
    const int lr = p * RPP + tid / TPR, lv = tid % TPR;
    const int64_t r = r0 + lr, c = c0 + (int64_t)lv * VE;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (r < A.rows) {
      if (A.vec_src && c + VE <= A.cols) {
        v = *reinterpret_cast<const u32x4*>(src + r * A.ld_src + c);
      } else {
        T e[VE];
#pragma unroll
        for (int k = 0; k < VE; ++k) e[k] = (c + k < A.cols) ? src[r * A.ld_src + c + k] : (T)0;
        if (sizeof(T) == 2) {
          v.x = (uint32_t)e[0] | ((uint32_t)e[1 % VE] << 16);
          v.y = (uint32_t)e[2 % VE] | ((uint32_t)e[3 % VE] << 16);
          v.z = (uint32_t)e[4 % VE] | ((uint32_t)e[5 % VE] << 16);
          v.w = (uint32_t)e[6 % VE] | ((uint32_t)e[7 % VE] << 16);
        } else {
          v.x = (uint32_t)e[0];
          v.y = (uint32_t)e[1 % VE];
          v.z = (uint32_t)e[2 % VE];
          v.w = (uint32_t)e[3 % VE];
        }
      }
    }
    uint32_t* w = &lds[lr][lv * 4];
    w[0] = v.x;
    w[1] = v.y;
    w[2] = v.z;
    w[3] = v.w;
  }
  __syncthreads();

  if (sizeof(T) == 2) {
    // thread (source rows 8*rg .. +7, source column pair cp): two destination rows, 16 bytes each
    const int rg = tid % 8, cp = tid / 8;
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = lds[8 * rg + j][cp];
    u32x4 lo, hi;
    lo.x = (w[0] & 0xffffu) | (w[1] << 16);
    lo.y = (w[2] & 0xffffu) | (w[3] << 16);
    lo.z = (w[4] & 0xffffu) | (w[5] << 16);
    lo.w = (w[6] & 0xffffu) | (w[7] << 16);
    hi.x = (w[0] >> 16) | (w[1] & 0xffff0000u);
    hi.y = (w[2] >> 16) | (w[3] & 0xffff0000u);
    hi.z = (w[4] >> 16) | (w[5] & 0xffff0000u);
    hi.w = (w[6] >> 16) | (w[7] & 0xffff0000u);
    const int64_t dr = c0 + 2 * cp, dc = r0 + 8 * rg;  // destination row (= source column), first column
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const u32x4 v = e ? hi : lo;
      if (dr + e >= A.cols) continue;
      if (A.vec_dst && dc + 8 <= A.rows) {
        *reinterpret_cast<u32x4*>(dst + (dr + e) * A.ld_dst + dc) = v;
      } else {
        const uint32_t q[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (dc + k < A.rows) dst[(dr + e) * A.ld_dst + dc + k] = (T)((q[k / 2] >> (16 * (k % 2))) & 0xffffu);
      }
    }
  } else {
    // thread (source rows 4*rg .. +3, source column c) of each of four passes
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int rg = tid % 16, c = p * 16 + tid / 16;
      u32x4 v;
      v.x = lds[4 * rg + 0][c];
      v.y = lds[4 * rg + 1][c];
      v.z = lds[4 * rg + 2][c];
      v.w = lds[4 * rg + 3][c];
      const int64_t dr = c0 + c, dc = r0 + 4 * rg;
      if (dr >= A.cols) continue;
      if (A.vec_dst && dc + 4 <= A.rows) {
        *reinterpret_cast<u32x4*>(dst + dr * A.ld_dst + dc) = v;
      } else {
        const uint32_t q[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (dc + k < A.rows) dst[dr * A.ld_dst + dc + k] = (T)q[k];
      }
    }
  }
}

}  // namespace unirl

using namespace unirl;

// Tile edge of a call: 256 x 256 tiles (one workgroup per compute unit, the fewest LDS reads per
// MFMA) from 256 rows, 128 x 128 below (measured: 0.25 against 0.30 ms at 256 rows, 0.44 against
// 0.52 ms at 512).
static int head_tile_edge(int64_t rows) { return rows >= (int64_t)tune_int("UNIRL_HEAD_BIG_ROWS", 256) ? 256 : 128; }

extern "C" size_t unirl_lmhead_logp_scratch_bytes(int64_t rows, int64_t V) {
  if (rows <= 0 || V <= 0) return 0;
  const int64_t n_tiles = (V + 127) / 128;  // the finer of the two tilings
  return (size_t)rows * (size_t)n_tiles * sizeof(float4) + (size_t)rows * sizeof(float) + 256;
}

template <int EDGE, bool DMA>
static int launch_head_tiles(const HeadArgs& A, dim3 grid, hipStream_t st) {
  dim3 block(kHdThreads);
  if (A.bias) {
    if (A.logits_out)
      hipLaunchKernelGGL((lmhead_tile_kernel<EDGE, EDGE, true, true, DMA>), grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((lmhead_tile_kernel<EDGE, EDGE, true, false, DMA>), grid, block, 0, st, A);
  } else {
    if (A.logits_out)
      hipLaunchKernelGGL((lmhead_tile_kernel<EDGE, EDGE, false, true, DMA>), grid, block, 0, st, A);
    else
      hipLaunchKernelGGL((lmhead_tile_kernel<EDGE, EDGE, false, false, DMA>), grid, block, 0, st, A);
  }
  return (int)hipGetLastError();
}

extern "C" int unirl_lmhead_logp(const void* hidden, int64_t ld_hidden, const void* weight, int64_t ld_weight,
                                 const void* bias, int64_t rows, int64_t V, int64_t K, const int64_t* ids,
                                 float temperature, float* logp_out, float* ent_out, float* lse_out, void* logits_out,
                                 int64_t ld_logits, void* scratch, size_t scratch_bytes, void* stream) {
  if (rows < 0 || V <= 0 || K <= 0 || ld_hidden < K || ld_weight < K) return UNIRL_E_SHAPE;
  if (K % kBK != 0 || ld_hidden % 8 != 0 || ld_weight % 8 != 0) return UNIRL_E_SHAPE;  // whole 64-wide K steps, 16-byte rows
  if (ld_hidden > (1 << 22) || ld_weight > (1 << 22)) return UNIRL_E_LIMIT;  // 32-bit byte offsets inside a 256-row tile
  if (logits_out && ld_logits < V) return UNIRL_E_SHAPE;
  if (rows == 0) return UNIRL_OK;
  if (!hidden || !weight || !scratch) return UNIRL_E_NULL;
  if (logp_out && !ids) return UNIRL_E_NULL;
  if (!aligned_to(hidden, 16) || !aligned_to(weight, 16) || !aligned_to(bias, 2) || !aligned_to(logits_out, 2) ||
      !aligned_to(scratch, 16) || !aligned_to(ids, 8) || !aligned_to(logp_out, 4) || !aligned_to(ent_out, 4) ||
      !aligned_to(lse_out, 4))
    return UNIRL_E_ALIGN;
  if (scratch_bytes < unirl_lmhead_logp_scratch_bytes(rows, V)) return UNIRL_E_WORKSPACE;
  const int edge = head_tile_edge(rows);
  const int64_t n_tiles = (V + edge - 1) / edge, m_blocks = (rows + edge - 1) / edge;
  if (n_tiles > 0x7fffffff || m_blocks > 0x7fffffff) return UNIRL_E_LIMIT;
  const long long total = (long long)n_tiles * m_blocks;
  const long long per_xcd = (total + kXcds - 1) / kXcds;
  if (per_xcd * kXcds > 0x7fffffffLL) return UNIRL_E_LIMIT;
  HeadArgs A = {};
  A.h = reinterpret_cast<const uint16_t*>(hidden);
  A.w = reinterpret_cast<const uint16_t*>(weight);
  A.bias = reinterpret_cast<const uint16_t*>(bias);
  A.ids = ids;
  A.M = rows;
  A.N = V;
  A.K = K;
  A.ldh = ld_hidden;
  A.ldw = ld_weight;
  const float T = temperature > 0.0f ? temperature : 1.0f;
  A.c = (float)(1.4426950408889634 / (double)T);
  A.state = reinterpret_cast<float4*>(scratch);
  A.xid = reinterpret_cast<float*>(reinterpret_cast<char*>(scratch) + (size_t)rows * (size_t)n_tiles * sizeof(float4));
  A.logits_out = reinterpret_cast<uint16_t*>(logits_out);
  A.ld_logits = ld_logits;
  A.n_tiles = (int)n_tiles;
  A.m_blocks = (int)m_blocks;
  A.group = (int)tune_int("UNIRL_HEAD_GROUP", 8);
  A.logp = logp_out;
  A.ent = ent_out;
  A.lse = lse_out;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((unsigned int)(per_xcd * kXcds));
  UNIRL_TRACE_SET(A, "lmhead_tile", grid.x);
  // from 512 rows the operands of the 256 x 256 tile travel global memory -> LDS directly
  const bool dma = edge == 256 && rows >= (int64_t)tune_int("UNIRL_HEAD_DMA_ROWS", 512);
  int rc = (edge == 256) ? (dma ? launch_head_tiles<256, true>(A, grid, st) : launch_head_tiles<256, false>(A, grid, st))
                         : launch_head_tiles<128, false>(A, grid, st);
  if (rc != 0) return rc;
  const int per_block = kHdThreads / kWave;
  hipLaunchKernelGGL(lmhead_merge_kernel, dim3((unsigned int)((rows + per_block - 1) / per_block)), dim3(kHdThreads), 0,
                     st, A);
  return (int)hipGetLastError();
}

extern "C" int unirl_transpose_2d(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, int64_t rows,
                                  int64_t cols, int elem_bytes, void* stream) {
  if (rows < 0 || cols < 0) return UNIRL_E_SHAPE;
  if (rows == 0 || cols == 0) return UNIRL_OK;
  if (!src || !dst) return UNIRL_E_NULL;
  if (elem_bytes != 2 && elem_bytes != 4) return UNIRL_E_DTYPE;
  if (ld_src < cols || ld_dst < rows) return UNIRL_E_SHAPE;
  if (!aligned_to(src, elem_bytes) || !aligned_to(dst, elem_bytes)) return UNIRL_E_ALIGN;
  const int64_t tiles_x = (cols + kTrTile - 1) / kTrTile, tiles_y = (rows + kTrTile - 1) / kTrTile;
  if (tiles_x > 0x7fffffffLL || tiles_y > 65535) return UNIRL_E_LIMIT;  // grid extents (y: 4 M source rows)
  TransposeArgs A;
  A.src = src;
  A.dst = dst;
  A.rows = rows;
  A.cols = cols;
  A.ld_src = ld_src;
  A.ld_dst = ld_dst;
  const int64_t ve = 16 / elem_bytes;
  A.vec_src = (aligned_to(src, 16) && ld_src % ve == 0) ? 1 : 0;
  A.vec_dst = (aligned_to(dst, 16) && ld_dst % ve == 0) ? 1 : 0;
  const dim3 grid((unsigned int)tiles_x, (unsigned int)tiles_y), block(kTrThreads);
  if (elem_bytes == 2) hipLaunchKernelGGL(transpose_tile_kernel<uint16_t>, grid, block, 0, (hipStream_t)stream, A);
  else hipLaunchKernelGGL(transpose_tile_kernel<uint32_t>, grid, block, 0, (hipStream_t)stream, A);
  return (int)hipGetLastError();
}
