// The prefill kernel of the dispatcher: 256 x 256 tiles on v_mfma_f32_16x16x32, weights in a ring of K-pair slots (or
// 64-byte-row stages when prepacked), activations in a ring of four stages. Own translation unit: it is the largest
// set of instances of the library and compiles beside kernels_tiled.hip, which keeps the 32x32x16 kernels.
#include <type_traits>

#include "fsw_internal.h"
#include "fsw_device.h"

namespace fsw {

typedef __attribute__((address_space(3))) void lds_void;

// ---- pair ring on v_mfma_f32_16x16x32 ----------------------------------------------------------------------------
// 256 x 256 workgroup tile, 4 waves of 128 x 128, K tiles of 32 elements. The wave tile is 8 x 8 blocks of 16 x 16 and
// ONE MFMA covers the whole 32-deep K tile. Per FLOP the 16x16x32 instruction moves half the accumulator registers of
// 32x32x16 (and twice the operand registers: 20 % less register-file traffic in total), and under the board's power
// cap that is what sets the clock: a register-only loop of either instruction issues at the same rate with all-zero
// operands (2445 vs 2480 TFLOP/s) and sustains 2090 vs 1822 TFLOP/s with random operands. Accumulators are a
// two-dimensional array indexed by constants only (a flat array made the register allocator move accumulators
// between MFMAs), and the MFMA is written out with its destination tied to the addend (mfma16_acc).
//
// Operands go global -> LDS with buffer_load ... lds. The activation operand is panel-blocked (blocks of
// [256 rows][32 elements], 16 KB contiguous) and keeps four 16 KB stages = two K pairs. The weight operand is
// ROW-MAJOR: read 32 K elements at a time it would yield 64-byte requests, half a cache line each, so it is fetched in
// K PAIRS (64 elements = one 128-byte line per row) into a ring of three 32 KB pair slots. 160 KB of LDS.
// The main loop walks K in pairs with ONE workgroup barrier per pair (see pair_iteration); the slot/stage pattern
// repeats every 6 pairs (lcm of 3 and 2), so the loop is unrolled sixfold with every LDS address a compile-time
// constant. Measured against one barrier per K tile (copies three tiles ahead): gate/up 1.285 -> 1.270 ms at
// 8192 x 4096 x 28672, bit-identical results (the K order is the same); with the barrier in the middle of the pair
// and reads and copies spread evenly over its quarters another 0.6 % (gate/up) and 1.6 % (down).
// LDS layouts: pair slot = [256 rows][128 B], chunk c of row r at position c ^ ((r >> 1) & 7); activation stage =
// [256 rows][64 B], chunk c at c ^ ((r >> 2) & 3): the 16 rows a fragment read touches at one logical chunk cover
// the 64 banks once. The swizzle is applied on the global side of the copy (which lane fetches which chunk), since
// an LDS-DMA instruction writes lane i at base + 16 i. For the gated kernel the even ("up") weight rows of a tile go
// to LDS rows 0..127 and the odd ("gate") rows to 128..255; a wave multiplies 64 of each against the same activation
// fragments, so up and gate of one output land in the same lane and register index.
// PBLK: the weight operand is panel-blocked as well (prepacked; for the gated kernel in de-interleaved row order). It
// then arrives like the activations, one 16 KB block per K tile; a pair slot holds the two blocks of a K pair, one
// after the other, as 64-byte rows, and the ring of three slots runs on the same schedule as for row-major weights.
// QROW: the activation operand is row-major as well (no blocked copy of it exists anywhere). It is then fetched
// exactly like row-major weights, in K pairs of one whole 128-byte line per row, into TWO pair slots that take the
// place of the four stages (same 64 KB, same schedule: the slot of pair I is free from the barrier of pair I on and
// is refilled with pair I + 2); rows past nq read as zero.
// SPLIT (row-major operands, plain product): blockIdx.y selects one of a.splits contiguous runs of 64-element K
// pairs; the workgroup multiplies that run only and stores its fp32 accumulators to a.partial[blockIdx.y][nq][np].
// OF32 (gated, row-major operands and output): H is float and receives the gated value unrounded.
template <class E, bool GATED, bool KTAIL, bool OBLK, bool PBLK = false, bool QROW = false, bool SPLIT = false,
          bool OF32 = false>
__global__ void __launch_bounds__(256)
tiled_pair16_kernel(const GemmArgs a_in, const int tiles_p, const int tiles_q, const int group) {
  static_assert(!SPLIT || (QROW && !GATED && !OBLK && !PBLK), "split-K: row-major operands, plain product");
  static_assert(!OF32 || (GATED && QROW && !OBLK && !PBLK), "fp32 output: the gated kernel on row-major operands");
  GemmArgs a = a_in;
  if constexpr (SPLIT) {  // the run of this workgroup as a product of its own: shifted operands, shorter K
    const int per = ((a_in.k + 63) / 64 + a_in.splits - 1) / a_in.splits * 64;
    const long long k0 = (long long)blockIdx.y * per;
    const long long left = a_in.k - k0;
    a.k = left < 0 ? 0 : (left < per ? (int)left : per);
    a.P = (const unsigned short*)a_in.P + k0;
    a.Q = (const unsigned short*)a_in.Q + k0;
  }
  constexpr int WP = 2, WQ = 2;
  constexpr int NB = 8;  // 16-row blocks per wave and operand
  constexpr int BP = 256, BQ = 256;
  constexpr int PSLOT = BP * 128, QSTAGE = BQ * 64;
  constexpr int LPH = 4;  // weight copy instructions per wave per HALF pair (8 rows x 128 B each)
  constexpr int LQ = 4;   // activation copy instructions per wave per K tile (16 rows x 64 B each)
  static_assert(!OBLK || GATED, "only H is ever written blocked");
  static_assert(!PBLK || !KTAIL || QROW, "blocked operands are zero padded in K");
  constexpr int PSTAGE = BP * 64;

  __shared__ __align__(1024) unsigned char ps0[PSLOT];
  __shared__ __align__(1024) unsigned char ps1[PSLOT];
  __shared__ __align__(1024) unsigned char ps2[PSLOT];
  // activations: four 16 KB stages, or (QROW) two 32 KB pair slots qs0, qs1; one array per stage or slot
  __shared__ __align__(1024) unsigned char qs0[QROW ? PSLOT : QSTAGE];
  __shared__ __align__(1024) unsigned char qs1[QROW ? PSLOT : QSTAGE];
  unsigned char* qs2 = nullptr;
  unsigned char* qs3 = nullptr;
  if constexpr (!QROW) {  // 160 KB are all there is: the two stages exist only where they are used
    __shared__ __align__(1024) unsigned char qs2_mem[QSTAGE];
    __shared__ __align__(1024) unsigned char qs3_mem[QSTAGE];
    qs2 = qs2_mem;
    qs3 = qs3_mem;
  }
  unsigned char* const ps[3] = {ps0, ps1, ps2};
  unsigned char* const qs[4] = {qs0, qs1, qs2, qs3};

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wq = wave % WQ;
  const int wp = wave / WQ;
  const int r16 = lane & 15;
  const int c4 = lane >> 4;

  int tp, tq;
  tile_coords(blockIdx.x, tiles_p, tiles_q, group, tp, tq);
  const int p0 = tp * BP;
  const int q0 = tq * BQ;
  const int nkt = (a.k + 31) / 32;
  const int npair = (nkt + 1) / 2;

  // weight copy: lane -> chunk position pcp of row rbp (+ 32 j), fetches logical chunk lcp of the 128-byte line
  const int pcp = t & 7;
  const int rbp = t >> 3;
  const int lcp = pcp ^ ((rbp >> 1) & 7);
  const unsigned char* pbase = PBLK ? (const unsigned char*)a.P + (long long)tp * nkt * PSTAGE
                                    : (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const __amdgpu_buffer_rsrc_t prs =
      make_rsrc(pbase, PBLK ? (long long)nkt * PSTAGE : ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  // Copy instruction j of a pair covers LDS rows rbp + 32 j, i.e. weight rows (GATED: 2 rbp + 64 (j & 3) + (j >> 2),
  // the even rows first, then the odd ones; else rbp + 32 j). Only the lane's part lives in a register; the part
  // that depends on j and on the K position is wave-uniform and is added where the copy is issued (one VALU add per
  // copy, in the shadow of the MFMAs): eight per-lane offsets held across the loop cost registers the accumulators
  // need. The sum goes into the instruction's vector offset, which the hardware bounds-checks (rows past the matrix
  // read as zero); its scalar offset is not checked.
  const unsigned ldp2 = (unsigned)a.ldp * 2u;
  const unsigned poff0 = (unsigned)(GATED ? 2 * rbp : rbp) * ldp2 + (unsigned)lcp * 16u;
  auto p_row_off = [&](int j) -> unsigned { return (unsigned)(GATED ? 64 * (j & 3) + (j >> 2) : 32 * j) * ldp2; };
  // activation copy from the blocked panel: lane -> chunk position pcq of row rbq (+ 64 j)
  const int pcq = t & 3;
  const int rbq = t >> 2;
  const int lcq = pcq ^ ((rbq >> 2) & 3);
  const unsigned char* qbase = QROW ? (const unsigned char*)a.Q + (long long)q0 * a.ldq * 2
                                    : (const unsigned char*)a.Q + (long long)tq * nkt * QSTAGE;
  const __amdgpu_buffer_rsrc_t qrs =
      make_rsrc(qbase, QROW ? ((long long)(a.nq - q0 - 1) * a.ldq + a.k) * 2 : (long long)nkt * QSTAGE);
  // Activation copy j covers rows rbq + 64 j of one K tile. Blocked panels are zero padded and need no bounds check:
  // the j and K parts go into the scalar offset. Row-major activations (QROW) are treated like row-major weights:
  // copy j covers rows rbp + 32 j of a K pair.
  const unsigned ldq2 = (unsigned)a.ldq * 2u;
  const unsigned qoff0 = QROW ? (unsigned)rbp * ldq2 + (unsigned)lcp * 16u : (unsigned)rbq * 64u + (unsigned)lcq * 16u;
  auto p_copy = [&](lds_void* dst, int j, int pair, bool in) {  // row-major weights: copy j (0 .. 7) of a K pair
    const unsigned voff = poff0 + (p_row_off(j) + (unsigned)pair * 128u);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, dst, 16, (int)(in ? voff : OOB_OFFSET), 0, 0, 0);
  };

  // operand fragment of a 16-row block: lane -> row r16, 16-byte K chunk c4 of the 32-element K tile
  const unsigned rd_p = PBLK ? (unsigned)((GATED ? wp * 64 : wp * 128) + r16) * 64u +
                                   (unsigned)((c4 ^ ((r16 >> 2) & 3)) * 16)
                             : (unsigned)((GATED ? wp * 64 : wp * 128) + r16) * 128u;
  const unsigned rd_q = QROW ? (unsigned)(wq * 128 + r16) * 128u
                             : (unsigned)(wq * 128 + r16) * 64u + (unsigned)((c4 ^ ((r16 >> 2) & 3)) * 16);
  unsigned xp[2];  // [half of the pair]
#pragma unroll
  for (int h = 0; h < 2; ++h) xp[h] = (unsigned)((((h << 2) | c4) ^ ((r16 >> 1) & 7)) * 16);
  auto p_block_off = [](int f) -> unsigned {
    constexpr unsigned RB = PBLK ? 64 : 128;  // bytes per weight row in LDS
    if (GATED) return (unsigned)(f < NB / 2 ? f * 16 : BP / 2 + (f - NB / 2) * 16) * RB;
    return (unsigned)(f * 16) * RB;
  };

  f32x4 acc[NB][NB];
#pragma unroll
  for (int f = 0; f < NB; ++f)
#pragma unroll
    for (int g = 0; g < NB; ++g) acc[f][g] = f32x4{0.f, 0.f, 0.f, 0.f};

  // two register sets of the 16 fragments of a K tile: [0..7] weight blocks, [8..15] activation blocks
  u32x4 fr[2][2 * NB];
  // ONE workgroup barrier per K PAIR (two K tiles, 128 MFMAs per wave), in the MIDDLE of the pair. Pair iteration I
  // multiplies tile a = 2I (fragments in register set 0) and tile b = 2I + 1 (set 1) in four quarters of 32 MFMAs;
  // every quarter carries 8 fragment reads and 4 copies, so that LDS and the copy queue see an even load:
  //   Q1  a, weight blocks 0..3   + the activation fragments of b      + weight copies 0..3 of pair I + 2
  //   Q2  a, weight blocks 4..7   + the weight fragments of b (first half of the quarter) + weight copies 4..7
  //   barrier: pair I + 1 has landed (all but the 8 weight copies just issued); every wave has read all of pair I
  //   Q3  b, weight blocks 0..3   + the activation fragments of tile a of pair I + 1 + activation copies 0..3 of
  //                                 pair I + 2 (into the two stages of pair I, free since the barrier)
  //   Q4  b, weight blocks 4..7   + the weight fragments of tile a of pair I + 1     + activation copies 4..7
  // The weight copies of pair I + 2 go into the slot pair I - 1 left at the previous barrier. Measured at
  // 8192 x 4096 x 14336 against the barrier at the end of Q3 (16 reads in Q2 and in Q4, 8 copies in Q1 and in Q3):
  // gate/up -0.6 %, down -1.6 %; weight copies issued a pair earlier still (in Q4): down +3.7 %.
  constexpr int VM = 2 * LPH;
  constexpr int WAIT_IMM = (VM & 15) | ((VM >> 4) << 14) | (7 << 4) | (0 << 8);
  auto read_one = [&](int set, int idx, const unsigned char* pslot, int half, const unsigned char* qstage) {
    if (idx == 0) {
      fr[set][0] = *(const u32x4*)(pslot + rd_p + p_block_off(0) + (PBLK ? 0u : xp[half]));
    } else if (idx <= NB) {
      fr[set][NB + idx - 1] = *(const u32x4*)(qstage + rd_q + (idx - 1) * 16 * (QROW ? 128 : 64) + (QROW ? xp[half] : 0u));
    } else {
      fr[set][idx - NB] = *(const u32x4*)(pslot + rd_p + p_block_off(idx - NB) + (PBLK ? 0u : xp[half]));
    }
  };
  // MFMA i of a K tile: weight block f = i / 8, activation block g walking forth on even f and back on odd f, so
  // that exactly one operand changes from any MFMA to the next (at the end of a row of blocks only the weight
  // fragment). Operand register reads cost power like everything else here: against restarting g at 0 the whole
  // forward at 8192 x 4096 x 14336 measures 0.5 % faster (1.8628 vs 1.8728 ms), bit-identical.
  auto mma_one = [&](int set, int i) {
    const int f = i / NB, g = (f & 1) ? NB - 1 - i % NB : i % NB;
    E::mfma16_acc(acc[f][g], fr[set][f], fr[set][NB + g]);
  };
  // activation copy j (0 .. 7) of pair `pair`: tile 2 pair + j / 4; tiles past the end arrive as zeros
  // (QROW: st_a is the pair slot, st_b unused; copy j covers rows 32 j .. 32 j + 31 of the pair, 128 bytes each)
  auto q_pair_copy = [&](unsigned char* st_a, unsigned char* st_b, int pair, int j) {
    if constexpr (QROW) {
      const bool qin = pair < npair && (!KTAIL || (pair * 64 + lcp * 8) < a.k);
      const unsigned voff = qoff0 + ((unsigned)(32 * j) * ldq2 + (unsigned)pair * 128u);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, (lds_void*)(st_a + j * 32 * 128 + wave * 1024), 16,
                                               (int)(qin ? voff : OOB_OFFSET), 0, 0, 0);
    } else {
      const int qt = 2 * pair + j / LQ;
      unsigned char* st = j < LQ ? st_a : st_b;
      lds_void* dst = (lds_void*)(st + (j % LQ) * 64 * 64 + wave * 1024);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, dst, 16, (int)(qt < nkt ? qoff0 : OOB_OFFSET),
                                               (j % LQ) * 64 * 64 + qt * QSTAGE, 0, 0);
    }
  };
  // weight copy j (0 .. 7) of pair `pair` into a pair slot: row-major: 32 rows of 128 bytes; prepacked: a quarter of
  // the block of K tile 2 pair + j / 4 (the second block of the pair sits PSTAGE bytes into the slot)
  auto p_pair_copy = [&](unsigned char* slot, int pair, int j) {
    if constexpr (PBLK) {
      const int pt = 2 * pair + j / LPH;
      unsigned char* st = slot + (j / LPH) * PSTAGE;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, (lds_void*)(st + (j % LPH) * 64 * 64 + wave * 1024), 16,
                                               (int)(pt < nkt ? (unsigned)rbq * 64u + (unsigned)lcq * 16u : OOB_OFFSET),
                                               (j % LPH) * 64 * 64 + pt * PSTAGE, 0, 0);
    } else {
      const int pc = pair < npair ? pair : npair - 1;  // past the end: re-read the last pair, never multiplied
      const bool in = !KTAIL || (pc * 64 + lcp * 8) < a.k;
      p_copy((lds_void*)(slot + j * 32 * 128 + wave * 1024), j, pc, in);
    }
  };
  auto pair_iteration = [&](auto i_c, int pr) {
    constexpr int I = decltype(i_c)::value;  // pair index modulo 6: LDS addresses are compile-time constants
    unsigned char* const pb = ps[I % 3] + (PBLK ? PSTAGE : 0);  // tile b of this pair
    unsigned char* const pna = ps[(I + 1) % 3];                 // tile a of the next pair
    unsigned char* const pfill = ps[(I + 2) % 3];               // slot of pair I - 1: refilled with pair I + 2
    // stages (QROW: the slot) of this pair: refilled with pair I + 2 after the barrier
    unsigned char* const qfa = QROW ? qs[I & 1] : qs[(2 * I) & 3];
    unsigned char* const qb = QROW ? qs[I & 1] : qs[(2 * I + 1) & 3];
    unsigned char* const qna = QROW ? qs[(I + 1) & 1] : qs[(2 * I + 2) & 3];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      mma_one(0, 4 * c + 0);
      read_one(1, 1 + c, pb, 1, qb);
      mma_one(0, 4 * c + 1);
      __builtin_amdgcn_sched_barrier(0);
      mma_one(0, 4 * c + 2);
      if (c & 1) {
        p_pair_copy(pfill, pr + 2, c >> 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      mma_one(0, 4 * c + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      mma_one(0, 4 * NB + 2 * c);
      read_one(1, c == 0 ? 0 : NB + c, pb, 1, qb);
      mma_one(0, 4 * NB + 2 * c + 1);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      mma_one(0, 4 * NB + 16 + 4 * c);
      mma_one(0, 4 * NB + 16 + 4 * c + 1);
      p_pair_copy(pfill, pr + 2, 4 + c);
      __builtin_amdgcn_sched_barrier(0);
      mma_one(0, 4 * NB + 16 + 4 * c + 2);
      mma_one(0, 4 * NB + 16 + 4 * c + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt %0\n\ts_barrier" ::"n"(WAIT_IMM) : "memory");
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      mma_one(1, 4 * c + 0);
      read_one(0, 1 + c, pna, 0, qna);
      mma_one(1, 4 * c + 1);
      __builtin_amdgcn_sched_barrier(0);
      mma_one(1, 4 * c + 2);
      if (c & 1) {
        q_pair_copy(qfa, qb, pr + 2, c >> 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      mma_one(1, 4 * c + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      mma_one(1, 4 * NB + 4 * c);
      read_one(0, c == 0 ? 0 : NB + c, pna, 0, qna);
      mma_one(1, 4 * NB + 4 * c + 1);
      __builtin_amdgcn_sched_barrier(0);
      mma_one(1, 4 * NB + 4 * c + 2);
      if (c & 1) {
        q_pair_copy(qfa, qb, pr + 2, 4 + (c >> 1));
        __builtin_amdgcn_sched_barrier(0);
      }
      mma_one(1, 4 * NB + 4 * c + 3);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  if (nkt > 0) {
    // pairs 0 and 1 of both operands; pair 0 has landed when the 16 copies of pair 1 are still in flight
#pragma unroll
    for (int j = 0; j < 8; ++j) p_pair_copy(ps0, 0, j);
#pragma unroll
    for (int j = 0; j < 8; ++j) q_pair_copy(qs0, qs1, 0, j);
#pragma unroll
    for (int j = 0; j < 8; ++j) p_pair_copy(ps1, 1, j);
#pragma unroll
    for (int j = 0; j < 8; ++j) q_pair_copy(QROW ? qs1 : qs2, qs3, 1, j);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * VM) : "memory");
#pragma unroll
    for (int i = 0; i < 2 * NB; ++i) read_one(0, i, ps0, 0, qs0);
  }
  int pr = 0;
  for (; pr + 5 < npair; pr += 6) {
    pair_iteration(std::integral_constant<int, 0>{}, pr);
    pair_iteration(std::integral_constant<int, 1>{}, pr + 1);
    pair_iteration(std::integral_constant<int, 2>{}, pr + 2);
    pair_iteration(std::integral_constant<int, 3>{}, pr + 3);
    pair_iteration(std::integral_constant<int, 4>{}, pr + 4);
    pair_iteration(std::integral_constant<int, 5>{}, pr + 5);
  }
#define FSW_PAIR16_TAIL(I)                                        \
  if (pr < npair) {                                             \
    pair_iteration(std::integral_constant<int, I>{}, pr);      \
    ++pr;                                                       \
  }
  FSW_PAIR16_TAIL(0)
  FSW_PAIR16_TAIL(1)
  FSW_PAIR16_TAIL(2)
  FSW_PAIR16_TAIL(3)
  FSW_PAIR16_TAIL(4)
#undef FSW_PAIR16_TAIL

  // epilogue: a lane owns activation row r16 of each block column and 4 consecutive features (4 c4 ..) per block row
  mfma_drain();
  // The lane's coordinates are derived again here (from the hardware lane count, not from the values the loop set-up
  // used): kept alive across the main loop they would not fit the register file beside the 256 accumulators and the
  // two fragment sets, and the compiler would park them in scratch memory.
  const int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  const int r16e = lane_e & 15, c4e = lane_e >> 4;
  // Output stores are 16 bytes per lane: a lane's accumulator block holds 4 consecutive features (8 bytes), so two
  // neighbouring 16-feature blocks (f, f + 1) are exchanged between the four 16-lane rows of the wave (lane = 16 c4 +
  // r16) with two swap instructions per register -- upper/lower 32 lanes, then odd/even rows -- after which row c4
  // holds features 8 (c4 & 1) .. + 7 of block f + (c4 >> 1): a store instruction then writes 64 contiguous bytes per
  // activation row (a whole 1 KB run of the blocked layout) instead of 32.
  auto widen = [](u32x2 lo, u32x2 hi) -> u32x4 {  // lo: block f, hi: block f + 1 (packed pairs of features)
    u32x4 out;
#pragma unroll
    for (int d = 0; d < 2; ++d) {
      const auto s32 = __builtin_amdgcn_permlane32_swap(lo[d], hi[d], false, false);
      const auto s16 = __builtin_amdgcn_permlane16_swap(s32[0], s32[1], false, false);
      out[d] = s16[0];
      out[2 + d] = s16[1];
    }
    return out;
  };
  if constexpr (OBLK) {
    // H panel-blocked (see store_tile_blocked): every row of the panel and every feature up to the next multiple
    // of 32 is written; padding comes out of zero operand rows
    const int nblocks = (a.np / 2 + 31) >> 5;
    unsigned char* O = (unsigned char*)a.O;
#pragma unroll
    for (int g = 0; g < NB; ++g) {
      const int row = wq * 128 + g * 16 + r16e;
#pragma unroll
      for (int f = 0; f < NB / 2; f += 2) {
        const int blk = tp * 4 + wp * 2 + (f >> 1);
        u32x2 pk[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[f + h][g][e] * silu_f32(acc[f + h + NB / 2][g][e]);
          pk[h] = u32x2{E::pack2(v[0], v[1]), E::pack2(v[2], v[3])};
        }
        const u32x4 w = widen(pk[0], pk[1]);
        if (blk < nblocks) *(u32x4*)(O + (((long long)tq * nblocks + blk) * 256 + row) * 64 + c4e * 16) = w;
      }
    }
  } else if constexpr (SPLIT) {
    float* const part = a.partial + (long long)blockIdx.y * a.nq * a.np;
    const bool vec_ok = (a.np & 3) == 0;
#pragma unroll
    for (int g = 0; g < NB; ++g) {
      const int m = q0 + wq * 128 + g * 16 + r16e;
      if (m >= a.nq) continue;
      float* prow = part + (long long)m * a.np;
#pragma unroll
      for (int f = 0; f < NB; ++f) {
        const int n = p0 + wp * 128 + f * 16 + c4e * 4;
        if (vec_ok && n + 3 < a.np) {
          *(f32x4*)(prow + n) = acc[f][g];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < a.np) prow[n + e] = acc[f][g][e];
        }
      }
    }
  } else if constexpr (OF32) {
    float* O = (float*)a.O;
    const int nout = a.np / 2;
    const bool vec_ok = ((a.ldo & 3) == 0) && ((((uintptr_t)a.O) & 15) == 0);
    const int nbase = p0 / 2 + wp * 64;
#pragma unroll
    for (int g = 0; g < NB; ++g) {
      const int m = q0 + wq * 128 + g * 16 + r16e;
      if (m >= a.nq) continue;
      float* orow = O + (long long)m * a.ldo;
#pragma unroll
      for (int f = 0; f < NB / 2; ++f) {
        f32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[f][g][e] * silu_f32(acc[f + NB / 2][g][e]);
        const int n = nbase + f * 16 + c4e * 4;
        if (vec_ok && n + 3 < nout) {
          *(f32x4*)(orow + n) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < nout) orow[n + e] = v[e];
        }
      }
    }
  } else {
    unsigned short* O = (unsigned short*)a.O;
    constexpr int FO = GATED ? NB / 2 : NB;
    const int nout = GATED ? a.np / 2 : a.np;
    const bool vec_ok = ((a.ldo & 3) == 0) && ((((uintptr_t)a.O) & 7) == 0);
    const bool vec16_ok = ((a.ldo & 7) == 0) && ((((uintptr_t)a.O) & 15) == 0);
    const int nbase = GATED ? p0 / 2 + wp * 64 : p0 + wp * 128;
#pragma unroll
    for (int g = 0; g < NB; ++g) {
      const int m = q0 + wq * 128 + g * 16 + r16e;
      unsigned short* orow = O + (long long)m * a.ldo;
#pragma unroll
      for (int f = 0; f < FO; f += 2) {
        float v[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            v[h][e] = GATED ? acc[f + h][g][e] * silu_f32(acc[f + h + FO][g][e]) : acc[f + h][g][e];
        if (vec16_ok && nbase + (f + 2) * 16 <= nout) {  // wave-uniform: both blocks lie inside the matrix
          const u32x4 w = widen(u32x2{E::pack2(v[0][0], v[0][1]), E::pack2(v[0][2], v[0][3])},
                                u32x2{E::pack2(v[1][0], v[1][1]), E::pack2(v[1][2], v[1][3])});
          if (m < a.nq) *(u32x4*)(orow + nbase + (f + (c4e >> 1)) * 16 + (c4e & 1) * 8) = w;
        } else if (m < a.nq) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int n = nbase + (f + h) * 16 + c4e * 4;
            if (vec_ok && n + 3 < nout) {
              u32x2 pk = {E::pack2(v[h][0], v[h][1]), E::pack2(v[h][2], v[h][3])};
              *(u32x2*)(orow + n) = pk;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < nout) orow[n + e] = E::cvt1(v[h][e]);
            }
          }
        }
      }
    }
  }
}

namespace {

// activations blocked, weights row-major
template <class E, bool GATED, bool OBLK>
hipError_t launch_pair16_blocked_x(const GemmArgs& a, hipStream_t stream) {
  const int tiles_p = (a.np + 255) / 256;
  const int tiles_q = (a.nq + 255) / 256;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q)), block(256);
  if (a.k % 64 == 0) {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, GATED, false, OBLK>), grid, block, 0, stream, a, tiles_p, tiles_q,
                       raster_group(GATED, tiles_q));
  } else {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, GATED, true, OBLK>), grid, block, 0, stream, a, tiles_p, tiles_q,
                       raster_group(GATED, tiles_q));
  }
  return hipGetLastError();
}

// both operands row-major (OBLK: H written blocked; OF32: H float)
template <class E, bool GATED, bool OBLK = false, bool OF32 = false>
hipError_t launch_pair16_rowmajor(const GemmArgs& a, hipStream_t stream) {
  const int tiles_p = (a.np + 255) / 256;
  const int tiles_q = (a.nq + 255) / 256;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q)), block(256);
  if (a.k % 64 == 0) {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, GATED, false, OBLK, false, true, false, OF32>), grid, block, 0, stream, a,
                       tiles_p, tiles_q, raster_group(GATED, tiles_q));
  } else {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, GATED, true, OBLK, false, true, false, OF32>), grid, block, 0, stream, a,
                       tiles_p, tiles_q, raster_group(GATED, tiles_q));
  }
  return hipGetLastError();
}

// both operands row-major, plain product, K split over blockIdx.y: fp32 partial tiles to a.partial
template <class E>
hipError_t launch_pair16_split(const GemmArgs& a, hipStream_t stream) {
  const int tiles_p = (a.np + 255) / 256;
  const int tiles_q = (a.nq + 255) / 256;
  if (tiles_p <= 0 || tiles_q <= 0 || a.splits <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q), (unsigned)a.splits), block(256);
  if (a.k % 64 == 0) {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, false, false, false, false, true, true>), grid, block, 0, stream, a,
                       tiles_p, tiles_q, raster_group(false, tiles_q));
  } else {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, false, true, false, false, true, true>), grid, block, 0, stream, a,
                       tiles_p, tiles_q, raster_group(false, tiles_q));
  }
  return hipGetLastError();
}

// weights blocked (prepacked): a stage ring for the weights; activations blocked, or (QROW) row-major in K pairs
template <class E, bool GATED, bool OBLK, bool QROW = false>
hipError_t launch_pair16_blocked_xw(const GemmArgs& a, hipStream_t stream) {
  const int tiles_p = (a.np + 255) / 256;
  const int tiles_q = (a.nq + 255) / 256;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q)), block(256);
  if (!QROW || a.k % 64 == 0) {  // blocked activations are zero padded in K; row-major ones need the K-tail checks
    hipLaunchKernelGGL((tiled_pair16_kernel<E, GATED, false, OBLK, true, QROW>), grid, block, 0, stream, a, tiles_p,
                       tiles_q, raster_group(GATED, tiles_q));
  } else if constexpr (QROW) {
    hipLaunchKernelGGL((tiled_pair16_kernel<E, GATED, true, OBLK, true, QROW>), grid, block, 0, stream, a, tiles_p,
                       tiles_q, raster_group(GATED, tiles_q));
  }
  return hipGetLastError();
}

template <class E>
hipError_t launch_pair16_typed(bool gated, const GemmArgs& a, hipStream_t stream) {
  if (gated && a.layout == 1) return launch_pair16_blocked_x<E, true, false>(a, stream);
  if (gated && a.layout == 3) return launch_pair16_blocked_x<E, true, true>(a, stream);
  if (!gated && a.layout == 1) return launch_pair16_blocked_x<E, false, false>(a, stream);
  if (gated && a.layout == 5) return launch_pair16_blocked_xw<E, true, false>(a, stream);
  if (gated && a.layout == 7) return launch_pair16_blocked_xw<E, true, true>(a, stream);
  if (!gated && a.layout == 5) return launch_pair16_blocked_xw<E, false, false>(a, stream);
  if (gated && a.layout == 2) return launch_pair16_rowmajor<E, true, true>(a, stream);
  if (gated && a.layout == 6) return launch_pair16_blocked_xw<E, true, true, true>(a, stream);
  if (gated && a.layout == 0 && a.out_f32) return launch_pair16_rowmajor<E, true, false, true>(a, stream);
  if (a.out_f32) return hipErrorInvalidValue;
  if (a.layout == 0) return gated ? launch_pair16_rowmajor<E, true>(a, stream) : launch_pair16_rowmajor<E, false>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace

// GemmArgs::layout: bit 0 = activations blocked, bit 1 = output blocked (gated only), bit 2 = weights blocked
hipError_t launch_pair16(int dtype, bool gated, const GemmArgs& a, hipStream_t stream) {
  return dtype == 0 ? launch_pair16_typed<Bf16>(gated, a, stream) : launch_pair16_typed<Fp16>(gated, a, stream);
}

// Row-major plain product with K split over a.splits workgroups per tile; fp32 partials to a.partial (not reduced).
hipError_t launch_pair16_splitk(int dtype, const GemmArgs& a, hipStream_t stream) {
  return dtype == 0 ? launch_pair16_split<Bf16>(a, stream) : launch_pair16_split<Fp16>(a, stream);
}

}  // namespace fsw
