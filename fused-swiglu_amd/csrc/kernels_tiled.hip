// LDS-tiled MFMA kernels for the compute-bound (prefill) regime on gfx950.
//
// One kernel template covers both GEMMs of the MLP forward:
//   GATED : H[m, j] = up * silu(gate), up = X[m,:].W13[2j,:], gate = X[m,:].W13[2j+1,:]
//           (the computation of swiglu.cu:111-394: main loop :290-343, gating epilogue :345-393)
//   plain : Y[m, n] = H[m,:].W2[n,:]   (no counterpart in the reference)
//
// Orientation. The MFMA "A" operand (rows of the 32x32 result) is fed with WEIGHT rows and the "B" operand
// (columns of the result) with ACTIVATION rows, so an accumulator lane owns one activation row m and runs of 4
// consecutive output features. That makes the stores 8-byte vectors along the contiguous dimension of the
// output, and, for the gated kernel, lets the de-interleave of W13 happen while the tile is copied into LDS:
// LDS rows [0, BP/2) receive the even ("up") rows of the weight tile and rows [BP/2, BP) the odd ("gate")
// rows. A wave then runs two accumulator sets over the same activation fragments, and up/gate of one (m, j)
// land in the same lane and register index: the gating is plain per-lane fp32 math, no cross-lane traffic.
//
// LDS layout. Each operand tile is [rows][64 elements] = 128 bytes per row, eight 16-byte chunks; chunk c of
// row r is stored at chunk position c ^ (r & 7). A wave's ds_read_b128 for an MFMA operand touches 32
// consecutive rows at one logical chunk (x2 for the two K halves), so any 8 consecutive lanes cover all 32
// banks exactly once; the global->LDS copy writes whole 128-byte rows per 8 lanes. Both are conflict-free.
#include <type_traits>

#include "fsw_internal.h"
#include "fsw_device.h"

namespace fsw {

// Epilogue shared by the tiled kernels. A lane owns activation row m = l32 of each Q fragment and, per group
// of 4 accumulator registers, 4 consecutive output features: feature = 8 * (i / 4) + 4 * hi + (i % 4) within
// the fragment. Gating (fp32 multiply and SiLU, swiglu.cu:380-381) happens here, then ONE rounding and an
// 8-byte store.
template <class E, bool GATED, int WP, int WQ, int FP, int FQ>
__device__ __forceinline__ void store_tile(f32x16 (&acc)[FP][FQ], const GemmArgs& a, int p0, int q0, int wp, int wq,
                                           int l32, int hi) {
  unsigned short* O = (unsigned short*)a.O;
  const int nout = GATED ? a.np / 2 : a.np;
  const bool vec_ok = ((a.ldo & 3) == 0) && ((((uintptr_t)a.O) & 7) == 0);
  constexpr int FO = GATED ? FP / 2 : FP;
#pragma unroll
  for (int g = 0; g < FQ; ++g) {
    const int m = q0 + (wq * FQ + g) * 32 + l32;
    if (m >= a.nq) continue;
    unsigned short* orow = O + (long long)m * a.ldo;
#pragma unroll
    for (int f = 0; f < FO; ++f) {
      const int nb = (GATED ? p0 / 2 + (wp * FO + f) * 32 : p0 + (wp * FO + f) * 32) + hi * 4;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (GATED) {
            v[e] = acc[f][g][i4 * 4 + e] * silu_f32(acc[f + FO][g][i4 * 4 + e]);
          } else {
            v[e] = acc[f][g][i4 * 4 + e];
          }
        }
        const int n = nb + i4 * 8;
        if (vec_ok && n + 3 < nout) {
          u32x2 pk = {E::pack2(v[0], v[1]), E::pack2(v[2], v[3])};
          *(u32x2*)(orow + n) = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < nout) orow[n + e] = E::cvt1(v[e]);
        }
      }
    }
  }
}

// Gated epilogue that writes H panel-blocked for the down projection: panels of 256 activation rows, blocks of
// 32 features, block (panel, j) = [256 rows][64 bytes] at ((panel * nblocks + j) * 256 + row) * 64. Every row of the
// panel and every feature up to the next multiple of 32 is written: rows past nq and features past ff come from
// out-of-range (zero) operand rows, so the padding the down projection's K loop reads is zero.
template <class E, int WP, int WQ, int FP, int FQ>
__device__ __forceinline__ void store_tile_blocked(f32x16 (&acc)[FP][FQ], const GemmArgs& a, int tp, int tq, int wp,
                                                   int wq, int l32, int hi) {
  constexpr int FO = FP / 2;
  constexpr int BH = WP * FO;  // 32-feature blocks per tile
  const int nblocks = (a.np / 2 + 31) >> 5;
  unsigned char* O = (unsigned char*)a.O;
#pragma unroll
  for (int g = 0; g < FQ; ++g) {
    const int row = (wq * FQ + g) * 32 + l32;
#pragma unroll
    for (int f = 0; f < FO; ++f) {
      const int blk = tp * BH + wp * FO + f;
      if (blk < nblocks) {
        unsigned char* dst = O + (((long long)tq * nblocks + blk) * 256 + row) * 64 + hi * 8;
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = acc[f][g][i4 * 4 + e] * silu_f32(acc[f + FO][g][i4 * 4 + e]);
          u32x2 pk = {E::pack2(v[0], v[1]), E::pack2(v[2], v[3])};
          *(u32x2*)(dst + i4 * 16) = pk;
        }
      }
    }
  }
}

// Split-K epilogue of the plain kernel: fp32 partial sums to partial[split][m][n], 16 bytes per lane.
template <int WP, int WQ, int FP, int FQ>
__device__ __forceinline__ void store_partial(f32x16 (&acc)[FP][FQ], const GemmArgs& a, int split, int p0, int q0,
                                              int wp, int wq, int l32, int hi) {
  float* base = a.partial + (long long)split * a.nq * a.np;
#pragma unroll
  for (int g = 0; g < FQ; ++g) {
    const int m = q0 + (wq * FQ + g) * 32 + l32;
    if (m >= a.nq) continue;
    float* row = base + (long long)m * a.np;
#pragma unroll
    for (int f = 0; f < FP; ++f) {
      const int nb = p0 + (wp * FP + f) * 32 + hi * 4;
#pragma unroll
      for (int i4 = 0; i4 < 4; ++i4) {
        const int n = nb + i4 * 8;
        if (((a.np & 3) == 0) && n + 3 < a.np) {
          f32x4 v = {acc[f][g][i4 * 4], acc[f][g][i4 * 4 + 1], acc[f][g][i4 * 4 + 2], acc[f][g][i4 * 4 + 3]};
          *(f32x4*)(row + n) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < a.np) row[n + e] = acc[f][g][i4 * 4 + e];
        }
      }
    }
  }
}

// O[m, n] = round(sum over splits of partial[s][m][n]); one thread per 4 consecutive n.
template <class E>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float* __restrict__ partial, int splits, int nq, int np, unsigned short* __restrict__ O,
                     long long ldo) {
  const int groups = (np + 3) >> 2;
  const long long id = (long long)blockIdx.x * 256 + threadIdx.x;
  if (id >= (long long)nq * groups) return;
  const int m = (int)(id / groups);
  const int n = (int)(id - (long long)m * groups) * 4;
  const long long plane = (long long)nq * np;
  const float* src = partial + (long long)m * np + n;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  const bool full = ((np & 3) == 0) && n + 3 < np;
  for (int s = 0; s < splits; ++s) {
    if (full) {
      const f32x4 t = *(const f32x4*)(src + s * plane);
      v[0] += t[0];
      v[1] += t[1];
      v[2] += t[2];
      v[3] += t[3];
    } else {
      for (int e = 0; e < 4; ++e)
        if (n + e < np) v[e] += src[s * plane + e];
    }
  }
  unsigned short* orow = O + (long long)m * ldo;
  if (full && ((ldo & 3) == 0) && ((((uintptr_t)O) & 7) == 0)) {
    u32x2 pk = {E::pack2(v[0], v[1]), E::pack2(v[2], v[3])};
    *(u32x2*)(orow + n) = pk;
  } else {
    for (int e = 0; e < 4; ++e)
      if (n + e < np) orow[n + e] = E::cvt1(v[e]);
  }
}

template <class E, bool GATED, int WP, int WQ, int FP, int FQ>
__global__ void __launch_bounds__(WP* WQ * 64)
tiled_kernel(const GemmArgs a, const int tiles_p, const int tiles_q, const int group) {
  constexpr int NT = WP * WQ * 64;
  constexpr int BP = WP * FP * 32;  // weight rows per workgroup tile
  constexpr int BQ = WQ * FQ * 32;  // activation rows per workgroup tile
  constexpr int BK = 64;            // K elements per LDS stage
  constexpr int ROWB = BK * 2;      // bytes per LDS row
  constexpr int RSTEP = NT / 8;     // row distance between a thread's successive 16-byte copies
  constexpr int LP = BP / RSTEP;    // copies per thread per stage, weight tile
  constexpr int LQ = BQ / RSTEP;    // copies per thread per stage, activation tile
  constexpr int STAGE = (BP + BQ) * ROWB;
  static_assert(BP % RSTEP == 0 && BQ % RSTEP == 0 && RSTEP % 8 == 0, "copy mapping");
  static_assert(!GATED || (FP % 2 == 0), "gated kernel pairs fragments");
  static_assert(2 * STAGE <= 160 * 1024, "LDS budget of a gfx950 CU");

  __shared__ __align__(16) unsigned char lds[2 * STAGE];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int wq = wave % WQ;
  const int wp = wave / WQ;
  const int l32 = lane & 31;
  const int hi = lane >> 5;

  int tp, tq;
  tile_coords(blockIdx.x, tiles_p, tiles_q, group, tp, tq);
  const int p0 = tp * BP;
  const int q0 = tq * BQ;

  // ---- global -> register copy mapping: thread copies chunk `c` of rows rb, rb+RSTEP, ...
  const int c = t & 7;
  const int rb = t >> 3;
  const unsigned char* pbase = (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const unsigned char* qbase = (const unsigned char*)a.Q + (long long)q0 * a.ldq * 2;
  const __amdgpu_buffer_rsrc_t prs = make_rsrc(pbase, ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  const __amdgpu_buffer_rsrc_t qrs = make_rsrc(qbase, ((long long)(a.nq - q0 - 1) * a.ldq + a.k) * 2);

  unsigned poff[LP], qoff[LQ];
#pragma unroll
  for (int i = 0; i < LP; ++i) {
    const int r = rb + i * RSTEP;
    const int grow = GATED ? (r < BP / 2 ? 2 * r : 2 * (r - BP / 2) + 1) : r;
    poff[i] = (unsigned)grow * (unsigned)a.ldp * 2u + (unsigned)c * 16u;
  }
#pragma unroll
  for (int i = 0; i < LQ; ++i) {
    const int r = rb + i * RSTEP;
    qoff[i] = (unsigned)r * (unsigned)a.ldq * 2u + (unsigned)c * 16u;
  }
  // LDS byte address of this thread's first copy; later copies add i * RSTEP * ROWB (RSTEP % 8 == 0 keeps r & 7).
  const unsigned wr_p = (unsigned)rb * ROWB + (unsigned)((c ^ (rb & 7)) * 16);
  const unsigned wr_q = (unsigned)BP * ROWB + wr_p;

  // ---- LDS -> MFMA fragment read mapping
  unsigned xo[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) xo[ks] = (unsigned)((((ks << 1) | hi) ^ (lane & 7)) * 16);
  const unsigned rd_p = (unsigned)((GATED ? wp * (FP / 2) * 32 : wp * FP * 32) + l32) * ROWB;
  const unsigned rd_q = (unsigned)(BP + wq * FQ * 32 + l32) * ROWB;
  auto p_frag_off = [](int f) -> unsigned {
    if (GATED) return (unsigned)((f < FP / 2 ? f * 32 : BP / 2 + (f - FP / 2) * 32) * ROWB);
    return (unsigned)(f * 32 * ROWB);
  };

  f32x16 acc[FP][FQ];
#pragma unroll
  for (int f = 0; f < FP; ++f)
#pragma unroll
    for (int g = 0; g < FQ; ++g)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[f][g][i] = 0.0f;

  u32x4 sp[LP], sq[LQ];
  const int nkt = (a.k + BK - 1) / BK;

  // Copies for K tile `kt`; tiles at or beyond K read as zero (hardware bounds check), so the pipeline below
  // can prefetch past the end without branching.
  // single tile of activation rows: every workgroup walks K from its own starting tile (see tiled_dma_kernel)
  const int rot = (tiles_q == 1 && nkt > 1) ? (int)(((unsigned)blockIdx.x * 2654435761u >> 12) % (unsigned)nkt) : 0;
  auto g_load = [&](int kt) {
    int ktr = kt + rot;
    if (ktr >= nkt) ktr -= nkt;
    const unsigned kb = (unsigned)ktr * (BK * 2);
    const bool in = kt < nkt && (ktr * BK + c * 8) < a.k;
#pragma unroll
    for (int i = 0; i < LP; ++i) sp[i] = buf_load16(prs, in ? poff[i] + kb : OOB_OFFSET);
#pragma unroll
    for (int i = 0; i < LQ; ++i) sq[i] = buf_load16(qrs, in ? qoff[i] + kb : OOB_OFFSET);
  };
  auto s_store = [&](int stage) {
    unsigned char* base = lds + stage * STAGE;
#pragma unroll
    for (int i = 0; i < LP; ++i) *(u32x4*)(base + wr_p + i * RSTEP * ROWB) = sp[i];
#pragma unroll
    for (int i = 0; i < LQ; ++i) *(u32x4*)(base + wr_q + i * RSTEP * ROWB) = sq[i];
  };

  u32x4 pf[2][FP], qf[2][FQ];
  // Fragment reads for K step `ks` of LDS stage `stage`, issued in the order the MFMAs consume them.
  auto f_read = [&](int fb, int stage, int ks) {
    const unsigned char* base = lds + stage * STAGE;
    pf[fb][0] = *(const u32x4*)(base + rd_p + p_frag_off(0) + xo[ks]);
#pragma unroll
    for (int g = 0; g < FQ; ++g) qf[fb][g] = *(const u32x4*)(base + rd_q + g * 32 * ROWB + xo[ks]);
#pragma unroll
    for (int f = 1; f < FP; ++f) pf[fb][f] = *(const u32x4*)(base + rd_p + p_frag_off(f) + xo[ks]);
  };
  auto mma = [&](int fb, int f_lo, int f_hi) {
#pragma unroll
    for (int f = f_lo; f < f_hi; ++f)
#pragma unroll
      for (int g = 0; g < FQ; ++g) acc[f][g] = E::mfma32(pf[fb][f], qf[fb][g], acc[f][g]);
  };

  // Software pipeline, one barrier per K tile of 64:
  //   K steps 0..2 : MFMAs of step s overlap the LDS fragment reads of step s+1 (same stage);
  //   K step 3, a  : first half of the MFMAs overlaps the ds_writes of tile kt+1 (in registers since the
  //                  previous iteration) into the other stage; barrier;
  //   K step 3, b  : second half of the MFMAs overlaps the fragment reads of step 0 of tile kt+1 and the
  //                  global loads of tile kt+2.
  // The other stage is free for writing during the whole iteration: every wave finished its reads of it
  // before the barrier of the previous iteration (they are issued in steps 0..2 and in 3b of the one before).
  g_load(0);
  s_store(0);
  g_load(1);
  __syncthreads();
  f_read(0, 0, 0);

  // Issue-order hints for the machine scheduler (masks: 0x008 MFMA, 0x020 VMEM read, 0x100 LDS read,
  // 0x200 LDS write). Without them the compiler sinks every fragment read next to its first use and the
  // LDS latency is exposed once per K step.
  constexpr int NM = FP * FQ;                      // MFMAs per K step
  constexpr int NR = FP + FQ;                      // fragment reads per K step
  constexpr int HF = FP / 2 > 0 ? FP / 2 : 1;      // fragments in the first half of step 3
  constexpr int MPR = NM / NR > 0 ? NM / NR : 1;   // MFMAs per fragment read
  auto hint_reads = [&]() {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  };
  for (int kt = 0; kt < nkt; ++kt) {
    const int cur = kt & 1;
    // K step 0
    f_read(1, cur, 1);
    mma(0, 0, FP);
    hint_reads();
    // K step 1
    f_read(0, cur, 2);
    mma(1, 0, FP);
    hint_reads();
    // K step 2
    f_read(1, cur, 3);
    mma(0, 0, FP);
    hint_reads();
    // K step 3a
    mma(1, 0, HF);
    s_store(cur ^ 1);
#pragma unroll
    for (int i = 0; i < HF * FQ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x200, (LP + LQ + HF * FQ - 1) / (HF * FQ), 0);
    }
    __syncthreads();
    // K step 3b
    f_read(0, cur ^ 1, 0);
    g_load(kt + 2);
    mma(1, HF, FP);
#pragma unroll
    for (int i = 0; i < (FP - HF) * FQ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x100, (NR + (FP - HF) * FQ - 1) / ((FP - HF) * FQ), 0);
      __builtin_amdgcn_sched_group_barrier(0x020, (LP + LQ + (FP - HF) * FQ - 1) / ((FP - HF) * FQ), 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
  }

  store_tile<E, GATED, WP, WQ, FP, FQ>(acc, a, p0, q0, wp, wq, l32, hi);
}

// ---- direct-to-LDS variant ---------------------------------------------------------------------------------
// Same tiling and epilogue, but the operand tiles go from global memory straight into LDS with
// buffer_load_dwordx4 ... lds (no staging registers, no ds_write: LDS writes by ds_write_b128 run at roughly a
// third of the read rate on this chip and were the largest single cost of the register-staged loop).
// An LDS-DMA instruction writes lane i's 16 bytes at base + 16 i, so a wave instruction fills 8 consecutive
// 128-byte rows; the swizzle is applied on the global side: the lane that lands on chunk position p of row r
// fetches logical chunk p ^ ((r >> 1) & 7). With that function any 16 consecutive rows at one logical chunk
// cover all 64 banks once (the LDS serves ds_read_b128 sixteen lanes per clock), so operand reads are
// conflict-free. The two stages are separate __shared__ objects so that the compiler's counter tracking can
// tell reads of the live stage from DMA writes into the other one.
typedef __attribute__((address_space(3))) void lds_void;

template <class E, bool GATED, bool KTAIL, int WP, int WQ, int FP, int FQ, bool STREAM_W = false, int NS = 2>
__global__ void __launch_bounds__(WP* WQ * 64)
tiled_dma_kernel(const GemmArgs a, const int tiles_p, const int tiles_q, const int group) {
  constexpr int NT = WP * WQ * 64;
  constexpr int BP = WP * FP * 32;
  constexpr int BQ = WQ * FQ * 32;
  constexpr int BK = 64;
  constexpr int ROWB = BK * 2;
  constexpr int RSTEP = NT / 8;
  constexpr int LP = BP / RSTEP;
  constexpr int LQ = BQ / RSTEP;
  constexpr int STAGE = (BP + BQ) * ROWB;
  static_assert(BP % RSTEP == 0 && BQ % RSTEP == 0 && RSTEP % 16 == 0, "copy mapping");
  static_assert(!GATED || (FP % 2 == 0), "gated kernel pairs fragments");
  static_assert(NS >= 2 && NS <= 5 && NS * STAGE <= 160 * 1024, "LDS budget of a gfx950 CU");

  __shared__ __align__(1024) unsigned char lds0[STAGE];
  __shared__ __align__(1024) unsigned char lds1[STAGE];
  __shared__ alignas(NS > 2 ? 1024 : 16) unsigned char lds2[NS > 2 ? STAGE : 16];
  __shared__ alignas(NS > 3 ? 1024 : 16) unsigned char lds3[NS > 3 ? STAGE : 16];
  __shared__ alignas(NS > 4 ? 1024 : 16) unsigned char lds4[NS > 4 ? STAGE : 16];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // wave-uniform: LDS-DMA bases live in SGPRs
  const int wq = wave % WQ;
  const int wp = wave / WQ;
  const int l32 = lane & 31;
  const int hi = lane >> 5;

  int tp, tq;
  tile_coords(blockIdx.x, tiles_p, tiles_q, group, tp, tq);
  const int p0 = tp * BP;
  const int q0 = tq * BQ;

  // ---- global -> LDS copy mapping: lane lands on chunk position pc of row rb (+ i * RSTEP)
  const int pc = t & 7;
  const int rb = t >> 3;
  const int lc = pc ^ ((rb >> 1) & 7);  // logical chunk this lane fetches (RSTEP % 16 == 0 keeps (row >> 1) & 7)
  const unsigned char* pbase = (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const unsigned char* qbase = (const unsigned char*)a.Q + (long long)q0 * a.ldq * 2;
  const __amdgpu_buffer_rsrc_t prs = make_rsrc(pbase, ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  const __amdgpu_buffer_rsrc_t qrs = make_rsrc(qbase, ((long long)(a.nq - q0 - 1) * a.ldq + a.k) * 2);
  unsigned poff[LP], qoff[LQ];
#pragma unroll
  for (int i = 0; i < LP; ++i) {
    const int r = rb + i * RSTEP;
    const int grow = GATED ? (r < BP / 2 ? 2 * r : 2 * (r - BP / 2) + 1) : r;
    poff[i] = (unsigned)grow * (unsigned)a.ldp * 2u + (unsigned)lc * 16u;
  }
#pragma unroll
  for (int i = 0; i < LQ; ++i) {
    const int r = rb + i * RSTEP;
    qoff[i] = (unsigned)r * (unsigned)a.ldq * 2u + (unsigned)lc * 16u;
  }

  // ---- LDS -> MFMA fragment read mapping
  unsigned xo[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) xo[ks] = (unsigned)((((ks << 1) | hi) ^ ((l32 >> 1) & 7)) * 16);
  const unsigned rd_p = (unsigned)((GATED ? wp * (FP / 2) * 32 : wp * FP * 32) + l32) * ROWB;
  const unsigned rd_q = (unsigned)(BP + wq * FQ * 32 + l32) * ROWB;
  auto p_frag_off = [](int f) -> unsigned {
    if (GATED) return (unsigned)((f < FP / 2 ? f * 32 : BP / 2 + (f - FP / 2) * 32) * ROWB);
    return (unsigned)(f * 32 * ROWB);
  };

  f32x16 acc[FP][FQ];
#pragma unroll
  for (int f = 0; f < FP; ++f)
#pragma unroll
    for (int g = 0; g < FQ; ++g)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[f][g][i] = 0.0f;

  // K range of this workgroup: everything, or one of a.splits contiguous runs of K tiles (blockIdx.y)
  const int nkt_all = (a.k + BK - 1) / BK;
  const int kt_per = (nkt_all + a.splits - 1) / a.splits;
  const int kt0 = (int)blockIdx.y * kt_per;
  const int nkt = nkt_all - kt0 < kt_per ? (nkt_all - kt0 > 0 ? nkt_all - kt0 : 0) : kt_per;

  // With a single tile of activation rows no two workgroups share a weight panel, every weight byte comes from
  // HBM, and workgroups that walk K in step all ask for the same column offset of rows a power of two apart: the
  // same few memory channels at any moment (measured 2.2 TB/s). Each workgroup therefore starts its walk at its own
  // K tile and wraps around; only the order of the fp32 summation changes. (With several activation tiles the
  // workgroups that share a panel must stay in step for the L2 to serve them, so there rot = 0.)
  const int rot = (tiles_q == 1 && nkt > 1) ? (int)(((unsigned)blockIdx.x * 2654435761u >> 12) % (unsigned)nkt) : 0;

  // STREAM_W: the weight copies carry the non-temporal cache policy, for launches with one or two tiles of activation rows,
  // where a weight line has at most two users: the single-use stream then neither displaces the activations nor has
  // to evict whatever the previous kernels left dirty in the L2s and the Infinity Cache. Measured at 4096 x 28672,
  // M = 128, caches filled with freshly written data before each call: gate/up 94 -> 67 us, down 63 -> 44 us;
  // back-to-back forwards 110 -> 106 us.
  // DMA of K tile `kt` into `stage`: wave-uniform LDS base per instruction, loop-invariant per-lane offset in a
  // VGPR, the K offset in an SGPR. Rows beyond the matrix are out of range for the buffer descriptor and arrive
  // as zeros. A prefetch past the last tile re-reads the last tile (never consumed). Only when K is not a
  // multiple of 64 (KTAIL) do lanes whose chunk lies at or beyond K redirect their offset out of range.
  auto dma = [&](unsigned char* stage, int kt) {
    int ktr = (kt < nkt ? kt : nkt - 1) + rot;
    if (ktr >= nkt) ktr -= nkt;
    const int ktc = kt0 + ktr;
    const int kb = ktc * (BK * 2);
    const bool in = !KTAIL || (ktc * BK + lc * 8) < a.k;
#pragma unroll
    for (int i = 0; i < LP; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, (lds_void*)(stage + i * RSTEP * ROWB + wave * 1024), 16,
                                               (int)(in ? poff[i] : OOB_OFFSET), kb, 0, STREAM_W ? 2 : 0);
#pragma unroll
    for (int i = 0; i < LQ; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, (lds_void*)(stage + (BP + i * RSTEP) * ROWB + wave * 1024), 16,
                                               (int)(in ? qoff[i] : OOB_OFFSET), kb, 0, 0);
  };

  u32x4 pf[2][FP], qf[2][FQ];
  auto f_read = [&](int fb, const unsigned char* base, int ks) {
    pf[fb][0] = *(const u32x4*)(base + rd_p + p_frag_off(0) + xo[ks]);
#pragma unroll
    for (int g = 0; g < FQ; ++g) qf[fb][g] = *(const u32x4*)(base + rd_q + g * 32 * ROWB + xo[ks]);
#pragma unroll
    for (int f = 1; f < FP; ++f) pf[fb][f] = *(const u32x4*)(base + rd_p + p_frag_off(f) + xo[ks]);
  };
  auto mma = [&](int fb, int f_lo, int f_hi) {
#pragma unroll
    for (int f = f_lo; f < f_hi; ++f)
#pragma unroll
      for (int g = 0; g < FQ; ++g) acc[f][g] = E::mfma32(pf[fb][f], qf[fb][g], acc[f][g]);
  };

  constexpr int NM = FP * FQ;
  constexpr int NR = FP + FQ;
  constexpr int NL = LP + LQ;
  constexpr int HF = FP / 2 > 0 ? FP / 2 : 1;
  constexpr int MPR = NM / NR > 0 ? NM / NR : 1;

  // One K tile. On entry: stage `cur` holds tile kt (made visible by the previous barrier) and its step-0
  // fragments are in pf[0]/qf[0]; every wave is done reading `oth`. The DMA of tile kt+1 into `oth` is issued
  // in step 0 and has the whole iteration to land before the barrier in step 3.
  auto iteration = [&](unsigned char* cur, unsigned char* oth, int kt) {
    dma(oth, kt + 1);
    f_read(1, cur, 1);
    mma(0, 0, FP);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
      __builtin_amdgcn_sched_group_barrier(0x010, (NL + NR - 1) / NR, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    f_read(0, cur, 2);
    mma(1, 0, FP);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    f_read(1, cur, 3);
    mma(0, 0, FP);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    mma(1, 0, HF);
    __syncthreads();  // waits for this wave's DMA (vmcnt) and LDS reads, then for every other wave
    f_read(0, oth, 0);
    mma(1, HF, FP);
#pragma unroll
    for (int i = 0; i < (FP - HF) * FQ; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x100, (NR + (FP - HF) * FQ - 1) / ((FP - HF) * FQ), 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
  };

  // NS stages: two for the compute-bound uses; three when every weight byte comes from HBM exactly once (a single
  // tile of activation rows, weights streamed non-temporally): the copy of tile kt + 2 is issued while tile kt is
  // multiplied, which doubles the bytes in flight per workgroup. Measured at 4096 x 28672, gate/up: M = 65: 67.6 ->
  // 43.9 us, M = 128: 67.0 -> 49.0 us (a fourth stage: level). The split-K down projection keeps two stages (three
  // cost it an LDS-limited workgroup per CU: 36.7 -> 40.4 us).
  if constexpr (NS == 2) {
    if (nkt > 0) dma(lds0, 0);
    __syncthreads();
    if (nkt > 0) f_read(0, lds0, 0);
    int kt = 0;
    for (; kt + 1 < nkt; kt += 2) {
      iteration(lds0, lds1, kt);
      iteration(lds1, lds0, kt + 1);
    }
    if (kt < nkt) iteration(lds0, lds1, kt);
  } else {
    unsigned char* const ring[5] = {lds0, lds1, lds2, lds3, lds4};
    constexpr int VM = (NS - 2) * NL;
    static_assert(VM <= 63, "vmcnt is a 6-bit counter");
    constexpr int WAIT_IMM = (VM & 15) | ((VM >> 4) << 14) | (7 << 4) | (0 << 8);
    auto ring_iteration = [&](unsigned char* cur, unsigned char* nxt, unsigned char* fill, int kt) {
      dma(fill, kt + NS - 1);
      f_read(1, cur, 1);
      mma(0, 0, FP);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, (NL + NR - 1) / NR, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      f_read(0, cur, 2);
      mma(1, 0, FP);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      f_read(1, cur, 3);
      mma(0, 0, FP);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      mma(1, 0, HF);
      asm volatile("s_waitcnt %0\n\ts_barrier" ::"n"(WAIT_IMM) : "memory");
      f_read(0, nxt, 0);
      mma(1, HF, FP);
#pragma unroll
      for (int i = 0; i < (FP - HF) * FQ; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, (NR + (FP - HF) * FQ - 1) / ((FP - HF) * FQ), 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
    };
    if (nkt > 0) {
#pragma unroll
      for (int j = 0; j < NS - 1; ++j) dma(ring[j], j);
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NS - 2) * NL) : "memory");
      f_read(0, lds0, 0);
    }
    int kt = 0;
    for (; kt + NS - 1 < nkt; kt += NS) {
#pragma unroll
      for (int j = 0; j < NS; ++j) ring_iteration(ring[j], ring[(j + 1) % NS], ring[(j + NS - 1) % NS], kt + j);
    }
#pragma unroll
    for (int j = 0; j < NS - 1; ++j) {
      if (kt < nkt) {
        ring_iteration(ring[j], ring[(j + 1) % NS], ring[(j + NS - 1) % NS], kt);
        ++kt;
      }
    }
  }

  if constexpr (!GATED) {
    if (a.splits > 1) {
      store_partial<WP, WQ, FP, FQ>(acc, a, (int)blockIdx.y, p0, q0, wp, wq, l32, hi);
      return;
    }
  }
  store_tile<E, GATED, WP, WQ, FP, FQ>(acc, a, p0, q0, wp, wq, l32, hi);
}

// ---- ring-of-stages direct-to-LDS variant --------------------------------------------------------------------
// K tiles of 32 elements in a ring of NS (4 or 5) LDS stages: the DMA of tile kt+NS-1 is issued while tile kt is
// being multiplied, so a copy has NS-1 iterations (~1000 MFMA cycles each) to land instead of one. That covers L2
// misses (Infinity Cache / HBM latency), which the two-stage kernels above expose at every barrier, and it keeps
// (NS-1) stages of bytes in flight per CU: the L2 -> LDS stream of these kernels is latency-bound, so its rate
// follows the bytes in flight. Five stages of a 256x256 tile are the whole 160 KB of LDS.
// LDS rows are 64 bytes (4 chunks of 16 B); chunk c of row r sits at position c ^ ((r >> 2) & 3): 16 consecutive
// rows at one logical chunk then cover the 64 banks once. The barrier waits for this wave's copy of tile kt+1
// only (vmcnt leaves the younger tiles in flight), hence the hand-written s_waitcnt.
// LAYOUT bits (256 x 256 tile only): 1 = the activation operand Q is panel-blocked (see block_rows_kernel),
// 2 = the output is written panel-blocked (gated kernel: H for the down projection), 4 = the weight operand P is
// panel-blocked (prepacked; for the gated kernel in de-interleaved row order). A blocked operand turns every copy
// instruction into one contiguous 1 KB read of whole cache lines; row-major, a 32-element K tile is 64 bytes per
// row, half a line per request. Measured at 8192 x 4096 x 14336: gate/up 1.52 -> 1.40 ms with X blocked, down
// 0.81 -> 0.70 ms with H blocked.
template <class E, bool GATED, bool KTAIL, int NS, int WP, int WQ, int FP, int FQ, int LAYOUT = 0>
__global__ void __launch_bounds__(WP* WQ * 64)
tiled_ring_kernel(const GemmArgs a, const int tiles_p, const int tiles_q, const int group) {
  constexpr int NT = WP * WQ * 64;
  constexpr int BP = WP * FP * 32;
  constexpr int BQ = WQ * FQ * 32;
  constexpr int BK = 32;
  constexpr int ROWB = BK * 2;      // 64
  constexpr int RSTEP = NT / 4;     // rows covered by one round of DMA instructions (16 rows per wave)
  constexpr int LP = BP / RSTEP;
  constexpr int LQ = BQ / RSTEP;
  constexpr int NL = LP + LQ;       // DMA instructions per wave per K tile
  constexpr int STAGE = (BP + BQ) * ROWB;
  static_assert(BP % RSTEP == 0 && BQ % RSTEP == 0 && RSTEP % 16 == 0, "copy mapping");
  static_assert(!GATED || (FP % 2 == 0), "gated kernel pairs fragments");
  static_assert(NS == 4 || NS == 5, "ring length");
  constexpr bool QBLK = (LAYOUT & 1) != 0, OBLK = (LAYOUT & 2) != 0, PBLK = (LAYOUT & 4) != 0;
  static_assert(LAYOUT == 0 || (BP == 256 && BQ == 256), "blocked layouts are defined for 256-row panels");
  static_assert(!OBLK || GATED, "only H is ever written blocked");
  static_assert(NS * STAGE <= 160 * 1024, "LDS budget of a gfx950 CU");

  // one array per stage: the compiler tracks outstanding LDS DMA per array
  __shared__ __align__(1024) unsigned char ring0[STAGE];
  __shared__ __align__(1024) unsigned char ring1[STAGE];
  __shared__ __align__(1024) unsigned char ring2[STAGE];
  __shared__ __align__(1024) unsigned char ring3[STAGE];
  __shared__ __align__(1024) unsigned char ring4[NS > 4 ? STAGE : 1024];
  unsigned char* const ring[5] = {ring0, ring1, ring2, ring3, ring4};

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wq = wave % WQ;
  const int wp = wave / WQ;
  const int l32 = lane & 31;
  const int hi = lane >> 5;

  int tp, tq;
  tile_coords(blockIdx.x, tiles_p, tiles_q, group, tp, tq);
  const int p0 = tp * BP;
  const int q0 = tq * BQ;

  const int pc = t & 3;
  const int rb = t >> 2;
  const int lc = pc ^ ((rb >> 2) & 3);
  const int nkt = (a.k + BK - 1) / BK;
  // a blocked panel: nkt blocks of [256 rows][64 bytes], block kt holds K elements 32 kt .. 32 kt + 31 (zero padded)
  constexpr int PBLOCK = BP * ROWB, QBLOCK = BQ * ROWB;
  const unsigned char* pbase = PBLK ? (const unsigned char*)a.P + (long long)tp * nkt * PBLOCK
                                    : (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const unsigned char* qbase = QBLK ? (const unsigned char*)a.Q + (long long)tq * nkt * QBLOCK
                                    : (const unsigned char*)a.Q + (long long)q0 * a.ldq * 2;
  const __amdgpu_buffer_rsrc_t prs =
      make_rsrc(pbase, PBLK ? (long long)nkt * PBLOCK : ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  const __amdgpu_buffer_rsrc_t qrs =
      make_rsrc(qbase, QBLK ? (long long)nkt * QBLOCK : ((long long)(a.nq - q0 - 1) * a.ldq + a.k) * 2);
  unsigned poff[LP], qoff[LQ];
#pragma unroll
  for (int i = 0; i < LP; ++i) {
    const int r = rb + i * RSTEP;
    const int grow = GATED ? (r < BP / 2 ? 2 * r : 2 * (r - BP / 2) + 1) : r;
    poff[i] = PBLK ? (unsigned)r * (unsigned)ROWB + (unsigned)lc * 16u
                   : (unsigned)grow * (unsigned)a.ldp * 2u + (unsigned)lc * 16u;
  }
#pragma unroll
  for (int i = 0; i < LQ; ++i) {
    const int r = rb + i * RSTEP;
    qoff[i] = QBLK ? (unsigned)r * (unsigned)ROWB + (unsigned)lc * 16u
                   : (unsigned)r * (unsigned)a.ldq * 2u + (unsigned)lc * 16u;
  }

  unsigned xo[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) xo[ks] = (unsigned)((((ks << 1) | hi) ^ ((l32 >> 2) & 3)) * 16);
  const unsigned rd_p = (unsigned)((GATED ? wp * (FP / 2) * 32 : wp * FP * 32) + l32) * ROWB;
  const unsigned rd_q = (unsigned)(BP + wq * FQ * 32 + l32) * ROWB;
  auto p_frag_off = [](int f) -> unsigned {
    if (GATED) return (unsigned)((f < FP / 2 ? f * 32 : BP / 2 + (f - FP / 2) * 32) * ROWB);
    return (unsigned)(f * 32 * ROWB);
  };

  f32x16 acc[FP][FQ];
#pragma unroll
  for (int f = 0; f < FP; ++f)
#pragma unroll
    for (int g = 0; g < FQ; ++g)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[f][g][i] = 0.0f;

  // single tile of activation rows: every workgroup walks K from its own starting tile (see tiled_dma_kernel)
  const int rot = (tiles_q == 1 && nkt > 1) ? (int)(((unsigned)blockIdx.x * 2654435761u >> 12) % (unsigned)nkt) : 0;
  // DMA instructions lo..hi-1 (of NL per wave: weight rows first, then activation rows) of K tile `kt`.
  auto dma = [&](unsigned char* stage, int kt, auto lo_c, auto hi_c) {
    constexpr int LO = decltype(lo_c)::value, HI = decltype(hi_c)::value;
    int ktc = (kt < nkt ? kt : nkt - 1) + rot;  // past the end: re-read the last tile, never consumed
    if (ktc >= nkt) ktc -= nkt;
    const int kb = ktc * (BK * 2);
    const bool in = !KTAIL || (ktc * BK + lc * 8) < a.k;
#pragma unroll
    for (int i = LO; i < HI; ++i) {
      // blocked operands are zero padded in K: no tail predicate, and the K tile selects a whole block
      if (i < LP) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, (lds_void*)(stage + i * RSTEP * ROWB + wave * 1024), 16,
                                                 (int)((PBLK || in) ? poff[i] : OOB_OFFSET), PBLK ? ktc * PBLOCK : kb, 0,
                                                 0);
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, (lds_void*)(stage + (BP + (i - LP) * RSTEP) * ROWB + wave * 1024),
                                                 16, (int)((QBLK || in) ? qoff[i - LP] : OOB_OFFSET),
                                                 QBLK ? ktc * QBLOCK : kb, 0, 0);
      }
    }
  };
  auto dma_all = [&](unsigned char* stage, int kt) {
    dma(stage, kt, std::integral_constant<int, 0>{}, std::integral_constant<int, NL>{});
  };

  u32x4 pf[2][FP], qf[2][FQ];
  auto f_read = [&](int fb, const unsigned char* base, int ks) {
    pf[fb][0] = *(const u32x4*)(base + rd_p + p_frag_off(0) + xo[ks]);
#pragma unroll
    for (int g = 0; g < FQ; ++g) qf[fb][g] = *(const u32x4*)(base + rd_q + g * 32 * ROWB + xo[ks]);
#pragma unroll
    for (int f = 1; f < FP; ++f) pf[fb][f] = *(const u32x4*)(base + rd_p + p_frag_off(f) + xo[ks]);
  };
  auto mma = [&](int fb, int f_lo, int f_hi) {
#pragma unroll
    for (int f = f_lo; f < f_hi; ++f)
#pragma unroll
      for (int g = 0; g < FQ; ++g) acc[f][g] = E::mfma32(pf[fb][f], qf[fb][g], acc[f][g]);
  };

  constexpr int NM = FP * FQ;
  constexpr int NR = FP + FQ;
  constexpr int HF = FP / 2 > 0 ? FP / 2 : 1;
  constexpr int MPR = NM / NR > 0 ? NM / NR : 1;
  // The NL copies of a K tile are issued in three parts spread over the iteration (a burst fills the texture
  // addresser's queue and stalls the wave, and with it the MFMA stream): DA in step 0, DB in the first half of
  // step 1, DC after the barrier.
  constexpr int DA = NL / 2, DB = (NL - DA) / 2, DC = NL - DA - DB;
  using C0 = std::integral_constant<int, 0>;
  using CA = std::integral_constant<int, DA>;
  using CB = std::integral_constant<int, DA + DB>;
  using CN = std::integral_constant<int, NL>;
  // s_waitcnt vmcnt(VM) lgkmcnt(0): this wave's copy of the next tile has landed (everything younger stays in
  // flight: the NS-3 tiles after it and parts A and B of the one after those) and its own LDS reads are complete;
  // then the workgroup barrier publishes every wave's part.
  constexpr int VM = (NS - 3) * NL + DA + DB;
  static_assert(VM <= 63, "vmcnt is a 6-bit counter");
  constexpr int WAIT_IMM = (VM & 15) | ((VM >> 4) << 14) | (7 << 4) | (0 << 8);
  auto ring_barrier = [&]() {
    asm volatile("s_waitcnt %0\n\ts_barrier" ::"n"(WAIT_IMM) : "memory");
  };

  // One K tile: `cur` holds tile kt with its step-0 fragments already in pf[0]/qf[0]; `nxt` holds (or is about
  // to hold) tile kt+1; `fill` is the stage every wave finished reading before the previous barrier.
  auto iteration = [&](unsigned char* cur, unsigned char* nxt, unsigned char* fill, int kt) {
    dma(fill, kt + NS - 1, C0{}, CA{});
    f_read(1, cur, 1);
    mma(0, 0, FP);
    if constexpr (FP == 4 && FQ == 4 && DA == 4) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, MPR, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, (DA + NR - 1) / NR, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
    dma(fill, kt + NS - 1, CA{}, CB{});
    mma(1, 0, HF);
#pragma unroll
    for (int i = 0; i < DB; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, (HF * FQ) / (DB > 0 ? DB : 1), 0);
      __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
    }
    ring_barrier();
    f_read(0, nxt, 0);
    dma(fill, kt + NS - 1, CB{}, CN{});
    mma(1, HF, FP);
    constexpr int MC = (FP - HF) * FQ;  // MFMAs after the barrier
#pragma unroll
    for (int j = 0; j < (DC > 0 ? DC : 1); ++j) {
#pragma unroll
      for (int i = 0; i < MC / (DC > 0 ? DC : 1); ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, (NR + MC - 1) / MC, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x010, DC > 0 ? 1 : 0, 0);
    }
  };

  static_assert((NS - 2) * NL <= 63, "vmcnt is a 6-bit counter");
  if (nkt > 0) {
#pragma unroll
    for (int j = 0; j < NS - 1; ++j) dma_all(ring[j], j);
    // tile 0 landed, tiles 1 .. NS-2 pending
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NS - 2) * NL) : "memory");
    f_read(0, ring0, 0);
  }
  int kt = 0;
  for (; kt + NS - 1 < nkt; kt += NS) {
#pragma unroll
    for (int j = 0; j < NS; ++j) iteration(ring[j], ring[(j + 1) % NS], ring[(j + NS - 1) % NS], kt + j);
  }
#pragma unroll
  for (int j = 0; j < NS - 1; ++j) {
    if (kt < nkt) {
      iteration(ring[j], ring[(j + 1) % NS], ring[(j + NS - 1) % NS], kt);
      ++kt;
    }
  }

  if constexpr (OBLK) {
    store_tile_blocked<E, WP, WQ, FP, FQ>(acc, a, tp, tq, wp, wq, l32, hi);
  } else {
    store_tile<E, GATED, WP, WQ, FP, FQ>(acc, a, p0, q0, wp, wq, l32, hi);
  }
}

// ---- pair ring: row-major weights in whole cache lines, blocked activations ----------------------------------
// 256 x 256 tile, 4 waves of 128 x 128, K tiles of 32 as in tiled_ring_kernel, for a ROW-MAJOR weight operand and
// a panel-blocked activation operand. A row-major operand read 32 K elements at a time yields 64-byte requests,
// half a cache line each; here the weight operand is fetched in K PAIRS (64 elements = one 128-byte line per row)
// into a ring of three 32 KB pair slots, half a pair per iteration, while the activations keep a ring of four
// 16 KB stages. A pair is issued four to three iterations before its first tile is multiplied, an activation tile
// three iterations before. The slot/stage pattern repeats every 12 K tiles (lcm of 6 and 4), so the loop is unrolled
// twelvefold with every LDS address a compile-time constant. 160 KB of LDS. The workgroup barrier sits between the two
// K steps of a tile and the instruction order of each half is written out by hand (see half_iteration).
// LDS layouts: pair slot = [256 rows][128 B], chunk c of row r at position c ^ ((r >> 1) & 7); activation stage =
// [256 rows][64 B], chunk c at c ^ ((r >> 2) & 3) (both conflict-free for the operand reads, see the kernels above).
template <class E, bool GATED, bool KTAIL, bool OBLK>
__global__ void __launch_bounds__(256)
tiled_pair_kernel(const GemmArgs a, const int tiles_p, const int tiles_q, const int group) {
  constexpr int WP = 2, WQ = 2, FP = 4, FQ = 4;
  constexpr int BP = 256, BQ = 256;
  constexpr int PSLOT = BP * 128, QSTAGE = BQ * 64;
  constexpr int LPH = 4;  // weight copy instructions per wave per HALF pair (8 rows x 128 B each)
  constexpr int LQ = 4;   // activation copy instructions per wave per K tile (16 rows x 64 B each)
  constexpr int NL = LPH + LQ;
  static_assert(!OBLK || GATED, "only H is ever written blocked");

  __shared__ __align__(1024) unsigned char ps0[PSLOT];
  __shared__ __align__(1024) unsigned char ps1[PSLOT];
  __shared__ __align__(1024) unsigned char ps2[PSLOT];
  __shared__ __align__(1024) unsigned char qs0[QSTAGE];
  __shared__ __align__(1024) unsigned char qs1[QSTAGE];
  __shared__ __align__(1024) unsigned char qs2[QSTAGE];
  __shared__ __align__(1024) unsigned char qs3[QSTAGE];
  unsigned char* const ps[3] = {ps0, ps1, ps2};
  unsigned char* const qs[4] = {qs0, qs1, qs2, qs3};

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wq = wave % WQ;
  const int wp = wave / WQ;
  const int l32 = lane & 31;
  const int hi = lane >> 5;

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
  const unsigned char* pbase = (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const __amdgpu_buffer_rsrc_t prs = make_rsrc(pbase, ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  unsigned poff[2 * LPH];
#pragma unroll
  for (int j = 0; j < 2 * LPH; ++j) {
    const int r = rbp + j * 32;
    const int grow = GATED ? (r < BP / 2 ? 2 * r : 2 * (r - BP / 2) + 1) : r;
    poff[j] = (unsigned)grow * (unsigned)a.ldp * 2u + (unsigned)lcp * 16u;
  }
  // activation copy from the blocked panel: lane -> chunk position pcq of row rbq (+ 64 j)
  const int pcq = t & 3;
  const int rbq = t >> 2;
  const int lcq = pcq ^ ((rbq >> 2) & 3);
  const unsigned char* qbase = (const unsigned char*)a.Q + (long long)tq * nkt * QSTAGE;
  const __amdgpu_buffer_rsrc_t qrs = make_rsrc(qbase, (long long)nkt * QSTAGE);
  unsigned qoff[LQ];
#pragma unroll
  for (int j = 0; j < LQ; ++j) qoff[j] = (unsigned)(rbq + j * 64) * 64u + (unsigned)lcq * 16u;

  // operand fragment reads
  const unsigned rd_p = (unsigned)((GATED ? wp * (FP / 2) * 32 : wp * FP * 32) + l32) * 128u;
  const unsigned rd_q = (unsigned)(wq * FQ * 32 + l32) * 64u;
  unsigned xp[2][2], xq[2];  // [half of the pair][K step] / [K step]
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    xq[ks] = (unsigned)((((ks << 1) | hi) ^ ((l32 >> 2) & 3)) * 16);
#pragma unroll
    for (int h = 0; h < 2; ++h) xp[h][ks] = (unsigned)((((h << 2) | (ks << 1) | hi) ^ ((l32 >> 1) & 7)) * 16);
  }
  auto p_frag_off = [](int f) -> unsigned {
    if (GATED) return (unsigned)((f < FP / 2 ? f * 32 : BP / 2 + (f - FP / 2) * 32) * 128);
    return (unsigned)(f * 32 * 128);
  };

  f32x16 acc[FP][FQ];
#pragma unroll
  for (int f = 0; f < FP; ++f)
#pragma unroll
    for (int g = 0; g < FQ; ++g)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[f][g][i] = 0.0f;

  // copy instruction idx of iteration kt: 0..3 = half (kt & 1) of weight pair (kt >> 1) + 2, 4..7 = activation tile
  // kt + 3. Past the end both re-read the last pair / tile (never consumed).
  auto dma = [&](int kt, unsigned char* pslot, unsigned char* qstage, auto lo_c, auto hi_c) {
    constexpr int LO = decltype(lo_c)::value, HI = decltype(hi_c)::value;
    const int pair = (kt >> 1) + 2 < npair ? (kt >> 1) + 2 : npair - 1;
    const int half = kt & 1;
    const int qt = kt + 3 < nkt ? kt + 3 : nkt - 1;
    const bool in = !KTAIL || (pair * 64 + lcp * 8) < a.k;
#pragma unroll
    for (int i = LO; i < HI; ++i) {
      if (i < LPH) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, (lds_void*)(pslot + (half * LPH + i) * 32 * 128 + wave * 1024), 16,
                                                 (int)(in ? poff[half * LPH + i] : OOB_OFFSET), pair * 128, 0, 0);
      } else {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, (lds_void*)(qstage + (i - LPH) * 64 * 64 + wave * 1024), 16,
                                                 (int)qoff[i - LPH], qt * QSTAGE, 0, 0);
      }
    }
  };
  // prologue copies: a whole weight pair / one activation tile
  auto dma_pair = [&](int pair_, unsigned char* pslot, int j_lo, int j_hi) {
    const int pair = pair_ < npair ? pair_ : npair - 1;
    const bool in = !KTAIL || (pair * 64 + lcp * 8) < a.k;
#pragma unroll
    for (int j = 0; j < 2 * LPH; ++j)
      if (j >= j_lo && j < j_hi)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, (lds_void*)(pslot + j * 32 * 128 + wave * 1024), 16,
                                                 (int)(in ? poff[j] : OOB_OFFSET), pair * 128, 0, 0);
  };
  auto dma_q = [&](int qt_, unsigned char* qstage) {
    const int qt = qt_ < nkt ? qt_ : nkt - 1;
#pragma unroll
    for (int j = 0; j < LQ; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, (lds_void*)(qstage + j * 64 * 64 + wave * 1024), 16, (int)qoff[j],
                                               qt * QSTAGE, 0, 0);
  };

  u32x4 pf[2][FP], qf[2][FQ];
  using C0 = std::integral_constant<int, 0>;
  using CH = std::integral_constant<int, LPH>;
  // The barrier sits in the middle of the iteration, between the two K steps. At the barrier of iteration kt
  // everything issued up to iteration kt - 2 has landed (tile kt + 1 and its weight pair among it); the copies of
  // iteration kt - 1 and the first half of this one stay in flight. lgkmcnt(0): this wave's reads of tile kt are
  // complete (the last one was issued eight MFMAs earlier), so its stage may be refilled from the next iteration on.
  constexpr int VM = NL + LPH;
  constexpr int WAIT_IMM = (VM & 15) | ((VM >> 4) << 14) | (7 << 4) | (0 << 8);

  // One fragment read / one MFMA by index, for the hand-ordered halves below. Read order: P fragment 0, the FQ
  // activation fragments, then P fragments 1 .. FP-1: the order the MFMAs (f major, g minor) first need them.
  auto read_one = [&](int fb, int idx, const unsigned char* pslot, int half, const unsigned char* qstage, int ks) {
    if (idx == 0) {
      pf[fb][0] = *(const u32x4*)(pslot + rd_p + p_frag_off(0) + xp[half][ks]);
    } else if (idx <= FQ) {
      qf[fb][idx - 1] = *(const u32x4*)(qstage + rd_q + (idx - 1) * 32 * 64 + xq[ks]);
    } else {
      pf[fb][idx - FQ] = *(const u32x4*)(pslot + rd_p + p_frag_off(idx - FQ) + xp[half][ks]);
    }
  };
  auto mma_one = [&](int fb, int i) {
    acc[i / FQ][i % FQ] = E::mfma32(pf[fb][i / FQ], qf[fb][i % FQ], acc[i / FQ][i % FQ]);
  };
  // Half an iteration: the 16 MFMAs of K step `ks_mma` with, between them, first the 8 fragment reads of the
  // following K step (one per MFMA) and then 4 copies (one per two MFMAs): at most one other instruction between two
  // MFMAs, in exactly this order (the scheduler is fenced after every group).
  auto half_iteration = [&](int fb_mma, int fb_rd, const unsigned char* pslot_rd, int half_rd,
                            const unsigned char* qstage_rd, int ks_rd, int kt, unsigned char* p_fill,
                            unsigned char* q_fill, auto lo_c) {
    constexpr int LO = decltype(lo_c)::value;
    static_assert(FP + FQ + 2 * LPH == FP * FQ && LPH == 4, "16 MFMAs = 8 read slots + 4 copy slots of two");
#pragma unroll
    for (int i = 0; i < FP + FQ; ++i) {
      mma_one(fb_mma, i);
      read_one(fb_rd, i, pslot_rd, half_rd, qstage_rd, ks_rd);
      __builtin_amdgcn_sched_barrier(0);
    }
    mma_one(fb_mma, FP + FQ + 0);
    mma_one(fb_mma, FP + FQ + 1);
    dma(kt, p_fill, q_fill, std::integral_constant<int, LO>{}, std::integral_constant<int, LO + 1>{});
    __builtin_amdgcn_sched_barrier(0);
    mma_one(fb_mma, FP + FQ + 2);
    mma_one(fb_mma, FP + FQ + 3);
    dma(kt, p_fill, q_fill, std::integral_constant<int, LO + 1>{}, std::integral_constant<int, LO + 2>{});
    __builtin_amdgcn_sched_barrier(0);
    mma_one(fb_mma, FP + FQ + 4);
    mma_one(fb_mma, FP + FQ + 5);
    dma(kt, p_fill, q_fill, std::integral_constant<int, LO + 2>{}, std::integral_constant<int, LO + 3>{});
    __builtin_amdgcn_sched_barrier(0);
    mma_one(fb_mma, FP + FQ + 6);
    mma_one(fb_mma, FP + FQ + 7);
    dma(kt, p_fill, q_fill, std::integral_constant<int, LO + 3>{}, std::integral_constant<int, LO + 4>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  // iteration j (mod 12) of the unrolled loop, K tile kt = base + j
  auto iteration = [&](auto j_c, int kt) {
    constexpr int J = decltype(j_c)::value;
    unsigned char* const p_cur = ps[(J >> 1) % 3];
    unsigned char* const p_nxt = ps[((J + 1) >> 1) % 3];
    unsigned char* const p_fill = ps[((J >> 1) + 2) % 3];
    unsigned char* const q_cur = qs[J & 3];
    unsigned char* const q_nxt = qs[(J + 1) & 3];
    unsigned char* const q_fill = qs[(J + 3) & 3];
    half_iteration(0, 1, p_cur, J & 1, q_cur, 1, kt, p_fill, q_fill, C0{});
    asm volatile("s_waitcnt %0\n\ts_barrier" ::"n"(WAIT_IMM) : "memory");
    half_iteration(1, 0, p_nxt, (J + 1) & 1, q_nxt, 0, kt, p_fill, q_fill, CH{});
  };

  if (nkt > 0) {
    // fill in the order the loop would have issued it: [pair 0, tile 0] [pair 1 first half, tile 1] [pair 1 second
    // half, tile 2]; then pair 0 and tile 0 have landed when 16 copies are still in flight
    dma_pair(0, ps0, 0, 2 * LPH);
    dma_q(0, qs0);
    dma_pair(1, ps1, 0, LPH);
    dma_q(1, qs1);
    dma_pair(1, ps1, LPH, 2 * LPH);
    dma_q(2, qs2);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * NL) : "memory");
#pragma unroll
    for (int i = 0; i < FP + FQ; ++i) read_one(0, i, ps0, 0, qs0, 0);
  }
  int kt = 0;
  for (; kt + 11 < nkt; kt += 12) {
    iteration(std::integral_constant<int, 0>{}, kt);
    iteration(std::integral_constant<int, 1>{}, kt + 1);
    iteration(std::integral_constant<int, 2>{}, kt + 2);
    iteration(std::integral_constant<int, 3>{}, kt + 3);
    iteration(std::integral_constant<int, 4>{}, kt + 4);
    iteration(std::integral_constant<int, 5>{}, kt + 5);
    iteration(std::integral_constant<int, 6>{}, kt + 6);
    iteration(std::integral_constant<int, 7>{}, kt + 7);
    iteration(std::integral_constant<int, 8>{}, kt + 8);
    iteration(std::integral_constant<int, 9>{}, kt + 9);
    iteration(std::integral_constant<int, 10>{}, kt + 10);
    iteration(std::integral_constant<int, 11>{}, kt + 11);
  }
#define FSW_PAIR_TAIL(J)                                     \
  if (kt < nkt) {                                            \
    iteration(std::integral_constant<int, J>{}, kt);         \
    ++kt;                                                    \
  }
  FSW_PAIR_TAIL(0)
  FSW_PAIR_TAIL(1)
  FSW_PAIR_TAIL(2)
  FSW_PAIR_TAIL(3)
  FSW_PAIR_TAIL(4)
  FSW_PAIR_TAIL(5)
  FSW_PAIR_TAIL(6)
  FSW_PAIR_TAIL(7)
  FSW_PAIR_TAIL(8)
  FSW_PAIR_TAIL(9)
  FSW_PAIR_TAIL(10)
#undef FSW_PAIR_TAIL

  if constexpr (OBLK) {
    store_tile_blocked<E, WP, WQ, FP, FQ>(acc, a, tp, tq, wp, wq, l32, hi);
  } else {
    store_tile<E, GATED, WP, WQ, FP, FQ>(acc, a, p0, q0, wp, wq, l32, hi);
  }
}

// ---- row-major -> panel-blocked copy ---------------------------------------------------------------------------
// dst block (panel, kt) = [256 rows][64 bytes]: rows 256 panel .. 256 panel + 255 of src, K elements 32 kt .. 32 kt + 31;
// rows past `rows` and elements past `k` are written as zeros. A workgroup copies four K tiles of one panel: reads
// are 256 contiguous bytes per row (16 lanes), writes 1 KB contiguous per 16 rows of a block.
// gated_order (W13): block row r < 128 is source row 2r of the panel (the "up" row of feature r), block row
// r >= 128 is source row 2(r - 128) + 1 (its "gate" row): the order the gated kernel keeps a weight tile in LDS.
__global__ void __launch_bounds__(256)
block_rows_kernel(const unsigned short* __restrict__ src, long long ld, int rows, int k, unsigned char* __restrict__ dst,
                  int nkt, int gated_order) {
  const int t = threadIdx.x;
  const int c16 = t & 15;
  const int r0 = t >> 4;
  const int panel = blockIdx.y;
  const int kt = (int)blockIdx.x * 4 + (c16 >> 2);
  if (kt >= nkt) return;
  const int k0 = (int)blockIdx.x * 128 + c16 * 8;
  unsigned char* block = dst + ((long long)panel * nkt + kt) * (256 * 64) + (c16 & 3) * 16;
#pragma unroll 4
  for (int pass = 0; pass < 16; ++pass) {
    const int row = pass * 16 + r0;
    const int srow = gated_order ? (row < 128 ? 2 * row : 2 * (row - 128) + 1) : row;
    const long long gr = (long long)panel * 256 + srow;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (gr < rows && k0 < k) v = *(const u32x4*)(src + gr * ld + k0);
    *(u32x4*)(block + row * 64) = v;
  }
}

// ---- variant table ------------------------------------------------------------------------------------
namespace {

const TiledVariant kVariants[] = {
    {"tiled_256x256", 256, 256, 256},  // large-M prefill: 4 waves, 128x128 accumulators per wave
    {"tiled_256x128", 256, 128, 256},
    {"tiled_128x128", 128, 128, 256},
    {"tiled_256x64", 256, 64, 256},
    {"tiled_256x32", 256, 32, 256},
    {"dma_256x256", 256, 256, 256},    // direct-to-LDS copies, conflict-free operand reads
    {"dma_256x128", 256, 128, 256},
    {"dma_128x128", 128, 128, 256},
    {"ring_256x256", 256, 256, 256},   // four-stage LDS ring, K tiles of 32
    {"ring_256x128", 256, 128, 256},
    {"ring8w_256x256_a", 256, 256, 512},  // 8 waves (2 per SIMD), wave tile 128 x 64
    {"ring8w_256x256_b", 256, 256, 512},  // 8 waves, wave tile 64 x 128
    {"dma8w_256x256", 256, 256, 512},
    {"ring5_256x256", 256, 256, 256},  // five-stage ring: all 160 KB of LDS, four K tiles in flight
    {"ring5_256x192", 256, 192, 256},  // 192 activation rows: within 5 % of the default either way, not dispatched
    {"dma_128x256", 128, 256, 256},    // 129 .. 256 activation rows in ONE tile: every weight byte is read once
    {"dma_128x192", 128, 192, 256},    // the same for 129 .. 192 rows
    {"dma8w_128x256", 128, 256, 512},  // 128 x 256 on 8 waves (two per SIMD), wave tile 64 x 64
    {"dma_128x64", 128, 64, 256},      // up to 64 activation rows in one tile
};

int g_raster_group = 0;  // 0 = per-launch default
int g_pair_ring = 2;     // row-major weights of the blocked entry points: pair ring on 16x16x32 MFMAs (2, default),
                         // pair ring on 32x32x16 (1) or plain ring (0)

// Activation-row tiles per raster band. Measured on the headline shapes: the gate/up product (many weight
// panels, 4096-deep K) prefers 4, the down product (few weight panels, 14336-deep K) prefers 2.
}  // namespace
int raster_group(bool gated) { return g_raster_group > 0 ? g_raster_group : (gated ? 4 : 2); }
namespace {

template <class E, bool GATED, int WP, int WQ, int FP, int FQ>
hipError_t launch_one(const GemmArgs& a, hipStream_t stream) {
  constexpr int BP = WP * FP * 32, BQ = WQ * FQ * 32;
  const int tiles_p = (a.np + BP - 1) / BP;
  const int tiles_q = (a.nq + BQ - 1) / BQ;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  hipLaunchKernelGGL((tiled_kernel<E, GATED, WP, WQ, FP, FQ>), dim3((unsigned)(tiles_p * tiles_q)), dim3(WP * WQ * 64), 0,
                     stream, a, tiles_p, tiles_q, raster_group(GATED));
  return hipGetLastError();
}

// two-stage direct-to-LDS kernel; the 128 x 128 instance streams its weights non-temporally when at most two tiles
// of activation rows share them
template <class E, bool GATED, bool KTAIL, int WP, int WQ, int FP, int FQ>
void launch_dma_kernel(const dim3 grid, hipStream_t stream, const GemmArgs& a, int tiles_p, int tiles_q, int group) {
  if constexpr (WP == 2 && FP == 2 && ((WQ == 2 && FQ >= 1 && FQ <= 4) || (WQ == 4 && FQ == 2))) {  // 128 weight rows x 128 / 192 / 256 activation rows
    // a single tile of activation rows: three stages (see NS). They leave room for one workgroup per compute unit,
    // so 128 x 128 launches of more than 256 workgroups keep two stages and two workgroups (8192 x 57344 at 65 rows,
    // 448 workgroups: 168 -> 158 us)
    if (tiles_q == 1 && (WQ * FQ >= 6 || (long long)grid.x * grid.y <= 256)) {
      hipLaunchKernelGGL((tiled_dma_kernel<E, GATED, KTAIL, WP, WQ, FP, FQ, true, 3>), grid, dim3(WP * WQ * 64), 0, stream,
                         a, tiles_p, tiles_q, group);
      return;
    }
    if (tiles_q <= 2) {
      hipLaunchKernelGGL((tiled_dma_kernel<E, GATED, KTAIL, WP, WQ, FP, FQ, true>), grid, dim3(WP * WQ * 64), 0, stream,
                         a, tiles_p, tiles_q, group);
      return;
    }
  }
  hipLaunchKernelGGL((tiled_dma_kernel<E, GATED, KTAIL, WP, WQ, FP, FQ>), grid, dim3(WP * WQ * 64), 0, stream, a, tiles_p,
                     tiles_q, group);
}

template <class E, bool GATED, int WP, int WQ, int FP, int FQ>
hipError_t launch_dma(const GemmArgs& a, hipStream_t stream) {
  constexpr int BP = WP * FP * 32, BQ = WQ * FQ * 32;
  const int tiles_p = (a.np + BP - 1) / BP;
  const int tiles_q = (a.nq + BQ - 1) / BQ;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q));
  if (a.k % 64 == 0) {
    launch_dma_kernel<E, GATED, false, WP, WQ, FP, FQ>(grid, stream, a, tiles_p, tiles_q, raster_group(GATED));
  } else {
    launch_dma_kernel<E, GATED, true, WP, WQ, FP, FQ>(grid, stream, a, tiles_p, tiles_q, raster_group(GATED));
  }
  return hipGetLastError();
}

template <class E, bool GATED, int NS, int WP, int WQ, int FP, int FQ>
hipError_t launch_ring(const GemmArgs& a, hipStream_t stream) {
  constexpr int BP = WP * FP * 32, BQ = WQ * FQ * 32;
  const int tiles_p = (a.np + BP - 1) / BP;
  const int tiles_q = (a.nq + BQ - 1) / BQ;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  if (a.k % 32 == 0) {
    hipLaunchKernelGGL((tiled_ring_kernel<E, GATED, false, NS, WP, WQ, FP, FQ>), dim3((unsigned)(tiles_p * tiles_q)),
                       dim3(WP * WQ * 64), 0, stream, a, tiles_p, tiles_q, raster_group(GATED));
  } else {
    hipLaunchKernelGGL((tiled_ring_kernel<E, GATED, true, NS, WP, WQ, FP, FQ>), dim3((unsigned)(tiles_p * tiles_q)),
                       dim3(WP * WQ * 64), 0, stream, a, tiles_p, tiles_q, raster_group(GATED));
  }
  return hipGetLastError();
}

// 256 x 256 ring kernel with blocked operands / output (GemmArgs::layout, bits as in tiled_ring_kernel)
template <class E, bool GATED, int NS, int LAYOUT>
hipError_t launch_ring_layout(const GemmArgs& a, hipStream_t stream) {
  const int tiles_p = (a.np + 255) / 256;
  const int tiles_q = (a.nq + 255) / 256;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q)), block(256);
  if constexpr ((LAYOUT & 4) != 0) {  // a blocked weight operand is zero padded in K as well: no K tail anywhere
    hipLaunchKernelGGL((tiled_ring_kernel<E, GATED, false, NS, 2, 2, 4, 4, LAYOUT>), grid, block, 0, stream, a, tiles_p,
                       tiles_q, raster_group(GATED));
  } else if (a.k % 32 == 0) {
    hipLaunchKernelGGL((tiled_ring_kernel<E, GATED, false, NS, 2, 2, 4, 4, LAYOUT>), grid, block, 0, stream, a, tiles_p,
                       tiles_q, raster_group(GATED));
  } else {
    hipLaunchKernelGGL((tiled_ring_kernel<E, GATED, true, NS, 2, 2, 4, 4, LAYOUT>), grid, block, 0, stream, a, tiles_p,
                       tiles_q, raster_group(GATED));
  }
  return hipGetLastError();
}

// Q blocked, P row-major: the pair ring (FSW_PAIR_RING) or the plain ring with LAYOUT 1 / 3
template <class E, bool GATED, bool OBLK>
hipError_t launch_pair(const GemmArgs& a, hipStream_t stream) {
  const int tiles_p = (a.np + 255) / 256;
  const int tiles_q = (a.nq + 255) / 256;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q)), block(256);
  if (a.k % 64 == 0) {
    hipLaunchKernelGGL((tiled_pair_kernel<E, GATED, false, OBLK>), grid, block, 0, stream, a, tiles_p, tiles_q,
                       raster_group(GATED));
  } else {
    hipLaunchKernelGGL((tiled_pair_kernel<E, GATED, true, OBLK>), grid, block, 0, stream, a, tiles_p, tiles_q,
                       raster_group(GATED));
  }
  return hipGetLastError();
}

template <class E>
hipError_t launch_blocked_typed(bool gated, const GemmArgs& a, hipStream_t stream) {
  if (a.layout == 0) return hipErrorInvalidValue;  // row-major operands: launch_tiled / the 16x16x32 kernel
  if (g_pair_ring) {
    if (gated && a.layout == 1) return launch_pair<E, true, false>(a, stream);
    if (gated && a.layout == 3) return launch_pair<E, true, true>(a, stream);
    if (!gated && a.layout == 1) return launch_pair<E, false, false>(a, stream);
  }
  if (gated) {
    if (a.layout == 1) return launch_ring_layout<E, true, 5, 1>(a, stream);
    if (a.layout == 3) return launch_ring_layout<E, true, 5, 3>(a, stream);
    if (a.layout == 5) return launch_ring_layout<E, true, 5, 5>(a, stream);
    if (a.layout == 7) return launch_ring_layout<E, true, 5, 7>(a, stream);
  } else {
    if (a.layout == 1) return launch_ring_layout<E, false, 4, 1>(a, stream);
    if (a.layout == 5) return launch_ring_layout<E, false, 4, 5>(a, stream);
  }
  return hipErrorInvalidValue;
}

template <class E, bool GATED>
hipError_t launch_variant(int variant, const GemmArgs& a, hipStream_t stream) {
  switch (variant) {
    case 0: return launch_one<E, GATED, 2, 2, 4, 4>(a, stream);
    case 1: return launch_one<E, GATED, 2, 2, 4, 2>(a, stream);
    case 2: return launch_one<E, GATED, 2, 2, 2, 2>(a, stream);
    case 3: return launch_one<E, GATED, 4, 1, 2, 2>(a, stream);
    case 4: return launch_one<E, GATED, 4, 1, 2, 1>(a, stream);
    case 5: return launch_dma<E, GATED, 2, 2, 4, 4>(a, stream);
    case 6: return launch_dma<E, GATED, 2, 2, 4, 2>(a, stream);
    case 7: return launch_dma<E, GATED, 2, 2, 2, 2>(a, stream);
    case 8: return launch_ring<E, GATED, 4, 2, 2, 4, 4>(a, stream);
    case 9: return launch_ring<E, GATED, 4, 2, 2, 4, 2>(a, stream);
    case 10: return launch_ring<E, GATED, 4, 2, 4, 4, 2>(a, stream);
    case 11: return launch_ring<E, GATED, 4, 4, 2, 2, 4>(a, stream);
    case 12: return launch_dma<E, GATED, 2, 4, 4, 2>(a, stream);
    case 13: return launch_ring<E, GATED, 5, 2, 2, 4, 4>(a, stream);
    case 14: return launch_ring<E, GATED, 5, 2, 2, 4, 3>(a, stream);
    case 15: return launch_dma<E, GATED, 2, 2, 2, 4>(a, stream);
    case 16: return launch_dma<E, GATED, 2, 2, 2, 3>(a, stream);
    case 17: return launch_dma<E, GATED, 2, 4, 2, 2>(a, stream);
    case 18: return launch_dma<E, GATED, 2, 2, 2, 1>(a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

SplitPlan tiled_split_plan(int np, int nq, int k) {
  const long long t128 = (long long)((np + 127) / 128) * ((nq + 127) / 128);
  const long long t256 = (long long)((np + 255) / 256) * ((nq + 255) / 256);
  SplitPlan p = {256, 1};
  // One or two activation tiles with more large tiles than half the compute units: no split (see pick_tiled).
  // More rows: splitting can still pay by evening out rounds (288 tiles are two rounds of K, 288 x 3 are four
  // rounds of K / 3), up to 512 tiles.
  if (t128 <= 0 || t256 > (nq > 256 ? 512 : 128)) return p;
  int by_k;
  long long tiles;
  if (t128 < 256) {
    p.tile = 128;
    tiles = t128;
    by_k = k / 512;  // at least 8 K tiles of 64 per partition
  } else {
    tiles = t256;
    by_k = k / 1024;
  }
  if (nq > 256) {
    // Several tiles of activation rows: all workgroups should be resident at once (two 128 x 128 workgroups or one
    // 256 x 256 workgroup per compute unit: a second, partly filled round costs a whole one; 640 rows of 4096 x
    // 14336: 160 tiles x 3 splits 86 us, x 4 splits 110 us), and every split adds a partial tile to write and read
    // back. Estimated time per candidate, in us on 256 compute units: MFMA work of the busiest compute unit at
    // ~5.1 TFLOP/s (a lone 128 x 128 workgroup runs at half of that, the small tile costs ~15 % more per flop, the
    // large one on 16x16x32 MFMAs ~15 % less) plus the fp32 partials at ~5 TB/s. Measured against it (4096 x 14336):
    // 257 rows 128/5 59 us, 640 rows 128/3 85 us, 1024 rows 256/4 106 us, 2048 rows 256/2 185 us, each within 5 % of
    // the fastest of 12 tile/split pairs tried.
    // From 129 large tiles up the unsplit alternative is the 16x16x32 kernel on blocked H (~8 % faster than on
    // row-major H, which the split kernel reads): there only large-tile splits are candidates, over several rounds
    // if need be, they must win by 15 %, and their partials stay under 256 MB.
    const int nkt = (k + 63) / 64;
    const bool large = t256 >= 129;
    double best = 0.0, unsplit = 0.0;
    p.tile = 128;
    p.splits = 1;
    for (int c = large ? 1 : 0; c < 2; ++c) {
      const int tile = c == 0 ? 128 : 256;
      const long long nt = c == 0 ? t128 : t256;
      const long long slots = c == 0 ? 512 : 256;
      long long smax = large ? 16 : slots / nt;
      const long long deep = c == 0 ? k / 512 : k / 1024;  // at least 8 (16) K tiles of 64 per partition
      if (smax > deep) smax = deep;
      if (smax > 16) smax = 16;
      if (smax < 1) smax = 1;
      for (int sp = 1; sp <= (int)smax; ++sp) {
        if (sp > 1 && 4.0 * sp * (double)nq * (double)np > 256e6) break;
        const double kper = 64.0 * ((nkt + sp - 1) / sp);
        // a partly filled round of large tiles runs at a higher clock: 0.6 .. 0.95 of a full one (4096 x 14336:
        // 16 tiles 0.57, 144 tiles 0.80, 176 tiles 0.83 of the 310 us a round of 256 takes)
        const long long wgs = nt * sp;
        const double rounds = c == 0 ? (double)((wgs + slots - 1) / slots)
                                     : (double)(wgs / slots) + (wgs % slots ? 0.6 + 0.35 * (wgs % slots) / slots : 0.0);
        const double mfma = 2.0 * kper * tile * tile * (c == 0 ? 2.0 * 1.15 : 0.85) * rounds / 5.1e6;
        const double partials = sp > 1 ? 8.0 * sp * (double)nq * (double)np / 5.0e6 : 0.0;
        if (sp == 1 && c == 1) unsplit = mfma;
        if (best == 0.0 || mfma + partials < best) {
          best = mfma + partials;
          p.tile = tile;
          p.splits = sp;
        }
      }
    }
    if (large && p.splits > 1 && best > 0.85 * unsplit) p.splits = 1;
    if (p.splits == 1) p.tile = large ? 256 : 128;  // unsplit mid-size problems keep the smaller tile
    return p;
  }
  // One tile of activation rows: three-stage workgroups, one per compute unit, beat two two-stage ones (less
  // partial-sum traffic as well); 129..256 rows take one 128 x 256 tile per workgroup for the same reason.
  int target = 512;
  if (nq <= 128) {
    target = 256;
  } else if (nq <= 256) {
    // ... as long as that still fills most compute units (narrow outputs: 1024 x 2816 at 256 rows, 40 wide
    // workgroups 18.3 us, unsplit 128 x 128 tiles 21.4 us)
    const long long wide = (np + 127) / 128;
    long long sw = (256 + wide - 1) / wide;
    if (sw > by_k) sw = by_k;
    if (sw > 16) sw = 16;
    if (wide * sw >= 192) {
      p.tile = nq <= 192 ? 130 : 129;  // 128 x 192 does a quarter less MFMA work where 192 rows are enough
      tiles = wide;
      target = 256;
    }
  }
  // all workgroups resident at once: rounding up put 40 tiles x 7 splits on 256 one-workgroup compute units
  // (5120 x 13824 at 256 rows: 86 us, against 68 us at 257 rows)
  int splits = (int)(target / tiles);
  if (splits > by_k) splits = by_k;
  if (splits > 16) splits = 16;
  p.splits = splits < 1 ? 1 : splits;
  if (p.splits == 1 && p.tile == 256) p.tile = 128;  // unsplit mid-size problems keep the smaller tile
  return p;
}

namespace {
template <class E>
hipError_t launch_splitk_reduce(const GemmArgs& a, hipStream_t stream) {
  const long long work = (long long)a.nq * ((a.np + 3) / 4);
  hipLaunchKernelGGL((splitk_reduce_kernel<E>), dim3((unsigned)((work + 255) / 256)), dim3(256), 0, stream, a.partial,
                     a.splits, a.nq, a.np, (unsigned short*)a.O, a.ldo);
  return hipGetLastError();
}

template <class E, int WP, int WQ, int FP, int FQ>
hipError_t launch_splitk_one(const GemmArgs& a, hipStream_t stream) {
  constexpr int BP = WP * FP * 32, BQ = WQ * FQ * 32;
  const int tiles_p = (a.np + BP - 1) / BP;
  const int tiles_q = (a.nq + BQ - 1) / BQ;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q), (unsigned)a.splits);
  const int group = raster_group(false);
  if (a.k % 64 == 0) {
    launch_dma_kernel<E, false, false, WP, WQ, FP, FQ>(grid, stream, a, tiles_p, tiles_q, group);
  } else {
    launch_dma_kernel<E, false, true, WP, WQ, FP, FQ>(grid, stream, a, tiles_p, tiles_q, group);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || a.splits <= 1) return e;
  return launch_splitk_reduce<E>(a, stream);
}
}  // namespace

hipError_t launch_tiled_splitk(int dtype, int tile, const GemmArgs& a, hipStream_t stream) {
  if (tile == 128) {
    return dtype == 0 ? launch_splitk_one<Bf16, 2, 2, 2, 2>(a, stream) : launch_splitk_one<Fp16, 2, 2, 2, 2>(a, stream);
  }
  if (tile == 130) {  // 128 output features x 192 activation rows
    return dtype == 0 ? launch_splitk_one<Bf16, 2, 2, 2, 3>(a, stream) : launch_splitk_one<Fp16, 2, 2, 2, 3>(a, stream);
  }
  if (tile == 129) {  // 128 output features x 256 activation rows, 8 waves
    return dtype == 0 ? launch_splitk_one<Bf16, 2, 4, 2, 2>(a, stream) : launch_splitk_one<Fp16, 2, 4, 2, 2>(a, stream);
  }
  if (g_pair_ring == 2 && a.splits > 1) {  // 256 x 256 on the 16x16x32 kernel
    const hipError_t e = launch_pair16_splitk(dtype, a, stream);
    if (e != hipSuccess) return e;
    return dtype == 0 ? launch_splitk_reduce<Bf16>(a, stream) : launch_splitk_reduce<Fp16>(a, stream);
  }
  return dtype == 0 ? launch_splitk_one<Bf16, 2, 2, 4, 4>(a, stream) : launch_splitk_one<Fp16, 2, 2, 4, 4>(a, stream);
}

hipError_t launch_tiled_blocked(int dtype, bool gated, const GemmArgs& a, hipStream_t stream) {
  if (g_pair_ring == 2) return launch_pair16(dtype, gated, a, stream);
  return dtype == 0 ? launch_blocked_typed<Bf16>(gated, a, stream) : launch_blocked_typed<Fp16>(gated, a, stream);
}

hipError_t launch_block_rows(const void* src, long long ld, int rows, int k, void* dst, bool gated_order,
                             hipStream_t stream) {
  const int nkt = (k + 31) / 32;
  const int panels = (rows + 255) / 256;
  if (nkt <= 0 || panels <= 0) return hipSuccess;
  hipLaunchKernelGGL(block_rows_kernel, dim3((unsigned)((nkt + 3) / 4), (unsigned)panels), dim3(256), 0, stream,
                     (const unsigned short*)src, ld, rows, k, (unsigned char*)dst, nkt, gated_order ? 1 : 0);
  return hipGetLastError();
}

void set_raster_group(int g) { g_raster_group = g > 0 ? g : 0; }
void set_pair_ring(int mode) { g_pair_ring = mode < 0 || mode > 2 ? 2 : mode; }
int pair_ring_mode() { return g_pair_ring; }
int tiled_variant_count() { return (int)(sizeof(kVariants) / sizeof(kVariants[0])); }
const TiledVariant& tiled_variant(int variant) { return kVariants[variant]; }

hipError_t launch_tiled(int variant, int dtype, bool gated, const GemmArgs& a, hipStream_t stream) {
  if (dtype == 0) {
    return gated ? launch_variant<Bf16, true>(variant, a, stream) : launch_variant<Bf16, false>(variant, a, stream);
  }
  return gated ? launch_variant<Fp16, true>(variant, a, stream) : launch_variant<Fp16, false>(variant, a, stream);
}

}  // namespace fsw
