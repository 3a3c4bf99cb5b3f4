// LDS-tiled MFMA kernels (v_mfma_f32_32x32x16) for small and mid-size problems on gfx950, the split-K reduction and
// the row-major -> panel-blocked copy. The 256 x 256 prefill kernel lives in kernels_pair16.hip.
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
                                           int l32, int hi, int p_end) {
  unsigned short* O = (unsigned short*)a.O;
  const int nout = GATED ? p_end / 2 : p_end;  // p_end: first weight row this workgroup does not own
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
  const int step_p = (a.tile_p > 0 && a.tile_p < BP) ? a.tile_p : BP;  // weight rows this workgroup owns
  const int p0 = tp * step_p;
  const int p_end = p0 + step_p < a.np ? p0 + step_p : a.np;
  const int q0 = tq * BQ;
  if (GATED && blockIdx.x == 0 && blockIdx.y == 0)  // counters of the kernel that follows in fsw_mlp (GemmArgs::zero_words)
    for (int i = t; i < a.n_zero_words; i += NT) a.zero_words[i] = 0u;

  // ---- global -> LDS copy mapping: lane lands on chunk position pc of row rb (+ i * RSTEP)
  const int pc = t & 7;
  const int rb = t >> 3;
  const int lc = pc ^ ((rb >> 1) & 7);  // logical chunk this lane fetches (RSTEP % 16 == 0 keeps (row >> 1) & 7)
  const unsigned char* pbase = (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const unsigned char* qbase = (const unsigned char*)a.Q + (long long)q0 * a.ldq * 2;
  const __amdgpu_buffer_rsrc_t prs = make_rsrc(pbase, ((long long)(p_end - p0 - 1) * a.ldp + a.k) * 2);
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
    // This wave's copy of tile kt + 1 has landed (vmcnt) and its reads of `cur` are complete (lgkmcnt), then the
    // workgroup barrier publishes every wave's part. Written out: the fences of __syncthreads() need not wait for
    // vmcnt, and nothing else orders another wave's direct-to-LDS copy against this wave's reads after the barrier.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
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
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
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
  store_tile<E, GATED, WP, WQ, FP, FQ>(acc, a, p0, q0, wp, wq, l32, hi, p_end);
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
    {"dma_128x128", 128, 128, 256},    // two- or three-stage direct-to-LDS copies, 4 waves of 64 x 64
    {"dma_128x256", 128, 256, 256},    // 129 .. 256 activation rows in ONE tile: every weight byte is read once
    {"dma_128x192", 128, 192, 256},    // the same for 129 .. 192 rows
    {"dma8w_128x256", 128, 256, 512},  // 128 x 256 on 8 waves (two per SIMD), wave tile 64 x 64
    {"dma_128x64", 128, 64, 256},      // up to 64 activation rows in one tile
    {"pair16_256x256", 256, 256, 256}, // v_mfma_f32_16x16x32 prefill kernel (kernels_pair16.hip), row-major operands
};
constexpr int kPair16Variant = 5;

}  // namespace

// Activation-row tiles per raster band of the 256 x 256 kernel (the 128-row kernels above use 4 for the gate/up and
// 2 for the down product): 4, i.e. the 32 tiles an XCD runs at once are 4 activation panels x 8 weight
// panels (12 operand panels through its L2 per round). The down product of tall problems (32 activation tiles or
// more, 16 weight panels, 14336-deep K) measures level to 1 % slower that way and keeps bands of 2; with fewer
// activation tiles bands of 4 win (4096 x 4096 x 11008: 244 -> 236 us, 2048 x 8192 x 28672 fp16: 639 -> 633 us).
int raster_group(bool gated, int tiles_q) { return gated ? 4 : (tiles_q >= 32 ? 2 : 4); }

namespace {

// the 128-row instances stream their weights non-temporally when at most two tiles of activation rows share them
template <class E, bool GATED, bool KTAIL, int WP, int WQ, int FP, int FQ>
void launch_dma_kernel(const dim3 grid, hipStream_t stream, const GemmArgs& a, int tiles_p, int tiles_q, int group) {
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
  hipLaunchKernelGGL((tiled_dma_kernel<E, GATED, KTAIL, WP, WQ, FP, FQ>), grid, dim3(WP * WQ * 64), 0, stream, a, tiles_p,
                     tiles_q, group);
}

template <class E, bool GATED, int WP, int WQ, int FP, int FQ>
hipError_t launch_dma(const GemmArgs& a, hipStream_t stream) {
  constexpr int BP = WP * FP * 32, BQ = WQ * FQ * 32;
  const int step_p = (a.tile_p > 0 && a.tile_p < BP) ? a.tile_p : BP;
  const int tiles_p = (a.np + step_p - 1) / step_p;
  const int tiles_q = (a.nq + BQ - 1) / BQ;
  if (tiles_p <= 0 || tiles_q <= 0) return hipSuccess;
  const dim3 grid((unsigned)(tiles_p * tiles_q));
  if (a.k % 64 == 0) {
    launch_dma_kernel<E, GATED, false, WP, WQ, FP, FQ>(grid, stream, a, tiles_p, tiles_q, GATED ? 4 : 2);
  } else {
    launch_dma_kernel<E, GATED, true, WP, WQ, FP, FQ>(grid, stream, a, tiles_p, tiles_q, GATED ? 4 : 2);
  }
  return hipGetLastError();
}

template <class E, bool GATED>
hipError_t launch_variant(int variant, const GemmArgs& a, hipStream_t stream) {
  switch (variant) {
    case 0: return launch_dma<E, GATED, 2, 2, 2, 2>(a, stream);
    case 1: return launch_dma<E, GATED, 2, 2, 2, 4>(a, stream);
    case 2: return launch_dma<E, GATED, 2, 2, 2, 3>(a, stream);
    case 3: return launch_dma<E, GATED, 2, 4, 2, 2>(a, stream);
    case 4: return launch_dma<E, GATED, 2, 2, 2, 1>(a, stream);
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
  const int group = 2;
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
  // 256 x 256 on the 16x16x32 kernel, then the reduction
  const hipError_t e = launch_pair16_splitk(dtype, a, stream);
  if (e != hipSuccess || a.splits <= 1) return e;
  return dtype == 0 ? launch_splitk_reduce<Bf16>(a, stream) : launch_splitk_reduce<Fp16>(a, stream);
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

int tiled_variant_count() { return (int)(sizeof(kVariants) / sizeof(kVariants[0])); }
int pair16_variant() { return kPair16Variant; }
const TiledVariant& tiled_variant(int variant) { return kVariants[variant]; }

// row-major operands; the 256 x 256 variant is the 16x16x32 kernel with GemmArgs::layout 0
hipError_t launch_tiled(int variant, int dtype, bool gated, const GemmArgs& a, hipStream_t stream) {
  if (variant == kPair16Variant) return launch_pair16(dtype, gated, a, stream);
  if (dtype == 0) {
    return gated ? launch_variant<Bf16, true>(variant, a, stream) : launch_variant<Bf16, false>(variant, a, stream);
  }
  return gated ? launch_variant<Fp16, true>(variant, a, stream) : launch_variant<Fp16, false>(variant, a, stream);
}

}  // namespace fsw
