// Weight-streaming kernels for the decode regime (at most 64 activation rows) on gfx950.
//
// With so few activation rows every weight byte is used once: the kernels are bound by HBM bandwidth, and the
// job is to keep ~100 KB of 16-byte loads in flight per CU with perfectly coalesced addresses.
//
// A workgroup owns one tile of 16 output features (16 weight rows; for the gated kernel the 16 "up" rows
// 2j and the 16 "gate" rows 2j+1, j in the tile) and its NW waves split K between them. Per step a wave
//   1. loads 128 K-elements (256 contiguous bytes) of each of its rows, 16 lanes per row, 16 bytes per lane
//      (each load instruction covers 4 rows x 256 B); the data of step s+1 is in flight while step s computes;
//   2. writes them to its private LDS slab and reads them back in MFMA operand order (lane = row, K chunk),
//      i.e. LDS is a per-wave transpose buffer: no barrier, LDS serves a wave's own accesses in order;
//   3. runs v_mfma_f32_16x16x32 with weight rows as the A operand and the (L2-resident) activation rows as
//      the B operand, so an accumulator lane owns activation row m = lane % 16 and 4 consecutive features.
// After the K loop the NW partial accumulators are summed through LDS (reusing the slabs) and the first MQ
// waves apply the epilogue (gating in fp32, one rounding) and store 8 bytes per lane.
//
// LDS slab layout: [row][16 chunks of 16 B]; chunk c of row r sits at position c ^ (r & 7), chosen by
// permuting which global chunk a lane fetches, so that the operand reads (16 rows at one logical chunk) hit
// every bank once per 8 lanes.
#include "fsw_internal.h"
#include "fsw_device.h"

namespace fsw {

template <class E, bool GATED, int MQ, int NW, bool XSLAB>
__global__ void __launch_bounds__(NW * 64)
skinny_kernel(const GemmArgs a) {
  constexpr int T = GATED ? 2 : 1;   // accumulator sets (up, gate)
  constexpr int R = 16 * T;          // weight rows per tile
  constexpr int NL = R / 4;          // weight loads per lane per step
  constexpr int KS = 128;            // K elements per step
  // Activations pass through the slab too: fetched like weights, 16 lanes per row, every 16-lane pass of a load
  // covers two whole cache lines; fetched in operand order (lane = row) every pass touches 16 lines, 256 tag
  // look-ups per 16-row step where 32 suffice. They go first (write, read back as fragments), then the weights
  // reuse the same bytes: LDS serves a wave's accesses in order. Measured on whole forwards at 4096 x 14336:
  // M = 16: 63.7 -> 61.0 us, M = 32: 85.8 -> 73.0, M = 64: 134.5 -> 98.1; with few activation rows the direct fetch
  // touches few lines per pass anyway (M = 3: 1.3 % faster, M = 8: level), so XSLAB is off for nq <= 8.
  constexpr int SLAB = R * 256;      // bytes of one wave's transpose buffer
  static_assert(MQ * T * 1024 <= SLAB, "the reduction reuses the slabs");
  __shared__ __align__(16) unsigned char lds[NW * SLAB];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int p0 = blockIdx.x * R;     // first weight row of the tile (interleaved numbering when gated)
  if (GATED && blockIdx.x == 0)      // counters of the kernel that follows in fsw_mlp (GemmArgs::zero_words)
    for (int i = t; i < a.n_zero_words; i += NW * 64) a.zero_words[i] = 0u;

  const unsigned char* pbase = (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const __amdgpu_buffer_rsrc_t prs = make_rsrc(pbase, ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  const __amdgpu_buffer_rsrc_t qrs = make_rsrc(a.Q, ((long long)(a.nq - 1) * a.ldq + a.k) * 2);

  // K partition: steps of KS, contiguous range per wave
  const int nsteps = (a.k + KS - 1) / KS;
  const int per = (nsteps + NW - 1) / NW;
  const int s_begin = wave * per;
  const int s_end = (s_begin + per < nsteps) ? s_begin + per : nsteps;

  // weight copy mapping: load i covers slab rows 4i .. 4i+3; lane -> (row, physical chunk), fetches logical chunk
  unsigned woff[NL];
  const int pc = lane & 15;
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int row = 4 * i + (lane >> 4);
    const int grow = GATED ? (row < 16 ? 2 * row : 2 * (row - 16) + 1) : row;
    const int lc = pc ^ (row & 7);
    woff[i] = (unsigned)grow * (unsigned)a.ldp * 2u + (unsigned)lc * 16u;
  }
  unsigned char* slab = lds + wave * SLAB;
  const unsigned wr = (unsigned)lane * 16u;   // + i * 1024

  // operand read mapping: set s (up / gate), K sub-step kk: row = 16 s + r16, logical chunk = 4 kk + q
  unsigned rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd[kk] = (unsigned)r16 * 256u + (unsigned)(((4 * kk + q) ^ (r16 & 7)) * 16);

  // activation fragments straight from global memory (L2 resident): lane -> row 16 mq + r16, K chunk q
  unsigned xoff[MQ];
#pragma unroll
  for (int mq = 0; mq < MQ; ++mq) xoff[mq] = (unsigned)(16 * mq + r16) * (unsigned)a.ldq * 2u + (unsigned)q * 16u;

  f32x4 acc[T][MQ];
#pragma unroll
  for (int s = 0; s < T; ++s)
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) acc[s][mq] = f32x4{0.f, 0.f, 0.f, 0.f};

  // coalesced activation mapping (XSLAB): load i covers rows 4i .. 4i+3 of the 16-row block, like the weights
  unsigned xoffc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 4 * i + (lane >> 4);
    xoffc[i] = (unsigned)row * (unsigned)a.ldq * 2u + (unsigned)(pc ^ (row & 7)) * 16u;
  }
  const unsigned xblock = 16u * (unsigned)a.ldq * 2u;  // bytes between 16-row activation blocks

  u32x4 wreg[NL];
  u32x4 xreg[MQ][4];
  auto g_load = [&](int step) {
    const int k0 = step * KS;
    const unsigned kb = (unsigned)k0 * 2u;
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int row = 4 * i + (lane >> 4);
      const int lc = pc ^ (row & 7);
      const bool in = (k0 + lc * 8) < a.k;
      wreg[i] = buf_load16_stream(prs, in ? woff[i] + kb : OOB_OFFSET);
    }
    if constexpr (XSLAB) {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = 4 * i + (lane >> 4);
          const int lc = pc ^ (row & 7);
          const bool in = (k0 + lc * 8) < a.k;
          xreg[mq][i] = buf_load16(qrs, in ? xoffc[i] + (unsigned)mq * xblock + kb : OOB_OFFSET);
        }
    } else {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const bool in = (k0 + kk * 32 + q * 8) < a.k;
          xreg[mq][kk] = buf_load16(qrs, in ? xoff[mq] + kb + (unsigned)kk * 64u : OOB_OFFSET);
        }
    }
  };

  if (s_begin < s_end) g_load(s_begin);
  for (int step = s_begin; step < s_end; ++step) {
    // registers -> slab (waits for this step's loads), then free the registers for the next step's loads
    u32x4 xcur[MQ][4];
    if constexpr (XSLAB) {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) {
#pragma unroll
        for (int i = 0; i < 4; ++i) *(u32x4*)(slab + wr + i * 1024) = xreg[mq][i];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) xcur[mq][kk] = *(const u32x4*)(slab + rd[kk]);
      }
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) *(u32x4*)(slab + wr + i * 1024) = wreg[i];
    if constexpr (!XSLAB) {
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) xcur[mq][kk] = xreg[mq][kk];
    }
    if (step + 1 < s_end) g_load(step + 1);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int s = 0; s < T; ++s) {
        const u32x4 wf = *(const u32x4*)(slab + s * 4096 + rd[kk]);
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq) acc[s][mq] = E::mfma16(wf, xcur[mq][kk], acc[s][mq]);
      }
    }
  }

  // ---- cross-wave reduction through LDS, then epilogue by the first MQ waves
  __syncthreads();  // every wave is done with its slab
  float* red = (float*)lds;  // [wave][s][mq][lane][4]
#pragma unroll
  for (int s = 0; s < T; ++s)
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq)
      *(f32x4*)(red + ((((wave * T + s) * MQ + mq) * 64 + lane) << 2)) = acc[s][mq];
  __syncthreads();
  if (wave < MQ) {
    const int mq = wave;
    f32x4 sum[T];
#pragma unroll
    for (int s = 0; s < T; ++s) {
      sum[s] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < NW; ++w) {
        const f32x4 v = *(const f32x4*)(red + ((((w * T + s) * MQ + mq) * 64 + lane) << 2));
        sum[s][0] += v[0];
        sum[s][1] += v[1];
        sum[s][2] += v[2];
        sum[s][3] += v[3];
      }
    }
    const int m = 16 * mq + r16;
    const int nout = GATED ? a.np / 2 : a.np;
    const int n = (GATED ? p0 / 2 : p0) + 4 * q;
    if (m < a.nq) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = GATED ? sum[0][e] * silu_f32(sum[T - 1][e]) : sum[0][e];
      if (GATED && a.out_f32) {  // H as float, unrounded
        float* orow32 = (float*)a.O + (long long)m * a.ldo;
        if (((a.ldo & 3) == 0) && ((((uintptr_t)a.O) & 15) == 0) && n + 3 < nout) {
          *(f32x4*)(orow32 + n) = f32x4{v[0], v[1], v[2], v[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < nout) orow32[n + e] = v[e];
        }
        return;
      }
      unsigned short* orow = (unsigned short*)a.O + (long long)m * a.ldo;
      const bool vec_ok = ((a.ldo & 3) == 0) && ((((uintptr_t)a.O) & 7) == 0);
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

namespace {

template <class E, bool GATED, int MQ, int NW>
hipError_t launch_skinny_one(const GemmArgs& a, hipStream_t stream) {
  constexpr int R = GATED ? 32 : 16;
  const int tiles = (a.np + R - 1) / R;
  if (tiles <= 0) return hipSuccess;
  if constexpr (MQ == 1) {
    if (a.nq <= 8) {
      hipLaunchKernelGGL((skinny_kernel<E, GATED, MQ, NW, false>), dim3((unsigned)tiles), dim3(NW * 64), 0, stream, a);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL((skinny_kernel<E, GATED, MQ, NW, true>), dim3((unsigned)tiles), dim3(NW * 64), 0, stream, a);
  return hipGetLastError();
}

template <class E, bool GATED, int MQ>
hipError_t launch_skinny_nw(int nw, const GemmArgs& a, hipStream_t stream) {
  if (nw == 4) return launch_skinny_one<E, GATED, MQ, 4>(a, stream);
  if constexpr (MQ == 1) {  // 16 waves leave 128 VGPRs per lane: enough for one activation tile only
    if (nw == 16) return launch_skinny_one<E, GATED, MQ, 16>(a, stream);
  }
  return launch_skinny_one<E, GATED, MQ, 8>(a, stream);
}

template <class E, bool GATED>
hipError_t launch_skinny_mq(int mq, int nw, const GemmArgs& a, hipStream_t stream) {
  switch (mq) {
    case 1: return launch_skinny_nw<E, GATED, 1>(nw, a, stream);
    case 2: return launch_skinny_nw<E, GATED, 2>(nw, a, stream);
    case 3: return launch_skinny_nw<E, GATED, 3>(nw, a, stream);
    case 4: return launch_skinny_nw<E, GATED, 4>(nw, a, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

// Waves per workgroup: enough waves in flight to cover HBM latency when there are few tiles, fewer (cheaper
// reduction, more workgroups per CU) when tiles are plentiful; never more waves than K steps.
SkinnyPlan skinny_plan(bool gated, int np, int nq, int k) {
  const int R = gated ? 32 : 16;
  const int tiles = (np + R - 1) / R;
  // measured on the M=16 down projection (256 tiles): 8 waves 25.8 us, 16 waves 27.2 us, 4 waves 28.4 us.
  // A register ring that keeps 2, 3, 4 or 6 steps of weight loads in flight per wave measured slower than the
  // one-step prefetch (27.5, 28.2, 29.2, 30.8 us): bytes in flight are not what limits this kernel.
  int nw = tiles <= 128 ? 16 : (tiles <= 640 ? 8 : 4);
  if (nq > 16 && nw > 8) nw = 8;
  const int nsteps = (k + 127) / 128;
  while (nw > 4 && nw > nsteps) nw >>= 1;
  SkinnyPlan p;
  p.splits = nw;
  p.workspace_bytes = 0;
  return p;
}

hipError_t launch_skinny(int dtype, bool gated, const GemmArgs& a, void* workspace, hipStream_t stream) {
  (void)workspace;
  if (a.nq > 64) return hipErrorInvalidValue;
  const int mq = (a.nq + 15) / 16;
  const int nw = skinny_plan(gated, a.np, a.nq, a.k).splits;
  if (dtype == 0) {
    return gated ? launch_skinny_mq<Bf16, true>(mq, nw, a, stream) : launch_skinny_mq<Bf16, false>(mq, nw, a, stream);
  }
  return gated ? launch_skinny_mq<Fp16, true>(mq, nw, a, stream) : launch_skinny_mq<Fp16, false>(mq, nw, a, stream);
}

}  // namespace fsw
