// Split-K weight-streaming kernel for the down projection of the decode regime (at most 32 activation rows) on
// gfx950: Y[m, n] = H[m, :] . W2[n, :] with every weight byte read once.
//
// Why another streaming kernel. skinny_kernel (kernels_skinny.hip) gives a workgroup 16 weight rows and the whole of
// K, so each of its workgroups reads ALL of H: for D = 4096 that is 256 workgroups x 458 KB = 117 MB of L2 -> CU
// traffic per 16 activation rows beside the 117 MB of weights, and its time grows with the rows (4096 x 14336:
// 18.3 us at one row, 21.4 us at 16, 27.5 us at 32). Here a workgroup owns 32 weight rows and ONE of S contiguous K
// ranges (blockIdx.y): the same number of workgroups for S = 2, half the H traffic.
//
// The S partial tiles of an output tile meet without a second launch and without waiting: a workgroup stores its
// fp32 partial sums write-through (agent-scope stores), waits for their acknowledgement and takes a ticket from the
// tile's counter (agent-scope atomic add). Whoever draws the last ticket re-reads all S partials in split order (its
// own included, so the summation order is fixed whatever the arrival order: the result is deterministic), rounds once
// and stores Y; it also puts the counter back to zero. Nobody spins, so the workgroups need not be resident together.
// The counters must be zero when the kernel starts: the gate/up kernel that runs before it in fsw_mlp zeroes them
// (GemmArgs::zero_words), which is why only fsw_mlp uses this kernel.
//
// Inside a workgroup: NW waves split the K range of the workgroup in contiguous runs of 128-element steps (256 bytes
// per row); every wave owns a ring of NS LDS stages filled by buffer_load ... lds, NS - 1 steps ahead (no staging
// registers, no ds_write; weights non-temporal). Stage layout: [32 weight rows][256 B] then [activation rows][256 B];
// chunk c (16 bytes) of row r sits at position c ^ (r & 15), applied on the global side of the copy (an LDS-DMA
// instruction writes lane i at base + 16 i, so a wave instruction fills 4 rows): the 16 rows an operand read touches
// at one logical chunk cover all 64 banks once. One __shared__ array per stage, each holding every wave's slab of that
// stage, and a loop unrolled NS-fold: the compiler tracks direct-to-LDS copies per array, so reads of the stage that
// has landed do not wait for the copies in flight into the others. Steps past a wave's range are issued with an
// out-of-range offset (zero data, no memory traffic) and multiplied like the others: the loop has no branch around a
// copy, the outstanding-copy count is the same in every iteration and the hand-written s_waitcnt is exact.
#include "fsw_internal.h"
#include "fsw_device.h"

namespace fsw {

typedef __attribute__((address_space(3))) void lds_void;

template <class E, int MQ, int NW, int NS>
__global__ void __launch_bounds__(NW * 64)
stream_split_kernel(const GemmArgs a, float* __restrict__ part, unsigned* __restrict__ tickets) {
  constexpr int T = 2;                  // 16-row weight blocks per tile
  constexpr int R = 16 * T;             // weight rows per tile
  constexpr int XR = 16 * MQ;           // activation rows (padded to whole MFMA blocks)
  constexpr int KS = 128;               // K elements per step
  constexpr int SLAB = (R + XR) * 256;  // bytes of one wave's part of a stage
  constexpr int NLW = R / 4, NLX = XR / 4, NL = NLW + NLX;  // copy instructions per step (4 rows each)
  static_assert(NS >= 2 && NS <= 4, "ring length");
  static_assert(NS * NW * SLAB <= 160 * 1024, "LDS budget of a gfx950 CU");
  static_assert((NS - 1) * NL <= 63, "vmcnt is a 6-bit counter");
  static_assert(T * MQ * 1024 <= SLAB, "the reduction reuses stage 0");
  static_assert(MQ <= NW, "one epilogue wave per activation block");

  __shared__ __align__(1024) unsigned char st0[NW * SLAB];
  __shared__ __align__(1024) unsigned char st1[NW * SLAB];
  __shared__ alignas(NS > 2 ? 1024 : 16) unsigned char st2[NS > 2 ? NW * SLAB : 16];
  __shared__ alignas(NS > 3 ? 1024 : 16) unsigned char st3[NS > 3 ? NW * SLAB : 16];
  __shared__ unsigned last_flag;
  unsigned char* const ring[4] = {st0, st1, st2, st3};

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);  // wave-uniform: LDS-DMA bases live in SGPRs
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int tile = blockIdx.x;
  const int split = blockIdx.y, nsplit = gridDim.y;
  const int p0 = tile * R;  // first weight row of the tile

  const unsigned char* pbase = (const unsigned char*)a.P + (long long)p0 * a.ldp * 2;
  const __amdgpu_buffer_rsrc_t prs = make_rsrc(pbase, ((long long)(a.np - p0 - 1) * a.ldp + a.k) * 2);
  const __amdgpu_buffer_rsrc_t qrs = make_rsrc(a.Q, ((long long)(a.nq - 1) * a.ldq + a.k) * 2);

  // K partition: steps of KS; a contiguous run per workgroup (split), inside it a contiguous run per wave
  const int nsteps = (a.k + KS - 1) / KS;
  const int per_wg = (nsteps + nsplit - 1) / nsplit;
  const int wg_begin = split * per_wg;
  const int wg_end = (wg_begin + per_wg < nsteps) ? wg_begin + per_wg : nsteps;
  const int per = (per_wg + NW - 1) / NW;
  const int s_begin = wg_begin + wave * per;
  const int s_end = (s_begin + per < wg_end) ? s_begin + per : wg_end;
  const int n = s_end > s_begin ? s_end - s_begin : 0;

  // copy mapping: instruction i fills slab rows 4i .. 4i+3; lane -> row 4i + q at chunk position r16, fetching the
  // logical chunk r16 ^ (row & 15) of that row
  unsigned woff[NLW], xoff[NLX];
  int wlc[NLW], xlc[NLX];
#pragma unroll
  for (int i = 0; i < NLW; ++i) {
    const int row = 4 * i + q;
    wlc[i] = (r16 ^ (row & 15)) * 8;
    woff[i] = (unsigned)row * (unsigned)a.ldp * 2u + (unsigned)wlc[i] * 2u;
  }
#pragma unroll
  for (int i = 0; i < NLX; ++i) {
    const int row = 4 * i + q;
    xlc[i] = (r16 ^ (row & 15)) * 8;
    xoff[i] = (unsigned)row * (unsigned)a.ldq * 2u + (unsigned)xlc[i] * 2u;
  }
  // copies of step `idx` of this wave (0-based within its range) into `stage`
  auto issue = [&](unsigned char* stage, int idx) {
    const int k0 = (s_begin + idx) * KS;
    const int krem = idx < n ? a.k - k0 : 0;  // past the range: everything out of range
    unsigned char* slab = stage + wave * SLAB;
#pragma unroll
    for (int i = 0; i < NLW; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(prs, (lds_void*)(slab + i * 1024), 16,
                                               (int)(wlc[i] < krem ? woff[i] : OOB_OFFSET), k0 * 2, 0, 2);  // non-temporal
#pragma unroll
    for (int i = 0; i < NLX; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(qrs, (lds_void*)(slab + R * 256 + i * 1024), 16,
                                               (int)(xlc[i] < krem ? xoff[i] : OOB_OFFSET), k0 * 2, 0, 0);
  };

  // operand reads: row r16 of a 16-row block, logical chunk 4 kk + q
  unsigned rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd[kk] = (unsigned)r16 * 256u + (unsigned)(((4 * kk + q) ^ r16) * 16);

  f32x4 acc[T][MQ];
#pragma unroll
  for (int s = 0; s < T; ++s)
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq) acc[s][mq] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto consume = [&](const unsigned char* stage) {
    const unsigned char* slab = stage + wave * SLAB;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      u32x4 xf[MQ];
#pragma unroll
      for (int mq = 0; mq < MQ; ++mq) xf[mq] = *(const u32x4*)(slab + R * 256 + mq * 4096 + rd[kk]);
#pragma unroll
      for (int s = 0; s < T; ++s) {
        const u32x4 wf = *(const u32x4*)(slab + s * 4096 + rd[kk]);
#pragma unroll
        for (int mq = 0; mq < MQ; ++mq) acc[s][mq] = E::mfma16(wf, xf[mq], acc[s][mq]);
      }
    }
  };

  // fill NS - 1 stages, then per step: refill the stage consumed last, wait for the oldest copy, multiply
#pragma unroll
  for (int j = 0; j < NS - 1; ++j) issue(ring[j], j);
  for (int base = 0; base < n; base += NS) {
#pragma unroll
    for (int j = 0; j < NS; ++j) {
      // the reads of the stage refilled here were consumed by the MFMAs of the previous step (program order)
      __builtin_amdgcn_sched_barrier(0);
      issue(ring[(j + NS - 1) % NS], base + j + NS - 1);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 1) * NL) : "memory");
      consume(ring[j]);
    }
  }

  // ---- cross-wave reduction through LDS: wave mq < MQ ends up with the workgroup's sums of activation block mq
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // no copy is still landing in any slab
  float* red = (float*)st0;  // [wave][s][mq][lane][4]
#pragma unroll
  for (int s = 0; s < T; ++s)
#pragma unroll
    for (int mq = 0; mq < MQ; ++mq)
      *(f32x4*)(red + ((((wave * T + s) * MQ + mq) * 64 + lane) << 2)) = acc[s][mq];
  __syncthreads();
  const int mq = wave;  // meaningful for wave < MQ
  f32x4 sum[T];
  if (wave < MQ) {
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
  }

  // ---- cross-workgroup reduction: partials write-through, a ticket per workgroup, the last one sums in split order
  if (nsplit > 1) {
    float* tile_part = part + (long long)tile * nsplit * (MQ * T * 256);
    if (wave < MQ) {
      unsigned* mine = (unsigned*)(tile_part + (split * MQ + mq) * (T * 256) + lane * 4);
#pragma unroll
      for (int s = 0; s < T; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float v = sum[s][e];  // a scalar copy: the bit cast of a vector ELEMENT reads the vector's first word
          __hip_atomic_store(mine + s * 256 + e, __builtin_bit_cast(unsigned, v), __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // every partial of this workgroup has been acknowledged by memory before the ticket is drawn.
    // The ordering between workgroups rests on three facts of this target, not on language-level fences: (i) the
    // agent-scope atomic stores above are written through to memory, and vmcnt reaches zero only when memory has
    // acknowledged them, so the ticket drawn below follows the partials; (ii) the agent-scope atomic loads of the
    // last workgroup are served by memory, never by a stale line of its own XCD's L2; (iii) a wave's memory
    // instructions issue in program order, and those loads sit behind the branch on the ticket. A release fence
    // and an acquire fence at agent scope would say the same in the language, but on this target they write the
    // whole L2 back and invalidate it: measured on a kernel of this family at 4096 x 14336, 23 -> 60 us. A later edit
    // that turns a partial store or load into a plain access breaks (i) or (ii) silently across the XCDs' L2s; the
    // bit-equality of repeated calls in the tests is what would show it.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (t == 0) {
      const unsigned ticket = __hip_atomic_fetch_add(tickets + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const unsigned last = ticket == (unsigned)nsplit - 1 ? 1u : 0u;
      if (last) __hip_atomic_store(tickets + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch
      last_flag = last;
    }
    __syncthreads();
    if (!last_flag) return;
    if (wave < MQ) {
#pragma unroll
      for (int s = 0; s < T; ++s) sum[s] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < nsplit; ++sp) {
        const unsigned* src = (const unsigned*)(tile_part + (sp * MQ + mq) * (T * 256) + lane * 4);
#pragma unroll
        for (int s = 0; s < T; ++s)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            sum[s][e] += __builtin_bit_cast(float, __hip_atomic_load(src + s * 256 + e, __ATOMIC_RELAXED,
                                                                     __HIP_MEMORY_SCOPE_AGENT));
      }
    }
  }

  // ---- epilogue: a lane owns activation row 16 mq + r16 and 4 consecutive features per weight block; one rounding
  if (wave < MQ) {
    const int m = 16 * mq + r16;
    if (m < a.nq) {
      unsigned short* orow = (unsigned short*)a.O + (long long)m * a.ldo;
      const bool vec_ok = ((a.ldo & 3) == 0) && ((((uintptr_t)a.O) & 7) == 0);
#pragma unroll
      for (int s = 0; s < T; ++s) {
        const int nn = p0 + 16 * s + 4 * q;
        if (vec_ok && nn + 3 < a.np) {
          u32x2 pk = {E::pack2(sum[s][0], sum[s][1]), E::pack2(sum[s][2], sum[s][3])};
          *(u32x2*)(orow + nn) = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (nn + e < a.np) orow[nn + e] = E::cvt1(sum[s][e]);
        }
      }
    }
  }
}

// Plan of the split-K streaming down projection: 32-row tiles, two K ranges. It pays where the 16-row kernel is bound
// by L2 delivery of H: enough weight rows that halving the workgroups' H reads matters, and a K deep enough to split.
StreamPlan stream_split_plan(int np, int nq, int k, bool forced) {
  StreamPlan p = {0, 0, 0, 0};
  if (nq < 1 || nq > 32 || np < 1 || k < 8) return p;
  // Measured at 4096 x 14336, whole forwards, 16-row kernel -> this one (us): 24 rows 63.3 -> 60.5, 32 rows 65.5 -> 62.1;
  // 16 rows 58.1 -> 58.5, 12 rows 56.7 -> 57.8, 9 rows 57.8 -> 59.6: up to 16 rows the three dependent round trips at the
  // end of a workgroup (partials acknowledged, ticket, partials read back) cost what the halved H traffic saves.
  if (!forced && (nq < 17 || np < 1024 || k < 2048)) return p;
  p.splits = 2;
  p.tiles = (np + 31) / 32;
  const int mq = (nq + 15) / 16;
  p.partial_bytes = (size_t)p.tiles * p.splits * mq * 2 * 1024;
  p.ticket_words = p.tiles;
  return p;
}

namespace {
template <class E>
hipError_t launch_stream_split_typed(const GemmArgs& a, const StreamPlan& p, float* part, unsigned* tickets,
                                     hipStream_t stream) {
  const dim3 grid((unsigned)p.tiles, (unsigned)p.splits);
  if (a.nq <= 16) {
    hipLaunchKernelGGL((stream_split_kernel<E, 1, 4, 3>), grid, dim3(256), 0, stream, a, part, tickets);
  } else {
    hipLaunchKernelGGL((stream_split_kernel<E, 2, 4, 2>), grid, dim3(256), 0, stream, a, part, tickets);
  }
  return hipGetLastError();
}
}  // namespace

// workspace: [partials: p.partial_bytes][tickets: p.ticket_words x 4 bytes, zero when the kernel starts]
hipError_t launch_stream_split(int dtype, const GemmArgs& a, const StreamPlan& p, void* workspace, hipStream_t stream) {
  if (p.splits < 2 || a.nq > 32) return hipErrorInvalidValue;
  float* part = (float*)workspace;
  unsigned* tickets = (unsigned*)((unsigned char*)workspace + p.partial_bytes);
  return dtype == 0 ? launch_stream_split_typed<Bf16>(a, p, part, tickets, stream)
                    : launch_stream_split_typed<Fp16>(a, p, part, tickets, stream);
}

}  // namespace fsw
