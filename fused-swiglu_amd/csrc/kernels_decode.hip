// Single-launch decode forward for at most 16 activation rows on gfx950: gate/up projection, a device-wide
// barrier, and the down projection in ONE persistent kernel (one 16-wave workgroup per CU).
//
// Why: at M = 16 the forward moves 353 MB of weights once; two back-to-back launches leave the GPU idle for
// ~6 us between them and each pays its own ramp-up and tail, which is 15-20 % of a ~60 us budget.
//
// Work split. Phase 1 walks tiles of 16 consecutive W13 rows (= 8 output features: even rows are "up", odd rows
// "gate", swiglu.cu:380-381), phase 2 tiles of 16 W2 rows; tile t belongs to workgroup t mod (number of
// workgroups). Inside a workgroup the 16 waves split K: wave w owns the same K slice of every tile, so its stream
// of 4 KB steps (16 rows x 256 B, 16 lanes per row, 16 B per lane) runs across tile boundaries with two steps in
// flight in registers. A step passes through the wave's private LDS slab (transpose to MFMA operand order, no
// barrier) and feeds v_mfma_f32_16x16x32 with weight rows as the A operand and activation rows (from L2) as the
// B operand. With the natural row order, accumulator registers 0/1 and 2/3 of a lane are up/gate of the same
// feature: gating is per-lane fp32 math. Per tile the 16 partial accumulators are summed through LDS.
//
// Device-wide barrier: arrive/depart counters in a file-scope __device__ array (zero at module load, restored to
// zero by the last workgroup to depart); the host hands concurrent launches different slots. Release/acquire at
// agent scope write back and invalidate the XCD-private L2s so that H written in phase 1 is read correctly by
// other XCDs in phase 2. The spin is bounded: if the workgroups are not all resident (someone else holds CUs)
// the kernel gives up, raises a flag the host checks on the next call, and exits instead of hanging.
#include "fsw_internal.h"
#include "fsw_device.h"

namespace fsw {

constexpr int DEC_NW = 16;           // waves per workgroup
constexpr int DEC_SLOTS = 64;        // barrier slots for concurrent launches
constexpr unsigned DEC_SPIN_LIMIT = 1u << 18;  // ~0.3 s of polling
static __device__ unsigned g_dec_barrier[DEC_SLOTS * 4];  // per slot: arrive, depart, failed, pad

template <class E, bool GATED>
__device__ __forceinline__ void decode_phase(const void* __restrict__ P, long long ldp, int np,
                                             const void* __restrict__ Q, long long ldq, int nq, int k,
                                             void* __restrict__ O, long long ldo, unsigned char* slab_all,
                                             float* part_all) {
  constexpr int KS = 128;
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int wg = blockIdx.x, nwg = gridDim.x;

  const int ntiles = (np + 15) >> 4;
  const int nt_mine = wg < ntiles ? (ntiles - wg + nwg - 1) / nwg : 0;
  const int nsteps = (k + KS - 1) / KS;
  const int per = (nsteps + DEC_NW - 1) / DEC_NW;
  const int s_begin = wave * per;
  const int s_cnt = (s_begin < nsteps) ? ((s_begin + per <= nsteps) ? per : nsteps - s_begin) : 0;
  const int nitems = nt_mine * s_cnt;

  const __amdgpu_buffer_rsrc_t prs = make_rsrc(P, ((long long)(np - 1) * ldp + k) * 2);
  const __amdgpu_buffer_rsrc_t qrs = make_rsrc(Q, ((long long)(nq - 1) * ldq + k) * 2);

  unsigned char* slab = slab_all + wave * 4096;
  const int pc = lane & 15;
  const unsigned wr = (unsigned)lane * 16u;
  unsigned rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd[kk] = (unsigned)r16 * 256u + (unsigned)(((4 * kk + q) ^ r16) * 16);
  const unsigned xoff = (unsigned)r16 * (unsigned)ldq * 2u + (unsigned)q * 16u;
  const unsigned row_bytes = (unsigned)ldp * 2u;

  u32x4 w0[4], w1[4], x0[4], x1[4];
  // loads of flattened item n (tile n / s_cnt, step s_begin + n % s_cnt): weights into w, activations into x
  // Items at or beyond nitems are issued too, with every offset redirected out of range (they read zeros and
  // touch no memory): the loop body then has no branch around a load, which lets the compiler count the loads
  // in flight exactly instead of waiting for all of them at every control-flow join.
  auto issue_w = [&](int n, u32x4 (&w)[4]) {
    const bool live = n < nitems;
    const int ti = n / s_cnt;
    const int step = s_begin + (n - ti * s_cnt);
    const int p0 = (wg + ti * nwg) << 4;
    const int k0 = step * KS;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 4 * i + (lane >> 4);
      const int lc = pc ^ row;  // slab chunk position pc of row `row` holds logical chunk pc ^ row (16 rows x 16 chunks)
      const bool in = live && (k0 + lc * 8) < k;
      const unsigned off = (unsigned)(p0 + row) * row_bytes + (unsigned)(k0 + lc * 8) * 2u;
      w[i] = buf_load16_stream(prs, in ? off : OOB_OFFSET);
    }
  };
  auto issue_x = [&](int n, u32x4 (&x)[4]) {
    const bool live = n < nitems;
    const int ti = n / s_cnt;
    const int k0 = (s_begin + (n - ti * s_cnt)) * KS;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const bool in = live && (k0 + kk * 32 + q * 8) < k;
      x[kk] = buf_load16(qrs, in ? xoff + (unsigned)(k0 + kk * 32) * 2u : OOB_OFFSET);
    }
  };

  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  int tiles_done = 0;
  // sum of the 16 partial accumulators of one tile, epilogue, store (wave 0 only, others go on streaming)
  auto finalize = [&](int ti) {
    float* part = part_all + (ti & 1) * (DEC_NW * 256);
    *(f32x4*)(part + ((wave * 64 + lane) << 2)) = acc;
    acc = f32x4{0.f, 0.f, 0.f, 0.f};
    // LDS-only barrier: __syncthreads() would also wait for the weight loads in flight (vmcnt(0)) and drain
    // the stream at every tile boundary
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (wave == 0) {
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
      for (int w = 0; w < DEC_NW; ++w) {
        const f32x4 v = *(const f32x4*)(part + ((w * 64 + lane) << 2));
        s[0] += v[0];
        s[1] += v[1];
        s[2] += v[2];
        s[3] += v[3];
      }
      const int p0 = (wg + ti * nwg) << 4;
      const int m = r16;
      if (m < nq) {
        unsigned short* orow = (unsigned short*)O + (long long)m * ldo;
        if (GATED) {
          const int n = (p0 >> 1) + 2 * q;  // rows 4q, 4q+1 -> feature p0/2 + 2q; rows 4q+2, 4q+3 -> the next one
          const int nout = np >> 1;
          const float h0 = s[0] * silu_f32(s[1]);
          const float h1 = s[2] * silu_f32(s[3]);
          if (((ldo & 1) == 0) && n + 1 < nout) {
            *(unsigned*)(orow + n) = E::pack2(h0, h1);
          } else {
            if (n < nout) orow[n] = E::cvt1(h0);
            if (n + 1 < nout) orow[n + 1] = E::cvt1(h1);
          }
        } else {
          const int n = p0 + 4 * q;
          if (((ldo & 3) == 0) && ((((uintptr_t)O) & 7) == 0) && n + 3 < np) {
            u32x2 pk = {E::pack2(s[0], s[1]), E::pack2(s[2], s[3])};
            *(u32x2*)(orow + n) = pk;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < np) orow[n + e] = E::cvt1(s[e]);
          }
        }
      }
    }
    ++tiles_done;
  };
  // registers -> slab frees w for the loads two items ahead; x is free again once the MFMAs have consumed it
  auto process = [&](int n, u32x4 (&w)[4], u32x4 (&x)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *(u32x4*)(slab + wr + i * 1024) = w[i];
    issue_w(n + 2, w);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const u32x4 wf = *(const u32x4*)(slab + rd[kk]);
      acc = E::mfma16(wf, x[kk], acc);
    }
    issue_x(n + 2, x);
    if (n < nitems && (n + 1) % s_cnt == 0) finalize(n / s_cnt);
  };

  if (nitems > 0) {  // s_cnt > 0 from here on
    issue_w(0, w0);
    issue_x(0, x0);
    issue_w(1, w1);
    issue_x(1, x1);
    for (int n = 0; n < nitems; n += 2) {
      process(n, w0, x0);
      process(n + 1, w1, x1);  // a dead item when nitems is odd: zero operands, no reduction
    }
  }
  // waves without a K slice still take part in every tile's reduction barrier
  while (tiles_done < nt_mine) finalize(tiles_done);
}

template <class E>
__global__ void __launch_bounds__(DEC_NW * 64)
decode_mlp_kernel(const DecodeArgs a, unsigned* bar) {
  __shared__ __align__(16) unsigned char slab[DEC_NW * 4096];
  __shared__ __align__(16) float part[2 * DEC_NW * 256];

  decode_phase<E, true>(a.W13, a.ldw13, 2 * a.ff, a.X, a.ldx, a.nq, a.d, a.H, a.ff, slab, part);

  // ---- device-wide barrier between the phases
  __syncthreads();  // every store of H by this workgroup has been issued and acknowledged
  if (threadIdx.x == 0) {
    __hip_atomic_fetch_add(bar + 0, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);  // writes back this XCD's L2
    unsigned spins = 0;
    // relaxed polling: an acquire load would invalidate the XCD's L2 on every iteration while other
    // workgroups are still streaming; one acquire fence after the barrier is enough
    while (__hip_atomic_load(bar + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < gridDim.x) {
      if (++spins > DEC_SPIN_LIMIT) {  // not all workgroups are resident: give up rather than hang
        __hip_atomic_store(bar + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(16);  // ~0.5 us between polls: 256 pollers must not load the counter's channel
    }
    // one acquire per workgroup: invalidates this CU's L1 and this XCD's L2 copies of lines other XCDs wrote
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    // depart: the last workgroup out restores the slot for the next launch that is handed it
    const unsigned left = __hip_atomic_fetch_add(bar + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (left == gridDim.x - 1) {
      __hip_atomic_store(bar + 0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(bar + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();

  decode_phase<E, false>(a.W2, a.ldw2, a.d, a.H, a.ff, a.nq, a.ff, a.Y, a.ldy, slab, part);
}

bool decode_mlp_supported(const DecodeArgs& a) {
  if (a.nq < 1 || a.nq > 16 || a.d < 8 || a.ff < 8) return false;
  // one buffer descriptor spans a whole matrix: byte offsets must stay below 2^31
  const long long lim = 0x7fffffffLL;
  if ((long long)2 * a.ff * a.ldw13 * 2 >= lim) return false;
  if ((long long)a.d * a.ldw2 * 2 >= lim) return false;
  return true;
}

hipError_t launch_decode_mlp(int dtype, const DecodeArgs& a, hipStream_t stream) {
  static int cu_count[64] = {0};
  static unsigned* bar_base[64] = {nullptr};
  static unsigned next_slot = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  if (cu_count[dev] == 0) {
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return e;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_dec_barrier));
    if (e != hipSuccess) return e;
    bar_base[dev] = (unsigned*)p;
    cu_count[dev] = prop.multiProcessorCount;
  }
  const unsigned slot = __atomic_fetch_add(&next_slot, 1u, __ATOMIC_RELAXED) % DEC_SLOTS;
  unsigned* bar = bar_base[dev] + slot * 4;
  const int tiles1 = (2 * a.ff + 15) / 16, tiles2 = (a.d + 15) / 16;
  int grid = cu_count[dev];  // one workgroup per CU: all resident at once, which the barrier relies on
  const int most = tiles1 > tiles2 ? tiles1 : tiles2;
  if (grid > most) grid = most;
  if (dtype == 0) {
    hipLaunchKernelGGL((decode_mlp_kernel<Bf16>), dim3((unsigned)grid), dim3(DEC_NW * 64), 0, stream, a, bar);
  } else {
    hipLaunchKernelGGL((decode_mlp_kernel<Fp16>), dim3((unsigned)grid), dim3(DEC_NW * 64), 0, stream, a, bar);
  }
  return hipGetLastError();
}

}  // namespace fsw
