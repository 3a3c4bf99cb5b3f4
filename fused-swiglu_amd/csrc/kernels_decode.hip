// Single-launch decode forward for at most 16 activation rows on gfx950: gate/up projection, a device-wide
// barrier, and the down projection in ONE persistent kernel (one 8-wave workgroup per CU, up to 256 VGPRs per lane).
//
// Why: at M = 16 the forward moves 353 MB of weights once; two back-to-back launches each pay a ramp-up and a
// tail, and the second cannot start fetching W2 before the first has drained. Here every wave has its first
// W2 steps in flight while the workgroups meet at the barrier, so the HBM stream does not stop between the
// projections.
//
// Work split. A workgroup owns a contiguous run of row tiles: in phase 1 tiles of 16 consecutive W13 rows (= 8
// output features: even rows are "up", odd rows "gate", swiglu.cu:380-381), in phase 2 tiles of 16 W2 rows. Its
// 8 waves split K: wave w owns the same K slice of every tile of the workgroup.
//   Phase 1: a wave keeps the activations of its K slice in registers (four 128-element steps at a time) and
//   streams the weight steps of up to 8 tiles past them into 8 accumulators (four steps in flight), so X is read
//   once per wave, not once per tile, and the 8 partial sums of all tiles are reduced through LDS once at the end.
//   Phase 2: one accumulator per tile, a register ring of 4 weight steps in flight (filled while waiting at the
//   barrier) and the matching H fragments (loaded after the barrier).
// A weight step is 16 rows x 256 B (16 lanes per row, 16 B per lane, non-temporal); it passes through the wave's
// private LDS slab (transpose to MFMA operand order, no barrier) and feeds v_mfma_f32_16x16x32 with weight rows
// as the A operand and activation rows as the B operand. With the natural W13 row order, accumulator registers
// 0/1 and 2/3 of a lane are up/gate of the same feature: gating is per-lane fp32 math.
// Loads past a wave's range are issued with an out-of-range offset (zero data, no memory traffic): the loops have
// no branch around a load, so the compiler counts the loads in flight exactly.
//
// Visibility of H across the eight XCD-private L2s without cache-wide write-back or invalidate: phase 1 stores H
// as relaxed agent-scope atomics (write-through to memory) and waits for their acknowledgement before arriving
// at the barrier; no L2 holds a copy of H's lines at that point (the dispatch invalidated the L2s and nothing in
// this kernel reads H before the barrier), so the plain loads of phase 2 miss and fetch the written data.
//
// Device-wide barrier: arrive/depart counters in a file-scope __device__ array (zero at module load, restored to
// zero by the last workgroup to depart). The host hands every single-launch forward a slot of its own and reuses a
// slot only when the event recorded behind its previous launch has completed; with no free slot, or on a stream
// that is being captured, the caller runs the two-launch path instead. The spin is bounded: if the workgroups are
// not all resident (someone else holds CUs) a workgroup gives up, writes the launch's own number (its epoch, unique
// per device) into the slot's `failed` word and SKIPS the down projection, as does every workgroup that reads its
// own epoch there after the barrier: a failed launch leaves Y incomplete and is counted in the slot's fourth word,
// which decode_barrier_failures() reports and clears; it never hangs and never multiplies a partial H. The mark
// belongs to the launch: a later launch that is handed the same slot carries another epoch and is not affected by
// a failure nobody has asked about yet.
#include <mutex>

#include "fsw_internal.h"
#include "fsw_device.h"

namespace fsw {

constexpr int DEC_NW = 8;            // waves per workgroup
constexpr int DEC_XS = 4;            // phase 1: K steps whose activations a wave holds at once = weight steps in flight
constexpr int DEC_TG = 8;            // phase 1: tiles (accumulators) per pass
constexpr int DEC_PF2 = 4;           // phase 2: weight steps in flight per wave
constexpr int DEC_POLL_SLEEP = 8;    // s_sleep between polls: 256 pollers must not saturate the counter's channel
constexpr int DEC_SLOTS = 64;        // barrier slots for launches in flight at the same time
constexpr unsigned DEC_SPIN_LIMIT = 1u << 18;  // ~0.3 s of polling
static __device__ unsigned g_dec_barrier[DEC_SLOTS * 4];  // per slot: arrive, depart, epoch of a failed launch, failures

// phases: bit 0 = gate/up, bit 1 = down; 3 = both with the device-wide barrier in between, which waits until
// `expected` workgroups have arrived (the grid size; a test passes more, so that the bounded wait gives up) for at
// most `spin_limit` polls.
template <class E>
__global__ void __launch_bounds__(DEC_NW * 64)
decode_mlp_kernel(const DecodeArgs a, unsigned* bar, const int phases, const unsigned expected,
                  const unsigned spin_limit, const unsigned epoch) {
  constexpr int KS = 128;
  // slabs of the waves first; the phase-1 reduction reuses everything, the phase-2 reduction has its own two
  // buffers behind the slabs
  constexpr int LDS_BYTES = (DEC_NW * DEC_TG * 1024 > 2 * DEC_NW * 4096 + 2 * DEC_NW * 1024) ? DEC_NW * DEC_TG * 1024
                                                                                            : 2 * DEC_NW * 4096 + 2 * DEC_NW * 1024;
  __shared__ __align__(16) unsigned char lds[LDS_BYTES];
  __shared__ unsigned barrier_failed;  // single launch: set by thread 0 when the device-wide barrier did not complete

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int r16 = lane & 15;
  const int q = lane >> 4;
  const int pc = lane & 15;
  const int wg = blockIdx.x, nwg = gridDim.x;
  unsigned char* slab = lds + wave * 4096;
  const unsigned wr = (unsigned)lane * 16u;
  unsigned rd[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) rd[kk] = (unsigned)r16 * 256u + (unsigned)(((4 * kk + q) ^ r16) * 16);

  // one weight step: rows row0 .. row0+15, K elements k0 .. k0+127; slab chunk position pc of row `row` holds
  // logical chunk pc ^ row (16 rows x 16 chunks). Per-lane parts of the address are loop constants (wl); the
  // tile's row offset is added per load, the K offset goes into the scalar offset. Validity never depends on
  // the scalar offset: rows past the matrix and dead items get an out-of-range vector offset, the K tail a
  // per-lane predicate.
  int lc8[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) lc8[i] = (pc ^ (4 * i + (lane >> 4))) * 8;
  auto lane_offsets = [&](unsigned row_bytes, unsigned (&wl)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) wl[i] = (unsigned)(4 * i + (lane >> 4)) * row_bytes + (unsigned)lc8[i] * 2u;
  };
  auto load_w = [&](__amdgpu_buffer_rsrc_t rs, const unsigned (&wl)[4], unsigned row_bytes, int row0, int k0, int kdim,
                    bool live, u32x4 (&w)[4]) {
    const unsigned rowpart = (unsigned)row0 * row_bytes;
    const int krem = live ? kdim - k0 : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned voff = lc8[i] < krem ? wl[i] + rowpart : OOB_OFFSET;
      w[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)voff, k0 * 2, 2);  // non-temporal: read exactly once
    }
  };
  // activation fragments of one step: lane -> row r16, K chunk q of each 32-element sub-step
  auto load_x = [&](__amdgpu_buffer_rsrc_t rs, unsigned xl, int k0, int kdim, bool live, u32x4 (&x)[4]) {
    const int krem = live ? kdim - k0 : 0;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const unsigned voff = (kk * 32 + q * 8) < krem ? xl : OOB_OFFSET;
      x[kk] = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)voff, k0 * 2 + kk * 64, 0);
    }
  };
  auto to_slab = [&](u32x4 (&w)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *(u32x4*)(slab + wr + i * 1024) = w[i];
  };
  // workgroup barrier that orders LDS only: __syncthreads() would also wait for the weight loads in flight
  auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  // ---------------------------------------------------------------- phase 1: H = (X Wu^T) * silu(X Wg^T)
  if (phases & 1) {
    const int np = 2 * a.ff, kdim = a.d;
    const int ntile = (np + 15) >> 4;
    const int tpw = (ntile + nwg - 1) / nwg;
    const int tile0 = wg * tpw;
    const int nsteps = (kdim + KS - 1) / KS;
    const int per = (nsteps + DEC_NW - 1) / DEC_NW;
    const int s_begin = wave * per;
    const __amdgpu_buffer_rsrc_t prs = make_rsrc(a.W13, ((long long)(np - 1) * a.ldw13 + kdim) * 2);
    const __amdgpu_buffer_rsrc_t qrs = make_rsrc(a.X, ((long long)(a.nq - 1) * a.ldx + kdim) * 2);
    const unsigned row_bytes = (unsigned)a.ldw13 * 2u;
    const unsigned xoff = (unsigned)r16 * (unsigned)a.ldx * 2u + (unsigned)q * 16u;
    unsigned wl[4];
    lane_offsets(row_bytes, wl);
    float* red = (float*)lds;  // [wave][tile][lane][4]

    for (int g0 = 0; g0 < tpw; g0 += DEC_TG) {
      f32x4 acc[DEC_TG];
#pragma unroll
      for (int i = 0; i < DEC_TG; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int kb = 0; kb < per; kb += DEC_XS) {
        u32x4 x[DEC_XS][4];
#pragma unroll
        for (int s = 0; s < DEC_XS; ++s) load_x(qrs, xoff, (s_begin + kb + s) * KS, kdim, kb + s < per, x[s]);
        // items: tile-major, step-minor; item idx uses ring slot idx % DEC_XS (= its step) and accumulator
        // idx / DEC_XS
        u32x4 w[DEC_XS][4];
        auto item_load = [&](int idx, u32x4 (&dst)[4]) {
          const int ti = idx / DEC_XS, s = idx % DEC_XS;
          const bool live = (g0 + ti < tpw) && (tile0 + g0 + ti < ntile) && (kb + s < per);
          load_w(prs, wl, row_bytes, (tile0 + g0 + ti) << 4, (s_begin + kb + s) * KS, kdim, live, dst);
        };
#pragma unroll
        for (int j = 0; j < DEC_XS; ++j) {
          item_load(j, w[j]);
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int idx = 0; idx < DEC_XS * DEC_TG; ++idx) {
          to_slab(w[idx % DEC_XS]);
          if (idx + DEC_XS < DEC_XS * DEC_TG) item_load(idx + DEC_XS, w[idx % DEC_XS]);
#pragma unroll
          for (int kk = 0; kk < 4; ++kk) {
            const u32x4 wf = *(const u32x4*)(slab + rd[kk]);
            acc[idx / DEC_XS] = E::mfma16(wf, x[idx % DEC_XS][kk], acc[idx / DEC_XS]);
          }
          __builtin_amdgcn_sched_barrier(0);  // keep the items apart: merged, they would drain the ring
        }
      }
      // sum of the 16 partial accumulators of every tile, gating, store
      __syncthreads();  // every wave is done with its slab
#pragma unroll
      for (int i = 0; i < DEC_TG; ++i) *(f32x4*)(red + (((wave * DEC_TG + i) * 64 + lane) << 2)) = acc[i];
      __syncthreads();
      if (wave < DEC_TG && g0 + wave < tpw && tile0 + g0 + wave < ntile) {
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
        for (int w2 = 0; w2 < DEC_NW; ++w2) {
          const f32x4 v = *(const f32x4*)(red + (((w2 * DEC_TG + wave) * 64 + lane) << 2));
          s[0] += v[0];
          s[1] += v[1];
          s[2] += v[2];
          s[3] += v[3];
        }
        const int p0 = (tile0 + g0 + wave) << 4;
        const int n = (p0 >> 1) + 2 * q;  // rows 4q, 4q+1 -> feature p0/2 + 2q; rows 4q+2, 4q+3 -> the next one
        const int nout = a.ff;
        if (r16 < a.nq && n < nout) {
          unsigned short* orow = (unsigned short*)a.H + (long long)r16 * a.ldh;
          const float h0 = s[0] * silu_f32(s[1]);
          const float h1 = s[2] * silu_f32(s[3]);
          // the single-launch forward requires the 4-byte path (decode_mlp_supported): its stores are write-through
          if (n + 1 < nout && ((a.ldh & 1) == 0) && ((((uintptr_t)a.H) & 3) == 0)) {
            __hip_atomic_store((unsigned*)(orow + n), E::pack2(h0, h1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          } else {
            orow[n] = E::cvt1(h0);
            if (n + 1 < nout) orow[n + 1] = E::cvt1(h1);
          }
        }
      }
      __syncthreads();  // the reduction buffer overlays the slabs
    }
  }

  // ---------------------------------------------------------------- phase 2 set-up and ring fill
  const int np2 = a.d, k2 = a.ff;
  const int ntile2 = (np2 + 15) >> 4;
  const int tpw2 = (ntile2 + nwg - 1) / nwg;
  const int tile0_2 = wg * tpw2;
  const int nsteps2 = (k2 + KS - 1) / KS;
  const int per2 = (nsteps2 + DEC_NW - 1) / DEC_NW;
  const int per2p = (per2 + DEC_PF2 - 1) / DEC_PF2 * DEC_PF2;  // a tile's steps padded to whole ring rounds
  const int nitems = tpw2 * per2p;  // the same for every wave of every workgroup
  const __amdgpu_buffer_rsrc_t w2rs = make_rsrc(a.W2, ((long long)(np2 - 1) * a.ldw2 + k2) * 2);
  const __amdgpu_buffer_rsrc_t hrs = make_rsrc(a.H, ((long long)(a.nq - 1) * a.ldh + k2) * 2);
  const unsigned row_bytes2 = (unsigned)a.ldw2 * 2u;
  // H steps are fetched like weight steps (16 lanes per row, whole cache lines) and transposed through a second
  // slab: fetched in operand order (lane = row), every 16-lane pass of a load touches 16 different cache lines,
  // 256 tag look-ups per step against 32, which cost a third of this phase.
  unsigned hl[4];
  lane_offsets((unsigned)a.ldh * 2u, hl);
  unsigned char* hslab = lds + (DEC_NW + wave) * 4096;
  unsigned wl2[4];
  lane_offsets(row_bytes2, wl2);
  // Both streams are consumed in item order, so each keeps a (tile, step) cursor instead of dividing the item
  // index: next_w / next_h load the cursor's item and advance it.
  int w_ti = 0, w_st = 0, h_ti = 0, h_st = 0;
  auto next_w = [&](u32x4 (&dst)[4]) {
    const bool live = (w_ti < tpw2) && (tile0_2 + w_ti < ntile2) && (w_st < per2);
    load_w(w2rs, wl2, row_bytes2, (tile0_2 + w_ti) << 4, (w_st * DEC_NW + wave) * KS, k2, live, dst);
    if (++w_st == per2p) {
      w_st = 0;
      ++w_ti;
    }
  };
  auto next_h = [&](u32x4 (&dst)[4]) {
    const int k0 = (h_st * DEC_NW + wave) * KS;
    const int krem = ((h_ti < tpw2) && (h_st < per2)) ? k2 - k0 : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      dst[i] = __builtin_amdgcn_raw_buffer_load_b128(hrs, (int)(lc8[i] < krem ? hl[i] : OOB_OFFSET), k0 * 2, 0);
    if (++h_st == per2p) {
      h_st = 0;
      ++h_ti;
    }
  };
  // ---------------------------------------------------------------- device-wide barrier and ring fill
  // Order: H stores acknowledged -> arrive -> fill the W2 ring -> wait for the others. A workgroup that finishes
  // phase 1 early spends its wait fetching W2; a late one arrives without waiting for its own ring.
  u32x4 w2[DEC_PF2][4];
  if (phases == 3) {
    // every store of H by this wave has been acknowledged by memory (written out: the fences of a workgroup
    // barrier need not wait for vmcnt), then every wave of the workgroup has got here
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (threadIdx.x == 0) __hip_atomic_fetch_add(bar + 0, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (phases & 2) {
#pragma unroll
    for (int j = 0; j < DEC_PF2; ++j) {
      next_w(w2[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  bool skip_down = false;
  if (phases == 3) {
    if (threadIdx.x == 0) {
      unsigned spins = 0, failed = 0;
      while (__hip_atomic_load(bar + 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < expected) {
        if (++spins > spin_limit) {  // not all workgroups are resident: give up rather than hang
          // mark the slot with this launch's epoch; the workgroup that changes the word counts the failure once
          if (__hip_atomic_exchange(bar + 2, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != epoch)
            __hip_atomic_fetch_add(bar + 3, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          failed = 1;
          break;
        }
        __builtin_amdgcn_s_sleep(DEC_POLL_SLEEP);
      }
      // a workgroup that got through still skips the down projection when another one has given up
      if (!failed) failed = __hip_atomic_load(bar + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == epoch ? 1u : 0u;
      barrier_failed = failed;
      // depart: the last workgroup out restores the slot for the next launch that is handed it
      const unsigned left = __hip_atomic_fetch_add(bar + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (left == gridDim.x - 1) {
        __hip_atomic_store(bar + 0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(bar + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    lds_barrier();  // no vmcnt wait: the ring stays in flight; also keeps loads of H below the barrier
    skip_down = barrier_failed != 0;
  }

  // ---------------------------------------------------------------- phase 2: Y = H W2^T
  if ((phases & 2) && !skip_down) {
    float* part_all = (float*)(lds + 2 * DEC_NW * 4096);  // two buffers of [wave][lane][4], by tile parity
    // H fragments ride the same ring distance as the weights and are issued before them: loads return in
    // order, so a younger, shorter H ring would make every step wait for the weight loads issued ahead of it
    u32x4 xh[DEC_PF2][4];
#pragma unroll
    for (int j = 0; j < DEC_PF2; ++j) {
      next_h(xh[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    f32x4 acc2 = {0.f, 0.f, 0.f, 0.f};
    int st_done = 0, ti_done = 0;
#pragma nounroll
    for (int i = 0; i < nitems; i += DEC_PF2) {
#pragma unroll
      for (int j = 0; j < DEC_PF2; ++j) {
        to_slab(w2[j]);
#pragma unroll
        for (int i2 = 0; i2 < 4; ++i2) *(u32x4*)(hslab + wr + i2 * 1024) = xh[j][i2];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const u32x4 wf = *(const u32x4*)(slab + rd[kk]);
          const u32x4 hf = *(const u32x4*)(hslab + rd[kk]);
          acc2 = E::mfma16(wf, hf, acc2);
        }
        next_h(xh[j]);
        next_w(w2[j]);
        __builtin_amdgcn_sched_barrier(0);
      }
      st_done += DEC_PF2;
      if (st_done == per2p) {  // a tile is complete (uniform over the workgroup)
        st_done = 0;
        const int tile = tile0_2 + ti_done;
        float* part = part_all + (ti_done & 1) * (DEC_NW * 256);
        ++ti_done;
        *(f32x4*)(part + ((wave * 64 + lane) << 2)) = acc2;
        acc2 = f32x4{0.f, 0.f, 0.f, 0.f};
        lds_barrier();
        if (wave == 0 && tile < ntile2) {
          f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
          for (int w = 0; w < DEC_NW; ++w) {
            const f32x4 v = *(const f32x4*)(part + ((w * 64 + lane) << 2));
            s[0] += v[0];
            s[1] += v[1];
            s[2] += v[2];
            s[3] += v[3];
          }
          const int n = (tile << 4) + 4 * q;
          if (r16 < a.nq) {
            unsigned short* orow = (unsigned short*)a.Y + (long long)r16 * a.ldy;
            if (((a.ldy & 3) == 0) && ((((uintptr_t)a.Y) & 7) == 0) && n + 3 < np2) {
              u32x2 pk = {E::pack2(s[0], s[1]), E::pack2(s[2], s[3])};
              *(u32x2*)(orow + n) = pk;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < np2) orow[n + e] = E::cvt1(s[e]);
            }
          }
        }
      }
    }
  }
}

bool decode_mlp_supported(const DecodeArgs& a, int phases) {
  if (a.nq < 1 || a.nq > 16 || a.d < 8 || a.ff < 1) return false;
  if ((phases & 2) && a.ff < 8) return false;
  // one launch for both phases: H must take the 4-byte write-through stores everywhere
  if (phases == 3 && ((a.ff & 1) || (a.ldh & 1) || (((uintptr_t)a.H) & 3))) return false;
  // one buffer descriptor spans a whole matrix and a partial last tile addresses up to 15 rows past it: byte
  // offsets must stay below 2^31
  const long long lim = 0x7fffffffLL;
  if ((phases & 1) && ((long long)2 * a.ff + 16) * a.ldw13 * 2 >= lim) return false;
  if ((phases & 2) && ((long long)a.d + 16) * a.ldw2 * 2 >= lim) return false;
  if ((phases & 2) && 16 * a.ldh * 2 >= lim) return false;
  return true;
}

namespace {

// per-device barrier slots of the single-launch forward
struct DecodeDevice {
  int cu_count = 0;
  unsigned* bar = nullptr;           // device address of g_dec_barrier on this device
  hipEvent_t done[DEC_SLOTS] = {};   // recorded behind the last launch that used the slot
  bool used[DEC_SLOTS] = {};
  unsigned next = 0;
  unsigned epoch = 0;                // number of the last single-launch forward on this device (never 0 in use)
};
std::mutex g_dec_mutex;
DecodeDevice g_dec_dev[64];

// device ordinal and its state, initialised on first use (under g_dec_mutex)
hipError_t decode_device(DecodeDevice*& out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= 64) return hipErrorInvalidDevice;
  DecodeDevice& d = g_dec_dev[dev];
  if (d.cu_count == 0) {
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return e;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_dec_barrier));
    if (e != hipSuccess) return e;
    d.bar = (unsigned*)p;
    d.cu_count = prop.multiProcessorCount;
  }
  out = &d;
  return hipSuccess;
}

}  // namespace

// phases 1 and 2 are plain launches. phases == 3 (one launch, device-wide barrier) needs a barrier slot that no
// launch in flight is using: *launched is set to false, and nothing is enqueued, when there is none or when `stream`
// is being captured (a replayed graph could run twice at once on one slot) -- the caller then runs two launches.
// test_unreachable: the barrier waits for one arrival more than the grid has and polls 64 times only, so that
// every workgroup takes the give-up path and the kernel still ends normally.
hipError_t launch_decode_mlp(int dtype, const DecodeArgs& a, hipStream_t stream, int phases, bool* launched,
                             bool test_unreachable) {
  if (launched) *launched = false;
  if (phases < 1 || phases > 3) return hipErrorInvalidValue;
  std::lock_guard<std::mutex> lock(g_dec_mutex);
  DecodeDevice* d = nullptr;
  hipError_t e = decode_device(d);
  if (e != hipSuccess) return e;
  const int tiles1 = (phases & 1) ? (2 * a.ff + 15) / 16 : 0, tiles2 = (phases & 2) ? (a.d + 15) / 16 : 0;
  int grid = d->cu_count;  // one workgroup per CU: all resident at once, which the barrier relies on
  const int most = tiles1 > tiles2 ? tiles1 : tiles2;
  if (grid > most) grid = most;
  int slot = -1;
  if (phases == 3) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    e = hipStreamIsCapturing(stream, &cap);
    if (e != hipSuccess) return e;
    if (cap != hipStreamCaptureStatusNone) return hipSuccess;
    for (int i = 0; i < DEC_SLOTS && slot < 0; ++i) {
      const int s = (int)((d->next + i) % DEC_SLOTS);
      if (!d->used[s]) {
        e = hipEventCreateWithFlags(&d->done[s], hipEventDisableTiming);
        if (e != hipSuccess) return e;
        slot = s;
      } else if (hipEventQuery(d->done[s]) == hipSuccess) {
        slot = s;
      }
    }
    (void)hipGetLastError();  // hipErrorNotReady of the queries is not an error of this call
    if (slot < 0) return hipSuccess;  // 64 single-launch forwards in flight
    d->used[slot] = true;
    d->next = (unsigned)slot + 1;
  }
  unsigned* bar = d->bar + (slot < 0 ? 0 : slot) * 4;
  unsigned epoch = 0;
  if (slot >= 0) {
    if (++d->epoch == 0) ++d->epoch;  // 0 is what an untouched slot holds
    epoch = d->epoch;
  }
  const unsigned expected = (unsigned)grid + (test_unreachable ? 1u : 0u);
  const unsigned spin_limit = test_unreachable ? 64u : DEC_SPIN_LIMIT;
  if (dtype == 0) {
    hipLaunchKernelGGL((decode_mlp_kernel<Bf16>), dim3((unsigned)grid), dim3(DEC_NW * 64), 0, stream, a, bar, phases,
                       expected, spin_limit, epoch);
  } else {
    hipLaunchKernelGGL((decode_mlp_kernel<Fp16>), dim3((unsigned)grid), dim3(DEC_NW * 64), 0, stream, a, bar, phases,
                       expected, spin_limit, epoch);
  }
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (launched) *launched = true;
  if (slot >= 0) e = hipEventRecord(d->done[slot], stream);
  return e;
}

// Number of single-launch forwards on the current device whose device-wide barrier gave up since the last call
// (their Y is incomplete); clears the marks. Synchronous copies: call it with no such forward in flight.
hipError_t decode_barrier_failures(int* count) {
  *count = 0;
  std::lock_guard<std::mutex> lock(g_dec_mutex);
  DecodeDevice* d = nullptr;
  hipError_t e = decode_device(d);
  if (e != hipSuccess) return e;
  unsigned host[DEC_SLOTS * 4];
  e = hipMemcpy(host, d->bar, sizeof(host), hipMemcpyDeviceToHost);
  if (e != hipSuccess) return e;
  const unsigned zero = 0;
  for (int s = 0; s < DEC_SLOTS; ++s) {
    if (host[s * 4 + 3] == 0) continue;
    *count += (int)host[s * 4 + 3];
    e = hipMemcpy(d->bar + s * 4 + 3, &zero, sizeof(zero), hipMemcpyHostToDevice);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace fsw
