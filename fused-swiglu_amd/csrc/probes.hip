// Two measurement kernels in a library of their own (libfsw_probe.so, include/fsw_probe.h; not part of the product
// library): what the matrix pipes and the memory system of THIS board sustain with nothing else in the way, measured
// in the same process as the product kernels.
// They are the yardsticks bench.py prints beside the roofline fractions (the published peaks assume a clock the
// board does not hold under a full MFMA load with random operands, and a read stream never sees the pin bandwidth).
// No counterpart in the reference.
#include <hip/hip_runtime.h>
#include <string.h>

#include "fsw.h"  // error codes only
#include "fsw_probe.h"
#include "fsw_device.h"

namespace fsw {

// Register-only loop of v_mfma_f32_16x16x32 in the shape the prefill kernel issues it: one wave per SIMD, 8 x 8
// accumulator blocks (256 accumulation registers), 16 operand fragments loaded once from `operands`
// (1024 x 16 bytes, the caller's data: random values give the data-dependent power draw of real inputs).
// iters x 64 MFMAs per wave, no memory traffic inside the loop.
template <class E>
__global__ void __launch_bounds__(256) probe_mfma_kernel(const u32x4* __restrict__ operands, float* __restrict__ out,
                                                         int iters) {
  u32x4 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = operands[(threadIdx.x + 64 * i) & 1023];
    b[i] = operands[(threadIdx.x * 3 + 17 * i + blockIdx.x) & 1023];
  }
  f32x4 acc[8][8];
#pragma unroll
  for (int f = 0; f < 8; ++f)
#pragma unroll
    for (int g = 0; g < 8; ++g) acc[f][g] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int f = 0; f < 8; ++f)
#pragma unroll
      for (int gg = 0; gg < 8; ++gg) {  // the prefill kernel's order: one operand changes per MFMA
        const int g = (f & 1) ? 7 - gg : gg;
        E::mfma16_acc(acc[f][g], a[f], b[g]);
      }
  }
  mfma_drain();
  float s = 0.f;
#pragma unroll
  for (int f = 0; f < 8; ++f)
#pragma unroll
    for (int g = 0; g < 8; ++g) s += acc[f][g][0] + acc[f][g][1] + acc[f][g][2] + acc[f][g][3];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Streaming read of `n16` 16-byte words with the non-temporal policy, four loads in flight per lane, grid-stride.
// Nothing is written unless the xor of all words is one particular value.
__global__ void __launch_bounds__(256) probe_read_kernel(const u32x4* __restrict__ p, size_t n16,
                                                         unsigned* __restrict__ out) {
  constexpr int U = 4;
  size_t i = (size_t)blockIdx.x * 256 * U + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256 * U;
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (; i + 256 * (U - 1) < n16; i += stride) {
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(p + i + 256 * u);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) out[0] = 1u;
}

}  // namespace fsw

namespace {
// the kernels are gfx950 code: anything else is refused before a launch
bool on_gfx950() {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return false;
  return strncmp(prop.gcnArchName, "gfx950", 6) == 0;
}
}  // namespace

extern "C" {

int fsw_probe_mfma(int dtype, int iters, const void* operands, void* out, int workgroups, void* stream) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (iters < 0 || workgroups < 1 || workgroups > 65536) return FSW_E_SHAPE;
  if (!operands || !out) return FSW_E_NULL;
  if (((uintptr_t)operands) & 15) return FSW_E_ALIGN;
  if (!on_gfx950()) return FSW_E_DEVICE;
  if (dtype == FSW_BF16) {
    hipLaunchKernelGGL((fsw::probe_mfma_kernel<fsw::Bf16>), dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const fsw::u32x4*)operands, (float*)out, iters);
  } else {
    hipLaunchKernelGGL((fsw::probe_mfma_kernel<fsw::Fp16>), dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                       (const fsw::u32x4*)operands, (float*)out, iters);
  }
  return hipGetLastError() == hipSuccess ? FSW_OK : FSW_E_LAUNCH;
}

int fsw_probe_read(const void* src, size_t bytes, void* out, int workgroups, void* stream) {
  if (!src || !out) return FSW_E_NULL;
  if ((((uintptr_t)src) & 15) || (bytes & 15)) return FSW_E_ALIGN;
  if (workgroups < 1 || workgroups > 65536) return FSW_E_SHAPE;
  if (!on_gfx950()) return FSW_E_DEVICE;
  hipLaunchKernelGGL(fsw::probe_read_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream,
                     (const fsw::u32x4*)src, bytes / 16, (unsigned*)out);
  return hipGetLastError() == hipSuccess ? FSW_OK : FSW_E_LAUNCH;
}

}  // extern "C"
