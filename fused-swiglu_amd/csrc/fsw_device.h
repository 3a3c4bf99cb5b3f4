// Device-side building blocks shared by the gfx950 kernels: element traits (MFMA + rounding), SiLU,
// raw-buffer loads with hardware bounds checking, and the XCD-aware tile rasteriser.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fsw {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

// bf16: v_mfma_f32_32x32x16_bf16 / v_mfma_f32_16x16x32_bf16, fp32 -> bf16 by v_cvt_pk_bf16_f32 (RNE, the
// rounding of cute::bfloat16_t(float) used at swiglu.cu:73-75).
struct Bf16 {
  static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  // The same instruction accumulating IN PLACE in accumulation registers ("+a": destination tied to the addend).
  // With 64 accumulator tiles live across an unrolled loop the register allocator does not always tie the builtin's
  // result to its addend and then moves accumulators between MFMAs; written out, the tie is part of the
  // instruction. The compiler does not see inside the statement: code that reads the accumulators with other
  // instructions afterwards must let the last MFMA drain first (mfma_drain).
  static __device__ __forceinline__ void mfma16_acc(f32x4& c, u32x4 a, u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(unsigned, v);
  }
  static __device__ __forceinline__ unsigned short cvt1(float x) {
    __bf16 v = (__bf16)x;
    return __builtin_bit_cast(unsigned short, v);
  }
};

// fp16: v_mfma_f32_32x32x16_f16 / v_mfma_f32_16x16x32_f16, fp32 -> fp16 by v_cvt_f16_f32 (RNE).
struct Fp16 {
  static __device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void mfma16_acc(f32x4& c, u32x4 a, u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
    f16x2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(unsigned, v);
  }
  static __device__ __forceinline__ unsigned short cvt1(float x) {
    _Float16 v = (_Float16)x;
    return __builtin_bit_cast(unsigned short, v);
  }
};

// Wait states between the last hand-written MFMA and the first other instruction that reads its accumulators
// (the longest requirement listed for matrix results read by vector instructions is 18).
__device__ __forceinline__ void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 7" ::: "memory"); }

// silu(x) = x / (1 + e^-x) (swiglu.cu:96) with v_exp_f32 (2^x) and v_rcp_f32; both are ~1 ulp fp32, far
// below the half-precision rounding applied afterwards. x -> -inf gives x * rcp(inf) = -0, no NaN for finite x.
__device__ __forceinline__ float silu_f32(float x) {
  float e = __builtin_amdgcn_exp2f(x * -1.4426950408889634f);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// Raw buffer descriptor over [base, base + bytes): loads whose byte offset falls outside return 0, which is
// how row tails (rows >= M / >= N) are zero-filled without branches.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, long long bytes) {
  if (bytes < 0) bytes = 0;
  if (bytes > 0x7fffffffLL) bytes = 0x7fffffffLL;  // tile-relative offsets stay far below 2 GiB
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0);
}
// Same load with the non-temporal cache policy: for weights that are read exactly once (decode). Measured on
// the M=16 forward: 7 % faster than the default policy, which lets 353 MB of single-use lines churn through
// the L2s and the 256 MB Infinity Cache and evict the activations that are reused.
__device__ __forceinline__ u32x4 buf_load16_stream(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
  return __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 2);
}
constexpr unsigned OOB_OFFSET = 0x80000000u;  // >= any num_records produced by make_rsrc

// Workgroup id -> tile coordinates. Hardware deals consecutive workgroup ids round-robin over the 8 XCDs
// (each with a private L2), so ids are first regrouped to give every XCD one contiguous run of logical tile
// ids, and logical ids walk the tile grid in bands of `group` activation-row tiles so that the ~32 tiles an
// XCD runs at once share a few X row panels and a few weight panels in that XCD's L2. (Same purpose as the
// threadblock swizzle at swiglu.cu:461-467, different mechanism.)
__device__ __forceinline__ void tile_coords(int bid, int tiles_p, int tiles_q, int group, int& tp, int& tq) {
  const int ntiles = tiles_p * tiles_q;
  const int per = (ntiles + 7) >> 3;
  int tall = ntiles & 7;
  if (tall == 0) tall = 8;
  const int xcd = bid & 7, loc = bid >> 3;
  const int id = (xcd < tall) ? xcd * per + loc : tall * per + (xcd - tall) * (per - 1) + loc;
  const int width = group * tiles_p;
  const int band = id / width;
  const int first_q = band * group;
  const int rows = (tiles_q - first_q < group) ? (tiles_q - first_q) : group;
  const int rem = id - band * width;
  tq = first_q + rem % rows;
  tp = rem / rows;
}

}  // namespace fsw
