// C-ABI dispatcher: argument validation (host only), regime selection by activation-row count, launches.
// Replaces the host launcher swiglu_fwd<TA,TB,TC> (swiglu.cu:397-525) and the convenience op's shape
// derivation (swiglu.cu:538-553); the public contract is include/fsw.h.
#include <hip/hip_runtime.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>

#include "fsw.h"
#include "fsw_internal.h"

namespace {

thread_local int g_last_hip_error = 0;
// Kernel override of fsw_set_variant, per calling thread: a thread's workspace queries and launches always agree,
// and no thread can change another's kernel choice. family 0 = gate/up, 1 = down.
thread_local int g_forced_variant[2] = {-1, -1};

constexpr int VARIANT_SKINNY = 100;          // id of the weight-streaming kernel in fsw_set_variant
constexpr int VARIANT_DECODE_STREAM = 102;   // M <= 16: the streaming kernel of kernels_decode.hip, one phase per launch
constexpr int VARIANT_DECODE_FUSED = 101;    // fsw_mlp only: single-launch decode forward (family 0)
constexpr int VARIANT_DECODE_FUSED_FAIL = 103;  // 101 with a device-wide barrier that cannot complete (failure-path test)
constexpr int VARIANT_STREAM_SPLIT = 104;    // family 1, fsw_mlp only: split-K streaming down projection for M <= 32
constexpr int64_t MAX_DIM = 1LL << 30;       // every size is cast to int inside the kernels
constexpr int64_t MAX_LD = 1LL << 21;        // keeps tile-relative byte offsets below 2^31

bool aligned16(const void* p) { return (((uintptr_t)p) & 15) == 0; }

// gfx950 check, cached per device ordinal.
int check_device() {
  static std::atomic<int> ok_mask[64];  // 0 unknown, 1 ok, 2 not gfx950 (zero-initialised; racing writers agree)
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return FSW_E_DEVICE;
  }
  if (dev < 0 || dev >= 64) return FSW_E_DEVICE;
  int state = ok_mask[dev].load(std::memory_order_relaxed);
  if (state == 0) {
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) {
      g_last_hip_error = (int)e;
      return FSW_E_DEVICE;
    }
    state = (strncmp(prop.gcnArchName, "gfx950", 6) == 0) ? 1 : 2;
    ok_mask[dev].store(state, std::memory_order_relaxed);
  }
  return state == 1 ? FSW_OK : FSW_E_DEVICE;
}

// indices of the tiled kernels (tiled_variant() of kernels_tiled.hip)
constexpr int V_128x128 = 0, V_128x192 = 2, V_8W_128x256 = 3, V_128x64 = 4, V_256x256 = 5;

// Variant choice for the tiled kernels: the widest tile whose activation-row extent is not mostly padding,
// stepping down to 128x128 when a 256-wide grid would leave most of the 256 CUs idle.
int pick_tiled(int family, int64_t m, int64_t np) {
  const int64_t tiles256 = ((np + 255) / 256) * ((m + 255) / 256);
  // 256 x 256 tiles down to half-filled compute units. Below that the down product splits K (see
  // tiled_split_plan); between 129 and 191 tiles one large tile per compute unit beats 128 x 128 tiles in
  // 1.1 .. 1.4 rounds (down, 4096 x 14336, M = 2304 .. 2816: 250-260 us against 355-365 us; gate/up, 4096 x 22016,
  // M = 257 .. 512: 79-81 us against 95-102 us).
  // Up to 128 activation rows are one weight stream whatever the tile count (8192 x 57344, M = 65 .. 128: 173 us on
  // 128 x 128 tiles, 201-203 us on half-empty large ones).
  if (tiles256 < 129 || m <= 128) {
    // 128 x 128, direct-to-LDS (with split-K for the down product, see fsw_down). The gate/up product of 129 .. 256
    // activation rows takes them in ONE 128 x 256 tile, so that every weight byte is still read exactly once
    // (4096 x 28672: M = 160: 85 -> 64 us, M = 256: 86 -> 68 us; at M = 128 the 128 x 128 tile is faster, 50 vs 66),
    // provided those tiles still cover half the compute units (1024 x 5632 at M = 256: 44 of them, 18.5 us against
    // 10.5 us for 88 tiles of 128 x 128).
    // Up to 192 rows the tile is 128 x 192: the single-tile kernels are bound by their MFMA and LDS work as much as
    // by the weight stream (4096 x 28672, M = 160: 65 -> 54 us; 5120 x 27648: 89 -> 68 us).
    // 193 .. 256 rows: 128 x 256 on 8 waves, two per SIMD (4096 x 28672: 72 -> 64 us, 5120 x 27648: 94 -> 79-87 us
    // against the 4-wave instance, variant 15).
    if (family == 0 && m > 128 && m <= 256 && (np + 127) / 128 >= 128) return m <= 192 ? V_128x192 : V_8W_128x256;
    // up to 64 rows the gate/up tile is 128 x 64 (4096 x 28672, M = 48: 39.4 -> 37.2 us)
    return (family == 0 && m <= 64) ? V_128x64 : V_128x128;
  }
  if (family == 0 && tiles256 > 256 && tiles256 <= 512) {
    // A few large tiles more than compute units: the second round is nearly empty, while 128 x 128 tiles (two per
    // compute unit, ~1.3-1.7 x the time per output element) come in rounds a quarter as long. Per round of 256
    // workgroups: ~33 us against ~75-100 us at K = 4096; the small tile must win by 20 % to be taken. 4096 x 36864,
    // M = 300 (288 tiles): 151 -> 130 us; 4096 x 22016, M = 640 (258 tiles): 148 -> 119 us.
    const int64_t tiles128 = ((np + 127) / 128) * ((m + 127) / 128);
    if (((tiles128 + 255) / 256) * 44 < ((tiles256 + 255) / 256) * 100) return V_128x128;
  }
  return V_256x256;
}

// Most activation rows that still run the weight-streaming kernels (which take up to 64). Their time grows with
// the rows (each workgroup re-reads every activation row from the L2), the tiled kernels' hardly does, and the
// larger the weight matrices the earlier the tiled kernels win. Whole forwards, weight-streaming vs tiled, us:
// 2048 x 8192: M = 32 32.5 / 37.1, 48 39.4 / 39.7, 64 46.0 / 41.7; 4096 x 11008: M = 32 57.7 / 60.4, 40 65.5 / 62.7,
// 64 77.6 / 64.9; 4096 x 14336: M = 24 72.5 / 75.2, 32 75.3 / 70.4, 64 99.6 / 70.6; 8192 x 28672: M = 17 252.8 /
// 228.3, 64 370.5 / 242.5. K == 0 stays with the weight-streaming kernels, which write the all-zero result.
int64_t decode_rows(int family, int64_t np, int64_t k) {
  if (k <= 0) return 64;
  const int64_t d_ff = family == 0 ? (np / 2) * k : np * k;
  return d_ff < ((int64_t)1 << 25) ? 48 : d_ff < ((int64_t)1 << 27) ? 32 : 16;
}

// Weight rows per workgroup of the 128-row tiled kernels when ONE tile of activation rows streams the whole weight
// matrix (gate/up): cut into 128-row tiles a matrix of fewer than 256 x 128 rows leaves compute units idle, and one
// compute unit fetches at most ~29 GB/s, so the stream is cut into one piece per compute unit instead (a multiple of 8
// rows; the kernel's copies of the rows past its piece are out of range and cost no traffic). Gate/up alone, 128-row
// tiles -> pieces, us: 16384 rows (128 tiles -> 256 x 64) M = 64 33.8 -> 31.0, M = 128 41.1 -> 39.3; 22016 rows (172 ->
// 251 x 88) 36.1 -> 34.2, 43.4 -> 41.9; 27648 rows (216 -> 247 x 112) M = 16 47.0 -> 45.3, M = 64 52.0 -> 49.4, M = 128
// 62.6 -> 60.0. Not with 224 tiles or more (28672 rows: 35.2 -> 35.8, the pieces' wasted MFMA and LDS work costs more
// than the 32 idle compute units) and not above 128 activation rows, where the matrix cores are the limit (16384 rows,
// M = 256: 53.5 -> 56.2). 0 = the kernel's own tile height.
int stream_tile_rows(int variant, int64_t m, int64_t np) {
  if (!(variant == V_128x64 && m <= 64) && !(variant == V_128x128 && m <= 128)) return 0;
  if ((np + 127) / 128 > 216) return 0;
  const int64_t rows = ((np + 255) / 256 + 7) / 8 * 8;
  return (rows >= 64 && rows < 128) ? (int)rows : 0;
}

int resolve_variant(int family, int64_t m, int64_t np, int64_t k) {
  const int forced = g_forced_variant[family];
  if (forced == VARIANT_DECODE_FUSED || forced == VARIANT_DECODE_FUSED_FAIL || forced == VARIANT_DECODE_STREAM ||
      forced == VARIANT_STREAM_SPLIT)
    return m <= 64 ? VARIANT_SKINNY : pick_tiled(family, m, np);
  if (forced >= 0 && !(forced == VARIANT_SKINNY && m > 64)) return forced;
  if (m <= decode_rows(family, np, k)) {  // decode and small batches: weight streaming, HBM bound
    // The gate/up product streams its weights faster through the three-stage 128 x 64 tiled kernel (direct-to-LDS
    // copies) than through the weight-streaming kernel when its tiles of 128 weight rows fill one round of compute
    // units and there are a dozen rows or more (gate/up, us: 4096 x 28672: M = 16 37.9 -> 35.6, 32 43.3 -> 36.0, M = 1
    // level; 5120 x 27648: M = 16 49.3 -> 47.3, M = 4 45.3 -> 47.2; 172 tiles of 4096 x 22016: 28.8 -> 33.7, no).
    const int64_t tiles = (np + 127) / 128;
    if (family == 0 && m >= 12 && k > 0 && tiles >= 200 && tiles <= 256) return V_128x64;
    return VARIANT_SKINNY;
  }
  return pick_tiled(family, m, np);
}

// the weight-streaming kernels need no scratch and no blocked operands
bool streams_weights(int family, int64_t m, int64_t np, int64_t k) {
  return m <= 64 && resolve_variant(family, m, np, k) == VARIANT_SKINNY;
}

// M <= 16 with very large weight matrices runs on the persistent streaming kernel of kernels_decode.hip (one phase
// per launch) unless the caller forces the skinny kernel. Measured whole forwards at M = 16, skinny vs streaming:
// 8192 x 28672: 254 vs 233 us; 5120 x 13824: 87.6 vs 90.3; 4096 x 14336: 61.1 vs 63.4; 4096 x 11008: 50.0 vs 54.5;
// 2048 x 8192: 26.9 vs 31.6: the streaming kernel needs many tiles per CU to balance and to amortise its single
// reduction. K == 0 stays with the skinny kernel, which writes the all-zero result.
bool decode_stream_wanted(int family, int64_t m, int64_t rows, int64_t k) {
  if (m > 16 || k <= 0 || g_forced_variant[family] == VARIANT_SKINNY) return false;
  if (g_forced_variant[family] == VARIANT_DECODE_STREAM) return true;
  return rows * k >= (family == 0 ? (int64_t)1 << 28 : (int64_t)1 << 27);  // = d * ff >= 2^27 for either projection
}

int finish(hipError_t e) {
  if (e != hipSuccess) {
    g_last_hip_error = (int)e;
    return FSW_E_LAUNCH;
  }
  return FSW_OK;
}

}  // namespace

extern "C" {

int fsw_version(void) { return 2000; }

const char* fsw_strerror(int code) {
  switch (code) {
    case FSW_OK: return "ok";
    case FSW_E_NULL: return "fsw: a required pointer is NULL";
    case FSW_E_DTYPE: return "fsw: unsupported element type (expected bf16 or fp16)";
    case FSW_E_SHAPE: return "fsw: bad shape (negative size, odd N, or size out of range)";
    case FSW_E_LD: return "fsw: leading dimension smaller than the row it strides";
    case FSW_E_ALIGN: return "fsw: K/FF and leading dimensions must be multiples of 8 and inputs 16-byte aligned";
    case FSW_E_WORKSPACE: return "fsw: workspace missing or too small";
    case FSW_E_LAUNCH: return "fsw: the HIP runtime rejected the kernel launch";
    case FSW_E_DEVICE: return "fsw: the current device is not a gfx950 GPU";
    case FSW_E_VARIANT: return "fsw: unknown kernel variant";
    case FSW_E_STATIC_LIMIT: return "fsw: the problem needs more scratch than the library's static 64 MiB; use fsw_mlp";
    default: return "fsw: unknown error code";
  }
}

int fsw_last_hip_error(void) { return g_last_hip_error; }

int fsw_decode_barrier_failures(void) {
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  int count = 0;
  const int rc = finish(fsw::decode_barrier_failures(&count));
  return rc != FSW_OK ? rc : count;
}

int fsw_set_variant(int family, int variant) {
  if (family < 0 || family > 1) return FSW_E_VARIANT;
  // the barrier that cannot complete exists for the failure-path test only: refused unless the process's
  // environment holds FSW_TEST_HOOKS=1, so a caller cannot leave it set by accident and get forwards without Y
  if (variant == VARIANT_DECODE_FUSED_FAIL) {
    const char* hooks = getenv("FSW_TEST_HOOKS");
    if (!hooks || strcmp(hooks, "1") != 0) return FSW_E_VARIANT;
  }
  if (variant >= 0 && variant != VARIANT_SKINNY && variant != VARIANT_DECODE_STREAM &&
      !(family == 0 && (variant == VARIANT_DECODE_FUSED || variant == VARIANT_DECODE_FUSED_FAIL)) &&
      !(family == 1 && variant == VARIANT_STREAM_SPLIT) &&
      variant >= fsw::tiled_variant_count())
    return FSW_E_VARIANT;
  g_forced_variant[family] = variant < 0 ? -1 : variant;
  return FSW_OK;
}

static fsw::StreamPlan mlp_stream_plan(int64_t M, int64_t D, int64_t FF);

const char* fsw_variant_name(int family, int dtype, int64_t M, int64_t N_or_D, int64_t K_or_FF) {
  (void)dtype;
  if (family == 2) {  // the down projection as fsw_mlp runs it
    if (mlp_stream_plan(M, N_or_D, K_or_FF).splits > 1) return "stream_split";
    family = 1;
  }
  if (family < 0 || family > 1) return "invalid";
  const int v = resolve_variant(family, M, N_or_D, K_or_FF);
  if (v == VARIANT_SKINNY) return decode_stream_wanted(family, M, N_or_D, K_or_FF) ? "decode_stream" : "skinny";
  if (family == 1 && g_forced_variant[1] < 0 && M <= MAX_DIM && N_or_D > 0 && N_or_D <= MAX_DIM && K_or_FF > 0 &&
      K_or_FF <= MAX_DIM) {
    const fsw::SplitPlan plan = fsw::tiled_split_plan((int)N_or_D, (int)M, (int)K_or_FF);
    if (plan.splits > 1) {
      if (plan.tile == 128) return "splitk_dma_128x128";
      if (plan.tile == 129) return "splitk_dma_128x256";
      if (plan.tile == 130) return "splitk_dma_128x192";
      return "splitk_pair16_256x256";
    }
  }
  return fsw::tiled_variant(v).name;
}

int fsw_validate_gateup(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13,
                        int64_t ldw, const void* H, int64_t ldh) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (M < 0 || N < 0 || K < 0 || (N & 1)) return FSW_E_SHAPE;
  if (M > MAX_DIM || N > MAX_DIM || K > MAX_DIM) return FSW_E_SHAPE;
  if (M == 0 || N == 0) return FSW_OK;  // nothing to read or write
  if (!H || (K > 0 && (!X || !W13))) return FSW_E_NULL;  // K == 0: X and W13 are never read
  if (ldx < K || ldw < K || ldh < N / 2) return FSW_E_LD;
  if (ldx > MAX_LD || ldw > MAX_LD || ldh > MAX_DIM) return FSW_E_SHAPE;
  if ((((uintptr_t)H) & 1)) return FSW_E_ALIGN;
  if (K == 0) return FSW_OK;
  if ((K & 7) || (ldx & 7) || (ldw & 7)) return FSW_E_ALIGN;
  if (!aligned16(X) || !aligned16(W13)) return FSW_E_ALIGN;
  return FSW_OK;
}

int fsw_validate_down(int dtype, int64_t M, int64_t D, int64_t FF, const void* H, int64_t ldh, const void* W2,
                      int64_t ldw2, const void* Y, int64_t ldy) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (M < 0 || D < 0 || FF < 0) return FSW_E_SHAPE;
  if (M > MAX_DIM || D > MAX_DIM || FF > MAX_DIM) return FSW_E_SHAPE;
  if (M == 0 || D == 0) return FSW_OK;
  if (!Y || (FF > 0 && (!H || !W2))) return FSW_E_NULL;  // FF == 0: H and W2 are never read
  if (ldh < FF || ldw2 < FF || ldy < D) return FSW_E_LD;
  if (ldh > MAX_LD || ldw2 > MAX_LD || ldy > MAX_DIM) return FSW_E_SHAPE;
  if ((((uintptr_t)Y) & 1)) return FSW_E_ALIGN;
  if (FF == 0) return FSW_OK;
  if ((FF & 7) || (ldh & 7) || (ldw2 & 7)) return FSW_E_ALIGN;
  if (!aligned16(H) || !aligned16(W2)) return FSW_E_ALIGN;
  return FSW_OK;
}

// zero_words / n_zero_words: see GemmArgs (only the decode-regime kernels honour them; the caller checks that)
static int gateup_impl(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13,
                       int64_t ldw, void* H, int64_t ldh, void* stream, unsigned* zero_words, int n_zero_words) {
  const int rc = fsw_validate_gateup(dtype, M, N, K, X, ldx, W13, ldw, H, ldh);
  if (rc != FSW_OK) return rc;
  if (M == 0 || N == 0) return FSW_OK;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  fsw::GemmArgs a;
  a.P = W13;
  a.Q = X;
  a.O = H;
  a.ldp = ldw;
  a.ldq = ldx;
  a.ldo = ldh;
  a.np = (int)N;
  a.nq = (int)M;
  a.k = (int)K;
  a.zero_words = zero_words;
  a.n_zero_words = n_zero_words;
  const int v = resolve_variant(0, M, N, K);
  a.tile_p = stream_tile_rows(v, M, N);
  if (v == VARIANT_SKINNY) {
    if (decode_stream_wanted(0, M, N, K)) {  // at most 16 rows: one 8-wave workgroup per CU, X held in registers
      fsw::DecodeArgs da = {};
      da.X = X;
      da.W13 = W13;
      da.H = H;
      da.ldx = ldx;
      da.ldw13 = ldw;
      da.ldh = ldh;
      da.nq = (int)M;
      da.d = (int)K;
      da.ff = (int)(N / 2);
      if (fsw::decode_mlp_supported(da, 1)) return finish(fsw::launch_decode_mlp(dtype, da, (hipStream_t)stream, 1));
    }
    return finish(fsw::launch_skinny(dtype, true, a, nullptr, (hipStream_t)stream));
  }
  return finish(fsw::launch_tiled(v, dtype, true, a, (hipStream_t)stream));
}

int fsw_gateup(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13, int64_t ldw,
               void* H, int64_t ldh, void* stream) {
  return gateup_impl(dtype, M, N, K, X, ldx, W13, ldw, H, ldh, stream, nullptr, 0);
}

// The reference's other build (C_TYPE float, constants.cuh:9-14; "C can work with either bf16 or fp32",
// swiglu.cu:470-471): H is float and receives the gated fp32 value without a rounding. Two kernels serve it: the
// weight-streaming kernel up to 64 rows, the 256 x 256 kernel on row-major operands above.
int fsw_gateup_f32out(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13,
                      int64_t ldw, float* H, int64_t ldh, void* stream) {
  const int rc = fsw_validate_gateup(dtype, M, N, K, X, ldx, W13, ldw, H, ldh);
  if (rc != FSW_OK) return rc;
  if (M == 0 || N == 0) return FSW_OK;
  if ((((uintptr_t)H) & 3)) return FSW_E_ALIGN;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  fsw::GemmArgs a;
  a.P = W13;
  a.Q = X;
  a.O = H;
  a.ldp = ldw;
  a.ldq = ldx;
  a.ldo = ldh;
  a.np = (int)N;
  a.nq = (int)M;
  a.k = (int)K;
  a.out_f32 = 1;
  if (M <= 64) return finish(fsw::launch_skinny(dtype, true, a, nullptr, (hipStream_t)stream));
  return finish(fsw::launch_pair16(dtype, true, a, (hipStream_t)stream));
}

// Inside fsw_mlp the down projection of up to 32 activation rows runs the split-K streaming kernel when (i) the
// gate/up product before it runs a kernel that zeroes the ticket counters (skinny_kernel or the 128 x 64 tiled
// kernel), (ii) the down projection is in the weight-streaming regime and (iii) the shape is large enough for the
// saved H traffic to matter (stream_split_plan) -- or when variant 104 forces it (then any shape it supports).
static fsw::StreamPlan mlp_stream_plan(int64_t M, int64_t D, int64_t FF) {
  const fsw::StreamPlan none = {0, 0, 0, 0};
  if (M < 1 || M > 32 || D <= 0 || FF <= 0 || D > MAX_DIM || FF > MAX_DIM / 2) return none;
  const int f1 = g_forced_variant[1];
  if (f1 >= 0 && f1 != VARIANT_STREAM_SPLIT) return none;
  const int f0 = g_forced_variant[0];
  if (f0 == VARIANT_DECODE_FUSED || f0 == VARIANT_DECODE_FUSED_FAIL) return none;
  const int v0 = resolve_variant(0, M, 2 * FF, D);
  const bool zeroes = (v0 == VARIANT_SKINNY && !decode_stream_wanted(0, M, 2 * FF, D)) || v0 == V_128x64;
  if (!zeroes) return none;
  if (f1 == VARIANT_STREAM_SPLIT) return fsw::stream_split_plan((int)D, (int)M, (int)FF, true);
  if (!streams_weights(1, M, D, FF) || decode_stream_wanted(1, M, D, FF)) return none;
  return fsw::stream_split_plan((int)D, (int)M, (int)FF, false);
}
static size_t stream_scratch_bytes(const fsw::StreamPlan& p) {
  return (p.partial_bytes + (size_t)p.ticket_words * 4 + 255) & ~(size_t)255;
}

size_t fsw_down_workspace_bytes(int dtype, int64_t M, int64_t D, int64_t FF) {
  (void)dtype;
  if (M <= 0 || M > MAX_DIM || D <= 0 || D > MAX_DIM || FF <= 0 || FF > MAX_DIM || streams_weights(1, M, D, FF)) return 0;
  if (g_forced_variant[1] >= 0) return 0;  // a forced kernel runs unsplit
  const fsw::SplitPlan plan = fsw::tiled_split_plan((int)D, (int)M, (int)FF);
  return plan.splits > 1 ? (size_t)plan.splits * (size_t)M * (size_t)D * sizeof(float) : 0;
}

int fsw_down(int dtype, int64_t M, int64_t D, int64_t FF, const void* H, int64_t ldh, const void* W2, int64_t ldw2,
             void* Y, int64_t ldy, void* workspace, size_t workspace_bytes, void* stream) {
  const int rc = fsw_validate_down(dtype, M, D, FF, H, ldh, W2, ldw2, Y, ldy);
  if (rc != FSW_OK) return rc;
  if (M == 0 || D == 0) return FSW_OK;
  const size_t need = fsw_down_workspace_bytes(dtype, M, D, FF);
  if (need > 0 && (!workspace || workspace_bytes < need)) return FSW_E_WORKSPACE;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  fsw::GemmArgs a;
  a.P = W2;
  a.Q = H;
  a.O = Y;
  a.ldp = ldw2;
  a.ldq = ldh;
  a.ldo = ldy;
  a.np = (int)D;
  a.nq = (int)M;
  a.k = (int)FF;
  const int v = resolve_variant(1, M, D, FF);
  if (v == VARIANT_SKINNY) {
    if (decode_stream_wanted(1, M, D, FF)) {
      fsw::DecodeArgs da = {};
      da.W2 = W2;
      da.H = const_cast<void*>(H);
      da.Y = Y;
      da.ldw2 = ldw2;
      da.ldy = ldy;
      da.ldh = ldh;
      da.nq = (int)M;
      da.d = (int)D;
      da.ff = (int)FF;
      if (fsw::decode_mlp_supported(da, 2)) return finish(fsw::launch_decode_mlp(dtype, da, (hipStream_t)stream, 2));
    }
    return finish(fsw::launch_skinny(dtype, false, a, workspace, (hipStream_t)stream));
  }
  if (need > 0 && g_forced_variant[1] < 0) {  // few output tiles, deep K: split K across workgroups
    if (!aligned16(workspace)) return FSW_E_ALIGN;
    const fsw::SplitPlan plan = fsw::tiled_split_plan((int)D, (int)M, (int)FF);
    a.splits = plan.splits;
    a.partial = (float*)workspace;
    return finish(fsw::launch_tiled_splitk(dtype, plan.tile, a, (hipStream_t)stream));
  }
  return finish(fsw::launch_tiled(v, dtype, false, a, (hipStream_t)stream));
}

// Large-tile regime of fsw_mlp: both projections run 256 x 256 tiles, and H never exists row-major: the gate/up
// epilogue writes it panel-blocked (whole 1 KB runs) and the down projection reads it blocked. Against row-major H
// the whole forward measures 0.8 % (8192 x 4096 x 14336) to 1.3 % (4096 x 4096 x 11008) faster; X is read row-major.
static bool blocked_regime(int64_t M, int64_t D, int64_t FF) {
  if (M <= 64 || D <= 0 || FF <= 0 || g_forced_variant[0] >= 0 || g_forced_variant[1] >= 0) return false;
  if (M > MAX_DIM || D > MAX_DIM || FF > MAX_DIM / 2) return false;
  return pick_tiled(0, M, 2 * FF) == V_256x256 && pick_tiled(1, M, D) == V_256x256 &&
         fsw::tiled_split_plan((int)D, (int)M, (int)FF).splits == 1;  // a split-K down projection reads row-major H
}

size_t fsw_blocked_bytes(int64_t rows, int64_t k) {
  if (rows <= 0 || k <= 0 || rows > MAX_DIM || k > MAX_DIM) return 0;
  return (size_t)fsw::blocked_bytes(rows, k);
}

// src: row-major [rows, k], 16-byte aligned, ld and k multiples of 8; dst: fsw_blocked_bytes(rows, k) bytes
static int block_rows_impl(int dtype, int64_t rows, int64_t k, const void* src, int64_t ld, void* dst, bool gated_order,
                           void* stream) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (rows < 0 || k < 0 || rows > MAX_DIM || k > MAX_DIM || (gated_order && (rows & 1))) return FSW_E_SHAPE;
  if (rows == 0 || k == 0) return FSW_OK;
  if (!src || !dst) return FSW_E_NULL;
  if (ld < k) return FSW_E_LD;
  if (ld > MAX_LD) return FSW_E_SHAPE;
  if ((k & 7) || (ld & 7) || !aligned16(src) || !aligned16(dst)) return FSW_E_ALIGN;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  return finish(fsw::launch_block_rows(src, ld, (int)rows, (int)k, dst, gated_order, (hipStream_t)stream));
}

int fsw_block_rows(int dtype, int64_t rows, int64_t k, const void* src, int64_t ld, void* dst, void* stream) {
  return block_rows_impl(dtype, rows, k, src, ld, dst, false, stream);
}

int fsw_prepack_w13(int dtype, int64_t N, int64_t K, const void* W13, int64_t ldw, void* dst, void* stream) {
  return block_rows_impl(dtype, N, K, W13, ldw, dst, true, stream);
}

int fsw_prepack_w2(int dtype, int64_t D, int64_t FF, const void* W2, int64_t ldw2, void* dst, void* stream) {
  return block_rows_impl(dtype, D, FF, W2, ldw2, dst, false, stream);
}

int fsw_gateup_blocked(int dtype, int64_t M, int64_t N, int64_t K, const void* Xb, const void* W13, int64_t ldw,
                       int w_blocked, void* Hb, int64_t ldh, void* stream) {

  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (M < 0 || N < 0 || K < 0 || (N & 1) || M > MAX_DIM || N > MAX_DIM || K > MAX_DIM) return FSW_E_SHAPE;
  if (M == 0 || N == 0) return FSW_OK;
  if (K == 0) return FSW_E_SHAPE;  // a blocked matrix with no columns has no representation
  if (!Xb || !W13 || !Hb) return FSW_E_NULL;
  if (!w_blocked && ldw < K) return FSW_E_LD;
  if (!w_blocked && ldw > MAX_LD) return FSW_E_SHAPE;
  if (ldh != 0 && ldh < N / 2) return FSW_E_LD;
  if (ldh > MAX_DIM) return FSW_E_SHAPE;
  if ((K & 7) || (!w_blocked && (ldw & 7))) return FSW_E_ALIGN;
  if (!aligned16(Xb) || !aligned16(W13) || (ldh == 0 ? !aligned16(Hb) : ((((uintptr_t)Hb) & 1) != 0))) return FSW_E_ALIGN;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  fsw::GemmArgs a;
  a.P = W13;
  a.Q = Xb;
  a.O = Hb;
  a.ldp = ldw;
  a.ldq = 0;
  a.ldo = ldh;
  a.np = (int)N;
  a.nq = (int)M;
  a.k = (int)K;
  a.layout = 1 | (ldh == 0 ? 2 : 0) | (w_blocked ? 4 : 0);
  return finish(fsw::launch_pair16(dtype, true, a, (hipStream_t)stream));
}

int fsw_gateup_hblocked(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13,
                        int64_t ldw, int w_blocked, void* Hb, void* stream) {
  // blocked weights have no leading dimension: validated as if their rows were K long
  const int rc = fsw_validate_gateup(dtype, M, N, K, X, ldx, W13, w_blocked ? K : ldw, Hb, N / 2);
  if (rc != FSW_OK) return rc;
  if (M == 0 || N == 0) return FSW_OK;
  if (K == 0) return FSW_E_SHAPE;  // a blocked matrix with no columns has no representation
  if (!aligned16(Hb)) return FSW_E_ALIGN;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  fsw::GemmArgs a;
  a.P = W13;
  a.Q = X;
  a.O = Hb;
  a.ldp = ldw;
  a.ldq = ldx;
  a.ldo = 0;
  a.np = (int)N;
  a.nq = (int)M;
  a.k = (int)K;
  a.layout = w_blocked ? 6 : 2;
  return finish(fsw::launch_pair16(dtype, true, a, (hipStream_t)stream));
}

int fsw_down_blocked(int dtype, int64_t M, int64_t D, int64_t FF, const void* Hb, const void* W2, int64_t ldw2,
                     int w_blocked, void* Y, int64_t ldy, void* stream) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (M < 0 || D < 0 || FF < 0 || M > MAX_DIM || D > MAX_DIM || FF > MAX_DIM) return FSW_E_SHAPE;
  if (M == 0 || D == 0) return FSW_OK;
  if (FF == 0) return FSW_E_SHAPE;
  if (!Hb || !W2 || !Y) return FSW_E_NULL;
  if ((!w_blocked && ldw2 < FF) || ldy < D) return FSW_E_LD;
  if ((!w_blocked && ldw2 > MAX_LD) || ldy > MAX_DIM) return FSW_E_SHAPE;
  if ((FF & 7) || (!w_blocked && (ldw2 & 7)) || (((uintptr_t)Y) & 1)) return FSW_E_ALIGN;
  if (!aligned16(Hb) || !aligned16(W2)) return FSW_E_ALIGN;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  fsw::GemmArgs a;
  a.P = W2;
  a.Q = Hb;
  a.O = Y;
  a.ldp = ldw2;
  a.ldq = 0;
  a.ldo = ldy;
  a.np = (int)D;
  a.nq = (int)M;
  a.k = (int)FF;
  a.layout = w_blocked ? 5 : 1;
  return finish(fsw::launch_pair16(dtype, false, a, (hipStream_t)stream));
}

// fsw_gateup never needs scratch: the large-tile kernel reads row-major X in whole cache lines (K pairs), which
// measures level with a blocked copy of X (8192 x 4096 x 28672: 1.2515 vs 1.2530 ms) and saves the copy. The two
// entry points stay for callers written against them.
size_t fsw_gateup_workspace_bytes(int dtype, int64_t M, int64_t N, int64_t K) {
  (void)dtype;
  (void)M;
  (void)N;
  (void)K;
  return 0;
}

int fsw_gateup_ws(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13, int64_t ldw,
                  void* H, int64_t ldh, void* workspace, size_t workspace_bytes, void* stream) {
  (void)workspace;
  (void)workspace_bytes;
  return fsw_gateup(dtype, M, N, K, X, ldx, W13, ldw, H, ldh, stream);
}

static size_t h_bytes(int64_t M, int64_t FF) {
  const size_t raw = (size_t)M * (size_t)FF * 2;
  return (raw + 255) & ~(size_t)255;
}

size_t fsw_mlp_workspace_bytes(int dtype, int64_t M, int64_t D, int64_t FF) {
  if (M <= 0 || D <= 0 || FF <= 0) return 0;
  if (blocked_regime(M, D, FF)) return (size_t)fsw::blocked_bytes(M, FF);  // H, panel-blocked
  const fsw::StreamPlan sp = mlp_stream_plan(M, D, FF);
  if (sp.splits > 1) return h_bytes(M, FF) + stream_scratch_bytes(sp);  // [H row-major][partials][ticket counters]
  // otherwise [H row-major][split-K scratch of the down projection]
  return h_bytes(M, FF) + ((fsw_down_workspace_bytes(dtype, M, D, FF) + 255) & ~(size_t)255);
}

// single_launch_ok: whether the opt-in single-launch decode forward may be used (it creates events on first use,
// which the entry point that must not allocate cannot afford)
static int mlp_impl(int dtype, int64_t M, int64_t D, int64_t FF, const void* X, int64_t ldx, const void* W13,
                    int64_t ldw13, const void* W2, int64_t ldw2, void* Y, int64_t ldy, void* workspace,
                    size_t workspace_bytes, void* stream, bool single_launch_ok) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (M < 0 || D < 0 || FF < 0 || M > MAX_DIM || D > MAX_DIM || FF > MAX_DIM / 2) return FSW_E_SHAPE;
  if (M == 0 || D == 0) return FSW_OK;  // Y is empty: nothing to read or write
  const size_t need = fsw_mlp_workspace_bytes(dtype, M, D, FF);
  if (need > 0 && (!workspace || workspace_bytes < need)) return FSW_E_WORKSPACE;
  if (need > 0 && !aligned16(workspace)) return FSW_E_ALIGN;
  // FF == 0 needs no H: any non-NULL pointer satisfies the validators and is never dereferenced
  void* Hbuf = need > 0 ? workspace : (void*)Y;
  // validate both halves before launching either, so a bad down-projection argument leaves nothing enqueued
  int rc = fsw_validate_gateup(dtype, M, 2 * FF, D, X, ldx, W13, ldw13, Hbuf, FF);
  if (rc != FSW_OK) return rc;
  rc = fsw_validate_down(dtype, M, D, FF, Hbuf, FF, W2, ldw2, Y, ldy);
  if (rc != FSW_OK) return rc;
  if (single_launch_ok && M <= 16 && FF > 0 &&
      (g_forced_variant[0] == VARIANT_DECODE_FUSED || g_forced_variant[0] == VARIANT_DECODE_FUSED_FAIL)) {
    // opt-in: one persistent launch does both projections with a device-wide barrier in between. Measured
    // slower than the two weight-streaming launches so far (stragglers before the barrier), so not the default.
    // Without a free barrier slot, or on a stream that is being captured, it is the two launches below.
    fsw::DecodeArgs da;
    da.X = X;
    da.W13 = W13;
    da.W2 = W2;
    da.H = Hbuf;
    da.Y = Y;
    da.ldx = ldx;
    da.ldw13 = ldw13;
    da.ldw2 = ldw2;
    da.ldy = ldy;
    da.ldh = FF;
    da.nq = (int)M;
    da.d = (int)D;
    da.ff = (int)FF;
    if (fsw::decode_mlp_supported(da, 3)) {
      const int drc = check_device();
      if (drc != FSW_OK) return drc;
      bool launched = false;
      const int lrc = finish(fsw::launch_decode_mlp(dtype, da, (hipStream_t)stream, 3, &launched,
                                                    g_forced_variant[0] == VARIANT_DECODE_FUSED_FAIL));
      if (lrc != FSW_OK || launched) return lrc;
    }
  }
  if (blocked_regime(M, D, FF)) {  // workspace = H, panel-blocked
    rc = fsw_gateup_hblocked(dtype, M, 2 * FF, D, X, ldx, W13, ldw13, 0, workspace, stream);
    if (rc != FSW_OK) return rc;
    return fsw_down_blocked(dtype, M, D, FF, workspace, W2, ldw2, 0, Y, ldy, stream);
  }
  unsigned char* ws2 = (unsigned char*)workspace + h_bytes(M, FF);
  const fsw::StreamPlan sp = mlp_stream_plan(M, D, FF);
  if (sp.splits > 1) {  // decode: the gate/up kernel zeroes the ticket counters of the split-K streaming down projection
    unsigned* tickets = (unsigned*)(ws2 + sp.partial_bytes);
    rc = gateup_impl(dtype, M, 2 * FF, D, X, ldx, W13, ldw13, Hbuf, FF, stream, tickets, sp.ticket_words);
    if (rc != FSW_OK) return rc;
    fsw::GemmArgs a;
    a.P = W2;
    a.Q = Hbuf;
    a.O = Y;
    a.ldp = ldw2;
    a.ldq = FF;
    a.ldo = ldy;
    a.np = (int)D;
    a.nq = (int)M;
    a.k = (int)FF;
    return finish(fsw::launch_stream_split(dtype, a, sp, ws2, (hipStream_t)stream));
  }
  const size_t down_ws = (fsw_down_workspace_bytes(dtype, M, D, FF) + 255) & ~(size_t)255;
  rc = fsw_gateup(dtype, M, 2 * FF, D, X, ldx, W13, ldw13, Hbuf, FF, stream);
  if (rc != FSW_OK) return rc;
  return fsw_down(dtype, M, D, FF, Hbuf, FF, W2, ldw2, Y, ldy, ws2, down_ws, stream);
}

int fsw_mlp(int dtype, int64_t M, int64_t D, int64_t FF, const void* X, int64_t ldx, const void* W13, int64_t ldw13,
            const void* W2, int64_t ldw2, void* Y, int64_t ldy, void* workspace, size_t workspace_bytes,
            void* stream) {
  return mlp_impl(dtype, M, D, FF, X, ldx, W13, ldw13, W2, ldw2, Y, ldy, workspace, workspace_bytes, stream, true);
}

// ---- the entry point that allocates nothing ------------------------------------------------------------------
// fsw_mlp with its workspace inside the library: a file-scope device array that every GPU the library runs on
// holds until the process ends. The array's name is a host-side stand-in, not a device address; its address on a
// device comes from hipGetSymbolAddress, asked once per device with that device current, and only that pointer is
// handed to kernels.
#define FSW_STATIC_SCRATCH_BYTES (64u << 20)
static __device__ __align__(256) unsigned char scratch[FSW_STATIC_SCRATCH_BYTES];

// device address of `scratch` on the current device (looked up on the first call per device, then cached)
static int static_scratch_ptr(void** out) {
  static std::atomic<void*> ptr_of_device[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= 64) {
    g_last_hip_error = (int)e;
    return FSW_E_DEVICE;
  }
  void* p = ptr_of_device[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      g_last_hip_error = (int)e;
      return FSW_E_LAUNCH;
    }
    ptr_of_device[dev].store(p, std::memory_order_release);  // racing first calls on one device store the same address
  }
  *out = p;
  return FSW_OK;
}

size_t fsw_mlp_static_max_bytes(void) { return FSW_STATIC_SCRATCH_BYTES; }

int fsw_mlp_static(int dtype, int64_t M, int64_t D, int64_t FF, const void* X, int64_t ldx, const void* W13,
                   int64_t ldw13, const void* W2, int64_t ldw2, void* Y, int64_t ldy, void* stream) {
  if (dtype != FSW_BF16 && dtype != FSW_FP16) return FSW_E_DTYPE;
  if (M < 0 || D < 0 || FF < 0 || M > MAX_DIM || D > MAX_DIM || FF > MAX_DIM / 2) return FSW_E_SHAPE;
  if (M == 0 || D == 0) return FSW_OK;
  if (fsw_mlp_workspace_bytes(dtype, M, D, FF) > FSW_STATIC_SCRATCH_BYTES) return FSW_E_STATIC_LIMIT;
  const int drc = check_device();
  if (drc != FSW_OK) return drc;
  void* ws = nullptr;
  const int rc = static_scratch_ptr(&ws);
  if (rc != FSW_OK) return rc;
  return mlp_impl(dtype, M, D, FF, X, ldx, W13, ldw13, W2, ldw2, Y, ldy, ws, FSW_STATIC_SCRATCH_BYTES, stream, false);
}

}  // extern "C"
