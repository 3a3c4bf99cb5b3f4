// Internal launcher interface between the C-ABI dispatcher (fsw_api.hip) and the kernel translation units.
// Nothing here is exported; the public surface is include/fsw.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fsw {

// One TN GEMM problem in "weight rows x activation rows" form.
//   P: weight operand, [np, k] row-major (W13 for the gated kernel, W2 for the down kernel)
//   Q: activation operand, [nq, k] row-major (X or H)
//   O: output, [nq, np/2] (gated) or [nq, np] (plain), row stride ldo
struct GemmArgs {
  const void* P;
  const void* Q;
  void* O;
  long long ldp, ldq, ldo;  // elements
  int np, nq, k;
  // split-K (plain kernel only): `splits` workgroups share one output tile, each over a contiguous K range, and
  // store fp32 partial sums to partial[split][nq][np]; splitk_reduce() sums them and rounds once.
  int splits = 1;
  float* partial = nullptr;
  // panel-blocked operands / output of the 256 x 256 kernel (launch_pair16): bit 0 = Q, bit 1 = O
  // (gated kernel), bit 2 = P. A blocked [rows, k] matrix is ceil(rows / 256) panels of ceil(k / 32) blocks of
  // [256 rows][64 bytes], zero padded (blocked_bytes()).
  int layout = 0;
  // words the FIRST workgroup of a gate/up launch sets to zero before anything else (tiled_dma_kernel and
  // skinny_kernel honour it): the ticket counters of the split-K streaming down projection that follows in fsw_mlp
  unsigned* zero_words = nullptr;
  int n_zero_words = 0;
  // gated kernels on row-major operands (skinny_kernel, the 256 x 256 kernel with layout 0): O is float [nq, np/2]
  // and receives the gated fp32 value unrounded (the reference's build with C_TYPE float, constants.cuh:9)
  int out_f32 = 0;
  // tiled_dma_kernel with one tile of activation rows: weight rows a workgroup owns when that is fewer than the
  // kernel's tile height (0 = the tile height). The tile then starts every tile_p rows, rows past tile_p are out
  // of range for its copies (zeros, no traffic) and are not stored: lets a weight stream be cut into exactly as
  // many pieces as there are compute units. A multiple of 8 (whole 8-byte stores of the gated output).
  int tile_p = 0;
};
inline long long blocked_bytes(long long rows, long long k) {
  return ((rows + 255) / 256) * ((k + 31) / 32) * (256 * 64);
}

// Tiled LDS/MFMA kernels (kernels_tiled.hip). `variant` indexes tiled_variant_table().
struct TiledVariant {
  const char* name;
  int bp, bq;        // workgroup tile: weight rows x activation rows
  int threads;
};
int tiled_variant_count();
int pair16_variant();  // index of the 256 x 256 kernel in the table
const TiledVariant& tiled_variant(int variant);
// row-major operands (GemmArgs::layout 0)
hipError_t launch_tiled(int variant, int dtype, bool gated, const GemmArgs& a, hipStream_t stream);
int raster_group(bool gated, int tiles_q);  // activation-row tiles per raster band of the tiled kernels
// The 256 x 256 kernel on v_mfma_f32_16x16x32 (kernels_pair16.hip) for GemmArgs::layout 0, 1, 3, 5, 7.
// gated: X blocked in (bit 0), H blocked out (bit 1) or row-major, W13 blocked (bit 2) or row-major: layouts 1, 3, 5, 7;
// plain: H blocked in, W2 row-major (1) or blocked (5); 0 = everything row-major
hipError_t launch_pair16(int dtype, bool gated, const GemmArgs& a, hipStream_t stream);
hipError_t launch_pair16_splitk(int dtype, const GemmArgs& a, hipStream_t stream);  // partials only, no reduction
// row-major [rows, k] (row stride ld elements) -> blocked; gated_order: W13's up/gate rows de-interleaved per panel
hipError_t launch_block_rows(const void* src, long long ld, int rows, int k, void* dst, bool gated_order,
                             hipStream_t stream);
// Plan for the plain (down-projection) product when the output has few tiles and K is deep: which direct-to-LDS
// tile (128 or 256 square) and how many K partitions, so that about two workgroups per CU are in flight.
// splits == 1 means the ordinary launch path.
struct SplitPlan {
  int tile;    // 128 or 256 (square), 129 = 128 output features x 256 activation rows, 130 = 128 x 192
  int splits;  // K partitions
};
SplitPlan tiled_split_plan(int np, int nq, int k);
hipError_t launch_tiled_splitk(int dtype, int tile, const GemmArgs& a, hipStream_t stream);  // a.splits, a.partial set

// Weight-streaming kernels for M <= 16 activation rows (kernels_skinny.hip).
struct SkinnyPlan {
  int splits;              // K partitions per weight-row tile across workgroups (1 = no scratch needed)
  size_t workspace_bytes;  // fp32 partials + arrival counters
};
SkinnyPlan skinny_plan(bool gated, int np, int nq, int k);
hipError_t launch_skinny(int dtype, bool gated, const GemmArgs& a, void* workspace, hipStream_t stream);

// Split-K weight-streaming down projection for at most 32 activation rows (kernels_stream.hip): 32-row tiles, the K
// range split over blockIdx.y, partial tiles reduced by the workgroup that draws a tile's last ticket.
struct StreamPlan {
  int splits;            // 0: the shape does not use this kernel
  int tiles;
  size_t partial_bytes;  // fp32 partial tiles, first in the scratch
  int ticket_words;      // one counter per tile behind the partials; must be zero when the kernel starts
};
StreamPlan stream_split_plan(int np, int nq, int k, bool forced);  // forced: any supported shape
hipError_t launch_stream_split(int dtype, const GemmArgs& a, const StreamPlan& p, void* workspace, hipStream_t stream);

}  // namespace fsw

namespace fsw {

// Single-launch decode forward (kernels_decode.hip): gate/up, device-wide barrier, down projection, for at most
// 16 activation rows. H is a caller-provided [nq, ff] scratch matrix (row stride ff).
struct DecodeArgs {
  const void* X;
  const void* W13;
  const void* W2;
  void* H;
  void* Y;
  long long ldx, ldw13, ldw2, ldy, ldh;  // elements
  int nq, d, ff;
};
bool decode_mlp_supported(const DecodeArgs& a, int phases = 3);
// phases: 1 = gate/up only, 2 = down only (H already written), 3 = both in one launch. With phases == 3 *launched
// tells whether the launch was enqueued: it is not (and the call still succeeds) when no barrier slot is free or the
// stream is being captured. test_unreachable makes the device-wide barrier give up at once (failure-path test).
hipError_t launch_decode_mlp(int dtype, const DecodeArgs& a, hipStream_t stream, int phases, bool* launched = nullptr,
                             bool test_unreachable = false);
hipError_t decode_barrier_failures(int* count);

}  // namespace fsw
