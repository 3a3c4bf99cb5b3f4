/*
 * fsw.h — C ABI of the MI355X (gfx950) fused SwiGLU MLP forward.
 *
 * The reference (bit-ml/Fused-SwiGLU) has no C ABI: its internal boundary is the C++ template
 * `swiglu_fwd<TA,TB,TC>` declared at csrc/torch_bindings.cpp:16-27 and defined at
 * csrc/SwiGLU/swiglu.cu:397-525, plus the convenience op `fused_swiglu_bf16` (swiglu.cu:538-553).
 * The entry points below are what a foreign-function binding for that path binds instead; the
 * PyTorch operator surface (torch_bindings.cpp:31-50) is rebuilt on top of them.
 *
 * Conventions (all entry points):
 *   - every data pointer is a DEVICE pointer owned by the caller; nothing is allocated or freed here;
 *   - leading dimensions (ld*) are in ELEMENTS, inner (K) stride is 1 as in swiglu.cu:411-414;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); launches are
 *     asynchronous, nothing here synchronises;
 *   - the return value is FSW_OK (0) or a negative FSW_E_* code; nothing throws or aborts;
 *   - the fsw_validate_* functions touch no GPU API and can be called on a machine without one;
 *   - entry points are re-entrant: there is no process-wide mutable state apart from caches of device properties
 *     (filled atomically), so any number of host threads may call them on any streams at the same time;
 *   - the library links the HIP runtime (libamdhip64). A process must hold ONE copy of it: inside a PyTorch-ROCm
 *     process, load torch (which brings its own) BEFORE this library, or launches fail with FSW_E_DEVICE.
 *
 * Weight formats (identical to the reference's):
 *   W13 [N = 2*ff, K] row-major, K-contiguous, rows interleaved: row 2j   = "up"  (linear) operand,
 *                                                                row 2j+1 = "gate" (SiLU) operand
 *       (swiglu.cu:380-381, numeric_tests.py:41-43);
 *   W2  [D, FF] row-major, FF-contiguous (the transpose of the mathematical Wd[FF, D]).
 */
#ifndef FSW_H
#define FSW_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* every entry point below is exported; everything else in the library has hidden visibility */
#define FSW_API __attribute__((visibility("default")))

/* element types */
#define FSW_BF16 0
#define FSW_FP16 1

/* error codes */
#define FSW_OK            0
#define FSW_E_NULL       -1   /* a required pointer is NULL */
#define FSW_E_DTYPE      -2   /* dtype is not FSW_BF16 / FSW_FP16 */
#define FSW_E_SHAPE      -3   /* negative size, odd N, or a size beyond the supported range */
#define FSW_E_LD         -4   /* leading dimension smaller than the row it strides */
#define FSW_E_ALIGN      -5   /* K (or FF), a leading dimension or a pointer breaks the 16-byte rule */
#define FSW_E_WORKSPACE  -6   /* workspace missing or smaller than fsw_*_workspace_bytes() */
#define FSW_E_LAUNCH     -7   /* the HIP runtime rejected a launch (see fsw_last_hip_error) */
#define FSW_E_DEVICE     -8   /* the current device is not a gfx950 GPU */
#define FSW_E_VARIANT    -9   /* unknown kernel variant requested through fsw_set_variant */
#define FSW_E_STATIC_LIMIT -10 /* fsw_mlp_static: the shape needs more scratch than the library's static array */

/*
 * Host-only argument validation of fsw_gateup (replaces the dtype TORCH_CHECKs of swiglu.cu:475-480 and adds
 * the shape/stride checks the reference leaves out). Rules: M >= 0; N >= 0 and even; K >= 0 and K % 8 == 0
 * (16-byte vectors; the reference needs K % 32 == 0, swiglu.cu:220-230); ldx >= K, ldw >= K, ldh >= N/2;
 * ldx % 8 == 0 and ldw % 8 == 0; pointers non-NULL and X, W13 16-byte aligned when the problem is non-empty
 * (M == 0 or N == 0 needs no pointers; K == 0 needs only H, which is then written with zeros).
 */
FSW_API int fsw_validate_gateup(int dtype, int64_t M, int64_t N, int64_t K,
                        const void* X, int64_t ldx, const void* W13, int64_t ldw,
                        const void* H, int64_t ldh);

/*
 * H[M, N/2] = up * silu(gate) with up = X @ W13[0::2].T, gate = X @ W13[1::2].T; fp32 accumulation,
 * fp32 gating, ONE round-to-nearest-even to the element type on store.
 * Replaces swiglu_fwd<bf16,bf16,bf16> (swiglu.cu:397-525; kernel swiglu.cu:103-394). N is the FULL 2*ff as in
 * the reference; ldh is the row stride of H itself (the reference's operator passes ldC/2, swiglu.cu:414).
 */
FSW_API int fsw_gateup(int dtype, int64_t M, int64_t N, int64_t K,
               const void* X, int64_t ldx, const void* W13, int64_t ldw,
               void* H, int64_t ldh, void* stream);

/*
 * fsw_gateup whose H is float [M, N/2] (row stride ldh in floats, 4-byte aligned): the gated fp32 value is stored
 * as it is, with no rounding. Replaces swiglu_fwd<bf16,bf16,float>, the reference's build with C_TYPE float
 * (constants.cuh:9-14; cast_mmaresult's to_float branch, swiglu.cu:47-82; "C can work with either bf16 or fp32",
 * swiglu.cu:470-471). Inputs as for fsw_gateup.
 */
FSW_API int fsw_gateup_f32out(int dtype, int64_t M, int64_t N, int64_t K,
                      const void* X, int64_t ldx, const void* W13, int64_t ldw,
                      float* H, int64_t ldh, void* stream);

/* Host-only validation of fsw_down: M, D, FF >= 0; FF % 8 == 0; ldh >= FF, ldw2 >= FF, ldy >= D;
 * ldh % 8 == 0, ldw2 % 8 == 0; H, W2 16-byte aligned. */
FSW_API int fsw_validate_down(int dtype, int64_t M, int64_t D, int64_t FF,
                      const void* H, int64_t ldh, const void* W2, int64_t ldw2,
                      const void* Y, int64_t ldy);

/* Bytes of device scratch fsw_down needs for this shape: fp32 split-K partials where few output tiles meet a deep K
 * (FSW_E_WORKSPACE without them), 0 otherwise. No counterpart in the reference, which has no down projection. */
FSW_API size_t fsw_down_workspace_bytes(int dtype, int64_t M, int64_t D, int64_t FF);

/*
 * Y[M, D] = H[M, FF] @ W2[D, FF].T, fp32 accumulation, one RNE rounding on store.
 * No counterpart in the reference (its op ends at H, swiglu.cu:538-553); it is the `@ Wd` step of the
 * full MLP forward (silu(X@Wg) * (X@Wu)) @ Wd.
 */
FSW_API int fsw_down(int dtype, int64_t M, int64_t D, int64_t FF,
             const void* H, int64_t ldh, const void* W2, int64_t ldw2,
             void* Y, int64_t ldy,
             void* workspace, size_t workspace_bytes, void* stream);

/* Bytes of device scratch fsw_mlp needs: the H[M, FF] intermediate (panel-blocked in the large-tile regime) plus the
 * scratch of its down projection. */
FSW_API size_t fsw_mlp_workspace_bytes(int dtype, int64_t M, int64_t D, int64_t FF);

/*
 * Whole forward: Y[M, D] = (silu(X @ Wg) * (X @ Wu)) @ Wd as fsw_gateup followed by fsw_down on the same
 * stream, with H held in `workspace`. X is [M, D]; W13 is [2*FF, D]; W2 is [D, FF].
 */
FSW_API int fsw_mlp(int dtype, int64_t M, int64_t D, int64_t FF,
            const void* X, int64_t ldx, const void* W13, int64_t ldw13,
            const void* W2, int64_t ldw2, void* Y, int64_t ldy,
            void* workspace, size_t workspace_bytes, void* stream);

/*
 * fsw_mlp for callers that cannot allocate device memory at all (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments without the workspace, same kernels, same result bit for
 * bit. No counterpart in the reference. The scratch (H, split-K partials and their ticket counters) lives in a static
 * device array of fsw_mlp_static_max_bytes() = 64 MiB inside the library, which every GPU the library runs on holds
 * until the process ends; shapes whose fsw_mlp_workspace_bytes() exceed it return FSW_E_STATIC_LIMIT (it covers
 * decode and small batches: at d = 4096, ff = 14336 every M <= 468). The call itself allocates and frees nothing;
 * the first call on a device looks the array's address up (make it outside graph capture). All calls on one GPU share
 * the one array: calls that overlap in time on the same GPU (different streams, concurrent graph replays) race on
 * it and must be serialised by the caller. The single-launch decode option of fsw_set_variant is ignored here.
 */
FSW_API size_t fsw_mlp_static_max_bytes(void);
FSW_API int fsw_mlp_static(int dtype, int64_t M, int64_t D, int64_t FF,
                           const void* X, int64_t ldx, const void* W13, int64_t ldw13,
                           const void* W2, int64_t ldw2, void* Y, int64_t ldy, void* stream);

/* Text for an FSW_E_* code (static storage, never NULL). */
FSW_API const char* fsw_strerror(int code);

/*
 * Panel-blocked layout (no counterpart in the reference; it is the offline/in-flight layout transform that lets the
 * large-tile kernels fetch whole cache lines). A blocked copy of a row-major [rows, k] matrix is ceil(rows / 256)
 * panels of ceil(k / 32) blocks; block (panel, kt) is [256 rows][32 elements] contiguous (16 KB) and holds rows
 * 256 panel .. 256 panel + 255, columns 32 kt .. 32 kt + 31, zero padded. fsw_mlp uses it internally for M > 64 when
 * both projections run 256 x 256 tiles: H is written and read blocked (fsw_gateup_hblocked, fsw_down_blocked); X is
 * read row-major. The entry points below expose the steps, and let a caller block the weights ONCE (fsw_prepack_*)
 * and pass them with w_blocked = 1. Constraints as for fsw_gateup / fsw_down (K, FF and row-major leading dimensions multiples of 8,
 * 16-byte aligned bases); the blocked kernels are the 256 x 256 tiled kernels, whatever M is.
 */
FSW_API size_t fsw_blocked_bytes(int64_t rows, int64_t k);
FSW_API int fsw_block_rows(int dtype, int64_t rows, int64_t k, const void* src, int64_t ld, void* dst_blocked,
                           void* stream);
/* W13 [N, K] interleaved as in swiglu.cu:380-381 -> blocked, with each panel's 128 "up" rows first, then its 128
 * "gate" rows (the order the gated kernel keeps a weight tile in LDS). */
FSW_API int fsw_prepack_w13(int dtype, int64_t N, int64_t K, const void* W13, int64_t ldw, void* dst_blocked,
                            void* stream);
FSW_API int fsw_prepack_w2(int dtype, int64_t D, int64_t FF, const void* W2, int64_t ldw2, void* dst_blocked,
                           void* stream);
/* H[M, N/2] = gate/up of X_blocked[M, K]; W13 row-major (w_blocked = 0, ldw) or from fsw_prepack_w13 (1); H is
 * written blocked when ldh == 0 (for fsw_down_blocked), else row-major with row stride ldh. */
FSW_API int fsw_gateup_blocked(int dtype, int64_t M, int64_t N, int64_t K, const void* X_blocked, const void* W13,
                               int64_t ldw, int w_blocked, void* H, int64_t ldh, void* stream);
/* fsw_gateup on row-major X (row stride ldx) whose H is written blocked, for fsw_down_blocked: the two halves of
 * fsw_mlp in the large-tile regime. W13 row-major (w_blocked = 0, ldw) or from fsw_prepack_w13 (1). K > 0;
 * constraints as for fsw_gateup; H 16-byte aligned. */
FSW_API int fsw_gateup_hblocked(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13,
                                int64_t ldw, int w_blocked, void* H_blocked, void* stream);
/* Y[M, D] (row-major, ldy) = H_blocked[M, FF] @ W2^T; W2 row-major (0, ldw2) or from fsw_prepack_w2 (1). */
FSW_API int fsw_down_blocked(int dtype, int64_t M, int64_t D, int64_t FF, const void* H_blocked, const void* W2,
                             int64_t ldw2, int w_blocked, void* Y, int64_t ldy, void* stream);

/* fsw_gateup with a scratch argument, kept for callers written against it: the query returns 0 for every shape and
 * the call is fsw_gateup (the large-tile kernel reads row-major X in whole cache lines; no blocked copy is made). */
FSW_API size_t fsw_gateup_workspace_bytes(int dtype, int64_t M, int64_t N, int64_t K);
FSW_API int fsw_gateup_ws(int dtype, int64_t M, int64_t N, int64_t K, const void* X, int64_t ldx, const void* W13,
                          int64_t ldw, void* H, int64_t ldh, void* workspace, size_t workspace_bytes, void* stream);

/* The hipError_t (as int) of the most recent failed launch on the calling thread, 0 if none. */
FSW_API int fsw_last_hip_error(void);

/* ABI version: major * 1000 + minor. 2000: the measurement kernels fsw_probe_* left this library (libfsw_probe.so,
 * fsw_probe.h); fsw_gateup_f32out and fsw_gateup_hblocked joined it; fsw_gateup_workspace_bytes returns 0. */
FSW_API int fsw_version(void);

/*
 * Kernel-selection override for tests and tuning, PER CALLING THREAD (thread-local): it changes the kernel choice
 * of later calls made by the same thread only, so a thread's fsw_*_workspace_bytes() queries and the launches
 * that follow them always agree. family: 0 = gate/up, 1 = down; variant < 0 restores the automatic choice by
 * shape; 0 .. 5 force one tiled kernel (dma_128x128, dma_128x256, dma_128x192, dma8w_128x256, dma_128x64,
 * pair16_256x256; a forced kernel runs unsplit and needs no scratch); 100 is the weight-streaming kernel (honoured
 * for M <= 64; the dispatcher itself picks it up to 16 .. 48 rows, the larger the weights the fewer); 102 is the
 * persistent streaming kernel (honoured for M <= 16; automatic only for d * ff >= 2^27); family 0 variant 101
 * makes fsw_mlp run M <= 16 as ONE persistent launch (gate/up, device-wide barrier, down) instead of two launches
 * -- see fsw_decode_barrier_failures(): a correctness-tested experiment that measures SLOWER than the two launches
 * (69.7 vs 61.0 us at M = 16, d = 4096, ff = 14336) and is kept for study only; 103 is 101 with a barrier that cannot
 * complete, a hook of the failure-path test that is refused (FSW_E_VARIANT) unless the environment holds
 * FSW_TEST_HOOKS=1;
 * family 1 variant 104 makes fsw_mlp run the down projection of M <= 32 rows on the split-K streaming kernel
 * (32-row tiles, two K ranges whose partial tiles meet through ticket counters that the gate/up kernel zeroes)
 * whatever the shape; the dispatcher picks it for 17 .. 32 rows of large weight matrices.
 * Returns FSW_E_VARIANT for unknown ids.
 */
FSW_API int fsw_set_variant(int family, int variant);

/*
 * The single-launch decode forward (fsw_set_variant(0, 101)) synchronises its workgroups with a device-wide barrier,
 * which completes only if all of them are resident at once. The wait is bounded: when other work holds compute units
 * the kernel gives up, skips the down projection (Y is left incomplete, never computed from a partial H) and marks
 * its barrier slot. This call returns how many such launches there were on the current device since it was last
 * called and clears the marks, or a negative FSW_E_* code. It copies synchronously: call it after synchronising the
 * stream, with no single-launch forward in flight. A caller that opts into variant 101 must check it before using Y.
 * With 64 single-launch forwards in flight, or on a stream that is being captured into a graph, fsw_mlp runs the
 * two-launch path instead. No counterpart in the reference.
 */
FSW_API int fsw_decode_barrier_failures(void);

/* Name of the kernel variant the dispatcher picks for this shape (static storage); "splitk_<kernel>" when the
 * down projection splits K (family 1; K_or_FF decides). family 2: the down projection as fsw_mlp runs it (differs
 * from family 1, which is fsw_down on its own, for 17 .. 32 rows: "stream_split"). */
FSW_API const char* fsw_variant_name(int family, int dtype, int64_t M, int64_t N_or_D, int64_t K_or_FF);

#ifdef __cplusplus
}
#endif
#endif /* FSW_H */
