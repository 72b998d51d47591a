/*
 * deepep_amd — C ABI of the MI355X (gfx950) dispatch / combine / W4A8-MoE hot path.
 *
 * Conventions
 *   - every function returns 0 on success, a negative DPEP_E* code otherwise, and never throws;
 *     dpep_last_error() returns a thread-local message for the last failure on this thread;
 *   - every pointer is a DEVICE pointer unless its name ends in _host;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); every call only
 *     enqueues work on that stream and returns without synchronising;
 *   - output buffers are allocated by the caller; the library owns only the workspace;
 *   - one call at a time per workspace (the host layer keeps the reference's per-buffer lock).
 *
 * Each entry point cites the reference interface it replaces (paths relative to the reference
 * checkout).
 */
#ifndef DEEPEP_AMD_H
#define DEEPEP_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DPEP_OK 0
#define DPEP_EINVAL (-1)  /* bad argument (maps to ValueError, like std::invalid_argument in csrc/ops) */
#define DPEP_ERUNTIME (-2) /* HIP failure (maps to RuntimeError, like std::runtime_error in csrc/ops) */

#define DPEP_MAX_TOPK 32
#define DPEP_MAX_LOCAL_EXPERTS 1024

const char* dpep_last_error(void);
int dpep_version(void);

/* Workspace: one hipMalloc'd HBM block standing in for the reference's symmetric SHMEM workspace
 * (csrc/runtime/session.cpp:40-140, Runtime(...) in csrc/bindings/module.cpp:54-71).  Holds the
 * layout scratch (per-chunk histograms) and the MegaMoE intermediates of one EP rank's share. */
int dpep_workspace_create(size_t bytes, void** ws);
int dpep_workspace_destroy(void* ws);
int dpep_workspace_capacity(void* ws, size_t* bytes);
/* Switches of a workspace for tests and diagnosis; no counterpart in the reference.  Keys:
 *   "layout_one_launch"             0: dpep_layout always takes two launches (count, assign); 1 (default): one
 *                                   launch whose workgroups exchange their histograms, where the input is small enough
 *   "layout_exchange_ticks"         bound of a workgroup's wait for the others' histograms in 10 ns ticks (default 2 s)
 *   "layout_exchange_extra_rows"    1: the workgroups wait for one histogram more than there are workgroups, so that
 *                                   the wait runs out (exercises the error path)
 *   "gemm_zero_fill"                1 (default): workgroups of dpep_megamoe_forward's first GEMM that get no tile zero
 *                                   the output rows of tokens no local expert serves; 0: the weighted reduce writes them
 *   "megamoe_served_only"           1: dpep_megamoe_forward leaves the rows of y whose token no local expert serves
 *                                   untouched (one rank's share of an EP job, where other ranks produce those rows);
 *                                   0 (default): they are zeroed
 *   "gemm_tile_rows"                0 (default): dpep_megamoe_forward chooses the row-tile height of its grouped GEMMs
 *                                   from the expected rows per expert; 64, 128 or 192: that height for both */
int dpep_workspace_tune(void* ws, const char* key, long long value);
/* Scratch bytes dpep_layout needs for T*K routes and L local experts
 * (notify_layout() workspace_bytes, csrc/ops/notify.cpp:98-110). */
size_t dpep_layout_workspace_bytes(int num_tokens, int num_topk, int num_local_experts);

/* Routing layout: validity, per-expert counts, prefix sums and the stable permutation.
 * Replaces notify() (csrc/ops/notify.cpp:112-190 -> notify_full_kernel, csrc/kernels/notify/notify.cpp:2026)
 * and the count/prefix half of expand() (csrc/direct/ops/expand.cpp:52-219).
 *   topk_idx      int64 [T,K]; a route is valid for this rank iff 0 <= e < num_experts and
 *                 expert_begin <= e < expert_begin + num_local
 *   counts        int32 [L]    rows per local expert (expert_totals slice / actual_expert_counts)
 *   psum          int32 [L]    inclusive prefix (psum_num_recv_tokens_per_expert)
 *   offsets       int32 [L+1]  exclusive prefix with leading 0 (expert_offsets)
 *   route_to_row  int32 [T*K]  row of route (t,s), -1 if it produces no row (recv_to_expanded_idx)
 *   row_to_route  int32 [T*K]  first R entries valid: flat route id t*K+s of each row (weight_return_meta)
 *   num_rows      int32 [1]    R */
int dpep_layout(void* ws, const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts,
                int expert_begin, int num_local, int32_t* counts, int32_t* psum, int32_t* offsets,
                int32_t* route_to_row, int32_t* row_to_route, int32_t* num_rows, void* stream);

/* dpep_layout for callers that cannot allocate: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference (whose notify always works in its pre-allocated symmetric
 * workspace).  Same inputs, outputs and results as dpep_layout, but no workspace: the histograms live in a device
 * array inside the library (84 KiB per GPU, held until the process ends), and the call allocates nothing - no
 * hipMalloc, hipFree or pinned memory, on the first call or any later one.  Always the two-launch form (count, then
 * assign); it reports nothing to the host, so R is read from num_rows on the device.  Limits: those of dpep_layout
 * (at most DPEP_MAX_LOCAL_EXPERTS local experts, T*K < 2^31), checked before anything is launched.  All calls on one
 * GPU share that GPU's array: calls whose kernels overlap on one GPU (different streams) race; calls on one stream
 * do not.  Nothing in the array has to be zero or is kept between calls. */
int dpep_layout_static(const int64_t* topk_idx, int num_tokens, int num_topk, int num_experts, int expert_begin,
                       int num_local, int32_t* counts, int32_t* psum, int32_t* offsets, int32_t* route_to_row,
                       int32_t* row_to_route, int32_t* num_rows, void* stream);

/* Host side of the layout's single synchronisation: blocks until the most recent dpep_layout launched on ws has
 * run, then returns R and (optionally) the rows per local expert.  Replaces the device-to-host read-back that sizes
 * the outputs of a fresh dispatch (deep_ep/backends/mesh_clos/elastic.py:1476, `.cpu()` of the notify outputs):
 * the layout kernel writes these few words straight into pinned host memory owned by the workspace and this
 * call polls them, which costs a few microseconds less than a copy plus a stream wait.
 *   counts_host   int32 [num_local] host memory, may be NULL; num_local must equal the launched layout's
 *   num_rows_host int32 [1] host memory
 *   timeout_us    DPEP_ERUNTIME if the kernel has not reported by then (a layout launch that failed never will)
 * One layout may be outstanding per workspace; the call does not wait for anything but the layout kernel. */
int dpep_layout_wait(void* ws, int32_t* counts_host, int num_local, int32_t* num_rows_host, long long timeout_us);

/* Expand-permute payload dispatch: out[row(t,s)] = x[t] for every route with a row.
 * Replaces dispatch() (csrc/ops/dispatch.cpp:82-211 -> dispatch_kernel, csrc/kernels/dispatch/dispatch.cpp:628)
 * and the scatter half of expand() (csrc/direct/kernels/expand/expand.cpp:334-520).
 *   row_bytes     bytes per payload row (BF16: 2H, FP8: H); must be a multiple of 16
 *   scales        optional fp32 [T, scale_cols] side rows moved with the payload (FP8 per-128 scales)
 *   topk_weights  optional fp32 [T,K]; out_weights[row] = topk_weights[t,s]
 *   num_rows      R (host value from dpep_layout_wait), or -1 when the host does not know R yet: the launch then
 *                 does not depend on R, out / out_scales / out_weights must hold T*K rows and the first R are
 *                 written.  A caller that allocates at capacity can thus queue layout and dispatch back to back
 *                 and read R (to narrow its outputs) while they run. */
int dpep_dispatch_copy(const void* x, const float* scales, const float* topk_weights,
                       const int32_t* route_to_row, const int32_t* row_to_route, int num_tokens,
                       int num_topk, int num_rows, int row_bytes, int scale_cols, void* out,
                       float* out_scales, float* out_weights, void* stream);

/* How dpep_dispatch_copy, dpep_dispatch_quant_fp8 and dpep_cast_to_fp8 store their payload rows; process-wide, no
 * counterpart in the reference (its rows leave through the transport).  Returns the policy in force before the call
 * (DPEP_STORE_QUERY changes nothing), or DPEP_EINVAL.
 *   DPEP_STORE_STREAMING  (default) non-temporal stores: the rows go to HBM past the caches, the kernel's time is the
 *                         time of its traffic and nothing is left for the next kernel to write back
 *   DPEP_STORE_THROUGH    write-through stores: the memory-side cache takes the rows first, so the kernel itself ends
 *                         sooner when that cache is clean and the kernel that follows pays for the write-back, unless it
 *                         is the reader of those rows and finds them there
 *   DPEP_STORE_CACHED     plain stores */
#define DPEP_STORE_THROUGH 0
#define DPEP_STORE_STREAMING 1
#define DPEP_STORE_CACHED 2
#define DPEP_STORE_QUERY 3
int dpep_dispatch_store_policy(int policy);

/* Fused per-128-element FP8 e4m3fn quantisation + expand-permute: the reference's caller-side
 * per_token_cast_to_fp8 (deep_ep/utils/math.py:45-61) followed by the FP8 dispatch above, in one pass.
 *   x             bf16 [T,H], H % 128 == 0
 *   out           fp8  [R,H]; out_scales fp32 [R, H/128]
 *   num_rows      R or -1, as for dpep_dispatch_copy */
int dpep_dispatch_quant_fp8(const void* x, const float* topk_weights, const int32_t* route_to_row,
                            const int32_t* row_to_route, int num_tokens, int num_topk, int num_rows,
                            int hidden, void* out, float* out_scales, float* out_weights, void* stream);

/* Routing layout and payload dispatch of a small batch (at most 2048 routes: a decode step) in ONE launch.
 * Replaces the low-latency dispatch (csrc/ops/low_latency.cpp:80-216 -> dispatch_low_latency, csrc/kernels/dispatch/
 * low_latency.cpp:73), which likewise derives the rows inside the payload kernel instead of running notify first; for
 * larger batches dpep_layout followed by dpep_dispatch_copy / dpep_dispatch_quant_fp8 produce the same results.
 * Every workgroup works out the rows of its own token from the whole routing table (which fits its LDS), so nothing
 * waits for a layout kernel.  Arguments as for dpep_layout plus dpep_dispatch_copy (quantize == 0: x of row_bytes
 * bytes per token, optional scales and weights) or dpep_dispatch_quant_fp8 (quantize != 0: x BF16, row_bytes = 2H,
 * H % 128 == 0, out FP8 + out_scales FP32 [.,H/128]).  out / out_scales / out_weights must hold T*K rows; the first R are
 * written.  The per-expert counts and R also go to the workspace's host mailbox: dpep_layout_wait works as after
 * dpep_layout. */
int dpep_layout_dispatch_small(void* ws, const int64_t* topk_idx, const void* x, const float* scales,
                               const float* topk_weights, int num_tokens, int num_topk, int num_experts, int expert_begin,
                               int num_local, int row_bytes, int scale_cols, int quantize, int32_t* counts, int32_t* psum,
                               int32_t* offsets, int32_t* route_to_row, int32_t* row_to_route, int32_t* num_rows, void* out,
                               float* out_scales, float* out_weights, void* stream);

/* Stand-alone per-128 quantiser (deep_ep/utils/math.py:45-61): x bf16 [T,H] -> fp8 [T,H], fp32 [T,ceil(H/128)].
 * H % 16 == 0; a last block shorter than 128 is quantised as if padded with zeros (math.py:52-53). */
int dpep_cast_to_fp8(const void* x, int num_tokens, int hidden, void* out, float* out_scales, void* stream);

/* The dequantiser the reference checks its FP8 path with: out = bf16(fp32(code) * scale), one scale per block of 128
 * columns (per_token_cast_back, deep_ep/utils/math.py:64-79).  scales: fp32 [T, ceil(H/128)], or, scales_are_e8m0_bytes
 * != 0, one exponent byte per block (the reference's int32 scale tensors hold four of them each, math.py:74-76).
 * H % 16 == 0; the last block of a row may be short.  codes e4m3fn [T,H] -> out bf16 [T,H]. */
int dpep_cast_back(const void* codes, const void* scales, int scales_are_e8m0_bytes, int num_tokens, int hidden, void* out,
                   void* stream);

/* Combine: out[t] = bf16_rne( sum over slots in order, skipping -1, of fp32(y[row]) (* w[row]) ).
 * Replaces combine() (csrc/ops/combine.cpp:198-326 -> combine_kernel, csrc/kernels/combine/combine.cpp:2965)
 * with row_weights == NULL, and aggregate() / the low-latency combine
 * (csrc/direct/ops/aggregate.cpp:44-143, csrc/direct/kernels/aggregate/aggregate_impl.h:166-226,
 * csrc/kernels/combine/low_latency.cpp:41) with row_weights != NULL.
 *   y             bf16 [R,H], H % 8 == 0
 *   row_weights   optional fp32 [R]: multiply each row before the add (separate mul and add)
 *   return_in     optional fp32 [R]: weight-return channel; return_out[t,s] = return_in[row], 0 without a row
 *   out           bf16 [T,H];  return_out fp32 [T,K] */
int dpep_combine(const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens,
                 int num_topk, int num_rows, int hidden, void* out, const float* return_in,
                 float* return_out, void* stream);

/* dpep_combine that writes only the tokens that own at least one row and leaves the others' rows of `out` untouched.
 * For one rank's receive share of an EP job most candidate tokens own no row here, and in the reference nothing is
 * produced for them on this rank at all (a rank returns rows only for the routes it served,
 * csrc/kernels/combine/combine.cpp:2965); dpep_combine zero-fills them, which is what a single-rank caller needs. */
int dpep_combine_served(const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens,
                        int num_topk, int num_rows, int hidden, void* out, const float* return_in,
                        float* return_out, void* stream);

/* The same combine for IEEE half rows and output (the low-latency path accepts BF16 or FP16 expert outputs and
 * returns the same dtype: deep_ep/backends/mesh_clos/elastic.py:596-606; oracle expected_combine,
 * tests/elastic/test_ep_low_latency.py:449-463): fp32 accumulation in slot order, one RNE rounding to half. */
int dpep_combine_fp16(const void* y, const float* row_weights, const int32_t* route_to_row, int num_tokens,
                      int num_topk, int num_rows, int hidden, void* out, const float* return_in,
                      float* return_out, void* stream);

/* MXFP8 activation quantiser, block 32 (quantize_input, experiments/megamoe/python/
 * deep_ep_experimental/megamoe/reference.py:44-54; device ComputeMxScale/QuantizeMxFp8Data).
 *   x bf16 [B,H], H % 32 == 0 -> codes e4m3 [B,H], scales e8m0 [B,H/32] */
int dpep_mx_quant(const void* x, int rows, int hidden, void* codes, uint8_t* scales, void* stream);

/* Host-only check of the grouped GEMM's copy/wait schedule; no counterpart in the reference (it is how this build
 * shows, without a GPU, that for a workgroup that walks `tiles_per_workgroup` tiles of `tile_rows` (64, 128 or 192)
 * rows and `ktiles` k tiles of 128 every asynchronous copy is covered by a counted wait before it is read, under
 * in-order completion of vector-memory operations: an item's operands before its MFMAs, the next tile's gather
 * indices before the copy cursor switches tiles), and that a ring slot of scale bytes is refilled only when the span of k
 * tiles it held has been read to the end.  epilogue_stores = stores a tile end issues (they only make the
 * counted waits stricter).  without_drain: bit 0 replays the schedule WITHOUT the cursor's wait at tile switches (what a
 * kernel that trusted every index fetch would do): the check then has to fail for tiles shorter than the copies run ahead;
 * bit 1 replays rings of two scale slots instead of the kernel's three: the check then has to fail where k is no multiple
 * of 512 and a workgroup has several tiles; that they do fail is how the tests know that the check can.
 * Returns 0, or DPEP_EINVAL with the first violation in dpep_last_error(). */
int dpep_megamoe_schedule_check(int tile_rows, int tiles_per_workgroup, int ktiles, int epilogue_stores, int without_drain);
/* The same check for the kernel that runs where K is a multiple of 512 (its waves split the tile's columns and load their
 * weights straight into registers; k tiles come in fours).  slack = operations the replayed wait allows in flight beyond
 * the kernel's own count: with slack > 0 the check has to fail, which is how the tests know that it can. */
int dpep_megamoe_schedule_check_column_waves(int tile_rows, int tiles_per_workgroup, int ktiles, int epilogue_stores, int slack);

/* Bytes of workspace dpep_megamoe_forward needs (buffer_size(), experiments/megamoe/csrc/forward.cpp:480).
 * num_shared = number of shared experts (0..8) whose rows (every token, each) are held next to the routed ones. */
size_t dpep_megamoe_workspace_bytes(int num_tokens, int num_topk, int hidden, int intermediate, int num_local,
                                    int num_shared);

/* What the grouped GEMM works on for a logical hidden or intermediate size: whole 256-column tiles and whole spans of
 * scales, at least 512 (dim <= 512 -> 512, else the next multiple of 256).  Prepared weights are padded to it when
 * they are prepared (zero codes, scale 1.0), input rows by a copy inside the forward; 0 for dim < 1.
 * (The reference accepts hidden % 64 == 0 and intermediate_hidden % 128 == 0, api.py:93-105.) */
int dpep_megamoe_padded_dim(int dim);

/* Shape of the prepared form of one raw weight tensor [L,N,K/2] + [L,N,K/32]: packed [L,padded_n,padded_k/2] and scales
 * [L,padded_n,scale_cols] (the scales are stored in spans of four k tiles = k 512, the last span padded).
 * N % 64 == 0 (gate_up: N = 2I with I % 128 == 0, both halves padded separately), K % 64 == 0.
 * (Part of the transform_weights_for_mega_moe contract below.) */
int dpep_megamoe_prepared_shape(int n, int k, int gate_up, int* padded_n, int* padded_k, int* scale_cols);

/* One-off weight re-layout (transform_weights_for_mega_moe, experiments/megamoe/python/.../api.py:311-379):
 * raw packed FP4 [L,N,K/2] + e8m0 [L,N,K/32]  ->  the tile order the GEMM kernel streams, padded as
 * dpep_megamoe_prepared_shape says (out_packed and out_scales have those sizes).  Byte shuffle only.
 * gate_up != 0 (first GEMM, N = 2I, gate rows then up rows) interleaves gate and up in groups of 32 output columns so
 * SwiGLU is lane-local (the counterpart of _interleave_gate_up_128, api.py:285-293). */
int dpep_megamoe_prepare_weights(const uint8_t* w_packed, const uint8_t* w_scales, int num_local, int n,
                                 int k, int gate_up, uint8_t* out_packed, uint8_t* out_scales, void* stream);

/* Diagnosis, no counterpart in the reference: what the idle workgroups of the most recent dpep_megamoe_forward's first
 * GEMM did (see "gemm_zero_fill").  Waits for `stream`, then reports the number of filler waves of that launch (0: the
 * launch had a tile for every workgroup, or zero fill is off) and the tokens they looked at before they were told to
 * stop.  The sizes are those of the forward call. */
int dpep_megamoe_fill_report(void* ws, int num_tokens, int num_topk, int hidden, int intermediate, int num_local,
                             int num_shared, int32_t* fillers_host, int64_t* tokens_filled_host, void* stream);

/* Fused W4A8 MoE forward for one rank's local experts (Plan::forward, experiments/megamoe/csrc/forward.cpp:340-478
 * -> mega_moe_kernel_do, kernel_launch.hpp:8-13):
 * layout -> gather rows -> GMM1 (MXFP8 x MXFP4) -> bf16 -> SwiGLU -> MXFP8 requant -> GMM2 -> bf16 ->
 * route-weighted fp32 reduce per token -> bf16.
 *   x_codes e4m3 [B,H], x_scales e8m0 [B,H/32], topk_idx int32 [B,K] (distinct, in [0,E)), topk_weights fp32 [B,K]
 *   H % 64 == 0, I % 128 == 0 (hidden / intermediate as the caller sees them)
 *   w1/s1: prepared GMM1 weights of the raw [L,2I,H/2] and scales; w2/s2: prepared GMM2 weights of the raw [L,H,I/2]
 *   and scales (sizes: dpep_megamoe_prepared_shape)
 *   shared_w1/s1/w2/s2: the same for num_shared shared experts ([S,2I,H/2] ...; sw1/sw2/ss1/ss2 of
 *   mega_moe_kernel_do), NULL when num_shared == 0.  A shared expert processes every token and its output is
 *   added with weight 1 after the routed experts' (golden.py:160-164).
 *   y bf16 [B,H]; expert_token_nums int32 [L] (routed experts only) */
int dpep_megamoe_forward(void* ws, const void* x_codes, const uint8_t* x_scales, const int32_t* topk_idx,
                         const float* topk_weights, const uint8_t* w1, const uint8_t* s1, const uint8_t* w2,
                         const uint8_t* s2, const uint8_t* shared_w1, const uint8_t* shared_s1,
                         const uint8_t* shared_w2, const uint8_t* shared_s2, int num_shared, int num_tokens, int hidden,
                         int intermediate, int num_topk, int num_experts, int expert_begin, int num_local, void* y,
                         int32_t* expert_token_nums, void* stream);

#ifdef __cplusplus
}
#endif
#endif
