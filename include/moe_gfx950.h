/*
 * moe_gfx950.h -- C ABI of libmoe_gfx950.so: the MoE dispatch / expert hot path as
 * hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions
 *  - every pointer is a DEVICE pointer unless the comment says "host";
 *  - every call only enqueues work on `stream` (a hipStream_t passed as void*); nothing here
 *    synchronises, allocates or frees device memory: outputs and workspaces are the caller's;
 *  - return value: MOE_OK or a negative MOE_ERR_* code; moe_last_error() gives the text for the
 *    calling thread;
 *  - counts / offsets / indices are int32, contiguous (reference utils.py:14-17,31);
 *  - `dtype` is the activation storage type (MOE_F32 or MOE_BF16); rows must be a multiple of
 *    16 bytes long (H % 4 == 0 for f32, H % 8 == 0 for bf16);
 *  - expert ex lives on rank ex / E_l as local expert ex % E_l (reference utils.py:217-218).
 *
 * The reference has no FFI: its operator API is Python (utils.py, the layers/ files).  Each entry
 * point below names the reference routine whose device work it replaces.
 */
#ifndef MOE_GFX950_H
#define MOE_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* moe_stream_t; /* hipStream_t */

enum { MOE_F32 = 0, MOE_BF16 = 1 };
enum { MOE_ACT_NONE = 0, MOE_ACT_GELU = 1, MOE_ACT_SILU = 2, MOE_ACT_SWIGLU = 3 };
enum {
    MOE_OK = 0,
    MOE_ERR_INVALID = -1,     /* bad argument (shape, alignment, null pointer) */
    MOE_ERR_UNSUPPORTED = -2, /* valid but outside what the kernels cover */
    MOE_ERR_WORKSPACE = -3,   /* workspace too small */
    MOE_ERR_LAUNCH = -4       /* HIP reported a launch error */
};

/* Limits of the kernels. */
#define MOE_MAX_EXPERTS 512
#define MOE_MAX_TOPK 16
#define MOE_COUNT_BLOCK 64 /* tokens per counting block */

int moe_abi_version(void);
/* Text of the last error on the calling thread ("" if none). host pointer, valid until the next call. */
const char* moe_last_error(void);

/* ---- a1: router softmax + top-k ------------------------------------------------------------
 * Replaces `F.softmax(einsum('th,he->te', tokens, router)); topk(...)` (reference utils.py:200-202).
 * Pinned fp32 arithmetic: h is cut into MOE_ROUTE_SEGMENTS contiguous segments of L = ceil(H/8) rounded up
 * to a multiple of 8 elements; s_p = fmaf chain over the h of segment p in ascending order from +0 (an
 * empty segment gives +0); logits[t,e] = ((..(s_0 + s_1) + ..) + s_7) + bias[e], fp32 additions in that
 * order.  Selection on the logits, descending, ties to the lower expert id; topk_gate = softmax
 * probability of each selected expert (not renormalised).  x [T,H], router [H,E] in `dtype`; bias fp32
 * [E] or NULL.  logits: fp32 [T,E] output (the raw logits).  ws: moe_route_workspace_bytes(T,E) bytes of
 * scratch (the segments' partial sums).   ws and logits must be 16-byte aligned. */
#define MOE_ROUTE_SEGMENTS 8
size_t moe_route_workspace_bytes(int T, int E);
int moe_route_topk(const void* x, const void* router, const float* bias, int dtype, int T, int H, int E,
                   int k, float* logits /*[T,E]*/, int32_t* topk_idx /*[T,k]*/, float* topk_gate /*[T,k]*/,
                   void* ws, size_t ws_bytes, moe_stream_t stream);

/* ---- a2/a4/a5/a6/a7 + payload order of a3 ----------------------------------------------------
 * Replaces the bucket loop and count/offset bookkeeping of route_and_pack_padding_free
 * (reference utils.py:204-238), build_expert_offsets (utils.py:20-31), _build_dst_offsets
 * (benchmark.py:44-49) and the local part of compute_capacity_from_pca (utils.py:118-121).
 * Outputs: send_counts [W,E_l]; expert_offs [W,E_l] (exclusive prefix inside each dst block);
 * dst_sizes [W]; dst_offsets [W]; caps[0] = max(1, max dst_sizes) (this shard's bound on M),
 * caps[1] = max(1, max send_counts) (its bound on CAP); pos [T,k] = row of slot (t,kk) in the
 * padding-free payload ((dst, el, token) order); row_token [T*k] = token of payload row r. */
size_t moe_count_workspace_bytes(int T, int k, int E);
int moe_count_and_offsets(const int32_t* topk_idx, int T, int k, int E, int W, int32_t* send_counts,
                          int32_t* expert_offs, int32_t* dst_sizes, int32_t* dst_offsets, int32_t* caps,
                          int32_t* pos, int32_t* row_token, void* ws, size_t ws_bytes, moe_stream_t stream);

/* moe_count_and_offsets for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  Same arguments and results
 * without the workspace: the scratch is a fixed MOE_COUNT_SCRATCH_BYTES array inside the library's device image,
 * one copy per GPU, held until the process ends.  Sizes whose moe_count_workspace_bytes(T,k,E) exceed it are
 * rejected with MOE_ERR_WORKSPACE.  All calls on one GPU share that array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and safe.  Nothing is allocated or freed. */
#define MOE_COUNT_SCRATCH_BYTES (4u << 20)
size_t moe_count_static_scratch_bytes(void);
int moe_count_and_offsets_static(const int32_t* topk_idx, int T, int k, int E, int W, int32_t* send_counts,
                                 int32_t* expert_offs, int32_t* dst_sizes, int32_t* dst_offsets, int32_t* caps,
                                 int32_t* pos, int32_t* row_token, moe_stream_t stream);

/* ---- a4/a5 on their own: build_expert_offsets (reference utils.py:20-31) and _build_dst_offsets
 * (benchmark.py:44-49) for a given counts [W,E_l].  dst_sizes / dst_offsets may be NULL. */
int moe_build_expert_offsets(const int32_t* counts, int W, int E_l, int32_t* expert_offs, int32_t* dst_sizes,
                             int32_t* dst_offsets, moe_stream_t stream);

/* ---- a7: M / CAP over several shards ---------------------------------------------------------
 * out[0] = max(1, max_i values[i]) (README.md:4-7 for M; utils.py:121 for the floor).  Stands
 * in for the all-reduce MAX of compute_capacity_from_pca when all shards live on one GPU. */
int moe_max_floor1(const int32_t* values, int n, int32_t* out, moe_stream_t stream);

/* ---- a3: padding-free payload (reference utils.py:235-246) ------------------------------------
 * payload[r,:] = x[row_token[r],:], r < R. */
int moe_pack_payload(const void* x, int dtype, int T, int H, const int32_t* row_token, int R, void* payload,
                     moe_stream_t stream);

/* ---- a8: fixed [W,M,H] send layout (reference README.md:5-7) ----------------------------------
 * send[dst,m,:] = x[row_token[dst_offsets[dst]+m],:] for m < dst_sizes[dst], else zeros.
 * map_ws: unused (kept for ABI stability; may be NULL).  status (nullable): set to 1 if some
 * dst_sizes[dst] > M (rows beyond M are dropped). */
int moe_pack(const void* x, int dtype, int T, int H, const int32_t* row_token, const int32_t* dst_sizes,
             const int32_t* dst_offsets, int W, int M, void* send_buf, int32_t* map_ws, int32_t* status,
             moe_stream_t stream);

/* The same send buffer, written token by token: every token row is read once and stored to the k slots
 * send[dst,m,:] with dst = topk_idx[t,kk] / E_l, m = pos[t,kk] - dst_offsets[dst] (pos as returned by
 * moe_count_and_offsets), padding rows zeroed; bit-identical to moe_pack with k times fewer token reads.
 * Restates the same README.md:5-7 layout from the per-token side of utils.py:210-219. */
int moe_pack_tokens(const void* x, int dtype, int T, int H, const int32_t* topk_idx, const int32_t* pos, int k,
                    int E_l, const int32_t* dst_sizes, const int32_t* dst_offsets, int W, int M, void* send_buf,
                    int32_t* status, moe_stream_t stream);

/* moe_pack_tokens that also ships each slot's top-k gate: send_gate[dst,m] = gate[t,kk] (fp32 [W,M], zero in the padding
 * slots), for a destination that multiplies the expert's result rows by their gates before it returns them
 * (moe_recv_row_map_gated, moe_grouped_gemm_mapped_gated) so that the source only adds (moe_combine with gate == NULL).
 * gate [T,k] as moe_route_topk returns it.  The reference drops the gates (utils.py:202) and has no return path: this
 * carries the same README.md:5-7 layout one column further. */
int moe_pack_tokens_gated(const void* x, int dtype, int T, int H, const int32_t* topk_idx, const int32_t* pos,
                          const float* gate, int k, int E_l, const int32_t* dst_sizes, const int32_t* dst_offsets, int W, int M,
                          void* send_buf, float* send_gate, int32_t* status, moe_stream_t stream);

/* The fp8 form of the same send buffer (BASELINE workload "quantized skew sweep": activations quantised per token to
 * e4m3 for the fp8 grouped GEMM).  Per-row quantisation commutes with moving rows, so the tokens can be quantised where
 * they are packed: send_q [W,M,H] codes and send_scale [W,M] hold, slot for slot, what moe_quantize_rows_fp8 would make
 * of moe_pack_tokens' bf16 buffer (padding slots: codes 0, scale 1), half the bytes cross, and the destination hands both
 * to moe_grouped_mlp_fp8_q_mapped without a quantisation pass of its own.  x is bf16.  Same README.md:5-7 layout. */
int moe_pack_tokens_fp8(const void* x_bf16, int T, int H, const int32_t* topk_idx, const int32_t* pos, int k, int E_l,
                        const int32_t* dst_sizes, const int32_t* dst_offsets, int W, int M, uint8_t* send_q,
                        float* send_scale, int32_t* status, moe_stream_t stream);

/* moe_pack_tokens_fp8 that also ships the gates (send_gate [W,M], as moe_pack_tokens_gated). */
int moe_pack_tokens_fp8_gated(const void* x_bf16, int T, int H, const int32_t* topk_idx, const int32_t* pos, const float* gate,
                              int k, int E_l, const int32_t* dst_sizes, const int32_t* dst_offsets, int W, int M, uint8_t* send_q,
                              float* send_scale, float* send_gate, int32_t* status, moe_stream_t stream);

/* ---- a9: receive layout (reference baseline.py:178-222; kernels.py:93-102,124-125) ------------
 * recv [W,M,H]: slot s holds what source s sent to this rank ((el, token) order, zero padded);
 * recv_counts [W,E_l]: recv_counts[s,e] rows from source s for local expert e.
 * token_buf[e,s,j,:] = recv[s, expert_offs_s[e]+j, :] for j < recv_counts[s,e], else zeros;
 * pca[e,s] = recv_counts[s,e].  status (nullable): 1 on count > CAP, or when a counted row lies at or
 * past row M of its slot (the sender's pack dropped it: it reads as zeros).
 * map_ws (here and in every entry point below that takes one): int32 scratch of
 * moe_recv_map_ints(W, E_l, n_out) elements (prefix tables over the counts; n_out = rows of the
 * output buffer, which no longer enters the size). */
size_t moe_recv_map_ints(int W, int E_l, int n_out);
int moe_unpack_token_buf(const void* recv, int dtype, int W, int M, int H, const int32_t* recv_counts, int E_l,
                         int CAP, void* token_buf, int32_t* pca, int32_t* map_ws, int32_t* status,
                         moe_stream_t stream);

/* Same placement from a padding-free flat payload (src-major, expert-minor blocks): the device
 * form of reorder_flat_to_token_buf (reference baseline.py:178-222).  flat [R,H]. */
int moe_reorder_flat_to_token_buf(const void* flat, int dtype, int R, int H, const int32_t* recv_counts, int W,
                                  int E_l, int CAP, void* token_buf, int32_t* map_ws, int32_t* status,
                                  moe_stream_t stream);

/* ---- a10: expert-major unpack (reference layers/token_shuffle.py:31-56; kernels.py:179-205) ---
 * shuffled[off[e,s]+j,:] = token_buf[e,s,j,:], off = exclusive prefix of pca over flattened (e,s).
 * S_rows = rows allocated in `shuffled` (>= sum pca); rows past the sum are zero-filled.
 * expert_cnt (nullable) [E_l] = sum_s pca[e,s] (reference layers/expert.py:26-27).
 */
int moe_shuffle(const void* token_buf, int dtype, int E_l, int W, int CAP, int H, const int32_t* pca,
                void* shuffled, int S_rows, int32_t* expert_cnt, int32_t* map_ws, moe_stream_t stream);

/* recv [W,M,H] -> shuffled [S_rows,H] directly (token_buf never materialised).  A counted row that lies at
 * or past row M of its slot was dropped by the sender's pack and reads as zeros. */
int moe_unpack_expert_major(const void* recv, int dtype, int W, int M, int H, const int32_t* recv_counts,
                            int E_l, void* shuffled, int S_rows, int32_t* expert_cnt, int32_t* map_ws,
                            moe_stream_t stream);

/* ---- a11: grouped GEMM (reference layers/expert.py:31-60; kernels.py:240-289) -----------------
 * out[rows of e] = tokens[rows of e] @ weights[e], fp32 accumulate, cast to `dtype`;
 * rows of e = [sum cnt[:e], +cnt[e]).  tokens [S_rows,K]; weights [E_l,K,N] (N contiguous, the
 * reference layout); out [S_rows,N].  Rows past sum(cnt) are left untouched.
 * For bf16 the weights are re-tiled into ws first (moe_prepack_bytes(...) bytes). */
size_t moe_prepack_bytes(int dtype, int E_l, int K, int N);
int moe_grouped_gemm(const void* tokens, const void* weights, const int32_t* expert_cnt, int dtype, int S_rows,
                     int K, int N, int E_l, void* out, void* ws, size_t ws_bytes, moe_stream_t stream);

/* One-time weight re-tiling for the MFMA kernels: [E_l,K,N] (N contiguous) -> K-contiguous rows grouped
 * in K slabs ([E_l][K/slab][Npad][slab], Npad = N rounded up to the kernel's N tile; the layout is
 * private to the kernels).  With w_up != NULL the two
 * matrices are interleaved in 32-column groups (gate, up, gate, up, ...) so one kernel computes
 * silu(x Wg) * (x Wu); the packed matrix then has 2N columns. */
int moe_prepack_weights(const void* w, const void* w_up, int dtype, int E_l, int K, int N, void* packed,
                        moe_stream_t stream);

/* One bf16 grouped GEMM on pre-packed weights with a fused epilogue: out [S_rows,N] =
 * act(tokens [S_rows,K] @ W[g]) per group; for MOE_ACT_SWIGLU `packed` holds (Wg,Wu) interleaved and
 * out = silu(x Wg) * (x Wu).  K % 64 == 0, N % 8 == 0.  (The two halves of moe_grouped_mlp.) */
int moe_grouped_gemm_packed(const void* tokens, const void* packed, const int32_t* expert_cnt, int S_rows, int K,
                            int N, int E_l, int act, void* out, moe_stream_t stream);

/* ---- a12: expert MLP (not in the reference; shapes from the workload descriptions) ------------
 * act GELU/SILU: y = act(x W1) W2;  SWIGLU: y = (silu(x Wg) * (x Wu)) Wd.
 * MOE_BF16: w1 = moe_prepack_weights(W1 or (Wg,Wu)) with K=H, N=F; w2 = moe_prepack_weights(W2)
 * with K=F, N=H; w_up must be NULL; H and F multiples of 64.
 * MOE_F32: w1 [E_l,H,F], w_up [E_l,H,F] (SwiGLU only, else NULL), w2 [E_l,F,H], reference layout.
 * hidden_ws: [S_rows,F] in `dtype`.  fp32 accumulation; hidden activation and output rounded
 * once to `dtype`. */
int moe_grouped_mlp(const void* tokens, const int32_t* expert_cnt, int dtype, int S_rows, int H, int F,
                    int E_l, int act, const void* w1, const void* w_up, const void* w2, void* hidden_ws,
                    void* out, moe_stream_t stream);

/* fp8 (OCP e4m3) SwiGLU expert.  Weights: e4m3 codes pre-packed like the bf16 ones (1 byte per
 * element) with per-output-channel fp32 scales (sg, su [E_l,F]; sd [E_l,H]).  The input rows (bf16) are quantised per
 * row inside (scale amax/448): xq_ws [S_rows,H] u8, xs_ws [S_rows] f32.  The hidden activation silu(g) * u is
 * quantised by the first GEMM's epilogue, from its fp32 values, in blocks of one row x 32 columns: scale 2^(b-127), the
 * smallest power of two under which the block's largest magnitude is at most 448, codes = e4m3(value / scale):
 * hq_ws [S_rows,F] u8 and hscale_ws [S_rows, F/32] u8 (the bytes b).  The down projection multiplies the codes with
 * the scales applied inside the matrix instruction; epilogue acc * s_ch[n] (* row_gate[m] where given).  H and F
 * multiples of 128. */
int moe_prepack_weights_fp8(const uint8_t* w, const uint8_t* w_up, int E_l, int K, int N, uint8_t* packed,
                            moe_stream_t stream);
int moe_quantize_rows_fp8(const void* x_bf16, int rows, int cols, uint8_t* q, float* scale,
                          const int32_t* n_rows_dev, moe_stream_t stream);
int moe_grouped_mlp_fp8(const void* tokens_bf16, const int32_t* expert_cnt, int S_rows, int H, int F, int E_l,
                        const uint8_t* wgu_packed, const float* sg, const float* su, const uint8_t* wd_packed,
                        const float* sd, uint8_t* xq_ws, float* xs_ws, uint8_t* hq_ws, uint8_t* hscale_ws, void* out,
                        moe_stream_t stream);

/* ---- a10 + a11/a12 + a13 without the two row copies ------------------------------------------------
 * The expert-major unpack (token_shuffle.py:31-56) and the return pack only move rows; the grouped GEMM
 * can read its input rows where the transfer left them and write its result rows where the way back
 * wants them.  Three entry points make that path:
 *   moe_recv_row_map        row_map[r] = row of the [W,M,H] receive buffer that holds expert-major row r
 *                           (r < n_rows; rows past the received total map to row 0; rows dropped by the
 *                           sender's pack, at or past row M of their slot, map to -1), expert_cnt (nullable)
 *                           as in moe_unpack_expert_major; map_ws: unused (kept for ABI stability; may be NULL).
 *                           The same map is the destination of result row r in the returned buffer.
 *   moe_grouped_gemm_mapped moe_grouped_gemm_packed with row indirection: logical row r is read from row
 *                           a_row_map[r] of a_base (a_rows rows of K, under 4 GiB) and written to row
 *                           c_row_map[r] of out (out_rows rows of N); either map may be NULL (identity).
 *                           Map entries must lie inside their buffers or be negative: a negative a_row_map
 *                           entry reads row 0, a negative c_row_map entry stores nothing.  part_ws (nullable, part_ws_bytes
 *                           bytes, moe_gemm_part_workspace_bytes() for the full benefit): scratch for fp32
 *                           partial sums; with it, when the last round of the persistent grid holds at most
 *                           a quarter of a grid of tiles, those tiles are cut along K over the idle compute
 *                           units and summed in a fixed order by a second kernel (same result for the same
 *                           shapes and counts on every call; last-bit differences against the unsplit sum).
 *   moe_zero_padding_rows   rows [sum_e recv_counts[s,e], M) of every slot s of buf [W,M,H] <- 0: what
 *                           moe_return_pack writes besides the result rows. */
int moe_recv_row_map(const int32_t* recv_counts, int W, int E_l, int M, int n_rows, int32_t* row_map,
                     int32_t* expert_cnt, int32_t* map_ws, moe_stream_t stream);
int moe_grouped_gemm_mapped(const void* a_base, int a_rows, const int32_t* a_row_map, const void* packed,
                            const int32_t* expert_cnt, int S_rows, int K, int N, int E_l, int act, void* out,
                            int out_rows, const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes,
                            moe_stream_t stream);
/* Two more forms of the row map, for the two ways the fused destination side is widened:
 *   moe_recv_row_map_flat   the receive buffer is a padding-free flat payload [sum recv_counts, H] instead of [W,M,H]:
 *                           source-major, expert-minor blocks, what each source's send_payload[dst_offsets[dst] ..] holds
 *                           (reference utils.py:235-246) and reorder_flat_to_token_buf reads (baseline.py:204-218);
 *                           row_map[r] = start of block (s,e) + j.  No row can have been dropped, nothing is padding; the
 *                           same map places result row r in a flat returned buffer.
 *   moe_recv_row_map_gated  M >= 1: moe_recv_row_map; M == 0: moe_recv_row_map_flat; with recv_gate (fp32, one per row of
 *                           the receive buffer, as moe_pack_tokens_gated ships them) also row_gate[r] = recv_gate[row_map[r]]
 *                           (0 for rows without a source), the row gates in the GEMM's row order.  Both or neither.
 *   moe_grouped_gemm_mapped_gated  moe_grouped_gemm_mapped without activation whose result row r is multiplied by
 *                           row_gate[r] in fp32 before the one rounding to bf16: the down projection of an expert MLP whose
 *                           rows return already weighted (the combine then only adds: moe_combine with gate == NULL). */
int moe_recv_row_map_flat(const int32_t* recv_counts, int W, int E_l, int n_rows, int32_t* row_map, int32_t* expert_cnt,
                          moe_stream_t stream);
int moe_recv_row_map_gated(const int32_t* recv_counts, int W, int E_l, int M, int n_rows, const float* recv_gate,
                           int32_t* row_map, float* row_gate, int32_t* expert_cnt, moe_stream_t stream);
int moe_grouped_gemm_mapped_gated(const void* a_base, int a_rows, const int32_t* a_row_map, const void* packed,
                                  const int32_t* expert_cnt, int S_rows, int K, int N, int E_l, const float* row_gate, void* out,
                                  int out_rows, const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes,
                                  moe_stream_t stream);
size_t moe_gemm_part_workspace_bytes(void);
/* How a launch with total_tiles output tiles, a persistent grid of `grid` workgroups, k_stages 64-byte stages of K
 * (even) and room for max_units part tiles in the workspace is walked: out[0] = tiles taken whole, out[1] = parts
 * per remaining tile (1: no split), out[2] = K stages per part, out[3] = work units in all.  Host-only arithmetic
 * (the kernels evaluate the same function); no counterpart in the reference. */
int moe_gemm_split_plan(int total_tiles, int grid, int k_stages, int max_units, int32_t* out);
int moe_zero_padding_rows(void* buf, int dtype, int W, int M, int H, const int32_t* recv_counts, int E_l,
                          moe_stream_t stream);
/* Gradient of moe_shuffle (the reference leaves TokenShuffle.backward empty, token_shuffle.py:58-60):
 * grad_token_buf[e,s,j,:] = grad_rows[off[e,s]+j,:] for j < pca[e,s], zeros in the padding; off as in moe_shuffle.
 * map_ws >= moe_recv_map_ints(W,E_l,0) ints. */
int moe_shuffle_backward(const void* grad_rows, int dtype, int E_l, int W, int CAP, int H, const int32_t* pca,
                         void* grad_token_buf, int32_t* map_ws, moe_stream_t stream);
/* moe_grouped_mlp_fp8 with the same row indirection: the row quantisation reads input row r from row
 * a_row_map[r] of a_base_bf16 (a_rows rows of H), the down GEMM writes result row r to row c_row_map[r]
 * of out (out_rows rows of H); either map may be NULL.  row_gate (nullable, fp32 [S_rows], as moe_recv_row_map_gated
 * returns it): result row r is multiplied by row_gate[r] before the one rounding (the gated return).  part_ws
 * (nullable): the K-split scratch of moe_grouped_gemm_mapped, used by both GEMMs in turn. */
int moe_grouped_mlp_fp8_mapped(const void* a_base_bf16, int a_rows, const int32_t* a_row_map,
                               const int32_t* expert_cnt, int S_rows, int H, int F, int E_l,
                               const uint8_t* wgu_packed, const float* sg, const float* su, const uint8_t* wd_packed,
                               const float* sd, uint8_t* xq_ws, float* xs_ws, uint8_t* hq_ws, uint8_t* hscale_ws,
                               const float* row_gate, void* out, int out_rows, const int32_t* c_row_map, void* part_ws,
                               size_t part_ws_bytes, moe_stream_t stream);

/* moe_grouped_mlp_fp8_mapped for rows that arrive quantised (moe_pack_tokens_fp8): a_q [a_rows,H] codes and a_scale
 * [a_rows] scales, gathered through a_row_map (nullable) by the first GEMM as it loads them; xs_ws [S_rows] receives the
 * scales in the GEMM's row order.  Everything else as in moe_grouped_mlp_fp8_mapped, whose result it reproduces bit for
 * bit when a_q / a_scale are the quantised rows of that call's input. */
int moe_grouped_mlp_fp8_q_mapped(const uint8_t* a_q, const float* a_scale, int a_rows, const int32_t* a_row_map,
                                 const int32_t* expert_cnt, int S_rows, int H, int F, int E_l, const uint8_t* wgu_packed,
                                 const float* sg, const float* su, const uint8_t* wd_packed, const float* sd, float* xs_ws,
                                 uint8_t* hq_ws, uint8_t* hscale_ws, const float* row_gate, void* out, int out_rows,
                                 const int32_t* c_row_map, void* part_ws, size_t part_ws_bytes, moe_stream_t stream);

/* ---- gradients (every backward of the reference is an empty stub: layers/expert.py:62-64,
 * layers/token_shuffle.py:58-60, layers/all_to_all.py:121-123) -----------------------------------------------------
 * For out[rows of g] = x[rows of g] @ w[g]:
 *   d x[rows of g] = d out[rows of g] @ w[g]^T : moe_grouped_gemm_mapped on weights re-tiled by
 *                    moe_prepack_weights_transposed (moe_prepack_bytes(dtype, E_l, N, K) bytes; with w_up the pair
 *                    (w, w_up) is transposed together in the fused gate/up column order, N = columns of ONE matrix,
 *                    twice the bytes); fp32: moe_transpose_weights_f32 then moe_grouped_gemm.
 *   d w[g]         = x[rows of g]^T @ d out[rows of g] : moe_grouped_gemm_dw, one launch for all groups, the ragged row
 *                    count being the reduction dimension (both operands are first rewritten row-index-fastest, every
 *                    group padded to a multiple of 64 rows with zeros, into ws of moe_dw_workspace_bytes bytes);
 *                    groups without rows get zeros.  split_F > 0 (bf16): dy is [S_rows, 2 split_F] in the fused
 *                    gate/up column order and dw comes out as [E_l, K, 2 split_F] = [d w_gate | d w_up] side by side.
 * moe_mlp_act_backward: gradient through the activation of the expert MLP; a1 = pre-activations ([rows,F]; SwiGLU:
 *   [rows,2F] in the fused gate/up column order, as moe_grouped_gemm_mapped produces them with MOE_ACT_NONE), dh [rows,F],
 *   d_a1 in the layout of a1.
 * moe_combine_backward: d ret[slot(t,kk)] = gate[t,kk] * d out[t] (padding slots zeroed, like the pack) and
 *   d gate[t,kk] = <d out[t], ret[slot(t,kk)]>.  The gradient of the fixed-M pack is moe_combine with unit gates; that of
 *   the expert-major unpack is moe_return_pack, and the other way round; moe_shuffle_backward is declared above. */
/* moe_grouped_gemm_act_keep: moe_grouped_gemm_mapped with an activation (act != MOE_ACT_NONE; bf16; rows of `out` are not
 *   remapped) that ALSO stores the values before the activation, for the backward pass of the expert MLP
 *   (layers/expert.py:62-64 of the reference is an empty stub): pre_act [S_rows, N] bf16, for SwiGLU [S_rows, 2N] in the
 *   column order of the fused gate / up product (32 gate columns, their 32 up columns, ...), which is what
 *   moe_mlp_act_backward takes.  Same values as a launch with MOE_ACT_NONE on the same weights would give. */
int moe_grouped_gemm_act_keep(const void* a_base, int a_rows, const int32_t* a_row_map, const void* packed,
                              const int32_t* expert_cnt, int S_rows, int K, int N, int E_l, int act, void* out, void* pre_act,
                              void* part_ws, size_t part_ws_bytes, moe_stream_t stream);
int moe_prepack_weights_transposed(const void* w, const void* w_up, int dtype, int E_l, int K, int N, void* packed,
                                   moe_stream_t stream);
size_t moe_dw_workspace_bytes(int S_rows, int E_l, int K, int N);
int moe_grouped_gemm_dw(const void* x, const void* dy, const int32_t* expert_cnt, int dtype, int S_rows, int K, int N,
                        int E_l, int split_F, void* dw, void* ws, size_t ws_bytes, moe_stream_t stream);
int moe_transpose_weights_f32(const float* w, int E_l, int K, int N, float* out, moe_stream_t stream);
int moe_mlp_act_backward(const void* a1, const void* dh, int dtype, int rows, int F, int act, void* d_a1,
                         moe_stream_t stream);
int moe_combine_backward(const void* d_out, const void* ret, int dtype, int W, int M, int H, const int32_t* topk_idx,
                         const int32_t* pos, const float* gate, const int32_t* dst_sizes, const int32_t* dst_offsets, int T,
                         int k, int E_l, void* d_ret, float* d_gate, moe_stream_t stream);

/* ---- a13: return path and combine (not in the reference; defined by the task statement) -------
 * ret[s, expert_offs_s[e]+j, :] = y[off[e,s]+j, :], zero padding: the [W,M,H] buffer this rank
 * sends back, slot s in the order source s sent its rows. */
int moe_return_pack(const void* y, int dtype, int S_rows, int H, const int32_t* recv_counts, int W, int E_l,
                    int M, void* ret, int32_t* map_ws, moe_stream_t stream);

/* out[t,:] = sum_kk gate[t,kk] * ret[dst, pos[t,kk]-dst_offsets[dst], :], dst = idx[t,kk]/E_l;
 * fp32 multiply then add in ascending kk (no fma), one rounding to `dtype`.  gate == NULL: the rows arrive weighted
 * (moe_grouped_gemm_mapped_gated) and are only added, in the same order.  A flat returned payload [R,H] in payload order
 * (row = pos[t,kk]) is the case W = 1, M = R, E_l = number of experts, dst_offsets = {0}.  A slot whose dst lies
 * outside [0,W) or whose row lies outside [0,M) -- a row the pack dropped because the pair capacity
 * was exceeded -- has no returned row: it is skipped and *status (nullable) is set to 1. */
int moe_combine(const void* ret, int dtype, int W, int M, int H, const int32_t* topk_idx, const int32_t* pos,
                const float* gate, const int32_t* dst_offsets, int T, int k, int E_l, void* out,
                int32_t* status, moe_stream_t stream);

/* ---- diagnostics (no counterpart in the reference, no part of the hot path) ------------------------------------------
 * moe_diag_mfma_loop: a register-only MFMA loop in the grouped GEMM's wave layout (4 waves per workgroup, 128 x 128 outputs per
 * wave; bf16 on 16x16x32, fp8 on 32x32x64), `workgroups` workgroups, `iters` passes over the wave's MFMA tiles; operands all
 * zero (random_data = 0) or drawn like N(0,1) (random_data = 1: the matrix cores run against a power limit, and what they
 * sustain depends on the operand values).  sink: moe_diag_mfma_loop_sink_floats() floats of scratch.  The caller times the
 * launch; moe_diag_mfma_loop_flops gives its flop count.  Used by `bench.py --mfma-ceiling`. */
size_t moe_diag_mfma_loop_sink_floats(void);
double moe_diag_mfma_loop_flops(int fp8, int iters, int workgroups);
int moe_diag_mfma_loop(int fp8, int random_data, int iters, int workgroups, float* sink, moe_stream_t stream);

/* moe_diag_gemm_trace: where time goes inside the grouped GEMM.  After a call with a device buffer of `words` >=
 * moe_diag_gemm_trace_words() 64-bit words, the forward grouped-GEMM launches of the calling process (through any entry point
 * above; 256-row tiles, no activation or SwiGLU) run an instantiation of the same kernel that writes the device's 100 MHz wall
 * clock into the buffer, take whole tiles only (no K split of the last round), and overwrite what the launch before left:
 *   words [256 w, 256 w + 256) of workgroup w: for each of its tiles in turn, the clock at the start of the tile's K loop, at the
 *     end of its K loop and at the end of its epilogue (the first 85 tiles);
 *   words [256 G, 256 G + 4096), G = number of workgroups = compute units: the clock at the end of every MFMA block (one 64-byte
 *     K stage of a 256 x 256 tile) of workgroup 0.
 * flags: bit 0: the epilogue computes but stores nothing (what the stores cost); 0x100: only launches without activation are
 * traced (the down projection); 0x200: only launches with one (gate/up).  trace == NULL ends it.  Not thread-safe; the
 * launches compute the same results (unless bit 0 is set).  Used by `bench.py --gemm-phases`. */
size_t moe_diag_gemm_trace_words(void);
int moe_diag_gemm_trace(unsigned long long* trace, size_t words, int flags);

#ifdef __cplusplus
}
#endif
#endif /* MOE_GFX950_H */
