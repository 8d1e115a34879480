/*
 * mvllm.h - C ABI of the MI355X (gfx950) paged-KV decode path.
 *
 * Every entry point is a plain C function: raw device pointers, sizes and
 * strides in ELEMENTS, an explicit hipStream_t (passed as void*), and an int
 * return code (0 = ok, negative = mv_status below).  No STEP call (anything that
 * takes a stream) allocates, frees or synchronises: the caller owns every buffer,
 * and all launches are legal under HIP stream capture.  The set-up and tear-down
 * calls of the communicators (mv_allreduce_init / _connect / _destroy,
 * mv_allgather_init) do allocate, map and free device memory and wait for the
 * device.  They say so where they are declared.  The entry points keep no state on the device
 * between calls except in the buffers the caller passes, so calls on different
 * streams (or threads) are independent as long as they are given different
 * workspaces; the one exception is mv_paged_attn_decode_noalloc, which says so.  All tensors are bf16 unless a parameter
 * says otherwise; accumulation is fp32.
 *
 * Each declaration names the reference call it stands in for
 * (paths relative to the micro-vllm checkout).
 */
#ifndef MVLLM_H
#define MVLLM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* mv_stream_t; /* hipStream_t */

enum mv_status {
    MV_OK = 0,
    MV_ERR_INVALID_ARG = -1, /* null pointer, non-positive size, misalignment */
    MV_ERR_UNSUPPORTED = -2, /* shape outside what the kernels are built for  */
    MV_ERR_LAUNCH = -3,      /* hipGetLastError() after the launch was not ok */
    MV_ERR_WORKSPACE = -4,   /* caller workspace too small                    */
    MV_ERR_GRAPH = -5        /* stream-capture / graph API failure            */
};

/* Library identity and error text. */
int mv_version(void);
const char* mv_status_string(int status);
/* Last HIP error string seen by this thread's most recent failing call. */
const char* mv_last_hip_error(void);

/* ------------------------------------------------------------------ norms */

/* y[r,:] = bf16( (x[r,:] * rsqrt(mean(x[r,:]^2) + eps)) * w ), fp32 math.
 * Replaces kernel/rmsnorm_add.py:170 rmsnorm_ (decode, writes a static
 * buffer) and kernel/rmsnorm_add.py:37 rmsnorm (prefill). */
int mv_rmsnorm(const void* x, const void* w, void* y, int rows, int n,
               int64_t stride_x, int64_t stride_y, float eps, mv_stream_t stream);

/* s = x + r (fp32); res_out = bf16(s); var from the UNROUNDED s;
 * y = bf16( (float(res_out) * rrms) * w ).
 * Replaces kernel/rmsnorm_residual.py:127 rmsnorm_residual_gemm and
 * kernel/rmsnorm_add.py:89 rmsnorm_residual_fused. */
int mv_rmsnorm_residual(const void* x, const void* r, const void* w, void* y, void* res_out,
                        int rows, int n, int64_t stride_x, int64_t stride_r, int64_t stride_y,
                        int64_t stride_res, float eps, mv_stream_t stream);

/* out[r,c] = bf16( gate*sigmoid(gate)*up ), up = gate_up[r,c], gate = gate_up[r,c+d].
 * Replaces kernel/swiglu.py:100 swiglu_gemm and :49 swiglu_fused. */
int mv_swiglu(const void* gate_up, void* out, int64_t rows, int d, mv_stream_t stream);

/* out = bf16(float(a) + float(b)), n elements (in place allowed: out == a).
 * Replaces the `.add_(self._residual[:bs])` of core/layer/model_graph.py:219
 * and the bias add of :147 (broadcast form: b has `n_b` elements, n % n_b == 0). */
int mv_add(const void* a, const void* b, void* out, int64_t n, int64_t n_b, mv_stream_t stream);

/* out[r,:] = table[ids[r],:].  Replaces model.transformer.wte(input_ids),
 * core/layer/model_graph.py:196.  ids are int64 (torch.long). */
int mv_embedding(const void* table, const int64_t* ids, void* out, int rows, int n,
                 int64_t vocab, mv_stream_t stream);

/* ------------------------------------------------- weight-streaming GEMM */

/* One-time relayout of a [N,K] row-major bf16 weight (torch Linear.weight,
 * y = x @ W^T) into wave tiles: tile (nt,kt) holds rows 16nt..16nt+15 and
 * columns 32kt..32kt+31 as 1 KiB, lane l owning W[16nt + (l&15)][32kt + 8(l>>4) + 0..7].
 * N % 16 == 0, K % 32 == 0.  Replaces the `.t().contiguous()` relayout of
 * core/layer/model_graph.py:87-118 prepare_weights. */
int mv_shuffle_weight(const void* w_nk, void* w_tiles, int n, int k, mv_stream_t stream);

/* Rows of `a` and `b` interleaved in groups of 8: out rows [16j,16j+8) = a rows
 * [8j,8j+8), out rows [16j+8,16j+16) = b rows [8j,8j+8).  Used to put `up`
 * and `gate` rows of one output column into the same wave tile. */
int mv_interleave_rows8(const void* a, const void* b, void* out, int rows_each, int k,
                        mv_stream_t stream);

/* Bytes of workspace mv_wgemm needs for the given problem (0 if none). */
size_t mv_wgemm_workspace_bytes(int m, int n, int k);

/* y[m, :] = bf16( bf16( bf16(x[m,:] @ W^T) + bias ) + residual[m,:] ), the two
 * optional terms each adding one bf16 rounding exactly where the reference's
 * `torch.matmul(out=)`, `.add_(bias)` and `.add_(residual)` round.
 * x: [M,K] (row stride ldx), W: tiles from mv_shuffle_weight, y: [M,N].
 * 1 <= M <= 64.  flags: MV_GEMM_* below.
 * Replaces the decode projections torch.matmul(..., out=) at
 * core/layer/model_graph.py:145,171,183,185 and model.lm_head (:223). */
enum {
    MV_GEMM_DEFAULT = 0,
    MV_GEMM_SWIGLU = 1, /* W rows are up/gate interleaved by 8 (mv_interleave_rows8);
                           y is [M, N/2] = swiglu(bf16(x @ W^T)), i.e. the matmul
                           + swiglu_gemm pair of model_graph.py:183-184 in one pass */
    MV_GEMM_OUT_F32 = 2, /* y is fp32 [M,N]: the un-rounded accumulators (tests) */
    MV_GEMM_SLABS = 4,   /* y is not written (may be NULL): the product is left in `workspace` as
                            mv_wgemm_slab_count(m, n, k) fp32 slabs [slab][M][N] whose sum, added in
                            slab order, is x @ W^T - for a caller whose next kernel adds them
                            (mv_allreduce_addnorm).  Workspace: mv_wgemm_postnorm_workspace_bytes. */
    MV_GEMM_PLAN_SLABS = 8 /* an ordinary call (y written, epilogue applied) that cuts k exactly as the
                            MV_GEMM_SLABS call of the same shape does, so that its sums are formed in
                            the same order: what a step built from separate kernels uses where the
                            fused step hands slabs to the next kernel (tests compare the two bit
                            for bit) */
};
int mv_wgemm(const void* x, int64_t ldx, const void* w_tiles, const void* bias,
             const void* residual, int64_t ld_res, void* y, int64_t ldy, int m, int n, int k,
             void* workspace, size_t workspace_bytes, int flags, mv_stream_t stream);

/* Number of slabs an MV_GEMM_SLABS call leaves for this problem (>= 1). */
int mv_wgemm_slab_count(int m, int n, int k);

/* mv_wgemm with the input transform of the preceding norm kernel folded in (1 <= M <= 4):
 *   add_r == NULL:  x' = rmsnorm(x) * ln_w                       (mv_rmsnorm, then mv_wgemm)
 *   add_r != NULL:  s = x + add_r; sum_out = bf16(s); x' = rmsnorm(s) * ln_w
 *                                                    (mv_rmsnorm_residual, then mv_wgemm)
 * with exactly the rounding of those two-kernel sequences (results are bit-identical to them).
 * norm_flags & MV_NORM_VAR_FROM_ROUNDED takes the variance from bf16(s) instead of the fp32 s:
 * that is `h = a.add_(r)` followed by rmsnorm_(h) (core/layer/model_graph.py:219 then :143).
 * Replaces rmsnorm_ + matmul (model_graph.py:143-145), rmsnorm_residual_gemm + matmul
 * (:213, :183) and ln_f + lm_head (:222-223) as single launches. */
enum { MV_NORM_VAR_FROM_ROUNDED = 1 };
int mv_wgemm_norm(const void* x, int64_t ldx, const void* add_r, int64_t ld_add_r,
                  const void* ln_w, float eps, void* sum_out, int64_t ld_sum_out, int norm_flags,
                  const void* w_tiles, const void* bias, const void* residual, int64_t ld_res,
                  void* y, int64_t ldy, int m, int n, int k, void* workspace,
                  size_t workspace_bytes, int flags, mv_stream_t stream);

/* mv_wgemm with the norm kernel that FOLLOWS the projection folded into the output (any M <= 64,
 * n <= 8192; the product goes through fp32 slabs in `workspace`, one launch sums them, applies
 * the epilogue and normalises the row):
 *   t = bf16(x @ W^T); t = bf16(t + bias); s = t + residual; y = bf16(s);
 *   normed = bf16((float(y) * rrms) * ln_w), rrms = 1/sqrt(mean(s^2) + eps)
 * i.e. matmul followed by rmsnorm_residual_gemm (core/layer/model_graph.py:171 then :213: the
 * variance is taken from the unrounded s), or, with MV_NORM_VAR_FROM_ROUNDED, matmul + residual
 * add followed by the next block's rmsnorm_ (:185, :219, :143: variance from y as stored).
 * Bit-identical to mv_wgemm followed by mv_rmsnorm_residual / mv_rmsnorm. */
size_t mv_wgemm_postnorm_workspace_bytes(int m, int n, int k);
int mv_wgemm_postnorm(const void* x, int64_t ldx, const void* w_tiles, const void* bias,
                      const void* residual, int64_t ld_res, void* y, int64_t ldy, const void* ln_w,
                      float eps, void* normed, int64_t ld_normed, int norm_flags, int m, int n, int k,
                      void* workspace, size_t workspace_bytes, mv_stream_t stream);

/* The QKV projection (with its RMSNorm prologue) and the paged attention of a decode step of 1, 2 or
 * 4 rows in ONE launch: what mv_wgemm_norm (x, ln_w, eps, w_tiles, bias -> qkv [m, n], n = (hq + 2 hkv) d)
 * followed by mv_paged_attn_decode (q | k | v = the columns of qkv) computes, bit for bit - the same
 * strips in the same wave shape, the same row assignment, softmax arithmetic and split merge - with
 * the attention's page ids and key/value rows requested at the very start of the launch, before q
 * exists.  core/layer/model_graph.py:143-147 and :161-168 of one block.  No counterpart in the
 * reference (which cannot start flash-attn's loads before cuBLAS has finished).
 * One 512-thread workgroup per (row, kv head, split), all resident at once: MV_ERR_UNSUPPORTED (issue
 * the two launches instead) unless CUs / 2 < m * hkv * num_splits <= CUs, num_splits >= 2, the head
 * shape is one the dot-product attention form serves with (d, hq / hkv) in {128} x {1, 2, 4} or
 * {64} x {1, 4}, and the stand-alone projection would run this shape as whole strips on 8 waves.
 * qkv is written (write-through) and may be read by later launches.  attn_workspace: as for
 * mv_paged_attn_decode.  sync_workspace: mv_qkv_attn_workspace_bytes() bytes, 16-byte aligned,
 * zero-filled once by the caller, for launches that are stream-ordered with each other; the launch
 * needs the whole GPU to itself (a workgroup waits for the others of its kv head).  A wait of more
 * than 2 s gives up, the results are then wrong, and *status_word - any int the device can write,
 * e.g. pinned host memory, zero before the first launch - is set to 1 + the workgroup that gave up. */
size_t mv_qkv_attn_workspace_bytes(void);
int mv_qkv_attn_decode(const void* x, int64_t ldx, const void* ln_w, float eps, const void* w_tiles,
                       const void* bias, void* qkv, int64_t ld_qkv, int m, int n, int k, void* k_cache,
                       void* v_cache, const void* rot_cos, const void* rot_sin, int rot_max_pos,
                       const int32_t* cache_seqlens, const int32_t* block_table, int bt_stride, void* out,
                       void* attn_workspace, size_t attn_workspace_bytes, void* sync_workspace,
                       size_t sync_workspace_bytes, int* status_word, int hq, int hkv, int d, int page,
                       int num_pages, float scale, int num_splits, mv_stream_t stream);

/* Launch-shape knobs for experiments (no counterpart in the reference; process-wide, read once
 * per call, safe to set from another thread):
 * key 0 = workgroups per CU the grid is sized for (1..8; 0 = planner, the default);
 * key 1 = forced number of k-slices per strip (0 = pick automatically);
 * key 2 = waves per workgroup of the M <= 4 kernel (8 or 16; 0 = planner);
 * key 3 = strips a workgroup of the M > 4 kernel multiplies together (1, 2, 4, 7; 0 = planner);
 * key 4 = tiles of a wave of the M <= 4 kernel consecutive (1) or interleaved (0, the default). */
int mv_wgemm_tune(int key, int value);

/* y[M,N] = x[M,K] . W^T for many rows (prefill) on the matrix cores, reading the same tile image
 * as mv_wgemm (mv_shuffle_weight / mv_interleave_rows8); flags, bias, residual, rounding and the
 * SWIGLU output width as for mv_wgemm.  K must be a multiple of 64, N of 16; any M >= 0.
 * Replaces torch.matmul at core/layer/model_prefill.py:42,54, the compiled _mlp (:58,
 * core/layer/model_graph.py:75-81) and lm_head (:62). */
int mv_gemm_prefill(const void* x, int64_t ldx, const void* w_tiles, const void* bias,
                    const void* residual, int64_t ld_res, void* y, int64_t ldy, int m, int n,
                    int k, int flags, mv_stream_t stream);

/* The same with a workspace for sums over parts of k.  When M x N alone gives fewer output tiles
 * than the chip has CUs (prompts of up to a few hundred tokens), k is cut into slices that run side
 * by side and a second launch adds them (fp32, in order) and applies the epilogue.  When there are
 * more 256-wide tiles than CUs and the last round of tiles would leave half the CUs or more idle,
 * the tiles of that round are cut along k between the workgroups of the one launch: the lower parts
 * leave their accumulators in the workspace (256 KiB per workgroup) and the workgroup with the last
 * part adds them, in part order, as it applies the epilogue.  The workspace starts with 4 KiB of
 * counters through which those parts count themselves in: zero-fill the workspace ONCE, when it is
 * allocated; every launch returns its counters to zero and writes its data behind them, so the
 * same workspace serves any later call of any shape that fits - one workspace per stream that
 * issues such calls.  Without the workspace (or with too small a one) the call behaves like
 * mv_gemm_prefill. */
size_t mv_gemm_prefill_workspace_bytes(int m, int n, int k);
int mv_gemm_prefill_ws(const void* x, int64_t ldx, const void* w_tiles, const void* bias,
                       const void* residual, int64_t ld_res, void* y, int64_t ldy, int m, int n,
                       int k, int flags, void* workspace, size_t workspace_bytes, mv_stream_t stream);
/* Which form a call of that shape takes on the current device (for tests and tools; no counterpart
 * in the reference): 0 = 128 x 256 tiles, two workgroups per CU, weights straight into registers;
 * 1 = 256 x 256 tiles, one workgroup per CU, both operands through LDS (taken when its tiles fill
 * at least half the CUs; MVLLM_PREFILL_WIDE=0/1 forces the choice for a process); 2 and 3 = the same
 * with tiles of 192 and of 224 columns, where those fill the CUs in fewer or fuller rounds
 * (MVLLM_PREFILL_WIDE_STRIPS=12/14/16 forces the width, in 16-column strips). */
int mv_gemm_prefill_form(int m, int n, int k);
/* Overrides for tests and A/B runs inside one process (no counterpart in the reference): cut = 0 / 1
 * switches the cutting of left-over tiles off / on, strips = 12 / 14 / 16 forces the tile width, for
 * every call that follows; -1 returns a choice to the environment (MVLLM_PREFILL_CUT,
 * MVLLM_PREFILL_WIDE_STRIPS) and the planner.  Process-wide; not for use beside running calls. */
void mv_debug_prefill_options(int cut, int strips);

/* ---------------------------------------------------- paged attention */

/* Bytes of workspace for the split-KV merge (0 for one split): a 1 MiB header of arrival
 * tickets, then the splits' log-sum-exps and fp32 partial outputs.  The caller zero-fills the
 * workspace ONCE, when it allocates it; every launch returns the tickets to zero, so the same
 * workspace serves any later call, of any shape that fits. */
size_t mv_paged_attn_decode_workspace_bytes(int bs, int hq, int d, int num_splits);

/* How many KV splits the library would pick for this shape (ctx_hint = typical
 * context length; <= 0 means unknown). */
int mv_paged_attn_decode_pick_splits(int bs, int hkv, int d, int ctx_hint);

/* Which form of the kernel mv_paged_attn_decode runs for this shape: 0 = dot-product form (scores,
 * softmax, P and P.V in fp32), 1 = matrix-core form (P rounded to bf16 before P.V, as
 * flash_attn_with_kvcache does: model_graph.py:161-168 is the call it stands in for); -1 = bad shape.
 * The two agree within that rounding: |diff| <= 2^-9 * sum_t p_t |v_t| + one bf16 unit. */
int mv_paged_attn_decode_form(int hq, int hkv, int d, int page);

/* Experiment knobs (no counterpart in the reference): key 0 = merge the KV splits inside the
 * attention kernel (1, default) or in a second launch (0); key 1 = workgroups per CU the
 * automatic split count aims at (1..8; 0 = the built-in rule, default); key 2 = the matrix-core
 * form of the kernel (head size 128, 4 or 8 query heads per kv head): 0 = built-in rule,
 * 1 = never, 2 = whenever it applies. */
int mv_paged_attn_tune(int key, int value);

/* Single-token paged attention with in-kernel NeoX RoPE and KV append.
 * For each row b with p = cache_seqlens[b]:
 *   q,k <- bf16(RoPE(q,k) at position p) using cos/sin[p, :D/2] (skipped when cos == NULL);
 *   k_cache/v_cache[block_table[b, p / page], p % page, h, :] <- k, v   (in place);
 *   out[b,hq,:] = bf16( softmax(q . K[0..p]^T * scale) V[0..p] ), q head hq reading kv head hq / (Hq/Hkv),
 *   scores, softmax, P and the P.V accumulation in fp32.
 * q: [bs,Hq,D] (row stride q_stride_b, heads contiguous), k_new/v_new: [bs,Hkv,D]
 * (kv_stride_b), caches: [num_pages, page, Hkv, D] contiguous, cache_seqlens: int32 [bs],
 * block_table: int32 [bs, bt_stride] (-1 = unallocated, never dereferenced for
 * indices <= p / page unless the caller broke the contract, in which case the key is
 * skipped), out: [bs,Hq,D] contiguous.  D in {64,128}; Hq/Hkv from 1 to 8.
 * workspace: see mv_paged_attn_decode_workspace_bytes (zero-filled once by the caller; calls
 * that may overlap on one GPU need a workspace each).
 * Replaces the flash_attn_with_kvcache call at core/layer/model_graph.py:161-168
 * (and core/paged_attention.py:281). */
int mv_paged_attn_decode(const void* q, int64_t q_stride_b, const void* k_new, const void* v_new,
                         int64_t kv_stride_b, void* k_cache, void* v_cache, const void* rot_cos,
                         const void* rot_sin, int rot_max_pos, const int32_t* cache_seqlens,
                         const int32_t* block_table, int bt_stride, void* out, void* workspace,
                         size_t workspace_bytes, int bs, int hq, int hkv, int d, int page,
                         int num_pages, float scale, int num_splits, mv_stream_t stream);

/* mv_paged_attn_decode with q | k_new | v_new taken as the QKV projection left them when it was cut
 * along k: qkv_slabs = fp32 [ksplit][bs][(Hq + 2 Hkv) D] (an MV_GEMM_SLABS call of mv_wgemm), whose
 * sum in slab order, rounded to bf16, plus qkv_bias ([(Hq + 2 Hkv) D] bf16 or NULL) rounded again,
 * is the row the projection's own slab reduction would have stored - bit for bit - so a decode
 * step for more than four rows saves that launch.  Everything else as mv_paged_attn_decode.  No
 * counterpart in the reference (its QKV projection is one cuBLAS call, core/layer/model_graph.py:
 * 141-148). */
int mv_paged_attn_decode_slabs(const void* qkv_slabs, int ksplit, const void* qkv_bias, void* k_cache,
                               void* v_cache, const void* rot_cos, const void* rot_sin, int rot_max_pos,
                               const int32_t* cache_seqlens, const int32_t* block_table, int bt_stride,
                               void* out, void* workspace, size_t workspace_bytes, int bs, int hq, int hkv,
                               int d, int page, int num_pages, float scale, int num_splits,
                               mv_stream_t stream);

/* mv_paged_attn_decode for callers that cannot allocate device memory (code under HIP stream
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same kernels and the same
 * results, bit for bit, with the split-KV workspace in an 8 MiB array that is part of the
 * library's device image instead of a caller buffer.  It has no counterpart in the reference.
 * The call allocates and frees nothing.  Limit: mv_paged_attn_decode_workspace_bytes(bs, hq, d,
 * num_splits) <= 8 MiB (e.g. 32 rows x 32 heads x 4 splits at d = 128), else MV_ERR_WORKSPACE
 * with the sizes in mv_last_hip_error().  Every GPU holds one copy of the array for the life of
 * the process and every call on a GPU uses it: calls that overlap on one GPU (two streams, two
 * threads) race and must not be made.  The first call on a device looks the array's address up
 * (make it outside stream capture). */
int mv_paged_attn_decode_noalloc(const void* q, int64_t q_stride_b, const void* k_new,
                                 const void* v_new, int64_t kv_stride_b, void* k_cache, void* v_cache,
                                 const void* rot_cos, const void* rot_sin, int rot_max_pos,
                                 const int32_t* cache_seqlens, const int32_t* block_table,
                                 int bt_stride, void* out, int bs, int hq, int hkv, int d, int page,
                                 int num_pages, float scale, int num_splits, mv_stream_t stream);

/* ---- prefill (many tokens per sequence) ---- */

/* NeoX rotation of `heads` heads of width d per row, y may alias x; row t uses cos/sin[t % seq].
 * Evaluated like the reference's bf16 tensor expression (every product and the sum/difference
 * round to bf16): core/layer/rope.py:10-39 (half-width table branch :28-33). */
int mv_rope_prefill(const void* x, int64_t x_stride, void* y, int64_t y_stride, const void* rot_cos,
                    const void* rot_sin, int rot_max_pos, int64_t tokens, int seq, int heads, int d,
                    mv_stream_t stream);

/* One launch for what the prefill runner does between the QKV projection and attention
 * (core/layer/model_prefill.py:45-52): rows of qkv are [q heads | k heads | v heads]; token i of
 * sequence b sits at position p = cache_seqlens[b] + i; q and k are rotated in place with
 * cos/sin[p] (mv_rope_prefill arithmetic; skipped when cos == NULL) and the rotated k and v are
 * written to k_cache/v_cache[block_table[b, p / page], p % page, h, :]. */
int mv_rope_store_prefill(void* qkv, int64_t row_stride, const void* rot_cos, const void* rot_sin,
                          int rot_max_pos, const int32_t* cache_seqlens, const int32_t* block_table,
                          int bt_stride, void* k_cache, void* v_cache, int bs, int seq, int hq,
                          int hkv, int d, int page, int num_pages, mv_stream_t stream);

/* Causal attention of `seq` new tokens per sequence over the paged cache, which must already
 * hold their keys and values (mv_rope_store_prefill / mv_store_kv): query i of sequence b sees
 * keys 0 .. cache_seqlens[b] + i (bottom-right aligned mask), q head h reads kv head h / (Hq/Hkv).
 * q rows: [bs*seq][q_stride] with heads contiguous; out rows likewise.  fp32 scores and softmax,
 * P rounded to bf16 as the matrix-core operand, fp32 accumulation, bf16 output.
 * D in {64,128}; Hq/Hkv from 1 to 8 (3, 5, 6 and 7 take the row stack of the next power of two: the rows of
 * the heads that do not exist are computed and dropped); page a power of two >= 64.
 * With the store above this replaces flash_attn_with_kvcache(q, k_cache, v_cache, k=, v=,
 * cache_seqlens=, block_table=, causal=True) at core/layer/model_prefill.py:49-52. */
int mv_paged_attn_prefill(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                          const int32_t* cache_seqlens, const int32_t* block_table, int bt_stride,
                          void* out, int64_t out_stride, int bs, int seq, int hq, int hkv, int d,
                          int page, int num_pages, float scale, mv_stream_t stream);
/* Waves per workgroup the call above takes for this shape on the current device (4 = 128 stacked query
 * rows per workgroup, 8 = 256; for tests and tools, no counterpart in the reference;
 * MVLLM_PREFILL_ATTN_WAVES=4/8 forces one for a process). */
int mv_paged_attn_prefill_form(int bs, int seq, int hq, int hkv);

/* key[t,h,:] -> k_cache[slot/page, slot%page, h, :] (same for value); slot -1 = skip.
 * key/value: [T,H,D] with token stride kv_stride_t; slot_mapping int32 [T].
 * Replaces core/cache_manager.py:143 store_kvcache (Triton store_kvcache_kernel :75). */
int mv_store_kv(const void* key, const void* value, int64_t kv_stride_t, void* k_cache,
                void* v_cache, const int32_t* slot_mapping, int tokens, int heads, int d,
                int page, int num_pages, mv_stream_t stream);

/* ------------------------------------------------------------- sampling */

/* ids[r] = argmax_c logits[r, c] over bf16 logits [rows, n] (row stride ld), lowest index on
 * ties; ids are int64.  The greedy (temperature -> 0) case of core/layer/sampler.py:21-43,
 * done on the device so the step needs no [bs,V] sort and no host round trip.
 * workspace (optional, mv_argmax_workspace_bytes() bytes, 16-byte aligned, zero-filled once by
 * the caller): where the parts of a long row meet when few rows are spread over many
 * workgroups; without it every row gets one workgroup (same result, slower). */
size_t mv_argmax_workspace_bytes(void);
int mv_argmax(const void* logits, int64_t ld, int rows, int n, int64_t* ids, void* workspace,
              size_t workspace_bytes, mv_stream_t stream);

/* Stochastic pick, one launch per batch: for each row, scale by 1/temperature[r], keep the
 * min(top_k, n, 1024) largest logits, softmax over them, keep the sorted prefix whose inclusive
 * cumulative probability is < top_p[r] (always at least the first), renormalise, and return the
 * entry at which the cumulative probability first exceeds uniforms[r] (a number in [0,1) the caller
 * draws).  Equal logits are ordered by ascending index, so the result is a deterministic function of
 * its inputs; temperature <= 0 returns the argmax.  n must be a multiple of 8.
 * The recipe of core/layer/sampler.py:21-43 (_sample_impl: topk, softmax, sort, cumsum < top_p,
 * multinomial), with the draw expressed through an explicit uniform number. */
int mv_sample_topk_topp(const void* logits, int64_t ld, int rows, int n, const float* temperatures,
                        const float* top_ps, int top_k, const float* uniforms, int64_t* ids,
                        mv_stream_t stream);

/* The same, for use inside a captured decode step: rows with temperature <= 0 take
 * greedy_ids[r] (the caller's mv_argmax result) without looking at the logits, so a step that
 * always contains this launch costs greedy batches nothing.  greedy_ids == NULL: as above. */
int mv_sample_or_greedy(const void* logits, int64_t ld, int rows, int n, const float* temperatures,
                        const float* top_ps, int top_k, const float* uniforms,
                        const int64_t* greedy_ids, int64_t* ids, mv_stream_t stream);

/* ------------------------------------------- tensor-parallel all-reduce */

/* One-shot all-reduce for the small [rows, n] bf16 messages of a tensor-parallel decode step, among
 * the (at most 8) GPUs of one node, one process per GPU.  Every rank pushes its partial into every
 * rank's exchange buffer over the direct xGMI links and sums what arrived in its own buffer in rank
 * order (fp32, rounded to bf16 once): all ranks get the same bits.  Stands in for
 * core/parallel_config.py:69-74 all_reduce at core/layer/model_graph.py:210,219; messages beyond the
 * communicator's capacity (prefill) stay with RCCL.
 *
 * Set-up, once per process (these three allocate / map device memory; the step calls do not):
 *   mv_allreduce_init        exchange buffer for messages of up to max_rows x max_n (max_rows <= 64,
 *                            max_n <= 8192, a multiple of 8) on the current device;
 *   mv_allreduce_get_handle  mv_allreduce_handle_bytes() bytes to pass to the other ranks by any host
 *                            channel (e.g. torch.distributed.all_gather_object);
 *   mv_allreduce_connect     `handles` = all ranks' handles in rank order; maps the peers' buffers.
 * The step calls take the stream, never synchronise and are legal under stream capture: flags carry an
 * epoch kept in device memory that only grows, so a captured step can be replayed.  All ranks must
 * issue the same sequence of calls with the same `rows`.  A rank that waits longer than
 * MVLLM_ALLREDUCE_TIMEOUT_MS (default 10 s) for a peer gives up, finishes with a wrong sum and sets
 * the communicator's status word (1 + the rank that did not arrive; 0 = no timeout so far).  The word
 * is host memory mapped into the device: mv_allreduce_status is a plain load that neither waits nor
 * touches the device, and tells about the step calls the caller has already waited for (so a serving
 * loop reads it right after the token read-back of a step, before it uses the tokens).  After a
 * timeout the ranks' epochs may be out of step: destroy the communicator, do not go on with it. */
size_t mv_allreduce_handle_bytes(void);
int mv_allreduce_init(int rank, int world, int max_rows, int max_n, void** comm_out);
int mv_allreduce_get_handle(void* comm, void* handle_out);
int mv_allreduce_connect(void* comm, const void* handles);
int mv_allreduce_status(void* comm, int* status_out);
/* How long later step calls wait for a peer (overrides MVLLM_ALLREDUCE_TIMEOUT_MS for this communicator). */
int mv_allreduce_set_timeout_ms(void* comm, double ms);
int mv_allreduce_destroy(void* comm);

/* out = bf16(sum over ranks of in), [rows, n] bf16; out may alias in. */
int mv_allreduce_step(void* comm, const void* in, int64_t ld_in, void* out, int64_t ld_out, int rows,
                      int n, mv_stream_t stream);

/* All-gather of [rows, n_local] bf16 slices into [rows, world * n_local] rows on every rank, through
 * a communicator of its own (same handle / connect / status / set_timeout / destroy calls as above):
 *   mv_allgather_init   exchange buffer for up to max_rows rows of world x n_local columns
 *                       (n_local a multiple of 8);
 *   mv_allgather_rows   rank r's `in` lands at columns [r * n_local, (r + 1) * n_local) of `out` on every
 *                       rank; takes the stream, never synchronises, legal under stream capture.
 * No counterpart in the reference, which keeps the LM head whole on every rank (core/layer/
 * model_graph.py:222-223): with the head cut by vocabulary rows each rank multiplies 1/world of it and
 * the ranks exchange their logits instead (at 8 ranks of the 8B shape 1/8 of the largest single
 * projection of a decode step). */
int mv_allgather_init(int rank, int world, int max_rows, int n_local, void** comm_out);
int mv_allgather_rows(void* comm, const void* in, int64_t ld_in, void* out, int64_t ld_out, int rows,
                      int n_local, mv_stream_t stream);

/* The all-reduce together with what a decoder block does next (core/layer/model_graph.py:210-213 and
 * :219 + :143 of the following block), one launch:
 *   t = bf16(sum over ranks of partial);  s = t + residual;  y = bf16(s);
 *   normed = bf16((float(y) * rrms) * ln_w),  rrms = 1 / sqrt(mean(s^2) + eps)
 * (mean over the unrounded s, or over y as stored with MV_NORM_VAR_FROM_ROUNDED: the two cases of
 * mv_wgemm_postnorm).  This rank's partial is either `in` (bf16 rows) or, with in == NULL, the sum of
 * the `ksplit` fp32 slabs [ksplit][rows][n] an MV_GEMM_SLABS projection left, rounded to bf16 - what
 * that projection's bf16 output would have been.  residual, y and (ln_w, normed) are optional. */
int mv_allreduce_addnorm(void* comm, const void* in, int64_t ld_in, const float* slabs, int ksplit,
                         const void* residual, int64_t ld_res, void* y, int64_t ldy, const void* ln_w,
                         float eps, void* normed, int64_t ld_normed, int norm_flags, int rows, int n,
                         mv_stream_t stream);

/* ------------------------------------------------------------ hipGraph */

/* Capture everything launched on `stream` between begin and end into an
 * executable hipGraph; replay it with mv_graph_launch.  Replaces the
 * torch.cuda.CUDAGraph capture/replay of core/layer/model_graph.py:241-259. */
int mv_graph_begin_capture(mv_stream_t stream);
int mv_graph_end_capture(mv_stream_t stream, void** graph_exec_out);
int mv_graph_launch(void* graph_exec, mv_stream_t stream);
int mv_graph_destroy(void* graph_exec);

/* ------------------------------------------------------------------------------------------------
 * Layer stacks with an fp32 residual stream, recurrent mixers and windowed attention over a RAGGED
 * step (csrc/linear_any.hip, stream_ops.hip, seq_mix.hip).  No counterpart in the reference, whose
 * only model family is the Llama-shaped one.
 *
 * A step's tokens lie back to back; row b (one sequence) owns tokens [row_start[b], row_start[b] +
 * row_len[b]) and had row_ctx[b] tokens before the step; tok_row[t] / tok_pos[t] give every token's
 * row and position.  Recurrent state lives in slot row_slot[b] of fp32 pools and is taken as zero
 * when row_ctx[b] == 0; keys and values live in pages named by block_table[b, pos / page].
 * `f32` selects the activation type of projection operands and cached keys/values: 0 = bf16,
 * 1 = fp32 (the whole model in 32 bits).  Everything else is fp32 in both.
 * ------------------------------------------------------------------------------------------------ */

/* y[M,N] (fp32) = x[M,K] . W[N,K]^T, row-major operands of the activation type, any M, N, K. */
int mv_linear_any(const void* x, int64_t ldx, const void* w, int64_t ldw, float* y, int64_t ldy, int m, int n,
                  int k, int f32, mv_stream_t stream);

/* x[r,:] = table[ids[r],:] * scale (fp32), h = the same in the activation type. */
int mv_embed_scaled(const void* table, const int32_t* ids, float* x, int64_t ldx, void* h, int64_t ldh, int rows,
                    int n, int vocab, float scale, int f32, mv_stream_t stream);

/* v = s1*y1 (+ s2*y2 when y2 != NULL); x += v / sqrt(mean(v^2) + eps) * (1 + w); h = act(x). */
int mv_postnorm_residual(const float* y1, int64_t ld1, const float* y2, int64_t ld2, float s1, float s2,
                         const float* w, float eps, float* x, int64_t ldx, void* h, int64_t ldh, int rows, int n,
                         int f32, mv_stream_t stream);

/* out[r,:] = act( x[idx[r],:] / sqrt(mean(.^2) + eps) * (1 + w) ); idx == NULL: row r itself. */
int mv_offset_rmsnorm_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, float eps, void* out,
                             int64_t ldo, int rows, int n, int f32, mv_stream_t stream);

/* out = act( max(in, 0)^2 ). */
int mv_relu_squared(const float* in, int64_t ldi, void* out, int64_t ldo, int rows, int n, int f32,
                    mv_stream_t stream);

/* v = cap * tanh(v / cap), in place. */
int mv_softcap(float* v, int64_t count, float cap, mv_stream_t stream);

/* out[t,c] = silu(bias[c] + sum_j w[c,j] * in[t - (taps-1) + j, c]) within each row, the inputs before
 * the row's first token taken from state[slot][taps-1][channels] (zeros for a new sequence); then the
 * state receives the row's last taps-1 inputs.  w: fp32 [channels, taps], last column = current token. */
int mv_conv_silu(const float* in, int64_t ldi, float* state, const float* w, const float* bias, float* out,
                 int64_t ldo, const int32_t* tok_row, const int32_t* row_start, const int32_t* row_len,
                 const int32_t* row_ctx, const int32_t* row_slot, int tokens, int rows, int channels, int taps,
                 mv_stream_t stream);

/* gain[t,h] = log(1 + exp(raw[t,h] + dt_bias[h])); log_decay[t,h] = -exp(a_log[h]) * gain[t,h] (may be NULL);
 * decay[t,h] = exp(log_decay[t,h]). */
int mv_softplus_decay(const float* raw, int64_t ld, const float* dt_bias, const float* a_log, float* gain,
                      float* decay, float* log_decay, int tokens, int heads, mv_stream_t stream);

/* Per row and head, token by token: S = decay[t,h] * S + gain[t,h] * k_t v_t^T (S: n x p, fp32, in
 * state[slot][head]); out[t, h*p ..] = S^T q_t (+ skip[h] * v_t).  q and k of head h are read at
 * column (h / q_div) * n and (h / k_div) * n (heads that share a group); gain == NULL: 1;
 * ld_decay == 0: decay[h] for every token.  max_len > 0: rows longer than that are left alone. */
int mv_scan_outer(const float* q, int64_t ldq, int q_div, const float* k, int64_t ldk, int k_div, const float* v,
                  int64_t ldv, const float* decay, int64_t ld_decay, const float* gain, int64_t ld_gain,
                  const float* skip, float* state, float* out, int64_t ldo, const int32_t* row_start,
                  const int32_t* row_len, const int32_t* row_ctx, const int32_t* row_slot, int rows, int heads, int n,
                  int p, int max_len, mv_stream_t stream);

/* The same recurrence for long rows, 64 tokens at a time, its products on the fp32 matrix instruction
 * (v_mfma_f32_16x16x4_f32; three launches: sums within each chunk, the states the chunks start from, their
 * contribution to the outputs).  Chunk c covers tokens ch_start[c] ..
 * + ch_len[c] (<= 64) of one row; row b owns chunks row_ch0[b] .. + row_nch[b] (0: the row is not taken -
 * mv_scan_outer with max_len > 0 leaves exactly the rows longer than max_len to this call).  The decay
 * comes as its logarithm ([tokens, heads], or [heads] with ld_ld == 0).  Scratch: ds [chunks, heads, n, p],
 * lsum [tokens, heads], atot [chunks, heads], all fp32.  Differs from the token-by-token form by the
 * order of the fp32 sums only.  MV_ERR_UNSUPPORTED when n and p need more LDS than a workgroup has
 * (mv_scan_chunked_lds_bytes(n, p) > 150 KiB). */
size_t mv_scan_chunked_lds_bytes(int n, int p);
int mv_scan_chunked(const float* q, int64_t ldq, int q_div, const float* k, int64_t ldk, int k_div, const float* v,
                    int64_t ldv, const float* log_decay, int64_t ld_ld, const float* gain, int64_t ld_gain,
                    const float* skip, float* state, float* out, int64_t ldo, float* ds, float* lsum, float* atot,
                    const int32_t* ch_start, const int32_t* ch_len, const int32_t* row_ch0, const int32_t* row_nch,
                    const int32_t* row_ctx, const int32_t* row_slot, int chunks, int rows, int heads, int n, int p,
                    mv_stream_t stream);

/* In place, per token and head of width dim: (u, v) = (x[i], x[i + rot/2]), i < rot/2, becomes
 * (u cos a - v sin a, v cos a + u sin a), a = tok_pos[t] * inv_freq[i] (formed in fp64); all dim values
 * are then multiplied by scale. */
int mv_rotary_pairs(float* x, int64_t ld, const double* inv_freq, const int32_t* tok_pos, int tokens, int heads,
                    int dim, int rot, float scale, mv_stream_t stream);

/* Rows cut into `groups` equal parts, each divided by its root mean square; gate_first: the part is
 * y * silu(gate) before that, else silu(gate) multiplies after; w (fp32 [n]) multiplies last or is NULL. */
int mv_gated_group_norm(const float* y, int64_t ldy, const float* gate, int64_t ldg, const float* w, void* out,
                        int64_t ldo, int rows, int n, int groups, int gate_first, float eps, int f32,
                        mv_stream_t stream);

/* Rows of qkv are [heads x d | kv_heads x d | kv_heads x dv] fp32.  Queries are divided by their root
 * mean square in place; keys likewise and written, with the values, to k_cache [pages, page, kv_heads, d]
 * and v_cache [pages, page, kv_heads, dv] at the token's position. */
int mv_qk_unitnorm_store(float* qkv, int64_t ld, void* k_cache, void* v_cache, const int32_t* tok_row,
                         const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int page, int tokens,
                         int heads, int kv_heads, int d, int dv, float eps, int f32, mv_stream_t stream);

/* Rows of qk are [heads x d | kv_heads x d] fp32, one projection's output.  Queries: q += q_bias (NULL: none), then
 * the first `rot` dimensions of each head rotated by angle pos * inv_freq[i] (fp64 table of rot/2 entries; adjacent:
 * dimension 2i with 2i+1, else i with i + rot/2), in place.  Keys: k += k_bias; the key as it then stands goes to
 * v_cache (attention whose values are its unrotated keys), its rotated form to k_cache, both [pages, page, kv_heads, d].
 * act_in != NULL: the same launch also forms act_out[t, :act_n] = mv_gated_act of act_in[t, :2 act_n] (gate | up columns
 * that the same projection left beside q and k: a layer whose mixer and feed-forward read one input). */
int mv_qk_rotary_store(float* qk, int64_t ld, const float* q_bias, const float* k_bias, void* k_cache, void* v_cache,
                       const double* inv_freq, const int32_t* tok_row, const int32_t* tok_pos,
                       const int32_t* block_table, int bt_stride, int page, int tokens, int heads, int kv_heads, int d,
                       int rot, int adjacent, const float* act_in, int64_t lda, void* act_out, int64_t ldao, int act_n,
                       int act_kind, float act_limit, float act_slope, int f32, mv_stream_t stream);

/* out[t, h*dv ..] = softmax_j( q_t . k_j * scale - slopes[h] * (pos - j) ) v_j over pos - window < j <= pos
 * from the pages (the step's own keys must already be stored).  dv <= 256.  keep_first > 0: positions below it
 * stay visible when the window has passed them, at their true positions.  sinks (fp32 [heads] or NULL): exp(sinks[h])
 * is one more term of the softmax's denominator, unscaled, with no value.  slopes NULL: no distance penalty.
 * part != NULL with splits >= 1 (fp32 [tokens * heads * splits * (dv + 2)]): the tokens the tiled kernel does not take
 * run one workgroup per (token, key/value head, up to eight of its query heads, split of the keys) - every key and value
 * is read once for those heads - and, with splits > 1, a second launch merges the splits' pieces.
 * short_tokens: how many of the step's tokens lie in rows of up to max_len tokens (-1: not known); 0 lets a step whose
 * rows all went to the tiled kernel skip the launch of the per-token form.  With a chunk table (chunks > 0:
 * rows of more than max_len tokens cut into runs of up to 64, as for mv_scan_chunked; row_len per row), bf16
 * and a head shape the tiled kernel is built for - (d, dv) in (32,32) (64,64) (96,96) (128,128) (128,64)
 * (64,128), 64-token pages - those rows run on the matrix cores, a workgroup per (chunk, head): q.k in bf16
 * (q rounded as the cached keys are), softmax in fp32, P.V with fp32 P.  Every other token takes the
 * one-workgroup-per-(token, head) form. */
int mv_window_attn(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, void* out, int64_t ldo,
                   const int32_t* tok_row, const int32_t* tok_pos, const int32_t* block_table, int bt_stride,
                   int page, const float* slopes, int tokens, int heads, int kv_heads, int d, int dv, float scale,
                   int window, int f32, const int32_t* row_len, const int32_t* ch_start, const int32_t* ch_len,
                   int chunks, int max_len, int keep_first, const float* sinks, float* part, int splits,
                   int short_tokens, mv_stream_t stream);
/* How many splits of the keys mv_window_attn should be given for a step of `tokens` tokens (1: none). */
int mv_window_attn_splits(int tokens, int heads, int kv_heads, int window, int keep_first);

/* ---- further row-wise steps of fp32-stream stacks (stream_ops.hip) ---------------------------------- */

/* n = tanh(alpha x) w + b (a norm that forms no statistics); h_t = act( n_t + (n_(t-1) - n_t) * mix ): every
 * token's normed vector blended with its predecessor's.  The predecessor of a row's first token is the vector
 * kept in state[slot] (zeros when row_ctx == 0); the row's last n is left there for its next step. */
int mv_dyt_shift(const float* x, int64_t ldx, const float* w, const float* b, const float* alpha, const float* mix,
                 float* state, void* h, int64_t ldh, const int32_t* tok_row, const int32_t* row_start,
                 const int32_t* row_len, const int32_t* row_ctx, const int32_t* row_slot, int tokens, int n, int f32,
                 mv_stream_t stream);
/* out[r,:] = act( tanh(alpha x[idx[r],:]) w + b ); idx == NULL: row r itself. */
int mv_dyt_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, const float* b, const float* alpha,
                  void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream);
/* x += tanh(alpha y) w + b; h = act(x) unless h == NULL; with w2 != NULL h = act( tanh(alpha2 x) w2 + b2 ), the next
 * sublayer's norm of the new x. */
int mv_dyt_residual(const float* y, int64_t ldy, const float* w, const float* b, const float* alpha, float* x,
                    int64_t ldx, void* h, int64_t ldh, const float* w2, const float* b2, const float* alpha2, int rows,
                    int n, int f32, mv_stream_t stream);
/* x += y / sqrt(mean(y^2) + eps) * w (plain weight); h = act(x) unless h == NULL. */
int mv_unitnorm_residual(const float* y, int64_t ldy, const float* w, float eps, float* x, int64_t ldx, void* h,
                         int64_t ldh, int rows, int n, int f32, mv_stream_t stream);
/* `per` groups of n values in each of `rows` rows: out = act( v / sqrt(mean(v^2) + eps) * w ), w [n] shared. */
int mv_rmsnorm_rows(const float* v, int64_t ld, int per, const float* w, float eps, void* out, int64_t ldo,
                    int rows, int n, int f32, mv_stream_t stream);
/* out[r,:] = act( gelu_tanh(a[r,:]) * table[ids[r]][off .. off+n) ), table rows of ldt values. */
int mv_gelu_gate_rows(const float* a, int64_t lda, const void* table, int64_t ldt, int off, const int32_t* ids,
                      int vocab, void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream);
/* out = act( silu(a[:, :n]) * a[:, n:2n] ). */
int mv_silu_mul(const float* a, int64_t lda, void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream);
/* out = act( f(a[:, :n]) * a[:, n:2n] ): kind 0 f = SiLU, 1 f = GELU in its tanh form; kind 2 the clamped gate,
 * g = min(a[:, :n], limit), u = clamp(a[:, n:2n], -limit, limit), out = act( g * sigmoid(slope * g) * (u + 1) ). */
int mv_gated_act(const float* a, int64_t lda, void* out, int64_t ldo, int rows, int n, int kind, float limit,
                 float slope, int f32, mv_stream_t stream);
/* x[r,:] = table[ids[r],:] * scale + pairs[j,:] (fp32), j = (prev[r] * mul_prev + ids[r] * mul_cur) mod buckets, or
 * j = buckets (the table's extra last row) where prev[r] < 0: the token has no predecessor.  Tables in the
 * activation type, `pairs` [buckets + 1, n].  norm_w != NULL: h = act( x / sqrt(mean(x^2) + eps) * norm_w ) as well. */
int mv_embed_pair(const void* table, const void* pairs, const int32_t* ids, const int32_t* prev, float* x, int64_t ldx,
                  int rows, int n, int vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur, float scale,
                  const float* norm_w, float eps, void* h, int64_t ldh, int f32, mv_stream_t stream);
/* x += y1 (+ y2) (y1 == NULL: x as it is); w != NULL: h = act( x / sqrt(mean(x^2) + eps) * w ). */
int mv_add_rmsnorm(const float* y1, int64_t ld1, const float* y2, int64_t ld2, float* x, int64_t ldx, const float* w,
                   float eps, void* h, int64_t ldh, int rows, int n, int f32, mv_stream_t stream);
/* out[r,:] = act( x[idx[r],:] / sqrt(mean(.^2) + eps) * (offset + w) ); idx == NULL: row r itself. */
int mv_rmsnorm_gather(const float* x, int64_t ldx, const int32_t* idx, const float* w, float eps, float offset,
                      void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream);
/* out = act( a * sigmoid(g) ); g == NULL: act(a). */
int mv_sigmoid_gate(const float* a, int64_t lda, const float* g, int64_t ldg, void* out, int64_t ldo, int rows, int n,
                    int f32, mv_stream_t stream);

/* ---- products per head and per segment (linear_any.hip) --------------------------------------------- */

/* `heads` products in one launch: y[:, h*zy .. +n] = x[:, h*zx .. +k] . W_h^T, W_h = w + h*zw ([n,k], row stride ldw). */
int mv_linear_heads(const void* x, int64_t ldx, int64_t zx, const void* w, int64_t ldw, int64_t zw, float* y,
                    int64_t ldy, int64_t zy, int m, int n, int k, int heads, int f32, mv_stream_t stream);
/* Output rows seg[e] .. seg[e+1] use weight w + e*zw; operand row of output row i is src[i] / src_div (src == NULL:
 * i).  max_rows bounds the rows of one segment, total_rows = seg[segments] (the rows of y). */
int mv_linear_segments(const void* x, int64_t ldx, const void* w, int64_t ldw, int64_t zw, float* y, int64_t ldy,
                       const int32_t* seg, const int32_t* src, int src_div, int segments, int max_rows, int total_rows,
                       int n, int k, int f32, mv_stream_t stream);

/* ---- gated recurrence without a key (seq_mix.hip) ---------------------------------------------------- */

/* q = silu(q), f = lower + (1 - lower) * sigmoid(f + bias) in place ([tokens, n] each, bias may be NULL). */
int mv_gate_lower_bound(float* q, int64_t ldq, float* f, int64_t ldf, const float* bias, const float* lower,
                        int tokens, int n, mv_stream_t stream);
/* S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t per head; q, f [T, heads*n], v, out [T, heads*p],
 * state [slots, heads, n, p] fp32 (taken as zero when row_ctx == 0).  chunks > 0: rows longer than max_len are cut
 * into chunks (ch_start / ch_len / row_ch0 / row_nch as for mv_scan_chunked) that run side by side from a zero
 * state and are then joined through the products of their gates (scratch: ds [chunks, heads, n, p], cum
 * [tokens, heads*n], fp32); differs from the token-by-token form by the order of the fp32 sums only. */
int mv_scan_gated(const float* q, int64_t ldq, const float* f, int64_t ldf, const float* v, int64_t ldv, float* state,
                  float* out, int64_t ldo, const int32_t* row_start, const int32_t* row_len, const int32_t* row_ctx,
                  const int32_t* row_slot, int rows, int heads, int n, int p, float* ds, float* cum,
                  const int32_t* ch_start, const int32_t* ch_len, const int32_t* row_ch0, const int32_t* row_nch,
                  int chunks, int max_len, mv_stream_t stream);

/* ---- attention over a cached latent (latent_attn.hip) ------------------------------------------------ */

/* Per token: cache[page row] = [ unit-RMS(dkv[:rank]) * w_norm | rotate(dkv[rank : rank + r]) ] in the activation
 * type; q_plain[t, h*d ..] = act(q[t, h*(d+r) .. +d]); q_abs[t, h*(rank+r) + rank ..] = rotate(q[t, h*(d+r) + d ..]).
 * Rotation by the token's position over the first `rot` of the r dimensions, pairs (2i, 2i+1) when `interleaved`,
 * else (i, i + rot/2); inv_freq [rot/2] fp64. */
int mv_latent_prep(const float* dkv, int64_t ldkv, const float* w_norm, float eps, void* cache, const float* q,
                   int64_t ldq, void* q_plain, int64_t ldqn, float* q_abs, int64_t ldqa, const double* inv_freq,
                   const int32_t* tok_row, const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int page,
                   int tokens, int heads, int d, int r, int rank, int rot, int interleaved, int f32,
                   mv_stream_t stream);
/* out[t, h*rank ..] = sum_j softmax_j( q_abs[t,h] . cache[j] * scale ) cache[j][:rank] over the keys j <= position
 * (window > 0: only the last `window` of them); sinks != NULL: exp(sinks[h]) joins the denominator.
 * chunks > 0: rows of more than max_len tokens, cut into chunks of up to 64 (ch_start / ch_len), run on the matrix
 * cores where the shape allows it (bf16, pages of 64, rank in {64,128,256,512}, r in {0,32,64}): q . k in bf16 (q
 * rounded as the cached latents are), softmax in fp32, P . V with fp32 P; every other token takes the
 * one-workgroup-per-(token, head group) form. */
int mv_latent_attn(const float* q_abs, int64_t ldq, const void* cache, void* out, int64_t ldo, const int32_t* tok_row,
                   const int32_t* tok_pos, const int32_t* block_table, int bt_stride, int page, const float* sinks,
                   int tokens, int heads, int rank, int r, float scale, int window, int f32, const int32_t* row_len,
                   const int32_t* ch_start, const int32_t* ch_len, int chunks, int max_len, mv_stream_t stream);

/* ---- routed experts (moe.hip) ------------------------------------------------------------------------ */

/* ids / weights [tokens, top]: the `top` largest of W_router h (fp32; ties to the lower index) and the softmax over
 * them; shared_gate[t] = sigmoid(w_shared_gate . h_t) when w_shared_gate != NULL. */
int mv_moe_route(const void* h, int64_t ldh, const float* w_router, const float* w_shared_gate, int32_t* ids,
                 float* weights, float* shared_gate, int tokens, int n, int experts, int top, int f32,
                 mv_stream_t stream);
/* scores = softmax over all `experts` router outputs of W_router h (fp32); the `top` largest of score + correction
 * (NULL: none; ties to the lower index) are chosen; weights = score / (sum of the chosen scores + sum_floor) * scale. */
int mv_moe_route_scored(const void* h, int64_t ldh, const float* w_router, const float* correction, int32_t* ids,
                        float* weights, int tokens, int n, int experts, int top, float scale, float sum_floor, int f32,
                        mv_stream_t stream);
/* (token, choice) pairs sorted by expert: seg [experts + 1], order [pairs] (pair in each row), place [pairs]. */
int mv_moe_plan(const int32_t* ids, int32_t* seg, int32_t* order, int32_t* place, int pairs, int experts,
                mv_stream_t stream);
/* s_t = sum_k weights[t,k] * expert_out[place[t*top+k]] (+ shared_gate[t] * shared_out[t]).  norm_w == NULL: y = s.
 * Else y is the residual stream: y += tanh(norm_alpha s) norm_w + norm_b, and h (optional) = act(y).
 * weights == NULL: every weight is one; shared_gate == NULL: the shared expert's output counts whole.
 * ids != NULL: a choice ids[t*top+k] >= first_pass has no expert row; it adds weights[t,k] * pass[t,:] (activation
 * type, row stride ldp): an expert that hands its input through. */
int mv_moe_combine(const float* expert_out, int64_t lde, const int32_t* place, const float* weights,
                   const float* shared_out, int64_t lds, const float* shared_gate, float* y, int64_t ldy,
                   const float* norm_w, const float* norm_b, const float* norm_alpha, void* h, int64_t ldh, int tokens,
                   int n, int top, int f32, const int32_t* ids, int first_pass, const void* pass, int64_t ldp,
                   mv_stream_t stream);

/* The `top` largest of W_router h (fp32; ties to the lower index); weights = sigmoid of each chosen output, not
 * renormalised. */
int mv_moe_route_sigmoid(const void* h, int64_t ldh, const float* w_router, int32_t* ids, float* weights, int tokens,
                         int n, int experts, int top, int f32, mv_stream_t stream);
/* mv_gated_act on rows sorted by expert, with both halves scaled first: out = act( f(s a[:, :n]) * (s a[:, n:2n]) ),
 * s = scale[order[row]] (order == NULL: scale[row]): an expert that reads weight * h, from the products of h. */
int mv_gated_act_scaled(const float* a, int64_t lda, void* out, int64_t ldo, int rows, int n, int kind, float limit,
                        float slope, const float* scale, const int32_t* order, int f32, mv_stream_t stream);

/* ---- gated residual stream, loop input (stream_ops.hip) ------------------------------------------------- */

/* mode 1: x += y * sigmoid(g + b) (b == NULL: no bias); mode 2: x = y + b; mode 0: x as it is.  w != NULL:
 * n = x / sqrt(mean(x^2) + eps) * (offset + w) of the new x, to n32 (fp32) and / or h (activation type). */
int mv_gated_residual_norm(const float* y, int64_t ldy, const float* g, int64_t ldg, const float* b, int mode, float* x,
                           int64_t ldx, const float* w, float eps, float offset, float* n32, int64_t ldn, void* h,
                           int64_t ldh, int rows, int n, int f32, mv_stream_t stream);
/* out[r, :n] = act(a[r, :]), out[r, n:2n] = act(b[r, :]). */
int mv_cast_concat(const float* a, int64_t lda, const float* b, int64_t ldb, void* out, int64_t ldo, int rows, int n,
                   int f32, mv_stream_t stream);
/* out = act( gelu(in) ), the tanh form. */
int mv_gelu_tanh(const float* in, int64_t ldi, void* out, int64_t ldo, int rows, int n, int f32, mv_stream_t stream);
/* v[i] *= factor. */
int mv_scale(float* v, int64_t count, float factor, mv_stream_t stream);

/* ---- short convolutions without activation, differential attention (seq_mix.hip, diff_attn.hip) ---------- */

/* y_t = (add_input ? u_t : 0) + sum_j w[c, j] u_(t - taps + 1 + j) per channel over a ragged step, inputs before
 * the step from state [slots, taps - 1, channels] (zeros for a row with row_ctx == 0); y to out32 (fp32) and / or
 * out_act (activation type); then the state keeps each row's last taps - 1 inputs. */
int mv_conv_taps(const float* in, int64_t ldi, float* state, const float* w, float* out32, int64_t ld32, void* out_act,
                 int64_t ldoa, int add_input, const int32_t* tok_row, const int32_t* row_start, const int32_t* row_len,
                 const int32_t* row_ctx, const int32_t* row_slot, int tokens, int rows, int channels, int taps, int f32,
                 mv_stream_t stream);
/* The same convolution (taps == 0: none) over the cq + ck + cv columns of one projection: the first cq to q (fp32),
 * the next ck into the token's row of k_cache [pages, page, ck], the last cv into v_cache [pages, page, cv]. */
int mv_conv_qkv_store(const float* in, int64_t ldi, float* state, const float* w, float* q, int64_t ldq, void* k_cache,
                      void* v_cache, const int32_t* tok_row, const int32_t* tok_pos, const int32_t* row_start,
                      const int32_t* row_len, const int32_t* row_ctx, const int32_t* row_slot,
                      const int32_t* block_table, int bt_stride, int page, int tokens, int rows, int cq, int ck, int cv,
                      int taps, int f32, mv_stream_t stream);
/* Two causal softmax maps per head over the same values: q [T, heads, 2, d] fp32, k_cache [pages, page, kv_heads, 2, d],
 * v_cache [pages, page, kv_heads, dv]; score = q.k * scale, then cap * tanh(score / cap) when cap > 0;
 * o = a1 - lambda a2; out[t, h, :] = act( o / sqrt(mean(o^2) + eps) * out_scale * sigmoid(gate[t, h]) ) (gate == NULL:
 * no gate).  chunks > 0: rows of more than max_len tokens run on the matrix cores where the shape allows it (bf16,
 * pages of 64, (d, dv) in {(32,32), (32,64), (64,64), (64,128), (128,128)}); short_tokens = tokens in the other rows
 * (-1: unknown). */
int mv_diff_attn(const float* q, int64_t ldq, const void* k_cache, const void* v_cache, void* out, int64_t ldo,
                 const float* gate, int64_t ldg, const int32_t* tok_row, const int32_t* tok_pos,
                 const int32_t* block_table, int bt_stride, int page, int tokens, int heads, int kv_heads, int d, int dv,
                 float scale, float cap, float lambda, float out_scale, float eps, int f32, const int32_t* row_len,
                 const int32_t* ch_start, const int32_t* ch_len, int chunks, int max_len, int short_tokens,
                 mv_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MVLLM_H */
