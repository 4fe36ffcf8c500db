/*
 * dflash_hip.h — C ABI of the MI355X (gfx950) DFlash speculative-verify kernels.
 *
 * One shared library, libdflash_hip.so.  Plain pointers and sizes only; no C++
 * types, no exceptions and no aborts cross this boundary.  Every array argument
 * is DEVICE memory owned by the caller unless a comment says "host".  Inputs are
 * never written, outputs are never allocated or freed here, and state_in may not
 * alias state_out.  All work is enqueued on the caller's stream (`stream` is a
 * hipStream_t passed as void*; NULL is the default stream) and the calls return
 * without synchronising.  The library is re-entrant.
 *
 * Return value of every `int` function:
 *    0                  work enqueued (DFLASH_OK)
 *    DFLASH_UNSUPPORTED the shape/dtype is outside what the kernels cover; nothing
 *                       was launched.  This is the analogue of the reference
 *                       returning nil / taking its ops path
 *                       (Sources/DFlash/DFlashKernels.swift:271-273, :744-758).
 *    DFLASH_INVALID     inconsistent arguments (NULL pointer, non-positive size,
 *                       Hv not a multiple of Hk, workspace too small ...).
 *    < 0                minus the hipError_t of a failed HIP call.
 * dflash_last_error() returns a thread-local description of the last failure.
 *
 * Layouts (row-major, last index fastest), as in the reference:
 *    q, k          [B, T, Hk, Dk]
 *    v, y, tape    [B, T, Hv, Dv]
 *    g             [B, T, Hv]        (g_ndim == 3, one decay per head)
 *                  [B, T, Hv, Dk]    (g_ndim == 4, one decay per key channel)
 *    beta          [B, T, Hv]
 *    state         [B, Hv, Dv, Dk]
 *    mask          [B, T]            a step runs when mask > 0.5
 *    g is the MULTIPLICATIVE decay (state * g), not its logarithm.
 *    Value head hv reads key head hv / (Hv / Hk).
 */
#ifndef DFLASH_HIP_H
#define DFLASH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DFLASH_OK 0
#define DFLASH_UNSUPPORTED 1
#define DFLASH_INVALID 2

/* Element types. */
#define DFLASH_F32 0
#define DFLASH_BF16 1
#define DFLASH_F16 2
#define DFLASH_U8 3 /* masks only */

#define DFLASH_MAX_BATCHED_LAYERS 64

int dflash_version(void);
const char* dflash_last_error(void);

/* Loads the code object on the current device and sizes the kernels' LDS
 * budgets.  Optional: every entry point does this on first use.  Thread-safe. */
int dflash_init(void);

/* ------------------------------------------------------------------------
 * Tape replay.  Replaces DFlashKernels.tapeReplayKernel
 * (Sources/DFlash/DFlashKernels.swift:252-301; Metal source :43-81; ops
 * restatement :371-407).  For t < T:  S <- S * g_t + tape_t (x) k_t ; a masked
 * step leaves S untouched.  The caller passes the accepted prefix
 * (T = nAccepted + 1, RecurrentRollbackCache.swift:115-125).
 *   tape_dtype : DFLASH_F32 (the recorded innovation tape) or == in_dtype
 *   in_dtype   : type of k and g
 *   state_dtype: DFLASH_F32, or == in_dtype in which case S is re-rounded to
 *                that type after every step as the Metal kernel does (:70).
 *   mask       : NULL, or [B,T] of mask_dtype (F32/BF16/F16/U8)
 * T == 0 copies state_in to state_out.
 * ---------------------------------------------------------------------- */
int dflash_tape_replay(void* stream,
                       const void* tape, int tape_dtype,
                       const void* k, const void* g, int in_dtype, int g_ndim,
                       const void* state_in, void* state_out, int state_dtype,
                       const void* mask, int mask_dtype,
                       int B, int T, int Hk, int Hv, int Dk, int Dv);

/* Replays `n_layers` independent caches in ONE launch.  Replaces the serial
 * loop over caches in DFlashRuntime.restoreTargetCacheAfterAcceptance
 * (Sources/DFlash/DFlashRuntime.swift:197-205), where every
 * RecurrentRollbackCache.rollback issues its own kernel.
 * The pointer arrays are HOST arrays of n_layers device pointers (copied into
 * the launch); all layers share shapes, dtypes and T_tape (the recorded tape
 * length, i.e. the stride-defining T of tape/k/g).
 * Steps replayed: `steps` when steps_dev == NULL, else min(*steps_dev, T_tape)
 * read on the device (an int32), which lets the accept kernel feed the replay
 * without a host round trip.  When skip_if_full != 0 and the step count equals
 * T_tape the kernel writes nothing: a fully accepted block keeps the state
 * the verify forward left in state_out (DFlashRuntime.swift:194,199-202).
 * n_layers <= DFLASH_MAX_BATCHED_LAYERS. */
int dflash_tape_replay_batched(void* stream, int n_layers,
                               const void* const* tape, int tape_dtype,
                               const void* const* k, const void* const* g, int in_dtype, int g_ndim,
                               const void* const* state_in, void* const* state_out, int state_dtype,
                               int steps, const int32_t* steps_dev, int skip_if_full,
                               int B, int T_tape, int Hk, int Hv, int Dk, int Dv);

/* ------------------------------------------------------------------------
 * GatedDelta forward that records the innovation tape.  Replaces
 * DFlashKernels.gatedDeltaKernelWithTape and the DFlashKernelProvider method of
 * the same name (DFlashKernels.swift:316-367, Metal :122-199, ops :409-466;
 * Sources/DFlash/DFlashKernelProvider.swift:8-14).  Per step:
 *   S' = S * g ; m = S' k ; delta = (v - m) * beta ; S = S' + delta (x) k ;
 *   y = S q.   A masked step keeps S and writes y = 0, delta = 0.
 *   q,k,v,g,beta : in_dtype          y : in_dtype        tape_out : float32
 *   state        : state_dtype (F32, or == in_dtype with per-step re-rounding,
 *                  DFlashKernels.swift:183-186)
 * state_out may be NULL: the post-block state is then not stored.  It is only
 * ever read when a block is accepted whole (DFlashRuntime.swift:194-202 keeps it
 * then; every other outcome replays from the snapshot and overwrites it), so a
 * host that rolls back with dflash_tape_replay* whatever was accepted
 * (skip_if_full = 0) does not need it, and the launch is about a tenth shorter
 * without the store.  Only the form used for verify blocks supports this (fp32
 * state, g_ndim == 3, Dk in {64,128,256}, Dv % 16 == 0, T >= 1); other shapes
 * return DFLASH_UNSUPPORTED when state_out is NULL.
 * ---------------------------------------------------------------------- */
int dflash_gated_delta_tape(void* stream,
                            const void* q, const void* k, const void* v,
                            const void* g, int g_ndim, const void* beta, int in_dtype,
                            const void* state_in, void* state_out, int state_dtype,
                            void* y, float* tape_out,
                            const void* mask, int mask_dtype,
                            int B, int T, int Hk, int Hv, int Dk, int Dv);

/* ------------------------------------------------------------------------
 * GatedDelta pre-ops: everything between the layer's projections and
 * dflash_gated_delta_tape, in one launch (layer code around the recurrence,
 * Sources/SwiftLM/KimiLinearDFlash.swift: ShortConv1d :274-293, q/k
 * normalisation :362-363, gates :390-391).
 *   mixed_qkv     [B, T, C], C = 2*Hk*Dk + Hv*Dv, channel order q | k | v
 *   conv_state_in [B, K-1, C] or NULL (zeros, :288); conv_weight [C, K], tap j
 *                 multiplies row t + j of concat(conv_state_in, mixed_qkv)
 *   out = silu(conv)                                                    (:291)
 *   q_out [B,T,Hk,Dk] = q_scale * rmsNorm(out_q, eps) per head; k_out likewise
 *                 with k_scale (:362-363); v_out [B,T,Hv,Dv] = out_v
 *   g_out = exp(-exp(A_log[h]) * softplus(a + dt_bias)), beta_out = sigmoid(b)
 *                 (:390-391); g_ndim 3: a [B,T,Hv], dt_bias [Hv];
 *                 g_ndim 4: a [B,T,Hv,Dk], dt_bias [Hv*Dk] (per-channel gate)
 *   conv_state_out [B, K-1, C] = last K-1 rows of the concatenation (:292) --
 *                 the window RecurrentRollbackCache snapshots; mixed_qkv itself is
 *                 what recordTape keeps as qkv (RecurrentRollbackCache.swift:139-158).
 * Tensors are `in_dtype` except A_log / dt_bias (float32 parameters).  2 <= K <= 8.
 * ---------------------------------------------------------------------- */
int dflash_gdn_prepare(void* stream,
                       const void* mixed_qkv, const void* conv_state_in, const void* conv_weight,
                       const void* a_logits, int g_ndim, const void* b_logits,
                       const float* A_log, const float* dt_bias, int in_dtype,
                       float q_scale, float k_scale, float norm_eps,
                       void* q_out, void* k_out, void* v_out, void* g_out, void* beta_out,
                       void* conv_state_out,
                       int B, int T, int Hk, int Hv, int Dk, int Dv, int K);

/* The layer's step after the recurrence (KimiLinearDFlash.swift:377-378, RMSNorm :341):
 *   out[b,t,h,:] = rmsNorm(y[b,t,h,:]; norm_weight [Dv], norm_eps) * act(gate[b,t,h,:])
 * gate_kind 0: act = sigmoid (the in-tree layer); 1: act = silu (the gated RMSNorm of
 * Qwen3-Next's linear-attention layer, whose source is not in the reference tree).
 * y, gate, out [B,T,Hv,Dv] and norm_weight in `in_dtype`.
 * ---------------------------------------------------------------------- */
int dflash_gdn_finish(void* stream, const void* y, const void* gate, const void* norm_weight, void* out,
                      int in_dtype, float norm_eps, int gate_kind, int B, int T, int Hv, int Dv);

/* ------------------------------------------------------------------------
 * One GatedDelta layer of the verify block, from its projections to the gated norm, in one call:
 * the body of the layer between its input and output projections
 * (Sources/SwiftLM/KimiLinearDFlash.swift:351-378: short conv + SiLU, q/k normalisation, gates,
 * the recurrence through DFlashKernelProvider.gatedDeltaKernelWithTape, oNorm(out) * act(gate)).
 * Equivalent to dflash_gdn_prepare -> dflash_gated_delta_tape -> dflash_gdn_finish, bit for bit,
 * in one launch instead of three: the pre-ops run inside the forward kernel's load phase, so
 * q, k, v, g and beta never travel through memory, and the gated norm -- which normalises over
 * the Dv rows of a head, spread by the forward over Dv/16 workgroups -- is done by whichever of
 * those workgroups finishes last (each counts itself in `arrivals`; none waits for another).
 *   inputs    mixed_qkv, conv_state_in (or NULL), conv_weight, a_logits [B,T,Hv], b_logits,
 *             A_log, dt_bias [Hv], q_scale, k_scale, norm_eps as for dflash_gdn_prepare;
 *             state_in [B,Hv,Dv,Dk] float32
 *   outputs   state_out (float32), tape_out [B,T,Hv,Dv] float32, y_out [B,T,Hv,Dv] (the
 *             recurrence's read-out before the norm), conv_state_out [B,K-1,C];
 *             k_out [B,T,Hk,Dk] and g_out [B,T,Hv]: what recordTape keeps for the replay
 *             (RecurrentRollbackCache.swift:75-85), NULL to skip;
 *             q_out, v_out, beta_out: optional copies of the other pre-op results, NULL to skip
 *   gate      NULL: stop after the recurrence.  Otherwise gate [B,T,Hv,Dv], out_norm_weight [Dv],
 *             out_norm_eps, gate_kind and out [B,T,Hv,Dv] as for dflash_gdn_finish (out must not
 *             alias y_out).
 *   arrivals  device int32 [B*Hv], all zero before the call; the call leaves it all zero, so one
 *             array zeroed once serves every later call that does not overlap with another one
 *             using the same array (calls on one stream never overlap).  NULL, or Dv > 256: the
 *             gated norm runs as a second launch, as dflash_gdn_finish.  A counter that is not
 *             zero when the launch begins (an array never cleared, or one a failed launch left
 *             half counted) makes `out` of that head meaningless; a count the launch itself
 *             cannot have produced sets DFLASH_STATUS_LAYER_ARRIVALS in the status word.
 *   aliasing  until the last workgroup of a head has written it, each row of `out` carries
 *             partial sums in its first Dv/16 floats.  The in-launch norm therefore needs `out`
 *             4-byte aligned and disjoint from gate and out_norm_weight; when it is not (a caller
 *             that norms in place, out == gate) the gated norm runs as the second launch, which
 *             allows that aliasing, and the results are the same bits.  out may never overlap y_out.
 * Covers the verify block: float32 state, one decay per head and step, no step mask, K == 4,
 * T <= 16, Dk in {64, 128, 256}, Dv a multiple of 16.  Anything else returns
 * DFLASH_UNSUPPORTED and the caller issues the three calls.
 * ---------------------------------------------------------------------- */
int dflash_gdn_layer(void* stream,
                     const void* mixed_qkv, const void* conv_state_in, const void* conv_weight,
                     const void* a_logits, const void* b_logits,
                     const float* A_log, const float* dt_bias, int in_dtype,
                     float q_scale, float k_scale, float norm_eps,
                     const void* state_in, void* state_out,
                     void* k_out, void* g_out, float* tape_out, void* conv_state_out, void* y_out,
                     const void* gate, const void* out_norm_weight, float out_norm_eps, int gate_kind,
                     void* out, int32_t* arrivals,
                     void* q_out, void* v_out, void* beta_out,
                     int B, int T, int Hk, int Hv, int Dk, int Dv, int K);

/* ------------------------------------------------------------------------
 * Block-causal batched GQA SDPA for the verify block.  Replaces
 * DFlashKernels.batchedSDPA2Pass (DFlashKernels.swift:737-815; Metal partials
 * :563-649, reduce :661-720); unlike it, covers every shape sdpaFallback
 * (:818-828) would be asked for at M == 16, so DFLASH_UNSUPPORTED mirrors the
 * reference's nil.
 *   q    [B, Hq, M, D]   contiguous, M must be 16 (:755)
 *   k,v  element (b, hk, n, d) at  b*kv_batch_stride + hk*kv_head_stride + n*D + d
 *        (strides in elements; a dense [B,Hk,N,D] has head stride N*D, batch
 *        stride Hk*N*D; a preallocated cache passes its capacity instead)
 *   N    number of keys INCLUDING the M block tokens; query row i sees keys
 *        0 .. N-M+i (:614).  hk = hq / (Hq/Hk) (:575).
 *   kv_len_dev  NULL, or device int32[B]: per-sequence key counts (ragged
 *        batches, or a count produced on the device); each must be in [M, N].
 *   out  [B, Hq, M, D] of `dtype`;  lse  NULL or float32 [B, Hq, M] receiving
 *        max + log(sum exp) of the scaled, masked scores (natural log).
 *   dtype DFLASH_BF16 or DFLASH_F16 (:756); D in {128, 256} (:757).
 *   workspace  device scratch of at least dflash_sdpa_workspace_bytes(...)
 *        bytes, 256-byte aligned; contents are undefined afterwards.
 * ---------------------------------------------------------------------- */
size_t dflash_sdpa_workspace_bytes(int B, int Hq, int Hk, int M, int N, int D);

int dflash_sdpa_block_causal(void* stream,
                             const void* q, const void* k, const void* v,
                             void* out, float* lse, int dtype, float scale,
                             int B, int Hq, int Hk, int M, int N, int D,
                             int64_t kv_batch_stride, int64_t kv_head_stride,
                             const int32_t* kv_len_dev,
                             void* workspace, size_t workspace_bytes);

/* dflash_sdpa_block_causal without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory where they
 * call it: code inside a HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The split-KV partial rows and their statistics go to an array of
 * DFLASH_SDPA_STATIC_SCRATCH_BYTES that lives in the library's code object (every GPU the library
 * runs on holds its own copy until the process ends); its address is looked up once per device by
 * dflash_init() -- call that once at set-up, outside any capture; afterwards this entry makes no
 * allocating call (no hipMalloc / hipFree, no allocating library routine).
 * Arguments, results and return codes are those of dflash_sdpa_block_causal; a shape whose split-KV
 * scratch exceeds the array (about B*Hq*16 rows x splits x (2*D + 8) bytes; the benchmark shape
 * B=1, Hq=16, Hk=2, D=256 needs 17.0 MB) returns DFLASH_UNSUPPORTED with the two sizes in
 * dflash_last_error(), and the caller uses the workspace entry.
 * Every call on a GPU shares that GPU's array and finds the previous call's contents in it (nothing
 * in it has to start at zero: each call writes every statistic it later reads).  Calls that overlap
 * on one GPU -- two streams, or two threads -- race on it; serialise them or use the workspace entry.
 * ---------------------------------------------------------------------- */
#define DFLASH_SDPA_STATIC_SCRATCH_BYTES (18 * 1024 * 1024)
int dflash_sdpa_block_causal_static(void* stream,
                                    const void* q, const void* k, const void* v,
                                    void* out, float* lse, int dtype, float scale,
                                    int B, int Hq, int Hk, int M, int N, int D,
                                    int64_t kv_batch_stride, int64_t kv_head_stride,
                                    const int32_t* kv_len_dev);

/* The same attention with the reference's optional additive mask (masked partials
 * kernel, DFlashKernels.swift:546-555; selected at :783-787).  mask [B, Hq, M, N]
 * contiguous, in `dtype` (the reference casts it to the input type, :784).  A key
 * is used when it passes the block-causal rule AND its mask value is at least the
 * lowest finite value of `dtype` (:551); the mask value is added to the scaled
 * score (:553).  A row without any usable key gets zeros (:711) and lse = -inf.
 * ---------------------------------------------------------------------- */
int dflash_sdpa_block_causal_masked(void* stream,
                                    const void* q, const void* k, const void* v, const void* mask,
                                    void* out, float* lse, int dtype, float scale,
                                    int B, int Hq, int Hk, int M, int N, int D,
                                    int64_t kv_batch_stride, int64_t kv_head_stride,
                                    const int32_t* kv_len_dev,
                                    void* workspace, size_t workspace_bytes);

/* The same attention with the block's K/V append fused in: the verify forward's
 * KVCacheSimple.update (mlx-swift-lm, reached from the attention layer the
 * reference's batchedSDPA2Pass was written for) followed by the SDPA, in one launch
 * pair.  k_new, v_new [B, Hk, M, D] are the block's rows; they stand for keys
 * N-M .. N-1 (per sequence: kv_len-M .. kv_len-1), are read from k_new/v_new by the
 * attention, and are stored into those rows of k_cache/v_cache (layout as k/v
 * above) by the same kernel, so a following call finds them in the cache.  N must
 * not exceed the cache's capacity in rows.  cache_len_dev (NULL, or device
 * int32[B]) counts the rows ALREADY in the cache, block excluded, i.e. the cache
 * offset the accept kernel maintains; sequence b then has cache_len_dev[b] + M keys,
 * which must not exceed N.
 * ---------------------------------------------------------------------- */
int dflash_sdpa_block_causal_append(void* stream,
                                    const void* q, void* k_cache, void* v_cache,
                                    const void* k_new, const void* v_new,
                                    void* out, float* lse, int dtype, float scale,
                                    int B, int Hq, int Hk, int M, int N, int D,
                                    int64_t kv_batch_stride, int64_t kv_head_stride,
                                    const int32_t* cache_len_dev,
                                    void* workspace, size_t workspace_bytes);

/* The same attention over a PAGED K/V cache.  The reference's cache is one dense
 * [B, Hk, N, D] array per layer (KVCacheSimple in mlx-swift-lm; the attention reads it
 * as DFlashKernels.swift:737-743 receives it), so paging has no counterpart there: the
 * entry computes exactly what dflash_sdpa_block_causal / _append compute on the dense
 * array that gathering the pages would give, bit for bit.
 *
 * k_pool, v_pool hold num_pages pages; page p, head h, row r, channel d sits at element
 * p * page_stride + h * head_stride + r * D + d (head_stride >= page_size * D, page_stride
 * >= (Hk-1) * head_stride + page_size * D, both multiples of 8).  page_size is a power of
 * two >= 32.  Key n of sequence b lives in page page_table[b * page_table_stride + n /
 * page_size] (device int32; page_table_stride * page_size >= N), row n % page_size.  Entries
 * are clamped to [0, num_pages) on the device, so a stale table cannot address outside the pool.
 *
 * k_new == v_new == NULL: plain attention, len_dev as kv_len_dev above (keys per sequence,
 * block included).  Otherwise k_new, v_new [B, Hk, M, D] are the block's rows as in the
 * append entry: read from there, stored into the pages that hold keys len..len+M-1 (which
 * the table must already map), and len_dev counts the rows already cached, block excluded.
 * No additive mask.  Returns DFLASH_UNSUPPORTED for a page size the kernel does not
 * take.
 * ---------------------------------------------------------------------- */
int dflash_sdpa_block_causal_paged(void* stream,
                                   const void* q, void* k_pool, void* v_pool,
                                   const int32_t* page_table, int page_table_stride,
                                   int page_size, int num_pages,
                                   int64_t page_stride, int64_t head_stride,
                                   const void* k_new, const void* v_new,
                                   void* out, float* lse, int dtype, float scale,
                                   int B, int Hq, int Hk, int M, int N, int D,
                                   const int32_t* len_dev,
                                   void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Acceptance.  dflash_match_acceptance_length replaces
 * DFlashRuntime.matchAcceptanceLength (Sources/DFlash/DFlashRuntime.swift:
 * 133-142): out[0] = number of leading positions with drafted[i] == posterior[i]
 * (0 when n == 0).  Tokens are uint32 on the device; out is a device int32.
 *
 * dflash_accept_commit does one verify cycle's integer bookkeeping on the
 * device (DFlashRuntime.swift:490-493, :525-530, :544-547, :571):
 *   verify_ids [V] = [staged_first, drafted...] ; posterior [V]
 *   out[0] = acceptanceLen = leading matches of verify_ids[1:] vs posterior[:V-1]
 *   out[1] = commitCount   = 1 + acceptanceLen  (= steps to replay)
 *   out[2] = stagedFirstNext = posterior[acceptanceLen]
 *   out[3] = *start_inout += commitCount (start_inout may be NULL -> commitCount)
 * ---------------------------------------------------------------------- */
int dflash_match_acceptance_length(void* stream, const uint32_t* drafted, const uint32_t* posterior,
                                   int n, int32_t* out);
int dflash_accept_commit(void* stream, const uint32_t* verify_ids, const uint32_t* posterior, int V,
                         int32_t* start_inout, int32_t* out4);

/* dflash_accept_commit and dflash_tape_replay_batched in ONE launch: the replay kernel
 * decides the acceptance itself (steps = commitCount = 1 + acceptanceLen; with
 * skip_if_full a fully accepted block, commitCount == T_tape, writes no state) and
 * leaves out4 / start_inout exactly as dflash_accept_commit would.  V <= T_tape + 1.
 * Arguments as for the two calls it replaces (DFlashRuntime.swift:525-547 followed
 * by the per-cache loop :197-205). */
int dflash_accept_commit_replay_batched(void* stream, const uint32_t* verify_ids, const uint32_t* posterior,
                                        int V, int32_t* start_inout, int32_t* out4, int n_layers,
                                        const void* const* tape, int tape_dtype, const void* const* k,
                                        const void* const* g, int in_dtype, int g_ndim,
                                        const void* const* state_in, void* const* state_out, int state_dtype,
                                        int skip_if_full, int B, int T_tape, int Hk, int Hv, int Dk, int Dv);

/* ------------------------------------------------------------------------
 * Greedy tokens over the verify logits.  dflash_greedy_tokens_with_mask replaces
 * DFlashRuntime.greedyTokensWithMask (DFlashRuntime.swift:118-128):
 *   tokens_out[t] = argmax_v where(suppress_mask[v], (dtype)(-1e9), logits[t, v])
 * with the lowest index winning a tie (the array library's argMax is not in the
 * reference tree; first-index is what its callers' tests and numpy/torch agree
 * on).  logits [T, V] row-major in `dtype` (f32/bf16/f16); suppress_mask NULL or
 * uint8 [V], non-zero = suppressed (buildSuppressTokenMask, :105-115).
 *
 * dflash_greedy_accept_commit does that and dflash_accept_commit's bookkeeping in
 * one call (the cycle's :513-547; two launches: per-chunk maxima, then one
 * workgroup that reduces them and does the bookkeeping): posterior_out [T] receives
 * the greedy tokens, out4 / start_inout are as for dflash_accept_commit with V == T.
 *
 * workspace: at least dflash_greedy_workspace_bytes(T, V) bytes, 256-byte
 * aligned; contents are undefined before and after.
 * ---------------------------------------------------------------------- */
size_t dflash_greedy_workspace_bytes(int T, int V);
int dflash_greedy_tokens_with_mask(void* stream, const void* logits, int dtype, int T, int V,
                                   const uint8_t* suppress_mask, uint32_t* tokens_out,
                                   void* workspace, size_t workspace_bytes);
int dflash_greedy_accept_commit(void* stream, const void* logits, int dtype, int T, int V,
                                const uint8_t* suppress_mask, const uint32_t* verify_ids,
                                int32_t* start_inout, int32_t* out4, uint32_t* posterior_out,
                                void* workspace, size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Conv-state rebuild after rollback.  Replaces
 * RecurrentRollbackCache.rebuildConvState (Sources/DFlash/
 * RecurrentRollbackCache.swift:139-158):
 *   out[b, j, :] = concat(snapshot_conv [B,keep,C], tape_qkv [B,T,C])[b, s + j, :]
 * for j < min(keep, keep + T - s), s = accepted_steps (or *steps_dev when not
 * NULL).  snapshot_conv == NULL stands for zeros (:147-152).  elem_bytes is the
 * element size (2 or 4).  Rows past the clamp are left untouched; the number of
 * valid rows is min(keep, keep + T - s) as in the reference's clamped slice.
 * ---------------------------------------------------------------------- */
int dflash_rebuild_conv_state(void* stream, const void* snapshot_conv, const void* tape_qkv, void* out,
                              int B, int keep, int T, int C, int elem_bytes,
                              int accepted_steps, const int32_t* steps_dev);

/* ------------------------------------------------------------------------
 * KV append for an attention layer at verify (the KVCacheSimple.update the
 * reference delegates to mlx-swift-lm, trimmed by DFlashRuntime.swift:212-218):
 * copies k_new/v_new [B, Hk, M, D] to rows [offset, offset+M) of a cache laid out
 * like k/v above.  offset comes from *offset_dev when not NULL.  new_len_dev, when
 * not NULL, receives offset + M (the cache's length after the append, which is
 * the N of the attention call that follows).  An append that would pass the
 * capacity writes nothing.
 * ---------------------------------------------------------------------- */
int dflash_kv_append(void* stream, void* k_cache, void* v_cache, const void* k_new, const void* v_new,
                     int B, int Hk, int M, int D, int elem_bytes,
                     int64_t kv_batch_stride, int64_t kv_head_stride,
                     int offset, const int32_t* offset_dev, int capacity, int32_t* new_len_dev);

/* ------------------------------------------------------------------------
 * Device-side status word (no counterpart in the reference, whose lengths all live on the host).
 * Several entries read a length from DEVICE memory (kv_len_dev / cache_len_dev, offset_dev, steps_dev),
 * so the host cannot check it before the launch.  A value outside the entry's contract never makes a kernel
 * read or write outside the caller's buffers -- it is clamped, or the write is skipped -- but the result is
 * then not the one asked for.  To see that it happened, register a device int32 with
 * dflash_set_status_word(): from then on (for launches enqueued by ANY thread, until it is replaced or
 * cleared with NULL) the kernels OR the bits below into it, and the caller reads it back whenever it likes,
 * e.g. together with the accept words.  The library never clears it.
 *   DFLASH_STATUS_SDPA_LEN      an attention entry found kv_len_dev[b] (or cache_len_dev[b] + M) outside [M, N]
 *                               and clamped it (a fused append then stored the block at the clamped position)
 *   DFLASH_STATUS_APPEND_RANGE  dflash_kv_append found rows [offset, offset + M) outside the capacity: nothing
 *                               was written and new_len_dev was left alone
 *   DFLASH_STATUS_CONV_STEPS    dflash_rebuild_conv_state found *steps_dev outside [0, T]: rows past the end of
 *                               the concatenation were left unwritten
 *   DFLASH_STATUS_LAYER_ARRIVALS dflash_gdn_layer found an arrival counter at or above Dv/16, which no launch on a
 *                               zeroed array produces: `arrivals` was not all zero before the call
 * The pointer is read when a call is ENQUEUED and travels in the kernel's arguments: a captured HIP graph keeps the
 * word that was registered at capture time and writes to it on every replay, so that word must outlive the graph
 * (clearing or replacing the registration later does not reach launches already captured).
 * ---------------------------------------------------------------------- */
#define DFLASH_STATUS_SDPA_LEN 1
#define DFLASH_STATUS_APPEND_RANGE 2
#define DFLASH_STATUS_CONV_STEPS 4
#define DFLASH_STATUS_LAYER_ARRIVALS 8
int dflash_set_status_word(int32_t* status_dev);

#ifdef __cplusplus
}
#endif
#endif /* DFLASH_HIP_H */
