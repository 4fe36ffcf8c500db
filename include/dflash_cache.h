/*
 * dflash_cache.h — host-side rollback caches and the accept/rollback step of
 * the DFlash verify loop, as opaque handles over the kernels of dflash_hip.h.
 *
 * These mirror the reference's cache objects.  A cache owns NO device memory:
 * like the reference's caches, which hold reference-counted arrays, a handle
 * holds the caller's device pointers for its two slots (slot 0 = conv window
 * [B, keep, C], slot 1 = recurrent state [B, Hv, Dv, Dk]) and, while armed,
 * pointers to the pre-verify slots (the snapshot) and to the recorded tape.
 * The caller keeps every buffer alive until the cycle's rollback or
 * clear_transients has been enqueued and has run.
 *
 * Functional update contract (the reference's arrays are immutable): the verify
 * forward must write the post-verify state and conv window into buffers
 * DIFFERENT from the ones that were in the slots when the cache was armed, then
 * store the new pointers with dflash_cache_set_slot.  On a partial acceptance
 * rollback() replays the tape from the snapshot INTO those post-verify buffers
 * (their content is the rejected state and is dead), so afterwards the slots
 * still point at them and hold the rolled-back state.
 *
 * Thread safety: a handle may be used by one thread at a time.
 */
#ifndef DFLASH_CACHE_H
#define DFLASH_CACHE_H

#include <stdint.h>

#include "dflash_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dflash_cache dflash_cache_t;

/* Cache kinds. */
#define DFLASH_CACHE_TAPE 0     /* RecurrentRollbackCache  (RecurrentRollbackCache.swift:34-182)  */
#define DFLASH_CACHE_SNAPSHOT 1 /* MambaSnapshotCache      (RecurrentRollbackCache.swift:193-232) */
#define DFLASH_CACHE_MAMBA 2    /* plain MambaCache: no rollback (DFlashRuntime.swift:206-211)    */
#define DFLASH_CACHE_KV 3       /* trimmable attention KV cache  (DFlashRuntime.swift:212-218)    */

/* conv_kernel_size: the GDN layer's depthwise-conv width; the conv window keeps
 * conv_kernel_size - 1 rows (RecurrentRollbackCache.defaultConvKernelSize = 4,
 * RecurrentRollbackCache.swift:135,141).  Ignored for KV caches.  NULL on failure. */
dflash_cache_t* dflash_cache_create(int kind, int conv_kernel_size);
void dflash_cache_destroy(dflash_cache_t* c);
int dflash_cache_kind(const dflash_cache_t* c);

/* Slots (`self[0]`, `self[1]` in the reference) and the token offset. */
int dflash_cache_set_slot(dflash_cache_t* c, int slot, void* dev_ptr);
void* dflash_cache_get_slot(const dflash_cache_t* c, int slot);
int64_t dflash_cache_offset(const dflash_cache_t* c);
int dflash_cache_set_offset(dflash_cache_t* c, int64_t offset);

/* DFlashRollbackCache protocol (RecurrentRollbackCache.swift:12-18). */
int dflash_cache_is_armed(const dflash_cache_t* c);
/* armRollback(prefixLen:): arm and snapshot both slots by reference (:63-71, :201-206). */
int dflash_cache_arm_rollback(dflash_cache_t* c, int64_t prefix_len);
/* recordTape(tape:k:g:qkv:) (:75-85).  Shapes of what was recorded:
 * tape [B,T,Hv,Dv] of tape_dtype, k [B,T,Hk,Dk] and g ([B,T,Hv] or
 * [B,T,Hv,Dk]) of in_dtype, qkv [B,T,C] with qkv_elem_bytes-sized elements
 * (may be NULL: the conv window is then left as it is, :140).  state_dtype is the
 * type of slot 1.  A snapshot-only cache ignores the call (:222-224). */
int dflash_cache_record_tape(dflash_cache_t* c, const void* tape, int tape_dtype, const void* k, const void* g,
                             int in_dtype, int g_ndim, const void* qkv, int qkv_elem_bytes, int state_dtype,
                             int B, int T, int Hk, int Hv, int Dk, int Dv, int C);
/* rollback(nAccepted:) (:95-131, :208-214): restores the snapshot, replays
 * acceptedSteps = nAccepted + 1 tape steps (:115) and rebuilds the conv window
 * (:139-158), enqueued on `stream`; then clears the transients. */
int dflash_cache_rollback(dflash_cache_t* c, void* stream, int n_accepted);
/* clearTransients() (:163-170, :216-220). */
int dflash_cache_clear_transients(dflash_cache_t* c);
/* trim(_:) (:175-181, :227-231): offset -= min(offset, n); returns the amount trimmed. */
int64_t dflash_cache_trim(dflash_cache_t* c, int64_t n);

/* DFlashRuntime.restoreTargetCacheAfterAcceptance (Sources/DFlash/
 * DFlashRuntime.swift:188-223), also what both DFlashEngine.rollback
 * implementations forward to (Sources/DFlash/DFlashEngine.swift:41-53, :71-83).
 * Fully accepted (drafted_tokens > 0 && acceptance_length == drafted_tokens):
 * rollback caches only clear their transients, no replay.  Otherwise tape caches
 * are rolled back (all tape caches that share shapes replay in ONE launch),
 * snapshot caches restore, plain Mamba caches take offset = target_len, KV caches
 * are trimmed to target_len.  *replay_ns (may be NULL) receives the host time
 * spent enqueuing the rollbacks, the quantity the reference returns. */
int dflash_restore_target_cache_after_acceptance(dflash_cache_t* const* caches, int n_caches, void* stream,
                                                 int64_t target_len, int acceptance_length, int drafted_tokens,
                                                 int64_t* replay_ns);

#ifdef __cplusplus
}
#endif
#endif /* DFLASH_CACHE_H */
