// Host-side rollback caches of the DFlash verify loop (no device code here).
// Mirrors Sources/DFlash/RecurrentRollbackCache.swift and
// DFlashRuntime.restoreTargetCacheAfterAcceptance (DFlashRuntime.swift:188-223).

#include <chrono>
#include <new>
#include <vector>

#include "../../include/dflash_cache.h"
#include "dflash_common.h"

struct dflash_cache {
    int kind = DFLASH_CACHE_TAPE;
    int keep = 3;                 // conv_kernel_size - 1
    void* slot[2] = {nullptr, nullptr};
    int64_t offset = 0;
    bool armed = false;
    bool has_snapshot = false;
    void* snap[2] = {nullptr, nullptr};
    // recorded tape
    bool has_tape = false;
    const void *tape = nullptr, *k = nullptr, *g = nullptr, *qkv = nullptr;
    int tape_dtype = 0, in_dtype = 0, g_ndim = 3, qkv_elem_bytes = 2, state_dtype = 0;
    int B = 0, T = 0, Hk = 0, Hv = 0, Dk = 0, Dv = 0, C = 0;
};

namespace {

using dflash::set_error;

bool is_rollback_kind(int kind) { return kind == DFLASH_CACHE_TAPE || kind == DFLASH_CACHE_SNAPSHOT; }

void clear_transients(dflash_cache* c) {   // RecurrentRollbackCache.swift:163-170
    c->armed = false;
    c->has_tape = false;
    c->tape = c->k = c->g = c->qkv = nullptr;
    c->has_snapshot = false;
    c->snap[0] = c->snap[1] = nullptr;
}

bool same_shape(const dflash_cache* a, const dflash_cache* b) {
    return a->tape_dtype == b->tape_dtype && a->in_dtype == b->in_dtype && a->g_ndim == b->g_ndim &&
           a->state_dtype == b->state_dtype && a->B == b->B && a->T == b->T && a->Hk == b->Hk && a->Hv == b->Hv &&
           a->Dk == b->Dk && a->Dv == b->Dv;
}

// What a tape cache has to do on rollback, after the snapshot has been restored.
struct ReplayJob {
    dflash_cache* c;
    void* post_state;
    void* post_conv;
    int steps;
};

// Checks a rollback WITHOUT changing the cache and says whether a tape replay will run
// (RecurrentRollbackCache.swift:95-128).  Validation is kept apart from the restore so that a call that is
// going to fail leaves every cache exactly as it was: still armed, tape and snapshot in place.
int validate_rollback(const dflash_cache* c, int n_accepted, bool* need_replay) {
    *need_replay = false;
    if (!c->has_snapshot) return DFLASH_OK;                       // :96-99, caller clears
    if (c->kind != DFLASH_CACHE_TAPE) return DFLASH_OK;           // snapshot-only: :208-214
    const void* restored1 = c->snap[1] ? c->snap[1] : c->slot[1]; // slot 1 as it will be after :108-109
    if (!(c->has_tape && restored1)) return DFLASH_OK;            // :112-113
    DFLASH_REQUIRE(n_accepted >= 0, "rollback: negative n_accepted");
    const void* post0 = c->slot[0];
    const void* post1 = c->slot[1];
    DFLASH_REQUIRE(post1 && post1 != c->snap[1],
                   "rollback: slot 1 still holds the pre-verify buffer; the forward must write a new one");
    if (c->qkv && c->keep > 0) {
        // The rebuilt window is written into the post-verify conv buffer while snapshot and qkv are read:
        // the three must not share memory (a slice of qkv handed over as the window is a view of it).
        const size_t win = (size_t)c->B * c->keep * c->C * c->qkv_elem_bytes;
        const size_t tape_bytes = (size_t)c->B * c->T * c->C * c->qkv_elem_bytes;
        const uintptr_t o = (uintptr_t)post0, q = (uintptr_t)c->qkv, sn = (uintptr_t)c->snap[0];
        const bool hits_qkv = o < q + tape_bytes && q < o + win;
        const bool hits_snap = sn && o < sn + win && sn < o + win;
        DFLASH_REQUIRE(post0 && !hits_qkv && !hits_snap,
                       "rollback: slot 0 must be a conv buffer that shares no memory with the snapshot or with qkv");
    }
    *need_replay = true;
    return DFLASH_OK;
}

// Restores the snapshot (:108-109) of a cache that passed validate_rollback and, when a replay is due, fills in
// the job.  Cannot fail.
void restore_snapshot(dflash_cache* c, int n_accepted, bool need_replay, ReplayJob* job) {
    if (!c->has_snapshot) return;
    void* post0 = c->slot[0];
    void* post1 = c->slot[1];
    if (c->snap[0]) c->slot[0] = c->snap[0];
    if (c->snap[1]) c->slot[1] = c->snap[1];
    if (!need_replay) return;
    int steps = n_accepted + 1;                                   // :115
    if (steps > c->T) steps = c->T;                               // slices clamp to the recorded length
    job->c = c; job->post_state = post1; job->post_conv = post0; job->steps = steps;
}

int finish_rollback(const ReplayJob& j, void* stream) {
    dflash_cache* c = j.c;
    c->slot[1] = j.post_state;                                    // :126, the replayed state
    if (c->keep <= 0) { c->slot[0] = nullptr; return DFLASH_OK; } // :142
    if (!c->qkv) return DFLASH_OK;                                // :140, keeps the restored window
    int rc = dflash_rebuild_conv_state(stream, c->snap[0], c->qkv, j.post_conv, c->B, c->keep, c->T, c->C,
                                       c->qkv_elem_bytes, j.steps, nullptr);
    if (rc) return rc;
    c->slot[0] = j.post_conv;                                     // :127
    return DFLASH_OK;
}

int replay_jobs(const std::vector<ReplayJob>& jobs, void* stream) {
    std::vector<bool> done(jobs.size(), false);
    for (size_t i = 0; i < jobs.size(); ++i) {
        if (done[i]) continue;
        const dflash_cache* a = jobs[i].c;
        std::vector<const void*> tape, k, g, sin;
        std::vector<void*> sout;
        for (size_t j = i; j < jobs.size() && tape.size() < DFLASH_MAX_BATCHED_LAYERS; ++j) {
            if (done[j] || jobs[j].steps != jobs[i].steps || !same_shape(a, jobs[j].c)) continue;
            done[j] = true;
            tape.push_back(jobs[j].c->tape); k.push_back(jobs[j].c->k); g.push_back(jobs[j].c->g);
            sin.push_back(jobs[j].c->snap[1]); sout.push_back(jobs[j].post_state);
        }
        int rc = dflash_tape_replay_batched(stream, (int)tape.size(), tape.data(), a->tape_dtype, k.data(), g.data(),
                                            a->in_dtype, a->g_ndim, sin.data(), sout.data(), a->state_dtype,
                                            jobs[i].steps, nullptr, 0, a->B, a->T, a->Hk, a->Hv, a->Dk, a->Dv);
        if (rc) return rc;
    }
    for (const ReplayJob& j : jobs) {
        int rc = finish_rollback(j, stream);
        if (rc) return rc;
    }
    return DFLASH_OK;
}

}  // namespace

extern "C" dflash_cache_t* dflash_cache_create(int kind, int conv_kernel_size) {
    if (kind < DFLASH_CACHE_TAPE || kind > DFLASH_CACHE_KV) { set_error("cache_create: bad kind %d", kind); return nullptr; }
    dflash_cache* c = new (std::nothrow) dflash_cache();
    if (!c) { set_error("cache_create: out of memory"); return nullptr; }
    c->kind = kind;
    c->keep = conv_kernel_size - 1;
    return c;
}

extern "C" void dflash_cache_destroy(dflash_cache_t* c) { delete c; }
extern "C" int dflash_cache_kind(const dflash_cache_t* c) { return c ? c->kind : -1; }

extern "C" int dflash_cache_set_slot(dflash_cache_t* c, int slot, void* p) {
    DFLASH_REQUIRE(c && (slot == 0 || slot == 1), "cache_set_slot: bad arguments");
    c->slot[slot] = p;
    return DFLASH_OK;
}
extern "C" void* dflash_cache_get_slot(const dflash_cache_t* c, int slot) {
    return (c && (slot == 0 || slot == 1)) ? c->slot[slot] : nullptr;
}
extern "C" int64_t dflash_cache_offset(const dflash_cache_t* c) { return c ? c->offset : -1; }
extern "C" int dflash_cache_set_offset(dflash_cache_t* c, int64_t offset) {
    DFLASH_REQUIRE(c && offset >= 0, "cache_set_offset: bad arguments");
    c->offset = offset;
    return DFLASH_OK;
}

extern "C" int dflash_cache_is_armed(const dflash_cache_t* c) { return c && c->armed ? 1 : 0; }

extern "C" int dflash_cache_arm_rollback(dflash_cache_t* c, int64_t /*prefix_len*/) {
    DFLASH_REQUIRE(c, "cache_arm_rollback: null handle");
    DFLASH_REQUIRE(is_rollback_kind(c->kind), "cache_arm_rollback: cache kind %d has no rollback", c->kind);
    c->armed = true;                                              // RecurrentRollbackCache.swift:64
    c->has_tape = false;
    c->tape = c->k = c->g = c->qkv = nullptr;                     // :65-68
    c->snap[0] = c->slot[0];                                      // :70, by reference
    c->snap[1] = c->slot[1];
    c->has_snapshot = true;
    return DFLASH_OK;
}

extern "C" int dflash_cache_record_tape(dflash_cache_t* c, const void* tape, int tape_dtype, const void* k,
                                        const void* g, int in_dtype, int g_ndim, const void* qkv, int qkv_elem_bytes,
                                        int state_dtype, int B, int T, int Hk, int Hv, int Dk, int Dv, int C) {
    DFLASH_REQUIRE(c, "cache_record_tape: null handle");
    DFLASH_REQUIRE(is_rollback_kind(c->kind), "cache_record_tape: cache kind %d records no tape", c->kind);
    if (c->kind == DFLASH_CACHE_SNAPSHOT) return DFLASH_OK;       // :222-224
    DFLASH_REQUIRE(tape && k && g, "cache_record_tape: null tape/k/g");
    DFLASH_REQUIRE(B > 0 && T > 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, "cache_record_tape: non-positive dimension");
    DFLASH_REQUIRE(!qkv || C > 0, "cache_record_tape: qkv given without its channel count");
    c->tape = tape; c->k = k; c->g = g; c->qkv = qkv;
    c->tape_dtype = tape_dtype; c->in_dtype = in_dtype; c->g_ndim = g_ndim; c->qkv_elem_bytes = qkv_elem_bytes;
    c->state_dtype = state_dtype;
    c->B = B; c->T = T; c->Hk = Hk; c->Hv = Hv; c->Dk = Dk; c->Dv = Dv; c->C = C;
    c->has_tape = true;
    return DFLASH_OK;
}

extern "C" int dflash_cache_rollback(dflash_cache_t* c, void* stream, int n_accepted) {
    DFLASH_REQUIRE(c, "cache_rollback: null handle");
    DFLASH_REQUIRE(is_rollback_kind(c->kind), "cache_rollback: cache kind %d has no rollback", c->kind);
    ReplayJob job;
    bool need = false;
    int rc = validate_rollback(c, n_accepted, &need);
    if (rc) return rc;                                            // nothing was touched: the cache is still armed
    restore_snapshot(c, n_accepted, need, &job);
    if (need) rc = replay_jobs(std::vector<ReplayJob>{job}, stream);
    clear_transients(c);                                          // :130
    return rc;
}

extern "C" int dflash_cache_clear_transients(dflash_cache_t* c) {
    DFLASH_REQUIRE(c, "cache_clear_transients: null handle");
    clear_transients(c);
    return DFLASH_OK;
}

extern "C" int64_t dflash_cache_trim(dflash_cache_t* c, int64_t n) {
    if (!c || n < 0) return 0;
    const int64_t trimmed = c->offset < n ? c->offset : n;        // :178-180
    c->offset -= trimmed;
    return trimmed;
}

extern "C" int dflash_restore_target_cache_after_acceptance(dflash_cache_t* const* caches, int n_caches, void* stream,
                                                            int64_t target_len, int acceptance_length,
                                                            int drafted_tokens, int64_t* replay_ns) {
    DFLASH_REQUIRE(n_caches >= 0 && (n_caches == 0 || caches), "restore_target_cache: bad arguments");
    const bool fully = drafted_tokens > 0 && acceptance_length == drafted_tokens;   // DFlashRuntime.swift:194
    int64_t ns = 0;
    int rc = DFLASH_OK;
    const auto t0 = std::chrono::steady_clock::now();
    // First pass: every handle and every rollback is checked; nothing is changed.  A failure here returns with
    // all caches as they were (armed, tapes and snapshots in place), so the caller can correct and call again.
    std::vector<char> need((size_t)n_caches, 0);
    for (int i = 0; i < n_caches; ++i) {
        const dflash_cache* c = caches[i];
        DFLASH_REQUIRE(c, "restore_target_cache: null cache handle at %d", i);
        if (is_rollback_kind(c->kind) && !fully) {
            bool n = false;
            rc = validate_rollback(c, acceptance_length, &n);
            if (rc) return rc;
            need[(size_t)i] = n;
        }
    }
    // Second pass: restore, collect the replays, fix the offsets.
    std::vector<ReplayJob> jobs;
    for (int i = 0; i < n_caches; ++i) {
        dflash_cache* c = caches[i];
        if (is_rollback_kind(c->kind)) {
            if (fully) { clear_transients(c); continue; }                          // :199-202
            ReplayJob job;
            restore_snapshot(c, acceptance_length, need[(size_t)i] != 0, &job);    // :204
            if (need[(size_t)i]) jobs.push_back(job);
        } else if (c->kind == DFLASH_CACHE_MAMBA) {
            c->offset = target_len;                                                // :211
        } else if (c->offset > target_len) {                                       // :212-218
            dflash_cache_trim(c, c->offset - target_len);
        }
    }
    if (!jobs.empty()) rc = replay_jobs(jobs, stream);
    if (!fully)
        for (int i = 0; i < n_caches; ++i)
            if (is_rollback_kind(caches[i]->kind)) clear_transients(caches[i]);
    ns = std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
    if (replay_ns) *replay_ns = ns;
    return rc;
}
