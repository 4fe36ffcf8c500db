/* A whole verify step without Python: a small hybrid stack (three GatedDelta layers and one attention layer, the
 * 3:1 pattern of the benchmark's stack) driven by a plain C host through include/dflash_hip.h and the HIP runtime's
 * C API only, the way a Swift (or any non-Python) host would drive it:
 *
 *   per step   3 x dflash_gated_delta_tape            pre-verify state -> post-verify state + innovation tape
 *              1 x dflash_sdpa_block_causal_append     the block's K/V rows appended at the device-side offset, attention
 *              1 x dflash_accept_commit_replay_batched acceptance, offset += commit count, rollback of all three caches
 *
 * Two steps (the two phases of the ping-pong state buffers) are captured with hipStreamBeginCapture on a fresh
 * stream, instantiated once and launched twice; nothing in a step needs the host (commit count, cache offset and
 * "fully accepted" stay on the device), which is what makes the capture legal.  The same four steps are then run
 * eagerly on a second set of buffers.  Checked: graph == eager byte for byte; accept words and offset against the
 * indexing of Sources/DFlash/DFlashRuntime.swift:525-547,:571; every layer's recurrent state against a double-precision
 * recurrence over exactly the committed tokens (the rollback contract, RecurrentRollbackCache.swift:95-131; rtol 1e-4
 * of the state's scale); the appended cache rows bit for bit; the last step's attention against a double-precision
 * softmax over the live keys (2e-2).  Exit code 0 = all checks passed. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "dflash_hip.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "HIP error %d (%s) at %s:%d\n", (int)e_, hipGetErrorString(e_), __FILE__, __LINE__); return 2; } } while (0)
#define CHECK_DF(x) do { int r_ = (x); if (r_ != DFLASH_OK) { fprintf(stderr, "dflash error %d at %s:%d: %s\n", r_, __FILE__, __LINE__, dflash_last_error()); return 3; } } while (0)

enum { T = 16, Hk = 2, Hv = 4, Dk = 128, Dv = 64, NGDN = 3,          /* GatedDelta layers */
       Hq = 4, Hkv = 2, D = 128, CONTEXT = 100, CAP = 256,           /* attention layer */
       NSTEPS = 4 };

static unsigned g_seed = 2024u;
static float rnd(void) { g_seed = g_seed * 1664525u + 1013904223u; return (float)((g_seed >> 8) & 0xffff) / 65536.0f - 0.5f; }

static uint16_t to_bf16(float x) {                   /* round to nearest even */
    uint32_t u; memcpy(&u, &x, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }

typedef struct {
    void *q, *k, *v, *g, *beta, *state[2], *y, *tape;             /* device */
} GdnLayer;
typedef struct {
    GdnLayer gdn[NGDN];
    void *aq, *k_new, *v_new, *k_cache, *v_cache, *out, *lse, *ws;
    size_t ws_bytes;
    int32_t *offset, *accept;                                      /* device int32 [1], [4] */
    uint32_t *ids[2], *post[2];                                    /* token ids of the step in flight, one slot per phase */
} Stack;

/* host copies of the activations (identical for both stacks) */
static uint16_t h_q[NGDN][T * Hk * Dk], h_k[NGDN][T * Hk * Dk], h_v[NGDN][T * Hv * Dv], h_g[NGDN][T * Hv], h_beta[NGDN][T * Hv];
static float h_state0[NGDN][Hv * Dv * Dk];
static uint16_t h_aq[Hq * T * D], h_knew[Hkv * T * D], h_vnew[Hkv * T * D], h_kc[Hkv * CAP * D], h_vc[Hkv * CAP * D];

static int upload(void** dst, const void* src, size_t bytes) {
    CHECK_HIP(hipMalloc(dst, bytes));
    if (src) CHECK_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
    else CHECK_HIP(hipMemset(*dst, 0, bytes));
    return 0;
}

static int make_stack(Stack* s) {
    for (int l = 0; l < NGDN; ++l) {
        GdnLayer* L = &s->gdn[l];
        if (upload(&L->q, h_q[l], sizeof h_q[l]) || upload(&L->k, h_k[l], sizeof h_k[l]) || upload(&L->v, h_v[l], sizeof h_v[l]) ||
            upload(&L->g, h_g[l], sizeof h_g[l]) || upload(&L->beta, h_beta[l], sizeof h_beta[l]) ||
            upload(&L->state[0], h_state0[l], sizeof h_state0[l]) || upload(&L->state[1], NULL, sizeof h_state0[l]) ||
            upload(&L->y, NULL, (size_t)T * Hv * Dv * 2) || upload(&L->tape, NULL, (size_t)T * Hv * Dv * 4)) return 2;
    }
    s->ws_bytes = dflash_sdpa_workspace_bytes(1, Hq, Hkv, T, CAP, D);
    if (!s->ws_bytes) { fprintf(stderr, "workspace query failed: %s\n", dflash_last_error()); return 3; }
    const int32_t off0 = CONTEXT;
    if (upload(&s->aq, h_aq, sizeof h_aq) || upload(&s->k_new, h_knew, sizeof h_knew) || upload(&s->v_new, h_vnew, sizeof h_vnew) ||
        upload(&s->k_cache, h_kc, sizeof h_kc) || upload(&s->v_cache, h_vc, sizeof h_vc) || upload(&s->out, NULL, sizeof h_aq) ||
        upload(&s->lse, NULL, (size_t)Hq * T * 4) || upload(&s->ws, NULL, s->ws_bytes) ||
        upload((void**)&s->offset, &off0, 4) || upload((void**)&s->accept, NULL, 16)) return 2;
    for (int p = 0; p < 2; ++p)
        if (upload((void**)&s->ids[p], NULL, T * 4) || upload((void**)&s->post[p], NULL, T * 4)) return 2;
    return 0;
}

/* One verify step, enqueued on `st` (never synchronises, never allocates): phase = which state buffer holds the
 * pre-verify state. */
static int enqueue_step(Stack* s, hipStream_t st, int phase) {
    const void *tapes[NGDN], *ks[NGDN], *gs[NGDN], *sin[NGDN];
    void* sout[NGDN];
    for (int l = 0; l < NGDN; ++l) {
        GdnLayer* L = &s->gdn[l];
        CHECK_DF(dflash_gated_delta_tape(st, L->q, L->k, L->v, L->g, 3, L->beta, DFLASH_BF16, L->state[phase], L->state[1 - phase],
                                         DFLASH_F32, L->y, (float*)L->tape, NULL, 0, 1, T, Hk, Hv, Dk, Dv));
        tapes[l] = L->tape; ks[l] = L->k; gs[l] = L->g; sin[l] = L->state[phase]; sout[l] = L->state[1 - phase];
    }
    CHECK_DF(dflash_sdpa_block_causal_append(st, s->aq, s->k_cache, s->v_cache, s->k_new, s->v_new, s->out, (float*)s->lse,
                                             DFLASH_BF16, 0.0883883f, 1, Hq, Hkv, T, CAP, D, (int64_t)Hkv * CAP * D, (int64_t)CAP * D,
                                             s->offset, s->ws, s->ws_bytes));
    CHECK_DF(dflash_accept_commit_replay_batched(st, s->ids[phase], s->post[phase], T, s->offset, s->accept, NGDN, tapes, DFLASH_F32,
                                                 ks, gs, DFLASH_BF16, 3, sin, sout, DFLASH_F32, /*skip_if_full=*/1, 1, T, Hk, Hv, Dk, Dv));
    return 0;
}

/* Token ids that make exactly `commit` tokens commit: posterior[i] == ids[i + 1] for i < commit - 1, then a mismatch. */
static void make_ids(int step, int commit, uint32_t* ids, uint32_t* post) {
    for (int i = 0; i < T; ++i) ids[i] = (uint32_t)(1000 * step + 10 + i);
    for (int i = 0; i < T - 1; ++i) post[i] = ids[i + 1];
    post[T - 1] = 7u;
    if (commit - 1 < T - 1) post[commit - 1] = ids[commit] + 1u;
}

/* The gated delta rule over the first n block tokens of layer l, in double (DFlashKernels.swift:409-466). */
static void host_forward(int l, double* S, int n) {
    for (int t = 0; t < n; ++t)
        for (int hv = 0; hv < Hv; ++hv) {
            const int hk = hv / (Hv / Hk);
            const double g = from_bf16(h_g[l][t * Hv + hv]), beta = from_bf16(h_beta[l][t * Hv + hv]);
            const uint16_t* kt = &h_k[l][(t * Hk + hk) * Dk];
            for (int dv = 0; dv < Dv; ++dv) {
                double* row = &S[((size_t)hv * Dv + dv) * Dk];
                double m = 0.0;
                for (int c = 0; c < Dk; ++c) { row[c] *= g; m += row[c] * from_bf16(kt[c]); }
                const double delta = (from_bf16(h_v[l][(t * Hv + hv) * Dv + dv]) - m) * beta;
                for (int c = 0; c < Dk; ++c) row[c] += delta * from_bf16(kt[c]);
            }
        }
}

int main(void) {
    /* ---- synthetic activations ---- */
    for (int l = 0; l < NGDN; ++l) {
        for (int i = 0; i < T * Hk * Dk; ++i) { h_q[l][i] = to_bf16(0.3f * rnd()); h_k[l][i] = to_bf16(0.3f * rnd()); }
        for (int i = 0; i < T * Hv * Dv; ++i) h_v[l][i] = to_bf16(2.0f * rnd());
        for (int i = 0; i < T * Hv; ++i) { h_g[l][i] = to_bf16(0.75f + 0.45f * rnd()); h_beta[l][i] = to_bf16(0.5f + 0.9f * rnd()); }
        for (int i = 0; i < Hv * Dv * Dk; ++i) h_state0[l][i] = 0.2f * rnd();
    }
    for (int i = 0; i < Hq * T * D; ++i) h_aq[i] = to_bf16(2.0f * rnd());
    for (int i = 0; i < Hkv * T * D; ++i) { h_knew[i] = to_bf16(2.0f * rnd()); h_vnew[i] = to_bf16(2.0f * rnd()); }
    for (int h = 0; h < Hkv; ++h)
        for (int n = 0; n < CAP; ++n)
            for (int c = 0; c < D; ++c) {
                const size_t i = ((size_t)h * CAP + n) * D + c;
                h_kc[i] = n < CONTEXT ? to_bf16(2.0f * rnd()) : 0;
                h_vc[i] = n < CONTEXT ? to_bf16(2.0f * rnd()) : 0;
            }
    const int commits[NSTEPS] = {4, 16, 1, 7};           /* partial, full (no replay), nothing accepted, partial */
    uint32_t ids[NSTEPS][T], post[NSTEPS][T];
    for (int s = 0; s < NSTEPS; ++s) make_ids(s, commits[s], ids[s], post[s]);

    CHECK_DF(dflash_init());                              /* code object and LDS limits: before any capture */
    static Stack graphed, eager;
    if (make_stack(&graphed) || make_stack(&eager)) return 2;

    /* ---- two steps captured on a fresh stream, launched twice ---- */
    hipStream_t st;
    CHECK_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
    hipGraph_t graph;
    hipGraphExec_t exec;
    CHECK_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeGlobal));
    if (enqueue_step(&graphed, st, 0) || enqueue_step(&graphed, st, 1)) return 3;
    CHECK_HIP(hipStreamEndCapture(st, &graph));
    CHECK_HIP(hipGraphInstantiate(&exec, graph, NULL, NULL, 0));
    for (int rep = 0; rep < 2; ++rep) {
        for (int p = 0; p < 2; ++p) {                     /* what the drafter and the target's argmax would leave on the device */
            CHECK_HIP(hipMemcpy(graphed.ids[p], ids[2 * rep + p], T * 4, hipMemcpyHostToDevice));
            CHECK_HIP(hipMemcpy(graphed.post[p], post[2 * rep + p], T * 4, hipMemcpyHostToDevice));
        }
        CHECK_HIP(hipGraphLaunch(exec, st));
        CHECK_HIP(hipStreamSynchronize(st));
    }
    /* ---- the same four steps, eagerly ---- */
    for (int s = 0; s < NSTEPS; ++s) {
        CHECK_HIP(hipMemcpy(eager.ids[s & 1], ids[s], T * 4, hipMemcpyHostToDevice));
        CHECK_HIP(hipMemcpy(eager.post[s & 1], post[s], T * 4, hipMemcpyHostToDevice));
        if (enqueue_step(&eager, st, s & 1)) return 3;
        CHECK_HIP(hipStreamSynchronize(st));
    }

    /* ---- integer bookkeeping: bit-exact ---- */
    int32_t off_g, off_e, acc_g[4], acc_e[4];
    CHECK_HIP(hipMemcpy(&off_g, graphed.offset, 4, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(&off_e, eager.offset, 4, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(acc_g, graphed.accept, 16, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(acc_e, eager.accept, 16, hipMemcpyDeviceToHost));
    int offs[NSTEPS + 1] = {CONTEXT};
    for (int s = 0; s < NSTEPS; ++s) offs[s + 1] = offs[s] + commits[s];
    const int last = commits[NSTEPS - 1];
    const int32_t want4[4] = {last - 1, last, (int32_t)post[NSTEPS - 1][last - 1], offs[NSTEPS]};
    printf("offset %d (graph) %d (eager), expected %d; accept words %d %d %d %d\n", off_g, off_e, offs[NSTEPS], acc_g[0], acc_g[1], acc_g[2], acc_g[3]);
    if (off_g != offs[NSTEPS] || off_e != offs[NSTEPS] || memcmp(acc_g, want4, 16) || memcmp(acc_e, want4, 16)) {
        fprintf(stderr, "offset / accept words mismatch\n"); return 1;
    }

    /* ---- recurrent states: graph == eager bytes, and both == the recurrence over the committed tokens ---- */
    const size_t ns = (size_t)Hv * Dv * Dk;
    float *sg = malloc(ns * 4), *se = malloc(ns * 4);
    double* S = malloc(ns * 8);
    const int final_phase = NSTEPS & 1;                   /* the buffer that holds the committed state after NSTEPS steps */
    double worst = 0.0;
    for (int l = 0; l < NGDN; ++l) {
        CHECK_HIP(hipMemcpy(sg, graphed.gdn[l].state[final_phase], ns * 4, hipMemcpyDeviceToHost));
        CHECK_HIP(hipMemcpy(se, eager.gdn[l].state[final_phase], ns * 4, hipMemcpyDeviceToHost));
        if (memcmp(sg, se, ns * 4)) { fprintf(stderr, "layer %d: graph replay and eager stepping left different states\n", l); return 1; }
        for (size_t i = 0; i < ns; ++i) S[i] = h_state0[l][i];
        for (int s = 0; s < NSTEPS; ++s) host_forward(l, S, commits[s]);
        double scale = 0.0, err = 0.0;
        for (size_t i = 0; i < ns; ++i) { if (fabs(S[i]) > scale) scale = fabs(S[i]); if (fabs(sg[i] - S[i]) > err) err = fabs(sg[i] - S[i]); }
        if (err / (1e-4 * scale) > worst) worst = err / (1e-4 * scale);
    }
    printf("recurrent states after %d steps: graph == eager; worst error is %.3g of the tolerance\n", NSTEPS, worst);
    if (!(worst <= 1.0)) { fprintf(stderr, "state mismatch\n"); return 1; }

    /* ---- KV cache: every step stored its block at its offset; a later step overwrote what lies beyond ITS offset ---- */
    static uint16_t kc[Hkv * CAP * D], vc[Hkv * CAP * D], kc_e[Hkv * CAP * D];
    CHECK_HIP(hipMemcpy(kc, graphed.k_cache, sizeof kc, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(vc, graphed.v_cache, sizeof vc, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(kc_e, eager.k_cache, sizeof kc_e, hipMemcpyDeviceToHost));
    if (memcmp(kc, kc_e, sizeof kc)) { fprintf(stderr, "graph replay and eager stepping left different K caches\n"); return 1; }
    for (int s = 0; s < NSTEPS; ++s) {
        const int rows = s == NSTEPS - 1 ? T : commits[s];
        for (int h = 0; h < Hkv; ++h)
            if (memcmp(&kc[((size_t)h * CAP + offs[s]) * D], &h_knew[(size_t)h * T * D], (size_t)rows * D * 2) ||
                memcmp(&vc[((size_t)h * CAP + offs[s]) * D], &h_vnew[(size_t)h * T * D], (size_t)rows * D * 2)) {
                fprintf(stderr, "step %d: appended rows differ\n", s); return 1;
            }
    }
    for (int h = 0; h < Hkv; ++h)
        if (memcmp(&kc[(size_t)h * CAP * D], &h_kc[(size_t)h * CAP * D], (size_t)CONTEXT * D * 2)) { fprintf(stderr, "context rows changed\n"); return 1; }

    /* ---- attention of the last step over offs[NSTEPS-1] + 16 keys, against a double-precision softmax on the cache as read back ---- */
    static uint16_t og[Hq * T * D], oe[Hq * T * D];
    CHECK_HIP(hipMemcpy(og, graphed.out, sizeof og, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(oe, eager.out, sizeof oe, hipMemcpyDeviceToHost));
    if (memcmp(og, oe, sizeof og)) { fprintf(stderr, "graph replay and eager stepping left different attention outputs\n"); return 1; }
    const int N = offs[NSTEPS - 1] + T;
    double worst_o = 0.0, sc[CAP];
    for (int h = 0; h < Hq; ++h) {
        const int hk = h / (Hq / Hkv);
        for (int i = 0; i < T; ++i) {
            const int vis = N - T + i;
            double mx = -1e300, sum = 0.0;
            for (int n = 0; n <= vis; ++n) {
                double d = 0.0;
                for (int c = 0; c < D; ++c) d += (double)from_bf16(h_aq[((size_t)h * T + i) * D + c]) * from_bf16(kc[((size_t)hk * CAP + n) * D + c]);
                sc[n] = d * 0.0883883;
                if (sc[n] > mx) mx = sc[n];
            }
            for (int n = 0; n <= vis; ++n) { sc[n] = exp(sc[n] - mx); sum += sc[n]; }
            for (int c = 0; c < D; ++c) {
                double o = 0.0;
                for (int n = 0; n <= vis; ++n) o += sc[n] * from_bf16(vc[((size_t)hk * CAP + n) * D + c]);
                o /= sum;
                const double excess = fabs(from_bf16(og[((size_t)h * T + i) * D + c]) - o) / (2e-2 * fabs(o) + 2e-2);
                if (excess > worst_o) worst_o = excess;
            }
        }
    }
    printf("attention of the last step over %d keys: worst error is %.3g of the tolerance\n", N, worst_o);
    if (!(worst_o <= 1.0)) { fprintf(stderr, "attention mismatch\n"); return 1; }

    CHECK_HIP(hipGraphExecDestroy(exec));
    CHECK_HIP(hipGraphDestroy(graph));
    CHECK_HIP(hipStreamDestroy(st));
    printf("verify-step check passed: %d steps through a captured graph and eagerly, C ABI only\n", NSTEPS);
    return 0;
}
