/* Plain C client of libdflash_hip.so: no Python, no torch, only the C ABI and the HIP runtime's C API.
 * Replays a small innovation tape (S <- S*g_t + delta_t (x) k_t, Sources/DFlash/DFlashKernels.swift:371-407),
 * runs the acceptance bookkeeping (DFlashRuntime.swift:133-142, :525-547) and the block-causal attention over a
 * dense and a paged cache, checking all against values computed here on the host.  Exit code 0 = all checks passed. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "dflash_hip.h"

#define CHECK_HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "HIP error %d at %s:%d\n", (int)e_, __FILE__, __LINE__); return 2; } } while (0)
#define CHECK_DF(x) do { int r_ = (x); if (r_ != DFLASH_OK) { fprintf(stderr, "dflash error %d at %s:%d: %s\n", r_, __FILE__, __LINE__, dflash_last_error()); return 3; } } while (0)

int main(void) {
    enum { B = 1, T = 6, Hk = 2, Hv = 4, Dk = 64, Dv = 32, NSTEPS = 4 };
    const size_t n_state = (size_t)B * Hv * Dv * Dk, n_tape = (size_t)B * T * Hv * Dv, n_k = (size_t)B * T * Hk * Dk,
                 n_g = (size_t)B * T * Hv;
    float *state = malloc(n_state * 4), *want = malloc(n_state * 4), *got = malloc(n_state * 4);
    float *tape = malloc(n_tape * 4), *k = malloc(n_k * 4), *g = malloc(n_g * 4);
    unsigned seed = 12345u;
    #define RND() ((seed = seed * 1664525u + 1013904223u), (float)((seed >> 8) & 0xffff) / 65536.0f - 0.5f)
    for (size_t i = 0; i < n_state; ++i) state[i] = RND();
    for (size_t i = 0; i < n_tape; ++i) tape[i] = RND();
    for (size_t i = 0; i < n_k; ++i) k[i] = RND() * 0.25f;
    for (size_t i = 0; i < n_g; ++i) g[i] = 0.75f + 0.5f * RND();

    /* host: the recurrence as written */
    memcpy(want, state, n_state * 4);
    for (int t = 0; t < NSTEPS; ++t)
        for (int hv = 0; hv < Hv; ++hv) {
            const int hk = hv / (Hv / Hk);
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk) {
                    float* s = &want[((size_t)hv * Dv + dv) * Dk + dk];
                    *s = *s * g[(size_t)t * Hv + hv] + tape[((size_t)t * Hv + hv) * Dv + dv] * k[((size_t)t * Hk + hk) * Dk + dk];
                }
        }

    CHECK_DF(dflash_init());
    void *d_state, *d_out, *d_tape, *d_k, *d_g;
    CHECK_HIP(hipMalloc(&d_state, n_state * 4)); CHECK_HIP(hipMalloc(&d_out, n_state * 4));
    CHECK_HIP(hipMalloc(&d_tape, n_tape * 4)); CHECK_HIP(hipMalloc(&d_k, n_k * 4)); CHECK_HIP(hipMalloc(&d_g, n_g * 4));
    CHECK_HIP(hipMemcpy(d_state, state, n_state * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_tape, tape, n_tape * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_k, k, n_k * 4, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_g, g, n_g * 4, hipMemcpyHostToDevice));
    /* replay the first NSTEPS of the T recorded steps: tape / k / g are passed with T = NSTEPS rows used */
    CHECK_DF(dflash_tape_replay(NULL, d_tape, DFLASH_F32, d_k, d_g, DFLASH_F32, 3, d_state, d_out, DFLASH_F32, NULL, 0,
                                B, NSTEPS, Hk, Hv, Dk, Dv));
    CHECK_HIP(hipDeviceSynchronize());
    CHECK_HIP(hipMemcpy(got, d_out, n_state * 4, hipMemcpyDeviceToHost));
    /* the bar of the parity tests: |got - want| <= 1e-4 |want| + 1e-6 */
    double worst = 0.0;
    for (size_t i = 0; i < n_state; ++i) {
        const double excess = fabs((double)got[i] - want[i]) / (1e-4 * fabs((double)want[i]) + 1e-6);
        if (excess > worst) worst = excess;
    }
    printf("tape replay: worst error is %.3g of the tolerance\n", worst);
    if (!(worst <= 1.0)) { fprintf(stderr, "tape replay mismatch\n"); return 1; }

    /* acceptance: verify = [7, 1, 2, 3, 4], posterior = [1, 2, 9, 4, 5] -> 2 drafted tokens accepted */
    const uint32_t verify[5] = {7, 1, 2, 3, 4}, post[5] = {1, 2, 9, 4, 5};
    int32_t start = 100, out4[4];
    void *d_v, *d_p, *d_s, *d_o;
    CHECK_HIP(hipMalloc(&d_v, sizeof verify)); CHECK_HIP(hipMalloc(&d_p, sizeof post));
    CHECK_HIP(hipMalloc(&d_s, 4)); CHECK_HIP(hipMalloc(&d_o, 16));
    CHECK_HIP(hipMemcpy(d_v, verify, sizeof verify, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_p, post, sizeof post, hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(d_s, &start, 4, hipMemcpyHostToDevice));
    CHECK_DF(dflash_accept_commit(NULL, (const uint32_t*)d_v, (const uint32_t*)d_p, 5, (int32_t*)d_s, (int32_t*)d_o));
    CHECK_HIP(hipMemcpy(out4, d_o, 16, hipMemcpyDeviceToHost));
    printf("accept: acceptance %d commit %d staged_next %d start %d\n", out4[0], out4[1], out4[2], out4[3]);
    if (out4[0] != 2 || out4[1] != 3 || out4[2] != 9 || out4[3] != 103) { fprintf(stderr, "accept mismatch\n"); return 1; }

    /* block-causal attention (DFlashKernels.swift:737-743: row i of the 16-row block sees keys 0 .. N-16+i), once over a
     * dense cache and once over the same keys in 32-key pages: identical bytes, and close to a double-precision softmax */
    {
        enum { Hq = 2, Hkv = 1, D = 128, N = 56, P = 32, PAGES = 3 };
        const size_t nq = (size_t)Hq * 16 * D, nkv = (size_t)Hkv * N * D, npool = (size_t)PAGES * Hkv * P * D;
        uint16_t *qh = malloc(nq * 2), *kh = malloc(nkv * 2), *vh = malloc(nkv * 2), *kp = calloc(npool, 2), *vp = calloc(npool, 2);
        uint16_t *o1 = malloc(nq * 2), *o2 = malloc(nq * 2);
        for (size_t i = 0; i < nq; ++i) { float x = 2.0f * RND(); uint32_t u; memcpy(&u, &x, 4); qh[i] = (uint16_t)(u >> 16); }
        for (size_t i = 0; i < nkv; ++i) { float x = 2.0f * RND(); uint32_t u; memcpy(&u, &x, 4); kh[i] = (uint16_t)(u >> 16); }
        for (size_t i = 0; i < nkv; ++i) { float x = 2.0f * RND(); uint32_t u; memcpy(&u, &x, 4); vh[i] = (uint16_t)(u >> 16); }
        const int32_t table[2] = {2, 0};                  /* keys 0..31 in page 2, keys 32..55 in page 0 */
        for (int n = 0; n < N; ++n) {
            memcpy(kp + ((size_t)table[n / P] * P + n % P) * D, kh + (size_t)n * D, D * 2);
            memcpy(vp + ((size_t)table[n / P] * P + n % P) * D, vh + (size_t)n * D, D * 2);
        }
        void *dq, *dk, *dv, *dkp, *dvp, *dt, *do1, *do2, *dws;
        const size_t ws = dflash_sdpa_workspace_bytes(1, Hq, Hkv, 16, N, D);
        if (ws == 0) { fprintf(stderr, "sdpa workspace query failed: %s\n", dflash_last_error()); return 1; }
        CHECK_HIP(hipMalloc(&dq, nq * 2)); CHECK_HIP(hipMalloc(&dk, nkv * 2)); CHECK_HIP(hipMalloc(&dv, nkv * 2));
        CHECK_HIP(hipMalloc(&dkp, npool * 2)); CHECK_HIP(hipMalloc(&dvp, npool * 2)); CHECK_HIP(hipMalloc(&dt, sizeof table));
        CHECK_HIP(hipMalloc(&do1, nq * 2)); CHECK_HIP(hipMalloc(&do2, nq * 2)); CHECK_HIP(hipMalloc(&dws, ws));
        CHECK_HIP(hipMemcpy(dq, qh, nq * 2, hipMemcpyHostToDevice)); CHECK_HIP(hipMemcpy(dk, kh, nkv * 2, hipMemcpyHostToDevice));
        CHECK_HIP(hipMemcpy(dv, vh, nkv * 2, hipMemcpyHostToDevice)); CHECK_HIP(hipMemcpy(dkp, kp, npool * 2, hipMemcpyHostToDevice));
        CHECK_HIP(hipMemcpy(dvp, vp, npool * 2, hipMemcpyHostToDevice)); CHECK_HIP(hipMemcpy(dt, table, sizeof table, hipMemcpyHostToDevice));
        const float scale = 0.0883883f;                   /* 1 / sqrt(128) */
        CHECK_DF(dflash_sdpa_block_causal(NULL, dq, dk, dv, do1, NULL, DFLASH_BF16, scale, 1, Hq, Hkv, 16, N, D,
                                          (int64_t)Hkv * N * D, (int64_t)N * D, NULL, dws, ws));
        CHECK_DF(dflash_sdpa_block_causal_paged(NULL, dq, dkp, dvp, (const int32_t*)dt, 2, P, PAGES, (int64_t)Hkv * P * D, (int64_t)P * D,
                                                NULL, NULL, do2, NULL, DFLASH_BF16, scale, 1, Hq, Hkv, 16, N, D, NULL, dws, ws));
        CHECK_HIP(hipDeviceSynchronize());
        CHECK_HIP(hipMemcpy(o1, do1, nq * 2, hipMemcpyDeviceToHost)); CHECK_HIP(hipMemcpy(o2, do2, nq * 2, hipMemcpyDeviceToHost));
        if (memcmp(o1, o2, nq * 2) != 0) { fprintf(stderr, "paged attention differs from dense\n"); return 1; }
        double worst_o = 0.0;
        for (int h = 0; h < Hq; ++h)
            for (int i = 0; i < 16; ++i) {
                double sc[N], mx = -1e300, sum = 0.0;
                const int vis = N - 16 + i;               /* last visible key */
                for (int n = 0; n <= vis; ++n) {
                    double d = 0.0;
                    for (int c = 0; c < D; ++c) {
                        uint32_t a = (uint32_t)qh[((size_t)h * 16 + i) * D + c] << 16, b = (uint32_t)kh[(size_t)n * D + c] << 16;
                        float fa, fb; memcpy(&fa, &a, 4); memcpy(&fb, &b, 4);
                        d += (double)fa * fb;
                    }
                    sc[n] = d * scale;
                    if (sc[n] > mx) mx = sc[n];
                }
                for (int n = 0; n <= vis; ++n) { sc[n] = exp(sc[n] - mx); sum += sc[n]; }
                for (int c = 0; c < D; ++c) {
                    double o = 0.0;
                    for (int n = 0; n <= vis; ++n) { uint32_t b = (uint32_t)vh[(size_t)n * D + c] << 16; float fb; memcpy(&fb, &b, 4); o += sc[n] * fb; }
                    o /= sum;
                    uint32_t g16 = (uint32_t)o1[((size_t)h * 16 + i) * D + c] << 16; float fg; memcpy(&fg, &g16, 4);
                    const double excess = fabs(fg - o) / (2e-2 * fabs(o) + 2e-2);
                    if (excess > worst_o) worst_o = excess;
                }
            }
        printf("attention: paged == dense; worst error is %.3g of the tolerance\n", worst_o);
        if (!(worst_o <= 1.0)) { fprintf(stderr, "attention mismatch\n"); return 1; }
    }

    /* an unsupported shape is reported, not crashed on */
    if (dflash_tape_replay(NULL, d_tape, DFLASH_F32, d_k, d_g, DFLASH_F32, 3, d_state, d_out, DFLASH_F32, NULL, 0,
                           B, NSTEPS, Hk, Hv, 48, Dv) != DFLASH_UNSUPPORTED) { fprintf(stderr, "Dk=48 should be unsupported\n"); return 1; }
    printf("C ABI check passed\n");
    return 0;
}
