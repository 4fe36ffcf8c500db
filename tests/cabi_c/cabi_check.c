/* Plain C client of libdflash_hip.so: no Python, no torch, only the C ABI and the HIP runtime's C API.
 * Replays a small innovation tape (S <- S*g_t + delta_t (x) k_t, Sources/DFlash/DFlashKernels.swift:371-407)
 * and runs the acceptance bookkeeping (DFlashRuntime.swift:133-142, :525-547), checking both against
 * values computed here on the host.  Exit code 0 = all checks passed. */
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

    /* an unsupported shape is reported, not crashed on */
    if (dflash_tape_replay(NULL, d_tape, DFLASH_F32, d_k, d_g, DFLASH_F32, 3, d_state, d_out, DFLASH_F32, NULL, 0,
                           B, NSTEPS, Hk, Hv, 48, Dv) != DFLASH_UNSUPPORTED) { fprintf(stderr, "Dk=48 should be unsupported\n"); return 1; }
    printf("C ABI check passed\n");
    return 0;
}
