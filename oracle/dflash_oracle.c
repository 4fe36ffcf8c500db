/*
 * CPU restatement of the DFlash verify hot path in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker and the timed CPU
 * baseline.  The shipped library never links or loads it.
 *
 * It restates the reference's *ops* implementations, which are what SwiftLM
 * executes on a CPU device (Sources/DFlash/DFlashKernels.swift:259-261,
 * :325-327):
 *   - tapeReplayOps            DFlashKernels.swift:371-407
 *   - gatedDeltaOpsWithTape    DFlashKernels.swift:409-466
 *   - sdpaFallback             DFlashKernels.swift:818-828 (softmax(QK^T)V with
 *                              the block-causal rule of :614)
 * Two flavours of each recurrence are provided: "opbyop" materialises one
 * full-state temporary per array operation per step, the way the ops graph is
 * evaluated (:388-405, :433-459); "fused" makes a single pass per step.
 * All arithmetic is float32; inputs arrive as float32 (already rounded to the
 * storage type by the caller).  Layouts: q,k [B,T,Hk,Dk]; v,tape,y [B,T,Hv,Dv];
 * g [B,T,Hv] (g_ndim 3) or [B,T,Hv,Dk] (g_ndim 4); beta [B,T,Hv];
 * state [B,Hv,Dv,Dk]; mask [B,T] (NULL = none).
 *
 * The underlying array library of the reference (MLX) is absent from the
 * reference tree and unpinned, so reduction order is not reproduced bit for
 * bit: "parity unpinned" at the bit level, checked against the numpy oracle and
 * the mathematical identities in tests/.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ---------------------------------------------------------------- replay -- */

/* DFlashKernels.swift:398: state = state * decay + delta * kT, fused per step. */
void oracle_tape_replay_fused(const float* tape, const float* k, const float* g, int g_ndim,
                              const float* state_in, float* state_out, const float* mask,
                              int B, int T, int Hk, int Hv, int Dk, int Dv) {
    const int rf = Hv / Hk;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b) {
        for (int hv = 0; hv < Hv; ++hv) {
            const int hk = hv / rf; /* consecutive repeat, :384 */
            const float* s_in = state_in + ((size_t)(b * Hv + hv)) * Dv * Dk;
            float* s = state_out + ((size_t)(b * Hv + hv)) * Dv * Dk;
            memcpy(s, s_in, sizeof(float) * (size_t)Dv * Dk);
            for (int t = 0; t < T; ++t) {
                if (mask && !(mask[b * T + t] > 0.5f)) continue; /* :399-403 */
                const float* kt = k + ((size_t)(b * T + t) * Hk + hk) * Dk;
                const float* dt = tape + ((size_t)(b * T + t) * Hv + hv) * Dv;
                const float* gt = g_ndim == 4 ? g + ((size_t)(b * T + t) * Hv + hv) * Dk
                                              : g + (size_t)(b * T + t) * Hv + hv;
                for (int dv = 0; dv < Dv; ++dv) {
                    float* row = s + (size_t)dv * Dk;
                    const float delta = dt[dv];
                    if (g_ndim == 4) {
                        for (int dk = 0; dk < Dk; ++dk) row[dk] = row[dk] * gt[dk] + delta * kt[dk];
                    } else {
                        const float decay = gt[0];
                        for (int dk = 0; dk < Dk; ++dk) row[dk] = row[dk] * decay + delta * kt[dk];
                    }
                }
            }
        }
    }
}

/* Same result, evaluated as the ops graph does: every array op of
 * DFlashKernels.swift:398-403 writes a whole [B,Hv,Dv,Dk] temporary. */
void oracle_tape_replay_opbyop(const float* tape, const float* k, const float* g, int g_ndim,
                               const float* state_in, float* state_out, const float* mask,
                               int B, int T, int Hk, int Hv, int Dk, int Dv) {
    const int rf = Hv / Hk;
    const size_t n = (size_t)B * Hv * Dv * Dk;
    float* t1 = (float*)malloc(n * sizeof(float)); /* state * decay   */
    float* t2 = (float*)malloc(n * sizeof(float)); /* delta * kT      */
    float* t3 = (float*)malloc(n * sizeof(float)); /* t1 + t2         */
    float* cur = (float*)malloc(n * sizeof(float));
    memcpy(cur, state_in, n * sizeof(float));
    for (int t = 0; t < T; ++t) {
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) {
            const int b = bh / Hv, hv = bh % Hv;
            const float* gt = g_ndim == 4 ? g + ((size_t)(b * T + t) * Hv + hv) * Dk
                                          : g + (size_t)(b * T + t) * Hv + hv;
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk) {
                    size_t i = ((size_t)bh * Dv + dv) * Dk + dk;
                    t1[i] = cur[i] * (g_ndim == 4 ? gt[dk] : gt[0]);
                }
        }
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) {
            const int b = bh / Hv, hv = bh % Hv, hk = hv / rf;
            const float* kt = k + ((size_t)(b * T + t) * Hk + hk) * Dk;
            const float* dt = tape + ((size_t)(b * T + t) * Hv + hv) * Dv;
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk)
                    t2[((size_t)bh * Dv + dv) * Dk + dk] = dt[dv] * kt[dk];
        }
#pragma omp parallel for schedule(static)
        for (size_t i = 0; i < n; ++i) t3[i] = t1[i] + t2[i];
        if (mask) {
            /* MLX.where(stepMask, state, prev), :402-403 */
#pragma omp parallel for schedule(static)
            for (int bh = 0; bh < B * Hv; ++bh) {
                const int b = bh / Hv;
                const int on = mask[b * T + t] > 0.5f;
                const size_t base = (size_t)bh * Dv * Dk;
                for (size_t i = 0; i < (size_t)Dv * Dk; ++i)
                    cur[base + i] = on ? t3[base + i] : cur[base + i];
            }
        } else {
            float* sw = cur; cur = t3; t3 = sw;
        }
    }
    memcpy(state_out, cur, n * sizeof(float));
    free(t1); free(t2); free(t3); free(cur);
}

/* ----------------------------------------------------------- gated delta -- */

/* DFlashKernels.swift:433-459, one fused pass per step. */
void oracle_gated_delta_fused(const float* q, const float* k, const float* v, const float* g,
                              int g_ndim, const float* beta, const float* state_in, float* y,
                              float* state_out, float* tape, const float* mask,
                              int B, int T, int Hk, int Hv, int Dk, int Dv) {
    const int rf = Hv / Hk;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; ++b) {
        for (int hv = 0; hv < Hv; ++hv) {
            const int hk = hv / rf;
            float* s = state_out + ((size_t)(b * Hv + hv)) * Dv * Dk;
            memcpy(s, state_in + ((size_t)(b * Hv + hv)) * Dv * Dk, sizeof(float) * (size_t)Dv * Dk);
            for (int t = 0; t < T; ++t) {
                const size_t tv = ((size_t)(b * T + t) * Hv + hv) * Dv;
                if (mask && !(mask[b * T + t] > 0.5f)) { /* :446-453 */
                    for (int dv = 0; dv < Dv; ++dv) { y[tv + dv] = 0.f; tape[tv + dv] = 0.f; }
                    continue;
                }
                const float* qt = q + ((size_t)(b * T + t) * Hk + hk) * Dk;
                const float* kt = k + ((size_t)(b * T + t) * Hk + hk) * Dk;
                const float* gt = g_ndim == 4 ? g + ((size_t)(b * T + t) * Hv + hv) * Dk
                                              : g + (size_t)(b * T + t) * Hv + hv;
                const float bt = beta[(size_t)(b * T + t) * Hv + hv];
                for (int dv = 0; dv < Dv; ++dv) {
                    float* row = s + (size_t)dv * Dk;
                    float kv_mem = 0.f;
                    for (int dk = 0; dk < Dk; ++dk) {
                        row[dk] *= (g_ndim == 4 ? gt[dk] : gt[0]);     /* :440 */
                        kv_mem += row[dk] * kt[dk];                    /* :441 */
                    }
                    const float delta = (v[tv + dv] - kv_mem) * bt;    /* :442 */
                    float out = 0.f;
                    for (int dk = 0; dk < Dk; ++dk) {
                        row[dk] += kt[dk] * delta;                     /* :443 */
                        out += row[dk] * qt[dk];                       /* :444 */
                    }
                    y[tv + dv] = out;
                    tape[tv + dv] = delta;
                }
            }
        }
    }
}

/* The same step list with one full-state temporary per array op (:440-444). */
void oracle_gated_delta_opbyop(const float* q, const float* k, const float* v, const float* g,
                               int g_ndim, const float* beta, const float* state_in, float* y,
                               float* state_out, float* tape, const float* mask,
                               int B, int T, int Hk, int Hv, int Dk, int Dv) {
    const int rf = Hv / Hk;
    const size_t n = (size_t)B * Hv * Dv * Dk;
    float* cur = (float*)malloc(n * sizeof(float));
    float* dec = (float*)malloc(n * sizeof(float)); /* decayedState      */
    float* tmp = (float*)malloc(n * sizeof(float)); /* product temporaries */
    float* nxt = (float*)malloc(n * sizeof(float)); /* newState          */
    float* kvm = (float*)malloc((size_t)B * Hv * Dv * sizeof(float));
    float* dlt = (float*)malloc((size_t)B * Hv * Dv * sizeof(float));
    memcpy(cur, state_in, n * sizeof(float));
    for (int t = 0; t < T; ++t) {
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) { /* decayedState = state * decay */
            const int b = bh / Hv, hv = bh % Hv;
            const float* gt = g_ndim == 4 ? g + ((size_t)(b * T + t) * Hv + hv) * Dk
                                          : g + (size_t)(b * T + t) * Hv + hv;
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk) {
                    size_t i = ((size_t)bh * Dv + dv) * Dk + dk;
                    dec[i] = cur[i] * (g_ndim == 4 ? gt[dk] : gt[0]);
                }
        }
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) { /* decayedState * k */
            const int b = bh / Hv, hv = bh % Hv, hk = hv / rf;
            const float* kt = k + ((size_t)(b * T + t) * Hk + hk) * Dk;
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk) {
                    size_t i = ((size_t)bh * Dv + dv) * Dk + dk;
                    tmp[i] = dec[i] * kt[dk];
                }
        }
#pragma omp parallel for schedule(static)
        for (int r = 0; r < B * Hv * Dv; ++r) { /* .sum(axis: -1) */
            float acc = 0.f;
            for (int dk = 0; dk < Dk; ++dk) acc += tmp[(size_t)r * Dk + dk];
            kvm[r] = acc;
        }
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) { /* delta = (v - kvMem) * beta */
            const int b = bh / Hv, hv = bh % Hv;
            const size_t tv = ((size_t)(b * T + t) * Hv + hv) * Dv;
            const float bt = beta[(size_t)(b * T + t) * Hv + hv];
            for (int dv = 0; dv < Dv; ++dv) dlt[(size_t)bh * Dv + dv] = (v[tv + dv] - kvm[(size_t)bh * Dv + dv]) * bt;
        }
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) { /* k * delta */
            const int b = bh / Hv, hv = bh % Hv, hk = hv / rf;
            const float* kt = k + ((size_t)(b * T + t) * Hk + hk) * Dk;
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk)
                    tmp[((size_t)bh * Dv + dv) * Dk + dk] = kt[dk] * dlt[(size_t)bh * Dv + dv];
        }
#pragma omp parallel for schedule(static)
        for (size_t i = 0; i < n; ++i) nxt[i] = dec[i] + tmp[i]; /* newState */
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) { /* newState * q */
            const int b = bh / Hv, hv = bh % Hv, hk = hv / rf;
            const float* qt = q + ((size_t)(b * T + t) * Hk + hk) * Dk;
            for (int dv = 0; dv < Dv; ++dv)
                for (int dk = 0; dk < Dk; ++dk) {
                    size_t i = ((size_t)bh * Dv + dv) * Dk + dk;
                    tmp[i] = nxt[i] * qt[dk];
                }
        }
#pragma omp parallel for schedule(static)
        for (int bh = 0; bh < B * Hv; ++bh) { /* y = .sum(axis: -1), gating, stores */
            const int b = bh / Hv, hv = bh % Hv;
            const size_t tv = ((size_t)(b * T + t) * Hv + hv) * Dv;
            const int on = mask ? (mask[b * T + t] > 0.5f) : 1;
            for (int dv = 0; dv < Dv; ++dv) {
                float acc = 0.f;
                const size_t r = (size_t)bh * Dv + dv;
                for (int dk = 0; dk < Dk; ++dk) acc += tmp[r * Dk + dk];
                y[tv + dv] = on ? acc : 0.f;
                tape[tv + dv] = on ? dlt[r] : 0.f;
            }
            const size_t base = (size_t)bh * Dv * Dk;
            if (on) memcpy(cur + base, nxt + base, sizeof(float) * (size_t)Dv * Dk);
        }
    }
    memcpy(state_out, cur, n * sizeof(float));
    free(cur); free(dec); free(tmp); free(nxt); free(kvm); free(dlt);
}

/* ------------------------------------------------------------------ sdpa -- */

/* softmax(scale * Q K^T + block-causal) V in float32 with a float32 logsumexp.
 * q [B,Hq,M,D]; k,v [B,Hk,N,D]; out [B,Hq,M,D]; lse [B,Hq,M] (may be NULL).
 * Row i sees keys 0 .. N-M+i (DFlashKernels.swift:614); hk = hq / (Hq/Hk) (:575);
 * scale folded into Q (:594). */
void oracle_sdpa_block_causal(const float* q, const float* k, const float* v, float scale,
                              float* out, float* lse, int B, int Hq, int Hk, int M, int N, int D) {
    const int rf = Hq / Hk;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int bh = 0; bh < B * Hq; ++bh) {
        for (int i = 0; i < M; ++i) {
            const int b = bh / Hq, h = bh % Hq, hk = h / rf;
            const float* qi = q + ((size_t)bh * M + i) * D;
            const float* kb = k + ((size_t)(b * Hk + hk)) * N * D;
            const float* vb = v + ((size_t)(b * Hk + hk)) * N * D;
            float* o = out + ((size_t)bh * M + i) * D;
            const int last = N - M + i;
            float* s = (float*)malloc(sizeof(float) * (size_t)(last + 1));
            float* qs = (float*)malloc(sizeof(float) * (size_t)D);
            for (int d = 0; d < D; ++d) qs[d] = scale * qi[d];
            float mx = -INFINITY;
            for (int n = 0; n <= last; ++n) {
                const float* kn = kb + (size_t)n * D;
                float acc = 0.f;
                for (int d = 0; d < D; ++d) acc += qs[d] * kn[d];
                s[n] = acc;
                if (acc > mx) mx = acc;
            }
            float sum = 0.f;
            for (int d = 0; d < D; ++d) o[d] = 0.f;
            for (int n = 0; n <= last; ++n) {
                const float p = expf(s[n] - mx);
                sum += p;
                const float* vn = vb + (size_t)n * D;
                for (int d = 0; d < D; ++d) o[d] += p * vn[d];
            }
            const float inv = 1.f / sum;
            for (int d = 0; d < D; ++d) o[d] *= inv;
            if (lse) lse[(size_t)bh * M + i] = mx + logf(sum);
            free(s); free(qs);
        }
    }
}

/* ---------------------------------------------------------------- accept -- */

/* sum(cumprod(drafted == posterior)), DFlashRuntime.swift:133-142. */
int oracle_match_acceptance_length(const uint32_t* drafted, const uint32_t* posterior, int n) {
    int acc = 0;
    for (int i = 0; i < n; ++i) {
        if (drafted[i] != posterior[i]) break;
        ++acc;
    }
    return acc;
}
