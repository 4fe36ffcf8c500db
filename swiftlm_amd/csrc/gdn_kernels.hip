// GatedDelta recurrent-state kernels for gfx950: tape replay and the forward
// pass that records the innovation tape.
//
// Both recurrences are independent per state row (b, hv, dv): a row of Dk
// floats is updated by rank-1 terms that only need k_t (shared by the head),
// the row's own delta_t and the head's decay.  The kernels therefore tile a
// head over Dv across workgroups (one head alone would occupy 32 of 256 CUs),
// keep each row slice in VGPRs for all T steps, and stage the per-step
// operands (k, q, v/tape slice, g, beta, mask) through LDS once per chunk of
// steps so the serial t-loop never waits on global memory.
//
// Semantics follow Sources/DFlash/DFlashKernels.swift: Metal kernels :43-81 and
// :122-199, ops restatements :371-407 and :409-466.

#include "dflash_common.h"

namespace dflash {

constexpr int kThreads = 256;

// 4 consecutive elements of run-time type -> float4
__device__ __forceinline__ float4 load4_rt(const void* base, int dtype, size_t idx) {
    switch (dtype) {
        case DFLASH_F32: return load4(reinterpret_cast<const float*>(base) + idx);
        case DFLASH_BF16: return load4(reinterpret_cast<const bf16_t*>(base) + idx);
        default: return load4(reinterpret_cast<const f16_t*>(base) + idx);
    }
}
__device__ __forceinline__ float load1_rt(const void* base, int dtype, size_t idx) {
    switch (dtype) {
        case DFLASH_F32: return reinterpret_cast<const float*>(base)[idx];
        case DFLASH_BF16: return to_float(reinterpret_cast<const bf16_t*>(base)[idx]);
        default: return to_float(reinterpret_cast<const f16_t*>(base)[idx]);
    }
}
__device__ __forceinline__ void store1_rt(void* base, int dtype, size_t idx, float v) {
    switch (dtype) {
        case DFLASH_F32: reinterpret_cast<float*>(base)[idx] = v; break;
        case DFLASH_BF16: reinterpret_cast<bf16_t*>(base)[idx] = from_float<bf16_t>(v); break;
        default: reinterpret_cast<f16_t*>(base)[idx] = from_float<f16_t>(v); break;
    }
}

// The same store and its load at agent scope: written through to, and read from, the level of the memory system
// that every workgroup of the launch shares (each XCD has an L2 of its own).  Data handed from one workgroup to
// another inside a launch goes this way; a release fence would instead write back the whole L2.
__device__ __forceinline__ void store1_rt_agent(void* base, int dtype, size_t idx, float v) {
    switch (dtype) {
        case DFLASH_F32: __hip_atomic_store(reinterpret_cast<float*>(base) + idx, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break;
        case DFLASH_BF16:
            __hip_atomic_store(reinterpret_cast<uint16_t*>(base) + idx, f32_to_bf16_bits(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
        default:
            __hip_atomic_store(reinterpret_cast<uint16_t*>(base) + idx, __builtin_bit_cast(uint16_t, (_Float16)v), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
            break;
    }
}
__device__ __forceinline__ float load_agent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const bf16_t* p) {
    return to_float(bf16_t{__hip_atomic_load(reinterpret_cast<const uint16_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)});
}
__device__ __forceinline__ float load_agent(const f16_t* p) {
    return (float)__builtin_bit_cast(_Float16, __hip_atomic_load(reinterpret_cast<const uint16_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

__device__ __forceinline__ float requant_rt(int dtype, float v) {      // v after a round trip through the type
    switch (dtype) {
        case DFLASH_F32: return v;
        case DFLASH_BF16: return requant<bf16_t>(v);
        default: return requant<f16_t>(v);
    }
}

// ===========================================================================
// Tape replay
// ===========================================================================

struct ReplayBatch {
    const void* tape[DFLASH_MAX_BATCHED_LAYERS];
    const void* k[DFLASH_MAX_BATCHED_LAYERS];
    const void* g[DFLASH_MAX_BATCHED_LAYERS];
    const void* state_in[DFLASH_MAX_BATCHED_LAYERS];
    void* state_out[DFLASH_MAX_BATCHED_LAYERS];
};

struct ReplayArgs {
    const void* mask;        // [B,T_tape] or null
    const int32_t* steps_dev;
    // fused acceptance (null verify_ids = off): steps = 1 + leading matches of verify_ids[1:] vs posterior
    const uint32_t* verify_ids;
    const uint32_t* posterior;
    int32_t* start_inout;
    int32_t* out4;
    int V;
    int mask_dtype, tape_dtype, in_dtype;
    int steps, skip_if_full;
    int T_tape, Hk, Hv, Dv;
};

constexpr int kReplayChunk = 16;  // steps staged in LDS at a time (8 for Dk = 256): one chunk covers the 16-token verify block

// One thread owns 4 consecutive key channels of NR state rows.  DK/4 threads
// span a row, so a 256-thread workgroup covers RPP = floor(1024/DK) rows per pass
// and NR passes (when DK/4 does not divide 256 the last few threads only help
// with staging).  Grid: x = Dv tiles, y = b*Hv + hv, z = layer.
template <typename StateT, bool VEC_G, int DK, int NR>
__global__ __launch_bounds__(kThreads) void tape_replay_kernel(ReplayBatch P, ReplayArgs A) {
    constexpr int TPR = DK / 4;
    constexpr int RPP = kThreads / TPR;
    constexpr int ROWS = RPP * NR;
    constexpr int TC = DK >= 256 ? kReplayChunk / 2 : kReplayChunk;   // keeps static LDS under 64 KB

    __shared__ float k_s[TC][DK];
    __shared__ float g_s[VEC_G ? TC : 1][VEC_G ? DK : TC];
    __shared__ float d_s[TC][ROWS];
    __shared__ int on_s[TC];

    // the scalar arguments in one burst of loads (the per-layer pointer tables are indexed by the layer and stay lazy)
    asm volatile("" ::"s"(A.mask), "s"(A.steps_dev), "s"(A.verify_ids), "s"(A.posterior), "s"(A.start_inout), "s"(A.out4),
                 "s"(A.V), "s"(A.mask_dtype), "s"(A.tape_dtype), "s"(A.in_dtype), "s"(A.steps), "s"(A.skip_if_full),
                 "s"(A.T_tape), "s"(A.Hk), "s"(A.Hv), "s"(A.Dv));
    const int layer = blockIdx.z;
    const int bh = blockIdx.y;
    const int b = bh / A.Hv, hv = bh % A.Hv;
    const int hk = hv / (A.Hv / A.Hk);
    const int row0 = blockIdx.x * ROWS;
    const int tid = threadIdx.x;
    const int c4 = (tid % TPR) * 4;
    const bool owner = tid < RPP * TPR;            // false only for the spare threads of an odd TPR
    const int rsub = owner ? tid / TPR : 0;

    int n;
    if (A.verify_ids) {
        // The cycle's acceptance (DFlashRuntime.swift:525-547) is decided here, by every workgroup for
        // itself (two 64-byte reads), so the rollback needs no launch ahead of it; workgroup 0 also does
        // the bookkeeping accept_commit_kernel would have done.
        __shared__ int n_s;
        if (tid < 64) {
            const int acc = A.V > 1 ? leading_matches(A.verify_ids + 1, A.posterior, A.V - 1) : 0;
            if (tid == 0) {
                n_s = 1 + acc;
                if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
                    A.out4[0] = acc;
                    A.out4[1] = 1 + acc;
                    A.out4[2] = (int32_t)A.posterior[acc];
                    int start = 1 + acc;
                    if (A.start_inout) { start += *A.start_inout; *A.start_inout = start; }
                    A.out4[3] = start;
                }
            }
        }
        __syncthreads();
        n = n_s;
    } else {
        n = A.steps;
        if (A.steps_dev) n = __builtin_amdgcn_readfirstlane(*A.steps_dev);   // (kept a branch: as a select of two addresses the host-side count lands in scratch)
    }
    n = n < 0 ? 0 : (n > A.T_tape ? A.T_tape : n);
    if (A.skip_if_full && n == A.T_tape) return;   // uniform over the grid

    const StateT* s_in = reinterpret_cast<const StateT*>(P.state_in[layer]) + (size_t)bh * A.Dv * DK;
    StateT* s_out = reinterpret_cast<StateT*>(P.state_out[layer]) + (size_t)bh * A.Dv * DK;
    const void* tape = P.tape[layer];
    const void* kk = P.k[layer];
    const void* gg = P.g[layer];

    // ---- loads ----
    // A chunk's operands are requested as raw bits, array by array, inside branches that hold nothing but loads,
    // and converted only after the last request has gone out; the state rows are requested in between.  (With a
    // conversion or an LDS store next to each load, the compiler waits for every load before it issues the next:
    // half a dozen dependent round trips per workgroup.)  Addresses are clamped instead of predicated, values that
    // must not count are dropped at the LDS store.
    constexpr int KI = (TC * TPR + kThreads - 1) / kThreads;      // k (and vector gate) groups of 4 per thread
    constexpr int DI = (TC * ROWS + kThreads - 1) / kThreads;     // tape values per thread
    const bool in32 = A.in_dtype == DFLASH_F32, tape32 = A.tape_dtype == DFLASH_F32;
    const bool in_bf16 = A.in_dtype == DFLASH_BF16, tape_bf16 = A.tape_dtype == DFLASH_BF16;
    uint4 k32[KI], g32[VEC_G ? KI : 1];
    uint2 k16[KI], g16[VEC_G ? KI : 1];
    float d32[DI], gs32;
    uint32_t d16[DI], gs16;                                   // 16-bit values, zero-extended
    int on_r;
    auto cvt16 = [](uint16_t bits, bool is_bf16) -> float {
        return is_bf16 ? __uint_as_float(((uint32_t)bits) << 16) : (float)__builtin_bit_cast(_Float16, bits);
    };
    auto cvt4 = [&](uint4 w, uint2 h) -> float4 {
        if (in32) return make_float4(__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z), __uint_as_float(w.w));
        return make_float4(cvt16((uint16_t)(h.x & 0xffffu), in_bf16), cvt16((uint16_t)(h.x >> 16), in_bf16),
                           cvt16((uint16_t)(h.y & 0xffffu), in_bf16), cvt16((uint16_t)(h.y >> 16), in_bf16));
    };
    auto request_chunk = [&](int t0, int tc) {
        size_t kidx[KI], gidx[KI], didx[DI];
#pragma unroll
        for (int u = 0; u < KI; ++u) {
            const int i = tid + u * kThreads, c = (i % TPR) * 4;
            const int t = (i / TPR) < tc ? (i / TPR) : tc - 1;
            const size_t bt = (size_t)b * A.T_tape + t0 + t;
            kidx[u] = (bt * A.Hk + hk) * DK + c;
            gidx[u] = (bt * A.Hv + hv) * DK + c;
        }
#pragma unroll
        for (int u = 0; u < DI; ++u) {
            const int i = tid + u * kThreads, r = i % ROWS;
            const int t = (i / ROWS) < tc ? (i / ROWS) : tc - 1;
            const int row = (row0 + r) < A.Dv ? row0 + r : A.Dv - 1;
            didx[u] = (((size_t)b * A.T_tape + t0 + t) * A.Hv + hv) * A.Dv + row;
        }
        const int tl = tid < tc ? tid : tc - 1;
        const size_t bts = (size_t)b * A.T_tape + t0 + tl;
        if (in32) {
#pragma unroll
            for (int u = 0; u < KI; ++u) {
                k32[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(kk) + kidx[u]);
                if (VEC_G) g32[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(gg) + gidx[u]);
            }
            if (!VEC_G) gs32 = reinterpret_cast<const float*>(gg)[bts * A.Hv + hv];
        } else {
#pragma unroll
            for (int u = 0; u < KI; ++u) {
                k16[u] = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(kk) + kidx[u]);
                if (VEC_G) g16[u] = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(gg) + gidx[u]);
            }
            if (!VEC_G) gs16 = reinterpret_cast<const uint16_t*>(gg)[bts * A.Hv + hv];
        }
        if (tape32) {
#pragma unroll
            for (int u = 0; u < DI; ++u) d32[u] = reinterpret_cast<const float*>(tape)[didx[u]];
        } else {
#pragma unroll
            for (int u = 0; u < DI; ++u) d16[u] = reinterpret_cast<const uint16_t*>(tape)[didx[u]];
        }
        on_r = A.mask ? (int)mask_on(A.mask, A.mask_dtype, (int)bts) : 1;
    };
    auto park_chunk = [&](int tc) {
#pragma unroll
        for (int u = 0; u < KI; ++u) {
            const int i = tid + u * kThreads, t = i / TPR, c = (i % TPR) * 4;
            if (t < tc) {
                store4(&k_s[t][c], cvt4(k32[u], k16[u]));
                if (VEC_G) store4(&g_s[t][c], cvt4(g32[VEC_G ? u : 0], g16[VEC_G ? u : 0]));
            }
        }
#pragma unroll
        for (int u = 0; u < DI; ++u) {
            const int i = tid + u * kThreads, t = i / ROWS, r = i % ROWS;
            if (t < tc) d_s[t][r] = (row0 + r) < A.Dv ? (tape32 ? d32[u] : cvt16((uint16_t)d16[u], tape_bf16)) : 0.f;
        }
        if (tid < tc) {
            if (!VEC_G) g_s[0][tid] = in32 ? gs32 : cvt16((uint16_t)gs16, in_bf16);
            on_s[tid] = on_r;
        }
    };

    const int tc0 = n < TC ? n : TC;
    if (n > 0) request_chunk(0, tc0);
    float4 s[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        int r = row0 + rsub + RPP * i;
        r = r < A.Dv ? r : A.Dv - 1;                       // clamped: rows outside are never stored
        s[i] = load4(s_in + (size_t)r * DK + c4);
    }

    for (int t0 = 0; t0 < n; t0 += TC) {
        const int tc = (n - t0) < TC ? (n - t0) : TC;
        if (t0) {
            __syncthreads();
            request_chunk(t0, tc);
        }
        park_chunk(tc);
        __syncthreads();
        // ---- serial steps, operands from LDS ----
        for (int t = 0; t < tc; ++t) {
            if (!on_s[t]) continue;                 // masked step: state untouched
            const float4 k4 = *reinterpret_cast<const float4*>(&k_s[t][c4]);
            float4 g4;
            if (VEC_G) g4 = *reinterpret_cast<const float4*>(&g_s[t][c4]);
            else { const float gs = g_s[0][t]; g4 = make_float4(gs, gs, gs, gs); }
#pragma unroll
            for (int i = 0; i < NR; ++i) {
                const float d = d_s[t][rsub + RPP * i];
                s[i].x = requant<StateT>(fmaf(k4.x, d, s[i].x * g4.x));
                s[i].y = requant<StateT>(fmaf(k4.y, d, s[i].y * g4.y));
                s[i].z = requant<StateT>(fmaf(k4.z, d, s[i].z * g4.z));
                s[i].w = requant<StateT>(fmaf(k4.w, d, s[i].w * g4.w));
            }
        }
    }

#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const int r = row0 + rsub + RPP * i;
        if (owner && r < A.Dv) store4(s_out + (size_t)r * DK + c4, s[i]);
    }
}

template <typename StateT, bool VEC_G, int DK>
static int launch_replay_nr(hipStream_t st, const ReplayBatch& P, const ReplayArgs& A, int B, int n_layers) {
    constexpr int RPP = kThreads / (DK / 4);
    // Fewer, fatter workgroups once the grid already covers the chip several times over.
    const long wg1 = (long)((A.Dv + RPP - 1) / RPP) * B * A.Hv * n_layers;
    const int cus = num_compute_units();
    LaunchBracket br(DFLASH_KERNEL_TAPE_REPLAY, st);
    if (wg1 >= 16L * cus && A.Dv >= RPP * 4) {
        dim3 grid((A.Dv + RPP * 4 - 1) / (RPP * 4), B * A.Hv, n_layers);
        br.launch(tape_replay_kernel<StateT, VEC_G, DK, 4>, grid, dim3(kThreads), 0, P, A);
    } else {
        dim3 grid((A.Dv + RPP - 1) / RPP, B * A.Hv, n_layers);
        br.launch(tape_replay_kernel<StateT, VEC_G, DK, 1>, grid, dim3(kThreads), 0, P, A);
    }
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

template <typename StateT>
static int launch_replay_state(hipStream_t st, const ReplayBatch& P, const ReplayArgs& A, int B, int n_layers,
                               int g_ndim, int Dk) {
    const bool vec = g_ndim == 4;
#define DFLASH_REPLAY_CASE(DKV)                                                              \
    case DKV:                                                                                \
        return vec ? launch_replay_nr<StateT, true, DKV>(st, P, A, B, n_layers)              \
                   : launch_replay_nr<StateT, false, DKV>(st, P, A, B, n_layers);
    switch (Dk) {
        DFLASH_REPLAY_CASE(32)
        DFLASH_REPLAY_CASE(64)
        DFLASH_REPLAY_CASE(96)
        DFLASH_REPLAY_CASE(128)
        DFLASH_REPLAY_CASE(160)
        DFLASH_REPLAY_CASE(192)
        DFLASH_REPLAY_CASE(224)
        DFLASH_REPLAY_CASE(256)
        default: break;
    }
#undef DFLASH_REPLAY_CASE
    // the reference's Metal kernels take every multiple of 32 (DFlashKernels.swift:271-273); beyond 256 the
    // caller is told to use its general path
    set_error("tape replay: Dk=%d is not a multiple of 32 in [32, 256]", Dk);
    return DFLASH_UNSUPPORTED;
}

struct FusedAccept {
    const uint32_t* verify_ids = nullptr;
    const uint32_t* posterior = nullptr;
    int32_t* start_inout = nullptr;
    int32_t* out4 = nullptr;
    int V = 0;
};

static int replay_common(hipStream_t st, int n_layers, const void* const* tape, int tape_dtype,
                         const void* const* k, const void* const* g, int in_dtype, int g_ndim,
                         const void* const* state_in, void* const* state_out, int state_dtype,
                         const void* mask, int mask_dtype, int steps, const int32_t* steps_dev, int skip_if_full,
                         int B, int T_tape, int Hk, int Hv, int Dk, int Dv, const FusedAccept& acc = FusedAccept()) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(n_layers >= 1 && n_layers <= DFLASH_MAX_BATCHED_LAYERS, "tape replay: n_layers=%d out of range", n_layers);
    DFLASH_REQUIRE(B > 0 && T_tape >= 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, "tape replay: non-positive dimension");
    DFLASH_REQUIRE(Hv % Hk == 0, "tape replay: Hv=%d is not a multiple of Hk=%d", Hv, Hk);
    DFLASH_REQUIRE(g_ndim == 3 || g_ndim == 4, "tape replay: g_ndim must be 3 or 4");
    DFLASH_REQUIRE(steps >= 0 && steps <= T_tape, "tape replay: steps=%d outside [0, T=%d]", steps, T_tape);
    DFLASH_REQUIRE((long)B * Hv <= 65535, "tape replay: B*Hv too large for one launch");
    DFLASH_SUPPORTED(in_dtype == DFLASH_F32 || in_dtype == DFLASH_BF16 || in_dtype == DFLASH_F16, "tape replay: bad in_dtype %d", in_dtype);
    DFLASH_SUPPORTED(tape_dtype == DFLASH_F32 || tape_dtype == in_dtype, "tape replay: tape dtype must be f32 or the input dtype");
    DFLASH_SUPPORTED(state_dtype == DFLASH_F32 || state_dtype == in_dtype, "tape replay: state dtype must be f32 or the input dtype");
    if (mask) DFLASH_REQUIRE(mask_dtype >= DFLASH_F32 && mask_dtype <= DFLASH_U8, "tape replay: bad mask dtype");

    ReplayBatch P;
    for (int l = 0; l < n_layers; ++l) {
        DFLASH_REQUIRE(state_in[l] && state_out[l], "tape replay: null state pointer (layer %d)", l);
        DFLASH_REQUIRE(state_in[l] != state_out[l], "tape replay: state_in aliases state_out (layer %d)", l);
        DFLASH_REQUIRE(T_tape == 0 || (tape[l] && k[l] && g[l]), "tape replay: null input pointer (layer %d)", l);
        P.tape[l] = tape[l]; P.k[l] = k[l]; P.g[l] = g[l];
        P.state_in[l] = state_in[l]; P.state_out[l] = state_out[l];
    }
    ReplayArgs A;
    A.mask = mask; A.steps_dev = steps_dev; A.mask_dtype = mask_dtype; A.tape_dtype = tape_dtype;
    A.verify_ids = acc.verify_ids; A.posterior = acc.posterior; A.start_inout = acc.start_inout; A.out4 = acc.out4; A.V = acc.V;
    A.in_dtype = in_dtype; A.steps = steps; A.skip_if_full = skip_if_full;
    A.T_tape = T_tape; A.Hk = Hk; A.Hv = Hv; A.Dv = Dv;

    switch (state_dtype) {
        case DFLASH_F32: return launch_replay_state<float>(st, P, A, B, n_layers, g_ndim, Dk);
        case DFLASH_BF16: return launch_replay_state<bf16_t>(st, P, A, B, n_layers, g_ndim, Dk);
        default: return launch_replay_state<f16_t>(st, P, A, B, n_layers, g_ndim, Dk);
    }
}

// ===========================================================================
// Gated delta forward with tape
// ===========================================================================

struct GdnArgs {
    const void *q, *k, *v, *g, *beta, *mask;
    const void* state_in;
    void* state_out;
    void* y;
    float* tape;
    int in_dtype, mask_dtype;
    int T, Hk, Hv, Dv;
    // chunked kernels only: value heads per key head and ceil(2^32 / group), so that hv / group is one multiply
    // (exact for hv, group < 2^16; group == 1 is handled apart, its reciprocal does not fit)
    uint32_t group, group_magic;
};

// Inputs of the layer's pre-ops when they run inside the forward kernel (gdn_layer_kernel): the short
// conv + SiLU over q|k|v, the q/k normalisation and the gate formulas of dflash_gdn_prepare.
struct GdnPrep {
    const void* x;            // mixed_qkv [B,T,C]
    const void* conv_in;      // [B,K-1,C] or null (zeros)
    const void* weight;       // [C,K]
    const void* a;            // [B,T,Hv]
    const void* b;            // [B,T,Hv]
    const float* a_log;       // [Hv]
    const float* dt_bias;     // [Hv]
    void *q_out, *k_out, *v_out, *g_out, *beta_out;   // each may be null
    void* conv_out;           // [B,K-1,C]
    float q_scale, k_scale, eps;
    int C;
    // The layer's post-op inside the same launch (all null / 0 when it is not asked for): the workgroup of a head
    // that finishes last -- counted in arrivals[b*Hv + hv], which is zero before the launch and zero again after
    // it -- normalises and gates the head's y rows.
    const void* fin_gate;     // [B,T,Hv,Dv]
    const void* fin_weight;   // [Dv]
    void* fin_out;            // [B,T,Hv,Dv]; until the last workgroup writes a row, its first Dv/16 floats hold
                              // the row tiles' sums of squares
    int32_t* arrivals;        // [B*Hv]
    int32_t* status;          // device status word (dflash_set_status_word), or null
    float fin_eps;
    int fin_silu;
};
constexpr int kLayerTaps = 4;
constexpr int kLayerFinishMaxDv = 256;   // head dim up to which the post-op runs inside the layer kernel  // conv kernel size the one-launch layer kernel is built for

constexpr int kGdnChunk = 16;  // steps staged in LDS at a time

// LPR lanes share one state row; each keeps DK/LPR channels as float4 pieces
// interleaved across the group (piece c of lane j covers channels
// c*4*LPR + 4j .. +3) so that state loads and stores are fully coalesced.
// Three row dot products are reduced together with DPP adds inside the 16-lane
// row: S'k for the innovation, S'q for the read-out and k.q, because
//   y = (S' + delta (x) k) q = S'q + delta * (k.q),
// so only S'k sits on the step-to-step critical path.  The kernel is bound by
// the latency of that serial chain (T dependent steps), not by bandwidth: each
// step's operands are therefore fetched from LDS one step ahead, and the dot
// products run as two half-length chains.
// Grid: x = Dv tiles of ROWS = 256/LPR rows, y = b*Hv + hv.
template <int CH> struct GdnStepOps {
    float4 k[CH], q[CH], g[CH];
    float gs, v, beta, kq;
    int on;
};

template <typename StateT, bool VEC_G, bool HAS_MASK, int DK, int LPR>
__global__ __launch_bounds__(kThreads) void gated_delta_tape_kernel(GdnArgs A) {
    constexpr int ROWS = kThreads / LPR;
    constexpr int CH = DK / (4 * LPR);
    constexpr int TC = kGdnChunk;
    constexpr int TPR = DK / 4;                                   // threads spanning one step's q (or k) row, 4 channels each
    static_assert(CH >= 1, "row slice must hold at least one float4");

    __shared__ float q_s[TC][DK];
    __shared__ float k_s[TC][DK];
    __shared__ float g_s[VEC_G ? TC : 1][VEC_G ? DK : TC];
    __shared__ float v_s[TC][ROWS];
    __shared__ float y_s[TC][ROWS];
    __shared__ float t_s[TC][ROWS];
    __shared__ float beta_s[TC];
    __shared__ int on_s[TC];

    // every argument in one burst of scalar loads (fetched where first used they are several dependent trips to memory)
    asm volatile("" ::"s"(A.q), "s"(A.k), "s"(A.v), "s"(A.g), "s"(A.beta), "s"(A.mask), "s"(A.state_in), "s"(A.state_out),
                 "s"(A.y), "s"(A.tape), "s"(A.in_dtype), "s"(A.mask_dtype), "s"(A.T), "s"(A.Hk), "s"(A.Hv), "s"(A.Dv));
    const int bh = blockIdx.y;
    const int b = bh / A.Hv, hv = bh % A.Hv;
    const int hk = hv / (A.Hv / A.Hk);
    const int row0 = blockIdx.x * ROWS;
    const int tid = threadIdx.x;
    const int j = tid % LPR;
    const int rloc = tid / LPR;
    const int row = row0 + rloc;
    const bool row_ok = row < A.Dv;

    const StateT* s_in = reinterpret_cast<const StateT*>(A.state_in) + ((size_t)bh * A.Dv + (row_ok ? row : 0)) * DK;
    StateT* s_out = reinterpret_cast<StateT*>(A.state_out) + ((size_t)bh * A.Dv + (row_ok ? row : 0)) * DK;

    // The state rows are the largest operand: their loads go out first.
    float4 s[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) s[c] = load4(s_in + c * 4 * LPR + 4 * j);

    // ---- a chunk's operands: requested as raw bits, array by array, inside branches that hold nothing but loads, and
    // converted only after the last request has gone out -- one memory round trip per chunk.  (With a conversion or an
    // LDS store next to each load, or a switch on the element type around it, the compiler waits for every load before
    // it issues the next: half a dozen dependent round trips per launch.)  Addresses are clamped instead of predicated;
    // values that must not count are dropped at the LDS store. ----
    constexpr int QI = (TC * TPR + kThreads - 1) / kThreads;      // q / k (and vector gate) groups of 4 per thread
    constexpr int VI = (TC * ROWS + kThreads - 1) / kThreads;     // v values per thread
    const bool in32 = A.in_dtype == DFLASH_F32, in_bf16 = A.in_dtype == DFLASH_BF16;
    uint4 q32[QI], k32[QI], g32[VEC_G ? QI : 1];
    uint2 q16[QI], k16[QI], g16[VEC_G ? QI : 1];
    float v32[VI], gs32 = 1.f, bs32 = 0.f;
    uint32_t v16[VI], gs16 = 0, bs16 = 0;                         // 16-bit values, zero-extended
    int on_r = 1;
    auto cvt16 = [](uint16_t bits, bool is_bf16) -> float {
        return is_bf16 ? __uint_as_float(((uint32_t)bits) << 16) : (float)__builtin_bit_cast(_Float16, bits);
    };
    auto cvt4 = [&](uint4 w, uint2 h) -> float4 {
        if (in32) return make_float4(__uint_as_float(w.x), __uint_as_float(w.y), __uint_as_float(w.z), __uint_as_float(w.w));
        return make_float4(cvt16((uint16_t)(h.x & 0xffffu), in_bf16), cvt16((uint16_t)(h.x >> 16), in_bf16),
                           cvt16((uint16_t)(h.y & 0xffffu), in_bf16), cvt16((uint16_t)(h.y >> 16), in_bf16));
    };
    auto request_chunk = [&](int t0, int tc) {
        size_t kidx[QI], gidx[QI], vidx[VI];
#pragma unroll
        for (int u = 0; u < QI; ++u) {
            const int i = tid + u * kThreads, c = (i % TPR) * 4;
            const int t = (i / TPR) < tc ? (i / TPR) : tc - 1;
            const size_t bt = (size_t)b * A.T + t0 + t;
            kidx[u] = (bt * A.Hk + hk) * DK + c;
            gidx[u] = (bt * A.Hv + hv) * DK + c;
        }
#pragma unroll
        for (int u = 0; u < VI; ++u) {
            const int i = tid + u * kThreads, r = i % ROWS;
            const int t = (i / ROWS) < tc ? (i / ROWS) : tc - 1;
            const int rr = (row0 + r) < A.Dv ? row0 + r : A.Dv - 1;
            vidx[u] = (((size_t)b * A.T + t0 + t) * A.Hv + hv) * A.Dv + rr;
        }
        const int tl = tid < tc ? tid : tc - 1;
        const size_t bts = (size_t)b * A.T + t0 + tl;
        if (in32) {
#pragma unroll
            for (int u = 0; u < QI; ++u) {
                q32[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(A.q) + kidx[u]);
                k32[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(A.k) + kidx[u]);
                if (VEC_G) g32[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(A.g) + gidx[u]);
            }
#pragma unroll
            for (int u = 0; u < VI; ++u) v32[u] = reinterpret_cast<const float*>(A.v)[vidx[u]];
            if (!VEC_G) gs32 = reinterpret_cast<const float*>(A.g)[bts * A.Hv + hv];
            bs32 = reinterpret_cast<const float*>(A.beta)[bts * A.Hv + hv];
        } else {
#pragma unroll
            for (int u = 0; u < QI; ++u) {
                q16[u] = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(A.q) + kidx[u]);
                k16[u] = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(A.k) + kidx[u]);
                if (VEC_G) g16[u] = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(A.g) + gidx[u]);
            }
#pragma unroll
            for (int u = 0; u < VI; ++u) v16[u] = reinterpret_cast<const uint16_t*>(A.v)[vidx[u]];
            if (!VEC_G) gs16 = reinterpret_cast<const uint16_t*>(A.g)[bts * A.Hv + hv];
            bs16 = reinterpret_cast<const uint16_t*>(A.beta)[bts * A.Hv + hv];
        }
        if (HAS_MASK) on_r = (int)mask_on(A.mask, A.mask_dtype, (int)bts);
    };
    auto park_chunk = [&](int tc) {
#pragma unroll
        for (int u = 0; u < QI; ++u) {
            const int i = tid + u * kThreads, t = i / TPR, c = (i % TPR) * 4;
            if (t < tc) {
                store4(&q_s[t][c], cvt4(q32[u], q16[u]));
                store4(&k_s[t][c], cvt4(k32[u], k16[u]));
                if (VEC_G) store4(&g_s[t][c], cvt4(g32[VEC_G ? u : 0], g16[VEC_G ? u : 0]));
            }
        }
#pragma unroll
        for (int u = 0; u < VI; ++u) {
            const int i = tid + u * kThreads, t = i / ROWS, r = i % ROWS;
            if (t < tc) v_s[t][r] = (row0 + r) < A.Dv ? (in32 ? v32[u] : cvt16((uint16_t)v16[u], in_bf16)) : 0.f;
        }
        if (tid < tc) {
            if (!VEC_G) g_s[0][tid] = in32 ? gs32 : cvt16((uint16_t)gs16, in_bf16);
            beta_s[tid] = in32 ? bs32 : cvt16((uint16_t)bs16, in_bf16);
            if (HAS_MASK) on_s[tid] = on_r;
        }
    };

    auto fetch = [&](int t, GdnStepOps<CH>& o) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int d = c * 4 * LPR + 4 * j;
            o.k[c] = *reinterpret_cast<const float4*>(&k_s[t][d]);
            o.q[c] = *reinterpret_cast<const float4*>(&q_s[t][d]);
            if (VEC_G) o.g[c] = *reinterpret_cast<const float4*>(&g_s[t][d]);
        }
        o.gs = VEC_G ? 1.f : g_s[0][t];
        o.v = v_s[t][rloc];
        o.beta = beta_s[t];
        o.on = HAS_MASK ? on_s[t] : 1;
        // k.q of the step (one value per head and step) from the lane's own channels; it does not depend on the
        // state, so its reduction runs beside the step-to-step chain, not on it
        float kq0 = 0.f, kq1 = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            kq0 = fmaf(o.k[c].x, o.q[c].x, kq0); kq1 = fmaf(o.k[c].y, o.q[c].y, kq1);
            kq0 = fmaf(o.k[c].z, o.q[c].z, kq0); kq1 = fmaf(o.k[c].w, o.q[c].w, kq1);
        }
        o.kq = group_sum<LPR>(kq0 + kq1);
    };

    if (A.T > 0) request_chunk(0, A.T < TC ? A.T : TC);
    for (int t0 = 0; t0 < A.T; t0 += TC) {
        const int tc = (A.T - t0) < TC ? (A.T - t0) : TC;
        if (t0) {
            __syncthreads();                      // every wave is done with the previous chunk's operands and outputs
            request_chunk(t0, tc);
        }
        park_chunk(tc);
        __syncthreads();

        // ---- serial steps, operands one step ahead (two operand sets, no register copies) ----
        auto step = [&](int t, const GdnStepOps<CH>& cur) {
            float yv = 0.f, delta = 0.f;
            if (!HAS_MASK || cur.on) {                // uniform across the workgroup
                float sk0 = 0.f, sk1 = 0.f, sq0 = 0.f, sq1 = 0.f;
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const float4 k4 = cur.k[c], q4 = cur.q[c];
                    const float4 g4 = VEC_G ? cur.g[c] : make_float4(cur.gs, cur.gs, cur.gs, cur.gs);
                    s[c].x *= g4.x; s[c].y *= g4.y; s[c].z *= g4.z; s[c].w *= g4.w;
                    sk0 = fmaf(s[c].x, k4.x, sk0); sk1 = fmaf(s[c].y, k4.y, sk1);
                    sk0 = fmaf(s[c].z, k4.z, sk0); sk1 = fmaf(s[c].w, k4.w, sk1);
                    sq0 = fmaf(s[c].x, q4.x, sq0); sq1 = fmaf(s[c].y, q4.y, sq1);
                    sq0 = fmaf(s[c].z, q4.z, sq0); sq1 = fmaf(s[c].w, q4.w, sq1);
                }
                const float sk = group_sum<LPR>(sk0 + sk1);
                const float sq = group_sum<LPR>(sq0 + sq1);
                delta = (cur.v - sk) * cur.beta;
                yv = fmaf(delta, cur.kq, sq);
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const float4 k4 = cur.k[c];
                    s[c].x = requant<StateT>(fmaf(k4.x, delta, s[c].x));
                    s[c].y = requant<StateT>(fmaf(k4.y, delta, s[c].y));
                    s[c].z = requant<StateT>(fmaf(k4.z, delta, s[c].z));
                    s[c].w = requant<StateT>(fmaf(k4.w, delta, s[c].w));
                }
            }
            if (j == 0) { y_s[t][rloc] = yv; t_s[t][rloc] = delta; }
        };
        if (tc == TC) {
            // A full chunk (the verify block) is straight-line code: operands are fetched kAhead steps ahead of their
            // use, so no step waits for LDS.
            constexpr int kAhead = 4;
            GdnStepOps<CH> ops[TC];
#pragma unroll
            for (int t = 0; t < kAhead; ++t) fetch(t, ops[t]);
#pragma unroll
            for (int t = 0; t < TC; ++t) {
                if (t + kAhead < TC) fetch(t + kAhead, ops[t + kAhead]);
                step(t, ops[t]);
            }
        } else {
            GdnStepOps<CH> opa, opb;
            fetch(0, opa);
            for (int t = 0; t < tc; t += 2) {
                if (t + 1 < tc) fetch(t + 1, opb);
                step(t, opa);
                if (t + 1 < tc) {
                    if (t + 2 < tc) fetch(t + 2, opa);
                    step(t + 1, opb);
                }
            }
        }
        __syncthreads();
        // ---- write this chunk's y and tape rows ----
        for (int i = tid; i < tc * ROWS; i += kThreads) {
            const int t = i / ROWS, r = i % ROWS;
            if (row0 + r < A.Dv) {
                const size_t o = (((size_t)b * A.T + t0 + t) * A.Hv + hv) * A.Dv + row0 + r;
                store1_rt(A.y, A.in_dtype, o, y_s[t][r]);
                A.tape[o] = t_s[t][r];
            }
        }
    }

    if (row_ok) {
#pragma unroll
        for (int c = 0; c < CH; ++c) store4(s_out + c * 4 * LPR + 4 * j, s[c]);
    }
}

// ---------------------------------------------------------------------------
// Chunked form (fp32 state, one decay per head and step).
//
// The serial kernel above spends its time in T dependent steps that each need
// two Dk-wide row reductions.  Unrolling the recurrence over a chunk of
// C <= 16 steps moves every Dk-wide contraction out of the serial part:
//
//   G[s][t]  = g_{s+1} * ... * g_t                (products, never quotients: no underflow ratio)
//   gam_t    = g_0 * ... * g_t
//   S_t      = gam_t S_0 + sum_{s<=t} G[s][t] delta_s (x) k_s
//   delta_t  = beta_t ( v_t - gam_t S_0 k_t - sum_{s<t} G[s][t] (k_s.k_t) delta_s )
//   y_t      = gam_t S_0 q_t + sum_{s<=t} G[s][t] (k_s.q_t) delta_s
//
// so one fp32 MFMA product  [S_0 rows ; k rows] x [k | q]^T  gives S_0 k_t, S_0 q_t, k_s.k_t
// and k_s.q_t at once, the step-to-step dependency shrinks to a 16x16 unit-triangular solve per
// state row (a few registers per lane, no Dk-wide reduction), and the state update is one rank-C
// MFMA product.  A masked or padded step is the identity step g = 1, beta = 0 (delta = 0) with
// y forced to 0 (DFlashKernels.swift:150-197 leaves the state untouched and emits zeros).
//
// Workgroup: 16 state rows of one head (grid x = Dv/16, y = b*Hv + hv), 4 waves.
// ---------------------------------------------------------------------------

constexpr int kChunkRows = 16;
constexpr int kChunkSteps = 16;

template <int DK> struct GdnChunkLds {
    static constexpr int LD = DK + 4;      // row pitch in floats: 16-byte pad spreads rows over the banks
    float x[32][LD];                       // rows 0..15 state tile, rows 16..31 k_t
    float y[32][LD];                       // rows 0..15 k_t, rows 16..31 q_t
    float p[16][33];                       // S_0 x [k | q]^T: p[r][t] = S_0 k_t, p[r][16 + t] = S_0 q_t of state row r
    float a[16][16];                       // a[s][t] = G[s][t] k_s.k_t for s < t, else 0
    float c[16][16];                       // c[s][t] = G[s][t] k_s.q_t for s <= t, else 0
    float dl[16][17];                      // delta_s of row r at dl[s][r]
    float v[16][16];                       // v_t of row r at v[t][r]
    float g[16], beta[16], gam[16], w[16]; // w[s] = G[s][15]: decay from step s to the end of the chunk
    int on[16];
    // bf16 inputs: the product's operands as bf16 (x rows 16..31 and y rows 16..31 are then unused).  The state tile
    // as three bf16 terms, S_0 = hi + mid + lo exactly (3 x 8 = 24 significand bits); k_t and q_t as they came.
    // Row pitch DK + 8: the 16 bytes of pad spread a column of rows over all banks for 16-byte reads.
    static constexpr int LB = DK + 8;
    uint16_t xs[3][16][LB];
    uint16_t kb[16][LB], qb[16][LB];
};

typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));

// The upper halves of two words as one: (a >> 16) | (b & 0xffff0000), one v_perm_b32.
__device__ __forceinline__ uint32_t upper_halves(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }
// Four floats that are bf16 values -> their 4 x 16 bits.
__device__ __forceinline__ uint2 pack4_bf16_exact(float4 v) {
    return make_uint2(upper_halves(__float_as_uint(v.x), __float_as_uint(v.y)), upper_halves(__float_as_uint(v.z), __float_as_uint(v.w)));
}
// x = hi + mid + lo with each term a bf16, by truncation: hi = the upper 16 bits of x, mid = the upper 16 bits of
// x - hi, lo = x - hi - mid.  hi takes 8 of x's 24 significand bits, mid the next 8 (or more, where zeros follow hi),
// so lo has at most 8 left and is a bf16 as it stands; both subtractions are exact, and the three terms add up to x
// bit for bit.  Four VALU operations per value and one v_perm per pair and term.
__device__ __forceinline__ void split3_bf16(float x, float& r1, float& r2) {
    r1 = x - __uint_as_float(__float_as_uint(x) & 0xffff0000u);
    r2 = r1 - __uint_as_float(__float_as_uint(r1) & 0xffff0000u);
}
__device__ __forceinline__ void split3_bf16(float x, uint16_t& hi, uint16_t& mid, uint16_t& lo) {
    float r1, r2;
    split3_bf16(x, r1, r2);
    hi = (uint16_t)(__float_as_uint(x) >> 16); mid = (uint16_t)(__float_as_uint(r1) >> 16); lo = (uint16_t)(__float_as_uint(r2) >> 16);
}
__device__ __forceinline__ void split3_bf16(float4 v, uint2& hi, uint2& mid, uint2& lo) {
    const float x[4] = {v.x, v.y, v.z, v.w};
    float r1[4], r2[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) split3_bf16(x[i], r1[i], r2[i]);
    hi = make_uint2(upper_halves(__float_as_uint(x[0]), __float_as_uint(x[1])), upper_halves(__float_as_uint(x[2]), __float_as_uint(x[3])));
    mid = make_uint2(upper_halves(__float_as_uint(r1[0]), __float_as_uint(r1[1])), upper_halves(__float_as_uint(r1[2]), __float_as_uint(r1[3])));
    lo = make_uint2(upper_halves(__float_as_uint(r2[0]), __float_as_uint(r2[1])), upper_halves(__float_as_uint(r2[2]), __float_as_uint(r2[3])));
}

typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef float f32x2v __attribute__((ext_vector_type(2)));
typedef float f32x16v __attribute__((ext_vector_type(16)));

template <int QUAD_LANE> __device__ __forceinline__ float quad_broadcast(float x) {
    constexpr int ctrl = QUAD_LANE | (QUAD_LANE << 2) | (QUAD_LANE << 4) | (QUAD_LANE << 6);
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), ctrl, 0xf, 0xf, true));
}

// Steps S..15 of the unit-triangular solve for one state row held by a quad (lane q owns steps 4q..4q+3).
// Every lane of the quad sees every delta; lane q keeps those of its own four steps in `mine` (a select per step,
// no branch) for the store that follows.
template <int S> struct SolveStep {
    static __device__ __forceinline__ void run(float (&acc)[4], const float4 (&arow)[16], const float (&bet)[16],
                                               float (&mine)[4], const int q) {
        const float d = quad_broadcast<S / 4>(bet[S] * acc[S % 4]);
        mine[S % 4] = q == S / 4 ? d : mine[S % 4];
        acc[0] = fmaf(-arow[S].x, d, acc[0]);
        acc[1] = fmaf(-arow[S].y, d, acc[1]);
        acc[2] = fmaf(-arow[S].z, d, acc[2]);
        acc[3] = fmaf(-arow[S].w, d, acc[3]);
        if constexpr (S + 1 < 16) SolveStep<S + 1>::run(acc, arow, bet, mine, q);
    }
};

// BF: the inputs are bf16 (fixed at compile time): the product then runs on bf16 MFMAs, exactly (see below).
template <bool HAS_MASK, int DK, bool FUSED, bool BF>
__device__ __forceinline__ void gdn_chunk_body(const GdnArgs& A, const GdnPrep& P) {
    using Lds = GdnChunkLds<DK>;
    extern __shared__ __align__(16) unsigned char gdn_chunk_smem[];
    Lds& L = *reinterpret_cast<Lds*>(gdn_chunk_smem);
    // Every kernel argument is asked for here, in one burst of scalar loads.  Left alone the compiler fetches
    // them where they are first used, in three or four dependent rounds, and each round that touches a new
    // cache line of the argument block is a trip to memory on the way to the first global load.
    if constexpr (FUSED)
        asm volatile("" ::"s"(A.state_in), "s"(A.state_out), "s"(A.y), "s"(A.tape), "s"(A.in_dtype), "s"(A.T), "s"(A.Hk),
                     "s"(A.Hv), "s"(A.Dv), "s"(A.group), "s"(A.group_magic), "s"(P.x), "s"(P.conv_in), "s"(P.weight), "s"(P.a), "s"(P.b), "s"(P.a_log),
                     "s"(P.dt_bias), "s"(P.q_out), "s"(P.k_out), "s"(P.v_out), "s"(P.g_out), "s"(P.beta_out), "s"(P.conv_out),
                     "s"(P.q_scale), "s"(P.k_scale), "s"(P.eps), "s"(P.C));
    if constexpr (FUSED)
        asm volatile("" ::"s"(P.fin_gate), "s"(P.fin_weight), "s"(P.fin_out), "s"(P.arrivals), "s"(P.status), "s"(P.fin_eps), "s"(P.fin_silu));
    // (The plain forward gets what its first loads need -- the state pointer, k, q and the sizes in their addresses -- in
    //  SGPRs at wave start, as leading kernel arguments; the rest of its arguments are named in one such statement
    //  further down, behind those loads, so that the wait for the argument block does not stand in front of them.)
    constexpr int E = DK / 64;             // channels per lane in the state-update product (16 lanes x E x 4 waves = DK)
    static_assert(DK % 64 == 0, "chunked gated delta needs Dk to be a multiple of 64");

    const int tid = threadIdx.x, lane = tid % 64, w = tid / 64;
    // Grid (Dv/16, Hv, B): no division on the way to the first address (an integer division is some twenty
    // dependent instructions, and everything ahead of the loads is on the critical path).  Element offsets into
    // q/k/v/g/beta/y/tape are 32-bit (the host checks the sizes), their per-thread parts 24-bit multiplies.
    const int b = blockIdx.z, hv = blockIdx.y;
    const int bh = b * A.Hv + hv;
    const int hk = A.group == 1 ? hv : (FUSED ? (int)__umulhi((uint32_t)hv, A.group_magic) : (int)((uint32_t)hv / A.group));
    const int row0 = blockIdx.x * kChunkRows;
    const float* s_in = reinterpret_cast<const float*>(A.state_in) + ((size_t)bh * A.Dv + row0) * DK;
    const size_t tile_off = ((size_t)bh * A.Dv + row0) * DK;          // of this workgroup's rows in the state arrays
    const uint32_t k_step = (uint32_t)A.Hk * DK, v_step = (uint32_t)A.Hv * A.Dv;       // elements per step

    constexpr int NV = kChunkRows * (DK / 4) / kThreads;      // float4 groups per thread of a 16 x DK tile
    const int ts = tid / 16, tt = tid % 16;        // (s, t) for the tables, (t, r) for v / y / tape

    if (A.T == 0) {                        // nothing to do but hand the state over
        if (A.state_out == nullptr) return;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int i = tid + u * kThreads, r = i / (DK / 4), c4 = (i % (DK / 4)) * 4;
            store4(reinterpret_cast<float*>(A.state_out) + tile_off + (size_t)r * DK + c4, load4(s_in + (size_t)r * DK + c4));
        }
        return;
    }

    // The state tile is the coldest and largest operand: its loads go out first, ahead of the index arithmetic of
    // everything else.
    float4 sv0[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int i = tid + u * kThreads, r = i / (DK / 4), c4 = (i % (DK / 4)) * 4;
        sv0[u] = load4(s_in + (uint32_t)(r * DK + c4));
    }

    // Where the staged operands go: fp32 rows for the fp32 product (x = [S_0 ; k], y = [k ; q]); with bf16 inputs the
    // product reads the bf16 arrays instead, and only what the state update needs stays fp32 (S_0 and k).
    auto store_state4 = [&](int r, int c4, float4 s4) {
        store4(&L.x[r][c4], s4);
        if constexpr (BF) {
            uint2 hi, mid, lo;
            split3_bf16(s4, hi, mid, lo);
            *reinterpret_cast<uint2*>(&L.xs[0][r][c4]) = hi;
            *reinterpret_cast<uint2*>(&L.xs[1][r][c4]) = mid;
            *reinterpret_cast<uint2*>(&L.xs[2][r][c4]) = lo;
        }
    };
    auto store_kq4 = [&](int t, int c4, float4 k4, float4 q4) {
        store4(&L.y[t][c4], k4);
        if constexpr (BF) {
            *reinterpret_cast<uint2*>(&L.kb[t][c4]) = pack4_bf16_exact(k4);
            *reinterpret_cast<uint2*>(&L.qb[t][c4]) = pack4_bf16_exact(q4);
        } else {
            store4(&L.x[16 + t][c4], k4);
            store4(&L.y[16 + t][c4], q4);
        }
    };

    // Stage one chunk: every global load of the chunk (the state tile is already on its way) is issued
    // before the first conversion or LDS store, so the chunk pays one memory round trip, not one per array.
    // Steps >= tc are identity steps.  Elem is the element type of q/k/v/g/beta.
    auto stage = [&](auto elem_tag, int t0, int tc, bool with_state) {
        using Elem = decltype(elem_tag);
        const Elem* kp = reinterpret_cast<const Elem*>(A.k);
        const Elem* qp = reinterpret_cast<const Elem*>(A.q);
        const Elem* vp = reinterpret_cast<const Elem*>(A.v);
        const Elem* gp = reinterpret_cast<const Elem*>(A.g);
        const Elem* bp = reinterpret_cast<const Elem*>(A.beta);
        float4 kv[NV], qv[NV];
        uint2 kraw[NV], qraw[NV];               // bf16 inputs: the rows as they come (q is never widened)
        const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
        const uint32_t bt0 = (uint32_t)b * A.T + t0;                       // first step of the chunk, all uniform
        const uint32_t k0 = (bt0 * A.Hk + hk) * DK, v0 = (bt0 * A.Hv + hv) * A.Dv + row0, g0 = bt0 * A.Hv + hv;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int i = tid + u * kThreads, t = i / (DK / 4), c4 = (i % (DK / 4)) * 4;
            const int tl = t < tc ? t : tc - 1;           // clamped: always a valid address, selected away below
            const uint32_t o = k0 + __umul24(tl, k_step) + c4;
            if constexpr (BF) {
                kraw[u] = *reinterpret_cast<const uint2*>(kp + o);
                qraw[u] = *reinterpret_cast<const uint2*>(qp + o);
            } else {
                kv[u] = load4(kp + o);
                qv[u] = load4(qp + o);
            }
        }
        const int tvl = ts < tc ? ts : tc - 1;
        const float vv = to_float(vp[v0 + __umul24(tvl, v_step) + tt]);
        float gv = 1.f, bv = 0.f;
        bool on = false;
        if (tid < kChunkSteps) {
            const int tl = tid < tc ? tid : tc - 1;
            const uint32_t go = g0 + __umul24(tl, A.Hv);
            gv = to_float(gp[go]);
            bv = to_float(bp[go]);
            on = HAS_MASK ? mask_on(A.mask, A.mask_dtype, (int)(bt0 + tl)) : true;
            on = on && tid < tc;
        }
        // The arguments that were not handed over in registers, in one burst of scalar loads, behind every load of the
        // chunk (pinned: the scheduler would otherwise lift the first use of one of them, and with it the wait for the
        // argument block, in front of the loads).
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::"s"(A.mask), "s"(A.state_out), "s"(A.y), "s"(A.tape), "s"(A.in_dtype), "s"(A.mask_dtype));
        if (with_state) {
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                const int i = tid + u * kThreads, r = i / (DK / 4), c4 = (i % (DK / 4)) * 4;
                store_state4(r, c4, sv0[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int i = tid + u * kThreads, t = i / (DK / 4), c4 = (i % (DK / 4)) * 4;
            if constexpr (BF) {
                const uint2 kr = t < tc ? kraw[u] : make_uint2(0u, 0u), qr = t < tc ? qraw[u] : make_uint2(0u, 0u);
                store4(&L.y[t][c4], make_float4(__uint_as_float(kr.x << 16), __uint_as_float(kr.x & 0xffff0000u),
                                                __uint_as_float(kr.y << 16), __uint_as_float(kr.y & 0xffff0000u)));
                *reinterpret_cast<uint2*>(&L.kb[t][c4]) = kr;
                *reinterpret_cast<uint2*>(&L.qb[t][c4]) = qr;
            } else {
                store_kq4(t, c4, t < tc ? kv[u] : zero4, t < tc ? qv[u] : zero4);
            }
        }
        L.v[ts][tt] = ts < tc ? vv : 0.f;
        if (tid < kChunkSteps) {
            L.on[tid] = on;
            L.g[tid] = on ? gv : 1.f;
            L.beta[tid] = on ? bv : 0.f;
        }
    };

    // The same with the layer's pre-ops done on the way in (one chunk, T <= 16, kLayerTaps conv taps): instead of
    // q, k, v, g, beta the workgroup reads the raw projections -- for every (step, 4 channels) of its key head the
    // K window rows of q and of k, for its 16 value rows K single elements per step -- and the conv taps, all in one
    // round trip with the state tile; conv -> SiLU -> per-head RMS scale (sum of squares over the DK/4 lanes that
    // share a step) -> rounded to the element type exactly as dflash_gdn_prepare stores them, so that the recurrence
    // sees bit-identical operands.  What the rollback cache records (k, g, the conv window) and the optional q, v,
    // beta are written by the first row tile of a head (q, k: of the first value head of the key head's group).
    auto stage_fused = [&](auto elem_tag, int tc) {
        using Elem = decltype(elem_tag);
        constexpr int KT = kLayerTaps, keep = KT - 1, LPT = DK / 4;
        const int C = P.C;
        const Elem* x = reinterpret_cast<const Elem*>(P.x) + (size_t)b * A.T * C;
        const Elem* cs = P.conv_in ? reinterpret_cast<const Elem*>(P.conv_in) + (size_t)b * keep * C : nullptr;
        const Elem* wt = reinterpret_cast<const Elem*>(P.weight);
        const int cq = hk * DK, ck = (A.Hk + hk) * DK, cv = 2 * A.Hk * DK + hv * A.Dv + row0;
        const int c4 = (tid % LPT) * 4;
        // Window row r of the concatenation [conv_in (keep rows) ; x (T rows)]; without conv_in its rows are zeros
        // (a valid address is read and the value dropped).  Selects, no branches: a branch around a load makes the
        // compiler wait for that load before it issues the next one.
        const Elem* csz = cs ? cs : x;
        auto win_row = [&](int r) -> const Elem* {
            const bool in_x = r >= keep;
            const int rr = in_x ? r - keep : (cs ? r : 0);
            return (in_x ? x : csz) + __umul24(rr, C);
        };
        float4 kw[NV][KT], qw[NV][KT], ktap[4], qtap[4], vtap;
        float vw[KT];
#pragma unroll
        for (int m = 0; m < 4; ++m) {               // [m] = the KT taps of channel c4 + m
            ktap[m] = load4(wt + (uint32_t)((ck + c4 + m) * KT));
            qtap[m] = load4(wt + (uint32_t)((cq + c4 + m) * KT));
        }
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int t = (tid + u * kThreads) / LPT, tl = t < tc ? t : tc - 1;
#pragma unroll
            for (int j = 0; j < KT; ++j) {
                const Elem* src = win_row(tl + j);
                kw[u][j] = load4(src + ck + c4);
                qw[u][j] = load4(src + cq + c4);
            }
        }
        const int tvl = ts < tc ? ts : tc - 1;
#pragma unroll
        for (int j = 0; j < KT; ++j) vw[j] = to_float(win_row(tvl + j)[cv + tt]);
        vtap = load4(wt + (uint32_t)((cv + tt) * KT));
        // gate inputs: every thread reads them (step tid mod 16), so that no load sits inside a branch
        const int tg = (tid % kChunkSteps) < tc ? (tid % kChunkSteps) : tc - 1;
        const uint32_t btg = ((uint32_t)b * A.T + tg) * A.Hv + hv;
        const float av = to_float(reinterpret_cast<const Elem*>(P.a)[btg]);
        const float bv = to_float(reinterpret_cast<const Elem*>(P.b)[btg]);
        const float alog = P.a_log[hv];
        const float dtb = P.dt_bias[hv];
        // ---- every load is out; now the arithmetic ----
        // (pinned: left to itself the scheduler starts on the state tile, whose loads were first, before the last
        //  window loads are issued, and those then leave a whole memory round trip later)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int i = tid + u * kThreads, r = i / (DK / 4), cc = (i % (DK / 4)) * 4;
            store_state4(r, cc, sv0[u]);
        }
        const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
        // Without a carried window the rows in front of the sequence are zeros: set once here, under a uniform branch
        // (selected tap by tap inside the conv it was a select per multiply on every call, carried window or not).
        if (!cs) {
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                const int t = (tid + u * kThreads) / LPT, tl = t < tc ? t : tc - 1;
#pragma unroll
                for (int j = 0; j < KT; ++j)
                    if (tl + j < keep) { kw[u][j] = zero4; qw[u][j] = zero4; }
            }
#pragma unroll
            for (int j = 0; j < KT; ++j)
                if (tvl + j < keep) vw[j] = 0.f;
        }
        const bool first_tile = blockIdx.x == 0;
        const bool qk_owner = first_tile && (hv % (A.Hv / A.Hk)) == 0;
        auto conv4 = [&](const float4 (&w)[KT], const float4 (&tap)[4], int tl) -> float4 {
            float o[4];
#pragma unroll
            for (int m = 0; m < 4; ++m) {
                const float tp[4] = {tap[m].x, tap[m].y, tap[m].z, tap[m].w};
                float acc = 0.f;
#pragma unroll
                for (int j = 0; j < KT; ++j) {
                    const float wj[4] = {w[j].x, w[j].y, w[j].z, w[j].w};
                    acc = fmaf(wj[m], tp[j], acc);
                }
                o[m] = silu_f(acc);
            }
            return make_float4(o[0], o[1], o[2], o[3]);
        };
        auto head_scale = [&](float4 y, float sc) -> float {
            float ss = __fadd_rn(__fadd_rn(__fmul_rn(y.x, y.x), __fmul_rn(y.y, y.y)),
                                 __fadd_rn(__fmul_rn(y.z, y.z), __fmul_rn(y.w, y.w)));
            return gdn_norm_scale(butterfly_sum<LPT>(ss), DK, P.eps, sc);
        };
        auto round4 = [](float4 y, float sc) -> float4 {
            return requant4<Elem>(make_float4(y.x * sc, y.y * sc, y.z * sc, y.w * sc));
        };
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int t = (tid + u * kThreads) / LPT, tl = t < tc ? t : tc - 1;
            const float4 kc = conv4(kw[u], ktap, tl), qc = conv4(qw[u], qtap, tl);
            const float4 k4 = round4(kc, head_scale(kc, P.k_scale)), q4 = round4(qc, head_scale(qc, P.q_scale));
            const bool live = t < tc;
            store_kq4(t, c4, live ? k4 : zero4, live ? q4 : zero4);
            if (qk_owner && live) {
                const size_t o = (((size_t)b * A.T + t) * A.Hk + hk) * DK + c4;
                if (P.k_out) store4(reinterpret_cast<Elem*>(P.k_out) + o, k4);
                if (P.q_out) store4(reinterpret_cast<Elem*>(P.q_out) + o, q4);
                if (t == tc - 1) {                  // the new conv window: rows 1..K-1 of the last step's window
                    Elem* dst = reinterpret_cast<Elem*>(P.conv_out) + (size_t)b * keep * C;
#pragma unroll
                    for (int j = 1; j < KT; ++j) {
                        store4(dst + (size_t)(j - 1) * C + ck + c4, kw[u][j]);
                        store4(dst + (size_t)(j - 1) * C + cq + c4, qw[u][j]);
                    }
                }
            }
        }
        {
            const float tp[4] = {vtap.x, vtap.y, vtap.z, vtap.w};
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < KT; ++j) acc = fmaf(vw[j], tp[j], acc);
            const float vv = requant<Elem>(silu_f(acc));
            L.v[ts][tt] = ts < tc ? vv : 0.f;
            if (ts < tc) {
                if (P.v_out)
                    reinterpret_cast<Elem*>(P.v_out)[(((size_t)b * A.T + ts) * A.Hv + hv) * A.Dv + row0 + tt] = from_float<Elem>(vv);
                if (ts == tc - 1) {
                    Elem* dst = reinterpret_cast<Elem*>(P.conv_out) + (size_t)b * keep * C + cv + tt;
#pragma unroll
                    for (int j = 1; j < KT; ++j)
                        dst[(size_t)(j - 1) * C] = from_float<Elem>(vw[j]);
                }
            }
        }
        if (tid < kChunkSteps) {
            const bool on = tid < tc;
            const float gv = requant<Elem>(gdn_decay(av, dtb, alog));
            const float be = requant<Elem>(sigmoid_f(bv));
            L.on[tid] = on;
            L.g[tid] = on ? gv : 1.f;
            L.beta[tid] = on ? be : 0.f;
            if (first_tile && on) {
                const size_t o = ((size_t)b * A.T + tid) * A.Hv + hv;
                if (P.g_out) reinterpret_cast<Elem*>(P.g_out)[o] = from_float<Elem>(gv);
                if (P.beta_out) reinterpret_cast<Elem*>(P.beta_out)[o] = from_float<Elem>(be);
            }
        }
    };

    // out = rmsNorm(y; weight, eps) * act(gate) for the 16 steps x Dv channels of this head: thread (t, j) takes
    // channels j, j + 16, ...; all of its loads go out together.
    auto finish_head = [&](auto elem_tag, int tc) {
        using Elem = decltype(elem_tag);
        constexpr int MAXI = kLayerFinishMaxDv / 16;
        const int t = ts < tc ? ts : tc - 1, tiles = (int)gridDim.x;
        const size_t row = (((size_t)b * A.T + t) * A.Hv + hv) * A.Dv;
        const Elem* yr = reinterpret_cast<const Elem*>(A.y) + row;
        const Elem* zr = reinterpret_cast<const Elem*>(P.fin_gate) + row;
        const Elem* wr = reinterpret_cast<const Elem*>(P.fin_weight);
        Elem* orow = reinterpret_cast<Elem*>(P.fin_out) + row;
        const float* part = reinterpret_cast<const float*>(orow);
        float yv[MAXI], zv[MAXI], wv[MAXI], pp[MAXI];
#pragma unroll
        for (int i = 0; i < MAXI; ++i) {
            const int d = tt + 16 * i, dl = d < A.Dv ? d : tt;
            yv[i] = load_agent(yr + dl);
            zv[i] = to_float(zr[dl]);
            wv[i] = to_float(wr[dl]);
            pp[i] = load_agent(part + (i < tiles ? i : 0));
        }
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < MAXI; ++i)
            if (i < tiles) ss = __fadd_rn(ss, pp[i]);
        const float inv = gdn_rms_inv(ss, A.Dv, P.fin_eps);
#pragma unroll
        for (int i = 0; i < MAXI; ++i) {
            const int d = tt + 16 * i;
            if (d < A.Dv && ts < tc) orow[d] = from_float<Elem>(gdn_gated_out(yv[i], inv, wv[i], zv[i], P.fin_silu != 0));
        }
    };

    // One chunk of up to 16 steps.  The first chunk (the only one of a verify block) is straight-line code ahead of
    // the loop over the rest: inside the loop the compiler hoists every invariant of the whole body above the first
    // load and carries waits round the back edge.
    auto run_chunk = [&](const int t0) {
        const int tc = (A.T - t0) < kChunkSteps ? (A.T - t0) : kChunkSteps;
        const bool last_chunk = t0 + kChunkSteps >= A.T;
        if constexpr (FUSED) {
            if constexpr (BF) stage_fused(bf16_t{}, tc);
            else if (A.in_dtype == DFLASH_F16) stage_fused(f16_t{}, tc);
            else stage_fused(float{}, tc);
        } else {
            if constexpr (BF) stage(bf16_t{}, t0, tc, t0 == 0);
            else if (A.in_dtype == DFLASH_F16) stage(f16_t{}, t0, tc, t0 == 0);
            else stage(float{}, t0, tc, t0 == 0);
        }
        __syncthreads();

        // ---- [S_0 ; k] x [k | q]^T: one 16x16 block per wave, over all DK channels ----
        //   wave 0: S_0 k_t -> p[r][t]     wave 1: S_0 q_t -> p[r][16+t]     wave 2: k_s.k_t -> a     wave 3: k_s.q_t -> c
        // A 16x16x4 fp32 MFMA takes lane l's a as row l%16, contraction index l/16 (b alike) and leaves lane l with
        // column l%16, rows 4*(l/16)+v; a float4 per lane feeds four MFMAs whose index sets are {16c + 4*(l/16) + e}.
        // No reduction across waves: the block's coefficients go from the accumulators straight into the tables.
        {
            const int n = lane % 16, kk = lane / 16;
            const int ws = __builtin_amdgcn_readfirstlane(w);
            constexpr int NB = DK / 16, PS = 4 * NB / 16;     // fp32 product: 4*NB MFMAs, 15 pieces
            constexpr int NK = DK / 32;                       // bf16 product: contraction steps of 32 channels
            float4 av[BF ? 1 : NB], bv[BF ? 1 : NB];
            bf16x8v ah[BF ? NK : 1], am[BF ? NK : 1], al[BF ? NK : 1], bb[BF ? NK : 1];
            if constexpr (BF) {
                // A 16x16x32 bf16 MFMA takes lane l's a as row l%16, channels 8*(l/16) .. +7 of the step (b alike).
                const uint16_t* bq = (ws & 1) ? &L.qb[n][8 * kk] : &L.kb[n][8 * kk];
                const int arow = ws < 2 ? 0 : 1;              // waves 2, 3 take k rows as their a operand
#pragma unroll
                for (int ks = 0; ks < NK; ++ks) {
                    bb[ks] = *reinterpret_cast<const bf16x8v*>(bq + 32 * ks);
                    ah[ks] = *reinterpret_cast<const bf16x8v*>((arow ? &L.kb[n][8 * kk] : &L.xs[0][n][8 * kk]) + 32 * ks);
                }
                if (ws < 2) {
#pragma unroll
                    for (int ks = 0; ks < NK; ++ks) {
                        am[ks] = *reinterpret_cast<const bf16x8v*>(&L.xs[1][n][8 * kk + 32 * ks]);
                        al[ks] = *reinterpret_cast<const bf16x8v*>(&L.xs[2][n][8 * kk + 32 * ks]);
                    }
                }
            } else {
                const float* ap = &L.x[(ws < 2 ? 0 : 16) + n][4 * kk];
                const float* bp = &L.y[(ws & 1 ? 16 : 0) + n][4 * kk];
#pragma unroll
                for (int c = 0; c < NB; ++c) {
                    av[c] = *reinterpret_cast<const float4*>(ap + 16 * c);
                    bv[c] = *reinterpret_cast<const float4*>(bp + 16 * c);
                }
            }
            float gj[kChunkSteps];
#pragma unroll
            for (int j4 = 0; j4 < kChunkSteps; j4 += 4) {
                const float4 g4 = *reinterpret_cast<const float4*>(&L.g[j4]);
                gj[j4] = g4.x; gj[j4 + 1] = g4.y; gj[j4 + 2] = g4.z; gj[j4 + 3] = g4.w;
            }
            // The decay products G[v] = g_{s+1} ... g_t of the lane's pairs (s, t) = (4*kk + v, n) (1 where s >= t)
            // are computed one factor at a time between the MFMAs: an instruction issued right behind an MFMA runs
            // while the matrix pipe works, one issued behind the last MFMA is on the critical path.  Piece i:
            // 0..11 the factors j = 4..15 of G[3], 12..14 one more factor for G[2], G[1], G[0], 15 the table
            // coefficients (a[s][t] = G k_s.k_t for s < t, c[s][t] = G k_s.q_t for s <= t, else 0).  All 16 decays
            // are read unconditionally and selected in registers.
            float G[4] = {1.f, 1.f, 1.f, 1.f}, coef[4];
            const int pitch = ws < 2 ? 33 : 16;
            float* const lds_f = reinterpret_cast<float*>(gdn_chunk_smem);
            int tbl = (int)((ws == 0 ? &L.p[0][0] : ws == 1 ? &L.p[0][16] : ws == 2 ? &L.a[0][0] : &L.c[0][0]) - &L.x[0][0]) +
                      4 * kk * pitch + n;               // float index of the lane's first table entry in LDS
            asm volatile("" : "+v"(tbl));
            auto g_piece = [&](int i) {
                if (i < 12) {
                    const int j = i + 4;
                    G[3] *= (j > 4 * kk + 3 && j <= n) ? gj[j] : 1.f;
                    asm volatile("" : "+v"(G[3]));   // pins the piece where it is written (the optimiser would sink it)
                } else if (i < 15) {
                    const int v = 14 - i;           // 2, 1, 0: g_{s+1} with s = 4*kk + v
                    float gs = 1.f;
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) gs = kk == q4 ? gj[4 * q4 + v + 1] : gs;
                    G[v] = G[v + 1] * (4 * kk + v + 1 <= n ? gs : 1.f);
                    asm volatile("" : "+v"(G[v]));
                } else if (i == 15) {               // what the block's entries are multiplied by on their way to the tables
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const int s = 4 * kk + v;
                        const bool keep = ws == 2 ? s < n : s <= n;
                        coef[v] = ws < 2 ? 1.f : (keep ? G[v] : 0.f);
                        asm volatile("" : "+v"(coef[v]));
                    }
                }
            };
            f32x4v acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (BF) {
                // With bf16 inputs the same product is exact on bf16 MFMAs: k and q are bf16, and the fp32 state
                // enters as three bf16 terms that add up to it bit for bit, so every partial product is exact in
                // fp32 and only the order of the additions differs from the fp32 MFMA.  3*NK MFMAs of 8 passes for
                // the state blocks, NK for the k blocks (whose waves also form the decay products), against 4*NB of
                // 8 passes in fp32.
                if (ws < 2) {
#pragma unroll
                    for (int ks = 0; ks < NK; ++ks) {
                        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[ks], bb[ks], acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(am[ks], bb[ks], acc1, 0, 0, 0);
                        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(al[ks], bb[ks], acc0, 0, 0, 0);
                    }
#pragma unroll
                    for (int v = 0; v < 4; ++v) coef[v] = 1.f;
                } else {
                    constexpr int PP = 16 / NK;         // pieces behind each MFMA
#pragma unroll
                    for (int ks = 0; ks < NK; ++ks) {
                        if (ks & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[ks], bb[ks], acc1, 0, 0, 0);
                        else acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ah[ks], bb[ks], acc0, 0, 0, 0);
#pragma unroll
                        for (int pc = 0; pc < PP; ++pc) g_piece(ks * PP + pc);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            if constexpr (!BF)
#pragma unroll
            for (int c = 0; c < NB; c += 2) {
                const float a0[4] = {av[c].x, av[c].y, av[c].z, av[c].w}, b0[4] = {bv[c].x, bv[c].y, bv[c].z, bv[c].w};
                const float a1[4] = {av[c + 1].x, av[c + 1].y, av[c + 1].z, av[c + 1].w};
                const float b1[4] = {bv[c + 1].x, bv[c + 1].y, bv[c + 1].z, bv[c + 1].w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = 4 * c + 2 * e;            // MFMA number; a piece behind every PS-th
                    acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[e], b0[e], acc0, 0, 0, 0);
                    g_piece(m % PS == 0 ? m / PS : 100);
                    __builtin_amdgcn_sched_barrier(0);
                    acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a1[e], b1[e], acc1, 0, 0, 0);
                    g_piece((m + 1) % PS == 0 ? (m + 1) / PS : 100);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // row 4*kk + v of the block: a state row (waves 0, 1) or step s (waves 2, 3); column n
#pragma unroll
            for (int v = 0; v < 4; ++v) lds_f[tbl + v * pitch] = coef[v] * (acc0[v] + acc1[v]);
            if (ws == 3) {
                if (kk == 0) L.gam[n] = gj[0] * G[0];
                if (n == kChunkSteps - 1) {
#pragma unroll
                    for (int v = 0; v < 4; ++v) L.w[4 * kk + v] = G[v];
                }
            }
        }
        __syncthreads();

        // ---- unit-triangular solve for delta: wave 0, one quad per state row, lane q owns steps 4q..4q+3 ----
        // The chain per step is multiply -> quad broadcast -> fused multiply-add; everything else (coefficients,
        // betas, the LDS stores of delta) is kept off it.
        if (w == 0) {
            const int r = lane / 4, q = lane % 4;
            float acc[4], bet[16], mine[4] = {0.f, 0.f, 0.f, 0.f};
            float4 arow[16];
            // every LDS read of the phase goes out before the first use (the compiler keeps the order written here:
            // with the start values first, the coefficient reads waited for them -- a second trip to LDS)
            float gm[4], pv[4], vv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) { gm[e] = L.gam[4 * q + e]; pv[e] = L.p[r][4 * q + e]; vv[e] = L.v[4 * q + e][r]; }
#pragma unroll
            for (int s = 0; s < 16; ++s) {
                arow[s] = *reinterpret_cast<const float4*>(&L.a[s][4 * q]);
                bet[s] = L.beta[s];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = fmaf(-gm[e], pv[e], vv[e]);
            SolveStep<0>::run(acc, arow, bet, mine, q);
#pragma unroll
            for (int e = 0; e < 4; ++e) L.dl[4 * q + e][r] = mine[e];
        }
        __syncthreads();

        // ---- read-out and tape: thread (t, r) ----
        {
            const int t = ts, r = tt;
            float yv = L.gam[t] * L.p[r][16 + t];
#pragma unroll
            for (int s = 0; s < kChunkSteps; ++s) yv = fmaf(L.c[s][t], L.dl[s][r], yv);
            yv = L.on[t] ? yv : 0.f;
            if (t < tc) {
                const uint32_t o = (((uint32_t)b * A.T + t0) * A.Hv + hv) * A.Dv + row0 + __umul24(t, v_step) + r;
                // Written through (agent scope): the 32- and 64-byte pieces then leave the L2s as they are produced
                // instead of waiting as partly dirty lines for the end-of-launch flush; the layer kernel's last
                // workgroup of a head re-reads y at that scope.
                store1_rt_agent(A.y, A.in_dtype, o, yv);
                __hip_atomic_store(A.tape + o, L.dl[t][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if constexpr (FUSED) {
                if (P.fin_gate) {          // this tile's share of sum(y^2) of step t, parked in the row of `out`
                    const float yq = requant_rt(A.in_dtype, yv);
                    const float sq = group_sum<16>(__fmul_rn(yq, yq));
                    if (r == 0 && t < tc) {
                        const size_t row = ((size_t)b * A.T + t) * A.Hv + hv;
                        const size_t esz = A.in_dtype == DFLASH_F32 ? 4 : 2;
                        __hip_atomic_store(reinterpret_cast<float*>(reinterpret_cast<unsigned char*>(P.fin_out) + row * A.Dv * esz) + blockIdx.x,
                                           sq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
        }

        // ---- state: S <- gam_15 S_0 + sum_s w_s delta_s (x) k_s, as 16x16x4 fp32 MFMAs ----
        // Lane l: a = row l%16, step 4*ks + l/16; b = column l%16 of the block; c = column l%16, rows 4*(l/16)+v.
        // Column n of MFMA e stands for channel base + E*n + e, so a lane ends up with E consecutive channels.
        {
            const int n = lane % 16, kk = lane / 16;
            const int base = w * 16 * E + E * n;
            const float gam_end = L.gam[kChunkSteps - 1];
            f32x4v cacc[E];
#pragma unroll
            for (int e = 0; e < E; ++e)
#pragma unroll
                for (int v = 0; v < 4; ++v) cacc[e][v] = gam_end * L.x[4 * kk + v][base + e];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const int s = 4 * ks + kk;
                const float av = L.w[s] * L.dl[s][n];
#pragma unroll
                for (int e = 0; e < E; ++e)
                    cacc[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, L.y[s][base + e], cacc[e], 0, 0, 0);
            }
            // first use of the pointer: down here (null when the caller does not want the post-block state)
            float* const s_out = A.state_out ? reinterpret_cast<float*>(A.state_out) + tile_off : nullptr;
            if (last_chunk) {
                // (layer kernel with the gated norm inside: the wave's y rows and sums of squares must be acknowledged
                //  before it counts itself in; waited for here, ahead of the state stores, the wait does not include
                //  those)
                if constexpr (FUSED)
                    if (P.fin_gate) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                // Written through (system scope) like y and the tape: the 2 MB of new state then drain while the launch
                // still runs instead of waiting dirty in the L2s for the end-of-launch flush (-0.7 % of a verify step).
                // A caller that rolls back from the tape whatever is accepted passes no state_out: nothing is stored.
                if (s_out != nullptr)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float* const ptr = s_out + (uint32_t)((4 * kk + v) * DK + base);
                    if constexpr (E == 1) {
                        asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"((uint64_t)ptr), "v"(cacc[0][v]) : "memory");
                    } else if constexpr (E == 2) {
                        const f32x2v val = {cacc[0][v], cacc[1][v]};
                        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1" ::"v"((uint64_t)ptr), "v"(val) : "memory");
                    } else {
                        static_assert(E == 1 || E == 2 || E == 4, "one store per row and lane");
                        const f32x4v val = {cacc[0][v], cacc[1][v], cacc[2][v], cacc[3][v]};
                        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"((uint64_t)ptr), "v"(val) : "memory");
                    }
                }
            } else {
                __syncthreads();           // every wave has read the old tile
                // One row at a time, with a compiler barrier between the rows: when the stores of rows 2 and 3 are
                // paired into one two-address LDS store (possible at DK = 64, where both offsets fit its 8-bit
                // fields) this compiler has emitted a wrong first offset.
#pragma unroll
                for (int v = 0; v < 4; ++v) {
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        L.x[4 * kk + v][base + e] = cacc[e][v];
                        if constexpr (BF) split3_bf16(cacc[e][v], L.xs[0][4 * kk + v][base + e], L.xs[1][4 * kk + v][base + e],
                                                      L.xs[2][4 * kk + v][base + e]);
                    }
                    asm volatile("" ::: "memory");
                }
                // the staging barrier of the next chunk orders these writes before their readers
            }
        }

        // ---- the layer's post-op, by the head's last workgroup ----
        // The hand-over between the workgroups of a head, in the order that makes it correct:
        //   1. store    every producer writes its y rows and sums of squares with agent-scope stores, which go through
        //               its XCD's L2 to the memory side that all XCDs share;
        //   2. ack      it waits until the memory side has acknowledged them (vmcnt(0), above, then the barrier below:
        //               every wave of the workgroup is past its own wait);
        //   3. count    only then does it add itself to the head's counter (an agent-scope read-modify-write, performed
        //               at that same shared level, hence ordered behind the acknowledged stores);
        //   4. observe  the workgroup whose own increment returns tiles - 1 has observed the increments of all others,
        //               each of which was issued behind that workgroup's acknowledged stores;
        //   5. load     and re-reads the head's y and the parked sums with agent-scope loads, which are served from that
        //               shared level and never from a copy its own XCD's caches may still hold; then it finishes the
        //               sums and writes `out`.
        // Steps 1-3 are a release of exactly the lines that are handed over (a release FENCE is a write-back of the whole
        // L2: 30 us per launch when it was tried, with the new state still stored write-back); 4-5 are the matching acquire, restricted
        // to the lines that are read.  An explicit invalidate in front of step 5 (the compiler's agent-scope acquire
        // fence, or a bare buffer_inv sc1) was measured at +3.4 us per launch (13.2 against 9.8 us) and adds nothing:
        // the only data that crosses workgroups is read by those agent-scope loads; gate and the norm weight are
        // inputs of the launch.  Nothing waits for anything: a workgroup that is not last is done.
        if constexpr (FUSED) {
            if (P.fin_gate) {
                __builtin_amdgcn_s_barrier();       // every wave is past its wait for the y rows (the state stores may be in flight)
                if (tid == 0) L.on[0] = __hip_atomic_fetch_add(P.arrivals + bh, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __syncthreads();
                const int arrived = L.on[0];
                // A count this launch cannot have produced: the array was not zero when the launch began (never
                // cleared, or left behind by a launch that did not finish).  `out` of this head is then not to be
                // trusted; say so where the caller can see it.
                if (arrived >= (int)gridDim.x && P.status && tid == 0) atomicOr(P.status, DFLASH_STATUS_LAYER_ARRIVALS);
                if (arrived != (int)gridDim.x - 1) return;
                if (tid == 0) __hip_atomic_store(P.arrivals + bh, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // as the next launch expects it
                if (A.in_dtype == DFLASH_BF16) finish_head(bf16_t{}, tc);
                else if (A.in_dtype == DFLASH_F16) finish_head(f16_t{}, tc);
                else finish_head(float{}, tc);
            }
        }
    };
    run_chunk(0);
    if constexpr (!FUSED)
        for (int t0 = kChunkSteps; t0 < A.T; t0 += kChunkSteps) run_chunk(t0);
}

// What stands between a wave's start and its loads -- the six input pointers and the sizes their addresses need --
// is passed as leading scalar arguments: the command processor hands those over in SGPRs when the wave starts (kernarg
// preload, 14 dwords at most, hence the sizes packed in pairs), so no load waits for a trip to the argument block.
// The rest of the arguments (outputs, mask, types) follow in the struct and are fetched while the loads are in flight.
template <bool HAS_MASK, int DK, bool BF>
__global__ __launch_bounds__(kThreads) void gated_delta_chunk_kernel(const void* state_in, const void* k, const void* q, const void* v,
                                                                     const void* g, const void* beta, uint32_t hv_dv, uint32_t hk_t,
                                                                     GdnArgs A) {
    A.state_in = state_in; A.k = k; A.q = q; A.v = v; A.g = g; A.beta = beta;
    A.Hv = (int)(hv_dv >> 16); A.Dv = (int)(hv_dv & 0xffffu); A.Hk = (int)(hk_t >> 16); A.T = (int)(hk_t & 0xffffu);
    A.group = (uint32_t)A.Hv / (uint32_t)A.Hk;
    A.group_magic = 0;                 // hk = hv / group is divided out below (scalar, once): the reciprocal did not fit the registers
    gdn_chunk_body<HAS_MASK, DK, false, BF>(A, GdnPrep{});
}

// One GatedDelta layer from its projections to the recurrence's outputs in one launch.
template <int DK, bool BF>
__global__ __launch_bounds__(kThreads) void gdn_layer_kernel(GdnArgs A, GdnPrep P) {
    gdn_chunk_body<false, DK, true, BF>(A, P);
}

// Whether the chunked kernels' 32-bit element offsets and 24-bit per-step strides cover this shape, and the
// reciprocal of the head group for them.
static bool chunk_index_setup(GdnArgs& A, int B, int Dk) {
    const uint64_t steps = (uint64_t)B * (uint64_t)(A.T > 0 ? A.T : 1);
    const uint64_t k_step = (uint64_t)A.Hk * Dk, v_step = (uint64_t)A.Hv * A.Dv, C = 2 * k_step + v_step;
    if (A.Hv > 65535 || B > 65535 || C >= (1u << 24) || steps * k_step >= (1ull << 31) || steps * v_step >= (1ull << 31)) return false;
    A.group = (uint32_t)(A.Hv / A.Hk);
    A.group_magic = A.group > 1 ? (uint32_t)(((1ull << 32) + A.group - 1) / A.group) : 0u;
    return true;
}

template <int DK>
static int launch_gdn_layer(hipStream_t st, const GdnArgs& A, const GdnPrep& P, int B) {
    const size_t lds = sizeof(GdnChunkLds<DK>);
    dim3 grid(A.Dv / kChunkRows, A.Hv, B);
    LaunchBracket br(DFLASH_KERNEL_GDN_LAYER, st);
    if (A.in_dtype == DFLASH_BF16) br.launch(gdn_layer_kernel<DK, true>, grid, dim3(kThreads), lds, A, P);
    else br.launch(gdn_layer_kernel<DK, false>, grid, dim3(kThreads), lds, A, P);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

template <int DK>
static int launch_gdn_chunk(hipStream_t st, const GdnArgs& A, int B) {
    const size_t lds = sizeof(GdnChunkLds<DK>);     // the attribute that allows it is set per device by gdn_device_setup()
    dim3 grid(A.Dv / kChunkRows, A.Hv, B);
    LaunchBracket br(DFLASH_KERNEL_GDN_FORWARD, st);
    const bool bf = A.in_dtype == DFLASH_BF16;
    const uint32_t hv_dv = ((uint32_t)A.Hv << 16) | (uint32_t)A.Dv, hk_t = ((uint32_t)A.Hk << 16) | (uint32_t)A.T;   // each below 2^16, checked by the caller
    if (A.mask && bf) br.launch(gated_delta_chunk_kernel<true, DK, true>, grid, dim3(kThreads), lds, A.state_in, A.k, A.q, A.v, A.g, A.beta, hv_dv, hk_t, A);
    else if (A.mask) br.launch(gated_delta_chunk_kernel<true, DK, false>, grid, dim3(kThreads), lds, A.state_in, A.k, A.q, A.v, A.g, A.beta, hv_dv, hk_t, A);
    else if (bf) br.launch(gated_delta_chunk_kernel<false, DK, true>, grid, dim3(kThreads), lds, A.state_in, A.k, A.q, A.v, A.g, A.beta, hv_dv, hk_t, A);
    else br.launch(gated_delta_chunk_kernel<false, DK, false>, grid, dim3(kThreads), lds, A.state_in, A.k, A.q, A.v, A.g, A.beta, hv_dv, hk_t, A);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

template <int DK>
static int gdn_chunk_setup() {
    const int lds = (int)sizeof(GdnChunkLds<DK>);
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)gated_delta_chunk_kernel<true, DK, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)gated_delta_chunk_kernel<true, DK, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)gated_delta_chunk_kernel<false, DK, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)gated_delta_chunk_kernel<false, DK, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)gdn_layer_kernel<DK, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)gdn_layer_kernel<DK, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    return DFLASH_OK;
}

int gdn_device_setup() {
    int rc = gdn_chunk_setup<64>();
    if (rc == DFLASH_OK) rc = gdn_chunk_setup<128>();
    if (rc == DFLASH_OK) rc = gdn_chunk_setup<256>();
    return rc;
}

template <typename StateT>
static int launch_gdn_state(hipStream_t st, const GdnArgs& A, int B, int g_ndim, int Dk) {
    const bool vec = g_ndim == 4;
#define DFLASH_GDN_CASE(DKV, LPRV)                                                                     \
    case DKV: {                                                                                        \
        dim3 grid((A.Dv + (kThreads / LPRV) - 1) / (kThreads / LPRV), B * A.Hv);                       \
        LaunchBracket br(DFLASH_KERNEL_GDN_FORWARD, st);                                               \
        if (vec && A.mask) br.launch(gated_delta_tape_kernel<StateT, true, true, DKV, LPRV>, grid, dim3(kThreads), 0, A);        \
        else if (vec) br.launch(gated_delta_tape_kernel<StateT, true, false, DKV, LPRV>, grid, dim3(kThreads), 0, A);            \
        else if (A.mask) br.launch(gated_delta_tape_kernel<StateT, false, true, DKV, LPRV>, grid, dim3(kThreads), 0, A);         \
        else br.launch(gated_delta_tape_kernel<StateT, false, false, DKV, LPRV>, grid, dim3(kThreads), 0, A);                    \
        DFLASH_HIP_TRY(hipGetLastError());                                                             \
        return DFLASH_OK;                                                                              \
    }
    switch (Dk) {
        DFLASH_GDN_CASE(32, 8)
        DFLASH_GDN_CASE(64, 16)
        DFLASH_GDN_CASE(96, 8)
        DFLASH_GDN_CASE(128, 16)
        DFLASH_GDN_CASE(160, 8)
        DFLASH_GDN_CASE(192, 16)
        DFLASH_GDN_CASE(224, 8)
        DFLASH_GDN_CASE(256, 16)
        default: break;
    }
#undef DFLASH_GDN_CASE
    set_error("gated delta: Dk=%d is not a multiple of 32 in [32, 256]", Dk);
    return DFLASH_UNSUPPORTED;
}

}  // namespace dflash

using namespace dflash;

extern "C" int dflash_tape_replay(void* stream, const void* tape, int tape_dtype, const void* k, const void* g,
                                  int in_dtype, int g_ndim, const void* state_in, void* state_out, int state_dtype,
                                  const void* mask, int mask_dtype, int B, int T, int Hk, int Hv, int Dk, int Dv) {
    const void* tp[1] = {tape};
    const void* kp[1] = {k};
    const void* gp[1] = {g};
    const void* si[1] = {state_in};
    void* so[1] = {state_out};
    return replay_common((hipStream_t)stream, 1, tp, tape_dtype, kp, gp, in_dtype, g_ndim, si, so, state_dtype,
                         mask, mask_dtype, T, nullptr, 0, B, T, Hk, Hv, Dk, Dv);
}

extern "C" int dflash_tape_replay_batched(void* stream, int n_layers, const void* const* tape, int tape_dtype,
                                          const void* const* k, const void* const* g, int in_dtype, int g_ndim,
                                          const void* const* state_in, void* const* state_out, int state_dtype,
                                          int steps, const int32_t* steps_dev, int skip_if_full, int B, int T_tape,
                                          int Hk, int Hv, int Dk, int Dv) {
    DFLASH_REQUIRE(tape && k && g && state_in && state_out, "tape replay (batched): null pointer array");
    return replay_common((hipStream_t)stream, n_layers, tape, tape_dtype, k, g, in_dtype, g_ndim, state_in, state_out,
                         state_dtype, nullptr, 0, steps, steps_dev, skip_if_full, B, T_tape, Hk, Hv, Dk, Dv);
}

extern "C" int dflash_accept_commit_replay_batched(void* stream, const uint32_t* verify_ids, const uint32_t* posterior,
                                                   int V, int32_t* start_inout, int32_t* out4, int n_layers,
                                                   const void* const* tape, int tape_dtype, const void* const* k,
                                                   const void* const* g, int in_dtype, int g_ndim,
                                                   const void* const* state_in, void* const* state_out,
                                                   int state_dtype, int skip_if_full, int B, int T_tape, int Hk, int Hv,
                                                   int Dk, int Dv) {
    DFLASH_REQUIRE(verify_ids && posterior && out4 && V >= 1, "accept + replay: bad acceptance arguments");
    DFLASH_REQUIRE(V - 1 <= T_tape, "accept + replay: %d verify positions for a tape of %d steps", V, T_tape);
    DFLASH_REQUIRE(tape && k && g && state_in && state_out, "accept + replay: null pointer array");
    FusedAccept acc;
    acc.verify_ids = verify_ids; acc.posterior = posterior; acc.start_inout = start_inout; acc.out4 = out4; acc.V = V;
    return replay_common((hipStream_t)stream, n_layers, tape, tape_dtype, k, g, in_dtype, g_ndim, state_in, state_out,
                         state_dtype, nullptr, 0, 0, nullptr, skip_if_full, B, T_tape, Hk, Hv, Dk, Dv, acc);
}

extern "C" int dflash_gated_delta_tape(void* stream, const void* q, const void* k, const void* v, const void* g,
                                       int g_ndim, const void* beta, int in_dtype, const void* state_in,
                                       void* state_out, int state_dtype, void* y, float* tape_out, const void* mask,
                                       int mask_dtype, int B, int T, int Hk, int Hv, int Dk, int Dv) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(B > 0 && T >= 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, "gated delta: non-positive dimension");
    DFLASH_REQUIRE(Hv % Hk == 0, "gated delta: Hv=%d is not a multiple of Hk=%d", Hv, Hk);
    DFLASH_REQUIRE(g_ndim == 3 || g_ndim == 4, "gated delta: g_ndim must be 3 or 4");
    DFLASH_REQUIRE(state_in, "gated delta: null state pointer");
    DFLASH_REQUIRE(state_in != state_out, "gated delta: state_in aliases state_out");
    DFLASH_REQUIRE(T == 0 || (q && k && v && g && beta && y && tape_out), "gated delta: null pointer");
    DFLASH_REQUIRE((long)B * Hv <= 65535, "gated delta: B*Hv too large for one launch");
    DFLASH_SUPPORTED(in_dtype == DFLASH_F32 || in_dtype == DFLASH_BF16 || in_dtype == DFLASH_F16, "gated delta: bad in_dtype %d", in_dtype);
    DFLASH_SUPPORTED(state_dtype == DFLASH_F32 || state_dtype == in_dtype, "gated delta: state dtype must be f32 or the input dtype");
    if (mask) DFLASH_REQUIRE(mask_dtype >= DFLASH_F32 && mask_dtype <= DFLASH_U8, "gated delta: bad mask dtype");

    GdnArgs A;
    A.q = q; A.k = k; A.v = v; A.g = g; A.beta = beta; A.mask = mask;
    A.state_in = state_in; A.state_out = state_out; A.y = y; A.tape = tape_out;
    A.in_dtype = in_dtype; A.mask_dtype = mask_dtype; A.T = T; A.Hk = Hk; A.Hv = Hv; A.Dv = Dv;
    if (state_dtype == DFLASH_F32 && g_ndim == 3 && Dv % kChunkRows == 0 && T > 0 && T < 65536 && Dv < 65536 && chunk_index_setup(A, B, Dk)) {
        // fp32 state with one decay per head and step: chunked form
        if (Dk == 64) return launch_gdn_chunk<64>((hipStream_t)stream, A, B);
        if (Dk == 128) return launch_gdn_chunk<128>((hipStream_t)stream, A, B);
        if (Dk == 256) return launch_gdn_chunk<256>((hipStream_t)stream, A, B);
    }
    DFLASH_SUPPORTED(state_out != nullptr, "gated delta: a call without state_out needs the chunked form (fp32 state, one decay "
                     "per head and step, Dk in {64, 128, 256}, Dv a multiple of 16, T >= 1)");
    switch (state_dtype) {
        case DFLASH_F32: return launch_gdn_state<float>((hipStream_t)stream, A, B, g_ndim, Dk);
        case DFLASH_BF16: return launch_gdn_state<bf16_t>((hipStream_t)stream, A, B, g_ndim, Dk);
        default: return launch_gdn_state<f16_t>((hipStream_t)stream, A, B, g_ndim, Dk);
    }
}

extern "C" int dflash_gdn_layer(void* stream, const void* mixed_qkv, const void* conv_state_in, const void* conv_weight,
                                const void* a_logits, const void* b_logits, const float* a_log, const float* dt_bias,
                                int in_dtype, float q_scale, float k_scale, float norm_eps, const void* state_in,
                                void* state_out, void* k_out, void* g_out, float* tape_out, void* conv_state_out,
                                void* y_out, const void* gate, const void* out_norm_weight, float out_norm_eps,
                                int gate_kind, void* out, int32_t* arrivals, void* q_out, void* v_out, void* beta_out,
                                int B, int T, int Hk, int Hv, int Dk, int Dv, int K) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(B > 0 && T > 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, "gdn_layer: non-positive dimension");
    DFLASH_REQUIRE(Hv % Hk == 0, "gdn_layer: Hv=%d is not a multiple of Hk=%d", Hv, Hk);
    DFLASH_REQUIRE(mixed_qkv && conv_weight && a_logits && b_logits && a_log && dt_bias, "gdn_layer: null input");
    DFLASH_REQUIRE(state_in && state_out && tape_out && y_out && conv_state_out, "gdn_layer: null output");
    DFLASH_REQUIRE(state_in != state_out, "gdn_layer: state_in aliases state_out");
    DFLASH_REQUIRE(conv_state_out != conv_state_in, "gdn_layer: conv_state_out aliases conv_state_in");
    DFLASH_REQUIRE(!gate || (out_norm_weight && out), "gdn_layer: a gate needs out_norm_weight and out");
    DFLASH_REQUIRE(!gate || out != y_out, "gdn_layer: out aliases y_out");
    DFLASH_REQUIRE(gate_kind == 0 || gate_kind == 1, "gdn_layer: gate_kind must be 0 (sigmoid) or 1 (silu)");
    DFLASH_REQUIRE((long)B * Hv <= 65535, "gdn_layer: B*Hv too large for one launch");
    DFLASH_SUPPORTED(in_dtype == DFLASH_F32 || in_dtype == DFLASH_BF16 || in_dtype == DFLASH_F16, "gdn_layer: bad in_dtype %d", in_dtype);
    DFLASH_SUPPORTED(K == kLayerTaps, "gdn_layer: conv kernel size %d (the one-launch layer is built for %d)", K, kLayerTaps);
    DFLASH_SUPPORTED(T <= kChunkSteps, "gdn_layer: T=%d above one chunk of %d steps", T, kChunkSteps);
    DFLASH_SUPPORTED(Dv % kChunkRows == 0 && (Dk == 64 || Dk == 128 || Dk == 256), "gdn_layer: Dk=%d / Dv=%d outside the chunked kernel", Dk, Dv);

    GdnArgs A;
    A.q = A.k = A.v = A.g = A.beta = A.mask = nullptr;
    A.state_in = state_in; A.state_out = state_out; A.y = y_out; A.tape = tape_out;
    A.in_dtype = in_dtype; A.mask_dtype = 0; A.T = T; A.Hk = Hk; A.Hv = Hv; A.Dv = Dv;
    DFLASH_SUPPORTED(chunk_index_setup(A, B, Dk), "gdn_layer: shape beyond the chunked kernel's 32-bit element offsets");
    GdnPrep P;
    P.x = mixed_qkv; P.conv_in = conv_state_in; P.weight = conv_weight; P.a = a_logits; P.b = b_logits;
    P.a_log = a_log; P.dt_bias = dt_bias; P.q_out = q_out; P.k_out = k_out; P.v_out = v_out; P.g_out = g_out;
    P.beta_out = beta_out; P.conv_out = conv_state_out; P.q_scale = q_scale; P.k_scale = k_scale; P.eps = norm_eps;
    P.C = 2 * Hk * Dk + Hv * Dv;
    // With a counter array the post-op runs inside the same launch; without one (or with a head dim the kernel's
    // post-op is not unrolled for) it is a second launch.
    // While the launch runs, the first Dv/16 floats of every row of `out` hold the row tiles' sums of squares, so the
    // in-launch norm needs `out` to be 4-byte aligned and disjoint from everything the last workgroup still reads
    // (gate, the norm weight); a caller that norms in place (out == gate) gets the second launch, which allows it.
    const size_t esz = in_dtype == DFLASH_F32 ? 4 : 2;
    const size_t out_bytes = (size_t)B * T * Hv * Dv * esz;
    auto overlaps = [&](const void* p, size_t bytes) {
        const uintptr_t a = (uintptr_t)out, b = (uintptr_t)p;
        return p && a < b + bytes && b < a + out_bytes;
    };
    DFLASH_REQUIRE(!gate || !overlaps(y_out, out_bytes), "gdn_layer: out overlaps y_out");
    const bool out_private = gate && (uintptr_t)out % 4 == 0 && !overlaps(gate, out_bytes) && !overlaps(out_norm_weight, (size_t)Dv * esz);
    const bool finish_inside = gate && arrivals && Dv <= kLayerFinishMaxDv && out_private;
    P.fin_gate = finish_inside ? gate : nullptr;
    P.fin_weight = finish_inside ? out_norm_weight : nullptr;
    P.fin_out = finish_inside ? out : nullptr;
    P.arrivals = finish_inside ? arrivals : nullptr;
    P.status = status_word();
    P.fin_eps = out_norm_eps;
    P.fin_silu = gate_kind;
    hipStream_t st = (hipStream_t)stream;
    if (Dk == 64) rc = launch_gdn_layer<64>(st, A, P, B);
    else if (Dk == 128) rc = launch_gdn_layer<128>(st, A, P, B);
    else rc = launch_gdn_layer<256>(st, A, P, B);
    if (rc || !gate || finish_inside) return rc;
    return dflash_gdn_finish(stream, y_out, gate, out_norm_weight, out, in_dtype, out_norm_eps, gate_kind, B, T, Hv, Dv);
}
