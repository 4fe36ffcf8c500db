// Shared helpers for the gfx950 DFlash kernels: element types, error plumbing,
// wave-level reductions.  Internal to the library.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dflash_hip.h"
#include "../../include/dflash_profile.h"

namespace dflash {

// ---- error plumbing ------------------------------------------------------

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define DFLASH_HIP_TRY(expr)                                                        \
    do {                                                                            \
        hipError_t _e = (expr);                                                     \
        if (_e != hipSuccess) {                                                     \
            ::dflash::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                                __FILE__, __LINE__);                                \
            return -(int)_e;                                                        \
        }                                                                           \
    } while (0)

#define DFLASH_REQUIRE(cond, ...)              \
    do {                                       \
        if (!(cond)) {                         \
            ::dflash::set_error(__VA_ARGS__);  \
            return DFLASH_INVALID;             \
        }                                      \
    } while (0)

#define DFLASH_SUPPORTED(cond, ...)            \
    do {                                       \
        if (!(cond)) {                         \
            ::dflash::set_error(__VA_ARGS__);  \
            return DFLASH_UNSUPPORTED;         \
        }                                      \
    } while (0)

int ensure_init();           // per-device one-time setup; 0 or negative hip error
int32_t* status_word();      // the device int32 registered with dflash_set_status_word(), or null
int num_compute_units();     // of the current device (cached)

// Per-device setup of the kernel files, run once per device by ensure_init() under its mutex with that
// device current: the dynamic-LDS limits of the kernels that need more than 64 KB (a function attribute is
// per device, and setting it is not legal while a stream is being captured, so it is done here and never
// at launch time).
int sdpa_device_setup();
int gdn_device_setup();

// Launches one kernel.  When the thread was armed by dflash_profile_next_launch() for this kernel id,
// the caller's events are attached to the dispatch itself (hipExtLaunchKernelGGL), so their elapsed
// time is the kernel's own begin-to-end duration, as a profiler reports it, not a bracket around it.
struct LaunchBracket {
    hipStream_t stream;
    hipEvent_t start, stop;
    LaunchBracket(int kernel_id, hipStream_t st);
    template <typename K, typename... Args>
    void launch(K kern, dim3 grid, dim3 block, size_t lds, Args... args) {
        if (start) hipExtLaunchKernelGGL(kern, grid, block, lds, stream, start, stop, 0, args...);
        else hipLaunchKernelGGL(kern, grid, block, lds, stream, args...);
    }
    LaunchBracket(const LaunchBracket&) = delete;
    LaunchBracket& operator=(const LaunchBracket&) = delete;
};

inline int dtype_size(int dt) {
    switch (dt) {
        case DFLASH_F32: return 4;
        case DFLASH_BF16: return 2;
        case DFLASH_F16: return 2;
        case DFLASH_U8: return 1;
        default: return 0;
    }
}

// n / d by one multiply: magic = floor(2^32 / d) (as close as 32 bits allow for d == 1) gives a quotient that is
// at most one too small for any n < 2^32; one comparison corrects it.  An integer division by a run-time value is
// some twenty-five dependent instructions, which matters ahead of a kernel's first load.
inline uint32_t fast_div_magic(uint32_t d) { return d <= 1 ? 0xFFFFFFFFu : (uint32_t)((1ull << 32) / d); }
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t d, uint32_t magic) {
    uint32_t q = __umulhi(n, magic);
    q += (n - q * d) >= d;
    return q;
}

// ---- element types -------------------------------------------------------

struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t x) { return (float)x.v; }

// round-to-nearest-even, NaN stays NaN: the hardware convert of gfx950 (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}

template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) { return bf16_t{f32_to_bf16_bits(f)}; }
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f) { return f16_t{(_Float16)f}; }

// value after a round trip through T (identity for float)
template <typename T> __device__ __forceinline__ float requant(float f) { return to_float(from_float<T>(f)); }
template <> __device__ __forceinline__ float requant<float>(float f) { return f; }

// requant of four values at once; bf16 converts in pairs (one v_cvt_pk_bf16_f32 per two values, the same rounding)
template <typename T> __device__ __forceinline__ float4 requant4(float4 v) {
    return make_float4(requant<T>(v.x), requant<T>(v.y), requant<T>(v.z), requant<T>(v.w));
}
template <> __device__ __forceinline__ float4 requant4<bf16_t>(float4 v) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t lo = {v.x, v.y}, hi = {v.z, v.w};
    const uint32_t a = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2_t));
    const uint32_t b = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2_t));
    return make_float4(__uint_as_float(a << 16), __uint_as_float(a & 0xffff0000u), __uint_as_float(b << 16), __uint_as_float(b & 0xffff0000u));
}

// 4 consecutive elements -> float4 (pointer aligned to 4 elements)
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    uint2 u = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                       __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ float4 load4(const f16_t* p) {
    return make_float4((float)p[0].v, (float)p[1].v, (float)p[2].v, (float)p[3].v);
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16_bits(v.x) | ((uint32_t)f32_to_bf16_bits(v.y) << 16);
    u.y = (uint32_t)f32_to_bf16_bits(v.z) | ((uint32_t)f32_to_bf16_bits(v.w) << 16);
    *reinterpret_cast<uint2*>(p) = u;
}
__device__ __forceinline__ void store4(f16_t* p, float4 v) {
    p[0].v = (_Float16)v.x; p[1].v = (_Float16)v.y; p[2].v = (_Float16)v.z; p[3].v = (_Float16)v.w;
}

// ---- GatedDelta layer formulas shared by the pre-op kernel and the one-launch layer kernel ----
// Both kernels must round identically, so the expressions live here once.
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(__expf(z)); }
// 1 / (1 + e^-z) with the hardware exponential and reciprocal (about 2 ulp)
__device__ __forceinline__ float sigmoid_f(float z) { return __builtin_amdgcn_rcpf(1.f + __expf(-z)); }
// The product is pinned as a float so that a following narrowing convert cannot be merged with the multiply
// (a merged multiply-convert rounds once, the two-step form twice: kernels that must agree bit for bit would not).
__device__ __forceinline__ float silu_f(float y) {
    float r = y * sigmoid_f(y);
    asm("" : "+v"(r));
    return r;
}
// g = exp(-exp(A_log) * softplus(a + dt_bias)) (Sources/SwiftLM/KimiLinearDFlash.swift:390)
__device__ __forceinline__ float gdn_decay(float a_logit, float dt_bias, float a_log) {
    const float z = a_logit + dt_bias;
    return __expf(-__expf(a_log) * softplus_f(z));
}
// scale * rsqrt(mean(x^2) + eps) for a head of `dim` channels whose squares sum to `sumsq` (:362-363)
__device__ __forceinline__ float gdn_norm_scale(float sumsq, int dim, float eps, float scale) {
    return scale * rsqrtf(sumsq / (float)dim + eps);
}

// The layer's gated output norm, out = rmsNorm(y; weight, eps) * act(gate) (KimiLinearDFlash.swift:377-378), is
// computed by the post-op kernel and by the one-launch layer kernel; both sum the squares of a row the same way --
// 16 consecutive channels by group_sum<16>, then those sums added one after the other from channel 0 up, starting
// from 0 -- and share these two expressions, so that they agree bit for bit.
__device__ __forceinline__ float gdn_rms_inv(float sumsq, int dim, float eps) { return rsqrtf(sumsq / (float)dim + eps); }
__device__ __forceinline__ float gdn_gated_out(float y, float inv, float w, float z, bool silu_gate) {
    const float act = silu_gate ? z * sigmoid_f(z) : sigmoid_f(z);
    return y * inv * w * act;
}

// mask element of run-time type -> "this step runs"
__device__ __forceinline__ bool mask_on(const void* mask, int mask_dtype, int idx) {
    float m;
    switch (mask_dtype) {
        case DFLASH_F32: m = reinterpret_cast<const float*>(mask)[idx]; break;
        case DFLASH_BF16: m = to_float(reinterpret_cast<const bf16_t*>(mask)[idx]); break;
        case DFLASH_F16: m = to_float(reinterpret_cast<const f16_t*>(mask)[idx]); break;
        default: m = (float)reinterpret_cast<const uint8_t*>(mask)[idx]; break;
    }
    return m > 0.5f;
}

// ---- cross-lane sums inside one 16-lane DPP row ---------------------------
// Data-parallel-primitive controls of GFX9: quad_perm, row_half_mirror, row_mirror.

// One wave.  Leading-match count = index of the first mismatch (n if none);
// equals sum(cumprod(drafted == posterior)) (DFlashRuntime.swift:139-141).
__device__ __forceinline__ int leading_matches(const uint32_t* a, const uint32_t* b, int n) {
    const int lane = threadIdx.x;
    int first = n;
    for (int base = 0; base < n; base += 64) {
        const int i = base + lane;
        const bool mismatch = i < n && a[i] != b[i];
        const unsigned long long bal = __builtin_amdgcn_ballot_w64(mismatch);
        if (bal) { first = base + __builtin_ctzll(bal); break; }   // uniform
    }
    return first;
}


template <int CTRL> __device__ __forceinline__ float dpp_add(float x) {
    int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false);
    return x + __int_as_float(y);
}

// Sum over groups of LANES (4, 8 or 16) consecutive lanes; every lane of the
// group receives the total.
template <int LANES> __device__ __forceinline__ float group_sum(float x) {
    static_assert(LANES == 4 || LANES == 8 || LANES == 16, "group must fit one DPP row");
    x = dpp_add<0xB1>(x);                          // quad_perm [1,0,3,2]
    x = dpp_add<0x4E>(x);                          // quad_perm [2,3,0,1]
    if (LANES >= 8) x = dpp_add<0x141>(x);         // row_half_mirror
    if (LANES >= 16) x = dpp_add<0x140>(x);        // row_mirror
    return x;
}

// Sum over groups of LANES (a power of two, 4..64) consecutive lanes as a butterfly: neighbours first (lane bit 0),
// then bit 1, and so on; every lane of the group receives the total.  Floating-point addition is commutative, so
// every lane holds the same bits, and two kernels that both use this order agree bit for bit.  Bits 0-3 stay inside
// a 16-lane DPP row; bit 4 and bit 5 use gfx950's v_permlane16_swap / v_permlane32_swap.
template <int LANES> __device__ __forceinline__ float butterfly_sum(float x) {
    static_assert(LANES == 4 || LANES == 8 || LANES == 16 || LANES == 32 || LANES == 64, "group size");
    x = group_sum<(LANES > 16 ? 16 : LANES)>(x);
    if (LANES >= 32) {
        auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        x = __fadd_rn(__uint_as_float(r[0]), __uint_as_float(r[1]));
    }
    if (LANES >= 64) {
        auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
        x = __fadd_rn(__uint_as_float(r[0]), __uint_as_float(r[1]));
    }
    return x;
}

// The same butterfly for the maximum (order does not matter for a maximum; this is only the fast path: DPP and
// lane swaps instead of six LDS permutes).
template <int CTRL> __device__ __forceinline__ float dpp_max(float x) {
    int y = __builtin_amdgcn_update_dpp(__float_as_int(x), __float_as_int(x), CTRL, 0xf, 0xf, false);
    return fmaxf(x, __int_as_float(y));
}
__device__ __forceinline__ float wave_max(float x) {
    x = dpp_max<0xB1>(x);
    x = dpp_max<0x4E>(x);
    x = dpp_max<0x141>(x);
    x = dpp_max<0x140>(x);
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    auto r2 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r2[0]), __uint_as_float(r2[1]));
}

}  // namespace dflash
