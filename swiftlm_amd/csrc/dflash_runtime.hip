// Library plumbing (init, error text) and the small integer/byte kernels of the
// verify step: acceptance length, accept/commit bookkeeping, conv-state
// rebuild, KV append.

#include <stdarg.h>
#include <string.h>

#include <mutex>

#include <type_traits>

#include <atomic>

#include "dflash_common.h"

namespace dflash {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

// A kernel that does nothing, launched with a caller-chosen grid, block and dynamic LDS size: what a launch of
// that shape costs on this device before any work is done (the floor under every kernel of a verify step).
__global__ void empty_kernel() {}

static std::mutex g_init_mu;
static int g_cus[64];
static bool g_ready[64];

int ensure_init() {
    int dev = 0;
    DFLASH_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) { set_error("device index %d out of range", dev); return DFLASH_INVALID; }
    std::lock_guard<std::mutex> lock(g_init_mu);
    if (g_ready[dev]) return 0;
    hipDeviceProp_t prop;
    DFLASH_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        set_error("this library is built for gfx950 only; device %d is %s", dev, prop.gcnArchName);
        return DFLASH_UNSUPPORTED;
    }
    DFLASH_HIP_TRY(hipFuncSetAttribute((const void*)empty_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    int rc = sdpa_device_setup();
    if (rc) return rc;
    rc = gdn_device_setup();
    if (rc) return rc;
    g_cus[dev] = prop.multiProcessorCount;
    g_ready[dev] = true;
    return 0;
}

int num_compute_units() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64 || !g_ready[dev]) return 256;
    return g_cus[dev];
}

// ---- measurement hook --------------------------------------------------------

struct ArmedBracket { hipEvent_t start = nullptr, stop = nullptr; };
static thread_local ArmedBracket g_bracket[DFLASH_KERNEL_COUNT];

LaunchBracket::LaunchBracket(int kernel_id, hipStream_t st) : stream(st), start(nullptr), stop(nullptr) {
    ArmedBracket& a = g_bracket[kernel_id];
    start = a.start;
    stop = a.stop;
    a.start = a.stop = nullptr;
}

// ---- acceptance ------------------------------------------------------------

__global__ __launch_bounds__(64) void match_acceptance_kernel(const uint32_t* drafted, const uint32_t* posterior,
                                                              int n, int32_t* out) {
    const int acc = leading_matches(drafted, posterior, n);
    if (threadIdx.x == 0) out[0] = acc;
}

__global__ __launch_bounds__(64) void accept_commit_kernel(const uint32_t* verify_ids, const uint32_t* posterior, int V,
                                                           int32_t* start_inout, int32_t* out4) {
    // drafted = verify_ids[1:], posterior[:V-1]  (DFlashRuntime.swift:525-530)
    const int acc = V > 1 ? leading_matches(verify_ids + 1, posterior, V - 1) : 0;
    if (threadIdx.x == 0) {
        const int commit = 1 + acc;                       // :544
        out4[0] = acc;
        out4[1] = commit;
        out4[2] = (int32_t)posterior[acc];                // :547
        int start = commit;
        if (start_inout) { start += *start_inout; *start_inout = start; }   // :571
        out4[3] = start;
    }
}

// ---- greedy tokens over the verify logits, fused with the acceptance ---------

// DFlashRuntime.greedyTokensWithMask (DFlashRuntime.swift:118-128): argmax over the vocabulary of
// where(mask, -1e9 rounded to the logits' type, logits); the first index wins a tie.  HBM-bound
// (T x V logits read once).  Two launches: greedy_partial_kernel (grid x = chunks of kArgmaxChunk
// vocabulary entries, y = row) leaves a (best value, best index) pair per workgroup in the
// workspace; greedy_finish_kernel (one workgroup) reduces them, writes posterior[T] and, when asked
// to, does the cycle's acceptance bookkeeping (accept_commit_kernel above).  A single launch with a
// "last workgroup finishes" ticket was measured slower: the device-scope fences and the atomic it
// needs add more dependent memory round trips than the second launch costs.
constexpr int kArgmaxThreads = 256;
constexpr int kArgmaxChunk = 8192;
constexpr int kArgmaxMaxRows = 1024;
constexpr int kArgmaxMaxPartials = 4096;   // T * chunks the last workgroup can hold in LDS

struct GreedyArgs {
    const void* logits;            // [T, V]
    const uint8_t* suppress;       // [V] non-zero = suppressed, or null
    const uint32_t* verify_ids;    // [T], or null: tokens only
    int32_t* start_inout;
    int32_t* out4;
    uint32_t* posterior;           // [T]
    float* part_val;               // [T, chunks]
    int32_t* part_idx;             // [T, chunks]
    int T, V, chunks;
};

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

template <typename Elem>
__global__ __launch_bounds__(kArgmaxThreads) void greedy_partial_kernel(GreedyArgs A) {
    __shared__ float val_s[kArgmaxThreads / 64];
    __shared__ int idx_s[kArgmaxThreads / 64];
    const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
    const Elem* lrow = reinterpret_cast<const Elem*>(A.logits) + (size_t)row * A.V;
    const float floor_v = to_float(from_float<Elem>(-1e9f));      // MLXArray(-1e9, dtype: logits.dtype) (:124)
    const int v0 = chunk * kArgmaxChunk;
    const int v1 = (v0 + kArgmaxChunk) < A.V ? (v0 + kArgmaxChunk) : A.V;

    float best = -INFINITY;
    int besti = 0x7fffffff;
    constexpr int VEC = 16 / sizeof(Elem);                        // elements per 16-byte load
    typedef typename std::conditional<VEC == 8, uint64_t, uint32_t>::type MaskWord;   // VEC mask bytes at once
    const bool aligned = ((size_t)row * A.V * sizeof(Elem)) % 16 == 0 && (uintptr_t)A.logits % 16 == 0 &&
                         (uintptr_t)A.suppress % sizeof(MaskWord) == 0;
    if (aligned) {
        for (int i = v0 + tid * VEC; i < v1; i += kArgmaxThreads * VEC) {
            if (i + VEC <= v1) {
                Elem e[VEC];
                *reinterpret_cast<uint4*>(e) = *reinterpret_cast<const uint4*>(lrow + i);
                const MaskWord mw = A.suppress ? *reinterpret_cast<const MaskWord*>(A.suppress + i) : (MaskWord)0;
#pragma unroll
                for (int u = 0; u < VEC; ++u) {
                    float x = to_float(e[u]);
                    if ((mw >> (8 * u)) & 0xff) x = floor_v;
                    if (x > best) { best = x; besti = i + u; }    // ascending indices: '>' keeps the first maximum
                }
            } else {
                for (int j = i; j < v1; ++j) {
                    float x = to_float(lrow[j]);
                    if (A.suppress && A.suppress[j]) x = floor_v;
                    if (x > best) { best = x; besti = j; }
                }
            }
        }
    } else {
        for (int j = v0 + tid; j < v1; j += kArgmaxThreads) {
            float x = to_float(lrow[j]);
            if (A.suppress && A.suppress[j]) x = floor_v;
            if (x > best) { best = x; besti = j; }
        }
    }
    for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(best, o);
        const int oi = __shfl_xor(besti, o);
        if (better(ov, oi, best, besti)) { best = ov; besti = oi; }
    }
    if ((tid & 63) == 0) { val_s[tid >> 6] = best; idx_s[tid >> 6] = besti; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < kArgmaxThreads / 64; ++w)
            if (better(val_s[w], idx_s[w], best, besti)) { best = val_s[w]; besti = idx_s[w]; }
        A.part_val[row * A.chunks + chunk] = best;
        A.part_idx[row * A.chunks + chunk] = besti;
    }
}

__global__ __launch_bounds__(kArgmaxThreads) void greedy_finish_kernel(GreedyArgs A) {
    const int tid = threadIdx.x;
    // every thread fetches partials at once (one memory round trip), then one wave reduces them per
    // row out of LDS
    __shared__ float pv_s[kArgmaxMaxPartials];
    __shared__ int pi_s[kArgmaxMaxPartials];
    const int total = A.T * A.chunks;
    for (int p = tid; p < total; p += kArgmaxThreads) {
        pv_s[p] = A.part_val[p];
        pi_s[p] = A.part_idx[p];
    }
    __syncthreads();
    if (tid >= 64) return;
    __shared__ uint32_t post_s[kArgmaxMaxRows];
    for (int r = tid; r < A.T; r += 64) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int c = 0; c < A.chunks; ++c)
            if (better(pv_s[r * A.chunks + c], pi_s[r * A.chunks + c], bv, bi)) { bv = pv_s[r * A.chunks + c]; bi = pi_s[r * A.chunks + c]; }
        // a row of NaNs never compares greater than anything: token 0, like a scan that starts at index 0
        const uint32_t tok = bi == 0x7fffffff ? 0u : (uint32_t)bi;
        post_s[r] = tok;
        A.posterior[r] = tok;
    }
    if (A.verify_ids) {
        __builtin_amdgcn_s_waitcnt(0xc07f);                       // lgkmcnt(0): this wave's LDS writes have landed
        __builtin_amdgcn_wave_barrier();
        const int acc = A.T > 1 ? leading_matches(A.verify_ids + 1, post_s, A.T - 1) : 0;
        if (tid == 0) {
            const int commit = 1 + acc;
            A.out4[0] = acc;
            A.out4[1] = commit;
            A.out4[2] = (int32_t)post_s[acc];
            int start = commit;
            if (A.start_inout) { start += *A.start_inout; *A.start_inout = start; }
            A.out4[3] = start;
        }
    }
}

// ---- conv-state rebuild ----------------------------------------------------

// out[b, j, :] = concat(snapshot [B,keep,C], qkv [B,T,C])[b, s + j, :], 16-byte pieces.
__global__ __launch_bounds__(256) void rebuild_conv_kernel(const uint4* snap, const uint4* qkv, uint4* out, int keep,
                                                           int T, int C16, int steps, const int32_t* steps_dev,
                                                           int32_t* status) {
    int s = steps_dev ? *steps_dev : steps;
    if (status && (s < 0 || s > T) && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x == 0)
        atomicOr(status, DFLASH_STATUS_CONV_STEPS);
    s = s < 0 ? 0 : s;
    const int b = blockIdx.z, j = blockIdx.y;
    const int src = s + j;
    if (src >= keep + T) return;     // clamped slice end (RecurrentRollbackCache.swift:156)
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < C16; i += gridDim.x * blockDim.x) {
        uint4 val;
        if (src < keep) val = snap ? snap[((size_t)b * keep + src) * C16 + i] : make_uint4(0, 0, 0, 0);
        else val = qkv[((size_t)b * T + (src - keep)) * C16 + i];
        out[((size_t)b * keep + j) * C16 + i] = val;
    }
}

// ---- KV append -------------------------------------------------------------

__global__ __launch_bounds__(256) void kv_append_kernel(uint4* k_cache, uint4* v_cache, const uint4* k_new,
                                                        const uint4* v_new, int Hk, int M, int D16, long batch_stride16,
                                                        long head_stride16, int offset, const int32_t* offset_dev,
                                                        int capacity, int32_t* new_len_dev, int32_t* status) {
    int off = offset_dev ? *offset_dev : offset;
    if (off < 0 || off + M > capacity) {          // never write outside the cache
        if (status && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) atomicOr(status, DFLASH_STATUS_APPEND_RANGE);
        return;
    }
    if (new_len_dev && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *new_len_dev = off + M;
    const int bh = blockIdx.y;
    const int b = bh / Hk, hk = bh % Hk;
    const int per = M * D16;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < per; i += gridDim.x * blockDim.x) {
        const size_t dst = (size_t)b * batch_stride16 + (size_t)hk * head_stride16 + (size_t)off * D16 + i;
        const size_t src = (size_t)bh * per + i;
        k_cache[dst] = k_new[src];
        v_cache[dst] = v_new[src];
    }
}

}  // namespace dflash

using namespace dflash;

static std::atomic<int32_t*> g_status_word{nullptr};
int32_t* dflash::status_word() { return g_status_word.load(std::memory_order_acquire); }
extern "C" int dflash_set_status_word(int32_t* status_dev) {
    g_status_word.store(status_dev, std::memory_order_release);
    return DFLASH_OK;
}

extern "C" int dflash_version(void) { return 100; }
extern "C" const char* dflash_last_error(void) { return g_err; }
extern "C" int dflash_init(void) { return ensure_init(); }

extern "C" int dflash_profile_next_launch(int kernel_id, void* start_event, void* stop_event) {
    DFLASH_REQUIRE(kernel_id >= 0 && kernel_id < DFLASH_KERNEL_COUNT, "profile_next_launch: bad kernel id %d", kernel_id);
    DFLASH_REQUIRE((start_event == nullptr) == (stop_event == nullptr), "profile_next_launch: pass both events or neither");
    g_bracket[kernel_id].start = (hipEvent_t)start_event;
    g_bracket[kernel_id].stop = (hipEvent_t)stop_event;
    return DFLASH_OK;
}

extern "C" int dflash_profile_empty_launch(void* stream, int grid_x, int grid_y, int grid_z, int threads, int lds_bytes) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(grid_x >= 1 && grid_y >= 1 && grid_z >= 1 && grid_y <= 65535 && grid_z <= 65535, "empty launch: bad grid");
    DFLASH_REQUIRE(threads >= 64 && threads <= 1024 && threads % 64 == 0, "empty launch: threads=%d is not a multiple of 64 in [64, 1024]", threads);
    DFLASH_REQUIRE(lds_bytes >= 0 && lds_bytes <= 160 * 1024, "empty launch: lds_bytes=%d outside [0, 160 KB]", lds_bytes);
    LaunchBracket br(DFLASH_KERNEL_EMPTY, (hipStream_t)stream);
    br.launch(empty_kernel, dim3(grid_x, grid_y, grid_z), dim3(threads), (size_t)lds_bytes);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

extern "C" int dflash_match_acceptance_length(void* stream, const uint32_t* drafted, const uint32_t* posterior, int n,
                                              int32_t* out) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(out && n >= 0 && (n == 0 || (drafted && posterior)), "match_acceptance_length: bad arguments");
    hipLaunchKernelGGL(match_acceptance_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, drafted, posterior, n, out);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

extern "C" int dflash_accept_commit(void* stream, const uint32_t* verify_ids, const uint32_t* posterior, int V,
                                    int32_t* start_inout, int32_t* out4) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(verify_ids && posterior && out4 && V >= 1, "accept_commit: bad arguments");
    hipLaunchKernelGGL(accept_commit_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, verify_ids, posterior, V,
                       start_inout, out4);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

static size_t greedy_ws_layout(int T, int V, size_t* off_idx) {
    const size_t chunks = (size_t)(V + kArgmaxChunk - 1) / kArgmaxChunk;
    size_t o = (size_t)T * chunks * sizeof(float);
    o = (o + 255) & ~(size_t)255;
    *off_idx = o;
    o += (size_t)T * chunks * sizeof(int32_t);
    return (o + 255) & ~(size_t)255;
}

extern "C" size_t dflash_greedy_workspace_bytes(int T, int V) {
    if (T <= 0 || V <= 0) return 0;
    size_t a;
    return greedy_ws_layout(T, V, &a);
}

static int greedy_common(void* stream, const void* logits, int dtype, int T, int V, const uint8_t* suppress,
                         const uint32_t* verify_ids, int32_t* start_inout, int32_t* out4, uint32_t* posterior,
                         void* workspace, size_t workspace_bytes) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(logits && posterior && T >= 1 && V >= 1, "greedy tokens: bad arguments");
    DFLASH_SUPPORTED(T <= kArgmaxMaxRows, "greedy tokens: T=%d rows exceed %d", T, kArgmaxMaxRows);
    DFLASH_SUPPORTED((long)T * ((V + kArgmaxChunk - 1) / kArgmaxChunk) <= kArgmaxMaxPartials,
                     "greedy tokens: T=%d x V=%d needs more than %d partial results", T, V, kArgmaxMaxPartials);
    DFLASH_SUPPORTED(dtype == DFLASH_F32 || dtype == DFLASH_BF16 || dtype == DFLASH_F16, "greedy tokens: bad dtype %d", dtype);
    size_t oi;
    const size_t need = greedy_ws_layout(T, V, &oi);
    DFLASH_REQUIRE(workspace && workspace_bytes >= need, "greedy tokens: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    DFLASH_REQUIRE((uintptr_t)workspace % 256 == 0, "greedy tokens: workspace must be 256-byte aligned");
    GreedyArgs A;
    A.logits = logits; A.suppress = suppress; A.verify_ids = verify_ids; A.start_inout = start_inout; A.out4 = out4;
    A.posterior = posterior;
    A.part_val = (float*)workspace;
    A.part_idx = (int32_t*)((char*)workspace + oi);
    A.T = T; A.V = V; A.chunks = (V + kArgmaxChunk - 1) / kArgmaxChunk;
    dim3 grid(A.chunks, T);
    hipStream_t st = (hipStream_t)stream;
    {
        LaunchBracket br(DFLASH_KERNEL_GREEDY_PARTIAL, st);
        if (dtype == DFLASH_F32) br.launch(greedy_partial_kernel<float>, grid, dim3(kArgmaxThreads), 0, A);
        else if (dtype == DFLASH_BF16) br.launch(greedy_partial_kernel<bf16_t>, grid, dim3(kArgmaxThreads), 0, A);
        else br.launch(greedy_partial_kernel<f16_t>, grid, dim3(kArgmaxThreads), 0, A);
    }
    DFLASH_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL(greedy_finish_kernel, dim3(1), dim3(kArgmaxThreads), 0, st, A);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

extern "C" int dflash_greedy_tokens_with_mask(void* stream, const void* logits, int dtype, int T, int V,
                                              const uint8_t* suppress_mask, uint32_t* tokens_out, void* workspace,
                                              size_t workspace_bytes) {
    return greedy_common(stream, logits, dtype, T, V, suppress_mask, nullptr, nullptr, nullptr, tokens_out, workspace,
                         workspace_bytes);
}

extern "C" int dflash_greedy_accept_commit(void* stream, const void* logits, int dtype, int T, int V,
                                           const uint8_t* suppress_mask, const uint32_t* verify_ids,
                                           int32_t* start_inout, int32_t* out4, uint32_t* posterior_out,
                                           void* workspace, size_t workspace_bytes) {
    DFLASH_REQUIRE(verify_ids && out4, "greedy accept: null pointer");
    return greedy_common(stream, logits, dtype, T, V, suppress_mask, verify_ids, start_inout, out4, posterior_out,
                         workspace, workspace_bytes);
}

extern "C" int dflash_rebuild_conv_state(void* stream, const void* snapshot_conv, const void* tape_qkv, void* out, int B,
                                         int keep, int T, int C, int elem_bytes, int accepted_steps,
                                         const int32_t* steps_dev) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(tape_qkv && out && B > 0 && keep > 0 && T >= 0 && C > 0, "rebuild_conv_state: bad arguments");
    DFLASH_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "rebuild_conv_state: element size must be 2 or 4");
    DFLASH_REQUIRE(accepted_steps >= 0, "rebuild_conv_state: negative accepted_steps");
    DFLASH_REQUIRE(((long)C * elem_bytes) % 16 == 0, "rebuild_conv_state: row of %d x %d bytes is not a multiple of 16", C, elem_bytes);
    DFLASH_REQUIRE(((uintptr_t)snapshot_conv | (uintptr_t)tape_qkv | (uintptr_t)out) % 16 == 0, "rebuild_conv_state: pointers must be 16-byte aligned");
    DFLASH_REQUIRE(keep <= 65535 && B <= 65535, "rebuild_conv_state: keep or B too large");
    {
        const size_t win = (size_t)B * keep * C * elem_bytes, tape_bytes = (size_t)B * T * C * elem_bytes;
        const uintptr_t o = (uintptr_t)out, q = (uintptr_t)tape_qkv, sn = (uintptr_t)snapshot_conv;
        DFLASH_REQUIRE(!(o < q + tape_bytes && q < o + win) && !(sn && o < sn + win && sn < o + win),
                       "rebuild_conv_state: out overlaps an input");
    }
    const int C16 = (int)(((long)C * elem_bytes) / 16);
    dim3 grid((C16 + 255) / 256, keep, B);
    hipLaunchKernelGGL(rebuild_conv_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint4*)snapshot_conv,
                       (const uint4*)tape_qkv, (uint4*)out, keep, T, C16, accepted_steps, steps_dev, status_word());
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

extern "C" int dflash_kv_append(void* stream, void* k_cache, void* v_cache, const void* k_new, const void* v_new, int B,
                                int Hk, int M, int D, int elem_bytes, int64_t kv_batch_stride, int64_t kv_head_stride,
                                int offset, const int32_t* offset_dev, int capacity, int32_t* new_len_dev) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(k_cache && v_cache && k_new && v_new, "kv_append: null pointer");
    DFLASH_REQUIRE(B > 0 && Hk > 0 && M > 0 && D > 0 && capacity > 0, "kv_append: non-positive dimension");
    DFLASH_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "kv_append: element size must be 2 or 4");
    DFLASH_REQUIRE(((long)D * elem_bytes) % 16 == 0, "kv_append: row bytes must be a multiple of 16");
    DFLASH_REQUIRE((kv_batch_stride * elem_bytes) % 16 == 0 && (kv_head_stride * elem_bytes) % 16 == 0, "kv_append: strides must be 16-byte multiples");
    DFLASH_REQUIRE(kv_head_stride >= (int64_t)capacity * D, "kv_append: head stride smaller than capacity*D");
    DFLASH_REQUIRE(kv_batch_stride >= (int64_t)(Hk - 1) * kv_head_stride + (int64_t)capacity * D, "kv_append: batch stride too small");
    DFLASH_REQUIRE(offset_dev || (offset >= 0 && offset + M <= capacity), "kv_append: rows [%d, %d) outside capacity %d", offset, offset + M, capacity);
    DFLASH_REQUIRE(((uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)k_new | (uintptr_t)v_new) % 16 == 0, "kv_append: pointers must be 16-byte aligned");
    DFLASH_REQUIRE((long)B * Hk <= 65535, "kv_append: B*Hk too large");
    const int D16 = (int)(((long)D * elem_bytes) / 16);
    dim3 grid((M * D16 + 255) / 256, B * Hk);
    hipLaunchKernelGGL(kv_append_kernel, grid, dim3(256), 0, (hipStream_t)stream, (uint4*)k_cache, (uint4*)v_cache,
                       (const uint4*)k_new, (const uint4*)v_new, Hk, M, D16, (long)(kv_batch_stride * elem_bytes / 16),
                       (long)(kv_head_stride * elem_bytes / 16), offset, offset_dev, capacity, new_len_dev, status_word());
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}
