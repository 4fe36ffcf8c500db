// Block-causal batched GQA attention for the 16-token verify block, gfx950.
//
// The problem is a stream of K/V rows (2 KV heads, tens of thousands of keys)
// scored against a tiny query tile, so it is bound by HBM bandwidth.  The
// design follows from that:
//   * all query heads of a GQA group (up to 8 heads x 16 block rows = 128 rows)
//     share one pass over their KV head's rows, so K/V are read once;
//   * the key axis is split over enough workgroups to cover every CU (split-KV),
//     each writing an unnormalised partial (O, max, sum); a second small kernel
//     combines the splits and emits O and the logsumexp;
//   * K/V tiles of 64 keys are double-buffered in LDS (prefetch of tile i+1 is in
//     flight while tile i is multiplied); Q K^T and P V run on bf16/f16 MFMA
//     (v_mfma_f32_32x32x16) with the online softmax held in registers.
//
// MFMA operand conventions used below (wave of 64 lanes, c = lane % 32,
// h = lane / 32):  A (32 x 16) lane holds row c, k-elements 8h..8h+7;
// B (16 x 32) lane holds column c, k-elements 8h..8h+7;  C/D (32 x 32) lane
// holds column c, register v holds row 8*(v/4) + 4h + (v%4).
// Scores are produced transposed, S^T = K Q^T, so each lane owns ONE query row
// (column c) and the softmax statistics need a single exchange with lane c+32.
// The same trick gives O^T = V^T P^T, whose accumulators are again one query row
// per lane, so the running rescale is a per-lane scalar.  P^T is taken straight
// from the S^T accumulators: the 8 k-elements a lane feeds to the second MFMA are
// whatever keys its accumulators hold, and V^T is laid out in LDS in that same
// key order (bits 2 and 3 of the key index swapped), which is legal because a
// contraction may enumerate its index in any order.
//
// Semantics follow Sources/DFlash/DFlashKernels.swift:737-815 (entry), :563-649
// (partials: causal rule :614, GQA mapping :575) and :661-720 (combine).

#include "dflash_common.h"

namespace dflash {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(8))) float f32x8_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;   // one 16-byte global/LDS access

constexpr int kSdpaThreads = 256;
constexpr int kBN = 64;             // keys per tile
constexpr int kM = 16;              // block rows per head
constexpr int kHeadsPerWG = 8;      // query heads sharing one K/V pass
constexpr int kMaxSplits = 512;

struct Bf16Tag {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ vec8 pack(f32x8_t x) { return __builtin_convertvector(x, vec8); }
    static __device__ __forceinline__ uint16_t cvt(float x) { return f32_to_bf16_bits(x); }
};
struct F16Tag {
    typedef f16x8_t vec8;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ vec8 pack(f32x8_t x) { return __builtin_convertvector(x, vec8); }
    static __device__ __forceinline__ uint16_t cvt(float x) {
        _Float16 hf = (_Float16)x;
        return *reinterpret_cast<uint16_t*>(&hf);
    }
};

struct SdpaArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    float* part_o;   // [B*Hq*16, S, D]
    float* part_m;   // [B*Hq*16, S]   running max, log2 units
    float* part_l;   // [B*Hq*16, S]   sum of exp2
    const int32_t* kv_len_dev;
    int64_t kv_batch_stride, kv_head_stride;
    float scale_log2;   // scale * log2(e)
    int Hq, Hk, G, N, S, groups_per_kv;
};

template <int D> struct SdpaLds {
    static constexpr int KS = D + 8;           // K row stride, elements
    static constexpr int VS = kBN + 8;         // V^T row stride, elements
    static constexpr int K_BYTES = kBN * KS * 2;
    static constexpr int V_BYTES = D * VS * 2;
    static constexpr int STAGE = K_BYTES + V_BYTES;
    static constexpr int OS = D + 4;           // epilogue O row stride, floats
    static constexpr int EPI = 4 * 32 * OS * 4;
    static constexpr int BYTES = 2 * STAGE > EPI ? 2 * STAGE : EPI;
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Grid: x = split, y = kv head * groups_per_kv + head group, z = batch.
template <typename Tag, int D>
__global__ __launch_bounds__(kSdpaThreads, 1) void sdpa_partial_kernel(SdpaArgs A) {
    typedef typename Tag::vec8 vec8;
    typedef SdpaLds<D> L;
    constexpr int KSTEPS = D / 16;     // MFMA k-steps over the head dimension
    constexpr int DB = D / 32;         // 32-wide output blocks over the head dimension
    constexpr int KCH = (kBN * D / 8) / kSdpaThreads;   // 16-byte K chunks per thread per tile
    constexpr int VBLK = (kBN / 8) * (D / 8);           // 8x8 V blocks per tile
    static_assert(VBLK <= kSdpaThreads, "one V block per thread");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int split = blockIdx.x;
    const int hk = blockIdx.y / A.groups_per_kv;
    const int hg0 = (blockIdx.y % A.groups_per_kv) * kHeadsPerWG;   // first head of the group handled here
    const int b = blockIdx.z;
    const int hcount = (A.G - hg0) < kHeadsPerWG ? (A.G - hg0) : kHeadsPerWG;

    int Nb = A.kv_len_dev ? A.kv_len_dev[b] : A.N;
    Nb = Nb < kM ? kM : (Nb > A.N ? A.N : Nb);
    const int nt = (Nb + kBN - 1) / kBN;
    const int t_begin = (int)(((long)split * nt) / A.S);
    const int t_end = (int)(((long)(split + 1) * nt) / A.S);

    // this wave's query rows: heads 2*wave, 2*wave+1 of the group, 16 rows each
    const int head_in_group = 2 * wave + (c >> 4);
    const bool row_valid = head_in_group < hcount;
    const bool wave_active = 2 * wave < hcount;
    const int hq = hk * A.G + hg0 + head_in_group;
    const int qi = c & 15;
    const size_t row_id = ((size_t)b * A.Hq + hq) * kM + qi;   // valid only when row_valid

    if (t_begin >= t_end) {   // empty split: tell the combine kernel to ignore it
        if (row_valid && h == 0) {
            A.part_m[row_id * A.S + split] = -INFINITY;
            A.part_l[row_id * A.S + split] = 0.f;
        }
        return;
    }

    const uint16_t* kbase = A.k + (size_t)b * A.kv_batch_stride + (size_t)hk * A.kv_head_stride;
    const uint16_t* vbase = A.v + (size_t)b * A.kv_batch_stride + (size_t)hk * A.kv_head_stride;

    // ---- Q as B operands: column c = query row, k-elements 16*s + 8h .. +7 ----
    vec8 qreg[KSTEPS];
    {
        const uint16_t* qrow = A.q + row_id * D;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            u32x4_t u = {0u, 0u, 0u, 0u};
            if (row_valid) u = *reinterpret_cast<const u32x4_t*>(qrow + 16 * s + 8 * h);
            qreg[s] = __builtin_bit_cast(vec8, u);
        }
    }

    f32x16_t oacc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    u32x4_t kreg[KCH];
    u32x4_t vreg[8];
    // V block owned by this thread: 8 keys (one LDS position group) x 8 channels
    const int v_kg = tid & 7, v_dc = tid >> 3;
    const int v_keybase = 32 * (v_kg >> 2) + 16 * ((v_kg >> 1) & 1) + 4 * (v_kg & 1);

    auto load_tile = [&](int t) {
        const int key0 = t * kBN;
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
            const int id = tid + kSdpaThreads * j;
            int key = key0 + id / (D / 8);
            key = key < Nb ? key : Nb - 1;
            kreg[j] = *reinterpret_cast<const u32x4_t*>(kbase + (size_t)key * D + (id % (D / 8)) * 8);
        }
        if (VBLK == kSdpaThreads || tid < VBLK) {
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                int key = key0 + v_keybase + 8 * (r >> 2) + (r & 3);
                key = key < Nb ? key : Nb - 1;
                vreg[r] = *reinterpret_cast<const u32x4_t*>(vbase + (size_t)key * D + v_dc * 8);
            }
        }
    };
    auto store_tile = [&](int buf) {
        uint16_t* ks = reinterpret_cast<uint16_t*>(smem + buf * L::STAGE);
        uint16_t* vt = reinterpret_cast<uint16_t*>(smem + buf * L::STAGE + L::K_BYTES);
#pragma unroll
        for (int j = 0; j < KCH; ++j) {
            const int id = tid + kSdpaThreads * j;
            *reinterpret_cast<u32x4_t*>(ks + (id / (D / 8)) * L::KS + (id % (D / 8)) * 8) = kreg[j];
        }
        if (VBLK == kSdpaThreads || tid < VBLK) {
            // 8x8 transpose of 16-bit elements: row r of vreg is key r, we need channel dd -> 8 keys
#pragma unroll
            for (int dd = 0; dd < 8; ++dd) {
                u32x4_t w;
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const uint32_t lo = vreg[2 * p][dd >> 1];
                    const uint32_t hi = vreg[2 * p + 1][dd >> 1];
                    w[p] = (dd & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
                }
                *reinterpret_cast<u32x4_t*>(vt + (v_dc * 8 + dd) * L::VS + v_kg * 8) = w;
            }
        }
    };

    load_tile(t_begin);
    store_tile(0);
    __syncthreads();

    for (int t = t_begin; t < t_end; ++t) {
        const int buf = (t - t_begin) & 1;
        const bool more = (t + 1) < t_end;
        if (more) load_tile(t + 1);

        if (wave_active) {
            const uint16_t* ks = reinterpret_cast<const uint16_t*>(smem + buf * L::STAGE);
            const uint16_t* vt = reinterpret_cast<const uint16_t*>(smem + buf * L::STAGE + L::K_BYTES);

            // ---- S^T = K Q^T for the tile's two 32-key blocks ----
            f32x16_t sacc[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) sacc[kb][v] = 0.f;
#pragma unroll
                for (int s = 0; s < KSTEPS; ++s) {
                    const vec8 a = *reinterpret_cast<const vec8*>(ks + (32 * kb + c) * L::KS + 16 * s + 8 * h);
                    sacc[kb] = Tag::mfma(a, qreg[s], sacc[kb]);
                }
            }

            // ---- scale, causal mask, online softmax (log2 domain) ----
            const int key0 = t * kBN;
            const bool need_mask = (key0 + kBN) > (Nb - kM);
            const int last_visible = Nb - kM + qi;     // row qi sees keys 0 .. Nb-16+qi
            float mloc = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    float x = sacc[kb][v] * A.scale_log2;
                    if (need_mask) {
                        const int key = key0 + 32 * kb + 8 * (v >> 2) + 4 * h + (v & 3);
                        x = key <= last_visible ? x : -INFINITY;
                    }
                    sacc[kb][v] = x;
                    mloc = fmaxf(mloc, x);
                }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
            const float m_new = fmaxf(m_run, mloc);
            const float m_safe = m_new == -INFINITY ? 0.f : m_new;
            const float alpha = fast_exp2(m_run - m_safe);
            m_run = m_new;
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float p = fast_exp2(sacc[kb][v] - m_safe);
                    sacc[kb][v] = p;
                    psum += p;
                }
            l_run = l_run * alpha + psum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
                for (int i = 0; i < DB; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) oacc[i][v] *= alpha;
            }

            // ---- O^T += V^T P^T ----
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int ksub = 0; ksub < 2; ++ksub) {
                    f32x8_t pf;
#pragma unroll
                    for (int e = 0; e < 8; ++e) pf[e] = sacc[kb][8 * ksub + e];
                    const vec8 pb = Tag::pack(pf);
#pragma unroll
                    for (int i = 0; i < DB; ++i) {
                        const vec8 a = *reinterpret_cast<const vec8*>(vt + (32 * i + c) * L::VS + 32 * kb + 16 * ksub + 8 * h);
                        oacc[i] = Tag::mfma(a, pb, oacc[i]);
                    }
                }
        }

        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: partial statistics and O rows (through LDS for coalesced stores) ----
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (row_valid && h == 0) {
        A.part_m[row_id * A.S + split] = m_run;
        A.part_l[row_id * A.S + split] = l_tot;
    }
    if (wave_active) {
        float* os = reinterpret_cast<float*>(smem) + wave * 32 * L::OS;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4) {
                float4 o = make_float4(oacc[i][4 * v4], oacc[i][4 * v4 + 1], oacc[i][4 * v4 + 2], oacc[i][4 * v4 + 3]);
                *reinterpret_cast<float4*>(os + c * L::OS + 32 * i + 8 * v4 + 4 * h) = o;
            }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): LDS writes of this wave are visible to it
        for (int r = 0; r < 32; ++r) {
            const int head = 2 * wave + (r >> 4);
            if (head >= hcount) break;
            const size_t rid = ((size_t)b * A.Hq + hk * A.G + hg0 + head) * kM + (r & 15);
            float* dst = A.part_o + (rid * A.S + split) * D;
            for (int d = lane * 4; d < D; d += 256)
                *reinterpret_cast<float4*>(dst + d) = *reinterpret_cast<const float4*>(os + r * L::OS + d);
        }
    }
}

// One workgroup per output row (b, hq, i): merges the S partials.
struct CombineArgs {
    const float* part_o;
    const float* part_m;
    const float* part_l;
    uint16_t* out;
    float* lse;
    int S;
};

template <typename Tag, int D>
__global__ __launch_bounds__(kSdpaThreads) void sdpa_combine_kernel(CombineArgs A) {
    constexpr int TPG = D / 4;                     // threads spanning one row as float4
    constexpr int NG = kSdpaThreads / TPG;         // split groups walking the partials in parallel
    __shared__ float w_s[kMaxSplits];
    __shared__ float red_s[kSdpaThreads / 64];
    __shared__ float4 acc_s[NG][TPG];

    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const float* pm = A.part_m + row * A.S;
    const float* pl = A.part_l + row * A.S;

    // global max
    float mx = -INFINITY;
    for (int s = tid; s < A.S; s += kSdpaThreads) mx = fmaxf(mx, pm[s]);
    for (int o = 32; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if ((tid & 63) == 0) red_s[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red_s[0], red_s[1]), fmaxf(red_s[2], red_s[3]));
    __syncthreads();
    // weights and denominator
    float lsum = 0.f;
    for (int s = tid; s < A.S; s += kSdpaThreads) {
        const float m = pm[s];
        const float w = m == -INFINITY ? 0.f : fast_exp2(m - mx);
        w_s[s] = w;
        lsum += w * pl[s];
    }
    for (int o = 32; o >= 1; o >>= 1) lsum += __shfl_xor(lsum, o);
    if ((tid & 63) == 0) red_s[tid >> 6] = lsum;
    __syncthreads();
    lsum = red_s[0] + red_s[1] + red_s[2] + red_s[3];

    // weighted sum of the partial rows
    const int grp = tid / TPG, d4 = (tid % TPG) * 4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    const float* po = A.part_o + row * A.S * D;
    for (int s = grp; s < A.S; s += NG) {
        const float w = w_s[s];
        if (w == 0.f) continue;
        const float4 o = *reinterpret_cast<const float4*>(po + (size_t)s * D + d4);
        acc.x = fmaf(w, o.x, acc.x); acc.y = fmaf(w, o.y, acc.y);
        acc.z = fmaf(w, o.z, acc.z); acc.w = fmaf(w, o.w, acc.w);
    }
    acc_s[grp][tid % TPG] = acc;
    __syncthreads();
    if (tid < TPG) {
        float4 r = acc_s[0][tid];
#pragma unroll
        for (int gI = 1; gI < NG; ++gI) {
            const float4 o = acc_s[gI][tid];
            r.x += o.x; r.y += o.y; r.z += o.z; r.w += o.w;
        }
        const float inv = lsum == 0.f ? 1.f : 1.f / lsum;   // divide unless the sum is 0 (DFlashKernels.swift:711)
        uint2 pk;
        pk.x = (uint32_t)Tag::cvt(r.x * inv) | ((uint32_t)Tag::cvt(r.y * inv) << 16);
        pk.y = (uint32_t)Tag::cvt(r.z * inv) | ((uint32_t)Tag::cvt(r.w * inv) << 16);
        *reinterpret_cast<uint2*>(A.out + row * D + tid * 4) = pk;
    }
    if (tid == 0 && A.lse) A.lse[row] = (mx + log2f(lsum)) * 0.6931471805599453f;
}

// ---- host side -------------------------------------------------------------

static int choose_splits(int B, int Hk, int groups_per_kv, int N) {
    const int nt = (N + kBN - 1) / kBN;
    const int cus = num_compute_units();
    const int per = B * Hk * groups_per_kv;
    int S = (cus + per - 1) / per;
    if (S > nt) S = nt;
    if (S > kMaxSplits) S = kMaxSplits;
    if (S < 1) S = 1;
    return S;
}

static size_t ws_layout(int B, int Hq, int S, int D, size_t* off_m, size_t* off_l) {
    const size_t rows = (size_t)B * Hq * kM;
    size_t o = rows * S * D * sizeof(float);
    o = (o + 255) & ~(size_t)255;
    *off_m = o;
    o += rows * S * sizeof(float);
    o = (o + 255) & ~(size_t)255;
    *off_l = o;
    o += rows * S * sizeof(float);
    return (o + 255) & ~(size_t)255;
}

template <typename Tag, int D>
static int launch_sdpa(hipStream_t st, const SdpaArgs& A, const CombineArgs& C, int B) {
    typedef SdpaLds<D> L;
    static_assert(L::BYTES <= 160 * 1024, "tile buffers must fit the 160 KB LDS of a gfx950 CU");
    auto kern = sdpa_partial_kernel<Tag, D>;
    // Raise the dynamic LDS limit above the 64 KB default, once per process.
    static const hipError_t attr_rc =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, L::BYTES);
    DFLASH_HIP_TRY(attr_rc);
    dim3 grid(A.S, A.Hk * A.groups_per_kv, B);
    hipLaunchKernelGGL(kern, grid, dim3(kSdpaThreads), L::BYTES, st, A);
    DFLASH_HIP_TRY(hipGetLastError());
    hipLaunchKernelGGL((sdpa_combine_kernel<Tag, D>), dim3(B * A.Hq * kM), dim3(kSdpaThreads), 0, st, C);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

}  // namespace dflash

using namespace dflash;

extern "C" size_t dflash_sdpa_workspace_bytes(int B, int Hq, int Hk, int M, int N, int D) {
    if (B <= 0 || Hq <= 0 || Hk <= 0 || M != kM || N < M || D <= 0 || Hq % Hk != 0) return 0;
    if (ensure_init()) return 0;
    const int G = Hq / Hk;
    const int groups = (G + kHeadsPerWG - 1) / kHeadsPerWG;
    size_t om, ol;
    return ws_layout(B, Hq, choose_splits(B, Hk, groups, N), D, &om, &ol);
}

extern "C" int dflash_sdpa_block_causal(void* stream, const void* q, const void* k, const void* v, void* out,
                                        float* lse, int dtype, float scale, int B, int Hq, int Hk, int M, int N,
                                        int D, int64_t kv_batch_stride, int64_t kv_head_stride,
                                        const int32_t* kv_len_dev, void* workspace, size_t workspace_bytes) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(q && k && v && out, "sdpa: null pointer");
    DFLASH_REQUIRE(B > 0 && Hq > 0 && Hk > 0 && N > 0 && D > 0, "sdpa: non-positive dimension");
    // the reference's guards (DFlashKernels.swift:755-758)
    DFLASH_SUPPORTED(M == kM, "sdpa: query length %d is not 16", M);
    DFLASH_SUPPORTED(dtype == DFLASH_BF16 || dtype == DFLASH_F16, "sdpa: dtype must be bf16 or f16");
    DFLASH_SUPPORTED(D == 128 || D == 256, "sdpa: head dim %d is not 128 or 256", D);
    DFLASH_SUPPORTED(Hq % Hk == 0, "sdpa: Hq=%d is not a multiple of Hk=%d", Hq, Hk);
    DFLASH_REQUIRE(N >= M, "sdpa: N=%d must include the %d block tokens", N, M);
    DFLASH_REQUIRE(kv_head_stride >= (int64_t)N * D, "sdpa: kv_head_stride smaller than N*D");
    DFLASH_REQUIRE(kv_batch_stride >= (int64_t)(Hk - 1) * kv_head_stride + (int64_t)N * D, "sdpa: kv_batch_stride too small");
    DFLASH_REQUIRE(kv_head_stride % 8 == 0 && kv_batch_stride % 8 == 0, "sdpa: kv strides must be multiples of 8 elements");
    DFLASH_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16 == 0, "sdpa: q/k/v/out must be 16-byte aligned");
    DFLASH_REQUIRE(B <= 65535 && (long)Hq * 2 <= 65535, "sdpa: batch or head count too large for one launch");

    const int G = Hq / Hk;
    const int groups = (G + kHeadsPerWG - 1) / kHeadsPerWG;
    const int S = choose_splits(B, Hk, groups, N);
    size_t om, ol;
    const size_t need = ws_layout(B, Hq, S, D, &om, &ol);
    DFLASH_REQUIRE(workspace && workspace_bytes >= need, "sdpa: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    DFLASH_REQUIRE((uintptr_t)workspace % 256 == 0, "sdpa: workspace must be 256-byte aligned");

    SdpaArgs A;
    A.q = (const uint16_t*)q; A.k = (const uint16_t*)k; A.v = (const uint16_t*)v;
    A.part_o = (float*)workspace;
    A.part_m = (float*)((char*)workspace + om);
    A.part_l = (float*)((char*)workspace + ol);
    A.kv_len_dev = kv_len_dev;
    A.kv_batch_stride = kv_batch_stride; A.kv_head_stride = kv_head_stride;
    A.scale_log2 = scale * 1.4426950408889634f;
    A.Hq = Hq; A.Hk = Hk; A.G = G; A.N = N; A.S = S; A.groups_per_kv = groups;
    CombineArgs C;
    C.part_o = A.part_o; C.part_m = A.part_m; C.part_l = A.part_l;
    C.out = (uint16_t*)out; C.lse = lse; C.S = S;

    hipStream_t st = (hipStream_t)stream;
    if (dtype == DFLASH_BF16) return D == 256 ? launch_sdpa<Bf16Tag, 256>(st, A, C, B) : launch_sdpa<Bf16Tag, 128>(st, A, C, B);
    return D == 256 ? launch_sdpa<F16Tag, 256>(st, A, C, B) : launch_sdpa<F16Tag, 128>(st, A, C, B);
}
