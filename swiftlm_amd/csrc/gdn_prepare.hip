// GatedDelta pre-ops for the verify block: short causal depthwise conv + SiLU over the
// concatenated q|k|v channels, per-head RMS normalisation of q and k, the gate formulas, and
// the conv window the rollback cache keeps.  One launch produces everything
// dflash_gated_delta_tape consumes.
//
// Semantics follow the layer code around the recurrence in
// Sources/SwiftLM/KimiLinearDFlash.swift: ShortConv1d :274-293 (window = concat(state, x),
// new state = its last K-1 rows), q/k normalisation :362-363, gates :390-391.
//
// The op moves a few hundred KB, so it is bound by launch latency and one round trip to HBM:
// every workgroup covers one head of one step (its Dk or Dv channels), each thread one
// channel, so all loads of a thread (K window rows, K taps) are issued at once.

#include "dflash_common.h"

namespace dflash {

struct PrepareArgs {
    const void* x;            // [B,T,C]
    const void* state_in;     // [B,K-1,C] or null
    const void* weight;       // [C,K]
    const void* a;            // [B,T,Hv] or [B,T,Hv,Dk]
    const void* b;            // [B,T,Hv]
    const float* a_log;       // [Hv]
    const float* dt_bias;     // [Hv] or [Hv*Dk]
    void *q, *k, *v, *g, *beta, *state_out;
    float q_scale, k_scale, eps;
    int in_dtype, vec_gate;
    int T, Hk, Hv, Dk, Dv, K, C;
};

constexpr int kPrepMaxTaps = 8;

// Grid: x = head block (Hk q heads, Hk k heads, Hv v heads, then gate blocks), y = t, z = b.
// Block: max(Dk, Dv) threads rounded up to a multiple of 64.
template <typename Elem>
__global__ void gdn_prepare_kernel(PrepareArgs A) {
    __shared__ float red_s[16];
    const int tid = threadIdx.x, t = blockIdx.y, b = blockIdx.z;
    int hb = blockIdx.x;
    const int n_conv = 2 * A.Hk + A.Hv;
    if (hb >= n_conv) {
        // ---- gates: g = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b) (:390-391) ----
        const size_t bt = (size_t)b * A.T + t;
        if (A.vec_gate) {
            const int h = hb - n_conv;                       // one block per value head, one thread per channel
            if (tid < A.Dk) {
                const size_t o = (bt * A.Hv + h) * A.Dk + tid;
                reinterpret_cast<Elem*>(A.g)[o] = from_float<Elem>(
                    gdn_decay(to_float(reinterpret_cast<const Elem*>(A.a)[o]), A.dt_bias[h * A.Dk + tid], A.a_log[h]));
            }
            if (tid == 0) {
                const size_t o = bt * A.Hv + h;
                reinterpret_cast<Elem*>(A.beta)[o] = from_float<Elem>(sigmoid_f(to_float(reinterpret_cast<const Elem*>(A.b)[o])));
            }
        } else {
            for (int h = tid; h < A.Hv; h += blockDim.x) {   // a single block
                const size_t o = bt * A.Hv + h;
                reinterpret_cast<Elem*>(A.g)[o] = from_float<Elem>(
                    gdn_decay(to_float(reinterpret_cast<const Elem*>(A.a)[o]), A.dt_bias[h], A.a_log[h]));
                reinterpret_cast<Elem*>(A.beta)[o] = from_float<Elem>(sigmoid_f(to_float(reinterpret_cast<const Elem*>(A.b)[o])));
            }
        }
        return;
    }

    // ---- conv + SiLU on one head's channels ----
    const int kind = hb < A.Hk ? 0 : (hb < 2 * A.Hk ? 1 : 2);        // q, k, v
    const int head = kind == 0 ? hb : (kind == 1 ? hb - A.Hk : hb - 2 * A.Hk);
    const int width = kind == 2 ? A.Dv : A.Dk;
    const int c0 = kind == 0 ? head * A.Dk : (kind == 1 ? A.Hk * A.Dk + head * A.Dk : 2 * A.Hk * A.Dk + head * A.Dv);
    const bool on = tid < width;
    const int c = c0 + (on ? tid : 0);
    const Elem* x = reinterpret_cast<const Elem*>(A.x) + (size_t)b * A.T * A.C;
    const Elem* st = reinterpret_cast<const Elem*>(A.state_in);
    const Elem* w = reinterpret_cast<const Elem*>(A.weight) + (size_t)c * A.K;
    const int keep = A.K - 1;

    // window row j of step t is row t + j of concat(state [keep rows], x [T rows])
    float win[kPrepMaxTaps], tap[kPrepMaxTaps];
#pragma unroll
    for (int j = 0; j < kPrepMaxTaps; ++j) {
        win[j] = 0.f;
        tap[j] = 0.f;
        if (j < A.K && on) {
            const int r = t + j;
            if (r >= keep) win[j] = to_float(x[(size_t)(r - keep) * A.C + c]);
            else if (st) win[j] = to_float(st[((size_t)b * keep + r) * A.C + c]);
            tap[j] = to_float(w[j]);
        }
    }
    float y = 0.f;
#pragma unroll
    for (int j = 0; j < kPrepMaxTaps; ++j) y = fmaf(win[j], tap[j], y);
    y = silu_f(y);                                                   // silu (:291)

    // the new conv window: the last K-1 rows of the concatenation (:292), i.e. rows 1..K-1 of the
    // window of the last step
    if (t == A.T - 1 && on) {
        Elem* so = reinterpret_cast<Elem*>(A.state_out) + (size_t)b * keep * A.C + c;
#pragma unroll
        for (int j = 1; j < kPrepMaxTaps; ++j)
            if (j < A.K) so[(size_t)(j - 1) * A.C] = from_float<Elem>(win[j]);
    }

    if (kind == 2) {
        if (on) reinterpret_cast<Elem*>(A.v)[(((size_t)b * A.T + t) * A.Hv + head) * A.Dv + tid] = from_float<Elem>(y);
        return;
    }
    // ---- q, k: scale * x * rsqrt(mean(x^2) + eps) over the head (:362-363) ----
    // The squares are summed pairwise, neighbours first (channel bit 0, then bit 1, ...), which is the order
    // the one-launch layer kernel reproduces with four channels per lane: both give the same bits.
    float ss = butterfly_sum<64>(on ? __fmul_rn(y, y) : 0.f);
    if ((tid & 63) == 0) red_s[tid >> 6] = ss;
    __syncthreads();
    const int nw = (int)(blockDim.x >> 6);
    float tot;
    if (nw == 4) tot = __fadd_rn(__fadd_rn(red_s[0], red_s[1]), __fadd_rn(red_s[2], red_s[3]));
    else {
        tot = red_s[0];
        for (int i = 1; i < nw; ++i) tot = __fadd_rn(tot, red_s[i]);
    }
    const float scale = gdn_norm_scale(tot, A.Dk, A.eps, kind == 0 ? A.q_scale : A.k_scale);
    if (on) {
        Elem* dst = reinterpret_cast<Elem*>(kind == 0 ? A.q : A.k);
        dst[(((size_t)b * A.T + t) * A.Hk + head) * A.Dk + tid] = from_float<Elem>(y * scale);
    }
}

// ---- post-op: out = rmsNorm(y; weight, eps) * act(gate) per head --------------------------
// (KimiLinearDFlash.swift:377-378: oNorm(out) * sigmoid(gate); RMSNorm with a learned weight of
// headDim elements, :341.)  One wave per (b, t, head) row of Dv elements.
struct FinishArgs {
    const void* y;        // [rows, Dv]
    const void* gate;     // [rows, Dv]
    const void* weight;   // [Dv]
    void* out;            // [rows, Dv]
    float eps;
    int rows, Dv, silu_gate;
};

template <typename Elem>
__global__ __launch_bounds__(256) void gdn_finish_kernel(FinishArgs A) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= A.rows) return;
    const Elem* y = reinterpret_cast<const Elem*>(A.y) + (size_t)row * A.Dv;
    const Elem* gt = reinterpret_cast<const Elem*>(A.gate) + (size_t)row * A.Dv;
    const Elem* wt = reinterpret_cast<const Elem*>(A.weight);
    Elem* out = reinterpret_cast<Elem*>(A.out) + (size_t)row * A.Dv;
    constexpr int kMaxPer = 16;                      // Dv <= 1024
    float v[kMaxPer], part[kMaxPer];
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) {
        const int d = lane + 64 * i;
        v[i] = d < A.Dv ? to_float(y[d]) : 0.f;
        part[i] = group_sum<16>(__fmul_rn(v[i], v[i]));      // channels 64 i + 16 (lane / 16) .. + 15
    }
    // the 16-channel sums in channel order (group g of pass i holds channels 64 i + 16 g ..)
    const int tiles = (A.Dv + 15) / 16;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) {
        if (4 * i >= tiles) break;                   // uniform
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float p = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(part[i]), 16 * g));
            if (4 * i + g < tiles) ss = __fadd_rn(ss, p);
        }
    }
    const float inv = gdn_rms_inv(ss, A.Dv, A.eps);
#pragma unroll
    for (int i = 0; i < kMaxPer; ++i) {
        const int d = lane + 64 * i;
        if (d < A.Dv) out[d] = from_float<Elem>(gdn_gated_out(v[i], inv, to_float(wt[d]), to_float(gt[d]), A.silu_gate != 0));
    }
}

}  // namespace dflash

using namespace dflash;

extern "C" int dflash_gdn_finish(void* stream, const void* y, const void* gate, const void* norm_weight, void* out,
                                 int in_dtype, float norm_eps, int gate_kind, int B, int T, int Hv, int Dv) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(y && gate && norm_weight && out, "gdn_finish: null pointer");
    DFLASH_REQUIRE(B > 0 && T > 0 && Hv > 0 && Dv > 0, "gdn_finish: non-positive dimension");
    DFLASH_REQUIRE(gate_kind == 0 || gate_kind == 1, "gdn_finish: gate_kind must be 0 (sigmoid) or 1 (silu)");
    DFLASH_SUPPORTED(Dv <= 1024, "gdn_finish: head dim above 1024");
    DFLASH_SUPPORTED(in_dtype == DFLASH_F32 || in_dtype == DFLASH_BF16 || in_dtype == DFLASH_F16, "gdn_finish: bad dtype %d", in_dtype);
    const long rows = (long)B * T * Hv;
    DFLASH_REQUIRE(rows <= 0x7fffffffL, "gdn_finish: too many rows");
    FinishArgs A;
    A.y = y; A.gate = gate; A.weight = norm_weight; A.out = out; A.eps = norm_eps;
    A.rows = (int)rows; A.Dv = Dv; A.silu_gate = gate_kind;
    dim3 grid((unsigned)((rows + 3) / 4));
    hipStream_t st = (hipStream_t)stream;
    LaunchBracket br(DFLASH_KERNEL_GDN_FINISH, st);
    if (in_dtype == DFLASH_F32) br.launch(gdn_finish_kernel<float>, grid, dim3(256), 0, A);
    else if (in_dtype == DFLASH_BF16) br.launch(gdn_finish_kernel<bf16_t>, grid, dim3(256), 0, A);
    else br.launch(gdn_finish_kernel<f16_t>, grid, dim3(256), 0, A);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

extern "C" int dflash_gdn_prepare(void* stream, const void* mixed_qkv, const void* conv_state_in,
                                  const void* conv_weight, const void* a_logits, int g_ndim, const void* b_logits,
                                  const float* a_log, const float* dt_bias, int in_dtype, float q_scale,
                                  float k_scale, float norm_eps, void* q_out, void* k_out, void* v_out, void* g_out,
                                  void* beta_out, void* conv_state_out, int B, int T, int Hk, int Hv, int Dk, int Dv,
                                  int K) {
    int rc = ensure_init();
    if (rc) return rc;
    DFLASH_REQUIRE(B > 0 && T > 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, "gdn_prepare: non-positive dimension");
    DFLASH_REQUIRE(mixed_qkv && conv_weight && a_logits && b_logits && a_log && dt_bias, "gdn_prepare: null input");
    DFLASH_REQUIRE(q_out && k_out && v_out && g_out && beta_out && conv_state_out, "gdn_prepare: null output");
    DFLASH_REQUIRE(g_ndim == 3 || g_ndim == 4, "gdn_prepare: g_ndim must be 3 or 4");
    DFLASH_REQUIRE(conv_state_out != conv_state_in, "gdn_prepare: conv_state_out aliases conv_state_in");
    DFLASH_SUPPORTED(K >= 2 && K <= kPrepMaxTaps, "gdn_prepare: conv kernel size %d outside [2, %d]", K, kPrepMaxTaps);
    DFLASH_SUPPORTED(Dk <= 1024 && Dv <= 1024, "gdn_prepare: head dim above 1024");
    DFLASH_SUPPORTED(in_dtype == DFLASH_F32 || in_dtype == DFLASH_BF16 || in_dtype == DFLASH_F16, "gdn_prepare: bad dtype %d", in_dtype);
    DFLASH_REQUIRE(T <= 65535 && B <= 65535, "gdn_prepare: T or B too large for one launch");

    PrepareArgs A;
    A.x = mixed_qkv; A.state_in = conv_state_in; A.weight = conv_weight; A.a = a_logits; A.b = b_logits;
    A.a_log = a_log; A.dt_bias = dt_bias; A.q = q_out; A.k = k_out; A.v = v_out; A.g = g_out; A.beta = beta_out;
    A.state_out = conv_state_out; A.q_scale = q_scale; A.k_scale = k_scale; A.eps = norm_eps; A.in_dtype = in_dtype;
    A.vec_gate = g_ndim == 4;
    A.T = T; A.Hk = Hk; A.Hv = Hv; A.Dk = Dk; A.Dv = Dv; A.K = K; A.C = 2 * Hk * Dk + Hv * Dv;
    const int widest = Dk > Dv ? Dk : Dv;
    const int threads = ((widest + 63) / 64) * 64;
    dim3 grid(2 * Hk + Hv + (A.vec_gate ? Hv : 1), T, B);
    hipStream_t st = (hipStream_t)stream;
    LaunchBracket br(DFLASH_KERNEL_GDN_PREPARE, st);
    if (in_dtype == DFLASH_F32) br.launch(gdn_prepare_kernel<float>, grid, dim3(threads), 0, A);
    else if (in_dtype == DFLASH_BF16) br.launch(gdn_prepare_kernel<bf16_t>, grid, dim3(threads), 0, A);
    else br.launch(gdn_prepare_kernel<f16_t>, grid, dim3(threads), 0, A);
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}
