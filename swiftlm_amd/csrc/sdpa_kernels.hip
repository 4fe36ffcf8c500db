// Block-causal batched GQA attention for the 16-token verify block, gfx950.
//
// The problem is a stream of K/V rows (2 KV heads, tens of thousands of keys)
// scored against a tiny query tile, so it is bound by HBM bandwidth.  The
// design follows from that:
//   * all query heads of a GQA group (up to 8 heads x 16 block rows = 128 rows)
//     share one pass over their KV head's rows, so K/V are read once;
//   * the key axis is split over enough workgroups to cover every CU (split-KV),
//     each writing a partial (O / l, max, l); a second small kernel combines the
//     splits and emits O and the logsumexp;
//   * K/V tiles of 32 keys go HBM -> LDS directly, several tiles ahead, requested
//     by two waves that do nothing else; four other waves run Q K^T and P V on
//     bf16/f16 MFMA (v_mfma_f32_32x32x16) with the online softmax in registers.
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
// whatever keys its accumulators hold, and the V^T operand is gathered from LDS
// in that same key order (two transposing reads of four keys each), which is
// legal because a contraction may enumerate its index in any order.
//
// Semantics follow Sources/DFlash/DFlashKernels.swift:737-815 (entry), :563-649
// (partials: causal rule :614, GQA mapping :575) and :661-720 (combine).

#include <type_traits>

#include "dflash_common.h"

namespace dflash {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(8))) float f32x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;   // one 16-byte global/LDS access
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

constexpr int kCombineThreads = 256;
constexpr int kBN = 32;             // keys per tile
constexpr int kM = 16;              // block rows per head
constexpr int kHeadsPerWG = 8;      // query heads sharing one K/V pass
constexpr int kMaxSplits = 512;
constexpr float kRescaleLog2 = 8.f;   // lazy-rescale threshold of the online softmax, log2 units

struct Bf16Tag {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ vec8 pack(f32x8_t x) { return __builtin_convertvector(x, vec8); }
    static __device__ __forceinline__ bf16x4_t pack4(f32x4_t x) { return __builtin_convertvector(x, bf16x4_t); }
    static __device__ __forceinline__ uint16_t cvt(float x) { return f32_to_bf16_bits(x); }
    static __device__ __forceinline__ float to_f32(uint16_t x) { return __uint_as_float(((uint32_t)x) << 16); }
};
struct F16Tag {
    typedef f16x8_t vec8;
    static __device__ __forceinline__ f32x16_t mfma(vec8 a, vec8 b, f32x16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ vec8 pack(f32x8_t x) { return __builtin_convertvector(x, vec8); }
    static __device__ __forceinline__ f16x4_t pack4(f32x4_t x) { return __builtin_convertvector(x, f16x4_t); }
    static __device__ __forceinline__ uint16_t cvt(float x) {
        _Float16 hf = (_Float16)x;
        return *reinterpret_cast<uint16_t*>(&hf);
    }
    static __device__ __forceinline__ float to_f32(uint16_t x) { return (float)__builtin_bit_cast(_Float16, x); }
};

struct SdpaArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    const uint16_t* k_new;   // [B,Hk,16,D] rows standing for keys Nb-16 .. Nb-1, or null
    const uint16_t* v_new;
    uint16_t* k_cache;       // where the fused append stores those rows (== k, v), or null
    uint16_t* v_cache;
    uint16_t* part_o;   // [S, B*Hq*16, D]  partial O / l in the input type (DFlashKernels.swift:647 stores it unnormalised)
    float* part_m;   // [B*Hq*16, S]   running max, log2 units
    float* part_l;   // [B*Hq*16, S]   sum of exp2
    const int32_t* kv_len_dev;
    const uint16_t* mask;    // additive mask [B,Hq,16,N] in the input type (DFlashKernels.swift:548-553), or null
    int64_t kv_batch_stride, kv_head_stride;
    float scale_log2;   // scale * log2(e)
    int Hq, Hk, G, N, S, groups_per_kv;
    int rows_total;     // B*Hq*16
    int len_bias;       // added to kv_len_dev[b]: 0, or 16 when the device count excludes the block
    // Paged K/V (PAGED instantiations): key n of sequence b lives in page page_table[b * table_stride + (n >> page_shift)]
    // of the pool, at row n & (page_size - 1); k, v point at the pools, kv_batch_stride is the page pitch and
    // kv_head_stride the head pitch inside a page.
    const int32_t* page_table;
    int page_shift, table_stride, num_pages;
    int32_t* status;         // device status word (dflash_set_status_word), or null
    uint32_t gpk_magic, S_magic;   // fast_div_magic of groups_per_kv and S
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;

// 64 lanes x 16 B from HBM straight into LDS at lds_base + 16 * lane (lds_base is wave-uniform and
// travels in M0).  Issued as inline assembly on purpose: the compiler then does not track these
// loads, so it cannot force a full vmcnt(0) drain ahead of every LDS read or barrier; completion
// is tracked by hand with wait_vmcnt<> below, which is what keeps several tiles in flight.
// K/V rows are read once per call, so their loads carry the non-temporal hint: the stream (800 MB per verify step
// at the benchmark's shape) then no longer pushes the recurrent state, the tapes and the split partials out of
// the 256 MB memory-side cache -- worth 8 % of the whole step, most of it in the OTHER kernels.
__device__ __forceinline__ void async_load_16B(const unsigned char* gbase, uint32_t goff, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :
                 : "v"(goff), "s"(gbase), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory", "m0");
}

// The same without the non-temporal hint (Q, which every workgroup of the head re-reads).
__device__ __forceinline__ void async_load_16B_plain(const unsigned char* gbase, uint32_t goff, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(goff), "s"(gbase), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory", "m0");
}

// Tells the compiler a wave-uniform pointer is uniform (inline-assembly "s" operands need SGPRs).
__device__ __forceinline__ const unsigned char* uniform_ptr(const unsigned char* p) {
    const uint64_t u = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return (const unsigned char*)(((uint64_t)hi << 32) | lo);
}

// Same, with a full per-lane 64-bit address (rows that come from different buffers).  STREAM: non-temporal, for
// K/V rows; Q, which every workgroup of the head re-reads, is loaded without the hint.
template <bool STREAM> __device__ __forceinline__ void async_load_16B_addr(const unsigned char* gptr, uint32_t lds_base) {
    if constexpr (STREAM)
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                     :
                     : "v"((uint64_t)gptr), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                     : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :
                     : "v"((uint64_t)gptr), "s"(__builtin_amdgcn_readfirstlane(lds_base))
                     : "memory", "m0");
}

// s_waitcnt vmcnt(n) only (expcnt and lgkmcnt left alone), GFX9 encoding.
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(((N >> 4) << 14) | (0xF << 8) | (0x7 << 4) | (N & 0xF));
}

// ---------------------------------------------------------------------------
// The partial kernel.  Grid: x = split, y = kv head * groups_per_kv + head group, z = batch.
//
// Roles.  A wave that issues HBM -> LDS loads is held at each load until the memory pipeline takes it; in the
// streaming steady state that is most of a tile's transfer time, and a wave that is held cannot feed its
// MFMAs.  So waves 0..3 only compute (32 query rows each: two heads of the group) and waves 4..5 only request
// tiles and wait for them: the holds fall on waves with nothing else to do.  Six waves put two on a SIMD, i.e.
// 256 registers per wave, of which the O^T accumulators take 128 at D = 256; Q therefore stays in LDS and is
// read per k-step like K.
//
// Data movement.  K/V rows go HBM -> LDS directly (global_load_lds_dwordx4, no VGPR staging).  A wave-wide load
// deposits 64 x 16 B contiguously in LDS in lane order, so the bank swizzle is applied on the way in: lane l,
// which fills piece l % CPR of its row, fetches piece (l % CPR) ^ f(row) from HBM.  K and Q use f = row % 16
// (conflict-free ds_read_b128 of one piece per row across 16 lanes); V uses f = 4 * (row % 4) (conflict-free
// ds_read_b64_tr_b16 of 4 key rows x 32 B per 16-lane group).  V^T operands come from that transposing read:
// in each 16-lane group, lane 4*j + q supplies the address of 4 channels of key row j; lane i receives channel
// (i % 4) of the address given by lane 4*r + i/4 as its r-th element, i.e. four consecutive keys of channel
// d0 + i when lane 4*j + q points at V[k0 + j][d0 + 4q].
//
// LDS: Q [128 rows] | K ring, kRingSlots tiles | V ring, kRingSlots tiles.  K and V advance separately because
// the scores run one tile ahead of the PV product: iteration t needs V(t) and K(t+1) ("group t").  Producers:
// request K(t0), Q, group t0, group t0+1; then per iteration
// t: wait for group t, barrier, request group t+2 (V(t+2) into the slot of V(t-1), K(t+3) into the slot of
// K(t), both free after the barrier).  One barrier per iteration, shared by all six waves.
//
// MASKED adds the reference's optional additive mask: a key is used when it passes the causal rule and its mask
// value is at least the lowest finite value of the input type, and the mask value is added to the scaled score
// (DFlashKernels.swift:550-553, :614-623).  The mask is read with plain loads inside the softmax; that
// instantiation is for signature parity, not for speed.  PAGED reads K/V through a page table.
// ---------------------------------------------------------------------------
constexpr int kPartialThreads = 384;    // 4 compute waves + 2 producer waves
constexpr int kRingSlots = 3;           // tiles per ring

template <int D> struct SdpaLds {
    static constexpr int ROWB = D * 2;
    static constexpr int CPR = D / 8;
    static constexpr int RPI = 64 / CPR;                     // rows per 1 KB load instruction
    static constexpr int KT = kBN * ROWB;                    // bytes of one K (or V) tile
    static constexpr int Q_BYTES = 4 * 32 * ROWB;            // 32 query rows per compute wave
    static constexpr int K_RING = Q_BYTES;
    static constexpr int V_RING = Q_BYTES + kRingSlots * KT;
    static constexpr int LPP = (kBN / RPI) / 2;              // load instructions per producer wave per K (or V) tile
    static constexpr int EROW = D * 2 + 16;                  // epilogue O row pitch, bytes
    static constexpr int EPI = 4 * 32 * EROW;
    static constexpr int RING_END = Q_BYTES + 2 * kRingSlots * KT;
    static constexpr int BYTES = RING_END > EPI ? RING_END : EPI;
};

// The t-th tile of a split: tiles are dealt in rows of S neighbouring tiles, one per split.
__device__ __forceinline__ int tile_index(int split, int t, int S) { return t * S + split; }

template <typename Tag, int D, bool MASKED, bool PAGED>
__global__ __launch_bounds__(kPartialThreads, 1) void sdpa_partial_kernel(SdpaArgs A) {
    typedef typename Tag::vec8 vec8;
    typedef SdpaLds<D> L;
    constexpr int KSTEPS = D / 16;
    constexpr int DB = D / 32;
    static_assert(4 * L::LPP <= 63, "vmcnt is a 6-bit counter");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t smem_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

    // All kernel arguments in one burst of scalar loads: fetched where they are first used they arrive in three
    // dependent rounds (with the device-side length in the middle), each a trip to memory ahead of the first tile.
    asm volatile("" ::"s"(A.q), "s"(A.k), "s"(A.v), "s"(A.k_new), "s"(A.v_new), "s"(A.k_cache), "s"(A.v_cache), "s"(A.part_o),
                 "s"(A.part_m), "s"(A.part_l), "s"(A.kv_len_dev), "s"(A.mask), "s"(A.kv_batch_stride), "s"(A.kv_head_stride));
    asm volatile("" ::"s"(A.scale_log2), "s"(A.Hq), "s"(A.Hk), "s"(A.G), "s"(A.N), "s"(A.S), "s"(A.groups_per_kv),
                 "s"(A.rows_total), "s"(A.len_bias), "s"(A.page_table), "s"(A.page_shift), "s"(A.table_stride), "s"(A.num_pages),
                 "s"(A.status), "s"(A.gpk_magic), "s"(A.S_magic));

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool producer = wave >= 4;
    const int c = lane & 31, h = lane >> 5;
    const int split = blockIdx.x;
    const int hk = (int)fast_div(blockIdx.y, (uint32_t)A.groups_per_kv, A.gpk_magic);
    const int hg0 = ((int)blockIdx.y - hk * A.groups_per_kv) * kHeadsPerWG;
    const int b = blockIdx.z;
    const int hcount = (A.G - hg0) < kHeadsPerWG ? (A.G - hg0) : kHeadsPerWG;

    // Paged: each producer wave keeps the page-table entries of this workgroup's next 64 tiles in a register, one
    // tile per lane (a single gather, so a cold table costs one round trip per 64 tiles and none inside the loop),
    // and the 64 after those in a second register that is fetched a whole batch ahead.  The first gather is issued
    // here, ahead of the device-side length, so that the two cold reads overlap; it therefore covers the tiles of
    // the host-side bound N, which the table spans by contract.
    int ent_cur = 0, ent_nxt = 0, ent_base = 0;
    auto load_entries = [&](int base) -> int {
        // no branch and no arithmetic on the value here: the wait for it then sits at its first use, not at the load
        const int nt_max = (A.N + kBN - 1) / kBN;
        int tile = tile_index(split, base + lane, A.S);
        tile = tile < nt_max ? tile : nt_max - 1;
        return A.page_table[(size_t)b * A.table_stride + ((tile * kBN) >> A.page_shift)];
    };
    if constexpr (PAGED) {
        if (producer) {
            ent_cur = load_entries(0);
            ent_nxt = load_entries(64);
        }
    }

    // The device-side key count is requested here, through the scalar cache, and awaited below the Q requests: a
    // scalar read counts on its own counter, so waiting for it does not wait for Q.  (Written as assembly because
    // the compiler would wait where the read is issued; the register is not touched between the two statements.
    // Without a device-side count a word of Q is read and dropped, which keeps the sequence free of branches.)
    int len_raw;
    {
        const int32_t* lp = A.kv_len_dev ? A.kv_len_dev + b : reinterpret_cast<const int32_t*>(A.q);
        asm volatile("s_load_dword %0, %1, 0x0" : "=s"(len_raw) : "s"(lp));
    }
    // Q does not depend on the key count, and the compute waves have nothing to do until the first tile lands: each
    // asks for its own 32 rows (heads 2w, 2w+1 of the group; an absent head re-reads the group's first head, its rows
    // are never stored) while the device-side count is still on its way and the producers get ready for K(t_begin).
    // Swizzled like a K tile, at w * 32 rows of the Q area.
    if (!producer) {
        const int ld_rsub = lane / L::CPR, ld_pos = lane % L::CPR;
        const unsigned char* qb = reinterpret_cast<const unsigned char*>(A.q) + ((size_t)b * A.Hq + hk * A.G + hg0) * kM * L::ROWB;
        if (2 * wave + 1 < hcount) {                 // uniform: both heads present, the 32 rows are contiguous
            const unsigned char* qw = uniform_ptr(qb + (size_t)wave * 32 * L::ROWB);
#pragma unroll
            for (int j = 0; j < 32 / L::RPI; ++j) {
                const int row = j * L::RPI + ld_rsub;
                async_load_16B_plain(qw, (uint32_t)(row * L::ROWB + ((ld_pos ^ (row & 15)) * 16)),
                                     smem_lds + (wave * 32 + j * L::RPI) * L::ROWB);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 32 / L::RPI; ++j) {
                const int row = wave * 32 + j * L::RPI + ld_rsub;
                const int head = (row >> 4) < hcount ? (row >> 4) : 0;
                async_load_16B_addr<false>(qb + (size_t)(head * kM + (row & 15)) * L::ROWB + ((ld_pos ^ (row & 15)) * 16),
                                    smem_lds + (wave * 32 + j * L::RPI) * L::ROWB);
            }
        }
    }
    // Everything that does not depend on the key count is worked out while the count is on its way (the bases are
    // operands of the wait below, so that they are in registers before it, not behind it).
    const int cw = producer ? 0 : wave;                      // compute wave index (producers: unused)
    const int head_in_group = 2 * cw + (c >> 4);
    const bool row_valid = !producer && head_in_group < hcount;
    const bool wave_active = !producer && 2 * cw < hcount;
    const int hq = hk * A.G + hg0 + head_in_group;
    const int qi = c & 15;
    const size_t row_id = ((size_t)b * A.Hq + hq) * kM + qi;

    // dense: the head's rows are contiguous; paged: the head's slice of page 0, the page is added per tile
    const size_t head_off = PAGED ? (size_t)hk * A.kv_head_stride * 2
                                  : ((size_t)b * A.kv_batch_stride + (size_t)hk * A.kv_head_stride) * 2;
    const unsigned char* kbase = reinterpret_cast<const unsigned char*>(A.k) + head_off;
    const unsigned char* vbase = reinterpret_cast<const unsigned char*>(A.v) + head_off;
    const unsigned char* knew = reinterpret_cast<const unsigned char*>(A.k_new) + ((size_t)b * A.Hk + hk) * kM * L::ROWB;
    const unsigned char* vnew = reinterpret_cast<const unsigned char*>(A.v_new) + ((size_t)b * A.Hk + hk) * kM * L::ROWB;
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(len_raw) : "s"(kbase), "s"(vbase), "s"(knew), "s"(vnew));
    int Nb = A.kv_len_dev ? len_raw + A.len_bias : A.N;
    if (A.status && (Nb < kM || Nb > A.N) && split == 0 && blockIdx.y == 0 && tid == 0) atomicOr(A.status, DFLASH_STATUS_SDPA_LEN);
    Nb = Nb < kM ? kM : (Nb > A.N ? A.N : Nb);
    const int nt = (Nb + kBN - 1) / kBN;
    // Tiles are dealt round-robin: split s takes tiles s, s + S, s + 2S, ...  At any moment the workgroups of a KV
    // head then read one contiguous stretch of the cache (S neighbouring tiles) instead of S stretches a split
    // apart, which the memory system serves faster.  Below, t counts this split's own tiles (0 .. t_end-1) and
    // key_of(t) is the first key of its t-th tile.
    const int t_begin = 0;
    const int t_full = (int)fast_div((uint32_t)nt, (uint32_t)A.S, A.S_magic);    // rows of S tiles that every split takes part in
    const int t_end = t_full + (tile_index(split, t_full, A.S) < nt ? 1 : 0);
    const int t_last = t_end - 1;
    auto key_of = [&](int t) { return tile_index(split, t, A.S) * kBN; };

    // Byte offset of key n's row from kbase / vbase (the K and V pools share one layout), for the rows that are
    // looked up one by one: those of the fused append.  Paged: the page comes from the table, clamped to the pool.
    // (Tiles take tile_off() below; a tile never straddles a page, page sizes being multiples of kBN.)
    const int page_mask = PAGED ? (1 << A.page_shift) - 1 : 0;
    auto row_off = [&](int key) -> size_t {
        if constexpr (PAGED) {
            int e = A.page_table[(size_t)b * A.table_stride + (key >> A.page_shift)];
            e = e < 0 ? 0 : (e >= A.num_pages ? A.num_pages - 1 : e);
            return (size_t)e * (size_t)A.kv_batch_stride * 2 + (size_t)(key & page_mask) * L::ROWB;
        } else {
            return (size_t)key * L::ROWB;
        }
    };
    // Fused append: keys Nb-16 .. Nb-1 are read from k_new / v_new, and the workgroups of the KV head store them
    // into the cache rows they stand for (paged: the 16 rows may straddle a page, so every row looks its page up).
    // The copy is spread over all splits of the KV head (done whole by one workgroup it was four dependent round trips
    // in that workgroup, which then finished last of the launch).
    const bool fused = A.k_new != nullptr;
    const int cache_rows = fused ? Nb - kM : Nb;       // keys below this index are read from the cache
    if (fused && A.k_cache && hg0 == 0 && wave == 0) {
        // 16-byte pieces of the block's rows, dealt evenly over the splits of the KV head: a handful per workgroup,
        // read and written by the first compute wave in one round trip.
        const int pieces = kM * L::CPR;
        const int per = (pieces + A.S - 1) / A.S;
        const u32x4_t* ksrc = reinterpret_cast<const u32x4_t*>(knew);
        const u32x4_t* vsrc = reinterpret_cast<const u32x4_t*>(vnew);
        for (int i0 = 0; i0 < per; i0 += 64) {
            const int i = split * per + i0 + lane;
            if (i0 + lane < per && i < pieces) {
                const u32x4_t kx = ksrc[i], vx = vsrc[i];
                const size_t off = head_off + row_off(cache_rows + i / L::CPR) + (size_t)(i % L::CPR) * 16;
                *reinterpret_cast<u32x4_t*>(reinterpret_cast<unsigned char*>(A.k_cache) + off) = kx;
                *reinterpret_cast<u32x4_t*>(reinterpret_cast<unsigned char*>(A.v_cache) + off) = vx;
            }
        }
    }

    if (t_begin >= t_end) {   // empty split: tell the combine kernel to ignore it
        wait_vmcnt<0>();                             // the Q requests must have landed before the wave ends
        if (row_valid && h == 0) {
            A.part_m[row_id * A.S + split] = -INFINITY;
            A.part_l[row_id * A.S + split] = 0.f;
        }
        return;
    }

    // =========================== producers ===========================
    if (producer) {
        const int pw = wave - 4;
        const int ld_rsub = lane / L::CPR, ld_pos = lane % L::CPR;
        // instruction j of this producer covers rows (2*j + pw) * RPI .. + RPI - 1 of a tile (or of Q)
        auto issue_rows = [&](const unsigned char* base, bool k_swizzle, int t, size_t toff, uint32_t lds_tile, bool is_k) {
            const int key0 = key_of(t);
            if (key0 + kBN <= cache_rows) {              // uniform: whole tile comes from the cache
                const unsigned char* tp = uniform_ptr(base + toff);
#pragma unroll
                for (int j = 0; j < L::LPP; ++j) {
                    const int rg = (2 * j + pw) * L::RPI;
                    const int row = rg + ld_rsub;
                    const uint32_t sw = k_swizzle ? (uint32_t)((ld_pos ^ (row & 15)) * 16) : (uint32_t)((ld_pos ^ (4 * (row & 3))) * 16);
                    async_load_16B(tp, (uint32_t)row * L::ROWB + sw, lds_tile + rg * L::ROWB);
                }
            } else {
                // Tail tile: rows past the end re-read the last key (masked later); with a fused append the
                // block's own 16 rows are taken from k_new / v_new instead of the cache.  Its cache rows sit behind
                // the tile's own offset like any other tile's (paged: a tile lies in one page).
#pragma unroll
                for (int j = 0; j < L::LPP; ++j) {
                    const int rg = (2 * j + pw) * L::RPI;
                    const int row = rg + ld_rsub;
                    int key = key0 + row;
                    key = key < Nb ? key : Nb - 1;
                    const uint32_t sw = k_swizzle ? (uint32_t)((ld_pos ^ (row & 15)) * 16) : (uint32_t)((ld_pos ^ (4 * (row & 3))) * 16);
                    const unsigned char* nw = is_k ? knew : vnew;
                    const unsigned char* src = key < cache_rows ? base + toff + (size_t)(key - key0) * L::ROWB
                                                                : nw + (size_t)(key - cache_rows) * L::ROWB;
                    async_load_16B_addr<true>(src + sw, lds_tile + rg * L::ROWB);
                }
            }
        };
        auto issue_k = [&](int t, size_t toff) {
            if (t < t_end) issue_rows(kbase, true, t, toff, smem_lds + L::K_RING + ((t - t_begin) % kRingSlots) * L::KT, true);
        };
        auto issue_v = [&](int t, size_t toff) {
            if (t < t_end) issue_rows(vbase, false, t, toff, smem_lds + L::V_RING + ((t - t_begin) % kRingSlots) * L::KT, false);
        };
        // Offset of tile t's first row (a wave-uniform value); paged: from the entries gathered at the top of the
        // kernel, refilled a batch ahead.  Tiles are asked for in increasing order.
        auto tile_off = [&](int t) -> size_t {
            if (t >= t_end) return 0;
            if constexpr (PAGED) {
                if (t - ent_base >= 64) {                                        // uniform
                    ent_cur = ent_nxt;
                    ent_base += 64;
                    ent_nxt = load_entries(ent_base + 64);
                    // Take the value here, once per 64 tiles.  Left pending, the compiler carries the load across the
                    // loop and puts a vmcnt(0) in front of every iteration's use, which drains the tile requests too.
                    asm volatile("" : "+v"(ent_nxt));
                }
                int e = __builtin_amdgcn_readlane(ent_cur, (t - ent_base) & 63);
                e = e < 0 ? 0 : (e >= A.num_pages ? A.num_pages - 1 : e);      // a stale table cannot leave the pool
                return (size_t)e * (size_t)A.kv_batch_stride * 2 + (size_t)(key_of(t) & page_mask) * L::ROWB;
            } else {
                return (size_t)key_of(t) * L::ROWB;
            }
        };
        // loads of group t still outstanding when one waits for the group before it
        auto group_loads = [&](int t) { return (t < t_end ? L::LPP : 0) + (t + 1 < t_end ? L::LPP : 0); };

        if constexpr (PAGED) asm volatile("" : "+v"(ent_cur), "+v"(ent_nxt));   // both gathers have landed from here on
        // Opening: only K(t_begin) (Q is already on its way) stands between the compute waves and their first
        // scores, so the first barrier waits for just these; the next two groups are requested behind it, while the
        // compute waves already work on tile t_begin.
        const size_t o0 = tile_off(t_begin), o1 = tile_off(t_begin + 1);
        issue_k(t_begin, o0);
        wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();                       // Q and K(t_begin) are in LDS
        issue_v(t_begin, o0); issue_k(t_begin + 1, o1);     // group t_begin
        issue_v(t_begin + 1, o1);                           // group t_begin + 1 ...
        size_t off_v = tile_off(t_begin + 2);                   // tile whose V the next iteration requests
        issue_k(t_begin + 2, off_v);                            // ... and its K
        size_t off_k = tile_off(t_begin + 3);                   // tile whose K the next iteration requests
        for (int t = t_begin; t <= t_last; ++t) {
            const int later = group_loads(t + 1);
            if (later >= 2 * L::LPP) wait_vmcnt<2 * L::LPP>();
            else if (later >= L::LPP) wait_vmcnt<L::LPP>();
            else wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();                   // group t is in LDS; iteration t-1 is over for every wave
            issue_v(t + 2, off_v); issue_k(t + 3, off_k);   // group t + 2, into the slots iteration t-1 released
            off_v = off_k;
            off_k = tile_off(t + 4);
        }
        return;
    }

    // =========================== compute waves ===========================
    // per-lane pieces of the operand addresses
    const int k_rd = c * L::ROWB;                        // K, Q: this lane's row
    const int k_sw = c & 15;
    const int tj = (lane & 15) >> 2, tq = lane & 3;      // V: transposing read, lane = 4*tj + tq in its group
    const int tg = lane >> 4;                            // group: channel half tg & 1, key half tg >> 1
    const int v_rd = (4 * (tg >> 1) + tj) * L::ROWB + (tq & 1) * 8;
    const int v_piece = 2 * (tg & 1) + (tq >> 1);        // 16-byte piece within a 32-channel block
    const unsigned char* q_rows = smem + cw * 32 * L::ROWB;

    auto k_slot = [&](int t) -> const unsigned char* { return smem + L::K_RING + ((t - t_begin) % kRingSlots) * L::KT; };
    auto v_slot = [&](int t) -> const unsigned char* { return smem + L::V_RING + ((t - t_begin) % kRingSlots) * L::KT; };
    // Operand offsets inside a tile.  The XOR swizzles only touch the low bits of the piece index, so a handful of
    // per-lane offsets plus compile-time constants (folded into the ds_read offset field) cover every k-step:
    //   K, Q: piece (2s+h) ^ (c & 15) = 16 * (s >> 3) + ((2 * (s & 7) + h) ^ (c & 15))
    //   V:    piece (4i + v_piece) ^ (4 tj) = 16 * (i >> 2) + 4 * ((i & 3) ^ tj) + v_piece
    uint32_t koff[8], voff[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) koff[j] = (uint32_t)(k_rd + (((2 * j + h) ^ k_sw) & (L::CPR - 1)) * 16);
#pragma unroll
    for (int m = 0; m < 4; ++m) voff[m] = (uint32_t)(v_rd + v_piece * 16 + ((m ^ tj) * 64));
    auto load_k = [&](const unsigned char* ks, int s) -> vec8 {
        return *reinterpret_cast<const vec8*>(ks + koff[s & 7] + 256 * (s >> 3));
    };
    auto load_q = [&](int s) -> vec8 {
        return *reinterpret_cast<const vec8*>(q_rows + koff[s & 7] + 256 * (s >> 3));
    };
    // V^T operand of PV step s: output block s % DB, key half s / DB.  The MFMA consumes accumulator registers
    // 8*ksub .. 8*ksub+7 of S^T, i.e. keys 16*ksub + {4h..4h+3} and 16*ksub + 8 + {4h..4h+3}: two transposing
    // reads of four keys each.
    auto load_v = [&](const unsigned char* vs, int s) -> vec8 {
        const int i = s % DB, ksub = s / DB;
        const unsigned char* p = vs + voff[i & 3] + 256 * (i >> 2);
        const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t*)(p + (16 * ksub) * L::ROWB));
        const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4_t*)(p + (16 * ksub + 8) * L::ROWB));
        return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    // operand reads run this many MFMA steps ahead; 2 at D = 256 keeps the wave inside its 256 registers without spills
    constexpr int kAhead = D == 256 ? 2 : 4;

    f32x16_t oacc[DB];
#pragma unroll
    for (int i = 0; i < DB; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[i][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    // ---- the per-tile work, arranged so that the softmax arithmetic hides behind the MFMAs ----
    // With one compute wave per SIMD nothing else fills the VALU while an MFMA runs, and the softmax of a tile
    // (16 scores per lane: scale, max, 16 quarter-rate exp2, sum, pack) costs about as many cycles as the tile's
    // 32 MFMAs.  A 32x32x16 MFMA occupies the matrix pipe for 32 cycles after a 4-cycle issue, and independent
    // VALU instructions of the same wave issue meanwhile.  So each iteration t runs two blocks:
    //   phase 1:  S^T(t+1) = K(t+1) Q^T  (MFMA)  with  P(t) = exp2(x(t) - m), row sums, pack  (VALU)
    //   phase 2:  O^T += V(t)^T P(t)^T   (MFMA)  with  x(t+1) = scale * S^T(t+1), row maximum  (VALU)
    // where x(t) are tile t's scaled scores.  sched_barrier(0) after every step pins the order.
    float x[16];                    // scaled (log2 domain) and masked scores of the current tile
    vec8 pb[2];                     // P^T of the current tile as MFMA operands (two key halves)
    f32x16_t sacc, sacc1;           // raw scores of the next tile, two accumulation chains
    float m_pending = -INFINITY;

    // S^T = K Q^T of one tile on its own (first tile only).  Two accumulators: a dependent 32x32x16 MFMA waits
    // out the pipeline latency of its predecessor, two interleaved chains hide half of it.
    auto qk_tile = [&](int t) {
        const unsigned char* ks = k_slot(t);
#pragma unroll
        for (int v = 0; v < 16; ++v) { sacc[v] = 0.f; sacc1[v] = 0.f; }
        vec8 ka[KSTEPS], qa[KSTEPS];
#pragma unroll
        for (int s = 0; s < kAhead; ++s) { ka[s] = load_k(ks, s); qa[s] = load_q(s); }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KSTEPS; s += 2) {
            if (s + kAhead < KSTEPS) {
                ka[s + kAhead] = load_k(ks, s + kAhead); ka[s + kAhead + 1] = load_k(ks, s + kAhead + 1);
                qa[s + kAhead] = load_q(s + kAhead); qa[s + kAhead + 1] = load_q(s + kAhead + 1);
            }
            sacc = Tag::mfma(ka[s], qa[s], sacc);
            sacc1 = Tag::mfma(ka[s + 1], qa[s + 1], sacc1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Phase 1 of iteration t.
    auto exp_qk = [&](int t) {
        const unsigned char* ks = k_slot(t + 1);
        const float m_safe = m_run == -INFINITY ? 0.f : m_run;
        float psum = 0.f;
        f32x8_t p0, p1;
#pragma unroll
        for (int v = 0; v < 16; ++v) { sacc[v] = 0.f; sacc1[v] = 0.f; }
        vec8 ka[KSTEPS], qa[KSTEPS];
#pragma unroll
        for (int s = 0; s < kAhead; ++s) { ka[s] = load_k(ks, s); qa[s] = load_q(s); }
        __builtin_amdgcn_sched_barrier(0);
        constexpr int PAIRS = KSTEPS / 2;
        constexpr int EPP = 16 / PAIRS;
#pragma unroll
        for (int s = 0; s < KSTEPS; s += 2) {
            if (s + kAhead < KSTEPS) {
                ka[s + kAhead] = load_k(ks, s + kAhead); ka[s + kAhead + 1] = load_k(ks, s + kAhead + 1);
                qa[s + kAhead] = load_q(s + kAhead); qa[s + kAhead + 1] = load_q(s + kAhead + 1);
            }
            sacc = Tag::mfma(ka[s], qa[s], sacc);
            sacc1 = Tag::mfma(ka[s + 1], qa[s + 1], sacc1);
            const int pr = s / 2;
#pragma unroll
            for (int e = pr * EPP; e < (pr + 1) * EPP; ++e) {
                const float pe = fast_exp2(x[e] - m_safe);
                psum += pe;
                if (e < 8) p0[e] = pe; else p1[e - 8] = pe;
            }
            if ((pr + 1) * EPP == 8) pb[0] = Tag::pack(p0);
            __builtin_amdgcn_sched_barrier(0);
        }
        pb[1] = Tag::pack(p1);
        l_run += psum;
    };
    // Phase 2 of iteration t: returns the running maximum of x(t+1) over this lane's 16 scores.
    auto pv_scale = [&](int t) -> float {
        const unsigned char* vs = v_slot(t);
        vec8 va[KSTEPS];
#pragma unroll
        for (int s = 0; s < kAhead; ++s) va[s] = load_v(vs, s);
        __builtin_amdgcn_sched_barrier(0);
        float mloc = -INFINITY;
        constexpr int EPS = 16 / KSTEPS;
        constexpr int LAG = 2;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            if (s + kAhead < KSTEPS) va[s + kAhead] = load_v(vs, s + kAhead);
            oacc[s % DB] = Tag::mfma(va[s], pb[s / DB], oacc[s % DB]);
            if (s >= LAG) {
#pragma unroll
                for (int e = (s - LAG) * EPS; e < (s - LAG + 1) * EPS; ++e) {
                    x[e] = (sacc[e] + sacc1[e]) * A.scale_log2;
                    mloc = fmaxf(mloc, x[e]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int e = (KSTEPS - LAG) * EPS; e < 16; ++e) {
            x[e] = (sacc[e] + sacc1[e]) * A.scale_log2;
            mloc = fmaxf(mloc, x[e]);
        }
        return mloc;
    };
    // Masks on x (tiles that reach the block's own keys: the causal rule; MASKED: the additive mask as well) and
    // the row maximum over both half-waves.  mloc is the maximum of the unmasked scores.
    auto mask_and_max = [&](int t, float mloc) -> float {
        const int key0 = key_of(t);
        const bool need_mask = (key0 + kBN) > (Nb - kM);
        if (MASKED || need_mask) {                  // uniform
            const int last_visible = Nb - kM + qi;  // row qi sees keys 0 .. Nb-16+qi
            float mk[16];
            if constexpr (MASKED) {
                const uint16_t* mrow = A.mask + row_id * (size_t)A.N;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    int key = key0 + 8 * (v >> 2) + 4 * h + (v & 3);
                    key = key < A.N ? key : A.N - 1;               // keys past the end fail the causal rule anyway
                    mk[v] = row_valid ? Tag::to_f32(mrow[key]) : 0.f;
                }
            }
            mloc = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                if constexpr (MASKED) {
                    // -inf (or NaN) drops the key; a finite mask value, however low, keeps it in the softmax
                    x[v] = mk[v] >= -3.4028234663852886e38f ? fmaxf(fmaf(mk[v], 1.4426950408889634f, x[v]), -3.4028234663852886e38f)
                                                             : -INFINITY;
                }
                const int key = key0 + 8 * (v >> 2) + 4 * h + (v & 3);
                x[v] = key <= last_visible ? x[v] : -INFINITY;
                mloc = fmaxf(mloc, x[v]);
            }
        }
        return fmaxf(mloc, __shfl_xor(mloc, 32));
    };
    // Lazy rescale: the exponent reference m_run only moves when a tile's maximum exceeds it by more than
    // kRescaleLog2 (P then stays below 2^kRescaleLog2, harmless in fp32/bf16).  Rows that are still empty take the
    // new reference at once; if rows that already accumulated data must move, false is returned and the caller
    // rescales the accumulators OUTSIDE the hot loop.  (With the rescale written inside it the register allocator
    // keeps a second copy of all 128 accumulator registers and refreshes it on every iteration.)
    auto accept_max = [&](float ml) -> bool {
        const bool bump = ml > m_run + kRescaleLog2;        // also true for the first finite maximum
        if (__builtin_amdgcn_ballot_w64(bump && m_run != -INFINITY) != 0) {
            m_pending = ml;
            return false;
        }
        if (bump) m_run = ml;
        return true;
    };
    // P(t) from x(t) without anything to hide behind (last tile)
    auto exp_tile = [&]() {
        const float m_safe = m_run == -INFINITY ? 0.f : m_run;
        float psum = 0.f;
        f32x8_t p0, p1;
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            p0[v] = fast_exp2(x[v] - m_safe);
            p1[v] = fast_exp2(x[v + 8] - m_safe);
            psum += p0[v] + p1[v];
        }
        l_run += psum;
        pb[0] = Tag::pack(p0);
        pb[1] = Tag::pack(p1);
    };
    auto pv_tile = [&](int t) {
        const unsigned char* vs = v_slot(t);
        vec8 va[KSTEPS];
#pragma unroll
        for (int s = 0; s < kAhead; ++s) va[s] = load_v(vs, s);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            if (s + kAhead < KSTEPS) va[s + kAhead] = load_v(vs, s + kAhead);
            oacc[s % DB] = Tag::mfma(va[s], pb[s / DB], oacc[s % DB]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    wait_vmcnt<0>();                                // this wave's Q rows have landed
    __builtin_amdgcn_s_barrier();                   // Q and K(t_begin) are in LDS
    if (wave_active) {
        qk_tile(t_begin);
        float mloc = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            x[v] = (sacc[v] + sacc1[v]) * A.scale_log2;
            mloc = fmaxf(mloc, x[v]);
        }
        accept_max(mask_and_max(t_begin, mloc));
    }
    int t = t_begin;
    while (t < t_last) {
        bool jumped = false;
        for (; t < t_last; ++t) {
            __builtin_amdgcn_s_barrier();           // V(t) and K(t+1) are in LDS; everyone is done with iteration t-1
            if (wave_active) {
                exp_qk(t);
                const float mloc = pv_scale(t);
                if (!accept_max(mask_and_max(t + 1, mloc))) {
                    jumped = true;
                    break;
                }
            }
        }
        if (jumped) {
            const bool bump = m_pending > m_run + kRescaleLog2;
            const float alpha = (bump && m_run != -INFINITY) ? fast_exp2(m_run - m_pending) : 1.f;
            if (bump) m_run = m_pending;
            l_run *= alpha;
            // (no AGPR pins here: with 256 registers per wave and no "a" constraint in the function the compiler
            //  keeps every MFMA accumulator in VGPRs, so this multiply works on them in place)
#pragma unroll
            for (int i = 0; i < DB; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) oacc[i][v] *= alpha;
            ++t;
        }
    }
    __builtin_amdgcn_s_barrier();                   // V(t_last) is in LDS
    if (wave_active) {
        exp_tile();
        pv_tile(t_last);
    }
    // The epilogue stages rows in the first EPI bytes of LDS (Q and the head of the K ring): nobody reads those
    // after the barrier above (the last scores were taken in iteration t_last - 1), and every load has landed
    // (the producers' last wait was vmcnt(0)).
    static_assert(L::EPI <= L::V_RING, "the epilogue staging must stay clear of the V ring");

    // ---- epilogue: partial statistics and O rows (through LDS for coalesced stores) ----
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (row_valid && h == 0) {      // written through like the partial rows: 4-byte fragments of lines shared with other splits
        __hip_atomic_store(A.part_m + row_id * A.S + split, m_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(A.part_l + row_id * A.S + split, l_tot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (wave_active) {
        const float inv_l = l_tot > 0.f ? 1.f / l_tot : 0.f;
        unsigned char* os = smem + cw * 32 * L::EROW;
#pragma unroll
        for (int i = 0; i < DB; ++i)
#pragma unroll
            for (int v4 = 0; v4 < 4; ++v4) {
                const f32x4_t o4 = {oacc[i][4 * v4] * inv_l, oacc[i][4 * v4 + 1] * inv_l, oacc[i][4 * v4 + 2] * inv_l,
                                    oacc[i][4 * v4 + 3] * inv_l};
                const u32x2_t pk = __builtin_bit_cast(u32x2_t, Tag::pack4(o4));
                *reinterpret_cast<u32x2_t*>(os + c * L::EROW + (32 * i + 8 * v4 + 4 * h) * 2) = pk;
            }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);
        const int rows = (hcount - 2 * cw) >= 2 ? 32 : 16;
        const size_t rid0 = ((size_t)b * A.Hq + hk * A.G + hg0 + 2 * cw) * kM;
        constexpr int PER_ROW = D / 8;
        constexpr int RPP = 64 / PER_ROW;
        const int rsub = lane / PER_ROW, d = (lane % PER_ROW) * 8;
        uint16_t* dst = A.part_o + ((size_t)split * A.rows_total + rid0) * D + d;
#pragma unroll
        for (int r0 = 0; r0 < 32; r0 += 8 * RPP) {
            u32x4_t o[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) o[u] = *reinterpret_cast<const u32x4_t*>(os + (r0 + u * RPP + rsub) * L::EROW + d * 2);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int r = r0 + u * RPP + rsub;
                // Written through (system scope): the 16.8 MB of partial rows then drain while other workgroups still
                // compute, instead of sitting dirty in the L2s until the end-of-launch flush (-0.7 us per launch).
                // (The s_nop is the wait state the hardware needs between a store of more than 64 bits and a VALU write
                //  of the registers that hold its data; the compiler inserts it for its own stores, not for assembly.)
                if (r < rows)
                    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"((uint64_t)(dst + (size_t)r * D)), "v"(o[u]) : "memory");
            }
        }
    }
}

// One workgroup per output row (b, hq, i): merges the S partials.
struct CombineArgs {
    const uint16_t* part_o;
    const float* part_m;
    const float* part_l;
    uint16_t* out;
    float* lse;
    int S;
};

template <typename Tag, int D>
__global__ __launch_bounds__(kCombineThreads) void sdpa_combine_kernel(CombineArgs A) {
    constexpr int TPG = D / 8;                     // threads spanning one row, 8 elements (16 B) each
    constexpr int NG = kCombineThreads / TPG;         // split groups walking the partials in parallel
    constexpr int UNROLL = 16;                     // row loads in flight per thread: one round trip for S <= 16 * NG
    __shared__ float w_s[kMaxSplits];
    __shared__ float redm_s[kCombineThreads / 64], reds_s[kCombineThreads / 64];
    __shared__ float acc_s[NG][D];
    static_assert(kMaxSplits <= 2 * kCombineThreads, "a thread holds the statistics of at most two splits");

    asm volatile("" ::"s"(A.part_o), "s"(A.part_m), "s"(A.part_l), "s"(A.out), "s"(A.lse), "s"(A.S));   // one burst of argument loads
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    const float* pm = A.part_m + row * A.S;
    const float* pl = A.part_l + row * A.S;
    const int grp = tid / TPG, d8 = (tid % TPG) * 8;
    const uint16_t* po = A.part_o + row * D + d8;

    // Everything the row needs is requested in one go: the statistics of this thread's splits (tid and, beyond 256
    // splits, tid + 256; addresses clamped, values dropped) and the first UNROLL partial rows of its group.  Asked
    // for one after the other -- maxima, then sums, then rows -- they are three dependent trips to memory.
    const int sa = tid < A.S ? tid : A.S - 1, sb = tid + kCombineThreads < A.S ? tid + kCombineThreads : A.S - 1;
    float m0 = pm[sa], m1 = pm[sb];
    const float l0 = pl[sa], l1 = pl[sb];
    u32x4_t raw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const int sp = grp + u * NG;
        // Loaded without looking at the weight (a branch per load makes the loads wait for one another); the rows of
        // empty splits hold no data, whatever was read from them is dropped below.
        raw[u] = *reinterpret_cast<const u32x4_t*>(po + (size_t)(sp < A.S ? sp : 0) * gridDim.x * D);
    }
    if (tid >= A.S) m0 = -INFINITY;
    if (tid + kCombineThreads >= A.S) m1 = -INFINITY;

    // global max
    float mx = wave_max(fmaxf(m0, m1));
    if ((tid & 63) == 0) redm_s[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(redm_s[0], redm_s[1]), fmaxf(redm_s[2], redm_s[3]));
    // weights and denominator (the partial rows are O / l: weight by l)
    const float w0 = m0 == -INFINITY ? 0.f : fast_exp2(m0 - mx) * l0;
    const float w1 = m1 == -INFINITY ? 0.f : fast_exp2(m1 - mx) * l1;
    if (tid < A.S) w_s[tid] = w0;
    if (tid + kCombineThreads < A.S) w_s[tid + kCombineThreads] = w1;
    float lsum = butterfly_sum<64>(w0 + w1);
    if ((tid & 63) == 0) reds_s[tid >> 6] = lsum;
    __syncthreads();
    lsum = reds_s[0] + reds_s[1] + reds_s[2] + reds_s[3];

    // weighted sum of the partial rows: group grp takes splits grp, grp + NG, ...
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    for (int s0 = grp; s0 < A.S; s0 += NG * UNROLL) {
        float w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int sp = s0 + u * NG;
            w[u] = sp < A.S ? w_s[sp] : 0.f;
            if (s0 != grp) raw[u] = *reinterpret_cast<const u32x4_t*>(po + (size_t)(sp < A.S ? sp : 0) * gridDim.x * D);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (w[u] == 0.f) raw[u][e] = 0u;
                acc[2 * e] = fmaf(w[u], Tag::to_f32((uint16_t)(raw[u][e] & 0xffffu)), acc[2 * e]);
                acc[2 * e + 1] = fmaf(w[u], Tag::to_f32((uint16_t)(raw[u][e] >> 16)), acc[2 * e + 1]);
            }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc_s[grp][d8 + e] = acc[e];
    __syncthreads();
    for (int d = tid; d < D; d += kCombineThreads) {
        float r = 0.f;
#pragma unroll
        for (int gI = 0; gI < NG; ++gI) r += acc_s[gI][d];
        const float inv = lsum == 0.f ? 1.f : 1.f / lsum;   // divide unless the sum is 0 (DFlashKernels.swift:711)
        A.out[row * D + d] = Tag::cvt(r * inv);
    }
    if (tid == 0 && A.lse) A.lse[row] = (mx + log2f(lsum)) * 0.6931471805599453f;
}

// ---- host side -------------------------------------------------------------

static int choose_splits(int B, int Hk, int groups_per_kv, int N) {
    const int nt = (N + kBN - 1) / kBN;
    const int cus = num_compute_units();
    const int per = B * Hk * groups_per_kv;      // workgroups per split index
    // How many workgroups W = per * S the key axis is spread over.  Every split pays a fixed price -- its partial rows,
    // written once and read back by the combine kernel, are as large as 4 tiles of K/V, and a launch drains them all at
    // once -- while a workgroup streams a tile in about 1.2 us.  Measured on split counts swept at 4K .. 100K keys
    // (Hq=16, Hk=2, D=256; microseconds for the pair of launches):
    //     keys     W=64   W=128   W=172   W=256
    //     4112     14.0   13.6      -     16.0          8208     17.8   15.7    -     17.6
    //     16400    19.8   20.6   19.8     20.9          32784      -    28.8   26.7   25.9
    // i.e. half the chip up to about two tiles per compute unit, the whole chip from eight tiles per compute unit on,
    // linear in between; never more workgroups than tiles.
    const long total_tiles = (long)per * nt;
    long W = cus / 2 + (total_tiles - 2L * cus) / 12;
    if (W < cus / 2) W = cus / 2;
    if (W > cus) W = cus;
    int S = (int)((W + per - 1) / per);
    if (S > nt) S = nt;
    if (S > kMaxSplits) S = kMaxSplits;
    if (S < 1) S = 1;
    // If a few more splits (at most a quarter, and never more workgroups than compute units) take one tile off the
    // longest split, take them: 129 tiles over 64 splits leave one split with three, over 65 splits none.
    const int longest = (nt + S - 1) / S;
    if (longest > 1) {
        const int more = (nt + longest - 2) / (longest - 1);          // splits for a longest one of longest - 1 tiles
        if (more <= S + S / 4 && (long)more * per <= cus && more <= kMaxSplits) S = more;
    }
    return S;
}

static size_t ws_layout(int B, int Hq, int S, int D, size_t* off_m, size_t* off_l) {
    const size_t rows = (size_t)B * Hq * kM;
    size_t o = rows * S * D * sizeof(uint16_t);
    o = (o + 255) & ~(size_t)255;
    *off_m = o;
    o += rows * S * sizeof(float);
    o = (o + 255) & ~(size_t)255;
    *off_l = o;
    o += rows * S * sizeof(float);
    return (o + 255) & ~(size_t)255;
}

template <typename Tag, int D, bool MASKED, bool PAGED>
static int launch_sdpa(hipStream_t st, const SdpaArgs& A, const CombineArgs& C, int B) {
    typedef SdpaLds<D> L;
    static_assert(L::BYTES <= 160 * 1024, "Q and the tile rings must fit the 160 KB LDS of a gfx950 CU");
    auto kern = sdpa_partial_kernel<Tag, D, MASKED, PAGED>;     // its dynamic-LDS limit is set per device by sdpa_device_setup()
    dim3 grid(A.S, A.Hk * A.groups_per_kv, B);
    {
        LaunchBracket br(DFLASH_KERNEL_SDPA_PARTIAL, st);
        br.launch(kern, grid, dim3(kPartialThreads), L::BYTES, A);
    }
    DFLASH_HIP_TRY(hipGetLastError());
    {
        LaunchBracket br(DFLASH_KERNEL_SDPA_COMBINE, st);
        br.launch(sdpa_combine_kernel<Tag, D>, dim3(B * A.Hq * kM), dim3(kCombineThreads), 0, C);
    }
    DFLASH_HIP_TRY(hipGetLastError());
    return DFLASH_OK;
}

template <typename Tag, int D>
static int sdpa_partial_setup() {
    const int lds = SdpaLds<D>::BYTES;
    DFLASH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sdpa_partial_kernel<Tag, D, false, false>), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sdpa_partial_kernel<Tag, D, true, false>), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    DFLASH_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sdpa_partial_kernel<Tag, D, false, true>), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    return DFLASH_OK;
}

// Split-KV workspace of dflash_sdpa_block_causal_static: the partial rows and their statistics live in this
// file-scope device array instead of a caller-provided workspace, so that entry allocates nothing.  Every GPU the
// library runs on holds its own copy, at its own address, until the process ends.  `scratch` itself is only the
// host-side handle of the symbol: device code is handed the address that hipGetSymbolAddress returned for the
// device at hand, never the name.
static __device__ __align__(256) unsigned char scratch[DFLASH_SDPA_STATIC_SCRATCH_BYTES];
static unsigned char* g_scratch_dev[64];     // per device; written once by sdpa_device_setup() under the init mutex

int sdpa_device_setup() {
    int rc = sdpa_partial_setup<Bf16Tag, 256>();
    if (rc == DFLASH_OK) rc = sdpa_partial_setup<Bf16Tag, 128>();
    if (rc == DFLASH_OK) rc = sdpa_partial_setup<F16Tag, 256>();
    if (rc == DFLASH_OK) rc = sdpa_partial_setup<F16Tag, 128>();
    if (rc != DFLASH_OK) return rc;
    int dev = 0;
    DFLASH_HIP_TRY(hipGetDevice(&dev));
    void* ptr = nullptr;
    DFLASH_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    DFLASH_REQUIRE(ptr != nullptr && (uintptr_t)ptr % 256 == 0, "sdpa: the static scratch array has no usable device address");
    g_scratch_dev[dev & 63] = static_cast<unsigned char*>(ptr);
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

// Page table of a paged K/V pool (null for the dense layout): kv_batch_stride is then the page pitch.
struct PagedKv {
    const int32_t* table;
    int table_stride, page_size, num_pages;
};

static int sdpa_common(void* stream, const void* q, const void* k, const void* v, const void* k_new, const void* v_new,
                       void* k_cache, void* v_cache, const void* mask, void* out, float* lse, int dtype, float scale, int B, int Hq, int Hk,
                       int M, int N, int D, int64_t kv_batch_stride, int64_t kv_head_stride, const int32_t* kv_len_dev,
                       void* workspace, size_t workspace_bytes, const PagedKv* paged = nullptr, bool static_scratch = false) {
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
    int page_shift = 0;
    if (paged) {
        DFLASH_REQUIRE(paged->table != nullptr, "sdpa (paged): null page table");
        DFLASH_SUPPORTED(!mask, "sdpa (paged): the additive mask is not supported with paged K/V");
        const int ps = paged->page_size;
        DFLASH_SUPPORTED(ps >= kBN && (ps & (ps - 1)) == 0, "sdpa (paged): page size %d is not a power of two >= %d", ps, kBN);
        while ((1 << page_shift) < ps) ++page_shift;
        DFLASH_REQUIRE(paged->num_pages > 0, "sdpa (paged): empty pool");
        DFLASH_REQUIRE((int64_t)paged->table_stride * ps >= N, "sdpa (paged): %d table entries of %d keys do not cover N=%d",
                       paged->table_stride, ps, N);
        DFLASH_REQUIRE(kv_head_stride >= (int64_t)ps * D, "sdpa (paged): head pitch smaller than page_size*D");
        DFLASH_REQUIRE(kv_batch_stride >= (int64_t)(Hk - 1) * kv_head_stride + (int64_t)ps * D, "sdpa (paged): page pitch too small");
    } else {
        DFLASH_REQUIRE(kv_head_stride >= (int64_t)N * D, "sdpa: kv_head_stride smaller than N*D");
        DFLASH_REQUIRE((int64_t)N * D * 2 < (1LL << 32), "sdpa: one KV head of %d keys exceeds the 4 GiB the kernel addresses", N);
        DFLASH_REQUIRE(kv_batch_stride >= (int64_t)(Hk - 1) * kv_head_stride + (int64_t)N * D, "sdpa: kv_batch_stride too small");
    }
    DFLASH_REQUIRE(kv_head_stride % 8 == 0 && kv_batch_stride % 8 == 0, "sdpa: kv strides must be multiples of 8 elements");
    DFLASH_REQUIRE(((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)k_new | (uintptr_t)v_new) % 16 == 0,
                   "sdpa: q/k/v/out must be 16-byte aligned");
    DFLASH_REQUIRE(B <= 65535 && (long)Hq * 2 <= 65535, "sdpa: batch or head count too large for one launch");

    const int G = Hq / Hk;
    const int groups = (G + kHeadsPerWG - 1) / kHeadsPerWG;
    const int S = choose_splits(B, Hk, groups, N);
    size_t om, ol;
    const size_t need = ws_layout(B, Hq, S, D, &om, &ol);
    if (static_scratch) {
        // the library's own per-device array stands in for the workspace (address looked up at init, with that device current)
        DFLASH_SUPPORTED(need <= (size_t)DFLASH_SDPA_STATIC_SCRATCH_BYTES,
                         "sdpa (static): this shape needs %zu bytes of split-KV scratch, the built-in array holds %zu; "
                         "use dflash_sdpa_block_causal with a workspace", need, (size_t)DFLASH_SDPA_STATIC_SCRATCH_BYTES);
        int dev = 0;
        DFLASH_HIP_TRY(hipGetDevice(&dev));
        workspace = g_scratch_dev[dev & 63];
        workspace_bytes = DFLASH_SDPA_STATIC_SCRATCH_BYTES;
    }
    DFLASH_REQUIRE(workspace && workspace_bytes >= need, "sdpa: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    DFLASH_REQUIRE((uintptr_t)workspace % 256 == 0, "sdpa: workspace must be 256-byte aligned");

    SdpaArgs A;
    A.q = (const uint16_t*)q; A.k = (const uint16_t*)k; A.v = (const uint16_t*)v;
    A.k_new = (const uint16_t*)k_new; A.v_new = (const uint16_t*)v_new;
    A.k_cache = (uint16_t*)k_cache; A.v_cache = (uint16_t*)v_cache;
    A.part_o = (uint16_t*)workspace;
    A.part_m = (float*)((char*)workspace + om);
    A.part_l = (float*)((char*)workspace + ol);
    A.kv_len_dev = kv_len_dev;
    A.mask = (const uint16_t*)mask;
    A.kv_batch_stride = kv_batch_stride; A.kv_head_stride = kv_head_stride;
    A.scale_log2 = scale * 1.4426950408889634f;
    A.Hq = Hq; A.Hk = Hk; A.G = G; A.N = N; A.S = S; A.groups_per_kv = groups; A.rows_total = B * Hq * kM;
    A.gpk_magic = fast_div_magic((uint32_t)groups); A.S_magic = fast_div_magic((uint32_t)S);
    A.len_bias = k_new ? kM : 0;
    A.page_table = paged ? paged->table : nullptr;
    A.page_shift = page_shift;
    A.table_stride = paged ? paged->table_stride : 0;
    A.num_pages = paged ? paged->num_pages : 0;
    A.status = status_word();
    CombineArgs C;
    C.part_o = A.part_o; C.part_m = A.part_m; C.part_l = A.part_l;
    C.out = (uint16_t*)out; C.lse = lse; C.S = S;

    hipStream_t st = (hipStream_t)stream;
#define DFLASH_SDPA_CASE(MASKED, PAGED)                                                                              \
    do {                                                                                                             \
        if (dtype == DFLASH_BF16)                                                                                    \
            return D == 256 ? launch_sdpa<Bf16Tag, 256, MASKED, PAGED>(st, A, C, B)                               \
                            : launch_sdpa<Bf16Tag, 128, MASKED, PAGED>(st, A, C, B);                              \
        return D == 256 ? launch_sdpa<F16Tag, 256, MASKED, PAGED>(st, A, C, B)                                    \
                        : launch_sdpa<F16Tag, 128, MASKED, PAGED>(st, A, C, B);                                   \
    } while (0)
    if (mask) DFLASH_SDPA_CASE(true, false);
    if (paged) DFLASH_SDPA_CASE(false, true);
    DFLASH_SDPA_CASE(false, false);
#undef DFLASH_SDPA_CASE
}

extern "C" int dflash_sdpa_block_causal(void* stream, const void* q, const void* k, const void* v, void* out,
                                        float* lse, int dtype, float scale, int B, int Hq, int Hk, int M, int N,
                                        int D, int64_t kv_batch_stride, int64_t kv_head_stride,
                                        const int32_t* kv_len_dev, void* workspace, size_t workspace_bytes) {
    return sdpa_common(stream, q, k, v, nullptr, nullptr, nullptr, nullptr, nullptr, out, lse, dtype, scale, B, Hq, Hk, M, N, D,
                       kv_batch_stride, kv_head_stride, kv_len_dev, workspace, workspace_bytes);
}

extern "C" int dflash_sdpa_block_causal_static(void* stream, const void* q, const void* k, const void* v, void* out,
                                               float* lse, int dtype, float scale, int B, int Hq, int Hk, int M, int N,
                                               int D, int64_t kv_batch_stride, int64_t kv_head_stride,
                                               const int32_t* kv_len_dev) {
    return sdpa_common(stream, q, k, v, nullptr, nullptr, nullptr, nullptr, nullptr, out, lse, dtype, scale, B, Hq, Hk, M, N, D,
                       kv_batch_stride, kv_head_stride, kv_len_dev, nullptr, 0, nullptr, true);
}

extern "C" int dflash_sdpa_block_causal_append(void* stream, const void* q, void* k_cache, void* v_cache,
                                               const void* k_new, const void* v_new, void* out, float* lse, int dtype,
                                               float scale, int B, int Hq, int Hk, int M, int N, int D,
                                               int64_t kv_batch_stride, int64_t kv_head_stride,
                                               const int32_t* cache_len_dev, void* workspace, size_t workspace_bytes) {
    DFLASH_REQUIRE(k_new && v_new && k_cache && v_cache, "sdpa (append): null pointer");
    return sdpa_common(stream, q, k_cache, v_cache, k_new, v_new, k_cache, v_cache, nullptr, out, lse, dtype, scale, B, Hq, Hk, M,
                       N, D, kv_batch_stride, kv_head_stride, cache_len_dev, workspace, workspace_bytes);
}

extern "C" int dflash_sdpa_block_causal_masked(void* stream, const void* q, const void* k, const void* v,
                                               const void* mask, void* out, float* lse, int dtype, float scale, int B,
                                               int Hq, int Hk, int M, int N, int D, int64_t kv_batch_stride,
                                               int64_t kv_head_stride, const int32_t* kv_len_dev, void* workspace,
                                               size_t workspace_bytes) {
    DFLASH_REQUIRE(mask, "sdpa (masked): null mask");
    return sdpa_common(stream, q, k, v, nullptr, nullptr, nullptr, nullptr, mask, out, lse, dtype, scale, B, Hq, Hk, M, N, D,
                       kv_batch_stride, kv_head_stride, kv_len_dev, workspace, workspace_bytes);
}

extern "C" int dflash_sdpa_block_causal_paged(void* stream, const void* q, void* k_pool, void* v_pool,
                                              const int32_t* page_table, int page_table_stride, int page_size, int num_pages,
                                              int64_t page_stride, int64_t head_stride, const void* k_new, const void* v_new,
                                              void* out, float* lse, int dtype, float scale, int B, int Hq, int Hk, int M, int N,
                                              int D, const int32_t* len_dev, void* workspace, size_t workspace_bytes) {
    DFLASH_REQUIRE(k_pool && v_pool, "sdpa (paged): null pool");
    DFLASH_REQUIRE((k_new == nullptr) == (v_new == nullptr), "sdpa (paged): k_new and v_new go together");
    PagedKv pg{page_table, page_table_stride, page_size, num_pages};
    return sdpa_common(stream, q, k_pool, v_pool, k_new, v_new, k_new ? k_pool : nullptr, k_new ? v_pool : nullptr, nullptr, out, lse,
                       dtype, scale, B, Hq, Hk, M, N, D, page_stride, head_stride, len_dev, workspace, workspace_bytes, &pg);
}
