// Split-KV decode attention over [packed low-bit prefix || fp16 residual window] + LSE combine.
//
// Replaces compute_attn_1rowblock_splitkv and combine_attn_seqk_parallel of the reference
// (csrc/bit_decode/src/flash_fwd_kernel.h:66-728, 1144-1327) with a wave64/MFMA design:
//
//  * A workgroup owns one (split, kv-head, batch).  Each wave streams whole work units of that
//    split: 64 packed tokens at 4 bits / 128 at 2 bits (about 9 KB with their parameters), or
//    16-token tiles of the fp16 window.  A unit is fetched with ten direct-to-LDS loads
//    (global_load_lds_dwordx4: 64 lanes x 16 B = one contiguous 1 KB row each, no staging
//    registers) into the wave's private LDS region and read back 16 bytes per lane just before
//    it is unpacked.  The rows are requested in the order they are consumed, a few ahead of the
//    one being read and running on into the wave's next unit.  With no load-staging registers the
//    kernel fits 3-4 waves per SIMD: a wave that waits for a row leaves the VALU to the others.
//  * Both products are computed transposed on v_mfma_f32_16x16x32_f16:
//        S^T = K * Q^T   (A = K codes, row = token; B = Q, column = query head of the GQA group)
//        O^T = V^T * P^T (A = V codes, row = channel; B = P^T)
//    so the accumulator registers of the first product are, lane for lane, the B operand of the
//    second one: P never leaves registers.
//  * Codes are never multiplied out.  A dword of codes becomes four half2 registers holding
//    (offset + code) through a mask and an exponent OR (dequantize.h:59-166 uses the same magic
//    numbers); the per-channel K scale is folded into Q once per group, the per-token V scale is
//    folded into P, and the offset/zero terms become one scalar bias per head:
//        q.k_n   = sum_c (q_c*s_c)*(off + code) + sum_c q_c*z_c - sum_c (q_c*s_c)*off
//        o_c     = sum_n (p_n*s_n)*(off + code) + sum_n p_n*z_n - sum_n (p_n*s_n)*off
//  * q*scale and p*scale do not fit fp16 (11+11 significant bits), and their rounding error would
//    multiply the large code*scale terms of outlier channels.  Each product is therefore kept as
//    an exact pair hi + lo (lo = fma(a, b, -hi)).  The 16 MFMA columns hold the GQA group twice:
//    columns 0-7 carry the hi parts of heads 0-7, columns 8-15 the lo parts, so both go through
//    the same MFMA and are added afterwards with one row-rotate (lane ^ 8) per accumulator.
//  * The offset/zero biases and the softmax row sums are themselves computed on the MFMA pipe
//    (A operand = the zero vector / the constant offsets / ones), which keeps the VALU for the
//    code unpacking; this kernel is VALU-issue bound long before it is MFMA bound.
//  * Online softmax in base 2 per head (softmax.h:250-310) in steps of 64 tokens: running max
//    shared by the four lanes of a head through two lane-half swaps, accumulators rescaled only
//    when some head's max actually moved.
//  * The waves of a workgroup merge through LDS, one wave per query head; splits merge in the
//    same launch: that wave publishes the head's record (O / sum in fp16, max, sum) without waiting
//    for the stores, an idle wave has meanwhile drawn a ticket from the head's counter, and the wave
//    whose head got the last ticket loads all records of the head, checks that none of their words
//    still reads "not written" (zero) and combines them.
#include <hip/hip_runtime.h>
#include <atomic>
#include <stddef.h>
#include <stdint.h>

#include "kernels.h"
#include "layout.h"
#include "qpack_chunk.h"

namespace bitdecode {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned int u4 __attribute__((ext_vector_type(4)));

// Optional per-wave timeline for kernel tuning (built only with -DBITDECODE_PROF).
#ifdef BITDECODE_PROF
__device__ unsigned long long* g_prof = nullptr;
#define PROF_DECL unsigned long long prof_ts[16] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#define PROF(slot)                                 \
    do {                                           \
        __builtin_amdgcn_sched_barrier(0);         \
        prof_ts[slot] = wall_clock64();            \
        __builtin_amdgcn_sched_barrier(0);         \
    } while (0)
#define PROF_FLUSH()                                                                                  \
    do {                                                                                              \
        unsigned long long* pb = g_prof;                                                              \
        if (pb && (threadIdx.x & 63) == 0) {                                                          \
            pb += ((size_t)blockIdx.x * 16 + (threadIdx.x >> 6)) * 16;                                 \
            for (int i_ = 0; i_ < 16; ++i_) pb[i_] = prof_ts[i_];                                     \
        }                                                                                             \
    } while (0)
#define PROF_AT(pts, slot)                          \
    do {                                           \
        __builtin_amdgcn_sched_barrier(0);         \
        (pts)[slot] = wall_clock64();              \
        __builtin_amdgcn_sched_barrier(0);         \
    } while (0)
#define PROF_TS prof_ts
#else
#define PROF_AT(pts, slot) do { } while (0)
#define PROF_TS nullptr
#define PROF_DECL do { } while (0)
#define PROF(slot) do { } while (0)
#define PROF_FLUSH() do { } while (0)
#endif

// Probabilities are kept as 2^shift * exp2(s - max) in fp16, and p * (V scale) must stay inside the fp16
// range as well.  A 4-bit V scale is at most 131008 / 15 = 8734: p up to 4 is safe and keeps two more bits of
// the small probabilities.  A 2-bit V scale reaches 131008 / 3 = 43669: p stays at 1 or below.
constexpr float p_shift(int bits) { return bits == 4 ? 2.0f : 0.0f; }
constexpr int kLdsRowHalves = 136;

__device__ __forceinline__ h2 pk_rtz(float a, float b) {
    return __builtin_bit_cast(h2, __builtin_amdgcn_cvt_pkrtz(a, b));
}

// 16 bytes of fp16 (or bf16 converted to fp16; exact inside the fp16 normal range)
template <bool BF16>
__device__ __forceinline__ h8 cvt_h8(u4 raw) {
    if constexpr (BF16) {
        h8 r;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            h2 t = pk_rtz(__uint_as_float(raw[x] << 16), __uint_as_float(raw[x] & 0xffff0000u));
            r[2 * x] = t[0];
            r[2 * x + 1] = t[1];
        }
        return r;
    } else {
        return __builtin_bit_cast(h8, raw);
    }
}

// n / d with the host's magic number for d (kernels.h)
__device__ __forceinline__ int div_magic(int n, uint32_t magic) {
    // (a select, not a branch: the index arithmetic of the prologue stays one basic block)
    const uint32_t q = __umulhi(static_cast<uint32_t>(n), magic), keep = magic ? 0u : 0xffffffffu;
    return static_cast<int>((q & ~keep) | (static_cast<uint32_t>(n) & keep));
}

__device__ __forceinline__ u4 ld_u4(const void* p) { return *reinterpret_cast<const u4*>(p); }
// the same with the non-temporal hint, for rows that are read once and whole by one instruction
__device__ __forceinline__ u4 ld_u4_stream(const void* p) { return __builtin_nontemporal_load(reinterpret_cast<const u4*>(p)); }

// The exponent patterns that turn a masked code field into offset + code (fp16).  They are kept
// in VGPRs behind an empty asm so that (w & mask) | magic becomes one v_and_or_b32 (mask from an
// SGPR, magic from a VGPR) instead of an AND and an OR with two literals.
struct Magic {
    uint32_t e1024, e256, e64, e16;
    __device__ __forceinline__ Magic() : e1024(0x64006400u), e256(0x5c005c00u), e64(0x54005400u), e16(0x4c004c00u) {
        asm volatile("" : "+v"(e1024), "+v"(e256), "+v"(e64), "+v"(e16));
    }
};

// 8 four-bit codes -> (1024+c0, 1024+c4, 64+c1, 64+c5, 1024+c2, 1024+c6, 64+c3, 64+c7)
__device__ __forceinline__ h8 dq4(uint32_t w, const Magic& mg) {
    u4 r;
    r[0] = (w & 0x000f000fu) | mg.e1024;
    r[1] = (w & 0x00f000f0u) | mg.e64;
    const uint32_t w8 = w >> 8;
    r[2] = (w8 & 0x000f000fu) | mg.e1024;
    r[3] = (w8 & 0x00f000f0u) | mg.e64;
    return __builtin_bit_cast(h8, r);
}
// 16 two-bit codes -> two k-steps; offsets per element (1024,1024,256,256,64,64,16,16)
__device__ __forceinline__ void dq2(uint32_t w, h8& a0, h8& a1, const Magic& mg) {
    u4 r;
    r[0] = (w & 0x00030003u) | mg.e1024;
    r[1] = (w & 0x000c000cu) | mg.e256;
    r[2] = (w & 0x00300030u) | mg.e64;
    r[3] = (w & 0x00c000c0u) | mg.e16;
    a0 = __builtin_bit_cast(h8, r);
    const uint32_t w8 = w >> 8;
    r[0] = (w8 & 0x00030003u) | mg.e1024;
    r[1] = (w8 & 0x000c000cu) | mg.e256;
    r[2] = (w8 & 0x00300030u) | mg.e64;
    r[3] = (w8 & 0x00c000c0u) | mg.e16;
    a1 = __builtin_bit_cast(h8, r);
}

template <int BITS>
__device__ __forceinline__ h8 code_offsets() {
    if constexpr (BITS == 4) {
        return h8{1024, 1024, 64, 64, 1024, 1024, 64, 64};
    } else {
        return h8{1024, 1024, 256, 256, 64, 64, 16, 16};
    }
}

__device__ __forceinline__ f4 mfma32(h8 a, h8 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f4 mfma16(h4 a, h4 b, f4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0);
}

// value held by the partner column (lane ^ 8 inside each row of 16 lanes): DPP row_ror:8
__device__ __forceinline__ float partner(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, true));
}
// (every lane has a source lane, so the "bound control" flag changes nothing but tells the compiler
// that no previous value of the result survives, which saves it a move)
__device__ __forceinline__ uint32_t partner(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(x), 0x128, 0xf, 0xf, true));
}
// max over the four lanes that share a column (lane, lane^16, lane^32, lane^48).
// v_permlane16_swap exchanges the odd 16-lane rows of its first register with the even rows of
// its second one, v_permlane32_swap does the same with 32-lane halves; fed two copies of x they
// leave (rows 0,0,2,2 / rows 1,1,3,3) and (lower,lower / upper,upper), whose element-wise max is
// the reduction.  Written as asm: the compiler builtin folds the two results into one here.
// The s_nop covers the wait states the swap needs after a VALU write of its operands.
__device__ __forceinline__ float colmax(float x) {
    float y = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    x = fmaxf(x, y);
    y = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(x), "+v"(y));
    return fmaxf(x, y);
}

template <int NCG>
struct WaveState {
    float m;          // running max of the raw scores (q.k units) of this lane's head
    f4 l;             // sum of p, accumulated by MFMA against a ones operand (hi columns only)
    f4 ob[NCG];       // V bias per channel group, accumulated by MFMA (all four rows equal)
    f4 o[8];          // O^T tiles: lane (head, q) holds channels 16*ct + 4*q + r
};

// Online-softmax step over N raw scores t (q.k units); on return t holds
// p = 2^pshift * exp2(scale * (t - running max)).  Accumulators are rescaled only when the
// running max of some head moved (wave-uniform branch).  With HALVES the hi column and the lo
// column of a head hold different halves of the step's scores, and the maximum is taken over both.
template <int N, int NCG, bool HALVES = false>
__device__ __forceinline__ void softmax_step(float (&t)[N], float scale, WaveState<NCG>& st, float mx, float pshift) {
    if constexpr (HALVES) mx = fmaxf(mx, partner(mx));
    mx = colmax(mx);
    const float m_new = fmaxf(st.m, mx);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
    if (__builtin_amdgcn_ballot_w64(m_new > st.m) != 0) {
        const float alpha = __builtin_amdgcn_exp2f((st.m - m_use) * scale);
        st.l *= alpha;
#pragma unroll
        for (int c = 0; c < NCG; ++c) st.ob[c] *= alpha;
#pragma unroll
        for (int ct = 0; ct < 8; ++ct) st.o[ct] *= alpha;
        st.m = m_new;
    }
    const float c0 = pshift - m_use * scale;
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(t[i], scale, c0));
}
template <int N, int NCG>
__device__ __forceinline__ void softmax_step(float (&t)[N], float scale, WaveState<NCG>& st, float pshift) {
    float mx = t[0];
#pragma unroll
    for (int i = 1; i < N; ++i) mx = fmaxf(mx, t[i]);
    softmax_step<N, NCG>(t, scale, st, mx, pshift);
}

// Accumulators of the four S^T tiles of a 64-token step -> probabilities as operands of the second
// product, per 32-token sub-block ks: p16 (every column), pz (p in the hi columns, 0 in the lo ones),
// pm (the reverse).  Element i = 4*T + r of a sub-block is tile 2*ks + T, accumulator register r.
// A tile's hi and lo columns hold the two parts of its scores; their sum is the score.
//
// Plain form: every lane adds up the 16 scores of its head and takes the 16 exponentials, the lo
// column repeating what the hi column does.
template <int NCG>
__device__ __forceinline__ void step_probabilities(const f4 (&sc)[4], uint32_t hi_cols, float scale, WaveState<NCG>& st,
                                                   h8 (&p16)[2], h8 (&pz)[2], h8 (&pm)[2]) {
    float t[16];
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
#pragma unroll
        for (int r = 0; r < 4; ++r) t[4 * tt + r] = sc[tt][r] + partner(sc[tt][r]);
    }
    softmax_step<16, NCG>(t, scale, st, p_shift(4));
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        u4 pw;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            pw[x] = __builtin_bit_cast(uint32_t, pk_rtz(t[8 * ks + 2 * x], t[8 * ks + 2 * x + 1]));
        }
        p16[ks] = __builtin_bit_cast(h8, pw);
        pz[ks] = __builtin_bit_cast(h8, pw & hi_cols);
        pm[ks] = __builtin_bit_cast(h8, pw & ~hi_cols);
    }
}
// Shared form, same values: the hi column takes sub-block 0 and the lo column sub-block 1 (eight sums
// and exponentials per lane instead of sixteen), and the packed probabilities are exchanged
// afterwards.  The sums of sub-block 0 are made in every lane; DPP adds that write only the two
// upper banks of each row of 16 lanes then put the sums of sub-block 1 over them in the lo columns.
// The compiler does not see that the asm reads MFMA results: the block takes all of them as operands,
// so that it comes after the last MFMA, and waits out the longest MFMA-to-VALU distance itself.
// Pays where a wave works through many units (2-4 % at 2 bits), not with one 4-bit unit per wave.
template <int NCG>
__device__ __forceinline__ void step_probabilities_shared(const f4 (&sc)[4], uint32_t hi_cols, float scale,
                                                          WaveState<NCG>& st, h8 (&p16)[2], h8 (&pz)[2],
                                                          h8 (&pm)[2]) {
    float t[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = sc[i / 4][i % 4] + partner(sc[i / 4][i % 4]);
    float mx;      // maximum of the lane's eight sums
    asm volatile("s_nop 7\n\ts_nop 3\n\t"
                 "v_add_f32_dpp %0, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %1, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %2, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %3, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %4, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %5, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %6, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_add_f32_dpp %7, %16, %16 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                 "v_max3_f32 %8, %0, %1, %2\n\t"
                 "v_max3_f32 %8, %8, %3, %4\n\t"
                 "v_max3_f32 %8, %8, %5, %6\n\t"
                 "v_max_f32 %8, %8, %7"
                 : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]),
                   "=&v"(mx)
                 : "v"(sc[2][0]), "v"(sc[2][1]), "v"(sc[2][2]), "v"(sc[2][3]), "v"(sc[3][0]), "v"(sc[3][1]),
                   "v"(sc[3][2]), "v"(sc[3][3]));
    softmax_step<8, NCG, true>(t, scale, st, mx, p_shift(2));
    u4 pw;
#pragma unroll
    for (int x = 0; x < 4; ++x) pw[x] = __builtin_bit_cast(uint32_t, pk_rtz(t[2 * x], t[2 * x + 1]));
    const u4 z0 = pw & hi_cols;       // the hi columns hold sub-block 0
    const u4 m1 = pw & ~hi_cols;      // the lo columns hold sub-block 1
    u4 z1, m0;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        z1[x] = partner(m1[x]);
        m0[x] = partner(z0[x]);
    }
    pz[0] = __builtin_bit_cast(h8, z0);
    pm[0] = __builtin_bit_cast(h8, m0);
    pz[1] = __builtin_bit_cast(h8, z1);
    pm[1] = __builtin_bit_cast(h8, m1);
    p16[0] = __builtin_bit_cast(h8, z0 | m0);
    p16[1] = __builtin_bit_cast(h8, z1 | m1);
}

// ---------------------------------------------------------------------------------------------
// packed units, streamed through LDS
// ---------------------------------------------------------------------------------------------
// FEW: the variant with 8 waves per workgroup and a deeper row pipeline (see launch_fwd_tt)
template <int BITS, int GS, bool FEW = false>
struct UnitCfg {
    static constexpr int UT = unit_tokens(BITS);             // tokens per unit (4 KB of K codes, 4 KB of V codes)
    static constexpr int UPC = kChunk / UT;                  // units per 128-token chunk
    static constexpr int NSTEP = UT / 64;                    // 64-token steps per unit (one softmax pass each)
    static constexpr int TPS = 4;                            // 16-token tiles per step
    static constexpr int NKS = 2;                            // 32-token k-steps (V sub-blocks) per step
    static constexpr int RPS = 4 / NSTEP;                    // 1 KB rows of K codes (and of V codes) per step
    static constexpr int TPG = GS / 16;                      // tiles per K group
    static constexpr int NGU = UT > GS ? UT / GS : 1;        // K groups a unit touches
    static constexpr int NCG = kHeadDim / GS;                // V channel groups
    static constexpr int KPB = unit_k_param_bytes(BITS, GS); // K parameter bytes per unit
    static constexpr int VPB = unit_v_param_bytes(BITS, GS); // V parameter bytes per unit
    static constexpr int KPB_T = UT * NCG * 4;                // K parameter bytes per unit in "k-tensor" mode (per token)
    static constexpr int NKP = (KPB + 1023) / 1024;          // load instructions for the K parameters
    static constexpr int NVP = (VPB + 1023) / 1024;          // ... for the V parameters
    static constexpr int KSIDE = NKP + 4;                    // loads of a unit's K side (parameters, 4 code rows)
    static constexpr int VSIDE = NVP + 4;                    // ... of its V side
    // LDS region of a wave: K rows | V rows | K parameters, two slots | V parameters
    static constexpr int OFF_KP = 8192, OFF_VP = 8192 + 2 * KPB;
    static constexpr int REGION = unit_region_bytes(BITS, GS);
    static constexpr int NW = FEW ? 8 : decode_waves(BITS, GS);        // waves per workgroup
    static constexpr int WANT_DEPTH = FEW ? 6 : 4;
    static constexpr int DEPTH = WANT_DEPTH < NKP + RPS + 1 ? WANT_DEPTH : NKP + RPS + 1;   // rows a wave keeps in flight
    static_assert(REGION == OFF_VP + VPB && REGION % 256 == 0, "region layout");
    static_assert(KPB_T <= KPB && (KPB_T + 1023) / 1024 == NKP, "the per-token K parameters use the same rows");
    static_assert(NW % 4 == 0, "the merge reads four wave weights per LDS access");
};

// 16 bytes per lane from global memory straight into LDS: lane l reads base + OFFSET + 16*l and its
// data lands at lds_base + OFFSET + 16*l (the instruction's immediate offset applies to both sides).
// The base is wave-uniform and travels in SGPRs, the per-lane part is one shared VGPR
// (lane16 = 16*lane), so the addresses of a whole unit cost no vector registers.  M0 carries the
// LDS byte address of the row.  The loads carry the non-temporal hint: the stream is read once, and
// marking it so is 1.3-5 % faster on every workload (same-box A/B) than the default policy, which lets it
// displace the partial results and parameters from the caches.
template <int OFFSET>
__device__ __forceinline__ void dma_row(const uint8_t* base, uint32_t lane16, uint32_t lds_base) {
    static_assert(OFFSET >= 0 && OFFSET < 4096, "immediate offset field");
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3 nt"
                 :
                 : "v"(lane16), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_base)), "n"(OFFSET)
                 : "memory", "m0");
}

// The same with only the first LANES lanes taking part, for a last row that is not full.  The lane
// mask goes into EXEC around the load inside one asm block (SALU moves only): a branch around the
// load would split the basic block the scheduler works in.
template <int OFFSET, int LANES>
__device__ __forceinline__ void dma_row_first_lanes(const uint8_t* base, uint32_t lane16, uint32_t lds_base) {
    static_assert(OFFSET >= 0 && OFFSET < 4096 && LANES > 0 && LANES < 64, "immediate offset field, partial row");
    const uint64_t mask = (1ull << LANES) - 1;
    uint64_t saved;
    asm volatile("s_mov_b32 m0, %3\n\t"
                 "s_mov_b64 %0, exec\n\t"
                 "s_and_b64 exec, exec, %5\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:%4 nt\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(lane16), "s"(base), "s"(__builtin_amdgcn_readfirstlane(lds_base)), "n"(OFFSET), "s"(mask)
                 : "memory", "m0", "scc");
}

// All of this wave's LDS reads have returned their data.  A direct-to-LDS load may be given an LDS
// location only after that: a read that has merely been issued can still be overtaken by the load's
// write when the data comes from a near cache and the LDS queue is long (seen as rare wrong results
// with twelve waves of the 4-bit, group-32 kernel and L2-resident caches).
__device__ __forceinline__ void wait_lds_reads() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

// s_waitcnt vmcnt(n): at most n of this wave's loads still in flight.  The compiler does not
// track the asm loads above, so the waits are explicit; the memory clobber keeps LDS reads below.
template <int N>
__device__ __forceinline__ void wait_vm() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// the same for a count that is a constant only after loop unrolling (the switch folds away)
__device__ __forceinline__ void wait_vm_n(int n) {
    switch (n) {
        case 0: wait_vm<0>(); break;
        case 1: wait_vm<1>(); break;
        case 2: wait_vm<2>(); break;
        case 3: wait_vm<3>(); break;
        case 4: wait_vm<4>(); break;
        case 5: wait_vm<5>(); break;
        case 6: wait_vm<6>(); break;
        case 7: wait_vm<7>(); break;
        case 8: wait_vm<8>(); break;
        case 9: wait_vm<9>(); break;
        case 10: wait_vm<10>(); break;
        case 11: wait_vm<11>(); break;
        default: wait_vm<0>(); break;      // waiting for more than needed is always safe
    }
}

// A 16-byte global load the compiler does not track (so that its automatic waits do not count
// the direct-to-LDS loads above as its own).  The loaded registers must not be touched before the
// matching wait_then_take, which waits and only then copies them into registers the compiler may
// use freely: the copy happens inside the same asm block as the wait, so nothing can be scheduled
// between them.
__device__ __forceinline__ u4 load_untracked(const void* gaddr) {
    u4 r;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r) : "v"(gaddr) : "memory");
    return r;
}
template <int N>
__device__ __forceinline__ void wait_then_take(u4& dst_a, u4& dst_b, const u4& a, const u4& b) {
    typedef unsigned int u2 __attribute__((ext_vector_type(2)));
    u2 a0, a1, b0, b1;
    asm volatile(
        "s_waitcnt vmcnt(%8)\n\t"
        "v_mov_b64 %0, %4\n\t"
        "v_mov_b64 %1, %5\n\t"
        "v_mov_b64 %2, %6\n\t"
        "v_mov_b64 %3, %7"
        : "=&v"(a0), "=&v"(a1), "=&v"(b0), "=&v"(b1)
        : "v"(u2{a[0], a[1]}), "v"(u2{a[2], a[3]}), "v"(u2{b[0], b[1]}), "v"(u2{b[2], b[3]}), "n"(N)
        : "memory");
    dst_a = u4{a0[0], a0[1], a1[0], a1[1]};
    dst_b = u4{b0[0], b0[1], b1[0], b1[1]};
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (const __attribute__((address_space(3))) void*)p));
}

// Base addresses of one unit of one (batch, kv-head): K codes, V codes, K parameters, V parameters.  The
// rows behind them are fetched one by one in the order they are consumed (see "the rows of a unit as a
// pipeline" below).
template <int BITS, int GS>
struct UnitAddr {
    const uint8_t* kc;
    const uint8_t* vc;
    const uint8_t* kp;
    const uint8_t* vp;
};
template <int BITS, int GS, bool KT = false>
__device__ __forceinline__ UnitAddr<BITS, GS> unit_addr(const FwdParams& P, int bi, int hk, int u) {
    using C = UnitCfg<BITS, GS>;
    const int uic = u % C::UPC;
    // region and chunk inside it, as layout.h::chunk_place; a paged cache looks the page up in the block
    // table with a scalar load written out here: a load the compiler tracks would be a vector load, and its
    // wait would also drain the direct-to-LDS loads in flight
    int ci = u / C::UPC;
    int64_t bh = static_cast<int64_t>(bi) * P.hk + hk;
    if (P.block_table) {
        const int slot = ci / P.chunks_per_page;
        int page;
        asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)"
                     : "=s"(page) : "s"(P.block_table + bi * P.bt_stride + slot) : "memory");
        bh = static_cast<int64_t>(page) * P.hk + hk;
        ci -= slot * P.chunks_per_page;
    }
    UnitAddr<BITS, GS> A;      // wave-uniform: everything here lives in SGPRs
    A.kc = P.k_pack + bh * P.kpack_bh + static_cast<int64_t>(ci) * chunk_code_bytes(BITS) + uic * 4096;
    A.vc = P.v_pack + bh * P.vpack_bh + static_cast<int64_t>(ci) * chunk_code_bytes(BITS) + uic * 4096;
    if constexpr (KT) {      // per-token K parameters: [64-token half][channel group][tile][token] per chunk
        A.kp = P.k_params + bh * P.kparams_bh + static_cast<int64_t>(ci) * v_param_chunk_bytes(GS) + uic * C::KPB_T;
    } else {
        A.kp = P.k_params + bh * P.kparams_bh +
               (static_cast<int64_t>(ci) * (kChunk / GS) + (uic * C::UT) / GS) * kKParamGroupBytes;
    }
    A.vp = P.v_params + bh * P.vparams_bh + static_cast<int64_t>(ci) * v_param_chunk_bytes(GS) + uic * C::VPB;
    return A;
}
// BYTES contiguous bytes (a multiple of 256) into LDS: whole 1 KB rows, the last one with only the
// first lanes, those that still have data.  Every wave executes every instruction, so the vmcnt
// bookkeeping below holds.
template <int BYTES, int R = 0>
__device__ __forceinline__ void dma_bytes(const uint8_t* src, uint32_t lane16, uint32_t lds_dst) {
    if constexpr (R * 1024 < BYTES) {
        constexpr int left = BYTES - R * 1024;
        if constexpr (left >= 1024) {
            dma_row<R * 1024>(src, lane16, lds_dst);
        } else {
            dma_row_first_lanes<R * 1024, left / 16>(src, lane16, lds_dst);
        }
        dma_bytes<BYTES, R + 1>(src, lane16, lds_dst);
    }
}
// ---- the rows of a unit as a pipeline
// A compute unit returns loads in the order it issued them, accepts only about 64 KB of them at a time,
// and while a wave's load waits to be accepted no other wave of that SIMD gets an LDS instruction
// through (measured: LDS reads of all waves stall for as long as load instructions queue up).  So a wave
// never sends a whole unit at once.  The rows of a unit are numbered in the order they are consumed:
//   K parameters | per 64-token step: its K rows, (first step: V parameters,) its V rows
// and a wave keeps kDepth of them in flight: the prologue issues rows 0 .. kDepth-2 of the wave's first
// unit, and just before the wave waits for row i it issues row i + kDepth - 1 (running on into the next
// unit of the wave).  With all waves of a workgroup doing this the rows of different waves interleave in
// the memory queue, the waves finish together, and what is left after the last byte of the stream is the
// work on one row per wave.  Before row i is read exactly kDepth - 1 younger loads may still be in flight
// (fewer at the end of the wave's last unit), which is what the s_waitcnt in front of every read says.

struct RowId {
    int kind;      // 0 K parameters, 1 K codes, 2 V parameters, 3 V codes
    int idx;       // 1 KB row inside its kind
};
template <int BITS, int GS>
constexpr RowId row_at(int i) {
    using C = UnitCfg<BITS, GS>;
    if (i < C::NKP) return RowId{0, i};
    int p = i - C::NKP;
    for (int s = 0; s < C::NSTEP; ++s) {
        if (p < C::RPS) return RowId{1, s * C::RPS + p};
        p -= C::RPS;
        if (s == 0) {
            if (p < C::NVP) return RowId{2, p};
            p -= C::NVP;
        }
        if (p < C::RPS) return RowId{3, s * C::RPS + p};
        p -= C::RPS;
    }
    return RowId{-1, 0};
}
// position of a row in that order
template <int BITS, int GS>
constexpr int pos_of(int kind, int idx) {
    using C = UnitCfg<BITS, GS>;
    for (int i = 0; i < C::KSIDE + C::VSIDE; ++i) {
        const RowId r = row_at<BITS, GS>(i);
        if (r.kind == kind && r.idx == idx) return i;
    }
    return -1;
}
// the load of row I of a unit into the wave's region; kslot names the K-parameter slot of that unit
template <int BITS, int GS, int I, bool KT = false>
__device__ __forceinline__ void issue_row(const UnitAddr<BITS, GS>& A, uint32_t lane16, uint32_t region, int kslot) {
    using C = UnitCfg<BITS, GS>;
    constexpr RowId r = row_at<BITS, GS>(I);
    static_assert(r.kind >= 0, "row inside the unit");
    if constexpr (r.kind == 0) {
        constexpr int left = (KT ? C::KPB_T : C::KPB) - r.idx * 1024;
        const uint32_t dst = region + C::OFF_KP + kslot * C::KPB;
        if constexpr (left >= 1024) {
            dma_row<r.idx * 1024>(A.kp, lane16, dst);
        } else {
            dma_row_first_lanes<r.idx * 1024, left / 16>(A.kp, lane16, dst);
        }
    } else if constexpr (r.kind == 1) {
        dma_row<r.idx * 1024>(A.kc, lane16, region);
    } else if constexpr (r.kind == 2) {
        constexpr int left = C::VPB - r.idx * 1024;
        if constexpr (left >= 1024) {
            dma_row<r.idx * 1024>(A.vp, lane16, region + C::OFF_VP);
        } else {
            dma_row_first_lanes<r.idx * 1024, left / 16>(A.vp, lane16, region + C::OFF_VP);
        }
    } else {
        dma_row<r.idx * 1024>(A.vc, lane16, region + 4096);
    }
}
// prologue of a wave: rows 0 .. kDepth-2 of its first unit
template <int BITS, int GS, bool KT = false, bool FEW = false, int I = 0>
__device__ __forceinline__ void issue_first_rows(const UnitAddr<BITS, GS>& A, uint32_t lane16, uint32_t region) {
    if constexpr (I < UnitCfg<BITS, GS, FEW>::DEPTH - 1) {
        issue_row<BITS, GS, I, KT>(A, lane16, region, 0);
        issue_first_rows<BITS, GS, KT, FEW, I + 1>(A, lane16, region);
    }
}
// In front of the read of row I of the current unit: send the row that keeps the pipeline full (of this
// unit, or of the next one if there is one), then wait until row I has landed.  The load may overwrite
// rows read earlier: every LDS read issued so far has to have returned its data first (a read that has
// only been issued can be overtaken by the load's write).
template <int BITS, int GS, bool HAS_NEXT, int I, bool KT = false, bool FEW = false>
__device__ __forceinline__ void row_ready(const UnitAddr<BITS, GS>& cur, const UnitAddr<BITS, GS>& next, uint32_t lane16,
                                          uint32_t region, int kslot) {
    using C = UnitCfg<BITS, GS, FEW>;
    constexpr int ROWS = C::KSIDE + C::VSIDE, kDepth = C::DEPTH, J = I + kDepth - 1;
    // rows of the next unit fetched from inside this one land on K-side rows only: the V parameters of this
    // unit are still in use up to its last row
    static_assert(kDepth - 1 <= C::NKP + C::RPS && kDepth - 1 < ROWS, "depth of the row pipeline");
    if constexpr (J < ROWS) {
        wait_lds_reads();
        issue_row<BITS, GS, J, KT>(cur, lane16, region, kslot);
        wait_vm<kDepth - 1>();
    } else if constexpr (HAS_NEXT) {
        wait_lds_reads();
        issue_row<BITS, GS, J - ROWS, KT>(next, lane16, region, kslot ^ 1);
        wait_vm<kDepth - 1>();
    } else {
        wait_vm<ROWS - 1 - I>();
    }
}

// Per-group state of the K side: Q with the group's scale folded in (exact hi/lo split) and the
// score bias  sum_c q_c*zero_c - sum_c (q_c*scale_c)*offset_c  built on the MFMA pipe.
struct KGroup {
    h8 qp[4];
    f4 kb;
};

// The workgroup's LDS copy of q: rows 0-7 = the eight head slots of the GQA group ([128] fp16
// values each; slots past the group repeat head 0 and are never written out), row 8 = zeros.
// A lane reads q three ways without any select: plain (its head), hi-only (zero row in the lo
// columns) and lo-only (zero row in the hi columns).
struct QRows {
    const uint8_t* q;    // row of this lane's head
    const uint8_t* qz;   // same row in the hi columns, zero row in the lo columns
    const uint8_t* qm;   // zero row in the hi columns, same row in the lo columns
};
// Rows are 272 bytes apart (256 + 16 of padding) so that the eight heads read by neighbouring
// lanes fall into different LDS banks.
constexpr int kQRowBytes = 272;
__device__ __forceinline__ QRows q_rows(const uint8_t* sq, int head, int kg, bool lo_part) {
    const uint8_t* row = sq + head * kQRowBytes + kg * 16;
    const uint8_t* zero = sq + 8 * kQRowBytes + kg * 16;
    return QRows{row, lo_part ? zero : row, lo_part ? row : zero};
}
__device__ __forceinline__ h8 q_load(const uint8_t* row, int j) {
    return __builtin_bit_cast(h8, *reinterpret_cast<const u4*>(row + 64 * j));
}

// a*b as an exact fp16 pair: hi columns get hi = round(a*b), lo columns get fma(a, b, -hi).
// a_lo_only is a in the lo columns and 0 in the hi columns, so no lane select is needed.
__device__ __forceinline__ h8 split_mul_masked(h8 a, h8 a_lo_only, h8 b) {
    const h8 hi_in_lo_cols = a_lo_only * b;
    return __builtin_elementwise_fma(a, b, -hi_in_lo_cols);
}

template <int BITS, bool BF16>
__device__ __forceinline__ void start_group(KGroup& G, const uint8_t* kpar, const QRows& Q, int kg) {
    const h8 noff = -code_offsets<BITS>();
    G.kb = f4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const h8 sc = cvt_h8<false>(*reinterpret_cast<const u4*>(kpar + (32 * j + 8 * kg) * 2));
        const h8 zr = cvt_h8<false>(*reinterpret_cast<const u4*>(kpar + 256 + (32 * j + 8 * kg) * 2));
        G.qp[j] = split_mul_masked(q_load(Q.q, j), q_load(Q.qm, j), sc);
        G.kb = mfma32(zr, q_load(Q.qz, j), G.kb);
        G.kb = mfma32(noff, G.qp[j], G.kb);
    }
}

// One packed unit from the wave's LDS region, in 64-token steps: S^T tiles of the step, online
// softmax update, O^T += V^T P^T for the same tokens.  Scores stay in q.k units; the softmax
// scale is applied inside the exponent.  On entry rows 0 .. kDepth-2 of the unit are in flight or landed;
// with HAS_NEXT the first rows of the wave's next unit are issued from here (see above); kslot says
// which K-parameter slot the current unit uses.
// With KT ("k-tensor" mode: K parameters per token and channel group) the K scale cannot be folded into q:
// a tile's raw sums  sum_c (offset + code) q_c  are taken per channel group with q as it is (hi columns
// only: q is exact in fp16), and each of the tile's tokens then applies its own scale and zero,
//   score = sum_g scale_g * (raw_g - sum_c offset_c q_c) + zero_g * sum_c q_c   (c in group g),
// with the two q sums of every group prepared once per wave (KQ).
template <int NCG>
struct TokenQ {
    h8 q[4];          // q of the lane's head in the hi columns, zero in the lo columns
    float noffq[NCG]; // - sum_c offset_c q_c per channel group, for the lane's column
    float qsum[NCG];  //   sum_c q_c
};
template <int BITS, int NCG>
__device__ __forceinline__ TokenQ<NCG> token_q(const QRows& Q) {
    TokenQ<NCG> T;
    const h8 noff = -code_offsets<BITS>();
    const h8 ones = h8{1, 1, 1, 1, 1, 1, 1, 1};
    f4 no[NCG], qs[NCG];       // every row of these products is the same
#pragma unroll
    for (int c = 0; c < NCG; ++c) no[c] = qs[c] = f4{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        T.q[j] = q_load(Q.qz, j);
        no[j * NCG / 4] = mfma32(noff, T.q[j], no[j * NCG / 4]);
        qs[j * NCG / 4] = mfma32(ones, T.q[j], qs[j * NCG / 4]);
    }
#pragma unroll
    for (int c = 0; c < NCG; ++c) {
        T.noffq[c] = no[c][0];
        T.qsum[c] = qs[c][0];
    }
    return T;
}

template <int BITS, int GS, bool BF16, bool HAS_NEXT, bool KT = false, bool FEW = false>
__device__ __forceinline__ void compute_unit(const uint8_t* reg, uint32_t region_lds, int kslot,
                                             const UnitAddr<BITS, GS>& cur, const UnitAddr<BITS, GS>& next,
                                             const QRows& Q, const FwdParams& P, int lane, bool lo_part, const Magic& mg,
                                             WaveState<kHeadDim / GS>& st, const TokenQ<kHeadDim / GS>* KQ = nullptr) {
    using C = UnitCfg<BITS, GS>;
    constexpr int NCG = C::NCG, TPS = C::TPS, NKS = C::NKS, TPG = C::TPG, CTPG = GS / 16;
    constexpr int NSTEP = C::NSTEP, RPS = C::RPS, TPR = TPS / RPS;      // tiles per K row
    const int kg = lane >> 4;
    const uint32_t lane16 = lane * 16;
    const h8 noff = -code_offsets<BITS>();
    const h8 ones = h8{1, 1, 1, 1, 1, 1, 1, 1};
    const uint32_t hi_cols = lo_part ? 0u : 0xffffffffu;
    const u4* kcode = reinterpret_cast<const u4*>(reg) + lane;             // row r: kcode[64 * r]
    const u4* vcode = reinterpret_cast<const u4*>(reg + 4096) + lane;
    const uint8_t* kpar = reg + C::OFF_KP + kslot * C::KPB;
    const uint8_t* vpar = reg + C::OFF_VP + kg * 16;
#define ROW_READY(kind, idx) row_ready<BITS, GS, HAS_NEXT, pos_of<BITS, GS>(kind, idx), KT, FEW>(cur, next, lane16, region_lds, kslot)

    // the K parameters lead the queue: the first K group is prepared while the code rows arrive
#pragma unroll
    for (int i = 0; i < C::NKP; ++i) {
        if (i == 0) ROW_READY(0, 0);
        if (i == 1) ROW_READY(0, 1);
    }
    static_assert(C::NKP <= 2 && C::NVP <= 2, "parameter rows of a unit");
    KGroup G;
    if constexpr (!KT) start_group<BITS, BF16>(G, kpar, Q, kg);
#pragma unroll
    for (int step = 0; step < NSTEP; ++step) {
        f4 sc[TPS];
#pragma unroll
        for (int tt = 0; tt < TPS; ++tt) {
            const int tile = step * TPS + tt;
            if (tt % TPR == 0) {       // the K row of this tile (4 bits: one tile per row, 2 bits: two)
                const int row = tile / TPR;
                if (row == 0) ROW_READY(1, 0);
                if (row == 1) ROW_READY(1, 1);
                if (row == 2) ROW_READY(1, 2);
                if (row == 3) ROW_READY(1, 3);
            }
            if constexpr (KT) {
                static_assert(!KT || BITS == 4, "per-token K parameters: 4 bits only");
                const u4 w = kcode[64 * tile];
                f4 raw[NCG];
#pragma unroll
                for (int c = 0; c < NCG; ++c) raw[c] = f4{KQ->noffq[c], KQ->noffq[c], KQ->noffq[c], KQ->noffq[c]};
#pragma unroll
                for (int j = 0; j < 4; ++j) raw[j * NCG / 4] = mfma32(dq4(w[j], mg), KQ->q[j], raw[j * NCG / 4]);
                f4 acc = {0, 0, 0, 0};
#pragma unroll
                for (int c = 0; c < NCG; ++c) {
                    // (scale, zero) of the tile's tokens 4*kg .. 4*kg+3 for channel group c
                    const h8 pr = *reinterpret_cast<const h8*>(kpar + (c * 4 + tile) * 64 + kg * 16);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        acc[r] = __builtin_fmaf(static_cast<float>(pr[2 * r]), raw[c][r],
                                                __builtin_fmaf(static_cast<float>(pr[2 * r + 1]), KQ->qsum[c], acc[r]));
                    }
                }
                sc[tt] = acc;
                continue;
            }
            if (tile != 0 && tile % TPG == 0) {
                start_group<BITS, BF16>(G, kpar + ((tile * 16) / GS) * kKParamGroupBytes, Q, kg);
            }
            f4 acc = G.kb;
            if constexpr (BITS == 4) {
                const u4 w = kcode[64 * tile];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc = mfma32(dq4(w[j], mg), G.qp[j], acc);
            } else {
                const u4 w = kcode[64 * (tile / 2)];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    h8 a0, a1;
                    dq2(w[2 * (tile % 2) + jj], a0, a1, mg);
                    acc = mfma32(a0, G.qp[2 * jj], acc);
                    acc = mfma32(a1, G.qp[2 * jj + 1], acc);
                }
            }
            sc[tt] = acc;
        }

        static_assert(TPS == 4 && NKS == 2, "four tiles, two sub-blocks per step");
        h8 p16[NKS], pz[NKS], pm[NKS];
        if constexpr (BITS == 2) {
            step_probabilities_shared<NCG>(sc, hi_cols, P.scale_log2, st, p16, pz, pm);
        } else {
            step_probabilities<NCG>(sc, hi_cols, P.scale_log2, st, p16, pz, pm);
        }
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) st.l = mfma32(ones, pz[ks], st.l);
        // V side of the step, row by row.  A row holds one channel half (tiles ct = 4*hf .. 4*hf+3) of one
        // 32-token sub-block (4 bits) or of the whole step (2 bits).
        if (step == 0) {
#pragma unroll
            for (int i = 0; i < C::NVP; ++i) {
                if (i == 0) ROW_READY(2, 0);
                if (i == 1) ROW_READY(2, 1);
            }
        }
        h8 pp[NCG][NKS];
        constexpr int CGH = NCG >= 2 ? NCG / 2 : 1;      // channel groups per channel half
#pragma unroll
        for (int r = 0; r < RPS; ++r) {
            const int hf = r % 2;
            const int ksr = (BITS == 4) ? r / 2 : 0;     // 4 bits: the row's sub-block
            // p * scale (exact hi/lo pair) and the bias terms of the channel groups this row starts
#pragma unroll
            for (int c = 0; c < CGH; ++c) {
                const int cg = NCG >= 2 ? hf * CGH + c : 0;
                if (NCG >= 2 || hf == 0) {
#pragma unroll
                    for (int ks = (BITS == 4 ? ksr : 0); ks < (BITS == 4 ? ksr + 1 : NKS); ++ks) {
                        const int sb = step * NKS + ks;               // 32-token sub-block inside the unit
                        const u4 rs = *reinterpret_cast<const u4*>(vpar + (sb * NCG + cg) * 128);
                        const u4 rz = *reinterpret_cast<const u4*>(vpar + (sb * NCG + cg) * 128 + 64);
                        pp[cg][ks] = split_mul_masked(p16[ks], pm[ks], cvt_h8<false>(rs));
                        st.ob[cg] = mfma32(cvt_h8<false>(rz), pz[ks], st.ob[cg]);
                        st.ob[cg] = mfma32(noff, pp[cg][ks], st.ob[cg]);
                    }
                }
            }
            const int vrow = step * RPS + r;
            if (vrow == 0) ROW_READY(3, 0);
            if (vrow == 1) ROW_READY(3, 1);
            if (vrow == 2) ROW_READY(3, 2);
            if (vrow == 3) ROW_READY(3, 3);
            const u4 w = vcode[64 * vrow];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int ct = 4 * hf + x, cg = ct / CTPG;
                if constexpr (BITS == 4) {
                    st.o[ct] = mfma32(dq4(w[x], mg), pp[cg][ksr], st.o[ct]);
                } else {
                    h8 a0, a1;
                    dq2(w[x], a0, a1, mg);
                    st.o[ct] = mfma32(a0, pp[cg][0], st.o[ct]);
                    st.o[ct] = mfma32(a1, pp[cg][1], st.o[ct]);
                }
            }
        }
    }
#undef ROW_READY
}

// Fields of the kernel's parameter block, re-read from the kernarg segment at the point of use.  The
// fields that only the append needs would otherwise sit in scalar registers through the whole kernel
// (the compiler loads every kernel argument up front), and the unit loop has none to spare: they get
// spilled to vector-register lanes inside it.  Scalar loads, written out so that they stay where they
// are; the kernel's only argument is the FwdParams block, at offset 0 of the segment.
template <int OFF>
__device__ __forceinline__ uint32_t karg_u32() {
    uint32_t v;
    asm volatile("s_load_dword %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                 : "=s"(v) : "s"(__builtin_amdgcn_kernarg_segment_ptr()), "n"(OFF) : "memory");
    return v;
}
template <int OFF>
__device__ __forceinline__ uint64_t karg_u64() {
    uint64_t v;
    asm volatile("s_load_dwordx2 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                 : "=s"(v) : "s"(__builtin_amdgcn_kernarg_segment_ptr()), "n"(OFF) : "memory");
    return v;
}
// sixteen consecutive dwords in one load, and a field picked out of them
typedef uint32_t kblock __attribute__((ext_vector_type(16)));
template <int OFF>
__device__ __forceinline__ kblock karg_block() {
    static_assert(OFF % 4 == 0 && OFF + 64 <= static_cast<int>(sizeof(FwdParams)), "inside the parameter block");
    kblock v;
    asm volatile("s_load_dwordx16 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                 : "=s"(v) : "s"(__builtin_amdgcn_kernarg_segment_ptr()), "n"(OFF) : "memory");
    return v;
}
// A value that an asm block delivered in scalar registers, told to the compiler as wave-uniform: it takes the
// results of an asm statement for lane-dependent and would carry everything computed from them (addresses above
// all) in vector registers.  The halves of a 64-bit value are widened as unsigned.
__device__ __forceinline__ uint32_t uni32(uint32_t x) {
    return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(x)));
}
__device__ __forceinline__ uint64_t uni64(uint64_t x) {
    return static_cast<uint64_t>(uni32(static_cast<uint32_t>(x))) | (static_cast<uint64_t>(uni32(static_cast<uint32_t>(x >> 32))) << 32);
}
template <int OFF, int FIELD_OFF>
__device__ __forceinline__ uint64_t block_u64(const kblock& v) {
    static_assert(FIELD_OFF >= OFF && FIELD_OFF + 8 <= OFF + 64 && (FIELD_OFF - OFF) % 4 == 0, "field inside the block");
    return v[(FIELD_OFF - OFF) / 4] | (static_cast<uint64_t>(v[(FIELD_OFF - OFF) / 4 + 1]) << 32);
}
template <int OFF, int FIELD_OFF>
__device__ __forceinline__ uint32_t block_u32(const kblock& v) {
    static_assert(FIELD_OFF >= OFF && FIELD_OFF + 4 <= OFF + 64 && (FIELD_OFF - OFF) % 4 == 0, "field inside the block");
    return v[(FIELD_OFF - OFF) / 4];
}
#define BLOCK_AT(field) offsetof(FwdParams, field)
#define BLOCK_PTR(type, blk, first, field) reinterpret_cast<type>(uni64(block_u64<BLOCK_AT(first), BLOCK_AT(field)>(blk)))
#define BLOCK_I64(blk, first, field) static_cast<int64_t>(uni64(block_u64<BLOCK_AT(first), BLOCK_AT(field)>(blk)))
#define BLOCK_I32(blk, first, field) static_cast<int>(uni32(block_u32<BLOCK_AT(first), BLOCK_AT(field)>(blk)))
#define LATE_I32(field) static_cast<int>(uni32(karg_u32<offsetof(FwdParams, field)>()))
#define LATE_I64(field) static_cast<int64_t>(uni64(karg_u64<offsetof(FwdParams, field)>()))
#define LATE_PTR(type, field) reinterpret_cast<type>(uni64(karg_u64<offsetof(FwdParams, field)>()))

// ---------------------------------------------------------------------------------------------
// 16-token tiles of the fp16 residual window (tokens n0 .. n0+15, valid below R)
// ---------------------------------------------------------------------------------------------
struct Fp16Tile {
    u4 k[4];   // lane (token col, kg): channels 32*j + 8*kg .. +7
    u4 v[4];   // lane (kg, col): token 4*x + kg, channels 8*col .. +7
};

// Where the window's rows are, for one (batch, kv-head).  With APPEND the window's row r_new is not in
// the window yet: it is the step's new token (kn, vn).
struct WindowSrc {
    const uint16_t* kr;
    const uint16_t* vr;
    int64_t k_st, v_st;
    const uint16_t* kn;
    const uint16_t* vn;
};
template <bool APPEND, bool LATE>
__device__ __forceinline__ WindowSrc window_src(const FwdParams& P, int bi, int hk) {
    WindowSrc W;
    if constexpr (!LATE) {
        W.kr = P.k_res + bi * P.kres_sb + hk * P.kres_sh;
        W.vr = P.v_res + bi * P.vres_sb + hk * P.vres_sh;
        W.k_st = P.kres_st;
        W.v_st = P.vres_st;
        W.kn = W.vn = nullptr;
        return W;
    }
    // The decode step needs more parameter fields than the scalar registers hold next to the unit loop's
    // state: what the loop does not use is fetched from the kernarg segment only here.
    const kblock kb = karg_block<BLOCK_AT(k_res)>();      // k_res ... vres_sh
    W.kr = BLOCK_PTR(const uint16_t*, kb, k_res, k_res) + bi * BLOCK_I64(kb, k_res, kres_sb) +
           hk * BLOCK_I64(kb, k_res, kres_sh);
    W.vr = BLOCK_PTR(const uint16_t*, kb, k_res, v_res) + bi * BLOCK_I64(kb, k_res, vres_sb) +
           hk * BLOCK_I64(kb, k_res, vres_sh);
    W.k_st = BLOCK_I64(kb, k_res, kres_st);
    W.v_st = BLOCK_I64(kb, k_res, vres_st);
    W.kn = W.vn = nullptr;
    if constexpr (APPEND) {
        W.kn = LATE_PTR(const uint16_t*, k_new) + bi * LATE_I64(knew_sb) + hk * LATE_I64(knew_sh);
        W.vn = LATE_PTR(const uint16_t*, v_new) + bi * LATE_I64(vnew_sb) + hk * LATE_I64(vnew_sh);
    }
    return W;
}
template <bool APPEND>
__device__ __forceinline__ void load_fp16_tile(Fp16Tile& T, const WindowSrc& W, int n0, int R, int lane, int r_new) {
    const int col = lane & 15, kg = lane >> 4;
    const int tok = n0 + col;
    const uint16_t* krow = (APPEND && tok == r_new) ? W.kn : W.kr + static_cast<int64_t>(tok) * W.k_st;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        T.k[j] = u4{0, 0, 0, 0};
        // default cache policy: an instruction takes 64 bytes of each token's 256-byte row, the other three
        // instructions find the rest of the lines in the cache (with the hint the fp16-only path is 5-8 % slower)
        if (tok < R) T.k[j] = ld_u4(krow + 32 * j + 8 * kg);
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const int tv = n0 + 4 * x + kg;
        const uint16_t* vrow = (APPEND && tv == r_new) ? W.vn : W.vr + static_cast<int64_t>(tv) * W.v_st;
        T.v[x] = u4{0, 0, 0, 0};
        // 16 lanes take a token's whole row: streamed (6-9 % faster on the fp16-only path, 0-1.5 % with a packed prefix)
        if (tv < R) T.v[x] = ld_u4_stream(vrow + col * 8);
    }
}

template <bool BF16, int NCG>
__device__ __forceinline__ void fp16_tile(const Fp16Tile& T, const FwdParams& P, int n0, int R, int lane,
                                          const QRows& Q, bool lo_part, WaveState<NCG>& st, uint16_t* lds, float pshift) {
    const int col = lane & 15, kg = lane >> 4;

    // V tile (16 tokens x 128 channels) goes through this wave's LDS slab to be read back
    // token-contiguous per channel (the MFMA A operand wants 4 tokens of one channel per lane).
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        *reinterpret_cast<u4*>(&lds[(4 * x + kg) * kLdsRowHalves + col * 8]) = T.v[x];
    }
    __builtin_amdgcn_wave_barrier();

    float s[4];
    {
        f4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // fp16 operands are exact: only the hi columns carry q
            acc = mfma32(cvt_h8<BF16>(T.k[j]), q_load(Q.qz, j), acc);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tk = n0 + 4 * kg + r;
            float tot = acc[r] + partner(acc[r]);   // outside the select: every lane executes the DPP
            s[r] = tk < R ? tot : -INFINITY;
        }
    }
    softmax_step<4, NCG>(s, P.scale_log2, st, pshift);
    const h2 p01 = pk_rtz(s[0], s[1]), p23 = pk_rtz(s[2], s[3]);
    h4 pb = {p01[0], p01[1], p23[0], p23[1]};
    if (lo_part) pb = h4{0, 0, 0, 0};
    st.l = mfma16(h4{1, 1, 1, 1}, pb, st.l);
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
        uint16_t e[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = lds[(4 * kg + i) * kLdsRowHalves + 16 * ct + col];
        h4 a;
        if constexpr (BF16) {
            h2 t0 = pk_rtz(__uint_as_float(static_cast<uint32_t>(e[0]) << 16),
                           __uint_as_float(static_cast<uint32_t>(e[1]) << 16));
            h2 t1 = pk_rtz(__uint_as_float(static_cast<uint32_t>(e[2]) << 16),
                           __uint_as_float(static_cast<uint32_t>(e[3]) << 16));
            a = h4{t0[0], t0[1], t1[0], t1[1]};
        } else {
            a = h4{__builtin_bit_cast(_Float16, e[0]), __builtin_bit_cast(_Float16, e[1]),
                   __builtin_bit_cast(_Float16, e[2]), __builtin_bit_cast(_Float16, e[3])};
        }
        st.o[ct] = mfma16(a, pb, st.o[ct]);
    }
}

// device-scope (agent) relaxed accesses of 8 bytes: write-through stores / loads served from the
// level all compute units share
__device__ __forceinline__ void st_dev2(float* p, float a, float b) {
    const uint64_t bits = __float_as_uint(a) | (static_cast<uint64_t>(__float_as_uint(b)) << 32);
    __hip_atomic_store(reinterpret_cast<uint64_t*>(p), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 ld_dev2(const float* p) {
    const uint64_t bits = __hip_atomic_load(reinterpret_cast<const uint64_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return float2{__uint_as_float(static_cast<uint32_t>(bits)), __uint_as_float(static_cast<uint32_t>(bits >> 32))};
}

// the same for 4 bytes
__device__ __forceinline__ void st_dev1(uint32_t* p, uint32_t v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A split's partial output as it crosses workgroups: normalised (O / L: a weighted mean of V rows, so inside the
// value range of V whatever the split's length) and rounded to nearest fp16, two channels per 32-bit word: half
// the bytes of fp32 partials for the workgroup that merges g x splits of them through one compute unit's memory
// path.  The rounding is at most 2^-11 of the value; a split whose output reaches 2 in some channel (so that the
// rounding could exceed 4.9e-4) also sends the residuals `lo` = value - hi, again as fp16 (22 significant bits
// together), which the merging wave adds: splits of large outputs that cancel stay inside the error bar (the
// reference keeps its partial outputs in fp32, flash_fwd_kernel.h:1280-1298).
// An all-zero word means "not written": (+0, +0) travels as (+0, -0), which adds up to the same sums.
__device__ __forceinline__ uint32_t pack_h2_nonzero(_Float16 a, _Float16 b) {
    const uint32_t w = static_cast<uint32_t>(__builtin_bit_cast(uint16_t, a)) | (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, b)) << 16);
    return w ? w : 0x80000000u;
}
struct PartialWords {
    float n0, n1;      // the normalised values
    _Float16 a, b;     // ... rounded
    __device__ __forceinline__ PartialWords(float O0, float O1, float L) {
        const float inv = L > 0.0f ? __builtin_amdgcn_rcpf(L) : 0.0f;
        n0 = O0 * inv;
        n1 = O1 * inv;
        a = static_cast<_Float16>(n0);
        b = static_cast<_Float16>(n1);
    }
    __device__ __forceinline__ uint32_t hi() const { return pack_h2_nonzero(a, b); }
    __device__ __forceinline__ uint32_t lo() const {
        return pack_h2_nonzero(static_cast<_Float16>(n0 - static_cast<float>(a)), static_cast<_Float16>(n1 - static_cast<float>(b)));
    }
    // some lane's value reaches the magnitude from which the residual words are sent
    __device__ __forceinline__ bool large(float from) const {
        return __builtin_amdgcn_ballot_w64(fmaxf(__builtin_fabsf(n0), __builtin_fabsf(n1)) >= from) != 0;
    }
};
constexpr float kPartialLoFrom = 2.0f;      // a split sends the residual words from this output magnitude on
__device__ __forceinline__ float half_lo(uint32_t w) { return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w))); }
__device__ __forceinline__ float half_hi(uint32_t w) { return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(w >> 16))); }

// x of lane `l` (wave-uniform index) as a scalar
__device__ __forceinline__ float lane_value(float x, int l) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), l));
}
// DPP row rotation: value of lane (l + N) % 16 of the same row of 16 lanes
template <int N>
__device__ __forceinline__ float row_ror(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + N, 0xf, 0xf, true));
}
// reductions over each row of 16 lanes, result in every lane of the row; the additions are grouped the
// same way in every run
__device__ __forceinline__ float row_max16(float x) {
    x = fmaxf(x, row_ror<8>(x));
    x = fmaxf(x, row_ror<4>(x));
    x = fmaxf(x, row_ror<2>(x));
    return fmaxf(x, row_ror<1>(x));
}
__device__ __forceinline__ float row_sum16(float x) {
    x += row_ror<8>(x);
    x += row_ror<4>(x);
    x += row_ror<2>(x);
    return x + row_ror<1>(x);
}
// the maximum over the whole wave, as a scalar
__device__ __forceinline__ float wave_max(float x) {
    x = row_max16(x);
    return fmaxf(fmaxf(lane_value(x, 0), lane_value(x, 16)), fmaxf(lane_value(x, 32), lane_value(x, 48)));
}

// 8 bytes per lane at (wave-uniform base) + (32-bit lane offset): the base stays in scalar registers
__device__ __forceinline__ float2 ld_dev2_at(const float* base, uint32_t lane_bytes) {
    return ld_dev2(reinterpret_cast<const float*>(reinterpret_cast<const uint8_t*>(base) + lane_bytes));
}

// 4 bytes per lane at (wave-uniform base) + (32-bit lane offset), device scope
__device__ __forceinline__ uint32_t ld_dev1_at(const uint32_t* base, uint32_t lane_bytes) {
    return __hip_atomic_load(reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(base) + lane_bytes),
                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// partial outputs (two channels per lane, 4 bytes) of splits s0 .. s0+N-1 of one query head.  The splits of a
// head lie 256 bytes apart, so the N loads differ only in the instruction's immediate offset and are issued back to
// back.  Past the head's last split the loads run on into the records behind it (the next head's, or the residual
// words that follow the partial outputs: the area behind the last head is longer than N records); the caller
// replaces what they return (settle_partials).
template <int N>
__device__ __forceinline__ void load_partials(uint32_t (&v)[N], const uint32_t* head_base, uint32_t lane_bytes, int s0) {
    const uint32_t* base = head_base + s0 * kPartialWords;
#pragma unroll
    for (int k = 0; k < N; ++k) v[k] = ld_dev1_at(base + k * kPartialWords, lane_bytes);
}
// words of splits that do not exist: a valid pair of ones (their weight is zero)
template <int N>
__device__ __forceinline__ void settle_partials(uint32_t (&v)[N], int cnt) {
    if (cnt < N) {
#pragma unroll
        for (int k = 0; k < N; ++k) v[k] = k < cnt ? v[k] : 0x3c003c00u;
    }
}

// Polls of a record that was not there yet, at most.  Every writer of a record the merging wave waits for has
// passed its workgroup's barrier and publishes without waiting for anybody, so the records arrive whatever else
// happens; the bound only keeps a misused workspace from hanging the launch.
constexpr int kMaxPolls = 1 << 16;

// Merge of the splits of one query head by one wave (flash_fwd_kernel.h:1217-1298 with normalised partials):
// out = sum_s w_s O_s / sum_s w_s with w_s = 2^(M_s - max M) L_s and O_s the split's normalised output.
// Lane l owns channels 2l and 2l+1.  Splits are taken N at a time (N = 32, or less when there are fewer splits):
// lane l holds the (M, L) pair of split s0 + l % 32, the weights go back to all lanes as scalars.  A record is
// valid when none of its words is zero; the loads of a block are repeated while one still reads "not written".
// A split that sent residual words (negative sum) has them added with the same weight.  The order of the
// additions is fixed: even and odd splits of a block are summed separately (two dependent chains instead of
// one) and added at the end, so the result does not depend on timing.  On return O0, O1 are the weighted sums
// and L the sum of the weights (the head's softmax denominator relative to M).  The partial-output area is
// below 2^31 bytes (checked by the host).
template <int N, int BLOCK>
__device__ __forceinline__ void merge_splits_n(uint32_t* o_part, uint32_t lo_words, float* ml_part, int64_t hrow,
                                               int nsplit, int lane, float& O0, float& O1, float& M, float& L, [[maybe_unused]] unsigned long long* pts = nullptr) {
    uint32_t* head_base = o_part + hrow * nsplit * kPartialWords;
    float* mlb = ml_part + hrow * nsplit * 2;
    const uint32_t lane_bytes = lane * 4;
    static_assert((BLOCK == 32 || BLOCK == 16) && N <= BLOCK, "splits per block");
    const int sl = lane & (BLOCK - 1);
    float lacc = 0.0f, Mu = 0.0f;
    float e0 = 0.0f, e1 = 0.0f, d0 = 0.0f, d1 = 0.0f;
    for (int s0 = 0; s0 < nsplit; s0 += BLOCK) {
        const bool mine = s0 + sl < nsplit;
        const uint32_t ml_lane = static_cast<uint32_t>(min(s0 + sl, nsplit - 1)) * 8;
        const float se0 = e0, se1 = e1, sd0 = d0, sd1 = d1;
        float2 ml;
        float w;
        // One flight of loads per attempt; the words are checked as they are used (none of them may be zero), and an
        // attempt that met a record still "not written" is thrown away and repeated.
        for (int spin = 0;; ++spin) {
            uint32_t v[N];
            // (the lane offset as a value of the attempt: the addresses of its loads are then formed here, from the
            // scalar base, and not kept in a pair of vector registers per load across the loop)
            uint32_t lb = lane_bytes, mlo = ml_lane;
            asm volatile("" : "+v"(lb), "+v"(mlo));
            PROF_AT(pts, 8);
            ml = ld_dev2_at(mlb, mlo);       // ahead of the bulk loads
            load_partials<N>(v, head_base, lb, s0);
            PROF_AT(pts, 9);
            uint32_t mn = __float_as_uint(ml.x) | __float_as_uint(ml.y);
            if (s0 == 0) {
                float mx = mine ? ml.x : -INFINITY;
                for (int s = BLOCK; s < nsplit; s += BLOCK) {        // more splits than a block holds: the other maxima
                    float2 t = float2{-INFINITY, 0.0f};
                    for (int spin2 = 0;; ++spin2) {
                        bool ok = true;
                        if (s + sl < nsplit) {
                            t = ld_dev2_at(mlb + 2 * s, sl * 8);
                            ok = (__float_as_uint(t.x) | __float_as_uint(t.y)) != 0;
                        }
                        if (__builtin_amdgcn_ballot_w64(!ok) == 0 || spin2 >= kMaxPolls) break;
                    }
                    mx = fmaxf(mx, t.x);
                }
                M = wave_max(mx);
                Mu = (M == -INFINITY) ? 0.0f : M;
            }
            w = mine ? __builtin_amdgcn_exp2f(ml.x - Mu) * __builtin_fabsf(ml.y) : 0.0f;
            settle_partials<N>(v, nsplit - s0);
#pragma unroll
            for (int k = 0; k < N; k += 2) {
                const float wa = lane_value(w, k), wb = lane_value(w, k + 1);
                mn = min(mn, min(v[k], v[k + 1]));
                e0 = __builtin_fmaf(wa, half_lo(v[k]), e0);
                e1 = __builtin_fmaf(wa, half_hi(v[k]), e1);
                d0 = __builtin_fmaf(wb, half_lo(v[k + 1]), d0);
                d1 = __builtin_fmaf(wb, half_hi(v[k + 1]), d1);
            }
            PROF_AT(pts, 10);
            if (__builtin_amdgcn_ballot_w64(mn == 0) == 0 || spin >= kMaxPolls) break;
            e0 = se0;
            e1 = se1;
            d0 = sd0;
            d1 = sd1;
        }
        lacc += w;
        // splits that sent residual words (rare: outputs of magnitude 2 or more), in ascending order; the words are set
        // back to "not written" here, by their only reader
        uint64_t sent = __builtin_amdgcn_ballot_w64(mine && lane < BLOCK && ml.y < 0.0f);
        while (sent) {
            const int s = __builtin_ctzll(sent);
            sent &= sent - 1;
            const float ws = lane_value(w, s);
            uint32_t* rec = head_base + lo_words + (s0 + s) * kPartialWords;
            uint32_t r = 0;
            for (int spin = 0;; ++spin) {
                r = ld_dev1_at(rec, lane_bytes);
                if (__builtin_amdgcn_ballot_w64(r == 0) == 0 || spin >= kMaxPolls) break;
            }
            e0 = __builtin_fmaf(ws, half_lo(r), e0);
            e1 = __builtin_fmaf(ws, half_hi(r), e1);
            st_dev1(rec + lane, 0u);
        }
    }
    O0 = e0 + d0;
    O1 = e1 + d1;
    // a block's terms lie in lanes 0 .. BLOCK-1 and again in the lanes behind them
    const float lrow = row_sum16(lacc);
    L = BLOCK == 32 ? lane_value(lrow, 0) + lane_value(lrow, 16) : lane_value(lrow, 0);
}
// MAXN: loads a lane may have in flight (32, or 16 in the kernels whose 16 waves leave a lane 128 registers: there
// more than 16 splits are merged in blocks of 16, one round trip per block)
template <int MAXN>
__device__ __forceinline__ void merge_splits(uint32_t* o_part, uint32_t lo_words, float* ml_part, int64_t hrow,
                                             int nsplit, int lane, float& O0, float& O1, float& M, float& L, [[maybe_unused]] unsigned long long* pts = nullptr) {
    // as many loads per lane as there are splits, rounded up to 4, 8, 16 or 32: every one of them is a round trip
    // of its own to the memory side (with 32 loads for 8 splits the 4K-token step took 0.5 us longer)
    if (nsplit <= 4) {
        merge_splits_n<4, 32>(o_part, lo_words, ml_part, hrow, nsplit, lane, O0, O1, M, L, pts);
    } else if (nsplit <= 8) {
        merge_splits_n<8, 32>(o_part, lo_words, ml_part, hrow, nsplit, lane, O0, O1, M, L, pts);
    } else if (nsplit <= 16) {
        merge_splits_n<16, 32>(o_part, lo_words, ml_part, hrow, nsplit, lane, O0, O1, M, L, pts);
    } else if constexpr (MAXN >= 32) {
        merge_splits_n<32, 32>(o_part, lo_words, ml_part, hrow, nsplit, lane, O0, O1, M, L, pts);
    } else {
        merge_splits_n<16, 16>(o_part, lo_words, ml_part, hrow, nsplit, lane, O0, O1, M, L, pts);
    }
}

template <bool BF16>
__device__ __forceinline__ uint16_t to_out(float f) {
    if constexpr (BF16) {
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
        u += 0x7fffu + ((u >> 16) & 1u);
        return static_cast<uint16_t>(u >> 16);
    } else {
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
    }
}

// Final values of one query head: lane l writes channels 2l, 2l+1 of O / L, lane 0 the natural-log LSE
// (softmax.h:303; +inf for a row without keys).  One reciprocal (within a unit in the last place of 1 / L) and two
// multiplications instead of two divisions: the wave that writes is the last thing running, and every
// instruction of it is on the critical path.
template <bool BF16>
__device__ __forceinline__ void write_head(uint16_t* out_row, float* lse, int lane, float O0, float O1, float M, float L,
                                           float pshift) {
    const bool none = !(L > 0.0f);
    const float inv = none ? 0.0f : __builtin_amdgcn_rcpf(L);
    const uint16_t a = to_out<BF16>(O0 * inv), b = to_out<BF16>(O1 * inv);
    if ((reinterpret_cast<uintptr_t>(out_row) & 3u) == 0) {
        reinterpret_cast<uint32_t*>(out_row)[lane] = a | (static_cast<uint32_t>(b) << 16);
    } else {
        out_row[2 * lane] = a;
        out_row[2 * lane + 1] = b;
    }
    if (lane == 0 && lse) *lse = none ? INFINITY : (M + __log2f(L) - pshift) * 0.69314718055994531f;
}

// ---------------------------------------------------------------------------------------------
// decode step with append: per-sequence length, the workgroup that stores and packs, the counter
// ---------------------------------------------------------------------------------------------
// The length is stable for every workgroup that reads it: it is advanced only after all workgroups of
// the sequence have drawn their tickets.
__device__ __forceinline__ int step_length(const FwdParams& P, int bi) { return P.lengths[bi]; }
// A sequence whose window is about to fill while its cache has no room for another chunk cannot
// take the token: it is attended, but neither stored nor counted.
__device__ __forceinline__ bool step_overflows(int capacity, int t) {
    const int r = t & (kChunk - 1);
    return t < 0 || (r == kChunk - 1 && t - r + kChunk > capacity);
}
// The workgroup that writes the output of a (batch, kv-head) is the last one of that pair to use the
// length and the window.  One of its threads draws a ticket as soon as that is settled; the holder of
// the last of the h_k tickets of a sequence knows that every workgroup of the sequence has read the
// length, advances it and resets the counter.  The tickets are relaxed device-scope atomics performed at the
// memory side (totally ordered); no data written in this launch is read through them, so no release or
// acquire is involved.  The new length and the reset counter are read again only by the next launch on the
// stream, and the end of a kernel makes plain stores visible to it: both may be plain stores, provided lengths
// and counters live in ordinary device memory (not host-coherent or fine-grained memory polled by another agent).
__device__ __forceinline__ void step_ticket(int* step_tickets, int* lengths, int n_heads_k, int capacity, int bi, int t) {
    const int drawn = __hip_atomic_fetch_add(&step_tickets[bi * kTicketStride], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (drawn == n_heads_k - 1) {
        // read again only by the next launch: plain stores
        step_tickets[bi * kTicketStride] = 0;
        if (!step_overflows(capacity, t)) lengths[bi] = t + 1;
    }
}

// Append of one (batch, kv-head) by the workgroup that finishes the pair, in two parts.  Both run after
// every other workgroup of the pair has finished, so nobody else reads the window any more.
//
// First part, as early as that is known, by the two last waves (the waves with the least to do in the
// merge, so that the round trips below overlap the other waves' work): 32 lanes of the last wave copy
// the new token into the window's next row, lane 0 of the wave before it sees to the length.
template <int NW>
__device__ __forceinline__ void step_begin(int bi, int hk, int t) {
    constexpr int first_wave = NW - 2;
    static_assert(NW >= 2, "two waves share the append");
    const int tid = threadIdx.x;
    const int capacity = LATE_I32(capacity);
    if (tid == first_wave * 64) {
        step_ticket(LATE_PTR(int*, step_tickets), LATE_PTR(int*, lengths), LATE_I32(hk), capacity, bi, t);
    }
    const int lt = tid - (first_wave + 1) * 64;
    if (lt < 0 || lt >= 32 || step_overflows(capacity, t)) return;
    const int r = t & (kChunk - 1);
    if (lt < 16) {
        const uint16_t* kn = LATE_PTR(const uint16_t*, k_new) + bi * LATE_I64(knew_sb) + hk * LATE_I64(knew_sh);
        uint16_t* kw = LATE_PTR(uint16_t*, k_res) + bi * LATE_I64(kres_sb) + hk * LATE_I64(kres_sh);
        *reinterpret_cast<u4*>(kw + r * LATE_I64(kres_st) + lt * 8) = ld_u4(kn + lt * 8);
    } else {
        const uint16_t* vn = LATE_PTR(const uint16_t*, v_new) + bi * LATE_I64(vnew_sb) + hk * LATE_I64(vnew_sh);
        uint16_t* vw = LATE_PTR(uint16_t*, v_res) + bi * LATE_I64(vres_sb) + hk * LATE_I64(vres_sh);
        *reinterpret_cast<u4*>(vw + r * LATE_I64(vres_st) + (lt - 16) * 8) = ld_u4(vn + (lt - 16) * 8);
    }
}
// Second part, by the whole workgroup once the output is written: a window that the token filled is
// quantize-packed (127 rows from the window, the last one from the new-token tensors) into the chunk
// behind the packed prefix.  `lds` is the workgroup's whole dynamic LDS.
template <int BITS, int GS, bool BF16, bool KT>
__device__ __forceinline__ void step_end(uint8_t* lds, int bi, int hk, int t) {
    const int tid = threadIdx.x;
    const int r = t & (kChunk - 1), packed = t - r;
    if (__builtin_expect(r == kChunk - 1, 0)) {      // uniform over the workgroup
        if (step_overflows(LATE_I32(capacity), t)) return;
        __syncthreads();        // the LDS still holds the merge weights some threads are reading
        const uint16_t* kn = LATE_PTR(const uint16_t*, k_new) + bi * LATE_I64(knew_sb) + hk * LATE_I64(knew_sh);
        const uint16_t* vn = LATE_PTR(const uint16_t*, v_new) + bi * LATE_I64(vnew_sb) + hk * LATE_I64(vnew_sh);
        const uint16_t* kw = LATE_PTR(const uint16_t*, k_res) + bi * LATE_I64(kres_sb) + hk * LATE_I64(kres_sh);
        const uint16_t* vw = LATE_PTR(const uint16_t*, v_res) + bi * LATE_I64(vres_sb) + hk * LATE_I64(vres_sh);
        const int64_t k_st = LATE_I64(kres_st), v_st = LATE_I64(vres_st);
        const ChunkPlace place = chunk_place(LATE_PTR(const int*, block_table), LATE_I64(bt_stride),
                                             LATE_I32(chunks_per_page), bi, hk, LATE_I32(hk), packed / kChunk);
        const qp::ChunkDst D = qp::chunk_dst<BITS, GS, KT>(
            LATE_PTR(uint8_t*, k_pack), LATE_PTR(uint8_t*, k_params), LATE_PTR(uint8_t*, v_pack),
            LATE_PTR(uint8_t*, v_params), LATE_I64(kpack_bh), LATE_I64(kparams_bh), LATE_I64(vpack_bh),
            LATE_I64(vparams_bh), place);
        qp::pack_chunk<BITS, GS, BF16, false, KT>(
            *reinterpret_cast<qp::PackLds<GS>*>(lds), tid, tid < qp::kPackThreads,
            [=](int n) { return n == kChunk - 1 ? kn : kw + n * k_st; },
            [=](int n) { return n == kChunk - 1 ? vn : vw + n * v_st; }, D);
    }
}

// With two workgroups per compute unit (the 8-wave kernels) and sequences of different lengths, the time of
// a launch is that of the unit whose two workgroups add up to the most.  The dispatcher fills the units
// round-robin, so the workgroups at batch positions p and p + b/2 share a unit: position p takes the p-th
// longest sequence and position ceil(b/2) + k the k-th shortest, which pairs the longest with the shortest.
// A permutation of the batch index computed by every wave from the device-side lengths (lane j holds sequence
// j; equal lengths are ordered by index), so every workgroup arrives at the same one; the lengths are not
// written during the launch.  Nothing else depends on it: results are indexed by the sequence.
__device__ __forceinline__ int sequence_of_position(const FwdParams& P, int p, int lane) {
    const int n = P.b;      // at most 64 (host)
    int len = -1;
    if (lane < n) len = min(max(P.seqlens[lane], 0), P.capacity);
    int rank = 0;           // sequences that come before this lane's in descending order of length
    for (int j = 0; j < n; ++j) {
        const int lj = __builtin_amdgcn_readlane(len, j);
        rank += (lj > len || (lj == len && j < lane)) ? 1 : 0;
    }
    const int half = (n + 1) >> 1;
    const int pos = rank < half ? rank : half + (n - 1 - rank);
    const unsigned long long hit = __ballot(lane < n && pos == p);
    // (pos is a permutation of 0 .. n-1, so exactly one lane answers; p itself if that were ever not so)
    return __builtin_amdgcn_readfirstlane(hit ? static_cast<int>(__builtin_ctzll(hit)) : p);
}

// ---------------------------------------------------------------------------------------------
// split-KV kernel: 1-D grid of num_splits * h_k * b workgroups of UnitCfg::NW waves.
// Split s of a (batch, kv-head) owns packed units [s*ups, (s+1)*ups) dealt round-robin to its
// waves; the 16-token tiles of the fp16 window are dealt round-robin over ALL waves of the head.
// With more than one split each head's wave writes its (O / sum in fp16, max, sum) and takes a ticket of the head;
// the wave that draws the last ticket merges all partials of the head
// (flash_fwd_kernel.h:1217-1298 formula) and resets the ticket.
//
// Dynamic LDS: [NW wave regions of UnitCfg::REGION bytes][q: 8 head rows + a zero row, 272 B apart]
// [sM, sL: per-wave max and sum, 8 heads x NW floats each][append flag][tickets and slots of the 8 heads].  A wave's region is reused as its
// V-transpose slab for fp16 tiles and as its slot of the cross-wave merge buffer (g x 128 floats <= 4 KB).
// ---------------------------------------------------------------------------------------------
template <int BITS, int GS, bool FEW>
constexpr int fwd_lds_bytes() {
    using C = UnitCfg<BITS, GS, FEW>;
    return C::NW * C::REGION + (kMaxGroupHeads + 1) * kQRowBytes + 2 * C::NW * kMaxGroupHeads * 4 + 16 + 2 * kMaxGroupHeads * 4;
}

template <int BITS, int GS, bool BF16, bool APPEND, bool KT, bool FEW>
// (second bound: waves per SIMD the register count has to leave room for.  Two workgroups of the 8-wave kernels share
// a compute unit when sequences differ in length, 4 waves per SIMD like the 16-wave kernels: 128 registers.  The
// per-token-K kernel of group size 32 needs more and runs one workgroup per unit.)
__global__ __launch_bounds__((UnitCfg<BITS, GS, FEW>::NW * 64), (FEW && !(KT && GS == 32) ? 4 : 1))
void fwd_splitkv_kernel(FwdParams P) {
    static_assert(!KT || BITS == 4, "per-token K parameters: 4 bits");
    // The decode step with append has more parameter fields than scalar registers, and the per-token-K kernels
    // have no vector register to spare for scalar spills: they fetch what only the window and the tail need from
    // the kernarg segment where it is used.
    constexpr bool kLateArgs = APPEND || KT;
    // Everything a workgroup needs before its first loads of the stream is asked for here, in the kernel's first
    // basic block (the fields are the head of the parameter block, kernels.h): left alone, the compiler fetches a
    // field behind the branch that first uses it, four or five rounds of scalar loads one after the other, half a
    // microsecond in which the memory system has nothing to do.  The rest is read where it is used.
    asm volatile("" : : "s"(P.nsplit), "s"(P.hk), "s"(P.g), "s"(P.b), "s"(P.nsplit_magic), "s"(P.hk_magic), "s"(P.seqlen),
                 "s"(P.reslen), "s"(P.capacity), "s"(P.res_cap), "s"(P.xcd_remap), "s"(P.seq_perm), "s"(P.seqlens),
                 "s"(P.reslens), "s"(P.q), "s"(P.q_sb), "s"(P.q_sh), "s"(P.k_pack), "s"(P.k_params), "s"(P.v_pack),
                 "s"(P.v_params), "s"(P.block_table), "s"(P.kpack_bh), "s"(P.kparams_bh), "s"(P.vpack_bh), "s"(P.vparams_bh),
                 "s"(P.bt_stride), "s"(P.chunks_per_page), "s"(P.neg_scale), "s"(P.scale_log2));
    if constexpr (kLateArgs && !KT) asm volatile("" : : "s"(P.tickets), "s"(P.h));      // (for the slot words below)
    if constexpr (!kLateArgs) {
        asm volatile("" : : "s"(P.k_res), "s"(P.v_res), "s"(P.kres_sb), "s"(P.kres_st), "s"(P.kres_sh), "s"(P.vres_sb),
                     "s"(P.vres_st), "s"(P.vres_sh), "s"(P.o_part), "s"(P.ml_part), "s"(P.tickets), "s"(P.out), "s"(P.out_sb),
                     "s"(P.out_sh), "s"(P.lse), "s"(P.h));
    }
    using C = UnitCfg<BITS, GS, FEW>;
    constexpr int NCG = C::NCG, NW = C::NW, REGION = C::REGION;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    static_assert(sizeof(qp::PackLds<GS>) <= NW * REGION, "the pack tile reuses the wave regions");
    uint8_t* const sq = lds + NW * REGION;                                   // [8 + zero row][128] 16-bit q
    float* const sM = reinterpret_cast<float*>(sq + (kMaxGroupHeads + 1) * kQRowBytes);   // [8][NW]
    float* const sL = sM + NW * kMaxGroupHeads;
    int* const s_last = reinterpret_cast<int*>(sL + NW * kMaxGroupHeads);
    int* const s_tick = s_last + 4;       // [8] tickets drawn for the heads of the group, -1 = not yet
    int* const s_cnt = s_tick + kMaxGroupHeads;      // [8] slot of this launch for each head of the group
    if (threadIdx.x < kMaxGroupHeads) s_tick[threadIdx.x] = -1;      // (read after the workgroup barrier of the tail)

    PROF_DECL;
    PROF(0);
    // Workgroups are handed to the 8 XCDs round-robin by linear id.  When the number of
    // (batch, kv-head) pairs is a multiple of 8, ids are remapped so that all splits of one pair run
    // on one XCD.
#ifdef BITDECODE_PROF
    asm volatile("" : : "s"(P.xcd_remap));
    PROF(11);
#endif
    int split, hk, bi;
    {
        const int lin = blockIdx.x;
        int bhid;
        if (P.xcd_remap) {
            const int xcd = lin & 7, r = lin >> 3;
            const int q = div_magic(r, P.nsplit_magic);
            bhid = q * 8 + xcd;
            split = r - q * P.nsplit;
        } else {
            bhid = div_magic(lin, P.nsplit_magic);
            split = lin - bhid * P.nsplit;
        }
        bi = div_magic(bhid, P.hk_magic);
        hk = bhid - bi * P.hk;
    }
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: unit addresses stay in SGPRs
    if constexpr (!APPEND) {
        if (P.seq_perm) bi = sequence_of_position(P, bi, lane);
    }
    const int col = lane & 15, kg = lane >> 4;
    const int head = col & 7;          // query head inside the GQA group
    const bool lo_part = col >= 8;     // columns 8-15 carry the lo halves of the split products
    const int g = P.g;
    const int64_t bh = static_cast<int64_t>(bi) * P.hk + hk;

    int S, R, r_new = -1, step_len = 0;
    if constexpr (APPEND) {
        step_len = step_length(P, bi);
        r_new = step_len & (kChunk - 1);
        S = min(step_len - r_new, P.capacity);     // a length beyond the capacity is the caller's error: stay inside
        R = r_new + 1;
    } else {
        // per-sequence values are device data the host never saw: keep them inside the cache and the window
        S = P.seqlens ? min(max(P.seqlens[bi], 0), P.capacity) : P.seqlen;
        R = P.reslens ? min(max(P.reslens[bi], 0), P.res_cap) : P.reslen;
    }
    const int nU = (S / kChunk) * C::UPC;
    const int ups = div_magic(nU + P.nsplit - 1, P.nsplit_magic);
    const int u0 = min(nU, split * ups);
    const int u1 = min(nU, u0 + ups);
    const int nT = (R + 15) / 16;
    PROF(12);

    uint8_t* const region = lds + wave * REGION;
    const uint32_t region_lds = lds_addr(region);

    // ---- every wave fetches q itself (two 16-byte loads per lane cover the eight head slots),
    // sends out the loads of its first unit, and then writes q, converted to fp16, to the
    // workgroup's LDS copy.  All waves write identical bytes, so no barrier is needed: q is the
    // oldest entry of each wave's own load queue.
    int u = u0 + wave;
    u4 qa_raw, qb_raw, qa, qb;
    {
        const int hq = lane >> 4;                         // head within a row of four
        const uint16_t* q0 = P.q + bi * P.q_sb + (hk * g) * P.q_sh + (lane & 15) * 8;
        qa_raw = load_untracked(q0 + (hq < g ? hq : 0) * P.q_sh);
        qb_raw = load_untracked(q0 + (hq + 4 < g ? hq + 4 : 0) * P.q_sh);
    }
    PROF(13);
    UnitAddr<BITS, GS> A;
    if (u < u1) {
        A = unit_addr<BITS, GS, KT>(P, bi, hk, u);
        PROF(14);
        issue_first_rows<BITS, GS, KT, FEW>(A, lane * 16, region_lds);
        PROF(15);
        wait_then_take<C::DEPTH - 1>(qa, qb, qa_raw, qb_raw);
    } else {
        wait_then_take<0>(qa, qb, qa_raw, qb_raw);
    }
    if (P.nsplit > 1 && wave == 0) {
        // Which slot of the split workspace this launch uses: a word per head next to its counter, flipped by the
        // wave that merges the head's splits when the launch is over for that head.  Lane j fetches head j's word
        // straight into LDS (device scope), behind the wave's first rows in its load queue (the waits of the row
        // pipeline count it as a row until it has landed, which holds the first rows back by one at most), so that
        // nobody ever waits for it: the tail reads it from LDS after the workgroup's barrier.
        const int* tk;
        if constexpr (KT) {
            const kblock ob = karg_block<BLOCK_AT(o_part)>();       // o_part ... bits
            tk = BLOCK_PTR(const int*, ob, o_part, tickets) +
                 (static_cast<int64_t>(bi) * BLOCK_I32(ob, o_part, h) + hk * g) * kTicketStride + kSlotWord;
        } else {
            tk = P.tickets + (static_cast<int64_t>(bi) * P.h + hk * g) * kTicketStride + kSlotWord;
        }
        const uint64_t heads = (1ull << g) - 1;
        uint64_t saved;
        asm volatile("s_mov_b32 m0, %3\n\t"
                     "s_mov_b64 %0, exec\n\t"
                     "s_and_b64 exec, exec, %4\n\t"
                     "global_load_lds_dword %1, %2 sc1\n\t"
                     "s_mov_b64 exec, %0"
                     : "=&s"(saved)
                     : "v"(lane * (kTicketStride * 4)), "s"(tk), "s"(__builtin_amdgcn_readfirstlane(lds_addr(s_cnt))), "s"(heads)
                     : "memory", "m0", "scc");
    }
    if (P.neg_scale) {      // softmax_scale < 0: scale_log2 holds |scale|, the sign goes into q
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            qa[i] ^= 0x80008000u;
            qb[i] ^= 0x80008000u;
        }
    }
    {
        uint8_t* dst = sq + (lane >> 4) * kQRowBytes + (lane & 15) * 16;
        *reinterpret_cast<h8*>(dst) = cvt_h8<BF16>(qa);
        *reinterpret_cast<h8*>(dst + 4 * kQRowBytes) = cvt_h8<BF16>(qb);
        if (lane < 16) *reinterpret_cast<u4*>(sq + 8 * kQRowBytes + lane * 16) = u4{0, 0, 0, 0};
    }
    // (head slots past the group hold head 0 again: finite values whose results are never stored)
    const QRows Q = q_rows(sq, head, kg, lo_part);
    PROF(1);

    WaveState<NCG> st;
    st.m = -INFINITY;
    st.l = f4{0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < NCG; ++c) st.ob[c] = f4{0, 0, 0, 0};
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) st.o[ct] = f4{0, 0, 0, 0};

    // ---- packed units of this wave
    if (u < u1) {
        const Magic mg;
#ifdef BITDECODE_PROF
        wait_vm<C::DEPTH - 2>();   // first row (K parameters) has arrived
        PROF(2);
#endif
        TokenQ<NCG> KQ;
        const TokenQ<NCG>* KQp = nullptr;
        if constexpr (KT) {
            KQ = token_q<BITS, NCG>(Q);
            KQp = &KQ;
        }
        int kslot = 0;
        for (int un = u + NW; un < u1; un += NW) {        // units that have a successor: it is fetched from inside
            const UnitAddr<BITS, GS> An = unit_addr<BITS, GS, KT>(P, bi, hk, un);
            compute_unit<BITS, GS, BF16, true, KT, FEW>(region, region_lds, kslot, A, An, Q, P, lane, lo_part, mg, st, KQp);
            A = An;
            kslot ^= 1;
        }
        compute_unit<BITS, GS, BF16, false, KT, FEW>(region, region_lds, kslot, A, A, Q, P, lane, lo_part, mg, st, KQp);
    }
    PROF(3);
    // ---- fp16 window tiles of this wave (the region becomes the V-transpose slab)
    {
        uint16_t* slab = reinterpret_cast<uint16_t*>(region);
        const int stride = NW * P.nsplit;
        int t = wave * P.nsplit + split;   // consecutive tiles go to different workgroups
        // (the lane index as a value of its own: what the tiles derive from it is then computed here, not carried
        // through the unit loop from the prologue, where the q loads derive the same; the loop has no register to spare)
        int lane_w = lane;
        asm volatile("" : "+v"(lane_w));
        if (t < nT) {
            wait_vm<0>();                  // q rows (a wave without packed units has not waited yet)
            const WindowSrc W = window_src<APPEND, kLateArgs>(P, bi, hk);
            Fp16Tile T;
            load_fp16_tile<APPEND>(T, W, t * 16, R, lane_w, r_new);
            while (true) {
                const int tn = t + stride;
                const bool more = tn < nT;
                fp16_tile<BF16, NCG>(T, P, t * 16, R, lane_w, Q, lo_part, st, slab, p_shift(BITS));
                if (!more) break;
                load_fp16_tile<APPEND>(T, W, tn * 16, R, lane_w, r_new);
                t = tn;
            }
        }
    }

    // (kLateArgs: what only the tail needs is fetched here, as for the window)
    uint16_t* out = P.out;
    int64_t out_sb = P.out_sb, out_sh = P.out_sh;
    float* lse_out = P.lse;
    uint32_t* o_part = P.o_part;
    float* ml_part = P.ml_part;
    int* tickets = P.tickets;
    int n_h = P.h;
    if constexpr (kLateArgs) {
        const kblock ob = karg_block<BLOCK_AT(o_part)>();       // o_part ... bits
        out = BLOCK_PTR(uint16_t*, ob, o_part, out);
        out_sb = BLOCK_I64(ob, o_part, out_sb);
        out_sh = BLOCK_I64(ob, o_part, out_sh);
        lse_out = BLOCK_PTR(float*, ob, o_part, lse);
        o_part = BLOCK_PTR(uint32_t*, ob, o_part, o_part);
        ml_part = BLOCK_PTR(float*, ob, o_part, ml_part);
        tickets = BLOCK_PTR(int*, ob, o_part, tickets);
        n_h = BLOCK_I32(ob, o_part, h);
    }
    // layout of the split workspace (kernels.h: split_slot_words): residual words behind the partial outputs of a
    // slot, the second slot behind the first
    const uint32_t lo_words = static_cast<uint32_t>(P.nsplit) * P.b * n_h * kPartialWords;
    const uint32_t slot_words = (lo_words / kPartialWords * (2 * kPartialWords + 2) + 63) / 64 * 64;
    // ---- merge the waves of this workgroup through LDS (each wave's slot is its own region)
    const float lsum = st.l[0] + partner(st.l[0]);      // rows are equal; lo columns hold 0
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = st.o[ct][r] + st.ob[ct / (GS / 16)][r];
            st.o[ct][r] = v + partner(v);      // hi + lo
        }
    }
    if (col < g) {
        float* sO = reinterpret_cast<float*>(region);
#pragma unroll
        for (int ct = 0; ct < 8; ++ct) {
            *reinterpret_cast<f4*>(&sO[col * kHeadDim + 16 * ct + 4 * kg]) = st.o[ct];
        }
    }
    if (kg == 0 && col < kMaxGroupHeads) {
        sM[col * NW + wave] = col < g ? st.m * P.scale_log2 : -INFINITY;     // base-2 units
        sL[col * NW + wave] = col < g ? lsum : 0.0f;
    }
    __syncthreads();
    PROF(4);
    if constexpr (APPEND) {
        if (P.nsplit == 1) step_begin<NW>(bi, hk, step_len);     // a single split: every wave is past the window
    }
    // From here on wave hh < g works alone on query head hh of the group, lane l on channels 2l and 2l+1;
    // nothing below needs another workgroup barrier (the decode step with append has one, to elect the
    // workgroup that appends).
    //
    // Protocol between the splits of one query head.  Workspace (ordinary device memory, all zero before its
    // first launch, used by one launch at a time and with one shape): a counter per head, and two slots of
    // records per (head, split): partial output (fp16 pairs), residual words, (max, sum).  A record is "not
    // written" while it holds a zero word; writers never store one.
    //  * Launches alternate between the two slots: a word next to each head's counter says which one is next; it is
    //    fetched into LDS while the workgroup streams, and flipped by the wave that ends the launch for the head.
    //  * After the workgroup's barrier an idle wave draws the head's ticket (device-scope atomic add, performed at
    //    the memory side, so tickets are totally ordered) while the head's own wave merges the workgroup's waves,
    //    writes its records into the launch's slot with device-scope write-through stores, and sets its records of
    //    the other slot back to "not written" for the next launch.  Nothing waits for the stores.
    //  * The wave whose head drew the last ticket of the launch knows that every other split of the head is past
    //    its barrier, so its records are written or about to be, by waves that wait for nobody.  It sets the
    //    counter back to zero, loads all records of the slot with device-scope loads and repeats the loads of a
    //    block while a record still reads "not written" (seldom: the ticket's round trip is longer than the way of
    //    the stores).
    // A record of the slot in use cannot be a leftover: its writer set it back two launches ago, after the launch
    // that read it had ended.  What would break it: a workspace in host-coherent or fine-grained memory with other
    // scope rules, two launches in flight on one workspace, another shape on a workspace that was not zeroed
    // again, or a workspace that was not zero at its first launch.
    bool last = false;
    float O0 = 0.0f, O1 = 0.0f, M = -INFINITY, L = 0.0f;
    // loads in flight of the wave that merges the splits (merge_splits): 16 where the kernel is at its register limit
    constexpr int kMergeLoads = (NW >= 16 || (KT && NW >= 12)) ? 16 : 32;
    const bool split_run = P.nsplit > 1;
    // With at least twice as many waves as heads in the group, wave g + j draws the ticket of head j as soon as the
    // workgroup is past its barrier, while wave j merges the workgroup's waves and publishes: the ticket's round
    // trip is over by the time wave j needs it.  The ticket travels through LDS (s_tick).
    const bool helpers = NW >= 2 * g;
    if (split_run && helpers && wave >= g && wave < 2 * g && lane == 0) {
        const int64_t hr = static_cast<int64_t>(bi) * n_h + hk * g + (wave - g);
        const int d = __hip_atomic_fetch_add(&tickets[hr * kTicketStride], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&s_tick[wave - g], d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    const int hq = hk * g + wave;                                  // this wave's query head
    const int64_t hrow = static_cast<int64_t>(bi) * n_h + hq;      // its row in [b][h] tables
    uint16_t* const out_row = out + bi * out_sb + hq * out_sh;
    if (wave < g) {
        // weights of the waves: lane (any row, w) takes wave w; the row reductions give every lane the
        // head's maximum, the weights travel to all lanes as scalars
        const int w16 = lane & 15;
        const float mw = w16 < NW ? sM[wave * NW + w16] : -INFINITY;
        const float lw = w16 < NW ? sL[wave * NW + w16] : 0.0f;
        M = row_max16(mw);
        const float Mu = (M == -INFINITY) ? 0.0f : M;
        const float aw = __builtin_amdgcn_exp2f(mw - Mu);
        L = lane_value(row_sum16(aw * lw), 0);
        const float* mine = reinterpret_cast<const float*>(lds) + wave * kHeadDim + 2 * lane;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float a = lane_value(aw, w);
            const float2 v = *reinterpret_cast<const float2*>(mine + w * (REGION / 4));
            O0 = __builtin_fmaf(a, v.x, O0);
            O1 = __builtin_fmaf(a, v.y, O1);
        }
        if (!split_run) {
            write_head<BF16>(out_row, lse_out ? lse_out + hrow : nullptr, lane, O0, O1, M, L, p_shift(BITS));
        } else {
            const int par = __builtin_amdgcn_readfirstlane(s_cnt[wave]) & 1;
            const uint32_t mine_words = par ? slot_words : 0u, other_words = par ? 0u : slot_words;
            const int64_t rec = hrow * P.nsplit + split;
            uint32_t* const rec_o = o_part + rec * kPartialWords + lane;
            float* const rec_ml = ml_part + rec * 2;
            const PartialWords W(O0, O1, L);
            const bool sends_lo = W.large(kPartialLoFrom);      // uniform
            if (sends_lo) st_dev1(rec_o + mine_words + lo_words, W.lo());
            st_dev1(rec_o + mine_words, W.hi());
            // (max, sum) is never two zero words: a zero maximum travels as -0; a negative sum says "residual words sent"
            if (lane == 0) st_dev2(rec_ml + mine_words, M == 0.0f ? -0.0f : M, sends_lo ? -L : L);
            PROF(5);
            int drawn = 0;
            if (!helpers && lane == 0) {
                drawn = __hip_atomic_fetch_add(&tickets[hrow * kTicketStride], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // this split's records of the other slot: "not written" again for the next launch
            st_dev1(rec_o + other_words, 0u);
            if (lane == 0) st_dev2(rec_ml + other_words, 0.0f, 0.0f);
            if (helpers) {
                do {
                    drawn = __hip_atomic_load(&s_tick[wave], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                } while (drawn < 0);
            }
            drawn = __builtin_amdgcn_readfirstlane(drawn);
            last = drawn == P.nsplit - 1;
            // the counter starts over and the next launch takes the other slot (both read again only by the next launch)
            if (last && lane == 0) {
                __hip_atomic_store(&tickets[hrow * kTicketStride], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&tickets[hrow * kTicketStride + kSlotWord], par ^ 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            PROF(6);
            o_part += mine_words;
            ml_part += mine_words;
            if constexpr (APPEND) {
                if (wave == 0) *s_last = last;
            } else if (last) {
                merge_splits<kMergeLoads>(o_part, lo_words, ml_part, hrow, P.nsplit, lane, O0, O1, M, L, PROF_TS);
                write_head<BF16>(out_row, lse_out ? lse_out + hrow : nullptr, lane, O0, O1, M, L, p_shift(BITS));
            }
        }
    }
    if constexpr (APPEND) {
        // The workgroup whose wave 0 holds the last ticket of the group's first head appends: every other
        // workgroup of the (batch, kv-head) is past its barrier, so none of them reads the window or the cache
        // any more.  Its last two waves store the token while the merging waves fetch the partials.
        bool appends = true;
        if (split_run) {
            __syncthreads();
            appends = *s_last != 0;
            if (appends) step_begin<NW>(bi, hk, step_len);
            if (wave < g && last) {
                merge_splits<kMergeLoads>(o_part, lo_words, ml_part, hrow, P.nsplit, lane, O0, O1, M, L, PROF_TS);
                write_head<BF16>(out_row, lse_out ? lse_out + hrow : nullptr, lane, O0, O1, M, L, p_shift(BITS));
            }
        }
        if (appends) step_end<BITS, GS, BF16, KT>(lds, bi, hk, step_len);
    }
    PROF(7);
    PROF_FLUSH();
}

template <int BITS, int GS, bool BF16, bool APPEND, bool KT, bool FEW>
hipError_t launch_fwd_ttt(const FwdParams& P, hipStream_t stream) {
    constexpr int kLds = fwd_lds_bytes<BITS, GS, FEW>();
    // the dynamic-LDS limit is raised once per kernel and device (idempotent, so a race between
    // two host threads only repeats the call)
    static std::atomic<bool> configured[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || !configured[dev].load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_splitkv_kernel<BITS, GS, BF16, APPEND, KT, FEW>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess) return e;
        if (dev >= 0 && dev < 64) configured[dev].store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((fwd_splitkv_kernel<BITS, GS, BF16, APPEND, KT, FEW>), dim3(P.nsplit * P.hk * P.b),
                       dim3(UnitCfg<BITS, GS, FEW>::NW * 64), kLds, stream, P);
    return hipGetLastError();
}

// The 4-bit kernels also exist with 8 waves per workgroup that keep six rows in flight each instead of 16 (12)
// waves with four (P.few_waves, decided on the host).  The prologue, which the waves of a SIMD issue in turn, and
// the merge of the waves shrink, and a wave's longer run of units hides more latency: 4-7 % faster from 4K to
// 128K tokens and from 1 to 16 sequences of equal length.  The 16 waves keep more bytes in flight per compute
// unit, which only pays when a few workgroups are left streaming alone (ragged batches).  A 2-bit unit admits
// only four rows in flight, and there the 8 waves lose 2-3 %: not built.
template <int BITS, int GS, bool BF16, bool APPEND, bool KT = false>
hipError_t launch_fwd_tt(const FwdParams& P, hipStream_t stream) {
    if constexpr (few_waves_variant(BITS, GS)) {
        if (P.few_waves) return launch_fwd_ttt<BITS, GS, BF16, APPEND, KT, true>(P, stream);
    }
    return launch_fwd_ttt<BITS, GS, BF16, APPEND, KT, false>(P, stream);
}

template <int BITS, int GS>
hipError_t launch_fwd_t(const FwdParams& P, hipStream_t stream) {
    if (P.ktensor) {      // "k-tensor" mode: 4 bits
        if constexpr (BITS == 4) {
            if (P.lengths) {
                return P.bf16 ? launch_fwd_tt<BITS, GS, true, true, true>(P, stream)
                              : launch_fwd_tt<BITS, GS, false, true, true>(P, stream);
            }
            return P.bf16 ? launch_fwd_tt<BITS, GS, true, false, true>(P, stream)
                          : launch_fwd_tt<BITS, GS, false, false, true>(P, stream);
        } else {
            return hipErrorInvalidValue;
        }
    }
    if (P.lengths) {
        return P.bf16 ? launch_fwd_tt<BITS, GS, true, true>(P, stream) : launch_fwd_tt<BITS, GS, false, true>(P, stream);
    }
    return P.bf16 ? launch_fwd_tt<BITS, GS, true, false>(P, stream) : launch_fwd_tt<BITS, GS, false, false>(P, stream);
}

}  // namespace

#ifdef BITDECODE_PROF
hipError_t set_prof_buffer(unsigned long long* p) {
    return hipMemcpyToSymbol(HIP_SYMBOL(g_prof), &p, sizeof(p));
}
#endif

hipError_t launch_fwd(const FwdParams& P, hipStream_t stream) {
    switch (P.bits * 1000 + P.gs) {
        case 4128: return launch_fwd_t<4, 128>(P, stream);
        case 4064: return launch_fwd_t<4, 64>(P, stream);
        case 4032: return launch_fwd_t<4, 32>(P, stream);
        case 2128: return launch_fwd_t<2, 128>(P, stream);
        case 2064: return launch_fwd_t<2, 64>(P, stream);
        case 2032: return launch_fwd_t<2, 32>(P, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace bitdecode
