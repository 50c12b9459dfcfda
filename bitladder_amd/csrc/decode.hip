// Split-KV decode attention over [packed low-bit prefix || fp16 residual window] + LSE combine.
//
// Replaces compute_attn_1rowblock_splitkv and combine_attn_seqk_parallel of the reference
// (csrc/bit_decode/src/flash_fwd_kernel.h:66-728, 1144-1327) with a wave64/MFMA design:
//
//  * A workgroup owns one (split, kv-head, batch); each of its waves streams whole work units of
//    that split: a packed 128-token chunk (~17 KB at 4 bits) or a 32-token fp16 block (16 KB).
//    All chunk data is fetched with 16-byte lane loads that form contiguous 1 KB wave rows.
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
//  * Online softmax in base 2 per head (softmax.h:250-310) in steps of 32 tokens (64 at 2 bits):
//    running max shared by the four lanes of a head through two lane-half swaps, accumulators
//    rescaled only when some head's max actually moved.
//  * The waves of a workgroup merge through LDS; splits merge in the same launch: the workgroup
//    that draws the last ticket of a (batch, kv-head) combines all partials.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"
#include "layout.h"

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
#define PROF_DECL unsigned long long prof_ts[8] = {0, 0, 0, 0, 0, 0, 0, 0}
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
            pb += ((((size_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * kNW +   \
                   (threadIdx.x >> 6)) * 8;                                                           \
            for (int i_ = 0; i_ < 8; ++i_) pb[i_] = prof_ts[i_];                                      \
        }                                                                                             \
    } while (0)
#else
#define PROF_DECL do { } while (0)
#define PROF(slot) do { } while (0)
#define PROF_FLUSH() do { } while (0)
#endif

constexpr int kNW = 8;            // waves per workgroup
constexpr float kPShift = 2.0f;   // probabilities are kept as 2^kPShift * exp2(s - max): a V scale
                                  // is at most 65504*2/3, so p*scale cannot overflow fp16
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

template <bool BF16>
__device__ __forceinline__ h8 ld_h8(const void* p) {
    return cvt_h8<BF16>(*reinterpret_cast<const u4*>(p));
}

__device__ __forceinline__ u4 ld_u4(const void* p) { return *reinterpret_cast<const u4*>(p); }

__device__ __forceinline__ float dot8(h8 a, h8 b, float c) {
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        h2 a2 = {a[2 * x], a[2 * x + 1]};
        h2 b2 = {b[2 * x], b[2 * x + 1]};
        c = __builtin_amdgcn_fdot2(a2, b2, c, false);
    }
    return c;
}

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
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x128, 0xf, 0xf, false));
}
// exact product a*b as hi + lo in fp16; returns the part this column carries
__device__ __forceinline__ h8 split_mul(h8 a, h8 b, bool lo_part) {
    const h8 hi = a * b;
    const h8 lo = __builtin_elementwise_fma(a, b, -hi);
    return lo_part ? lo : hi;
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
// p = 2^kPShift * exp2(scale * (t - running max)).  Accumulators are rescaled only when the
// running max of some head moved (wave-uniform branch).
template <int N, int NCG>
__device__ __forceinline__ void softmax_step(float (&t)[N], float scale, WaveState<NCG>& st) {
    float mx = t[0];
#pragma unroll
    for (int i = 1; i < N; ++i) mx = fmaxf(mx, t[i]);
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
    const float c0 = kPShift - m_use * scale;
#pragma unroll
    for (int i = 0; i < N; ++i) t[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(t[i], scale, c0));
}

// ---------------------------------------------------------------------------------------------
// packed 128-token chunks
// ---------------------------------------------------------------------------------------------
// Registers holding one chunk's global loads.  K side and V side are separate so that the next
// chunk's K loads can be issued as soon as this chunk's K registers are consumed (and likewise
// for V): with one chunk per wave every load of the kernel is in flight from the first cycle.
template <int BITS, int GS>
struct KSide {
    static constexpr int NG = kChunk / GS;
    static constexpr int NW4 = BITS == 4 ? 8 : 4;     // 16-byte lane loads of codes per chunk
    static constexpr int PF = NG <= 2 ? NG : 1;       // parameter groups fetched with the chunk
    u4 code[NW4];
    u4 ps[PF][4], pz[PF][4];
};
template <int BITS, int GS>
struct VSide {
    static constexpr int NCG = kHeadDim / GS;
    static constexpr int NW4 = BITS == 4 ? 8 : 4;
    static constexpr int PF = NCG == 1 ? 4 : 0;       // sub-blocks whose params are fetched with the chunk
    u4 code[NW4];
    u4 ps[PF ? PF : 1], pz[PF ? PF : 1];
};

template <int BITS, int GS>
__device__ __forceinline__ void load_kside(KSide<BITS, GS>& K, const FwdParams& P, int64_t bh, int ci, int lane) {
    constexpr int NG = kChunk / GS;
    const int kg = lane >> 4;
    const uint8_t* kc = P.k_pack + bh * P.kpack_bh + static_cast<int64_t>(ci) * chunk_code_bytes(BITS);
    const uint8_t* kp = P.k_params + bh * P.kparams_bh + static_cast<int64_t>(ci) * NG * kKParamGroupBytes;
    const uint32_t poff = kg * 16, coff = lane * 16;     // per-lane byte offsets from uniform bases
#pragma unroll
    for (int g = 0; g < KSide<BITS, GS>::PF; ++g) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            K.ps[g][j] = ld_u4(kp + (g * kKParamGroupBytes + 64 * j) + poff);
            K.pz[g][j] = ld_u4(kp + (g * kKParamGroupBytes + 256 + 64 * j) + poff);
        }
    }
#pragma unroll
    for (int x = 0; x < KSide<BITS, GS>::NW4; ++x) K.code[x] = ld_u4(kc + x * 1024 + coff);
}

template <int BITS, int GS>
__device__ __forceinline__ void load_vside(VSide<BITS, GS>& V, const FwdParams& P, int64_t bh, int ci, int lane) {
    const int kg = lane >> 4;
    const uint8_t* vc = P.v_pack + bh * P.vpack_bh + static_cast<int64_t>(ci) * chunk_code_bytes(BITS);
    const uint8_t* vp = P.v_params + bh * P.vparams_bh + static_cast<int64_t>(ci) * v_param_chunk_bytes(GS);
    const uint32_t poff = kg * 16, coff = lane * 16;
#pragma unroll
    for (int sb = 0; sb < VSide<BITS, GS>::PF; ++sb) {
        V.ps[sb] = ld_u4(vp + sb * 128 + poff);
        V.pz[sb] = ld_u4(vp + (sb * 128 + 64) + poff);
    }
#pragma unroll
    for (int x = 0; x < VSide<BITS, GS>::NW4; ++x) V.code[x] = ld_u4(vc + x * 1024 + coff);
}

// One packed chunk in steps of 32 tokens (4-bit) or 64 tokens (2-bit): S^T tiles of the step,
// online-softmax update, O^T += V^T P^T for the same tokens.  Scores stay in q.k units; the
// softmax scale is applied inside the exponent.
template <int BITS, int GS, bool BF16>
__device__ __forceinline__ void packed_chunk(const KSide<BITS, GS>& K, const VSide<BITS, GS>& V, const FwdParams& P,
                                             int64_t bh, int ci, int lane, const h8 (&qB)[4], bool lo_part,
                                             const Magic& mg, WaveState<kHeadDim / GS>& st) {
    constexpr int NG = kChunk / GS;
    constexpr int NCG = kHeadDim / GS;
    constexpr int TPG = GS / 16;                 // 16-token tiles per K group
    constexpr int CTPG = GS / 16;                // 16-channel tiles per V channel group
    constexpr int TPS = BITS == 4 ? 2 : 4;       // tiles per step
    constexpr int NSTEP = 8 / TPS;
    constexpr int KPF = KSide<BITS, GS>::PF;
    constexpr int VPF = VSide<BITS, GS>::PF;
    const int kg = lane >> 4;
    const h8 noff = -code_offsets<BITS>();
    const h8 ones = h8{1, 1, 1, 1, 1, 1, 1, 1};
    const h8 zero8 = h8{0, 0, 0, 0, 0, 0, 0, 0};
    const uint8_t* kp = P.k_params + bh * P.kparams_bh + static_cast<int64_t>(ci) * NG * kKParamGroupBytes;
    const uint8_t* vp = P.v_params + bh * P.vparams_bh + static_cast<int64_t>(ci) * v_param_chunk_bytes(GS);

    h8 qp[4];
    f4 kb = {0, 0, 0, 0};
#pragma unroll
    for (int step = 0; step < NSTEP; ++step) {
        float t[4 * TPS];
#pragma unroll
        for (int tt = 0; tt < TPS; ++tt) {
            const int tile = step * TPS + tt;
            if (tile % TPG == 0) {
                // new K group: fold its scale into Q (exact hi/lo split) and build the score bias
                // sum_c q_c*zero_c - sum_c (q_c*scale_c)*offset_c on the MFMA pipe
                const int grp = tile / TPG;
                kb = f4{0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    u4 rs, rz;
                    if (grp < KPF) {
                        rs = K.ps[grp < KPF ? grp : 0][j];
                        rz = K.pz[grp < KPF ? grp : 0][j];
                    } else {
                        rs = ld_u4(kp + (grp * kKParamGroupBytes + 64 * j) + kg * 16);
                        rz = ld_u4(kp + (grp * kKParamGroupBytes + 256 + 64 * j) + kg * 16);
                    }
                    qp[j] = split_mul(qB[j], cvt_h8<BF16>(rs), lo_part);
                    kb = mfma32(cvt_h8<BF16>(rz), lo_part ? zero8 : qB[j], kb);
                    kb = mfma32(noff, qp[j], kb);
                }
            }
            f4 acc = kb;
            if constexpr (BITS == 4) {
                const u4 w = K.code[tile];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc = mfma32(dq4(w[j], mg), qp[j], acc);
            } else {
                const u4 w = K.code[tile / 2];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    h8 a0, a1;
                    dq2(w[2 * (tile % 2) + jj], a0, a1, mg);
                    acc = mfma32(a0, qp[2 * jj], acc);
                    acc = mfma32(a1, qp[2 * jj + 1], acc);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) t[4 * tt + r] = acc[r] + partner(acc[r]);   // hi + lo
        }

        softmax_step<4 * TPS, NCG>(t, P.scale_log2, st);

        // ---- O^T += V^T P^T for the tokens of this step
        constexpr int NKS = TPS / 2;                  // 32-token k-steps in this step
        h8 p16[NKS], pz[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                // element i = 4*T + r  <->  tile 2*ks + T of the step, accumulator register r
                const h2 pr = pk_rtz(t[8 * ks + 2 * x], t[8 * ks + 2 * x + 1]);
                p16[ks][2 * x] = pr[0];
                p16[ks][2 * x + 1] = pr[1];
            }
            pz[ks] = lo_part ? zero8 : p16[ks];       // p itself only in the hi columns
            st.l = mfma32(ones, pz[ks], st.l);
        }
        const u4 w0 = V.code[2 * step], w1 = V.code[2 * step + 1];
#pragma unroll
        for (int cg = 0; cg < NCG; ++cg) {
            h8 pp[NKS];
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const int sb = step * NKS + ks;
                u4 rs, rz;
                if (VPF) {
                    rs = V.ps[VPF ? sb : 0];
                    rz = V.pz[VPF ? sb : 0];
                } else {
                    rs = ld_u4(vp + (sb * NCG + cg) * 128 + kg * 16);
                    rz = ld_u4(vp + ((sb * NCG + cg) * 128 + 64) + kg * 16);
                }
                pp[ks] = split_mul(p16[ks], cvt_h8<BF16>(rs), lo_part);
                st.ob[cg] = mfma32(cvt_h8<BF16>(rz), pz[ks], st.ob[cg]);
                st.ob[cg] = mfma32(noff, pp[ks], st.ob[cg]);
            }
#pragma unroll
            for (int x = 0; x < CTPG; ++x) {
                const int ct = cg * CTPG + x;
                const uint32_t w = ct < 4 ? w0[ct & 3] : w1[ct & 3];
                if constexpr (BITS == 4) {
                    st.o[ct] = mfma32(dq4(w, mg), pp[0], st.o[ct]);
                } else {
                    h8 a0, a1;
                    dq2(w, a0, a1, mg);
                    st.o[ct] = mfma32(a0, pp[0], st.o[ct]);
                    st.o[ct] = mfma32(a1, pp[NKS - 1], st.o[ct]);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// 16-token tiles of the fp16 residual window (tokens n0 .. n0+15, valid below R)
// ---------------------------------------------------------------------------------------------
struct Fp16Tile {
    u4 k[4];   // lane (token col, kg): channels 32*j + 8*kg .. +7
    u4 v[4];   // lane (kg, col): token 4*x + kg, channels 8*col .. +7
};

__device__ __forceinline__ void load_fp16_tile(Fp16Tile& T, const FwdParams& P, int bi, int hk, int n0, int R,
                                               int lane) {
    const int col = lane & 15, kg = lane >> 4;
    const uint16_t* kr = P.k_res + bi * P.kres_sb + hk * P.kres_sh;
    const uint16_t* vr = P.v_res + bi * P.vres_sb + hk * P.vres_sh;
    const int tok = n0 + col;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        T.k[j] = u4{0, 0, 0, 0};
        if (tok < R) T.k[j] = ld_u4(kr + static_cast<int64_t>(tok) * P.kres_st + 32 * j + 8 * kg);
    }
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        const int tv = n0 + 4 * x + kg;
        T.v[x] = u4{0, 0, 0, 0};
        if (tv < R) T.v[x] = ld_u4(vr + static_cast<int64_t>(tv) * P.vres_st + col * 8);
    }
}

template <bool BF16, int NCG>
__device__ __forceinline__ void fp16_tile(const Fp16Tile& T, const FwdParams& P, int n0, int R, int lane,
                                          const h8 (&qB)[4], bool lo_part, WaveState<NCG>& st, uint16_t* lds) {
    const int col = lane & 15, kg = lane >> 4;
    const h8 zero8 = h8{0, 0, 0, 0, 0, 0, 0, 0};

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
            acc = mfma32(cvt_h8<BF16>(T.k[j]), lo_part ? zero8 : qB[j], acc);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tk = n0 + 4 * kg + r;
            const float tot = acc[r] + partner(acc[r]);   // outside the select: every lane executes the DPP
            s[r] = tk < R ? tot : -INFINITY;
        }
    }
    softmax_step<4, NCG>(s, P.scale_log2, st);
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

// device-scope (agent) relaxed accesses: write-through stores / cache-coherent loads
__device__ __forceinline__ void st_dev(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_dev(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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

// ---------------------------------------------------------------------------------------------
// split-KV kernel: grid (num_splits, h_k, b), kNW waves.
// Split s of a (batch, kv-head) owns packed chunks [s*cps, (s+1)*cps) dealt round-robin to its
// waves; the 16-token tiles of the fp16 window are dealt round-robin over ALL waves of the head.
// With more than one split each workgroup writes a normalised partial and takes a ticket; the
// workgroup that draws the last ticket of its (batch, kv-head) merges all partials
// (flash_fwd_kernel.h:1217-1298 formula) and resets the ticket.
// ---------------------------------------------------------------------------------------------
template <int BITS, int GS, bool BF16>
__global__ __launch_bounds__(kNW * 64) void fwd_splitkv_kernel(FwdParams P) {
    constexpr int NCG = kHeadDim / GS;
    constexpr int kSlabHalves = 16 * kLdsRowHalves;
    constexpr int kMergeFloats = kNW * kMaxGroupHeads * kHeadDim;
    constexpr int kLdsBytes = (kMergeFloats * 4 > kNW * kSlabHalves * 2) ? kMergeFloats * 4 : kNW * kSlabHalves * 2;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[kLdsBytes];
    __shared__ float sM[kNW][kMaxGroupHeads], sL[kNW][kMaxGroupHeads];
    __shared__ int s_last;

    PROF_DECL;
    PROF(0);
    const int split = blockIdx.x, hk = blockIdx.y, bi = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: chunk addresses stay in SGPRs
    const int col = lane & 15, kg = lane >> 4;
    const int head = col & 7;          // query head inside the GQA group
    const bool lo_part = col >= 8;     // columns 8-15 carry the lo halves of the split products
    const int g = P.g;
    const int64_t bh = static_cast<int64_t>(bi) * P.hk + hk;

    const int S = P.seqlens ? P.seqlens[bi] : P.seqlen;
    const int R = P.reslens ? P.reslens[bi] : P.reslen;
    const int nP = S / kChunk;
    const int cps = (nP + P.nsplit - 1) / P.nsplit;
    const int c0 = min(nP, split * cps);
    const int c1 = min(nP, c0 + cps);
    const int nT = (R + 15) / 16;

    // Q is fetched unconditionally (padding columns re-read head 0 and are zeroed after the
    // chunk loads have been issued) so that no wait sits in front of the big loads.
    u4 qraw[4];
    {
        const uint16_t* qp = P.q + bi * P.q_sb + (hk * g + (head < g ? head : 0)) * P.q_sh + 8 * kg;
#pragma unroll
        for (int j = 0; j < 4; ++j) qraw[j] = ld_u4(qp + 32 * j);
    }
    auto q_operand = [&](h8 (&qB)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (head >= g) qraw[j] = u4{0, 0, 0, 0};
            qB[j] = cvt_h8<BF16>(qraw[j]);
            if (P.neg_scale) qB[j] = -qB[j];     // scale_log2 holds |scale|: running max needs scale >= 0
        }
    };

    WaveState<NCG> st;
    st.m = -INFINITY;
    st.l = f4{0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < NCG; ++c) st.ob[c] = f4{0, 0, 0, 0};
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) st.o[ct] = f4{0, 0, 0, 0};

    // ---- packed chunks of this wave, software-pipelined one side ahead
    h8 qB[4];
    {
        int ci = c0 + wave;
        if (ci >= c1) {
            q_operand(qB);
        } else {
            KSide<BITS, GS> K;
            VSide<BITS, GS> V;
            const Magic mg;
            PROF(1);
            load_kside<BITS, GS>(K, P, bh, ci, lane);
            load_vside<BITS, GS>(V, P, bh, ci, lane);
            // every load of the chunk is issued before any of it is used: keep the scheduler from
            // sinking the V loads below the QK^T work
            __builtin_amdgcn_sched_barrier(0);
            PROF(2);
            q_operand(qB);
            while (true) {
                packed_chunk<BITS, GS, BF16>(K, V, P, bh, ci, lane, qB, lo_part, mg, st);
                PROF(3);
                const int cn = ci + kNW;
                if (cn >= c1) break;
                load_kside<BITS, GS>(K, P, bh, cn, lane);
                load_vside<BITS, GS>(V, P, bh, cn, lane);
                __builtin_amdgcn_sched_barrier(0);
                ci = cn;
            }
        }
    }
    // ---- fp16 window tiles of this wave
    {
        uint16_t* slab = reinterpret_cast<uint16_t*>(lds_raw) + wave * kSlabHalves;
        const int stride = kNW * P.nsplit;
        int t = wave * P.nsplit + split;   // consecutive tiles go to different workgroups
        if (t < nT) {
            Fp16Tile T;
            load_fp16_tile(T, P, bi, hk, t * 16, R, lane);
            while (true) {
                const int tn = t + stride;
                Fp16Tile N;
                const bool more = tn < nT;
                if (more) load_fp16_tile(N, P, bi, hk, tn * 16, R, lane);
                fp16_tile<BF16, NCG>(T, P, t * 16, R, lane, qB, lo_part, st, slab);
                if (!more) break;
                T = N;
                t = tn;
            }
        }
    }

    PROF(4);
    // ---- merge the waves of this workgroup through LDS
    const float lsum = st.l[0] + partner(st.l[0]);      // rows are equal; lo columns hold 0
#pragma unroll
    for (int ct = 0; ct < 8; ++ct) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float v = st.o[ct][r] + st.ob[ct / (GS / 16)][r];
            st.o[ct][r] = v + partner(v);      // hi + lo
        }
    }
    __syncthreads();   // slabs are dead from here on
    float* sO = reinterpret_cast<float*>(lds_raw);
    if (col < g) {
#pragma unroll
        for (int ct = 0; ct < 8; ++ct) {
            *reinterpret_cast<f4*>(&sO[(wave * kMaxGroupHeads + col) * kHeadDim + 16 * ct + 4 * kg]) = st.o[ct];
        }
        if (kg == 0) {
            sM[wave][col] = st.m * P.scale_log2;     // base-2 units
            sL[wave][col] = lsum;
        }
    }
    __syncthreads();
    const int64_t hstride = static_cast<int64_t>(P.b) * P.h;       // rows per split in the workspace
    for (int idx = tid; idx < g * kHeadDim; idx += kNW * 64) {
        const int hh = idx >> 7, c = idx & 127;
        float M = sM[0][hh];
#pragma unroll
        for (int w = 1; w < kNW; ++w) M = fmaxf(M, sM[w][hh]);
        const float Mu = (M == -INFINITY) ? 0.0f : M;
        float L = 0.0f, O = 0.0f;
#pragma unroll
        for (int w = 0; w < kNW; ++w) {
            const float a = __builtin_amdgcn_exp2f(sM[w][hh] - Mu);
            L += a * sL[w][hh];
            O += a * sO[(w * kMaxGroupHeads + hh) * kHeadDim + c];
        }
        const bool empty = !(L > 0.0f);
        const float o = empty ? 0.0f : O / L;
        // natural-log LSE of this split (softmax.h:303); -inf marks an empty split
        const float lse = empty ? -INFINITY : (M + __log2f(L) - kPShift) * 0.69314718055994531f;
        const int hq = hk * g + hh;
        if (P.nsplit == 1) {
            P.out[bi * P.out_sb + hq * P.out_sh + c] = to_out<BF16>(o);
            if (c == 0 && P.lse) P.lse[bi * P.h + hq] = empty ? INFINITY : lse;
        } else {
            const int64_t row = split * hstride + bi * P.h + hq;
            st_dev(&P.o_part[row * kHeadDim + c], o);
            if (c == 0) st_dev(&P.lse_part[row], lse);
        }
    }
    PROF(5);
    if (P.nsplit == 1) {
        PROF_FLUSH();
        return;
    }

    // ---- the workgroup that draws the last ticket of this (batch, kv-head) merges the splits.
    // Partials are written with device-scope (write-through) stores; once a thread's stores have
    // completed (vmcnt 0) and the workgroup has met at the barrier, thread 0 takes the ticket.
    // The merging workgroup reads the partials with device-scope loads, so no cache-wide
    // write-back or invalidate is needed on either side.
    __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this thread's partial stores are complete
    __syncthreads();
    if (tid == 0) {
        const int old = __hip_atomic_fetch_add(&P.tickets[bh], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old == P.nsplit - 1);
        if (s_last) __hip_atomic_store(&P.tickets[bh], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    PROF(6);
    if (!s_last) {
        PROF_FLUSH();
        return;
    }
    // every thread owns one (head, channel) and fetches the partial outputs and LSEs of up to 32
    // splits in one batch, so that the whole merge costs one memory round trip
    for (int idx = tid; idx < g * kHeadDim; idx += kNW * 64) {
        const int hh = idx >> 7, c = idx & 127;
        const int hq = hk * g + hh;
        const int64_t row0 = bi * P.h + hq;
        float M = -INFINITY, sum = 0.0f, o = 0.0f;
        for (int s0 = 0; s0 < P.nsplit; s0 += 32) {
            float v[32], e[32];
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                const int sidx = min(s0 + k, P.nsplit - 1);
                v[k] = ld_dev(&P.o_part[(sidx * hstride + row0) * kHeadDim + c]);
                e[k] = ld_dev(&P.lse_part[sidx * hstride + row0]);
            }
            float mb = -INFINITY;
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                if (s0 + k >= P.nsplit) e[k] = -INFINITY;
                mb = fmaxf(mb, e[k]);
            }
            const float Mn = fmaxf(M, mb);
            const float Mu = (Mn == -INFINITY) ? 0.0f : Mn;
            const float a = __expf(M - Mu);
            sum *= a;
            o *= a;
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                const float w = __expf(e[k] - Mu);
                sum += w;
                o += w * v[k];
            }
            M = Mn;
        }
        const bool none = (sum == 0.0f || sum != sum);
        P.out[bi * P.out_sb + hq * P.out_sh + c] = to_out<BF16>(none ? 0.0f : o / sum);
        if (c == 0 && P.lse) P.lse[row0] = none ? INFINITY : __logf(sum) + M;
    }
    PROF(7);
    PROF_FLUSH();
}

template <int BITS, int GS>
hipError_t launch_fwd_t(const FwdParams& P, hipStream_t stream) {
    dim3 grid(P.nsplit, P.hk, P.b);
    if (P.bf16) {
        hipLaunchKernelGGL((fwd_splitkv_kernel<BITS, GS, true>), grid, dim3(kNW * 64), 0, stream, P);
    } else {
        hipLaunchKernelGGL((fwd_splitkv_kernel<BITS, GS, false>), grid, dim3(kNW * 64), 0, stream, P);
    }
    return hipGetLastError();
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
