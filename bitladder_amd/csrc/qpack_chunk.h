// Quantize-pack of one 128-token chunk of one (batch, kv-head) by 256 threads of a workgroup: the
// body shared by the stand-alone pack kernel and by the decode step that packs a full window.
// Arithmetic follows csrc/bit_decode/src/include/qpack.h:224-296 of the reference in IEEE fp32 (no
// contraction, correctly rounded divisions), so codes and parameters are bit-exact against the CPU
// restatement.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

namespace bitdecode {
namespace qp {

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

constexpr int kRowHalves = 136;  // 128 + 8 halves of padding: 272-byte rows, conflict-free b128 reads
constexpr int kPackThreads = 256;

template <bool BF16>
__device__ __forceinline__ float to_f32(uint16_t h) {
    if constexpr (BF16) {
        return __uint_as_float(static_cast<uint32_t>(h) << 16);
    } else {
        _Float16 x;
        __builtin_memcpy(&x, &h, 2);
        return static_cast<float>(x);
    }
}

template <bool BF16>
__device__ __forceinline__ uint16_t from_f32(float f) {
    if constexpr (BF16) {
        uint32_t u = __float_as_uint(f);
        if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
        u += 0x7fffu + ((u >> 16) & 1u);
        return static_cast<uint16_t>(u >> 16);
    } else {
        _Float16 x = static_cast<_Float16>(f);  // v_cvt_f16_f32: round to nearest even
        uint16_t h;
        __builtin_memcpy(&h, &x, 2);
        return h;
    }
}

// Parameter as stored in the cache.  Scale and zero are rounded to the element type (fp16, or bf16
// for bf16 inputs: that is the value the quantizer defines) and then written as fp16 bits in both
// cases, because the decode kernel's MFMA operands are fp16.  For bf16 this is exact whenever the
// value lies in the fp16 normal range, which is the domain the decode kernel supports anyway.
template <bool BF16>
__device__ __forceinline__ uint16_t param_bits(float v) {
    if constexpr (BF16) v = to_f32<true>(from_f32<true>(v));
    return from_f32<false>(v);
}

// qpack.h:243-251: scale_inv = range > 0 ? M / range : 0; stored scale = 1 / scale_inv (or 0)
// (Plain operators under the pragma, not the __f*_rn intrinsics: those are inline functions of the
// HIP headers whose operations carry the translation unit's default contraction mode, so the
// compiler may still fuse a multiply of one with an add of another.)
__device__ __forceinline__ void group_params(float mn, float mx, float M, float& sinv, float& scale) {
#pragma clang fp contract(off)
    const float range = mx - mn;
    sinv = (range > 0.0f) ? M / range : 0.0f;
    scale = (sinv == 0.0f) ? 0.0f : 1.0f / sinv;
}

// qpack.h:272-285: clamp(roundf((x - min) * scale_inv), 0, M); roundf = halves away from zero.
// t is never negative here (min is the minimum of the group x belongs to, scale_inv >= 0), and for
// t >= 0  roundf(t) == floor(t + 0.49999997f)  in fp32 round-to-nearest-even arithmetic: the constant
// is the float just below 0.5, so t = 0.49999997 stays at 0 while every t = k + 0.5 still reaches
// k + 1 (checked over every float in [0, 64]).  The upper clamp can never act: with d = fl(x - min)
// <= range = fl(max - min) and scale_inv = fl(M / range), t = fl(d * scale_inv) <= M * (1 + 2^-22),
// far below M + 0.5; an infinite range gives scale_inv = 0 and t = 0 or NaN, and v_cvt_u32_f32 maps
// NaN to 0.  The conversion truncates, which is the floor of a non-negative value.
__device__ __forceinline__ uint32_t quant_code(float x, float mn, float sinv) {
#pragma clang fp contract(off)
    const float d = x - mn;
    const float t = d * sinv;
    const float u = t + 0.49999997f;      // must stay a separate rounding: a fused multiply-add breaks ties differently
    return static_cast<uint32_t>(u);
}

// LDS of one chunk in flight
template <int GS>
struct PackLds {
    static constexpr int NG = kChunk / GS;       // K groups per chunk
    static constexpr int NCG = kHeadDim / GS;    // V channel groups per token
    __attribute__((aligned(16))) uint16_t tile[kChunk * kRowHalves];
    float k_qmin[4][kHeadDim], k_qmax[4][kHeadDim];      // per 32-token quarter
    float k_sinv[NG][kHeadDim], k_mn[NG][kHeadDim];
    float v_sinv[kChunk][NCG], v_mn[kChunk][NCG];
};

// where the chunk goes: its K codes, K parameters, V codes, V parameters
struct ChunkDst {
    uint8_t* kc;
    uint8_t* kp;
    uint8_t* vc;
    uint8_t* vp;
};
template <int BITS, int GS, bool KT = false>
__device__ __forceinline__ ChunkDst chunk_dst(uint8_t* k_pack, uint8_t* k_params, uint8_t* v_pack, uint8_t* v_params,
                                              int64_t kpack_bh, int64_t kparams_bh, int64_t vpack_bh,
                                              int64_t vparams_bh, const ChunkPlace& place) {
    const int64_t bh = place.region, ci = place.chunk;
    ChunkDst D;
    D.kc = k_pack + bh * kpack_bh + ci * chunk_code_bytes(BITS);
    // ("k-tensor": K parameters per token and channel group, as many bytes per chunk as V's)
    D.kp = k_params + bh * kparams_bh + ci * (KT ? v_param_chunk_bytes(GS) : (kChunk / GS) * kKParamGroupBytes);
    D.vc = v_pack + bh * vpack_bh + ci * chunk_code_bytes(BITS);
    D.vp = v_params + bh * vparams_bh + ci * v_param_chunk_bytes(GS);
    return D;
}

// Threads 0..255 of the workgroup (`active`) pack the chunk whose token n has its 128 K values at
// krow(n) and its 128 V values at vrow(n); every thread of the workgroup must make the call (the
// barriers inside are workgroup-wide).  The K tile is staged in LDS while the V tile's global loads are
// still in flight (PREFETCH_V; without it the V tile is fetched when the K side is done, which keeps
// 32 registers free), per-channel statistics are taken column-wise, per-token statistics row-wise,
// and each thread then assembles whole 16-byte lane slots of the packed layout so that the stores
// are full 1 KB wave rows.
// Minimum and maximum of every (token, channel group) of the tile in LDS: thread -> token tid/2, 64-channel
// half tid%2.  store(n, cg, mn, mx) is called once per group by the thread that holds its statistics.
template <int GS, bool BF16, class Store>
__device__ __forceinline__ void row_group_stats(const uint16_t* tile, int tid, Store store) {
    const int n = tid >> 1, hf = tid & 1;   // token, 64-channel half
    constexpr int PARTS = (GS >= 64) ? 1 : 2;        // groups fully inside this thread's half
    constexpr int PW = 64 / PARTS;                   // channels per part
    float pmn[PARTS], pmx[PARTS];
#pragma unroll
    for (int pt = 0; pt < PARTS; ++pt) {
        const uint16_t* row = &tile[n * kRowHalves + 64 * hf + PW * pt];
        float mn = to_f32<BF16>(row[0]), mx = mn;
#pragma unroll
        for (int c = 1; c < PW; ++c) {
            float x = to_f32<BF16>(row[c]);
            mn = fminf(mn, x);
            mx = fmaxf(mx, x);
        }
        pmn[pt] = mn;
        pmx[pt] = mx;
    }
    if constexpr (GS == 128) {
        pmn[0] = fminf(pmn[0], __shfl_xor(pmn[0], 1));
        pmx[0] = fmaxf(pmx[0], __shfl_xor(pmx[0], 1));
    }
#pragma unroll
    for (int pt = 0; pt < PARTS; ++pt) {
        const int cg = (GS == 128) ? 0 : (GS == 64 ? hf : 2 * hf + pt);
        if (GS == 128 && hf != 0) break;
        store(n, cg, pmn[pt], pmx[pt]);
    }
}

// 16-byte global load / store of the chunk routine.  STREAM marks data that is touched once (the bulk pack of
// a long prefix: fp16 rows in, packed rows out) with the non-temporal hint: 11-13 % faster there.  A pack of a
// single block per sequence keeps the default policy: its output is read by the very next decode step, and the
// small launch ends sooner when its stores may complete in the cache (6.5 against 7.4-8.0 us).
template <bool STREAM>
__device__ __forceinline__ u4 ld16(const void* p) {
    if constexpr (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    else return *reinterpret_cast<const u4*>(p);
}
template <bool STREAM>
__device__ __forceinline__ void st16(void* p, u4 v) {
    if constexpr (STREAM) __builtin_nontemporal_store(v, reinterpret_cast<u4*>(p));
    else *reinterpret_cast<u4*>(p) = v;
}

// With KT ("k-tensor" mode, qpack.h:378-470 of the reference) K is quantized like V, per token over groups
// of GS channels; its codes keep the K layout, its parameters go per chunk as
// [64-token half][channel group][16-token tile][token] (scale, zero) pairs.
template <int BITS, int GS, bool BF16, bool PREFETCH_V, bool KT = false, bool STREAM = false, class RowK, class RowV>
__device__ __forceinline__ void pack_chunk(PackLds<GS>& L, int tid, bool active, RowK krow, RowV vrow,
                                           const ChunkDst& D) {
#pragma clang fp contract(off)
    constexpr int NG = kChunk / GS, NCG = kHeadDim / GS;
    constexpr float M = static_cast<float>((1 << BITS) - 1);
    uint16_t* const tile = L.tile;

    // ---- global loads of both tiles: thread -> row tid/16 + 16*x, 16-byte column block tid%16
    const int lrow = (tid >> 4) & 15, lcol = (tid & 15) * 8;
    u4 kreg[8], vreg[8];
    if (active) {
#pragma unroll
        for (int x = 0; x < 8; ++x) kreg[x] = ld16<STREAM>(krow(lrow + 16 * x) + lcol);
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            if constexpr (PREFETCH_V) vreg[x] = ld16<STREAM>(vrow(lrow + 16 * x) + lcol);
        }
#pragma unroll
        for (int x = 0; x < 8; ++x) *reinterpret_cast<u4*>(&tile[(lrow + 16 * x) * kRowHalves + lcol]) = kreg[x];
    }
    __syncthreads();

    // ================= K: per-channel groups of GS tokens (KT: per-token groups of GS channels) =================
    if constexpr (KT) {
        if (active) {
            row_group_stats<GS, BF16>(tile, tid, [&](int n, int cg, float mn, float mx) {
                float sinv, scale;
                group_params(mn, mx, M, sinv, scale);
                L.v_sinv[n][cg] = sinv;
                L.v_mn[n][cg] = mn;
                uint16_t* dst = reinterpret_cast<uint16_t*>(
                    D.kp + ((((n >> 6) * NCG + cg) * 4 + ((n >> 4) & 3)) * 16 + (n & 15)) * 4);
                dst[0] = param_bits<BF16>(scale);
                dst[1] = param_bits<BF16>(mn);
            });
        }
        __syncthreads();
    }
    if (!KT && active) {
        const int c = tid & 127, part = tid >> 7;
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            const int quarter = 2 * part + qq;
            float mn = to_f32<BF16>(tile[(32 * quarter) * kRowHalves + c]);
            float mx = mn;
#pragma unroll 8
            for (int n = 1; n < 32; ++n) {
                float x = to_f32<BF16>(tile[(32 * quarter + n) * kRowHalves + c]);
                mn = fminf(mn, x);
                mx = fmaxf(mx, x);
            }
            L.k_qmin[quarter][c] = mn;
            L.k_qmax[quarter][c] = mx;
        }
    }
    if constexpr (!KT) __syncthreads();
    if (!KT && active) {
        for (int idx = tid; idx < NG * kHeadDim; idx += kPackThreads) {
            const int grp = idx >> 7, c = idx & 127;
            constexpr int QPG = GS / 32;  // quarters per group
            float mn = L.k_qmin[grp * QPG][c], mx = L.k_qmax[grp * QPG][c];
#pragma unroll
            for (int x = 1; x < QPG; ++x) {
                mn = fminf(mn, L.k_qmin[grp * QPG + x][c]);
                mx = fmaxf(mx, L.k_qmax[grp * QPG + x][c]);
            }
            float sinv, scale;
            group_params(mn, mx, M, sinv, scale);
            L.k_sinv[grp][c] = sinv;
            L.k_mn[grp][c] = mn;
            uint16_t* kp = reinterpret_cast<uint16_t*>(D.kp + grp * kKParamGroupBytes);
            kp[c] = param_bits<BF16>(scale);
            kp[kHeadDim + c] = param_bits<BF16>(mn);
        }
    }
    if constexpr (!KT) __syncthreads();
    if (active) {
        uint8_t* const kc = D.kc;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int rep = 0; rep < 2; ++rep) {
                const int slot = tid + kPackThreads * rep;
                const int t = slot >> 6, l = slot & 63, m = l & 15, kg = l >> 4;
                const int n = 16 * t + m, grp = n / GS;
                u4 out;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int ch0 = 32 * j + 8 * kg;
                    uint32_t w = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        float x = to_f32<BF16>(tile[n * kRowHalves + ch0 + i]);
                        uint32_t code = KT ? quant_code(x, L.v_mn[n][(ch0 + i) / GS], L.v_sinv[n][(ch0 + i) / GS])
                                           : quant_code(x, L.k_mn[grp][ch0 + i], L.k_sinv[grp][ch0 + i]);
                        const int p = i / 2 + 4 * (i % 2);
                        w |= code << (4 * p);
                    }
                    out[j] = w;
                }
                st16<STREAM>(kc + t * 1024 + l * 16, out);
            }
        } else {
            const int tp = tid >> 6, l = tid & 63, m = l & 15, kg = l >> 4;
            u4 out;
#pragma unroll
            for (int tin = 0; tin < 2; ++tin) {
                const int n = 16 * (2 * tp + tin) + m, grp = n / GS;
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    uint32_t w = 0;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int j = 2 * jj + e / 8, i = e % 8;
                        const int ch = 32 * j + 8 * kg + i;
                        float x = to_f32<BF16>(tile[n * kRowHalves + ch]);
                        uint32_t code = KT ? quant_code(x, L.v_mn[n][ch / GS], L.v_sinv[n][ch / GS])
                                           : quant_code(x, L.k_mn[grp][ch], L.k_sinv[grp][ch]);
                        const int f = e / 2 + 8 * (e % 2);
                        w |= code << (2 * f);
                    }
                    out[2 * tin + jj] = w;
                }
            }
            st16<STREAM>(kc + tp * 1024 + l * 16, out);
        }
    }
    __syncthreads();

    // ================= V: per-token groups of GS channels =================
    if (active) {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            if constexpr (!PREFETCH_V) vreg[x] = ld16<STREAM>(vrow(lrow + 16 * x) + lcol);
        }
#pragma unroll
        for (int x = 0; x < 8; ++x) *reinterpret_cast<u4*>(&tile[(lrow + 16 * x) * kRowHalves + lcol]) = vreg[x];
    }
    __syncthreads();
    if (active) {
        row_group_stats<GS, BF16>(tile, tid, [&](int n, int cg, float mn, float mx) {
            const int sb = n >> 5, T = (n >> 4) & 1, q = (n >> 2) & 3, r = n & 3, i = 4 * T + r;
            float sinv, scale;
            group_params(mn, mx, M, sinv, scale);
            L.v_sinv[n][cg] = sinv;
            L.v_mn[n][cg] = mn;
            uint16_t* dst = reinterpret_cast<uint16_t*>(D.vp + (sb * NCG + cg) * 128 + q * 16 + i * 2);
            dst[0] = param_bits<BF16>(scale);
            dst[32] = param_bits<BF16>(mn);   // zeros start 64 bytes after the scales
        });
    }
    __syncthreads();
    if (active) {
        uint8_t* const vc = D.vc;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int rep = 0; rep < 2; ++rep) {
                const int slot = tid + kPackThreads * rep;
                const int sb = slot >> 7, hf = (slot >> 6) & 1, l = slot & 63, c = l & 15, kg = l >> 4;
                u4 out;
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const int ch = 16 * (4 * hf + x) + c, cg = ch / GS;
                    uint32_t w = 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int tok = 32 * sb + 16 * (i / 4) + 4 * kg + (i % 4);
                        float xv = to_f32<BF16>(tile[tok * kRowHalves + ch]);
                        uint32_t code = quant_code(xv, L.v_mn[tok][cg], L.v_sinv[tok][cg]);
                        const int p = i / 2 + 4 * (i % 2);
                        w |= code << (4 * p);
                    }
                    out[x] = w;
                }
                st16<STREAM>(vc + sb * 2048 + hf * 1024 + l * 16, out);
            }
        } else {
            const int sb2 = tid >> 7, hf = (tid >> 6) & 1, l = tid & 63, c = l & 15, kg = l >> 4;
            u4 out;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int ch = 16 * (4 * hf + x) + c, cg = ch / GS;
                uint32_t w = 0;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int ks = e / 8, i = e % 8;
                    const int tok = 64 * sb2 + 32 * ks + 16 * (i / 4) + 4 * kg + (i % 4);
                    float xv = to_f32<BF16>(tile[tok * kRowHalves + ch]);
                    uint32_t code = quant_code(xv, L.v_mn[tok][cg], L.v_sinv[tok][cg]);
                    const int f = e / 2 + 8 * (e % 2);
                    w |= code << (2 * f);
                }
                out[x] = w;
            }
            st16<STREAM>(vc + sb2 * 2048 + hf * 1024 + l * 16, out);
        }
    }
}

}  // namespace qp
}  // namespace bitdecode
