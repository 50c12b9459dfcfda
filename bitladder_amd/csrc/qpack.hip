// Quantize-pack kernel: fp16/bf16 K,V -> 2/4-bit codes + scale/zero in the gfx950 layout of
// layout.h.  Arithmetic follows csrc/bit_decode/src/include/qpack.h:224-296 of the reference
// in IEEE fp32 (no contraction, correctly rounded divisions), so codes and parameters are
// bit-exact against the CPU restatement.
//
// One workgroup (256 threads) packs one 128-token chunk of one (batch, kv-head): the K tile is
// staged in LDS while the V tile's global loads are still in flight, per-channel statistics are
// taken column-wise, per-token statistics row-wise, and each thread then assembles whole
// 16-byte lane slots of the packed layout so that the stores are full 1 KB wave rows.
// HBM-bound: reads 64 KB, writes chunk_code_bytes*2 + params per chunk.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"
#include "layout.h"

namespace bitdecode {
namespace {

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

constexpr int kRowHalves = 136;  // 128 + 8 halves of padding: 272-byte rows, conflict-free b128 reads

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
__device__ __forceinline__ void group_params(float mn, float mx, float M, float& sinv, float& scale) {
    float range = __fsub_rn(mx, mn);
    sinv = (range > 0.0f) ? __fdiv_rn(M, range) : 0.0f;
    scale = (sinv == 0.0f) ? 0.0f : __fdiv_rn(1.0f, sinv);
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
    const float t = __fmul_rn(__fsub_rn(x, mn), sinv);
    return static_cast<uint32_t>(__fadd_rn(t, 0.49999997f));
}

template <int BITS, int GS, bool BF16>
__global__ __launch_bounds__(256) void qpack_kernel(QpackParams P) {
    constexpr int NG = kChunk / GS;       // K groups per chunk
    constexpr int NCG = kHeadDim / GS;    // V channel groups per token
    constexpr float M = static_cast<float>((1 << BITS) - 1);

    __shared__ __attribute__((aligned(16))) uint16_t tile[kChunk * kRowHalves];
    __shared__ float k_qmin[4][kHeadDim], k_qmax[4][kHeadDim];      // per 32-token quarter
    __shared__ float k_sinv[NG][kHeadDim], k_mn[NG][kHeadDim];
    __shared__ float v_sinv[kChunk][NCG], v_mn[kChunk][NCG];

    const int tid = threadIdx.x;
    const int ci_src = blockIdx.x, hk = blockIdx.y, bi = blockIdx.z;
    const int dst_base = P.dst_offsets ? P.dst_offsets[bi] : P.dst_offset;
    if (dst_base < 0) return;       // a negative per-sequence offset skips that sequence (whole workgroup)
    const int dst_tok = dst_base + ci_src * kChunk;
    const ChunkPlace place = chunk_place(P.block_table, P.bt_stride, P.chunks_per_page, bi, hk, P.hk, dst_tok / kChunk);
    const int ci = place.chunk;
    const int64_t bh = place.region;

    // ---- global loads of both tiles: thread -> row tid/16 + 16*x, 16-byte column block tid%16
    const int lrow = tid >> 4, lcol = (tid & 15) * 8;
    u4 kreg[8], vreg[8];
    {
        const uint16_t* ks = P.k + bi * P.k_sb + static_cast<int64_t>(ci_src) * kChunk * P.k_st + hk * P.k_sh + lcol;
        const uint16_t* vs = P.v + bi * P.v_sb + static_cast<int64_t>(ci_src) * kChunk * P.v_st + hk * P.v_sh + lcol;
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            kreg[x] = *reinterpret_cast<const u4*>(ks + static_cast<int64_t>(lrow + 16 * x) * P.k_st);
        }
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            vreg[x] = *reinterpret_cast<const u4*>(vs + static_cast<int64_t>(lrow + 16 * x) * P.v_st);
        }
    }
#pragma unroll
    for (int x = 0; x < 8; ++x) {
        *reinterpret_cast<u4*>(&tile[(lrow + 16 * x) * kRowHalves + lcol]) = kreg[x];
    }
    __syncthreads();

    // ================= K: per-channel groups of GS tokens =================
    {
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
            k_qmin[quarter][c] = mn;
            k_qmax[quarter][c] = mx;
        }
    }
    __syncthreads();
    for (int idx = tid; idx < NG * kHeadDim; idx += 256) {
        const int grp = idx >> 7, c = idx & 127;
        constexpr int QPG = GS / 32;  // quarters per group
        float mn = k_qmin[grp * QPG][c], mx = k_qmax[grp * QPG][c];
#pragma unroll
        for (int x = 1; x < QPG; ++x) {
            mn = fminf(mn, k_qmin[grp * QPG + x][c]);
            mx = fmaxf(mx, k_qmax[grp * QPG + x][c]);
        }
        float sinv, scale;
        group_params(mn, mx, M, sinv, scale);
        k_sinv[grp][c] = sinv;
        k_mn[grp][c] = mn;
        uint16_t* kp = reinterpret_cast<uint16_t*>(
            P.k_params + bh * P.kparams_bh + (static_cast<int64_t>(ci) * NG + grp) * kKParamGroupBytes);
        kp[c] = param_bits<BF16>(scale);
        kp[kHeadDim + c] = param_bits<BF16>(mn);
    }
    __syncthreads();
    {
        uint8_t* kc = P.k_pack + bh * P.kpack_bh + static_cast<int64_t>(ci) * chunk_code_bytes(BITS);
        if constexpr (BITS == 4) {
#pragma unroll
            for (int rep = 0; rep < 2; ++rep) {
                const int slot = tid + 256 * rep;
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
                        uint32_t code = quant_code(x, k_mn[grp][ch0 + i], k_sinv[grp][ch0 + i]);
                        const int p = i / 2 + 4 * (i % 2);
                        w |= code << (4 * p);
                    }
                    out[j] = w;
                }
                *reinterpret_cast<u4*>(kc + t * 1024 + l * 16) = out;
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
                        uint32_t code = quant_code(x, k_mn[grp][ch], k_sinv[grp][ch]);
                        const int f = e / 2 + 8 * (e % 2);
                        w |= code << (2 * f);
                    }
                    out[2 * tin + jj] = w;
                }
            }
            *reinterpret_cast<u4*>(kc + tp * 1024 + l * 16) = out;
        }
    }
    __syncthreads();

    // ================= V: per-token groups of GS channels =================
#pragma unroll
    for (int x = 0; x < 8; ++x) {
        *reinterpret_cast<u4*>(&tile[(lrow + 16 * x) * kRowHalves + lcol]) = vreg[x];
    }
    __syncthreads();
    {
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
        uint8_t* vp = P.v_params + bh * P.vparams_bh + static_cast<int64_t>(ci) * v_param_chunk_bytes(GS);
        const int sb = n >> 5, T = (n >> 4) & 1, q = (n >> 2) & 3, r = n & 3, i = 4 * T + r;
#pragma unroll
        for (int pt = 0; pt < PARTS; ++pt) {
            const int cg = (GS == 128) ? 0 : (GS == 64 ? hf : 2 * hf + pt);
            if (GS == 128 && hf != 0) break;
            float sinv, scale;
            group_params(pmn[pt], pmx[pt], M, sinv, scale);
            v_sinv[n][cg] = sinv;
            v_mn[n][cg] = pmn[pt];
            uint16_t* dst = reinterpret_cast<uint16_t*>(vp + (sb * NCG + cg) * 128 + q * 16 + i * 2);
            dst[0] = param_bits<BF16>(scale);
            dst[32] = param_bits<BF16>(pmn[pt]);   // zeros start 64 bytes after the scales
        }
    }
    __syncthreads();
    {
        uint8_t* vc = P.v_pack + bh * P.vpack_bh + static_cast<int64_t>(ci) * chunk_code_bytes(BITS);
        if constexpr (BITS == 4) {
#pragma unroll
            for (int rep = 0; rep < 2; ++rep) {
                const int slot = tid + 256 * rep;
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
                        uint32_t code = quant_code(xv, v_mn[tok][cg], v_sinv[tok][cg]);
                        const int p = i / 2 + 4 * (i % 2);
                        w |= code << (4 * p);
                    }
                    out[x] = w;
                }
                *reinterpret_cast<u4*>(vc + sb * 2048 + hf * 1024 + l * 16) = out;
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
                    uint32_t code = quant_code(xv, v_mn[tok][cg], v_sinv[tok][cg]);
                    const int f = e / 2 + 8 * (e % 2);
                    w |= code << (2 * f);
                }
                out[x] = w;
            }
            *reinterpret_cast<u4*>(vc + sb2 * 2048 + hf * 1024 + l * 16) = out;
        }
    }
}

template <int BITS, int GS>
hipError_t launch_qpack_t(const QpackParams& P, hipStream_t stream) {
    dim3 grid(P.n_tokens / kChunk, P.hk, P.b);
    if (P.bf16) {
        hipLaunchKernelGGL((qpack_kernel<BITS, GS, true>), grid, dim3(256), 0, stream, P);
    } else {
        hipLaunchKernelGGL((qpack_kernel<BITS, GS, false>), grid, dim3(256), 0, stream, P);
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_qpack(const QpackParams& P, hipStream_t stream) {
    if (P.n_tokens == 0 || P.b == 0) return hipSuccess;
    switch (P.bits * 1000 + P.gs) {
        case 4128: return launch_qpack_t<4, 128>(P, stream);
        case 4064: return launch_qpack_t<4, 64>(P, stream);
        case 4032: return launch_qpack_t<4, 32>(P, stream);
        case 2128: return launch_qpack_t<2, 128>(P, stream);
        case 2064: return launch_qpack_t<2, 64>(P, stream);
        case 2032: return launch_qpack_t<2, 32>(P, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace bitdecode
