// Physical layout of the packed KV cache for gfx950 (wave64, 16-byte lane loads, MFMA 16x16x32).
//
// The caller allocates the four tensors with the reference's shapes
//   k_pack   (b, S/pn, h_k, 128) u16      k_params (b, S/gs, h_k, 128) f32 (= 2 x fp16)
//   v_pack   (b, S,    h_k, 128/pn) u16   v_params (b, 128/gs, h_k, S) f32 (= 2 x fp16)
// (pn = 16/bits; reference: evaluation/test.py:76-83).  Only the byte budget of those shapes is
// kept; the arrangement of bytes inside is private to this library's pack and decode kernels
// and is described here.  S below is the capacity in tokens implied by the tensor shape.
//
// Every tensor is split into one contiguous region per (batch, kv-head), region index
// b * h_k + h, and every region into 128-token chunks, so a decode wave streams one chunk of
// one head as a run of fully coalesced 1 KB wave loads (64 lanes x 16 B).
//
// MFMA view used by the decode kernel (v_mfma_f32_16x16x32_f16, lane = col + 16*kg):
//   QK^T is computed transposed, S^T = K * Q^T: A operand = K codes, row = token,
//        8 k-values per lane = 8 channels;  B operand = Q, column = query head.
//   PV is computed transposed, O^T = V^T * P^T: A operand = V codes, row = channel,
//        8 k-values per lane = 8 tokens;  B operand = P^T straight out of the QK^T
//        accumulator registers (no LDS round trip), which fixes the token order below.
//
// K codes, 4-bit: chunk = 8 tiles of 16 tokens, tile = 1 KB = 64 lanes x 4 dwords.
//   lane l = m + 16*kg holds token 16*t + m; dword j, element i (0..7) is channel 32*j + 8*kg + i;
//   element i sits in nibble p = i/2 + 4*(i%2) (so that two masks and one shift unpack a dword
//   into four half2 registers).
// K codes, 2-bit: chunk = 4 tile pairs, pair = 1 KB = 64 lanes x 4 dwords; dword dd = 2*tin + jj
//   holds token 16*(2*tp + tin) + m, k-steps j = 2*jj and 2*jj+1: element e = 8*(j%2) + i sits in
//   field f = e/2 + 8*(e%2), channel 32*j + 8*kg + i.
// V codes, 4-bit: chunk = 4 sub-blocks of 32 tokens, sub-block = 2 halves x 1 KB; half hf,
//   lane l = c + 16*kg, dword x: channel 16*(4*hf + x) + c; element i is token
//   32*sb + 16*(i/4) + 4*kg + i%4, nibble p = i/2 + 4*(i%2).
// V codes, 2-bit: chunk = 2 sub-blocks of 64 tokens, same halves/lanes/dwords; element
//   e = 8*ks + i is token 64*sb2 + 32*ks + 16*(i/4) + 4*kg + i%4, field f = e/2 + 8*(e%2).
// Parameters (scale, zero) are stored as fp16 bit patterns for both element types; a bf16 cache
// stores fp16(bf16 value), which is the same number inside the fp16 normal range.
// K params: per group of gs tokens 512 B: scale[128] then zero[128], natural channel order.
// V params: per chunk 4 sub-blocks x ncg channel groups x 128 B: scale[q][i] (64 B) then
//   zero[q][i] (64 B), q = 0..3, i = 0..7, token 32*sb + 16*(i/4) + 4*q + i%4.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bitdecode {

constexpr int kHeadDim = 128;
constexpr int kChunk = 128;               // tokens per chunk (pack granularity)
constexpr int kMaxGroupHeads = 8;         // query heads per kv head handled by one MFMA tile

// bytes of K (or V) codes per chunk
constexpr int chunk_code_bytes(int bits) { return kChunk * kHeadDim * bits / 8; }
// bytes of K params per token group / of V params per chunk
constexpr int kKParamGroupBytes = 4 * kHeadDim;
constexpr int v_param_chunk_bytes(int gs) { return kChunk * (kHeadDim / gs) * 4; }

// per-(batch, kv-head) region sizes in bytes for a cache with capacity S tokens
constexpr int64_t code_region_bytes(int64_t S, int bits) { return S * kHeadDim * bits / 8; }
constexpr int64_t k_param_region_bytes(int64_t S, int gs) { return (S / gs) * kKParamGroupBytes; }
constexpr int64_t v_param_region_bytes(int64_t S, int gs) { return S * (kHeadDim / gs) * 4; }

// Region and chunk-in-region of chunk `ci` of sequence `bi`, kv-head `hk`.  Contiguous cache: region
// bi * h_k + hk holds all chunks of the sequence.  Paged cache: the block table names the page of every
// `chunks_per_page` chunks and regions are (page, kv-head).
struct ChunkPlace {
    int64_t region;
    int chunk;
};
__host__ __device__ inline ChunkPlace chunk_place(const int* block_table, int64_t bt_stride, int chunks_per_page,
                                                  int bi, int hk, int n_heads_k, int ci) {
    if (!block_table) return ChunkPlace{static_cast<int64_t>(bi) * n_heads_k + hk, ci};
    const int slot = ci / chunks_per_page;
    const int page = block_table[bi * bt_stride + slot];
    return ChunkPlace{static_cast<int64_t>(page) * n_heads_k + hk, ci - slot * chunks_per_page};
}

// ---- decode work units (shared by the kernel and the host-side split choice)
// A decode wave streams units of 4 KB of K codes + 4 KB of V codes + their parameters through its
// private LDS region: 64 tokens at 4 bits, 128 tokens at 2 bits.  The region holds the code rows, two
// slots of K parameters (the next unit's are fetched while the current ones are in use) and one slot of
// V parameters.
constexpr int unit_tokens(int bits) { return bits == 4 ? 64 : 128; }
constexpr int unit_k_param_bytes(int bits, int gs) {
    const int ut = unit_tokens(bits);
    return (ut > gs ? ut / gs : 1) * kKParamGroupBytes;
}
constexpr int unit_v_param_bytes(int bits, int gs) { return unit_tokens(bits) * (kHeadDim / gs) * 4; }
constexpr int unit_region_bytes(int bits, int gs) {
    return 8192 + 2 * unit_k_param_bytes(bits, gs) + unit_v_param_bytes(bits, gs);
}
// waves per decode workgroup: as many as 160 KB of LDS (less shared scratch) and the register file allow
constexpr int decode_waves(int bits, int gs) {
    return unit_region_bytes(bits, gs) <= 9728 ? 16 : (unit_region_bytes(bits, gs) <= 12288 ? 12 : 8);
}

// The decode kernels that also exist with 8 waves per workgroup (for launches with little work per
// workgroup), and the number of waves of a launch.
constexpr bool few_waves_variant(int bits, int gs) { return bits == 4 && decode_waves(bits, gs) > 8; }
constexpr int kFewWaves = 8;

}  // namespace bitdecode