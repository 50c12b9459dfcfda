// Internal launch interface between the C ABI (api.hip) and the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bitdecode {

// Arrival counters of different query heads are drawn from compute units all over the chip at about the
// same time: each sits in a 256-byte block of its own (counters that share a cache line cost several
// microseconds per launch on a multi-die GPU, measured).
constexpr int kTicketStride = 64;      // ints
constexpr int kSlotWord = 32;          // ints behind a head's counter, in the other 128-byte half of its block: which record slot the next launch uses
constexpr int kPartialWords = 64;      // 32-bit words of one split's partial output of one query head: 128 channels as fp16

struct QpackParams {
    const uint16_t* k;
    const uint16_t* v;
    int64_t k_sb, k_st, k_sh, v_sb, v_st, v_sh;      // element strides
    uint8_t* k_pack;
    uint8_t* k_params;
    uint8_t* v_pack;
    uint8_t* v_params;
    int64_t kpack_bh, kparams_bh, vpack_bh, vparams_bh;  // bytes per (batch, kv-head) region
    int b, n_tokens, hk;
    int dst_offset;
    const int* dst_offsets;
    int capacity;               // tokens a sequence can hold: a device-side offset beyond it skips the sequence
    int bits, gs, bf16;
    int ktensor;                // "k-tensor" mode: K quantized per token over channel groups, like V
    const int* block_table;     // paged cache: page of (sequence, page slot); regions are then (page, kv-head)
    int64_t bt_stride;
    int chunks_per_page;
};

// The decode kernel fetches its arguments in 64-byte blocks with scalar loads of its own (decode.hip): the first
// three blocks, everything a workgroup needs up to its first loads of the stream, in one round at its entry;
// k_res ... vres_sh and o_part ... bits where they are used.  Keep each group contiguous and in this order;
// static_asserts in decode.hip check the offsets.
struct FwdParams {
    // ---- block 0: shape, lengths
    int nsplit, hk, g, b;
    // n / nsplit and n / hk as one multiply: magic = ceil(2^32 / d), or 0 for d = 1; exact for n * d < 2^32
    // (a runtime integer division costs the prologue of every workgroup some 100 cycles, and there were five)
    uint32_t nsplit_magic, hk_magic;
    int seqlen, reslen;
    int capacity;               // packed tokens a sequence can hold (set for every call; clamps device-side lengths)
    int res_cap;                // rows of the fp16 window (clamps device-side window lengths)
    int xcd_remap;              // (b * hk) % 8 == 0: keep the splits of one (batch, kv-head) on one XCD
    int seq_perm;               // workgroups take their sequence by rank of length (decode.hip: sequence_of_position)
    const int* seqlens;
    const int* reslens;
    // ---- block 1: q and the packed cache
    const uint16_t* q;
    int64_t q_sb, q_sh;
    const uint8_t* k_pack;
    const uint8_t* k_params;
    const uint8_t* v_pack;
    const uint8_t* v_params;
    const int* block_table;     // paged cache: page of (sequence, page slot); regions are then (page, kv-head)
    // ---- block 2
    int64_t kpack_bh, kparams_bh, vpack_bh, vparams_bh;
    int64_t bt_stride;
    int chunks_per_page;
    int neg_scale;              // softmax_scale < 0: the sign is folded into q
    float scale, scale_log2;    // scale_log2 = |softmax_scale| * log2(e)
    int few_waves;              // run the 8-wave variant of the kernel (layout.h: few_waves_variant)
    int ktensor;                // "k-tensor" mode, as in QpackParams (4 bits)
    // ---- fp16 window
    const uint16_t* k_res;
    const uint16_t* v_res;
    int64_t kres_sb, kres_st, kres_sh, vres_sb, vres_st, vres_sh;
    // ---- outputs and the split workspace: a counter per (batch, query head), and two slots of records that
    // launches use in turn (decode.hip, "protocol between the splits").  o_part / ml_part point into slot 0; slot 1
    // lies split_slot_words(...) 32-bit words behind, a split's residual words behind all partial outputs of its slot.
    uint32_t* o_part;   // [b][h][split][64] partial outputs: normalised (O / sum), two fp16 channels per word
    float* ml_part;     // [b][h][split][2] maximum (base-2 units) and sum of each split
    int* tickets;       // [b][h] arrival counters, kTicketStride ints apart, zero between launches; kSlotWord ints behind
                        // each, the slot of the next launch
    uint16_t* out;
    int64_t out_sb, out_sh;
    float* lse;         // optional [b][h]
    int h, bits;
    // ---- the rest
    int gs, bf16;
    // Decode step with append (lengths != nullptr): sequence i holds lengths[i] tokens, the last
    // lengths[i] % 128 of them in the fp16 window; its new token (k_new, v_new) is attended as the
    // window's next row, stored there, and a window that becomes full is packed behind the prefix.
    // seqlens / reslens / seqlen / reslen are not used then.
    int* lengths;               // [b], advanced by one by the last workgroup of each sequence
    int* step_tickets;          // [b] arrival counters, kTicketStride ints apart, zero between calls
    const uint16_t* k_new;
    const uint16_t* v_new;
    int64_t knew_sb, knew_sh, vnew_sb, vnew_sh;
};

// 32-bit words of one slot of the split workspace: partial outputs, residual words, (max, sum) pairs
// (a whole number of 256-byte blocks, so that the records of both slots are aligned alike)
inline size_t split_slot_words(size_t rows, size_t nsplit) {
    return (rows * nsplit * (2 * kPartialWords + 2) + 63) / 64 * 64;
}

inline uint32_t division_magic(uint32_t d) { return d <= 1 ? 0u : static_cast<uint32_t>(((1ull << 32) + d - 1) / d); }

hipError_t launch_qpack(const QpackParams& p, hipStream_t stream);
hipError_t launch_fwd(const FwdParams& p, hipStream_t stream);
#ifdef BITDECODE_PROF
hipError_t set_prof_buffer(unsigned long long* p);   // per-wave timeline buffer (tuning builds only)
#endif

}  // namespace bitdecode
