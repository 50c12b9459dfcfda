/* C ABI of the MI355X low-bit KV-cache decode library (libbitdecode.so).
 *
 * These entry points are what the reference's Python package binds for this path through
 * its pybind module `bit_decode_cuda` (csrc/bit_decode/decode_api.cpp:605-611):
 *   kvcache_pack_i2/_i4  ->  bitdecode_qpack
 *   fwd_kvcache_i2/_i4   ->  bitdecode_fwd
 * All pointers are device pointers unless stated; strides are in elements; every call is
 * asynchronous on `stream` (a hipStream_t passed as void*), keeps no state between calls
 * and returns 0 on success or a BITDECODE_E* code (no exceptions cross the boundary;
 * bitdecode_last_error() gives the message for the calling thread).
 */
#ifndef BITDECODE_H_
#define BITDECODE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BITDECODE_ABI_VERSION 5

enum {
    BITDECODE_OK = 0,
    BITDECODE_EINVAL = 1,      /* bad argument (shape, divisibility, null pointer)        */
    BITDECODE_EUNSUPPORTED = 2,/* valid request the kernels do not implement              */
    BITDECODE_EWORKSPACE = 3,  /* workspace too small                                     */
    BITDECODE_ELAUNCH = 4      /* HIP reported an error at launch                         */
};

enum { BITDECODE_FP16 = 0, BITDECODE_BF16 = 1 };

/* quant_mode of the reference's entry points (bit_decode_interface.py:17,50): K quantized per channel over
 * groups of tokens ("k-channel"), or per token over groups of channels like V ("k-tensor":
 * csrc/bit_decode/src/include/qpack.h:378-470, dequantize.h:403-475; its dispatch is commented out in the
 * reference, decode_api.cpp:195-203, 217-225).  "k-tensor" is implemented for 4 bits, as in the reference,
 * in every entry point; k_params then has v_params' shape. */
enum { BITDECODE_K_CHANNEL = 0, BITDECODE_K_TENSOR = 1 };

/* Quantize-pack n_tokens new tokens of K and V into the packed cache.
 * Replaces kvcache_qpack<num_bits> (csrc/bit_decode/decode_api.cpp:517-603) and the kernel it
 * launches (csrc/bit_decode/src/flash_fwd_kernel.h:732-1091).  K is quantized per channel over
 * groups of group_size consecutive tokens, V per token over groups of group_size consecutive
 * channels; scale and zero (= group minimum) are rounded to the element type and stored as fp16
 * bit patterns (for bf16: the bf16 value converted to fp16, the same number inside the fp16
 * normal range). */
typedef struct bitdecode_qpack_args {
    const void* k;             /* [b, n_tokens, h_k, 128] fp16/bf16, last dim contiguous    */
    const void* v;
    int64_t k_stride_b, k_stride_t, k_stride_h;
    int64_t v_stride_b, v_stride_t, v_stride_h;
    void* k_pack;              /* caller-allocated, reference shapes (see layout)           */
    void* k_params;
    void* v_pack;
    void* v_params;
    int32_t b, n_tokens, h_k, d;   /* d must be 128; n_tokens a multiple of 128            */
    int32_t cache_tokens;      /* capacity S of the packed tensors, multiple of 128         */
    int32_t dst_offset;        /* token offset of the first written chunk (multiple of 128) */
    const int32_t* dst_offsets;/* optional device int32[b]: per-sequence dst offset; a
                                  negative entry skips that sequence                        */
    int32_t bits;              /* 2 or 4                                                    */
    int32_t group_size;        /* 32, 64 or 128                                             */
    int32_t dtype;             /* BITDECODE_FP16 / BITDECODE_BF16                           */
    /* paged cache (csrc/bit_decode/decode_api.cpp:328-352, 420-425): with block_table set, the
     * four cache tensors are pools of pages, cache_tokens is the page size in tokens (a multiple
     * of 128) and token t of sequence i lives in page block_table[i * stride + t / cache_tokens].
     * Entries must lie in [0, num_pages): they are device data and are not checked. */
    const int32_t* block_table;/* optional device int32[b, max_pages_per_seq]               */
    int64_t block_table_stride;/* elements between the rows of two sequences                */
    int32_t max_pages_per_seq; /* columns of block_table                                    */
    int32_t num_pages;         /* pages in the pool (leading dimension of the cache)        */
    int32_t quant_mode;        /* BITDECODE_K_CHANNEL / BITDECODE_K_TENSOR                  */
} bitdecode_qpack_args;

int bitdecode_qpack(const bitdecode_qpack_args* args, void* stream);

/* Decode attention of one query token per sequence over [packed prefix || fp16 residual].
 * Replaces mha_fwd_kvcache<num_bits> (csrc/bit_decode/decode_api.cpp:301-441), the split-KV
 * kernel (flash_fwd_kernel.h:66-728) and the combine kernel (flash_fwd_kernel.h:1144-1327). */
typedef struct bitdecode_fwd_args {
    const void* q;             /* [b, 1, h, 128], last dim contiguous                       */
    int64_t q_stride_b, q_stride_h;
    const void* k_pack;
    const void* k_params;
    const void* v_pack;
    const void* v_params;
    int32_t cache_tokens;      /* capacity S of the packed tensors                          */
    int32_t seqlen_k;          /* valid packed tokens (multiple of 128), all sequences      */
    const int32_t* seqlens_k;  /* optional device int32[b] overriding seqlen_k              */
    const void* k_res;         /* optional fp16/bf16 residual window [b, R, h_k, 128]       */
    const void* v_res;
    int64_t kres_stride_b, kres_stride_t, kres_stride_h;
    int64_t vres_stride_b, vres_stride_t, vres_stride_h;
    int32_t res_len;           /* valid residual tokens, all sequences                      */
    const int32_t* res_lens;   /* optional device int32[b] overriding res_len               */
    int32_t max_seqlen_k;      /* upper bound of seqlens_k (host value, sizes the grid)     */
    int32_t max_res_len;       /* upper bound of res_lens                                   */
    void* out;                 /* [b, 1, h, 128] element type of q                          */
    int64_t out_stride_b, out_stride_h;
    float* softmax_lse;        /* optional [b, h] natural-log LSE                           */
    void* workspace;           /* >= bitdecode_fwd_workspace_bytes(...) or NULL if 1 split;
                                  ordinary device memory (hipMalloc, not host-coherent or
                                  fine-grained memory), 16-byte aligned.  ALL of it must be
                                  zero before the first call that uses it, and again before a
                                  call with another (b, h, num_splits) than the calls before:
                                  the kernel tells a split's record that is written from one
                                  that is not by its words being non-zero, and leaves the
                                  workspace ready for the next call of the same shape.  Calls
                                  that share a workspace must not overlap in time            */
    size_t workspace_bytes;
    int32_t b, h, h_k, d;      /* d must be 128, h % h_k == 0, h / h_k <= 8                 */
    int32_t bits, group_size, dtype;
    float softmax_scale;
    int32_t num_splits;        /* 0 = choose (bitdecode_num_splits); at most 512            */
    /* paged cache, as in bitdecode_qpack_args: cache_tokens is then the page size */
    const int32_t* block_table;
    int64_t block_table_stride;
    int32_t max_pages_per_seq;
    int32_t num_pages;
    int32_t quant_mode;        /* BITDECODE_K_CHANNEL / BITDECODE_K_TENSOR                  */
} bitdecode_fwd_args;

int bitdecode_fwd(const bitdecode_fwd_args* args, void* stream);

/* bitdecode_fwd for callers that cannot allocate device memory (code under HIP-graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results as bitdecode_fwd, except that `workspace` / `workspace_bytes` are ignored: partial outputs and
 * arrival counters live in an 8 MiB array inside the library's code object (one copy per GPU, held until the
 * process ends), and the call allocates nothing.  Limits: b * h <= 4096 and
 * bitdecode_fwd_workspace_bytes(b, h, num_splits) - 256 * b * h <= 7 MiB (1040 bytes per split and query
 * head), otherwise BITDECODE_EWORKSPACE.  Every call clears the part of the array it uses with a small fill
 * kernel in front of the decode kernel (calls of different shapes follow one another on the one array), so a
 * call is two or three launches.  All calls on one GPU share that array: calls that overlap in time on one
 * GPU (two streams, two host threads) race; calls on one stream do not.  The first call on a device looks up
 * the array's address (hipGetSymbolAddress): make it outside any stream capture. */
int bitdecode_fwd_static(const bitdecode_fwd_args* args, void* stream);

/* One decode step in one launch: attend the new token together with everything held, append it, and
 * quantize-pack the fp16 window when it fills.  This is the "residual kernel" the reference's figures
 * describe (imgs/overview.png, imgs/scheme.png) and its kernel traits still name
 * (csrc/bit_decode/src/include/kernel_traits.h:76,85: residual_block_size); the reference's main
 * branch ships no code for it.  Sequence i holds lengths[i] tokens before the call: the first
 * lengths[i] / 128 * 128 in the packed cache, the rest in rows 0.. of its window.  The call
 *   - attends q over [packed prefix || window || new token],
 *   - stores the new token in the window's next row,
 *   - if that makes 128 rows, packs them into the cache behind the prefix (they were attended in
 *     fp16 in this call and are read as codes from the next one on),
 *   - sets lengths[i] += 1.
 * A sequence whose window fills while its cache has no room for another 128 tokens is attended but
 * left unchanged (its length does not advance).  Lengths stay on the device, so a captured HIP graph of
 * this call can be replayed step after step with no host work.
 * In `fwd`: seqlen_k, seqlens_k, res_len, res_lens and max_seqlen_k are ignored; k_res / v_res are the
 * window (written), max_res_len its capacity in tokens (at least 128); the packed cache is written;
 * workspace must hold bitdecode_fwd_append_workspace_bytes(...) bytes, required for any split count,
 * all zero before the first call and before a call with another (b, h, num_splits), as for bitdecode_fwd. */
typedef struct bitdecode_fwd_append_args {
    bitdecode_fwd_args fwd;
    int32_t* lengths;          /* device int32[b], read and advanced                        */
    const void* k_new;         /* [b, 1, h_k, 128] element type of q, last dim contiguous   */
    const void* v_new;
    int64_t knew_stride_b, knew_stride_h;
    int64_t vnew_stride_b, vnew_stride_h;
    int32_t max_len;           /* host upper bound of lengths before the step (sizes the grid) */
} bitdecode_fwd_append_args;

int bitdecode_fwd_append(const bitdecode_fwd_append_args* args, void* stream);
size_t bitdecode_fwd_append_workspace_bytes(int32_t b, int32_t h, int32_t num_splits);

/* Split count the library would choose for this problem (host function, no GPU work);
 * replaces num_splits_heuristic (csrc/bit_decode/decode_api.cpp:234-268), retuned for 256 CUs.
 * num_cus <= 0 queries the current device; returns -1 for an unsupported (bits, group_size). */
int bitdecode_num_splits(int32_t b, int32_t h_k, int32_t max_seqlen_k, int32_t max_res_len,
                         int32_t num_cus, int32_t bits, int32_t group_size);

/* The same for a call that takes per-sequence lengths from the device (bitdecode_fwd_args.seqlens_k) when
 * per_sequence_lengths != 0: a batch of unequal sequences gets up to two workgroups per compute unit, dealt
 * out so that long sequences share a unit with short ones.  This is the count bitdecode_fwd chooses itself
 * with num_splits = 0.  No counterpart in the reference, whose heuristic only sees the longest sequence. */
int bitdecode_num_splits_for(int32_t b, int32_t h_k, int32_t max_seqlen_k, int32_t max_res_len,
                             int32_t num_cus, int32_t bits, int32_t group_size, int32_t per_sequence_lengths);

/* Workspace the split path needs: a 256-byte block per query head (arrival counter and the slot the next call
 * uses), then two slots of records that calls use in turn; a record per (query head, split) is a partial output
 * (normalised, 64 words of two fp16), 64 residual words for outputs too large for fp16 alone, and an fp32
 * (max, sum) pair: 256 * b * h + 2 * round_up(1040 * b * h * num_splits, 256) bytes (replaces the per-call
 * torch::empty of out_accum / softmax_lse_accum, csrc/bit_decode/decode_api.cpp:292-295). */
size_t bitdecode_fwd_workspace_bytes(int32_t b, int32_t h, int32_t num_splits);

int bitdecode_abi_version(void);
const char* bitdecode_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* BITDECODE_H_ */
