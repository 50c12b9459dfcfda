// C ABI of libbitdecode.so: argument validation, split choice, workspace carving, launches.
// Host-side counterpart of csrc/bit_decode/decode_api.cpp:301-441 (decode) and :517-603 (pack)
// in the reference; unsupported configurations return an error instead of silently doing nothing
// (decode_api.cpp:190-202 leaves the output uninitialised there).
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include <algorithm>
#include <atomic>
#include <cmath>

#include "../../include/bitdecode.h"
#include "kernels.h"
#include "layout.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Scratch of bitdecode_fwd_static: device memory that belongs to the library's code object, so the call
// needs no allocation.  Every GPU that loads the library holds its own copy until the process ends.
// Layout: arrival counters for up to kStaticHeads (batch x query head) rows, one 256-byte block each,
// then the two record slots of the splits.  Calls of different shapes follow one another on this one
// array, and the decode kernel expects the part it uses to be zero when a shape starts on it: every
// call therefore clears its counters and record slots with a small fill kernel in front of the decode
// kernel (a kernel, not a memset node: the call may be recorded into a HIP graph).
constexpr size_t kStaticHeads = 4096;
constexpr size_t kStaticCounterBytes = kStaticHeads * bitdecode::kTicketStride * sizeof(int);     // 1 MiB
constexpr size_t kStaticScratchBytes = size_t(8) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
// address of `scratch` on each device (the name itself is only a host-side handle)
std::atomic<unsigned char*> g_scratch_ptr[64] = {};

// 16-byte stores of zero over [p, p + n16 * 16)
__global__ void zero_fill_kernel(uint4* p, size_t n16) {
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) p[i] = uint4{0, 0, 0, 0};
}
hipError_t zero_fill(void* p, size_t bytes, hipStream_t stream) {      // bytes: a multiple of 16
    const size_t n16 = bytes / 16;
    if (n16 == 0) return hipSuccess;
    const unsigned int blocks = static_cast<unsigned int>(std::min<size_t>((n16 + 255) / 256, 1024));
    hipLaunchKernelGGL(zero_fill_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<uint4*>(p), n16);
    return hipGetLastError();
}

int check_quant(int bits, int gs, int dtype, int d) {
    if (d != bitdecode::kHeadDim) return fail(BITDECODE_EUNSUPPORTED, "head_dim %d unsupported (only 128)", d);
    if (bits != 2 && bits != 4) return fail(BITDECODE_EUNSUPPORTED, "num_bits %d unsupported (2 or 4)", bits);
    if (gs != 32 && gs != 64 && gs != 128)
        return fail(BITDECODE_EUNSUPPORTED, "group_size %d unsupported (32, 64 or 128)", gs);
    if (dtype != BITDECODE_FP16 && dtype != BITDECODE_BF16)
        return fail(BITDECODE_EUNSUPPORTED, "dtype %d unsupported (fp16=0, bf16=1)", dtype);
    return 0;
}

int check_mode(int quant_mode, int bits) {
    if (quant_mode != BITDECODE_K_CHANNEL && quant_mode != BITDECODE_K_TENSOR)
        return fail(BITDECODE_EINVAL, "quant_mode %d (k-channel=0, k-tensor=1)", quant_mode);
    if (quant_mode == BITDECODE_K_TENSOR && bits != 4)
        return fail(BITDECODE_EUNSUPPORTED, "quant_mode k-tensor is implemented for 4 bits only (as in the reference)");
    return 0;
}

int query_cus() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    return n;
}

// A wave streams whole packed units (64 tokens at 4 bits, 128 at 2 bits) plus a share of the 16-token
// fp16 tiles, and a workgroup has 16 or 12 waves.  Pick the number of splits so that the grid is about
// one workgroup per CU (a second round of workgroups costs far more than idle waves) while a
// workgroup still gets at least one unit for every second wave (or four fp16 tiles per unit when
// nothing is packed); measured optimum over 4K-128K tokens, 1-128 (batch, kv-head) pairs.
int choose_splits(int b, int hk, int max_seqlen_k, int max_res_len, int num_cus, int bits, int gs) {
    const int nw = bitdecode::decode_waves(bits, gs);
    const int packed_units = max_seqlen_k / bitdecode::unit_tokens(bits);
    const int tiles = (max_res_len + 15) / 16;
    const int units = packed_units > 0 ? packed_units : (tiles + 3) / 4;
    if (units <= 0) return 1;
    const int heads = std::max(1, b * hk);
    const int by_occupancy = std::max(1, (num_cus + heads - 1) / heads);
    const int by_work = std::max(1, (2 * units + nw - 1) / nw);
    int n = std::min(std::min(by_occupancy, by_work), 256);
    // drop splits that would be empty: ceil(units / n) units per split
    const int ups = (units + n - 1) / n;
    n = (units + ups - 1) / ups;
    return std::max(1, n);
}

// The 4-bit kernels also exist with 8 waves per workgroup (decode.hip: launch_fwd_tt), used whenever the packed
// prefix is the bulk of the work.  With per-sequence lengths on the device the workgroups of the longest
// sequences can be left streaming alone at the end, where 16 waves keep more bytes in flight per compute
// unit: then only up to 32 units per workgroup (measured on a batch of 16 sequences of 1.9K-8K tokens: 26.2
// against 26.6 us; equal-length batches of every size measured gain 1-7 % from the 8 waves).
bool use_few_waves(int bits, int gs, int max_s, int max_r, int nsplit, bool device_lengths) {
    const int packed_units = max_s / bitdecode::unit_tokens(bits);
    const int units_per_wg = (packed_units + nsplit - 1) / nsplit;
    return bitdecode::few_waves_variant(bits, gs) && units_per_wg >= 1 && max_r <= 512 &&
           (!device_lengths || units_per_wg <= 32);
}

// Split count for a call; `ragged` = per-sequence lengths come from the device (the host only has their bound).
// Two workgroups of the 8-wave kernels fit a compute unit (78 KB of LDS and 125 registers each).  A batch of
// unequal sequences is better served by twice as many workgroups of half the size: the two that share a unit
// add up, and the kernel orders the sequences so that the longest shares with the shortest (decode.hip:
// sequence_of_position).  16 sequences of 1.9K-8K tokens: 62 units on the busiest unit with one workgroup
// per unit, 49.5 with two.  Only for batches that fill the machine with one or two splits: the host cannot tell a
// ragged batch from an equal one, and equal sequences lose by the doubling what the extra splits cost
// (32 x 8 heads: nothing; 16 x 8: 1.5 %; 8 x 8 and 4 x 8, where 4 and 8 splits would become 8 and 16: 9-12 %).
int choose_splits_for(int b, int hk, int max_s, int max_r, int num_cus, int bits, int gs, bool ragged) {
    const int n1 = choose_splits(b, hk, max_s, max_r, num_cus, bits, gs);
    if (!ragged || b < 2 || n1 > 2) return n1;
    const int n2 = choose_splits(b, hk, max_s, max_r, 2 * num_cus, bits, gs);
    if (n2 > n1 && static_cast<int64_t>(n2) * b * hk <= 2 * num_cus && use_few_waves(bits, gs, max_s, max_r, n2, true))
        return n2;
    return n1;
}

}  // namespace

extern "C" {

int bitdecode_abi_version(void) { return BITDECODE_ABI_VERSION; }

const char* bitdecode_last_error(void) { return g_err; }

int bitdecode_num_splits(int32_t b, int32_t h_k, int32_t max_seqlen_k, int32_t max_res_len, int32_t num_cus,
                         int32_t bits, int32_t group_size) {
    if (num_cus <= 0) num_cus = query_cus();
    if (check_quant(bits, group_size, BITDECODE_FP16, bitdecode::kHeadDim)) return -1;
    return choose_splits(b, h_k, max_seqlen_k, max_res_len, num_cus, bits, group_size);
}

int bitdecode_num_splits_for(int32_t b, int32_t h_k, int32_t max_seqlen_k, int32_t max_res_len, int32_t num_cus,
                             int32_t bits, int32_t group_size, int32_t per_sequence_lengths) {
    if (num_cus <= 0) num_cus = query_cus();
    if (check_quant(bits, group_size, BITDECODE_FP16, bitdecode::kHeadDim)) return -1;
    return choose_splits_for(b, h_k, max_seqlen_k, max_res_len, num_cus, bits, group_size, per_sequence_lengths != 0);
}

// [tickets: one 256-byte block per (batch, query head)][o_part][ml_part]
static size_t ticket_bytes(int32_t b, int32_t h) { return static_cast<size_t>(b) * h * bitdecode::kTicketStride * sizeof(int); }

// two slots of records behind the counters (kernels.h: split_slot_words)
static size_t slots_bytes(int32_t b, int32_t h, int32_t num_splits) {
    return 2 * bitdecode::split_slot_words(static_cast<size_t>(b) * h, static_cast<size_t>(num_splits)) * sizeof(uint32_t);
}

size_t bitdecode_fwd_workspace_bytes(int32_t b, int32_t h, int32_t num_splits) {
    if (num_splits <= 1) return 0;
    return ticket_bytes(b, h) + slots_bytes(b, h, num_splits);
}

// paged cache: cache_tokens is the page size; the table must cover `tokens` per sequence
static int check_paging(const int32_t* block_table, int64_t stride, int32_t max_pages, int32_t num_pages,
                        int32_t page_tokens, int32_t tokens) {
    if (!block_table) return BITDECODE_OK;
    if (max_pages <= 0 || num_pages <= 0 || stride < max_pages)
        return fail(BITDECODE_EINVAL, "block_table: %d pages per sequence, stride %lld, pool of %d pages", max_pages,
                    static_cast<long long>(stride), num_pages);
    if (static_cast<int64_t>(tokens) > static_cast<int64_t>(max_pages) * page_tokens)
        return fail(BITDECODE_EINVAL, "block_table covers %d x %d tokens per sequence, %d needed", max_pages, page_tokens,
                    tokens);
    return BITDECODE_OK;
}

int bitdecode_qpack(const bitdecode_qpack_args* a, void* stream) {
    using namespace bitdecode;
    if (!a) return fail(BITDECODE_EINVAL, "args is null");
    if (int rc = check_quant(a->bits, a->group_size, a->dtype, a->d)) return rc;
    if (int rc = check_mode(a->quant_mode, a->bits)) return rc;
    if (a->b < 0 || a->h_k <= 0 || a->n_tokens < 0) return fail(BITDECODE_EINVAL, "negative size");
    if (a->n_tokens % kChunk) return fail(BITDECODE_EINVAL, "n_tokens %d is not a multiple of 128", a->n_tokens);
    if (a->cache_tokens % kChunk || a->cache_tokens <= 0)
        return fail(BITDECODE_EINVAL, "cache_tokens %d is not a positive multiple of 128", a->cache_tokens);
    // tokens one sequence can hold: the tensor capacity, or what its row of the block table covers
    const int64_t capacity = a->block_table ? static_cast<int64_t>(a->max_pages_per_seq) * a->cache_tokens
                                            : a->cache_tokens;
    if (!a->dst_offsets) {
        if (a->dst_offset < 0 || a->dst_offset % kChunk)
            return fail(BITDECODE_EINVAL, "dst_offset %d is not a multiple of 128", a->dst_offset);
        if (static_cast<int64_t>(a->dst_offset) + a->n_tokens > capacity)
            return fail(BITDECODE_EINVAL, "dst_offset %d + n_tokens %d exceeds cache capacity %lld", a->dst_offset,
                        a->n_tokens, static_cast<long long>(capacity));
    } else if (a->n_tokens > capacity) {
        return fail(BITDECODE_EINVAL, "n_tokens %d exceeds cache capacity %lld", a->n_tokens,
                    static_cast<long long>(capacity));
    }
    if (int rc = check_paging(a->block_table, a->block_table_stride, a->max_pages_per_seq, a->num_pages,
                              a->cache_tokens, 0))
        return rc;
    if (a->n_tokens == 0 || a->b == 0) return BITDECODE_OK;
    if (!a->k || !a->v || !a->k_pack || !a->k_params || !a->v_pack || !a->v_params)
        return fail(BITDECODE_EINVAL, "null tensor pointer");
    if (!aligned16(a->k) || !aligned16(a->v) || !aligned16(a->k_pack) || !aligned16(a->k_params) ||
        !aligned16(a->v_pack) || !aligned16(a->v_params))
        return fail(BITDECODE_EINVAL, "tensor pointers must be 16-byte aligned");
    const int64_t strides[6] = {a->k_stride_b, a->k_stride_t, a->k_stride_h, a->v_stride_b, a->v_stride_t, a->v_stride_h};
    for (int64_t s : strides)
        if (s % 8) return fail(BITDECODE_EINVAL, "K/V strides must be multiples of 8 elements");

    QpackParams P{};
    P.k = static_cast<const uint16_t*>(a->k);
    P.v = static_cast<const uint16_t*>(a->v);
    P.k_sb = a->k_stride_b; P.k_st = a->k_stride_t; P.k_sh = a->k_stride_h;
    P.v_sb = a->v_stride_b; P.v_st = a->v_stride_t; P.v_sh = a->v_stride_h;
    P.k_pack = static_cast<uint8_t*>(a->k_pack);
    P.k_params = static_cast<uint8_t*>(a->k_params);
    P.v_pack = static_cast<uint8_t*>(a->v_pack);
    P.v_params = static_cast<uint8_t*>(a->v_params);
    P.kpack_bh = code_region_bytes(a->cache_tokens, a->bits);
    P.vpack_bh = P.kpack_bh;
    P.ktensor = a->quant_mode == BITDECODE_K_TENSOR;
    P.kparams_bh = P.ktensor ? v_param_region_bytes(a->cache_tokens, a->group_size)
                             : k_param_region_bytes(a->cache_tokens, a->group_size);
    P.vparams_bh = v_param_region_bytes(a->cache_tokens, a->group_size);
    P.b = a->b; P.n_tokens = a->n_tokens; P.hk = a->h_k;
    P.dst_offset = a->dst_offset;
    P.dst_offsets = a->dst_offsets;
    P.capacity = static_cast<int>(std::min<int64_t>(capacity, INT32_MAX / 2));
    P.bits = a->bits; P.gs = a->group_size; P.bf16 = a->dtype == BITDECODE_BF16;
    P.block_table = a->block_table; P.bt_stride = a->block_table_stride;
    P.chunks_per_page = a->cache_tokens / kChunk;
    hipError_t e = launch_qpack(P, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(BITDECODE_ELAUNCH, "qpack launch failed: %s", hipGetErrorString(e));
    return BITDECODE_OK;
}

// bytes of the per-sequence step counters that lead a step workspace
static size_t step_ticket_bytes(int32_t b) { return static_cast<size_t>(b) * bitdecode::kTicketStride * sizeof(int); }

size_t bitdecode_fwd_append_workspace_bytes(int32_t b, int32_t h, int32_t num_splits) {
    return step_ticket_bytes(b) + bitdecode_fwd_workspace_bytes(b, h, num_splits);
}

// decode, or (step != null) decode step with append
static int run_fwd(const bitdecode_fwd_args* a, const bitdecode_fwd_append_args* step, void* stream,
                   unsigned char* static_scratch = nullptr) {
    using namespace bitdecode;
    if (!a) return fail(BITDECODE_EINVAL, "args is null");
    if (int rc = check_quant(a->bits, a->group_size, a->dtype, a->d)) return rc;
    if (int rc = check_mode(a->quant_mode, a->bits)) return rc;
    if (a->b <= 0 || a->h <= 0 || a->h_k <= 0) return fail(BITDECODE_EINVAL, "batch and head counts must be positive");
    if (a->h % a->h_k) return fail(BITDECODE_EINVAL, "h %d is not a multiple of h_k %d", a->h, a->h_k);
    const int g = a->h / a->h_k;
    if (g > kMaxGroupHeads)
        return fail(BITDECODE_EUNSUPPORTED, "%d query heads per kv head unsupported (at most %d)", g, kMaxGroupHeads);
    int max_s = a->seqlens_k ? a->max_seqlen_k : a->seqlen_k;
    int max_r = a->res_lens ? a->max_res_len : a->res_len;
    if (step) {
        // lengths live on the device; the host bound sizes the grid: up to max_len tokens before the
        // step, of which whole chunks are packed, and a window of up to 128 tokens with the new one
        if (!step->lengths || !step->k_new || !step->v_new)
            return fail(BITDECODE_EINVAL, "decode step: lengths, k_new and v_new are required");
        if (step->max_len < 0) return fail(BITDECODE_EINVAL, "decode step: max_len %d is negative", step->max_len);
        if (!a->k_res || !a->v_res || a->max_res_len < kChunk)
            return fail(BITDECODE_EINVAL, "decode step: a residual window of at least 128 tokens is required "
                                          "(max_res_len = its capacity, got %d)", a->max_res_len);
        if (!aligned16(step->k_new) || !aligned16(step->v_new))
            return fail(BITDECODE_EINVAL, "tensor pointers must be 16-byte aligned");
        const int64_t ns[4] = {step->knew_stride_b, step->knew_stride_h, step->vnew_stride_b, step->vnew_stride_h};
        for (int64_t s : ns)
            if (s % 8) return fail(BITDECODE_EINVAL, "k_new / v_new strides must be multiples of 8 elements");
        max_s = step->max_len / kChunk * kChunk;
        max_r = kChunk;
    }
    if (max_s < 0 || max_r < 0) return fail(BITDECODE_EINVAL, "negative length");
    if (max_s % kChunk) return fail(BITDECODE_EINVAL, "packed length %d is not a multiple of 128", max_s);
    if (!a->block_table && max_s > a->cache_tokens)
        return fail(BITDECODE_EINVAL, "packed length %d exceeds cache capacity %d", max_s, a->cache_tokens);
    if (a->block_table && (a->cache_tokens <= 0 || a->cache_tokens % kChunk))
        return fail(BITDECODE_EINVAL, "page size %d is not a positive multiple of 128", a->cache_tokens);
    if (int rc = check_paging(a->block_table, a->block_table_stride, a->max_pages_per_seq, a->num_pages,
                              a->cache_tokens, max_s))
        return rc;
    if (max_s > 0 && (a->cache_tokens % kChunk)) return fail(BITDECODE_EINVAL, "cache_tokens must be a multiple of 128");
    if (!a->q || !a->out) return fail(BITDECODE_EINVAL, "q/out is null");
    if ((max_s > 0 || step) && (!a->k_pack || !a->k_params || !a->v_pack || !a->v_params))
        return fail(BITDECODE_EINVAL, "null packed-cache pointer");
    if (step && (a->cache_tokens <= 0 || a->cache_tokens % kChunk))
        return fail(BITDECODE_EINVAL, "cache_tokens %d is not a positive multiple of 128", a->cache_tokens);
    if (max_r > 0 && (!a->k_res || !a->v_res)) return fail(BITDECODE_EINVAL, "null residual pointer");
    if (!aligned16(a->q) || !aligned16(a->k_pack) || !aligned16(a->k_params) || !aligned16(a->v_pack) ||
        !aligned16(a->v_params) || !aligned16(a->k_res) || !aligned16(a->v_res))
        return fail(BITDECODE_EINVAL, "tensor pointers must be 16-byte aligned");
    const int64_t strides[8] = {a->q_stride_b, a->q_stride_h, a->kres_stride_b, a->kres_stride_t, a->kres_stride_h,
                                a->vres_stride_b, a->vres_stride_t, a->vres_stride_h};
    for (int64_t s : strides)
        if (s % 8) return fail(BITDECODE_EINVAL, "q and residual strides must be multiples of 8 elements");

    int nsplit = a->num_splits;
    if (nsplit < 0) return fail(BITDECODE_EINVAL, "num_splits %d is negative", nsplit);
    if (nsplit > 512) return fail(BITDECODE_EINVAL, "num_splits %d is above the limit of 512", nsplit);
    const int cus = query_cus();
    if (nsplit == 0)
        nsplit = choose_splits_for(a->b, a->h_k, max_s, max_r, cus, a->bits, a->group_size, a->seqlens_k && !step);
    if (nsplit > 1 && slots_bytes(a->b, a->h, nsplit) >= (size_t(1) << 31))
        return fail(BITDECODE_EUNSUPPORTED, "%d splits x %d x %d heads: partial outputs of 2 GiB or more", nsplit, a->b, a->h);
    // the kernel divides workgroup ids and unit counts by the split count and the head count with a
    // multiply (kernels.h: division_magic), exact while numerator x divisor stays below 2^32
    {
        const uint64_t wgs = static_cast<uint64_t>(nsplit) * a->b * a->h_k;
        // lengths read on the device are clamped to the capacity by the kernel, not to max_seqlen_k: that is the bound
        const uint64_t cap_tokens = a->block_table ? static_cast<uint64_t>(a->max_pages_per_seq) * a->cache_tokens
                                                   : static_cast<uint64_t>(a->cache_tokens);
        const uint64_t longest = (a->seqlens_k || step) ? std::max<uint64_t>(cap_tokens, max_s) : static_cast<uint64_t>(max_s);
        const uint64_t units = longest / 64 + static_cast<uint64_t>(nsplit);
        if (wgs * std::max(nsplit, a->h_k) >= (1ull << 32) || units * nsplit >= (1ull << 32))
            return fail(BITDECODE_EUNSUPPORTED, "%d splits x %d x %d kv heads: too many workgroups", nsplit, a->b, a->h_k);
    }
    if (static_scratch) {
        const size_t rows = static_cast<size_t>(a->b) * a->h;
        const size_t need = nsplit > 1 ? slots_bytes(a->b, a->h, nsplit) : 0;
        if (rows > kStaticHeads || need > kStaticScratchBytes - kStaticCounterBytes)
            return fail(BITDECODE_EWORKSPACE, "bitdecode_fwd_static: %d splits x %zu (batch x head) rows need %zu bytes; the "
                        "built-in scratch holds %zu rows and %zu bytes (use bitdecode_fwd with a workspace)", nsplit, rows,
                        need, kStaticHeads, kStaticScratchBytes - kStaticCounterBytes);
    } else if (nsplit > 1 || step) {
        const size_t need = step ? bitdecode_fwd_append_workspace_bytes(a->b, a->h, nsplit)
                                 : bitdecode_fwd_workspace_bytes(a->b, a->h, nsplit);
        if (!a->workspace || a->workspace_bytes < need)
            return fail(BITDECODE_EWORKSPACE, "workspace of %zu bytes needed for %d splits, got %zu", need, nsplit,
                        a->workspace ? a->workspace_bytes : size_t(0));
        if (!aligned16(a->workspace)) return fail(BITDECODE_EINVAL, "workspace must be 16-byte aligned");
    }

    FwdParams P{};
    P.q = static_cast<const uint16_t*>(a->q);
    P.q_sb = a->q_stride_b; P.q_sh = a->q_stride_h;
    P.k_pack = static_cast<const uint8_t*>(a->k_pack);
    P.k_params = static_cast<const uint8_t*>(a->k_params);
    P.v_pack = static_cast<const uint8_t*>(a->v_pack);
    P.v_params = static_cast<const uint8_t*>(a->v_params);
    P.kpack_bh = code_region_bytes(a->cache_tokens, a->bits);
    P.vpack_bh = P.kpack_bh;
    P.ktensor = a->quant_mode == BITDECODE_K_TENSOR;
    P.kparams_bh = P.ktensor ? v_param_region_bytes(a->cache_tokens, a->group_size)
                             : k_param_region_bytes(a->cache_tokens, a->group_size);
    P.vparams_bh = v_param_region_bytes(a->cache_tokens, a->group_size);
    P.k_res = static_cast<const uint16_t*>(a->k_res);
    P.v_res = static_cast<const uint16_t*>(a->v_res);
    P.kres_sb = a->kres_stride_b; P.kres_st = a->kres_stride_t; P.kres_sh = a->kres_stride_h;
    P.vres_sb = a->vres_stride_b; P.vres_st = a->vres_stride_t; P.vres_sh = a->vres_stride_h;
    P.seqlens = a->seqlens_k; P.reslens = a->res_lens;
    P.seqlen = a->seqlen_k; P.reslen = a->res_len;
    P.out = static_cast<uint16_t*>(a->out);
    P.out_sb = a->out_stride_b; P.out_sh = a->out_stride_h;
    P.lse = a->softmax_lse;
    P.b = a->b; P.h = a->h; P.hk = a->h_k; P.g = g; P.nsplit = nsplit;
    P.scale = a->softmax_scale;
    P.scale_log2 = fabsf(a->softmax_scale) * 1.4426950408889634f;   // decode_api.cpp:128-142
    P.neg_scale = a->softmax_scale < 0.0f;
    P.xcd_remap = (a->b * a->h_k) % 8 == 0 && nsplit > 1;
    P.few_waves = use_few_waves(a->bits, a->group_size, max_s, max_r, nsplit, a->seqlens_k != nullptr || step != nullptr);
    // more than one workgroup per compute unit and lengths that differ: the kernel deals the sequences out so
    // that long ones share a unit with short ones (a pure permutation of the batch index, from the lengths
    // on the device; not in the step with append, whose launch itself advances the lengths)
    P.seq_perm = a->seqlens_k && !step && a->b >= 2 && a->b <= 64 && static_cast<int64_t>(nsplit) * a->b * a->h_k > cus;
    P.nsplit_magic = division_magic(static_cast<uint32_t>(nsplit));
    P.hk_magic = division_magic(static_cast<uint32_t>(a->h_k));
    P.block_table = a->block_table; P.bt_stride = a->block_table_stride;
    P.chunks_per_page = a->block_table ? a->cache_tokens / kChunk : 1;
    P.bits = a->bits; P.gs = a->group_size; P.bf16 = a->dtype == BITDECODE_BF16;
    {
        const int64_t cap = a->block_table ? static_cast<int64_t>(a->max_pages_per_seq) * a->cache_tokens : a->cache_tokens;
        P.capacity = static_cast<int>(std::min<int64_t>(cap, INT32_MAX / 2));
        P.res_cap = max_r;
    }
    uint8_t* ws = static_cast<uint8_t*>(a->workspace);
    if (step) {
        P.lengths = step->lengths;
        P.step_tickets = reinterpret_cast<int*>(ws);
        ws += step_ticket_bytes(a->b);
        P.k_new = static_cast<const uint16_t*>(step->k_new);
        P.v_new = static_cast<const uint16_t*>(step->v_new);
        P.knew_sb = step->knew_stride_b; P.knew_sh = step->knew_stride_h;
        P.vnew_sb = step->vnew_stride_b; P.vnew_sh = step->vnew_stride_h;
    }
    if (nsplit > 1) {
        const size_t records = static_cast<size_t>(nsplit) * a->b * a->h;
        if (static_scratch) {
            P.tickets = reinterpret_cast<int*>(static_scratch);
            P.o_part = reinterpret_cast<uint32_t*>(static_scratch + kStaticCounterBytes);
        } else {
            P.tickets = reinterpret_cast<int*>(ws);
            P.o_part = reinterpret_cast<uint32_t*>(ws + ticket_bytes(a->b, a->h));
        }
        P.ml_part = reinterpret_cast<float*>(P.o_part + 2 * records * kPartialWords);
        if (static_scratch) {
            // another shape may have used the array before: counters and record slots of this call start at zero
            hipError_t e = zero_fill(P.tickets, ticket_bytes(a->b, a->h), static_cast<hipStream_t>(stream));
            if (e == hipSuccess) e = zero_fill(P.o_part, slots_bytes(a->b, a->h, nsplit), static_cast<hipStream_t>(stream));
            if (e != hipSuccess) return fail(BITDECODE_ELAUNCH, "decode launch failed: %s", hipGetErrorString(e));
        }
    }
    hipError_t e = launch_fwd(P, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(BITDECODE_ELAUNCH, "decode launch failed: %s", hipGetErrorString(e));
    return BITDECODE_OK;
}

int bitdecode_fwd(const bitdecode_fwd_args* a, void* stream) { return run_fwd(a, nullptr, stream); }

int bitdecode_fwd_static(const bitdecode_fwd_args* a, void* stream) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess || dev < 0 || dev >= 64)
        return fail(BITDECODE_ELAUNCH, "bitdecode_fwd_static: no current device (%s)", hipGetErrorString(e));
    unsigned char* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // once per device, with that device current: where this device keeps its copy of the array
        if (hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)); e != hipSuccess || !ptr)
            return fail(BITDECODE_ELAUNCH, "bitdecode_fwd_static: address of the built-in scratch: %s", hipGetErrorString(e));
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    return run_fwd(a, nullptr, stream, ptr);
}

int bitdecode_fwd_append(const bitdecode_fwd_append_args* a, void* stream) {
    if (!a) return fail(BITDECODE_EINVAL, "args is null");
    return run_fwd(&a->fwd, a, stream);
}

#ifdef BITDECODE_PROF
int bitdecode_prof_set(void* p) { return bitdecode::set_prof_buffer(static_cast<unsigned long long*>(p)) != hipSuccess; }
#endif

}  // extern "C"
