// Quantize-pack kernel: fp16/bf16 K,V -> 2/4-bit codes + scale/zero in the gfx950 layout of
// layout.h.  One workgroup (256 threads) packs one 128-token chunk of one (batch, kv-head) with the
// shared chunk routine of qpack_chunk.h.  HBM-bound: reads 64 KB, writes chunk_code_bytes*2 + params
// per chunk.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"
#include "layout.h"
#include "qpack_chunk.h"

namespace bitdecode {
namespace {

template <int BITS, int GS, bool BF16, bool KT, bool STREAM>
__global__ __launch_bounds__(qp::kPackThreads) void qpack_kernel(QpackParams P) {
    __shared__ qp::PackLds<GS> L;
    const int tid = threadIdx.x;
    const int ci_src = blockIdx.x, hk = blockIdx.y, bi = blockIdx.z;
    const int dst_base = P.dst_offsets ? P.dst_offsets[bi] : P.dst_offset;
    if (dst_base < 0) return;       // a negative per-sequence offset skips that sequence (whole workgroup)
    const int dst_tok = dst_base + ci_src * kChunk;
    // a device-side offset the host never saw: not on a chunk boundary, or past the cache -> nothing is written
    if ((dst_base & (kChunk - 1)) != 0 || dst_tok + kChunk > P.capacity) return;
    const ChunkPlace place = chunk_place(P.block_table, P.bt_stride, P.chunks_per_page, bi, hk, P.hk, dst_tok / kChunk);
    const qp::ChunkDst D = qp::chunk_dst<BITS, GS, KT>(P.k_pack, P.k_params, P.v_pack, P.v_params, P.kpack_bh, P.kparams_bh,
                                                   P.vpack_bh, P.vparams_bh, place);
    const uint16_t* ks = P.k + bi * P.k_sb + static_cast<int64_t>(ci_src) * kChunk * P.k_st + hk * P.k_sh;
    const uint16_t* vs = P.v + bi * P.v_sb + static_cast<int64_t>(ci_src) * kChunk * P.v_st + hk * P.v_sh;
    const int64_t k_st = P.k_st, v_st = P.v_st;
    // 4 bits, group 128: with the V tile prefetched the kernel needs 133 registers and only three
    // workgroups fit a CU; fetched after the K side it needs 114, a fourth workgroup fits (LDS: 40 KB
    // each) and the kernel is 10 % faster.  (At group 64 a fourth workgroup was measured 3 % slower.)
    qp::pack_chunk<BITS, GS, BF16, !(BITS == 4 && GS == 128), KT, STREAM>(
        L, tid, true, [=](int n) { return ks + n * k_st; }, [=](int n) { return vs + n * v_st; }, D);
}

template <int BITS, int GS, bool KT, bool STREAM>
hipError_t launch_qpack_tt(const QpackParams& P, dim3 grid, hipStream_t stream) {
    if (P.bf16) {
        hipLaunchKernelGGL((qpack_kernel<BITS, GS, true, KT, STREAM>), grid, dim3(256), 0, stream, P);
    } else {
        hipLaunchKernelGGL((qpack_kernel<BITS, GS, false, KT, STREAM>), grid, dim3(256), 0, stream, P);
    }
    return hipGetLastError();
}

template <int BITS, int GS>
hipError_t launch_qpack_t(const QpackParams& P, hipStream_t stream) {
    dim3 grid(P.n_tokens / kChunk, P.hk, P.b);
    // a bulk pack (more chunks than two rounds of workgroups over the 256 compute units) streams its input
    // and output past the caches; an append of a block per sequence does not
    const bool stream_data = static_cast<int64_t>(grid.x) * grid.y * grid.z >= 512;
    if (P.ktensor) {      // K quantized per token like V: 4 bits only, as in the reference (qpack.h:385)
        if constexpr (BITS == 4) {
            return stream_data ? launch_qpack_tt<BITS, GS, true, true>(P, grid, stream)
                               : launch_qpack_tt<BITS, GS, true, false>(P, grid, stream);
        } else {
            return hipErrorInvalidValue;
        }
    }
    return stream_data ? launch_qpack_tt<BITS, GS, false, true>(P, grid, stream)
                       : launch_qpack_tt<BITS, GS, false, false>(P, grid, stream);
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
