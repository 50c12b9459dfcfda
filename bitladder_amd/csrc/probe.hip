// Read probe: kernels that do nothing but read a buffer, in the launch shapes a decode kernel could use.
// Their time over the bytes of a decode step is what the memory system alone allows for that step; the
// benchmark reports the best of them next to the decode kernel's time.  Built into a library of its own
// (libbitdecode_probe.so) that only the benchmark loads: it is no part of the decode path or its C ABI.
//
//   int bitprobe_read(src, bytes, grid, block, mode, depth, nt, pattern, stream)
//     grid, block  workgroups and threads per workgroup (block a multiple of 64, at most 1024)
//     mode         0: 16-byte loads into registers, `depth` independent loads per lane in flight
//                  1: direct-to-LDS loads (global_load_lds_dwordx4, 1 KB per wave and instruction), a ring of
//                     `depth` rows per wave, as the decode kernel streams its packed units
//     nt           1: non-temporal hint on the loads
//     pattern      0: 1 KB rows dealt round-robin over all waves of the grid
//                  1: every workgroup reads one contiguous share, its waves interleaved row by row
//   returns 0, or -1 for a combination that is not built / a buffer that is not 1 KB-granular.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {

typedef unsigned int u4 __attribute__((ext_vector_type(4)));

struct Rows {
    size_t first, step, limit;      // 1 KB rows of this wave: first, first + step, ... below limit
};
__device__ __forceinline__ Rows rows_of_wave(size_t total_rows, int pattern) {
    const size_t nw = blockDim.x >> 6;
    const size_t wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    if (pattern == 0) return Rows{blockIdx.x * nw + wave, static_cast<size_t>(gridDim.x) * nw, total_rows};
    const size_t per_wg = (total_rows + gridDim.x - 1) / gridDim.x;
    const size_t lo = blockIdx.x * per_wg;
    const size_t hi = lo + per_wg < total_rows ? lo + per_wg : total_rows;
    return Rows{lo + wave, nw, hi};
}

template <bool NT>
__device__ __forceinline__ u4 ld16(const u4* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    return *p;
}

template <int DEPTH, bool NT>
__global__ __launch_bounds__(1024) void probe_regs(const u4* src, size_t total_rows, int pattern, unsigned int* sink) {
    const Rows R = rows_of_wave(total_rows, pattern);
    const u4* lane_src = src + (threadIdx.x & 63);
    u4 acc = {0, 0, 0, 0};
    size_t r = R.first;
    for (; r + (DEPTH - 1) * R.step < R.limit; r += DEPTH * R.step) {
        u4 x[DEPTH];
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) x[k] = ld16<NT>(lane_src + (r + k * R.step) * 64);
#pragma unroll
        for (int k = 0; k < DEPTH; ++k) acc ^= x[k];
    }
    for (; r < R.limit; r += R.step) acc ^= ld16<NT>(lane_src + r * 64);
    // never true for real data; keeps the loads alive
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink) *sink = acc[0];
}

template <bool NT>
__device__ __forceinline__ void dma_row(const uint8_t* row, uint32_t lane16, uint32_t lds_row) {
    if constexpr (NT) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     : : "v"(lane16), "s"(row), "s"(lds_row) : "memory", "m0");
    } else {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     : : "v"(lane16), "s"(row), "s"(lds_row) : "memory", "m0");
    }
}

template <int DEPTH, bool NT>
__global__ __launch_bounds__(1024) void probe_lds(const uint8_t* src, size_t total_rows, int pattern, unsigned int* sink) {
    extern __shared__ __attribute__((aligned(16))) uint8_t ring[];      // [waves][DEPTH] rows of 1 KB
    const Rows R = rows_of_wave(total_rows, pattern);
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const uint32_t lane16 = (threadIdx.x & 63) * 16;
    const uint32_t base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
                              (const __attribute__((address_space(3))) void*)ring)) + wave * DEPTH * 1024;
    int slot = 0, issued = 0;
    for (size_t r = R.first; r < R.limit; r += R.step) {
        if (issued >= DEPTH) asm volatile("s_waitcnt vmcnt(%0)" : : "n"(DEPTH - 1) : "memory");
        dma_row<NT>(src + r * 1024, lane16, __builtin_amdgcn_readfirstlane(base + slot * 1024));
        slot = slot + 1 == DEPTH ? 0 : slot + 1;
        ++issued;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (sink && total_rows == 0) *sink = ring[0];
}

template <int DEPTH, bool NT>
hipError_t launch_regs(const void* src, size_t rows, int grid, int block, int pattern, hipStream_t s) {
    hipLaunchKernelGGL((probe_regs<DEPTH, NT>), dim3(grid), dim3(block), 0, s, static_cast<const u4*>(src), rows, pattern,
                       static_cast<unsigned int*>(nullptr));
    return hipGetLastError();
}
template <int DEPTH, bool NT>
hipError_t launch_lds(const void* src, size_t rows, int grid, int block, int pattern, hipStream_t s) {
    const int lds = (block / 64) * DEPTH * 1024;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    static bool configured[64] = {};
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || !configured[dev]) {
        if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&probe_lds<DEPTH, NT>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            e != hipSuccess)
            return e;
        if (dev >= 0 && dev < 64) configured[dev] = true;
    }
    hipLaunchKernelGGL((probe_lds<DEPTH, NT>), dim3(grid), dim3(block), lds, s, static_cast<const uint8_t*>(src), rows, pattern,
                       static_cast<unsigned int*>(nullptr));
    return hipGetLastError();
}

template <bool NT>
hipError_t pick(const void* src, size_t rows, int grid, int block, int mode, int depth, int pattern, hipStream_t s) {
    if (mode == 0) {
        switch (depth) {
            case 2: return launch_regs<2, NT>(src, rows, grid, block, pattern, s);
            case 4: return launch_regs<4, NT>(src, rows, grid, block, pattern, s);
            case 8: return launch_regs<8, NT>(src, rows, grid, block, pattern, s);
            case 16: return launch_regs<16, NT>(src, rows, grid, block, pattern, s);
        }
    } else if (mode == 1) {
        switch (depth) {
            case 2: return launch_lds<2, NT>(src, rows, grid, block, pattern, s);
            case 4: return launch_lds<4, NT>(src, rows, grid, block, pattern, s);
            case 6: return launch_lds<6, NT>(src, rows, grid, block, pattern, s);
            case 8: return launch_lds<8, NT>(src, rows, grid, block, pattern, s);
            case 16: return launch_lds<16, NT>(src, rows, grid, block, pattern, s);
        }
    }
    return hipErrorInvalidValue;
}

}  // namespace

extern "C" int bitprobe_read(const void* src, size_t bytes, int grid, int block, int mode, int depth, int nt, int pattern,
                             void* stream) {
    if (!src || (reinterpret_cast<uintptr_t>(src) & 15u) || bytes % 1024 || grid <= 0 || block <= 0 || block % 64 ||
        block > 1024 || (pattern != 0 && pattern != 1))
        return -1;
    if (bytes == 0) return 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const hipError_t e = nt ? pick<true>(src, bytes / 1024, grid, block, mode, depth, pattern, s)
                            : pick<false>(src, bytes / 1024, grid, block, mode, depth, pattern, s);
    return e == hipSuccess ? 0 : -1;
}
