// Native test driver for the C ABI of libbitdecode.so: pack a K/V cache, decode one query token
// against it, and check the output -- no Python, no torch.  It plays the role of the reference's
// libtorch drivers (csrc/bit_decode/src/test_single_packdecode.cu:15-105 for one sequence,
// test_batch_packdecode.cu:16-170 for a batch): same flow (random fp16 Q/K/V with a fixed seed, pack,
// decode, compare with attention on the unquantized tensors under the reference's thresholds,
// mean-abs-err and mean-squared-err < 1e-1), plus the strict bar of this build: max-abs-err against
// dequantize-then-attend from the C restatement of the quantizer (oracle/liboracle_c.so, loaded with
// dlopen: test infrastructure, never linked into the product) must stay below 2e-3.
//
// usage: packdecode_driver <libbitdecode.so> <liboracle_c.so>
// exit status 0 = every case passed.  The same source also builds as a shared library whose
// packdecode_driver_run(lib, oracle) the Python test suite calls in-process (a GPU test must not
// start another program from a process that already uses the GPU).
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/bitdecode.h"

#define HIP_OK(x)                                                                         \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            std::exit(2);                                                                 \
        }                                                                                 \
    } while (0)

namespace {

// entry points of the library under test, bound at run time like a foreign-function binding would
struct Api {
    int (*abi_version)(void);
    const char* (*last_error)(void);
    int (*num_splits)(int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t);
    size_t (*workspace_bytes)(int32_t, int32_t, int32_t);
    int (*qpack)(const bitdecode_qpack_args*, void*);
    int (*fwd)(const bitdecode_fwd_args*, void*);
    int (*fwd_append)(const bitdecode_fwd_append_args*, void*);
    size_t (*fwd_append_workspace_bytes)(int32_t, int32_t, int32_t);
};
typedef void (*quantize_fn)(const float*, const float*, int, int, int, int, int, int, int, uint8_t*, float*, float*,
                            uint8_t*, float*, float*);
typedef void (*attend_fn)(const float*, const uint8_t*, const float*, const float*, const uint8_t*, const float*,
                          const float*, const float*, const float*, const int*, const int*, int, int, int, int, int,
                          int, int, float, float*, float*);
typedef float (*round_fn)(float);

template <class T>
T sym(void* h, const char* name) {
    void* p = dlsym(h, name);
    if (!p) {
        std::fprintf(stderr, "missing symbol %s\n", name);
        std::exit(2);
    }
    return reinterpret_cast<T>(p);
}

uint16_t f32_to_f16_bits(float f) {   // f is already representable in fp16
    _Float16 h = static_cast<_Float16>(f);
    uint16_t u;
    std::memcpy(&u, &h, 2);
    return u;
}
float f16_bits_to_f32(uint16_t u) {
    _Float16 h;
    std::memcpy(&h, &u, 2);
    return static_cast<float>(h);
}

template <class T>
T* to_device(const std::vector<T>& v) {
    T* d = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&d), v.size() * sizeof(T) + 16));
    HIP_OK(hipMemcpy(d, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

// softmax(q k^T * scale) v on the unquantized tensors, fp32 (the reference drivers' single_mha)
void plain_attention(const std::vector<float>& q, const std::vector<float>& k, const std::vector<float>& v, int b, int h,
                     int hk, int n, float scale, std::vector<float>& out) {
    const int d = 128, g = h / hk;
    std::vector<float> s(n);
    for (int bi = 0; bi < b; ++bi)
        for (int hq = 0; hq < h; ++hq) {
            const float* qp = &q[(static_cast<size_t>(bi) * h + hq) * d];
            const int kh = hq / g;
            float mx = -INFINITY;
            for (int t = 0; t < n; ++t) {
                const float* kp = &k[((static_cast<size_t>(bi) * n + t) * hk + kh) * d];
                float acc = 0.f;
                for (int c = 0; c < d; ++c) acc += qp[c] * kp[c];
                s[t] = acc * scale;
                mx = std::fmax(mx, s[t]);
            }
            double sum = 0;
            for (int t = 0; t < n; ++t) sum += (s[t] = std::exp(s[t] - mx));
            float* op = &out[(static_cast<size_t>(bi) * h + hq) * d];
            for (int c = 0; c < d; ++c) {
                double acc = 0;
                for (int t = 0; t < n; ++t) acc += s[t] * v[((static_cast<size_t>(bi) * n + t) * hk + kh) * d + c];
                op[c] = static_cast<float>(acc / sum);
            }
        }
}

struct Case {
    int b, h, hk, S, R, bits, gs;
};

bool run_case(const Api& api, quantize_fn quantize, attend_fn attend, round_fn round16, const Case& c) {
    const int d = 128, pn = 16 / c.bits, n = c.S + c.R;
    std::mt19937 rng(42);   // seed of test_single_packdecode.cu:19
    std::normal_distribution<float> gauss(0.f, 1.f);
    std::uniform_real_distribution<float> uni(0.f, 1.f);
    std::vector<float> q(static_cast<size_t>(c.b) * c.h * d), k(static_cast<size_t>(c.b) * n * c.hk * d), v(k.size());
    for (auto& x : q) x = round16(uni(rng));
    for (auto& x : k) x = round16(gauss(rng));
    for (auto& x : v) x = round16(gauss(rng));

    std::vector<uint16_t> qh(q.size()), kh(k.size()), vh(v.size());
    for (size_t i = 0; i < q.size(); ++i) qh[i] = f32_to_f16_bits(q[i]);
    for (size_t i = 0; i < k.size(); ++i) kh[i] = f32_to_f16_bits(k[i]);
    for (size_t i = 0; i < v.size(); ++i) vh[i] = f32_to_f16_bits(v[i]);
    uint16_t *dq = to_device(qh), *dk = to_device(kh), *dv = to_device(vh);

    // caller-allocated cache with the reference's shapes (test_single_packdecode.cu:33-43)
    const size_t pack_bytes = static_cast<size_t>(c.b) * c.S / pn * c.hk * d * 2;
    const size_t param_bytes = static_cast<size_t>(c.b) * c.S / c.gs * c.hk * d * 4;
    void *k_pack, *k_params, *v_pack, *v_params, *out;
    HIP_OK(hipMalloc(&k_pack, pack_bytes));
    HIP_OK(hipMalloc(&v_pack, pack_bytes));
    HIP_OK(hipMalloc(&k_params, param_bytes));
    HIP_OK(hipMalloc(&v_params, param_bytes));
    HIP_OK(hipMalloc(&out, static_cast<size_t>(c.b) * c.h * d * 2));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    bitdecode_qpack_args pa;
    std::memset(&pa, 0, sizeof pa);
    pa.k = dk;
    pa.v = dv;
    pa.k_stride_b = pa.v_stride_b = static_cast<int64_t>(n) * c.hk * d;
    pa.k_stride_t = pa.v_stride_t = static_cast<int64_t>(c.hk) * d;
    pa.k_stride_h = pa.v_stride_h = d;
    pa.k_pack = k_pack; pa.k_params = k_params; pa.v_pack = v_pack; pa.v_params = v_params;
    pa.b = c.b; pa.n_tokens = c.S; pa.h_k = c.hk; pa.d = d;
    pa.cache_tokens = c.S;
    pa.bits = c.bits; pa.group_size = c.gs; pa.dtype = BITDECODE_FP16;
    if (int rc = api.qpack(&pa, stream)) {
        std::fprintf(stderr, "bitdecode_qpack failed (%d): %s\n", rc, api.last_error());
        return false;
    }

    const float scale = 1.f / std::sqrt(static_cast<float>(d));
    bitdecode_fwd_args fa;
    std::memset(&fa, 0, sizeof fa);
    fa.q = dq; fa.q_stride_b = static_cast<int64_t>(c.h) * d; fa.q_stride_h = d;
    fa.k_pack = k_pack; fa.k_params = k_params; fa.v_pack = v_pack; fa.v_params = v_params;
    fa.cache_tokens = fa.seqlen_k = fa.max_seqlen_k = c.S;
    if (c.R) {
        fa.k_res = dk + static_cast<size_t>(c.S) * c.hk * d;      // the last R tokens stay fp16
        fa.v_res = dv + static_cast<size_t>(c.S) * c.hk * d;
        fa.kres_stride_b = fa.vres_stride_b = pa.k_stride_b;
        fa.kres_stride_t = fa.vres_stride_t = pa.k_stride_t;
        fa.kres_stride_h = fa.vres_stride_h = d;
        fa.res_len = fa.max_res_len = c.R;
    }
    fa.out = out; fa.out_stride_b = static_cast<int64_t>(c.h) * d; fa.out_stride_h = d;
    fa.b = c.b; fa.h = c.h; fa.h_k = c.hk; fa.d = d;
    fa.bits = c.bits; fa.group_size = c.gs; fa.dtype = BITDECODE_FP16;
    fa.softmax_scale = scale;
    fa.num_splits = api.num_splits(c.b, c.hk, c.S, c.R, 0, c.bits, c.gs);
    const size_t ws = api.workspace_bytes(c.b, c.h, fa.num_splits);
    void* workspace = nullptr;
    if (ws) {
        HIP_OK(hipMalloc(&workspace, ws));
        HIP_OK(hipMemsetAsync(workspace, 0, ws, stream));
        fa.workspace = workspace;
        fa.workspace_bytes = ws;
    }
    for (int rep = 0; rep < 2; ++rep) {        // twice: the workspace must come back reusable
        if (int rc = api.fwd(&fa, stream)) {
            std::fprintf(stderr, "bitdecode_fwd failed (%d): %s\n", rc, api.last_error());
            return false;
        }
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> oh(static_cast<size_t>(c.b) * c.h * d);
    HIP_OK(hipMemcpy(oh.data(), out, oh.size() * 2, hipMemcpyDeviceToHost));

    // checker 1: dequantize-then-attend from the C restatement (packed prefix contiguous per batch)
    std::vector<float> kp(static_cast<size_t>(c.b) * c.S * c.hk * d), vp(kp.size()), kr, vr;
    if (c.R) { kr.resize(static_cast<size_t>(c.b) * c.R * c.hk * d); vr.resize(kr.size()); }
    const size_t row = static_cast<size_t>(c.hk) * d;
    for (int bi = 0; bi < c.b; ++bi) {
        std::memcpy(&kp[bi * c.S * row], &k[static_cast<size_t>(bi) * n * row], c.S * row * 4);
        std::memcpy(&vp[bi * c.S * row], &v[static_cast<size_t>(bi) * n * row], c.S * row * 4);
        if (c.R) {
            std::memcpy(&kr[bi * c.R * row], &k[(static_cast<size_t>(bi) * n + c.S) * row], c.R * row * 4);
            std::memcpy(&vr[bi * c.R * row], &v[(static_cast<size_t>(bi) * n + c.S) * row], c.R * row * 4);
        }
    }
    std::vector<uint8_t> kc(kp.size()), vc(kp.size());
    std::vector<float> ks(kp.size() / c.gs), kz(ks.size()), vs(ks.size()), vz(ks.size());
    quantize(kp.data(), vp.data(), c.b, c.S, c.hk, d, c.bits, c.gs, 0, kc.data(), ks.data(), kz.data(), vc.data(),
             vs.data(), vz.data());
    std::vector<float> want(oh.size()), lse(static_cast<size_t>(c.b) * c.h), plain(oh.size());
    attend(q.data(), kc.data(), ks.data(), kz.data(), vc.data(), vs.data(), vz.data(), c.R ? kr.data() : nullptr,
           c.R ? vr.data() : nullptr, nullptr, nullptr, c.b, c.h, c.hk, d, c.S, c.R, c.gs, scale, want.data(),
           lse.data());
    // checker 2: the reference drivers' criterion against unquantized attention
    plain_attention(q, k, v, c.b, c.h, c.hk, n, scale, plain);

    double max_err = 0, mae = 0, mse = 0;
    for (size_t i = 0; i < oh.size(); ++i) {
        const float o = f16_bits_to_f32(oh[i]);
        max_err = std::fmax(max_err, std::fabs(o - want[i]));
        mae += std::fabs(o - plain[i]);
        mse += (o - plain[i]) * (o - plain[i]);
    }
    mae /= oh.size();
    mse /= oh.size();
    const bool ok = max_err < 2e-3 && mae < 1e-1 && mse < 1e-1;
    std::printf("b %d heads %d/%d packed %d + fp16 %d tokens, %d-bit g%d, %d splits: max|out - dequant-attend| %.2e, "
                "vs unquantized mae %.2e mse %.2e -> %s\n",
                c.b, c.h, c.hk, c.S, c.R, c.bits, c.gs, fa.num_splits, max_err, mae, mse, ok ? "pass" : "FAIL");
    std::fflush(stdout);

    for (void* p : {static_cast<void*>(dq), static_cast<void*>(dk), static_cast<void*>(dv), k_pack, k_params, v_pack,
                    v_params, out, workspace})
        if (p) HIP_OK(hipFree(p));
    HIP_OK(hipStreamDestroy(stream));
    return ok;
}

// A decode loop on the one-launch entry point: every sequence starts with `start` tokens (whole 128-token
// blocks packed with bitdecode_qpack, the rest copied into its fp16 window) and takes `steps` calls of
// bitdecode_fwd_append, each with a new token and a new query; lengths stay on the device.  Checked at the
// end: the length counters, and the last call's output against the C restatement on the token history
// (blocks that were packed -- by the pack call or inside a step -- read as codes, the rest as fp16).
bool run_step_case(const Api& api, quantize_fn quantize, attend_fn attend, round_fn round16, int b, int h, int hk,
                   int start, int steps, int bits, int gs) {
    const int d = 128, pn = 16 / bits, n = start + steps;
    const int cap = (n + 127) / 128 * 128;
    std::mt19937 rng(7);
    std::normal_distribution<float> gauss(0.f, 1.f);
    const size_t row = static_cast<size_t>(hk) * d;
    std::vector<float> q(static_cast<size_t>(steps) * b * h * d), k(static_cast<size_t>(b) * n * row), v(k.size());
    for (auto& x : q) x = round16(gauss(rng));
    for (auto& x : k) x = round16(gauss(rng));
    for (auto& x : v) x = round16(gauss(rng));
    std::vector<uint16_t> qh(q.size()), kh(k.size()), vh(v.size());
    for (size_t i = 0; i < q.size(); ++i) qh[i] = f32_to_f16_bits(q[i]);
    for (size_t i = 0; i < k.size(); ++i) kh[i] = f32_to_f16_bits(k[i]);
    for (size_t i = 0; i < v.size(); ++i) vh[i] = f32_to_f16_bits(v[i]);
    uint16_t *dq = to_device(qh), *dk = to_device(kh), *dv = to_device(vh);

    const size_t pack_bytes = static_cast<size_t>(b) * cap / pn * row * 2;
    const size_t param_bytes = static_cast<size_t>(b) * cap / gs * row * 4;
    const size_t win_bytes = static_cast<size_t>(b) * 128 * row * 2;
    void *k_pack, *k_params, *v_pack, *v_params, *out, *k_win, *v_win, *lengths, *workspace;
    HIP_OK(hipMalloc(&k_pack, pack_bytes));
    HIP_OK(hipMalloc(&v_pack, pack_bytes));
    HIP_OK(hipMalloc(&k_params, param_bytes));
    HIP_OK(hipMalloc(&v_params, param_bytes));
    HIP_OK(hipMalloc(&out, static_cast<size_t>(b) * h * d * 2));
    HIP_OK(hipMalloc(&k_win, win_bytes));
    HIP_OK(hipMalloc(&v_win, win_bytes));
    HIP_OK(hipMalloc(&lengths, b * sizeof(int32_t)));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    // prefill: whole blocks packed, the remainder into the window
    const int packed0 = start / 128 * 128, r0 = start - packed0;
    if (packed0) {
        bitdecode_qpack_args pa;
        std::memset(&pa, 0, sizeof pa);
        pa.k = dk; pa.v = dv;
        pa.k_stride_b = pa.v_stride_b = static_cast<int64_t>(n) * row;
        pa.k_stride_t = pa.v_stride_t = static_cast<int64_t>(row);
        pa.k_stride_h = pa.v_stride_h = d;
        pa.k_pack = k_pack; pa.k_params = k_params; pa.v_pack = v_pack; pa.v_params = v_params;
        pa.b = b; pa.n_tokens = packed0; pa.h_k = hk; pa.d = d;
        pa.cache_tokens = cap;
        pa.bits = bits; pa.group_size = gs; pa.dtype = BITDECODE_FP16;
        if (int rc = api.qpack(&pa, stream)) {
            std::fprintf(stderr, "bitdecode_qpack failed (%d): %s\n", rc, api.last_error());
            return false;
        }
    }
    for (int bi = 0; bi < b && r0; ++bi) {
        const size_t src = (static_cast<size_t>(bi) * n + packed0) * row, dst = static_cast<size_t>(bi) * 128 * row;
        HIP_OK(hipMemcpyAsync(static_cast<uint16_t*>(k_win) + dst, dk + src, r0 * row * 2, hipMemcpyDeviceToDevice, stream));
        HIP_OK(hipMemcpyAsync(static_cast<uint16_t*>(v_win) + dst, dv + src, r0 * row * 2, hipMemcpyDeviceToDevice, stream));
    }
    std::vector<int32_t> len0(b, start);
    HIP_OK(hipMemcpyAsync(lengths, len0.data(), b * sizeof(int32_t), hipMemcpyHostToDevice, stream));

    const float scale = 1.f / std::sqrt(static_cast<float>(d));
    bitdecode_fwd_append_args sa;
    std::memset(&sa, 0, sizeof sa);
    bitdecode_fwd_args& fa = sa.fwd;
    fa.q_stride_b = static_cast<int64_t>(h) * d; fa.q_stride_h = d;
    fa.k_pack = k_pack; fa.k_params = k_params; fa.v_pack = v_pack; fa.v_params = v_params;
    fa.cache_tokens = cap;
    fa.k_res = k_win; fa.v_res = v_win;
    fa.kres_stride_b = fa.vres_stride_b = 128 * static_cast<int64_t>(row);
    fa.kres_stride_t = fa.vres_stride_t = static_cast<int64_t>(row);
    fa.kres_stride_h = fa.vres_stride_h = d;
    fa.max_res_len = 128;                        // capacity of the window
    fa.out = out; fa.out_stride_b = static_cast<int64_t>(h) * d; fa.out_stride_h = d;
    fa.b = b; fa.h = h; fa.h_k = hk; fa.d = d;
    fa.bits = bits; fa.group_size = gs; fa.dtype = BITDECODE_FP16;
    fa.softmax_scale = scale;
    fa.num_splits = api.num_splits(b, hk, cap, 128, 0, bits, gs);   // one grid for every step
    const size_t ws = api.fwd_append_workspace_bytes(b, h, fa.num_splits);
    HIP_OK(hipMalloc(&workspace, ws));
    HIP_OK(hipMemsetAsync(workspace, 0, ws, stream));
    fa.workspace = workspace;
    fa.workspace_bytes = ws;
    sa.lengths = static_cast<int32_t*>(lengths);
    sa.knew_stride_b = sa.vnew_stride_b = static_cast<int64_t>(n) * row;
    sa.knew_stride_h = sa.vnew_stride_h = d;
    sa.max_len = cap + 127;
    for (int s = 0; s < steps; ++s) {
        fa.q = dq + static_cast<size_t>(s) * b * h * d;
        sa.k_new = dk + static_cast<size_t>(start + s) * row;     // token start + s of every sequence
        sa.v_new = dv + static_cast<size_t>(start + s) * row;
        if (int rc = api.fwd_append(&sa, stream)) {
            std::fprintf(stderr, "bitdecode_fwd_append failed (%d): %s\n", rc, api.last_error());
            return false;
        }
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> oh(static_cast<size_t>(b) * h * d);
    std::vector<int32_t> len1(b);
    HIP_OK(hipMemcpy(oh.data(), out, oh.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(len1.data(), lengths, b * sizeof(int32_t), hipMemcpyDeviceToHost));
    bool ok = true;
    for (int bi = 0; bi < b; ++bi) ok = ok && len1[bi] == n;

    // the last call saw n - 1 tokens plus its new one: blocks below `packed` as codes, the rest fp16
    const int packed = (n - 1) / 128 * 128, R = n - packed;
    std::vector<float> kp(static_cast<size_t>(b) * packed * row), vp(kp.size()), kr(static_cast<size_t>(b) * R * row), vr(kr.size());
    for (int bi = 0; bi < b; ++bi) {
        if (packed) {
            std::memcpy(&kp[static_cast<size_t>(bi) * packed * row], &k[static_cast<size_t>(bi) * n * row], packed * row * 4);
            std::memcpy(&vp[static_cast<size_t>(bi) * packed * row], &v[static_cast<size_t>(bi) * n * row], packed * row * 4);
        }
        std::memcpy(&kr[static_cast<size_t>(bi) * R * row], &k[(static_cast<size_t>(bi) * n + packed) * row], R * row * 4);
        std::memcpy(&vr[static_cast<size_t>(bi) * R * row], &v[(static_cast<size_t>(bi) * n + packed) * row], R * row * 4);
    }
    std::vector<uint8_t> kc(kp.size() + 1), vc(kp.size() + 1);
    std::vector<float> ks(kp.size() / gs + 1), kz(ks.size()), vs(ks.size()), vz(ks.size());
    if (packed)
        quantize(kp.data(), vp.data(), b, packed, hk, d, bits, gs, 0, kc.data(), ks.data(), kz.data(), vc.data(), vs.data(),
                 vz.data());
    std::vector<float> want(oh.size()), lse(static_cast<size_t>(b) * h);
    attend(&q[static_cast<size_t>(steps - 1) * b * h * d], kc.data(), ks.data(), kz.data(), vc.data(), vs.data(), vz.data(),
           kr.data(), vr.data(), nullptr, nullptr, b, h, hk, d, packed, R, gs, scale, want.data(), lse.data());
    double max_err = 0;
    for (size_t i = 0; i < oh.size(); ++i) max_err = std::fmax(max_err, std::fabs(f16_bits_to_f32(oh[i]) - want[i]));
    ok = ok && max_err < 2e-3;
    std::printf("decode loop, b %d heads %d/%d, %d tokens + %d steps of bitdecode_fwd_append, %d-bit g%d, %d splits: "
                "lengths %d, last step max|out - dequant-attend| %.2e -> %s\n",
                b, h, hk, start, steps, bits, gs, fa.num_splits, len1[0], max_err, ok ? "pass" : "FAIL");
    std::fflush(stdout);
    for (void* p : {static_cast<void*>(dq), static_cast<void*>(dk), static_cast<void*>(dv), k_pack, k_params, v_pack,
                    v_params, out, k_win, v_win, lengths, workspace})
        HIP_OK(hipFree(p));
    HIP_OK(hipStreamDestroy(stream));
    return ok;
}

}  // namespace

extern "C" int packdecode_driver_run(const char* lib_path, const char* oracle_path) {
    void* lib = dlopen(lib_path, RTLD_NOW | RTLD_LOCAL);
    void* ora = dlopen(oracle_path, RTLD_NOW | RTLD_LOCAL);
    if (!lib || !ora) {
        std::fprintf(stderr, "dlopen: %s\n", dlerror());
        return 2;
    }
    Api api;
    api.abi_version = sym<int (*)(void)>(lib, "bitdecode_abi_version");
    api.last_error = sym<const char* (*)(void)>(lib, "bitdecode_last_error");
    api.num_splits = sym<decltype(api.num_splits)>(lib, "bitdecode_num_splits");
    api.workspace_bytes = sym<decltype(api.workspace_bytes)>(lib, "bitdecode_fwd_workspace_bytes");
    api.qpack = sym<decltype(api.qpack)>(lib, "bitdecode_qpack");
    api.fwd = sym<decltype(api.fwd)>(lib, "bitdecode_fwd");
    api.fwd_append = sym<decltype(api.fwd_append)>(lib, "bitdecode_fwd_append");
    api.fwd_append_workspace_bytes = sym<decltype(api.fwd_append_workspace_bytes)>(lib, "bitdecode_fwd_append_workspace_bytes");
    if (api.abi_version() != BITDECODE_ABI_VERSION) {
        std::fprintf(stderr, "ABI version %d, header says %d\n", api.abi_version(), BITDECODE_ABI_VERSION);
        return 2;
    }
    quantize_fn quantize = sym<quantize_fn>(ora, "oracle_quantize_kv");
    attend_fn attend = sym<attend_fn>(ora, "oracle_attend");
    round_fn round16 = sym<round_fn>(ora, "oracle_round_fp16");

    // shapes of the reference drivers (one sequence, MHA and GQA, 2 and 4 bits, group 32 and 128;
    // a batch), scaled to what the scalar checker finishes in seconds, plus the fp16 window
    const Case cases[] = {
        {1, 32, 32, 1024, 0, 4, 128}, {1, 32, 8, 2048, 0, 4, 128},  {1, 32, 8, 2048, 0, 2, 128},
        {1, 32, 8, 1024, 0, 4, 32},   {1, 32, 8, 1024, 0, 2, 32},   {1, 32, 8, 4096, 128, 4, 128},
        {4, 32, 8, 1024, 100, 4, 128}, {2, 16, 2, 2048, 77, 2, 64},
    };
    int failed = 0;
    for (const Case& c : cases) failed += !run_case(api, quantize, attend, round16, c);
    // decode loops across a window that fills (once, and twice with an empty start)
    failed += !run_step_case(api, quantize, attend, round16, 2, 32, 8, 1024 + 100, 40, 4, 128);
    failed += !run_step_case(api, quantize, attend, round16, 1, 16, 2, 0, 260, 2, 64);
    std::printf("%d case(s) failed\n", failed);
    std::fflush(stdout);
    return failed ? 1 : 0;
}

#ifndef PACKDECODE_DRIVER_AS_LIBRARY
int main(int argc, char** argv) {
    if (argc != 3) {
        std::fprintf(stderr, "usage: %s <libbitdecode.so> <liboracle_c.so>\n", argv[0]);
        return 2;
    }
    return packdecode_driver_run(argv[1], argv[2]);
}
#endif
