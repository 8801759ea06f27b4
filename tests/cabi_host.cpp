// A host program without torch or Python: it binds the C ABI the way any C or C++ caller would
// (include/aicomp_kv.h, link libaicomp_kv.so), runs a fused append + decode step on a small bf16
// problem and checks the result against double-precision attention computed on the host.
// Built by aicomp_amd/build.py; run by tests/test_gpu_cabi_host.py.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "aicomp_kv.h"

#define HIP_OK(x)                                                                    \
    do {                                                                             \
        hipError_t e__ = (x);                                                        \
        if (e__ != hipSuccess) {                                                     \
            std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e__), __FILE__, __LINE__); \
            return 2;                                                                \
        }                                                                            \
    } while (0)

static uint16_t f32_to_bf16(float f) {           // round to nearest even
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float bf16_to_f32(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
static float lcg(uint32_t& s) {                  // uniform in [-1, 1)
    s = s * 1664525u + 1013904223u;
    return (float)((s >> 8) & 0xffff) / 32768.f - 1.f;
}

int main() {
    const int B = 3, Hq = 8, Hkv = 2, D = 128, BS = 16, G = Hq / Hkv;
    const int ctx[B] = {1, 37, 300};             // lengths including the token appended by this step
    const int max_blocks = (300 + BS - 1) / BS;
    const int num_blocks = B * max_blocks + 1;
    uint32_t seed = 12345u;

    std::vector<uint16_t> k_pool((size_t)num_blocks * Hkv * BS * D), v_pool(k_pool.size());
    for (auto& x : k_pool) x = f32_to_bf16(lcg(seed) * 0.7f);
    for (auto& x : v_pool) x = f32_to_bf16(lcg(seed) * 0.7f);
    std::vector<int32_t> table((size_t)B * max_blocks);
    for (int b = 0; b < B; ++b)                  // blocks dealt out in reverse, so the table is not the identity
        for (int j = 0; j < max_blocks; ++j) table[(size_t)b * max_blocks + j] = num_blocks - 1 - (b * max_blocks + j);
    std::vector<uint16_t> q((size_t)B * Hq * D), nk((size_t)B * Hkv * D), nv(nk.size());
    for (auto& x : q) x = f32_to_bf16(lcg(seed));
    for (auto& x : nk) x = f32_to_bf16(lcg(seed) * 0.7f);
    for (auto& x : nv) x = f32_to_bf16(lcg(seed) * 0.7f);
    const float scale = 1.f / std::sqrt((float)D);

    // expected: the new row takes slot ctx-1, then softmax(q K^T scale) V over ctx tokens, in double
    std::vector<uint16_t> k_ref = k_pool, v_ref = v_pool;
    auto slot_of = [&](int b, int t) { return (size_t)table[(size_t)b * max_blocks + t / BS] * BS + t % BS; };
    auto at = [&](size_t slot, int h) { return ((slot / BS) * Hkv + h) * BS * D + (slot % BS) * D; };
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < Hkv; ++h)
            for (int d = 0; d < D; ++d) {
                k_ref[at(slot_of(b, ctx[b] - 1), h) + d] = nk[((size_t)b * Hkv + h) * D + d];
                v_ref[at(slot_of(b, ctx[b] - 1), h) + d] = nv[((size_t)b * Hkv + h) * D + d];
            }
    std::vector<double> want((size_t)B * Hq * D, 0.0);
    for (int b = 0; b < B; ++b)
        for (int h = 0; h < Hq; ++h) {
            std::vector<double> s(ctx[b]);
            double mx = -1e300;
            for (int t = 0; t < ctx[b]; ++t) {
                double dot = 0;
                for (int d = 0; d < D; ++d)
                    dot += (double)bf16_to_f32(q[((size_t)b * Hq + h) * D + d]) *
                           bf16_to_f32(k_ref[at(slot_of(b, t), h / G) + d]);
                s[t] = dot * scale;
                mx = std::fmax(mx, s[t]);
            }
            double den = 0;
            for (int t = 0; t < ctx[b]; ++t) { s[t] = std::exp(s[t] - mx); den += s[t]; }
            for (int t = 0; t < ctx[b]; ++t)
                for (int d = 0; d < D; ++d)
                    want[((size_t)b * Hq + h) * D + d] += s[t] / den * bf16_to_f32(v_ref[at(slot_of(b, t), h / G) + d]);
        }

    void *d_k, *d_v, *d_q, *d_out, *d_nk, *d_nv, *d_table, *d_ctx, *d_ws = nullptr;
    HIP_OK(hipMalloc(&d_k, k_pool.size() * 2));
    HIP_OK(hipMalloc(&d_v, v_pool.size() * 2));
    HIP_OK(hipMalloc(&d_q, q.size() * 2));
    HIP_OK(hipMalloc(&d_out, q.size() * 2));
    HIP_OK(hipMalloc(&d_nk, nk.size() * 2));
    HIP_OK(hipMalloc(&d_nv, nv.size() * 2));
    HIP_OK(hipMalloc(&d_table, table.size() * 4));
    HIP_OK(hipMalloc(&d_ctx, sizeof(ctx)));
    HIP_OK(hipMemcpy(d_k, k_pool.data(), k_pool.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_v, v_pool.data(), v_pool.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_q, q.data(), q.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_nk, nk.data(), nk.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_nv, nv.data(), nv.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_table, table.data(), table.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d_ctx, ctx, sizeof(ctx), hipMemcpyHostToDevice));
    const size_t need = aicomp_paged_decode_workspace_bytes(B, Hq, Hkv, D, BS, max_blocks, AICOMP_KV_BF16,
                                                            AICOMP_KV_BF16, 0);
    if (need) HIP_OK(hipMalloc(&d_ws, need));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));

    const int rc = aicomp_paged_decode_attn_append(d_out, d_q, d_nk, d_nv, (int64_t)Hkv * D, D, d_k, d_v,
                                                   (const int32_t*)d_table, max_blocks, (const int32_t*)d_ctx, B,
                                                   Hq, Hkv, D, BS, max_blocks, num_blocks, scale, AICOMP_KV_BF16,
                                                   AICOMP_KV_BF16, nullptr, nullptr, 0, d_ws, need, stream);
    if (rc != AICOMP_KV_OK) {
        std::printf("aicomp_paged_decode_attn_append failed: %d %s\n", rc, aicomp_kv_last_error());
        return 1;
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<uint16_t> out(q.size()), k_got(k_pool.size()), v_got(v_pool.size());
    HIP_OK(hipMemcpy(out.data(), d_out, out.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(k_got.data(), d_k, k_got.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(v_got.data(), d_v, v_got.size() * 2, hipMemcpyDeviceToHost));
    if (k_got != k_ref || v_got != v_ref) {
        std::printf("pools differ from the expected append\n");
        return 1;
    }
    double worst = 0;
    for (size_t i = 0; i < out.size(); ++i) worst = std::fmax(worst, std::fabs(bf16_to_f32(out[i]) - want[i]));
    // an argument error must come back as a code and a message, not as a launch
    const int bad = aicomp_paged_decode_attn(d_out, d_q, d_k, d_v, (const int32_t*)d_table, max_blocks,
                                             (const int32_t*)d_ctx, B, Hq, 3, D, BS, max_blocks, num_blocks, scale,
                                             AICOMP_KV_BF16, AICOMP_KV_BF16, nullptr, nullptr, 0, d_ws, need, stream);
    std::printf("library %d, append bit-exact, decode max abs err %.3e, bad call -> %d (%s)\n",
                aicomp_kv_version(), worst, bad, aicomp_kv_last_error());
    return (worst <= 1e-2 && bad == AICOMP_KV_EINVAL) ? 0 : 1;
}
