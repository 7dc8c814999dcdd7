// A caller of libelectrock_moe.so that is not Python: plain C++ over the HIP runtime, the way a compiled serving
// engine would bind the layer (include/electrock_moe.h, nothing else).  It runs one MoE layer call per batch size
// on small shapes, restates the layer in float on the host (router of fused_moe.py:130-164 with ties to the lowest
// index, expert MLP of models/modeling_mixtral.py:632-670) and compares:
//   * topk_ids left in the workspace: equal to the host's,
//   * num_tokens_post_pad: the sum over experts of the row counts rounded up to the block size,
//   * the fp32 output of the default mode: max-abs <= 2e-2 and mean relative error <= 1e-3.
// Exit status 0 and a last line "host_check ok" on success.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/electrock_moe.h"

#define HIP_OK(call)                                                                          \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            std::printf("%s failed: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__); \
            return 1;                                                                         \
        }                                                                                     \
    } while (0)

namespace {

uint16_t to_bf16(float f) {  // round to nearest even
    uint32_t b;
    std::memcpy(&b, &f, 4);
    return static_cast<uint16_t>((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}
float from_bf16(uint16_t h) {
    const uint32_t b = static_cast<uint32_t>(h) << 16;
    float f;
    std::memcpy(&f, &b, 4);
    return f;
}

struct Lcg {  // small deterministic generator: uniform in [-1, 1)
    uint64_t s;
    float next() {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        return static_cast<float>(static_cast<int32_t>(s >> 32)) * (1.0f / 2147483648.0f);
    }
};

void fill(std::vector<uint16_t>& v, Lcg& g, float scale) {
    for (auto& e : v) e = to_bf16(scale * g.next());
}

int run_case(int64_t T, int H, int I, int E, int k) {
    std::printf("host_check: T=%lld H=%d I=%d E=%d top-%d\n", static_cast<long long>(T), H, I, E, k);
    std::fflush(stdout);
    Lcg g{static_cast<uint64_t>(T) * 977 + H};
    std::vector<uint16_t> x(T * H), w13(static_cast<size_t>(E) * 2 * I * H), w2(static_cast<size_t>(E) * H * I);
    std::vector<float> logits(T * E);
    fill(x, g, 1.7f);
    fill(w13, g, 0.035f);
    fill(w2, g, 0.035f);
    for (auto& l : logits) l = 2.0f * g.next();

    em_moe_layout L;
    if (em_moe_workspace_layout(T, H, I, E, k, EM_FLAG_OUT_F32, &L) != 0) return 1;
    const size_t ws_bytes = em_moe_workspace_bytes(T, H, I, E, k, EM_FLAG_OUT_F32);
    if (ws_bytes != static_cast<size_t>(L.total_bytes)) return 1;

    void *dx, *dw13, *dw2, *dl, *dout, *dws;
    HIP_OK(hipMalloc(&dx, x.size() * 2));
    HIP_OK(hipMalloc(&dw13, w13.size() * 2));
    HIP_OK(hipMalloc(&dw2, w2.size() * 2));
    HIP_OK(hipMalloc(&dl, logits.size() * 4));
    HIP_OK(hipMalloc(&dout, static_cast<size_t>(T) * H * 4));
    HIP_OK(hipMalloc(&dws, ws_bytes));
    HIP_OK(hipMemcpy(dx, x.data(), x.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dw13, w13.data(), w13.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dw2, w2.data(), w2.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dl, logits.data(), logits.size() * 4, hipMemcpyHostToDevice));

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    const int rc = em_moe_forward(dx, dl, EM_DTYPE_F32, dw13, dw2, dout, T, H, I, E, k, 1, dws, ws_bytes,
                                  EM_FLAG_OUT_F32, stream);
    if (rc != 0) {
        std::printf("em_moe_forward: %s\n", em_error_string(rc));
        return 1;
    }
    HIP_OK(hipStreamSynchronize(stream));

    std::vector<float> out(T * H);
    std::vector<int32_t> ids(T * k);
    int32_t post_pad = -1;
    HIP_OK(hipMemcpy(out.data(), dout, out.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(ids.data(), static_cast<char*>(dws) + L.topk_ids_off, ids.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(&post_pad, static_cast<char*>(dws) + L.post_pad_off, 4, hipMemcpyDeviceToHost));
    int32_t saturated = -1;  // activations clamped to the fp16 range: none with these operands
    HIP_OK(hipMemcpy(&saturated, static_cast<char*>(dws) + L.saturated_off, 4, hipMemcpyDeviceToHost));
    if (saturated != 0) {
        std::printf("saturated counter reads %d, expected 0\n", saturated);
        return 1;
    }

    // ---- the layer on the host, in float ----
    std::vector<float> ref(T * H, 0.0f), act(I);
    std::vector<int64_t> rows_of(E, 0);
    double sum_abs_ref = 0, sum_abs_err = 0, max_err = 0;
    for (int64_t t = 0; t < T; ++t) {
        const float* l = &logits[t * E];
        float mx = l[0];
        for (int e = 1; e < E; ++e) mx = std::fmax(mx, l[e]);
        float den = 0;
        for (int e = 0; e < E; ++e) den += std::exp(l[e] - mx);
        std::vector<bool> taken(E, false);
        std::vector<int> sel(k);
        float wsum = 0;
        for (int j = 0; j < k; ++j) {
            int best = -1;
            for (int e = 0; e < E; ++e)  // strict '>': a tie keeps the lower index
                if (!taken[e] && (best < 0 || l[e] > l[best])) best = e;
            taken[best] = true;
            sel[j] = best;
            wsum += std::exp(l[best] - mx) / den;
            if (ids[t * k + j] != best) {
                std::printf("topk_ids[%lld][%d] = %d, host says %d\n", static_cast<long long>(t), j, ids[t * k + j], best);
                return 1;
            }
        }
        for (int j = 0; j < k; ++j) {
            const int e = sel[j];
            ++rows_of[e];
            const float wgt = std::exp(l[e] - mx) / den / wsum;
            const uint16_t* wg = &w13[static_cast<size_t>(e) * 2 * I * H];
            const uint16_t* wu = wg + static_cast<size_t>(I) * H;
            for (int i = 0; i < I; ++i) {
                float gs = 0, us = 0;
                for (int h = 0; h < H; ++h) {
                    const float xv = from_bf16(x[t * H + h]);
                    gs += xv * from_bf16(wg[static_cast<size_t>(i) * H + h]);
                    us += xv * from_bf16(wu[static_cast<size_t>(i) * H + h]);
                }
                act[i] = gs / (1.0f + std::exp(-gs)) * us;
            }
            const uint16_t* wd = &w2[static_cast<size_t>(e) * H * I];
            for (int h = 0; h < H; ++h) {
                float s = 0;
                for (int i = 0; i < I; ++i) s += act[i] * from_bf16(wd[static_cast<size_t>(h) * I + i]);
                ref[t * H + h] += wgt * s;
            }
        }
    }
    int64_t padded = 0;
    for (int e = 0; e < E; ++e) padded += (rows_of[e] + L.block_size - 1) / L.block_size * L.block_size;
    if (post_pad != padded) {
        std::printf("num_tokens_post_pad = %d, host says %lld\n", post_pad, static_cast<long long>(padded));
        return 1;
    }
    for (size_t i = 0; i < ref.size(); ++i) {
        const double d = std::fabs(static_cast<double>(out[i]) - ref[i]);
        sum_abs_err += d;
        sum_abs_ref += std::fabs(ref[i]);
        max_err = d > max_err ? d : max_err;
    }
    const double mean_rel = sum_abs_err / sum_abs_ref;
    std::printf("  block %lld, ksplit %lld, padded rows %d; max-abs %.3e mean-rel %.3e\n",
                static_cast<long long>(L.block_size), static_cast<long long>(L.ksplit), post_pad, max_err, mean_rel);
    if (!(max_err <= 2e-2) || !(mean_rel <= 1e-3)) {
        std::printf("output outside the tolerance\n");
        return 1;
    }
    HIP_OK(hipStreamDestroy(stream));
    HIP_OK(hipFree(dx));
    HIP_OK(hipFree(dw13));
    HIP_OK(hipFree(dw2));
    HIP_OK(hipFree(dl));
    HIP_OK(hipFree(dout));
    HIP_OK(hipFree(dws));
    return 0;
}

}  // namespace

int main() {
    std::printf("libelectrock_moe version %d\n", em_version());
    // streaming kernels, 64- / 128-row tiles, 256-row tiles, and a shape only the generic kernels take
    const int64_t batches[] = {3, 40, 150, 400, 700};
    for (int64_t T : batches)
        if (run_case(T, 256, 512, 8, 2) != 0) return 1;
    if (run_case(33, 136, 200, 4, 2) != 0) return 1;
    std::printf("host_check ok\n");
    return 0;
}
