// Times the C++ attention layer (include/sentinel_hip/HipCausalSelfAttention.hpp) forward and backward with flash
// attention on and off, the way the reference's train profile fills its "attention fwd/bwd ms" bucket
// (sentinel/NeuralNet/Cuda/CudaLanguageModel.cu:4259-4263, :4306-4315, printed at :4378): device events around
// attention.forward(input, attended, sequenceLength) and attention.backward(gradient, inputGradient, four weight
// gradients), averaged over the timed steps.  Shapes are the reference's flash-parity ones (main.cpp:640-643:
// (E, H, T) = (768,12,128), (768,12,256), (768,12,1024)), packed to `columns` tokens per step like its packed batches.
// A third timing has the projection products in mixed precision as well (HipAmp::preferMixedPrecision, fp16 operands,
// the reference's CudaAmp::preferMixedPrecision); the weights' 16-bit copies are kept across steps, as between two
// optimizer steps.
//
//   bench_layer [columns=4096] [steps=20] [warmup=3] [only=all|flash|dense|flash_mixed_projections] [seq_len=0]
// (`only`: time one of the three configurations, `seq_len`: one of the three shapes; e.g. under a profiler)
// prints one JSON object on stdout; bench.py --layer-path runs it and puts that object into its line.
#include "../../include/sentinel_hip/HipCausalSelfAttention.hpp"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

using namespace sentinel_hip_host;

static std::vector<float> lcg(size_t count, unsigned& state, float scale) {
    std::vector<float> out(count);
    for (size_t i = 0; i < count; ++i) {
        state = state * 1664525u + 1013904223u;
        out[i] = ((static_cast<float>(state >> 8) / 16777216.0f) * 2.0f - 1.0f) * scale;
    }
    return out;
}

struct Timing {
    float forwardMs = 0.0f;
    float backwardMs = 0.0f;
};

static Timing timeLayer(int e, int heads, int T, int packs, bool preferFlash, bool mixedProjections, int steps, int warmup) {
    const int d = e / heads, cols = packs * T;
    unsigned state = 271u;
    const float bound = 1.0f / std::sqrt(static_cast<float>(e));
    HostAttentionWeights host;
    host.queryWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.keyWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.valueWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.outputWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.embeddingDim = e;
    host.headCount = heads;
    host.kvHeadCount = heads;
    host.headDimension = d;
    host.maximumPositionCount = T;
    HipAmp::preferMixedPrecision() = mixedProjections;
    const unsigned long long mixedBefore = HipAmp::mixedProductCount();
    HipCausalSelfAttention layer = HipCausalSelfAttention::createFrom(host);
    layer.preferFlashAttention = preferFlash;

    HipMatrix input, gradient, out, inputGradient, dWq, dWk, dWv, dWo;
    input.upload(lcg(static_cast<size_t>(e) * cols, state, 1.0f), e, cols);
    gradient.upload(lcg(static_cast<size_t>(e) * cols, state, 1.0f), e, cols);

    hipEvent_t marks[3];
    for (hipEvent_t& m : marks) throwIfHipFailed(hipEventCreate(&m), "hipEventCreate");
    const hipStream_t stream = HipFlashAttention::activeStream();
    Timing sum;
    for (int step = 0; step < warmup + steps; ++step) {
        throwIfHipFailed(hipEventRecord(marks[0], stream), "hipEventRecord");
        layer.forward(input, out, T);
        throwIfHipFailed(hipEventRecord(marks[1], stream), "hipEventRecord");
        layer.backward(gradient, inputGradient, dWq, dWk, dWv, dWo);
        throwIfHipFailed(hipEventRecord(marks[2], stream), "hipEventRecord");
        throwIfHipFailed(hipEventSynchronize(marks[2]), "hipEventSynchronize");
        if (layer.usedFlashAttention != preferFlash) throw std::logic_error("bench_layer: unexpected attention path");
        if (step < warmup) continue;
        float f = 0.0f, b = 0.0f;
        throwIfHipFailed(hipEventElapsedTime(&f, marks[0], marks[1]), "hipEventElapsedTime");
        throwIfHipFailed(hipEventElapsedTime(&b, marks[1], marks[2]), "hipEventElapsedTime");
        sum.forwardMs += f;
        sum.backwardMs += b;
    }
    for (hipEvent_t& m : marks) throwIfHipFailed(hipEventDestroy(m), "hipEventDestroy");
    HipAmp::preferMixedPrecision() = false;
    if ((HipAmp::mixedProductCount() != mixedBefore) != mixedProjections)
        throw std::logic_error("bench_layer: unexpected projection arithmetic");
    sum.forwardMs /= static_cast<float>(steps);
    sum.backwardMs /= static_cast<float>(steps);
    return sum;
}

int main(int argc, char** argv) {
    const int columns = argc > 1 ? std::atoi(argv[1]) : 4096;
    const int steps = argc > 2 ? std::atoi(argv[2]) : 20;
    const int warmup = argc > 3 ? std::atoi(argv[3]) : 3;
    const std::string only = argc > 4 ? argv[4] : "all";
    const int onlyLength = argc > 5 ? std::atoi(argv[5]) : 0;
    if (columns <= 0 || steps <= 0 || warmup < 0 ||
        (only != "all" && only != "flash" && only != "dense" && only != "flash_mixed_projections")) {
        std::fprintf(stderr, "usage: bench_layer [columns] [steps] [warmup] [all|flash|dense|flash_mixed_projections]\n");
        return 2;
    }
    try {
        HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_BF16;
        const int shapes[3][3] = {{768, 12, 128}, {768, 12, 256}, {768, 12, 1024}};
        std::string json = "{\"compute\": \"bf16 attention arithmetic; projections fp32 (rocBLAS sgemm) in flash / dense, fp16 operands with "
                           "fp32 accumulation (rocblas_gemm_ex) in flash_mixed_projections\", \"columns_per_step\": " +
                           std::to_string(columns) + ", \"steps\": " + std::to_string(steps) + ", \"shapes\": [";
        bool first = true;
        for (int i = 0; i < 3; ++i) {
            const int e = shapes[i][0], heads = shapes[i][1], T = shapes[i][2];
            if (onlyLength > 0 && T != onlyLength) continue;
            const int packs = columns / T > 0 ? columns / T : 1;
            char row[768];
            int at = std::snprintf(row, sizeof row, "%s{\"embedding_dim\": %d, \"heads\": %d, \"seq_len\": %d, \"packs\": %d",
                                   first ? "" : ", ", e, heads, T, packs);
            first = false;
            const char* names[3] = {"flash", "dense", "flash_mixed_projections"};
            for (int mode = 0; mode < 3; ++mode) {
                if (only != "all" && only != names[mode]) continue;
                const Timing t = timeLayer(e, heads, T, packs, mode != 1, mode == 2, steps, warmup);
                at += std::snprintf(row + at, sizeof row - at,
                                    ", \"%s\": {\"attention_fwd_ms\": %.4f, \"attention_bwd_ms\": %.4f}, \"tokens_per_s_%s\": %.0f",
                                    names[mode], t.forwardMs, t.backwardMs, names[mode],
                                    packs * T / ((t.forwardMs + t.backwardMs) * 1e-3));
            }
            std::snprintf(row + at, sizeof row - at, "}");
            json += row;
        }
        json += "]}";
        std::printf("%s\n", json.c_str());
    } catch (const std::exception& ex) {
        std::fprintf(stderr, "bench_layer: %s\n", ex.what());
        return 1;
    }
    return 0;
}
