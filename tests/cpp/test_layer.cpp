// GPU test of the C++ attention layer (include/sentinel_hip/HipCausalSelfAttention.hpp) against the CPU oracle's
// layer (training step and prefill / decode generation), on the shapes of the reference's own device smoke tests (CudaCausalSelfAttention::runFlashParitySmokeDemo:
// E=64, H=4, T=48; runGqaCudaSmokeDemo: grouped heads) plus packed batches and head_dim 64 / 128 with MFMA arithmetic.
// With preferFlashAttention = false the same cases run on the dense materialising path, and flash and dense are compared
// with each other on the shapes of the reference's flash parity runs (main.cpp:640-643: (E, H, T) = (64,4,48), (768,12,128),
// (768,12,256)). Multi-head cases (kvHeads == heads) run with the stacked QKV weights.
// Test infrastructure: the oracle is linked here only as the checker.
#include "../../include/sentinel_hip/HipCausalSelfAttention.hpp"
#include "../../oracle/sentinel_attention_oracle.h"

#include <cmath>
#include <cstdio>
#include <stdexcept>
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

static float relErr(const std::vector<float>& got, const std::vector<float>& want) {
    float err = 0.0f, top = 0.0f;
    for (size_t i = 0; i < got.size(); ++i) {
        err = std::max(err, std::fabs(got[i] - want[i]));
        top = std::max(top, std::fabs(want[i]));
    }
    return err / std::max(top, 1e-30f);
}

template <typename Fn>
static void expectThrow(const char* what, Fn fn) {
    try {
        fn();
    } catch (const std::exception&) {
        return;
    }
    throw std::runtime_error(std::string("expected an exception: ") + what);
}

static void runCase(const char* name, int e, int heads, int kvHeads, int d, int T, int packs, int compute, float tol,
                    int windowSize = 0, int globalTokenCount = 0, bool preferFlash = true) {
    const int qRows = heads * d, kvRows = kvHeads * d, cols = packs * T;
    unsigned state = 2024u + static_cast<unsigned>(e + T);
    const float bound = 1.0f / std::sqrt(static_cast<float>(e));
    HostAttentionWeights host;
    host.queryWeight = lcg(static_cast<size_t>(qRows) * e, state, bound);
    host.keyWeight = lcg(static_cast<size_t>(kvRows) * e, state, bound);
    host.valueWeight = lcg(static_cast<size_t>(kvRows) * e, state, bound);
    host.outputWeight = lcg(static_cast<size_t>(e) * qRows, state, bound);
    host.embeddingDim = e;
    host.headCount = heads;
    host.kvHeadCount = kvHeads;
    host.headDimension = d;
    host.maximumPositionCount = T + 5;
    host.windowSize = windowSize;
    host.globalTokenCount = globalTokenCount;
    auto hx = lcg(static_cast<size_t>(e) * cols, state, 1.0f);
    auto hg = lcg(static_cast<size_t>(e) * cols, state, 1.0f);

    // oracle: one sequence at a time, weight gradients summed over the batch (what the train loop accumulates)
    std::vector<float> wy(hx.size()), wdx(hx.size()), wdq(host.queryWeight.size(), 0.0f), wdk(host.keyWeight.size(), 0.0f),
        wdv(host.valueWeight.size(), 0.0f), wdo(host.outputWeight.size(), 0.0f);
    for (int p = 0; p < packs; ++p) {
        std::vector<float> x(static_cast<size_t>(e) * T), g(x.size()), y(x.size()), dx(x.size()), dq(wdq.size()), dk(wdk.size()),
            dv(wdv.size()), dwo(wdo.size());
        for (int r = 0; r < e; ++r)
            for (int c = 0; c < T; ++c) {
                x[static_cast<size_t>(r) * T + c] = hx[static_cast<size_t>(r) * cols + p * T + c];
                g[static_cast<size_t>(r) * T + c] = hg[static_cast<size_t>(r) * cols + p * T + c];
            }
        if (sentinel_oracle_layer_sparse(x.data(), host.queryWeight.data(), host.keyWeight.data(), host.valueWeight.data(),
                                         host.outputWeight.data(), g.data(), y.data(), dx.data(), dq.data(), dk.data(),
                                         dv.data(), dwo.data(), e, heads, kvHeads, d, T, host.ropeBase,
                                         host.maximumPositionCount, windowSize, globalTokenCount) != 0)
            throw std::runtime_error("oracle layer failed");
        for (int r = 0; r < e; ++r)
            for (int c = 0; c < T; ++c) {
                wy[static_cast<size_t>(r) * cols + p * T + c] = y[static_cast<size_t>(r) * T + c];
                wdx[static_cast<size_t>(r) * cols + p * T + c] = dx[static_cast<size_t>(r) * T + c];
            }
        for (size_t i = 0; i < wdq.size(); ++i) wdq[i] += dq[i];
        for (size_t i = 0; i < wdk.size(); ++i) wdk[i] += dk[i];
        for (size_t i = 0; i < wdv.size(); ++i) wdv[i] += dv[i];
        for (size_t i = 0; i < wdo.size(); ++i) wdo[i] += dwo[i];
    }

    HipFlashAttention::computeType() = compute;
    HipCausalSelfAttention layer = HipCausalSelfAttention::createFrom(host);
    layer.preferFlashAttention = preferFlash;
    if (layer.usesFusedQkv() != (heads == kvHeads) || layer.qkvWeight.empty() == (heads == kvHeads))
        throw std::runtime_error("stacked QKV weights must exist exactly for multi-head layers");
    HipMatrix x, g, y, dx, dwq, dwk, dwv, dwo;
    x.upload(hx, e, cols);
    g.upload(hg, e, cols);
    layer.forward(x, y, T);
    layer.backward(g, dx, dwq, dwk, dwv, dwo);
    const float ey = relErr(y.download(), wy), ex = relErr(dx.download(), wdx), eq = relErr(dwq.download(), wdq),
                ek = relErr(dwk.download(), wdk), ev = relErr(dwv.download(), wdv), eo = relErr(dwo.download(), wdo);
    std::printf("  %-40s  Y=%.2e dX=%.2e dWq=%.2e dWk=%.2e dWv=%.2e dWo=%.2e\n", name, ey, ex, eq, ek, ev, eo);
    if (ey > tol || ex > tol || eq > tol || ek > tol || ev > tol || eo > tol) throw std::runtime_error(std::string(name) + " parity failed");
    if (layer.usedFlashAttention != preferFlash || layer.activePackCount != packs || layer.activeSegmentLength != T)
        throw std::runtime_error("layer bookkeeping");
    if (compute != SENTINEL_HIP_COMPUTE_AUTO && preferFlash) {
        // MFMA arithmetic: the backward call above used the 16-bit operands the forward call left behind; converting
        // them again instead (keepFlashOperands = false) runs the same kernels on the same values
        if (!layer.flashOperands.filled) throw std::runtime_error(std::string(name) + " forward did not keep its 16-bit operands");
        const std::vector<float> keptDx = dx.download(), keptDwq = dwq.download(), keptDwk = dwk.download(), keptDwv = dwv.download();
        layer.keepFlashOperands = false;
        HipMatrix y2, dx2, a, b, c, o2;
        layer.forward(x, y2, T);
        layer.backward(g, dx2, a, b, c, o2);
        if (dx2.download() != keptDx || a.download() != keptDwq || b.download() != keptDwk || c.download() != keptDwv)
            throw std::runtime_error(std::string(name) + " kept 16-bit operands changed the gradients");
        layer.keepFlashOperands = true;
        layer.forward(x, y2, T);  // leave the layer as the checks below expect it: operands kept
    } else if (layer.flashOperands.filled) {
        throw std::runtime_error(std::string(name) + " exact fp32 arithmetic keeps no 16-bit operands");
    }
    if (heads == kvHeads) {
        // the stacked weight gradient alone (materializeSplitWeightGrads = false) holds the same three blocks
        HipMatrix dx2, a, b, c, o2;
        layer.backward(g, dx2, a, b, c, o2, false);
        if (!a.empty() || !b.empty() || !c.empty()) throw std::runtime_error("split weight gradients were materialised");
        std::vector<float> stacked = layer.qkvWeightGradient.download(), want3(wdq);
        want3.insert(want3.end(), wdk.begin(), wdk.end());
        want3.insert(want3.end(), wdv.begin(), wdv.end());
        if (stacked.size() != want3.size() || relErr(stacked, want3) > tol || relErr(dx2.download(), wdx) > tol)
            throw std::runtime_error(std::string(name) + " stacked weight gradient parity failed");
    }
}

// flash and dense paths of one layer on the same input: outputs and all gradients within tol of each other
static void runFlashVersusDense(const char* name, int e, int heads, int T, float tol) {
    const int d = e / heads;
    unsigned state = 77u + static_cast<unsigned>(e + T);
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
    auto hx = lcg(static_cast<size_t>(e) * T, state, 1.0f);
    auto hg = lcg(static_cast<size_t>(e) * T, state, 1.0f);
    HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;
    std::vector<std::vector<float>> results[2];
    for (int pass = 0; pass < 2; ++pass) {
        HipCausalSelfAttention layer = HipCausalSelfAttention::createFrom(host);
        layer.preferFlashAttention = pass == 0;
        HipMatrix x, g, y, dx, dwq, dwk, dwv, dwo;
        x.upload(hx, e, T);
        g.upload(hg, e, T);
        layer.forward(x, y);
        layer.backward(g, dx, dwq, dwk, dwv, dwo);
        if (layer.usedFlashAttention != (pass == 0)) throw std::runtime_error("wrong attention path");
        results[pass] = {y.download(), dx.download(), dwq.download(), dwk.download(), dwv.download(), dwo.download()};
    }
    float worst = 0.0f;
    for (size_t i = 0; i < results[0].size(); ++i) worst = std::max(worst, relErr(results[0][i], results[1][i]));
    std::printf("  %-40s  flash vs dense worst %.2e\n", name, worst);
    if (worst > tol) throw std::runtime_error(std::string(name) + " flash / dense parity failed");
}

// Generation: prefill `prompt` columns, then decode the rest one token at a time. Step t must reproduce column t of
// the oracle's full forward over columns 0..t (causal attention: earlier columns do not depend on later ones, so
// one oracle call over all columns gives every step's answer).
static void runGeneration(const char* name, int e, int heads, int kvHeads, int d, int prompt, int total, int compute, float tol,
                          int windowSize = 0, int globalTokenCount = 0, bool preferFlash = true) {
    const int qRows = heads * d, kvRows = kvHeads * d;
    unsigned state = 4711u + static_cast<unsigned>(e + total);
    const float bound = 1.0f / std::sqrt(static_cast<float>(e));
    HostAttentionWeights host;
    host.queryWeight = lcg(static_cast<size_t>(qRows) * e, state, bound);
    host.keyWeight = lcg(static_cast<size_t>(kvRows) * e, state, bound);
    host.valueWeight = lcg(static_cast<size_t>(kvRows) * e, state, bound);
    host.outputWeight = lcg(static_cast<size_t>(e) * qRows, state, bound);
    host.embeddingDim = e;
    host.headCount = heads;
    host.kvHeadCount = kvHeads;
    host.headDimension = d;
    host.maximumPositionCount = total;
    host.windowSize = windowSize;
    host.globalTokenCount = globalTokenCount;
    auto hx = lcg(static_cast<size_t>(e) * total, state, 1.0f);
    std::vector<float> want(hx.size());
    if (sentinel_oracle_layer_sparse(hx.data(), host.queryWeight.data(), host.keyWeight.data(), host.valueWeight.data(),
                                     host.outputWeight.data(), nullptr, want.data(), nullptr, nullptr, nullptr, nullptr, nullptr, e,
                                     heads, kvHeads, d, total, host.ropeBase, host.maximumPositionCount, windowSize,
                                     globalTokenCount) != 0)
        throw std::runtime_error("oracle layer failed");

    HipFlashAttention::computeType() = compute;
    HipCausalSelfAttention layer = HipCausalSelfAttention::createFrom(host);
    layer.preferFlashAttention = preferFlash;
    HipKvCache cache;
    auto columns = [&](const std::vector<float>& m, int c0, int count) {
        std::vector<float> out(static_cast<size_t>(e) * count);
        for (int r = 0; r < e; ++r)
            for (int c = 0; c < count; ++c) out[static_cast<size_t>(r) * count + c] = m[static_cast<size_t>(r) * total + c0 + c];
        return out;
    };
    HipMatrix x, y;
    x.upload(columns(hx, 0, prompt), e, prompt);
    layer.prefill(x, cache, y);
    float worst = relErr(y.download(), columns(want, 0, prompt));
    if (cache.length != prompt) throw std::runtime_error("prefill did not fill the cache");
    for (int t = prompt; t < total; ++t) {
        x.upload(columns(hx, t, 1), e, 1);
        layer.decode(x, cache, y);
        worst = std::max(worst, relErr(y.download(), columns(want, t, 1)));
    }
    std::printf("  %-40s  worst step error %.2e\n", name, worst);
    if (worst > tol) throw std::runtime_error(std::string(name) + " generation parity failed");
    if (cache.length != total) throw std::runtime_error("decode did not extend the cache");
    x.upload(columns(hx, 0, 1), e, 1);
    expectThrow("cache full", [&] { layer.decode(x, cache, y); });
    // prefill resets the cache
    x.upload(columns(hx, 0, prompt), e, prompt);
    layer.prefill(x, cache, y);
    if (cache.length != prompt) throw std::runtime_error("prefill did not reset the cache");
}

// HipAmp::preferMixedPrecision (CudaAmp::preferMixedPrecision): the projection products through 16-bit operand copies
// with fp32 accumulation, against the same fp32 oracle layer; which path ran is read from HipAmp::mixedProductCount.
static void runMixedPrecision() {
    struct Restore {
        ~Restore() {
            HipAmp::preferMixedPrecision() = false;
            HipAmp::operandType() = SENTINEL_HIP_F16;
            HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;
        }
    } restore;
    HipAmp::preferMixedPrecision() = true;
    const int types[2] = {SENTINEL_HIP_F16, SENTINEL_HIP_BF16};
    for (int type : types) {
        HipAmp::operandType() = type;
        const char* tag = type == SENTINEL_HIP_F16 ? "fp16" : "bf16";
        unsigned long long before = HipAmp::mixedProductCount();
        runCase((std::string("amp ") + tag + " GEMMs, bf16 attention E256 H4 d64 T128 packs2").c_str(), 256, 4, 4, 64, 128, 2,
                SENTINEL_HIP_COMPUTE_BF16, 2e-2f);
        if (HipAmp::mixedProductCount() < before + 6) throw std::runtime_error("stacked-QKV layer: the 16-bit products did not run");
        before = HipAmp::mixedProductCount();
        runCase((std::string("amp ") + tag + " GEMMs, fp16 attention GQA 4q/1kv d128 T256").c_str(), 256, 4, 1, 128, 256, 1,
                SENTINEL_HIP_COMPUTE_F16, 2e-2f);
        if (HipAmp::mixedProductCount() < before + 12) throw std::runtime_error("grouped-query layer: the 16-bit products did not run");
        runCase((std::string("amp ") + tag + " GEMMs, fp32 attention E256 H8 d32 T96 packs3").c_str(), 256, 8, 8, 32, 96, 3,
                SENTINEL_HIP_COMPUTE_AUTO, 2e-2f);
        runCase((std::string("amp ") + tag + " GEMMs, dense attention E256 H4 d64 T128 packs2").c_str(), 256, 4, 4, 64, 128, 2,
                SENTINEL_HIP_COMPUTE_AUTO, 2e-2f, 0, 0, false);
    }
    HipAmp::operandType() = SENTINEL_HIP_F16;
    // products below the reference's size rule (contraction < 256) stay fp32: same bits as with the switch off
    {
        const unsigned long long before = HipAmp::mixedProductCount();
        runCase("amp on, E64: products too small, fp32", 64, 4, 4, 16, 48, 1, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        if (HipAmp::mixedProductCount() != before) throw std::runtime_error("a product below the size rule took the 16-bit path");
    }
    // master weights: the 16-bit copy is kept until invalidateMasterWeightHalves, registrations follow the layer
    const int e = 256, heads = 4, d = 64, T = 256;  // every product of the step passes the size rule
    unsigned state = 77u;
    HostAttentionWeights host;
    host.embeddingDim = e;
    host.headCount = heads;
    host.headDimension = d;
    host.maximumPositionCount = T;
    const float bound = 1.0f / std::sqrt(static_cast<float>(e));
    host.queryWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.keyWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.valueWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    host.outputWeight = lcg(static_cast<size_t>(e) * e, state, bound);
    HipMatrix x, y1, y2, y3, y4;
    x.upload(lcg(static_cast<size_t>(e) * T, state, 1.0f), e, T);
    const float* deadWeight = nullptr;
    size_t deadCount = 0;
    {
        HipCausalSelfAttention built = HipCausalSelfAttention::createFrom(host);
        HipCausalSelfAttention layer = std::move(built);  // registrations move with the buffers
        layer.forward(x, y1, T);
        deadWeight = layer.outputWeight.buffer.deviceData;
        deadCount = layer.outputWeight.elementCount();
        if (HipAmp::masterWeightHalfOrNull(deadWeight, deadCount, SENTINEL_HIP_F16) == nullptr ||
            HipAmp::masterWeightHalfOrNull(layer.qkvWeight.buffer.deviceData, layer.qkvWeight.elementCount(), SENTINEL_HIP_F16) == nullptr)
            throw std::runtime_error("the layer's weights are not registered with HipAmp");
        // the optimizer's step: new output weights in the same buffer
        layer.outputWeight.upload(lcg(static_cast<size_t>(e) * e, state, bound), e, e);
        if (layer.outputWeight.buffer.deviceData != deadWeight) throw std::runtime_error("upload moved the weight");
        layer.forward(x, y2, T);  // the kept copy still serves: the caller has not said that the weights changed
        if (y2.download() != y1.download()) throw std::runtime_error("the kept 16-bit weight copy was not used");
        HipAmp::invalidateMasterWeightHalves();
        layer.forward(x, y3, T);
        {
            // a training step with warm weight copies casts four activations: input and attended in the forward call (kept
            // for the backward call), output gradient and stacked projection gradient in the backward call
            HipMatrix g, dx, a, b, c, o;
            g.upload(lcg(static_cast<size_t>(e) * T, state, 1.0f), e, T);
            const unsigned long long casts = HipAmp::castCount(), products = HipAmp::mixedProductCount();
            layer.forward(x, y3, T);
            layer.backward(g, dx, a, b, c, o);
            if (HipAmp::mixedProductCount() != products + 6 || HipAmp::castCount() != casts + 4)
                throw std::runtime_error("mixed-precision step: expected 6 products and 4 casts, got " +
                                         std::to_string(HipAmp::mixedProductCount() - products) + " and " +
                                         std::to_string(HipAmp::castCount() - casts));
        }
        HipAmp::preferMixedPrecision() = false;
        layer.forward(x, y4, T);
        HipAmp::preferMixedPrecision() = true;
        const float fresh = relErr(y3.download(), y4.download()), stale = relErr(y1.download(), y4.download());
        std::printf("  %-40s  new weights: %.2e from fp32, old copy: %.2e\n", "amp master weight copies", fresh, stale);
        if (fresh > 2e-2f || stale < 0.1f) throw std::runtime_error("invalidateMasterWeightHalves did not refresh the copy");
    }
    if (HipAmp::masterWeightHalfOrNull(deadWeight, deadCount, SENTINEL_HIP_F16) != nullptr)
        throw std::runtime_error("a dead layer's weight is still registered with HipAmp");
    expectThrow("operand type", [&] {
        HipAmp::operandType() = SENTINEL_HIP_F32;
        HipCausalSelfAttention layer = HipCausalSelfAttention::createFrom(host);
        layer.forward(x, y1, T);
    });
}

int main() {
    try {
        if (!sentinel_hip_device_available()) {
            std::printf("  no HIP device\n");
            return 2;
        }
        runCase("fp32 E64 H4 d16 T48", 64, 4, 4, 16, 48, 1, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        runCase("fp32 E64 H4 d16 T48 packs4", 64, 4, 4, 16, 48, 4, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        runCase("fp32 GQA E64 8q/2kv d8 T16 packs3", 64, 8, 2, 8, 16, 3, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        runCase("fp32 E96 H3 d32 T70 packs2", 96, 3, 3, 32, 70, 2, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        // MFMA arithmetic for the attention core (projections stay fp32), rotation fused into the conversion passes
        runCase("bf16 E256 H4 d64 T128 packs2", 256, 4, 4, 64, 128, 2, SENTINEL_HIP_COMPUTE_BF16, 2e-2f);
        runCase("fp16 GQA E256 4q/1kv d128 T200", 256, 4, 1, 128, 200, 1, SENTINEL_HIP_COMPUTE_F16, 2e-2f);
        // head dims without a tiling of their own (zero-padded to 64 / 128 inside the conversion pass), rotation fused
        runCase("bf16 E288 H3 d96 T130 packs2", 288, 3, 3, 96, 130, 2, SENTINEL_HIP_COMPUTE_BF16, 2e-2f);
        runCase("fp16 GQA E128 4q/2kv d32 T70", 128, 4, 2, 32, 70, 1, SENTINEL_HIP_COMPUTE_F16, 2e-2f);
        // the sparse mask: the shape of runSparseComputeSmokeDemo (E=32, H=2, T=16, W=4, G=2) and larger ones
        HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;
        runCase("sparse fp32 E32 H2 d16 T16 W4 G2", 32, 2, 2, 16, 16, 1, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 4, 2);
        runCase("sparse fp32 GQA 8q/2kv d8 T90 W17 G3 packs2", 64, 8, 2, 8, 90, 2, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 17, 3);
        runCase("sparse bf16 E256 H4 d64 T300 W70 G10", 256, 4, 4, 64, 300, 1, SENTINEL_HIP_COMPUTE_BF16, 2e-2f, 70, 10);
        runCase("sparse fp16 GQA 4q/1kv d128 T200 W33 packs2", 256, 4, 1, 128, 200, 2, SENTINEL_HIP_COMPUTE_F16, 2e-2f, 33, 0);
        HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;
        // the dense materialising path (flash switched off) against the oracle layer, then against the flash path
        runCase("dense fp32 E64 H4 d16 T48", 64, 4, 4, 16, 48, 1, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 0, 0, false);
        runCase("dense fp32 E64 H4 d16 T48 packs4", 64, 4, 4, 16, 48, 4, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 0, 0, false);
        runCase("dense fp32 GQA 8q/2kv d8 T16 packs3", 64, 8, 2, 8, 16, 3, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 0, 0, false);
        runCase("dense fp32 E96 H3 d32 T70 packs2", 96, 3, 3, 32, 70, 2, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 0, 0, false);
        runCase("dense fp32 GQA 4q/1kv d128 T200", 256, 4, 1, 128, 200, 1, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 0, 0, false);
        runCase("dense sparse fp32 E32 H2 d16 T16 W4 G2", 32, 2, 2, 16, 16, 1, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 4, 2, false);
        runCase("dense sparse GQA 8q/2kv d8 T90 W17 G3 packs2", 64, 8, 2, 8, 90, 2, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 17, 3, false);
        runFlashVersusDense("E64 H4 T48", 64, 4, 48, 1e-4f);
        runFlashVersusDense("E768 H12 T128", 768, 12, 128, 1e-4f);
        runFlashVersusDense("E768 H12 T256", 768, 12, 256, 1e-4f);
        // the shapes of runKvCacheSmokeDemo (E=64, H=4, T=32 of 64 positions), grouped heads, a cache of several chunks
        runGeneration("generate fp32 E64 H4 d16 32+32", 64, 4, 4, 16, 32, 64, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        runGeneration("generate fp32 GQA 8q/2kv d8 5+20", 64, 8, 2, 8, 5, 25, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        runGeneration("generate fp32 E128 H2 d64 1+300", 128, 2, 2, 64, 1, 301, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f);
        runGeneration("generate bf16 prefill GQA 4q/1kv d128", 256, 4, 1, 128, 130, 140, SENTINEL_HIP_COMPUTE_BF16, 2e-2f);
        runGeneration("generate sparse fp32 H4 d16 20+60 W9 G2", 64, 4, 4, 16, 20, 80, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 9, 2);
        runGeneration("generate sparse fp32 GQA d64 3+400 W100 G70", 128, 4, 2, 64, 3, 403, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 100, 70);
        runGeneration("generate dense prefill H4 d16 32+32", 64, 4, 4, 16, 32, 64, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 0, 0, false);
        runGeneration("generate dense prefill sparse GQA W9 G2", 64, 4, 2, 16, 20, 60, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 9, 2, false);
        HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;
        runMixedPrecision();

        // configurations this layer does not run are refused, not approximated
        HostAttentionWeights host;
        unsigned st = 9u;
        host.embeddingDim = 32;
        host.headCount = 2;
        host.headDimension = 16;
        host.maximumPositionCount = 32;
        host.queryWeight = lcg(32 * 32, st, 0.1f);
        host.keyWeight = host.queryWeight;
        host.valueWeight = host.queryWeight;
        host.outputWeight = host.queryWeight;
        HipMatrix x, y;
        x.ensureSize(32, 16);
        x.fill(0.1f);
        {
            // split weights replaced by matrices of their own are stacked again by syncFusedQkvWeight; the split weights
            // of a fresh layer are views of the stacked matrix (no copy to keep in step)
            HipCausalSelfAttention layer = HipCausalSelfAttention::createFrom(host);
            if (layer.queryWeight.buffer.deviceData != layer.qkvWeight.buffer.deviceData || layer.keyWeight.buffer.ownsMemory)
                throw std::runtime_error("split weights are not views of the stacked weights");
            HipMatrix before, after, varied;  // columns that differ, so that the keys matter
            varied.upload(lcg(32 * 16, st, 1.0f), 32, 16);
            layer.forward(varied, before);
            HipMatrix own;
            own.upload(lcg(32 * 32, st, 0.2f), 32, 32);
            layer.keyWeight = std::move(own);
            layer.syncFusedQkvWeight();
            if (layer.keyWeight.buffer.ownsMemory || layer.keyWeight.buffer.deviceData != layer.qkvWeight.buffer.deviceData + 32 * 32)
                throw std::runtime_error("syncFusedQkvWeight did not re-stack");
            layer.forward(varied, after);
            if (relErr(after.download(), before.download()) < 1e-3f) throw std::runtime_error("new key weights had no effect");
            layer.releaseActivationScratch();
            if (!layer.query.empty() || !layer.inputCache.empty() || layer.qkvWeight.empty())
                throw std::runtime_error("releaseActivationScratch");
            layer.forward(x, after);
        }
        HipCausalSelfAttention dense = HipCausalSelfAttention::createFrom(host);
        expectThrow("columns not a multiple of the segment", [&] { dense.forward(x, y, 5); });
        HipMatrix longer;
        longer.ensureSize(32, 40);
        longer.fill(0.1f);
        expectThrow("sequence longer than the RoPE table", [&] { dense.forward(longer, y); });
        HipMatrix dx, a, b, c, d;
        HipCausalSelfAttention fresh = HipCausalSelfAttention::createFrom(host);
        expectThrow("backward before forward", [&] { fresh.backward(x, dx, a, b, c, d); });
        host.kvHeadCount = 3;
        expectThrow("heads not divisible", [&] { HipCausalSelfAttention::createFrom(host); });
        std::printf("  layer ok\n");
        return 0;
    } catch (const std::exception& ex) {
        std::printf("  FAILED: %s\n", ex.what());
        return 1;
    }
}
