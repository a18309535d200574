// GPU test of the C++ shim: reads like the reference's own smoke demos (LCG inputs, max-abs-diff against the
// CPU path, throw on threshold breach; Cuda/CudaCausalSelfAttention.cu:577-697, :896-997), with the CPU side
// played by the oracle library.  Exit code 0 = pass.
#include "../../include/sentinel_hip/HipFlashAttention.hpp"
#include "../../oracle/sentinel_attention_oracle.h"

#include <cmath>
#include <cstdio>
#include <stdexcept>
#include <vector>

using namespace sentinel_hip_host;

static std::vector<float> lcg(size_t count, unsigned& state) {  // Layers/CausalSelfAttention.cpp:566-574
    std::vector<float> out(count);
    for (size_t i = 0; i < count; ++i) {
        state = state * 1664525u + 1013904223u;
        out[i] = (static_cast<float>(state >> 8) / 16777216.0f) * 2.0f - 1.0f;
    }
    return out;
}

static float maxAbsDiff(const std::vector<float>& a, const std::vector<float>& b, size_t stride, size_t col0, size_t cols) {
    float diff = 0.0f;
    for (size_t r = 0; r < a.size() / stride; ++r)
        for (size_t c = col0; c < col0 + cols; ++c) diff = std::max(diff, std::fabs(a[r * stride + c] - b[r * stride + c]));
    return diff;
}

template <typename Fn>
static void expectInvalid(const char* what, Fn fn) {
    try {
        fn();
    } catch (const std::invalid_argument&) {
        return;
    }
    throw std::runtime_error(std::string("expected std::invalid_argument: ") + what);
}

static void runCase(const char* name, int heads, int kvHeads, int d, int T, int packs, int col0, int pad, int compute,
                    float fwdTol, float bwdTol) {
    const int stride = col0 + packs * T + pad;
    unsigned state = 123u;
    auto hq = lcg(static_cast<size_t>(heads) * d * stride, state);
    auto hk = lcg(static_cast<size_t>(kvHeads) * d * stride, state);
    auto hv = lcg(static_cast<size_t>(kvHeads) * d * stride, state);
    auto hg = lcg(static_cast<size_t>(heads) * d * stride, state);
    const float scale = 1.0f / std::sqrt(static_cast<float>(d));

    std::vector<float> ro(hq.size()), rl(static_cast<size_t>(heads) * stride), rdq(hq.size()), rdk(hk.size()), rdv(hv.size());
    if (sentinel_oracle_attention(hq.data(), hk.data(), hv.data(), ro.data(), rl.data(), hg.data(), rdq.data(), rdk.data(),
                                  rdv.data(), heads, kvHeads, d, stride, col0, T, packs, scale, 1, 0) != 0)
        throw std::runtime_error("oracle failed");

    HipMatrix q, k, v, g, out, lse, dq, dk, dv, delta;
    q.upload(hq, static_cast<size_t>(heads) * d, stride);
    k.upload(hk, static_cast<size_t>(kvHeads) * d, stride);
    v.upload(hv, static_cast<size_t>(kvHeads) * d, stride);
    g.upload(hg, static_cast<size_t>(heads) * d, stride);
    HipFlashAttention::computeType() = compute;
    HipFlashAttention::forwardMultiHead(q, k, v, out, lse, heads, d, scale, true, col0, T, packs, kvHeads);
    HipFlashAttention::backwardMultiHead(q, k, v, out, lse, g, dq, dk, dv, delta, heads, d, scale, true, col0, T, packs, kvHeads);
    const size_t cols = static_cast<size_t>(packs) * T;
    const float eo = maxAbsDiff(out.download(), ro, stride, col0, cols);
    const float el = maxAbsDiff(lse.download(), rl, stride, col0, cols);
    const float eq = maxAbsDiff(dq.download(), rdq, stride, col0, cols);
    const float ek = maxAbsDiff(dk.download(), rdk, stride, col0, cols);
    const float ev = maxAbsDiff(dv.download(), rdv, stride, col0, cols);
    std::printf("  %-34s  out=%.2e lse=%.2e dQ=%.2e dK=%.2e dV=%.2e\n", name, eo, el, eq, ek, ev);
    if (eo > fwdTol || el > fwdTol || eq > bwdTol || ek > bwdTol || ev > bwdTol) throw std::runtime_error(std::string(name) + " parity failed");
    if (delta.rows != static_cast<size_t>(heads) || delta.cols != cols) throw std::runtime_error("delta workspace shape");
}

int main() {
    try {
        if (!sentinel_hip_device_available()) {
            std::printf("  no HIP device\n");
            return 2;
        }
        // flash parity shapes of the reference (main.cpp:640-643 uses E=64,H=4,T=48) and its GQA smoke (8q/2kv, T=16)
        runCase("fp32 E64 H4 T48 packs4", 4, 4, 16, 48, 4, 0, 0, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 1e-4f);
        runCase("fp32 GQA 8q/2kv d8 T16", 8, 2, 8, 16, 1, 0, 0, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 1e-4f);
        runCase("fp32 window col0=8 T100 packs2", 2, 1, 32, 100, 2, 8, 12, SENTINEL_HIP_COMPUTE_AUTO, 1e-4f, 1e-4f);
        // MFMA arithmetic on Sentinel's fp32 layout (what the CUDA WMMA path does with fp16 tiles); the reference's own
        // flash thresholds for this are 1e-3 forward / 1e-1 backward (Cuda/CudaCausalSelfAttention.cu:970, :984)
        runCase("bf16-mfma E768 H12 T128", 12, 12, 64, 128, 1, 0, 0, SENTINEL_HIP_COMPUTE_BF16, 2e-2f, 1e-1f);
        runCase("fp16-mfma GQA 8q/2kv d128 T200 x2", 8, 2, 128, 200, 2, 4, 4, SENTINEL_HIP_COMPUTE_F16, 5e-3f, 5e-2f);
        HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;

        HipMatrix q, out, lse;
        q.ensureSize(64, 192);
        q.fill(0.1f);
        expectInvalid("head geometry", [&] { HipFlashAttention::forwardMultiHead(q, q, q, out, lse, 0, 16, 0.25f); });
        expectInvalid("rows mismatch", [&] { HipFlashAttention::forwardMultiHead(q, q, q, out, lse, 3, 16, 0.25f); });
        expectInvalid("column window", [&] { HipFlashAttention::forwardMultiHead(q, q, q, out, lse, 4, 16, 0.25f, true, 100, 100, 1); });
        expectInvalid("pack window", [&] { HipFlashAttention::forwardMultiHead(q, q, q, out, lse, 4, 16, 0.25f, true, 0, 48, 5); });
        HipMatrix big;
        big.ensureSize(256, 8);
        big.fill(0.0f);
        expectInvalid("maxHeadDimension", [&] { HipFlashAttention::forwardMultiHead(big, big, big, out, lse, 1, 256, 0.25f); });
        // rotary embedding: bit-identical to the oracle, inverse undoes it, reference exception on a short table
        {
            const int heads = 3, d = 32, cols = 70, positions = 80;
            unsigned st = 7u;
            auto hx = lcg(static_cast<size_t>(heads) * d * cols, st);
            std::vector<float> hc(static_cast<size_t>(positions) * d / 2), hs(hc.size());
            if (sentinel_oracle_rope_tables(d, positions, 10000.0f, hc.data(), hs.data()) != 0) throw std::runtime_error("oracle tables");
            std::vector<float> want = hx;
            if (sentinel_oracle_rope_rotate(want.data(), heads, d, cols, 0, cols, 5, 0, hc.data(), hs.data(), positions, 0) != 0)
                throw std::runtime_error("oracle rope");
            HipMatrix x, ct, stb;
            x.upload(hx, static_cast<size_t>(heads) * d, cols);
            ct.upload(hc, positions, d / 2);
            stb.upload(hs, positions, d / 2);
            HipOps::rotaryRotateInPlace(x, heads, d, d / 2, ct, stb, 5);
            if (x.download() != want) throw std::runtime_error("rope rotate differs from the oracle");
            HipOps::rotaryRotateInverseInPlace(x, heads, d, d / 2, ct, stb, 5);
            const float back = maxAbsDiff(x.download(), hx, cols, 0, cols);
            std::printf("  %-34s  bit-exact, inverse round trip %.2e\n", "rope H3 d32 T70 offset 5", back);
            if (back > 2e-6f) throw std::runtime_error("rope inverse round trip");
            expectInvalid("rope table too short", [&] { HipOps::rotaryRotateInPlace(x, heads, d, d / 2, ct, stb, 11); });
            expectInvalid("rope dims", [&] { HipOps::rotaryRotateInPlace(x, heads, d, 0, ct, stb); });
        }
        // kept operands belong to the matrices they were made from: a backward call that is handed another key matrix
        // (or another mask) together with the forward call's KeptOperands converts everything again
        {
            const int heads = 2, d = 64, T = 96;
            const float scale = 0.125f;
            unsigned st = 99u;
            HipMatrix q, k, k2, v, g, out, lse, dq, dk, dv, delta, dq2, dk2, dv2, delta2;
            q.upload(lcg(static_cast<size_t>(heads) * d * T, st), static_cast<size_t>(heads) * d, T);
            k.upload(lcg(static_cast<size_t>(heads) * d * T, st), static_cast<size_t>(heads) * d, T);
            k2.upload(lcg(static_cast<size_t>(heads) * d * T, st), static_cast<size_t>(heads) * d, T);
            v.upload(lcg(static_cast<size_t>(heads) * d * T, st), static_cast<size_t>(heads) * d, T);
            g.upload(lcg(static_cast<size_t>(heads) * d * T, st), static_cast<size_t>(heads) * d, T);
            HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_BF16;
            HipFlashAttention::KeptOperands kept;
            HipFlashAttention::forwardMultiHead(q, k, v, out, lse, heads, d, scale, true, 0, T, 1, 0, &kept);
            if (!kept.filled) throw std::runtime_error("forward did not keep its operands");
            HipFlashAttention::backwardMultiHead(q, k2, v, out, lse, g, dq, dk, dv, delta, heads, d, scale, true, 0, T, 1, 0, &kept);
            HipFlashAttention::backwardMultiHead(q, k2, v, out, lse, g, dq2, dk2, dv2, delta2, heads, d, scale, true, 0, T, 1, 0, nullptr);
            if (dq.download() != dq2.download() || dk.download() != dk2.download() || dv.download() != dv2.download())
                throw std::runtime_error("backward reused 16-bit copies of another key matrix");
            HipFlashAttention::backwardMultiHead(q, k, v, out, lse, g, dq, dk, dv, delta, heads, d, scale, false, 0, T, 1, 0, &kept);
            HipFlashAttention::backwardMultiHead(q, k, v, out, lse, g, dq2, dk2, dv2, delta2, heads, d, scale, false, 0, T, 1, 0, nullptr);
            if (dq.download() != dq2.download() || dk.download() != dk2.download() || dv.download() != dv2.download())
                throw std::runtime_error("backward under another mask differs with kept operands");
            kept.invalidate();
            HipFlashAttention::backwardMultiHead(q, k, v, out, lse, g, dq, dk, dv, delta, heads, d, scale, true, 0, T, 1, 0, &kept);
            HipFlashAttention::backwardMultiHead(q, k, v, out, lse, g, dq2, dk2, dv2, delta2, heads, d, scale, true, 0, T, 1, 0, nullptr);
            if (dq.download() != dq2.download()) throw std::runtime_error("backward after invalidate() differs");
            HipFlashAttention::computeType() = SENTINEL_HIP_COMPUTE_AUTO;
            std::printf("  %-34s  ok\n", "kept operands tied to their tensors");
        }
        // single-head wrappers
        HipMatrix one, o1, l1, d1, d2, d3;
        one.ensureSize(16, 40);
        one.fill(0.05f);
        HipFlashAttention::forward(one, one, one, o1, l1, 0.25f);
        HipFlashAttention::backward(one, one, one, o1, l1, one, d1, d2, d3, 0.25f);
        if (o1.rows != 16 || l1.rows != 1 || d1.cols != 40) throw std::runtime_error("single-head wrapper shapes");
        std::printf("  shim ok\n");
        return 0;
    } catch (const std::exception& e) {
        std::printf("  FAILED: %s\n", e.what());
        return 1;
    }
}
