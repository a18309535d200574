// Exact fp32 attention forward / backward for gfx950: plain FMA arithmetic, one query (or key) per lane.
//
// This is the path for fp32 tensors that must match Sentinel's CPU attention to 1e-4 (the quickstart
// LM shape, head_dim 16): no operand is rounded below fp32.  It works on any element strides, so it
// reads Sentinel's column layout directly (lanes walk the contiguous column axis, which makes the
// per-lane global loads coalesced there) as well as [B,H,T,d].
//
// Stands for the scalar kernels CudaFlashAttentionForwardFixedEntry / ForwardEntry
// (sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:467-574, :337-438), CudaFlashAttentionDeltaEntry
// (:576-596) and the backward pair BackwardQueryFixedEntry / BackwardKeyEntry (:857-1005, :599-719),
// with two changes of design: dK/dV come from a key-outer kernel and dQ from a query-outer kernel, so
// no gradient needs atomics or pre-zeroed buffers, and grouped K/V heads are read in place.
#include "flash_common.h"

#include <math.h>

namespace sentinel_hip {
namespace {

constexpr int kLanes = 64;     // one wavefront per workgroup
constexpr int kKeyStage = 32;  // keys staged in LDS per step (forward, dQ)
constexpr int kQueryStage = 16;  // queries staged in LDS per step (dK/dV)

// Copy a [rows x DP] fp32 tile of one head into LDS as tile[row][c], zero-filled outside (T, d).
template <int DP, int ROWS>
__device__ __forceinline__ void stage_rows(float* tile, const float* base, const TensorMap& m, int row0, int T, int d,
                                           int lane) {
    for (int idx = lane; idx < ROWS * DP; idx += kLanes) {
        int r, c;
        if (m.t_stride == 1) {  // column layout: consecutive lanes walk tokens
            c = idx / ROWS;
            r = idx % ROWS;
        } else {
            r = idx / DP;
            c = idx % DP;
        }
        const int t = row0 + r;
        float x = 0.0f;
        if (t < T && c < d) x = base[t * m.t_stride + c * m.c_stride];
        tile[r * DP + c] = x;
    }
}

template <int DP>
__global__ __launch_bounds__(kLanes) void fwd_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                          const float* __restrict__ v, float* __restrict__ out,
                                                          float* __restrict__ lse, TensorMap qm, TensorMap km, RowMap lm,
                                                          AttnGeom g) {
    __shared__ __attribute__((aligned(16))) float ks[kKeyStage * DP];
    __shared__ __attribute__((aligned(16))) float vs[kKeyStage * DP];

    const int lane = threadIdx.x;
    const int tile = gridDim.x - 1 - blockIdx.x;  // longest rows first under the causal mask
    const int h = blockIdx.y;
    const int b = blockIdx.z;
    const int kvh = h / (g.q_heads / g.kv_heads);
    const int d = g.head_dim;
    const int T = g.seq_len;
    const int qi = tile * kLanes + lane;
    const int qload = qi < T ? qi : T - 1;

    const float* qp = q + b * qm.pack_stride + h * qm.head_stride + qload * qm.t_stride;
    const float* kbase = k + b * km.pack_stride + kvh * km.head_stride;
    const float* vbase = v + b * km.pack_stride + kvh * km.head_stride;

    float qr[DP];
    float acc[DP];
#pragma unroll
    for (int c = 0; c < DP; ++c) {
        qr[c] = c < d ? qp[c * qm.c_stride] : 0.0f;
        acc[c] = 0.0f;
    }

    const float c2 = g.scale * kLog2e;
    float m = -INFINITY;
    float l = 0.0f;
    const int kv_end = g.causal ? min(T, tile * kLanes + kLanes) : T;

    // first key any query of this tile still sees through its window (stages before it matter only for global tokens)
    const int window_lo = g.window > 0 ? tile * kLanes - g.window + 1 : 0;

    for (int k0 = 0; k0 < kv_end; k0 += kKeyStage) {
        if (k0 >= g.global_tokens && k0 + kKeyStage <= window_lo) continue;  // workgroup-uniform: nothing visible in this stage
        __syncthreads();
        stage_rows<DP, kKeyStage>(ks, kbase, km, k0, T, d, lane);
        stage_rows<DP, kKeyStage>(vs, vbase, km, k0, T, d, lane);
        __syncthreads();

        for (int j0 = 0; j0 < kKeyStage; j0 += 8) {
            if (k0 + j0 >= kv_end) break;
            float s[8];
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                const float* kr = ks + (j0 + jj) * DP;
                float dot = 0.0f;
#pragma unroll
                for (int c = 0; c < DP; ++c) dot += qr[c] * kr[c];
                const int kj = k0 + j0 + jj;
                s[jj] = (kj >= T || (g.causal && kj > qi) || outside_window(g, qi, kj)) ? -INFINITY : dot;
            }
            float mx = m;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) mx = fmaxf(mx, s[jj]);
            const float mref = (mx == -INFINITY) ? 0.0f : mx;
            const float alpha = exp2f((m - mref) * c2);
            float p[8];
            float psum = 0.0f;
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) {
                p[jj] = exp2f((s[jj] - mref) * c2);
                psum += p[jj];
            }
            l = l * alpha + psum;
#pragma unroll
            for (int c = 0; c < DP; ++c) {
                float a = acc[c] * alpha;
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) a += p[jj] * vs[(j0 + jj) * DP + c];
                acc[c] = a;
            }
            m = mx;
        }
    }

    if (qi < T) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        float* op = out + b * qm.pack_stride + h * qm.head_stride + qi * qm.t_stride;
#pragma unroll
        for (int c = 0; c < DP; ++c)
            if (c < d) op[c * qm.c_stride] = acc[c] * inv;
        lse[b * lm.pack_stride + h * lm.head_stride + qi] = m * g.scale + (l > 0.0f ? logf(l) : 0.0f);
    }
}

// dQ: one query per lane, keys streamed through LDS.  Runs first: the lane holds its query's dO row anyway, so it also
// forms D[h][b*T + t] = sum_c out * d_out (dims in increasing order, as the reference's Delta kernel sums them,
// CudaFlashAttention.cu:576-596) and leaves it in `delta` for the dK / dV kernel: no launch of its own for that.
template <int DP>
__global__ __launch_bounds__(kLanes) void bwd_dq_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                             const float* __restrict__ v, const float* __restrict__ out,
                                                             const float* __restrict__ lse,
                                                             const float* __restrict__ d_out, float* __restrict__ delta,
                                                             float* __restrict__ dq, TensorMap qm, TensorMap km, RowMap lm,
                                                             AttnGeom g) {
    __shared__ __attribute__((aligned(16))) float ks[kKeyStage * DP];
    __shared__ __attribute__((aligned(16))) float vs[kKeyStage * DP];

    const int lane = threadIdx.x;
    const int tile = gridDim.x - 1 - blockIdx.x;
    const int h = blockIdx.y;
    const int b = blockIdx.z;
    const int kvh = h / (g.q_heads / g.kv_heads);
    const int d = g.head_dim;
    const int T = g.seq_len;
    const int qi = tile * kLanes + lane;
    const int qload = qi < T ? qi : T - 1;

    const long long qoff = b * qm.pack_stride + h * qm.head_stride + qload * qm.t_stride;
    const float* kbase = k + b * km.pack_stride + kvh * km.head_stride;
    const float* vbase = v + b * km.pack_stride + kvh * km.head_stride;

    float qr[DP];
    float gr[DP];
    float acc[DP];
#pragma unroll
    for (int c = 0; c < DP; ++c) {
        qr[c] = c < d ? q[qoff + c * qm.c_stride] : 0.0f;
        gr[c] = c < d ? d_out[qoff + c * qm.c_stride] : 0.0f;
        acc[c] = 0.0f;
    }
    const float c2 = g.scale * kLog2e;
    const float lse2 = lse[b * lm.pack_stride + h * lm.head_stride + qload] * kLog2e;
    float dl = 0.0f;
    for (int c = 0; c < d; ++c) dl += out[qoff + c * qm.c_stride] * d_out[qoff + c * qm.c_stride];
    if (qi < T) delta[(long long)h * g.packs * T + (long long)b * T + qi] = dl;
    const int kv_end = g.causal ? min(T, tile * kLanes + kLanes) : T;
    const int window_lo = g.window > 0 ? tile * kLanes - g.window + 1 : 0;

    for (int k0 = 0; k0 < kv_end; k0 += kKeyStage) {
        if (k0 >= g.global_tokens && k0 + kKeyStage <= window_lo) continue;  // workgroup-uniform: nothing visible in this stage
        __syncthreads();
        stage_rows<DP, kKeyStage>(ks, kbase, km, k0, T, d, lane);
        stage_rows<DP, kKeyStage>(vs, vbase, km, k0, T, d, lane);
        __syncthreads();
        for (int j = 0; j < kKeyStage; ++j) {
            const int kj = k0 + j;
            if (kj >= kv_end) break;
            const float* kr = ks + j * DP;
            const float* vr = vs + j * DP;
            float s = 0.0f;
            float dp = 0.0f;
#pragma unroll
            for (int c = 0; c < DP; ++c) {
                s += qr[c] * kr[c];
                dp += gr[c] * vr[c];
            }
            const float p = ((g.causal && kj > qi) || outside_window(g, qi, kj)) ? 0.0f : exp2f(s * c2 - lse2);
            const float ds = p * (dp - dl) * g.scale;
#pragma unroll
            for (int c = 0; c < DP; ++c) acc[c] += ds * kr[c];
        }
    }
    if (qi < T) {
        float* dst = dq + b * qm.pack_stride + h * qm.head_stride + qi * qm.t_stride;
#pragma unroll
        for (int c = 0; c < DP; ++c)
            if (c < d) dst[c * qm.c_stride] = acc[c];
    }
}

// dK, dV: one key per lane; the group's query heads and their query tiles are streamed through LDS.
// Dynamic LDS: kt[DP][64], vt[DP][64] (own keys, transposed so lanes read consecutive words),
// qs[16][DP], gs[16][DP], lse2s[16], dls[16].
template <int DP>
__global__ __launch_bounds__(kLanes) void bwd_dkdv_f32_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                               const float* __restrict__ v,
                                                               const float* __restrict__ lse,
                                                               const float* __restrict__ d_out,
                                                               const float* __restrict__ delta, float* __restrict__ dk,
                                                               float* __restrict__ dv, TensorMap qm, TensorMap km,
                                                               RowMap lm, AttnGeom g) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* kt = smem;
    float* vt = kt + DP * kLanes;
    float* qs = vt + DP * kLanes;
    float* gs = qs + kQueryStage * DP;
    float* lse2s = gs + kQueryStage * DP;
    float* dls = lse2s + kQueryStage;

    const int lane = threadIdx.x;
    const int ktile = blockIdx.x;
    const int kvh = blockIdx.y;
    const int b = blockIdx.z;
    const int d = g.head_dim;
    const int T = g.seq_len;
    const int group = g.q_heads / g.kv_heads;
    const int kj = ktile * kLanes + lane;
    const int kload = kj < T ? kj : T - 1;

    {
        const long long koff = b * km.pack_stride + kvh * km.head_stride + kload * km.t_stride;
        for (int c = 0; c < DP; ++c) {
            kt[c * kLanes + lane] = c < d ? k[koff + c * km.c_stride] : 0.0f;
            vt[c * kLanes + lane] = c < d ? v[koff + c * km.c_stride] : 0.0f;
        }
    }
    float dkr[DP];
    float dvr[DP];
#pragma unroll
    for (int c = 0; c < DP; ++c) {
        dkr[c] = 0.0f;
        dvr[c] = 0.0f;
    }
    const float c2 = g.scale * kLog2e;
    const int q_begin = g.causal ? ktile * kLanes : 0;
    // a tile without global tokens is seen by the queries up to its last key + window - 1 only
    const int q_end = (g.window > 0 && ktile * kLanes >= g.global_tokens) ? min(T, ktile * kLanes + kLanes + g.window - 1) : T;

    for (int gi = 0; gi < group; ++gi) {
        const int h = kvh * group + gi;
        const float* qbase = q + b * qm.pack_stride + h * qm.head_stride;
        const float* gbase = d_out + b * qm.pack_stride + h * qm.head_stride;
        const float* lrow = lse + b * lm.pack_stride + h * lm.head_stride;
        const float* drow = delta + (long long)h * g.packs * T + (long long)b * T;
        for (int q0 = q_begin; q0 < q_end; q0 += kQueryStage) {
            __syncthreads();
            stage_rows<DP, kQueryStage>(qs, qbase, qm, q0, T, d, lane);
            stage_rows<DP, kQueryStage>(gs, gbase, qm, q0, T, d, lane);
            if (lane < kQueryStage) {
                const int t = q0 + lane;
                lse2s[lane] = t < T ? lrow[t] * kLog2e : INFINITY;
                dls[lane] = t < T ? drow[t] : 0.0f;
            }
            __syncthreads();
            for (int i = 0; i < kQueryStage; ++i) {
                const int qi = q0 + i;
                if (qi >= T) break;
                const float* qrow = qs + i * DP;
                const float* grow = gs + i * DP;
                float s = 0.0f;
                float dp = 0.0f;
#pragma unroll
                for (int c = 0; c < DP; ++c) {
                    s += qrow[c] * kt[c * kLanes + lane];
                    dp += grow[c] * vt[c * kLanes + lane];
                }
                const float p = (kj >= T || (g.causal && kj > qi) || outside_window(g, qi, kj)) ? 0.0f : exp2f(s * c2 - lse2s[i]);
                const float ds = p * (dp - dls[i]) * g.scale;
#pragma unroll
                for (int c = 0; c < DP; ++c) {
                    dvr[c] += p * grow[c];
                    dkr[c] += ds * qrow[c];
                }
            }
        }
    }
    if (kj < T) {
        const long long koff = b * km.pack_stride + kvh * km.head_stride + kj * km.t_stride;
#pragma unroll
        for (int c = 0; c < DP; ++c)
            if (c < d) {
                dk[koff + c * km.c_stride] = dkr[c];
                dv[koff + c * km.c_stride] = dvr[c];
            }
    }
}

template <int DP>
size_t dkdv_lds_bytes() {
    return sizeof(float) * (2 * DP * kLanes + 2 * kQueryStage * DP + 2 * kQueryStage);
}

template <int DP>
hipError_t run_fwd(const float* q, const float* k, const float* v, float* out, float* lse, TensorMap qm, TensorMap kvm,
                   RowMap lm, AttnGeom g, hipStream_t stream) {
    const dim3 grid((g.seq_len + kLanes - 1) / kLanes, g.q_heads, g.packs);
    KernelTimer timer("fwd_f32", stream);
    hipLaunchKernelGGL(fwd_f32_kernel<DP>, grid, dim3(kLanes), 0, stream, q, k, v, out, lse, qm, kvm, lm, g);
    return hipGetLastError();
}

template <int DP>
hipError_t run_bwd(const float* q, const float* k, const float* v, const float* out, const float* lse, const float* d_out,
                   float* delta, float* dq, float* dk, float* dv, TensorMap qm, TensorMap kvm, RowMap lm, AttnGeom g,
                   hipStream_t stream) {
    const int tiles = (g.seq_len + kLanes - 1) / kLanes;
    hipError_t err;
    {
        KernelTimer timer("dq_f32", stream);
        hipLaunchKernelGGL(bwd_dq_f32_kernel<DP>, dim3(tiles, g.q_heads, g.packs), dim3(kLanes), 0, stream, q, k, v, out, lse,
                           d_out, delta, dq, qm, kvm, lm, g);
        err = hipGetLastError();
    }
    if (err != hipSuccess) return err;

    const size_t lds = dkdv_lds_bytes<DP>();
    static bool raised = false;  // one-time opt-in to more than 64 KiB of LDS, no per-call state change
    if (!raised && lds > 64 * 1024) {
        err = hipFuncSetAttribute(reinterpret_cast<const void*>(bwd_dkdv_f32_kernel<DP>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (err != hipSuccess) return err;
        raised = true;
    }
    KernelTimer timer("dkdv_f32", stream);
    hipLaunchKernelGGL(bwd_dkdv_f32_kernel<DP>, dim3(tiles, g.kv_heads, g.packs), dim3(kLanes), lds, stream, q, k, v, lse,
                       d_out, delta, dk, dv, qm, kvm, lm, g);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_fwd_f32(const float* q, const float* k, const float* v, float* out, float* lse, TensorMap qm,
                          TensorMap kvm, RowMap lm, AttnGeom g, hipStream_t stream) {
    if (g.head_dim <= 16) return run_fwd<16>(q, k, v, out, lse, qm, kvm, lm, g, stream);
    if (g.head_dim <= 32) return run_fwd<32>(q, k, v, out, lse, qm, kvm, lm, g, stream);
    if (g.head_dim <= 64) return run_fwd<64>(q, k, v, out, lse, qm, kvm, lm, g, stream);
    return run_fwd<128>(q, k, v, out, lse, qm, kvm, lm, g, stream);
}

hipError_t launch_bwd_f32(const float* q, const float* k, const float* v, const float* out, const float* lse,
                          const float* d_out, float* dq, float* dk, float* dv, float* delta, TensorMap qm, TensorMap kvm,
                          RowMap lm, AttnGeom g, hipStream_t stream) {
    if (g.head_dim <= 16) return run_bwd<16>(q, k, v, out, lse, d_out, delta, dq, dk, dv, qm, kvm, lm, g, stream);
    if (g.head_dim <= 32) return run_bwd<32>(q, k, v, out, lse, d_out, delta, dq, dk, dv, qm, kvm, lm, g, stream);
    if (g.head_dim <= 64) return run_bwd<64>(q, k, v, out, lse, d_out, delta, dq, dk, dv, qm, kvm, lm, g, stream);
    return run_bwd<128>(q, k, v, out, lse, d_out, delta, dq, dk, dv, qm, kvm, lm, g, stream);
}

}  // namespace sentinel_hip
