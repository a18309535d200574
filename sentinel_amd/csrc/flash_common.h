// Internal declarations shared by the attention kernels and the C ABI (not installed).
#ifndef SENTINEL_HIP_FLASH_COMMON_H
#define SENTINEL_HIP_FLASH_COMMON_H

#include <hip/hip_runtime.h>

namespace sentinel_hip {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Problem geometry common to every kernel.
struct AttnGeom {
    int q_heads;
    int kv_heads;
    int head_dim;
    int seq_len;
    int packs;
    float scale;
    int causal;
    // Sentinel's sparse mask on top of the causal one (CausalSelfAttention::allowsKey,
    // sentinel/NeuralNet/Layers/CausalSelfAttention.cpp:95-100): with window > 0 a key at or past global_tokens is
    // visible only to the queries key .. key + window - 1.  window == 0: full causal (global_tokens is then 0 too).
    int window;
    int global_tokens;
};

// true when the sparse mask forbids the pair (the causal rule key <= query is checked separately)
__host__ __device__ inline bool outside_window(const AttnGeom& g, int query, int key) {
    return g.window > 0 && key >= g.global_tokens && query - key >= g.window;
}

// element(pack, head, t, c) = base[pack * pack_stride + head * head_stride + t * t_stride + c * c_stride]
// Sentinel's column layout: pack_stride = seq_len, head_stride = head_dim * stride_columns, t_stride = 1,
// c_stride = stride_columns (base already advanced by column_start).
// [B,H,T,d]: pack_stride = heads * T * d, head_stride = T * d, t_stride = d, c_stride = 1.
struct TensorMap {
    long long pack_stride;
    long long head_stride;
    long long t_stride;
    long long c_stride;
};

// row(pack, head, t) = base[pack * pack_stride + head * head_stride + t]   (lse, delta)
struct RowMap {
    long long pack_stride;
    long long head_stride;
};

enum class Elem : int { F32 = 0, BF16 = 1, F16 = 2 };

// ---- fp32 FMA path (flash_fp32.hip): any head_dim <= 128, any layout ----
hipError_t launch_fwd_f32(const float* q, const float* k, const float* v, float* out, float* lse, TensorMap qm,
                          TensorMap kvm, RowMap lm, AttnGeom g, hipStream_t stream);
hipError_t launch_bwd_f32(const float* q, const float* k, const float* v, const float* out, const float* lse,
                          const float* d_out, float* dq, float* dk, float* dv, float* delta, TensorMap qm, TensorMap kvm,
                          RowMap lm, AttnGeom g, hipStream_t stream);

// Rotary embedding tables [positions][head_dim / 2] (cos == nullptr: no rotation); token t of a pack uses
// table row offset + t.
struct RopeTables {
    const float* cos;
    const float* sin;
    int offset;
    int positions;  // rows of each table
};

// A result tensor in Sentinel's column layout, fp32 [(head * head_dim + dim), column], for the MFMA kernels to write
// straight from their accumulators (base == nullptr: none).  The kernels hold results transposed, one head dim of 32
// consecutive tokens per register, which is 128 contiguous bytes of a row of that matrix: no conversion pass is
// needed on the way out.  `base` is already advanced to the first column of pack 0; pack p starts seq_len columns on.
// `inverse_rope`: the rotary embedding's inverse applied on the way (dQ, dK), as bhtd_to_columns does.
// `head_dim`: rows per head of that matrix (a multiple of 8); where it is smaller than the kernels' own head dim (operands
// zero-padded to the next tiling, see launch_columns_to_bhtd_jobs) only that many head dims are written.
struct ColumnSink {
    float* base;
    long long stride;  // columns per row
    RopeTables inverse_rope;
    int head_dim;
};
constexpr ColumnSink kNoColumnSink = {nullptr, 0, {nullptr, nullptr, 0, 0}, 0};

// ---- MFMA path (flash_mfma_*.hip): bf16 / fp16 [B,H,T,d] tensors, head_dim 64 or 128 ----
bool mfma_supported(int head_dim);
// the tiling a head dim is zero-padded to when it has none of its own (multiples of 8 up to 128), 0 if there is none
inline int mfma_padded_head_dim(int head_dim) {
    if (head_dim <= 0 || head_dim > 128 || head_dim % 8 != 0) return 0;
    return head_dim <= 64 ? 64 : 128;
}
// lse rows are addressed through `lm`; delta is q_heads x (packs * seq_len).
// out_columns: O is written there as well (the 16-bit `out` is always written: the backward reads it)
hipError_t launch_fwd_mfma(Elem type, const void* q, const void* k, const void* v, void* out, float* lse, RowMap lm,
                           AttnGeom g, hipStream_t stream, ColumnSink out_columns = kNoColumnSink);
// dq_columns / dk_columns / dv_columns: where given, that gradient goes there instead of to its 16-bit tensor (which may
// then be nullptr).
hipError_t launch_bwd_mfma(Elem type, const void* q, const void* k, const void* v, const void* out, const float* lse,
                           RowMap lm, const void* d_out, void* dq, void* dk, void* dv, float* delta, AttnGeom g,
                           hipStream_t stream, ColumnSink dq_columns = kNoColumnSink,
                           ColumnSink dk_columns = kNoColumnSink, ColumnSink dv_columns = kNoColumnSink);

// ---- layout adapter (layout_adapter.hip): Sentinel column layout fp32 <-> [B,H,T,d] bf16 / fp16 ----
// several tensors of one shape family (same head_dim, stride, sequence length, packs; head counts may differ) through one
// launch; `rotate`: apply the rotary tables to this tensor; z_end is filled in by the launcher.  padded_dim (0: head_dim):
// head dims per token on the 16-bit side, the ones from head_dim on are zeros (written / skipped)
constexpr int kMaxConvertJobs = 5;
struct ConvertJob {
    const float* src;     // first column of pack 0
    unsigned short* dst;  // [packs, heads, seq_len, head_dim]
    int heads;
    int rotate;
    int z_end;
};
struct ConvertJobs {
    ConvertJob job[kMaxConvertJobs];
    int count;
};
hipError_t launch_columns_to_bhtd_jobs(Elem type, ConvertJobs jobs, int head_dim, int stride_columns, int seq_len, int packs,
                                       RopeTables rope, hipStream_t stream, int padded_dim = 0);
hipError_t launch_columns_to_bhtd(Elem type, const float* src, void* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, RopeTables rope, hipStream_t stream, int padded_dim = 0);
hipError_t launch_bhtd_to_columns(Elem type, const void* src, float* dst, int heads, int head_dim, int stride_columns,
                                  int seq_len, int packs, RopeTables inverse_rope, hipStream_t stream, int padded_dim = 0);
// flat cast of `count` fp32 values to bf16 / fp16, round to nearest even (operands of the layer's mixed-precision GEMMs)
hipError_t launch_cast_f32_to_16bit(Elem type, const float* src, void* dst, size_t count, hipStream_t stream);
// single-query attention against the K/V cache (fp32 column layout, `stride` positions per row, `length` used)
size_t decode_workspace_bytes(int q_heads, int head_dim, int length);
// window / global_tokens: the layer's sparse mask for the query at position length - 1 (window <= 0: none)
hipError_t launch_decode_attention(const float* query, const float* key_cache, const float* value_cache, float* out,
                                   int q_heads, int kv_heads, int head_dim, int stride, int length, float scale,
                                   int window, int global_tokens, float* workspace, hipStream_t stream);
// size of the file-scope device array behind the allocation-free decode entry point, and its address on the current
// device (looked up once per device)
constexpr size_t kDecodeStaticScratchBytes = 4u << 20;
hipError_t decode_static_scratch_address(float** address);
// in-place rotation of fp32 column-layout rows (tensor already advanced to the first column)
hipError_t launch_rope_rotate_f32(float* tensor, int heads, int head_dim, int stride_columns, int columns,
                                  int position_offset, int segment_length, const float* cos, const float* sin, bool inverse,
                                  hipStream_t stream);

// ---- dense (materialising) path of the layer (dense_softmax.hip): keys x queries fp32 score matrices ----
// in place: P = softmax over keys of (scale * S, forbidden pairs at -1e9); matrix b starts at scores + b * batch_stride
hipError_t launch_dense_softmax_fwd(float* scores, int batch, long long batch_stride, int key_count, int query_count,
                                    int query_position_start, int window, int global_tokens, int segment_length, float scale,
                                    hipStream_t stream);
// in place over gradient: dS = scale * P * (dP - sum_keys dP * P), zero on forbidden pairs
hipError_t launch_dense_softmax_bwd(const float* probabilities, long long probability_batch_stride, float* gradient,
                                    long long gradient_batch_stride, int batch, int key_count, int query_count,
                                    int query_position_start, int window, int global_tokens, int segment_length, float scale,
                                    hipStream_t stream);

// ---- optional per-kernel hipEvent timing (kernel_timing.hip) ----
class KernelTimer {
public:
    KernelTimer(const char* name, hipStream_t stream);
    ~KernelTimer();
    KernelTimer(const KernelTimer&) = delete;
    KernelTimer& operator=(const KernelTimer&) = delete;

private:
    const char* name_;
    hipStream_t stream_;
    hipEvent_t start_;
};
int timing_set_enabled(int enabled);
int timing_collect(const char** names, float* total_ms, int* launches, int capacity);

}  // namespace sentinel_hip
#endif
