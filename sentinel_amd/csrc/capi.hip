// C ABI of the attention library: argument validation, layout resolution and kernel dispatch.
// Validation follows CudaFlashAttention's host code (sentinel/NeuralNet/Cuda/CudaFlashAttention.cu:
// validateMultiHeadShape :1458-1471, resolveColumnWindow :1533-1539, pack window :1551-1552,
// device check :1545-1546) with return codes in place of exceptions.
#include "../../include/sentinel_hip_attn.h"

#include "flash_common.h"

#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

using namespace sentinel_hip;

namespace {

thread_local char g_last_error[256] = "";

int fail(int code, const char* fmt, ...) {
    va_list args;
    va_start(args, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, args);
    va_end(args);
    return code;
}

int fail_hip(const char* what, hipError_t err) {
    return fail(SENTINEL_HIP_RUNTIME, "%s: %s", what, hipGetErrorString(err));
}

size_t align_up(size_t x) { return (x + 255) & ~static_cast<size_t>(255); }

struct Resolved {
    AttnGeom g;
    int io;        // SENTINEL_HIP_F32 / BF16 / F16
    int compute;   // resolved compute type
    int layout;
    long long stride;  // column layout only
    int column_start;
    bool adapter;  // column layout fp32 tensors converted to [B,H,T,d] 16-bit for the MFMA kernels
    int source_dim;  // the caller's head dim; g.head_dim is larger when the conversion pads it to a tiling the MFMA kernels have
    bool keep;     // forward: lay the converted operands out where the backward expects them (SENTINEL_HIP_WORKSPACE_KEEP)
    bool reuse;    // backward: q, k, v, out of the workspace are the forward's (SENTINEL_HIP_WORKSPACE_REUSE)
};

// Geometry checks shared by both entry points. `op` names the operation in messages.
int resolve(const char* op, int io_dtype, int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
            int stride_columns, int column_start, int seq_len, int pack_count, float scale, int causal, Resolved* r) {
    if (io_dtype < SENTINEL_HIP_F32 || io_dtype > SENTINEL_HIP_F16) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s unknown io dtype %d", op, io_dtype);
    if (compute_dtype < SENTINEL_HIP_COMPUTE_AUTO || compute_dtype > SENTINEL_HIP_COMPUTE_F16)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s unknown compute dtype %d", op, compute_dtype);
    constexpr int kFlags = SENTINEL_HIP_WORKSPACE_KEEP | SENTINEL_HIP_WORKSPACE_REUSE;
    const int workspace_flags = layout & kFlags;
    layout &= ~kFlags;
    if (layout != SENTINEL_HIP_LAYOUT_COLUMNS && layout != SENTINEL_HIP_LAYOUT_BHTD)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s unknown layout %d", op, layout);
    if (q_heads <= 0 || head_dim <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s invalid head geometry", op);
    if (kv_heads <= 0) kv_heads = q_heads;
    if (q_heads % kv_heads != 0)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s headCount must be divisible by kvHeadCount", op);
    if (head_dim > sentinel_hip_flash_max_head_dim())
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s headDim exceeds maxHeadDimension", op);
    if (pack_count <= 0) pack_count = 1;
    if (layout == SENTINEL_HIP_LAYOUT_COLUMNS) {
        if (stride_columns <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty input", op);
        if (seq_len <= 0) seq_len = stride_columns - column_start;  // resolveColumnWindow
        if (column_start < 0 || seq_len <= 0 || (long long)column_start + seq_len > stride_columns)
            return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s invalid column window", op);
        if ((long long)column_start + (long long)pack_count * seq_len > stride_columns)
            return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s pack window exceeds columns", op);
    } else {
        if (seq_len <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty input", op);
        stride_columns = 0;
        column_start = 0;
    }
    if (!(scale > 0.0f) || !std::isfinite(scale))
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s scale must be positive and finite", op);

    int compute = compute_dtype;
    if (compute == SENTINEL_HIP_COMPUTE_AUTO) compute = io_dtype;
    bool adapter = false;
    if (compute == SENTINEL_HIP_COMPUTE_F32) {
        if (io_dtype != SENTINEL_HIP_F32)
            return fail(SENTINEL_HIP_UNSUPPORTED, "%s fp32 arithmetic needs fp32 tensors", op);
    } else {
        if (io_dtype == SENTINEL_HIP_F32) {
            if (layout != SENTINEL_HIP_LAYOUT_COLUMNS)
                return fail(SENTINEL_HIP_UNSUPPORTED, "%s fp32 tensors with MFMA arithmetic need the column layout", op);
            // the conversion pass pads head dims without a tiling of their own with zeros (no product changes)
            if (mfma_padded_head_dim(head_dim) == 0)
                return fail(SENTINEL_HIP_UNSUPPORTED, "%s MFMA arithmetic needs a head_dim that is a multiple of 8, got %d", op, head_dim);
            adapter = true;
        } else {
            if (!mfma_supported(head_dim))
                return fail(SENTINEL_HIP_UNSUPPORTED, "%s 16-bit tensors: the MFMA kernels cover head_dim 64 and 128, got %d", op, head_dim);
            if (io_dtype != compute)
                return fail(SENTINEL_HIP_UNSUPPORTED, "%s 16-bit tensors must be multiplied in their own type", op);
            if (layout != SENTINEL_HIP_LAYOUT_BHTD)
                return fail(SENTINEL_HIP_UNSUPPORTED, "%s 16-bit tensors need the [B,H,T,d] layout", op);
        }
    }
    // every kernel indexes one tensor with 64-bit offsets but tiles with int
    if ((long long)pack_count * seq_len > 0x7fffffffLL / 4)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s too many columns", op);
    if (compute != SENTINEL_HIP_COMPUTE_F32) {
        // the MFMA kernels address one head through a 32-bit buffer range and int byte offsets inside it
        if ((long long)seq_len * (adapter ? mfma_padded_head_dim(head_dim) : head_dim) * 2 > 0x7fffffffLL)
            return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s one head exceeds 2 GiB (seq_len * head_dim * 2 bytes)", op);
        // the layout conversion launches one grid plane per (pack, head)
        if (adapter && (long long)pack_count * q_heads > 65535)
            return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s more than 65535 (pack, head) pairs in the column layout", op);
    }

    r->source_dim = head_dim;
    if (adapter) head_dim = mfma_padded_head_dim(head_dim);
    r->g = AttnGeom{q_heads, kv_heads, head_dim, seq_len, pack_count, scale, causal ? 1 : 0, 0, 0};
    r->io = io_dtype;
    r->compute = compute;
    r->layout = layout;
    r->stride = stride_columns;
    r->column_start = column_start;
    r->adapter = adapter;
    // without a conversion pass there is nothing to keep: the flags are then accepted and mean nothing
    r->keep = adapter && (workspace_flags & SENTINEL_HIP_WORKSPACE_KEEP);
    r->reuse = adapter && (workspace_flags & SENTINEL_HIP_WORKSPACE_REUSE);
    return SENTINEL_HIP_OK;
}

TensorMap tensor_map(const Resolved& r, int heads) {
    if (r.layout == SENTINEL_HIP_LAYOUT_COLUMNS)
        return TensorMap{r.g.seq_len, (long long)r.g.head_dim * r.stride, 1, r.stride};
    return TensorMap{(long long)heads * r.g.seq_len * r.g.head_dim, (long long)r.g.seq_len * r.g.head_dim, r.g.head_dim, 1};
}

RowMap lse_map(const Resolved& r) {
    if (r.layout == SENTINEL_HIP_LAYOUT_COLUMNS) return RowMap{r.g.seq_len, r.stride};
    return RowMap{(long long)r.g.q_heads * r.g.seq_len, r.g.seq_len};
}

bool misaligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

size_t q_bytes16(const AttnGeom& g) { return align_up((size_t)g.packs * g.q_heads * g.seq_len * g.head_dim * 2); }
size_t kv_bytes16(const AttnGeom& g) { return align_up((size_t)g.packs * g.kv_heads * g.seq_len * g.head_dim * 2); }

// 16-bit copies of the column-layout tensors (adapter)
size_t conversion_bytes(const Resolved& r, bool backward) {
    if (!r.adapter) return 0;
    const size_t nq = q_bytes16(r.g);
    const size_t nkv = kv_bytes16(r.g);
    return backward ? 4 * nq + 4 * nkv : 2 * nq + 2 * nkv;
}
// The kernels write fp32 column matrices with 32-bit byte offsets inside a head's rows: head_dim rows must span less
// than 2 GiB (and likewise the rotary tables, which resolve_rope has bounded).
bool direct_columns(const Resolved& r) { return (long long)r.g.head_dim * r.stride * 4 < 0x7fffffffLL; }

size_t workspace_need(const Resolved& r, bool backward) { return conversion_bytes(r, backward); }

}  // namespace

extern "C" int sentinel_hip_flash_max_head_dim(void) { return 128; }

extern "C" int sentinel_hip_device_available(void) {
    // asked once per process: the answer cannot change under a running program, and a runtime query on every
    // forward / backward call is host work on the launch path
    static const int available = [] {
        int count = 0;
        if (hipGetDeviceCount(&count) != hipSuccess) {
            (void)hipGetLastError();
            return 0;
        }
        return count > 0 ? 1 : 0;
    }();
    return available;
}

extern "C" const char* sentinel_hip_strerror(int code) {
    switch (code) {
        case SENTINEL_HIP_OK: return "ok";
        case SENTINEL_HIP_INVALID_ARGUMENT: return "invalid argument";
        case SENTINEL_HIP_UNSUPPORTED: return "unsupported configuration";
        case SENTINEL_HIP_RUNTIME: return "HIP runtime failure";
        default: return "unknown code";
    }
}

extern "C" const char* sentinel_hip_last_error(void) { return g_last_error; }

extern "C" int sentinel_hip_flash_set_timing(int enabled) { return timing_set_enabled(enabled); }

extern "C" int sentinel_hip_flash_collect_timings(const char** names_out, float* total_ms_out, int* launches_out,
                                                  int capacity) {
    if (!names_out || !total_ms_out || !launches_out || capacity <= 0) return 0;
    return timing_collect(names_out, total_ms_out, launches_out, capacity);
}

extern "C" size_t sentinel_hip_flash_workspace_bytes(int io_dtype, int compute_dtype, int layout, int q_heads, int kv_heads,
                                                     int head_dim, int seq_len, int pack_count, int backward) {
    Resolved r;
    // stride / window are irrelevant to the size: use a window that always validates
    const int packs = pack_count <= 0 ? 1 : pack_count;
    if (seq_len <= 0) return 0;
    if ((long long)packs * seq_len > 0x7fffffffLL / 4) return 0;
    if (resolve("sentinel_hip_flash_workspace_bytes", io_dtype, compute_dtype, layout, q_heads, kv_heads, head_dim,
                packs * seq_len, 0, seq_len, packs, 1.0f, 1, &r) != SENTINEL_HIP_OK)
        return 0;
    return workspace_need(r, backward != 0);
}

namespace {

// Checks of the rotary tables shared by the fused entry points and sentinel_hip_rope_rotate; messages follow
// CudaOps::rotaryRotateInPlace (Cuda/CudaOps.cu:1319-1330).
int check_rope(const char* op, const float* cos_table, const float* sin_table, int table_positions, int head_dim,
               int position_offset, int positions_needed) {
    if (!cos_table || !sin_table || table_positions <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty tables", op);
    if (head_dim <= 0 || head_dim % 2 != 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s invalid rope dims", op);
    if (position_offset < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s negative positionOffset", op);
    if ((long long)position_offset + positions_needed > table_positions)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s position exceeds RoPE table", op);
    return SENTINEL_HIP_OK;
}

// Rotary tables as handed in by the caller; validated against the RESOLVED sequence length (seq_len <= 0 means "the
// rest of the window" in the column layout), never against the raw argument.
struct RopeRequest {
    const float* cos;
    const float* sin;
    int table_positions;
    int position_offset;
    bool requested;
};
const RopeRequest kNoRope = {nullptr, nullptr, 0, 0, false};

int resolve_rope(const char* op, const RopeRequest& req, const Resolved& r, RopeTables* rope) {
    *rope = RopeTables{nullptr, nullptr, 0, 0};
    if (!req.requested) return SENTINEL_HIP_OK;
    const int rc = check_rope(op, req.cos, req.sin, req.table_positions, r.source_dim, req.position_offset, r.g.seq_len);
    if (rc != SENTINEL_HIP_OK) return rc;
    if (misaligned(req.cos) || misaligned(req.sin))
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s rope tables must be 16-byte aligned", op);
    if (!r.adapter)
        return fail(SENTINEL_HIP_UNSUPPORTED,
                    "%s the rotation is fused into the layout conversion of fp32 column tensors with 16-bit arithmetic; "
                    "rotate other tensors with sentinel_hip_rope_rotate",
                    op);
    *rope = RopeTables{req.cos, req.sin, req.position_offset, req.table_positions};
    return SENTINEL_HIP_OK;
}

// The layer's sparse mask (windowSize, globalTokenCount).  A window that covers the sequence is no window, and
// without a window the global tokens change nothing: both collapse to the plain causal mask.
struct SparseMask {
    int window;
    int global_tokens;
};
const SparseMask kNoSparseMask = {0, 0};

int apply_sparse_mask(const char* op, SparseMask mask, AttnGeom* g) {
    if (mask.global_tokens < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s globalTokenCount must be >= 0", op);
    if (mask.window <= 0 || mask.window >= g->seq_len) return SENTINEL_HIP_OK;
    if (!g->causal) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s the sliding window refines the causal mask: causal must be set", op);
    g->window = mask.window;
    g->global_tokens = mask.global_tokens < g->seq_len ? mask.global_tokens : g->seq_len;
    return SENTINEL_HIP_OK;
}

int flash_fwd(const char* op, const void* q, const void* k, const void* v, void* out, float* lse, int io_dtype,
              int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim, int stride_columns, int column_start,
              int seq_len, int pack_count, float scale, int causal, void* workspace, size_t workspace_bytes,
              void* stream_ptr, const RopeRequest& rope_request, SparseMask mask = kNoSparseMask) {
    if (!q || !k || !v || !out || !lse) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty input", op);
    Resolved r;
    const int rc = resolve(op, io_dtype, compute_dtype, layout, q_heads, kv_heads, head_dim, stride_columns, column_start,
                           seq_len, pack_count, scale, causal, &r);
    if (rc != SENTINEL_HIP_OK) return rc;
    const int mask_rc = apply_sparse_mask(op, mask, &r.g);
    if (mask_rc != SENTINEL_HIP_OK) return mask_rc;
    RopeTables rope;
    const int rope_rc = resolve_rope(op, rope_request, r, &rope);
    if (rope_rc != SENTINEL_HIP_OK) return rope_rc;
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
    const AttnGeom& g = r.g;

    if (r.compute == SENTINEL_HIP_COMPUTE_F32) {
        const long long off = r.column_start;
        const hipError_t err = launch_fwd_f32(static_cast<const float*>(q) + off, static_cast<const float*>(k) + off,
                                              static_cast<const float*>(v) + off, static_cast<float*>(out) + off, lse + off,
                                              tensor_map(r, g.q_heads), tensor_map(r, g.kv_heads), lse_map(r), g, stream);
        if (err != hipSuccess) return fail_hip("fp32 forward launch", err);
        return SENTINEL_HIP_OK;
    }

    const Elem type = static_cast<Elem>(r.compute);
    if (!r.adapter) {
        if (misaligned(q) || misaligned(k) || misaligned(v) || misaligned(out))
            return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s 16-bit tensors must be 16-byte aligned", op);
        const hipError_t err = launch_fwd_mfma(type, q, k, v, out, lse, lse_map(r), g, stream);
        if (err != hipSuccess) return fail_hip("MFMA forward launch", err);
        return SENTINEL_HIP_OK;
    }

    // column-layout fp32 tensors: convert operands, run the MFMA kernel, convert the result back
    // SENTINEL_HIP_WORKSPACE_KEEP: the workspace is the backward's, and q, out, k, v go where the backward looks for them
    const size_t need = workspace_need(r, r.keep);
    if (!workspace || workspace_bytes < need || misaligned(workspace))
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s needs %zu bytes of 16-byte aligned workspace", op, need);
    char* ws = static_cast<char*>(workspace);
    void* q16 = ws;
    void* o16 = ws + q_bytes16(g);
    void* k16 = ws + (r.keep ? 4 : 2) * q_bytes16(g);
    void* v16 = static_cast<char*>(k16) + kv_bytes16(g);
    const long long off = r.column_start;
    const int stride = static_cast<int>(r.stride);
    const RopeTables none = {nullptr, nullptr, 0, 0};
    // Q, K (rotated where the call rotates) and V in one launch
    ConvertJobs in;
    in.count = 3;
    in.job[0] = ConvertJob{static_cast<const float*>(q) + off, static_cast<unsigned short*>(q16), g.q_heads, 1, 0};
    in.job[1] = ConvertJob{static_cast<const float*>(k) + off, static_cast<unsigned short*>(k16), g.kv_heads, 1, 0};
    in.job[2] = ConvertJob{static_cast<const float*>(v) + off, static_cast<unsigned short*>(v16), g.kv_heads, 0, 0};
    hipError_t err = launch_columns_to_bhtd_jobs(type, in, r.source_dim, stride, g.seq_len, g.packs, rope, stream, g.head_dim);
    // O goes to the caller's matrix straight from the kernel's accumulators (and in 16 bit to the workspace, for the
    // backward); a conversion pass only where the kernel's 32-bit row offsets would not reach
    const bool direct = direct_columns(r);
    if (err == hipSuccess)
        err = launch_fwd_mfma(type, q16, k16, v16, o16, lse + off, lse_map(r), g, stream,
                              direct ? ColumnSink{static_cast<float*>(out) + off, r.stride, none, r.source_dim} : kNoColumnSink);
    if (err == hipSuccess && !direct)
        err = launch_bhtd_to_columns(type, o16, static_cast<float*>(out) + off, g.q_heads, r.source_dim, stride, g.seq_len,
                                     g.packs, none, stream, g.head_dim);
    if (err != hipSuccess) return fail_hip("MFMA forward (column layout) launch", err);
    return SENTINEL_HIP_OK;
}


int flash_bwd(const char* op, const void* q, const void* k, const void* v, const void* out, const float* lse,
              const void* d_out, void* dq, void* dk, void* dv, float* delta, int io_dtype, int compute_dtype, int layout,
              int q_heads, int kv_heads, int head_dim, int stride_columns, int column_start, int seq_len, int pack_count,
              float scale, int causal, void* workspace, size_t workspace_bytes, void* stream_ptr,
              const RopeRequest& rope_request, SparseMask mask = kNoSparseMask) {
    if (!q || !k || !v || !out || !lse || !d_out || !dq || !dk || !dv || !delta)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty input", op);
    Resolved r;
    const int rc = resolve(op, io_dtype, compute_dtype, layout, q_heads, kv_heads, head_dim, stride_columns, column_start,
                           seq_len, pack_count, scale, causal, &r);
    if (rc != SENTINEL_HIP_OK) return rc;
    const int mask_rc = apply_sparse_mask(op, mask, &r.g);
    if (mask_rc != SENTINEL_HIP_OK) return mask_rc;
    RopeTables rope;
    const int rope_rc = resolve_rope(op, rope_request, r, &rope);
    if (rope_rc != SENTINEL_HIP_OK) return rope_rc;
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    hipStream_t stream = static_cast<hipStream_t>(stream_ptr);
    const AttnGeom& g = r.g;

    if (r.compute == SENTINEL_HIP_COMPUTE_F32) {
        const long long off = r.column_start;
        const hipError_t err = launch_bwd_f32(
            static_cast<const float*>(q) + off, static_cast<const float*>(k) + off, static_cast<const float*>(v) + off,
            static_cast<const float*>(out) + off, lse + off, static_cast<const float*>(d_out) + off,
            static_cast<float*>(dq) + off, static_cast<float*>(dk) + off, static_cast<float*>(dv) + off, delta,
            tensor_map(r, g.q_heads), tensor_map(r, g.kv_heads), lse_map(r), g, stream);
        if (err != hipSuccess) return fail_hip("fp32 backward launch", err);
        return SENTINEL_HIP_OK;
    }

    const Elem type = static_cast<Elem>(r.compute);
    if (!r.adapter) {
        if (misaligned(q) || misaligned(k) || misaligned(v) || misaligned(out) || misaligned(d_out) || misaligned(dq) ||
            misaligned(dk) || misaligned(dv))
            return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s 16-bit tensors must be 16-byte aligned", op);
        const hipError_t err = launch_bwd_mfma(type, q, k, v, out, lse, lse_map(r), d_out, dq, dk, dv, delta, g, stream);
        if (err != hipSuccess) return fail_hip("MFMA backward launch", err);
        return SENTINEL_HIP_OK;
    }

    const size_t need = workspace_need(r, true);
    if (!workspace || workspace_bytes < need || misaligned(workspace))
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s needs %zu bytes of 16-byte aligned workspace", op, need);
    char* ws = static_cast<char*>(workspace);
    const size_t nq = q_bytes16(g);
    const size_t nkv = kv_bytes16(g);
    void* q16 = ws;
    void* o16 = ws + nq;
    void* g16 = ws + 2 * nq;
    void* dq16 = ws + 3 * nq;
    void* k16 = ws + 4 * nq;
    void* v16 = ws + 4 * nq + nkv;
    void* dk16 = ws + 4 * nq + 2 * nkv;
    void* dv16 = ws + 4 * nq + 3 * nkv;
    const long long off = r.column_start;
    const int stride = static_cast<int>(r.stride);
    const int T = g.seq_len;
    const RopeTables none = {nullptr, nullptr, 0, 0};
    // SENTINEL_HIP_WORKSPACE_REUSE: q16, o16, k16, v16 are still the ones the forward call left there (rotated Q, K and
    // the 16-bit O the kernel itself wrote, which is the O that D = rowsum(dO o O) should be formed from anyway)
    // one launch converts dO and, unless the forward call left them, Q, K (rotated where the call rotates), V and O
    ConvertJobs in;
    in.count = 0;
    in.job[in.count++] = ConvertJob{static_cast<const float*>(d_out) + off, static_cast<unsigned short*>(g16), g.q_heads, 0, 0};
    if (!r.reuse) {
        in.job[in.count++] = ConvertJob{static_cast<const float*>(q) + off, static_cast<unsigned short*>(q16), g.q_heads, 1, 0};
        in.job[in.count++] = ConvertJob{static_cast<const float*>(out) + off, static_cast<unsigned short*>(o16), g.q_heads, 0, 0};
        in.job[in.count++] = ConvertJob{static_cast<const float*>(k) + off, static_cast<unsigned short*>(k16), g.kv_heads, 1, 0};
        in.job[in.count++] = ConvertJob{static_cast<const float*>(v) + off, static_cast<unsigned short*>(v16), g.kv_heads, 0, 0};
    }
    hipError_t err = launch_columns_to_bhtd_jobs(type, in, r.source_dim, stride, T, g.packs, rope, stream, g.head_dim);
    // The gradients leave the kernels as fp32 columns, straight from the accumulators, rotated back on the way (they are
    // gradients with respect to the unrotated Q, K).  Matrices beyond the kernels' 32-bit row offsets write 16-bit
    // tensors and convert them in passes of their own.
    if (direct_columns(r)) {
        if (err == hipSuccess)
            err = launch_bwd_mfma(type, q16, k16, v16, o16, lse + off, lse_map(r), g16, dq16, dk16, dv16, delta, g, stream,
                                  ColumnSink{static_cast<float*>(dq) + off, r.stride, rope, r.source_dim},
                                  ColumnSink{static_cast<float*>(dk) + off, r.stride, rope, r.source_dim},
                                  ColumnSink{static_cast<float*>(dv) + off, r.stride, none, r.source_dim});
        if (err != hipSuccess) return fail_hip("MFMA backward (column layout) launch", err);
        return SENTINEL_HIP_OK;
    }
    if (err == hipSuccess)
        err = launch_bwd_mfma(type, q16, k16, v16, o16, lse + off, lse_map(r), g16, dq16, dk16, dv16, delta, g, stream);
    if (err == hipSuccess)
        err = launch_bhtd_to_columns(type, dq16, static_cast<float*>(dq) + off, g.q_heads, r.source_dim, stride, T, g.packs,
                                     rope, stream, g.head_dim);
    if (err == hipSuccess)
        err = launch_bhtd_to_columns(type, dk16, static_cast<float*>(dk) + off, g.kv_heads, r.source_dim, stride, T, g.packs,
                                     rope, stream, g.head_dim);
    if (err == hipSuccess)
        err = launch_bhtd_to_columns(type, dv16, static_cast<float*>(dv) + off, g.kv_heads, r.source_dim, stride, T, g.packs,
                                     none, stream, g.head_dim);
    if (err != hipSuccess) return fail_hip("MFMA backward (column layout) launch", err);
    return SENTINEL_HIP_OK;
}

}  // namespace

extern "C" int sentinel_hip_flash_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int io_dtype,
                                      int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                      int stride_columns, int column_start, int seq_len, int pack_count, float scale,
                                      int causal, void* workspace, size_t workspace_bytes, void* stream_ptr) {
    return flash_fwd("sentinel_hip_flash_fwd", q, k, v, out, lse, io_dtype, compute_dtype, layout, q_heads, kv_heads,
                     head_dim, stride_columns, column_start, seq_len, pack_count, scale, causal, workspace, workspace_bytes,
                     stream_ptr, kNoRope);
}

extern "C" int sentinel_hip_flash_bwd(const void* q, const void* k, const void* v, const void* out, const float* lse,
                                      const void* d_out, void* dq, void* dk, void* dv, float* delta, int io_dtype,
                                      int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                      int stride_columns, int column_start, int seq_len, int pack_count, float scale,
                                      int causal, void* workspace, size_t workspace_bytes, void* stream_ptr) {
    return flash_bwd("sentinel_hip_flash_bwd", q, k, v, out, lse, d_out, dq, dk, dv, delta, io_dtype, compute_dtype, layout,
                     q_heads, kv_heads, head_dim, stride_columns, column_start, seq_len, pack_count, scale, causal,
                     workspace, workspace_bytes, stream_ptr, kNoRope);
}

extern "C" int sentinel_hip_flash_fwd_rope(const void* q, const void* k, const void* v, void* out, float* lse,
                                           const float* cos_table, const float* sin_table, int table_positions,
                                           int position_offset, int io_dtype, int compute_dtype, int layout, int q_heads,
                                           int kv_heads, int head_dim, int stride_columns, int column_start, int seq_len,
                                           int pack_count, float scale, int causal, void* workspace,
                                           size_t workspace_bytes, void* stream_ptr) {
    const RopeRequest rope = {cos_table, sin_table, table_positions, position_offset, true};
    return flash_fwd("sentinel_hip_flash_fwd_rope", q, k, v, out, lse, io_dtype, compute_dtype, layout, q_heads, kv_heads,
                     head_dim, stride_columns, column_start, seq_len, pack_count, scale, causal, workspace, workspace_bytes,
                     stream_ptr, rope);
}

extern "C" int sentinel_hip_flash_bwd_rope(const void* q, const void* k, const void* v, const void* out, const float* lse,
                                           const void* d_out, void* dq, void* dk, void* dv, float* delta,
                                           const float* cos_table, const float* sin_table, int table_positions,
                                           int position_offset, int io_dtype, int compute_dtype, int layout, int q_heads,
                                           int kv_heads, int head_dim, int stride_columns, int column_start, int seq_len,
                                           int pack_count, float scale, int causal, void* workspace,
                                           size_t workspace_bytes, void* stream_ptr) {
    const RopeRequest rope = {cos_table, sin_table, table_positions, position_offset, true};
    return flash_bwd("sentinel_hip_flash_bwd_rope", q, k, v, out, lse, d_out, dq, dk, dv, delta, io_dtype, compute_dtype,
                     layout, q_heads, kv_heads, head_dim, stride_columns, column_start, seq_len, pack_count, scale, causal,
                     workspace, workspace_bytes, stream_ptr, rope);
}

extern "C" int sentinel_hip_flash_fwd_sparse(const void* q, const void* k, const void* v, void* out, float* lse,
                                             const float* cos_table, const float* sin_table, int table_positions,
                                             int position_offset, int window_size, int global_token_count, int io_dtype,
                                             int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                             int stride_columns, int column_start, int seq_len, int pack_count, float scale,
                                             int causal, void* workspace, size_t workspace_bytes, void* stream_ptr) {
    // both tables NULL: no rotation; one without the other is reported as "empty tables"
    const RopeRequest rope = {cos_table, sin_table, table_positions, position_offset, cos_table || sin_table};
    return flash_fwd("sentinel_hip_flash_fwd_sparse", q, k, v, out, lse, io_dtype, compute_dtype, layout, q_heads, kv_heads,
                     head_dim, stride_columns, column_start, seq_len, pack_count, scale, causal, workspace, workspace_bytes,
                     stream_ptr, rope, SparseMask{window_size, global_token_count});
}

extern "C" int sentinel_hip_flash_bwd_sparse(const void* q, const void* k, const void* v, const void* out, const float* lse,
                                             const void* d_out, void* dq, void* dk, void* dv, float* delta,
                                             const float* cos_table, const float* sin_table, int table_positions,
                                             int position_offset, int window_size, int global_token_count, int io_dtype,
                                             int compute_dtype, int layout, int q_heads, int kv_heads, int head_dim,
                                             int stride_columns, int column_start, int seq_len, int pack_count, float scale,
                                             int causal, void* workspace, size_t workspace_bytes, void* stream_ptr) {
    const RopeRequest rope = {cos_table, sin_table, table_positions, position_offset, cos_table || sin_table};
    return flash_bwd("sentinel_hip_flash_bwd_sparse", q, k, v, out, lse, d_out, dq, dk, dv, delta, io_dtype, compute_dtype,
                     layout, q_heads, kv_heads, head_dim, stride_columns, column_start, seq_len, pack_count, scale, causal,
                     workspace, workspace_bytes, stream_ptr, rope, SparseMask{window_size, global_token_count});
}

extern "C" int sentinel_hip_rope_rotate(float* tensor, int heads, int head_dim, int stride_columns, int column_start,
                                        int columns, int position_offset, int segment_length, const float* cos_table,
                                        const float* sin_table, int table_positions, int inverse, void* stream_ptr) {
    const char* op = inverse ? "sentinel_hip_rope_rotate (inverse)" : "sentinel_hip_rope_rotate";
    if (!tensor) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty tensor", op);
    if (heads <= 0 || head_dim <= 0 || head_dim % 2 != 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s invalid rope dims", op);
    if (columns <= 0 || column_start < 0 || (long long)column_start + columns > stride_columns)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s column window outside the matrix", op);
    if (segment_length < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s segmentLength must be >= 0", op);
    if (segment_length > 0 && segment_length > table_positions)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s segmentLength exceeds RoPE table", op);
    const int rc = check_rope(op, cos_table, sin_table, table_positions, head_dim, segment_length > 0 ? 0 : position_offset,
                              segment_length > 0 ? segment_length : columns);
    if (rc != SENTINEL_HIP_OK) return rc;
    if (position_offset < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s negative positionOffset", op);
    if ((long long)heads * (head_dim / 2) > 65535)  // one grid row per (head, pair)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s more than 65535 (head, pair) rows", op);
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    const hipError_t err = launch_rope_rotate_f32(tensor + column_start, heads, head_dim, stride_columns, columns,
                                                  position_offset, segment_length, cos_table, sin_table, inverse != 0,
                                                  static_cast<hipStream_t>(stream_ptr));
    if (err != hipSuccess) return fail_hip("rope rotate launch", err);
    return SENTINEL_HIP_OK;
}

extern "C" int sentinel_hip_cast_to_16bit(const float* source, void* destination, size_t element_count, int dtype,
                                          void* stream_ptr) {
    const char* op = "sentinel_hip_cast_to_16bit";
    if (dtype != SENTINEL_HIP_BF16 && dtype != SENTINEL_HIP_F16)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s dtype must be SENTINEL_HIP_BF16 or SENTINEL_HIP_F16", op);
    if (element_count == 0) return SENTINEL_HIP_OK;
    if (!source || !destination) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty buffer", op);
    if (reinterpret_cast<uintptr_t>(source) % 4 != 0 || reinterpret_cast<uintptr_t>(destination) % 2 != 0)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s misaligned buffer", op);
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    const hipError_t err = launch_cast_f32_to_16bit(static_cast<Elem>(dtype), source, destination, element_count,
                                                    static_cast<hipStream_t>(stream_ptr));
    if (err != hipSuccess) return fail_hip("cast launch", err);
    return SENTINEL_HIP_OK;
}

namespace {

// argument checks shared by the dense path's two softmax entry points; messages follow
// CudaOps::applySparseAttentionMaskInPlace (Cuda/CudaOps.cu:1262-1267)
int check_dense(const char* op, const void* a, const void* b, int batch, long long stride_a, long long stride_b, int key_count,
                int query_count, int query_position_start, int global_token_count, int segment_length, float scale) {
    if (!a || !b || batch <= 0 || key_count <= 0 || query_count <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty scores", op);
    const long long elements = (long long)key_count * query_count;
    if (batch > 65535) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s more than 65535 matrices in one call", op);
    if (batch > 1 && (stride_a < elements || stride_b < elements))
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s batch stride smaller than one matrix", op);
    if (global_token_count < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s globalTokenCount must be >= 0", op);
    if (query_position_start < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s queryPositionStart must be >= 0", op);
    if (segment_length < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s segmentLength must be >= 0", op);
    if (!std::isfinite(scale)) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s scale must be finite", op);
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    return SENTINEL_HIP_OK;
}

}  // namespace

extern "C" int sentinel_hip_dense_softmax_fwd(float* scores, int batch, long long batch_stride, int key_count, int query_count,
                                              int query_position_start, int window_size, int global_token_count,
                                              int segment_length, float scale, void* stream_ptr) {
    const char* op = "sentinel_hip_dense_softmax_fwd";
    const int rc = check_dense(op, scores, scores, batch, batch_stride, batch_stride, key_count, query_count, query_position_start,
                               global_token_count, segment_length, scale);
    if (rc != SENTINEL_HIP_OK) return rc;
    const hipError_t err = launch_dense_softmax_fwd(scores, batch, batch_stride, key_count, query_count, query_position_start,
                                                    window_size, global_token_count, segment_length, scale,
                                                    static_cast<hipStream_t>(stream_ptr));
    if (err != hipSuccess) return fail_hip("dense softmax launch", err);
    return SENTINEL_HIP_OK;
}

extern "C" int sentinel_hip_dense_softmax_bwd(const float* probabilities, long long probability_batch_stride,
                                              float* probability_gradient, long long gradient_batch_stride, int batch,
                                              int key_count, int query_count, int query_position_start, int window_size,
                                              int global_token_count, int segment_length, float scale, void* stream_ptr) {
    const char* op = "sentinel_hip_dense_softmax_bwd";
    const int rc = check_dense(op, probabilities, probability_gradient, batch, probability_batch_stride, gradient_batch_stride,
                               key_count, query_count, query_position_start, global_token_count, segment_length, scale);
    if (rc != SENTINEL_HIP_OK) return rc;
    const hipError_t err = launch_dense_softmax_bwd(probabilities, probability_batch_stride, probability_gradient,
                                                    gradient_batch_stride, batch, key_count, query_count, query_position_start,
                                                    window_size, global_token_count, segment_length, scale,
                                                    static_cast<hipStream_t>(stream_ptr));
    if (err != hipSuccess) return fail_hip("dense softmax backward launch", err);
    return SENTINEL_HIP_OK;
}

extern "C" size_t sentinel_hip_decode_workspace_bytes(int q_heads, int head_dim, int length) {
    if (q_heads <= 0 || head_dim <= 0 || length <= 0) return 0;
    return align_up(decode_workspace_bytes(q_heads, head_dim, length));
}

namespace {

// argument checks shared by the two decode entry points (everything but the workspace)
int check_decode(const char* op, const float* query, const float* key_cache, const float* value_cache, const float* out,
                 int q_heads, int kv_heads, int head_dim, int cache_stride, int length, float scale, int global_token_count) {
    if (!query || !key_cache || !value_cache || !out) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s empty input", op);
    if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s invalid head geometry", op);
    if (q_heads % kv_heads != 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s headCount must be divisible by kvHeadCount", op);
    if (head_dim > sentinel_hip_flash_max_head_dim()) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s headDim exceeds maxHeadDimension", op);
    if (length <= 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s cache is empty", op);
    if (length > cache_stride) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s cache length exceeds its capacity", op);
    if (!(scale > 0.0f) || !std::isfinite(scale)) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s scale must be positive and finite", op);
    if (global_token_count < 0) return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s globalTokenCount must be >= 0", op);
    const int group = q_heads / kv_heads;
    if (group != 1 && group != 2 && group != 4 && group != 8)
        return fail(SENTINEL_HIP_UNSUPPORTED, "%s query heads per K/V head must be 1, 2, 4 or 8 (got %d)", op, group);
    if (head_dim % 8 != 0) return fail(SENTINEL_HIP_UNSUPPORTED, "%s head_dim must be a multiple of 8", op);
    return SENTINEL_HIP_OK;
}

}  // namespace

extern "C" int sentinel_hip_decode_attention(const float* query, const float* key_cache, const float* value_cache, float* out,
                                             int q_heads, int kv_heads, int head_dim, int cache_stride, int length,
                                             float scale, int window_size, int global_token_count, void* workspace,
                                             size_t workspace_bytes, void* stream_ptr) {
    const char* op = "sentinel_hip_decode_attention";
    const int rc = check_decode(op, query, key_cache, value_cache, out, q_heads, kv_heads, head_dim, cache_stride, length, scale,
                                global_token_count);
    if (rc != SENTINEL_HIP_OK) return rc;
    const size_t need = sentinel_hip_decode_workspace_bytes(q_heads, head_dim, length);
    if (!workspace || workspace_bytes < need || misaligned(workspace))
        return fail(SENTINEL_HIP_INVALID_ARGUMENT, "%s needs %zu bytes of 16-byte aligned workspace", op, need);
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    const hipError_t err = launch_decode_attention(query, key_cache, value_cache, out, q_heads, kv_heads, head_dim,
                                                   cache_stride, length, scale, window_size, global_token_count,
                                                   static_cast<float*>(workspace), static_cast<hipStream_t>(stream_ptr));
    if (err != hipSuccess) return fail_hip("decode attention launch", err);
    return SENTINEL_HIP_OK;
}

extern "C" int sentinel_hip_decode_attention_static(const float* query, const float* key_cache, const float* value_cache,
                                                    float* out, int q_heads, int kv_heads, int head_dim, int cache_stride,
                                                    int length, float scale, int window_size, int global_token_count,
                                                    void* stream_ptr) {
    const char* op = "sentinel_hip_decode_attention_static";
    const int rc = check_decode(op, query, key_cache, value_cache, out, q_heads, kv_heads, head_dim, cache_stride, length, scale,
                                global_token_count);
    if (rc != SENTINEL_HIP_OK) return rc;
    const size_t need = sentinel_hip_decode_workspace_bytes(q_heads, head_dim, length);
    if (need > kDecodeStaticScratchBytes)
        return fail(SENTINEL_HIP_INVALID_ARGUMENT,
                    "%s needs %zu bytes of scratch, the built-in area holds %zu: use sentinel_hip_decode_attention with a "
                    "workspace of your own",
                    op, need, (size_t)kDecodeStaticScratchBytes);
    if (!sentinel_hip_device_available()) return fail(SENTINEL_HIP_RUNTIME, "%s no HIP device", op);
    float* scratch = nullptr;  // this device's copy of the array: an address from the runtime, never the array's name
    hipError_t err = decode_static_scratch_address(&scratch);
    if (err != hipSuccess) return fail_hip("decode attention scratch lookup", err);
    // nothing in the area has to start at zero: decode_partial writes every record that decode_merge reads
    err = launch_decode_attention(query, key_cache, value_cache, out, q_heads, kv_heads, head_dim, cache_stride, length, scale,
                                  window_size, global_token_count, scratch, static_cast<hipStream_t>(stream_ptr));
    if (err != hipSuccess) return fail_hip("decode attention launch", err);
    return SENTINEL_HIP_OK;
}
