// extern "C" surface of libhawk_hip.so: argument validation, then dispatch to the kernel
// translation units.  Validation happens before any HIP call, so bad arguments are
// reported without touching a GPU.
#include "hawk_scan.h"

#include <stdint.h>

namespace {

inline bool dtype_ok(int d) { return d == HAWK_DTYPE_BF16 || d == HAWK_DTYPE_F32; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
// y and dy of the gated scan may be slices of wider tensors: element alignment is enough
inline bool aligned_elem(const void* p, int dtype) {
    return (reinterpret_cast<uintptr_t>(p) & (dtype == HAWK_DTYPE_F32 ? 3u : 1u)) == 0;
}
inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

constexpr int kMaxGridY = 65535;
constexpr long long kMaxTiles = 0x7fffffffLL;
constexpr long long kMaxRowStride = 1LL << 24;  // elements; keeps 16 rows of any dtype within 32-bit byte offsets

int check_scan_shape(int B, int T, int D) {
    if (B < 1 || T < 1 || D < 1) return HAWK_ERR_BAD_SHAPE;
    // the kernels form row and tile byte offsets in 32 bits
    if (D > kMaxRowStride) return HAWK_ERR_BAD_SHAPE;
    // tiles are at least 64 rows x 64 channels; the flattened grid must fit 31 bits
    const long long tiles = (long long)B * ((T + 63) / 64) * ((D + 63) / 64);
    if (tiles > kMaxTiles) return HAWK_ERR_BAD_SHAPE;
    return HAWK_OK;
}

}  // namespace

extern "C" {

int hawk_version(void) { return 100; }

int hawk_stream_capture_id(void* stream, unsigned long long* id) {
    if (!id) return HAWK_ERR_NULL_POINTER;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long cid = 0;
    if (hipStreamGetCaptureInfo(as_stream(stream), &status, &cid) != hipSuccess) return HAWK_ERR_LAUNCH;
    *id = status == hipStreamCaptureStatusActive ? cid : 0ull;
    return HAWK_OK;
}

const char* hawk_status_string(int status) {
    switch (status) {
        case HAWK_OK: return "ok";
        case HAWK_ERR_NULL_POINTER: return "a required pointer is NULL";
        case HAWK_ERR_BAD_SHAPE: return "bad shape: sizes must be >= 1 and within the documented limits";
        case HAWK_ERR_BAD_DTYPE: return "unsupported dtype (expected HAWK_DTYPE_BF16 or HAWK_DTYPE_F32)";
        case HAWK_ERR_WORKSPACE: return "workspace is NULL or smaller than the size query reports";
        case HAWK_ERR_LAUNCH: return "the HIP runtime refused a kernel launch or copy";
        case HAWK_ERR_ALIGNMENT: return "tensor pointers must be 16-byte aligned";
        case HAWK_ERR_SCRATCH_LIMIT:
            return "shape needs more carry words than the library's fixed 16 MiB scratch array holds: "
                   "hawk_rglru_scan_fwd_static_bytes(B, T, D, dtype) must fit; use the entry point that takes a workspace";
        default: return "unknown status";
    }
}

size_t hawk_scan_workspace_bytes(int B, int T, int D, int dtype) {
    if (check_scan_shape(B, T, D) != HAWK_OK || !dtype_ok(dtype)) return 0;
    return hawk::scan_workspace_bytes(B, T, D, dtype);
}

int hawk_scan_workspace_init(void* workspace_device, size_t workspace_bytes, void* stream) {
    if (workspace_device == nullptr) return HAWK_ERR_NULL_POINTER;
    if (!aligned16(workspace_device)) return HAWK_ERR_ALIGNMENT;
    if (workspace_bytes < 256) return HAWK_ERR_WORKSPACE;
    return hawk::workspace_init(workspace_device, workspace_bytes, as_stream(stream));
}

int hawk_scan_workspace_status(const void* workspace_device, void* stream, int* flag) {
    if (flag == nullptr) return HAWK_ERR_NULL_POINTER;
    if (workspace_device == nullptr) return hawk::static_scratch_status(as_stream(stream), flag);
    return hawk::workspace_status(workspace_device, as_stream(stream), flag);
}

int hawk_rglru_scan_fwd_mixed(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                              void* h, int B, int T, int D, int in_dtype, int out_dtype, void* workspace_device,
                              size_t workspace_bytes, void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !h) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !hawk::scan_dtypes_supported(in_dtype, out_dtype))
        return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(h)) return HAWK_ERR_ALIGNMENT;
    if (workspace_device && !aligned16(workspace_device)) return HAWK_ERR_ALIGNMENT;
    return hawk::scan_fwd(x, x_rg_lru, a_rg_lru, a_param, h, B, T, D, in_dtype, out_dtype, workspace_device,
                          workspace_bytes, as_stream(stream));
}

int hawk_rglru_scan_fwd(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param, void* h,
                        int B, int T, int D, int dtype, void* workspace_device, size_t workspace_bytes,
                        void* stream) {
    return hawk_rglru_scan_fwd_mixed(x, x_rg_lru, a_rg_lru, a_param, h, B, T, D, dtype, dtype, workspace_device,
                                     workspace_bytes, stream);
}

int hawk_rglru_scan_fwd_static(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                               void* h, int B, int T, int D, int dtype, void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !h) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(dtype)) return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(h)) return HAWK_ERR_ALIGNMENT;
    return hawk::scan_fwd_static(x, x_rg_lru, a_rg_lru, a_param, h, B, T, D, dtype, as_stream(stream));
}

size_t hawk_rglru_scan_fwd_static_bytes(int B, int T, int D, int dtype) {
    if (check_scan_shape(B, T, D) != HAWK_OK || !dtype_ok(dtype)) return 0;
    return hawk::scan_fwd_static_bytes(B, T, D, dtype);
}

int hawk_rglru_scan_bwd_mixed(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                              const void* h_saved, const void* grad_out, void* dx, void* dx_rg_lru, void* da_rg_lru,
                              float* da_param, int B, int T, int D, int in_dtype, int state_dtype,
                              void* workspace_device, size_t workspace_bytes, void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !h_saved || !grad_out || !dx || !dx_rg_lru || !da_rg_lru ||
        !da_param)
        return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(in_dtype) || !dtype_ok(state_dtype) || !hawk::scan_dtypes_supported(in_dtype, state_dtype))
        return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(h_saved) ||
        !aligned16(grad_out) || !aligned16(dx) || !aligned16(dx_rg_lru) || !aligned16(da_rg_lru))
        return HAWK_ERR_ALIGNMENT;
    if (workspace_device == nullptr) return HAWK_ERR_WORKSPACE;
    if (!aligned16(workspace_device)) return HAWK_ERR_ALIGNMENT;
    return hawk::scan_bwd(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out, dx, dx_rg_lru, da_rg_lru, da_param, B,
                          T, D, in_dtype, state_dtype, workspace_device, workspace_bytes, as_stream(stream));
}

int hawk_rglru_scan_bwd(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                        const void* h_saved, const void* grad_out, void* dx, void* dx_rg_lru, void* da_rg_lru,
                        float* da_param, int B, int T, int D, int dtype, void* workspace_device,
                        size_t workspace_bytes, void* stream) {
    return hawk_rglru_scan_bwd_mixed(x, x_rg_lru, a_rg_lru, a_param, h_saved, grad_out, dx, dx_rg_lru, da_rg_lru,
                                     da_param, B, T, D, dtype, dtype, workspace_device, workspace_bytes, stream);
}

int hawk_rglru_scan_gated_fwd(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                              const void* y, long long ldy, void* h, void* out, void* h_last, int B, int T, int D,
                              int in_dtype, int out_dtype, void* workspace_device, size_t workspace_bytes,
                              void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !y || !out) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype) || !hawk::scan_dtypes_supported(in_dtype, out_dtype))
        return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    if (ldy < D || ldy > kMaxRowStride) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned_elem(y, out_dtype) ||
        !aligned16(out) || (h && !aligned16(h)) || (h_last && !aligned16(h_last)))
        return HAWK_ERR_ALIGNMENT;
    if (workspace_device && !aligned16(workspace_device)) return HAWK_ERR_ALIGNMENT;
    return hawk::scan_gated_fwd(x, x_rg_lru, a_rg_lru, a_param, y, ldy, h, out, h_last, B, T, D, in_dtype, out_dtype,
                                workspace_device, workspace_bytes, as_stream(stream));
}

int hawk_rglru_scan_gated_bwd(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                              const void* y, long long ldy, const void* h_saved, const void* grad_out, void* dx,
                              void* dx_rg_lru, void* da_rg_lru, void* dy, long long lddy, float* da_param, int B,
                              int T, int D, int in_dtype, int state_dtype, void* workspace_device,
                              size_t workspace_bytes, void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !y || !h_saved || !grad_out || !dx || !dx_rg_lru || !da_rg_lru ||
        !dy || !da_param)
        return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(in_dtype) || !dtype_ok(state_dtype) || !hawk::scan_dtypes_supported(in_dtype, state_dtype))
        return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    if (ldy < D || ldy > kMaxRowStride || lddy < D || lddy > kMaxRowStride) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned_elem(y, state_dtype) ||
        !aligned16(h_saved) || !aligned16(grad_out) || !aligned16(dx) || !aligned16(dx_rg_lru) ||
        !aligned16(da_rg_lru) || !aligned_elem(dy, state_dtype))
        return HAWK_ERR_ALIGNMENT;
    if (workspace_device == nullptr) return HAWK_ERR_WORKSPACE;
    if (!aligned16(workspace_device)) return HAWK_ERR_ALIGNMENT;
    return hawk::scan_gated_bwd(x, x_rg_lru, a_rg_lru, a_param, y, ldy, h_saved, grad_out, dx, dx_rg_lru, da_rg_lru,
                                dy, lddy, da_param, B, T, D, in_dtype, state_dtype, workspace_device, workspace_bytes,
                                as_stream(stream));
}

int hawk_conv1d_fwd_strided(const void* x, long long x_row_stride, const float* w, const float* bias,
                            const void* state, void* y, long long y_row_stride, int B, int T, int D, int W,
                            int x_dtype, int y_dtype, void* stream) {
    if (!x || !w || !bias || !y) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (B < 1 || T < 1 || D < 1 || W < 1 || W > 8 || B > kMaxGridY) return HAWK_ERR_BAD_SHAPE;
    if (W != 4 && T > kMaxGridY) return HAWK_ERR_BAD_SHAPE;
    if (x_row_stride < D || y_row_stride < D || x_row_stride > kMaxRowStride || y_row_stride > kMaxRowStride)
        return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(y) || (state && !aligned16(state))) return HAWK_ERR_ALIGNMENT;
    return hawk::conv1d_fwd(x, x_row_stride, w, bias, state, y, y_row_stride, B, T, D, W, x_dtype, y_dtype,
                            as_stream(stream));
}

int hawk_conv1d_fwd(const void* x, const float* w, const float* bias, const void* state, void* y, int B, int T,
                    int D, int W, int x_dtype, int y_dtype, void* stream) {
    return hawk_conv1d_fwd_strided(x, D, w, bias, state, y, D, B, T, D, W, x_dtype, y_dtype, stream);
}

size_t hawk_conv1d_bwd_workspace_bytes(int B, int T, int D, int W) {
    if (B < 1 || T < 1 || D < 1 || W < 1 || W > 8) return 0;
    return hawk::conv1d_bwd_workspace_bytes(B, T, D, W);
}

int hawk_conv1d_bwd_strided(const void* grad_y, const void* x, long long x_row_stride, const float* w, void* dx,
                            long long dx_row_stride, float* dw, float* db, int B, int T, int D, int W, int x_dtype,
                            int gy_dtype, void* workspace_device, size_t workspace_bytes, void* stream) {
    if (!grad_y || !x || !w || !dx || !dw || !db) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(x_dtype) || !dtype_ok(gy_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (B < 1 || T < 1 || D < 1 || W < 1 || W > 8 || B > kMaxGridY) return HAWK_ERR_BAD_SHAPE;
    if (x_row_stride < D || dx_row_stride < D || x_row_stride > kMaxRowStride || dx_row_stride > kMaxRowStride)
        return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(grad_y) || !aligned16(x) || !aligned16(dx)) return HAWK_ERR_ALIGNMENT;
    if (workspace_device == nullptr) return HAWK_ERR_WORKSPACE;
    return hawk::conv1d_bwd(grad_y, x, x_row_stride, w, dx, dx_row_stride, dw, db, B, T, D, W, x_dtype, gy_dtype,
                            workspace_device, workspace_bytes, as_stream(stream));
}

int hawk_conv1d_bwd(const void* grad_y, const void* x, const float* w, void* dx, float* dw, float* db, int B, int T,
                    int D, int W, int x_dtype, int gy_dtype, void* workspace_device, size_t workspace_bytes,
                    void* stream) {
    return hawk_conv1d_bwd_strided(grad_y, x, D, w, dx, D, dw, db, B, T, D, W, x_dtype, gy_dtype, workspace_device,
                                   workspace_bytes, stream);
}

int hawk_conv1d_step(void* conv_state, const void* x_new, const float* w, const float* bias, void* y, int B, int D,
                     int W, int dtype, int y_dtype, void* stream) {
    if (!x_new || !w || !bias || !y || (W > 1 && !conv_state)) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(dtype) || !dtype_ok(y_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (B < 1 || D < 1 || W < 1 || W > 8 || B > kMaxGridY) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x_new) || !aligned16(y) || (conv_state && !aligned16(conv_state))) return HAWK_ERR_ALIGNMENT;
    return hawk::conv1d_step(conv_state, x_new, w, bias, y, B, D, W, dtype, y_dtype, as_stream(stream));
}

int hawk_rglru_step(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* a_param,
                    void* recc_state, void* h_out, int B, int D, int dtype, int state_dtype, void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !recc_state || !h_out) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(dtype) || !dtype_ok(state_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (B < 1 || D < 1 || B > kMaxGridY) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(recc_state) || !aligned16(h_out))
        return HAWK_ERR_ALIGNMENT;
    return hawk::rglru_step(x, x_rg_lru, a_rg_lru, a_param, recc_state, h_out, B, D, dtype, state_dtype,
                            as_stream(stream));
}

int hawk_rglru_step_gated(const void* x, const void* x_rg_lru, const void* a_rg_lru, const float* bias_i,
                          const float* bias_a, const float* a_param, const void* y, long long ldy, void* recc_state,
                          void* h_out, void* out, int B, int D, int dtype, int state_dtype, void* stream) {
    if (!x || !x_rg_lru || !a_rg_lru || !a_param || !recc_state || !y || !out) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(dtype) || !dtype_ok(state_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (B < 1 || D < 1 || B > kMaxGridY || ldy < D) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(recc_state) || !aligned16(out) ||
        (h_out && !aligned16(h_out)) || !aligned_elem(y, dtype))
        return HAWK_ERR_ALIGNMENT;
    return hawk::rglru_step_gated(x, x_rg_lru, a_rg_lru, bias_i, bias_a, a_param, y, ldy, recc_state, h_out, out, B,
                                  D, dtype, state_dtype, as_stream(stream));
}

int hawk_gate_proj_supported(int D, int num_blocks) {
    if (D < 1 || num_blocks < 1 || D % num_blocks != 0) return 0;
    return hawk::gate_proj_block_width_supported(D / num_blocks) ? 1 : 0;
}

int hawk_decode_core_supported(int D, int num_blocks, int W) {
    return (W >= 1 && W <= 8 && hawk_gate_proj_supported(D, num_blocks)) ? 1 : 0;
}

size_t hawk_decode_core_workspace_bytes(int B, int D, int num_blocks) {
    if (B < 1 || !hawk_gate_proj_supported(D, num_blocks)) return 0;
    return hawk::decode_core_workspace_bytes(B, D, num_blocks);
}

int hawk_decode_core_step_ws(void* conv_state, const void* x_new, long long ldx, const float* conv_w,
                             const float* conv_b, const void* w_i, const float* b_i, const void* w_a, const float* b_a,
                             const float* a_param, const void* y, long long ldy, void* recc_state, void* out, int B,
                             int D, int num_blocks, int W, int dtype, int w_dtype, int state_dtype,
                             void* workspace_device, size_t workspace_bytes, void* stream) {
    if (!x_new || !conv_w || !conv_b || !w_i || !w_a || !a_param || !y || !recc_state || !out ||
        (W > 1 && !conv_state))
        return HAWK_ERR_NULL_POINTER;
    if (dtype != HAWK_DTYPE_BF16 || !dtype_ok(w_dtype) || !dtype_ok(state_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (B < 1 || !hawk_decode_core_supported(D, num_blocks, W)) return HAWK_ERR_BAD_SHAPE;
    // rows of x_new are read 16 bytes at a time
    if (ldx < D || (ldx % 8) != 0 || ldx > kMaxRowStride || ldy < D || ldy > kMaxRowStride) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x_new) || (conv_state && !aligned16(conv_state)) || !aligned16(w_i) || !aligned16(w_a) ||
        !aligned_elem(y, dtype) || !aligned_elem(recc_state, state_dtype) || !aligned_elem(out, dtype))
        return HAWK_ERR_ALIGNMENT;
    if (workspace_device != nullptr) {
        if ((reinterpret_cast<uintptr_t>(workspace_device) & 3u) != 0) return HAWK_ERR_ALIGNMENT;
        if (workspace_bytes < hawk::decode_core_workspace_bytes(B, D, num_blocks)) return HAWK_ERR_WORKSPACE;
    }
    return hawk::decode_core_step(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, a_param, y, ldy,
                                  recc_state, out, B, D, num_blocks, W, w_dtype, state_dtype, workspace_device,
                                  workspace_bytes, as_stream(stream));
}

int hawk_decode_core_step(void* conv_state, const void* x_new, long long ldx, const float* conv_w,
                          const float* conv_b, const void* w_i, const float* b_i, const void* w_a, const float* b_a,
                          const float* a_param, const void* y, long long ldy, void* recc_state, void* out, int B, int D,
                          int num_blocks, int W, int dtype, int w_dtype, int state_dtype, void* stream) {
    return hawk_decode_core_step_ws(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, a_param, y, ldy,
                                    recc_state, out, B, D, num_blocks, W, dtype, w_dtype, state_dtype, nullptr, 0,
                                    stream);
}

int hawk_gate_proj_fwd(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a,
                       void* x_rg_lru, void* a_rg_lru, int M, int D, int num_blocks, int x_dtype, int w_dtype,
                       int out_dtype, void* stream) {
    if (!x || !w_i || !w_a || !x_rg_lru || !a_rg_lru) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(x_dtype) || !dtype_ok(w_dtype) || !dtype_ok(out_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (M < 1 || !hawk_gate_proj_supported(D, num_blocks)) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(w_i) || !aligned16(w_a))
        return HAWK_ERR_ALIGNMENT;
    return hawk::gate_proj_fwd(x, w_i, b_i, w_a, b_a, x_rg_lru, a_rg_lru, M, D, num_blocks, x_dtype, w_dtype,
                               out_dtype, as_stream(stream));
}

int hawk_conv_gate_proj_fwd(const void* x, long long x_row_stride, const float* conv_w, const float* conv_b,
                            const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* u,
                            void* x_rg_lru, void* a_rg_lru, int B, int T, int D, int num_blocks, int temporal_width,
                            int w_dtype, void* stream) {
    if (!x || !conv_w || !conv_b || !w_i || !w_a || !u || !x_rg_lru || !a_rg_lru) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(w_dtype)) return HAWK_ERR_BAD_DTYPE;
    // one wrap of the position per 32-row tile, 32-bit byte offsets over a tile and its history
    if (B < 1 || T < 32 || temporal_width != 4 || !hawk_gate_proj_supported(D, num_blocks) ||
        (long long)B * T > 0x7fffffffLL || x_row_stride < D || x_row_stride > kMaxRowStride || x_row_stride % 8 != 0)
        return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(u) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(w_i) ||
        !aligned16(w_a))
        return HAWK_ERR_ALIGNMENT;
    return hawk::conv_gate_proj_fwd(x, x_row_stride, conv_w, conv_b, w_i, b_i, w_a, b_a, u, x_rg_lru, a_rg_lru, B, T,
                                    D, num_blocks, w_dtype, as_stream(stream));
}

int hawk_gate_proj_bwd_input(const void* d_x_rg_lru, const void* d_a_rg_lru, const void* w_i, const void* w_a,
                             const void* addend, void* dx, int M, int D, int num_blocks, int g_dtype, int w_dtype,
                             int dx_dtype, void* stream) {
    if (!d_x_rg_lru || !d_a_rg_lru || !w_i || !w_a || !dx) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(g_dtype) || !dtype_ok(w_dtype) || !dtype_ok(dx_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (M < 1 || !hawk_gate_proj_supported(D, num_blocks)) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(d_x_rg_lru) || !aligned16(d_a_rg_lru) || !aligned16(dx) || !aligned16(w_i) || !aligned16(w_a) ||
        (addend && !aligned16(addend)))
        return HAWK_ERR_ALIGNMENT;
    return hawk::gate_proj_bwd_input(d_x_rg_lru, d_a_rg_lru, w_i, w_a, addend, dx, M, D, num_blocks, g_dtype, w_dtype,
                                     dx_dtype, as_stream(stream));
}

size_t hawk_gate_proj_bwd_weights_workspace_bytes(int M, int D, int num_blocks) {
    if (M < 1 || !hawk_gate_proj_supported(D, num_blocks)) return 0;
    return hawk::gate_proj_bwd_weights_workspace_bytes(M, D, num_blocks);
}

int hawk_gate_proj_bwd_weights(const void* x, const void* d_x_rg_lru, const void* d_a_rg_lru, float* dw_i,
                               float* db_i, float* dw_a, float* db_a, int M, int D, int num_blocks, int x_dtype,
                               int g_dtype, void* workspace_device, size_t workspace_bytes, void* stream) {
    if (!x || !d_x_rg_lru || !d_a_rg_lru || !dw_i || !dw_a) return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(x_dtype) || !dtype_ok(g_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (M < 1 || !hawk_gate_proj_supported(D, num_blocks)) return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(x) || !aligned16(d_x_rg_lru) || !aligned16(d_a_rg_lru)) return HAWK_ERR_ALIGNMENT;
    if (workspace_device == nullptr) return HAWK_ERR_WORKSPACE;
    if (!aligned16(workspace_device)) return HAWK_ERR_ALIGNMENT;
    return hawk::gate_proj_bwd_weights(x, d_x_rg_lru, d_a_rg_lru, dw_i, db_i, dw_a, db_a, M, D, num_blocks, x_dtype,
                                       g_dtype, workspace_device, workspace_bytes, as_stream(stream));
}

int hawk_gate_weights_to_bf16(const float* w_i, const float* w_a, void* w_i_bf16, void* w_a_bf16, int num_blocks,
                              int block_width, void* stream) {
    if (!w_i || !w_a || !w_i_bf16 || !w_a_bf16) return HAWK_ERR_NULL_POINTER;
    if (num_blocks < 1 || block_width < 1 || block_width % 4 != 0 ||
        (long long)num_blocks * block_width * block_width > 0x7fffffffLL)
        return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(w_i) || !aligned16(w_a) || !aligned16(w_i_bf16) || !aligned16(w_a_bf16)) return HAWK_ERR_ALIGNMENT;
    return hawk::gate_weights_to_bf16(w_i, w_a, w_i_bf16, w_a_bf16, (size_t)num_blocks * block_width * block_width,
                                      as_stream(stream));
}

int hawk_block_core_fwd(const void* xy, long long xy_row_stride, const float* conv_w, const float* conv_b,
                        const void* w_i, const float* b_i, const void* w_a, const float* b_a, int w_dtype,
                        void* w_bf16, const float* a_param, void* u, void* x_rg_lru, void* a_rg_lru, void* h, void* out,
                        void* h_last, int B, int T, int D, int num_blocks, int temporal_width,
                        void* scan_workspace, size_t scan_workspace_bytes, void* stream) {
    if (!xy || !conv_w || !conv_b || !w_i || !w_a || !a_param || !u || !x_rg_lru || !a_rg_lru || !out)
        return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(w_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    // the conv in front of the projections: one wrap of the position per 32-row tile, 32-bit byte
    // offsets over a tile and its history; y = xy + D must stay 16-byte aligned row by row
    if (T < 32 || temporal_width != 4 || !hawk_gate_proj_supported(D, num_blocks) || D % 8 != 0 ||
        (long long)B * T > 0x7fffffffLL || xy_row_stride < 2LL * D || xy_row_stride > kMaxRowStride ||
        xy_row_stride % 8 != 0)
        return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(xy) || !aligned16(u) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(w_i) ||
        !aligned16(w_a) || !aligned16(out) || (h && !aligned16(h)) || (h_last && !aligned16(h_last)) ||
        (w_bf16 && !aligned16(w_bf16)) || (scan_workspace && !aligned16(scan_workspace)))
        return HAWK_ERR_ALIGNMENT;
    return hawk::block_core_fwd(xy, xy_row_stride, conv_w, conv_b, w_i, b_i, w_a, b_a, w_dtype, w_bf16, a_param, u,
                                x_rg_lru, a_rg_lru, h, out, h_last, B, T, D, num_blocks, scan_workspace,
                                scan_workspace_bytes, as_stream(stream));
}

int hawk_block_core_bwd(const void* xy, long long xy_row_stride, const void* u, const void* x_rg_lru,
                        const void* a_rg_lru, const void* h_saved, const float* conv_w, const void* w_i,
                        const void* w_a, int w_dtype, const float* a_param, const void* grad_out, void* d_xy,
                        long long d_xy_row_stride, void* du, void* d_x_rg_lru, void* d_a_rg_lru, float* d_conv_w,
                        float* d_conv_b, float* dw_i, float* db_i, float* dw_a, float* db_a, float* da_param, int B,
                        int T, int D, int num_blocks, int temporal_width, void* scan_workspace,
                        size_t scan_workspace_bytes, void* gate_workspace, size_t gate_workspace_bytes,
                        void* conv_workspace, size_t conv_workspace_bytes, void* stream) {
    if (!xy || !u || !x_rg_lru || !a_rg_lru || !h_saved || !conv_w || !w_i || !w_a || !a_param || !grad_out || !d_xy ||
        !du || !d_x_rg_lru || !d_a_rg_lru || !d_conv_w || !d_conv_b || !dw_i || !dw_a || !da_param)
        return HAWK_ERR_NULL_POINTER;
    if (!dtype_ok(w_dtype)) return HAWK_ERR_BAD_DTYPE;
    if (int rc = check_scan_shape(B, T, D)) return rc;
    if (temporal_width < 1 || temporal_width > 8 || B > kMaxGridY || !hawk_gate_proj_supported(D, num_blocks) ||
        D % 8 != 0 || (long long)B * T > 0x7fffffffLL || xy_row_stride < 2LL * D || xy_row_stride > kMaxRowStride ||
        xy_row_stride % 8 != 0 || d_xy_row_stride < 2LL * D || d_xy_row_stride > kMaxRowStride ||
        d_xy_row_stride % 8 != 0)
        return HAWK_ERR_BAD_SHAPE;
    if (!aligned16(xy) || !aligned16(u) || !aligned16(x_rg_lru) || !aligned16(a_rg_lru) || !aligned16(h_saved) ||
        !aligned16(w_i) || !aligned16(w_a) || !aligned16(grad_out) || !aligned16(d_xy) || !aligned16(du) ||
        !aligned16(d_x_rg_lru) || !aligned16(d_a_rg_lru))
        return HAWK_ERR_ALIGNMENT;
    if (!scan_workspace || !gate_workspace || !conv_workspace) return HAWK_ERR_WORKSPACE;
    if (!aligned16(scan_workspace) || !aligned16(gate_workspace) || !aligned16(conv_workspace))
        return HAWK_ERR_ALIGNMENT;
    return hawk::block_core_bwd(xy, xy_row_stride, u, x_rg_lru, a_rg_lru, h_saved, conv_w, w_i, w_a, w_dtype, a_param,
                                grad_out, d_xy, d_xy_row_stride, du, d_x_rg_lru, d_a_rg_lru, d_conv_w, d_conv_b, dw_i,
                                db_i, dw_a, db_a, da_param, B, T, D, num_blocks, temporal_width, scan_workspace,
                                scan_workspace_bytes, gate_workspace, gate_workspace_bytes, conv_workspace,
                                conv_workspace_bytes, as_stream(stream));
}

int hawk_stream_probe(const void* const* reads, int n_reads, void* const* writes, int n_writes, size_t bytes,
                      size_t row_pitch_bytes, int shape, void* stream) {
    if (!reads || !writes) return HAWK_ERR_NULL_POINTER;
    if (n_reads < 1 || n_reads > 5 || n_writes < 1 || n_writes > 3) return HAWK_ERR_BAD_SHAPE;
    for (int i = 0; i < n_reads; ++i) {
        if (!reads[i]) return HAWK_ERR_NULL_POINTER;
        if (!aligned16(reads[i])) return HAWK_ERR_ALIGNMENT;
    }
    for (int i = 0; i < n_writes; ++i) {
        if (!writes[i]) return HAWK_ERR_NULL_POINTER;
        if (!aligned16(writes[i])) return HAWK_ERR_ALIGNMENT;
    }
    if (!hawk::stream_probe_shape_ok(bytes, row_pitch_bytes, shape)) return HAWK_ERR_BAD_SHAPE;
    return hawk::stream_probe(reads, n_reads, writes, n_writes, bytes, row_pitch_bytes, shape, as_stream(stream));
}

}  // extern "C"
