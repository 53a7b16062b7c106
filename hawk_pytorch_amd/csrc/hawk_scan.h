// Internal C++ interface between the C ABI (hawk_capi.hip) and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>

#include "../../include/hawk_hip.h"
#include "hawk_reduce.h"

namespace hawk {

// The backward entry points below that take a `deferred` pointer end in a small reduction of
// per-tile partial sums; with the pointer set they hand its description back instead of
// launching it, and the caller runs it (block_core_bwd: three of them in one launch).

// hawk_scan.hip
size_t scan_workspace_bytes(int B, int T, int D, int dtype);
int workspace_init(void* ws, size_t bytes, hipStream_t st);
int workspace_status(const void* ws, hipStream_t st, int* flag);
// in_dtype: x, x_rg_lru, a_rg_lru (and, in the backward, their gradients);
// out_dtype / state_dtype: h (and, in the backward, the saved h and grad_out).
bool scan_dtypes_supported(int in_dtype, int state_dtype);
int scan_fwd(const void* x, const void* xg, const void* ag, const float* lam, void* h, int B, int T, int D,
             int in_dtype, int out_dtype, void* ws, size_t ws_bytes, hipStream_t st);
int scan_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* hs, const void* gout,
             void* dx, void* dxg, void* dag, float* dlam, int B, int T, int D, int in_dtype, int state_dtype,
             void* ws, size_t ws_bytes, hipStream_t st);
// Forward scan on the library's fixed per-device carry array; allocates nothing.
int scan_fwd_static(const void* x, const void* xg, const void* ag, const float* lam, void* h, int B, int T, int D,
                    int dtype, hipStream_t st);
int static_scratch_status(hipStream_t st, int* flag);
// bytes of the fixed array a shape needs (0 when T fits one tile)
size_t scan_fwd_static_bytes(int B, int T, int D, int dtype);
// Gated variants: out = gelu(y) * h.  y (and dy) are [B, T, D] with ldy (lddy) elements between rows.
int scan_gated_fwd(const void* x, const void* xg, const void* ag, const float* lam, const void* y, long long ldy,
                   void* h, void* out, void* h_last, int B, int T, int D, int in_dtype, int out_dtype, void* ws,
                   size_t ws_bytes, hipStream_t st);
int scan_gated_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* y, long long ldy,
                   const void* hs, const void* gout, void* dx, void* dxg, void* dag, void* dy, long long lddy,
                   float* dlam, int B, int T, int D, int in_dtype, int state_dtype, void* ws, size_t ws_bytes,
                   hipStream_t st, ColsumTask* deferred = nullptr);

// hawk_conv.hip
// ldx, ldy, lddx: row strides in elements (>= D); batch rows lie T rows apart
int conv1d_fwd(const void* x, long long ldx, const float* w, const float* bias, const void* state, void* y,
               long long ldy, int B, int T, int D, int W, int x_dtype, int y_dtype, hipStream_t st);
size_t conv1d_bwd_workspace_bytes(int B, int T, int D, int W);
int conv1d_bwd(const void* gy, const void* x, long long ldx, const float* w, void* dx, long long lddx, float* dw,
               float* db, int B, int T, int D, int W, int x_dtype, int gy_dtype, void* ws, size_t ws_bytes,
               hipStream_t st, ColsumTask* deferred = nullptr);

// hawk_step.hip
int conv1d_step(void* conv_state, const void* x_new, const float* w, const float* bias, void* y, int B, int D,
                int W, int dtype, int y_dtype, hipStream_t st);
int rglru_step(const void* x, const void* xg, const void* ag, const float* lam, void* state, void* h_out, int B,
               int D, int dtype, int state_dtype, hipStream_t st);
int rglru_step_gated(const void* x, const void* xg, const void* ag, const float* bias_i, const float* bias_a,
                     const float* lam, const void* y, long long ldy, void* state, void* h_out, void* out, int B,
                     int D, int dtype, int state_dtype, hipStream_t st);

// hawk_gates.hip
bool gate_proj_block_width_supported(int bw);
int gate_proj_fwd(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* out_i,
                  void* out_a, int M, int D, int nb, int x_dtype, int w_dtype, int out_dtype, hipStream_t st);
// temporal conv (width 4, bf16 in and out, x rows ldx elements apart) and both projections of
// its output in one kernel; u receives the conv output
int conv_gate_proj_fwd(const void* x, long long ldx, const float* conv_w, const float* conv_b, const void* w_i,
                       const float* b_i, const void* w_a, const float* b_a, void* u, void* out_i, void* out_a, int B,
                       int T, int D, int nb, int w_dtype, hipStream_t st);
int gate_proj_bwd_input(const void* dxg, const void* dag, const void* w_i, const void* w_a, const void* addend,
                        void* dx, int M, int D, int nb, int g_dtype, int w_dtype, int dx_dtype, hipStream_t st);
// conv window roll + conv, both projections, state update and output gate of one decode step
// (bf16 activations and conv window; W <= 8)
int decode_core_step(void* conv_state, const void* x_new, long long ldx, const float* conv_w, const float* conv_b,
                     const void* w_i, const float* b_i, const void* w_a, const float* b_a, const float* lam,
                     const void* y, long long ldy, void* state, void* out, int B, int D, int nb, int W, int w_dtype,
                     int state_dtype, void* workspace, size_t workspace_bytes, hipStream_t st);
// counters (one 32-bit word per 32 rows and block, zero between launches) that let a launch cut a
// block's output columns over several workgroups
size_t decode_core_workspace_bytes(int B, int D, int nb);
size_t gate_proj_bwd_weights_workspace_bytes(int M, int D, int nb);
int gate_proj_bwd_weights(const void* x, const void* dg_i, const void* dg_a, float* dw_i, float* db_i, float* dw_a,
                          float* db_a, int M, int D, int nb, int x_dtype, int g_dtype, void* ws, size_t ws_bytes,
                          hipStream_t st, GateReduceTask* deferred = nullptr);

// hawk_block.hip
// two fp32 arrays of `count` elements (a multiple of 4) rounded to bf16 by one launch
int gate_weights_to_bf16(const float* w_i, const float* w_a, void* w_i16, void* w_a16, size_t count, hipStream_t st);
// conv + both projections + gated scan on the [B,T,2D] bf16 projection output xy (rows ld elements
// apart: x half, then y half).  fp32 weights are rounded once into w16 ([2][nb][bw][bw] bf16) when
// it is not NULL, and the kernels read those.
int block_core_fwd(const void* xy, long long ld, const float* conv_w, const float* conv_b, const void* w_i,
                   const float* b_i, const void* w_a, const float* b_a, int w_dtype, void* w16, const float* lam,
                   void* u, void* xg, void* ag, void* h, void* out, void* h_last, int B, int T, int D, int nb,
                   void* scan_ws, size_t scan_ws_bytes, hipStream_t st);
// The backward of all of it; du, dxg, dag: [B,T,D] bf16 scratch for the gradients in between.
int block_core_bwd(const void* xy, long long ld, const void* u, const void* xg, const void* ag, const void* h,
                   const float* conv_w, const void* w_i, const void* w_a, int w_dtype, const float* lam,
                   const void* gout, void* d_xy, long long ldd, void* du, void* dxg, void* dag, float* d_conv_w,
                   float* d_conv_b, float* dw_i, float* db_i, float* dw_a, float* db_a, float* dlam, int B, int T,
                   int D, int nb, int W, void* scan_ws, size_t scan_ws_bytes, void* gate_ws, size_t gate_ws_bytes,
                   void* conv_ws, size_t conv_ws_bytes, hipStream_t st);

// hawk_probe.hip
bool stream_probe_shape_ok(size_t bytes, size_t row_pitch, int shape);
int stream_probe(const void* const* reads, int n_reads, void* const* writes, int n_writes, size_t bytes,
                 size_t row_pitch, int shape, hipStream_t st);

}  // namespace hawk
