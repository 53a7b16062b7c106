// The recurrent core of a Hawk block (temporal conv -> both gate projections -> RG-LRU scan
// fused with the output gate; hawk/hawk.py:172-198 upstream) as one host call per direction.
// The kernels are the ones the single entry points launch; what this file adds is the launch
// sequence with fewer small kernels around them: the fp32 gate weights are rounded to bf16 by
// one launch for both gates, and the three closing reductions of the backward (dLambda, the
// conv's dw / db, the projections' dw / db) run as one launch behind the last large kernel.
#include "hawk_scan.h"

namespace hawk {
namespace {

// fp32 -> bf16 (round to nearest even) of two arrays of `count` elements, count % 4 == 0.
__global__ __launch_bounds__(256) void round_pair_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                         bf16_t* __restrict__ a16, bf16_t* __restrict__ b16,
                                                         size_t quads) {
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < 2 * quads; i += step) {
        const bool second = i >= quads;
        const size_t q = second ? i - quads : i;
        const f32x4 v = reinterpret_cast<const f32x4*>(second ? b : a)[q];
        const u32x2 r = {pack_bf16x2(v.x, v.y), pack_bf16x2(v.z, v.w)};
        reinterpret_cast<u32x2*>(second ? b16 : a16)[q] = r;
    }
}

// Blocks [0, n0) run the dLambda reduction, [n0, n0 + n1) the conv's, the rest the projections'.
__global__ __launch_bounds__(kColsumThreads) void block_finish_kernel(ColsumTask dlam, ColsumTask conv,
                                                                      GateReduceTask gates, int n0, int n1) {
    __shared__ float s[kColsumSlices][kColsumCols];
    const int blk = (int)blockIdx.x;
    if (blk < n0) {
        colsum_block(dlam, blk, s);
    } else if (blk < n0 + n1) {
        colsum_block(conv, blk - n0, s);
    } else {
        const size_t nb = (size_t)((int)gridDim.x - n0 - n1);
        gate_reduce_span(gates, (size_t)(blk - n0 - n1) * kColsumThreads + threadIdx.x, nb * kColsumThreads);
    }
}

}  // namespace

int gate_weights_to_bf16(const float* w_i, const float* w_a, void* w_i16, void* w_a16, size_t count, hipStream_t st) {
    const size_t quads = count / 4;
    size_t blocks = (2 * quads + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    if (blocks == 0) return HAWK_OK;
    hipLaunchKernelGGL(round_pair_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w_i, w_a,
                       static_cast<bf16_t*>(w_i16), static_cast<bf16_t*>(w_a16), quads);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

int block_core_fwd(const void* xy, long long ld, const float* conv_w, const float* conv_b, const void* w_i,
                   const float* b_i, const void* w_a, const float* b_a, int w_dtype, void* w16, const float* lam,
                   void* u, void* xg, void* ag, void* h, void* out, void* h_last, int B, int T, int D, int nb,
                   void* scan_ws, size_t scan_ws_bytes, hipStream_t st) {
    const size_t wcount = (size_t)nb * (D / nb) * (D / nb);
    if (w_dtype == HAWK_DTYPE_F32 && w16 != nullptr) {
        bf16_t* dst = static_cast<bf16_t*>(w16);
        if (int rc = gate_weights_to_bf16(static_cast<const float*>(w_i), static_cast<const float*>(w_a), dst,
                                          dst + wcount, wcount, st))
            return rc;
        w_i = dst;
        w_a = dst + wcount;
        w_dtype = HAWK_DTYPE_BF16;
    }
    if (int rc = conv_gate_proj_fwd(xy, ld, conv_w, conv_b, w_i, b_i, w_a, b_a, u, xg, ag, B, T, D, nb, w_dtype, st))
        return rc;
    const void* y = static_cast<const bf16_t*>(xy) + D;
    return scan_gated_fwd(u, xg, ag, lam, y, ld, h, out, h_last, B, T, D, HAWK_DTYPE_BF16, HAWK_DTYPE_BF16, scan_ws,
                          scan_ws_bytes, st);
}

int block_core_bwd(const void* xy, long long ld, const void* u, const void* xg, const void* ag, const void* h,
                   const float* conv_w, const void* w_i, const void* w_a, int w_dtype, const float* lam,
                   const void* gout, void* d_xy, long long ldd, void* du, void* dxg, void* dag, float* d_conv_w,
                   float* d_conv_b, float* dw_i, float* db_i, float* dw_a, float* db_a, float* dlam, int B, int T,
                   int D, int nb, int W, void* scan_ws, size_t scan_ws_bytes, void* gate_ws, size_t gate_ws_bytes,
                   void* conv_ws, size_t conv_ws_bytes, hipStream_t st) {
    constexpr int bf = HAWK_DTYPE_BF16;
    const int M = B * T;
    const void* y = static_cast<const bf16_t*>(xy) + D;
    void* dy = static_cast<bf16_t*>(d_xy) + D;
    ColsumTask r_dlam, r_conv;
    GateReduceTask r_gates;
    if (int rc = scan_gated_bwd(u, xg, ag, lam, y, ld, h, gout, du, dxg, dag, dy, ldd, dlam, B, T, D, bf, bf, scan_ws,
                                scan_ws_bytes, st, &r_dlam))
        return rc;
    // the projections' input gradient accumulates onto the scan's, in place
    if (int rc = gate_proj_bwd_input(dxg, dag, w_i, w_a, du, du, M, D, nb, bf, w_dtype, bf, st)) return rc;
    // the conv's backward right behind the kernel that wrote its input gradient (part of that
    // tensor is then still in the memory-side cache), the weight gradients last
    if (int rc = conv1d_bwd(du, xy, ld, conv_w, d_xy, ldd, d_conv_w, d_conv_b, B, T, D, W, bf, bf, conv_ws,
                            conv_ws_bytes, st, &r_conv))
        return rc;
    if (int rc = gate_proj_bwd_weights(u, dxg, dag, dw_i, db_i, dw_a, db_a, M, D, nb, bf, bf, gate_ws, gate_ws_bytes,
                                       st, &r_gates))
        return rc;
    const int n0 = r_dlam.blocks(), n1 = r_conv.blocks();
    size_t n2 = (r_gates.items() + kColsumThreads - 1) / kColsumThreads;
    if (n2 > 2048) n2 = 2048;
    hipLaunchKernelGGL(block_finish_kernel, dim3((unsigned)(n0 + n1 + (int)n2)), dim3(kColsumThreads), 0, st, r_dlam,
                       r_conv, r_gates, n0, n1);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace hawk
