// Decode-step kernels for gfx950: one new token per batch row.
//
// Upstream issues about thirty small eager launches per layer and token for this
// (hawk/hawk.py:137-151, :169-179, :196-198; hawk/cache.py:29-43).  Here the conv window
// roll + conv is one launch and the RG-LRU state update is one launch; both update the
// cache buffers in place and work for any batch size.
#include "hawk_scan.h"

#include <stdint.h>

#include "hawk_device.h"

namespace hawk {

namespace {

constexpr int kMaxW = 8;

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// One thread per (batch row, V channels).  The thread reads its W-1 state rows and the new
// row, writes the conv output, then writes the state back shifted by one row.
template <typename ST, typename YT, int V>
__global__ __launch_bounds__(256) void conv1d_step_kernel(ST* __restrict__ state, const ST* __restrict__ x_new,
                                                         const float* __restrict__ w,
                                                         const float* __restrict__ bias, YT* __restrict__ y,
                                                         int D, int W, int nvec) {
    typedef typename Raw<ST, V>::type sraw_t;
    typedef typename Raw<YT, V>::type yraw_t;
    const int vc = blockIdx.x * blockDim.x + threadIdx.x;
    const int b = blockIdx.y;
    if (vc >= nvec) return;
    const int c0 = vc * V;
    const int H = W - 1;
    ST* sb = state + (size_t)b * H * D + c0;

    sraw_t rows[kMaxW];
#pragma unroll
    for (int j = 0; j < kMaxW - 1; ++j) {
        if (j < H) rows[j] = load_raw<ST, V>(sb + (size_t)j * D);
    }
    const sraw_t newest = load_raw<ST, V>(x_new + (size_t)b * D + c0);

    float acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = bias[c0 + v];
#pragma unroll
    for (int j = 0; j < kMaxW - 1; ++j) {
        if (j < H) {
            float xv[V];
            unpack(rows[j], xv);
#pragma unroll
            for (int v = 0; v < V; ++v) acc[v] = fmaf(w[(size_t)j * D + c0 + v], xv[v], acc[v]);
        }
    }
    {
        float xv[V];
        unpack(newest, xv);
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = fmaf(w[(size_t)H * D + c0 + v], xv[v], acc[v]);
    }
    yraw_t r;
    pack(acc, r);
    *reinterpret_cast<yraw_t*>(y + (size_t)b * D + c0) = r;

#pragma unroll
    for (int j = 0; j < kMaxW - 1; ++j) {
        if (j + 1 < H) *reinterpret_cast<sraw_t*>(sb + (size_t)j * D) = rows[j + 1];
    }
    if (H > 0) *reinterpret_cast<sraw_t*>(sb + (size_t)(H - 1) * D) = newest;
}

// h = alpha * state + sqrt(1 - alpha^2) * (sigmoid(x_rg_lru) * x); state <- h; h_out <- h.
// Optional, each switched by a non-null pointer (uniform over the launch):
//   bias_i, bias_a [D] fp32   added to the two gate logits first (the block-diagonal
//                             projections' biases), so the projections can skip them
//   y (rows ldy apart), out   out <- gelu(y) * h, the block's gate
template <typename ET, typename ST, int V>
__global__ __launch_bounds__(256) void rglru_step_kernel(const ET* __restrict__ x, const ET* __restrict__ xg,
                                                        const ET* __restrict__ ag,
                                                        const float* __restrict__ bias_i,
                                                        const float* __restrict__ bias_a,
                                                        const float* __restrict__ lam, const ET* __restrict__ y,
                                                        size_t ldy, ST* __restrict__ state, ET* __restrict__ h_out,
                                                        ET* __restrict__ out, int D, int nvec) {
    typedef typename Raw<ET, V>::type eraw_t;
    typedef typename Raw<ST, V>::type sraw_t;
    const int vc = blockIdx.x * blockDim.x + threadIdx.x;
    const int b = blockIdx.y;
    if (vc >= nvec) return;
    const int c0 = vc * V;
    const size_t o = (size_t)b * D + c0;
    float fx[V], fxg[V], fag[V], fs[V], hn[V];
    unpack(load_raw<ET, V>(x + o), fx);
    unpack(load_raw<ET, V>(xg + o), fxg);
    unpack(load_raw<ET, V>(ag + o), fag);
    unpack(load_raw<ST, V>(state + o), fs);
#pragma unroll
    for (int v = 0; v < V; ++v) {
        if (bias_i != nullptr) fxg[v] += bias_i[c0 + v];
        if (bias_a != nullptr) fag[v] += bias_a[c0 + v];
        hn[v] = rglru_step_value(fx[v], fxg[v], fag[v], softplus_precise(lam[c0 + v]), fs[v]);
    }
    eraw_t rh;
    sraw_t rs;
    pack(hn, rh);
    pack(hn, rs);
    if (h_out != nullptr) *reinterpret_cast<eraw_t*>(h_out + o) = rh;
    *reinterpret_cast<sraw_t*>(state + o) = rs;
    if (y != nullptr) {
        float fy[V], g[V];
        unpack(load_raw<ET, V>(y + (size_t)b * ldy + c0), fy);
#pragma unroll
        for (int v = 0; v < V; ++v) g[v] = gelu_times(fy[v], hn[v]);
        eraw_t ro;
        pack(g, ro);
        *reinterpret_cast<eraw_t*>(out + o) = ro;
    }
}

int pick_v(int D) { return (D % 4 == 0) ? 4 : ((D % 2 == 0) ? 2 : 1); }

template <typename ST, typename YT>
int conv_step_dispatch(void* state, const void* x_new, const float* w, const float* bias, void* y, int B, int D,
                       int W, hipStream_t st) {
    const int V = pick_v(D);
    const int nvec = D / V;
    const dim3 grid((unsigned)ceil_div(nvec, 256), (unsigned)B), block(256);
    ST* sp = static_cast<ST*>(state);
    const ST* xp = static_cast<const ST*>(x_new);
    YT* yp = static_cast<YT*>(y);
    if (V == 4) hipLaunchKernelGGL((conv1d_step_kernel<ST, YT, 4>), grid, block, 0, st, sp, xp, w, bias, yp, D, W, nvec);
    else if (V == 2) hipLaunchKernelGGL((conv1d_step_kernel<ST, YT, 2>), grid, block, 0, st, sp, xp, w, bias, yp, D, W, nvec);
    else hipLaunchKernelGGL((conv1d_step_kernel<ST, YT, 1>), grid, block, 0, st, sp, xp, w, bias, yp, D, W, nvec);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename ET, typename ST>
int rglru_step_dispatch(const void* x, const void* xg, const void* ag, const float* bias_i, const float* bias_a,
                        const float* lam, const void* y, long long ldy, void* state, void* h_out, void* out,
                        int B, int D, hipStream_t st) {
    int V = pick_v(D);
    // y may be a slice of a wider row: its vectors must stay aligned in every row
    while (V > 1 && y != nullptr &&
           ((ldy % V) != 0 || (reinterpret_cast<uintptr_t>(y) % (V * sizeof(ET))) != 0))
        V /= 2;
    const int nvec = D / V;
    const dim3 grid((unsigned)ceil_div(nvec, 256), (unsigned)B), block(256);
    const ET* xp = static_cast<const ET*>(x);
    const ET* xgp = static_cast<const ET*>(xg);
    const ET* agp = static_cast<const ET*>(ag);
    ST* sp = static_cast<ST*>(state);
    ET* hp = static_cast<ET*>(h_out);
    const ET* yp = static_cast<const ET*>(y);
    ET* op = static_cast<ET*>(out);
    const size_t ld = (size_t)ldy;
    if (V == 4)
        hipLaunchKernelGGL((rglru_step_kernel<ET, ST, 4>), grid, block, 0, st, xp, xgp, agp, bias_i, bias_a, lam, yp, ld,
                           sp, hp, op, D, nvec);
    else if (V == 2)
        hipLaunchKernelGGL((rglru_step_kernel<ET, ST, 2>), grid, block, 0, st, xp, xgp, agp, bias_i, bias_a, lam, yp, ld,
                           sp, hp, op, D, nvec);
    else
        hipLaunchKernelGGL((rglru_step_kernel<ET, ST, 1>), grid, block, 0, st, xp, xgp, agp, bias_i, bias_a, lam, yp, ld,
                           sp, hp, op, D, nvec);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace

int conv1d_step(void* conv_state, const void* x_new, const float* w, const float* bias, void* y, int B, int D,
                int W, int dtype, int y_dtype, hipStream_t st) {
    if (dtype == HAWK_DTYPE_BF16) {
        if (y_dtype == HAWK_DTYPE_BF16) return conv_step_dispatch<bf16_t, bf16_t>(conv_state, x_new, w, bias, y, B, D, W, st);
        return conv_step_dispatch<bf16_t, float>(conv_state, x_new, w, bias, y, B, D, W, st);
    }
    if (y_dtype == HAWK_DTYPE_BF16) return conv_step_dispatch<float, bf16_t>(conv_state, x_new, w, bias, y, B, D, W, st);
    return conv_step_dispatch<float, float>(conv_state, x_new, w, bias, y, B, D, W, st);
}

int rglru_step_gated(const void* x, const void* xg, const void* ag, const float* bias_i, const float* bias_a,
                     const float* lam, const void* y, long long ldy, void* state, void* h_out, void* out, int B,
                     int D, int dtype, int state_dtype, hipStream_t st) {
    if (dtype == HAWK_DTYPE_BF16) {
        if (state_dtype == HAWK_DTYPE_BF16)
            return rglru_step_dispatch<bf16_t, bf16_t>(x, xg, ag, bias_i, bias_a, lam, y, ldy, state, h_out, out, B, D, st);
        return rglru_step_dispatch<bf16_t, float>(x, xg, ag, bias_i, bias_a, lam, y, ldy, state, h_out, out, B, D, st);
    }
    if (state_dtype == HAWK_DTYPE_BF16)
        return rglru_step_dispatch<float, bf16_t>(x, xg, ag, bias_i, bias_a, lam, y, ldy, state, h_out, out, B, D, st);
    return rglru_step_dispatch<float, float>(x, xg, ag, bias_i, bias_a, lam, y, ldy, state, h_out, out, B, D, st);
}

int rglru_step(const void* x, const void* xg, const void* ag, const float* lam, void* state, void* h_out, int B,
               int D, int dtype, int state_dtype, hipStream_t st) {
    return rglru_step_gated(x, xg, ag, nullptr, nullptr, lam, nullptr, 0, state, h_out, nullptr, B, D, dtype,
                            state_dtype, st);
}

}  // namespace hawk
