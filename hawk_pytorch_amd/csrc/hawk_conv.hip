// Temporal causal depthwise conv1d for gfx950 (forward, backward, parameter-gradient reduce).
//
// Replaces Conv1D.doc_mask_forward of the upstream tree (hawk/external.py:49-95), which
// runs W x (slice, zero-pad, concat, multiply, add) full-tensor passes, and the autograd
// mirror of those passes.  Here forward and backward are one streaming pass each:
// a lane owns V adjacent channels and RT consecutive rows and keeps the W-1 halo rows in
// registers.  In the forward a workgroup's four waves take adjacent row chunks and hand each
// other their last W-1 rows through LDS, so only the first wave fetches history rows from memory
// (fetched by every wave they were 16 % more bytes read from memory, counted by rocprofv3; the
// kernel went from 56 to 51.5 us at B=8, T=4096, D=2560).  The backward's
// halo rows do come from cache (6 % more reads; keeping them in registers across a wave's
// chunks instead changed nothing).
#include "hawk_scan.h"

#include "hawk_device.h"

namespace hawk {

namespace {

constexpr int kConvWaves = 4;   // waves per workgroup, each on its own row chunk
constexpr int kConvRT = 16;     // rows per lane per chunk
constexpr int kConvMaxW = 8;

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// ---------------------------------------------------------------------------------------
// Forward, temporal width fixed at compile time.
// grid.x = row-chunk groups * channel tiles, grid.y = B; block = kConvWaves * 64.
// ---------------------------------------------------------------------------------------
template <typename XT, typename YT, int V, int W, int RT>
__global__ __launch_bounds__(kConvWaves * kWave) void conv1d_fwd_kernel(
    const XT* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
    const XT* __restrict__ state, YT* __restrict__ y, int T, int D, int nct, size_t ldx, size_t ldy) {
    typedef typename Raw<XT, V>::type xraw_t;
    typedef typename Raw<YT, V>::type yraw_t;
    constexpr int H = W - 1;
    // the last H rows of every wave's chunk, for the wave that owns the next chunk: only the
    // workgroup's first wave fetches its history rows from memory
    __shared__ xraw_t s_tail[kConvWaves][H > 0 ? H : 1][kWave];

    const int lane = threadIdx.x & (kWave - 1);
    const int wv = threadIdx.x / kWave;
    const int ct = blockIdx.x % nct;
    const int rg = blockIdx.x / nct;
    const int b = blockIdx.y;
    const int c_want = ct * kWave * V + lane * V;
    const bool lane_on = c_want < D;
    const int c0 = lane_on ? c_want : 0;
    const int t0 = (rg * kConvWaves + wv) * RT;

    const XT* xb = x + (size_t)b * T * ldx + c0;
    xraw_t raw[RT + H];
#pragma unroll
    for (int j = 0; j < RT; ++j) {
        const int t = t0 + j;
        raw[H + j] = (lane_on && t < T) ? load_raw<XT, V>(xb + (size_t)t * ldx) : raw_zero<xraw_t>();
    }
    if (wv == 0) {
#pragma unroll
        for (int j = 0; j < H; ++j) {
            const int t = t0 - H + j;
            if (!lane_on) raw[j] = raw_zero<xraw_t>();
            else if (t >= 0) raw[j] = load_raw<XT, V>(xb + (size_t)t * ldx);
            else if (state != nullptr) raw[j] = load_raw<XT, V>(state + ((size_t)b * H + (H + t)) * D + c0);
            else raw[j] = raw_zero<xraw_t>();
        }
    }
    if constexpr (H > 0) {
#pragma unroll
        for (int j = 0; j < H; ++j) s_tail[wv][j][lane] = raw[RT + j];
        __syncthreads();
        if (wv > 0) {
#pragma unroll
            for (int j = 0; j < H; ++j) raw[j] = s_tail[wv - 1][j][lane];
        }
    }
    if (!lane_on || t0 >= T) return;

    float wk[W][V], bk[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        bk[v] = bias[c0 + v];
#pragma unroll
        for (int k = 0; k < W; ++k) wk[k][v] = w[(size_t)k * D + c0 + v];
    }
    float win[W][V];
#pragma unroll
    for (int k = 0; k < H; ++k) unpack(raw[k], win[k]);

    YT* yb = y + (size_t)b * T * ldy + c0;
#pragma unroll
    for (int j = 0; j < RT; ++j) {
        unpack(raw[H + j], win[H]);
        float out[V];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float acc = bk[v];
#pragma unroll
            for (int k = 0; k < W; ++k) acc = fmaf(wk[k][v], win[k][v], acc);  // win[k] is row t-(W-1-k)
            out[v] = acc;
        }
        if (t0 + j < T) {
            yraw_t r;
            pack(out, r);
            store_raw<YT, V>(yb + (size_t)(t0 + j) * ldy, r);
        }
#pragma unroll
        for (int k = 0; k < H; ++k) {
#pragma unroll
            for (int v = 0; v < V; ++v) win[k][v] = win[k + 1][v];
        }
    }
}

// Forward for any 1 <= W <= kConvMaxW: one thread per (row, V channels); history rows are
// re-read through the cache.  Not a tuned path (Hawk uses W = 4).
template <typename XT, typename YT, int V>
__global__ __launch_bounds__(256) void conv1d_fwd_anyw_kernel(
    const XT* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
    const XT* __restrict__ state, YT* __restrict__ y, int T, int D, int W, int nvec, size_t ldx, size_t ldy) {
    typedef typename Raw<YT, V>::type yraw_t;
    const int vc = blockIdx.x * blockDim.x + threadIdx.x;
    const int t = blockIdx.y;
    const int b = blockIdx.z;
    if (vc >= nvec) return;
    const int c0 = vc * V;
    const int H = W - 1;
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = bias[c0 + v];
    for (int s = 0; s < W; ++s) {
        const int tt = t - s;
        float xv[V];
        if (tt >= 0) {
            unpack(load_raw<XT, V>(x + ((size_t)b * T + tt) * ldx + c0), xv);
        } else if (state != nullptr) {
            unpack(load_raw<XT, V>(state + ((size_t)b * H + (H + tt)) * D + c0), xv);
        } else {
            continue;
        }
#pragma unroll
        for (int v = 0; v < V; ++v) acc[v] = fmaf(w[(size_t)(W - 1 - s) * D + c0 + v], xv[v], acc[v]);
    }
    yraw_t r;
    pack(acc, r);
    store_raw<YT, V>(y + ((size_t)b * T + t) * ldy + c0, r);
}

// ---------------------------------------------------------------------------------------
// Backward, temporal width fixed at compile time.  A wave walks `chunks` consecutive
// row chunks, accumulating dw / db for its channels in registers; the workgroup's waves
// are then summed through LDS into one row of the [rows, (W+1) D] partial buffer.
// grid.x = row groups * channel tiles, grid.y = B.
// ---------------------------------------------------------------------------------------
template <typename XT, typename GT, int V, int W, int RT>
__global__ __launch_bounds__(kConvWaves * kWave) void conv1d_bwd_kernel(
    const GT* __restrict__ gy, const XT* __restrict__ x, const float* __restrict__ w,
    XT* __restrict__ dx, float* __restrict__ part, int T, int D, int nct, int chunks, size_t ldx, size_t lddx) {
    typedef typename Raw<XT, V>::type xraw_t;
    typedef typename Raw<GT, V>::type graw_t;
    constexpr int H = W - 1;
    constexpr int CT = kWave * V;

    __shared__ float s_acc[kConvWaves][W + 1][CT];

    const int lane = threadIdx.x & (kWave - 1);
    const int wv = threadIdx.x / kWave;
    const int ct = blockIdx.x % nct;
    const int rg = blockIdx.x / nct;
    const int b = blockIdx.y;
    const int c_want = ct * CT + lane * V;
    const bool lane_on = c_want < D;
    const int c0 = lane_on ? c_want : 0;

    float wk[W][V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
#pragma unroll
        for (int k = 0; k < W; ++k) wk[k][v] = w[(size_t)k * D + c0 + v];
    }
    float dwk[W][V], dbk[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        dbk[v] = 0.0f;
#pragma unroll
        for (int k = 0; k < W; ++k) dwk[k][v] = 0.0f;
    }

    const GT* gb = gy + (size_t)b * T * D + c0;
    const XT* xb = x + (size_t)b * T * ldx + c0;
    XT* dxb = dx + (size_t)b * T * lddx + c0;

    for (int ch = 0; ch < chunks; ++ch) {
        const int t0 = ((rg * kConvWaves + wv) * chunks + ch) * RT;
        if (t0 >= T || !lane_on) break;
        graw_t graw[RT + H];  // grad_y rows t0 .. t0+RT+H-1
        xraw_t xraw[RT + H];  // x rows t0-H .. t0+RT-1
#pragma unroll
        for (int j = 0; j < RT + H; ++j) {
            const int tg = t0 + j;
            graw[j] = (tg < T) ? load_raw<GT, V>(gb + (size_t)tg * D) : raw_zero<graw_t>();
            const int tx = t0 - H + j;
            xraw[j] = (tx >= 0 && tx < T) ? load_raw<XT, V>(xb + (size_t)tx * ldx) : raw_zero<xraw_t>();
        }
        float gwin[W][V], xwin[W][V];
#pragma unroll
        for (int k = 0; k < H; ++k) {
            unpack(graw[k], gwin[k]);
            unpack(xraw[k], xwin[k]);
        }
#pragma unroll
        for (int j = 0; j < RT; ++j) {
            // gwin[k] = grad_y row t+k, xwin[k] = x row t-(W-1-k), for t = t0 + j
            unpack(graw[H + j], gwin[H]);
            unpack(xraw[H + j], xwin[H]);
            float out[V];
#pragma unroll
            for (int v = 0; v < V; ++v) {
                float acc = 0.0f;
#pragma unroll
                for (int s = 0; s < W; ++s) acc = fmaf(wk[W - 1 - s][v], gwin[s][v], acc);
                out[v] = acc;
                const float g = gwin[0][v];  // zero past T
                dbk[v] += g;
#pragma unroll
                for (int k = 0; k < W; ++k) dwk[k][v] = fmaf(g, xwin[k][v], dwk[k][v]);
            }
            if (t0 + j < T) {
                xraw_t r;
                pack(out, r);
                store_raw<XT, V>(dxb + (size_t)(t0 + j) * lddx, r);
            }
#pragma unroll
            for (int k = 0; k < H; ++k) {
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    gwin[k][v] = gwin[k + 1][v];
                    xwin[k][v] = xwin[k + 1][v];
                }
            }
        }
    }

#pragma unroll
    for (int v = 0; v < V; ++v) {
#pragma unroll
        for (int k = 0; k < W; ++k) s_acc[wv][k][lane * V + v] = dwk[k][v];
        s_acc[wv][W][lane * V + v] = dbk[v];
    }
    __syncthreads();
    if (wv == 0 && lane_on) {
        float* prow = part + ((size_t)rg * gridDim.y + b) * (size_t)(W + 1) * D;
#pragma unroll
        for (int k = 0; k <= W; ++k) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                float sum = 0.0f;
#pragma unroll
                for (int q = 0; q < kConvWaves; ++q) sum += s_acc[q][k][lane * V + v];
                prow[(size_t)k * D + c0 + v] = sum;
            }
        }
    }
}

// Backward for any W: dx by direct evaluation, dw/db partials per (row group, batch).
template <typename XT, typename GT>
__global__ __launch_bounds__(256) void conv1d_bwd_anyw_kernel(
    const GT* __restrict__ gy, const XT* __restrict__ x, const float* __restrict__ w,
    XT* __restrict__ dx, float* __restrict__ part, int T, int D, int W, int rows_per_group, size_t ldx, size_t lddx) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int rg = blockIdx.y;
    const int b = blockIdx.z;
    if (c >= D) return;
    float dwk[kConvMaxW], dbk = 0.0f;
#pragma unroll
    for (int k = 0; k < kConvMaxW; ++k) dwk[k] = 0.0f;
    const int t_begin = rg * rows_per_group;
    const int t_end = min(T, t_begin + rows_per_group);
    for (int t = t_begin; t < t_end; ++t) {
        float acc = 0.0f;
        float g0[1];
        unpack(load_raw<GT, 1>(gy + ((size_t)b * T + t) * D + c), g0);
#pragma unroll
        for (int s = 0; s < kConvMaxW; ++s) {
            if (s < W) {
                if (t + s < T) {
                    float gv[1];
                    unpack(load_raw<GT, 1>(gy + ((size_t)b * T + t + s) * D + c), gv);
                    acc = fmaf(w[(size_t)(W - 1 - s) * D + c], gv[0], acc);
                }
                if (t - s >= 0) {
                    float xv[1];
                    unpack(load_raw<XT, 1>(x + ((size_t)b * T + t - s) * ldx + c), xv);
                    dwk[s] = fmaf(g0[0], xv[0], dwk[s]);  // slot s holds dw[W-1-s]
                }
            }
        }
        dbk += g0[0];
        float o[1] = {acc};
        typename Raw<XT, 1>::type r;
        pack(o, r);
        store_raw<XT, 1>(dx + ((size_t)b * T + t) * lddx + c, r);
    }
    float* prow = part + ((size_t)rg * gridDim.z + b) * (size_t)(W + 1) * D;
#pragma unroll
    for (int s = 0; s < kConvMaxW; ++s) {
        if (s < W) prow[(size_t)(W - 1 - s) * D + c] = dwk[s];
    }
    prow[(size_t)W * D + c] = dbk;
}

// Column sums of the [rows, (W + 1) D] partials in a fixed order: dw, then db.
__global__ __launch_bounds__(kColsumThreads) void colsum_kernel(ColsumTask t) {
    __shared__ float s[kColsumSlices][kColsumCols];
    colsum_block(t, (int)blockIdx.x, s);
}

// Channels per lane: every row of every tensor must start on a multiple of it.
int pick_v4(int D, size_t ld_a, size_t ld_b) {
    if (D % 4 == 0 && ld_a % 4 == 0 && ld_b % 4 == 0) return 4;
    if (D % 2 == 0 && ld_a % 2 == 0 && ld_b % 2 == 0) return 2;
    return 1;
}

// Rows of time covered by one backward workgroup (all its waves and chunks).
int bwd_rows_per_group(int T) {
    const int chunks = T >= 4096 ? 4 : (T >= 1024 ? 2 : 1);
    return chunks;
}

template <typename XT, typename YT>
int fwd_dispatch(const void* x, const float* w, const float* bias, const void* state, void* y, int B, int T, int D,
                 int W, size_t ldx, size_t ldy, hipStream_t st) {
    const XT* xp = static_cast<const XT*>(x);
    const XT* sp = static_cast<const XT*>(state);
    YT* yp = static_cast<YT*>(y);
    const int V = pick_v4(D, ldx, ldy);
    if (W == 4) {
        const int nct = ceil_div(D, kWave * V);
        const int nrg = ceil_div(T, kConvWaves * kConvRT);
        const dim3 grid((unsigned)(nct * nrg), (unsigned)B), block(kConvWaves * kWave);
        if (V == 4) hipLaunchKernelGGL((conv1d_fwd_kernel<XT, YT, 4, 4, kConvRT>), grid, block, 0, st, xp, w, bias, sp, yp, T, D, nct, ldx, ldy);
        else if (V == 2) hipLaunchKernelGGL((conv1d_fwd_kernel<XT, YT, 2, 4, kConvRT>), grid, block, 0, st, xp, w, bias, sp, yp, T, D, nct, ldx, ldy);
        else hipLaunchKernelGGL((conv1d_fwd_kernel<XT, YT, 1, 4, kConvRT>), grid, block, 0, st, xp, w, bias, sp, yp, T, D, nct, ldx, ldy);
    } else {
        const int nvec = D / V;
        const dim3 grid((unsigned)ceil_div(nvec, 256), (unsigned)T, (unsigned)B), block(256);
        if (V == 4) hipLaunchKernelGGL((conv1d_fwd_anyw_kernel<XT, YT, 4>), grid, block, 0, st, xp, w, bias, sp, yp, T, D, W, nvec, ldx, ldy);
        else if (V == 2) hipLaunchKernelGGL((conv1d_fwd_anyw_kernel<XT, YT, 2>), grid, block, 0, st, xp, w, bias, sp, yp, T, D, W, nvec, ldx, ldy);
        else hipLaunchKernelGGL((conv1d_fwd_anyw_kernel<XT, YT, 1>), grid, block, 0, st, xp, w, bias, sp, yp, T, D, W, nvec, ldx, ldy);
    }
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

struct BwdPlan {
    int chunks, rows_per_group, ngroups;
};
BwdPlan bwd_plan(int T, int W) {
    BwdPlan p;
    if (W == 4) {
        p.chunks = bwd_rows_per_group(T);
        p.rows_per_group = kConvWaves * kConvRT * p.chunks;
    } else {
        p.chunks = 1;
        p.rows_per_group = 64;
    }
    p.ngroups = ceil_div(T, p.rows_per_group);
    return p;
}

template <typename XT, typename GT>
int bwd_dispatch(const void* gy, const void* x, const float* w, void* dx, float* dw, float* db, int B, int T, int D,
                 int W, size_t ldx, size_t lddx, float* part, hipStream_t st, ColsumTask* deferred) {
    const GT* gp = static_cast<const GT*>(gy);
    const XT* xp = static_cast<const XT*>(x);
    XT* dxp = static_cast<XT*>(dx);
    const BwdPlan p = bwd_plan(T, W);
    if (W == 4) {
        const int V = pick_v4(D, ldx, lddx);
        const int nct = ceil_div(D, kWave * V);
        const dim3 grid((unsigned)(nct * p.ngroups), (unsigned)B), block(kConvWaves * kWave);
        if (V == 4) hipLaunchKernelGGL((conv1d_bwd_kernel<XT, GT, 4, 4, kConvRT>), grid, block, 0, st, gp, xp, w, dxp, part, T, D, nct, p.chunks, ldx, lddx);
        else if (V == 2) hipLaunchKernelGGL((conv1d_bwd_kernel<XT, GT, 2, 4, kConvRT>), grid, block, 0, st, gp, xp, w, dxp, part, T, D, nct, p.chunks, ldx, lddx);
        else hipLaunchKernelGGL((conv1d_bwd_kernel<XT, GT, 1, 4, kConvRT>), grid, block, 0, st, gp, xp, w, dxp, part, T, D, nct, p.chunks, ldx, lddx);
    } else {
        const dim3 grid((unsigned)ceil_div(D, 256), (unsigned)p.ngroups, (unsigned)B), block(256);
        hipLaunchKernelGGL((conv1d_bwd_anyw_kernel<XT, GT>), grid, block, 0, st, gp, xp, w, dxp, part, T, D, W, p.rows_per_group, ldx, lddx);
    }
    if (hipGetLastError() != hipSuccess) return HAWK_ERR_LAUNCH;
    const ColsumTask reduce{part, dw, db, nullptr, p.ngroups * B, (W + 1) * D, W * D};
    if (deferred != nullptr) {   // the caller runs it, together with its other closing reductions
        *deferred = reduce;
        return HAWK_OK;
    }
    hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)reduce.blocks()), dim3(kColsumThreads), 0, st, reduce);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace

int conv1d_fwd(const void* x, long long ldx, const float* w, const float* bias, const void* state, void* y,
               long long ldy, int B, int T, int D, int W, int x_dtype, int y_dtype, hipStream_t st) {
    const size_t lx = (size_t)ldx, ly = (size_t)ldy;
    if (x_dtype == HAWK_DTYPE_BF16) {
        if (y_dtype == HAWK_DTYPE_BF16) return fwd_dispatch<bf16_t, bf16_t>(x, w, bias, state, y, B, T, D, W, lx, ly, st);
        return fwd_dispatch<bf16_t, float>(x, w, bias, state, y, B, T, D, W, lx, ly, st);
    }
    if (y_dtype == HAWK_DTYPE_BF16) return fwd_dispatch<float, bf16_t>(x, w, bias, state, y, B, T, D, W, lx, ly, st);
    return fwd_dispatch<float, float>(x, w, bias, state, y, B, T, D, W, lx, ly, st);
}

size_t conv1d_bwd_workspace_bytes(int B, int T, int D, int W) {
    const BwdPlan p = bwd_plan(T, W);
    return align_up((size_t)p.ngroups * B * (size_t)(W + 1) * D * sizeof(float), 256);
}

int conv1d_bwd(const void* gy, const void* x, long long ldx, const float* w, void* dx, long long lddx, float* dw,
               float* db, int B, int T, int D, int W, int x_dtype, int gy_dtype, void* ws, size_t ws_bytes,
               hipStream_t st, ColsumTask* deferred) {
    if (ws == nullptr || ws_bytes < conv1d_bwd_workspace_bytes(B, T, D, W)) return HAWK_ERR_WORKSPACE;
    float* part = static_cast<float*>(ws);
    const size_t lx = (size_t)ldx, ld = (size_t)lddx;
    if (x_dtype == HAWK_DTYPE_BF16) {
        if (gy_dtype == HAWK_DTYPE_BF16)
            return bwd_dispatch<bf16_t, bf16_t>(gy, x, w, dx, dw, db, B, T, D, W, lx, ld, part, st, deferred);
        return bwd_dispatch<bf16_t, float>(gy, x, w, dx, dw, db, B, T, D, W, lx, ld, part, st, deferred);
    }
    if (gy_dtype == HAWK_DTYPE_BF16) return bwd_dispatch<float, bf16_t>(gy, x, w, dx, dw, db, B, T, D, W, lx, ld, part, st, deferred);
    return bwd_dispatch<float, float>(gy, x, w, dx, dw, db, B, T, D, W, lx, ld, part, st, deferred);
}

}  // namespace hawk
