// RG-LRU linear scan for gfx950: forward h_t = alpha_t h_{t-1} + beta_t and the reverse-time
// backward, each as ONE pass over HBM.
//
// Replaces the two Triton kernels of the upstream tree (hawk/scan_fused.py:34-109 and
// :112-317), which walk all T steps serially in one wavefront per (batch, 64 channels).
//
// Layout.  Activations are [B,T,D] row-major.  A workgroup owns one tile of
//   TS = NW*TC consecutive time rows  x  CT = 64*V consecutive channels  of one batch row.
// Each lane owns V adjacent channels (one V*sizeof(elem)-byte load per row, so a wavefront
// reads 64*V contiguous elements of a row) and TC consecutive rows; wave w of the
// workgroup owns time slice w of the tile.  The whole tile stays in registers between the
// local scan and the carry fix-up, so every input byte is read once and every output byte
// written once.
//
// The recurrence is associative under (P,H) o (P',H') = (P P', P' H + H'):
//   1. each lane scans its TC rows from a zero state, keeping per row the running product
//      P_j and the local state H_j, and ends with the slice aggregate (P, H);
//   2. slice aggregates are combined across the NW waves through LDS;
//   3. tile aggregates are combined across workgroups with a look-back over per-channel
//      words in a caller-provided workspace: a tile publishes its aggregate, folds the
//      aggregates of its predecessors back to the nearest checkpoint tile, and adds that
//      checkpoint's inclusive state (checkpoint tiles publish theirs once they have it);
//   4. the carry is applied: h_j = H_j + P_j * carry, rounded once and stored.
// The backward runs the same machinery in reverse time on c_t = alpha_t (gout_t + c_{t+1}).
//
// Look-back words are 64 bits: a 32-bit launch tag and an fp32 payload, written and read
// with single relaxed device-scope atomics, so no fences are needed and a stale word from
// an earlier launch can never be mistaken for a fresh one.  Tiles take their position in
// the chain from an atomic ticket, so a tile only ever waits for tiles that have already
// started; the wait is also bounded, and a tile that exhausts it raises the workspace's
// error word and finishes (with a wrong carry) instead of hanging.
#include "hawk_scan.h"

#include "hawk_device.h"

namespace hawk {

namespace {

constexpr uint32_t kSpinLimit = 1u << 22;

enum CtrlWord { kTicket = 0, kDone = 1, kEpoch = 2, kError = 3 };

struct ScanWsPtrs {
    uint32_t* ctrl;
    unsigned long long* incl;  // [nseg][B][D] inclusive state at the end of a tile
    unsigned long long* agg_p; // [nseg][B][D] tile aggregate: product of alpha
    unsigned long long* agg_h; // [nseg][B][D] tile aggregate: state from zero
    float* dlam_part;          // [nseg][B][D] per-tile partial sums for dLambda
};

__device__ __forceinline__ void publish(unsigned long long* p, uint32_t tag, float v) {
    unsigned long long w = ((unsigned long long)tag << 32) | (unsigned long long)__float_as_uint(v);
    __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool try_read(const unsigned long long* p, uint32_t tag, float& v) {
    unsigned long long w = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v = __uint_as_float((uint32_t)w);
    return (uint32_t)(w >> 32) == tag;
}

// Every kCheckpointEvery-th chain position is a checkpoint: it publishes the inclusive
// state at its end; every other position publishes only its own aggregate.  A tile folds
// the aggregates of its predecessors back to the nearest checkpoint and finishes with that
// checkpoint's inclusive state.  The order of the floating-point operations is therefore
// fixed by the position alone, never by timing, so results are bitwise reproducible, and
// the serial dependency runs over checkpoints only (nseg / kCheckpointEvery hops).
constexpr int kCheckpointEvery = 8;

__device__ __forceinline__ bool is_checkpoint(int pos) { return (pos % kCheckpointEvery) == 0; }

// Return the state carried into chain position `pos` (pos >= 1) for one channel.  `stride`
// is the distance in words between consecutive chain positions of the same channel.
__device__ __forceinline__ float look_back(const ScanWsPtrs& ws, size_t idx_pos0, size_t stride,
                                           int pos, uint32_t tag) {
    float acc_p = 1.0f, acc_h = 0.0f;
    int j = pos - 1;
    uint32_t spins = 0;
    while (true) {
        const size_t idx = idx_pos0 + (size_t)j * stride;
        if (is_checkpoint(j)) {
            float vi;
            if (try_read(ws.incl + idx, tag, vi)) return fmaf(acc_p, vi, acc_h);
        } else {
            float vp, vh;
            const bool okp = try_read(ws.agg_p + idx, tag, vp);
            const bool okh = try_read(ws.agg_h + idx, tag, vh);
            if (okp && okh) {
                acc_h = fmaf(acc_p, vh, acc_h);
                acc_p *= vp;
                --j;
                continue;
            }
        }
        if (++spins > kSpinLimit) {
            __hip_atomic_store(ws.ctrl + kError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return acc_h;
        }
        __builtin_amdgcn_s_sleep(4);
    }
}

// Take a ticket (chain-ordered tile index) and the launch tag.  One barrier.
__device__ __forceinline__ void take_ticket(uint32_t* ctrl, uint32_t* s_ticket, uint32_t& ticket,
                                            uint32_t& tag) {
    if (threadIdx.x == 0) {
        s_ticket[0] = __hip_atomic_fetch_add(ctrl + kTicket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_ticket[1] = __hip_atomic_load(ctrl + kEpoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
    }
    __syncthreads();
    ticket = s_ticket[0];
    tag = s_ticket[1];
}

// Last tile out re-arms the control block for the next launch on the same workspace.
__device__ __forceinline__ void retire(uint32_t* ctrl, uint32_t total, uint32_t tag) {
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t d = __hip_atomic_fetch_add(ctrl + kDone, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d == total - 1u) {
            __hip_atomic_store(ctrl + kTicket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(ctrl + kDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(ctrl + kEpoch, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// ---------------------------------------------------------------------------------------
// Forward
// ---------------------------------------------------------------------------------------
template <typename ET, int V, int TC, int NW, bool PRECISE>
__global__ __launch_bounds__(NW * kWave) void rglru_scan_fwd_kernel(
    const ET* __restrict__ x, const ET* __restrict__ xg, const ET* __restrict__ ag,
    const float* __restrict__ lam, ET* __restrict__ h, int B, int T, int D, int nseg, int nct,
    ScanWsPtrs ws) {
    typedef typename Raw<ET, V>::type raw_t;
    constexpr int CT = kWave * V;
    constexpr int TS = NW * TC;

    __shared__ float2 s_agg[NW][CT];
    __shared__ float s_cin[CT];
    __shared__ uint32_t s_ticket[2];

    uint32_t ticket = blockIdx.x, tag = 0;
    const uint32_t total = (uint32_t)nseg * (uint32_t)B * (uint32_t)nct;
    if (nseg > 1) take_ticket(ws.ctrl, s_ticket, ticket, tag);

    const int per_seg = B * nct;
    const int seg = ticket / per_seg;
    const int rem = ticket - seg * per_seg;
    const int b = rem / nct;
    const int ct = rem - b * nct;

    const int lane = threadIdx.x & (kWave - 1);
    const int w = threadIdx.x / kWave;
    const int c_want = ct * CT + lane * V;
    const bool lane_on = c_want < D;
    const int c0 = lane_on ? c_want : D - V;  // idle lanes shadow the last valid channels
    const int t0 = seg * TS + w * TC;

    const size_t base = ((size_t)b * T + t0) * D + c0;
    raw_t rx[TC], rxg[TC], rag[TC];
    const bool full = (t0 + TC <= T);
    if (full) {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const size_t o = base + (size_t)j * D;
            rx[j] = load_raw<ET, V>(x + o);
            rxg[j] = load_raw<ET, V>(xg + o);
            rag[j] = load_raw<ET, V>(ag + o);
        }
    } else {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const size_t o = base + (size_t)j * D;
            const bool ok = t0 + j < T;
            rx[j] = ok ? load_raw<ET, V>(x + o) : raw_zero<raw_t>();
            rxg[j] = ok ? load_raw<ET, V>(xg + o) : raw_zero<raw_t>();
            rag[j] = ok ? load_raw<ET, V>(ag + o) : raw_zero<raw_t>();
        }
    }

    // Per-channel constants: log2(alpha) = c2 * r, 2 ln(alpha) = cn * r.
    float c2[V], cn[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float s = softplus_precise(lam[c0 + v]);
        c2[v] = -8.0f * kLog2e * s;
        cn[v] = -16.0f * s;
    }

    // 1. local scan from a zero state
    float pj[TC][V], hj[TC][V];
    float p_run[V], h_run[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { p_run[v] = 1.0f; h_run[v] = 0.0f; }
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        float fx[V], fxg[V], fag[V];
        unpack(rx[j], fx);
        unpack(rxg[j], fxg);
        unpack(rag[j], fag);
        const bool ok = full || (t0 + j < T);
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float i = sigmoid_fast(fxg[v]);
            const float r = sigmoid_fast(fag[v]);
            float alpha = hw_exp2(c2[v] * r);
            const float z = PRECISE ? one_minus_exp(cn[v] * r) : clamp01(fmaf(-alpha, alpha, 1.0f));
            float beta = hw_sqrt(z) * (i * fx[v]);
            if (!ok) { alpha = 1.0f; beta = 0.0f; }  // rows past T are the identity
            h_run[v] = fmaf(alpha, h_run[v], beta);
            p_run[v] *= alpha;
            pj[j][v] = p_run[v];
            hj[j][v] = h_run[v];
        }
    }

    // 2. combine the NW time slices of this tile
#pragma unroll
    for (int v = 0; v < V; ++v) s_agg[w][lane * V + v] = make_float2(p_run[v], h_run[v]);
    __syncthreads();
    float p_pre[V], h_pre[V], p_tot[V], h_tot[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { p_tot[v] = 1.0f; h_tot[v] = 0.0f; p_pre[v] = 1.0f; h_pre[v] = 0.0f; }
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if (ww == w) { p_pre[v] = p_tot[v]; h_pre[v] = h_tot[v]; }
            const float2 a = s_agg[ww][lane * V + v];
            h_tot[v] = fmaf(a.x, h_tot[v], a.y);
            p_tot[v] *= a.x;
        }
    }

    // 3. carry across tiles
    float cin[V];
#pragma unroll
    for (int v = 0; v < V; ++v) cin[v] = 0.0f;
    if (nseg > 1) {
        if (w == 0) {
            const size_t stride = (size_t)B * D;
            const size_t idx0 = (size_t)b * D + c0;  // chain position 0 of this channel
            const size_t idx = idx0 + (size_t)seg * stride;
            const bool publishes = seg + 1 < nseg;
            if (publishes && !is_checkpoint(seg)) {
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    publish(ws.agg_p + idx + v, tag, p_tot[v]);
                    publish(ws.agg_h + idx + v, tag, h_tot[v]);
                }
                asm volatile("" ::: "memory");
            }
            if (seg > 0) {
#pragma unroll
                for (int v = 0; v < V; ++v) cin[v] = look_back(ws, idx0 + v, stride, seg, tag);
            }
            if (publishes && is_checkpoint(seg)) {
#pragma unroll
                for (int v = 0; v < V; ++v) publish(ws.incl + idx + v, tag, fmaf(p_tot[v], cin[v], h_tot[v]));
            }
#pragma unroll
            for (int v = 0; v < V; ++v) s_cin[lane * V + v] = cin[v];
        }
        __syncthreads();
#pragma unroll
        for (int v = 0; v < V; ++v) cin[v] = s_cin[lane * V + v];
    }

    // 4. apply the carry and store
    float cw[V];
#pragma unroll
    for (int v = 0; v < V; ++v) cw[v] = fmaf(p_pre[v], cin[v], h_pre[v]);
    if (lane_on) {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            if (full || (t0 + j < T)) {
                float out[V];
#pragma unroll
                for (int v = 0; v < V; ++v) out[v] = fmaf(pj[j][v], cw[v], hj[j][v]);
                raw_t r;
                pack(out, r);
                store_raw<ET, V>(h + base + (size_t)j * D, r);
            }
        }
    }

    if (nseg > 1) retire(ws.ctrl, total, tag);
}

// ---------------------------------------------------------------------------------------
// Backward.  Reverse chain on c_t = alpha_t (gout_t + c_{t+1}); g_t = gout_t + c_{t+1}.
// Per element, everything that multiplies g_t is precomputed in the local pass:
//   dx = g K1, dx_rg_lru = g K2, da_rg_lru = g K3, dLambda += g K4 (scaled per channel later)
//   K1 = m i;  K2 = m x i (1-i);  K4 = (h_{t-1} alpha - i x alpha^2 2 csg(1-alpha^2)) r;
//   K3 = K4 (1-r) (-8 softplus(Lambda)).
// ---------------------------------------------------------------------------------------
template <typename ET, int V, int TC, int NW, bool PRECISE>
__global__ __launch_bounds__(NW * kWave) void rglru_scan_bwd_kernel(
    const ET* __restrict__ x, const ET* __restrict__ xg, const ET* __restrict__ ag,
    const float* __restrict__ lam, const ET* __restrict__ hs, const ET* __restrict__ gout,
    ET* __restrict__ dx, ET* __restrict__ dxg, ET* __restrict__ dag, int B, int T, int D, int nseg,
    int nct, ScanWsPtrs ws) {
    typedef typename Raw<ET, V>::type raw_t;
    constexpr int CT = kWave * V;
    constexpr int TS = NW * TC;

    __shared__ float2 s_agg[NW][CT];
    __shared__ float s_cin[CT];
    __shared__ float s_dl[NW][CT];
    __shared__ uint32_t s_ticket[2];

    uint32_t ticket = blockIdx.x, tag = 0;
    const uint32_t total = (uint32_t)nseg * (uint32_t)B * (uint32_t)nct;
    if (nseg > 1) take_ticket(ws.ctrl, s_ticket, ticket, tag);

    const int per_seg = B * nct;
    const int pos = ticket / per_seg;  // chain position: 0 is the LAST time tile
    const int seg = nseg - 1 - pos;
    const int rem = ticket - pos * per_seg;
    const int b = rem / nct;
    const int ct = rem - b * nct;

    const int lane = threadIdx.x & (kWave - 1);
    const int w = threadIdx.x / kWave;
    const int c_want = ct * CT + lane * V;
    const bool lane_on = c_want < D;
    const int c0 = lane_on ? c_want : D - V;
    const int t0 = seg * TS + w * TC;

    const size_t base = ((size_t)b * T + t0) * D + c0;
    raw_t rx[TC], rxg[TC], rag[TC], rgo[TC], rhp[TC];
    const bool full = (t0 + TC <= T) && (t0 > 0);
    if (full) {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const size_t o = base + (size_t)j * D;
            rx[j] = load_raw<ET, V>(x + o);
            rxg[j] = load_raw<ET, V>(xg + o);
            rag[j] = load_raw<ET, V>(ag + o);
            rgo[j] = load_raw<ET, V>(gout + o);
            rhp[j] = load_raw<ET, V>(hs + o - D);
        }
    } else {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            const size_t o = base + (size_t)j * D;
            const bool ok = t0 + j < T;
            rx[j] = ok ? load_raw<ET, V>(x + o) : raw_zero<raw_t>();
            rxg[j] = ok ? load_raw<ET, V>(xg + o) : raw_zero<raw_t>();
            rag[j] = ok ? load_raw<ET, V>(ag + o) : raw_zero<raw_t>();
            rgo[j] = ok ? load_raw<ET, V>(gout + o) : raw_zero<raw_t>();
            rhp[j] = (ok && t0 + j > 0) ? load_raw<ET, V>(hs + o - D) : raw_zero<raw_t>();
        }
    }

    float c2[V], cs[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float s = softplus_precise(lam[c0 + v]);
        c2[v] = -8.0f * kLog2e * s;
        cs[v] = -8.0f * s;
    }

    // 1. local reverse scan from a zero carry
    float qn[TC][V], gl[TC][V], k1[TC][V], k2[TC][V], k3[TC][V];
    float q_run[V], c_run[V], acc_a[V], acc_q[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { q_run[v] = 1.0f; c_run[v] = 0.0f; acc_a[v] = 0.0f; acc_q[v] = 0.0f; }
#pragma unroll
    for (int j = TC - 1; j >= 0; --j) {
        float fx[V], fxg[V], fag[V], fgo[V], fhp[V];
        unpack(rx[j], fx);
        unpack(rxg[j], fxg);
        unpack(rag[j], fag);
        unpack(rgo[j], fgo);
        unpack(rhp[j], fhp);
        const bool ok = full || (t0 + j < T);
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float i = sigmoid_fast(fxg[v]);
            const float r = sigmoid_fast(fag[v]);
            float alpha = hw_exp2(c2[v] * r);
            const float a2 = alpha * alpha;
            const float z = PRECISE ? one_minus_exp(2.0f * cs[v] * r) : clamp01(1.0f - a2);
            const float rs = hw_rsq(fmaxf(z, 1e-30f));
            const float m = z * rs;
            // 2 * clipped sqrt derivative: 1/sqrt(max(4z,1e-6)) = 0.5/sqrt(max(z,2.5e-7))
            const float csg2 = (z >= 2.5e-7f) ? rs : 2000.0f;
            const float ix = i * fx[v];
            const float mi = m * i;
            float k4 = fmaf(fhp[v], alpha, -(ix * a2) * csg2) * r;
            if (!ok) { alpha = 1.0f; k4 = 0.0f; }
            k1[j][v] = mi;
            k2[j][v] = (m * ix) * (1.0f - i);
            k3[j][v] = (k4 * (1.0f - r)) * cs[v];
            const float g_loc = fgo[v] + c_run[v];
            gl[j][v] = g_loc;
            qn[j][v] = q_run[v];
            acc_a[v] = fmaf(g_loc, k4, acc_a[v]);
            acc_q[v] = fmaf(q_run[v], k4, acc_q[v]);
            c_run[v] = alpha * g_loc;
            q_run[v] *= alpha;
        }
    }

    // 2. combine the time slices; later slices come first in the reverse chain
#pragma unroll
    for (int v = 0; v < V; ++v) s_agg[w][lane * V + v] = make_float2(q_run[v], c_run[v]);
    __syncthreads();
    float p_pre[V], h_pre[V], p_tot[V], h_tot[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { p_tot[v] = 1.0f; h_tot[v] = 0.0f; p_pre[v] = 1.0f; h_pre[v] = 0.0f; }
#pragma unroll
    for (int ww = NW - 1; ww >= 0; --ww) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if (ww == w) { p_pre[v] = p_tot[v]; h_pre[v] = h_tot[v]; }
            const float2 a = s_agg[ww][lane * V + v];
            h_tot[v] = fmaf(a.x, h_tot[v], a.y);
            p_tot[v] *= a.x;
        }
    }

    // 3. carry across tiles
    float cin[V];
#pragma unroll
    for (int v = 0; v < V; ++v) cin[v] = 0.0f;
    if (nseg > 1) {
        if (w == 0) {
            const size_t stride = (size_t)B * D;
            const size_t idx0 = (size_t)b * D + c0;
            const size_t idx = idx0 + (size_t)pos * stride;
            const bool publishes = pos + 1 < nseg;
            if (publishes && !is_checkpoint(pos)) {
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    publish(ws.agg_p + idx + v, tag, p_tot[v]);
                    publish(ws.agg_h + idx + v, tag, h_tot[v]);
                }
                asm volatile("" ::: "memory");
            }
            if (pos > 0) {
#pragma unroll
                for (int v = 0; v < V; ++v) cin[v] = look_back(ws, idx0 + v, stride, pos, tag);
            }
            if (publishes && is_checkpoint(pos)) {
#pragma unroll
                for (int v = 0; v < V; ++v) publish(ws.incl + idx + v, tag, fmaf(p_tot[v], cin[v], h_tot[v]));
            }
#pragma unroll
            for (int v = 0; v < V; ++v) s_cin[lane * V + v] = cin[v];
        }
        __syncthreads();
#pragma unroll
        for (int v = 0; v < V; ++v) cin[v] = s_cin[lane * V + v];
    }

    // 4. apply the carry, store the three gradients, reduce the dLambda partial
    float cw[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        cw[v] = fmaf(p_pre[v], cin[v], h_pre[v]);
        s_dl[w][lane * V + v] = fmaf(cw[v], acc_q[v], acc_a[v]);
    }
    if (lane_on) {
#pragma unroll
        for (int j = 0; j < TC; ++j) {
            if (full || (t0 + j < T)) {
                float o1[V], o2[V], o3[V];
#pragma unroll
                for (int v = 0; v < V; ++v) {
                    const float g = fmaf(qn[j][v], cw[v], gl[j][v]);
                    o1[v] = g * k1[j][v];
                    o2[v] = g * k2[j][v];
                    o3[v] = g * k3[j][v];
                }
                raw_t r1, r2, r3;
                pack(o1, r1);
                pack(o2, r2);
                pack(o3, r3);
                const size_t o = base + (size_t)j * D;
                store_raw<ET, V>(dx + o, r1);
                store_raw<ET, V>(dxg + o, r2);
                store_raw<ET, V>(dag + o, r3);
            }
        }
    }
    __syncthreads();
    if (w == 0 && lane_on) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float sum = 0.0f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) sum += s_dl[ww][lane * V + v];
            ws.dlam_part[((size_t)seg * B + b) * D + c0 + v] = sum;
        }
    }

    if (nseg > 1) retire(ws.ctrl, total, tag);
}

// dLambda[c] = -8 sigmoid(Lambda_c) * sum over rows of the [rows, D] partials.
// 64 channels x 16 row slices per block; fixed summation order, so the result is
// reproducible run to run.
__global__ __launch_bounds__(1024) void dlam_reduce_kernel(const float* __restrict__ part,
                                                          const float* __restrict__ lam,
                                                          float* __restrict__ dlam, int rows, int D) {
    __shared__ float s[16][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int c = blockIdx.x * kWave + lane;
    float sum = 0.0f;
    if (c < D) {
        for (int r = slice; r < rows; r += 16) sum += part[(size_t)r * D + c];
    }
    s[slice][lane] = sum;
    __syncthreads();
    if (slice == 0 && c < D) {
        float tot = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) tot += s[k][lane];
        dlam[c] = -8.0f * sigmoid_precise(lam[c]) * tot;
    }
}

__global__ void fill_u32_kernel(uint32_t* p, size_t n, uint32_t v) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) p[i] = v;
}

// ---------------------------------------------------------------------------------------
// Host side: tile-shape choice, workspace carving, launches.
// ---------------------------------------------------------------------------------------
constexpr size_t kCtrlBytes = 256;

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct TileShape {
    int V, TC, NW;
    int rows() const { return TC * NW; }
    int chans() const { return kWave * V; }
};

// Widest per-lane vector that divides D and keeps every row start aligned.
int pick_v(int D, int dtype, int vmax) {
    int v = vmax;
    while (v > 1 && (D % v) != 0) v >>= 1;
    (void)dtype;
    return v;
}

TileShape fwd_shape(int D, int dtype) {
    TileShape s;
    s.V = pick_v(D, dtype, 2);
    if (dtype == HAWK_DTYPE_BF16) { s.TC = 16; s.NW = 8; }
    else { s.TC = 8; s.NW = 8; }
    return s;
}
TileShape bwd_shape(int D, int dtype) {
    TileShape s;
    s.V = pick_v(D, dtype, 2);
    s.TC = 8;
    s.NW = 8;
    return s;
}

int ceil_div(int a, int b) { return (a + b - 1) / b; }

struct WsLayout {
    size_t off_incl, off_aggp, off_aggh, off_dlam, total;
};
WsLayout layout_for(int B, int D, int nseg_chain, int nseg_dlam) {
    WsLayout l;
    const size_t words = (size_t)nseg_chain * B * D * sizeof(unsigned long long);
    l.off_incl = kCtrlBytes;
    l.off_aggp = align_up(l.off_incl + words, 256);
    l.off_aggh = align_up(l.off_aggp + words, 256);
    l.off_dlam = align_up(l.off_aggh + words, 256);
    l.total = align_up(l.off_dlam + (size_t)nseg_dlam * B * D * sizeof(float), 256);
    return l;
}
ScanWsPtrs carve(void* ws, const WsLayout& l) {
    char* p = static_cast<char*>(ws);
    ScanWsPtrs r;
    r.ctrl = reinterpret_cast<uint32_t*>(p);
    r.incl = reinterpret_cast<unsigned long long*>(p + l.off_incl);
    r.agg_p = reinterpret_cast<unsigned long long*>(p + l.off_aggp);
    r.agg_h = reinterpret_cast<unsigned long long*>(p + l.off_aggh);
    r.dlam_part = reinterpret_cast<float*>(p + l.off_dlam);
    return r;
}

template <typename ET, int V, int TC, int NW, bool PRECISE>
int launch_fwd(const void* x, const void* xg, const void* ag, const float* lam, void* h, int B, int T,
               int D, int nseg, int nct, ScanWsPtrs ws, hipStream_t st) {
    const unsigned grid = (unsigned)nseg * B * nct;
    hipLaunchKernelGGL((rglru_scan_fwd_kernel<ET, V, TC, NW, PRECISE>), dim3(grid), dim3(NW * kWave), 0, st,
                       static_cast<const ET*>(x), static_cast<const ET*>(xg), static_cast<const ET*>(ag), lam,
                       static_cast<ET*>(h), B, T, D, nseg, nct, ws);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename ET, int V, int TC, int NW, bool PRECISE>
int launch_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* hs,
               const void* gout, void* dx, void* dxg, void* dag, int B, int T, int D, int nseg, int nct,
               ScanWsPtrs ws, hipStream_t st) {
    const unsigned grid = (unsigned)nseg * B * nct;
    hipLaunchKernelGGL((rglru_scan_bwd_kernel<ET, V, TC, NW, PRECISE>), dim3(grid), dim3(NW * kWave), 0, st,
                       static_cast<const ET*>(x), static_cast<const ET*>(xg), static_cast<const ET*>(ag), lam,
                       static_cast<const ET*>(hs), static_cast<const ET*>(gout), static_cast<ET*>(dx),
                       static_cast<ET*>(dxg), static_cast<ET*>(dag), B, T, D, nseg, nct, ws);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace

size_t scan_workspace_bytes(int B, int T, int D, int dtype) {
    const TileShape f = fwd_shape(D, dtype), r = bwd_shape(D, dtype);
    const int nf = ceil_div(T, f.rows()), nr = ceil_div(T, r.rows());
    return layout_for(B, D, nf > nr ? nf : nr, nr).total;
}

int workspace_init(void* ws, size_t bytes, hipStream_t st) {
    const size_t n = bytes / sizeof(uint32_t);
    if (n == 0) return HAWK_OK;
    size_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, st, static_cast<uint32_t*>(ws), n, 0u);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

int workspace_status(const void* ws, hipStream_t st, int* flag) {
    uint32_t v = 0;
    if (hipMemcpyAsync(&v, static_cast<const uint32_t*>(ws) + kError, sizeof(v), hipMemcpyDeviceToHost, st) != hipSuccess)
        return HAWK_ERR_LAUNCH;
    if (hipStreamSynchronize(st) != hipSuccess) return HAWK_ERR_LAUNCH;
    *flag = (int)v;
    return HAWK_OK;
}

int scan_fwd(const void* x, const void* xg, const void* ag, const float* lam, void* h, int B, int T, int D,
             int dtype, void* ws, size_t ws_bytes, hipStream_t st) {
    const TileShape s = fwd_shape(D, dtype);
    const int nseg = ceil_div(T, s.rows());
    const int nct = ceil_div(D, s.chans());
    ScanWsPtrs p = {};
    if (nseg > 1) {
        const WsLayout l = layout_for(B, D, nseg, 0);
        if (ws == nullptr || ws_bytes < l.total) return HAWK_ERR_WORKSPACE;
        p = carve(ws, l);
    }
#define HAWK_FWD(ET, V_, TC_, NW_, PR) \
    return launch_fwd<ET, V_, TC_, NW_, PR>(x, xg, ag, lam, h, B, T, D, nseg, nct, p, st)
    if (dtype == HAWK_DTYPE_BF16) {
        if (s.V == 2) HAWK_FWD(bf16_t, 2, 16, 8, false);
        HAWK_FWD(bf16_t, 1, 16, 8, false);
    } else {
        if (s.V == 2) HAWK_FWD(float, 2, 8, 8, true);
        HAWK_FWD(float, 1, 8, 8, true);
    }
#undef HAWK_FWD
}

int scan_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* hs, const void* gout,
             void* dx, void* dxg, void* dag, float* dlam, int B, int T, int D, int dtype, void* ws,
             size_t ws_bytes, hipStream_t st) {
    const TileShape s = bwd_shape(D, dtype);
    const int nseg = ceil_div(T, s.rows());
    const int nct = ceil_div(D, s.chans());
    const WsLayout l = layout_for(B, D, nseg, nseg);
    if (ws == nullptr || ws_bytes < l.total) return HAWK_ERR_WORKSPACE;
    const ScanWsPtrs p = carve(ws, l);
    int rc;
#define HAWK_BWD(ET, V_, TC_, NW_, PR) \
    rc = launch_bwd<ET, V_, TC_, NW_, PR>(x, xg, ag, lam, hs, gout, dx, dxg, dag, B, T, D, nseg, nct, p, st)
    if (dtype == HAWK_DTYPE_BF16) {
        if (s.V == 2) HAWK_BWD(bf16_t, 2, 8, 8, false);
        else HAWK_BWD(bf16_t, 1, 8, 8, false);
    } else {
        if (s.V == 2) HAWK_BWD(float, 2, 8, 8, true);
        else HAWK_BWD(float, 1, 8, 8, true);
    }
#undef HAWK_BWD
    if (rc != HAWK_OK) return rc;
    hipLaunchKernelGGL(dlam_reduce_kernel, dim3((unsigned)ceil_div(D, kWave)), dim3(1024), 0, st, p.dlam_part, lam,
                       dlam, nseg * B, D);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace hawk
