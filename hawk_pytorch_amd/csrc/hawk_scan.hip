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
// error word and finishes (with a wrong carry) instead of hanging.  Results do not depend
// on timing: the combination order is a function of the tile position only.
#include "hawk_scan.h"

#include <stdint.h>

#include <mutex>

#include "hawk_device.h"

namespace hawk {

namespace {

constexpr uint32_t kSpinLimit = 1u << 22;

// Occupancy the register allocator must leave room for (waves per SIMD).
#ifndef HAWK_FWD_WAVES_PER_SIMD
#define HAWK_FWD_WAVES_PER_SIMD 4
#endif
#ifndef HAWK_BWD_WAVES_PER_SIMD
#define HAWK_BWD_WAVES_PER_SIMD 4
#endif
#ifndef HAWK_BWD_KEEP_ALPHA
#define HAWK_BWD_KEEP_ALPHA 1
#endif

// Control block at the start of the workspace:
//   bytes 0-7   one 64-bit word: launch epoch (high half) and ticket counter (low half)
//   bytes 8-11  error flag (a tile gave up waiting for a carry)
struct ScanWsPtrs {
    unsigned long long* ctrl;
    unsigned long long* incl;  // [nseg][B][D] inclusive state at the end of a checkpoint tile
    unsigned long long* agg_p; // [nseg][B][D] tile aggregate: product of alpha
    unsigned long long* agg_h; // [nseg][B][D] tile aggregate: state from zero
    float* dlam_part;          // [nseg][B][D] per-tile partial sums for dLambda
    int lookback;              // distance between checkpoints of the carry chain (power of two)
    uint32_t div_tiles[2];     // ticket / (B * nct) and ... / nct by multiplication (FastDiv)
    uint32_t div_nct[2];
};

// Division of a 32-bit number by a launch constant as a multiplication and two shifts
// (Granlund and Montgomery's round-up method, exact for every 32-bit dividend): a tile's first
// instructions after its ticket arrives are two such divisions, and nothing else can start
// before them.  m = floor(2^32 (2^l - d) / d) + 1 with l = ceil(log2 d); l == 0 means d == 1.
struct FastDiv {
    uint32_t m, l;
};
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t m, uint32_t l) {
    if (l == 0u) return n;
    const uint32_t t = __umulhi(n, m);
    return (t + ((n - t) >> 1)) >> (l - 1u);
}

__device__ __forceinline__ void publish(unsigned long long* p, uint32_t tag, float v) {
    unsigned long long w = ((unsigned long long)tag << 32) | (unsigned long long)__float_as_uint(v);
    __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool try_read(const unsigned long long* p, uint32_t tag, float& v) {
    unsigned long long w = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    v = __uint_as_float((uint32_t)w);
    return (uint32_t)(w >> 32) == tag;
}

// Every lookback-th chain position is a checkpoint: it publishes the inclusive state at
// its end; every other position publishes only its own aggregate.  A tile reads the
// aggregates of its predecessors back to the nearest checkpoint, plus that checkpoint's
// inclusive state, all in parallel (wave k fetches predecessors k, k + NW, ...), and folds them
// oldest first.  The order of the floating-point operations is fixed by the position and the
// launch's shape alone, never by timing, so results are bitwise reproducible, and the serial
// dependency runs over checkpoints only (nseg / lookback hops of one memory round trip each).
// The distance is chosen per launch: 4 when there are enough independent chains (B x channel
// tiles) to keep the memory system busy while each chain waits on its hops, 8 when there are
// few and the hops themselves set the pace (one long sequence of a narrow model: 8 chains run
// 22 % faster, 16 chains 4 %); with 60 or more chains the wider window costs 2-3 % instead.
// With 128 or more chains the distance is 2: a tile then reads at most two predecessors'
// words, and even at one memory round trip per two positions the chain stays ahead of the
// rate at which the launch gets through a position of all its chains (0.5 % faster).
// With 8 chains or fewer the hops are all there is to wait for, and the distance grows to 16
// (5 to 8 chains: 6 % / 3 % faster forward / backward than 8; 12 or more chains are 2 % slower
// with it) and to 32 (up to 4 chains: one chain, B = 1 and D = 128, runs twice as fast as with 8,
// 4 chains 28 % / 20 % faster).
constexpr int kMaxLookback = 32;
constexpr int kFewChains = 24;
constexpr int kFewerChains = 8, kFewestChains = 4;   // distance 16 and 32
#ifndef HAWK_LOOKBACK_MANY
#define HAWK_LOOKBACK_MANY 2
#endif

__device__ __forceinline__ bool is_checkpoint(int pos, int lookback) { return (pos & (lookback - 1)) == 0; }
__device__ __forceinline__ int checkpoint_before(int pos, int lookback) { return (pos - 1) & ~(lookback - 1); }

// One 64-bit atomic hands out the tile's position in the chain (ticket) together with the
// launch tag, so a tile only ever waits for tiles that have already started.  The tile
// that takes the last ticket re-arms the word for the next launch on this workspace
// (epoch + 1, ticket 0) with a second atomic; nothing else ever writes it.
__device__ __forceinline__ void take_ticket(unsigned long long* ctrl, uint32_t total, uint32_t* s_ticket,
                                            uint32_t& ticket, uint32_t& tag) {
    if (threadIdx.x == 0) {
        const unsigned long long v =
            __hip_atomic_fetch_add(ctrl, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t t = (uint32_t)v;
        if (t == total - 1u) {
            __hip_atomic_fetch_add(ctrl, (1ull << 32) - (unsigned long long)total, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        s_ticket[0] = t;
        s_ticket[1] = (uint32_t)(v >> 32) + 1u;
    }
    __syncthreads();
    ticket = __builtin_amdgcn_readfirstlane(s_ticket[0]);
    tag = __builtin_amdgcn_readfirstlane(s_ticket[1]);
}

// Carry into chain position `pos` for the V channels of this lane.
//   tot_p/tot_h  aggregate of this whole tile (every wave holds it)
//   s_prev       LDS [kMaxLookback][CT] staging of the predecessors' words
// Wave 0 publishes the tile's own word; wave k fetches predecessors pos-1-k, pos-1-k-NW, ...;
// after one barrier every wave folds the staged words.
template <int V, int NW>
__device__ __forceinline__ void exchange_carry(const ScanWsPtrs& ws, int pos, int nseg, size_t idx_pos0,
                                               size_t stride, uint32_t tag, int w, int lane,
                                               const float (&tot_p)[V], const float (&tot_h)[V],
                                               float2 (*s_prev)[kWave * V], float (&cin)[V]) {
    const int lookback = ws.lookback;
    const bool publishes = pos + 1 < nseg;
    const size_t idx_self = idx_pos0 + (size_t)pos * stride;
    if (w == 0 && publishes && !is_checkpoint(pos, lookback)) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            publish(ws.agg_p + idx_self + v, tag, tot_p[v]);
            publish(ws.agg_h + idx_self + v, tag, tot_h[v]);
        }
        asm volatile("" ::: "memory");
    }
    const int npred = (pos > 0) ? pos - checkpoint_before(pos, lookback) : 0;
    for (int k = w; k < npred; k += NW) {
        const int j = pos - 1 - k;
        const size_t idx = idx_pos0 + (size_t)j * stride;
        const bool cp = (k == npred - 1);
        float vp[V], vh[V];
        bool ok = false;
        uint32_t spins = 0;
        while (!ok) {
            ok = true;
#pragma unroll
            for (int v = 0; v < V; ++v) {
                if (cp) {
                    vp[v] = 0.0f;
                    ok &= try_read(ws.incl + idx + v, tag, vh[v]);
                } else {
                    ok &= try_read(ws.agg_p + idx + v, tag, vp[v]);
                    ok &= try_read(ws.agg_h + idx + v, tag, vh[v]);
                }
            }
            if (!ok) {
                if (++spins > kSpinLimit) {
                    __hip_atomic_store(reinterpret_cast<uint32_t*>(ws.ctrl) + 2, 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int v = 0; v < V; ++v) { vp[v] = 0.0f; vh[v] = 0.0f; }
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
        }
#pragma unroll
        for (int v = 0; v < V; ++v) s_prev[k][lane * V + v] = make_float2(vp[v], vh[v]);
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < V; ++v) cin[v] = 0.0f;
    for (int k = npred - 1; k >= 0; --k) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float2 a = s_prev[k][lane * V + v];
            cin[v] = fmaf(a.x, cin[v], a.y);
        }
    }
    if (w == 0 && publishes && is_checkpoint(pos, lookback)) {
#pragma unroll
        for (int v = 0; v < V; ++v) publish(ws.incl + idx_self + v, tag, fmaf(tot_p[v], cin[v], tot_h[v]));
    }
}

// Slice aggregates of the NW waves -> prefix for wave `w` and tile total, in chain order
// (forward: wave 0 first; backward: wave NW-1 first).
// LEAN: read the staged aggregates four at a time instead of all at once (fewer registers).
template <int V, int NW, bool REVERSE, bool LEAN = false>
__device__ __forceinline__ void combine_slices(float2 (*s_agg)[kWave * V], int w, int lane, float (&pre_p)[V],
                                               float (&pre_h)[V], float (&tot_p)[V], float (&tot_h)[V]) {
#pragma unroll
    for (int v = 0; v < V; ++v) { tot_p[v] = 1.0f; tot_h[v] = 0.0f; pre_p[v] = 1.0f; pre_h[v] = 0.0f; }
#pragma unroll
    for (int q = 0; q < NW; ++q) {
        const int ww = REVERSE ? NW - 1 - q : q;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if (ww == w) { pre_p[v] = tot_p[v]; pre_h[v] = tot_h[v]; }
            const float2 a = s_agg[ww][lane * V + v];
            tot_h[v] = fmaf(a.x, tot_h[v], a.y);
            tot_p[v] *= a.x;
        }
        if (LEAN && (q % 4) == 3) __builtin_amdgcn_sched_barrier(0);
    }
}

// Operands of the gated variants (out = gelu(y) * h, the step that follows the scan in a
// Hawk block).  y and dy are [B, T, D] views whose rows may be further apart than D
// elements (y is one half of a wider projection); batches are T rows apart.
template <typename OT>
struct GateFwdArgs {
    const OT* y;      // gate input
    OT* out;          // gelu(y) * h, dense [B, T, D]
    OT* h_last;       // optional [B, D]: h at t = T-1 (the decode cache's recurrent state)
    uint32_t ldy;     // elements between consecutive rows of y
};
template <typename ST>
struct GateBwdArgs {
    const ST* y;
    ST* dy;
    uint32_t ldy, lddy;
};

// Bytes of a [rows, D - c_tile] window of a row-strided tensor, for its buffer resource.
__device__ __forceinline__ uint32_t strided_window_bytes(int rows, uint32_t row_bytes, uint32_t last_row_bytes) {
    return rows > 0 ? (uint32_t)(rows - 1) * row_bytes + last_row_bytes : 0u;
}

// ---------------------------------------------------------------------------------------
// Forward tile.  FULL: every row of the tile is inside [0, T).
// GATED: also reads y and writes out = gelu(y) * h; h itself is stored only if h != nullptr.
// ---------------------------------------------------------------------------------------
template <typename IT, typename OT, int V, int TC, int NW, bool PRECISE, bool FULL, bool GATED, bool STORE_H>
__device__ __forceinline__ void fwd_tile(const IT* __restrict__ x, const IT* __restrict__ xg,
                                         const IT* __restrict__ ag, const float* __restrict__ lam,
                                         OT* __restrict__ h, const GateFwdArgs<OT>& gate, int B, int T, int D,
                                         int nseg, int seg, int b, int ct, uint32_t tag, const ScanWsPtrs& ws,
                                         float2 (*s_agg)[kWave * V], float2 (*s_prev)[kWave * V]) {
    typedef typename Raw<IT, V>::type raw_t;
    typedef typename Raw<OT, V>::type out_raw_t;
    constexpr int CT = kWave * V;
    constexpr int TS = NW * TC;

    const int lane = threadIdx.x & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int c_tile = ct * CT;
    const bool lane_on = c_tile + lane * V < D;
    const unsigned lane_off = lane_on ? lane * V : D - V - c_tile;  // idle lanes shadow the last valid channels
    const int t0 = seg * TS + w * TC;
    const size_t tile_off = ((size_t)b * T + t0) * D + c_tile;  // wave-uniform
    const int rows_in = FULL ? TC : __builtin_amdgcn_readfirstlane(min(max(T - t0, 0), TC));  // rows inside [0, T)
    const uint32_t row_bytes = (uint32_t)D * sizeof(IT);
    const uint32_t out_row_bytes = (uint32_t)D * sizeof(OT);
    const uint32_t slab = (uint32_t)rows_in * row_bytes;
    const uint32_t lane_bytes = lane_off * sizeof(IT);
    const rsrc_t bx = make_rsrc(x + tile_off, slab), bxg = make_rsrc(xg + tile_off, slab),
                 bag = make_rsrc(ag + tile_off, slab);
    const rsrc_t bh = make_rsrc(STORE_H ? h + tile_off : nullptr, STORE_H ? (uint32_t)rows_in * out_row_bytes : 0u);
    // idle lanes store at an offset beyond any slab, which the range check drops
    const uint32_t store_bytes = lane_on ? lane_off * (uint32_t)sizeof(OT) : 0x80000000u;

    raw_t rx[TC], rxg[TC], rag[TC];
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        rx[j] = buffer_load<raw_t>(bx, lane_bytes, j * row_bytes);
        rxg[j] = buffer_load<raw_t>(bxg, lane_bytes, j * row_bytes);
        rag[j] = buffer_load<raw_t>(bag, lane_bytes, j * row_bytes);
    }

    // Per-channel constants: log2(alpha) = c2 * r, 2 ln(alpha) = cn * r.
    float c2[V], cn[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float s = softplus_fast(lam[c_tile + lane_off + v]);
        c2[v] = -8.0f * kLog2e * s;
        cn[v] = -16.0f * s;
    }

    // 1. local scan from a zero state.  Kept per row: the local state (fp32) and the
    //    running product of alpha, which for bf16 activations with two channels per lane
    //    is stored as an fp16 pair (it only ever scales the carry).
    constexpr bool PACK_P = (V == 2) && (sizeof(OT) == 2);
    float hj[TC][V];
    float pj[PACK_P ? 1 : TC][V];
    uint32_t pjh[PACK_P ? TC : 1];
    float p_run[V], h_run[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { p_run[v] = 1.0f; h_run[v] = 0.0f; }
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        float fx[V], fxg[V], fag[V];
        unpack(rx[j], fx);
        unpack(rxg[j], fxg);
        unpack(rag[j], fag);
        const bool ok = FULL || (t0 + j < T);  // wave-uniform
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
            if (!PACK_P) pj[j][v] = p_run[v];
            hj[j][v] = h_run[v];
        }
        // (packed now: left alone, the conversion sinks below the exchange and the products stay in fp32)
        if (PACK_P) pjh[j] = opaque(pack_f16x2(p_run[0], p_run[V - 1]));
        __builtin_amdgcn_sched_barrier(0);  // one row's temporaries live at a time
    }

    // The gate rows are fetched now, into registers the raw inputs occupied until here,
    // and arrive during the carry exchange.
    out_raw_t ry[GATED ? TC : 1];
    if constexpr (GATED) {
        __builtin_amdgcn_sched_barrier(0);  // not before the local pass has freed the inputs' registers
        const uint32_t y_row_bytes = gate.ldy * (uint32_t)sizeof(OT);
        const rsrc_t by = make_rsrc(gate.y + ((size_t)b * T + t0) * gate.ldy + c_tile,
                                    strided_window_bytes(rows_in, y_row_bytes, (uint32_t)(D - c_tile) * sizeof(OT)));
#pragma unroll
        for (int j = 0; j < TC; ++j)
            ry[j] = buffer_load<out_raw_t>(by, lane_off * (uint32_t)sizeof(OT), j * y_row_bytes);
    }

    // 2. combine the NW time slices of this tile
#pragma unroll
    for (int v = 0; v < V; ++v) s_agg[w][lane * V + v] = make_float2(p_run[v], h_run[v]);
    __syncthreads();
    float pre_p[V], pre_h[V], tot_p[V], tot_h[V];
    combine_slices<V, NW, false, true>(s_agg, w, lane, pre_p, pre_h, tot_p, tot_h);
    // This wave's prefix is picked here: left to itself the compiler keeps all NW candidates in
    // registers through the carry exchange and picks afterwards (30 registers at 16 rows).
#pragma unroll
    for (int v = 0; v < V; ++v) { pre_p[v] = opaque(pre_p[v]); pre_h[v] = opaque(pre_h[v]); }

    // 3. carry across tiles
    float cin[V];
#pragma unroll
    for (int v = 0; v < V; ++v) cin[v] = 0.0f;
    if (nseg > 1) {
        exchange_carry<V, NW>(ws, seg, nseg, (size_t)b * D + c_tile + lane_off, (size_t)B * D, tag, w, lane,
                              tot_p, tot_h, s_prev, cin);
    }

    // 4. apply the carry and store
    float cw[V];
#pragma unroll
    for (int v = 0; v < V; ++v) cw[v] = fmaf(pre_p[v], cin[v], pre_h[v]);
    const rsrc_t bout = make_rsrc(GATED ? gate.out + tile_off : nullptr, GATED ? (uint32_t)rows_in * out_row_bytes : 0u);
    const int j_last = T - 1 - t0;  // row of this slice that is t = T-1, if any (wave-uniform)
    out_raw_t r_last = raw_zero<out_raw_t>();
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        float out[V];
        if (PACK_P) {
            out[0] = fmaf(f16_lo(pjh[j]), cw[0], hj[j][0]);
            out[V - 1] = fmaf(f16_hi(pjh[j]), cw[V - 1], hj[j][V - 1]);
        } else {
#pragma unroll
            for (int v = 0; v < V; ++v) out[v] = fmaf(pj[j][v], cw[v], hj[j][v]);
        }
        out_raw_t r;
        pack(out, r);
        if constexpr (GATED) {
            float fy[V], o[V];
            if constexpr (sizeof(out_raw_t) == 4) {
                unpack(opaque(ry[j]), fy);  // keeps the gate's arithmetic below the exchange, one row at a time
            } else {
                unpack(ry[j], fy);
            }
#pragma unroll
            for (int v = 0; v < V; ++v) {
                float cdf, e;
                normal_cdf<PRECISE>(fy[v], cdf, e);
                o[v] = (fy[v] * cdf) * out[v];
            }
            out_raw_t ro;
            pack(o, ro);
            buffer_store<out_raw_t>(ro, bout, store_bytes, j * out_row_bytes);
            if constexpr (STORE_H) buffer_store<out_raw_t>(r, bh, store_bytes, j * out_row_bytes);
            r_last = (j == j_last) ? r : r_last;
            __builtin_amdgcn_sched_barrier(0);  // one row's temporaries live at a time
        } else {
            buffer_store<out_raw_t>(r, bh, store_bytes, j * out_row_bytes);  // rows past T and idle lanes are dropped
        }
    }
    if constexpr (GATED) {
        if (gate.h_last != nullptr && j_last >= 0 && j_last < TC) {
            const rsrc_t bl = make_rsrc(gate.h_last + (size_t)b * D + c_tile, (uint32_t)(D - c_tile) * sizeof(OT));
            buffer_store<out_raw_t>(r_last, bl, store_bytes, 0u);
        }
    }
}

template <typename IT, typename OT, int V, int TC, int NW, bool PRECISE, bool GATED, bool STORE_H>
__global__ __launch_bounds__(NW * kWave, HAWK_FWD_WAVES_PER_SIMD) void rglru_scan_fwd_kernel(
    const IT* __restrict__ x, const IT* __restrict__ xg, const IT* __restrict__ ag,
    const float* __restrict__ lam, OT* __restrict__ h, GateFwdArgs<OT> gate, int B, int T, int D, int nseg,
    int nct, ScanWsPtrs ws) {
    constexpr int CT = kWave * V;
    constexpr int TS = NW * TC;
    __shared__ float2 s_agg[NW][CT];
    __shared__ float2 s_prev[kMaxLookback][CT];
    __shared__ uint32_t s_ticket[2];

    uint32_t ticket = blockIdx.x, tag = 0;
    if (nseg > 1) take_ticket(ws.ctrl, (uint32_t)nseg * (uint32_t)B * (uint32_t)nct, s_ticket, ticket, tag);

    const int per_seg = B * nct;
    const int seg = (int)fast_div(ticket, ws.div_tiles[0], ws.div_tiles[1]);
    const int rem = ticket - seg * per_seg;
    const int b = (int)fast_div((uint32_t)rem, ws.div_nct[0], ws.div_nct[1]);
    const int ct = rem - b * nct;
    if (seg * TS + TS <= T)
        fwd_tile<IT, OT, V, TC, NW, PRECISE, true, GATED, STORE_H>(x, xg, ag, lam, h, gate, B, T, D, nseg, seg, b, ct,
                                                                   tag, ws, s_agg, s_prev);
    else
        fwd_tile<IT, OT, V, TC, NW, PRECISE, false, GATED, STORE_H>(x, xg, ag, lam, h, gate, B, T, D, nseg, seg, b, ct,
                                                                    tag, ws, s_agg, s_prev);
}

// ---------------------------------------------------------------------------------------
// Backward.  Reverse chain on c_t = alpha_t (gout_t + c_{t+1}); g_t = gout_t + c_{t+1}.
// The chain itself needs only alpha and gout, so the local pass evaluates just those (and
// keeps r); once the carry into the slice is known, the recurrence is replayed
// exactly and each row's gradients are formed and stored on the spot:
//   dx = g m i;  dx_rg_lru = g m x i (1-i);
//   dlog_a = g (h_{t-1} alpha - i x alpha^2 2 csg(1-alpha^2));
//   da_rg_lru = dlog_a r (1-r) (-8 softplus(Lambda));  dLambda += dlog_a r  (scaled per channel later)
// FULL: every row of the tile is inside [1, T) (row 0 has no h_{t-1}).
// GATED: gout is the gradient of out = gelu(y) * h; the gradient reaching h is
//   gout gelu(y), and dy = gout h_t gelu'(y) is stored as a fourth output.
// ---------------------------------------------------------------------------------------
template <typename IT, typename ST, int V, int TC, int NW, bool PRECISE, bool FULL, bool GATED>
__device__ __forceinline__ void bwd_tile(const IT* __restrict__ x, const IT* __restrict__ xg,
                                         const IT* __restrict__ ag, const float* __restrict__ lam,
                                         const ST* __restrict__ hs, const ST* __restrict__ gout,
                                         IT* __restrict__ dx, IT* __restrict__ dxg, IT* __restrict__ dag,
                                         const GateBwdArgs<ST>& gate, int B, int T, int D, int nseg, int seg, int pos,
                                         int b, int ct, uint32_t tag, const ScanWsPtrs& ws,
                                         float2 (*s_agg)[kWave * V], float2 (*s_prev)[kWave * V],
                                         float (*s_dl)[kWave * V]) {
    typedef typename Raw<IT, V>::type raw_t;      // x, x_rg_lru, a_rg_lru and the three gradients
    typedef typename Raw<ST, V>::type sraw_t;     // saved h and grad_out
    constexpr int CT = kWave * V;
    constexpr int TS = NW * TC;

    const int lane = threadIdx.x & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int c_tile = ct * CT;
    const bool lane_on = c_tile + lane * V < D;
    const unsigned lane_off = lane_on ? lane * V : D - V - c_tile;
    const int t0 = seg * TS + w * TC;
    const size_t tile_off = ((size_t)b * T + t0) * D + c_tile;
    const int rows_in = FULL ? TC : __builtin_amdgcn_readfirstlane(min(max(T - t0, 0), TC));
    const uint32_t row_bytes = (uint32_t)D * sizeof(IT);
    const uint32_t srow_bytes = (uint32_t)D * sizeof(ST);
    const uint32_t slab = (uint32_t)rows_in * row_bytes;
    const uint32_t lane_bytes = lane_off * sizeof(IT);
    const uint32_t slane_bytes = lane_off * sizeof(ST);
    const rsrc_t bx = make_rsrc(x + tile_off, slab), bxg = make_rsrc(xg + tile_off, slab),
                 bag = make_rsrc(ag + tile_off, slab),
                 bgo = make_rsrc(gout + tile_off, (uint32_t)rows_in * srow_bytes),
                 bhs = make_rsrc(hs + tile_off, (uint32_t)rows_in * srow_bytes);
    // h_{t-1} of the slice's first row lives one row before the slab; absent at t = 0
    const bool has_prev = FULL || (t0 > 0 && rows_in > 0);
    const rsrc_t bhm1 = make_rsrc(has_prev ? hs + tile_off - D : hs, has_prev ? srow_bytes : 0u);
    const rsrc_t bdx = make_rsrc(dx + tile_off, slab), bdxg = make_rsrc(dxg + tile_off, slab),
                 bdag = make_rsrc(dag + tile_off, slab);
    // idle lanes store at an offset beyond any slab, which the range check drops
    const uint32_t store_bytes = lane_on ? lane_bytes : 0x80000000u;

    // The local pass needs only a_rg_lru and grad_out; x, x_rg_lru and h are fetched after
    // it (their registers would otherwise sit idle through it) and arrive during the carry
    // exchange.  This is what lets a lane own TC rows within 128 registers.
    raw_t rx[TC], rxg[TC], rag[TC];
    sraw_t rgo[TC], rhp[TC];
    sraw_t ry[GATED ? TC : 1], rh_end = raw_zero<sraw_t>();
    const uint32_t y_row_bytes = GATED ? gate.ldy * (uint32_t)sizeof(ST) : 0u;
    const uint32_t dy_row_bytes = GATED ? gate.lddy * (uint32_t)sizeof(ST) : 0u;
    rsrc_t by, bdy;
    if constexpr (GATED) {
        const uint32_t last = (uint32_t)(D - c_tile) * sizeof(ST);
        by = make_rsrc(gate.y + ((size_t)b * T + t0) * gate.ldy + c_tile,
                       strided_window_bytes(rows_in, y_row_bytes, last));
        bdy = make_rsrc(gate.dy + ((size_t)b * T + t0) * gate.lddy + c_tile,
                        strided_window_bytes(rows_in, dy_row_bytes, last));
    }
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        rag[j] = buffer_load<raw_t>(bag, lane_bytes, j * row_bytes);
        rgo[j] = buffer_load<sraw_t>(bgo, slane_bytes, j * srow_bytes);
        if constexpr (GATED) ry[j] = buffer_load<sraw_t>(by, slane_bytes, j * y_row_bytes);
    }

    float c2[V], cs[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const float s = softplus_fast(lam[c_tile + lane_off + v]);
        c2[v] = -8.0f * kLog2e * s;
        cs[v] = -8.0f * s;
    }

    // 1. local reverse scan of c from a zero carry: needs only alpha and gout.  r
    //    is kept; everything else is evaluated after the carry is known.
    // r is kept as an fp16 pair for bf16 activations (2^-11 relative, well inside the bf16
    // rounding of the gradients), in fp32 otherwise.
    constexpr bool PACK_R = (V == 2) && (sizeof(IT) == 2);
    float rr[PACK_R ? 1 : TC][V];
    uint32_t rrh[PACK_R ? TC : 1];
    // alpha is kept for the replay where the registers are there for it (short tiles)
    constexpr bool KEEP_ALPHA = HAWK_BWD_KEEP_ALPHA && TC <= 8;
    float al[KEEP_ALPHA ? TC : 1][V];
    float q_run[V], c_run[V];
#pragma unroll
    for (int v = 0; v < V; ++v) { q_run[v] = 1.0f; c_run[v] = 0.0f; }
#pragma unroll
    for (int j = TC - 1; j >= 0; --j) {
        float fag[V], fgo[V], rv[V];
        unpack(rag[j], fag);
        unpack(rgo[j], fgo);
        if constexpr (GATED) {
            // The gate is evaluated once.  gout gelu(y), the gradient that reaches h, takes
            // gout's registers, and gout gelu'(y), which the replay multiplies by h_t to get
            // dy, takes y's: both in the state dtype, which is also where an unfused
            // gelu(y) * h backward would round them.
            float fy[V], gd[V];
            unpack(ry[j], fy);
#pragma unroll
            for (int v = 0; v < V; ++v) {
                float cdf, e;
                normal_cdf<PRECISE>(fy[v], cdf, e);
                gd[v] = fgo[v] * fmaf(fy[v] * kInvSqrt2Pi, e, cdf);
                fgo[v] *= fy[v] * cdf;
            }
            // (pinned here: left alone, the compiler sinks the conversions to their uses after
            // the exchange and keeps two floats per element alive instead of one packed word)
            pack(fgo, rgo[j]);
            pack(gd, ry[j]);
            rgo[j] = opaque(rgo[j]);
            ry[j] = opaque(ry[j]);
            unpack(rgo[j], fgo);  // the chain must see exactly the gradient the replay will see
        }
        const bool ok = FULL || (t0 + j < T);
#pragma unroll
        for (int v = 0; v < V; ++v) rv[v] = sigmoid_fast(fag[v]);
        if (PACK_R) {
            // the chain must see exactly the r the replay will see
            rrh[j] = pack_f16x2(rv[0], rv[V - 1]);
            rv[0] = f16_lo(rrh[j]);
            rv[V - 1] = f16_hi(rrh[j]);
        }
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float alpha = hw_exp2(c2[v] * rv[v]);
            if (!ok) alpha = 1.0f;  // rows past T are the identity
            if (!PACK_R) rr[j][v] = rv[v];
            if (KEEP_ALPHA) al[j][v] = alpha;
            c_run[v] = alpha * (fgo[v] + c_run[v]);
            q_run[v] *= alpha;
        }
        if constexpr (GATED) __builtin_amdgcn_sched_barrier(0);  // one row's gate temporaries at a time
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < TC; ++j) {
        rx[j] = buffer_load<raw_t>(bx, lane_bytes, j * row_bytes);
        rxg[j] = buffer_load<raw_t>(bxg, lane_bytes, j * row_bytes);
        rhp[j] = (j == 0) ? buffer_load<sraw_t>(bhm1, slane_bytes, 0u)
                          : buffer_load<sraw_t>(bhs, slane_bytes, (j - 1) * srow_bytes);
    }
    if constexpr (GATED) rh_end = buffer_load<sraw_t>(bhs, slane_bytes, (TC - 1) * srow_bytes);
    __builtin_amdgcn_sched_barrier(0);

    // 2. combine the time slices; later slices come first in the reverse chain
#pragma unroll
    for (int v = 0; v < V; ++v) s_agg[w][lane * V + v] = make_float2(q_run[v], c_run[v]);
    __syncthreads();
    float pre_p[V], pre_h[V], tot_p[V], tot_h[V];
    combine_slices<V, NW, true, true>(s_agg, w, lane, pre_p, pre_h, tot_p, tot_h);
#pragma unroll
    for (int v = 0; v < V; ++v) { pre_p[v] = opaque(pre_p[v]); pre_h[v] = opaque(pre_h[v]); }  // as in the forward

    // 3. carry across tiles
    float cin[V];
#pragma unroll
    for (int v = 0; v < V; ++v) cin[v] = 0.0f;
    if (nseg > 1) {
        exchange_carry<V, NW>(ws, pos, nseg, (size_t)b * D + c_tile + lane_off, (size_t)B * D, tag, w, lane,
                              tot_p, tot_h, s_prev, cin);
    }

    // 4. the exact recurrence from the true carry, with the gradients of each row computed
    //    and stored as its g_t becomes known
    float c_true[V], acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        c_true[v] = fmaf(pre_p[v], cin[v], pre_h[v]);
        acc[v] = 0.0f;
    }
#pragma unroll
    for (int j = TC - 1; j >= 0; --j) {
        float fx[V], fxg[V], fgo[V], fhp[V];
        unpack(rx[j], fx);
        unpack(rxg[j], fxg);
        if constexpr (sizeof(sraw_t) == 4 && sizeof(ST) == 2) {
            // unpack again rather than keep the local pass's floats alive across the exchange
            unpack(opaque(rgo[j]), fgo);
        } else {
            unpack(rgo[j], fgo);
        }
        unpack(rhp[j], fhp);
        float o4[V];
        if constexpr (GATED) {
            // dy = (gout gelu'(y)) h_t; h_t is the next row's h_{t-1}
            float fd[V], fh[V];
            if constexpr (sizeof(sraw_t) == 4 && sizeof(ST) == 2) {
                unpack(opaque(ry[j]), fd);
            } else {
                unpack(ry[j], fd);
            }
            unpack(j == TC - 1 ? rh_end : rhp[j == TC - 1 ? j : j + 1], fh);
#pragma unroll
            for (int v = 0; v < V; ++v) o4[v] = fd[v] * fh[v];
        }
        const bool ok = FULL || (t0 + j < T);
        const uint32_t rpair = PACK_R ? opaque(rrh[j]) : 0u;
        float o1[V], o2[V], o3[V];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float r = PACK_R ? (v == 0 ? f16_lo(rpair) : f16_hi(rpair)) : opaque(rr[j][v]);
            float alpha;
            if (KEEP_ALPHA) {
                alpha = opaque(al[j][v]);
            } else {
                alpha = hw_exp2(c2[v] * r);  // cheaper to re-evaluate than to keep in a register
                if (!ok) alpha = 1.0f;
            }
            const float g = fgo[v] + c_true[v];
            c_true[v] = alpha * g;
            const float i = sigmoid_fast(fxg[v]);
            const float z = PRECISE ? one_minus_exp(2.0f * cs[v] * r) : clamp01(fmaf(-alpha, alpha, 1.0f));
            const float m = hw_sqrt(z);
            // 2 * clipped sqrt derivative: 1/sqrt(max(4z,1e-6)) = 0.5/sqrt(max(z,2.5e-7)), at most 2000
            const float csg2 = hw_rsq(fmaxf(z, 2.5e-7f));
            const float ix = i * fx[v];
            const float gm = g * m;
            const float ixa2 = PRECISE ? ix * (alpha * alpha) : fmaf(-ix, z, ix);  // i x alpha^2
            float k4 = fmaf(fhp[v], alpha, -ixa2 * csg2) * r;  // dlog_a / g * r
            if (!ok) k4 = 0.0f;
            const float gk4 = g * k4;
            o1[v] = gm * i;
            const float t2 = o1[v] * fx[v];   // g m i x
            o2[v] = fmaf(-t2, i, t2);         // ... (1 - i)
            const float t3 = gk4 * cs[v];
            o3[v] = fmaf(-t3, r, t3);         // g k4 (-8 s) (1 - r)
            acc[v] += gk4;
        }
        raw_t r1, r2, r3;
        pack(o1, r1);
        pack(o2, r2);
        pack(o3, r3);
        buffer_store<raw_t>(r1, bdx, store_bytes, j * row_bytes);
        buffer_store<raw_t>(r2, bdxg, store_bytes, j * row_bytes);
        buffer_store<raw_t>(r3, bdag, store_bytes, j * row_bytes);
        if constexpr (GATED) {
            sraw_t r4;
            pack(o4, r4);
            buffer_store<sraw_t>(r4, bdy, lane_on ? slane_bytes : 0x80000000u, j * dy_row_bytes);
        }
        __builtin_amdgcn_sched_barrier(0);  // one row's temporaries live at a time
    }
#pragma unroll
    for (int v = 0; v < V; ++v) s_dl[w][lane * V + v] = acc[v];
    __syncthreads();
    if (w == 0 && lane_on) {
#pragma unroll
        for (int v = 0; v < V; ++v) {
            float sum = 0.0f;
#pragma unroll
            for (int ww = 0; ww < NW; ++ww) sum += s_dl[ww][lane * V + v];
            ws.dlam_part[((size_t)seg * B + b) * D + c_tile + lane_off + v] = sum;
        }
    }
}

template <typename IT, typename ST, int V, int TC, int NW, bool PRECISE, bool GATED>
__global__ __launch_bounds__(NW * kWave, HAWK_BWD_WAVES_PER_SIMD) void rglru_scan_bwd_kernel(
    const IT* __restrict__ x, const IT* __restrict__ xg, const IT* __restrict__ ag,
    const float* __restrict__ lam, const ST* __restrict__ hs, const ST* __restrict__ gout,
    IT* __restrict__ dx, IT* __restrict__ dxg, IT* __restrict__ dag, GateBwdArgs<ST> gate, int B, int T, int D,
    int nseg, int nct, ScanWsPtrs ws) {
    constexpr int CT = kWave * V;
    constexpr int TS = NW * TC;
    __shared__ float2 s_agg[NW][CT];
    __shared__ float2 s_prev[kMaxLookback][CT];
    __shared__ float s_dl[NW][CT];
    __shared__ uint32_t s_ticket[2];

    uint32_t ticket = blockIdx.x, tag = 0;
    if (nseg > 1) take_ticket(ws.ctrl, (uint32_t)nseg * (uint32_t)B * (uint32_t)nct, s_ticket, ticket, tag);

    const int per_seg = B * nct;
    const int pos = (int)fast_div(ticket, ws.div_tiles[0], ws.div_tiles[1]);  // chain position: 0 is the LAST time tile
    const int seg = nseg - 1 - pos;
    const int rem = ticket - pos * per_seg;
    const int b = (int)fast_div((uint32_t)rem, ws.div_nct[0], ws.div_nct[1]);
    const int ct = rem - b * nct;
    if (seg > 0 && seg * TS + TS <= T)
        bwd_tile<IT, ST, V, TC, NW, PRECISE, true, GATED>(x, xg, ag, lam, hs, gout, dx, dxg, dag, gate, B, T, D, nseg,
                                                          seg, pos, b, ct, tag, ws, s_agg, s_prev, s_dl);
    else
        bwd_tile<IT, ST, V, TC, NW, PRECISE, false, GATED>(x, xg, ag, lam, hs, gout, dx, dxg, dag, gate, B, T, D, nseg,
                                                           seg, pos, b, ct, tag, ws, s_agg, s_prev, s_dl);
}

// dLambda[c] = -8 sigmoid(Lambda_c) * sum over rows of the [rows, D] partials.
// 32 channels x 32 row slices per block; fixed summation order, so the result is
// reproducible run to run.
__global__ __launch_bounds__(kColsumThreads) void dlam_reduce_kernel(ColsumTask t) {
    __shared__ float s[kColsumSlices][kColsumCols];
    colsum_block(t, (int)blockIdx.x, s);
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

// Tile shapes.  A lane moves 4 bytes per row access: two bf16 channels (one when D is
// odd) or one fp32 channel, so a wave covers 256 contiguous bytes of a row.  The forward
// keeps 2 floats per element across the carry exchange, the backward keeps the packed
// inputs and one float.  Two workgroups of 8 waves share a CU (4 waves per SIMD, 128 VGPRs each);
// the heights below are the fastest measured, not the tallest that fit: the forward kernels use
// 86 (102 gated) registers at 16 rows, and 20 to 28 rows, or three workgroups of 10 to 14 rows, are
// 1-10 % slower.
#ifndef HAWK_FWD_TC
#define HAWK_FWD_TC 16
#endif
#ifndef HAWK_FWD_NW
#define HAWK_FWD_NW 8
#endif
#ifndef HAWK_BWD_TC
#define HAWK_BWD_TC 12
#endif
#ifndef HAWK_BWD_NW
#define HAWK_BWD_NW 8
#endif
#ifndef HAWK_FWD_GATED_TC
#define HAWK_FWD_GATED_TC 16
#endif
#ifndef HAWK_BWD_GATED_TC
#define HAWK_BWD_GATED_TC 10
#endif
#ifndef HAWK_BWD_GATED_TC1
#define HAWK_BWD_GATED_TC1 12
#endif
constexpr int kFwdTC = HAWK_FWD_TC, kFwdNW = HAWK_FWD_NW;
constexpr int kBwdTC = HAWK_BWD_TC, kBwdNW = HAWK_BWD_NW;
// with two channels per lane the gate's operands cost two more registers per row and the tile
// is two rows shorter; with one channel per lane the plain kernel's tile height still fits
constexpr int kBwdGatedTC = HAWK_BWD_GATED_TC, kBwdGatedTC1 = HAWK_BWD_GATED_TC1;
// With many independent chains in a launch (B x channel tiles) the backward runs 1-3 % faster on
// 64-row tiles: more, shorter-lived tiles, and enough chains to keep the memory system busy
// while each waits on its carry.  With few chains the longer carry chain of short tiles
// costs more than that (4 % at B=2, T=32768, D=4096), so those keep the tall tiles.
#ifndef HAWK_BWD_MANY_TC
#define HAWK_BWD_MANY_TC 8
#endif
#ifndef HAWK_BWD_MANY_CHAINS
#define HAWK_BWD_MANY_CHAINS 128
#endif
constexpr int kBwdManyTC = HAWK_BWD_MANY_TC;
constexpr int kManyChains = HAWK_BWD_MANY_CHAINS;
constexpr int kFwdGatedTC = HAWK_FWD_GATED_TC;  // two channels per lane; one channel keeps kFwdTC

#ifndef HAWK_MAX_V
#define HAWK_MAX_V 2
#endif
int pick_v(int D, int dtype) { return (HAWK_MAX_V >= 2 && dtype == HAWK_DTYPE_BF16 && (D % 2) == 0) ? 2 : 1; }

TileShape fwd_shape(int D, int dtype) { return TileShape{pick_v(D, dtype), kFwdTC, kFwdNW}; }
bool many_chains(int B, int D, int V) { return (long long)B * ((D + kWave * V - 1) / (kWave * V)) >= kManyChains; }
TileShape bwd_shape(int D, int dtype, bool many) {
    return TileShape{pick_v(D, dtype), many ? kBwdManyTC : kBwdTC, kBwdNW};
}
TileShape fwd_gated_shape(int V) { return TileShape{V, V == 2 ? kFwdGatedTC : kFwdTC, kFwdNW}; }
TileShape bwd_gated_shape(int V, bool many) {
    return TileShape{V, many ? kBwdManyTC : (V == 2 ? kBwdGatedTC : kBwdGatedTC1), kBwdNW};
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
int lookback_for(int B, int nct) {
#ifdef HAWK_LOOKBACK
    return HAWK_LOOKBACK;
#else
    const long long chains = (long long)B * nct;
    if (chains <= kFewestChains) return 32;
    if (chains <= kFewerChains) return 16;
    return chains <= kFewChains ? 8 : (chains >= kManyChains ? HAWK_LOOKBACK_MANY : 4);
#endif
}
FastDiv fast_div_for(uint32_t d) {
    FastDiv f;
    f.l = 0;
    while ((1ull << f.l) < d) ++f.l;
    f.m = (uint32_t)(((1ull << 32) * ((1ull << f.l) - d)) / d + 1);
    return f;
}
void set_divisors(ScanWsPtrs& p, int B, int nct) {
    const FastDiv a = fast_div_for((uint32_t)B * (uint32_t)nct), b = fast_div_for((uint32_t)nct);
    p.div_tiles[0] = a.m, p.div_tiles[1] = a.l;
    p.div_nct[0] = b.m, p.div_nct[1] = b.l;
}
ScanWsPtrs carve(void* ws, const WsLayout& l, int lookback) {
    char* p = static_cast<char*>(ws);
    ScanWsPtrs r;
    r.lookback = lookback;
    r.ctrl = reinterpret_cast<unsigned long long*>(p);
    r.incl = reinterpret_cast<unsigned long long*>(p + l.off_incl);
    r.agg_p = reinterpret_cast<unsigned long long*>(p + l.off_aggp);
    r.agg_h = reinterpret_cast<unsigned long long*>(p + l.off_aggh);
    r.dlam_part = reinterpret_cast<float*>(p + l.off_dlam);
    return r;
}

// Type-erased gate operands as they arrive from the C ABI; y == nullptr means "not gated".
struct GateFwdHost {
    const void* y = nullptr;
    void* out = nullptr;
    void* h_last = nullptr;
    uint32_t ldy = 0;
};
struct GateBwdHost {
    const void* y = nullptr;
    void* dy = nullptr;
    uint32_t ldy = 0, lddy = 0;
    ColsumTask* deferred = nullptr;   // not NULL: receives the dLambda reduction instead of a launch
};

template <typename IT, typename OT, int V, int TC, int NW, bool PRECISE, bool GATED>
int launch_fwd(const void* x, const void* xg, const void* ag, const float* lam, void* h, const GateFwdHost& g,
               int B, int T, int D, int nseg, int nct, ScanWsPtrs ws, hipStream_t st) {
    const unsigned grid = (unsigned)nseg * B * nct;
    const GateFwdArgs<OT> gate = {static_cast<const OT*>(g.y), static_cast<OT*>(g.out), static_cast<OT*>(g.h_last),
                                  g.ldy};
    if constexpr (!GATED) {
        hipLaunchKernelGGL((rglru_scan_fwd_kernel<IT, OT, V, TC, NW, PRECISE, false, true>), dim3(grid),
                           dim3(NW * kWave), 0, st, static_cast<const IT*>(x), static_cast<const IT*>(xg),
                           static_cast<const IT*>(ag), lam, static_cast<OT*>(h), gate, B, T, D, nseg, nct, ws);
    } else if (h != nullptr) {
        hipLaunchKernelGGL((rglru_scan_fwd_kernel<IT, OT, V, TC, NW, PRECISE, GATED, true>), dim3(grid),
                           dim3(NW * kWave), 0, st, static_cast<const IT*>(x), static_cast<const IT*>(xg),
                           static_cast<const IT*>(ag), lam, static_cast<OT*>(h), gate, B, T, D, nseg, nct, ws);
    } else {
        hipLaunchKernelGGL((rglru_scan_fwd_kernel<IT, OT, V, TC, NW, PRECISE, GATED, false>), dim3(grid),
                           dim3(NW * kWave), 0, st, static_cast<const IT*>(x), static_cast<const IT*>(xg),
                           static_cast<const IT*>(ag), lam, static_cast<OT*>(h), gate, B, T, D, nseg, nct, ws);
    }
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename IT, typename ST, int V, int TC, int NW, bool PRECISE, bool GATED>
int launch_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* hs,
               const void* gout, void* dx, void* dxg, void* dag, const GateBwdHost& g, int B, int T, int D,
               int nseg, int nct, ScanWsPtrs ws, hipStream_t st) {
    const unsigned grid = (unsigned)nseg * B * nct;
    const GateBwdArgs<ST> gate = {static_cast<const ST*>(g.y), static_cast<ST*>(g.dy), g.ldy, g.lddy};
    hipLaunchKernelGGL((rglru_scan_bwd_kernel<IT, ST, V, TC, NW, PRECISE, GATED>), dim3(grid), dim3(NW * kWave), 0,
                       st, static_cast<const IT*>(x), static_cast<const IT*>(xg), static_cast<const IT*>(ag), lam,
                       static_cast<const ST*>(hs), static_cast<const ST*>(gout), static_cast<IT*>(dx),
                       static_cast<IT*>(dxg), static_cast<IT*>(dag), gate, B, T, D, nseg, nct, ws);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <bool GATED>
int scan_fwd_impl(const void* x, const void* xg, const void* ag, const float* lam, void* h, const GateFwdHost& g,
                  int B, int T, int D, int in_dtype, int out_dtype, void* ws, size_t ws_bytes, hipStream_t st) {
    TileShape s = fwd_shape(D, in_dtype);
    // a lane's pair of bf16 must stay 4-byte aligned in every row of y
    if (GATED) s = fwd_gated_shape(((g.ldy % 2) != 0 || (reinterpret_cast<uintptr_t>(g.y) & 3u) != 0) ? 1 : s.V);
    constexpr int TC2 = GATED ? kFwdGatedTC : kFwdTC;
    const int nseg = ceil_div(T, s.rows());
    const int nct = ceil_div(D, s.chans());
    ScanWsPtrs p = {};
    p.lookback = 4;
    set_divisors(p, B, nct);
    if (nseg > 1) {
        const WsLayout l = layout_for(B, D, nseg, 0);
        if (ws == nullptr || ws_bytes < l.total) return HAWK_ERR_WORKSPACE;
        p = carve(ws, l, lookback_for(B, nct));
        set_divisors(p, B, nct);
    }
    if (in_dtype == HAWK_DTYPE_BF16) {
        if (s.V == 2)
            return launch_fwd<bf16_t, bf16_t, 2, TC2, kFwdNW, false, GATED>(x, xg, ag, lam, h, g, B, T, D, nseg, nct,
                                                                               p, st);
        return launch_fwd<bf16_t, bf16_t, 1, kFwdTC, kFwdNW, false, GATED>(x, xg, ag, lam, h, g, B, T, D, nseg, nct, p,
                                                                           st);
    }
    if (out_dtype == HAWK_DTYPE_BF16)
        return launch_fwd<float, bf16_t, 1, kFwdTC, kFwdNW, false, GATED>(x, xg, ag, lam, h, g, B, T, D, nseg, nct, p,
                                                                          st);
    return launch_fwd<float, float, 1, kFwdTC, kFwdNW, true, GATED>(x, xg, ag, lam, h, g, B, T, D, nseg, nct, p, st);
}

template <bool GATED, bool MANY>
int scan_bwd_shaped(const void* x, const void* xg, const void* ag, const float* lam, const void* hs, const void* gout,
                    void* dx, void* dxg, void* dag, float* dlam, const GateBwdHost& g, int B, int T, int D,
                    int in_dtype, int state_dtype, int V, void* ws, size_t ws_bytes, hipStream_t st) {
    constexpr int TC2 = MANY ? kBwdManyTC : (GATED ? kBwdGatedTC : kBwdTC);
    constexpr int TC1 = MANY ? kBwdManyTC : (GATED ? kBwdGatedTC1 : kBwdTC);
    const TileShape s = GATED ? bwd_gated_shape(V, MANY) : TileShape{V, MANY ? kBwdManyTC : kBwdTC, kBwdNW};
    const int nseg = ceil_div(T, s.rows());
    const int nct = ceil_div(D, s.chans());
    const WsLayout l = layout_for(B, D, nseg, nseg);
    if (ws == nullptr || ws_bytes < l.total) return HAWK_ERR_WORKSPACE;
    ScanWsPtrs p = carve(ws, l, lookback_for(B, nct));
    set_divisors(p, B, nct);
    int rc;
    if (in_dtype == HAWK_DTYPE_BF16) {
        if (s.V == 2)
            rc = launch_bwd<bf16_t, bf16_t, 2, TC2, kBwdNW, false, GATED>(x, xg, ag, lam, hs, gout, dx, dxg, dag, g, B, T,
                                                                         D, nseg, nct, p, st);
        else
            rc = launch_bwd<bf16_t, bf16_t, 1, TC1, kBwdNW, false, GATED>(x, xg, ag, lam, hs, gout, dx, dxg, dag, g, B, T,
                                                                         D, nseg, nct, p, st);
    } else if (state_dtype == HAWK_DTYPE_BF16) {
        rc = launch_bwd<float, bf16_t, 1, TC1, kBwdNW, false, GATED>(x, xg, ag, lam, hs, gout, dx, dxg, dag, g, B, T, D,
                                                                    nseg, nct, p, st);
    } else {
        rc = launch_bwd<float, float, 1, TC1, kBwdNW, true, GATED>(x, xg, ag, lam, hs, gout, dx, dxg, dag, g, B, T, D,
                                                                  nseg, nct, p, st);
    }
    if (rc != HAWK_OK) return rc;
    const ColsumTask reduce{p.dlam_part, dlam, nullptr, lam, nseg * B, D, D};
    if (g.deferred != nullptr) {   // the caller runs it, together with its other closing reductions
        *g.deferred = reduce;
        return HAWK_OK;
    }
    hipLaunchKernelGGL(dlam_reduce_kernel, dim3((unsigned)reduce.blocks()), dim3(kColsumThreads), 0, st, reduce);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <bool GATED>
int scan_bwd_impl(const void* x, const void* xg, const void* ag, const float* lam, const void* hs, const void* gout,
                  void* dx, void* dxg, void* dag, float* dlam, const GateBwdHost& g, int B, int T, int D,
                  int in_dtype, int state_dtype, void* ws, size_t ws_bytes, hipStream_t st) {
    int V = pick_v(D, in_dtype);
    if (GATED) {
        const bool pairs_aligned = (g.ldy % 2) == 0 && (g.lddy % 2) == 0 &&
                                   ((reinterpret_cast<uintptr_t>(g.y) | reinterpret_cast<uintptr_t>(g.dy)) & 3u) == 0;
        if (!pairs_aligned) V = 1;
    }
    if (many_chains(B, D, V))
        return scan_bwd_shaped<GATED, true>(x, xg, ag, lam, hs, gout, dx, dxg, dag, dlam, g, B, T, D, in_dtype,
                                            state_dtype, V, ws, ws_bytes, st);
    return scan_bwd_shaped<GATED, false>(x, xg, ag, lam, hs, gout, dx, dxg, dag, dlam, g, B, T, D, in_dtype,
                                         state_dtype, V, ws, ws_bytes, st);
}

}  // namespace

size_t scan_workspace_bytes(int B, int T, int D, int dtype) {
    // one size serves every scan entry point: the longest chain (shortest tile) decides
    const int V = pick_v(D, dtype);
    const bool many1 = many_chains(B, D, 1), manyv = many_chains(B, D, V);
    const int rows[6] = {fwd_shape(D, dtype).rows(),        fwd_gated_shape(1).rows(),       fwd_gated_shape(2).rows(),
                         bwd_shape(D, dtype, manyv).rows(), bwd_gated_shape(1, many1).rows(), bwd_gated_shape(2, manyv).rows()};
    int n_chain = 0, n_dlam = 0;
    for (int k = 0; k < 6; ++k) {
        const int n = ceil_div(T, rows[k]);
        if (n > n_chain) n_chain = n;
        if (k >= 3 && n > n_dlam) n_dlam = n;  // only the backward kernels write dLambda partials
    }
    return layout_for(B, D, n_chain, n_dlam).total;
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
    if (hipMemcpyAsync(&v, static_cast<const uint32_t*>(ws) + 2, sizeof(v), hipMemcpyDeviceToHost, st) != hipSuccess)
        return HAWK_ERR_LAUNCH;
    if (hipStreamSynchronize(st) != hipSuccess) return HAWK_ERR_LAUNCH;
    *flag = (int)v;
    return HAWK_OK;
}

// ---------------------------------------------------------------------------------------
// Forward scan on the library's own carry buffer, for callers that cannot allocate.
// `scratch` is one fixed array per GPU (each device that loads this code object holds its
// own copy at its own address, from the first use of the library on that device until the
// process ends).  On the host the array's name is only a handle: the device address is
// asked for once per device, with that device current, and kept; kernels, fills and copies
// only ever see that address.
// ---------------------------------------------------------------------------------------
namespace {

static __device__ __align__(256) unsigned char scratch[HAWK_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of the current device's scratch array.
int static_scratch_ptr(void** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return HAWK_ERR_LAUNCH;
    std::lock_guard<std::mutex> guard(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return HAWK_ERR_LAUNCH;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return HAWK_OK;
}

}  // namespace

size_t scan_fwd_static_bytes(int B, int T, int D, int dtype) {
    const TileShape s = fwd_shape(D, dtype);
    const int nseg = ceil_div(T, s.rows());
    return nseg > 1 ? layout_for(B, D, nseg, 0).total : 0;
}

int scan_fwd_static(const void* x, const void* xg, const void* ag, const float* lam, void* h, int B, int T, int D,
                    int dtype, hipStream_t st) {
    if (scan_fwd_static_bytes(B, T, D, dtype) > (size_t)HAWK_STATIC_SCRATCH_BYTES) return HAWK_ERR_SCRATCH_LIMIT;
    // Nothing is cleared, here or ever: the array starts as zeros like any object of static
    // storage, the ticket half of its control word is back at zero when a launch ends, and the
    // words of earlier calls carry older launch tags.  (A clearing kernel on the first caller's
    // stream would race with a second thread's first call on another stream.)
    void* ws = nullptr;
    if (int rc = static_scratch_ptr(&ws)) return rc;
    return scan_fwd_impl<false>(x, xg, ag, lam, h, GateFwdHost{}, B, T, D, dtype, dtype, ws,
                                (size_t)HAWK_STATIC_SCRATCH_BYTES, st);
}

int static_scratch_status(hipStream_t st, int* flag) {
    void* ws = nullptr;
    if (int rc = static_scratch_ptr(&ws)) return rc;
    if (int rc = workspace_status(ws, st, flag)) return rc;
    if (*flag != 0) {
        // the array cannot be re-initialised by the caller, so reading a raised flag lowers it
        // (one word, with the fill kernel: nothing is allocated)
        hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, static_cast<uint32_t*>(ws) + 2, (size_t)1, 0u);
        if (hipGetLastError() != hipSuccess) return HAWK_ERR_LAUNCH;
    }
    return HAWK_OK;
}

bool scan_dtypes_supported(int in_dtype, int state_dtype) {
    if (in_dtype == HAWK_DTYPE_BF16) return state_dtype == HAWK_DTYPE_BF16;
    return in_dtype == HAWK_DTYPE_F32 && (state_dtype == HAWK_DTYPE_F32 || state_dtype == HAWK_DTYPE_BF16);
}

int scan_fwd(const void* x, const void* xg, const void* ag, const float* lam, void* h, int B, int T, int D,
             int in_dtype, int out_dtype, void* ws, size_t ws_bytes, hipStream_t st) {
    return scan_fwd_impl<false>(x, xg, ag, lam, h, GateFwdHost{}, B, T, D, in_dtype, out_dtype, ws, ws_bytes, st);
}

int scan_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* hs, const void* gout,
             void* dx, void* dxg, void* dag, float* dlam, int B, int T, int D, int in_dtype, int state_dtype,
             void* ws, size_t ws_bytes, hipStream_t st) {
    return scan_bwd_impl<false>(x, xg, ag, lam, hs, gout, dx, dxg, dag, dlam, GateBwdHost{}, B, T, D, in_dtype,
                                state_dtype, ws, ws_bytes, st);
}

int scan_gated_fwd(const void* x, const void* xg, const void* ag, const float* lam, const void* y, long long ldy,
                   void* h, void* out, void* h_last, int B, int T, int D, int in_dtype, int out_dtype, void* ws,
                   size_t ws_bytes, hipStream_t st) {
    GateFwdHost g;
    g.y = y;
    g.out = out;
    g.h_last = h_last;
    g.ldy = (uint32_t)ldy;
    return scan_fwd_impl<true>(x, xg, ag, lam, h, g, B, T, D, in_dtype, out_dtype, ws, ws_bytes, st);
}

int scan_gated_bwd(const void* x, const void* xg, const void* ag, const float* lam, const void* y, long long ldy,
                   const void* hs, const void* gout, void* dx, void* dxg, void* dag, void* dy, long long lddy,
                   float* dlam, int B, int T, int D, int in_dtype, int state_dtype, void* ws, size_t ws_bytes,
                   hipStream_t st, ColsumTask* deferred) {
    GateBwdHost g;
    g.y = y;
    g.dy = dy;
    g.ldy = (uint32_t)ldy;
    g.lddy = (uint32_t)lddy;
    g.deferred = deferred;
    return scan_bwd_impl<true>(x, xg, ag, lam, hs, gout, dx, dxg, dag, dlam, g, B, T, D, in_dtype, state_dtype, ws,
                               ws_bytes, st);
}

}  // namespace hawk
