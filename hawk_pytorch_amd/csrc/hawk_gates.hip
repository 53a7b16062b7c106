// Block-diagonal gate projections of the RG-LRU for gfx950 (MFMA, bf16 inputs, fp32 accumulate).
//
// Upstream evaluates the two gate logits of every token with two separate block-diagonal
// linear layers (hawk/external.py:224-233, called at hawk/hawk.py:181-182): two batched
// GEMMs that each read the conv output, plus two bias adds.  Here one kernel reads the
// activations once and writes both logits, bias included:
//   x_rg_lru[m, h*bw + j] = b_i[h, j] + sum_i x[m, h*bw + i] w_i[h, i, j]
//   a_rg_lru[m, h*bw + j] = b_a[h, j] + sum_i x[m, h*bw + i] w_a[h, i, j]
//
// Work decomposition (one workgroup of 16 waves per CU, persistent over row tiles):
//   * a workgroup owns 256 adjacent channels (256 / bw whole blocks) and walks over tiles
//     of 32 rows;
//   * wave (g, c), g = gate, c = 0..7, owns the 32 output columns [32c, 32c+32) of gate g
//     and keeps that slice of the weights, bw x 32, in registers as MFMA B operands for the
//     whole kernel (64 VGPRs at bw = 256): the weights are read once per workgroup;
//   * the 32 x 256 activation tile goes global -> registers -> LDS with 16-byte accesses
//     along rows (fp32 activations are rounded to bf16 on the way); two register sets and
//     two LDS buffers keep the next two tiles in flight; all 16 waves read the tile back as
//     MFMA A operands;
//   * results pass through LDS once more so that each row leaves in 512-byte (bf16) or
//     1-KiB (fp32) pieces.
// Per 32-row tile a CU moves 16 KiB in and 32 KiB out (bf16) against 16 waves x bw/16 MFMAs
// of 32x32x16.  At bw = 256 that is about 2 k cycles of matrix-core time and, because every
// MFMA takes a fresh 1 KiB A operand from LDS, as many cycles of LDS time, against about 5 k
// cycles of HBM time at 5 TB/s; with the result pass and the barriers a tile takes about 6 k.
#include "hawk_scan.h"

#include <stdint.h>

#include <atomic>

#include "hawk_device.h"

namespace hawk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16x8 bf16x8_t;
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kGroup = 256;                    // channels per workgroup
constexpr int kTileRows = 32;                  // rows per MFMA tile
constexpr int kGateThreads = 1024;             // 16 waves
constexpr int kARowBytes = kGroup * 2 + 16;    // bf16 row + pad: 8 lanes' 16-byte reads cover all banks
constexpr int kATileBytes = kTileRows * kARowBytes;
constexpr int kDefaultNumCU = 256;   // MI355X; used when the device cannot be asked
// Row counts up to this one take the forward kernel that is cut by output columns.
#ifndef HAWK_GATE_MIN_SPLIT_TILES
#define HAWK_GATE_MIN_SPLIT_TILES 4
#endif
#ifndef HAWK_GATE_SMALL_M
#define HAWK_GATE_SMALL_M 512
#endif
// Tiles in flight per workgroup of the weight-gradient kernel (bf16 operands; half as many fp32).
#ifndef HAWK_GATE_DW_SETS
#define HAWK_GATE_DW_SETS 2
#endif


// Weight fetches that go through a buffer resource (scalar base, one per-lane offset, scalar
// per-access offset) use the default cache policy: every workgroup re-reads them.
// eight consecutive weights as a bf16 MFMA operand (scaled by `live`, 0 or 1)
__device__ __forceinline__ bf16x8_t load_weight8(rsrc_t r, uint32_t lane_bytes, uint32_t off_bytes, float live,
                                                 const float*) {
    const u32x4 a = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, lane_bytes, off_bytes, kAuxDefault));
    const u32x4 b = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, lane_bytes, off_bytes + 16, kAuxDefault));
    const u32x4 packed = {pack_bf16x2(live * __uint_as_float(a.x), live * __uint_as_float(a.y)),
                          pack_bf16x2(live * __uint_as_float(a.z), live * __uint_as_float(a.w)),
                          pack_bf16x2(live * __uint_as_float(b.x), live * __uint_as_float(b.y)),
                          pack_bf16x2(live * __uint_as_float(b.z), live * __uint_as_float(b.w))};
    return __builtin_bit_cast(bf16x8_t, packed);
}
__device__ __forceinline__ bf16x8_t load_weight8(rsrc_t r, uint32_t lane_bytes, uint32_t off_bytes, float live,
                                                 const bf16_t*) {
    u32x4 a = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, lane_bytes, off_bytes, kAuxDefault));
    if (live == 0.0f) a = u32x4{0u, 0u, 0u, 0u};
    return __builtin_bit_cast(bf16x8_t, a);
}

// Eight consecutive activations as they sit in registers between the global load and the LDS store.
template <typename XT>
struct Row8;
template <>
struct Row8<bf16_t> {
    u32x4 v;
    __device__ __forceinline__ void load(const bf16_t* p, bool ok) {
        v = ok ? *reinterpret_cast<const u32x4*>(p) : u32x4{0u, 0u, 0u, 0u};
    }
    // through a buffer resource: bytes outside it read as zeros, without a branch
    __device__ __forceinline__ void load_buf(rsrc_t r, uint32_t off) { v = buffer_load<u32x4>(r, off, 0u); }
    __device__ __forceinline__ void load_buf_default(rsrc_t r, uint32_t off) {
        v = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, off, 0u, kAuxDefault));
    }
    __device__ __forceinline__ u32x4 as_bf16() const { return v; }
    __device__ __forceinline__ void as_f32(f32x4& a, f32x4& b) const {
        a = f32x4{bf16_lo(v.x), bf16_hi(v.x), bf16_lo(v.y), bf16_hi(v.y)};
        b = f32x4{bf16_lo(v.z), bf16_hi(v.z), bf16_lo(v.w), bf16_hi(v.w)};
    }
};
template <>
struct Row8<float> {
    f32x4 lo, hi;
    __device__ __forceinline__ void load(const float* p, bool ok) {
        const f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
        lo = ok ? *reinterpret_cast<const f32x4*>(p) : z;
        hi = ok ? *reinterpret_cast<const f32x4*>(p + 4) : z;
    }
    __device__ __forceinline__ void load_buf(rsrc_t r, uint32_t off) {
        lo = buffer_load<f32x4>(r, off, 0u);
        hi = buffer_load<f32x4>(r, off, 16u);
    }
    __device__ __forceinline__ u32x4 as_bf16() const {
        return u32x4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y),
                     pack_bf16x2(hi.z, hi.w)};
    }
    __device__ __forceinline__ void as_f32(f32x4& a, f32x4& b) const {
        a = lo;
        b = hi;
    }
};

// Eight consecutive output columns of four consecutive input channels of a weight matrix, as
// they arrive from memory, and the same 32 values as bf16 regrouped by output column
// (column e: input channels 0..3 in two dwords), which is what the LDS transposition writes.
template <typename WT>
struct WeightQuad;
template <>
struct WeightQuad<bf16_t> {
    static constexpr int kDwords = 16;
    u32x4 q[4];
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int r = 0; r < 4; ++r) q[r] = u32x4{0u, 0u, 0u, 0u};
    }
    __device__ __forceinline__ void load(const bf16_t* p, size_t row_stride) {
#pragma unroll
        for (int r = 0; r < 4; ++r) q[r] = *reinterpret_cast<const u32x4*>(p + r * row_stride);
    }
    __device__ __forceinline__ u32x2 column(int e) const {
        const uint32_t a = q[0][e / 2], b = q[1][e / 2], c = q[2][e / 2], d = q[3][e / 2];
        if (e % 2 == 0) return u32x2{(a & 0xffffu) | (b << 16), (c & 0xffffu) | (d << 16)};
        return u32x2{(a >> 16) | (b & 0xffff0000u), (c >> 16) | (d & 0xffff0000u)};
    }
};
template <>
struct WeightQuad<float> {
    static constexpr int kDwords = 32;
    f32x4 q[4][2];
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int r = 0; r < 4; ++r) q[r][0] = q[r][1] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    __device__ __forceinline__ void load(const float* p, size_t row_stride) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            q[r][0] = *reinterpret_cast<const f32x4*>(p + r * row_stride);
            q[r][1] = *reinterpret_cast<const f32x4*>(p + r * row_stride + 4);
        }
    }
    __device__ __forceinline__ u32x2 column(int e) const {
        return u32x2{pack_bf16x2(q[0][e / 4][e % 4], q[1][e / 4][e % 4]),
                     pack_bf16x2(q[2][e / 4][e % 4], q[3][e / 4][e % 4])};
    }
};

__device__ __forceinline__ void store_out(unsigned char* p, float v, bf16_t*) {
    *reinterpret_cast<uint16_t*>(p) = to_bf16_bits(v);
}
__device__ __forceinline__ void store_out(unsigned char* p, float v, float*) { *reinterpret_cast<float*>(p) = v; }

// LDS scratch of the forward kernel's weight transposition: [2 gates][256 columns][kPassK + 8] bf16.
template <int BW>
struct WeightStage {
    static constexpr int kPassK = BW < 64 ? BW : 64;
    static constexpr int kRowBytes = kPassK * 2 + 16;
    static constexpr int kBytes = 2 * kGroup * kRowBytes;
};

// With CONV the kernel's input is the temporal conv's input (hawk/hawk.py:172-176 upstream:
// conv, then both gates) and the kernel applies the width-4 causal depthwise conv itself: a
// raw tile lands in LDS with the three rows in front of it, every thread forms one row piece of
// the conv output from four raw rows (fp32, taps oldest first, the arithmetic of
// conv1d_fwd_kernel), writes it into the MFMA A tile and to memory, where the scan reads it.
// The conv output is then never read back by this kernel: one pass over a tensor less.
struct ConvFront {
    const float* w;   // [4, D], tap 3 multiplies the row itself
    const float* b;   // [D]
    bf16_t* u;        // conv output, dense [M, D]
    int T;            // rows per sequence: rows of one sequence never see another's
    long long ldx;    // row stride of x in elements
};
constexpr int kConvTaps = 4;
constexpr int kRTileBytes = (kTileRows + kConvTaps - 1) * kARowBytes;   // a raw tile and its history rows
template <typename OT>
constexpr size_t gate_fwd_lds_bytes(bool conv) {
    return 2 * kATileBytes + (sizeof(OT) > 2 ? 1 : 2) * (size_t)kTileRows * (2 * kGroup * sizeof(OT) + 16) +
           (conv ? 2 * (size_t)kRTileBytes + (kConvTaps + 1) * kGroup * sizeof(float) : 0);
}

template <typename XT, typename WT, typename OT, int BW, bool CONV>
__global__ __launch_bounds__(kGateThreads, 1) void gate_proj_fwd_kernel(
    const XT* __restrict__ x, const WT* __restrict__ w_i, const float* __restrict__ b_i,
    const WT* __restrict__ w_a, const float* __restrict__ b_a, OT* __restrict__ out_i, OT* __restrict__ out_a,
    int M, int D, int nb, int ntiles, ConvFront cf) {
    static_assert(BW == 32 || BW == 64 || BW == 128 || BW == 256, "block width");
    static_assert(!CONV || sizeof(XT) == 2, "the fused conv runs on bf16 activations");
    constexpr int KS = BW / 16;                                     // MFMA k-steps per output tile
    constexpr int G = kGroup / BW;                                  // whole blocks per workgroup
    constexpr int kORowBytes = 2 * kGroup * (int)sizeof(OT) + 16;   // both gates' columns of one row + pad
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* sA = smem;                     // two activation tiles
    constexpr bool kTwoResultTiles = sizeof(OT) == 2;                     // fp32 results: no room for two
    constexpr int kOBuf = kTwoResultTiles ? kTileRows * kORowBytes : 0;   // distance between the two result tiles
    unsigned char* sO = smem + 2 * kATileBytes;                           // result tiles
    unsigned char* sR = sO + (kTwoResultTiles ? 2 : 1) * kTileRows * kORowBytes;   // CONV: two raw tiles
    float* sCW = reinterpret_cast<float*>(sR + 2 * kRTileBytes);          // CONV: taps and bias of the group

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int group = blockIdx.y, worker = blockIdx.x, nworkers = gridDim.x;

    // ---- this wave's slice of the weights, as MFMA B operands: lane holds output column
    //      (lane % 32) and 8 consecutive input channels starting at 16 s + 8 (lane / 32)
    const int g = w >> 3, c = w & 7;
    const int blk = (32 * c) / BW;                 // block within the group
    const int col = lane & 31, khalf = 8 * (lane >> 5);
    const float* bsel = g ? b_a : b_i;
    const int ch = group * kGroup + 32 * c + col;  // channel of the layer
    const float bias = (bsel != nullptr && ch < D) ? bsel[ch] : 0.0f;

    // ---- tile traffic: thread -> (row, 8 consecutive channels)
    const int lrow = tid >> 5, lc8 = tid & 31;
    const int lcol = group * kGroup + lc8 * 8;
    const bool col_ok = lcol < D;
    // (through a buffer resource that covers the rows of the tile which exist: no branch)
    const uint32_t x_row_bytes = (uint32_t)D * (uint32_t)sizeof(XT);
    const uint32_t x_off = col_ok ? (uint32_t)(lrow * D + lcol) * (uint32_t)sizeof(XT) : 0x80000000u;
    auto load_tile = [&](int it, Row8<XT>& r) {
        const int t = min(worker + it * nworkers, ntiles);   // past the last tile: an empty window
        const int row0 = min(t * kTileRows, M);
        if constexpr (sizeof(XT) == 2)
            r.load_buf_default(make_rsrc(x + (size_t)row0 * D, (uint32_t)min(M - row0, kTileRows) * x_row_bytes), x_off);
        else
            r.load_buf(make_rsrc(x + (size_t)row0 * D, (uint32_t)min(M - row0, kTileRows) * x_row_bytes), x_off);
    };
    auto stage_tile = [&](int buf, const Row8<XT>& r) {
        *reinterpret_cast<u32x4*>(sA + buf * kATileBytes + lrow * kARowBytes + lc8 * 16) = r.as_bf16();
    };
    // CONV: a raw tile is its 32 rows and the three rows in front of them (threads of the first
    // three rows fetch one history piece each; every other thread's second load is out of range
    // and costs no memory access).  Rows in front of the tensor do not exist and are masked later.
    const uint32_t ldx_bytes = CONV ? (uint32_t)cf.ldx * 2u : 0u;
    auto load_raw_tile = [&](int it, auto& r, auto& hist) {
        const int t = min(worker + it * nworkers, ntiles);
        const int row0 = min(t * kTileRows, M);
        const int hb = row0 >= kConvTaps - 1 ? kConvTaps - 1 : 0;
        const int nrows = min(M - row0, kTileRows) + hb;
        const rsrc_t rs = make_rsrc(x + (size_t)(row0 - hb) * (size_t)cf.ldx,
                                    nrows > 0 ? (uint32_t)(nrows - 1) * ldx_bytes + (uint32_t)D * 2u : 0u);
        const uint32_t col_bytes = (uint32_t)lcol * 2u;
        r.load_buf_default(rs, col_ok ? (uint32_t)(hb + lrow) * ldx_bytes + col_bytes : 0x80000000u);
        hist.load_buf_default(rs, (col_ok && lrow < hb) ? (uint32_t)lrow * ldx_bytes + col_bytes : 0x80000000u);
    };
    auto stage_raw_tile = [&](int buf, const auto& r, const auto& hist) {
        unsigned char* dst = sR + buf * kRTileBytes + lrow * kARowBytes + lc8 * 16;
        *reinterpret_cast<u32x4*>(dst + (kConvTaps - 1) * kARowBytes) = r.as_bf16();
        if (lrow < kConvTaps - 1) *reinterpret_cast<u32x4*>(dst) = hist.as_bf16();
    };
    // conv of tile j from raw buffer `buf` into A buffer `buf`, and out to memory
    auto conv_tile = [&](int j, int buf) {
        const int tt = worker + j * nworkers;
        if (tt >= ntiles) return;
        const int row0 = tt * kTileRows;
        int t = row0 % cf.T + lrow;   // position in the sequence (T >= 32: at most one wrap)
        if (t >= cf.T) t -= cf.T;
        const unsigned char* src = sR + buf * kRTileBytes + lrow * kARowBytes + lc8 * 16;
        const float* cw = sCW + lc8 * 8;
        // four channels at a time: the weights of the matrix products leave few registers
        u32x4 o;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const f32x4 b4 = *reinterpret_cast<const f32x4*>(cw + kConvTaps * kGroup + 4 * hf);
            float acc[4] = {b4[0], b4[1], b4[2], b4[3]};
#pragma unroll
            for (int k = 0; k < kConvTaps; ++k) {
                u32x2 v = *reinterpret_cast<const u32x2*>(src + k * kARowBytes + 8 * hf);   // row t - (3 - k)
                if (t < kConvTaps - 1 - k) v = u32x2{0u, 0u};                               // before the sequence starts
                const f32x4 w4 = *reinterpret_cast<const f32x4*>(cw + k * kGroup + 4 * hf);
                acc[0] = fmaf(w4[0], bf16_lo(v.x), acc[0]);
                acc[1] = fmaf(w4[1], bf16_hi(v.x), acc[1]);
                acc[2] = fmaf(w4[2], bf16_lo(v.y), acc[2]);
                acc[3] = fmaf(w4[3], bf16_hi(v.y), acc[3]);
            }
            o[2 * hf] = pack_bf16x2(acc[0], acc[1]);
            o[2 * hf + 1] = pack_bf16x2(acc[2], acc[3]);
        }
        *reinterpret_cast<u32x4*>(sA + buf * kATileBytes + lrow * kARowBytes + lc8 * 16) = o;
        const int row = row0 + lrow;
        if (row < M && col_ok)
            __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(cf.u + (size_t)row * D + lcol));
    };

    // Two register sets alternate as landing places for the prefetched tiles (tile it+1 is
    // staged into LDS during iteration it, and its registers are reloaded with tile it+3), and
    // the loop is unrolled by two so that buffers and registers are fixed per half.  With CONV a
    // tile is staged raw one iteration earlier (tile it+2 during iteration it, its registers
    // reloaded with tile it+4) and convolved into the A buffer during iteration it+1's stores.
    Row8<XT> ra, rb, ha, hb_;
    if constexpr (CONV) {
        load_raw_tile(0, ra, ha);
        load_raw_tile(1, rb, hb_);
        if (tid < kGroup) {
            const int cch = group * kGroup + tid;
#pragma unroll
            for (int k = 0; k < kConvTaps; ++k) sCW[k * kGroup + tid] = cch < D ? cf.w[(size_t)k * D + cch] : 0.0f;
            sCW[kConvTaps * kGroup + tid] = cch < D ? cf.b[cch] : 0.0f;
        }
    } else {
        load_tile(0, ra);
        load_tile(1, rb);
    }
    __builtin_amdgcn_sched_barrier(0);  // the first tiles travel while the weights are fetched

    // ---- the weights.  A lane's B operand is 8 consecutive input channels of one output
    //      column, which lie bw elements apart in memory, so they are fetched the way memory
    //      wants it (a thread reads 8 consecutive output columns of 4 consecutive input
    //      channels, 16 or 32 bytes each) and transposed through LDS with 8-byte writes, up to
    //      64 input channels of both gates per pass.  A group past the last block (D not a
    //      multiple of 256) gets zeros.
    constexpr int kPassK = WeightStage<BW>::kPassK, kTRowBytes = WeightStage<BW>::kRowBytes;
    constexpr int kQuads = kPassK / 4, kTasks = 2 * kQuads * (kGroup / 8);
    bf16x8 bfrag[KS];
    {
        const int tgate = tid / (kQuads * (kGroup / 8)), trem = tid % (kQuads * (kGroup / 8));
        const int tkq = trem % kQuads, tn8 = (trem / kQuads) * 8;  // thread -> (4 input channels, 8 output columns)
        const int tblk = tn8 / BW;
        const bool twrites = tid < kTasks;
        const bool tloads = twrites && group * G + tblk < nb;
        const WT* tsrc_w = (tgate ? w_a : w_i) + ((size_t)(group * G + tblk) * BW + 4 * tkq) * BW + (tn8 - tblk * BW);
        unsigned char* tdst = smem + (tgate * kGroup + tn8) * kTRowBytes + tkq * 8;
        const unsigned char* tsrc = smem + ((g * kGroup + 32 * c + col) * kTRowBytes + khalf * 2);
        // as many passes are kept in flight as fit in 64 registers; the registers of the
        // matrix operands fill up as those of the raw rows drain
        constexpr int NP = BW / kPassK;
        constexpr int kAhead = 64 / WeightQuad<WT>::kDwords < NP ? 64 / WeightQuad<WT>::kDwords : NP;
        WeightQuad<WT> raw[NP];
#pragma unroll
        for (int pass = 0; pass < NP; ++pass) raw[pass].clear();
        if (tloads) {
#pragma unroll
            for (int pass = 0; pass < kAhead; ++pass) raw[pass].load(tsrc_w + (size_t)pass * kPassK * BW, BW);
        }
#pragma unroll
        for (int pass = 0; pass < NP; ++pass) {
            u32x2 cols[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) cols[e] = raw[pass].column(e);
            if (pass + kAhead < NP && tloads)
                raw[pass + kAhead].load(tsrc_w + (size_t)(pass + kAhead) * kPassK * BW, BW);
            if (pass > 0) __syncthreads();  // the previous pass has been read
            if (twrites) {
#pragma unroll
                for (int e = 0; e < 8; ++e) *reinterpret_cast<u32x2*>(tdst + e * kTRowBytes) = cols[e];
            }
            __syncthreads();
#pragma unroll
            for (int s2 = 0; s2 < kPassK / 16; ++s2)
                bfrag[pass * (kPassK / 16) + s2] = *reinterpret_cast<const bf16x8*>(tsrc + 32 * s2);
        }
        __syncthreads();
    }

    if constexpr (CONV) {
        stage_raw_tile(0, ra, ha);
        load_raw_tile(2, ra, ha);
        stage_raw_tile(1, rb, hb_);
        load_raw_tile(3, rb, hb_);
        __syncthreads();
        conv_tile(0, 0);
    } else {
        stage_tile(0, ra);
        load_tile(2, ra);
    }
    __syncthreads();

    const int a_off = col * kARowBytes + (blk * BW + khalf) * 2;
    unsigned char* o_base = sO + (4 * (lane >> 5)) * kORowBytes + (g * kGroup + 32 * c + col) * (int)sizeof(OT);

    auto step = [&](int it, int cur, Row8<XT>& rnext, Row8<XT>& hnext) {
        // 32 x 32 output tile of this wave: A operands from LDS, B operands resident.  The A
        // operands are fetched four k-steps at a time: the weights leave no room for more.
        f32x16 acc = {};
        const unsigned char* a_base = sA + cur * kATileBytes + a_off;
        constexpr int kBatch = KS < 4 ? KS : 4;
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += kBatch) {
            bf16x8 a[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) a[j] = *reinterpret_cast<const bf16x8*>(a_base + (s0 + j) * 32);
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], bfrag[s0 + j], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // accumulator register r of a lane is row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = 8 * (r / 4) + (r % 4);
            store_out(o_base + cur * kOBuf + m * kORowBytes, acc[r] + bias, static_cast<OT*>(nullptr));
        }
        if constexpr (CONV) {
            // the conv of tile it+1 (raw since the last step) into the other A buffer, then raw tile
            // it+2 into the raw buffer tile it has left and tile it+4 into its registers
            if constexpr (kTwoResultTiles) conv_tile(it + 1, cur ^ 1);
            stage_raw_tile(cur, rnext, hnext);
            load_raw_tile(it + 4, rnext, hnext);
        } else {
            // tile it+1 into the other buffer, tile it+3 into the registers it leaves
            stage_tile(cur ^ 1, rnext);
            load_tile(it + 3, rnext);
        }
        __syncthreads();
        // a gate's row of the group is 32 (bf16) or 64 (fp32) pieces of 16 bytes; consecutive
        // threads take consecutive pieces, so that every store instruction writes whole rows
        constexpr int kPieces = kGroup * (int)sizeof(OT) / 16;
        constexpr int kPerThread = kTileRows * kPieces / kGateThreads;
#pragma unroll
        for (int q = 0; q < kPerThread; ++q) {
            const int piece = tid + q * kGateThreads;
            const int prow = piece / kPieces, pc = piece % kPieces;
            const int row = (worker + it * nworkers) * kTileRows + prow;
            const int ocol = group * kGroup + pc * (16 / (int)sizeof(OT));
            if (ocol < D && row < M) {
                const unsigned char* src = sO + cur * kOBuf + prow * kORowBytes + pc * 16;
                const u32x4 vi = *reinterpret_cast<const u32x4*>(src);
                const u32x4 va = *reinterpret_cast<const u32x4*>(src + kGroup * (int)sizeof(OT));
                __builtin_nontemporal_store(vi, reinterpret_cast<u32x4*>(out_i + (size_t)row * D + ocol));
                __builtin_nontemporal_store(va, reinterpret_cast<u32x4*>(out_a + (size_t)row * D + ocol));
            }
        }
        // (issued behind the matrix products instead, the conv spills and the kernel takes 194 us
        // against 150 us at 32768 rows of 2560 channels)
        // Without the conv the next tile's results go to the other result tile, and the barrier in
        // the middle of the next step orders everything else: a wave that is done with its stores
        // goes straight on to the next tile's products.
        if constexpr (!kTwoResultTiles) {
            if constexpr (CONV) conv_tile(it + 1, cur ^ 1);
            __syncthreads();
        }
    };

    for (int it = 0; worker + it * nworkers < ntiles; it += 2) {
        if constexpr (CONV) step(it, 0, ra, ha); else step(it, 0, rb, hb_);
        if (worker + (it + 1) * nworkers >= ntiles) break;
        if constexpr (CONV) step(it + 1, 1, rb, hb_); else step(it + 1, 1, ra, ha);
    }
}

// ---------------------------------------------------------------------------------------
// The same projections for few rows (decode: one row per sequence).  With M/32 row tiles the
// kernel above keeps at most (M/32) x (D/256) compute units busy and each of them spends most
// of its time fetching a 256-column slice of the weights for a single tile.  Here the work is
// cut the other way: a workgroup of 8 waves owns 32 output columns of one gate.  It reads
// that bw x 32 slice of the weights once with 16-byte accesses along the rows of the weight
// matrix (64 contiguous bytes each), transposes it through LDS so that a lane finds its 8
// consecutive input channels of one output column in 16 contiguous bytes, and every wave takes
// its B operands from there.  Wave w then walks over row tiles w, w + 8 x gridDim.y, ...: A
// operands come straight from memory (a lane's 8 consecutive input channels are 16 contiguous
// bytes), results leave from the accumulator registers (64 contiguous bytes per row and half
// wave, which is acceptable while M is small).
// ---------------------------------------------------------------------------------------
constexpr int kSmallWaves = 8;

template <typename XT, typename WT, typename OT, int BW>
__global__ __launch_bounds__(kSmallWaves* kWave, sizeof(XT) == 2 ? 4 : 2) void gate_proj_fwd_small_kernel(
    const XT* __restrict__ x, const WT* __restrict__ w_i, const float* __restrict__ b_i,
    const WT* __restrict__ w_a, const float* __restrict__ b_a, OT* __restrict__ out_i, OT* __restrict__ out_a,
    int M, int D, int ntiles) {
    constexpr int KS = BW / 16;
    constexpr int kWRowBytes = BW * 2 + 16;        // one output column's bw weights + pad
    __shared__ __align__(16) unsigned char sW[32 * kWRowBytes];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int ncol = D / 32;                       // D is a multiple of bw, bw a multiple of 32
    const int g = (int)blockIdx.x / ncol;          // gate
    const int c0 = ((int)blockIdx.x - g * ncol) * 32;
    const int h = c0 / BW;                         // a 32-column tile never straddles two blocks
    const int col = lane & 31, khalf = 8 * (lane >> 5);
    const WT* wsel = g ? w_a : w_i;
    const float* bsel = g ? b_a : b_i;
    OT* out = g ? out_a : out_i;
    int rt = (int)blockIdx.y * kSmallWaves + w;
    const int rstep = (int)gridDim.y * kSmallWaves;

    // A operands of the first row tile travel while the weights are staged
    const XT* xcol = x + (size_t)h * BW + khalf;
    u32x4 abf[KS];
    auto load_rows = [&](int t) {
        const int row = t * kTileRows + col;
        const bool ok = t < ntiles && row < M;
        const XT* p = xcol + (ok ? (size_t)row * D : 0);
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            Row8<XT> r;
            r.load(p + 16 * s, ok);
            abf[s] = r.as_bf16();
        }
    };
    load_rows(rt);
    __builtin_amdgcn_sched_barrier(0);

    // weights: thread -> (4 input channels, 8 consecutive output columns), written transposed
    if (tid < BW) {
        const int tkq = tid % (BW / 4), tn8 = (tid / (BW / 4)) * 8;
        WeightQuad<WT> raw;
        raw.load(wsel + ((size_t)h * BW + 4 * tkq) * BW + (c0 - h * BW) + tn8, BW);
#pragma unroll
        for (int e = 0; e < 8; ++e)
            *reinterpret_cast<u32x2*>(sW + (tn8 + e) * kWRowBytes + tkq * 8) = raw.column(e);
    }
    const float bias = bsel != nullptr ? bsel[c0 + col] : 0.0f;
    __syncthreads();
    // B operands stay in LDS and are read per use: the registers go to the A operands, and
    // two workgroups fit a compute unit (one with fp32 activations, whose rows take twice the
    // registers while they travel)
    const unsigned char* bsrc = sW + col * kWRowBytes + khalf * 2;

    for (; rt < ntiles; rt += rstep) {
        f32x16 acc = {};
        constexpr int kBatch = KS < 4 ? KS : 4;
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += kBatch) {
            bf16x8 b[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) b[j] = *reinterpret_cast<const bf16x8*>(bsrc + 32 * (s0 + j));
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, abf[s0 + j]), b[j], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (rt + rstep < ntiles) load_rows(rt + rstep);
        __builtin_amdgcn_sched_barrier(0);
        // accumulator register r of a lane is row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32
        const int row0 = rt * kTileRows + 4 * (lane >> 5);
        OT* obase = out + (size_t)row0 * D + c0 + col;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = 8 * (r / 4) + (r % 4);
            if (row0 + m < M)
                store_out(reinterpret_cast<unsigned char*>(obase + (size_t)m * D), acc[r] + bias,
                          static_cast<OT*>(nullptr));
        }
    }
}

// ---------------------------------------------------------------------------------------
// One decode step of a layer's whole recurrent core in one launch: the conv window roll and
// conv, both gate projections, the RG-LRU state update and the output gate
// (hawk/hawk.py:137-151, :169-182, :196-198 and hawk/cache.py:37-43 upstream; the three launches
// hawk_conv1d_step, hawk_gate_proj_fwd, hawk_rglru_step_gated here).  Every kernel of a decode
// step runs for about as long as it takes to start, so what this saves is two starts per layer.
//
// A workgroup of 8 waves owns 32 batch rows of one block of the projections, i.e. every
// channel that those rows' outputs in the block depend on:
//   1. all waves: conv of the rows' bw channels from the window in conv_state and the new row;
//      the window is rolled in place, the result goes to LDS as bf16 (the MFMA A operand, and x
//      of the recurrence);
//   2. wave c < bw/32: the bw x 32 slices of both weight matrices that produce output columns
//      32c.. of the block, transposed through a wave-private LDS region into B operands, one
//      gate after the other (the second gate's weights travel while the first is multiplied);
//   3. the same wave adds the biases and leaves its 32 x 32 logits in LDS as bf16, over the
//      weights, which are done with by then;
//   4. all waves: recurrence and output gate, thread -> (row, 8 consecutive channels) with
//      16-byte accesses to y, recc_state (updated in place) and out.  (Applied straight to the
//      accumulators, with 2-byte gathers and scatters per element, this step alone made the
//      kernel 13 us slower at a block width of 32 and 2 us at 128.)
// Intermediate roundings are those of the three separate launches (conv output and logits to
// bf16), so the two paths give the same bits.
// At 256 rows, replayed from a graph: 18.6 us at a block width of 256 against 19.4 us for the
// three launches it replaces, 8.4 against 14.5 us at a width of 128, 8.9 against 14.1 us at 32.
// At 256 the time is the launch, staging, matrix products, operand loads and stores (8 us),
// fetching a block's 256 KiB of weights into one compute unit (4.8 us; fetching the second
// gate's earlier does not shorten it), the conv (2.9 us) and the recurrence (1.6 us).  One
// workgroup per (32 rows, block) is 80 workgroups there: what the launch saves in starts it
// loses to running on a third of the device, and its gain is on the host side (one call
// instead of three plus a copy).
//
// With a workspace of counters the output columns of a block are cut over NS workgroups
// (NS = 2 or 4: 64 KiB of weights each at a width of 256 instead of 256 KiB through one L1, and
// four times the compute units).  Every one of them needs the conv output of all the block's
// channels, so each computes it from the window, but none rolls the window while reading: a
// workgroup that has read it (its loads have returned) counts itself in on the (rows, block)
// counter, and in the one that counts in last, when no reader is left, the waves that have no
// matrix products to do roll the window while the others multiply, and set the counter back to
// zero for the next launch.  (Rolling at the end of the workgroup's work instead put the rows'
// round trip on the critical path.)  At a width of 256 and 10 blocks: 13.5 us at 256 rows with two
// workgroups per block against 18.4 us with one, 8.8 against 17.4 us at 32 rows with four.
// ---------------------------------------------------------------------------------------
constexpr int kCoreWaves = 8;
constexpr int kCoreMaxW = 8;

template <int BW>
struct CoreLds {
    static constexpr int kRowBytes = BW * 2 + 16;                       // bf16 row + pad
    static constexpr int kUBytes = kTileRows * kRowBytes;               // conv output tile
    static constexpr int kWaveBytes = 32 * kRowBytes;                   // one wave's 32 weight columns
    static constexpr int kWaves = BW / 32 < kCoreWaves ? BW / 32 : kCoreWaves;
    static constexpr int kORowBytes = 2 * BW * 2 + 16;                  // both gates' logits of one row + pad
    static constexpr int kWeightBytes = kWaves * kWaveBytes;
    static constexpr int kLogitBytes = kTileRows * kORowBytes;          // reuses the weights' space
    static constexpr int kBytes = kUBytes + (kWeightBytes > kLogitBytes ? kWeightBytes : kLogitBytes);
};

// all LDS traffic of this wave issued so far has completed, and the compiler keeps what
// follows behind it
__device__ __forceinline__ void wave_lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// WC: the conv window's width when it is known at compile time (4, upstream's), else 0: with a
// known width the window's loads are straight-line code, all in flight together, instead of a
// chain of branches each waiting for its own load.
template <typename WT, typename ST, int BW, int NS, int WC>
__global__ __launch_bounds__(kCoreWaves* kWave, 1) void decode_core_kernel(
    bf16_t* __restrict__ conv_state, const bf16_t* __restrict__ x_new, size_t ldx, const float* __restrict__ conv_w,
    const float* __restrict__ conv_b, const WT* __restrict__ w_i, const float* __restrict__ b_i,
    const WT* __restrict__ w_a, const float* __restrict__ b_a, const float* __restrict__ lam,
    const bf16_t* __restrict__ y, size_t ldy, ST* __restrict__ state, bf16_t* __restrict__ out, int M, int D,
    int W_runtime, int ntiles, bool vec_io, uint32_t* __restrict__ counters) {
    const int W = WC > 0 ? WC : W_runtime;
    static_assert(BW % 32 == 0 && BW <= 32 * kCoreWaves, "one wave per 32 output columns of a block");
    static_assert(NS >= 1 && (BW / NS) % 32 == 0, "whole 32-column slices per workgroup");
    static_assert(NS == 1 || BW / NS / 32 < kCoreWaves, "a cut workgroup needs a wave without matrix products");
    constexpr int KS = BW / 16;
    constexpr int CW = BW / NS;       // output columns of the block that this workgroup produces
    constexpr int NT = CW / 32;
    constexpr int kRowBytes = CoreLds<BW>::kRowBytes;
    constexpr int TPL = BW >= kWave ? BW / kWave : 1;   // weight tasks per lane and gate
    extern __shared__ __align__(16) unsigned char core_smem[];
    unsigned char* sU = core_smem;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
    // the NS workgroups of a (rows, block) pair are neighbours in the grid: they start together
    const int part = (int)blockIdx.x % NS;
    const int pair = (int)blockIdx.x / NS;
    const int h = pair / ntiles;
    const int rt = pair - h * ntiles;
    const int c_first = part * CW;    // first of this workgroup's output columns within the block
    const bool computes = w < NT;
    __shared__ uint32_t s_arrival;           // this workgroup's place among the NS of its pair
    constexpr uint32_t kNotArrived = 0xffffffffu;
    if (NS > 1 && tid == 0) s_arrival = kNotArrived;   // visible after the barrier that ends the conv

    // This wave's slice of a weight matrix: thread -> (4 input channels, 8 consecutive output
    // columns).  Sixteen lanes take sixteen consecutive channel quads of one column octet (their
    // 8-byte LDS writes then cover every bank once), the next sixteen the next octet of the same
    // rows, so that one load instruction touches 16 rows of 64 contiguous bytes and every
    // cache line is asked for by one instruction only.
    constexpr int KQN = BW / 4 < 16 ? BW / 4 : 16;
    WeightQuad<WT> raw[TPL];
    auto fetch_weights = [&](const WT* wsel) {
#pragma unroll
        for (int q = 0; q < TPL; ++q) {
            const int task = lane + q * kWave;
            const int tkq = task % KQN + KQN * (task / (4 * KQN)), tn8 = ((task / KQN) % 4) * 8;
            if (task < BW) raw[q].load(wsel + ((size_t)h * BW + 4 * tkq) * BW + c_first + w * 32 + tn8, BW);
            else raw[q].clear();
        }
    };
    unsigned char* sW = core_smem + CoreLds<BW>::kUBytes + (computes ? w : 0) * CoreLds<BW>::kWaveBytes;
    auto stage_weights = [&]() {
#pragma unroll
        for (int q = 0; q < TPL; ++q) {
            const int task = lane + q * kWave;
            const int tkq = task % KQN + KQN * (task / (4 * KQN)), tn8 = ((task / KQN) % 4) * 8;
            if (task < BW) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    *reinterpret_cast<u32x2*>(sW + (tn8 + e) * kRowBytes + tkq * 8) = raw[q].column(e);
            }
        }
    };
    if (computes) fetch_weights(w_i);

    // Everything the later steps read from memory and whose address is known now is asked for
    // now, so that the kernel pays one memory round trip and not one per step: the recurrence's
    // y and state rows (step 4), the biases of this wave's columns (step 3) and Lambda (step 2).
    // (Not with fp32 weights: their raw rows fill the register file, and these would spill.)
    constexpr bool kEarly = sizeof(WT) == 2;
    typedef typename Raw<ST, 8>::type sraw8_t;
    constexpr int kRecCH = CW / 8;
    constexpr int kRecPerThread = (kTileRows * kRecCH + kCoreWaves * kWave - 1) / (kCoreWaves * kWave);
    u32x4 early_y[kRecPerThread];
    sraw8_t early_s[kRecPerThread];
    if (kEarly && vec_io) {
#pragma unroll
        for (int q = 0; q < kRecPerThread; ++q) {
            const int task = min(tid + q * kCoreWaves * kWave, kTileRows * kRecCH - 1);
            const int rl = task / kRecCH, ch = c_first / 8 + (task - rl * kRecCH);
            const int row = min(rt * kTileRows + rl, M - 1);
            const int c = h * BW + ch * 8;
            early_y[q] = load_raw<bf16_t, 8>(y + (size_t)row * ldy + c);
            early_s[q] = load_raw<ST, 8>(state + (size_t)row * D + c);
        }
    }
    float early_bias_i = 0.0f, early_bias_a = 0.0f;
    if (computes) {
        const int c_out = h * BW + c_first + w * 32 + (lane & 31);
        if (b_i != nullptr) early_bias_i = b_i[c_out];
        if (b_a != nullptr) early_bias_a = b_a[c_out];
    }
    const float early_lam = tid < BW ? lam[h * BW + tid] : 0.0f;

    // ---- 1. conv window roll + conv: 16-byte chunks of 8 channels
    {
        constexpr int CH = BW / 8;
        const int H = W - 1;
        for (int task = tid; task < kTileRows * CH; task += kCoreWaves * kWave) {
            const int rl = task / CH, ch = task - rl * CH;
            const int row = rt * kTileRows + rl;
            const int c = h * BW + ch * 8;
            u32x4 ubits = {0u, 0u, 0u, 0u};
            if (row < M) {
                bf16_t* sb = conv_state + (size_t)row * H * D + c;
                // every load of the task is issued before the first of them is used
                u32x4 win[kCoreMaxW - 1];
                f32x4 cw[kCoreMaxW][2];
#pragma unroll
                for (int j = 0; j < kCoreMaxW - 1; ++j) {
                    if (j < H) win[j] = *reinterpret_cast<const u32x4*>(sb + (size_t)j * D);
                }
                const u32x4 newest = *reinterpret_cast<const u32x4*>(x_new + (size_t)row * ldx + c);
#pragma unroll
                for (int j = 0; j < kCoreMaxW; ++j) {
                    if (j <= H) {
                        cw[j][0] = *reinterpret_cast<const f32x4*>(conv_w + (size_t)j * D + c);
                        cw[j][1] = *reinterpret_cast<const f32x4*>(conv_w + (size_t)j * D + c + 4);
                    }
                }
                const f32x4 cb0 = *reinterpret_cast<const f32x4*>(conv_b + c);
                const f32x4 cb1 = *reinterpret_cast<const f32x4*>(conv_b + c + 4);
                float acc[8], xv[8];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    acc[v] = cb0[v];
                    acc[4 + v] = cb1[v];
                }
#pragma unroll
                for (int j = 0; j < kCoreMaxW - 1; ++j) {
                    if (j < H) {
                        unpack(win[j], xv);
#pragma unroll
                        for (int v = 0; v < 8; ++v) acc[v] = fmaf(cw[j][v / 4][v % 4], xv[v], acc[v]);
                    }
                }
                unpack(newest, xv);
                {
                    f32x4 last0 = cw[0][0], last1 = cw[0][1];   // row H of the weights
#pragma unroll
                    for (int j = 1; j < kCoreMaxW; ++j) {
                        if (j == H) {
                            last0 = cw[j][0];
                            last1 = cw[j][1];
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        acc[v] = fmaf(last0[v], xv[v], acc[v]);
                        acc[4 + v] = fmaf(last1[v], xv[4 + v], acc[4 + v]);
                    }
                }
                pack(acc, ubits);
                if constexpr (NS == 1) {   // the only reader of these rows rolls them on the spot
#pragma unroll
                    for (int j = 0; j < kCoreMaxW - 1; ++j) {
                        if (j + 1 < H) *reinterpret_cast<u32x4*>(sb + (size_t)j * D) = win[j + 1];
                    }
                    if (H > 0) *reinterpret_cast<u32x4*>(sb + (size_t)(H - 1) * D) = newest;
                }
            }
            *reinterpret_cast<u32x4*>(sU + rl * kRowBytes + ch * 16) = ubits;
        }
    }

    // ---- 2. gate projections of this wave's 32 output columns
    const int col = lane & 31, khalf = 8 * (lane >> 5);
    // softplus(Lambda) of the block's channels, once per workgroup
    float* sSp = reinterpret_cast<float*>(core_smem + CoreLds<BW>::kBytes);
    if (tid < BW) sSp[tid] = softplus_precise(early_lam);
    if (computes) {
        stage_weights();
        fetch_weights(w_a);
    }
    wave_lds_fence();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (NS > 1) {
        // Every thread's window loads have returned (their values went to LDS before the
        // barrier): this workgroup no longer reads the window.  The waves without matrix products
        // count it in, and in the workgroup that counts in last, when no reader is left anywhere,
        // they roll the window while the other waves multiply.  They ask for the rows before they
        // know the count, so that the loads travel together with the counter's round trip.
        if (!computes && W > 1) {
            constexpr int CH = BW / 8;
            constexpr int kIdle = (kCoreWaves - NT) * kWave;
            const int H = W - 1;
            const int itid = tid - NT * kWave;
            if (itid == 0) {
                const uint32_t a = __hip_atomic_fetch_add(counters + pair, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(&s_arrival, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            // all of a thread's rows are asked for at once (one round trip, not one per task)
            constexpr int kPerThread = (kTileRows * CH + kIdle - 1) / kIdle;
            u32x4 win[kPerThread][kCoreMaxW - 1], newest[kPerThread];
#pragma unroll
            for (int q = 0; q < kPerThread; ++q) {
                const int task = min(itid + q * kIdle, kTileRows * CH - 1);
                const int rl = task / CH, ch = task - rl * CH;
                const int row = min(rt * kTileRows + rl, M - 1);
                const int c = h * BW + ch * 8;
                const bf16_t* sb = conv_state + (size_t)row * H * D + c;
#pragma unroll
                for (int j = 1; j < kCoreMaxW - 1; ++j) {
                    if (j < H) win[q][j] = *reinterpret_cast<const u32x4*>(sb + (size_t)j * D);
                }
                newest[q] = *reinterpret_cast<const u32x4*>(x_new + (size_t)row * ldx + c);
            }
            uint32_t arrived = kNotArrived;
            while (arrived == kNotArrived) {
                arrived = __hip_atomic_load(&s_arrival, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                if (arrived == kNotArrived) __builtin_amdgcn_s_sleep(1);
            }
            if (arrived == (uint32_t)(NS - 1)) {
#pragma unroll
                for (int q = 0; q < kPerThread; ++q) {
                    const int task = itid + q * kIdle;
                    const int rl = task / CH, ch = task - rl * CH;
                    const int row = rt * kTileRows + rl;
                    if (task < kTileRows * CH && row < M) {
                        bf16_t* sb = conv_state + (size_t)row * H * D + h * BW + ch * 8;
#pragma unroll
                        for (int j = 0; j < kCoreMaxW - 1; ++j) {
                            if (j + 1 < H) *reinterpret_cast<u32x4*>(sb + (size_t)j * D) = win[q][j + 1];
                        }
                        *reinterpret_cast<u32x4*>(sb + (size_t)(H - 1) * D) = newest[q];
                    }
                }
            }
            // every part has counted in: the counter can go back to zero for the next launch
            if (itid == 0 && arrived == (uint32_t)(NS - 1))
                __hip_atomic_store(counters + pair, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    f32x16 acc_i = {}, acc_a = {};
    if (computes) {
        const unsigned char* asrc = sU + col * kRowBytes + khalf * 2;
        const unsigned char* bsrc = sW + col * kRowBytes + khalf * 2;
#pragma unroll
        for (int s = 0; s < KS; ++s)
            acc_i = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(asrc + 32 * s),
                                                            *reinterpret_cast<const bf16x8*>(bsrc + 32 * s), acc_i, 0, 0,
                                                            0);
        wave_lds_fence();   // the first gate's operands have been read: the region can be overwritten
        stage_weights();
        wave_lds_fence();
#pragma unroll
        for (int s = 0; s < KS; ++s)
            acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(asrc + 32 * s),
                                                            *reinterpret_cast<const bf16x8*>(bsrc + 32 * s), acc_a, 0, 0,
                                                            0);
    }

    // ---- 3. the logits (biases added, rounded to bf16) go to LDS over the weights, which every
    //         wave has finished with, so that the recurrence can run on all threads with 16-byte
    //         accesses: thread -> (row, 8 consecutive channels), as in the conv
    constexpr int kORowBytes = CoreLds<BW>::kORowBytes;
    unsigned char* sO = core_smem + CoreLds<BW>::kUBytes;
    wave_lds_fence();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (computes) {
        const float bias_i = early_bias_i, bias_a = early_bias_a;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int rl = 4 * (lane >> 5) + 8 * (r / 4) + (r % 4);
            unsigned char* o = sO + rl * kORowBytes + (c_first + w * 32 + col) * 2;
            *reinterpret_cast<uint16_t*>(o) = to_bf16_bits(acc_i[r] + bias_i);
            *reinterpret_cast<uint16_t*>(o + BW * 2) = to_bf16_bits(acc_a[r] + bias_a);
        }
    }
    wave_lds_fence();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // ---- 4. recurrence and output gate
    {
        constexpr int CH = CW / 8;
#pragma unroll
        for (int q = 0; q < kRecPerThread; ++q) {
            const int task = tid + q * kCoreWaves * kWave;
            if (task >= kTileRows * CH) break;
            const int rl = task / CH, ch = c_first / 8 + (task - rl * CH);
            const int row = rt * kTileRows + rl;
            if (row >= M) continue;
            const int c = h * BW + ch * 8;
            float u[8], xg[8], ag[8], fy[8], so[8], hn[8], go[8];
            unpack(*reinterpret_cast<const u32x4*>(sU + rl * kRowBytes + ch * 16), u);
            unpack(*reinterpret_cast<const u32x4*>(sO + rl * kORowBytes + ch * 16), xg);
            unpack(*reinterpret_cast<const u32x4*>(sO + rl * kORowBytes + BW * 2 + ch * 16), ag);
            const bf16_t* yp = y + (size_t)row * ldy + c;
            ST* sp = state + (size_t)row * D + c;
            bf16_t* op = out + (size_t)row * D + c;
            if (kEarly && vec_io) {
                unpack(early_y[q], fy);
                unpack(early_s[q], so);
            } else if (vec_io) {
                unpack(load_raw<bf16_t, 8>(yp), fy);
                unpack(load_raw<ST, 8>(sp), so);
            } else {
#pragma unroll
                for (int v = 0; v < 8; ++v) {
                    float t1[1], t2[1];
                    unpack(load_raw<bf16_t, 1>(yp + v), t1);
                    unpack(load_raw<ST, 1>(sp + v), t2);
                    fy[v] = t1[0];
                    so[v] = t2[0];
                }
            }
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                hn[v] = rglru_step_value(u[v], xg[v], ag[v], sSp[ch * 8 + v], so[v]);
                go[v] = gelu_times(fy[v], hn[v]);
            }
            if (vec_io) {
                sraw8_t rs;
                u32x4 ro;
                pack(hn, rs);
                pack(go, ro);
                *reinterpret_cast<sraw8_t*>(sp) = rs;
                *reinterpret_cast<u32x4*>(op) = ro;
            } else {
#pragma unroll
                for (int v = 0; v < 8; ++v) {
                    const float h1[1] = {hn[v]};
                    typename Raw<ST, 1>::type r1;
                    pack(h1, r1);
                    *reinterpret_cast<typename Raw<ST, 1>::type*>(sp + v) = r1;
                    *reinterpret_cast<uint16_t*>(op + v) = to_bf16_bits(go[v]);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Input gradient of the two projections:
//   dx[m, h*bw + i] = sum_j dxg[m, h*bw + j] w_i[h, i, j] + sum_j dag[m, h*bw + j] w_a[h, i, j]
//                     (+ addend[m, h*bw + i], the gradient x receives from its other consumers)
// Same decomposition as the forward: wave (g, c) keeps w_g[h, 32c.., :] (rows of the weight
// matrix, contiguous in memory) as B operands, reads gate g's gradient tile from LDS as A
// operands, and the two gates' partial tiles are added on the way out.
// ---------------------------------------------------------------------------------------
template <typename GT, typename WT, typename DT, int BW, bool ADD>
__global__ __launch_bounds__(kGateThreads, 1) void gate_proj_bwd_input_kernel(
    const GT* __restrict__ dxg, const GT* __restrict__ dag, const WT* __restrict__ w_i, const WT* __restrict__ w_a,
    const DT* __restrict__ addend, DT* __restrict__ dx, int M, int D, int nb, int ntiles) {
    constexpr int KS = BW / 16;
    constexpr int G = kGroup / BW;
    constexpr int kORowBytes = kGroup * 4 + 16;             // fp32 partial sums of one gate, one row
    constexpr int kOTileBytes = kTileRows * kORowBytes;
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* sA = smem;                               // [stage][gate] gradient tiles
    unsigned char* sO = smem + 4 * kATileBytes;             // [gate] partial result tiles

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int group = blockIdx.y, worker = blockIdx.x, nworkers = gridDim.x;
    const int g = w >> 3, c = w & 7;
    const int blk = (32 * c) / BW;
    const int h = group * G + blk;
    const int col = lane & 31, khalf = 8 * (lane >> 5);
    const int i_in = 32 * c - blk * BW + col;               // input channel within the block
    const WT* wsel = g ? w_a : w_i;

    const int lrow = tid >> 5, lc8 = tid & 31;
    const int lcol = group * kGroup + lc8 * 8;
    const bool col_ok = lcol < D;
    const uint32_t g_row_bytes = (uint32_t)D * (uint32_t)sizeof(GT);
    const uint32_t g_off = col_ok ? (uint32_t)(lrow * D + lcol) * (uint32_t)sizeof(GT) : 0x80000000u;
    auto load_tile = [&](int it, Row8<GT>& r0, Row8<GT>& r1) {
        const int t = min(worker + it * nworkers, ntiles);   // past the last tile: an empty window
        const int row0 = min(t * kTileRows, M);
        const uint32_t window = (uint32_t)min(M - row0, kTileRows) * g_row_bytes;
        r0.load_buf(make_rsrc(dxg + (size_t)row0 * D, window), g_off);
        r1.load_buf(make_rsrc(dag + (size_t)row0 * D, window), g_off);
    };
    auto stage_tile = [&](int buf, const Row8<GT>& r0, const Row8<GT>& r1) {
        unsigned char* p = sA + (2 * buf) * kATileBytes + lrow * kARowBytes + lc8 * 16;
        *reinterpret_cast<u32x4*>(p) = r0.as_bf16();
        *reinterpret_cast<u32x4*>(p + kATileBytes) = r1.as_bf16();
    };

    Row8<GT> ra0, ra1, rb0, rb1;
    load_tile(0, ra0, ra1);
    load_tile(1, rb0, rb1);
    __builtin_amdgcn_sched_barrier(0);

    // weights: lane holds row i of w_g[h] and 8 consecutive j per k-step (contiguous)
    const float live = (h < nb) ? 1.0f : 0.0f;
    const rsrc_t wres = make_rsrc(wsel, (uint32_t)((size_t)nb * BW * BW * sizeof(WT)));
    const uint32_t wlane = (uint32_t)((((size_t)min(h, nb - 1) * BW + i_in) * BW + khalf) * sizeof(WT));
    bf16x8 bfrag[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        bfrag[s] = load_weight8(wres, wlane, (uint32_t)(16 * s * sizeof(WT)), live, static_cast<const WT*>(nullptr));
        if (s % 4 == 3) __builtin_amdgcn_sched_barrier(0);
    }

    stage_tile(0, ra0, ra1);
    load_tile(2, ra0, ra1);
    __syncthreads();

    const int a_off = g * kATileBytes + col * kARowBytes + (blk * BW + khalf) * 2;
    unsigned char* o_base = sO + g * kOTileBytes + (4 * (lane >> 5)) * kORowBytes + (32 * c + col) * 4;
    const unsigned char* o_src = sO + lrow * kORowBytes + lc8 * 32;

    auto step = [&](int it, int cur, Row8<GT>& rn0, Row8<GT>& rn1) {
        // the addend's piece of this tile is asked for now and used after the tile's arithmetic
        const int row = (worker + it * nworkers) * kTileRows + lrow;
        const bool out_ok = col_ok && row < M;
        Row8<DT> radd;
        if constexpr (ADD) {
            const int arow0 = min((worker + it * nworkers) * kTileRows, M);
            const uint32_t a_row_bytes = (uint32_t)D * (uint32_t)sizeof(DT);
            radd.load_buf(make_rsrc(addend + (size_t)arow0 * D, (uint32_t)min(M - arow0, kTileRows) * a_row_bytes),
                          col_ok ? (uint32_t)(lrow * D + lcol) * (uint32_t)sizeof(DT) : 0x80000000u);
        }
        f32x16 acc = {};
        const unsigned char* a_base = sA + (2 * cur) * kATileBytes + a_off;
        constexpr int kBatch = KS < 4 ? KS : 4;
#pragma unroll
        for (int s0 = 0; s0 < KS; s0 += kBatch) {
            bf16x8 a[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) a[j] = *reinterpret_cast<const bf16x8*>(a_base + (s0 + j) * 32);
#pragma unroll
            for (int j = 0; j < kBatch; ++j)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[j], bfrag[s0 + j], acc, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = 8 * (r / 4) + (r % 4);
            *reinterpret_cast<float*>(o_base + m * kORowBytes) = acc[r];
        }
        stage_tile(cur ^ 1, rn0, rn1);
        load_tile(it + 3, rn0, rn1);
        __syncthreads();
        if (out_ok) {
            const f32x4 p0 = *reinterpret_cast<const f32x4*>(o_src), p1 = *reinterpret_cast<const f32x4*>(o_src + 16);
            const f32x4 q0 = *reinterpret_cast<const f32x4*>(o_src + kOTileBytes);
            const f32x4 q1 = *reinterpret_cast<const f32x4*>(o_src + kOTileBytes + 16);
            f32x4 s0 = p0 + q0, s1 = p1 + q1;
            if constexpr (ADD) {
                f32x4 e0, e1;
                radd.as_f32(e0, e1);
                s0 += e0;
                s1 += e1;
            }
            DT* dst = dx + (size_t)row * D + lcol;
            if constexpr (sizeof(DT) == 4) {
                __builtin_nontemporal_store(s0, reinterpret_cast<f32x4*>(dst));
                __builtin_nontemporal_store(s1, reinterpret_cast<f32x4*>(dst) + 1);
            } else {
                const u32x4 packed = {pack_bf16x2(s0.x, s0.y), pack_bf16x2(s0.z, s0.w), pack_bf16x2(s1.x, s1.y),
                                      pack_bf16x2(s1.z, s1.w)};
                __builtin_nontemporal_store(packed, reinterpret_cast<u32x4*>(dst));
            }
        }
        __syncthreads();
    };

    for (int it = 0; worker + it * nworkers < ntiles; it += 2) {
        step(it, 0, rb0, rb1);
        if (worker + (it + 1) * nworkers >= ntiles) break;
        step(it + 1, 1, ra0, ra1);
    }
}

// ---------------------------------------------------------------------------------------
// Weight and bias gradients:
//   dw_g[h, i, j] = sum_m x[m, h*bw + i] dg[m, h*bw + j],   db_g[c] = sum_m dg[m, c]
// The contraction runs over the rows, so both operands are needed "column-wise".  A
// workgroup (msplit, 256-channel group, gate) walks over its share of the row tiles (32 rows
// each, dealt round-robin to the splits);
// waves 0-7 fetch the x tile and waves 8-15 the gradient tile, each lane 8 rows of two
// adjacent channels, transpose them in registers and write them to LDS as
// [8-row chunk][channel][8 rows], which is exactly the 16 bytes an MFMA operand lane needs
// (bank-conflict free both ways).  Every wave accumulates up to 2 x 2 output tiles of
// 32 x 32 in registers over the whole row range and writes them to a per-split partial
// buffer; a second kernel adds the splits in a fixed order.
// ---------------------------------------------------------------------------------------
constexpr int kChunkBytes = kGroup * 16;          // one 8-row chunk of a transposed tile
constexpr int kTTileBytes = 4 * kChunkBytes;      // 32 rows

template <typename ET>
__device__ __forceinline__ uint32_t pair_as_bf16(const uint32_t (&raw)[2]) {
    if constexpr (sizeof(ET) == 2) return raw[0];
    return pack_bf16x2(__uint_as_float(raw[0]), __uint_as_float(raw[1]));
}

template <typename XT, typename GT, int BW>
__global__ __launch_bounds__(kGateThreads, 1) void gate_proj_bwd_weights_kernel(
    const XT* __restrict__ x, const GT* __restrict__ dg_i, const GT* __restrict__ dg_a, float* __restrict__ part_w,
    float* __restrict__ part_b, int M, int D, int nb) {
    constexpr int G = kGroup / BW;                 // blocks per group
    constexpr int NT = BW / 32;                    // 32-wide tiles per block side
    constexpr int TI = BW >= 256 ? 2 : 1;          // output tiles per wave: TI x TJ
    constexpr int TJ = BW >= 128 ? 2 : 1;
    constexpr int WPB = (NT * NT) / (TI * TJ);     // waves per block
    constexpr int RAWW = (sizeof(XT) > 2 || sizeof(GT) > 2) ? 2 : 1;
    __shared__ __align__(16) unsigned char sT[2][2][kTTileBytes];   // [stage][x | dg][chunk][channel][8 rows]
    __shared__ float s_db[4][kGroup];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int split = blockIdx.x, group = blockIdx.y, gate = blockIdx.z;
    const GT* dg = gate ? dg_a : dg_i;
    // Row tiles are dealt out round-robin: split s takes tiles s, s + nsplit, ...  All workgroups
    // of the launch then read neighbouring rows at any moment, three sequential streams (x and
    // the two gradients) instead of three per split; memory serves few streams faster.
    const int nsplit = gridDim.x;
    const int all_tiles = (M + kTileRows - 1) / kTileRows;
    const int ntiles = split < all_tiles ? (all_tiles - split + nsplit - 1) / nsplit : 0;

    // ---- loader role: 8 rows x 2 channels per lane
    const bool loads_x = w < 8;
    const int q = (w & 7) >> 1;                                  // 8-row chunk of the tile
    const int c2 = (w & 1) * 64 + lane;                          // channel pair within the group
    const int lch = group * kGroup + 2 * c2;
    const bool ch_ok = lch < D;
    // Register sets that hold tiles on their way from memory: tile k lands in set k % kSets and is
    // staged into LDS kSets - 1 steps after its loads were issued.  A step lasts well under a
    // microsecond and a load under traffic takes several, so the depth of this ring, not the
    // arithmetic, sets the pace of the loop.
    constexpr int kSets = (RAWW == 1) ? HAWK_GATE_DW_SETS : (HAWK_GATE_DW_SETS / 4 >= 1 ? (HAWK_GATE_DW_SETS / 4) * 2 : 2);
    static_assert(kSets >= 2 && kSets % 2 == 0, "an even number of register sets");
    uint32_t rs[kSets][8][RAWW];
    // Loads go through a buffer resource that covers the rows of the tile which exist: rows past
    // M, tiles past the last one and the channels past D of the last group read as zeros without a
    // branch, so the loop body is straight-line code and the compiler can wait for exactly the
    // loads a step needs while younger ones stay in flight.
    constexpr bool kSameWidth = sizeof(XT) == sizeof(GT);
    const char* src = loads_x ? reinterpret_cast<const char*>(x) : reinterpret_cast<const char*>(dg);
    const uint32_t esz = loads_x ? (uint32_t)sizeof(XT) : (uint32_t)sizeof(GT);
    const uint32_t row_bytes = (uint32_t)D * esz;
    const uint32_t lane_bytes = ch_ok ? (uint32_t)lch * esz : 0x80000000u;
    auto load_rows = [&](int t, uint32_t (&r)[8][RAWW]) {
        const int row0 = min((split + t * nsplit) * kTileRows + 8 * q, M);
        const int rows = (t < ntiles) ? min(M - row0, 8) : 0;
        const rsrc_t rs_ = make_rsrc(src + (size_t)row0 * row_bytes, (uint32_t)rows * row_bytes);
        auto narrow = [&](int k) {
            r[k][0] = __builtin_amdgcn_raw_buffer_load_b32(rs_, lane_bytes, k * row_bytes, kAuxDefault);
            if (RAWW > 1) r[k][RAWW - 1] = 0u;
        };
        auto wide = [&](int k) {
            const u32x2 v = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rs_, lane_bytes, k * row_bytes,
                                                                                           kAuxDefault));
            r[k][0] = v.x;
            r[k][RAWW - 1] = v.y;
        };
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            if constexpr (kSameWidth) {
                if constexpr (sizeof(XT) == 2) narrow(k);
                else wide(k);
            } else if ((sizeof(XT) == 2) == loads_x) {   // the two roles differ in width: a wave-uniform branch
                narrow(k);
            } else {
                wide(k);
            }
        }
    };
    float colsum[2] = {0.0f, 0.0f};
    auto stage_rows = [&](int buf, const uint32_t (&r)[8][RAWW]) {
        uint32_t d[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            uint32_t tmp[2] = {r[k][0], RAWW > 1 ? r[k][RAWW - 1] : 0u};
            if constexpr (sizeof(XT) == sizeof(GT)) d[k] = pair_as_bf16<XT>(tmp);
            else d[k] = loads_x ? pair_as_bf16<XT>(tmp) : pair_as_bf16<GT>(tmp);
        }
        // column sums of the gradient tile, for the bias gradient (the x loaders add up x's
        // columns too, which nobody reads: cheaper than a branch in the tile loop)
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            colsum[0] += bf16_lo(d[k]);
            colsum[1] += bf16_hi(d[k]);
        }
        // channel 2 c2 takes the low halves, channel 2 c2 + 1 the high halves; rows in order
        u32x4 lo, hi;
        lo.x = __builtin_amdgcn_perm(d[1], d[0], 0x05040100u);
        lo.y = __builtin_amdgcn_perm(d[3], d[2], 0x05040100u);
        lo.z = __builtin_amdgcn_perm(d[5], d[4], 0x05040100u);
        lo.w = __builtin_amdgcn_perm(d[7], d[6], 0x05040100u);
        hi.x = __builtin_amdgcn_perm(d[1], d[0], 0x07060302u);
        hi.y = __builtin_amdgcn_perm(d[3], d[2], 0x07060302u);
        hi.z = __builtin_amdgcn_perm(d[5], d[4], 0x07060302u);
        hi.w = __builtin_amdgcn_perm(d[7], d[6], 0x07060302u);
        unsigned char* p = &sT[buf][loads_x ? 0 : 1][q * kChunkBytes + (2 * c2) * 16];
        *reinterpret_cast<u32x4*>(p) = lo;
        *reinterpret_cast<u32x4*>(p + 16) = hi;
    };

    // ---- compute role: TI x TJ output tiles of block `blk`
    const int blk_raw = w / WPB;                   // block within the group (idle if >= G)
    const int wi = w % WPB;
    const int i0 = (wi / (NT / TJ)) * TI, j0 = (wi % (NT / TJ)) * TJ;
    const int h = group * G + blk_raw;
    const bool computes = blk_raw < G && h < nb;
    // waves without a block of their own run the same instruction stream on block 0 (their sums
    // are dropped), so that the tile loop has no branch and the matrix products of a tile can be
    // interleaved with the staging of the next one
    const int blk = computes ? blk_raw : 0;
    const int col = lane & 31;
    const int a_off = (lane >> 5) * kChunkBytes + (blk * BW + i0 * 32 + col) * 16;
    const int b_off = (lane >> 5) * kChunkBytes + (blk * BW + j0 * 32 + col) * 16;
    f32x16 acc[TI][TJ];
#pragma unroll
    for (int a = 0; a < TI; ++a)
#pragma unroll
        for (int b = 0; b < TJ; ++b) acc[a][b] = f32x16{};

#pragma unroll
    for (int k = 0; k < kSets; ++k) load_rows(k, rs[k]);
    stage_rows(0, rs[0]);
    load_rows(kSets, rs[0]);
    __syncthreads();

    auto step = [&](int t, int cur, uint32_t (&rnext)[8][RAWW]) {
        {
            bf16x8 fa[2][TI], fb[2][TJ];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
                for (int a = 0; a < TI; ++a)
                    fa[ks][a] = *reinterpret_cast<const bf16x8*>(&sT[cur][0][2 * ks * kChunkBytes + a_off + a * 32 * 16]);
#pragma unroll
                for (int b = 0; b < TJ; ++b)
                    fb[ks][b] = *reinterpret_cast<const bf16x8*>(&sT[cur][1][2 * ks * kChunkBytes + b_off + b * 32 * 16]);
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int a = 0; a < TI; ++a)
#pragma unroll
                    for (int b = 0; b < TJ; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks][a], fb[ks][b], acc[a][b], 0, 0, 0);
        }
        // tile t + 1 into the other LDS stage, tile t + 1 + kSets into the registers it leaves
        stage_rows(cur ^ 1, rnext);
        load_rows(t + 1 + kSets, rnext);
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += kSets) {
#pragma unroll
        for (int k = 0; k < kSets; ++k) {
            if (t + k < ntiles) step(t + k, k & 1, rs[(k + 1) % kSets]);
        }
    }

    // ---- partial results of this split
    if (computes) {
        float* dst = part_w + (((size_t)split * 2 + gate) * nb + h) * BW * BW;
#pragma unroll
        for (int a = 0; a < TI; ++a)
#pragma unroll
            for (int b = 0; b < TJ; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int i = (i0 + a) * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
                    const int j = (j0 + b) * 32 + col;
                    dst[(size_t)i * BW + j] = acc[a][b][r];
                }
    }
    if (!loads_x) {
        s_db[q][2 * c2] = colsum[0];
        s_db[q][2 * c2 + 1] = colsum[1];
    }
    __syncthreads();
    if (tid < kGroup && group * kGroup + tid < D)
        part_b[((size_t)split * 2 + gate) * D + group * kGroup + tid] =
            (s_db[0][tid] + s_db[1][tid]) + (s_db[2][tid] + s_db[3][tid]);
}

// dw_g = sum over splits of the partial tiles, db_g likewise; fixed order.
__global__ void gate_proj_reduce_kernel(GateReduceTask t) {
    gate_reduce_span(t, (size_t)blockIdx.x * blockDim.x + threadIdx.x, (size_t)gridDim.x * blockDim.x);
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Compute units of the current device (asked once per device): the persistent kernels launch one
// workgroup per compute unit, and the size of the weight-gradient workspace follows from it.
int num_cu() {
    static std::atomic<int> cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return kDefaultNumCU;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = kDefaultNumCU;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Raises a kernel's dynamic LDS limit once per device instead of on every launch.
template <auto Kernel>
bool allow_dynamic_lds(size_t bytes) {
    static std::atomic<unsigned long long> done{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)bytes) != hipSuccess)
        return false;
    done.fetch_or(bit, std::memory_order_release);
    return true;
}

template <typename XT, typename WT, typename OT, int BW>
int launch_gate_fwd(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* out_i,
                    void* out_a, int M, int D, int nb, hipStream_t st) {
    const int ngroups = ceil_div(D, kGroup);
    const int ntiles = ceil_div(M, kTileRows);
    if (M <= HAWK_GATE_SMALL_M) {
        // enough workgroups to give every compute unit a few waves; each wave keeps its weights
        // for all the row tiles it walks over
        const int ncolblocks = 2 * (D / 32);
        int rsplit = ceil_div(8 * num_cu(), ncolblocks * kSmallWaves);
        const int max_split = ceil_div(ntiles, kSmallWaves);
        if (rsplit > max_split) rsplit = max_split;
        hipLaunchKernelGGL((gate_proj_fwd_small_kernel<XT, WT, OT, BW>), dim3((unsigned)ncolblocks, (unsigned)rsplit),
                           dim3(kSmallWaves * kWave), 0, st, static_cast<const XT*>(x), static_cast<const WT*>(w_i),
                           b_i, static_cast<const WT*>(w_a), b_a, static_cast<OT*>(out_i), static_cast<OT*>(out_a), M,
                           D, ntiles);
        return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
    }
    int nworkers = num_cu() / ngroups;
    if (nworkers < 1) nworkers = 1;
    if (nworkers > ntiles) nworkers = ntiles;
    size_t smem = gate_fwd_lds_bytes<OT>(false);
    if (smem < (size_t)WeightStage<BW>::kBytes) smem = WeightStage<BW>::kBytes;
    constexpr auto kernel = gate_proj_fwd_kernel<XT, WT, OT, BW, false>;
    if (!allow_dynamic_lds<kernel>(smem)) return HAWK_ERR_LAUNCH;
    hipLaunchKernelGGL(kernel, dim3((unsigned)nworkers, (unsigned)ngroups), dim3(kGateThreads), smem, st,
                       static_cast<const XT*>(x), static_cast<const WT*>(w_i), b_i, static_cast<const WT*>(w_a), b_a,
                       static_cast<OT*>(out_i), static_cast<OT*>(out_a), M, D, nb, ntiles, ConvFront{});
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

// The forward with the temporal conv in front (bf16 activations; the weight-transposition scratch
// of the prologue must stay clear of the conv taps at the end of the LDS block).
template <typename WT, int BW>
int launch_conv_gate_fwd(const void* x, long long ldx, const float* conv_w, const float* conv_b, const void* w_i,
                         const float* b_i, const void* w_a, const float* b_a, void* u, void* out_i, void* out_a,
                         int M, int T, int D, int nb, hipStream_t st) {
    const int ngroups = ceil_div(D, kGroup);
    const int ntiles = ceil_div(M, kTileRows);
    int nworkers = num_cu() / ngroups;
    if (nworkers < 1) nworkers = 1;
    if (nworkers > ntiles) nworkers = ntiles;
    constexpr size_t smem = gate_fwd_lds_bytes<bf16_t>(true);
    static_assert((size_t)WeightStage<BW>::kBytes <= smem - (kConvTaps + 1) * kGroup * sizeof(float), "LDS layout");
    constexpr auto kernel = gate_proj_fwd_kernel<bf16_t, WT, bf16_t, BW, true>;
    if (!allow_dynamic_lds<kernel>(smem)) return HAWK_ERR_LAUNCH;
    const ConvFront cf = {conv_w, conv_b, static_cast<bf16_t*>(u), T, ldx};
    hipLaunchKernelGGL(kernel, dim3((unsigned)nworkers, (unsigned)ngroups), dim3(kGateThreads), smem, st,
                       static_cast<const bf16_t*>(x), static_cast<const WT*>(w_i), b_i, static_cast<const WT*>(w_a),
                       b_a, static_cast<bf16_t*>(out_i), static_cast<bf16_t*>(out_a), M, D, nb, ntiles, cf);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename WT>
int conv_gate_fwd_bw(const void* x, long long ldx, const float* conv_w, const float* conv_b, const void* w_i,
                     const float* b_i, const void* w_a, const float* b_a, void* u, void* out_i, void* out_a, int M,
                     int T, int D, int nb, int bw, hipStream_t st) {
    switch (bw) {
        case 32: return launch_conv_gate_fwd<WT, 32>(x, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, u, out_i, out_a, M, T, D, nb, st);
        case 64: return launch_conv_gate_fwd<WT, 64>(x, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, u, out_i, out_a, M, T, D, nb, st);
        case 128: return launch_conv_gate_fwd<WT, 128>(x, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, u, out_i, out_a, M, T, D, nb, st);
        case 256: return launch_conv_gate_fwd<WT, 256>(x, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, u, out_i, out_a, M, T, D, nb, st);
        default: return HAWK_ERR_BAD_SHAPE;
    }
}

template <typename XT, typename WT, typename OT>
int gate_fwd_bw(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* out_i,
                void* out_a, int M, int D, int nb, int bw, hipStream_t st) {
    switch (bw) {
        case 32: return launch_gate_fwd<XT, WT, OT, 32>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, st);
        case 64: return launch_gate_fwd<XT, WT, OT, 64>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, st);
        case 128: return launch_gate_fwd<XT, WT, OT, 128>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, st);
        case 256: return launch_gate_fwd<XT, WT, OT, 256>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, st);
        default: return HAWK_ERR_BAD_SHAPE;
    }
}

template <typename XT, typename WT>
int gate_fwd_out(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* out_i,
                 void* out_a, int M, int D, int nb, int bw, int out_dtype, hipStream_t st) {
    if (out_dtype == HAWK_DTYPE_BF16)
        return gate_fwd_bw<XT, WT, bf16_t>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, bw, st);
    return gate_fwd_bw<XT, WT, float>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, bw, st);
}

template <typename GT, typename WT, typename DT, int BW>
int launch_gate_bwd_input(const void* dxg, const void* dag, const void* w_i, const void* w_a, const void* addend,
                          void* dx, int M, int D, int nb, hipStream_t st) {
    const int ngroups = ceil_div(D, kGroup);
    const int ntiles = ceil_div(M, kTileRows);
    int nworkers = num_cu() / ngroups;
    if (nworkers < 1) nworkers = 1;
    if (nworkers > ntiles) nworkers = ntiles;
    const size_t smem = 4 * kATileBytes + 2 * (size_t)kTileRows * (kGroup * 4 + 16);
    constexpr auto with_addend = gate_proj_bwd_input_kernel<GT, WT, DT, BW, true>;
    constexpr auto without = gate_proj_bwd_input_kernel<GT, WT, DT, BW, false>;
    if (!(addend != nullptr ? allow_dynamic_lds<with_addend>(smem) : allow_dynamic_lds<without>(smem)))
        return HAWK_ERR_LAUNCH;
    hipLaunchKernelGGL(addend != nullptr ? with_addend : without, dim3((unsigned)nworkers, (unsigned)ngroups),
                       dim3(kGateThreads), smem, st,
                       static_cast<const GT*>(dxg), static_cast<const GT*>(dag), static_cast<const WT*>(w_i),
                       static_cast<const WT*>(w_a), static_cast<const DT*>(addend), static_cast<DT*>(dx), M, D, nb,
                       ntiles);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename GT, typename WT, typename DT>
int gate_bwd_input_bw(const void* dxg, const void* dag, const void* w_i, const void* w_a, const void* addend,
                      void* dx, int M, int D, int nb, int bw, hipStream_t st) {
    switch (bw) {
        case 32: return launch_gate_bwd_input<GT, WT, DT, 32>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, st);
        case 64: return launch_gate_bwd_input<GT, WT, DT, 64>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, st);
        case 128: return launch_gate_bwd_input<GT, WT, DT, 128>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, st);
        case 256: return launch_gate_bwd_input<GT, WT, DT, 256>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, st);
        default: return HAWK_ERR_BAD_SHAPE;
    }
}

template <typename GT, typename WT>
int gate_bwd_input_out(const void* dxg, const void* dag, const void* w_i, const void* w_a, const void* addend,
                       void* dx, int M, int D, int nb, int bw, int dx_dtype, hipStream_t st) {
    if (dx_dtype == HAWK_DTYPE_BF16)
        return gate_bwd_input_bw<GT, WT, bf16_t>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, bw, st);
    return gate_bwd_input_bw<GT, WT, float>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, bw, st);
}

int weight_splits(int M, int D) {
    const int ngroups = ceil_div(D, kGroup);
    int n = num_cu() / (2 * ngroups);
    if (n < 1) n = 1;
    // at least HAWK_GATE_MIN_SPLIT_TILES row tiles per split: every split costs a pass over its
    // partial sums in the reduction
    const int cap = (ceil_div(M, kTileRows) + HAWK_GATE_MIN_SPLIT_TILES - 1) / HAWK_GATE_MIN_SPLIT_TILES;
    return n > cap ? cap : n;
}

template <typename XT, typename GT, int BW>
int launch_gate_bwd_weights(const void* x, const void* dg_i, const void* dg_a, float* part_w, float* part_b, int M,
                            int D, int nb, int nsplit, hipStream_t st) {
    hipLaunchKernelGGL((gate_proj_bwd_weights_kernel<XT, GT, BW>),
                       dim3((unsigned)nsplit, (unsigned)ceil_div(D, kGroup), 2u), dim3(kGateThreads), 0, st,
                       static_cast<const XT*>(x), static_cast<const GT*>(dg_i), static_cast<const GT*>(dg_a), part_w,
                       part_b, M, D, nb);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename XT, typename GT>
int gate_bwd_weights_bw(const void* x, const void* dg_i, const void* dg_a, float* part_w, float* part_b, int M, int D,
                        int nb, int bw, int nsplit, hipStream_t st) {
    switch (bw) {
        case 32: return launch_gate_bwd_weights<XT, GT, 32>(x, dg_i, dg_a, part_w, part_b, M, D, nb, nsplit, st);
        case 64: return launch_gate_bwd_weights<XT, GT, 64>(x, dg_i, dg_a, part_w, part_b, M, D, nb, nsplit, st);
        case 128: return launch_gate_bwd_weights<XT, GT, 128>(x, dg_i, dg_a, part_w, part_b, M, D, nb, nsplit, st);
        case 256: return launch_gate_bwd_weights<XT, GT, 256>(x, dg_i, dg_a, part_w, part_b, M, D, nb, nsplit, st);
        default: return HAWK_ERR_BAD_SHAPE;
    }
}

// Workgroups that share a block's output columns, when the caller brought counters for them.
// Each of them repeats the block's conv, so the cut pays only where fetching the weights is the
// larger part, at a block width of 256 (256 KiB per block; at 128 the cut was measured slower:
// 9.5 against 8.1 us at 256 rows), and only while the launch fits the device in one round:
// at 256 rows and 10 blocks two workgroups per block take 14.9 us against 18.7 for one and 21.8
// for four (320 workgroups); at 32 rows four take 10.3 against 17.6 us.
// (the grid is kept within one workgroup per compute unit of the device)
int num_cu();
inline int decode_core_parts(int pairs, int bw, bool have_counters) {
    if (!have_counters || bw < 256) return 1;
    const int max_grid = num_cu();
    if ((long long)pairs * 4 <= max_grid) return 4;
    if ((long long)pairs * 2 <= max_grid) return 2;
    return 1;
}

template <typename WT, typename ST, int BW, int NS, int WC>
int launch_decode_core_nsw(void* conv_state, const void* x_new, long long ldx, const float* conv_w, const float* conv_b,
                          const void* w_i, const float* b_i, const void* w_a, const float* b_a, const float* lam,
                          const void* y, long long ldy, void* state, void* out, int B, int D, int nb, int W,
                          uint32_t* counters, hipStream_t st) {
    const int ntiles = ceil_div(B, kTileRows);
    const long long grid = (long long)nb * ntiles * NS;
    if (grid > 0x7fffffffLL) return HAWK_ERR_BAD_SHAPE;
    constexpr auto kernel = decode_core_kernel<WT, ST, BW, NS, WC>;
    constexpr size_t smem = CoreLds<BW>::kBytes + BW * sizeof(float);   // + softplus(Lambda) of the block
    // 16-byte accesses to y, recc_state and out when their rows allow it
    const bool vec_io = (ldy % 8) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0 &&
                        (reinterpret_cast<uintptr_t>(state) & 31u) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    if (!allow_dynamic_lds<kernel>(smem)) return HAWK_ERR_LAUNCH;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kCoreWaves * kWave), smem, st,
                       static_cast<bf16_t*>(conv_state), static_cast<const bf16_t*>(x_new), (size_t)ldx, conv_w,
                       conv_b, static_cast<const WT*>(w_i), b_i, static_cast<const WT*>(w_a), b_a, lam,
                       static_cast<const bf16_t*>(y), (size_t)ldy, static_cast<ST*>(state), static_cast<bf16_t*>(out),
                       B, D, W, ntiles, vec_io, counters);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

template <typename WT, typename ST, int BW, int NS>
int launch_decode_core_ns(void* conv_state, const void* x_new, long long ldx, const float* conv_w, const float* conv_b,
                          const void* w_i, const float* b_i, const void* w_a, const float* b_a, const float* lam,
                          const void* y, long long ldy, void* state, void* out, int B, int D, int nb, int W,
                          uint32_t* counters, hipStream_t st) {
    if (W == 4)
        return launch_decode_core_nsw<WT, ST, BW, NS, 4>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam,
                                                         y, ldy, state, out, B, D, nb, W, counters, st);
    return launch_decode_core_nsw<WT, ST, BW, NS, 0>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y,
                                                     ldy, state, out, B, D, nb, W, counters, st);
}

template <typename WT, typename ST, int BW>
int launch_decode_core(void* conv_state, const void* x_new, long long ldx, const float* conv_w, const float* conv_b,
                       const void* w_i, const float* b_i, const void* w_a, const float* b_a, const float* lam,
                       const void* y, long long ldy, void* state, void* out, int B, int D, int nb, int W,
                       uint32_t* counters, hipStream_t st) {
    const int parts = decode_core_parts(nb * ceil_div(B, kTileRows), BW, counters != nullptr);
    if constexpr (BW >= 128) {
        if (parts == 4)
            return launch_decode_core_ns<WT, ST, BW, 4>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y,
                                                        ldy, state, out, B, D, nb, W, counters, st);
    }
    if constexpr (BW >= 64) {
        if (parts == 2)
            return launch_decode_core_ns<WT, ST, BW, 2>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y,
                                                        ldy, state, out, B, D, nb, W, counters, st);
    }
    return launch_decode_core_ns<WT, ST, BW, 1>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy,
                                                state, out, B, D, nb, W, nullptr, st);
}

template <typename WT, typename ST>
int decode_core_bw(void* conv_state, const void* x_new, long long ldx, const float* conv_w, const float* conv_b,
                   const void* w_i, const float* b_i, const void* w_a, const float* b_a, const float* lam,
                   const void* y, long long ldy, void* state, void* out, int B, int D, int nb, int W, uint32_t* counters,
                   hipStream_t st) {
    switch (D / nb) {
        case 32: return launch_decode_core<WT, ST, 32>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
        case 64: return launch_decode_core<WT, ST, 64>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
        case 128: return launch_decode_core<WT, ST, 128>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
        case 256: return launch_decode_core<WT, ST, 256>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
        default: return HAWK_ERR_BAD_SHAPE;
    }
}

}  // namespace

bool gate_proj_block_width_supported(int bw) { return bw == 32 || bw == 64 || bw == 128 || bw == 256; }

size_t decode_core_workspace_bytes(int B, int D, int nb) {
    (void)D;
    return (size_t)nb * ceil_div(B, kTileRows) * sizeof(uint32_t);
}

int decode_core_step(void* conv_state, const void* x_new, long long ldx, const float* conv_w, const float* conv_b,
                     const void* w_i, const float* b_i, const void* w_a, const float* b_a, const float* lam,
                     const void* y, long long ldy, void* state, void* out, int B, int D, int nb, int W, int w_dtype,
                     int state_dtype, void* workspace, size_t workspace_bytes, hipStream_t st) {
    // counters for cutting a block's columns over several workgroups, if the caller brought enough
    uint32_t* counters = (workspace != nullptr && workspace_bytes >= decode_core_workspace_bytes(B, D, nb))
                             ? static_cast<uint32_t*>(workspace)
                             : nullptr;
    if (w_dtype == HAWK_DTYPE_BF16) {
        if (state_dtype == HAWK_DTYPE_BF16)
            return decode_core_bw<bf16_t, bf16_t>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
        return decode_core_bw<bf16_t, float>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
    }
    if (state_dtype == HAWK_DTYPE_BF16)
        return decode_core_bw<float, bf16_t>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
    return decode_core_bw<float, float>(conv_state, x_new, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, lam, y, ldy, state, out, B, D, nb, W, counters, st);
}

int gate_proj_fwd(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* out_i,
                  void* out_a, int M, int D, int nb, int x_dtype, int w_dtype, int out_dtype, hipStream_t st) {
    const int bw = D / nb;
    if (x_dtype == HAWK_DTYPE_BF16) {
        if (w_dtype == HAWK_DTYPE_BF16)
            return gate_fwd_out<bf16_t, bf16_t>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, bw, out_dtype, st);
        return gate_fwd_out<bf16_t, float>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, bw, out_dtype, st);
    }
    if (w_dtype == HAWK_DTYPE_BF16)
        return gate_fwd_out<float, bf16_t>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, bw, out_dtype, st);
    return gate_fwd_out<float, float>(x, w_i, b_i, w_a, b_a, out_i, out_a, M, D, nb, bw, out_dtype, st);
}

int conv_gate_proj_fwd(const void* x, long long ldx, const float* conv_w, const float* conv_b, const void* w_i,
                       const float* b_i, const void* w_a, const float* b_a, void* u, void* out_i, void* out_a, int B,
                       int T, int D, int nb, int w_dtype, hipStream_t st) {
    const int bw = D / nb, M = B * T;
    if (w_dtype == HAWK_DTYPE_BF16)
        return conv_gate_fwd_bw<bf16_t>(x, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, u, out_i, out_a, M, T, D, nb, bw, st);
    return conv_gate_fwd_bw<float>(x, ldx, conv_w, conv_b, w_i, b_i, w_a, b_a, u, out_i, out_a, M, T, D, nb, bw, st);
}

int gate_proj_bwd_input(const void* dxg, const void* dag, const void* w_i, const void* w_a, const void* addend,
                        void* dx, int M, int D, int nb, int g_dtype, int w_dtype, int dx_dtype, hipStream_t st) {
    const int bw = D / nb;
    if (g_dtype == HAWK_DTYPE_BF16) {
        if (w_dtype == HAWK_DTYPE_BF16)
            return gate_bwd_input_out<bf16_t, bf16_t>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, bw, dx_dtype, st);
        return gate_bwd_input_out<bf16_t, float>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, bw, dx_dtype, st);
    }
    if (w_dtype == HAWK_DTYPE_BF16)
        return gate_bwd_input_out<float, bf16_t>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, bw, dx_dtype, st);
    return gate_bwd_input_out<float, float>(dxg, dag, w_i, w_a, addend, dx, M, D, nb, bw, dx_dtype, st);
}

size_t gate_proj_bwd_weights_workspace_bytes(int M, int D, int nb) {
    const size_t bw = (size_t)(D / nb);
    return (size_t)weight_splits(M, D) * 2 * ((size_t)nb * bw * bw + (size_t)D) * sizeof(float);
}

int gate_proj_bwd_weights(const void* x, const void* dg_i, const void* dg_a, float* dw_i, float* db_i, float* dw_a,
                          float* db_a, int M, int D, int nb, int x_dtype, int g_dtype, void* ws, size_t ws_bytes,
                          hipStream_t st, GateReduceTask* deferred) {
    const int bw = D / nb;
    const int nsplit = weight_splits(M, D);
    const size_t wcount = (size_t)nb * bw * bw;
    if (ws == nullptr || ws_bytes < gate_proj_bwd_weights_workspace_bytes(M, D, nb)) return HAWK_ERR_WORKSPACE;
    float* part_w = static_cast<float*>(ws);
    float* part_b = part_w + (size_t)nsplit * 2 * wcount;
    int rc;
    if (x_dtype == HAWK_DTYPE_BF16) {
        rc = g_dtype == HAWK_DTYPE_BF16
                 ? gate_bwd_weights_bw<bf16_t, bf16_t>(x, dg_i, dg_a, part_w, part_b, M, D, nb, bw, nsplit, st)
                 : gate_bwd_weights_bw<bf16_t, float>(x, dg_i, dg_a, part_w, part_b, M, D, nb, bw, nsplit, st);
    } else {
        rc = g_dtype == HAWK_DTYPE_BF16
                 ? gate_bwd_weights_bw<float, bf16_t>(x, dg_i, dg_a, part_w, part_b, M, D, nb, bw, nsplit, st)
                 : gate_bwd_weights_bw<float, float>(x, dg_i, dg_a, part_w, part_b, M, D, nb, bw, nsplit, st);
    }
    if (rc != HAWK_OK) return rc;
    const GateReduceTask reduce{part_w, part_b, dw_i, dw_a, db_i, db_a, nsplit, D, wcount};
    if (deferred != nullptr) {   // the caller runs it, together with its other closing reductions
        *deferred = reduce;
        return HAWK_OK;
    }
    size_t blocks = (reduce.items() + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(gate_proj_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, st, reduce);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace hawk

