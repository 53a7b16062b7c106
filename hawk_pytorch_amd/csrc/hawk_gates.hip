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
//     along rows (fp32 activations are rounded to bf16 on the way), is prefetched three
//     tiles ahead, and is read back as MFMA A operands by all 16 waves;
//   * results pass through LDS once more so that each row leaves in 512-byte (bf16) or
//     1-KiB (fp32) pieces.
// Per 32-row tile a CU moves 16 KiB in and 32 KiB out (bf16) against 16 waves x bw/16 MFMAs
// of 32x32x16; at bw = 256 that is about 2 k cycles of matrix-core time against about 5 k
// cycles of HBM time at 5 TB/s, so the kernel is bound by HBM.
#include "hawk_scan.h"

#include <stdint.h>

#include "hawk_device.h"

namespace hawk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kGroup = 256;                    // channels per workgroup
constexpr int kTileRows = 32;                  // rows per MFMA tile
constexpr int kGateThreads = 1024;             // 16 waves
constexpr int kARowBytes = kGroup * 2 + 16;    // bf16 row + pad: 8 lanes' 16-byte reads cover all banks
constexpr int kATileBytes = kTileRows * kARowBytes;
constexpr int kNumCU = 256;

__device__ __forceinline__ float elem_to_f32(float v) { return v; }
__device__ __forceinline__ float elem_to_f32(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }

// Eight consecutive activations as they sit in registers between the global load and the LDS store.
template <typename XT>
struct Row8;
template <>
struct Row8<bf16_t> {
    u32x4 v;
    __device__ __forceinline__ void load(const bf16_t* p, bool ok) {
        v = ok ? *reinterpret_cast<const u32x4*>(p) : u32x4{0u, 0u, 0u, 0u};
    }
    __device__ __forceinline__ u32x4 as_bf16() const { return v; }
};
template <>
struct Row8<float> {
    f32x4 lo, hi;
    __device__ __forceinline__ void load(const float* p, bool ok) {
        const f32x4 z = {0.0f, 0.0f, 0.0f, 0.0f};
        lo = ok ? *reinterpret_cast<const f32x4*>(p) : z;
        hi = ok ? *reinterpret_cast<const f32x4*>(p + 4) : z;
    }
    __device__ __forceinline__ u32x4 as_bf16() const {
        return u32x4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y),
                     pack_bf16x2(hi.z, hi.w)};
    }
};

__device__ __forceinline__ void store_out(unsigned char* p, float v, bf16_t*) {
    *reinterpret_cast<uint16_t*>(p) = to_bf16_bits(v);
}
__device__ __forceinline__ void store_out(unsigned char* p, float v, float*) { *reinterpret_cast<float*>(p) = v; }

template <typename XT, typename WT, typename OT, int BW>
__global__ __launch_bounds__(kGateThreads, 1) void gate_proj_fwd_kernel(
    const XT* __restrict__ x, const WT* __restrict__ w_i, const float* __restrict__ b_i,
    const WT* __restrict__ w_a, const float* __restrict__ b_a, OT* __restrict__ out_i, OT* __restrict__ out_a,
    int M, int D, int nb, int ntiles) {
    static_assert(BW == 32 || BW == 64 || BW == 128 || BW == 256, "block width");
    constexpr int KS = BW / 16;                                     // MFMA k-steps per output tile
    constexpr int G = kGroup / BW;                                  // whole blocks per workgroup
    constexpr int kORowBytes = 2 * kGroup * (int)sizeof(OT) + 16;   // both gates' columns of one row + pad
    extern __shared__ __align__(16) unsigned char smem[];
    unsigned char* sA = smem;                     // two activation tiles
    unsigned char* sO = smem + 2 * kATileBytes;   // one result tile

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int w = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int group = blockIdx.y, worker = blockIdx.x, nworkers = gridDim.x;

    // ---- this wave's slice of the weights, as MFMA B operands: lane holds output column
    //      (lane % 32) and 8 consecutive input channels starting at 16 s + 8 (lane / 32)
    const int g = w >> 3, c = w & 7;
    const int blk = (32 * c) / BW;                 // block within the group
    const int h = group * G + blk;                 // block of the layer
    const int col = lane & 31, khalf = 8 * (lane >> 5);
    const int n = 32 * c - blk * BW + col;         // output column within the block
    const WT* wsel = g ? w_a : w_i;
    const float* bsel = g ? b_a : b_i;
    const int ch = group * kGroup + 32 * c + col;  // channel of the layer
    const float bias = (bsel != nullptr && ch < D) ? bsel[ch] : 0.0f;

    // ---- tile traffic: thread -> (row, 8 consecutive channels)
    const int lrow = tid >> 5, lc8 = tid & 31;
    const int lcol = group * kGroup + lc8 * 8;
    const bool col_ok = lcol < D;
    auto load_tile = [&](int it, Row8<XT>& r) {
        const int t = worker + it * nworkers;
        const int row = t * kTileRows + lrow;
        const bool ok = col_ok && t < ntiles && row < M;
        r.load(x + (ok ? (size_t)row * D + lcol : 0), ok);
    };
    auto stage_tile = [&](int buf, const Row8<XT>& r) {
        *reinterpret_cast<u32x4*>(sA + buf * kATileBytes + lrow * kARowBytes + lc8 * 16) = r.as_bf16();
    };

    // Two register sets alternate as landing places for the prefetched tiles (tile it+1 is
    // staged into LDS during iteration it, and its registers are reloaded with tile it+3), and
    // the loop is unrolled by two so that buffers and registers are fixed per half.
    Row8<XT> ra, rb;
    load_tile(0, ra);
    load_tile(1, rb);
    __builtin_amdgcn_sched_barrier(0);  // the first tiles travel while the weights are fetched

    // ---- the weights: 8 strided loads per k-step and lane (coalesced across lanes), issued
    //      four k-steps at a time so that they fit the registers left beside their own
    //      destination; a group past the last block (D not a multiple of 256) reads block
    //      nb-1 and zeroes it
    const float live = (h < nb) ? 1.0f : 0.0f;
    const WT* wblk = wsel + ((size_t)min(h, nb - 1) * BW + khalf) * BW + n;
    bf16x8 bfrag[KS];
    constexpr int kWBatch = KS < 4 ? KS : 4;
#pragma unroll
    for (int s0 = 0; s0 < KS; s0 += kWBatch) {
        float v[kWBatch][8];
#pragma unroll
        for (int j = 0; j < kWBatch; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] = elem_to_f32(wblk[(size_t)(16 * (s0 + j) + e) * BW]);
#pragma unroll
        for (int j = 0; j < kWBatch; ++j) {
            const u32x4 packed = {pack_bf16x2(live * v[j][0], live * v[j][1]), pack_bf16x2(live * v[j][2], live * v[j][3]),
                                  pack_bf16x2(live * v[j][4], live * v[j][5]), pack_bf16x2(live * v[j][6], live * v[j][7])};
            bfrag[s0 + j] = __builtin_bit_cast(bf16x8, packed);
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    stage_tile(0, ra);
    load_tile(2, ra);
    __syncthreads();

    const int a_off = col * kARowBytes + (blk * BW + khalf) * 2;
    unsigned char* o_base = sO + (4 * (lane >> 5)) * kORowBytes + (g * kGroup + 32 * c + col) * (int)sizeof(OT);
    const unsigned char* o_src = sO + lrow * kORowBytes + lc8 * 8 * (int)sizeof(OT);

    auto step = [&](int it, int cur, Row8<XT>& rnext) {
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
            store_out(o_base + m * kORowBytes, acc[r] + bias, static_cast<OT*>(nullptr));
        }
        // tile it+1 into the other buffer, tile it+3 into the registers it leaves
        stage_tile(cur ^ 1, rnext);
        load_tile(it + 3, rnext);
        __syncthreads();
        const int row = (worker + it * nworkers) * kTileRows + lrow;
        if (col_ok && row < M) {
            constexpr int kVecs = (int)sizeof(OT) / 2;  // 16-byte pieces per 8 elements
            OT* dst_i = out_i + (size_t)row * D + lcol;
            OT* dst_a = out_a + (size_t)row * D + lcol;
#pragma unroll
            for (int q = 0; q < kVecs; ++q) {
                const u32x4 vi = *reinterpret_cast<const u32x4*>(o_src + q * 16);
                const u32x4 va = *reinterpret_cast<const u32x4*>(o_src + kGroup * (int)sizeof(OT) + q * 16);
                __builtin_nontemporal_store(vi, reinterpret_cast<u32x4*>(dst_i) + q);
                __builtin_nontemporal_store(va, reinterpret_cast<u32x4*>(dst_a) + q);
            }
        }
        __syncthreads();
    };

    for (int it = 0; worker + it * nworkers < ntiles; it += 2) {
        step(it, 0, rb);
        if (worker + (it + 1) * nworkers >= ntiles) break;
        step(it + 1, 1, ra);
    }
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

template <typename XT, typename WT, typename OT, int BW>
int launch_gate_fwd(const void* x, const void* w_i, const float* b_i, const void* w_a, const float* b_a, void* out_i,
                    void* out_a, int M, int D, int nb, hipStream_t st) {
    const int ngroups = ceil_div(D, kGroup);
    const int ntiles = ceil_div(M, kTileRows);
    int nworkers = kNumCU / ngroups;
    if (nworkers < 1) nworkers = 1;
    if (nworkers > ntiles) nworkers = ntiles;
    const size_t smem = 2 * kATileBytes + (size_t)kTileRows * (2 * kGroup * sizeof(OT) + 16);
    auto kernel = gate_proj_fwd_kernel<XT, WT, OT, BW>;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
        return HAWK_ERR_LAUNCH;
    hipLaunchKernelGGL(kernel, dim3((unsigned)nworkers, (unsigned)ngroups), dim3(kGateThreads), smem, st,
                       static_cast<const XT*>(x), static_cast<const WT*>(w_i), b_i, static_cast<const WT*>(w_a), b_a,
                       static_cast<OT*>(out_i), static_cast<OT*>(out_a), M, D, nb, ntiles);
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
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

}  // namespace

bool gate_proj_block_width_supported(int bw) { return bw == 32 || bw == 64 || bw == 128 || bw == 256; }

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

}  // namespace hawk
