// The small closing reductions of the backward kernels (per-tile partial sums -> dLambda, the
// conv's dw / db, the gate projections' dw / db), as device functions over a task description:
// each entry point launches its own as a last kernel, and the backward of a whole recurrent
// core launches one kernel that runs all three, from the same code, so both give the same bits.
#pragma once

#include "hawk_device.h"

namespace hawk {

constexpr int kColsumThreads = 1024;   // kColsumCols columns x kColsumSlices row slices per block
constexpr int kColsumCols = 32, kColsumSlices = kColsumThreads / kColsumCols;

// Column sums of a [rows, cols] fp32 matrix in a fixed order.  Columns below n_first go to
// out_first, the rest to out_second.  With `lam` the sums are the partials of dLambda:
// out_first[c] = -8 sigmoid(lam[c]) * sum.
struct ColsumTask {
    const float* part;
    float* out_first;
    float* out_second;
    const float* lam;
    int rows, cols, n_first;
    int blocks() const { return (cols + kColsumCols - 1) / kColsumCols; }
};

// Block `block` of the task, by a workgroup of kColsumThreads threads: kColsumCols adjacent columns
// (one 128-byte line of a row) x kColsumSlices row slices; `s` is its LDS scratch.  The few rows a
// thread takes are all asked for at once: the launch is a handful of memory round trips long, so
// their number, not the bytes, sets its duration.
__device__ __forceinline__ void colsum_block(const ColsumTask& t, int block, float (*s)[kColsumCols]) {
    const int lane = threadIdx.x & (kColsumCols - 1);
    const int slice = threadIdx.x / kColsumCols;
    const int c = block * kColsumCols + lane;
    float sum = 0.0f;
    if (c < t.cols) {
        // eight independent loads in flight per thread; the order of additions is fixed
        int r = slice;
        for (; r + kColsumSlices * 7 < t.rows; r += kColsumSlices * 8) {
            float v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = t.part[(size_t)(r + kColsumSlices * k) * t.cols + c];
#pragma unroll
            for (int k = 0; k < 8; ++k) sum += v[k];
        }
        for (; r < t.rows; r += kColsumSlices) sum += t.part[(size_t)r * t.cols + c];
    }
    s[slice][lane] = sum;
    __syncthreads();
    if (slice == 0 && c < t.cols) {
        float tot = 0.0f;
#pragma unroll
        for (int k = 0; k < kColsumSlices; ++k) tot += s[k][lane];
        if (t.lam != nullptr) tot *= -8.0f * sigmoid_precise(t.lam[c]);
        if (c < t.n_first) t.out_first[c] = tot;
        else t.out_second[c - t.n_first] = tot;
    }
}

// dw_g = sum over the row splits of the gate projections' partial tiles, db_g likewise, splits
// in order.  Element idx of [dw_i | dw_a | db_i | db_a].
struct GateReduceTask {
    const float* part_w;
    const float* part_b;
    float* dw_i;
    float* dw_a;
    float* db_i;
    float* db_a;
    int nsplit, D;
    size_t wcount;
    __host__ __device__ size_t total() const { return 2 * wcount + 2 * (size_t)D; }
    // four adjacent elements at a time: sizes are multiples of four and every tensor starts on 16 bytes
    __host__ __device__ bool by_four() const {
        const uintptr_t ptrs = reinterpret_cast<uintptr_t>(part_w) | reinterpret_cast<uintptr_t>(part_b) |
                               reinterpret_cast<uintptr_t>(dw_i) | reinterpret_cast<uintptr_t>(dw_a) |
                               reinterpret_cast<uintptr_t>(db_i) | reinterpret_cast<uintptr_t>(db_a);
        return wcount % 4 == 0 && D % 4 == 0 && (ptrs & 15u) == 0;
    }
    // work items of the task: one per element, or one per four
    __host__ __device__ size_t items() const { return by_four() ? total() / 4 : total(); }
};

// Work items first, first + stride, ... of the task.
__device__ __forceinline__ void gate_reduce_one(const GateReduceTask& t, size_t idx) {
    float sum = 0.0f;
    if (idx < 2 * t.wcount) {
        for (int s = 0; s < t.nsplit; ++s) sum += t.part_w[(size_t)s * 2 * t.wcount + idx];
        if (idx < t.wcount) t.dw_i[idx] = sum;
        else t.dw_a[idx - t.wcount] = sum;
    } else {
        const size_t k = idx - 2 * t.wcount;
        for (int s = 0; s < t.nsplit; ++s) sum += t.part_b[(size_t)s * 2 * t.D + k];
        if (k < (size_t)t.D) {
            if (t.db_i != nullptr) t.db_i[k] = sum;
        } else if (t.db_a != nullptr) {
            t.db_a[k - t.D] = sum;
        }
    }
}
__device__ __forceinline__ void gate_reduce_span(const GateReduceTask& t, size_t first, size_t stride) {
    const size_t total = t.total();
    if (!t.by_four()) {
        for (size_t idx = first; idx < total; idx += stride) gate_reduce_one(t, idx);
        return;
    }
    // the same additions in the same order, element by element: splits in order
    for (size_t q = first; q < total / 4; q += stride) {
        const size_t idx = 4 * q;
        f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
        if (idx < 2 * t.wcount) {
            const f32x4* src = reinterpret_cast<const f32x4*>(t.part_w + idx);
            const size_t step = 2 * t.wcount / 4;
            // four splits' loads in flight at a time; the additions stay in split order
            int sp = 0;
            for (; sp + 4 <= t.nsplit; sp += 4) {
                f32x4 v[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = __builtin_nontemporal_load(src + (size_t)(sp + k) * step);
#pragma unroll
                for (int k = 0; k < 4; ++k) sum += v[k];
            }
            for (; sp < t.nsplit; ++sp) sum += __builtin_nontemporal_load(src + (size_t)sp * step);
            f32x4* dst = reinterpret_cast<f32x4*>(idx < t.wcount ? t.dw_i + idx : t.dw_a + (idx - t.wcount));
            *dst = sum;
        } else {
            const size_t k = idx - 2 * t.wcount;
            const f32x4* src = reinterpret_cast<const f32x4*>(t.part_b + k);
            const size_t step = 2 * (size_t)t.D / 4;
            for (int s = 0; s < t.nsplit; ++s) sum += src[(size_t)s * step];
            float* out = k < (size_t)t.D ? t.db_i : t.db_a;
            if (out != nullptr) *reinterpret_cast<f32x4*>(out + (k < (size_t)t.D ? k : k - t.D)) = sum;
        }
    }
}

}  // namespace hawk
