// Streaming probes: copy kernels that move NR tensors in and NW tensors out with the scan
// kernels' own memory instructions (non-temporal buffer loads and stores through a resource in
// scalar registers) and no arithmetic to speak of, in two shapes: flat (a 256-thread workgroup
// takes 16 KiB of every tensor, 16 bytes a lane) and in the scan's workgroup shape (eight waves
// stacked in time, each on 16 rows x 256 bytes with 4 bytes a lane; the tiles are taken in memory
// order or in the order a scan launch takes them, position along the sequence slowest).  They
// exist so that a benchmark can state, on its own tensors and in its own process, what the part
// delivers for the scan's mix of reads and writes with and without the scan's access shape.
// Every output element receives the sum of the inputs' 32-bit words at its place plus the
// output's index, so a test can check that all of every tensor was moved.
#include "hawk_scan.h"

namespace hawk {
namespace {

constexpr int kMaxProbeReads = 5, kMaxProbeWrites = 3;
struct ProbeTensors {
    const void* r[kMaxProbeReads];
    void* w[kMaxProbeWrites];
};

constexpr int kFlatBytes = 16384;   // of every tensor per workgroup

template <int NR, int NW>
__global__ __launch_bounds__(256) void stream_probe_flat_kernel(ProbeTensors t) {
    const size_t origin = (size_t)blockIdx.x * kFlatBytes;
    const uint32_t lane_bytes = threadIdx.x * 16u;
    u32x4 acc[4] = {};
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const rsrc_t rs = make_rsrc(static_cast<const char*>(t.r[i]) + origin, kFlatBytes);
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[k] += buffer_load<u32x4>(rs, lane_bytes, k * 4096u);
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const rsrc_t rs = make_rsrc(static_cast<char*>(t.w[i]) + origin, kFlatBytes);
#pragma unroll
        for (int k = 0; k < 4; ++k) buffer_store<u32x4>(acc[k] + (uint32_t)i, rs, lane_bytes, k * 4096u);
    }
}

constexpr int kTileWaves = 8, kTileRowsPerWave = 16, kTileRowBytes = 256;

template <int NR, int NW>
__global__ __launch_bounds__(kTileWaves* kWave) void stream_probe_tile_kernel(ProbeTensors t, uint32_t row_pitch,
                                                                             int column_tiles, int groups_per_seq,
                                                                             int sequences) {
    // the scan's launch order: position along the sequence slowest, then sequence, then column tile
    const int tile = (int)blockIdx.x, per_pos = sequences * column_tiles;
    const int seg = tile / per_pos, rem = tile - seg * per_pos;
    const int seq = rem / column_tiles, ct = rem - seq * column_tiles;
    const int rg = seq * groups_per_seq + seg;
    const int w = __builtin_amdgcn_readfirstlane((int)threadIdx.x / kWave);
    const size_t origin = ((size_t)rg * kTileWaves + w) * kTileRowsPerWave * row_pitch + (size_t)ct * kTileRowBytes;
    const uint32_t window = (kTileRowsPerWave - 1) * row_pitch + kTileRowBytes;
    const uint32_t lane_bytes = (threadIdx.x & (kWave - 1)) * 4u;
    uint32_t acc[kTileRowsPerWave] = {};
#pragma unroll
    for (int i = 0; i < NR; ++i) {
        const rsrc_t rs = make_rsrc(static_cast<const char*>(t.r[i]) + origin, window);
#pragma unroll
        for (int k = 0; k < kTileRowsPerWave; ++k) acc[k] += buffer_load<uint32_t>(rs, lane_bytes, k * row_pitch);
    }
#pragma unroll
    for (int i = 0; i < NW; ++i) {
        const rsrc_t rs = make_rsrc(static_cast<char*>(t.w[i]) + origin, window);
#pragma unroll
        for (int k = 0; k < kTileRowsPerWave; ++k)
            buffer_store<uint32_t>(acc[k] + (uint32_t)i, rs, lane_bytes, k * row_pitch);
    }
}

template <int NR, int NW>
int launch_probe(const ProbeTensors& t, size_t bytes, uint32_t row_pitch, int shape, hipStream_t st) {
    if (shape == 0) {
        hipLaunchKernelGGL((stream_probe_flat_kernel<NR, NW>), dim3((unsigned)(bytes / kFlatBytes)), dim3(256), 0, st, t);
    } else {
        const int column_tiles = (int)(row_pitch / kTileRowBytes);
        const size_t row_groups = bytes / row_pitch / (kTileWaves * kTileRowsPerWave);
        hipLaunchKernelGGL((stream_probe_tile_kernel<NR, NW>), dim3((unsigned)(row_groups * column_tiles)),
                           dim3(kTileWaves * kWave), 0, st, t, row_pitch, column_tiles, shape,
                           (int)(row_groups / (size_t)shape));
    }
    return hipGetLastError() == hipSuccess ? HAWK_OK : HAWK_ERR_LAUNCH;
}

}  // namespace

bool stream_probe_shape_ok(size_t bytes, size_t row_pitch, int shape) {
    if (bytes == 0 || bytes / kFlatBytes > 0x7fffffffull) return false;
    if (shape == 0) return bytes % kFlatBytes == 0;
    if (shape < 1 || row_pitch == 0 || row_pitch % kTileRowBytes != 0 || row_pitch > (1u << 24)) return false;
    if (bytes % row_pitch != 0 || (bytes / row_pitch) % (kTileWaves * kTileRowsPerWave) != 0) return false;
    const size_t row_groups = bytes / row_pitch / (kTileWaves * kTileRowsPerWave);
    return row_groups % (size_t)shape == 0 && row_groups * (row_pitch / kTileRowBytes) <= 0x7fffffffull;
}

int stream_probe(const void* const* reads, int n_reads, void* const* writes, int n_writes, size_t bytes,
                 size_t row_pitch, int shape, hipStream_t st) {
    ProbeTensors t = {};
    for (int i = 0; i < n_reads; ++i) t.r[i] = reads[i];
    for (int i = 0; i < n_writes; ++i) t.w[i] = writes[i];
    const uint32_t rp = (uint32_t)row_pitch;
    switch (n_reads * 10 + n_writes) {
        case 11: return launch_probe<1, 1>(t, bytes, rp, shape, st);
        case 12: return launch_probe<1, 2>(t, bytes, rp, shape, st);
        case 13: return launch_probe<1, 3>(t, bytes, rp, shape, st);
        case 21: return launch_probe<2, 1>(t, bytes, rp, shape, st);
        case 31: return launch_probe<3, 1>(t, bytes, rp, shape, st);
        case 53: return launch_probe<5, 3>(t, bytes, rp, shape, st);
        default: return HAWK_ERR_BAD_SHAPE;
    }
}

}  // namespace hawk
