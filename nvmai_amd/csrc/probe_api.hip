// A measuring stick, not part of the path: a kernel that only reads a buffer, so that the fraction of
// the HBM peak a streaming kernel of this library reaches can be set beside what a plain read reaches on
// the same device in the same run (bench.py --workload read).
#include "ctx.hpp"

using namespace nvmai;

namespace {

// A wave reads UNROLL KiB at a time, every load of a round in flight before the first is used; waves stride
// over the buffer.  The sum leaves the kernel only under a condition that never holds, which is enough to
// keep the loads.
template <int UNROLL>
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ p, uint64_t n_vec, uint32_t* sink) {
    const uint64_t wave = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6), waves = (uint64_t)gridDim.x * 4;
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t acc = 0;
    uint64_t base = wave * UNROLL * 64;
    for (; base + UNROLL * 64 <= n_vec; base += waves * UNROLL * 64) {
        uint4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = p[base + u * 64 + lane];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (uint64_t i = base + lane; i < n_vec && i < base + UNROLL * 64; i += 64) {      // the ragged end
        const uint4 v = p[i];
        acc += v.x ^ v.y ^ v.z ^ v.w;
    }
    if (acc == 0x9E3779B9u && sink) sink[0] = acc;
}

}  // namespace

extern "C" int nvmai_hip_read_probe(nvmai_hip_ctx* ctx, nvmai_stream stream, const void* data, uint64_t bytes,
                                    uint32_t* sink) {
    if (!ctx) return NVMAI_ERR_INVALID_ARG;
    if (bytes == 0) return NVMAI_OK;
    if (!data) return NVMAI_ERR_INVALID_ARG;
    if (!aligned16(data) || bytes % 16) return NVMAI_ERR_ALIGNMENT;
    const uint64_t n_vec = bytes / 16;
    const uint64_t rounds = (n_vec + 8 * 64 - 1) / (8 * 64);            // 8 KiB per wave and round
    const uint32_t blocks = (uint32_t)(rounds / 4 < 8192 ? (rounds + 3) / 4 : 8192);
    read_probe_kernel<8><<<blocks, 256, 0, (hipStream_t)stream>>>(reinterpret_cast<const uint4*>(data), n_vec, sink);
    return launch_status();
}
