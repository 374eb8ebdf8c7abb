// Read-bandwidth probe: what the memory system of this GPU gives a kernel that only reads, with the access pattern of
// the decode kernels (every wavefront walks its own contiguous range in 1 KiB pieces, one 16-byte load per lane, a fixed
// number of loads in flight) or with the textbook grid-stride pattern.  The yardstick next to the fused GEMV's rate; the
// counterpart of the reference's bench/micro/bwprobe.cu:23-60 (stride and per-warp chunk kernels, load-hint modes).
//
// Measurement only: built into libbf16n_probe.so, which the benchmark programs load next to the product library (the
// product library exports no probe).  One C entry point, bf16n_probe_read.
#include "dev_w64.h"

#include <hip/hip_runtime.h>

namespace bf16n {
namespace dev {

namespace {

__device__ __forceinline__ uint32_t fold(uint32_t s, const uint4 v) { return s ^ v.x ^ v.y ^ v.z ^ v.w; }

// wavefront w reads pieces [w * per_wave, (w + 1) * per_wave) of 1 KiB each, DEPTH loads in flight
template <int DEPTH, bool ONCE>
__global__ void __launch_bounds__(512) k_probe_ranges(const uint4 * __restrict__ src, uint64_t pieces, uint64_t per_wave,
                                                      uint32_t * __restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const uint64_t w = (uint64_t) blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    const uint64_t first = w * per_wave;
    if (first >= pieces) {
        return;
    }
    const uint64_t n = pieces - first < per_wave ? pieces - first : per_wave;
    const range_t r = make_range(src + first * 64, (uint32_t) (n * 1024));
    uint32_t off = 16 * (uint32_t) lane, s = 0;
    uint4 q[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
        q[d] = range_load16<ONCE>(r, off);
        off += 1024;
    }
    for (uint64_t i = 0; i < n; i += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            s = fold(s, q[d]);                      // pieces past the end read as zeros
            q[d] = range_load16<ONCE>(r, off);
            off += 1024;
        }
    }
    if (s == 0x9E3779B9u) {
        sink[0] = s; // never true for the buffers the probe is run on; keeps the loads alive
    }
}

// thread i reads 16-byte element i, i + threads, ...: U independent loads per iteration
template <int U, bool ONCE>
__global__ void __launch_bounds__(256) k_probe_stride(const uint4 * __restrict__ src, uint64_t n16, uint32_t * __restrict__ sink) {
    const uint64_t step = (uint64_t) gridDim.x * blockDim.x;
    uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t s = 0;
    for (; i + (U - 1) * step < n16; i += U * step) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            v[u] = ONCE ? load_once(src + i + u * step) : src[i + u * step];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            s = fold(s, v[u]);
        }
    }
    for (; i < n16; i += step) {
        s = fold(s, ONCE ? load_once(src + i) : src[i]);
    }
    if (s == 0x9E3779B9u) {
        sink[0] = s;
    }
}

} // namespace

// pattern 0: per-wavefront ranges, non-temporal loads; 1: the same with plain loads; 2 / 3: grid-stride, non-temporal
// / plain.  bytes is rounded down to whole KiB.  waves_per_cu wavefronts per CU (0: 16, the fused GEMV's occupancy).
static void launch_read_probe(const void * src, uint64_t bytes, int pattern, int waves_per_cu, uint32_t * sink, int cus, hipStream_t stream) {
    const uint64_t pieces = bytes / 1024;
    if (pattern <= 1) {
        const uint64_t waves = (uint64_t) cus * (waves_per_cu > 0 ? waves_per_cu : 16);
        const uint64_t per_wave = (pieces + waves - 1) / waves;
        const unsigned blocks = (unsigned) ((waves + 7) / 8);
        if (pattern == 0) {
            hipLaunchKernelGGL((k_probe_ranges<4, true>), dim3(blocks), dim3(512), 0, stream, (const uint4 *) src, pieces, per_wave, sink);
        } else {
            hipLaunchKernelGGL((k_probe_ranges<4, false>), dim3(blocks), dim3(512), 0, stream, (const uint4 *) src, pieces, per_wave, sink);
        }
    } else {
        const unsigned blocks = (unsigned) (cus * (waves_per_cu > 0 ? waves_per_cu : 16) / 4);
        if (pattern == 2) {
            hipLaunchKernelGGL((k_probe_stride<4, true>), dim3(blocks), dim3(256), 0, stream, (const uint4 *) src, pieces * 64, sink);
        } else {
            hipLaunchKernelGGL((k_probe_stride<4, false>), dim3(blocks), dim3(256), 0, stream, (const uint4 *) src, pieces * 64, sink);
        }
    }
}

} // namespace dev
} // namespace bf16n

// Returns 0, or 1 for arguments out of range, or 2 for a HIP error.  src 16-byte aligned; bytes >= 1024; pattern 0..3;
// waves_per_cu 0..32; sink: one device word (never written for ordinary data); stream: hipStream_t.
extern "C" int bf16n_probe_read(const void * src, uint64_t bytes, int pattern, int waves_per_cu, uint32_t * sink, void * stream) {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
            return 2;
        }
        cus = prop.multiProcessorCount;
    }
    if (!src || !sink || ((uintptr_t) src & 15) != 0 || pattern < 0 || pattern > 3 || bytes < 1024 || waves_per_cu < 0 || waves_per_cu > 32) {
        return 1;
    }
    // a wavefront's range is addressed with 32-bit offsets
    if (bytes / 1024 / ((uint64_t) cus * (waves_per_cu > 0 ? waves_per_cu : 16)) >= (1u << 21)) {
        return 1;
    }
    bf16n::dev::launch_read_probe(src, bytes, pattern, waves_per_cu, sink, cus, (hipStream_t) stream);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
