// Measurement aids: what the memory paths the gathers live on deliver on the device at hand, so that a rate can be
// held against a measured ceiling and not only against a product of nominal figures.  No counterpart in the
// reference; nothing in the library's own paths calls these.
//
//   nnueft_probe_l2_gather   every CU gathers pieces of `span` contiguous bytes at random places of a set that is
//                            resident in its XCD's L2 (workgroup id % 8 = XCD, each XCD its own set), `depth`
//                            loads in flight per lane: the access pattern of the row gathers through L2
//   nnueft_probe_lds_read    every CU reads 16 bytes per lane from a 96 KB LDS tile: a wave 1 KB in a row
//                            (pattern 0) or each 8-lane group a whole 128-byte row at a random row (pattern 1:
//                            the gather out of LDS tiles)
#include "internal.h"

namespace {

using nnueft_blocked::kXcd;
typedef float f4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t lcg(uint32_t& s) {
    s = s * 1664525u + 1013904223u;
    return s >> 8;
}

template <int DEPTH>
__global__ __launch_bounds__(256) void k_probe_l2_gather(const char* __restrict__ src, float* __restrict__ sink,
                                                         uint32_t set_bytes, uint32_t span, int iters) {
    const int lane = threadIdx.x & 63;
    const int x = blockIdx.x % kXcd;
    const char* set = src + (size_t)x * set_bytes;
    const uint32_t nspans = set_bytes / span;
    const uint32_t lanes_per_span = span / 16;                 // 8 for a 128-byte line, 64 for 1 KB
    const uint32_t group = lane / lanes_per_span;              // which of the wave's spans this lane reads
    const uint32_t in_span = (lane % lanes_per_span) * 16;
    uint32_t s = (blockIdx.x * 256u + (threadIdx.x & ~63u)) * 2654435761u + 12345u + group * 7919u;
    f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
        f4 v[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
            v[d] = *reinterpret_cast<const f4*>(set + (size_t)(lcg(s) % nspans) * span + in_span);
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) acc += v[d];
    }
    if (acc.x + acc.y + acc.z + acc.w == 1.2345e-30f) sink[0] = acc.x;
}

constexpr int kProbeTile = 96 * 1024;

template <int PATTERN>
__global__ __launch_bounds__(1024) void k_probe_lds_read(float* __restrict__ sink, int iters) {
    extern __shared__ float4 probe_lds[];
    char* tb = reinterpret_cast<char*>(probe_lds);
    const int tid = threadIdx.x, lane = tid & 63;
    for (int i = tid; i < kProbeTile / 16; i += 1024) probe_lds[i] = make_float4(1.f, 0.f, 0.f, 0.f);
    __syncthreads();
    typedef __attribute__((address_space(3))) const f4 lds_f4;
    const uint32_t base = (uint32_t)(uintptr_t)tb;
    // eight places per lane group, drawn once; every round moves them on by an odd step inside the first 64 KB of
    // the tile (512 rows of 128 bytes, 64 pieces of 1 KB), so the loop is reads and little else
    uint32_t s = (blockIdx.x * 1024u + (PATTERN == 1 ? (tid >> 3) : (tid >> 6))) * 2654435761u + 99u;
    uint32_t place[8];
#pragma unroll
    for (int d = 0; d < 8; ++d) place[d] = lcg(s);
    const uint32_t lane_off = PATTERN == 1 ? base + (lane & 7) * 16 : base + lane * 16;
    f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
        f4 v[8];
#pragma unroll
        for (int d = 0; d < 8; ++d) {
            place[d] += 0x9e3779b1u;
            const uint32_t addr = PATTERN == 1 ? lane_off + ((place[d] >> 23) << 7) : lane_off + ((place[d] >> 26) << 10);
            v[d] = *reinterpret_cast<lds_f4*>(addr);
        }
#pragma unroll
        for (int d = 0; d < 8; ++d) acc += v[d];
    }
    if (acc.x + acc.y + acc.z + acc.w == 1.2345e-30f) sink[0] = acc.x;
}

}  // namespace

extern "C" int nnueft_probe_l2_gather(const void* src, size_t src_bytes, float* sink, int set_bytes, int span, int depth,
                                      int iters, long long* bytes_read, void* stream) {
    if (!src || !sink || set_bytes <= 0 || (span != 128 && span != 1024) || set_bytes % span || iters <= 0) return NNUEFT_E_ARG;
    if ((depth != 4 && depth != 8 && depth != 16) || src_bytes < (size_t)kXcd * set_bytes) return NNUEFT_E_ARG;
    const nnueft_dev::DeviceInfo* info = nullptr;
    const int rc = nnueft_dev::device_info(nullptr, &info);
    if (rc) return rc;
    const int grid = info->cus / kXcd * kXcd * 8;   // 8 workgroups of 4 waves a CU
    if (grid <= 0) return NNUEFT_E_UNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    const char* p = (const char*)src;
    if (depth == 4)
        hipLaunchKernelGGL(k_probe_l2_gather<4>, dim3(grid), dim3(256), 0, st, p, sink, (uint32_t)set_bytes, (uint32_t)span, iters);
    else if (depth == 8)
        hipLaunchKernelGGL(k_probe_l2_gather<8>, dim3(grid), dim3(256), 0, st, p, sink, (uint32_t)set_bytes, (uint32_t)span, iters);
    else
        hipLaunchKernelGGL(k_probe_l2_gather<16>, dim3(grid), dim3(256), 0, st, p, sink, (uint32_t)set_bytes, (uint32_t)span, iters);
    NNUEFT_LAUNCH_CHECK();
    if (bytes_read) *bytes_read = (long long)grid * 256 * 16 * depth * iters;
    return 0;
}

extern "C" int nnueft_probe_lds_read(float* sink, int pattern, int iters, long long* bytes_read, void* stream) {
    if (!sink || (pattern != 0 && pattern != 1) || iters <= 0) return NNUEFT_E_ARG;
    int device = 0;
    const nnueft_dev::DeviceInfo* info = nullptr;
    const int rc = nnueft_dev::device_info(&device, &info);
    if (rc) return rc;
    if (info->max_lds < kProbeTile) return NNUEFT_E_UNSUPPORTED;
    // the permission to use more than 64 KB of LDS belongs to the loaded kernel; asking again costs nothing
    hipError_t e = hipFuncSetAttribute((const void*)k_probe_lds_read<0>, hipFuncAttributeMaxDynamicSharedMemorySize, kProbeTile);
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)k_probe_lds_read<1>, hipFuncAttributeMaxDynamicSharedMemorySize, kProbeTile);
    if (e != hipSuccess) return (int)e;
    hipStream_t st = (hipStream_t)stream;
    const int grid = info->cus;
    if (pattern == 0)
        hipLaunchKernelGGL(k_probe_lds_read<0>, dim3(grid), dim3(1024), kProbeTile, st, sink, iters);
    else
        hipLaunchKernelGGL(k_probe_lds_read<1>, dim3(grid), dim3(1024), kProbeTile, st, sink, iters);
    NNUEFT_LAUNCH_CHECK();
    if (bytes_read) *bytes_read = (long long)grid * 1024 * 16 * 8 * iters;
    return 0;
}
