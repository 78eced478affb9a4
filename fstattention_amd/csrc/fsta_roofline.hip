// Two measuring aids behind the C ABI, used by bench.py to put this GPU's own ceilings beside the
// attention kernels' figures: what a launch costs when the kernel does nothing, and what a kernel
// that only reads gets out of HBM.  Neither has a counterpart in the reference.
#include "fsta_common.h"

namespace fsta {
namespace {

__global__ void empty_kernel() {}

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int kReadThreads = 256;

// Every lane reads 16 bytes per load, consecutive lanes consecutive addresses (a wave = 1 KiB per
// instruction), kReadUnroll independent loads before the first use; the xor of everything read
// is compared with a value it never takes, so that the loads cannot be dropped.  CONTIG: a workgroup
// walks one contiguous piece of the buffer (its loads of one round are 4 KiB apart) instead of
// striding over the whole buffer with the grid.
template <int kReadUnroll, bool NT, bool CONTIG>
__global__ __launch_bounds__(kReadThreads) void hbm_read_kernel(const u32x4* __restrict__ src, size_t chunks,
                                                               uint32_t* __restrict__ sink) {
    size_t stride = (size_t)gridDim.x * kReadThreads;
    size_t i = (size_t)blockIdx.x * kReadThreads + threadIdx.x;
    if (CONTIG) {
        const size_t per_wg = (chunks / gridDim.x) & ~(size_t)(kReadThreads * kReadUnroll - 1);
        src += (size_t)blockIdx.x * per_wg;
        chunks = per_wg;
        stride = kReadThreads;
        i = threadIdx.x;
    }
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (; i + (kReadUnroll - 1) * stride < chunks; i += kReadUnroll * stride) {
        u32x4 x[kReadUnroll];
#pragma unroll
        for (int u = 0; u < kReadUnroll; ++u) x[u] = NT ? __builtin_nontemporal_load(src + i + u * stride) : src[i + u * stride];
#pragma unroll
        for (int u = 0; u < kReadUnroll; ++u) acc ^= x[u];
    }
    for (; i < chunks; i += stride) acc ^= src[i];
    const uint32_t all = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (all == 0x5ca1ab1eu && sink) sink[0] = all;
}

}  // namespace
}  // namespace fsta

extern "C" int fsta_probe_empty_launch(int32_t workgroups, int32_t threads, void* stream) {
    if (workgroups < 1 || threads < 1 || threads > 1024)
        return fsta::fail(FSTA_EINVAL, "fsta_probe_empty_launch: workgroups=%d threads=%d", workgroups, threads);
    hipLaunchKernelGGL(fsta::empty_kernel, dim3((unsigned)workgroups), dim3((unsigned)threads), 0,
                       static_cast<hipStream_t>(stream));
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

extern "C" int fsta_probe_hbm_read(const void* src, size_t bytes, int32_t workgroups, int32_t variant, uint32_t* sink,
                                   void* stream) {
    if (!src || bytes < 16 || workgroups < 1 || variant < 0 || variant > 7 || fsta::misaligned(src, 16) || fsta::misaligned(sink, 4))
        return fsta::fail(FSTA_EINVAL, "fsta_probe_hbm_read: src=%p (16-byte aligned), bytes=%zu, workgroups=%d, variant=%d", src,
                          bytes, workgroups, variant);
    using namespace fsta;
    const dim3 grid((unsigned)workgroups), block(kReadThreads);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const u32x4* p = static_cast<const u32x4*>(src);
    const size_t chunks = bytes / 16;
    switch (variant) {      // bit 0: 16 instead of 8 loads in flight; bit 1: non-temporal loads; bit 2: contiguous pieces per workgroup
        case 0: hipLaunchKernelGGL((hbm_read_kernel<8, false, false>), grid, block, 0, s, p, chunks, sink); break;
        case 1: hipLaunchKernelGGL((hbm_read_kernel<16, false, false>), grid, block, 0, s, p, chunks, sink); break;
        case 2: hipLaunchKernelGGL((hbm_read_kernel<8, true, false>), grid, block, 0, s, p, chunks, sink); break;
        case 3: hipLaunchKernelGGL((hbm_read_kernel<16, true, false>), grid, block, 0, s, p, chunks, sink); break;
        case 4: hipLaunchKernelGGL((hbm_read_kernel<8, false, true>), grid, block, 0, s, p, chunks, sink); break;
        case 5: hipLaunchKernelGGL((hbm_read_kernel<16, false, true>), grid, block, 0, s, p, chunks, sink); break;
        case 6: hipLaunchKernelGGL((hbm_read_kernel<8, true, true>), grid, block, 0, s, p, chunks, sink); break;
        default: hipLaunchKernelGGL((hbm_read_kernel<16, true, true>), grid, block, 0, s, p, chunks, sink); break;
    }
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}
