// Measuring tool, part of the instrumented library only (libfsta_timeline.so, `build.py --timeline`):
// how fast one SIMD of this GPU issues the bf16 matrix instructions the attention kernels are made
// of, alone and with vector-ALU instructions between them.  `python -m fstattention_amd.mfma_rate`
// launches the kernels below and prints the table.  The figures put a number on the issue time a
// kernel's counters imply (instructions x cycles each), which the published peak (one 16x16x32
// instruction per 16 cycles and SIMD) does not give.
#ifdef FSTA_TIMELINE
#include "fsta_common.h"

namespace fsta {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));

// The shader clock under the load of the loop: s_memtime counts shader cycles, s_memrealtime the constant 100 MHz
// clock; the first wave of the grid notes how far each got between its first and last instruction, behind the
// results (out[threads], out[threads + 1]).
struct ProbeClocks { uint64_t cycles, ticks; };
__device__ __forceinline__ ProbeClocks probe_clocks() {
    return ProbeClocks{(uint64_t)__builtin_readcyclecounter(), (uint64_t)__builtin_amdgcn_s_memrealtime()};
}
__device__ __forceinline__ void probe_note_clocks(const ProbeClocks& begin, float* out) {
    const ProbeClocks end = probe_clocks();
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        out[gridDim.x * blockDim.x] = (float)(end.cycles - begin.cycles);
        out[gridDim.x * blockDim.x + 1] = (float)(end.ticks - begin.ticks);
    }
}

// One workgroup of 4 waves per launch slot; every wave runs `iters` rounds of 8 matrix instructions that
// accumulate into ACCS accumulators in turn (1 = a chain on one accumulator), each followed by VALU
// independent multiply-adds.  The dynamic LDS size of the launch fixes how many workgroups share a CU.
template <int SHAPE, int ACCS, int VALU>
__global__ __launch_bounds__(256) void probe_mfma_kernel(const uint32_t* in, float* out, int iters) {
    extern __shared__ float probe_pad[];
    if (iters < 0) out[0] = probe_pad[threadIdx.x];
    const ProbeClocks clocks_begin = probe_clocks();
    probe_u32x4 a, b;
    for (int i = 0; i < 4; ++i) { a[i] = in[i * 256 + threadIdx.x]; b[i] = in[(4 + i) * 256 + threadIdx.x]; }
    const probe_bf16x8 A = __builtin_bit_cast(probe_bf16x8, a), B = __builtin_bit_cast(probe_bf16x8, b);
    float s = 0.f;
    float v[8];
    for (int i = 0; i < 8; ++i) v[i] = 1.f + i;
    // The matrix instructions are written as assembly with the accumulator as an in-out operand: through the
    // builtin the compiler rotates several accumulators through other registers with dozens of copies per round,
    // which is then what the loop measures.
    if (SHAPE == 16) {
        probe_f32x4 acc[ACCS];
        for (int i = 0; i < ACCS; ++i) acc[i] = probe_f32x4{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[j % ACCS]) : "v"(A), "v"(B));
#pragma unroll
                for (int u = 0; u < VALU; ++u) v[u & 7] = __builtin_fmaf(v[u & 7], 1.0001f, 0.5f);
            }
        }
        for (int i = 0; i < ACCS; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    } else {
        probe_f32x16 acc[ACCS];
        for (int i = 0; i < ACCS; ++i)
            for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j % ACCS]) : "v"(A), "v"(B));
#pragma unroll
                for (int u = 0; u < VALU; ++u) v[u & 7] = __builtin_fmaf(v[u & 7], 1.0001f, 0.5f);
            }
        }
        for (int i = 0; i < ACCS; ++i)
            for (int e = 0; e < 16; ++e) s += acc[i][e];
    }
    for (int i = 0; i < 8; ++i) s += v[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    probe_note_clocks(clocks_begin, out);
}

// vector ALU alone: the same multiply-adds without a matrix instruction between them
template <int VALU>
__global__ __launch_bounds__(256) void probe_valu_kernel(const uint32_t* in, float* out, int iters) {
    extern __shared__ float probe_pad[];
    if (iters < 0) out[0] = probe_pad[threadIdx.x];
    const ProbeClocks clocks_begin = probe_clocks();
    float v[8];
    for (int i = 0; i < 8; ++i) v[i] = 1.f + i + (float)in[threadIdx.x];
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int u = 0; u < VALU; ++u) v[u & 7] = __builtin_fmaf(v[u & 7], 1.0001f, 0.5f);
    }
    float s = 0.f;
    for (int i = 0; i < 8; ++i) s += v[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    probe_note_clocks(clocks_begin, out);
}

template <typename K> int probe_launch(K kernel, const uint32_t* in, float* out, int iters, int waves_per_simd, hipStream_t s) {
    // one workgroup per CU of an MI355X (256) and wave per SIMD, or two: 100 KB of LDS per workgroup lets one share a CU, 70 KB two
    const size_t lds = waves_per_simd == 1 ? 100 * 1024 : 70 * 1024;
    FSTA_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(kernel, dim3(256 * waves_per_simd), dim3(256), lds, s, in, out, iters);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

}  // namespace
}  // namespace fsta

using namespace fsta;

// shape 16 (16x16x32) or 32 (32x32x16), 0 = vector ALU only; accumulators 1, 2, 4 or 8; 0, 2, 4 or 8 multiply-adds
// per matrix instruction; 1 or 2 waves per SIMD.  `in`: 2048 uint32 (bf16 pairs), `out`: 2 * 256 * 256 + 2 floats.
extern "C" int fsta_probe_mfma_rate(int32_t shape, int32_t accumulators, int32_t valu, int32_t waves_per_simd,
                                    int32_t iters, const uint32_t* in, float* out, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (waves_per_simd != 1 && waves_per_simd != 2) return fail(FSTA_EINVAL, "fsta_probe_mfma_rate: waves_per_simd");
#define FSTA_PROBE_CASE(SH, AC, VA) \
    if (shape == SH && accumulators == AC && valu == VA) return probe_launch(&probe_mfma_kernel<SH, AC, VA>, in, out, iters, waves_per_simd, s);
    FSTA_PROBE_CASE(16, 1, 0) FSTA_PROBE_CASE(16, 2, 0) FSTA_PROBE_CASE(16, 4, 0) FSTA_PROBE_CASE(16, 8, 0)
    FSTA_PROBE_CASE(16, 1, 4) FSTA_PROBE_CASE(16, 8, 2) FSTA_PROBE_CASE(16, 8, 4) FSTA_PROBE_CASE(16, 8, 8)
    FSTA_PROBE_CASE(32, 1, 0) FSTA_PROBE_CASE(32, 4, 0) FSTA_PROBE_CASE(32, 4, 4) FSTA_PROBE_CASE(32, 4, 8)
#undef FSTA_PROBE_CASE
    if (shape == 0 && valu == 2) return probe_launch(&probe_valu_kernel<2>, in, out, iters, waves_per_simd, s);
    if (shape == 0 && valu == 4) return probe_launch(&probe_valu_kernel<4>, in, out, iters, waves_per_simd, s);
    if (shape == 0 && valu == 8) return probe_launch(&probe_valu_kernel<8>, in, out, iters, waves_per_simd, s);
    return fail(FSTA_EINVAL, "fsta_probe_mfma_rate: no such case (shape %d, %d accumulators, %d multiply-adds)", shape,
                accumulators, valu);
}
#endif  // FSTA_TIMELINE
