// Merge of two partial attention results over disjoint key sets (same queries): the step that
// lets the dense shared prefix of reference fstattention.py:113-136 be computed by another
// kernel (a paged / flash kernel over a real KV cache) and joined with the tree part through the
// base-2 log-sum-exp of fstattention.py:139-141.  Element-wise, HBM-bound: per row 3 x D
// elements and 3 floats move once; 16 bytes per lane and access.
#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kMergeThreads = 256;

template <typename T> struct Vec16;   // 16 bytes of T
template <> struct Vec16<float> { static constexpr int n = 4; };
template <> struct Vec16<__half> { static constexpr int n = 8; };
template <> struct Vec16<__hip_bfloat16> { static constexpr int n = 8; };

template <typename T>
__global__ __launch_bounds__(kMergeThreads) void merge_states_kernel(
    const T* __restrict__ o_a, const float* __restrict__ lse_a, const T* __restrict__ o_b,
    const float* __restrict__ lse_b, T* __restrict__ o_out, float* __restrict__ lse_out, int64_t rows,
    int32_t chunks_per_row) {
    constexpr int kN = Vec16<T>::n;
    const int64_t idx = (int64_t)blockIdx.x * kMergeThreads + threadIdx.x;
    // (a 64-bit division costs ~170 instructions per thread: 32-bit arithmetic where the index fits)
    const int64_t row = rows * chunks_per_row <= 0x7fffffff ? (int64_t)((uint32_t)idx / (uint32_t)chunks_per_row)
                                                            : idx / chunks_per_row;
    if (row >= rows) return;
    const int chunk = (int)(idx - row * chunks_per_row);
    const float la = lse_a[row], lb = lse_b[row];
    const float m = fmaxf(la, lb);
    // weights of the two parts; a part without keys has lse = -inf and weight 0
    const float wa = m == -INFINITY ? 0.f : exp2f(la - m);
    const float wb = m == -INFINITY ? 0.f : exp2f(lb - m);
    const float sum = wa + wb;
    const float inv = sum > 0.f ? 1.f / sum : 0.f;
    const float fa = wa * inv, fb = wb * inv;
    const size_t off = ((size_t)row * chunks_per_row + chunk) * kN;
    struct alignas(16) Pack { T v[kN]; };
    const Pack a = *reinterpret_cast<const Pack*>(o_a + off);
    const Pack b = *reinterpret_cast<const Pack*>(o_b + off);
    Pack out;
#pragma unroll
    for (int i = 0; i < kN; ++i) {
        // a weight of exactly 0 drops its part whatever that part holds
        const float xa = fa > 0.f ? to_float(a.v[i]) * fa : 0.f;
        const float xb = fb > 0.f ? to_float(b.v[i]) * fb : 0.f;
        out.v[i] = from_float<T>(xa + xb);
    }
    *reinterpret_cast<Pack*>(o_out + off) = out;
    if (lse_out && chunk == 0) lse_out[row] = sum > 0.f ? m + log2f(sum) : -INFINITY;
}

// Joins the partial results of a key-split attention launch: `splits` normalised float32 rows
// with their base-2 log-sum-exps per query row.  4 floats per lane and part.
template <typename T>
__global__ __launch_bounds__(kMergeThreads) void merge_splits_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_lse, int splits, int64_t rows,
    int32_t chunks_per_row, T* __restrict__ o, float* __restrict__ lse) {
    const int64_t idx = (int64_t)blockIdx.x * kMergeThreads + threadIdx.x;
    const int64_t row = rows * chunks_per_row <= 0x7fffffff ? (int64_t)((uint32_t)idx / (uint32_t)chunks_per_row)
                                                            : idx / chunks_per_row;
    if (row >= rows) return;
    const int chunk = (int)(idx - row * chunks_per_row);
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, part_lse[(size_t)s * rows + row]);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float sum = 0.f;
    const size_t part_stride = (size_t)rows * chunks_per_row;   // in float4
    const float4* src = reinterpret_cast<const float4*>(part_o) + (size_t)row * chunks_per_row + chunk;
    for (int s = 0; s < splits; ++s) {
        const float l = part_lse[(size_t)s * rows + row];
        const float w = l == -INFINITY ? 0.f : exp2f(l - m);   // a part without keys drops out
        const float4 x = src[(size_t)s * part_stride];
        if (w > 0.f) {
            acc[0] += w * x.x; acc[1] += w * x.y; acc[2] += w * x.z; acc[3] += w * x.w;
            sum += w;
        }
    }
    const float inv = sum > 0.f ? 1.f / sum : 0.f;
    struct alignas(sizeof(T) * 4) Pack { T v[4]; };
    Pack out;
#pragma unroll
    for (int i = 0; i < 4; ++i) out.v[i] = from_float<T>(acc[i] * inv);
    *reinterpret_cast<Pack*>(o + ((size_t)row * chunks_per_row + chunk) * 4) = out;
    if (lse && chunk == 0) lse[row] = sum > 0.f ? m + log2f(sum) : -INFINITY;
}

template <typename T>
int launch_merge(const void* o_a, const float* lse_a, const void* o_b, const float* lse_b, void* o_out,
                 float* lse_out, int64_t rows, int32_t head_dim, hipStream_t stream) {
    const int chunks = head_dim / Vec16<T>::n;
    const int64_t threads = rows * chunks;
    const int64_t blocks = (threads + kMergeThreads - 1) / kMergeThreads;
    if (blocks > 0x7fffffff) return fail(FSTA_EUNSUPPORTED, "fsta_merge_states: %lld rows", (long long)rows);
    hipLaunchKernelGGL(merge_states_kernel<T>, dim3((unsigned)blocks), dim3(kMergeThreads), 0, stream,
                       static_cast<const T*>(o_a), lse_a, static_cast<const T*>(o_b), lse_b,
                       static_cast<T*>(o_out), lse_out, rows, chunks);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

}  // namespace

int launch_merge_splits(const float* part_o, const float* part_lse, int splits, int64_t rows, int head_dim,
                        void* o, int out_dtype, float* lse, hipStream_t stream) {
    const int chunks = head_dim / 4;
    const int64_t blocks = (rows * chunks + kMergeThreads - 1) / kMergeThreads;
    if (blocks > 0x7fffffff) return fail(FSTA_EUNSUPPORTED, "merge of key splits: %lld rows", (long long)rows);
    const dim3 grid((unsigned)blocks), block(kMergeThreads);
    switch (out_dtype) {
        case FSTA_F32:
            hipLaunchKernelGGL(merge_splits_kernel<float>, grid, block, 0, stream, part_o, part_lse, splits, rows,
                               chunks, static_cast<float*>(o), lse);
            break;
        case FSTA_F16:
            hipLaunchKernelGGL(merge_splits_kernel<__half>, grid, block, 0, stream, part_o, part_lse, splits, rows,
                               chunks, static_cast<__half*>(o), lse);
            break;
        case FSTA_BF16:
            hipLaunchKernelGGL(merge_splits_kernel<__hip_bfloat16>, grid, block, 0, stream, part_o, part_lse, splits,
                               rows, chunks, static_cast<__hip_bfloat16*>(o), lse);
            break;
        default: return fail(FSTA_EINVAL, "merge of key splits: out_dtype=%d", out_dtype);
    }
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

}  // namespace fsta

using namespace fsta;

extern "C" int fsta_merge_states(const void* o_a, const float* lse_a, const void* o_b, const float* lse_b,
                                 void* o_out, float* lse_out, int64_t rows, int32_t head_dim, int32_t dtype,
                                 void* stream) {
    if (rows < 0 || head_dim < 8 || head_dim % 8 != 0)
        return fail(FSTA_EINVAL, "fsta_merge_states: rows=%lld head_dim=%d (need a multiple of 8)",
                    (long long)rows, head_dim);
    if (rows == 0) return FSTA_OK;
    if (!o_a || !lse_a || !o_b || !lse_b || !o_out) return fail(FSTA_EINVAL, "fsta_merge_states: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case FSTA_F32: return launch_merge<float>(o_a, lse_a, o_b, lse_b, o_out, lse_out, rows, head_dim, s);
        case FSTA_F16: return launch_merge<__half>(o_a, lse_a, o_b, lse_b, o_out, lse_out, rows, head_dim, s);
        case FSTA_BF16: return launch_merge<__hip_bfloat16>(o_a, lse_a, o_b, lse_b, o_out, lse_out, rows, head_dim, s);
    }
    return fail(FSTA_EINVAL, "fsta_merge_states: dtype=%d", dtype);
}
