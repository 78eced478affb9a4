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
    const int64_t row = idx / chunks_per_row;
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
