// Scalar-ALU tree attention kernel: any of f32/f16/bf16, every head_dim and
// block size the API admits.  It is the float32 path (float32 has no fast matrix
// core format on gfx950) and a second, independently written implementation the
// matrix-core kernel is cross-checked against.
//
// One workgroup owns one query block of one (batch, head) slice, as one Triton
// program does in reference fstattention.py:42-45.  Keys are visited in tiles of
// 32: first the block's unique ancestors (masked per row by the packed tree
// mask), then the block's own rows through the diagonal "leaf" path
// (fstattention.py:86-91), then the dense shared prefix (fstattention.py:113-136).
// All three feed one online softmax in float32 (base 2, fstattention.py:55-59).
#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kThreads = 256;
constexpr int kTileN = 32;

template <int D, int M>
constexpr size_t generic_lds_bytes() {
    return sizeof(float) * (size_t)(M * (D + 1) + kTileN * (D + 1) + kTileN * D + M * (kTileN + 1) + 2 * M)
           + sizeof(int) * kTileN;
}

template <typename T, int D, int M>
__global__ __launch_bounds__(kThreads) void attn_generic_kernel(AttnParams p) {
    extern __shared__ float smem[];
    float* q_s = smem;                        // [M][D+1]
    float* k_s = q_s + M * (D + 1);           // [kTileN][D+1]
    float* v_s = k_s + kTileN * (D + 1);      // [kTileN][D]
    float* s_s = v_s + kTileN * D;            // [M][kTileN+1] scores, then weights
    float* alpha_s = s_s + M * (kTileN + 1);  // [M] rescale of the running sums
    float* stat_s = alpha_s + M;              // [M] 1/l for the epilogue
    int* key_s = reinterpret_cast<int*>(stat_s + M);  // [kTileN] K/V row of each tile column

    const int tid = threadIdx.x;
    const int j = blockIdx.x;
    const int hz = blockIdx.y;
    const int row0 = j * M;
    const T* qb = static_cast<const T*>(p.q) + (size_t)hz * p.nq * D;
    const T* kb = static_cast<const T*>(p.k) + (size_t)hz * p.nk * D;
    const T* vb = static_cast<const T*>(p.v) + (size_t)hz * p.nk * D;

    for (int e = tid; e < M * D; e += kThreads) {
        const int m = e / D, d = e % D;
        const int row = row0 + m;
        q_s[m * (D + 1) + d] = row < p.nq ? to_float(qb[(size_t)row * D + d]) : 0.f;
    }

    constexpr int kAcc = M * D / kThreads;
    float acc[kAcc];
#pragma unroll
    for (int i = 0; i < kAcc; ++i) acc[i] = 0.f;
    float m_i = -INFINITY, l_i = 0.f;  // running max / sum of row `tid` (tid < M)

    int n_anc = p.anc_count ? p.anc_count[j] : p.max_anc;
    n_anc = min(max(n_anc, 0), p.max_anc);
    const int anc_tiles = (n_anc + kTileN - 1) / kTileN;
    const int leaf_tiles = (M + kTileN - 1) / kTileN;
    const int prefix_tiles = (p.prefix + kTileN - 1) / kTileN;
    const int total_tiles = anc_tiles + leaf_tiles + prefix_tiles;

    for (int t = 0; t < total_tiles; ++t) {
        // kind 0: ancestors, 1: leaves (diagonal), 2: shared prefix
        int kind, base;
        if (t < anc_tiles) { kind = 0; base = t * kTileN; }
        else if (t < anc_tiles + leaf_tiles) { kind = 1; base = (t - anc_tiles) * kTileN; }
        else { kind = 2; base = (t - anc_tiles - leaf_tiles) * kTileN; }

        if (tid < kTileN) {
            int64_t idx = -1;
            const int c = base + tid;
            if (kind == 0) { if (c < n_anc) idx = p.ancestor_idx[(size_t)j * p.max_anc + c]; }
            else if (kind == 1) { if (c < M) idx = p.leaf_idx[(size_t)j * M + c]; }
            else { if (c < p.prefix) idx = c; }
            key_s[tid] = (idx >= 0 && idx < p.nk) ? (int)idx : -1;
        }
        __syncthreads();

        for (int e = tid; e < kTileN * D; e += kThreads) {
            const int n = e / D, d = e % D;
            const int key = key_s[n];
            float kf = 0.f, vf = 0.f;
            if (key >= 0) {
                kf = to_float(kb[(size_t)key * D + d]);
                vf = to_float(vb[(size_t)key * D + d]);
            }
            k_s[n * (D + 1) + d] = kf;
            v_s[n * D + d] = vf;
        }
        __syncthreads();

        for (int e = tid; e < M * kTileN; e += kThreads) {
            const int m = e / kTileN, n = e % kTileN;
            bool ok = key_s[n] >= 0;
            if (kind == 0) {
                const uint32_t w = p.mask_bits[((size_t)j * p.mask_words + (base >> 5)) * M + m];
                ok = ok && ((w >> n) & 1u);
            } else if (kind == 1) {
                ok = ok && (m == base + n);
            }
            float s = -INFINITY;
            if (ok) {
                float dot = 0.f;
#pragma unroll 8
                for (int d = 0; d < D; ++d) dot += q_s[m * (D + 1) + d] * k_s[n * (D + 1) + d];
                s = dot * p.scale_log2e;
            }
            s_s[m * (kTileN + 1) + n] = s;
        }
        __syncthreads();

        if (tid < M) {
            float mx = m_i;
            for (int n = 0; n < kTileN; ++n) mx = fmaxf(mx, s_s[tid * (kTileN + 1) + n]);
            const float alpha = (mx == -INFINITY) ? 1.f : exp2f(m_i - mx);
            float sum = 0.f;
            for (int n = 0; n < kTileN; ++n) {
                const float s = s_s[tid * (kTileN + 1) + n];
                const float w = (s == -INFINITY) ? 0.f : exp2f(s - mx);
                s_s[tid * (kTileN + 1) + n] = w;
                sum += w;
            }
            l_i = l_i * alpha + sum;
            m_i = mx;
            alpha_s[tid] = alpha;
        }
        __syncthreads();

#pragma unroll
        for (int i = 0; i < kAcc; ++i) {
            const int e = tid + i * kThreads;
            const int m = e / D, d = e % D;
            float a = acc[i] * alpha_s[m];
#pragma unroll 8
            for (int n = 0; n < kTileN; ++n) a += s_s[m * (kTileN + 1) + n] * v_s[n * D + d];
            acc[i] = a;
        }
        __syncthreads();
    }

    if (tid < M) {
        stat_s[tid] = l_i;
        const int row = row0 + tid;
        if (p.lse && row < p.nq)
            p.lse[(size_t)hz * p.nq + row] = l_i > 0.f ? m_i + log2f(l_i) : -INFINITY;
    }
    __syncthreads();

#pragma unroll
    for (int i = 0; i < kAcc; ++i) {
        const int e = tid + i * kThreads;
        const int m = e / D, d = e % D;
        const int row = row0 + m;
        if (row >= p.nq) continue;
        const float l = stat_s[m];
        const float val = l > 0.f ? acc[i] / l : 0.f;
        const size_t off = ((size_t)hz * p.nq + row) * D + d;
        if (p.out_f32) static_cast<float*>(p.o)[off] = val;
        else static_cast<T*>(p.o)[off] = from_float<T>(val);
    }
}

template <typename T, int D, int M>
int launch_one(const AttnParams& p, hipStream_t stream) {
    constexpr size_t lds = generic_lds_bytes<D, M>();
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&attn_generic_kernel<T, D, M>>();
        if (rc != FSTA_OK) return rc;
    }
    dim3 grid(p.nb, p.heads_total);
    hipLaunchKernelGGL((attn_generic_kernel<T, D, M>), grid, dim3(kThreads), lds, stream, p);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

template <typename T, int D>
int launch_m(const AttnParams& p, hipStream_t stream) {
    switch (p.block_m) {
        case 16: return launch_one<T, D, 16>(p, stream);
        case 32: return launch_one<T, D, 32>(p, stream);
        case 64: return launch_one<T, D, 64>(p, stream);
        case 128: return launch_one<T, D, 128>(p, stream);
    }
    return fail(FSTA_EUNSUPPORTED, "block_m=%d (supported: 16, 32, 64, 128)", p.block_m);
}

template <typename T>
int launch_d(const AttnParams& p, int head_dim, hipStream_t stream) {
    switch (head_dim) {
        case 16: return launch_m<T, 16>(p, stream);
        case 32: return launch_m<T, 32>(p, stream);
        case 64: return launch_m<T, 64>(p, stream);
        case 128: return launch_m<T, 128>(p, stream);
    }
    return fail(FSTA_EUNSUPPORTED, "head_dim=%d (supported: 16, 32, 64, 128)", head_dim);
}

}  // namespace

int launch_attention_generic(const AttnParams& p, int dtype, int head_dim, hipStream_t stream) {
    switch (dtype) {
        case FSTA_F32: return launch_d<float>(p, head_dim, stream);
        case FSTA_F16: return launch_d<__half>(p, head_dim, stream);
        case FSTA_BF16: return launch_d<__hip_bfloat16>(p, head_dim, stream);
    }
    return fail(FSTA_EINVAL, "dtype=%d", dtype);
}

}  // namespace fsta
