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
#include <type_traits>

#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kThreads = 256;
constexpr int kTileN = 32;
constexpr int kPad = 4;     // floats of padding per LDS row: rows stay 16-byte aligned for vector reads

// 16 bytes of T -> floats
template <typename T> struct Vec16 { static constexpr int n = 16 / (int)sizeof(T); };
template <typename T>
__device__ __forceinline__ void load16(const T* src, float (&out)[Vec16<T>::n]) {
    struct alignas(16) Pack { T v[Vec16<T>::n]; };
    const Pack p = *reinterpret_cast<const Pack*>(src);
#pragma unroll
    for (int i = 0; i < Vec16<T>::n; ++i) out[i] = to_float(p.v[i]);
}

template <int D, int M>
constexpr size_t generic_lds_bytes() {
    return sizeof(float) * (size_t)(M * (D + kPad) + 2 * kTileN * (D + kPad) + M * (kTileN + kPad) + 2 * M)
           + sizeof(int) * 2 * kTileN;
}

// Register tiles: a thread owns kRowsS x 4 scores of a tile (4 neighbouring keys) and kRowsO x 4
// output values (4 neighbouring head dims), and reads its operands from LDS 16 bytes at a time.
template <typename T, int D, int M>
__global__ __launch_bounds__(kThreads) void attn_generic_kernel(AttnParams p) {
    constexpr int kPitch = D + kPad;            // floats per row of q_s / k_s / v_s
    constexpr int kPitchS = kTileN + kPad;      // floats per row of s_s
    constexpr int kColGroupsS = kTileN / 4;     // 8 groups of 4 keys
    constexpr int kRowSlotsS = kThreads / kColGroupsS;                 // 32 row slots
    constexpr int kRowsS = (M + kRowSlotsS - 1) / kRowSlotsS;          // score rows per thread
    constexpr int kColGroupsO = D / 4;          // groups of 4 head dims
    constexpr int kRowSlotsO = kThreads / kColGroupsO;
    constexpr int kRowsO = (M + kRowSlotsO - 1) / kRowSlotsO;          // output rows per thread
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* q_s = smem;                          // [M][kPitch]
    float* k_s = q_s + M * kPitch;              // [kTileN][kPitch]
    float* v_s = k_s + kTileN * kPitch;         // [kTileN][kPitch]
    float* s_s = v_s + kTileN * kPitch;         // [M][kPitchS] scores, then weights
    float* alpha_s = s_s + M * kPitchS;         // [M] rescale of the running sums
    float* stat_s = alpha_s + M;                // [M] 1/l for the epilogue
    int* key_s = reinterpret_cast<int*>(stat_s + M);  // [2][kTileN] K/V row of each tile column, tiles t and t + 1

    const int tid = threadIdx.x;
    const int j = blockIdx.x;
    const int hz = blockIdx.y;
    const int row0 = j * M;
    const T* qb = static_cast<const T*>(p.q) + (size_t)hz * p.nq * D;
    const T* kb = static_cast<const T*>(p.k) + (size_t)hz * p.nk * D;
    const T* vb = static_cast<const T*>(p.v) + (size_t)hz * p.nk * D;

    constexpr int kVec = Vec16<T>::n;           // elements per 16-byte global load

    // this thread's tiles
    const int sc = (tid % kColGroupsS) * 4;     // first key column of the score tile
    const int sr = tid / kColGroupsS;           // score rows sr + kRowSlotsS * i
    const int oc = (tid % kColGroupsO) * 4;     // first head dim of the output tile
    const int orow = tid / kColGroupsO;         // output rows orow + kRowSlotsO * i
    float acc[kRowsO][4];
#pragma unroll
    for (int i = 0; i < kRowsO; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[i][c] = 0.f;
    // running maximum / sum of this thread's score rows (the 8 threads that share a row hold the same values)
    float m_i[kRowsS], l_i[kRowsS];
#pragma unroll
    for (int i = 0; i < kRowsS; ++i) { m_i[i] = -INFINITY; l_i[i] = 0.f; }

    // the block's ancestor count and the first entries of both lists are requested together: which of the
    // two lists tile 0 (and tile 1) comes from depends on the count, and the count is one more round trip
    int64_t first_anc0 = -1, first_anc1 = -1, first_leaf0 = -1, first_leaf1 = -1;
    if (tid < kTileN) {
        if (tid < p.max_anc) first_anc0 = p.ancestor_idx[(size_t)j * p.max_anc + tid];
        if (kTileN + tid < p.max_anc) first_anc1 = p.ancestor_idx[(size_t)j * p.max_anc + kTileN + tid];
        if (tid < M) first_leaf0 = p.leaf_idx[(size_t)j * M + tid];
        if (kTileN + tid < M) first_leaf1 = p.leaf_idx[(size_t)j * M + kTileN + tid];
    }
    int n_anc = p.anc_count ? p.anc_count[j] : p.max_anc;
    n_anc = min(max(n_anc, 0), p.max_anc);
    const int anc_tiles = (n_anc + kTileN - 1) / kTileN;
    const int leaf_tiles = (M + kTileN - 1) / kTileN;
    const int prefix_tiles = (p.prefix + kTileN - 1) / kTileN;
    const int total_tiles = anc_tiles + leaf_tiles + prefix_tiles;

    // kind 0: ancestors, 1: leaves (diagonal), 2: shared prefix
    auto tile_kind = [&](int t, int& base) {
        if (t < anc_tiles) { base = t * kTileN; return 0; }
        if (t < anc_tiles + leaf_tiles) { base = (t - anc_tiles) * kTileN; return 1; }
        base = (t - anc_tiles - leaf_tiles) * kTileN;
        return 2;
    };
    // The tile loop is a software pipeline: while tile t is worked on, the K/V rows of tile t + 1 are
    // on their way into registers and the key list of tile t + 2 into a register of the first 32
    // threads; each tile costs compute time only, not two dependent memory round trips as well.
    auto load_key = [&](int t) -> int {          // threads 0 .. 31: K/V row of column tid of tile t, or -1
        if (t >= total_tiles) return -1;
        int base;
        const int kind = tile_kind(t, base);
        int64_t idx = -1;
        const int c = base + tid;
        if (kind == 0) { if (c < n_anc) idx = p.ancestor_idx[(size_t)j * p.max_anc + c]; }
        else if (kind == 1) { if (c < M) idx = p.leaf_idx[(size_t)j * M + c]; }
        else { if (c < p.prefix) idx = c; }
        return (idx >= 0 && idx < p.nk) ? (int)idx : -1;
    };
    constexpr int kLoads = (kTileN * D / kVec + kThreads - 1) / kThreads;   // 16-byte pieces of K (and of V) per thread
    float kreg[kLoads][kVec], vreg[kLoads][kVec];
    auto fetch_rows = [&](const int* keys) {     // K/V rows of the tile whose key list is `keys` -> registers
#pragma unroll
        for (int it = 0; it < kLoads; ++it) {
            const int e = tid + it * kThreads;
#pragma unroll
            for (int i = 0; i < kVec; ++i) { kreg[it][i] = 0.f; vreg[it][i] = 0.f; }
            if (e < kTileN * D / kVec) {
                const int n = e / (D / kVec), d = (e % (D / kVec)) * kVec;
                const int key = keys[n];
                if (key >= 0) {
                    load16(kb + (size_t)key * D + d, kreg[it]);
                    load16(vb + (size_t)key * D + d, vreg[it]);
                }
            }
        }
    };
    if (tid < kTileN) {
        // tiles 0 and 1 from the entries requested above where they are ancestor or leaf tiles
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            int key = -1;
            if (t < total_tiles) {
                int base;
                const int kind = tile_kind(t, base);
                if (kind == 2 || base >= 2 * kTileN) {
                    key = load_key(t);
                } else {
                    const int c = base + tid;
                    // (unary plus: a choice between values, not between addresses)
                    const int64_t from_anc = base == 0 ? +first_anc0 : +first_anc1;
                    const int64_t from_leaf = base == 0 ? +first_leaf0 : +first_leaf1;
                    const int64_t idx = kind == 0 ? (c < n_anc ? from_anc : -1) : (c < M ? from_leaf : -1);
                    key = (idx >= 0 && idx < p.nk) ? (int)idx : -1;
                }
            }
            key_s[t * kTileN + tid] = key;
        }
    }
    __syncthreads();
    if (total_tiles > 0) fetch_rows(key_s);
    // The Q rows are requested behind the first tile's K/V rows (both are needed at the same moment, the first
    // score tile): in front of the key lists they would put one more memory round trip into the start-up chain.
    for (int e = tid; e < M * D / kVec; e += kThreads) {
        const int m = e / (D / kVec), d = (e % (D / kVec)) * kVec;
        const int row = row0 + m;
        float x[kVec];
#pragma unroll
        for (int i = 0; i < kVec; ++i) x[i] = 0.f;
        if (row < p.nq) load16(qb + (size_t)row * D + d, x);
#pragma unroll
        for (int i = 0; i < kVec; ++i) q_s[m * kPitch + d + i] = x[i];
    }


    for (int t = 0; t < total_tiles; ++t) {
        int base;
        const int kind = tile_kind(t, base);
        const int* keys = key_s + (t & 1) * kTileN;
        // rows of tile t: registers -> LDS; then the requests for tile t + 1 and the list of tile t + 2
#pragma unroll
        for (int it = 0; it < kLoads; ++it) {
            const int e = tid + it * kThreads;
            if (e < kTileN * D / kVec) {
                const int n = e / (D / kVec), d = (e % (D / kVec)) * kVec;
#pragma unroll
                for (int i = 0; i < kVec; ++i) {
                    k_s[n * kPitch + d + i] = kreg[it][i];
                    v_s[n * kPitch + d + i] = vreg[it][i];
                }
            }
        }
        if (t + 1 < total_tiles) fetch_rows(key_s + ((t + 1) & 1) * kTileN);
        int key_after_next = -1;
        if (tid < kTileN) key_after_next = load_key(t + 2);
        __syncthreads();

        // scores of this thread's tile: rows sr + 32 i, keys sc .. sc + 3
        if (sr < M) {
            float dot[kRowsS][4];
#pragma unroll
            for (int i = 0; i < kRowsS; ++i)
#pragma unroll
                for (int c = 0; c < 4; ++c) dot[i][c] = 0.f;
            if (kind == 1) {
                // leaf tile: row m sees its own key only (column m - base): one dot product per row, by the thread
                // whose four columns hold it
#pragma unroll
                for (int i = 0; i < kRowsS; ++i) {
                    const int m = sr + kRowSlotsS * i;
                    const int own = m - base - sc;
                    if ((kRowsS * kRowSlotsS > M && m >= M) || own < 0 || own >= 4) continue;
                    float part = 0.f;
#pragma unroll 4
                    for (int d = 0; d < D; d += 4) {
                        const float4 kk = *reinterpret_cast<const float4*>(k_s + (sc + own) * kPitch + d);
                        const float4 qq = *reinterpret_cast<const float4*>(q_s + m * kPitch + d);
                        part += qq.x * kk.x + qq.y * kk.y + qq.z * kk.z + qq.w * kk.w;
                    }
#pragma unroll
                    for (int c = 0; c < 4; ++c) dot[i][c] = c == own ? part : dot[i][c];
                }
            } else {
#pragma unroll 4
                for (int d = 0; d < D; d += 4) {
                    float4 kq[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) kq[c] = *reinterpret_cast<const float4*>(k_s + (sc + c) * kPitch + d);
#pragma unroll
                    for (int i = 0; i < kRowsS; ++i) {
                        const int m = sr + kRowSlotsS * i;
                        if (kRowsS * kRowSlotsS > M && m >= M) continue;
                        const float4 qq = *reinterpret_cast<const float4*>(q_s + m * kPitch + d);
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            dot[i][c] += qq.x * kq[c].x + qq.y * kq[c].y + qq.z * kq[c].z + qq.w * kq[c].w;
                    }
                }
            }
            // mask, then the online softmax of the row among the 8 threads that share it (neighbouring lanes:
            // maximum and sum by lane exchanges), weights into s_s for the O tiles
#pragma unroll
            for (int i = 0; i < kRowsS; ++i) {
                const int m = sr + kRowSlotsS * i;
                if (kRowsS * kRowSlotsS > M && m >= M) continue;     // (whole waves: M is a multiple of 16, a wave holds 8 rows)
                uint32_t w = 0xffffffffu;
                if (kind == 0) w = p.mask_bits[((size_t)j * p.mask_words + (base >> 5)) * M + m];
                float sv[4];
                float mx = -INFINITY;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int n = sc + c;
                    bool ok = keys[n] >= 0 && ((w >> n) & 1u);
                    if (kind == 1) ok = ok && (m == base + n);
                    sv[c] = ok ? dot[i][c] * p.scale_log2e : -INFINITY;
                    mx = fmaxf(mx, sv[c]);
                }
#pragma unroll
                for (int dlt = 1; dlt < kColGroupsS; dlt <<= 1) mx = fmaxf(mx, __shfl_xor(mx, dlt));
                const float m_new = fmaxf(m_i[i], mx);
                const float alpha = (m_new == -INFINITY) ? 1.f : exp2f(m_i[i] - m_new);
                float sum = 0.f;
                float wv[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    wv[c] = (sv[c] == -INFINITY) ? 0.f : exp2f(sv[c] - m_new);
                    sum += wv[c];
                }
                *reinterpret_cast<float4*>(s_s + m * kPitchS + sc) = make_float4(wv[0], wv[1], wv[2], wv[3]);
#pragma unroll
                for (int dlt = 1; dlt < kColGroupsS; dlt <<= 1) sum += __shfl_xor(sum, dlt);
                l_i[i] = l_i[i] * alpha + sum;
                m_i[i] = m_new;
                if (sc == 0) alpha_s[m] = alpha;
            }
        }
        __syncthreads();

        // O tile: rows orow + kRowSlotsO i, head dims oc .. oc + 3
        if (orow < M) {
#pragma unroll
            for (int i = 0; i < kRowsO; ++i) {
                const int m = orow + kRowSlotsO * i;
                if (kRowsO * kRowSlotsO > M && m >= M) continue;
                const float a = alpha_s[m];
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[i][c] *= a;
            }
            if (kind == 1) {
                // leaf tile: a row's only weight sits on its own key
#pragma unroll
                for (int i = 0; i < kRowsO; ++i) {
                    const int m = orow + kRowSlotsO * i;
                    const int own = m - base;
                    if ((kRowsO * kRowSlotsO > M && m >= M) || own < 0 || own >= kTileN) continue;
                    const float w = s_s[m * kPitchS + own];
                    const float4 vv = *reinterpret_cast<const float4*>(v_s + own * kPitch + oc);
                    acc[i][0] += w * vv.x;
                    acc[i][1] += w * vv.y;
                    acc[i][2] += w * vv.z;
                    acc[i][3] += w * vv.w;
                }
            } else {
#pragma unroll 2
                for (int n = 0; n < kTileN; n += 4) {
                    float4 vv[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) vv[u] = *reinterpret_cast<const float4*>(v_s + (n + u) * kPitch + oc);
#pragma unroll
                    for (int i = 0; i < kRowsO; ++i) {
                        const int m = orow + kRowSlotsO * i;
                        if (kRowsO * kRowSlotsO > M && m >= M) continue;
                        const float4 w = *reinterpret_cast<const float4*>(s_s + m * kPitchS + n);
                        acc[i][0] += w.x * vv[0].x + w.y * vv[1].x + w.z * vv[2].x + w.w * vv[3].x;
                        acc[i][1] += w.x * vv[0].y + w.y * vv[1].y + w.z * vv[2].y + w.w * vv[3].y;
                        acc[i][2] += w.x * vv[0].z + w.y * vv[1].z + w.z * vv[2].z + w.w * vv[3].z;
                        acc[i][3] += w.x * vv[0].w + w.y * vv[1].w + w.z * vv[2].w + w.w * vv[3].w;
                    }
                }
            }
        }
        if (tid < kTileN) key_s[(t & 1) * kTileN + tid] = key_after_next;   // (tile t's list was last read in the score phase)
        __syncthreads();
    }

    if (sr < M && sc == 0) {
#pragma unroll
        for (int i = 0; i < kRowsS; ++i) {
            const int m = sr + kRowSlotsS * i;
            if (kRowsS * kRowSlotsS > M && m >= M) continue;
            stat_s[m] = l_i[i];
            const int row = row0 + m;
            if (p.lse && row < p.nq)
                p.lse[(size_t)hz * p.nq + row] = l_i[i] > 0.f ? m_i[i] + log2f(l_i[i]) : -INFINITY;
        }
    }
    __syncthreads();

    if (orow < M) {
#pragma unroll
        for (int i = 0; i < kRowsO; ++i) {
            const int m = orow + kRowSlotsO * i;
            const int row = row0 + m;
            if ((kRowsO * kRowSlotsO > M && m >= M) || row >= p.nq) continue;
            const float l = stat_s[m];
            const size_t off = ((size_t)hz * p.nq + row) * D + oc;
            // four neighbouring head dims leave in one store (non-temporal: nobody in this launch reads the output again)
            typedef float f32x4 __attribute__((ext_vector_type(4)));
            typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
            float val[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) val[c] = l > 0.f ? acc[i][c] / l : 0.f;
            if (p.out_f32 || sizeof(T) == 4) {
                const f32x4 v = {val[0], val[1], val[2], val[3]};
                __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(p.o) + off));
            } else {
                T h[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) h[c] = from_float<T>(val[c]);
                u32x2 pk;
                __builtin_memcpy(&pk, h, sizeof(pk) < sizeof(h) ? sizeof(pk) : sizeof(h));
                __builtin_nontemporal_store(pk, reinterpret_cast<u32x2*>(static_cast<T*>(p.o) + off));
            }
        }
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
    note_launch({"attn_generic_kernel", sizeof(T) == 4 ? "float" : (std::is_same<T, __half>::value ? "__half" : "__hip_bfloat16"),
                 {D, M, 0, 0, 0}, 2, 0u, 0, 0});
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
