// Dense shared-prefix attention for gfx950 (reference fstattention.py:113-136: every query of the
// tree sees every key of the prefix, no mask): a flash-style kernel of its own for long prefixes.
//
// The tree kernel walks the prefix with 16 query rows per wave and the mask machinery of the tree
// tiles, and every query block of a head pulls every prefix tile into its own LDS.  Here a
// workgroup owns 128 query rows (4 waves x 32 rows) and a run of prefix keys; a wave keeps TWO
// groups of 16 query rows and feeds every K / V fragment it reads from LDS to both (half the LDS
// traffic per product) and no mask words exist.
// Each workgroup writes a normalised float32 partial result and its base-2 log-sum-exp into the
// caller's workspace; the launch of the tree part (tree kernel, prefix left out) reads them back and
// joins them with its own.  Bound: matrix cores and HBM at once (256 flop per K/V byte at 256 query
// rows per head against a machine balance of ~310): both have to be kept busy.
#include <type_traits>

#include "fsta_mfma_common.h"

namespace fsta {
namespace {

using namespace mfma;

constexpr int kPfxRows = 128;      // query rows per workgroup
constexpr int kPfxWaves = 4;       // 32 rows each
constexpr int kPfxStages = 5;      // ring depth, 16 KB per stage at head_dim 128: two workgroups fill a CU's 160 KB

// SPLIT: bf16 weights as hi + lo pairs (two matrix instructions per product)
template <bool BF16, int D, bool SPLIT>
__global__ __launch_bounds__(kPfxWaves * 64, 2) void prefix_attn_kernel(AttnParams p) {
    using MM = Mma<BF16>;
    using T = typename MM::elem;
    using Frag = typename MM::frag;
    constexpr int kCpr = D / 8;                    // 16-byte chunks per row
    constexpr int kRowsPerDma = 64 / kCpr;         // rows one wave-wide 1 KiB transfer covers
    constexpr int kDmaPerTile = 2 * kTileN / kRowsPerDma;
    constexpr int kDmaPerWave = kDmaPerTile / kPfxWaves;
    static_assert(kDmaPerWave >= 2 && kDmaPerWave % 2 == 0, "a wave's transfers are K/V pairs of whole row groups");
    constexpr int kRowGroups = kDmaPerWave / 2;
    constexpr int kSteps = D / 32;                 // MFMAs per 16-key half of S^T
    constexpr int kDTiles = D / 16;                // 16-row tiles of O^T
    constexpr int kTileElems = kTileN * D;
    constexpr float kTrustedSum = BF16 ? 16777216.f : 32768.f;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* ring = reinterpret_cast<T*>(smem);          // [kPfxStages][K tile | V tile]

    // grid (8 XCDs x key runs, row chunks, slices per XCD), as the tree kernel's: blockIdx.x % 8 is the XCD
    const int xcd = blockIdx.x % kXcds;
    const int run = blockIdx.x / kXcds;
    const int hz = blockIdx.z * kXcds + xcd;
    const int row_base = blockIdx.y * kPfxRows;
    if (hz >= p.heads_total) return;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ql = lane & 15, g = lane >> 4;

    const T* qb = static_cast<const T*>(p.q) + (size_t)hz * p.nq * D;
    const unsigned char* kb = static_cast<const unsigned char*>(p.k) + (size_t)hz * p.nk * D * 2;
    const unsigned char* vb = static_cast<const unsigned char*>(p.v) + (size_t)hz * p.nk * D * 2;

    // this workgroup's run of prefix tiles
    const int all_tiles = (p.prefix + kTileN - 1) / kTileN;
    const int first_tile = min(run * p.split_tiles, all_tiles);
    const int total = min(first_tile + p.split_tiles, all_tiles) - first_tile;

    // ---- gather ring: tile t of the run lives in slot t % kPfxStages --------------------------------
    const int dma_row = lane / kCpr, dma_slot = lane % kCpr;
    uint32_t dma_k[kRowGroups], dma_v[kRowGroups];   // chunk offsets of this lane's K and V pieces (swizzled)
#pragma unroll
    for (int i = 0; i < kRowGroups; ++i) {
        const int r = (wave * kRowGroups + i) * kRowsPerDma + dma_row;
        dma_k[i] = (uint32_t)k_chunk<D>(r, dma_slot) * 16u;
        dma_v[i] = (uint32_t)v16_chunk<D>(r, dma_slot) * 16u;
    }
    auto issue = [&](int t) {
        T* dst = ring + (t % kPfxStages) * 2 * kTileElems;
#pragma unroll
        for (int i = 0; i < kRowGroups; ++i) {
            const int u = wave * kRowGroups + i;
            const int row = min((first_tile + t) * kTileN + u * kRowsPerDma + dma_row, p.prefix - 1);
            const uint32_t off = (uint32_t)row * (uint32_t)(D * 2);
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(kb + (size_t)(off + dma_k[i])),
                                             (void __attribute__((address_space(3)))*)(dst + u * 512), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(vb + (size_t)(off + dma_v[i])),
                                             (void __attribute__((address_space(3)))*)(dst + kTileElems + u * 512), 16, 0, 0);
        }
    };
    int issued = 0;
    for (; issued < total && issued < kPfxStages; ++issued) issue(issued);

    // ---- Q fragments of the wave's two row groups, straight from memory (B operand of S^T = K.Q^T:
    //      lane holds Q[q][32 s + 8 g .. + 7]); rows past the end are read as the last row, never stored
    Frag qf[2][kSteps];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row = min(row_base + wave * 32 + h * 16 + ql, p.nq - 1);
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            // (non-temporal: the Q rows of a run are read once)
            const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(qb + (size_t)row * D + 32 * s + 8 * g));
            qf[h][s] = __builtin_bit_cast(Frag, raw);
        }
    }

    float m_i[2] = {-INFINITY, -INFINITY}, l_i[2] = {0.f, 0.f};
    f32x4 o[2][kDTiles];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt) o[h][dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    constexpr int kHalfTileBytes = 16 * D * 2;
    const uint32_t k_lane0 = (uint32_t)(ql * D + k_chunk<D>(ql, g) * 8) * 2;
    const int tr_r0 = 4 * g + (ql >> 2), tr_col = 4 * (ql & 3);
    const uint32_t v_lane0 = (uint32_t)(tr_r0 * D + v16_chunk<D>(tr_r0, tr_col >> 3) * 8 + (tr_col & 7)) * 2;
    const float sc = p.scale_log2e;

    // S^T = K_tile . Q^T for both row groups: every K fragment feeds two products
    typedef const u32x4 __attribute__((address_space(3))) * lds_u32x4;
    auto scores = [&](int t, f32x4 (&s)[2][2]) {
        const uint32_t k_addr0 = lds_addr(ring + (t % kPfxStages) * 2 * kTileElems) + k_lane0;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            s[0][sub] = f32x4{0.f, 0.f, 0.f, 0.f};
            s[1][sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < kSteps; ++ks) {
                const u32x4 raw = *(lds_u32x4)(uintptr_t)((k_addr0 ^ (uint32_t)(ks << 6)) + sub * kHalfTileBytes);
                const Frag kf = __builtin_bit_cast(Frag, raw);
                s[0][sub] = mfma16(kf, qf[0][ks], s[0][sub]);
                s[1][sub] = mfma16(kf, qf[1][ks], s[1][sub]);
            }
        }
    };

    // Software pipeline over the tiles: the scores of tile t + 1 go to the matrix cores in front of the
    // softmax of tile t, in one straight piece of code, so that the vector ALU works on one tile while the
    // matrix pipeline works on the next.  Tile t (its V rows) and tile t + 1 (its K rows) are resident, the
    // tiles behind them in flight.  (The last step computes the scores of the last tile once more and drops
    // them: no branch in the loop body.)  Only the last tile of the prefix can be partial: `tail` masks it.
    f32x4 s[2][2];
    if (total > 0) {
        wait_tiles_outstanding<kDmaPerWave>(min(issued - 1, 3));
        ring_barrier();
        scores(0, s);
    }
    auto step = [&](int t, auto tail) {
        constexpr bool kTail = decltype(tail)::value;
        // tile t + 1 has landed for everyone, everyone is done with tile t - 1: its slot is refilled
        wait_tiles_outstanding<kDmaPerWave>(min(max(issued - t - 2, 0), 3));
        ring_barrier();
        if (t > 0 && issued < total) { issue(issued); ++issued; }
        const T* vt = ring + (t % kPfxStages) * 2 * kTileElems + kTileElems;
        // Scores of tile t + 1 and, between the matrix instructions (16 cycles of the matrix pipeline each), the
        // weights of tile t against the running maximum as it stands (exact as long as no weight gets large: a
        // power of two on a row's weights cancels in O / l; the row maximum is only looked at when that fails).
        // Written interleaved because the compiler keeps this order: per K fragment its two products, then the
        // exponentials of two scores; the next fragment is requested before the products of this one.
        f32x4 s_next[2][2];
        float pw[2][8], rowsum[2] = {0.f, 0.f};
        float sv[2][8];
        float neg_m[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) neg_m[h] = m_i[h] == -INFINITY ? 0.f : -m_i[h];
        {
            constexpr int kFrags = 2 * kSteps;                 // K fragments of a tile
            constexpr int kPerFrag = 16 / kFrags;              // scores of tile t handled per fragment
            const uint32_t k_addr0 = lds_addr(ring + (min(t + 1, total - 1) % kPfxStages) * 2 * kTileElems) + k_lane0;
            auto frag_addr = [&](int i) { return (k_addr0 ^ (uint32_t)((i % kSteps) << 6)) + (i / kSteps) * kHalfTileBytes; };
            u32x4 raw = *(lds_u32x4)(uintptr_t)frag_addr(0);
#pragma unroll
            for (int i = 0; i < kFrags; ++i) {
                const int sub = i / kSteps, ks = i % kSteps;
                const Frag kf = __builtin_bit_cast(Frag, raw);
                if (i + 1 < kFrags) raw = *(lds_u32x4)(uintptr_t)frag_addr(i + 1);
                if (ks == 0) {
                    s_next[0][sub] = f32x4{0.f, 0.f, 0.f, 0.f};
                    s_next[1][sub] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
                s_next[0][sub] = mfma16(kf, qf[0][ks], s_next[0][sub]);
                s_next[1][sub] = mfma16(kf, qf[1][ks], s_next[1][sub]);
#pragma unroll
                for (int e = i * kPerFrag; e < (i + 1) * kPerFrag; ++e) {
                    const int h = e / 8, r = e % 8;
                    float score = s[h][r / 4][r % 4];
                    if (kTail) {
                        const int left = p.prefix - (first_tile + t) * kTileN;     // keys of this tile that exist
                        if (16 * (r / 4) + 4 * g + (r % 4) >= left) score = -INFINITY;
                    }
                    sv[h][r] = score;
                    pw[h][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(score, sc, neg_m[h]));
                    rowsum[h] += pw[h][r];
                }
            }
        }
        const bool redo = !(rowsum[0] <= kTrustedSum) || !(rowsum[1] <= kTrustedSum) || m_i[0] == -INFINITY || m_i[1] == -INFINITY;
        if (__ballot(redo) != 0ull) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float mx_raw = fmaxf(fmaxf(fmaxf(sv[h][0], sv[h][1]), fmaxf(sv[h][2], sv[h][3])),
                                     fmaxf(fmaxf(sv[h][4], sv[h][5]), fmaxf(sv[h][6], sv[h][7])));
                mx_raw = max_quarters(mx_raw);
                const float mx = mx_raw * sc;   // the scale is positive here
                const bool raise = mx > m_i[h] + kRescaleSlack || (m_i[h] == -INFINITY && mx > -INFINITY);
                const float alpha = raise ? __builtin_amdgcn_exp2f(m_i[h] - mx) : 1.f;   // exp2(-inf) = 0
                if (raise) m_i[h] = mx;
                l_i[h] *= alpha;
#pragma unroll
                for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[h][dt][r] *= alpha;
                const float neg_m = m_i[h] == -INFINITY ? 0.f : -m_i[h];
                rowsum[h] = 0.f;
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    pw[h][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[h][r], sc, neg_m));
                    rowsum[h] += pw[h][r];
                }
            }
        }
        Frag ph[2], pl[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            l_i[h] += rowsum[h];
            u32x4 hi4, lo4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = pw[h][2 * e], b = pw[h][2 * e + 1];
                const uint32_t hi = MM::pack(a, b);
                hi4[e] = hi;
                if (SPLIT) lo4[e] = MM::pack(a - MM::low(hi), b - MM::high(hi));
            }
            ph[h] = __builtin_bit_cast(Frag, hi4);
            if (SPLIT) pl[h] = __builtin_bit_cast(Frag, lo4);
        }
        // O^T += V_tile^T . P^T for both row groups: every V fragment feeds two (four) products
        // (the fragments of the next two head-dim tiles are requested before the products of these two)
        const uint32_t v_addr0 = lds_addr(vt) + v_lane0;
        auto read_v = [&](VPair (&f)[2], int dt) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const uint32_t addr = v_addr0 ^ (uint32_t)((dt + i) << 5);
                f[i].a = lds_read_tr16(addr);
                f[i].b = lds_read_tr16_at<kHalfTileBytes>(addr);
            }
        };
        VPair fa[2], fb[2];
        read_v(fa, 0);
#pragma unroll
        for (int dt = 0; dt < kDTiles; dt += 2) {
            VPair (&cur)[2] = (dt & 2) ? fb : fa;
            VPair (&nxt)[2] = (dt & 2) ? fa : fb;
            if (dt + 2 < kDTiles) {
                read_v(nxt, dt + 2);
                asm volatile("s_waitcnt lgkmcnt(4)" ::: "memory");   // the four reads of `cur` are in, the next four in flight
            } else {
                lds_wait();
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                lds_tie(cur[i].a);
                lds_tie(cur[i].b);
                const Frag vf = __builtin_bit_cast(Frag, cur[i]);
                o[0][dt + i] = mfma16(vf, ph[0], o[0][dt + i]);
                o[1][dt + i] = mfma16(vf, ph[1], o[1][dt + i]);
                if (SPLIT) {
                    o[0][dt + i] = mfma16(vf, pl[0], o[0][dt + i]);
                    o[1][dt + i] = mfma16(vf, pl[1], o[1][dt + i]);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) s[h][sub] = s_next[h][sub];
    };
    const bool partial_tail = first_tile + total == all_tiles && p.prefix % kTileN != 0;
    for (int t = 0; t + 1 < total; ++t) step(t, std::false_type{});
    if (total > 0) {
        if (partial_tail) step(total - 1, std::true_type{});
        else step(total - 1, std::false_type{});
    }

    // ---- normalised float32 partial result and its log-sum-exp into the workspace slot of this run ----
    // slot 0 belongs to the tree part; accumulator rows 4g .. 4g+3 of tile dt are 4 consecutive head dims
    const int slot = 1 + run;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const float l_tot = sum_quarters(l_i[h]);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const int row = row_base + wave * 32 + h * 16 + ql;
        if (row < p.nq) {
            const size_t out_row = ((size_t)slot * p.heads_total + hz) * p.nq + row;
            if (g == 0) p.part_lse[out_row] = l_tot > 0.f ? m_i[h] + log2f(l_tot) : -INFINITY;
            float* dst = p.part_o + out_row * D;
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt) {
                const f32x4 val = {o[h][dt][0] * inv, o[h][dt][1] * inv, o[h][dt][2] * inv, o[h][dt][3] * inv};
                *reinterpret_cast<f32x4*>(dst + 16 * dt + 4 * g) = val;
            }
        }
    }
}

template <bool BF16, int D, bool SPLIT>
int launch_prefix(const AttnParams& p, hipStream_t stream) {
    const size_t lds = (size_t)kPfxStages * 2 * kTileN * D * 2;
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&prefix_attn_kernel<BF16, D, SPLIT>>();
        if (rc != FSTA_OK) return rc;
    }
    const int chunks = (p.nq + kPfxRows - 1) / kPfxRows;
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    if (chunks > 65535 || slices_per_xcd > 65535) return FSTA_EUNSUPPORTED;
    const dim3 grid((unsigned)(kXcds * p.key_splits), (unsigned)chunks, (unsigned)slices_per_xcd);
    hipLaunchKernelGGL((prefix_attn_kernel<BF16, D, SPLIT>), grid, dim3(kPfxWaves * 64), lds, stream, p);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

}  // namespace

// Runs of prefix keys [run * split_tiles, ...) x chunks of 128 query rows x (batch, head) slices ->
// partial results in slots 1 .. key_splits of p.part_o / p.part_lse.
int launch_attention_prefix(const AttnParams& p, int dtype, int head_dim, bool fast_pv, hipStream_t stream) {
    if ((uint64_t)p.nk * (uint64_t)head_dim * 2u > 0xffffffffull) return FSTA_EUNSUPPORTED;
    // bfloat16 weights go to the matrix cores as hi + lo pairs, as in the tree kernel: fed as single values they
    // leave errors of up to 1e-2 in O when one or two keys carry most of a row's weight (measured), whatever the
    // length of the prefix
    const bool split = dtype == FSTA_BF16 && !fast_pv;
    if (dtype == FSTA_F16) {
        if (head_dim == 128) return launch_prefix<false, 128, false>(p, stream);
        if (head_dim == 64) return launch_prefix<false, 64, false>(p, stream);
    } else if (dtype == FSTA_BF16) {
        if (head_dim == 128) return split ? launch_prefix<true, 128, true>(p, stream) : launch_prefix<true, 128, false>(p, stream);
        if (head_dim == 64) return split ? launch_prefix<true, 64, true>(p, stream) : launch_prefix<true, 64, false>(p, stream);
    }
    return FSTA_EUNSUPPORTED;
}

bool prefix_kernel_supported(int dtype, int head_dim) {
    return (dtype == FSTA_F16 || dtype == FSTA_BF16) && (head_dim == 64 || head_dim == 128);
}

}  // namespace fsta
