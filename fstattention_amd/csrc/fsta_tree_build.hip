// Draft-head probabilities -> parent array of the tree of the most probable candidate paths
// (a Medusa-style tree), in one workgroup and launch, so that a tree that changes every decoding
// step is built without leaving the device or the stream (the reference builds its trees on the
// host, utils.py:27-77; README.md:16 rebuilds the kernel inputs once per step).
//
// A candidate is a path of ranks (r1..rd), 1 <= d <= depths, 0 <= r < topk; it scores
// probs[0][r1] * probs[1][r2] * ... (float64, multiplied left to right).  Candidates are indexed
// by (depth, ranks) ascending: index = start[d] + value, value = the ranks read as a base-topk
// number.  The n-1 best candidates are kept, ties going to the smaller index; node 0 is the empty
// path, the kept candidates are numbered 1.. in index order (so parent < child), and the parent
// of a path is the path without its last rank.
//
//   1. scores of all candidates into LDS
//   2. the (n-1)-th largest score by radix selection on the bit patterns (up to 8 passes of 8 bits,
//      ending as soon as the candidates left all belong to the kept ones; non-negative doubles
//      order like their bit patterns)
//   3. "kept" flags (above the threshold, or equal to it and among the first ties), numbered by
//      a prefix sum over the candidate index
//   4. parent ids through the numbering of the parents' candidates
// When nearly all candidates sit on the last level (four heads of ten ranks: 10000 of 11110), that
// level is never stored: the (n-1)-th largest score of the shorter paths bounds the threshold from
// below, the last level is scored on the fly against that bound, and steps 2-4 run over the short
// list of paths that reach it (same result, a tenth of the keys; 18.5 -> 13.3 us for that shape).
#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kBuildThreads = 1024;
constexpr int kBuildWaves = kBuildThreads / 64;
constexpr int kBuildRows = 16;                                  // candidate c belongs to thread c % 1024, row c / 1024
constexpr int kBuildMaxCand = kBuildThreads * kBuildRows;       // 16384: 128 KB of scores
constexpr int kBuildMaxProbs = 1024;                            // depths * topk
constexpr int kBuildShort = 2048;                               // short list of the threshold search (scores and indices: 24 KB)
constexpr int kBuildWords = kBuildMaxCand / 32;                 // a bitmap over the candidate index: 512 words
// paths of the last level from which its part of the score array holds the short list and three bitmaps
constexpr int kBuildTailCand = (kBuildShort * 12 + 3 * kBuildWords * 4) / 8;

template <typename T>
__global__ __launch_bounds__(kBuildThreads) void medusa_tree_kernel(const T* __restrict__ probs, int depths, int topk,
                                                                    int n_cand, int keep, int64_t* __restrict__ parent,
                                                                    uint32_t* __restrict__ status) {
    asm volatile("" ::"s"(probs), "s"(depths), "s"(topk), "s"(n_cand), "s"(keep), "s"(parent), "s"(status));   // one batch of argument loads
    extern __shared__ __attribute__((aligned(16))) unsigned char build_s[];
    uint64_t* key_s = reinterpret_cast<uint64_t*>(build_s);                    // [n_cand] score bits, later node ids
    double* prob_s = reinterpret_cast<double*>(key_s + n_cand);                // [depths * topk]
    uint32_t* hist_s = reinterpret_cast<uint32_t*>(prob_s + depths * topk);    // [256] bytes; later counts per (row, wave)
    uint32_t* misc_s = hist_s + 256;   // [0] chosen byte, [1] candidates still wanted, [2] selection finished, [3] length of the short list
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int rows = (n_cand + kBuildThreads - 1) / kBuildThreads;

    if (keep == 0) {      // the root alone
        if (tid == 0) parent[0] = -1;
        return;
    }
    for (int e = tid; e < depths * topk; e += kBuildThreads) prob_s[e] = (double)probs[e];
    __syncthreads();

    // select(src, count, k): the k-th largest of src[0 .. count) and how many of the keys equal to it belong to the k
    // largest, by radix selection, 8 bits per pass from the top (non-negative doubles order like their bit
    // patterns); a pass ends the search as soon as every key left is wanted.
    uint64_t threshold = 0ull;
    uint32_t want = 0u;
    auto select = [&](const uint64_t* src, int count, uint32_t k) {
        const int src_rows = (count + kBuildThreads - 1) / kBuildThreads;
        uint64_t prefix = 0ull;        // the bytes of the threshold found so far (in place, lower bytes zero)
        uint32_t left = k;
        if (tid < 3) misc_s[tid] = 0u;
        for (int shift = 56; shift >= 0; shift -= 8) {
            if (tid < 256) hist_s[tid] = 0u;
            __syncthreads();
            const uint64_t high_mask = shift == 56 ? 0ull : ~0ull << (shift + 8);
#pragma unroll 1
            for (int r = 0; r < src_rows; ++r) {
                const int c = tid + r * kBuildThreads;
                const uint64_t key = c < count ? src[c] : 0ull;
                const bool in = c < count && (key & high_mask) == prefix;
                const uint32_t bin = (uint32_t)(key >> shift) & 255u;
                // The leading bytes of the scores are nearly all alike: 64 atomics of a wave would queue
                // on one or two words.  For up to two byte values one lane counts for all lanes that
                // hold it; what is left after that is spread over many words and goes lane by lane.
                uint64_t voters = __ballot(in);
#pragma unroll
                for (int round = 0; round < 2; ++round) {
                    if (voters != 0ull) {
                        const int leader = __ffsll((long long)voters) - 1;
                        const uint32_t first = __builtin_amdgcn_readlane(bin, leader);
                        const uint64_t same = __ballot(in && bin == first);
                        if (lane == leader) atomicAdd(&hist_s[first], (uint32_t)__popcll(same));
                        voters &= ~same;
                    }
                }
                if ((voters >> lane) & 1ull) atomicAdd(&hist_s[bin], 1u);
            }
            __syncthreads();
            if (tid < 64) {
                // lane l owns bins 255 - 4l .. 252 - 4l; counts accumulate from the largest byte down
                uint32_t mine[4], local = 0u;
#pragma unroll
                for (int b = 0; b < 4; ++b) { mine[b] = hist_s[255 - 4 * tid - b]; local += mine[b]; }
                uint32_t incl = local;
#pragma unroll
                for (int dlt = 1; dlt < 64; dlt <<= 1) {
                    const uint32_t up = __shfl_up(incl, dlt, 64);
                    if (tid >= dlt) incl += up;
                }
                uint32_t before = incl - local;       // candidates in larger bins
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    if (before < left && left <= before + mine[b]) {
                        misc_s[0] = (uint32_t)(255 - 4 * tid - b);
                        misc_s[1] = left - before;
                        // every candidate of this byte value is wanted: the lower bytes need no look
                        if (left - before == mine[b]) misc_s[2] = 1u;
                    }
                    before += mine[b];
                }
            }
            __syncthreads();
            prefix |= (uint64_t)misc_s[0] << shift;
            left = misc_s[1];
            // (uniform: everyone reads the flag between the same two barriers)
            if (misc_s[2] != 0u) break;   // threshold = the prefix with zero lower bytes, all `left` candidates from it up
        }
        __syncthreads();   // (the next search clears the words read above)
        threshold = prefix;
        want = left;
    };
    // Scores of the levels from `d` on, as long as they start below `limit`: a path's score is its prefix's score
    // times the probability of its last rank (the left-to-right product); one division by topk per candidate, done
    // as a multiplication by 2^32 / topk rounded up (exact below 2^32 / topk, i.e. for every index here).
    const uint32_t magic = (uint32_t)((0x100000000ull + (uint32_t)topk - 1u) / (uint32_t)max(topk, 1));
    int lvl = 0, start = 0, prev_start = 0, count = topk;      // the next level to score
    auto score_levels = [&](int limit) {
        for (; start < limit; ++lvl) {
            for (int v = tid; v < count; v += kBuildThreads) {
                const uint32_t q = __umulhi((uint32_t)v, magic);          // v / topk
                const uint32_t r = (uint32_t)v - q * (uint32_t)topk;
                const double head = lvl == 0 ? 1.0 : __longlong_as_double((long long)key_s[prev_start + q]);
                key_s[start + v] = (uint64_t)__double_as_longlong(head * prob_s[lvl * topk + r]);
            }
            __syncthreads();
            prev_start = start;
            start += count;
            count *= topk;
        }
    };

    // ---- many candidates, nearly all of them on the last level: the last level is never stored -----------------
    // The keep-th largest score of the shorter paths (the head: every level but the last) is a lower bound of the
    // threshold: the keep-th largest of any subset cannot exceed the keep-th largest of all.  The paths of the last
    // level are scored on the fly and only those at or above the bound join a short list, together with the head's;
    // the list contains every kept path, so the search over it finds the same threshold and the same number of kept
    // ties.  Kept paths are then numbered through a bitmap over the candidate index (ids in index order = bits below)
    // and their parents looked up in the same bitmap.  The tail of the score array, which the last level does not
    // use here, holds the list and the bitmaps.  A list that overflows sends the launch down the general way below.
    {
        int last = 1;
        for (int d = 0; d < depths && last <= kBuildMaxCand; ++d) last *= topk;     // paths of the last level
        const int n_head = n_cand - last;
        if (depths >= 2 && topk >= 2 && last >= kBuildTailCand && n_head >= keep && n_head <= kBuildShort) {
            uint64_t* skey_s = key_s + n_head;                                   // [kBuildShort] scores of the listed paths
            uint32_t* sidx_s = reinterpret_cast<uint32_t*>(skey_s + kBuildShort);   // [kBuildShort] their candidate indices
            uint32_t* kept_s = sidx_s + kBuildShort;       // [512] bitmap over the candidate index: kept
            uint32_t* tie_s = kept_s + kBuildWords;        // [512] equal to the threshold
            uint32_t* below_s = tie_s + kBuildWords;       // [512] bits set in the words before (of the bitmap scanned last)
            score_levels(n_head);
            select(key_s, n_head, (uint32_t)keep);
            const uint64_t bound = threshold;
            for (int w = tid; w < 2 * kBuildWords; w += kBuildThreads) kept_s[w] = 0u;       // kept and tie bitmaps
            if (tid == 0) misc_s[3] = 0u;
            __syncthreads();
            const uint64_t lanes_below = (1ull << lane) - 1ull;
            auto list = [&](bool take, uint64_t key, int index) {      // (called by whole waves)
                const uint64_t takers = __ballot(take);
                if (takers == 0ull) return;
                uint32_t base = 0u;
                if (lane == 0) base = atomicAdd(&misc_s[3], (uint32_t)__popcll(takers));
                base = __builtin_amdgcn_readfirstlane(base);
                const uint32_t pos = base + (uint32_t)__popcll(takers & lanes_below);
                if (take && pos < (uint32_t)kBuildShort) {
                    skey_s[pos] = key;
                    sidx_s[pos] = (uint32_t)index;
                }
            };
#pragma unroll 1
            for (int c0 = 0; c0 < n_head; c0 += kBuildThreads) {
                const int c = c0 + tid;
                const uint64_t key = c < n_head ? key_s[c] : 0ull;
                list(c < n_head && key >= bound, key, c);
            }
#pragma unroll 1
            for (int v0 = 0; v0 < last; v0 += kBuildThreads) {
                const int v = v0 + tid;
                const bool valid = v < last;
                const uint32_t q = __umulhi((uint32_t)(valid ? v : 0), magic);
                const uint32_t r = (uint32_t)(valid ? v : 0) - q * (uint32_t)topk;
                const double head = __longlong_as_double((long long)key_s[prev_start + q]);
                const uint64_t key = (uint64_t)__double_as_longlong(head * prob_s[lvl * topk + r]);
                list(valid && key >= bound, key, n_head + v);
            }
            __syncthreads();
            const int n_short = (int)misc_s[3];
            if (n_short <= kBuildShort) {       // (uniform)
                select(skey_s, n_short, (uint32_t)keep);
                // bitmaps: above the threshold -> kept; equal to it -> tie
                for (int e = tid; e < n_short; e += kBuildThreads) {
                    const uint64_t key = skey_s[e];
                    const uint32_t c = sidx_s[e];
                    if (key > threshold) atomicOr(&kept_s[c >> 5], 1u << (c & 31));
                    else if (key == threshold) atomicOr(&tie_s[c >> 5], 1u << (c & 31));
                }
                __syncthreads();
                // below_s[w] = bits set in words [0, w) of a bitmap: one wave, 8 words per lane
                auto count_below = [&](const uint32_t* bits) {
                    if (tid < 64) {
                        uint32_t mine[8], local = 0u;
#pragma unroll
                        for (int i = 0; i < 8; ++i) { mine[i] = (uint32_t)__popc(bits[8 * tid + i]); local += mine[i]; }
                        uint32_t incl = local;
#pragma unroll
                        for (int dlt = 1; dlt < 64; dlt <<= 1) {
                            const uint32_t up = __shfl_up(incl, dlt, 64);
                            if (tid >= dlt) incl += up;
                        }
                        uint32_t before = incl - local;
#pragma unroll
                        for (int i = 0; i < 8; ++i) { below_s[8 * tid + i] = before; before += mine[i]; }
                    }
                    __syncthreads();
                };
                auto rank_in = [&](const uint32_t* bits, uint32_t c) {      // bits set below position c
                    return below_s[c >> 5] + (uint32_t)__popc(bits[c >> 5] & ((1u << (c & 31)) - 1u));
                };
                // the first `want` ties in index order are kept as well
                count_below(tie_s);
                for (int e = tid; e < n_short; e += kBuildThreads) {
                    const uint32_t c = sidx_s[e];
                    if (skey_s[e] == threshold && rank_in(tie_s, c) < want) atomicOr(&kept_s[c >> 5], 1u << (c & 31));
                }
                __syncthreads();
                count_below(kept_s);
                // ids = 1 + kept paths below in index order; the parent of a path is the path without its last rank
                if (tid == 0) parent[0] = -1;
                bool broken = false;
                for (int e = tid; e < n_short; e += kBuildThreads) {
                    const uint32_t c = sidx_s[e];
                    if (!((kept_s[c >> 5] >> (c & 31)) & 1u)) continue;
                    int s0 = 0, cnt = topk, p0 = 0;
                    while ((int)c >= s0 + cnt) { p0 = s0; s0 += cnt; cnt *= topk; }
                    int64_t par = 0;      // paths of one rank hang off the root
                    if (s0 > 0) {
                        const uint32_t pc = (uint32_t)p0 + ((uint32_t)c - (uint32_t)s0) / (uint32_t)topk;
                        if ((kept_s[pc >> 5] >> (pc & 31)) & 1u) par = 1 + (int64_t)rank_in(kept_s, pc);
                        else broken = true;     // the parent path was not kept: probabilities above 1 or not numbers
                    }
                    parent[1 + rank_in(kept_s, c)] = par;
                }
                if (broken) atomicOr(status, FSTA_TREE_NOT_PREFIX_CLOSED);
                return;
            }
            // (the list overflowed: scores of more than kBuildShort paths reach the bound)
            __syncthreads();
        }
    }

    // ---- the general way: every score stored, the search over all of them -----------------------------------------
    // 1. scores, depth by depth
    if (topk == 1) {       // a single chain: one path per depth
        if (tid == 0) {
            double score = 1.0;
            for (int d = 0; d < depths; ++d) {
                score *= prob_s[d];
                key_s[d] = (uint64_t)__double_as_longlong(score);
            }
        }
        __syncthreads();
    } else {
        score_levels(n_cand);
    }

    // 2. threshold = the keep-th largest key, and how many of the keys equal to it are kept
    select(key_s, n_cand, (uint32_t)keep);

    // 3. numbering of the kept candidates in index order.  Index order = row by row, wave by wave,
    //    lane by lane: counts per (row, wave) from ballots (above the threshold | equal to it << 16),
    //    an exclusive scan over those 256 counts, and the lanes below within the wave.
    uint32_t* count_s = hist_s;
    __syncthreads();
    if (tid < 256 && tid >= rows * kBuildWaves) count_s[tid] = 0u;   // rows this launch does not have
#pragma unroll 1
    for (int k = 0; k < rows; ++k) {
        const int c = tid + k * kBuildThreads;
        const uint64_t key = c < n_cand ? key_s[c] : 0ull;
        const uint64_t over = __ballot(c < n_cand && key > threshold);
        const uint64_t tie = __ballot(c < n_cand && key == threshold);
        if (lane == 0) count_s[k * kBuildWaves + wave] = (uint32_t)__popcll(over) | ((uint32_t)__popcll(tie) << 16);
    }
    __syncthreads();
    if (tid < 64) {
        uint32_t mine[4], local = 0u;
#pragma unroll
        for (int b = 0; b < 4; ++b) { mine[b] = count_s[4 * tid + b]; local += mine[b]; }
        uint32_t incl = local;        // n_cand <= 16384: no carry between the halves
#pragma unroll
        for (int dlt = 1; dlt < 64; dlt <<= 1) {
            const uint32_t up = __shfl_up(incl, dlt, 64);
            if (tid >= dlt) incl += up;
        }
        uint32_t before = incl - local;
#pragma unroll
        for (int b = 0; b < 4; ++b) { count_s[4 * tid + b] = before; before += mine[b]; }
    }
    __syncthreads();
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll 1
    for (int k = 0; k < rows; ++k) {
        const int c = tid + k * kBuildThreads;
        const uint64_t key = c < n_cand ? key_s[c] : 0ull;
        const bool is_over = c < n_cand && key > threshold, is_tie = c < n_cand && key == threshold;
        const uint64_t over = __ballot(is_over);
        const uint64_t tie = __ballot(is_tie);
        const uint32_t base = count_s[k * kBuildWaves + wave];
        const uint32_t above_before = (base & 0xffffu) + (uint32_t)__popcll(over & below);
        const uint32_t equal_before = (base >> 16) + (uint32_t)__popcll(tie & below);
        // kept candidates before this one: those above the threshold and the kept ties
        const bool kept = is_over || (is_tie && equal_before < want);
        // node ids (0 = not kept) take the place of the scores
        if (c < n_cand) key_s[c] = kept ? 1u + above_before + min(equal_before, want) : 0u;
    }
    __syncthreads();

    // 4. parents
    if (tid == 0) parent[0] = -1;
    bool broken = false;
#pragma unroll 1
    for (int c = tid; c < n_cand; c += kBuildThreads) {
        const uint32_t id = (uint32_t)key_s[c];
        if (id == 0u) continue;
        int start = 0, count = topk, prev_start = 0;
        while (c >= start + count) { prev_start = start; start += count; count *= topk; }
        int64_t par = 0;      // paths of one rank hang off the root
        if (start > 0) {
            par = (int64_t)(uint32_t)key_s[prev_start + (c - start) / topk];
            if (par == 0) broken = true;     // the parent path was not kept: probabilities above 1 or not numbers
        }
        parent[id] = par;
    }
    if (broken) atomicOr(status, FSTA_TREE_NOT_PREFIX_CLOSED);
}


// ---- more candidates than one workgroup's LDS holds (up to kBigMaxCand) -----------------------------
// The same four steps over arrays in device memory (the caller's workspace), one launch per step and
// per radix pass; workgroup w owns candidates [4096 w, 4096 w + 4096), row k of it = candidates
// 4096 w + 1024 k + thread.  Everything is integer work on 8 bytes per candidate that stay in L2.
//   workspace: keys [n_cand] u64 (scores, later node ids) | hist [8][256] u32 | state [8] u32 |
//              counts [workgroups][2] u32 (above the threshold, equal to it)
constexpr int kBigRows = 4;
constexpr int kBigChunk = kBuildThreads * kBigRows;            // candidates per workgroup
constexpr int64_t kBigMaxCand = (int64_t)1 << 24;
constexpr int kBigPasses = 8;
// state words: [0] passes decided, [1] candidates still wanted, [2] selection finished, [4..5] threshold bytes found
struct BigLayout {
    uint64_t* keys;
    uint32_t* hist;
    uint32_t* state;
    uint32_t* counts;
};
__host__ __device__ inline size_t big_workspace_bytes(int64_t n_cand) {
    const int64_t wgs = (n_cand + kBigChunk - 1) / kBigChunk;
    return (size_t)n_cand * 8 + kBigPasses * 256 * 4 + 8 * 4 + (size_t)wgs * 2 * 4;
}
__host__ __device__ inline BigLayout big_layout(void* workspace, int64_t n_cand) {
    BigLayout l;
    l.keys = static_cast<uint64_t*>(workspace);
    l.hist = reinterpret_cast<uint32_t*>(l.keys + n_cand);
    l.state = l.hist + kBigPasses * 256;
    l.counts = l.state + 8;
    return l;
}

// 1. scores: every candidate multiplies its ranks' probabilities from the first rank on (the order of the
//    level-by-level products above and of the host builder); workgroup 0 also clears the histograms and the state
template <typename T>
__global__ __launch_bounds__(kBuildThreads) void big_scores_kernel(const T* __restrict__ probs, int depths, int topk,
                                                                   int n_cand, int keep, BigLayout w) {
    __shared__ double prob_s[kBuildMaxProbs];
    const int tid = threadIdx.x;
    for (int e = tid; e < depths * topk; e += kBuildThreads) prob_s[e] = (double)probs[e];
    if (blockIdx.x == 0) {
        for (int e = tid; e < kBigPasses * 256; e += kBuildThreads) w.hist[e] = 0u;
        if (tid < 8) w.state[tid] = tid == 1 ? (uint32_t)keep : 0u;
    }
    __syncthreads();
#pragma unroll 1
    for (int k = 0; k < kBigRows; ++k) {
        const int c = blockIdx.x * kBigChunk + k * kBuildThreads + tid;
        if (c >= n_cand) continue;
        int start = 0, count = topk, d = 0;
        while (c >= start + count) { start += count; count *= topk; ++d; }     // path of d + 1 ranks
        int v = c - start, pow = count;
        double score = 1.0;
        for (int i = 0; i <= d; ++i) {
            pow /= topk;
            const int r = v / pow;
            v -= r * pow;
            score *= prob_s[i * topk + r];
        }
        w.keys[c] = (uint64_t)__double_as_longlong(score);
    }
}

// The byte the previous pass decided on: lane l of wave 0 owns bins 255 - 4l .. 252 - 4l of its histogram.
// Returns (through LDS) the threshold bytes found so far, how many candidates are still wanted among
// the keys that share them, and whether the selection is complete.  Every workgroup computes the same.
__device__ __forceinline__ void big_decide(const BigLayout& w, int pass, int keep, uint32_t* sh /* [4] */) {
    // replays the decisions of passes 0 .. pass - 1 from their histograms
    const int tid = threadIdx.x;
    if (tid < 64) {
        uint64_t prefix = 0ull;
        uint32_t want = (uint32_t)keep, done = 0u;
        for (int q = 0; q < pass && !done; ++q) {
            const int shift = 56 - 8 * q;
            uint32_t mine[4], local = 0u;
#pragma unroll
            for (int b = 0; b < 4; ++b) { mine[b] = w.hist[q * 256 + 255 - 4 * tid - b]; local += mine[b]; }
            uint32_t incl = local;
#pragma unroll
            for (int dlt = 1; dlt < 64; dlt <<= 1) {
                const uint32_t up = __shfl_up(incl, dlt, 64);
                if (tid >= dlt) incl += up;
            }
            uint32_t before = incl - local;
            uint32_t byte = 0u, next_want = 0u, fin = 0u, hit = 0u;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                if (before < want && want <= before + mine[b]) {
                    hit = 1u;
                    byte = (uint32_t)(255 - 4 * tid - b);
                    next_want = want - before;
                    fin = next_want == mine[b] ? 1u : 0u;
                }
                before += mine[b];
            }
            const uint64_t who = __ballot(hit != 0u);          // exactly one lane
            const int src = __ffsll((long long)who) - 1;
            byte = __shfl(byte, src, 64);
            want = __shfl(next_want, src, 64);
            done = __shfl(fin, src, 64);
            prefix |= (uint64_t)byte << shift;
        }
        if (tid == 0) {
            sh[0] = (uint32_t)prefix;
            sh[1] = (uint32_t)(prefix >> 32);
            sh[2] = want;
            sh[3] = done;
        }
    }
    __syncthreads();
}

// 2. one radix pass: histogram of byte `pass` (from the top) over the keys that share the bytes found so far
__global__ __launch_bounds__(kBuildThreads) void big_hist_kernel(int n_cand, int keep, int pass, BigLayout w) {
    __shared__ uint32_t hist_s[256];
    __shared__ uint32_t sh[4];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    if (tid < 256) hist_s[tid] = 0u;
    big_decide(w, pass, keep, sh);
    if (sh[3] != 0u) return;                       // (uniform) the selection was complete before this pass
    const uint64_t prefix = (uint64_t)sh[0] | ((uint64_t)sh[1] << 32);
    const int shift = 56 - 8 * pass;
    const uint64_t high_mask = pass == 0 ? 0ull : ~0ull << (shift + 8);
#pragma unroll 1
    for (int k = 0; k < kBigRows; ++k) {
        const int c = blockIdx.x * kBigChunk + k * kBuildThreads + tid;
        const uint64_t key = c < n_cand ? w.keys[c] : 0ull;
        const bool in = c < n_cand && (key & high_mask) == prefix;
        const uint32_t bin = (uint32_t)(key >> shift) & 255u;
        uint64_t voters = __ballot(in);
#pragma unroll
        for (int round = 0; round < 2; ++round) {
            if (voters != 0ull) {
                const int leader = __ffsll((long long)voters) - 1;
                const uint32_t first = __builtin_amdgcn_readlane(bin, leader);
                const uint64_t same = __ballot(in && bin == first);
                if (lane == leader) atomicAdd(&hist_s[first], (uint32_t)__popcll(same));
                voters &= ~same;
            }
        }
        if ((voters >> lane) & 1ull) atomicAdd(&hist_s[bin], 1u);
    }
    __syncthreads();
    if (tid < 256 && hist_s[tid] != 0u) atomicAdd(&w.hist[pass * 256 + tid], hist_s[tid]);
}

// 3a. threshold known: kept candidates per workgroup (above the threshold, equal to it)
__global__ __launch_bounds__(kBuildThreads) void big_count_kernel(int n_cand, int keep, BigLayout w) {
    __shared__ uint32_t sh[4];
    __shared__ uint32_t over_s, tie_s;
    const int tid = threadIdx.x;
    if (tid == 0) { over_s = 0u; tie_s = 0u; }
    big_decide(w, kBigPasses, keep, sh);
    const uint64_t threshold = (uint64_t)sh[0] | ((uint64_t)sh[1] << 32);
    uint32_t over = 0u, tie = 0u;
#pragma unroll 1
    for (int k = 0; k < kBigRows; ++k) {
        const int c = blockIdx.x * kBigChunk + k * kBuildThreads + tid;
        const uint64_t key = c < n_cand ? w.keys[c] : 0ull;
        over += (uint32_t)__popcll(__ballot(c < n_cand && key > threshold));
        tie += (uint32_t)__popcll(__ballot(c < n_cand && key == threshold));
    }
    if ((tid & 63) == 0) { atomicAdd(&over_s, over); atomicAdd(&tie_s, tie); }
    __syncthreads();
    if (tid == 0) {
        w.counts[2 * blockIdx.x] = over_s;
        w.counts[2 * blockIdx.x + 1] = tie_s;
        if (blockIdx.x == 0) { w.state[4] = sh[0]; w.state[5] = sh[1]; w.state[1] = sh[2]; }
    }
}

// 3b. numbering in index order: kept candidates of the workgroups in front (sum of their counts), of the rows and
//     waves in front inside the workgroup, of the lanes below; node ids (0 = not kept) take the place of the scores
__global__ __launch_bounds__(kBuildThreads) void big_number_kernel(int n_cand, BigLayout w) {
    __shared__ uint32_t red_s[2][kBuildWaves];
    __shared__ uint32_t cnt_s[kBigRows * kBuildWaves];
    __shared__ uint32_t base_s[2];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const uint64_t threshold = (uint64_t)w.state[4] | ((uint64_t)w.state[5] << 32);
    const uint32_t want = w.state[1];
    // kept candidates in the workgroups in front of this one
    uint32_t over = 0u, tie = 0u;
    for (int g = tid; g < (int)blockIdx.x; g += kBuildThreads) { over += w.counts[2 * g]; tie += w.counts[2 * g + 1]; }
#pragma unroll
    for (int dlt = 32; dlt >= 1; dlt >>= 1) { over += __shfl_xor(over, dlt, 64); tie += __shfl_xor(tie, dlt, 64); }
    if (lane == 0) { red_s[0][wave] = over; red_s[1][wave] = tie; }
    uint64_t keys[kBigRows];
#pragma unroll
    for (int k = 0; k < kBigRows; ++k) {
        const int c = blockIdx.x * kBigChunk + k * kBuildThreads + tid;
        keys[k] = c < n_cand ? w.keys[c] : 0ull;
        const uint64_t o = __ballot(c < n_cand && keys[k] > threshold);
        const uint64_t t = __ballot(c < n_cand && keys[k] == threshold);
        if (lane == 0) cnt_s[k * kBuildWaves + wave] = (uint32_t)__popcll(o) | ((uint32_t)__popcll(t) << 16);
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t a = 0u, b = 0u;
        for (int i = 0; i < kBuildWaves; ++i) { a += red_s[0][i]; b += red_s[1][i]; }
        base_s[0] = a;
        base_s[1] = b;
    }
    if (tid == 64) {       // exclusive scan of the 64 (row, wave) counts: at most 64 candidates each, 16 bits hold a workgroup's
        uint32_t run = 0u;
        for (int i = 0; i < kBigRows * kBuildWaves; ++i) { const uint32_t x = cnt_s[i]; cnt_s[i] = run; run += x; }
    }
    __syncthreads();
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
    for (int k = 0; k < kBigRows; ++k) {
        const int c = blockIdx.x * kBigChunk + k * kBuildThreads + tid;
        const bool is_over = c < n_cand && keys[k] > threshold, is_tie = c < n_cand && keys[k] == threshold;
        const uint64_t o = __ballot(is_over);
        const uint64_t t = __ballot(is_tie);
        const uint32_t base = cnt_s[k * kBuildWaves + wave];
        const uint32_t above_before = base_s[0] + (base & 0xffffu) + (uint32_t)__popcll(o & below);
        const uint32_t equal_before = base_s[1] + (base >> 16) + (uint32_t)__popcll(t & below);
        const bool kept = is_over || (is_tie && equal_before < want);
        if (c < n_cand) w.keys[c] = kept ? 1u + above_before + min(equal_before, want) : 0u;
    }
}

// 4. parents through the numbering of the parents' candidates
__global__ __launch_bounds__(kBuildThreads) void big_parents_kernel(int topk, int n_cand, BigLayout w,
                                                                    int64_t* __restrict__ parent, uint32_t* __restrict__ status) {
    const int tid = threadIdx.x;
    if (blockIdx.x == 0 && tid == 0) parent[0] = -1;
    bool broken = false;
#pragma unroll 1
    for (int k = 0; k < kBigRows; ++k) {
        const int c = blockIdx.x * kBigChunk + k * kBuildThreads + tid;
        if (c >= n_cand) continue;
        const uint32_t id = (uint32_t)w.keys[c];
        if (id == 0u) continue;
        int start = 0, count = topk, prev_start = 0;
        while (c >= start + count) { prev_start = start; start += count; count *= topk; }
        int64_t par = 0;
        if (start > 0) {
            par = (int64_t)(uint32_t)w.keys[prev_start + (c - start) / topk];
            if (par == 0) broken = true;
        }
        parent[id] = par;
    }
    if (broken) atomicOr(status, FSTA_TREE_NOT_PREFIX_CLOSED);
}

template <typename T>
int launch_big_tree(const T* probs, int depths, int topk, int64_t n_cand, int n_nodes, int64_t* parent, uint32_t* status,
                    void* workspace, hipStream_t s) {
    const BigLayout w = big_layout(workspace, n_cand);
    const unsigned wgs = (unsigned)((n_cand + kBigChunk - 1) / kBigChunk);
    const int keep = n_nodes - 1;
    hipLaunchKernelGGL(big_scores_kernel<T>, dim3(wgs), dim3(kBuildThreads), 0, s, probs, depths, topk, (int)n_cand, keep, w);
    for (int pass = 0; pass < kBigPasses; ++pass)
        hipLaunchKernelGGL(big_hist_kernel, dim3(wgs), dim3(kBuildThreads), 0, s, (int)n_cand, keep, pass, w);
    hipLaunchKernelGGL(big_count_kernel, dim3(wgs), dim3(kBuildThreads), 0, s, (int)n_cand, keep, w);
    hipLaunchKernelGGL(big_number_kernel, dim3(wgs), dim3(kBuildThreads), 0, s, (int)n_cand, w);
    hipLaunchKernelGGL(big_parents_kernel, dim3(wgs), dim3(kBuildThreads), 0, s, topk, (int)n_cand, w, parent, status);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

}  // namespace
}  // namespace fsta

using namespace fsta;

extern "C" int fsta_medusa_tree(const void* probs, int32_t probs_dtype, int32_t depths, int32_t topk, int32_t n_nodes,
                                int64_t* parent, uint32_t* status, void* stream) {
    if (depths < 1 || topk < 1 || n_nodes < 1)
        return fail(FSTA_EINVAL, "fsta_medusa_tree: depths=%d topk=%d n_nodes=%d", depths, topk, n_nodes);
    if (probs_dtype != FSTA_F32 && probs_dtype != FSTA_F64)
        return fail(FSTA_EINVAL, "fsta_medusa_tree: probs_dtype=%d (float32 or float64)", probs_dtype);
    int64_t n_cand = 0, level = 1;
    for (int d = 0; d < depths; ++d) {
        level *= topk;
        n_cand += level;
        if (n_cand > kBuildMaxCand) break;
    }
    if (n_cand > kBuildMaxCand || (int64_t)depths * topk > kBuildMaxProbs)
        return fail(FSTA_EUNSUPPORTED, "fsta_medusa_tree: depths=%d topk=%d give more than %d candidate paths",
                    depths, topk, kBuildMaxCand);
    if (n_nodes - 1 > n_cand)
        return fail(FSTA_EINVAL, "fsta_medusa_tree: n_nodes=%d but only %lld candidate paths (+ the root)", n_nodes,
                    (long long)n_cand);
    if (!probs || !parent || !status) return fail(FSTA_EINVAL, "fsta_medusa_tree: null pointer");
    const size_t lds = (size_t)n_cand * 8 + (size_t)depths * topk * 8 + (256 + 4) * 4;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (probs_dtype == FSTA_F32) {
        if (lds > 64 * 1024) {
            const int rc = allow_full_lds<&medusa_tree_kernel<float>>();
            if (rc != FSTA_OK) return rc;
        }
        hipLaunchKernelGGL(medusa_tree_kernel<float>, dim3(1), dim3(kBuildThreads), lds, s,
                           static_cast<const float*>(probs), depths, topk, (int)n_cand, n_nodes - 1, parent, status);
    } else {
        if (lds > 64 * 1024) {
            const int rc = allow_full_lds<&medusa_tree_kernel<double>>();
            if (rc != FSTA_OK) return rc;
        }
        hipLaunchKernelGGL(medusa_tree_kernel<double>, dim3(1), dim3(kBuildThreads), lds, s,
                           static_cast<const double*>(probs), depths, topk, (int)n_cand, n_nodes - 1, parent, status);
    }
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

namespace {

// candidate paths of (depths, topk), or -1 beyond `limit`
int64_t count_candidates(int depths, int topk, int64_t limit) {
    int64_t n_cand = 0, level = 1;
    for (int d = 0; d < depths; ++d) {
        level *= topk;
        n_cand += level;
        if (n_cand > limit) return -1;
    }
    return n_cand;
}

}  // namespace

extern "C" size_t fsta_medusa_workspace_bytes(int32_t depths, int32_t topk) {
    if (depths < 1 || topk < 1) return 0;
    const int64_t n_cand = count_candidates(depths, topk, kBigMaxCand);
    if (n_cand < 0 || n_cand <= kBuildMaxCand) return 0;
    return big_workspace_bytes(n_cand);
}

extern "C" int fsta_medusa_tree_ws(const void* probs, int32_t probs_dtype, int32_t depths, int32_t topk, int32_t n_nodes,
                                   int64_t* parent, uint32_t* status, void* workspace, size_t workspace_bytes,
                                   void* stream) {
    if (depths < 1 || topk < 1 || n_nodes < 1)
        return fail(FSTA_EINVAL, "fsta_medusa_tree_ws: depths=%d topk=%d n_nodes=%d", depths, topk, n_nodes);
    const int64_t small = count_candidates(depths, topk, kBuildMaxCand);
    if (small >= 0) return fsta_medusa_tree(probs, probs_dtype, depths, topk, n_nodes, parent, status, stream);
    if (probs_dtype != FSTA_F32 && probs_dtype != FSTA_F64)
        return fail(FSTA_EINVAL, "fsta_medusa_tree_ws: probs_dtype=%d (float32 or float64)", probs_dtype);
    const int64_t n_cand = count_candidates(depths, topk, kBigMaxCand);
    if (n_cand < 0 || (int64_t)depths * topk > kBuildMaxProbs)
        return fail(FSTA_EUNSUPPORTED, "fsta_medusa_tree_ws: depths=%d topk=%d give more than %lld candidate paths",
                    depths, topk, (long long)kBigMaxCand);
    if (n_nodes - 1 > n_cand)
        return fail(FSTA_EINVAL, "fsta_medusa_tree_ws: n_nodes=%d but only %lld candidate paths (+ the root)", n_nodes,
                    (long long)n_cand);
    if (!probs || !parent || !status) return fail(FSTA_EINVAL, "fsta_medusa_tree_ws: null pointer");
    if (!workspace || workspace_bytes < big_workspace_bytes(n_cand))
        return fail(FSTA_EINVAL, "fsta_medusa_tree_ws: %lld candidate paths need a workspace of %zu bytes (given: %zu)",
                    (long long)n_cand, big_workspace_bytes(n_cand), workspace ? workspace_bytes : (size_t)0);
    if (misaligned(workspace, 8) || misaligned(parent, 8) || misaligned(status, 4) ||
        misaligned(probs, probs_dtype == FSTA_F64 ? 8 : 4))
        return fail(FSTA_EINVAL, "fsta_medusa_tree_ws: workspace and parent must be 8-byte aligned, probs and status to their element size");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n_nodes == 1) {      // the root alone: the single-workgroup kernel's first branch
        hipLaunchKernelGGL(medusa_tree_kernel<float>, dim3(1), dim3(kBuildThreads), 0, s, static_cast<const float*>(probs),
                           depths, topk, 0, 0, parent, status);
        FSTA_HIP_OK(hipGetLastError());
        return FSTA_OK;
    }
    if (probs_dtype == FSTA_F32)
        return launch_big_tree(static_cast<const float*>(probs), depths, topk, n_cand, n_nodes, parent, status, workspace, s);
    return launch_big_tree(static_cast<const double*>(probs), depths, topk, n_cand, n_nodes, parent, status, workspace, s);
}

