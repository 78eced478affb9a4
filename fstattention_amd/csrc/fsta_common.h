// Shared declarations of libfsta's translation units (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/fsta.h"

namespace fsta {

constexpr float kLog2e = 1.4426950408889634f;

// Block plan (include/fsta.h, fsta_block_plan_bytes): per query block a record of 32-bit words,
//   header [kPlanHeaderWords] | ancestor keys [32 * tiles] | per 32 rows: leaf keys [32], mask words [tiles][32]
constexpr int kPlanHeaderWords = 8;   // [0] ancestor count, [4..7] leaf validity per 32 rows
constexpr int kPlanLeafValid = 4;
struct PlanLayout {
    int tiles;          // ancestor tiles of 32 slots
    int common_words;   // header + ancestor keys
    int group_words;    // one group of 32 rows: leaf keys + mask words
    int block_words;    // whole record
};
__host__ __device__ inline PlanLayout plan_layout(int block_m, int max_anc) {
    PlanLayout l;
    l.tiles = (max_anc + 31) / 32;
    l.common_words = kPlanHeaderWords + 32 * l.tiles;
    l.group_words = 32 * (1 + l.tiles);
    l.block_words = l.common_words + (block_m / 32) * l.group_words;
    return l;
}
inline bool plan_block_size_ok(int block_m) { return block_m == 32 || block_m == 64 || block_m == 128; }

// Argument block of every attention kernel.  Plain data, passed by value.
struct AttnParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    float* lse;                   // may be null
    const int64_t* ancestor_idx;  // [nb, max_anc]
    const uint32_t* mask_bits;    // [nb, mask_words, block_m]
    const int32_t* anc_count;     // [nb]
    const int64_t* leaf_idx;      // [nb, block_m]
    const uint32_t* plan;         // block plan of the same lists, or null
    int32_t key_shift;            // added to the plan's keys
    int32_t nq, nk, prefix;       // prefix = nk - nq
    int32_t block_m, max_anc, mask_words, nb;
    int32_t heads_total;          // batch * heads
    int32_t out_f32;              // o is float32 instead of the input type
    float scale_log2e;            // sm_scale * log2(e)
    // Key splits of the shared prefix (narrow matrix-core kernel only; 1 = off): workgroup s of a
    // block takes prefix tiles [s * split_tiles, (s + 1) * split_tiles) and writes a normalised
    // float32 partial result part_o[s][batch*heads][nq][D] with log-sum-exp part_lse[s][batch*heads][nq].
    int32_t key_splits, split_tiles;
    int32_t share_tiles;          // tuning: wave pairs of a row group always share the tiles, never the head dimension
    float* part_o;
    float* part_lse;
    // With merge_parts > 0 the kernel with key runs writes no partial result of its own: it joins its (tree) part
    // with the partial results in slots 1 .. merge_parts of part_o / part_lse (the dense prefix kernel's, already
    // written on the stream) and stores the final rows in o / lse.
    int32_t merge_parts;
    int32_t dry_run;              // launchers return what they would return without launching anything
    int32_t stream_mode;          // streaming kernel (workgroups that walk a list of blocks): 1 = wherever the shape allows, else never (it is slower than one workgroup per block on every shape measured)
    // 8-bit K/V (fsta_attention_fwd_kv8): k and v hold OCP e4m3 bytes; one float32 scale per
    // (batch, head) slice each, or null for 1
    const float* k_scale;
    const float* v_scale;
};

// true when a non-null pointer is not a multiple of `bytes` (null pointers are judged elsewhere)
inline bool misaligned(const void* ptr, unsigned bytes) { return reinterpret_cast<uintptr_t>(ptr) % bytes != 0; }

// Records a message for fsta_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

#define FSTA_HIP_OK(expr)                                                          \
    do {                                                                           \
        hipError_t err__ = (expr);                                                 \
        if (err__ != hipSuccess)                                                   \
            return ::fsta::fail(FSTA_EHIP, "%s: %s", #expr, hipGetErrorString(err__)); \
    } while (0)

// Raises the dynamic-LDS limit of one kernel to what the 160 KB of a gfx950 CU leave, once per device and
// process (the attribute call costs microseconds on the host; setting it twice in a race is harmless).
template <auto Kernel>
int allow_full_lds() {
    static bool done[64] = {};
    int dev = 0;
    FSTA_HIP_OK(hipGetDevice(&dev));
    const bool tracked = dev >= 0 && dev < 64;
    if (tracked && done[dev]) return FSTA_OK;
    // static LDS of the kernel (its own or a library routine's) counts against the same 160 KB
    hipFuncAttributes attr;
    FSTA_HIP_OK(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(Kernel)));
    FSTA_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    160 * 1024 - (int)attr.sharedSizeBytes));
    if (tracked) done[dev] = true;
    return FSTA_OK;
}

// Which attention kernel the calling thread launched last (fsta_last_attention_kernel): the kernel's
// name and up to seven template arguments, kept as numbers and turned into text only when asked for.
struct LaunchNote {
    const char* kernel;   // string literal
    const char* first;    // first template argument as text, e.g. "true" or "float"
    int args[6];
    int n_args;
    unsigned bool_args;   // bit i: args[i] is a bool template argument
    int half_blocks, early_start;   // launch options of the narrow matrix-core kernel
};
void note_launch(const LaunchNote& note);

// launchers, one per translation unit
int launch_attention_generic(const AttnParams& p, int dtype, int head_dim, hipStream_t stream);
int launch_attention_mfma(const AttnParams& p, int dtype, int head_dim, bool fast_pv,
                          hipStream_t stream);
int launch_attention_mfma16(const AttnParams& p, int dtype, int head_dim, bool fast_pv,
                            hipStream_t stream);
// dense shared prefix, run by run, into slots 1 .. key_splits of p.part_o / p.part_lse
int launch_attention_prefix(const AttnParams& p, int dtype, int head_dim, bool fast_pv, hipStream_t stream);
bool prefix_kernel_supported(int dtype, int head_dim);
// workgroups that stay and walk a list of (block, slice) pairs; FSTA_EUNSUPPORTED where the launch has too few pairs or a prefix
int launch_attention_stream(const AttnParams& p, int dtype, int head_dim, bool fast_pv, hipStream_t stream);
int launch_attention_mfma16_kv8(const AttnParams& p, int dtype, int head_dim, hipStream_t stream);
bool mfma_supported(int dtype, int head_dim, int block_m);
// joins `splits` partial results (layout of AttnParams::part_o / part_lse) into o (and lse, may be null)
int launch_merge_splits(const float* part_o, const float* part_lse, int splits, int64_t rows, int head_dim,
                        void* o, int out_dtype, float* lse, hipStream_t stream);

// ---- element conversion -------------------------------------------------
__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(__half x) { return __half2float(x); }
__device__ __forceinline__ float to_float(__hip_bfloat16 x) { return __bfloat162float(x); }

template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ __half from_float<__half>(float x) { return __float2half_rn(x); }
template <> __device__ __forceinline__ __hip_bfloat16 from_float<__hip_bfloat16>(float x) {
    return __float2bfloat16(x);
}

}  // namespace fsta
