// extern "C" surface of libfsta: argument validation, error text, kernel dispatch.
#include <cstdarg>
#include <cstdio>

#include "fsta_common.h"

namespace fsta {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

static thread_local LaunchNote g_note = {nullptr, "", {0, 0, 0, 0, 0, 0}, 0, 0u, 0, 0};
static thread_local char g_note_text[192] = "";

void note_launch(const LaunchNote& note) { g_note = note; }

}  // namespace fsta

using namespace fsta;

extern "C" const char* fsta_last_attention_kernel(void) {
    if (!g_note.kernel) return "";
    int len = snprintf(g_note_text, sizeof(g_note_text), "%s<%s", g_note.kernel, g_note.first);
    for (int i = 0; i < g_note.n_args && len < (int)sizeof(g_note_text); ++i)
        len += (g_note.bool_args >> i) & 1u
                   ? snprintf(g_note_text + len, sizeof(g_note_text) - len, ", %s", g_note.args[i] ? "true" : "false")
                   : snprintf(g_note_text + len, sizeof(g_note_text) - len, ", %d", g_note.args[i]);
    if (len < (int)sizeof(g_note_text))
        snprintf(g_note_text + len, sizeof(g_note_text) - len, ">%s%s", g_note.half_blocks ? " half-blocks" : "",
                 g_note.early_start ? " early-start" : "");
    return g_note_text;
}

extern "C" int fsta_abi_version(void) { return FSTA_ABI_VERSION; }

extern "C" const char* fsta_last_error(void) { return g_error; }

namespace {

constexpr int kKeyTile = 32;        // keys per tile of the attention kernels
constexpr int kMinRunTiles = 8;     // shortest run of prefix tiles worth a workgroup of its own
constexpr int kTargetGroups = 512;  // two workgroups per CU
constexpr int kDenseMinRunTiles = 16;   // the same for the dense prefix kernel, whose partial results the tree part's launch reads back
                                        // (2048 keys: 4 runs 33.7 us, 8 runs 38.1; 4096 keys: 4 and 8 runs alike)

// How the shared prefix is cut for a launch of the narrow matrix-core kernel: number of runs
// (1 = no split) and prefix tiles per run.  Depends on the shape and flags only, so that the
// workspace query and the launch agree.
int plan_key_splits(int64_t slices, int nq, int nk, int head_dim, int dtype, int block_m, float sm_scale,
                    uint32_t flags, int* split_tiles) {
    const int tiles = (nk - nq + kKeyTile - 1) / kKeyTile;
    *split_tiles = tiles;
    if (tiles < 2 || slices <= 0 || nq <= 0) return 1;
    if ((flags & (FSTA_FLAG_GENERIC | FSTA_FLAG_WIDE_WAVES)) || !(sm_scale > 0.f) ||
        !mfma_supported(dtype, head_dim, block_m))
        return 1;
    const int forced = (int)((flags >> 8) & 0xffu);
    int64_t want = forced;
    if (!forced) {
        const int64_t groups = ((slices + 7) / 8) * 8 * ((nq + block_m - 1) / block_m);
        want = (kTargetGroups + groups - 1) / groups;
        if (want > tiles / kMinRunTiles) want = tiles / kMinRunTiles;
    }
    if (want > tiles) want = tiles;
    if (want > 255) want = 255;
    if (want <= 1) return 1;
    const int per = (int)((tiles + want - 1) / want);
    *split_tiles = per;
    return (tiles + per - 1) / per;
}

size_t key_split_bytes(int splits, int64_t slices, int nq, int head_dim) {
    return (size_t)splits * (size_t)slices * (size_t)nq * (size_t)(head_dim + 1) * sizeof(float);
}

constexpr int kDenseMinKeys = 2048;   // shortest prefix handed to the dense prefix kernel (below: two more launches cost more than they save)
constexpr int kDenseRows = 128;       // query rows per workgroup of that kernel

// Whether (and how) the prefix goes to the dense prefix kernel: number of key runs (0 = not at all) and
// prefix tiles per run.  The tree part then takes one more workspace slot.  Shape and flags only.
int plan_dense_prefix(int64_t slices, int nq, int nk, int head_dim, int dtype, int block_m, float sm_scale,
                      uint32_t flags, int* split_tiles) {
    const int prefix = nk - nq;
    if (slices <= 0 || nq <= 0 || prefix < kDenseMinKeys) return 0;
    if ((flags & (FSTA_FLAG_GENERIC | FSTA_FLAG_WIDE_WAVES)) || !(sm_scale > 0.f) ||
        !mfma_supported(dtype, head_dim, block_m) || !prefix_kernel_supported(dtype, head_dim))
        return 0;
    const int forced = (int)((flags >> 8) & 0xffu);
    if (forced == 1) return 0;        // "never split": the prefix stays in the tree kernel's own loop
    const int tiles = (prefix + kKeyTile - 1) / kKeyTile;
    int64_t want = forced;
    if (!forced) {
        const int64_t groups = ((slices + 7) / 8) * 8 * ((nq + kDenseRows - 1) / kDenseRows);
        want = (kTargetGroups + groups - 1) / groups;
        if (want > tiles / kDenseMinRunTiles) want = tiles / kDenseMinRunTiles;
        if (want < 1) want = 1;
    }
    if (want > tiles) want = tiles;
    if (want > 254) want = 254;
    const int per = (int)((tiles + want - 1) / want);
    *split_tiles = per;
    return (tiles + per - 1) / per;
}

}  // namespace

extern "C" size_t fsta_attention_workspace_bytes(int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                                                 int32_t head_dim, int32_t dtype, int32_t block_m,
                                                 int32_t max_ancestors, float sm_scale, uint32_t flags) {
    (void)max_ancestors;
    if (batch <= 0 || heads <= 0 || nq <= 0 || nk <= nq || block_m <= 0) return 0;
    int split_tiles = 0;
    const int64_t slices = (int64_t)batch * heads;
    const int runs = plan_dense_prefix(slices, nq, nk, head_dim, dtype, block_m, sm_scale, flags, &split_tiles);
    if (runs > 0) return key_split_bytes(runs + 1, slices, nq, head_dim);
    const int splits = plan_key_splits(slices, nq, nk, head_dim, dtype, block_m, sm_scale, flags, &split_tiles);
    return splits > 1 ? key_split_bytes(splits, slices, nq, head_dim) : 0;
}

extern "C" int fsta_attention_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                                  const int64_t* ancestor_idx, const uint32_t* mask_bits,
                                  const int32_t* anc_count, const int64_t* leaf_idx,
                                  const uint32_t* block_plan, int32_t plan_key_shift,
                                  int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                                  int32_t head_dim, int32_t dtype, int32_t out_dtype,
                                  int32_t block_m, int32_t max_ancestors, int32_t num_blocks,
                                  float sm_scale, uint32_t flags, void* stream) {
    return fsta_attention_fwd_ws(q, k, v, o, lse, ancestor_idx, mask_bits, anc_count, leaf_idx, block_plan,
                                 plan_key_shift, batch, heads, nq,
                                 nk, head_dim, dtype, out_dtype, block_m, max_ancestors, num_blocks, sm_scale,
                                 flags, nullptr, 0, stream);
}

extern "C" int fsta_attention_fwd_ws(const void* q, const void* k, const void* v, void* o, float* lse,
                                     const int64_t* ancestor_idx, const uint32_t* mask_bits,
                                     const int32_t* anc_count, const int64_t* leaf_idx,
                                     const uint32_t* block_plan, int32_t plan_key_shift,
                                     int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                                     int32_t head_dim, int32_t dtype, int32_t out_dtype,
                                     int32_t block_m, int32_t max_ancestors, int32_t num_blocks,
                                     float sm_scale, uint32_t flags, void* workspace, size_t workspace_bytes,
                                     void* stream) {
    if (batch < 0 || heads < 0 || nq < 0 || nk < nq)
        return fail(FSTA_EINVAL, "fsta_attention_fwd: batch=%d heads=%d nq=%d nk=%d (need nk >= nq >= 0)",
                    batch, heads, nq, nk);
    if (dtype != FSTA_F32 && dtype != FSTA_F16 && dtype != FSTA_BF16)
        return fail(FSTA_EINVAL, "fsta_attention_fwd: dtype=%d", dtype);
    if (out_dtype != dtype && out_dtype != FSTA_F32)
        return fail(FSTA_EINVAL, "fsta_attention_fwd: out_dtype=%d must equal dtype=%d or be float32",
                    out_dtype, dtype);
    if (head_dim != 16 && head_dim != 32 && head_dim != 64 && head_dim != 128)
        return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd: head_dim=%d (supported: 16, 32, 64, 128)", head_dim);
    if (block_m != 16 && block_m != 32 && block_m != 64 && block_m != 128)
        return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd: block_m=%d (supported: 16, 32, 64, 128)", block_m);
    if (max_ancestors < 1)
        return fail(FSTA_EINVAL, "fsta_attention_fwd: max_ancestors=%d", max_ancestors);
    if (num_blocks != (nq + block_m - 1) / block_m)
        return fail(FSTA_EINVAL, "fsta_attention_fwd: num_blocks=%d but ceil(nq=%d / block_m=%d) = %d",
                    num_blocks, nq, block_m, (nq + block_m - 1) / block_m);
    const int64_t slices = (int64_t)batch * heads;
    if (slices > 65535)
        return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd: batch*heads=%lld > 65535", (long long)slices);
    if (slices == 0 || nq == 0) return FSTA_OK;
    if (!q || !k || !v || !o || !ancestor_idx || !mask_bits || !leaf_idx)
        return fail(FSTA_EINVAL, "fsta_attention_fwd: null pointer");
    // rows and plan records are moved 16 bytes at a time, list entries 8, mask words and counts 4
    if (misaligned(q, 16) || misaligned(k, 16) || misaligned(v, 16) || misaligned(o, 16))
        return fail(FSTA_EINVAL, "fsta_attention_fwd: q, k, v and o must be 16-byte aligned");
    if (misaligned(block_plan, 16))
        return fail(FSTA_EINVAL, "fsta_attention_fwd: block_plan must be 16-byte aligned");
    if (misaligned(ancestor_idx, 8) || misaligned(leaf_idx, 8))
        return fail(FSTA_EINVAL, "fsta_attention_fwd: ancestor_idx and leaf_idx must be 8-byte aligned");
    if (misaligned(mask_bits, 4) || misaligned(anc_count, 4) || misaligned(lse, 4))
        return fail(FSTA_EINVAL, "fsta_attention_fwd: mask_bits, anc_count and lse must be 4-byte aligned");
    if (block_plan && (plan_key_shift < 0 || plan_key_shift > nk))
        return fail(FSTA_EINVAL, "fsta_attention_fwd: plan_key_shift=%d outside [0, nk=%d]", plan_key_shift, nk);

    AttnParams p;
    p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
    p.ancestor_idx = ancestor_idx; p.mask_bits = mask_bits; p.anc_count = anc_count;
    p.leaf_idx = leaf_idx;
    p.plan = plan_block_size_ok(block_m) ? block_plan : nullptr;
    p.key_shift = plan_key_shift;
    p.nq = nq; p.nk = nk; p.prefix = nk - nq;
    p.block_m = block_m; p.max_anc = max_ancestors; p.mask_words = fsta_mask_words(max_ancestors);
    p.nb = num_blocks;
    p.heads_total = (int32_t)slices;
    p.out_f32 = (out_dtype == FSTA_F32) ? 1 : 0;
    p.scale_log2e = sm_scale * kLog2e;
    p.key_splits = 1; p.split_tiles = 0; p.part_o = nullptr; p.part_lse = nullptr;
    p.share_tiles = (flags & FSTA_FLAG_SHARE_TILES) ? 1 : 0;
    p.k_scale = nullptr; p.v_scale = nullptr;
    p.merge_parts = 0; p.dry_run = 0;
    p.stream_mode = (flags & FSTA_FLAG_STREAM) ? 1 : 0;

    hipStream_t s = static_cast<hipStream_t>(stream);
    if (workspace && p.plan) {
        // a long prefix goes to the dense prefix kernel, run by run (slots 1 .. runs of the workspace); the tree
        // kernel then does the tree part and, in its epilogue, joins it with those partial results into o / lse
        int run_tiles = 0;
        const int runs = plan_dense_prefix(slices, nq, nk, head_dim, dtype, block_m, sm_scale, flags, &run_tiles);
        if (runs > 0 && workspace_bytes >= key_split_bytes(runs + 1, slices, nq, head_dim)) {
            if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
                return fail(FSTA_EINVAL, "fsta_attention_fwd_ws: workspace must be 16-byte aligned");
            const bool fast_pv = (flags & FSTA_FLAG_FAST_PV) != 0;
            AttnParams pt = p;
            pt.part_o = static_cast<float*>(workspace);
            pt.part_lse = pt.part_o + (size_t)(runs + 1) * slices * nq * head_dim;
            pt.key_splits = 1;
            pt.split_tiles = 0;        // no prefix tile for the tree kernel
            pt.merge_parts = runs;
            pt.dry_run = 1;            // (would the tree kernel take this shape? asked before anything is launched)
            int rc = launch_attention_mfma16(pt, dtype, head_dim, fast_pv, s);
            if (rc == FSTA_OK) {
                AttnParams pp = pt;
                pp.dry_run = 0;
                pp.merge_parts = 0;
                pp.key_splits = runs;
                pp.split_tiles = run_tiles;
                rc = launch_attention_prefix(pp, dtype, head_dim, fast_pv, s);
                if (rc != FSTA_OK) return rc;
                pt.dry_run = 0;
                return launch_attention_mfma16(pt, dtype, head_dim, fast_pv, s);
            }
            if (rc != FSTA_EUNSUPPORTED) return rc;
            // (ancestor lists too long for the kernel with key runs: the launches below)
        }
        int split_tiles = 0;
        // (a workspace too small for what fsta_attention_workspace_bytes asked for: no split of any kind)
        const int splits = runs > 0 ? 1 : plan_key_splits(slices, nq, nk, head_dim, dtype, block_m, sm_scale, flags, &split_tiles);
        if (splits > 1 && workspace_bytes >= key_split_bytes(splits, slices, nq, head_dim)) {
            if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
                return fail(FSTA_EINVAL, "fsta_attention_fwd_ws: workspace must be 16-byte aligned");
            AttnParams ps = p;
            ps.key_splits = splits;
            ps.split_tiles = split_tiles;
            ps.part_o = static_cast<float*>(workspace);
            ps.part_lse = ps.part_o + (size_t)splits * slices * nq * head_dim;
            const int rc = launch_attention_mfma16(ps, dtype, head_dim, (flags & FSTA_FLAG_FAST_PV) != 0, s);
            if (rc == FSTA_OK)
                return launch_merge_splits(ps.part_o, ps.part_lse, splits, slices * nq, head_dim, o, out_dtype, lse, s);
            // (this shape cannot take the narrow kernel: one launch without key splits below)
            if (rc != FSTA_EUNSUPPORTED) return rc;
        }
    }
    // the matrix-core kernel takes row maxima before scaling, which needs a positive scale
    if (!(flags & FSTA_FLAG_GENERIC) && sm_scale > 0.f && mfma_supported(dtype, head_dim, block_m)) {
        const bool fast_pv = (flags & FSTA_FLAG_FAST_PV) != 0;
        // (the kernel with 16 rows per wave reads the block plan only; it hands launches it cannot
        // take on to the other matrix-core kernel itself)
        int rc = FSTA_EUNSUPPORTED;
        if (!(flags & FSTA_FLAG_WIDE_WAVES)) rc = launch_attention_stream(p, dtype, head_dim, fast_pv, s);
        if (rc == FSTA_EUNSUPPORTED)
            rc = (flags & FSTA_FLAG_WIDE_WAVES) || !p.plan ? launch_attention_mfma(p, dtype, head_dim, fast_pv, s)
                                                           : launch_attention_mfma16(p, dtype, head_dim, fast_pv, s);
        // ancestor lists too long for the LDS-resident lists of these kernels: the scalar kernel
        // streams them and takes any length
        if (rc != FSTA_EUNSUPPORTED) return rc;
    }
    return launch_attention_generic(p, dtype, head_dim, s);
}

extern "C" int fsta_attention_fwd_kv8(const void* q, const void* k8, const void* v8, const float* k_scale,
                                      const float* v_scale, void* o, float* lse, const uint32_t* block_plan,
                                      int32_t plan_key_shift, int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                                      int32_t head_dim, int32_t dtype, int32_t out_dtype, int32_t block_m,
                                      int32_t max_ancestors, int32_t num_blocks, float sm_scale, void* stream) {
    if (batch < 0 || heads < 0 || nq < 0 || nk < nq)
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: batch=%d heads=%d nq=%d nk=%d (need nk >= nq >= 0)", batch,
                    heads, nq, nk);
    if (dtype != FSTA_F16 && dtype != FSTA_BF16)
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: dtype=%d (q must be float16 or bfloat16)", dtype);
    if (out_dtype != dtype && out_dtype != FSTA_F32)
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: out_dtype=%d must equal dtype=%d or be float32", out_dtype, dtype);
    if (head_dim != 64 && head_dim != 128)
        return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd_kv8: head_dim=%d (supported: 64, 128)", head_dim);
    if (!plan_block_size_ok(block_m))
        return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd_kv8: block_m=%d (supported: 32, 64, 128)", block_m);
    if (max_ancestors < 1) return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: max_ancestors=%d", max_ancestors);
    if (num_blocks != (nq + block_m - 1) / block_m)
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: num_blocks=%d but ceil(nq=%d / block_m=%d) = %d", num_blocks, nq,
                    block_m, (nq + block_m - 1) / block_m);
    if (!(sm_scale > 0.f)) return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd_kv8: sm_scale must be positive");
    const int64_t slices = (int64_t)batch * heads;
    if (slices > 65535) return fail(FSTA_EUNSUPPORTED, "fsta_attention_fwd_kv8: batch*heads=%lld > 65535", (long long)slices);
    if (slices == 0 || nq == 0) return FSTA_OK;
    if (!q || !k8 || !v8 || !o || !block_plan) return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: null pointer");
    if (misaligned(q, 16) || misaligned(k8, 16) || misaligned(v8, 16) || misaligned(o, 16) || misaligned(block_plan, 16))
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: q, k8, v8, o and block_plan must be 16-byte aligned");
    if (misaligned(k_scale, 4) || misaligned(v_scale, 4) || misaligned(lse, 4))
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: k_scale, v_scale and lse must be 4-byte aligned");
    if (plan_key_shift < 0 || plan_key_shift > nk)
        return fail(FSTA_EINVAL, "fsta_attention_fwd_kv8: plan_key_shift=%d outside [0, nk=%d]", plan_key_shift, nk);
    AttnParams p;
    p.q = q; p.k = k8; p.v = v8; p.o = o; p.lse = lse;
    p.ancestor_idx = nullptr; p.mask_bits = nullptr; p.anc_count = nullptr; p.leaf_idx = nullptr;
    p.plan = block_plan; p.key_shift = plan_key_shift;
    p.nq = nq; p.nk = nk; p.prefix = nk - nq;
    p.block_m = block_m; p.max_anc = max_ancestors; p.mask_words = fsta_mask_words(max_ancestors);
    p.nb = num_blocks;
    p.heads_total = (int32_t)slices;
    p.out_f32 = (out_dtype == FSTA_F32) ? 1 : 0;
    p.scale_log2e = sm_scale * kLog2e;
    p.key_splits = 1; p.split_tiles = 0; p.part_o = nullptr; p.part_lse = nullptr;
    p.share_tiles = 0;
    p.k_scale = k_scale; p.v_scale = v_scale;
    p.merge_parts = 0; p.dry_run = 0; p.stream_mode = 0;
    return launch_attention_mfma16_kv8(p, dtype, head_dim, static_cast<hipStream_t>(stream));
}
