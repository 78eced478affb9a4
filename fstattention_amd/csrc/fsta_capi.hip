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

}  // namespace fsta

using namespace fsta;

extern "C" int fsta_abi_version(void) { return FSTA_ABI_VERSION; }

extern "C" const char* fsta_last_error(void) { return g_error; }

extern "C" int fsta_attention_fwd(const void* q, const void* k, const void* v, void* o, float* lse,
                                  const int64_t* ancestor_idx, const uint32_t* mask_bits,
                                  const int32_t* anc_count, const int64_t* leaf_idx,
                                  int32_t batch, int32_t heads, int32_t nq, int32_t nk,
                                  int32_t head_dim, int32_t dtype, int32_t out_dtype,
                                  int32_t block_m, int32_t max_ancestors, int32_t num_blocks,
                                  float sm_scale, uint32_t flags, void* stream) {
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

    AttnParams p;
    p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
    p.ancestor_idx = ancestor_idx; p.mask_bits = mask_bits; p.anc_count = anc_count;
    p.leaf_idx = leaf_idx;
    p.nq = nq; p.nk = nk; p.prefix = nk - nq;
    p.block_m = block_m; p.max_anc = max_ancestors; p.mask_words = fsta_mask_words(max_ancestors);
    p.nb = num_blocks;
    p.heads_total = (int32_t)slices;
    p.out_f32 = (out_dtype == FSTA_F32) ? 1 : 0;
    p.scale_log2e = sm_scale * kLog2e;

    hipStream_t s = static_cast<hipStream_t>(stream);
    // the matrix-core kernel takes row maxima before scaling, which needs a positive scale
    if (!(flags & FSTA_FLAG_GENERIC) && sm_scale > 0.f && mfma_supported(dtype, head_dim, block_m)) {
        const bool fast_pv = (flags & FSTA_FLAG_FAST_PV) != 0;
        const int rc = (flags & FSTA_FLAG_WIDE_WAVES) ? launch_attention_mfma(p, dtype, head_dim, fast_pv, s)
                                                      : launch_attention_mfma16(p, dtype, head_dim, fast_pv, s);
        // ancestor lists too long for the LDS-resident lists of these kernels: the scalar kernel
        // streams them and takes any length
        if (rc != FSTA_EUNSUPPORTED) return rc;
    }
    return launch_attention_generic(p, dtype, head_dim, s);
}
