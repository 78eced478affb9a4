// PyTorch operator registration of the two entry points of the path (host code only, no kernels):
//   torch.ops.fsta.attention_fwd(...)  ->  fsta_attention_fwd_ws / fsta_attention_fwd_kv8 of libfsta.so
//   torch.ops.fsta.precompute(...)     ->  fsta_precompute (reference utils.py:104-129)
// on torch's current HIP stream of the tensors' device.  It does in C++ what the operator wrapper of
// reference fstattention.py:153-181 does in Python (shape checks, allocation of o and L, launch), so
// that an eager caller pays the dispatcher and one allocation per call instead of a page of Python.
// Device memory, streams and the device guard are torch's; everything below the C ABI is libfsta's.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <tuple>

#include "../../include/fsta.h"

namespace {

int dtype_code(at::ScalarType t) {
    switch (t) {
        case at::kFloat: return FSTA_F32;
        case at::kHalf: return FSTA_F16;
        case at::kBFloat16: return FSTA_BF16;
        default: return -1;
    }
}

void check_rc(int rc) {
    TORCH_CHECK(rc == FSTA_OK, "libfsta error ", rc, ": ", fsta_last_error());
}

const void* ptr_or_null(const c10::optional<at::Tensor>& t) { return t.has_value() && t->defined() ? t->data_ptr() : nullptr; }

// q [Z,H,Nq,D], k/v [Z,H,Nk,D] (16-bit or float32; k/v float8_e4m3fn for 8-bit storage with optional
// per-slice scales), the reference's index tensors, their packed forms, the block plan (or None).
// out_dtype_code: FSTA_* code of o; flags: FSTA_FLAG_*.  Returns (o, lse); lse is empty unless asked for.
std::tuple<at::Tensor, at::Tensor> attention_fwd(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                                 const at::Tensor& ancestor_idx, const at::Tensor& mask_bits,
                                                 const at::Tensor& anc_count, const at::Tensor& leaf_idx,
                                                 const c10::optional<at::Tensor>& plan, int64_t key_shift,
                                                 double sm_scale, int64_t block_m, int64_t max_ancestors,
                                                 int64_t out_dtype_code, bool return_lse, int64_t flags,
                                                 const c10::optional<at::Tensor>& k_scale,
                                                 const c10::optional<at::Tensor>& v_scale) {
    TORCH_CHECK_VALUE(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, "q, k, v must be [batch, heads, seq, head_dim]");
    TORCH_CHECK_VALUE(q.is_cuda() && k.is_cuda() && v.is_cuda(), "fst_attention runs on the GPU only (no CPU fallback)");
    TORCH_CHECK_VALUE(q.device() == k.device() && q.device() == v.device() && q.device() == ancestor_idx.device() &&
                    q.device() == leaf_idx.device() && q.device() == mask_bits.device() && q.device() == anc_count.device(),
                "all tensors must live on the same device");
    TORCH_CHECK_VALUE(q.is_contiguous() && k.is_contiguous() && v.is_contiguous(), "q, k, v must be contiguous");
    const int64_t Z = q.size(0), H = q.size(1), Nq = q.size(2), D = q.size(3), Nk = k.size(2);
    TORCH_CHECK_VALUE(k.size(0) == Z && k.size(1) == H && k.size(3) == D && v.sizes() == k.sizes(), "k/v shapes do not match q");
    TORCH_CHECK_VALUE(Nk >= Nq, "k has fewer rows than q");
    const int64_t nb = (Nq + block_m - 1) / block_m;
    TORCH_CHECK_VALUE(ancestor_idx.scalar_type() == at::kLong && leaf_idx.scalar_type() == at::kLong,
                "ancestor_idx and leaf_idx must be int64");
    TORCH_CHECK_VALUE(ancestor_idx.dim() == 2 && ancestor_idx.size(0) == nb && ancestor_idx.size(1) == max_ancestors,
                      "ancestor_idx is not [ceil(Nq/BLOCK_M)=", nb, ", MAX_ANCESTORS=", max_ancestors, "]");
    TORCH_CHECK_VALUE(leaf_idx.dim() == 2 && leaf_idx.size(0) == nb && leaf_idx.size(1) == block_m,
                      "leaf_idx is not [", nb, ", BLOCK_M=", block_m, "]");
    const at::Tensor a_idx = ancestor_idx.contiguous(), l_idx = leaf_idx.contiguous();
    TORCH_CHECK_VALUE(mask_bits.numel() == nb * fsta_mask_words((int32_t)max_ancestors) * block_m && anc_count.numel() == nb,
                "packed mask was built for another block size / ancestor count");
    if (plan.has_value() && plan->defined())
        TORCH_CHECK_VALUE((size_t)plan->numel() * plan->element_size() >=
                            fsta_block_plan_bytes((int32_t)nb, (int32_t)block_m, (int32_t)max_ancestors) &&
                        plan->device() == q.device(),
                    "block plan was built for another block size / ancestor count");
    const bool kv8 = k.scalar_type() == at::kFloat8_e4m3fn;
    const int code = dtype_code(q.scalar_type());
    TORCH_CHECK_VALUE(code >= 0, "q must be float32, float16 or bfloat16");
    TORCH_CHECK_VALUE(kv8 ? v.scalar_type() == at::kFloat8_e4m3fn : (k.scalar_type() == q.scalar_type() && v.scalar_type() == q.scalar_type()),
                "q/k/v must share one dtype (or k and v both be float8_e4m3fn)");
    TORCH_CHECK_VALUE(out_dtype_code == code || out_dtype_code == FSTA_F32, "out_dtype must be the input dtype or float32");
    TORCH_CHECK_VALUE(kv8 || (!k_scale.has_value() && !v_scale.has_value()),
                      "k_scale / v_scale belong to 8-bit K/V (float8_e4m3fn k and v)");
    TORCH_CHECK_VALUE(!kv8 || (flags == 0 && code != FSTA_F32),
                      "8-bit K/V: q must be float16/bfloat16, and there is one kernel (no kernel-selection switches)");

    const c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
    const hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(q.device().index()).stream();
    at::Tensor o = at::empty(q.sizes(), q.options().dtype(out_dtype_code == FSTA_F32 ? at::kFloat : q.scalar_type()));
    // the reference allocates L and drops it (fstattention.py:158-160,181); here it only exists when asked for
    at::Tensor lse = return_lse ? at::empty({Z * H, Nq}, q.options().dtype(at::kFloat)) : at::Tensor();
    float* lse_ptr = return_lse ? lse.data_ptr<float>() : nullptr;
    const uint32_t* plan_ptr = static_cast<const uint32_t*>(ptr_or_null(plan));
    if (kv8) {
        TORCH_CHECK_VALUE(plan_ptr != nullptr, "8-bit K/V needs BLOCK_M of 32, 64 or 128");
        for (const auto* s : {&k_scale, &v_scale})
            TORCH_CHECK_VALUE(!s->has_value() || ((*s)->scalar_type() == at::kFloat && (*s)->numel() == Z * H &&
                                             (*s)->is_contiguous() && (*s)->device() == q.device()),
                        "k_scale / v_scale must be contiguous float32 tensors of batch*heads entries on q's device");
        check_rc(fsta_attention_fwd_kv8(q.data_ptr(), k.data_ptr(), v.data_ptr(), static_cast<const float*>(ptr_or_null(k_scale)),
                                        static_cast<const float*>(ptr_or_null(v_scale)), o.data_ptr(), lse_ptr, plan_ptr,
                                        (int32_t)key_shift, (int32_t)Z, (int32_t)H, (int32_t)Nq, (int32_t)Nk, (int32_t)D, code,
                                        (int32_t)out_dtype_code, (int32_t)block_m, (int32_t)max_ancestors, (int32_t)nb,
                                        (float)sm_scale, stream));
        return {o, lse};
    }
    // a shared prefix may be worth cutting into key runs: the library says how much workspace that takes
    at::Tensor work;
    size_t work_bytes = 0;
    if (Nk > Nq) {
        work_bytes = fsta_attention_workspace_bytes((int32_t)Z, (int32_t)H, (int32_t)Nq, (int32_t)Nk, (int32_t)D, code,
                                                    (int32_t)block_m, (int32_t)max_ancestors, (float)sm_scale, (uint32_t)flags);
        if (work_bytes) work = at::empty({(int64_t)work_bytes}, q.options().dtype(at::kByte));
    }
    check_rc(fsta_attention_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse_ptr,
                                   a_idx.data_ptr<int64_t>(), static_cast<const uint32_t*>(mask_bits.data_ptr()),
                                   static_cast<const int32_t*>(anc_count.data_ptr()), l_idx.data_ptr<int64_t>(), plan_ptr,
                                   (int32_t)key_shift, (int32_t)Z, (int32_t)H, (int32_t)Nq, (int32_t)Nk, (int32_t)D, code,
                                   (int32_t)out_dtype_code, (int32_t)block_m, (int32_t)max_ancestors, (int32_t)nb,
                                   (float)sm_scale, (uint32_t)flags, work_bytes ? work.data_ptr() : nullptr, work_bytes, stream));
    return {o, lse};
}

// lineage [N, W] int64 (contiguous; written to when mutate_lineage, as utils.py:124-125 writes to the caller's
// tensor), level_lookup [N] int64, on the GPU.  Returns the three tensors of the reference (ancestor_mask empty
// unless want_bool_mask), the packed mask, the per-block ancestor counts, the block plan (empty for block sizes
// the matrix-core kernels do not take) and the status word (FSTA_PRE_* bits; the caller's own zeroed word if one
// was passed, so that the stages of a front-end chain share one).
std::tuple<at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor, at::Tensor> precompute(
    at::Tensor& lineage, const at::Tensor& level_lookup, int64_t block_m, int64_t max_ancestors, bool mutate_lineage,
    bool want_bool_mask, const c10::optional<at::Tensor>& status) {
    TORCH_CHECK_VALUE(lineage.dim() == 2 && level_lookup.dim() == 1 && level_lookup.size(0) == lineage.size(0),
                      "lineage must be [N, W] and level_lookup [N]");
    TORCH_CHECK_VALUE(lineage.scalar_type() == at::kLong && level_lookup.scalar_type() == at::kLong,
                      "lineage and level_lookup must be int64");
    TORCH_CHECK_VALUE(lineage.is_cuda() && level_lookup.device() == lineage.device(),
                      "the precompute runs on the GPU only (no CPU fallback); both tensors on one device");
    TORCH_CHECK_VALUE(lineage.is_contiguous() && level_lookup.is_contiguous(), "lineage and level_lookup must be contiguous");
    TORCH_CHECK_VALUE(block_m > 0 && max_ancestors > 0, "block_m and max_ancestors must be positive");
    const int64_t n = lineage.size(0), width = lineage.size(1);
    const int64_t nb = (n + block_m - 1) / block_m;
    const auto i64 = lineage.options();
    const auto i32 = lineage.options().dtype(at::kInt);
    at::Tensor a_idx = at::empty({nb, max_ancestors}, i64);
    at::Tensor a_mask = want_bool_mask ? at::empty({nb, block_m, max_ancestors}, lineage.options().dtype(at::kBool)) : at::Tensor();
    at::Tensor l_idx = at::empty({nb, block_m}, i64);
    at::Tensor bits = at::empty({nb, (int64_t)fsta_mask_words((int32_t)max_ancestors), block_m}, i32);
    at::Tensor count = at::empty({nb}, i32);
    const size_t plan_bytes = fsta_block_plan_bytes((int32_t)nb, (int32_t)block_m, (int32_t)max_ancestors);
    at::Tensor plan = plan_bytes ? at::empty({(int64_t)(plan_bytes / 4)}, i32) : at::Tensor();
    at::Tensor st;
    if (status.has_value() && status->defined()) {
        TORCH_CHECK_VALUE(status->scalar_type() == at::kInt && status->numel() == 1 && status->device() == lineage.device(),
                          "status must be one int32 on the tensors' device");
        st = *status;
    } else {
        st = at::zeros({1}, i32);
    }
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(lineage.device());
    const hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(lineage.device().index()).stream();
    check_rc(fsta_precompute(lineage.data_ptr<int64_t>(), level_lookup.data_ptr<int64_t>(), n, width, (int32_t)block_m,
                             (int32_t)max_ancestors, mutate_lineage ? 1 : 0, a_idx.data_ptr<int64_t>(),
                             want_bool_mask ? static_cast<uint8_t*>(a_mask.data_ptr()) : nullptr, l_idx.data_ptr<int64_t>(),
                             static_cast<uint32_t*>(bits.data_ptr()), count.data_ptr<int32_t>(),
                             plan_bytes ? static_cast<uint32_t*>(plan.data_ptr()) : nullptr,
                             static_cast<uint32_t*>(st.data_ptr()), stream));
    return {a_idx, a_mask, l_idx, bits, count, plan, st};
}

}  // namespace

TORCH_LIBRARY(fsta, m) {
    m.def("precompute(Tensor(a!) lineage, Tensor level_lookup, int block_m, int max_ancestors, bool mutate_lineage, "
          "bool want_bool_mask, Tensor(b!)? status) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
    m.def("attention_fwd(Tensor q, Tensor k, Tensor v, Tensor ancestor_idx, Tensor mask_bits, Tensor anc_count, "
          "Tensor leaf_idx, Tensor? plan, int key_shift, float sm_scale, int block_m, int max_ancestors, "
          "int out_dtype_code, bool return_lse, int flags, Tensor? k_scale, Tensor? v_scale) -> (Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(fsta, CUDA, m) {
    m.impl("attention_fwd", &attention_fwd);
    m.impl("precompute", &precompute);
}
// tensors that all live on the host end up here: same message as for a mixed call
TORCH_LIBRARY_IMPL(fsta, CPU, m) {
    m.impl("attention_fwd", &attention_fwd);
    m.impl("precompute", &precompute);
}
