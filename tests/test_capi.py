"""The C ABI library loads and exports what include/fsta.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

from fstattention_amd import _lib

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "fsta.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fsta_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_functions()
    assert "fsta_attention_fwd" in names and "fsta_precompute" in names
    assert sorted(_lib.SIGNATURES) == names


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} has not been built (python -m fstattention_amd.build)")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in fsta.h but not exported"


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """include/fsta.h is what a C, cgo or FFI binding includes: it has to compile as C99 without the
    HIP headers, and a C program has to link against the library and reach its host-side checks."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} has not been built (python -m fstattention_amd.build)")
    src = tmp_path / "use_fsta.c"
    src.write_text(
        '#include "fsta.h"\n#include <stdio.h>\n#include <string.h>\n'
        "int main(void) {\n"
        "    if (fsta_abi_version() != FSTA_ABI_VERSION) return 1;\n"
        "    if (fsta_mask_words(80) != 3) return 2;\n"
        "    /* rejected on the host, before any GPU work: head_dim 48 is not supported */\n"
        "    int rc = fsta_attention_fwd(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 64, 64, 48, FSTA_BF16, FSTA_BF16,\n"
        "                                64, 64, 1, 0.125f, 0, 0);\n"
        "    if (rc == FSTA_OK || strlen(fsta_last_error()) == 0) return 3;\n"
        '    printf("ok\\n");\n    return 0;\n}\n')
    exe = tmp_path / "use_fsta"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.dirname(HEADER),
                    str(src), "-o", str(exe), "-L", libdir, "-l:" + os.path.basename(_lib.LIB_PATH),
                    "-Wl,-rpath," + libdir, "-Wl,--allow-shlib-undefined"], check=True, capture_output=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "ok", (out.returncode, out.stdout, out.stderr)


def test_constants_match_header():
    text = open(HEADER).read()
    defs = dict(re.findall(r"#define\s+(FSTA_[A-Z_0-9]+)\s+(-?\d+)u?\b", text))
    assert int(defs["FSTA_ABI_VERSION"]) == _lib.ABI_VERSION
    assert int(defs["FSTA_DFS_ORDER_MAX_NODES"]) == _lib.DFS_ORDER_MAX_NODES
    assert int(defs["FSTA_DFS_ORDER_STATIC_MAX_NODES"]) == _lib.DFS_ORDER_STATIC_MAX_NODES
    assert "(6 * (size_t)(n) + 8)" in text and _lib.dfs_order_workspace_ints(10) == 68
    assert (int(defs["FSTA_F32"]), int(defs["FSTA_F16"]), int(defs["FSTA_BF16"]), int(defs["FSTA_F64"])) == \
        (_lib.F32, _lib.F16, _lib.BF16, _lib.F64)
    assert int(defs["FSTA_TREE_NOT_PREFIX_CLOSED"]) == _lib.TREE_NOT_PREFIX_CLOSED
    assert (int(defs["FSTA_OK"]), int(defs["FSTA_EINVAL"]), int(defs["FSTA_EUNSUPPORTED"]),
            int(defs["FSTA_EHIP"])) == (_lib.OK, _lib.EINVAL, _lib.EUNSUPPORTED, _lib.EHIP)
    assert (int(defs["FSTA_FLAG_FAST_PV"]), int(defs["FSTA_FLAG_GENERIC"]), int(defs["FSTA_FLAG_WIDE_WAVES"]),
            int(defs["FSTA_FLAG_SHARE_TILES"])) == \
        (_lib.FLAG_FAST_PV, _lib.FLAG_GENERIC, _lib.FLAG_WIDE_WAVES, _lib.FLAG_SHARE_TILES)
    assert (int(defs["FSTA_PRE_TOO_MANY_ANCESTORS"]), int(defs["FSTA_PRE_BAD_NODE_ID"]),
            int(defs["FSTA_PRE_BAD_LEVEL"])) == (_lib.PRE_TOO_MANY_ANCESTORS, _lib.PRE_BAD_NODE_ID, _lib.PRE_BAD_LEVEL)


def test_argument_validation_happens_before_any_gpu_work():
    lib = _lib.load()
    assert lib.fsta_abi_version() == _lib.ABI_VERSION
    assert lib.fsta_mask_words(1) == 1 and lib.fsta_mask_words(32) == 1 and lib.fsta_mask_words(33) == 2
    # every call below is rejected on its arguments; nothing is launched
    bad_dtype = lib.fsta_attention_fwd(None, None, None, None, None, None, None, None, None, None, 0,
                                       1, 1, 16, 16, 64, 7, 7, 16, 8, 1, 1.0, 0, None)
    assert bad_dtype == _lib.EINVAL and b"dtype" in lib.fsta_last_error()
    bad_dim = lib.fsta_attention_fwd(None, None, None, None, None, None, None, None, None, None, 0,
                                     1, 1, 16, 16, 48, _lib.F16, _lib.F16, 16, 8, 1, 1.0, 0, None)
    assert bad_dim == _lib.EUNSUPPORTED and b"head_dim" in lib.fsta_last_error()
    short_k = lib.fsta_attention_fwd(None, None, None, None, None, None, None, None, None, None, 0,
                                     1, 1, 16, 8, 64, _lib.F16, _lib.F16, 16, 8, 1, 1.0, 0, None)
    assert short_k == _lib.EINVAL
    blocks = lib.fsta_attention_fwd(None, None, None, None, None, None, None, None, None, None, 0,
                                    1, 1, 40, 40, 64, _lib.F16, _lib.F16, 16, 8, 2, 1.0, 0, None)
    assert blocks == _lib.EINVAL and b"num_blocks" in lib.fsta_last_error()
    null_ptr = lib.fsta_attention_fwd(None, None, None, None, None, None, None, None, None, None, 0,
                                      1, 1, 16, 16, 64, _lib.F16, _lib.F16, 16, 8, 1, 1.0, 0, None)
    assert null_ptr == _lib.EINVAL and b"null" in lib.fsta_last_error()
    # pointer alignment: rows and plan records move 16 bytes at a time, list entries 8, words 4
    ok = dict(q=256, k=256, v=256, o=256, lse=256, a=256, bits=256, cnt=256, leaf=256, plan=256)

    def attn(**ptr):
        a = dict(ok, **ptr)
        return lib.fsta_attention_fwd(a["q"], a["k"], a["v"], a["o"], a["lse"], a["a"], a["bits"], a["cnt"], a["leaf"],
                                      a["plan"], 0, 1, 1, 64, 64, 64, _lib.BF16, _lib.BF16, 64, 32, 1, 0.125, 0, None)
    for name, off, word in (("q", 8, b"16-byte"), ("k", 8, b"16-byte"), ("v", 4, b"16-byte"), ("o", 8, b"16-byte"),
                            ("plan", 8, b"block_plan"), ("a", 4, b"8-byte"), ("leaf", 4, b"8-byte"),
                            ("bits", 2, b"4-byte"), ("cnt", 2, b"4-byte"), ("lse", 2, b"4-byte")):
        assert attn(**{name: 256 + off}) == _lib.EINVAL and word in lib.fsta_last_error(), name
    assert lib.fsta_attention_fwd(256, 256, 256, 256, None, 256, 256, 256, 256, 256, -1, 1, 1, 64, 64, 64, _lib.BF16,
                                  _lib.BF16, 64, 32, 1, 0.125, 0, None) == _lib.EINVAL      # negative key shift
    assert lib.fsta_precompute(256, 256, 64, 4, 64, 32, 0, 260, None, 256, None, None, None, 256, None) == _lib.EINVAL
    assert b"8-byte" in lib.fsta_last_error()
    assert lib.fsta_precompute(256, 256, 64, 4, 64, 32, 0, 256, None, 256, 258, None, None, 256, None) == _lib.EINVAL
    assert lib.fsta_precompute(256, 256, 64, 4, 64, 32, 0, 256, None, 256, None, None, 264, 256, None) == _lib.EINVAL
    assert lib.fsta_precompute(256, 256, 64, 4, 16, 32, 0, 256, None, 256, None, None, 256, 256, None) == _lib.EINVAL
    assert b"block plan" in lib.fsta_last_error()       # block sizes of the plan: 32, 64, 128
    assert lib.fsta_pack_mask(260, 256, None, 2, 64, 32, 0, 256, 256, None, None) == _lib.EINVAL
    assert lib.fsta_pack_mask(256, 256, None, 2, 64, 32, 0, 256, 256, 256, None) == _lib.EINVAL     # plan without leaf_idx
    assert lib.fsta_pack_mask(256, 256, 256, 2, 64, 32, 64, 256, 256, 264, None) == _lib.EINVAL     # plan alignment
    assert lib.fsta_block_plan_bytes(4, 64, 64) == 4 * (8 + 64 + 2 * (32 + 64)) * 4
    assert lib.fsta_block_plan_bytes(4, 16, 64) == 0 and lib.fsta_block_plan_bytes(0, 64, 64) == 0
    assert lib.fsta_precompute(None, None, 10, 0, 4, 4, 0, None, None, None, None, None, None, None, None) == _lib.EINVAL
    assert lib.fsta_precompute(None, None, 0, 1, 4, 4, 0, None, None, None, None, None, None, None, None) == _lib.OK
    assert lib.fsta_pack_mask(None, None, None, 0, 16, 8, 0, None, None, None, None) == _lib.OK
    assert lib.fsta_pack_mask(None, None, None, 2, 16, 0, 0, None, None, None, None) == _lib.EINVAL
    assert lib.fsta_lineage_from_parents(None, 5, 0, None, None, None, None) == _lib.EINVAL
    assert lib.fsta_dfs_order(None, -1, 0, None, None, None, None, None) == _lib.EINVAL
    assert lib.fsta_dfs_order(None, 1 << 20, 0, None, None, None, None, None) == _lib.EUNSUPPORTED
    assert lib.fsta_dfs_order(None, 8, 0, None, None, None, None, None) == _lib.EINVAL      # null pointers
    assert lib.fsta_renumber_parents(None, None, -1, None, None) == _lib.EINVAL
    assert lib.fsta_renumber_parents(None, None, 0, None, None) == _lib.OK
    assert lib.fsta_renumber_parents(None, None, 8, None, None) == _lib.EINVAL and b"null" in lib.fsta_last_error()
    assert lib.fsta_merge_states(None, None, None, None, None, None, 4, 12, _lib.BF16, None) == _lib.EINVAL   # head dim
    assert lib.fsta_merge_states(None, None, None, None, None, None, 4, 64, 7, None) == _lib.EINVAL          # null pointers come first
    assert lib.fsta_merge_states(None, None, None, None, None, None, 0, 64, _lib.BF16, None) == _lib.OK       # nothing to do
    with pytest.raises(_lib.FstaError):
        _lib.check(_lib.EINVAL)


def test_tree_builder_rejects_bad_arguments_before_any_gpu_work():
    lib = _lib.load()
    call = lambda *a: lib.fsta_medusa_tree(*a)
    assert call(8, _lib.F64, 0, 10, 5, 8, 8, None) == _lib.EINVAL
    assert call(8, _lib.BF16, 4, 10, 5, 8, 8, None) == _lib.EINVAL and b"probs_dtype" in lib.fsta_last_error()
    assert call(8, _lib.F64, 4, 12, 5, 8, 8, None) == _lib.EUNSUPPORTED      # 22620 candidate paths
    assert call(8, _lib.F64, 2, 600, 5, 8, 8, None) == _lib.EUNSUPPORTED     # 1200 probabilities
    assert call(8, _lib.F64, 2, 3, 14, 8, 8, None) == _lib.EINVAL            # 12 paths + root < 14 nodes
    assert call(None, _lib.F64, 2, 3, 5, 8, 8, None) == _lib.EINVAL and b"null" in lib.fsta_last_error()
    # more candidate paths than one workgroup ranks: the workspace variant, with its own checks
    ws = lambda *a: lib.fsta_medusa_tree_ws(*a)
    assert lib.fsta_medusa_workspace_bytes(4, 10) == 0                        # 11110 paths: one launch, no workspace
    need = lib.fsta_medusa_workspace_bytes(5, 10)                             # 111110 paths, 28 workgroups of 4096
    assert need == 111110 * 8 + 8 * 256 * 4 + 8 * 4 + 28 * 2 * 4
    assert lib.fsta_medusa_workspace_bytes(8, 10) == 0                        # beyond 2^24 paths: out of range
    assert ws(8, _lib.F64, 5, 10, 300, 8, 8, None, 0, None) == _lib.EINVAL and b"workspace" in lib.fsta_last_error()
    assert ws(8, _lib.F64, 5, 10, 300, 8, 8, 64, need - 1, None) == _lib.EINVAL
    assert ws(8, _lib.F64, 5, 10, 300, 8, 8, 68, need, None) == _lib.EINVAL and b"aligned" in lib.fsta_last_error()
    assert ws(8, _lib.BF16, 5, 10, 300, 8, 8, 64, need, None) == _lib.EINVAL and b"probs_dtype" in lib.fsta_last_error()
    assert ws(8, _lib.F64, 8, 10, 300, 8, 8, 64, need, None) == _lib.EUNSUPPORTED
    assert ws(8, _lib.F64, 2, 200, 50000, 8, 8, 64, 1 << 30, None) == _lib.EINVAL       # 40200 paths + root < 50000 nodes
    assert ws(None, _lib.F64, 5, 10, 300, 8, 8, 64, need, None) == _lib.EINVAL and b"null" in lib.fsta_last_error()
    assert ws(8, _lib.F64, 0, 10, 5, 8, 8, None, 0, None) == _lib.EINVAL      # small problems: the checks of fsta_medusa_tree


def test_workspace_planning_is_host_arithmetic():
    """How a shared prefix is cut into runs of keys depends on the shape and flags only."""
    lib = _lib.load()
    per_run = 32 * 256 * (128 + 1) * 4       # float32 partial rows + their log-sum-exps of one run
    size = lambda *a: lib.fsta_attention_workspace_bytes(*a)
    # one sequence, 32 heads, 256 rows behind 16384 prefix keys: the prefix goes to the dense prefix kernel, 64 workgroups
    # of 128 rows per run -> 8 runs, plus one slot for the tree part
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, 0) == 9 * per_run
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, _lib.flag_key_splits(7)) == 8 * per_run
    # enough workgroups to begin with: one run (the dense kernel still takes the prefix)
    assert size(8, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, 0) == 2 * 8 * per_run
    # head dims the dense kernel does not take: runs of keys inside the tree kernel (4 for 128 workgroups)
    assert size(1, 32, 256, 256 + 16384, 32, _lib.BF16, 64, 64, 0.1, 0) == 4 * 32 * 256 * (32 + 1) * 4
    # nothing to cut: no prefix, a short one, enough blocks already, never-split flag
    assert size(1, 32, 256, 256, 128, _lib.BF16, 64, 64, 0.1, 0) == 0
    assert size(1, 32, 256, 256 + 256, 128, _lib.BF16, 64, 64, 0.1, 0) == 0
    # a prefix too short for the dense kernel: runs of keys inside the tree kernel
    assert size(1, 32, 256, 256 + 1024, 128, _lib.BF16, 64, 64, 0.1, 0) == 4 * per_run
    assert size(8, 32, 256, 256 + 16384, 32, _lib.BF16, 64, 64, 0.1, 0) == 0
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, _lib.flag_key_splits(1)) == 0
    # kernels without key runs: float32, the scalar and wide-wave kernels, non-positive scales
    assert size(1, 32, 256, 256 + 16384, 128, _lib.F32, 64, 64, 0.1, 0) == 0
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, _lib.FLAG_GENERIC) == 0
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, _lib.FLAG_WIDE_WAVES) == 0
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.0, 0) == 0
    assert size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 16, 64, 0.1, 0) == 0
    # more runs than tiles are not made; malformed shapes want nothing
    assert size(1, 1, 32, 32 + 64, 64, _lib.F16, 32, 16, 0.1, _lib.flag_key_splits(9)) == 2 * 32 * (64 + 1) * 4
    assert size(0, 32, 256, 512, 128, _lib.BF16, 64, 64, 0.1, 0) == 0
    assert size(1, 32, 256, 100, 128, _lib.BF16, 64, 64, 0.1, 0) == 0
    # the workspace variant validates like the plain one, and wants an aligned workspace
    bad = lib.fsta_attention_fwd_ws(None, None, None, None, None, None, None, None, None, None, 0,
                                    1, 1, 16, 16, 64, 7, 7, 16, 8, 1, 1.0, 0, None, 0, None)
    assert bad == _lib.EINVAL and b"dtype" in lib.fsta_last_error()
    need = size(1, 32, 256, 256 + 16384, 128, _lib.BF16, 64, 64, 0.1, 0)
    odd = lib.fsta_attention_fwd_ws(16, 16, 16, 16, None, 8, 8, None, 8, 16, 0, 1, 32, 256, 256 + 16384, 128, _lib.BF16,
                                    _lib.BF16, 64, 64, 4, 0.1, 0, 4100, need, None)
    assert odd == _lib.EINVAL and b"aligned" in lib.fsta_last_error()


def test_python_entry_points_refuse_to_run_without_a_gpu_path():
    import torch
    from fstattention_amd import create_fst_attention_kernel_inputs, fst_attention, trees
    q = torch.zeros(1, 1, 16, 16, dtype=torch.float16)
    idx = torch.full((1, 8), -1, dtype=torch.int64)
    mask = torch.zeros(1, 16, 8, dtype=torch.bool)
    leaf = torch.arange(16).view(1, 16)
    with pytest.raises(ValueError, match="GPU"):
        fst_attention(q, q, q, idx, mask, leaf, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)
    from fstattention_amd import dfs_order_gpu, medusa_parents_gpu, merge_attention_states
    lse = torch.zeros(16)
    with pytest.raises(ValueError, match="GPU"):
        merge_attention_states(q, lse, q, lse)
    with pytest.raises(ValueError, match="GPU"):
        dfs_order_gpu(torch.tensor([-1, 0], dtype=torch.int64))
    with pytest.raises(ValueError, match="GPU"):
        medusa_parents_gpu(torch.ones(2, 3), 4)
    if not torch.cuda.is_available():
        lineage, level = trees.lineage_from_parents([-1, 0, 1])
        with pytest.raises(RuntimeError, match="GPU"):
            create_fst_attention_kernel_inputs(lineage, level, 4, 4)


def test_operator_library_registers_both_operators_and_rejects_host_tensors():
    """``_fsta_torch.so`` registers ``fsta::attention_fwd`` and ``fsta::precompute`` with torch's dispatcher;
    both check their arguments on the host and refuse tensors that are not on the GPU."""
    import torch
    if not os.path.exists(_lib.TORCH_OPS_PATH):
        pytest.fail(f"{_lib.TORCH_OPS_PATH} has not been built (python -m fstattention_amd.build)")
    ops = _lib.load_torch_ops()
    pre = ops.precompute.default._schema
    assert [a.name for a in pre.arguments] == ["lineage", "level_lookup", "block_m", "max_ancestors", "mutate_lineage",
                                               "want_bool_mask", "status"]
    assert len(pre.returns) == 7
    assert pre.arguments[0].alias_info is not None and pre.arguments[0].alias_info.is_write   # lineage is written
    fwd = ops.attention_fwd.default._schema
    assert [a.name for a in fwd.arguments][:6] == ["q", "k", "v", "ancestor_idx", "mask_bits", "anc_count"]
    lineage = torch.tensor([[0, -1], [0, 1]], dtype=torch.int64)
    level = torch.tensor([0, 1], dtype=torch.int64)
    with pytest.raises(ValueError, match="GPU"):
        ops.precompute(lineage, level, 2, 2, True, True, None)
    with pytest.raises(ValueError, match="int64"):
        ops.precompute(lineage.int(), level, 2, 2, True, True, None)
