"""CPU-only checks of the boundary: libpf8.so loads and exports every symbol the headers under
include/ declare, the ctypes table matches the header's arity, argument validation rejects bad input
without touching a GPU, and the host-side mirror raises instead of falling back."""
import ctypes as C
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_decls():
    inc = os.path.join(ROOT, "include")
    text = "".join(open(os.path.join(inc, f)).read() for f in sorted(os.listdir(inc)) if f.endswith(".h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(?:int|const char\*)\s+(pf8_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        n = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        decls[m.group(1)] = n
    return decls


@pytest.fixture(scope="module")
def lib():
    from paddleformers_amd import _lib

    return _lib.lib()


def test_library_exports_every_declared_symbol(lib):
    decls = _header_decls()
    assert len(decls) >= 20
    for name in decls:
        assert hasattr(lib, name), f"{name} declared under include/ but not exported"


def test_ctypes_table_matches_header_arity():
    from paddleformers_amd import _lib

    decls = _header_decls()
    for name, argtypes in _lib.SIGNATURES.items():
        assert name in decls, f"{name} bound in _lib.py but not declared"
        assert len(argtypes) == decls[name], f"{name}: {len(argtypes)} bound arguments vs {decls[name]} declared"
    assert set(decls) - set(_lib.SIGNATURES) == {"pf8_last_error"}


def test_version_and_cu_budget(lib):
    assert lib.pf8_version() >= 100
    prev = lib.pf8_set_num_cus(112)
    assert lib.pf8_get_num_cus() == 112
    lib.pf8_set_num_cus(prev)
    assert lib.pf8_get_num_cus() == prev


def test_argument_validation_without_a_gpu(lib):
    """Every rejection happens before any launch, so it can be exercised on a CPU-only host."""
    from paddleformers_amd import _lib

    buf = (C.c_char * 64)()
    p = C.cast(buf, C.c_void_p)
    aligned = C.c_void_p((p.value + 15) & ~15)
    # K not a multiple of 128
    assert lib.pf8_quant_1x128(aligned, 4, 100, 100, aligned, aligned, 0, 0, None) == -1
    assert "multiple of 128" in _lib.last_error()
    # null pointers
    assert lib.pf8_quant_1x128(None, 4, 128, 128, aligned, aligned, 0, 0, None) == -1
    # misaligned pointer
    assert lib.pf8_quant_1x128(C.c_void_p(aligned.value + 2), 4, 128, 128, aligned, aligned, 0, 0, None) == -1
    # bad layout flag
    assert lib.pf8_quant_1x128(aligned, 4, 128, 128, aligned, aligned, 7, 0, None) == -1
    # zero-sized problems are legal no-ops
    assert lib.pf8_quant_1x128(None, 0, 128, 128, None, None, 0, 0, None) == 0
    assert lib.pf8_gemm_nt(None, None, 0, None, None, 0, 128, 128, None, 128, None) == 0
    assert lib.pf8_grouped_gemm_nt_contiguous(None, None, 0, None, None, 4, 0, 128, 128, None, None, None) == 0
    # grouped: rows not padded to 128
    assert lib.pf8_grouped_gemm_nt_contiguous(aligned, aligned, 0, aligned, aligned, 1, 100, 128, 128, aligned, aligned, None) == -1
    rows = (C.c_int64 * 2)(128, 100)
    assert lib.pf8_transpose_split_quant(aligned, None, 0, 0, rows, 2, 128, aligned, aligned, 0, None) == -1
    assert lib.pf8_grouped_wgrad(aligned, aligned, aligned, aligned, rows, 2, 128, 128, aligned, 1, None) == -1
    # q/s must come as pairs
    assert lib.pf8_quant_128x128(aligned, 128, 128, aligned, None, None, None, 0, None) == -1
    # the one-read row-wise + transposed quantizer: ragged segment, missing row-wise outputs, misaligned input
    good = (C.c_int64 * 2)(128, 128)
    assert lib.pf8_quant_and_transpose_split(aligned, rows, 2, 128, aligned, aligned, 0, aligned, aligned, 1, None) == -1
    assert "multiples of 128" in _lib.last_error()
    assert lib.pf8_quant_and_transpose_split(aligned, good, 2, 128, None, None, 0, aligned, aligned, 1, None) == -1
    assert lib.pf8_quant_and_transpose_split(C.c_void_p(aligned.value + 2), good, 2, 128, aligned, aligned, 0, aligned, aligned, 1, None) == -1
    assert lib.pf8_quant_and_transpose_split(aligned, good, 2, 100, aligned, aligned, 0, aligned, aligned, 1, None) == -1
    # UE8M0 GEMM: N must be a multiple of 128 and at least 256, K at least 384
    assert lib.pf8_gemm_nt_ue8m0(aligned, aligned, 128, aligned, aligned, 128, 128, 512, aligned, 128, None) == -1
    assert lib.pf8_gemm_nt_ue8m0(aligned, aligned, 128, aligned, aligned, 128, 384, 256, aligned, 384, None) == -1
    assert lib.pf8_gemm_nt_ue8m0(aligned, aligned, 128, aligned, aligned, 128, 320, 512, aligned, 320, None) == -1


def test_cpu_tensors_raise_instead_of_falling_back():
    from paddleformers_amd import deep_gemm
    from paddleformers_amd import functional as F8

    x = torch.zeros((128, 128), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        F8.fp8_quant_blockwise(x, quant_method="1x128")
    with pytest.raises(RuntimeError, match="no CPU path"):
        F8.fused_stack_transpose_quant([x])
    q = torch.zeros((128, 128), dtype=torch.float8_e4m3fn)
    s = torch.ones((128, 1))
    with pytest.raises(RuntimeError, match="no CPU path"):
        deep_gemm.fp8_gemm_nt((q, s), (q, torch.ones((1, 1))), torch.zeros((128, 128), dtype=torch.bfloat16))


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "paddleformers_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("CPU checker", ""), f"{f} mentions the oracle"


def test_padding_rule_matches_the_reference_branches():
    """transformers/fp8_utils.py:140-152 always lands on the next multiple of 512."""
    from paddleformers_amd.fp8_utils import FP8LinearFunctionBase as B

    for n in (1, 127, 128, 129, 300, 384, 385, 511, 512, 513, 640, 900, 1024, 1100):
        out = B.padding(torch.ones((n, 4)), 0)
        exp = n if n % 512 == 0 else (n // 512 + 1) * 512
        assert out.shape[0] == exp, (n, out.shape[0], exp)
        assert torch.equal(out[:n], torch.ones((n, 4))) and (out[n:] == 0).all()
        out = B.padding(torch.ones((4, n)), 1)
        assert out.shape[1] == exp


def test_zipf_expert_counts_generator():
    from tests import _gen as G

    counts, padded = G.zipf_counts(8192, 32, 1.1, seed=3)
    assert counts.sum() == 8192 and (counts == 0).sum() >= 2
    assert (padded % 128 == 0).all() and (padded >= counts).all() and (padded - counts < 128).all()
    c2, _ = G.zipf_counts(8192, 32, 1.1, seed=3)
    assert np.array_equal(counts, c2)


def test_ernie_and_inference_mirrors_host_logic_without_a_gpu():
    """The host logic of the ERNIE wrappers and of the inference-style linear that needs no kernel: the
    padding rule, the config switch lookup, the cached-weight lookup, the scale registration, the plain
    linear on a wide weight; quantised work on CPU tensors raises instead of falling back."""
    from paddleformers_amd import ernie_fp8_linear as EL
    from paddleformers_amd import ernie_fp8_utils as EU
    from paddleformers_amd import fp8_linear as FL
    from paddleformers_amd import kernel as K8

    for n in (1, 128, 300, 384, 512, 900):
        exp = n if n % 512 == 0 else (n // 512 + 1) * 512
        assert EL.padding(torch.ones((n, 4)), 0).shape[0] == exp and EL.padding(torch.ones((4, n)), 1).shape[1] == exp
    assert EU.has_config({"spaq": True}, "spaq") and not EU.has_config({"spaq": False}, "spaq") and not EU.has_config({}, "spaq")

    class W:
        pass

    w = W()
    w.fp8_weight_stacked, w.fp8_scale_stacked = "q", "s"
    w.fp8_weight_stacked_transpose, w.fp8_scale_stacked_transpose = "qt", "st"
    assert EU.fused_stack_transpose_quant([w], transpose=False) == ("q", "s")
    assert EU.fused_stack_transpose_quant([w], transpose=True) == ("qt", "st")

    layer = FL.Linear(300, 200, bias=True, dtype=torch.float8_e4m3fn, device="cpu")
    assert tuple(layer.weight_scale_inv.shape) == (3, 2) and layer.weight._scale is layer.weight_scale_inv
    plain = FL.Linear(8, 4, bias=True, dtype=torch.float32, device="cpu")
    assert not hasattr(plain, "weight_scale_inv")
    x = torch.ones((2, 8))
    assert torch.equal(plain(x), x @ plain.weight + plain.bias)
    with pytest.raises(RuntimeError, match="no CPU path"):
        layer(torch.ones((2, 300), dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="no CPU path"):
        K8.act_quant(torch.zeros((4, 128), dtype=torch.bfloat16))
    with pytest.raises(AssertionError):
        K8.act_quant(torch.zeros((4, 100), dtype=torch.bfloat16))


def _remark(name, scratch):
    tag = "[-Rpass-analysis=kernel-resource-usage]"
    return [f"x.hip:1:1: remark: Function Name: {name} {tag}", f"x.hip:1:1: remark:     VGPRs: 200 {tag}",
            f"x.hip:1:1: remark:     ScratchSize [bytes/lane]: {scratch} {tag}", f"x.hip:1:1: remark:     VGPRs Spill: 0 {tag}"]


def test_build_scratch_check_on_canned_remarks(monkeypatch):
    """The build refuses a kernel that spills to scratch, can be told to warn instead, and fails when the remarks it
    reads are missing rather than passing vacuously."""
    from paddleformers_amd import build as B

    clean = [l for k in B.EXPECTED_KERNELS for l in _remark(f"_ZN3pf8{len(k)}{k}ILi0EEEvNS_8GemmArgsE", 0)]
    seen, spilling = B.kernels_with_scratch(clean)
    assert len(seen) == len(B.EXPECTED_KERNELS) and spilling == []
    assert B.check_scratch(clean) == ""
    dirty = clean + _remark("_ZN3pf814k_rms_norm_fwdILi2EEEvPKt", 156)
    monkeypatch.delenv("PF8_ALLOW_SCRATCH", raising=False)
    with pytest.raises(RuntimeError, match="k_rms_norm_fwd.*156"):
        B.check_scratch(dirty)
    monkeypatch.setenv("PF8_ALLOW_SCRATCH", "1")
    assert B.check_scratch(dirty).startswith("warning:") and "156" in B.check_scratch(dirty)
    # remarks in a wording the parser does not know: nothing is seen, and that is an error of its own
    reworded = [l.replace("ScratchSize [bytes/lane]:", "Scratch bytes per lane =") for l in dirty]
    with pytest.raises(RuntimeError, match="resource remarks not found"):
        B.check_scratch(reworded)
    with pytest.raises(RuntimeError, match="resource remarks not found"):
        B.check_scratch(["clang: warning: something else"])


def test_packed_expert_results_behave_like_the_lists_the_reference_returns():
    """fused_transpose_split_quant hands its per-expert tensors out as views made on demand; code written for the
    reference's Python lists (indexing, negative indices, slices, iteration, len, concatenation) must not notice."""
    import torch

    from paddleformers_amd.functional import _PackedExperts

    rows, K = [256, 0, 128, 384], 4
    q = torch.arange(sum(rows) * K, dtype=torch.int32)
    s = torch.arange((sum(rows) // 128) * K, dtype=torch.float32)
    pq, ps = _PackedExperts(q, rows, K, False), _PackedExperts(s, rows, K, True)
    assert len(pq) == len(ps) == 4
    off = 0
    for e, r in enumerate(rows):
        assert pq[e].shape == (K, r) and ps[e].shape == (r // 128, K)
        assert torch.equal(pq[e].reshape(-1), q[off * K:(off + r) * K])
        assert torch.equal(ps[e].reshape(-1), s[(off // 128) * K:((off + r) // 128) * K])
        assert pq[e].data_ptr() == q.data_ptr() + off * K * 4 or r == 0        # views, not copies
        off += r
    assert pq[-1] is pq[3] and pq[1].numel() == 0
    assert [t.shape for t in pq[1:3]] == [(K, 0), (K, 128)]
    assert [t.shape[1] for t in pq] == rows
    both = pq + ps
    assert isinstance(both, list) and len(both) == 8 and both[4] is ps[0]
    assert ([pq[0]] + ps)[1] is ps[0]
    with pytest.raises(IndexError):
        pq[4]
    (only,), = [_PackedExperts(q[:128 * K], [128], K, False)]
    assert only.shape == (K, 128)



def test_build_scans_inline_assembly_for_scalar_address_hazards():
    """A vector-memory instruction may read a scalar address register the vector unit wrote only five wait states later;
    the compiler pads its own instructions but not inline assembly, so the build scans the device assembly itself."""
    from paddleformers_amd.build import sgpr_address_hazards

    bad = "\tv_readlane_b32 s0, v225, 47\n\tv_readlane_b32 s1, v225, 48\n\tglobal_atomic_add v196, v178, v198, s[0:1] sc0\n"
    hz = sgpr_address_hazards(bad)
    assert [(h[2], h[3]) for h in hz] == [(0, 1), (1, 0)]
    padded = "\tv_readlane_b32 s0, v225, 47\n\tv_readlane_b32 s1, v225, 48\n\ts_nop 4\n\tglobal_atomic_add v196, v178, v198, s[0:1] sc0\n"
    assert sgpr_address_hazards(padded) == []
    far = "\tv_readfirstlane_b32 s4, v1\n" + "\tv_mov_b32_e32 v2, v3\n" * 5 + "\tglobal_load_dwordx4 v[0:3], v8, s[4:5]\n"
    assert sgpr_address_hazards(far) == []
    near = "\tv_readfirstlane_b32 s4, v1\n" + "\tv_mov_b32_e32 v2, v3\n" * 4 + "\tglobal_load_dwordx4 v[0:3], v8, s[4:5]\n"
    assert len(sgpr_address_hazards(near)) == 1
