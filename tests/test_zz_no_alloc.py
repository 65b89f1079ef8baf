"""GPU test of the allocation-free grouped UE8M0 GEMM entry point, through the raw C ABI: its output must
be bit-identical to pf8_grouped_items_build + pf8_grouped_gemm_nt_contiguous_ue8m0 (itself checked against the
oracle in tests/test_gpu_gemm_ue8m0.py), on two calls in a row that share the built-in work-item list, the
second with a smaller input, and no device memory may be allocated while it runs."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


def _case(rows, N, K, seed):
    E, Mtot = len(rows), int(sum(rows))
    a, sa = O.quant_1x128(G.bf16_normal((Mtot, K), seed=seed, outlier_frac=1e-3, outlier_scale=30.0), 1, pow2=True)     # scales [K/128, Mtot]
    bs, sbs = [], []
    for e in range(E):
        b, sb, _, _ = O.quant_128x128(G.bf16_normal((N, K), seed=seed + 10 + e, std=0.02), pow2=True)
        bs.append(b)
        sbs.append(sb)
    t = dict(a=G.to_torch_fp8(a), sa=torch.from_numpy(O.scales_to_ue8m0(sa)).cuda(), b=G.to_torch_fp8(np.stack(bs)),
             sb=torch.from_numpy(O.scales_to_ue8m0(np.stack(sbs))).cuda(),
             m=torch.from_numpy(np.repeat(np.arange(E, dtype=np.int32), rows)).cuda())
    return t, (a, sa, np.stack(bs), np.stack(sbs)), E, Mtot


def _with_list(lib, t, E, Mtot, N, K, st):
    items = torch.empty(4 + 4 * (Mtot // 128), dtype=torch.int32, device="cuda")
    out = torch.full((Mtot, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    lib.call("pf8_grouped_items_build", t["m"].data_ptr(), Mtot, items.data_ptr(), st)
    lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0", t["a"].data_ptr(), t["sa"].data_ptr(), t["sa"].stride(0), t["b"].data_ptr(),
             t["sb"].data_ptr(), E, Mtot, N, K, t["m"].data_ptr(), items.data_ptr(), out.data_ptr(), st)
    return out


@pytest.mark.parametrize("cus", [0, 8])      # 8: the paired 256-row tiles (the kernel that reads the list items) take these small loads
def test_no_alloc_entry_point_matches_the_caller_built_list(cus):
    from paddleformers_amd import _lib as lib

    lib.lib().pf8_set_num_cus(cus)
    try:
        N, K = 512, 1024
        st = torch.cuda.current_stream().cuda_stream
        first, first_np, E1, M1 = _case([640, 128, 0, 384, 256, 768], N, K, seed=1)
        second, _, E2, M2 = _case([256, 128], N, K, seed=2)
        exp1 = _with_list(lib, first, E1, M1, N, K, st)
        exp2 = _with_list(lib, second, E2, M2, N, K, st)
        out1 = torch.full((M1, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        out2 = torch.full((M2, N), float("nan"), dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        reserved, allocated = torch.cuda.memory_reserved(), torch.cuda.memory_allocated()
        free_before = torch.cuda.mem_get_info()[0]
        for t, E, M, out in ((first, E1, M1, out1), (second, E2, M2, out2)):      # back to back: the second call overwrites the list
            lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0_noalloc", t["a"].data_ptr(), t["sa"].data_ptr(), t["sa"].stride(0),
                     t["b"].data_ptr(), t["sb"].data_ptr(), E, M, N, K, t["m"].data_ptr(), out.data_ptr(), st)
        torch.cuda.synchronize()
        assert torch.cuda.memory_reserved() == reserved and torch.cuda.memory_allocated() == allocated
        assert torch.cuda.mem_get_info()[0] >= free_before          # nothing was taken from the device either
        assert torch.equal(out1.view(torch.int16), exp1.view(torch.int16))
        assert torch.equal(out2.view(torch.int16), exp2.view(torch.int16))
        # and the numbers are the oracle's
        a, sa, b, sb = first_np
        ref = O.grouped_gemm_nt_contiguous(a, np.ascontiguousarray(sa.T), b, sb, first["m"].cpu().numpy())
        assert G.rel_fro(O.bf16_bits_to_f32(G.from_torch_bf16(out1)), O.bf16_bits_to_f32(ref)) <= 8e-4
    finally:
        lib.lib().pf8_set_num_cus(0)


def test_no_alloc_entry_point_rejects_more_rows_than_its_list_holds():
    from paddleformers_amd import _lib as lib

    buf = torch.zeros(64, dtype=torch.uint8, device="cuda")
    p = buf.data_ptr()
    with pytest.raises(ValueError, match="1,048,576 rows"):
        lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0_noalloc", p, p, 128 * 8193, p, p, 1, 128 * 8193, 512, 1024, p, p, None)
    with pytest.raises(ValueError):
        lib.call("pf8_grouped_gemm_nt_contiguous_ue8m0_noalloc", p, p, 200, p, p, 1, 200, 512, 1024, p, p, None)
