"""GPU parity of moe_permute / moe_unpermute against the numpy oracle (bit for bit: the operators
only move rows, and the way back sums in fp32 in slot order), plus size-independent properties at
the full config 5 size.  The operators' home is a binary the reference does not ship; the oracle
restates what the reference's call sites rely on (see oracle/pf8_oracle.py)."""
import numpy as np
import pytest

from oracle import pf8_oracle as O
from tests import _gen as G

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def F():
    from paddleformers_amd import _lib
    from paddleformers_amd import functional as F8

    _lib.lib()
    return F8


def routing(T, topk, E, seed, drop=0.1):
    rng = np.random.default_rng(seed)
    rm = np.stack([rng.permutation(E)[:topk] for _ in range(T)]).astype(np.int32) if T else np.zeros((0, topk), np.int32)
    rm[rng.random(rm.shape) < drop] = -1
    counts = [int((rm == e).sum()) for e in range(E)]
    probs = rng.random(rm.shape).astype(np.float32)
    return rm, probs, counts


@pytest.mark.parametrize("T,H,topk,E,align", [(37, 256, 4, 8, 128), (300, 1408, 2, 5, 128), (64, 7168, 8, 16, 128), (9, 128, 1, 3, 16), (1, 128, 3, 4, 128)])
def test_permute_unpermute_bf16(F, T, H, topk, E, align):
    rm, probs, counts = routing(T, topk, E, seed=T + H)
    bits = G.bf16_normal((T, H), seed=T * 3 + 1)
    ox, orow, op, _ = O.moe_permute(bits, None, rm, probs, E, counts, align)
    x = G.to_torch_bf16(bits)
    gx, grow, gp, gs = F.moe_permute(x, None, torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda(), E, counts, align)
    assert gs is None
    assert (grow.cpu().numpy() == orow).all(), "row map"
    assert (G.from_torch_bf16(gx) == ox).all(), "permuted rows (padding rows are zero)"
    assert (gp.cpu().numpy() == op).all(), "permuted probabilities"
    # rows of one expert keep token order
    for e in range(E):
        col = orow[:, e][orow[:, e] >= 0]
        assert (np.diff(col) == 1).all()
    # the way back: a different tensor in the permuted layout, e.g. the expert outputs
    ubits = G.bf16_normal(ox.shape, seed=7)
    eo, ep = O.moe_unpermute(ubits, orow, rm, op, T, E)
    go, gpp = F.moe_unpermute(G.to_torch_bf16(ubits), grow, torch.from_numpy(rm).cuda(), gp, T, E)
    assert (G.from_torch_bf16(go) == eo).all(), "summed rows"
    assert (gpp.cpu().numpy() == ep).all() and (ep[rm >= 0] == probs[rm >= 0]).all(), "probabilities back in [T, topk] order"


def test_permute_fp8_with_scales(F):
    T, H, topk, E = 130, 512, 4, 6
    rm, probs, counts = routing(T, topk, E, seed=3)
    rng = np.random.default_rng(4)
    q = rng.integers(0, 255, size=(T, H), dtype=np.uint8)
    s = rng.random((T, H // 128)).astype(np.float32)
    ox, orow, op, osc = O.moe_permute(q, s, rm, probs, E, counts, 128)
    gx, grow, gp, gs = F.moe_permute(G.to_torch_fp8(q), torch.from_numpy(s).cuda(), torch.from_numpy(rm).cuda(),
                                     torch.from_numpy(probs).cuda(), E, counts, 128)
    assert (G.from_torch_fp8(gx) == ox).all() and (grow.cpu().numpy() == orow).all()
    assert (gs.cpu().numpy() == osc).all() and (gp.cpu().numpy() == op).all()


def test_full_size_round_trip_properties(F):
    """Config 5 sized: 16384 tokens x top-8 over 128 experts, H = 4096.  With small-integer rows the
    sums are exact: unpermute(permute(x)) == (routed slots of the token) * x; every padded segment
    is a multiple of 128 rows; the row map is a bijection onto the non-padding rows."""
    T, H, topk, E = 16384, 4096, 8, 128
    rm, probs, counts = routing(T, topk, E, seed=5, drop=0.0)
    rng = np.random.default_rng(6)
    xv = rng.integers(-8, 9, size=(T, H)).astype(np.float32)
    x = torch.from_numpy(xv).cuda().to(torch.bfloat16)
    gx, grow, gp, _ = F.moe_permute(x, None, torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda(), E, counts, 128)
    assert gx.shape[0] == sum((c + 127) // 128 * 128 for c in counts)
    rows = grow[grow >= 0]
    assert rows.numel() == T * topk and torch.unique(rows).numel() == T * topk
    back, pb = F.moe_unpermute(gx, grow, torch.from_numpy(rm).cuda(), gp, T, E)
    assert torch.equal(back.float(), (x.float() * topk))
    assert torch.equal(pb.cpu(), torch.from_numpy(probs))
    # padding rows are zero and carry probability 0
    used = torch.zeros(gx.shape[0], dtype=torch.bool, device="cuda")
    used[rows.long()] = True
    assert not gx[~used].any() and not gp[~used].any()


def test_permute_rejects_inconsistent_counts_and_bad_arguments(F):
    T, H, topk, E = 20, 128, 2, 4
    rm, probs, counts = routing(T, topk, E, seed=9, drop=0.0)
    x = G.to_torch_bf16(G.bf16_normal((T, H), seed=1))
    short = list(counts)
    short[int(np.argmax(counts))] -= 1
    with pytest.raises(ValueError, match="tokens_per_expert"):
        F.moe_permute(x, None, torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda(), E, short, 128, validate=True)
    # a count that overstates what the routing sends: flagged, and with the check skipped the rows no token
    # lands on hold zeros (probability 0), like padding rows, not whatever the allocation held
    big = int(np.argmax(counts))
    over = list(counts)
    over[big] += 3
    with pytest.raises(ValueError, match="fewer tokens"):
        F.moe_permute(x, None, torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda(), E, over, 128, validate=True)
    torch.full((E * 256, H), float("nan"), dtype=torch.bfloat16, device="cuda")     # poison what the allocator hands out next
    ox, orow, op, _ = F.moe_permute(x, None, torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda(), E, over, 128)
    # the default call reads nothing back: the flag stays on the device until somebody asks, and asking clears it
    with pytest.raises(ValueError, match="fewer tokens"):
        F.moe_permute_check()
    F.moe_permute_check()
    start = sum((c + 127) // 128 * 128 for c in over[:big])
    assert not ox[start + counts[big]:start + over[big]].any() and not op[start + counts[big]:start + over[big]].any()
    gx, _, gp, _ = F.moe_permute(x, None, torch.from_numpy(rm).cuda(), torch.from_numpy(probs).cuda(), E, counts, 128)
    assert torch.equal(ox[start:start + counts[big]], gx[start:start + counts[big]])
    with pytest.raises(ValueError):
        F.moe_permute(x, None, torch.from_numpy(rm).cuda(), None, E, counts[:-1], 128)
    with pytest.raises(RuntimeError):
        F.moe_permute(x.cpu(), None, torch.from_numpy(rm), None, E, counts, 128)
    with pytest.raises(ValueError):
        F.moe_permute(x.float(), None, torch.from_numpy(rm).cuda(), None, E, counts, 128)
    ox, orow, op, _ = F.moe_permute(torch.zeros((0, H), dtype=torch.bfloat16, device="cuda"), None,
                                    torch.zeros((0, topk), dtype=torch.int32, device="cuda"), None, E, [0] * E, 128)
    assert ox.shape == (0, H) and orow.shape == (0, E)
