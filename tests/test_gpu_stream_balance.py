"""The weight-streaming GEMM1 with its overflow blocks cut along k (shares on helper blocks, partial sums handed
over through device memory, the last share to arrive finishing the block) against the same launch uncut: the
same bits, at shapes where the cut is made, through the layer entry and through the operator entry with a
workspace whose counters the caller has zeroed once."""
import pytest
import torch

from tests.helpers import Layer, gen, tokens

pytestmark = pytest.mark.gpu

H, I = 7168, 2048   # blocks of 917 KB: the cut pays from a few dozen overflow blocks on


def _routing(T, E, K, seed):
    g = gen(seed)
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32).cuda()
    w = torch.rand(T, K, generator=g).cuda()
    return w, ids


@pytest.mark.parametrize("T,n_local", [(64, 9), (16, 9), (3, 12)])
def test_layer_with_and_without_the_cut(tuning, T, n_local):
    """9 local experts + the shared one at 64 tokens are 11 row blocks x 32 column blocks = 352 blocks on 256 compute
    units: 96 overflow blocks, cut 2 or 4 ways.  16 tokens: 10 x 32 = 320 blocks, 64 overflow blocks.  3 tokens on
    12 experts: about 9 x 32 blocks."""
    from omni_infer_amd import hip_ops as ops
    K = 4
    lay = Layer(n_local, H, I, seed=301, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    x = tokens(T, H, 302 + T).cuda()
    w, ids = _routing(T, n_local, K, 303 + T)
    outs = {}
    for setting in (0, 1):
        tuning(OMNI_MOE_STREAM_BALANCE=setting)
        for rep in range(3):   # the counters are left at zero: a second and third call on the same workspace agree
            out = ops.moe_w8a8_layer(x, None, w, ids, 0, n_local, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I)
            torch.cuda.synchronize()
            if rep == 0:
                outs[setting] = out.clone()
            else:
                assert torch.equal(out, outs[setting]), f"call {rep} differs from the first, balance={setting}"
    assert bool(torch.isfinite(outs[1].float()).all())
    assert torch.equal(outs[0], outs[1]), "the layer with its overflow blocks cut along k differs from the uncut launch"


def test_operator_entry_with_zeroed_workspace(tuning):
    """omni_moe_gemm1_swiglu_quant with OMNI_GEMM1_WS_ZEROED on a workspace zero-filled once: three calls in a row
    (the kernel leaves its counters at zero), int8 rows and scales equal to the call without the flag and to the
    uncut launch."""
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    n_local, T, K = 9, 64, 4
    lay = Layer(n_local, H, I, seed=311, shared=True)
    d = lay.to_device()
    x = tokens(T, H, 312).cuda()
    _, ids = _routing(T, n_local, K, 313)
    xq, xs = ops.npu_dynamic_quant(x)
    p = ops.moe_permute(ids, 0, n_local, L.OMNI_IDX_TOKEN_MAJOR)
    M_cap = T * K + T

    def run(flags, ws):
        hq, hs, _ = ops.grouped_gemm1_swiglu_quant(xq, xs, p.sorted_src, L.OMNI_IDX_TOKEN_MAJOR, K, d["w13"], d["s13"],
                                                   p.offsets, H, I, M_cap, extra=(d["sh13"], d["sh_s13"]), extra_rows=T,
                                                   flags=flags, workspace=ws)
        torch.cuda.synchronize()
        return hq.clone(), hs.clone()

    kept = int(p.offsets[-1].item()) + T   # rows the groups own; the rest of the capacity is never written
    tuning(OMNI_MOE_STREAM_BALANCE=0)
    want_q, want_s = run(0, None)
    tuning(OMNI_MOE_STREAM_BALANCE=1)
    got_q, got_s = run(0, None)
    assert torch.equal(got_q[:kept], want_q[:kept]) and torch.equal(got_s[:kept], want_s[:kept])
    ws = torch.zeros(L.lib().omni_moe_gemm1_workspace_bytes(T, K, n_local, T, M_cap, H, I), dtype=torch.uint8, device="cuda")
    for rep in range(3):
        q, s = run(L.OMNI_GEMM1_WS_ZEROED, ws)
        assert torch.equal(q[:kept], want_q[:kept]) and torch.equal(s[:kept], want_s[:kept]), f"flagged call {rep}"
