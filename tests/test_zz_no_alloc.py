"""The layer entry point that runs on the library's static scratch (no workspace argument, no
allocation) against the workspace entry point: same bits, on two calls in a row, the second
smaller than the first (the scratch then still holds the first call's contents)."""
import pytest
import torch

from tests.helpers import Layer, gen, tokens

pytestmark = pytest.mark.gpu


def _inputs(T, H, E, K, n, seed):
    g = gen(seed)
    x = tokens(T, H, seed).cuda()
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32).cuda()
    w = torch.rand(T, K, generator=g).cuda()
    return x, w, ids


@pytest.mark.parametrize("rows_dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_entry_matches_workspace_entry(rows_dtype):
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    H, I, n, E, K = 7168, 2048, 8, 16, 4
    lay = Layer(n, H, I, seed=91, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    lo = 3   # local experts are global ids 3..10: some assignments fall outside and are dropped
    for T, seed in ((64, 92), (17, 93)):   # about 16 and 4 rows per local expert: the weight-streaming kernels
        x, w, ids = _inputs(T, H, E, K, n, seed)
        want = ops.moe_w8a8_layer(x, None, w, ids, lo, lo + n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I,
                                  rows_dtype=rows_dtype)
        out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]   # allocations made so far
        got = ops.moe_w8a8_layer_static(x, None, w, ids, lo, lo + n, d["w13"], d["s13"], d["w2"], d["s2"], shared,
                                        H=H, I=I, out=out, rows_dtype=rows_dtype)
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "the wrapper allocated through torch"
        torch.cuda.synchronize()
        assert got.data_ptr() == out.data_ptr()
        assert bool(torch.isfinite(got.float()).all())
        assert torch.equal(got, want), f"T={T}: static-scratch result differs from the workspace entry's"


@pytest.mark.parametrize("case", ["int8_tokens", "no_shared_expert"])
def test_static_scratch_entry_other_inputs(case):
    """Tokens that arrive quantised (int8 + scales) and a layer without the shared expert (another scratch layout)
    on the static scratch, two calls in a row, the second smaller: the bits of the workspace entry."""
    from omni_infer_amd import hip_ops as ops
    H, I, n, E, K = 2048, 1024, 8, 16, 4
    with_shared = case != "no_shared_expert"
    lay = Layer(n, H, I, seed=95, shared=with_shared)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"]) if with_shared else None
    for T, seed in ((64, 96), (20, 97)):
        x, w, ids = _inputs(T, H, E, K, n, seed)
        xs = None
        if case == "int8_tokens":
            x, xs = ops.npu_dynamic_quant(x)
        want = ops.moe_w8a8_layer(x, xs, w, ids, 0, n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I)
        out = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device="cuda")
        got = ops.moe_w8a8_layer_static(x, xs, w, ids, 0, n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I, out=out)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"{case} T={T}"


def test_static_scratch_entry_rejects_what_does_not_fit():
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    H, I, n, K = 7168, 2048, 32, 8
    T = 4096
    assert L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n, H, I, 1, L.OMNI_DT_F32) > L.OMNI_STATIC_SCRATCH_BYTES
    x = torch.zeros(T, H, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(T, K, device="cuda")
    ids = torch.zeros(T, K, dtype=torch.int32, device="cuda")
    p = x   # any valid device pointer: the size check comes before anything is read
    with pytest.raises(RuntimeError, match="static scratch"):
        ops.moe_w8a8_layer_static(x, None, w, ids, 0, n, p, p, p, p, None, H=H, I=I)
