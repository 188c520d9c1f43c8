"""The gate projection on the fp32 matrix cores (fixed summation order) and its fusion with the router,
against the CPU oracle: logits, routing ids and routing weights bit exact."""
import types

import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import gen, tokens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available()
    from omni_infer_amd import hip_ops
    return hip_ops


def _bits_equal(a, b):
    return torch.equal(a.cpu().contiguous().view(torch.int32), b.cpu().contiguous().view(torch.int32))


@pytest.mark.parametrize("T,H,E,xdt,wdt", [
    (64, 7168, 256, torch.bfloat16, torch.float32),    # the decode configuration
    (1, 7168, 256, torch.bfloat16, torch.float32),
    (130, 1024, 160, torch.bfloat16, torch.float32),   # ragged token and expert tiles, one group of slices
    (33, 1152, 8, torch.float32, torch.float32),       # fp32 tokens (the reference's hidden_states.float()), 9 slices
    (40, 2048, 64, torch.bfloat16, torch.bfloat16),    # bf16 gate
])
def test_gate_logits_bit_exact(ops, T, H, E, xdt, wdt):
    g = gen(7)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(xdt)
    w = (torch.randn(E, H, generator=g) * 0.02).to(wdt)
    ref = O.gate_logits_spec(x, w, round_bf16=wdt == torch.bfloat16)
    got = ops.gate_logits(x.cuda(), w.cuda(), round_logits_bf16=wdt == torch.bfloat16)
    assert got.shape == (T, E) and got.dtype == torch.float32
    assert _bits_equal(got, ref), f"{int((got.cpu() != ref).sum())} of {ref.numel()} logits differ"
    assert float((got.cpu().double() - x.double() @ w.double().t()).abs().max()) < 1e-2


def test_gate_logits_do_not_depend_on_the_batch(ops):
    """Small batches give one slice of 128 to a wavefront, large ones a group of 8 slices; a token's logits
    must be the same bits in both (and whatever its position in the batch)."""
    g = gen(8)
    H, E = 7168, 256
    x = torch.randn(4096, H, generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn(E, H, generator=g) * 0.02).cuda()
    big = ops.gate_logits(x, w)
    small = ops.gate_logits(x[1000:1064].contiguous(), w)
    one = ops.gate_logits(x[4095:4096].contiguous(), w)
    assert _bits_equal(big[1000:1064], small) and _bits_equal(big[4095:4096], one)
    ref = O.gate_logits_spec(x[1000:1008].cpu(), w.cpu())
    assert _bits_equal(big[1000:1008], ref)


@pytest.mark.parametrize("xdt,wdt", [(torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                     (torch.float32, torch.float32), (torch.float32, torch.bfloat16)])
def test_gate_logits_large_batch_kernel(ops, xdt, wdt):
    """From 2048 tokens on a block of four wavefronts passes the operands through LDS (128 tokens x 64 experts
    x a group of 8 slices).  Ragged token and expert tiles, a last group of 2 slices; the result must be the
    bits of the small-batch kernel (64 tokens at a time) and of the oracle."""
    g = gen(9)
    T, H, E = 2048 + 77, 7168 + 256, 160
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(xdt).cuda()
    w = (torch.randn(E, H, generator=g) * 0.02).to(wdt).cuda()
    rb = wdt == torch.bfloat16
    big = ops.gate_logits(x, w, round_logits_bf16=rb)
    assert big.shape == (T, E)
    for t0 in (0, 64, 1024, 2048, 2112):
        small = ops.gate_logits(x[t0:t0 + 64].contiguous(), w, round_logits_bf16=rb)
        assert _bits_equal(big[t0:t0 + 64], small), f"tokens {t0}.."
    rows = torch.tensor([0, 63, 64, 127, 128, 2047, 2124])
    ref = O.gate_logits_spec(x[rows.cuda()].cpu(), w.cpu(), round_bf16=rb)
    assert _bits_equal(big[rows.cuda()], ref)


@pytest.mark.parametrize("T,H,E", [(64, 7168, 256), (7, 1024, 64)])
def test_gate_route_fused_equals_two_steps_and_oracle(ops, T, H, E):
    """omni_moe_gate_route = gate logits + the sigmoid/bias grouped router, one call: ids and weights equal
    those of the router run on the library's own logits, and those of the oracle end to end."""
    from omni_infer_amd.layers.layer import FusedMoE
    g = gen(9)
    x = tokens(T, H, 9)
    w = torch.randn(E, H, generator=g) * 0.05
    bias = torch.randn(E, generator=g) * 0.01
    ng, tg, K = (8, 4, 8) if E == 256 else (4, 2, 6)
    logits_ref = O.gate_logits_spec(x, w)
    w_ref, id_ref = O.route_noaux_tc(logits_ref, bias, K, ng, tg, 2.5)
    tw, ids, row, logits = FusedMoE.gate_and_select_experts(x.cuda(), w.cuda(), K, True, True, tg, ng, None, "sigmoid",
                                                             bias.cuda(), 2.5, want_logits=True)
    assert _bits_equal(logits, logits_ref)
    assert torch.equal(ids.cpu(), id_ref) and torch.equal(tw.cpu(), w_ref)
    tw2, ids2, _ = FusedMoE.select_experts(x.cuda(), ops.gate_logits(x.cuda().float(), w.cuda()), K, True, True, tg, ng,
                                           None, "sigmoid", bias.cuda(), 2.5)
    assert torch.equal(ids2, ids) and torch.equal(tw2, tw)
    # the other two routers through the same entry
    wg_ref, idg_ref, _ = O.route_grouped_topk(logits_ref, K, True, ng, tg, "softmax", None)
    tw, ids, _, _ = FusedMoE.gate_and_select_experts(x.cuda(), w.cuda(), K, True, True, tg, ng, None, "softmax", None, 2.5)
    assert torch.equal(ids.cpu(), idg_ref) and torch.equal(tw.cpu(), wg_ref * 2.5)
    ws_ref, ids_ref, _ = O.route_softmax_topk(logits_ref, 2, True)
    tw, ids, _, _ = FusedMoE.gate_and_select_experts(x.cuda(), w.cuda(), 2, False, True)
    assert torch.equal(ids.cpu(), ids_ref) and torch.equal(tw.cpu(), ws_ref)


def test_block_with_its_own_gate_against_oracle(ops):
    """The whole block (gate included) against the oracle with nothing shared but the inputs: DeepSeek-V3
    widths, 4 local experts of 32, 64 tokens, both bodies of the block."""
    from tests import test_gpu_layer as tl
    from omni_infer_amd import _lib as L, config, distributed
    env = types.SimpleNamespace(L=L, ops=ops, config=config, dist=distributed)
    blk, lay, gate_w, bias, lo = tl._dsv3_block(env, 4, 8, 2)
    x = tokens(64, 7168, 71)
    logits_ref = O.gate_logits_spec(x, gate_w)
    out_ref, st = tl._block_reference(lay, x, logits_ref, bias, lo, 4)
    for fused in (True, False):
        blk.fused = fused
        out, _ = blk(x.cuda(), None, None, 3)
        assert torch.equal(out.float().cpu(), out_ref.float()), f"fused={fused}"


def test_gate_argument_errors(ops):
    x = torch.zeros(4, 100, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(8, 100, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ops.gate_logits(x, w)
    with pytest.raises(ValueError):
        ops.gate_logits(x, torch.zeros(8, 128, device="cuda"))
    with pytest.raises(ValueError):
        ops.gate_logits(x.to(torch.float16), w)


def test_unquantised_replicated_linear_that_is_not_a_gate():
    """A replicated linear the ``ignore`` list keeps unquantised, with a width the gate kernel does not take (7168
    outputs), or fp16 parameters: the plain product of the reference's unquantised linear method, not an error."""
    from omni_infer_amd.layers.linear import ReplicatedLinear
    from omni_infer_amd.quantization.compressed_tensors import AscendCompressedTensorsConfig
    cfg = AscendCompressedTensorsConfig(ignore=["down_proj"])
    g = torch.Generator().manual_seed(5)
    lin = ReplicatedLinear(2048, 7168, bias=False, quant_config=cfg, params_dtype=torch.bfloat16,
                           prefix="model.layers.3.mlp.shared_experts.down_proj", device="cuda")
    assert lin.quant_method is None
    lin.weight.data.copy_((torch.randn(7168, 2048, generator=g) * 0.02).to(torch.bfloat16))
    x = torch.randn(5, 2048, generator=g).to(torch.bfloat16).cuda()
    out, _ = lin(x)
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (5, 7168)
    want = x.float().cpu() @ lin.weight.data.float().cpu().t()
    assert float((out.float().cpu() - want).norm() / want.norm()) < 1e-2
    half = ReplicatedLinear(256, 64, bias=False, quant_config=None, params_dtype=torch.float16, prefix="gate", device="cuda")
    half.weight.data.copy_((torch.randn(64, 256, generator=g) * 0.05).to(torch.float16))
    out, _ = half(torch.randn(3, 256, generator=g).to(torch.float16).cuda())
    assert out.dtype == torch.float16 and tuple(out.shape) == (3, 64)
