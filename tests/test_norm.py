"""Residual add + RMSNorm (+ dynamic quantisation): the oracle pinned against independent routines
and closed forms (CPU), the HIP kernel against the oracle bit for bit (GPU)."""
import math

import pytest
import torch

from oracle import moe_oracle as O
from tests.helpers import gen


def _inputs(T, H, seed, scale=1.0):
    g = gen(seed)
    x = (torch.randn(T, H, generator=g) * scale).to(torch.bfloat16)
    r = (torch.randn(T, H, generator=g) * 3.0).to(torch.bfloat16)
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
    return x, r, w


# ------------------------------------------------------------------ oracle pins (CPU)
def test_oracle_add_rms_norm_against_fp64_library_routine():
    """torch.nn.functional.rms_norm in fp64 on the fp32 sum is the independent routine: the oracle's
    bf16 result may differ from the rounded fp64 result by one bf16 step at most, and only rarely."""
    x, r, w = _inputs(16, 7168, 1)
    y, res = O.add_rms_norm(x, r, w, 1e-6)
    s = x.float() + r.float()
    assert torch.equal(res, s.to(torch.bfloat16))               # the residual leaves as the rounded sum
    ref = torch.nn.functional.rms_norm(s.double(), (7168,), w.double(), 1e-6)
    ref_bf = ref.to(torch.bfloat16)
    diff = (y.float() - ref_bf.float()).abs()
    ulp = (ref_bf.float().abs() * 2.0 ** -7).clamp(min=1e-30)
    assert bool((diff <= ulp).all())
    assert float((diff > 0).float().mean()) < 0.02


def test_oracle_add_rms_norm_closed_forms():
    H = 1024
    w = torch.full((H,), 0.5, dtype=torch.bfloat16)
    # constant rows: mean(s^2) = c^2 exactly, y = c / sqrt(c^2 + eps) * w
    for c in (1.0, -2.0, 0.25):
        x = torch.full((2, H), c, dtype=torch.bfloat16)
        y, _ = O.add_rms_norm(x, torch.zeros_like(x), w, 1e-6)
        f = torch.tensor(c, dtype=torch.float32)
        want = ((f * (1.0 / torch.sqrt(f * f + torch.tensor(1e-6)))) * 0.5).to(torch.bfloat16)
        assert bool((y == want).all())
    # a zero row stays zero (eps keeps the root finite), its quantisation is (0, 0)
    z = torch.zeros(1, H, dtype=torch.bfloat16)
    q, sc, res = O.add_rms_norm_dynamic_quant(z, z, w, 1e-6)
    assert int(q.abs().sum()) == 0 and float(sc[0]) == 0.0 and float(res.abs().sum()) == 0.0
    # no residual = residual of zeros
    x, _, w2 = _inputs(5, 2048, 3)
    y0, r0 = O.add_rms_norm(x, None, w2, 1e-5)
    y1, _ = O.add_rms_norm(x, torch.zeros_like(x), w2, 1e-5)
    assert r0 is None and torch.equal(y0, y1)


def test_oracle_rms_norm_scale_invariance_and_unit_rms():
    """Scaling the input by a power of two changes nothing when eps = 0 (every product is exact), and
    with unit weights the output has RMS 1 up to bf16 rounding."""
    x, r, _ = _inputs(8, 4096, 4)
    ones = torch.ones(4096, dtype=torch.bfloat16)
    y1, _ = O.add_rms_norm(x, r, ones, 0.0)
    y4, _ = O.add_rms_norm((x.float() * 4).to(torch.bfloat16), (r.float() * 4).to(torch.bfloat16), ones, 0.0)
    assert torch.equal(y1, y4)
    rms = y1.float().pow(2).mean(dim=-1).sqrt()
    assert bool(((rms - 1.0).abs() < 4e-3).all())


def test_oracle_norm_quant_is_the_quantisation_of_the_normalised_tensor():
    x, r, w = _inputs(6, 7168, 5)
    q, sc, res = O.add_rms_norm_dynamic_quant(x, r, w, 1e-6)
    y, res2 = O.add_rms_norm(x, r, w, 1e-6)
    # quantisation invariants on the normalised rows (they do not restate the formula)
    assert torch.equal(res, res2)
    assert bool((q.abs().amax(dim=-1) == 127).all())
    assert bool(((y.float() - q.float() * sc.unsqueeze(-1)).abs() <= sc.unsqueeze(-1) / 2 * (1 + 1e-6)).all())


def test_oracle_square_root_is_correctly_rounded():
    import numpy as np
    v = (torch.rand(200000, generator=gen(6)) * 50 + 1e-6).float()
    assert np.array_equal(O._sqrt_rn(v).numpy(), np.sqrt(v.numpy()))


# ------------------------------------------------------------------ kernel parity (GPU)
@pytest.mark.gpu
@pytest.mark.parametrize("T,H,eps", [(64, 7168, 1e-6), (3, 1024, 1e-5), (17, 7680, 1e-6), (1, 8, 1e-6), (5, 8192, 1e-6)])
def test_kernel_add_rms_norm_quant_bit_exact(T, H, eps):
    from omni_infer_amd import hip_ops as ops
    x, r, w = _inputs(T, H, 10 + T)
    if T > 2:
        x[1].zero_(); r[1].zero_()          # a zero row
    q_ref, s_ref, res_ref = O.add_rms_norm_dynamic_quant(x, r, w, eps)
    y_ref, _ = O.add_rms_norm(x, r, w, eps)
    y, res, q, sc = ops.add_rms_norm_quant(x.cuda(), r.cuda(), w.cuda(), eps, want_y=True, want_quant=True)
    assert torch.equal(res.cpu(), res_ref), "residual out"
    assert torch.equal(y.cpu(), y_ref), "normalised rows"
    assert torch.equal(sc.cpu(), s_ref), "per-token scales"
    assert torch.equal(q.cpu(), q_ref), "int8 rows"
    # the quantised-only form, residual updated in place
    rd = r.cuda().clone()
    y2, res2, q2, sc2 = ops.add_rms_norm_quant(x.cuda(), rd, w.cuda(), eps, want_y=False, want_quant=True,
                                               inplace_residual=True)
    assert y2 is None and res2.data_ptr() == rd.data_ptr()
    assert torch.equal(rd.cpu(), res_ref) and torch.equal(q2.cpu(), q_ref) and torch.equal(sc2.cpu(), s_ref)
    # no residual
    y3, res3, _, _ = ops.add_rms_norm_quant(x.cuda(), None, w.cuda(), eps)
    assert res3 is None and torch.equal(y3.cpu(), O.add_rms_norm(x, None, w, eps)[0])


@pytest.mark.gpu
def test_kernel_norm_argument_errors():
    from omni_infer_amd import hip_ops as ops
    x, r, w = _inputs(2, 1024, 0)
    with pytest.raises(ValueError):
        ops.add_rms_norm_quant(x.cuda().float(), r.cuda(), w.cuda(), 1e-6)
    with pytest.raises(RuntimeError):
        ops.add_rms_norm_quant(torch.zeros(2, 12, dtype=torch.bfloat16).cuda(), None,
                               torch.ones(12, dtype=torch.bfloat16).cuda(), 1e-6)      # H % 8 != 0


@pytest.mark.gpu
def test_rmsnorm_layer_hands_int8_rows_to_the_block():
    """RMSNorm.forward in its three forms, and the block fed by forward_moe_input gives the same
    bits as the block fed by the normalised bf16 rows (it then quantises them itself)."""
    import types
    from omni_infer_amd import config, distributed
    from omni_infer_amd.layers.layernorm import RMSNorm
    from tests.test_gpu_layer import _dsv3_block
    env = types.SimpleNamespace(config=config, dist=distributed)
    blk, lay, gate_w, bias, lo = _dsv3_block(env, 4, 8, 2, H=1024, I=512, seed=4)
    norm = RMSNorm(1024, 1e-6, params_dtype=torch.bfloat16, device="cuda")
    x, r, w = _inputs(40, 1024, 31)
    norm.weight.data.copy_(w)
    y_ref, res_ref = O.add_rms_norm(x, r, w, 1e-6)
    y, res = norm(x.cuda(), r.cuda())
    assert torch.equal(y.cpu(), y_ref) and torch.equal(res.cpu(), res_ref)
    d, res2 = norm(x.cuda(), r.cuda(), quant_symbol=True)
    q_ref, s_ref, _ = O.add_rms_norm_dynamic_quant(x, r, w, 1e-6)
    assert set(d) == {"x_int8", "pertoken_scale"} and torch.equal(d["x_int8"].cpu(), q_ref)
    assert torch.equal(d["pertoken_scale"].cpu(), s_ref) and torch.equal(res2.cpu(), res_ref)
    assert torch.equal(norm(x.cuda()).cpu(), O.add_rms_norm(x, None, w, 1e-6)[0])
    handed, _ = norm.forward_moe_input(x.cuda(), r.cuda())
    out_a, _ = blk(handed, None, None, 3)
    out_b, _ = blk(y, None, None, 3)
    assert torch.equal(out_a, out_b)
