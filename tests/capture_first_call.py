"""Run as a program by tests/test_gpu_capture_first_call.py, in a process of its own: the very first layer call of
the process is recorded into a HIP graph (so everything the library looks up once per process or per device, the
occupancy of its kernels, the compute-unit count, the device address of its static arrays, is looked up inside the
capture), the graph is replayed, and the replays are compared with an eager call made afterwards."""
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from tests.helpers import Layer, gen, tokens  # noqa: E402


def main(routed: bool) -> int:
    from omni_infer_amd import _lib as L
    from omni_infer_amd import hip_ops as ops
    E, n, H, I, K, T = 32, 4, 1024, 512, 8, 48
    lay = Layer(n, H, I, seed=801, shared=True)
    d = lay.to_device()
    shared = (d["sh13"], d["sh_s13"], d["sh2"], d["sh_s2"])
    g = gen(802)
    x = tokens(T, H, 803).cuda()
    logits = torch.randn(T, E, generator=g).cuda()
    bias = (torch.randn(E, generator=g) * 0.01).cuda()
    ids = torch.rand(T, E, generator=g).argsort(dim=1)[:, :K].to(torch.int32).cuda()
    w = torch.rand(T, K, generator=g).cuda()
    ws = torch.empty(L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, n, H, I, 1, L.OMNI_DT_F32), dtype=torch.uint8, device="cuda")
    out = torch.empty(T, H, dtype=torch.bfloat16, device="cuda")
    tw = torch.empty(T, K, dtype=torch.float32, device="cuda")
    ti = torch.empty(T, K, dtype=torch.int32, device="cuda")
    route = dict(top_k=K, n_group=8, topk_group=4, score_fn="sigmoid", group_mode=L.OMNI_GROUP_TOP2SUM,
                 masked_fill_zero=False, weight_from_c=False, renorm=True, scale=2.5, eps=1e-20)

    def step():
        if routed:
            return ops.moe_w8a8_layer_routed(x, None, logits, bias, lo=0, hi=n, w13_packed=d["w13"], w13_scale=d["s13"],
                                             w2_packed=d["w2"], w2_scale=d["s2"], shared=shared, H=H, I=I, workspace=ws,
                                             out=out, topk_w=tw, topk_ids=ti, **route)[0]
        return ops.moe_w8a8_layer(x, None, w, ids, 0, n, d["w13"], d["s13"], d["w2"], d["s2"], shared, H=H, I=I,
                                  workspace=ws, out=out)

    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    replays = []
    for rep in range(2):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        replays.append(out.clone())
    eager = step().clone()
    torch.cuda.synchronize()
    ok = all(torch.equal(r, eager) for r in replays) and bool(torch.isfinite(eager.float()).all())
    print("capture-first-call", "routed" if routed else "layer", "OK" if ok else "MISMATCH", flush=True)
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main(len(sys.argv) > 1 and sys.argv[1] == "routed"))
