"""A step's per-layer calls recorded into a HIP graph: after one eager warm-up (which sizes the workspaces) the calls
neither allocate nor wait, so a caller may capture them.  Replays, with eager work and waits in between, must give
the eager result bit for bit."""
import pytest

import harness as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kv,past,new", [("u8", [700, 64, 1300, 31], [1, 1, 1, 1]),       # decode kernel, one split
                                         ("u8", [9000], [1]),                             # several splits + merge
                                         ("bf16", [300, 40, 0], [1, 1, 70]),              # matrix kernel, mixed step
                                         ("u8", [300, 40, 0], [1, 1, 70]),                # decode kernel on the second stream beside the matrix kernel
                                         ("bf16", [700, 64, 1300, 31], [1, 1, 1, 1]),     # 16-bit decode kernel (appends too)
                                         ("bf16", [9000, 20], [1, 1])])                   # the same with several splits
def test_graph_replays_equal_eager(pkg, kv, past, new):
    import torch
    dev = torch.device("cuda:0")
    q = "bf16" if kv == "bf16" else "f16"
    case = H.build_case(H.case_from_lens("graph", 8, 2, 128, 32, q, kv, past, new), 77)
    layers = 3
    s = torch.cuda.Stream(dev)
    with torch.cuda.stream(s):
        op = pkg.PagedAttention(8, 2, 128, 32, q, kv, num_layers=layers, device=0, stream=s)
        op.step_begin(case["past_lens"], case["subsequence_begins"], case["block_indices_begins"],
                      int((case["past_lens"] + case["new_lens"]).max()), None, 0, case["scale"])
        op.set_block_indices(case["block_indices"], case["num_blocks"])
        kc = [torch.from_numpy(case["key_cache0"]).to(dev) for _ in range(layers)]
        vc = [torch.from_numpy(case["value_cache0"]).to(dev) for _ in range(layers)]
        qd, kd, vd = (H.to_device_16(torch, case[x], q, dev) for x in ("query", "key", "value"))
        outs = [torch.zeros_like(qd) for _ in range(layers)]
        scores = [torch.zeros(op.total_scores, dtype=torch.float32, device=dev) for _ in range(layers)]

        def step():
            for l in range(layers):
                op.forward(qd, kd, vd, kc[l], vc[l], outs[l], scores[l], layer=l)

        step()  # eager: also sizes every workspace
        s.synchronize()
        want_out = [o.clone() for o in outs]
        want_sc = [x.clone() for x in scores]
        want_kc = [x.clone() for x in kc]
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            step()
        for rep in range(3):
            for o, x in zip(outs, scores):  # eager work between the replays: the outputs are wiped
                o.zero_()
                x.fill_(-1.0)
            s.synchronize()
            g.replay()
            s.synchronize()
            for l in range(layers):
                assert torch.equal(outs[l], want_out[l]), (rep, l)
                assert torch.equal(scores[l], want_sc[l]), (rep, l)
                assert torch.equal(kc[l], want_kc[l]), (rep, l)  # the append rewrote the same rows
        assert float(want_sc[0].sum()) > 0
