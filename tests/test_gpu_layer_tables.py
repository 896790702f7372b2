"""`block_indices.<L>` of several layers set by one call: the same tables, descriptors and results as one call per layer."""
import numpy as np
import pytest

import harness as H

from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    return torch.device("cuda:0")


CASES = [
    H.case_from_lens("decode_u8", 8, 2, 128, 32, "f16", "u8", [37, 130, 64, 700], [1, 1, 1, 1]),
    H.case_from_lens("mixed_bf16", 8, 2, 128, 32, "bf16", "bf16", [0, 130, 64], [70, 1, 33]),
    H.case_from_lens("mixed_u8_block16", 4, 4, 64, 16, "f16", "u8", [5, 300], [1, 40]),
]
LAYERS = 3


def _run_layers(torch, op, dev, cases, set_tables):
    c0 = cases[0]
    op.step_begin(c0["past_lens"], c0["subsequence_begins"], c0["block_indices_begins"],
                  int((c0["past_lens"] + c0["new_lens"]).max()), None, 0, c0["scale"])
    set_tables()
    res = []
    for l, c in enumerate(cases):
        q, k, v = (H.to_device_16(torch, c[n], c["q_dtype"], dev) for n in ("query", "key", "value"))
        kc, vc = torch.from_numpy(c["key_cache0"]).to(dev), torch.from_numpy(c["value_cache0"]).to(dev)
        out = torch.zeros_like(q)
        scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
        op.forward(q, k, v, kc, vc, out, scores, layer=l)
        op.synchronize()
        res.append((out.view(torch.int16).cpu().numpy(), scores.cpu().numpy(), kc.cpu().numpy(), vc.cpu().numpy()))
    return res


@pytest.mark.parametrize("case", CASES, ids=lambda c: c["name"])
def test_tables_of_all_layers_in_one_call_give_the_results_of_a_call_per_layer(pkg, dev, case):
    import torch
    cases = [H.build_case(case, seed=40 + l) for l in range(LAYERS)]   # same lengths, a table and contents per layer
    c0 = cases[0]
    op = pkg.PagedAttention(c0["Hq"], c0["Hkv"], c0["D"], c0["bs"], c0["q_dtype"], c0["kv_dtype"], num_layers=LAYERS,
                            device=0, stream=torch.cuda.current_stream(dev))
    pool = c0["num_blocks"]

    def one_by_one():
        for l, c in enumerate(cases):
            op.set_block_indices(c["block_indices"], pool, layer=l)

    def together():
        op.set_block_indices_per_layer([c["block_indices"] for c in cases], pool)

    def part_and_rest():  # layers 1.. in one call, layer 0 on its own, in that order
        op.set_block_indices_per_layer([c["block_indices"] for c in cases[1:]], pool, first_layer=1)
        op.set_block_indices(cases[0]["block_indices"], pool, layer=0)

    want = _run_layers(torch, op, dev, cases, one_by_one)
    ref = H.run_case_on_checker(cases[1])   # (the per-layer path itself against the checker, one layer)
    H.assert_close(O.from_bits(want[1][0].view(np.uint16), H.DT[c0["q_dtype"]]), ref["out"], c0["q_dtype"])
    assert np.array_equal(want[1][2], ref["key_cache"]) and np.array_equal(want[1][3], ref["value_cache"])
    for how in (together, part_and_rest, one_by_one, together):
        got = _run_layers(torch, op, dev, cases, how)
        for l in range(LAYERS):
            for g, w, what in zip(got[l], want[l], ("out", "scores", "key_cache", "value_cache")):
                assert np.array_equal(g, w, equal_nan=True), (how.__name__, l, what)


def test_bad_table_of_any_layer_is_refused_and_changes_nothing(pkg, dev):
    import torch
    cases = [H.build_case(CASES[0], seed=50 + l) for l in range(LAYERS)]
    c0 = cases[0]
    op = pkg.PagedAttention(c0["Hq"], c0["Hkv"], c0["D"], c0["bs"], c0["q_dtype"], c0["kv_dtype"], num_layers=LAYERS,
                            device=0, stream=torch.cuda.current_stream(dev))
    pool = c0["num_blocks"]
    op.step_begin(c0["past_lens"], c0["subsequence_begins"], c0["block_indices_begins"])
    tables = [c["block_indices"].copy() for c in cases]
    tables[2][5] = pool                      # one id of the last layer outside the cache
    with pytest.raises(pkg.PaError) as e:
        op.set_block_indices_per_layer(tables, pool)
    assert e.value.status == -6
    q = H.to_device_16(torch, c0["query"], c0["q_dtype"], dev)
    kc = torch.from_numpy(c0["key_cache0"]).to(dev)
    with pytest.raises(pkg.PaError):         # no layer's table was set by the refused call
        op.attention(q, kc, kc, torch.zeros_like(q), layer=0)
    with pytest.raises(pkg.PaError) as e:    # more layers than the context has
        op.set_block_indices_per_layer([c["block_indices"] for c in cases], pool, first_layer=1)
    assert e.value.status == -6
    with pytest.raises(pkg.PaError) as e:    # wrong number of ids
        op.set_block_indices_per_layer([c["block_indices"][:-1] for c in cases], pool)
    assert e.value.status == -4
    op.set_block_indices_per_layer([c["block_indices"] for c in cases], pool)
    # a cache smaller than a layer's largest id + 1 is refused at the layer call, per layer
    small = int(cases[1]["block_indices"].max())
    short = torch.zeros(small, *kc.shape[1:], dtype=torch.uint8, device=dev)
    with pytest.raises(pkg.PaError) as e:
        op.attention(q, short, short, torch.zeros_like(q), layer=1)
    assert e.value.status == -6
    op.attention(q, kc, kc, torch.zeros_like(q), layer=1)
    op.synchronize()
