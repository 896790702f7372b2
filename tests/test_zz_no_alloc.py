"""pa_attention_static (the entry point that allocates nothing) against pa_attention, through the C-ABI."""
import numpy as np
import pytest

import harness as H

pytestmark = pytest.mark.gpu


def _device_inputs(torch, case, dev):
    q = H.to_device_16(torch, case["query"], case["q_dtype"], dev)
    kc = torch.from_numpy(case["key_cache0"]).to(dev)
    vc = torch.from_numpy(case["value_cache0"]).to(dev)
    return q, kc, vc


def _run(torch, op, case, dev, static, want_scores=True):
    q, kc, vc = _device_inputs(torch, case, dev)
    op.step_begin(case["past_lens"], case["subsequence_begins"], case["block_indices_begins"],
                  int((case["past_lens"] + case["new_lens"]).max()), case["score_aggregation_window"],
                  case["sliding_window"], case["scale"])
    op.set_block_indices(case["block_indices"], case["num_blocks"])
    out = torch.full_like(q, float("nan"))
    scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev) if want_scores else None
    torch.cuda.synchronize(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]
    (op.attention_static if static else op.attention)(q, kc, vc, out, scores)
    op.synchronize()
    if static:  # nothing was allocated (or freed) on the device inside the call
        assert torch.cuda.mem_get_info(dev)[0] == free_before
    torch.cuda.synchronize(dev)
    return (out.view(torch.int16).cpu().numpy().view(np.uint16), scores.cpu().numpy() if want_scores else None,
            op.num_splits)


@pytest.mark.parametrize("kv_dtype,q_dtype,heads", [("u8", "f16", (32, 8, 128)), ("bf16", "bf16", (32, 8, 128)),
                                                    ("u8", "bf16", (16, 8, 256)), ("f16", "f16", (12, 4, 96))])
def test_static_entry_point_matches_pa_attention_on_two_calls_in_a_row(pkg, kv_dtype, q_dtype, heads):
    """Two calls in a row on the shared scratch, the second with a smaller input: outputs and scores are those of
    pa_attention bit for bit (same kernels, other workspace) and within tolerance of the CPU checker."""
    import torch
    dev = torch.device("cuda:0")
    Hq, Hkv, D = heads
    big = H.build_case(H.case_from_lens("static_big", Hq, Hkv, D, 32, q_dtype, kv_dtype,
                                        [9000, 4500, 7000, 123, 8100, 6400], [1] * 6), seed=11)
    small = H.build_case(H.case_from_lens("static_small", Hq, Hkv, D, 32, q_dtype, kv_dtype, [700, 33, 1500], [1] * 3), seed=12)
    ref_op = pkg.PagedAttention(Hq, Hkv, D, 32, q_dtype, kv_dtype, 1, 0, torch.cuda.current_stream(dev))
    st_op = pkg.PagedAttention(Hq, Hkv, D, 32, q_dtype, kv_dtype, 1, 0, torch.cuda.current_stream(dev))
    splits = []
    for case in (big, small):  # the static calls follow each other on the same scratch
        out_s, sc_s, ns = _run(torch, st_op, case, dev, static=True)
        out_r, sc_r, nr = _run(torch, ref_op, case, dev, static=False)
        assert ns == nr
        splits.append(ns)
        assert np.array_equal(out_s, out_r), case["name"]
        assert np.array_equal(sc_s, sc_r), case["name"]
        # and against the checker (the caches already hold the step's rows: attention only)
        from oracle import oracle as O
        qd, kd = H.DT[q_dtype], H.DT[kv_dtype]
        out, out16, scores = O.paged_attention(case["query"], qd, case["key_cache0"], case["value_cache0"], kd,
                                               case["past_lens"], case["subsequence_begins"], case["block_indices"],
                                               case["block_indices_begins"], Hq, Hkv, D, 32, case["scale"], 0, None, True, 8)
        H.assert_close(O.from_bits(out_s, qd), out, q_dtype)
        H.assert_close(sc_s, scores, "f16", "scores")
    assert splits[0] > 1, "the first case is meant to use the split partials of the scratch"
    # a third call without scores on the same scratch
    out_s, _, _ = _run(torch, st_op, small, dev, static=True, want_scores=False)
    out_r, _, _ = _run(torch, ref_op, small, dev, static=False, want_scores=False)
    assert np.array_equal(out_s, out_r)


def test_static_entry_point_refuses_what_it_cannot_serve(pkg):
    import torch
    from openvino_genai_amd import _lib as L
    dev = torch.device("cuda:0")
    # more workspace than the scratch holds: the per-head split probabilities of 40 sequences x 30000 positions, 77 MB
    op = pkg.PagedAttention(32, 8, 128, 32, "f16", "u8", 1, 0, torch.cuda.current_stream(dev))
    B, past = 40, 30000
    nblk = (past + 1 + 31) // 32
    bib = np.arange(B + 1, dtype=np.int32) * nblk
    op.step_begin(np.full(B, past, np.int32), np.arange(B + 1, dtype=np.int32), bib, past + 1)
    op.set_block_indices(np.arange(B * nblk, dtype=np.int32) % 64, 64)
    q = torch.zeros(B, 32 * 128, dtype=torch.float16, device=dev)
    kc = torch.zeros(64, 8, 32, 136, dtype=torch.uint8, device=dev)
    out = torch.zeros_like(q)
    scores = torch.zeros(op.total_scores, dtype=torch.float32, device=dev)
    with pytest.raises(L.PaError) as e:
        op.attention_static(q, kc, kc, out, scores)
    assert e.value.status == -6 and "fixed scratch" in str(e.value)
    # a step with a prefill chunk is not served
    op.step_begin(np.array([0, 64], np.int32), np.array([0, 40, 41], np.int32), np.array([0, 2, 5], np.int32), 65)
    op.set_block_indices(np.arange(5, dtype=np.int32), 64)
    q = torch.zeros(41, 32 * 128, dtype=torch.float16, device=dev)
    out = torch.zeros_like(q)
    with pytest.raises(L.PaError) as e:
        op.attention_static(q, kc, kc, out, None)
    assert e.value.status == -2


def test_static_entry_point_serves_the_largest_single_token_workload(pkg):
    """256 sequences x 8193 positions, 32 heads over 8 kv heads: the per-kv-head score sums alone are 33.6 MB, the
    largest workspace among the single-token workloads this path is measured on, and inside the scratch.  The block
    tables walk a pool of 129 real blocks over and over, so the case costs megabytes, not gigabytes."""
    import torch
    from oracle import oracle as O
    dev = torch.device("cuda:0")
    Hq, Hkv, D, bs, B, ctx_len = 32, 8, 128, 32, 256, 8193
    pool = H.build_case(H.case_from_lens("static_pool", Hq, Hkv, D, bs, "f16", "u8", [4095], [1]), seed=21, pool_factor=1.0)
    nb, nblk = pool["num_blocks"], (ctx_len + bs - 1) // bs
    rng = np.random.default_rng(22)
    case = dict(pool, name="static_256x8193", B=B, past_lens=np.full(B, ctx_len - 1, np.int32), new_lens=np.ones(B, np.int32),
                subsequence_begins=np.arange(B + 1, dtype=np.int32),
                block_indices_begins=(np.arange(B + 1) * nblk).astype(np.int32),
                block_indices=rng.integers(0, nb, B * nblk).astype(np.int32),
                query=O.to_bits(rng.standard_normal((B, Hq * D)).astype(np.float32), H.DT["f16"]))
    ref_op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "u8", 1, 0, torch.cuda.current_stream(dev))
    st_op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "u8", 1, 0, torch.cuda.current_stream(dev))
    out_s, sc_s, ns = _run(torch, st_op, case, dev, static=True)
    out_r, sc_r, nr = _run(torch, ref_op, case, dev, static=False)
    assert ns == nr == 1
    assert Hkv * sc_s.size * 2 > 32 << 20
    assert np.array_equal(out_s, out_r)
    assert np.array_equal(sc_s, sc_r)
    out, out16, scores = O.paged_attention(case["query"], H.DT["f16"], case["key_cache0"], case["value_cache0"], H.DT["u8"],
                                           case["past_lens"], case["subsequence_begins"], case["block_indices"],
                                           case["block_indices_begins"], Hq, Hkv, D, bs, case["scale"], 0, None, True, 8)
    H.assert_close(O.from_bits(out_s, H.DT["f16"]), out, "f16")
    H.assert_close(sc_s, scores, "f16", "scores")
