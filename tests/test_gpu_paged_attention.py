"""GPU parity of the HIP path against the CPU checker, through the C-ABI.

KV rows (u8 codes, f32 headers, 16-bit copies) must be bit-exact; outputs and scores within 2e-3 relative / 1e-3
absolute (plus half an ulp of the bf16 output format where the output is bf16).  Full-size workloads are checked
through size-independent properties."""
import numpy as np
import pytest

import harness as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


def _check(pkg, dev, case, seed, outliers=False, want_scores=True):
    print(f"case {case['name']} seed {seed}", flush=True)
    c = H.build_case(case, seed, outliers=outliers)
    got = H.run_case_on_gpu(pkg, c, dev, want_scores)
    ref = H.run_case_on_checker(c, want_scores=want_scores)
    assert np.array_equal(got["key_cache"], ref["key_cache"]), "key cache bytes differ"
    assert np.array_equal(got["value_cache"], ref["value_cache"]), "value cache bytes differ"
    H.assert_close(got["out"], ref["out"], c["q_dtype"])
    if want_scores:
        assert np.isfinite(got["scores"]).all(), "scores not fully written"
        H.assert_close(got["scores"], ref["scores"], "f16", "scores")
    return got, ref, c


def _outliers(torch, x, g, frac=0.01):
    """Replaces `frac` of the elements by +-8 (the workloads' outlier recipe), in place."""
    m = torch.rand(x.shape, generator=g, device=x.device) < frac
    s = torch.where(torch.rand(x.shape, generator=g, device=x.device) < 0.5, 8.0, -8.0).to(x.dtype)
    x[m] = s[m]
    return x


def _check_whole_batch(spec, q, kc, vc, out, scores, W, qd, kd, sw):
    """Every sequence of a full-size workload against the checker: the blocks the tables name are gathered into a
    compact copy of the caches (table = 0, 1, 2, ...) on the device, copied to the host, and the whole batch goes
    through one checker call."""
    import torch
    O = H.O
    Hq, Hkv, D, bs = spec["Hq"], spec["Hkv"], spec["D"], spec["bs"]
    ids = torch.from_numpy(spec["block_indices"].astype(np.int64)).to(kc.device)
    kcs, vcs = kc[ids].cpu().numpy(), vc[ids].cpu().numpy()
    qs = q.view(torch.int16).cpu().numpy().view(np.uint16)
    ref_out, _, ref_sc = O.paged_attention(
        qs, H.DT[qd], kcs, vcs, H.DT[kd], spec["past_lens"], spec["subsequence_begins"],
        np.arange(len(spec["block_indices"]), dtype=np.int32), spec["block_indices_begins"], Hq, Hkv, D, bs,
        spec["scale"], sw, W, want_scores=True, num_threads=16)
    H.assert_close(out.float().cpu().numpy(), ref_out, qd)
    H.assert_close(scores.cpu().numpy(), ref_sc, "f16", "scores")



APPEND_CASES = [("f16", "u8", 128), ("f16", "u8", 64), ("bf16", "u8", 128), ("f16", "f16", 64), ("bf16", "bf16", 128),
                ("f16", "bf16", 128), ("bf16", "f16", 64),
                ("f16", "u8", 96), ("bf16", "u8", 256), ("f16", "f16", 96), ("bf16", "bf16", 256), ("f16", "bf16", 96),
                ("bf16", "f16", 256)]


@pytest.mark.parametrize("qd,kd,D", APPEND_CASES)
def test_kv_append_bit_exact(pkg, dev, qd, kd, D):
    case = H.case_from_lens(f"append_{qd}_{kd}_{D}", 4, 2, D, 32, qd, kd, [0, 31, 32, 100, 7], [40, 1, 33, 1, 25])
    _check(pkg, dev, case, 3, outliers=True, want_scores=False)


MANY_ROWS = [
    # (query type, cache type, D, Hkv, block size): steps of 16384 or more (token, kv head, K | V) rows take the
    # append kernel with a row per 16 lanes
    ("f16", "u8", 128, 4, 32), ("bf16", "u8", 128, 8, 32), ("f16", "u8", 64, 4, 32), ("bf16", "u8", 64, 2, 32),
    ("f16", "u8", 128, 4, 16), ("f16", "f16", 128, 4, 32), ("bf16", "bf16", 64, 4, 32), ("f16", "bf16", 128, 4, 32),
    ("bf16", "f16", 64, 2, 16), ("f16", "u8", 96, 4, 32), ("bf16", "u8", 256, 2, 32), ("f16", "f16", 96, 3, 16),
    ("bf16", "bf16", 256, 2, 64),
]


@pytest.mark.parametrize("qd,kd,D,Hkv,bs", MANY_ROWS)
def test_kv_append_many_rows_bit_exact(pkg, dev, qd, kd, D, Hkv, bs):
    T_min = 16384 // (2 * Hkv) + 70
    _append_many(pkg, dev, qd, kd, D, Hkv, bs, [T_min - 700, 333, 1, 300, 65, 1], 16384)


MANY_TOKENS = [
    # steps of 8192 or more tokens take the append kernel in which 16 lanes own a token and walk its rows four at a
    # time (3 kv heads: the last group of rows is not full)
    ("f16", "u8", 128, 8, 32), ("bf16", "u8", 64, 3, 32), ("f16", "u8", 128, 1, 16), ("bf16", "bf16", 128, 4, 32),
    ("f16", "bf16", 64, 3, 64), ("bf16", "f16", 128, 2, 32),
    ("f16", "u8", 96, 3, 32), ("bf16", "u8", 256, 2, 32), ("bf16", "bf16", 96, 2, 16), ("f16", "f16", 256, 1, 64),
]


@pytest.mark.parametrize("qd,kd,D,Hkv,bs", MANY_TOKENS)
def test_kv_append_many_tokens_bit_exact(pkg, dev, qd, kd, D, Hkv, bs):
    _append_many(pkg, dev, qd, kd, D, Hkv, bs, [7000, 333, 1, 1300, 65, 1], 8192 * Hkv * 2)


def _append_many(pkg, dev, qd, kd, D, Hkv, bs, new, min_rows):
    import torch
    from oracle import oracle as O
    case = H.case_from_lens(f"append_many_{qd}_{kd}_{D}", Hkv, Hkv, D, bs, qd, kd, [0, 31, 4000, 100, 7, 0], new)
    print(f"case {case['name']} seed 9", flush=True)
    c = H.build_case(case, 9, outliers=True)
    assert int(c["subsequence_begins"][-1]) * Hkv * 2 >= min_rows
    # rows with a zero range, a huge range and exact ties, in the middle of the long sequence
    x = np.zeros((3, Hkv * D), np.float32)
    x[0] = 3.25
    x[1, ::2], x[1, 1::2] = -60000.0, 60000.0
    x[2] = np.tile(np.arange(D, dtype=np.float32) * 0.5, Hkv)
    c["key"][500:503] = O.to_bits(x, H.DT[qd])
    c["value"][800:803] = O.to_bits(x[::-1].copy(), H.DT[qd])
    kc_ref, vc_ref = c["key_cache0"].copy(), c["value_cache0"].copy()
    O.kv_append(c["key"], c["value"], H.DT[qd], kc_ref, vc_ref, H.DT[kd], c["past_lens"], c["subsequence_begins"],
                c["block_indices"], c["block_indices_begins"], Hkv, D, bs)
    op = pkg.PagedAttention(Hkv, Hkv, D, bs, qd, kd, 1, 0, torch.cuda.current_stream(dev))
    k = H.to_device_16(torch, c["key"], qd, dev)
    v = H.to_device_16(torch, c["value"], qd, dev)
    kc, vc = torch.from_numpy(c["key_cache0"]).to(dev), torch.from_numpy(c["value_cache0"]).to(dev)
    op.step_begin(c["past_lens"], c["subsequence_begins"], c["block_indices_begins"],
                  int((c["past_lens"] + c["new_lens"]).max()))
    op.set_block_indices(c["block_indices"], c["num_blocks"])
    op.kv_append(k, v, kc, vc)
    op.synchronize()
    assert np.array_equal(kc.cpu().numpy(), kc_ref), "key cache bytes differ"
    assert np.array_equal(vc.cpu().numpy(), vc_ref), "value cache bytes differ"


def test_step_arrays_outgrow_the_pinned_staging_area(pkg, dev):
    """A context's step arrays pass through a pinned staging area that starts small: a step of 40000 tokens does not
    fit it (the area is waited for and grows in the middle of the step's uploads), and the steps before and after it
    on the same context use what is there."""
    import torch
    from oracle import oracle as O
    Hkv, D, bs, qd, kd = 2, 64, 32, "f16", "u8"
    op = pkg.PagedAttention(Hkv, Hkv, D, bs, qd, kd, 1, 0, torch.cuda.current_stream(dev))
    for i, (past, new) in enumerate([([5, 0], [3, 40]), ([0, 31, 100], [25000, 14000, 1000]), ([7], [9])]):
        c = H.build_case(H.case_from_lens(f"staging_{i}", Hkv, Hkv, D, bs, qd, kd, past, new), 90 + i)
        kc_ref, vc_ref = c["key_cache0"].copy(), c["value_cache0"].copy()
        O.kv_append(c["key"], c["value"], H.DT[qd], kc_ref, vc_ref, H.DT[kd], c["past_lens"], c["subsequence_begins"],
                    c["block_indices"], c["block_indices_begins"], Hkv, D, bs)
        k, v = H.to_device_16(torch, c["key"], qd, dev), H.to_device_16(torch, c["value"], qd, dev)
        kc, vc = torch.from_numpy(c["key_cache0"]).to(dev), torch.from_numpy(c["value_cache0"]).to(dev)
        op.step_begin(c["past_lens"], c["subsequence_begins"], c["block_indices_begins"],
                      int((c["past_lens"] + c["new_lens"]).max()))
        op.set_block_indices(c["block_indices"], c["num_blocks"])
        op.kv_append(k, v, kc, vc)
        op.synchronize()
        assert np.array_equal(kc.cpu().numpy(), kc_ref), f"step {i}: key cache bytes differ"
        assert np.array_equal(vc.cpu().numpy(), vc_ref), f"step {i}: value cache bytes differ"


def test_kv_append_constant_and_extreme_rows(pkg, dev):
    # constant rows (zero range), huge range, and exact .5 ties
    import torch
    case = H.case_from_lens("append_edge", 2, 1, 128, 32, "f16", "u8", [5], [4])
    c = H.build_case(case, 1)
    rows = np.zeros((4, 128), np.float32)
    rows[0, :] = 1.25
    rows[1, :] = np.linspace(-60000, 60000, 128)
    rows[2, :] = np.concatenate([[0.0, 255.0], np.arange(126) + 0.5])
    rows[3, :] = 0.0
    c["key"] = H.O.to_bits(rows, H.O.DT_F16)
    c["value"] = H.O.to_bits(rows[::-1].copy(), H.O.DT_F16)
    got = H.run_case_on_gpu(pkg, c, dev, False)
    ref = H.run_case_on_checker(c, want_scores=False)
    assert np.array_equal(got["key_cache"], ref["key_cache"])
    assert np.array_equal(got["value_cache"], ref["value_cache"])


def test_cfg1_tinyllama_decode_f16(pkg, dev):
    rng = np.random.default_rng(1001)
    past = rng.integers(64, 2049, 16)
    _check(pkg, dev, H.case_from_lens("cfg1", 32, 4, 64, 32, "f16", "f16", past, np.ones(16, int)), 1001)


def test_cfg2_shape_decode_u8_reduced(pkg, dev):
    # Llama-3-8B shape, u8 KV with 1 % outliers, batch 6, contexts around 4096 reduced to keep the checker quick
    _check(pkg, dev, H.case_from_lens("cfg2_small", 32, 8, 128, 32, "f16", "u8", [1024, 4096, 333, 32, 31, 2047],
                                      np.ones(6, int)), 1002, outliers=True)


def test_cfg3_shape_mixed_prefill_decode_bf16(pkg, dev):
    past = [0, 256, 512, 100, 700, 64, 1023]
    new = [96, 64, 33, 1, 1, 1, 1]
    _check(pkg, dev, H.case_from_lens("cfg3_small", 28, 4, 128, 32, "bf16", "bf16", past, new,
                                      score_aggregation_window=[8, 64, 0, 1, 1, 1, 0]), 1003)


def test_cfg5_shape_long_context_and_sliding_window(pkg, dev):
    _check(pkg, dev, H.case_from_lens("cfg5_small", 40, 8, 128, 32, "f16", "u8", [6000, 5000], [1, 1]), 1005)
    _check(pkg, dev, H.case_from_lens("cfg5_window", 40, 8, 128, 32, "f16", "u8", [6000, 100, 511], [1, 1, 1],
                                      sliding_window=512), 1005)


@pytest.mark.parametrize("name,args", [
    ("prefill_from_empty_u8", (8, 2, 128, 32, "f16", "u8", [0, 0], [70, 1])),
    ("block16_gqa1", (4, 4, 64, 16, "f16", "f16", [17, 48, 0], [1, 5, 16])),
    ("gqa8_d64_bf16q_u8", (16, 2, 64, 32, "bf16", "u8", [200, 90], [1, 3])),
    ("window_prefill", (8, 2, 128, 32, "f16", "f16", [100, 0], [40, 90])),
    ("single_token_context", (8, 8, 128, 32, "f16", "u8", [0], [1])),
])
def test_edge_shapes(pkg, dev, name, args):
    sw = 48 if name == "window_prefill" else 0
    saw = [40, 7] if name == "window_prefill" else None
    _check(pkg, dev, H.case_from_lens(name, *args, sliding_window=sw, score_aggregation_window=saw), 77)


@pytest.mark.parametrize("name,args,kw", [
    ("dec_u8_d128_g4_multi_split", (8, 2, 128, 32, "f16", "u8", [3000, 2500, 17], [1, 1, 1]), {}),
    ("dec_u8_d64_g8", (16, 2, 64, 32, "f16", "u8", [700, 64, 31, 32, 33, 1500], [1] * 6), {}),
    ("dec_u8_d128_g16_bf16q", (16, 1, 128, 32, "bf16", "u8", [900, 100], [1, 1]), {}),
    ("dec_u8_g1", (4, 4, 128, 32, "f16", "u8", [257, 1024], [1, 1]), {}),
    ("dec_u8_window_multi_split", (8, 2, 128, 32, "f16", "u8", [5000, 900, 40], [1, 1, 1]), {"sliding_window": 1000}),
    ("dec_u8_window_unaligned", (8, 2, 128, 32, "f16", "u8", [300, 77], [1, 1]), {"sliding_window": 45}),
    ("dec_u8_w0_mix", (8, 2, 128, 32, "f16", "u8", [300, 77, 500], [1, 1, 1]), {"score_aggregation_window": [1, 0, 1]}),
    ("dec_u8_many_seqs", (32, 8, 128, 32, "f16", "u8", list(range(1, 600, 9)), [1] * 67), {}),
    # head sizes 96 (six value channels per lane, append by the shape-generic kernel) and 256 (one workgroup per CU)
    ("dec_u8_d96_mha_multi_split", (6, 6, 96, 32, "f16", "u8", [3000, 2500, 17], [1, 1, 1]), {}),
    ("dec_u8_d96_g3_bs16_bf16q", (12, 4, 96, 16, "bf16", "u8", [700, 64, 31, 32, 33, 1500], [1] * 6), {}),
    ("dec_u8_d96_bs128_window", (8, 2, 96, 128, "f16", "u8", [5000, 900, 40], [1, 1, 1]), {"sliding_window": 1000}),
    ("dec_u8_d96_many_seqs", (32, 32, 96, 32, "f16", "u8", list(range(1, 600, 9)), [1] * 67), {}),
    ("dec_u8_d256_g2_multi_split", (16, 8, 256, 32, "f16", "u8", [3000, 2500, 17], [1, 1, 1]), {}),
    ("dec_u8_d256_mha_bf16q_bs64", (4, 4, 256, 64, "bf16", "u8", [700, 64, 31, 32, 33, 1500], [1] * 6), {}),
    ("dec_u8_d256_g16_window", (16, 1, 256, 32, "f16", "u8", [5000, 900, 40], [1, 1, 1]), {"sliding_window": 1000}),
    ("dec_u8_d256_w0_mix", (8, 2, 256, 32, "bf16", "u8", [300, 77, 500], [1, 1, 1]), {"score_aggregation_window": [1, 0, 1]}),
    ("dec_u8_d256_many_seqs", (16, 8, 256, 32, "f16", "u8", list(range(1, 600, 9)), [1] * 67), {}),
])
def test_decode_u8_kernel_shapes(pkg, dev, name, args, kw):
    got, ref, c = _check(pkg, dev, H.case_from_lens(name, *args, **kw), 31, outliers=True)
    # and without scores (no probabilities kept)
    got2 = H.run_case_on_gpu(pkg, c, dev, want_scores=False)
    H.assert_close(got2["out"], ref["out"], c["q_dtype"])


@pytest.mark.parametrize("name,args,kw", [
    ("pf16_bf16_g7_mixed", (28, 4, 128, 32, "bf16", "bf16", [0, 700, 333, 40, 2000], [150, 37, 1, 1, 64]),
     {"score_aggregation_window": [8, 37, 1, 0, 3]}),
    ("pf16_f16_d64_g8", (32, 4, 64, 32, "f16", "f16", [0, 31, 32, 500], [33, 100, 1, 17]), {}),
    ("pf16_f16_g1_window", (4, 4, 128, 32, "f16", "f16", [300, 0], [200, 130]), {"sliding_window": 100}),
    ("pf16_bf16_g16", (16, 1, 128, 32, "bf16", "bf16", [64, 0], [9, 8]), {}),
    ("pf16_f16_g3_long_chunk", (6, 2, 128, 32, "f16", "f16", [1500], [700]), {"score_aggregation_window": [16]}),
    # many long single-token sequences next to two short chunks: their work items are listed between the chunks' items
    ("pf16_bf16_interleaved_items", (28, 4, 128, 32, "bf16", "bf16",
                                     [100, 0] + [900 + 37 * i for i in range(14)], [64, 40] + [1] * 14), {}),
    # long single-token sequences next to chunks, scores wanted: their items keep the probabilities in LDS (several
    # items per sequence) and a small kernel forms the scores; windows of 0 and 1 rows, a sliding window, G = 16
    ("pf16_bf16_g7_long_singles", (28, 4, 128, 32, "bf16", "bf16", [0, 5000, 4097, 1375, 1376, 1377, 9000],
                                   [100, 1, 1, 1, 1, 1, 1]), {"score_aggregation_window": [4, 1, 0, 1, 1, 1, 1]}),
    ("pf16_f16_g16_long_singles_window", (16, 1, 128, 32, "f16", "f16", [64, 3000, 700, 6000], [40, 1, 1, 1]),
     {"sliding_window": 2500}),
    ("pf16_f16_d64_g1_long_singles", (4, 4, 64, 32, "f16", "f16", [10, 7000, 33], [70, 1, 1]), {}),
    ("pf16_bf16_block16_long_singles", (8, 2, 128, 16, "bf16", "bf16", [0, 5000, 2049], [50, 1, 1]), {}),
    ("pf16_f16_interleaved_items_window", (8, 2, 64, 32, "f16", "f16",
                                           [300] + [700 + 11 * i for i in range(9)], [50] + [1] * 9),
     {"sliding_window": 600, "score_aggregation_window": [5] + [1] * 9}),
    # more than 64 query heads, contexts cut into several ranges: the score rows fold the ranges' maxima and
    # denominators row by row (a wave's lanes hold at most 64 heads' pairs)
    ("pf16_bf16_128_heads_ranges", (128, 8, 128, 32, "bf16", "bf16", [1500, 2000, 40], [300, 1, 1]), {}),
    ("pf16_f16_96_heads_ranges_window_rows", (96, 8, 128, 32, "f16", "f16", [1200, 900], [200, 1]),
     {"score_aggregation_window": [5, 1]}),
    # head sizes 96 and 256 over 16-bit caches: the one-row-group variant (256: one workgroup per CU, two load units
    # per thread), single-token sequences of a mixed step as its work items
    ("pf16_bf16_d256_mixed", (16, 8, 256, 32, "bf16", "bf16", [0, 700, 333, 40, 2000, 90], [150, 37, 1, 1, 64, 1]),
     {"score_aggregation_window": [8, 37, 1, 0, 3, 1]}),
    ("pf16_f16_d256_ranges_bs16", (8, 2, 256, 16, "f16", "f16", [3000, 0, 900], [300, 130, 1]), {}),
    ("pf16_f16_d256_window", (4, 4, 256, 128, "f16", "f16", [300, 0, 1000], [200, 130, 1]), {"sliding_window": 100}),
    ("pf16_bf16_d96_mixed", (12, 4, 96, 32, "bf16", "bf16", [0, 700, 333, 40, 2000, 90], [150, 37, 1, 1, 64, 1]),
     {"score_aggregation_window": [8, 37, 1, 0, 3, 1]}),
    ("pf16_f16_d96_ranges_bs64", (6, 6, 96, 64, "f16", "f16", [3000, 0, 900], [300, 130, 1]), {}),
])
def test_prefill16_kernel_shapes(pkg, dev, name, args, kw):
    _check(pkg, dev, H.case_from_lens(name, *args, **kw), 41)


@pytest.mark.parametrize("name,args,kw", [
    # multi-token sequences over a u8 cache run on the matrix kernel, single-token ones on the decode kernel
    ("pf_u8_g4_mixed", (32, 8, 128, 32, "f16", "u8", [0, 700, 333, 40, 2000, 90], [150, 37, 1, 1, 64, 1]),
     {"score_aggregation_window": [8, 37, 1, 0, 3, 1]}),
    ("pf_u8_bf16q_d64_g8", (16, 2, 64, 32, "bf16", "u8", [0, 31, 32, 500], [33, 100, 1, 17]), {}),
    ("pf_u8_window", (8, 2, 128, 32, "f16", "u8", [300, 0, 1000], [200, 130, 1]), {"sliding_window": 100}),
    ("pf_u8_prefill_only_long", (8, 2, 128, 32, "f16", "u8", [1500], [700]), {"score_aggregation_window": [16]}),
    ("pf_u8_g32_all_on_matrix_kernel", (32, 1, 128, 32, "f16", "u8", [64, 0, 300], [9, 8, 1]), {}),
    # head size 96: chunks on the matrix kernel's one-row-group variant, single-token sequences on the decode kernel
    ("pf_u8_d96_mixed", (12, 4, 96, 32, "f16", "u8", [0, 700, 333, 40, 2000, 90], [150, 37, 1, 1, 64, 1]),
     {"score_aggregation_window": [8, 37, 1, 0, 3, 1]}),
    ("pf_u8_d96_mha_bf16q_window", (6, 6, 96, 64, "bf16", "u8", [300, 0, 1000], [200, 130, 1]), {"sliding_window": 100}),
    # head size 256: chunks on the one-row-group variant with one workgroup per CU
    ("pf_u8_d256_mixed", (8, 4, 256, 32, "f16", "u8", [0, 700, 40], [50, 1, 1]), {}),
    ("pf_u8_d256_ranges_window_rows", (16, 8, 256, 64, "bf16", "u8", [3000, 0, 900], [300, 130, 1]),
     {"score_aggregation_window": [5, 130, 1]}),
    ("pf_u8_d256_sliding_window", (4, 1, 256, 32, "f16", "u8", [300, 0, 1000], [200, 130, 1]), {"sliding_window": 100}),
    ("pf_u8_decode_multi_split_beside_prefill", (8, 2, 128, 32, "f16", "u8", [3000, 0, 2500], [1, 40, 1]), {}),
    ("pf_u8_96_heads_ranges", (96, 8, 128, 32, "f16", "u8", [1200, 2500, 60], [200, 1, 1]), {}),
])
def test_prefill_u8_kernel_shapes(pkg, dev, name, args, kw):
    got, ref, c = _check(pkg, dev, H.case_from_lens(name, *args, **kw), 43, outliers=True)
    got2 = H.run_case_on_gpu(pkg, c, dev, want_scores=False)
    H.assert_close(got2["out"], ref["out"], c["q_dtype"])


@pytest.mark.parametrize("qd,sw", [("f16", 0), ("bf16", 0), ("bf16", 3000)])
def test_pure_decode_over_16bit_caches_with_scores(pkg, dev, qd, sw):
    """A decode-only step over a 16-bit cache with scores: the 16-bit decode kernel keeps its probabilities in LDS and
    writes the scores itself (no second pass over K).  Windows of 0, 1 and more rows; several KV ranges per row."""
    case = H.case_from_lens(f"decode16_{qd}_sw{sw}", 16, 8, 128, 32, qd, qd, [6100, 4097, 31, 5555, 7000, 0], [1] * 6,
                            sliding_window=sw, score_aggregation_window=[1, 0, 1, 5, 1, 1])
    got, ref, c = _check(pkg, dev, case, 17, outliers=True)
    again = H.run_case_on_gpu(pkg, c, dev, op=got["op"])
    assert np.array_equal(again["out16"], got["out16"]) and np.array_equal(again["scores"], got["scores"])


DECODE16 = [
    ("f16_d128_g4", (8, 2, 128, 32, "f16", "f16", [37, 130, 64, 4097, 0, 31, 32, 33], [1] * 8), {}),
    ("bf16_d128_g7", (28, 4, 128, 32, "bf16", "bf16", [1000, 2047, 5], [1] * 3), {}),
    ("f16_d64_g1", (4, 4, 64, 32, "f16", "f16", [300, 64, 63, 1], [1] * 4), {}),
    ("bf16_d64_g16", (32, 2, 64, 32, "bf16", "bf16", [700, 90], [1] * 2), {}),
    ("f16_long_splits", (8, 2, 128, 32, "f16", "f16", [15000], [1]), {}),
    ("bf16_long_splits_window", (16, 8, 128, 32, "bf16", "bf16", [9000, 4000], [1, 1]), {"sliding_window": 2500}),
    ("f16_window_inside_block", (8, 2, 128, 32, "f16", "f16", [100, 45, 700], [1] * 3), {"sliding_window": 40}),
    ("bf16_mixed_with_chunks", (8, 2, 128, 32, "bf16", "bf16", [500, 0, 2000, 64], [1, 70, 1, 300]), {}),
    # odd products of blocks x heads: the per-block maxima in LDS are packed G to a block
    ("bf16_d128_g5_odd_blocks", (10, 2, 128, 32, "bf16", "bf16", [4127, 95, 33], [1] * 3), {}),
    ("f16_d128_g5_long_splits", (5, 1, 128, 32, "f16", "f16", [12001], [1]), {}),
    ("f16_g17_stays_on_the_matrix_kernel", (17, 1, 64, 32, "f16", "f16", [200, 77], [1, 1]), {}),
    # head sizes 96 and 256 (256: one workgroup per CU)
    ("f16_d96_mha", (6, 6, 96, 32, "f16", "f16", [37, 130, 64, 4097, 0, 31, 32, 33], [1] * 8), {}),
    ("bf16_d96_g3_bs16_long_splits", (12, 4, 96, 16, "bf16", "bf16", [9000, 4000], [1, 1]), {"sliding_window": 2500}),
    ("bf16_d256_g2", (16, 8, 256, 32, "bf16", "bf16", [37, 130, 64, 4097, 0, 31, 32, 33], [1] * 8), {}),
    ("f16_d256_g16_long_splits_bs64", (16, 1, 256, 64, "f16", "f16", [15000], [1]), {}),
    ("f16_d256_bs16_window_inside_block", (4, 4, 256, 16, "f16", "f16", [100, 45, 700], [1] * 3), {"sliding_window": 40}),
    ("f16_d96_g17_runs_on_the_generic_kernel", (17, 1, 96, 32, "f16", "f16", [200, 77], [1, 1]), {}),
]


@pytest.mark.parametrize("name,args,kw", DECODE16, ids=[c[0] for c in DECODE16])
def test_decode16_kernel_shapes(pkg, dev, name, args, kw):
    """Single-token sequences over 16-bit caches: the 16-bit decode kernel in steps without dense chunks (with and
    without scores), the matrix kernel otherwise; all against the checker."""
    case = H.case_from_lens(name, *args, **kw)
    got, ref, c = _check(pkg, dev, case, 23, outliers=True, want_scores=False)
    with_scores = H.run_case_on_gpu(pkg, c, dev, True, op=got["op"])
    full = H.run_case_on_checker(c)
    H.assert_close(with_scores["out"], full["out"], c["q_dtype"])
    H.assert_close(with_scores["scores"], full["scores"], "f16", "scores")
    again = H.run_case_on_gpu(pkg, c, dev, False, op=got["op"])
    assert np.array_equal(again["out16"], got["out16"])  # same kernel, same result, whatever ran in between


BLOCK16 = [
    # 16-token cache blocks: a 32-token tile of the decode kernels is two blocks (a last tile may hold one)
    ("b16_u8_d128_g4", (8, 2, 128, 16, "f16", "u8", [0, 14, 15, 16, 17, 31, 32, 33, 47, 48, 49, 700], [1] * 12), {}),
    ("b16_u8_d64_g8_bf16q", (16, 2, 64, 16, "bf16", "u8", [700, 64, 31, 16, 33, 1500], [1] * 6), {}),
    ("b16_u8_multi_split", (8, 2, 128, 16, "f16", "u8", [3000, 2500, 17], [1, 1, 1]), {}),
    ("b16_u8_window", (8, 2, 128, 16, "f16", "u8", [5000, 900, 40, 300], [1] * 4), {"sliding_window": 1000}),
    ("b16_u8_window_unaligned", (8, 2, 128, 16, "f16", "u8", [300, 77, 23], [1] * 3), {"sliding_window": 45}),
    ("b16_u8_g16_w0_mix", (16, 1, 128, 16, "f16", "u8", [300, 77, 500], [1] * 3), {"score_aggregation_window": [1, 0, 1]}),
    ("b16_u8_long", (32, 8, 128, 16, "f16", "u8", [9000, 4100, 33], [1] * 3), {}),
    ("b16_f16_d128_g4", (8, 2, 128, 16, "f16", "f16", [37, 130, 64, 4097, 0, 15, 16, 17, 31, 32, 33], [1] * 11), {}),
    ("b16_bf16_d128_g7", (28, 4, 128, 16, "bf16", "bf16", [1000, 2047, 5], [1] * 3), {}),
    ("b16_f16_d64_g1", (4, 4, 64, 16, "f16", "f16", [300, 64, 63, 1, 16], [1] * 5), {}),
    ("b16_bf16_long_splits_window", (16, 8, 128, 16, "bf16", "bf16", [9000, 4000], [1, 1]), {"sliding_window": 2500}),
    # steps with multi-token sequences: the matrix kernel's 32-token tiles are two blocks as well
    ("b16_u8_mixed_step", (8, 2, 128, 16, "f16", "u8", [300, 0, 77], [1, 40, 1]), {}),
    ("b16_f16_mixed_step", (8, 2, 128, 16, "f16", "f16", [300, 0, 77], [1, 40, 1]), {}),
    ("b16_bf16_g7_mixed", (28, 4, 128, 16, "bf16", "bf16", [0, 700, 333, 40, 2000], [150, 37, 1, 1, 64]),
     {"score_aggregation_window": [8, 37, 1, 0, 3]}),
    ("b16_f16_d64_g8", (32, 4, 64, 16, "f16", "f16", [0, 15, 16, 500], [33, 100, 1, 17]), {}),
    ("b16_f16_chunks_only_window", (4, 4, 128, 16, "f16", "f16", [300, 0], [200, 130]), {"sliding_window": 100}),
    ("b16_bf16_long_chunk", (6, 2, 128, 16, "bf16", "bf16", [1500], [700]), {"score_aggregation_window": [16]}),
    ("b16_u8_g4_mixed", (32, 8, 128, 16, "f16", "u8", [0, 700, 333, 40, 2000, 90], [150, 37, 1, 1, 64, 1]),
     {"score_aggregation_window": [8, 37, 1, 0, 3, 1]}),
    ("b16_u8_bf16q_d64_g8", (16, 2, 64, 16, "bf16", "u8", [0, 31, 16, 500], [33, 100, 1, 17]), {}),
    ("b16_u8_window", (8, 2, 128, 16, "f16", "u8", [300, 0, 1000], [200, 130, 1]), {"sliding_window": 100}),
    ("b16_u8_odd_block_counts", (8, 2, 128, 16, "f16", "u8", [0, 3, 20], [17, 45, 60]), {}),
    # blocks of 64, 128 and 256 tokens (256 is what the reference's GPU plugin uses with XAttention): a tile is a
    # 32-token part of a block
    ("b64_u8_decode", (8, 2, 128, 64, "f16", "u8", [0, 31, 32, 63, 64, 65, 700, 3000], [1] * 8), {}),
    ("b256_u8_decode_multi_split", (32, 8, 128, 256, "f16", "u8", [9000, 4100, 255, 256, 257, 33], [1] * 6), {}),
    ("b128_u8_decode_window", (8, 2, 64, 128, "bf16", "u8", [5000, 900, 40, 300], [1] * 4), {"sliding_window": 1000}),
    ("b256_bf16_decode", (28, 4, 128, 256, "bf16", "bf16", [1000, 2047, 5, 255, 256], [1] * 5), {}),
    ("b64_f16_decode_long", (8, 2, 128, 64, "f16", "f16", [15000, 63], [1, 1]), {}),
    ("b256_bf16_g7_mixed", (28, 4, 128, 256, "bf16", "bf16", [0, 700, 333, 40, 2000], [150, 37, 1, 1, 64]),
     {"score_aggregation_window": [8, 37, 1, 0, 3]}),
    ("b128_f16_chunks_only_window", (4, 4, 128, 128, "f16", "f16", [300, 0], [200, 130]), {"sliding_window": 100}),
    ("b256_u8_g4_mixed", (32, 8, 128, 256, "f16", "u8", [0, 700, 333, 40, 2000, 90], [150, 37, 1, 1, 64, 1]),
     {"score_aggregation_window": [8, 37, 1, 0, 3, 1]}),
    ("b64_u8_bf16q_d64_g8", (16, 2, 64, 64, "bf16", "u8", [0, 31, 64, 500], [33, 100, 1, 17]), {}),
    ("b256_bf16_long_singles", (8, 2, 128, 256, "bf16", "bf16", [0, 5000, 2049], [50, 1, 1]), {}),
]


@pytest.mark.parametrize("name,args,kw", BLOCK16, ids=[c[0] for c in BLOCK16])
def test_block_size_16_steps(pkg, dev, name, args, kw):
    """Caches of 16-token blocks (the block size of the reference's GPU plugin) and of 64 to 256 tokens on the tuned
    kernels, whose 32-token tiles are then two blocks, or a part of one: single-token steps, chunks and mixed steps, with
    and without scores, appended rows included."""
    got, ref, c = _check(pkg, dev, H.case_from_lens(name, *args, **kw), 59, outliers=True)
    got2 = H.run_case_on_gpu(pkg, c, dev, want_scores=False)
    H.assert_close(got2["out"], ref["out"], c["q_dtype"])
    assert np.array_equal(got2["key_cache"], ref["key_cache"]) and np.array_equal(got2["value_cache"], ref["value_cache"])


def test_block_size_16_runs_the_decode_kernels(pkg, dev):
    """The tuned kernels, not the generic one, serve single-token steps over 16-token blocks: pa_attention_static, which
    refuses every step the decode kernels do not take, accepts them and returns what pa_attention returns."""
    import torch
    for qd, kd in (("f16", "u8"), ("bf16", "bf16")):
        c = H.build_case(H.case_from_lens(f"b16_which_{kd}", 8, 2, 128, 16, qd, kd, [5000, 3000, 15], [1, 1, 1]), 5)
        op = pkg.PagedAttention(8, 2, 128, 16, qd, kd, 1, 0, torch.cuda.current_stream(dev))
        q = H.to_device_16(torch, c["query"], qd, dev)
        kc, vc = torch.from_numpy(c["key_cache0"]).to(dev), torch.from_numpy(c["value_cache0"]).to(dev)
        op.step_begin(c["past_lens"], c["subsequence_begins"], c["block_indices_begins"],
                      int((c["past_lens"] + c["new_lens"]).max()), c["score_aggregation_window"], 0, c["scale"])
        op.set_block_indices(c["block_indices"], c["num_blocks"])
        outs = []
        for call in (op.attention_static, op.attention):
            out = torch.full_like(q, float("nan"))
            scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
            call(q, kc, vc, out, scores)
            op.synchronize()
            outs.append((out.view(torch.int16).cpu().numpy(), scores.cpu().numpy()))
        assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
        assert np.isfinite(outs[0][1]).all()


_SHORT = list(range(5, 1500, 23))
WIDE_WORKGROUP = [
    # (name, args, kw, splits): contexts whose probabilities do not fit half a CU's LDS, in steps with at least 256
    # (sequence, kv head) pairs: one workgroup of eight waves per CU takes them with fewer splits than two of four waves
    ("dec_u8_wide_one_split", (32, 8, 128, 32, "f16", "u8", [8100, 6200, 7000] + _SHORT[:29], [1] * 32), {}, 1),
    ("dec_u8_wide_two_splits", (32, 8, 128, 32, "f16", "u8", [13000, 12001] + _SHORT[:30], [1] * 32), {}, 2),
    ("dec_u8_wide_d64_g8_bf16q", (32, 4, 64, 32, "bf16", "u8", [5000, 4100] + _SHORT[:62], [1] * 64), {}, 1),
    ("dec_u8_wide_window", (32, 8, 128, 32, "f16", "u8", [13000, 9000] + _SHORT[:30], [1] * 32),
     {"sliding_window": 7001}, 1),
    ("dec_u8_wide_all_long", (32, 8, 128, 32, "f16", "u8", [6500 + 37 * i for i in range(32)], [1] * 32), {}, 1),
    # next to dense chunks (the matrix kernel takes those; the single-token sequences are listed for the decode kernel)
    ("dec_u8_wide_next_to_chunks", (32, 8, 128, 32, "f16", "u8", [700, 8100, 0] + _SHORT[:32] + [6999],
                                    [130, 1, 40] + [1] * 33), {}, None),
]


@pytest.mark.parametrize("name,args,kw,splits", WIDE_WORKGROUP, ids=[c[0] for c in WIDE_WORKGROUP])
def test_decode_u8_wide_workgroup(pkg, dev, name, args, kw, splits):
    got, ref, c = _check(pkg, dev, H.case_from_lens(name, *args, **kw), 57, outliers=True)
    if splits is not None:
        assert got["op"].num_splits == splits, got["op"].num_splits
    # without scores no probabilities are kept and the plan is the four-wave one
    got2 = H.run_case_on_gpu(pkg, c, dev, want_scores=False)
    H.assert_close(got2["out"], ref["out"], c["q_dtype"])


def test_profiling_and_split_count(pkg, dev):
    """pa_set_profiling / pa_last_kernel_ms / pa_get_num_splits: a long single sequence is cut into KV ranges, a short
    batch is not; the timed kernel reports a plausible duration, and only when timing was asked for."""
    for kd, past, splits in (("u8", [9000], True), ("u8", [100, 40, 77, 300], False), ("bf16", [12000], True)):
        qd = "bf16" if kd == "bf16" else "f16"
        c = H.build_case(H.case_from_lens("prof", 8, 2, 128, 32, qd, kd, past, [1] * len(past)), 9)
        got = H.run_case_on_gpu(pkg, c, dev)
        op = got["op"]
        assert (op.num_splits > 1) == splits, (kd, past, op.num_splits)
        with pytest.raises(pkg.PaError) as e:
            op.last_kernel_ms()
        assert e.value.status == -4
        op.set_profiling(True)
        again = H.run_case_on_gpu(pkg, c, dev, op=op)
        ms = op.last_kernel_ms()
        assert 0.0 < ms < 50.0, ms
        assert np.array_equal(again["out16"], got["out16"]) and np.array_equal(again["scores"], got["scores"])
        op.set_profiling(False)


def _plant_dominant_new_rows(c, logit=16.0, v_plant=3.0):
    """Rewrites the step's new K / V rows (single-token sequences) so that, for the first head of every kv head's
    group, the new token takes nearly all of the softmax mass: K = q * logit / (scale |q|^2), V = a constant.  A
    kernel that attends over the cache before its own append has landed then misses `out` by O(1) and the last score
    by about one per kv head."""
    from oracle import oracle as O
    Hq, Hkv, D = c["Hq"], c["Hkv"], c["D"]
    G = Hq // Hkv
    qd = H.DT[c["q_dtype"]]
    q = O.from_bits(c["query"], qd).reshape(-1, Hq, D)
    k = np.zeros((q.shape[0], Hkv, D), np.float32)
    for h in range(Hkv):
        q0 = q[:, h * G, :]
        k[:, h, :] = q0 * (logit / (c["scale"] * np.maximum((q0 * q0).sum(axis=1, keepdims=True), 1e-6)))
    c["key"] = O.to_bits(k.reshape(q.shape[0], Hkv * D), qd)
    c["value"] = O.to_bits(np.full((q.shape[0], Hkv * D), v_plant, np.float32), qd)


LATE_APPEND = [
    # (query type, cache type, block size, sequences, contexts): single-token steps in which the wave that appends a
    # sequence's new row has fetched other tiles first; one workgroup per (sequence, kv head) and several
    ("f16", "u8", 32, 64, (1100, 1300)), ("bf16", "u8", 16, 64, (1100, 1300)), ("f16", "u8", 64, 64, (1100, 1300)),
    ("f16", "u8", 32, 8, (20000, 33000)), ("bf16", "u8", 32, 8, (26000, 33000)),
    ("f16", "f16", 32, 64, (1100, 1300)), ("bf16", "bf16", 16, 64, (1100, 1300)), ("bf16", "bf16", 32, 8, (20000, 33000)),
    # head size 256 (a seventh field: query heads, kv heads, head size)
    ("f16", "u8", 32, 64, (1100, 1300), (16, 8, 256)), ("bf16", "u8", 64, 8, (20000, 33000), (16, 8, 256)),
    ("bf16", "bf16", 32, 64, (1100, 1300), (16, 8, 256)), ("f16", "f16", 16, 8, (20000, 33000), (12, 4, 96)),
    ("f16", "u8", 32, 64, (1100, 1300), (12, 4, 96)), ("bf16", "u8", 16, 8, (20000, 33000), (6, 6, 96)),
]
LATE_APPEND = [c if len(c) == 6 else c + ((32, 8, 128),) for c in LATE_APPEND]


@pytest.mark.parametrize("qd,kd,bs,B,ctx,heads", LATE_APPEND)
def test_fused_append_row_is_seen_by_the_launch_that_writes_it(pkg, dev, qd, kd, bs, B, ctx, heads):
    """The new token dominates the softmax of one head per kv head, so a stale read of its row fails `out` and
    `scores` outright instead of hiding in the tolerance."""
    Hq, Hkv, D = heads
    past = np.linspace(ctx[0], ctx[1], B).astype(np.int64) | 1  # odd: the new row is never a block's first
    case = H.case_from_lens(f"late_append_{qd}_{kd}_bs{bs}_B{B}_D{D}", Hq, Hkv, D, bs, qd, kd, past, [1] * B)
    print(f"case {case['name']}", flush=True)
    c = H.build_case(case, 4242)
    _plant_dominant_new_rows(c)
    got = H.run_case_on_gpu(pkg, c, dev)
    ref = H.run_case_on_checker(c)
    # the step went down the path this test is about: some sequence's last workgroup walks 17 tiles or more, so the
    # wave that owns the last tile has four tiles in front of it
    n = got["op"].num_splits
    tiles = (past + 1 + 31) // 32
    per = (tiles + n - 1) // n
    assert ((tiles - (n - 1) * per) >= 17).any(), (n, tiles.tolist())
    assert (n > 1) == (B < 32), n
    assert np.array_equal(got["key_cache"], ref["key_cache"]) and np.array_equal(got["value_cache"], ref["value_cache"])
    H.assert_close(got["out"], ref["out"], qd)
    H.assert_close(got["scores"], ref["scores"], "f16", "scores")
    # ... and the planted rows do dominate: the first head of every group returns the planted V row
    G = Hq // Hkv
    o = got["out"].reshape(B, Hq, D)[:, ::G, :]
    assert np.abs(o - 3.0).max() < 0.05, np.abs(o - 3.0).max()



@pytest.mark.parametrize("qd,kd,new", [("f16", "u8", [1, 1]), ("bf16", "bf16", [1, 1]), ("f16", "u8", [1, 300]), ("bf16", "bf16", [1, 300])])
def test_contexts_of_128k_tokens(pkg, dev, qd, kd, new):
    """Two sequences behind 131071 and 70000 cached tokens, decoding or with a chunk beside the long one: the split
    plans at their limits (64 splits, the most tiles a workgroup's LDS holds), int32 offsets far from their ends."""
    case = H.case_from_lens(f"ctx128k_{qd}_{kd}_{new[1]}", 8, 2, 128, 32, qd, kd, [131071, 70000], new,
                            score_aggregation_window=[1, min(new[1], 4)])
    _check(pkg, dev, case, 99)


@pytest.mark.parametrize("qd,kd,mixed", [("f16", "u8", False), ("bf16", "bf16", False), ("f16", "u8", True), ("f16", "f16", True)])
def test_steps_of_three_thousand_sequences(pkg, dev, qd, kd, mixed):
    """Many short sequences in one step (grids, descriptors and lists far beyond the benchmark's batch sizes), all
    decoding or every seventh one with a short chunk."""
    rng = np.random.default_rng(5)
    B = 3000
    past = rng.integers(0, 120, B).tolist()
    new = [int(rng.integers(2, 40)) if mixed and i % 7 == 0 else 1 for i in range(B)]
    case = H.case_from_lens(f"many_seqs_{qd}_{kd}_{mixed}", 8, 2, 64, 32, qd, kd, past, new)
    _check(pkg, dev, case, 17)


def test_decode_u8_ignores_garbage_beyond_the_context(pkg, dev):
    """Rows past kv_len in the last block (and unused blocks) may hold anything, NaN headers included."""
    case = H.case_from_lens("garbage_tail", 8, 2, 128, 32, "f16", "u8", [40, 90], [1, 1])
    c = H.build_case(case, 5)
    ref = H.run_case_on_checker(c)
    rng = np.random.default_rng(0)
    for b in range(2):
        kv = int(c["past_lens"][b]) + 1
        blk = c["block_indices"][c["block_indices_begins"][b] + kv // 32]
        for cache in (c["key_cache0"], c["value_cache0"]):
            cache[blk, :, kv % 32:, :] = rng.integers(0, 256, cache[blk, :, kv % 32:, :].shape, dtype=np.uint8)
            cache[blk, :, kv % 32:, :8] = 0xFF  # NaN scale and zero point
    got = H.run_case_on_gpu(pkg, c, dev)
    H.assert_close(got["out"], ref["out"], "f16")
    H.assert_close(got["scores"], ref["scores"], "f16", "scores")


@pytest.mark.parametrize("qd,kd", [("f16", "u8"), ("bf16", "u8"), ("f16", "f16"), ("bf16", "bf16")])
def test_prefill_ignores_garbage_beyond_the_context(pkg, dev, qd, kd):
    """Same for multi-token sequences: all-ones bytes are NaN as u8 headers, as f16 and as bf16 values."""
    case = H.case_from_lens(f"garbage_tail_prefill_{qd}_{kd}", 8, 2, 128, 32, qd, kd, [40, 90, 0], [9, 1, 33])
    c = H.build_case(case, 6)
    ref = H.run_case_on_checker(c)
    for b in range(3):
        kv = int(c["past_lens"][b] + c["new_lens"][b])
        blk = c["block_indices"][c["block_indices_begins"][b] + (kv - 1) // 32]
        if kv % 32:
            for cache in (c["key_cache0"], c["value_cache0"]):
                cache[blk, :, kv % 32:, :] = 0xFF
    got = H.run_case_on_gpu(pkg, c, dev)
    H.assert_close(got["out"], ref["out"], qd)
    H.assert_close(got["scores"], ref["scores"], "f16", "scores")


class _ByteOffset:
    """Stands for a tensor that starts ``nbytes`` into ``t`` (the binding only asks a tensor for its address)."""

    def __init__(self, t, nbytes):
        self._t, self._n = t, nbytes

    def data_ptr(self):
        return self._t.data_ptr() + self._n


def test_errors_are_reported_not_thrown_across_the_abi(pkg, dev):
    import torch
    op = pkg.PagedAttention(8, 2, 128, 32, "f16", "u8", device=0, stream=torch.cuda.current_stream(dev))
    with pytest.raises(pkg.PaError) as e:  # block table shorter than the context
        op.step_begin([100], [0, 1], [0, 3])
    assert e.value.status == -6
    op.step_begin([100], [0, 1], [0, 4])
    with pytest.raises(pkg.PaError) as e:  # physical id outside the cache
        op.set_block_indices([0, 1, 2, 9], num_blocks=8)
    assert e.value.status == -6
    with pytest.raises(pkg.PaError) as e:  # wrong number of ids
        op.set_block_indices([0, 1, 2], num_blocks=8)
    assert e.value.status == -4
    q = torch.zeros(1, 8 * 128, dtype=torch.float16, device=dev)
    kc = torch.zeros(8, 2, 32, 136, dtype=torch.uint8, device=dev)
    with pytest.raises(pkg.PaError):  # tables not set for this step
        op.attention(q, kc, kc, q)
    with pytest.raises(pkg.PaError):
        pkg.PagedAttention(8, 3, 128)  # heads not a multiple of kv heads
    # a table validated against a large cache, then a layer call with a smaller one: refused before any launch
    op.set_block_indices([0, 1, 2, 40], num_blocks=64)
    for call in (lambda: op.attention(q, kc, kc, q), lambda: op.kv_append(q[:, :256], q[:, :256], kc, kc),
                 lambda: op.forward(q, q[:, :256], q[:, :256], kc, kc, q)):
        with pytest.raises(pkg.PaError) as e:
            call()
        assert e.value.status == -6, str(e.value)
    big = torch.zeros(41, 2, 32, 136, dtype=torch.uint8, device=dev)
    op.attention(q, big, big, torch.zeros_like(q))  # 41 blocks hold id 40
    op.synchronize()
    # tensors off the 16-byte grid the kernels move rows on (views into larger buffers): refused, nothing launched
    pad_q = torch.zeros(8 * 128 + 8, dtype=torch.float16, device=dev)
    pad_c = torch.zeros(big.numel() + 16, dtype=torch.uint8, device=dev)
    off_q, off_c = pad_q[1:1 + 8 * 128].view(1, -1), pad_c[8:8 + big.numel()].view(big.shape)
    sc = torch.zeros(101 + 1, dtype=torch.float32, device=dev)
    for call in (lambda: op.attention(off_q, big, big, torch.zeros_like(q)), lambda: op.attention(q, big, big, off_q),
                 lambda: op.attention(q, off_c, big, torch.zeros_like(q)), lambda: op.attention(q, big, off_c, torch.zeros_like(q)),
                 lambda: op.kv_append(off_q[:, :256], q[:, :256], big, big),
                 lambda: op.attention(q, big, big, torch.zeros_like(q), _ByteOffset(sc, 2))):
        with pytest.raises(pkg.PaError) as e:
            call()
        assert e.value.status == -14, str(e.value)
    op.attention(q, big, big, torch.zeros_like(q), sc[1:])  # a 4-byte offset is fine for scores
    op.synchronize()


def test_full_size_cfg2_properties(pkg, dev):
    """Headline workload at full size: append -> attend round trip, permutation invariance, score mass, and the
    whole batch against the checker."""
    import torch
    wl = __import__("openvino_genai_amd.workloads", fromlist=["x"])
    spec = wl.make_spec(2)
    B, Hq, Hkv, D, bs = spec["B"], spec["Hq"], spec["Hkv"], spec["D"], spec["bs"]
    g = torch.Generator(device=dev).manual_seed(1002)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "u8", device=0, stream=torch.cuda.current_stream(dev))
    nb = spec["num_blocks"]
    kc = torch.zeros(nb, Hkv, bs, D + 8, dtype=torch.uint8, device=dev)
    vc = torch.zeros_like(kc)
    past = spec["past_lens"]
    # fill the past by one prefill-sized append per sequence group (the product's own append, bit-exact by the tests above)
    psb = np.concatenate([[0], np.cumsum(past)]).astype(np.int32)
    Tp = int(psb[-1])
    # (the workload's contents: normal values with 1 % of the elements at +-8)
    kp = _outliers(torch, torch.randn(Tp, Hkv * D, generator=g, device=dev, dtype=torch.float16), g)
    vp = _outliers(torch, torch.randn(Tp, Hkv * D, generator=g, device=dev, dtype=torch.float16), g)
    op.step_begin(np.zeros(B, np.int32), psb, spec["block_indices_begins"])
    op.set_block_indices(spec["block_indices"], nb)
    op.kv_append(kp, vp, kc, vc)
    q = torch.randn(B, Hq * D, generator=g, device=dev, dtype=torch.float16)
    k = torch.randn(B, Hkv * D, generator=g, device=dev, dtype=torch.float16)
    v = torch.randn(B, Hkv * D, generator=g, device=dev, dtype=torch.float16)
    out = torch.zeros_like(q)
    op.step_begin(past, spec["subsequence_begins"], spec["block_indices_begins"])
    op.set_block_indices(spec["block_indices"], nb)
    scores = torch.zeros(op.total_scores, dtype=torch.float32, device=dev)
    op.forward(q, k, v, kc, vc, out, scores)
    op.synchronize()
    assert torch.isfinite(out).all()
    # every softmax row sums to one: a sequence's scores sum to the number of query heads
    mass = scores.view(B, -1).sum(dim=1).cpu().numpy()
    np.testing.assert_allclose(mass, Hq, rtol=1e-3)
    # dequantised rows reproduce the source within half a quantisation step
    seq, tok = 5, 1234
    phys = int(spec["block_indices"][spec["block_indices_begins"][seq] + tok // bs])
    row = kc[phys, 3, tok % bs].cpu().numpy()
    sc, zp = row[:8].view(np.float32)
    src = kp[psb[seq] + tok, 3 * D:4 * D].float().cpu().numpy()
    assert np.all(np.abs((row[8:].astype(np.float32) - zp) * sc - src) <= 0.5 * sc * 1.001 + 1e-6)
    # the same logical cache under another physical placement gives the same bits
    perm = torch.randperm(nb, generator=g, device=dev)
    inv = torch.argsort(perm)
    kc2, vc2 = kc[perm], vc[perm]
    table2 = inv[torch.from_numpy(spec["block_indices"].astype(np.int64)).to(dev)].cpu().numpy().astype(np.int32)
    out2 = torch.zeros_like(q)
    scores2 = torch.zeros_like(scores)
    op.step_begin(past, spec["subsequence_begins"], spec["block_indices_begins"])
    op.set_block_indices(table2, nb)
    op.attention(q, kc2, vc2, out2, scores2)
    op.synchronize()
    assert torch.equal(out, out2) and torch.equal(scores, scores2)
    # every sequence of the batch against the checker at full context
    _check_whole_batch(spec, q, kc, vc, out, scores, None, "f16", "u8", 0)


def _random_case(rng, idx):
    """A random step: shapes, cache type, sequence mix, sliding window and score windows drawn from the ranges the
    kernels are built for (and a few outside, which take the generic path)."""
    D = int(rng.choice([64, 128]))
    Hkv = int(rng.choice([1, 2, 4]))
    G = int(rng.choice([1, 2, 3, 4, 7, 8, 16, 20]))
    qd = str(rng.choice(["f16", "bf16"]))
    kd = str(rng.choice(["u8", qd]))
    bs = 32 if rng.random() < 0.85 else 16
    B = int(rng.integers(1, 7))
    kind = rng.choice(["decode", "prefill", "mixed"])
    past, new = [], []
    for _ in range(B):
        if kind == "decode" or (kind == "mixed" and rng.random() < 0.5):
            past.append(int(rng.integers(0, 900)))
            new.append(1)
        else:
            past.append(int(rng.choice([0, int(rng.integers(1, 600))])))
            new.append(int(rng.integers(2, 200)))
    sw = int(rng.choice([0, 0, int(rng.integers(8, 300))]))
    saw = [int(rng.integers(0, n + 1)) for n in new] if rng.random() < 0.6 else None
    return H.case_from_lens(f"random_{idx}_{kind}_{qd}_{kd}_D{D}_H{Hkv}x{G}_bs{bs}_sw{sw}", Hkv * G, Hkv, D, bs, qd, kd, past, new,
                            sliding_window=sw, score_aggregation_window=saw)


@pytest.mark.parametrize("idx", range(48))
def test_random_steps_against_the_checker(pkg, dev, idx):
    rng = np.random.default_rng(9000 + idx)
    case = _random_case(rng, idx)
    got, ref, c = _check(pkg, dev, case, 9000 + idx, outliers=bool(idx % 2))
    # the same step again on a fresh context: identical bits (no dependence on timing between waves or workgroups)
    again = H.run_case_on_gpu(pkg, c, dev)
    assert np.array_equal(again["out16"], got["out16"]), "output differs between two runs of the same step"
    assert np.array_equal(again["scores"].view(np.uint32), got["scores"].view(np.uint32)), "scores differ between runs"


# Steps that once missed the tolerance on single rows of the u8 matrix path, found by running thousands of random
# steps beyond the ones above (seed = the seed of the generated tensors; all with planted +-8 outliers):
#   a tie in the f16 rounding of a dominant softmax weight, seen differently by the matrix product and the
#   zero-point term; an 11-bit weight on a row that leans on few tokens with opposite V values; a 5000-token context
#   whose accumulator lost half a unit in the last place per product.
SOAK_FINDS = [
    (50239, 80, 4, 128, "f16", [116, 0, 78, 211], [197, 183, 3, 64], 34, [106, 46, 1, 13]),
    (50331, 80, 4, 128, "bf16", [124, 0, 0], [1, 163, 188], 0, [0, 82, 140]),
    (50391, 16, 4, 64, "f16", [0, 0], [126, 197], 0, None),
    (60349, 40, 2, 128, "f16", [721, 898, 380], [1, 1, 197], 0, None),
    (90007, 128, 8, 64, "bf16", [7410, 3598, 3839, 0, 5010, 11125, 13833], [1, 1, 99, 621, 616, 1, 1], 0, None),
]


@pytest.mark.parametrize("seed,Hq,Hkv,D,qd,past,new,sw,saw", SOAK_FINDS, ids=lambda v: str(v) if isinstance(v, int) and v > 1000 else None)
def test_steps_that_once_missed_the_tolerance(pkg, dev, seed, Hq, Hkv, D, qd, past, new, sw, saw):
    case = H.case_from_lens(f"soak_find_{seed}", Hq, Hkv, D, 32, qd, "u8", past, new, sliding_window=sw,
                            score_aggregation_window=saw)
    _check(pkg, dev, case, seed, outliers=True)


def test_peaked_single_token_row_over_u8_cache(pkg, dev):
    """Logits scaled x2 and planted +-8 outliers: head 12 of the sequence at past 4073 leans on a few tokens whose V
    values cancel in one channel; with the softmax weights as one f16 value per token the u8 decode kernel was
    1.1e-3 off there (row magnitude 1.6).  The weights now enter as f16 value + remainder."""
    case = H.case_from_lens("peaked_1600094", 64, 4, 64, 32, "f16", "u8", [7456, 0, 4073, 1006, 4055, 6396, 0],
                            [1, 233, 1, 1, 216, 1, 202], scale=0.25)
    _check(pkg, dev, case, 1600094, outliers=True)


@pytest.mark.parametrize("cfg,kw", [(3, {}), (5, {}), (5, {"sliding_window": 4096}), (1, {}), (4, {})])
def test_full_size_properties_of_the_other_workloads(pkg, dev, cfg, kw):
    """Full-size workloads: append -> attend, score mass per sequence (every softmax row
    sums to one, so a sequence's scores sum to Hq x W), zero scores outside the sliding window, identical bits under
    another physical placement of the blocks, and the whole batch against the checker."""
    import torch
    wl = __import__("openvino_genai_amd.workloads", fromlist=["x"])
    spec = wl.make_spec(cfg, **kw)
    B, Hq, Hkv, D, bs = spec["B"], spec["Hq"], spec["Hkv"], spec["D"], spec["bs"]
    qd, kd = spec["q_dtype"], spec["kv_dtype"]
    print(f"case full-size cfg {cfg} {kw} {qd}/{kd}", flush=True)
    tdt = torch.float16 if qd == "f16" else torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(2000 + cfg)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, qd, kd, device=0, stream=torch.cuda.current_stream(dev))
    nb = spec["num_blocks"]
    kc = torch.zeros(nb, Hkv, bs, pkg.row_bytes(D, kd), dtype=torch.uint8, device=dev)
    vc = torch.zeros_like(kc)
    past, sb, bib = spec["past_lens"], spec["subsequence_begins"], spec["block_indices_begins"]
    new = np.diff(sb)
    psb = np.concatenate([[0], np.cumsum(past)]).astype(np.int32)
    Tp, T = int(psb[-1]), int(sb[-1])
    rnd = lambda n, w: torch.randn(n, w, generator=g, device=dev, dtype=torch.float32).to(tdt)
    sel = [b for b in range(B) if past[b] > 0]  # the past is written by one prefill-sized append of those that have one
    ids = np.concatenate([spec["block_indices"][bib[b]:bib[b + 1]] for b in sel]).astype(np.int32)
    op.step_begin(np.zeros(len(sel), np.int32), np.concatenate([[0], np.cumsum(past[sel])]).astype(np.int32),
                  np.concatenate([[0], np.cumsum([bib[b + 1] - bib[b] for b in sel])]).astype(np.int32))
    op.set_block_indices(ids, nb)
    op.kv_append(rnd(Tp, Hkv * D), rnd(Tp, Hkv * D), kc, vc)
    q, k, v = rnd(T, Hq * D), rnd(T, Hkv * D), rnd(T, Hkv * D)
    out = torch.zeros_like(q)
    W = np.minimum(new, 3).astype(np.int32)  # last three query tokens of every chunk, one for single tokens
    sw = spec["sliding_window"]
    op.step_begin(past, sb, bib, spec["max_context_len"], W, sw, spec["scale"])
    op.set_block_indices(spec["block_indices"], nb)
    scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
    op.forward(q, k, v, kc, vc, out, scores)
    op.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(scores).all()
    sc = scores.cpu().numpy()
    off = np.concatenate([[0], np.cumsum(past + new)])
    for b in range(B):
        s = sc[off[b]:off[b + 1]]
        assert abs(s.sum() - Hq * W[b]) <= 2e-3 * Hq * W[b] + 1e-3, (b, s.sum())
        if sw > 0:  # the last W tokens see nothing before (first of them) + 1 - window
            first_seen = max(0, past[b] + new[b] - W[b] + 1 - sw)
            assert not s[:first_seen].any()
    # another physical placement of the same logical cache: the same bits
    perm = torch.randperm(nb, generator=g, device=dev)
    inv = torch.argsort(perm)
    table2 = inv[torch.from_numpy(spec["block_indices"].astype(np.int64)).to(dev)].cpu().numpy().astype(np.int32)
    out2, scores2 = torch.zeros_like(q), torch.zeros_like(scores)
    op.step_begin(past, sb, bib, spec["max_context_len"], W, sw, spec["scale"])
    op.set_block_indices(table2, nb)
    op.attention(q, kc[perm], vc[perm], out2, scores2)
    op.synchronize()
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16)) and torch.equal(scores, scores2)
    # every sequence of the batch against the checker (config 3's chunks are a minute of checker time)
    _check_whole_batch(spec, q, kc, vc, out, scores, W, qd, kd, sw)


@pytest.mark.parametrize("qd,kd,new", [("f16", "u8", [1, 1, 1, 1]), ("bf16", "bf16", [1, 1, 1, 1]), ("f16", "u8", [1, 40, 1, 3]),
                                       ("bf16", "bf16", [1, 40, 1, 3]), ("f16", "f16", [33, 1, 1, 1])])
def test_sequences_that_share_the_blocks_of_a_common_prefix(pkg, dev, qd, kd, new):
    """Prefix caching hands several sequences the SAME physical blocks for their common prefix (the reference's block
    manager, src/cpp/src/continuous_batching/cache/block_manager.hpp:23-58: blocks with a reference count above one): the tables of four sequences name one set
    of blocks for their first 20 blocks and blocks of their own behind it.  Attention reads the shared blocks once
    per sequence; the step's new rows go to the sequences' own blocks."""
    past = [1000, 700, 2000, 640]
    case = H.case_from_lens(f"shared_prefix_{qd}_{kd}", 8, 2, 128, 32, qd, kd, past, new)
    c = H.build_case(case, 61, outliers=True)
    shared = 20
    bib = c["block_indices_begins"]
    for b in range(1, len(past)):
        c["block_indices"][bib[b]:bib[b] + shared] = c["block_indices"][bib[0]:bib[0] + shared]
    got = H.run_case_on_gpu(pkg, c, dev)
    ref = H.run_case_on_checker(c)
    assert np.array_equal(got["key_cache"], ref["key_cache"]) and np.array_equal(got["value_cache"], ref["value_cache"])
    H.assert_close(got["out"], ref["out"], qd)
    H.assert_close(got["scores"], ref["scores"], "f16", "scores")
    # the shared blocks were not written by the step (every new row lies behind the prefix)
    ids = c["block_indices"][bib[0]:bib[0] + shared]
    assert np.array_equal(got["key_cache"][ids], c["key_cache0"][ids])
