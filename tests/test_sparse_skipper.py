"""Tri-shape sparse prefill block skipper: the CPU checker and the library's host code against the reference's 43
cases (tests/cpp/sparse_attention.cpp:23-72), and a skipped-block step through the packing and the attention kernels."""
import json
import os

import pytest

from oracle import oracle as O

KATS = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sparse_skipper_kats.json")))


def test_all_reference_cases_were_transcribed():
    assert len(KATS["cases"]) == 43


@pytest.mark.parametrize("case", KATS["cases"], ids=[c["id"] for c in KATS["cases"]])
def test_checker(case):
    got = O.trishape_skipped_blocks(KATS["block_size"], case["num_last_dense_tokens_in_prefill"],
                                    case["num_retained_start_tokens_in_cache"], case["num_retained_recent_tokens_in_cache"],
                                    case["prompt_len"], case["num_tokens_in_cache"], case["num_tokens_in_new_chunk"])
    assert got == set(case["skipped"])


@pytest.mark.parametrize("case", KATS["cases"], ids=[c["id"] for c in KATS["cases"]])
def test_library(pkg, case):
    sk = pkg.TriShapeSparseAttentionTokenSkipper(KATS["block_size"], case["num_last_dense_tokens_in_prefill"],
                                                 case["num_retained_start_tokens_in_cache"],
                                                 case["num_retained_recent_tokens_in_cache"])
    assert sk.get_skipped_blocks(case["prompt_len"], case["num_tokens_in_cache"], case["num_tokens_in_new_chunk"]) == set(case["skipped"])


def test_library_rejects_bad_arguments(pkg):
    with pytest.raises(pkg.PaError):
        pkg.TriShapeSparseAttentionTokenSkipper(32, 5, 33, 32)
    sk = pkg.TriShapeSparseAttentionTokenSkipper(32, 5, 32, 32)
    with pytest.raises(pkg.PaError):
        sk.get_skipped_blocks(10, 8, 3)  # chunk runs past the prompt


@pytest.mark.gpu
def test_skipped_blocks_step_on_gpu(pkg):
    """A prefill chunk with skipped blocks is an ordinary step over a shorter table: past_lens shrinks by the skipped
    tokens (model_runner.hpp:804,818) and the table lists the kept blocks (:1452-1463).  Parity with the checker run
    on the same packed inputs."""
    import torch
    import harness as H
    dev = torch.device("cuda:0")
    bs, prompt_len, processed, chunk = 32, 300, 250, 11
    sk = pkg.TriShapeSparseAttentionTokenSkipper(bs, 10, 32, 32)
    skipped = sk.get_skipped_blocks(prompt_len, processed, chunk)
    assert skipped == {1, 2, 3, 4, 5}
    n_logical = (processed + chunk + bs - 1) // bs
    past, sb, bib, mx = pkg.pack_step([processed], [0], [len(skipped)], [chunk], [n_logical], bs)
    assert past[0] == processed - len(skipped) * bs and bib[1] == n_logical - len(skipped) and mx == processed + chunk
    case = H.case_from_lens("sparse_chunk", 8, 2, 128, bs, "f16", "u8", past, [chunk])
    c = H.build_case(case, 9)
    got = H.run_case_on_gpu(pkg, c, dev)
    ref = H.run_case_on_checker(c)
    H.assert_close(got["out"], ref["out"], "f16")
    H.assert_close(got["scores"], ref["scores"], "f16", "scores")
    assert len(got["scores"]) == past[0] + chunk
