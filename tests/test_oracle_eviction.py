"""Pins the CPU checker's eviction restatement to the reference's own known-answer vectors."""
import types

import pytest

import eviction_kats as K
from oracle import oracle as O

IMPL = types.SimpleNamespace(
    ScoreManager=O.ScoreManager, CacheEvictionAlgorithm=O.CacheEvictionAlgorithm, add_with_skips=O.add_with_skips,
    snapkv_num_scores=O.snapkv_num_scores,
    MODES={"SUM": O.MODE_SUM, "NORM_SUM": O.MODE_NORM_SUM, "ADAPTIVE_RKV": O.MODE_ADAPTIVE_RKV})
KATS = K.KATS


@pytest.mark.parametrize("case", KATS["add_with_skips"]["cases"])
def test_add_with_skips(case):
    K.check_add_with_skips(IMPL, case)


@pytest.mark.parametrize("case", KATS["register_scores"]["cases"], ids=lambda c: c["id"])
def test_register_scores(case):
    K.check_register_scores(IMPL, case, KATS["register_scores"]["abs_tol"])


@pytest.mark.parametrize("case", KATS["adaptive_rkv_register_scores"]["cases"], ids=lambda c: c["id"])
def test_adaptive_rkv_register_scores(case):
    K.check_adaptive_rkv(IMPL, case, KATS["adaptive_rkv_register_scores"]["abs_tol"])


@pytest.mark.parametrize("case", KATS["snapkv_counters"]["cases"], ids=lambda c: c["id"])
def test_snapkv_counters(case):
    K.check_snapkv_counters(IMPL, case)


@pytest.mark.parametrize("case", KATS["remove_scores"]["cases"], ids=lambda c: c["id"])
def test_remove_scores(case):
    K.check_remove_scores(IMPL, case, KATS["remove_scores"]["abs_tol"])


@pytest.mark.parametrize("case", KATS["snapkv_score_aggregator"]["cases"], ids=lambda c: c["id"])
def test_snapkv_score_aggregator(case):
    assert O.snapkv_num_scores(case["snapkv"], case["prompt_len"], case["num_scheduled"], case["num_processed"]) == case["ref"]


@pytest.mark.parametrize("n", KATS["no_eviction_token_counts"]["counts"])
def test_no_eviction_below_total_size(n):
    K.check_no_eviction_below_total_size(IMPL, n)


@pytest.mark.parametrize("case", KATS["range_calculation"]["cases"], ids=lambda c: str(c["num_tokens"]))
def test_evictable_range(case):
    K.check_range(IMPL, case)


def test_starts_evicting_once_max_size_exceeded():
    K.check_starts_evicting(IMPL)


@pytest.mark.parametrize("case", KATS["low_score_block_eviction"]["cases"], ids=lambda c: c["id"])
def test_low_score_blocks(case):
    K.check_low_score(IMPL, case)


@pytest.mark.parametrize("case", KATS["normalization_setting"]["cases"],
                         ids=lambda c: f'{c["mode"]}_{c["power"]}_{"rising" if c["rising"] else "falling"}')
def test_normalization_setting(case):
    K.check_normalization(IMPL, case)


@pytest.mark.parametrize("mode", KATS["scores_are_accumulated"]["modes"])
def test_scores_are_accumulated(mode):
    K.check_scores_are_accumulated(IMPL, mode)


@pytest.mark.parametrize("c", KATS["invalid_config"]["config_cases"])
def test_invalid_config(c):
    with pytest.raises(ValueError):
        O.CacheEvictionAlgorithm(c[0], c[1], c[2], O.MODE_NORM_SUM, 8, 1, 1, 1)


@pytest.mark.parametrize("c", KATS["invalid_config"]["algo_cases"])
def test_invalid_algo_config(c):
    with pytest.raises(ValueError):
        O.CacheEvictionAlgorithm(c["start"], c["recent"], c["max"], O.MODE_NORM_SUM, 8, c["block_size"], c["layers"], 1)


@pytest.mark.parametrize("layers", [1, 4, 13, 23, 42])  # tests/cpp/cache_eviction.cpp:814-821
def test_evicted_blocks_are_layered_as_configured(layers):
    algo = K.make_algo(IMPL, "DEFAULT", 1, layers=layers)
    assert len(algo.evict_logical_blocks()) == layers
