"""A bounded slice of the parity soak: twenty seeded random steps of every kind through the C-ABI against the CPU
checker.  Odd cases get planted +-8 outliers (every ``peaked`` case does)."""
import numpy as np
import pytest

import harness as H
import soak_cases as S
import test_gpu_paged_attention as T
import test_gpu_xattention as TX

pytestmark = pytest.mark.gpu

KINDS = {"small": T._random_case, "big": S.big_case, "peaked": S.peaked_case, "wide": S.wide_case, "sparse": S.sparse_case,
         "heads": S.heads_case}


@pytest.fixture(scope="module")
def dev():
    import torch
    return torch.device("cuda:0")


@pytest.mark.parametrize("i", range(20))
@pytest.mark.parametrize("kind", list(KINDS))
def test_soak_slice(pkg, dev, kind, i):
    seed = 70000 + 1000 * list(KINDS).index(kind) + i
    case = KINDS[kind](np.random.default_rng(seed), seed)
    if kind == "sparse":
        TX._check(pkg, dev, H.build_case(case, seed, outliers=bool(i % 2)), case["thresholds"], case["xb"], case["S"],
                  min_decided=0.0)
    else:
        T._check(pkg, dev, case, seed, outliers=kind == "peaked" or bool(i % 2))
