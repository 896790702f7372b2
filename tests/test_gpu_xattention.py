"""Block-sparse prefill (XAttention) through the C-ABI against the CPU checker.

Three links are checked separately, so that a near-tie in the selection cannot hide behind a tolerance:
  * the block importances against the checker's (floating point, tolerance below);
  * the kept block pairs against the checker's selection *from the GPU's importances*: exact;
  * outputs and scores against the checker's attention *under the GPU's mask*: the usual tolerance.
And, end to end, the kept pairs against the checker's own wherever the checker's decision has slack.
"""
import numpy as np
import pytest

import harness as H
import xattention_cases as X
from oracle import oracle as O

pytestmark = pytest.mark.gpu

# The block importances are an internal quantity (the op's outputs are held to the tolerance of the path); they
# are compared with the checker's binary64 values at 2e-3 relative for 16-bit caches.  Over u8 caches the keys enter
# the matrix cores dequantised and rounded to f16 (11 bits; the quantisation that produced the codes moved every key
# element by up to half a step, 40 times as much), which moves a logit by a few 1e-3 where queries and keys hold
# planted +-8 outliers and the stride is 1, and a probability by as much in relative terms: the largest deviation in
# 1900 random block-sparse steps was 7e-3; 1e-2 there.  The selection is checked exactly against the checker's
# selection from these very sums, and the op's outputs under the resulting mask at the tolerance of the path.
SUM_RTOL, SUM_ATOL = {"f16": 2e-3, "bf16": 2e-3, "u8": 1e-2}, 2e-5


@pytest.fixture(scope="module")
def env():
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    assert torch.cuda.is_available()
    return pkg, torch.device("cuda:0")


def _run(pkg, dev, c, thresholds, xb, S, want_scores=True):
    import torch
    op = pkg.PagedAttention(c["Hq"], c["Hkv"], c["D"], c["bs"], c["q_dtype"], c["kv_dtype"], num_layers=1,
                            device=dev.index or 0, stream=torch.cuda.current_stream(dev))
    q = H.to_device_16(torch, c["query"], c["q_dtype"], dev)
    k = H.to_device_16(torch, c["key"], c["q_dtype"], dev)
    v = H.to_device_16(torch, c["value"], c["q_dtype"], dev)
    kc = torch.from_numpy(c["key_cache0"]).to(dev)
    vc = torch.from_numpy(c["value_cache0"]).to(dev)
    out = torch.zeros_like(q)
    op.step_begin(c["past_lens"], c["subsequence_begins"], c["block_indices_begins"],
                  int((c["past_lens"] + c["new_lens"]).max()), c["score_aggregation_window"], c["sliding_window"],
                  c["scale"])
    op.set_block_indices(c["block_indices"], c["num_blocks"])
    op.set_xattention(thresholds, xb, S)
    scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev) if want_scores else None
    op.forward(q, k, v, kc, vc, out, scores)
    op.synchronize()
    torch.cuda.synchronize(dev)
    sums, kept = [], []
    for b in range(c["B"]):
        if op.xattention_shape(b)[1] > 0:
            sums.append(op.xattention_block_sums(b))
            kept.append(op.xattention_retained(b))
        else:
            sums.append(None)
            kept.append(None)
    return dict(out=out.float().cpu().numpy(), scores=scores.cpu().numpy() if want_scores else None,
                key_cache=kc.cpu().numpy(), sums=sums, kept=kept, op=op)


def _check(pkg, dev, c, thresholds, xb, S, want_scores=True, min_decided=0.5):
    got = _run(pkg, dev, c, thresholds, xb, S, want_scores)
    decided = total = 0
    for b in range(c["B"]):
        sparse = thresholds[b] > 0 and c["new_lens"][b] > 1
        assert (got["kept"][b] is not None) == sparse, f"sequence {b}"
        if not sparse:
            continue
        qb0 = int(c["past_lens"][b]) // xb
        ref_sums = X.checker_block_sums(c, got["key_cache"], b, xb, S)
        err = np.abs(got["sums"][b] - ref_sums)
        assert (err <= SUM_ATOL + SUM_RTOL[c["kv_dtype"]] * np.abs(ref_sums)).all(), f"block sums of sequence {b}: worst {err.max():.3g}"
        same_input, _ = O.xattention_select(got["sums"][b].astype(np.float64), qb0, thresholds[b])
        assert np.array_equal(got["kept"][b], same_input), f"selection of sequence {b} from the same block sums"
        own, slack = O.xattention_select(ref_sums, qb0, thresholds[b])
        rows_equal = (got["kept"][b] == own).all(axis=2)
        # a decision with less room than the estimates differ by may fall either way
        row_err = err.max(axis=2) / ref_sums.sum(axis=2)
        clear = slack > 20 * row_err + 1e-6
        assert rows_equal[clear].all(), f"selection of sequence {b} differs where the decision is clear"
        decided += int(clear.sum())
        total += clear.size
    if total:
        assert decided >= min_decided * total, f"only {decided} of {total} rows have a clear decision"
    ref = X.checker_step(c, got["kept"], xb, want_scores)
    H.assert_close(got["out"], ref["out"], c["q_dtype"])
    if want_scores:
        H.assert_close(got["scores"], ref["scores"], c["q_dtype"], "scores")
    return got


CASES = [
    # name, Hq, Hkv, D, q, kv, past, new, xb, S, scale multiple
    ("f16_aligned", 8, 2, 128, "f16", "f16", [0, 512], [512, 256], 64, 8, 4.0),
    ("bf16_unaligned", 14, 2, 128, "bf16", "bf16", [37, 1000, 3], [300, 171, 80], 64, 8, 4.0),
    ("u8_f16", 8, 2, 128, "f16", "u8", [100, 777], [260, 333], 64, 8, 4.0),
    ("u8_bf16_d64", 8, 4, 64, "bf16", "u8", [64, 0], [200, 129], 32, 4, 6.0),
    ("f16_d64_big_blocks", 4, 4, 64, "f16", "f16", [1000], [500], 128, 16, 6.0),
    ("stride_1", 4, 2, 64, "f16", "f16", [50], [150], 32, 1, 6.0),
    ("stride_32", 8, 2, 128, "bf16", "bf16", [640], [384], 256, 32, 4.0),
    ("long_context_split", 8, 2, 128, "f16", "u8", [6000], [512], 64, 8, 4.0),
    ("gqa_7", 28, 4, 128, "bf16", "bf16", [2048], [512], 64, 8, 3.0),
    # head size 256: four 64-channel stages per slot, the matrix kernel's one-row-group variant with one workgroup per CU
    ("d256_f16", 8, 4, 256, "f16", "f16", [37, 1000], [300, 171], 64, 8, 4.0),
    ("d256_u8_bf16", 16, 8, 256, "bf16", "u8", [100, 2500], [260, 333], 64, 8, 4.0),
]


@pytest.mark.parametrize("name,Hq,Hkv,D,qd,kd,past,new,xb,S,mult", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("threshold", [0.6, 0.9])
def test_sparse_prefill(env, name, Hq, Hkv, D, qd, kd, past, new, xb, S, mult, threshold):
    pkg, dev = env
    case = H.case_from_lens(name, Hq, Hkv, D, 32, qd, kd, past, new, scale=mult / np.sqrt(D),
                            score_aggregation_window=[min(8, n) for n in new])
    c = H.build_case(case, 4242 + len(name), outliers=True)
    # ~100 key blocks of nearly equal importance under f16-rounded u8 keys: few rows are decided with room to spare
    # there; the three links above still hold for every row
    got = _check(pkg, dev, c, np.full(len(past), threshold, np.float32), xb, S,
                 min_decided=0.0 if name == "long_context_split" else 0.5)
    kept = np.concatenate([k.ravel() for k in got["kept"]])
    assert kept.mean() < 1.0  # something was left out, or the case says nothing about masking


def test_mixed_step(env):
    """Sparse chunks, a dense chunk (threshold 0) and single-token sequences in one step, with a sliding window."""
    pkg, dev = env
    past = [300, 40, 2000, 511, 900]
    new = [200, 1, 130, 1, 64]
    for kd, sw in (("u8", 0), ("bf16", 0), ("u8", 700)):
        case = H.case_from_lens("mixed", 16, 4, 128, 32, "bf16", kd, past, new, scale=4.0 / np.sqrt(128), sliding_window=sw,
                                score_aggregation_window=[4, 1, 0, 1, 64])
        c = H.build_case(case, 99, outliers=True)
        _check(pkg, dev, c, np.array([0.8, 0.8, 0.0, 0.0, 0.7], np.float32), 64, 8)


def test_mixed_step_with_256_token_cache_blocks(env):
    """The block size the reference's GPU plugin uses with XAttention: 256-token cache blocks, key blocks of 256 and of
    64 positions."""
    pkg, dev = env
    past = [300, 40, 2000, 511, 900]
    new = [200, 1, 130, 1, 64]
    for kd, xb, bs in (("u8", 256, 256), ("bf16", 64, 256), ("bf16", 128, 64)):
        case = H.case_from_lens("mixed_b256", 16, 4, 128, bs, "bf16", kd, past, new, scale=4.0 / np.sqrt(128),
                                score_aggregation_window=[4, 1, 0, 1, 64])
        c = H.build_case(case, 98, outliers=True)
        _check(pkg, dev, c, np.array([0.8, 0.8, 0.0, 0.0, 0.7], np.float32), xb, 8)


def test_threshold_zero_is_dense(env):
    pkg, dev = env
    case = H.case_from_lens("dense", 8, 2, 128, 32, "f16", "u8", [100, 30], [200, 1])
    c = H.build_case(case, 5)
    plain = H.run_case_on_gpu(pkg, c, dev)
    for thr in (None, np.zeros(2, np.float32)):
        got = _run(pkg, dev, c, thr, 64, 8)
        assert got["kept"] == [None, None]
        assert np.array_equal(got["out"], plain["out"]) and np.array_equal(got["scores"], plain["scores"])


def test_threshold_one_keeps_everything_visible(env):
    pkg, dev = env
    case = H.case_from_lens("all", 4, 2, 64, 32, "f16", "f16", [128], [256])
    c = H.build_case(case, 6)
    got = _run(pkg, dev, c, np.ones(1, np.float32), 64, 8)
    dense = H.run_case_on_checker(c)
    H.assert_close(got["out"], dense["out"], "f16")
    kept = got["kept"][0]
    for i in range(kept.shape[1]):
        # all but at most the least important block of a row: the running sum may reach the total one step early
        assert kept[:, i, :2 + i + 1].sum(axis=1).min() >= 2 + i


def test_step_after_a_sparse_one_is_dense_again(env):
    pkg, dev = env
    case = H.case_from_lens("again", 8, 2, 128, 32, "f16", "f16", [256], [256], scale=4.0 / np.sqrt(128))
    c = H.build_case(case, 8)
    got = _check(pkg, dev, c, np.array([0.5], np.float32), 64, 8)
    plain = H.run_case_on_gpu(pkg, c, dev, op=got["op"])  # same context, no set_xattention in this step
    dense = H.run_case_on_checker(c)
    H.assert_close(plain["out"], dense["out"], "f16")
    assert got["op"].xattention_shape(0) == (0, 0, 0)


def test_rejected_configurations(env):
    import torch
    pkg, dev = env
    op = pkg.PagedAttention(8, 2, 128, 32, "f16", "u8", device=0, stream=torch.cuda.current_stream(dev))
    thr = np.array([0.5], np.float32)
    with pytest.raises(pkg.PaError) as e:
        op.set_xattention(thr, 64, 8)
    assert e.value.status == -4  # no step yet
    op.step_begin([0], [0, 64], [0, 2])
    for xb, S in ((48, 8), (16, 8), (64, 3), (64, 64)):
        with pytest.raises(pkg.PaError) as e:
            op.set_xattention(thr, xb, S)
        assert e.value.status == -2, (xb, S)
    for bad in (-0.1, 1.5, float("nan")):
        with pytest.raises(pkg.PaError) as e:
            op.set_xattention(np.array([bad], np.float32), 64, 8)
        assert e.value.status == -4
    op.set_xattention(thr, 64, 8)
    assert op.xattention_shape(0) == (0, 1, 1)
    with pytest.raises(pkg.PaError) as e:  # nothing has been computed yet
        op.xattention_retained(0)
    assert e.value.status == -4
    with pytest.raises(pkg.PaError):
        op.xattention_shape(1)
    # a shape the matrix kernel does not take
    op2 = pkg.PagedAttention(8, 2, 128, 16, "f16", "f16", device=0, stream=torch.cuda.current_stream(dev))
    op2.step_begin([0], [0, 64], [0, 4])
    with pytest.raises(pkg.PaError) as e:
        op2.set_xattention(thr, 64, 8)
    assert e.value.status == -2
    op2.set_xattention(np.zeros(1, np.float32), 64, 8)  # nothing sparse: nothing to refuse


@pytest.mark.parametrize("kv_dtype", ["u8", "f16"])
def test_chunked_prefill_like_the_pipeline(env, kv_dtype):
    """A prompt prefilled in scheduler-sized chunks next to a sequence that decodes, thresholds from the scheduler's
    rule (sparse chunks first, the chunk near the prompt's end dense), one context and one pair of caches carried
    across the steps: every step's outputs against the checker under the step's own masks, caches bit for bit."""
    import torch
    pkg, dev = env
    Hq, Hkv, D, bs, chunk, prompt = 8, 2, 128, 32, 200, 1130
    cfg = pkg.SparseAttentionConfig(mode=pkg.SparseAttentionMode.XATTENTION, xattention_threshold=0.8,
                                    num_last_dense_tokens_in_prefill=150)
    rng = np.random.default_rng(77)
    qd = O.DT_F16
    n_blocks = 200
    perm = rng.permutation(n_blocks)
    tab_a, tab_b = perm[:(prompt + 40) // bs + 1], perm[60:60 + 12]   # two sequences' block tables
    rb = O.row_bytes(D, H.DT[kv_dtype])
    kc_h = np.zeros((n_blocks, Hkv, bs, rb), np.uint8)
    vc_h = np.zeros_like(kc_h)
    kc, vc = torch.from_numpy(kc_h).to(dev), torch.from_numpy(vc_h).to(dev)
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", kv_dtype, device=0, stream=torch.cuda.current_stream(dev))
    done_a, past_b = 0, 0
    sparse_steps = dense_steps = 0
    while done_a < prompt + 3:
        new_a = min(chunk, prompt - done_a) if done_a < prompt else 1
        new_b = 37 if past_b == 0 else 1                                # sequence b: a short prompt, then decoding
        thr_a = pkg.schedule_xattention_threshold(cfg, prompt, done_a, new_a, done_a >= prompt)
        thr_b = pkg.schedule_xattention_threshold(cfg, 37, past_b, new_b, past_b >= 37)
        past = np.array([done_a, past_b], np.int32)
        new = np.array([new_a, new_b], np.int32)
        c = dict(B=2, Hq=Hq, Hkv=Hkv, D=D, bs=bs, q_dtype="f16", kv_dtype=kv_dtype, past_lens=past, new_lens=new,
                 subsequence_begins=np.array([0, new_a, new_a + new_b], np.int32), sliding_window=0,
                 score_aggregation_window=np.array([min(new_a, 8), 1], np.int32), scale=3.0 / np.sqrt(D),
                 num_blocks=n_blocks)
        nb = [(done_a + new_a + bs - 1) // bs, (past_b + new_b + bs - 1) // bs]
        c["block_indices"] = np.concatenate([tab_a[:nb[0]], tab_b[:nb[1]]]).astype(np.int32)
        c["block_indices_begins"] = np.array([0, nb[0], nb[0] + nb[1]], np.int32)
        T = new_a + new_b
        c["query"], c["key"], c["value"] = (O.to_bits(rng.standard_normal((T, w)).astype(np.float32), qd)
                                            for w in (Hq * D, Hkv * D, Hkv * D))
        c["key_cache0"], c["value_cache0"] = kc_h, vc_h
        thr = np.array([thr_a, thr_b], np.float32)
        q, k, v = (H.to_device_16(torch, c[n], "f16", dev) for n in ("query", "key", "value"))
        out = torch.zeros_like(q)
        op.step_begin(past, c["subsequence_begins"], c["block_indices_begins"], int((past + new).max()),
                      c["score_aggregation_window"], 0, c["scale"])
        op.set_block_indices(c["block_indices"], n_blocks)
        op.set_xattention(thr, cfg.xattention_block_size, cfg.xattention_stride)
        scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
        op.forward(q, k, v, kc, vc, out, scores)
        op.synchronize()
        kept = [op.xattention_retained(b) if op.xattention_shape(b)[1] else None for b in range(2)]
        assert [x is not None for x in kept] == [bool(t > 0 and n > 1) for t, n in zip(thr, new)]
        sparse_steps += kept[0] is not None
        dense_steps += kept[0] is None
        ref = X.checker_step(c, kept, cfg.xattention_block_size)
        H.assert_close(out.float().cpu().numpy(), ref["out"], "f16")
        H.assert_close(scores.cpu().numpy(), ref["scores"], "f16", "scores")
        kc_h, vc_h = ref["key_cache"], ref["value_cache"]
        assert np.array_equal(kc.cpu().numpy(), kc_h) and np.array_equal(vc.cpu().numpy(), vc_h)
        done_a += new_a
        past_b += new_b
    assert sparse_steps >= 4 and dense_steps >= 3  # chunks before the dense tail; the tail and the decode steps
