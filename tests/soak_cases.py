"""Generators of random steps beyond the suite's own: longer contexts and chunks (``big``), logits scaled so that few
tokens carry a row (``peaked``), decode steps that take the eight-wave plan of the u8 decode kernel (``wide``) and
block-sparse prefill steps (``sparse``), and steps at head sizes 96 and 256 (``heads``).  Used by
``test_gpu_soak_slice.py``."""
import numpy as np

import harness as H


def big_case(rng, idx):
    D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 8])); G = int(rng.choice([1, 4, 5, 8, 16]))
    qd = str(rng.choice(["f16", "bf16"])); kd = str(rng.choice(["u8", "u8", qd]))
    B = int(rng.integers(1, 10))
    kind = rng.choice(["decode", "prefill", "mixed"])
    past, new = [], []
    for _ in range(B):
        if kind == "decode" or (kind == "mixed" and rng.random() < 0.6):
            past.append(int(rng.choice([int(rng.integers(0, 3000)), int(rng.integers(3000, 14000))])))
            new.append(1)
        else:
            past.append(int(rng.choice([0, int(rng.integers(1, 6000))])))
            new.append(int(rng.integers(2, 700)))
    sw = int(rng.choice([0, 0, 0, int(rng.integers(64, 5000))]))
    saw = [int(rng.integers(0, min(n, 16) + 1)) for n in new] if rng.random() < 0.7 else None
    bs = 16 if idx % 4 == 3 else 32  # (from the index, not the generator: the other cases stay what they were)
    return H.case_from_lens(f"big_{idx}_{kind}_{qd}_{kd}_D{D}_H{Hkv}x{G}_sw{sw}_b{bs}", Hkv * G, Hkv, D, bs, qd, kd, past, new,
                            sliding_window=sw, score_aggregation_window=saw)


def heads_case(rng, idx):
    """Head sizes 96 and 256: the tuned kernels' instantiations with six value channels per lane / one workgroup per
    CU (and, with more than 16 heads per kv head or 16-token blocks at 256 over u8, the shape-generic kernel)."""
    D = int(rng.choice([96, 256])); Hkv = int(rng.choice([1, 2, 8])); G = int(rng.choice([1, 2, 3, 4, 8, 16, 20]))
    qd = str(rng.choice(["f16", "bf16"])); kd = str(rng.choice(["u8", "u8", qd]))
    bs = int(rng.choice([16, 32, 32, 32, 64, 128]))
    B = int(rng.integers(1, 9))
    kind = rng.choice(["decode", "decode", "prefill", "mixed"])
    past, new = [], []
    for _ in range(B):
        if kind == "decode" or (kind == "mixed" and rng.random() < 0.6):
            past.append(int(rng.choice([int(rng.integers(0, 2000)), int(rng.integers(2000, 9000))])))
            new.append(1)
        else:
            past.append(int(rng.choice([0, int(rng.integers(1, 4000))])))
            new.append(int(rng.integers(2, 400)))
    sw = int(rng.choice([0, 0, 0, int(rng.integers(40, 3000))]))
    saw = [int(rng.integers(0, min(n, 16) + 1)) for n in new] if rng.random() < 0.7 else None
    mult = float(rng.choice([1.0, 1.0, 1.0, 4.0]))
    return H.case_from_lens(f"heads_{idx}_{kind}_{qd}_{kd}_D{D}_H{Hkv}x{G}_sw{sw}_b{bs}_x{mult}", Hkv * G, Hkv, D, bs, qd, kd,
                            past, new, sliding_window=sw, score_aggregation_window=saw, scale=mult / np.sqrt(D))


def peaked_case(rng, idx):
    D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4])); G = int(rng.choice([1, 4, 8, 16]))
    qd = str(rng.choice(["f16", "bf16"])); kd = str(rng.choice(["u8", "u8", qd]))
    B = int(rng.integers(1, 8))
    kind = rng.choice(["decode", "prefill", "mixed"])
    past, new = [], []
    for _ in range(B):
        if kind == "decode" or (kind == "mixed" and rng.random() < 0.6):
            past.append(int(rng.integers(0, 9000)))
            new.append(1)
        else:
            past.append(int(rng.choice([0, int(rng.integers(1, 5000))])))
            new.append(int(rng.integers(2, 300)))
    mult = float(rng.choice([2.0, 4.0, 8.0]))
    bs = 16 if idx % 4 == 3 else 32
    return H.case_from_lens(f"peaked_{idx}_{kind}_{qd}_{kd}_D{D}_H{Hkv}x{G}_x{mult}_b{bs}", Hkv * G, Hkv, D, bs, qd, kd, past, new,
                            scale=mult / np.sqrt(D))


def wide_case(rng, idx):
    D = int(rng.choice([64, 128])); Hkv = int(rng.choice([4, 8])); G = int(rng.choice([1, 2, 4, 5, 8, 16]))
    qd = str(rng.choice(["f16", "bf16"]))
    B = 256 // Hkv + int(rng.integers(0, 12))
    cap4 = (80640 - 4 * 32 * (D + 8) - 1024) // (64 + 64 * G + 4)   # blocks a four-wave workgroup can keep
    lo = 32 * cap4 + 1
    past = [int(rng.integers(lo, min(3 * lo, 20000))) for _ in range(int(rng.integers(1, 4)))]
    past += [int(rng.integers(0, 1500)) for _ in range(B - len(past))]
    past = [past[i] for i in rng.permutation(B)]
    sw = int(rng.choice([0, 0, int(rng.integers(lo, 2 * lo))]))
    mult = float(rng.choice([1.0, 1.0, 2.0, 4.0]))
    saw = [int(rng.integers(0, 2)) for _ in range(B)] if rng.random() < 0.3 else None
    return H.case_from_lens(f"wide_{idx}_{qd}_D{D}_H{Hkv}x{G}_sw{sw}_x{mult}", Hkv * G, Hkv, D, 32, qd, "u8", past, [1] * B,
                            sliding_window=sw, score_aggregation_window=saw, scale=mult / np.sqrt(D))


def sparse_case(rng, idx):
    D = int(rng.choice([64, 128])); Hkv = int(rng.choice([1, 2, 4])); G = int(rng.choice([1, 2, 4, 7, 8]))
    qd = str(rng.choice(["f16", "bf16"])); kd = str(rng.choice(["u8", qd]))
    B = int(rng.integers(1, 6))
    past, new, thr = [], [], []
    for _ in range(B):
        r = rng.random()
        if r < 0.25:    # single-token sequence: never sparse, whatever its threshold
            past.append(int(rng.integers(0, 3000))); new.append(1); thr.append(float(rng.choice([0.0, 0.8])))
        elif r < 0.4:   # dense chunk
            past.append(int(rng.choice([0, int(rng.integers(1, 3000))]))); new.append(int(rng.integers(2, 300))); thr.append(0.0)
        else:
            past.append(int(rng.choice([0, int(rng.integers(1, 2000)), int(rng.integers(2000, 7000))])))
            new.append(int(rng.integers(2, 600))); thr.append(float(rng.choice([0.3, 0.6, 0.8, 0.9, 0.95, 1.0])))
    xb = int(rng.choice([32, 64, 64, 128, 256])); S = int(rng.choice([1, 4, 8, 8, 16, 32]))
    if S == 1 and max(p + n for p, n in zip(past, new)) > 3000:
        S = 8  # keep the checker's share of the soak short
    sw = int(rng.choice([0, 0, 0, int(rng.integers(200, 3000))]))
    saw = [int(rng.integers(0, min(n, 16) + 1)) for n in new] if rng.random() < 0.7 else None
    mult = float(rng.choice([1.0, 3.0, 6.0]))
    case = H.case_from_lens(f"sparse_{idx}_{qd}_{kd}_D{D}_H{Hkv}x{G}_xb{xb}_S{S}_sw{sw}", Hkv * G, Hkv, D, 32, qd, kd, past, new,
                            sliding_window=sw, score_aggregation_window=saw, scale=mult / np.sqrt(D))
    case["thresholds"], case["xb"], case["S"] = np.array(thr, np.float32), xb, S
    return case
