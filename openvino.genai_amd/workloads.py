"""Shapes and step metadata of the benchmark workloads (synthetic; no tensor contents here).

Each spec is the integer side of one PagedAttention call: per-sequence past lengths and new-token counts, a block
table drawn as a random permutation prefix over a 2x oversized pool, and the op's constants.  Seeds follow
``numpy.random.Generator(PCG64(1000 + config index))``.
"""
import numpy as np

CONFIGS = {
    # TinyLlama-1.1B-shape decode, fp16 KV
    1: dict(name="tinyllama_decode_f16", Hq=32, Hkv=4, D=64, bs=32, q_dtype="f16", kv_dtype="f16", B=16,
            past=("uniform", 64, 2048), new=1, sliding_window=0),
    # Llama-3-8B-shape decode, u8 KV, batch 64 x 4096 context: the headline workload
    2: dict(name="llama3_8b_decode_u8_b64_ctx4096", Hq=32, Hkv=8, D=128, bs=32, q_dtype="f16", kv_dtype="u8", B=64,
            past=("const", 4096), new=1, sliding_window=0),
    # Qwen2.5-7B-shape mixed chunked prefill + decode, bf16
    3: dict(name="qwen25_7b_mixed_bf16", Hq=28, Hkv=4, D=128, bs=32, q_dtype="bf16", kv_dtype="bf16", B=64,
            past=("mixed", [0, 2048, 4096, 8192], 60, 512, 8192), new=("mixed", 512, 1), sliding_window=0),
    # cache-eviction scoring, Llama-3-8B shape, batch 256 x 8192
    4: dict(name="llama3_8b_eviction_u8_b256_ctx8192", Hq=32, Hkv=8, D=128, bs=32, q_dtype="f16", kv_dtype="u8",
            B=256, past=("const", 8192), new=1, sliding_window=0),
    # long-context decode, 32B-class shape, batch 8 x 32768 (variant: sliding window 4096)
    5: dict(name="long_context_decode_u8_b8_ctx32768", Hq=40, Hkv=8, D=128, bs=32, q_dtype="f16", kv_dtype="u8", B=8,
            past=("const", 32768), new=1, sliding_window=0),
    # diagnostics beyond the five benchmark workloads: the headline step at the other head sizes the tuned kernels
    # are instantiated for (Phi-3-mini-like: 32 heads without grouping, head size 96; Gemma-2-9B-like: 16 / 8, 256)
    6: dict(name="phi3_mini_decode_u8_b64_ctx4096", Hq=32, Hkv=32, D=96, bs=32, q_dtype="f16", kv_dtype="u8", B=64,
            past=("const", 4096), new=1, sliding_window=0),
    7: dict(name="gemma2_9b_decode_u8_b64_ctx4096", Hq=16, Hkv=8, D=256, bs=32, q_dtype="f16", kv_dtype="u8", B=64,
            past=("const", 4096), new=1, sliding_window=0),
    # ... and larger prefill steps than the mixed workload's four 512-token chunks (Qwen2.5-7B shape, bf16): one
    # 2048-token chunk behind 30000 cached tokens, and an 8192-token prompt from scratch
    8: dict(name="qwen25_7b_prefill_bf16_2048_behind_30000", Hq=28, Hkv=4, D=128, bs=32, q_dtype="bf16", kv_dtype="bf16",
            B=1, past=("mixed", [30000], 0, 1, 1), new=("mixed", 2048, 1), sliding_window=0),
    9: dict(name="qwen25_7b_prefill_bf16_8192_from_scratch", Hq=28, Hkv=4, D=128, bs=32, q_dtype="bf16", kv_dtype="bf16",
            B=1, past=("mixed", [0], 0, 1, 1), new=("mixed", 8192, 1), sliding_window=0),
}


def make_spec(cfg, seed=None, batch=None, context_scale=1.0, sliding_window=None, pool_factor=2.0, block_size=None,
              new_tokens=None):
    """Step metadata of config ``cfg`` (1..9); ``batch`` / ``context_scale`` shrink it for parity tests;
    ``new_tokens``: every sequence of a decode workload schedules that many tokens instead of one (the shape of a
    speculative-decoding validation step)."""
    c = dict(CONFIGS[cfg])
    rng = np.random.Generator(np.random.PCG64(1000 + cfg if seed is None else seed))
    B = c["B"] if batch is None else batch
    kind = c["past"][0]
    sc = lambda v: max(0, int(round(v * context_scale)))
    if kind == "const":
        past = np.full(B, sc(c["past"][1]), np.int64)
        new = np.full(B, c["new"] if new_tokens is None else new_tokens, np.int64)
    elif kind == "uniform":
        past = rng.integers(sc(c["past"][1]), sc(c["past"][2]) + 1, size=B)
        new = np.full(B, c["new"] if new_tokens is None else new_tokens, np.int64)
    else:  # mixed: prefill chunks first, then decode sequences
        _, chunk_pasts, n_dec, lo, hi = c["past"]
        _, chunk_len, _ = c["new"]
        n_dec = n_dec if batch is None else max(0, batch - len(chunk_pasts))
        past = np.concatenate([[sc(p) for p in chunk_pasts], rng.integers(sc(lo), sc(hi) + 1, size=n_dec)])
        new = np.concatenate([np.full(len(chunk_pasts), max(1, sc(chunk_len))), np.ones(n_dec, np.int64)])
        B = len(past)
    bs = c["bs"] if block_size is None else int(block_size)
    nblk = (past + new + bs - 1) // bs
    bib = np.concatenate([[0], np.cumsum(nblk)])
    pool = int(np.ceil(pool_factor * bib[-1]))
    table = rng.permutation(pool)[:bib[-1]]
    return dict(
        name=c["name"], cfg=cfg, B=int(B), Hq=c["Hq"], Hkv=c["Hkv"], D=c["D"], bs=bs, q_dtype=c["q_dtype"],
        kv_dtype=c["kv_dtype"], past_lens=past.astype(np.int32),
        subsequence_begins=np.concatenate([[0], np.cumsum(new)]).astype(np.int32),
        block_indices_begins=bib.astype(np.int32), block_indices=table.astype(np.int32), num_blocks=pool,
        max_context_len=int((past + new).max()), scale=float(1.0 / np.sqrt(c["D"])),
        sliding_window=c["sliding_window"] if sliding_window is None else sliding_window,
        score_aggregation_window=None)


def algorithmic_bytes(spec, with_scores=True):
    """HBM bytes one attention call must move: every visible K and V row once, Q in, output out, the int32 step
    arrays and block ids, and the f32 scores."""
    past = spec["past_lens"].astype(np.int64)
    new = np.diff(spec["subsequence_begins"]).astype(np.int64)
    kv = past + new
    if spec["sliding_window"] > 0:
        kv = np.minimum(kv, spec["sliding_window"])
    D = spec["D"]
    rb = D + 8 if spec["kv_dtype"] == "u8" else 2 * D
    T = int(new.sum())
    # rows read: every query row of a chunk re-reads nothing extra at the HBM level (a chunk reads its rows once)
    kv_bytes = int(kv.sum()) * spec["Hkv"] * 2 * rb
    q_out = 2 * T * spec["Hq"] * D * 2
    ints = 4 * len(spec["block_indices"]) + 4 * (3 * spec["B"] + 2)
    scores = 4 * int((past + new).sum()) if with_scores else 0
    return dict(kv=kv_bytes, q_out=q_out, ints=ints, scores=scores, total=kv_bytes + q_out + ints + scores)


def attention_flops(spec, multi_token_only=False):
    """Matrix flops of one attention call: 4 * D per (query row, visible position), all query heads
    (multi_token_only: of the sequences that schedule more than one token)."""
    past = spec["past_lens"].astype(np.int64)
    new = np.diff(spec["subsequence_begins"]).astype(np.int64)
    pairs = 0
    for p, n in zip(past, new):
        if multi_token_only and n <= 1:
            continue
        last = p + np.arange(n, dtype=np.int64)  # last visible position of each new token
        vis = last + 1
        if spec["sliding_window"] > 0:
            vis = np.minimum(vis, spec["sliding_window"])
        pairs += int(vis.sum())
    return 4 * spec["Hq"] * spec["D"] * pairs
