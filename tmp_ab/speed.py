"""Speed of shapes that run on the shape-generic kernels: Phi-3-mini-like (32 heads, MHA, D = 96) and Gemma-like (D = 256, G = 2)."""
import sys, os
import numpy as np
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import torch
import __graft_entry__ as entry
pkg = entry.load_package()
dev = torch.device("cuda:0")
def run(name, Hq, Hkv, D, kd, past, new):
    bs = 32
    qd = "f16"
    op = pkg.PagedAttention(Hq, Hkv, D, bs, qd, kd, 1, 0, torch.cuda.current_stream(dev))
    past, new = np.asarray(past, np.int32), np.asarray(new, np.int32)
    B = len(past)
    sb = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    nblk = (past + new + bs - 1) // bs
    bib = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
    pool = int(bib[-1]) + 1
    table = np.random.default_rng(0).permutation(pool)[:bib[-1]].astype(np.int32)
    rb = pkg.row_bytes(D, kd)
    kc = torch.zeros(pool, Hkv, bs, rb, dtype=torch.uint8, device=dev)
    if kd == "u8":
        kc.view(torch.float32).view(pool, Hkv, bs, rb // 4)[..., 0] = 0.01
        kc.view(torch.float32).view(pool, Hkv, bs, rb // 4)[..., 1] = 128.0
    vc = kc.clone()
    T = int(sb[-1])
    q = torch.randn(T, Hq * D, device=dev).to(torch.float16)
    k = torch.randn(T, Hkv * D, device=dev).to(torch.float16)
    out = torch.zeros_like(q)
    op.step_begin(past, sb, bib, int((past + new).max()))
    op.set_block_indices(table, pool)
    scores = torch.zeros(op.total_scores, dtype=torch.float32, device=dev)
    for _ in range(2):
        op.forward(q, k, k, kc, vc, out, scores)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    n = 5
    for _ in range(n):
        op.forward(q, k, k, kc, vc, out, scores)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / n
    kv_bytes = float(((past + new).astype(np.int64)).sum()) * Hkv * 2 * rb
    pairs = float(sum(int(n) * int(p) + int(n) * (int(n) + 1) // 2 for p, n in zip(past, new)))
    fl = 4.0 * Hq * D * pairs
    print(f"{name}: {ms*1e3:.0f} us per step; {fl/1e9:.1f} GFLOP -> {fl/ms/1e9:.0f} TFLOP/s; KV once {kv_bytes/1e6:.0f} MB", flush=True)

for kd in ("f16", "u8"):
    run(f"1 x 8192 from scratch, 28/4 D128 {kd}", 28, 4, 128, kd, [0], [8192])
    run(f"1 x 2048 behind 30000, 28/4 D128 {kd}", 28, 4, 128, kd, [30000], [2048])
    run(f"8 x 1024 from scratch, 32/8 D128 {kd}", 32, 8, 128, kd, [0] * 8, [1024] * 8)
    run(f"1 x 512 behind 8192, 32/8 D128 {kd}", 32, 8, 128, kd, [8192], [512])
    run(f"32 x 128 behind 1000, 32/8 D128 {kd}", 32, 8, 128, kd, [1000] * 32, [128] * 32)
    run(f"1 x 16384 from scratch, 32/8 D128 {kd}", 32, 8, 128, kd, [0], [16384])
