"""What KVCacheManager accepts beyond the tuned shapes -- head sizes other than 64 / 128, a value head size and a value
precision of their own, u4 rows, a 16-bit cache of the other 16-bit type -- through the C-ABI against the CPU checker:
cache rows bit-exact, outputs and scores within tolerance."""
import numpy as np
import pytest

import harness as H
from oracle import oracle as O

pytestmark = pytest.mark.gpu

MIXES = [
    # (query type, Dk, Dv, key cache type, value cache type, block size, Hq, Hkv)
    ("f16", 80, 80, "f16", "f16", 32, 8, 2), ("bf16", 96, 96, "u8", "u8", 16, 6, 2), ("f16", 256, 256, "u8", "u8", 32, 4, 4),
    ("bf16", 256, 256, "bf16", "bf16", 32, 4, 1), ("f16", 128, 64, "u8", "f16", 32, 8, 2), ("bf16", 64, 128, "bf16", "u8", 32, 8, 2),
    ("f16", 192, 128, "f16", "u4", 32, 6, 3), ("bf16", 128, 128, "u4", "u4", 32, 8, 2), ("f16", 72, 40, "u4", "bf16", 24, 4, 2),
    ("f16", 128, 128, "bf16", "bf16", 32, 8, 2), ("f16", 512, 8, "u8", "u8", 32, 2, 1),
    # head size 96 (K and V alike, a u8 cache or one of the query's type): the matrix kernel's one-row-group variants
    ("f16", 96, 96, "f16", "f16", 32, 8, 8), ("bf16", 96, 96, "bf16", "bf16", 32, 6, 2), ("f16", 96, 96, "u8", "u8", 32, 12, 4),
    ("bf16", 96, 96, "u8", "u8", 64, 4, 1),
]


def _case(rng, qd, Dk, Dv, kd, vd, bs, Hq, Hkv, past, new):
    qdt, kdt, vdt = H.DT[qd], O.DT_U4 if kd == "u4" else H.DT[kd], O.DT_U4 if vd == "u4" else H.DT[vd]
    past, new = np.asarray(past, np.int32), np.asarray(new, np.int32)
    B = len(past)
    sb = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    nblk = (past + new + bs - 1) // bs
    bib = np.concatenate([[0], np.cumsum(nblk)]).astype(np.int32)
    pool = 2 * int(bib[-1]) + 1
    table = rng.permutation(pool)[:bib[-1]].astype(np.int32)
    kc = np.zeros((pool, Hkv, bs, O.row_bytes(Dk, kdt)), np.uint8)
    vc = np.zeros((pool, Hkv, bs, O.row_bytes(Dv, vdt)), np.uint8)

    def synth(n, w):
        x = rng.standard_normal((n, w)).astype(np.float32)
        m = rng.random(x.shape) < 0.01
        x[m] = np.where(rng.random(int(m.sum())) < 0.5, 8.0, -8.0)
        return O.to_bits(x, qdt)

    if past.sum() > 0:
        psb = np.concatenate([[0], np.cumsum(past)]).astype(np.int32)
        O.kv_append_kv(synth(int(psb[-1]), Hkv * Dk), synth(int(psb[-1]), Hkv * Dv), qdt, kc, vc, kdt, vdt,
                       np.zeros(B, np.int32), psb, table, bib, Hkv, Dk, Dv, bs)
    T = int(sb[-1])
    return dict(qdt=qdt, kdt=kdt, vdt=vdt, past=past, new=new, sb=sb, bib=bib, table=table, pool=pool, kc=kc, vc=vc,
                q=synth(T, Hq * Dk), k=synth(T, Hkv * Dk), v=synth(T, Hkv * Dv))


@pytest.mark.parametrize("qd,Dk,Dv,kd,vd,bs,Hq,Hkv", MIXES)
@pytest.mark.parametrize("kind", ["mixed", "decode"])
def test_shapes_beyond_the_tuned_ones(pkg, qd, Dk, Dv, kd, vd, bs, Hq, Hkv, kind):
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(Dk * 131 + Dv + bs)
    past, new = ([0, 45, 700, 9], [37, 1, 1, 70]) if kind == "mixed" else ([300, 5, 1500], [1, 1, 1])
    print(f"case generic {qd} Dk{Dk} Dv{Dv} {kd}/{vd} bs{bs} {kind}", flush=True)
    c = _case(rng, qd, Dk, Dv, kd, vd, bs, Hq, Hkv, past, new)
    W = np.minimum(c["new"], 2).astype(np.int32)
    sw = 0 if kind == "mixed" else 600
    scale = float(1.0 / np.sqrt(Dk))
    # the checker
    kc_ref, vc_ref = c["kc"].copy(), c["vc"].copy()
    O.kv_append_kv(c["k"], c["v"], c["qdt"], kc_ref, vc_ref, c["kdt"], c["vdt"], c["past"], c["sb"], c["table"], c["bib"],
                   Hkv, Dk, Dv, bs)
    ref_out, _, ref_sc = O.paged_attention_kv(c["q"], c["qdt"], kc_ref, vc_ref, c["kdt"], c["vdt"], c["past"], c["sb"],
                                              c["table"], c["bib"], Hq, Hkv, Dk, Dv, bs, scale, sw, W, True, 8)
    # the library
    op = pkg.PagedAttention(Hq, Hkv, Dk, bs, qd, kd, 1, 0, torch.cuda.current_stream(dev), v_head_size=Dv,
                            value_cache_dtype=vd)
    q, k, v = (H.to_device_16(torch, c[n], qd, dev) for n in ("q", "k", "v"))
    kc, vc = torch.from_numpy(c["kc"]).to(dev), torch.from_numpy(c["vc"]).to(dev)
    out = torch.zeros(q.shape[0], Hq * Dv, dtype=q.dtype, device=dev)
    op.step_begin(c["past"], c["sb"], c["bib"], int((c["past"] + c["new"]).max()), W, sw, scale)
    op.set_block_indices(c["table"], c["pool"])
    scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
    op.forward(q, k, v, kc, vc, out, scores)
    op.synchronize()
    assert np.array_equal(kc.cpu().numpy(), kc_ref), "key cache bytes differ"
    assert np.array_equal(vc.cpu().numpy(), vc_ref), "value cache bytes differ"
    H.assert_close(out.float().cpu().numpy(), ref_out, qd)
    H.assert_close(scores.cpu().numpy(), ref_sc, "f16", "scores")


def test_refused_configurations(pkg):
    for kw in (dict(head_size=100), dict(head_size=520), dict(head_size=128, v_head_size=12), dict(head_size=0)):
        hs = kw.pop("head_size")
        with pytest.raises(pkg.PaError):
            pkg.PagedAttention(8, 2, hs, 32, "f16", "u8", **kw)


ALIBI = [
    # (query type, Dk, Dv, key cache type, value cache type, block size, Hq, Hkv): tuned shapes (which a context with
    # slopes leaves for the shape-generic kernels) and others
    ("f16", 128, 128, "u8", "u8", 32, 8, 2), ("bf16", 128, 128, "bf16", "bf16", 32, 28, 4), ("f16", 64, 64, "f16", "f16", 16, 4, 4),
    ("bf16", 96, 96, "u8", "u8", 32, 6, 2), ("f16", 128, 64, "u4", "f16", 32, 8, 1),
]


@pytest.mark.parametrize("qd,Dk,Dv,kd,vd,bs,Hq,Hkv", ALIBI)
@pytest.mark.parametrize("kind", ["mixed", "decode"])
def test_alibi_slopes(pkg, qd, Dk, Dv, kd, vd, bs, Hq, Hkv, kind):
    """The op's alibi_slopes input: outputs and scores against the checker's form with slopes; with all-zero slopes
    and after taking the slopes away again the context is back on its own kernels with their results."""
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(Dk * 17 + Hq)
    past, new = ([0, 45, 700, 9], [37, 1, 1, 70]) if kind == "mixed" else ([300, 5, 1500], [1, 1, 1])
    print(f"case alibi {qd} Dk{Dk} Dv{Dv} {kd}/{vd} bs{bs} {kind}", flush=True)
    c = _case(rng, qd, Dk, Dv, kd, vd, bs, Hq, Hkv, past, new)
    W = np.minimum(c["new"], 2).astype(np.int32)
    sw = 0 if kind == "mixed" else 600
    scale = float(1.0 / np.sqrt(Dk))
    # slopes of the paper's geometric kind, one head without a slope
    slopes = (2.0 ** -(8.0 * (np.arange(Hq) + 1) / Hq)).astype(np.float32)
    slopes[Hq // 2] = 0.0
    kc_ref, vc_ref = c["kc"].copy(), c["vc"].copy()
    O.kv_append_kv(c["k"], c["v"], c["qdt"], kc_ref, vc_ref, c["kdt"], c["vdt"], c["past"], c["sb"], c["table"], c["bib"],
                   Hkv, Dk, Dv, bs)
    ref_out, _, ref_sc = O.paged_attention_alibi(c["q"], c["qdt"], kc_ref, vc_ref, c["kdt"], c["vdt"], c["past"], c["sb"],
                                                 c["table"], c["bib"], Hq, Hkv, Dk, Dv, bs, scale, slopes, sw, W, True, 8)
    plain_out, _, plain_sc = O.paged_attention_kv(c["q"], c["qdt"], kc_ref, vc_ref, c["kdt"], c["vdt"], c["past"], c["sb"],
                                                  c["table"], c["bib"], Hq, Hkv, Dk, Dv, bs, scale, sw, W, True, 8)
    assert np.abs(ref_out - plain_out).max() > 1e-2   # (the slopes matter on this data)
    op = pkg.PagedAttention(Hq, Hkv, Dk, bs, qd, kd, 1, 0, torch.cuda.current_stream(dev), v_head_size=Dv,
                            value_cache_dtype=vd)
    q, k, v = (H.to_device_16(torch, c[n], qd, dev) for n in ("q", "k", "v"))

    def run(want):
        kc, vc = torch.from_numpy(c["kc"]).to(dev), torch.from_numpy(c["vc"]).to(dev)
        out = torch.zeros(q.shape[0], Hq * Dv, dtype=q.dtype, device=dev)
        op.step_begin(c["past"], c["sb"], c["bib"], int((c["past"] + c["new"]).max()), W, sw, scale)
        op.set_block_indices(c["table"], c["pool"])
        scores = torch.full((op.total_scores,), float("nan"), dtype=torch.float32, device=dev)
        op.forward(q, k, v, kc, vc, out, scores)
        op.synchronize()
        assert np.array_equal(kc.cpu().numpy(), kc_ref) and np.array_equal(vc.cpu().numpy(), vc_ref), "cache bytes differ"
        H.assert_close(out.float().cpu().numpy(), want[0], qd)
        H.assert_close(scores.cpu().numpy(), want[1], "f16", "scores")
        return out.view(torch.int16).cpu().numpy(), scores.cpu().numpy()

    before = run((plain_out, plain_sc))
    op.set_alibi_slopes(slopes)
    with pytest.raises(pkg.PaError):   # the step's plan is void after the change: it has to begin again
        op.attention(q, torch.from_numpy(c["kc"]).to(dev), torch.from_numpy(c["vc"]).to(dev),
                     torch.zeros(q.shape[0], Hq * Dv, dtype=q.dtype, device=dev))
    run((ref_out, ref_sc))
    op.set_alibi_slopes(np.zeros(Hq, np.float32))
    after = run((plain_out, plain_sc))
    assert np.array_equal(before[0], after[0]) and np.array_equal(before[1], after[1])
    op.set_alibi_slopes(slopes)
    run((ref_out, ref_sc))
    op.set_alibi_slopes(None)
    after = run((plain_out, plain_sc))
    assert np.array_equal(before[0], after[0])
    with pytest.raises(pkg.PaError):   # one slope per query head
        op.set_alibi_slopes(slopes[:-1])
