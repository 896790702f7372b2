"""KV cache tensors on the device (pa_kv_cache_*), after the reference's tests/cpp/cache_manager.cpp:28-108 --
cache_size / num_kv_blocks -> allocated bytes, dynamic growth -- plus what those tests take for granted: growth keeps
the blocks' contents (kv_cache_manager.hpp:215-240), copy_blocks copies every layer's K and V block
(kv_cache_manager.hpp:278-335), and the tensors work as `key_cache.<L>` / `value_cache.<L>` of the op."""
import ctypes as C

import numpy as np
import pytest

import harness as H
from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    assert torch.cuda.is_available()
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    return pkg, torch.device("cuda:0"), hip


class _Dev:
    """A raw device pointer where the op wrapper expects a tensor."""

    def __init__(self, ptr, num_blocks):
        self._p = ptr
        self.shape = (num_blocks,)

    def data_ptr(self):
        return self._p


def _read(hip, ptr, nbytes):
    out = np.zeros(nbytes, np.uint8)
    assert hip.hipMemcpy(out.ctypes.data, C.c_void_p(ptr), nbytes, 2) == 0  # device to host
    return out


def _write(hip, ptr, arr):
    a = np.ascontiguousarray(arr)
    assert hip.hipMemcpy(C.c_void_p(ptr), a.ctypes.data, a.nbytes, 1) == 0  # host to device


def test_cache_size_param(env):
    """TestCacheManager.test_cache_size_param: cache_size (GiB) -> blocks -> allocated bytes."""
    pkg, _, _ = env
    layers = 12
    mgr = pkg.KVCacheManager(layers, 2, 64, 32, "u8")
    assert mgr.get_num_layers() == layers and mgr.get_block_size() == 32
    bb = mgr.get_block_size_in_bytes()
    assert bb == 2 * layers * 2 * 32 * (64 + 8)
    cache_size = 1
    blocks = pkg.normalize_num_kv_blocks(0, cache_size, 32, bb, 200 << 30)
    mgr.allocate_cache_if_needed(blocks)
    allocated = mgr.get_num_allocated_kv_blocks() * bb
    assert allocated == (cache_size << 30) // bb * bb
    for l in range(layers):
        assert mgr.get_key_cache(l) and mgr.get_value_cache(l) and mgr.get_key_cache(l) != mgr.get_value_cache(l)


def test_kv_blocks_param_and_dynamic_cache_increase(env):
    """TestCacheManager.test_kv_blocks_param / test_dynamic_cache_increase, and the contents survive the growth."""
    pkg, _, hip = env
    layers = 3
    mgr = pkg.KVCacheManager(layers, 2, 128, 32, "f16")
    bb = mgr.get_block_size_in_bytes()
    per_layer = bb // (2 * layers)
    assert pkg.normalize_num_kv_blocks(150, 0, 32, bb, 200 << 30) == 150
    assert mgr.get_num_allocated_kv_blocks() == 0
    mgr.allocate_cache_if_needed(100)
    assert mgr.get_num_allocated_kv_blocks() * bb == 100 * bb
    rng = np.random.default_rng(1)
    want = {}
    for l in range(layers):
        for which, ptr in (("k", mgr.get_key_cache(l)), ("v", mgr.get_value_cache(l))):
            want[l, which] = rng.integers(0, 256, 100 * per_layer, dtype=np.uint8)
            _write(hip, ptr, want[l, which])
    mgr.allocate_cache_if_needed(200)
    assert mgr.get_num_allocated_kv_blocks() == 200
    for l in range(layers):
        for which, ptr in (("k", mgr.get_key_cache(l)), ("v", mgr.get_value_cache(l))):
            assert np.array_equal(_read(hip, ptr, 100 * per_layer), want[l, which]), (l, which)
    before = [mgr.get_key_cache(l) for l in range(layers)]
    mgr.allocate_cache_if_needed(200)   # nothing new: nothing moves
    mgr.allocate_cache_if_needed(50)    # never shrinks
    assert mgr.get_num_allocated_kv_blocks() == 200
    assert [mgr.get_key_cache(l) for l in range(layers)] == before


def test_copy_blocks_and_use_as_op_tensors(env):
    """Copy-on-write: after copy_blocks a table that points at the copies attends exactly like the original."""
    import torch
    pkg, dev, hip = env
    Hq, Hkv, D, bs, layers = 8, 2, 128, 32, 2
    case = H.build_case(H.case_from_lens("cow", Hq, Hkv, D, bs, "f16", "u8", [70, 33], [1, 1]), 3)
    nb = case["num_blocks"]
    mgr = pkg.KVCacheManager(layers, Hkv, D, bs, "u8")
    mgr.allocate_cache_if_needed(nb)
    for l in range(layers):
        _write(hip, mgr.get_key_cache(l), case["key_cache0"])
        _write(hip, mgr.get_value_cache(l), case["value_cache0"])
    op = pkg.PagedAttention(Hq, Hkv, D, bs, "f16", "u8", num_layers=layers, device=0, stream=torch.cuda.current_stream(dev))
    q, k, v = (H.to_device_16(torch, case[x], "f16", dev) for x in ("query", "key", "value"))

    def run(table, num_blocks):
        outs = []
        op.step_begin(case["past_lens"], case["subsequence_begins"], case["block_indices_begins"])
        op.set_block_indices(table, num_blocks)
        for l in range(layers):
            out = torch.zeros_like(q)
            sc = torch.zeros(op.total_scores, dtype=torch.float32, device=dev)
            op.forward(q, k, v, _Dev(mgr.get_key_cache(l), num_blocks), _Dev(mgr.get_value_cache(l), num_blocks), out, sc, layer=l)
            op.synchronize()
            outs.append((out.cpu().numpy().view(np.uint16).copy(), sc.cpu().numpy().copy()))
        return outs

    first = run(case["block_indices"], nb)
    ref = H.run_case_on_checker(case)
    for out16, sc in first:
        H.assert_close(O.from_bits(out16, O.DT_F16), ref["out"], "f16")
        H.assert_close(sc, ref["scores"], "f16", "scores")
    # grow, then give every block of the table a copy among the new blocks
    mgr.allocate_cache_if_needed(2 * nb)
    copies = {int(src): [nb + i] for i, src in enumerate(case["block_indices"])}
    mgr.copy_blocks(copies)
    moved = np.array([copies[int(b)][0] for b in case["block_indices"]], np.int32)
    second = run(moved, 2 * nb)   # (appends the same new rows again, into the copies)
    for (o1, s1), (o2, s2) in zip(first, second):
        assert np.array_equal(o1, o2) and np.array_equal(s1, s2)
    with pytest.raises(pkg.PaError):
        mgr.copy_blocks({0: [2 * nb]})  # outside the cache


def test_growth_moves_nothing_and_new_blocks_are_zero(env):
    """Growth maps memory behind what is there: base addresses stay, old blocks stay in place, new ones read as 0."""
    pkg, _, hip = env
    layers = 2
    mgr = pkg.KVCacheManager(layers, 4, 128, 32, "u8")
    per_layer = mgr.get_block_size_in_bytes() // (2 * layers)
    mgr.allocate_cache_if_needed(7)
    ptrs = [(mgr.get_key_cache(l), mgr.get_value_cache(l)) for l in range(layers)]
    rng = np.random.default_rng(5)
    want = {}
    for l in range(layers):
        for w in range(2):
            want[l, w] = rng.integers(0, 256, 7 * per_layer, dtype=np.uint8)
            _write(hip, ptrs[l][w], want[l, w])
    for n in (8, 300, 5000):   # within the first mapping's slack, then across several mappings
        mgr.allocate_cache_if_needed(n)
        assert [(mgr.get_key_cache(l), mgr.get_value_cache(l)) for l in range(layers)] == ptrs
        for l in range(layers):
            for w in range(2):
                got = _read(hip, ptrs[l][w], n * per_layer)
                assert np.array_equal(got[:7 * per_layer], want[l, w]), (n, l, w)
                assert not got[7 * per_layer:].any(), (n, l, w)


def test_failed_growth_leaves_the_cache_as_it_was(env):
    pkg, _, hip = env
    mgr = pkg.KVCacheManager(2, 4, 128, 32, "u8")
    per_layer = mgr.get_block_size_in_bytes() // 4
    mgr.allocate_cache_if_needed(10)
    ptr = mgr.get_key_cache(1)
    data = np.arange(10 * per_layer, dtype=np.uint32).astype(np.uint8)
    _write(hip, ptr, data)
    with pytest.raises(pkg.PaError) as e:   # more than the device holds
        mgr.allocate_cache_if_needed((400 << 30) // mgr.get_block_size_in_bytes())
    assert e.value.status == -10 and "larger than available memory" in str(e.value)
    assert mgr.get_num_allocated_kv_blocks() == 10 and mgr.get_key_cache(1) == ptr
    assert np.array_equal(_read(hip, ptr, 10 * per_layer), data)
    mgr.allocate_cache_if_needed(20)        # and it still grows
    assert np.array_equal(_read(hip, ptr, 10 * per_layer), data)


def test_growth_past_half_of_the_free_memory(env):
    """From N to 2N blocks with N above a third of the free memory: a growth that copied into a new allocation could
    not hold both; here nothing is copied, addresses stay valid and the contents stay where they are."""
    import torch
    pkg, dev, hip = env
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info(dev)
    layers = 4
    mgr = pkg.KVCacheManager(layers, 8, 128, 32, "u8")
    bb = mgr.get_block_size_in_bytes()
    per_layer = bb // (2 * layers)
    n = int(0.36 * free) // bb
    mgr.allocate_cache_if_needed(n)
    ptrs = [(mgr.get_key_cache(l), mgr.get_value_cache(l)) for l in range(layers)]
    rng = np.random.default_rng(9)
    marks = {}
    for l in range(layers):
        for w in range(2):
            for blk in (0, n // 2, n - 1):
                marks[l, w, blk] = rng.integers(0, 256, per_layer, dtype=np.uint8)
                _write(hip, ptrs[l][w] + blk * per_layer, marks[l, w, blk])
    mgr.allocate_cache_if_needed(2 * n)
    assert mgr.get_num_allocated_kv_blocks() == 2 * n
    assert 2 * n * bb > 0.7 * free
    assert [(mgr.get_key_cache(l), mgr.get_value_cache(l)) for l in range(layers)] == ptrs
    for (l, w, blk), data in marks.items():
        assert np.array_equal(_read(hip, ptrs[l][w] + blk * per_layer, per_layer), data), (l, w, blk)
    last = ptrs[layers - 1][1] + (2 * n - 1) * per_layer
    assert not _read(hip, last, per_layer).any()
    _write(hip, last, marks[0, 0, 0])
    assert np.array_equal(_read(hip, last, per_layer), marks[0, 0, 0])
    del mgr
    torch.cuda.synchronize(dev)
    assert torch.cuda.mem_get_info(dev)[0] > 0.9 * free   # everything was given back


def test_copy_blocks_of_a_whole_batch_is_exact_and_ordered(env):
    """256 pairs x 32 layers in one call; then pairs that feed each other, which the reference copies one after the
    other (kv_cache_manager.hpp:278-335)."""
    import time
    pkg, _, hip = env
    layers = 32
    mgr = pkg.KVCacheManager(layers, 8, 128, 32, "u8")
    per_layer = mgr.get_block_size_in_bytes() // (2 * layers)
    nb = 600
    mgr.allocate_cache_if_needed(nb)
    rng = np.random.default_rng(3)
    content = {}
    for l in range(layers):
        for w in range(2):
            content[l, w] = rng.integers(0, 256, (nb, per_layer), dtype=np.uint8)
            _write(hip, (mgr.get_key_cache(l), mgr.get_value_cache(l))[w], content[l, w])
    src = rng.permutation(300)[:256]
    copy_map = {int(s): [300 + i] for i, s in enumerate(src)}
    t0 = time.perf_counter()
    mgr.copy_blocks(copy_map)
    dt = time.perf_counter() - t0
    print("copy_blocks: 256 blocks x 32 layers (%.0f MB read + written) in %.3f ms host time" %
          (2 * 256 * mgr.get_block_size_in_bytes() / 1e6, dt * 1e3))
    for l in (0, 13, 31):
        for w in range(2):
            got = _read(hip, (mgr.get_key_cache(l), mgr.get_value_cache(l))[w], nb * per_layer).reshape(nb, per_layer)
            want = content[l, w].copy()
            for s, ds in copy_map.items():
                want[ds[0]] = content[l, w][s]
            assert np.array_equal(got, want), (l, w)
    # 0 -> 1, then 1 -> 2: block 2 ends up with what block 0 held; one source, several destinations
    base0 = _read(hip, mgr.get_key_cache(5), 3 * per_layer).reshape(3, per_layer)
    mgr.copy_blocks({0: [1, 590, 591], 1: [2]})
    got = _read(hip, mgr.get_key_cache(5), nb * per_layer).reshape(nb, per_layer)
    for blk in (1, 2, 590, 591):
        assert np.array_equal(got[blk], base0[0]), blk


def test_shape_and_precision_per_layer_and_per_tensor(env):
    """Layers whose K and V tensors differ in kv heads, head size and precision (u4 included): block bytes add up as
    the reference adds them (kv_cache_manager.hpp:74-92), growth keeps every tensor's blocks, copy_blocks copies each
    tensor's own block size."""
    pkg, _, hip = env
    layers = [((8, 32, 128, "u8"), (8, 32, 128, "u8")), ((4, 32, 192, "bf16"), (4, 32, 128, "u4")),
              ((2, 32, 80, "f16"), (2, 32, 256, "u8")), ((8, 32, 64, "u4"), (8, 32, 64, "f16"))]
    rb = {"u8": lambda d: d + 8, "u4": lambda d: d // 2 + 8, "f16": lambda d: 2 * d, "bf16": lambda d: 2 * d}
    per = [[h * b * rb[t](d) for (h, b, d, t) in kv] for kv in layers]
    mgr = pkg.KVCacheManager(len(layers), 8, 128, 32, "u8", layers=layers)
    assert mgr.get_block_size_in_bytes() == sum(sum(p) for p in per)
    nb = 40
    mgr.allocate_cache_if_needed(nb)
    rng = np.random.default_rng(11)
    content = {}
    for l in range(len(layers)):
        for w in range(2):
            content[l, w] = rng.integers(0, 256, (nb, per[l][w]), dtype=np.uint8)
            _write(hip, (mgr.get_key_cache(l), mgr.get_value_cache(l))[w], content[l, w])
    ptrs = [(mgr.get_key_cache(l), mgr.get_value_cache(l)) for l in range(len(layers))]
    mgr.allocate_cache_if_needed(4 * nb)  # growth: same addresses, old blocks kept, new ones zero
    assert ptrs == [(mgr.get_key_cache(l), mgr.get_value_cache(l)) for l in range(len(layers))]
    mgr.copy_blocks({3: [nb + 5, 7], 9: [4 * nb - 1]})
    for l in range(len(layers)):
        for w in range(2):
            got = _read(hip, ptrs[l][w], 4 * nb * per[l][w]).reshape(4 * nb, per[l][w])
            want = np.zeros_like(got)
            want[:nb] = content[l, w]
            want[nb + 5] = want[7] = content[l, w][3]
            want[4 * nb - 1] = content[l, w][9]
            assert np.array_equal(got, want), (l, w)
    with pytest.raises(pkg.PaError):
        pkg.KVCacheManager(1, 8, 128, 32, "u8", layers=[((8, 32, 0, "u8"), (8, 32, 128, "u8"))])
