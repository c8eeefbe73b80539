"""Pins the pack / unpack / grad-sum oracle (oracle/fa2a.py).

The reference holds no golden data for these kernels: its tests compare the CUDA kernels
with pure-torch simulators on random tensors (tests/test_fa2a_metadata.py:8-59,
tests/all_to_all/test_grad_sum_kernel.py:84-98).  The oracle is therefore pinned by a
hand-computed known answer, by the invariants the reference's own tests rely on, and by an
independent bit-level model of the bf16 / fp16 rounding."""
import numpy as np
import torch

from oracle import fa2a


def test_known_answer_non_cp():
    """3 shards of a 5-token tensor, 16-byte tokens, written out by hand from the kernel's
    rule buffer[offset_s + (t - start_s)*token_bytes] = tensor[t] (memcpy.cu:55-67)."""
    t = np.arange(5 * 16, dtype=np.uint8).reshape(5, 16)         # token i = bytes 16i .. 16i+15
    lens, offs = [2, 0, 3], [48, 0, 0]                           # shard 0 -> bytes 48.., shard 2 -> bytes 0..
    buf = np.full(96, 0xEE, dtype=np.uint8)
    fa2a.copy_non_cp(t, buf, offs, lens, None, True)
    expected = np.concatenate([np.arange(32, 80), np.arange(0, 32), np.full(16, 0xEE)]).astype(np.uint8)
    assert np.array_equal(buf, expected)
    back = np.zeros_like(t)
    fa2a.copy_non_cp(back, buf, offs, lens, None, False)
    assert np.array_equal(back, t)


def test_known_answer_cp():
    """One 3-token tensor, shards [1, 2], two replicas; replica 1 carries only shard 1
    (do_shard[s, c], offsets[c, s]: memcpy.cu:120-121)."""
    t = np.arange(3 * 16, dtype=np.uint8).reshape(3, 16)
    do_shard = np.array([[1, 0], [1, 1]], dtype=np.int8)
    offs = np.array([[32, 0], [999, 48]], dtype=np.int64)        # (replica 1, shard 0) unused
    buf = np.full(80, 0xEE, dtype=np.uint8)
    fa2a.copy_cp(t, buf, do_shard, offs, [1, 2], True)
    expected = np.concatenate([np.arange(16, 48), np.arange(0, 16), np.arange(16, 48)]).astype(np.uint8)
    assert np.array_equal(buf, expected)
    planes = np.zeros((2, 3, 16), dtype=np.uint8)
    fa2a.copy_cp(planes, buf, do_shard, offs, [1, 2], False)
    assert np.array_equal(planes[0], t)
    assert np.array_equal(planes[1, 1:], t[1:]) and not planes[1, 0].any()


def _case(seed, nshard=11, tb=32, empty=True):
    rng = np.random.default_rng(seed)
    lens = rng.integers(0 if empty else 1, 9, size=nshard).astype(np.int64)
    T = int(lens.sum())
    perm = rng.permutation(nshard)
    off = np.zeros(nshard, dtype=np.int64)
    cur = 0
    for s in perm:
        off[s] = cur
        cur += int(lens[s]) * tb + 16 * int(rng.integers(0, 3))
    t = rng.integers(0, 256, size=(T, tb), dtype=np.uint8)
    return rng, lens, off, cur, t


def test_slice_form_equals_token_loop_and_round_trip():
    for seed in range(5):
        rng, lens, off, nbuf, t = _case(seed)
        mask = (rng.random(len(lens)) < 0.5).astype(np.int8)
        for m in (None, mask):
            a = np.full(nbuf, 7, np.uint8); b = a.copy()
            fa2a.copy_non_cp(t, a, off, lens, m, True)
            fa2a.copy_non_cp_tokenwise(t, b, off, lens, m, True)
            assert np.array_equal(a, b)
        back = np.zeros_like(t)
        full = np.zeros(nbuf, np.uint8)
        fa2a.copy_non_cp(t, full, off, lens, None, True)
        fa2a.copy_non_cp(back, full, off, lens, None, False)
        assert np.array_equal(back, t)                         # pack then unpack = identity
        back2 = np.zeros_like(t)
        fa2a.copy_non_cp_tokenwise(back2, full, off, lens, None, False)
        assert np.array_equal(back2, t)


def test_masked_shards_leave_buffer_untouched_and_mask_ignored_on_unpack():
    rng, lens, off, nbuf, t = _case(9, empty=False)
    mask = np.zeros(len(lens), np.int8); mask[::2] = 1
    buf = np.full(nbuf, 0x5A, np.uint8)
    fa2a.copy_non_cp(t, buf, off, lens, mask, True)
    start = 0
    for s, ln in enumerate(lens):
        region = buf[off[s]:off[s] + ln * t.shape[1]]
        if mask[s]:
            assert np.array_equal(region, t[start:start + ln].reshape(-1))
        else:
            assert (region == 0x5A).all()
        start += ln
    # the reference launches the unmasked kernel whenever it unpacks (memcpy.cu:272-278)
    full = np.zeros(nbuf, np.uint8)
    fa2a.copy_non_cp(t, full, off, lens, None, True)
    back = np.zeros_like(t)
    fa2a.copy_non_cp(back, full, off, lens, mask, False)
    assert np.array_equal(back, t)


def test_rows_beyond_tensor_are_never_touched():
    t = np.arange(4 * 16, dtype=np.uint8).reshape(4, 16)
    buf = np.zeros(16 * 8, np.uint8)
    fa2a.copy_non_cp(t, buf, [0, 64], [3, 5], None, True)       # shard 1 claims 5 tokens, only 1 exists
    assert np.array_equal(buf[:48], t[:3].reshape(-1)) and np.array_equal(buf[64:80], t[3]) and not buf[80:].any()


def test_cp_unpack_of_pack_summed_over_planes_is_source_times_replicas():
    """tests/test_shard_info_to_fa2a.py:212-227 relies on this for the K/V gradient path."""
    rng = np.random.default_rng(3)
    nshard, max_cp, tb = 6, 3, 32
    lens = rng.integers(1, 7, size=nshard).astype(np.int64)
    T = int(lens.sum())
    do_shard = (rng.random((nshard, max_cp)) < 0.6).astype(np.int8)
    off = np.zeros((max_cp, nshard), np.int64); cur = 0
    for c in range(max_cp):
        for s in rng.permutation(nshard):
            off[c, s] = cur; cur += int(lens[s]) * tb
    src = rng.integers(1, 50, size=(T, tb // 4)).astype(np.float32)
    buf = np.zeros(cur, np.uint8)
    fa2a.copy_cp(src, buf, do_shard, off, lens, True)
    planes = np.zeros((max_cp, T, tb // 4), np.float32)
    fa2a.copy_cp(planes, buf, do_shard, off, lens, False)
    reps = np.repeat(do_shard.sum(1), lens)[:, None]
    assert np.array_equal(planes.sum(0), src * reps)


def _round_bf16(x32: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (as fp32 values), round to nearest even, by integer arithmetic."""
    u = x32.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32)


def test_grad_sum_rounds_once_per_copy_in_copy_order():
    g = torch.Generator().manual_seed(1)
    lens = [3, 2, 3, 3]                                          # shard 0 main with copies at shards 2, 3
    data = (torch.randn((11, 8), generator=g) * 100).to(torch.bfloat16)
    num_copies = [2, 0, 0, 0]
    starts = [[5, 8], [0, 0], [0, 0], [0, 0]]
    got = data.clone()
    fa2a.grad_sum(got, num_copies, starts, lens)
    x = data.float().numpy()
    step1 = _round_bf16(x[0:3] + x[5:8])
    step2 = _round_bf16(step1 + x[8:11])
    assert np.array_equal(got[0:3].float().numpy(), step2)
    assert torch.equal(got[3:], data[3:])                        # copies and plain shards untouched
    # a single rounding of the exact sum differs somewhere: the per-copy rounding is observable
    assert not np.array_equal(_round_bf16(x[0:3] + x[5:8] + x[8:11]), step2)


def test_grad_sum_fp32_and_no_copies():
    data = torch.arange(24, dtype=torch.float32).reshape(6, 4)
    same = data.clone()
    fa2a.grad_sum(same, [0, 0], [[0], [0]], [2, 4])
    assert torch.equal(same, data)
    got = data.clone()
    fa2a.grad_sum(got, [1, 0, 0], [[4], [0], [0]], [2, 2, 2])
    assert torch.equal(got[0:2], data[0:2] + data[4:6]) and torch.equal(got[2:], data[2:])
