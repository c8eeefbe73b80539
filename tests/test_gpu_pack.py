"""GPU parity (bit-exact) of the shard pack / unpack / grad-sum kernels against the oracle."""
import numpy as np
import pytest
import torch

from oracle import fa2a

pytestmark = pytest.mark.gpu


def _layout(rng, lens, token_bytes, slack=64):
    perm = rng.permutation(len(lens))
    off = np.zeros(len(lens), dtype=np.int64)
    cur = 16 * int(rng.integers(0, 4))
    for s in perm:
        off[s] = cur
        cur += int(lens[s]) * token_bytes + 16 * int(rng.integers(0, slack))
    return off, cur


@pytest.mark.parametrize("hidden,dtype", [(128, torch.bfloat16), (1024, torch.bfloat16), (4096, torch.bfloat16), (24, torch.float32), (8320, torch.uint8)])
@pytest.mark.parametrize("nshard", [1, 7, 300])
def test_non_cp_pack_unpack(cuda, hidden, dtype, nshard):
    from distca_amd.ops import a2a_memcpy_non_cp
    rng = np.random.default_rng(hidden * 1000 + nshard)
    lens = rng.integers(0, 40, size=nshard).astype(np.int64)
    lens[rng.integers(0, nshard)] += 5
    T = int(lens.sum())
    esz = torch.empty((), dtype=dtype).element_size()
    tb = hidden * esz
    off, nbuf = _layout(rng, lens, tb)
    src = torch.from_numpy(rng.integers(0, 256, size=(T, tb), dtype=np.uint8)).view(dtype).reshape(T, hidden)
    mask = (rng.random(nshard) < 0.7).astype(np.int8)
    for use_mask in (False, True):
        buf0 = rng.integers(0, 256, size=nbuf, dtype=np.uint8)
        exp = buf0.copy()
        fa2a.copy_non_cp(src.view(torch.uint8).numpy().reshape(T, tb), exp, off, lens, mask if use_mask else None, True)
        dbuf = torch.from_numpy(buf0.copy()).to(cuda)
        print(f"pack hidden={hidden} {dtype} nshard={nshard} mask={use_mask}", flush=True)
        a2a_memcpy_non_cp(src.to(cuda), torch.from_numpy(off).to(cuda), torch.from_numpy(lens).to(cuda), True,
                          torch.from_numpy(mask).to(cuda) if use_mask else None, buffer=dbuf)
        torch.cuda.synchronize()
        assert np.array_equal(dbuf.cpu().numpy(), exp)
    # unpack the unmasked pack into a poisoned tensor: identity
    dst = torch.full((T, tb), 0xA5, dtype=torch.uint8, device=cuda).view(dtype).reshape(T, hidden)
    a2a_memcpy_non_cp(dst, torch.from_numpy(off).to(cuda), torch.from_numpy(lens).to(cuda), False, None, buffer=dbuf if not use_mask else torch.from_numpy(exp).to(cuda))
    exp_t = np.full((T, tb), 0xA5, dtype=np.uint8)
    fa2a.copy_non_cp(exp_t, exp, off, lens, None, False)
    torch.cuda.synchronize()
    assert np.array_equal(dst.view(torch.uint8).reshape(T, tb).cpu().numpy(), exp_t)


@pytest.mark.parametrize("scale", [1, 60])
def test_several_tensors_in_one_launch(cuda, scale):
    """a2a_memcpy_non_cp_multi (q, k, v of a tick against one buffer in one launch) leaves the bytes the oracle leaves
    after three separate copies: packing with and without per-shard masks, then unpacking into poisoned tensors.
    `scale` 60 makes shards of up to 2 400 tokens (19 MB): slices of several loop rounds that cross shard ends."""
    from distca_amd.ops import a2a_memcpy_non_cp_multi
    rng = np.random.default_rng(500 + scale)
    hiddens = [4096, 1024, 1024, 520]                      # bf16 q, k, v and an odd fourth tensor (1040-byte tokens)
    shard_counts = [11, 17, 17, 3]
    lens = [(rng.integers(0, 40, size=n) * scale).astype(np.int64) for n in shard_counts]
    for l in lens:
        l[rng.integers(0, len(l))] += 5
    lens[2] = lens[1].copy()
    tbs = [h * 2 for h in hiddens]
    offs, base = [], 0
    for l, tb in zip(lens, tbs):
        o, n = _layout(rng, l, tb)
        offs.append(o + base)
        base += n
    srcs = [rng.integers(0, 256, size=(int(l.sum()), tb), dtype=np.uint8) for l, tb in zip(lens, tbs)]
    masks = [(rng.random(len(l)) < 0.6).astype(np.int8) for l in lens]
    dev = lambda a: torch.from_numpy(a).to(cuda)
    d_srcs = [dev(a).view(torch.bfloat16) for a in srcs]
    d_offs, d_lens, d_masks = [dev(o) for o in offs], [dev(l) for l in lens], [dev(m) for m in masks]
    for use_mask in (True, False):
        buf0 = rng.integers(0, 256, size=base, dtype=np.uint8)
        exp = buf0.copy()
        for a, o, l, m, tb in zip(srcs, offs, lens, masks, tbs):
            fa2a.copy_non_cp(a, exp, o, l, m if use_mask else None, True)
        dbuf = dev(buf0.copy())
        print(f"multi pack scale={scale} mask={use_mask} buffer {base} B", flush=True)
        a2a_memcpy_non_cp_multi(d_srcs, d_offs, d_lens, True, d_masks if use_mask else None, buffer=dbuf)
        torch.cuda.synchronize()
        assert np.array_equal(dbuf.cpu().numpy(), exp)
    dsts = [torch.full(a.shape, 0x5A, dtype=torch.uint8, device=cuda).view(torch.bfloat16) for a in srcs]
    print(f"multi unpack scale={scale}", flush=True)
    a2a_memcpy_non_cp_multi(dsts, d_offs, d_lens, False, d_masks, buffer=dbuf)     # masks are ignored when unpacking
    torch.cuda.synchronize()
    for a, d in zip(srcs, dsts):
        assert np.array_equal(d.view(torch.uint8).cpu().numpy(), a)
    # fewer jobs, one of them empty
    empty = torch.empty((0, 1024), dtype=torch.bfloat16, device=cuda)
    z = torch.zeros(0, dtype=torch.int64, device=cuda)
    dbuf2 = dev(np.zeros(base, dtype=np.uint8))
    a2a_memcpy_non_cp_multi([d_srcs[0], empty], [d_offs[0], z], [d_lens[0], z], True, buffer=dbuf2)
    torch.cuda.synchronize()
    exp2 = np.zeros(base, dtype=np.uint8)
    fa2a.copy_non_cp(srcs[0], exp2, offs[0], lens[0], None, True)
    assert np.array_equal(dbuf2.cpu().numpy(), exp2)


@pytest.mark.parametrize("max_cp", [1, 3])
def test_cp_pack_unpack(cuda, max_cp):
    from distca_amd.ops import a2a_memcpy_cp
    rng = np.random.default_rng(77 + max_cp)
    nshard, hidden = 9, 1024
    lens = rng.integers(1, 50, size=nshard).astype(np.int64)
    T = int(lens.sum())
    tb = hidden * 2
    do_shard = (rng.random((nshard, max_cp)) < 0.6).astype(np.int8)
    do_shard[:, 0] = 1
    off = np.zeros((max_cp, nshard), dtype=np.int64)
    cur = 0
    for c in range(max_cp):
        for s in rng.permutation(nshard):
            off[c, s] = cur
            cur += int(lens[s]) * tb
    src = torch.from_numpy(rng.integers(0, 256, size=(T, tb), dtype=np.uint8))
    exp = np.zeros(cur, dtype=np.uint8)
    fa2a.copy_cp(src.numpy(), exp, do_shard, off, lens, True)
    dbuf = torch.zeros(cur, dtype=torch.uint8, device=cuda)
    d_do, d_off, d_len = (torch.from_numpy(x).to(cuda) for x in (do_shard, off, lens))
    print(f"cp pack max_cp={max_cp}", flush=True)
    a2a_memcpy_cp(src.view(torch.bfloat16).to(cuda), d_do, d_off, d_len, True, buffer=dbuf)
    torch.cuda.synchronize()
    assert np.array_equal(dbuf.cpu().numpy(), exp)
    planes = torch.zeros((max_cp, T, hidden), dtype=torch.bfloat16, device=cuda)
    a2a_memcpy_cp(planes, d_do, d_off, d_len, False, buffer=dbuf)
    exp_p = np.zeros((max_cp, T, tb), dtype=np.uint8)
    fa2a.copy_cp(exp_p, exp, do_shard, off, lens, False)
    torch.cuda.synchronize()
    assert np.array_equal(planes.view(torch.uint8).reshape(max_cp, T, tb).cpu().numpy(), exp_p)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("hidden", [128, 1024, 20])
def test_grad_sum(cuda, dtype, hidden):
    from distca_amd.ops import pre_a2a_grad_acc
    rng = np.random.default_rng(hidden)
    # shards: mains with copies interleaved with plain shards
    lens, num_copies, starts = [], [], []
    spec = [(37, 2), (5, 0), (64, 1), (1, 3), (12, 0)]
    order = []
    for i, (ln, nc) in enumerate(spec):
        order.append((i, ln, nc, True))
        for c in range(nc):
            order.append((i, ln, 0, False))
    perm = rng.permutation(len(order))
    order = [order[i] for i in perm]
    pos, main_idx, copy_pos = 0, {}, {}
    for j, (i, ln, nc, is_main) in enumerate(order):
        if is_main:
            main_idx[i] = j
        else:
            copy_pos.setdefault(i, []).append(pos)
        lens.append(ln)
        pos += ln
    T = pos
    max_copies = 3
    nc_arr = np.zeros(len(order), dtype=np.int32)
    cs = np.zeros((len(order), max_copies), dtype=np.int64)
    for i, (ln, nc) in enumerate(spec):
        nc_arr[main_idx[i]] = nc
        for c, p in enumerate(copy_pos.get(i, [])):
            cs[main_idx[i], c] = p
    g = torch.Generator().manual_seed(hidden)
    data = (torch.randn((T, hidden), generator=g) * 3).to(dtype)
    exp = data.clone()
    fa2a.grad_sum(exp, nc_arr, cs, lens)
    d = data.to(cuda)
    print(f"grad_sum {dtype} hidden={hidden}", flush=True)
    pre_a2a_grad_acc(d, torch.from_numpy(nc_arr).to(cuda), torch.from_numpy(cs).to(cuda), torch.tensor(lens, dtype=torch.int64, device=cuda))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().view(torch.uint8), exp.view(torch.uint8))


def test_through_torch_ops(cuda):
    """The same kernels called as `torch.ops.distca_amd.*` with the reference's op names and argument
    order (csrc/bindings/all_to_all.cpp:102-113,182-254): pack, replicating pack and duplicate sum."""
    from distca_amd import torch_ops  # noqa: F401  (registers the ops)
    rng = np.random.default_rng(5)
    nshard, hidden = 6, 256
    lens = rng.integers(1, 30, size=nshard).astype(np.int64)
    T, tb = int(lens.sum()), hidden * 2
    off, nbuf = _layout(rng, lens, tb)
    src = torch.from_numpy(rng.integers(0, 256, size=(T, tb), dtype=np.uint8))
    mask = np.array([1, 0, 1, 1, 0, 1], dtype=np.int8)
    exp = np.full(nbuf, 0x33, dtype=np.uint8)
    fa2a.copy_non_cp(src.numpy(), exp, off, lens, mask, True)
    dbuf = torch.full((nbuf,), 0x33, dtype=torch.uint8, device=cuda)
    d_off, d_len = torch.from_numpy(off).to(cuda), torch.from_numpy(lens).to(cuda)
    print("torch.ops non_cp", flush=True)
    torch.ops.distca_amd.fast_a2a_memcpy_non_cp_debug(src.view(torch.bfloat16).to(cuda), d_off, d_len, torch.from_numpy(mask).to(cuda), True, dbuf)
    torch.cuda.synchronize()
    assert np.array_equal(dbuf.cpu().numpy(), exp)

    max_cp = 2
    do_shard = np.ones((nshard, max_cp), dtype=np.int8)
    do_shard[2, 1] = 0
    off2 = np.zeros((max_cp, nshard), dtype=np.int64)
    cur = 0
    for c in range(max_cp):
        for s in rng.permutation(nshard):
            off2[c, s] = cur
            cur += int(lens[s]) * tb
    exp2 = np.zeros(cur, dtype=np.uint8)
    fa2a.copy_cp(src.numpy(), exp2, do_shard, off2, lens, True)
    dbuf2 = torch.zeros(cur, dtype=torch.uint8, device=cuda)
    print("torch.ops cp", flush=True)
    torch.ops.distca_amd.fast_a2a_memcpy_cp_debug(src.view(torch.bfloat16).to(cuda), torch.from_numpy(do_shard).to(cuda),
                                                  torch.from_numpy(off2).to(cuda), d_len, True, dbuf2)
    torch.cuda.synchronize()
    assert np.array_equal(dbuf2.cpu().numpy(), exp2)

    # rows 0..9 are a main shard with one copy in rows 10..19
    g = torch.Generator().manual_seed(9)
    data = torch.randn((20, hidden), generator=g).to(torch.bfloat16)
    nc = np.array([1, 0], dtype=np.int32)
    cs = np.array([[10], [0]], dtype=np.int64)
    ln = [10, 10]
    expd = data.clone()
    fa2a.grad_sum(expd, nc, cs, ln)
    d = data.to(cuda)
    print("torch.ops grad_acc", flush=True)
    torch.ops.distca_amd.fast_a2a_grad_acc(d, torch.from_numpy(nc).to(cuda), torch.from_numpy(cs).to(cuda), torch.tensor(ln, dtype=torch.int64, device=cuda))
    torch.cuda.synchronize()
    assert torch.equal(d.cpu().view(torch.uint8), expd.view(torch.uint8))
