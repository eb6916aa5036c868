"""The entry point that allocates nothing (`tl_flash_attention_static`, csrc/no_alloc.h), called
through ctypes as a caller without torch's allocator would: its output against that of
`tl_flash_attention`, which takes its scratch from the caller, on two calls in a row, the second
with a smaller input; and its refusal of sizes beyond the static array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
c_void_p, c_int, c_int64, c_float = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float


def ptr(t):
    return c_void_p(0 if t is None else t.data_ptr())


def decode_batch(lens, nq, nkv, hd, bs, seed):
    """One new token per request over `lens` cached keys each: q, caches, block tables, positions."""
    g = torch.Generator().manual_seed(seed)
    mb = max(-(-l // bs) for l in lens)
    nb = sum(-(-l // bs) for l in lens) + 3
    perm = torch.randperm(nb, generator=g).tolist()
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    for r, l in enumerate(lens):
        for b in range(-(-l // bs)):
            bt[r, b] = perm.pop()
    q = torch.randn(len(lens), nq * hd, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(nb, nkv, bs, hd, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(nb, nkv, bs, hd, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([l - 1 for l in lens], dtype=torch.int32, device=DEV)
    return q, k, v, bt.to(DEV), pos


def call(lib, static, batch, nq, nkv, hd, bs, n_splits, out, scratch=None):
    q, k, v, bt, pos = batch
    T = q.shape[0]
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (ptr(q), c_int64(q.stride(0)), ptr(k), ptr(v), ptr(bt), c_int(bt.shape[1]), ptr(None), ptr(None), ptr(None),
            ptr(pos), ptr(out), c_int64(out.stride(0)))
    tail = (c_int(T), c_int(T), c_int(nq), c_int(nkv), c_int(hd), c_int(bs), c_float(hd ** -0.5), c_int(0),
            c_int(n_splits), ptr(None), ptr(None), c_int(0), stream)
    if static:
        return lib.tl_flash_attention_static(*head, *tail)
    part_o = scratch[: n_splits * T * nq * hd]
    part_ml = scratch[n_splits * T * nq * hd:]
    return lib.tl_flash_attention(*head, ptr(part_o), ptr(part_ml), *tail)


def test_static_scratch_entry_point_matches_the_one_that_takes_scratch():
    from tiny_llm_amd.kernels import library
    lib = library.load()
    lib.tl_static_scratch_floats.restype = c_int64
    limit = lib.tl_static_scratch_floats()
    assert limit == 1 << 20
    nq, nkv, hd, bs = 32, 4, 64, 16
    # everything the calls touch exists before the first of them: the entry point itself allocates nothing
    big = decode_batch([700, 1500, 64, 1029, 513, 2047], nq, nkv, hd, bs, 1)
    small = decode_batch([900, 130], nq, nkv, hd, bs, 2)
    outs = {name: torch.full((b[0].shape[0], nq * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
            for name, b in (("big_s", big), ("big_r", big), ("small_s", small), ("small_r", small))}
    scratch = torch.full((limit,), float("nan"), dtype=torch.float32, device=DEV)
    # a first call on this device looks the array's address up (and loads the code, array included)
    warm = torch.empty_like(outs["small_s"])
    assert call(lib, True, small, nq, nkv, hd, bs, 2, warm) == 0
    torch.cuda.synchronize()
    # the device's own count of free memory: an allocation made inside the library, which torch's
    # allocator knows nothing of, would show here
    free_before = torch.cuda.mem_get_info()[0]
    assert call(lib, True, big, nq, nkv, hd, bs, 5, outs["big_s"]) == 0
    assert call(lib, True, small, nq, nkv, hd, bs, 3, outs["small_s"]) == 0      # smaller, right after
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free_before
    assert call(lib, False, big, nq, nkv, hd, bs, 5, outs["big_r"], scratch) == 0
    assert call(lib, False, small, nq, nkv, hd, bs, 3, outs["small_r"], scratch) == 0
    torch.cuda.synchronize()
    for name in ("big", "small"):
        got, want = outs[name + "_s"].float().cpu(), outs[name + "_r"].float().cpu()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), name           # the same kernels on the same numbers: the same bits
    # and the existing entry point is right: against plain attention over the gathered keys
    q, k, v, bt, pos = small
    for r in range(q.shape[0]):
        L = int(pos[r]) + 1
        blocks = bt[r, : -(-L // bs)].long()
        keys = k[blocks].permute(1, 0, 2, 3).reshape(nkv, -1, hd)[:, :L].float()
        vals = v[blocks].permute(1, 0, 2, 3).reshape(nkv, -1, hd)[:, :L].float()
        qr = q[r].view(nkv, nq // nkv, hd).float()
        p = torch.softmax(torch.einsum("ngd,nld->ngl", qr, keys) * hd ** -0.5, -1)
        ref = torch.einsum("ngl,nld->ngd", p, vals).reshape(-1)
        assert float((outs["small_s"][r].float() - ref).abs().max()) < 2e-2 * float(ref.abs().max())
    # one split needs no scratch at all
    one = torch.full_like(outs["small_s"], float("nan"))
    assert call(lib, True, small, nq, nkv, hd, bs, 1, one) == 0
    torch.cuda.synchronize()
    assert float((one.float() - outs["small_s"].float()).abs().max()) < 2e-2
    # beyond the static array: refused with its own status, nothing launched
    untouched = torch.full_like(outs["big_s"], 7.0)
    assert 86 * 6 * nq * (hd + 2) > limit
    assert call(lib, True, big, nq, nkv, hd, bs, 86, untouched) == 3
    torch.cuda.synchronize()
    assert bool((untouched == 7.0).all())


def test_refusal_reads_clearly_through_the_python_face():
    from tiny_llm_amd.kernels import ops
    nq, nkv, hd, bs = 32, 4, 64, 16
    q, k, v, bt, pos = decode_batch([300] * 6, nq, nkv, hd, bs, 3)
    out = torch.empty_like(q)
    with pytest.raises(ops.KernelError) as e:
        ops.flash_attention(q, k, v, bt, None, pos, out, nq, nkv, hd, hd ** -0.5, n_splits=86, static_scratch=True)
    assert "static" in str(e.value) and str(1 << 20) in str(e.value)
    ops.flash_attention(q, k, v, bt, None, pos, out, nq, nkv, hd, hd ** -0.5, n_splits=4, static_scratch=True)
    ref = torch.empty_like(q)
    ops.flash_attention(q, k, v, bt, None, pos, ref, nq, nkv, hd, hd ** -0.5, n_splits=4,
                        scratch=torch.empty(4 * 6 * nq * (hd + 2), dtype=torch.float32, device=DEV))
    assert torch.equal(out.cpu().float(), ref.cpu().float())
