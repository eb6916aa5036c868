"""Each HIP kernel alone against a plain float64 reference, at sizes other than the
engine's: odd widths, head sizes in steps of 16, page sizes 8/16/32, far keys,
a window's edge.  Vectors marked (ref) are the ones the reference's own tests hold."""
import math

import pytest
import torch

import plain_llama as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def ops():
    from tiny_llm_amd.kernels import ops as o
    return o


def tol(dtype, f32=1e-5, bf16=1.2e-2):
    return f32 if dtype == torch.float32 else bf16


def rel(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


# ------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_rows(dtype):
    # (ref) tests/ops/cuda/test_embedding.cpp:19-43: rows 2,3,1,7,9,0 of a table of width 2011
    table = (torch.arange(10 * 2011, dtype=torch.float32).reshape(10, 2011) % 97 / 97).to(dtype).to(DEV)
    ids = torch.tensor([2, 3, 1, 7, 9, 0], dtype=torch.int32, device=DEV)
    out = torch.empty(6, 2011, dtype=torch.float32, device=DEV)
    ops().embedding(ids, table, out)
    assert torch.equal(out.cpu(), table.float().cpu()[ids.cpu().long()])


# --------------------------------------------------------------------- rmsnorm
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [241, 64, 2048, 5120])
def test_rmsnorm(dtype, hidden):
    # width 241 and eps 1.192e-7 as in tests/ops/cuda/test_norm.cpp:8-47
    g = torch.Generator().manual_seed(1)
    x = torch.randn(23, hidden, generator=g) * 3
    w = (1 + 0.1 * torch.randn(hidden, generator=g))
    for wdt in (torch.float32, dtype):
        out = torch.empty(23, hidden, dtype=dtype, device=DEV)
        ops().rmsnorm(x.to(DEV), w.to(wdt).to(DEV), 1.192e-7, out)
        ref = plain.rms_norm(x.double(), w.to(wdt).double(), 1.192e-7)
        assert rel(out, ref) < tol(dtype, 2e-6, 5e-3)


def test_rmsnorm_gathers_rows():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(10, 96, generator=g)
    w = torch.randn(96, generator=g)
    rows = torch.tensor([9, 0, 4], dtype=torch.int32, device=DEV)
    out = torch.empty(3, 96, dtype=torch.float32, device=DEV)
    ops().rmsnorm(x.to(DEV), w.to(DEV), 1e-5, out, rows)
    ref = plain.rms_norm(x.double()[[9, 0, 4]], w.double(), 1e-5)
    assert rel(out, ref) < 2e-6


def test_rmsnorm_reduces_to_library_routine():
    x = torch.randn(5, 128, generator=torch.Generator().manual_seed(3))
    out = torch.empty(5, 128, dtype=torch.float32, device=DEV)
    ops().rmsnorm(x.to(DEV), torch.ones(128, device=DEV), 1e-6, out)
    ref = torch.nn.functional.rms_norm(x.double(), (128,), eps=1e-6)
    assert rel(out, ref) < 2e-6


# ---------------------------------------------------------------------- linear
def test_linear_reference_vectors():
    # (ref) tests/ops/cuda/test_gemm.cpp:8-40
    a = torch.tensor([[0., 1, 2], [3, 4, 5]], device=DEV)
    w = torch.arange(12, dtype=torch.float32, device=DEV).reshape(4, 3)
    out = torch.empty(2, 4, device=DEV)
    ops().linear(a, w, out)
    assert out.cpu().tolist() == [[5, 14, 23, 32], [14, 50, 86, 122]]
    # one row (the reference's q == 1 path) gives the same numbers
    out1 = torch.empty(1, 4, device=DEV)
    ops().linear(a[1:2], w, out1)
    assert out1.cpu().tolist() == [[14, 50, 86, 122]]


def test_lm_head_last_rows_reference_vector():
    # (ref) tests/runtime/cuda/test_linear_runtime.cpp:332-387: rows 1, 4, 9 of a [10, 3] ramp
    x = torch.arange(30, dtype=torch.float32, device=DEV).reshape(10, 3)
    w = torch.tensor([[0., 1, 2], [3, 4, 5]], device=DEV)
    rows = x[[1, 4, 9]].contiguous()
    out = torch.empty(3, 2, device=DEV)
    ops().linear(rows, w, out)
    assert out.cpu().tolist() == [[14, 50], [41, 158], [86, 338]]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,N", [(127, 255, 353), (1, 64, 251), (7, 176, 64), (130, 96, 517), (64, 2048, 256),
                                   (300, 5632, 136), (9, 5640, 520), (16, 4104, 40), (8, 5640, 524), (3, 2056, 2044),
                                   (5, 9000, 72), (8, 64, 4100), (12, 96, 8200), (16, 72, 12300), (7, 64, 8200),
                                   (5, 64, 2500), (16, 96, 3302), (17, 2048, 32000), (40, 64, 16390),
                                   (64, 2048, 32000), (33, 128, 128256), (12, 96, 1500), (16, 2048, 2048),
                                   (10, 64, 20000), (8, 128, 40004), (4, 2048, 1100), (36, 2048, 2560), (8, 64, 28672),
                                   (16, 72, 27650)])
def test_linear_sizes(dtype, M, K, N):
    if dtype == torch.bfloat16 and K % 8:
        K = K + 8 - K % 8
    g = torch.Generator().manual_seed(M * 1000 + N)
    a = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(dtype)
    res = torch.randn(M, N, generator=g)
    ref = a.double() @ w.double().T
    for out_dtype in {dtype, torch.float32}:
        out = torch.empty(M, N, dtype=out_dtype, device=DEV)
        ops().linear(a.to(DEV), w.to(DEV), out)
        assert rel(out, ref) < (1e-5 if out_dtype == torch.float32 and dtype == torch.float32 else
                                1e-5 if out_dtype == torch.float32 else 6e-3)
    out = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), out, res.to(DEV))
    assert rel(out, ref + res.double()) < 1e-5
    # in place on the residual, as the blocks use it
    x = res.clone().to(DEV)
    ops().linear(a.to(DEV), w.to(DEV), x, x)
    assert rel(x, ref + res.double()) < 1e-5


@pytest.mark.parametrize("tile", [1, 2, 3, 4])
@pytest.mark.parametrize("M,K,N", [(65, 64, 2), (257, 200, 258), (300, 72, 516), (513, 136, 130), (256, 128, 512),
                                   (130, 1096, 700)])
def test_linear_every_tile(tile, M, K, N):
    """Each tile shape of the bfloat16 product on sizes that end inside a tile (rows, columns and
    inner size), with every epilogue: by size alone the large tiles are only chosen for large,
    regular products."""
    g = torch.Generator().manual_seed(tile * 100 + M + N)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g)
    scale = torch.rand(M, generator=g) + 0.5
    ref = a.double() @ w.double().T
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), out, tile=tile)
    assert rel(out, ref) < 6e-3
    x = res.clone().to(DEV)
    ops().linear(a.to(DEV), w.to(DEV), x, x, row_scale=scale.to(DEV), tile=tile)
    assert rel(x, ref * scale.double()[:, None] + res.double()) < 1e-5
    z = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w[:N // 2 * 2].contiguous().to(DEV), z, epilogue="swiglu", tile=tile)
    assert rel(z, plain.silu(ref[:, 0:N // 2 * 2:2]) * ref[:, 1:N // 2 * 2:2]) < 6e-3
    # a view with a row stride of its own, as the q columns of a qkv buffer
    wide = torch.zeros(M, N + 24, dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), wide[:, 8:8 + N] if N % 8 == 0 else wide[:, :N], tile=tile)
    assert rel(wide[:, 8:8 + N] if N % 8 == 0 else wide[:, :N], ref) < 6e-3
    assert float(wide[:, N + 8:].abs().sum()) == 0.0


@pytest.mark.parametrize("M", [1, 5, 16, 17, 40, 64, 65, 200])
@pytest.mark.parametrize("K,N", [(64, 251), (2048, 96), (176, 64), (5632, 40), (96, 516)])
def test_linear_norm(M, K, N):
    """The product that carries an RMSNorm: (bf16(w * x) @ W^T) / rms, in one kernel for few rows and
    as pre-scale + tiled product for many; with a row gather, a residual, the SiLU-gate epilogue."""
    g = torch.Generator().manual_seed(M * 7 + N)
    x = torch.randn(M + 3, K, generator=g) * 2
    nw = 1 + 0.1 * torch.randn(K, generator=g)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g)
    rows = torch.randperm(M + 3, generator=g)[:M].to(torch.int32)
    for nwt in (torch.float32, torch.bfloat16):
        for use_rows in (False, True):
            src = (x[rows.long()] if use_rows else x[:M]).double()
            wn = nw.to(nwt).double()
            inv = 1.0 / torch.sqrt((src * src).mean(dim=-1, keepdim=True) + 1e-5)
            ref = ((wn * src).to(torch.bfloat16).double() @ w.double().T) * inv + res.double()
            out = torch.empty(M, N, dtype=torch.float32, device=DEV)
            ops().linear_norm(x.to(DEV) if use_rows else x[:M].contiguous().to(DEV), nw.to(nwt).to(DEV), 1e-5,
                              w.to(DEV), out, res.to(DEV), rows.to(DEV) if use_rows else None)
            assert rel(out, ref) < 1e-5
            # and it is an RMSNorm followed by a product, up to the rounding of the operand
            assert rel(out, plain.rms_norm(src, wn, 1e-5) @ w.double().T + res.double()) < 1e-2
    src = x[:M].double()
    inv = 1.0 / torch.sqrt((src * src).mean(dim=-1, keepdim=True) + 1e-5)
    c = ((nw.double() * src).to(torch.bfloat16).double() @ w.double().T) * inv
    z = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
    ops().linear_norm(x[:M].contiguous().to(DEV), nw.to(DEV), 1e-5, w[:N // 2 * 2].contiguous().to(DEV), z,
                      epilogue="swiglu")
    assert rel(z, plain.silu(c[:, 0:N // 2 * 2:2]) * c[:, 1:N // 2 * 2:2]) < 6e-3
    ob = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops().linear_norm(x[:M].contiguous().to(DEV), nw.to(DEV), 1e-5, w.to(DEV), ob)
    assert rel(ob, c) < 6e-3


@pytest.mark.parametrize("M", [1, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("K,N,N2", [(64, 248, 96), (5632, 2048, 516), (176, 64, 40), (96, 520, 1030), (2120, 1000, 72),
                                    (64, 4200, 40), (64, 64, 8300), (64, 2600, 3000), (72, 2048, 32000), (64, 64, 16390),
                                    (64, 5120, 72), (72, 10000, 40), (64, 16376, 24)])
def test_linear_handoff(M, K, N, N2):
    """A norm handed from the product that writes the residual stream to the product that reads
    it: the first also writes bf16(w * x) and partial sums of x^2, the second applies 1 / rms."""
    g = torch.Generator().manual_seed(M * 11 + N)
    z = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g)
    w2 = (torch.randn(N2, N, generator=g) / math.sqrt(N)).to(torch.bfloat16)
    x_ref = z.double() @ w1.double().T + res.double()
    for nwt in (torch.float32, torch.bfloat16):
        nw = (1 + 0.1 * torch.randn(N, generator=g)).to(nwt)
        x = res.clone().to(DEV)
        operand = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        sumsq = torch.full((M, ops().handoff_parts(M, N, K)), float("nan"), dtype=torch.float32, device=DEV)
        ops().linear_handoff(z.to(DEV), w1.to(DEV), x, x, emit=(nw.to(DEV), operand, sumsq))
        assert rel(x, x_ref) < 1e-5
        xs = x.cpu().double()
        # the operand is the rounded product of the weight and the float32 result, element by element
        assert torch.equal(operand.cpu(), (nw.float() * x.cpu()).to(torch.bfloat16))
        assert rel(sumsq.sum(dim=1), (xs * xs).sum(dim=1)) < 1e-6
        inv = 1.0 / torch.sqrt((xs * xs).mean(dim=-1, keepdim=True) + 1e-5)
        c = (operand.cpu().double() @ w2.double().T) * inv
        out = torch.empty(M, N2, dtype=torch.float32, device=DEV)
        ops().linear_handoff(operand, w2.to(DEV), out, prepared=(sumsq, 1e-5, N))
        assert rel(out, c) < 1e-5
        assert rel(out, plain.rms_norm(xs, nw.double(), 1e-5) @ w2.double().T) < 1e-2
        # with a gather of rows, as the output head takes the wanted positions
        rows = torch.randperm(M, generator=g)[:max(1, M // 2)].to(torch.int32)
        outg = torch.empty(rows.numel(), N2, dtype=torch.float32, device=DEV)
        ops().linear_handoff(operand, w2.to(DEV), outg, rows=rows.to(DEV), prepared=(sumsq, 1e-5, N))
        assert rel(outg, c[rows.long()]) < 1e-5
        # with the SiLU-gate epilogue, as the feed-forward's first product
        zz = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device=DEV)
        ops().linear_handoff(operand, w2.to(DEV), zz, epilogue="swiglu", prepared=(sumsq, 1e-5, N))
        assert rel(zz, plain.silu(c[:, 0::2]) * c[:, 1::2]) < 6e-3
    with pytest.raises(Exception):      # a gather of more rows than the few-row product takes
        ops().linear_handoff(torch.zeros(80, K, dtype=torch.bfloat16, device=DEV), w1.to(DEV),
                             torch.empty(65, N, dtype=torch.float32, device=DEV),
                             rows=torch.arange(65, dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("M,K,N,N2", [(65, 64, 128, 200), (300, 256, 1024, 1030), (2048, 64, 8576, 96),
                                      (512, 512, 2048, 1024), (1000, 136, 320, 16390)])
def test_linear_handoff_many_rows(M, K, N, N2):
    """The hand-off of a norm through the tiled kernel: the producer writes the operand and a sum
    of squares per 64 columns (also when it is launched in two parts), the consumer works the row
    factor out of the parts in its epilogue."""
    g = torch.Generator().manual_seed(M + N)
    z = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g)
    w2 = (torch.randn(N2, N, generator=g) / math.sqrt(N)).to(torch.bfloat16)
    x_ref = z.double() @ w1.double().T + res.double()
    assert ops().can_hand_off(M, N, K, torch.bfloat16)
    for nwt in (torch.float32, torch.bfloat16):
        nw = (1 + 0.1 * torch.randn(N, generator=g)).to(nwt)
        x = res.clone().to(DEV)
        operand = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        sumsq = torch.full((M, ops().handoff_parts(M, N, K)), float("nan"), dtype=torch.float32, device=DEV)
        ops().linear_handoff(z.to(DEV), w1.to(DEV), x, x, emit=(nw.to(DEV), operand, sumsq))
        assert rel(x, x_ref) < 1e-5
        xs = x.cpu().double()
        assert torch.equal(operand.cpu(), (nw.float() * x.cpu()).to(torch.bfloat16))
        assert not torch.isnan(sumsq).any()
        assert rel(sumsq.sum(dim=1), (xs * xs).sum(dim=1)) < 1e-6
        inv = 1.0 / torch.sqrt((xs * xs).mean(dim=-1, keepdim=True) + 1e-5)
        c = (operand.cpu().double() @ w2.double().T) * inv
        out = torch.empty(M, N2, dtype=torch.float32, device=DEV)
        ops().linear_handoff(operand, w2.to(DEV), out, prepared=(sumsq, 1e-5, N))
        assert rel(out, c) < 1e-5
        ob = torch.empty(M, N2, dtype=torch.bfloat16, device=DEV)
        ops().linear_handoff(operand, w2.to(DEV), ob, prepared=(sumsq, 1e-5, N))
        assert rel(ob, c) < 6e-3
        zz = torch.empty(M, N2 // 2, dtype=torch.bfloat16, device=DEV)
        ops().linear_handoff(operand, w2.to(DEV), zz, epilogue="swiglu", prepared=(sumsq, 1e-5, N))
        assert rel(zz, plain.silu(c[:, 0::2]) * c[:, 1::2]) < 6e-3


@pytest.mark.parametrize("M,K,N", [(2048, 64, 8576), (1000, 136, 16390)])
def test_linear_two_part_launch(M, K, N):
    """Wide products are launched in two parts (whole rounds of the largest tile, then the rest with
    another tile): every epilogue must land in the right columns of both parts."""
    g = torch.Generator().manual_seed(N)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g)
    scale = torch.rand(M, generator=g) + 0.5
    ref = a.double() @ w.double().T
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), out)
    assert rel(out, ref) < 6e-3
    x = res.clone().to(DEV)
    ops().linear(a.to(DEV), w.to(DEV), x, x, row_scale=scale.to(DEV))
    assert rel(x, ref * scale.double()[:, None] + res.double()) < 1e-5
    z = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), z, epilogue="swiglu")
    assert rel(z, plain.silu(ref[:, 0::2]) * ref[:, 1::2]) < 6e-3
    # the same values as one launch with one tile shape
    one = torch.empty(M, N, dtype=torch.float32, device=DEV)
    two = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), one, tile=3)
    ops().linear(a.to(DEV), w.to(DEV), two)
    assert rel(two, one.double()) < 1e-6


@pytest.mark.parametrize("M", [17, 50, 64, 65, 200, 512])
@pytest.mark.parametrize("K,N", [(5632, 2048), (2048, 4100), (1096, 518), (2048, 2046), (256, 2560), (4096, 6144)])
def test_linear_split_k(M, K, N):
    """Products with few output tiles split their inner size over workgroups and add the parts up
    in a second kernel, which also applies every epilogue and both sides of the norm hand-off."""
    g = torch.Generator().manual_seed(M + K + N)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(torch.bfloat16)
    res = torch.randn(M, N, generator=g)
    scale = torch.rand(M, generator=g) + 0.5
    ref = a.double() @ w.double().T
    splits = ops().split_k(M, N, K)
    few_tiles = -(-M // 128) * -(-N // 128) < 160
    if M <= 64:      # few rows: small weight matrices stay with the few-row kernel, large or deep ones are split
        must_split = K % 64 == 0 and (N * K > (17 << 20) or (N * K > (6 << 20) and (K > 4096 or M > 28)) or M >= 56) \
            and not (N > 128 * 128 and M <= 32)
    else:
        must_split = K >= 512 and few_tiles
    if must_split:
        assert splits > 1                     # these sizes are here because they are split
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), out)
    assert rel(out, ref) < 6e-3
    x = res.clone().to(DEV)
    ops().linear(a.to(DEV), w.to(DEV), x, x, row_scale=scale.to(DEV))
    assert rel(x, ref * scale.double()[:, None] + res.double()) < 1e-5
    z = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), z, epilogue="swiglu")
    assert rel(z, plain.silu(ref[:, 0::2]) * ref[:, 1::2]) < 6e-3
    y = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), y)
    assert rel(y, ref) < 1e-5
    y2 = torch.empty(M, N, dtype=torch.float32, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), y2)
    assert torch.equal(y, y2)                 # the parts are added in a fixed order
    if not ops().can_hand_off(M, N, K, torch.bfloat16) or N % 8:
        return
    # producer side of the norm hand-off, then a consumer
    nw = 1 + 0.1 * torch.randn(N, generator=g)
    x = res.clone().to(DEV)
    operand = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    sumsq = torch.full((M, ops().handoff_parts(M, N, K)), float("nan"), dtype=torch.float32, device=DEV)
    ops().linear_handoff(a.to(DEV), w.to(DEV), x, x, emit=(nw.to(DEV), operand, sumsq))
    assert rel(x, ref + res.double()) < 1e-5
    xs = x.cpu().double()
    assert torch.equal(operand.cpu(), (nw * x.cpu()).to(torch.bfloat16))
    assert rel(sumsq.sum(dim=1), (xs * xs).sum(dim=1)) < 1e-6
    w2 = (torch.randn(5000, N, generator=g) / math.sqrt(N)).to(torch.bfloat16)
    inv = 1.0 / torch.sqrt((xs * xs).mean(dim=-1, keepdim=True) + 1e-5)
    c = (operand.cpu().double() @ w2.double().T) * inv
    zz = torch.empty(M, 2500, dtype=torch.bfloat16, device=DEV)
    ops().linear_handoff(operand, w2.to(DEV), zz, epilogue="swiglu", prepared=(sumsq, 1e-5, N))
    assert rel(zz, plain.silu(c[:, 0::2]) * c[:, 1::2]) < 6e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("M,K,N", [(1, 64, 352), (9, 96, 400), (64, 2048, 96), (65, 176, 128), (300, 256, 1030),
                                   (8, 64, 28672), (16, 72, 27648), (12, 64, 22010)])
def test_linear_swiglu_epilogue(dtype, M, K, N):
    g = torch.Generator().manual_seed(M + N)
    a = torch.randn(M, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K) * 2).to(dtype)
    z = torch.empty(M, N // 2, dtype=dtype, device=DEV)
    ops().linear(a.to(DEV), w.to(DEV), z, epilogue="swiglu")
    c = a.double() @ w.double().T
    assert rel(z, plain.silu(c[:, 0::2]) * c[:, 1::2]) < tol(dtype, 1e-5, 6e-3)
    from tiny_llm_amd.kernels import KernelError
    with pytest.raises(KernelError):
        ops().linear(a.to(DEV), w.to(DEV), torch.empty(M, N, dtype=dtype, device=DEV), epilogue="swiglu")


@pytest.mark.parametrize("M", [1, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("K,N", [(64, 250), (2048, 2560), (176, 96), (4096, 64), (5120, 520), (2048, 11264), (300, 4100),
                                 (1024, 12300)])
def test_linear_norm_f32(M, K, N):
    """Float32, few rows: the norm inside the product's kernel against norm, then product, in double;
    with the SiLU-gate epilogue and with a residual; and a row gives the same bits alone and in a batch."""
    g = torch.Generator().manual_seed(M * 7 + N)
    x = (torch.randn(M, K, generator=g) * 1.7).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(DEV)
    res = torch.randn(M, N, generator=g).to(DEV)
    eps = 1e-5
    assert ops().linear_norm_f32_ok(M, N, K, K)
    ref = plain.rms_norm(x.double().cpu(), nw.double().cpu(), eps) @ w.double().cpu().T
    out = torch.full((M, N), float("nan"), device=DEV)
    ops().linear_norm_f32(x, nw, eps, w, out)
    assert rel(out, ref) < 1e-5
    out_r = torch.empty(M, N, device=DEV)
    ops().linear_norm_f32(x, nw, eps, w, out_r, residual=res)
    assert rel(out_r, ref + res.double().cpu()) < 1e-5
    if N % 2 == 0:
        z = torch.empty(M, N // 2, device=DEV)
        ops().linear_norm_f32(x, nw, eps, w, z, epilogue="swiglu")
        assert rel(z, plain.silu(ref[:, 0::2]) * ref[:, 1::2]) < 1e-5
    # against the norm's own kernel followed by the plain product: the same function, other rounding
    h = torch.empty(M, K, device=DEV)
    ops().rmsnorm(x, nw, eps, h)
    two = torch.empty(M, N, device=DEV)
    ops().linear(h, w, two)
    assert rel(out, two.double().cpu()) < 1e-5
    m = M // 2
    alone = torch.empty(1, N, device=DEV)
    ops().linear_norm_f32(x[m:m + 1].contiguous(), nw, eps, w, alone)
    assert torch.equal(alone, out[m:m + 1])
    assert not ops().linear_norm_f32_ok(65, N, K, K)
    # the norm as two kernels (what steps of more rows take, and wide products, where a workgroup of
    # the plain product owns two or three column tiles): the same BITS, with every epilogue, also
    # when the rows sit among many others (the tiled product) and when they are gathered
    tiles = -(-N // 16)
    ct = ops().linear_f32_col_tiles(M, N, K)
    assert (2 <= ct <= 3) if M <= 16 and tiles > 256 else ct == 1
    hp, inv = ops().norm_prescale_f32(x, nw, eps)
    assert rel(hp, (x * nw).double().cpu()) == 0.0
    two = torch.full((M, N), float("nan"), device=DEV)
    ops().linear(hp, w, two, row_scale=inv)
    assert torch.equal(two, out)
    ops().linear(hp, w, two, residual=res, row_scale=inv)
    assert torch.equal(two, out_r)
    if N % 2 == 0:
        z2 = torch.empty(M, N // 2, device=DEV)
        ops().linear(hp, w, z2, epilogue="swiglu", row_scale=inv)
        assert torch.equal(z2, z)
    many = torch.cat([x, (torch.randn(90, K, generator=g) * 0.3).to(DEV)])[torch.randperm(M + 90, generator=g).to(DEV)]
    where = torch.tensor([int((many == x[i]).all(dim=1).nonzero()[0]) for i in range(M)], dtype=torch.int32, device=DEV)
    hm, invm = ops().norm_prescale_f32(many, nw, eps)
    big = torch.empty(M + 90, N, device=DEV)
    ops().linear(hm, w, big, row_scale=invm)
    assert torch.equal(big[where.long()], out)
    hg, invg = ops().norm_prescale_f32(many, nw, eps, rows=where)
    ops().linear(hg, w, two, row_scale=invg)
    assert torch.equal(two, out)


@pytest.mark.parametrize("K", [70, 258, 1001])
def test_norm_prescale_f32_any_inner_size(K):
    """Inner sizes that are no multiple of 4 (no fused route exists for them): against the plain norm."""
    g = torch.Generator().manual_seed(K)
    M, N, eps = 19, 37, 1e-6
    x = torch.randn(M, K, generator=g).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(DEV)
    h, inv = ops().norm_prescale_f32(x, nw, eps)
    out = torch.empty(M, N, device=DEV)
    ops().linear(h, w, out, row_scale=inv)
    assert rel(out, plain.rms_norm(x.double().cpu(), nw.double().cpu(), eps) @ w.double().cpu().T) < 1e-5
    alone = torch.empty(1, N, device=DEV)
    h1, inv1 = ops().norm_prescale_f32(x[7:8].contiguous(), nw, eps)
    ops().linear(h1, w, alone, row_scale=inv1)
    assert torch.equal(alone, out[7:8])


@pytest.mark.parametrize("K,N", [(200, 90), (1000, 72), (5632, 130), (256, 8), (258, 34), (700, 48), (2308, 24),
                                 (1536, 2050)])
def test_linear_row_alone_equals_row_in_batch_fp32(K, N):
    """In float32 a row gives the same bits alone, among a few rows and among many: the tiled kernel
    (more than 256 rows, or an inner size that is no multiple of 4) and the few-row kernel add in one
    order, also where the few-row kernel puts two k blocks into one matrix tile (up to 8 rows and 2,048
    columns; an odd number of blocks, a last block that is not whole).  With residual and with the
    SiLU-gate epilogue too."""
    g = torch.Generator().manual_seed(5 + K)
    a = torch.randn(300, K, generator=g).to(DEV)       # 300 rows: the tiled kernel whatever the other sizes
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(DEV)
    res = torch.randn(300, N, generator=g).to(DEV)
    for kwargs in ({}, {"residual": True}, {"epilogue": "swiglu"}):
        width = N // 2 if "epilogue" in kwargs else N
        def run(rows):
            x = a[rows].contiguous()
            out = torch.empty(x.shape[0], width, device=DEV)
            r = res[rows].contiguous() if kwargs.get("residual") else None
            ops().linear(x, w, out, r, epilogue=kwargs.get("epilogue"))
            return out
        full = run(slice(0, 300))
        assert torch.equal(full[100:230], run(slice(100, 230)))      # 65 to 256 rows: either kernel, by estimate
        assert torch.equal(full[0:256], run(slice(0, 256)))
        assert torch.equal(full[37:38], run(slice(37, 38)))
        assert torch.equal(full[30:43], run(slice(30, 43)))
        assert torch.equal(full[30:38], run(slice(30, 38)))
        assert torch.equal(full[11:14], run(slice(11, 14)))
        assert torch.equal(full[3:67], run(slice(3, 67)))
        ref = a.double() @ w.double().T
        if kwargs.get("residual"):
            ref = ref + res.double()
        if "epilogue" in kwargs:
            ref = plain.silu(ref[:, 0::2]) * ref[:, 1::2]
        assert rel(full, ref) < 1e-5


def test_linear_fp32_tile_shapes_give_the_same_bits():
    """The float32 product picks 128 x 128 tiles for 1100 x 2100 outputs, 64 x 64 tiles for a
    512-row slice of them and the few-row kernel for a single row: one order of addition in all."""
    g = torch.Generator().manual_seed(77)
    K, N = 520, 2100
    a = torch.randn(1100, K, generator=g).to(DEV)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).to(DEV)
    res = torch.randn(1100, N, generator=g).to(DEV)
    def run(rows, residual):
        x = a[rows].contiguous()
        out = torch.empty(x.shape[0], N, device=DEV)
        ops().linear(x, w, out, res[rows].contiguous() if residual else None)
        return out
    for residual in (False, True):
        full = run(slice(0, 1100), residual)
        assert torch.equal(full[100:612], run(slice(100, 612), residual))
        assert torch.equal(full[5:6], run(slice(5, 6), residual))
        assert torch.equal(full[1000:1100], run(slice(1000, 1100), residual))
        ref = a.double() @ w.double().T + (res.double() if residual else 0)
        assert rel(full, ref) < 1e-5


def test_linear_refuses_bad_inner_size_in_bf16():
    from tiny_llm_amd.kernels import KernelError
    a = torch.zeros(4, 12, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 12, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(KernelError):
        ops().linear(a, w, torch.empty(4, 8, dtype=torch.bfloat16, device=DEV))


# -------------------------------------------------------------------- silu_mul
@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    # (ref) tests/ops/cuda/test_silu.cpp:8-28: silu(0) = 0, silu(1) = 1 / (1 + e^-1)
    gu = torch.tensor([[0., 1., -2., 2., 3., 0.5]], dtype=dtype, device=DEV)
    out = torch.empty(1, 3, dtype=dtype, device=DEV)
    ops().silu_mul(gu, out)
    ref = torch.tensor([[0.0, 1 / (1 + math.exp(-1)) * 3, -2 / (1 + math.exp(2)) * 0.5]])
    assert rel(out, ref) < tol(dtype, 1e-6, 4e-3)
    g = torch.Generator().manual_seed(7)
    gu = torch.randn(9, 2 * 176, generator=g).to(dtype)
    out = torch.empty(9, 176, dtype=dtype, device=DEV)
    ops().silu_mul(gu.to(DEV), out)
    ref = plain.silu(gu.double()[:, :176]) * gu.double()[:, 176:]
    assert rel(out, ref) < tol(dtype, 1e-6, 4e-3)


# ------------------------------------------------------------------ rope_store
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,nq,nkv,bs", [(96, 4, 4, 8), (16, 4, 2, 16), (48, 3, 1, 32), (128, 8, 2, 16)])
def test_rope_store(dtype, hd, nq, nkv, bs):
    # head size 96 and base 1e4 as in tests/ops/cuda/test_rope.cpp:8-37; the paged write follows
    # test_rope.cpp:100-213 (positions deep in a block table, neighbours must stay untouched)
    from tiny_llm_amd.parts.rotary import RotaryEmbedding
    T, max_pos, nblocks = 11, 64, 12
    rot = RotaryEmbedding("r", dtype, DEV, head_dim=hd, theta=10000.0, max_position=max_pos)
    cos, sin, rd = rot.rotary_tables()
    pc, ps = plain.rope_table(max_pos, hd, 10000.0)
    assert torch.equal(cos.cpu().double(), pc) and torch.equal(sin.cpu().double(), ps)
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd, generator=g).to(dtype)
    positions = torch.tensor([0, 1, 2, 3, 4, 5, 6, 40, 41, 17, 63], dtype=torch.int32)
    slots = torch.tensor([3 * bs + 0, 3 * bs + 1, 3 * bs + 2, 3 * bs + 3, 3 * bs + 4, 3 * bs + 5, 3 * bs + 6,
                          7 * bs + bs - 1, 9 * bs, 1 * bs + 1, -1], dtype=torch.int32)
    kc = torch.ones(nblocks, nkv, bs, hd, dtype=dtype, device=DEV)
    vc = torch.ones(nblocks, nkv, bs, hd, dtype=dtype, device=DEV)
    dq = qkv.clone().to(DEV)
    ops().rope_store(dq, positions.to(DEV), cos, sin, slots.to(DEV), kc, vc, nq, nkv, hd, rd)
    q_ref = plain.apply_rope(qkv.double()[:, :nq * hd].reshape(T, nq, hd), positions.tolist(), pc, ps)
    k_ref = plain.apply_rope(qkv.double()[:, nq * hd:(nq + nkv) * hd].reshape(T, nkv, hd), positions.tolist(), pc, ps)
    v_ref = qkv.double()[:, (nq + nkv) * hd:].reshape(T, nkv, hd)
    t = tol(dtype, 1e-6, 4e-3)
    assert rel(dq[:, :nq * hd].reshape(T, nq, hd), q_ref) < t
    exp_k = torch.ones(nblocks, nkv, bs, hd, dtype=torch.float64)
    exp_v = torch.ones(nblocks, nkv, bs, hd, dtype=torch.float64)
    for i in range(T):
        s = int(slots[i])
        if s < 0:
            continue
        exp_k[s // bs, :, s % bs] = k_ref[i].to(dtype).double()
        exp_v[s // bs, :, s % bs] = v_ref[i]
    assert rel(kc, exp_k) < t
    assert torch.equal(vc.cpu().double(), exp_v)
    untouched = exp_k == 1.0
    assert torch.equal(kc.cpu().double()[untouched], exp_k[untouched])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,rd", [(32, 32), (48, 16), (128, 128)])
def test_rope_store_interleaved_pairing_and_scaled_positions(dtype, hd, rd):
    """The part's other pairing, (2i, 2i + 1), and positions divided by a factor, against the plain
    functions; pairings and scalings that are not built are refused by name."""
    from tiny_llm_amd.parts.rotary import RotaryEmbedding
    nq, nkv, bs, T, max_pos = 3, 2, 8, 9, 80
    rot = RotaryEmbedding("r", dtype, DEV, head_dim=hd, rotary_dim=rd, theta=300.0, max_position=max_pos,
                          pairing="interleaved", scaling={"kind": "linear", "factor": 4.0})
    cos, sin, got_rd = rot.rotary_tables()
    assert got_rd == rd and rot.pairing == "interleaved"
    pc, ps = plain.rope_table_fast(max_pos, rd, 300.0, position_factor=4.0)
    assert torch.equal(cos.cpu().double(), pc) and torch.equal(sin.cpu().double(), ps)
    assert torch.equal(pc[4 * 7], plain.rope_table_fast(max_pos, rd, 300.0)[0][7])      # position 28 has the angles of 7
    g = torch.Generator().manual_seed(hd)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd, generator=g).to(dtype)
    positions = torch.tensor([0, 1, 2, 3, 30, 31, 79, 5, 64], dtype=torch.int32)
    slots = torch.tensor([0, 1, 2, 3, 3 * bs + 6, 3 * bs + 7, 5 * bs, -1, 2 * bs + 1], dtype=torch.int32)
    kc = torch.ones(7, nkv, bs, hd, dtype=dtype, device=DEV)
    vc = torch.ones(7, nkv, bs, hd, dtype=dtype, device=DEV)
    dq = qkv.clone().to(DEV)
    ops().rope_store(dq, positions.to(DEV), cos, sin, slots.to(DEV), kc, vc, nq, nkv, hd, rd, pairing="interleaved")

    def ref(x, heads):
        x = x.reshape(T, heads, hd).clone()
        x[..., :rd] = plain.apply_rope_interleaved(x[..., :rd], positions.tolist(), pc, ps)
        return x
    t = tol(dtype, 1e-6, 4e-3)
    assert rel(dq[:, :nq * hd].reshape(T, nq, hd), ref(qkv.double()[:, :nq * hd], nq)) < t
    k_ref = ref(qkv.double()[:, nq * hd:(nq + nkv) * hd], nkv)
    for i in range(T):
        sl = int(slots[i])
        if sl >= 0:
            assert rel(kc[sl // bs, :, sl % bs], k_ref[i].to(dtype).double()) < t
            assert torch.equal(vc[sl // bs, :, sl % bs].cpu(), qkv[i, (nq + nkv) * hd:].reshape(nkv, hd))
    # the two pairings are one rotation under a permutation of the dims (even dims first)
    x = torch.randn(T, 2, rd, generator=g, dtype=torch.float64)
    perm = list(range(0, rd, 2)) + list(range(1, rd, 2))
    assert torch.allclose(plain.apply_rope_interleaved(x, positions.tolist(), pc, ps)[..., perm],
                          plain.apply_rope(x[..., perm], positions.tolist(), pc, ps), atol=1e-12)
    with pytest.raises(ValueError, match="pairing"):
        RotaryEmbedding("r", dtype, DEV, head_dim=hd, theta=1e4, max_position=8, pairing="quarters")
    with pytest.raises(ValueError, match="scaling"):
        RotaryEmbedding("r", dtype, DEV, head_dim=hd, theta=1e4, max_position=8, scaling={"kind": "spiral", "factor": 2})
    with pytest.raises(Exception, match="pairing"):
        ops().rope_store(dq, positions.to(DEV), cos, sin, slots.to(DEV), kc, vc, nq, nkv, hd, rd, pairing="quarters")


def test_rope_invariants():
    """Position 0 is the identity; pair norms are kept; q.k depends only on the distance."""
    from tiny_llm_amd.parts.rotary import RotaryEmbedding
    hd = 32
    rot = RotaryEmbedding("r", torch.float32, DEV, head_dim=hd, theta=500000.0, max_position=512)
    cos, sin, rd = rot.rotary_tables()
    g = torch.Generator().manual_seed(13)
    base = torch.randn(1, 3 * hd, generator=g)     # one q head, one k head, one v head

    def rotated(p):
        """(q rotated in place, k as it lands in the cache) for a token at position p."""
        x = base.clone().to(DEV)
        kc = torch.zeros(1, 1, 4, hd, device=DEV)
        vc = torch.zeros(1, 1, 4, hd, device=DEV)
        ops().rope_store(x, torch.tensor([p], dtype=torch.int32, device=DEV), cos, sin,
                         torch.tensor([2], dtype=torch.int32, device=DEV), kc, vc, 1, 1, hd, rd)
        assert torch.equal(vc.cpu()[0, 0, 2], base[0, 2 * hd:])
        return x.cpu()[0, :hd], kc.cpu()[0, 0, 2]

    q0, k0 = rotated(0)
    assert torch.equal(q0, base[0, :hd]) and torch.equal(k0, base[0, hd:2 * hd])
    q7, _ = rotated(7)
    pair = lambda v: v[:hd // 2] ** 2 + v[hd // 2:] ** 2
    assert torch.allclose(pair(q7), pair(base[0, :hd]), rtol=1e-5, atol=1e-6)
    dots = []
    for m, n in [(5, 2), (105, 102), (303, 300)]:
        qm, _ = rotated(m)
        _, kn = rotated(n)
        dots.append(float(qm.double() @ kn.double()))
    assert abs(dots[0] - dots[1]) < 1e-4 and abs(dots[0] - dots[2]) < 1e-4
    qa, _ = rotated(9)
    _, kb = rotated(2)
    assert abs(float(qa.double() @ kb.double()) - dots[0]) > 1e-3   # another distance, another score


# ------------------------------------------------------------- paged attention
def _paged_case(dtype, lens, q_lens, nq, nkv, hd, bs, window=0, seed=0, boost=None, shuffle=True,
                impl="generic", n_splits=1, tile_tokens=None):
    """Builds a batch: request r has lens[r] cached tokens, the last q_lens[r] are this step's
    queries.  Returns engine output and the plain result, both [T, nq, hd]."""
    g = torch.Generator().manual_seed(seed)
    R = len(lens)
    nblocks = sum(-(-l // bs) for l in lens) + 3
    perm = torch.randperm(nblocks, generator=g).tolist() if shuffle else list(range(nblocks))
    kc = torch.full((nblocks, nkv, bs, hd), float("nan"), dtype=dtype)
    vc = torch.full((nblocks, nkv, bs, hd), float("nan"), dtype=dtype)
    max_blocks = max(-(-l // bs) for l in lens)
    bt = torch.zeros(R, max_blocks, dtype=torch.int32)
    qs, refs, req_of, pos = [], [], [], []
    for r, (L, ql) in enumerate(zip(lens, q_lens)):
        k = torch.randn(L, nkv, hd, generator=g).to(dtype)
        v = torch.randn(L, nkv, hd, generator=g).to(dtype)
        q = torch.randn(L, nq, hd, generator=g).to(dtype)
        if boost is not None and boost < L:     # make one far key stand out for the last query
            far = boost
            k[far] = 0
            k[far, :, 0] = 6.0
            q[L - 1] = 0
            q[L - 1, :, 0] = 3.0 * math.sqrt(hd)          # score 18 against random ones of order 1
        for b in range(-(-L // bs)):
            blk = perm.pop()
            bt[r, b] = blk
            n = min(bs, L - b * bs)
            kc[blk, :, :n] = k[b * bs:b * bs + n].transpose(0, 1)
            vc[blk, :, :n] = v[b * bs:b * bs + n].transpose(0, 1)
        full = plain.attention_fast(q.double(), k.double(), v.double(), list(range(L)), window)
        qs.append(q[L - ql:])
        refs.append(full[L - ql:])
        req_of += [r] * ql
        pos += list(range(L - ql, L))
    q = torch.cat(qs).reshape(-1, nq * hd).contiguous()
    out = torch.empty_like(q).to(DEV)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    if impl == "generic":
        ops().paged_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), i32(req_of), i32(pos), out, nq, nkv,
                              hd, 1.0 / math.sqrt(hd), window)
    else:
        # query tiles of at most 16 // (nq / nkv) tokens, as the step context builds them
        per = (16 // (nq // nkv)) * ((8 if impl == "prefill" else 4) if impl.startswith("prefill") else 1)
        if tile_tokens is not None:
            per = tile_tokens
        t_req, t_tok0, t_ntok, t = [], [], [], 0
        for r, ql in enumerate(q_lens):
            for s0 in range(0, ql, per):
                t_req.append(r)
                t_tok0.append(t + s0)
                t_ntok.append(min(per, ql - s0))
            t += ql
        T = q.shape[0]
        if impl.startswith("prefill"):
            scratch = torch.full((max(1, n_splits * T * nq * (hd + 2)),), float("nan"), device=DEV)
            ops().flash_prefill(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), (i32(t_req), i32(t_tok0), i32(t_ntok)),
                                i32(pos), out, nq, nkv, hd, 1.0 / math.sqrt(hd), window, 8 if impl == "prefill" else 4,
                                n_splits, scratch)
            return out.reshape(-1, nq, hd), torch.cat(refs)
        scratch = torch.full((max(1, n_splits * T * nq * (hd + 2)),), float("nan"), device=DEV)
        if impl == "f32":       # n_splits stands for the number of 256-key chunks given to workgroups of their own
            tiles = None if (n_splits == -1) else (i32(t_req), i32(t_tok0), i32(t_ntok))
            chunks = max(1, abs(n_splits))
            scratch = torch.full((max(1, chunks * T * nq * (hd + 2)),), float("nan"), device=DEV)
            ops().attention_f32(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), tiles, i32(pos), out, nq, nkv, hd,
                                1.0 / math.sqrt(hd), window, chunks, scratch)
            return out.reshape(-1, nq, hd), torch.cat(refs)
        ops().flash_attention(q.to(DEV), kc.to(DEV), vc.to(DEV), bt.to(DEV), (i32(t_req), i32(t_tok0), i32(t_ntok)),
                              i32(pos), out, nq, nkv, hd, 1.0 / math.sqrt(hd), window, n_splits, scratch)
    return out.reshape(-1, nq, hd), torch.cat(refs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,bs", [(4, 2, 48, 32), (4, 2, 64, 16), (3, 1, 32, 8), (8, 8, 16, 16),
                                          (6, 2, 80, 16), (2, 1, 128, 64), (5, 5, 112, 8), (2, 2, 256, 16)])
def test_paged_attention_mixed_batch(dtype, nq, nkv, hd, bs):
    # shapes after tests/ops/cuda/test_flash_attention.cpp:172-271 (q 107, kv 123, heads 4:2), generalised:
    # a whole prompt, a portion with earlier context, single decoded tokens, a one-token request
    out, ref = _paged_case(dtype, lens=[123, 107, 65, 1, 300], q_lens=[123, 40, 1, 1, 1], nq=nq, nkv=nkv,
                           hd=hd, bs=bs, seed=hd + bs)
    assert not torch.isnan(out).any()
    assert rel(out, ref) < tol(dtype, 2e-6, 8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_far_key_among_hundreds(dtype):
    # one early key dominates the last query: a kernel that drops or misplaces it shows at once
    for far in (0, 15, 16, 255, 256, 511):
        out, ref = _paged_case(dtype, lens=[700], q_lens=[1], nq=4, nkv=2, hd=64, bs=16, seed=far, boost=far)
        assert rel(out, ref) < tol(dtype, 2e-6, 8e-3), far


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 7, 16, 33])
def test_paged_attention_window_edge(dtype, window):
    out, ref = _paged_case(dtype, lens=[90, 40, 64], q_lens=[90, 1, 5], nq=4, nkv=2, hd=32, bs=8,
                           window=window, seed=window)
    assert rel(out, ref) < tol(dtype, 2e-6, 8e-3)


FLASH_SHAPES = [(4, 2, 48, 32), (32, 4, 64, 16), (3, 1, 32, 8), (8, 8, 16, 16), (6, 2, 80, 16), (16, 1, 128, 64),
                (5, 5, 112, 8), (12, 4, 96, 16), (8, 2, 64, 24), (4, 4, 32, 1), (2, 1, 64, 100)]


@pytest.mark.parametrize("n_splits", [1, 3])
@pytest.mark.parametrize("nq,nkv,hd,bs", FLASH_SHAPES)
def test_flash_attention_mixed_batch(nq, nkv, hd, bs, n_splits):
    out, ref = _paged_case(torch.bfloat16, lens=[123, 107, 65, 1, 300, 2], q_lens=[123, 40, 1, 1, 1, 2], nq=nq,
                           nkv=nkv, hd=hd, bs=bs, seed=hd + bs, impl="flash", n_splits=n_splits)
    assert not torch.isnan(out).any()
    assert rel(out, ref) < 8e-3


@pytest.mark.parametrize("impl,n_splits", [("prefill", 1), ("prefill4", 1), ("prefill4", 3), ("prefill", 2)])
@pytest.mark.parametrize("nq,nkv,hd,bs", FLASH_SHAPES)
def test_flash_prefill_mixed_batch(nq, nkv, hd, bs, impl, n_splits):
    out, ref = _paged_case(torch.bfloat16, lens=[123, 107, 65, 1, 300, 2, 513], q_lens=[123, 40, 1, 1, 1, 2, 257],
                           nq=nq, nkv=nkv, hd=hd, bs=bs, seed=hd + bs, impl=impl, n_splits=n_splits)
    assert not torch.isnan(out).any()
    assert rel(out, ref) < 8e-3


@pytest.mark.parametrize("window", [1, 7, 16, 33, 100])
def test_flash_prefill_window_edge(window):
    for n_splits in (1, 2):
        out, ref = _paged_case(torch.bfloat16, lens=[190, 40, 64, 130], q_lens=[190, 1, 5, 70], nq=4, nkv=2, hd=32,
                               bs=8, window=window, seed=window, impl="prefill", n_splits=n_splits)
        assert not torch.isnan(out).any()
        assert rel(out, ref) < 8e-3


def test_flash_prefill_far_key_among_hundreds():
    for far in (0, 15, 16, 63, 64, 255, 256, 511, 699):
        for impl, n_splits in (("prefill", 1), ("prefill4", 1), ("prefill4", 4)):
            out, ref = _paged_case(torch.bfloat16, lens=[700], q_lens=[30], nq=8, nkv=1, hd=64, bs=16, seed=far,
                                   boost=far, impl=impl, n_splits=n_splits)
            assert rel(out, ref) < 8e-3, far


@pytest.mark.parametrize("hd", [64, 128])
def test_flash_prefill_eight_splits_over_a_long_context(hd):
    """A portion of 40 tokens at the end of 5,000, its keys shared out over eight workgroups (what the
    engine asks for from 32,768 tokens of context on), beside a portion that is a whole short prompt."""
    for far in (3, 2047, 2048, 4960, 4999):
        out, ref = _paged_case(torch.bfloat16, lens=[5000, 90], q_lens=[40, 90], nq=8, nkv=2, hd=hd, bs=16, seed=far,
                               boost=far, impl="prefill4", n_splits=8)
        assert not torch.isnan(out).any()
        assert rel(out, ref) < 8e-3, far


@pytest.mark.parametrize("n_splits", [1, 2, 7])
def test_flash_attention_far_key_among_hundreds(n_splits):
    for far in (0, 15, 16, 63, 64, 255, 256, 511, 699):
        out, ref = _paged_case(torch.bfloat16, lens=[700], q_lens=[1], nq=8, nkv=1, hd=64, bs=16, seed=far,
                               boost=far, impl="flash", n_splits=n_splits)
        assert rel(out, ref) < 8e-3, far


@pytest.mark.parametrize("hd,n_splits", [(64, 32), (64, 64), (128, 33), (128, 64)])
def test_flash_attention_many_splits_over_a_long_context(hd, n_splits):
    """Thirty-two to sixty-four workgroups share the keys of one request (what the engine asks for at
    contexts of tens of thousands of tokens), more than the merge kernel takes in one round trip; one
    key among 5,000 stands out, near the start, at a split's edge, at the end; a second request is so
    short that most splits hold none of its keys."""
    for far in (3, 2047, 2048, 4999):
        out, ref = _paged_case(torch.bfloat16, lens=[5000, 70], q_lens=[1, 1], nq=8, nkv=2, hd=hd, bs=16, seed=far,
                               boost=far, impl="flash", n_splits=n_splits)
        assert not torch.isnan(out).any()
        assert rel(out, ref) < 8e-3, far


@pytest.mark.parametrize("window", [1, 7, 16, 33, 100])
def test_flash_attention_window_edge(window):
    for n_splits in (1, 2):
        out, ref = _paged_case(torch.bfloat16, lens=[190, 40, 64, 130], q_lens=[190, 1, 5, 1], nq=4, nkv=2, hd=32,
                               bs=8, window=window, seed=window, impl="flash", n_splits=n_splits)
        assert not torch.isnan(out).any()
        assert rel(out, ref) < 8e-3


# ---------------------------------------------- float32 attention on the matrix cores
@pytest.mark.parametrize("chunks", [1, 3])
@pytest.mark.parametrize("nq,nkv,hd,bs", FLASH_SHAPES)
def test_attention_f32_mixed_batch(nq, nkv, hd, bs, chunks):
    out, ref = _paged_case(torch.float32, lens=[123, 107, 65, 1, 300, 2, 513], q_lens=[123, 40, 1, 1, 1, 2, 257],
                           nq=nq, nkv=nkv, hd=hd, bs=bs, seed=hd + bs, impl="f32", n_splits=chunks)
    assert not torch.isnan(out).any()
    assert rel(out, ref) < 2e-6


def test_attention_f32_far_key_window_edge_and_decode_batch():
    for far in (0, 15, 16, 63, 64, 255, 256, 511, 512, 699):
        for chunks in (1, 3):
            out, ref = _paged_case(torch.float32, lens=[700], q_lens=[30 if chunks == 1 else 1], nq=8, nkv=1, hd=64,
                                   bs=16, seed=far, boost=far, impl="f32", n_splits=chunks)
            assert rel(out, ref) < 2e-6, far
    for window in (1, 7, 16, 33, 100, 600):
        out, ref = _paged_case(torch.float32, lens=[190, 40, 64, 130, 1300], q_lens=[190, 1, 5, 70, 2], nq=4, nkv=2,
                               hd=32, bs=8, window=window, seed=window, impl="f32", n_splits=6)
        assert not torch.isnan(out).any()
        assert rel(out, ref) < 2e-6, window
    lens = [1, 2, 63, 64, 65, 127, 128, 129, 500, 1000, 17, 256, 512, 513, 1024, 1025]
    for chunks in (1, 5, -5):       # -5: without tile arrays (row i is request i), as a decode step runs
        out, ref = _paged_case(torch.float32, lens=lens, q_lens=[1] * len(lens), nq=32, nkv=4, hd=64, bs=16,
                               seed=5, impl="f32", n_splits=chunks)
        assert rel(out, ref) < 2e-6


def test_attention_f32_gives_the_same_bits_however_the_work_is_cut():
    """A query row's result, to the bit: alone or in a batch, in tiles of one token or of several,
    keys walked by one workgroup or chunks of 256 given to several."""
    lens, nq, nkv, hd, bs = [1100, 77, 513], 8, 2, 64, 16
    base, _ = _paged_case(torch.float32, lens=lens, q_lens=[300, 77, 1], nq=nq, nkv=nkv, hd=hd, bs=bs, seed=3, impl="f32")
    for kw in (dict(n_splits=5), dict(tile_tokens=1), dict(tile_tokens=3, n_splits=7), dict(tile_tokens=2, n_splits=1)):
        other, _ = _paged_case(torch.float32, lens=lens, q_lens=[300, 77, 1], nq=nq, nkv=nkv, hd=hd, bs=bs, seed=3,
                               impl="f32", **kw)
        assert torch.equal(other.cpu(), base.cpu()), kw
    # the last rows of the first request alone, as single decoded tokens would come
    tail, _ = _paged_case(torch.float32, lens=lens, q_lens=[1, 1, 1], nq=nq, nkv=nkv, hd=hd, bs=bs, seed=3,
                          impl="f32", n_splits=-5)
    assert torch.equal(tail.cpu()[0], base.cpu()[299]) and torch.equal(tail.cpu()[1], base.cpu()[376])


@pytest.mark.parametrize("nq,nkv,hd,window", [(8, 4, 64, 0), (4, 4, 32, 0), (16, 2, 128, 0), (8, 4, 48, 300)])
def test_attention_f32_of_many_query_tiles_has_the_bits_of_few(nq, nkv, hd, window):
    """A step of a thousand query tiles and more (whole prompts) runs a wave per tile, four neighbouring
    tiles a workgroup; the same rows as a step of chunks given to workgroups of their own (what decode
    steps run), and in tiles of one token: the same bits, and the plain result within rounding."""
    per = 16 // (nq // nkv)
    lens = [per * (1024 // nkv), 700, 65, 1]        # whole prompts: at least 1,024 tiles x kv heads
    assert sum(-(-n // per) for n in lens) * nkv >= 1024
    kw = dict(lens=lens, q_lens=lens, nq=nq, nkv=nkv, hd=hd, bs=16, seed=11, window=window, impl="f32")
    many, ref = _paged_case(torch.float32, **kw)
    assert not torch.isnan(many).any()
    assert rel(many, ref) < 2e-6
    chunks = -(-max(lens) // 256)
    few, _ = _paged_case(torch.float32, n_splits=chunks, **kw)
    assert torch.equal(many.cpu(), few.cpu())
    if nq == nkv:      # tiles of one token are tiles of one row per head group only where a tile holds 16 tokens
        single, _ = _paged_case(torch.float32, tile_tokens=3, **kw)
        assert torch.equal(many.cpu(), single.cpu())


def test_flash_attention_decode_batch():
    """Single decoded tokens of many requests of very different lengths, keys split over workgroups."""
    lens = [1, 2, 63, 64, 65, 127, 128, 129, 500, 1000, 17, 256]
    for n_splits in (1, 4):
        out, ref = _paged_case(torch.bfloat16, lens=lens, q_lens=[1] * len(lens), nq=32, nkv=4, hd=64, bs=16,
                               seed=5, impl="flash", n_splits=n_splits)
        assert rel(out, ref) < 8e-3


@pytest.mark.parametrize("nq,nkv,hd,bs", [(32, 4, 64, 16), (3, 1, 32, 8), (8, 8, 16, 16), (16, 2, 128, 32), (6, 2, 80, 16),
                                          (3, 1, 112, 12), (4, 1, 48, 16)])
@pytest.mark.parametrize("n_splits", [1, 3])
@pytest.mark.parametrize("window", [0, 150])
def test_flash_attention_fused_rotation_and_cache_write(nq, nkv, hd, bs, n_splits, window):
    """Decode step with rotation and cache write inside the attention kernel == rope_store + attention.
    The long requests give a wave several key tiles in turn (the new token's in the last), the
    window lets a wave's first tile be another than the one whose pages it looked up ahead."""
    _fused_against_separate(nq, nkv, hd, bs, n_splits, window, nq + hd)


def test_flash_attention_fused_rotation_random_sizes():
    """The same at sizes drawn at random: every head size the kernel takes, 1 to 16 heads a kv head,
    pages of 1 to 100 tokens, up to 16 key splits, windows from 1 to beyond the longest context.
    Both ways write the same rows of the cache."""
    import random
    for seed in range(120):
        rng = random.Random(seed)
        hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
        nkv = rng.choice([1, 2, 3, 4, 8])
        group = rng.choice([1, 2, 3, 4, 5, 8, 16])
        bs = rng.choice([1, 2, 3, 4, 8, 16, 32, 64, 12, 100])
        n_splits = rng.choice([1, 2, 3, 4, 8, 16])
        window = rng.choice([0, 0, 1, 2, 16, 64, 65, 150, 300, 1000])
        try:
            _fused_against_separate(nkv * group, nkv, hd, bs, n_splits, window, seed)
        except AssertionError as e:
            raise AssertionError(f"seed {seed}: {nkv * group}/{nkv} heads of {hd}, page {bs}, {n_splits} splits, "
                                 f"window {window}") from e


def _fused_against_separate(nq, nkv, hd, bs, n_splits, window, seed):
    from tiny_llm_amd.parts.rotary import RotaryEmbedding
    g = torch.Generator().manual_seed(seed)
    lens = [1, 2, 63, 64, 65, 129, 300, 17, 600, 1100]
    R = len(lens)
    rot = RotaryEmbedding("r", torch.bfloat16, DEV, head_dim=hd, theta=10000.0, max_position=1200)
    cos, sin, rd = rot.rotary_tables()
    nblocks = sum(-(-l // bs) for l in lens) + 2
    perm = torch.randperm(nblocks, generator=g).tolist()
    mb = max(-(-l // bs) for l in lens)
    bt = torch.zeros(R, mb, dtype=torch.int32)
    kc = (torch.randn(nblocks, nkv, bs, hd, generator=g)).to(torch.bfloat16)
    vc = (torch.randn(nblocks, nkv, bs, hd, generator=g)).to(torch.bfloat16)
    slots = []
    for r, L in enumerate(lens):
        for b in range(-(-L // bs)):
            bt[r, b] = perm.pop()
        slots.append(int(bt[r, (L - 1) // bs]) * bs + (L - 1) % bs)
    qkv = torch.randn(R, (nq + 2 * nkv) * hd, generator=g).to(torch.bfloat16)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    pos = i32([l - 1 for l in lens])
    tiles = (i32(list(range(R))), i32(list(range(R))), i32([1] * R))
    scratch = torch.full((n_splits * R * nq * (hd + 2),), float("nan"), device=DEV)
    # separate kernels
    kc1, vc1, qkv1 = kc.clone().to(DEV), vc.clone().to(DEV), qkv.clone().to(DEV)
    ops().rope_store(qkv1, pos, cos, sin, i32(slots), kc1, vc1, nq, nkv, hd, rd)
    out1 = torch.empty(R, nq * hd, dtype=torch.bfloat16, device=DEV)
    ops().flash_attention(qkv1[:, :nq * hd], kc1, vc1, bt.to(DEV), tiles, pos, out1, nq, nkv, hd, hd ** -0.5, window,
                          n_splits, scratch)
    # fused
    kc2, vc2, qkv2 = kc.clone().to(DEV), vc.clone().to(DEV), qkv.clone().to(DEV)
    out2 = torch.empty(R, nq * hd, dtype=torch.bfloat16, device=DEV)
    ops().flash_attention(qkv2[:, :nq * hd], kc2, vc2, bt.to(DEV), tiles, pos, out2, nq, nkv, hd, hd ** -0.5, window,
                          n_splits, scratch, fused_rope=(cos, sin))
    # The same rows with the same values: the values are copied, the keys rotated by the same
    # expression in both kernels, whose multiplications and additions the compiler fuses as it likes
    # in each: once in some ten thousand elements the last bit of a key differs (and then, by as
    # little, outputs that the key or the query, rotated the same way, enters).  A row lost or
    # misplaced is off by the size of the values.
    assert torch.equal(vc1, vc2)
    k1, k2 = kc1.float(), kc2.float()
    assert ((k1 - k2).abs() <= k1.abs() * 2.0 ** -7).all() and (k1 != k2).float().mean() < 1e-3
    assert torch.equal(qkv2.cpu(), qkv)                          # the input rows are left as they were
    assert rel(out2, out1.double()) < 1e-2
    assert (out2 != out1).float().mean() < 0.02
    # without tile arrays: row i is the one new token of request i
    kc3, vc3 = kc.clone().to(DEV), vc.clone().to(DEV)
    out3 = torch.empty(R, nq * hd, dtype=torch.bfloat16, device=DEV)
    ops().flash_attention(qkv2[:, :nq * hd], kc3, vc3, bt.to(DEV), None, pos, out3, nq, nkv, hd, hd ** -0.5, window,
                          n_splits, scratch, fused_rope=(cos, sin))
    assert torch.equal(out3, out2) and torch.equal(kc3, kc2) and torch.equal(vc3, vc2)


@pytest.mark.parametrize("hd", [48, 80, 112])
def test_fused_rotation_head_sizes_that_end_inside_a_k_step(hd):
    """Head sizes that are no multiple of 32: the last k step of the score product has slots beyond
    the head, where the query operand is zero.  The new token's key, which the fused kernel holds in
    registers, must be finite there too (0 * NaN is NaN, and the sum then drops the whole row to
    zero).  What an unwritten register holds changes from case to case, hence the many cases."""
    from tiny_llm_amd.parts.rotary import RotaryEmbedding
    nq, nkv, bs = 3, 1, 16
    rot = RotaryEmbedding("r", torch.bfloat16, DEV, head_dim=hd, theta=10000.0, max_position=400)
    cos, sin, rd = rot.rotary_tables()
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for seed in range(40):
        g = torch.Generator().manual_seed(seed)
        for L in (40, 81, 300):
            nb = -(-L // bs)
            bt = torch.arange(nb, dtype=torch.int32, device=DEV).reshape(1, nb)
            kc = torch.randn(nb, nkv, bs, hd, generator=g).to(torch.bfloat16).to(DEV)
            vc = torch.randn(nb, nkv, bs, hd, generator=g).to(torch.bfloat16).to(DEV)
            qkv = torch.randn(1, (nq + 2 * nkv) * hd, generator=g).to(torch.bfloat16).to(DEV)
            pos, slots = i32([L - 1]), i32([L - 1])
            kc1, vc1, qkv1 = kc.clone(), vc.clone(), qkv.clone()
            ops().rope_store(qkv1, pos, cos, sin, slots, kc1, vc1, nq, nkv, hd, rd)
            out1 = torch.empty(1, nq * hd, dtype=torch.bfloat16, device=DEV)
            ops().flash_attention(qkv1[:, :nq * hd], kc1, vc1, bt, None, pos, out1, nq, nkv, hd, hd ** -0.5, 0, 1, None)
            out2 = torch.empty(1, nq * hd, dtype=torch.bfloat16, device=DEV)
            ops().flash_attention(qkv[:, :nq * hd], kc, vc, bt, None, pos, out2, nq, nkv, hd, hd ** -0.5, 0, 1, None,
                                  fused_rope=(cos, sin))
            assert rel(out2, out1.double()) < 1e-2, (hd, seed, L)      # a row dropped to zero gives 1


def test_paged_attention_reduces_to_library_routine():
    """One request, whole prompt, identity block table: plain causal attention."""
    nq = nkv = 2
    hd, L, bs = 64, 50, 16
    g = torch.Generator().manual_seed(17)
    q, k, v = (torch.randn(L, nq, hd, generator=g) for _ in range(3))
    nb = -(-L // bs)
    kc = torch.zeros(nb, nkv, bs, hd)
    vc = torch.zeros(nb, nkv, bs, hd)
    for b in range(nb):
        n = min(bs, L - b * bs)
        kc[b, :, :n] = k[b * bs:b * bs + n].transpose(0, 1)
        vc[b, :, :n] = v[b * bs:b * bs + n].transpose(0, 1)
    out = torch.empty(L, nq * hd, device=DEV)
    ops().paged_attention(q.reshape(L, -1).to(DEV), kc.to(DEV), vc.to(DEV),
                          torch.arange(nb, dtype=torch.int32, device=DEV).reshape(1, nb),
                          torch.zeros(L, dtype=torch.int32, device=DEV),
                          torch.arange(L, dtype=torch.int32, device=DEV), out, nq, nkv, hd, hd ** -0.5, 0)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.double().transpose(0, 1), k.double().transpose(0, 1), v.double().transpose(0, 1), is_causal=True)
    assert rel(out.reshape(L, nq, hd), ref.transpose(0, 1)) < 2e-6


# -------------------------------------------------------------------- sampling
def _sample(logits, **kw):
    n = logits.shape[0]
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    dev = {k: (v.to(DEV) if v is not None else None) for k, v in kw.items()}
    ops().sample(logits.to(DEV), out, **dev)
    return out.cpu().tolist()


def test_argmax_reference_vector_and_first_maximum():
    # (ref) tests/logit_processors/test_argmax_processor.cpp:19-31: ramps -> id 19
    ramps = torch.arange(40, dtype=torch.float32).reshape(2, 20)
    assert _sample(ramps) == [19, 19]
    ties = torch.zeros(3, 1000)
    ties[0, [5, 700]] = 2.0
    ties[1, 999] = 1.0
    ties[2] = -1.0
    assert _sample(ties) == [5, 999, 0]
    big = torch.randn(4, 32003, generator=torch.Generator().manual_seed(19))
    assert _sample(big) == big.argmax(dim=1).tolist()


def test_sampling_single_finite_logit():
    # (ref) tests/logit_processors/test_sample_processors.cpp:20-34: one finite logit is always drawn
    l = torch.full((2, 64), -1e30)
    l[0, 17] = 0.3
    l[1, 63] = -2.0
    got = _sample(l, temperature=torch.tensor([1.0, 0.5]), top_k=torch.tensor([0, 0], dtype=torch.int32),
                  top_p=torch.tensor([1.0, 1.0]), seeds=torch.tensor([1, 2]), counters=torch.tensor([0, 9], dtype=torch.int32))
    assert got == [17, 63]


def test_sampling_matches_plain_chain():
    """Temperature -> top-k -> top-p -> multinomial gives the plain chain's token for the same u."""
    g = torch.Generator().manual_seed(23)
    cases = []
    for vocab in (20, 251, 517, 32000):
        for (t, k, p) in [(0.7, 50, 0.95), (1.0, 0, 1.0), (0.8, 5, 1.0), (1.3, 0, 0.2), (0.5, 1, 0.9),
                          (1.0, 10, 0.0), (2.0, 0, 0.6)]:
            cases.append((vocab, t, min(k, vocab), p))
    mismatches = 0
    for vocab, t, k, p in cases:
        n = 12
        logits = torch.randn(n, vocab, generator=g) * 3
        seeds = torch.arange(n, dtype=torch.int64) * 7919 + vocab
        ctrs = torch.arange(n, dtype=torch.int32) + 3
        got = _sample(logits, temperature=torch.full((n,), t), top_k=torch.full((n,), k, dtype=torch.int32),
                      top_p=torch.full((n,), p), seeds=seeds, counters=ctrs)
        for i in range(n):
            u = plain.uniform_for(int(seeds[i]), int(ctrs[i]))
            want = plain.sample_token(logits[i], t, k, p, u)
            if got[i] != want:
                # allowed only when u sits on a boundary of the cumulative distribution (rounding)
                near = {plain.sample_token(logits[i], t, k, p, min(max(u + d, 0.0), 0.999999)) for d in (-2e-6, 2e-6)}
                assert got[i] in near, (vocab, t, k, p, i, got[i], want)
                mismatches += 1
    assert mismatches <= 2


def test_sampling_top_p_reference_vectors():
    # (ref) tests/logit_processors/test_sort_processors.cpp:120-200: with logits i/40 and logit[0] = 0.5,
    # p = 0.2 keeps ids {0, 19, 18, 17}; with logit[0] = 2 it keeps {0, 19}
    for first, keep in ((0.5, {0, 19, 18, 17}), (2.0, {0, 19})):
        l = (torch.arange(20, dtype=torch.float32) / 40) + (0.5 if first == 2.0 else 0.0)
        l[0] = first
        assert set(plain.top_k_top_p_ids(l, 0, 0.2)) == keep
        n = 400
        got = _sample(l.repeat(n, 1), temperature=torch.ones(n), top_k=torch.zeros(n, dtype=torch.int32),
                      top_p=torch.full((n,), 0.2), seeds=torch.arange(n, dtype=torch.int64),
                      counters=torch.zeros(n, dtype=torch.int32))
        assert set(got) == keep


def test_sampling_distribution():
    """Frequencies follow softmax(logits / T) over the kept ids."""
    l = torch.tensor([2.0, 1.0, 0.0, -1.0, 3.0, 0.5])
    n = 20000
    got = _sample(l.repeat(n, 1), temperature=torch.full((n,), 0.8), top_k=torch.full((n,), 4, dtype=torch.int32),
                  top_p=torch.ones(n), seeds=torch.full((n,), 12345, dtype=torch.int64),
                  counters=torch.arange(n, dtype=torch.int32))
    kept = [4, 0, 1, 5]
    probs = torch.softmax(l[kept].double() / 0.8, 0)
    counts = torch.tensor([got.count(i) for i in kept], dtype=torch.float64) / n
    assert set(got) == set(kept)
    assert (counts - probs).abs().max() < 0.015


# ------------------------------------------------------------ seeded numbers
@pytest.mark.parametrize("dtype", DTYPES)
def test_seeded_numbers_are_the_same_bits_on_host_and_device(dtype):
    """Random-weights mode: a tensor made on the device equals the one made on the host (which
    is what a written model folder holds), for matrices, norm weights and the rounding to bfloat16."""
    from tiny_llm_amd.parts.base import WeightSpec
    from tiny_llm_amd.weights.loader import random_tensor
    for spec, std, nstd in ((WeightSpec("model.layers.0.mlp.up_proj.weight", (1031, 517)), 0.02, 0.0),
                            (WeightSpec("a.weight", (3, 5, 7)), 1.7, 0.0),
                            (WeightSpec("n.weight", (4099,), role="vector", init="ones"), 0.02, 0.1),
                            (WeightSpec("n.weight", (33,), role="vector", init="ones"), 0.02, 0.0),
                            (WeightSpec("big.weight", (3000, 2048)), 0.02, 0.0)):
        host = random_tensor(spec, 77, std, nstd, dtype=dtype)
        dev = random_tensor(spec, 77, std, nstd, device=DEV, dtype=dtype)
        assert dev.dtype == dtype and dev.shape == host.shape
        assert torch.equal(dev.cpu(), host), spec.name
    other = random_tensor(WeightSpec("a.weight", (3, 5, 7)), 78, 1.7, 0.0, device=DEV, dtype=dtype)
    assert not torch.equal(other.cpu(), random_tensor(WeightSpec("a.weight", (3, 5, 7)), 77, 1.7, 0.0, dtype=dtype))


def test_handover_probe_runs_and_its_waits_are_bounded():
    """The measurement of a hand-over among resident workgroups: values arrive right, a round takes
    microseconds; with a wait of one poll the kernel gives up instead of waiting, and still ends."""
    us = ops().peak_handover(workgroups=256, rounds=200, payload=16)
    assert 0.2 < us < 200.0
    assert ops().peak_handover(workgroups=8, rounds=50, payload=300) > 0.0
    try:
        ops().peak_handover(workgroups=256, rounds=50, payload=16, spin_limit=1)
    except ops().KernelError as e:
        assert "ran out" in str(e)
    torch.cuda.synchronize()
