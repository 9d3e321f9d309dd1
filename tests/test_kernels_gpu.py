"""Each HIP kernel alone against its plain PyTorch counterpart (tests/kernel_refs.py),
at sizes other than the engine's tiny models: widths and vocabularies that are no
powers of two, several head sizes and group counts, ragged batches, pages out of order.
"""
import math
import types

import numpy as np
import pytest
import torch

import kernel_refs as R
from yalis_amd.engine.batch import SeqSpan, attention_tiles, attention_token_columns, build_host_batch, named_arrays

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from yalis_amd.ops.hip import HipOps

    return HipOps(DEV)


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def device_cache(ops, kc, vc):
    """Pages written in the plain order -> what the kernels expect, on the GPU."""
    if ops.cache_tiled(kc.dtype, kc.shape[3], kc.shape[2]):
        kc, vc = R.tile_cache(kc.cpu(), vc.cpu())
    return kc.to(DEV), vc.to(DEV)


def plain_cache(ops, kc, vc):
    """Pages as the kernels keep them -> the plain order, on the CPU."""
    if ops.cache_tiled(kc.dtype, kc.shape[3], kc.shape[2]):
        return R.untile_cache(kc.cpu(), vc.cpu())
    return kc.cpu(), vc.cpu()


def close(got, want, atol, rtol=0.0):
    got = got.float().cpu()
    want = want.float().cpu()
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert torch.isfinite(got).all(), "kernel produced non-finite values"
    assert (err <= bound).all(), f"max err {err.max().item():.3e} (bound {bound.min().item():.3e})"


# ------------------------------------------------------------------------- embedding
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed(ops, dtype):
    table = rnd((515, 192), dtype, 0)
    ids = torch.tensor([0, 514, 3, 3, 77, 200], dtype=torch.int32, device=DEV)
    got = ops.embed(ids, table)
    assert got.dtype == torch.float32
    assert torch.equal(got.cpu(), R.embed(ids.cpu(), table.cpu()))


# ------------------------------------------------------------------------------ norm
# (from 1,024 rows on a thread of the fast form holds two pieces of its row)
@pytest.mark.parametrize("width,rows", [(192, 7), (4096, 33), (1000, 3), (6144, 2), (3080, 1030), (72, 1025)])
@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm(ops, width, rows, act, wdtype):
    res = rnd((rows, width), torch.float32, 1)
    res[0] *= 1e-4  # a near-zero row: eps matters
    delta = rnd((rows, width), act, 2)
    w = (1 + 0.1 * rnd((width,), torch.float32, 3)).to(wdtype)
    for eps, unit in ((1e-5, False), (1e-6, True)):
        for d in (delta, None):
            r_gpu = res.clone()
            r_ref = res.clone().cpu()
            got = ops.add_rmsnorm(r_gpu, d, w, eps, unit, act)
            want = R.add_rmsnorm(r_ref, None if d is None else d.cpu(), w.cpu(), eps, unit, torch.float32)
            close(r_gpu, r_ref, 1e-6)
            if act == torch.float32:
                close(got, want, 2e-5, 2e-5)
            else:
                close(got, want, 1e-3, 2**-8)


@pytest.mark.parametrize("width", [192, 4096, 1001])
@pytest.mark.parametrize("tdtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_starts_from_embedding_rows(ops, width, tdtype):
    """The first norm gathers the embedding's rows itself: the residual it leaves and the
    normed rows are those of the embedding kernel followed by the norm."""
    table = rnd((515, width), tdtype, 70)
    ids = torch.tensor([0, 514, 3, 3, 77, 200, 1], dtype=torch.int32, device=DEV)
    w = rnd((width,), tdtype, 71) + 1
    res_a = ops.embed(ids, table)
    out_a = ops.add_rmsnorm(res_a, None, w, 1e-5, False, torch.bfloat16)
    res_b, rows = ops.embedded_rows(ids, table)
    res_b.fill_(float("nan"))  # never read
    out_b = ops.add_rmsnorm(res_b, rows, w, 1e-5, False, torch.bfloat16)
    assert torch.equal(res_a, res_b) and torch.equal(out_a, out_b)
    assert torch.equal(rows.gather(), res_a)


def test_gather_add_rmsnorm(ops):
    res = rnd((20, 320), torch.float32, 1)
    delta = rnd((20, 320), torch.bfloat16, 2)
    w = rnd((320,), torch.bfloat16, 3)
    rows = torch.tensor([19, 0, 7, 7], dtype=torch.int32, device=DEV)
    keep = res.clone()
    got = ops.gather_add_rmsnorm(res, delta, rows, w, 1e-5, False, torch.float32)
    want = R.gather_add_rmsnorm(keep.cpu(), delta.cpu(), rows.cpu(), w.cpu(), 1e-5, False, torch.float32)
    assert torch.equal(res, keep), "the gathered form must not change the residual"
    close(got, want, 2e-5, 2e-5)


# ------------------------------------------------------------------------------ gemm
@pytest.mark.parametrize("m,n,k", [(5, 37, 19), (70, 130, 100), (1, 515, 192), (64, 64, 64), (129, 65, 33)])
@pytest.mark.parametrize("xd,wd,od", [
    (torch.float32, torch.float32, torch.float32),
    (torch.bfloat16, torch.float32, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16, torch.float32),
    (torch.float32, torch.bfloat16, torch.float32),
])
def test_gemm_fma(ops, m, n, k, xd, wd, od):
    x = rnd((m, k), xd, 4)
    w = rnd((n, k), wd, 5)
    got = ops.gemm_fma(x, w, od)
    want = x.double().cpu() @ w.double().cpu().T
    if od == torch.float32:
        close(got, want, 1e-5 * math.sqrt(k), 1e-5)
    else:
        close(got, want, 1e-3, 2**-8)


def test_gemm_fma_is_true_float32(ops):
    """Inputs that a reduced-precision matrix mode would truncate: 1 + 2^-12 has more
    mantissa bits than bfloat16 (8) or a 10-bit tensor-float mode keep, and every partial
    sum of its squares is still exact enough in float32."""
    k = 64
    x = torch.full((4, k), 1.0 + 2.0**-12, device=DEV)
    w = torch.full((8, k), 1.0 + 2.0**-12, device=DEV)
    got = ops.gemm_fma(x, w, torch.float32)
    want = k * (1.0 + 2.0**-12) ** 2  # 64.03125...; truncated inputs would give 64
    assert abs(got[0, 0].item() - want) < 2e-5


@pytest.mark.parametrize("m,n,k", [
    (1, 96, 64), (3, 515, 192), (16, 100, 200), (17, 64, 4096), (33, 130, 72), (64, 520, 328),
    (8, 4096, 4096), (100, 515, 192), (1, 16, 8),
])
@pytest.mark.parametrize("od", [torch.float32, torch.bfloat16])
def test_gemm_mfma_skinny(ops, m, n, k, od):
    x = rnd((m, k), torch.bfloat16, 6)
    w = rnd((n, k), torch.bfloat16, 7)
    got = ops.gemm_mfma_skinny(x, w, od)
    want = x.double().cpu() @ w.double().cpu().T
    if od == torch.float32:
        close(got, want, 2e-5 * math.sqrt(k), 1e-5)
    else:
        close(got, want, 1e-2, 2**-8)


@pytest.fixture
def forced(ops):
    """``forced(chunk=, waves=, slices=)`` forces the few-row product's plan for one test."""
    yield ops.force_skinny_plan
    ops.force_skinny_plan()


@pytest.mark.parametrize("chunk", [128, 256])
def test_gemm_mfma_skinny_chunk_lengths(ops, chunk, forced):
    """The few-row product walks K in chunks of 256 or 128, chosen by the length of a
    workgroup's slice; here each length is forced in turn on every row-tile count, on split
    and unsplit products, on K that is no multiple of the chunk, and on the fused activation."""
    forced(chunk=chunk)
    for m, n, k in [(8, 200, 4096), (3, 515, 200), (24, 130, 2056), (40, 96, 1000), (64, 520, 328), (100, 64, 4096)]:
        x = rnd((m, k), torch.bfloat16, 6)
        w = rnd((n, k), torch.bfloat16, 7)
        close(ops.gemm_mfma_skinny(x, w, torch.float32), x.double().cpu() @ w.double().cpu().T, 2e-5 * math.sqrt(k), 1e-5)
    for m, k, inter in [(8, 4096, 512), (30, 392, 200), (64, 1024, 264)]:
        x = rnd((m, k), torch.bfloat16, 30, 0.7)
        packed, group = ops.pack_gate_up(rnd((inter, k), torch.bfloat16, 31, 0.05), rnd((inter, k), torch.bfloat16, 32, 0.05))
        got = ops.gate_up_act(x, packed, group, "silu", torch.bfloat16)
        assert torch.equal(got, ops.gated_act(ops.linear(x, packed, torch.bfloat16), "silu", torch.bfloat16, group=group))


def test_gemm_mfma_skinny_eight_waves(ops, forced):
    """With more than 32 rows of x a workgroup may have eight waves (128 weight rows on one
    staged copy of x): the same sums in the same order as with four, so the same bits, on
    sizes that are no multiples of the workgroup's rows or of the chunk, split and unsplit,
    plain and with the activation in the epilogue.  Eight waves asked for with fewer rows of
    x are four."""
    for m, n, k in [(64, 200, 4096), (50, 515, 328), (40, 1040, 2056), (33, 96, 1000)]:
        x = rnd((m, k), torch.bfloat16, 6)
        w = rnd((n, k), torch.bfloat16, 7)
        for slices in (1, 3):
            forced(waves=4, slices=slices)
            four = ops.gemm_mfma_skinny(x, w, torch.float32)
            forced(waves=8, slices=slices)
            eight = ops.gemm_mfma_skinny(x, w, torch.float32)
            assert torch.equal(four, eight), (m, n, k, slices)
            close(eight, x.double().cpu() @ w.double().cpu().T, 2e-5 * math.sqrt(k), 1e-5)
    x = rnd((64, 1024), torch.bfloat16, 30, 0.7)
    packed, group = ops.pack_gate_up(rnd((264, 1024), torch.bfloat16, 31, 0.05), rnd((264, 1024), torch.bfloat16, 32, 0.05))
    forced(waves=8)
    got = ops.gate_up_act(x, packed, group, "silu", torch.bfloat16)
    assert torch.equal(got, ops.gated_act(ops.linear(x, packed, torch.bfloat16), "silu", torch.bfloat16, group=group))
    few = rnd((8, 1024), torch.bfloat16, 33)
    eight = ops.gemm_mfma_skinny(few, packed, torch.float32)
    forced(waves=4)
    assert torch.equal(eight, ops.gemm_mfma_skinny(few, packed, torch.float32))


def test_gemm_mfma_skinny_two_chunks_in_flight(ops, forced):
    """Long slices of K with 33 to 64 rows of x and eight waves walk in short chunks, two in
    flight per wave (a register set each, by turns): the same sums in the same order as one
    long chunk at a time, so the same bits; slices of an even and of an odd number of chunks,
    K no multiple of the chunk, the last slice shorter, one chunk only in a slice."""
    for m, n, k, slices in [(64, 200, 16384, 2), (48, 136, 4096 + 2600, 1), (33, 520, 3 * 4224 + 72, 3), (64, 96, 4352, 1), (40, 130, 4200, 1)]:
        x = rnd((m, k), torch.bfloat16, 6)
        w = rnd((n, k), torch.bfloat16, 7)
        forced(waves=8, slices=slices)
        two = ops.gemm_mfma_skinny(x, w, torch.float32)   # the rule's own choice for these slices
        forced(waves=8, slices=slices, chunk=256)
        one = ops.gemm_mfma_skinny(x, w, torch.float32)
        forced(waves=4, slices=slices, chunk=128)
        four = ops.gemm_mfma_skinny(x, w, torch.float32)
        assert torch.equal(two, one) and torch.equal(two, four), (m, n, k, slices)
        close(two, x.double().cpu() @ w.double().cpu().T, 2e-5 * math.sqrt(k), 1e-5)


@pytest.mark.parametrize("chunk", [128, 256])
@pytest.mark.parametrize("waves", [4, 8])
def test_gemm_mfma_skinny_wide_form(ops, forced, chunk, waves):
    """33 to 64 rows of x in the wide form (32 x 32 x 16 products, a wave owns 32 weight rows),
    forced here on every shape: sizes that are no multiples of a wave's 32 rows, of the chunk or
    of 64 rows of x, one-hot operands that name the element every lane must hold, split and
    unsplit, float32 and bfloat16 results, the activation in the epilogue (with a last tile
    that holds one gate/up pair only); by the library's own rule it is taken at an unsliced K of 8,192."""
    try:
        ops.wide_skinny_products(2)
        forced(chunk=chunk, waves=waves)
        for m, n, k in [(64, 200, 4096), (50, 515, 328), (40, 1040, 2056), (33, 96, 1000), (100, 72, 520)]:
            x = rnd((m, k), torch.bfloat16, 6)
            w = rnd((n, k), torch.bfloat16, 7)
            want = x.double().cpu() @ w.double().cpu().T
            for slices in (1, 3):
                forced(chunk=chunk, waves=waves, slices=slices)
                close(ops.gemm_mfma_skinny(x, w, torch.float32), want, 2e-5 * math.sqrt(k), 1e-5)
                part = ops.linear(x, w, torch.bfloat16, partial_ok=True)
                close(part.reduce() if hasattr(part, "reduce") else part, want, 2e-2, 2**-7)
            forced(chunk=chunk, waves=waves)
        m, n, k = 40, 48, 64
        for kk in (0, 7, 8, 15, 16, 40, 63):
            x = torch.zeros((m, k), dtype=torch.bfloat16, device=DEV)
            w = torch.zeros((n, k), dtype=torch.bfloat16, device=DEV)
            x[:, kk] = torch.arange(1, m + 1, dtype=torch.bfloat16)
            w[:, kk] = torch.arange(1, n + 1, dtype=torch.bfloat16) * 0.5
            got = ops.gemm_mfma_skinny(x, w, torch.float32).cpu()
            assert torch.equal(got, torch.outer(torch.arange(1, m + 1).float(), torch.arange(1, n + 1).float() * 0.5)), f"k={kk}"
        for inter in (264, 512, 40):  # 528, 1024 and 80 rows of gate/up: the last tile is half, none, half
            x = rnd((64, 1024), torch.bfloat16, 30, 0.7)
            packed, group = ops.pack_gate_up(rnd((inter, 1024), torch.bfloat16, 31, 0.05), rnd((inter, 1024), torch.bfloat16, 32, 0.05))
            got = ops.gate_up_act(x[:50], packed, group, "silu", torch.bfloat16)
            plain = ops.gated_act(ops.linear(x[:50], packed, torch.bfloat16), "silu", torch.bfloat16, group=group)
            assert torch.equal(got, plain), inter
            ops.wide_skinny_products(0)
            assert torch.equal(got, ops.gate_up_act(x[:50], packed, group, "silu", torch.bfloat16))
            ops.wide_skinny_products(2)
        ops.wide_skinny_products(1)
        forced()
        forced(slices=1)
        x, w = rnd((48, 8192), torch.bfloat16, 8, 0.3), rnd((136, 8192), torch.bfloat16, 9, 0.05)
        by_rule = ops.gemm_mfma_skinny(x, w, torch.float32)
        close(by_rule, x.double().cpu() @ w.double().cpu().T, 2e-5 * math.sqrt(8192), 1e-5)
        # with more than 48 rows of x the rule keeps two long chunks in flight per wave: the same
        # bits as one at a time (a forced chunk length), on a K of an odd number of chunks and a tail
        for m, k in ((64, 8192 + 256 + 72), (49, 8192)):
            x, w = rnd((m, k), torch.bfloat16, 8, 0.3), rnd((136, k), torch.bfloat16, 9, 0.05)
            forced(slices=1)
            two = ops.gemm_mfma_skinny(x, w, torch.float32)
            forced(slices=1, chunk=256)
            assert torch.equal(two, ops.gemm_mfma_skinny(x, w, torch.float32))
            close(two, x.double().cpu() @ w.double().cpu().T, 2e-5 * math.sqrt(k), 1e-5)
            packed, group = ops.pack_gate_up(rnd((72, k), torch.bfloat16, 31, 0.05), rnd((72, k), torch.bfloat16, 32, 0.05))
            forced()
            got = ops.gate_up_act(x, packed, group, "silu", torch.bfloat16)
            forced(chunk=256)
            assert torch.equal(got, ops.gate_up_act(x, packed, group, "silu", torch.bfloat16))
        forced()
    finally:
        ops.wide_skinny_products(1)


def test_gemm_tile(ops):
    """The product in tiles of 128 x 128 for some dozens to a few hundred rows: sizes that are no
    multiples of the tile or of the step of 64 along K, one-hot operands, K cut into 1 to 8 slices
    (an odd number of steps in a slice, a last slice shorter than the others), float32 and
    bfloat16 results, slices kept for a consumer; and where ``linear`` takes it by itself."""
    from yalis_amd.ops.hip import SplitSum

    try:
        for m, n, k in [(65, 200, 4096), (128, 128, 64), (130, 515, 328), (256, 1040, 2056), (200, 96, 1000), (300, 136, 8192), (1, 8, 8)]:
            x = rnd((m, k), torch.bfloat16, 6)
            w = rnd((n, k), torch.bfloat16, 7)
            want = x.double().cpu() @ w.double().cpu().T
            for slices in (0, 1, 2, 3, 8):
                ops.force_tile_slices(slices)
                close(ops.gemm_tile(x, w, torch.float32), want, 2e-5 * math.sqrt(k), 1e-5)
                part = ops.gemm_tile(x, w, torch.bfloat16, partial_ok=True)
                if isinstance(part, SplitSum):
                    assert part.out_dtype == torch.bfloat16 and 1 < part.n_splits <= max(slices, 8)
                    close(part.reduce(), want, 2e-2, 2**-7)
                    res = rnd((m, n), torch.float32, 8)
                    got = ops.add_rmsnorm(res.clone(), part, torch.ones(n, device=DEV), 1e-5, False, torch.float32)
                    part = ops.gemm_tile(x, w, torch.bfloat16, partial_ok=True)
                    summed = part.tensor[0].clone()  # the consumers add the slices one after the other
                    for sl in range(1, part.n_splits):
                        summed += part.tensor[sl]
                    plain = ops.add_rmsnorm(res.clone(), summed.to(torch.bfloat16), torch.ones(n, device=DEV), 1e-5, False, torch.float32)
                    assert torch.equal(got, plain), "the slices' consumers round their sum as the product's output would have been"
                else:
                    close(part, want, 2e-2, 2**-7)
        ops.force_tile_slices(0)
        m, n, k = 150, 140, 128
        for kk in (0, 7, 8, 15, 16, 63, 64, 127):
            x = torch.zeros((m, k), dtype=torch.bfloat16, device=DEV)
            w = torch.zeros((n, k), dtype=torch.bfloat16, device=DEV)
            x[:, kk] = torch.arange(1, m + 1, dtype=torch.bfloat16)
            w[:, kk] = torch.arange(1, n + 1, dtype=torch.bfloat16) * 0.5
            got = ops.gemm_tile(x, w, torch.float32).cpu()
            assert torch.equal(got, torch.outer(torch.arange(1, m + 1).float(), torch.arange(1, n + 1).float() * 0.5)), f"k={kk}"
        # rows of x and w with gaps between them
        xs, wsrc = rnd((100, 4096 + 16), torch.bfloat16, 9), rnd((72, 4096 + 8), torch.bfloat16, 10)
        close(ops.gemm_tile(xs[:, :4096], wsrc[:, :4096], torch.float32), xs[:, :4096].double().cpu() @ wsrc[:, :4096].double().cpu().T, 2e-5 * 64, 1e-5)
        # a down projection of 65 to 256 rows is this kernel's by linear's own choice
        assert ops.long_matrix_tiles(128, 4096, 14336) and not ops.long_matrix_tiles(64, 4096, 14336)
        assert not ops.long_matrix_tiles(300, 4096, 14336) and not ops.long_matrix_tiles(128, 4096, 4096)
        x, w = rnd((100, 4096), torch.bfloat16, 11, 0.3), rnd((520, 4096), torch.bfloat16, 12, 0.05)
        y = ops.linear(x, w, torch.bfloat16, partial_ok=True)
        assert isinstance(y, SplitSum)
        close(y.reduce(), x.double().cpu() @ w.double().cpu().T, 2e-2, 2**-7)
        close(ops.linear(x, w, torch.bfloat16), x.double().cpu() @ w.double().cpu().T, 2e-2, 2**-7)
    finally:
        ops.force_tile_slices(0)


def test_forced_slice_counts_reach_the_consumers(ops, forced):
    """The number of K slices a product leaves behind is what the launch says it wrote, also
    when the plan is forced after the library was first asked about the shape."""
    from yalis_amd.ops.hip import SplitSum

    x, w = rnd((8, 4096), torch.bfloat16, 61), rnd((520, 4096), torch.bfloat16, 62)
    want = x.double().cpu() @ w.double().cpu().T
    auto = ops.linear(x, w, torch.bfloat16, partial_ok=True)
    for slices in (1, 3, 16):
        forced(slices=slices)
        y = ops.linear(x, w, torch.bfloat16, partial_ok=True)
        assert (y.n_splits if isinstance(y, SplitSum) else 1) == slices
        close(y.reduce() if isinstance(y, SplitSum) else y, want, 2e-2, 2**-7)
    forced()
    again = ops.linear(x, w, torch.bfloat16, partial_ok=True)
    assert (again.n_splits if isinstance(again, SplitSum) else 1) == (auto.n_splits if isinstance(auto, SplitSum) else 1)
    with pytest.raises(Exception, match="128 or 256"):
        forced(chunk=100)


def test_gemm_mfma_operand_order(ops):
    """One-hot operands name the element each lane must hold: y[m, n] = x[m, kx] * w[n, kx]
    for a single k picks out any mismatch between the two operands' k order."""
    m, n, k = 16, 16, 64
    for kk in (0, 7, 8, 31, 32, 63):
        x = torch.zeros((m, k), dtype=torch.bfloat16, device=DEV)
        w = torch.zeros((n, k), dtype=torch.bfloat16, device=DEV)
        x[:, kk] = torch.arange(1, m + 1, dtype=torch.bfloat16)
        w[:, kk] = torch.arange(1, n + 1, dtype=torch.bfloat16) * 0.5
        got = ops.gemm_mfma_skinny(x, w, torch.float32).cpu()
        want = torch.outer(torch.arange(1, m + 1).float(), torch.arange(1, n + 1).float() * 0.5)
        assert torch.equal(got, want), f"k={kk}"


def test_split_sums_feed_their_consumers(ops):
    """A few-row product may stay as unreduced K slices; norm, rotary + append and the
    gated activation add them up themselves, round the sum as the product's output would
    have been rounded, and so give the same bits as the reduced path."""
    from yalis_amd.ops.hip import SplitSum

    m, k = 5, 4096
    x = rnd((m, k), torch.bfloat16, 20, 0.5)
    w = rnd((256, k), torch.bfloat16, 21, 0.05)
    part = ops.linear(x, w, torch.bfloat16, partial_ok=True)
    assert isinstance(part, SplitSum) and part.n_splits > 1, "this shape was meant to split K"
    assert part.out_dtype == torch.bfloat16
    # (the slices live in the library's workspace until the next product; a copy of this test's
    # own can be fed to every consumer below)
    part = SplitSum(part.tensor.clone(), part.out_dtype)
    full = part.tensor.sum(0)
    assert (full.cpu() - (x.double().cpu() @ w.double().cpu().T).float()).abs().max() < 1e-3
    reduced = ops.linear(x, w, torch.bfloat16)  # the same slices, summed and rounded by the product
    assert torch.equal(part.reduce(), reduced.float())
    # norm
    res = rnd((m, 256), torch.float32, 22)
    nw = (1 + 0.1 * rnd((256,), torch.float32, 23)).to(torch.bfloat16)
    r1, r2 = res.clone(), res.clone()
    got = ops.add_rmsnorm(r1, part, nw, 1e-5, False, torch.bfloat16)
    want = ops.add_rmsnorm(r2, reduced, nw, 1e-5, False, torch.bfloat16)
    assert torch.equal(r1, r2) and torch.equal(got, want)
    close(r1, res.cpu() + full.cpu(), 1e-2, 2**-7)
    rows = torch.tensor([4, 0], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.gather_add_rmsnorm(res, part, rows, nw, 1e-5, False, torch.float32),
                       ops.gather_add_rmsnorm(res, reduced, rows, nw, 1e-5, False, torch.float32))
    # gated activation
    assert torch.equal(ops.gated_act(part, "silu", torch.bfloat16), ops.gated_act(reduced, "silu"))
    close(ops.gated_act(part, "silu", torch.float32), R.gated_act(reduced.float().cpu(), "silu"), 1e-5, 1e-5)
    # rotary + append: 2 query heads, 1 kv head of 64 -> 256 columns
    cos, sin = _tables(64, 100)
    positions = torch.tensor([3, 4, 50, 0, 99], dtype=torch.int32, device=DEV)
    slots = torch.tensor([5, 6, 40, 0, 63], dtype=torch.int32, device=DEV)
    kc = torch.zeros((4, 1, 16, 64), dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros((4, 1, 64, 16), dtype=torch.bfloat16, device=DEV)
    q = ops.rope_append(part, 2, 1, 64, positions, cos, sin, 64, False, kc, vc, slots, 16)
    assert q.shape == (m, 128) and q.dtype == torch.bfloat16
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q2 = ops.rope_append(reduced.clone(), 2, 1, 64, positions, cos, sin, 64, False, kc2, vc2, slots, 16)
    assert torch.equal(q, q2[:, :128]) and torch.equal(kc, kc2) and torch.equal(vc, vc2)
    kr, vr = torch.zeros((4, 1, 16, 64)), torch.zeros((4, 1, 64, 16))
    ref2 = full.clone().cpu()
    R.rope_append(ref2, 2, 1, 64, positions.cpu(), cos.cpu(), sin.cpu(), 64, False, kr, vr, slots.cpu(), 16)
    close(q, ref2[:, :128], 1e-2, 2**-7)
    close(kc, kr, 1e-2, 2**-7)
    close(vc, vr, 1e-2, 2**-7)
    # slices of a product asked for in float32 are added without rounding
    part32 = ops.linear(x, w, torch.float32, partial_ok=True)
    assert isinstance(part32, SplitSum) and part32.out_dtype == torch.float32
    r3 = res.clone()
    ops.add_rmsnorm(r3, part32, nw, 1e-5, False, torch.bfloat16)
    close(r3, res.cpu() + full.cpu(), 2e-6, 2e-6)


@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("m,k,inter", [(1, 4096, 1024), (8, 512, 2048), (40, 320, 520), (64, 4096, 14336 // 4),
                                       (5, 8192, 64), (70, 256, 328), (9, 192, 100)])
def test_gate_up_act(ops, act, m, k, inter):
    """Both projections and the activation: as one kernel where the product has few rows and
    is not split over K, else product + activation kernel over the packed columns; the
    same bits either way, and the plain arithmetic on [gate; up] within rounding."""
    x = rnd((m, k), torch.bfloat16, 30, 0.7)
    wg = rnd((inter, k), torch.bfloat16, 31, 0.05)
    wu = rnd((inter, k), torch.bfloat16, 32, 0.05)
    packed, group = ops.pack_gate_up(wg, wu)
    assert group == (8 if inter % 8 == 0 else 0) and packed.shape == (2 * inter, k)
    got = ops.gate_up_act(x, packed, group, act, torch.bfloat16)
    assert got.shape == (m, inter)
    # product, then the activation kernel on the packed columns
    gu = ops.linear(x, packed, torch.bfloat16)
    two_steps = ops.gated_act(gu, act, torch.bfloat16, group=group)
    assert torch.equal(got, two_steps)
    gate = (x.double().cpu() @ wg.double().cpu().T).to(torch.bfloat16)
    up = (x.double().cpu() @ wu.double().cpu().T).to(torch.bfloat16)
    want = R.gated_act(torch.cat([gate, up], dim=1).float(), act)
    close(got, want, 3e-2, 2**-7)
    # float32 weights are never packed
    assert ops.pack_gate_up(wg.float(), wu.float())[1] == 0


def test_gated_act_grouped_columns(ops):
    gu = rnd((7, 2 * 72), torch.bfloat16, 33, 2.0)
    for group in (0, 4, 8, 24):
        close(ops.gated_act(gu, "silu", group=group), R.gated_act(gu.float().cpu(), "silu", group=group), 1e-2, 2**-7)
    part = rnd((3, 7, 2 * 72), torch.float32, 34, 1.0)
    from yalis_amd.ops.hip import SplitSum
    close(ops.gated_act(SplitSum(part, torch.bfloat16), "silu", torch.bfloat16, group=8),
          R.gated_act(part.sum(0).to(torch.bfloat16).float().cpu(), "silu", group=8), 1e-2, 2**-7)


def test_linear_dispatch(ops):
    x = rnd((200, 192), torch.bfloat16, 8)
    w = rnd((515, 192), torch.bfloat16, 9)
    want = x.double().cpu() @ w.double().cpu().T
    close(ops.linear(x, w, torch.bfloat16), want, 1e-2, 2**-7)
    close(ops.linear(x, w, torch.float32), want, 1e-4, 1e-5)
    close(ops.linear(x[:5], w, torch.bfloat16), want[:5], 1e-2, 2**-7)
    # 65 to 192 rows where the vendor library would have few tiles: the few-row kernel, in row tiles of 64
    assert ops.few_library_tiles(100, 515) and not ops.few_library_tiles(200, 515) and not ops.few_library_tiles(128, 28672)
    assert ops.few_library_tiles(128, 4096) and not ops.few_library_tiles(128, 6144) and not ops.few_library_tiles(160, 4096)
    for rows in (65, 100, 128, 192):
        close(ops.linear(x[:rows], w, torch.bfloat16), want[:rows], 1e-2, 2**-7)
        part = ops.linear(x[:rows], w, torch.bfloat16, partial_ok=True)
        close(part.reduce() if hasattr(part, "reduce") else part, want[:rows], 1e-2, 2**-7)
    wf = w.float()
    close(ops.linear(x, wf, torch.bfloat16), want, 1e-2, 2**-7)


@pytest.mark.parametrize("tuned", [False, True])
def test_library_product(ops, tuned):
    """The vendor library's product, called directly: rows of x and w with gaps between them,
    both result types, shapes that are timed when first met (up to 256 rows) and shapes that are
    not, and the same values again from the kept plan."""
    ops.tune_library_products(tuned)
    try:
        for seed, (m, n, k, pad) in enumerate(((70, 520, 200, 0), (200, 1032, 136, 8), (300, 264, 512, 16), (129, 4096, 256, 0))):
            # (other leading dimensions for the two settings, so that each makes plans of its own)
            pad += 8 if tuned else 0
            xs = rnd((m, k + pad), torch.bfloat16, 50 + seed)
            wsrc = rnd((n, k + pad), torch.bfloat16, 60 + seed)
            x, w = xs[:, :k], wsrc[:, :k]
            want = x.double().cpu() @ w.double().cpu().T
            first = ops.gemm_library(x, w, torch.bfloat16)
            close(first, want, 1e-2, 2**-7)
            assert torch.equal(first, ops.gemm_library(x, w, torch.bfloat16))
            close(ops.gemm_library(x, w, torch.float32), want, 1e-4, 1e-5)
    finally:
        ops.tune_library_products(False)
    from yalis_amd.ops.hip import KernelError

    with pytest.raises(KernelError, match="gemm_library"):
        ops.gemm_library(rnd((70, 64), torch.float32, 1), rnd((64, 64), torch.bfloat16, 2), torch.bfloat16)


# ---------------------------------------------------------------- rotary + cache append
def _tables(rotary_dim, positions, theta=10000.0):
    inv = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2).float() / rotary_dim))
    ang = torch.outer(torch.arange(positions).float(), inv)
    return torch.cos(ang).to(DEV), torch.sin(ang).to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("h,g,d,rd,inter", [(4, 2, 16, 16, False), (6, 3, 64, 64, False), (8, 1, 128, 64, True), (3, 3, 48, 32, False), (5, 0, 32, 32, False)])
def test_rope_append(ops, dtype, h, g, d, rd, inter):
    n, page, n_pages = 37, 16, 9
    qkv = rnd((n, (h + 2 * g) * d), dtype, 10)
    cos, sin = _tables(rd, 200)
    positions = torch.randint(0, 200, (n,), generator=torch.Generator().manual_seed(1), dtype=torch.int32).to(DEV)
    slots = torch.randperm(page * n_pages, generator=torch.Generator().manual_seed(2))[:n].to(torch.int32).to(DEV)
    kc = torch.zeros((n_pages, max(g, 1), page, d), dtype=dtype, device=DEV)
    vc = torch.zeros((n_pages, max(g, 1), d, page), dtype=dtype, device=DEV)
    kc_r, vc_r, qkv_r = kc.cpu().clone(), vc.cpu().clone(), qkv.cpu().clone()
    if g == 0:
        ops.rope_append(qkv, h, 0, d, positions, cos, sin, rd, inter, None, None, None, page)
        R.rope_append(qkv_r, h, 0, d, positions.cpu(), cos.cpu(), sin.cpu(), rd, inter, None, None, None, page)
    else:
        ops.rope_append(qkv, h, g, d, positions, cos, sin, rd, inter, kc, vc, slots, page)
        R.rope_append(qkv_r, h, g, d, positions.cpu(), cos.cpu(), sin.cpu(), rd, inter, kc_r, vc_r, slots.cpu(), page)
    tol = 1e-6 if dtype == torch.float32 else 2**-7
    close(qkv.view(n, -1, d)[:, :h], qkv_r.view(n, -1, d)[:, :h], tol, tol)
    if g:
        close(kc, kc_r, tol, tol)
        assert torch.equal(vc.cpu(), vc_r), "values are copied, not changed"


@pytest.mark.parametrize("h,g,d,rd,page", [(8, 2, 128, 128, 64), (6, 3, 64, 32, 16), (4, 4, 48, 48, 32), (5, 1, 80, 16, 16), (6, 3, 64, 32, 128)])
def test_rope_append_prompt_portions(ops, h, g, d, rd, page):
    """Many bfloat16 tokens: portions whose slots run on from a multiple of 8 (values stored
    as 16-byte pieces), portions that start anywhere, scattered single tokens, a token count
    that is no multiple of 8; everything else in the pages stays as it was."""
    u = 64  # slots are laid out in units of 64 whatever the page size
    n_pages = 12 * u // page
    runs = [(3 * u, 40), (7 * u + 5, 19), (0, u), (9 * u + 8, 11)]  # (first slot, tokens)
    slots, positions = [], []
    for first, count in runs:
        slots += list(range(first, first + count))
        positions += list(range(first % 50, first % 50 + count))
    scattered = [5 * u + 3, 2 * u + 9, 11 * u + 1]
    slots += scattered
    positions += [190, 0, 77]
    n = len(slots)
    assert n % 8 != 0 and len(set(slots)) == n
    qkv = rnd((n, (h + 2 * g) * d), torch.bfloat16, 40)
    cos, sin = _tables(rd, 200)
    positions = torch.tensor(positions, dtype=torch.int32, device=DEV)
    slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
    kc_r, vc_r = rnd((n_pages, g, page, d), torch.bfloat16, 41).cpu(), rnd((n_pages, g, d, page), torch.bfloat16, 42).cpu()
    kc, vc = device_cache(ops, kc_r.clone(), vc_r.clone())
    qkv_r = qkv.cpu().clone()
    ops.rope_append(qkv, h, g, d, positions, cos, sin, rd, False, kc, vc, slots, page)
    R.rope_append(qkv_r, h, g, d, positions.cpu(), cos.cpu(), sin.cpu(), rd, False, kc_r, vc_r, slots.cpu(), page)
    close(qkv.view(n, -1, d)[:, :h], qkv_r.view(n, -1, d)[:, :h], 2**-7, 2**-7)
    kc_p, vc_p = plain_cache(ops, kc, vc)
    close(kc_p, kc_r, 2**-7, 2**-7)
    assert torch.equal(vc_p, vc_r), "values are copied, not changed"
    # the same rows one token at a time (the scalar kernel) give the same bits
    qkv1 = rnd((n, (h + 2 * g) * d), torch.bfloat16, 40)
    kc1, vc1 = device_cache(ops, rnd((n_pages, g, page, d), torch.bfloat16, 41), rnd((n_pages, g, d, page), torch.bfloat16, 42))
    for i in range(n):
        ops.rope_append(qkv1[i : i + 1], h, g, d, positions[i : i + 1], cos, sin, rd, False, kc1, vc1, slots[i : i + 1], page)
    assert torch.equal(qkv1.view(n, -1, d)[:, :h], qkv.view(n, -1, d)[:, :h]) and torch.equal(kc1, kc) and torch.equal(vc1, vc)


# ------------------------------------------------------------------------- attention
def _attention_case(ops, dtype, h, g, d, page, spans, window, seed, poison=True, n_pages=64, plan=None, long_plan=None, col_tiles=1, with_cols=False,
                    pool_pages=None):
    """spans: list of (cached tokens before the step, new tokens).  Builds pages in a
    shuffled order, fills cache for the earlier tokens, runs rope-free attention.
    pool_pages: the pages are the last n_pages of a pool of so many (never initialised below them)."""
    gen = torch.Generator().manual_seed(seed)
    order = torch.randperm(n_pages, generator=gen).tolist()
    kc = torch.zeros((n_pages, g, page, d), dtype=dtype)
    vc = torch.zeros((n_pages, g, d, page), dtype=dtype)
    if poison:
        kc.fill_(float("nan"))
        vc.fill_(float("nan"))
    seqs = []
    used = 0
    for cached, new in spans:
        total = cached + new
        n_p = -(-total // page)
        table = np.array(order[used : used + n_p], dtype=np.int32)
        used += n_p
        assert used <= n_pages
        k = torch.randn((total, g, d), generator=gen).to(dtype)
        v = torch.randn((total, g, d), generator=gen).to(dtype)
        for pos in range(total):
            kc[table[pos // page], :, pos % page, :] = k[pos]
            vc[table[pos // page], :, :, pos % page] = v[pos]
        seqs.append(SeqSpan(tokens=[0] * new, first_position=cached, block_tables=[table + (pool_pages - n_pages if pool_pages else 0)], state_slot=0))
    hb = build_host_batch(seqs, 1, page)
    tpt = ops.attention_tokens_per_tile(h, g)
    big = ops.attention_long_span_tile(h, g)
    big_c = ops.attention_long_span_tile(h, g, col_tiles)  # tokens of a long tile with col_tiles column tiles a wave
    arrays = named_arrays(hb, {"tiles": lambda b: attention_tiles(b, tpt, 1, big), "long_tiles": lambda b: attention_tiles(b, big_c, big + 1, longest_first=(seed % 2 == 0)),
                               "cols": lambda b: attention_token_columns(b, tpt, 1, big)})
    ctx = types.SimpleNamespace(
        arrays={k: torch.from_numpy(np.ascontiguousarray(v)).to(DEV) for k, v in arrays.items()},
        max_ctx=hb.max_ctx,
    )
    ctx_cpu = types.SimpleNamespace(arrays={k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in arrays.items()})
    n = hb.n_tokens
    q = (torch.randn((n, h * d), generator=gen) * 1.5).to(dtype)
    scale = 1.0 / math.sqrt(d)
    kc_d, vc_d = device_cache(ops, kc, vc)
    if pool_pages:
        pool_k = torch.empty((pool_pages,) + tuple(kc_d.shape[1:]), dtype=dtype, device=DEV)
        pool_v = torch.empty((pool_pages,) + tuple(vc_d.shape[1:]), dtype=dtype, device=DEV)
        pool_k[pool_pages - n_pages:] = kc_d
        pool_v[pool_pages - n_pages:] = vc_d
        kc_d, vc_d = pool_k, pool_v
    got = ops.attention(q.to(DEV), h, g, d, kc_d, vc_d, page, scale, window, ctx, 0, ctx.arrays["tiles"], ctx.arrays["long_tiles"], plan=plan, long_plan=long_plan, long_col_tiles=col_tiles,
                        token_cols=ctx.arrays["cols"] if with_cols else None)
    if pool_pages:
        return got, None  # (the plain implementation would need the pool on the host)
    want = R.attention(q.float(), h, g, d, kc.float(), vc.float(), page, scale, window, ctx_cpu, 0, None)
    return got, want


SPANS = [(0, 5), (17, 1), (0, 70), (63, 2), (100, 1), (31, 34), (0, 1)]


@pytest.mark.parametrize("h,g,d,page", [(4, 2, 16, 16), (4, 1, 32, 32), (6, 3, 48, 16), (5, 5, 80, 64), (2, 1, 256, 16)])
@pytest.mark.parametrize("window", [0, 24])
def test_attention_generic_f32(ops, h, g, d, page, window):
    got, want = _attention_case(ops, torch.float32, h, g, d, page, SPANS, window, seed=3)
    close(got, want, 2e-5, 1e-5)


@pytest.mark.parametrize("h,g,d,page", [(4, 2, 16, 16), (6, 3, 48, 32)])
def test_attention_generic_bf16(ops, h, g, d, page):
    got, want = _attention_case(ops, torch.bfloat16, h, g, d, page, SPANS, 0, seed=4)
    close(got, want, 1e-2, 2**-7)


@pytest.mark.parametrize("h,g,d,page", [
    (8, 2, 128, 64), (6, 3, 64, 16), (4, 4, 64, 32), (32, 1, 128, 16), (5, 1, 64, 48), (24, 8, 128, 64), (40, 2, 64, 16),
    (4, 4, 64, 128), (12, 3, 128, 192),
])
@pytest.mark.parametrize("window", [0, 40])
def test_attention_mfma(ops, h, g, d, page, window):
    got, want = _attention_case(ops, torch.bfloat16, h, g, d, page, SPANS, window, seed=5)
    close(got, want, 2e-2, 2**-6)


def test_attention_mfma_long_context_splits(ops):
    """Few waves and many keys: the launch splits the keys and merges the parts."""
    spans = [(1500, 1), (900, 3), (0, 2)]
    got, want = _attention_case(ops, torch.bfloat16, 8, 2, 128, 64, spans, 0, seed=6, n_pages=48)
    close(got, want, 2e-2, 2**-6)
    got, want = _attention_case(ops, torch.bfloat16, 8, 2, 128, 64, spans, 700, seed=6, n_pages=48)
    close(got, want, 2e-2, 2**-6)


@pytest.mark.parametrize("plan", [(1, 1), (4, 1), (1, 5), (4, 3), (4, 7)])
@pytest.mark.parametrize("d,page", [(64, 32), (128, 32), (64, 64), (128, 128)])
def test_attention_mfma_every_way_of_dividing_keys(ops, plan, d, page):
    """Keys divided among the waves of a workgroup, among workgroups, or both, give the
    same result; spans include ones with fewer key blocks than waves (idle waves hold
    an empty part) and windows that cut the first block.  Pages of 32 tokens are plain,
    those of 64 and 128 tiled."""
    spans = [(1500, 1), (900, 3), (0, 2), (63, 1), (64, 1), (200, 2)]
    for window in (0, 700, 33):
        got, want = _attention_case(ops, torch.bfloat16, 8, 2, d, page, spans, window, seed=16, n_pages=3072 // page + 6, plan=plan)
        close(got, want, 2e-2, 2**-6)


@pytest.mark.parametrize("plan", [(4, 2), (4, 5), (1, 3)])
@pytest.mark.parametrize("h,g,d,page", [(8, 2, 128, 64), (6, 3, 64, 32), (32, 8, 128, 64), (24, 8, 128, 64), (32, 1, 128, 32)])
def test_attention_splits_merged_by_the_product(ops, plan, h, g, d, page, monkeypatch):
    """A step of up to 16 tokens leaves its splits unmerged for the product that follows:
    merged on their own they are the attention's output, and the product fed by the splits
    gives the bits of the product fed by the merged tensor (tiles of 8, 4, 5 and 1 tokens;
    heads that need two chunks; a product that keeps its K slices, one that does not, and
    one whose K slices are too long, which merges first)."""
    import yalis_amd.ops.hip as hip_ops
    from yalis_amd.ops.hip import SplitAttention, SplitSum

    monkeypatch.setattr(hip_ops, "MERGE_IN_PRODUCT_MAX_TOKENS", 16)  # as far as the kernel goes, not as far as it pays
    spans = [(700, 1), (64, 2), (300, 1), (0, 3), (1500, 1), (63, 2)]
    plain, _ = _attention_case(ops, torch.bfloat16, h, g, d, page, spans, 0, seed=21, n_pages=2700 // page + 8, plan=plan)
    # (the unmerged splits live in the library's workspace until the next attention: made last)
    got, want = _attention_case(ops, torch.bfloat16, h, g, d, page, spans, 0, seed=21, n_pages=2700 // page + 8, plan=plan, with_cols=True)
    assert isinstance(got, SplitAttention) and got.n_splits == plan[1] and got.shape == (10, h * d)
    merged = got.merge()
    close(merged, want, 2e-2, 2**-6)
    assert torch.equal(plain, merged)
    fed = 0
    for n_out, out_dtype, partial_ok in ((h * d, torch.bfloat16, True), (515, torch.float32, False), (48, torch.bfloat16, True)):
        w = rnd((n_out, h * d), torch.bfloat16, 22)
        fed += bool(ops._ask("yk_gemm_skinny_from_attention_ok", 10, n_out, h * d))
        y = ops.linear(got, w, out_dtype, partial_ok=partial_ok)
        a = y.tensor.clone() if isinstance(y, SplitSum) else y.clone()
        y = ops.linear(merged, w, out_dtype, partial_ok=partial_ok)
        b = y.tensor if isinstance(y, SplitSum) else y
        assert a.shape == b.shape and torch.equal(a, b), (n_out, out_dtype)
        close(a.sum(0) if partial_ok and a.dim() == 3 else a, merged.double().cpu() @ w.double().cpu().T, 3e-2, 2**-6)
    assert fed >= 1, "no product here took the splits itself"
    # more than 16 tokens: merged by the attention itself
    got, want = _attention_case(ops, torch.bfloat16, h, g, d, page, spans + [(5, 9)], 0, seed=21, n_pages=2700 // page + 8, plan=plan, with_cols=True)
    assert isinstance(got, torch.Tensor)
    close(got, want, 2e-2, 2**-6)


def _bits(t):
    return t.contiguous().view(torch.int16)


def _rotary_inside_cases():
    shapes = [(32, 8, 128, 128, 64, False), (6, 2, 128, 128, 64, False), (6, 3, 64, 32, 16, False), (8, 1, 64, 64, 128, True),
              (32, 1, 128, 64, 32, False), (24, 8, 128, 128, 64, False), (4, 4, 64, 0, 64, False)]
    for shape in shapes:
        for slices in (1, 3):
            for plan in (None, (1, 1), (4, 1), (4, 3), (1, 4)):
                yield (*shape, slices, plan, 0)
    # a window: its edge inside the block that holds the token, in an earlier block, in a split
    # that another workgroup owns; pages below it given back
    for shape in shapes[:4] + shapes[6:]:
        for window in (24, 100):
            for slices, plan in ((1, None), (3, (4, 3)), (1, (1, 4)), (3, (4, 1))):
                yield (*shape, slices, plan, window)


@pytest.mark.parametrize("h,g,d,rd,page,inter,slices,plan,window", list(_rotary_inside_cases()))
def test_attention_rotates_and_appends_in_its_launch(ops, plan, slices, h, g, d, rd, page, inter, window):
    """A step of single tokens: rotary + append inside the attention launch give the bits of
    rotary + append followed by attention, in the output and in the pages, whether the
    projection comes as bfloat16 rows or as float32 K slices, however the keys are divided,
    with the token's own key first, last or in the middle of a block of 64 (the slot it goes to
    holds NaN before), in tiled and in plain pages; and both agree with the plain reference.
    With a window: contexts one short of it, equal to it and beyond, the pages that lie wholly
    below the window given back (-1 in the block table, NaN where they were), and the key just
    outside the window made large, so that a window off by one would let it take the output."""
    from yalis_amd.ops.hip import RopeInLaunch, SplitSum

    cached = [0, 1, 31, 32, 63, 64, 65, 700, 1500, 127, 190]
    if window:
        cached += [window - 1, window, window + 1]
    n = len(cached)
    gen = torch.Generator().manual_seed(31)
    n_pages = sum(-(-(c + 1) // page) for c in cached) + 3
    order = torch.randperm(n_pages, generator=gen).tolist()
    kc = torch.full((n_pages, g, page, d), float("nan"), dtype=torch.bfloat16)
    vc = torch.full((n_pages, g, d, page), float("nan"), dtype=torch.bfloat16)
    seqs, used = [], 0
    for c in cached:
        n_p = -(-(c + 1) // page)
        table = np.array(order[used : used + n_p], dtype=np.int32)
        used += n_p
        k = torch.randn((c, g, d), generator=gen).to(torch.bfloat16)
        v = torch.randn((c, g, d), generator=gen).to(torch.bfloat16)
        first_seen = max(0, c - window + 1) if window else 0  # the oldest key the token at position c sees
        if window and first_seen > 0:
            k[first_seen - 1] *= 40.0  # just outside: were it seen, it would take half the heads' outputs
            table[: first_seen // page] = -1  # pages wholly below the window: given back, never filled
        for pos in range(c):
            if table[pos // page] >= 0:
                kc[table[pos // page], :, pos % page, :] = k[pos]
                vc[table[pos // page], :, :, pos % page] = v[pos]
        seqs.append(SeqSpan(tokens=[0], first_position=c, block_tables=[table], state_slot=0))
    hb = build_host_batch(seqs, 1, page)
    tpt, big = ops.attention_tokens_per_tile(h, g), ops.attention_long_span_tile(h, g)
    arrays = named_arrays(hb, {"tiles": lambda b: attention_tiles(b, tpt, 1, big), "cols": lambda b: attention_token_columns(b, tpt, 1, big)})
    dev = {k: torch.from_numpy(np.ascontiguousarray(v)).to(DEV) for k, v in arrays.items()}
    ctx = types.SimpleNamespace(arrays=dev, max_ctx=hb.max_ctx, max_qlen=1)
    cols = (h + 2 * g) * d
    if slices == 1:
        raw = (torch.randn((n, cols), generator=gen) * 1.2).to(torch.bfloat16).to(DEV)
        give = lambda: raw.clone()
        summed = raw.float().cpu()
    else:
        parts = (torch.randn((slices, n, cols), generator=gen) * 0.7).to(DEV)
        give = lambda: SplitSum(parts.clone(), torch.bfloat16)
        summed = (parts[0] + parts[1] + parts[2]).to(torch.bfloat16).float().cpu()
    cos, sin = _tables(rd, 1600) if rd else (None, None)
    scale = 1.0 / math.sqrt(d)
    positions, slots = dev["positions"], dev["slots_g0"]
    # rotary + append, then attention
    kc_a, vc_a = device_cache(ops, kc.clone(), vc.clone())
    q = ops.rope_append(give(), h, g, d, positions, cos, sin, rd, inter, kc_a, vc_a, slots, page)
    out_a = ops.attention(q, h, g, d, kc_a, vc_a, page, scale, window, ctx, 0, dev["tiles"], plan=plan)
    # both in one launch
    kc_b, vc_b = device_cache(ops, kc.clone(), vc.clone())
    out_b = ops.attention(give(), h, g, d, kc_b, vc_b, page, scale, window, ctx, 0, dev["tiles"], plan=plan,
                          rope=RopeInLaunch(cos, sin, rd, inter, True))
    assert torch.isfinite(out_b.float()).all()
    assert torch.equal(_bits(out_a), _bits(out_b))
    assert torch.equal(_bits(kc_a), _bits(kc_b)) and torch.equal(_bits(vc_a), _bits(vc_b))
    # queries only, against pages that already hold the tokens' keys and values (a run entry
    # that reads another entry's cache)
    q_rows = give()
    q_rows = SplitSum(q_rows.tensor[:, :, : h * d].contiguous(), torch.bfloat16) if slices > 1 else q_rows[:, : h * d].contiguous()
    out_c = ops.attention(q_rows, h, g, d, kc_b, vc_b, page, scale, window, ctx, 0, dev["tiles"], plan=plan,
                          rope=RopeInLaunch(cos, sin, rd, inter, False))
    assert torch.equal(_bits(out_a), _bits(out_c))
    # the plain reference
    qkv_r = summed.clone()
    kc_r, vc_r = kc.float(), vc.float()
    cpu = {k: torch.from_numpy(np.ascontiguousarray(v)) for k, v in arrays.items()}
    R.rope_append(qkv_r, h, g, d, cpu["positions"], None if cos is None else cos.cpu(), None if sin is None else sin.cpu(), rd, inter, kc_r, vc_r, cpu["slots_g0"], page)
    kc_r, vc_r = kc_r.to(torch.bfloat16).float(), vc_r.to(torch.bfloat16).float()
    q_r = qkv_r.view(n, -1, d)[:, :h].reshape(n, h * d).to(torch.bfloat16).float()
    want = R.attention(q_r, h, g, d, kc_r, vc_r, page, scale, window, types.SimpleNamespace(arrays=cpu), 0, None)
    close(out_b, want, 2e-2, 2**-6)


def test_attention_with_rotary_inside_leaves_splits_for_the_product(ops):
    """One or two tokens whose keys are split across workgroups: the launch with rotary inside
    leaves its splits unmerged too, and merged they are the two-kernel path's output."""
    from yalis_amd.ops.hip import RopeInLaunch, SplitAttention

    h, g, d, page = 32, 8, 128, 64
    gen = torch.Generator().manual_seed(5)
    cached = [1100, 300]
    n_pages = 30
    kc = torch.randn((n_pages, g, page, d), generator=gen).to(torch.bfloat16)
    vc = torch.randn((n_pages, g, d, page), generator=gen).to(torch.bfloat16)
    tables = [np.arange(0, 18, dtype=np.int32), np.arange(20, 25, dtype=np.int32)]
    seqs = [SeqSpan(tokens=[0], first_position=c, block_tables=[t], state_slot=0) for c, t in zip(cached, tables)]
    hb = build_host_batch(seqs, 1, page)
    tpt, big = ops.attention_tokens_per_tile(h, g), ops.attention_long_span_tile(h, g)
    arrays = named_arrays(hb, {"tiles": lambda b: attention_tiles(b, tpt, 1, big), "cols": lambda b: attention_token_columns(b, tpt, 1, big)})
    dev = {k: torch.from_numpy(np.ascontiguousarray(v)).to(DEV) for k, v in arrays.items()}
    ctx = types.SimpleNamespace(arrays=dev, max_ctx=hb.max_ctx, max_qlen=1)
    raw = torch.randn((2, (h + 2 * g) * d), generator=gen).to(torch.bfloat16).to(DEV)
    cos, sin = _tables(d, 1200)
    kc_a, vc_a = device_cache(ops, kc.clone(), vc.clone())
    q = ops.rope_append(raw.clone(), h, g, d, dev["positions"], cos, sin, d, False, kc_a, vc_a, dev["slots_g0"], page)
    out_a = ops.attention(q, h, g, d, kc_a, vc_a, page, 0.09, 0, ctx, 0, dev["tiles"], plan=(4, 4))
    kc_b, vc_b = device_cache(ops, kc.clone(), vc.clone())
    got = ops.attention(raw.clone(), h, g, d, kc_b, vc_b, page, 0.09, 0, ctx, 0, dev["tiles"], plan=(4, 4), token_cols=dev["cols"],
                        rope=RopeInLaunch(cos, sin, d, False, True))
    assert isinstance(got, SplitAttention)
    assert torch.equal(_bits(got.merge()), _bits(out_a)) and torch.equal(_bits(kc_a), _bits(kc_b)) and torch.equal(_bits(vc_a), _bits(vc_b))
    # refused for steps that hold more than single tokens
    ctx.max_qlen = 2
    with pytest.raises(Exception, match="single tokens"):
        ops.attention(raw.clone(), h, g, d, kc_b, vc_b, page, 0.09, 0, ctx, 0, dev["tiles"], rope=RopeInLaunch(cos, sin, d, False, True))


@pytest.mark.parametrize("col_tiles", [1, 2])
@pytest.mark.parametrize("splits", [1, 2, 5, 16])
@pytest.mark.parametrize("h,g,d,page", [(8, 2, 128, 64), (6, 3, 64, 16), (32, 1, 128, 32), (6, 2, 64, 128)])
def test_attention_long_spans_with_split_keys(ops, splits, h, g, d, page, col_tiles):
    """Portions of prompts against a long cached context, the keys split across workgroups
    and merged: spans that end a tile early, a window, more splits than some tiles have key
    blocks (empty parts); one and two column tiles per wave (tiles of twice the tokens)."""
    spans = [(900, 70), (0, 130), (1500, 33), (40, 100)]
    for window in (0, 300):
        got, want = _attention_case(ops, torch.bfloat16, h, g, d, page, spans, window, seed=18, n_pages=3000 // page + 8, long_plan=splits, col_tiles=col_tiles)
        close(got, want, 2e-2, 2**-6)


def test_attention_policies_keep_their_invariants():
    """What the launch policies must hold whatever their constants are: a plan has one or four
    waves and at least one split, never more waves than key blocks could feed; the long-span
    kernel gets one or two column tiles, and splits only as far as all workgroups stay on the
    GPU at once."""
    from yalis_amd.ops.hip import HipOps

    for groups in (1, 8, 64, 512, 5000):
        for key_blocks in (1, 2, 5, 16, 128, 2048):
            waves, splits = HipOps.attention_plan(groups, key_blocks)
            assert waves in (1, 4) and 1 <= splits <= 256
            assert key_blocks > 1 or (waves, splits) == (1, 1)
            assert waves * splits < 2 * 8 + key_blocks * 2
    for workgroups in (1, 8, 120, 256, 400, 1024, 5000):
        for fewest in (0, 512, 1024, 7000):
            assert HipOps.attention_long_col_tiles(workgroups, fewest) in (1, 2)
        for key_blocks in (1, 4, 20, 64, 400):
            for col_tiles in (1, 2):
                splits = HipOps.attention_long_splits(workgroups, key_blocks, col_tiles)
                assert 1 <= splits <= 16
                assert splits == 1 or (splits * workgroups <= (768 if col_tiles == 1 else 512) and key_blocks // splits >= 8)


@pytest.mark.parametrize("h,g,d,page", [(32, 8, 128, 64), (24, 8, 128, 64), (32, 8, 64, 64)])
def test_attention_gives_one_result_under_every_plan_its_policies_choose(ops, h, g, d, page):
    """The policies decide from the batch how the keys are divided (waves, splits, column tiles of
    the long-span kernel).  For workloads on which they decide differently, the result under the
    policy's own choice is, within rounding, the result with nothing divided and the plain
    reference's: retuning a policy can change speed only."""
    from yalis_amd.ops.hip import HipOps

    workloads = {
        "single tokens behind long contexts": [(2000, 1), (900, 1), (64, 1)],
        "a few tokens each": [(1500, 3), (0, 2), (700, 4)],
        "a portion behind a long cached context": [(1400, 200)],
        "a prompt from nothing": [(0, 300)],
        "portions beside single tokens": [(1100, 150), (600, 1), (0, 90), (1300, 1)],
    }
    seen = set()
    for what, spans in workloads.items():
        n_pages = sum(-(-(c + n) // page) for c, n in spans) + 2
        chosen, want = _attention_case(ops, torch.bfloat16, h, g, d, page, spans, 0, seed=30, n_pages=n_pages)
        undivided, _ = _attention_case(ops, torch.bfloat16, h, g, d, page, spans, 0, seed=30, n_pages=n_pages, plan=(1, 1), long_plan=1)
        two, _ = _attention_case(ops, torch.bfloat16, h, g, d, page, spans, 0, seed=30, n_pages=n_pages, col_tiles=2)
        close(chosen, want, 2e-2, 2**-6)
        close(undivided, want, 2e-2, 2**-6)
        close(two, want, 2e-2, 2**-6)
        # (the parts of a division are merged in float32 and rounded once: what a division can
        # change is the order of float32 sums, a unit of bfloat16 at most)
        close(chosen, undivided.float().cpu(), 2e-2, 2**-7)
        longest = max(c + n for c, n in spans)
        seen.add(HipOps.attention_plan(len(spans) * g, -(-longest // 64)))
    assert len(seen) > 1, "the workloads were meant to make the policy choose differently"


@pytest.mark.parametrize("dtype,h,g,d,page", [(torch.bfloat16, 32, 8, 128, 64), (torch.bfloat16, 6, 3, 64, 16), (torch.float32, 4, 2, 48, 32)])
def test_attention_in_a_pool_beyond_4_gib(ops, dtype, h, g, d, page):
    """Pages whose offsets in the pool do not fit 32 bits (a pool of more than 4 GiB of keys, and
    as much of values; more than 2^31 elements): the same bits as from the same pages at the
    start of a small pool, for single tokens, short and long spans, keys split and not."""
    free = torch.cuda.mem_get_info()[0]
    per_page = g * page * d * (2 if dtype == torch.bfloat16 else 4)
    pool_pages = (2**31 + 2**28) // (g * page * d)
    if free < 2.5 * pool_pages * per_page:
        pytest.skip("not enough free device memory for the pool")
    assert pool_pages * g * page * d > 2**31
    spans = [(0, 5), (17, 1), (0, 300), (63, 2), (700, 1), (31, 34), (200, 130)]
    for plan, long_plan in ((None, None), ((4, 3), 2)):
        small, want = _attention_case(ops, dtype, h, g, d, page, spans, 0, seed=5, plan=plan, long_plan=long_plan, n_pages=128)
        big, _ = _attention_case(ops, dtype, h, g, d, page, spans, 0, seed=5, plan=plan, long_plan=long_plan, n_pages=128, pool_pages=pool_pages)
        assert torch.equal(small, big)
        close(small, want, 2e-5 if dtype == torch.float32 else 2e-2, 0 if dtype == torch.float32 else 2**-7)
        torch.cuda.empty_cache()


def test_attention_far_key_stands_out(ops):
    """One far key gets a large score: if a kernel skipped or misplaced it, the output
    would be the average of the others instead of (almost exactly) that key's value."""
    h, g, d, page = 8, 2, 128, 64
    n_ctx = 777
    for dtype in (torch.bfloat16, torch.float32):
        gen = torch.Generator().manual_seed(11)
        kc = torch.zeros((16, g, page, d), dtype=dtype)
        vc = torch.zeros((16, g, d, page), dtype=dtype)
        table = np.arange(15, 15 - 13, -1).astype(np.int32)  # pages in reverse
        k = torch.randn((n_ctx, g, d), generator=gen) * 0.1
        v = torch.randn((n_ctx, g, d), generator=gen)
        far = 5  # an early key, hundreds of tokens back
        q = torch.randn((1, h * d), generator=gen) * 0.1
        k[far] = 0
        k[far, 0, :] = q.view(h, d)[1] * 200.0  # head 1 (group 0) loves key `far`
        for pos in range(n_ctx):
            kc[table[pos // page], :, pos % page, :] = k[pos].to(dtype)
            vc[table[pos // page], :, :, pos % page] = v[pos].to(dtype)
        span = SeqSpan(tokens=[0], first_position=n_ctx - 1, block_tables=[table], state_slot=0)
        hb = build_host_batch([span], 1, page)
        tpt = ops.attention_tokens_per_tile(h, g)
        arrays = named_arrays(hb, {"tiles": lambda b: attention_tiles(b, tpt)})
        ctx = types.SimpleNamespace(
            arrays={kk: torch.from_numpy(np.ascontiguousarray(vv)).to(DEV) for kk, vv in arrays.items()},
            max_ctx=hb.max_ctx,
        )
        kc_d, vc_d = device_cache(ops, kc, vc)
        got = ops.attention(q.to(dtype).to(DEV), h, g, d, kc_d, vc_d, page, 1.0 / math.sqrt(d), 0, ctx, 0, ctx.arrays["tiles"])
        head1 = got.view(h, d)[1].float().cpu()
        close(head1, v[far, 0].to(dtype).float(), 2e-2, 2**-6)


# ------------------------------------------------------------------------ activation
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["silu", "gelu_tanh"])
def test_gated_act(ops, dtype, act):
    gu = rnd((9, 2 * 328), dtype, 12, scale=3.0)
    got = ops.gated_act(gu, act)
    want = R.gated_act(gu.float().cpu(), act)
    if dtype == torch.float32:
        close(got, want, 1e-6, 1e-5)
    else:
        close(got, want, 1e-3, 2**-8)


# -------------------------------------------------------------------------- sampling
def test_argmax_lowest_index_on_ties(ops):
    logits = rnd((5, 1000), torch.float32, 13)
    logits[0, 17] = 50.0
    logits[0, 900] = 50.0
    logits[1, 999] = 60.0
    got = ops.argmax(logits).cpu()
    want = torch.argmax(logits.cpu(), dim=-1)
    assert got[0].item() == 17 and got[1].item() == 999
    assert torch.equal(got[2:].long(), want[2:])


def _sample(ops, logits, temperature, top_k, top_p, seed, draw, whole_row=False):
    rows = logits.shape[0]
    f = lambda v, dt: torch.full((rows,), v, dtype=dt, device=DEV)
    return ops.sample(
        logits, f(temperature, torch.float32), f(top_k, torch.int32), f(top_p, torch.float32),
        f(seed, torch.int32), torch.arange(draw, draw + rows, dtype=torch.int32, device=DEV), whole_row=whole_row,
    ).cpu()


def test_sample_matches_plain(ops):
    import plain_llama as P

    logits = rnd((1, 515), torch.float32, 14, scale=2.0)
    for temperature, top_k, top_p in [(0.7, 0, 1.0), (1.0, 5, 1.0), (1.3, 0, 0.8), (0.9, 50, 0.5), (0.0, 0, 1.0), (1.0, 1, 1.0), (1.0, 0, 0.0)]:
        for draw in range(20):
            got = _sample(ops, logits, temperature, top_k, top_p, 99, draw)[0].item()
            want = P.sample_token(logits[0].cpu(), temperature, top_k or None, top_p, 99, draw)
            assert got == want, (temperature, top_k, top_p, draw)


SAMPLE_SETTINGS = [(0.7, 0, 1.0), (1.0, 5, 1.0), (1.3, 0, 0.8), (0.9, 50, 0.5), (1.0, 1, 1.0), (1.0, 0, 0.0),
                   (0.8, 3000, 0.95), (1.0, 6000, 0.9), (2.0, 0, 0.999), (1.1, 700, 1.0), (0.6, 5000, 1.0)]


@pytest.mark.parametrize("vocab,kind", [(32003, "peaked"), (128256, "peaked"), (20000, "flat"), (9001, "ties")])
def test_sample_large_vocabulary_matches_plain(ops, vocab, kind):
    """Rows larger than the candidate store: peaked rows narrow down to a few tokens, a
    flat row under top_p alone and a row of thousands of equal logits fall back to the
    whole-row path; every way gives the plain implementation's token, and the forced
    whole-row path agrees."""
    import plain_llama as P

    gen = torch.Generator().manual_seed(vocab)
    if kind == "peaked":
        logits = torch.randn((1, vocab), generator=gen) * 3.0
    elif kind == "flat":
        logits = torch.randn((1, vocab), generator=gen) * 0.01
    else:
        logits = torch.randn((1, vocab), generator=gen).round()  # a handful of distinct values
    logits = logits.to(DEV)
    for temperature, top_k, top_p in SAMPLE_SETTINGS:
        if kind == "ties" and top_p < 1.0:
            # which of several equally likely tokens top_p keeps is left to the sort in the
            # reference (yalis/external/sampling.py:24); the kernel drops them together
            continue
        for draw in range(4):
            want = P.sample_token(logits[0].cpu(), temperature, top_k or None, top_p, 7, draw)
            got = _sample(ops, logits, temperature, top_k, top_p, 7, draw)[0].item()
            slow = _sample(ops, logits, temperature, top_k, top_p, 7, draw, whole_row=True)[0].item()
            assert got == want and slow == want, (kind, temperature, top_k, top_p, draw, got, slow, want)


@pytest.mark.parametrize("kind", ["peaked", "flat"])
def test_sample_divided_rows(ops, kind):
    """Rows of a large vocabulary are divided among workgroups: rows with different settings in
    one launch give the plain implementation's tokens, and each goes the way its settings
    say: greedy, a race over the row (plain temperature; top_p once its threshold is known),
    settled among the candidates (top_k), or left to one workgroup (more candidates than fit)."""
    import plain_llama as P

    vocab = 128256
    settings = [(0.0, 0, 1.0, 0), (1.0, 0, 1.0, 1), (1.0, 0, 0.8, 1), (1.0, 50, 1.0, 3), (0.7, 50, 0.8, 3),
                (2.0, 0, 0.9, 1), (1.0, 6000, 1.0, 4), (0.5, 1, 1.0, 3), (1.3, 0, 0.0, 1), (0.9, 3000, 0.95, 3)]
    gen = torch.Generator().manual_seed(77)
    logits = torch.randn((len(settings), vocab), generator=gen) * (3.0 if kind == "peaked" else 0.3)
    if kind == "peaked":
        logits[:, 1000:1040] += 9.0
    logits[1, 5] = float("-inf")  # a masked token: never drawn, and no part of the bins' extent
    dev = logits.to(DEV)
    col = lambda j, dt: torch.tensor([st[j] for st in settings], dtype=dt, device=DEV)
    seeds = torch.arange(len(settings), dtype=torch.int32, device=DEV) + 11
    for draw in range(3):
        draws = torch.full((len(settings),), draw, dtype=torch.int32, device=DEV)
        paths = torch.full((len(settings),), -1, dtype=torch.int32, device=DEV)
        got = ops.sample(dev, col(0, torch.float32), col(1, torch.int32), col(2, torch.float32), seeds, draws, paths=paths).cpu()
        assert paths.cpu().tolist() == [st[3] for st in settings]
        for i, (temperature, top_k, top_p, _) in enumerate(settings):
            want = P.sample_token(logits[i], temperature, top_k or None, top_p, 11 + i, draw)
            assert got[i].item() == want, (kind, i, settings[i], draw, got[i].item(), want)


def test_sample_rows_are_independent(ops):
    """Many rows with different settings in one launch give what each gives alone."""
    vocab = 50000
    logits = rnd((6, vocab), torch.float32, 41, scale=2.5)
    temperature = torch.tensor([0.0, 0.7, 1.0, 1.2, 0.9, 1.0], dtype=torch.float32, device=DEV)
    top_k = torch.tensor([0, 40, 0, 5000, 0, 1], dtype=torch.int32, device=DEV)
    top_p = torch.tensor([1.0, 0.9, 0.5, 1.0, 1.0, 0.3], dtype=torch.float32, device=DEV)
    seeds = torch.arange(6, dtype=torch.int32, device=DEV) + 100
    draws = torch.arange(6, dtype=torch.int32, device=DEV) * 3
    both = ops.sample(logits, temperature, top_k, top_p, seeds, draws).cpu()
    for i in range(6):
        alone = ops.sample(logits[i : i + 1].contiguous(), temperature[i : i + 1], top_k[i : i + 1], top_p[i : i + 1],
                           seeds[i : i + 1], draws[i : i + 1]).cpu()
        assert both[i].item() == alone[0].item()


def test_sample_frequencies(ops):
    """Draws follow softmax(logits / T): chi-square over many draws."""
    vocab, draws, temperature = 12, 20000, 0.8
    logits = torch.linspace(-2, 2, vocab, device=DEV).repeat(draws, 1).contiguous()
    got = _sample(ops, logits, temperature, 0, 1.0, 5, 0)
    counts = torch.bincount(got.long(), minlength=vocab).double()
    p = torch.softmax(logits[0].cpu().double() / temperature, dim=0)
    chi2 = ((counts - draws * p) ** 2 / (draws * p)).sum().item()
    assert chi2 < 40.0, chi2  # 11 degrees of freedom: 40 is beyond the 99.99th percentile


def test_tiled_pages_layout(ops):
    """Which pages are tiled, and that the description of the order which the tests work
    from is the one the kernels write: a token's key and value land where it says."""
    assert ops.cache_tiled(torch.bfloat16, 128, 64) and ops.cache_tiled(torch.bfloat16, 64, 192)
    assert not ops.cache_tiled(torch.float32, 128, 64) and not ops.cache_tiled(torch.bfloat16, 128, 32)
    assert not ops.cache_tiled(torch.bfloat16, 48, 64) and not ops.cache_tiled(torch.bfloat16, 256, 64)
    h, g, d, page = 2, 1, 64, 128
    cos, sin = _tables(d, 4)
    for slot in (0, 5, 37, 64, 127, 128 + 70):
        qkv = rnd((1, (h + 2 * g) * d), torch.bfloat16, slot)
        kc = torch.zeros((2, g, page, d), dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros((2, g, d, page), dtype=torch.bfloat16, device=DEV)
        want_k, want_v = qkv[0, h * d : (h + 1) * d].clone(), qkv[0, (h + 1) * d :].clone()
        ops.rope_append(qkv, h, g, d, torch.zeros(1, dtype=torch.int32, device=DEV), cos, sin, d, False, kc, vc,
                        torch.tensor([slot], dtype=torch.int32, device=DEV), page)  # position 0: no rotation
        kp, vp = R.untile_cache(kc.cpu(), vc.cpu())
        assert torch.equal(kp[slot // page, 0, slot % page], want_k.cpu()) and kp.ne(0).sum() == want_k.ne(0).sum()
        assert torch.equal(vp[slot // page, 0, :, slot % page], want_v.cpu()) and vp.ne(0).sum() == want_v.ne(0).sum()


def test_machine_probes_run_and_refuse_bad_sizes(ops):
    """The benchmark's two probes: they leave their input and (for ordinary data) their sink
    alone, count their flops, and refuse sizes their kernels do not take."""
    from yalis_amd.ops.hip import KernelError

    data = rnd((1 << 16,), torch.float32, 0)
    before = data.clone()
    sink = torch.zeros(1, dtype=torch.float32, device=DEV)
    for workgroups in (1, 7, 300):
        ops.probe_stream_read(data, workgroups, sink, nontemporal=workgroups == 7)
    assert ops.probe_mfma_bf16(3, 32, sink) == 3 * 4 * 32 * 4 * 16384
    torch.cuda.synchronize()
    assert torch.equal(data, before) and sink.item() == 0.0
    with pytest.raises(KernelError):
        ops.probe_stream_read(data[1:4], 4, sink)  # neither aligned nor whole 16-byte pieces
    with pytest.raises(KernelError):
        ops.probe_mfma_bf16(3, 10, sink)
