"""Each HIP kernel alone against a plain float32 torch reference of the same op, at sizes other than
the engine's tiny configurations (odd widths, vocabularies that are no power of two, several head
sizes and group sizes), in float32 and bfloat16."""

from __future__ import annotations

import math

import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def K():
    from mini_engine_amd.ops import kernels

    return kernels


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype is torch.float32 else dict(rtol=2e-2, atol=2e-2)


def dev(t):
    return t.cuda().contiguous()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,vocab", [(72, 301), (1024, 1000)])
def test_embed(dtype, hidden, vocab):
    table = torch.randn(vocab, hidden).to(dtype)
    ids = torch.randint(0, vocab, (37,), dtype=torch.int32)
    out = K().embed(dev(ids), dev(table))
    assert out.dtype is torch.float32
    assert torch.equal(out.cpu(), table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,dim", [(5, 72), (3, 1000), (2, 5120), (1, 16), (300, 1000), (257, 4096), (260, 72),
                                      (256, 520), (17, 1024), (64, 1000), (40, 4100)])
def test_add_rmsnorm(dtype, rows, dim):
    x, delta, w = torch.randn(rows, dim) * 3, torch.randn(rows, dim).to(dtype), 1 + 0.1 * torch.randn(dim)
    xd = dev(x.clone())
    h = K().add_rmsnorm(xd, dev(delta), dev(w), 1e-5, dtype)
    s = x + delta.float()
    torch.testing.assert_close(xd.cpu(), s, rtol=1e-6, atol=1e-6)  # the residual sum is a float32 sum
    torch.testing.assert_close(h.float().cpu(), plain.rms_norm(s, w, 1e-5), **tol(dtype))
    # no delta: x untouched; rows: gather without writing x
    xd2 = dev(x.clone())
    h2 = K().add_rmsnorm(xd2, None, dev(w), 1e-5, dtype)
    assert torch.equal(xd2.cpu(), x)
    torch.testing.assert_close(h2.float().cpu(), plain.rms_norm(x, w, 1e-5), **tol(dtype))
    pick = torch.tensor([rows - 1, 0], dtype=torch.int32)
    h3 = K().add_rmsnorm(xd2, dev(delta), dev(w), 1e-5, dtype, rows=dev(pick), write_x=False)
    assert torch.equal(xd2.cpu(), x)
    torch.testing.assert_close(h3.float().cpu(), plain.rms_norm(s[pick.long()], w, 1e-5), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_rows(dtype):
    x, w = torch.randn(4, 3, 48).to(dtype), torch.randn(48)
    out = K().rmsnorm(dev(x), dev(w), 1e-6)
    torch.testing.assert_close(out.float().cpu(), plain.rms_norm(x.float(), w, 1e-6), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,inter", [(7, 160), (3, 1001)])
def test_swiglu(dtype, tokens, inter):
    gu = (torch.randn(tokens, 2 * inter) * 2).to(dtype)
    g, u = gu.float()[:, :inter], gu.float()[:, inter:]
    torch.testing.assert_close(K().swiglu(dev(gu)).float().cpu(), plain.silu(g) * u, **tol(dtype))
    gelu = K().swiglu(dev(gu), activation="gelu_tanh").float().cpu()
    torch.testing.assert_close(gelu, torch.nn.functional.gelu(g, approximate="tanh") * u, **tol(dtype))
    with pytest.raises(ValueError, match="activation"):
        K().swiglu(dev(gu), activation="relu")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [2, 16, 33, 64, 130, 300])
def test_gated_products_with_either_activation(dtype, rows):
    """``linear(..., gated=name)`` at the row counts of every kernel that computes the gate as its epilogue
    (the small and the streaming kernel, the tiled one) or after a library product, against the formula."""
    g = torch.Generator().manual_seed(rows)
    x = torch.randn(rows, 128, generator=g).to(dtype)
    w = (torch.randn(2 * 200, 128, generator=g) * 0.1).to(dtype)
    y = x.float() @ w.float().T
    for name, act in (("silu", plain.silu), ("gelu_tanh", lambda z: torch.nn.functional.gelu(z, approximate="tanh"))):
        want = act(y[:, :200]) * y[:, 200:]
        got = K().linear(dev(x), dev(w), gated=name).float().cpu()
        t = tol(dtype)
        torch.testing.assert_close(got, want, rtol=t["rtol"], atol=t["atol"] * max(1.0, want.abs().max().item()))
    assert (act(y[:, :200]) - plain.silu(y[:, :200])).abs().max() > 0.05  # the two activations differ at these values


@pytest.mark.parametrize("m,n,k", [(1, 50, 33), (5, 130, 72), (70, 64, 100), (129, 257, 48), (64, 33, 1028), (65, 300, 1024),
                                   (200, 96, 2050), (32, 31, 16), (33, 160, 2)])
def test_gemm_f32(m, n, k):
    """The float32 product at row counts on both sides of its tile shapes' limits (32, 64), columns that are no
    multiple of a tile, k that is no multiple of the tile's 16, of 4 (no 16-byte loads) or of the instruction's 2;
    one column and one row stand out, so that a tile that stops short of them or runs past them shows."""
    g = torch.Generator().manual_seed(m * 7 + n + k)
    x, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g)
    w[n - 1] *= 8
    x[m - 1] *= 8
    out = K().gemm_f32(dev(x), dev(w))
    want = (x.double() @ w.double().T).float()
    torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=1e-5 * max(1.0, want.abs().max().item()))
    shifted = dev(torch.cat([torch.zeros(1, k), x]))[1:]  # rows that start 4 k bytes into an allocation: not always 16-byte aligned
    assert torch.equal(K().gemm_f32(shifted, dev(w)).cpu(), out.cpu())  # scalar and 16-byte loads give the same sums


@pytest.mark.parametrize("m,n,k,gated", [(130, 200, 128, False), (257, 96, 192, True), (2048, 1024, 1024, False),
                                         (77, 50, 64, True), (300, 333, 256, False), (513, 1000, 320, True), (1100, 200, 128, True)])
@pytest.mark.parametrize("shape", [0, 1, 2, 6, 7, 8, 9, 12])
def test_gemm_bf16_tiled(m, n, k, gated, shape):
    """The LDS-tiled matrix-core product at sizes that are no multiple of its tiles, against a float32
    product of the same bfloat16 inputs; every block tile shape, plain and with the SwiGLU epilogue."""
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n * (2 if gated else 1), k, generator=g) * 0.1).bfloat16()
    want = x.float() @ w.float().T
    if gated:
        want = plain.silu(want[:, :n]) * want[:, n:]
    out_types = (torch.bfloat16,) if gated else (torch.bfloat16, torch.float32)
    for out_dtype in out_types:
        got = K().gemm_bf16_tiled(dev(x), dev(w), out_dtype, gated, shape=shape).float().cpu()
        scale = max(1.0, want.abs().max().item())
        tol_abs = (2**-7 if out_dtype is torch.bfloat16 else 1e-4) * scale
        assert (got - want).abs().max().item() <= tol_abs, (out_dtype, (got - want).abs().max().item(), scale)
    from mini_engine_amd.ops.library import KernelError

    with pytest.raises(KernelError, match="multiple of 64"):
        K().gemm_bf16_tiled(dev(x[:, : k - 8].contiguous()), dev(w[:, : k - 8].contiguous()), torch.bfloat16, gated)


@pytest.mark.parametrize("m,n,k", [(130, 200, 128), (2048, 1024, 1024), (70, 50, 72), (300, 333, 75), (65, 1001, 40), (1, 64, 64)])
def test_gemm_bf16_library(m, n, k):
    """Plain products through the GEMM library, called directly where it has an algorithm for the sizes
    and through torch where not (odd widths), as bfloat16 and as float32, also replayed from a graph."""
    g = torch.Generator().manual_seed(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    want = x.float() @ w.float().T
    scale = max(1.0, want.abs().max().item())
    xd, wd = dev(x), dev(w)
    for out_dtype in (torch.bfloat16, torch.float32):
        got = K().gemm_bf16_library(xd, wd, out_dtype)
        assert got.dtype is out_dtype
        tol_abs = (2**-7 if out_dtype is torch.bfloat16 else 1e-4) * scale
        assert (got.float().cpu() - want).abs().max().item() <= tol_abs, (out_dtype, (got.float().cpu() - want).abs().max().item(), scale)
    out = torch.zeros(m, n, dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        K().gemm_bf16_library(xd, wd, torch.bfloat16, out=out)
    for _ in range(2):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert (out.float().cpu() - want).abs().max().item() <= 2**-7 * scale


@pytest.mark.parametrize("m,n,k,splits", [(17, 1024, 2048, 4), (64, 1000, 3072, 4), (33, 48, 520, 2), (40, 16, 4096, 8)])
def test_small_gemm_partial_sums_and_their_add_rmsnorm(m, n, k, splits):
    """A product of 17 to 64 rows cut into runs of k: the parts add up to the product, and add_rmsnorm
    takes them where it takes a delta."""
    g = torch.Generator().manual_seed(k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    parts = K().gemm_bf16_small(dev(x), dev(w), torch.float32, k_splits=splits)
    assert parts.shape == (splits, m, n)
    want = x.float() @ w.float().T
    torch.testing.assert_close(parts.sum(0).cpu(), want, rtol=1e-4, atol=1e-4 * max(1.0, want.abs().max().item()))
    if k >= 64 * splits:
        assert all(parts[i].abs().max() > 0 for i in range(splits))  # every run did some of the work
    res = torch.randn(m, n, generator=g) * 2
    wn = 1 + 0.1 * torch.randn(n, generator=g)
    xd = dev(res.clone())
    h = K().add_rmsnorm(xd, K().PartialSums(parts), dev(wn), 1e-5, torch.bfloat16)
    s = res + want
    torch.testing.assert_close(xd.cpu(), s, rtol=1e-4, atol=1e-4 * max(1.0, s.abs().max().item()))
    torch.testing.assert_close(h.float().cpu(), plain.rms_norm(s, wn, 1e-5), **tol(torch.bfloat16))
    pick = torch.tensor([m - 1, 0], dtype=torch.int32)
    xd2 = dev(res.clone())
    h2 = K().add_rmsnorm(xd2, K().PartialSums(parts), dev(wn), 1e-5, torch.bfloat16, rows=dev(pick), write_x=False)
    assert torch.equal(xd2.cpu(), res)
    torch.testing.assert_close(h2.float().cpu(), plain.rms_norm(s[pick.long()], wn, 1e-5), **tol(torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,dim,num_parts", [(3, 5120, 7), (40, 5120, 7), (64, 8192, 16), (8, 1000, 5), (20, 16384, 2), (2, 20000, 3),
                                                (5, 1002, 4), (1, 16, 9)])
def test_add_rmsnorm_with_partial_sums_at_every_row_length(dtype, rows, dim, num_parts):
    """Partial sums stand where a delta stands, for few rows and many, rows of one vector and of several vectors per
    thread, lengths that are no multiple of 4 and lengths beyond the vectorised kernel's."""
    g = torch.Generator().manual_seed(rows * dim + num_parts)
    x, w = torch.randn(rows, dim, generator=g) * 3, 1 + 0.1 * torch.randn(dim, generator=g)
    parts = torch.randn(num_parts, rows, dim, generator=g)
    xd = dev(x.clone())
    h = K().add_rmsnorm(xd, K().PartialSums(dev(parts)), dev(w), 1e-5, dtype)
    s = x + parts.sum(0)
    torch.testing.assert_close(xd.cpu(), s, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h.float().cpu(), plain.rms_norm(s, w, 1e-5), **tol(dtype))
    pick = torch.tensor([rows - 1, 0], dtype=torch.int32)
    xd2 = dev(x.clone())
    h2 = K().add_rmsnorm(xd2, K().PartialSums(dev(parts)), dev(w), 1e-5, dtype, rows=dev(pick), write_x=False)
    assert torch.equal(xd2.cpu(), x)
    torch.testing.assert_close(h2.float().cpu(), plain.rms_norm(s[pick.long()], w, 1e-5), **tol(dtype))


def test_linear_hands_back_partial_sums_only_when_asked():
    """A bfloat16 product that is only ever a delta of the residual stream comes back as float32 partial sums, never
    rounded to bfloat16: several runs of k from the streaming kernel up to 64 rows, one sum from the library beyond,
    and for sizes the streaming kernel does not take."""
    x = dev(torch.randn(40, 2048).bfloat16())
    w = dev((torch.randn(1024, 2048) * 0.02).bfloat16())
    plain_out = K().linear(x, w)
    assert isinstance(plain_out, torch.Tensor)
    exact = x.float() @ w.float().T
    delta = K().linear(x, w, as_delta=True)
    assert isinstance(delta, K().PartialSums) and delta.shape == (40, 1024) and delta.parts.shape[0] > 1
    torch.testing.assert_close(delta.parts.sum(0), exact, rtol=1e-4, atol=1e-4)  # float32 all the way
    few = K().linear(x[:8].contiguous(), w, as_delta=True)  # few rows too: k is cut so that every compute unit streams
    assert isinstance(few, K().PartialSums) and few.shape == (8, 1024) and few.parts.shape[0] > 1
    torch.testing.assert_close(few.parts.sum(0), exact[:8], rtol=1e-4, atol=1e-4)
    narrow = dev((torch.randn(1024, 2048 - 4) * 0.02).bfloat16())  # k no multiple of 8: not the streaming kernel's
    odd = K().linear(x[:, :2044].contiguous(), narrow, as_delta=True)
    assert isinstance(odd, K().PartialSums) and odd.parts.shape == (1, 40, 1024) and odd.parts.dtype is torch.float32
    many = K().linear(dev(torch.randn(300, 2048).bfloat16()), w, as_delta=True)  # beyond 64 rows: one sum from the library
    assert isinstance(many, K().PartialSums) and many.parts.shape == (1, 300, 1024) and many.parts.dtype is torch.float32
    short = K().linear(x[:, :256].contiguous(), dev((torch.randn(1024, 256) * 0.02).bfloat16()), as_delta=True)  # one run of k
    assert isinstance(short, K().PartialSums) and short.parts.shape == (1, 40, 1024)


def test_gemm_f32_rows_do_not_depend_on_the_batch():
    """The value of a row is bit-identical whatever other rows are in the product."""
    x, w = torch.randn(200, 200), torch.randn(77, 200)
    whole = K().gemm_f32(dev(x), dev(w)).cpu()  # tiles of 128 rows
    for lo, hi in [(0, 1), (63, 65), (89, 90), (10, 80), (100, 132), (136, 200), (0, 65)]:  # one-wave tiles, and large ones
        assert torch.equal(K().gemm_f32(dev(x[lo:hi]), dev(w)).cpu(), whole[lo:hi])


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 100, 72), (17, 1000, 1024), (64, 33, 160), (33, 151, 3072)])
def test_gemm_bf16_skinny(m, n, k, out_dtype):
    x, w = torch.randn(m, k).bfloat16(), (torch.randn(n, k) * 0.05).bfloat16()
    out = K().gemm_bf16_skinny(dev(x), dev(w), out_dtype)
    want = (x.double() @ w.double().T).float()
    t = dict(rtol=1e-4, atol=1e-4) if out_dtype is torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(out.float().cpu(), want, **t)


@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 96, 72), (16, 1000, 1024), (33, 64, 160), (64, 160, 3072)])
@pytest.mark.parametrize("with_delta", [True, False])
@pytest.mark.parametrize("gated", [True, False])
def test_gemm_bf16_small_with_norm_prologue_and_swiglu_epilogue(m, n, k, with_delta, gated):
    """The fused form against its unfused definition: rmsnorm(x + delta) * w, product, silu(gate) * up;
    the residual stream comes out in the second buffer and the first is left untouched."""
    g = torch.Generator().manual_seed(m * 1000 + n)
    x = torch.randn(m, k, generator=g) * 2
    delta = torch.randn(m, k, generator=g).bfloat16() if with_delta else None
    wn = 1 + 0.2 * torch.randn(k, generator=g)
    w = (torch.randn(2 * n if gated else n, k, generator=g) * 0.05).bfloat16()
    xd, spare = dev(x.clone()), dev(torch.full((m, k), 7.0))
    h = K().NormedInput(xd, None if delta is None else dev(delta), dev(wn), 1e-5, torch.bfloat16, spare)
    # linear() fuses up to 16 rows (a row or two go to the weight-streaming kernel's prologue instead); the kernel takes 64
    in_stream = m <= 2 and K().stream_norm_fits(m, k)
    assert h.fusion(dev(w)) == (K().NORM_IN_STREAM if in_stream else K().NORM_IN_SMALL if m <= 16 else K().NORM_ALONE)
    out = K().gemm_bf16_small(h, dev(w), torch.bfloat16, gated).float().cpu()
    s = x + (delta.float() if with_delta else 0)
    y = plain.rms_norm(s, wn, 1e-5) @ w.float().T
    want = plain.silu(y[:, :n]) * y[:, n:] if gated else y
    torch.testing.assert_close(out, want, rtol=2e-2, atol=2e-2 * max(1.0, want.abs().max().item()))
    assert torch.equal(xd.cpu(), x)  # the input buffer is only read
    if with_delta:
        assert h.residual is spare
        torch.testing.assert_close(spare.cpu(), s, rtol=1e-6, atol=1e-6)  # a float32 sum
    else:
        assert h.residual is xd and torch.equal(spare.cpu(), torch.full((m, k), 7.0))


@pytest.mark.parametrize("m,n,k", [(1, 32768, 64), (2, 33001, 520), (8, 40010, 1024), (16, 33001, 2056), (3, 32768 + 17, 72)])
def test_gemm_bf16_small_with_very_many_columns(m, n, k):
    """From 32,768 columns on (an output head) and three rows on, a block computes four tiles of 16
    columns from one set of loads of x: column counts that are no multiple of 64, k over several rounds, both output types."""
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.1).bfloat16()
    w[-1] *= 5  # the last column stands out: a tile that stops short of it, or runs past it, shows
    want = x.float() @ w.float().T
    for out_dtype in (torch.float32, torch.bfloat16):
        got = K().gemm_bf16_small(dev(x), dev(w), out_dtype).float().cpu()
        scale = max(1.0, want.abs().max().item())
        tol_abs = (2**-7 if out_dtype is torch.bfloat16 else 1e-4) * scale
        assert (got - want).abs().max().item() <= tol_abs, (out_dtype, (got - want).abs().max().item(), scale)


@pytest.mark.parametrize("m,n,k", [(3, 1024, 2048), (8, 1024, 3072), (16, 1032, 520), (5, 104, 72), (33, 2048, 1000), (64, 4096, 264),
                                   (70, 520, 136), (130, 1024, 1024)])
def test_a_norm_carried_from_one_product_to_the_next(m, n, k):
    """The delta of the residual stream added to it in the product's epilogue, with bf16(x * w) and partial sums of
    squares left for the product behind the RMS norm, which multiplies its rows by rsqrt(mean + eps): against the
    float32 add, norm and products, for both kernels that take the second product, gated and not. One row of the
    stream is a thousand times the others, so that a scale taken from another row's sums shows."""
    g = torch.Generator().manual_seed(m * 31 + n + k)
    a = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    x = torch.randn(m, n, generator=g)
    x[m // 2] *= 1000.0
    wn = 1.0 + 0.3 * torch.randn(n, generator=g)
    eps = 1e-3
    x_dev = dev(x.clone())
    h, ss = K().gemm_bf16_stream_carry(dev(a), dev(w), x_dev, dev(wn))
    want_x = x + a.float() @ w.float().T
    assert (x_dev.cpu() - want_x).abs().max().item() <= 1e-4 * want_x.abs().max().item()
    assert ss.shape == (m, K().stream_carry_blocks(m, n, k))
    assert torch.allclose(ss.sum(1).cpu(), (want_x**2).sum(1), rtol=1e-4)
    want_h = want_x * wn
    assert ((h.float().cpu() - want_h).abs() <= 2**-7 * want_h.abs() + 1e-5 * want_x.abs().max()).all()  # one rounding to bfloat16
    normed = plain.rms_norm(want_x, wn, eps)
    for n2 in (96, 3 * 1024 + 8):
        w2 = (torch.randn(2 * n2, n, generator=g) * 0.05).bfloat16()
        y = normed @ w2.float().T
        for gated in (False, True):
            want = plain.silu(y[:, :n2]) * y[:, n2:] if gated else y
            for kernel in ("small", "stream"):
                if kernel == "small" and m > 64:
                    continue
                got = K().gemm_bf16_scaled(h, dev(w2), ss, n, eps, gated, torch.bfloat16, kernel).float().cpu()
                assert got.shape == want.shape
                assert ((got - want).abs().max(1).values <= 2**-6 * want.abs().max(1).values.clamp_min(1e-3)).all(), (n2, gated, kernel)


@pytest.mark.parametrize("m,n,k", [(1, 16, 128), (7, 100, 72), (16, 1040, 1000), (17, 4099, 1536), (33, 200, 2056), (48, 68, 8200),
                                   (64, 9000, 648), (64, 40, 136), (2, 3072, 264), (8, 6140, 128), (3, 6142, 136), (5, 1000, 3072),
                                   (64, 4096, 16384), (40, 2100, 24576), (33, 4098, 8704), (65, 520, 264), (130, 3072, 1024),
                                   (256, 68, 136), (200, 1030, 520)])
@pytest.mark.parametrize("gated", [True, False])
def test_gemm_bf16_stream(m, n, k, gated):
    """The weight-streaming product at every row-tile count, with column counts that are no multiple of a
    block's (every arrangement of a block's waves: many, some and few columns), k that is no multiple of a
    step, both output types, the gated form, and partial sums over runs of k whose sum is the product. Four
    shapes of up to 8 rows are dealt to more blocks than they have runs of a block's columns (whole rounds of the
    compute units), so that blocks begin and end inside a tile of 16, at column counts that are a multiple of 16,
    of 4, or of neither; the last three (more than 32 rows, thousands of columns, long k) take blocks of 128 columns,
    two tiles a wave, for their partial sums. More than 64 rows go to groups of blocks, 64 rows a group, the last
    group with fewer."""
    g = torch.Generator().manual_seed(m * 977 + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(2 * n if gated else n, k, generator=g) * 0.05).bfloat16()
    w[n - 1] *= 4  # the last column stands out: a tile that stops short of it, or runs past it, shows
    y = x.float() @ w.float().T
    want = plain.silu(y[:, :n]) * y[:, n:] if gated else y
    scale = max(1.0, want.abs().max().item())
    got = K().gemm_bf16_stream(dev(x), dev(w), torch.bfloat16, gated).float().cpu()
    assert (got - want).abs().max().item() <= 2**-7 * scale
    if gated:
        return
    got = K().gemm_bf16_stream(dev(x), dev(w), torch.float32).cpu()
    assert (got - want).abs().max().item() <= 1e-4 * scale
    steps = -(-k // 128)
    for splits in sorted({K().stream_splits(n, k, rows=m), K().stream_splits(n, k), 2, 3, min(steps, 64)} - {1}):
        if steps < splits or -(-steps // -(-steps // splits)) != splits:
            continue  # runs are whole steps, none of them empty
        parts = K().gemm_bf16_stream(dev(x), dev(w), torch.float32, k_splits=splits).cpu()
        assert parts.shape == (splits, m, n)
        assert (parts.sum(0) - want).abs().max().item() <= 1e-4 * scale
        assert parts[-1].abs().max() > 0


@pytest.mark.parametrize("m,n,k", [(1, 4096, 1024), (2, 100, 1000), (3, 1040, 72), (4, 68, 2056), (1, 16, 128), (2, 9000, 648),
                                   (1, 3072, 1024), (2, 6142, 264), (2, 520, 2048), (1, 100, 4096)])
@pytest.mark.parametrize("delta", ["none", "tensor", "parts3", "parts6", "parts11", "parts16"])
@pytest.mark.parametrize("gated", [False, "silu", "gelu_tanh"])
def test_gemm_bf16_stream_norm(m, n, k, delta, gated):
    """Residual add, RMSNorm and product in one launch of the weight-streaming kernel, for a row or a few: every
    arrangement of a block's waves, k that is no multiple of a step, k of 2,048 and 4,096 (whose walk over k starts at
    another step in every block), each kind of delta (none, a tensor, partial sums in odd and even numbers: fewer than the
    prologue requests at once, which are 4, 8 or 16 for one row and 8 for more, as many, and more), both output
    types and both gates; the sum goes to the second buffer and only there."""
    g = torch.Generator().manual_seed(m * 31 + n + k)
    x, wn = torch.randn(m, k, generator=g) * 2, 1 + 0.2 * torch.randn(k, generator=g)
    w = (torch.randn(2 * n if gated else n, k, generator=g) * 0.05).bfloat16()
    w[n - 1] *= 4
    s, d = x.clone(), None
    if delta == "tensor":
        d = torch.randn(m, k, generator=g).bfloat16()
        s = x + d.float()
        d = dev(d)
    elif delta.startswith("parts"):
        parts = torch.randn(int(delta[5:]), m, k, generator=g)
        s = x + parts.sum(0)
        d = K().PartialSums(dev(parts))
    normed = plain.rms_norm(s, wn, 1e-5)
    y = normed @ w.float().T
    act = {"silu": plain.silu, "gelu_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh")}.get(gated)
    want = act(y[:, :n]) * y[:, n:] if gated else y
    scale = max(1.0, want.abs().max().item())
    for out_dtype in ((torch.bfloat16,) if gated else (torch.bfloat16, torch.float32)):
        xd, spare = dev(x.clone()), dev(torch.full((m, k), 7.0))
        h = K().NormedInput(xd, d, dev(wn), 1e-5, torch.bfloat16, spare)
        got = K().gemm_bf16_stream_norm(h, dev(w), out_dtype, gated).float().cpu()
        # the operand is rounded to bfloat16 once, as the add-and-norm kernel rounds it: 2^-8 of the largest product
        assert (got - want).abs().max().item() <= 2**-6 * scale
        assert torch.equal(xd.cpu(), x)  # other blocks still read it
        if delta == "none":
            assert h.residual is xd and torch.equal(spare.cpu(), torch.full((m, k), 7.0))
        else:
            assert h.residual is spare
            torch.testing.assert_close(spare.cpu(), s, rtol=1e-6, atol=1e-6)


def test_stream_plan_deals_columns_in_whole_rounds():
    """What the plan promises, on any number of compute units: the blocks cover all columns, a block has at most
    its waves' 16 columns each, and the runs of k are whole steps of which none is empty. On 256 compute units: the
    shapes this file tests the uneven deal with do get one, and the layer shapes the choice was measured on get
    what was measured best."""
    cus = K().compute_units(torch.device("cuda:0"))
    for m in (1, 8, 16, 17, 64):
        for n, k in ((16, 128), (1000, 3072), (3072, 1024), (4096, 4096), (6142, 136), (10240, 5120), (25600, 5120), (151936, 1024)):
            for gated in (False, True):
                for may_split in (False, True):
                    splits = K().stream_splits(n, k, rows=m) if may_split and not gated else 1
                    wn, runs, grid = K().stream_plan(m, n, k, gated, splits)
                    assert wn in (1, 2, 4, 8) and runs == splits  # tiles of 16 columns per block
                    fours = -(-n // 4)
                    assert grid >= -(-n // (16 * wn)) and -(-fours // grid) * 4 <= 16 * wn, (m, n, k, gated, wn, runs, grid)
                    steps = -(-k // 128)
                    assert -(-steps // -(-steps // runs)) == runs
    if cus != 256:
        return
    assert K().stream_plan(2, 3072, 264, True) == (1, 1, 256)  # 192 tiles of 16 columns on 256 blocks of 12
    assert K().stream_plan(8, 6140, 128) == (2, 1, 256)
    assert K().stream_plan(5, 1000, 3072, False, K().stream_splits(1000, 3072, rows=5)) == (2, 6, 42)
    assert K().stream_plan(1, 25600, 5120, True) == (4, 1, 512) and K().stream_plan(1, 6144, 4096) == (2, 1, 256)
    assert K().stream_plan(1, 4096, 12288, False, K().stream_splits(4096, 12288)) == (4, 4, 64)
    assert K().stream_plan(64, 10240, 5120) == (4, 1, 160)  # many rows: wide blocks before whole rounds
    for m, n, k in ((64, 4096, 16384), (40, 2100, 24576), (33, 4098, 8704)):  # blocks of 128 columns, two tiles a wave
        assert K().stream_plan(m, n, k, False, K().stream_splits(n, k, rows=m))[0] == 8
    assert K().stream_plan(64, 4096, 4096, False, K().stream_splits(4096, 4096, rows=64))[0] == 4  # its partial sums would weigh too much


def test_gemm_bf16_stream_norm_refuses_what_it_cannot_do():
    wn, w = dev(torch.ones(64)), dev(torch.zeros(32, 64).bfloat16())
    x = dev(torch.zeros(17, 64))
    with pytest.raises(ValueError, match="17 rows"):
        K().gemm_bf16_stream_norm(K().NormedInput(x, None, wn, 1e-6, torch.bfloat16, None), w)
    assert not K().stream_norm_fits(4, 8192) and K().stream_norm_fits(2, 8192)  # the rows stay in the block's memory
    x = dev(torch.zeros(2, 64))
    with pytest.raises(ValueError, match="second buffer"):
        K().gemm_bf16_stream_norm(K().NormedInput(x, dev(torch.zeros(2, 64).bfloat16()), wn, 1e-6, torch.bfloat16, None), w)
    with pytest.raises(ValueError, match="residual stream itself"):
        K().gemm_bf16_stream_norm(K().NormedInput(x, dev(torch.zeros(2, 64).bfloat16()), wn, 1e-6, torch.bfloat16, x), w)


def test_gemm_bf16_stream_refuses_what_it_cannot_do():
    x, w = dev(torch.zeros(257, 64).bfloat16()), dev(torch.zeros(32, 64).bfloat16())
    with pytest.raises(ValueError):
        K().gemm_bf16_stream(x, w)
    x = dev(torch.zeros(4, 68).bfloat16())
    with pytest.raises(RuntimeError, match="multiple of 8"):
        K().gemm_bf16_stream(x, dev(torch.zeros(32, 68).bfloat16()))
    x = dev(torch.zeros(4, 256).bfloat16())
    with pytest.raises(RuntimeError, match="runs of whole steps"):
        K().gemm_bf16_stream(x, dev(torch.zeros(32, 256).bfloat16()), torch.float32, k_splits=3)
    with pytest.raises(RuntimeError, match="plain float32"):
        K().gemm_bf16_stream(x, dev(torch.zeros(32, 256).bfloat16()), torch.bfloat16, k_splits=2)


def test_normed_input_falls_back_to_the_separate_kernels():
    """More than 64 rows or float32: the add-and-norm kernel runs, in place, and the product follows."""
    for dtype, m in ((torch.bfloat16, 100), (torch.float32, 5)):
        x, delta = torch.randn(m, 64), torch.randn(m, 64).to(dtype)
        wn, w = 1 + 0.1 * torch.randn(64), (torch.randn(48, 64) * 0.1).to(dtype)
        xd = dev(x.clone())
        h = K().NormedInput(xd, dev(delta), dev(wn), 1e-6, dtype, dev(torch.zeros(m, 64)))
        out = K().linear(h, dev(w), gated=True).float().cpu()
        s = x + delta.float()
        y = plain.rms_norm(s, wn, 1e-6) @ w.float().T
        torch.testing.assert_close(out, plain.silu(y[:, :24]) * y[:, 24:], **tol(dtype))
        assert h.residual is xd
        torch.testing.assert_close(xd.cpu(), s, rtol=1e-6, atol=1e-6)


def test_gemm_bf16_skinny_refuses_what_it_cannot_do():
    from mini_engine_amd.ops.library import KernelError

    x, w = dev(torch.randn(4, 20).bfloat16()), dev(torch.randn(8, 20).bfloat16())
    with pytest.raises(KernelError, match="multiple of 8"):
        K().gemm_bf16_skinny(x, w)
    with pytest.raises(ValueError, match="at most 64"):
        K().gemm_bf16_skinny(dev(torch.randn(65, 16).bfloat16()), dev(torch.randn(8, 16).bfloat16()))


@pytest.mark.parametrize("m,n,k", [(3, 40, 20), (200, 96, 72), (100, 70, 64)])
def test_linear_bf16_takes_every_shape(m, n, k):
    x, w = torch.randn(m, k).bfloat16(), (torch.randn(n, k) * 0.1).bfloat16()
    want = (x.double() @ w.double().T).float()
    torch.testing.assert_close(K().linear(dev(x), dev(w)).float().cpu(), want, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(K().linear(dev(x), dev(w), torch.float32).cpu(), want, rtol=1e-2, atol=1e-2)


# ------------------------------------------------- q/k norm + rotary + page write, and attention
def make_paged(items, nkv, d, bs, dtype, num_pages=64, seed=0):
    """items: list of (cached, new). Returns full k/v per item, scattered tables and the cache holding
    the cached part of every item (pages used by nobody are filled with large garbage)."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_pages, generator=g).tolist()
    k_cache = torch.full((num_pages, nkv, bs, d), 50.0).to(dtype)
    v_cache = torch.full((num_pages, nkv, d, bs), -70.0).to(dtype)
    tables, ks, vs = [], [], []
    for cached, new in items:
        n = cached + new
        table = [perm.pop() for _ in range(-(-n // bs))]
        k, v = torch.randn(n, nkv, d, generator=g).to(dtype), torch.randn(n, nkv, d, generator=g).to(dtype)
        for pos in range(cached):
            k_cache[table[pos // bs], :, pos % bs, :] = k[pos]
            v_cache[table[pos // bs], :, :, pos % bs] = v[pos]
        tables.append(table)
        ks.append(k)
        vs.append(v)
    width = max(len(t) for t in tables)
    table_t = torch.tensor([t + [0] * (width - len(t)) for t in tables], dtype=torch.int32)
    positions = torch.tensor([p for c, n in items for p in range(c, c + n)], dtype=torch.int32)
    token_item = torch.tensor([i for i, (c, n) in enumerate(items) for _ in range(n)], dtype=torch.int32)
    return k_cache, v_cache, tables, table_t, positions, token_item, ks, vs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,bs,rd,norm", [(4, 2, 16, 4, 16, True), (6, 1, 32, 8, 32, True),
                                                  (3, 3, 48, 16, 32, False), (16, 8, 128, 16, 128, True),
                                                  (2, 1, 256, 32, 0, True)])
def test_qk_norm_rope_scatter(dtype, nh, nkv, d, bs, rd, norm):
    items = [(0, 7), (9, 1), (8, 5)]
    k_cache, v_cache, tables, table_t, positions, token_item, _, _ = make_paged(items, nkv, d, bs, dtype)
    t = positions.numel()
    qkv = torch.randn(t, (nh + 2 * nkv) * d).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(d), 1 + 0.2 * torch.randn(d)
    theta, eps = 5000.0, 1e-5
    inv_freq = (1.0 / (theta ** (torch.arange(0, rd, 2, dtype=torch.float32) / rd))) if rd else None
    kc, vc = dev(k_cache.clone()), dev(v_cache.clone())
    q_out = K().qk_norm_rope_scatter(dev(qkv), dev(qw) if norm else None, dev(kw) if norm else None,
                                     K().rope_table(dev(inv_freq), int(positions.max()) + 1) if rd else None, dev(positions),
                                     dev(token_item), dev(table_t),
                                     kc, vc, nh, nkv, d, eps)
    f = qkv.float()
    q, k, v = (f[:, : nh * d].view(t, nh, d), f[:, nh * d : (nh + nkv) * d].view(t, nkv, d),
               f[:, (nh + nkv) * d :].view(t, nkv, d))
    if norm:
        q, k = plain.rms_norm(q, qw, eps), plain.rms_norm(k, kw, eps)
    if rd:
        cos, sin = plain.rope_tables(positions, rd, theta)
        q = torch.cat((plain.apply_rope(q[..., :rd], cos, sin), q[..., rd:]), -1)
        k = torch.cat((plain.apply_rope(k[..., :rd], cos, sin), k[..., rd:]), -1)
    torch.testing.assert_close(q_out.float().cpu(), q, **tol(dtype))
    kc, vc = kc.float().cpu(), vc.float().cpu()
    touched = torch.zeros(k_cache.shape[0], bs, dtype=torch.bool)
    for i in range(t):
        table, pos = tables[token_item[i]], int(positions[i])
        page, slot = table[pos // bs], pos % bs
        touched[page, slot] = True
        torch.testing.assert_close(kc[page, :, slot, :], k[i], **tol(dtype))
        torch.testing.assert_close(vc[page, :, :, slot], v[i], **tol(dtype))
    # every other slot keeps what it held
    keep = ~touched
    assert torch.equal(kc.permute(0, 2, 1, 3)[keep], k_cache.float().permute(0, 2, 1, 3)[keep])
    assert torch.equal(vc.permute(0, 3, 1, 2)[keep], v_cache.float().permute(0, 3, 1, 2)[keep])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,bs", [(4, 2, 32, 16), (16, 8, 128, 16), (3, 1, 64, 32), (2, 2, 48, 8)])
def test_qk_norm_rope_scatter_writes_values_by_page_tiles(dtype, nh, nkv, d, bs):
    """Many tokens: the values go through the page-tile kernel (pages of a multiple of 16 slots). Items
    start inside a page, end inside a page, span many pages, and one has a single token; slots that
    the step does not touch keep what they held. Same cache as the element-wise path."""
    items = [(5, 70), (0, 33), (31, 1), (16, 16), (47, 100)]
    k_cache, v_cache, tables, table_t, positions, token_item, _, _ = make_paged(items, nkv, d, bs, dtype, num_pages=96)
    t = positions.numel()
    qkv = torch.randn(t, (nh + 2 * nkv) * d).to(dtype)
    qw, kw = 1 + 0.2 * torch.randn(d), 1 + 0.2 * torch.randn(d)
    rope = K().rope_table(dev(1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))), 256)
    qlens = [n for _, n in items]
    item_start = torch.tensor([0] + torch.tensor(qlens).cumsum(0).tolist(), dtype=torch.int32)
    out = {}
    for tiled in (False, True):
        kc, vc = dev(k_cache.clone()), dev(v_cache.clone())
        extra = dict(item_start=dev(item_start), starts=[c for c, _ in items], qlens=qlens) if tiled else {}
        q = K().qk_norm_rope_scatter(dev(qkv), dev(qw), dev(kw), rope, dev(positions), dev(token_item), dev(table_t),
                                     kc, vc, nh, nkv, d, 1e-6, **extra)
        out[tiled] = (q.cpu(), kc.cpu(), vc.cpu())
    for a, b in zip(out[False], out[True]):
        assert torch.equal(a, b)
    v = qkv[:, (nh + nkv) * d :].view(t, nkv, d)
    vc = out[True][2]
    for i in range(t):
        table, pos = tables[token_item[i]], int(positions[i])
        assert torch.equal(vc[table[pos // bs], :, :, pos % bs], v[i])


def assert_attention_close(got: torch.Tensor, want: torch.Tensor, bits: int = 7) -> None:
    """bfloat16 attention outputs against the float32 result from the same bfloat16 inputs, token by token: no element
    further off than 2^-bits of that token's largest output. The outputs are softmax averages over hundreds of values,
    well below 1 in size, so an absolute tolerance would be a sizeable share of the signal; a result rounded to
    bfloat16 is 2^-9 off at most, and the softmax weights rounded to bfloat16 add less than that."""
    got, want = got.float().cpu().reshape(want.shape[0], -1), want.reshape(want.shape[0], -1)
    err = (got - want).abs().amax(dim=-1)
    bound = 2.0**-bits * want.abs().amax(dim=-1)
    bad = (err > bound).nonzero()
    assert bad.numel() == 0, (f"token {int(bad[0])}: error {err[bad[0]].item():.3e} against a bound of {bound[bad[0]].item():.3e} "
                              f"(largest output {want[bad[0]].abs().max().item():.3e}); {bad.numel()} of {want.shape[0]} tokens off")


def dense_reference(qs, ks, vs, items, scale, window):
    outs = []
    for q, k, v, (cached, new) in zip(qs, ks, vs, items):
        outs.append(plain.grouped_causal_attention(q.float(), k.float(), v.float(), scale, window))
    return torch.cat(outs).reshape(sum(n for _, n in items), -1)


def fill_new(k_cache, v_cache, tables, ks, vs, items, bs):
    for table, k, v, (cached, new) in zip(tables, ks, vs, items):
        for pos in range(cached, cached + new):
            k_cache[table[pos // bs], :, pos % bs, :] = k[pos]
            v_cache[table[pos // bs], :, :, pos % bs] = v[pos]


ATTN_SHAPES = [(4, 2, 16, 4), (6, 1, 32, 8), (5, 5, 48, 16), (16, 8, 128, 16), (8, 2, 64, 32), (4, 4, 256, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,bs", ATTN_SHAPES)
@pytest.mark.parametrize("window", [0, 5])
def test_attention_general_mixed_batch(dtype, nh, nkv, d, bs, window):
    """A fresh prompt, single decoded tokens at several context lengths and a continued portion in
    one launch, with scattered tables (reference tests/test_attention.py:20 and test_gpu.py:29)."""
    items = [(0, 7), (9, 1), (8, 5), (0, 1), (15, 1), (16, 1), (63, 2), (130, 1), (60, 70)]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=128)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(5)
    qs = [torch.randn(n, nh, d, generator=g).to(dtype) for _, n in items]
    scale = d**-0.5
    out = K().attention_general(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(positions), dev(token_item),
                                dev(table_t), scale, window)
    want = dense_reference(qs, ks, vs, items, scale, window)
    if dtype is torch.float32:
        torch.testing.assert_close(out.cpu(), want, rtol=1e-5, atol=1e-5)
    else:
        assert_attention_close(out, want)


@pytest.mark.parametrize("nh,nkv,d,bs", ATTN_SHAPES + [(14, 2, 96, 16), (16, 1, 64, 16), (3, 1, 20, 4)])
@pytest.mark.parametrize("window", [0, 5, 100])
def test_attention_general_shares_tiles_without_changing_a_bit(nh, nkv, d, bs, window):
    """float32 steps with several tokens per item run in the kernel whose blocks share the tiles of keys and values
    among their tokens: the same bits as a wave per token and head fetching its own, for prompts, portions behind a
    context, single tokens between them (blocks that serve several items one after the other), windows that end inside
    and outside a block's tokens, contexts of several chunks, and every group size up to 16 heads per kv head. With few
    heads the kernel it is held against runs eight waves per token and head, which share the chunks; with many, one."""
    items = [(0, 7), (9, 1), (8, 5), (0, 1), (63, 2), (130, 1), (60, 70), (0, 200), (250, 3), (5, 64),
             (1000, 40), (767, 2), (255, 1), (256, 1), (511, 3)]  # the last five: several chunks of 256 keys, and their edges
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, torch.float32, num_pages=1200)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(6)
    q = torch.cat([torch.randn(n, nh, d, generator=g) for _, n in items])
    args = (dev(q), dev(k_cache), dev(v_cache), dev(positions), dev(token_item), dev(table_t), d**-0.5, window)
    shared = K().attention_general(*args)
    alone = K().attention_general(*args, shared_tiles=False)
    assert torch.equal(shared, alone)
    want = dense_reference(list(torch.split(q, [n for _, n in items])), ks, vs, items, d**-0.5, window)
    torch.testing.assert_close(shared.cpu(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key_at_every_page_edge(dtype):
    """One key's score is made to stand out by scaling it and the query; the output must be that
    key's value. Places: first key, both sides of page and tile edges, the last key."""
    nh, nkv, d, bs, ctx = 4, 2, 32, 16, 300
    for hot in [0, 15, 16, 17, 63, 64, 65, 127, 128, 255, 256, 298, 299]:
        items = [(ctx - 1, 1)]
        k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, seed=hot)
        direction = torch.randn(d)
        direction /= direction.norm()
        ks[0] = (ks[0].float() * 0.1).to(dtype)
        ks[0][hot] = (direction * 8).to(dtype)
        k_cache.fill_(0)
        fill_new(k_cache, v_cache, tables, ks, vs, [(0, ctx)], bs)
        q = (direction * 40).expand(1, nh, d).to(dtype)
        out = K().attention_general(dev(q), dev(k_cache), dev(v_cache), dev(positions), dev(token_item), dev(table_t),
                                    d**-0.5, 0)
        want = vs[0][hot].float().repeat_interleave(nh // nkv, dim=0).reshape(1, -1)
        torch.testing.assert_close(out.float().cpu(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_window_edge(dtype):
    """The key just outside the window must be ignored even when it would dominate, and the key just
    inside must be found."""
    nh, nkv, d, bs, ctx, window = 2, 1, 16, 8, 100, 37
    for hot, seen in [(ctx - window - 1, False), (ctx - window, True)]:
        items = [(ctx - 1, 1)]
        k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, seed=3)
        direction = torch.zeros(d)
        direction[3] = 1.0
        ks[0] = (ks[0].float() * 0.05).to(dtype)
        ks[0][hot] = (direction * 8).to(dtype)
        fill_new(k_cache, v_cache, tables, ks, vs, [(0, ctx)], bs)
        q = (direction * 40).expand(1, nh, d).to(dtype)
        out = K().attention_general(dev(q), dev(k_cache), dev(v_cache), dev(positions), dev(token_item), dev(table_t),
                                    d**-0.5, window).float().cpu()
        hot_v = vs[0][hot].float().repeat_interleave(nh, dim=0).reshape(1, -1)
        if seen:
            torch.testing.assert_close(out, hot_v, rtol=1e-2, atol=1e-2)
        else:
            want = dense_reference([q], ks, vs, [(ctx - 1, 1)], d**-0.5, window)
            assert_attention_close(out, want, bits=7 if dtype is torch.bfloat16 else 16)
            assert (out - hot_v).abs().max() > 0.3


def test_attention_refuses_bad_sizes():
    from mini_engine_amd.ops.library import KernelError

    q = dev(torch.zeros(1, 3, 16))
    kc, vc = dev(torch.zeros(2, 2, 4, 16)), dev(torch.zeros(2, 2, 16, 4))
    idx = dev(torch.zeros(1, dtype=torch.int32))
    with pytest.raises(KernelError, match="multiple"):
        K().attention_general(q, kc, vc, idx, idx, dev(torch.zeros(1, 1, dtype=torch.int32)), 1.0)


# -------------------------------------------------------------------------------------- sampling
@pytest.mark.parametrize("vocab", [7, 384, 5000, 151936])
def test_argmax_takes_the_first_maximum(vocab):
    logits = torch.randn(5, vocab)
    logits[1, vocab - 1] = 99.0
    logits[2, 0] = 99.0
    logits[3, vocab // 2] = 50.0
    logits[3, vocab // 3] = 50.0  # two equal maxima: the lower index wins
    out = K().sample(dev(logits)).cpu()
    assert out.tolist() == logits.argmax(-1).tolist()
    assert out[3] == vocab // 3


def test_temperature_sampling_is_keyed_repeatable_and_follows_softmax():
    from mini_engine_amd.sampling import draw_key

    logits = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5, -3.0, 1.5]])
    n = 20000
    rows = dev(logits.expand(n, -1).contiguous())
    temps = dev(torch.full((n,), 0.8))
    keys = dev(torch.tensor([draw_key(0, 5, i) for i in range(n)], dtype=torch.int64))
    a = K().sample(rows, temps, keys).cpu()
    b = K().sample(rows, temps, keys).cpu()
    assert torch.equal(a, b)  # a draw is a function of its key
    freq = torch.bincount(a.long(), minlength=7).float() / n
    want = plain.temperature_probs(logits, 0.8)[0]
    assert (freq - want).abs().max() < 4 * math.sqrt(0.25 / n) + 1e-3, (freq, want)
    other = K().sample(rows, temps, dev(torch.tensor([draw_key(1, 5, i) for i in range(n)], dtype=torch.int64))).cpu()
    assert not torch.equal(a, other)
    # temperature 0 rows in the same launch are plain argmax; a tiny temperature acts as argmax too
    mixed = dev(torch.tensor([0.0, 1e-7] * (n // 2)))
    assert set(K().sample(rows, mixed, keys).cpu().tolist()) == {0}


# -------------------------------------------------------- matrix-core attention kernels (bfloat16)
MFMA_SHAPES = [(4, 2, 32, 16), (6, 1, 32, 16), (16, 8, 128, 16), (8, 8, 64, 32), (16, 1, 64, 16), (3, 1, 96, 64),
               (2, 2, 256, 16), (40, 2, 32, 16), (4, 2, 192, 16), (4, 4, 128, 128), (2, 1, 64, 256)]


@pytest.mark.parametrize("nh,nkv,d,bs", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 37])
def test_attention_decode_mfma(nh, nkv, d, bs, window):
    """One new token per item at context lengths around page, tile and split edges (reference
    tests/test_gpu.py:29 uses [1, 16, 17, 33, 100, 255])."""
    dtype = torch.bfloat16
    ctxs = [1, 16, 17, 33, 100, 255, 64, 65, 700]
    items = [(c - 1, 1) for c in ctxs]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=160)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(9)
    qs = [torch.randn(1, nh, d, generator=g).to(dtype) for _ in items]
    scale = d**-0.5
    want = dense_reference(qs, ks, vs, items, scale, window)
    item_ctx = torch.tensor(ctxs, dtype=torch.int32)
    for max_ctx in (max(ctxs), 4096):  # a tight bound, and a graph's fixed bound with mostly empty splits
        width = -(-max_ctx // bs)
        wide = torch.zeros(len(items), max(width, table_t.shape[1]), dtype=torch.int32)
        wide[:, : table_t.shape[1]] = table_t
        out = K().attention_decode_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide),
                                        scale, window, max_ctx)
        assert_attention_close(out, want)


@pytest.mark.parametrize("nh,nkv,d,bs,max_ctx", [(16, 8, 128, 16, 8192), (8, 8, 64, 32, 16384)])
def test_attention_decode_of_a_launch_large_enough_to_stream(nh, nkv, d, bs, max_ctx):
    """A launch whose items may hold 256 MB and more of keys and values loads them as data that passes through once,
    unless the step's flags say that the items share pages: the same result either way, and as without flags."""
    dtype = torch.bfloat16
    ctxs = [1, 16, 17, 33, 100, 255, 64, 65, 700, 1000]
    assert len(ctxs) * max_ctx * nkv * d * 4 >= 256 << 20
    items = [(c - 1, 1) for c in ctxs]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=200)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(10)
    qs = [torch.randn(1, nh, d, generator=g).to(dtype) for _ in items]
    scale = d**-0.5
    want = dense_reference(qs, ks, vs, items, scale, 0)
    item_ctx = torch.tensor(ctxs, dtype=torch.int32)
    wide = torch.zeros(len(items), max_ctx // bs, dtype=torch.int32)
    wide[:, : table_t.shape[1]] = table_t
    outs = []
    for flags in (None, 0, 1):
        word = None if flags is None else dev(torch.tensor([flags], dtype=torch.int32))
        out = K().attention_decode_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide), scale, 0,
                                        max_ctx, step_flags=word)
        assert_attention_close(out, want)
        outs.append(out)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])  # the kind of load changes no bit


@pytest.mark.parametrize("nh,nkv,d,width", [(16, 8, 128, 1024), (32, 8, 128, 4096), (6, 2, 64, 200), (64, 8, 128, 5120),
                                            (3, 1, 64, 72)])
@pytest.mark.parametrize("rows", [1, 2, 3, 4])
def test_output_projection_that_adds_up_the_splits_of_decode_attention(nh, nkv, d, width, rows):
    """A decode step of very few items leaves the splits' partial results to its output projection: the product equals
    the one of the finished attention output (the second kernel's, rounded to bfloat16) with the same weight, summed
    over its runs of k; a far key that dominates lies in another split than the rest."""
    dtype = torch.bfloat16
    bs, max_ctx = 16, 4096
    ctxs = [700, 3000, 65, 4096][:rows]
    items = [(c - 1, 1) for c in ctxs]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=520)
    g = torch.Generator().manual_seed(21)
    qs = [torch.randn(1, nh, d, generator=g).to(dtype) for _ in items]
    ks[0][5] = (qs[0][0, 0].float() * 3).to(dtype)  # one early key that the first head of item 0 finds among hundreds
    fill_new(k_cache, v_cache, tables, ks, vs, [(0, c) for c in ctxs], bs)
    scale = d**-0.5
    item_ctx = torch.tensor(ctxs, dtype=torch.int32)
    wide = torch.zeros(len(items), max_ctx // bs, dtype=torch.int32)
    wide[:, : table_t.shape[1]] = table_t
    weight = (torch.randn(width, nh * d, generator=g) * (nh * d) ** -0.5).to(dtype)
    args = (dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide), scale, 0, max_ctx)
    out = K().attention_decode_bf16(*args)
    assert_attention_close(out, dense_reference(qs, ks, vs, items, scale, 0))
    part_o, part_ml, splits = K().attention_decode_bf16(*args, leave_parts=True)
    assert K().attention_decode_leaves_parts(rows, nh, nkv, d, splits)
    if not K().attention_out_product_supported(rows, nh, d, width, splits):
        from mini_engine_amd.ops.library import KernelError

        with pytest.raises(KernelError, match="not supported"):
            K().attention_out_product_bf16(part_o, part_ml, splits, dev(weight), rows, nh)
        return  # (more (row, head) pairs than a block takes, or too many heads for a run of k)
    parts = K().attention_out_product_bf16(part_o, part_ml, splits, dev(weight), rows, nh)
    want = out.float().cpu() @ weight.float().T
    got = parts.sum(0).cpu()
    assert parts.shape[1:] == (rows, width)
    torch.testing.assert_close(got, want, rtol=0, atol=2**-12 * float(want.abs().max()))


@pytest.mark.parametrize("nh,nkv,d,bs", [(16, 8, 128, 16), (4, 2, 64, 16), (6, 1, 96, 32)])
def test_attention_decode_with_fewer_live_items_than_the_grid_holds(nh, nkv, d, bs):
    """A launch laid out for as few as `least` live items (a replayed graph: the rest is padding) has
    more splits than a fuller step needs; the kernel takes as many as the live items call for. Every
    count of live items from `least` to all gives the same result as a launch without padding."""
    dtype = torch.bfloat16
    ctxs = [700, 16, 17, 333, 1000, 255, 64, 65, 1, 1, 1, 1, 130, 1, 1, 1]
    items = [(c - 1, 1) for c in ctxs]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=260)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(4)
    qs = [torch.randn(1, nh, d, generator=g).to(dtype) for _ in items]
    scale = d**-0.5
    want = dense_reference(qs, ks, vs, items, scale, 0)
    item_ctx = torch.tensor(ctxs, dtype=torch.int32)
    max_ctx = 4096
    wide = torch.zeros(len(items), max_ctx // bs, dtype=torch.int32)
    wide[:, : table_t.shape[1]] = table_t
    args = (dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide), scale, 0, max_ctx)
    plain_out = K().attention_decode_bf16(*args)
    assert_attention_close(plain_out, want)
    least = 9
    chunks = -(-(nh // nkv) // 16)
    grid_splits, full_splits = (K().decode_splits(n, nkv * chunks, max_ctx)[1] for n in (least, len(items)))
    assert grid_splits >= full_splits and (grid_splits > full_splits or nkv < 8)
    for live in (9, 12, 16):
        count = dev(torch.tensor([live], dtype=torch.int32))
        out = K().attention_decode_bf16(*args, live=(count, least))
        assert_attention_close(out, want)


@pytest.mark.parametrize("nh,nkv,d,bs", [(16, 8, 128, 16), (4, 2, 64, 16), (6, 1, 96, 32), (8, 8, 256, 16), (32, 2, 64, 16)])
@pytest.mark.parametrize("window", [0, 100])
def test_attention_decode_with_few_splits_in_one_block(nh, nkv, d, bs, window):
    """Steps of many items have few splits per item: one block then takes all splits of its heads, a wave
    each, and writes the finished output (no second kernel). Items of very different lengths, among them
    some shorter than the number of splits, with and without the norm / rotary / page-write prologue."""
    dtype = torch.bfloat16
    ctxs = [500, 16, 17, 333, 450, 255, 64, 65, 1, 2, 3, 40] * 3
    items = [(c - 1, 1) for c in ctxs]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=700)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(6)
    qs = [torch.randn(1, nh, d, generator=g).to(dtype) for _ in items]
    scale = d**-0.5
    want = dense_reference(qs, ks, vs, items, scale, window)
    item_ctx = torch.tensor(ctxs, dtype=torch.int32)
    max_ctx = 512
    chunks = -(-(nh // nkv) // 16)
    splits = K().decode_splits(len(items), nkv * chunks, max_ctx)[1]
    assert 1 < splits <= (8 if d <= 128 else 4), splits  # few enough for one block
    wide = torch.zeros(len(items), max_ctx // bs, dtype=torch.int32)
    wide[:, : table_t.shape[1]] = table_t
    out = K().attention_decode_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide), scale,
                                    window, max_ctx)
    assert_attention_close(out, want)
    # padding behind the live items: fewer live items, more of the block's waves at work
    count = dev(torch.tensor([len(items) - 7], dtype=torch.int32))
    out = K().attention_decode_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide), scale,
                                    window, max_ctx, live=(count, len(items) - 10))
    assert_attention_close(out, want)


def test_attention_decode_many_splits():
    """A long context of one item is cut into more splits than a wave has lanes; a far key is made to
    dominate so that a split that is dropped or weighted wrongly shows."""
    dtype = torch.bfloat16
    nh, nkv, d, bs = 4, 1, 64, 16
    ctx = 9000
    items = [(ctx - 1, 1), (4999, 1)]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=900)
    g = torch.Generator().manual_seed(3)
    qs = [torch.randn(1, nh, d, generator=g).to(dtype) for _ in items]
    ks[0][1234] = (qs[0][0, 1:2].float() * 2.0).to(dtype)  # head 1 of item 0 looks at key 1234 almost alone
    k_cache[tables[0][1234 // bs], :, 1234 % bs, :] = ks[0][1234]
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    scale = d**-0.5
    want = dense_reference(qs, ks, vs, items, scale, 0)
    item_ctx = torch.tensor([ctx, 5000], dtype=torch.int32)
    max_ctx = 16384
    wide = torch.zeros(len(items), max_ctx // bs, dtype=torch.int32)
    wide[:, : table_t.shape[1]] = table_t
    assert K().decode_splits(len(items), nkv, max_ctx)[1] > 64
    out = K().attention_decode_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(item_ctx), dev(wide), scale, 0,
                                    max_ctx)
    assert_attention_close(out, want)


@pytest.mark.parametrize("nh,nkv,d,bs", [s for s in MFMA_SHAPES if s[0] // s[1] <= 16])
@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("wide", [False, True])
def test_attention_prefill_mfma(nh, nkv, d, bs, window, wide):
    """Blocks of 128 and of 256 query columns (the step's size chooses between them in the engine)."""
    dtype = torch.bfloat16
    items = [(0, 7), (9, 1), (8, 5), (0, 1), (15, 1), (16, 33), (63, 2), (130, 1), (60, 70), (0, 200), (300, 129)]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=256)
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    g = torch.Generator().manual_seed(5)
    qs = [torch.randn(n, nh, d, generator=g).to(dtype) for _, n in items]
    scale = d**-0.5
    qlens = [n for _, n in items]
    item_start = torch.tensor([0] + torch.tensor(qlens).cumsum(0).tolist(), dtype=torch.int32)
    plan = K().prefill_plan([c for c, _ in items], qlens, nh, nkv, d, window, torch.device("cuda:0"), wide=wide)
    assert plan.columns == (256 if wide else 128)
    out = K().attention_prefill_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(positions), dev(item_start),
                                     qlens, dev(table_t), scale, window, plan=plan)
    want = dense_reference(qs, ks, vs, items, scale, window)
    assert_attention_close(out, want)


@pytest.mark.parametrize("nh,nkv,d,bs,window", [(4, 2, 64, 16, 0), (16, 8, 128, 16, 0), (3, 1, 96, 64, 900)])
@pytest.mark.parametrize("wide", [False, True])
def test_attention_prefill_cuts_long_tiles_when_the_step_is_small(nh, nkv, d, bs, window, wide):
    """A short portion over a long context: too few tiles to fill the chip, so their keys are cut into
    ranges and added up by the second kernel. One far key dominates a head, so that a range that is
    dropped or weighted wrongly shows; a second, short item stays in one piece beside it."""
    dtype = torch.bfloat16
    items = [(3000, 70), (0, 5)]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=256)
    g = torch.Generator().manual_seed(11)
    qs = [torch.randn(n, nh, d, generator=g).to(dtype) for _, n in items]
    far = 2500
    ks[0][far, 0] = (qs[0][3, 0].float() * 1.5).to(dtype)  # token 3, head 0 of item 0 looks at key 2500
    k_cache[tables[0][far // bs], :, far % bs, :] = ks[0][far]
    fill_new(k_cache, v_cache, tables, ks, vs, items, bs)
    scale = d**-0.5
    qlens = [n for _, n in items]
    starts = [c for c, _ in items]
    item_start = torch.tensor([0] + torch.tensor(qlens).cumsum(0).tolist(), dtype=torch.int32)
    plan = K().prefill_plan(starts, qlens, nh, nkv, d, window, torch.device("cuda:0"), wide=wide)
    assert plan.max_chunks > 1 and plan.columns == (256 if wide else 128)
    out = K().attention_prefill_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(positions), dev(item_start),
                                     qlens, dev(table_t), scale, window, plan=plan)
    want = dense_reference(qs, ks, vs, items, scale, window)
    assert_attention_close(out, want)
    # and without a plan from the caller: the item starts are read back from the positions
    out2 = K().attention_prefill_bf16(dev(torch.cat(qs)), dev(k_cache), dev(v_cache), dev(positions), dev(item_start),
                                      qlens, dev(table_t), scale, window)
    assert_attention_close(out2, want)


@pytest.mark.parametrize("nh,nkv,d,bs", [(4, 2, 64, 16), (16, 8, 128, 16), (6, 1, 128, 32), (2, 2, 256, 16)])
@pytest.mark.parametrize("norm,rotary,window", [(True, True, 0), (False, True, 37), (True, False, 0)])
def test_attention_decode_fused_equals_the_two_kernels(nh, nkv, d, bs, norm, rotary, window):
    """The decode kernel with the norm / rotary / page-write prologue against qk_norm_rope_scatter
    followed by the plain decode kernel: same cache contents, same output."""
    dtype = torch.bfloat16
    ctxs = [1, 16, 17, 33, 100, 255, 64, 65, 700]
    items = [(c - 1, 1) for c in ctxs]
    k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, num_pages=160)
    assert K().attention_decode_fused_supported(d, bs, d if rotary else 0, nh // nkv)
    g = torch.Generator().manual_seed(2)
    qkv = torch.randn(len(items), (nh + 2 * nkv) * d, generator=g).to(dtype)
    qw, kw = (dev(1 + 0.2 * torch.randn(d, generator=g)), dev(1 + 0.2 * torch.randn(d, generator=g))) if norm else (None, None)
    inv_freq = 1.0 / (1e4 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    rope = K().rope_table(dev(inv_freq), 4096) if rotary else None
    item_ctx, scale = dev(torch.tensor(ctxs, dtype=torch.int32)), d**-0.5
    wide = torch.zeros(len(items), 4096 // bs, dtype=torch.int32)
    wide[:, : table_t.shape[1]] = table_t
    kc1, vc1, kc2, vc2 = dev(k_cache.clone()), dev(v_cache.clone()), dev(k_cache.clone()), dev(v_cache.clone())
    q = K().qk_norm_rope_scatter(dev(qkv), qw, kw, rope, dev(positions), dev(token_item), dev(wide), kc1, vc1, nh, nkv, d, 1e-5)
    want = K().attention_decode_bf16(q, kc1, vc1, item_ctx, dev(wide), scale, window, 4096)
    got = K().attention_decode_fused_bf16(dev(qkv), qw, kw, rope, 1e-5, True, kc2, vc2, item_ctx, dev(wide), nh, scale,
                                          window, 4096)
    # values are copied bit for bit; keys go through a float32 norm whose sum the two kernels take in
    # different orders, so a key may differ in its last bfloat16 bit
    assert torch.equal(vc1, vc2)
    torch.testing.assert_close(kc1.float(), kc2.float(), rtol=2**-7, atol=1e-6)
    torch.testing.assert_close(got.float(), want.float(), rtol=1e-2, atol=1e-2)
    assert not K().attention_decode_fused_supported(96, 16, 96, 1)
    assert not K().attention_decode_fused_supported(128, 16, 64, 1)


@pytest.mark.parametrize("kernel", ["decode", "prefill"])
def test_mfma_attention_finds_one_far_key_and_respects_the_window_edge(kernel):
    dtype, nh, nkv, d, bs, ctx = torch.bfloat16, 4, 2, 64, 16, 600
    for hot, window in [(0, 0), (15, 0), (16, 0), (63, 0), (64, 0), (511, 0), (512, 0), (598, 0), (599, 0),
                        (ctx - 100, 100), (ctx - 101, 100)]:
        items = [(ctx - 1, 1)]
        k_cache, v_cache, tables, table_t, positions, token_item, ks, vs = make_paged(items, nkv, d, bs, dtype, seed=hot)
        direction = torch.randn(d)
        direction /= direction.norm()
        ks[0] = (ks[0].float() * 0.05).to(dtype)
        ks[0][hot] = (direction * 8).to(dtype)
        fill_new(k_cache, v_cache, tables, ks, vs, [(0, ctx)], bs)
        q = (direction * 40).expand(1, nh, d).to(dtype).contiguous()
        if kernel == "decode":
            out = K().attention_decode_bf16(dev(q), dev(k_cache), dev(v_cache), dev(torch.tensor([ctx], dtype=torch.int32)),
                                            dev(table_t), d**-0.5, window, ctx)
        else:
            out = K().attention_prefill_bf16(dev(q), dev(k_cache), dev(v_cache), dev(positions),
                                             dev(torch.tensor([0, 1], dtype=torch.int32)), [1], dev(table_t), d**-0.5, window)
        out = out.float().cpu()
        hot_v = vs[0][hot].float().repeat_interleave(nh // nkv, dim=0).reshape(1, -1)
        seen = window == 0 or hot >= ctx - window
        if seen:
            assert_attention_close(out, hot_v)
        else:
            assert (out - hot_v).abs().max() > 0.3
            assert_attention_close(out, dense_reference([q], ks, vs, items, d**-0.5, window))


def test_mfma_attention_refuses_unsupported_sizes():
    assert not K().attention_mfma_supported(16, 16)
    assert not K().attention_mfma_supported(128, 8) and not K().attention_mfma_supported(128, 48)
    assert K().attention_mfma_supported(128, 16) and not K().attention_mfma_supported(128, 16, group=17)
    from mini_engine_amd.ops.library import KernelError

    q = dev(torch.zeros(1, 2, 16, dtype=torch.bfloat16))
    kc, vc = dev(torch.zeros(2, 1, 16, 16, dtype=torch.bfloat16)), dev(torch.zeros(2, 1, 16, 16, dtype=torch.bfloat16))
    with pytest.raises(KernelError, match="not supported"):
        K().attention_decode_bf16(q, kc, vc, dev(torch.ones(1, dtype=torch.int32)), dev(torch.zeros(1, 1, dtype=torch.int32)), 1.0, 0, 16)
