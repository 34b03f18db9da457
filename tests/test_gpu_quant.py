"""GPU parity: fp8 e4m3fn block quantiser vs the closed-form oracle (bit-exact bytes and scales).
The reference has no such kernel: parity unpinned against it, pinned by closed forms."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("lens", [[256], [300, 1, 128], [80]])
def test_quant_fp8_block_bit_exact(dev, dtype, lens):
    import flashomni_amd as fo
    heads = 3
    g = torch.Generator().manual_seed(sum(lens))
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    x = (torch.randn(int(indptr[-1]), heads, 128, generator=g) * 3).to(dtype)
    x[:64, 1] = 0          # an all-zero (head, block) slab where a block has <= 64 rows
    if x.shape[0] >= 128:
        x[:128, 1] = 0     # all-zero full block -> scale 1
    x8, scale = fo.quant_fp8_block(x.to(dev), indptr)
    e8, es = oracle.quant_fp8_block(x, indptr)
    assert torch.equal(scale.cpu(), es)
    assert torch.equal(x8.cpu().view(torch.uint8), e8.view(torch.uint8))
    # closed forms: every non-zero block reaches +-448; dequantisation error <= 2^-4 relative (+ denormal floor)
    deq = oracle.dequant_fp8_block(x8.cpu(), scale.cpu(), indptr)
    err = (deq - x.float()).abs()
    bound = x.float().abs() * 2 ** -4 + scale.cpu().max() * 2 ** -9
    assert bool((err <= bound).all())


@pytest.mark.parametrize("lens", [[256], [300, 1, 128]])
def test_quant_fp8_block_residual(dev, lens):
    """The second term is the same rounding applied to what the first left: bit-exact against the
    oracle, and the two terms together carry x to 2^-8 relative (two 3-bit-mantissa roundings)."""
    import flashomni_amd as fo
    heads = 2
    g = torch.Generator().manual_seed(7 + sum(lens))
    indptr = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    x = (torch.randn(int(indptr[-1]), heads, 128, generator=g) * 2).to(torch.bfloat16)
    x8, scale, lo = fo.quant_fp8_block(x.to(dev), indptr, residual=True)
    e8, es, elo = oracle.quant_fp8_block(x, indptr, residual=True)
    assert torch.equal(scale.cpu(), es)
    assert torch.equal(x8.cpu().view(torch.uint8), e8.view(torch.uint8))
    assert torch.equal(lo.cpu().view(torch.uint8), elo.view(torch.uint8))
    one = oracle.dequant_fp8_block(x8.cpu(), scale.cpu(), indptr)
    two = one + oracle.dequant_fp8_block(lo.cpu(), scale.cpu(), indptr)
    floor = scale.cpu().max() * 2 ** -10
    assert bool(((two - x.float()).abs() <= x.float().abs() * 2 ** -8 + floor).all())
    assert float((two - x.float()).norm()) < 0.1 * float((one - x.float()).norm())
    # without residual=True the result is the two-tuple it always was
    assert len(fo.quant_fp8_block(x.to(dev), indptr)) == 2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quant_fp8_every_16_bit_value(dev, dtype):
    """Every 16-bit pattern of x (signed zeros and denormals included) under 40 absmax values, the
    residual term as well.  The kernel forms x / scale from the reciprocal of the scale and two fused
    corrections; slabs whose scale is below 2^-80 take the division itself: both ways must give the
    oracle's bytes.  Patterns that are not finite or exceed the slab's absmax are replaced by it."""
    import flashomni_amd as fo
    g = torch.Generator().manual_seed(11)
    every = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype).clone()
    # absmax values: random normal-range patterns, powers of two, values whose scale is tiny
    pats = torch.randint(0x0400 if dtype == torch.float16 else 0x2000, 0x7bff if dtype == torch.float16 else 0x5f00,
                         (32,), generator=g).to(torch.int16).view(dtype)
    if dtype == torch.bfloat16:
        extra = torch.tensor([1.0, 1.75, 448.0, 3.0e38, 2.0 ** -60, 2.0 ** -75, 2.0 ** -100, 2.0 ** -130])
    else:
        extra = torch.tensor([1.0, 1.75, 448.0, 65504.0, 2.0 ** -10, 2.0 ** -14, 2.0 ** -20, 2.0 ** -24])
    amaxes = torch.cat([pats, extra.to(dtype)])
    slabs = []
    for a in amaxes:
        v = every.clone()
        bad = ~torch.isfinite(v.float()) | (v.float().abs() > float(a))
        v[bad] = a
        slabs.append(v.view(4 * 128, 1, 128))  # four 128-token blocks hold the 65536 values
    x = torch.cat(slabs)
    indptr = torch.tensor([0, x.shape[0]], dtype=torch.int32)
    x8, scale, lo = fo.quant_fp8_block(x.to(dev), indptr, residual=True)
    e8, es, elo = oracle.quant_fp8_block(x, indptr, residual=True)
    assert torch.equal(scale.cpu(), es)
    assert torch.equal(x8.cpu().view(torch.uint8), e8.view(torch.uint8))
    assert torch.equal(lo.cpu().view(torch.uint8), elo.view(torch.uint8))
