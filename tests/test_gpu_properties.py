"""Size-independent properties of the HIP path at the full benchmark sizes, where the CPU oracle would take minutes.

Every property below is exact -- bit for bit -- because it leaves the order of the float32 additions of an output
untouched and changes the operands only in ways float16 / float32 arithmetic carries without rounding:

* doubling the activations, or the group scales, doubles every product exactly (a power of two, no overflow and
  nothing subnormal at these magnitudes), hence every partial sum and the rounded output;
* permuting the rows of x permutes the rows of y: an output's sum over k does not depend on the row it sits in;
* permuting the weight rows (packed words and scales together) permutes the columns of y: nor on its column.

A kernel that dropped, duplicated or misplaced a tile, a K window or a row at full size fails them; the oracle
comparisons at these sizes (sampled rows, in the parity tests) pin the values themselves."""
import pytest
import torch

pytestmark = pytest.mark.gpu

LLAMA7B = [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]
LLAMA13B = [(15360, 5120), (5120, 5120), (27648, 5120), (5120, 13824)]
CASES = ([(4, 32, n, k, m) for n, k in LLAMA7B for m in (1, 8, 512, 2048)] +
         [(8, 128, n, k, m) for n, k in LLAMA13B for m in (1, 16, 256)])


def _case(bits, group, n, k, m, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    per = 32 // bits
    wq = torch.randint(-2**31, 2**31 - 1, (n, k // per), dtype=torch.int32, device="cuda", generator=g)
    s = (torch.rand((n, k // group), device="cuda", generator=g) * 0.015 + 0.005).to(torch.float16)
    x = torch.randn((m, k), device="cuda", generator=g).to(torch.float16)
    return x, wq, s


def _same(got, want, what):
    """Bit-equal wherever the expected value is a normal float16 with room to spare; below that (a handful of
    outputs that happen to lie within 2^-13 of zero) a subnormal's fixed spacing makes round(2 a) differ from
    2 round(a), so those compare to within one subnormal step."""
    got, want = got.contiguous(), want.contiguous()
    assert got.shape == want.shape, what
    normal = want.float().abs() >= 2.0 ** -12
    assert torch.equal(got.view(torch.int16)[normal], want.view(torch.int16)[normal]), what
    rest = ~normal
    assert int(rest.sum()) <= max(4, want.numel() // 1000), (what, "too many near-zero outputs")
    assert bool(((got.float() - want.float()).abs()[rest] <= 2.0 ** -23).all()), (what, "near-zero outputs")


@pytest.mark.parametrize("bits,group,n,k,m", CASES)
def test_exact_properties_at_full_size(bits, group, n, k, m):
    import relax_amd

    x, wq, s = _case(bits, group, n, k, m, 4000 + bits + n % 97 + k % 89 + m)
    y = relax_amd.wq_matmul(x, wq, s, bits, group)
    torch.cuda.synchronize()
    assert torch.isfinite(y).all()
    assert float(y.float().abs().max()) < 16000.0  # doubling stays finite
    assert float(y.float().abs().mean()) > 0.05    # and the outputs are no zeros

    # doubling x, doubling the scales
    y2x = relax_amd.wq_matmul(x * 2, wq, s, bits, group)
    y2s = relax_amd.wq_matmul(x, wq, s * 2, bits, group)
    torch.cuda.synchronize()
    _same(y2x, y * 2, "y(2x) != 2 y(x)")
    _same(y2s, y * 2, "y(2s) != 2 y(s)")

    # rows of x permuted
    g = torch.Generator(device="cuda").manual_seed(77)
    if m > 1:
        pm = torch.randperm(m, device="cuda", generator=g)
        yp = relax_amd.wq_matmul(x[pm].contiguous(), wq, s, bits, group)
        torch.cuda.synchronize()
        assert torch.equal(yp.view(torch.int16), y[pm].contiguous().view(torch.int16)), "rows of x permuted"

    # weight rows permuted
    pn = torch.randperm(n, device="cuda", generator=g)
    yn = relax_amd.wq_matmul(x, wq[pn].contiguous(), s[pn].contiguous(), bits, group)
    torch.cuda.synchronize()
    assert torch.equal(yn.view(torch.int16), y[:, pn].contiguous().view(torch.int16)), "weight rows permuted"
