"""elu(x) + 1 as one HIP launch for queries and keys: the rounding steps of torch's `F.elu(x) + 1.0`
(16-bit types: elu rounded, then + 1 rounded again; the bits agree up to the last place of the two
exp routines), the float64 closed form within rounding,
the derivative against autograd of the torch expression; sizes that are not multiples of a
16-byte vector, empty tensors, views off a 16-byte boundary and non-contiguous inputs."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _closed_form(x64):
    return np.where(x64 > 0, x64 + 1.0, np.exp(x64))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 300, 64), (1, 7), (5,), (3, 1, 129), (0, 8), (2, 4096, 640)])
def test_forward_matches_torch_and_the_closed_form(shape, dtype):
    from flash_bla.ops.feature_map import elu_plus_one
    g = torch.Generator().manual_seed(sum(shape))
    x = (3.0 * torch.randn(*shape, generator=g)).to(dtype).cuda()
    y = (3.0 * torch.randn(*shape, generator=g)).to(dtype).cuda()
    a, b = elu_plus_one(x, y)
    single = elu_plus_one(x)
    for got, inp in ((a, x), (b, y), (single, x)):
        want = F.elu(inp) + 1.0
        assert got.shape == inp.shape and got.dtype == inp.dtype
        if dtype == torch.float32:  # exp may differ in the last bit between the two libraries
            torch.testing.assert_close(got, want, rtol=2e-6, atol=1e-7)
        elif inp.numel():
            # the same rounding steps as torch: the bits agree except where the two exp routines
            # differ in the last place of the fp32 value right at a rounding boundary
            ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
            diff = (got.float() - want.float()).abs()
            assert (diff <= ulp * want.float().abs()).all()
            assert (diff > 0).float().mean().item() < 1e-3
        if inp.numel():
            ref = _closed_form(inp.double().cpu().numpy())
            tol = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2e-6}[dtype]
            err = np.abs(got.double().cpu().numpy() - ref) / np.maximum(np.abs(ref), 1.0)
            assert err.max() <= tol, err.max()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_backward_matches_autograd_of_the_torch_expression(dtype):
    from flash_bla.ops.feature_map import elu_plus_one
    g = torch.Generator().manual_seed(5)
    xs = [(2.0 * torch.randn(3, 257, 40, generator=g)).to(dtype).cuda() for _ in range(2)]
    gs = [torch.randn(3, 257, 40, generator=g).to(dtype).cuda() for _ in range(2)]
    ours = [t.clone().requires_grad_() for t in xs]
    a, b = elu_plus_one(*ours)
    (a * gs[0]).sum().backward(retain_graph=True)
    (b * gs[1]).sum().backward()
    for x, go, leaf in zip(xs, gs, ours):
        ref = x.clone().requires_grad_()
        ((F.elu(ref) + 1.0) * go).sum().backward()
        if dtype == torch.float32:
            torch.testing.assert_close(leaf.grad, ref.grad, rtol=2e-6, atol=1e-7)
        else:  # one rounding here, torch rounds exp(x) and the product separately
            torch.testing.assert_close(leaf.grad.float(), ref.grad.float(),
                                       rtol={torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype], atol=1e-6)
        want = go.double() * torch.where(x.double() > 0, torch.ones_like(x, dtype=torch.float64), x.double().exp())
        tol = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, torch.float32: 2e-6}[dtype]
        err = (leaf.grad.double() - want).abs() / want.abs().clamp_min(1e-3)
        assert err.max().item() <= tol


def test_views_and_non_contiguous_inputs():
    from flash_bla.ops.feature_map import elu_plus_one
    base = torch.randn(4 * 100 + 3, device="cuda").half()
    off = base[3:].view(4, 100)           # first element 6 bytes past a 16-byte boundary
    strided = torch.randn(6, 50, 32, device="cuda").half().transpose(0, 1)
    a, b = elu_plus_one(off, off * 2)
    torch.testing.assert_close(a, F.elu(off) + 1.0, rtol=1e-3, atol=0)
    torch.testing.assert_close(b, F.elu(off * 2) + 1.0, rtol=1e-3, atol=0)
    c = elu_plus_one(strided)
    assert c.shape == strided.shape
    torch.testing.assert_close(c, F.elu(strided) + 1.0, rtol=1e-3, atol=0)


def test_rejects_cpu_tensors_and_mixed_types():
    from flash_bla.ops.feature_map import elu_plus_one
    with pytest.raises(ValueError):
        elu_plus_one(torch.randn(4, 4))
    with pytest.raises(ValueError):
        elu_plus_one(torch.randn(4, 4, device="cuda").half(), torch.randn(4, 4, device="cuda"))
    with pytest.raises(TypeError):
        elu_plus_one(torch.ones(4, 4, device="cuda", dtype=torch.int32))
