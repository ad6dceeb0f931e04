"""Layer counterparts: `mode='torch'` runs anywhere (CPU shapes check), on the GPU
`mode='triton'` (the HIP operators) must agree with it for the output and the
input gradient, with the acceptance rule of the reference layers' self-tests
(flash_bla/utils.py:55-67 with ratio 0.06; layers/linfusion.py:116-141 etc.)."""
import ast
import os

import numpy as np
import pytest
import torch

from flash_bla.layers import (FocusedLinearAttention, GeneralizedLinearAttention, MambaLikeLinearAttention,
                              PolaLinearAttention, RALALinearAttention)
from flash_bla.utils import assert_close

CASES = {
    "linfusion": (lambda: GeneralizedLinearAttention(256, heads=4, dim_head=64), (2, 144, 256), ()),
    "mlla": (lambda: MambaLikeLinearAttention(128, (12, 12), 4), (2, 144, 128), ()),
    "rala": (lambda: RALALinearAttention(128, (12, 12), 4), (2, 144, 128), ()),
    "focused": (lambda: FocusedLinearAttention(256, 144, num_heads=4), (2, 144, 256), (12, 12)),
    "pola": (lambda: PolaLinearAttention(128, 144, num_heads=4), (2, 144, 128), (12, 12)),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_torch_mode_on_cpu(name):
    torch.manual_seed(0)
    make, shape, extra = CASES[name]
    layer = make()
    x = torch.randn(shape, requires_grad=True)
    y = layer(x, *extra, mode='torch')
    assert y.shape == x.shape and torch.isfinite(y).all()
    y.sum().backward()
    assert torch.isfinite(x.grad).all()
    with pytest.raises(NotImplementedError):
        layer(x, *extra, mode='flash')


def test_linfusion_state_dict_names():
    names = set(GeneralizedLinearAttention(64, heads=1, dim_head=64).state_dict())
    assert {"to_q.weight", "to_k.weight", "to_v.weight", "to_out.0.weight", "to_out.0.bias",
            "to_q_.0.weight", "to_q_.1.weight", "to_q_.3.bias", "to_k_.3.weight"} <= names
    assert "to_q.bias" not in names


def test_state_dict_names_and_shapes_follow_the_reference_modules():
    """A checkpoint of the reference's blocks must load: parameter / buffer names and shapes as the
    reference's constructors create them (layers/mlla.py:29,54-57, rala.py:30-34,
    focused_la.py:24-39, polaformer.py:22-40; qkv_bias defaults to False in the PVT-style blocks,
    True in MLLA / RALA)."""
    dim, heads, res = 64, 4, (4, 4)
    want = {
        "mlla": (MambaLikeLinearAttention(dim, res, heads), {
            "qk.weight": (2 * dim, dim), "qk.bias": (2 * dim,), "lepe.weight": (dim, 1, 3, 3), "lepe.bias": (dim,),
            "rope.rotations": (*res, dim // 2, 2)}),
        "rala": (RALALinearAttention(dim, res, heads), {
            "qkvo.weight": (4 * dim, dim), "qkvo.bias": (4 * dim,), "lepe.weight": (dim, 1, 5, 5),
            "lepe.bias": (dim,), "rope.rotations": (*res, dim // heads // 2, 2), "proj.weight": (dim, dim),
            "proj.bias": (dim,)}),
        "focused": (FocusedLinearAttention(dim, 16, num_heads=heads, sr_ratio=2), {
            "q.weight": (dim, dim), "kv.weight": (2 * dim, dim), "proj.weight": (dim, dim), "proj.bias": (dim,),
            "sr.weight": (dim, dim, 2, 2), "sr.bias": (dim,), "norm.weight": (dim,), "norm.bias": (dim,),
            "dwc.weight": (dim // heads, 1, 5, 5), "dwc.bias": (dim // heads,), "scale": (1, 1, dim),
            "positional_encoding": (1, 16 // 4, dim)}),
        "pola": (PolaLinearAttention(dim, 16, num_heads=heads, sr_ratio=2), {
            "qg.weight": (2 * dim, dim), "kv.weight": (2 * dim, dim), "proj.weight": (dim, dim), "proj.bias": (dim,),
            "sr.weight": (dim, dim, 2, 2), "sr.bias": (dim,), "norm.weight": (dim,), "norm.bias": (dim,),
            "dwc.weight": (dim // heads, 1, 5, 5), "dwc.bias": (dim // heads,), "power": (1, heads, 1, dim // heads),
            "scale": (1, 1, dim), "positional_encoding": (1, 16 // 4, dim)}),
    }
    for name, (module, shapes) in want.items():
        got = {k: tuple(v.shape) for k, v in module.state_dict().items()}
        assert got == shapes, name


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
GOLDEN_BLOCKS = {"mlla": MambaLikeLinearAttention, "rala": RALALinearAttention, "focused": FocusedLinearAttention,
                 "focused_sr2": FocusedLinearAttention, "pola": PolaLinearAttention, "pola_sr2": PolaLinearAttention}


def _golden_block(name, device="cpu", dtype=None):
    """Our block with the constructor arguments and the parameters of the fixture
    tests/golden/layer_<name>.npz (written by tests/golden/make_layer_golden.py from the reference's
    own block in mode='torch'), and the fixture's x, dy, y, dx."""
    data = np.load(os.path.join(GOLDEN, f"layer_{name}.npz"))
    kwargs = ast.literal_eval(str(data["kwargs"]))
    state = {k[len("param."):]: torch.from_numpy(data[k]) for k in data.files if k.startswith("param.")}
    ref_dtype = torch.from_numpy(data["y"]).dtype
    block = GOLDEN_BLOCKS[name](**kwargs).to(ref_dtype)
    block.load_state_dict(state, strict=True)   # every name and shape of the reference's state dict
    block = block.to(device, dtype or ref_dtype).eval()
    tensors = {k: torch.from_numpy(data[k]).to(device, dtype or ref_dtype) for k in ("x", "dy", "y", "dx")}
    return block, tensors, tuple(int(v) for v in data["extra"])


@pytest.mark.parametrize("name", sorted(GOLDEN_BLOCKS))
def test_torch_mode_reproduces_the_reference_block(name):
    """Arithmetic of the blocks against the reference's own modules (RoPE pair layout, RALA's
    efficiency weighting, the focusing power, the spatial reduction, the polarity split)."""
    block, t, extra = _golden_block(name)
    x = t["x"].clone().requires_grad_()
    y = block(x, *extra, mode="torch")
    y.backward(t["dy"])
    tol = 1e-9 if y.dtype == torch.float64 else 1e-5
    assert (y - t["y"]).abs().max() <= tol * t["y"].abs().max(), name
    assert (x.grad - t["dx"]).abs().max() <= tol * t["dx"].abs().max(), name


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(GOLDEN_BLOCKS))
def test_fast_mode_reproduces_the_reference_block(name):
    """mode='triton' (the HIP operators, fp32) against the reference block's torch-mode output."""
    block, t, extra = _golden_block(name, "cuda", torch.float32)
    x = t["x"].clone().requires_grad_()
    y = block(x, *extra, mode="triton")
    y.backward(t["dy"])
    assert (y - t["y"]).abs().max() <= 2e-5 * t["y"].abs().max(), name
    assert (x.grad - t["dx"]).abs().max() <= 2e-5 * t["dx"].abs().max(), name


GPU_CASES = {
    # the shapes of the reference self-tests
    "linfusion": (lambda: GeneralizedLinearAttention(1024, heads=16, dim_head=64), (2, 4096, 1024), ()),
    "mlla": (lambda: MambaLikeLinearAttention(512, (16, 16), 16), (4, 256, 512), ()),
    "rala": (lambda: RALALinearAttention(512, (16, 16), 16), (4, 256, 512), ()),
    "focused": (lambda: FocusedLinearAttention(1024, 256, num_heads=16), (4, 256, 1024), (16, 16)),
    "pola": (lambda: PolaLinearAttention(256, 256, num_heads=8), (4, 256, 256), (16, 16)),
    # keys and values reduced 2 x 2 spatially: 64 of them for 256 queries
    "focused_sr2": (lambda: FocusedLinearAttention(256, 256, num_heads=4, sr_ratio=2), (4, 256, 256), (16, 16)),
    "pola_sr2": (lambda: PolaLinearAttention(512, 256, num_heads=8, sr_ratio=2), (4, 256, 512), (16, 16)),
}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16], ids=str)
@pytest.mark.parametrize("name", sorted(GPU_CASES))
def test_fast_mode_matches_torch_mode(name, dtype):
    torch.manual_seed(1)
    make, shape, extra = GPU_CASES[name]
    layer = make().to("cuda", dtype)
    x = torch.randn(shape, device="cuda", dtype=dtype, requires_grad=True)
    do = torch.randn(shape, device="cuda", dtype=dtype)
    ref = layer(x, *extra, mode='torch')
    ref.backward(do)
    ref_dx, x.grad = x.grad.clone(), None
    out = layer(x, *extra, mode='triton')
    out.backward(do)
    assert_close("o", ref, out, 0.06)
    assert_close("dx", ref_dx, x.grad, 0.06)
    if dtype == torch.float32:
        assert (out - ref).abs().max() <= 1e-3 * ref.abs().max() + 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,channels,heads", [(4096, 640, 10), (1024, 1280, 20)])
def test_linfusion_sdxl_shapes_fp16(tokens, channels, heads):
    """BASELINE config 4: SDXL self-attention shapes, B=2, fp16, forward only."""
    torch.manual_seed(42)
    layer = GeneralizedLinearAttention(channels, heads=heads, dim_head=64).to("cuda", torch.float16)
    x = torch.randn(2, tokens, channels, device="cuda", dtype=torch.float16)
    with torch.no_grad():
        out = layer(x, mode='triton')
        ref = layer.float()(x.float(), mode='torch')
    assert_close("o", ref, out.float(), 0.06)
    assert (out.float() - ref).abs().max() <= 5e-3 * ref.abs().max()


@pytest.mark.gpu
def test_captured_forward_replays_the_block_bit_for_bit():
    """The LinFusion block's inference forward recorded into a HIP graph: replays on new inputs,
    with eager work in between, equal the eager block bit for bit."""
    from flash_bla.utils import CapturedForward
    torch.manual_seed(3)
    layer = GeneralizedLinearAttention(640, heads=10, dim_head=64).to("cuda", torch.float16).eval()
    x = torch.randn(2, 1024, 640, device="cuda", dtype=torch.float16)
    graphed = CapturedForward(layer, x, mode="triton")
    for i in range(4):
        xi = torch.randn(2, 1024, 640, device="cuda", dtype=torch.float16)
        with torch.no_grad():
            eager = layer(xi, mode="triton")
            torch.cuda.synchronize()
            got = graphed(xi).clone()
        assert torch.equal(got, eager), f"replay {i}"
