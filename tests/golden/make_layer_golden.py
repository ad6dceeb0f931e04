#!/usr/bin/env python3
"""Writes tests/golden/layer_<name>.npz: the arithmetic of the reference's attention blocks
(flash_bla/layers/{mlla,rala,focused_la,polaformer}.py) in mode='torch', on the CPU, at tiny
shapes (float64, float32 for the two blocks with RoPE): seeded parameters (the state dict), an input, the output and the input gradient.

Run once in the build container, where /root/reference exists:

    python tests/golden/make_layer_golden.py

Nothing else pins these blocks' arithmetic (RoPE pair layout, RALA's efficiency weighting, the
norm-preserving focusing power, the PVT spatial reduction, the polarity split): the reference has
no test for them, and their self-tests compare the two modes of one block with each other.  Each
reference file is loaded by path, alone; `flash_bla.ops.*` and `flash_bla.utils`, which the files
import at the top but do not use in mode='torch', resolve to this repository's package, so no
Triton kernel is imported or run.  rala.py takes RoPE from the reference's mlla.py.  The fixtures
hold data only (arrays), no source text.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF_LAYERS = "/root/reference/flash_bla/layers"
sys.path.insert(0, os.path.join(ROOT, "flash-bidirectional-linear-attention_amd"))


def load_reference(name, stand_ins=None):
    """The reference's layers/<name>.py as a module of its own (`ref_<name>`)."""
    saved = {}
    for mod_name, module in (stand_ins or {}).items():
        saved[mod_name] = sys.modules.get(mod_name)
        sys.modules[mod_name] = module
    try:
        spec = importlib.util.spec_from_file_location("ref_" + name, os.path.join(REF_LAYERS, name + ".py"))
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
    finally:
        for mod_name, old in saved.items():
            if old is None:
                sys.modules.pop(mod_name, None)
            else:
                sys.modules[mod_name] = old
    return module


# name -> (reference file, class, constructor kwargs, input shape, extra forward args, dtype).  The blocks
# take the token grid as square (h = w = sqrt(n)); RoPE computes in float32 whatever it is given
# (mlla.py:32-33), so the two blocks that use it are evaluated in float32, the others in float64.
CASES = {
    "mlla": ("mlla", "MambaLikeLinearAttention", dict(dim=32, input_resolution=(5, 5), num_heads=2), (2, 25, 32), (),
             torch.float32),
    "rala": ("rala", "RALALinearAttention", dict(dim=32, input_resolution=(5, 5), num_heads=2), (2, 25, 32), (),
             torch.float32),
    "focused": ("focused_la", "FocusedLinearAttention", dict(dim=32, num_patches=25, num_heads=2),
                (2, 25, 32), (5, 5), torch.float64),
    "focused_sr2": ("focused_la", "FocusedLinearAttention", dict(dim=32, num_patches=16, num_heads=2, sr_ratio=2),
                    (2, 16, 32), (4, 4), torch.float64),
    "pola": ("polaformer", "PolaLinearAttention", dict(dim=32, num_patches=25, num_heads=2), (2, 25, 32), (5, 5),
             torch.float64),
    "pola_sr2": ("polaformer", "PolaLinearAttention", dict(dim=32, num_patches=16, num_heads=2, sr_ratio=2),
                 (2, 16, 32), (4, 4), torch.float64),
}


def main():
    ref_mlla = load_reference("mlla")
    modules = {"mlla": ref_mlla,
               "rala": load_reference("rala", {"flash_bla.layers.mlla": ref_mlla}),
               "focused_la": load_reference("focused_la"),
               "polaformer": load_reference("polaformer")}
    for name, (file, cls, kwargs, shape, extra, dtype) in CASES.items():
        torch.manual_seed(1234)
        block = getattr(modules[file], cls)(**kwargs).to(dtype).eval()
        with torch.no_grad():  # parameters that start at zero or one would hide their own use
            for pname, prm in block.named_parameters():
                if prm.ndim >= 1 and (prm.abs().max() == 0 or (prm == 1).all()):
                    prm.add_(0.3 * torch.randn(prm.shape, dtype=prm.dtype))
        x = torch.randn(shape, dtype=dtype, requires_grad=True)
        dy = torch.randn(shape, dtype=dtype)
        y = block(x, *extra, mode="torch")
        y.backward(dy)
        arrays = {"param." + k: v.detach().numpy() for k, v in block.state_dict().items()}
        arrays.update(x=x.detach().numpy(), dy=dy.numpy(), y=y.detach().numpy(), dx=x.grad.numpy())
        arrays["kwargs"] = np.array(repr(kwargs))
        arrays["extra"] = np.array(extra, dtype=np.int64)
        out = os.path.join(HERE, f"layer_{name}.npz")
        np.savez_compressed(out, **arrays)
        print(f"{out}: {len(arrays)} arrays, |y| max {y.abs().max().item():.4f}")


if __name__ == "__main__":
    main()
