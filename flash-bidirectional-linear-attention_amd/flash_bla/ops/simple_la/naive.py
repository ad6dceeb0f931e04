"""Plain-torch formula of simple_la (counterpart of flash_bla/ops/simple_la/naive.py:8-20)."""


def naive_simple_la(q, k, v, scale=None):
    if scale is None:
        scale = q.shape[-1] ** -0.5
    s = k.transpose(-2, -1) @ (v * scale)
    return q @ s
