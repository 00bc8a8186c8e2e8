import numpy as np
import torch


def rel_err(got, want):
    """(max-norm relative error, L2 relative error) of got vs want, both taken in fp64 on the host."""
    g = torch.as_tensor(got).detach().to("cpu", torch.float64)
    w = torch.as_tensor(want).detach().to("cpu", torch.float64)
    assert g.shape == w.shape, (g.shape, w.shape)
    scale = w.abs().max().item()
    l2 = w.norm().item()
    if scale == 0.0:
        return g.abs().max().item(), g.norm().item()
    return (g - w).abs().max().item() / scale, (g - w).norm().item() / l2


def assert_close(got, want, tol, what="", floor=None):
    """floor: magnitude below which `want` counts as zero (a gradient that vanishes identically,
    e.g. the key bias under softmax); errors are then taken relative to the floor instead."""
    if floor is not None and torch.as_tensor(want).abs().max().item() < 1e-6 * floor:
        g = torch.as_tensor(got).detach().to("cpu", torch.float64)
        mx = g.abs().max().item() / floor
        assert mx <= tol, "%s: |got| %.3e vs floor %.3e > tol %.1e" % (what, mx * floor, floor, tol)
        return mx, mx
    mx, l2 = rel_err(got, want)
    assert mx <= tol and l2 <= tol, "%s: rel max %.3e, rel l2 %.3e > tol %.1e" % (what, mx, l2, tol)
    return mx, l2


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a) if isinstance(a, np.ndarray) else a)
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda().contiguous()


def grad_scale(grads, name):
    """Magnitude a weight gradient is judged on: its own largest entry, except for the key bias of an attention layer, whose
    gradient vanishes identically (a key bias shifts every score of a row equally) - that one is judged on the query bias's."""
    ref = name.replace("/key/bias", "/query/bias") if name.endswith("/key/bias") else name
    return float(grads[ref].abs().max())
