"""Shared helpers of the test-suite: synthetic configurations and error metrics."""
import numpy as np
import torch


def rel_err(got, ref):
    """max |got - ref| / max |ref| in float64 (0/0 -> 0)."""
    got = got.detach().to("cpu", torch.float64)
    ref = ref.detach().to("cpu", torch.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if ref.numel() == 0:
        return 0.0
    scale = ref.abs().max().item()
    err = (got - ref).abs().max().item()
    return err / scale if scale > 0 else err


def close_stats(got, ref, floor=1.0):
    """(normwise, elementwise, rms) error of ``got`` against the float64 reference:
    normwise    = max|d| / max|ref|;
    elementwise = max over elements of |d| / (|ref| + floor * rms(ref)): an element much smaller
                  than the typical magnitude is held to an absolute bound of tol * floor * rms, every
                  other element to a relative one;
    rms         = rms(d) / rms(ref): rounding noise averages out in it, a systematic error (a missing
                  or doubled term of a sum) does not."""
    got = got.detach().to("cpu", torch.float64)
    ref = ref.detach().to("cpu", torch.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if ref.numel() == 0:
        return 0.0, 0.0, 0.0
    diff = (got - ref).abs()
    scale = ref.abs().max().item()
    rms = ref.pow(2).mean().sqrt().item()
    if rms == 0:
        worst = diff.max().item()
        return worst, worst, worst
    return diff.max().item() / scale, (diff / (ref.abs() + floor * rms)).max().item(), diff.pow(2).mean().sqrt().item() / rms


def assert_close(got, ref, tol, what="", floor=1.0):
    """Three bounds: max|d| <= tol max|ref|; |d| <= tol (|ref| + floor rms(ref)) for every element;
    rms(d) <= tol / 2 * rms(ref)."""
    norm, elem, rms = close_stats(got, ref, floor)
    assert norm <= tol and elem <= tol and rms <= tol / 2, \
        f"{what}: normwise {norm:.3e}, elementwise {elem:.3e}, rms {rms:.3e}, tolerance {tol:.1e}"


# tolerance of the comparison against the float64 oracle, per compute dtype
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2, torch.float64: 1e-10}


def zipf_experts(n, n_expert, s, gen):
    p = (torch.arange(1, n_expert + 1, dtype=torch.float64)) ** (-s)
    p = p / p.sum()
    perm = torch.randperm(n_expert, generator=gen)
    return perm[torch.multinomial(p, n, replacement=True, generator=gen)]


def ragged_counts(total, n_expert, gen, empties=1):
    """Random expert counts summing to `total`, with `empties` experts forced to 0."""
    w = torch.rand(n_expert, generator=gen) + 0.05
    if n_expert > empties:
        w[torch.randperm(n_expert, generator=gen)[:empties]] = 0
    c = torch.floor(w / w.sum() * total).long()
    c[int(torch.argmax(w))] += total - int(c.sum())
    return c
