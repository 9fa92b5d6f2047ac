"""Error figures shared by the GPU parity tests."""
import torch


def rel(a, b):
    """max |a - b| over max |b|, the whole tensor as one scale."""
    b = b.detach().float().cpu()
    return float((a.detach().float().cpu() - b).abs().max() / b.abs().max().clamp_min(1e-20))


def rel_per_expert(a, b, with_rms=False):
    """Per-expert figure for tensors whose first dimension is the expert: every slice [e] is measured against its OWN
    scale max |b[e]|, so that the gradient of a one-row or near-empty group (a few % of the largest group's) cannot
    hide behind the global maximum.  A slice whose reference is exactly zero (a group without rows) must be exactly
    zero too.  Returns the worst slice's max-relative error (and, on request, the worst slice's RMS-relative error)."""
    a = a.detach().float().cpu()
    b = b.detach().float().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    worst, worst_rms = 0.0, 0.0
    for e in range(b.shape[0]):
        scale = float(b[e].abs().max())
        if scale == 0.0:
            if float(a[e].abs().max()) != 0.0:
                worst, worst_rms = float("inf"), float("inf")
            continue
        diff = a[e] - b[e]
        worst = max(worst, float(diff.abs().max()) / scale)
        worst_rms = max(worst_rms, float(diff.pow(2).mean().sqrt() / b[e].pow(2).mean().sqrt()))
    return (worst, worst_rms) if with_rms else worst
