"""Shared helpers of the parity tests."""
import torch

OUTLIER_CHANNELS = (7, 33, 71, 101)


def make_qkv(B, Hq, Hkv, Lq, Lk, D, dtype, seed=0, outliers=False, device="cpu"):
    """Seeded N(0,1) inputs generated on the host in fp32, then cast (and moved)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, Hq, Lq, D, generator=g)
    k = torch.randn(B, Hkv, Lk, D, generator=g)
    v = torch.randn(B, Hkv, Lk, D, generator=g)
    if outliers:
        for c in OUTLIER_CHANNELS:
            if c < D:
                k[..., c] *= 8.0
    return q.to(dtype).to(device), k.to(dtype).to(device), v.to(dtype).to(device)


def rel_err(a, b):
    a, b = a.detach().float().cpu(), b.detach().float().cpu()
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def support(mask_dense):
    return (mask_dense.detach().float().cpu() != 0)


def tie_aware_equal(sel_a, sel_b, scores):
    """sel_*: bool (R, n) selections of k entries per row; scores (R, n). True when, per row,
    both picked every entry strictly above the k-th score and the same number at it."""
    sel_a, sel_b, scores = sel_a.cpu(), sel_b.cpu(), scores.float().cpu()
    for r in range(scores.shape[0]):
        sa, sb = scores[r][sel_a[r]], scores[r][sel_b[r]]
        if sa.numel() != sb.numel():
            return False
        if sa.numel() == 0:
            continue
        thr = sa.min()
        if sb.min() != thr:
            return False
        above = scores[r] > thr
        if not (torch.equal(sel_a[r] & above, above) and torch.equal(sel_b[r] & above, above)):
            return False
    return True
