"""Pure-torch CPU restatement of the reference's V1/V2 paths -- TEST INFRASTRUCTURE ONLY.

These follow the *flow* of the reference's pure-PyTorch versions (which ATen ops
run, in which order, what is saved for backward) so that timing them on host
cores is a fair stand-in for "the reference on CPU", and so that they give a
second, independently written check beside the C restatement in plo_oracle.c.

  lsr      : V2, hand-derived backward   pytorch_loss/label_smooth.py:60-121
  focal    : V2, hand-derived backward   focal_loss.py:50-123 (repository root copy)
  lmargin  : V2, hand-derived backward   large_margin_softmax.py:68-140 (root copy, -inf mask)
  lovasz   : V1, autograd                pytorch_loss/lovasz_softmax.py:14-68
             with the V3 output convention (per-class losses; reduction over C).
"""
import torch
import torch.nn.functional as F


def _ignore_split(labels, ignore_index):
    ignored = labels == ignore_index
    return ignored, labels.masked_fill(ignored, 0)


class _LSRV2(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, smooth, ignore_index):
        n_cls = logits.size(1)
        w_pos, w_neg = 1.0 - smooth, smooth / n_cls
        ignored, safe = _ignore_split(labels, ignore_index)
        target = torch.full_like(logits, w_neg).scatter_(1, safe.unsqueeze(1), w_pos)
        target.masked_fill_(ignored.unsqueeze(1), 0.0)
        ctx.coeff = (n_cls - 1) * w_neg + w_pos
        ctx.save_for_backward(logits, target, ignored)
        return torch.log_softmax(logits, dim=1).neg_().mul_(target).sum(dim=1)

    @staticmethod
    def backward(ctx, grad_output):
        logits, target, ignored = ctx.saved_tensors
        grad = torch.softmax(logits, dim=1).mul_(ctx.coeff).sub_(target)
        grad.mul_(grad_output.unsqueeze(1))
        grad.masked_fill_(ignored.unsqueeze(1), 0.0)
        return grad, None, None, None


def lsr(logits, labels, lb_smooth=0.1, reduction="mean", ignore_index=-100):
    losses = _LSRV2.apply(logits, labels, lb_smooth, ignore_index)
    if reduction == "sum":
        return losses.sum()
    if reduction == "mean":
        return losses.sum() / (labels != ignore_index).sum()
    return losses


def _focal_logs(x):
    pos = x >= 0
    log_p = torch.where(pos, F.softplus(x, -1, 50), x - F.softplus(x, 1, 50))
    log_1p = torch.where(pos, F.softplus(x, -1, 50) - x, -F.softplus(x, 1, 50))
    return log_p, log_1p


class _FocalV2(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, alpha, gamma):
        probs = torch.sigmoid(logits)
        coeff = (labels - probs).abs_().pow_(gamma).neg_()
        log_p, log_1p = _focal_logs(logits)
        ce = log_p.mul_(labels).mul_(alpha).add_(log_1p.mul_(1.0 - labels).mul_(1.0 - alpha))
        ctx.stash = (coeff, probs, ce, labels, gamma, alpha)
        return ce * coeff

    @staticmethod
    def backward(ctx, grad_output):
        coeff, probs, ce, labels, gamma, alpha = ctx.stash
        d_coeff = (labels - probs).abs_().pow_(gamma - 1.0).mul_(gamma).mul_(probs).mul_(1.0 - probs)
        d_coeff = torch.where(labels < probs, d_coeff.neg(), d_coeff)
        d_ce = labels * alpha - probs * (1.0 - labels - alpha + 2.0 * labels * alpha)
        grad = d_coeff.mul_(ce).add_(d_ce.mul_(coeff)).mul_(grad_output)
        return grad, None, None, None


def focal(logits, labels, alpha=0.25, gamma=2, reduction="mean"):
    losses = _FocalV2.apply(logits, labels, alpha, gamma)
    if reduction == "mean":
        return losses.mean()
    if reduction == "sum":
        return losses.sum()
    return losses


class _LMarginV2(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, lam):
        coeff = 1.0 / (logits.size(1) - 1.0)
        hot = torch.zeros_like(logits, dtype=torch.bool).scatter_(1, labels.unsqueeze(1), True)
        others = logits.masked_fill(hot, float("-inf"))
        q = others.softmax(dim=1)
        log_q = others.log_softmax(dim=1)
        margin = q.sub_(coeff).mul_(log_q).mul_(lam / 2.0)
        margin.masked_fill_(hot, 0.0)
        ctx.stash = (logits, hot, coeff, lam)
        return margin.sum(dim=1).add_(F.cross_entropy(logits, labels, reduction="none"))

    @staticmethod
    def backward(ctx, grad_output):
        logits, hot, coeff, lam = ctx.stash
        p = logits.softmax(dim=1)
        others = logits.masked_fill(hot, float("-inf"))
        q = others.softmax(dim=1)
        qx = (q * others).masked_fill_(hot, 0.0)
        grad = (q * (others + 1.0 - qx.sum(dim=1, keepdim=True)) - coeff) * lam / 2.0
        grad.masked_fill_(hot, -1.0)
        grad = grad.add_(p).mul_(grad_output.unsqueeze(1))
        return grad, None, None


def lmargin(logits, labels, lam=0.3, reduction="mean", ignore_index=255, per_pixel=False):
    """reduction 'none' in the V2 module returns only the valid pixels; ``per_pixel=True``
    returns the V3 layout instead (full label shape, zeros at ignored pixels)."""
    ignored, safe = _ignore_split(labels, ignore_index)
    losses = _LMarginV2.apply(logits, safe, lam)
    if reduction == "mean":
        return losses[~ignored].mean()
    if reduction == "sum":
        return losses[~ignored].sum()
    if per_pixel:
        return losses * (~ignored).to(losses.dtype)
    return losses[~ignored]


def lovasz_per_class(logits, labels, ignore_index=-100):
    """-> (losses[C], errs[C, n_valid]); differentiable through torch autograd."""
    n_cls = logits.size(1)
    flat = logits.transpose(0, 1).reshape(n_cls, -1)
    labels = labels.reshape(-1)
    keep = (labels != ignore_index).nonzero(as_tuple=False).reshape(-1)
    probs = flat.softmax(dim=0)[:, keep]
    lab = labels[keep]
    hot = torch.zeros_like(probs).scatter_(0, lab.unsqueeze(0), 1.0).detach()
    errs = (hot - probs).abs()
    # stable descending order: equal errors keep pixel order
    errs_sorted, order = torch.sort(errs, dim=1, descending=True, stable=True)
    with torch.no_grad():
        hot_sorted = torch.gather(hot, 1, order)
        n_pos = hot_sorted.sum(dim=1, keepdim=True)
        inter = n_pos - hot_sorted.cumsum(dim=1)
        union = n_pos + (1.0 - hot_sorted).cumsum(dim=1)
        jacc = 1.0 - inter / union
        if errs.size(1) > 1:
            jacc[:, 1:] = jacc[:, 1:] - jacc[:, :-1]
    return torch.einsum("ab,ab->a", errs_sorted, jacc), errs


def lovasz(logits, labels, reduction="mean", ignore_index=-100):
    losses, _ = lovasz_per_class(logits, labels, ignore_index)
    if reduction == "sum":
        return losses.sum()
    if reduction == "mean":
        return losses.mean()
    return losses


def ohem_labels(logits, labels, ignore_index, score_thresh, n_min):
    """The relabelling of ohem_cpp.score_ohem_label as torch ops (csrc/ohem_label_kernel.cu:171-263):
    score = softmax probability at the label (1 at ignored pixels), stable ascending sort, every
    pixel at position >= n_min with score > score_thresh becomes ignore_index."""
    flat = labels.reshape(-1)
    if n_min >= flat.numel():
        return labels
    ign = labels == ignore_index
    probs = torch.softmax(logits.detach().float(), dim=1)
    score = probs.gather(1, labels.masked_fill(ign, 0).unsqueeze(1)).squeeze(1)
    score = score.masked_fill(ign, 1.0).reshape(-1)
    order = torch.sort(score, stable=True).indices[max(n_min, 0):]
    drop = order[score[order] > score_thresh]
    out = flat.clone()
    out[drop] = ignore_index
    return out.reshape(labels.shape)


def ohem_ce(logits, labels, score_thresh, n_min=None, ignore_index=255):
    """OhemCELoss.forward (pytorch_loss/ohem_loss.py:22-27)."""
    n_min = labels.numel() // 16 if n_min is None else n_min
    new_labels = ohem_labels(logits, labels, ignore_index, score_thresh, n_min)
    return F.cross_entropy(logits, new_labels, ignore_index=ignore_index, reduction="mean")


def taylor_log_softmax(x, dim=1, n=4):
    """LogTaylorSoftmaxV1 (pytorch_loss/taylor_softmax.py:35-44): exp replaced by its order-n series."""
    fn = torch.ones_like(x)
    denor = 1.0
    for i in range(1, n + 1):
        denor *= i
        fn = fn + x.pow(i) / denor
    return (fn / fn.sum(dim=dim, keepdim=True)).log()


def taylor_ce(logits, labels, n=4, reduction="mean", ignore_index=-1):
    """TaylorCrossEntropyLossV1.forward (pytorch_loss/taylor_softmax.py:160-173)."""
    return F.nll_loss(taylor_log_softmax(logits, 1, n), labels, reduction=reduction, ignore_index=ignore_index)


def soft_dice(logits, labels, p=1, smooth=1.0):
    """Soft dice over everything as one row (pytorch_loss/soft_dice_loss.py:10-33 with the denominator of the
    fused kernel, csrc/soft_dice_kernel_v2.cu:90, where the label is not raised to p):
    1 - (2 sum(sigmoid(x) y) + smooth) / (sum(sigmoid(x)^p + y) + smooth)."""
    probs = torch.sigmoid(logits)
    numer = 2 * (probs * labels).sum() + smooth
    denor = (probs.pow(p) + labels).sum() + smooth
    return 1.0 - numer / denor


def layer_norm(x, eps=1e-6):
    """(N, C, M) normalised over C with autograd's own backward (pytorch_loss/layer_norm.py:32-38)."""
    mean = x.mean(dim=1, keepdim=True)
    std = (x.var(dim=1, keepdim=True, unbiased=False) + eps).rsqrt()
    return (x - mean) * std
