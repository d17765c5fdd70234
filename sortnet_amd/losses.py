"""Training losses on (logits, worst-case margins, targets), the reference's `--loss` choices (main.py:329-379).

`outputs` are the logits of the clean input, `worst_outputs` the worst-case margins of every class against the
target (0 in the target column) that the models return beside the logits (ell_inf_models.py:45-50).  Each loss is
a plain function; the classes below carry the reference's names, constructor arguments and the
`loss.update(ratio)` / `loss(outputs, worst_outputs, targets)` protocol of main.py:85-92, so a loss spec such as
`mixture(lam0=0.05,lam_end=0.0005)` maps onto them unchanged.
"""
import math

import torch
import torch.nn.functional as TF


def lam_schedule(lam0, lam_end, ratio):
    """Weight of the clean cross-entropy term: lam0 (lam_end / lam0)^ratio, ratio = training progress in [0, 1]
    (main.py:338-347); 0 stays 0."""
    return 0.0 if lam0 == 0 else lam0 * math.exp(math.log(lam_end / lam0) * ratio)


def hinge_loss(worst_outputs, mix=0.25):
    """main.py:329-335: largest positive margin per sample, mixed with the mean over all classes."""
    res = worst_outputs.clamp(min=0)
    return (1 - mix) * res.max(dim=1)[0].mean() + mix * res.mean()


def crossentropy_loss(outputs, worst_outputs, targets, lam):
    """main.py:353-355."""
    return TF.cross_entropy(worst_outputs, targets) + lam * TF.cross_entropy(outputs, targets)


def mixture_loss(outputs, worst_outputs, targets, lam, clip=1.0):
    """main.py:358-365: clipped hinge on the worst margin plus the decaying clean cross entropy."""
    res = worst_outputs.clamp(min=0, max=clip)
    return res.max(dim=1)[0].mean() + lam * TF.cross_entropy(outputs, targets)


def ce_hinge_loss(outputs, worst_outputs, targets, lam):
    """main.py:368-373: unit-margin hinge between the worst margins, counted only for samples the clean logits
    classify correctly."""
    correct = (outputs.argmax(dim=1) == targets).to(outputs.dtype)
    col = targets.view(-1, 1)
    margin = (worst_outputs - worst_outputs.gather(1, col) + 1).scatter(1, col, 0)
    return (correct * margin.max(dim=1)[0]).mean() + lam * TF.cross_entropy(outputs, targets)


def ce_mixture_loss(outputs, worst_outputs, targets, lam):
    """main.py:376-379: cross entropy of the worst margins on correctly classified samples."""
    correct = (outputs.argmax(dim=1) == targets).to(outputs.dtype)
    return (correct * TF.cross_entropy(worst_outputs, targets, reduction="none")).mean() + \
        lam * TF.cross_entropy(outputs, targets)


class hinge:
    def __init__(self, mix=0.25):
        self.mix = mix

    def update(self, ratio):
        pass

    def __call__(self, outputs, worst_outputs, targets):
        return hinge_loss(worst_outputs, self.mix)


class _Decaying:
    fn = None

    def __init__(self, lam0=1.0, lam_end=0.01, **extra):
        self.lam_start, self.lam_end, self.lam, self.extra = lam0, lam_end, lam0, extra

    def update(self, ratio):
        self.lam = lam_schedule(self.lam_start, self.lam_end, ratio)

    def __call__(self, outputs, worst_outputs, targets):
        return type(self).fn(outputs, worst_outputs, targets, self.lam, **self.extra)


class crossentropy(_Decaying):
    fn = staticmethod(crossentropy_loss)


class mixture(_Decaying):
    fn = staticmethod(mixture_loss)

    def __init__(self, lam0=1.0, lam_end=0.01, clip=1):
        super().__init__(lam0, lam_end, clip=clip)


class ce_hinge(_Decaying):
    fn = staticmethod(ce_hinge_loss)


class ce_mixture(_Decaying):
    fn = staticmethod(ce_mixture_loss)


LOSSES = {c.__name__: c for c in (hinge, crossentropy, mixture, ce_hinge, ce_mixture)}
