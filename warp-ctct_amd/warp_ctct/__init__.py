"""CTC-Transducer loss for AMD MI355X (gfx950) with the warp_ctct API.

Drop-in for ``warp_ctct`` of maxwellzh/warp-ctct: the public functions
``ctct_loss`` and ``ctct_simple_loss`` keep the reference's signatures,
assertions, reduction / average_frames semantics and autograd contract
(warp_ctct/__init__.py:88-147 and :150-236 of the reference); blank = 0.

All device work is done by hand-written HIP kernels in libwarpctct_hip.so,
reached through the torch binding ``warp_ctct._C``.  There is no CPU or eager
fallback: importing this package without the built extension raises.
"""
from typing import Optional

import torch

try:
    from . import _C as core
except ImportError as exc:  # pragma: no cover - exercised only on a broken install
    raise ImportError(
        "warp_ctct._C (the HIP extension) is not built; run "
        "`python setup.py build_ext --inplace` in warp-ctct_amd/ "
        "(needs hipcc, --offload-arch=gfx950)"
    ) from exc

# The reference exports exactly these two (warp_ctct/__init__.py:17), so that
# `from warp_ctct import *` binds the same names.  ctct_loss_with_logits,
# ctct_loss_compact and label_range_violated are additions of this build and are
# reached by name (warp_ctct.ctct_loss_with_logits, ...).
__all__ = ["ctct_loss", "ctct_simple_loss"]


def _package_version():
    """Version of the installed distribution (the reference reads it the same
    way, warp_ctct/__init__.py:14), which is the reference distribution's 0.3.0;
    the same string from _version.py when the package is used from a source tree
    without distribution metadata.  The kernel library has an ABI version of its
    own: warp_ctct._C.library_version()."""
    try:
        from importlib.metadata import version
        return version("warp_ctct")
    except Exception:
        from ._version import __version__ as source_version
        return source_version


__version__ = _package_version()


# ctct_loss allocates and clears the joint's gradient during the forward (in the
# lattice kernel's launch, beside the sweeps) when the joint requires a gradient.  The
# buffer then lives from the forward to the backward; set this to False to
# allocate and clear it in the backward instead.
CLEAR_GRADIENT_IN_FORWARD = True

# The kernels clamp labels into [0, V) before they use them as column indices,
# so that a corrupt label cannot make the GPU fault; the reference's
# torch.gather raises on such an index (warp_ctct/__init__.py:131).  A clamped
# label is recorded on the device and shows up in label_range_violated() /
# status() without any synchronisation in the loss itself.  Set this to True to
# get the reference's behaviour back while debugging a data pipeline: every call
# then checks its labels on the host (one device-to-host synchronisation).
CHECK_LABEL_RANGE = False


STATUS_LABEL_RANGE, STATUS_NAN_INPUT, STATUS_LOST_HAND_OVER, STATUS_LINEAR_FELL_BACK = 1, 2, 4, 8


def status(reset: bool = True, device=None) -> int:
    """Sticky status bits of a GPU (the current one by default), set by the
    kernels of every call since the last reset:

    * ``STATUS_LABEL_RANGE``: a label outside [0, V) was met and clamped (the
      reference raises for it, warp_ctct/__init__.py:131);
    * ``STATUS_NAN_INPUT``: a gathered log-probability was NaN (the lattice
      treats such a unit as log 0);
    * ``STATUS_LOST_HAND_OVER``: a lattice was not swept to its end (its costs
      and gradients are NaN by construction, not because of the inputs);
    * ``STATUS_LINEAR_FELL_BACK``: ``ctct_simple_loss`` swept a batch in the
      linear domain, its check refused the result, and the log-domain kernels
      computed the batch again (the results are right; see
      ``joiner_linear_lattice``).

    Nothing in ``ctct_loss`` / ``ctct_simple_loss`` synchronises with the host;
    this call does (it waits for the device), so use it where a pipeline would
    check anyway: once per epoch, or when a loss looks wrong."""
    if device is None:
        return int(core.status(bool(reset)))
    with torch.cuda.device(device):
        return int(core.status(bool(reset)))


def joiner_linear_lattice(from_frames: int = -1) -> int:
    """From how many frames on ``ctct_simple_loss`` sweeps its lattices on path
    masses instead of their logarithms (half the time per frame; the result is
    checked on the GPU, and the log-domain kernels, queued behind, compute a
    batch again whose check fails: ``STATUS_LINEAR_FELL_BACK``).  0: never,
    1: always, negative: the defaults (768 frames, 384 with normalisation, and
    only batches of up to 768 wavefronts of sweeps, 2 N ceil((U+1)/62), or 256
    where a lattice needs one per direction: larger batches are bound by the
    memory system, where the linear form has nothing to gain).  A limit set here
    holds for batches of any size.  One setting for the process; returns the
    previous one (negative: the defaults).  The reference sweeps in the log domain only (csrc/simple.cu)."""
    return int(core.joiner_linear_lattice(int(from_frames)))


def label_range_violated(reset: bool = True, device=None) -> bool:
    """True if any call since the last reset met a label outside [0, V)."""
    bits = status(reset=False, device=device)
    if reset and bits & STATUS_LABEL_RANGE:
        status(reset=True, device=device)
    return bool(bits & STATUS_LABEL_RANGE)


def _check_labels(labels, vocabulary):
    if CHECK_LABEL_RANGE and labels.numel() > 0:
        lo, hi = int(labels.min()), int(labels.max())
        if lo < 0 or hi >= vocabulary:
            raise IndexError("labels must lie in [0, %d): found values from %d to %d"
                             % (vocabulary, lo, hi))


def _no_autocast():
    return torch.autocast(device_type="cuda", enabled=False)


def _as_int(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.int).contiguous()


def _reduce(costs, frames_lengths, reduction, average_frames):
    # warp_ctct/__init__.py:138-147 of the reference
    if average_frames:
        costs = costs / frames_lengths
    if reduction == "none" or reduction is None:
        return costs
    if reduction == "sum":
        return costs.sum()
    if reduction == "mean":
        return costs.mean()
    return costs


_REDUCTION_CODE = {None: 0, "none": 0, "sum": 1, "mean": 2}
_NATIVE_DTYPES = (torch.float32, torch.float16, torch.bfloat16)


# The fused losses are autograd functions of the binding (csrc/binding.cpp:
# JointLoss, LogitsLoss, JoinerLoss): one crossing into C++ per call, and the
# backward runs without Python.
#
# JointLoss (ctct_loss on the un-gathered joint, reduction included) is the
# counterpart of the reference's gather (warp_ctct/__init__.py:124-131), the cast
# to float (:135), CTCTLoss (:20-33) and the reduction (:138-147).  Its forward
# runs gather, both lattices and the batch reduction on the GPU and keeps their
# workspace.  The dense gradient is all zeros but <= 3 entries per live row, so
# its buffer is allocated in the forward and cleared, at HBM write bandwidth,
# inside the launch of the lattice kernel (whose sweeps are bound by latency and
# leave the memory system idle); the backward then only writes the non-zero
# entries, already weighted by the upstream gradient and by the reduction's own
# factor (1/N, 1/lx[n]), so autograd launches nothing else.  A float16 or
# bfloat16 joint is read as it is and its gradient is written in the same type
# (the lattice itself always runs in float32 / float64).  The cleared buffer
# serves one backward: a second backward through the same graph
# (retain_graph=True) clears and fills a buffer of its own.
#
# LogitsLoss is ctct_loss(logits.log_softmax(-1), ...) without the
# log-probability tensor: the forward takes the row-wise logsumexp inside the
# gather and keeps it next to the lattices; the backward writes d(loss)/d(logits)
# = w * (G - softmax * sum(G)) in one pass, G being the <= 3 non-zero
# gather-backward entries of the row.  Rows of padding are never read.
#
# JoinerLoss (ctct_simple_loss on the un-gathered f (N,T,V) and g (N,U+1,V)) is
# the counterpart of the reference's LogMMExp (warp_ctct/__init__.py:36-52), the
# two gathers (:204-215) and SimpleCTCTLoss (:55-85): the forward computes den
# (if normalized), the lattice and the compact gradients wrt the gathered f, g
# and den; the backward expands them to dense gradients wrt f and g, including
# the path through den, scaled by grad_output[n].


class CTCTLoss(torch.autograd.Function):
    """The reference's autograd function on GATHERED log-probabilities
    (warp_ctct/__init__.py:20-33): ``log_probs`` is (N, T, U, 3) =
    joint[..., [0, y[u-1], y[u]]].  Kept for code that imports it by name;
    :func:`ctct_loss` does not go through it (it works on the joint itself)."""

    @staticmethod
    def forward(ctx, log_probs, labels, lx, ly, requires_grad):
        costs, grads = core.ctct_loss_fwd(log_probs, labels, lx, ly, requires_grad)
        if requires_grad:
            ctx.save_for_backward(grads)
        return costs

    @staticmethod
    def backward(ctx, grad_outputs):
        (grads,) = ctx.saved_tensors
        return grad_outputs.reshape(-1, 1, 1, 1) * grads, None, None, None, None


class LogMMExp(torch.autograd.Function):
    """Differentiable log-semiring matrix product (warp_ctct/__init__.py:36-52
    of the reference): ``out[b, i, j] = logsumexp_k(lhs[b, i, k] + rhs[b, k, j])``
    for float32 operands (B, M, K) and (B, K, N); strided operands are fine."""

    @staticmethod
    def forward(ctx, lhs, rhs, track_l=True, track_r=True):
        out = core.log_matmul(lhs, rhs)
        if track_l or track_r:
            ctx.save_for_backward(lhs, rhs, out)
            ctx.track = [bool(track_l), bool(track_r)]
        return out

    @staticmethod
    def backward(ctx, grad_outputs):
        lhs, rhs, out = ctx.saved_tensors
        grad_lhs, grad_rhs = core.log_matmul_backward(grad_outputs.contiguous(), lhs, rhs, out,
                                                      ctx.track)
        return grad_lhs, grad_rhs, None, None


class SimpleCTCTLoss(torch.autograd.Function):
    """The reference's autograd function of the log-add joiner on GATHERED
    operands (warp_ctct/__init__.py:55-85): ``f`` (N, T, U), ``g`` (N, U, 3),
    ``den`` (N, T, U) or None for the unnormalised variant.  Kept for code that
    imports it by name; :func:`ctct_simple_loss` works on the un-gathered
    operands instead."""

    @staticmethod
    def forward(ctx, f, g, den, labels, lx, ly, rg_f, rg_g):
        normalized = den is not None and den.dim() == 3
        stand_in = den if normalized else f.new_empty(1)
        need = bool(rg_f or rg_g)
        costs, grad_f, grad_g, grad_den = core.ctct_loss_simple_fwd(f, g, labels, stand_in, lx, ly,
                                                                    need)
        ctx.which = (bool(rg_f), bool(rg_g), normalized and need)
        ctx.save_for_backward(*[t for t, keep in zip((grad_f, grad_g, grad_den), ctx.which)
                                if keep])
        return costs

    @staticmethod
    def backward(ctx, grad_outputs):
        saved = list(ctx.saved_tensors)
        w = grad_outputs.reshape(-1, 1, 1)
        grads = [saved.pop(0) * w if keep else None for keep in ctx.which]
        return grads[0], grads[1], grads[2], None, None, None, None, None


def ctct_loss(log_probs: torch.Tensor,
              labels: torch.Tensor,
              frames_lengths: torch.Tensor,
              labels_lengths: torch.Tensor,
              reduction: Optional[str] = "mean",
              average_frames: bool = False) -> torch.Tensor:
    """The CTC-Transducer loss.

    Args:
        log_probs: (N, T, U, V) joint log-probabilities, where N is the batch
            size, T the maximum number of frames, U the maximum number of
            labels + 1 and V the vocabulary size including the blank (index 0).
        labels: (N, U-1) reference labels.
        frames_lengths: (N,) number of frames of each sample.
        labels_lengths: (N,) number of labels of each sample.
        reduction: 'none' | 'mean' | 'sum' (None behaves like 'none').
        average_frames: divide each sample's loss by its number of frames.

    Memory: when ``log_probs`` requires a gradient, the forward allocates the
    gradient's buffer (the shape and type of ``log_probs``: 2 GB for a
    (32, 250, 61, 1024) float32 joint) and clears it beside the lattice sweeps;
    the buffer lives until the backward has run or the graph is freed.  Code
    that evaluates several losses before one backward holds one such buffer per
    loss; ``warp_ctct.CLEAR_GRADIENT_IN_FORWARD = False`` allocates and clears
    it in the backward instead, as the reference's autograd does (one more
    launch per step).
    """
    assert average_frames is None or isinstance(average_frames, bool)
    assert reduction is None or reduction in ("none", "mean", "sum")
    assert log_probs.dim() == 4
    assert labels.dim() == 2
    assert log_probs.size(2) == labels.size(1) + 1
    assert log_probs.size(0) == labels.size(0) == frames_lengths.size(0) == labels_lengths.size(0)

    if log_probs.size(0) == 0:
        # nothing to launch; costs of an empty batch, still attached to the graph
        return _reduce(log_probs.float().sum(dim=(1, 2, 3)), frames_lengths, reduction,
                       average_frames)
    _check_labels(labels, log_probs.size(3))
    if log_probs.dtype not in _NATIVE_DTYPES:
        log_probs = log_probs.float()      # as the reference does for every dtype (:135)
    # (the reference computes under autocast(enabled=False), :134; nothing in
    # here is subject to autocast.)  A strided view is gathered through its
    # strides, not copied.
    return core.ctct_loss(log_probs, labels, frames_lengths, labels_lengths,
                          _REDUCTION_CODE[reduction], bool(average_frames),
                          bool(CLEAR_GRADIENT_IN_FORWARD))


def ctct_loss_compact(log_probs: torch.Tensor,
                      labels: torch.Tensor,
                      frames_lengths: torch.Tensor,
                      labels_lengths: torch.Tensor):
    """Per-sample costs and their gradient in compact form, without autograd.

    For callers that own the joiner and want to apply the gradient themselves
    instead of receiving a dense (N, T, U, V) tensor that is zero almost
    everywhere.  Returns ``(costs, unit_grads, index)``:
    ``costs`` (N,) float32; ``unit_grads`` (N, T, U, 3) float32 with
    ``unit_grads[n, t, u, k] = d costs[n] / d log_probs[n, t, u, index[n, u, k]]``
    (zero outside ``t < frames_lengths[n]``, ``u <= labels_lengths[n]``);
    ``index`` (N, U, 3) int64 = ``[0, labels[u-1], labels[u]]`` with 0 where no
    label exists, the gather index of the reference
    (warp_ctct/__init__.py:124-131).  ``dense.scatter_add_(3, index[:, None]
    .expand_as(unit_grads), unit_grads)`` rebuilds the dense gradient."""
    assert log_probs.dim() == 4
    assert labels.dim() == 2
    assert log_probs.size(2) == labels.size(1) + 1
    assert log_probs.size(0) == labels.size(0) == frames_lengths.size(0) == labels_lengths.size(0)
    if log_probs.dtype not in _NATIVE_DTYPES:
        log_probs = log_probs.float()
    labels_i = _as_int(labels)
    with torch.no_grad(), _no_autocast():
        costs, unit_grads = core.ctct_loss_compact_fwd(
            log_probs.detach().contiguous(), labels_i, _as_int(frames_lengths),
            _as_int(labels_lengths))
        n, u = labels_i.shape
        index = torch.zeros(n, u + 1, 3, dtype=torch.long, device=labels_i.device)
        index[:, 1:, 1] = labels_i
        index[:, :-1, 2] = labels_i
    return costs, unit_grads, index


def ctct_loss_with_logits(logits: torch.Tensor,
                          labels: torch.Tensor,
                          frames_lengths: torch.Tensor,
                          labels_lengths: torch.Tensor,
                          reduction: Optional[str] = "mean",
                          average_frames: bool = False) -> torch.Tensor:
    """``ctct_loss(logits.log_softmax(-1), ...)`` in one pass over the logits.

    The reference expects normalised log-probabilities, so its callers run
    ``log_softmax`` over the (N, T, U, V) joiner output first and autograd
    pushes the dense gradient back through it.  This function takes the
    joiner output itself: the normalisation happens inside the gather, its
    backward inside the kernel that writes the gradient, and the
    log-probability tensor is never materialised.  Arguments and result are
    those of :func:`ctct_loss`; ``logits`` may be float32, float16 or
    bfloat16 (other types are converted to float32)."""
    assert average_frames is None or isinstance(average_frames, bool)
    assert reduction is None or reduction in ("none", "mean", "sum")
    assert logits.dim() == 4
    assert labels.dim() == 2
    assert logits.size(2) == labels.size(1) + 1
    assert logits.size(0) == labels.size(0) == frames_lengths.size(0) == labels_lengths.size(0)

    if logits.size(0) == 0:
        return _reduce(logits.float().sum(dim=(1, 2, 3)), frames_lengths, reduction,
                       average_frames)
    _check_labels(labels, logits.size(3))
    if logits.dtype not in _NATIVE_DTYPES:
        logits = logits.float()
    return core.ctct_loss_with_logits(logits, labels, frames_lengths, labels_lengths,
                                      _REDUCTION_CODE[reduction], bool(average_frames))


def ctct_simple_loss(f: torch.Tensor,
                     g: torch.Tensor,
                     labels: torch.Tensor,
                     frames_lengths: torch.Tensor,
                     labels_lengths: torch.Tensor,
                     reduction: Optional[str] = "mean",
                     average_frames: bool = False,
                     normalized: bool = True) -> torch.Tensor:
    """The CTC-Transducer loss with the log-add joiner  joint = f (+) g.

    Args:
        f: (N, T, V) encoder scores.
        g: (N, U, V) predictor scores, U = maximum number of labels + 1.
        labels, frames_lengths, labels_lengths, reduction, average_frames: as
            in :func:`ctct_loss`.
        normalized: subtract logsumexp_v(f + g) per (t, u) (a proper
            distribution); False scores paths with the raw sums.
    """
    assert average_frames is None or isinstance(average_frames, bool)
    assert reduction is None or reduction in ("none", "mean", "sum")
    assert f.dim() == 3 and g.dim() == 3
    assert labels.dim() == 2
    assert g.size(1) == labels.size(1) + 1
    assert f.size(0) == g.size(0) == labels.size(0) == frames_lengths.size(0) == labels_lengths.size(0)

    _check_labels(labels, f.size(-1))
    return core.ctct_simple_loss(f, g, labels, frames_lengths, labels_lengths, bool(normalized),
                                 _REDUCTION_CODE[reduction], bool(average_frames))
