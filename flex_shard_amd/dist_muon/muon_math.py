"""Muon math on an owner's whole matrices, on HIP kernels.

The functions keep the names and argument meaning of the reference's
optimizer math (dist_muon/optimizer.py:2031-2151, cost model :1147-1155):
``_adjust_muon_learning_rate``, ``_prepare_muon_input``,
``_compute_muon_direction``, ``_apply_muon_update``,
``_zeropower_via_newtonschulz``.  ``OwnedMuon`` strings them together for the
comm-free case the reference runs on ``BucketedOwned`` storage
(dist_muon/_optimizer_reshard_runtime.py:645-661): every parameter is a whole
matrix on this rank, so a step is prepare -> Newton-Schulz -> apply with no
exchange.  Matrices of one shape are orthogonalized as one batch.
"""

from __future__ import annotations

import math
from collections.abc import Iterable, Sequence

import torch

from .. import hip_ops

DEFAULT_NS_COEFFICIENTS = (3.4445, -4.7750, 2.0315)


def _adjust_muon_learning_rate(lr: float, adjust_lr_fn: str | None, compute_matrix_shape: Sequence[int]) -> float:
    """Scale ``lr`` for the matrix aspect ratio."""
    rows, columns = compute_matrix_shape[-2:]
    if adjust_lr_fn is None or adjust_lr_fn == "original":
        ratio = math.sqrt(max(1.0, rows / columns))
    elif adjust_lr_fn == "match_rms_adamw":
        ratio = 0.2 * math.sqrt(max(rows, columns))
    elif adjust_lr_fn == "spectral_unclamped":
        ratio = math.sqrt(rows / columns)
    else:
        raise ValueError(f"unsupported adjust_lr_fn {adjust_lr_fn!r}")
    return lr * ratio


def _estimate_muon_compute_cost(matrix_shape: Sequence[int], ns_steps: int) -> int:
    """Multiply-accumulate count of Newton-Schulz: per step two s*s*l products
    and one s*s*s product (s the short side); FLOPs are twice this."""
    *batch, rows, columns = matrix_shape
    short, long = sorted((rows, columns))
    return math.prod(batch) * ns_steps * short * short * (2 * long + short)


def _require_bf16_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError("Muon kernels run on the GPU; this package has no CPU compute path.")
        if t.dtype != torch.bfloat16:
            raise NotImplementedError(f"the Newton-Schulz kernels operate on bf16 tensors, got {t.dtype}")
        if not t.is_contiguous():
            raise ValueError("the Muon kernels need contiguous tensors")


def _require_master_gpu(*tensors: torch.Tensor) -> None:
    """Parameters, gradients and momentum buffers: bf16 or fp32 (the
    reference's optimizer math is dtype-generic; its own tests run fp32)."""
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError("Muon kernels run on the GPU; this package has no CPU compute path.")
        if t.dtype not in (torch.bfloat16, torch.float32):
            raise NotImplementedError(f"the Muon kernels update bf16 or fp32 tensors, got {t.dtype}")
        if not t.is_contiguous():
            raise ValueError("the Muon kernels need contiguous tensors")


def _prepare_muon_input(
    gradient: torch.Tensor, momentum_buffer: torch.Tensor, *, momentum: float, nesterov: bool, out: torch.Tensor
) -> torch.Tensor:
    """``momentum_buffer.lerp_(gradient, 1 - momentum)`` and then either
    ``lerp(gradient, momentum_buffer, momentum)`` (Nesterov) or a copy of the
    buffer into ``out``; one fused launch.  Gradient and momentum buffer are
    both bf16 or both fp32; ``out`` is the bf16 tensor the orthogonalization
    reads (the reference casts its input to bf16 as its first step)."""
    _require_master_gpu(gradient, momentum_buffer)
    _require_bf16_gpu(out)
    if gradient.dtype != momentum_buffer.dtype:
        raise ValueError(f"gradient {gradient.dtype} and momentum buffer {momentum_buffer.dtype} differ in dtype")
    hip_ops.muon_prepare(momentum_buffer, gradient, out, momentum=momentum, nesterov=nesterov)
    return out


def _zeropower_via_newtonschulz(
    update: torch.Tensor,
    *,
    ns_coefficients: tuple[float, float, float] = DEFAULT_NS_COEFFICIENTS,
    ns_steps: int = 5,
    eps: float = 1e-7,
    workspace: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Approximate polar factor of each matrix of ``update`` ([..., rows, cols]):
    bf16 copy, Frobenius normalization, ``ns_steps`` quintic iterations with
    fp32-accumulated MFMA products rounded to bf16.  Returns a new bf16 tensor
    (or ``out``); ``update`` is left untouched unless it *is* ``out``."""
    if update.device.type != "cuda":
        raise RuntimeError("Newton-Schulz runs on the GPU; this package has no CPU compute path.")
    if update.ndim < 2:
        raise ValueError(f"expected a matrix or a batch of matrices, got shape {tuple(update.shape)}")
    if out is None:
        out = update.to(dtype=torch.bfloat16, copy=True).contiguous()
    elif out is not update:
        out.copy_(update)
    _require_bf16_gpu(out)
    hip_ops.newton_schulz(out.view(-1, *out.shape[-2:]), ns_coefficients, ns_steps, eps, workspace)
    return out


def _compute_muon_direction(
    prepared: torch.Tensor,
    *,
    lr_reference_shape: Sequence[int] | None = None,
    adjust_lr_fn: str | None = None,
    ns_coefficients: tuple[float, float, float] = DEFAULT_NS_COEFFICIENTS,
    ns_steps: int = 5,
    eps: float = 1e-7,
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """Orthogonalize ``prepared`` ([..., rows, cols], bf16) in place.  When the
    learning-rate shape factor of the matrices differs from the one of
    ``lr_reference_shape`` the direction is rescaled by their ratio (whole
    parameters use their own shape as reference, so the factor is 1)."""
    _zeropower_via_newtonschulz(
        prepared, ns_coefficients=ns_coefficients, ns_steps=ns_steps, eps=eps, workspace=workspace, out=prepared
    )
    if lr_reference_shape is not None:
        ratio = _adjust_muon_learning_rate(1.0, adjust_lr_fn, prepared.shape[-2:])
        reference = _adjust_muon_learning_rate(1.0, adjust_lr_fn, lr_reference_shape)
        if ratio != reference:
            prepared.mul_(ratio / reference)
    return prepared


def _apply_muon_update(
    parameter: torch.Tensor,
    direction: torch.Tensor,
    *,
    lr: float,
    weight_decay: float,
    adjust_lr_fn: str | None,
    compute_matrix_shape: Sequence[int],
) -> torch.Tensor:
    """``parameter *= 1 - lr*weight_decay; parameter += -adjusted_lr * direction``
    in one launch: with a bf16 rounding after each on a bf16 parameter, in
    fp32 on an fp32 one.  ``direction`` is the bf16 orthogonalized matrix."""
    _require_master_gpu(parameter)
    _require_bf16_gpu(direction)
    adjusted = _adjust_muon_learning_rate(lr, adjust_lr_fn, compute_matrix_shape)
    hip_ops.muon_apply(parameter, direction, decay_factor=1 - lr * weight_decay, neg_adjusted_lr=-adjusted)
    return parameter


class OwnedMuon:
    """Muon over whole bf16 or fp32 matrices owned by this rank (momentum
    buffers in the parameter's dtype, gradients too); a parameter with leading
    dimensions is a batch of matrices.

    Defaults follow the reference (dist_muon/optimizer.py:205-222): lr 1e-3,
    weight decay 0.1, momentum 0.95, Nesterov, 5 Newton-Schulz steps with the
    quintic coefficients, eps 1e-7.  ``step(grads)`` takes one gradient per
    parameter, in order; a missing gradient raises before anything is updated.
    """

    def __init__(
        self,
        params: Iterable[torch.Tensor],
        *,
        lr: float = 1e-3,
        weight_decay: float = 0.1,
        momentum: float = 0.95,
        nesterov: bool = True,
        ns_coefficients: tuple[float, float, float] = DEFAULT_NS_COEFFICIENTS,
        ns_steps: int = 5,
        eps: float = 1e-7,
        adjust_lr_fn: str | None = None,
    ) -> None:
        self.params = list(params)
        if not self.params:
            raise ValueError("OwnedMuon needs at least one parameter")
        for p in self.params:
            if p.ndim < 2:
                raise ValueError(f"Muon updates matrices; got a parameter of shape {tuple(p.shape)}")
        _require_master_gpu(*self.params)
        self.lr, self.weight_decay, self.momentum, self.nesterov = lr, weight_decay, momentum, nesterov
        self.ns_coefficients, self.ns_steps, self.eps, self.adjust_lr_fn = ns_coefficients, ns_steps, eps, adjust_lr_fn
        self.momentum_buffers = [torch.zeros_like(p) for p in self.params]
        # A parameter with leading dimensions ([experts, rows, cols]) is a
        # batch of independent matrices (the reference views it as one,
        # dist_muon/optimizer.py:2082-2091): the step works on 2-D views.
        self._matrix_counts = [math.prod(p.shape[:-2]) for p in self.params]
        self._stacked = any(p.ndim > 2 for p in self.params)
        self._matrices = self._as_matrices(self.params)
        self._momentum_matrices = self._as_matrices(self.momentum_buffers)
        # Matrices of one shape and dtype are orthogonalized as one batch; the step's
        # launch tables (address tables, batch buffers, workspaces) are built once.
        self._groups: dict[tuple[int, int, torch.dtype], list[int]] = {}  # (rows, cols, dtype) -> matrix indices
        # Matrices whose rows or columns are not multiples of 8 (the batched
        # step's 16-byte rows) take the per-matrix kernels, padded inside
        # the orthogonalization.
        self._odd: list[int] = []
        for index, m in enumerate(self._matrices):
            if m.shape[0] % 8 or m.shape[1] % 8:
                self._odd.append(index)
            else:
                self._groups.setdefault((*m.shape, m.dtype), []).append(index)
        self._plan = None
        if self._groups:
            self._plan = hip_ops.MuonStepPlan(
                [
                    # whole parameters are their own learning-rate reference shape: direction scale 1
                    (key[:2], len(members), -_adjust_muon_learning_rate(lr, adjust_lr_fn, key[:2]), 1.0, key[2])
                    for key, members in self._groups.items()
                ],
                self.params[0].device,
            )
            self._batch = dict(zip(self._groups, self._plan.batches))
            self._workspace = dict(zip(self._groups, self._plan.workspaces))

    @staticmethod
    def _as_matrices(tensors: Sequence[torch.Tensor]) -> list[torch.Tensor]:
        """The 2-D matrices of the tensors, in order, as views."""
        matrices = []
        for t in tensors:
            matrices.extend(t.view(-1, *t.shape[-2:]).unbind(0) if t.ndim > 2 else (t,))
        return matrices

    def flops_per_step(self) -> int:
        return 2 * sum(_estimate_muon_compute_cost(tuple(p.shape), self.ns_steps) for p in self.params)

    @torch.no_grad()
    def step(self, grads: Sequence[torch.Tensor | None]) -> None:
        if len(grads) != len(self.params):
            raise ValueError(f"expected {len(self.params)} gradients, got {len(grads)}")
        missing = [i for i, g in enumerate(grads) if g is None]
        if missing:
            raise RuntimeError(f"Muon parameters {missing} have no gradient; no parameter was updated")
        for p, g in zip(self.params, grads):
            if g.shape != p.shape or g.dtype != p.dtype:
                raise ValueError(
                    f"gradient {tuple(g.shape)} {g.dtype} does not match parameter {tuple(p.shape)} {p.dtype}"
                )
        _require_master_gpu(*grads)
        # One C call: per shape group a momentum launch over all its matrices
        # (which also leaves the sums of squares the normalization needs),
        # Newton-Schulz with every product issued for all groups together, and
        # an update launch per group.  Same bits as _prepare_muon_input ->
        # _compute_muon_direction -> _apply_muon_update per matrix.
        grad_matrices = self._as_matrices(grads)
        if self._stacked:
            # views of a stacked parameter are taken per step: they follow a
            # parameter whose storage was replaced (``p.data = ...``) since
            self._matrices = self._as_matrices(self.params)
        for index in self._odd:
            p, g = self._matrices[index], grad_matrices[index]
            direction = _prepare_muon_input(
                g, self._momentum_matrices[index], momentum=self.momentum, nesterov=self.nesterov,
                out=torch.empty(p.shape, dtype=torch.bfloat16, device=p.device),
            )
            _compute_muon_direction(direction, ns_coefficients=self.ns_coefficients, ns_steps=self.ns_steps, eps=self.eps)
            _apply_muon_update(
                p, direction, lr=self.lr, weight_decay=self.weight_decay, adjust_lr_fn=self.adjust_lr_fn,
                compute_matrix_shape=p.shape,
            )
        if self._plan is None:
            return
        members = list(self._groups.values())
        self._plan.step(
            [[self._matrices[i] for i in group] for group in members],
            [[self._momentum_matrices[i] for i in group] for group in members],
            [[grad_matrices[i] for i in group] for group in members],
            lerp_weight=1 - self.momentum, nesterov_weight=self.momentum, nesterov=self.nesterov,
            decay_factor=1 - self.lr * self.weight_decay, coefficients=self.ns_coefficients, steps=self.ns_steps,
            eps=self.eps,
            # lr and adjust_lr_fn are read on every step, like the weight decay
            # beside them: a scheduler that changes opt.lr moves both halves of
            # the update together.
            neg_adjusted_lrs=[-_adjust_muon_learning_rate(self.lr, self.adjust_lr_fn, key[:2]) for key in self._groups],
        )
