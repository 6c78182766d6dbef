"""Norms fused with the residual add that precedes them."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from ..kernels.limits import NORM_MAX_WIDTH, beyond
from ..weights.loader import Expect
from .base import BuildContext, NormedBranches, Part, Residual, RowVector, ScaledBranch, WeightedBranch, register_part


def partial_slab(pending) -> Optional[torch.Tensor]:
    """The float32 [S, T, d] tensor whose slabs, in order, ``pending`` lists (a branch that arrives as
    partial sums of a product split over K), or None."""
    if len(pending) < 2 or any(isinstance(branch, ScaledBranch) for branch in pending):
        return None
    base = pending[0]._base
    if (base is None or base.dim() != 3 or base.dtype != torch.float32 or base.shape[0] != len(pending)
            or not base.is_contiguous()):
        return None
    for index, slab in enumerate(pending):
        if slab._base is not base or slab.shape != base.shape[1:] or slab.data_ptr() != base[index].data_ptr():
            return None
    return base


def add_normed_branches(h: torch.Tensor, normed: NormedBranches, vector: Optional[torch.Tensor] = None) -> None:
    """h += layer norm of the weighted sum of ``normed``'s branches (+ ``vector`` on every row); nothing is normed
    behind it."""
    branches = list(normed.branches)
    extra = None
    while len(branches) > LAYERNORM_BRANCHES:               # more than the kernel sums: the first ones are added up first
        first, factor = branches.pop(0)
        if extra is None:
            extra = torch.zeros(h.shape, dtype=torch.float32, device=h.device)
        ops.stream_add(extra, first, factor, None)
    if extra is not None:
        second, factor = branches.pop(0)
        ops.stream_add(extra, second, factor, None)
        branches.insert(0, (extra, 1.0))
    ops.add_layernorm(h, branches, vector, None, None, 0.0, None, branch_norm=(normed.weight, normed.bias, normed.eps))


def fold_weighted(residual: Residual, keep_weighted: bool = False) -> None:
    """Add the ``WeightedBranch``es, ``NormedBranches`` and ``RowVector``s among the pending branches to the stream
    with the kernel that knows them, and leave the others pending: for a norm whose own kernel fuses none of them
    (``keep_weighted``: the weighted branches stay pending too, for a norm that adds them itself)."""
    kept = []
    for branch in residual.pending:
        if isinstance(branch, NormedBranches):
            add_normed_branches(residual.h, branch)
        elif isinstance(branch, WeightedBranch) and keep_weighted:
            kept.append(branch)
        elif isinstance(branch, WeightedBranch):
            ops.stream_add(residual.h, branch.rows, branch.factor, None)
        elif isinstance(branch, RowVector):
            ops.stream_add(residual.h, None, 1.0, branch.vector)
        else:
            kept.append(branch)
    if len(kept) != len(residual.pending):
        residual.pending = kept


def fold_pending(residual: Residual) -> None:
    """Add everything that is pending to the stream, with no norm behind it."""
    fold_weighted(residual)
    for branch in residual.pending:
        if isinstance(branch, ScaledBranch):
            raise NotImplementedError("a branch scaled by feature joins the stream in a norm's kernel")
        ops.stream_add(residual.h, branch, 1.0, None)
    residual.pending = []


@register_part("rmsnorm")
class RmsNorm(Part):
    """y = x / sqrt(mean(x^2) + eps) * (w + weight_offset), statistics in float32
    (reference: src/model_weights.rs:563-565, golden src/decoder.rs:10331-10334).  The offset (1 for a weight
    stored around zero) is added once, in float32, when the part is built."""
    graph_safe = True
    kernel_modules = ("common",)

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        return [Expect(f"{prefix}.weight", ((hidden_size,),), init="zero_centred" if spec.weight_offset else "norm")]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return beyond("rmsnorm", "hidden_size", hidden_size, NORM_MAX_WIDTH, "the norm stages a float32 row in 64 KiB of LDS")

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.eps = spec.eps
        self.build = build
        self.weight = (tensors[f"{prefix}.weight"].to(torch.float32) + float(spec.weight_offset)).contiguous().to(build.device)

    def _add(self, h: torch.Tensor, branch) -> None:
        if isinstance(branch, ScaledBranch):
            ops.add_scaled_rmsnorm(h, branch.rows, branch.scale, self.weight, self.eps, None)
        else:
            ops.add_rmsnorm(h, [branch], self.weight, self.eps, None)

    def rms_prologue(self):
        return self.weight, self.eps

    def forward(self, residual: Residual, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Add the pending branch outputs to the residual stream and return its normed rows
        (all of them, or only ``rows``; with ``rows`` the stream itself is left unchanged)."""
        if any(isinstance(branch, (RowVector, NormedBranches)) for branch in residual.pending):
            fold_weighted(residual, keep_weighted=True)
        if any(isinstance(branch, WeightedBranch) for branch in residual.pending):
            if any(isinstance(branch, ScaledBranch) for branch in residual.pending):
                fold_weighted(residual)
            else:
                return self._forward_weighted(residual, rows)
        pending = residual.pending
        slab = partial_slab(pending)
        if slab is not None and slab.shape[0] <= 16 and residual.h.shape[1] % 4 == 0:
            # partial sums of one branch: added and normed in one launch (with a gather: added here,
            # the gather below then norms the rows of the stream itself)
            out = None
            if rows is None:
                out = torch.empty(residual.h.shape, dtype=self.build.dtype, device=residual.h.device)
            ops.add_partials_rmsnorm(residual.h, slab, self.weight, self.eps, out)
            residual.pending = pending = []
            if rows is None:
                return out
        if any(isinstance(branch, ScaledBranch) for branch in pending):
            # branches with a scale of their own: each is added by the kernel that knows the scale, the last one
            # together with the norm
            for branch in pending[:-1]:
                self._add(residual.h, branch)
            last = pending[-1]
            if not isinstance(last, ScaledBranch):
                pending = [last]
            else:
                count = residual.h.shape[0] if rows is None else rows.numel()
                out = torch.empty((count, residual.h.shape[1]), dtype=self.build.dtype, device=residual.h.device)
                ops.add_scaled_rmsnorm(residual.h, last.rows, last.scale, self.weight, self.eps, out, rows)
                residual.pending = [] if rows is None else [last]
                return out
        while len(pending) > 2:                    # more than two branches: add the extra ones first
            ops.add_rmsnorm(residual.h, pending[:2], self.weight, self.eps, None)
            pending = pending[2:]
        count = residual.h.shape[0] if rows is None else rows.numel()
        out = torch.empty((count, residual.h.shape[1]), dtype=self.build.dtype, device=residual.h.device)
        ops.add_rmsnorm(residual.h, pending, self.weight, self.eps, out, rows)
        if rows is None:
            residual.pending = []
        return out


    def _forward_weighted(self, residual: Residual, rows: Optional[torch.Tensor]) -> torch.Tensor:
        """Branches that join the stream times a number each: the norm's kernel adds up to two of one dtype with
        their factors in its own launch (the products in float32); what is left over is added before."""
        pairs = [(branch.rows, float(branch.factor)) if isinstance(branch, WeightedBranch) else (branch, 1.0)
                 for branch in residual.pending]
        pairs = [(tensor if tensor.is_contiguous() else tensor.contiguous(), factor) for tensor, factor in pairs]
        while len(pairs) > 2 or (len(pairs) == 2 and pairs[0][0].dtype != pairs[1][0].dtype):
            tensor, factor = pairs.pop(0)
            ops.stream_add(residual.h, tensor, factor, None)
        count = residual.h.shape[0] if rows is None else rows.numel()
        out = torch.empty((count, residual.h.shape[1]), dtype=self.build.dtype, device=residual.h.device)
        ops.add_rmsnorm(residual.h, [tensor for tensor, _ in pairs], self.weight, self.eps, out, rows,
                        factors=[factor for _, factor in pairs])
        # with a gather the stream itself was not changed by the norm's kernel: its branches stay pending
        residual.pending = [] if rows is None else [WeightedBranch(tensor, factor) for tensor, factor in pairs]
        return out


LAYERNORM_BRANCHES = 3          # branches that the layer norm's kernel adds in its own launch


@register_part("layernorm")
class LayerNorm(Part):
    """y = (x - mean) / sqrt(variance + eps) * weight + bias over a row, mean and variance (the mean of the squared
    deviations, taken in a second pass over the row) in float32.  The kernel first adds what is pending to the
    stream: up to three branches, each times a number of its own, and one vector for every row."""
    graph_safe = True
    kernel_modules = ("common",)

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        return [Expect(f"{prefix}.weight", ((hidden_size,),), init="norm"),
                Expect(f"{prefix}.bias", ((hidden_size,),), init="bias")]

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return beyond("layernorm", "hidden_size", hidden_size, NORM_MAX_WIDTH, "the norm stages a float32 row in 64 KiB of LDS")

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.eps = spec.eps
        self.build = build
        self.weight = tensors[f"{prefix}.weight"].to(torch.float32).contiguous().to(build.device)
        self.bias = tensors[f"{prefix}.bias"].to(torch.float32).contiguous().to(build.device)

    def forward(self, residual: Residual, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Add the pending branches to the stream and return its normed rows (all, or only ``rows``; with ``rows``
        the stream itself is left unchanged and the branches stay pending)."""
        branches, vector, normed = [], None, None
        for branch in residual.pending:
            if isinstance(branch, NormedBranches):
                # the one the kernel takes through its own norm on the way into the stream; others before it
                if normed is not None or rows is not None or len(branch.branches) > LAYERNORM_BRANCHES:
                    add_normed_branches(residual.h, branch)
                else:
                    normed = branch
            elif isinstance(branch, RowVector):
                if vector is None:
                    vector = branch.vector
                else:                                      # a second vector: added by the plain kernel
                    ops.stream_add(residual.h, None, 1.0, branch.vector)
            elif isinstance(branch, ScaledBranch):         # a scale by feature: the kernel that knows it adds it
                ops.add_scaled_rmsnorm(residual.h, branch.rows, branch.scale, self.weight, self.eps, None)
            elif isinstance(branch, WeightedBranch):
                branches.append((branch.rows, float(branch.factor)))
            else:
                branches.append((branch, 1.0))
        if normed is not None and branches:
            # plain branches beside a normed group: the plain ones go first, the kernel's branch slots are the group's
            for tensor, factor in branches:
                ops.stream_add(residual.h, tensor, factor, None)
            branches = []
        while len(branches) > LAYERNORM_BRANCHES:
            first, factor = branches.pop(0)
            ops.stream_add(residual.h, first, factor, None)
        count = residual.h.shape[0] if rows is None else rows.numel()
        out = torch.empty((count, residual.h.shape[1]), dtype=self.build.dtype, device=residual.h.device)
        if normed is not None:
            ops.add_layernorm(residual.h, normed.branches, vector, self.weight, self.bias, self.eps, out,
                              branch_norm=(normed.weight, normed.bias, normed.eps))
            residual.pending = []
            return out
        ops.add_layernorm(residual.h, branches, vector, self.weight, self.bias, self.eps, out, rows)
        if rows is None:
            residual.pending = []
        else:
            # the stream was not changed: what this call could not fuse was added above, the rest stays pending
            kept = [WeightedBranch(tensor, factor) for tensor, factor in branches]
            residual.pending = kept + ([RowVector(vector)] if vector is not None else [])
        return out
