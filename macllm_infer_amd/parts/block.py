"""Arrangements of parts in a layer."""
from __future__ import annotations

from typing import Dict

import torch

from ..weights.loader import Expect
from .base import BuildContext, NormedBranches, Residual, ScaledBranch, WeightedBranch, part_class

_ARRANGEMENTS: Dict[str, type] = {}
_FUSIONS: Dict[str, object] = {}

OVERLAP_MIN_TOKENS = 256       # prompt portions from this size on run their two mixers on two streams
_side_streams: Dict[int, list] = {}


def side_stream(device: torch.device, beside: "torch.cuda.Stream") -> "torch.cuda.Stream":
    """A second stream of the device (default priority) that is not ``beside``.  Streams come from a pool of a
    few dozen that hands them out in turn, so the one drawn may be the very stream a graph is being captured on:
    work recorded "beside" it would queue behind (a 2,048-token prompt of the 0.5B shape: 7.2 ms instead of 6.3)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    streams = _side_streams.setdefault(index, [])
    for stream in streams:
        if stream != beside:
            return stream
    while True:
        streams.append(torch.cuda.Stream(device=device))
        if streams[-1] != beside:
            return streams[-1]


def overlap_pays(mixers, rows: int, device: torch.device) -> bool:
    """Whether two mixers of a layer that read the same rows should run beside each other on two streams: in a
    captured graph only (launched one by one the step waits for the host, which the second stream costs more),
    for portions long enough to be worth the hops between the queues, and if both only queue work."""
    return (len(mixers) == 2 and rows >= OVERLAP_MIN_TOKENS and device.type == "cuda"
            and torch.cuda.is_current_stream_capturing()
            and all(getattr(mixer, "graph_safe", False) for mixer in mixers))


def register_fusion(arrangement: str):
    """Register ``factory(block, build) -> fusion or None`` for layers of ``arrangement``: a fusion runs the
    whole layer through fewer launches where its parts and sizes allow
    (``forward(residual, step, caches) -> bool``: True when it ran the layer)."""
    def decorate(factory):
        _FUSIONS[arrangement] = factory
        return factory
    return decorate


def register_arrangement(name: str):
    def decorate(cls):
        _ARRANGEMENTS[name] = cls
        return cls
    return decorate


def arrangement_class(name: str) -> type:
    if name not in _ARRANGEMENTS:
        raise KeyError(f"no arrangement named {name!r}; registered: {sorted(_ARRANGEMENTS)}")
    return _ARRANGEMENTS[name]


@register_arrangement("parallel_prenorm")
class ParallelPreNormBlock:
    """n = norm(h); h += sum over mixers of mixer(n); h += ffn(norm(h)).
    All mixers read the same normed input and their outputs are summed into the residual
    (reference: src/decoder.rs:2658-2682, 2684-2699).  With one mixer this is the ordinary
    sequential pre-norm layer.  A layer may scale either branch feature by feature before the add
    (``mixer_scale_name`` / ``ffn_scale_name``: h += scale * branch, the product in float32) or multiply both by
    one number (``branch_multiplier``), and may have no feed-forward at all (``ffn`` None).  A mixer may have an RMS
    norm of its own on its output (``MixerSlot.post_norm``): the normed outputs are summed with the mixers' weights
    in one launch, in float32, and that sum is the branch."""

    @classmethod
    def expected_tensors(cls, layer, hidden_size: int):
        out = []
        out += part_class(layer.mixer_norm).expected_tensors(
            layer.mixer_norm, f"{layer.prefix}.{layer.mixer_norm_name}", hidden_size)
        for slot in layer.mixers:
            out += part_class(slot.spec).expected_tensors(slot.spec, f"{layer.prefix}.{slot.name}", hidden_size)
            if getattr(slot, "post_norm", None) is not None:
                out += part_class(slot.post_norm).expected_tensors(
                    slot.post_norm, f"{layer.prefix}.{slot.name}.{slot.post_norm_name}", hidden_size)
        if layer.mixer_scale_name:
            out.append(Expect(f"{layer.prefix}.{layer.mixer_scale_name}", ((hidden_size,),), init="scale"))
        second = part_class(layer.ffn_norm).expected_tensors(
            layer.ffn_norm, f"{layer.prefix}.{layer.ffn_norm_name}", hidden_size)
        if layer.ffn_scale_name:
            second.append(Expect(f"{layer.prefix}.{layer.ffn_scale_name}", ((hidden_size,),), init="scale"))
        if layer.ffn is None:
            # a layer without a feed-forward uses neither; a checkpoint that holds them all the same is accepted
            return out + [Expect(one.name, one.shapes, one.init, one.integer, optional=True) for one in second]
        out += second
        out += part_class(layer.ffn).expected_tensors(layer.ffn, f"{layer.prefix}.{layer.ffn_name}", hidden_size)
        return out

    @staticmethod
    def _part_specs(layer):
        second = [] if layer.ffn is None else [layer.ffn_norm, layer.ffn]
        return [layer.mixer_norm] + second + [slot.spec for slot in layer.mixers]

    @classmethod
    def limits(cls, layer, hidden_size: int):
        """What the kernels of this layer's parts refuse (see ``Part.limits``)."""
        out = []
        for spec in cls._part_specs(layer):
            out += part_class(spec).limits(spec, hidden_size)
        return out

    @classmethod
    def kernel_modules(cls, layer):
        modules = []
        for spec in cls._part_specs(layer):
            modules += list(part_class(spec).kernel_modules)
        return modules

    def __init__(self, layer, tensors, build: BuildContext):
        self.layer = layer
        self.mixer_norm = part_class(layer.mixer_norm)(
            layer.mixer_norm, f"{layer.prefix}.{layer.mixer_norm_name}", tensors, build)
        self.mixers = [(slot.name, part_class(slot.spec)(slot.spec, f"{layer.prefix}.{slot.name}", tensors, build))
                       for slot in layer.mixers]
        self.ffn_norm = self.ffn = None
        if layer.ffn is not None:
            self.ffn_norm = part_class(layer.ffn_norm)(
                layer.ffn_norm, f"{layer.prefix}.{layer.ffn_norm_name}", tensors, build)
            self.ffn = part_class(layer.ffn)(layer.ffn, f"{layer.prefix}.{layer.ffn_name}", tensors, build)

        def scale(name):
            if not name:
                return None
            return tensors[f"{layer.prefix}.{name}"].to(torch.float32).contiguous().to(build.device)
        self.mixer_scale = scale(layer.mixer_scale_name)
        self.ffn_scale = scale(layer.ffn_scale_name) if layer.ffn is not None else None
        factory = _FUSIONS.get(layer.arrangement)
        # the fast path knows plain branches and a feed-forward behind them; None when parts or sizes do not fit
        self.branch_multiplier = float(getattr(layer, "branch_multiplier", 1.0))
        self.mixer_weights = [float(getattr(slot, "weight", 1.0)) for slot in layer.mixers]
        # (weight, eps) of the RMS norm on a mixer's output, or None
        self.mixer_posts = []
        for slot in layer.mixers:
            post = getattr(slot, "post_norm", None)
            if post is None:
                self.mixer_posts.append(None)
                continue
            if post.kind != "rmsnorm":
                raise ValueError(f"layer {layer.prefix}: the norm on a mixer's output is an RMS norm")
            norm = part_class(post)(post, f"{layer.prefix}.{slot.name}.{slot.post_norm_name}", tensors, build)
            self.mixer_posts.append((norm.weight, float(post.eps)))
        plain = (self.mixer_scale is None and all(post is None for post in self.mixer_posts) and self.ffn_scale is None and self.ffn is not None
                 and self.branch_multiplier == 1.0 and all(weight == 1.0 for weight in self.mixer_weights))
        self.fusion = factory(self, build) if factory is not None and plain else None

    @property
    def graph_safe(self) -> bool:
        parts = [self.mixer_norm] + [mixer for _, mixer in self.mixers]
        parts += [self.ffn_norm, self.ffn] if self.ffn is not None else []
        return all(getattr(part, "graph_safe", False) for part in parts)

    def tune(self, peers) -> None:
        """Called once every layer of the model is built, with all of them: what a layer can only decide by
        timing itself among the others."""
        tune = getattr(self.fusion, "tune_chain", None)
        if tune is not None:
            tune([getattr(peer, "fusion", None) for peer in peers])

    @property
    def first_norm(self):
        """The norm this arrangement starts with: what a layer before it may prepare the stream for."""
        return self.mixer_norm

    def forward(self, residual: Residual, step, caches) -> None:
        """``caches``: mixer name -> EntryCache of this run of the layer."""
        fusion = self.fusion
        if fusion is not None and fusion.forward(residual, step, caches):
            return
        normed = self.mixer_norm.forward(residual)
        outputs = self.run_mixers(normed, step, caches)
        if any(post is not None for post in self.mixer_posts):
            outputs = self.normed_outputs(outputs)
        elif self.mixer_scale is not None:
            outputs = [ScaledBranch(rows, self.mixer_scale) for rows in outputs]
        elif self.branch_multiplier != 1.0 or any(weight != 1.0 for weight in self.mixer_weights):
            outputs = [WeightedBranch(rows, self.branch_multiplier * weight)
                       for rows, weight in zip(outputs, self.mixer_weights)]
        residual.pending = outputs
        if self.ffn is None:
            return
        normed = self.ffn_norm.forward(residual)
        rows = self.ffn.forward(normed)
        if self.ffn_scale is not None:
            residual.pending = [ScaledBranch(rows, self.ffn_scale)]
        elif self.branch_multiplier != 1.0:
            residual.pending = [WeightedBranch(rows, self.branch_multiplier)]
        else:
            residual.pending = [rows]

    def normed_outputs(self, outputs: list) -> list:
        """The mixers' outputs behind their own RMS norms: the normed ones summed with their weights in one launch
        (float32), the others as weighted branches beside that sum."""
        from ..kernels import ops
        if self.mixer_scale is not None:
            raise NotImplementedError("a scale by feature beside norms on the mixers' outputs")
        normed = [(rows, weight, *post) for rows, weight, post in zip(outputs, self.mixer_weights, self.mixer_posts)
                  if post is not None]
        total = torch.empty(outputs[0].shape, dtype=torch.float32, device=outputs[0].device)
        if len(normed) > ops.NORMED_SUM_MOST:
            raise NotImplementedError(f"more than {ops.NORMED_SUM_MOST} mixers with norms on their outputs")
        ops.normed_sum(normed, total)
        branches = [WeightedBranch(total, self.branch_multiplier)]
        branches += [WeightedBranch(rows, self.branch_multiplier * weight)
                     for rows, weight, post in zip(outputs, self.mixer_weights, self.mixer_posts) if post is None]
        return branches

    def run_mixers(self, normed: torch.Tensor, step, caches) -> list:
        """Every mixer's output for the normed rows, in the mixers' order."""
        if overlap_pays([mixer for _, mixer in self.mixers], normed.shape[0], normed.device):
            # the second mixer is recorded first and stays on the queue of the kernels around it (see the fast
            # path's ``forward_general``); what either allocates is its own stream's until the join
            (first_name, first), (second_name, second) = self.mixers
            main = torch.cuda.current_stream(normed.device)
            side = side_stream(normed.device, main)
            side.wait_stream(main)
            second_out = second.forward(normed, step, caches[second_name])
            with torch.cuda.stream(side):
                first_out = first.forward(normed, step, caches[first_name])
            main.wait_stream(side)
            return [first_out, second_out]
        return [mixer.forward(normed, step, caches[name]) for name, mixer in self.mixers]


@register_arrangement("sandwich")
class SandwichBlock(ParallelPreNormBlock):
    """A norm before and a norm after each branch: h += post1(sum over mixers of weight_m * mixer_m(norm1(h)));
    h += post2(ffn(norm2(h))).  The weighted sum of a branch and its post-norm wait in ``Residual.pending`` as one
    ``NormedBranches`` entry, so the norm that follows (this layer's second, or the next layer's first) takes the
    branch through its post-norm, adds it to the stream and normalizes the stream in one launch."""

    @classmethod
    def expected_tensors(cls, layer, hidden_size: int):
        out = super().expected_tensors(layer, hidden_size)
        post = part_class(layer.mixer_post_norm).expected_tensors(
            layer.mixer_post_norm, f"{layer.prefix}.{layer.mixer_post_norm_name}", hidden_size)
        second = part_class(layer.ffn_post_norm).expected_tensors(
            layer.ffn_post_norm, f"{layer.prefix}.{layer.ffn_post_norm_name}", hidden_size)
        if layer.ffn is None:
            second = [Expect(one.name, one.shapes, one.init, one.integer, optional=True) for one in second]
        return out + post + second

    @staticmethod
    def _part_specs(layer):
        return ParallelPreNormBlock._part_specs(layer) + [layer.mixer_post_norm]

    def __init__(self, layer, tensors, build: BuildContext):
        super().__init__(layer, tensors, build)
        self.fusion = None
        if layer.mixer_post_norm.kind != "layernorm" or (layer.ffn is not None and layer.ffn_post_norm.kind != "layernorm"):
            raise ValueError(f"layer {layer.prefix}: the norms behind the branches of a sandwich layer are layer norms")

        def post(spec, name):
            norm = part_class(spec)(spec, f"{layer.prefix}.{name}", tensors, build)
            return norm.weight, norm.bias, float(spec.eps)
        self.mixer_post = post(layer.mixer_post_norm, layer.mixer_post_norm_name)
        self.ffn_post = post(layer.ffn_post_norm, layer.ffn_post_norm_name) if layer.ffn is not None else None

    def forward(self, residual: Residual, step, caches) -> None:
        normed = self.mixer_norm.forward(residual)
        outputs = self.run_mixers(normed, step, caches)
        branches = [(rows, self.branch_multiplier * weight) for rows, weight in zip(outputs, self.mixer_weights)]
        residual.pending = [NormedBranches(branches, *self.mixer_post)]
        if self.ffn is None:
            return
        normed = self.ffn_norm.forward(residual)
        residual.pending = [NormedBranches([(self.ffn.forward(normed), self.branch_multiplier)], *self.ffn_post)]
