"""Feed-forwards that route every token to a few of many small experts."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..kernels.limits import MOE_MAX_EXPERTS, beyond
from ..weights.loader import Expect
from .base import BuildContext, FeedForward, register_part
from .linear import Linear


@register_part("routed_experts")
class RoutedExperts(FeedForward):
    """sum over a token's ``top_k`` experts of weight * expert(x), plus sigmoid(w_sg . x) * shared(x).

    An expert is down(act(gate(x), up(x))) with the clamped gated activation of ``ClampedGLUSpec`` and no biases, or
    (an activation that is not ``gated``) down(max(up(x), 0)^2) with no gate matrix.  With ``routing``
    "top_then_softmax" the router's logits get a bias, the largest are chosen and weighted by the softmax over the
    chosen ones alone.  The router's logits are a float32 product (its weight is kept in 32 bits, with the shared expert's gate vector as
    one more row); one kernel forms the softmax, adds the correction, picks the experts and their weights.  The
    tokens' rows are then grouped by expert on the device (no count travels to the host: the launch sizes depend on
    the number of tokens alone): each expert's rows fill whole tiles of the grouped products, gate/up with the
    activation in its epilogue, then down into float32 rows, which a last kernel weights and sums token by token, in
    the order of the token's choices, together with the gated shared expert.  A token's result does not depend on
    which other tokens share its expert's tiles: a row of a tile is summed on its own.  The output is float32."""
    graph_safe = True
    kernel_modules = ("common", "gemm", "moe")

    @classmethod
    def expected_tensors(cls, spec, prefix: str, hidden_size: int):
        out = [Expect(f"{prefix}.router.weight", ((spec.num_experts, hidden_size),))]
        if spec.routing == "top_then_softmax":
            out.append(Expect(f"{prefix}.router.bias", ((spec.num_experts,),), init="bias"))
        else:
            out.append(Expect(f"{prefix}.correction", ((spec.num_experts,),), init="bias"))
        gated = getattr(spec.activation, "gated", True)
        for number in range(spec.num_experts):
            if gated:
                out.append(Expect(f"{prefix}.e{number}.gate.weight", ((spec.expert_size, hidden_size),)))
            out += [Expect(f"{prefix}.e{number}.up.weight", ((spec.expert_size, hidden_size),)),
                    Expect(f"{prefix}.e{number}.down.weight", ((hidden_size, spec.expert_size),))]
        if spec.shared_size is not None:
            out += [Expect(f"{prefix}.shared.gate.weight", ((spec.shared_size, hidden_size),)),
                    Expect(f"{prefix}.shared.up.weight", ((spec.shared_size, hidden_size),)),
                    Expect(f"{prefix}.shared.down.weight", ((hidden_size, spec.shared_size),)),
                    Expect(f"{prefix}.shared.sg.weight", ((1, hidden_size),))]
        return out

    @classmethod
    def limits(cls, spec, hidden_size: int):
        return beyond("routed_experts", "num_experts", spec.num_experts, MOE_MAX_EXPERTS,
                      "the experts' counts and a token's scores are kept in LDS and registers")

    def __init__(self, spec, prefix: str, tensors, build: BuildContext):
        self.spec = spec
        self.build = build
        get = lambda name: tensors[f"{prefix}.{name}"]
        experts, inner, hidden = spec.num_experts, spec.expert_size, build.hidden_size
        # rows of 16-byte pieces for the bfloat16 matrix cores, else the float32 kernel (any width)
        keep = torch.float32 if (build.dtype == torch.float32 or hidden % 8 or inner % 8) else torch.bfloat16
        self.gated = getattr(spec.activation, "gated", True)
        if self.gated:
            first = [torch.cat([get(f"e{number}.gate.weight"), get(f"e{number}.up.weight")]) for number in range(experts)]
        else:
            first = [get(f"e{number}.up.weight") for number in range(experts)]
        self.gate_up = torch.stack(first).to(keep).contiguous().to(build.device)
        self.down = torch.stack([get(f"e{number}.down.weight") for number in range(experts)]) \
            .to(keep).contiguous().to(build.device)
        # the router's product has float32 sums; a weight stored in bfloat16 beside bfloat16 rows gives exact float32
        # products on the matrix cores, so it stays as it is stored; any other keeps 32 bits and the float32 kernel
        stored = {get("router.weight").dtype} | ({get("shared.sg.weight").dtype} if spec.shared_size is not None else set())
        route_dtype = torch.bfloat16 if (build.dtype == torch.bfloat16 and stored == {torch.bfloat16} and hidden % 8 == 0) \
            else torch.float32
        router = [get("router.weight").to(route_dtype)]
        self.shared = spec.shared_size is not None
        if self.shared:
            router.append(get("shared.sg.weight").to(route_dtype).reshape(1, hidden))
            self.shared_gate_up = Linear([get("shared.gate.weight"), get("shared.up.weight")], [None, None], build)
            self.shared_down = Linear([get("shared.down.weight")], [None], build)
        self.router = torch.cat(router).contiguous().to(build.device)
        # what is added to a token's scores before the choice: a correction of the softmax, or the logits' bias
        added = "router.bias" if spec.routing == "top_then_softmax" else "correction"
        self.correction = get(added).to(torch.float32).contiguous().to(build.device)
        # rows and matrices in whole 16-byte pieces: the widest tiles of the grouped products take nothing else
        piece = 4 if keep == torch.float32 else 8
        self.whole_pieces = hidden % piece == 0 and inner % piece == 0

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        spec = self.spec
        tokens, hidden = x.shape
        logits = ops.linear(x, self.router, None, keep_float32=True)          # float32 [T, experts (+ 1)]
        chosen, weights, gate = ops.moe_route(logits, spec.num_experts, spec.top_k, self.correction, spec.route_scale,
                                              spec.weight_eps, self.shared, routing=spec.routing)
        plan = ops.moe_plan(chosen, spec.num_experts,
                            ops.moe_tile_rows(tokens, spec.top_k, spec.num_experts, self.whole_pieces))
        rows = x if x.dtype == self.gate_up.dtype else x.to(self.gate_up.dtype)
        inner = torch.empty((plan.capacity, spec.expert_size), dtype=rows.dtype, device=x.device)
        ops.moe_expert_gemm(rows, plan, self.gate_up, inner, gather=True, glu=spec.activation if self.gated else None,
                            squared_relu=not self.gated)
        down = torch.empty((plan.capacity, hidden), dtype=torch.float32, device=x.device)
        ops.moe_expert_gemm(inner, plan, self.down, down, gather=False, glu=None)
        shared_rows = None
        if self.shared:
            act = spec.shared_activation
            gate_up = self.shared_gate_up(x)
            activated = torch.empty((tokens, spec.shared_size), dtype=gate_up.dtype, device=x.device)
            ops.clamped_glu(gate_up, act.limit, act.alpha, act.up_offset, activated)
            shared_rows = self.shared_down(activated)
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=x.device)
        ops.moe_combine(down, plan, weights, shared_rows, gate, out)
        return out
