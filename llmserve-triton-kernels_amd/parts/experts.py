"""A feed-forward of many small experts, of which each token uses `top`.

Parameters (a `PartSpec` of kind "experts"): hidden, intermediate (of one expert), experts, top, limit,
renormalize (default False: the weights are the chosen scores as they are), names (local names: "router", and the
pattern of an expert's matrices, default "e{e}.gate", "e{e}.up", "e{e}.down"), and, with defaults that leave them
out: scores ("sigmoid" or "softmax" over all experts), groups and keep (the experts form `groups` equal groups of
neighbours, a group's score is its largest, only experts of the `keep` best groups can be chosen), renorm_eps (added
to the sum that `renormalize` divides by), weight_on ("input": the weight multiplies the expert's input; "output":
its result), unit ("clamped" or "silu"), router_bias (True: a bias per expert, tensor "<router>.b", is added to z),
shared ({"intermediate": I, "gate": True or False}: one more SiLU-gated unit of its own width that every token uses,
tensors "shared.gate", "shared.up", "shared.down"; with "gate" its result is multiplied by sigmoid(w_sg . h), one number
per token, tensor "shared.sg" [1, hidden]).

Router: z = W_router h in 32-bit, scores sigmoid(z) or softmax(z), the `top` largest chosen.  With weight_on
"input" y = sum over chosen e of expert_e(w_e h), with "output" y = sum of w_e expert_e(h).  Expert, unit "clamped":
a = min(W_gate x, limit), b = clamp(W_up x, -limit, limit), W_down (a sigmoid(1.702 a) (b + 1)); unit "silu":
W_down (a sigmoid(a) b) with a = W_gate x, b = W_up x.  No biases.

One step: route, sort the (token, choice) pairs by expert on the device (stably, so a pair's place does not depend
on what else is in the batch beyond which rows share its tile), scatter the weighted inputs into that order, two
products with a weight per segment of rows (the first with the gated unit in its epilogue: gate and up rows
lie in blocks of 32 in one stacked weight), and a sum over each token's choices in their order.  Nothing is read back: the
grids are sized by the number of pairs.
"""

from __future__ import annotations

import torch

from ..ops import library as ops
from .registry import FeedForward, register_feed_forward
from .spec import ParamInfo

_DEFAULT_NAMES = {"router": "router", "gate": "e{e}.gate", "up": "e{e}.up", "down": "e{e}.down", "router_bias": "router.b",
                  "shared_gate": "shared.gate", "shared_up": "shared.up", "shared_down": "shared.down", "shared_sg": "shared.sg"}


@register_feed_forward("experts")
class Experts(FeedForward):
    graph_safe = True

    def __init__(self, spec, ctx):
        super().__init__(spec, ctx)
        self.hidden = int(spec["hidden"])
        self.intermediate = int(spec["intermediate"])
        self.experts = int(spec["experts"])
        self.top = int(spec["top"])
        self.unit = spec.get("unit", "clamped")
        self.limit = float(spec["limit"]) if self.unit == "clamped" else 0.0
        self.renormalize = bool(spec.get("renormalize", False))
        self.renorm_eps = float(spec.get("renorm_eps", 0.0))
        self.scores = spec.get("scores", "sigmoid")
        self.groups = int(spec.get("groups") or 1)
        self.keep = int(spec.get("keep") or self.groups)
        self.weight_on = spec.get("weight_on", "input")
        if self.unit not in ("clamped", "silu") or self.scores not in ("sigmoid", "softmax") or \
                self.weight_on not in ("input", "output"):
            raise ValueError(f"unit={self.unit!r}, scores={self.scores!r}, weight_on={self.weight_on!r}")
        if self.experts % self.groups or not 1 <= self.keep <= self.groups or \
                (self.groups > 1 and self.top > self.keep * (self.experts // self.groups)):
            raise ValueError(f"{self.groups} groups of which {self.keep} are kept do not fit {self.experts} experts "
                             f"of which {self.top} are chosen")
        self.names = dict(_DEFAULT_NAMES, **(spec.get("names") or {}))
        self.router_bias = bool(spec.get("router_bias", False))
        shared = spec.get("shared") or None
        self.shared_intermediate = int(shared["intermediate"]) if shared else 0
        self.shared_gated = bool(shared.get("gate", False)) if shared else False
        if shared and self.shared_intermediate < 1:
            raise ValueError("the shared unit needs a positive width")
        self.b_router = None
        self.shared_unit = None  # the shared expert: the engine's dense gated feed-forward under its own tensor names
        if shared:
            from .registry import FEED_FORWARDS
            from .spec import PartSpec

            n = self.names
            self.shared_unit = FEED_FORWARDS.build(PartSpec("swiglu", {
                "hidden": self.hidden, "intermediate": self.shared_intermediate, "result": "float32",
                "names": {"gate": n["shared_gate"], "up": n["shared_up"], "down": n["shared_down"]}}), ctx)
        if not 1 <= self.top <= min(self.experts, ops.MOE_MAX_TOP):
            raise ValueError(f"top={self.top} of {self.experts} experts (at most {ops.MOE_MAX_TOP})")
        self.w_router = self.w_gate_up = self.w_down = None

    def libraries(self, dtype_name):
        return ("moe", "grouped_gemm")

    def param_infos(self):
        h, i, n = self.hidden, self.intermediate, self.names
        infos = {n["router"]: ParamInfo((self.experts, h))}
        for e in range(self.experts):
            infos[n["gate"].format(e=e)] = ParamInfo((i, h))
            infos[n["up"].format(e=e)] = ParamInfo((i, h))
            infos[n["down"].format(e=e)] = ParamInfo((h, i))
        if self.router_bias:
            infos[n["router_bias"]] = ParamInfo((self.experts,), "around_zero")
        if self.shared_unit is not None:
            infos.update(self.shared_unit.param_infos())
            if self.shared_gated:
                infos[n["shared_sg"]] = ParamInfo((1, h))
        return infos

    def load(self, tensors):
        n = self.names
        self.w_router = tensors[n["router"]].contiguous()
        if self.router_bias:
            self.b_router = tensors[n["router_bias"]].float().contiguous()
        if self.shared_unit is not None:
            self.shared_unit.load({name: tensors[name] for name in self.shared_unit.param_infos()})
            if self.shared_gated:  # the gate's row lies behind the experts' in the router's matrix: one kernel forms both
                self.w_router = torch.cat([self.w_router, tensors[n["shared_sg"]].reshape(1, self.hidden)], dim=0).contiguous()
        # [E, 64 ceil(I / 32), H]: blocks of 32 gate rows and the 32 up rows of the same units, so that a thread of
        # the product holds both of a unit
        self.w_gate_up = ops.stack_paired(torch.stack([tensors[n["gate"].format(e=e)] for e in range(self.experts)]),
                                          torch.stack([tensors[n["up"].format(e=e)] for e in range(self.experts)]))
        self.w_down = torch.stack([tensors[n["down"].format(e=e)] for e in range(self.experts)]).contiguous()

    def forward(self, x):
        rows, dev = x.shape[0], x.device
        pairs = rows * self.top
        chosen = torch.empty((rows, self.top), dtype=torch.int32, device=dev)
        weight = torch.empty((rows, self.top), dtype=torch.float32, device=dev)
        shared_gate = torch.empty((rows, 1), dtype=torch.float32, device=dev) if self.shared_gated else None
        ops.moe_router(chosen, weight, x, self.w_router, renormalize=self.renormalize, scores=self.scores,
                       groups=self.groups, keep=self.keep, renorm_eps=self.renorm_eps, bias=self.b_router,
                       extra_out=shared_gate)
        shared = self.shared_unit.forward(x) if self.shared_unit is not None else None
        on_input = self.weight_on == "input"
        sorted_in = torch.empty((pairs, self.hidden), dtype=x.dtype, device=dev)
        place = torch.empty(pairs, dtype=torch.int32, device=dev)
        if 0 < pairs <= ops.MOE_FEW_PAIRS:  # (decoding: one launch instead of three)
            seg, tiles = ops.moe_place_few(sorted_in, place, x, chosen, weight if on_input else None, self.experts)
        else:
            rank, seg, tiles = ops.moe_sort(chosen, self.experts)
            ops.moe_scatter(sorted_in, place, x, chosen, weight if on_input else None, rank, seg)
        act = torch.empty((pairs, self.intermediate), dtype=x.dtype, device=dev)
        ops.grouped_product(act, sorted_in, self.w_gate_up, epilogue="paired", segments=(seg, tiles), limit=self.limit,
                            units=self.intermediate, unit=self.unit)
        # (few rows: the last product's K is shared out, and the sum over a token's choices adds the shares up as well)
        parts = ops.grouped_k_parts(act, self.w_down, ops.compute_units(dev))
        shape = (pairs, self.hidden) if parts == 1 else (parts, pairs, self.hidden)
        results = torch.empty(shape, dtype=torch.float32, device=dev)
        ops.grouped_product(results, act, self.w_down, segments=(seg, tiles), k_parts=parts)
        return ops.moe_combine(torch.empty((rows, self.hidden), dtype=torch.float32, device=dev), results, place,
                               None if on_input else weight, always=shared,
                               always_gate=None if shared_gate is None else shared_gate.view(rows))
