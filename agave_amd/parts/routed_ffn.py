"""A routed feed-forward: a mixture of gated experts with a shared expert.

The router's logits are a 32-bit product of the feed-forward's input with the router matrix (kept in
32-bit).  Scores are the softmax over all router outputs; the choice goes by score + correction among the
outputs of the best groups, the weights are the plain scores times a factor (see
``agave_amd.config.spec.RoutedFfnSpec``); or (``score="softmax_top"``) the largest logits plus a bias are chosen and
weighted by the softmax over the chosen alone.  Outputs past the experts with weights are identity experts:
their result is the input row.  The chosen experts' rows are summed with their weights, the shared
expert's row is added, times the sigmoid of a logit per token where it has a gate (the gate's vector rides along
as one more row of the router matrix, so its product costs no kernel).

Nothing on the host depends on the choice: every launch has the same shape whatever the tokens are, so a
decode step is recorded into a graph like any other.
"""
from __future__ import annotations

from typing import List

import torch

from ..config.spec import RoutedFfnSpec
from ..ops import kernels, routed
from ..weights.loader import TensorNeed
from .base import BuildEnv, register
from .ffn import GatedFfn


class RoutedFfn:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("routed_ffn",)

    def __init__(self, spec: RoutedFfnSpec, weights, env: BuildEnv):
        s = spec
        if s.activation not in kernels.GATE_ACTIVATIONS:
            raise ValueError(f"routed feed-forward: unsupported activation {s.activation!r}; known: {sorted(kernels.GATE_ACTIVATIONS)}")
        self.n_outputs = s.n_experts + s.n_identity
        if self.n_outputs < 1 or self.n_outputs > routed.MAX_OUTPUTS:
            raise ValueError(f"routed feed-forward: {self.n_outputs} router outputs (1 to {routed.MAX_OUTPUTS})")
        if s.groups < 1 or s.groups > 64 or self.n_outputs % s.groups:
            raise ValueError(f"routed feed-forward: {self.n_outputs} router outputs do not form {s.groups} equal groups (at most 64)")
        if not 1 <= s.keep_groups <= s.groups:
            raise ValueError(f"routed feed-forward: {s.keep_groups} of {s.groups} groups kept")
        if not 1 <= s.top <= s.keep_groups * (self.n_outputs // s.groups):
            raise ValueError(f"routed feed-forward: {s.top} experts chosen of {s.keep_groups * (self.n_outputs // s.groups)} that can be")
        if s.score not in ("softmax_all", "softmax_top", "sigmoid"):
            raise ValueError(f"routed feed-forward: unknown way of scoring {s.score!r} (softmax_all, softmax_top, sigmoid)")
        if s.group_top not in (1, 2) or (s.normalise and (s.top > 64 or s.score == "softmax_top")):
            raise ValueError("routed feed-forward: a group counts by its largest or its two largest scores; weights are divided "
                             "by their sum for at most 64 chosen experts")
        if s.score == "softmax_top" and (s.groups != 1 or s.top > 64 or s.n_identity):
            raise ValueError("routed feed-forward: the softmax over the chosen logits takes no groups, no identity experts "
                             "and at most 64 chosen")
        if s.shared_gate and s.shared is None:
            raise ValueError("routed feed-forward: a gate on the shared expert needs a shared expert")
        self.spec, self.env = spec, env
        self.act = kernels.GATE_ACTIVATIONS[s.activation]
        dev = env.device
        # the router stays 32-bit in both engines
        rows = [weights.get(s.router).to(torch.float32)]
        if s.shared_gate:
            rows.append(weights.get(s.shared_gate).to(torch.float32).view(1, s.hidden))
        self.router = torch.cat(rows, 0).contiguous().to(dev)
        self.correction = weights.get(s.correction).to(torch.float32).contiguous().to(dev) if s.correction else None

        def stack(which: str) -> torch.Tensor:
            mats = [weights.get(f"{s.expert_prefix}{i}.{which}") for i in range(s.n_experts)]
            return torch.stack([m.to(env.dtype) for m in mats]).contiguous().to(dev)     # [experts, out, in]
        # bfloat16 experts whose sizes are multiples of 32 are kept in the matrix cores' tile order (only that copy)
        self.tile_order = bool(s.n_experts) and env.dtype == torch.bfloat16 and s.hidden % 32 == 0 and s.intermediate % 32 == 0
        if s.n_experts:
            self.w_gate, self.w_up, self.w_down = stack(s.gate_name), stack(s.up_name), stack(s.down_name)
            if self.tile_order:
                self.w_gate, self.w_up, self.w_down = (routed.pack_expert_weights(w) for w in (self.w_gate, self.w_up, self.w_down))
        else:
            self.w_gate = self.w_up = self.w_down = None
        self.shared = GatedFfn(s.shared, weights, env) if s.shared is not None else None

    @staticmethod
    def tensor_needs(spec: RoutedFfnSpec) -> List[TensorNeed]:
        s = spec
        r = s.n_experts + s.n_identity
        needs = []
        for i in range(s.n_experts):
            p = f"{s.expert_prefix}{i}."
            needs += [TensorNeed(p + s.gate_name, (s.intermediate, s.hidden)), TensorNeed(p + s.up_name, (s.intermediate, s.hidden)),
                      TensorNeed(p + s.down_name, (s.hidden, s.intermediate))]
        needs.append(TensorNeed(s.router, (r, s.hidden)))
        if s.correction:
            needs.append(TensorNeed(s.correction, (r,)))
        if s.shared is not None:
            needs += GatedFfn.tensor_needs(s.shared)
        if s.shared_gate:
            needs.append(TensorNeed(s.shared_gate, (1, s.hidden)))
        return needs

    def forward(self, x: torch.Tensor, step) -> torch.Tensor:
        s, ws = self.spec, self.env.workspace
        n, r, top = x.shape[0], self.n_outputs, s.top
        choice = ws.get("router_choice", n, top, torch.int32)
        weight = ws.get("router_weight", n, top, torch.float32)
        # the router's 32-bit product and the choice in one kernel
        shared_gate = ws.get("router_shared_gate", n, 1, torch.float32) if s.shared_gate else None
        routed.route_rows(x, self.router, self.correction, s.groups, s.keep_groups, top, s.route_scale, choice, weight,
                          softmax_top=s.score == "softmax_top", extra_out=shared_gate, sigmoid=s.score == "sigmoid",
                          group_top=s.group_top, normalise=s.normalise)
        y = place = None
        if self.tile_order and not routed.mfma_ok(x, s.intermediate):
            raise ValueError("routed feed-forward: its experts are kept in tile order, which takes aligned bfloat16 rows")
        if s.n_experts and self.w_gate.dtype == torch.bfloat16 and routed.mfma_ok(x, s.intermediate):
            # the pairs sorted by expert on the device, then the experts' products tile by tile on the matrix cores
            tm, tiles, cap = routed.tile_plan(n * top, s.n_experts)
            place = ws.get("expert_place", n * top, 1, torch.int32).view(-1)
            sorted_pair = ws.get(f"expert_sorted{tm}", cap, 1, torch.int32).view(-1)
            tile_expert = ws.get(f"expert_tiles{tm}", tiles, 1, torch.int32).view(-1)
            routed.route_sort(choice.view(-1), s.n_experts, tm, tiles, place, sorted_pair, tile_expert)
            act_rows = ws.get("expert_act", cap, s.intermediate, x.dtype)
            y = ws.get("expert_rows", cap, s.hidden, torch.float32)
            routed.experts_mfma(x, sorted_pair, tile_expert, self.w_gate, self.w_up, self.w_down, act_rows, y, tm, tiles, top,
                                self.act, tile_order=self.tile_order, p0=s.act_limit, p1=s.act_alpha)
        elif s.n_experts:
            act_rows = ws.get("expert_act", n * top, s.intermediate, x.dtype)
            y = ws.get("expert_rows", n * top, s.hidden, torch.float32)
            routed.experts_plain(x, choice.view(-1), self.w_gate, self.w_up, self.w_down, act_rows, y, top, self.act,
                                 s.act_limit, s.act_alpha)
        shared = self.shared.forward(x, step, slices_ok=False, tag="shared_ffn") if self.shared is not None else None
        out = ws.get("routed_out", n, s.hidden, x.dtype)
        routed.combine(y, place, choice.view(-1), weight.view(-1), x, shared, out, top, s.n_experts,
                       shared_gate.view(-1) if shared_gate is not None else None)
        return out


register("ffn", "routed", RoutedFfn)
