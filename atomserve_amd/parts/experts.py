"""Feed-forward layers made of experts: every token runs through a few of several small gated
feed-forwards, down_e(act(gate_e h) * (up_e h)), and their outputs are added with a weight each.

Which experts a token uses is found on the GPU, so a step never waits for the host and a decode step can
be replayed as a graph.  `TableExperts` reads them from a table indexed by the token's id (no router of
its own: every chosen expert weighs 1 / top); another way of choosing is another `route`.
"""

import torch

from atomserve_amd.kernels import ops
from atomserve_amd.parts.base import FeedForward, WeightDecl, register


class TableExperts(FeedForward):
    capturable = True

    def __init__(self, spec, env):
        super().__init__(spec, env)
        if spec.activation != "silu":
            raise ValueError(f"activation {spec.activation!r} has no kernel (only 'silu')")
        if not 1 <= spec.top <= spec.num_experts <= ops.MOE_MAX_EXPERTS:
            raise ValueError(f"{spec.top} of {spec.num_experts} experts (at most {ops.MOE_MAX_EXPERTS}) cannot be chosen")

    def weight_decls(self) -> dict:
        s = self.spec
        return {
            "gate.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "up.weight": WeightDecl((s.num_experts, s.intermediate_size, s.hidden_size)),
            "down.weight": WeightDecl((s.num_experts, s.hidden_size, s.intermediate_size)),
            "table": WeightDecl((s.vocab_size, s.top), role="table_int"),
        }

    def bind(self, tensors: dict) -> None:
        super().bind(tensors)
        # every expert's gate rows, then its up rows: what the first grouped product reads
        self.gate_up_weight = torch.cat([self.gate_weight, self.up_weight], dim=1).contiguous()
        del self.gate_weight, self.up_weight

    def route(self, step):
        """The step's (token, expert) pairs sorted by expert; every layer with the same table object shares it."""
        key = ("table_experts", self.table.data_ptr())
        found = step.shared.get(key)
        if found is None:
            found = step.shared[key] = ops.moe_route_table(step.token_ids, self.table, self.spec.num_experts)
        return found

    def forward(self, h, step):
        s, env = self.spec, self.env
        T, dev = h.shape[0], h.device
        route = self.route(step)
        pairs = T * s.top
        act = torch.empty((pairs, s.intermediate_size), dtype=env.dtype, device=dev)
        ops.moe_gemm(h, self.gate_up_weight, route, act, gated=True, per_token=True)
        if s.top == 1:
            y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
            ops.moe_gemm(act, self.down_weight, route, y, gated=False, per_token=False)
            return y
        each = torch.empty((pairs, s.hidden_size), dtype=torch.float32, device=dev)
        ops.moe_gemm(act, self.down_weight, route, each, gated=False, per_token=False)
        y = torch.empty((T, s.hidden_size), dtype=env.dtype, device=dev)
        ops.moe_combine(each, s.top, 1.0 / s.top, y)
        return y


register("feed_forward", "table_experts", TableExperts)
