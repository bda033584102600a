"""A feed-forward of many small experts, of which every token uses a few.

An expert is down(act(up(x))) without biases, act the square of relu.  Which experts a token uses is read from
a table by its token id (``table_experts``: a row of ``top`` distinct experts per id, each weighted 1 / top;
there is no router).  An optional shared expert of the same form runs for every token and is added.

The step's (token, choice) entries are put in the order of their experts on the device, the two products run
over tiles of that order, and a token's outputs are added in the order of its choices: no sum depends on what
else the step holds, nothing is decided on the host, and a captured step replays.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .base import MATRIX, TABLE, FeedForward, PartError, TensorReq, register_part


@register_part("ffn", "table_experts")
class TableExperts(FeedForward):
    NEEDS_STEP = True            # the experts are chosen by the step's token ids
    LAUNCHES = 9
    GRAPH_SAFE_PORTIONS = True   # every grid follows the step's shape; the choices are read on the device

    def __init__(self, hidden_size: int, vocab_size: int, num_experts: int, top: int, expert_size: int,
                 shared_size: int = 0):
        if not 1 <= int(top) <= int(num_experts):
            raise PartError(f"table_experts: {top} of {num_experts} experts a token")
        self.hidden_size, self.vocab_size = int(hidden_size), int(vocab_size)
        self.num_experts, self.top, self.expert_size = int(num_experts), int(top), int(expert_size)
        self.shared_size = int(shared_size or 0)
        self.table = self.up_t = self.down_t = self.shared_up = self.shared_down = None

    def tensors(self):
        h, f = self.hidden_size, self.expert_size
        t = {"table": TensorReq((self.vocab_size, self.top), TABLE, high=self.num_experts)}
        for e in range(self.num_experts):
            t[f"e{e}.up"] = TensorReq((f, h), MATRIX)
            t[f"e{e}.down"] = TensorReq((h, f), MATRIX)
        if self.shared_size:
            t["shared.up"] = TensorReq((self.shared_size, h), MATRIX)
            t["shared.down"] = TensorReq((h, self.shared_size), MATRIX)
        return t

    def load(self, tensors, dtype, device):
        n = self.num_experts
        self.table = tensors["table"]
        # one tensor [expert, out, in] per product
        self.up_t = K.GroupedWeight(torch.stack([tensors[f"e{e}.up"] for e in range(n)]))
        self.down_t = K.GroupedWeight(torch.stack([tensors[f"e{e}.down"] for e in range(n)]))
        if self.shared_size:
            self.shared_up = K.prepare_weight(tensors["shared.up"])
            self.shared_down = K.prepare_weight(tensors["shared.down"])

    def forward(self, x, step=None):
        if step is None:
            raise PartError("table_experts: the step's token ids are needed to choose the experts")
        choice = K.moe_choices_by_table(step.token_ids, self.table, self.num_experts)
        eo = K.moe_order(choice, self.num_experts, self.top)
        mid = K.moe_linear(x, self.up_t, eo, from_tokens=True, relu_squared_epilogue=True)
        y = K.moe_linear(mid, self.down_t, eo, from_tokens=False, out_dtype=torch.float32)
        base: Optional[torch.Tensor] = None
        if self.shared_size:
            base = K.as_tensor(K.linear(K.relu_squared(K.linear(x, self.shared_up)), self.shared_down))
        return K.moe_combine(y, eo, 1.0 / self.top, base, x.dtype)
