"""Top-k routed MoE layers built on the grouped FP8 modules.

Same classes and data flow as the two FP8 layers of the reference's example (fp8_gmm/example.py:
``Fp8LinearModule`` :72-103, ``Fp8MlpModule`` :106-130): a bf16 gating linear, softmax + top-k, grouping of the
(token, choice) pairs by expert, ``gather`` into expert order, the grouped expert computation, and the weighted
``scatter`` back to token order.  The routing operators come from :mod:`fp8_gmm_amd.moe_ops` instead of
megablocks.  Experts that receive no token are allowed (the reference's modules assert against them,
grouped_linear.py:205, grouped_mlp.py:348).
"""
import numpy as np
import torch

from . import moe_ops
from .grouped_linear import GroupedLinear
from .grouped_mlp import GroupedMlp


class _RoutedModule(torch.nn.Module):
    def __init__(self, n_embd, n_inner, n_experts, top_k, dtype, device):
        super().__init__()
        self.n_embd = n_embd
        self.n_inner = n_inner
        self.n_experts = n_experts
        self.top_k = top_k
        self.sort_end_bit = max(int(np.ceil(np.log2(n_experts))), 1)
        self.gating_network = torch.nn.Linear(n_embd, n_experts, bias=False).to(dtype).to(device)
        self._counts_host = None    # page-locked landing place of the per-expert counts, and the event of its copy
        self._counts_ready = None

    def experts(self, x, batch_sizes):
        raise NotImplementedError

    def start_experts(self):
        """Enqueue what the experts' pass can do before the host knows the split (nothing, by default)."""

    def compute(self, x, tokens_per_expert, indices, bin_ids, expert_weights, bins, top_k):
        x = x.view(-1, x.size(-1))
        # The host needs the split to plan the expert launches.  Its copy is enqueued ahead of the gather and of the
        # experts' weight casts, which need nothing from the host: the GPU has that work to do while the host waits
        # for the counts and plans the launches.
        if self._counts_host is None or self._counts_host.numel() != tokens_per_expert.numel():
            self._counts_host = torch.empty(tokens_per_expert.shape, dtype=tokens_per_expert.dtype, pin_memory=True)
            self._counts_ready = torch.cuda.Event()
        self._counts_host.copy_(tokens_per_expert, non_blocking=True)
        self._counts_ready.record()
        x = moe_ops.gather(x, indices, bin_ids, bins, top_k)
        self.start_experts()
        self._counts_ready.synchronize()
        batch_sizes = self._counts_host.to(torch.long, copy=True)   # the page-locked buffer is reused by the next step
        out = self.experts(x, batch_sizes)
        return moe_ops.scatter(out, indices, bin_ids, expert_weights, bins, top_k)

    def forward(self, input):
        input = input.view(-1, input.size(-1))
        routing_logits = self.gating_network(input)
        weights0, selected_experts = moe_ops.topk(routing_logits, self.top_k)
        expert_weights = weights0.flatten()
        top_experts = selected_experts.flatten()
        with torch.no_grad():
            indices, bin_ids, bins, tokens_per_expert = moe_ops.indices_and_bins(
                top_experts, self.sort_end_bit, self.n_experts)
        return self.compute(input, tokens_per_expert, indices, bin_ids, expert_weights, bins, self.top_k)


class Fp8LinearModule(_RoutedModule):
    """Two ``GroupedLinear`` layers with an (erf) GELU between them (fp8_gmm/example.py:72-103)."""

    def __init__(self, n_embd, n_inner, n_experts, top_k, dtype=torch.bfloat16, cutlass=False, device="cuda"):
        super().__init__(n_embd, n_inner, n_experts, top_k, dtype, device)
        self.grouped_linear1 = GroupedLinear(n_embd, n_inner, n_experts, dtype=dtype, cutlass=cutlass, device=device)
        self.grouped_linear2 = GroupedLinear(n_inner, n_embd, n_experts, dtype=dtype, cutlass=cutlass, device=device)
        self.act = torch.nn.GELU()

    def start_experts(self):
        self.grouped_linear1.cast_weights_ahead()
        self.grouped_linear2.cast_weights_ahead()

    def experts(self, x, batch_sizes):
        return self.grouped_linear2(self.act(self.grouped_linear1(x, batch_sizes)), batch_sizes)


class Fp8MlpModule(_RoutedModule):
    """One ``GroupedMlp`` (tanh-GELU fused into the first GEMM) as the experts (fp8_gmm/example.py:106-130)."""

    def __init__(self, n_embd, n_inner, n_experts, top_k, dtype=torch.bfloat16, device="cuda"):
        super().__init__(n_embd, n_inner, n_experts, top_k, dtype, device)
        self.grouped_mlp = GroupedMlp(n_embd, n_inner, n_experts, dtype=dtype, device=device)

    def start_experts(self):
        self.grouped_mlp.cast_weights_ahead()

    def experts(self, x, batch_sizes):
        return self.grouped_mlp(x, batch_sizes)
