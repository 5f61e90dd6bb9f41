"""The routers PiKVMoE instantiates (core/single/routing_strategy.py): ExpertRouter,
LoadBalancingRouter, ImportanceAwareRouter and their blend, AdaptiveRouter - same
constructors, parameter names (a reference state_dict loads) and return tuples.

What stays in torch: the small MLPs (gate, importance predictor, router selector) and the
losses built on their outputs.  What runs natively: every softmax + top-k + renormalise
(`pikv_router_tail`, one wavefront per token), with this build's total order - value
descending, lower expert first among equal float32 values - where torch.topk leaves ties
unspecified.  Values come from the kernel; when gradients are wanted, the same quantities
recomputed by torch carry them (value = kernel, gradient = torch), as in routing.py.
"""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops


def _with_grad(value: torch.Tensor, differentiable: torch.Tensor) -> torch.Tensor:
    """`value` with the gradient of `differentiable` (same quantity, torch arithmetic)."""
    if not (torch.is_grad_enabled() and differentiable.requires_grad):
        return value
    return value + (differentiable - differentiable.detach())


def _softmax_topk(logits: torch.Tensor, top_k: int):
    """softmax -> top-k -> renormalise of [B,S,E] logits through the native tail
    (core/single/routing_strategy.py:47-53).  Returns (probs [B,S,E], idx [B,S,k] int64,
    weights [B,S,k])."""
    B, S, E = logits.shape
    flat = logits.detach().reshape(B * S, E).float().contiguous()
    r = ops.router_tail(flat, top_k=top_k)
    probs = r.probs.view(B, S, E)
    idx = r.topk_idx.long().view(B, S, -1)
    w = r.topk_w.view(B, S, -1)
    if torch.is_grad_enabled() and logits.requires_grad:
        p_t = F.softmax(logits.float(), dim=-1)
        sel = p_t.gather(-1, idx)
        probs = _with_grad(probs, p_t)
        w = _with_grad(w, sel / sel.sum(dim=-1, keepdim=True))
    return probs, idx, w


class ExpertRouter(nn.Module):
    """core/single/routing_strategy.py:6-55."""

    def __init__(self, hidden_size, num_experts, top_k=2, temperature=1.0):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_experts = num_experts
        self.top_k = top_k
        self.temperature = temperature
        self.router = nn.Sequential(
            nn.Linear(hidden_size, hidden_size),
            nn.ReLU(),
            nn.Linear(hidden_size, num_experts),
        )
        self.expert_capacity = nn.Parameter(torch.ones(num_experts))

    def forward(self, x, expert_mask=None):
        """x [B,S,H]; expert_mask [E] is ADDED to the logits (:45-46).  Returns
        (routing_weights [B,S,E], expert_indices [B,S,k], top_k_weights [B,S,k])."""
        if not x.is_cuda:
            raise ValueError("pikv_amd routers run on the GPU only")
        logits = self.router(x) / self.temperature
        if expert_mask is not None:
            logits = logits + expert_mask.unsqueeze(0).unsqueeze(0)
        return _softmax_topk(logits, min(self.top_k, self.num_experts))


class LoadBalancingRouter(ExpertRouter):
    """core/single/routing_strategy.py:57-71."""

    def __init__(self, hidden_size, num_experts, top_k=2, temperature=1.0, balance_weight=0.01):
        super().__init__(hidden_size, num_experts, top_k, temperature)
        self.balance_weight = balance_weight

    def forward(self, x, expert_mask=None):
        routing_weights, expert_indices, top_k_weights = super().forward(x, expert_mask)
        expert_usage = routing_weights.mean(dim=0).mean(dim=0)
        load_balance_loss = self.balance_weight * (expert_usage.std() / expert_usage.mean())
        return routing_weights, expert_indices, top_k_weights, load_balance_loss


class ImportanceAwareRouter(ExpertRouter):
    """core/single/routing_strategy.py:73-98."""

    def __init__(self, hidden_size, num_experts, top_k=2, temperature=1.0):
        super().__init__(hidden_size, num_experts, top_k, temperature)
        self.importance_predictor = nn.Sequential(
            nn.Linear(hidden_size, hidden_size // 2),
            nn.ReLU(),
            nn.Linear(hidden_size // 2, 1),
            nn.Sigmoid(),
        )

    def forward(self, x, expert_mask=None):
        importance = self.importance_predictor(x)
        routing_weights, expert_indices, top_k_weights = super().forward(x, expert_mask)
        routing_weights = routing_weights * importance
        routing_weights = routing_weights / routing_weights.sum(dim=-1, keepdim=True)
        return routing_weights, expert_indices, top_k_weights, importance


class AdaptiveRouter(nn.Module):
    """core/single/routing_strategy.py:100-150: a per-sequence blend of the two routers
    above, then top-k of the blended weights and renormalisation."""

    def __init__(self, hidden_size, num_experts, top_k=2, temperature=1.0):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_experts = num_experts
        self.top_k = top_k
        self.temperature = temperature
        self.load_balancing_router = LoadBalancingRouter(hidden_size, num_experts, top_k, temperature)
        self.importance_router = ImportanceAwareRouter(hidden_size, num_experts, top_k, temperature)
        self.router_selector = nn.Sequential(
            nn.Linear(hidden_size, hidden_size // 2),
            nn.ReLU(),
            nn.Linear(hidden_size // 2, 2),
            nn.Softmax(dim=-1),
        )

    def forward(self, x, expert_mask=None):
        if x.dim() == 2:
            x = x.unsqueeze(-1).expand(-1, -1, self.hidden_size)
        elif x.dim() == 1:
            x = x.unsqueeze(0).unsqueeze(-1).expand(-1, -1, self.hidden_size)
        x_mean = x.mean(dim=1)
        router_weights = self.router_selector(x_mean)
        lb_weights, _, _, lb_loss = self.load_balancing_router(x, expert_mask)
        imp_weights, _, _, importance = self.importance_router(x, expert_mask)
        routing_weights = (router_weights[:, 0:1, None] * lb_weights +
                           router_weights[:, 1:2, None] * imp_weights)
        # top-k of the blended weights themselves (no second softmax): the native raw top-k
        B, S, E = routing_weights.shape
        k = min(self.top_k, E)
        r = ops.router_tail(routing_weights.detach().reshape(B * S, E).float().contiguous(), top_k=k,
                            use_softmax=False)
        expert_indices = r.topk_idx.long().view(B, S, k)
        top_k_weights = routing_weights.gather(-1, expert_indices)
        top_k_weights = top_k_weights / top_k_weights.sum(dim=-1, keepdim=True)
        return routing_weights, expert_indices, top_k_weights, lb_loss, importance
