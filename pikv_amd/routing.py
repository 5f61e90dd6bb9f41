"""Routers with the reference's interface (core/single/pikv_routing.py), whose
tail - last gate Linear, logit scaling / mask, softmax, top-k, renormalisation,
capacity slots - runs in the fused HIP router.

  BaseRouter ........... :7-161    forward(hidden_states, expert_mask=None)
                                   -> (dispatch, combine, router_probs, aux_loss)
  TopKBalancedRouter ... :163-222  (+ entropy / cv / l2 balance term)
  PiKVRouter ........... :380-549  two gates chosen per token by an importance
                                   mask, cache-usage correction factor, 5-tuple
  EPLBRouter ........... :551-735  /temperature then *expert_weights, KL + z loss
  HierarchicalRouter ... :737-860  group softmax x in-group softmax, top-k of the
                                   products (the per-group MLPs stay in torch)

The hidden layers of the gate MLPs and the auxiliary losses stay in torch (dense
GEMMs and scalar reductions); everything after the last hidden activation goes
through pikv_router_fused / pikv_router_tail.  Capacity slots follow the
token-major sequential rule of core/single/module/pikv_routing.py:93-104 (the
vectorised loop of core/single/pikv_routing.py:107-128 gives every token of a
round the same slot; it is not reproduced).  Ties in the top-k go to the lower
expert index.

Gradients: the integer decisions (expert indices, slots, counts) have none.  The float
outputs (router_probs, top-k weights, logits, and the losses built on them) carry the
native kernel's VALUES and, whenever autograd is recording and a gate parameter or the
input requires grad, the GRADIENT of the same formula evaluated in torch on the selected
experts (value + (torch - torch.detach())), so the gate MLPs train as in the reference.
Under torch.no_grad() nothing is recomputed.

Every forward also accepts return_compact=True and then returns the RouterOut
(topk_idx, topk_w, slot, count, probs) instead of the dense tensors, which at
production shapes cannot exist ([T, E, capacity] floats).
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

# dense [T, E, capacity] tensors are only built below this many elements
DENSE_LIMIT = 1 << 28


def _dense_dispatch_combine(r: ops.RouterOut, batch_size, seq_len, num_experts, capacity):
    T = batch_size * seq_len
    if T * num_experts * max(capacity, 1) > DENSE_LIMIT:
        raise ValueError(
            f"dense dispatch/combine tensors of shape [{T},{num_experts},{capacity}] are too large; "
            "call forward(..., return_compact=True)")
    dev = r.topk_idx.device
    disp = torch.zeros(T, num_experts, capacity, device=dev)
    comb = torch.zeros(T, num_experts, capacity, device=dev)
    keep = r.slot >= 0
    t_idx = torch.arange(T, device=dev).unsqueeze(1).expand_as(r.slot)[keep]
    e_idx = r.topk_idx[keep].long()
    s_idx = r.slot[keep].long()
    disp[t_idx, e_idx, s_idx] = 1.0
    comb[t_idx, e_idx, s_idx] = r.topk_w[keep]
    return (disp.view(batch_size, seq_len, num_experts, capacity),
            comb.view(batch_size, seq_len, num_experts, capacity))


def _dense_legacy_fairscale(r: ops.RouterOut, batch_size, seq_len, num_experts, capacity):
    """Dense tensors the way the fairscale branch of core/single/pikv_routing.py:102-128 fills
    them: round j of the top-k is handled for all tokens at once, every token of the round that
    picked expert e lands on position used[e], and used[e] grows by ONE per round however many
    tokens picked e (an indexed += does not accumulate duplicates).  Small shapes only."""
    T = batch_size * seq_len
    dev = r.topk_idx.device
    disp = torch.zeros(T, num_experts, capacity, device=dev)
    comb = torch.zeros(T, num_experts, capacity, device=dev)
    used = torch.zeros(num_experts, dtype=torch.long, device=dev)
    tok = torch.arange(T, device=dev)
    for j in range(r.topk_idx.shape[1]):
        e = r.topk_idx[:, j].long()
        room = used[e] < capacity
        e_in, t_in = e[room], tok[room]
        pos = used[e_in]
        picked = torch.zeros(num_experts, dtype=torch.bool, device=dev)
        picked[e_in] = True
        used = used + picked.long()
        disp[t_in, e_in, pos] = 1.0
        comb[t_in, e_in, pos] = r.topk_w[:, j][room]
    return (disp.view(batch_size, seq_len, num_experts, capacity),
            comb.view(batch_size, seq_len, num_experts, capacity))


def _dense_basic(r: ops.RouterOut, batch_size, seq_len, num_experts):
    """The non-fairscale branch (core/single/pikv_routing.py:133-153): one position per expert."""
    T = batch_size * seq_len
    dev = r.topk_idx.device
    disp = torch.zeros(T, num_experts, 1, device=dev)
    comb = torch.zeros(T, num_experts, 1, device=dev)
    t_idx = torch.arange(T, device=dev).unsqueeze(1).expand_as(r.topk_idx)
    disp[t_idx, r.topk_idx.long(), 0] = 1.0
    comb[t_idx, r.topk_idx.long(), 0] = r.topk_w
    return disp.view(batch_size, seq_len, num_experts, 1), comb.view(batch_size, seq_len, num_experts, 1)


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _attach_grad(r: ops.RouterOut, logits: torch.Tensor, *, temperature=1.0, expert_scale=None,
                 expert_mask=None, module_arithmetic=False, renorm_eps=0.0) -> ops.RouterOut:
    """Give the float outputs of the native router the gradient of the reference's formula
    (core/single/pikv_routing.py:65-82, :653-660) evaluated in torch on raw gate `logits`
    [T,E] that are part of the autograd graph.  Values stay the kernel's."""
    lg = logits.float()
    if expert_scale is not None:
        expert_scale = torch.as_tensor(expert_scale, dtype=lg.dtype, device=lg.device)
    if expert_mask is not None:
        expert_mask = torch.as_tensor(expert_mask, dtype=lg.dtype, device=lg.device)
    if module_arithmetic:
        if expert_scale is not None:
            lg = lg * expert_scale
        if temperature != 1.0:
            lg = lg / temperature
        penalty = torch.finfo(torch.float32).min
    else:
        if temperature != 1.0:
            lg = lg / temperature
        if expert_scale is not None:
            lg = lg * expert_scale
        penalty = -1e9
    if expert_mask is not None:
        lg = lg + (1.0 - expert_mask) * penalty
    probs = F.softmax(lg, dim=-1)
    w = probs.gather(-1, r.topk_idx.long())
    w = w / (w.sum(dim=-1, keepdim=True) + renorm_eps)
    r.probs = r.probs + (probs - probs.detach())
    r.topk_w = r.topk_w + (w - w.detach())
    if r.logits is not None:
        r.logits = r.logits + (lg - lg.detach())
    return r


def _gate_tail(hidden: torch.Tensor, linear: nn.Linear, **kw) -> ops.RouterOut:
    """hidden [T,H'] (activation before the last Linear) -> fused router."""
    x = hidden.contiguous()
    w = linear.weight.detach().to(x.dtype).contiguous()
    b = None if linear.bias is None else linear.bias.detach().float()
    return ops.router_fused(x, w, b, **kw)


class BaseRouter(nn.Module):
    # The reference has a second copy of its routers (core/single/module/pikv_routing.py) whose
    # arithmetic differs in three places: * expert weights BEFORE / temperature (:596-600), mask
    # penalty finfo.min instead of -1e9 (:133-134), and + 1e-8 in the renormalisation (:143).
    # Set router.module_arithmetic = True to get that copy's numbers.
    module_arithmetic = False
    # Dense dispatch/combine tensors follow the token-major capacity rule.  legacy_fairscale = True
    # reproduces the vectorised fill of core/single/pikv_routing.py:102-128 instead (all tokens of
    # a round share a position); expert_backend != "fairscale" gives the [B,S,E,1] tensors of :133-153.
    legacy_fairscale = False

    def _arith_kw(self):
        return dict(module_arithmetic=True, renorm_eps=1e-8) if self.module_arithmetic else {}

    def __init__(self, hidden_size: int, num_experts: int, top_k: int = 2,
                 capacity_factor: float = 1.5, expert_backend: str = "fairscale"):
        super().__init__()
        self.hidden_size = hidden_size
        self.num_experts = num_experts
        self.top_k = min(top_k, num_experts)
        self.capacity_factor = capacity_factor
        self.expert_backend = expert_backend
        self.router = nn.Sequential(nn.Linear(hidden_size, hidden_size), nn.ReLU(),
                                    nn.Linear(hidden_size, num_experts))

    def _compute_capacity(self, batch_size: int, seq_len: int) -> int:
        return int(batch_size * seq_len * self.capacity_factor * self.top_k / self.num_experts)

    def _hidden_before_gate(self, seq: nn.Sequential, x2d: torch.Tensor) -> torch.Tensor:
        h = x2d
        for layer in list(seq)[:-1]:
            h = layer(h)
        return h

    def _route(self, hidden_states, expert_mask=None, *, seq=None, **scale_kw) -> ops.RouterOut:
        B, S, H = hidden_states.shape
        seq = self.router if seq is None else seq
        x2d = hidden_states.reshape(B * S, H)
        # ONE pass through the gate's hidden layers (one dropout mask, if any is active): the kernel gets
        # the activation's values, the torch tail - when gradients are wanted - continues from the same
        # tensor, so values and gradients belong to the same function
        grad = _wants_grad(hidden_states, *seq.parameters())
        with torch.set_grad_enabled(grad):
            h = self._hidden_before_gate(seq, x2d)
        cap = self._compute_capacity(B, S)
        r = _gate_tail(h.detach(), seq[-1], top_k=self.top_k, capacity=cap, expert_mask=expert_mask,
                       **self._arith_kw(), **scale_kw)
        if grad:
            r = _attach_grad(r, seq[-1](h), expert_mask=expert_mask, **self._arith_kw(), **scale_kw)
        return r

    def _aux_loss(self, router_probs: torch.Tensor) -> torch.Tensor:
        p = router_probs.mean(dim=[0, 1])
        return torch.sum(p * torch.log(p * self.num_experts + 1e-9))

    def _finish(self, r, B, S, return_compact):
        probs = r.probs.view(B, S, self.num_experts)
        if return_compact:
            return r, probs
        if self.expert_backend != "fairscale":
            return _dense_basic(r, B, S, self.num_experts), probs
        if self.legacy_fairscale:
            return _dense_legacy_fairscale(r, B, S, self.num_experts, r.capacity), probs
        disp, comb = _dense_dispatch_combine(r, B, S, self.num_experts, r.capacity)
        return (disp, comb), probs

    def forward(self, hidden_states: torch.Tensor, expert_mask: Optional[torch.Tensor] = None,
                return_compact: bool = False):
        B, S, _ = hidden_states.shape
        r = self._route(hidden_states, expert_mask)
        out, probs = self._finish(r, B, S, return_compact)
        aux = self._aux_loss(probs)
        if return_compact:
            return out, probs, aux
        return out[0], out[1], probs, aux


class TopKBalancedRouter(BaseRouter):
    def __init__(self, hidden_size, num_experts, top_k=2, capacity_factor=1.5,
                 expert_backend="fairscale", balance_coefficient=0.01, balance_mode="entropy"):
        super().__init__(hidden_size, num_experts, top_k, capacity_factor, expert_backend)
        self.balance_coefficient = balance_coefficient
        self.balance_mode = balance_mode

    def _balance(self, probs):
        p = probs.mean(dim=[0, 1])
        if self.balance_mode == "entropy":
            term = -torch.sum(p * torch.log(p + 1e-9)) / math.log(self.num_experts)
            return -self.balance_coefficient * term
        if self.balance_mode == "cv":
            return self.balance_coefficient * (p.std() / (p.mean() + 1e-9))
        uniform = torch.ones_like(p) / self.num_experts
        return self.balance_coefficient * torch.sum((p - uniform) ** 2)

    def forward(self, hidden_states, expert_mask=None, return_compact=False):
        res = super().forward(hidden_states, expert_mask, return_compact)
        probs = res[-2]
        aux = res[-1] + self._balance(probs)
        return (*res[:-1], aux)


class EPLBRouter(BaseRouter):
    def __init__(self, hidden_size, num_experts, top_k=2, capacity_factor=1.5,
                 expert_backend="fairscale", balance_coefficient=0.01, temperature=1.0,
                 use_auxiliary_loss=True, use_z_loss=True, z_loss_coefficient=1e-3):
        super().__init__(hidden_size, num_experts, top_k, capacity_factor, expert_backend)
        self.balance_coefficient = balance_coefficient
        self.temperature = temperature
        self.use_auxiliary_loss = use_auxiliary_loss
        self.use_z_loss = use_z_loss
        self.z_loss_coefficient = z_loss_coefficient
        self.global_step = 0
        self.router = nn.Sequential(nn.Linear(hidden_size, hidden_size * 2), nn.GELU(), nn.Dropout(0.1),
                                    nn.Linear(hidden_size * 2, hidden_size), nn.GELU(), nn.Dropout(0.1),
                                    nn.Linear(hidden_size, num_experts))
        self.register_buffer("expert_weights", torch.ones(num_experts))

    def _update_expert_weights(self, expert_usage):
        # core/single/pikv_routing.py:628-640 (the "momentum" there is the identity)
        self.expert_weights = expert_usage.mean() / (expert_usage + 1e-8)

    def forward(self, hidden_states, expert_mask=None, return_compact=False):
        B, S, _ = hidden_states.shape
        B_S = B * S
        # /temperature, then *expert_weights, then mask: the order of :653-660
        seq = self.router
        x2d = hidden_states.reshape(B_S, -1)
        # one pass through the hidden layers and their dropout: values (kernel) and gradients (torch tail)
        # come from the same activation, drawn with one mask
        grad = _wants_grad(hidden_states, *seq.parameters())
        with torch.set_grad_enabled(grad):
            h = self._hidden_before_gate(seq, x2d)
        cap = self._compute_capacity(B, S)
        hv = h.detach()
        r = ops.router_fused(hv.contiguous(), seq[-1].weight.detach().to(hv.dtype).contiguous(),
                             seq[-1].bias.detach().float(), top_k=self.top_k, capacity=cap,
                             expert_scale=self.expert_weights, expert_mask=expert_mask,
                             temperature=self.temperature, return_logits=True, **self._arith_kw())
        if grad:
            r = _attach_grad(r, seq[-1](h), temperature=self.temperature, expert_scale=self.expert_weights,
                             expert_mask=expert_mask, **self._arith_kw())
        out, probs = self._finish(r, B, S, return_compact)
        aux = torch.zeros((), device=probs.device)
        usage = r.count.float()
        if self.use_auxiliary_loss:
            u = usage / (B_S * self.top_k)
            kl = F.kl_div(torch.log(u + 1e-8), torch.full_like(u, 1.0 / self.num_experts), reduction="sum")
            aux = aux + self.balance_coefficient * kl
        if self.use_z_loss:
            aux = aux + self.z_loss_coefficient * torch.mean(torch.logsumexp(r.logits, dim=-1) ** 2)
        self._update_expert_weights(usage)
        self.global_step += 1
        if return_compact:
            return out, probs, aux
        return out[0], out[1], probs, aux


class AdaptiveRouter(BaseRouter):
    """core/single/pikv_routing.py:224-377: importance predictor + two gates."""

    def __init__(self, hidden_size, num_experts, top_k=2, capacity_factor=1.5,
                 expert_backend="fairscale", imp_threshold=0.5):
        super().__init__(hidden_size, num_experts, top_k, capacity_factor, expert_backend)
        self.importance_predictor = nn.Sequential(nn.Linear(hidden_size, hidden_size // 2), nn.ReLU(),
                                                  nn.Linear(hidden_size // 2, 1), nn.Sigmoid())
        self.imp_threshold = imp_threshold
        mk = lambda: nn.Sequential(nn.Linear(hidden_size, hidden_size), nn.ReLU(),
                                   nn.Linear(hidden_size, num_experts))
        self.router_important = mk()
        self.router_unimportant = mk()

    def _two_gate_route(self, hidden_states, importance, expert_mask, expert_scale=None):
        B, S, H = hidden_states.shape
        x2 = hidden_states.reshape(B * S, H)
        grad = _wants_grad(hidden_states, expert_scale, *self.router_important.parameters(),
                           *self.router_unimportant.parameters())
        with torch.set_grad_enabled(grad):      # both gates run once; the kernel takes their values
            la_t = self.router_important(x2).float()
            lb_t = self.router_unimportant(x2).float()
        la, lb = la_t.detach().contiguous(), lb_t.detach().contiguous()
        sel = (importance.reshape(-1) > self.imp_threshold)
        cap = self._compute_capacity(B, S)
        scale_v = None if expert_scale is None else expert_scale.detach()
        r = ops.router_tail(la, top_k=self.top_k, capacity=cap, logits_b=lb, select=sel,
                            expert_scale=scale_v, expert_mask=expert_mask, **self._arith_kw())
        if grad:
            # the per-token choice between the two gates (core/single/pikv_routing.py:450-458)
            lg = torch.where(sel.unsqueeze(1), la_t, lb_t)
            r = _attach_grad(r, lg, expert_scale=expert_scale, expert_mask=expert_mask, **self._arith_kw())
        return r


class PiKVRouter(AdaptiveRouter):
    def __init__(self, hidden_size, num_experts, top_k=2, capacity_factor=1.5,
                 expert_backend="fairscale", imp_threshold=0.5, cache_update_interval=100):
        super().__init__(hidden_size, num_experts, top_k, capacity_factor, expert_backend, imp_threshold)
        self.register_buffer("cache_usage_history", torch.zeros(num_experts))
        self.kv_importance_model = nn.Sequential(nn.Linear(hidden_size, hidden_size // 2), nn.ReLU(),
                                                 nn.Linear(hidden_size // 2, 1), nn.Sigmoid())
        self.cache_correction_factor = nn.Parameter(torch.ones(num_experts))
        self.register_buffer("update_counter", torch.tensor(0))
        self.cache_update_interval = cache_update_interval

    def update_cache_usage(self, usage_vector: torch.Tensor):
        self.cache_usage_history = 0.9 * self.cache_usage_history + 0.1 * usage_vector
        self.update_counter += 1
        if self.update_counter % self.cache_update_interval == 0:
            f = 1.0 / (self.cache_usage_history + 0.5)
            self.cache_correction_factor.data = f / f.mean()

    def forward(self, hidden_states, kv_states=None, expert_mask=None, return_compact=False):
        B, S, _ = hidden_states.shape
        importance = self.importance_predictor(hidden_states)
        if kv_states is not None:
            importance = (importance + self.kv_importance_model(kv_states)) / 2
        r = self._two_gate_route(hidden_states, importance.detach(), expert_mask,
                                 expert_scale=self.cache_correction_factor)
        out, probs = self._finish(r, B, S, return_compact)
        usage = probs.sum(dim=[0, 1])
        usage_norm = usage / usage.sum()
        self.update_cache_usage(usage_norm.detach())
        p = probs.mean(dim=[0, 1])
        aux = torch.sum(p * torch.log(p * self.num_experts + 1e-9))
        aux = aux + 0.05 * torch.sum(self.cache_usage_history * usage_norm)
        if return_compact:
            return out, probs, aux, importance
        return out[0], out[1], probs, aux, importance


class HierarchicalRouter(BaseRouter):
    """core/single/pikv_routing.py:737-860: router_probs[t, e] = softmax(group logits)[group of e]
    * softmax(logits of e's group router)[e], optionally times the expert mask; the k largest
    products are renormalised.  The two small softmaxes are torch; the top-k (ties to the lower
    expert index) and the capacity slots are the native tail on the products.  The reference
    writes every selected expert to slot 0 of its dense tensors (:838-846, marked "simplified");
    here the slots follow the token-major capacity rule like every other router."""

    def __init__(self, hidden_size: int, num_experts: int, top_k: int = 2, capacity_factor: float = 1.5,
                 expert_backend: str = "fairscale", num_groups: int = 4, group_top_k: int = 1):
        super().__init__(hidden_size, num_experts, top_k, capacity_factor, expert_backend)
        if num_experts % num_groups:
            raise ValueError("num_experts must be a multiple of num_groups")
        self.num_groups = num_groups
        self.group_top_k = group_top_k
        self.experts_per_group = num_experts // num_groups
        self.group_router = nn.Sequential(nn.Linear(hidden_size, hidden_size), nn.ReLU(),
                                          nn.Linear(hidden_size, num_groups))
        self.expert_routers = nn.ModuleList([
            nn.Sequential(nn.Linear(hidden_size, hidden_size // 2), nn.ReLU(),
                          nn.Linear(hidden_size // 2, self.experts_per_group))
            for _ in range(num_groups)])

    def router_probs(self, hidden_states: torch.Tensor, expert_mask: Optional[torch.Tensor] = None):
        group_probs = F.softmax(self.group_router(hidden_states), dim=-1)              # [B,S,G]
        parts = [group_probs[..., g:g + 1] * F.softmax(r(hidden_states), dim=-1)
                 for g, r in enumerate(self.expert_routers)]
        probs = torch.cat(parts, dim=-1)                                                 # [B,S,E]
        if expert_mask is not None:
            probs = probs * expert_mask.view(1, 1, -1)
        return probs

    def forward(self, hidden_states: torch.Tensor, expert_mask: Optional[torch.Tensor] = None,
                return_compact: bool = False):
        B, S, _ = hidden_states.shape
        probs = self.router_probs(hidden_states, expert_mask)
        flat = probs.detach().reshape(B * S, self.num_experts).float().contiguous()
        r = ops.router_tail(flat, top_k=self.top_k, capacity=self._compute_capacity(B, S), use_softmax=False)
        w = probs.reshape(B * S, self.num_experts).float().gather(-1, r.topk_idx.long())   # differentiable
        r.topk_w = w / w.sum(dim=-1, keepdim=True)
        r.probs = flat
        p = probs.mean(dim=[0, 1])
        aux = torch.sum(p * torch.log(p * self.num_experts + 1e-9))
        if return_compact:
            return r, probs, aux
        disp, comb = _dense_dispatch_combine(r, B, S, self.num_experts, r.capacity)
        return disp, comb, probs, aux
