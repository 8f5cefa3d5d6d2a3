"""Grouped top-k routing with a selection bias in plain tensor ops: a restatement of the selection rule of
python/sglang/srt/layers/moe/topk.py:665-738 that the tests hold the fused gate kernel against on the GPU (the numpy
oracle states the same rule for the CPU tests)."""
from typing import Optional, Tuple

import torch


def biased_grouped_topk_impl(
    hidden_states: torch.Tensor,
    gating_output: torch.Tensor,
    correction_bias: torch.Tensor,
    topk: int,
    renormalize: bool,
    num_expert_group: Optional[int] = None,
    topk_group: Optional[int] = None,
    routed_scaling_factor: Optional[float] = None,
    apply_routed_scaling_factor_on_output: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Same interface and selection rule as python/sglang/srt/layers/moe/topk.py:665-738: an expert's choice value
    is sigmoid(logit) + bias; a group is worth the sum of its two best choice values; only experts of the
    `topk_group` best groups compete for the `topk` places; the routing weights are the un-biased sigmoid values of
    the winners, normalised to sum 1 when `renormalize`."""
    tokens, experts = gating_output.shape
    assert hidden_states.shape[0] == tokens, "Number of tokens mismatch"
    per_group = experts // num_expert_group
    prob = torch.sigmoid(gating_output)
    choice = (prob + correction_bias).view(tokens, num_expert_group, per_group)
    group_worth = torch.topk(choice, 2, dim=2).values.sum(dim=2)                      # [tokens, groups]
    kept_groups = torch.topk(group_worth, topk_group, dim=1, sorted=False).indices     # [tokens, topk_group]
    group_open = torch.zeros((tokens, num_expert_group), dtype=torch.bool, device=choice.device)
    group_open.scatter_(1, kept_groups, True)
    candidates = torch.where(group_open.unsqueeze(2), choice, choice.new_full((), float("-inf"))).view(tokens, experts)
    winners = torch.topk(candidates, topk, dim=1, sorted=False).indices
    weights = torch.gather(prob, 1, winners)
    if renormalize:
        weights = weights / weights.sum(dim=1, keepdim=True)
        if apply_routed_scaling_factor_on_output:
            weights = weights * routed_scaling_factor
    return weights.float(), winners.int()


