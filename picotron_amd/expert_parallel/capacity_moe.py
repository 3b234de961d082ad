"""Capacity-capped, static-memory MoE dispatch on the GPU (single rank).

Same entry points as picotron/expert_parallel/capacity_moe.py: ``compute_capacity`` (:33-41),
``_slot_assignment`` (:44-57) and ``capacity_moe`` (:60-120).  Two modes: one capped round that drops the
overflow (``dropless=False``) or successive capped rounds that process everything (``dropless=True``).

Mechanism: a row's rank inside its expert comes out of the same stable counting sort that builds the
permutation, so the rows an expert keeps in a round are a prefix window of its sorted segment.  The kept
rows are laid out compactly, expert after expert, and the expert FFN runs on exactly those rows: the
zero-padded ``[num_experts*capacity, d]`` buffer of the reference (whose padding rows cost GEMM time and
yield zeros) is never materialised.  The per-token accumulation keeps the reference's rounding: within a
round the gate-weighted rows of a token are summed in fp32 and rounded once (what ``index_add`` into a zeroed
buffer does on the CPU), and the rounds are added one after another in the tensor dtype.
"""

import torch

from picotron_amd import _lib, _ops


def compute_capacity(num_tokens, top_k, num_experts, capacity_factor):
    """Per-expert row capacity for one round: ``capacity_factor * tokens*top_k/num_experts`` rounded up, min 1."""
    avg = (num_tokens * top_k) / num_experts
    return max(1, int(capacity_factor * avg + 0.999))


def _slot_assignment(expert_idx, num_experts):
    """(within int64 [N], counts int64 [E]): ``within[r]`` = number of earlier rows routed to row r's expert."""
    plan = _ops.permute_plan(expert_idx, num_experts, want_within=True)
    return plan.within.to(torch.int64), plan.counts


def _capped_rounds(src, div, expert_idx, weights_tk, num_tokens, top_k, num_experts, expert_fn, capacity, dropless, max_rounds):
    """Shared core: ``src`` holds one row per token (div = top_k) or one row per routed pick (div = 1)."""
    n_rows = expert_idx.numel()
    plan0 = _ops.permute_plan(expert_idx, num_experts, capacity=capacity, round_index=0)
    if dropless:
        need = int((int(plan0.counts.max().item()) + capacity - 1) // capacity) if num_experts else 1
        rounds = max(1, min(need, max_rounds))
    else:
        rounds = 1
    output = None
    for r in range(rounds):
        plan = plan0 if r == 0 else _ops.permute_plan(expert_idx, num_experts, capacity=capacity, round_index=r)
        x_sorted = _ops.expand_permute(src, plan.order, plan.inv_order, div, n_rows)
        y_sorted = expert_fn(x_sorted, plan.kept_counts)
        y = _ops.unpermute_combine(y_sorted, weights_tk, plan.inv_order, plan.order, num_tokens, top_k, zero_fill=True)
        output = y if output is None else output + y
    return output, plan0


def capacity_moe(
    routed, expert_idx, weights, token_idx, num_tokens, expert_dim, num_experts, num_local_experts, ep_world_size,
    group, expert_fn, capacity, dropless, max_rounds,
):
    """Run the routed experts under a per-expert capacity and sum the gate-weighted results per token.

    ``routed`` [N, expert_dim] holds one row per (token, pick) in token-major order (row ``t*top_k + j``;
    ``token_idx`` must be that expansion), ``expert_idx`` / ``weights`` [N] its expert and gate weight.
    ``expert_fn(x_grouped, counts)`` runs the experts on rows grouped by expert.  Single rank only.
    """
    if ep_world_size != 1:
        raise _lib.PicomoeError("capacity_moe: this build runs the single-rank (EP=1) path only")
    _lib.require_cuda(routed, expert_idx, weights)
    n_rows = routed.shape[0]
    if num_tokens == 0 or n_rows % num_tokens != 0:
        raise _lib.PicomoeError("capacity_moe: routed rows must be the token-major expansion (N = num_tokens * top_k)")
    top_k = n_rows // num_tokens
    out, _ = _capped_rounds(routed, 1, expert_idx, weights.reshape(num_tokens, top_k), num_tokens, top_k, num_experts,
                            expert_fn, capacity, dropless, max_rounds)
    return out
