"""Mixture-of-Experts layer for one MI355X (all experts local, EP = 1).

Drop-in for picotron/expert_parallel/expert_parallel.py: ``MoELayer`` (:38-439) keeps its constructor
knobs, attributes, parameter names and private helpers (``_route`` :168, ``_balance`` folded into the
router kernel, ``_expand_routed`` :214, ``_combine_topk`` :219, ``_moe_naive`` :271, ``_moe_capped`` :286,
``_grouped_experts`` :311, ``_run_local_experts`` :331) and ``collect_aux_loss`` (:442-454).

With one rank the dispatch / combine all-to-alls are local permutations, so the layer is:
router kernel -> stable counting-sort plan -> one gather (expand + permute) -> grouped SwiGLU GEMMs ->
one gather-sum (un-permute + gate-weighted combine).  The paths that exist only for several ranks
(``_dispatch_combine``, ``_moe_tiled``, ``_moe_deepep``) have no counterpart here.
Everything runs on the GPU through libpicomoe.so; CPU tensors are refused.
"""

import types

import torch
import torch.nn as nn

from picotron_amd import _lib, _ops
from picotron_amd.expert_parallel import megakernel
from picotron_amd.expert_parallel.capacity_moe import _capped_rounds, compute_capacity
from picotron_amd.model import MLP


def _argsort_inv(key, num_keys=None):
    """Stable argsort by small integer keys plus its inverse permutation (``x[order][inv_order] == x``)."""
    n = int(key.max().item()) + 1 if num_keys is None else num_keys
    plan = _ops.permute_plan(key, n)
    return plan.order.to(torch.int64), plan.inv_order.to(torch.int64)


_side_streams = {}


def _side_stream(device):
    """One extra stream per device (default priority), created on first use and shared by every layer: the layers of a
    model run one after the other, so their shared experts never compete for it."""
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    stream = _side_streams.get(key)
    if stream is None:
        stream = _side_streams[key] = torch.cuda.Stream(device=key)
    return stream


class _StackedWeights(torch.autograd.Function):
    """Presents E per-expert parameters as one [E, ...] tensor without copying: ``stack`` already shares
    storage with them.  Backward hands each parameter its slice of the stacked gradient."""

    @staticmethod
    def forward(ctx, stack, *params):
        return stack.view_as(stack)

    @staticmethod
    def backward(ctx, grad):
        return (None, *grad.unbind(0))


class MoELayer(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.hidden_size = config.hidden_size
        self.num_experts = config.num_experts
        self.top_k = config.num_experts_per_tok
        self.norm_topk_prob = getattr(config, "norm_topk_prob", True)

        # one GPU: every expert is local
        self.ep_world_size = 1
        self.ep_rank = 0
        self.num_local_experts = self.num_experts

        self.latent_dim = getattr(config, "moe_latent_dim", 0)
        self.latent = 0 < self.latent_dim < self.hidden_size
        self.expert_dim = self.latent_dim if self.latent else self.hidden_size

        self.gate = nn.Linear(config.hidden_size, self.num_experts, bias=False)
        if self.latent:
            self.down_proj_latent = nn.Linear(self.hidden_size, self.latent_dim, bias=False)
            self.up_proj_latent = nn.Linear(self.latent_dim, self.hidden_size, bias=False)
        expert_config = types.SimpleNamespace(hidden_size=self.expert_dim, intermediate_size=config.intermediate_size)
        self.local_experts = nn.ModuleList([MLP(expert_config) for _ in range(self.num_local_experts)])
        self.num_shared_experts = getattr(config, "num_shared_experts", 0)
        if self.num_shared_experts > 0:
            shared_config = types.SimpleNamespace(
                hidden_size=self.hidden_size, intermediate_size=config.intermediate_size * self.num_shared_experts
            )
            self.shared_expert = MLP(shared_config)
        else:
            self.shared_expert = None

        # ep_overlap: the shared expert runs on a second stream beside the routed path (see _shared_start); the other
        # knobs of the multi-rank paths are kept as attributes (callers set them) but have no effect here
        self.ep_overlap = getattr(config, "ep_overlap", True)
        self.ep_num_tiles = getattr(config, "ep_num_tiles", 1)
        self.ep_backend = getattr(config, "ep_backend", "torch")
        self.ep_fp8_dispatch = getattr(config, "ep_fp8_dispatch", False)
        # not in the reference: with the FP8 dispatch on, feed the forward gate/up GEMM with the E4M3 codes on FP8 MFMA
        # (weights quantised per output row) instead of the dequantised rows on bf16 MFMA; "all" also runs the forward
        # down GEMM on FP8 MFMA (SwiGLU output quantised per row).  The backward is bf16 either way.
        self.ep_fp8_gemm = getattr(config, "ep_fp8_gemm", False)
        self._fp8_weights = None

        self.ep_capacity_factor = getattr(config, "ep_capacity_factor", 0.0)
        self.ep_capacity_dropless = getattr(config, "ep_capacity_dropless", True)
        self.ep_max_rounds = getattr(config, "ep_max_rounds", 8)

        self.router_aux_loss_coef = getattr(config, "router_aux_loss_coef", 0.0)
        self.router_bias_update_rate = getattr(config, "router_bias_update_rate", 0.0)
        self.use_loss_free = self.router_bias_update_rate > 0
        self.register_buffer("expert_bias", torch.zeros(self.num_experts), persistent=True)
        self.aux_loss = None

        self._stacks = None  # [E,I,H], [E,I,H], [E,H,I] buffers the per-expert parameters are views of
        self.reset_parameters()

    def reset_parameters(self):
        self.gate.reset_parameters()
        if self.latent:
            self.down_proj_latent.reset_parameters()
            self.up_proj_latent.reset_parameters()
        for expert in self.local_experts:
            expert.reset_parameters()
        if self.shared_expert is not None:
            self.shared_expert.reset_parameters()

    # ---- expert weights as stacked tensors ------------------------------------------------------
    def _expert_params(self):
        ex = self.local_experts
        return ([e.gate_proj.weight for e in ex], [e.up_proj.weight for e in ex], [e.down_proj.weight for e in ex])

    def _stacked_weights(self):
        """(gate_w [E,I,H], up_w [E,I,H], down_w [E,H,I]) sharing storage with the per-expert parameters.

        The first call (and any call after the parameters were moved, cast or re-assigned) copies the
        weights once into three contiguous buffers and re-points every ``local_experts[i].*_proj.weight``
        at its slice; afterwards optimizer steps and ``load_state_dict`` update the buffers in place and
        no per-forward ``stack`` is needed."""
        groups = self._expert_params()
        p0 = groups[0][0]
        ok = self._stacks is not None and all(s.dtype == p0.dtype and s.device == p0.device for s in self._stacks)
        if ok:
            for stack, params in zip(self._stacks, groups):
                step = stack.stride(0) * stack.element_size()
                base = stack.data_ptr()
                if any(p.data_ptr() != base + i * step or p.shape != stack.shape[1:] for i, p in enumerate(params)):
                    ok = False
                    break
        if not ok:
            with torch.no_grad():
                stacks = []
                for params in groups:
                    stack = torch.stack([p.detach() for p in params]).contiguous()
                    for i, p in enumerate(params):
                        p.data = stack[i]
                    stacks.append(stack)
                self._stacks = tuple(stacks)
        return tuple(_StackedWeights.apply(stack, *params) for stack, params in zip(self._stacks, groups))

    # ---- forward ----------------------------------------------------------------------------------
    def forward(self, x):
        batch_size, seq_length, _ = x.shape
        tokens = x.reshape(-1, self.hidden_size)
        tokens, router_logits = self._gate(tokens)
        topk_idx, topk_weights = self._route(tokens, router_logits)
        if self.ep_capacity_factor > 0:
            expert_out = self._moe_capped(tokens, topk_idx, topk_weights)
        else:
            expert_out = self._moe_naive(tokens, topk_idx, topk_weights)
        return expert_out.view(batch_size, seq_length, self.hidden_size)

    def _gate(self, tokens):
        """(tokens, router logits).  With a gate the fused kernel takes (no bias, at most 16 experts, no module hooks to
        honour) and a token gradient to carry, the tokens come back as the second output of the gate's autograd node, so that
        their whole gradient -- through the router and through everything else that reads them -- is written by one kernel."""
        gate = self.gate
        fused = (gate.bias is None and torch.is_grad_enabled() and tokens.requires_grad
                 and _ops.gate_dgrad_supported(tokens, gate.weight)
                 and not (gate._forward_hooks or gate._forward_pre_hooks or gate._backward_hooks or gate._backward_pre_hooks))
        if not fused:
            return tokens, gate(tokens)
        router_logits, tokens = _ops.gate_tap(tokens.contiguous(), gate.weight)
        return tokens, router_logits

    def _route(self, tokens, router_logits=None):
        """Router: top-k expert selection + gate weights; stashes the aux loss and steps the loss-free bias
        (training only), all inside the router kernels."""
        _lib.require_cuda(tokens)
        if router_logits is None:
            router_logits = self.gate(tokens)
        balance = self.training and (self.router_aux_loss_coef > 0 or self.use_loss_free)
        # fp32 view or copy of the bias: the router kernel reads it for the selection, the balance kernel that
        # follows on the same stream steps it in place
        bias_f32 = self.expert_bias.float() if self.use_loss_free else None
        topk_idx, topk_weights, aux = _ops.route(
            router_logits, bias_f32, self.top_k, self.norm_topk_prob, balance,
            self.router_aux_loss_coef if balance else 0.0, self.router_bias_update_rate if (balance and self.use_loss_free) else 0.0,
        )
        self.aux_loss = aux if (balance and self.router_aux_loss_coef > 0) else None
        if balance and self.use_loss_free:
            with torch.no_grad():
                self.expert_bias.copy_(bias_f32)
        return topk_idx, topk_weights.to(tokens.dtype)  # the reference's cast (expert_parallel.py:184)

    def _expand_routed(self, tokens, topk_idx, topk_weights):
        """One routed row per (token, selected expert), token-major."""
        n = tokens.shape[0] * self.top_k
        return _ops.expand_permute(tokens, None, None, self.top_k, n), topk_idx.reshape(-1), topk_weights.reshape(-1)

    def _combine_topk(self, y, weights, num_tokens):
        """Weight each routed row by its gate weight and sum a token's top-k rows."""
        return _ops.unpermute_combine(y, weights.reshape(num_tokens, self.top_k), None, None, num_tokens, self.top_k)

    def _maybe_down(self, tokens):
        return self.down_proj_latent(tokens) if self.latent else tokens

    def _shared_start(self, tokens):
        """Starts the shared expert.  With ``ep_overlap`` it is enqueued on a second HIP stream (default priority), so its
        kernels run beside the routed path's: at small batches neither the shared expert's launches (one expert: few
        tiles) nor the routed ones fill the 256 CUs alone.  The reference overlaps the shared expert with the dispatch
        exchange the same way (expert_parallel.py:230-248); autograd replays each backward op on the stream its forward
        ran on, so the backward overlaps too."""
        if self.shared_expert is None:
            return None, None
        if not (self.ep_overlap and tokens.is_cuda and self._launches_leave_cus_idle(tokens.shape[0])):
            return self.shared_expert(tokens), None
        main = torch.cuda.current_stream(tokens.device)
        side = _side_stream(tokens.device)
        side.wait_stream(main)                   # tokens are ready once the work already queued on this stream is done
        with torch.cuda.stream(side):
            out = self.shared_expert(tokens)
        tokens.record_stream(side)               # the allocator must not hand tokens' memory out before the side stream is done
        return out, side

    def _launches_leave_cus_idle(self, num_tokens):
        """Whether a second stream can pay: the routed gate/up launch has fewer than four rounds of 256 x 256 tiles for the
        256 CUs, so its last round (and every launch of the one-expert shared FFN) leaves a good part of them without a
        tile.  Measured: a 2048-token train step of 8 experts gains 4-5 %; at 16384 tokens x 64 experts the step time is
        the same with and without, and the kernels of the two streams only stretch each other."""
        inter = self.local_experts[0].gate_proj.weight.shape[0]
        row_tiles = (num_tokens * self.top_k) // 256 + self.num_local_experts
        return row_tiles * ((inter + 127) // 128) < 4 * 256

    def _finalize(self, y_expert, shared):
        y = self.up_proj_latent(y_expert) if self.latent else y_expert
        shared_out, side = shared
        if shared_out is None:
            return y
        if side is not None:
            main = torch.cuda.current_stream(y.device)
            main.wait_stream(side)
            shared_out.record_stream(main)
        return y + shared_out

    def _moe_naive(self, tokens, topk_idx, topk_weights):
        _lib.require_cuda(tokens, topk_idx, topk_weights)
        num_tokens = tokens.shape[0]
        shared = self._shared_start(tokens)
        latent = self._maybe_down(tokens)
        n_rows = num_tokens * self.top_k
        plan = _ops.permute_plan(topk_idx.reshape(-1), self.num_local_experts)
        codes = None
        if self.ep_fp8_dispatch:
            # One pass over the tokens: quantise -> dequantise (one per token equals one per routed row, a row op on
            # identical rows) written straight to the rows' sorted positions, with the codes beside them for the FP8 GEMM
            x_sorted, q_sorted, scale_sorted = _ops.dispatch_fp8(latent, plan.inv_order, self.top_k, n_rows,
                                                                 with_codes=self._use_fp8_gemm(latent))
            if q_sorted is not None:
                codes = (q_sorted, scale_sorted)
        else:
            x_sorted = _ops.expand_permute(latent, plan.order, plan.inv_order, self.top_k, n_rows)
        y_sorted = self._grouped_experts(x_sorted, plan.counts, codes)
        y = _ops.unpermute_combine(y_sorted, topk_weights, plan.inv_order, plan.order, num_tokens, self.top_k)
        return self._finalize(y, shared)

    def _moe_capped(self, tokens, topk_idx, topk_weights):
        """MoE under a fixed per-expert capacity: one round with drops, or dropless rounds (see capacity_moe.py)."""
        _lib.require_cuda(tokens, topk_idx, topk_weights)
        num_tokens = tokens.shape[0]
        shared = self._shared_start(tokens)
        latent = self._maybe_down(tokens)
        capacity = compute_capacity(num_tokens, self.top_k, self.num_experts, self.ep_capacity_factor)
        y, _ = _capped_rounds(
            latent, self.top_k, topk_idx.reshape(-1), topk_weights, num_tokens, self.top_k, self.num_experts,
            self._grouped_experts, capacity, self.ep_capacity_dropless, self.ep_max_rounds,
        )
        return self._finalize(y, shared)

    def _use_fp8_gemm(self, x):
        return (self.ep_fp8_gemm and x.dtype == torch.bfloat16 and x.shape[0] > 0
                and megakernel.fp8_gemm_supported(self.expert_dim, self.local_experts[0].gate_proj.weight.shape[0]))

    def _quantized_weights(self):
        """E4M3 codes + per-row scales of the stacked gate / up (and, with ``ep_fp8_gemm == "all"``, down) weights, kept
        until a parameter's version counter moves: an optimizer step updates the parameters in place and so moves
        them, the micro-batches of a gradient-accumulation step in between reuse the codes.  After a write that
        bypasses the counters (``p.data``) call ``invalidate_fp8_weights``."""
        gates, ups, downs = self._expert_params()
        with_down = self.ep_fp8_gemm == "all"
        params = gates + ups + (downs if with_down else [])
        key = (with_down, self._stacks[0].data_ptr(), self._stacks[1].data_ptr(), self._stacks[2].data_ptr(),
               tuple(p._version for p in params))
        if self._fp8_weights is None or self._fp8_weights[0] != key:
            with torch.no_grad():
                quantized = megakernel.quantize_expert_weights(self._stacks[0]) + megakernel.quantize_expert_weights(self._stacks[1])
                if with_down:
                    quantized += megakernel.quantize_expert_weights(self._stacks[2])
            self._fp8_weights = (key, quantized)
        return self._fp8_weights[1]

    def invalidate_fp8_weights(self):
        self._fp8_weights = None

    def _grouped_experts(self, x_sorted, counts, codes=None):
        """Run the local experts on rows already grouped by expert; ``counts[e]`` rows go to expert ``e``.
        ``codes`` (optional): ``(E4M3 codes [N,H] uint8, scale [N])`` of the same rows for the FP8 gate/up GEMM."""
        if x_sorted.shape[0] == 0:
            return x_sorted
        _lib.require_cuda(x_sorted)
        gate_w, up_w, down_w = self._stacked_weights()
        fp8 = None
        if codes is not None:
            fp8 = (codes[0], codes[1]) + self._quantized_weights()
        return megakernel.fused_moe(x_sorted, counts, gate_w, up_w, down_w, fp8=fp8)

    def _run_local_experts(self, x, local_expert_idx):
        """Run the local experts on ``x`` given each row's expert id, preserving the input order."""
        if x.shape[0] == 0:
            return x
        n = x.shape[0]
        plan = _ops.permute_plan(local_expert_idx, self.num_local_experts)
        x_sorted = _ops.expand_permute(x, plan.order, plan.inv_order, 1, n)
        y_sorted = self._grouped_experts(x_sorted, plan.counts)
        return _ops.unpermute_combine(y_sorted, None, plan.inv_order, plan.order, n, 1)


def collect_aux_loss(model):
    """Sum and drain the aux loss stashed on every ``MoELayer`` by its last forward (``None`` if there is none)."""
    total = None
    for module in model.modules():
        if isinstance(module, MoELayer) and module.aux_loss is not None:
            total = module.aux_loss if total is None else total + module.aux_loss
            module.aux_loss = None
    return total
