"""MoE layer with the constructor, parameters, buffers and forward signature of
the reference (xma/layers/moe/__init__.py:22-262) and a ``KernelBackend.rocm``
branch that runs on the gfx950 kernels of libxma_rocm.so."""

from __future__ import annotations

from typing import Callable

import torch
import torch.nn as nn
import torch.nn.functional as F

from ...accelerator import Accelerator, KernelBackend
from ...functional import continuous_count


class Experts(nn.Module):
    """E stacked linear layers: weight (E, out, in), optional bias (E, out), uint32 buffers N_array / K_array
    (reference: moe/__init__.py:22-43, 112-119)."""

    def __init__(
        self, num_experts: int, in_features: int, out_features: int, add_bias: bool = True, std: float | None = None
    ) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.in_features = in_features
        self.out_features = out_features
        self.std = std

        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features))
        self.bias = nn.Parameter(torch.empty(num_experts, out_features)) if add_bias else None

        self.register_buffer("N_array", torch.empty((num_experts,), dtype=torch.uint32))
        self.register_buffer("K_array", torch.empty((num_experts,), dtype=torch.uint32))

        self.reset_parameters()

    def torch_forward(
        self, x: torch.Tensor | list[torch.Tensor], expert_frequency: torch.Tensor | None, return_list: bool = False
    ) -> list[torch.Tensor] | torch.Tensor:
        """one F.linear per expert over the expert-sorted rows (reference: moe/__init__.py:89-105)"""
        if isinstance(x, torch.Tensor):
            x = x.split(expert_frequency.tolist(), dim=0)
        else:
            assert expert_frequency is None
        x = [F.linear(x[e], self.weight[e], None if self.bias is None else self.bias[e]) for e in range(self.num_experts)]
        return x if return_list else torch.cat(x, dim=0)

    def extra_repr(self) -> str:
        return f"num_experts={self.num_experts}, in_features={self.in_features}, out_features={self.out_features}"

    @torch.no_grad()
    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0, std=self.std)
        if self.bias is not None:
            self.bias.zero_()
        self.N_array.fill_(self.out_features)
        self.K_array.fill_(self.in_features)


class MoE(nn.Module):
    def __init__(
        self,
        num_experts: int,
        num_experts_per_tok: int,
        hidden_size: int,
        intermediate_size: int,
        activation_function: Callable,
        is_glu: bool,
        add_bias: bool,
        std: float,
    ) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.top_k = num_experts_per_tok
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.is_glu = is_glu
        # rocm backend with the fused SwiGLU path only (not a constructor argument: the signature is the reference's).
        # False: keep x and the pre-activations between forward and backward and recompute the activations and the expert
        # outputs in the backward, as the reference's backward does (triton_implementation/__init__.py:117-128).
        self.save_activations = True

        self.gate = nn.Linear(in_features=hidden_size, out_features=num_experts, bias=False)
        self.c_fc = Experts(
            num_experts=num_experts,
            in_features=hidden_size,
            out_features=2 * intermediate_size if is_glu else intermediate_size,
            add_bias=add_bias,
            std=std,
        )
        self.act = activation_function
        self.c_proj = Experts(
            num_experts=num_experts, in_features=intermediate_size, out_features=hidden_size, add_bias=add_bias, std=std
        )

    def forward(self, x: torch.Tensor, *, kernel_backend: KernelBackend | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        original_shape = x.shape
        x = x.view(-1, self.hidden_size)
        router_logits, router_weights, selected_experts = self._compute_routing_weights(x, kernel_backend=kernel_backend)
        x = self._compute_experts(x, router_weights, selected_experts, kernel_backend=kernel_backend)
        return x.view(original_shape), router_logits

    def _compute_routing_weights(
        self, x: torch.Tensor, *, kernel_backend: KernelBackend | None = None
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        # (T, H) -> logits (T, E), weights (T, k) = fp32 softmax over the k selected logits, experts (T, k)
        if kernel_backend is None:
            kernel_backend = Accelerator.get_kernel_backend()
        if kernel_backend == KernelBackend.rocm and x.is_cuda:
            from . import rocm_implementation as R

            # equal logits go to the lower expert index
            if self.gate.bias is None and R.router_gate_topk_supported(x, self.gate.weight, self.top_k):
                # gate GEMM, top-k, softmax, cast and int32 expert ids in one kernel: x is read once
                return R.router_gate_topk(x, self.gate.weight, self.top_k)
            router_logits = self.gate(x)
            router_weights, selected_experts = R.router_topk(router_logits, self.top_k)
            return router_logits, router_weights, selected_experts
        router_logits = self.gate(x)
        router_weights, selected_experts = self._get_topk(router_logits)
        router_weights = F.softmax(router_weights.float(), dim=-1).type_as(x)
        return router_logits, router_weights, selected_experts

    def _compute_experts(
        self,
        x: torch.Tensor,
        router_weights: torch.Tensor,
        selected_experts: torch.Tensor,
        *,
        kernel_backend: KernelBackend | None = None,
    ) -> torch.Tensor:
        if kernel_backend is None:
            kernel_backend = Accelerator.get_kernel_backend()
        else:
            assert kernel_backend.verify_accelerator()

        T = x.size(0)

        if kernel_backend == KernelBackend.rocm:
            from . import rocm_implementation as R

            _, expert_offsets, _, sorted_expert_idxs, sorted_scattered_idxs = R.route(selected_experts, self.num_experts)
            x = x.contiguous()
            w_fc, w_proj = self.c_fc.weight.permute(0, 2, 1), self.c_proj.weight.permute(0, 2, 1)
            # the experts' biases (the reference applies them on its torch path only, :96-100; its Triton path asserts
            # that there are none, :53 and :75) enter the grouped GEMMs as the first term of their fp32 sums
            b_fc, b_proj = self.c_fc.bias, self.c_proj.bias

            if self.is_glu and getattr(self.act, "_xma_fused_activation", None) == "swiglu_packed":
                x = R.fused_swiglu_experts(x, w_fc, w_proj, router_weights, sorted_scattered_idxs, expert_offsets, b_fc,
                                           b_proj, self.save_activations)
            else:
                x = R.up_projection_experts(x, w_fc, self.top_k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets,
                                            b_fc)
                x = self.act(x)
                x = R.down_projection_experts(
                    x.contiguous(), w_proj, 1, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, router_weights,
                    b_proj
                )
        elif kernel_backend == KernelBackend.torch:
            # the reference's torch path (moe/__init__.py:210-211, 235-250)
            sorted_expert_idxs, sorted_scattered_idxs = selected_experts.flatten().sort(stable=True)
            expert_frequency = continuous_count(sorted_expert_idxs, self.num_experts, kernel_backend=KernelBackend.torch)

            fan_in_index = sorted_scattered_idxs // self.top_k
            batch_gates = router_weights.flatten()[sorted_scattered_idxs]

            x = x[fan_in_index]
            x = self.c_fc.torch_forward(x=x, expert_frequency=expert_frequency, return_list=True)
            x = [self.act(i) for i in x]
            x = self.c_proj.torch_forward(x=x, expert_frequency=None, return_list=False)

            x = x * batch_gates.unsqueeze(-1)
            zeros = torch.zeros((T, self.hidden_size), dtype=x.dtype, device=x.device)
            x = zeros.index_add(0, fan_in_index, x)
        else:
            raise ValueError(f"unexpected kernel_backend ({kernel_backend})")

        return x

    def _get_topk(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        if self.top_k == 1:
            return x.max(dim=-1, keepdim=True)
        return x.topk(self.top_k, dim=-1)
