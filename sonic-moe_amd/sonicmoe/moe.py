"""`MoE` module: drop-in for the reference module (constructor, parameter names/shapes and forward signature of
sonicmoe/moe.py:58-257).

    router.weight (E, H)   c_fc.weight (E, 2I, H) [gate rows even, up rows odd]   c_proj.weight (E, H, I)

kernel_backend_moe = sonicmoe runs the HIP kernels; kernel_backend_moe = torch is the plain-PyTorch evaluation of the
same layer (runs on CPU or GPU) that the reference uses as its own parity target.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .count_cumsum import count_cumsum
from .enums import ActivationType, KernelBackendMoE, is_glu
from .functional import moe_TC_softmax_topk_layer, switch_loss


def _split_gate_up(h: torch.Tensor):
    return h[..., ::2], h[..., 1::2]


def _apply_activation(h: torch.Tensor, kind: ActivationType) -> torch.Tensor:
    if kind == ActivationType.SWIGLU:
        g, u = _split_gate_up(h)
        return F.silu(g) * u
    if kind == ActivationType.GEGLU:
        g, u = _split_gate_up(h)
        return (F.gelu(g.float()) * u).to(g.dtype)
    if kind == ActivationType.REGLU:
        g, u = _split_gate_up(h)
        return (F.relu(g) * u).to(g.dtype)
    if kind == ActivationType.GELU:
        return F.gelu(h.float()).to(h.dtype)
    if kind == ActivationType.RELU:
        return F.relu(h)
    if kind == ActivationType.RELU_SQ:
        return F.relu(h) ** 2
    if kind == ActivationType.SILU:
        return F.silu(h)
    raise ValueError(f"unknown activation {kind}")


class Experts(nn.Module):
    """E stacked linear maps: weight (E, out_features, in_features), optional bias (E, out_features)."""

    def __init__(
        self, num_experts: int, in_features: int, out_features: int, add_bias: bool = True, std: float | None = None
    ) -> None:
        super().__init__()
        self.num_experts, self.in_features, self.out_features = num_experts, in_features, out_features
        self.std = std
        self.weight = nn.Parameter(torch.empty(num_experts, out_features, in_features))
        self.bias = nn.Parameter(torch.empty(num_experts, out_features)) if add_bias else None
        self.reset_parameters()

    @torch.no_grad()
    def reset_parameters(self) -> None:
        nn.init.normal_(self.weight, mean=0, std=self.std)
        if self.bias is not None:
            self.bias.zero_()

    def torch_forward(self, chunks: list[torch.Tensor]) -> list[torch.Tensor]:
        """chunks[e] (n_e, in) -> (n_e, out) with expert e's map."""
        weights = self.weight.unbind(0)  # one autograd node for all experts' weight gradients
        biases = [None] * self.num_experts if self.bias is None else self.bias.unbind(0)
        return [F.linear(c, w, b) for c, w, b in zip(chunks, weights, biases)]

    def extra_repr(self) -> str:
        return f"num_experts={self.num_experts}, in_features={self.in_features}, out_features={self.out_features}"


class MoE(nn.Module):
    def __init__(
        self,
        num_experts: int,
        num_experts_per_tok: int,
        hidden_size: int,
        intermediate_size: int,
        activation_function: ActivationType,
        add_bias: bool,
        std: float,
    ) -> None:
        super().__init__()
        self.num_experts = num_experts
        self.top_k = num_experts_per_tok
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.activation_function = activation_function

        self.router = nn.Linear(in_features=hidden_size, out_features=num_experts, bias=False)
        up_out = 2 * intermediate_size if is_glu(activation_function) else intermediate_size
        self.c_fc = Experts(num_experts, hidden_size, up_out, add_bias=add_bias, std=std)
        self.c_proj = Experts(num_experts, intermediate_size, hidden_size, add_bias=add_bias, std=std)

        # the stream the expert kernels are launched on; 0 (the default stream) when built without a GPU
        self.stream_id = torch.cuda.current_stream().cuda_stream if torch.cuda.is_available() else 0

    def forward(
        self,
        hidden_states: torch.Tensor,
        kernel_backend_moe: KernelBackendMoE = KernelBackendMoE.sonicmoe,
        is_inference_mode: bool = False,
    ) -> tuple[torch.Tensor, torch.Tensor]:
        shape = hidden_states.shape
        x = hidden_states.view(-1, self.hidden_size)

        if kernel_backend_moe == KernelBackendMoE.sonicmoe:
            out, router_logits, expert_frequency = moe_TC_softmax_topk_layer(
                x,
                self.router.weight,
                self.c_fc.weight.permute(1, 2, 0),
                self.c_fc.bias,
                self.c_proj.weight.permute(1, 2, 0),
                self.c_proj.bias,
                self.top_k,
                self.stream_id,
                self.activation_function,
                is_inference_mode or not self.training,
            )
        elif kernel_backend_moe == KernelBackendMoE.torch:
            router_logits, gates, selected = self._compute_routing_weights(x)
            out, expert_frequency = self._compute_experts(x, gates, selected, kernel_backend_moe)
        elif kernel_backend_moe == KernelBackendMoE.scattermoe:
            raise NotImplementedError("the scattermoe backend is an external comparison backend and is not provided")
        else:
            raise ValueError(f"unexpected kernel_backend_moe ({kernel_backend_moe})")

        out = out.view(shape)
        if kernel_backend_moe == KernelBackendMoE.sonicmoe:
            # same value as _compute_switch_loss below, one pass over the logits instead of six torch kernels
            aux_loss = switch_loss(router_logits, expert_frequency)
        else:
            aux_loss = self._compute_switch_loss(
                logits=router_logits,
                probs=F.softmax(router_logits, dim=-1, dtype=torch.float32),
                expert_frequency=expert_frequency,
            )
        return out, aux_loss

    def _compute_switch_loss(
        self, logits: torch.Tensor, probs: torch.Tensor, expert_frequency: torch.Tensor
    ) -> torch.Tensor:
        """E * <normalised mean router probability, normalised expert load>."""
        probs = probs.view(-1, probs.size(-1))
        p = F.normalize(probs.sum(0), p=1, dim=0)
        f = F.normalize(expert_frequency.float(), p=1, dim=0)
        return probs.size(-1) * (p * f).sum()

    def _get_topk(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        if self.top_k == 1:
            return x.max(dim=-1, keepdim=True)
        return x.topk(self.top_k, dim=-1)

    def _compute_routing_weights(self, x: torch.Tensor):
        router_logits = self.router(x)
        top_logits, selected = self._get_topk(router_logits)
        gates = F.softmax(top_logits.float(), dim=-1).type_as(x)
        return router_logits, gates, selected

    def _compute_experts(self, x, gates, selected, kernel_backend_moe):
        """Plain-PyTorch expert evaluation: sort the routed pairs by expert, run each expert on its slice,
        scale by the gate and scatter-add into an fp32 (T, H) buffer."""
        if kernel_backend_moe != KernelBackendMoE.torch:
            raise ValueError(f"unexpected kernel_backend_moe ({kernel_backend_moe})")
        T = x.size(0)
        flat = selected.flatten()
        with torch.no_grad():
            _, order = flat.sort()
        if flat.is_cuda and self.num_experts % 4 == 0:
            expert_frequency, _ = count_cumsum(flat, self.num_experts, do_cumsum=True)
        else:
            expert_frequency = flat.bincount(minlength=self.num_experts).to(torch.int32)
        token_of_row = order // self.top_k
        gate_of_row = gates.flatten()[order]
        chunks = list(x[token_of_row].split(expert_frequency.tolist(), dim=0))
        hidden = [_apply_activation(h, self.activation_function) for h in self.c_fc.torch_forward(chunks)]
        y = torch.cat(self.c_proj.torch_forward(hidden), dim=0) * gate_of_row.unsqueeze(-1)
        out = torch.zeros((T, self.hidden_size), dtype=torch.float32, device=x.device).index_add(0, token_of_row, y)
        return out, expert_frequency
