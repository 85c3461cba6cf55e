"""The expert module of the alltoall dispatcher on MI355X: ``GmmExpertsImpl`` and a self-contained ``GroupedMLP``.

``GmmExpertsImpl`` mirrors mindspeed/core/transformer/moe/moe_feature/gmm/experts.py:14-193: the mix-in that
MindSpeed puts in front of Megatron's ``GroupedMLP``.  Same constructor ``(num_local_experts, config)``, same
``forward(permuted_local_hidden_states, tokens_per_expert, permuted_probs=None) -> (output, None)``:

* flat parameters ``weight1 [hidden, E * 2 * ffn]`` and ``weight2 [E * ffn, hidden]`` viewed per expert at use
  (``weight1.view(E, hidden, -1)``, ``weight2.view(E, -1, hidden)``, experts.py:90-91);
* ``gg.ops.gmm(x, w, tokens_per_expert, trans_b=False, gemm_fusion=..., original_weight=...)`` for both matmuls
  (experts.py:113-120,146-153) with ``activation_func_with_probs`` between them (experts.py:41-44,121-127);
* the ``CheckpointWithoutOutput`` switch for activation recomputation (experts.py:121-127,183-191);
* with no tokens on the rank, plain matmuls on the flat weights so that the parameters still get (zero) gradients
  (experts.py:154-181).

Where nothing asks for the op-by-op sequence (no ``gemm_gradient_accumulation_fusion``, 16-bit vector-access
operands, SiLU gate) the whole body is one autograd node, ``ops.grouped_mlp``, whose values are those of the separate
kernels bit for bit; ``config.moe_fuse_expert_mlp = False`` keeps the reference's sequence.  The quantised branches
of the reference (``qat_scheme``, fp8 grouped matmuls) are outside this path and raise.

``GroupedMLP`` supplies what Megatron's class of that name gives the mix-in (the two flat parameters and
``activation_func``), so the module can be built without Megatron: ``GroupedMLP(num_local_experts, config)`` with
``config.hidden_size``, ``config.moe_ffn_hidden_size`` (or ``ffn_hidden_size``), ``config.gated_linear_unit``,
``config.activation_func``, ``config.params_dtype`` and optionally ``config.init_method``.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import fusions
from .ops import fused_swiglu, grouped_mlp, swiglu_with_probs
from .recompute import CheckpointWithoutOutput

__all__ = ["GmmExpertsImpl", "GroupedMLP", "should_recompute_activation"]


def should_recompute_activation(config, layer_number):
    """mindspeed/model/transformer.py:142-159 without the pipeline-bubble schedules: recompute when
    ``recompute_activation_function`` is set, the module knows its layer number, and the layer lies within
    ``recompute_activation_function_num_layers`` (all layers when that is None)."""
    if not getattr(config, "recompute_activation_function", False) or layer_number is None:
        return False
    limit = getattr(config, "recompute_activation_function_num_layers", None)
    if limit is None:
        return True
    if limit < 0:
        raise AssertionError("--recompute-activation-function-num-layers cannot be less than 0.")
    return layer_number <= limit


class GmmExpertsImpl:
    """Mix-in in front of a class that creates ``weight1`` / ``weight2`` / ``activation_func`` (Megatron's
    ``GroupedMLP``, or :class:`GroupedMLP` below)."""

    def __init__(self, num_local_experts, config=None):
        self.num_local_experts = num_local_experts
        self.config = config
        self.layer_number = None
        self.weight1 = None
        self.weight2 = None
        self.activation_checkpoint_manager = None
        super().__init__(num_local_experts, config)
        if self.config.gated_linear_unit:
            assert self.config.activation_func == F.silu, "Activation function must be silu when using fused_swiglu."
            self.activation_func = fused_swiglu

        def activation_func_with_probs(x, probs):
            if self.activation_func is fused_swiglu and x.dim() == 2 and x.size(0) != 0:
                # one kernel for activation and probability: silu(gate) * up * probs in fp32, rounded once
                return swiglu_with_probs(x, probs)
            dtype = x.dtype
            res = self.activation_func(x) * probs
            return res.to(dtype)

        self.activation_func_with_probs = activation_func_with_probs

    def _one_node(self, hidden_states, gemm_fusion):
        """Whether the whole body may run as ``ops.grouped_mlp``: gated SiLU, no in-place gradient accumulation, and the
        layout the fused kernels need."""
        cfg = self.config
        if gemm_fusion or not cfg.gated_linear_unit or not getattr(cfg, "moe_fuse_expert_mlp", True):
            return False
        w1, w2 = self.weight1, self.weight2
        ffn2 = w1.numel() // (self.num_local_experts * cfg.hidden_size)
        return (hidden_states.dtype in (torch.bfloat16, torch.float16) and w1.dtype == hidden_states.dtype
                and w2.dtype == hidden_states.dtype and cfg.hidden_size % 8 == 0 and ffn2 % 16 == 0
                and hidden_states.data_ptr() % 16 == 0 and w1.data_ptr() % 16 == 0 and w2.data_ptr() % 16 == 0)

    def forward(self, permuted_local_hidden_states, tokens_per_expert, permuted_probs=None):
        cfg = self.config
        is_recompute_activation = (
            should_recompute_activation(cfg, self.layer_number)
            and not getattr(cfg, "moe_alltoall_overlap_comm", False)
            and not getattr(cfg, "moe_allgather_overlap_comm", False)
        )
        gemm_fusion = getattr(cfg, "gemm_gradient_accumulation_fusion", False)
        if getattr(cfg, "qat_scheme", None) is not None:
            raise NotImplementedError("quantisation-aware expert weights (qat_scheme) are outside the MI355X expert path")
        E, H = self.num_local_experts, cfg.hidden_size
        probs = permuted_probs.unsqueeze(-1) if permuted_probs is not None else None
        act_fn = self.activation_func_with_probs if probs is not None else (lambda x, _p=None: self.activation_func(x))

        if permuted_local_hidden_states.nelement() != 0:
            w1 = self.weight1.view(E, H, -1)
            w2 = self.weight2.view(E, -1, H)
            if self._one_node(permuted_local_hidden_states, gemm_fusion):
                counts = tokens_per_expert.to(device=permuted_local_hidden_states.device, dtype=torch.int64,
                                              non_blocking=True)
                return grouped_mlp(permuted_local_hidden_states, w1, w2, counts, permuted_probs,
                                   recompute_activation=is_recompute_activation), None
            fc1_output = fusions.Ops.gmm(permuted_local_hidden_states, w1, tokens_per_expert, trans_b=False,
                                         gemm_fusion=gemm_fusion, original_weight=self.weight1)
            if not is_recompute_activation:
                intermediate_parallel = act_fn(fc1_output, probs)
            else:
                self.activation_checkpoint_manager = CheckpointWithoutOutput()
                intermediate_parallel = self.activation_checkpoint_manager.checkpoint(
                    act_fn, False, *((fc1_output, probs) if probs is not None else (fc1_output,)))
            fc2_output = fusions.Ops.gmm(intermediate_parallel, w2, tokens_per_expert, trans_b=False,
                                         gemm_fusion=gemm_fusion, original_weight=self.weight2)
        else:
            # No tokens on this rank: the grouped matmul has nothing to launch; 2-D matmuls on the flat weights keep
            # the parameters in the graph, so they still receive (zero) gradients.
            assert torch.count_nonzero(tokens_per_expert) == 0
            w1 = self.weight1.view(H, -1)
            w2 = self.weight2.view(-1, H)
            h = torch.matmul(permuted_local_hidden_states, w1)
            empty_act = (lambda x, p: (self._empty_activation(x) * p).to(x.dtype)) if probs is not None \
                else (lambda x, _p=None: self._empty_activation(x))
            if not is_recompute_activation:
                intermediate_parallel = empty_act(h, probs)
            else:
                self.activation_checkpoint_manager = CheckpointWithoutOutput()
                intermediate_parallel = self.activation_checkpoint_manager.checkpoint(
                    empty_act, False, *((h, probs) if probs is not None else (h,)))
            fc2_output = torch.matmul(intermediate_parallel, w2)

        if is_recompute_activation:
            # the activation's storage is released here and rebuilt from fc1 when the gradient of the second
            # matmul's output arrives (experts.py:183-191)
            self.activation_checkpoint_manager.discard_output()
            if fc2_output.requires_grad:
                fc2_output.register_hook(self.activation_checkpoint_manager.recompute)
        return fc2_output, None

    def _empty_activation(self, x):
        """The activation on a tensor without rows: nothing to launch, only shapes and graph edges."""
        if self.config.gated_linear_unit:
            gate, up = torch.chunk(x, 2, dim=-1)
            return F.silu(gate) * up
        return self.config.activation_func(x)


class _GroupedMLPParameters(torch.nn.Module):
    """What Megatron's ``GroupedMLP.__init__`` leaves behind for the mix-in: the flat expert weights and the
    activation (megatron/core/transformer/moe/experts.py, restated in the reference at experts.py:87-91 by the views
    it takes of them)."""

    def __init__(self, num_local_experts, config):
        super().__init__()
        ffn = getattr(config, "moe_ffn_hidden_size", None) or config.ffn_hidden_size
        fc1_out = ffn * 2 if config.gated_linear_unit else ffn
        dtype = getattr(config, "params_dtype", torch.float32)
        device = getattr(config, "device", None)
        self.weight1 = torch.nn.Parameter(torch.empty(config.hidden_size, num_local_experts * fc1_out, dtype=dtype,
                                                      device=device))
        self.weight2 = torch.nn.Parameter(torch.empty(num_local_experts * ffn, config.hidden_size, dtype=dtype,
                                                      device=device))
        init = getattr(config, "init_method", None) or (lambda w: torch.nn.init.normal_(w, mean=0.0, std=0.02))
        with torch.no_grad():
            init(self.weight1)
            (getattr(config, "output_layer_init_method", None) or init)(self.weight2)
        # the flag the grouped matmul's deferred weight-gradient path looks for (weight_grad_store.py:75)
        self.weight1.gmm_weight = True
        self.weight2.gmm_weight = True
        self.activation_func = config.activation_func


class GroupedMLP(GmmExpertsImpl, _GroupedMLPParameters):
    """``GmmExpertsImpl`` over parameters of its own: the expert module without Megatron."""
