"""Feed-forward parts: the dense SwiGLU and the routed mixture of SwiGLU experts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..ops.profile import active as profiling, section
from .base import ParamSpec, Part, ResidualStream, StepContext, TensorSource
from .norm import RMSNorm


def _fuse_rows(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """[.., Ia, H] and [.., Ib, H] -> [.., Ia + Ib, H] (gate rows first, up rows second)."""
    dt = torch.float32 if torch.float32 in (a.dtype, b.dtype) else a.dtype
    shape = list(a.shape)
    shape[-2] = a.shape[-2] + b.shape[-2]
    out = torch.empty(shape, dtype=dt, device=a.device)
    out[..., : a.shape[-2], :].copy_(a)
    out[..., a.shape[-2]:, :].copy_(b)
    return out


def _rows(w) -> torch.Tensor:
    return ops.unpack_weight(w) if isinstance(w, ops.PackedWeight) else w


def _activation_code(name: str) -> int:
    try:
        return ops.ACTIVATIONS[name]
    except KeyError:
        raise ValueError(f"activation {name!r} is not known ({', '.join(sorted(ops.ACTIVATIONS))})") from None


class DenseSwiGLU(Part):
    """down( act(gate x) * (up x) ) (reference: src/SharpInference.Engine/ForwardPass.cs:2006-2015;
    silu(g) = g / (1 + exp(-g)), src/SharpInference.Cpu/SimdKernels.cs:4377-4408).  ``activation``
    names the gate's function: "silu" (the reference's) or "gelu_tanh"."""

    def __init__(self, hidden: int, intermediate: int, activation: str = "silu"):
        self.hidden, self.inter = int(hidden), int(intermediate)
        self.act = _activation_code(activation)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        return {
            prefix + "gate_proj.weight": ParamSpec((self.inter, self.hidden)),
            prefix + "up_proj.weight": ParamSpec((self.inter, self.hidden)),
            prefix + "down_proj.weight": ParamSpec((self.hidden, self.inter)),
        }

    def load(self, prefix: str, source: TensorSource) -> None:
        g = source.get(prefix + "gate_proj.weight")
        u = source.get(prefix + "up_proj.weight")
        # both also in the order the few-rows kernel streams them; the rows stay for prompt-sized steps
        self.w_gate_up = ops.pack_weight(_fuse_rows(g, u))
        del g, u
        self.w_down = ops.pack_weight(source.get(prefix + "down_proj.weight"))

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        T = x.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        with section("dense feed-forward", nbytes=width * 3 * self.inter * self.hidden + width * T * (2 * self.hidden + 3 * self.inter),
                     flops=6.0 * T * self.inter * self.hidden):
            gu = ops.linear(x, self.w_gate_up, ctx.act_dtype)
            act = ops.gated_act(gu, None, self.act)
            return ops.linear(act, self.w_down, ctx.act_dtype)


class MoESwiGLU(Part):
    """Router -> top-k experts (+ an always-on shared expert)
    (reference: src/SharpInference.Engine/ForwardPass.cs:2021-2098).

    The router's logits, gate and picks are float and stay on the device.  With
    ``score_on_input`` the gate and up products of a chosen expert are multiplied by its score
    before the SiLU (ForwardPass.cs:2083-2089); without it the expert runs on the unscaled input
    and its output is multiplied by the score where the outputs are summed (the reference's other
    order, src/SharpInference.Cuda/CudaKernels.cs:112-157 llm_moe_weighted_reduce).  The shared
    expert sees the unscaled input (2060-2066); the outputs are summed (2096-2097).  ``gate`` is "sigmoid" or "softmax"
    (2031-2034); ``renormalise`` divides the k scores by their sum (2156-2162); ``activation`` names the
    experts' gate function ("silu", the reference's, or "gelu_tanh")."""

    MERGE_MAX_TOKENS = 16   # one row block of the few-rows kernel for the shared group (measured: up to 64 tokens
                            # the merged launches and the library's product for the shared expert are as fast)
    MERGE_MIN_MANY_TOKENS = None   # tokens from which the shared expert is one more group of the many-rows grouped
                                   # product; off: measured at 2,048 tokens, 1.48 ms a layer against 0.93 + 0.45 with
                                   # the library's product for the shared expert (which runs at the matrix cores' peak)

    def __init__(self, hidden: int, num_experts: int, top_k: int, expert_intermediate: int,
                 shared_intermediate: Optional[int] = None, gate: str = "sigmoid", renormalise: bool = False,
                 score_on_input: bool = True, activation: str = "silu"):
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top_k {top_k} must lie in 1..{num_experts}")
        if num_experts > ops.ROUTER_MAX_EXPERTS:
            raise ValueError(f"{num_experts} experts are not taken: the routing kernels hold scores for {ops.ROUTER_MAX_EXPERTS}")
        if gate not in ("sigmoid", "softmax"):
            raise ValueError(f"router gate {gate!r} is not known (sigmoid, softmax)")
        self.hidden, self.E, self.k = int(hidden), int(num_experts), int(top_k)
        self.inter = int(expert_intermediate)
        self.act = _activation_code(activation)
        self.shared = DenseSwiGLU(hidden, shared_intermediate, activation) if shared_intermediate else None
        self.gate = ops.GATE_SIGMOID if gate == "sigmoid" else ops.GATE_SOFTMAX
        self.renormalise = bool(renormalise)
        self.score_on_input = bool(score_on_input)
        self.w_router: Optional[torch.Tensor] = None
        self.w_gate_up: Optional[torch.Tensor] = None     # [E, 2*I, H]
        self.w_down: Optional[torch.Tensor] = None        # [E, H, I]

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        out = {
            prefix + "router.weight": ParamSpec((self.E, self.hidden)),
            prefix + "experts.gate_proj": ParamSpec((self.E, self.inter, self.hidden)),
            prefix + "experts.up_proj": ParamSpec((self.E, self.inter, self.hidden)),
            prefix + "experts.down_proj": ParamSpec((self.E, self.hidden, self.inter)),
        }
        if self.shared is not None:
            out.update(self.shared.param_specs(prefix + "shared_expert."))
        return out

    def load(self, prefix: str, source: TensorSource) -> None:
        self.w_router = source.get(prefix + "router.weight")
        g = source.get(prefix + "experts.gate_proj")
        u = source.get(prefix + "experts.up_proj")
        d = source.get(prefix + "experts.down_proj")
        self.merged = False
        sh = self.shared
        if sh is not None:
            sh.load(prefix + "shared_expert.", source)
        bf16 = g.dtype == u.dtype == d.dtype == torch.bfloat16
        # The experts' matrices are kept only in the order the kernels stream them (no rows: both
        # the few-rows and the many-rows product of the experts read that order), if the sizes allow.
        pack = bf16 and self.inter % 128 == 0 and self.hidden % 128 == 0
        merge = (bf16 and sh is not None and sh.inter == self.inter and sh.w_gate_up.dtype == torch.bfloat16
                 and sh.w_down.dtype == torch.bfloat16)   # (dtype: of a tensor or of a packed weight)
        if not bf16:
            self.w_gate_up, self.w_down = _fuse_rows(g, u), d
            return
        # With a shared expert of the experts' width, it becomes expert E of their tensors: few-row
        # steps then run it in the same launches as the routed ones.
        n = self.E + (1 if merge else 0)
        gu = torch.empty(n, 2 * self.inter, self.hidden, dtype=torch.bfloat16, device=g.device)
        dn = torch.empty(n, self.hidden, self.inter, dtype=torch.bfloat16, device=d.device)
        put = ops.pack_into if pack else (lambda dst, src: dst.copy_(src))
        for e in range(self.E):
            put(gu[e, :self.inter], g[e])
            put(gu[e, self.inter:], u[e])
            put(dn[e], d[e])
        del g, u, d
        if merge:
            sgu, sdn = _rows(sh.w_gate_up), _rows(sh.w_down)
            put(gu[self.E, :self.inter], sgu[:self.inter])
            put(gu[self.E, self.inter:], sgu[self.inter:])
            put(dn[self.E], sdn)
            if pack:   # the shared expert's own packed copies give way to these
                sh.w_gate_up, sh.w_down = ops.PackedWeight(gu[self.E], sgu), ops.PackedWeight(dn[self.E], sdn)
            else:      # its own tensors turn into views
                sh.w_gate_up, sh.w_down = gu[self.E], dn[self.E]
            self.merged = True
        self.w_gate_up = ops.PackedWeight(gu, None) if pack else gu
        self.w_down = ops.PackedWeight(dn, None) if pack else dn

    def _experts_section(self, ids: torch.Tensor, T: int, with_shared: bool):
        """The profiler's span of the experts' two products: every expert that a token picked is
        read once (the count is taken from the picks, only while profiling)."""
        if not profiling():
            return section("experts")
        width = 2 if self.w_gate_up.dtype == torch.bfloat16 else 4
        used = int(ids.unique().numel()) + (1 if with_shared else 0)
        rows = T * self.k + (T if with_shared else 0)
        per_expert = 3 * self.inter * self.hidden
        return section("experts" + (" + shared" if with_shared else ""), nbytes=width * (used * per_expert + rows * (2 * self.hidden + 3 * self.inter)),
                       flops=2.0 * rows * per_expert)

    def _few_tokens(self, T: int, ctx: StepContext) -> bool:
        """A few decode tokens in bfloat16 (at most 64 picks): the experts' two products find their
        rows from the picks themselves."""
        packed = isinstance(self.w_gate_up, ops.PackedWeight)
        return (ctx.act_dtype == torch.bfloat16 and self.w_gate_up.dtype == torch.bfloat16
                and ops.picked_ok(T, self.k, 2 * self.inter, self.hidden, True, packed)
                and ops.picked_ok(T, self.k, self.hidden, self.inter, False, packed))

    def _picked(self, x: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, ctx: StepContext):
        """No sorting kernel: pair by pair in the picks' own order.  With up to MERGE_MAX_TOKENS
        tokens the shared expert rides along as one more group of the same two launches (its rows
        after the pairs'); with more it goes through the library."""
        T = x.shape[0]
        trace = ctx.extras.get("router_trace")
        if trace is not None:      # the picks of this step, layer by layer (reference: ForwardPass.cs:2042-2056)
            trace.append((ids, wts, x))
        along = self.merged and T <= self.MERGE_MAX_TOKENS
        shared = None if along or self.shared is None else self.shared.forward(x, ctx)
        with self._experts_section(ids, T, along):
            act = ops.gemm_skinny_picked(x, self.w_gate_up, ids, wts if self.score_on_input else None, along, True,
                                         self.act, ctx.act_dtype)
            y = ops.gemm_skinny_picked(act, self.w_down, ids, None, along, False, False, ctx.act_dtype)
        return ops.ExpertSum(y, ops.counting(T * self.k, x.device), y[T * self.k:] if along else shared, T, self.k,
                             None if self.score_on_input else wts)

    def forward_from_stream(self, stream: ResidualStream, norm: Part, ctx: StepContext):
        """The block's second half from the residual stream: normalise and feed forward.  With a
        few decode tokens the norm and the router are one launch (the bits of the two)."""
        T = stream.h.shape[0]
        if (self._few_tokens(T, ctx) and isinstance(norm, RMSNorm)
                and ops.norm_router_ok(stream.h, stream.pending, ctx.act_dtype)):
            with section("norm + router", nbytes=T * self.hidden * 10 + 2 * self.E * self.hidden):
                x, ids, wts = ops.add_rmsnorm_router(stream.h, stream.pending, norm.weight, norm.eps, self.w_router, self.k,
                                                     self.gate, self.renormalise)
            stream.pending = None
            return self._picked(x, ids, wts, ctx)
        return self.forward(norm.forward(stream, ctx.act_dtype), ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        T = x.shape[0]
        trace = ctx.extras.get("router_trace")
        if self._few_tokens(T, ctx):
            with section("router", nbytes=2 * T * self.hidden + 2 * self.E * self.hidden):
                ids, wts = ops.router_topk(x, self.w_router, self.k, self.gate, self.renormalise)
            return self._picked(x, ids, wts, ctx)
        many = self.MERGE_MIN_MANY_TOKENS is not None and T >= self.MERGE_MIN_MANY_TOKENS
        merge = self.merged and ctx.act_dtype == torch.bfloat16 and (T <= self.MERGE_MAX_TOKENS or many)
        with section("router", nbytes=2 * T * self.hidden + 2 * self.E * self.hidden):
            ids, wts, rt = ops.route(x, self.w_router, self.k, self.gate, self.renormalise, shared_group=merge)
        if trace is not None:      # the picks of this step, layer by layer (reference: ForwardPass.cs:2042-2056)
            trace.append((ids, wts, x))
        after = None if self.score_on_input else wts     # scores applied where the outputs are summed
        if merge:
            # few rows: the shared expert rides along as one more group of the same two launches
            with self._experts_section(ids, T, True):
                act = ops.grouped_swiglu(x, self.w_gate_up, rt, ctx.act_dtype, scaled=self.score_on_input, act=self.act)
                y = ops.grouped_linear(act, self.w_down, rt, False, ctx.act_dtype)
            # left as a sum: the next norm forms it while it reads the residual stream
            return ops.ExpertSum(y, rt.inv_pos, y[T * self.k:], T, self.k, after)
        shared = self.shared.forward(x, ctx) if self.shared is not None else None
        with self._experts_section(ids, T, False):
            act = ops.grouped_swiglu(x, self.w_gate_up, rt, ctx.act_dtype, scaled=self.score_on_input, act=self.act)
            y = ops.grouped_linear(act, self.w_down, rt, False, ctx.act_dtype)
        return ops.ExpertSum(y, rt.inv_pos, shared, T, self.k, after)   # formed by the next norm (or by whoever asks for a tensor)
