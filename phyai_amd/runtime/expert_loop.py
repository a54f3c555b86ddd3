"""The action expert's flow-matching denoise loop, unrolled into one hipGraph.

Mirrors the part of the reference's ``PI05ExpertRunner`` that drives the quantized-linear path
(``phyai/src/phyai/models/pi05/model_runner_pi05.py:560-738``): ``bind_euler_schedule`` projects
the per-step AdaRMS modulation tables once, outside the graph (``:560-607``); ``setup`` records
``_fwd_loop`` - ``num_steps`` Euler steps of ``_one_step`` = action embedding, all decoder layers,
final adaptive norm, action projection, ``x_t <- x_t + dt * v_t`` (``:689-738``) - as ONE graph;
``run`` replays it.  The decoder layer is ``PI05ExpertLayer.forward``
(``models/pi05/modeling_pi05.py:801-835``).

What is NOT mirrored is the reference's attention back end (paged KV pool, flashinfer planning):
attention is a callback ``attend(fused_qkv, layer_index) -> [M, heads * head_dim]``.
:class:`PrefixAttentionStandIn` is a plain-torch one (RoPE + SDPA over a fixed prefix KV plus the
chunk's own keys and values) so that data really chains through the layers; it is a stand-in,
not a kernel of this package.

Three forms of the layer run on the same weights:

``fused``    norm + quantizer in one kernel, GEMM on its codes, attention, GEMM with the gated
             residual in its epilogue, norm + quantizer, GEMM + GeGLU epilogue, GEMM + gated
             residual: 8 kernels of this library per layer;
``unfused``  the reference's structure on this library's kernels: norm, quantized linear,
             attention, quantized linear, ``torch.addcmul``, norm, MLP, ``torch.addcmul``
             (12 kernels per layer).  Bit-equal to ``fused``;
``torch``    the reference's own arithmetic as torch library calls (norm and quantizer
             expressions, ``torch._scaled_mm``, ``gelu * up``, ``addcmul``): the yardstick the
             other two are held to, layer by layer.
"""

from __future__ import annotations

import dataclasses
from typing import Callable, Sequence

import torch
import torch.nn.functional as F
from torch import nn

from phyai_amd.linear import QKVParallelLinear, ReplicatedLinear, RowParallelLinear
from phyai_amd.mlp import DenseMLP
from phyai_amd.norm import AdaRMSNorm
from phyai_amd.quant import Fp8Spec
from phyai_amd.runtime.graph import HipGraph

VARIANTS = ("fused", "unfused", "torch")
Attend = Callable[[torch.Tensor, int], torch.Tensor]


@dataclasses.dataclass
class ExpertLayerModulation:
    """One step's projected ``scale | shift | gate`` rows of a layer's two adaptive norms."""

    input_ln: torch.Tensor            # [1, 3 * hidden]
    post_attention_ln: torch.Tensor   # [1, 3 * hidden]


def _torch_adarmsnorm(h: torch.Tensor, mod: torch.Tensor, eps: float):
    scale, shift, gate = mod.float().chunk(3, dim=-1)
    hf = h.float()
    n = hf * torch.rsqrt(hf.pow(2).mean(-1, keepdim=True) + eps)
    return (n * (1.0 + scale) + shift).to(h.dtype), gate.to(h.dtype)


def _torch_fp8_linear(x: torch.Tensor, layer: nn.Module, act: bool = False) -> torch.Tensor:
    """``Fp8Spec.quantize_activation`` + ``TorchKernel._fp8_per_channel`` (reference
    ``layers/quant/fp8.py:152-154``, ``layers/linear/backends/torch.py:166-175``) as torch calls."""
    a = x.abs().amax(dim=-1, keepdim=True).clamp_min(1e-12)
    s = (a / 448.0).to(torch.float32)
    xq = (x / s).to(torch.float8_e4m3fn)
    y = torch._scaled_mm(xq, layer.weight.t(), scale_a=s, scale_b=layer.weight_scale.reshape(1, -1),
                         bias=layer.bias, out_dtype=x.dtype)
    if act:
        half = y.shape[-1] // 2
        y = F.gelu(y[:, :half], approximate="tanh") * y[:, half:]
    return y


class ExpertLayer(nn.Module):
    """Pre-AdaRMS self-attention + gated MLP (``PI05ExpertLayer``, ``modeling_pi05.py:704-835``) with
    fp8 W8A8 linears; attention itself is the caller's."""

    def __init__(self, hidden_size: int = 1024, head_dim: int = 256, num_heads: int = 8, num_kv_heads: int = 1,
                 intermediate_size: int = 4096, cond_dim: int = 1024, eps: float = 1e-6, *, spec=None,
                 params_dtype: torch.dtype = torch.bfloat16, prefix: str = "") -> None:
        super().__init__()
        spec_of = (lambda: spec) if spec is not None else Fp8Spec
        child = (lambda n: f"{prefix}.{n}" if prefix else n)
        self.hidden_size, self.eps = hidden_size, eps
        self.input_layernorm = AdaRMSNorm(hidden_size, cond_dim, eps, dtype=params_dtype, prefix=child("input_layernorm"))
        self.qkv_proj = QKVParallelLinear(hidden_size, head_dim, num_heads, num_kv_heads, bias=False,
                                          params_dtype=params_dtype, spec=spec_of(), prefix=child("self_attn.qkv_proj"))
        self.o_proj = RowParallelLinear(num_heads * head_dim, hidden_size, bias=False, params_dtype=params_dtype,
                                        spec=spec_of(), prefix=child("self_attn.o_proj"))
        self.post_attention_layernorm = AdaRMSNorm(hidden_size, cond_dim, eps, dtype=params_dtype,
                                                   prefix=child("post_attention_layernorm"))
        self.mlp = DenseMLP(hidden_size, intermediate_size, activation="gelu_tanh", params_dtype=params_dtype,
                            spec_in=spec_of(), spec_out=spec_of(), prefix=child("mlp"))

    def forward(self, h: torch.Tensor, attend: Attend, index: int, modulation: ExpertLayerModulation,
                variant: str = "fused") -> torch.Tensor:
        residual = h
        if variant == "fused":
            view, gate_attn = self.input_layernorm.forward_fp8(h, modulation=modulation.input_ln)
            fused, _ = self.qkv_proj(view)
            h = self.o_proj.forward_addcmul(attend(fused, index), residual, gate_attn)
            view, gate_mlp = self.post_attention_layernorm.forward_fp8(h, modulation=modulation.post_attention_ln)
            act = self.mlp.gate_up_proj.forward_fused(view, "geglu_tanh")
            return self.mlp.down_proj.forward_addcmul(act, h, gate_mlp)
        if variant == "unfused":
            n, gate_attn = self.input_layernorm(h, modulation=modulation.input_ln)
            fused, _ = self.qkv_proj(n)
            out, _ = self.o_proj(attend(fused, index))
            h = torch.addcmul(residual, out, gate_attn)
            m, gate_mlp = self.post_attention_layernorm(h, modulation=modulation.post_attention_ln)
            return torch.addcmul(h, self.mlp(m), gate_mlp)
        if variant == "torch":
            n, gate_attn = _torch_adarmsnorm(h, modulation.input_ln, self.eps)
            fused = _torch_fp8_linear(n, self.qkv_proj)
            h = torch.addcmul(residual, _torch_fp8_linear(attend(fused, index), self.o_proj), gate_attn)
            m, gate_mlp = _torch_adarmsnorm(h, modulation.post_attention_ln, self.eps)
            act = _torch_fp8_linear(m, self.mlp.gate_up_proj, act=True)
            return torch.addcmul(h, _torch_fp8_linear(act, self.mlp.down_proj), gate_mlp)
        raise ValueError(f"unknown variant {variant!r}; expected one of {VARIANTS}")


class PrefixAttentionStandIn:
    """Plain-torch joint attention of the action chunk over a fixed prefix: RoPE on q / k, the chunk's
    keys and values appended behind ``prefix_len`` cached positions per layer, SDPA with one KV head
    shared by all query heads.  Stands in for the reference's attention back end so that the loop's
    data chains; every variant of the loop uses the same one."""

    def __init__(self, n_layers: int, chunk: int, prefix_len: int, num_heads: int = 8, head_dim: int = 256, *,
                 device, dtype: torch.dtype = torch.bfloat16, seed: int = 4242) -> None:
        g = torch.Generator().manual_seed(seed)
        self.chunk, self.prefix_len, self.heads, self.hd = chunk, prefix_len, num_heads, head_dim

        def cache():
            pre = torch.randn(prefix_len, 1, head_dim, generator=g).to(dtype)
            return torch.cat([pre, torch.zeros(chunk, 1, head_dim, dtype=dtype)]).to(device)

        self.k_cache = [cache() for _ in range(n_layers)]
        self.v_cache = [cache() for _ in range(n_layers)]
        pos = torch.arange(prefix_len, prefix_len + chunk, dtype=torch.float32)
        inv = 1.0 / (10000.0 ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
        ang = pos[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos()[:, None, :].to(device), ang.sin()[:, None, :].to(device)

    def _rope(self, t: torch.Tensor) -> torch.Tensor:
        half = self.hd // 2
        t1, t2 = t[..., :half].float(), t[..., half:].float()
        return torch.cat([t1 * self.cos - t2 * self.sin, t2 * self.cos + t1 * self.sin], dim=-1).to(t.dtype)

    def __call__(self, fused: torch.Tensor, index: int) -> torch.Tensor:
        M, H, HD, P = self.chunk, self.heads, self.hd, self.prefix_len
        q, k, v = fused.split([H * HD, HD, HD], dim=-1)
        q, k = self._rope(q.reshape(M, H, HD)), self._rope(k.reshape(M, 1, HD))
        self.k_cache[index][P:].copy_(k)
        self.v_cache[index][P:].copy_(v.reshape(M, 1, HD))
        S = P + M
        o = F.scaled_dot_product_attention(q.transpose(0, 1)[None],
                                           self.k_cache[index].transpose(0, 1)[None].expand(1, H, S, HD),
                                           self.v_cache[index].transpose(0, 1)[None].expand(1, H, S, HD))
        return o[0].transpose(0, 1).reshape(M, H * HD)


class ExpertDenoiseLoop(nn.Module):
    """``num_steps`` Euler steps of the expert stack as one graph (batch 1).

    ``heads``: ``embed_action`` (action_dim -> hidden) and ``project_action`` (hidden -> action_dim)
    are plain bf16 linears, outside the quantized path as in the reference."""

    def __init__(self, layers: Sequence[ExpertLayer], attend: Attend, *, chunk_size: int = 50, action_dim: int = 32,
                 hidden_size: int = 1024, cond_dim: int = 1024, eps: float = 1e-6, variant: str = "fused",
                 use_graph: bool = True, params_dtype: torch.dtype = torch.bfloat16) -> None:
        super().__init__()
        if variant not in VARIANTS:
            raise ValueError(f"unknown variant {variant!r}; expected one of {VARIANTS}")
        self.layers = nn.ModuleList(layers)
        self.attend, self.variant, self.use_graph = attend, variant, use_graph
        self.chunk_size, self.action_dim, self.hidden_size = chunk_size, action_dim, hidden_size
        self.params_dtype = params_dtype
        self.embed_action = ReplicatedLinear(action_dim, hidden_size, bias=True, params_dtype=params_dtype, prefix="embed_action")
        self.project_action = ReplicatedLinear(hidden_size, action_dim, bias=True, params_dtype=params_dtype, prefix="project_action")
        self.final_norm = AdaRMSNorm(hidden_size, cond_dim, eps, dtype=params_dtype, prefix="norm")
        self._time_emb_table: torch.Tensor | None = None
        self._mod_tables: list[list[ExpertLayerModulation]] | None = None   # [step][layer]
        self._final_mod: list[torch.Tensor] | None = None                  # [step]
        self._num_steps, self._dt = 0, 0.0
        self.graph: HipGraph | None = None

    # ---- schedule (model_runner_pi05.py:560-607) ------------------------------------------------
    def bind_euler_schedule(self, time_emb_table: torch.Tensor, dt: float, num_steps: int) -> None:
        if time_emb_table.shape[0] != num_steps:
            raise ValueError(f"time_emb_table has {time_emb_table.shape[0]} rows but num_steps={num_steps}.")
        self._time_emb_table, self._dt, self._num_steps = time_emb_table, float(dt), int(num_steps)
        self._build_modulation_tables()

    def _build_modulation_tables(self) -> None:
        """One projection of the whole time-embedding table per norm; a same-shape re-bind copies
        in place, so that a recorded graph keeps reading the same storage."""
        table = self._time_emb_table
        per_layer = [(lay.input_layernorm.project_modulation(table), lay.post_attention_layernorm.project_modulation(table))
                     for lay in self.layers]
        final = self.final_norm.project_modulation(table)
        new_tables = [[ExpertLayerModulation(a[s:s + 1], b[s:s + 1]) for a, b in per_layer] for s in range(self._num_steps)]
        new_final = [final[s:s + 1] for s in range(self._num_steps)]
        if self._mod_tables is not None and len(self._mod_tables) == len(new_tables):
            for old_step, new_step in zip(self._mod_tables, new_tables):
                for old, new in zip(old_step, new_step):
                    old.input_ln.copy_(new.input_ln)
                    old.post_attention_ln.copy_(new.post_attention_ln)
            for old, new in zip(self._final_mod, new_final):
                old.copy_(new)
        else:
            self._mod_tables, self._final_mod = new_tables, new_final

    # ---- setup (model_runner_pi05.py:613-686) ---------------------------------------------------
    def setup(self) -> None:
        if self._time_emb_table is None or self._num_steps <= 0:
            raise RuntimeError("ExpertDenoiseLoop.setup() called before bind_euler_schedule(); the recorded graph "
                               "unrolls the Euler loop and needs the time-embedding table and step count.")
        if self.use_graph:
            self._capture_graph()

    def _capture_graph(self) -> None:
        dev = self.embed_action.weight.device
        example = {"noise": torch.zeros(self.chunk_size, self.action_dim, dtype=self.params_dtype, device=dev)}
        self.graph = HipGraph()
        self.graph.capture(self._fwd_loop, example)

    # ---- forward path (model_runner_pi05.py:689-738) -------------------------------------------
    def _one_step(self, x_t: torch.Tensor, step: int, trace: list | None = None) -> torch.Tensor:
        h, _ = self.embed_action(x_t)
        for i, layer in enumerate(self.layers):
            if trace is not None:
                trace.append(h)
            h = layer(h, self.attend, i, self._mod_tables[step][i], self.variant)
        if trace is not None:
            trace.append(h)
        if self.variant == "torch":
            n, _ = _torch_adarmsnorm(h, self._final_mod[step], self.final_norm.variance_epsilon)
        else:
            n, _ = self.final_norm(h, modulation=self._final_mod[step])
        v_t, _ = self.project_action(n)
        return v_t

    def _fwd_loop(self, *, noise: torch.Tensor, trace: list | None = None) -> torch.Tensor:
        x_t = noise
        for step in range(self._num_steps):
            v_t = self._one_step(x_t, step, trace)
            x_t = x_t + self._dt * v_t.to(x_t.dtype)
        return x_t

    def run(self, noise: torch.Tensor) -> torch.Tensor:
        """Final ``x_t`` for one action chunk: a graph replay when recorded, else the eager loop."""
        if self.graph is not None:
            return self.graph.replay({"noise": noise})
        return self._fwd_loop(noise=noise)


__all__ = ["ExpertLayer", "ExpertLayerModulation", "ExpertDenoiseLoop", "PrefixAttentionStandIn", "VARIANTS"]
