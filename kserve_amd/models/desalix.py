"""Desalix: a decoder of chunk-local attention layers with routed experts,
part of which is run several times over.

The layers are listed one by one in the config. A span of them (``loop``) is
run ``times`` times in a row with the same weights; every pass keeps KV pages
of its own, re-injects the embedding output (from the second pass on) and adds
a learned per-pass vector before its first layer.

A layer wraps each sublayer in two norms and a per-channel scale,

    x += ls1 * norm1b(mixer(norm1(x)))
    x += ls2 * norm2b(ff(norm2(x)))          (if the layer has a feed-forward)

where every norm is an RMS norm with ONE learned gain for all channels. The
mixer is ``RotaryChunkSinkAttention`` (per-head q/k norm, partial rotation,
unit-norm rotated values, chunk-local mask, sink), the feed-forward
``RoutedClampedMoE``. The residual stream is fp32 whatever the activation
dtype; "close the previous sublayer (post-norm, layer scale, add), add what a
new pass adds, norm for the next sublayer" is one kernel.
"""

from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kserve_amd import ops
from kserve_amd.engine.config import (
    GLUSpec,
    HybridLayerSpec,
    HybridModelConfig,
    MoESpec,
)
from kserve_amd.models.mixers import (
    ClampedGLU,
    RotaryChunkSinkAttention,
    RoutedClampedMoE,
)
from kserve_amd.parallel import comm


def _scalar():
    return nn.Parameter(torch.empty((), dtype=torch.float32), requires_grad=False)


class DesalixLayer(nn.Module):
    def __init__(self, width: int, spec: HybridLayerSpec, eps: float, dtype):
        super().__init__()
        if spec.attention is None or spec.ssm is not None:
            raise ValueError("a Desalix layer has an attention mixer and nothing else")
        self.spec = spec
        self.attn = RotaryChunkSinkAttention(width, spec.attention, eps, dtype)
        if isinstance(spec.mlp, MoESpec):
            self.mlp = RoutedClampedMoE(width, spec.mlp, dtype)
        elif isinstance(spec.mlp, GLUSpec):
            self.mlp = ClampedGLU(width, spec.mlp, dtype)
        else:
            self.mlp = None
        self.norm1 = _scalar()
        self.norm1b = _scalar()
        self.ls1 = nn.Parameter(
            torch.empty(width, dtype=torch.float32), requires_grad=False
        )
        if self.mlp is not None:
            self.norm2 = _scalar()
            self.norm2b = _scalar()
            self.ls2 = nn.Parameter(
                torch.empty(width, dtype=torch.float32), requires_grad=False
            )
        # the scalar gains as host numbers (kernel arguments)
        self.g1 = self.g1b = self.g2 = self.g2b = 1.0

    def finish_load(self):
        self.g1, self.g1b = float(self.norm1), float(self.norm1b)
        if self.mlp is not None:
            self.g2, self.g2b = float(self.norm2), float(self.norm2b)


class DesalixForCausalLM(nn.Module):
    # every step attends through the paged cache (no separate un-paged
    # prefill kernel); there is no recurrent state
    paged_prefill_only = True
    needs_state_slots = False

    def __init__(
        self,
        config: HybridModelConfig,
        dtype: Optional[torch.dtype] = None,
        device: str = "cpu",
    ):
        super().__init__()
        st = comm.get_state()
        if st.tp_size != 1 or st.pp_size != 1:
            raise NotImplementedError(
                "Desalix runs on one GPU per replica (no tensor/pipeline split)"
            )
        self.config = config
        dtype = dtype or (
            torch.bfloat16 if config.dtype == "bfloat16" else torch.float32
        )
        self.dtype = dtype
        W = config.hidden_size
        self.embed = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.layers = nn.ModuleList(
            [DesalixLayer(W, spec, config.rms_norm_eps, dtype) for spec in config.layers]
        )
        self.runs = config.layer_runs()
        self.loop_start = config.loop.start if config.loop is not None else -1
        times = max([t + 1 for _, t in self.runs if t is not None], default=0)
        self.loop_step = (
            nn.Parameter(torch.empty(times, W, dtype=torch.float32), requires_grad=False)
            if times else None
        )
        self.num_local_layers = len(self.runs)
        self.final_norm = _scalar()
        self.g_final = 1.0
        self.head = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.eps = config.rms_norm_eps
        # largest decode batch worth capturing: above it the routed experts
        # switch to their sorted form, which synchronises with the host
        caps = [
            l.mlp.dense_max_tokens for l in self.layers
            if isinstance(l.mlp, RoutedClampedMoE)
        ]
        self.decode_graph_max_tokens = min(caps) if caps else None
        # when a list, forward() appends the residual stream after each layer run
        self.debug_residuals: Optional[List[torch.Tensor]] = None
        self.to(device)

    # -- cache layout (read by the model runner) ------------------------------
    def cache_layout(self):
        """One entry per layer RUN (a looped layer once per pass):
        (kv_heads, dim, vdim) and no recurrent state."""
        out = []
        for i, _ in self.runs:
            a = self.layers[i].spec.attention
            out.append(((a.kv_heads, a.dim, a.vdim), {}))
        return out

    # -- init -----------------------------------------------------------------
    @torch.no_grad()
    def random_init(self, std: float = 0.02, seed: int = 0):
        dev = self.embed.device
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("q_norm", "k_norm") or p.dim() == 0:
                p.fill_(1.0)
            elif leaf in ("ls1", "ls2"):
                p.fill_(0.5)
            elif p.dim() >= 2 and leaf != "loop_step":
                # keep activations O(1) through the stack
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)
            else:
                p.normal_(0.0, 0.1, generator=gen)
        self._finish_load()
        return self

    def _finish_load(self):
        for layer in self.layers:
            layer.finish_load()
        self.g_final = float(self.final_norm)

    # -- forward --------------------------------------------------------------
    def forward(self, input_ids, positions, caches, meta):
        emb = ops.embed_scale_sinpos(
            self.embed, input_ids, positions, None, self.config.embedding_scale
        )
        looped = self.loop_step is not None and self.loop_step.shape[0] > 1
        x = emb.clone() if looped else emb
        pending = (None, 1.0, None)  # (sublayer output, post gain, layer scale)
        dbg = self.debug_residuals
        for (i, t), cache in zip(self.runs, caches):
            layer = self.layers[i]
            add_rows = add_vec = None
            if t is not None and i == self.loop_start:
                add_rows = emb if t > 0 else None
                add_vec = self.loop_step[t]
            h = self._close_open(x, pending, layer.g1, add_rows, add_vec)
            pending = (layer.attn(h, positions, cache, meta), layer.g1b, layer.ls1)
            if layer.mlp is not None:
                h = self._close_open(x, pending, layer.g2)
                pending = (layer.mlp(h), layer.g2b, layer.ls2)
            if dbg is not None:
                r = x.clone()
                ops.post_norm_add_rms_norm(
                    r, pending[0], pending[1], pending[2], self.eps, 1.0,
                    self.dtype, want_out=False,
                )
                dbg.append(r)
        return self._close_open(x, pending, self.g_final)

    def _close_open(self, x, pending, next_gain, add_rows=None, add_vec=None):
        d, g, ls = pending
        return ops.post_norm_add_rms_norm(
            x, d, g, ls, self.eps, next_gain, self.dtype, add_rows, add_vec
        )

    def compute_logits(self, hidden):
        return F.linear(hidden, self.head)

    # -- weights ----------------------------------------------------------------
    @torch.no_grad()
    def load_hf_state_dict(self, tensors) -> None:
        """Tensor names: embed, loop.step, l<i>.norm1|norm1b|norm2|norm2b,
        l<i>.ls1|ls2, l<i>.mix.q|k|v|o|q.norm|k.norm|sink,
        l<i>.mlp.router, l<i>.mlp.e<j>.gate|up|down,
        l<i>.mlp.shared.gate|up|down, final.norm, head."""

        def get(name):
            t = tensors[name]
            return t() if callable(t) else t

        self.embed.copy_(get("embed").to(self.dtype))
        self.head.copy_(get("head").to(self.dtype))
        self.final_norm.copy_(get("final.norm").float().reshape(()))
        if self.loop_step is not None:
            self.loop_step.copy_(get("loop.step").float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.copy_(get(p + "norm1").float().reshape(()))
            layer.norm1b.copy_(get(p + "norm1b").float().reshape(()))
            layer.ls1.copy_(get(p + "ls1").float())
            layer.attn.load(get, p + "mix.")
            if layer.mlp is not None:
                layer.norm2.copy_(get(p + "norm2").float().reshape(()))
                layer.norm2b.copy_(get(p + "norm2b").float().reshape(()))
                layer.ls2.copy_(get(p + "ls2").float())
                layer.mlp.load(get, p + "mlp.")
        self._finish_load()

    def num_parameters(self) -> int:
        return sum(p.numel() for p in self.parameters())
