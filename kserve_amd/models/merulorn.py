"""Merulorn: a decoder whose layers are listed one by one in the config.

A layer is pre-norm: x += mixer(norm1(x)), then (if it has one)
x += ff(norm2(x)). Mixers are a state-space sublayer alone ("mamba2") or an
attention sublayer beside a state-space one, both reading the same normed
input, their outputs added with fixed scales ("parallel"). Norm weights are
stored around zero and applied as (1 + w). The embedding is scaled and gets
interleaved sinusoidal positions; there is no rotation inside attention.

The residual stream is fp32 whatever the activation dtype; every
"add the sublayer's output, norm for the next sublayer" pair is one kernel,
and a parallel mixer runs ONE projection GEMM for both of its branches.
"""

from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kserve_amd import ops
from kserve_amd.engine.config import HybridLayerSpec, HybridModelConfig
from kserve_amd.models.mixers import (
    ClampedGLU,
    LayerCache,
    NormedGatedAttention,
    SSDMixer,
)
from kserve_amd.ops.torch_ref import sinusoid_inv_freq
from kserve_amd.parallel import comm


class MerulornLayer(nn.Module):
    def __init__(self, width: int, spec: HybridLayerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        self.norm1 = nn.Parameter(
            torch.empty(width, dtype=torch.float32), requires_grad=False
        )
        self.attn = (
            NormedGatedAttention(width, spec.attention, eps, dtype)
            if spec.attention is not None
            else None
        )
        self.ssm = SSDMixer(width, spec.ssm, eps, dtype) if spec.ssm is not None else None
        self.mlp = ClampedGLU(width, spec.mlp, dtype) if spec.mlp is not None else None
        self.norm2 = (
            nn.Parameter(torch.empty(width, dtype=torch.float32), requires_grad=False)
            if self.mlp is not None
            else None
        )
        # both branches read the same input: fuse their projections
        self.fused_proj = None
        self.fused_bias = None

    def finish_load(self):
        if self.attn is not None and self.ssm is not None:
            self.fused_proj = nn.Parameter(
                torch.cat([self.attn.qkvg.data, self.ssm.in_proj.data], dim=0),
                requires_grad=False,
            )
            self.fused_bias = nn.Parameter(
                torch.cat(
                    [
                        self.attn.qkvg_bias.data,
                        torch.zeros(
                            self.ssm.spec.proj_width,
                            dtype=self.dtype,
                            device=self.attn.qkvg_bias.device,
                        ),
                    ]
                ),
                requires_grad=False,
            )
            # the branch modules keep views of the fused storage
            a = self.attn.proj_width
            self.attn.qkvg.data = self.fused_proj.data[:a]
            self.attn.qkvg_bias.data = self.fused_bias.data[:a]
            self.ssm.in_proj.data = self.fused_proj.data[a:]

    def mixer(self, h, positions, cache: LayerCache, meta):
        """Returns (delta0, scale0, delta1, scale1) to add to the stream."""
        if self.attn is not None and self.ssm is not None:
            proj = F.linear(h, self.fused_proj, self.fused_bias)
            a = self.attn.proj_width
            left = self.attn.mix(proj[:, :a], positions, cache, meta)
            right = self.ssm.mix(proj[:, a:], positions, cache, meta)
            return left, self.spec.attention_scale, right, self.spec.ssm_scale
        if self.ssm is not None:
            return self.ssm(h, positions, cache, meta), 1.0, None, 1.0
        return self.attn(h, positions, cache, meta), 1.0, None, 1.0


class MerulornForCausalLM(nn.Module):
    # every step attends through the paged cache (no separate un-paged
    # prefill kernel), and steps carry per-sequence state slots
    paged_prefill_only = True
    needs_state_slots = True

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
                "Merulorn runs on one GPU per replica (no tensor/pipeline split)"
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
            [MerulornLayer(W, spec, config.rms_norm_eps, dtype) for spec in config.layers]
        )
        self.num_local_layers = len(self.layers)
        self.final_norm = nn.Parameter(
            torch.empty(W, dtype=torch.float32), requires_grad=False
        )
        self.head = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.register_buffer("inv_freq", sinusoid_inv_freq(W), persistent=False)
        self.eps = config.rms_norm_eps
        # when a list, forward() appends the residual stream after each layer
        self.debug_residuals: Optional[List[torch.Tensor]] = None
        self.to(device)

    # -- cache layout (read by the model runner) ------------------------------
    def cache_layout(self):
        """Per layer: (kv_heads, dim, vdim) or None, and
        {name: (shape_per_slot, dtype)} of recurrent state or {}."""
        out = []
        for layer in self.layers:
            a = layer.spec.attention
            kv = (a.kv_heads, a.dim, a.vdim) if a is not None else None
            state = layer.ssm.state_shapes() if layer.ssm is not None else {}
            out.append((kv, state))
        return out

    # -- init -----------------------------------------------------------------
    @torch.no_grad()
    def random_init(self, std: float = 0.02, seed: int = 0):
        dev = self.embed.device
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        for name, p in self.named_parameters():
            if "fused_" in name:
                continue
            leaf = name.rsplit(".", 1)[-1]
            if p.dim() >= 2 and leaf != "conv_w":
                # keep activations O(1) through the stack
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)
            elif leaf == "conv_w":
                p.normal_(0.0, 0.5, generator=gen)
            elif leaf in ("q_norm", "k_norm", "norm_w"):
                p.fill_(1.0)
            elif leaf == "a_log":
                p.uniform_(-1.0, 1.0, generator=gen)
            elif leaf == "d_skip":
                p.fill_(1.0)
            elif leaf == "dt_bias":
                p.uniform_(-3.0, 0.0, generator=gen)
            else:
                p.normal_(0.0, 0.1, generator=gen)
        for layer in self.layers:
            layer.finish_load()
        return self

    # -- forward --------------------------------------------------------------
    def forward(self, input_ids, positions, caches, meta):
        x = ops.embed_scale_sinpos(
            self.embed, input_ids, positions, self.inv_freq,
            self.config.embedding_scale,
        )
        pending = (None, 1.0, None, 1.0)
        dbg = self.debug_residuals
        for layer, cache in zip(self.layers, caches):
            h = self._add_norm(x, layer.norm1, pending)
            pending = layer.mixer(h, positions, cache, meta)
            if layer.mlp is not None:
                h = self._add_norm(x, layer.norm2, pending)
                pending = (layer.mlp(h), 1.0, None, 1.0)
            if dbg is not None:
                r = x.clone()
                for d, s in ((pending[0], pending[1]), (pending[2], pending[3])):
                    if d is not None:
                        r += s * d.float()
                dbg.append(r)
        return self._add_norm(x, self.final_norm, pending)

    def _add_norm(self, x, weight, pending):
        d0, s0, d1, s1 = pending
        return ops.add_rms_norm_f32res(
            x, weight, self.eps, 1.0, self.dtype, d0, s0, d1, s1
        )

    def compute_logits(self, hidden):
        return F.linear(hidden, self.head)

    # -- weights ----------------------------------------------------------------
    @torch.no_grad()
    def load_hf_state_dict(self, tensors) -> None:
        """Tensor names: embed, l<i>.norm1|norm2, l<i>.mix.* (or
        l<i>.mix.left.* / l<i>.mix.right.* in a parallel mixer),
        l<i>.mlp.gate|up|down, final.norm, head."""

        def get(name):
            t = tensors[name]
            return t() if callable(t) else t

        self.embed.copy_(get("embed").to(self.dtype))
        self.head.copy_(get("head").to(self.dtype))
        self.final_norm.copy_(get("final.norm").float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.copy_(get(p + "norm1").float())
            if layer.attn is not None and layer.ssm is not None:
                layer.attn.load(get, p + "mix.left.")
                layer.ssm.load(get, p + "mix.right.")
            elif layer.ssm is not None:
                layer.ssm.load(get, p + "mix.")
            else:
                layer.attn.load(get, p + "mix.")
            if layer.mlp is not None:
                layer.norm2.copy_(get(p + "norm2").float())
                layer.mlp.load(get, p + "mlp.")
            layer.finish_load()

    def num_parameters(self) -> int:
        return sum(
            p.numel() for n, p in self.named_parameters() if "fused_" not in n
        )
