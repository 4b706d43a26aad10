"""Sequence mixers and feed-forwards for models with a 32-bit residual stream.

Each module owns its weights and runs one sublayer on a flat token batch
``[T, width]`` in the activation dtype (bf16 or fp32). Matrix products go to
the vendor GEMM; everything around them is a HIP kernel from ``kserve_amd.ops``
(CPU tensors take the plain torch forms). Small vectors that enter fp32
arithmetic (norm weights, convolution taps, decay and step parameters) are
kept in fp32 regardless of the activation dtype.

Per-step inputs come from ``AttentionMetadata``: besides the paged-KV fields
they need ``cu_seqlens`` / ``seq_of_token`` (flat-batch layout) and
``state_slots`` (one row of the recurrent-state pools per sequence).
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kserve_amd import ops
from kserve_amd.engine.config import AttentionMixerSpec, GLUSpec, SSMMixerSpec


class LayerCache(NamedTuple):
    """What one layer keeps between steps; absent parts are None."""

    k: Optional[torch.Tensor] = None      # [blocks, kv_heads, block, dim]
    v: Optional[torch.Tensor] = None      # [blocks, kv_heads, block, vdim]
    conv: Optional[torch.Tensor] = None   # [slots, taps-1, channels]
    ssm: Optional[torch.Tensor] = None    # [slots, heads, vdim, state] fp32


def _param(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


class SSDMixer(nn.Module):
    """State-space sublayer (Mamba-2 form): in-projection to
    [z | x | B | C | dt], causal conv + silu over x|B|C, the scan, a gated
    grouped RMS norm, out-projection."""

    def __init__(self, width: int, spec: SSMMixerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        self.in_proj = _param(spec.proj_width, width, dtype=dtype)
        self.conv_w = _param(spec.conv_channels, spec.conv, dtype=torch.float32)
        self.conv_b = _param(spec.conv_channels, dtype=torch.float32)
        self.dt_bias = _param(spec.heads, dtype=torch.float32)
        self.a_log = _param(spec.heads, dtype=torch.float32)
        self.d_skip = _param(spec.heads, dtype=torch.float32)
        self.norm_w = _param(spec.inner, dtype=torch.float32)
        self.o_proj = _param(width, spec.inner, dtype=dtype)

    def state_shapes(self):
        s = self.spec
        return {
            "conv": ((max(s.conv - 1, 1), s.conv_channels), self.dtype),
            "ssm": ((s.heads, s.vdim, s.state), torch.float32),
        }

    def load(self, get, prefix: str):
        self.in_proj.copy_(get(prefix + "in").to(self.dtype))
        self.conv_w.copy_(get(prefix + "conv").float())
        self.conv_b.copy_(get(prefix + "conv.b").float())
        self.dt_bias.copy_(get(prefix + "dt_bias").float())
        self.a_log.copy_(get(prefix + "A_log").float())
        self.d_skip.copy_(get(prefix + "D").float())
        self.norm_w.copy_(get(prefix + "norm").float())
        self.o_proj.copy_(get(prefix + "o").to(self.dtype))

    def mix(self, proj, positions, cache: LayerCache, meta):
        """``proj``: [T, proj_width] rows of this mixer's in-projection (may be
        a column slice of a wider fused projection)."""
        s = self.spec
        z = proj[:, : s.inner]
        xbc_raw = proj[:, s.inner : s.inner + s.conv_channels]
        dt_raw = proj[:, s.inner + s.conv_channels :]
        xbc = ops.causal_conv_silu(
            xbc_raw, self.conv_w, self.conv_b, cache.conv, positions,
            meta.seq_of_token, meta.cu_seqlens, meta.state_slots,
        )
        y = ops.ssd_scan(
            xbc, dt_raw, self.dt_bias, self.a_log, self.d_skip, cache.ssm,
            positions, meta.cu_seqlens, meta.state_slots, s.groups,
        )
        yn = ops.gated_group_rms_norm(
            y, z, self.norm_w, self.eps, s.norm_groups, self.dtype
        )
        return F.linear(yn, self.o_proj)

    def forward(self, h, positions, cache: LayerCache, meta):
        return self.mix(F.linear(h, self.in_proj), positions, cache, meta)


class NormedGatedAttention(nn.Module):
    """Causal softmax attention without rotation: biased q/k/v projections,
    RMS norm over the whole q (and k) projection, a position-dependent query
    temperature, fp32 scores against the paged cache, a sigmoid output gate
    per head read from the sublayer input, out-projection. The q|k|v|gate
    projections are one fused GEMM."""

    def __init__(self, width: int, spec: AttentionMixerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        self.q_w = spec.heads * spec.dim
        self.k_w = spec.kv_heads * spec.dim
        self.v_w = spec.kv_heads * spec.vdim
        self.proj_width = self.q_w + self.k_w + self.v_w + spec.heads
        self.qkvg = _param(self.proj_width, width, dtype=dtype)
        self.qkvg_bias = _param(self.proj_width, dtype=dtype)
        self.q_norm = _param(self.q_w, dtype=torch.float32)
        self.k_norm = _param(self.k_w, dtype=torch.float32)
        self.o_proj = _param(width, spec.heads * spec.vdim, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.dtype
        w = torch.cat(
            [get(prefix + n).to(dt) for n in ("q", "k", "v", "g")], dim=0
        )
        b = torch.cat(
            [get(prefix + n + ".b").to(dt) for n in ("q", "k", "v")]
            + [torch.zeros(self.spec.heads, dtype=dt)]
        )
        self.qkvg.copy_(w)
        self.qkvg_bias.copy_(b)
        self.q_norm.copy_(get(prefix + "q.norm").float())
        self.k_norm.copy_(get(prefix + "k.norm").float())
        self.o_proj.copy_(get(prefix + "o").to(dt))

    def mix(self, proj, positions, cache: LayerCache, meta):
        s = self.spec
        a, b, c = self.q_w, self.q_w + self.k_w, self.q_w + self.k_w + self.v_w
        q, k, v, gate = proj[:, :a], proj[:, a:b], proj[:, b:c], proj[:, c:]
        qn = ops.qk_norm_temp_cache(
            q, k, v, self.q_norm, self.k_norm, positions, meta.slot_mapping,
            cache.k, cache.v, self.eps, s.q_temp_coef, s.q_temp_every, s.heads,
        )
        o = ops.ctx_attention_f32(
            qn, cache.k, cache.v, meta.block_tables, meta.cu_seqlens,
            meta.context_lens, s.scale, meta.max_seqlen, s.heads, gate=gate,
            out_dtype=self.dtype,
        )
        return F.linear(o, self.o_proj)

    def forward(self, h, positions, cache: LayerCache, meta):
        return self.mix(
            F.linear(h, self.qkvg, self.qkvg_bias), positions, cache, meta
        )


class ClampedGLU(nn.Module):
    """y = g * sigmoid(alpha g) * (u + 1), g = min(W_gate h, limit),
    u = clamp(W_up h, -limit, limit); gate|up are one fused GEMM."""

    ALPHA = 1.702

    def __init__(self, width: int, spec: GLUSpec, dtype):
        super().__init__()
        self.spec = spec
        self.gate_up = _param(2 * spec.ff, width, dtype=dtype)
        self.down = _param(width, spec.ff, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.gate_up.dtype
        self.gate_up.copy_(
            torch.cat([get(prefix + "gate").to(dt), get(prefix + "up").to(dt)], dim=0)
        )
        self.down.copy_(get(prefix + "down").to(dt))

    def forward(self, h):
        act = ops.clamped_swiglu(
            F.linear(h, self.gate_up), self.ALPHA, self.spec.limit
        )
        return F.linear(act, self.down)
