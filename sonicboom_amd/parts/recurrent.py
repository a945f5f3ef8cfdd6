"""Gated recurrences: mixers whose memory of a sequence is one float32 vector.

``mingru``: the gates read the current token only,

    z_t = sigmoid(W_z h_t + b_z),  u_t = W_x h_t + b_x,
    cand_t = u_t + 1/2 where u_t >= 0, sigmoid(u_t) where u_t < 0,
    S_t = (1 - z_t) S_{t-1} + z_t cand_t   (element by element, S = 0 before the first token),
    x_t += out_scale * W_o (S_t * silu(W_g h_t)).

The three input projections are stacked into one matrix, so a step runs one product; its rows
leave in float32 and the scan kernel takes sigmoid, candidate, update and output gate from there in
float32.  The state is per-sequence state of the cache (one row per slot, zeroed when the slot is
handed out, moved on by every step), so prompts cut into steps, batches and decoding all run the
same recurrence.  In the 32-bit path every step runs the serial kernel, whose sums are those of
token-by-token decoding to the bit; in bfloat16 a step that brings a sequence more rows than a chunk
runs the chunked form.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Mixer, StateSpec, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec


def mingru_spec(prefix: str, width: int, inner: int, out_scale: float = 1.0) -> PartSpec:
    """Tensors ``<prefix>z``, ``z.b``, ``x``, ``x.b``, ``g``, ``o``."""
    return PartSpec("mixer", "mingru", {"width": width, "inner": inner, "out_scale": float(out_scale)}, {
        "z_weight": TensorSpec(prefix + "z", (inner, width)), "z_bias": TensorSpec(prefix + "z.b", (inner,)),
        "x_weight": TensorSpec(prefix + "x", (inner, width)), "x_bias": TensorSpec(prefix + "x.b", (inner,)),
        "g_weight": TensorSpec(prefix + "g", (inner, width)), "o_weight": TensorSpec(prefix + "o", (width, inner)),
    })


@register_part("mixer", "mingru")
class MinGRU(Mixer):
    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width, self.inner = int(p["width"]), int(p["inner"])
        self.out_scale = float(p.get("out_scale", 1.0))
        ws = [tensors["z_weight"], tensors["x_weight"], tensors["g_weight"]]
        if not all(w.dtype == ws[0].dtype for w in ws):
            ws = [w.float() for w in ws]
        bias = torch.cat([tensors["z_bias"].float(), tensors["x_bias"].float(),
                          torch.zeros(self.inner, dtype=torch.float32, device=ws[0].device)])
        self.zxg = Linear(torch.cat(ws, dim=0), bias, rt.fast_kernels)
        self.out = Linear(tensors["o_weight"], None, rt.fast_kernels)
        # the chunked form takes a step's rows in runs of this many (the context lists them)
        self.chunk = ops.mingru_chunk_rows() if rt.act_dtype != torch.float32 and ws[0].is_cuda else 0
        self.row_tile = self.chunk or None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.inner,), torch.float32)

    def forward(self, h, x, ctx, binding, then_norm=None):
        pre = self.zxg(h, torch.float32)                       # [rows, 3 * inner]: z | x | g before their activations
        chunks = ctx.row_tiles(self.chunk) if self.chunk and ctx.max_new > self.chunk else None
        y = ops.mingru_scan(pre, binding.state, ctx.cu_rows, ctx.slots, ctx.n_seqs, self.rt.act_dtype, chunks)
        return self.out.add_into(y, x, then_norm, self.rt.act_dtype, scale=self.out_scale)
