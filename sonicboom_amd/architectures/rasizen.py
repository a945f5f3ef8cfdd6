"""The Rasizen decoder as a model spec.

A list of pre-norm layers, each with one mixer and at most one feed-forward, every branch
multiplied by ``residual_mult`` before it joins the stream:

    x += m * mixer(norm1(x));   x += m * ff(norm2(x))   (layers without a feed-forward stop after the first)

* norms: RMS norm taken over ``norm.groups`` equal consecutive parts of the row, one weight over
  the whole row (``parts/norm.py``);
* mixer ``mingru``: a gated recurrence with a float32 state per sequence (``parts/recurrent.py``);
* mixer ``latent_attention``: attention over a cached latent row per token, rotated key part shared
  by the heads, neighbouring-pair rotation, sliding window, sigmoid output gate
  (``parts/latent_attention.py``); a layer with ``kv_from`` reads the rows of that earlier layer:
  its order entry names the other's cache and does not write it;
* feed-forward ``dense``: W_down xIELU(W_up h) with the layer's two numbers (``parts/ffn.py``);
* the head is the embedding table, after the model's norm.

Tensor names: ``embed``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.<role>``, ``l<i>.mlp.<role>``.
"""
from __future__ import annotations

from ..config.rasizen import LatentAttentionConfig, MinGRUConfig, RasizenConfig
from ..config.registry import register_architecture
from ..parts.block import prenorm_block_spec
from ..parts.embedding import embedding_spec, head_spec
from ..parts.ffn import dense_ffn_spec
from ..parts.latent_attention import latent_attention_spec
from ..parts.norm import rmsnorm_spec
from ..parts.position import rope_interleaved_spec
from ..parts.recurrent import mingru_spec
from ..parts.spec import ModelSpec, OrderEntry, PartSpec

EMBED = "embed"


def build_spec(cfg: RasizenConfig) -> ModelSpec:
    d, m = cfg.width, cfg.residual_mult

    def norm(name):
        return rmsnorm_spec(name, d, cfg.norm_eps, cfg.norm_groups)

    blocks, order = [], []
    for i, layer in enumerate(cfg.layers):
        p, mx = f"l{i}.", layer.mixer
        if isinstance(mx, MinGRUConfig):
            mixer = mingru_spec(p + "mix.", d, mx.width, out_scale=m)
            order.append(OrderEntry(block=i, cache=None))
        elif isinstance(mx, LatentAttentionConfig):
            position = rope_interleaved_spec(mx.rot_dims, mx.rot_base) if mx.rot_dims else PartSpec("position", "none")
            own = mx.kv_from is None
            mixer = latent_attention_spec(p + "mix.", d, mx.heads, mx.dim, mx.rot_dim, mx.vdim, mx.kv_rank, mx.scale,
                                          position, window=mx.window, eps=cfg.norm_eps, own_latent=own, out_scale=m)
            order.append(OrderEntry(block=i, cache=i if own else mx.kv_from, writes_cache=own))
        else:
            raise ValueError(f"layer {i}: no mixer for {layer.type!r}")
        ffn = ffn_norm = None
        if layer.mlp is not None:
            ffn_norm = norm(p + "norm2")
            ffn = dense_ffn_spec(p + "mlp.up", p + "mlp.down", d, layer.mlp.ff, "xielu", act_name=p + "mlp.act",
                                 out_scale=m)
        blocks.append(prenorm_block_spec(norm(p + "norm1"), mixer, ffn_norm, ffn))
    spec = ModelSpec(
        architecture=cfg.architecture, width=d, vocab=cfg.vocab,
        embedding=embedding_spec(EMBED, cfg.vocab, d),
        blocks=blocks, order=order,
        final_norm=norm("final.norm"),
        head=head_spec(EMBED, cfg.vocab, d),
        max_positions=0,
        stop_tokens=tuple(cfg.eos_token_ids),
    )
    spec.validate()
    return spec


register_architecture("Rasizen", RasizenConfig, build_spec)
