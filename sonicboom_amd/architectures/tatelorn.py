"""The Tatelorn decoder as a model spec.

A list of layers that read the residual stream as it is and norm what their sublayers give back:

    x += un(mixer(x), norm1);   x += un(ff(x), norm2)      (layers without a feed-forward stop after the first)

* un: RMS norm whose file weight is the multiplier minus one, v / sqrt(mean(v^2) + eps) * (1 + w) (``parts/norm.py``
  with an offset of 1);
* the stream starts as un(table[token] * embedding.scale + pos[position]) (``parts/embedding.py``,
  the ``positional`` kind);
* mixer ``attention`` (``parts/attention.py``): no biases, no rotation, every head of q and k
  normed with a plain weight that the heads share, values of their own size, scores times ``scale``
  then capped by a tanh, a sink in the softmax, and values mixed with those of the first layer
  whose configuration says ``v_mix``;
* feed-forward ``dense``: W_down (relu(W_gate f) * W_up f) (``parts/ffn.py``); ``moe``: routed
  experts with a clamped swish pair, and an expert that every token takes (``parts/moe.py``);
* the head is the embedding table (unscaled) after the model's norm, times ``logit_scale``.

Tensor names: ``embed``, ``pos``, ``embed.norm``, ``final.norm``, and per layer i ``l<i>.norm1``,
``l<i>.norm2``, ``l<i>.mix.<role>``, ``l<i>.mlp.<role>``.
"""
from __future__ import annotations

from ..config.registry import register_architecture
from ..config.tatelorn import DenseFFConfig, MoEFFConfig, TatelornConfig
from ..parts.attention import attention_spec
from ..parts.block import outnorm_block_spec
from ..parts.embedding import head_spec, positional_embedding_spec
from ..parts.ffn import gated_ffn_spec
from ..parts.moe import moe_ffn_spec
from ..parts.norm import rmsnorm_spec
from ..parts.spec import ModelSpec, OrderEntry, PartSpec

EMBED = "embed"
SWISH_ALPHA = 1.702        # the experts' g sigmoid(alpha g)
MIX_NAMES = {"q_weight": "q", "k_weight": "k", "v_weight": "v", "o_weight": "o", "q_norm": "q.norm", "k_norm": "k.norm",
             "value_mix": "vmix"}


def build_spec(cfg: TatelornConfig) -> ModelSpec:
    d = cfg.width

    def norm(name):
        return rmsnorm_spec(name, d, cfg.norm_eps, offset=1.0)

    blocks, order, ignorable = [], [], []
    mixing = False
    for i, layer in enumerate(cfg.layers):
        p, mx = f"l{i}.", layer.mixer
        value_mix = None
        if mx.v_mix:
            value_mix = "mix" if mixing else "first"
            mixing = True
        else:
            ignorable.append(p + "mix.vmix")
        mixer = attention_spec(p + "mix.", d, mx.heads, mx.kv_heads, mx.dim, PartSpec("position", "none"),
                               scale=mx.scale, qkv_bias=False, v_dim=mx.vdim, qk_norm=True, qk_norm_eps=cfg.norm_eps,
                               softcap=mx.softcap, sink=True, value_mix=value_mix, names=MIX_NAMES)
        order.append(OrderEntry(block=i, cache=i))
        ffn = ffn_norm = None
        f = layer.mlp
        if isinstance(f, DenseFFConfig):
            ffn = gated_ffn_spec(p + "mlp.", d, f.ff, activation="relu", names=("gate", "up", "down"))
        elif isinstance(f, MoEFFConfig):
            ffn = moe_ffn_spec(p + "mlp.", d, f.experts, f.top, f.ff, f.limit, SWISH_ALPHA, f.shared_ff, f.shared_limit)
        if ffn is not None:
            ffn_norm = norm(p + "norm2")
        else:
            ignorable.append(p + "norm2")
        blocks.append(outnorm_block_spec(norm(p + "norm1"), mixer, ffn_norm, ffn))
    spec = ModelSpec(
        architecture=cfg.architecture, width=d, vocab=cfg.vocab,
        embedding=positional_embedding_spec(EMBED, cfg.vocab, d, cfg.embedding_scale, "pos", cfg.max_positions,
                                            "embed.norm", cfg.norm_eps, 1.0),
        blocks=blocks, order=order,
        final_norm=norm("final.norm"),
        head=head_spec(EMBED, cfg.vocab, d, scale=cfg.logit_scale),
        max_positions=cfg.max_positions,
        stop_tokens=tuple(cfg.eos_token_ids),
        ignorable_tensors=tuple(ignorable),
    )
    spec.validate()
    return spec


register_architecture("Tatelorn", TatelornConfig, build_spec)
