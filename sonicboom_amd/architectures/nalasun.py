"""The Nalasun decoder as a model spec.

A list of pre-norm layers whose mixer reads the normed stream through a short convolution over time:

    h = rms(x, norm1);  h <- h + tconv(h, canon1);  x += mixer(h);  x += ff(rms(x, norm2))
    (layers without a feed-forward stop after the first)

* the stream starts as table[token] + pos[position] (``parts/embedding.py``, the ``positional`` kind
  without a norm);
* the block is the ``prenorm`` kind with a convolution on the mixer's input (``parts/block.py``);
* mixer ``mamba2``: the ``ssd`` part, ``channel_delta``: the part of that name (``parts/state_space.py``);
* mixer ``attention``: the ``shared_attention`` part (``parts/shared_attention.py``): biases on q and k, the values
  are the keys as projected, norms over the whole projections, a query temperature, a bias by the
  logarithm of the distance, and the heads' weights mixed by a matrix;
* feed-forward ``moe`` (``parts/moe.py``): sigmoid scores, the chosen experts' scores times
  ``router.scale`` as weights, SiLU-gated experts and an ungated shared expert;
* the head is the embedding table after the model's norm.

Tensor names: ``embed``, ``pos``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.canon1``, ``l<i>.mix.<role>``, ``l<i>.mlp.<role>``.
"""
from __future__ import annotations

from ..config.nalasun import NalasunConfig
from ..config.registry import register_architecture
from ..parts.block import prenorm_block_spec
from ..parts.embedding import head_spec, positional_embedding_spec
from ..parts.moe import moe_ffn_spec
from ..parts.norm import rmsnorm_spec
from ..parts.shared_attention import shared_attention_spec
from ..parts.spec import ModelSpec, OrderEntry
from ..parts.state_space import channel_delta_spec, ssd_spec

EMBED = "embed"


def build_spec(cfg: NalasunConfig) -> ModelSpec:
    d, eps = cfg.width, cfg.norm_eps
    blocks, order, ignorable = [], [], []
    for i, layer in enumerate(cfg.layers):
        p, mx = f"l{i}.", layer.mixer
        cache = None
        if layer.type == "mamba2":
            mixer = ssd_spec(p + "mix.", d, mx.heads, mx.vdim, mx.state, mx.groups, mx.conv, mx.norm_groups, eps)
        elif layer.type == "channel_delta":
            mixer = channel_delta_spec(p + "mix.", d, mx.heads, mx.kv_heads, mx.dim, mx.vdim, mx.conv, eps,
                                       decay_rank=mx.decay_rank, gate_rank=mx.gate_rank)
        else:
            mixer = shared_attention_spec(p + "mix.", d, mx.heads, mx.kv_heads, mx.dim, eps, scale=mx.scale,
                                          temp_coef=mx.temp_coef, temp_every=mx.temp_every)
            cache = i
        order.append(OrderEntry(block=i, cache=cache))
        ffn = ffn_norm = None
        f = layer.mlp
        if f is not None:
            ffn = moe_ffn_spec(p + "mlp.", d, f.experts, f.top, f.ff, 0.0, 1.0, f.shared_ff, 0.0, activation="silu",
                               router_score="sigmoid", router_scale=f.scale, shared_gate=False)
            ffn_norm = rmsnorm_spec(p + "norm2", d, eps)
        else:
            ignorable.append(p + "norm2")
        blocks.append(prenorm_block_spec(rmsnorm_spec(p + "norm1", d, eps), mixer, ffn_norm, ffn,
                                         input_conv_name=p + "canon1", input_taps=cfg.canon_taps, width=d))
    spec = ModelSpec(
        architecture=cfg.architecture, width=d, vocab=cfg.vocab,
        embedding=positional_embedding_spec(EMBED, cfg.vocab, d, 1.0, "pos", cfg.max_positions),
        blocks=blocks, order=order,
        final_norm=rmsnorm_spec("final.norm", d, eps),
        head=head_spec(EMBED, cfg.vocab, d),
        max_positions=cfg.max_positions,
        stop_tokens=tuple(cfg.eos_token_ids),
        ignorable_tensors=tuple(ignorable),
    )
    spec.validate()
    return spec


register_architecture("Nalasun", NalasunConfig, build_spec)
