"""The Fitatar decoder as a model spec.

A list of layers whose two branches read the same stream, each through a norm of its own:

    x += mixer(norm1(x)) + ff(norm2(x))        (layers without a feed-forward: the mixer's branch alone)

* the stream starts as table[token] * embedding.scale (``parts/embedding.py``);
* norms: RMS norm with a plain weight (``parts/norm.py``);
* mixer ``latent_attention`` (``parts/latent_attention.py``): queries through a normed latent of their
  own, keys and values from one cached latent row per token with a rotated key part that the heads
  share, neighbouring-pair rotation whose slow pairs are stretched with a ramp and whose cosines and
  sines carry a magnitude, a sigmoid output gate of one number a head; a layer with ``kv_from`` reads
  the rows of that earlier layer (its order entry names the other's cache and does not write it);
* mixer ``attention`` (``parts/attention.py``): grouped-query attention without biases, keys and values
  of sizes of their own, rotate-half rotation of the first ``rot.dims`` numbers with every frequency
  divided by a factor, a sink whose score is a number of the head's own, a sigmoid output gate number
  by number;
* feed-forward ``dense``: W_down gelu(W_up h + b) + b with the error-function gelu (``parts/ffn.py``);
  ``moe``: experts W_down max(W_up h, 0)^2 chosen by softmax scores within the best groups, weights not
  renormalized, plus a gated expert that every token takes (``parts/moe.py``);
* logits: the model's norm, the head's own matrix, then cap * tanh(logits / cap).

Tensor names: ``embed``, ``head``, ``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.<role>``, ``l<i>.mlp.<role>``.
"""
from __future__ import annotations

from ..config.fitatar import AttentionConfig, DenseFFConfig, FitatarConfig, LatentAttentionConfig, MoEFFConfig
from ..config.registry import register_architecture
from ..parts.attention import attention_spec
from ..parts.block import parallel_block_spec
from ..parts.embedding import head_spec, positional_embedding_spec
from ..parts.ffn import dense_ffn_spec
from ..parts.latent_attention import latent_attention_spec
from ..parts.moe import moe_ffn_spec
from ..parts.norm import rmsnorm_spec
from ..parts.position import rope_interleaved_spec, rope_spec, stretched_frequencies
from ..parts.spec import ModelSpec, OrderEntry, PartSpec

ATTENTION_NAMES = {"q_weight": "q", "k_weight": "k", "v_weight": "v", "o_weight": "o", "sink": "sink", "g_weight": "g"}


def _frequencies(rot, kind):
    """(frequencies, magnitude) of a layer's rotation; ``kind`` is what a factor means for this mixer."""
    if not rot.factor:
        return stretched_frequencies(rot.dims, rot.base)
    return stretched_frequencies(rot.dims, rot.base, kind, rot.factor, rot.original, rot.fast, rot.slow)


def build_spec(cfg: FitatarConfig) -> ModelSpec:
    d = cfg.width

    def norm(name):
        return rmsnorm_spec(name, d, cfg.norm_eps)

    blocks, order, ignorable = [], [], []
    for i, layer in enumerate(cfg.layers):
        p, mx = f"l{i}.", layer.mixer
        if isinstance(mx, LatentAttentionConfig):
            position = PartSpec("position", "none")
            if mx.rot.dims:
                freq, magnitude = _frequencies(mx.rot, "ramp")
                position = rope_interleaved_spec(mx.rot.dims, mx.rot.base, frequencies=freq, magnitude=magnitude)
            own = mx.kv_from is None
            mixer = latent_attention_spec(p + "mix.", d, mx.heads, mx.dim, mx.rot_dim, mx.vdim, mx.kv_rank, mx.scale,
                                          position, eps=cfg.norm_eps, own_latent=own, q_rank=mx.q_rank, gate_per_head=True)
            order.append(OrderEntry(block=i, cache=i if own else mx.kv_from, writes_cache=own))
        elif isinstance(mx, AttentionConfig):
            position = PartSpec("position", "none")
            if mx.rot.dims:
                freq, magnitude = _frequencies(mx.rot, "linear")
                position = rope_spec(mx.dim, mx.rot.base, rot_dims=mx.rot.dims, frequencies=freq, magnitude=magnitude)
            mixer = attention_spec(p + "mix.", d, mx.heads, mx.kv_heads, mx.dim, position, scale=mx.scale, qkv_bias=False,
                                   v_dim=mx.vdim, sink=True, sink_scores=True, out_gate=True, names=ATTENTION_NAMES)
            order.append(OrderEntry(block=i, cache=i))
        else:
            raise ValueError(f"layer {i}: no mixer for {layer.type!r}")
        ffn = ffn_norm = None
        f = layer.mlp
        if isinstance(f, DenseFFConfig):
            ffn = dense_ffn_spec(p + "mlp.up", p + "mlp.down", d, f.ff, "gelu_erf", up_bias_name=p + "mlp.up.b",
                                 down_bias_name=p + "mlp.down.b")
        elif isinstance(f, MoEFFConfig):
            ffn = moe_ffn_spec(p + "mlp.", d, f.experts, f.top, f.ff, 0.0, shared_inner=f.shared_ff, activation="relu_sq",
                               router_score="softmax_all", groups=f.groups, keep_groups=f.keep)
        if ffn is not None:
            ffn_norm = norm(p + "norm2")
        else:
            ignorable.append(p + "norm2")
        blocks.append(parallel_block_spec(norm(p + "norm1"), mixer, ffn_norm, ffn))
    spec = ModelSpec(
        architecture=cfg.architecture, width=d, vocab=cfg.vocab,
        embedding=positional_embedding_spec("embed", cfg.vocab, d, cfg.embedding_scale),
        blocks=blocks, order=order,
        final_norm=norm("final.norm"),
        head=head_spec("head", cfg.vocab, d, softcap=cfg.logit_softcap),
        max_positions=0,
        stop_tokens=tuple(cfg.eos_token_ids),
        ignorable_tensors=tuple(ignorable),
    )
    spec.validate()
    return spec


register_architecture("Fitatar", FitatarConfig, build_spec)
