"""Negosun: a decoder whose layers run attention and a feed-forward of routed experts side by side, assembled from parts.

Per layer both sublayers read the same stream, each through an RMS norm of its own; their outputs are multiplied
element by element by learned scales and added to the stream under one multiplier (`ParallelBlock`). Attention has
biases on q, k and v, norms q and k over the whole projection, knows positions only through a query temperature that
grows with their logarithm, and, in layers that say so, blends its values with those the first such layer made for
the same token before caching them (`Attention` with its prologue options). The feed-forward chooses a few of many
small gated experts per token, optionally only among the best groups of neighbours, beside an optional expert every
token passes (`RoutedExperts`, `SwiGLU`). A final norm, then the embedding matrix as the head, with an optional soft
cap on the logits.

Checkpoint names: `embed`, `l<i>.norm1|norm2|ls1|ls2`, `l<i>.mix.q|k|v|o` with `.b` and `.norm` behind q, k (and v for
the bias), `l<i>.mix.vmix`, `l<i>.mlp.router`, `l<i>.mlp.e<j>.gate|up|down`, `l<i>.mlp.shared.gate|up|down`, `final.norm`.
"""
from __future__ import annotations

from ..config.model_config import NegosunConfig
from ..parts.base import LayerCall, make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import register_architecture
from .model import DecoderModel, WeightSource


@register_architecture("Negosun")
def build_negosun(cfg: NegosunConfig) -> DecoderModel:
    h, eps = cfg.hidden_size, cfg.norm_eps
    norm = lambda: make_part("norm", "rms", size=h, eps=eps)
    layers, sources, optional = [], {}, set()
    first_mixed = None                        # the first layer with value mixing: the others blend with its values
    for i, layer in enumerate(cfg.layers):
        m, ck, me = layer.mixer, f"l{i}.mix.", f"layers.{i}.mixer."
        mix = None
        if m["v_mix"]:
            mix = "first" if first_mixed is None else "blend"
            first_mixed = i if first_mixed is None else first_mixed
        mixer = make_part("mixer", "attention", hidden_size=h, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"],
                          value_dim=m["vdim"], scale=m["scale"], qk_norm_eps=eps, qk_norm_over="projection", qkv_bias=True,
                          q_temperature=None if m["temp_every"] is None else (m["temp_coef"], m["temp_every"]), value_mix=mix)
        q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
        sources[me + "qkv.weight"] = [WeightSource(ck + "q", 0, q), WeightSource(ck + "k", q, k), WeightSource(ck + "v", q + k, v)]
        sources[me + "qkv_bias"] = [WeightSource(ck + "q.b", 0, q), WeightSource(ck + "k.b", q, k), WeightSource(ck + "v.b", q + k, v)]
        sources[me + "q_norm_weight"] = [WeightSource(ck + "q.norm")]
        sources[me + "k_norm_weight"] = [WeightSource(ck + "k.norm")]
        sources[me + "o.weight"] = [WeightSource(ck + "o")]
        if mix == "blend":
            sources[me + "vmix"] = [WeightSource(ck + "vmix")]
        else:
            optional.add(ck + "vmix")          # stored for every layer, used from the second mixing layer on
        ffn = norm2 = None
        f = layer.mlp
        if f is not None:
            shared = None
            ck, me = f"l{i}.mlp.", f"layers.{i}.feed_forward."
            if f["shared_ff"] is not None:
                shared = make_part("feed_forward", "swiglu", hidden_size=h, intermediate_size=f["shared_ff"])
                sources[me + "shared.gate_up.weight"] = [WeightSource(ck + "shared.gate", 0, f["shared_ff"]),
                                                         WeightSource(ck + "shared.up", f["shared_ff"], f["shared_ff"])]
                sources[me + "shared.down.weight"] = [WeightSource(ck + "shared.down")]
            ffn = make_part("feed_forward", "moe", hidden_size=h, intermediate_size=f["ff"], num_experts=f["experts"], top=f["top"],
                            group_count=f["group_count"], group_keep=f["group_keep"], shared=shared)
            F = f["ff"]
            sources[me + "router"] = [WeightSource(ck + "router")]
            sources[me + "gate_up"] = [src for e in range(f["experts"])
                                       for src in (WeightSource(f"{ck}e{e}.gate", 2 * e * F, F), WeightSource(f"{ck}e{e}.up", (2 * e + 1) * F, F))]
            sources[me + "down"] = [WeightSource(f"{ck}e{e}.down", e * h, h) for e in range(f["experts"])]
            norm2 = norm()
            sources[f"layers.{i}.norm2.weight"] = [WeightSource(f"l{i}.norm2")]
            sources[f"layers.{i}.scale2"] = [WeightSource(f"l{i}.ls2")]
        else:
            optional.update((f"l{i}.norm2", f"l{i}.ls2"))
        layers.append(make_part("block", "parallel", norm1=norm(), mixer=mixer, norm2=norm2, feed_forward=ffn,
                                residual_mult=cfg.residual_mult, layer_scale=True))
        sources[f"layers.{i}.norm1.weight"] = [WeightSource(f"l{i}.norm1")]
        sources[f"layers.{i}.scale1"] = [WeightSource(f"l{i}.ls1")]
    embedding = TokenEmbedding(cfg.vocab_size, h)
    head = LMHead(cfg.vocab_size, h, tied_to=embedding, softcap=cfg.logit_softcap)
    sources["embedding.weight"] = [WeightSource("embed")]
    sources["final_norm.weight"] = [WeightSource("final.norm")]
    return DecoderModel(cfg, embedding, layers, [LayerCall(i) for i in range(len(layers))], norm(), head, sources, optional)
