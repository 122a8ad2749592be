"""Sigosun: a decoder whose layers each name their own mixer, assembled from parts by its config.

Per layer the norm sits on the sublayer's output only (`OutputNormBlock`; weights stored around zero). Mixers:
softmax attention under a block mask with per-head q/k norm, a rotation of the first dimensions of each head in
adjacent pairs, grouped key/value heads of their own value size, a sigmoid gate per head, and optionally the keys
and values of an earlier layer in place of its own (`Attention`); a selective state-space recurrence
(`SelectiveStateSpace`); linear attention with one decay per head (`LinearAttention`). A layer may have a dense
feed-forward with a squared-relu activation. A final norm of the same kind, then the head.

Checkpoint names: `embed`, `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.<tensor>`, `l<i>.mlp.up|down`, `final.norm`, `head`.
"""
from __future__ import annotations

from ..config.model_config import SigosunConfig
from ..parts.base import LayerCall, make_part
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import register_architecture
from .model import DecoderModel, WeightSource


def _kernel_head_size(dim: int, vdim: int) -> int:
    """One head size for keys and values: the larger of the two, in whole steps of 16 (what the matrix-core
    attention kernels take)."""
    return -(-max(dim, vdim) // 16) * 16


@register_architecture("Sigosun")
def build_sigosun(cfg: SigosunConfig) -> DecoderModel:
    h, eps = cfg.hidden_size, cfg.norm_eps
    norm = lambda: make_part("norm", "rms", size=h, eps=eps, one_plus=True)
    layers, order, sources = [], [], {}
    rotations: dict = {}                      # layers with equal rotations share one table
    for i, layer in enumerate(cfg.layers):
        m, ck, me = layer.mixer, f"l{i}.mix.", f"layers.{i}.mixer."
        if layer.kind == "attention":
            own = m["kv_from"] is None
            D = _kernel_head_size(m["dim"], m["vdim"])
            key = (D, m["dim"], m["rot_dims"], m["rot_base"])
            if key not in rotations:
                rotations[key] = make_part("position_encoding", "rotary", head_dim=D, theta=m["rot_base"], stored_dim=m["dim"],
                                           rotary_dims=m["rot_dims"], interleaved=True, exact_angles=True)
            mixer = make_part("mixer", "attention", hidden_size=h, num_heads=m["heads"], num_kv_heads=m["kv_heads"],
                              head_dim=m["dim"], value_dim=m["vdim"], scale=m["scale"], qk_norm_eps=eps,
                              position=rotations[key], chunk=m["mask_size"], head_gate=True, own_kv=own)
            q, k, v = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            blocks = [WeightSource(ck + "q", 0, q)]
            if own:
                blocks += [WeightSource(ck + "k", q, k), WeightSource(ck + "v", q + k, v)]
                sources[me + "k_norm_weight"] = [WeightSource(ck + "k.norm")]
            blocks.append(WeightSource(ck + "g", q + (k + v if own else 0), m["heads"]))
            sources[me + "qkv.weight"] = blocks
            sources[me + "q_norm_weight"] = [WeightSource(ck + "q.norm")]
            sources[me + "o.weight"] = [WeightSource(ck + "o")]
            order.append(LayerCall(i, cache_of=m["kv_from"]))
        elif layer.kind == "mamba2":
            mixer = make_part("mixer", "mamba2", hidden_size=h, num_heads=m["heads"], value_dim=m["vdim"], state_dim=m["state"],
                              groups=m["groups"], taps=m["conv"], norm_groups=m["norm_groups"], norm_eps=eps)
            for mine, stored in (("in_proj.weight", "in"), ("conv_weight", "conv"), ("conv_bias", "conv.b"), ("dt_bias", "dt_bias"),
                                 ("A_log", "A_log"), ("D", "D"), ("norm_weight", "norm"), ("o.weight", "o")):
                sources[me + mine] = [WeightSource(ck + stored)]
            order.append(LayerCall(i))
        else:
            mixer = make_part("mixer", "lightning", hidden_size=h, num_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"],
                              decay=m["decay"], norm_eps=eps)
            qk, inner = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            sources[me + "qkvg.weight"] = [WeightSource(ck + "q", 0, qk), WeightSource(ck + "k", qk, qk),
                                           WeightSource(ck + "v", 2 * qk, inner), WeightSource(ck + "g", 2 * qk + inner, inner)]
            sources[me + "norm_weight"] = [WeightSource(ck + "norm")]
            sources[me + "o.weight"] = [WeightSource(ck + "o")]
            order.append(LayerCall(i))
        ffn = norm2 = None
        if layer.ff is not None:
            ffn, norm2 = make_part("feed_forward", "dense", hidden_size=h, intermediate_size=layer.ff, activation="relu2"), norm()
            sources[f"layers.{i}.norm2.weight"] = [WeightSource(f"l{i}.norm2")]
            sources[f"layers.{i}.feed_forward.up.weight"] = [WeightSource(f"l{i}.mlp.up")]
            sources[f"layers.{i}.feed_forward.down.weight"] = [WeightSource(f"l{i}.mlp.down")]
        layers.append(make_part("block", "output_norm", norm1=norm(), mixer=mixer, norm2=norm2, feed_forward=ffn))
        sources[f"layers.{i}.norm1.weight"] = [WeightSource(f"l{i}.norm1")]
    embedding = TokenEmbedding(cfg.vocab_size, h)
    head = LMHead(cfg.vocab_size, h)
    sources["embedding.weight"] = [WeightSource("embed")]
    sources["final_norm.weight"] = [WeightSource("final.norm")]
    sources["head.weight"] = [WeightSource("head")]
    return DecoderModel(cfg, embedding, layers, order, norm(), head, sources)
