"""``Suripel``: a decoder whose layers mix time in three ways, put together from parts.

Every layer is a pre-norm block with LayerNorm (a weight, no bias) whose sublayers read their
input through a short causal convolution added to it (``prenorm_filtered``); the mixer is
sliding-window attention with pooled blocks, a gated delta rule or retention, layer by layer as
config.json lists them; the feed-forward is dense with the PolyNorm activation, or absent.
Tensors: ``embed``, ``l<i>.norm1``/``norm2``, ``l<i>.canon1``/``canon2``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``.

An attention layer with ``kv_from`` reads the cache of the layer it names (``ExecStep.cache_of``);
the owner's cache then reaches back as far as the longest reach among its readers.
"""
from __future__ import annotations

from ..config import ExecStep, LayerSpec, ModelSpec, PartSpec, register_architecture
from ..config.suripel import SuripelConfig


def _mixer_spec(cfg: SuripelConfig, i: int, prefix: str) -> PartSpec:
    m = cfg.layers[i].mixer
    E = cfg.width
    if m.kind == "attention":
        owner = i if m.kv_from is None else m.kv_from
        family = [l.mixer for j, l in enumerate(cfg.layers)
                  if l.mixer.kind == "attention" and (j == owner or l.mixer.kv_from == owner)]
        keep = max(max(x.window, x.pool) for x in family)
        return PartSpec("pooled_window_attention", {
            "hidden_size": E, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim,
            "window": m.window, "pool": m.pool, "scale": m.scale, "conv_taps": m.conv, "keep": keep,
            "kv_shared": m.kv_from is not None}, prefix=prefix)
    if m.kind == "delta":
        return PartSpec("gated_delta", {
            "hidden_size": E, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "v_head_dim": m.vdim,
            "conv_taps": m.conv, "eps": cfg.eps}, prefix=prefix)
    position = None
    if m.rot_dims:
        position = PartSpec("rotary", {"head_dim": m.dim, "theta": m.rot_base, "rotary_dim": m.rot_dims})
    return PartSpec("retention", {
        "hidden_size": E, "num_heads": m.heads, "head_dim": m.dim, "v_head_dim": m.vdim, "decay": list(m.decay),
        "eps": cfg.eps, "position": position}, prefix=prefix)


def build_suripel_spec(cfg: SuripelConfig) -> ModelSpec:
    E = cfg.width
    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        has_ff = layer.ff is not None

        def norm(name, optional=False):
            # 32-bit rows: the convolution behind the norm carries them from token to token
            return PartSpec("layernorm", {"size": E, "eps": cfg.eps, "weight_name": name, "out_dtype": "float32",
                                          "optional": optional}, prefix=p)

        def canon(name, optional=False):
            return PartSpec("causal_conv", {"channels": E, "taps": cfg.canon_taps, "residual": True, "weight_name": name,
                                            "optional": optional}, prefix=p)

        layers.append(LayerSpec(
            mixer=_mixer_spec(cfg, i, p + "mix."),
            feed_forward=PartSpec("dense_mlp", {"hidden_size": E, "intermediate_size": layer.ff, "activation": "polynorm",
                                                "eps": cfg.eps}, prefix=p + "mlp.") if has_ff else None,
            # a layer without a feed-forward has no use for its second norm and filter; a file may still bring them
            norms={"mixer_norm": norm("norm1"), "feed_forward_norm": norm("norm2", optional=not has_ff)},
            filters={"mixer_filter": canon("canon1"), "feed_forward_filter": canon("canon2", optional=not has_ff)},
            block="prenorm_filtered"))
        order.append(ExecStep(i, cache_of=layer.mixer.kv_from))
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=E, vocab_size=cfg.vocab, max_position=cfg.max_position,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": E, "weight_name": "embed"}),
        layers=layers, order=order,
        final_norm=PartSpec("layernorm", {"size": E, "eps": cfg.eps, "weight_name": "norm"}, prefix="final."),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": E, "tied": False, "weight_name": "head"}))


register_architecture("Suripel", SuripelConfig.from_dict, build_suripel_spec)
