"""``Sugosun``: a decoder of linear-attention and latent-attention layers over several residual
streams, put together from parts.

The embedding adds a row of a hashed table of token pairs to the token's row and norms the sum.
Every layer is a pre-norm block with RMSNorm; the mixer is lightning attention (retention with SiLU
on q, k and v, the heads' read-outs normed together and a sigmoid gate) or latent attention (keys and
values from one cached latent a token, a rotated key part shared by the heads, a sliding window),
layer by layer as config.json lists them; the feed-forward is a gated one with both branches clamped,
a set of routed experts, or absent.  With ``streams`` the layers keep that many copies of the residual
stream and every sublayer has connection weights (``prenorm_streams``); without, the plain sum.
A span of layers may run several times in a row with the same weights; every pass is an entry of
the run order with a cache and state of its own.
Tensors: ``embed``, ``bigram``, ``embed.norm``, ``l<i>.norm1``/``norm2``, ``l<i>.hc1.*``/``hc2.*``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config import ExecStep, LayerSpec, ModelSpec, PartSpec, register_architecture
from ..config.sugosun import SugosunConfig


def _mixer_spec(cfg: SugosunConfig, i: int, prefix: str) -> PartSpec:
    m = cfg.layers[i].mixer
    E = cfg.width
    if m.kind == "lightning":
        return PartSpec("retention", {
            "hidden_size": E, "num_heads": m.heads, "head_dim": m.dim, "v_head_dim": m.vdim, "decay": list(m.decay),
            "eps": cfg.eps, "qkv_activation": "silu", "key_scale": 1.0, "norm_over": "row", "norm_name": "norm",
            "gate_activation": "sigmoid"}, prefix=prefix)
    return PartSpec("latent_attention", {
        "hidden_size": E, "num_heads": m.heads, "head_dim": m.dim, "rot_dim": m.rot_dim, "v_head_dim": m.vdim,
        "q_rank": m.q_rank, "kv_rank": m.kv_rank, "scale": m.scale, "eps": cfg.eps, "rot_dims": m.rot_dims,
        "rot_base": m.rot_base, "window": m.window}, prefix=prefix)


def _mlp_spec(cfg: SugosunConfig, i: int, prefix: str):
    mlp = cfg.layers[i].mlp
    if mlp is None:
        return None
    if mlp.kind == "dense":
        return PartSpec("gated_mlp", {
            "hidden_size": cfg.width, "intermediate_size": mlp.ff, "activation": "clamped_swish", "activation_param": mlp.limit,
            "gate_name": "gate", "up_name": "up", "down_name": "down", "weight_suffix": ""}, prefix=prefix)
    return PartSpec("routed_experts", {
        "hidden_size": cfg.width, "intermediate_size": mlp.ff, "num_experts": mlp.experts, "top": mlp.top}, prefix=prefix)


def build_sugosun_spec(cfg: SugosunConfig) -> ModelSpec:
    E, S = cfg.width, cfg.streams
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        has_ff = layer.mlp is not None

        def norm(name, optional=False):
            return PartSpec("rmsnorm", {"size": E, "eps": cfg.eps, "weight_name": name, "optional": optional}, prefix=p)

        def connection(name, optional=False):
            return PartSpec("stream_connection", {"streams": S, "optional": optional}, prefix=p + name + ".")

        # a layer without a feed-forward has no use for its second norm and connection; a file may still bring them
        layers.append(LayerSpec(
            mixer=_mixer_spec(cfg, i, p + "mix."), feed_forward=_mlp_spec(cfg, i, p + "mlp."),
            norms={"mixer_norm": norm("norm1"), "feed_forward_norm": norm("norm2", optional=not has_ff)},
            connections=({"mixer_connection": connection("hc1"), "feed_forward_connection": connection("hc2", optional=not has_ff)}
                         if S is not None else {}),
            block="prenorm_streams" if S is not None else "prenorm_optional"))
    big = cfg.bigram
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=E, vocab_size=cfg.vocab, max_position=cfg.max_position,
        embedding=PartSpec("pair_hash_embedding", {
            "vocab_size": cfg.vocab, "hidden_size": E, "buckets": big.buckets if big else 0,
            "mul_prev": big.mul_prev if big else 0, "mul_cur": big.mul_cur if big else 0, "eps": cfg.eps,
            "weight_name": "embed", "pairs_name": "bigram", "norm_name": "embed.norm"}),
        layers=layers, order=[ExecStep(i) for i in cfg.run_order()],
        final_norm=PartSpec("rmsnorm", {"size": E, "eps": cfg.eps, "weight_name": "norm"}, prefix="final."),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": E, "tied": False, "weight_name": "head"}),
        streams=S)


register_architecture("Sugosun", SugosunConfig.from_dict, build_sugosun_spec)
