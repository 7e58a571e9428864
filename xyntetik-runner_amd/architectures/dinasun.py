"""``Dinasun``: a decoder of time-mixing and attention layers whose sublayers are normed before and
after by dynamic tanh, put together from parts.

The embedding's rows are scaled by a constant.  Every layer is a "sandwich" block:
``x += m post(mixer(pre(x))); x += m post'(feed_forward(pre'(x)))`` with dynamic tanh for all four norms
and one factor ``m`` for the model.  The mixer is wkv time mixing (a decay a token, head and key channel;
mixes of every row with the row before it) or attention whose values are its keys as projected, with
queries and keys normed head by head, a query temperature that grows with the position, no rotation, and a
bias on the scores that grows with the distance: ``2^(-8 (h + 1) / H) (i - j)`` for head h of H, which is
what this design fixes.  The feed-forward is a set of gated experts chosen by a stored table from the
token's id, each with the weight 1 / top, plus a shared expert; a layer may have none.  A span of layers
may run several times in a row with the same weights: every pass is entered through ``x <- W [x; x0]``
(``x0``: the embedding's rows) and has a cache and state of its own.  The head is the embedding table
itself, without the embedding's scale.
Tensors: ``embed``, ``loop.in``, ``l<i>.norm1``/``norm1b``/``norm2``/``norm2b`` (each with ``.b`` and ``.alpha``),
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``.
"""
from __future__ import annotations

from ..config import ExecStep, LayerSpec, ModelSpec, PartSpec, register_architecture
from ..config.dinasun import DinasunConfig

SLOPE_EXPONENT = 8.0        # head h of H: 2^(-8 (h + 1) / H)


def distance_slopes(heads: int):
    return [2.0 ** (-SLOPE_EXPONENT * (h + 1) / heads) for h in range(heads)]


def _mixer_spec(cfg: DinasunConfig, i: int, prefix: str) -> PartSpec:
    m = cfg.layers[i].mixer
    E = cfg.width
    if m.kind == "wkv":
        return PartSpec("wkv_time_mix", {"hidden_size": E, "num_heads": m.heads, "head_dim": m.dim, "eps": cfg.eps}, prefix=prefix)
    return PartSpec("paged_attention", {
        "hidden_size": E, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "scale": m.scale,
        "bias": True, "out_bias": False, "values": "keys", "slopes": distance_slopes(m.heads),
        "q_name": "q", "k_name": "k", "o_name": "o", "weight_suffix": "", "bias_suffix": ".b",
        "qk_transform": PartSpec("head_rmsnorm", {"head_dim": m.dim, "eps": cfg.eps, "q_name": "q.norm", "k_name": "k.norm",
                                                  "temp_coef": m.temp_coef, "temp_every": m.temp_every})}, prefix=prefix)


def _mlp_spec(cfg: DinasunConfig, i: int, prefix: str):
    mlp = cfg.layers[i].mlp
    if mlp is None:
        return None
    return PartSpec("routed_experts", {
        "hidden_size": cfg.width, "intermediate_size": mlp.ff, "num_experts": mlp.experts, "top": mlp.top,
        "activation": "swiglu", "routing": "table", "vocab_size": cfg.vocab, "shared_size": mlp.shared_ff}, prefix=prefix)


def build_dinasun_spec(cfg: DinasunConfig) -> ModelSpec:
    E = cfg.width
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        has_ff = layer.mlp is not None

        def norm(name, optional=False, out_dtype="compute"):
            return PartSpec("dynamic_tanh", {"size": E, "weight_name": name, "optional": optional, "out_dtype": out_dtype}, prefix=p)

        # time mixing forms its mixes of a row and the row before in 32 bits: its input is not rounded on the way
        layers.append(LayerSpec(
            mixer=_mixer_spec(cfg, i, p + "mix."), feed_forward=_mlp_spec(cfg, i, p + "mlp."),
            norms={"mixer_norm": norm("norm1", out_dtype="float32" if layer.mixer.kind == "wkv" else "compute"),
                   "mixer_post_norm": norm("norm1b"),
                   "feed_forward_norm": norm("norm2", optional=not has_ff),
                   "feed_forward_post_norm": norm("norm2b", optional=not has_ff)},
            block="sandwich", block_params={"residual_mult": cfg.residual_mult}))
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=E, vocab_size=cfg.vocab, max_position=cfg.max_position,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": E, "scale": cfg.embedding_scale,
                                               "weight_name": "embed"}),
        layers=layers, order=[ExecStep(i, enters=enters) for i, enters in cfg.run_order()],
        final_norm=PartSpec("dynamic_tanh", {"size": E, "weight_name": "norm"}, prefix="final."),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": E, "tied": True}),
        injection=(PartSpec("concat_projection", {"hidden_size": E, "weight_name": "in"}, prefix="loop.")
                   if cfg.loop is not None else None))


register_architecture("Dinasun", DinasunConfig.from_dict, build_dinasun_spec)
