"""``Kegorax``: a decoder whose layers run two mixers side by side or a gated delta rule, put together from parts.

The embedding's rows are scaled by a constant.  Every layer is pre-norm (RMS norms with plain weights):
``x += mixer(norm1(x)); x += feed_forward(norm2(x))``, the feed-forward optional.  Mixers by ``type``:

* "parallel": attention (grouped key/value heads, a rotation of the first channels of every head in the
  rotate-half layout, a mask of chunks counted from position 0, a learned sink a head in the softmax's
  denominator, a sigmoid gate a head on the output) beside gated linear attention (a decay a token and key
  channel, ``sigmoid(z)^(1/tau)``); each side's result is RMS-normed over the model's width with a weight of
  its own, and the mixer's result is half their sum: what this design fixes.
* "parallel_2": attention with biased projections, queries and keys normed head by head, no rotation, a bias
  ``2^(-8 (h + 1) / H) (i - j)`` on the scores, a sliding window that keeps the first tokens, and one added to
  the softmax's denominator, beside retention (a fixed decay a head); the result is a weighted sum of the two
  with the configuration's weights.
* "channel_delta": the gated delta rule with a decay a head and key channel through two thin factors, short
  convolutions on q, k and v, and a sigmoid gate through two thin factors.

The feed-forward is dense and gated with the tanh form of GELU, or a set of SiLU-gated experts chosen by
sigmoid scores with a correction, limited to the best groups, weighted by score times a constant.  A span of
layers may run several times in a row with the same weights, each pass with a cache and state of its own: before
every pass but the first the embedding's rows are added again, and before every pass a vector of that pass.
The head is the embedding table itself, without the embedding's scale.
Tensors: ``embed``, ``loop.step``, ``l<i>.norm1``/``norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``.
"""
from __future__ import annotations

from ..config import ExecStep, LayerSpec, ModelSpec, PartSpec, register_architecture
from ..config.kegorax import KegoraxConfig

SLOPE_EXPONENT = 8.0        # head h of H: 2^(-8 (h + 1) / H)
PARALLEL_WEIGHT = 0.5       # a "parallel" mixer is half the sum of its normed sides


def distance_slopes(heads: int):
    return [2.0 ** (-SLOPE_EXPONENT * (h + 1) / heads) for h in range(heads)]


def _attention(cfg: KegoraxConfig, a, **more) -> PartSpec:
    return PartSpec("paged_attention", dict({
        "hidden_size": cfg.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
        "v_head_dim": a.vdim, "scale": a.scale, "out_bias": False, "q_name": "q", "k_name": "k", "v_name": "v",
        "o_name": "o", "weight_suffix": "", "bias_suffix": ".b"}, **more))


def _mixer_spec(cfg: KegoraxConfig, i: int, prefix: str) -> PartSpec:
    m = cfg.layers[i].mixer
    E, r = cfg.width, cfg.layers[i].mixer.right
    if m.kind == "channel_delta":
        return PartSpec("gated_delta", {
            "hidden_size": E, "num_heads": r.heads, "num_kv_heads": r.kv_heads, "head_dim": r.dim, "v_head_dim": r.vdim,
            "conv_taps": r.conv, "eps": cfg.eps, "decay": "channel", "gate": "low_rank", "gate_activation": "sigmoid"},
            prefix=prefix)
    a = m.left
    if m.kind == "parallel":
        position = (PartSpec("rotary", {"head_dim": a.dim, "theta": a.rot_base, "rotary_dim": a.rot_dims})
                    if a.rot_dims else None)
        left = _attention(cfg, a, bias=False, position=position, chunk=a.mask_size, sink="learned", sink_name="sink",
                          gate_name="g")
        right = PartSpec("gated_linear_attention", {"hidden_size": E, "num_heads": r.heads, "head_dim": r.dim,
                                                    "v_head_dim": r.vdim, "tau": r.tau, "eps": cfg.eps})
        return PartSpec("parallel_mixers", {"hidden_size": E, "left": left, "right": right, "left_scale": PARALLEL_WEIGHT,
                                            "right_scale": PARALLEL_WEIGHT, "out_norm": True, "eps": cfg.eps}, prefix=prefix)
    left = _attention(cfg, a, bias=True, window=a.mask_size, keep_first=a.keep_first, sink="zero",
                      slopes=distance_slopes(a.heads),
                      qk_transform=PartSpec("head_rmsnorm", {"head_dim": a.dim, "eps": cfg.eps, "q_name": "q.norm",
                                                             "k_name": "k.norm"}))
    right = PartSpec("retention", {"hidden_size": E, "num_heads": r.heads, "head_dim": r.dim, "v_head_dim": r.vdim,
                                   "decay": list(r.decay), "eps": cfg.eps})
    return PartSpec("parallel_mixers", {"hidden_size": E, "left": left, "right": right, "left_scale": m.left_scale,
                                        "right_scale": m.right_scale}, prefix=prefix)


def _mlp_spec(cfg: KegoraxConfig, i: int, prefix: str):
    mlp = cfg.layers[i].mlp
    if mlp is None:
        return None
    if mlp.kind == "dense":
        return PartSpec("gated_mlp", {"hidden_size": cfg.width, "intermediate_size": mlp.ff, "activation": "gelu_tanh",
                                      "gate_name": "gate", "up_name": "up", "down_name": "down", "weight_suffix": ""},
                        prefix=prefix)
    return PartSpec("routed_experts", {
        "hidden_size": cfg.width, "intermediate_size": mlp.ff, "num_experts": mlp.experts, "top": mlp.top,
        "activation": "swiglu", "scores": "sigmoid", "groups": mlp.groups, "keep_groups": mlp.keep_groups,
        "weight_scale": mlp.scale}, prefix=prefix)


def build_kegorax_spec(cfg: KegoraxConfig) -> ModelSpec:
    E = cfg.width
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        has_ff = layer.mlp is not None

        def norm(name, optional=False):
            return PartSpec("rmsnorm", {"size": E, "eps": cfg.eps, "weight_name": name, "optional": optional}, prefix=p)

        layers.append(LayerSpec(
            mixer=_mixer_spec(cfg, i, p + "mix."), feed_forward=_mlp_spec(cfg, i, p + "mlp."),
            norms={"mixer_norm": norm("norm1"), "feed_forward_norm": norm("norm2", optional=not has_ff)},
            block="prenorm_optional"))
    order = [ExecStep(i, enters=t is not None, pass_index=t or 0) for i, t in cfg.run_order()]
    return ModelSpec(
        architecture=cfg.architecture, hidden_size=E, vocab_size=cfg.vocab, max_position=cfg.max_position,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": E, "scale": cfg.embedding_scale,
                                               "weight_name": "embed"}),
        layers=layers, order=order,
        final_norm=PartSpec("rmsnorm", {"size": E, "eps": cfg.eps, "weight_name": "norm"}, prefix="final."),
        head=PartSpec("linear", {"vocab_size": cfg.vocab, "hidden_size": E, "tied": True}),
        injection=(PartSpec("step_addition", {"hidden_size": E, "passes": cfg.loop[2], "weight_name": "step"}, prefix="loop.")
                   if cfg.loop is not None else None))


register_architecture("Kegorax", KegoraxConfig.from_dict, build_kegorax_spec)
