"""``Tumitar``: how its configuration turns into layers and the order they run in.

A decoder with RMS pre-norms whose layers have one of two mixers: ``parallel`` (attention without
rotation, with normed queries and keys, a query factor that grows with the position and a softmax sink,
beside a Mamba-2 mixer; the layer's mixer output is a weighted sum of the two) or ``rglru`` (Griffin's
recurrent block).  Feed-forwards are dense with a squared relu, routed experts weighted by their own
sigmoid scores, or absent.  A run of layers may be looped: it runs several times with the same weights,
every pass with caches and states of its own, and from the second pass on the embedding output is added
to the stream in front of the run.  The head is the embedding table.  Tensor names: ``embed``,
``l<i>.norm1`` / ``.norm2``, ``l<i>.mix.*`` (``.left.*`` / ``.right.*`` in a parallel layer),
``l<i>.mlp.*``, ``final.norm``.
"""
from __future__ import annotations

from tensorline_amd.config.registry import Architecture, register_architecture
from tensorline_amd.config.tumitar_config import TumitarConfig
from tensorline_amd.parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _mixer(kind: str, m: dict, eps: float) -> PartSpec:
    if kind == "rglru":
        return PartSpec("rglru", {"width": m["width"], "blocks": m["blocks"], "conv": m["conv"]}, prefix="mix.")
    a, s = m["left"], m["right"]
    left = PartSpec("normed_attention", {
        "heads": a["heads"], "kv_heads": a["kv_heads"], "dim": a["dim"], "vdim": a["vdim"], "scale": a["scale"], "eps": eps,
        "bias": True, "qk_norm": True, "q_temp": a.get("q_temp"), "sink": True}, prefix="left.")
    right = PartSpec("ssd", {"heads": s["heads"], "vdim": s["vdim"], "state": s["state"], "groups": s["groups"],
                             "conv": s["conv"], "norm_groups": s["norm_groups"], "eps": eps}, prefix="right.")
    return PartSpec("parallel", {"left": left, "right": right, "left_scale": m["left_scale"],
                                 "right_scale": m["right_scale"]}, prefix="mix.")


def _feed_forward(mlp: dict | None) -> PartSpec | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartSpec("up_down", {"ff": mlp["ff"], "activation": "relu2"}, prefix="mlp.")
    return PartSpec("routed_experts", {
        "experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "ff": mlp["expert"]["ff"],
        "weighting": "sigmoid", "router_scale": mlp["router"]["scale"], "router_bias": False, "activation": "swiglu"},
        prefix="mlp.")


def tumitar_spec(cfg: TumitarConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        ffn = _feed_forward(layer.get("mlp"))
        layers.append(LayerSpec(
            prefix=f"l{i}.", mixer=_mixer(layer["type"], layer["mixer"], cfg.norm_eps), feed_forward=ffn,
            mixer_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "norm1"}),
            feed_forward_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "norm2"}) if ffn is not None else None,
            block="prenorm_token_input"))
    spec = ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"name": "embed", "scale": cfg.embedding_scale}),
        layers=tuple(layers),
        final_norm=PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": "final.norm"}),
        head=PartSpec("lm_head", {"name": "head", "tied": True}),
        schedule=tuple(ScheduleEntry(i, add_input=again) for i, again in cfg.run_order()),
        max_position=cfg.max_position_embeddings, eos_token_ids=tuple(cfg.eos_token_id))
    spec.validate()
    return spec


TUMITAR = register_architecture(Architecture("Tumitar", TumitarConfig, tumitar_spec), replace=True)
