"""``Samovik``: how its configuration turns into layers.

A decoder whose layers differ: each has one of three mixers (attention over a compressed latent,
linear attention with a decay per head, time mixing with a data-dependent decay), a routed
feed-forward with a shared expert (or none), Dynamic Tanh where other models have norms, and a
per-layer input from the token ids at its end.  Tensor names: ``embed``, ``side.embed``,
``l<i>.norm1`` / ``.norm2`` (with ``.b`` and ``.alpha``), ``l<i>.mix.*``, ``l<i>.mlp.*``,
``l<i>.side.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from tensorline_amd.config.registry import Architecture, register_architecture
from tensorline_amd.config.samovik_config import SamovikConfig
from tensorline_amd.parts.spec import LayerSpec, ModelSpec, PartSpec


def _mixer(kind: str, m: dict, eps: float) -> PartSpec:
    if kind == "latent_attention":
        return PartSpec("latent_attention", {
            "heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"], "kv_rank": m["kv_rank"],
            "scale": m["scale"], "rot": m["rot"], "eps": eps}, prefix="mix.")
    if kind == "lightning":
        return PartSpec("lightning_attention", {"heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"],
                                                "decay": tuple(m["decay"]), "eps": eps}, prefix="mix.")
    if "decay_rank" not in m:
        raise ValueError("a wkv mixer's decay_rank is not known: read the configuration with the checkpoint's shapes "
                         "(load_model_config) or name it")
    return PartSpec("wkv", {"heads": m["heads"], "dim": m["dim"], "decay_rank": m["decay_rank"], "eps": eps}, prefix="mix.")


def samovik_spec(cfg: SamovikConfig) -> ModelSpec:
    layers = []
    for i, layer in enumerate(cfg.layers):
        mlp = layer.get("mlp")
        ffn = None
        if mlp is not None:
            ffn = PartSpec("routed_experts", {
                "experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "ff": mlp["expert"]["ff"],
                "limit": mlp["expert"]["limit"], "shared": mlp.get("shared") or None}, prefix="mlp.")
        side = None
        if cfg.token_side_dim:
            side = PartSpec("gated_token_slice", {
                "table": "side.embed", "vocab_size": cfg.vocab_size, "dim": cfg.token_side_dim, "index": i,
                "slices": len(cfg.layers), "eps": cfg.norm_eps}, prefix="side.")
        layers.append(LayerSpec(
            prefix=f"l{i}.", mixer=_mixer(layer["type"], layer["mixer"], cfg.norm_eps), feed_forward=ffn,
            mixer_norm=PartSpec("dyt", {"name": "norm1"}),
            feed_forward_norm=PartSpec("dyt", {"name": "norm2"}) if ffn is not None else None,
            block="prenorm_token_input", token_input=side))
    spec = ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token_embedding", {"name": "embed"}),
        layers=tuple(layers),
        final_norm=PartSpec("dyt", {"name": "final.norm"}),
        head=PartSpec("lm_head", {"name": "head", "tied": False}),
        max_position=cfg.max_position_embeddings, eos_token_ids=tuple(cfg.eos_token_id))
    spec.validate()
    return spec


SAMOVIK = register_architecture(Architecture("Samovik", SamovikConfig, samovik_spec), replace=True)
