"""Dedelorn: the description of the design in parts.

A decoder whose layers are listed one by one in config.json.  Every layer is a parallel block (one RMS norm, the
mixer and the feed-forward both read it, both results are added to the stream) around one of two mixers, a gated
delta rule (state per request) or windowed latent attention (paged cache; a layer may read an earlier layer's
cache instead of keeping one), and one of two feed-forwards, a dense gated one with the tanh form of GELU or
routed experts, or none.  The embedding is RMS-normed before the first layer.

Tensor names: ``embed``, ``embed.norm``, ``l<i>.norm1``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>`` (experts
``l<i>.mlp.e<j>.up`` / ``.down``), ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, ScheduleStep
from ..config.model_config import DedelornConfig
from ..config.registry import register_architecture


def _mixer(cfg: DedelornConfig, i: int) -> PartSpec:
    layer, p = cfg.layers[i], f"l{i}.mix."
    m = layer["mixer"]
    if layer["type"] == "delta":
        return PartSpec(
            "gated_delta_rule",
            {"hidden_size": cfg.hidden_size, "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "dim": int(m["dim"]),
             "vdim": int(m["vdim"]), "conv": int(m["conv"]), "eps": cfg.norm_eps},
            {"q": p + "q", "q_conv": p + "q.conv", "k": p + "k", "k_conv": p + "k.conv", "v": p + "v",
             "v_conv": p + "v.conv", "b": p + "b", "a": p + "a", "A_log": p + "A_log", "dt_bias": p + "dt_bias",
             "norm": p + "norm", "g": p + "g", "o": p + "o"})
    rot = int(m["rot_dim"])
    shares = m.get("kv_from") is not None
    position = PartSpec("rope_pairs", {"head_dim": rot, "rotary_dim": int(m["rot"]["dims"]), "theta": float(m["rot"]["base"])})
    names = {"q": p + "q", "uk": p + "uk", "uv": p + "uv", "o": p + "o"}
    if not shares:
        names.update({"dkv": p + "dkv", "dkv_norm": p + "dkv.norm"})
    return PartSpec(
        "latent_attention",
        {"hidden_size": cfg.hidden_size, "heads": int(m["heads"]), "dim": int(m["dim"]), "rot_dim": rot,
         "vdim": int(m["vdim"]), "kv_rank": int(m["kv_rank"]), "scale": float(m["scale"]),
         "window": int((m.get("mask") or {}).get("size", 0)), "eps": cfg.norm_eps, "shares_cache": shares,
         "position": position},
        names)


def _feed_forward(cfg: DedelornConfig, i: int) -> PartSpec:
    mlp, p = cfg.layers[i].get("mlp"), f"l{i}.mlp."
    if mlp is None:
        return PartSpec("none")
    if mlp["kind"] == "dense":
        return PartSpec("gated_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": int(mlp["ff"]),
                                      "activation": "gelu_tanh"},
                        {"gate": p + "gate", "up": p + "up", "down": p + "down"})
    E = int(mlp["router"]["experts"])
    names = {"router": p + "router", "correction": p + "correction"}
    for e in range(E):
        names[f"up_{e}"] = f"{p}e{e}.up"
        names[f"down_{e}"] = f"{p}e{e}.down"
    return PartSpec("routed_experts", {"hidden_size": cfg.hidden_size, "experts": E, "top": int(mlp["router"]["top"]),
                                       "ff": int(mlp["expert"]["ff"]), "scale": float(mlp["router"].get("scale", 1.0))},
                    names)


def dedelorn_forward_config(cfg: DedelornConfig) -> ModelForwardConfig:
    H, eps = cfg.hidden_size, cfg.norm_eps
    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        norms = {"input": PartSpec("rmsnorm", {"dim": H, "eps": eps}, {"weight": f"l{i}.norm1"})}
        layers.append(LayerSpec("parallel", _mixer(cfg, i), _feed_forward(cfg, i), norms))
        src = layer["mixer"].get("kv_from") if layer["type"] == "latent_attention" else None
        # a layer that reads another layer's latents runs on that layer's cache and stores nothing
        schedule.append(ScheduleStep(layer=i, cache=i if src is None else int(src), writes_cache=src is None))
    fc = ModelForwardConfig(
        architecture="Dedelorn", hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H, "norm_eps": eps},
                           {"weight": "embed", "norm": "embed.norm"}),
        layers=tuple(layers), schedule=tuple(schedule),
        final_norm=PartSpec("rmsnorm", {"dim": H, "eps": eps}, {"weight": "final.norm"}),
        lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids, max_position_embeddings=0,
        family={"mixers": [layer["type"] for layer in cfg.layers], "norm_eps": eps})
    fc.validate()
    return fc


register_architecture("Dedelorn", DedelornConfig, dedelorn_forward_config, aliases=("dedelorn",))
