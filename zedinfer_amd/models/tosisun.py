"""Tosisun: the description of the design in parts.

A decoder whose layers are listed one by one in config.json.  Every layer adds the layer-normed OUTPUT of its
sublayers to the stream, x <- x + LN1(mixer(x)), x <- x + LN2(ff(x)), and the sublayers read the stream itself.  The
mixer is grouped-query attention whose q/k/v projections (with biases) pass a short causal convolution, an RMS norm
over the whole of q and of k, and a rotation of the first dims of every head with stretched long wavelengths; its
softmax has a learned sink per head.  The feed-forward is dense, down(relu(up x)^2), or a mixture of clamped gated
experts chosen by their router logits, with a shared expert; or none.  A layer may run with an earlier layer's
tensors and a cache and state of its own.  The logits pass a layer norm, the head and a soft cap.

Tensor names: ``embed``, ``l<i>.norm1`` / ``.norm2`` (biases with ``.b`` added), ``l<i>.mix.q`` / ``.k`` / ``.v``
(``.b``, ``.conv``, ``.norm`` added), ``l<i>.mix.sink``, ``l<i>.mix.o``, ``l<i>.mlp.up`` / ``.down``, experts
``l<i>.mlp.e<j>.gate`` / ``.up`` / ``.down``, ``l<i>.mlp.router`` (``.b``), ``l<i>.mlp.shared.*``, ``final.norm``
(``.b``), ``head``.
"""
from __future__ import annotations

from ..config.forward_config import LayerSpec, ModelForwardConfig, PartSpec, ScheduleStep
from ..config.model_config import TosisunConfig
from ..config.registry import register_architecture


def _mixer(cfg: TosisunConfig, i: int) -> PartSpec:
    m, p = cfg.layers[i]["mixer"], f"l{i}.mix."
    rot = m["rot"]
    dims = int(rot["dims"])
    if dims:
        position = PartSpec("rope_neox", {"head_dim": int(m["dim"]), "rotary_dim": dims, "theta": float(rot["base"]),
                                          "scaling": dict(rot["scaling"]) if rot.get("scaling") else None})
    else:
        position = PartSpec("none")
    names = {"o": p + "o", "sink": p + "sink"}
    for x in ("q", "k", "v"):
        names.update({x: p + x, x + "_bias": p + x + ".b", x + "_conv": p + x + ".conv"})
    names.update({"q_norm": p + "q.norm", "k_norm": p + "k.norm"})
    return PartSpec(
        "conv_attention",
        {"hidden_size": cfg.hidden_size, "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]),
         "head_dim": int(m["dim"]), "value_dim": int(m["vdim"]), "conv": int(m["conv"]), "scale": float(m["scale"]),
         "eps": cfg.norm_eps, "position": position},
        names)


def _feed_forward(cfg: TosisunConfig, i: int) -> PartSpec:
    mlp, p = cfg.layers[i].get("mlp"), f"l{i}.mlp."
    if mlp is None:
        return PartSpec("none")
    if mlp["kind"] == "dense":
        return PartSpec("relu2_mlp", {"hidden_size": cfg.hidden_size, "intermediate_size": int(mlp["ff"])},
                        {"up": p + "up", "down": p + "down"})
    E = int(mlp["router"]["experts"])
    names = {"router": p + "router", "router_bias": p + "router.b"}
    for e in range(E):
        names.update({f"gate_{e}": f"{p}e{e}.gate", f"up_{e}": f"{p}e{e}.up", f"down_{e}": f"{p}e{e}.down"})
    sh = mlp.get("shared")
    if sh is not None:
        names.update({"shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down"})
    return PartSpec("clamped_experts",
                    {"hidden_size": cfg.hidden_size, "experts": E, "top": int(mlp["router"]["top"]),
                     "ff": int(mlp["expert"]["ff"]), "limit": float(mlp["expert"]["limit"]),
                     "shared_ff": int(sh["ff"]) if sh is not None else 0,
                     "shared_limit": float(sh["limit"]) if sh is not None else 0.0},
                    names)


def _norm(cfg: TosisunConfig, name: str) -> PartSpec:
    return PartSpec("layernorm", {"dim": cfg.hidden_size, "eps": cfg.norm_eps}, {"weight": name, "bias": name + ".b"})


def tosisun_forward_config(cfg: TosisunConfig) -> ModelForwardConfig:
    H = cfg.hidden_size
    layers, schedule, built = [], [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.get("weights_of") is None:
            built[i] = len(layers)
            layers.append(LayerSpec("output_norm", _mixer(cfg, i), _feed_forward(cfg, i),
                                    {"mixer_out": _norm(cfg, f"l{i}.norm1"), "ff_out": _norm(cfg, f"l{i}.norm2")}))
    for i in range(len(cfg.layers)):
        # a layer that runs with another's tensors is that layer's parts once more, on a cache and state of its own
        schedule.append(ScheduleStep(layer=built[cfg.owner_of(i)], cache=i))
    fc = ModelForwardConfig(
        architecture="Tosisun", hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("token", {"vocab_size": cfg.vocab_size, "hidden_size": H}, {"weight": "embed"}),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=_norm(cfg, "final.norm"),
        lm_head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H, "tied_to": None,
                                    "softcap": cfg.logit_softcap or None}, {"weight": "head"}),
        eos_token_ids=cfg.eos_token_ids, max_position_embeddings=0,
        family={"mixers": [cfg.layers[cfg.owner_of(i)]["type"] for i in range(len(cfg.layers))], "norm_eps": cfg.norm_eps})
    fc.validate()
    return fc


register_architecture("Tosisun", TosisunConfig, tosisun_forward_config, aliases=("tosisun",))
