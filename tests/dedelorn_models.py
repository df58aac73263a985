"""Small Dedelorn configurations of the tests and their random weights.

The sizes differ from layer to layer and between the configurations in everything the format lets differ: heads
against q/k heads (equal, 3 and 4 to 1), dim against vdim against rot_dim, 2 to 5 convolution taps, one expert of
five and all three of three, a layer without a feed-forward, a layer that reads another layer's latents through
a wider window than its owner's, a layer that sees all keys, a width that is no multiple of 8.

Weights are drawn here (not by the engine's random-weights mode): wide enough that attention is peaked and the
router's choice close, with decays, step biases and router corrections that are not their neutral values."""
import json
import os

import torch

ALL = dict(
    architecture="Dedelorn", width=80, vocab=300, norm=dict(eps=2e-6),
    layers=[
        dict(type="latent_attention",
             mixer=dict(heads=3, dim=24, rot_dim=8, vdim=40, kv_rank=48, scale=0.19, mask=dict(size=20),
                        rot=dict(base=5000.0, dims=8)),
             mlp=dict(kind="moe", expert=dict(ff=56), router=dict(experts=6, top=3, scale=1.5))),
        dict(type="delta", mixer=dict(heads=6, kv_heads=2, dim=24, vdim=40, conv=4), mlp=dict(kind="dense", ff=104)),
        dict(type="latent_attention",
             mixer=dict(heads=5, dim=16, rot_dim=8, vdim=24, kv_rank=48, scale=0.3, mask=dict(size=33), kv_from=0,
                        rot=dict(base=5000.0, dims=8)),
             mlp=None),
        dict(type="delta", mixer=dict(heads=2, kv_heads=2, dim=40, vdim=16, conv=2),
             mlp=dict(kind="moe", expert=dict(ff=40), router=dict(experts=5, top=1, scale=1.0))),
    ])

LATENT_ONLY = dict(
    architecture="Dedelorn", width=64, vocab=200, norm=dict(eps=1e-5),
    layers=[
        dict(type="latent_attention",
             mixer=dict(heads=2, dim=16, rot_dim=16, vdim=16, kv_rank=32, scale=0.25, mask=dict(size=9),
                        rot=dict(base=100.0, dims=16)),
             mlp=dict(kind="dense", ff=96)),
        dict(type="latent_attention",
             mixer=dict(heads=4, dim=8, rot_dim=4, vdim=24, kv_rank=72, scale=0.4, rot=dict(base=30000.0, dims=4)),
             mlp=dict(kind="dense", ff=48)),
    ])

DELTA_ONLY = dict(
    architecture="Dedelorn", width=84, vocab=150, norm=dict(eps=1e-6),
    layers=[
        dict(type="delta", mixer=dict(heads=3, kv_heads=3, dim=72, vdim=20, conv=3), mlp=dict(kind="dense", ff=60)),
        dict(type="delta", mixer=dict(heads=4, kv_heads=1, dim=8, vdim=72, conv=5),
             mlp=dict(kind="moe", expert=dict(ff=36), router=dict(experts=3, top=3, scale=0.7))),
    ])

CONFIGS = {"all": ALL, "latent": LATENT_ONLY, "delta": DELTA_ONLY}


def tensor_shapes(cfg):
    """name -> shape of every tensor a model of ``cfg`` has."""
    W, out = cfg["width"], {}
    out["embed"], out["embed.norm"] = (cfg["vocab"], W), (W,)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (W,)
        if layer["type"] == "delta":
            qk, v = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            out.update({p + "mix.q": (qk, W), p + "mix.q.conv": (qk, m["conv"]), p + "mix.k": (qk, W),
                        p + "mix.k.conv": (qk, m["conv"]), p + "mix.v": (v, W), p + "mix.v.conv": (v, m["conv"]),
                        p + "mix.b": (m["heads"], W), p + "mix.a": (m["heads"], W), p + "mix.A_log": (m["heads"],),
                        p + "mix.dt_bias": (m["heads"],), p + "mix.norm": (m["vdim"],), p + "mix.g": (v, W),
                        p + "mix.o": (W, v)})
        else:
            H = m["heads"]
            out.update({p + "mix.q": (H * (m["dim"] + m["rot_dim"]), W), p + "mix.uk": (H * m["dim"], m["kv_rank"]),
                        p + "mix.uv": (H * m["vdim"], m["kv_rank"]), p + "mix.o": (W, H * m["vdim"])})
            if m.get("kv_from") is None:
                out.update({p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], W), p + "mix.dkv.norm": (m["kv_rank"],)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            out.update({p + "mlp.gate": (mlp["ff"], W), p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            out.update({p + "mlp.router": (E, W), p + "mlp.correction": (E,)})
            for e in range(E):
                out.update({f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
    out["final.norm"], out["head"] = (W,), (cfg["vocab"], W)
    return out


def make_weights(cfg, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if last in ("norm", "norm1"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif last in ("A_log", "dt_bias"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif last == "correction":
            t = 0.05 * torch.randn(shape, generator=g)
        elif last == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.0 / shape[-1] ** 0.5)
        w[name] = t.to(dtype)
    return w


def write_model(folder, name, seed=0, dtype=torch.float32):
    """config.json and model.safetensors of configuration ``name``; returns the folder."""
    from zedinfer_amd.weights.safetensors_io import write_safetensors
    cfg = CONFIGS[name]
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), make_weights(cfg, seed, dtype), metadata={"format": "pt"})
    return folder


def random_config(seed):
    """A configuration drawn at random: sizes, head counts, the order of layers, windows (from 1 key to more than a
    sequence), which layers read whose latents, rotation bases, taps, experts and how many are chosen, norm eps."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 64, 96, 128, 160])
    cfg = dict(architecture="Dedelorn", width=width, vocab=rng.choice([97, 256, 411]), norm=dict(eps=rng.choice([1e-6, 1e-5, 3e-6])),
               layers=[])
    owners = []                  # latent layers that keep a cache of their own
    for i in range(rng.randint(2, 6)):
        if rng.random() < 0.5:
            kvh = rng.choice([1, 2, 3])
            mixer = dict(heads=kvh * rng.choice([1, 2, 4]), kv_heads=kvh, dim=rng.choice([8, 16, 24, 40, 64, 96]),
                         vdim=rng.choice([8, 16, 24, 40, 64]), conv=rng.choice([1, 2, 3, 4, 6]))
            kind = "delta"
        else:
            kind = "latent_attention"
            if owners and rng.random() < 0.5:
                src = rng.choice(owners)
                o = cfg["layers"][src]["mixer"]
                mixer = dict(kv_rank=o["kv_rank"], rot_dim=o["rot_dim"], rot=dict(o["rot"]), kv_from=src)
            else:
                rot = rng.choice([2, 4, 8, 16, 24, 32])
                mixer = dict(kv_rank=rng.choice([16, 24, 40, 64, 96, 136]), rot_dim=rot,
                             rot=dict(base=rng.choice([50.0, 10000.0, 500000.0]), dims=rot))
                owners.append(i)
            mixer.update(heads=rng.choice([1, 2, 3, 5, 8, 17]), dim=rng.choice([8, 16, 24, 32, 48]), vdim=rng.choice([8, 16, 24, 40]),
                         scale=rng.choice([0.1, 0.25, 0.5]), mask=dict(size=rng.choice([1, 2, 7, 16, 31, 64, 100, 500])))
        r = rng.random()
        if r < 0.2:
            mlp = None
        elif r < 0.6:
            mlp = dict(kind="dense", ff=rng.choice([32, 72, 136]))
        else:
            experts = rng.choice([2, 4, 7, 16, 40])
            mlp = dict(kind="moe", expert=dict(ff=rng.choice([16, 40, 72])),
                       router=dict(experts=experts, top=rng.randint(1, min(experts, 6)), scale=rng.choice([1.0, 2.5, 0.5])))
        cfg["layers"].append(dict(type=kind, mixer=mixer, mlp=mlp))
    return cfg
