"""Small Tosisun configurations of the tests and their random weights.

The sizes differ from layer to layer and between the configurations in everything the format lets differ: heads
against key/value heads (equal, 3 and 4 to 1), dim against vdim (smaller, larger, equal), 1 to 5 convolution taps,
rotated dims (none, some, the whole head), frequency stretching whose three branches all occur, layers that run with
another layer's tensors, one expert of five and three of six, with and without a shared expert, a layer without a
feed-forward, no soft cap, a width that is no multiple of 8.

Weights are drawn here (not by the engine's random-weights mode): gains and biases of the norms away from their
neutral values, sinks of both signs, router biases, wide convolution taps."""
import json
import os

import torch

MAIN = dict(
    architecture="Tosisun", width=96, vocab=310, norm=dict(eps=3e-6), logit_softcap=9.0,
    layers=[
        dict(type="attention",
             mixer=dict(heads=6, kv_heads=2, dim=32, vdim=16, conv=4, scale=0.2,
                        rot=dict(base=10000.0, dims=8, scaling=dict(factor=8.0, low=1.0, high=4.0, original=64))),
             mlp=dict(kind="dense", ff=136)),
        dict(type="attention",
             mixer=dict(heads=4, kv_heads=4, dim=16, vdim=48, conv=2, scale=0.3, rot=dict(base=500.0, dims=16)),
             mlp=dict(kind="moe", expert=dict(ff=40, limit=1.5), router=dict(experts=6, top=3), shared=dict(ff=56, limit=0.7))),
        dict(type="attention",
             mixer=dict(heads=4, kv_heads=4, dim=16, vdim=48, conv=2, scale=0.3, rot=dict(base=500.0, dims=16)),
             mlp=dict(kind="moe", expert=dict(ff=40, limit=1.5), router=dict(experts=6, top=3), shared=dict(ff=56, limit=0.7)),
             weights_of=1),
        dict(type="attention",
             mixer=dict(heads=3, kv_heads=1, dim=24, vdim=24, conv=1, scale=0.25, rot=dict(base=1.0, dims=0)),
             mlp=None),
        dict(type="attention",
             mixer=dict(heads=6, kv_heads=2, dim=32, vdim=16, conv=4, scale=0.2,
                        rot=dict(base=10000.0, dims=8, scaling=dict(factor=8.0, low=1.0, high=4.0, original=64))),
             mlp=dict(kind="dense", ff=136), weights_of=0),
        dict(type="attention",
             mixer=dict(heads=8, kv_heads=2, dim=64, vdim=64, conv=3, scale=0.11,
                        rot=dict(base=1000000.0, dims=32, scaling=dict(factor=4.0, low=1.0, high=4.0, original=32))),
             mlp=dict(kind="moe", expert=dict(ff=24, limit=3.0), router=dict(experts=5, top=1))),
    ])

# a width that is no multiple of 8, heads that no matrix-core kernel takes as they are, no cap on the logits
ODD = dict(
    architecture="Tosisun", width=84, vocab=150, norm=dict(eps=1e-5),
    layers=[
        dict(type="attention",
             mixer=dict(heads=5, kv_heads=5, dim=20, vdim=12, conv=5, scale=0.3, rot=dict(base=100.0, dims=20)),
             mlp=dict(kind="moe", expert=dict(ff=36, limit=1.0), router=dict(experts=3, top=3), shared=dict(ff=20, limit=2.0))),
        dict(type="attention",
             mixer=dict(heads=2, kv_heads=1, dim=8, vdim=72, conv=2, scale=0.5, rot=dict(base=30000.0, dims=4)),
             mlp=dict(kind="dense", ff=60)),
    ])

# heads of 128 and of more than any matrix-core kernel takes, many query heads a key/value head
WIDE = dict(
    architecture="Tosisun", width=128, vocab=200, norm=dict(eps=1e-6), logit_softcap=30.0,
    layers=[
        dict(type="attention",
             mixer=dict(heads=2, kv_heads=1, dim=128, vdim=96, conv=3, scale=0.09,
                        rot=dict(base=10000.0, dims=64, scaling=dict(factor=2.0, low=1.0, high=2.0, original=16))),
             mlp=dict(kind="dense", ff=64)),
        dict(type="attention",
             mixer=dict(heads=20, kv_heads=1, dim=16, vdim=16, conv=2, scale=0.25, rot=dict(base=50.0, dims=8)),
             mlp=None),
        dict(type="attention",
             mixer=dict(heads=1, kv_heads=1, dim=144, vdim=40, conv=2, scale=0.08, rot=dict(base=1000.0, dims=144)),
             mlp=dict(kind="dense", ff=32)),
    ])

CONFIGS = {"main": MAIN, "odd": ODD, "wide": WIDE}


def tensor_shapes(cfg):
    """name -> shape of every tensor a model of ``cfg`` has (layers that run with another's tensors have none)."""
    W, out = cfg["width"], {}
    out["embed"] = (cfg["vocab"], W)
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        for n in ("norm1", "norm2"):
            out[p + n], out[p + n + ".b"] = (W,), (W,)
        Qd, Kd, Vd = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
        for x, rows in (("q", Qd), ("k", Kd), ("v", Vd)):
            out.update({f"{p}mix.{x}": (rows, W), f"{p}mix.{x}.b": (rows,), f"{p}mix.{x}.conv": (rows, m["conv"])})
        out.update({p + "mix.q.norm": (Qd,), p + "mix.k.norm": (Kd,), p + "mix.sink": (m["heads"],),
                    p + "mix.o": (W, m["heads"] * m["vdim"])})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            out.update({p + "mlp.up": (mlp["ff"], W), p + "mlp.down": (W, mlp["ff"])})
        else:
            E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            out.update({p + "mlp.router": (E, W), p + "mlp.router.b": (E,)})
            for e in range(E):
                out.update({f"{p}mlp.e{e}.gate": (ff, W), f"{p}mlp.e{e}.up": (ff, W), f"{p}mlp.e{e}.down": (W, ff)})
            if mlp.get("shared") is not None:
                sf = mlp["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (sf, W), p + "mlp.shared.up": (sf, W), p + "mlp.shared.down": (W, sf)})
    out["final.norm"], out["final.norm.b"], out["head"] = (W,), (W,), (cfg["vocab"], W)
    return out


def make_weights(cfg, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        parts = name.split(".")
        last = parts[-1]
        if last in ("norm1", "norm2") or name == "final.norm":
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif last == "norm":                      # q.norm, k.norm
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif last == "b" and parts[-2] in ("norm1", "norm2", "norm"):
            t = 0.1 * torch.randn(shape, generator=g)
        elif last == "b":                         # projection and router biases
            t = 0.3 * torch.randn(shape, generator=g)
        elif last == "conv":
            t = 0.6 * torch.randn(shape, generator=g)
        elif last == "sink":
            t = 1.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) * (1.0 / shape[-1] ** 0.5)
        w[name] = t.to(dtype)
    return w


def write_config(folder, cfg, weights):
    from zedinfer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"), weights, metadata={"format": "pt"})
    return folder


def write_model(folder, name, seed=0, dtype=torch.float32):
    """config.json and model.safetensors of configuration ``name``; returns the folder."""
    return write_config(folder, CONFIGS[name], make_weights(CONFIGS[name], seed, dtype))


def random_config(seed):
    """A configuration drawn at random: sizes, head counts, the order of layers and which run with whose tensors,
    taps, rotated dims, bases and stretching, scales, experts and how many are chosen, limits, eps, the cap."""
    import random
    rng = random.Random(seed)
    width = rng.choice([48, 64, 72, 96, 128, 160])
    cfg = dict(architecture="Tosisun", width=width, vocab=rng.choice([97, 256, 411]),
               norm=dict(eps=rng.choice([1e-6, 1e-5, 3e-6])), layers=[])
    if rng.random() < 0.7:
        cfg["logit_softcap"] = rng.choice([5.0, 12.0, 40.0])
    owners = []
    for i in range(rng.randint(2, 6)):
        if owners and rng.random() < 0.35:
            src = rng.choice(owners)
            layer = json.loads(json.dumps(cfg["layers"][src]))
            layer["weights_of"] = src
            cfg["layers"].append(layer)
            continue
        kvh = rng.choice([1, 2, 3, 4])
        dim = rng.choice([8, 16, 24, 32, 48, 64, 96, 128])
        dims = rng.choice([0, 2, dim // 2, dim]) // 2 * 2
        rot = dict(base=rng.choice([50.0, 10000.0, 1000000.0]), dims=dims)
        if dims and rng.random() < 0.6:
            rot["scaling"] = dict(factor=rng.choice([2.0, 4.0, 8.0]), low=1.0, high=rng.choice([2.0, 4.0]),
                                  original=rng.choice([16, 64, 256]))
        mixer = dict(heads=kvh * rng.choice([1, 2, 4, 6]), kv_heads=kvh, dim=dim, vdim=rng.choice([8, 16, 24, 40, 64, 128]),
                     conv=rng.choice([1, 2, 3, 4, 6]), scale=rng.choice([0.05, 0.1, 0.2]) * (32.0 / dim) ** 0.5, rot=rot)
        r = rng.random()
        if r < 0.15:
            mlp = None
        elif r < 0.5:
            mlp = dict(kind="dense", ff=rng.choice([32, 72, 136]))
        else:
            experts = rng.choice([2, 4, 7, 16, 40])
            mlp = dict(kind="moe", expert=dict(ff=rng.choice([16, 40, 72]), limit=rng.choice([0.5, 2.0, 7.0])),
                       router=dict(experts=experts, top=rng.randint(1, min(experts, 6))))
            if rng.random() < 0.6:
                mlp["shared"] = dict(ff=rng.choice([16, 48, 100]), limit=rng.choice([1.0, 3.0]))
        owners.append(i)
        cfg["layers"].append(dict(type="attention", mixer=mixer, mlp=mlp))
    return cfg
