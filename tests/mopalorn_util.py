"""Small random Mopalorn checkpoints for the tests: a config dict and a name -> tensor dict in the checkpoint's naming, optionally written to a folder
(config.json + model.safetensors) so the tests go through the registry and the loader like a user does."""

import json
import os

import torch


def latent(heads=3, dim=24, rot_dim=16, vdim=40, kv_rank=48, size=11, rot_dims=None, base=5000.0, scale=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "mask": {"size": size},
                                                  "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base}, "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}}


def capped(heads=4, kv_heads=2, dim=24, vdim=40, coef=0.7, every=9, softcap=6.0, v_mix=True, scale=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "q_temp": {"coef": coef, "every": every}, "softcap": softcap,
                                           "v_mix": v_mix, "scale": dim ** -0.5 if scale is None else scale}}


def pooled(heads=4, kv_heads=2, dim=24, vdim=40, size=13, pool=5, v_mix=True, scale=None, sink=True):
    return {"type": "attention_2", "sink": sink, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size, "pool": pool}, "v_mix": v_mix,
                                                           "scale": dim ** -0.5 if scale is None else scale}}


def dense(ff=88):
    return {"kind": "dense", "ff": ff}


def make_config(layers, width=72, vocab=131, eps=1e-5, logit_scale=0.8):
    """layers: list of (mixer entry, mlp entry or None).  The 'sink' key of a mixer entry only steers make_weights and is not part of the config."""
    out = []
    for mixer, mlp in layers:
        e = {k: v for k, v in mixer.items() if k != "sink"}
        e["mlp"] = mlp
        out.append(e)
    return {"architecture": "Mopalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale, "layers": out}, [m.get("sink", False) for m, _ in layers]


def make_weights(cfg_sinks, seed=0):
    cfg, sinks = cfg_sinks
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / i ** 0.5).to(torch.bfloat16)

    def vec(n, mean=1.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(torch.bfloat16), "final.norm": vec(W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"], w[p + "norm1b"] = vec(W), vec(W, 0.8, 0.2)
        x = p + "mix."
        if layer["type"] == "latent_attention":
            H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w[x + "q"], w[x + "dkv"], w[x + "dkv.norm"] = lin(H * (dn + dr), W, 3.0), lin(R + dr, W, 2.0), vec(R, 1.0, 0.2)
            w[x + "uk"], w[x + "uv"], w[x + "g"], w[x + "o"] = lin(H * dn, R, 2.0), lin(H * dv, R), lin(H * dv, W, 2.0), lin(W, H * dv)
        else:
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[x + "q"], w[x + "k"], w[x + "v"], w[x + "o"] = lin(H * d, W, 3.0), lin(G * d, W, 2.0), lin(G * dv, W), lin(W, H * dv)
            if m.get("v_mix"):
                w[x + "vmix"] = (0.2 + 0.5 * torch.rand((), generator=g)).to(torch.bfloat16)
            if sinks[i]:
                w[x + "sink"] = vec(H, 0.5, 1.0)
        mlp = layer.get("mlp")
        if mlp:
            w[p + "norm2"], w[p + "norm2b"] = vec(W), vec(W, 0.8, 0.2)
            e = p + "mlp."
            w[e + "up"], w[e + "down"], w[e + "act"] = lin(mlp["ff"], W, 2.0), lin(W, mlp["ff"]), vec(2, 0.3, 0.8)
    return w


def save(folder, cfg_sinks, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg_sinks[0], f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def default_layers():
    """Every mixer; grouped queries 2:1, 1:1 and 3:1; windows shorter than the prompts; a pool that does not divide its window; a value-mixing chain that starts in a
    pooled layer, skips one layer and goes through both attention types; a layer without feed-forward; a partial rotation."""
    return [(latent(), dense()),
            (pooled(), dense(ff=50)),
            (capped(v_mix=False, heads=3, kv_heads=3, dim=16, vdim=24), None),
            (capped(), dense()),
            (latent(heads=2, dim=40, rot_dim=24, vdim=16, kv_rank=72, size=7, rot_dims=12, base=300.0), dense(ff=40)),
            (pooled(heads=6, kv_heads=2, size=9, pool=4, sink=False), dense())]
