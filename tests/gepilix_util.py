"""Small random Gepilix checkpoints for the tests: a config dict and a name -> tensor dict in the checkpoint's naming, optionally written to a folder
(config.json + model.safetensors) so the tests go through the registry and the loader like a user does."""

import json
import os

import torch


def chunked(heads=4, kv_heads=2, dim=24, vdim=40, size=13, scale=None, softcap=5.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "scale": dim ** -0.5 if scale is None else scale}
    if softcap:
        m["softcap"] = softcap
    return m


def windowed(heads=6, kv_heads=2, dim=16, vdim=24, size=11, rot_dims=12, base=5000.0, scaling=(4.0, 1.0, 4.0, 64), scale=None, softcap=8.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size}, "scale": dim ** -0.5 if scale is None else scale,
         "rot": {"dims": rot_dims, "base": base}}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if softcap:
        m["softcap"] = softcap
    return m


def parallel(left=None, width=48, blocks=3, conv=4):
    return {"type": "parallel", "mixer": {"left": left or chunked(), "right": {"width": width, "blocks": blocks, "conv": conv}}}


def parallel_2(left=None, heads=4, vdim=20, state=24, groups=2, norm_groups=4, conv=4, left_scale=0.7, right_scale=1.3):
    return {"type": "parallel_2", "mixer": {"left": left or windowed(), "left_scale": left_scale, "right_scale": right_scale,
                                            "right": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}}}


def wkv(heads=3, dim=24, rank=10):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "_rank": rank}


def dense(ff=88):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=3, ff=40, shared=56):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def make_config(layers, width=72, vocab=131, eps=1e-5):
    """layers: list of (mixer entry, mlp entry or None).  Returns (config, {layer: decay rank}) -- the rank is no config entry, a tensor's shape gives it."""
    out, ranks = [], {}
    for i, (mixer, mlp) in enumerate(layers):
        e = {k: v for k, v in mixer.items() if not k.startswith("_")}
        e["mlp"] = mlp
        out.append(e)
        if "_rank" in mixer:
            ranks[i] = mixer["_rank"]
    return {"architecture": "Gepilix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": out}, ranks


def make_weights(cfg_ranks, seed=0):
    cfg, ranks = cfg_ranks
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    bf = torch.bfloat16

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / i ** 0.5).to(bf)

    def vec(n, mean=1.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(bf)

    def norm(name, w):
        w[name], w[name + ".b"], w[name + ".alpha"] = vec(W), vec(W, 0.0, 0.1), (0.5 + 0.5 * torch.rand((), generator=g)).to(bf)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(bf), "head": lin(cfg["vocab"], W)}
    norm("final.norm", w)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        norm(p + "norm1", w)
        w[p + "ls1"] = vec(W, 0.8, 0.2)
        x = p + "mix."
        if layer["type"] == "wkv":
            H, d, r = m["heads"], m["dim"], ranks[i]
            for s in "rkvgw":
                w[x + "mu." + s] = torch.rand(W, generator=g).to(bf)
            w[x + "r"], w[x + "k"], w[x + "v"], w[x + "g"] = lin(H * d, W), lin(H * d, W), lin(H * d, W), lin(H * d, W)
            w[x + "w1"], w[x + "w2"], w[x + "w0"] = lin(r, W, 2.0), lin(H * d, r, 2.0), vec(H * d, -1.5, 1.0)
            w[x + "u"], w[x + "norm"], w[x + "o"] = vec(H * d, 0.5, 0.5).reshape(H, d), vec(H * d), lin(W, H * d)
        else:
            L, R = m["left"], m["right"]
            H, G, d, dv = L["heads"], L["kv_heads"], L["dim"], L["vdim"]
            l, r = x + "left.", x + "right."
            w[l + "q"], w[l + "k"], w[l + "v"], w[l + "o"] = lin(H * d, W, 3.0), lin(G * d, W, 2.0), lin(G * dv, W), lin(W, H * dv)
            if layer["type"] == "parallel":
                w[l + "q.b"], w[l + "k.b"], w[l + "v.b"] = vec(H * d, 0.0, 0.3), vec(G * d, 0.0, 0.3), vec(G * dv, 0.0, 0.3)
                w[l + "g"] = lin(H, W, 2.0)
                C, nb, taps = R["width"], R["blocks"], R["conv"]
                n = C // nb
                w[r + "y"], w[r + "y.b"], w[r + "x"], w[r + "x.b"] = lin(C, W), vec(C, 0.0, 0.2), lin(C, W), vec(C, 0.0, 0.2)
                w[r + "conv"], w[r + "conv.b"] = (0.4 * torch.randn(C, taps, generator=g)).to(bf), vec(C, 0.0, 0.2)
                w[r + "ra"], w[r + "ra.b"] = (torch.randn(nb, n, n, generator=g) / n ** 0.5).to(bf), vec(nb * n, 0.0, 0.5).reshape(nb, n)
                w[r + "ri"], w[r + "ri.b"] = (torch.randn(nb, n, n, generator=g) / n ** 0.5).to(bf), vec(nb * n, 0.0, 0.5).reshape(nb, n)
                w[r + "lam"], w[r + "o"] = vec(C, -2.0, 1.5), lin(W, C)
                w[x + "left.out"], w[x + "right.out"] = vec(W), vec(W, 0.7, 0.2)
            else:
                Hs, P, N, Gs, taps = R["heads"], R["vdim"], R["state"], R["groups"], R["conv"]
                inner, Cc = Hs * P, Hs * P + 2 * Gs * N
                w[r + "in"] = lin(2 * inner + 2 * Gs * N + Hs, W)
                w[r + "conv"], w[r + "conv.b"] = (0.4 * torch.randn(Cc, taps, generator=g)).to(bf), vec(Cc, 0.0, 0.2)
                w[r + "dt_bias"], w[r + "A_log"], w[r + "D"] = vec(Hs, -1.0, 1.0), vec(Hs, 0.0, 1.0), vec(Hs, 1.0, 0.5)
                w[r + "norm"], w[r + "o"] = vec(inner), lin(W, inner)
        mlp = layer.get("mlp")
        if mlp:
            norm(p + "norm2", w)
            w[p + "ls2"] = vec(W, 0.8, 0.2)
            e = p + "mlp."
            if mlp["kind"] == "dense":
                w[e + "up"], w[e + "down"] = lin(mlp["ff"], W, 1.5), lin(W, mlp["ff"])
            else:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                w[e + "router"], w[e + "router.b"] = lin(E, W, 4.0), vec(E, 0.0, 0.5)
                for j in range(E):
                    w[f"{e}e{j}.gate"], w[f"{e}e{j}.up"], w[f"{e}e{j}.down"] = lin(F, W, 1.5), lin(F, W, 1.5), lin(W, F)
                if mlp.get("shared"):
                    Fs = mlp["shared"]["ff"]
                    w[e + "shared.gate"], w[e + "shared.up"], w[e + "shared.down"] = lin(Fs, W, 1.5), lin(Fs, W, 1.5), lin(W, Fs)
    return w


def save(folder, cfg_ranks, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg_ranks[0], f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def default_layers():
    """Every mixer and feed-forward; grouped queries 2:1 and 3:1; chunks and windows shorter than the prompts; a partial rotation with rescaled frequencies;
    a layer without feed-forward; a mixture with and one without a shared expert."""
    return [(wkv(), dense()),
            (parallel(), moe()),
            (parallel_2(), dense(ff=50)),
            (wkv(heads=2, dim=40, rank=6), None),
            (parallel_2(left=windowed(heads=3, kv_heads=3, dim=24, vdim=16, size=7, rot_dims=24, scaling=None, softcap=0.0), heads=6, vdim=8, state=16, groups=3, norm_groups=1, conv=2),
             moe(experts=5, top=1, ff=24, shared=0)),
            (parallel(left=chunked(heads=6, kv_heads=2, dim=16, vdim=16, size=8), width=40, blocks=1, conv=2), dense())]
