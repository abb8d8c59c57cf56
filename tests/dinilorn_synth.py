"""Small Dinilorn models for tests: configurations of chosen sizes, random bf16 weights from a seed, written as a folder
(config.json + model.safetensors) the loader reads.  The sizes are deliberately odd ones - head counts, head sizes, expert
counts and widths that share no factor with the kernels' tile sizes."""
from __future__ import annotations

import json
import os

import torch


def moe(experts=6, top=2, groups=(3, 2), ff=24, limit=1.2, shared=(40, 1.6)):
    """groups: (count, keep) or None; shared: (ff, limit) or None."""
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}
    if shared:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def retention(heads=3, dim=20, vdim=12, rot_dims=8, base=5000.0, decay=None, mlp=None):
    mixer = {"decay": list(decay) if decay else [1.0 - 0.3 * 2.0 ** (-1 - h) for h in range(heads)], "dim": dim, "heads": heads, "vdim": vdim}
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "retention", "mixer": mixer, "mlp": mlp}


def attention(heads=6, kv_heads=2, dim=24, vdim=20, scale=0.25, softcap=7.0, rel_rows=10, bias_max=40, q_temp=(0.4, 5), mlp=None):
    """rel_rows: rows of the distance-bias table - it lives in the tensor's shape only, so it travels beside the configuration."""
    mixer = {"bias_max": bias_max, "dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if softcap:
        mixer["softcap"] = softcap
    if q_temp:
        mixer["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": mixer, "mlp": mlp, "_rel_rows": rel_rows}


def attention_2(heads=4, kv_heads=2, dim=12, vdim=28, scale=0.3, rot_dims=8, base=3000.0, scaling=(4.0, 1.0, 3.0, 64), size=9, keep_first=3, diff=0.35, mlp=None):
    """scaling: (factor, low, high, original) or None."""
    mixer = {"diff": diff, "dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if size:
        mixer["mask"] = {"keep_first": keep_first, "size": size}
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
        if scaling:
            mixer["rot"]["scaling"] = {"factor": scaling[0], "low": scaling[1], "high": scaling[2], "original": scaling[3]}
    return {"type": "attention_2", "mixer": mixer, "mlp": mlp}


def config(layers, width=72, vocab=97, eps=1e-5, loop=None):
    """loop: (start, stop, times) or None."""
    cfg = {"architecture": "Dinilorn", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = {}
    width, vocab = cfg["width"], cfg["vocab"]

    def mat(n, k, gain=1.0):
        return (torch.randn(n, k, generator=g) * gain / k ** 0.5).to(torch.bfloat16)

    def vec(n, std=0.1, mean=0.0):
        return (torch.randn(n, generator=g) * std + mean).to(torch.bfloat16)

    W["embed"] = (torch.randn(vocab, width, generator=g) * 0.5).to(torch.bfloat16)
    W["head"] = mat(vocab, width)
    W["final.norm"] = vec(width, 0.2)
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        H, D, VD = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        W[p + "norm1"] = vec(width, 0.2)
        W[p + "norm1b"] = vec(width, 0.2)
        if lc["type"] == "retention":
            W[p + "mix.q"] = mat(H * D, width, 1.5)
            W[p + "mix.k"] = mat(H * D, width, 1.5)
            W[p + "mix.v"] = mat(H * VD, width, 1.5)
            W[p + "mix.g"] = mat(H * VD, width, 1.5)
        else:
            maps = 2 if lc["type"] == "attention_2" else 1
            for nm, rows in (("q", H * maps * D), ("k", G * maps * D), ("v", G * VD)):
                W[p + "mix." + nm] = mat(rows, width, 1.5)
                W[p + "mix." + nm + ".b"] = vec(rows, 0.3)
            W[p + "mix.o.b"] = vec(width, 0.3)
            if maps == 1:
                W[p + "mix.rel"] = (torch.randn(lc["_rel_rows"], H, generator=g) * 1.0).to(torch.bfloat16)
                W[p + "mix.g"] = mat(H, width, 2.0)
            else:
                for nm in ("lq1", "lk1", "lq2", "lk2"):
                    W[p + "mix." + nm] = vec(D, 0.3)
                W[p + "mix.g"] = mat(H * VD, width, 2.0)
        W[p + "mix.o"] = mat(width, H * VD)
        mlp = lc.get("mlp")
        if mlp:
            W[p + "norm2"] = vec(width, 0.2)
            W[p + "norm2b"] = vec(width, 0.2)
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                W[p + f"mlp.e{e}.gate"] = mat(ff, width, 2.0)
                W[p + f"mlp.e{e}.up"] = mat(ff, width, 2.0)
                W[p + f"mlp.e{e}.down"] = mat(width, ff)
            W[p + "mlp.router"] = mat(mlp["router"]["experts"], width, 2.0)
            W[p + "mlp.correction"] = vec(mlp["router"]["experts"], 0.4)
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                W[p + "mlp.shared.gate"] = mat(sf, width, 2.0)
                W[p + "mlp.shared.up"] = mat(sf, width, 2.0)
                W[p + "mlp.shared.down"] = mat(width, sf)
                W[p + "mlp.shared.sg"] = mat(1, width, 2.0)
    return W


def write(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    clean = json.loads(json.dumps(cfg))
    for lc in clean["layers"]:
        lc.pop("_rel_rows", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(clean, f, indent=1)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)
