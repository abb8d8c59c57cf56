"""Small Tuterax models for tests: configurations of chosen sizes, random bf16 weights from a seed, written as a folder
(config.json + model.safetensors) the loader reads.  The sizes are deliberately odd ones - head counts, head sizes, tap
counts and widths that share no factor with the kernels' tile sizes."""
from __future__ import annotations

import json
import os

import torch


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def attention(heads=6, kv_heads=2, dim=24, vdim=20, rot_dims=8, base=5000.0, scale=0.3, softcap=6.0, mlp=None):
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim, "rot": {"base": base, "dims": rot_dims}}
    if softcap:
        mixer["softcap"] = softcap
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def delta(heads=4, kv_heads=2, dim=12, vdim=20, conv=4, mlp=None):
    return {"type": "delta", "mixer": {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}, "mlp": mlp}


def channel_delta(heads=3, kv_heads=3, dim=20, vdim=12, conv=3, ranks=(5, 7), mlp=None):
    """ranks: inner sizes of the low-rank decay and gate projections; they live in the tensors' shapes only, so they travel beside the configuration."""
    return {"type": "channel_delta", "mixer": {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}, "mlp": mlp, "_ranks": list(ranks)}


def config(layers, width=72, vocab=97, eps=1e-5, embed_scale=2.5):
    return {"architecture": "Tuterax", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def weights(cfg, seed=0, hold=False):
    """hold: decays close to one (the matrix memory keeps what it was told for hundreds of tokens)."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    width, vocab = cfg["width"], cfg["vocab"]

    def mat(n, k, gain=1.0):
        return (torch.randn(n, k, generator=g) * gain / k ** 0.5).to(torch.bfloat16)

    def vec(n, std=0.1, mean=0.0):
        return (torch.randn(n, generator=g) * std + mean).to(torch.bfloat16)

    W["embed"] = (torch.randn(vocab, width, generator=g) * 0.5).to(torch.bfloat16)
    W["final.norm"] = vec(width, 0.2)
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        H, G, D, VD = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = vec(width, 0.2)
        if lc["type"] == "attention":
            W[p + "mix.q"] = mat(H * D, width, 1.5)
            W[p + "mix.k"] = mat(G * D, width, 1.5)
            W[p + "mix.v"] = mat(G * VD, width, 1.5)
            W[p + "mix.q.norm"] = vec(D, 0.3, 1.5)
            W[p + "mix.k.norm"] = vec(D, 0.3, 1.5)
            W[p + "mix.sink"] = vec(H, 1.0, 0.5)
        else:
            taps = m["conv"]
            for nm, rows in (("q", G * D), ("k", G * D), ("v", H * VD)):
                W[p + "mix." + nm] = mat(rows, width, 2.0)
                W[p + "mix." + nm + ".conv"] = (torch.randn(rows, taps, generator=g) * 0.6).to(torch.bfloat16)
            W[p + "mix.b"] = mat(H, width, 2.0)
            W[p + "mix.A_log"] = vec(H, 0.5, -6.0 if hold else -0.5)
            W[p + "mix.norm"] = vec(VD, 0.2, 1.0)
            if lc["type"] == "channel_delta":
                ra, rg = lc["_ranks"]
                W[p + "mix.a1"] = mat(ra, width, 1.5)
                W[p + "mix.a2"] = mat(H * D, ra, 1.5)
                W[p + "mix.dt_bias"] = vec(H * D, 0.7)
                W[p + "mix.g1"] = mat(rg, width, 1.5)
                W[p + "mix.g2"] = mat(H * VD, rg, 1.5)
            else:
                W[p + "mix.a"] = mat(H, width, 1.5)
                W[p + "mix.dt_bias"] = vec(H, 0.7)
                W[p + "mix.g"] = mat(H * VD, width, 1.5)
        W[p + "mix.o"] = mat(width, H * VD)
        if lc.get("mlp"):
            ff = lc["mlp"]["ff"]
            W[p + "norm2"] = vec(width, 0.2)
            W[p + "mlp.gate"] = mat(ff, width, 1.5)
            W[p + "mlp.up"] = mat(ff, width, 1.5)
            W[p + "mlp.down"] = mat(width, ff)
    return W


def write(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    clean = json.loads(json.dumps(cfg))
    for lc in clean["layers"]:
        lc.pop("_ranks", None)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(clean, f, indent=1)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)
