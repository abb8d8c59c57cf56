"""Writer of synthetic Tuterax folders (config.json + model.safetensors) with seeded random bf16 weights, numpy only: what bench.py loads when no real
checkpoint is at hand (novorax_synth.py and fidepel_synth.py are the same for the other folder designs).  The sizes resemble the layers of real models
of that width: attention and delta-rule mixers alternate, every layer closes with a gated feed-forward."""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np

from .novorax_synth import _bf16


@dataclass
class TuteraxSize:
    """`pattern` is repeated `repeat` times: D = delta, C = channel_delta, A = attention, each followed by d (dense feed-forward) or nothing."""
    name: str
    width: int
    vocab: int
    heads: int             # attention
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int
    d_heads: int           # delta rule: value heads, query / key heads, sizes, taps, inner sizes of the per-channel decay and gate
    d_kv_heads: int
    d_dim: int
    d_vdim: int
    conv: int
    rank_a: int
    rank_g: int
    ff: int
    pattern: tuple = ("Dd", "Ad", "Cd", "Ad")
    repeat: int = 1


SIZES = {
    "w1024": TuteraxSize("w1024", 1024, 32000, 16, 4, 64, 64, 32, 8, 4, 128, 128, 4, 64, 64, 2816),
    "w2048": TuteraxSize("w2048", 2048, 32000, 16, 4, 128, 128, 64, 16, 8, 128, 128, 4, 96, 96, 5632),
    "w4096": TuteraxSize("w4096", 4096, 32000, 32, 8, 128, 128, 64, 32, 16, 128, 128, 4, 128, 128, 11008),
}


def config_of(s: TuteraxSize) -> dict:
    layers, ranks = [], {}
    for _ in range(s.repeat):
        for code in s.pattern:
            if code[0] == "A":
                lc = {"type": "attention", "mixer": {"dim": s.dim, "heads": s.heads, "kv_heads": s.kv_heads, "rot": {"base": 500000.0, "dims": s.rot_dims},
                                                     "scale": float(s.dim ** -0.5), "softcap": 30.0, "vdim": s.vdim}}
            else:
                lc = {"type": "delta" if code[0] == "D" else "channel_delta",
                      "mixer": {"conv": s.conv, "dim": s.d_dim, "heads": s.d_heads, "kv_heads": s.d_kv_heads, "vdim": s.d_vdim}}
            lc["mlp"] = {"kind": "dense", "ff": s.ff} if code[1:] == "d" else None
            layers.append(lc)
    return {"architecture": "Tuterax", "embedding": {"scale": float(s.width ** 0.5)}, "layers": layers, "norm": {"eps": 1e-5}, "vocab": s.vocab, "width": s.width}


def tensor_shapes(cfg: dict, rank_a: int = 16, rank_g: int = 16) -> list:
    """(name, shape) of every tensor the configuration asks for (all bf16).  The inner sizes of the low-rank decay and gate projections are not part of
    the configuration - the loader takes them from the tensors - so they are given here."""
    W, V = cfg["width"], cfg["vocab"]
    out = [("embed", (V, W)), ("final.norm", (W,))]
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        H, G, D, VD = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out.append((p + "norm1", (W,)))
        if lc["type"] == "attention":
            out += [(p + "mix.q", (H * D, W)), (p + "mix.k", (G * D, W)), (p + "mix.v", (G * VD, W)), (p + "mix.q.norm", (D,)), (p + "mix.k.norm", (D,)),
                    (p + "mix.sink", (H,)), (p + "mix.o", (W, H * VD))]
        else:
            t = m["conv"]
            out += [(p + "mix.q", (G * D, W)), (p + "mix.q.conv", (G * D, t)), (p + "mix.k", (G * D, W)), (p + "mix.k.conv", (G * D, t)),
                    (p + "mix.v", (H * VD, W)), (p + "mix.v.conv", (H * VD, t)), (p + "mix.b", (H, W)), (p + "mix.A_log", (H,)), (p + "mix.norm", (VD,))]
            if lc["type"] == "channel_delta":
                out += [(p + "mix.a1", (rank_a, W)), (p + "mix.a2", (H * D, rank_a)), (p + "mix.dt_bias", (H * D,)),
                        (p + "mix.g1", (rank_g, W)), (p + "mix.g2", (H * VD, rank_g))]
            else:
                out += [(p + "mix.a", (H, W)), (p + "mix.dt_bias", (H,)), (p + "mix.g", (H * VD, W))]
            out.append((p + "mix.o", (W, H * VD)))
        if lc.get("mlp"):
            ff = lc["mlp"]["ff"]
            out += [(p + "norm2", (W,)), (p + "mlp.gate", (ff, W)), (p + "mlp.up", (ff, W)), (p + "mlp.down", (W, ff))]
    return out


def write_synthetic_tuterax(folder: str, size, seed: int = 0) -> dict:
    """Writes the folder; returns the configuration.  Matrices are N(0, 1 / in); norm weights that the design centres on zero, sinks, decay rates and
    step biases N(0, 0.1); the other vectors N(1, 0.1)."""
    s = SIZES[size] if isinstance(size, str) else size
    cfg = config_of(s)
    rng = np.random.default_rng(seed)
    os.makedirs(folder, exist_ok=True)
    shapes = tensor_shapes(cfg, s.rank_a, s.rank_g)
    head, off = {}, 0
    for name, shape in shapes:
        n = int(np.prod(shape, dtype=np.int64)) * 2
        head[name] = {"dtype": "BF16", "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
    hj = json.dumps(head, separators=(",", ":")).encode()
    hj += b" " * ((8 - len(hj) % 8) % 8)
    tmp = os.path.join(folder, "model.safetensors.tmp")
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for name, shape in shapes:
            if len(shape) == 2:
                rows_left = shape[0]
                gain = np.float32(1.0 if name == "embed" else shape[1] ** -0.5)
                while rows_left > 0:                        # in slabs: a wide table would be gigabytes of floats at once
                    r = min(rows_left, 4096)
                    f.write(_bf16(rng.standard_normal((r, shape[1]), dtype=np.float32) * gain).astype("<u2").tobytes())
                    rows_left -= r
            else:
                around_one = name.endswith(("q.norm", "k.norm", "mix.norm"))
                f.write(_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(0.1) + np.float32(1.0 if around_one else 0.0)).astype("<u2").tobytes())
    os.replace(tmp, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return cfg


def weight_bytes_per_token(cfg: dict, rank_a: int = 16, rank_g: int = 16) -> int:
    """Weight bytes one decoded token reads: every layer's projections (both halves of the low-rank ones), its output projection and feed-forward, one
    embedding row, and the embedding table once more as the output head."""
    W, V = cfg["width"], cfg["vocab"]
    total = 2 * (W + V * W)
    for lc in cfg["layers"]:
        m = lc["mixer"]
        H, G, D, VD = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if lc["type"] == "attention":
            rows = H * D + G * D + G * VD
        elif lc["type"] == "channel_delta":
            rows = 2 * G * D + H * VD + H + rank_a + rank_g
            total += 2 * (H * D * rank_a + H * VD * rank_g)
        else:
            rows = 2 * G * D + H * VD + H + H + H * VD
        total += 2 * (rows * W + W * H * VD)
        if lc.get("mlp"):
            total += 2 * 3 * lc["mlp"]["ff"] * W
    return total
