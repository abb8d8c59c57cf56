"""Writer of synthetic Dinilorn folders (config.json + model.safetensors) with seeded random bf16 weights, numpy only: what bench.py loads when no real
checkpoint is at hand (novorax_synth.py, fidepel_synth.py and tuterax_synth.py are the same for the other folder designs).  The sizes resemble the layers
of real models of that width: retention, attention and two-map attention in turns, every layer closes with routed experts and a shared expert."""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np

from .novorax_synth import _bf16


@dataclass
class DinilornSize:
    """`pattern`: R = retention, A = attention, B = two-map attention, each followed by m (routed experts) or nothing."""
    name: str
    width: int
    vocab: int
    heads: int             # both attentions
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int          # two-map attention
    window: int
    keep_first: int
    r_heads: int           # retention
    r_dim: int
    r_vdim: int
    n_expert: int
    top: int
    expert_ff: int
    groups: tuple          # (count, keep)
    shared_ff: int
    rel_rows: int = 32
    bias_max: int = 4096
    pattern: tuple = ("Rm", "Am", "Bm", "Am")
    loop: tuple | None = None          # (start, stop, times)


SIZES = {
    "w1024": DinilornSize("w1024", 1024, 32000, 16, 4, 64, 64, 32, 1024, 4, 8, 128, 128, 8, 2, 704, (4, 2), 704),
    "w2048": DinilornSize("w2048", 2048, 32000, 16, 4, 128, 128, 64, 1024, 4, 16, 128, 128, 16, 2, 960, (4, 2), 1856),
    "w4096": DinilornSize("w4096", 4096, 32000, 32, 8, 128, 128, 64, 1024, 4, 32, 128, 128, 32, 4, 960, (8, 4), 1856),
}


def config_of(s: DinilornSize) -> dict:
    layers = []
    for code in s.pattern:
        if code[0] == "R":
            lc = {"type": "retention", "mixer": {"decay": [float(1.0 - 0.75 * 2.0 ** (-5 - 3 * h / max(s.r_heads - 1, 1))) for h in range(s.r_heads)], "dim": s.r_dim, "heads": s.r_heads,
                                                 "rot": {"base": 500000.0, "dims": s.r_dim}, "vdim": s.r_vdim}}
        elif code[0] == "A":
            lc = {"type": "attention", "mixer": {"bias_max": s.bias_max, "dim": s.dim, "heads": s.heads, "kv_heads": s.kv_heads, "q_temp": {"coef": 0.1, "every": 256},
                                                 "scale": float(s.dim ** -0.5), "softcap": 30.0, "vdim": s.vdim}}
        else:
            lc = {"type": "attention_2", "mixer": {"diff": 0.5, "dim": s.dim // 2, "heads": s.heads, "kv_heads": s.kv_heads, "mask": {"keep_first": s.keep_first, "size": s.window},
                                                   "rot": {"base": 500000.0, "dims": s.rot_dims, "scaling": {"factor": 8.0, "high": 4.0, "low": 1.0, "original": 8192}},
                                                   "scale": float((s.dim // 2) ** -0.5), "vdim": s.vdim}}
        lc["mlp"] = {"kind": "moe", "expert": {"ff": s.expert_ff, "limit": 7.0},
                     "router": {"experts": s.n_expert, "groups": {"count": s.groups[0], "keep": s.groups[1]}, "top": s.top},
                     "shared": {"ff": s.shared_ff, "limit": 7.0}} if code[1:] == "m" else None
        layers.append(lc)
    cfg = {"architecture": "Dinilorn", "layers": layers, "norm": {"eps": 1e-5}, "vocab": s.vocab, "width": s.width}
    if s.loop:
        cfg["loop"] = {"start": s.loop[0], "stop": s.loop[1], "times": s.loop[2]}
    return cfg


def tensor_shapes(cfg: dict, rel_rows: int = 32) -> list:
    """(name, shape) of every tensor the configuration asks for (all bf16).  The rows of the distance-bias table are not part of the configuration - the
    loader takes them from the tensor - so they are given here."""
    W, V = cfg["width"], cfg["vocab"]
    out = [("embed", (V, W)), ("head", (V, W)), ("final.norm", (W,))]
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        H, D, VD = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        out += [(p + "norm1", (W,)), (p + "norm1b", (W,))]
        if lc["type"] == "retention":
            out += [(p + "mix.q", (H * D, W)), (p + "mix.k", (H * D, W)), (p + "mix.v", (H * VD, W)), (p + "mix.g", (H * VD, W))]
        else:
            maps = 2 if lc["type"] == "attention_2" else 1
            out += [(p + "mix.q", (H * maps * D, W)), (p + "mix.q.b", (H * maps * D,)), (p + "mix.k", (G * maps * D, W)), (p + "mix.k.b", (G * maps * D,)),
                    (p + "mix.v", (G * VD, W)), (p + "mix.v.b", (G * VD,)), (p + "mix.o.b", (W,))]
            if maps == 1:
                out += [(p + "mix.rel", (rel_rows, H)), (p + "mix.g", (H, W))]
            else:
                out += [(p + "mix." + nm, (D,)) for nm in ("lq1", "lk1", "lq2", "lk2")] + [(p + "mix.g", (H * VD, W))]
        out.append((p + "mix.o", (W, H * VD)))
        mlp = lc.get("mlp")
        if mlp:
            ff = mlp["expert"]["ff"]
            out += [(p + "norm2", (W,)), (p + "norm2b", (W,))]
            for e in range(mlp["router"]["experts"]):
                out += [(f"{p}mlp.e{e}.gate", (ff, W)), (f"{p}mlp.e{e}.up", (ff, W)), (f"{p}mlp.e{e}.down", (W, ff))]
            out += [(p + "mlp.router", (mlp["router"]["experts"], W)), (p + "mlp.correction", (mlp["router"]["experts"],))]
            if mlp.get("shared"):
                sf = mlp["shared"]["ff"]
                out += [(p + "mlp.shared.gate", (sf, W)), (p + "mlp.shared.up", (sf, W)), (p + "mlp.shared.down", (W, sf)), (p + "mlp.shared.sg", (1, W))]
    return out


def write_synthetic_dinilorn(folder: str, size, seed: int = 0) -> dict:
    """Writes the folder; returns the configuration.  Matrices are N(0, 1 / in) (the embedding N(0, 1), the bias table N(0, 1)), vectors N(0, 0.1)."""
    s = SIZES[size] if isinstance(size, str) else size
    cfg = config_of(s)
    rng = np.random.default_rng(seed)
    os.makedirs(folder, exist_ok=True)
    shapes = tensor_shapes(cfg, s.rel_rows)
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
                gain = np.float32(1.0 if name == "embed" or name.endswith("mix.rel") else shape[1] ** -0.5)
                while rows_left > 0:                        # in slabs: a wide table would be gigabytes of floats at once
                    r = min(rows_left, 4096)
                    f.write(_bf16(rng.standard_normal((r, shape[1]), dtype=np.float32) * gain).astype("<u2").tobytes())
                    rows_left -= r
            else:
                f.write(_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(0.1)).astype("<u2").tobytes())
    os.replace(tmp, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return cfg


def weight_bytes_per_token(cfg: dict) -> int:
    """Weight bytes one decoded token reads: the projections and the output projection of every layer RUN, the router and the shared gate, of the routed
    experts only the chosen ones, the shared expert, one embedding row, the head."""
    W, V = cfg["width"], cfg["vocab"]
    loop = cfg.get("loop")
    runs = list(range(len(cfg["layers"])))
    if loop:
        a, b, n = loop["start"], loop["stop"], loop["times"]
        runs = list(range(a)) + list(range(a, b)) * n + list(range(b, len(cfg["layers"])))
    total = 2 * (W + V * W)
    for il in runs:
        lc = cfg["layers"][il]
        m = lc["mixer"]
        H, D, VD = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        if lc["type"] == "retention":
            rows = 2 * H * D + 2 * H * VD
        elif lc["type"] == "attention":
            rows = H * D + G * D + G * VD + H
        else:
            rows = 2 * H * D + 2 * G * D + G * VD + H * VD
        total += 2 * (rows * W + W * H * VD)
        mlp = lc.get("mlp")
        if mlp:
            total += 2 * (mlp["router"]["experts"] * W + 3 * mlp["expert"]["ff"] * W * mlp["router"]["top"])
            if mlp.get("shared"):
                total += 2 * (3 * mlp["shared"]["ff"] * W + W)
    return total
