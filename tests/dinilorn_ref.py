"""Plain, slow restatement of the Dinilorn design in float64 torch, one function per mechanism.

Test infrastructure only: it shares no code with the product path (cortex.llamacpp_amd/), runs on the CPU and
processes whole sequences at once - no cache, no batching, the recurrence token by token.  Weights are a dict
name -> tensor, the configuration is the dict a model's config.json holds.

Notation: x [T, width] the residual stream of one sequence, positions 0 .. T-1; n(y, w) = y / rms(y) * (1 + w).
  layer:      x <- x + n(mixer(n(x, n1)), n1b);  x <- x + n(ff(n(x, n2)), n2b)
  loop:       layers start .. stop-1 run `times` times with the same weights; every pass but the first opens with x <- x + x0
              (x0 the embedding rows)
  retention:  q = Wq h, k = Wk h, v = Wv h per head;  the first `dims` entries of q / k turn (entry i with i + dims/2) by
              p * base^(-2i/dims);  k <- k / sqrt(dim);  S <- decay_head S + k v^T;  o = S^T q;  o / rms(o) per head;
              times silu(Wg h);  Wo
  attention:  q, k, v with biases;  q_p <- q_p (1 + coef ln(floor((p+1)/every) + 1));  s(i, j) = cap tanh(q_i.k_j scale / cap)
              + rel[bucket(i-j), head], j <= i;  weight = exp(s) / (1 + sum_j exp(s));  head's sum times sigmoid(Wg h)[head];  Wo + b
  attention_2: two score maps per head (q, k rows [head][map][dim]) over the same values;  interleaved turn (entry 2i with 2i+1)
              with the three-band frequency scaling;  j <= i and (i - j < size or j < keep_first);  plain softmax per map;
              o = a1 - lam a2, lam = exp(lq1.lk1) - exp(lq2.lk2) + diff;  o / rms(o) (1 - diff);  times sigmoid(Wg h) per entry;  Wo + b
  experts:    s = sigmoid(Wr h);  c = s + correction;  groups of neighbours score as the sum of their two largest c, the `keep`
              best groups stay open;  the `top` open experts with the largest c, weights s (as they are);
              expert(h) = Wdown (g sigmoid(1.702 g) (u + 1)), g = min(Wgate h, limit), u = clamp(Wup h, -limit, limit);
              plus sigmoid(Wsg h) * shared expert(h)
  output:     logits = head n(x, final)
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w.to(F64))


def lin(x, W, name, bias=False):
    y = x @ W[name].to(F64).T
    return y + W[name + ".b"].to(F64) if bias else y


# ---------------------------------------------------------------------------------------------- positions
def plain_frequencies(dims, base):
    return float(base) ** (-2.0 * torch.arange(dims // 2, dtype=F64) / dims)


def banded_frequencies(dims, base, scaling):
    """Radians per position of every pair; with `scaling` {factor, low, high, original}: short wavelengths stay, long ones slow down by
    `factor`, the band between them blends the two linearly in original / wavelength."""
    f = plain_frequencies(dims, base)
    if not scaling:
        return f
    factor, low, high, orig = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"]), float(scaling["original"])
    out = f.clone()
    for i in range(f.numel()):
        wl = 2.0 * math.pi / float(f[i])
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[i] = f[i] / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out


def turn_halves(x, positions, freq):
    """x [T, heads, D]: entry i < len(freq) pairs with entry i + len(freq); entries from 2 len(freq) on pass."""
    half = freq.numel()
    if not half:
        return x
    ang = positions.to(F64)[:, None, None] * freq[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., 2 * half:]], dim=-1)


def turn_neighbours(x, positions, freq):
    """x [T, heads, D]: entry 2i pairs with entry 2i + 1; entries from 2 len(freq) on pass."""
    half = freq.numel()
    if not half:
        return x
    ang = positions.to(F64)[:, None, None] * freq[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
    out = x.clone()
    out[..., 0:2 * half:2] = a * c - b * s
    out[..., 1:2 * half:2] = b * c + a * s
    return out


# ---------------------------------------------------------------------------------------------- retention
def retention_scan(q, k, v, decay):
    """q, k [T, H, D], v [T, H, VD], decay [H] -> o [T, H, VD]; the state starts at zero."""
    T, H, D = q.shape
    S = torch.zeros(H, D, v.shape[-1], dtype=F64)
    out = []
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hdv,hd->hv", S, q[t]))
    return torch.stack(out)


def retention(h, W, p, mx, eps, without=()):
    """`without`: "state" (every token sees only itself)."""
    T = h.shape[0]
    H, D, VD = mx["heads"], mx["dim"], mx["vdim"]
    rot = mx.get("rot") or {}
    freq = plain_frequencies(int(rot.get("dims", 0)), rot.get("base", 10000.0)) if rot.get("dims") else torch.zeros(0, dtype=F64)
    pos = torch.arange(T)
    q = turn_halves(lin(h, W, p + "q").reshape(T, H, D), pos, freq)
    k = turn_halves(lin(h, W, p + "k").reshape(T, H, D), pos, freq) * D ** -0.5
    v = lin(h, W, p + "v").reshape(T, H, VD)
    decay = torch.tensor(mx["decay"], dtype=F64) * (0.0 if "state" in without else 1.0)
    o = rms_unit(retention_scan(q, k, v, decay), eps).reshape(T, H * VD)
    g = lin(h, W, p + "g")
    return lin(o * g * torch.sigmoid(g), W, p + "o")


# ---------------------------------------------------------------------------------------------- attention with a distance bias
def distance_bucket(n, B, far):
    """Row of the bias table for distance n >= 0: one row per distance below B // 2, then rows spaced evenly in the logarithm up to `far`."""
    half = B // 2
    if n < half:
        return n
    return min(B - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (B - half))))


def query_temperature(positions, coef, every):
    return 1.0 + coef * torch.log(torch.floor((positions.to(F64) + 1.0) / every) + 1.0)


def softmax_one_more(s, seen):
    """rows of s over the seen columns with 1 added to the denominator (a term of score 0 that has no value)."""
    s = s.masked_fill(~seen, float("-inf"))
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(-m))


def attention(h, W, p, mx, without=()):
    """`without` names parts to leave out - "sink", "bias", "softcap", "temperature", "gate" - so that a test can show its inputs tell them apart."""
    T = h.shape[0]
    H, G, D, VD = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    pos = torch.arange(T)
    q = lin(h, W, p + "q", True).reshape(T, H, D)
    k = lin(h, W, p + "k", True).reshape(T, G, D)
    v = lin(h, W, p + "v", True).reshape(T, G, VD)
    qt = mx.get("q_temp")
    if qt and "temperature" not in without:
        q = q * query_temperature(pos, float(qt["coef"]), float(qt["every"]))[:, None, None]
    rel = W[p + "rel"].to(F64)
    B = rel.shape[0]
    dist = pos[:, None] - pos[None, :]
    seen = dist >= 0
    bucket = torch.tensor([[distance_bucket(int(n), B, mx["bias_max"]) if n >= 0 else 0 for n in row] for row in dist.tolist()])
    cap = float(mx.get("softcap") or 0.0)
    gate = torch.sigmoid(lin(h, W, p + "g"))
    heads = []
    for a in range(H):
        s = (q[:, a] @ k[:, a // (H // G)].T) * mx["scale"]
        if cap and "softcap" not in without:
            s = cap * torch.tanh(s / cap)
        if "bias" not in without:
            s = s + rel[bucket, a]
        w = torch.softmax(s.masked_fill(~seen, float("-inf")), -1) if "sink" in without else softmax_one_more(s, seen)
        o = w @ v[:, a // (H // G)]
        heads.append(o if "gate" in without else o * gate[:, a:a + 1])
    return lin(torch.cat(heads, -1), W, p + "o", True)


# ---------------------------------------------------------------------------------------------- two-map attention
def window_with_first(T, size, keep_first):
    pos = torch.arange(T)
    dist = pos[:, None] - pos[None, :]
    return (dist >= 0) & ((dist < size) | (pos[None, :] < keep_first))


def attention_two_maps(h, W, p, mx, eps, without=()):
    """`without`: "keep_first" (the first positions are lost like any other), "window_wider" (one more position seen), "second_map" (lambda = 0)."""
    T = h.shape[0]
    H, G, D, VD = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    pos = torch.arange(T)
    rot = mx.get("rot") or {}
    freq = banded_frequencies(int(rot["dims"]), rot.get("base", 10000.0), rot.get("scaling")) if rot.get("dims") else torch.zeros(0, dtype=F64)
    q = turn_neighbours(lin(h, W, p + "q", True).reshape(T, H * 2, D), pos, freq).reshape(T, H, 2, D)
    k = turn_neighbours(lin(h, W, p + "k", True).reshape(T, G * 2, D), pos, freq).reshape(T, G, 2, D)
    v = lin(h, W, p + "v", True).reshape(T, G, VD)
    mask = mx.get("mask") or {}
    if mask.get("size"):
        seen = window_with_first(T, int(mask["size"]) + (1 if "window_wider" in without else 0), 0 if "keep_first" in without else int(mask.get("keep_first", 0)))
    else:
        seen = window_with_first(T, T + 1, 0)
    diff = float(mx["diff"])
    lam = math.exp(float((W[p + "lq1"].to(F64) * W[p + "lk1"].to(F64)).sum())) - math.exp(float((W[p + "lq2"].to(F64) * W[p + "lk2"].to(F64)).sum())) + diff
    if "second_map" in without:
        lam = 0.0
    heads = []
    for a in range(H):
        g = a // (H // G)
        maps = []
        for m in range(2):
            s = (q[:, a, m] @ k[:, g, m].T) * mx["scale"]
            maps.append(torch.softmax(s.masked_fill(~seen, float("-inf")), -1) @ v[:, g])
        heads.append(rms_unit(maps[0] - lam * maps[1], eps) * (1.0 - diff))
    o = torch.cat(heads, -1) * torch.sigmoid(lin(h, W, p + "g"))
    return lin(o, W, p + "o", True)


# ---------------------------------------------------------------------------------------------- experts
def expert(h, W, p, limit):
    g = torch.clamp(lin(h, W, p + "gate"), max=limit)
    u = torch.clamp(lin(h, W, p + "up"), min=-limit, max=limit)
    return lin(g * torch.sigmoid(1.702 * g) * (u + 1.0), W, p + "down")


def route(z, correction, top, groups, keep):
    """z [T, E] router logits -> (ids [T, top], weights [T, top]); ties go to the lower index."""
    s = torch.sigmoid(z)
    c = s + correction.to(F64)
    T, E = c.shape
    per = E // groups
    gs = c.reshape(T, groups, per).topk(min(2, per), -1).values.sum(-1)
    open_groups = torch.zeros(T, groups, dtype=torch.bool)
    for t in range(T):
        order = sorted(range(groups), key=lambda g: (-float(gs[t, g]), g))[:keep]
        open_groups[t, order] = True
    c = c.masked_fill(~open_groups.repeat_interleave(per, 1), float("-inf"))
    ids = torch.stack([torch.tensor(sorted(range(E), key=lambda e: (-float(c[t, e]), e))[:top]) for t in range(T)])
    return ids, s.gather(1, ids)


def experts(h, W, p, mlp, without=()):
    rt = mlp["router"]
    gr = rt.get("groups") or {"count": 1, "keep": 1}
    if "groups" in without:
        gr = {"count": 1, "keep": 1}
    corr = W[p + "correction"] * (0.0 if "correction" in without else 1.0)
    ids, w = route(lin(h, W, p + "router"), corr, rt["top"], gr["count"], gr["keep"])
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            out[t] += w[t, j] * expert(h[t:t + 1], W, p + "e%d." % int(ids[t, j]), float(mlp["expert"]["limit"]))[0]
    sh = mlp.get("shared")
    if sh and "shared" not in without:
        out = out + torch.sigmoid(lin(h, W, p + "shared.sg")) * expert(h, W, p + "shared.", float(sh["limit"]))
    return out


# ---------------------------------------------------------------------------------------------- the model
def layer_runs(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {}
    a, b, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
    if b <= a or times < 1:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens, taps=None, without=()):
    """logits [T, vocab] of one sequence; taps (a list) receives the stream after every layer run; `without` bends mechanisms (see the mixers; "reopen": the
    passes of the looped span do not take the embedding rows in again; "correction": the router picks by its scores alone; "groups": every group stays open)."""
    eps = float(cfg["norm"]["eps"])
    x0 = W["embed"].to(F64)[torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    for il, reopen in layer_runs(cfg):
        lc = cfg["layers"][il]
        p = "l%d." % il
        if reopen and "reopen" not in without:
            x = x + x0
        h = norm(x, W[p + "norm1"], eps)
        if lc["type"] == "retention":
            y = retention(h, W, p + "mix.", lc["mixer"], eps, without)
        elif lc["type"] == "attention":
            y = attention(h, W, p + "mix.", lc["mixer"], without)
        elif lc["type"] == "attention_2":
            y = attention_two_maps(h, W, p + "mix.", lc["mixer"], eps, without)
        else:
            raise ValueError(lc["type"])
        x = x + norm(y, W[p + "norm1b"], eps)
        if lc.get("mlp"):
            x = x + norm(experts(norm(x, W[p + "norm2"], eps), W, p + "mlp.", lc["mlp"], without), W[p + "norm2b"], eps)
        if taps is not None:
            taps.append(x.clone())
    return lin(norm(x, W["final.norm"], eps), W, "head")
