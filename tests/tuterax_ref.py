"""Plain, slow restatement of the Tuterax design in float64 torch, one function per mechanism.

Test infrastructure only: it shares no code with the product path (cortex.llamacpp_amd/), runs on the CPU and
processes whole sequences at once - no cache, no batching, the recurrences token by token.  Weights are a dict
name -> tensor, the configuration is the dict a model's config.json holds.

Notation: x [T, width] the residual stream of one sequence, positions 0 .. T-1.
  layer:      x <- x + post(mixer(x), n1);  x <- x + post(ff(x), n2)    - the sublayers read x itself, the norm sits on their OUTPUT
  post:       y / rms(y) * (1 + n)
  attend:     q = Wq x, k = Wk x, v = Wv x;  q, k <- y / rms(y) * w per head (w shared by the heads);  the first `dims` entries of
              every q / k head turn (entry i with i + dims/2) by p * base^(-2i/dims);  every value head turns over ALL its entries
              (entry m with m + vdim/2) by its own position j;  s(i, j) = cap * tanh(q_i . k_j * scale / cap), j <= i;
              weight = exp(s) / (sum_j exp(s) + exp(sink_head));  the head's weighted sum of turned values turns back by -i;  Wo
  delta:      q, k, v = silu(short causal convolution of Wq x, Wk x, Wv x);  q, k <- unit vectors per head, q / sqrt(dim);
              b = sigmoid(Wb x);  a = exp(-exp(A) * softplus(Wa x + dt));
              S <- a S;  u = b (v - S^T k);  S <- S + k u^T;  o = S^T q;   out = o / rms(o) * w * silu(Wg x);  Wo
  channel_delta: the same with one decay per (head, key channel) - a = exp(-exp(A_head) * softplus(Wa2 Wa1 x + dt)), row d of S
              times a[d] - and the output gate sigmoid(Wg2 Wg1 x)
  ff:         Wdown (gelu_tanh(Wgate x) * (Wup x))
  output:     logits = E post-normed rows, E the embedding table (rows enter the stream times embedding.scale)
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def post_norm(y, n, eps):
    return rms_unit(y, eps) * (1.0 + n.to(F64))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def turn_halves(x, positions, dims, base, sign=1.0):
    """x [T, heads, D]: entry i < dims/2 pairs with entry i + dims/2 and turns by sign * position * base^(-2i/dims); entries from dims on pass."""
    if not dims:
        return x
    half = dims // 2
    f = float(base) ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    ang = sign * positions.to(F64)[:, None, None] * f[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def softcap(s, cap):
    return cap * torch.tanh(s / cap) if cap else s


def sink_softmax(s, seen, sink):
    """rows of s over the seen columns, with one more term exp(sink) in the denominator (no key, no value)."""
    s = s.masked_fill(~seen, float("-inf"))
    m = torch.maximum(s.max(-1, keepdim=True).values, sink.reshape(1, 1))
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - m))


def attend(x, W, p, mx, eps, without=()):
    """`without` names parts to leave out or bend - "sink", "value_turn", "softcap", "causal" (a row then also sees the next position) - so that a test can
    show that its inputs tell the right mechanism from a wrong one."""
    T = x.shape[0]
    H, G, D, VD = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    rot = mx.get("rot") or {}
    dims, base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
    pos = torch.arange(T)
    q = (x @ W[p + "q"].to(F64).T).reshape(T, H, D)
    k = (x @ W[p + "k"].to(F64).T).reshape(T, G, D)
    v = (x @ W[p + "v"].to(F64).T).reshape(T, G, VD)
    q = rms_unit(q, eps) * W[p + "q.norm"].to(F64)
    k = rms_unit(k, eps) * W[p + "k.norm"].to(F64)
    q = turn_halves(q, pos, dims, base)
    k = turn_halves(k, pos, dims, base)
    turn_v = bool(rot) and "value_turn" not in without
    if turn_v:
        v = turn_halves(v, pos, VD, base)
    seen = pos[None, :] <= pos[:, None] + (1 if "causal" in without else 0)
    sink = W[p + "sink"].to(F64) if "sink" not in without else torch.full((H,), float("-inf"), dtype=F64)
    cap = 0.0 if "softcap" in without else float(mx.get("softcap") or 0.0)
    heads = []
    for a in range(H):
        b = a // (H // G)
        s = softcap((q[:, a] @ k[:, b].T) * float(mx.get("scale", 1.0)), cap)
        heads.append(sink_softmax(s, seen, sink[a]) @ v[:, b])
    o = torch.stack(heads, 1)
    if turn_v:
        o = turn_halves(o, pos, VD, base, sign=-1.0)
    return o.reshape(T, H * VD) @ W[p + "o"].to(F64).T


def short_conv_silu(y, w):
    """y [T, C], w [C, taps]: out[t] = silu(sum_j w[:, taps-1-j] * y[t-j]), zeros before the start."""
    T, C = y.shape
    taps = w.shape[1]
    w = w.to(F64)
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), y], 0)
    out = torch.zeros(T, C, dtype=F64)
    for j in range(taps):
        out = out + pad[taps - 1 - j: taps - 1 - j + T] * w[:, taps - 1 - j]
    return out * torch.sigmoid(out)


def unit_vector(y):
    return y / torch.sqrt((y * y).sum(-1, keepdim=True) + 1e-6)


def delta_scan(q, k, v, beta, decay):
    """q, k [T, H, D]; v [T, H, VD]; beta [T, H]; decay [T, H, D] (a per-head decay is the same number for every d).  Returns [T, H, VD]."""
    T, H, D = q.shape
    VD = v.shape[-1]
    S = torch.zeros(H, D, VD, dtype=F64)
    out = torch.zeros(T, H, VD, dtype=F64)
    for t in range(T):
        S = S * decay[t][:, :, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def delta_mixer(x, W, p, mx, eps, per_channel):
    T = x.shape[0]
    H, G, D, VD = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = short_conv_silu(x @ W[p + "q"].to(F64).T, W[p + "q.conv"]).reshape(T, G, D)
    k = short_conv_silu(x @ W[p + "k"].to(F64).T, W[p + "k.conv"]).reshape(T, G, D)
    v = short_conv_silu(x @ W[p + "v"].to(F64).T, W[p + "v.conv"]).reshape(T, H, VD)
    q = unit_vector(q) * D ** -0.5
    k = unit_vector(k)
    rep = H // G
    q = q.repeat_interleave(rep, 1)
    k = k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(x @ W[p + "b"].to(F64).T)
    A = torch.exp(W[p + "A_log"].to(F64))
    dt = W[p + "dt_bias"].to(F64)
    sp = torch.nn.functional.softplus
    if per_channel:
        z = (x @ W[p + "a1"].to(F64).T) @ W[p + "a2"].to(F64).T + dt
        decay = torch.exp(-A[None, :, None] * sp(z).reshape(T, H, D))
        gate = torch.sigmoid((x @ W[p + "g1"].to(F64).T) @ W[p + "g2"].to(F64).T)
    else:
        z = x @ W[p + "a"].to(F64).T + dt
        decay = torch.exp(-A[None, :] * sp(z))[:, :, None].expand(T, H, D)
        g = x @ W[p + "g"].to(F64).T
        gate = g * torch.sigmoid(g)
    o = delta_scan(q, k, v, beta, decay)
    o = rms_unit(o, eps) * W[p + "norm"].to(F64)
    return (o.reshape(T, H * VD) * gate) @ W[p + "o"].to(F64).T


def feed_forward(x, W, p):
    return (gelu_tanh(x @ W[p + "gate"].to(F64).T) * (x @ W[p + "up"].to(F64).T)) @ W[p + "down"].to(F64).T


def mixer(x, W, p, lc, eps, without=()):
    if lc["type"] == "attention":
        return attend(x, W, p, lc["mixer"], eps, without)
    return delta_mixer(x, W, p, lc["mixer"], eps, per_channel=lc["type"] == "channel_delta")


def forward(cfg, W, tokens, taps=None, without=()):
    """Logits [T, vocab] of one sequence; taps (a list) receives the stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    E = W["embed"].to(F64)
    x = E[torch.as_tensor(tokens, dtype=torch.long)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    for il, lc in enumerate(cfg["layers"]):
        p = f"l{il}."
        x = x + post_norm(mixer(x, W, p + "mix.", lc, eps, without), W[p + "norm1"], eps)
        if lc.get("mlp"):
            x = x + post_norm(feed_forward(x, W, p + "mlp."), W[p + "norm2"], eps)
        if taps is not None:
            taps.append(x.clone())
    return post_norm(x, W["final.norm"], eps) @ E.T
